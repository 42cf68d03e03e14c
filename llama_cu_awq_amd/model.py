"""Host-side mirror of build_transformer / run_transformer / generate_thread (llama2_q4.cu:541-757) over the C-ABI."""
import ctypes as C

import numpy as np

from ._lib import ConfigC, LayerWeightsC, RunStateC, check, lib
from .ops import DeviceBuffer, QWeight

SCHEDULE_REFERENCE = 0
SCHEDULE_FUSED = 1
SCHEDULE_PERSISTENT = 2
EOS_TOKEN = 2  # tokenizer.h:10


class Transformer:
    def __init__(self, ctx, image=None, path=None):
        self.ctx = ctx
        h = C.c_void_p()
        if path is not None:
            check(lib.awq_transformer_load_file(ctx.h, path.encode(), C.byref(h)))
        else:
            image = np.ascontiguousarray(image)
            check(lib.awq_transformer_load_image(ctx.h, image.ctypes.data, image.nbytes, C.byref(h)))
        self.h = h
        cfg = ConfigC()
        check(lib.awq_transformer_config(h, C.byref(cfg)))
        self.config = {n: getattr(cfg, n) for n, _ in ConfigC._fields_}
        st = RunStateC()
        check(lib.awq_transformer_state(h, C.byref(st)))
        self.state = st
        self._tokens = (C.c_int * (self.config["seq_len"] + 1)).from_address(st.shared_tokens)
        self._pos = C.c_int.from_address(st.shared_pos)

    def close(self):
        if self.h:
            check(lib.awq_transformer_free(self.h))
            self.h = None

    # run state access ----------------------------------------------------
    def buffer(self, name, nbytes):
        return DeviceBuffer(self.ctx, nbytes, ptr=getattr(self.state, name))

    def download(self, name, count, dtype=np.uint16):
        return self.buffer(name, count * np.dtype(dtype).itemsize).download(dtype, count)

    def layer(self, l):
        lw = LayerWeightsC()
        check(lib.awq_transformer_layer(self.h, l, C.byref(lw)))
        out = {"rms_att_weight": lw.rms_att_weight, "rms_ffn_weight": lw.rms_ffn_weight}
        for n in ("wq_q", "wq_k", "wq_v", "wq_o", "wq_gate", "wq_up", "wq_down"):
            q = getattr(lw, n)
            out[n] = QWeight(q.weight, q.zeros, q.scales)
        return out

    @property
    def pos(self):
        return self._pos.value

    def token(self, i):
        return self._tokens[i]

    # decode ----------------------------------------------------------------
    def reset(self, prompt_tokens):
        arr = (C.c_int * len(prompt_tokens))(*[int(t) for t in prompt_tokens])
        check(lib.awq_transformer_reset(self.h, arr, len(prompt_tokens)))

    def set_pos(self, pos, token):
        check(lib.awq_transformer_set_pos(self.h, pos, token))

    def forward(self, gen_token=True, use_graph=False, mode=SCHEDULE_FUSED):
        check(lib.awq_transformer_forward(self.h, int(gen_token), int(use_graph), mode))

    def capture(self, max_positions, mode=SCHEDULE_FUSED):
        """Record the launch sequences of every sequence-length bin below max_positions ahead of time."""
        check(lib.awq_transformer_capture(self.h, mode, max_positions))

    LAUNCH_KINDS = ("embed", "qkv", "attention", "oproj", "gate_up", "down", "classifier")

    def time_launches(self, passes=4):
        """Mean GPU microseconds per launch of the fused schedule at the current position, by launch kind."""
        us = (C.c_float * len(self.LAUNCH_KINDS))()
        n = (C.c_int * len(self.LAUNCH_KINDS))()
        check(lib.awq_transformer_time_launches(self.h, passes, us, n))
        return {k: {"us": round(us[i], 3), "launches": n[i]} for i, k in enumerate(self.LAUNCH_KINDS)}

    def forward_logits(self, use_graph=False, mode=SCHEDULE_FUSED):
        """run_llama_network() alone: this position's logits, no sampler."""
        check(lib.awq_transformer_forward_logits(self.h, int(use_graph), mode))

    def sample(self, sampler, gen_token=True):
        """sample() (sampler.h:77-115) on this model's logits and token list."""
        check(lib.awq_transformer_sample(self.h, sampler.h, int(gen_token)))

    def prefill(self, n_tokens, gen_token=True):
        """Consume n_tokens prompt tokens (already in the token list, from the current position) in one batched pass."""
        check(lib.awq_transformer_prefill(self.h, n_tokens, int(gen_token)))

    def generate(self, prompt_tokens, steps, ignore_eos=False, use_graph=False, mode=SCHEDULE_FUSED, on_logits=None):
        """The loop of generate_thread (llama2_q4.cu:697-745) without text output.

        Returns (tokens[0..pos], pos).  on_logits(pos, fp16 bits) is called after each pass when given
        (this adds a synchronisation per token and is meant for tests).
        """
        vocab = self.config["vocab_size"]
        self.reset(prompt_tokens)
        n_prompt = len(prompt_tokens)
        pos = 0
        while pos < steps:
            self.ctx.sync()  # wait for the previous token (llama2_q4.cu:713)
            self.forward(pos >= n_prompt - 1, use_graph, mode)
            if on_logits is not None:
                on_logits(pos, self.download("logits", vocab))
            if pos > 0:
                nxt = self._tokens[pos]
                if nxt >= vocab:
                    nxt = 0
                if nxt == EOS_TOKEN and not ignore_eos:
                    break
            pos += 1
        self.ctx.sync()
        return [self._tokens[i] for i in range(pos + 1)], pos
