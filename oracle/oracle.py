"""ctypes binding of the CPU oracle (oracle/libawq_oracle.so).  TEST INFRASTRUCTURE ONLY.

Imported by tests, the smoke check and the benchmark's cpu_baseline leg; never by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libawq_oracle.so")


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def _load():
    if not os.path.exists(_SO):
        build()
    h = C.CDLL(_SO)
    vp, i, f = C.c_void_p, C.c_int, C.c_float
    sig = {
        "orc_half_to_float_sw": ([C.c_uint16], f),
        "orc_float_to_half_sw": ([f], C.c_uint16),
        "orc_half_to_float": ([C.c_uint16], f),
        "orc_float_to_half": ([f], C.c_uint16),
        "orc_num_threads": ([], i),
        "orc_set_exact_sums": ([i], None),
        "orc_dequant": ([vp, vp, vp, vp, i, i], None),
        "orc_matvec_int4": ([vp, vp, vp, vp, vp, i, i, i, i, i, vp], i),
        "orc_qkv_matvec": ([vp] * 13 + [i, i, i, vp], i),
        "orc_ffn_matvec_silu": ([vp] * 8 + [i, i], i),
        "orc_embed": ([vp, vp, i, vp, vp], None),
        "orc_rmsnorm": ([vp, vp, vp, i], None),
        "orc_matvec_f16": ([vp, vp, vp, i, i], i),
        "orc_rope": ([vp, vp, i, i, i, vp, i, f], None),
        "orc_attention": ([vp, vp, vp, vp, vp, i, i, i, vp], None),
        "orc_argmax_advance": ([vp, i, vp, vp, vp, i], i),
        "orc_random_f32": ([vp], f),
        "orc_softmax_logits": ([vp, i, f], None),
        "orc_sample_top_p": ([vp, i, f, i, vp, vp, vp], i),
        "orc_top_p_pick_fp16_scan": ([vp, i, f, i, i, i, i], i),
        "orc_model_file_bytes": ([vp], C.c_size_t),
        "orc_model_open": ([vp, C.c_size_t], vp),
        "orc_model_close": ([vp], None),
        "orc_model_reset": ([vp, vp, i], None),
        "orc_model_set_pos": ([vp, i, i], None),
        "orc_model_buffer": ([vp, C.c_char_p], vp),
        "orc_model_tokens": ([vp], vp),
        "orc_model_pos": ([vp], i),
        "orc_model_forward": ([vp, i], i),
        "orc_generate": ([vp, vp, i, i, i, vp], i),
    }
    for name, (args, res) in sig.items():
        fn = getattr(h, name)
        fn.argtypes = args
        fn.restype = res
    return h


lib = _load()


def _p(a):
    return a.ctypes.data if a is not None else None


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def num_threads():
    return lib.orc_num_threads()


def set_exact_sums(on):
    """Diagnostic: matrix-vector sums in double precision (rounded to fp32 once) instead of the reference's fp32 order.
    Process-wide; switch it off again after use."""
    lib.orc_set_exact_sums(int(on))


def dequant(weight, zeros, scales, K, N):
    w, z, s = _c(weight, np.uint32), _c(zeros, np.uint32), _c(scales.view(np.uint16), np.uint16)
    out = np.empty((N, K), dtype=np.uint16)
    lib.orc_dequant(_p(out), _p(w), _p(z), _p(s), K, N)
    return out.view(np.float16)


def matvec_int4(out, x, weight, zeros, scales, K, N, accum=False, gpu_count=1, loff=-1, pos=None):
    """out: fp16 array updated in place (viewed as uint16)."""
    w, z, s = _c(weight, np.uint32), _c(zeros, np.uint32), _c(scales.view(np.uint16), np.uint16)
    xx = _c(x.view(np.uint16), np.uint16)
    p = np.array([pos if pos is not None else 0], dtype=np.int32)
    assert out.flags["C_CONTIGUOUS"]
    return lib.orc_matvec_int4(_p(out), _p(xx), _p(w), _p(z), _p(s), K, N, int(accum), gpu_count, loff, _p(p))


def qkv_matvec(q, kc, vc, x, qw, kw, vw, K, N, loff, pos):
    arrs = []
    for m in (qw, kw, vw):
        arrs += [_c(m[0], np.uint32), _c(m[1], np.uint32), _c(m[2].view(np.uint16), np.uint16)]
    xx = _c(x.view(np.uint16), np.uint16)
    p = np.array([pos], dtype=np.int32)
    return lib.orc_qkv_matvec(_p(q), _p(kc), _p(vc), _p(xx), *[_p(a) for a in arrs], K, N, loff, _p(p))


def ffn_matvec_silu(out, x, gate, up, K, N):
    arrs = []
    for m in (gate, up):
        arrs += [_c(m[0], np.uint32), _c(m[1], np.uint32), _c(m[2].view(np.uint16), np.uint16)]
    xx = _c(x.view(np.uint16), np.uint16)
    return lib.orc_ffn_matvec_silu(_p(out), _p(xx), *[_p(a) for a in arrs], K, N)


def rmsnorm(x, weight):
    xx, ww = _c(x.view(np.uint16), np.uint16), _c(weight.view(np.uint16), np.uint16)
    o = np.empty_like(xx)
    lib.orc_rmsnorm(_p(o), _p(xx), _p(ww), xx.size)
    return o.view(np.float16)


def matvec_f16(x, w, n, d):
    xx, ww = _c(x.view(np.uint16), np.uint16), _c(w.view(np.uint16), np.uint16)
    o = np.empty(d, dtype=np.uint16)
    r = lib.orc_matvec_f16(_p(o), _p(xx), _p(ww), n, d)
    return r, o.view(np.float16)


def rope(q, k_base, num_heads, num_kv_heads, head_size, pos, loff, theta):
    """q, k_base: uint16 arrays modified in place."""
    p = np.array([pos], dtype=np.int32)
    lib.orc_rope(_p(q), _p(k_base), num_heads, num_kv_heads, head_size, _p(p), loff, theta)


def attention(q, key_cache, value_cache, num_heads, head_size, kv_mul, pos):
    """key_cache/value_cache: uint16 (seq, kv_dim) of one layer. Returns (out fp16, att fp16 (heads, pos+1))."""
    p = np.array([pos], dtype=np.int32)
    out = np.empty(num_heads * head_size, dtype=np.uint16)
    att = np.empty(num_heads * (pos + 1), dtype=np.uint16)
    qq = _c(q.view(np.uint16), np.uint16)
    lib.orc_attention(_p(out), _p(qq), _p(key_cache), _p(value_cache), _p(att), num_heads, head_size, kv_mul, _p(p))
    return out.view(np.float16), att.view(np.float16).reshape(num_heads, pos + 1)


def argmax_advance(logits, tokens, pos_host, pos_dev, write_token):
    ll = _c(logits.view(np.uint16), np.uint16)
    return lib.orc_argmax_advance(_p(ll), ll.size, _p(tokens), _p(pos_host), _p(pos_dev), int(write_token))


def random_f32(state):
    """state: np.uint64 array of 1 (updated in place). sampler.h:65-74."""
    return float(lib.orc_random_f32(_p(state)))


def softmax_logits(logits, temperature):
    """Returns the fp16 probabilities (uint16 view in, new array out)."""
    ll = np.array(logits.view(np.uint16), dtype=np.uint16, copy=True)
    lib.orc_softmax_logits(_p(ll), ll.size, float(temperature))
    return ll.view(np.float16)


def sample_top_p(probs, threshold, sorted_, tokens, pos_host, pos_dev):
    pp = _c(probs.view(np.uint16), np.uint16)
    return lib.orc_sample_top_p(_p(pp), pp.size, float(threshold), int(sorted_), _p(tokens), _p(pos_host), _p(pos_dev))


def top_p_pick_fp16_scan(probs, threshold, sorted_, mode, threads=128, items=16):
    """The top-p pick when the prefix sum is added in fp16: mode 0 sequentially, mode 1 in tiles of threads x items."""
    pp = _c(probs.view(np.uint16), np.uint16)
    return lib.orc_top_p_pick_fp16_scan(_p(pp), pp.size, float(threshold), int(sorted_), int(mode), int(threads), int(items))


class Model:
    def __init__(self, image):
        self.image = np.ascontiguousarray(image)  # must outlive the model
        self.h = lib.orc_model_open(_p(self.image), self.image.nbytes)
        if not self.h:
            raise ValueError("oracle: bad model image")
        hdr = self.image[:28].view(np.int32)
        self.config = dict(zip(("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len"), map(int, hdr)))

    def close(self):
        if self.h:
            lib.orc_model_close(self.h)
            self.h = None

    def buffer(self, name, count):
        ptr = lib.orc_model_buffer(self.h, name.encode())
        return np.ctypeslib.as_array((C.c_uint16 * count).from_address(ptr))

    def tokens(self, n):
        ptr = lib.orc_model_tokens(self.h)
        return list(np.ctypeslib.as_array((C.c_int * n).from_address(ptr)))

    def reset(self, prompt):
        arr = np.array(prompt, dtype=np.int32)
        lib.orc_model_reset(self.h, _p(arr), arr.size)

    def set_pos(self, pos, token):
        lib.orc_model_set_pos(self.h, pos, token)

    @property
    def pos(self):
        return lib.orc_model_pos(self.h)

    def forward(self, gen_token=True):
        return lib.orc_model_forward(self.h, int(gen_token))

    def generate(self, prompt, steps, ignore_eos=False, want_logits=False):
        arr = np.array(prompt, dtype=np.int32)
        logits = np.zeros((steps, self.config["vocab_size"]), dtype=np.uint16) if want_logits else None
        pos = lib.orc_generate(self.h, _p(arr), arr.size, steps, int(ignore_eos), _p(logits))
        return self.tokens(pos + 1), pos, (logits.view(np.float16) if want_logits else None)
