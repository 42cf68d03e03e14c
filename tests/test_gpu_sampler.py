"""GPU parity of the temperature / top-p sampler (through the C-ABI) against the CPU oracle.

softmax of the logits: within 2 fp16 steps of the oracle (expf of the two platforms may differ in the last bit of
fp32, which can move an fp16 rounding).  The selection (order, exact prefix sums, first crossing) is integer work: the
token must be IDENTICAL to the oracle's on the same fp16 probabilities.
"""
import ctypes as C

import numpy as np
import pytest

import llama_cu_awq_amd as A
from llama_cu_awq_amd import synth
from llama_cu_awq_amd._lib import AWQ_ERR_SHAPE
from oracle import oracle
from tests.helpers import f16, ulp_diff_f16

pytestmark = pytest.mark.gpu


class Pinned:
    """SharedData-like pinned block: pos at byte 0, tokens from byte 16."""

    def __init__(self, ctx, n=64):
        self.ctx = ctx
        self.host = ctx.alloc_host(16 + 4 * n)
        self.pos = C.c_int.from_address(self.host)
        self.tokens = (C.c_int * n).from_address(self.host + 16)
        self.dpos = ctx.upload(np.array([0], dtype=np.int32))

    def set_pos(self, p):
        self.ctx.sync()
        self.pos.value = p
        self.dpos = self.ctx.upload(np.array([p], dtype=np.int32))

    def close(self):
        self.ctx.free_host(self.host)


def _logits(seed, n, scale):
    return (np.random.default_rng(seed).normal(0, scale, n)).astype(np.float16)


@pytest.mark.parametrize("n,temperature,scale", [(32000, 0.5, 2.0), (32000, 1.0, 5.0), (1000, 0.7, 1.0), (5, 0.3, 1.0), (1025, 2.0, 8.0), (65535, 0.9, 3.0), (40000, 0.7, 2.0), (32768, 0.6, 3.0), (32769, 0.6, 3.0), (65536, 0.8, 3.0), (128256, 0.7, 4.0)])
def test_softmax_logits(ctx, n, temperature, scale):
    l = _logits(3, n, scale)
    d = ctx.upload(l.view(np.uint16))
    A.softmax_logits(ctx, d, n, temperature)
    got = f16(d.download(np.uint16))
    want = oracle.softmax_logits(l, temperature)
    assert ulp_diff_f16(got, want).max() <= 2
    assert abs(float(got.astype(np.float64).sum()) - 1.0) < 2e-3


def _oracle_pick(probs, threshold, sorted_):
    tokens = np.zeros(4, dtype=np.int32)
    ph = np.array([0], dtype=np.int32)
    pd = np.array([0], dtype=np.int32)
    return oracle.sample_top_p(probs, threshold, sorted_, tokens, ph, pd)


@pytest.mark.parametrize("sorted_", [0, 1])
@pytest.mark.parametrize("case", range(12))
def test_sample_top_p_identical_to_oracle(ctx, case, sorted_):
    rng = np.random.default_rng(200 + case)
    n = [32000, 32000, 4097, 777, 64, 3, 65535, 1024, 40000, 49153, 65536, 128256][case]  # up to 32768 / 49152 / 65535 / beyond: the forms of the kernels
    if case == 7:
        probs = np.full(n, 1.0 / 1024, dtype=np.float16)  # all equal: pure tie-breaking by index
    elif case == 6:
        probs = oracle.softmax_logits(_logits(case, n, 0.2), 1.0)  # nearly flat: thousands of equal values per bin
    else:
        probs = oracle.softmax_logits(_logits(case, n, [2.0, 7.0, 1.0, 3.0, 0.5, 1.0, 0, 0, 2.0, 4.0, 0.3, 5.0][case]), 0.8)
    d = ctx.upload(probs.view(np.uint16))
    pin = Pinned(ctx)
    thresholds = list(rng.uniform(0, 1, 20)) + [0.0, 1e-8, 2.0 ** -24, 0.5, 0.999, 1.0, 1.0005, 1.5]
    for i, th in enumerate(thresholds):
        pin.set_pos(7)
        A.sample_top_p(ctx, d, n, th, sorted_, pin.host + 16, pin.host, pin.dpos)
        ctx.sync()
        want = _oracle_pick(probs, th, sorted_)
        assert pin.tokens[8] == want, (n, th, sorted_)
        assert pin.pos.value == 8 and pin.dpos.download(np.int32)[0] == 8
    assert np.array_equal(d.download(np.uint16), probs.view(np.uint16))  # probabilities untouched
    pin.close()


def test_sample_top_p_rejects_large_vocabulary(ctx):
    pin = Pinned(ctx)
    d = ctx.zeros(16)
    with pytest.raises(A.AwqError) as e:
        A.sample_top_p(ctx, d, (1 << 20) + 1, 0.5, 1, pin.host + 16, pin.host, pin.dpos)
    assert e.value.code == AWQ_ERR_SHAPE
    pin.close()


@pytest.mark.parametrize("V", [32000, 128256])
@pytest.mark.parametrize("temperature,topp", [(0.5, 0.6), (1.0, 0.9), (0.8, 1.0), (1.3, 0.0), (0.0, 0.6)])
def test_sampler_object_follows_reference_sample(ctx, temperature, topp, V):
    """awq_sampler_sample = coin from xorshift*, greedy when temperature is 0 or the token is not generated, else
    softmax + (top-p | plain) selection with threshold coin * topp | coin."""
    seed = 4242
    s = A.Sampler(ctx, V, temperature, topp, seed)
    state = np.array([seed], dtype=np.uint64)
    pin = Pinned(ctx)
    for step in range(12):
        l = _logits(50 + step, V, 3.0)
        d = ctx.upload(l.view(np.uint16))
        gen = step % 4 != 3
        pin.set_pos(step)
        pin.tokens[step + 1] = -1
        s.sample(d, pin.host + 16, pin.host, pin.dpos, gen)
        ctx.sync()
        coin = oracle.random_f32(state)  # drawn on every call
        assert pin.pos.value == step + 1
        if not gen:
            assert pin.tokens[step + 1] == -1
        elif temperature == 0.0:
            assert pin.tokens[step + 1] == int(np.argmax(l.astype(np.float32)))
        else:
            probs = f16(d.download(np.uint16))  # the logits now hold the probabilities
            assert ulp_diff_f16(probs, oracle.softmax_logits(l, temperature)).max() <= 2
            nucleus = 0.0 < topp < 1.0
            th = np.float32(coin) * np.float32(topp) if nucleus else np.float32(coin)
            assert pin.tokens[step + 1] == _oracle_pick(probs, float(th), 1 if nucleus else 0)
    s.close()
    pin.close()


@pytest.mark.parametrize("use_graph", [False, True])
def test_transformer_sample_loop(ctx, use_graph):
    """forward_logits + sample on a small model: greedy sampler == the fused forward; stochastic sampler picks what
    the oracle picks from the GPU's own probabilities, and the token feeds the next step.  With use_graph the network
    is a replayed recording (llama2_q4.cu:552-590) and the sampler is launched behind it."""
    cfg = dict(dim=256, hidden_dim=768, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=2048, seq_len=64, rope_theta=10000.0)
    img = synth.make_model_image(cfg, seed=5)
    prompt = [3, 9, 27]
    t = A.Transformer(ctx, image=img)
    # greedy through the sampler object
    g = A.Sampler(ctx, cfg["vocab_size"], 0.0, 0.9, 1)
    t.reset(prompt)
    for pos in range(12):
        ctx.sync()
        t.forward_logits(use_graph)
        t.sample(g, pos >= len(prompt) - 1)
    ctx.sync()
    greedy = [t.token(i) for i in range(13)]
    t.reset(prompt)
    for pos in range(12):
        ctx.sync()
        t.forward(pos >= len(prompt) - 1, use_graph)
    ctx.sync()
    assert greedy == [t.token(i) for i in range(13)]
    g.close()
    # stochastic
    seed, temperature, topp = 99, 0.9, 0.8
    s = A.Sampler(ctx, cfg["vocab_size"], temperature, topp, seed)
    state = np.array([seed], dtype=np.uint64)
    t.reset(prompt)
    for pos in range(16):
        ctx.sync()
        t.forward_logits(use_graph)
        gen = pos >= len(prompt) - 1
        t.sample(s, gen)
        ctx.sync()
        coin = oracle.random_f32(state)
        assert t.pos == pos + 1
        if gen:
            probs = f16(t.download("logits", cfg["vocab_size"]))
            want = _oracle_pick(probs, float(np.float32(coin) * np.float32(topp)), 1)
            assert t.token(pos + 1) == want
        else:
            assert t.token(pos + 1) == prompt[pos + 1]
    s.close()
    t.close()


def test_recorded_network_equals_eager_across_bins(ctx):
    """forward_logits as a replayed recording gives the logits of the eager launch sequence, bit for bit, on both sides
    of the 128-position bin boundary (the recordings are keyed by bin; positions are read from device memory), and
    prompt steps of forward(use_graph) leave the prompt's tokens alone."""
    cfg = dict(dim=256, hidden_dim=768, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=512, seq_len=300, rope_theta=10000.0)
    img = synth.make_model_image(cfg, seed=8)
    prompt = [int(x) for x in synth.prompt_tokens(3, 140, cfg["vocab_size"])]
    g = A.Sampler(ctx, cfg["vocab_size"], 0.0, 0.9, 1)
    logits = {}
    for use_graph in (False, True):
        t = A.Transformer(ctx, image=img)
        t.reset(prompt)
        rows = []
        for pos in range(150):
            ctx.sync()
            t.forward_logits(use_graph)
            ctx.sync()
            if pos in (0, 5, 126, 127, 128, 129, 140, 149):
                rows.append(t.download("logits", cfg["vocab_size"]).copy())
            t.sample(g, pos >= len(prompt) - 1)
        ctx.sync()
        logits[use_graph] = (rows, [t.token(i) for i in range(151)])
        t.close()
    for a, b in zip(logits[False][0], logits[True][0]):
        assert np.array_equal(a, b)
    assert logits[False][1] == logits[True][1]
    assert logits[True][1][: len(prompt)] == prompt
    # forward(use_graph) through the prompt: recorded network + sampler that only advances
    t = A.Transformer(ctx, image=img)
    t.reset(prompt)
    for pos in range(150):
        ctx.sync()
        t.forward(pos >= len(prompt) - 1, True)
    ctx.sync()
    assert [t.token(i) for i in range(151)] == logits[False][1]
    t.close()
    g.close()
