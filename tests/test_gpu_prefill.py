"""GPU parity of the multi-token prefill path: the int4 x fp16 MFMA GEMM against fp64, and a whole prefill against
the oracle's token-by-token run (KV cache contents and last-token logits within rel-L2 1e-2, same next token)."""
import numpy as np
import pytest

import llama_cu_awq_amd as A
from llama_cu_awq_amd import synth
from oracle import oracle
from tests.helpers import f16, rel_l2

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,K,N", [(128, 128, 128), (1, 256, 128), (37, 512, 256), (512, 4096, 256), (200, 11008, 128), (130, 1024, 384)])
def test_gemm_int4_vs_fp64(ctx, M, K, N):
    key = synth.stream_key(30, M, K, N)
    w, z, s = synth.make_qweight(key, K, N)
    a = synth.normal_f16(synth.stream_key(key, "a"), M * K)
    qw = A.QWeight.upload(ctx, w, z, s)
    dout = ctx.zeros(M * N * 2)
    A.gemm_q(ctx, dout, N, ctx.upload(a), K, M, qw, K, N)
    got = f16(dout.download(np.uint16)).reshape(M, N)
    # truth: the dequantised fp16 weights (bit-exact definition) times the activations in fp64
    w16 = synth.dequantize(w, z, s, K).astype(np.float32).astype(np.float16).astype(np.float64)
    truth = a.astype(np.float64).reshape(M, K) @ w16.T
    assert rel_l2(got, truth) <= 1e-3
    # residual epilogue
    resid = synth.normal_f16(synth.stream_key(key, "r"), M * N)
    dout = ctx.upload(resid)
    A.gemm_q(ctx, dout, N, ctx.upload(a), K, M, qw, K, N, accum=True)
    got = f16(dout.download(np.uint16)).reshape(M, N)
    assert rel_l2(got, truth + resid.astype(np.float64).reshape(M, N)) <= 1e-3


def test_gemm_shape_guard(ctx):
    buf = ctx.alloc(1 << 16)
    qw = A.QWeight(buf, buf, buf)
    for M, K, N in ((4, 48, 128), (4, 64, 64), (0, 64, 128)):
        with pytest.raises(A.AwqError) as e:
            A.gemm_q(ctx, buf, N, buf, K, M, qw, K, N)
        assert e.value.code == -2


CFG = dict(dim=512, hidden_dim=1536, n_layers=3, n_heads=4, n_kv_heads=4, vocab_size=1024, seq_len=192, rope_theta=10000.0)
CFG_GQA = dict(dim=512, hidden_dim=1280, n_layers=2, n_heads=8, n_kv_heads=2, vocab_size=512, seq_len=96, rope_theta=10000.0)
# 128-wide heads with grouped KV: the matrix-core attention kernel with kv_mul > 1
CFG_GQA128 = dict(dim=1024, hidden_dim=1536, n_layers=2, n_heads=8, n_kv_heads=2, vocab_size=512, seq_len=128, rope_theta=10000.0)


# 128-wide heads and a prompt longer than one 512-token chunk: the second chunk attends to more than 512 keys (several
# rounds of key blocks per wave, the two-pass softmax, more than two rounds of value tiles)
CFG_LONG128 = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=512, seq_len=1024, rope_theta=10000.0)


@pytest.mark.parametrize("cfg,n_prompt", [(CFG, 130), (CFG, 16), (CFG, 1), (CFG, 97), (CFG_GQA, 70), (CFG_GQA128, 75),
                                          (CFG_LONG128, 700), (CFG_LONG128, 1000)])
def test_prefill_matches_token_by_token_oracle(ctx, cfg, n_prompt):
    img = synth.make_model_image(cfg, seed=31)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    prompt = synth.prompt_tokens(31, n_prompt, cfg["vocab_size"])
    o.reset(prompt)
    for i in range(n_prompt):
        o.forward(i >= n_prompt - 1)
    t.reset(prompt)
    t.prefill(n_prompt, gen_token=True)
    ctx.sync()
    assert t.pos == n_prompt
    kv_dim = cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"]
    n_layers, seq = cfg["n_layers"], cfg["seq_len"]
    for name in ("key_cache", "value_cache"):
        got = f16(t.download(name, n_layers * seq * kv_dim)).reshape(n_layers, seq, kv_dim)[:, :n_prompt]
        want = f16(o.buffer(name, n_layers * seq * kv_dim)).reshape(n_layers, seq, kv_dim)[:, :n_prompt]
        assert rel_l2(got, want) <= 1e-2, name
        for l in range(n_layers):
            assert rel_l2(got[l], want[l]) <= 1e-2, (name, l)
    got_logits = f16(t.download("logits", cfg["vocab_size"]))
    want_logits = f16(o.buffer("logits", cfg["vocab_size"]))
    assert rel_l2(got_logits, want_logits) <= 1e-2
    assert t.token(n_prompt) == o.tokens(n_prompt + 1)[n_prompt]
    # decoding continues from the prefilled state and keeps matching the oracle
    for i in range(8):
        ctx.sync()
        t.forward(True, False, A.SCHEDULE_FUSED)
        o.forward(True)
    ctx.sync()
    assert [t.token(i) for i in range(n_prompt + 9)] == o.tokens(n_prompt + 9)
    t.close()
    o.close()


def test_prefill_in_two_parts_equals_one(ctx):
    """A prompt consumed as prefill(40) + prefill(30) leaves the same state as prefill(70)."""
    img = synth.make_model_image(CFG, seed=32)
    prompt = synth.prompt_tokens(32, 70, CFG["vocab_size"])
    kv = CFG["n_layers"] * CFG["seq_len"] * CFG["dim"]
    states = []
    for parts in ((70,), (40, 30)):
        t = A.Transformer(ctx, image=img)
        t.reset(prompt)
        for i, n in enumerate(parts):
            t.prefill(n, gen_token=(i == len(parts) - 1))
        ctx.sync()
        states.append((t.download("key_cache", kv), t.download("value_cache", kv), t.download("logits", CFG["vocab_size"]), t.pos, t.token(70)))
        t.close()
    a, b = states
    assert a[3] == b[3] == 70 and a[4] == b[4]
    assert rel_l2(f16(a[0]), f16(b[0])) <= 1e-3 and rel_l2(f16(a[1]), f16(b[1])) <= 1e-3 and rel_l2(f16(a[2]), f16(b[2])) <= 2e-3


# 128-wide heads and a context past what the batched attention keeps in LDS (1920 positions): the tokens beyond that bound
# go through the matrix-vector path one at a time inside the same call (position hand-over, token list, the
# position-split attention from 1024 positions on).
CFG_LONG2K = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=512, seq_len=2176, rope_theta=10000.0)


# the same with grouped queries: four heads share one KV head (the position-split attention and the single QKV launch
# with fewer K and V rows, at long context)
CFG_LONG2K_GQA = dict(dim=512, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=1, vocab_size=512, seq_len=2176, rope_theta=10000.0)


@pytest.mark.parametrize("cfg", [CFG_LONG2K, CFG_LONG2K_GQA], ids=["2-heads", "grouped-queries"])
def test_prefill_past_the_batched_attention_bound(ctx, cfg):
    n_prompt = 2000
    img = synth.make_model_image(cfg, seed=33, scale_mult=0.5)
    prompt = synth.prompt_tokens(33, n_prompt, cfg["vocab_size"])
    o = oracle.Model(img)
    o.reset(prompt)
    for i in range(n_prompt):
        o.forward(i >= n_prompt - 1)
    kv_dim, L, seq, vocab = cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"], cfg["n_layers"], cfg["seq_len"], cfg["vocab_size"]
    want_kv = {n: f16(o.buffer(n, L * seq * kv_dim)).reshape(L, seq, kv_dim)[:, :n_prompt].copy() for n in ("key_cache", "value_cache")}
    want_logits = f16(o.buffer("logits", vocab)).copy()
    want_next = o.tokens(n_prompt + 1)[n_prompt]

    def state(t):
        ctx.sync()
        kv = {n: f16(t.download(n, L * seq * kv_dim)).reshape(L, seq, kv_dim)[:, :n_prompt] for n in ("key_cache", "value_cache")}
        return kv, f16(t.download("logits", vocab)), t.token(n_prompt), t.pos

    results = {}
    for name, parts in (("one call", (2000,)), ("1900 + 100", (1900, 100)), ("token by token", None)):
        t = A.Transformer(ctx, image=img)
        t.reset(prompt)
        if parts is None:
            for i in range(n_prompt):
                t.forward(i >= n_prompt - 1, False, A.SCHEDULE_FUSED)
        else:
            for i, n in enumerate(parts):
                t.prefill(n, gen_token=(i == len(parts) - 1))
        results[name] = state(t)
        kv, logits, nxt, pos = results[name]
        assert pos == n_prompt, name
        for n in ("key_cache", "value_cache"):
            for l in range(L):
                assert rel_l2(kv[n][l], want_kv[n][l]) <= 1e-2, (name, n, l)
                # the rows written one at a time past the bound, on their own
                assert rel_l2(kv[n][l][1920:], want_kv[n][l][1920:]) <= 1e-2, (name, n, l)
        assert rel_l2(logits, want_logits) <= 1e-2, name
        assert nxt == want_next, name
        # decoding continues from there
        for i in range(4):
            ctx.sync()
            t.forward(True, False, A.SCHEDULE_FUSED)
        ctx.sync()
        assert t.pos == n_prompt + 4
        results[name] += ([t.token(n_prompt + 1 + i) for i in range(4)],)
        t.close()
    for i in range(4):
        o.forward(True)
    want_more = o.tokens(n_prompt + 5)[n_prompt + 1 :]
    for name, r in results.items():
        assert r[4] == want_more, name
    o.close()
