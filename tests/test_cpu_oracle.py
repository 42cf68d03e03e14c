"""CPU tests that pin the oracle (oracle/awq_oracle.cpp) without any reference execution.

Each oracle function is checked against something independent of its own code: numpy restatements written from the
layout / formula definitions, fp64 closed forms, invariants and brute force on small inputs.
"""
import numpy as np
import pytest

from llama_cu_awq_amd import synth
from oracle import oracle
from tests.helpers import f16, rel_l2, ulp_diff_f16


# ---------------------------------------------------------------- fp16 conversions
def test_half_to_float_all_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got_hw = np.array([oracle.lib.orc_half_to_float(int(b)) for b in bits[::7]], dtype=np.float32)
    got_sw = np.array([oracle.lib.orc_half_to_float_sw(int(b)) for b in bits], dtype=np.float32)
    assert np.array_equal(got_sw.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got_sw[np.isnan(want)]).all()
    w7 = want[::7]
    assert np.array_equal(got_hw.view(np.uint32)[~np.isnan(w7)], w7.view(np.uint32)[~np.isnan(w7)])


def test_float_to_half_rne_against_numpy():
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.normal(0, 1, 20000), rng.normal(0, 1e-4, 5000), rng.normal(0, 3e4, 5000),
        # exact ties between adjacent halves, subnormal region, overflow boundary
        np.array([1.0 + 2**-11, 1.0 + 3 * 2**-11, 2**-24, 2**-25, 1.5 * 2**-25, 65504.0, 65519.9, 65520.0, 1e6, -0.0, 0.0, 6.1e-5, 5.96e-8]),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got_hw = np.array([oracle.lib.orc_float_to_half(float(v)) for v in vals], dtype=np.uint16)
    got_sw = np.array([oracle.lib.orc_float_to_half_sw(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got_hw, want)
    assert np.array_equal(got_sw, want)


# ---------------------------------------------------------------- layout
@pytest.mark.parametrize("K,N", [(128, 8), (256, 16), (1056, 24), (4096, 64), (11008, 8), (200, 8)])
def test_dequant_matches_layout_definition(K, N):
    w, z, s = synth.make_qweight(synth.stream_key(11, K, N), K, N)
    got = oracle.dequant(w, z, s, K, N).view(np.uint16)
    # numpy restatement from the layout: element k in nibble k%8 of dword k/8; group k/128; single rounding of the exact product
    want = synth.dequantize(w, z, s, K).astype(np.float32).astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_pack_unpack_round_trip_and_bit_positions():
    rng = np.random.default_rng(1)
    q = rng.integers(0, 16, size=(5, 40), dtype=np.uint8)
    p = synth.pack_nibbles(q, 5)
    assert np.array_equal(synth.unpack_nibbles(p, 40), q)
    # element 9 of a row sits in bits 4..7 of dword 1
    one = np.zeros((1, 16), dtype=np.uint8)
    one[0, 9] = 0xA
    assert synth.pack_nibbles(one, 2)[0, 1] == 0xA << 4 and synth.pack_nibbles(one, 2)[0, 0] == 0


def test_dequant_single_weight_by_hand():
    """One non-zero nibble: w[n=1][k=130] = (q - z) * s with z, s of group 1."""
    K, N = 256, 2
    pwh, pzh, sh = synth.strides(K)
    w = np.zeros((N, pwh), dtype=np.uint32)
    z = np.zeros((N, pzh), dtype=np.uint32)
    s = np.zeros((N, sh), dtype=np.float16)
    w[1, 130 // 8] = 13 << (4 * (130 % 8))
    z[1, 0] = 5 << 4  # group 1 -> nibble 1
    s[1, 1] = 0.0123
    d = oracle.dequant(w, z, s, K, N)
    assert d[1, 130] == np.float16(np.float32(8) * np.float32(np.float16(0.0123)))
    assert d[1, 129] == np.float16(np.float32(-5) * np.float32(np.float16(0.0123)))  # q = 0 elsewhere in group 1
    assert not d[0].any() and not d[1, :128].any()  # scale 0 in group 0


# ---------------------------------------------------------------- int4 matvec family
@pytest.mark.parametrize("K,N", [(128, 8), (1024, 16), (1056, 8), (4096, 128), (11008, 32), (6656, 16)])
def test_matvec_int4_vs_fp64(K, N):
    w, z, s = synth.make_qweight(synth.stream_key(12, K, N), K, N)
    x = synth.normal_f16(synth.stream_key(12, "x", K), K)
    out = np.zeros(N, dtype=np.uint16)
    assert oracle.matvec_int4(out, x, w, z, s, K, N) == 0
    truth = synth.dequantize(w, z, s, K) @ x.astype(np.float64)
    got = f16(out).astype(np.float64)
    # fp32 accumulation then one fp16 rounding: half an fp16 step plus ~1e-6 of the magnitude
    assert np.all(np.abs(got - truth) <= np.abs(truth) * 2**-11 + 2e-5 * np.sqrt(K))
    assert rel_l2(got, truth) <= 4e-4


def test_matvec_int4_epilogues():
    K, N = 256, 16
    w, z, s = synth.make_qweight(synth.stream_key(13), K, N)
    x = synth.normal_f16(synth.stream_key(13, "x"), K)
    truth = synth.dequantize(w, z, s, K) @ x.astype(np.float64)
    resid = synth.normal_f16(synth.stream_key(13, "r"), N)
    out = resid.view(np.uint16).copy()
    oracle.matvec_int4(out, x, w, z, s, K, N, accum=True, gpu_count=1)
    assert rel_l2(f16(out), truth + resid.astype(np.float64)) <= 1e-3
    out = resid.view(np.uint16).copy()
    oracle.matvec_int4(out, x, w, z, s, K, N, accum=True, gpu_count=4)  # residual pre-divided
    assert rel_l2(f16(out), truth + resid.astype(np.float64) / 4) <= 1e-3
    # KV-cache row offset: exactly N halves written at loff + pos*N
    cache = np.full(6 * N, 0x1234, dtype=np.uint16)
    oracle.matvec_int4(cache, x, w, z, s, K, N, loff=2 * N, pos=3)
    assert (cache[: 5 * N] == 0x1234).all() and rel_l2(f16(cache[5 * N :]), truth) <= 1e-3
    # shape guard: K or N not a multiple of 8
    assert oracle.matvec_int4(np.zeros(16, np.uint16), x, w, z, s, 12, 16) == -1
    assert oracle.matvec_int4(np.zeros(16, np.uint16), x, w, z, s, 256, 12) == -1


def test_zero_weights_accum_is_identity():
    K, N = 256, 8
    pwh, pzh, sh = synth.strides(K)
    w = np.full((N, pwh), 0x77777777, dtype=np.uint32)
    z = np.full((N, pzh), 0x77777777, dtype=np.uint32)
    s = np.full((N, sh), 0.01, dtype=np.float16)
    x = synth.normal_f16(synth.stream_key(14), K)
    resid = synth.normal_f16(synth.stream_key(14, "r"), N)
    out = resid.view(np.uint16).copy()
    oracle.matvec_int4(out, x, w, z, s, K, N, accum=True)
    assert np.array_equal(out, resid.view(np.uint16))


def test_qkv_and_ffn_vs_fp64():
    K, N = 512, 64
    mats = [synth.make_qweight(synth.stream_key(15, i), K, N) for i in range(3)]
    x = synth.normal_f16(synth.stream_key(15, "x"), K)
    xd = x.astype(np.float64)
    q = np.zeros(N, np.uint16)
    kc = np.zeros(4 * N, np.uint16)
    vc = np.zeros(4 * N, np.uint16)
    assert oracle.qkv_matvec(q, kc, vc, x, *mats, K, N, N, 2) == 0
    assert rel_l2(f16(q), synth.dequantize(*mats[0], K) @ xd) <= 1e-3
    assert rel_l2(f16(kc[3 * N :]), synth.dequantize(*mats[1], K) @ xd) <= 1e-3
    assert rel_l2(f16(vc[3 * N :]), synth.dequantize(*mats[2], K) @ xd) <= 1e-3
    assert not kc[: 3 * N].any() and not vc[: 3 * N].any()
    out = np.zeros(N, np.uint16)
    assert oracle.ffn_matvec_silu(out, x, mats[0], mats[1], K, N) == 0
    g = synth.dequantize(*mats[0], K) @ xd
    u = synth.dequantize(*mats[1], K) @ xd
    assert rel_l2(f16(out), g / (1 + np.exp(-g)) * u) <= 1e-3
    # gate and up are not interchangeable (silu is applied to the first matrix)
    out2 = np.zeros(N, np.uint16)
    oracle.ffn_matvec_silu(out2, x, mats[1], mats[0], K, N)
    assert rel_l2(f16(out2), u / (1 + np.exp(-u)) * g) <= 1e-3 and not np.array_equal(out, out2)


# ---------------------------------------------------------------- fp16 ops
@pytest.mark.parametrize("size", [8, 100, 1024, 4096, 5000])
def test_rmsnorm_closed_form(size):
    x = synth.normal_f16(synth.stream_key(16, size), size, 0, 3.0)
    w = synth.normal_f16(synth.stream_key(16, "w", size), size, 1.0, 0.05)
    got = oracle.rmsnorm(x, w).astype(np.float64)
    xd = x.astype(np.float64)
    truth = xd / np.sqrt((xd * xd).mean() + 1e-5) * w.astype(np.float64)
    assert rel_l2(got, truth) <= 4e-4
    # w = 1, x = c  ->  c / sqrt(c^2 + 1e-5)
    c = np.full(size, 0.5, dtype=np.float16)
    got = oracle.rmsnorm(c, np.ones(size, dtype=np.float16)).astype(np.float64)
    assert np.allclose(got, 0.5 / np.sqrt(0.25 + 1e-5), rtol=1e-3)
    # scale equivariance: norm(2x) == norm(x) up to rounding (eps negligible)
    a = oracle.rmsnorm(x, w).astype(np.float64)
    b = oracle.rmsnorm((x.astype(np.float32) * 2).astype(np.float16), w).astype(np.float64)
    assert rel_l2(a, b) <= 1e-3


@pytest.mark.parametrize("heads,kv_heads,head,pos", [(4, 4, 128, 0), (4, 4, 128, 7), (8, 2, 64, 100), (2, 2, 256, 2047)])
def test_rope_closed_form(heads, kv_heads, head, pos):
    q = synth.normal_f16(synth.stream_key(17, heads, pos), heads * head)
    seq = pos + 1
    kc = synth.normal_f16(synth.stream_key(17, "k", heads, pos), seq * kv_heads * head)
    q_bits, k_bits = q.view(np.uint16).copy(), kc.view(np.uint16).copy()
    oracle.rope(q_bits, k_bits, heads, kv_heads, head, pos, 0, 10000.0)
    i = np.arange(head // 2)
    ang = pos * (1.0 / np.power(10000.0, 2.0 * i / head))

    def rot(v):  # pairs (i, i + head/2)
        a, b = v[..., : head // 2], v[..., head // 2 :]
        return np.concatenate([a * np.cos(ang) - b * np.sin(ang), a * np.sin(ang) + b * np.cos(ang)], axis=-1)

    tol = 2e-3 if pos > 1000 else 6e-4  # float32 angle at large positions
    assert rel_l2(f16(q_bits), rot(q.astype(np.float64).reshape(heads, head)).reshape(-1)) <= tol
    krow = kc.astype(np.float64).reshape(seq, kv_heads, head)[pos]
    assert rel_l2(f16(k_bits).reshape(seq, kv_heads, head)[pos].reshape(-1), rot(krow).reshape(-1)) <= tol
    assert np.array_equal(k_bits[: pos * kv_heads * head], kc.view(np.uint16)[: pos * kv_heads * head])  # other rows untouched
    if pos == 0:
        assert np.array_equal(q_bits, q.view(np.uint16))  # identity
    # rotation preserves the norm of each pair
    qq = f16(q_bits).astype(np.float64).reshape(heads, head)
    q0 = q.astype(np.float64).reshape(heads, head)
    n_new = qq[:, : head // 2] ** 2 + qq[:, head // 2 :] ** 2
    n_old = q0[:, : head // 2] ** 2 + q0[:, head // 2 :] ** 2
    assert np.allclose(n_new, n_old, rtol=5e-3, atol=1e-4)


@pytest.mark.parametrize("heads,head,kv_mul,pos", [(4, 128, 1, 0), (4, 128, 1, 33), (8, 64, 4, 200), (2, 256, 1, 1100)])
def test_attention_brute_force(heads, head, kv_mul, pos):
    kv_dim = heads * head // kv_mul
    seq = pos + 1
    key = synth.stream_key(18, heads, head, pos)
    q = synth.normal_f16(synth.stream_key(key, "q"), heads * head)
    kc = synth.normal_f16(synth.stream_key(key, "k"), seq * kv_dim)
    vc = synth.normal_f16(synth.stream_key(key, "v"), seq * kv_dim)
    out, att = oracle.attention(q, kc.view(np.uint16), vc.view(np.uint16), heads, head, kv_mul, pos)
    Q = q.astype(np.float64).reshape(heads, head)
    Kc = kc.astype(np.float64).reshape(seq, heads // kv_mul, head)
    Vc = vc.astype(np.float64).reshape(seq, heads // kv_mul, head)
    for h in range(heads):
        sc = Kc[:, h // kv_mul, :] @ Q[h] / np.sqrt(head)
        p = np.exp(sc - sc.max())
        p /= p.sum()
        assert rel_l2(out.reshape(heads, head)[h], p @ Vc[:, h // kv_mul, :]) <= 5e-3
        assert np.allclose(att[h].astype(np.float64), p, atol=2e-3)
        assert abs(att[h].astype(np.float64).sum() - 1) <= 5e-3
    if pos == 0:
        # one position: probability 1, so every head returns its KV head's value row bit for bit
        want = np.repeat(vc.view(np.uint16).reshape(heads // kv_mul, head), kv_mul, axis=0).reshape(-1)
        assert np.array_equal(out.view(np.uint16), want)


def test_attention_identical_keys_give_uniform_probabilities():
    heads, head, pos = 2, 64, 9
    q = synth.normal_f16(synth.stream_key(19, "q"), heads * head)
    krow = synth.normal_f16(synth.stream_key(19, "k"), heads * head)
    kc = np.tile(krow, pos + 1)
    vc = synth.normal_f16(synth.stream_key(19, "v"), (pos + 1) * heads * head)
    out, att = oracle.attention(q, kc.view(np.uint16), vc.view(np.uint16), heads, head, 1, pos)
    assert np.allclose(att.astype(np.float64), 0.1, atol=1e-4)
    assert rel_l2(out, vc.astype(np.float64).reshape(pos + 1, heads * head).mean(axis=0)) <= 2e-3


@pytest.mark.parametrize("n,d", [(8, 8), (264, 16), (4096, 64)])
def test_matvec_f16_vs_fp64(n, d):
    w = synth.normal_f16(synth.stream_key(20, n, d), n * d, 0, 0.05)
    x = synth.normal_f16(synth.stream_key(20, "x", n), n)
    r, got = oracle.matvec_f16(x, w, n, d)
    assert r == 0
    assert rel_l2(got, w.astype(np.float64).reshape(d, n) @ x.astype(np.float64)) <= 5e-4
    assert oracle.matvec_f16(x, w, 12, 8)[0] == -1


def test_argmax_lowest_index_on_ties_and_position_advance():
    logits = np.array([1.0, 5.0, -2.0, 5.0, 3.0, 5.0, 0.0, 1.0], dtype=np.float16)
    tokens = np.full(8, -1, dtype=np.int32)
    ph = np.array([2], dtype=np.int32)
    pd = np.array([2], dtype=np.int32)
    assert oracle.argmax_advance(logits, tokens, ph, pd, True) == 1
    assert ph[0] == 3 and pd[0] == 3 and tokens[3] == 1
    assert oracle.argmax_advance(logits, tokens, ph, pd, False) == 1  # prompt phase: advance only
    assert ph[0] == 4 and tokens[4] == -1
    rng = np.random.default_rng(3)
    big = rng.normal(0, 1, 32000).astype(np.float16)
    assert oracle.argmax_advance(big, np.zeros(4, np.int32), np.array([0], np.int32), np.array([0], np.int32), False) == int(np.argmax(big.astype(np.float32)))


# ---------------------------------------------------------------- schedule and decode loop
TOY = dict(dim=128, hidden_dim=256, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=64, seq_len=16, rope_theta=10000.0)


def _views(img, cfg):
    """Split an image into tensors by the documented file order (independent of the oracle's own parser)."""
    dim, hid, V = cfg["dim"], cfg["hidden_dim"], cfg["vocab_size"]
    off = 32

    def take(nbytes, dtype):
        nonlocal off
        a = img[off : off + nbytes].view(dtype)
        off += nbytes
        return a

    def qw(K, N):
        pwh, pzh, sh = synth.strides(K)
        return (take(N * pwh * 4, np.uint32).reshape(N, pwh), take(N * pzh * 4, np.uint32).reshape(N, pzh), take(N * sh * 2, np.float16).reshape(N, sh))

    t = {"embed": take(V * dim * 2, np.float16), "wcls": take(V * dim * 2, np.float16), "final": take(dim * 2, np.float16), "layers": []}
    for _ in range(cfg["n_layers"]):
        L = {}
        for name, K, N in (("q", dim, dim), ("k", dim, dim), ("v", dim, dim), ("o", dim, dim), ("up", dim, hid), ("gate", dim, hid), ("down", hid, dim)):
            L[name] = qw(K, N)
        L["rms_att"] = take(dim * 2, np.float16)
        L["rms_ffn"] = take(dim * 2, np.float16)
        t["layers"].append(L)
    assert off == img.nbytes
    return t


def test_forward_is_the_documented_schedule():
    """orc_model_forward == the op sequence of run_llama_network composed by hand from the single ops, bit for bit."""
    cfg = TOY
    img = synth.make_model_image(cfg, seed=21, threads=1)
    t = _views(img, cfg)
    dim, hid, heads, head, seq = cfg["dim"], cfg["hidden_dim"], cfg["n_heads"], cfg["dim"] // cfg["n_heads"], cfg["seq_len"]
    m = oracle.Model(img)
    prompt = [5, 9, 33]
    m.reset(prompt)
    kc = np.zeros(cfg["n_layers"] * seq * dim, np.uint16)
    vc = np.zeros(cfg["n_layers"] * seq * dim, np.uint16)
    tokens = list(prompt) + [0] * 8
    for pos in range(5):
        x = t["embed"].reshape(-1, dim)[tokens[pos]].copy()
        for l, L in enumerate(t["layers"]):
            xb = oracle.rmsnorm(x, L["rms_att"])
            loff = l * seq * dim
            q = np.zeros(dim, np.uint16)
            oracle.qkv_matvec(q, kc, vc, xb, L["q"], L["k"], L["v"], dim, dim, loff, pos)
            oracle.rope(q, kc, heads, heads, head, pos, loff, 10000.0)
            att_out, _ = oracle.attention(f16(q), kc[loff : loff + seq * dim], vc[loff : loff + seq * dim], heads, head, 1, pos)
            xa = x.view(np.uint16).copy()
            oracle.matvec_int4(xa, att_out, *L["o"], dim, dim, accum=True)
            x = f16(xa)
            xb = oracle.rmsnorm(x, L["rms_ffn"])
            hb = np.zeros(hid, np.uint16)
            oracle.ffn_matvec_silu(hb, xb, L["gate"], L["up"], dim, hid)
            xa = x.view(np.uint16).copy()
            oracle.matvec_int4(xa, f16(hb), *L["down"], hid, dim, accum=True)
            x = f16(xa)
        x = oracle.rmsnorm(x, t["final"])
        _, logits = oracle.matvec_f16(x, t["wcls"], dim, cfg["vocab_size"])
        gen = pos >= len(prompt) - 1
        tok = m.forward(gen)
        assert np.array_equal(m.buffer("logits", cfg["vocab_size"]), logits.view(np.uint16)), pos
        assert tok == int(np.argmax(logits.astype(np.float32)))
        if gen:
            tokens[pos + 1] = tok
        assert m.tokens(pos + 2)[: pos + 2] == tokens[: pos + 2]
    m.close()


def test_decode_loop_state_machine():
    cfg = TOY
    img = synth.make_model_image(cfg, seed=22, threads=1)
    m = oracle.Model(img)
    prompt = [7, 8, 9, 10]
    toks, pos, logits = m.generate(prompt, 12, ignore_eos=True, want_logits=True)
    assert pos == 12 and toks[:4] == prompt and len(toks) == 13
    # every generated token is the argmax of the logits of the step before it
    for p in range(3, 12):
        assert toks[p + 1] == int(np.argmax(logits[p].astype(np.float32)))
    # steps shorter than the prompt: only prompt tokens are echoed
    toks, pos, _ = m.generate(prompt, 2, ignore_eos=True)
    assert pos == 2 and toks[:3] == prompt[:3]
    # EOS (2) read back at position p stops the loop with pos == p
    toks, pos, _ = m.generate([5, 6, 2, 11], 10)
    assert pos == 2
    # deterministic
    a = m.generate(prompt, 12, ignore_eos=True)[0]
    b = m.generate(prompt, 12, ignore_eos=True)[0]
    assert a == b
    m.close()


def test_model_open_rejects_short_image():
    img = synth.make_model_image(TOY, seed=23, threads=1)
    with pytest.raises(ValueError):
        oracle.Model(img[:1000])
