"""GPU parity: every op of the C-ABI against the CPU oracle and against fp64 closed forms.

Tolerances: unpack/dequant bit-exact; matrix-vector outputs rel-L2 <= 1e-3 of the fp64 product of the exactly
dequantised weights (the stated bound) and, tighter, within 2 fp16 steps of the oracle's fp32 restatement
(summation order differs); fp16 element-wise ops within 1 fp16 step of the oracle.
"""
import ctypes as C
import functools

import numpy as np
import pytest

import llama_cu_awq_amd as A
from llama_cu_awq_amd import synth
from llama_cu_awq_amd._lib import AWQ_ERR_SHAPE, lib
from oracle import oracle
from tests.helpers import assert_close_f16, f16, rel_l2, ulp_diff_f16

pytestmark = pytest.mark.gpu

SHAPES = [(4096, 4096), (4096, 11008), (11008, 4096), (5120, 5120), (13824, 5120), (6656, 1024), (17920, 512), (128, 8), (200, 24), (1056, 40),
          (53248, 4608)]  # the last: rows so long that one workgroup per compute unit walks the row groups (288 groups on 256 units)


@functools.lru_cache(maxsize=16)
def _case(K, N, tag=0):
    key = synth.stream_key(0, "case", K, N, tag)
    w, z, s = synth.make_qweight(key, K, N)
    x = synth.normal_f16(synth.stream_key(key, "x"), K)
    for a in (w, z, s, x):
        a.setflags(write=False)  # shared between the tests that ask for the same case
    return w, z, s, x


@functools.lru_cache(maxsize=6)
def _exact(K, N, tag):
    """The exactly dequantised matrix of _case(K, N, tag) in fp64 (kept across the parametrisations that reuse it)."""
    w, z, s, _ = _case(K, N, tag)
    m = synth.dequantize(w, z, s, K)
    m.setflags(write=False)
    return m


@pytest.mark.parametrize("K,N", [(4096, 512), (11008, 64), (200, 24), (128, 8), (13824, 32)])
def test_dequant_bit_exact(ctx, K, N):
    w, z, s, _ = _case(K, N)
    qw = A.QWeight.upload(ctx, w, z, s)
    out = ctx.alloc(N * K * 2)
    A.dequant(ctx, out, qw, K, N)
    got = out.download(np.uint16).reshape(N, K)
    want = oracle.dequant(w, z, s, K, N).view(np.uint16)
    assert np.array_equal(got, want)
    # and against the layout definition in numpy (single rounding of the exact product)
    ref = synth.dequantize(w, z, s, K).astype(np.float32).astype(np.float16).view(np.uint16)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("K,N", SHAPES)
def test_matvec_int4_plain(ctx, K, N):
    w, z, s, x = _case(K, N)
    qw = A.QWeight.upload(ctx, w, z, s)
    dx = ctx.upload(x)
    dout = ctx.zeros(N * 2)
    A.matmul_q(ctx, dout, dx, qw, K, N)
    got = f16(dout.download(np.uint16))
    truth = synth.dequantize(w, z, s, K) @ x.astype(np.float64)
    assert rel_l2(got, truth) <= 1e-3
    want = np.zeros(N, dtype=np.uint16)
    assert oracle.matvec_int4(want, x, w, z, s, K, N) == 0
    assert_close_f16(got, f16(want), ulps=2)
    assert rel_l2(got, f16(want)) <= 3e-4
    # How good the fp32 sum is before the one rounding to fp16: the share of outputs that are not the correctly rounded
    # exact result.  The reference's sequential fp32 order misses 0.1 - 0.3 % of them; an accumulation that drops low
    # bits shows up here long before it shows in rel-L2 (4.6 % with the nibbles taken as denormals in bits 3..0, whose
    # products v_dot2_f32_f16 adds in a window anchored 6 - 10 bits too high).
    if N >= 512:
        best = truth.astype(np.float16)
        assert (got != best).mean() <= max(2 * (f16(want) != best).mean(), 4e-3)


# ---- shapes chosen to reach every branch of the launch geometry (waves per workgroup 4 / 8 / 10 / 13 / 16, one, two or
# four rows side by side in a wave, two or three passes in flight, partly filled last workgroups and row groups, row
# lengths that are no multiple of a pass or of a quantisation group), in the three forms.
SWEEP_K = [8, 96, 136, 256, 512, 544, 1000, 2560, 2592, 3072, 4096, 5120, 6144, 6656, 8192, 8224, 10240, 11008, 13824, 17920, 20480,
           28672, 28704, 53248, 65536]  # the last three: more than 64 KB of LDS per workgroup
SWEEP_N = [8, 40, 264, 1000]


@pytest.mark.parametrize("K", SWEEP_K)
def test_matvec_int4_shape_sweep(ctx, K):
    for N in SWEEP_N + ([5120] if K in (5120, 13824) else []) + ([6656] if K in (6656, 17920) else []):
        w, z, s, x = _case(K, N, 7)
        truth = synth.dequantize(w, z, s, K) @ x.astype(np.float64)
        qw = A.QWeight.upload(ctx, w, z, s)
        dx = ctx.upload(x)
        # single matrix, with the residual added
        resid = synth.normal_f16(synth.stream_key(7, "res", K, N), N)
        dout = ctx.upload(resid)
        A.matmul_q(ctx, dout, dx, qw, K, N, accum=True)
        got = f16(dout.download(np.uint16))
        want = resid.view(np.uint16).copy()
        oracle.matvec_int4(want, x, w, z, s, K, N, accum=True)
        assert_close_f16(got, f16(want), ulps=2)
        assert rel_l2(got, truth + resid.astype(np.float64)) <= 1e-3, ("single", K, N)
        # the three-matrix form (the same matrix three times: q, and one row each of the two caches)
        pos, loff, rows = 1, N, 3
        dq, dk, dv = ctx.zeros(N * 2), ctx.zeros(rows * N * 2), ctx.zeros(rows * N * 2)
        dpos = ctx.upload(np.array([pos], dtype=np.int32))
        A.qkv_matvec(ctx, dq, dk, dv, dx, qw, qw, qw, K, N, loff, dpos)
        plain = np.zeros(N, dtype=np.uint16)
        oracle.matvec_int4(plain, x, w, z, s, K, N)
        for buf, off in ((dq, 0), (dk, loff + pos * N), (dv, loff + pos * N)):
            g = buf.download(np.uint16)
            assert_close_f16(f16(g[off : off + N]), f16(plain), ulps=2)
            assert not g[:off].any() and not g[off + N :].any(), ("qkv", K, N)
        # gate/up with SiLU (the matrix against a second one)
        w2, z2, s2, _ = _case(K, N, 8)
        qw2 = A.QWeight.upload(ctx, w2, z2, s2)
        xs = (x.astype(np.float32) * np.float32(0.25)).astype(np.float16)  # keeps SiLU(g) * u inside fp16 at the long rows
        dh = ctx.zeros(N * 2)
        A.ffn_matvec_silu(ctx, dh, ctx.upload(xs), qw, qw2, K, N)
        hw = np.zeros(N, dtype=np.uint16)
        oracle.ffn_matvec_silu(hw, xs, (w, z, s), (w2, z2, s2), K, N)
        gh, hw = f16(dh.download(np.uint16)), f16(hw)
        assert np.isfinite(hw.astype(np.float32)).all()
        assert rel_l2(gh, hw) <= 1e-3, ("ffn", K, N)
        assert_close_f16(gh, hw, ulps=4)


# ---- activations far from unit magnitude.  The reference multiplies (q - z) * s * x in fp32 whatever the size of x
# (gpu_kernels.h:203-207), so a vector that is small as a whole (the attention output in front of the O projection,
# SiLU(gate) * up in front of the down projection) must come out as accurately as a vector of order one.  The scaled
# vectors are exact multiples of the N(0,1) one until elements fall into the fp16 denormal range (2^-14 takes most of them
# there: those are then inputs in their own right, with few significant bits).
X_SCALES = [-8, -12, -14, 8]


def _scaled(x, e):
    return (x.astype(np.float32) * np.float32(2.0**e)).astype(np.float16)


def _fp16_rounding_floor(truth):
    """rel-L2 that rounding the exact result to fp16 costs by itself (large only where outputs are fp16 denormals)."""
    with np.errstate(over="ignore"):
        return rel_l2(truth.astype(np.float16), truth)


@pytest.mark.parametrize("e", X_SCALES)
@pytest.mark.parametrize("K,N", [(4096, 4096), (11008, 4096)])
def test_matvec_int4_scaled_activations(ctx, K, N, e):
    w, z, s, x = _case(K, N, 30)
    x = _scaled(x, e)
    qw = A.QWeight.upload(ctx, w, z, s)
    dout = ctx.zeros(N * 2)
    A.matmul_q(ctx, dout, ctx.upload(x), qw, K, N)
    got = f16(dout.download(np.uint16))
    truth = _exact(K, N, 30) @ x.astype(np.float64)
    floor = _fp16_rounding_floor(truth)
    assert floor <= 5e-4  # the outputs are representable: the stated bound applies as it is
    assert rel_l2(got, truth) <= 1e-3
    assert rel_l2(got, truth) <= floor + 1.5e-4  # and nearly all of it is the output's own rounding
    want = np.zeros(N, dtype=np.uint16)
    assert oracle.matvec_int4(want, x, w, z, s, K, N) == 0
    assert_close_f16(got, f16(want), ulps=2)
    # residual form: the product must survive next to a residual of its own size
    resid = _scaled(synth.normal_f16(synth.stream_key(30, "res", K), N), e + 2)
    dout = ctx.upload(resid)
    A.matmul_q(ctx, dout, ctx.upload(x), qw, K, N, accum=True)
    want = resid.view(np.uint16).copy()
    oracle.matvec_int4(want, x, w, z, s, K, N, accum=True)
    assert_close_f16(f16(dout.download(np.uint16)), f16(want), ulps=2)


@pytest.mark.parametrize("e", X_SCALES)
@pytest.mark.parametrize("K,N", [(4096, 4096), (11008, 4096)])
def test_qkv_matvec_scaled_activations(ctx, K, N, e):
    mats = [_case(K, N, t)[:3] for t in (31, 32, 33)]
    x = _scaled(_case(K, N, 34)[3], e)
    qws = [A.QWeight.upload(ctx, *m) for m in mats]
    pos, loff, rows = 1, 0, 2
    dq, dk, dv = ctx.zeros(N * 2), ctx.zeros(rows * N * 2), ctx.zeros(rows * N * 2)
    dpos = ctx.upload(np.array([pos], dtype=np.int32))
    A.qkv_matvec(ctx, dq, dk, dv, ctx.upload(x), *qws, K, N, loff, dpos)
    q = np.zeros(N, dtype=np.uint16)
    kc = np.zeros(rows * N, dtype=np.uint16)
    vc = np.zeros(rows * N, dtype=np.uint16)
    oracle.qkv_matvec(q, kc, vc, x, *mats, K, N, loff, pos)
    for got, want in ((dq.download(np.uint16), q), (dk.download(np.uint16), kc), (dv.download(np.uint16), vc)):
        assert_close_f16(f16(got), f16(want), ulps=2)
    for got, tag in ((dq.download(np.uint16), 31), (dv.download(np.uint16)[pos * N : (pos + 1) * N], 33)):
        truth = _exact(K, N, tag) @ x.astype(np.float64)
        assert rel_l2(f16(got), truth) <= 1e-3


@pytest.mark.parametrize("e", X_SCALES)
@pytest.mark.parametrize("K,N", [(4096, 11008), (11008, 4096)])
def test_ffn_matvec_silu_scaled_activations(ctx, K, N, e):
    """SiLU(g) * u is quadratic in a small x, so below 2^-8 the exact results themselves are fp16 denormals or zero:
    there the comparison is with the oracle in fp16 steps (a step is a denormal quantum), and with fp64 as far as the
    output format allows."""
    gate, up = _case(K, N, 35)[:3], _case(K, N, 36)[:3]
    x = _scaled(_case(K, N, 37)[3], e)
    if e > 0:  # keep the product of two sums inside fp16 range
        x = _scaled(x, -6)
    dout = ctx.zeros(N * 2)
    A.ffn_matvec_silu(ctx, dout, ctx.upload(x), A.QWeight.upload(ctx, *gate), A.QWeight.upload(ctx, *up), K, N)
    got = f16(dout.download(np.uint16))
    want = np.zeros(N, dtype=np.uint16)
    oracle.ffn_matvec_silu(want, x, gate, up, K, N)
    assert np.isfinite(f16(want).astype(np.float32)).all()
    assert_close_f16(got, f16(want), ulps=4)
    xd = x.astype(np.float64)
    g = _exact(K, N, 35) @ xd
    u = _exact(K, N, 36) @ xd
    truth = g / (1.0 + np.exp(-g)) * u
    assert rel_l2(got, truth) <= 1e-3 + _fp16_rounding_floor(truth)


@pytest.mark.parametrize("e", X_SCALES)
@pytest.mark.parametrize("parts", [1, 3])
def test_matvec_int4_parts_scaled_activations(ctx, e, parts):
    """The product whose input arrives as fp32 partial sums (the O projection behind the position-split attention):
    x = half(p0 + p1 + ...) added in part order, then the same arithmetic as the plain product."""
    K = N = 4096
    w, z, s, x = _case(K, N, 38)
    xf = x.astype(np.float32) * np.float32(2.0**e)
    split = np.abs(synth.normal_f16(synth.stream_key(38, "split", parts), parts * K).astype(np.float32).reshape(parts, K)) + 0.125
    p = (split / split.sum(axis=0, keepdims=True) * xf).astype(np.float32)  # positive fractions of every element
    acc = p[0].copy()
    for i in range(1, parts):
        acc = acc + p[i]
    xh = acc.astype(np.float16)
    qw = A.QWeight.upload(ctx, w, z, s)
    resid = _scaled(synth.normal_f16(synth.stream_key(38, "res"), N), e + 2)
    d1, d2 = ctx.upload(resid), ctx.upload(resid)
    A.matmul_q_parts(ctx, d1, ctx.upload(p.reshape(-1)), parts, qw, K, N, accum=True)
    A.matmul_q(ctx, d2, ctx.upload(xh), qw, K, N, accum=True)
    assert np.array_equal(d1.download(np.uint16), d2.download(np.uint16))
    want = resid.view(np.uint16).copy()
    oracle.matvec_int4(want, xh, w, z, s, K, N, accum=True)
    assert_close_f16(f16(d1.download(np.uint16)), f16(want), ulps=2)
    truth = synth.dequantize(w, z, s, K) @ xh.astype(np.float64) + resid.astype(np.float64)
    assert rel_l2(f16(d1.download(np.uint16)), truth) <= 1e-3


@pytest.mark.parametrize("K,N", [(4096, 4096), (5120, 5120), (6656, 264), (416, 40)])  # 64-lane rows; two rows per wave
def test_matvec_int4_accum_and_kv_offset(ctx, K, N):
    w, z, s, x = _case(K, N, 1)
    qw = A.QWeight.upload(ctx, w, z, s)
    dx = ctx.upload(x)
    resid = synth.normal_f16(synth.stream_key(1, "res"), N)
    # residual epilogue: out = half(Wx + out)
    dout = ctx.upload(resid)
    A.matmul_q(ctx, dout, dx, qw, K, N, accum=True, gpu_count=1)
    got = f16(dout.download(np.uint16))
    want = resid.view(np.uint16).copy()
    oracle.matvec_int4(want, x, w, z, s, K, N, accum=True)
    assert_close_f16(got, f16(want), ulps=2)
    truth = synth.dequantize(w, z, s, K) @ x.astype(np.float64) + resid.astype(np.float64)
    assert rel_l2(got, truth) <= 1e-3
    # gpu_count = 2 pre-divides the residual (gpu_kernels.h:237-238)
    dout = ctx.upload(resid)
    A.matmul_q(ctx, dout, dx, qw, K, N, accum=True, gpu_count=2)
    got = f16(dout.download(np.uint16))
    truth = synth.dequantize(w, z, s, K) @ x.astype(np.float64) + resid.astype(np.float64) / 2
    assert rel_l2(got, truth) <= 1e-3
    # KV-cache row epilogue: written at loff + pos*N, nothing else touched
    pos, loff, rows = 3, 2 * N, 8
    cache = np.full(rows * N, 0x3C00, dtype=np.uint16)
    dcache = ctx.upload(cache)
    dpos = ctx.upload(np.array([pos], dtype=np.int32))
    A.matmul_q(ctx, dcache, dx, qw, K, N, loff=loff, pPos=dpos)
    got = dcache.download(np.uint16)
    want = cache.copy()
    oracle.matvec_int4(want, x, w, z, s, K, N, loff=loff, pos=pos)
    assert np.array_equal(got[: loff + pos * N], want[: loff + pos * N])
    assert np.array_equal(got[loff + (pos + 1) * N :], want[loff + (pos + 1) * N :])
    assert_close_f16(f16(got), f16(want), ulps=2)


def test_zero_weights_leave_residual(ctx):
    """accum with W == 0 (q == z everywhere) returns the residual.  The kernel forms sum q*x - z * sum x with each sum
    rounded in fp32 on its own, so W x comes out as fp32 rounding noise (about 1e-7 here) instead of an exact zero:
    the residual comes back bit for bit except where that noise crosses an fp16 rounding boundary (one step)."""
    K, N = 256, 64
    pwh, pzh, sh = synth.strides(K)
    w = np.full((N, pwh), 0x55555555, dtype=np.uint32)
    z = np.full((N, pzh), 0x55555555, dtype=np.uint32)
    s = np.full((N, sh), 0.01, dtype=np.float16)
    x = synth.normal_f16(synth.stream_key(2, "x"), K)
    resid = synth.normal_f16(synth.stream_key(2, "r"), N)
    qw = A.QWeight.upload(ctx, w, z, s)
    dout = ctx.upload(resid)
    A.matmul_q(ctx, dout, ctx.upload(x), qw, K, N, accum=True)
    got = dout.download(np.uint16)
    steps = ulp_diff_f16(f16(got), resid)
    assert steps.max() <= 1 and (steps == 0).mean() >= 0.9
    # W x itself: zero to within fp32 rounding of its two partial sums
    dout = ctx.zeros(N * 2)
    A.matmul_q(ctx, dout, ctx.upload(x), qw, K, N)
    assert np.abs(f16(dout.download(np.uint16)).astype(np.float64)).max() <= 1e-5


@pytest.mark.parametrize("K,N", [(4096, 4096), (5120, 5120), (256, 64), (6656, 6656), (512, 6656)])  # the last two: 10-wave workgroups, the last one partly filled
def test_qkv_matvec(ctx, K, N):
    mats = [_case(K, N, t)[:3] for t in (10, 11, 12)]
    x = _case(K, N, 13)[3]
    qws = [A.QWeight.upload(ctx, *m) for m in mats]
    pos, loff, rows = 2, N, 5
    dq = ctx.zeros(N * 2)
    dk = ctx.zeros(rows * N * 2)
    dv = ctx.zeros(rows * N * 2)
    dpos = ctx.upload(np.array([pos], dtype=np.int32))
    A.qkv_matvec(ctx, dq, dk, dv, ctx.upload(x), *qws, K, N, loff, dpos)
    q = np.zeros(N, dtype=np.uint16)
    kc = np.zeros(rows * N, dtype=np.uint16)
    vc = np.zeros(rows * N, dtype=np.uint16)
    oracle.qkv_matvec(q, kc, vc, x, *mats, K, N, loff, pos)
    for got, want in ((dq.download(np.uint16), q), (dk.download(np.uint16), kc), (dv.download(np.uint16), vc)):
        assert_close_f16(f16(got), f16(want), ulps=2)
    # only the addressed cache row is written
    kgot = dk.download(np.uint16)
    assert not kgot[: loff + pos * N].any() and not kgot[loff + (pos + 1) * N :].any()
    truth = synth.dequantize(*mats[1], K) @ x.astype(np.float64)
    assert rel_l2(f16(kgot[loff + pos * N : loff + (pos + 1) * N]), truth) <= 1e-3


@pytest.mark.parametrize("K,N", [(4096, 11008), (5120, 13824), (6656, 17920), (256, 72), (1024, 4480), (8192, 1024), (2560, 264), (136, 40), (10240, 520)])
def test_rmsnorm_ffn_matvec_silu_equals_the_two_calls(ctx, K, N):
    """The one-launch form of rmsnorm + ffn_matvec_silu (what the fused schedule runs) against the oracle's two steps:
    the normalised vector must be the same fp16 values, so the outputs agree as closely as the plain kernel's do."""
    gate = _case(K, N, 23)[:3]
    up = _case(K, N, 24)[:3]
    x = (_case(K, N, 25)[3].astype(np.float32) * 3.0).astype(np.float16)  # a residual stream, not a normalised vector
    nw = synth.normal_f16(synth.stream_key(1, "nw", K), K, 1.0, 0.02)
    dout = ctx.zeros(N * 2)
    A.rmsnorm_ffn_matvec_silu(ctx, dout, ctx.upload(x), ctx.upload(nw), A.QWeight.upload(ctx, *gate), A.QWeight.upload(ctx, *up), K, N)
    got = f16(dout.download(np.uint16))
    xn = oracle.rmsnorm(x, nw)
    want = np.zeros(N, dtype=np.uint16)
    oracle.ffn_matvec_silu(want, xn, gate, up, K, N)
    xd = xn.astype(np.float64)
    g = synth.dequantize(*gate, K) @ xd
    u = synth.dequantize(*up, K) @ xd
    assert rel_l2(got, g / (1.0 + np.exp(-g)) * u) <= 1e-3
    assert rel_l2(got, f16(want)) <= 3e-4
    # and against the library's own two launches
    dxn, d2 = ctx.zeros(K * 2), ctx.zeros(N * 2)
    A.rmsnorm(ctx, dxn, ctx.upload(x), ctx.upload(nw), K)
    assert ulp_diff_f16(f16(dxn.download(np.uint16)), xn).max() <= 1  # the sum of squares is added in another order
    A.ffn_matvec_silu(ctx, d2, dxn, A.QWeight.upload(ctx, *gate), A.QWeight.upload(ctx, *up), K, N)
    assert_close_f16(got, f16(d2.download(np.uint16)), ulps=2)


@pytest.mark.parametrize("K,N", [(4096, 11008), (5120, 13824), (6656, 1792), (256, 72)])
def test_ffn_matvec_silu(ctx, K, N):
    gate = _case(K, N, 20)[:3]
    up = _case(K, N, 21)[:3]
    x = _case(K, N, 22)[3]
    dout = ctx.zeros(N * 2)
    A.ffn_matvec_silu(ctx, dout, ctx.upload(x), A.QWeight.upload(ctx, *gate), A.QWeight.upload(ctx, *up), K, N)
    got = f16(dout.download(np.uint16))
    want = np.zeros(N, dtype=np.uint16)
    oracle.ffn_matvec_silu(want, x, gate, up, K, N)
    xd = x.astype(np.float64)
    g = synth.dequantize(*gate, K) @ xd
    u = synth.dequantize(*up, K) @ xd
    truth = g / (1.0 + np.exp(-g)) * u
    assert rel_l2(got, truth) <= 1e-3
    assert rel_l2(got, f16(want)) <= 3e-4
    assert_close_f16(got, f16(want), ulps=4)


@pytest.mark.parametrize("K,N", [(12, 8), (8, 12), (4096, 4100), (0, 8), (65568, 8)])
def test_shape_guard(ctx, K, N):
    """The reference prints 'Unsupported matmul size' and exits; the library returns AWQ_ERR_SHAPE."""
    buf = ctx.alloc(1 << 16)
    qw = A.QWeight(buf, buf, buf)
    with pytest.raises(A.AwqError) as e:
        A.matmul_q(ctx, buf, buf, qw, K, N)
    assert e.value.code == AWQ_ERR_SHAPE
    with pytest.raises(A.AwqError):
        A.ffn_matvec_silu(ctx, buf, buf, qw, qw, K, N)
    with pytest.raises(A.AwqError):
        A.matmul(ctx, buf, buf, buf, K, N)


def test_partial_sum_input_guards(ctx):
    """The matrix-vector product that takes its input as fp32 partial sums: 1 to 4 of them, K up to 8192, the usual shape
    rules; the split attention rejects head sizes and head counts it has no kernel for.  Nothing is launched."""
    buf = ctx.alloc(1 << 16)
    qw = A.QWeight(buf, buf, buf)
    for parts, K, N in ((0, 4096, 4096), (5, 4096, 4096), (2, 8192 + 128, 4096), (2, 12, 8), (2, 4096, 4100)):
        with pytest.raises(A.AwqError) as e:
            A.matmul_q_parts(ctx, buf, buf, parts, qw, K, N)
        assert e.value.code == AWQ_ERR_SHAPE, (parts, K, N)
    pos = ctx.upload(np.array([300], dtype=np.int32))
    for heads, head, kv_mul in ((32, 96, 1), (300, 128, 1), (32, 128, 3)):
        with pytest.raises(A.AwqError) as e:
            A.MultiHeadAttention_partial(ctx, buf, buf, buf, buf, buf, heads, head, kv_mul, 512, pos)
        assert e.value.code == AWQ_ERR_SHAPE, (heads, head, kv_mul)


@pytest.mark.parametrize("size", [4096, 5120, 6656, 8, 1000])
def test_rmsnorm(ctx, size):
    x = synth.normal_f16(synth.stream_key(3, "x", size), size, 0.0, 2.0)
    w = synth.normal_f16(synth.stream_key(3, "w", size), size, 1.0, 0.02)
    dx = ctx.upload(x)
    do = ctx.zeros(size * 2)
    A.rmsnorm(ctx, do, dx, ctx.upload(w), size)
    got = f16(do.download(np.uint16))
    want = oracle.rmsnorm(x, w)
    assert_close_f16(got, want, ulps=1)
    xd = x.astype(np.float64)
    truth = xd / np.sqrt((xd * xd).mean() + 1e-5) * w.astype(np.float64)
    assert rel_l2(got, truth) <= 5e-4
    # in place (the final norm of the network runs in place)
    A.rmsnorm(ctx, dx, dx, ctx.upload(w), size)
    assert np.array_equal(dx.download(np.uint16), do.download(np.uint16))


@pytest.mark.parametrize("heads,kv_heads,head,pos", [(32, 32, 128, 0), (32, 32, 128, 17), (8, 2, 64, 2047), (4, 4, 256, 100), (40, 40, 128, 1791)])
def test_rope(ctx, heads, kv_heads, head, pos):
    seq, loff = pos + 2, 0
    q = synth.normal_f16(synth.stream_key(4, "q", heads, pos), heads * head).view(np.uint16).copy()
    kc = synth.normal_f16(synth.stream_key(4, "k", heads, pos), 2 * seq * kv_heads * head).view(np.uint16).copy()
    loff = seq * kv_heads * head
    dq, dk = ctx.upload(q), ctx.upload(kc)
    dpos = ctx.upload(np.array([pos], dtype=np.int32))
    A.RoPERotation(ctx, dq, dk, heads, kv_heads, head, dpos, loff, 10000.0)
    q0, k0 = q.copy(), kc.copy()
    oracle.rope(q, kc, heads, kv_heads, head, pos, loff, 10000.0)
    gq, gk = dq.download(np.uint16), dk.download(np.uint16)
    # device powf may differ from libm's in the last place of freq; at pos ~2000 that moves the angle by ~1e-4,
    # i.e. the outputs by ~1e-4 of |q|: 2 fp16 steps, or 5e-4 of the rms for elements near zero
    if pos == 0:
        assert np.array_equal(gq, q) and np.array_equal(gk, kc)
    else:
        assert_close_f16(f16(gq), f16(q), ulps=2, floor=5e-4)
        assert_close_f16(f16(gk), f16(kc), ulps=2, floor=5e-4)
    if pos == 0:
        assert np.array_equal(gq, q0) and np.array_equal(gk, k0)
    # rows other than the addressed K row are untouched
    row = loff + pos * kv_heads * head
    assert np.array_equal(gk[:row], k0[:row]) and np.array_equal(gk[row + kv_heads * head :], k0[row + kv_heads * head :])
    # fp64 closed form on q
    i = np.arange(head // 2)
    ang = pos * (1.0 / np.power(10000.0, 2.0 * i / head))
    qq = f16(q0).astype(np.float64).reshape(heads, head)
    a, b = qq[:, : head // 2], qq[:, head // 2 :]
    truth = np.concatenate([a * np.cos(ang) - b * np.sin(ang), a * np.sin(ang) + b * np.cos(ang)], axis=1).reshape(-1)
    assert rel_l2(f16(gq), truth) <= (2e-3 if pos > 1000 else 6e-4)


@pytest.mark.parametrize(
    "heads,head,kv_mul,pos,max_seq",
    [(32, 128, 1, 0, 1), (32, 128, 1, 16, 17), (32, 128, 1, 271, 512), (40, 128, 1, 1791, 2048), (8, 64, 4, 300, 301), (4, 256, 2, 1023, 1024), (52, 128, 1, 2047, 2048), (8, 128, 2, 2500, 4096), (8, 64, 4, 700, 1024),
     (8, 128, 2, 9000, 16384),  # beyond the reference's 8192-position shared-memory form (gpu_kernels.h:411-454)
     (64, 128, 8, 300, 512)],
)
def test_attention(ctx, heads, head, kv_mul, pos, max_seq):
    kv_dim = heads * head // kv_mul
    seq = pos + 1
    key = synth.stream_key(5, heads, head, kv_mul, pos)
    q = synth.normal_f16(synth.stream_key(key, "q"), heads * head)
    kc = synth.normal_f16(synth.stream_key(key, "k"), seq * kv_dim)
    vc = synth.normal_f16(synth.stream_key(key, "v"), seq * kv_dim)
    dout = ctx.zeros(heads * head * 2)
    datt = ctx.zeros(heads * max(max_seq, seq) * 2)
    dpos = ctx.upload(np.array([pos], dtype=np.int32))
    A.MultiHeadAttention(ctx, dout, ctx.upload(q), ctx.upload(kc), ctx.upload(vc), datt, heads, head, kv_mul, max_seq, dpos)
    got = f16(dout.download(np.uint16))
    want, _ = oracle.attention(q, kc.view(np.uint16), vc.view(np.uint16), heads, head, kv_mul, pos)
    # fp64 brute force softmax(qK^T/sqrt(d))V
    Q = q.astype(np.float64).reshape(heads, head)
    Kc = kc.astype(np.float64).reshape(seq, heads // kv_mul, head)
    Vc = vc.astype(np.float64).reshape(seq, heads // kv_mul, head)
    truth = np.empty((heads, head))
    for h in range(heads):
        sc = Kc[:, h // kv_mul, :] @ Q[h] / np.sqrt(head)
        p = np.exp(sc - sc.max())
        p /= p.sum()
        truth[h] = p @ Vc[:, h // kv_mul, :]
    # the fp16 rounding of scores and probabilities (reference behaviour) costs ~1e-3 vs fp64
    assert rel_l2(got, truth.reshape(-1)) <= 4e-3
    assert rel_l2(want, truth.reshape(-1)) <= 4e-3
    assert rel_l2(got, want) <= 1.5e-3
    # a second call gives the same bits
    A.MultiHeadAttention(ctx, dout, ctx.upload(q), ctx.upload(kc), ctx.upload(vc), datt, heads, head, kv_mul, max_seq, dpos)
    assert np.array_equal(dout.download(np.uint16), got.view(np.uint16))


@pytest.mark.parametrize(
    "heads,head,kv_mul,pos,max_seq",
    [(32, 128, 1, 256, 257), (32, 128, 1, 271, 512), (40, 128, 1, 1791, 2048), (52, 128, 1, 2047, 2048), (8, 64, 4, 300, 512), (4, 256, 2, 1023, 1024), (32, 128, 1, 2, 512),
     (8, 128, 2, 9000, 16384), (64, 128, 8, 1500, 2048)],  # the last: Llama-2-70B's heads (8 share a KV head), K = 8192 into the O projection
)
def test_attention_split_over_positions_then_o_projection(ctx, heads, head, kv_mul, pos, max_seq):
    """The long-context form of the fused schedule: P.V as fp32 partial sums per range of positions, added up and
    rounded to fp16 inside the O projection's staging.  The rounded sum of the partials must be the attention output
    (same probabilities, only the fp32 order of the sum over positions differs), and the product taken from the
    partials must be the product of that vector."""
    kv_dim, dim = heads * head // kv_mul, heads * head
    seq = pos + 1
    key = synth.stream_key(55, heads, head, kv_mul, pos)
    q = synth.normal_f16(synth.stream_key(key, "q"), dim)
    kc = synth.normal_f16(synth.stream_key(key, "k"), seq * kv_dim)
    vc = synth.normal_f16(synth.stream_key(key, "v"), seq * kv_dim)
    dq, dk, dv = ctx.upload(q), ctx.upload(kc), ctx.upload(vc)
    datt = ctx.zeros(heads * max(max_seq, seq) * 2)
    dpos = ctx.upload(np.array([pos], dtype=np.int32))
    dpart = ctx.upload(np.full(4 * dim, np.nan, dtype=np.float32))  # whatever the chunks do not write would poison the sum
    chunks = A.MultiHeadAttention_partial(ctx, dpart, dq, dk, dv, datt, heads, head, kv_mul, max_seq, dpos)
    assert 1 <= chunks <= 4
    part = dpart.download(np.float32).reshape(4, dim)[:chunks]
    acc = part[0].copy()
    for c in range(1, chunks):
        acc = acc + part[c]  # fp32, chunk order: what the consumer does
    got = acc.astype(np.float16)
    want, want_att = oracle.attention(q, kc.view(np.uint16), vc.view(np.uint16), heads, head, kv_mul, pos)
    assert rel_l2(got, want) <= 1.5e-3
    dout = ctx.zeros(dim * 2)
    A.MultiHeadAttention(ctx, dout, dq, dk, dv, datt, heads, head, kv_mul, max_seq, dpos)
    assert_close_f16(got, f16(dout.download(np.uint16)), ulps=2)
    # the O projection fed with the partials == the O projection fed with their rounded sum
    if dim <= 8192:
        N = 256
        w, z, sc, _ = _case(dim, N, 56)
        qw = A.QWeight.upload(ctx, w, z, sc)
        resid = synth.normal_f16(synth.stream_key(key, "r"), N)
        d1, d2 = ctx.upload(resid), ctx.upload(resid)
        A.matmul_q_parts(ctx, d1, dpart, chunks, qw, dim, N, accum=True)
        A.matmul_q(ctx, d2, ctx.upload(got), qw, dim, N, accum=True)
        assert np.array_equal(d1.download(np.uint16), d2.download(np.uint16))


def test_attention_pos0_returns_v0(ctx):
    heads, head = 32, 128
    q = synth.normal_f16(synth.stream_key(6, "q"), heads * head)
    kc = synth.normal_f16(synth.stream_key(6, "k"), heads * head)
    vc = synth.normal_f16(synth.stream_key(6, "v"), heads * head)
    dout = ctx.zeros(heads * head * 2)
    A.MultiHeadAttention(ctx, dout, ctx.upload(q), ctx.upload(kc), ctx.upload(vc), ctx.zeros(heads * 2), heads, head, 1, 1, ctx.upload(np.array([0], dtype=np.int32)))
    assert np.array_equal(dout.download(np.uint16), vc.view(np.uint16))


@pytest.mark.parametrize("n,d", [(4096, 32000), (5120, 32000), (6656, 1024), (8, 8), (264, 40)])
def test_matvec_f16(ctx, n, d):
    key = synth.stream_key(7, n, d)
    w = synth.normal_f16(synth.stream_key(key, "w"), n * d, 0.0, 0.02)
    x = synth.normal_f16(synth.stream_key(key, "x"), n)
    dout = ctx.zeros(d * 2)
    A.matmul(ctx, dout, ctx.upload(x), ctx.upload(w), n, d)
    got = f16(dout.download(np.uint16))
    r, want = oracle.matvec_f16(x, w, n, d)
    assert r == 0
    truth = w.astype(np.float64).reshape(d, n) @ x.astype(np.float64)
    assert rel_l2(got, truth) <= 1e-3
    assert_close_f16(got, want, ulps=2)


def test_argmax_advance_and_ties(ctx):
    V = 32000
    logits = synth.normal_f16(synth.stream_key(8, "l"), V)
    m = np.float16(logits.max() + 1)
    logits[[31999, 17, 20000]] = m  # a three-way tie: lowest index wins
    host = ctx.alloc_host(4 * 64)
    pos_host = C.c_int.from_address(host)
    tokens = (C.c_int * 32).from_address(host + 16)
    for i in range(32):
        tokens[i] = -1
    pos_host.value = 4
    dpos = ctx.upload(np.array([4], dtype=np.int32))
    A.argmax_advance(ctx, ctx.upload(logits), V, host + 16, host, dpos, True)
    ctx.sync()
    assert pos_host.value == 5 and tokens[5] == 17 and dpos.download(np.int32)[0] == 5
    # write_token = False only advances the position
    A.argmax_advance(ctx, ctx.upload(logits), V, host + 16, host, dpos, False)
    ctx.sync()
    assert pos_host.value == 6 and tokens[6] == -1 and dpos.download(np.int32)[0] == 6
    ctx.free_host(host)


def test_embed(ctx):
    dim, V = 4096, 64
    table = synth.normal_f16(synth.stream_key(9, "t"), V * dim).view(np.uint16)
    toks = np.array([5, 63, 0, 7], dtype=np.int32)
    dx = ctx.zeros(dim * 2)
    A.copy_embedding(ctx, dx, ctx.upload(table), dim, ctx.upload(toks), ctx.upload(np.array([1], dtype=np.int32)))
    assert np.array_equal(dx.download(np.uint16), table[63 * dim : 64 * dim])
