"""The batched int4 GEMM entry point that allocates nothing (awq_gemm_int4_static) against awq_gemm_int4.

Both run the same kernel with the same work split; only where the split-K workspace lives differs (a device array
inside the library instead of memory allocated on first use), and the two-term sum of the K halves does not depend
on which half arrives first, so the outputs must agree bit for bit.  Two calls in a row share the array: the second
is smaller and must not see anything the first left behind.
"""
import numpy as np
import pytest

import llama_cu_awq_amd as A
from llama_cu_awq_amd import synth
from tests.helpers import f16, rel_l2

pytestmark = pytest.mark.gpu


def _case(ctx, M, K, N, tag):
    key = synth.stream_key(77, M, K, N, tag)
    w, z, s = synth.make_qweight(key, K, N)
    a = synth.normal_f16(synth.stream_key(key, "a"), M * K)
    resid = synth.normal_f16(synth.stream_key(key, "r"), M * N)
    return A.QWeight.upload(ctx, w, z, s), ctx.upload(a), resid, (w, z, s, a)


def _run(fn, ctx, qw, da, resid, M, K, N, accum):
    dout = ctx.upload(resid) if accum else ctx.zeros(M * N * 2)
    fn(ctx, dout, N, da, K, M, qw, K, N, accum=accum)
    return dout.download(np.uint16)


def test_static_workspace_matches_allocating_entry_point_twice_in_a_row(ctx):
    # (512, 4096, 4096): 128 output tiles < 256, K = 64 steps -> the split-K form, every tile of the workspace the
    # 7B-shape O projection uses; then (130, 1024, 384): 6 tiles, ragged last row tile, a fraction of the array
    shapes = [(512, 4096, 4096), (130, 1024, 384)]
    for accum in (False, True):
        static_out, plain_out, truth = [], [], []
        cases = [_case(ctx, M, K, N, int(accum)) for M, K, N in shapes]
        # the two static calls back to back on the same stream, nothing in between
        for (M, K, N), (qw, da, resid, _) in zip(shapes, cases):
            static_out.append(_run(A.gemm_q_static, ctx, qw, da, resid, M, K, N, accum))
        for (M, K, N), (qw, da, resid, host) in zip(shapes, cases):
            plain_out.append(_run(A.gemm_q, ctx, qw, da, resid, M, K, N, accum))
            w, z, s, a = host
            w16 = synth.dequantize(w, z, s, K).astype(np.float32).astype(np.float16).astype(np.float64)
            t = a.astype(np.float64).reshape(M, K) @ w16.T
            truth.append(t + resid.astype(np.float64).reshape(M, N) if accum else t)
        for got, want, t, (M, K, N) in zip(static_out, plain_out, truth, shapes):
            assert np.array_equal(got, want), (M, K, N, accum)
            assert rel_l2(f16(got).reshape(M, N), t) <= 1e-3


def test_static_workspace_without_split(ctx):
    """More than 255 output tiles: no split, no workspace; still the same result."""
    M, K, N = 256, 256, 16384  # 2 x 128 tiles
    qw, da, resid, _ = _case(ctx, M, K, N, 9)
    got = _run(A.gemm_q_static, ctx, qw, da, resid, M, K, N, False)
    want = _run(A.gemm_q, ctx, qw, da, resid, M, K, N, False)
    assert np.array_equal(got, want)


def test_static_workspace_shape_guard(ctx):
    buf = ctx.alloc(1 << 16)
    qw = A.QWeight(buf, buf, buf)
    for M, K, N in ((4, 48, 128), (4, 64, 64), (0, 64, 128)):
        with pytest.raises(A.AwqError) as e:
            A.gemm_q_static(ctx, buf, N, buf, K, M, qw, K, N)
        assert e.value.code == -2
