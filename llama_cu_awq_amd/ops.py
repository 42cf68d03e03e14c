"""Host-side mirror of the reference's launcher set (llama2_q4.cu:347-427, sampler.h:77-84) over the C-ABI.

Names and argument order follow the reference's launchers; buffers are DeviceBuffer objects (or raw integer
device addresses).  Every call is asynchronous on the context's stream, as in the reference.
"""
import ctypes as C

import numpy as np

from ._lib import QWeightC, check, lib


def _addr(b):
    if b is None:
        return None
    if isinstance(b, DeviceBuffer):
        return b.ptr
    return int(b)


class Context:
    """Device ordinal + stream (cudaSetDevice/cudaStreamCreate, llama2_q4.cu:685,695)."""

    def __init__(self, device=0, stream=None):
        h = C.c_void_p()
        if stream is None:
            check(lib.awq_ctx_create(device, C.byref(h)))
        else:
            check(lib.awq_ctx_create_on_stream(device, stream, C.byref(h)))
        self.h = h
        self.device = device

    def sync(self):
        check(lib.awq_stream_sync(self.h))

    def close(self):
        if self.h:
            check(lib.awq_ctx_destroy(self.h))
            self.h = None

    # memory -------------------------------------------------------------
    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def upload(self, array):
        a = np.ascontiguousarray(array)
        b = DeviceBuffer(self, a.nbytes)
        if a.nbytes:
            check(lib.awq_memcpy_h2d(self.h, b.ptr, a.ctypes.data, a.nbytes))
        return b

    def zeros(self, nbytes):
        b = DeviceBuffer(self, nbytes)
        check(lib.awq_memset_async(self.h, b.ptr, 0, nbytes))
        return b

    def alloc_host(self, nbytes):
        p = C.c_void_p()
        check(lib.awq_malloc_host(self.h, C.byref(p), nbytes))
        return p.value

    def free_host(self, ptr):
        check(lib.awq_free_host(self.h, ptr))

    # timing -------------------------------------------------------------
    def event(self):
        e = C.c_void_p()
        check(lib.awq_event_create(self.h, C.byref(e)))
        return e

    def record(self, e):
        check(lib.awq_event_record(self.h, e))

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        check(lib.awq_event_elapsed_ms(self.h, start, stop, C.byref(ms)))
        return ms.value


class DeviceBuffer:
    def __init__(self, ctx, nbytes, ptr=None):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        self.owned = ptr is None
        if ptr is None:
            p = C.c_void_p()
            check(lib.awq_malloc(ctx.h, C.byref(p), self.nbytes))
            ptr = p.value
        self.ptr = ptr

    def download(self, dtype, count=None, offset_bytes=0):
        dtype = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset_bytes) // dtype.itemsize
        out = np.empty(count, dtype=dtype)
        if out.nbytes:
            check(lib.awq_memcpy_d2h(self.ctx.h, out.ctypes.data, self.ptr + offset_bytes, out.nbytes))
        return out

    def write(self, array, offset_bytes=0):
        a = np.ascontiguousarray(array)
        assert offset_bytes + a.nbytes <= self.nbytes
        check(lib.awq_memcpy_h2d(self.ctx.h, self.ptr + offset_bytes, a.ctypes.data, a.nbytes))

    def free(self):
        if self.owned and self.ptr:
            check(lib.awq_free(self.ctx.h, self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class QWeight:
    """QWeight (common.h:26-30): device (weight, zeros, scales) of one packed matrix."""

    def __init__(self, weight, zeros, scales):
        self.weight, self.zeros, self.scales = weight, zeros, scales
        self.c = QWeightC(_addr(weight), _addr(zeros), _addr(scales))

    @classmethod
    def upload(cls, ctx, weight, zeros, scales):
        return cls(ctx.upload(weight), ctx.upload(zeros), ctx.upload(scales))


def copy_embedding(ctx, x, table, dim, tokens, pPos):
    """copy_embedding_kernel launch, llama2_q4.cu:441."""
    check(lib.awq_embed(ctx.h, _addr(x), _addr(table), dim, _addr(tokens), _addr(pPos)))


def rmsnorm(ctx, o, x, weight, size):
    """rmsnorm(), llama2_q4.cu:347-350."""
    check(lib.awq_rmsnorm(ctx.h, _addr(o), _addr(x), _addr(weight), size))


def matmul(ctx, xout, x, w, n, d):
    """matmul(half), llama2_q4.cu:357-365 (classifier form)."""
    check(lib.awq_matvec_f16(ctx.h, _addr(xout), _addr(x), _addr(w), n, d))


def matmul_q(ctx, xout, x, w, inpSize, opSize, accum=False, gpu_count=1, loff=-1, pPos=None):
    """matmul(QWeight), llama2_q4.cu:367-376."""
    check(lib.awq_matvec_int4(ctx.h, _addr(xout), _addr(x), C.byref(w.c), inpSize, opSize, int(accum), gpu_count, loff, _addr(pPos)))


def qkv_matvec(ctx, q, key_cache, value_cache, x, qw, kw, vw, inpSize, opSize, loff, pPos):
    """qkv_matvec(), llama2_q4.cu:378-391."""
    check(
        lib.awq_qkv_matvec(
            ctx.h, _addr(q), _addr(key_cache), _addr(value_cache), _addr(x), C.byref(qw.c), C.byref(kw.c), C.byref(vw.c),
            inpSize, opSize, loff, _addr(pPos),
        )
    )


def ffn_matvec_silu(ctx, xout, x, gate_w, up_w, inpSize, opSize):
    """ffn_matvec_silu(), llama2_q4.cu:393-404."""
    check(lib.awq_ffn_matvec_silu(ctx.h, _addr(xout), _addr(x), C.byref(gate_w.c), C.byref(up_w.c), inpSize, opSize))


def rmsnorm_ffn_matvec_silu(ctx, xout, x, norm_weight, gate_w, up_w, inpSize, opSize):
    """rmsnorm() + ffn_matvec_silu() (llama2_q4.cu:496-498) in one launch: what the fused schedule issues."""
    check(lib.awq_rmsnorm_ffn_matvec_silu(ctx.h, _addr(xout), _addr(x), _addr(norm_weight), C.byref(gate_w.c), C.byref(up_w.c), inpSize, opSize))


def RoPERotation(ctx, q, k, num_heads, num_kv_heads, head_size, pPos, loff, rope_theta):
    """RoPERotation(), llama2_q4.cu:406-408."""
    check(lib.awq_rope(ctx.h, _addr(q), _addr(k), num_heads, num_kv_heads, head_size, _addr(pPos), loff, rope_theta))


def MultiHeadAttention(ctx, output, q, key_cache, value_cache, att, num_heads, head_size, kv_mul, max_seq_len, pPos):
    """MultiHeadAttention(), llama2_q4.cu:410-427."""
    check(
        lib.awq_attention(
            ctx.h, _addr(output), _addr(q), _addr(key_cache), _addr(value_cache), _addr(att), num_heads, head_size, kv_mul,
            max_seq_len, _addr(pPos),
        )
    )


def MultiHeadAttention_partial(ctx, part, q, key_cache, value_cache, att, num_heads, head_size, kv_mul, max_seq_len, pPos):
    """Scores + position-split P.V (fp32 partial sums per range of positions); returns the number of ranges."""
    n = C.c_int()
    check(
        lib.awq_attention_partial(
            ctx.h, _addr(part), C.byref(n), _addr(q), _addr(key_cache), _addr(value_cache), _addr(att), num_heads, head_size,
            kv_mul, max_seq_len, _addr(pPos),
        )
    )
    return n.value


def matmul_q_parts(ctx, xout, part, parts, w, inpSize, opSize, accum=False):
    """matmul(QWeight) whose input vector is half(sum of `parts` fp32 vectors) (the O projection behind the split attention)."""
    check(lib.awq_matvec_int4_parts(ctx.h, _addr(xout), _addr(part), parts, C.byref(w.c), inpSize, opSize, int(accum)))


def argmax_advance(ctx, logits, size, tokens, pos_host, pos_dev, write_token):
    """sample() greedy branch, sampler.h:77-84."""
    check(lib.awq_argmax_advance(ctx.h, _addr(logits), size, _addr(tokens), _addr(pos_host), _addr(pos_dev), int(write_token)))


def softmax_logits(ctx, logits, size, temperature):
    """softmax_logits_kernel launch, sampler.h:87 (in place)."""
    check(lib.awq_softmax_logits(ctx.h, _addr(logits), size, float(temperature)))


def sample_top_p(ctx, probs, size, threshold, sorted_, tokens, pos_host, pos_dev):
    """Sort + prefix sum + sample_top_p_kernel, sampler.h:94-115."""
    check(lib.awq_sample_top_p(ctx.h, _addr(probs), size, float(threshold), int(sorted_), _addr(tokens), _addr(pos_host), _addr(pos_dev)))


class Sampler:
    """Sampler + build_sampler() / sample(), sampler.h:10-47, 77-115."""

    def __init__(self, ctx, vocab_size, temperature, topp, rng_seed):
        self.ctx = ctx
        h = C.c_void_p()
        check(lib.awq_sampler_create(ctx.h, vocab_size, float(temperature), float(topp), int(rng_seed), C.byref(h)))
        self.h = h

    def sample(self, logits, tokens, pos_host, pos_dev, gen_token):
        check(lib.awq_sampler_sample(self.h, _addr(logits), _addr(tokens), _addr(pos_host), _addr(pos_dev), int(gen_token)))

    def close(self):
        if self.h:
            check(lib.awq_sampler_destroy(self.h))
            self.h = None


def dequant(ctx, out, w, K, N):
    """(q - z) * scale materialised in fp16 (gpu_kernels.h:204-205)."""
    check(lib.awq_dequant(ctx.h, _addr(out), C.byref(w.c), K, N))


def gemm_q(ctx, out, ldo, a, lda, M, w, K, N, accum=False):
    """Batched form of matmul(QWeight) for M activation rows (prefill); no launcher of this kind exists in the reference."""
    check(lib.awq_gemm_int4(ctx.h, _addr(out), ldo, _addr(a), lda, M, C.byref(w.c), K, N, int(accum)))


def gemm_q_static(ctx, out, ldo, a, lda, M, w, K, N, accum=False):
    """gemm_q() with the split-K workspace in the library's own device array: allocates nothing (for callers under graph capture)."""
    check(lib.awq_gemm_int4_static(ctx.h, _addr(out), ldo, _addr(a), lda, M, C.byref(w.c), K, N, int(accum)))
