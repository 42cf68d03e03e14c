"""Deterministic synthetic tensors and weight_packer-format model images (no checkpoints exist offline).

A counter-based splitmix64 generator: every tensor has its own stream key derived from (seed, layer, name), so
tensors can be generated independently, in any order and in parallel, and are identical on every machine.

Distributions (the benchmark configurations'): 4-bit weights and zero points uniform on {0..15}; scales
half(U[0.002, 0.02]); activations and KV pre-fill N(0,1); embedding / classifier N(0, 0.02); norm weights
1 + N(0, 0.02).  Padding nibbles are zero.
"""
from concurrent.futures import ThreadPoolExecutor

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_CHUNK = 1 << 22


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def stream_key(seed, *ids):
    """Key of the stream named by (seed, ids...); ids are ints or strings."""
    with np.errstate(over="ignore"):
        k = _mix(np.uint64(seed) + _GOLDEN)
        for i in ids:
            if isinstance(i, str):
                for b in i.encode():
                    k = _mix(k ^ (np.uint64(b) + _GOLDEN))
            else:
                k = _mix(k ^ (np.uint64(int(i) & 0xFFFFFFFFFFFFFFFF) + _GOLDEN))
    return k


def random_u64(key, n, start=0):
    """Outputs start .. start+n-1 of the stream: mix(key + (i+1)*golden)."""
    out = np.empty(n, dtype=np.uint64)
    with np.errstate(over="ignore"):
        for o in range(0, n, _CHUNK):
            m = min(_CHUNK, n - o)
            idx = np.arange(start + o + 1, start + o + m + 1, dtype=np.uint64)
            out[o : o + m] = _mix(key + idx * _GOLDEN)
    return out


def random_u32(key, n):
    return random_u64(key, (n + 1) // 2).view(np.uint32)[:n]


def uniform01(key, n, start=0):
    return (random_u64(key, n, start) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def normal(key, n, mean=0.0, std=1.0):
    """Box-Muller (cosine branch) in double precision."""
    out = np.empty(n, dtype=np.float64)
    for o in range(0, n, _CHUNK):
        m = min(_CHUNK, n - o)
        u = random_u64(key, 2 * m, 2 * o)
        u1 = ((u[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / (1 << 53))  # (0, 1]
        u2 = (u[1::2] >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
        out[o : o + m] = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return out * std + mean


def normal_f16(key, n, mean=0.0, std=1.0):
    return normal(key, n, mean, std).astype(np.float16)


# ---------------------------------------------------------------- packed matrices
def strides(K):
    """(pwh dwords, pzh dwords, sh halves) per row for reduction length K (llama2_q4.cu:106-129)."""
    sh = (K + 127) // 128
    return ((K + 31) // 32) * 4, (sh + 7) // 8, sh


def pack_nibbles(vals, width_dwords):
    """vals: (rows, n) ints in 0..15 -> (rows, width_dwords) uint32, element j in bits 4*(j%8) of dword j/8."""
    rows, n = vals.shape
    padded = np.zeros((rows, width_dwords * 8), dtype=np.uint32)
    padded[:, :n] = vals
    shifts = (np.arange(8, dtype=np.uint32) * 4)[None, None, :]
    return (padded.reshape(rows, width_dwords, 8) << shifts).sum(axis=2, dtype=np.uint32)


def unpack_nibbles(packed, n):
    """Inverse of pack_nibbles: (rows, width) uint32 -> (rows, n) uint8."""
    rows, width = packed.shape
    shifts = (np.arange(8, dtype=np.uint32) * 4)[None, None, :]
    return ((packed[:, :, None] >> shifts) & np.uint32(0xF)).reshape(rows, width * 8)[:, :n].astype(np.uint8)


def make_qweight(key, K, N, scale_mult=1.0):
    """Random packed matrix: returns (weight (N,pwh) u32, zeros (N,pzh) u32, scales (N,sh) f16).

    scale_mult multiplies the scale range U[0.002, 0.02] (1.0 = the benchmark distribution)."""
    pwh, pzh, sh = strides(K)
    weight = random_u32(stream_key(key, "w"), N * pwh).reshape(N, pwh).copy()
    if K % 32:
        q = unpack_nibbles(weight, K)
        weight = pack_nibbles(q, pwh)
    z = (random_u64(stream_key(key, "z"), N * sh) >> np.uint64(60)).astype(np.uint32).reshape(N, sh)
    zeros = pack_nibbles(z, pzh)
    scales = (scale_mult * (0.002 + 0.018 * uniform01(stream_key(key, "s"), N * sh))).astype(np.float16).reshape(N, sh)
    return weight, zeros, scales


def dequantize(weight, zeros, scales, K):
    """Exact (q - z) * s as float64 (N, K) from the layout definition (numpy restatement, independent of the C code)."""
    N = weight.shape[0]
    sh = (K + 127) // 128
    q = unpack_nibbles(weight, K).astype(np.float64)
    z = unpack_nibbles(zeros, sh).astype(np.float64)
    s = scales.astype(np.float64)
    g = np.arange(K) // 128
    return (q - z[:, g]) * s[:, g]


# ---------------------------------------------------------------- model images
def model_bytes(cfg):
    dim, hid, L, V = cfg["dim"], cfg["hidden_dim"], cfg["n_layers"], cfg["vocab_size"]
    kv_dim = dim * cfg["n_kv_heads"] // cfg["n_heads"]

    def qb(K, N):
        pwh, pzh, sh = strides(K)
        return N * (pwh * 4 + pzh * 4 + sh * 2)

    layer = 2 * qb(dim, dim) + 2 * qb(dim, kv_dim) + 2 * qb(dim, hid) + qb(hid, dim) + 4 * dim
    return 32 + 4 * V * dim + 2 * dim + L * layer


def make_model_image(cfg, seed=0, threads=8, scale_mult=1.0):
    """A weight_packer-format .bin image (llama2_q4.cu:220-246 order) of random weights, as a uint8 array.

    scale_mult shrinks (or grows) every quantisation scale: with the benchmark distribution (1.0) each layer adds a
    few hundred to the residual stream, which leaves fp16 range in models of 40 and more layers; a smaller range
    keeps such a model finite so that its outputs can be checked."""
    dim, hid, L, V = cfg["dim"], cfg["hidden_dim"], cfg["n_layers"], cfg["vocab_size"]
    kv_dim = dim * cfg["n_kv_heads"] // cfg["n_heads"]
    img = np.empty(model_bytes(cfg), dtype=np.uint8)
    hdr = np.array([dim, hid, L, cfg["n_heads"], cfg["n_kv_heads"], V, cfg["seq_len"]], dtype=np.int32)
    img[:28] = hdr.view(np.uint8)
    img[28:32] = np.array([cfg.get("rope_theta", 10000.0)], dtype=np.float32).view(np.uint8)
    jobs = []  # (offset, nbytes, fn)
    off = [32]

    def put(nbytes, fn):
        jobs.append((off[0], nbytes, fn))
        off[0] += nbytes

    def dense(name, n, mean, std, layer=-1):
        put(2 * n, lambda: normal_f16(stream_key(seed, layer, name), n, mean, std).view(np.uint8))

    def qweight(name, K, N, layer):
        pwh, pzh, sh = strides(K)

        def gen():
            w, z, s = make_qweight(stream_key(seed, layer, name), K, N, scale_mult)
            return np.concatenate([w.reshape(-1).view(np.uint8), z.reshape(-1).view(np.uint8), s.reshape(-1).view(np.uint8)])

        put(N * (pwh * 4 + pzh * 4 + sh * 2), gen)

    dense("embed", V * dim, 0.0, 0.02)
    dense("wcls", V * dim, 0.0, 0.02)
    dense("rms_final", dim, 1.0, 0.02)
    for l in range(L):
        qweight("wq_q", dim, dim, l)
        qweight("wq_k", dim, kv_dim, l)
        qweight("wq_v", dim, kv_dim, l)
        qweight("wq_o", dim, dim, l)
        qweight("wq_up", dim, hid, l)
        qweight("wq_gate", dim, hid, l)
        qweight("wq_down", hid, dim, l)
        dense("rms_att", dim, 1.0, 0.02, l)
        dense("rms_ffn", dim, 1.0, 0.02, l)
    assert off[0] == img.nbytes

    def run(job):
        o, n, fn = job
        data = fn()
        assert data.nbytes == n
        img[o : o + n] = data

    if threads > 1:
        with ThreadPoolExecutor(threads) as ex:
            list(ex.map(run, jobs))
    else:
        for j in jobs:
            run(j)
    return img


def prompt_tokens(seed, n, vocab):
    """n random token ids in [3, vocab)."""
    u = random_u64(stream_key(seed, "prompt"), n)
    return [int(3 + (int(v) % (vocab - 3))) for v in u]


CONFIG_7B = dict(dim=4096, hidden_dim=11008, n_layers=32, n_heads=32, n_kv_heads=32, vocab_size=32000, seq_len=2048, rope_theta=10000.0)
CONFIG_13B = dict(dim=5120, hidden_dim=13824, n_layers=40, n_heads=40, n_kv_heads=40, vocab_size=32000, seq_len=2048, rope_theta=10000.0)
CONFIG_33B = dict(dim=6656, hidden_dim=17920, n_layers=60, n_heads=52, n_kv_heads=52, vocab_size=32000, seq_len=2048, rope_theta=10000.0)
# beyond the benchmark's configurations: Llama-2-70B's shape (grouped queries: 64 heads share 8 KV heads), 36.6 GB packed
CONFIG_70B = dict(dim=8192, hidden_dim=28672, n_layers=80, n_heads=64, n_kv_heads=8, vocab_size=32000, seq_len=2048, rope_theta=10000.0)
