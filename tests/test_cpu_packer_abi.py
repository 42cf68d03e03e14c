"""CPU tests: the .bin format against the reference's own weight_packer output (golden fixture), model-size
arithmetic against the published layer sizes, and the C-ABI surface of libawq_hip.so (no GPU calls)."""
import ctypes
import os
import re

import numpy as np
import pytest

from llama_cu_awq_amd import packer, synth
from oracle import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CFG = dict(dim=128, hidden_dim=384, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=32, seq_len=32, rope_theta=10000.0)


@pytest.fixture(scope="module")
def fixture():
    return np.load(os.path.join(ROOT, "tests", "golden", "packer_fixture.npz"))


def _own_image(fx):
    dim, hid = CFG["dim"], CFG["hidden_dim"]
    t = {"embed": fx["model.embed_tokens.weight"], "lm_head": fx["lm_head.weight"], "norm": fx["model.norm.weight"]}
    names = {"q_proj": ("self_attn.q_proj", dim, dim), "k_proj": ("self_attn.k_proj", dim, dim), "v_proj": ("self_attn.v_proj", dim, dim),
             "o_proj": ("self_attn.o_proj", dim, dim), "up_proj": ("mlp.up_proj", dim, hid), "gate_proj": ("mlp.gate_proj", dim, hid),
             "down_proj": ("mlp.down_proj", hid, dim)}
    for l in range(CFG["n_layers"]):
        for short, (full, K, N) in names.items():
            base = f"model.layers.{l}.{full}"
            t[f"{l}.{short}"] = packer.repack_old_awq(fx[base + ".qweight"], fx[base + ".qzeros"], fx[base + ".scales"], K, N)
        t[f"{l}.input_layernorm"] = fx[f"model.layers.{l}.input_layernorm.weight"]
        t[f"{l}.post_attention_layernorm"] = fx[f"model.layers.{l}.post_attention_layernorm.weight"]
    return packer.write_model(None, CFG, t)


def _valid_nibble_masks(cfg):
    """(low, high) per-byte masks: False where the nibble is padding of a zeros row, which the reference tool fills
    with whatever lay beyond its buffer (weight_packer.cpp:117-121 with a group count that is not a multiple of 8)."""
    dim, hid, V = cfg["dim"], cfg["hidden_dim"], cfg["vocab_size"]
    lo = np.ones(synth.model_bytes(cfg), dtype=bool)
    hi = np.ones(synth.model_bytes(cfg), dtype=bool)
    off = 32 + 2 * V * dim * 2 + dim * 2
    for _ in range(cfg["n_layers"]):
        for K, N in ((dim, dim), (dim, dim), (dim, dim), (dim, dim), (dim, hid), (dim, hid), (hid, dim)):
            pwh, pzh, sh = synth.strides(K)
            off += N * pwh * 4
            nib = np.arange(pzh * 8) < sh  # nibble j of a zeros row is valid iff j < groups
            lo[off : off + N * pzh * 4] = np.tile(nib[0::2], N)
            hi[off : off + N * pzh * 4] = np.tile(nib[1::2], N)
            off += N * pzh * 4 + N * sh * 2
        off += 2 * dim * 2
    assert off == lo.size
    return lo, hi


def test_own_packer_reproduces_reference_weight_packer(fixture):
    ref = fixture["reference_bin"]
    own = _own_image(fixture)
    assert ref.size == own.size == synth.model_bytes(CFG)
    assert np.array_equal(ref[:32], own[:32])  # header: 7 int32 + rope_theta
    lo, hi = _valid_nibble_masks(CFG)
    assert np.array_equal((ref & 0xF)[lo], (own & 0xF)[lo])
    assert np.array_equal((ref >> 4)[hi], (own >> 4)[hi])
    assert (~lo).sum() + (~hi).sum() > 0  # the fixture does exercise padding nibbles


def test_reference_bin_dequantises_to_the_awq_definition(fixture):
    """Weights decoded from the reference tool's .bin equal (q - z) * s decoded directly from the AWQ tensors."""
    ref = fixture["reference_bin"]
    dim, hid = CFG["dim"], CFG["hidden_dim"]
    m = oracle.Model(ref)
    assert m.config["dim"] == dim and m.config["hidden_dim"] == hid
    m.close()
    # down_proj of layer 1 straight from the AWQ tensors
    base = "model.layers.1.mlp.down_proj"
    K, N = hid, dim
    q = packer.deinterleave(fixture[base + ".qweight"])[:K, :N].astype(np.float64)  # [K][N]
    z = packer.deinterleave(fixture[base + ".qzeros"])[: K // 128, :N].astype(np.float64)
    s = fixture[base + ".scales"].astype(np.float64)
    g = np.arange(K) // 128
    want = ((q - z[g]) * s[g]).T  # [N][K]
    # the same tensor located in the reference .bin by the documented order
    off = 32 + 2 * CFG["vocab_size"] * dim * 2 + dim * 2
    sizes = [(dim, dim)] * 4 + [(dim, hid)] * 2 + [(hid, dim)]
    per_layer = sum(Nn * (synth.strides(Kk)[0] * 4 + synth.strides(Kk)[1] * 4 + synth.strides(Kk)[2] * 2) for Kk, Nn in sizes) + 4 * dim
    off += per_layer  # layer 0
    for Kk, Nn in sizes[:-1]:
        pwh, pzh, sh = synth.strides(Kk)
        off += Nn * (pwh * 4 + pzh * 4 + sh * 2)
    pwh, pzh, sh = synth.strides(K)
    w = ref[off : off + N * pwh * 4].view(np.uint32).reshape(N, pwh)
    off += N * pwh * 4
    zz = ref[off : off + N * pzh * 4].view(np.uint32).reshape(N, pzh)
    off += N * pzh * 4
    sc = ref[off : off + N * sh * 2].view(np.float16).reshape(N, sh)
    assert np.array_equal(synth.dequantize(w, zz, sc, K), want)
    got = oracle.dequant(w, zz, sc, K, N)
    assert np.array_equal(got.view(np.uint16), want.astype(np.float32).astype(np.float16).view(np.uint16))


def test_interleave_round_trip():
    rng = np.random.default_rng(4)
    v = rng.integers(0, 16, size=(6, 32), dtype=np.uint8)
    assert np.array_equal(packer.deinterleave(packer.interleave(v)), v)
    # nibble i of the source dword is column order_map[i] (weight_packer.cpp:96-107)
    one = np.array([[0x76543210]], dtype=np.uint32)
    assert list(packer.deinterleave(one)[0]) == [0, 4, 1, 5, 2, 6, 3, 7]


def test_model_sizes_match_the_published_shapes():
    assert synth.model_bytes(synth.CONFIG_7B) == 3889438752
    assert synth.model_bytes(synth.CONFIG_13B) == 7248291872
    assert synth.model_bytes(synth.CONFIG_33B) == 17539945504
    # one 4096x4096 matrix: weights + zeros + scales
    pwh, pzh, sh = synth.strides(4096)
    assert 4096 * (pwh * 4 + pzh * 4 + sh * 2) == 8716288
    pwh, pzh, sh = synth.strides(11008)
    assert (pwh, pzh, sh) == (1376, 11, 86) and 4096 * (pwh * 4 + pzh * 4 + sh * 2) == 23429120


def test_synthetic_streams_are_deterministic_and_distinct():
    a = synth.random_u64(synth.stream_key(0, 3, "wq_q"), 1000)
    b = synth.random_u64(synth.stream_key(0, 3, "wq_q"), 1000)
    c = synth.random_u64(synth.stream_key(0, 4, "wq_q"), 1000)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    # chunked generation equals one-shot generation
    big = synth.random_u64(synth.stream_key(1), (1 << 22) + 17)
    assert np.array_equal(big[-17:], synth.random_u64(synth.stream_key(1), 17, start=1 << 22))
    n = synth.normal(synth.stream_key(2), 200000)
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1) < 0.01
    w, z, s = synth.make_qweight(synth.stream_key(5), 200, 16)  # K % 32 != 0: padding nibbles are zero
    assert not (synth.unpack_nibbles(w, 224)[:, 200:]).any()
    assert s.min() >= np.float16(0.002) and s.max() <= np.float16(0.02)


def test_library_exports_every_declared_symbol():
    """Every awq_* function declared in include/awq_hip.h is exported by the built library (no compute calls)."""
    hdr = open(os.path.join(ROOT, "include", "awq_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(awq_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) >= 35
    so = os.path.join(ROOT, "llama_cu_awq_amd", "libawq_hip.so")
    if not os.path.exists(so):
        import __graft_entry__

        __graft_entry__.build()
    lib = ctypes.CDLL(so)
    missing = [n for n in sorted(declared) if not hasattr(lib, n)]
    assert not missing, missing
    # the Python binding lists the same functions
    from llama_cu_awq_amd import _lib

    bound = set(_lib.PROTOTYPES) | set(_lib.NON_STATUS)
    assert declared == bound, (declared - bound, bound - declared)
    # status codes and struct sizes the header promises
    assert ctypes.sizeof(_lib.ConfigC) == 32
    lib.awq_last_error.restype = ctypes.c_char_p
    assert isinstance(lib.awq_last_error(), bytes)
