"""CPU tests of the weight_packer command-line tool (llama_cu_awq_amd/csrc/driver/weight_packer.cpp).

Golden data: tests/golden/packer_fixture.npz holds old-format AWQ tensors and the .bin that the reference's own
weight_packer (compiled from its source) produced from them.  Where the compiled reference tool is present
(oracle/_ref/weight_packer, built by `make -C oracle`), the new-format path is also compared with it directly.
Padding nibbles of the zeros rows are masked: the reference fills them with whatever lay behind its buffer.
"""
import json
import os
import subprocess

import numpy as np
import pytest

from llama_cu_awq_amd import synth
from tests.test_cpu_packer_abi import CFG, ROOT, _own_image, _valid_nibble_masks

SRC = os.path.join(ROOT, "llama_cu_awq_amd", "csrc", "driver", "weight_packer.cpp")
REF_TOOL = os.path.join(ROOT, "oracle", "_ref", "weight_packer")
HF = {"hidden_size": "dim", "intermediate_size": "hidden_dim", "num_hidden_layers": "n_layers", "num_attention_heads": "n_heads",
      "num_key_value_heads": "n_kv_heads", "vocab_size": "vocab_size", "max_position_embeddings": "seq_len"}


@pytest.fixture(scope="module")
def tool(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("packer") / "weight_packer")
    subprocess.run(["g++", "-O2", "-std=c++17", "-Wall", "-Werror", SRC, "-o", exe], check=True)
    return exe


@pytest.fixture(scope="module")
def fixture():
    return np.load(os.path.join(ROOT, "tests", "golden", "packer_fixture.npz"))


def _write_config(path, cfg, compact=True, drop=()):
    d = {hf: cfg[own] for hf, own in HF.items() if hf not in drop}
    d["rope_theta"] = cfg["rope_theta"]
    for k in drop:
        d.pop(k, None)
    with open(path, "w") as f:
        f.write(json.dumps(d, separators=(",", ":")) if compact else json.dumps(d, indent=4, separators=(",", " : ")))


def _dump_old(dirname, fx):
    os.makedirs(dirname, exist_ok=True)
    for name in fx.files:
        if name != "reference_bin":
            fx[name].tofile(os.path.join(dirname, name + ".bin"))


def _masked_equal(a, b, cfg):
    lo, hi = _valid_nibble_masks(cfg)
    return bool(np.array_equal((a & 0x0F)[lo], (b & 0x0F)[lo]) and np.array_equal((a >> 4)[hi], (b >> 4)[hi]))


def test_old_format_matches_reference_output(tool, fixture, tmp_path):
    _dump_old(tmp_path / "in", fixture)
    _write_config(tmp_path / "config.json", CFG)
    out = tmp_path / "model.bin"
    r = subprocess.run([tool, str(tmp_path / "config.json"), str(tmp_path / "in"), str(out), "1"], capture_output=True)
    assert r.returncode == 0, r.stderr
    got = np.fromfile(out, dtype=np.uint8)
    ref = fixture["reference_bin"]
    assert got.size == ref.size == synth.model_bytes(CFG)
    assert _masked_equal(got, ref, CFG)
    # and byte for byte what the Python packer writes (both zero the padding nibbles)
    assert np.array_equal(got, _own_image(fixture))


def _dump_new(dirname, image, cfg):
    """Split a model image back into per-tensor files in the new AWQ layout (scale rows padded to 8 groups)."""
    os.makedirs(dirname, exist_ok=True)
    dim, hid, V = cfg["dim"], cfg["hidden_dim"], cfg["vocab_size"]
    off = 32

    def take(n):
        nonlocal off
        part = image[off : off + n]
        off += n
        return part

    take(V * dim * 2).tofile(os.path.join(dirname, "model.embed_tokens.weight.bin"))
    take(V * dim * 2).tofile(os.path.join(dirname, "lm_head.weight.bin"))
    take(dim * 2).tofile(os.path.join(dirname, "model.norm.weight.bin"))
    mats = [("self_attn.q_proj", dim, dim), ("self_attn.k_proj", dim, dim), ("self_attn.v_proj", dim, dim), ("self_attn.o_proj", dim, dim),
            ("mlp.up_proj", dim, hid), ("mlp.gate_proj", dim, hid), ("mlp.down_proj", hid, dim)]
    for l in range(cfg["n_layers"]):
        base = os.path.join(dirname, f"model.layers.{l}.")
        for name, K, N in mats:
            pwh, pzh, sh = synth.strides(K)
            take(N * pwh * 4).tofile(base + name + ".qweight.bin")
            take(N * pzh * 4).tofile(base + name + ".qzeros.bin")
            s = take(N * sh * 2).view(np.uint16).reshape(N, sh)
            padded = np.full((N, pzh * 8), 0x7E00, dtype=np.uint16)  # padding that must not survive
            padded[:, :sh] = s
            padded.tofile(base + name + ".scales.bin")
        take(dim * 2).tofile(base + "input_layernorm.weight.bin")
        take(dim * 2).tofile(base + "post_attention_layernorm.weight.bin")
    assert off == image.size


def test_new_format_strips_scale_padding(tool, fixture, tmp_path):
    image = _own_image(fixture)
    _dump_new(tmp_path / "in", image, CFG)
    _write_config(tmp_path / "config.json", CFG, compact=False)  # whitespace around the colons
    out = tmp_path / "model.bin"
    r = subprocess.run([tool, str(tmp_path / "config.json"), str(tmp_path / "in"), str(out), "0"], capture_output=True)
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(out, dtype=np.uint8), image)
    if os.path.exists(REF_TOOL):  # the compiled reference tool on the same inputs (it needs the compact "key": spelling)
        _write_config(tmp_path / "config_compact.json", CFG)
        ref_out = tmp_path / "ref.bin"
        rr = subprocess.run([REF_TOOL, str(tmp_path / "config_compact.json"), str(tmp_path / "in"), str(ref_out), "0"], capture_output=True)
        assert rr.returncode == 0
        assert _masked_equal(np.fromfile(ref_out, dtype=np.uint8), image, CFG)


def test_optional_keys_and_header(tool, fixture, tmp_path):
    _dump_old(tmp_path / "in", fixture)
    cfg_path = tmp_path / "config.json"
    d = {hf: CFG[own] for hf, own in HF.items() if hf != "num_key_value_heads"}  # no kv heads, no rope_theta
    cfg_path.write_text(json.dumps(d))
    out = tmp_path / "model.bin"
    r = subprocess.run([tool, str(cfg_path), str(tmp_path / "in"), str(out), "1"], capture_output=True)
    assert r.returncode == 0, r.stderr
    head = np.fromfile(out, dtype=np.int32, count=8)
    assert list(head[:7]) == [CFG["dim"], CFG["hidden_dim"], CFG["n_layers"], CFG["n_heads"], CFG["n_heads"], CFG["vocab_size"], CFG["seq_len"]]
    assert head[7:8].view(np.float32)[0] == np.float32(10000.0)


def test_rejects_bad_inputs(tool, fixture, tmp_path):
    _dump_old(tmp_path / "in", fixture)
    _write_config(tmp_path / "config.json", CFG)
    out = tmp_path / "model.bin"
    # a truncated tensor file
    victim = tmp_path / "in" / "model.layers.1.mlp.down_proj.qzeros.bin"
    data = victim.read_bytes()
    victim.write_bytes(data[:-4])
    r = subprocess.run([tool, str(tmp_path / "config.json"), str(tmp_path / "in"), str(out), "1"], capture_output=True)
    assert r.returncode != 0 and b"down_proj.qzeros" in r.stderr
    victim.write_bytes(data)
    # a dimension the loader cannot read back
    bad = dict(CFG, dim=136)
    _write_config(tmp_path / "bad.json", bad)
    r = subprocess.run([tool, str(tmp_path / "bad.json"), str(tmp_path / "in"), str(out), "1"], capture_output=True)
    assert r.returncode != 0 and b"multiples of 32" in r.stderr
    # a missing mandatory key
    _write_config(tmp_path / "short.json", CFG, drop=("vocab_size",))
    r = subprocess.run([tool, str(tmp_path / "short.json"), str(tmp_path / "in"), str(out), "1"], capture_output=True)
    assert r.returncode != 0 and b"vocab_size" in r.stderr
    # wrong argument count prints the usage like the reference tool
    r = subprocess.run([tool], capture_output=True)
    assert r.returncode == 0 and b"usage: weight_packer" in r.stdout
