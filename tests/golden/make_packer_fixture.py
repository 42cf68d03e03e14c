"""Writes tests/golden/packer_fixture.npz: a tiny old-format AWQ checkpoint and the .bin that the REFERENCE's own
weight_packer (compiled from its source by oracle/Makefile into oracle/_ref/weight_packer) makes of it.

Run in the build container (needs oracle/_ref/weight_packer):  python tests/golden/make_packer_fixture.py
The fixture is data only: random input tensors and the bytes the reference tool wrote.
"""
import json
import os
import subprocess
import sys
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from llama_cu_awq_amd import packer, synth  # noqa: E402

CFG = dict(dim=128, hidden_dim=384, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=32, seq_len=32)
# hidden 384 = 3 groups: the zeros rows have 5 padding nibbles, which the reference tool fills with stale bytes


def main():
    tool = os.path.join(ROOT, "oracle", "_ref", "weight_packer")
    if not os.path.exists(tool):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "ref"])
    rng = np.random.default_rng(1234)
    dim, hid, V = CFG["dim"], CFG["hidden_dim"], CFG["vocab_size"]
    arrays = {}
    with tempfile.TemporaryDirectory() as d:
        with open(os.path.join(d, "config.json"), "w") as f:
            # the tool scrapes `"key":` without a space before the colon (weight_packer.cpp:22-72)
            f.write(json.dumps({"hidden_size": dim, "intermediate_size": hid, "num_hidden_layers": CFG["n_layers"], "num_attention_heads": CFG["n_heads"],
                                "num_key_value_heads": CFG["n_kv_heads"], "vocab_size": V, "max_position_embeddings": CFG["seq_len"], "rope_theta": 10000.0},
                               separators=(",", ":")))

        def dump(name, a):
            arrays[name] = a
            a.tofile(os.path.join(d, name + ".bin"))

        dump("model.embed_tokens.weight", rng.normal(0, 0.02, V * dim).astype(np.float16))
        dump("lm_head.weight", rng.normal(0, 0.02, V * dim).astype(np.float16))
        dump("model.norm.weight", (1 + rng.normal(0, 0.02, dim)).astype(np.float16))
        for l in range(CFG["n_layers"]):
            for name, K, N in (("self_attn.q_proj", dim, dim), ("self_attn.k_proj", dim, dim), ("self_attn.v_proj", dim, dim), ("self_attn.o_proj", dim, dim),
                               ("mlp.up_proj", dim, hid), ("mlp.gate_proj", dim, hid), ("mlp.down_proj", hid, dim)):
                G = (K + 127) // 128
                base = f"model.layers.{l}.{name}"
                dump(base + ".qweight", rng.integers(0, 2**32, size=(K, N // 8), dtype=np.uint32))
                dump(base + ".qzeros", rng.integers(0, 2**32, size=(G, N // 8), dtype=np.uint32))
                dump(base + ".scales", rng.uniform(0.002, 0.02, size=(G, N)).astype(np.float16))
            dump(f"model.layers.{l}.input_layernorm.weight", (1 + rng.normal(0, 0.02, dim)).astype(np.float16))
            dump(f"model.layers.{l}.post_attention_layernorm.weight", (1 + rng.normal(0, 0.02, dim)).astype(np.float16))
        out = os.path.join(d, "model.bin")
        subprocess.check_call([tool, os.path.join(d, "config.json"), d, out, "1"], stdout=subprocess.DEVNULL)
        ref_bin = np.fromfile(out, dtype=np.uint8)
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "packer_fixture.npz"), reference_bin=ref_bin, **arrays)
    print("wrote packer_fixture.npz:", ref_bin.nbytes, "bytes of reference output,", len(arrays), "input tensors")


if __name__ == "__main__":
    main()
