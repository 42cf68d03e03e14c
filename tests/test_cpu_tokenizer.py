"""CPU test: the driver's tokenizer (llama_cu_awq_amd/csrc/driver/tokenizer.hpp) against golden vectors produced by
the reference's own tokenizer.h (tests/golden/make_tokenizer_vectors.py) on the vocabulary file the reference ships."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(ROOT, "tests", "golden")


def _tool():
    exe = os.path.join(ROOT, "llama_cu_awq_amd", "bin", "tokenize")
    src = os.path.join(ROOT, "llama_cu_awq_amd", "csrc", "driver", "tokenize_main.cpp")
    if not os.path.exists(exe):
        os.makedirs(os.path.dirname(exe), exist_ok=True)
        subprocess.check_call(["g++", "-O2", "-std=c++17", src, "-o", exe])
    return exe


def test_encode_and_decode_match_reference_vectors():
    raw = open(os.path.join(GOLD, "tokenizer_vectors.txt"), "rb").read()
    texts, want = raw.split(b"====\n", 1)
    got = subprocess.run([_tool(), os.path.join(GOLD, "tokenizer.bin"), "32000"], input=texts, capture_output=True, check=True).stdout
    assert got == want
    # sanity on the vectors themselves: every text starts with BOS, the empty text is BOS alone
    lines = want.decode().splitlines()
    enc = [l for l in lines if l.startswith("E")]
    assert enc[0] == "E 1" and all(l.startswith("E 1") for l in enc) and len(enc) == texts.count(b"\n")


def test_missing_tokenizer_file_is_reported():
    r = subprocess.run([_tool(), "/nonexistent/tokenizer.bin", "32000"], input=b"x\n", capture_output=True)
    assert r.returncode != 0 and b"couldn't load" in r.stderr
