"""Writes tests/golden/tokenizer_vectors.txt: token ids and decoded pieces that the REFERENCE's tokenizer produces for a
list of texts (run in the build container; needs oracle/_ref/ref_tokenizer, built from the reference's tokenizer.h by
oracle/Makefile).  tests/golden/tokenizer.bin is the vocabulary data file the reference ships."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
TEXTS = [
    "",
    "Write a poem on GPUs",
    "Hello, world!",
    " leading space",
    "trailing space ",
    "two  spaces and\ttab",
    "line one\\nline two",
    "Tell me a story about a dragon who learns to program in C++ and HIP.",
    "naïve café déjà vu — “quotes” … ünïcödé",
    "日本語のテキスト",
    "emoji 🚀🔥 test",
    "1234567890 3.14159 0x1F",
    "[INST] <<SYS>>You are a helpful assistant<</SYS>> Hi [/INST]",
    "aaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaa",
    "The quick brown fox jumps over the lazy dog. THE QUICK BROWN FOX JUMPS OVER THE LAZY DOG.",
    "\x01\x02 control \x7f bytes",
]


def main():
    tool = os.path.join(ROOT, "oracle", "_ref", "ref_tokenizer")
    tok = os.path.join(ROOT, "tests", "golden", "tokenizer.bin")
    out = subprocess.run([tool, tok, "32000"], input=("\n".join(TEXTS) + "\n").encode("utf-8"), capture_output=True, check=True)
    with open(os.path.join(ROOT, "tests", "golden", "tokenizer_vectors.txt"), "wb") as f:
        f.write(("\n".join(TEXTS) + "\n").encode("utf-8"))
        f.write(b"====\n")
        f.write(out.stdout)
    print("wrote tokenizer_vectors.txt:", len(out.stdout), "bytes")


if __name__ == "__main__":
    main()
