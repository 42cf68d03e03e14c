"""CPU tests that pin the oracle's temperature / top-p sampler (sampler.h:65-115, gpu_kernels.h:507-592).

Independent checks: the xorshift* recurrence computed with Python integers; fp64 softmax; numpy's stable argsort with
integer cumulative sums (fp16 values are exact multiples of 2^-24) and numpy's own float16 rounding; hand-built
distributions whose crossing position is known in advance.
"""
import numpy as np
import pytest

from oracle import oracle


def test_random_f32_matches_integer_recurrence():
    state = np.array([1234567], dtype=np.uint64)
    s = 1234567
    mask = (1 << 64) - 1
    for _ in range(50):
        s ^= s >> 12
        s ^= (s << 25) & mask
        s ^= s >> 27
        want = ((((s * 0x2545F4914F6CDD1D) & mask) >> 32) >> 8) / 16777216.0
        got = oracle.random_f32(state)
        assert got == np.float32(want)
        assert int(state[0]) == s


def _logits(seed, n, scale):
    rng = np.random.default_rng(seed)
    return (rng.normal(0, scale, n)).astype(np.float16)


@pytest.mark.parametrize("n,temperature,scale", [(32000, 0.5, 2.0), (32000, 1.0, 4.0), (1000, 0.7, 1.0), (5, 0.3, 1.0), (1025, 2.0, 8.0)])
def test_softmax_logits_against_fp64(n, temperature, scale):
    l = _logits(1, n, scale)
    got = oracle.softmax_logits(l, temperature).astype(np.float64)
    t = (l.astype(np.float32) / np.float32(temperature)).astype(np.float16).astype(np.float64)  # first rounding point
    e = np.exp(t - t.max())
    want = e / e.sum()
    # two fp16 roundings (of exp and of the quotient): relative error <= ~2^-10 for normal values, absolute 2^-24 below
    assert np.all(np.abs(got - want) <= want * 1.2e-3 + 2.0 ** -24)
    assert abs(got.sum() - 1.0) < 2e-3


def _reference_pick(probs, threshold, sorted_):
    """Straight restatement with numpy: stable descending order, exact integer prefix, one rounding to fp16."""
    p = np.asarray(probs, dtype=np.float16)
    order = np.argsort(-p.astype(np.float32), kind="stable") if sorted_ else np.arange(p.size)
    units = np.round(p[order].astype(np.float64) * 2.0 ** 24).astype(np.int64)  # exact: multiples of 2^-24
    prefix = np.cumsum(units)
    # exact integer -> float64 (exact below 2^53) -> float16 with numpy's round-to-nearest-even
    rounded = (prefix.astype(np.float64) / 2.0 ** 24).astype(np.float16).astype(np.float32)
    hit = np.nonzero(rounded >= np.float32(threshold))[0]
    pos = int(hit[0]) if hit.size else p.size - 1
    return int(order[pos])


@pytest.mark.parametrize("sorted_", [0, 1])
@pytest.mark.parametrize("seed", range(6))
def test_sample_top_p_against_numpy(seed, sorted_):
    rng = np.random.default_rng(100 + seed)
    n = [32000, 32000, 4097, 777, 64, 3][seed]
    probs = oracle.softmax_logits(_logits(seed, n, [2.0, 6.0, 1.0, 3.0, 0.5, 1.0][seed]), 0.8)
    for threshold in list(rng.uniform(0, 1, 12)) + [0.0, 1e-8, 0.999, 1.0, 1.5]:
        tokens = np.zeros(8, dtype=np.int32)
        pos_h = np.array([2], dtype=np.int32)
        pos_d = np.array([2], dtype=np.int32)
        tok = oracle.sample_top_p(probs, threshold, sorted_, tokens, pos_h, pos_d)
        assert tok == _reference_pick(probs, threshold, sorted_), (n, threshold)
        assert tokens[3] == tok and pos_h[0] == 3 and pos_d[0] == 3


def test_sample_top_p_known_answers():
    # three quarters on token 5, the rest spread: the sorted order starts with token 5
    p = np.zeros(16, dtype=np.float16)
    p[5] = 0.75
    p[9] = 0.125
    p[2] = 0.125
    z = lambda: (np.zeros(4, dtype=np.int32), np.array([0], dtype=np.int32), np.array([0], dtype=np.int32))
    assert oracle.sample_top_p(p, 0.5, 1, *z()) == 5
    assert oracle.sample_top_p(p, 0.75, 1, *z()) == 5       # reaches the threshold exactly
    assert oracle.sample_top_p(p, 0.76, 1, *z()) == 2       # equal probabilities keep index order: 2 before 9
    assert oracle.sample_top_p(p, 0.9, 1, *z()) == 9
    assert oracle.sample_top_p(p, 1.5, 1, *z()) == 15       # never reached: last of the sorted order (a zero, largest index)
    assert oracle.sample_top_p(p, 0.1, 0, *z()) == 2        # index order
    assert oracle.sample_top_p(p, 0.2, 0, *z()) == 5
    assert oracle.sample_top_p(p, 0.9, 0, *z()) == 9
    assert oracle.sample_top_p(p, 1.5, 0, *z()) == 15
    # rounding of the prefix: 1 + 2^-11 rounds to 1 (tie to even), so a threshold just above 1 is not reached by it
    q = np.array([1.0, 2.0 ** -11, 2.0 ** -11], dtype=np.float16)
    assert oracle.sample_top_p(q, 1.0, 1, *z()) == 0
    assert oracle.sample_top_p(q, 1.0004, 1, *z()) == 2     # 1 + 2^-10 is representable and >= 1.0004? no: 1.000977 >= 1.0004
