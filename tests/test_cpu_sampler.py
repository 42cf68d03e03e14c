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


# ---------------------------------------------------------------------------------------------------------------------
# How much does the order of the fp16 additions in the reference's prefix sum matter?  (sampler.h:107-111 runs
# cub::DeviceScan::InclusiveSum on half data; CUB picks the order, the reference does not fix it.)  The oracle carries
# two such orders next to its own exact-sum definition; they are pinned here against numpy's float16 arithmetic and
# then compared with each other.

def _sorted_probs(probs):
    p = np.asarray(probs, dtype=np.float16)
    order = np.argsort(-p.astype(np.float32), kind="stable")
    return p[order], order


def _numpy_tiled_scan(ps, threads, items):
    """The tiled order written with numpy float16 operations (every + below rounds to fp16)."""
    out = np.empty_like(ps)
    carry = None
    tile = threads * items
    for base in range(0, ps.size, tile):
        chunk = ps[base:base + tile]
        owners = [chunk[t * items:(t + 1) * items] for t in range(threads)]
        owners = [o for o in owners if o.size]
        totals = [np.add.accumulate(o, dtype=np.float16)[-1] for o in owners]
        excl = []
        groups = carry
        for g in range(0, len(totals), 32):
            lanes = list(totals[g:g + 32])
            off = 1
            while off < 32:
                prev = list(lanes)
                for l in range(off, len(lanes)):
                    lanes[l] = np.float16(prev[l - off] + prev[l])
                off *= 2
            for l in range(len(lanes)):
                before = None if l == 0 else lanes[l - 1]
                if groups is None:
                    excl.append(before)
                else:
                    excl.append(groups if before is None else np.float16(groups + before))
            groups = lanes[-1] if groups is None else np.float16(groups + lanes[-1])
        for t, o in enumerate(owners):
            seeded = o if excl[t] is None else np.concatenate([[excl[t]], o]).astype(np.float16)
            acc = np.add.accumulate(seeded, dtype=np.float16)
            out[base + t * items: base + t * items + o.size] = acc if excl[t] is None else acc[1:]
        carry = groups
    return out


def _pick_from_prefix(prefix, order, threshold):
    hit = np.nonzero(prefix.astype(np.float32) >= np.float32(threshold))[0]
    return int(order[int(hit[0]) if hit.size else order.size - 1])


@pytest.mark.parametrize("n,scale", [(32000, 2.0), (4097, 1.0), (777, 3.0), (130, 0.5), (5, 1.0)])
def test_fp16_scan_orders_against_numpy_float16(n, scale):
    probs = oracle.softmax_logits(_logits(n, n, scale), 0.8)
    ps, order = _sorted_probs(probs)
    seq = np.add.accumulate(ps, dtype=np.float16)
    tiled = _numpy_tiled_scan(ps, 128, 16)
    small = _numpy_tiled_scan(ps, 32, 3)
    rng = np.random.default_rng(n)
    for threshold in list(rng.uniform(0, 1, 25)) + [0.0, 1.0, 1.5]:
        assert oracle.top_p_pick_fp16_scan(probs, threshold, 1, 0) == _pick_from_prefix(seq, order, threshold)
        assert oracle.top_p_pick_fp16_scan(probs, threshold, 1, 1, 128, 16) == _pick_from_prefix(tiled, order, threshold)
        assert oracle.top_p_pick_fp16_scan(probs, threshold, 1, 1, 32, 3) == _pick_from_prefix(small, order, threshold)
        # one thread holding everything is the sequential order
        assert oracle.top_p_pick_fp16_scan(probs, threshold, 1, 1, 1, n) == oracle.top_p_pick_fp16_scan(probs, threshold, 1, 0)


def test_fp16_scan_orders_agree_when_every_partial_sum_is_representable():
    # descending powers of two: every partial sum of every order fits 11 bits, so nothing rounds and all definitions agree
    p = np.array([2.0 ** -k for k in range(1, 11)] + [2.0 ** -10], dtype=np.float16)
    z = lambda: (np.zeros(4, dtype=np.int32), np.array([0], dtype=np.int32), np.array([0], dtype=np.int32))
    for threshold in np.linspace(0.0, 1.0, 41):
        want = oracle.sample_top_p(p, threshold, 1, *z())
        assert oracle.top_p_pick_fp16_scan(p, threshold, 1, 0) == want
        assert oracle.top_p_pick_fp16_scan(p, threshold, 1, 1, 4, 2) == want


def test_top_p_pick_depends_on_the_scan_order_and_by_how_much(capsys):
    """The measured figure: over vocabulary-sized distributions and thresholds coin * topp, how often the exact-sum
    definition (this library's), a sequential fp16 scan and two tilings of a CUB-style fp16 scan pick different
    tokens, and how far apart the picks are in the sorted order and in probability mass."""
    rng = np.random.default_rng(7)
    rows = []
    for n, scale, temp in [(32000, 8.0, 0.5), (32000, 6.0, 0.8), (32000, 4.0, 1.0), (32000, 2.0, 0.8), (32000, 1.0, 1.0), (4097, 1.0, 0.8)]:
        probs = oracle.softmax_logits(_logits(n + int(scale * 10), n, scale), temp)
        ps, order = _sorted_probs(probs)
        rank = np.empty(n, dtype=np.int64)
        rank[order] = np.arange(n)
        mass = np.cumsum(ps.astype(np.float64))
        N = 150
        diff_seq = diff_t16 = diff_t12 = diff_tt = stalled = 0
        rank_shift, mass_shift = [], []
        for _ in range(N):
            threshold = rng.uniform() * 0.9
            z = (np.zeros(4, dtype=np.int32), np.array([0], dtype=np.int32), np.array([0], dtype=np.int32))
            exact = oracle.sample_top_p(probs, threshold, 1, *z)
            seq = oracle.top_p_pick_fp16_scan(probs, threshold, 1, 0)
            t16 = oracle.top_p_pick_fp16_scan(probs, threshold, 1, 1, 128, 16)
            t12 = oracle.top_p_pick_fp16_scan(probs, threshold, 1, 1, 128, 12)
            diff_seq += exact != seq
            diff_t16 += exact != t16
            diff_t12 += exact != t12
            diff_tt += t16 != t12
            stalled += rank[seq] == n - 1
            for t in (t16, t12):
                rank_shift.append(abs(int(rank[exact]) - int(rank[t])))
                mass_shift.append(abs(mass[rank[exact]] - mass[rank[t]]))
        rows.append((n, scale, temp, float(probs.max()), diff_seq / N, diff_t16 / N, diff_t12 / N, diff_tt / N, stalled / N, max(rank_shift), max(mass_shift)))
    with capsys.disabled():
        print("\n n     scale T    p_max   exact!=seq exact!=128x16 exact!=128x12 128x16!=128x12 seq-stalls max-rank-shift max-mass-shift")
        for r in rows:
            print(" %-5d %-5.1f %-4.1f %-7.4f %-10.2f %-13.2f %-13.2f %-14.2f %-10.2f %-14d %.4f" % r)
    for n, scale, temp, pmax, d_seq, d16, d12, dtt, stalled, rshift, mshift in rows:
        # the tilings never move the pick by more than a few dozen places or two percent of probability mass ...
        assert rshift <= 64 and mshift <= 2e-2
        # ... and a peaked distribution leaves no room for any disagreement
        if pmax >= 0.7:
            assert d_seq == d16 == d12 == dtt == 0
    # on flat distributions the two tilings disagree with each other about as often as either disagrees with the exact
    # sum: the reference's own answer is a property of CUB's tuning for the GPU it runs on, not of the algorithm
    flat = [r for r in rows if r[3] < 0.06]
    assert all(r[7] > 0.25 * max(r[5], r[6]) for r in flat)
    # a strictly sequential fp16 sum stops growing once the terms fall below half an ulp of the running sum and then
    # never reaches the threshold: it falls through to the least likely token
    assert max(r[8] for r in flat) > 0.1
