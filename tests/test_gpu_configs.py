"""The benchmark's model configurations at their own sizes, against the CPU oracle.

The other model-level tests use models of a few layers and at most 192 positions.  These run the 7B, 13B and 33B
shapes and the 512-token prefill as the benchmark does: 32 / 40 / 60 layers, 52 heads, positions that cross the
128 -> 256 -> 512 sequence-length bins of the recorded launch sequences (llama2_q4.cu:553-575) and the switch from
the one-launch to the two-launch attention at 256 positions, a KV cache pre-filled to position 1536, split-K and
RoPE / SiLU epilogues of the batched GEMM at M = 512.

Bar: greedy tokens identical to the oracle's, logits within rel-L2 1e-2 (the benchmark definition) wherever the
model lets two correct implementations agree that closely.  With the benchmark's weight distributions a 32-layer model
does not: attention scores have a standard deviation of about 30, so the softmax is close to an argmax and a
difference of one fp16 step in a score moves probabilities by 6 %.  The oracle run twice, once with the reference's
fp32 summation order and once with every matrix-vector sum rounded once from double precision (the value any fp32
order approximates), gives logits 0.4 % apart at position 0 and 1 - 3 % apart from position 10 on.  Each model's
bar is therefore derived from that measured distance (`_conditioning`): 1e-2 where the model is well conditioned,
a multiple of the oracle's own sensitivity where it is not.  One full-size model with a narrower scale range (well
conditioned) is held to 1e-2 outright.  Where the oracle would take minutes (60 layers, 512-token prompts through 32
layers) the check is a property the GPU paths must share among themselves, stated at the test.
"""
import os

import numpy as np
import pytest

import llama_cu_awq_amd as A
from llama_cu_awq_amd import synth
from oracle import oracle
from tests.helpers import f16, rel_l2

pytestmark = pytest.mark.gpu

THREADS = min(16, os.cpu_count() or 8)


def _kv_dim(cfg):
    return cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"]


def _prefill_kv_both(t, o, cfg, seed, upto):
    """N(0,1) keys and values below position `upto` in every layer, identical on the GPU and in the oracle."""
    kv_dim, seq, L = _kv_dim(cfg), cfg["seq_len"], cfg["n_layers"]
    for name in ("key_cache", "value_cache"):
        dev = t.buffer(name, L * seq * kv_dim * 2)
        host = o.buffer(name, L * seq * kv_dim).reshape(L, seq, kv_dim) if o is not None else None
        for l in range(L):
            vals = synth.normal_f16(synth.stream_key(seed, name, l), upto * kv_dim)
            dev.write(vals, offset_bytes=l * seq * kv_dim * 2)
            if host is not None:
                host[l, :upto] = vals.view(np.uint16).reshape(upto, kv_dim)


def _oracle_record(o, n_prompt, steps, first_pos=0):
    """Run `steps` passes of the oracle from its current state; per pass the logits and (once the prompt is consumed)
    the token it wrote.  Pass i runs at position first_pos + i."""
    vocab = o.config["vocab_size"]
    rec = []
    for i in range(steps):
        gen = i >= n_prompt - 1
        o.forward(gen)
        pos = first_pos + i
        rec.append((f16(o.buffer("logits", vocab)).copy(), o.tokens(pos + 2)[pos + 1] if gen else None))
    return rec


def _conditioning(o, ref, n_prompt, first_pos=0):
    """How far the oracle's logits move when its matrix-vector sums are rounded once from double precision instead
    of being added in the reference's fp32 order: the same passes again from the oracle's state before `ref` was
    recorded (the caller restores that state), kept on ref's tokens.  Returns the per-pass rel-L2 distances and the
    logits of the exactly summed passes."""
    vocab = o.config["vocab_size"]
    dist, exact = [], []
    oracle.set_exact_sums(True)
    try:
        for i, (want_logits, want_tok) in enumerate(ref):
            gen = i >= n_prompt - 1
            o.forward(gen)
            pos = first_pos + i
            exact.append(f16(o.buffer("logits", vocab)).copy())
            dist.append(rel_l2(exact[-1], want_logits))
            if gen and o.tokens(pos + 2)[pos + 1] != want_tok:
                o.set_pos(pos + 1, int(want_tok))
    finally:
        oracle.set_exact_sums(False)
    return dist, exact


# How much farther from the exactly summed logits than the reference's own fp32 order a GPU run may be.  Any fp32
# summation order is one sample of the same rounding noise, amplified through 32 to 60 layers of near-argmax softmax by
# a factor that differs from pass to pass; and the passes of a run share their history (each reads the KV rows its
# predecessors wrote), so a run is one sample of a trajectory, not 16 or 48 independent ones.  Measured over the five
# scenarios below the ratio GPU / reference order of the median distance is 0.99 .. 1.54 and of the worst pass
# 0.89 .. 2.05.  The comparison is therefore between the two runs' distributions over the passes: median and mean
# within EXACT_FACTOR, the worst pass within EXACT_WORST of the reference order's worst.  Position 0 (no attention,
# nothing amplified, no history) is compared on its own by the callers that start there, and the arithmetic of a
# single product is held much tighter in tests/test_gpu_ops.py (how many outputs round differently from the exact sum).
EXACT_FACTOR = 2.0
EXACT_WORST = 2.5


def _check_against_exact(rec, exact, dist, what):
    """The comparison the arithmetic fixes, whatever the model's conditioning: the GPU's logits are no farther from the
    exactly summed ones (every matrix-vector sum rounded once from double precision, same token history) than the
    reference's fp32 summation order is."""
    g = [rel_l2(logits, ex) for (logits, _), ex in zip(rec, exact)]
    med_g, med_d = float(np.median(g)), float(np.median(dist))
    print(f"{what}: distance from exactly summed logits, GPU / the reference's fp32 order, per pass:")
    print("  " + " ".join(f"{a:.4f}/{b:.4f}" for a, b in zip(g, dist)))
    print(f"  GPU worst {max(g):.4g} mean {np.mean(g):.4g} median {med_g:.4g}; reference order worst {max(dist):.4g} "
          f"mean {np.mean(dist):.4g} median {med_d:.4g}")
    assert med_g <= EXACT_FACTOR * med_d, (med_g, med_d)
    assert float(np.mean(g)) <= EXACT_FACTOR * float(np.mean(dist)), (float(np.mean(g)), float(np.mean(dist)))
    assert max(g) <= EXACT_WORST * max(dist), (max(g), max(dist))
    return g


def _bars(dist):
    """(per-pass bar, median bar) for GPU-vs-oracle logits from the oracle's own sensitivity `dist`: two
    implementations that each differ from the exactly rounded sums by about that much differ from each other by more
    (independent differences, different exponentials), hence the factors; never below the benchmark's 1e-2."""
    return max(1e-2, 4 * max(dist)), max(1e-2, 2.5 * float(np.median(dist)))


def _gpu_record(t, n_prompt, steps, use_graph, mode, first_pos=0, ref=None, bar=1e-2):
    """The same passes on the GPU (synchronise, launch, read back: the reference loop).  With `ref` (a record of the
    oracle or of another GPU run) every pass is compared with it: the rel-L2 distance of the logits is returned for the
    caller to hold against its bar, and the greedy token must be the same or a tie as defined below.

    Random weights put the largest of 32000 fp16 logits a few fp16 steps apart, and exact ties are common (the
    oracle's own 7B run has five among its first 32 generated tokens; it breaks them by lowest index), so two correct
    implementations that add in a different order cannot agree on every token.  A different token is accepted as a tie
    only when the reference's own logits of the two tokens are closer than 4 * bar * rms(logits) (four standard
    deviations of the per-logit difference that the logits bar `bar` allows: 13 fp16 steps at the benchmark's 1e-2)
    AND within twice the largest logit difference between the two runs at that pass, i.e. when the flip is explained
    by differences inside the logits bar.  The GPU is then put back on the reference's token so that the comparison
    goes on over the same history.  Returns (record, per-pass rel-L2, number of ties)."""
    vocab = t.config["vocab_size"]
    rec, errs, ties = [], [], 0
    for i in range(steps):
        gen = i >= n_prompt - 1
        pos = first_pos + i
        t.ctx.sync()
        t.forward(gen, use_graph, mode)
        t.ctx.sync()
        assert t.pos == pos + 1
        logits = f16(t.download("logits", vocab))
        tok = t.token(pos + 1) if gen else None
        if ref is not None:
            want_logits, want_tok = ref[i]
            errs.append(rel_l2(logits, want_logits))
            if gen and tok != want_tok:
                a, b = float(want_logits[want_tok]), float(want_logits[tok])
                margin = abs(a - b)
                step = float(np.spacing(np.float16(max(abs(a), abs(b)))))
                apart = float(np.abs(logits.astype(np.float64) - want_logits.astype(np.float64)).max())
                rms = float(np.sqrt(np.mean(want_logits.astype(np.float64) ** 2)))
                assert margin <= 4 * bar * rms and margin <= 2 * apart, (
                    f"pass {i} (position {pos}): token {tok}, reference {want_tok}; their reference logits {a} and {b} are "
                    f"{margin / step:.0f} fp16 steps apart, largest logit difference between the runs {apart:.4g}")
                ties += 1
                print(f"tie at position {pos}: {tok} for {want_tok}, reference margin {margin / step:.0f} fp16 steps")
                t.set_pos(pos + 1, int(want_tok))
                tok = want_tok
        rec.append((logits, tok))
    if ref is not None:
        print(f"{steps} passes from position {first_pos}: logits rel-L2 worst {max(errs):.3g}, median {np.median(errs):.3g}; {ties} ties")
    return rec, errs, ties


def _check(errs, bars):
    assert max(errs) <= bars[0], (max(errs), bars)
    assert float(np.median(errs)) <= bars[1], (float(np.median(errs)), bars)


# ------------------------------------------------------------------ 7B shape (32 layers, 32 heads)
@pytest.fixture(scope="module")
def model_7b(ctx):
    img = synth.make_model_image(synth.CONFIG_7B, seed=0, threads=THREADS)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    yield synth.CONFIG_7B, t, o, {}
    t.close()
    o.close()


def _bars_7b(model_7b):
    """The 7B model's bars (and the oracle record they come from), computed on first use: the oracle's 16 + 32 passes
    in the reference's summation order, then again with sums rounded once."""
    cfg, _, o, shared = model_7b
    if "bars" not in shared:
        n_prompt, steps = 16, 16 + 32
        prompt = synth.prompt_tokens(0, n_prompt, cfg["vocab_size"])
        o.reset(prompt)
        ref = _oracle_record(o, n_prompt, steps)
        assert all(np.isfinite(l.astype(np.float32)).all() for l, _ in ref)
        o.reset(prompt)
        dist, exact = _conditioning(o, ref, n_prompt)
        print(f"oracle, reference summation order vs sums rounded once: logits rel-L2 worst {max(dist):.3g}, median {np.median(dist):.3g}")
        assert max(dist) > 1e-2  # the reason for the derived bar; if this stops holding, hold the run to 1e-2 outright
        shared["bars"] = _bars(dist)
        shared["ref"] = (prompt, ref)
        shared["exact"] = (dist, exact)
    return shared["bars"]


def test_7b_prompt_then_32_greedy_steps(model_7b):
    """The benchmark run's first 48 positions: 16 prompt tokens, 32 generated, fused schedule under graph replay."""
    cfg, t, o, shared = model_7b
    n_prompt, steps = 16, 16 + 32
    _bars_7b(model_7b)
    prompt, ref = shared["ref"]
    t.reset(prompt)
    rec, errs, ties = _gpu_record(t, n_prompt, steps, True, A.SCHEDULE_FUSED, ref=ref, bar=shared["bars"][0])
    _check(errs, shared["bars"])
    g = _check_against_exact(rec, shared["exact"][1], shared["exact"][0], "7B shape, 16 prompt + 32 generated tokens")
    assert errs[0] <= 1e-2  # position 0 has no attention to amplify anything:
    assert g[0] <= 1.5 * shared["exact"][0][0]  # there the single pass is comparable
    assert [t.token(i) for i in range(n_prompt)] == prompt
    assert [tok for _, tok in rec] == [tok for _, tok in ref]
    assert ties <= 10, ties  # the oracle's own 32 steps have 5 pairs of top logits within 2 fp16 steps, 3 of them exact ties


@pytest.mark.parametrize("start", [120, 250])
def test_7b_decode_across_sequence_length_bins(model_7b, start):
    """16 steps from a pre-filled cache at 120 (bin 128 -> 256) and at 250 (bin 256 -> 512, which is also where the
    one-launch attention hands over to the two-launch form), eagerly and under graph replay; set_pos on both sides."""
    cfg, t, o, shared = model_7b
    steps = 16
    bars = _bars_7b(model_7b)
    tok0 = synth.prompt_tokens(start, 1, cfg["vocab_size"])[0]
    o.reset([tok0])
    t.reset([tok0])
    _prefill_kv_both(t, o, cfg, seed=start, upto=start)
    o.set_pos(start, tok0)
    ref = _oracle_record(o, 1, steps, first_pos=start)
    o.set_pos(start, tok0)
    dist, exact = _conditioning(o, ref, 1, first_pos=start)
    for use_graph in (False, True):
        t.set_pos(start, tok0)  # the rows from `start` on are rewritten by the passes themselves
        rec, errs, ties = _gpu_record(t, 1, steps, use_graph, A.SCHEDULE_FUSED, first_pos=start, ref=ref, bar=bars[0])
        assert t.pos == start + steps
        _check(errs, bars)
        _check_against_exact(rec, exact, dist, f"7B shape, 16 passes from position {start}")
        assert ties <= 4, ties


def test_7b_back_to_back_passes_without_synchronising(model_7b):
    """Passes issued back to back (no stream synchronisation between them) across the 128-position bin edge and the
    256-position attention switch give the tokens of the synchronised loop: the launch sizes come from the host-side
    count of issued passes, not from the pinned position."""
    cfg, t, _, _ = model_7b
    tok0 = synth.prompt_tokens(5, 1, cfg["vocab_size"])[0]
    runs = []
    for sync_each in (True, False):
        for start, steps in ((122, 12), (250, 12)):
            t.reset([tok0])
            _prefill_kv_both(t, None, cfg, seed=9, upto=start)
            t.set_pos(start, tok0)
            for i in range(steps):
                if sync_each:
                    t.ctx.sync()
                t.forward(True, False, A.SCHEDULE_FUSED)
            t.ctx.sync()
            assert t.pos == start + steps
            runs.append([t.token(start + 1 + i) for i in range(steps)])
    assert runs[0] == runs[2] and runs[1] == runs[3]


def test_7b_prefill_512_equals_token_by_token_decode(model_7b):
    """All 32 layers, 512 prompt tokens in one batched pass against the GPU's own single-token passes (which the
    tests above tie to the oracle): KV rows and last-token logits within 1e-2, same next token."""
    cfg, t, _, shared = model_7b
    M = 512
    prompt = synth.prompt_tokens(1, M, cfg["vocab_size"])
    kv_dim, seq, L, vocab = _kv_dim(cfg), cfg["seq_len"], cfg["n_layers"], cfg["vocab_size"]
    layers = (0, 1, 15, 31)

    def snapshot():
        rows = {}
        for name in ("key_cache", "value_cache"):
            buf = t.buffer(name, L * seq * kv_dim * 2)
            for l in layers:
                rows[name, l] = f16(buf.download(np.uint16, M * kv_dim, offset_bytes=l * seq * kv_dim * 2))
        return rows, f16(t.download("logits", vocab)), t.token(M)

    t.reset(prompt)
    for i in range(M):
        t.forward(i >= M - 1, True, A.SCHEDULE_FUSED)
    t.ctx.sync()
    assert t.pos == M
    want_rows, want_logits, want_next = snapshot()
    t.reset(prompt)
    t.prefill(M, gen_token=True)
    t.ctx.sync()
    assert t.pos == M
    got_rows, got_logits, got_next = snapshot()
    assert np.isfinite(want_logits.astype(np.float32)).all()
    bar = _bars_7b(model_7b)[0]  # 512 positions through 32 layers: the ill-conditioned model's bar
    for key in want_rows:
        assert rel_l2(got_rows[key], want_rows[key]) <= (1e-3 if key[1] == 0 else bar), key
    assert rel_l2(got_logits, want_logits) <= bar
    # same next token, unless the two largest logits are closer than the two runs' logits are to each other
    top2 = np.sort(want_logits.astype(np.float64))[-2:]
    apart = np.abs(got_logits.astype(np.float64) - want_logits.astype(np.float64)).max()
    assert got_next == want_next or top2[1] - top2[0] <= 2 * apart


def test_7b_shape_well_conditioned_model_meets_1e_2(ctx):
    """All 32 layers at the 7B shape with an eighth of the benchmark's scale range (attention scores of order 1, so
    rounding differences are not amplified): the benchmark's bar as stated, 8 prompt + 16 generated tokens."""
    cfg = dict(synth.CONFIG_7B, seq_len=256)
    img = synth.make_model_image(cfg, seed=6, threads=THREADS, scale_mult=0.125)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    try:
        n_prompt, steps = 8, 8 + 16
        prompt = synth.prompt_tokens(6, n_prompt, cfg["vocab_size"])
        o.reset(prompt)
        ref = _oracle_record(o, n_prompt, steps)
        for mode, graph in ((A.SCHEDULE_FUSED, True), (A.SCHEDULE_REFERENCE, False)):
            t.reset(prompt)
            _, errs, ties = _gpu_record(t, n_prompt, steps, graph, mode, ref=ref)
            assert max(errs) <= 1e-2, (mode, graph, max(errs))
            assert ties <= 4, ties
    finally:
        t.close()
        o.close()


# ------------------------------------------------------------------ 7B-shape layers, 512-token prefill vs the oracle
def test_7b_shape_prefill_512_matches_token_by_token_oracle(ctx):
    """dim 4096 / hidden 11008 / 32 heads with 2 layers: every GEMM of the 512-token prefill at its 7B shape (QKV with
    RoPE in the epilogue, O and down with K split in two, gate/up with the SiLU hand-over, causal attention over 512
    positions on the matrix cores) against the oracle run token by token.  A quarter of the benchmark's scale range:
    with the full range attention over 500 positions amplifies rounding differences past 1e-2 in two layers (the
    decode steps after the prefill come out 1.0 - 1.4e-2 from the oracle), and this test is about the batched path
    meeting the bar as stated."""
    cfg = dict(synth.CONFIG_7B, n_layers=2, seq_len=640)
    M = 512
    img = synth.make_model_image(cfg, seed=4, threads=THREADS, scale_mult=0.25)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    try:
        prompt = synth.prompt_tokens(4, M, cfg["vocab_size"])
        o.reset(prompt)
        for i in range(M):
            o.forward(i >= M - 1)
        t.reset(prompt)
        t.prefill(M, gen_token=True)
        ctx.sync()
        assert t.pos == M == o.pos
        kv_dim, seq, L = _kv_dim(cfg), cfg["seq_len"], cfg["n_layers"]
        for name in ("key_cache", "value_cache"):
            got = f16(t.download(name, L * seq * kv_dim)).reshape(L, seq, kv_dim)[:, :M]
            want = f16(o.buffer(name, L * seq * kv_dim)).reshape(L, seq, kv_dim)[:, :M]
            for l in range(L):
                assert rel_l2(got[l], want[l]) <= 1e-2, (name, l)
                # no row is off on its own (a misplaced tile or position would hide in the aggregate)
                err = np.linalg.norm(got[l].astype(np.float64) - want[l].astype(np.float64), axis=1)
                ref = np.linalg.norm(want[l].astype(np.float64), axis=1)
                assert (err <= 2e-2 * ref).all(), (name, l, int(np.argmax(err / ref)))
        assert rel_l2(f16(t.download("logits", cfg["vocab_size"])), f16(o.buffer("logits", cfg["vocab_size"]))) <= 1e-2
        want_logits = f16(o.buffer("logits", cfg["vocab_size"]))
        want_next, got_next = o.tokens(M + 1)[M], t.token(M)
        if got_next != want_next:  # only as a tie of the oracle's own logits (see _gpu_record)
            a, b = np.float16(want_logits[want_next]), np.float16(want_logits[got_next])
            assert abs(float(a) - float(b)) <= 2 * float(np.spacing(np.float16(max(abs(a), abs(b)))))
            t.set_pos(M, int(want_next))
        # decoding continues from the prefilled state and keeps matching the oracle
        ref = _oracle_record(o, 1, 4, first_pos=M)
        _, errs, _ = _gpu_record(t, 1, 4, False, A.SCHEDULE_FUSED, first_pos=M, ref=ref)
        assert max(errs) <= 1e-2
    finally:
        t.close()
        o.close()


# ------------------------------------------------------------------ 13B shape, long context
def test_13b_decode_from_kv_prefilled_to_1536(ctx):
    """40 layers, 40 heads, K = 5120 / 13824; cache pre-filled with N(0,1) below position 1536 as the benchmark's
    long-context configuration does; 6 greedy steps, eagerly and under graph replay."""
    cfg = synth.CONFIG_13B
    start, steps = 1536, 6
    img = synth.make_model_image(cfg, seed=0, threads=THREADS)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    try:
        tok0 = synth.prompt_tokens(13, 1, cfg["vocab_size"])[0]
        t.reset([tok0])
        o.reset([tok0])
        _prefill_kv_both(t, o, cfg, seed=13, upto=start)
        t.set_pos(start, tok0)
        o.set_pos(start, tok0)
        ref = _oracle_record(o, 1, steps, first_pos=start)
        assert all(np.isfinite(l.astype(np.float32)).all() for l, _ in ref)
        o.set_pos(start, tok0)
        dist, exact = _conditioning(o, ref, 1, first_pos=start)
        print(f"oracle, reference summation order vs sums rounded once: logits rel-L2 worst {max(dist):.3g}, median {np.median(dist):.3g}")
        for use_graph in (False, True):
            t.set_pos(start, tok0)  # the rows from `start` on are rewritten by the passes themselves
            rec, errs, ties = _gpu_record(t, 1, steps, use_graph, A.SCHEDULE_FUSED, first_pos=start, ref=ref, bar=_bars(dist)[0])
            _check(errs, _bars(dist))
            _check_against_exact(rec, exact, dist, "13B shape from a cache pre-filled to 1536")
            assert ties <= 2, ties
    finally:
        t.close()
        o.close()


# ------------------------------------------------------------------ 33B shape (52 heads, K = 6656 / 17920)
# With the benchmark's scale range U[0.002, 0.02] the residual stream of a 60-layer model leaves fp16 range (on the
# GPU and in the oracle alike), so these models use half that range; shapes and layouts are unchanged.
SCALE_33B = 0.5


def test_33b_shape_four_layers_matches_oracle(ctx):
    cfg = dict(synth.CONFIG_33B, n_layers=4, seq_len=256)
    img = synth.make_model_image(cfg, seed=3, threads=THREADS, scale_mult=SCALE_33B)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    try:
        n_prompt, steps = 8, 8 + 24
        prompt = synth.prompt_tokens(33, n_prompt, cfg["vocab_size"])
        o.reset(prompt)
        ref = _oracle_record(o, n_prompt, steps)
        assert all(np.isfinite(l.astype(np.float32)).all() for l, _ in ref)
        for mode, graph in ((A.SCHEDULE_FUSED, True), (A.SCHEDULE_REFERENCE, False)):
            t.reset(prompt)
            _, errs, ties = _gpu_record(t, n_prompt, steps, graph, mode, ref=ref)
            assert max(errs) <= 1e-2, (mode, graph, max(errs))
            assert ties <= 6, ties
    finally:
        t.close()
        o.close()


def test_70b_shape_grouped_queries_four_layers_matches_oracle(ctx):
    """Llama-2-70B's layer shape (dim 8192, hidden 28672, 64 heads sharing 8 KV heads), four layers: the grouped-query
    branch of the reference's schedule (llama2_q4.cu:457-464) against the single fused launch, rows of 28672 elements in
    the down projection, and attention heads that share their key and value rows."""
    cfg = dict(dim=8192, hidden_dim=28672, n_layers=4, n_heads=64, n_kv_heads=8, vocab_size=32000, seq_len=256, rope_theta=10000.0)
    img = synth.make_model_image(cfg, seed=70, threads=THREADS, scale_mult=0.35)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    try:
        n_prompt, steps = 6, 6 + 14
        prompt = synth.prompt_tokens(70, n_prompt, cfg["vocab_size"])
        o.reset(prompt)
        ref = _oracle_record(o, n_prompt, steps)
        assert all(np.isfinite(l.astype(np.float32)).all() for l, _ in ref)
        for mode, graph in ((A.SCHEDULE_FUSED, True), (A.SCHEDULE_REFERENCE, False)):
            t.reset(prompt)
            _, errs, ties = _gpu_record(t, n_prompt, steps, graph, mode, ref=ref)
            assert max(errs) <= 1e-2, (mode, graph, max(errs))
            assert ties <= 4, ties
    finally:
        t.close()
        o.close()


def test_405b_shape_grouped_queries_two_layers_matches_oracle(ctx):
    """Llama-3.1-405B's layer shape (dim 16384, hidden 53248, 128 heads sharing 8 KV heads), two layers: rows of 53248
    elements in the down projection take 113 KB of LDS per workgroup, beyond the 64 KB a kernel may use unless its limit
    is raised; the first launches here are recorded ones."""
    cfg = dict(dim=16384, hidden_dim=53248, n_layers=2, n_heads=128, n_kv_heads=8, vocab_size=4096, seq_len=128, rope_theta=500000.0)
    img = synth.make_model_image(cfg, seed=405, threads=THREADS, scale_mult=0.25)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    try:
        n_prompt, steps = 4, 4 + 8
        prompt = synth.prompt_tokens(405, n_prompt, cfg["vocab_size"])
        o.reset(prompt)
        ref = _oracle_record(o, n_prompt, steps)
        assert all(np.isfinite(l.astype(np.float32)).all() for l, _ in ref)
        for mode, graph in ((A.SCHEDULE_FUSED, True), (A.SCHEDULE_FUSED, False), (A.SCHEDULE_REFERENCE, False)):
            t.reset(prompt)
            _, errs, ties = _gpu_record(t, n_prompt, steps, graph, mode, ref=ref)
            assert max(errs) <= 1e-2, (mode, graph, max(errs))
            assert ties <= 3, ties
    finally:
        t.close()
        o.close()


def test_33b_full_model_schedules_agree_and_stay_finite(ctx):
    """All 60 layers (17.5 GB of weights on the one GPU): the oracle would need minutes, so the check is that the two
    multi-kernel schedules, which share no matrix-vector launch geometry for the norm-fused steps, produce the same
    16 greedy tokens with finite logits, eagerly and under graph replay, plus 3 generated tokens of the oracle itself."""
    cfg = synth.CONFIG_33B
    img = synth.make_model_image(cfg, seed=3, threads=THREADS, scale_mult=SCALE_33B)
    t = A.Transformer(ctx, image=img)
    o = oracle.Model(img)
    try:
        n_prompt, steps = 4, 4 + 16
        prompt = synth.prompt_tokens(34, n_prompt, cfg["vocab_size"])
        t.reset(prompt)
        base, _, _ = _gpu_record(t, n_prompt, steps, False, A.SCHEDULE_REFERENCE)
        assert all(np.isfinite(l.astype(np.float32)).all() for l, _ in base)
        o.reset(prompt)
        ref = _oracle_record(o, n_prompt, n_prompt + 3)
        o.reset(prompt)
        dist, exact = _conditioning(o, ref, n_prompt)
        print(f"oracle, reference summation order vs sums rounded once: logits rel-L2 worst {max(dist):.3g}, median {np.median(dist):.3g}")
        bars = _bars(dist)
        for graph in (False, True):
            t.reset(prompt)
            _, errs, ties = _gpu_record(t, n_prompt, steps, graph, A.SCHEDULE_FUSED, ref=base, bar=bars[0])
            _check(errs, bars)
            assert ties <= 4, ties
        t.reset(prompt)
        rec, errs, _ = _gpu_record(t, n_prompt, n_prompt + 3, True, A.SCHEDULE_FUSED, ref=ref, bar=bars[0])
        _check(errs, bars)
        _check_against_exact(rec, exact, dist, "33B shape, all 60 layers, half the scale range")
    finally:
        t.close()
        o.close()
