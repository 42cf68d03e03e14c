#!/usr/bin/env python3
"""Benchmark: batch-1 greedy decode of a Llama-2-7B-shape AWQ int4-g128 model on one MI355X.

A step is one token through the whole network (one pass of the hot path).  The default run consumes a 16-token
random prompt as warm-up and times exactly 256 decode steps; weights are random (no checkpoints offline) with the
real layout and distributions, resident in HBM before the timed region starts.

Prints ONE JSON line: tokens/s (`value`) of the run the flags ask for; `config1`, the benchmark's own run (16-token
prompt + 256 decode steps from position 0) whatever the flags were; `config2` and `config3`, 256 decode steps of the 13B
shape from a KV cache pre-filled to position 1536 and of the 33B shape; `shape_70b`, 128 steps of Llama-2-70B's shape
(grouped queries, 36.6 GB packed; not one of the benchmark's configurations); the roofline of the dominant kernel as the timed
schedule launches it (RMSNorm-fused gate/up int4 matrix-vector product, timed live with HIP events over the 32
layers' distinct weights); `config0`, the single 4096 x 4096 product back to back on one stream and dealt over 2 and 4
plain streams; the 512-token prefill; and the CPU oracle timed on a bounded sample of the same workload.
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # MI355X published HBM3E bandwidth, bytes/s

# Figures that cannot be measured inside this process (hardware counters, profiler durations) are read, at run time,
# from the rocprofv3 summaries committed under profiles/: the table rows of the kernels named here.
TRACE_MD = "profiles/decode_7b_fused_kernel_trace.md"
PMC_MD = "profiles/gemv_int4_ffn_7b_pmc.md"
FFN_KERNEL = "gemv_int4_kernel<4, 1, 2, 2, true, false, false, 1>"  # norm-fused gate/up, the launch of the fused schedule
GEMV_4096_KERNEL = "gemv_int4_kernel<8, 1, 2, 0, false, false, false, 1>"  # O projection and the 4096 x 4096 loops
COPY_ROW = "__amd_rocclr_copyBuffer, 256 MiB"


def _table_row(path, starts_with):
    """Cells (stripped) of the first markdown table row of `path` whose first cell starts with `starts_with`."""
    with open(os.path.join(ROOT, path)) as f:
        for line in f:
            if line.startswith("|"):
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if cells and cells[0].startswith(starts_with):
                    return cells
    raise KeyError(f"{path}: no table row for {starts_with}")


def profiled_figures():
    """rocprofv3 figures of the 7B-shape kernels from the committed summaries: average kernel durations (us) of the
    kernel trace, and the HBM bytes per launch of the roofline kernel from the FETCH_SIZE / WRITE_SIZE counters (KiB per
    dispatch), each scaled by what the same counter reads for a 256 MiB device copy."""
    num = lambda c: float(c.replace(",", ""))
    ffn_us = num(_table_row(TRACE_MD, FFN_KERNEL)[2])
    gemv_us = num(_table_row(TRACE_MD, GEMV_4096_KERNEL)[2])
    copy = _table_row(PMC_MD, COPY_ROW)
    ffn = _table_row(PMC_MD, FFN_KERNEL)
    fetch_scale = 262144.0 / num(copy[2])  # KiB actually read by the copy / KiB the counter shows for it
    write_scale = 262144.0 / num(copy[3])
    fetch_scale, write_scale = round(fetch_scale, 1), round(write_scale, 1)  # the factors as the summary states them
    traffic = int(round((num(ffn[2]) * fetch_scale + num(ffn[3]) * write_scale) * 1024))
    return {"ffn_kernel_us": ffn_us, "gemv_4096_kernel_us": gemv_us, "ffn_traffic_bytes": traffic,
            "fetch_scale": fetch_scale, "write_scale": write_scale}


def qweight_bytes(K, N):
    sh = (K + 127) // 128
    return N * (((K + 31) // 32) * 16 + ((sh + 7) // 8) * 4 + sh * 2)


def weight_bytes_per_token(cfg):
    dim, hid, L, V = cfg["dim"], cfg["hidden_dim"], cfg["n_layers"], cfg["vocab_size"]
    kv_dim = dim * cfg["n_kv_heads"] // cfg["n_heads"]
    layer = 2 * qweight_bytes(dim, dim) + 2 * qweight_bytes(dim, kv_dim) + 2 * qweight_bytes(dim, hid) + qweight_bytes(hid, dim) + 4 * dim
    return L * layer + 2 * V * dim + 2 * dim + 2 * dim  # + classifier + final norm + one embedding row


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", default="7b", choices=["7b", "13b", "33b", "70b"])
    ap.add_argument("--scale-mult", type=float, default=None, help="multiplies the weights' scale range U[0.002, 0.02]; default 1.0, 0.5 for --config 33b and 0.25 for 70b (60 and 80 layers leave fp16 range at 1.0)")
    ap.add_argument("--start-pos", type=int, default=0, help="pre-fill the KV cache with N(0,1) up to this position first")
    ap.add_argument("--schedule", default="fused", choices=["persistent", "fused", "reference"])
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=12, help="tokens of the same model timed on the CPU oracle (0 = skip)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--prefill", type=int, default=512, help="also time a batched prefill of this many prompt tokens (0 = skip)")
    ap.add_argument("--no-extra-configs", action="store_true", help="skip the 13B-shape and 33B-shape runs that a 7B run appends")
    ap.add_argument("--only-kernels", action="store_true", help="skip the decode loop: run only the per-kernel loops and a 256 MiB device copy (for counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the whole model on ONE GPU (no collectives); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np

    import llama_cu_awq_amd as A
    from llama_cu_awq_amd import synth

    cfg = {"7b": synth.CONFIG_7B, "13b": synth.CONFIG_13B, "33b": synth.CONFIG_33B, "70b": synth.CONFIG_70B}[args.config]
    n_prompt = max(1, args.warmup)
    total = n_prompt + args.steps
    assert args.start_pos + total <= cfg["seq_len"], "warmup + steps exceeds seq_len"
    mode = {"persistent": A.SCHEDULE_PERSISTENT, "fused": A.SCHEDULE_FUSED, "reference": A.SCHEDULE_REFERENCE}[args.schedule]
    use_graph = not args.no_graph

    t0 = time.time()
    scale_mult = args.scale_mult if args.scale_mult is not None else {"33b": 0.5, "70b": 0.25}.get(args.config, 1.0)
    image = synth.make_model_image(cfg, seed=args.seed, threads=min(16, os.cpu_count() or 8), scale_mult=scale_mult)
    print(f"[bench] model image {image.nbytes / 1e9:.2f} GB generated in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    ctx = A.Context(0)
    t0 = time.time()
    model = A.Transformer(ctx, image=image)
    print(f"[bench] uploaded in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)

    vocab = cfg["vocab_size"]
    kv_dim = cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"]
    prompt = synth.prompt_tokens(args.seed, n_prompt, vocab)

    def fill_kv(model, cfg, upto):
        """KV cache pre-filled with N(0,1) below position `upto` (the long-context configuration)."""
        kvd = cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"]
        for name in ("key_cache", "value_cache"):
            buf = model.buffer(name, cfg["n_layers"] * cfg["seq_len"] * kvd * 2)
            for l in range(cfg["n_layers"]):
                vals = synth.normal_f16(synth.stream_key(args.seed, name, l), upto * kvd)
                buf.write(vals, offset_bytes=l * cfg["seq_len"] * kvd * 2)

    if args.start_pos:
        fill_kv(model, cfg, args.start_pos)

    def run_decode(model, cfg, n_prompt, n_steps, start_pos=0):
        """Prompt as warm-up, then n_steps timed decode steps with the reference's synchronise-then-launch loop
        (llama2_q4.cu:713).  Every recorded launch sequence the run will replay is recorded before the clock starts."""
        toks = synth.prompt_tokens(args.seed, n_prompt, cfg["vocab_size"])
        model.reset(toks)
        if start_pos:
            model.set_pos(start_pos, toks[0])
            np.ctypeslib.as_array(model._tokens)[start_pos : start_pos + n_prompt] = toks
            for i, tk in enumerate(toks):  # the device mirror of the token list, which the fused schedule reads
                model.set_pos(start_pos + i, tk)
            model.set_pos(start_pos, toks[0])
        if use_graph and mode != A.SCHEDULE_PERSISTENT:
            model.capture(start_pos + n_prompt + n_steps, mode)
        for i in range(n_prompt):
            ctx.sync()
            model.forward(gen_token=(i >= n_prompt - 1), use_graph=use_graph, mode=mode)
        ctx.sync()
        ctx.record(ev0)
        w0 = time.perf_counter()
        for i in range(n_steps):
            ctx.sync()
            model.forward(gen_token=True, use_graph=use_graph, mode=mode)
        ctx.record(ev1)
        ctx.sync()
        wall = time.perf_counter() - w0
        first = start_pos + n_prompt
        return wall, ctx.elapsed_ms(ev0, ev1), [model.token(first + i) for i in range(min(8, n_steps))]

    ev0, ev1 = ctx.event(), ctx.event()
    if args.only_kernels:
        # calibration for HBM counters: a device-to-device copy of known size (reads 256 MiB, writes 256 MiB)
        from llama_cu_awq_amd._lib import check, lib

        nbytes = 256 << 20
        src, dst = ctx.alloc(nbytes), ctx.alloc(nbytes)
        check(lib.awq_memset_async(ctx.h, src.ptr, 1, nbytes))
        for _ in range(4):
            check(lib.awq_memcpy_d2d_async(ctx.h, dst.ptr, src.ptr, nbytes))
        ctx.sync()
        args.steps, n_prompt, total = 1, 1, 2
    wall, gpu_ms, gen = run_decode(model, cfg, n_prompt, args.steps, args.start_pos)
    tok_s = args.steps / wall

    wbytes = weight_bytes_per_token(cfg)
    avg_kv = 2 * cfg["n_layers"] * kv_dim * 2 * (args.start_pos + n_prompt + (args.steps + 1) / 2.0)
    decode_gbps = (wbytes + avg_kv) * tok_s / 1e9

    # ---- dominant kernel, as the timed (fused) schedule launches it: RMSNorm folded into the staging of x, gate and up
    # rows walked together, SiLU(gate) * up in the epilogue; one launch per layer over that layer's own weights (1.5 GB
    # of distinct matrices at 7B, so the 256 MB memory-side cache cannot serve them), timed with events on the
    # context's stream.  The plain form (separate RMSNorm, what the reference schedule launches) is timed beside it.
    dim, hid = cfg["dim"], cfg["hidden_dim"]
    layers = [model.layer(l) for l in range(cfg["n_layers"])]
    xres = model.buffer("x", dim * 2)
    xb = model.buffer("xb", dim * 2)
    hb = model.buffer("hb", hid * 2)
    reps = 8

    def timed(fn):
        fn()
        ctx.sync()
        ctx.record(ev0)
        for _ in range(reps):
            fn()
        ctx.record(ev1)
        ctx.sync()
        return ctx.elapsed_ms(ev0, ev1) * 1e3 / reps

    def ffn_fused_pass():
        for L in layers:
            A.rmsnorm_ffn_matvec_silu(ctx, hb, xres, L["rms_ffn_weight"], L["wq_gate"], L["wq_up"], dim, hid)

    def ffn_plain_pass():
        for L in layers:
            A.ffn_matvec_silu(ctx, hb, xb, L["wq_gate"], L["wq_up"], dim, hid)

    ffn_loop_us = timed(ffn_fused_pass) / len(layers)
    ffn_plain_us = timed(ffn_plain_pass) / len(layers)
    # ... and where it actually runs: every kernel of the fused schedule timed in place (eager passes at the middle
    # position of the timed run, each kernel launched with an event pair stamped with its own start and end)
    mid = args.start_pos + n_prompt + args.steps // 2
    model.set_pos(min(mid, cfg["seq_len"] - 1), prompt[0])
    in_place = model.time_launches(passes=4)
    ffn_us = in_place["gate_up"]["us"]
    # every launch kind of the fused schedule against the HBM roofline: algorithmic bytes per launch (packed weights,
    # activations in and out, norm weights; attention: the key and value rows up to the position) over its time in place
    kv_rows_bytes = 2 * (min(mid, cfg["seq_len"] - 1) + 1) * kv_dim * 2
    launch_bytes = {
        "embed": 2 * dim * 2,
        "qkv": qweight_bytes(dim, dim) + 2 * qweight_bytes(dim, kv_dim) + 2 * dim * 2 + (dim + 2 * kv_dim) * 2,
        "attention": kv_rows_bytes + 2 * dim * 2,
        "oproj": qweight_bytes(dim, dim) + 3 * dim * 2,
        "gate_up": 2 * qweight_bytes(dim, hid) + 2 * dim * 2 + hid * 2,
        "down": qweight_bytes(hid, dim) + hid * 2 + 2 * dim * 2,
        "classifier": vocab * dim * 2 + 2 * dim * 2 + vocab * 2,
    }
    launch_table = {
        k: {"us": v["us"], "bytes": launch_bytes[k], "gbps": round(launch_bytes[k] / v["us"] / 1e3, 1) if v["us"] else None,
            "frac_of_hbm_peak": round(launch_bytes[k] / v["us"] / 1e3 / (HBM_PEAK / 1e9), 4) if v["us"] else None}
        for k, v in in_place.items()
    }
    ffn_bytes = 2 * qweight_bytes(dim, hid) + dim * 2 + dim * 2 + hid * 2  # weights, x, norm weights, out
    ffn_gbps = ffn_bytes / ffn_us / 1e3
    ffn_waves = 4 if dim <= 8192 else 16

    # ---- configuration 0: the single dim x dim product (q/k/v/o shapes), rotating over every layer's four matrices
    def gemv_pass():
        for L in layers:
            for n in ("wq_q", "wq_k", "wq_v", "wq_o"):
                A.matmul_q(ctx, hb, xb, L[n], dim, dim)

    gemv_us = timed(gemv_pass) / (len(layers) * 4)
    gemv_bytes = qweight_bytes(dim, dim) + 4 * dim
    gemv_gbps = gemv_bytes / gemv_us / 1e3
    config0 = {
        "shape": [dim, dim],
        "bytes_per_product": gemv_bytes,
        "one_stream_back_to_back": {"us_per_product": round(gemv_us, 3), "gbps": round(gemv_gbps, 1), "frac": round(gemv_gbps * 1e9 / HBM_PEAK, 4)},
    }
    is_7b = (dim, hid) == (4096, 11008)
    prof = profiled_figures() if is_7b else None
    if is_7b:
        us = prof["gemv_4096_kernel_us"]
        config0["rocprof_kernel_duration"] = {"us_per_product": us, "gbps": round(gemv_bytes / us / 1e3, 1), "frac": round(gemv_bytes / us / 1e3 / 8000.0, 4), "source": TRACE_MD}
    # the same product through the C-ABI from one host thread per stream: 1, 2 and 4 plain streams over 64 distinct
    # matrices (558 MB), so that the fixed cost of a dependent launch overlaps the streaming of the other streams
    tool = os.path.join(ROOT, "llama_cu_awq_amd", "bin", "gemv_bench")
    if os.path.exists(tool) and not args.only_kernels:
        try:
            res = subprocess.run([tool, str(dim), str(dim), "64", "8"], capture_output=True, text=True, timeout=120)
            if res.returncode == 0:
                config0["independent_streams"] = json.loads(res.stdout.strip().splitlines()[-1])
            else:
                config0["independent_streams"] = {"error": res.stderr.strip()[-200:]}
        except Exception as e:  # the tool is a side measurement; the benchmark line does not depend on it
            config0["independent_streams"] = {"error": str(e)[-200:]}

    # ---- configuration 1 (the benchmark's own run), whatever --steps / --warmup were
    config1 = None
    if args.config == "7b" and not args.only_kernels:
        if (n_prompt, args.steps, args.start_pos) == (16, 256, 0):
            c_wall, c_gpu_ms, c_gen = wall, gpu_ms, gen
        else:
            c_wall, c_gpu_ms, c_gen = run_decode(model, cfg, 16, 256, 0)
        config1 = {
            "workload": "16-token prompt then 256 decode steps from position 0",
            "tok_per_s": round(256 / c_wall, 2),
            "ms_per_step": round(c_wall * 1e3 / 256, 4),
            "gpu_ms_per_step": round(c_gpu_ms / 256, 4),
            "frac_of_weight_roofline": round(256 / c_wall / (HBM_PEAK / weight_bytes_per_token(cfg)), 4),
            "first_tokens": c_gen,
        }

    # ---- prefill (7B shape, M prompt tokens in one batched pass on the matrix cores)
    prefill = None
    if args.prefill > 0 and not args.only_kernels and args.prefill <= cfg["seq_len"]:
        M = args.prefill
        ptoks = synth.prompt_tokens(args.seed + 1, M, vocab)
        times = []
        for rep in range(3):
            model.reset(ptoks)
            ctx.sync()
            ctx.record(ev0)
            model.prefill(M, gen_token=True)
            ctx.record(ev1)
            ctx.sync()
            times.append(ctx.elapsed_ms(ev0, ev1))
        pf_ms = min(times[1:])
        L, V = cfg["n_layers"], vocab
        proj_flops = 2.0 * M * L * (2 * dim * dim + 2 * dim * kv_dim + 3 * dim * hid) + 2.0 * dim * V
        attn_flops = 2.0 * 2 * L * cfg["n_heads"] * (dim // cfg["n_heads"]) * (M * (M + 1) / 2)
        prefill = {
            "tokens": M,
            "ms": round(pf_ms, 3),
            "tok_per_s": round(M / pf_ms * 1e3, 1),
            "tflops": round((proj_flops + attn_flops) / pf_ms / 1e9, 1),
            "mfma_frac_of_2.5PFLOPs": round((proj_flops + attn_flops) / (pf_ms * 1e-3) / 2.5e15, 4),
            "next_token": model.token(M),
        }

    # ---- CPU baseline: the oracle on the same model, a bounded number of tokens
    cpu = None
    if args.cpu_tokens > 0:
        from oracle import oracle

        o = oracle.Model(image)
        o.reset(prompt)
        o.forward(False)  # touch the weights once
        c0 = time.perf_counter()
        for _ in range(args.cpu_tokens):
            o.forward(False)
        cpu_s = time.perf_counter() - c0
        cpu = {
            "value": round(args.cpu_tokens / cpu_s, 4),
            "unit": "tok/s",
            "cores": oracle.num_threads(),
            "kind": "port",
            "sample": f"{args.cpu_tokens} tokens of the same {args.config} model (positions 1..{args.cpu_tokens}) through the scalar C++/OpenMP oracle, after 1 untimed token",
        }
        o.close()
        # configuration 0 on the host: the single 4096 x 4096 product through the oracle, 32 distinct matrices (279 MB)
        # x 4 rounds
        mats = [synth.make_qweight(synth.stream_key(args.seed, "config0", i), 4096, 4096) for i in range(32)]
        x0 = synth.normal_f16(synth.stream_key(args.seed, "config0", "x"), 4096)
        y0 = np.zeros(4096, dtype=np.float16)
        for w, z, sc in mats[:4]:
            oracle.matvec_int4(y0, x0, w, z, sc, 4096, 4096)
        c0 = time.perf_counter()
        for _ in range(4):
            for w, z, sc in mats:
                oracle.matvec_int4(y0, x0, w, z, sc, 4096, 4096)
        c_us = (time.perf_counter() - c0) * 1e6 / (4 * len(mats))
        cpu["config0"] = {"us_per_product": round(c_us, 1), "gbps": round((qweight_bytes(4096, 4096) + 4 * 4096) / c_us / 1e3, 2),
                          "sample": "128 products over 32 distinct 4096 x 4096 matrices"}
        del mats

    # ---- configurations 2 and 3 (13B shape from a cache pre-filled to 1536; 33B shape), compact, after everything that
    # needs the 7B model.  The 33B image takes half the benchmark's scale range: with the full range the residual stream
    # of a 60-layer model leaves fp16 range (in the oracle as on the GPU) and its tokens would mean nothing.
    extra = {}
    if args.config == "7b" and not args.only_kernels and not args.no_extra_configs:
        model.close()
        model = None
        del image
        for key, name, start, steps, scale in (("config2", "13b", 1536, 256, 1.0), ("config3", "33b", 0, 256, 0.5), ("shape_70b", "70b", 0, 128, 0.25)):
            xcfg = {"13b": synth.CONFIG_13B, "33b": synth.CONFIG_33B, "70b": synth.CONFIG_70B}[name]
            t0 = time.time()
            ximg = synth.make_model_image(xcfg, seed=args.seed, threads=min(16, os.cpu_count() or 8), scale_mult=scale)
            xm = A.Transformer(ctx, image=ximg)
            print(f"[bench] {name} image {ximg.nbytes / 1e9:.2f} GB generated and uploaded in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
            del ximg
            if start:
                fill_kv(xm, xcfg, start)
            x_wall, x_gpu_ms, x_gen = run_decode(xm, xcfg, 4, steps, start)
            xw = weight_bytes_per_token(xcfg)
            xkv = 2 * xcfg["n_layers"] * (xcfg["dim"] * xcfg["n_kv_heads"] // xcfg["n_heads"]) * 2 * (start + 4 + (steps + 1) / 2.0)
            x_tok_s = steps / x_wall
            extra[key] = {
                "workload": f"llama-{name}-shape: 4-token prompt then {steps} decode steps from position {start}" + (" (KV cache pre-filled with N(0,1))" if start else "") + (f", scale range x {scale}" if scale != 1.0 else ""),
                "tok_per_s": round(x_tok_s, 2),
                "ms_per_step": round(x_wall * 1e3 / steps, 4),
                "gpu_ms_per_step": round(x_gpu_ms / steps, 4),
                "weight_bytes_per_token": xw,
                "avg_kv_bytes_per_token": int(xkv),
                "frac_of_weight_roofline": round(x_tok_s / (HBM_PEAK / xw), 4),
                "frac_of_weight_plus_kv_roofline": round(x_tok_s / (HBM_PEAK / (xw + xkv)), 4),
                "first_tokens": x_gen,
            }
            xm.close()

    out = {
        "metric": "decode tok/s bs=1 @7B shape; int4 GEMV HBM GB/s vs ~8 TB/s peak",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int4 weights x fp16 activations, fp32 accumulate",
        "data": "synthetic (random int4-g128 weights, fp16 scales, random prompt ids; seed %d)" % args.seed,
        "config": {
            "workload": f"llama-2-{args.config}-shape bs=1 greedy decode: {n_prompt}-token prompt then {args.steps} decode steps from position {args.start_pos}",
            "schedule": args.schedule,
            "graph": use_graph,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "gemv_int4_kernel<W=%d waves, R=1 gate/up row pair per wave, D=2 passes in flight, KIND_FFN, NORM=true, ROPE=false> "
            "(RMSNorm while staging x, SiLU(gate)*up epilogue; the launch of the fused schedule), K=%d N=%d" % (ffn_waves, dim, hid),
            "achieved": round(ffn_gbps, 1),
            "peak": HBM_PEAK / 1e9,
            "unit": "GB/s",
            # achieved and frac follow from ONE measurement: this process's HIP events around the launches in place
            # (us_per_launch below); the committed rocprofv3 trace of the same command is carried beside it as frac_rocprof
            "frac": round(ffn_gbps * 1e9 / HBM_PEAK, 4),
            "frac_source": "HIP events in this run (us_per_launch)",
            "frac_rocprof": round(ffn_bytes / prof["ffn_kernel_us"] / 1e3 / (HBM_PEAK / 1e9), 4) if is_7b else None,
            # HBM bytes per launch cannot be counted from inside the run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this
            # kernel at the 7B shape, from the committed summary
            "traffic": prof["ffn_traffic_bytes"] if is_7b else None,
            "traffic_source": PMC_MD if is_7b else None,
            "bytes_per_launch": ffn_bytes,
            "us_per_launch": round(ffn_us, 3),
            "how_timed": "start/stop HIP events attached to each of the %d gate/up launches (kernel start to kernel end) in 4 eager passes of the fused schedule at position %d, on the context's stream" % (cfg["n_layers"], mid),
            "isolated_loop_us_per_launch": round(ffn_loop_us, 3),
            "rocprof_us_per_launch": prof["ffn_kernel_us"] if is_7b else None,
            "rocprof_source": TRACE_MD if is_7b else None,
            "plain_form_us_per_launch": round(ffn_plain_us, 3),
        },
        "cpu_baseline": cpu,
        "prefill": prefill,
        "decode": {
            "gpu_ms_per_step": round(gpu_ms / args.steps, 4),
            "weight_bytes_per_token": wbytes,
            "avg_kv_bytes_per_token": int(avg_kv),
            "hbm_gbps": round(decode_gbps, 1),
            "frac_of_weight_roofline": round(tok_s / (HBM_PEAK / wbytes), 4),
            "first_tokens": gen,
        },
        "launches_in_place_us": {k: v["us"] for k, v in in_place.items()},
        "launches_in_place": launch_table,
        "config0": config0,
        "config1": config1,
    }
    out.update(extra)
    print(json.dumps(out), flush=True)
    if model is not None:
        model.close()
    ctx.close()


if __name__ == "__main__":
    main()
