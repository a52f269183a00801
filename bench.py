#!/usr/bin/env python3
"""Batch-1 greedy decode throughput of the 40-layer 35B-A3B-shaped 4-bit model on one MI355X.

A step is one decode token at batch 1 (embed -> 40 layers -> final norm -> lm_head -> argmax).
The model is synthetic (seeded, generated in HBM); a 512-token uniform-random prompt is prefilled
before the timed region; tokens feed back on the device in chains, as the reference's default
decode does (chainedStepArgmax, K = 8).

Prints one JSON line: throughput, the roofline of the dominant kernel (the persistent step kernel
k_decode_flow: one launch runs a chain of `--chain` tokens, each fed back on the device; launches are
timed with HIP events on the engine's stream; roofline.avg_ms and bytes_per_launch are those of one
launch = `--chain` tokens), and the CPU baseline (the oracle, timed on this host's cores on a bounded
sample of the same workload).  After the timed decode region the same engine also times the batched
paths on the same weights and reports them as extra objects of the line: `lane_batch` (32 sequences at mixed contexts of 1K-16K tokens
stepped together), `verify` (4-row verify steps) and `prefill` (a 2048-token prompt in chunks of 1024
rows, exact rows and hybrid on the matrix cores), `context_sweep` (decode after prompts of 4096, 8192 and 32768
tokens, with the stage times of an attention layer at each context), `blocks` (the single blocks of the reference's
configurations 0-2, one launch each) and `stage_timeline`;
`--lanes 0 --verify-rows 0 --prefill-chunk 0 --context-sweep= --blocks 0 --stage-timeline 0` skips them.
`--microbench 1` prints the machine-limit micro-benchmarks instead (dependent exchanges between workgroups, the
4-bit GEMV streaming rate, matrix-instruction issue), the figures the design notes price the step against.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_FP16_PEAK_TFLOPS = 2500.0
PROMPT_LEN = 512
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "k_decode_flow_decode_b1_40layer_hbm_traffic_pmc.txt")


def traffic_bytes_per_token():
    """HBM bytes per decoded token as the counters saw them: the tracked rocprofv3 FETCH_SIZE / WRITE_SIZE summary of
    the k_decode_flow launches of this same command (copy-calibrated; the file names the commands).  None when the
    summary is missing, so the figure can never outlive the profile it came from."""
    import re
    try:
        with open(TRAFFIC_PROFILE) as f:
            m = re.search(r"traffic = (\d+) bytes per launch of (\d+) tokens", f.read())
        return int(m.group(1)) // int(m.group(2)) if m else None
    except OSError:
        return None


def step_bytes(cfg, ctx):
    """Algorithmic HBM bytes of one decode step: every needed weight/scale/bias byte once, plus
    recurrent state and conv history read+written, plus the KV prefix read."""
    q4 = lambda n, k: n * k // 2 + n * k // 16
    H, I, E = 2048, 512, cfg.n_experts
    moe = E * H * 2 + 8 * (2 * q4(I, H) + q4(H, I)) + (2 * q4(I, H) + q4(H, I)) + H * 2
    gdn = q4(12352, H) + q4(H, 4096) + 8192 * 4 * 4 + 2 * 3 * 8192 * 2 + 2 * 32 * 128 * 128 * 4
    attn = q4(9216, H) + q4(H, 4096) + 2 * 2 * ctx * 256 * 2
    n_attn = sum(0 if cfg.is_linear(i) else 1 for i in range(cfg.n_layers))
    n_gdn = cfg.n_layers - n_attn
    head = q4(cfg.vocab, H)
    norms = (2 * cfg.n_layers + 1) * H * 2
    return cfg.n_layers * moe + n_gdn * gdn + n_attn * attn + head + norms, head


def lane_step_bytes(cfg, ctxs):
    """Algorithmic HBM bytes of one step of len(ctxs) lanes (row b = lane b's next token): what the lanes share is
    counted once (dense projections, router, shared expert, norms, head), every routed expert the batch touches once
    (expected count per layer under the uniform routing of random weights: E (1 - (1 - 8/E)^B)), and per lane its
    recurrent state and conv history read + written and its KV prefix read."""
    q4 = lambda n, k: n * k // 2 + n * k // 16
    H, I, E, B = 2048, 512, cfg.n_experts, len(ctxs)
    expert = 2 * q4(I, H) + q4(H, I)
    touched = E * (1.0 - (1.0 - 8.0 / E) ** B)
    moe = E * H * 2 + expert + H * 2 + touched * expert
    gdn_w = q4(12352, H) + q4(H, 4096) + 8192 * 4 * 4
    gdn_lane = 2 * 3 * 8192 * 2 + 2 * 32 * 128 * 128 * 4
    attn_w = q4(9216, H) + q4(H, 4096)
    kv = sum(2 * 2 * c * 256 * 2 for c in ctxs)
    n_attn = sum(0 if cfg.is_linear(i) else 1 for i in range(cfg.n_layers))
    n_gdn = cfg.n_layers - n_attn
    shared = cfg.n_layers * moe + n_gdn * gdn_w + n_attn * attn_w + q4(cfg.vocab, H) + (2 * cfg.n_layers + 1) * H * 2
    return int(shared + n_gdn * B * gdn_lane + n_attn * kv)


def prefill_flops(cfg, n):
    """Multiply-adds x 2 of a prompt of n tokens: every projection row a token uses (router, shared expert and 8 routed
    experts, the mixers' projections), causal attention scores and weighted sums (16 heads x 256 dims, key j <= row),
    the gated delta rule per row (state [32 heads][128][128]: decay, k S, rank-1 update, S q) and the head on the last row."""
    H, I, E = 2048, 512, cfg.n_experts
    moe = (E + 1) * H + 9 * 3 * I * H
    gdn = 12352 * H + H * 4096 + 4 * 32 * 128 * 128
    attn = 9216 * H + H * 4096
    n_attn = sum(0 if cfg.is_linear(i) else 1 for i in range(cfg.n_layers))
    n_gdn = cfg.n_layers - n_attn
    per_token = cfg.n_layers * moe + n_gdn * gdn + n_attn * attn
    scores = n_attn * 16 * 256 * 2 * (n * (n + 1) // 2)
    return 2 * (n * per_token + scores + cfg.vocab * H)


def block_benchmarks(eng, cfg, np, torch):
    """Benchmark configurations 0-2: one MoE block, one GDN layer, one attention layer over 4K / 8K / 32K keys, batch 1,
    through the block entry points (the kernel-per-stage sequence: 3 kernels per MoE block, 3 per GDN layer, 5 per
    attention layer), timed with HIP events around each call's kernels.  "cold": successive calls go to different
    layers of the model (40 / 30 / 10 distinct weight sets, 0.7 / 0.7 / 0.15-0.8 GB, more than the 256 MB last-level
    cache), so weights come from HBM; "hot": the same layer every time.  The method follows the reference's kernel
    micro-benchmarks (PrefixCachePoC.swift:111-162).  Inside the single-launch decode step the same blocks cost what
    the stage timeline reports."""
    H = 2048
    q4 = lambda n, k: n * k // 2 + n * k // 16
    moe_b = cfg.n_experts * H * 2 + 9 * (2 * q4(512, H) + q4(H, 512)) + H * 2
    gdn_b = q4(12352, H) + q4(H, 4096) + 8192 * 4 * 4 + 2 * 3 * 8192 * 2 + 2 * 32 * 128 * 128 * 4
    att_w = q4(9216, H) + q4(H, 4096)
    lin = [i for i in range(cfg.n_layers) if cfg.is_linear(i)]
    att = [i for i in range(cfg.n_layers) if not cfg.is_linear(i)]
    rng = np.random.default_rng(1000)
    xs = [rng.normal(0, 1, (1, H)).astype(np.float16) for _ in range(8)]
    REPS, DROP = 30, 5                                    # the reference's 30 repetitions with the first 5 dropped

    def timed(e, fn, layers, nbytes):
        out = {}
        for name, seq in (("cold", [layers[i % len(layers)] for i in range(REPS)]), ("hot", [layers[0]] * REPS)):
            ms = []
            for i, li in enumerate(seq):
                y = fn(e, li, xs[i % len(xs)])
                assert y is not None, e.gpu_fault
                ms.append(e.last_gpu_ms)
            us = float(np.median(ms[DROP:])) * 1e3
            out[name] = {"us": us, "GBs": nbytes / us / 1e3, "frac_of_peak": nbytes / us / 1e3 / HBM_PEAK_GBS}
        out["bytes"] = nbytes
        out["roofline_us"] = nbytes / HBM_PEAK_GBS / 1e3
        return out

    rep = {"method": f"block entry points (one launch per block: the step kernel's stages for that block), batch 1, HIP events, median of {REPS - DROP} calls"}
    lane = eng.new_lane(max_m=1, max_seq_len=64)
    rep["moe_block"] = timed(lane, lambda e, li, x: e.moe_block_rows(li, x), list(range(cfg.n_layers)), moe_b)
    if lin:
        rep["gdn_layer"] = timed(lane, lambda e, li, x: e.gdn_layer_rows(li, x), lin, gdn_b)
    lane.close()
    if att:
        rep["attention_layer"] = {}
        for S in (4096, 8192, 32768):
            lane = eng.new_lane(max_m=1, max_seq_len=S + 2 * REPS + 8)
            kv = np.random.default_rng(1310).normal(0, 1, (2, S, 256)).astype(np.float16)
            for li in att:
                assert lane.load_layer_cache(li, kv, kv)
            rep["attention_layer"][str(S)] = timed(lane, lambda e, li, x: e.attn_layer_rows(li, x), att, att_w + 2048 * S)
            lane.close()
    return rep


def microbench(L):
    """The three machine limits the design notes quote, measured by the library's own micro-benchmark kernels
    (qwisp_amd/csrc/sl_ubench.hip); every figure is the best of three runs."""
    import ctypes as C
    f, g = C.c_float(), C.c_float()

    def best(call, pick=min):
        vals = []
        for _ in range(3):
            r = call()
            assert r == 0, f"micro-benchmark failed with status {r}"
            vals.append((f.value, g.value))
        return pick(vals)
    ex = {}
    for mode, name in ((0, "allgather_2048_words_barrier_per_round"), (1, "allgather_2048_words_one_barrier"),
                       (2, "allgather_2048_words_every_thread_its_pair"), (3, "256_words_among_32_workgroups_of_one_xcd"),
                       (4, "256_words_among_32_workgroups_across_xcds")):
        ex[name] = round(best(lambda: L.dll.sl_ubench_exchange(mode, 2008, C.byref(f)))[0], 3)
    gm = {}
    for mode, name in ((0, "loads_only"), (1, "with_dot"), (2, "with_dot_and_row_reduction")):
        for grid in (256, 512):
            gm[f"{name}_grid{grid}"] = round(best(lambda: L.dll.sl_ubench_gemv_stream(mode, grid, C.byref(f)), max)[0], 3)
    mf = {}
    for wps in (1, 2):
        for lds in (0, 1):
            for valu in (0, 1, 2, 4, 8):
                if lds and valu > 2:
                    continue
                t = best(lambda: L.dll.sl_ubench_mfma_issue(valu, lds, wps, C.byref(f), C.byref(g)), max)
                mf[f"valu_steps{valu}_lds{lds}_waves{wps}"] = {"tflops": round(t[0], 1), "ns_per_mfma_per_simd": round(t[1], 2)}
    return {"microbench": {"exchange_us_per_dependent_round": ex, "gemv_stream_tb_per_s": gm, "mfma_issue": mf,
                           "notes": "exchange: 256 workgroups x 1024 threads, 2000 dependent rounds; gemv: 2.4 GB of K = 2048 "
                                    "4-bit rows; mfma: v_mfma_f32_32x32x16_f16, a valu step = 3 vector instructions on a half pair"}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--chain", type=int, default=8, help="tokens per on-device chain")
    ap.add_argument("--layers", type=int, default=40, help="for quick functional runs only")
    ap.add_argument("--cpu-tokens", type=int, default=96,
                    help="decode tokens the CPU oracle generates after the same 512-token prompt: timed as the CPU baseline and "
                         "compared with the GPU stream token by token (0 = skip)")
    ap.add_argument("--blocks", type=int, default=1,
                    help="also time the single blocks (MoE block, GDN layer, attention layer at 4K / 8K / 32K keys) through their "
                         "block entry points, weights cold (rotating over the model's layers) and hot (0 = skip)")
    ap.add_argument("--stage-timeline", type=int, default=1,
                    help="also run one chain with the stage clock on and report where a step's time goes (0 = skip)")
    ap.add_argument("--lanes", type=int, default=32, metavar="B",
                    help="also time B lanes stepped as one batch of rows on the same weights (extra object in the JSON line; 0 = skip)")
    ap.add_argument("--lane-contexts", choices=("mixed", "short"), default="mixed",
                    help="contexts of the --lanes sequences: mixed = 1K to 16K tokens spread evenly over the lanes (prefilled "
                         "on the matrix cores first), short = 8 to 56 tokens")
    ap.add_argument("--prefill-chunk", type=int, default=2048, metavar="M",
                    help="also time a prefill in chunks of M rows, exact rows and hybrid (matrix cores), on lanes "
                         "of the same weights (extra object in the JSON line; 0 = skip); 2048 is the chunk of the "
                         "reference's batched configuration")
    ap.add_argument("--prefill-also", default="1024", metavar="M,M",
                    help="further chunk sizes timed in hybrid mode only (the reference's own default chunk is 1024)")
    ap.add_argument("--prefill-tokens", type=int, default=2048, metavar="N",
                    help="prompt length of the --prefill-chunk measurement (the reference's batched configuration uses 2048)")
    ap.add_argument("--verify-rows", type=int, default=4, metavar="R",
                    help="also time verify steps of R rows ([token] + R-1 drafts through stepArgmax) at the decode context "
                         "(extra object in the JSON line; 0 = skip)")
    ap.add_argument("--context-sweep", type=str, default="4096,8192,32768", metavar="S1,S2",
                    help="also time batch-1 decode after prompts of these lengths (hybrid prefill in chunks of 1024; extra "
                         "object in the JSON line; empty = skip)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="only run a plain device copy of this many MiB (reference for rocprofv3 FETCH_SIZE/WRITE_SIZE) and exit")
    ap.add_argument("--microbench", type=int, default=0,
                    help="only run the library's micro-benchmarks of the machine limits that bound the kernels (dependent "
                         "hand-over between 256 resident workgroups, 4-bit row streaming through the dot, issue cost of vector "
                         "instructions beside matrix instructions), print their figures as one JSON line and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).")

    import numpy as np
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X; no GPU is visible.")
    torch.cuda.set_device(0)
    if args.copy_calibration:
        n = args.copy_calibration << 20
        src = torch.full((n,), 3, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes": n, "copies": 3}))
        return
    from qwisp_amd import lib, synth
    from qwisp_amd.engine import SeedlessFusedForward
    if args.microbench:
        print(json.dumps(microbench(lib.get())))
        return

    cfg = synth.ModelConfig(n_layers=args.layers)
    t0 = time.time()
    dev = synth.generate_device(cfg, lib.get())
    t_gen = time.time() - t0
    max_seq = PROMPT_LEN + args.warmup + args.steps + 16 + 24 * max(args.verify_rows, 0)
    eng = SeedlessFusedForward(cfg, dev, max_m=max(64, args.verify_rows), max_seq_len=max_seq)
    host = None
    if args.cpu_tokens > 0:
        host = {k: (v.cpu().numpy().view(np.uint32) if v.dtype == torch.int32 else v.cpu().numpy()) for k, v in dev.items()}
    del dev
    torch.cuda.empty_cache()

    prompt = np.random.default_rng(3000).integers(0, cfg.vocab, PROMPT_LEN).astype(np.int32)
    t0 = time.time()
    first = eng.greedy_generate(prompt, 1, chain_k=args.chain)
    assert first is not None, eng.gpu_fault
    t_prefill = time.time() - t0
    cur = int(first[0])
    stream = [cur]

    def run(n):
        nonlocal cur
        done = 0
        while done < n:
            k = min(args.chain, n - done)
            out = eng.chained_step_argmax(cur, k)
            assert out is not None, eng.gpu_fault
            stream.extend(out.tolist())
            cur = int(out[-1])
            done += k

    run(args.warmup)
    eng.profile_head(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(args.steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    head_ms, head_n = eng.profile_head_read()
    eng.profile_head(False)

    ctx_mid = PROMPT_LEN + args.warmup + args.steps // 2
    total_b, head_b = step_bytes(cfg, ctx_mid)
    ms_step = elapsed * 1e3 / args.steps
    tok_s = args.steps / elapsed
    tok_per_launch = args.steps / max(head_n, 1)          # a launch of k_decode_flow runs a whole chain
    head_avg_ms = head_ms / max(head_n, 1)
    launch_b = int(total_b * tok_per_launch)
    head_gbs = launch_b / (head_avg_ms * 1e-3) / 1e9 if head_n else 0.0
    step_gbs = total_b / (ms_step * 1e-3) / 1e9

    lanes_report = None
    if args.lanes > 1:
        B = args.lanes
        # the batched configuration of the reference: concurrent sequences at mixed contexts of 1K to 16K tokens
        # (spread evenly over the lanes; --lane-contexts short keeps them at 8-56 tokens for quick runs)
        mixed = args.lane_contexts == "mixed"
        ctxs = [1024 + (15 * 1024 * i) // max(B - 1, 1) for i in range(B)] if mixed else [8 + (i * 5) % 40 for i in range(B)]
        lane_m = max(B, 256) if mixed else B
        lanes = [eng.new_lane(max_m=lane_m, max_seq_len=(max(ctxs) + 64 if mixed else 256)) for _ in range(B)]
        rng = np.random.default_rng(4000)
        toks = []
        t_fill = time.time()
        for i, lane in enumerate(lanes):
            pr = rng.integers(0, cfg.vocab, ctxs[i]).astype(np.int32)
            if mixed:                                    # prompts through the hybrid prefill in chunks of lane_m rows
                lane.set_hybrid(True)
                o = lane.greedy_generate(pr, 1, chain_k=1)
                assert o is not None, lane.gpu_fault
                lane.set_hybrid(False)
                toks.append(int(o[0]))
            else:
                o = None
                for j in range(0, len(pr), B):
                    o = lane.step_argmax(pr[j:j + B])
                    assert o is not None, lane.gpu_fault
                toks.append(int(o[-1]))
        t_fill = time.time() - t_fill
        step = type(eng).lane_step_argmax
        for _ in range(2):
            toks = step(lanes, toks).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        n_lane_steps = 8
        for _ in range(n_lane_steps):
            toks = step(lanes, toks).tolist()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        lanes_report = {"lanes": B, "ms_per_step": dt * 1e3 / n_lane_steps, "tok_s_aggregate": B * n_lane_steps / dt,
                        "contexts": f"{min(ctxs)}-{max(ctxs)} tokens, mean {sum(ctxs) // B}", "fill_s": t_fill, "path": "rows of the kernel-per-stage path; from 32 lanes on two launch sequences side by side, 16 lanes each"}
        lane_b = lane_step_bytes(cfg, ctxs)             # the step's own byte roofline (shared weights once, touched experts once)
        lanes_report["bytes_per_step"] = lane_b
        lanes_report["frac_of_peak"] = lane_b / (dt / n_lane_steps) / 1e9 / HBM_PEAK_GBS
        if B >= 16:                                     # the same batch with projections, experts and lm_head on the matrix cores
            lanes[0].set_hybrid(True)
            for _ in range(2):
                toks = step(lanes, toks).tolist()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n_lane_steps):
                toks = step(lanes, toks).tolist()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            lanes_report["hybrid_matrix_cores"] = {"ms_per_step": dt * 1e3 / n_lane_steps, "tok_s_aggregate": B * n_lane_steps / dt,
                                                   "frac_of_peak": lane_b / (dt / n_lane_steps) / 1e9 / HBM_PEAK_GBS}
            lanes[0].set_hybrid(False)
        for lane in lanes:
            lane.close()

    verify_report = None
    if args.verify_rows > 1:
        R = args.verify_rows
        rng = np.random.default_rng(5000)
        reps = 16
        rows = [np.concatenate([[cur], rng.integers(0, cfg.vocab, R - 1)]).astype(np.int32) for _ in range(reps + 4)]
        for r in rows[:4]:
            assert eng.step_argmax(r) is not None, eng.gpu_fault
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for r in rows[4:]:
            o = eng.step_argmax(r)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert o is not None, eng.gpu_fault
        verify_report = {"rows": R, "ms_per_step": dt * 1e3 / reps, "ms_per_row": dt * 1e3 / reps / R,
                         "context": PROMPT_LEN + args.warmup + args.steps + 4 * R,
                         "path": "rows of the kernel-per-stage path; every row accepted (the context advances R per step)"}

    prefill_report = None
    if args.prefill_chunk > 0:
        PF = args.prefill_tokens
        pf_prompt = np.random.default_rng(3000).integers(0, cfg.vocab, PF).astype(np.int32)
        prefill_report = {"prompt": PF, "chunk_rows": args.prefill_chunk}
        for name, hyb in (("exact_rows", False), ("hybrid_matrix_cores", True)):
            times = []
            for rep in range(2):                           # the first pass warms code and caches
                lane = eng.new_lane(max_m=args.prefill_chunk, max_seq_len=PF + 8)
                lane.set_hybrid(hyb)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                o = lane.greedy_generate(pf_prompt, 1, chain_k=1)
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                assert o is not None, lane.gpu_fault
                lane.close()
            prefill_report[name] = {"ms": times[-1] * 1e3, "tok_s": PF / times[-1]}
            if hyb:                                        # against the dense fp16 rate of the matrix cores
                prefill_report[name]["tflops"] = prefill_flops(cfg, PF) / times[-1] / 1e12
                prefill_report[name]["frac_of_fp16_peak"] = prefill_report[name]["tflops"] / MFMA_FP16_PEAK_TFLOPS
        for m in [int(x) for x in args.prefill_also.split(",") if x]:
            times = []
            for rep in range(2):
                lane = eng.new_lane(max_m=m, max_seq_len=PF + 8)
                lane.set_hybrid(True)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                o = lane.greedy_generate(pf_prompt, 1, chain_k=1)
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                assert o is not None, lane.gpu_fault
                lane.close()
            prefill_report.setdefault("hybrid_other_chunks", {})[str(m)] = {"ms": times[-1] * 1e3, "tok_s": PF / times[-1]}

    sweep_report = None
    if args.context_sweep:
        sweep_report = []
        for S in [int(x) for x in args.context_sweep.split(",") if x]:
            lane = eng.new_lane(max_m=1024, max_seq_len=S + 128)
            lane.set_hybrid(True)
            pr = np.random.default_rng(6000 + S).integers(0, cfg.vocab, S).astype(np.int32)
            o = lane.greedy_generate(pr, 1, chain_k=args.chain)
            assert o is not None, lane.gpu_fault
            t = int(o[0])
            o = lane.chained_step_argmax(t, args.chain)          # warm-up chain
            t = int(o[-1])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            n_tok = 8 * args.chain
            for _ in range(8):
                o = lane.chained_step_argmax(t, args.chain)
                t = int(o[-1])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            assert o is not None, lane.gpu_fault
            b_tok, _ = step_bytes(cfg, S + args.chain + n_tok // 2)
            entry = {"context": S, "ms_per_token": dt * 1e3 / n_tok, "tok_s": n_tok / dt, "bytes_per_token": b_tok,
                     "frac_of_peak": b_tok / (dt / n_tok) / 1e9 / HBM_PEAK_GBS}
            if args.stage_timeline:
                # where an attention layer's time goes at this context: one more chain on the stamping variant of the kernel
                from qwisp_amd import stage_timeline
                lib.get().dll.sl_debug_stage_clock(lane.h, 1, None, 0)
                o = lane.chained_step_argmax(t, args.chain)
                o = lane.chained_step_argmax(int(o[-1]), args.chain)
                assert o is not None, lane.gpu_fault
                att = stage_timeline.collect(lane).summary().get("attention_layer")
                lib.get().dll.sl_debug_stage_clock(lane.h, 0, None, 0)
                if att:
                    entry["attention_layer_us"] = {"layer": att["us"], "mixer": att["mixer_us"], "moe_block": att["moe_block_us"],
                                                   "in-proj": att["in-proj"]["total_us"], "tile units": att["core"]["total_us"],
                                                   "merge + out-proj": att["out-proj"]["total_us"]}
            sweep_report.append(entry)
            lane.close()

    blocks_report = None
    if args.blocks:
        blocks_report = block_benchmarks(eng, cfg, np, torch)

    timeline_report = None
    if args.stage_timeline:
        from qwisp_amd import stage_timeline
        lib.get().dll.sl_debug_stage_clock(eng.h, 1, None, 0)
        out = eng.chained_step_argmax(cur, args.chain)            # warms the stamping variant's code
        out = eng.chained_step_argmax(int(out[-1]), args.chain)
        assert out is not None, eng.gpu_fault
        tl = stage_timeline.collect(eng)
        lib.get().dll.sl_debug_stage_clock(eng.h, 0, None, 0)
        print(tl.table(), file=sys.stderr)
        timeline_report = tl.summary()

    cpu = None
    stream_check = None
    if host is not None:
        # the oracle on the same workload: the same 512-token prompt (untimed), then `--cpu-tokens` greedy tokens, timed
        # as the CPU baseline and compared with the stream the GPU produced above, token by token
        from oracle import orc
        ora = orc.Oracle(cfg, host, max_m=64, max_seq_len=PROMPT_LEN + args.cpu_tokens + 8)
        t0 = time.perf_counter()
        nr = None
        for i in range(0, PROMPT_LEN, 64):
            nr = ora.forward_tokens(prompt[i:i + 64])
        cpu_prefill = time.perf_counter() - t0
        ocur = int(ora.head_argmax(nr[-1:])[0])
        ostream = [ocur]
        t0 = time.perf_counter()
        for _ in range(args.cpu_tokens):
            ocur = int(ora.step_argmax([ocur])[0])
            ostream.append(ocur)
        cpu_elapsed = time.perf_counter() - t0
        n_cmp = min(len(ostream), len(stream))
        bad = [i for i in range(n_cmp) if ostream[i] != stream[i]]
        assert not bad, f"GPU stream leaves the oracle's at token {bad[0]}: {stream[bad[0]]} vs {ostream[bad[0]]}"
        stream_check = {"tokens_compared": n_cmp, "equal": True}
        cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
        cpu = {"value": args.cpu_tokens / cpu_elapsed, "unit": "tok/s", "cores": min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))),
               "kind": "port",
               "sample": f"{args.cpu_tokens} decode tokens after the same {PROMPT_LEN}-token prompt, the same {cfg.n_layers}-layer model and "
                         f"weights (oracle, g++ -O3 OpenMP; decode {cpu_elapsed:.1f} s, prompt {cpu_prefill:.1f} s untimed)"}

    print(json.dumps({
        "metric": "batch-1 decode tok/s (35B-A3B shape, 4-bit) + achieved HBM GB/s as % of peak",
        "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u4 weights, f16 activations, f32 accumulate", "data": "synthetic",
        "config": {"workload": f"{cfg.n_layers}-layer 35B-A3B hybrid (3 GDN : 1 attention, 256-expert top-8 MoE + shared), "
                               f"vocab {cfg.vocab}, 4-bit g64; greedy decode after a {PROMPT_LEN}-token prompt, batch 1",
                   "chain_k": args.chain, "context": [PROMPT_LEN + args.warmup, PROMPT_LEN + args.warmup + args.steps]},
        "roofline": {"bound": "hbm", "kernel": "k_decode_flow (persistent batch-1 step: 40 layers + lm_head + argmax)",
                     "achieved": head_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head_gbs / HBM_PEAK_GBS,
                     "traffic": (int(traffic_bytes_per_token() * tok_per_launch) if traffic_bytes_per_token() else None),
                     "launches": head_n, "avg_ms": head_avg_ms,
                     "bytes_per_launch": launch_b, "tokens_per_launch": tok_per_launch, "bytes_per_token": total_b,
                     "avg_ms_per_token": head_avg_ms / tok_per_launch},
        "step_hbm": {"bytes_per_token": total_b, "achieved_GBs": step_gbs, "frac_of_peak": step_gbs / HBM_PEAK_GBS},
        "cpu_baseline": cpu,
        "stream_vs_oracle": stream_check,
        "blocks": blocks_report,
        "stage_timeline": timeline_report,
        "lane_batch": lanes_report,
        "prefill": prefill_report,
        "verify": verify_report,
        "context_sweep": sweep_report,
        "setup_s": {"generate": t_gen, "prefill_512": t_prefill},
        "tokens_head": stream[:8],
    }))


if __name__ == "__main__":
    main()
