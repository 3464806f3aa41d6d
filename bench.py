#!/usr/bin/env python3
"""Benchmark of the MoE expert forward path on one MI355X.

A step is one pass of the whole path (router logits in, combined hidden states
out: routing, permute, activation quantisation, both grouped fp8 GEMMs, shared
expert, combine) over one batch of synthetic input that is already resident in
HBM.  The headline workload is the DeepSeek-V3-style prefill layer; the same
run also measures the decode shape (HBM-bound) and reports it under "decode".

Prints ONE JSON line.  FLOPs counted: 6*R*D*I (routed) + 6*M*D*SI (shared); the
router matmul and tile padding are not counted.  Decode bytes counted: fp8
weights (and their scales) of the experts actually touched plus the shared
expert; activations are not counted.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0     # MI355X dense fp8 MFMA (published)
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E (published)


def measured_traffic(workload, kernel="gateup_routed"):
    """HBM-side bytes per launch of one of the workload's routed grouped GEMM launches (kernel = gateup_routed or
    down_routed), as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE: read at run time from the committed
    summary under profiles/, which carries the commands and the calibration next to a line
        traffic: workload=<name> kernel=<kernel> fetch_bytes=<n> write_bytes=<n>
    Returns (bytes or None, the file it came from or None)."""
    import glob
    import re
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*hbm_traffic*.txt"))):
        for ln in open(path):
            m = re.match(r"\s*traffic:\s+workload=(\S+)\s+kernel=(\S+)\s+fetch_bytes=(\d+)\s+write_bytes=(\d+)", ln)
            if m and m.group(1) == workload and m.group(2) == kernel:
                return float(m.group(3)) + float(m.group(4)), os.path.relpath(path, ROOT)
    return None, None


GATEUP_NAME = "grouped_gemm_kernel<0>, routed launch (gate/up + SwiGLU + h quantisation)"
DOWN_NAME = "grouped_gemm_kernel<1>, routed launch (down, bf16 rows)"


def kernel_roofline(bound, kern, workload, kernel_key, name):
    """The roofline object of one launch timed alone (HIP events on the stream it is launched on): achieved =
    algorithmic FLOPs (or algorithmic weight bytes) per launch / average launch duration."""
    traffic, src = measured_traffic(workload, kernel_key)
    if bound == "mfma":
        ach, peak, unit = kern["tflops"], PEAK_FP8_TFLOPS, "TFLOP/s"
    else:
        ach, peak, unit = kern["gbs"], PEAK_HBM_GBS, "GB/s"
    return {"bound": bound, "achieved": ach, "peak": peak, "unit": unit, "frac": ach / peak, "traffic": traffic,
            "traffic_source": src, "kernel": name, "avg_launch_ms": kern["avg_launch_ms"],
            "flops_per_launch": kern["flops_per_launch"], "algorithmic_bytes_per_launch": kern["bytes_per_launch"]}


WORKLOADS = {
    # benchmark configs 3 and 4 (BASELINE.json): DeepSeek-V3-style layer
    "deepseek_v3_prefill": dict(M=8192, D=7168, E=256, k=8, I=2048, SI=2048, routing="sigmoid_grouped",
                                n_group=8, topk_group=4),
    "deepseek_v3_decode": dict(M=64, D=7168, E=256, k=8, I=2048, SI=2048, routing="sigmoid_grouped",
                               n_group=8, topk_group=4),
    # benchmark config 2 (BASELINE.json): Qwen3-MoE-style layer
    "qwen3_moe_prefill": dict(M=4096, D=2048, E=128, k=8, I=768, SI=0, routing="softmax", n_group=1, topk_group=1),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_weights(jg, torch, E, N, K, gen, std=0.02, chunk=16):
    """(E, N, K) N(0, std) weights, block-quantised on the GPU chunk by chunk (never on the host)."""
    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    sw = torch.empty((E, N // 128, K // 128), dtype=torch.float32, device="cuda")
    for e0 in range(0, E, chunk):
        n = min(chunk, E - e0)
        w = (torch.randn((n, N, K), dtype=torch.float32, device="cuda", generator=gen) * std).to(torch.bfloat16)
        d = jg.quantize_weight_block(w)
        wq[e0:e0 + n] = d["w"]
        sw[e0:e0 + n] = d["scale_inv"]
        del w, d
    return {"w": wq, "scale_inv": sw}


def make_layer(jg, torch, cfg, seed=0, bias_std=0.1):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    D, E, I, SI = cfg["D"], cfg["E"], cfg["I"], cfg["SI"]
    experts = dict(gate_proj=make_weights(jg, torch, E, I, D, gen), up_proj=make_weights(jg, torch, E, I, D, gen),
                   down_proj=make_weights(jg, torch, E, D, I, gen))
    shared = None
    if SI:
        shared = dict(gate_proj=make_weights(jg, torch, 1, SI, D, gen), up_proj=make_weights(jg, torch, 1, SI, D, gen),
                      down_proj=make_weights(jg, torch, 1, D, SI, gen))
    bias = None
    if cfg["routing"] == "sigmoid_grouped":
        bias = torch.randn((E,), dtype=torch.float32, device="cuda", generator=gen) * bias_std
    return experts, shared, bias, gen


def make_inputs(torch, cfg, gen):
    x = torch.randn((cfg["M"], cfg["D"]), dtype=torch.float32, device="cuda", generator=gen).to(torch.bfloat16)
    logits = torch.randn((cfg["M"], cfg["E"]), dtype=torch.float32, device="cuda", generator=gen)
    return x, logits


def timed(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall


def run_workload(jg, torch, name, cfg, layer, steps, warmup, graph=True):
    experts, shared, bias, gen = layer
    x, logits = make_inputs(torch, cfg, gen)
    kw = dict(top_k=cfg["k"], experts=experts, shared=shared, routing=cfg["routing"], bias=bias,
              n_group=cfg["n_group"], topk_group=cfg["topk_group"])
    out, dbg = jg.moe_experts(x, logits, return_debug=True, **kw)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all(), "non-finite output"
    gs = dbg["group_sizes"].cpu()
    touched = int((gs > 0).sum())
    assert int(gs.sum()) == cfg["M"] * cfg["k"]
    log(f"{name}: rows per expert, ascending: {sorted(int(v) for v in gs)}")
    ev_ms, wall_ms = timed(torch, lambda: jg.moe_experts(x, logits, **kw), steps, warmup)
    M, D, E, k, I, SI = (cfg[n] for n in ("M", "D", "E", "k", "I", "SI"))
    R = M * k
    flops = 6.0 * R * D * I + 6.0 * M * D * SI
    per_expert_bytes = 3 * D * I + 3 * (D // 128) * (I // 128) * 4
    shared_bytes = (3 * D * SI + 3 * (D // 128) * (SI // 128) * 4) if SI else 0
    weight_bytes = touched * per_expert_bytes + shared_bytes
    res = dict(workload=name, ms_per_step=ev_ms, wall_ms_per_step=wall_ms, flops=flops, tflops=flops / ev_ms / 1e9,
               touched_experts=touched, weight_bytes=weight_bytes, gbs=weight_bytes / ev_ms / 1e6)

    # the same step captured once in a HIP graph and replayed (no per-launch host work): matters for
    # decode-sized batches, where a dozen dependent launches share a millisecond
    res["graph_ms_per_step"] = None
    try:
        if not graph:
            raise RuntimeError("not asked for")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                jg.moe_experts(x, logits, **kw)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out_g = jg.moe_experts(x, logits, **kw)
        graph.replay()
        torch.cuda.synchronize()
        if not torch.equal(out_g, out):
            raise RuntimeError("graph replay differs from the eager result")
        # replayed and eager steps in turn (two rounds each): a captured step and an eager one are then compared under
        # the same clocks and temperatures (measured one after the other, whichever comes second reads 2-3 % slower)
        g_runs, e_runs = [], []
        for _ in range(2):
            g_runs.append(timed(torch, graph.replay, steps, 2)[0])
            e_runs.append(timed(torch, lambda: jg.moe_experts(x, logits, **kw), steps, 2)[0])
        if not torch.equal(out_g, out):
            raise RuntimeError("graph replay differs from the eager result after the timed replays")
        g_ms = sum(g_runs) / len(g_runs)
        res["graph_ms_per_step"] = g_ms
        res["eager_ms_per_step_beside_graph"] = sum(e_runs) / len(e_runs)
        res["graph_gbs"] = weight_bytes / g_ms / 1e6
        res["graph_tflops"] = flops / g_ms / 1e9
        del graph, out_g
    except Exception as exc:  # noqa: BLE001 - the eager figure stands on its own
        log(f"graph replay measurement skipped: {exc!r}")

    # the dominant kernel alone: the routed launch of the gate/up grouped GEMM, HIP events on the
    # stream it is launched on (torch's current stream is the stream handed to the C ABI)
    sg = jg.permute(dbg["indices"], E)
    xq, sx = jg.quant_act(x)
    # as moe_forward launches it: large batches read their activation scales block-major, in sorted row order
    blocked = R > 2048
    sxk = jg.gather_scales(sx, sg["sorted_token_ids"]) if blocked else sx

    def gateup():
        jg.gemm_gateup_swiglu(xq, sxk, experts["gate_proj"], experts["up_proj"], sg["group_offsets"],
                              row_ids=sg["sorted_token_ids"], block_major=blocked)

    k_ms, _ = timed(torch, gateup, steps, max(2, warmup // 2))
    k_flops = 4.0 * R * D * I
    k_bytes = touched * per_expert_bytes * 2 / 3
    res["gateup_kernel"] = dict(avg_launch_ms=k_ms, flops_per_launch=k_flops, tflops=k_flops / k_ms / 1e9,
                                bytes_per_launch=k_bytes, gbs=k_bytes / k_ms / 1e6)
    # the routed down launch, timed alone the same way, on the h that the gate/up launch wrote
    hq, sh = jg.gemm_gateup_swiglu(xq, sxk, experts["gate_proj"], experts["up_proj"], sg["group_offsets"],
                                   row_ids=sg["sorted_token_ids"], block_major=blocked)
    d_ms, _ = timed(torch, lambda: jg.gemm_down(hq, sh, experts["down_proj"], sg["group_offsets"], block_major=blocked),
                    steps, max(2, warmup // 2))
    d_flops = 2.0 * R * D * I
    d_bytes = touched * per_expert_bytes / 3
    res["down_kernel"] = dict(avg_launch_ms=d_ms, flops_per_launch=d_flops, tflops=d_flops / d_ms / 1e9,
                              bytes_per_launch=d_bytes, gbs=d_bytes / d_ms / 1e6)
    return res


def run_ep_shard(jg, torch, steps, warmup, seed=5):
    """Benchmark config 5: one GPU's expert-parallel shard.  32 local experts of the DeepSeek-V3 shape receive
    16384 pre-dispatched rows (already in expert order: row_ids = NULL), group sizes from Zipf(1.2) with empty
    experts, combine with top-8 weights from Dirichlet(1) into 2048 tokens.  A step = gate/up GEMM, down GEMM,
    combine."""
    import numpy as np
    E, D, I, k, M = 32, 7168, 2048, 8, 2048
    R = M * k
    rng = np.random.Generator(np.random.Philox(seed))
    p = 1.0 / np.arange(1, E + 1) ** 1.2
    p[[5, 17, 30]] = 0.0                                       # forced empty experts
    p /= p.sum()
    group_sizes = np.bincount(rng.choice(E, size=R, p=p), minlength=E).astype(np.int32)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(group_sizes)]).astype(np.int32)).cuda()
    weights = torch.from_numpy(rng.dirichlet(np.ones(k), size=M).astype(np.float32)).cuda()
    inv_perm = torch.from_numpy(rng.permutation(R).astype(np.int32)).cuda()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    experts = dict(gate_proj=make_weights(jg, torch, E, I, D, gen), up_proj=make_weights(jg, torch, E, I, D, gen),
                   down_proj=make_weights(jg, torch, E, D, I, gen))
    xq, sx = jg.quant_act(torch.randn((R, D), dtype=torch.float32, device="cuda", generator=gen).to(torch.bfloat16))
    log(f"ep_shard_skewed: rows per expert, ascending: {sorted(int(v) for v in group_sizes)}")

    def step():   # (the rows arrive with row-major scales, as a dispatch all-to-all delivers them: the gather is part of the step)
        sxb = jg.gather_scales(sx)
        hq, sh = jg.gemm_gateup_swiglu(xq, sxb, experts["gate_proj"], experts["up_proj"], off, block_major=True)
        y = jg.gemm_down(hq, sh, experts["down_proj"], off, block_major=True)
        return jg.combine(y, weights, inv_perm)

    out = step()
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all(), "non-finite output"
    ms, _ = timed(torch, step, steps, warmup)
    sxb = jg.gather_scales(sx)
    k_ms, _ = timed(torch, lambda: jg.gemm_gateup_swiglu(xq, sxb, experts["gate_proj"], experts["up_proj"], off,
                                                         block_major=True), steps, max(2, warmup // 2))
    hq, sh = jg.gemm_gateup_swiglu(xq, sxb, experts["gate_proj"], experts["up_proj"], off, block_major=True)
    d_ms, _ = timed(torch, lambda: jg.gemm_down(hq, sh, experts["down_proj"], off, block_major=True), steps, max(2, warmup // 2))
    flops = 6.0 * R * D * I
    k_flops, d_flops = 4.0 * R * D * I, 2.0 * R * D * I
    touched = int((group_sizes > 0).sum())
    per_expert_bytes = 3 * D * I + 3 * (D // 128) * (I // 128) * 4
    gk = dict(avg_launch_ms=k_ms, flops_per_launch=k_flops, tflops=k_flops / k_ms / 1e9,
              bytes_per_launch=touched * per_expert_bytes * 2 / 3, gbs=touched * per_expert_bytes * 2 / 3 / k_ms / 1e6)
    dk = dict(avg_launch_ms=d_ms, flops_per_launch=d_flops, tflops=d_flops / d_ms / 1e9,
              bytes_per_launch=touched * per_expert_bytes / 3, gbs=touched * per_expert_bytes / 3 / d_ms / 1e6)
    return {"metric": "expert-parallel shard fp8 TFLOP/s (pre-dispatched rows, gate/up + down + combine)",
            "value": flops / ms / 1e9, "unit": "TFLOP/s", "ms_per_step": ms, "frac_of_peak": flops / ms / 1e9 / PEAK_FP8_TFLOPS,
            "config": {"workload": "ep_shard_skewed", "local_experts": E, "rows": R, "D": D, "I": I, "k": k, "tokens": M,
                       "touched_experts": touched, "largest_group": int(group_sizes.max()), "group_sizes": "Zipf(1.2)"},
            "roofline": kernel_roofline("mfma", gk, "ep_shard_skewed", "gateup_routed", GATEUP_NAME + ", rows in expert order"),
            "down_kernel": kernel_roofline("mfma", dk, "ep_shard_skewed", "down_routed", DOWN_NAME)}


def run_probe(reps):
    """`--probe`: the ceilings of the grouped GEMM's K loop on this box (jax-gpt_amd/csrc/moe_probe.hip: skeletons of
    the loop on all 256 CUs, no epilogue, results meaningless).  Prints one JSON line with a list of measurements."""
    import ctypes as C
    path = os.path.join(ROOT, "jax-gpt_amd", "libmoe_probe.so")
    if not os.path.exists(path):
        import __graft_entry__
        __graft_entry__.build()
    lib = C.CDLL(path)
    lib.moe_probe_variant_name.restype = C.c_char_p
    lib.moe_probe_gemm_loop.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double),
                                        C.POINTER(C.c_double)]
    sources = ["every weight line an L2 hit", "weights from HBM, 4 workgroups share a slab", "weights from HBM, every workgroup its own slab"]
    out = []
    for random_data in (1, 0):
        for v in range(lib.moe_probe_variants()):
            name = lib.moe_probe_variant_name(v).decode()
            for src in range(3):
                if "compute only" in name and src:
                    continue                      # (no copies: the source makes no difference)
                if not random_data and not (name.startswith("A  structure") or "compute only" in name):
                    continue                      # (constant data: only to show what the data cost)
                ms, tf, gbs = C.c_double(), C.c_double(), C.c_double()
                if lib.moe_probe_gemm_loop(v, src, random_data, reps, C.byref(ms), C.byref(tf), C.byref(gbs)):
                    raise RuntimeError("moe_probe_gemm_loop failed")
                rec = {"variant": name, "weights": sources[src] if "compute only" not in name else "-",
                       "data": "random fp8 codes" if random_data else "constant bytes", "ms_per_launch": ms.value,
                       "tflops": tf.value, "frac_of_fp8_peak": tf.value / PEAK_FP8_TFLOPS,
                       "weight_tile_copy_gbs": gbs.value if "compute only" not in name else 0.0}
                out.append(rec)
                log(f"{rec['data']:17s} {rec['weights']:46s} {ms.value:7.3f} ms {tf.value:7.0f} TFLOP/s {rec['weight_tile_copy_gbs']:7.0f} GB/s  {name}")
    print(json.dumps({"probe": "grouped GEMM K loop skeletons, 256 workgroups x 16 items x 56 K steps", "reps": reps,
                      "peak_fp8_tflops": PEAK_FP8_TFLOPS, "measurements": out}), flush=True)


def cpu_baseline(cfg, seconds_budget=25.0):
    """The reference's dataflow (oracle/reference_dataflow.py, a port) on the host cores, on a bounded
    sample of the prefill workload: a few experts at their mean row count."""
    import torch
    from oracle import reference_dataflow as RD
    cores = os.cpu_count() or 1
    threads = min(cores, 16)                  # a one-GPU box gives this job 16 cores' worth
    rows = max(cfg["M"] * cfg["k"] // cfg["E"], 1)
    n_exp = 32                                # about 10-20 s of host work in total
    t0 = time.perf_counter()
    r = RD.time_expert_sample(cfg["D"], cfg["I"], n_exp, rows, top_k=cfg["k"], reps=3, threads=threads)
    log(f"cpu baseline: {r['sample']}: {r['seconds']:.2f} s/pass, total {time.perf_counter() - t0:.1f} s")
    return {"value": r["flops"] / r["seconds"] / 1e12, "unit": "TFLOP/s", "cores": r["cores"], "kind": "port",
            "sample": r["sample"]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="deepseek_v3_prefill", choices=sorted(WORKLOADS))
    ap.add_argument("--no-decode", action="store_true", help="skip the decode measurement")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-extra", action="store_true", help="skip the Qwen3-MoE prefill and the expert-parallel shard parts")
    ap.add_argument("--parts", default="decode,balanced,qwen3,ep_shard",
                    help="which measurements ride along with the default prefill workload (comma-separated subset of "
                         "decode, balanced, qwen3, ep_shard; counter runs take one at a time so that a grid size names a launch)")
    ap.add_argument("--probe", action="store_true",
                    help="instead of the benchmark: time the skeletons of the grouped GEMM's K loop (compute pattern alone, "
                         "copies from L2 / HBM, alternative structures) and print their rates as one JSON line")
    ap.add_argument("--bias-std", type=float, default=0.1,
                    help="standard deviation of the selection bias of sigmoid_grouped routing (0.1 = the workload as "
                         "specified: the same 7 of 8 groups win almost every token; 0 = balanced routing)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (expert parallelism is shown as one "
              "GPU's shard); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.probe:
        run_probe(max(args.steps, 20) * 5)
        return
    import torch
    import jax_gpt_amd as jg
    from jax_gpt_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    jg.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    cfg = WORKLOADS[args.workload]
    t0 = time.perf_counter()
    layer = make_layer(jg, torch, cfg, bias_std=args.bias_std)
    torch.cuda.synchronize()
    log(f"weights for {args.workload} generated in {time.perf_counter() - t0:.1f} s")
    main_res = run_workload(jg, torch, args.workload, cfg, layer, args.steps, args.warmup)
    log(json.dumps(main_res))
    is_decode = args.workload.endswith("decode")

    decode = None
    parts = set(p for p in args.parts.split(",") if p)
    if args.no_decode:
        parts -= {"decode", "balanced"}
    if args.no_extra:
        parts -= {"balanced", "qwen3", "ep_shard"}
    if args.workload != "deepseek_v3_prefill":
        parts = set()
    if "decode" in parts:
        dcfg = WORKLOADS["deepseek_v3_decode"]
        decode = run_workload(jg, torch, "deepseek_v3_decode", dcfg, layer, max(args.steps, 20), args.warmup)
        log(json.dumps(decode))
    # the same two shapes under balanced routing (selection bias 0: every expert gets 256 +- 16 rows at prefill, about
    # 221 experts of two or three rows are touched at decode), in the default run only
    balanced = None
    if "balanced" in parts and args.bias_std != 0.0:
        flat = (layer[0], layer[1], torch.zeros_like(layer[2]), layer[3])
        balanced = (run_workload(jg, torch, "deepseek_v3_prefill_balanced", cfg, flat, args.steps, args.warmup, graph=False),
                    run_workload(jg, torch, "deepseek_v3_decode_balanced", WORKLOADS["deepseek_v3_decode"], flat,
                                 max(args.steps, 20), args.warmup))
        log(json.dumps(balanced))
    # the other two MFMA-bound configurations of the benchmark, measured in the same run (the default run only)
    qwen3 = ep_shard = None
    if parts & {"qwen3", "ep_shard"}:
        del layer
        torch.cuda.empty_cache()
    if "qwen3" in parts:
        qcfg = WORKLOADS["qwen3_moe_prefill"]
        qwen3 = run_workload(jg, torch, "qwen3_moe_prefill", qcfg, make_layer(jg, torch, qcfg, seed=2), max(args.steps, 20), args.warmup)
        log(json.dumps(qwen3))
    if "ep_shard" in parts:
        ep_shard = run_ep_shard(jg, torch, max(args.steps, 20), args.warmup)
        log(json.dumps(ep_shard))

    def prefill_obj(res, workload, cfg_):
        return {"metric": "MoE layer fp8 TFLOP/s (prefill)", "value": res["tflops"], "unit": "TFLOP/s",
                "ms_per_step": res["ms_per_step"], "graph_replay_ms_per_step": res["graph_ms_per_step"],
                "frac_of_peak": res["tflops"] / PEAK_FP8_TFLOPS,
                "config": {"workload": workload, **{k: cfg_[k] for k in ("M", "D", "E", "k", "I", "SI", "routing")},
                           "touched_experts": res["touched_experts"]},
                "roofline": kernel_roofline("mfma", res["gateup_kernel"], workload, "gateup_routed", GATEUP_NAME),
                "down_kernel": kernel_roofline("mfma", res["down_kernel"], workload, "down_routed", DOWN_NAME)}

    def decode_obj(res, workload):
        return {"metric": "HBM GB/s over touched fp8 expert weights", "value": res["gbs"], "unit": "GB/s",
                "ms_per_step": res["ms_per_step"], "graph_replay_ms_per_step": res["graph_ms_per_step"],
                "eager_ms_per_step_beside_graph_replay": res.get("eager_ms_per_step_beside_graph"),
                "graph_replay_value": res.get("graph_gbs"), "touched_experts": res["touched_experts"],
                "weight_bytes": res["weight_bytes"], "frac_of_peak": res["gbs"] / PEAK_HBM_GBS,
                "roofline": kernel_roofline("hbm", res["gateup_kernel"], workload, "gateup_routed", GATEUP_NAME),
                "down_kernel": kernel_roofline("hbm", res["down_kernel"], workload, "down_routed", DOWN_NAME)}

    tag = args.workload if args.bias_std == 0.1 else args.workload + "_bias%g" % args.bias_std
    if is_decode:
        metric, value, unit = "MoE layer HBM GB/s over touched fp8 expert weights (decode)", main_res["gbs"], "GB/s"
        head = decode_obj(main_res, tag)
    else:
        metric, value, unit = "MoE layer fp8 TFLOP/s (prefill)", main_res["tflops"], "TFLOP/s"
        head = prefill_obj(main_res, tag, cfg)
    line = {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3", "data": "synthetic",
        "config": {"workload": args.workload, **{k: cfg[k] for k in ("M", "D", "E", "k", "I", "SI", "routing")},
                   "touched_experts": main_res["touched_experts"], "bias_std": args.bias_std},
        "frac_of_peak": (value / PEAK_HBM_GBS) if is_decode else (value / PEAK_FP8_TFLOPS),
        "graph_replay_ms_per_step": main_res["graph_ms_per_step"],
        "roofline": head["roofline"], "down_kernel": head["down_kernel"],
    }
    if decode:
        line["decode"] = decode_obj(decode, "deepseek_v3_decode")
    if qwen3:
        line["qwen3_moe_prefill"] = prefill_obj(qwen3, "qwen3_moe_prefill", WORKLOADS["qwen3_moe_prefill"])
    if balanced:
        line["prefill_balanced"] = prefill_obj(balanced[0], "deepseek_v3_prefill_balanced", WORKLOADS["deepseek_v3_prefill"])
        line["prefill_balanced"]["config"]["bias_std"] = 0.0
        line["decode_balanced"] = decode_obj(balanced[1], "deepseek_v3_decode_balanced")
        line["decode_balanced"]["bias_std"] = 0.0
    if ep_shard:
        line["ep_shard_skewed"] = ep_shard
    if not args.no_cpu:
        pcfg = cfg if not is_decode else WORKLOADS["deepseek_v3_prefill"]
        line["cpu_baseline"] = cpu_baseline(pcfg)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
