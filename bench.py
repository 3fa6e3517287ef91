#!/usr/bin/env python3
"""MoE FFN layer benchmark on one MI355X.

A step is one pass of the hot path over one batch: router GEMV -> softmax top-k -> routed experts -> shared expert
-> combine for `--batch` tokens through ONE resident MoE layer. Steps cycle through `--layers` resident layers
(distinct weights, so the 256 MB Infinity Cache cannot hold the working set) and through a pool of activations, so
the router picks different experts every step. Inputs are resident in HBM before the timed region starts.

Prints one JSON line (metric: microseconds per token for one MoE layer; lower is better), with
  roofline       the dominant kernel's algorithmic bytes per launch / its measured launch duration, vs 8 TB/s
  cpu_baseline   the CPU oracle (a port of the reference's scalar double-accumulating path) on this host's cores
  batch_sweep    the ragged small batches (B = 2, 4, 8): drawn hot routing as an input, and the layer's own router
  <layout>_sweep the same on the mixed-precision layout and the two layouts with the expert formats of the reference's target file
  prefill_sweep  chunks of 512 / 2048 tokens on the MFMA tile kernels: TFLOP/s against the fp16 matrix-core peak and the HBM cap
  mid_sweep      12 .. 48 tokens through the layer's own router (iq2; f2 at 16 and 32), between the small batches and the chunks
  stack          48 layers back to back for one token (residual + RMS-norm around every layer), us per token and GB/s
  yardsticks     this machine's own streaming-read rate and fp16 matrix-core rate, measured in the same run
  topk_pool      the file-backed top-k pool (redmetal_topk_*) on a synthetic GGUF file: one token through a device slot table and a chunk of 512
                 tokens, on raw slots and with the fast path's re-laid copies; all-IQ2_XXS experts, and all-IQ2_XS ones (`iq2_xs_experts`)
The headline is timed as HIP graph replays (what a decode loop issues); the eager figure is printed beside it.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

CAL_BYTES = 256 << 20
HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=480)
    ap.add_argument("--warmup", type=int, default=96)
    ap.add_argument("--layout", choices=["iq2", "f2", "xs", "m"], default="iq2",
                    help="iq2: the benchmark definition's config 1 (all IQ2_XXS, F32 router); f2: its config 2 layout; xs / m: routed experts IQ2_XS / IQ1_M "
                         "(the formats of the reference's target file), Q6_K shared expert")
    ap.add_argument("--layers", type=int, default=48, help="resident layers the steps cycle through")
    ap.add_argument("--routing", choices=["router", "hot", "zipf"], default="router",
                    help="router: the layer's own router on the activations (router GEMV + selection inside the timed step); hot: drawn logits N(0,1) + 2.0 on "
                         "32 hot experts (the ragged small-batch config); zipf: top-k drawn from a Zipf(1.1) expert popularity (the prefill-chunk config). hot / zipf: the routing is "
                         "an input, the timed step is grouping + experts + combine")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-micro", action="store_true", help="skip the single-GEMV microbench (only run for --layout iq2 --batch 1)")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--calibrate", action="store_true", help="also run the plain copy kernel of known size (for rocprofv3 --pmc runs)")
    ap.add_argument("--f2-layers", type=int, default=48, help="layers of the handles of the other layouts that the default run's sweep adds (0: leave those sweeps out)")
    ap.add_argument("--sweep-layouts", default="f2,xs,m", help="layouts the default run adds a sweep for on handles of their own (one token through the layer's "
                                                               "own router, then B=2/4/8 with hot routing); key <layout>_sweep of the result")
    ap.add_argument("--no-sweep", action="store_true", help="skip the B=2/4/8 hot-routing sweep that the default (B=1, own router) run appends")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill-chunk sweep (512 / 2048 tokens) that the default run appends")
    ap.add_argument("--prefill-layers", type=int, default=8, help="resident layers of the chunk handles (a chunk reads about 0.4 GB of experts per layer)")
    ap.add_argument("--no-yardsticks", action="store_true", help="skip the streaming-read and matrix-core yardsticks")
    ap.add_argument("--no-pool", action="store_true", help="skip the file-backed top-k pool entries that the default run appends")
    ap.add_argument("--prime", type=int, default=2000, help="untimed steps before the warm-up that bring the clocks up (reported as clock_priming_steps)")
    return ap.parse_args()


def layer_bytes(cfg, distinct_experts, batch):
    """Algorithmic bytes of one step: weights that must be read once + activations in and out."""
    from dwarfstar_red_lite_amd import synth
    H, F, E = cfg["hidden"], cfg["ffn"], cfg["n_expert"]
    expert = 2 * F * synth.row_bytes(cfg["gate_up_type"], H) + H * synth.row_bytes(cfg["down_type"], F)
    shared = 2 * F * synth.row_bytes(cfg["sh_gate_up_type"], H) + H * synth.row_bytes(cfg["sh_down_type"], F)
    router = E * synth.row_bytes(cfg["router_type"], H)
    return {"expert_bytes": distinct_experts * expert + shared, "router_bytes": router, "gate_inp_bytes": 4 * H,
            "act_bytes": 2 * 4 * H * batch, "one_expert": expert, "shared": shared}


def oracle_given_routing(orc, cfg, lay, x, ids, w, threads):
    """CPU oracle of the experts behind a given routing: routed experts in selection order (double) + the gated shared expert"""
    import numpy as np
    H, F = cfg["hidden"], cfg["ffn"]
    L = orc.lib()
    p = lambda a: a.ctypes.data_as(orc.C.c_void_p)
    out = np.empty((x.shape[0], H), np.float32)
    for t in range(x.shape[0]):
        routed = np.empty(H, np.float64)
        idt, wt = np.ascontiguousarray(ids[t], np.uint32), np.ascontiguousarray(w[t], np.float32)
        assert L.orc_routed_topk(cfg["gate_up_type"], cfg["down_type"], p(lay["gate"]), p(lay["up"]), p(lay["down"]), lay["gate"][0].nbytes,
                                 lay["up"][0].nbytes, lay["down"][0].nbytes, p(idt), p(wt), idt.size, H, F, p(np.ascontiguousarray(x[t])), p(routed))
        sh, sc = orc.shared_expert(cfg["sh_gate_up_type"], cfg["sh_down_type"], lay["sh_gate"], lay["sh_up"], lay["sh_down"], lay["sh_gate_inp"],
                                   H, F, x[t], threads=threads)
        out[t] = (routed + sh.astype(np.float64) * sc).astype(np.float32)
    return out


def time_steps(torch, stream, step, K, W, outs, rows_written, use_graph, replays=15):
    """W untimed + exactly K timed eager steps (synchronised on both sides); then the same K steps recorded once into a HIP graph
    (kernel launches only) and replayed: every replay is checked bit for bit against the eager outputs on the rows the K steps write,
    and the median over `replays` timed replays (each exactly K steps between two synchronisations) is what a decode loop that issues
    graphs would see. That median is the reported time whenever the replays are bit-identical to the eager run."""
    with torch.cuda.stream(stream):
        for i in range(W):
            step(i)
        stream.synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            step(W + i)
        stream.synchronize()
        torch.cuda.synchronize()
        eager_ms = (time.perf_counter() - t0) * 1e3 / K
    res = {"eager_ms": eager_ms, "graph_ms": None, "ms": eager_ms, "mode": "eager", "replays_timed": 0}
    if not use_graph:
        return res
    idx = torch.tensor(sorted(rows_written), device="cuda")
    eager_rows = outs[idx].clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for i in range(K):
            step(W + i)
    times = []
    for r in range(2 + replays):                # the first two replays are untimed (the first one uploads the graph)
        outs.zero_()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        if not torch.equal(outs[idx], eager_rows):
            print("GRAPH REPLAY MISMATCH on replay %d: the eager timing is reported" % r, file=sys.stderr)
            res["replay_mismatch"] = True
            return res
        if r >= 2:
            times.append((t1 - t0) * 1e3 / K)
    times.sort()
    res["graph_ms"] = times[len(times) // 2]
    res["graph_ms_min"] = times[0]
    res["replays_timed"] = len(times)
    # one fixed mode: graph replay (the eager figure is reported beside it)
    res["ms"], res["mode"] = res["graph_ms"], "hip_graph"
    return res


def stage_profile(lib, stream, torch, step, K, W):
    """the same K steps with per-kernel begin/end timestamps (HIP events on the launch stream)"""
    n_stage = lib.redhip_profile_stage_count()
    with torch.cuda.stream(stream):
        lib.redhip_profile_begin()
        for i in range(K):
            step(W + i)
        stage_ms = (C.c_double * n_stage)()
        stage_n = (C.c_uint32 * n_stage)()
        lib.redhip_profile_end(stage_ms, stage_n, n_stage)
    return {lib.redhip_profile_stage_name(s).decode(): {"ms_total": stage_ms[s], "launches": int(stage_n[s]), "us_avg": 1e3 * stage_ms[s] / stage_n[s]}
            for s in range(n_stage) if stage_n[s]}


def kernel_roofline(cfg, synth, stages, K, B, mean_distinct, lb, traffic_key):
    """the stage with the largest summed kernel time, its algorithmic bytes (or flops) per launch and what it achieves"""
    # (chunks of a mixed layout run the shared expert's dense products on a second stream under the batch_* stage names: their durations
    # include the wait for compute units behind the routed tile kernels, so they are no candidates there)
    cand = [k for k in stages if not ("prefill_gateup" in stages and k in ("batch_gateup", "batch_down"))]
    dom = max(cand, key=lambda k: stages[k]["ms_total"])
    H, F = cfg["hidden"], cfg["ffn"]
    gate_up = lb["one_expert"] - H * synth.row_bytes(cfg["down_type"], F)
    sh_gate_up = 2 * F * synth.row_bytes(cfg["sh_gate_up_type"], H)
    sh_down = H * synth.row_bytes(cfg["sh_down_type"], F)
    down = lb["one_expert"] - gate_up
    # weights each kernel has to read once + its activations in and out (f32 x, fp16 hi/lo activations)
    per_launch = {
        "router_gemv": lb["router_bytes"] + 4 * H + B * (4 * H + 4 * cfg["n_expert"]),
        # the packed path computes the shared expert's gate/up in the same launch; the generic one has its own stage
        "gateup": mean_distinct * gate_up + (0 if "shared_gateup" in stages else sh_gate_up) + 4 * H,
        "shared_gateup": sh_gate_up + 4 * H,
        "down_combine": mean_distinct * down + sh_down + 4 * H,
        "fused_experts": lb["expert_bytes"] + 2 * 4 * H,
        "batch_gateup": mean_distinct * gate_up + sh_gate_up + B * 4 * H,
        "batch_down": mean_distinct * down + sh_down + B * 4 * H,
        "route_select": B * 4 * (cfg["n_expert"] + 1),
        # the partial output vectors of the one-token expert slices, read once, and the output
        "slice_sum": (cfg["top_k"] + 1) * (F // 32) * H * 4 + 4 * H,
    }
    dom_bytes = per_launch.get(dom)
    dom_us = stages[dom]["us_avg"] * (stages[dom]["launches"] / K)        # per step, if launched more than once per step
    # HBM bytes per launch of the dominant kernel, from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs recorded under
    # profiles/ (counters cannot be collected from inside this process); null for workloads that were not profiled
    traffic = None
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as fh:
            rec = json.load(fh).get(traffic_key, {}).get("stages", {}).get(dom)
        if rec:
            traffic = int(rec["fetch_bytes"] + rec["write_bytes"])
    except (OSError, ValueError, KeyError):
        traffic = None
    if dom in ("prefill_gateup", "prefill_down"):
        # prefill tiles run on the MFMA units: algorithmic flops of the stage (2 per multiply-add, every (token, expert) pair
        # and every token's shared expert once; the fp16 hi/lo split that doubles the issued MFMAs is not counted)
        pairs = B * (cfg["top_k"] + (0 if "batch_gateup" in stages else 1))      # (mixed layouts: the shared expert runs as dense f32 products beside the tiles)
        flops = pairs * 2.0 * H * F * (2 if dom == "prefill_gateup" else 1)
        achieved = flops / (dom_us * 1e-6) / 1e12
        return {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 2), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 4), "traffic": traffic, "flops_per_launch": int(flops), "launch_us": round(dom_us, 3)}
    if dom_bytes:
        achieved = dom_bytes / (dom_us * 1e-6) / 1e9
        return {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "bytes_per_launch": int(dom_bytes), "launch_us": round(dom_us, 3)}
    return None


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    import oracle_lib as orc
    from dwarfstar_red_lite_amd import load, synth
    from dwarfstar_red_lite_amd.moe import ResidentMoe

    lib = load()
    torch.cuda.init()
    B, NL = args.batch, args.layers
    K, W = args.steps, args.warmup
    grids = None
    if args.layout in ("xs", "m") or "xs" in args.sweep_layouts.split(",") or "m" in args.sweep_layouts.split(","):
        # these two decode through codebooks the caller supplies: the reference's, from the fixture
        from dwarfstar_red_lite_amd import moe as moe_api
        g = json.load(open(os.path.join(ROOT, "tests", "golden", "iq_grids.json")))
        grids = [np.frombuffer(bytes.fromhex(g[k]), np.int8) for k in ("iq2_xs", "iq1_m")]
        moe_api.set_codebooks(*grids)
        orc.set_codebooks(*grids)
    # the default run (one token, the layer's own router) appends the small-batch sweep on the same resident handle
    sweep = [] if (args.no_sweep or B != 1 or args.routing != "router") else [2, 4, 8]
    sweep_layouts = [l for l in args.sweep_layouts.split(",") if l] if (sweep and args.layout == "iq2" and args.f2_layers > 0) else []
    for l in sweep_layouts:
        if l not in ("f2", "xs", "m"):
            raise SystemExit("bench.py: unknown layout %r in --sweep-layouts" % l)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(20241125)
    stream = torch.cuda.Stream()
    NX_DECODE = 64

    def resident_handle(layout, NL, max_tokens):
        """a handle with NL layers of the layout resident (weights drawn on the GPU), layer 0 also on the host for the oracle"""
        cfg = synth.layer_config(layout=layout)
        moe = ResidentMoe(cfg, n_layer=NL, max_tokens=max_tokens)
        layer0 = None
        for l in range(NL):
            a = synth.make_layer_gpu(torch, gen, cfg)
            moe.load_layer(l, a)
            if l == 0:
                layer0 = synth.layer_to_host(a, cfg)
            del a
        torch.cuda.synchronize()
        return {"layout": layout, "cfg": cfg, "moe": moe, "NL": NL, "layer0": layer0, "ref": orc.Layer(cfg, **layer0)}

    def run_workload(ctx, B, routing):
        """parity gate on layer 0, then timing, per-kernel profile and the dominant kernel's roofline for batches of B tokens"""
        cfg, moe, NL, layer0, ref = ctx["cfg"], ctx["moe"], ctx["NL"], ctx["layer0"], ctx["ref"]
        H = cfg["hidden"]
        NX = NX_DECODE if B <= 64 else max(4, 4096 // B)          # activation sets the steps cycle through (chunks: fewer, larger ones)
        prime = args.prime if B <= 64 else max(50, args.prime // 10)
        xs_host = synth.normed_x(np.random.default_rng(99 + B), NX * B, H).reshape(NX, B, H)
        xs = torch.from_numpy(xs_host).cuda()
        outs = torch.zeros_like(xs)
        # drawn routing (the ragged small-batch and prefill-chunk configurations): ids / weights per activation set, made on the host
        route_ids = route_w = ids_h = w_h = None
        if routing != "router":
            rr = np.random.default_rng(7)
            K_, E_ = cfg["top_k"], cfg["n_expert"]
            ids_h = np.empty((NX, B, K_), np.uint32)
            w_h = np.empty((NX, B, K_), np.float32)
            for i in range(NX):
                if routing == "hot":
                    lg = synth.hot_logits(rr, B, E_)
                    for t in range(B):
                        ids_h[i, t], w_h[i, t] = orc.router_select(lg[t], K_)
                else:
                    ids_h[i] = synth.zipf_topk(rr, B, E_, K_)
                    ww = rr.random((B, K_)).astype(np.float32) + 0.1
                    w_h[i] = ww / ww.sum(axis=1, keepdims=True)
            route_ids = torch.from_numpy(ids_h.astype(np.int32)).cuda()
            route_w = torch.from_numpy(w_h).cuda()

        def step(i):
            if route_ids is None:
                moe.forward(i % NL, xs[i % NX], outs[i % NX])
            else:
                moe.experts(i % NL, xs[i % NX], route_ids[i % NX], route_w[i % NX], outs[i % NX])

        # ---- parity gate on the very tensors the timed steps use (layer 0, CPU oracle) ----
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            step(0)
            if route_ids is None:
                gids, _, _ = moe.last_route(B)
            stream.synchronize()
        if route_ids is None:           # (chunks: the first eight tokens - tokens are independent of each other)
            n_chk = min(B, 8)
            want, cids, _, _ = ref.forward(xs_host[0][:n_chk], threads=os.cpu_count() or 1)
            got = outs[0][:n_chk].cpu().numpy()
            ids_ok = bool(np.array_equal(gids[:n_chk], cids))
        else:           # drawn routing: the oracle's routed experts + gated shared expert for the first tokens of the step
            n_chk = min(B, 8)
            want = oracle_given_routing(orc, cfg, layer0, xs_host[0][:n_chk], ids_h[0][:n_chk], w_h[0][:n_chk], os.cpu_count() or 1)
            got = outs[0][:n_chk].cpu().numpy()
            ids_ok = True
        rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
        if not rel <= 1e-3 or not ids_ok:
            print("PARITY FAILURE (B=%d, routing %s): rel L2 %.3g vs the CPU oracle, router ids identical: %s" % (B, routing, rel, ids_ok), file=sys.stderr)
            sys.exit(1)

        # ---- untimed clock priming, then the timed region ----
        with torch.cuda.stream(stream):
            for i in range(prime):
                step(i)
            stream.synchronize()
        rows_written = {(W + i) % NX for i in range(K)}
        tm = time_steps(torch, stream, step, K, W, outs, rows_written, not args.no_graph)
        stages = stage_profile(lib, stream, torch, step, K, W)
        # distinct routed experts per step (B > 1 shares experts between tokens)
        distinct = []
        with torch.cuda.stream(stream):
            for i in range(min(K, NX)):
                if route_ids is None:
                    step(W + i)
                    ids, _, _ = moe.last_route(B)
                else:
                    ids = ids_h[(W + i) % NX]
                distinct.append(len(set(ids.ravel().tolist())))
        mean_distinct = float(np.mean(distinct))
        lb = layer_bytes(cfg, mean_distinct, B)
        roof = kernel_roofline(cfg, synth, stages, K, B, mean_distinct, lb, "%s_b%d" % (ctx["layout"], B) + ("" if routing == "router" else "_" + routing))
        return {"B": B, "routing": routing, "timing": tm, "stages": stages, "mean_distinct": mean_distinct, "lb": lb, "roofline": roof, "rel": rel,
                "ids_ok": ids_ok, "xs": xs, "xs_host": xs_host, "NX": NX}

    main_ctx = resident_handle(args.layout, NL, max([B] + sweep))
    cfg, moe = main_ctx["cfg"], main_ctx["moe"]
    H, F = cfg["hidden"], cfg["ffn"]
    ref = main_ctx["ref"]
    head = run_workload(main_ctx, B, args.routing)
    tm, stages, lb, mean_distinct = head["timing"], head["stages"], head["lb"], head["mean_distinct"]
    ms_per_step = tm["ms"]
    xs, xs_host = head["xs"], head["xs_host"]
    n_stage = lib.redhip_profile_stage_count()
    if args.calibrate:         # yardstick for FETCH_SIZE / WRITE_SIZE: copies of exactly CAL_BYTES in, CAL_BYTES out
        cal_src = torch.empty(CAL_BYTES, dtype=torch.uint8, device="cuda").random_(0, 256)
        cal_dst = torch.empty_like(cal_src)
        for _ in range(4):
            assert lib.redhip_calibration_copy(cal_dst.data_ptr(), cal_src.data_ptr(), CAL_BYTES, None)
        torch.cuda.synchronize()

    us_per_token = ms_per_step * 1e3 / B
    total_bytes = lb["expert_bytes"] + lb["router_bytes"] + lb["gate_inp_bytes"] + lb["act_bytes"]
    result = {
        "metric": "moe_ffn_layer_us_per_token", "value": round(us_per_token, 3), "unit": "us/token", "n_gpus": 1,
        "steps": K, "warmup": W, "ms_per_step": round(ms_per_step, 6), "launch_mode": tm["mode"],
        "eager_ms_per_step": round(tm["eager_ms"], 6),
        "graph_ms_per_step": None if tm["graph_ms"] is None else round(tm["graph_ms"], 6),
        "graph_replays_timed": tm["replays_timed"], "clock_priming_steps": args.prime,
        "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: one MoE FFN layer, B=%d decode token(s), hidden 2048, 512 experts top-10 + shared, ffn 512, layout %s, "
                               "all experts of %d layers resident" % ({"iq2": "config1", "f2": "config2"}.get(args.layout, "target-file expert format"),
                                                                      B, args.layout, NL),
                   "layout": args.layout, "batch": B, "routing": args.routing, "resident_layers": NL, "resident_gb": round(moe.resident_bytes / 1e9, 2),
                   "mean_distinct_routed_experts": mean_distinct,
                   "arithmetic": "weights exact in fp16 (integer codebook values, block scales applied in f32), activations as fp16 hi + lo halves "
                                 "(22 significant bits), f32 accumulation"},
        "layer_gbps": {"expert_bytes": int(lb["expert_bytes"]), "layer_bytes": int(total_bytes),
                       "expert_gbps": round(lb["expert_bytes"] / (ms_per_step * 1e-3) / 1e9, 1),
                       "layer_gbps": round(total_bytes / (ms_per_step * 1e-3) / 1e9, 1),
                       "frac_of_peak_on_expert_bytes": round(lb["expert_bytes"] / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
        "stages_us": {k: round(v["us_avg"] * v["launches"] / K, 3) for k, v in stages.items()},
        "parity": {"rel_l2_vs_cpu_oracle": head["rel"], "router_ids_identical": head["ids_ok"]},
        "roofline": head["roofline"],
    }

    # ---- what the launches alone cost on this machine: the same number of dependent launches per step with the same grids, empty kernels ----
    if B == 1 and not args.no_graph:
        shapes = [(136, 256), (176, 1024), (64, 256)]          # router, expert slices, sum of the partial vectors
        with torch.cuda.stream(stream):
            for g_, b_ in shapes:
                assert lib.redhip_calibration_empty(g_, b_, stream.cuda_stream)
            stream.synchronize()
            gf = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gf, stream=stream):
                for _ in range(K):
                    for g_, b_ in shapes:
                        lib.redhip_calibration_empty(g_, b_, stream.cuda_stream)
        ts = []
        for r in range(12):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            gf.replay()
            torch.cuda.synchronize()
            ts.append((time.perf_counter() - t0) * 1e6 / K)
        ts = sorted(ts[2:])
        result["launch_floor_us"] = round(ts[len(ts) // 2], 3)
        result["launch_floor_note"] = "three dependent launches of empty kernels per step (grids of %s), %d steps per graph replay, median of %d replays" % (
            " / ".join("%dx%d" % sh for sh in shapes), K, len(ts))

    # ---- the ragged small-batch configuration on the same resident handle: B = 2, 4, 8; drawn logits with 32 hot experts (the routing is an
    # input, as the configuration defines it), and the same batches through the layer's own router (router GEMV + selection in the step) ----
    def sweep_entry(ctx, b, routing):
        r = run_workload(ctx, b, routing)
        t = r["timing"]
        rf = r["roofline"] or {}
        return {"batch": b, "routing": routing, "us_per_step": round(t["ms"] * 1e3, 3), "us_per_token": round(t["ms"] * 1e3 / b, 3), "launch_mode": t["mode"],
                "eager_us_per_step": round(t["eager_ms"] * 1e3, 3), "mean_distinct_routed_experts": r["mean_distinct"],
                "stages_us": {k: round(v["us_avg"] * v["launches"] / K, 3) for k, v in r["stages"].items()},
                "dominant_kernel": rf.get("kernel"), "kernel_us": rf.get("launch_us"), "kernel_gbps": rf.get("achieved"), "kernel_frac_of_peak": rf.get("frac"),
                "kernel_traffic_bytes": rf.get("traffic"), "expert_bytes": int(r["lb"]["expert_bytes"]),
                "step_gbps_on_expert_bytes": round(r["lb"]["expert_bytes"] / (t["ms"] * 1e-3) / 1e9, 1), "rel_l2_vs_cpu_oracle": r["rel"]}

    # ---- prefill chunks on the MFMA tile kernels: algorithmic flops (2 per multiply-add, every (token, expert) pair's three products and every
    # token's shared expert once; the fp16 hi / lo split doubles the MFMAs issued and is not counted) against the dense fp16 matrix-core peak,
    # and the HBM cap: the bytes of the distinct experts the chunk touches (+ shared expert + router) against 8 TB/s ----
    def chunk_entry(ctx, ntok, routing):
        r = run_workload(ctx, ntok, routing)
        c, t, lb = ctx["cfg"], r["timing"], r["lb"]
        us = t["ms"] * 1e3
        flops = ntok * (c["top_k"] + 1) * 3 * 2.0 * c["hidden"] * c["ffn"]
        cap_bytes = lb["expert_bytes"] + lb["router_bytes"] + lb["gate_inp_bytes"] + lb["act_bytes"]
        return {"layout": ctx["layout"], "tokens": ntok, "routing": routing, "us_per_chunk": round(us, 2), "us_per_token": round(us / ntok, 4),
                "launch_mode": t["mode"], "eager_us_per_chunk": round(t["eager_ms"] * 1e3, 2), "resident_layers": ctx["NL"],
                "mean_distinct_routed_experts": r["mean_distinct"],
                "stages_us": {k: round(v["us_avg"] * v["launches"] / K, 3) for k, v in r["stages"].items()},
                "roofline": r["roofline"],
                "chunk_flops": int(flops), "chunk_tflops": round(flops / (us * 1e-6) / 1e12, 2),
                "chunk_frac_of_mfma_peak": round(flops / (us * 1e-6) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                "hbm_cap": {"bytes": int(cap_bytes), "us_at_peak": round(cap_bytes / HBM_PEAK_GBS / 1e3, 2), "achieved_gbps": round(cap_bytes / (us * 1e-6) / 1e9, 1),
                            "frac": round(cap_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)},
                "rel_l2_vs_cpu_oracle": r["rel"], "router_ids_identical": r["ids_ok"]}

    # ---- 48 layers back to back for one token: x <- (x + branch) + layer_l(rmsnorm(x + branch)) for l = 0 .. NL - 1, every layer's input the
    # previous layer's output (the residual add and RMS-norm ride in the layer's own launches). Gate: layer 0's block step against the oracle. ----
    def stack_entry(ctx, n_tok=10):
        c, m, NL = ctx["cfg"], ctx["moe"], ctx["NL"]
        Hc = c["hidden"]
        rs = np.random.default_rng(4242)
        x0 = (2.0 * rs.standard_normal((1, Hc))).astype(np.float32)
        br = (0.5 * rs.standard_normal((NX_DECODE, 1, Hc))).astype(np.float32)
        pw = np.ones(Hc, np.float32)
        brd, pwd = torch.from_numpy(br).cuda(), torch.from_numpy(pw).cuda()
        xd = torch.from_numpy(x0).cuda()
        with torch.cuda.stream(stream):
            got = m.forward_block(0, xd, brd[0], pwd, 1e-6).cpu().numpy()
            gids, _, _ = m.last_route(1)
        resid = (x0 + br[0]).astype(np.float32)
        normed = np.empty_like(resid)
        orc.lib().orc_rmsnorm(resid[0].ctypes.data, pw.ctypes.data, Hc, 1e-6, normed[0].ctypes.data)
        ffn, cids, _, _ = ctx["ref"].forward(normed, threads=os.cpu_count() or 1)
        want = resid + ffn.astype(np.float32)
        rel = float(np.linalg.norm((got - resid) - (want - resid)) / np.linalg.norm(want - resid))
        if not rel <= 1e-3 or not np.array_equal(gids, cids):
            print("PARITY FAILURE (stack, %s): block step of layer 0 rel L2 %.3g" % (ctx["layout"], rel), file=sys.stderr)
            sys.exit(1)

        def token(i):
            for l in range(NL):
                m.forward_block(l, xd, brd[(i * NL + l) % NX_DECODE], pwd, 1e-6, out=xd)
        with torch.cuda.stream(stream):
            for i in range(20):
                token(i)
            stream.synchronize()
            t0 = time.perf_counter()
            for i in range(n_tok):
                token(i)
            stream.synchronize()
            eager_us = (time.perf_counter() - t0) * 1e6 / n_tok
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for i in range(n_tok):
                    token(i)
        ts = []
        for rpl in range(12):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            g.replay()
            torch.cuda.synchronize()
            ts.append((time.perf_counter() - t0) * 1e6 / n_tok)
        ts = sorted(ts[2:])
        us = ts[len(ts) // 2]
        finite = bool(torch.isfinite(xd).all().item())
        lb1 = layer_bytes(c, c["top_k"], 1)
        per_layer = lb1["expert_bytes"] + lb1["router_bytes"] + lb1["gate_inp_bytes"]
        return {"layout": ctx["layout"], "layers": NL, "batch": 1, "us_per_token": round(us, 2), "us_per_layer": round(us / NL, 3), "launch_mode": "hip_graph",
                "eager_us_per_token": round(eager_us, 2), "tokens_per_replay": n_tok, "replays_timed": len(ts),
                "bytes_per_token": int(per_layer * NL), "gbps": round(per_layer * NL / us / 1e3, 1), "frac_of_hbm_peak": round(per_layer * NL / us / 1e3 / HBM_PEAK_GBS, 4),
                "us_at_60pct_of_peak": round(per_layer * NL / (0.6 * HBM_PEAK_GBS) / 1e3, 1), "output_finite": finite,
                "rel_l2_vs_cpu_oracle_layer0_block": rel}

    if sweep:
        result["batch_sweep"] = [sweep_entry(main_ctx, b, "hot") for b in sweep] + [sweep_entry(main_ctx, b, "router") for b in sweep]
        if NL >= 48:
            result["stack"] = [stack_entry(main_ctx)]
        # ---- the other layouts, each on a handle of its own: the mixed-precision layout of config 2 (f2) and the layouts with the expert
        # formats of the reference's target file (xs: IQ2_XS, m: IQ1_M experts). One token with the layer's own router, then the same ragged
        # batches; all 48 layers resident like the headline handle ----
        for lay in sweep_layouts:
            ctx = resident_handle(lay, args.f2_layers, max(sweep))
            result[lay + "_sweep"] = {"resident_layers": args.f2_layers, "resident_gb": round(ctx["moe"].resident_bytes / 1e9, 2),
                                      "runs": [sweep_entry(ctx, 1, "router")] + [sweep_entry(ctx, b, "hot") for b in sweep] +
                                              ([sweep_entry(ctx, b, "router") for b in sweep] if lay == "f2" else [])}
            if lay == "f2" and args.f2_layers >= 48:
                result.setdefault("stack", []).append(stack_entry(ctx))
            ctx["moe"].close()
            del ctx
            torch.cuda.empty_cache()

    # ---- prefill chunks (handles of their own, made for chunks: they also hold the tile-major copies) ----
    if sweep and not args.no_prefill:
        moe.close()                                   # the headline handle is no longer needed: its memory goes to the chunk handles
        main_ctx["moe"] = None
        torch.cuda.empty_cache()
        pre = []
        ctx = resident_handle("iq2", args.prefill_layers, 2048)
        pre.append(chunk_entry(ctx, 512, "router"))
        pre.append(chunk_entry(ctx, 512, "zipf"))
        pre.append(chunk_entry(ctx, 2048, "router"))
        # between the small batches and the chunks: 12 .. 32 tokens through the layer's own router (one batch of expert slices), 48 on the tiles
        mid = [dict(sweep_entry(ctx, b, "router"), layout="iq2") for b in (12, 16, 24, 32, 48)]
        ctx["moe"].close()
        del ctx
        torch.cuda.empty_cache()
        ctx = resident_handle("f2", args.prefill_layers, 2048)
        pre.append(chunk_entry(ctx, 512, "zipf"))
        pre.append(chunk_entry(ctx, 512, "router"))
        pre.append(chunk_entry(ctx, 2048, "zipf"))
        mid += [dict(sweep_entry(ctx, b, "router"), layout="f2") for b in (16, 32)]
        ctx["moe"].close()
        del ctx
        torch.cuda.empty_cache()
        result["prefill_sweep"] = pre
        result["mid_sweep"] = mid

    # ---- this machine's own yardsticks, in the same run: streaming read of 1 GiB (four times the 256 MB last-level cache) and a dense fp16
    # matrix-core loop on register operands ----
    if not args.no_yardsticks:
        n_stage_ = lib.redhip_profile_stage_count()
        buf = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 256)
        sink = torch.zeros(4, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()

        def timed(launch, reps):
            with torch.cuda.stream(stream):
                for _ in range(2):
                    launch()
                stream.synchronize()
                lib.redhip_profile_begin()
                for _ in range(reps):
                    launch()
                sm_, sn_ = (C.c_double * n_stage_)(), (C.c_uint32 * n_stage_)()
                lib.redhip_profile_end(sm_, sn_, n_stage_)
            return 1e3 * sum(sm_) / max(sum(sn_), 1)          # average kernel duration in us
        rd_us = timed(lambda: lib.redhip_calibration_read(buf.data_ptr(), buf.numel(), sink.data_ptr(), stream.cuda_stream), 8)
        cp_src, cp_dst = buf[:CAL_BYTES], torch.empty(CAL_BYTES, dtype=torch.uint8, device="cuda")
        cp_us = timed(lambda: lib.redhip_calibration_copy(cp_dst.data_ptr(), cp_src.data_ptr(), CAL_BYTES, stream.cuda_stream), 8)
        fl = C.c_uint64(0)
        mf_us = timed(lambda: lib.redhip_calibration_mfma(2048, 2048, sink.data_ptr(), C.byref(fl), stream.cuda_stream), 4)
        result["yardsticks"] = {
            "streaming_read": {"bytes": int(buf.numel()), "us": round(rd_us, 2), "gbps": round(buf.numel() / rd_us / 1e3, 1),
                               "frac_of_published_peak": round(buf.numel() / rd_us / 1e3 / HBM_PEAK_GBS, 4)},
            "copy": {"bytes_in": CAL_BYTES, "bytes_out": CAL_BYTES, "us": round(cp_us, 2), "gbps_in_plus_out": round(2 * CAL_BYTES / cp_us / 1e3, 1)},
            "mfma_f16_16x16x32": {"flops": int(fl.value), "us": round(mf_us, 2), "tflops": round(fl.value / mf_us / 1e6, 1),
                                  "frac_of_published_peak": round(fl.value / mf_us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4)},
            "note": "kernel durations from the dispatches' own timestamps; published peaks: HBM 8 TB/s, dense fp16 MFMA 2.5 PFLOP/s"}
        del buf, cp_dst

    # ---- per-kernel microbench of config 1: one IQ2_XXS dequant-GEMV [512 x 2048] x [2048] on raw GGUF rows ----
    if args.layout == "iq2" and B == 1 and not args.no_micro:
        NM, reps = 1024, 2048                   # 1024 distinct matrices = 277 MB, more than the 256 MB last-level cache
        mats = torch.randint(0, 256, (NM, F * synth.row_bytes(synth.TYPE_IQ2_XXS, H)), dtype=torch.uint8, device="cuda", generator=gen)
        mats.view(NM * F * (H // 256), 66)[:, 1] = 0x1E            # d in [2^-8, 2^-7): finite whatever the random low byte
        yv = torch.empty((NM, F), dtype=torch.float32, device="cuda")
        xg = xs[0, 0].contiguous()
        torch.cuda.synchronize()                # the matrices were filled on the default stream, the launches go to `stream`

        def gemv(i):
            ok = lib.redhip_gemv_rows(synth.TYPE_IQ2_XXS, mats[i % NM].data_ptr(), H, 0, F, xg.data_ptr(), yv[i % NM].data_ptr(),
                                      stream.cuda_stream)
            assert ok
        with torch.cuda.stream(stream):
            for i in range(64):
                gemv(i)
            stream.synchronize()
            want_row = orc.matvec(synth.TYPE_IQ2_XXS, mats[5].cpu().numpy(), H, xs_host[0, 0])
            got_row = yv[5].cpu().numpy()
            micro_rel = float(np.linalg.norm(got_row - want_row) / np.linalg.norm(want_row))
            g2 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g2, stream=stream):
                for i in range(reps):
                    gemv(i)
            g2.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            g2.replay()
            torch.cuda.synchronize()
            gemv_us = (time.perf_counter() - t0) * 1e6 / reps
            lib.redhip_profile_begin()
            for i in range(reps):
                gemv(i)
            sm, sn = (C.c_double * n_stage)(), (C.c_uint32 * n_stage)()
            lib.redhip_profile_end(sm, sn, n_stage)
        kern_us = 1e3 * sum(sm) / max(sum(sn), 1)
        gemv_bytes = F * synth.row_bytes(synth.TYPE_IQ2_XXS, H) + 4 * H + 4 * F
        fused_us = sum(v for k, v in result["stages_us"].items() if k in ("gateup", "down_combine", "fused_experts", "slice_sum"))
        result["microbench"] = {
            "iq2_xxs_gemv_512x2048": {"us_back_to_back": round(gemv_us, 3), "kernel_us": round(kern_us, 3), "bytes": gemv_bytes,
                                      "gbps_back_to_back": round(gemv_bytes / gemv_us / 1e3, 1), "gbps_kernel": round(gemv_bytes / kern_us / 1e3, 1),
                                      "rel_l2_vs_cpu_oracle": micro_rel,
                                      "note": "%d launches replayed from one HIP graph over %d distinct matrices; kernel_us = the dispatches' own "
                                              "begin/end timestamps" % (reps, NM)},
            "fused_experts_10_routed_1_shared": {"us": round(fused_us, 3), "bytes": int(lb["expert_bytes"]),
                                                 "gbps": round(lb["expert_bytes"] / fused_us / 1e3, 1),
                                                 "note": "the expert launches of the timed steps (everything behind the router launch)"}}
        if not micro_rel <= 1e-3:
            print("PARITY FAILURE in the GEMV microbench: rel L2 %.3g" % micro_rel, file=sys.stderr)
            sys.exit(1)

    # ---- the file-backed top-k pool (redmetal_topk_*), the surface the reference's engine binds: ten experts for one token through a device
    # slot table (encode_device_into) and a chunk of 512 tokens x top-10 (encode_batched), on raw GGUF slots and on a pool with the fast
    # path's re-laid copies; 512 experts of the config shape read from a synthetic GGUF file: all IQ2_XXS, and (`iq2_xs_experts`) all IQ2_XS ----
    def pool_entry(playout, word, codebooks):
        import tempfile

        from dwarfstar_red_lite_amd.gguf_writer import write_moe_gguf
        from dwarfstar_red_lite_amd.moe import gguf_expert_layout
        from dwarfstar_red_lite_amd.redmetal_topk import ExpertLayout, RedMetalTopKPool
        PE, PK, PT = 512, cfg["top_k"], 512
        pcfg = synth.layer_config(hidden=H, ffn=F, n_expert=PE, top_k=PK, layout=playout)
        play = synth.make_layer(4242, pcfg)
        tmpd = tempfile.mkdtemp(prefix="redhip_pool_")
        gguf = os.path.join(tmpd, "pool.gguf")
        write_moe_gguf(gguf, pcfg, [play])
        lays = []
        for e in range(PE):
            d = gguf_expert_layout(gguf, PE, 0, e)
            lays.append(ExpertLayout(d["gate_offset"], d["gate_bytes"], d["up_offset"], d["up_bytes"], d["down_offset"], d["down_bytes"]))
        payload = 2 * lays[0].gate_bytes + lays[0].down_bytes
        up_ = lambda v, a_: (v + a_ - 1) // a_ * a_
        cb_xs, cb_m = codebooks
        prng = np.random.default_rng(77)
        NLIST = 32
        lists = [prng.permutation(PE)[:PK] for _ in range(NLIST)]
        pw = [(prng.random(PK).astype(np.float32) + 0.1) for _ in range(NLIST)]
        px = torch.from_numpy(synth.normed_x(prng, max(NLIST, PT), H)).cuda()
        logit = prng.standard_normal((PT, PE))
        bids = np.argsort(-logit, axis=1)[:, :PK].astype(np.uint32)
        bw = prng.random((PT, PK)).astype(np.float32) + 0.05
        uid, start, ptok, pweight, tpair = orc.group_pairs(bids, bw, PE)
        entry = {"experts": PE, "expert_bytes": int(payload), "note": "graph replay of 128 single-token calls over 32 different expert lists; batched: 16 calls "
                 "queued back to back, device time per call; raw = the pool as the reference defines it (raw GGUF bytes per slot), fast = "
                 "redhip_topk_pool_enable_fast_path with tile-major copies"}
        for mode in ("raw", "fast"):
            # (a slot of the fast pool: raw bytes, the re-laid copy - 8 bytes per 32 weights + 2 per 256, IQ2_XS 9 per 32 - and the tile-major one)
            copy_b = 3 * (H * F // 32 * (9 if word == 17 else 8) + H * F // 256 * 2)
            phys = up_(up_(payload, 256) + up_(copy_b, 256) + copy_b, 4096) if mode == "fast" else up_(payload, 4096)
            pool = RedMetalTopKPool(gguf, (PE + 2) * phys, payload, slots_per_slab=64, iq2_xs_grid=cb_xs, iq1_m_grid=cb_m)
            if mode == "fast":
                pool.enable_fast_path(word, H, F, tiles=True)
            for e in range(PE):
                pool.load(e, lays[e])
            addr = [pool.addresses(e, lays[e])[0] for e in range(PE)]
            tabs = [torch.from_numpy(np.array([addr[e] for e in l], np.uint64).view(np.int64)).cuda() for l in lists]
            wdev = [torch.from_numpy(w_).cuda() for w_ in pw]
            pouts = torch.zeros(NLIST, H, device="cuda")
            gb = lays[0].gate_bytes

            def run_lists(st):
                for i in range(NLIST):
                    pool.encode_device_into(st, tabs[i].data_ptr(), wdev[i].data_ptr(), PK, word, H, F, gb, gb, px[i].data_ptr(), pouts[i].data_ptr())
            with torch.cuda.stream(stream):
                run_lists(stream.cuda_stream)
                stream.synchronize()
                want = sum(float(w_) * orc.expert_ffn(word, word, play["gate"][e], play["up"][e], play["down"][e], H, F, px[0].cpu().numpy())
                           for e, w_ in zip(lists[0], pw[0]))
                prel = float(np.linalg.norm(pouts[0].cpu().numpy() - want) / np.linalg.norm(want))
                if not prel <= 1e-3:
                    print("PARITY FAILURE in the top-k pool (%s): rel L2 %.3g" % (mode, prel), file=sys.stderr)
                    sys.exit(1)
                pgraph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(pgraph, stream=stream):
                    for _ in range(4):
                        run_lists(stream.cuda_stream)
                ts = []
                for _ in range(10):
                    stream.synchronize()
                    t0_ = time.perf_counter()
                    pgraph.replay()
                    stream.synchronize()
                    ts.append((time.perf_counter() - t0_) * 1e6 / (4 * NLIST))
                one_us_ = sorted(ts[2:])[len(ts[2:]) // 2]
                del pgraph
                # the chunk
                bout = torch.zeros(PT, H, device="cuda")
                slots_b = [int(e) for e in uid]
                lays_b = [lays[int(e)] for e in uid]

                # (the C entry point itself, its host arrays made once: the Python bridge spends 0.2 ms per call turning 512 layout tuples into arrays)
                ids_a = np.ascontiguousarray(slots_b, np.uint32)
                gb_a, ub_a, db_a = (np.ascontiguousarray([getattr(l_, f_) for l_ in lays_b], np.uint64) for f_ in ("gate_bytes", "up_bytes", "down_bytes"))
                pt_a, pw_a = np.ascontiguousarray(ptok, np.uint32), np.ascontiguousarray(pweight, np.float32)
                es_a, tp_a = np.ascontiguousarray(start, np.uint32), np.ascontiguousarray(tpair, np.uint32)

                def run_chunk():
                    if not pool.lib.redmetal_topk_pool_encode_batched(pool.handle, stream.cuda_stream, ids_a.ctypes.data, gb_a.ctypes.data, ub_a.ctypes.data,
                                                                      db_a.ctypes.data, ids_a.size, word, H, F, 0, PT, PK, pt_a.size, pt_a.ctypes.data, pw_a.ctypes.data,
                                                                      es_a.ctypes.data, tp_a.ctypes.data, px.data_ptr(), 0, bout.data_ptr(), 0):
                        raise SystemExit("encode_batched failed: " + pool._last_error())
                for _ in range(2):
                    run_chunk()
                stream.synchronize()
                row = bout[5].cpu().numpy()
                want_b = sum(float(w_) * orc.expert_ffn(word, word, play["gate"][e], play["up"][e], play["down"][e], H, F, px[5].cpu().numpy())
                             for e, w_ in zip(bids[5], bw[5]))
                brel = float(np.linalg.norm(row - want_b) / np.linalg.norm(want_b))
                if not brel <= 1e-3:
                    print("PARITY FAILURE in the batched top-k pool (%s): rel L2 %.3g" % (mode, brel), file=sys.stderr)
                    sys.exit(1)
                nrep = 16 if mode == "fast" else 4
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(nrep):
                    run_chunk()
                e1.record(stream)
                stream.synchronize()
                chunk_us = e0.elapsed_time(e1) * 1e3 / nrep
                pool.release(slots_b)
            entry[mode] = {"encode_device_into_us": round(one_us_, 2), "encode_device_into_gbps": round(PK * payload / one_us_ / 1e3, 1),
                           "encode_batched_512_tokens_us": round(chunk_us, 1), "distinct_experts_in_chunk": int(len(uid)),
                           "pool_bytes": int(pool.telemetry()["allocated_bytes"]), "rel_l2_vs_cpu_oracle": prel, "rel_l2_batched_row": brel}
            pool.close()
            del tabs, wdev, pouts, bout
            torch.cuda.empty_cache()
        try:
            os.remove(gguf)
            os.rmdir(tmpd)
        except OSError:
            pass
        return entry

    if args.layout == "iq2" and B == 1 and sweep and not args.no_pool:
        result["topk_pool"] = pool_entry("iq2", 16, (np.zeros(512 * 8, np.int8), np.zeros(2048 * 8, np.int8)))      # (codebooks of formats this file does not use)
        if grids is not None:      # the same with IQ2_XS experts, the format of the reference's target file
            result["topk_pool"]["iq2_xs_experts"] = pool_entry("xs", 17, grids)

    # ---- CPU baseline: the oracle on this host's cores, layer 0, same activations ----
    if not args.no_cpu:
        cores = min(os.cpu_count() or 1, 64)
        reps, t_cpu, budget = 0, 0.0, 12.0
        while t_cpu < budget and reps < 2000:
            tc = time.perf_counter()
            ref.forward(xs_host[reps % head["NX"]], threads=cores)
            t_cpu += time.perf_counter() - tc
            reps += 1
        cpu_us = t_cpu * 1e6 / (reps * B)
        t1c = time.perf_counter()
        ref.forward(xs_host[0], threads=1)
        one_us = (time.perf_counter() - t1c) * 1e6 / B
        result["cpu_baseline"] = {"value": round(cpu_us, 1), "unit": "us/token", "cores": cores, "kind": "port",
                                  "sample": "%d forwards of layer 0 (same weights and activations as the GPU run), rows split over %d pthreads "
                                            "per matvec like the reference; 1 thread: %.0f us/token" % (reps, cores, one_us),
                                  "gpu_speedup": round(cpu_us / us_per_token, 1)}
    print(json.dumps(result))
    moe.close()


if __name__ == "__main__":
    main()
