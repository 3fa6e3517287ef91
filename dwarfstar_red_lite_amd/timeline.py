"""Phase table of the expert-slice kernels from their in-kernel stamps (a library built with `python dwarfstar_red_lite_amd/build.py
--timeline`, loaded through REDHIP_LIBRARY). Runs a few steps of one workload over several resident layers (weights from HBM), then
reads the stamps the last expert launch left: per phase the time since the previous stamp of the same workgroup, and when the
workgroups started and ended relative to the first one (the dispatch rounds of the grid).

    REDHIP_LIBRARY=dwarfstar_red_lite_amd/libredmetal_hip_timeline.so python -m dwarfstar_red_lite_amd.timeline --batch 8 --routing hot
"""
import argparse
import ctypes as C
import os
import sys

import numpy as np

PHASES_BATCH = ["entry -> pass entry read", "-> weights requested, tables written", "-> table barrier", "-> gate/up of wave 0 multiplied",
                "-> barrier (every wave)", "-> SwiGLU + barrier", "-> down slice multiplied, stores issued"]
PHASES_ONE = ["entry -> selection + tables (barrier)", "-> weights requested", "-> first unit arrived and multiplied", "-> gate/up of wave 0 multiplied",
              "-> barrier (every wave)", "-> SwiGLU + barrier", "-> down slice multiplied, stores issued"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layout", default="iq2", choices=["iq2", "f2"])
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--routing", default="router", choices=["router", "hot"])
    ap.add_argument("--layers", type=int, default=8)
    ap.add_argument("--steps", type=int, default=24)
    args = ap.parse_args()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for p in (root, os.path.join(root, "oracle")):
        if p not in sys.path:
            sys.path.insert(0, p)
    import torch

    from dwarfstar_red_lite_amd import load, synth
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    lib = load()
    cfg = synth.layer_config(layout=args.layout)
    B, NL = args.batch, args.layers
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    m = ResidentMoe(cfg, n_layer=NL, max_tokens=max(B, 1))
    for l in range(NL):
        m.load_layer(l, synth.make_layer_gpu(torch, gen, cfg))
    rng = np.random.default_rng(3)
    NX = 16
    xs = torch.from_numpy(synth.normed_x(rng, NX * B, cfg["hidden"]).reshape(NX, B, -1)).cuda()
    out = torch.empty_like(xs[0])
    ids = w = None
    if args.routing == "hot":
        import oracle_lib as orc
        ids_h = np.empty((NX, B, cfg["top_k"]), np.uint32)
        w_h = np.empty((NX, B, cfg["top_k"]), np.float32)
        for i in range(NX):
            lg = synth.hot_logits(rng, B, cfg["n_expert"])
            for t in range(B):
                ids_h[i, t], w_h[i, t] = orc.router_select(lg[t], cfg["top_k"])
        ids, w = torch.from_numpy(ids_h.astype(np.int32)).cuda(), torch.from_numpy(w_h).cuda()
    for i in range(args.steps):
        if ids is None:
            m.forward(i % NL, xs[i % NX], out)
        else:
            m.experts(i % NL, xs[i % NX], ids[i % NX], w[i % NX], out)
    torch.cuda.synchronize()
    G, S = 2048, 16
    buf = (C.c_uint64 * (G * S))()
    if not lib.redhip_timeline_read(buf, G, 0):
        raise SystemExit("this library holds no phase stamps: build it with build.py --timeline and set REDHIP_LIBRARY")
    t = np.frombuffer(buf, dtype=np.uint64).reshape(G, S).astype(np.int64)
    ran = t[:, 7] > 0                                   # workgroups that reached the last stamp in the last launch that wrote any
    last = t[ran][:, 0].max()
    ran &= t[:, 0] > last - 100000                      # ... within a millisecond of the newest start (older launches had other grids)
    ran &= (np.diff(t[:, :8], axis=1) >= 0).all(axis=1)  # a workgroup that left early this time still shows an older launch's later stamps
    t = t[ran]
    t0 = t[:, 0].min()
    print("workload: layout %s, %d token(s), routing %s; %d workgroups ran all phases; kernel span %.2f us (first start to last end)" % (
        args.layout, B, args.routing, len(t), (t[:, 7].max() - t0) * 0.01))
    names = PHASES_ONE if B == 1 else PHASES_BATCH
    d = (t[:, 1:8] - t[:, 0:7]) * 0.01
    print("| phase | mean us | median | p90 | max |")
    print("|---|---|---|---|---|")
    for k, name in enumerate(names):
        print("| %s | %.2f | %.2f | %.2f | %.2f |" % (name, d[:, k].mean(), np.median(d[:, k]), np.percentile(d[:, k], 90), d[:, k].max()))
    if B == 1 and args.routing == "router" and (t[:, 12] > 0).any():      # the selecting wave's own stamps (workgroups of routed slots)
        sel = t[t[:, 12] > t[:, 0]]
        ds = np.stack([sel[:, 8] - sel[:, 0], sel[:, 9] - sel[:, 8], sel[:, 10] - sel[:, 9], sel[:, 11] - sel[:, 10], sel[:, 12] - sel[:, 11], sel[:, 1] - sel[:, 12]], axis=1) * 0.01
        for k, name in enumerate(["selection: entry -> logits loaded, maximum", "selection: exponentials, denominator", "selection: threshold, candidate count",
                                  "selection: candidates compacted and ranked", "selection: weights", "selection: end -> barrier passed"]):
            print("| %s | %.2f | %.2f | %.2f | %.2f |" % (name, ds[:, k].mean(), np.median(ds[:, k]), np.percentile(ds[:, k], 90), ds[:, k].max()))
    life = (t[:, 7] - t[:, 0]) * 0.01
    start = (t[:, 0] - t0) * 0.01
    print("| workgroup lifetime | %.2f | %.2f | %.2f | %.2f |" % (life.mean(), np.median(life), np.percentile(life, 90), life.max()))
    print("| workgroup start after the first | %.2f | %.2f | %.2f | %.2f |" % (start.mean(), np.median(start), np.percentile(start, 90), start.max()))
    dw, dc = (t[:, 4] - t[:, 3]).sum(), (t[:, 14] - t[:, 13]).sum()
    if dw > 0:
        print("shader clock counter over the gate/up phase: %.0f counts per us of wall clock" % (dc / (dw * 0.01)))
    cus = len(set(t[:, 15].tolist()))
    print("compute units used: %d; workgroups per compute unit: mean %.2f, max %d" % (cus, len(t) / max(cus, 1), np.bincount(np.unique(t[:, 15], return_inverse=True)[1]).max()))
    m.close()


if __name__ == "__main__":
    main()
