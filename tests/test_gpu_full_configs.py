"""GPU parity at the full size of the two benchmark configurations that the smaller tests only sample:
the 512-token Zipf-routed prefill chunk (512 experts, top-10) and the 48-layer resident mixed-precision stack."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth
from gpu_common import REL_L2_TOL, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

WORKERS = 16


def oracle_tokens_parallel(cfg, lay, x, ids, w):
    """The CPU path token by token (routed experts in selection order in double + the gated shared expert), tokens spread
    over host threads (the C calls release the interpreter lock)."""
    H, F = cfg["hidden"], cfg["ffn"]
    L = orc.lib()
    p = lambda a: a.ctypes.data_as(orc.C.c_void_p)
    out = np.empty((x.shape[0], H), np.float32)

    def one(t):
        routed = np.empty(H, np.float64)
        idt, wt = np.ascontiguousarray(ids[t], np.uint32), np.ascontiguousarray(w[t], np.float32)
        xt = np.ascontiguousarray(x[t])
        assert L.orc_routed_topk(cfg["gate_up_type"], cfg["down_type"], p(lay["gate"]), p(lay["up"]), p(lay["down"]),
                                 lay["gate"][0].nbytes, lay["up"][0].nbytes, lay["down"][0].nbytes, p(idt), p(wt), idt.size, H, F,
                                 p(xt), p(routed))
        sh, s = orc.shared_expert(cfg["sh_gate_up_type"], cfg["sh_down_type"], lay["sh_gate"], lay["sh_up"], lay["sh_down"],
                                  lay["sh_gate_inp"], H, F, xt, threads=1)
        out[t] = (routed + sh.astype(np.float64) * s).astype(np.float32)

    with ThreadPoolExecutor(WORKERS) as ex:
        list(ex.map(one, range(x.shape[0])))
    return out


def test_prefill_chunk_512_tokens_zipf_mixed_layout():
    """The prefill-chunk configuration as written: gate/up IQ2_XXS, down IQ3_S, Q6_K shared expert; hidden 2048, ffn 512, 512 experts,
    top-10 drawn from a Zipf(1.1) popularity, 512 tokens in one call. Every token against the CPU path."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(layout="f2")
    ntok, E, K = 512, cfg["n_expert"], cfg["top_k"]
    lay = synth.make_layer(4004, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    rng = np.random.default_rng(44)
    x = synth.normed_x(rng, ntok, cfg["hidden"])
    ids = synth.zipf_topk(rng, ntok, E, K)
    w = rng.random((ntok, K)).astype(np.float32) + 0.1
    w /= w.sum(axis=1, keepdims=True)
    counts = np.bincount(ids.ravel(), minlength=E)
    # the shape of the load this configuration is about: experts with hundreds of pairs (many tiles of 16, a partial last one),
    # experts with a single pair, experts with none
    assert counts.max() > 256 and (counts == 1).any() and (counts == 0).any() and (counts % 16 != 0).any()
    got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
    want = oracle_tokens_parallel(cfg, lay, x, ids, w)
    worst = max(rel_l2(got[t], want[t]) for t in range(ntok))
    assert worst <= REL_L2_TOL, worst
    # the grouping of the same routing: the host loop's arrays up to the order of the groups
    uid, start, ptok, pw, tp = m.group(torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda())
    cuid, cstart, cptok, cpw, ctp = orc.group_pairs(ids, w, E)
    assert np.array_equal(uid.cpu().numpy().astype(np.uint32), cuid) and np.array_equal(start.cpu().numpy().astype(np.uint32), cstart)
    assert np.array_equal(ptok.cpu().numpy().astype(np.uint32), cptok) and np.array_equal(tp.cpu().numpy().astype(np.uint32), ctp)
    assert np.array_equal(pw.cpu().numpy(), cpw)
    m.close()


@pytest.mark.parametrize("layout", ["iq2", "f2"])
def test_prefill_chunk_2048_tokens(layout):
    """The largest chunk the reference's prefill hands over (B <= 2048, native/redmetal_engine_prefill.m:1246-1277) at the benchmark shape:
    20,480 pairs, sorted block by block of 512 tokens, about 40 pairs per expert (runs of 32 and remainders). 192 tokens - the first and
    last of every block of 512 and a random draw - against the CPU path; the grouping against the host sort."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(layout=layout)
    ntok, E, K = 2048, cfg["n_expert"], cfg["top_k"]
    lay = synth.make_layer(4010, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    rng = np.random.default_rng(45)
    x = synth.normed_x(rng, ntok, cfg["hidden"])
    ids = synth.zipf_topk(rng, ntok, E, K) if layout == "f2" else np.stack([rng.permutation(E)[:K] for _ in range(ntok)]).astype(np.uint32)
    w = rng.random((ntok, K)).astype(np.float32) + 0.1
    w /= w.sum(axis=1, keepdims=True)
    got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
    pick = sorted(set([0, 511, 512, 1023, 1024, 1535, 1536, 2047]) | set(rng.choice(ntok, 184, replace=False).tolist()))
    want = oracle_tokens_parallel(cfg, lay, x[pick], ids[pick], w[pick])
    worst = max(rel_l2(got[t], want[i]) for i, t in enumerate(pick))
    assert worst <= REL_L2_TOL, worst
    uid, start, ptok, pw, tp = m.group(torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda())
    cuid, cstart, cptok, cpw, ctp = orc.group_pairs(ids, w, E)
    assert np.array_equal(uid.cpu().numpy().astype(np.uint32), cuid) and np.array_equal(start.cpu().numpy().astype(np.uint32), cstart)
    assert np.array_equal(ptok.cpu().numpy().astype(np.uint32), cptok) and np.array_equal(tp.cpu().numpy().astype(np.uint32), ctp)
    assert np.array_equal(pw.cpu().numpy(), cpw)
    # ... and through the layer's own router: ids as the CPU path selects them on a sample of the tokens
    out = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
    gids, gw, _ = m.last_route(ntok)
    ref = orc.Layer(cfg, **lay)
    for t in pick[:24]:
        cw_out, cids, cw, _ = ref.forward(x[t][None], threads=8)
        if np.array_equal(gids[t], cids[0]):               # (a near tie in the logits may order two experts differently)
            assert rel_l2(out[t], cw_out[0]) <= REL_L2_TOL, t
        else:
            assert sorted(gids[t].tolist()) == sorted(cids[0].tolist()) or len(set(gids[t].tolist()) ^ set(cids[0].tolist())) <= 2, t
    m.close()


def test_prefill_chunk_512_tokens_own_router_packed_layout():
    """512 tokens through forward() on the all-IQ2_XXS layer: the layer's own F32 router on every token (ids as the CPU path selects
    them), selection, grouping, tiles, combine."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_layer import ids_match_up_to_ties
    cfg = synth.layer_config(layout="iq2")
    ntok = 512
    lay = synth.make_layer(4005, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    rng = np.random.default_rng(45)
    x = synth.normed_x(rng, ntok, cfg["hidden"])
    x[300] = x[17]                                          # two requests with the same row
    got = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
    gids, gw, glog = m.last_route(ntok)
    # CPU routing of every token, then the CPU experts behind the CPU routing
    cids = np.empty_like(gids)
    cw = np.empty_like(gw)
    clog = np.empty_like(glog)
    for t in range(ntok):
        clog[t] = orc.router_logits(cfg["router_type"], lay["router"], cfg["hidden"], cfg["n_expert"], x[t])
        cids[t], cw[t] = orc.router_select(clog[t], cfg["top_k"])
    assert all(ids_match_up_to_ties(gids[t], cids[t], clog[t]) for t in range(ntok))
    same = [t for t in range(ntok) if np.array_equal(gids[t], cids[t])]
    assert len(same) >= ntok - 2                            # (a tie within 1e-6 may swap two ids; none expected)
    assert np.abs(gw[same] - cw[same]).max() <= 1e-5
    want = oracle_tokens_parallel(cfg, lay, x, gids, gw)     # experts behind the routing the GPU used (identical where `same`)
    worst = max(rel_l2(got[t], want[t]) for t in range(ntok))
    assert worst <= REL_L2_TOL, worst
    assert np.array_equal(got[300], got[17])
    m.close()


def test_resident_stack_48_layers_mixed_layout():
    """The 48-layer resident stack of the mixed-precision layout at full shape (24 GB of GGUF bytes plus the packed, word-packed and
    f32 copies), weights drawn on the GPU: one token through layers 0, 23 and 47 against the CPU path on the same bytes."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_layer import ids_match_up_to_ties
    cfg = synth.layer_config(layout="f2")
    NL, check = 48, (0, 23, 47)
    m = ResidentMoe(cfg, n_layer=NL, max_tokens=8)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4848)
    host = {}
    for l in range(NL):
        a = synth.make_layer_gpu(torch, gen, cfg)
        m.load_layer(l, a)
        if l in check:
            host[l] = synth.layer_to_host(a, cfg)
        del a
    torch.cuda.synchronize()
    assert m.resident_bytes > 48 * 512 * 991232             # at least the GGUF bytes of the routed experts
    xs = synth.normed_x(np.random.default_rng(48), 4, cfg["hidden"])
    for l in check:
        ref = orc.Layer(cfg, **host[l])
        # the resident copies of this layer decode to the bytes that were uploaded for it (and not for a neighbour)
        for e, which in ((0, 0), (511, 1), (257, 2), (512, 0), (512, 2)):
            key = ("sh_" if e == 512 else "") + ("gate", "up", "down")[which]
            raw = host[l][key] if e == 512 else host[l][key][e]
            t = cfg[("sh_" if e == 512 else "") + ("gate_up_type" if which < 2 else "down_type")]
            want = orc.dequant_rows(t, raw.reshape(-1), cfg["hidden"] if which < 2 else cfg["ffn"])
            got = m.dequant_resident(l, e, which).cpu().numpy()
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (l, e, which)
        out = m.forward(l, torch.from_numpy(xs[:1]).cuda()).cpu().numpy()[0]
        gids, gw, glog = m.last_route(1)
        want, cids, cw, clog = ref.forward(xs[0], threads=WORKERS)
        assert ids_match_up_to_ties(gids[0], cids[0], clog[0]), l
        assert rel_l2(out, want[0]) <= REL_L2_TOL, l
    # a batch of four on the last layer (the grouped kernels index the same strides)
    out = m.forward(47, torch.from_numpy(xs).cuda()).cpu().numpy()
    want, cids, cw, clog = orc.Layer(cfg, **host[47]).forward(xs, threads=WORKERS)
    gids, _, _ = m.last_route(4)
    assert np.array_equal(gids, cids)
    for t in range(4):
        assert rel_l2(out[t], want[t]) <= REL_L2_TOL, t
    m.close()
