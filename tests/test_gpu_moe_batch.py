"""GPU parity of small ragged batches (parallel requests + MTP verify pair) and of a prefill-sized chunk: token->expert
grouping, every distinct expert applied once to all its tokens, weighted combine in selection order. Checked
against the CPU oracle run token by token."""
import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth
from gpu_common import REL_L2_TOL, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def oracle_tokens(cfg, lay, x, ids, w):
    """routed experts with the given routing + gated shared expert, token by token (float32 [ntok, hidden])"""
    H, F = cfg["hidden"], cfg["ffn"]
    L = orc.lib()
    p = lambda a: a.ctypes.data_as(orc.C.c_void_p)
    out = np.empty((x.shape[0], H), np.float32)
    for t in range(x.shape[0]):
        routed = np.empty(H, np.float64)
        idt, wt = np.ascontiguousarray(ids[t], np.uint32), np.ascontiguousarray(w[t], np.float32)
        assert L.orc_routed_topk(cfg["gate_up_type"], cfg["down_type"], p(lay["gate"]), p(lay["up"]), p(lay["down"]),
                                 lay["gate"][0].nbytes, lay["up"][0].nbytes, lay["down"][0].nbytes, p(idt), p(wt), idt.size, H, F,
                                 p(np.ascontiguousarray(x[t])), p(routed))
        sh, s = orc.shared_expert(cfg["sh_gate_up_type"], cfg["sh_down_type"], lay["sh_gate"], lay["sh_up"], lay["sh_down"],
                                  lay["sh_gate_inp"], H, F, x[t], threads=8)
        out[t] = (routed + sh.astype(np.float64) * s).astype(np.float32)
    return out


@pytest.mark.parametrize("layout", ["iq2", "f2", "xs", "m"])
def test_ragged_small_batches_hot_experts(layout, golden_dir):
    """Ragged small batches: 2..8 tokens, logits N(0,1) + 2.0 on 32 hot experts, benchmark layer shape."""
    import json
    import os
    from dwarfstar_red_lite_amd import moe as moe_api
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    if layout in ("xs", "m"):
        g = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
        grids = [np.frombuffer(bytes.fromhex(g[k]), np.int8) for k in ("iq2_xs", "iq1_m")]
        moe_api.set_codebooks(*grids)
        orc.set_codebooks(*grids)
    cfg = synth.layer_config(layout=layout)
    lay = synth.make_layer(77, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=8)
    m.load_layer(0, lay)
    # the column-sliced copies of the routed down matrices that these batches read dequantise bit-exactly
    for e in (0, 311, cfg["n_expert"] - 1):
        want = orc.dequant_rows(cfg["down_type"], lay["down"][e].reshape(-1), cfg["ffn"])
        got = m.dequant_resident(0, e, 4).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (layout, e)
    rng = np.random.default_rng(31)
    for ntok in (1, 2, 3, 8):                                                      # (one token: the caller's routing on the single-token kernels)
        x = synth.normed_x(rng, ntok, cfg["hidden"])
        logits = synth.hot_logits(rng, ntok, cfg["n_expert"])
        sel = [orc.router_select(logits[t], cfg["top_k"]) for t in range(ntok)]
        ids = np.stack([s[0] for s in sel])
        w = np.stack([s[1] for s in sel])
        assert ntok == 1 or len(set(ids.ravel().tolist())) < ntok * cfg["top_k"]            # tokens do share experts
        got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
        want = oracle_tokens(cfg, lay, x, ids, w)
        for t in range(ntok):
            assert rel_l2(got[t], want[t]) <= REL_L2_TOL, (layout, ntok, t)
    # end to end with the layer's own router: every token routed as the CPU path routes it
    x = synth.normed_x(rng, 5, cfg["hidden"])
    x[1] = x[0]                                                                    # the verify pair sees identical rows
    got = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
    gids, gw, glog = m.last_route(5)
    want, cids, cw, clog = orc.Layer(cfg, **lay).forward(x, threads=8)
    assert np.array_equal(gids, cids)
    assert np.array_equal(got[0], got[1])
    for t in range(5):
        assert rel_l2(got[t], want[t]) <= REL_L2_TOL
    # a full batch in which three requests carry the same row: groups of one, two and three pairs, read once each
    x = synth.normed_x(rng, 8, cfg["hidden"])
    x[3] = x[0]
    x[6] = x[0]
    x[7] = x[2]
    got = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
    gids, gw, glog = m.last_route(8)
    want, cids, cw, clog = orc.Layer(cfg, **lay).forward(x, threads=8)
    assert np.array_equal(gids, cids)
    assert np.array_equal(got[0], got[3]) and np.array_equal(got[0], got[6]) and np.array_equal(got[2], got[7])
    for t in range(8):
        assert rel_l2(got[t], want[t]) <= REL_L2_TOL, (layout, t)
    m.close()


@pytest.mark.parametrize("hidden,ffn,ntok", [(512, 256, 96), (1024, 512, 40), (2048, 512, 33), (1024, 768, 24)])
def test_prefill_sized_chunk_zipf(hidden, ffn, ntok):
    """Prefill chunk on the mixed layout: Zipf(1.1) expert popularity, variable token count per expert. Routed gate/up tiles on
    packed IQ2_XXS, routed IQ3_S down tiles, the Q6_K shared expert as dense f32 products; ffn 768 takes the raw-row kernels."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(hidden=hidden, ffn=ffn, n_expert=64, top_k=4, layout="f2")
    lay = synth.make_layer(5, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    rng = np.random.default_rng(8)
    x = synth.normed_x(rng, ntok, hidden)
    ids = synth.zipf_topk(rng, ntok, 64, 4)
    w = rng.random((ntok, 4)).astype(np.float32)
    w /= w.sum(axis=1, keepdims=True)
    counts = np.bincount(ids.ravel(), minlength=64)
    assert counts.max() > 8 and counts.min() < 4          # ragged: some experts busy, some nearly idle
    got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
    want = oracle_tokens(cfg, lay, x, ids, w)
    assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL
    m.close()


@pytest.mark.parametrize("hidden,ffn,ntok", [(1024, 512, 96), (512, 256, 40), (2048, 768, 33)])
def test_prefill_chunk_packed_tiles(hidden, ffn, ntok):
    """Prefill chunk on the packed IQ2_XXS layout (tiles of 16 pairs per expert on the 16x16x16 MFMA): Zipf routing, so
    one expert fills several tiles, others have a single pair, some none; the last tile of a group is partial."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(hidden=hidden, ffn=ffn, n_expert=64, top_k=4, layout="iq2")
    lay = synth.make_layer(6, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    rng = np.random.default_rng(9)
    x = synth.normed_x(rng, ntok, hidden)
    ids = synth.zipf_topk(rng, ntok, 64, 4)
    w = rng.random((ntok, 4)).astype(np.float32)
    w /= w.sum(axis=1, keepdims=True)
    counts = np.bincount(ids.ravel(), minlength=64)
    assert counts.max() > 16 and counts.min() < 4
    got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
    want = oracle_tokens(cfg, lay, x, ids, w)
    assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL
    m.close()


@pytest.mark.parametrize("layout,hidden", [("iq2", 1024), ("f2", 2048)])
def test_prefill_chunk_tile_list_edges(layout, hidden):
    """Experts with exactly 16, 17, 32, 33, 48 and 49 pairs in one chunk: the gate/up tiles are cut into runs of 32 pairs (two sets of 16
    share every decoded weight) with remainders of 17 .. 31 as one more such tile and remainders of 1 .. 16 on the 16-pair kernel; the
    down tiles stay 16 pairs. Every boundary of that split in one call."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    ntok, E, K = 128, 64, 2
    cfg = synth.layer_config(hidden=hidden, ffn=512, n_expert=E, top_k=K, layout=layout)
    lay = synth.make_layer(12, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    order = [0] * 16 + [1] * 17 + [2] * 32 + [3] * 33 + [4] * 48 + [5] * 49
    order += [6 + i % (E - 6) for i in range(ntok * K - len(order))]
    ids = np.stack([order[:ntok], order[ntok:]], axis=1).astype(np.uint32)             # token t: pairs t and t + ntok of the run list
    assert all(ids[t, 0] != ids[t, 1] for t in range(ntok))
    counts = np.bincount(ids.ravel(), minlength=E)
    assert list(counts[:6]) == [16, 17, 32, 33, 48, 49]
    rng = np.random.default_rng(13)
    x = synth.normed_x(rng, ntok, hidden)
    w = rng.random((ntok, K)).astype(np.float32) + 0.1
    w /= w.sum(axis=1, keepdims=True)
    got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
    want = oracle_tokens(cfg, lay, x, ids, w)
    assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL
    m.close()


@pytest.mark.parametrize("layout", ["iq2", "f2", "xs", "m"])
def test_drawn_routing_every_batch_size_class(layout, golden_dir):
    """Seeded routing at every batch size class of the dispatch (one token, small batches, two small batches, chunks), spread over all
    experts or concentrated on top_k of them (every token the same experts: the largest tiles a chunk can have), on every layout:
    caller-given routing and the layer's own router against the CPU path."""
    import json
    import os
    from dwarfstar_red_lite_amd import moe as moe_api
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    if layout in ("xs", "m"):
        g = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
        grids = [np.frombuffer(bytes.fromhex(g[k]), np.int8) for k in ("iq2_xs", "iq1_m")]
        moe_api.set_codebooks(*grids)
        orc.set_codebooks(*grids)
    H, F, E, K = 1024, 256, 24, 6
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout=layout)
    lay = synth.make_layer(21, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=130)
    m.load_layer(0, lay)
    ref = orc.Layer(cfg, **lay)
    rng = np.random.default_rng(22)
    for ntok, hot in ((1, E), (2, K), (7, E), (9, K), (16, 11), (33, K), (130, K), (130, E)):
        x = synth.normed_x(rng, ntok, H)
        ids = np.stack([rng.permutation(hot)[:K] for _ in range(ntok)]).astype(np.uint32)
        w = rng.random((ntok, K)).astype(np.float32) + 0.05
        w /= w.sum(axis=1, keepdims=True)
        got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
        want = oracle_tokens(cfg, lay, x, ids, w)
        assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL, (layout, ntok, hot)
        got = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        gids, _, _ = m.last_route(ntok)
        want, cids, _, _ = ref.forward(x, threads=8)
        agree = [t for t in range(ntok) if np.array_equal(gids[t], cids[t])]             # (a near tie in the logits may order two experts differently)
        assert len(agree) >= ntok - 1
        assert max(rel_l2(got[t], want[t]) for t in agree) <= REL_L2_TOL, (layout, ntok)
    m.close()


@pytest.mark.parametrize("shape,sizes", [((2048, 512, 512, 10), (17, 32, 33)), ((1024, 256, 32, 8), (20, 24, 25, 32)), ((512, 256, 64, 16), (31, 32))])
def test_batches_up_to_32_tokens_behind_the_own_router(shape, sizes):
    """all-IQ2_XXS layers take up to 32 tokens (512 pairs) as one batch of expert slices: through forward() the selection launch sorts the
    pairs and writes the pass list, with the routing given a launch of its own does. Few experts: every expert serves many tokens
    (passes of two pairs); 64 experts x top-16: 512 pairs."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_layer import ids_match_up_to_ties
    H, F, E, K = shape
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout="iq2")
    lay = synth.make_layer(91, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=max(sizes))
    m.load_layer(0, lay)
    ref = orc.Layer(cfg, **lay)
    rng = np.random.default_rng(92)
    for ntok in sizes:
        x = synth.normed_x(rng, ntok, H)
        got = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        gids, gw, _ = m.last_route(ntok)
        want, cids, cw, clog = ref.forward(x, threads=8)
        assert all(ids_match_up_to_ties(gids[t], cids[t], clog[t]) for t in range(ntok)), (shape, ntok)
        assert np.abs(gw - cw).max() <= 1e-5
        assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL, (shape, ntok)
        # the same sizes with the routing given: every token picks among `hot` experts, so an expert serves many tokens of the batch
        hot = min(E, 3 * K)
        ids = np.stack([rng.permutation(hot)[:K] for _ in range(ntok)]).astype(np.uint32)
        w = rng.random((ntok, K)).astype(np.float32) + 0.05
        w /= w.sum(axis=1, keepdims=True)
        got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
        want = oracle_tokens(cfg, lay, x, ids, w)
        assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL, (shape, ntok, "given")
    m.close()


@pytest.mark.parametrize("layout", ["f2", "xs", "m"])
@pytest.mark.parametrize("shape,sizes", [((2048, 512, 512, 10), (17, 32)), ((1024, 256, 32, 8), (9, 16, 24, 25, 31, 33))])
def test_mixed_layout_batches_up_to_32_tokens_behind_the_own_router(layout, shape, sizes, golden_dir):
    """the mixed layouts whose small batches run as expert slices take 9..32 tokens through forward() as one batch: the router launch of the
    eight-token batches once per eight tokens, one selection + pair sort launch, slices per pass"""
    import json
    import os
    from dwarfstar_red_lite_amd import moe as moe_api
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_layer import ids_match_up_to_ties
    if layout in ("xs", "m"):
        g = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
        grids = [np.frombuffer(bytes.fromhex(g[k]), np.int8) for k in ("iq2_xs", "iq1_m")]
        moe_api.set_codebooks(*grids)
        orc.set_codebooks(*grids)
    H, F, E, K = shape
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout=layout)
    lay = synth.make_layer(93, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=max(sizes))
    m.load_layer(0, lay)
    ref = orc.Layer(cfg, **lay)
    rng = np.random.default_rng(94)
    for ntok in sizes:
        x = synth.normed_x(rng, ntok, H)
        got = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        gids, gw, _ = m.last_route(ntok)
        want, cids, cw, clog = ref.forward(x, threads=8)
        assert all(ids_match_up_to_ties(gids[t], cids[t], clog[t]) for t in range(ntok)), (layout, shape, ntok)
        agree = [t for t in range(ntok) if np.array_equal(gids[t], cids[t])]
        assert len(agree) >= ntok - 1
        assert max(rel_l2(got[t], want[t]) for t in agree) <= REL_L2_TOL, (layout, shape, ntok)
        # the same sizes with the routing given (up to 24 tokens as slices, behind a pair sort launch of its own): few experts, shared by many tokens
        hot = min(E, 3 * K)
        ids = np.stack([rng.permutation(hot)[:K] for _ in range(ntok)]).astype(np.uint32)
        w = rng.random((ntok, K)).astype(np.float32) + 0.05
        w /= w.sum(axis=1, keepdims=True)
        got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
        want = oracle_tokens(cfg, lay, x, ids, w)
        assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL, (layout, shape, ntok, "given")
    m.close()


@pytest.mark.parametrize("layout", ["iq2", "f2"])
def test_prefill_chunk_forward_config_shape(layout):
    """A 24-token chunk at the benchmark shape through forward(): router (tiled, a Q6_K router through its f32 copy), selection, grouping,
    tiles, combine."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(layout=layout)
    lay = synth.make_layer(78, cfg)
    ntok = 24
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    x = synth.normed_x(np.random.default_rng(32), ntok, cfg["hidden"])
    got = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
    gids, gw, _ = m.last_route(ntok)
    want, cids, cw, clog = orc.Layer(cfg, **lay).forward(x, threads=8)
    from test_gpu_moe_layer import ids_match_up_to_ties
    assert all(ids_match_up_to_ties(gids[t], cids[t], clog[t]) for t in range(ntok))
    assert np.abs(gw - cw).max() <= 1e-5
    assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL
    m.close()


@pytest.mark.parametrize("down_type", [synth.TYPE_Q6_K, synth.TYPE_IQ2_XXS])
def test_mixed_layout_raw_down_rows(down_type):
    """mixed layers whose routed down matrices have no packed copy (Q6_K, or IQ2_XXS beside a Q6_K shared expert): the raw-row down
    kernels for one token, a pair, grouped batches and a chunk"""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(hidden=1024, ffn=512, n_expert=32, top_k=6, layout="f2")
    cfg["down_type"] = down_type
    lay = synth.make_layer(911, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=20)
    m.load_layer(0, lay)
    ref = orc.Layer(cfg, **lay)
    xs = synth.normed_x(np.random.default_rng(3), 20, cfg["hidden"])
    xs[6] = xs[2]
    for ntok in (1, 2, 5, 8, 20):
        out = m.forward(0, torch.from_numpy(xs[:ntok].copy()).cuda()).cpu().numpy()
        gids, gw, glog = m.last_route(ntok)
        want, cids, cw, clog = ref.forward(xs[:ntok], threads=8)
        assert np.array_equal(gids, cids)
        for i in range(ntok):
            assert rel_l2(out[i], want[i]) <= REL_L2_TOL, (down_type, ntok, i)
        if ntok >= 8:
            assert np.array_equal(out[6], out[2])
    m.close()


def test_chunk_as_slices_of_small_batches():
    """a layout without tile kernels (ffn 768): forward() of 20 tokens runs as slices of 8 on the grouped small-batch kernels, the route
    of every token at its place in the chunk"""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(hidden=1024, ffn=768, n_expert=24, top_k=12, layout="f2")
    lay = synth.make_layer(505, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=20)
    m.load_layer(0, lay)
    xs = synth.normed_x(np.random.default_rng(9), 20, cfg["hidden"])
    out = m.forward(0, torch.from_numpy(xs).cuda()).cpu().numpy()
    gids, gw, glog = m.last_route(20)
    want, cids, cw, clog = orc.Layer(cfg, **lay).forward(xs, threads=8)
    assert np.array_equal(gids, cids)
    assert np.all(np.abs(gw - cw) <= 1e-6 + 1e-5 * cw)
    for i in range(20):
        assert rel_l2(out[i], want[i]) <= REL_L2_TOL, i
    m.close()

