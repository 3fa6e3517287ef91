"""GPU parity of the two formats that decode through caller-supplied codebooks, IQ2_XS (type 17) and IQ1_M (type 29), on the
surfaces that accept them: the dequantisation / GEMV taps, redmetal_quant_rows and the single-expert pool. The codebooks are the
reference's own tables (golden fixture), handed over the way the reference hands them."""
import json
import os
import struct

import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import expert_type_word, synth
from gpu_common import REL_L2_TOL, T_IQ2, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

T_XS, T_M = 17, 29


def dev(a):
    return torch.from_numpy(np.array(a, copy=True)).cuda()


@pytest.fixture(scope="module")
def grids(golden_dir):
    from dwarfstar_red_lite_amd import moe
    g = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
    xs = np.frombuffer(bytes.fromhex(g["iq2_xs"]), np.int8)
    m = np.frombuffer(bytes.fromhex(g["iq1_m"]), np.int8)
    moe.set_codebooks(xs, m)
    return xs, m


def edge_rows(t, ncols):
    """all-zero, all-one and extreme-scale blocks beside seeded ones"""
    rng = np.random.default_rng(4321 + t)
    rows = synth.quant_rows(rng, t, 6, ncols)
    bb = synth.BLOCK_BYTES[t]
    r = rows.reshape(6, -1, bb)
    r[1] = 0
    r[2] = 0xFF                  # every index, sign and scale bit set; d = NaN pattern for IQ2_XS is avoided below
    if t == T_XS:
        r[2, :, 0], r[2, :, 1] = 0x00, 0x3C          # d = 1
        r[3, :, 0], r[3, :, 1] = 0x01, 0x00          # smallest subnormal d
        r[4, :, 1] |= 0x80                           # negative d
        r[5, :, 0], r[5, :, 1] = 0xFF, 0x7B          # 65504
    else:
        for i, nib in enumerate((0x0, 0x0, 0xC, 0x3)):          # d = 1.0 spread over the four top nibbles
            r[2, :, 49 + 2 * i] = (r[2, :, 49 + 2 * i] & 0x0F) | (nib << 4)
        r[3, :, 49::2] &= 0x0F                        # d = 0
        r[3, :, 49] |= 0x10                           # ... then the smallest subnormal
        r[4, :, 55] |= 0x80                           # negative d
        for i, nib in enumerate((0xF, 0xF, 0xB, 0x7)):          # 65504
            r[5, :, 49 + 2 * i] = (r[5, :, 49 + 2 * i] & 0x0F) | (nib << 4)
    return rows


@pytest.mark.parametrize("t", [T_XS, T_M])
def test_dequant_bit_exact(t, grids):
    from dwarfstar_red_lite_amd import moe
    grid = grids[0] if t == T_XS else grids[1]
    rng = np.random.default_rng(300 + t)
    for ncols in (256, 512, 2048):
        rows = np.concatenate([synth.quant_rows(rng, t, 37, ncols), edge_rows(t, ncols)])
        got = moe.dequant_rows(t, dev(rows), ncols).cpu().numpy()
        want = orc.dequant_rows_grid(t, rows, ncols, grid)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (t, ncols)


def test_golden_rows(golden_dir, grids):
    """the rows the compiled reference was run on: dequantisation against the oracle, the dot against the reference's own"""
    from dwarfstar_red_lite_amd import moe
    g = json.load(open(os.path.join(golden_dir, "quant_rows_xs_m.json")))
    for c in g["cases"]:
        t, n = c["type"], c["ncols"]
        row = np.frombuffer(bytes.fromhex(c["row"]), np.uint8).reshape(1, -1)
        x = np.frombuffer(bytes.fromhex(c["x"]), np.float32)
        want = struct.unpack("<d", bytes.fromhex(c["dot"]))[0]
        w = orc.dequant_rows_grid(t, row, n, grids[0] if t == T_XS else grids[1])
        got_w = moe.dequant_rows(t, dev(row), n).cpu().numpy()
        assert np.array_equal(got_w.view(np.uint32), w.view(np.uint32)), (t, n, c["fill"])
        got = float(moe.gemv_rows(t, dev(row), n, dev(x)).cpu().numpy()[0])
        scale = float(np.abs(w.astype(np.float64) * x).sum())
        assert abs(got - want) <= 2e-5 * scale + 1e-30, (t, n, c["fill"], got, want)


@pytest.mark.parametrize("t", [T_XS, T_M])
def test_gemv_rows(t, grids):
    from dwarfstar_red_lite_amd import moe
    grid = grids[0] if t == T_XS else grids[1]
    rng = np.random.default_rng(400 + t)
    for ncols in (256, 512, 1024, 2048):
        nrows = 37
        w = synth.quant_rows(rng, t, nrows, ncols)
        x = rng.standard_normal(ncols).astype(np.float32)
        want = np.array([orc.row_dot_grid(t, w[r], x, grid) for r in range(nrows)])
        got = moe.gemv_rows(t, dev(w), ncols, dev(x)).cpu().numpy()
        scale = np.abs(orc.dequant_rows_grid(t, w, ncols, grid).astype(np.float64) * x).sum(axis=1)
        assert np.max(np.abs(got - want) / scale) <= 2e-5, (t, ncols)
        assert rel_l2(got, want) <= REL_L2_TOL
        part = moe.gemv_rows(t, dev(w), ncols, dev(x), row_start=5, row_count=9).cpu().numpy()
        assert np.array_equal(part, got[5:14])


@pytest.fixture(scope="module")
def model_file(tmp_path_factory):
    H, F = 512, 256
    rng = np.random.default_rng(78)
    parts, off, index = [np.zeros(10, np.uint8)], 10, {}
    for fam, gu, dn in (("xs", T_XS, T_XS), ("m", T_M, T_M), ("m_xs", T_M, T_XS), ("xs_iq2", T_XS, T_IQ2)):
        for name, t, nr, nc in (("gate", gu, F, H), ("up", gu, F, H), ("down", dn, H, F)):
            b = synth.quant_rows(rng, t, nr, nc).ravel()
            index[fam + "." + name] = (off, b.size)
            parts.append(b)
            off += b.size
    blob = np.concatenate(parts)
    path = tmp_path_factory.mktemp("model_xs_m") / "raw_blocks.bin"
    blob.tofile(path)
    return str(path), blob, index, H, F


def test_quant_rows(model_file, grids):
    from dwarfstar_red_lite_amd import RedHipError
    from dwarfstar_red_lite_amd.redmetal_quant import RedMetalQuantBridge
    path, blob, index, H, F = model_file
    br = RedMetalQuantBridge()
    x = synth.normed_x(np.random.default_rng(5), 1, H)[0]
    for name, t, ncols, nrows, grid in (("xs.gate", T_XS, H, F, grids[0]), ("m.down", T_M, F, H, grids[1])):
        off, n = index[name]
        xin = x[:ncols]
        out, _, _ = br.rows(path, off, n, t, ncols, nrows, 3, 11, xin, grid=grid)
        w = blob[off:off + n].reshape(nrows, -1)
        want = np.array([orc.row_dot_grid(t, w[r], xin, grid) for r in range(3, 14)])
        assert rel_l2(out, want) <= REL_L2_TOL, name
        with pytest.raises(RedHipError, match="grid size mismatch"):
            br.rows(path, off, n, t, ncols, nrows, 0, 1, xin)
        with pytest.raises(RedHipError, match="grid size mismatch"):
            br.rows(path, off, n, t, ncols, nrows, 0, 1, xin, grid=grid[:-8])


def test_ffn_pool(model_file, grids):
    from dwarfstar_red_lite_amd.redmetal_ffn import ExpertLayout, RedMetalFfnPool
    path, blob, index, H, F = model_file
    xs, m = grids
    x = synth.normed_x(np.random.default_rng(6), 1, H)[0]
    slot_bytes = max(sum(index[f + "." + n][1] for n in ("gate", "up", "down")) for f in ("xs", "m", "m_xs", "xs_iq2"))
    sl = lambda o, n: blob[o:o + n]
    with RedMetalFfnPool(path, 8 * (slot_bytes + 4096), slot_bytes, iq2_xs_grid=xs, iq1_m_grid=m) as pool:
        for slot, (fam, gu, dn) in enumerate((("xs", T_XS, T_XS), ("m", T_M, T_M), ("m_xs", T_M, T_XS), ("xs_iq2", T_XS, T_IQ2))):
            lay = ExpertLayout(*index[fam + ".gate"], *index[fam + ".up"], *index[fam + ".down"])
            pool.load(slot, lay)
            want = orc.expert_ffn_grid(gu, dn, sl(lay.gate_offset, lay.gate_bytes), sl(lay.up_offset, lay.up_bytes),
                                       sl(lay.down_offset, lay.down_bytes), H, F, x, xs, m)
            out, _ = pool.execute(slot, lay, expert_type_word(gu, dn), H, F, 0, H, x)
            assert rel_l2(out, want) <= REL_L2_TOL, fam
            win, _ = pool.execute(slot, lay, expert_type_word(gu, dn), H, F, 500, 12, x)
            assert np.array_equal(win, out[500:])
    # a pool made without codebooks serves the other formats and says so for these two
    with RedMetalFfnPool(path, 2 * (slot_bytes + 4096), slot_bytes) as pool:
        lay = ExpertLayout(*index["xs.gate"], *index["xs.up"], *index["xs.down"])
        pool.load(0, lay)
        with pytest.raises(ValueError, match="need the pool created with"):
            pool.execute(0, lay, T_XS, H, F, 0, H, x)

def test_pools_with_different_codebooks_do_not_decode_through_each_others_tables(model_file, grids):
    """the process holds one device copy of the two codebooks: while a pool that has run an IQ2_XS expert is alive, a pool (or a one-shot
    GEMV) that brings other tables is refused with a message; once the first pool is gone the second one runs on its own tables"""
    from dwarfstar_red_lite_amd import moe
    from dwarfstar_red_lite_amd._lib import RedHipError
    from dwarfstar_red_lite_amd.redmetal_ffn import ExpertLayout, RedMetalFfnPool
    from dwarfstar_red_lite_amd.redmetal_quant import RedMetalQuantBridge
    path, blob, index, H, F = model_file
    xs, m = grids
    xs2 = np.roll(xs.reshape(512, 8), 1, axis=0).copy().reshape(-1)          # the same entries under other indices
    x = synth.normed_x(np.random.default_rng(16), 1, H)[0]
    slot_bytes = sum(index["xs." + n][1] for n in ("gate", "up", "down"))
    lay = ExpertLayout(*index["xs.gate"], *index["xs.up"], *index["xs.down"])
    sl = lambda o, n: blob[o:o + n]
    want = {id(g): orc.expert_ffn_grid(T_XS, T_XS, sl(lay.gate_offset, lay.gate_bytes), sl(lay.up_offset, lay.up_bytes),
                                       sl(lay.down_offset, lay.down_bytes), H, F, x, g, m) for g in (xs, xs2)}
    first = RedMetalFfnPool(path, 2 * (slot_bytes + 4096), slot_bytes, iq2_xs_grid=xs, iq1_m_grid=m)
    second = RedMetalFfnPool(path, 2 * (slot_bytes + 4096), slot_bytes, iq2_xs_grid=xs2, iq1_m_grid=m)
    try:
        first.load(0, lay)
        second.load(0, lay)
        out, _ = first.execute(0, lay, T_XS, H, F, 0, H, x)
        assert rel_l2(out, want[id(xs)]) <= REL_L2_TOL
        with pytest.raises(RedHipError, match="codebooks differ"):
            second.execute(0, lay, T_XS, H, F, 0, H, x)
        off, n = index["xs.gate"]
        with pytest.raises(RedHipError, match="codebooks differ"):
            RedMetalQuantBridge().rows(path, off, n, T_XS, H, F, 0, 4, x, grid=xs2)
        out, _ = first.execute(0, lay, T_XS, H, F, 0, H, x)                   # the bound pool is unaffected
        assert rel_l2(out, want[id(xs)]) <= REL_L2_TOL
        first.close()
        out2, _ = second.execute(0, lay, T_XS, H, F, 0, H, x)
        assert rel_l2(out2, want[id(xs2)]) <= REL_L2_TOL
        assert rel_l2(out2, want[id(xs)]) > 10 * REL_L2_TOL                   # (the two tables do decode differently)
    finally:
        first.close()
        second.close()
    moe.set_codebooks(xs, m)                                                  # what the tests after this one expect on the device


@pytest.mark.parametrize("layout", ["xs", "m"])
@pytest.mark.parametrize("shape", [(512, 256, 16, 4), (2048, 512, 64, 10)])
def test_resident_layer(layout, shape, grids):
    """the resident layer with IQ2_XS / IQ1_M routed experts (what the reference's target file holds): one token, a ragged small
    batch and a chunk, against the oracle's layer forward"""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_layer import ids_match_up_to_ties
    orc.set_codebooks(*grids)
    H, F, E, K = shape
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout=layout)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=24)
    lay = synth.make_layer(60 + H, cfg)
    m.load_layer(0, lay)
    ref = orc.Layer(cfg, **lay)
    t = cfg["gate_up_type"]
    for e, which in ((0, 0), (E - 1, 1), (E // 2, 2)):
        want = orc.dequant_rows(t, lay[("gate", "up", "down")[which]][e].reshape(-1), H if which < 2 else F)
        got = m.dequant_resident(0, e, which).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    xs = synth.normed_x(np.random.default_rng(8), 24, H)
    for ntok in (1, 5, 24):
        out = m.forward(0, torch.from_numpy(xs[:ntok].copy()).cuda()).cpu().numpy()
        gids, gw, glog = m.last_route(ntok)
        want, cids, cw, clog = ref.forward(xs[:ntok], threads=8)
        for i in range(ntok):
            assert ids_match_up_to_ties(gids[i], cids[i], clog[i])
            assert rel_l2(out[i], want[i]) <= REL_L2_TOL, (layout, shape, ntok, i)
    m.close()


@pytest.mark.parametrize("layout", ["f2", "xs", "m"])
@pytest.mark.parametrize("shape", [(1024, 768, 24, 12), (4096, 1024, 16, 2), (2048, 1024, 16, 4), (512, 256, 16, 4), (512, 256, 4, 1), (1024, 256, 2, 2)])
def test_mixed_layouts_other_shapes(layout, shape, grids):
    """mixed-precision layers away from the benchmark shape: 13 slots (the 16-wave kernels), ffn 768 / 1024 (two column chunks per
    lane), hidden 512 .. 4096; one token, a pair, grouped batches, with dequantisation from the copies the kernels read"""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_layer import ids_match_up_to_ties
    orc.set_codebooks(*grids)
    H, F, E, K = shape
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout=layout)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=8)
    lay = synth.make_layer(90 + H + F, cfg)
    m.load_layer(0, lay)
    ref = orc.Layer(cfg, **lay)
    for e, which in ((1, 0), (E - 1, 1), (E // 2, 2), (0, 2)):
        t = cfg["gate_up_type" if which < 2 else "down_type"]
        want = orc.dequant_rows(t, lay[("gate", "up", "down")[which]][e].reshape(-1), H if which < 2 else F)
        got = m.dequant_resident(0, e, which).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (layout, shape, e, which)
    xs = synth.normed_x(np.random.default_rng(17), 8, H)
    xs[5] = xs[1]                                        # two requests with the same row: groups of two pairs
    for ntok in (1, 2, 5, 8):
        out = m.forward(0, torch.from_numpy(xs[:ntok].copy()).cuda()).cpu().numpy()
        gids, gw, glog = m.last_route(ntok)
        want, cids, cw, clog = ref.forward(xs[:ntok], threads=8)
        for i in range(ntok):
            assert ids_match_up_to_ties(gids[i], cids[i], clog[i])
            assert rel_l2(out[i], want[i]) <= REL_L2_TOL, (layout, shape, ntok, i)
        if ntok == 8:
            assert np.array_equal(out[5], out[1])
    m.close()


@pytest.mark.parametrize("layout", ["xs", "m"])
@pytest.mark.parametrize("shape,ntok", [((1024, 512, 16, 4), 48), ((512, 256, 16, 4), 33)])
def test_codebook_layout_chunks(layout, shape, ntok, grids):
    """prefill chunks on IQ2_XS / IQ1_M layers (tile kernels on the row-major streams): experts with several tiles (twenty requests carry
    the same row), partial last tiles, experts nobody selected"""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_layer import ids_match_up_to_ties
    orc.set_codebooks(*grids)
    H, F, E, K = shape
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout=layout)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    lay = synth.make_layer(7 + H, cfg)
    m.load_layer(0, lay)
    xs = synth.normed_x(np.random.default_rng(23), ntok, H)
    xs[5:25] = xs[4]
    out = m.forward(0, torch.from_numpy(xs).cuda()).cpu().numpy()
    gids, gw, glog = m.last_route(ntok)
    want, cids, cw, clog = orc.Layer(cfg, **lay).forward(xs, threads=8)
    for i in range(ntok):
        assert ids_match_up_to_ties(gids[i], cids[i], clog[i])
        assert rel_l2(out[i], want[i]) <= REL_L2_TOL, (layout, shape, i)
    assert np.array_equal(out[7], out[4])
    m.close()


@pytest.mark.parametrize("layout", ["xs", "m"])
def test_codebook_layout_given_routing(layout, grids):
    """caller-given routing (drawn logits with hot experts, so tokens share experts) on IQ2_XS / IQ1_M layers: one token (single-token kernels), batches of 2, 3
    and 8 (grouped kernels, the pair sort riding in the shared gate/up launch) and a chunk of 40 tokens, against the oracle run token by token"""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_batch import oracle_tokens
    orc.set_codebooks(*grids)
    cfg = synth.layer_config(hidden=1024, ffn=512, n_expert=64, top_k=6, layout=layout)
    lay = synth.make_layer(321, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=40)
    m.load_layer(0, lay)
    rng = np.random.default_rng(77)
    for ntok in (1, 2, 3, 8, 40):
        x = synth.normed_x(rng, ntok, cfg["hidden"])
        logits = synth.hot_logits(rng, ntok, cfg["n_expert"])
        sel = [orc.router_select(logits[t], cfg["top_k"]) for t in range(ntok)]
        ids = np.stack([s[0] for s in sel])
        w = np.stack([s[1] for s in sel])
        got = m.experts(0, torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
        want = oracle_tokens(cfg, lay, x, ids, w)
        for t in range(ntok):
            assert rel_l2(got[t], want[t]) <= REL_L2_TOL, (layout, ntok, t)
    m.close()


@pytest.mark.parametrize("layout", ["f2", "xs"])
def test_chunk_in_a_graph_with_the_shared_expert_on_its_own_stream(layout, grids):
    """A chunk on a mixed layout forks the shared expert's dense products onto a second stream and joins them before the combine.
    Captured into a HIP graph (two layers, so that a fork follows a join) and replayed with new inputs, eager work and
    synchronisations in between: every replay must equal the eager result bit for bit, and the eager result the oracle."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    orc.set_codebooks(*grids)
    cfg = synth.layer_config(hidden=1024, ffn=512, n_expert=32, top_k=6, layout=layout)
    lays = [synth.make_layer(900 + i, cfg) for i in range(2)]
    ntok = 40
    m = ResidentMoe(cfg, n_layer=2, max_tokens=ntok)
    for i, lay in enumerate(lays):
        m.load_layer(i, lay)
    rng = np.random.default_rng(5)
    xs = [synth.normed_x(rng, ntok, cfg["hidden"]) for _ in range(3)]
    x_dev = torch.empty((ntok, cfg["hidden"]), dtype=torch.float32, device="cuda")
    mid = torch.empty_like(x_dev)
    out = torch.empty_like(x_dev)

    def two_layers():
        m.forward(0, x_dev, out=mid)
        m.forward(1, mid, out=out)

    eager = []
    for x in xs:
        x_dev.copy_(torch.from_numpy(x))
        two_layers()
        torch.cuda.synchronize()
        eager.append((mid.clone(), out.clone()))
    want0, *_ = orc.Layer(cfg, **lays[0]).forward(xs[0], threads=8)
    for t in range(ntok):
        assert rel_l2(eager[0][0][t].cpu().numpy(), want0[t]) <= REL_L2_TOL, (layout, t)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        two_layers()                                # warm-up on the capture stream
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=stream):
        two_layers()
    for rnd in range(2):
        for x, (e_mid, e_out) in zip(xs, eager):
            x_dev.copy_(torch.from_numpy(x))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(mid, e_mid) and torch.equal(out, e_out), (layout, rnd)
            two_layers()                            # the program's own eager work between replays
            torch.cuda.synchronize()
            assert torch.equal(out, e_out), (layout, rnd)
    m.close()
