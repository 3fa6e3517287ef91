"""The resident top-k expert pool (redmetal_topk_*) through the C ABI against the CPU path: experts are read from a GGUF file into
slots at the byte ranges the file's directory gives, then the weighted top-k FFN runs over slot lists - host arrays (execute),
stream-ordered with host lists (encode, encode_batched, encode_mapped) and with the slot table and weights read on the device
(encode_device_into / _into2 / _tail). Expected values: the CPU path's expert FFN in double, summed in list order."""
import json
import os

import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth
from dwarfstar_red_lite_amd._lib import RedHipError
from dwarfstar_red_lite_amd.gguf_writer import write_moe_gguf
from gpu_common import REL_L2_TOL, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def grids(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
    xs = np.frombuffer(bytes.fromhex(g["iq2_xs"]), np.int8)
    m = np.frombuffer(bytes.fromhex(g["iq1_m"]), np.int8)
    orc.set_codebooks(xs, m)
    return xs, m


def read_device(ptr, nbytes, dtype):
    """bytes at a device address the library handed out (not a torch allocation), through the library's own copy kernel"""
    from dwarfstar_red_lite_amd._lib import load
    assert nbytes % 16 == 0
    dst = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    assert load().redhip_calibration_copy(dst.data_ptr(), ptr, nbytes, torch.cuda.current_stream().cuda_stream)
    return dst.cpu().numpy().view(dtype)


def type_word(cfg):
    return cfg["gate_up_type"] if cfg["gate_up_type"] == cfg["down_type"] else cfg["gate_up_type"] | (cfg["down_type"] << 8)


class Case:
    """a one-layer GGUF file of `layout`, a pool over it, experts 0 .. n_load - 1 loaded into slots in a scrambled order"""

    def __init__(self, tmp_path, grids, layout, hidden=512, ffn=256, n_expert=16, n_load=None, seed=700, fast=False, tiles=False, **pool_kw):
        from dwarfstar_red_lite_amd.moe import gguf_expert_layout
        from dwarfstar_red_lite_amd.redmetal_topk import ExpertLayout, RedMetalTopKPool
        self.cfg = cfg = synth.layer_config(hidden=hidden, ffn=ffn, n_expert=n_expert, top_k=4, layout=layout)
        self.lay = synth.make_layer(seed, cfg)
        self.path = str(tmp_path / ("topk_%s_%d.gguf" % (layout, hidden)))
        write_moe_gguf(self.path, cfg, [self.lay])
        self.layouts = []
        for e in range(n_expert):
            d = gguf_expert_layout(self.path, n_expert, 0, e)
            self.layouts.append(ExpertLayout(d["gate_offset"], d["gate_bytes"], d["up_offset"], d["up_bytes"], d["down_offset"], d["down_bytes"]))
        self.slot_bytes = self.layouts[0].gate_bytes * 2 + self.layouts[0].down_bytes
        n_load = n_expert if n_load is None else n_load
        kw = dict(slots_per_slab=5)
        kw.update(pool_kw)
        up = lambda v, a: (v + a - 1) // a * a
        # with the fast path a slot also holds the re-laid copy of its expert, 256-aligned behind the raw bytes (and with tiles a third,
        # tile-major one). The copy: 8 bytes per 32 weights + 2 per 256; IQ2_XS 9 per 32; IQ3_S down matrices 16 per 32
        per32 = lambda t: {17: 9, 21: 16}.get(t, 8)
        n_w = hidden * ffn
        self.copy_bytes = 2 * (n_w // 32 * per32(cfg["gate_up_type"]) + n_w // 256 * 2) + n_w // 32 * per32(cfg["down_type"]) + n_w // 256 * 2
        if tiles:
            self.slot_phys = up(up(self.slot_bytes, 256) + up(self.copy_bytes, 256) + self.copy_bytes, 4096)
        else:
            self.slot_phys = up(up(self.slot_bytes, 256) + self.copy_bytes, 4096) if fast else up(self.slot_bytes, 4096)
        self.pool = RedMetalTopKPool(self.path, (n_load + 3) * self.slot_phys, self.slot_bytes, iq2_xs_grid=grids[0], iq1_m_grid=grids[1], **kw)
        self.word = type_word(cfg)
        if fast:
            assert self.pool.capacity > n_load + 3
            self.pool.enable_fast_path(self.word, hidden, ffn, tiles=tiles)
            assert self.pool.capacity == n_load + 3
        self.slot_of = {}
        for i, e in enumerate(np.random.default_rng(seed).permutation(n_load)):
            self.slot_of[int(e)] = i
            got = self.pool.load(i, self.layouts[e])
            assert got["bytes_read"] == self.slot_bytes

    def want(self, experts, weights, x, row_start=0, row_count=None):
        cfg, lay = self.cfg, self.lay
        acc = None
        for e, w in zip(experts, weights):
            y = orc.expert_ffn(cfg["gate_up_type"], cfg["down_type"], lay["gate"][e], lay["up"][e], lay["down"][e], cfg["hidden"], cfg["ffn"], x,
                               row_start, row_count)
            acc = float(w) * y if acc is None else acc + float(w) * y
        return acc


@pytest.mark.parametrize("layout,fast", [("iq2", False), ("f2", False), ("xs", False), ("m", False), ("iq2", True), ("f2", True), ("xs", True), ("m", True)])
def test_execute_against_cpu_path(tmp_path, grids, layout, fast):
    """fast: the calls with whole output rows run on the slots' re-laid copies, the row windows on the raw rows"""
    c = Case(tmp_path, grids, layout, fast=fast)
    H, F = c.cfg["hidden"], c.cfg["ffn"]
    rng = np.random.default_rng(5)
    for top_k, row_start, row_count in ((4, 0, H), (1, 0, H), (7, 128, 200), (16, H - 1, 1)):
        experts = rng.permutation(16)[:top_k]
        w = rng.random(top_k).astype(np.float32) + 0.05
        x = synth.normed_x(rng, 1, H)[0]
        got, ms = c.pool.execute([c.slot_of[int(e)] for e in experts], [c.layouts[e] for e in experts], w, c.word, H, F, row_start, row_count, x)
        assert got.shape == (row_count,) and ms > 0.0
        assert rel_l2(got, c.want(experts, w, x, row_start, row_count)) <= REL_L2_TOL, (layout, top_k, row_start)
        assert not any(c.pool.slot_inflight(s) for s in range(c.pool.capacity))
    t = c.pool.telemetry()
    assert t["bytes_read"] == 16 * c.slot_bytes and t["read_calls"] >= 48 and t["slab_count"] == 4 and t["capacity"] == 19
    c.pool.close()


@pytest.mark.parametrize("layout,fast,hidden", [("f2", False, 2048), ("f2", True, 2048), ("xs", True, 2048), ("m", True, 2048),
                                                ("f2", True, 1024), ("xs", True, 1024), ("m", True, 1024)])
def test_execute_full_shape_top10(tmp_path, grids, layout, fast, hidden):
    """hidden 2048 (and 1024), ffn 512, ten experts of the mixed-precision layout (gate/up IQ2_XXS, down IQ3_S) and of the IQ2_XS / IQ1_M
    layouts; fast: on the slots' re-laid copies"""
    c = Case(tmp_path, grids, layout, hidden=hidden, ffn=512, n_expert=12, fast=fast)
    rng = np.random.default_rng(6)
    experts = rng.permutation(12)[:10]
    w = rng.random(10).astype(np.float32)
    w /= w.sum()
    x = synth.normed_x(rng, 1, hidden)[0]
    got, _ = c.pool.execute([c.slot_of[int(e)] for e in experts], [c.layouts[e] for e in experts], w, c.word, hidden, 512, 0, hidden, x)
    assert rel_l2(got, c.want(experts, w, x)) <= REL_L2_TOL
    c.pool.close()


def test_validation_and_slot_bookkeeping(tmp_path, grids):
    c = Case(tmp_path, grids, "iq2", n_load=6)
    H, F, L = c.cfg["hidden"], c.cfg["ffn"], c.layouts
    x = np.zeros(H, np.float32)
    ok = lambda ids, lays, w, **kw: c.pool.execute(ids, lays, w, kw.get("word", c.word), kw.get("H", H), F, kw.get("start", 0), kw.get("count", H), kw.get("x", x))
    with pytest.raises(RedHipError, match="duplicate slot 2"):
        ok([1, 2, 2], [L[0]] * 3, [1, 1, 1])
    with pytest.raises(RedHipError, match="exceeds capacity"):
        ok([1, 99], [L[0]] * 2, [1, 1])
    with pytest.raises(RedHipError, match=r"top_k=0 must be in \[1,512\]"):
        ok([], [], [])
    with pytest.raises(RedHipError, match="matrix byte mismatch"):
        ok([1], [L[0]._replace(down_bytes=L[0].down_bytes - 2)], [1])
    with pytest.raises(RedHipError, match="invalid top-k dimensions"):
        ok([1], [L[0]], [1], start=H)
    with pytest.raises(RedHipError, match="unsupported top-k GGML type word"):
        ok([1], [L[0]], [1], word=2)
    # generations count the loads of a slot; a slot in flight is not overwritten
    assert c.pool.slot_generation(0) == 1 and c.pool.slot_generation(8) == 0
    c.pool.load(0, L[3])
    assert c.pool.slot_generation(0) == 2
    xd, od = torch.zeros(H, device="cuda"), torch.zeros(H, device="cuda")
    c.pool.encode(None, [0, 1], [L[3], L[0]], [0.5, 0.5], c.word, H, F, 0, H, xd.data_ptr(), od.data_ptr())
    assert c.pool.slot_inflight(0) and c.pool.slot_inflight(1) and not c.pool.slot_inflight(2)
    with pytest.raises(RedHipError, match="refusing to overwrite in-flight top-k slot 0"):
        c.pool.load(0, L[2])
    torch.cuda.synchronize()
    c.pool.release([0, 1])
    assert not c.pool.slot_inflight(0)
    c.pool.load(0, L[2])
    with pytest.raises(RedHipError, match="payload exceeds slot size"):
        c.pool.load(1, L[0]._replace(gate_bytes=L[0].gate_bytes + 8192))
    with pytest.raises(RedHipError, match="invalid pread range"):
        c.pool.load(1, L[0]._replace(gate_offset=10 ** 12))
    with pytest.raises(RedHipError, match="must be set before any slab"):
        c.pool.set_classes([c.slot_bytes], [4])
    c.pool.close()


def test_slot_classes_and_budget(tmp_path, grids):
    from dwarfstar_red_lite_amd.redmetal_topk import RedMetalTopKPool
    c = Case(tmp_path, grids, "f2", n_load=0)
    big = (c.slot_bytes + 4095) // 4096 * 4096
    pool = RedMetalTopKPool(c.path, 10 * big, c.slot_bytes, slots_per_slab=2, iq2_xs_grid=grids[0], iq1_m_grid=grids[1])
    assert pool.capacity == 10
    with pytest.raises(RedHipError, match="exceed the cache budget"):
        pool.set_classes([big, 4096], [10, 1])
    pool.set_classes([8192, c.slot_bytes], [3, 5])                  # slots 0..2 small, 3..7 expert sized
    assert pool.capacity == 8
    with pytest.raises(RedHipError, match="payload exceeds slot size"):
        pool.load(1, c.layouts[0])
    pool.load(3, c.layouts[4])
    pool.load(7, c.layouts[9])
    g3, u3, d3 = pool.addresses(3, c.layouts[4])
    g4, _, _ = pool.addresses(4, c.layouts[4])
    assert u3 - g3 == c.layouts[4].gate_bytes and d3 - u3 == c.layouts[4].up_bytes and g4 - g3 == big
    t = pool.telemetry()
    assert t["slab_count"] == 2 and t["allocated_bytes"] == 2 * big + 1 * big       # slab of slots 3,4 and slab of slot 7 alone
    rng = np.random.default_rng(8)
    x = synth.normed_x(rng, 1, c.cfg["hidden"])[0]
    got, _ = pool.execute([7, 3], [c.layouts[9], c.layouts[4]], [0.25, 0.75], c.word, c.cfg["hidden"], c.cfg["ffn"], 0, c.cfg["hidden"], x)
    assert rel_l2(got, c.want([9, 4], [0.25, 0.75], x)) <= REL_L2_TOL
    pool.allocate_all()
    assert pool.telemetry()["slab_count"] == 2 + 3
    pool.close()
    c.pool.close()


@pytest.mark.parametrize("layout,fast", [("iq2", False), ("f2", False), ("iq2", True), ("f2", True), ("xs", True), ("m", True)])
def test_device_driven_forms(tmp_path, grids, layout, fast):
    """slot addresses gathered on the device from the residency table, weights on the device: into, into with the sum left to the
    caller, two input vectors, and the fused tail; replayed from a HIP graph as well (these forms copy nothing from the host).
    fast: on the slots' re-laid copies (the sum left to the caller stays on the raw rows)"""
    c = Case(tmp_path, grids, layout, fast=fast)
    H, F, E = c.cfg["hidden"], c.cfg["ffn"], 16
    gb = c.layouts[0].gate_bytes
    table_ptr = c.pool.residency_table_init(3, E)
    for e in range(E):
        c.pool.residency_set(1, e, c.slot_of[e])
    c.pool.residency_clear(1, 5)
    g_addr = [c.pool.addresses(c.slot_of[e], c.layouts[e])[0] for e in range(E)]
    host_table = read_device(table_ptr, 3 * E * 8, np.uint64).reshape(3, E)
    assert host_table[0].sum() == 0 and host_table[2].sum() == 0 and host_table[1][5] == 0
    assert all(int(host_table[1][e]) == g_addr[e] for e in range(E) if e != 5)
    rng = np.random.default_rng(9)
    experts = np.array([3, 11, 0, 7, 9, 14])
    w = (rng.random(6).astype(np.float32) + 0.1)
    x = synth.normed_x(rng, 2, H)
    slots_dev = torch.from_numpy(np.array([g_addr[e] for e in experts], np.uint64).view(np.int64)).cuda()
    w_dev, x_dev = torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda()
    out = torch.zeros(H, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    c.pool.encode_device_into(stream, slots_dev.data_ptr(), w_dev.data_ptr(), 6, c.word, H, F, gb, gb, x_dev.data_ptr(), out.data_ptr())
    want0 = c.want(experts, w, x[0])
    assert rel_l2(out.cpu().numpy(), want0) <= REL_L2_TOL
    # the sum left to the caller: tmp[e][r] in the pool's buffer
    c.pool.encode_device_into(stream, slots_dev.data_ptr(), w_dev.data_ptr(), 6, c.word, H, F, gb, gb, x_dev.data_ptr(), None)
    torch.cuda.synchronize()
    tmp = read_device(c.pool.tmp_buffer(), 6 * H * 4, np.float32).reshape(6, H)
    for k, e in enumerate(experts):
        assert rel_l2(tmp[k], c.want([e], [1.0], x[0])) <= REL_L2_TOL
    # two input vectors: experts 0..3 on x[0], 4..5 on x[1]
    c.pool.encode_device_into(stream, slots_dev.data_ptr(), w_dev.data_ptr(), 6, c.word, H, F, gb, gb, x_dev[0].data_ptr(), out.data_ptr(),
                              x1_dev=x_dev[1].data_ptr(), x_split=4)
    want2 = c.want(experts[:4], w[:4], x[0]) + c.want(experts[4:], w[4:], x[1])
    assert rel_l2(out.cpu().numpy(), want2) <= REL_L2_TOL
    # fused tail: x = layer_out = resid + (routed + shared * scalar)
    resid, shared = torch.from_numpy(synth.normed_x(rng, 2, H)).cuda()
    scalar = torch.tensor([0.37], device="cuda")
    x_out, layer_out = torch.zeros(H, device="cuda"), torch.zeros(H, device="cuda")
    assert c.pool.encode_device_tail(stream, slots_dev.data_ptr(), w_dev.data_ptr(), 6, c.word, H, F, gb, gb, x_dev.data_ptr(), resid.data_ptr(),
                                     shared.data_ptr(), scalar.data_ptr(), x_out.data_ptr(), layer_out.data_ptr()) == 1
    want_tail = resid.cpu().numpy().astype(np.float64) + (want0 + shared.cpu().numpy().astype(np.float64) * 0.37)
    assert torch.equal(x_out, layer_out) and rel_l2(x_out.cpu().numpy(), want_tail) <= REL_L2_TOL
    big = torch.zeros(65, dtype=torch.int64, device="cuda")
    assert c.pool.encode_device_tail(stream, big.data_ptr(), w_dev.data_ptr(), 65, c.word, H, F, gb, gb, x_dev.data_ptr(), resid.data_ptr(),
                                     shared.data_ptr(), scalar.data_ptr(), x_out.data_ptr(), layer_out.data_ptr()) == -1
    with pytest.raises(RedHipError, match="matrix byte mismatch"):
        c.pool.encode_device_into(stream, slots_dev.data_ptr(), w_dev.data_ptr(), 6, c.word, H, F, gb + 66, gb, x_dev.data_ptr(), out.data_ptr())
    # graph replays of the device-driven form against its eager result
    eager = torch.zeros(H, device="cuda")
    c.pool.encode_device_into(stream, slots_dev.data_ptr(), w_dev.data_ptr(), 6, c.word, H, F, gb, gb, x_dev.data_ptr(), eager.data_ptr())
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    gout = torch.zeros(H, device="cuda")
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            c.pool.encode_device_into(side.cuda_stream, slots_dev.data_ptr(), w_dev.data_ptr(), 6, c.word, H, F, gb, gb, x_dev.data_ptr(), gout.data_ptr())
    for _ in range(3):
        gout.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(gout, eager)
        c.pool.encode_device_into(stream, slots_dev.data_ptr(), w_dev.data_ptr(), 6, c.word, H, F, gb, gb, x_dev[1].data_ptr(), out.data_ptr())
        torch.cuda.synchronize()
    del graph
    c.pool.close()


@pytest.mark.parametrize("layout,tiles", [("iq2", False), ("f2", False), ("xs", False), ("iq2", True), ("f2", True), ("xs", True), ("m", True)])
def test_batched_and_mapped_pairs(tmp_path, grids, layout, tiles):
    """prefill form: pairs sorted by expert over a ragged routing (an expert with 19 pairs, experts with one, experts with none), tokens
    tok_first .. of a larger buffer; the same pairs on experts read in place from device copies of the whole tensors.
    tiles: the batched form on the tile-major copies of the slots (the mapped form, which has no slots, stays on the raw rows)"""
    c = Case(tmp_path, grids, layout, fast=tiles, tiles=tiles)
    H, F, E, K = c.cfg["hidden"], c.cfg["ffn"], 16, 3
    rng = np.random.default_rng(10)
    tok_first, ntok = 2, 21
    ids = np.stack([rng.permutation(12)[:K] for _ in range(ntok)]).astype(np.uint32)
    ids[:19, 1] = 13                                                   # a popular expert: three slices of eight pairs
    ids[:19, 0] = np.where(ids[:19, 0] == 13, 14, ids[:19, 0])
    ids[:19, 2] = np.where(ids[:19, 2] == 13, 15, ids[:19, 2])
    for t in range(ntok):
        assert len(set(ids[t].tolist())) == K
    w = (rng.random((ntok, K)).astype(np.float32) + 0.1)
    uid, start, ptok, pw, tp = orc.group_pairs(ids, w, E)
    x = synth.normed_x(rng, tok_first + ntok, H)
    x_dev = torch.from_numpy(x).cuda()
    out = torch.full((tok_first + ntok, H), 7.0, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    slots = [c.slot_of[int(e)] for e in uid]
    c.pool.encode_batched(stream, slots, [c.layouts[int(e)] for e in uid], c.word, H, F, tok_first, ntok, K, ptok + tok_first, pw, start, tp,
                          x_dev.data_ptr(), out.data_ptr())
    assert all(c.pool.slot_inflight(s) for s in slots)
    torch.cuda.synchronize()
    c.pool.release(slots)
    got = out.cpu().numpy()
    assert (got[:tok_first] == 7.0).all()                              # rows before tok_first are not written
    for t in range(ntok):
        assert rel_l2(got[tok_first + t], c.want(ids[t], w[t], x[tok_first + t])) <= REL_L2_TOL, t
    # mapped: whole tensors on the device, experts addressed by id
    g_dev, u_dev, d_dev = (torch.from_numpy(np.ascontiguousarray(c.lay[k])).cuda() for k in ("gate", "up", "down"))
    out2 = torch.zeros_like(out)
    L0 = c.layouts[0]
    c.pool.encode_mapped(stream, g_dev.data_ptr(), u_dev.data_ptr(), d_dev.data_ptr(), L0.gate_bytes, L0.up_bytes, L0.down_bytes, uid, c.word, H, F,
                         tok_first, ntok, K, ptok + tok_first, pw, start, tp, x_dev.data_ptr(), out2.data_ptr())
    torch.cuda.synchronize()
    if tiles:
        assert rel_l2(out2[tok_first:].cpu().numpy(), out[tok_first:].cpu().numpy()) <= REL_L2_TOL
    else:
        assert torch.equal(out2[tok_first:], out[tok_first:])          # same kernels on the same bytes
    with pytest.raises(RedHipError, match="expert_start is inconsistent"):
        c.pool.encode_batched(stream, slots, [c.layouts[int(e)] for e in uid], c.word, H, F, tok_first, ntok, K, ptok + tok_first, pw, start[::-1].copy(), tp,
                              x_dev.data_ptr(), out.data_ptr())
    with pytest.raises(RedHipError, match="pair token out of range"):
        c.pool.encode_batched(stream, slots, [c.layouts[int(e)] for e in uid], c.word, H, F, 0, ntok, K, ptok + tok_first, pw, start, tp,
                              x_dev.data_ptr(), out.data_ptr())
    c.pool.close()


def test_batched_pairs_with_more_than_sixteen_experts_per_token(tmp_path, grids):
    """the batched form takes any top_k the pool does (the reference's sum loops over top_k): 17 and 20 experts per token run the looped
    combine, in selection order, against the CPU path"""
    c = Case(tmp_path, grids, "iq2", n_expert=24)
    H, F, E = c.cfg["hidden"], c.cfg["ffn"], 24
    rng = np.random.default_rng(44)
    stream = torch.cuda.current_stream().cuda_stream
    for K, ntok in ((17, 3), (20, 5)):
        ids = np.stack([rng.permutation(E)[:K] for _ in range(ntok)]).astype(np.uint32)
        w = rng.random((ntok, K)).astype(np.float32) + 0.1
        uid, start, ptok, pw, tp = orc.group_pairs(ids, w, E)
        x = synth.normed_x(rng, ntok, H)
        x_dev = torch.from_numpy(x).cuda()
        out = torch.zeros((ntok, H), device="cuda")
        slots = [c.slot_of[int(e)] for e in uid]
        c.pool.encode_batched(stream, slots, [c.layouts[int(e)] for e in uid], c.word, H, F, 0, ntok, K, ptok, pw, start, tp, x_dev.data_ptr(), out.data_ptr())
        torch.cuda.synchronize()
        c.pool.release(slots)
        got = out.cpu().numpy()
        for t in range(ntok):
            assert rel_l2(got[t], c.want(ids[t], w[t], x[t])) <= REL_L2_TOL, (K, t)
    c.pool.close()


def test_fast_path_copies_follow_the_slots(tmp_path, grids):
    """the re-laid copy of a slot is rewritten whenever the slot is loaded: after a slot changes its expert, calls through the copies
    (whole rows) and through the raw rows (a row window) both see the new expert; shapes and moments the fast path refuses"""
    from dwarfstar_red_lite_amd.redmetal_topk import RedMetalTopKPool
    c = Case(tmp_path, grids, "iq2", hidden=1024, ffn=512, n_expert=12, n_load=8, fast=True)
    H, F, L = 1024, 512, c.layouts
    rng = np.random.default_rng(71)
    x = synth.normed_x(rng, 1, H)[0]
    w = rng.random(5).astype(np.float32) + 0.1
    experts = [0, 3, 5, 6, 7]
    slots = [c.slot_of[e] for e in experts]
    got, _ = c.pool.execute(slots, [L[e] for e in experts], w, c.word, H, F, 0, H, x)
    assert rel_l2(got, c.want(experts, w, x)) <= REL_L2_TOL
    # slot of expert 3 now holds expert 10, the slot of expert 6 expert 11
    c.pool.load(c.slot_of[3], L[10])
    c.pool.load(c.slot_of[6], L[11])
    now = [0, 10, 5, 11, 7]
    got, _ = c.pool.execute(slots, [L[e] for e in now], w, c.word, H, F, 0, H, x)
    assert rel_l2(got, c.want(now, w, x)) <= REL_L2_TOL
    part, _ = c.pool.execute(slots, [L[e] for e in now], w, c.word, H, F, 100, 300, x)
    assert rel_l2(part, c.want(now, w, x, 100, 300)) <= REL_L2_TOL
    assert rel_l2(part, got[100:400]) <= 2 * REL_L2_TOL
    with pytest.raises(RedHipError, match="before any slab"):
        c.pool.enable_fast_path(c.word, H, F)
    c.pool.close()
    pool = RedMetalTopKPool(c.path, 8 * c.slot_phys, c.slot_bytes, iq2_xs_grid=grids[0], iq1_m_grid=grids[1])
    with pytest.raises(RedHipError, match="all-IQ2_XXS"):
        pool.enable_fast_path(14, H, F)
    with pytest.raises(RedHipError, match="all-IQ2_XXS"):
        pool.enable_fast_path(17 | (29 << 8), H, F)
    with pytest.raises(RedHipError, match="tile-major copies"):
        pool.enable_fast_path(16, 4096, F, tiles=True)
    with pytest.raises(RedHipError, match="all-IQ2_XXS"):
        pool.enable_fast_path(16, 768, F)
    pool.enable_fast_path(16, H, F)
    with pytest.raises(RedHipError, match="already enabled"):
        pool.enable_fast_path(16, H, F)
    with pytest.raises(RedHipError, match="before the fast path"):
        pool.set_classes([c.slot_bytes], [2])
    pool.close()


@pytest.mark.parametrize("layout", ["iq2", "f2", "xs"])
def test_batched_chunk_of_512_tokens_on_the_tile_copies(tmp_path, grids, layout):
    """a prefill chunk at the full expert shape (hidden 2048, ffn 512, ten of 48 experts per token, 512 tokens) through the batched form
    on the slots' tile-major copies: every 16th token against the CPU path, every token against the same call on a pool without copies
    (the raw-row kernels)"""
    H, F, E, K, ntok = 2048, 512, 48, 10, 512
    fast = Case(tmp_path, grids, layout, hidden=H, ffn=F, n_expert=E, fast=True, tiles=True, slots_per_slab=7)
    (tmp_path / "raw").mkdir()
    raw = Case(tmp_path / "raw", grids, layout, hidden=H, ffn=F, n_expert=E)
    rng = np.random.default_rng(12)
    logits = rng.standard_normal((ntok, E)) + 1.5 * (np.arange(E) < 3)                # three popular experts: wide tiles, narrow ones, singles
    ids = np.argsort(-logits, axis=1)[:, :K].astype(np.uint32)
    w = rng.random((ntok, K)).astype(np.float32) + 0.05
    w /= w.sum(axis=1, keepdims=True)
    uid, start, ptok, pw, tp = orc.group_pairs(ids, w, E)
    x = synth.normed_x(rng, ntok, H)
    x_dev = torch.from_numpy(x).cuda()
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for c in (fast, raw):
        out = torch.zeros((ntok, H), device="cuda")
        slots = [c.slot_of[int(e)] for e in uid]
        c.pool.encode_batched(stream, slots, [c.layouts[int(e)] for e in uid], c.word, H, F, 0, ntok, K, ptok, pw, start, tp, x_dev.data_ptr(), out.data_ptr())
        torch.cuda.synchronize()
        c.pool.release(slots)
        outs.append(out.cpu().numpy())
    for t in range(0, ntok, 16):
        assert rel_l2(outs[0][t], fast.want(ids[t], w[t], x[t])) <= REL_L2_TOL, t
    for t in range(ntok):
        assert rel_l2(outs[0][t], outs[1][t]) <= REL_L2_TOL, t
    fast.pool.close()
    raw.pool.close()


def test_fast_path_up_to_64_experts_per_call(tmp_path, grids):
    """the copies serve calls of up to 64 experts (the partial vectors are sized for that); a call with more runs on the raw rows of the
    same pool: both against the CPU path, through the device-driven form"""
    c = Case(tmp_path, grids, "iq2", n_expert=72, fast=True)
    H, F = c.cfg["hidden"], c.cfg["ffn"]
    gb = c.layouts[0].gate_bytes
    rng = np.random.default_rng(81)
    x = synth.normed_x(rng, 1, H)[0]
    x_dev = torch.from_numpy(x).cuda()
    stream = torch.cuda.current_stream().cuda_stream
    g_addr = [c.pool.addresses(c.slot_of[e], c.layouts[e])[0] for e in range(72)]
    for top_k in (64, 66):
        experts = rng.permutation(72)[:top_k]
        w = rng.random(top_k).astype(np.float32) + 0.05
        slots_dev = torch.from_numpy(np.array([g_addr[e] for e in experts], np.uint64).view(np.int64)).cuda()
        w_dev = torch.from_numpy(w).cuda()
        out = torch.zeros(H, device="cuda")
        c.pool.encode_device_into(stream, slots_dev.data_ptr(), w_dev.data_ptr(), top_k, c.word, H, F, gb, gb, x_dev.data_ptr(), out.data_ptr())
        assert rel_l2(out.cpu().numpy(), c.want(experts, w, x)) <= REL_L2_TOL, top_k
    c.pool.close()
