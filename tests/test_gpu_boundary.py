"""GPU parity of the drop-in boundary: redmetal_quant_rows, the redmetal_ffn pool and rl_native_router_gpu_f32,
driven the way the reference's dev tools drive them (a file of raw blocks plus byte offsets)."""
import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import expert_type_word, synth
from gpu_common import REL_L2_TOL, T_F32, T_IQ2, T_IQ3, T_Q6K, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def model_file(tmp_path_factory):
    """raw synthetic 'model': 6 experts x (gate|up|down) in two layouts, a router, at odd (even-aligned) offsets"""
    H, F = 512, 256
    rng = np.random.default_rng(77)
    parts, off, index = [], 0, {}

    def add(name, arr):
        nonlocal off
        b = np.ascontiguousarray(arr).view(np.uint8).ravel()
        index[name] = (off, b.size)
        parts.append(b)
        off += b.size

    add("pad", np.zeros(6, np.uint8))
    for e in range(3):
        add("iq2.gate.%d" % e, synth.quant_rows(rng, T_IQ2, F, H))
        add("iq2.up.%d" % e, synth.quant_rows(rng, T_IQ2, F, H))
        add("iq2.down.%d" % e, synth.quant_rows(rng, T_IQ2, H, F))
    for e in range(3):
        add("f2.gate.%d" % e, synth.quant_rows(rng, T_IQ2, F, H))
        add("f2.up.%d" % e, synth.quant_rows(rng, T_IQ2, F, H))
        add("f2.down.%d" % e, synth.quant_rows(rng, T_IQ3, H, F))
    add("q6.gate", synth.quant_rows(rng, T_Q6K, F, H))
    add("q6.up", synth.quant_rows(rng, T_Q6K, F, H))
    add("q6.down", synth.quant_rows(rng, T_Q6K, H, F))
    add("router.f32", (0.02 * rng.standard_normal((16, H))).astype(np.float32))
    add("router.q6k", synth.quant_rows(rng, T_Q6K, 16, H, d_range=(1e-5, 3e-5)))
    blob = np.concatenate(parts)
    path = tmp_path_factory.mktemp("model") / "raw_blocks.bin"
    blob.tofile(path)
    return str(path), blob, index, H, F


def test_quant_rows(model_file):
    from dwarfstar_red_lite_amd.redmetal_quant import RedMetalQuantBridge
    from dwarfstar_red_lite_amd import RedHipError
    path, blob, index, H, F = model_file
    br = RedMetalQuantBridge()
    x = synth.normed_x(np.random.default_rng(1), 1, H)[0]
    for name, t, ncols, nrows in (("iq2.gate.1", T_IQ2, H, F), ("f2.down.2", T_IQ3, F, H), ("q6.up", T_Q6K, H, F), ("router.f32", T_F32, H, 16)):
        off, n = index[name]
        xin = x[:ncols]
        out, io_ms, gpu_ms = br.rows(path, off, n, t, ncols, nrows, 3, 11, xin)
        want = orc.matvec(t, blob[off:off + n], ncols, xin, row_start=3, row_count=11)
        assert rel_l2(out, want) <= REL_L2_TOL and io_ms >= 0 and gpu_ms >= 0
    off, n = index["iq2.gate.0"]
    with pytest.raises(RedHipError, match="matrix byte size mismatch"):
        br.rows(path, off, n - 66, T_IQ2, H, F, 0, 1, x)
    with pytest.raises(RedHipError, match="unsupported GGML type"):
        br.rows(path, off, n, 18, H, F, 0, 1, x)
    with pytest.raises(RedHipError, match="invalid mixed-quant dimensions"):
        br.rows(path, off, n, T_IQ2, H, F, F, 1, x)
    with pytest.raises(RedHipError, match="invalid pread range"):
        br.rows(path, blob.size - 10, n, T_IQ2, H, F, 0, 1, x)


def test_ffn_pool(model_file):
    from dwarfstar_red_lite_amd.redmetal_ffn import ExpertLayout, RedMetalFfnPool
    from dwarfstar_red_lite_amd import RedHipError
    path, blob, index, H, F = model_file
    x = synth.normed_x(np.random.default_rng(2), 1, H)[0]
    slot_bytes = 2 * index["q6.gate"][1] + index["q6.down"][1]      # the largest of the three families
    aligned = (slot_bytes + 4095) // 4096 * 4096
    with RedMetalFfnPool(path, 5 * aligned + 100, slot_bytes, slots_per_slab=2) as pool:
        assert pool.capacity == 5 and pool.telemetry()["slab_count"] == 0
        for fam, gu, dn in (("iq2", T_IQ2, T_IQ2), ("f2", T_IQ2, T_IQ3), ("q6", T_Q6K, T_Q6K)):
            for e in range(3 if fam != "q6" else 1):
                sfx = ".%d" % e if fam != "q6" else ""
                lay = ExpertLayout(*index[fam + ".gate" + sfx], *index[fam + ".up" + sfx], *index[fam + ".down" + sfx])
                slot = 4 if fam == "q6" else (e + 1) % 5      # slots 1..4: three slabs of two slots, the last one short
                info = pool.load(slot, lay)
                assert info["bytes_read"] == lay.gate_bytes + lay.up_bytes + lay.down_bytes
                g, u, d = pool.addresses(slot, lay)
                assert u == g + lay.gate_bytes and d == u + lay.up_bytes and g % 4096 == 0
                sl = lambda o, n: blob[o:o + n]
                want = orc.expert_ffn(gu, dn, sl(lay.gate_offset, lay.gate_bytes), sl(lay.up_offset, lay.up_bytes),
                                      sl(lay.down_offset, lay.down_bytes), H, F, x)
                out, ms = pool.execute(slot, lay, expert_type_word(gu, dn), H, F, 0, H, x)
                assert rel_l2(out, want) <= REL_L2_TOL, (fam, e)
                win, _ = pool.execute(slot, lay, expert_type_word(gu, dn), H, F, 500, 12, x)
                assert np.array_equal(win, out[500:])
                assert not pool.slot_inflight(slot)
        tel = pool.telemetry()
        assert tel["slab_count"] == 3 and tel["allocated_bytes"] == 5 * aligned and tel["read_calls"] >= 21
        lay = ExpertLayout(*index["iq2.gate.0"], *index["iq2.up.0"], *index["iq2.down.0"])
        with pytest.raises(RedHipError, match="unsupported FFN GGML type"):
            pool.execute(1, lay, 18, H, F, 0, H, x)
        with pytest.raises(RedHipError, match="FFN matrix byte mismatch"):
            pool.execute(1, lay._replace(gate_bytes=lay.gate_bytes - 66), T_IQ2, H, F, 0, H, x)
        with pytest.raises(RedHipError, match="invalid FFN dimensions"):
            pool.execute(1, lay, T_IQ2, H, F, H, 1, x)
        with pytest.raises(RedHipError, match="exceeds slot size"):
            pool.load(0, lay._replace(down_bytes=aligned))
    with pytest.raises(RedHipError, match="cannot fit one aligned expert slot"):
        RedMetalFfnPool(path, 4096, 8192)


def test_router_gpu(model_file):
    from dwarfstar_red_lite_amd import redmetal_quant as rq
    from dwarfstar_red_lite_amd import RedHipError
    path, blob, index, H, F = model_file
    x = synth.normed_x(np.random.default_rng(3), 1, H)[0]
    for name, t in (("router.f32", T_F32), ("router.q6k", T_Q6K)):
        off, n = index[name]
        logits, tel = rq.router_gpu(path, t, H, 16, off, n, x)
        want = orc.router_logits(t, blob[off:off + n], H, 16, x)
        assert np.max(np.abs(logits - want)) <= 1e-3 * max(1.0, float(np.abs(want).max())) and rel_l2(logits, want) <= REL_L2_TOL
        ids, w = rq.router_select(logits, 4)
        ci, cw = orc.router_select(want, 4)
        assert np.array_equal(ids, ci) and np.all(np.abs(w - cw) <= 1e-5)
    off, n = index["router.f32"]
    with pytest.raises(RedHipError, match="shape/span mismatch"):
        rq.router_gpu(path, T_F32, H, 16, off, n - 4, x)
    with pytest.raises(RedHipError, match="invalid HIP router arguments"):
        rq.router_gpu(path, T_IQ2, H, 16, off, n, x)
