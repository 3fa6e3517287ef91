"""Router selection, expert FFN, shared expert, layer composition and grouping of the CPU oracle (no GPU).

Pins: the reference's golden vectors (tests/golden/router_select.json, shared_expert.json), the known answers of
native/redlite_native_router_offline_test.c:7-38 and tests/test_ffn.py:8-13, closed forms and brute force.
"""
import json
import math
import os
import struct

import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth

T_F32, T_Q6K, T_IQ2, T_IQ3 = 0, 14, 16, 21


def unhex(s, dtype):
    return np.frombuffer(bytes.fromhex(s), dtype=dtype).copy()


def test_router_known_answers():
    ids, w = orc.router_select(np.array([0, 1, 2, 3], np.float32), 2)
    assert list(ids) == [3, 2]
    assert abs(w[0] - 0.7310585786) < 1e-6 and abs(w[1] - 0.2689414214) < 1e-6 and abs(w.sum() - 1) < 1e-6
    ids, _ = orc.router_select(np.array([1, 1, 0, 0], np.float32), 2)
    assert list(ids) == [0, 1]
    with pytest.raises(ValueError):
        orc.router_select(np.array([np.nan, 1.0], np.float32), 1)
    with pytest.raises(ValueError):
        orc.router_select(np.array([0.0, 1.0], np.float32), 3)


def test_router_golden(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "router_select.json")))
    assert len(g["cases"]) >= 10
    for c in g["cases"]:
        logits = unhex(c["logits"], np.float32)
        ids, w, probs = orc.router_select(logits, c["top_k"], want_probs=True)
        assert list(ids) == c["ids"]
        assert np.array_equal(w.view(np.uint32), unhex(c["weights"], np.uint32))
        assert np.array_equal(probs.view(np.uint32), unhex(c["probs"], np.uint32))


def test_router_documented_case():
    l = np.array([np.float32(math.sin(0.37 * i) * 3.0) + (np.float32(0.5) if i % 7 == 0 else np.float32(0)) for i in range(512)], np.float32)
    ids, w = orc.router_select(l, 10)
    assert list(ids) == [259, 140, 378, 21, 497, 462, 56, 343, 175, 224]
    assert np.allclose(w, [0.108234048, 0.108041741, 0.107689209, 0.107116669, 0.106419519, 0.0965727493, 0.0947094038,
                           0.0925658271, 0.0904977918, 0.0881530568], atol=2e-7)


def test_router_invariants_bruteforce():
    rng = np.random.default_rng(11)
    for E, K in ((8, 3), (33, 5), (512, 10)):
        for _ in range(20):
            l = rng.standard_normal(E).astype(np.float32)
            if rng.random() < 0.5:
                l[rng.integers(0, E, 4)] = l[0]          # exact ties
            ids, w, p = orc.router_select(l, K, want_probs=True)
            assert len(set(ids)) == K and abs(float(w.sum()) - 1.0) < 1e-6
            order = sorted(range(E), key=lambda i: (-p[i], i))[:K]
            assert list(ids) == order
            assert np.all(np.diff(p[ids]) <= 0)


def test_silu_mul_known_values():
    L = orc.lib()
    assert L.orc_silu_mul(0.0, 2.0) == 0.0
    assert abs(L.orc_silu_mul(1.0, 2.0) - 2.0 / (1.0 + math.exp(-1.0))) < 1e-15
    assert abs(L.orc_silu_mul(-1.0, 2.0) + 2.0 * math.exp(-1.0) / (1.0 + math.exp(-1.0))) < 1e-15
    assert abs(L.orc_silu_mul(-800.0, 1.0)) == 0.0 and L.orc_silu_mul(800.0, 1.0) == 800.0


def test_shared_expert_golden(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "shared_expert.json")))
    for c in g["cases"]:
        H, F, E, gu, dn = c["hidden"], c["ffn"], c["experts"], c["gate_up_type"], c["down_type"]
        f = unhex(c["file"], np.uint8)
        x = unhex(c["x"], np.float32)
        n_inp, n_g, n_d = 4 * H, F * orc.row_bytes(gu, H), H * orc.row_bytes(dn, F)
        gate_inp = f[:n_inp].view(np.float32)
        gate, up = f[n_inp:n_inp + n_g], f[n_inp + n_g:n_inp + 2 * n_g]
        down = f[n_inp + 2 * n_g:n_inp + 2 * n_g + n_d]
        router = f[n_inp + 2 * n_g + n_d:]
        out, s = orc.shared_expert_standalone(gu, dn, gate, up, down, gate_inp, H, F, x)
        assert s == struct.unpack("<d", bytes.fromhex(c["scalar_gate"]))[0]
        assert np.array_equal(out, unhex(c["out"], np.float64))
        part, _ = orc.shared_expert_standalone(gu, dn, gate, up, down, gate_inp, H, F, x, row_start=100, row_count=17)
        assert np.array_equal(part, out[100:117])
        logits = orc.router_logits(T_F32, router, H, E, x)
        assert np.array_equal(logits, unhex(c["router_logits"], np.float32))
        # engine-style variant (double exp, float hand-offs) differs only by rounding of the activation
        eng, s2 = orc.shared_expert(gu, dn, gate, up, down, gate_inp, H, F, x)
        assert abs(s2 - s) < 1e-15
        rel = np.linalg.norm(eng.astype(np.float64) * s2 - out) / np.linalg.norm(out)
        assert rel < 1e-5


def _unit_iq2_rows(nrows, ncols):
    """IQ2_XXS rows whose every weight is exactly +1 (d = 1, grid entry 0, scale 0, no signs)."""
    rows = np.zeros((nrows, 66 * (ncols // 256)), np.uint8)
    rows[:, 1::66] = 0x3C
    return rows


def test_expert_ffn_closed_form():
    H, F = 512, 256
    x = synth.normed_x(np.random.default_rng(3), 1, H)[0]
    gate, up, down = _unit_iq2_rows(F, H), _unit_iq2_rows(F, H), _unit_iq2_rows(H, F)
    s = float(x.astype(np.float64).sum())
    act = s / (1 + math.exp(-s)) * s
    out = orc.expert_ffn(T_IQ2, T_IQ2, gate, up, down, H, F, x)
    assert np.allclose(out, F * act, rtol=1e-12)
    # weighted combine with weights summing to one returns the same vector
    ids = np.array([0, 0, 0], np.uint32)
    w = np.array([0.5, 0.25, 0.25], np.float32)
    res = np.empty(H, np.float64)
    L = orc.lib()
    p = lambda a: a.ctypes.data_as(orc.C.c_void_p)
    assert L.orc_routed_topk(T_IQ2, T_IQ2, p(gate), p(up), p(down), gate.nbytes, up.nbytes, down.nbytes, p(ids), p(w), 3, H, F, p(x), p(res))
    assert np.allclose(res, F * act, rtol=1e-12)


@pytest.mark.parametrize("layout", ["iq2", "f2"])
def test_expert_ffn_equals_composition(layout):
    """orc_expert_ffn == down(row_dot_d) o silu_mul o gate/up(row_dot), the pinned pieces, for every type pairing."""
    cfg = synth.layer_config(hidden=512, ffn=256, n_expert=4, top_k=2, layout=layout)
    lay = synth.make_layer(21, cfg)
    x = synth.normed_x(np.random.default_rng(4), 1, 512)[0]
    gu, dn = cfg["gate_up_type"], cfg["down_type"]
    e = 2
    gate = lay["gate"][e].reshape(256, -1)
    up = lay["up"][e].reshape(256, -1)
    down = lay["down"][e].reshape(512, -1)
    act = np.array([orc.lib().orc_silu_mul(orc.row_dot(gu, gate[r], x), orc.row_dot(gu, up[r], x)) for r in range(256)])
    want = np.array([orc.row_dot(dn, down[r], act) for r in range(512)])
    got = orc.expert_ffn(gu, dn, lay["gate"][e], lay["up"][e], lay["down"][e], 512, 256, x)
    assert np.array_equal(got, want)
    win = orc.expert_ffn(gu, dn, lay["gate"][e], lay["up"][e], lay["down"][e], 512, 256, x, row_start=500, row_count=12)
    assert np.array_equal(win, want[500:])


@pytest.mark.parametrize("layout", ["iq2", "f2"])
def test_layer_equals_composition(layout):
    cfg = synth.layer_config(hidden=512, ffn=256, n_expert=16, top_k=4, layout=layout)
    lay = synth.make_layer(33, cfg)
    x = synth.normed_x(np.random.default_rng(6), 2, 512)
    L = orc.Layer(cfg, **lay)
    out, ids, w, logits = L.forward(x, threads=3)
    out1, ids1, w1, _ = L.forward(x, threads=1)
    assert np.array_equal(out, out1) and np.array_equal(ids, ids1)
    for t in range(2):
        lg = orc.router_logits(cfg["router_type"], lay["router"], 512, 16, x[t])
        assert np.array_equal(lg, logits[t])
        i2, w2 = orc.router_select(lg, 4)
        assert np.array_equal(i2, ids[t]) and np.array_equal(w2, w[t])
        routed = np.zeros(512, np.float64)
        for k in range(4):
            e = int(i2[k])
            routed += np.float64(w2[k]) * orc.expert_ffn(cfg["gate_up_type"], cfg["down_type"], lay["gate"][e], lay["up"][e], lay["down"][e], 512, 256, x[t])
        sh, s = orc.shared_expert(cfg["sh_gate_up_type"], cfg["sh_down_type"], lay["sh_gate"], lay["sh_up"], lay["sh_down"],
                                  lay["sh_gate_inp"], 512, 256, x[t])
        want = (routed + sh.astype(np.float64) * s).astype(np.float32)
        assert np.array_equal(out[t], want)
        assert abs(s - 1 / (1 + math.exp(-float(np.dot(lay["sh_gate_inp"].astype(np.float64), x[t].astype(np.float64)))))) < 1e-12


def _group_bruteforce(ids, weights):
    ntok, K = ids.shape
    uid = []
    for t in range(ntok):
        for k in range(K):
            if ids[t, k] not in uid:
                uid.append(int(ids[t, k]))
    pairs = {u: [] for u in uid}
    for t in range(ntok):
        for k in range(K):
            pairs[int(ids[t, k])].append((t, k))
    start, ptok, pw, tp = [0], [], [], np.zeros(ntok * K, np.uint32)
    for u in uid:
        for (t, k) in pairs[u]:
            tp[t * K + k] = len(ptok)
            ptok.append(t)
            pw.append(weights[t, k])
        start.append(len(ptok))
    return np.array(uid, np.uint32), np.array(start, np.uint32), np.array(ptok, np.uint32), np.array(pw, np.float32), tp


def test_grouping_bruteforce_and_invariants():
    rng = np.random.default_rng(8)
    for ntok, E, K in ((1, 512, 10), (2, 512, 10), (8, 512, 10), (5, 16, 4), (64, 64, 8)):
        l = synth.hot_logits(rng, ntok, E, n_hot=min(32, E // 2))
        ids = np.stack([orc.router_select(l[t], K)[0] for t in range(ntok)])
        w = np.stack([orc.router_select(l[t], K)[1] for t in range(ntok)])
        uid, start, ptok, pw, tp = orc.group_pairs(ids, w, E)
        b = _group_bruteforce(ids, w)
        for got, want in zip((uid, start, ptok, pw, tp), b):
            assert np.array_equal(got, want)
        P = ntok * K
        assert start[0] == 0 and start[-1] == P and np.all(np.diff(start.astype(np.int64)) > 0)
        assert sorted(tp) == list(range(P))
        assert np.all(np.bincount(ptok, minlength=ntok) == K)
        for u in range(len(uid)):
            seg = ptok[start[u]:start[u + 1]]
            assert np.all(np.diff(seg.astype(np.int64)) > 0)     # token order inside an expert, no token twice
    with pytest.raises(ValueError):
        orc.group_pairs(np.array([[600]], np.uint32), np.ones((1, 1), np.float32), 512)


def test_rmsnorm():
    x = np.arange(1, 9, dtype=np.float32)
    out = np.empty(8, np.float32)
    orc.lib().orc_rmsnorm(x.ctypes.data, None, 8, 1e-6, out.ctypes.data)
    assert np.allclose(out, x / math.sqrt(float((x.astype(np.float64) ** 2).mean()) + 1e-6), rtol=1e-7)


def test_routed_topk_against_the_compiled_reference(golden_dir, tmp_path):
    """orc_routed_topk / orc_expert_ffn_grid bit for bit against rl_native_reference_topk (native/redlite_native_reference.c:251-382) on the
    formats that function accepts: IQ2_XS, IQ1_M, IQ3_S and two mixed gate/up vs down pairings. This is the direct pin of the expert step
    (gate and up in double, SiLU * up in double, down rows on double activations, experts added in selection order)."""
    import sys
    import zlib
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from dwarfstar_red_lite_amd.gguf_writer import write_topk_case
    grids = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
    xs_grid, m_grid = (np.frombuffer(bytes.fromhex(grids[k]), np.int8) for k in ("iq2_xs", "iq1_m"))
    orc.set_codebooks(xs_grid, m_grid)
    g = json.load(open(os.path.join(golden_dir, "reference_topk.json")))
    assert len(g["cases"]) == 5
    for c in g["cases"]:
        spec = c["spec"]
        path = str(tmp_path / (spec["name"] + ".gguf"))
        cfg, lay = write_topk_case(path, spec)
        assert zlib.crc32(open(path, "rb").read()) == c["file_crc32"], spec["name"]      # the very bytes the reference read
        H, F = spec["hidden"], spec["ffn"]
        i = np.arange(H, dtype=np.int64)
        x = (((i * 17 + 3) % 61 - 30) / 32.0).astype(np.float32)
        L = orc.lib()
        p = lambda a: a.ctypes.data_as(orc.C.c_void_p)
        for call in c["calls"]:
            ids, w = np.asarray(call["ids"], np.uint32), unhex(call["weights_f32_hex"], np.float32)
            want = unhex(call["output_f64_hex"], np.float64)
            r0, n = call["row_start"], call["row_count"]
            full = np.zeros(H, np.float64)
            assert L.orc_routed_topk(spec["gate_up_type"], spec["down_type"], p(lay["gate"]), p(lay["up"]), p(lay["down"]), lay["gate"][0].nbytes,
                                     lay["up"][0].nbytes, lay["down"][0].nbytes, p(ids), p(w), ids.size, H, F, p(x), p(full))
            assert np.array_equal(full[r0:r0 + n].view(np.uint64), want.view(np.uint64)), (spec["name"], call["ids"])
            # the single-expert form on the same row window, weighted and added in selection order as the reference does
            acc = np.zeros(n, np.float64)
            for e, we in zip(ids, w):
                acc += np.float64(we) * orc.expert_ffn_grid(spec["gate_up_type"], spec["down_type"], lay["gate"][e], lay["up"][e], lay["down"][e], H, F, x,
                                                            xs_grid, m_grid, r0, n)
            assert np.array_equal(acc.view(np.uint64), want.view(np.uint64)), (spec["name"], "windowed")
