"""GPU parity of the kernels over raw GGUF rows, through the C ABI, against the CPU oracle and the golden vectors.
Shaped like the reference's model-free kernel self-test (native/redmetal_engine_selftest.m:64-118,159-210)."""
import json
import os

import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth
from gpu_common import REL_L2_TOL, T_F32, T_IQ2, T_IQ3, T_Q6K, edge_rows, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def dev(a):
    return torch.from_numpy(np.array(a, copy=True)).cuda()


@pytest.mark.parametrize("t", [T_IQ2, T_IQ3, T_Q6K])
def test_dequant_bit_exact(t):
    from dwarfstar_red_lite_amd import moe
    rng = np.random.default_rng(100 + t)
    for ncols in (256, 512, 2048):
        rows = np.concatenate([synth.quant_rows(rng, t, 37, ncols), edge_rows(t, ncols)])
        if t == T_Q6K:
            rows = np.concatenate([rows, synth.quant_rows(rng, t, 8, ncols, d_range=(1e-5, 3e-5))])   # subnormal d
        got = moe.dequant_rows(t, dev(rows), ncols).cpu().numpy()
        want = orc.dequant_rows(t, rows, ncols)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (t, ncols)


def test_dequant_golden(golden_dir):
    from dwarfstar_red_lite_amd import moe
    g = json.load(open(os.path.join(golden_dir, "quant_rows.json")))
    n = 0
    for c in g["cases"]:
        if c["type"] == T_F32:
            continue
        row = np.frombuffer(bytes.fromhex(c["row"]), np.uint8).reshape(1, -1)
        got = moe.dequant_rows(c["type"], dev(row), c["ncols"]).cpu().numpy()
        assert np.array_equal(got.view(np.uint32).ravel(), np.frombuffer(bytes.fromhex(c["dequant"]), np.uint32))
        n += 1
    assert n >= 30


@pytest.mark.parametrize("t", [T_IQ2, T_IQ3, T_Q6K, T_F32])
def test_gemv_rows(t):
    from dwarfstar_red_lite_amd import moe
    rng = np.random.default_rng(200 + t)
    for ncols in (256, 512, 1024, 2048):
        nrows = 37
        if t == T_F32:
            w = (0.02 * rng.standard_normal((nrows, ncols))).astype(np.float32).view(np.uint8).reshape(nrows, -1)
        else:
            w = synth.quant_rows(rng, t, nrows, ncols)
        x = rng.standard_normal(ncols).astype(np.float32)
        want = np.array([orc.row_dot(t, w[r], x) for r in range(nrows)])
        got = moe.gemv_rows(t, dev(w), ncols, dev(x)).cpu().numpy()
        # the reference self-test's metric: error relative to sum |w x| of the row
        deq = orc.dequant_rows(t, w, ncols) if t != T_F32 else w.view(np.float32).reshape(nrows, ncols)
        scale = np.abs(deq.astype(np.float64) * x).sum(axis=1)
        assert np.max(np.abs(got - want) / scale) <= 2e-5, (t, ncols)
        assert rel_l2(got, want) <= REL_L2_TOL
        part = moe.gemv_rows(t, dev(w), ncols, dev(x), row_start=5, row_count=9).cpu().numpy()
        assert np.array_equal(part, got[5:14])


def test_gemv_golden(golden_dir):
    from dwarfstar_red_lite_amd import moe
    g = json.load(open(os.path.join(golden_dir, "quant_rows.json")))
    for c in g["cases"]:
        row = np.frombuffer(bytes.fromhex(c["row"]), np.uint8).reshape(1, -1)
        x = np.frombuffer(bytes.fromhex(c["x"]), np.float32)
        want = np.frombuffer(bytes.fromhex(c["dot"]), np.float64)[0]
        got = float(moe.gemv_rows(c["type"], dev(row), c["ncols"], dev(x)).cpu().numpy()[0])
        if c["type"] == T_F32:
            scale = float(np.abs(row.view(np.float32).astype(np.float64) * x).sum())
        else:
            scale = float(np.abs(np.frombuffer(bytes.fromhex(c["dequant"]), np.float32).astype(np.float64) * x).sum())
        assert abs(got - want) <= 2e-5 * scale + 1e-30, (c["type"], c["ncols"], c["fill"], got, want)


def test_router_select_golden(golden_dir):
    from dwarfstar_red_lite_amd import redmetal_quant as rq
    g = json.load(open(os.path.join(golden_dir, "router_select.json")))
    for c in g["cases"]:
        logits = np.frombuffer(bytes.fromhex(c["logits"]), np.float32)
        ids, w, probs = rq.router_select(logits, c["top_k"], want_probs=True)
        want_w = np.frombuffer(bytes.fromhex(c["weights"]), np.float32)
        want_p = np.frombuffer(bytes.fromhex(c["probs"]), np.float32)
        assert list(ids) == c["ids"]
        assert np.all(np.abs(w - want_w) <= 1e-6 + 1e-5 * want_w)
        assert np.all(np.abs(probs - want_p) <= 1e-7 + 1e-5 * want_p)
    with pytest.raises(Exception):
        rq.router_select(np.array([np.nan, 1.0], np.float32), 1)
    with pytest.raises(Exception):
        rq.router_select(np.array([0.0, 1.0], np.float32), 3)


def test_router_select_random_and_ties():
    """64 cases incl. exact ties: ids identical to the CPU selection, weights within 1e-6 + 1e-5 w."""
    from dwarfstar_red_lite_amd import redmetal_quant as rq
    rng = np.random.default_rng(7)
    for case in range(64):
        E = (512, 512, 64, 1000)[case % 4]
        K = (10, 10, 4, 16)[case % 4]
        l = rng.standard_normal(E).astype(np.float32) * np.float32(1 + case % 5)
        if case % 2:
            l[rng.integers(0, E, 12)] = l[3]
        ids, w = rq.router_select(l, K)
        ci, cw = orc.router_select(l, K)
        assert np.array_equal(ids, ci), case
        assert np.all(np.abs(w - cw) <= 1e-6 + 1e-5 * cw)


def test_router_select_adversarial(golden_dir):
    """The selection must pick what the CPU's argmax loop over probabilities picks, also where different logits share a probability:
    logits one to a few ulps apart around the K-th place (the lower index a little smaller, so that logit order and the CPU's order
    differ whenever the probabilities collapse), tight clusters, logits spread until the tail underflows, all equal, and the golden
    cases of the reference (here without the probabilities output)."""
    from dwarfstar_red_lite_amd import redmetal_quant as rq
    rng = np.random.default_rng(2024)
    cases = []
    for c in json.load(open(os.path.join(golden_dir, "router_select.json")))["cases"]:
        cases.append((np.frombuffer(bytes.fromhex(c["logits"]), np.float32).copy(), c["top_k"]))
    for case in range(96):
        E, K = (512, 10) if case % 3 else (64, 4)
        l = (rng.standard_normal(E) * (0.9, 3.0, 40.0, 300.0)[case % 4]).astype(np.float32)
        order = np.argsort(-l)
        kind = case % 6
        if kind == 0:            # the K-th and (K+1)-th one ulp apart, the smaller logit at the lower index
            hi, lo = sorted((int(order[K - 1]), int(order[K])))
            l[hi] = l[order[K - 1]]
            l[lo] = np.nextafter(l[hi], np.float32(-np.inf))
        elif kind == 1:          # a ladder of ulps through the top K + 4
            base = l[order[0]]
            for r, i in enumerate(sorted(int(j) for j in order[:K + 4])):
                v = base
                for _ in range(3 * r):
                    v = np.nextafter(v, np.float32(-np.inf))
                l[i] = v
        elif kind == 2:          # twenty logits within 1e-6 of each other at the top
            top = order[:20]
            l[top] = l[order[0]] + (rng.random(20) * 1e-6).astype(np.float32)
        elif kind == 3:          # exact ties across the boundary
            l[order[K - 3:K + 5]] = l[order[K - 1]]
        elif kind == 4:          # fewer than K probabilities above zero: the tail is picked by index
            l = (rng.standard_normal(E) * 400.0).astype(np.float32)
        # kind 5: plain random
        cases.append((l, K))
    cases.append((np.zeros(512, np.float32), 10))
    cases.append((np.full(512, -3.25, np.float32), 10))
    for n, (l, K) in enumerate(cases):
        ids, w = rq.router_select(l, K)
        ci, cw = orc.router_select(l, K)
        assert np.array_equal(ids, ci), (n, ids, ci)
        assert np.all(np.abs(w - cw) <= 1e-6 + 1e-5 * cw), n


def test_grouping_matches_host_sort():
    from dwarfstar_red_lite_amd import moe
    cfg = synth.layer_config(hidden=256, ffn=256, n_expert=512, top_k=10)
    m = moe.ResidentMoe(cfg, n_layer=1, max_tokens=2048)
    rng = np.random.default_rng(12)
    for ntok in (1, 2, 3, 8, 33, 512, 513, 1024, 1600, 2048):          # (more than 512 tokens: the pair sort places block by block)
        l = synth.hot_logits(rng, ntok, 512)
        sel = [orc.router_select(l[t], 10) for t in range(ntok)]
        ids = np.stack([s[0] for s in sel])
        w = np.stack([s[1] for s in sel])
        want = orc.group_pairs(ids, w, 512)
        got = m.group(dev(ids.astype(np.int32)), dev(w))
        for a, b in zip(got, want):
            assert np.array_equal(a.cpu().numpy().view(b.dtype), b), ntok
    for ntok in (512, 2048):
        ids = synth.zipf_topk(rng, ntok, 512, 10)
        w = rng.random((ntok, 10)).astype(np.float32)
        want = orc.group_pairs(ids, w, 512)
        got = m.group(dev(ids.astype(np.int32)), dev(w))
        for a, b in zip(got, want):
            assert np.array_equal(a.cpu().numpy().view(b.dtype), b), ntok
    m.close()
    # the widest expert table (1024) with a partial last block of tokens
    cfg = synth.layer_config(hidden=256, ffn=256, n_expert=1024, top_k=4)
    m = moe.ResidentMoe(cfg, n_layer=1, max_tokens=1500)
    ids = synth.zipf_topk(rng, 1500, 1024, 4)
    w = rng.random((1500, 4)).astype(np.float32)
    want = orc.group_pairs(ids, w, 1024)
    got = m.group(dev(ids.astype(np.int32)), dev(w))
    for a, b in zip(got, want):
        assert np.array_equal(a.cpu().numpy().view(b.dtype), b)
    m.close()
