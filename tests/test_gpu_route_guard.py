"""Routing handed in by a caller is untrusted: an expert id beyond the layer's experts must not be turned into an address, and both
contract violations (id out of range, an expert named twice by one token) must be reported by the next last_route(). The kernels
clamp such ids before they index anything, so these calls are ordinary, fault-free launches."""
import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth
from dwarfstar_red_lite_amd._lib import RedHipError
from gpu_common import REL_L2_TOL, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def test_pair_sort_of_a_large_chunk_reports_the_same_way():
    """More than 512 tokens: the pair sort runs on many workgroups (spans of 64 tokens); an id out of range in one span and an expert named
    twice in another are clamped / reported, the sorted arrays are those of the clamped routing."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    E, K, ntok = 64, 4, 700
    cfg = synth.layer_config(hidden=512, ffn=256, n_expert=E, top_k=K, layout="iq2")
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    rng = np.random.default_rng(3)
    ids = np.stack([rng.choice(E - 1, size=K, replace=False) for _ in range(ntok)]).astype(np.uint32)      # (expert E - 1 unused: the clamp lands there)
    w = rng.random((ntok, K)).astype(np.float32)
    got = m.group(torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda())
    m.last_route(1)                                          # no report
    for a, b in zip(got, orc.group_pairs(ids, w, E)):
        assert np.array_equal(a.cpu().numpy().view(b.dtype), b)
    bad = ids.copy()
    bad[650, 2] = E + 77
    got = m.group(torch.from_numpy(bad.astype(np.int32)).cuda(), torch.from_numpy(w).cuda())
    with pytest.raises(RedHipError, match="n_expert"):
        m.last_route(1)
    clamped = bad.copy()
    clamped[650, 2] = E - 1
    for a, b in zip(got, orc.group_pairs(clamped, w, E)):
        assert np.array_equal(a.cpu().numpy().view(b.dtype), b)
    dup = ids.copy()
    dup[130, 3] = dup[130, 1]
    m.group(torch.from_numpy(dup.astype(np.int32)).cuda(), torch.from_numpy(w).cuda())
    with pytest.raises(RedHipError, match="twice"):
        m.last_route(1)
    got = m.group(torch.from_numpy(ids.astype(np.int32)).cuda(), torch.from_numpy(w).cuda())               # the scratch is ready for the next chunk
    m.last_route(1)
    for a, b in zip(got, orc.group_pairs(ids, w, E)):
        assert np.array_equal(a.cpu().numpy().view(b.dtype), b)
    m.close()


@pytest.mark.parametrize("layout,shape", [("iq2", (512, 256, 32, 4)), ("f2", (512, 256, 32, 4)), ("f2", (768, 256, 24, 3))])
def test_out_of_range_and_repeated_ids_are_clamped_and_reported(layout, shape):
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_batch import oracle_tokens
    H, F, E, K = shape                                       # (768: no packed path, the generic kernels)
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout=layout)
    lay = synth.make_layer(321, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=40)
    m.load_layer(0, lay)
    rng = np.random.default_rng(2)
    for ntok in (1, 3, 40):                                  # one token, a grouped small batch, a chunk
        x = synth.normed_x(rng, ntok, H)
        ids = np.stack([rng.choice(E, size=K, replace=False) for _ in range(ntok)]).astype(np.uint32)
        w = rng.random((ntok, K)).astype(np.float32) + 0.1
        w /= w.sum(axis=1, keepdims=True)
        xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
        # a valid call: no report, the oracle's result
        got = m.experts(0, xd, torch.from_numpy(ids.astype(np.int32)).cuda(), wd).cpu().numpy()
        m.last_route(ntok)
        want = oracle_tokens(cfg, lay, x, ids, w)
        assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL
        # an id far beyond the experts: clamped (computes expert E - 1 in its place), reported once
        bad = ids.copy()
        bad[ntok - 1, K - 1] = E + 1000 if (E - 1) not in ids[ntok - 1] else bad[ntok - 1, K - 1]
        if bad[ntok - 1, K - 1] >= E:
            got = m.experts(0, xd, torch.from_numpy(bad.astype(np.int64).astype(np.int32)).cuda(), wd).cpu().numpy()
            with pytest.raises(RedHipError, match="n_expert"):
                m.last_route(ntok)
            clamped = bad.copy()
            clamped[ntok - 1, K - 1] = E - 1
            want = oracle_tokens(cfg, lay, x, clamped, w)
            assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL
            m.last_route(ntok)                               # the report was cleared
        if ntok > 1:                                         # a token that names an expert twice: reported by the pair sort
            dup = ids.copy()
            dup[0, 1] = dup[0, 0]
            m.experts(0, xd, torch.from_numpy(dup.astype(np.int32)).cuda(), wd)
            with pytest.raises(RedHipError, match="twice"):
                m.last_route(ntok)
    # the stand-alone pair sort reports the same way
    dup = np.stack([rng.choice(E, size=K, replace=False) for _ in range(20)]).astype(np.uint32)
    dup[7, 2] = dup[7, 0]
    dup[3, 1] = E + 5
    m.group(torch.from_numpy(dup.astype(np.int32)).cuda(), torch.ones((20, K), dtype=torch.float32, device="cuda"))
    with pytest.raises(RedHipError, match="n_expert.*twice"):
        m.last_route(1)
    m.close()


@pytest.mark.parametrize("layout", ["iq2", "f2"])
def test_worst_case_repeats_stay_inside_the_pair_arrays(layout):
    """The fullest small batch (8 tokens x top_k 15 = 120 of at most 128 pairs) whose first token names one expert fifteen times, an expert
    that every other token names too: the repeated pairs take no place of their own in the group arrays (before, each counted the whole
    group again and the pair / pass lists ran past their ends into the neighbouring scratch). Reported, and the next valid call on the
    same handle is right."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from test_gpu_moe_batch import oracle_tokens
    H, F, E, K, ntok = 512, 256, 32, 15, 8
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout=layout)
    lay = synth.make_layer(99, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    rng = np.random.default_rng(12)
    x = synth.normed_x(rng, ntok, H)
    ids = np.stack([np.concatenate([[5], rng.choice(np.setdiff1d(np.arange(E), [5]), size=K - 1, replace=False)]) for _ in range(ntok)]).astype(np.uint32)
    w = rng.random((ntok, K)).astype(np.float32) + 0.1
    w /= w.sum(axis=1, keepdims=True)
    xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    for bad_tok in (0, 3, ntok - 1):
        bad = ids.copy()
        bad[bad_tok, :] = 5
        m.experts(0, xd, torch.from_numpy(bad.astype(np.int32)).cuda(), wd)
        with pytest.raises(RedHipError, match="twice"):
            m.last_route(ntok)
        got = m.experts(0, xd, torch.from_numpy(ids.astype(np.int32)).cuda(), wd).cpu().numpy()
        m.last_route(ntok)
        want = oracle_tokens(cfg, lay, x, ids, w)
        assert max(rel_l2(got[t], want[t]) for t in range(ntok)) <= REL_L2_TOL
    m.close()


def test_top_k_limits_are_settled_at_create():
    """top_k = 16 (17 slots with the shared expert) and top_k = 1 run on the generic kernels instead of failing mid-forward"""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    for layout, K in (("iq2", 16), ("f2", 1), ("f2", 16)):
        cfg = synth.layer_config(hidden=512, ffn=256, n_expert=32, top_k=K, layout=layout)
        lay = synth.make_layer(77 + K, cfg)
        m = ResidentMoe(cfg, n_layer=1, max_tokens=4)
        m.load_layer(0, lay)
        x = synth.normed_x(np.random.default_rng(K), 3, 512)
        ref = orc.Layer(cfg, **lay)
        for ntok in (1, 3):
            out = m.forward(0, torch.from_numpy(x[:ntok].copy()).cuda()).cpu().numpy()
            gids, _, _ = m.last_route(ntok)
            want, cids, _, _ = ref.forward(x[:ntok], threads=4)
            assert np.array_equal(gids, cids)
            assert max(rel_l2(out[t], want[t]) for t in range(ntok)) <= REL_L2_TOL, (layout, K, ntok)
            ids = torch.from_numpy(cids.astype(np.int32)).cuda()
            _, cw, _ = m.last_route(ntok)
            out2 = m.experts(0, torch.from_numpy(x[:ntok].copy()).cuda(), ids, torch.from_numpy(cw).cuda()).cpu().numpy()
            assert max(rel_l2(out2[t], want[t]) for t in range(ntok)) <= REL_L2_TOL, (layout, K, ntok)
        m.close()
