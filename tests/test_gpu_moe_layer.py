"""GPU parity of the resident MoE layer (router -> top-k -> experts -> shared -> combine) against the CPU oracle."""
import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth
from gpu_common import REL_L2_TOL, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def ids_match_up_to_ties(gpu_ids, cpu_ids, cpu_logits, tol=1e-6):
    """identical ids, except where two logits tie within tol (then the sets may differ by the tied experts)"""
    if np.array_equal(gpu_ids, cpu_ids):
        return True
    diff = set(gpu_ids.tolist()) ^ set(cpu_ids.tolist())
    if not diff:                                           # same set, order swapped between near-tied logits
        swapped = [k for k in range(len(cpu_ids)) if gpu_ids[k] != cpu_ids[k]]
        return all(abs(cpu_logits[gpu_ids[k]] - cpu_logits[cpu_ids[k]]) <= tol for k in swapped)
    vals = sorted(cpu_logits[list(diff)])
    return vals[-1] - vals[0] <= tol


@pytest.mark.parametrize("layout", ["iq2", "f2"])
@pytest.mark.parametrize("shape", [(512, 256, 16, 4), (2048, 512, 64, 10)])
def test_layer_single_token(layout, shape):
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    H, F, E, K = shape
    cfg = synth.layer_config(hidden=H, ffn=F, n_expert=E, top_k=K, layout=layout)
    m = ResidentMoe(cfg, n_layer=2, max_tokens=1)
    layers = [synth.make_layer(40 + l, cfg) for l in range(2)]
    for l in range(2):
        m.load_layer(l, layers[l])
    xs = synth.normed_x(np.random.default_rng(5), 3, H)
    for l in range(2):
        ref = orc.Layer(cfg, **layers[l])
        # resident weights dequantise bit-exactly from the layout the kernels read
        for e, which in ((0, 0), (E - 1, 1), (E // 2, 2), (E, 0), (E, 2)):
            key = ("sh_" if e == E else "") + ("gate", "up", "down")[which]
            raw = layers[l][key] if e == E else layers[l][key][e]
            t = cfg[("sh_" if e == E else "") + ("gate_up_type" if which < 2 else "down_type")]
            want = orc.dequant_rows(t, raw.reshape(-1), H if which < 2 else F)
            got = m.dequant_resident(l, e, which).cpu().numpy()
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
            if which == 2 and (layout == "iq2" or e != E):   # and from the column-sliced copy (all of iq2; the routed IQ3_S matrices of f2)
                got = m.dequant_resident(l, e, 4).cpu().numpy()
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        for t in range(3):
            out = m.forward(l, torch.from_numpy(xs[t:t + 1]).cuda()).cpu().numpy()[0]
            gids, gw, glog = m.last_route(1)
            want, cids, cw, clog = ref.forward(xs[t], threads=8)
            assert rel_l2(glog[0], clog[0]) <= REL_L2_TOL
            assert ids_match_up_to_ties(gids[0], cids[0], clog[0])
            assert np.all(np.abs(gw[0] - cw[0]) <= 1e-5 + 1e-3 * cw[0])
            assert rel_l2(out, want[0]) <= REL_L2_TOL, (layout, shape, l, t)
    m.close()


def test_layer_full_size_config0():
    """The benchmark layer at its real shape: hidden 2048, 512 experts, top-10 + shared, ffn 512, all IQ2_XXS, F32 router."""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config()
    m = ResidentMoe(cfg, n_layer=1, max_tokens=1)
    lay = synth.make_layer(2024, cfg)
    m.load_layer(0, lay)
    ref = orc.Layer(cfg, **lay)
    xs = synth.normed_x(np.random.default_rng(6), 2, 2048)
    for t in range(2):
        out = m.forward(0, torch.from_numpy(xs[t:t + 1]).cuda()).cpu().numpy()[0]
        gids, gw, glog = m.last_route(1)
        want, cids, cw, clog = ref.forward(xs[t], threads=16)
        assert ids_match_up_to_ties(gids[0], cids[0], clog[0])
        assert rel_l2(out, want[0]) <= REL_L2_TOL
        # route / experts pieces give the same result as forward
        x = torch.from_numpy(xs[t:t + 1]).cuda()
        ids, w, logits = m.route(0, x)
        out2 = m.experts(0, x, ids, w).cpu().numpy()[0]
        # the same kernels as forward() with the selection as a launch of its own: same terms, same order of addition
        assert np.array_equal(out2, out)
    m.close()
