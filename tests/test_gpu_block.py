"""GPU parity of the layer with the steps around it (native/redlite_native_engine_cpu.c:418-427): residual add + RMS-norm in
front, residual add behind. Oracle: the same three steps composed on the CPU (float residual, double-precision norm, the
layer oracle, float add)."""
import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth
from gpu_common import REL_L2_TOL, rel_l2

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def oracle_block(cfg, lay, x, branch, w, eps):
    resid = (x + branch).astype(np.float32)
    normed = np.empty_like(resid)
    for t in range(x.shape[0]):
        orc.lib().orc_rmsnorm(resid[t].ctypes.data, w.ctypes.data, resid.shape[1], eps, normed[t].ctypes.data)
    ffn, ids, _, _ = orc.Layer(cfg, **lay).forward(normed, threads=8)
    return (resid + ffn.astype(np.float32)).astype(np.float32), normed, ids


@pytest.mark.parametrize("layout,ntok", [("iq2", 1), ("f2", 1), ("iq2", 3), ("f2", 2), ("f2", 6), ("iq2", 12), ("f2", 13), ("iq2", 24)])
def test_block_step_matches_cpu(layout, ntok):
    """one token (norm inside the router launch, residual in the down kernel) on both layouts, a small batch, a batch on the
    generic kernels, and a chunk (separate norm kernel, tiled router, MFMA tiles, residual in the combine kernel)"""
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(layout=layout)
    lay = synth.make_layer(123, cfg)
    m = ResidentMoe(cfg, n_layer=1, max_tokens=ntok)
    m.load_layer(0, lay)
    rng = np.random.default_rng(1000 + ntok)
    H = cfg["hidden"]
    x = (3.0 * rng.standard_normal((ntok, H))).astype(np.float32)             # not normalised: the step has to do it
    branch = (0.5 * rng.standard_normal((ntok, H))).astype(np.float32)
    w = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    eps = 1e-6
    want, normed, cids = oracle_block(cfg, lay, x, branch, w, eps)
    xg = torch.from_numpy(x).cuda()
    got = m.forward_block(0, xg, torch.from_numpy(branch).cuda(), torch.from_numpy(w).cuda(), eps).cpu().numpy()
    gids, _, _ = m.last_route(ntok)
    assert np.array_equal(gids, cids)
    # the FFN part alone (output minus the exact float residual) meets the usual bar, so does the whole
    resid = (x + branch).astype(np.float32)
    for t in range(ntok):
        assert rel_l2(got[t] - resid[t], want[t] - resid[t]) <= REL_L2_TOL, (layout, ntok, t)
        assert rel_l2(got[t], want[t]) <= REL_L2_TOL
    # in place: x_out may be x
    got2 = m.forward_block(0, xg, torch.from_numpy(branch).cuda(), torch.from_numpy(w).cuda(), eps, out=xg).cpu().numpy()
    assert np.array_equal(got2, got)
    m.close()
