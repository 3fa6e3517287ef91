"""The reference's own FFN acceptance harness (`redlite-ffn parity`, native/redlite_native_ffn_parity_cli.c:93-332) run against the
resident-layer path on seeded synthetic blocks of the benchmark shape: its deterministic input (:45), its refusal conditions on the router
(:205-220) and its per-row gate on the expert outputs (:77-91, :273-284), with the CPU oracle standing where the reference's CPU path
stands."""
import json
import os

import numpy as np
import pytest

import oracle_lib as orc
from dwarfstar_red_lite_amd import synth

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

LOGIT_ABS, WEIGHT_ABS = 1e-3, 1e-5          # native/redlite_native_ffn_parity_cli.c:216-220


def row_gate(gpu, cpu):
    """|gpu - cpu| <= 1e-3 + 1e-4 |cpu| for every output row (native/redlite_native_ffn_parity_cli.c:77-91)"""
    gpu, cpu = np.asarray(gpu, np.float64), np.asarray(cpu, np.float64)
    return bool(np.all(np.abs(gpu - cpu) <= 1e-3 + 1e-4 * np.abs(cpu)))


@pytest.mark.parametrize("layout", ["iq2", "f2", "xs", "m"])
def test_reference_acceptance_harness(layout, golden_dir):
    from dwarfstar_red_lite_amd import moe as moe_api
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    if layout in ("xs", "m"):
        g = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
        grids = [np.frombuffer(bytes.fromhex(g[k]), np.int8) for k in ("iq2_xs", "iq1_m")]
        moe_api.set_codebooks(*grids)
        orc.set_codebooks(*grids)
    cfg = synth.layer_config(layout=layout)
    H, F, K = cfg["hidden"], cfg["ffn"], cfg["top_k"]
    lays = [synth.make_layer(500 + l, cfg) for l in range(2)]
    m = ResidentMoe(cfg, n_layer=2, max_tokens=1)
    for l, lay in enumerate(lays):
        m.load_layer(l, lay)
    x = np.array([((i * 17 + 3) % 61 - 30) / 32.0 for i in range(H)], np.float32)          # native/redlite_native_ffn_parity_cli.c:45
    xd = torch.from_numpy(x).cuda()
    for l, lay in enumerate(lays):
        want, cids, cw, clog = orc.Layer(cfg, **lay).forward(x[None], threads=8)
        # router: logits, selection and weights on both sides; any disagreement refuses the comparison
        gids, gw, glog = m.route(l, xd)
        gids, gw, glog = gids.cpu().numpy(), gw.cpu().numpy(), glog.cpu().numpy()
        assert np.max(np.abs(glog[0].astype(np.float64) - clog[0])) <= LOGIT_ABS, (layout, l)
        assert np.array_equal(gids[0].astype(np.uint32), cids[0]), (layout, l)
        assert np.max(np.abs(gw[0].astype(np.float64) - cw[0])) <= WEIGHT_ABS, (layout, l)
        # the layer end to end (its own router), then the routed experts with the CPU's routing: every row inside the gate
        got = m.forward(l, xd).cpu().numpy()[0]
        assert row_gate(got, want[0]), (layout, l)
        got = m.experts(l, xd, torch.from_numpy(cids.astype(np.int32)).cuda(), torch.from_numpy(cw).cuda()).cpu().numpy()[0]
        assert row_gate(got, want[0]), (layout, l)
        # the shared expert alone (all router weights zero): the rows and, through them, the scalar gate
        sh, s = orc.shared_expert(cfg["sh_gate_up_type"], cfg["sh_down_type"], lay["sh_gate"], lay["sh_up"], lay["sh_down"],
                                  lay["sh_gate_inp"], H, F, x, threads=8)
        got_sh = m.experts(l, xd, torch.from_numpy(cids.astype(np.int32)).cuda(), torch.zeros((1, K), dtype=torch.float32).cuda()).cpu().numpy()[0]
        assert row_gate(got_sh, sh.astype(np.float64) * s), (layout, l)
        # ... and the routed part by difference
        assert row_gate(got.astype(np.float64) - got_sh, want[0].astype(np.float64) - sh.astype(np.float64) * s), (layout, l)
    m.close()
