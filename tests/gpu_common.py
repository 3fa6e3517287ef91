"""Shared helpers of the GPU parity tests."""
import numpy as np

T_F32, T_Q6K, T_IQ2, T_IQ3 = 0, 14, 16, 21

# parity tolerance: GEMV / FFN outputs within 1e-3 relative L2 of the double-accumulating CPU path
REL_L2_TOL = 1e-3


def rel_l2(got, want):
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-300))


def edge_rows(t, ncols):
    """rows with subnormal / zero / negative / maximal d and all-zero / all-one payloads"""
    from dwarfstar_red_lite_amd import synth
    rng = np.random.default_rng(1234 + t)
    rows = synth.quant_rows(rng, t, 8, ncols)
    bb, off = synth.BLOCK_BYTES[t], synth.D_OFFSET[t]
    r = rows.reshape(8, -1, bb)
    r[1, :, off], r[1, :, off + 1] = 0x01, 0x00          # smallest subnormal
    r[2, :, off], r[2, :, off + 1] = 0xFF, 0x03          # largest subnormal
    r[3, :, off], r[3, :, off + 1] = 0x00, 0x00          # zero
    r[4, :, off + 1] |= 0x80                             # negative d
    r[5, :, :] = 0
    r[5, :, off + 1] = 0x3C
    r[6, :, :] = 0xFF
    r[6, :, off], r[6, :, off + 1] = 0x00, 0x3C
    r[7, :, off], r[7, :, off + 1] = 0xFF, 0x7B          # 65504
    return rows
