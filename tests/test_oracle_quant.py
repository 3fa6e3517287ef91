"""The CPU oracle against the reference's golden vectors and known answers (no GPU).

Golden fixtures come from the reference's own C (tests/golden/make_golden.c). Known answers are the ones in
the reference's model-free tests: native/redlite_native_shared_exec_offline_test.c:18-55,
native/redlite_native_quant_cpu.c:364-393, tests/test_redmetal.py:25-29.
"""
import json
import os
import struct

import numpy as np
import pytest

import oracle_lib as orc

T_F32, T_Q6K, T_IQ2, T_IQ3 = 0, 14, 16, 21


def unhex(s, dtype):
    return np.frombuffer(bytes.fromhex(s), dtype=dtype).copy()


def test_f16_exhaustive(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "f16.json")))
    mine = np.empty(65536, np.float32)
    orc.lib().orc_f16_all(mine.ctypes.data_as(orc.C.c_void_p))
    assert "%08x" % orc.lib().orc_crc32(mine.ctypes.data, mine.nbytes) == g["crc32_of_f32_le"]
    for k, v in g["spot"].items():
        assert "%08x" % mine[int(k, 16)].view(np.uint32) == v
    # independent of the reference: numpy's IEEE half conversion, all non-NaN patterns
    ref = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    ok = ~np.isnan(ref)
    assert np.array_equal(mine[ok].view(np.uint32), ref[ok].view(np.uint32))
    assert mine[1] == 2.0 ** -24


def test_codebooks():
    L = orc.lib()
    g2 = np.ctypeslib.as_array(L.orc_iq2xxs_grid(), (2048,))
    g3 = np.ctypeslib.as_array(L.orc_iq3s_grid(), (512,))
    assert "%08x" % L.orc_crc32(g2.ctypes.data, 2048) == "9924ff02"
    assert "%08x" % L.orc_crc32(g3.ctypes.data, 2048) == "f576e4f3"
    assert set(np.unique(g2)) == {8, 25, 43}
    assert list(g2[:8]) == [8] * 8 and list(g2[8:16]) == [43] + [8] * 7
    assert list(g2[255 * 8:]) == [8, 25, 8, 8, 25, 43, 43, 43]
    # spot values the reference's IQ3 selftest checks (native/redlite_native_iq3.c:398)
    assert g3[0] == 0x01010101 and g3[511] == 0x0f0f0101 and g3[1] == 0x01010103 and g3[256] == 0x05090507
    b = g3.view(np.uint8)
    assert np.all(b % 2 == 1) and b.max() == 15 and b.min() == 1


def test_row_sizes():
    assert orc.row_bytes(T_Q6K, 256) == 210 and orc.row_bytes(T_IQ2, 256) == 66 and orc.row_bytes(T_IQ3, 2048) == 880
    assert orc.row_bytes(T_IQ2, 2048) == 528 and orc.row_bytes(T_IQ2, 512) == 132 and orc.row_bytes(T_F32, 2048) == 8192
    assert orc.row_bytes(T_IQ2, 100) == 0 and orc.row_bytes(18, 256) == 0


def test_golden_rows(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "quant_rows.json")))
    seen = set()
    for c in g["cases"]:
        t, n = c["type"], c["ncols"]
        row = unhex(c["row"], np.uint8)
        x = unhex(c["x"], np.float32)
        want = struct.unpack("<d", bytes.fromhex(c["dot"]))[0]
        got = orc.row_dot(t, row, x)
        assert got == want, (t, n, c["fill"], got, want)          # same order of double operations: bit-equal
        if t != T_F32:
            w = orc.dequant_rows(t, row, n)[0]
            assert np.array_equal(w.view(np.uint32), unhex(c["dequant"], np.uint32)), (t, n, c["fill"])
            assert "%08x" % orc.lib().orc_crc32(w.ctypes.data, w.nbytes) == c["dequant_crc32"]
            # the digest check of the reference's offline test: double dot of the dequantised row agrees
            brute = float(np.dot(w.astype(np.float64), x.astype(np.float64)))
            assert abs(brute - want) <= 1e-9 * max(1.0, np.abs(w.astype(np.float64) * x).sum())
        if "dot_d" in c:
            xd = unhex(c["xd"], np.float64)
            assert orc.row_dot(t, row, xd) == struct.unpack("<d", bytes.fromhex(c["dot_d"]))[0]
        seen.add((t, c["fill"]))
    assert {(16, 0), (21, 0), (14, 0), (0, 0), (16, 3), (21, 3), (14, 3)} <= seen


def test_appendix_rows():
    """Two-block rows with formula bytes; expected values were produced by the compiled reference."""
    want = {
        T_IQ2: ("d10d4eca", "877d1af2", -12.7415771484375, [-0.923828125, 0.923828125, 0.537109375, -0.537109375], -1.25976562, 0.421875),
        T_IQ3: ("99a6997b", "30688e0b", 8.427734375, [-1.265625, 3.796875, -5.484375, -2.953125], 3.515625, -1.421875),
        T_Q6K: ("9c223205", "47004699", 484.328125, [-22.359375, 26.5, 9.109375, -8.28125], -0.9375, -28.4375),
    }
    x = np.array([((i * 7 + 3) % 31 - 15) / 16.0 for i in range(512)], np.float32)
    for t, (crc_row, crc_w, dot, w03, w255, w511) in want.items():
        bb = orc.lib().orc_block_bytes(t)
        row = np.zeros(2 * bb, np.uint8)
        for b in range(2):
            for i in range(bb):
                row[b * bb + i] = (i * 37 + 11 + b * 101) & 255
            off = 208 if t == T_Q6K else 0
            row[b * bb + off], row[b * bb + off + 1] = 0x00, 0x24
        assert "%08x" % orc.lib().orc_crc32(row.ctypes.data, row.nbytes) == crc_row
        w = orc.dequant_rows(t, row, 512)[0]
        assert "%08x" % orc.lib().orc_crc32(w.ctypes.data, w.nbytes) == crc_w
        assert list(w[:4]) == w03 and abs(w[255] - w255) < 1e-7 and w[511] == w511
        assert orc.row_dot(t, row, x) == dot


def test_known_answer_blocks():
    ones = np.ones(256, np.float32)
    q6 = np.zeros(210, np.uint8)
    q6[:128] = 0x11
    q6[128:192] = 0xAA
    q6[192:208] = 1
    q6[208], q6[209] = 0x00, 0x3C
    assert orc.row_dot(T_Q6K, q6, ones) == 256.0
    assert np.all(orc.dequant_rows(T_Q6K, q6, 256) == 1.0)
    q6[208], q6[209] = 0x01, 0x00                      # smallest fp16 subnormal
    assert abs(orc.row_dot(T_Q6K, q6, ones) - 2.0 ** -16) < 1e-12
    q6z = np.zeros(210, np.uint8)
    q6z[192:208] = 1
    q6z[209] = 0x3C
    assert orc.row_dot(T_Q6K, q6z, ones) == -8192.0
    assert np.all(orc.dequant_rows(T_Q6K, q6z, 256) == -32.0)
    iq2 = np.zeros(66, np.uint8)
    iq2[1] = 0x3C
    assert orc.row_dot(T_IQ2, iq2, ones) == 256.0
    x = np.array([((i * 17 + 3) % 61 - 30) / 32.0 for i in range(256)], np.float32)
    assert abs(orc.row_dot(T_IQ2, iq2, x) - float(x.astype(np.float64).sum())) < 1e-9


def test_iq2xxs_sign_parity_and_exactness():
    rng = np.random.default_rng(5)
    from dwarfstar_red_lite_amd import synth
    rows = synth.quant_rows(rng, T_IQ2, 8, 512)
    w = orc.dequant_rows(T_IQ2, rows, 512)
    neg = (w < 0).reshape(8, 64, 8).sum(axis=2)
    assert np.all(neg % 2 == 0)                         # each group of 8 holds an even number of minus signs
    mags = np.abs(w).reshape(8, 2, 8, 32)
    # |w| / db must be a grid magnitude: ratios within one 32-group are ratios of {8,25,43}
    r = mags / mags.min(axis=3, keepdims=True)
    allowed = np.array([1.0, 25 / 8, 43 / 8, 43 / 25, 25 / 25])
    assert np.all(np.min(np.abs(r[..., None] - allowed), axis=-1) < 1e-6)


def _py_iq3s_block(bp, grid):
    """independent pure-python decoder of one IQ3_S block from the published ggml layout"""
    d = np.frombuffer(bytes(bp[:2]), np.float16)[0].astype(np.float32)
    qs, qh, signs, scales = bp[2:66], bp[66:74], bp[74:106], bp[106:110]
    y = np.zeros(256, np.float32)
    for ib32 in range(8):
        nib = (int(scales[ib32 // 2]) >> (4 * (ib32 % 2))) & 15
        db = np.float32(d * np.float32(1 + 2 * nib))
        for l in range(4):
            for half in range(2):
                idx = int(qs[8 * ib32 + 2 * l + half]) | (((int(qh[ib32]) >> (2 * l + half)) & 1) << 8)
                word = int(grid[idx])
                for j in range(4):
                    s = -1.0 if (int(signs[4 * ib32 + l]) >> (4 * half + j)) & 1 else 1.0
                    y[32 * ib32 + 8 * l + 4 * half + j] = np.float32(db * np.float32((word >> (8 * j)) & 255)) * np.float32(s)
    return y


def test_iq3s_against_independent_decoder():
    from dwarfstar_red_lite_amd import synth
    rng = np.random.default_rng(9)
    grid = np.ctypeslib.as_array(orc.lib().orc_iq3s_grid(), (512,))
    rows = synth.quant_rows(rng, T_IQ3, 3, 256)
    for r in rows:
        assert np.array_equal(orc.dequant_rows(T_IQ3, r, 256)[0], _py_iq3s_block(r, grid))


def test_matvec_threads_identical():
    from dwarfstar_red_lite_amd import synth
    rng = np.random.default_rng(2)
    w = synth.quant_rows(rng, T_IQ2, 96, 512)
    x = rng.standard_normal(512).astype(np.float32)
    a = orc.matvec(T_IQ2, w, 512, x, threads=1)
    b = orc.matvec(T_IQ2, w, 512, x, threads=5)
    c = orc.matvec(T_IQ2, w, 512, x, row_start=10, row_count=20, threads=3)
    assert np.array_equal(a, b) and np.array_equal(a[10:30], c)
    assert a[7] == np.float32(orc.row_dot(T_IQ2, w[7], x))


def load_iq_grids(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
    return np.frombuffer(bytes.fromhex(g["iq2_xs"]), np.int8), np.frombuffer(bytes.fromhex(g["iq1_m"]), np.int8), g


def fnv1a64(data):
    h = 1469598103934665603          # the reference's offset basis (native/redlite_native_tables.c:272), not the textbook one
    for b in data.tobytes():
        h = ((h ^ b) * 0x100000001b3) & 0xffffffffffffffff
    return h


def test_iq2xs_iq1m_codebooks(golden_dir):
    xs, m, g = load_iq_grids(golden_dir)
    assert xs.size == 512 * 8 and m.size == 2048 * 8
    assert set(np.unique(xs).tolist()) == {8, 25, 43} and set(np.unique(m).tolist()) == {-1, 0, 1}
    # the digests the reference computes over the same tables (rl_native_quant_table_fnv1a)
    assert "%016x" % fnv1a64(xs) == g["iq2_xs_fnv1a"] and "%016x" % fnv1a64(m) == g["iq1_m_fnv1a"]
    assert len({xs[8 * i:8 * i + 8].tobytes() for i in range(512)}) == 512          # a codebook has no repeated entry
    assert len({m[8 * i:8 * i + 8].tobytes() for i in range(2048)}) == 2048


def test_golden_rows_iq2xs_iq1m(golden_dir):
    """the reference's own row dot (rl_native_quant_row_dot) on seeded rows, bit for bit; the dequantised row is exact in
    f32, so its double dot with x must agree with the reference's to rounding"""
    xs, m, _ = load_iq_grids(golden_dir)
    g = json.load(open(os.path.join(golden_dir, "quant_rows_xs_m.json")))
    seen = set()
    for c in g["cases"]:
        t, n = c["type"], c["ncols"]
        grid = xs if t == 17 else m
        row = unhex(c["row"], np.uint8)
        x = unhex(c["x"], np.float32)
        want = struct.unpack("<d", bytes.fromhex(c["dot"]))[0]
        assert orc.row_dot_grid(t, row, x, grid) == want, (t, n, c["fill"])
        w = orc.dequant_rows_grid(t, row, n, grid)[0]
        brute = float(np.dot(w.astype(np.float64), x.astype(np.float64)))
        assert abs(brute - want) <= 1e-9 * max(1.0, np.abs(w.astype(np.float64) * x).sum())
        seen.add((t, c["fill"]))
    assert {(17, 0), (29, 0), (17, 3), (29, 3), (17, 4), (29, 4)} <= seen


def test_iq2xs_iq1m_known_blocks(golden_dir):
    """hand-built blocks: every field decoded where the format says it is"""
    xs, m, _ = load_iq_grids(golden_dir)
    blk = np.zeros(74, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(2.0).tobytes(), np.uint8)
    q = 5 | (0b0000011 << 9)                    # entry 5, signs on weights 0 and 1, even parity: weight 7 positive
    blk[2 + 2 * 3:2 + 2 * 3 + 2] = [q & 255, q >> 8]         # group 1, part 1 -> weights 24..31
    blk[66] = 0x70                              # scale 7 for group 1 (high nibble of byte 0)
    w = orc.dequant_rows_grid(17, blk[None, :], 256, xs)[0]
    db = 2.0 * (0.5 + 7) * 0.25
    want = db * xs[40:48].astype(np.float64) * np.array([-1, -1, 1, 1, 1, 1, 1, 1])
    assert np.array_equal(w[24:32], want.astype(np.float32))
    assert np.array_equal(w[0:8], (2.0 * 0.5 * 0.25 * xs[0:8]).astype(np.float32))      # entry 0, scale 0, no signs
    blk = np.zeros(56, np.uint8)
    d = int(np.frombuffer(np.float16(0.5).tobytes(), np.uint16)[0])
    sc = [((d >> (4 * i)) & 15) << 12 for i in range(4)]
    sc[0] |= 3 << 3                             # scale index 1 (groups 2, 3) = 3
    for i in range(4):
        blk[48 + 2 * i] = sc[i] & 255
        blk[49 + 2 * i] = sc[i] >> 8
    blk[2] = 0x34                               # group 2: low grid bits
    blk[32 + 1] = 0x0a                          # group 2 nibble: delta negative, high grid bits 2
    w = orc.dequant_rows_grid(29, blk[None, :], 256, m)[0]
    gi = 0x34 | (2 << 8)
    want = 0.5 * 7 * (m[8 * gi:8 * gi + 8].astype(np.float64) - 0.125)
    assert np.array_equal(w[16:24], want.astype(np.float32))
    assert np.array_equal(w[0:8], (0.5 * 1 * (m[0:8].astype(np.float64) + 0.125)).astype(np.float32))


def test_expert_ffn_grid_composition(golden_dir):
    """orc_expert_ffn_grid: the other formats give orc_expert_ffn bit for bit; with a codebook format on either side gate/up are
    the pinned row dots and the down rows agree with a numpy double product over the exactly dequantised weights."""
    from dwarfstar_red_lite_amd import synth
    xs, m, _ = load_iq_grids(golden_dir)
    H, F = 512, 256
    rng = np.random.default_rng(91)
    x = synth.normed_x(rng, 1, H)[0]
    gate, up, down = synth.quant_rows(rng, 16, F, H), synth.quant_rows(rng, 16, F, H), synth.quant_rows(rng, 21, H, F)
    assert np.array_equal(orc.expert_ffn_grid(16, 21, gate, up, down, H, F, x, xs, m), orc.expert_ffn(16, 21, gate, up, down, H, F, x))
    for gu, dn in ((17, 17), (29, 29), (29, 17), (17, 16)):
        gate, up, down = synth.quant_rows(rng, gu, F, H), synth.quant_rows(rng, gu, F, H), synth.quant_rows(rng, dn, H, F)
        ggrid = xs if gu == 17 else m
        act = np.array([orc.lib().orc_silu_mul(orc.row_dot_grid(gu, gate[r], x, ggrid), orc.row_dot_grid(gu, up[r], x, ggrid)) for r in range(F)])
        wd = orc.dequant_rows_grid(dn, down, F, xs if dn == 17 else m) if dn in (17, 29) else orc.dequant_rows(dn, down, F)
        want = wd.astype(np.float64) @ act
        got = orc.expert_ffn_grid(gu, dn, gate, up, down, H, F, x, xs, m)
        bound = 1e-12 * (np.abs(wd.astype(np.float64)) @ np.abs(act))
        assert np.all(np.abs(got - want) <= bound + 1e-300), (gu, dn)
        win = orc.expert_ffn_grid(gu, dn, gate, up, down, H, F, x, xs, m, row_start=500, row_count=12)
        assert np.array_equal(win, got[500:])
    # a Q6_K (and an IQ2_XXS, an IQ3_S) down matrix fed double activations: the row dot with a double input vector against a numpy
    # double product over the exactly dequantised row (each term is one rounding of an exact product, the sum is sequential)
    for dn in (14, 16, 21):
        down = synth.quant_rows(rng, dn, H, F)
        act = rng.standard_normal(F) * np.exp(rng.uniform(-3, 3, F))
        wd = orc.dequant_rows(dn, down, F).astype(np.float64)
        got = np.array([orc.row_dot(dn, down[r], act) for r in range(H)])          # float64 input: orc_row_dot_d
        bound = 1e-12 * (np.abs(wd) @ np.abs(act))
        assert np.all(np.abs(got - wd @ act) <= bound + 1e-300), dn
        # and it is what the expert FFN feeds its down projection with
        gate, up = synth.quant_rows(rng, 16, F, H), synth.quant_rows(rng, 16, F, H)
        a64 = np.array([orc.lib().orc_silu_mul(orc.row_dot(16, gate[r], x), orc.row_dot(16, up[r], x)) for r in range(F)])
        ffn = orc.expert_ffn(16, dn, gate, up, down, H, F, x)
        assert np.array_equal(ffn, np.array([orc.row_dot(dn, down[r], a64) for r in range(H)])), dn


def test_kept_codebooks_match_grid_arguments(golden_dir):
    """the functions without a grid argument, after set_codebooks, give what the grid-taking ones give, bit for bit"""
    from dwarfstar_red_lite_amd import synth
    xs, m, _ = load_iq_grids(golden_dir)
    orc.set_codebooks(xs, m)
    H, F = 512, 256
    rng = np.random.default_rng(92)
    x = synth.normed_x(rng, 1, H)[0]
    for t, grid in ((17, xs), (29, m)):
        rows = synth.quant_rows(rng, t, 5, H)
        assert orc.row_bytes(t, H) == rows.shape[1]
        assert np.array_equal(orc.dequant_rows(t, rows, H), orc.dequant_rows_grid(t, rows, H, grid))
        assert [orc.row_dot(t, rows[r], x) for r in range(5)] == [orc.row_dot_grid(t, rows[r], x, grid) for r in range(5)]
        gate, up, down = synth.quant_rows(rng, t, F, H), synth.quant_rows(rng, t, F, H), synth.quant_rows(rng, t, H, F)
        assert np.array_equal(orc.expert_ffn(t, t, gate, up, down, H, F, x), orc.expert_ffn_grid(t, t, gate, up, down, H, F, x, xs, m))
