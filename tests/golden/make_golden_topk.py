"""Writes tests/golden/reference_topk.json. Runs ONLY in the build container, where the reference checkout exists: small GGUF files
with routed experts in the formats the reference's routed-expert CPU path accepts (IQ2_XS 17, IQ1_M 29, IQ3_S 21, and mixed gate/up
vs down types) are written by dwarfstar_red_lite_amd/gguf_writer.py, and the reference's own C (native/redlite_native_reference.c:307-382
rl_native_reference_topk, compiled unchanged into oracle/_ref/libref.so by oracle/Makefile) computes the weighted top-k expert
FFN on them in double. The fixture is data: each file's recipe and CRC-32, the routing, and the reference's answers as the hex of
their float64 bytes; nothing of its source text.

    make -C oracle ref && python3 tests/golden/make_golden_topk.py
"""
import ctypes as C
import json
import os
import sys
import tempfile
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "tests"), HERE]
from make_golden_gguf import ExpertMap      # noqa: E402
from dwarfstar_red_lite_amd.gguf_writer import write_topk_case      # noqa: E402

# (gate/up type, down type): the reference runs the down rows on double activations (the step no other fixture reaches)
CASES = [
    dict(name="iq2_xs", gate_up_type=17, down_type=17, hidden=256, ffn=256, n_expert=8, seed=9500),
    dict(name="iq1_m", gate_up_type=29, down_type=29, hidden=512, ffn=256, n_expert=8, seed=9501),
    dict(name="iq2_xs_gate_up_iq3_s_down", gate_up_type=17, down_type=21, hidden=256, ffn=512, n_expert=6, seed=9502),
    dict(name="iq3_s", gate_up_type=21, down_type=21, hidden=256, ffn=256, n_expert=6, seed=9503),
    dict(name="iq1_m_gate_up_iq2_xs_down", gate_up_type=29, down_type=17, hidden=256, ffn=256, n_expert=6, seed=9504),
]
# (expert ids in selection order, router weights, row_start, row_count or None for every row)
CALLS = [
    ([3, 0, 5], [0.5, 0.3, 0.2], 0, None),
    ([1], [1.0], 0, None),
    ([4, 2, 0, 1], [0.4, 0.3, 0.2, 0.1], 100, 37),
]


def harness_input(n):       # the deterministic activation vector of the reference's parity tool (native/redlite_native_ffn_parity_cli.c)
    i = np.arange(n, dtype=np.int64)
    return (((i * 17 + 3) % 61 - 30) / 32.0).astype(np.float32)


def main():
    ref = C.CDLL(os.path.join(ROOT, "oracle", "_ref", "libref.so"))
    ref.rl_native_build_expert_map.argtypes = [C.c_char_p, C.c_uint32, C.POINTER(ExpertMap), C.c_char_p, C.c_size_t]
    ref.rl_native_free_expert_map.argtypes = [C.POINTER(ExpertMap)]
    ref.rl_native_reference_topk.argtypes = [C.c_char_p, C.POINTER(ExpertMap), C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32,
                                             C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32, C.c_void_p, C.c_char_p, C.c_size_t]
    out = []
    with tempfile.TemporaryDirectory() as tmp:
        for spec in CASES:
            path = os.path.join(tmp, spec["name"] + ".gguf")
            write_topk_case(path, spec)
            raw = open(path, "rb").read()
            m, err = ExpertMap(), C.create_string_buffer(256)
            assert ref.rl_native_build_expert_map(path.encode(), spec["n_expert"], C.byref(m), err, 256), err.value
            H = spec["hidden"]
            x = harness_input(H)
            rec = {"spec": spec, "file_crc32": zlib.crc32(raw), "calls": []}
            for ids, w, row_start, row_count in CALLS:
                n = H - row_start if row_count is None else row_count
                ida, wa, res = np.asarray(ids, np.uint32), np.asarray(w, np.float32), np.zeros(n, np.float64)
                ok = ref.rl_native_reference_topk(path.encode(), C.byref(m), 0, ida.ctypes.data, wa.ctypes.data, len(ids), row_start, n,
                                                  x.ctypes.data, H, res.ctypes.data, n, None, err, 256)
                assert ok, err.value
                rec["calls"].append({"ids": ids, "weights_f32_hex": wa.tobytes().hex(), "row_start": row_start, "row_count": n,
                                     "output_f64_hex": res.tobytes().hex()})
            ref.rl_native_free_expert_map(C.byref(m))
            out.append(rec)
    with open(os.path.join(HERE, "reference_topk.json"), "w") as fh:
        json.dump({"source": "rl_native_reference_topk of the reference's unmodified C on synthetic GGUF files (see make_golden_topk.py)",
                   "input": "x[i] = ((i * 17 + 3) % 61 - 30) / 32", "cases": out}, fh, indent=1)
    print("wrote %d cases" % len(out))


if __name__ == "__main__":
    main()
