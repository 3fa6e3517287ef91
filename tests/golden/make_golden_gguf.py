"""Writes tests/golden/gguf_expert_layout.json. Runs ONLY in the build container, where the reference checkout exists: small GGUF
files are written by dwarfstar_red_lite_amd/gguf_writer.py, parsed by the reference's own C (native/redlite_native_gguf.c, compiled unchanged into
oracle/_ref/libref.so by oracle/Makefile) through rl_native_build_expert_map (:199-397) and rl_native_expert_layout (:399-440), and
what the reference answers is stored next to the recipe of each file and the file's CRC-32. The fixture is data: the reference's
answers; nothing of its source text.

    make -C oracle ref && python3 tests/golden/make_golden_gguf.py
"""
import ctypes as C
import json
import os
import sys
import tempfile
import zlib

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "tests")]
from dwarfstar_red_lite_amd.gguf_writer import write_case      # noqa: E402


class ExpertTensor(C.Structure):         # rl_expert_tensor, native/redlite_native_gguf.h:19-31
    _fields_ = [("layer", C.c_uint32), ("kind", C.c_int), ("ggml_type", C.c_uint32), ("n_dims", C.c_uint32), ("shape", C.c_uint64 * 8),
                ("tensor_offset", C.c_uint64), ("tensor_span_bytes", C.c_uint64), ("payload_bytes", C.c_uint64),
                ("tail_padding_bytes", C.c_uint64), ("expert_stride_bytes", C.c_uint64), ("slice_safe", C.c_int)]


class ExpertMap(C.Structure):            # rl_expert_map, native/redlite_native_gguf.h:33-45
    _fields_ = [("version", C.c_uint32), ("alignment", C.c_uint32), ("tensor_count", C.c_uint64), ("kv_count", C.c_uint64),
                ("expert_count", C.c_uint32), ("layer_count", C.c_uint32), ("routed_tensor_count", C.c_uint32),
                ("total_routed_payload_bytes", C.c_uint64), ("max_expert_triplet_bytes", C.c_uint64), ("all_slice_safe", C.c_int),
                ("routed", C.POINTER(ExpertTensor))]


class ExpertLayout(C.Structure):         # rl_expert_layout, native/redlite_native_gguf.h:47-59
    _fields_ = [(n, C.c_uint32) for n in ("layer", "expert", "ggml_type", "down_type")] + \
               [(n, C.c_uint64) for n in ("gate_offset", "gate_bytes", "up_offset", "up_bytes", "down_offset", "down_bytes", "total_bytes")]


CASES = [
    dict(name="packed_two_layers", layouts=["iq2", "iq2"], hidden=256, ffn=256, n_expert=32, top_k=4, seed=9100, first_layer=3,
         alignment=32, extra_floats=101),
    dict(name="mixed_precision_trailing_bytes", layouts=["f2"], hidden=512, ffn=256, n_expert=16, top_k=4, seed=9200, first_layer=0,
         alignment=64, trailing_bytes=7),
    dict(name="format_runs", layouts=["xs", "m", "m"], hidden=256, ffn=256, n_expert=32, top_k=2, seed=9300, first_layer=0,
         alignment=32, extra_floats=7),
    dict(name="gate_up_types_differ", layouts=["iq2"], hidden=256, ffn=256, n_expert=8, top_k=2, seed=9400, first_layer=0,
         alignment=32, up_type=17),                          # the up tensors labelled IQ2_XS, the gate tensors IQ2_XXS
]


def main():
    ref = C.CDLL(os.path.join(ROOT, "oracle", "_ref", "libref.so"))
    ref.rl_native_build_expert_map.argtypes = [C.c_char_p, C.c_uint32, C.POINTER(ExpertMap), C.c_char_p, C.c_size_t]
    ref.rl_native_expert_layout.argtypes = [C.POINTER(ExpertMap), C.c_uint32, C.c_uint32, C.POINTER(ExpertLayout), C.c_char_p, C.c_size_t]
    ref.rl_native_free_expert_map.argtypes = [C.POINTER(ExpertMap)]
    out = []
    with tempfile.TemporaryDirectory() as tmp:
        for spec in CASES:
            spec = dict(spec)
            path = os.path.join(tmp, spec["name"] + ".gguf")
            write_case(path, spec)
            raw = open(path, "rb").read()
            m, err = ExpertMap(), C.create_string_buffer(256)
            ok = ref.rl_native_build_expert_map(path.encode(), spec["n_expert"], C.byref(m), err, 256)
            rec = {"spec": spec, "file_size": len(raw), "file_crc32": zlib.crc32(raw), "map_ok": int(ok), "map_error": err.value.decode()}
            if ok:
                rec["map"] = {n: int(getattr(m, n)) for n, _ in ExpertMap._fields_ if n != "routed"}
                rec["routed"] = [{n: (list(getattr(m.routed[i], n)) if n == "shape" else int(getattr(m.routed[i], n))) for n, _ in ExpertTensor._fields_}
                                 for i in range(m.routed_tensor_count)]
                first, nl, E = spec["first_layer"], len(spec["layouts"]), spec["n_expert"]
                rec["layouts"], rec["refused"] = [], []
                for layer in range(first, first + nl):
                    for e in range(E):
                        lo = ExpertLayout()
                        if ref.rl_native_expert_layout(C.byref(m), layer, e, C.byref(lo), err, 256):
                            rec["layouts"].append({n: int(getattr(lo, n)) for n, _ in ExpertLayout._fields_})
                        else:
                            rec["refused"].append({"layer": layer, "expert": e, "error": err.value.decode()})
                for layer, e in ((first, E), (first + nl, 0), (first + nl + 5, 1)):       # beyond the experts, beyond the layers
                    lo = ExpertLayout()
                    r = ref.rl_native_expert_layout(C.byref(m), layer, e, C.byref(lo), err, 256)
                    assert not r
                    rec["refused"].append({"layer": layer, "expert": e, "error": err.value.decode()})
                ref.rl_native_free_expert_map(C.byref(m))
            out.append(rec)
            print(spec["name"], "map_ok", ok, "layouts", len(rec.get("layouts", [])), "refused", len(rec.get("refused", [])))
    with open(os.path.join(HERE, "gguf_expert_layout.json"), "w") as fh:
        json.dump({"cases": out}, fh, indent=0, separators=(",", ":"))


if __name__ == "__main__":
    main()
