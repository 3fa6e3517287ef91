"""Writes a GGUF v3 file holding the MoE tensors of synthetic layers (for the tests and the benchmark of the file-backed pool). Format as the reference parses it
(native/redlite_native_gguf.c:196-330): header, metadata key/values, tensor directory, aligned data."""
import struct

import numpy as np

GGUF_U32, GGUF_STRING = 4, 8


def _s(b):
    b = b.encode() if isinstance(b, str) else b
    return struct.pack("<Q", len(b)) + b


def write_moe_gguf(path, cfg, layers, first_layer=0, alignment=32, arch="qwen3next", extra_tensors=()):
    """layers: list of dicts from synth.make_layer; cfg: their configuration, or a list with one per layer. Tensors per layer: router, sh_gate_inp, shared gate/up/down, routed
    gate/up/down (expert-major). extra_tensors: (name, np.ndarray) pairs placed first (other model tensors)."""
    cfgs = list(cfg) if isinstance(cfg, (list, tuple)) else [cfg] * len(layers)      # one dict, or one per layer (mixed formats)
    cfg = cfgs[0]
    H, F, E = cfg["hidden"], cfg["ffn"], cfg["n_expert"]
    tensors = list((n, a, (a.size,), 0) for n, a in extra_tensors)
    for i, lay in enumerate(layers):
        l = first_layer + i
        cfg = cfgs[i]
        tensors += [
            ("blk.%d.ffn_gate_inp.weight" % l, lay["router"], (H, E), cfg["router_type"]),
            ("blk.%d.ffn_gate_inp_shexp.weight" % l, lay["sh_gate_inp"], (H,), 0),
            ("blk.%d.ffn_gate_shexp.weight" % l, lay["sh_gate"], (H, F), cfg["sh_gate_up_type"]),
            ("blk.%d.ffn_up_shexp.weight" % l, lay["sh_up"], (H, F), cfg["sh_gate_up_type"]),
            ("blk.%d.ffn_down_shexp.weight" % l, lay["sh_down"], (F, H), cfg["sh_down_type"]),
            ("blk.%d.ffn_gate_exps.weight" % l, lay["gate"], (H, F, E), cfg["gate_up_type"]),
            ("blk.%d.ffn_up_exps.weight" % l, lay["up"], (H, F, E), cfg.get("up_type", cfg["gate_up_type"])),
            ("blk.%d.ffn_down_exps.weight" % l, lay["down"], (F, H, E), cfg["down_type"]),
        ]
    kv = [("general.architecture", GGUF_STRING, arch), ("general.alignment", GGUF_U32, alignment),
          (arch + ".block_count", GGUF_U32, first_layer + len(layers)), (arch + ".expert_count", GGUF_U32, E),
          (arch + ".expert_used_count", GGUF_U32, cfg["top_k"]),
          ("tokenizer.ggml.tokens", 9, ["a", "bc", "def"])]          # an array of strings, to be skipped by the parser
    head = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(kv))
    for k, t, v in kv:
        head += _s(k) + struct.pack("<I", t)
        if t == GGUF_STRING:
            head += _s(v)
        elif t == GGUF_U32:
            head += struct.pack("<I", v)
        else:
            head += struct.pack("<IQ", GGUF_STRING, len(v)) + b"".join(_s(x) for x in v)
    directory, blobs, off = b"", [], 0
    for name, arr, dims, typ in tensors:
        raw = np.ascontiguousarray(arr).tobytes()
        directory += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", typ, off)
        blobs.append((off, raw))
        off = (off + len(raw) + alignment - 1) // alignment * alignment
    start = (len(head) + len(directory) + alignment - 1) // alignment * alignment
    with open(path, "wb") as fh:
        fh.write(head + directory)
        fh.write(b"\0" * (start - len(head) - len(directory)))
        for o, raw in blobs:
            fh.seek(start + o)
            fh.write(raw)
        fh.truncate(start + off)


def write_case(path, spec):
    """One of the fixture files of tests/golden/gguf_expert_layout.json, rebuilt from its `spec` (the same bytes every time: the
    fixture holds the file's CRC-32). Returns (list of per-layer configurations, list of layers)."""
    from dwarfstar_red_lite_amd import synth
    cfgs = []
    for layout in spec["layouts"]:
        c = synth.layer_config(hidden=spec["hidden"], ffn=spec["ffn"], n_expert=spec["n_expert"], top_k=spec["top_k"], layout=layout)
        if spec.get("up_type") is not None:
            c["up_type"] = spec["up_type"]                   # a file the reference refuses: gate and up of different types
        cfgs.append(c)
    layers = [synth.make_layer(spec["seed"] + i, c) for i, c in enumerate(cfgs)]
    extra = [("token_embd.weight", np.arange(spec["extra_floats"], dtype=np.float32))] if spec.get("extra_floats") else []
    write_moe_gguf(path, cfgs, layers, first_layer=spec["first_layer"], alignment=spec["alignment"], extra_tensors=extra)
    if spec.get("trailing_bytes"):
        with open(path, "ab") as fh:
            fh.write(b"\xa5" * spec["trailing_bytes"])
    return cfgs, layers


def write_topk_case(path, spec):
    """One of the fixture files of tests/golden/reference_topk.json: a single layer whose routed experts have the given gate/up and
    down formats (the same bytes every time). Returns (configuration, layer)."""
    from dwarfstar_red_lite_amd import synth
    c = synth.layer_config(hidden=spec["hidden"], ffn=spec["ffn"], n_expert=spec["n_expert"], top_k=2, layout="xs")
    c["gate_up_type"], c["down_type"] = spec["gate_up_type"], spec["down_type"]
    layer = synth.make_layer(spec["seed"], c)
    write_moe_gguf(path, c, [layer])
    return c, layer
