"""GGUF side: directory parsing and configuration probe on the host; upload from a file on the GPU, where the layer loaded from
the file must behave exactly as the same layer uploaded from memory."""
import numpy as np
import pytest

from dwarfstar_red_lite_amd import synth
from dwarfstar_red_lite_amd._lib import RedHipError
from dwarfstar_red_lite_amd.gguf_writer import write_moe_gguf


def small_cfg(layout):
    return synth.layer_config(hidden=512, ffn=256, n_expert=16, top_k=4, layout=layout)


@pytest.mark.parametrize("layout", ["iq2", "f2"])
def test_config_probe(tmp_path, layout):
    from dwarfstar_red_lite_amd.moe import gguf_moe_config
    cfg = small_cfg(layout)
    layers = [synth.make_layer(40 + i, cfg) for i in range(3)]
    path = tmp_path / "moe.gguf"
    write_moe_gguf(path, cfg, layers, first_layer=2, extra_tensors=[("token_embd.weight", np.arange(100, dtype=np.float32))])
    got, n = gguf_moe_config(str(path), first_layer=2)
    assert n == 3
    for k in ("hidden", "ffn", "n_expert", "top_k", "router_type", "gate_up_type", "down_type", "sh_gate_up_type", "sh_down_type"):
        assert got[k] == cfg[k], k
    with pytest.raises(RedHipError, match="lacks one of the MoE tensors"):
        gguf_moe_config(str(path), first_layer=0)


def test_rejects_broken_files(tmp_path):
    from dwarfstar_red_lite_amd.moe import gguf_moe_config
    p = tmp_path / "bad.gguf"
    p.write_bytes(b"GGML" + b"\0" * 64)
    with pytest.raises(RedHipError, match="invalid or unsupported GGUF header"):
        gguf_moe_config(str(p))
    cfg = small_cfg("iq2")
    good = tmp_path / "good.gguf"
    write_moe_gguf(good, cfg, [synth.make_layer(1, cfg)])
    cut = tmp_path / "cut.gguf"
    cut.write_bytes(good.read_bytes()[:-1000])
    with pytest.raises(RedHipError, match="beyond the end of the file"):
        gguf_moe_config(str(cut))
    with pytest.raises(RedHipError, match="open .* failed"):
        gguf_moe_config(str(tmp_path / "missing.gguf"))


@pytest.mark.gpu
@pytest.mark.parametrize("layout", ["iq2", "f2"])
def test_load_from_file_equals_load_from_memory(tmp_path, layout):
    torch = pytest.importorskip("torch")
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = small_cfg(layout)
    layers = [synth.make_layer(50 + i, cfg) for i in range(2)]
    path = tmp_path / "moe.gguf"
    write_moe_gguf(path, cfg, layers, first_layer=5)
    a = ResidentMoe.from_gguf(str(path), first_layer=5, max_tokens=3)
    assert a.n_layer == 2 and a.cfg["top_k"] == 4
    b = ResidentMoe(cfg, n_layer=2, max_tokens=3)
    x = torch.from_numpy(synth.normed_x(np.random.default_rng(3), 3, cfg["hidden"])).cuda()
    for l in range(2):
        b.load_layer(l, layers[l])
        for nt in (1, 3):
            assert torch.equal(a.forward(l, x[:nt]), b.forward(l, x[:nt]))
        for which in range(3):
            assert torch.equal(a.dequant_resident(l, 3, which), b.dequant_resident(l, 3, which))
    a.close()
    b.close()


def test_config_probe_walks_format_runs(tmp_path):
    """layers 0-1 IQ2_XS, 2-4 IQ1_M, 5 IQ2_XS (the reference's target file changes its expert format this way): one run per format"""
    from dwarfstar_red_lite_amd.moe import gguf_moe_config
    cx, cm = small_cfg("xs"), small_cfg("m")
    cfgs = [cx, cx, cm, cm, cm, cx]
    layers = [synth.make_layer(70 + i, c) for i, c in enumerate(cfgs)]
    path = tmp_path / "mixed.gguf"
    write_moe_gguf(path, cfgs, layers)
    for first, n, t in ((0, 2, 17), (1, 1, 17), (2, 3, 29), (5, 1, 17)):
        cfg, n_layer = gguf_moe_config(str(path), first)
        assert n_layer == n and cfg["gate_up_type"] == t and cfg["down_type"] == t and cfg["sh_gate_up_type"] == 14


@pytest.mark.gpu
def test_load_format_runs_from_file(tmp_path, golden_dir):
    import json
    import os
    torch = pytest.importorskip("torch")
    from dwarfstar_red_lite_amd import moe
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    g = json.load(open(os.path.join(golden_dir, "iq_grids.json")))
    moe.set_codebooks(np.frombuffer(bytes.fromhex(g["iq2_xs"]), np.int8), np.frombuffer(bytes.fromhex(g["iq1_m"]), np.int8))
    cx, cm = small_cfg("xs"), small_cfg("m")
    cfgs = [cx, cm, cm]
    layers = [synth.make_layer(80 + i, c) for i, c in enumerate(cfgs)]
    path = tmp_path / "mixed.gguf"
    write_moe_gguf(path, cfgs, layers)
    x = torch.from_numpy(synth.normed_x(np.random.default_rng(4), 3, cx["hidden"])).cuda()
    for first, n, cfg in ((0, 1, cx), (1, 2, cm)):
        a = ResidentMoe.from_gguf(str(path), first_layer=first, max_tokens=3)
        assert a.n_layer == n and a.cfg["gate_up_type"] == cfg["gate_up_type"]
        b = ResidentMoe(cfg, n_layer=n, max_tokens=3)
        for l in range(n):
            b.load_layer(l, layers[first + l])
            for nt in (1, 3):
                assert torch.equal(a.forward(l, x[:nt]), b.forward(l, x[:nt]))
        a.close()
        b.close()


# ---- the reader against the reference's own parser: tests/golden/gguf_expert_layout.json holds what rl_native_build_expert_map and
# ---- rl_native_expert_layout (native/redlite_native_gguf.c:199-440) answered for files that write_case() rebuilds byte for byte

def layout_cases(golden_dir):
    import json
    import os
    return json.load(open(os.path.join(golden_dir, "gguf_expert_layout.json")))["cases"]


LAYOUT_FIELDS = ("layer", "expert", "ggml_type", "down_type", "gate_offset", "gate_bytes", "up_offset", "up_bytes", "down_offset",
                 "down_bytes", "total_bytes")


def test_expert_layout_equals_the_reference_parser(tmp_path, golden_dir):
    import zlib
    from dwarfstar_red_lite_amd.moe import gguf_expert_layout
    from dwarfstar_red_lite_amd.gguf_writer import write_case
    seen = 0
    for case in layout_cases(golden_dir):
        spec = case["spec"]
        path = tmp_path / (spec["name"] + ".gguf")
        cfgs, layers = write_case(path, spec)
        raw = path.read_bytes()
        assert len(raw) == case["file_size"] and zlib.crc32(raw) == case["file_crc32"], spec["name"]      # the bytes the reference parsed
        assert case["map_ok"] == 1 and case["map"]["expert_count"] == spec["n_expert"]
        for want in case["layouts"]:
            got = gguf_expert_layout(str(path), spec["n_expert"], want["layer"], want["expert"])
            assert [got[k] for k in LAYOUT_FIELDS] == [want[k] for k in LAYOUT_FIELDS], (spec["name"], want["layer"], want["expert"])
            # and the ranges hold the bytes that went in for that expert
            lay = layers[want["layer"] - spec["first_layer"]]
            for key in ("gate", "up", "down"):
                o, n = want[key + "_offset"], want[key + "_bytes"]
                assert raw[o:o + n] == lay[key][want["expert"]].tobytes(), (spec["name"], key)
            seen += 1
        for refusal in case["refused"]:                   # what the reference refuses, this reader refuses
            with pytest.raises(RedHipError):
                gguf_expert_layout(str(path), spec["n_expert"], refusal["layer"], refusal["expert"])
    assert seen == 64 + 16 + 96


def test_expert_layout_strides_are_the_reference_spans(golden_dir):
    """The reference sizes an expert from the distance to the next tensor in the file, this reader from the tensor's type and shape:
    on the fixture files the two rules give the same stride for every routed tensor (and the 7 stray bytes behind the last tensor of
    one file are the reference's tail padding, not payload)."""
    for case in layout_cases(golden_dir):
        if case["spec"].get("up_type") is not None:
            continue
        for t in case["routed"]:
            rows = t["shape"][1]
            assert t["slice_safe"] == 1 and t["expert_stride_bytes"] == rows * synth.row_bytes(t["ggml_type"], t["shape"][0])
        assert sum(t["tail_padding_bytes"] for t in case["routed"]) == case["spec"].get("trailing_bytes", 0)


@pytest.mark.gpu
def test_layer_loaded_from_file_equals_cpu_path_on_the_reference_byte_ranges(tmp_path, golden_dir):
    """End to end: the file is loaded by this library's reader, the CPU path gets the experts cut out of the file at the offsets the
    REFERENCE's parser reported. A reader that placed a tensor or an expert wrongly fails here."""
    torch = pytest.importorskip("torch")
    import oracle_lib as orc
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    from gpu_common import REL_L2_TOL, rel_l2
    from dwarfstar_red_lite_amd.gguf_writer import write_case
    from test_gpu_moe_layer import ids_match_up_to_ties
    for case in layout_cases(golden_dir)[:2]:
        spec = case["spec"]
        path = tmp_path / (spec["name"] + ".gguf")
        cfgs, layers = write_case(path, spec)
        raw = np.frombuffer(path.read_bytes(), np.uint8)
        m = ResidentMoe.from_gguf(str(path), first_layer=spec["first_layer"], max_tokens=3)
        assert m.n_layer == len(layers)
        x = synth.normed_x(np.random.default_rng(spec["seed"]), 3, spec["hidden"])
        for l, (cfg, lay) in enumerate(zip(cfgs, layers)):
            cut = {k: v for k, v in lay.items() if k not in ("gate", "up", "down")}
            per = [w for w in case["layouts"] if w["layer"] == spec["first_layer"] + l]
            assert [w["expert"] for w in per] == list(range(spec["n_expert"]))
            for key in ("gate", "up", "down"):
                cut[key] = np.stack([raw[w[key + "_offset"]:w[key + "_offset"] + w[key + "_bytes"]] for w in per])
            ref = orc.Layer(cfg, **cut)
            got = m.forward(l, torch.from_numpy(x).cuda()).cpu().numpy()
            gids, gw, glog = m.last_route(3)
            want, cids, cw, clog = ref.forward(x)
            for t in range(3):
                assert ids_match_up_to_ties(gids[t], cids[t], clog[t])
                if np.array_equal(gids[t], cids[t]):
                    assert rel_l2(got[t], want[t]) <= REL_L2_TOL, (spec["name"], l, t)
        m.close()
