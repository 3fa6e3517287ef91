"""The C-ABI library loads and exports every symbol include/*.h declares (no GPU, no compute calls)."""
import ctypes
import glob
import os
import re

import pytest

from dwarfstar_red_lite_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        text = re.sub(r"//.*", "", text)
        for m in re.finditer(r"\b((?:redmetal|redhip|rl_native)_[a-z0-9_]+)\s*\(", text):
            names.add(m.group(1))
    return names


def test_headers_and_library_agree():
    if not os.path.isfile(_lib.LIB_PATH):
        pytest.fail("libredmetal_hip.so is not built: run python -m dwarfstar_red_lite_amd.build")
    names = declared_symbols()
    assert len(names) >= 35
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in sorted(names):
        assert hasattr(lib, n), "library does not export " + n
    assert names == set(_lib.ABI), names ^ set(_lib.ABI)
    assert _lib.load().redmetal_ffn_abi_version() == 1


def test_error_strings_without_device_work():
    lib = _lib.load()
    assert lib.redmetal_ffn_pool_create(None, 0, 0, 0, None, 0, None, 0) is None
    assert b"invalid Red Metal FFN pool arguments" in lib.redmetal_ffn_last_error()
    lib.redmetal_ffn_pool_destroy(None)
    lib.redhip_moe_destroy(None)
    assert lib.redhip_moe_create(None) is None
    assert b"null MoE config" in lib.redhip_moe_last_error()
    assert lib.redmetal_topk_pool_create(None, 0, 0, 0, None, 0, None, 0) is None
    assert b"invalid Red Metal top-k pool arguments" in lib.redmetal_topk_last_error()
    lib.redmetal_topk_pool_destroy(None)
    assert lib.redmetal_topk_pool_capacity(None) == 0 and lib.redmetal_topk_pool_tmp_buffer(None) is None
    assert lib.redmetal_topk_pool_slab_residency_set(None) is None
    assert lib.redmetal_quant_rows(None, 0, 0, 16, 256, 1, 0, 1, None, 256, None, 0, None, 1, None, None) == 0
    assert b"invalid Red Metal mixed-quant arguments" in lib.redmetal_quant_last_error()


def test_codebook_formats_refused_before_codebooks():
    """this process never uploads a codebook: a resident layer with IQ2_XS / IQ1_M experts is refused, not decoded through zeros;
    wrong codebook sizes are refused too"""
    lib = _lib.load()
    cfg = _lib.MoeConfig(hidden=512, ffn=256, n_expert=16, top_k=4, router_type=0, expert_type_word=17, shared_type_word=14,
                         n_layer=1, max_tokens=1)
    assert lib.redhip_moe_create(ctypes.byref(cfg)) is None
    assert b"redhip_set_codebooks" in lib.redhip_moe_last_error()
    buf = (ctypes.c_int8 * 4096)()
    assert lib.redhip_set_codebooks(buf, 4000, None, 0) == 0
    assert b"codebook size mismatch" in lib.redhip_moe_last_error()
