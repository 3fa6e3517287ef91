"""TEST INFRASTRUCTURE - ctypes view of oracle/libmoe_oracle.so (the CPU restatement of the reference path).

Imported only by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg. The shipped library never
touches it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmoe_oracle.so")

u8p = C.POINTER(C.c_uint8)
f32p = C.POINTER(C.c_float)
f64p = C.POINTER(C.c_double)
u32p = C.POINTER(C.c_uint32)


class OrcLayer(C.Structure):
    _fields_ = [
        ("hidden", C.c_uint32), ("ffn", C.c_uint32), ("n_expert", C.c_uint32), ("top_k", C.c_uint32),
        ("router_type", C.c_uint32), ("gate_up_type", C.c_uint32), ("down_type", C.c_uint32),
        ("sh_gate_up_type", C.c_uint32), ("sh_down_type", C.c_uint32),
        ("router", C.c_void_p), ("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p),
        ("sh_gate", C.c_void_p), ("sh_up", C.c_void_p), ("sh_down", C.c_void_p), ("sh_gate_inp", C.c_void_p),
    ]


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "libmoe_oracle.so"] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f16_all.restype = None
        L.orc_f16_all.argtypes = [C.c_void_p]
        L.orc_iq2xxs_grid.restype = u8p
        L.orc_iq3s_grid.restype = u32p
        L.orc_crc32.restype = C.c_uint32
        L.orc_crc32.argtypes = [C.c_void_p, C.c_size_t]
        L.orc_block_bytes.restype = C.c_size_t
        L.orc_block_bytes.argtypes = [C.c_uint32]
        L.orc_row_bytes.restype = C.c_size_t
        L.orc_row_bytes.argtypes = [C.c_uint32, C.c_uint32]
        L.orc_dequant_row.argtypes = [C.c_uint32, C.c_void_p, C.c_uint32, C.c_void_p]
        L.orc_row_dot.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint32, f64p]
        L.orc_row_dot_d.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint32, f64p]
        L.orc_dequant_row_grid.argtypes = [C.c_uint32, C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p]
        L.orc_set_codebooks.argtypes = [C.c_void_p, C.c_void_p]
        L.orc_set_codebooks.restype = None
        L.orc_row_dot_grid.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p, f64p]
        L.orc_expert_ffn_grid.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32,
                                          C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_matvec.argtypes = [C.c_uint32, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_int]
        L.orc_rmsnorm.restype = None
        L.orc_rmsnorm.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_float, C.c_void_p]
        L.orc_router_logits.argtypes = [C.c_uint32, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        L.orc_router_select.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_silu_mul.restype = C.c_double
        L.orc_silu_mul.argtypes = [C.c_double, C.c_double]
        L.orc_expert_ffn.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32,
                                     C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        L.orc_routed_topk.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                      C.c_size_t, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        L.orc_shared_expert.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                        C.c_uint32, C.c_void_p, C.c_void_p, f64p, C.c_int]
        L.orc_shared_expert_standalone.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                                   C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, f64p]
        L.orc_moe_layer.argtypes = [C.POINTER(OrcLayer), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.orc_moe_layer_batch.argtypes = [C.POINTER(OrcLayer), C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.orc_group_pairs.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _bytes(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint8
    return a


def row_bytes(t, ncols):
    return int(lib().orc_row_bytes(t, ncols))


def dequant_rows(t, rows, ncols):
    """rows: uint8 [nrows, row_bytes] -> float32 [nrows, ncols]"""
    rows = _bytes(rows).reshape(-1, row_bytes(t, ncols))
    out = np.empty((rows.shape[0], ncols), np.float32)
    for r in range(rows.shape[0]):
        assert lib().orc_dequant_row(t, _p(rows[r]), ncols, _p(out[r]))
    return out


def row_dot(t, row, x):
    row = _bytes(row)
    x = np.ascontiguousarray(x)
    d = C.c_double()
    if x.dtype == np.float64:
        ok = lib().orc_row_dot_d(t, _p(row), _p(x), x.size, C.byref(d))
    else:
        assert x.dtype == np.float32
        ok = lib().orc_row_dot(t, _p(row), _p(x), x.size, C.byref(d))
    assert ok
    return d.value


def matvec(t, w, ncols, x, row_start=0, row_count=None, threads=1):
    w = _bytes(w)
    nrows = w.size // row_bytes(t, ncols)
    if row_count is None:
        row_count = nrows - row_start
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(row_count, np.float32)
    assert lib().orc_matvec(t, _p(w), ncols, row_start, row_count, _p(x), _p(out), threads)
    return out


def router_logits(t, w, hidden, experts, x):
    w = _bytes(w) if w.dtype == np.uint8 else np.ascontiguousarray(w, np.float32)
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(experts, np.float32)
    assert lib().orc_router_logits(t, _p(w), hidden, experts, _p(x), _p(out))
    return out


def router_select(logits, top_k, want_probs=False):
    logits = np.ascontiguousarray(logits, np.float32)
    ids = np.empty(top_k, np.uint32)
    w = np.empty(top_k, np.float32)
    probs = np.empty(logits.size, np.float32) if want_probs else None
    ok = lib().orc_router_select(_p(logits), logits.size, top_k, _p(ids), _p(w), _p(probs))
    if not ok:
        raise ValueError("router selection failed")
    return (ids, w, probs) if want_probs else (ids, w)


def expert_ffn(gu_t, dn_t, gate, up, down, hidden, ffn, x, row_start=0, row_count=None):
    if row_count is None:
        row_count = hidden - row_start
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(row_count, np.float64)
    assert lib().orc_expert_ffn(gu_t, dn_t, _p(_bytes(gate)), _p(_bytes(up)), _p(_bytes(down)), hidden, ffn,
                                row_start, row_count, _p(x), _p(out))
    return out


def shared_expert(gu_t, dn_t, gate, up, down, gate_inp, hidden, ffn, x, threads=1):
    x = np.ascontiguousarray(x, np.float32)
    gate_inp = np.ascontiguousarray(gate_inp, np.float32)
    out = np.empty(hidden, np.float32)
    s = C.c_double()
    assert lib().orc_shared_expert(gu_t, dn_t, _p(_bytes(gate)), _p(_bytes(up)), _p(_bytes(down)), _p(gate_inp),
                                   hidden, ffn, _p(x), _p(out), C.byref(s), threads)
    return out, s.value


def shared_expert_standalone(gu_t, dn_t, gate, up, down, gate_inp, hidden, ffn, x, row_start=0, row_count=None):
    if row_count is None:
        row_count = hidden - row_start
    x = np.ascontiguousarray(x, np.float32)
    gate_inp = np.ascontiguousarray(gate_inp, np.float32)
    out = np.empty(row_count, np.float64)
    s = C.c_double()
    assert lib().orc_shared_expert_standalone(gu_t, dn_t, _p(_bytes(gate)), _p(_bytes(up)), _p(_bytes(down)),
                                              _p(gate_inp), hidden, ffn, row_start, row_count, _p(x), _p(out), C.byref(s))
    return out, s.value


class Layer:
    """Keeps the numpy buffers alive next to the C struct."""

    def __init__(self, cfg, router, gate, up, down, sh_gate, sh_up, sh_down, sh_gate_inp):
        self.keep = [np.ascontiguousarray(a) for a in (router, gate, up, down, sh_gate, sh_up, sh_down, sh_gate_inp)]
        k = self.keep
        self.c = OrcLayer(cfg["hidden"], cfg["ffn"], cfg["n_expert"], cfg["top_k"], cfg["router_type"],
                          cfg["gate_up_type"], cfg["down_type"], cfg["sh_gate_up_type"], cfg["sh_down_type"],
                          *[a.ctypes.data for a in k])
        self.cfg = cfg

    def forward(self, x, threads=1):
        cfg = self.cfg
        x = np.ascontiguousarray(x, np.float32).reshape(-1, cfg["hidden"])
        n = x.shape[0]
        out = np.empty((n, cfg["hidden"]), np.float32)
        ids = np.empty((n, cfg["top_k"]), np.uint32)
        w = np.empty((n, cfg["top_k"]), np.float32)
        logits = np.empty((n, cfg["n_expert"]), np.float32)
        for t in range(n):
            assert lib().orc_moe_layer(C.byref(self.c), _p(x[t]), _p(out[t]), _p(ids[t]), _p(w[t]), _p(logits[t]), threads)
        return out, ids, w, logits


def group_pairs(ids, weights, n_expert):
    ids = np.ascontiguousarray(ids, np.uint32)
    weights = np.ascontiguousarray(weights, np.float32)
    ntok, top_k = ids.shape
    P = ntok * top_k
    uid = np.zeros(min(P, n_expert), np.uint32)
    start = np.zeros(min(P, n_expert) + 1, np.uint32)
    ptok = np.zeros(P, np.uint32)
    pw = np.zeros(P, np.float32)
    tp = np.zeros(P, np.uint32)
    U = lib().orc_group_pairs(_p(ids), _p(weights), ntok, top_k, n_expert, _p(uid), _p(start), _p(ptok), _p(pw), _p(tp))
    if U < 0:
        raise ValueError("bad grouping arguments")
    return uid[:U].copy(), start[:U + 1].copy(), ptok, pw, tp


def dequant_rows_grid(t, rows, ncols, grid):
    """float32 [nrows, ncols] of IQ2_XS (17) / IQ1_M (29) rows; grid: int8 codebook of the type."""
    rows = np.ascontiguousarray(rows, np.uint8).reshape(-1, rows.shape[-1])
    grid = np.ascontiguousarray(grid, np.int8)
    out = np.empty((rows.shape[0], ncols), np.float32)
    for r in range(rows.shape[0]):
        assert lib().orc_dequant_row_grid(t, _p(rows[r]), ncols, _p(grid), _p(out[r]))
    return out


def row_dot_grid(t, row, x, grid):
    row, x, grid = np.ascontiguousarray(row, np.uint8), np.ascontiguousarray(x, np.float32), np.ascontiguousarray(grid, np.int8)
    d = C.c_double()
    assert lib().orc_row_dot_grid(t, _p(row), _p(x), x.size, _p(grid), C.byref(d))
    return d.value


def expert_ffn_grid(gu_t, dn_t, gate, up, down, hidden, ffn, x, xs_grid, m_grid, row_start=0, row_count=None):
    """single-expert FFN in double where either side may be IQ2_XS (17) / IQ1_M (29)."""
    row_count = hidden - row_start if row_count is None else row_count
    x = np.ascontiguousarray(x, np.float32)
    xs_grid, m_grid = np.ascontiguousarray(xs_grid, np.int8), np.ascontiguousarray(m_grid, np.int8)
    out = np.zeros(row_count, np.float64)
    assert lib().orc_expert_ffn_grid(gu_t, dn_t, _p(_bytes(gate)), _p(_bytes(up)), _p(_bytes(down)), hidden, ffn, row_start, row_count,
                                     _p(x), _p(xs_grid), _p(m_grid), _p(out))
    return out


def set_codebooks(iq2_xs=None, iq1_m=None):
    """keep the codebooks for the functions that take no grid (row_dot, matvec, expert_ffn, Layer.forward on types 17 / 29)."""
    a = np.ascontiguousarray(iq2_xs, np.int8) if iq2_xs is not None else None
    b = np.ascontiguousarray(iq1_m, np.int8) if iq1_m is not None else None
    assert (a is None or a.size == 4096) and (b is None or b.size == 16384)
    lib().orc_set_codebooks(_p(a), _p(b))
