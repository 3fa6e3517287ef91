"""Host-side mirror of redlite/redmetal_quant.py:9-95 (one-shot quantised GEMV from a file) and of the router
entry points of native/redlite_native_router_exec.h over libredmetal_hip.so."""
import ctypes as C
import os

import numpy as np

from ._lib import RedHipError, RouterTelemetry, RouterTensorInfo, load


class RedMetalQuantBridge:
    def __init__(self):
        self.lib = load()

    def _last_error(self):
        raw = self.lib.redmetal_quant_last_error()
        return raw.decode("utf-8", errors="replace") if raw else "unknown Red Metal quant error"

    def rows(self, model, matrix_file_offset, matrix_bytes, ggml_type, ncols, nrows, row_start, row_count, input_values, grid=None):
        x = np.ascontiguousarray(input_values, np.float32)
        if x.size != ncols:
            raise ValueError("input has %d values, expected %d" % (x.size, ncols))
        g = np.ascontiguousarray(grid, np.int8) if grid is not None else None
        out = np.zeros(max(row_count, 1), np.float32)
        io_ms, gpu_ms = C.c_double(), C.c_double()
        ok = self.lib.redmetal_quant_rows(os.fsencode(os.path.abspath(os.path.expanduser(str(model)))), int(matrix_file_offset),
                                          int(matrix_bytes), int(ggml_type), int(ncols), int(nrows), int(row_start), int(row_count),
                                          x.ctypes.data, ncols, g.ctypes.data if g is not None else None, g.size if g is not None else 0,
                                          out.ctypes.data, row_count, C.byref(io_ms), C.byref(gpu_ms))
        if not ok:
            raise RedHipError(self._last_error())
        return out[:row_count], float(io_ms.value), float(gpu_ms.value)


def router_gpu(model, ggml_type, hidden, experts, tensor_offset, span_bytes, input_values):
    """rl_native_router_gpu_f32: logits of the (hidden, experts) tensor at tensor_offset of the file."""
    lib = load()
    info = RouterTensorInfo(layer=0, ggml_type=ggml_type, n_dims=2, tensor_offset=tensor_offset, tensor_span_bytes=span_bytes)
    info.shape[0], info.shape[1] = hidden, experts
    x = np.ascontiguousarray(input_values, np.float32)
    logits = np.zeros(experts, np.float32)
    tel = RouterTelemetry()
    err = C.create_string_buffer(256)
    ok = lib.rl_native_router_gpu_f32(os.fsencode(str(model)), C.byref(info), x.ctypes.data, x.size, logits.ctypes.data, experts,
                                      C.byref(tel), err, len(err))
    if not ok:
        raise RedHipError(err.value.decode())
    return logits, {"read_ms": tel.read_ms, "compute_ms": tel.compute_ms}


def router_select(logits, top_k, want_probs=False):
    """rl_native_router_select_softmax_topk on the GPU."""
    lib = load()
    l = np.ascontiguousarray(logits, np.float32)
    ids = np.zeros(top_k, np.uint32)
    w = np.zeros(top_k, np.float32)
    probs = np.zeros(l.size, np.float32) if want_probs else None
    err = C.create_string_buffer(256)
    ok = lib.rl_native_router_select_softmax_topk(l.ctypes.data, l.size, top_k, ids.ctypes.data, w.ctypes.data,
                                                  probs.ctypes.data if want_probs else None, err, len(err))
    if not ok:
        raise RedHipError(err.value.decode())
    return (ids, w, probs) if want_probs else (ids, w)
