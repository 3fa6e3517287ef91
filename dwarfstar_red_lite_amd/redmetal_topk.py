"""Host-side mirror of the reference's resident top-k pool bridge (redlite/redmetal_topk.py:13-260) over libredmetal_hip.so: same
methods and argument meaning (create / load / addresses / execute / telemetry), numpy arrays instead of Python lists, plus the
stream-ordered entry points of include/redmetal_topk.h on device addresses."""
import ctypes as C
import os

import numpy as np

from ._lib import RedHipError, load
from .redmetal_ffn import ExpertLayout          # noqa: F401  (byte ranges of one expert inside the model file)

TOPK_MAX = 512


def _u32(a):
    return np.ascontiguousarray(a, np.uint32)


def _u64(a):
    return np.ascontiguousarray(a, np.uint64)


class RedMetalTopKPool:
    def __init__(self, model, budget_bytes, slot_bytes, *, slots_per_slab=64, iq2_xs_grid, iq1_m_grid):
        if budget_bytes <= 0 or slot_bytes <= 0:
            raise ValueError("budget_bytes and slot_bytes must be positive")
        self.lib = load()
        # the reference reads the two codebooks from a llama.cpp checkout (redlite/quant_tables.py); here the caller passes them
        self._iq2 = np.ascontiguousarray(iq2_xs_grid, np.int8).ravel()
        self._iq1 = np.ascontiguousarray(iq1_m_grid, np.int8).ravel()
        self.model = os.path.abspath(os.path.expanduser(str(model)))
        self.handle = self.lib.redmetal_topk_pool_create(os.fsencode(self.model), int(budget_bytes), int(slot_bytes), int(slots_per_slab),
                                                         self._iq2.ctypes.data, self._iq2.size, self._iq1.ctypes.data, self._iq1.size)
        if not self.handle:
            raise RedHipError(self._last_error())

    def _last_error(self):
        raw = self.lib.redmetal_topk_last_error()
        return raw.decode("utf-8", errors="replace") if raw else "unknown Red Metal top-k error"

    def _check(self, ok):
        if not ok:
            raise RedHipError(self._last_error())

    def close(self):
        if self.handle:
            self.lib.redmetal_topk_pool_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *_):
        self.close()

    @property
    def capacity(self):
        return int(self.lib.redmetal_topk_pool_capacity(self.handle))

    def set_classes(self, slot_bytes, capacity):
        sb, cp = _u64(slot_bytes), _u32(capacity)
        self._check(self.lib.redmetal_topk_pool_set_classes(self.handle, sb.size, sb.ctypes.data, cp.ctypes.data))

    def enable_fast_path(self, type_word, hidden, ffn, tiles=False):
        """experts of this shape (all IQ2_XXS) also keep a copy in the fused kernels' layout behind their slot's raw bytes (written at
        load); their single-token calls then run on it, and with `tiles` (a third, tile-major copy) the batched form runs on the prefill
        tile kernels. Before the first slab exists; the copies count against the budget."""
        self._check(self.lib.redhip_topk_pool_enable_fast_path(self.handle, int(type_word), int(hidden), int(ffn), 1 if tiles else 0))

    def slot_inflight(self, slot_id):
        return bool(self.lib.redmetal_topk_pool_slot_inflight(self.handle, slot_id))

    def slot_generation(self, slot_id):
        return int(self.lib.redmetal_topk_pool_slot_generation(self.handle, slot_id))

    def load(self, slot_id, layout):
        read, ms = C.c_uint64(), C.c_double()
        self._check(self.lib.redmetal_topk_pool_load_expert(self.handle, slot_id, layout.gate_offset, layout.gate_bytes, layout.up_offset,
                                                            layout.up_bytes, layout.down_offset, layout.down_bytes, C.byref(read), C.byref(ms)))
        return {"bytes_read": int(read.value), "elapsed_ms": float(ms.value)}

    def addresses(self, slot_id, layout):
        g, u, d = C.c_uint64(), C.c_uint64(), C.c_uint64()
        self._check(self.lib.redmetal_topk_pool_slot_addresses(self.handle, slot_id, layout.gate_bytes, layout.up_bytes, layout.down_bytes,
                                                               C.byref(g), C.byref(u), C.byref(d)))
        return int(g.value), int(u.value), int(d.value)

    @staticmethod
    def _lists(slot_ids, layouts):
        ids = _u32(slot_ids)
        return ids, _u64([l.gate_bytes for l in layouts]), _u64([l.up_bytes for l in layouts]), _u64([l.down_bytes for l in layouts])

    def execute(self, slot_ids, layouts, router_weights, ggml_type, hidden_size, ffn_size, output_row_start, output_row_count, input_values):
        """redlite/redmetal_topk.py:192-250: (output rows, elapsed ms) of the weighted top-k FFN over resident slots, host arrays"""
        ids, gb, ub, db = self._lists(slot_ids, layouts)
        w = np.ascontiguousarray(router_weights, np.float32)
        x = np.ascontiguousarray(input_values, np.float32)
        if not (ids.size == w.size == len(layouts)):
            raise ValueError("slot_ids, layouts and router_weights must have the same length")
        if x.size != hidden_size:
            raise ValueError("input has %d values, expected %d" % (x.size, hidden_size))
        out = np.zeros(max(output_row_count, 1), np.float32)
        ms = C.c_double()
        self._check(self.lib.redmetal_topk_pool_execute(self.handle, ids.ctypes.data, gb.ctypes.data, ub.ctypes.data, db.ctypes.data, w.ctypes.data,
                                                        ids.size, int(ggml_type), hidden_size, ffn_size, output_row_start, output_row_count,
                                                        x.ctypes.data, x.size, out.ctypes.data, output_row_count, C.byref(ms)))
        return out[:output_row_count], float(ms.value)

    # ---- stream-ordered forms: device addresses (int), `stream` a hipStream_t value or None ----

    def encode(self, stream, slot_ids, layouts, router_weights, ggml_type, hidden_size, ffn_size, output_row_start, output_row_count,
               x_dev, out_dev, x_offset=0, out_offset=0):
        ids, gb, ub, db = self._lists(slot_ids, layouts)
        w = np.ascontiguousarray(router_weights, np.float32)
        self._check(self.lib.redmetal_topk_pool_encode(self.handle, stream, ids.ctypes.data, gb.ctypes.data, ub.ctypes.data, db.ctypes.data, w.ctypes.data,
                                                       ids.size, int(ggml_type), hidden_size, ffn_size, output_row_start, output_row_count,
                                                       int(x_dev), x_offset, int(out_dev), out_offset))

    def release(self, slot_ids):
        ids = _u32(slot_ids)
        self.lib.redmetal_topk_pool_release(self.handle, ids.ctypes.data, ids.size)

    def residency_table_init(self, layers, experts):
        self._check(self.lib.redmetal_topk_pool_residency_table_init(self.handle, layers, experts))
        return int(self.lib.redmetal_topk_pool_residency_table(self.handle))

    def residency_set(self, layer, expert, slot_id):
        self._check(self.lib.redmetal_topk_pool_residency_set(self.handle, layer, expert, slot_id))

    def residency_clear(self, layer, expert):
        self.lib.redmetal_topk_pool_residency_clear(self.handle, layer, expert)

    def allocate_all(self):
        self._check(self.lib.redmetal_topk_pool_allocate_all(self.handle))

    def tmp_buffer(self):
        return self.lib.redmetal_topk_pool_tmp_buffer(self.handle)

    def encode_device_into(self, stream, slot_table_dev, weight_dev, top_k, ggml_type, hidden_size, ffn_size, gate_bytes, up_bytes, x_dev, out_dev,
                           x1_dev=None, x_split=0, table_offset=0, weight_offset=0):
        """slot base addresses (uint64) and weights (float32) read from device memory; out_dev None leaves tmp[e][r] to the caller;
        with x1_dev the experts from x_split on read the second vector"""
        if x1_dev is None:
            ok = self.lib.redmetal_topk_pool_encode_device_into(self.handle, stream, int(slot_table_dev), table_offset, int(weight_dev), weight_offset,
                                                                top_k, int(ggml_type), hidden_size, ffn_size, gate_bytes, up_bytes, int(x_dev), 0,
                                                                None if out_dev is None else int(out_dev), 0)
        else:
            ok = self.lib.redmetal_topk_pool_encode_device_into2(self.handle, stream, int(slot_table_dev), table_offset, int(weight_dev), weight_offset,
                                                                 top_k, int(ggml_type), hidden_size, ffn_size, gate_bytes, up_bytes, int(x_dev), 0,
                                                                 None if out_dev is None else int(out_dev), 0, int(x1_dev), 0, x_split)
        self._check(ok)

    def encode_device_tail(self, stream, slot_table_dev, weight_dev, top_k, ggml_type, hidden_size, ffn_size, gate_bytes, up_bytes, x_in_dev,
                           resid_dev, shared_dev, scalar_dev, x_dev, layer_out_dev):
        r = self.lib.redmetal_topk_pool_encode_device_tail(self.handle, stream, int(slot_table_dev), 0, int(weight_dev), 0, top_k, int(ggml_type),
                                                           hidden_size, ffn_size, gate_bytes, up_bytes, int(x_in_dev), 0, int(resid_dev), int(shared_dev),
                                                           int(scalar_dev), int(x_dev), int(layer_out_dev), 0)
        if r == 0:
            raise RedHipError(self._last_error())
        return r                                   # 1 enqueued, -1 shape not served by the fused tail

    def encode_batched(self, stream, slot_ids, layouts, ggml_type, hidden_size, ffn_size, tok_first, ntok, top_k, pair_token, pair_weight,
                       expert_start, tok_pair, x_dev, out_dev):
        ids, gb, ub, db = self._lists(slot_ids, layouts)
        pt, pw, es, tp = _u32(pair_token), np.ascontiguousarray(pair_weight, np.float32), _u32(expert_start), _u32(tok_pair)
        self._check(self.lib.redmetal_topk_pool_encode_batched(self.handle, stream, ids.ctypes.data, gb.ctypes.data, ub.ctypes.data, db.ctypes.data,
                                                               ids.size, int(ggml_type), hidden_size, ffn_size, tok_first, ntok, top_k, pt.size,
                                                               pt.ctypes.data, pw.ctypes.data, es.ctypes.data, tp.ctypes.data,
                                                               int(x_dev), 0, int(out_dev), 0))

    def encode_mapped(self, stream, gate_addr0, up_addr0, down_addr0, gate_bytes, up_bytes, down_bytes, expert_ids, ggml_type, hidden_size, ffn_size,
                      tok_first, ntok, top_k, pair_token, pair_weight, expert_start, tok_pair, x_dev, out_dev):
        ids = _u32(expert_ids)
        pt, pw, es, tp = _u32(pair_token), np.ascontiguousarray(pair_weight, np.float32), _u32(expert_start), _u32(tok_pair)
        self._check(self.lib.redmetal_topk_pool_encode_mapped(self.handle, stream, None, int(gate_addr0), None, int(up_addr0), None, int(down_addr0),
                                                              gate_bytes, up_bytes, down_bytes, ids.ctypes.data, ids.size, int(ggml_type),
                                                              hidden_size, ffn_size, tok_first, ntok, top_k, pt.size, pt.ctypes.data, pw.ctypes.data,
                                                              es.ctypes.data, tp.ctypes.data, int(x_dev), 0, int(out_dev), 0))

    def telemetry(self):
        L, h = self.lib, self.handle
        return {"capacity": self.capacity, "slab_count": int(L.redmetal_topk_pool_slab_count(h)),
                "allocated_bytes": int(L.redmetal_topk_pool_allocated_bytes(h)), "bytes_read": int(L.redmetal_topk_pool_bytes_read(h)),
                "read_calls": int(L.redmetal_topk_pool_read_calls(h)), "read_ms": float(L.redmetal_topk_pool_read_ms(h))}
