"""Host-side mirror of the reference's single-expert FFN pool bridge (redlite/redmetal_ffn.py:13-225) over
libredmetal_hip.so. Same methods and argument meaning; numpy arrays instead of Python lists."""
import ctypes as C
import os
from collections import namedtuple

import numpy as np

from ._lib import RedHipError, load

# byte range of one expert's three matrices inside the model file (the reference's ExpertLayout parts)
ExpertLayout = namedtuple("ExpertLayout", "gate_offset gate_bytes up_offset up_bytes down_offset down_bytes")


class RedMetalFfnPool:
    def __init__(self, model, budget_bytes, slot_bytes, *, slots_per_slab=64, iq2_xs_grid=None, iq1_m_grid=None):
        if budget_bytes <= 0 or slot_bytes <= 0:
            raise ValueError("budget_bytes and slot_bytes must be positive")
        self.lib = load()
        # the reference's signature: two int8 codebooks with exact element counts (it reads them from a llama.cpp checkout,
        # redlite/quant_tables.py). The caller passes them here; without them the pool still serves the formats that carry
        # their own tables, and execute() refuses IQ2_XS / IQ1_M
        self._have_grids = iq2_xs_grid is not None and iq1_m_grid is not None
        self._iq2 = (C.c_int8 * (512 * 8))(*(np.asarray(iq2_xs_grid, np.int8).ravel().tolist() if iq2_xs_grid is not None else ()))
        self._iq1 = (C.c_int8 * (2048 * 8))(*(np.asarray(iq1_m_grid, np.int8).ravel().tolist() if iq1_m_grid is not None else ()))
        self.model = os.path.abspath(os.path.expanduser(str(model)))
        self.handle = self.lib.redmetal_ffn_pool_create(os.fsencode(self.model), int(budget_bytes), int(slot_bytes),
                                                        int(slots_per_slab), self._iq2, len(self._iq2), self._iq1, len(self._iq1))
        if not self.handle:
            raise RedHipError(self._last_error())

    def _last_error(self):
        raw = self.lib.redmetal_ffn_last_error()
        return raw.decode("utf-8", errors="replace") if raw else "unknown Red Metal FFN error"

    def close(self):
        if self.handle:
            self.lib.redmetal_ffn_pool_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *_):
        self.close()

    @property
    def capacity(self):
        return int(self.lib.redmetal_ffn_pool_capacity(self.handle))

    def slot_inflight(self, slot_id):
        return bool(self.lib.redmetal_ffn_pool_slot_inflight(self.handle, slot_id))

    def load(self, slot_id, layout):
        read, ms = C.c_uint64(), C.c_double()
        ok = self.lib.redmetal_ffn_pool_load_expert(self.handle, slot_id, layout.gate_offset, layout.gate_bytes, layout.up_offset,
                                                    layout.up_bytes, layout.down_offset, layout.down_bytes, C.byref(read), C.byref(ms))
        if not ok:
            raise RedHipError(self._last_error())
        return {"bytes_read": int(read.value), "elapsed_ms": float(ms.value)}

    def addresses(self, slot_id, layout):
        g, u, d = C.c_uint64(), C.c_uint64(), C.c_uint64()
        ok = self.lib.redmetal_ffn_pool_slot_addresses(self.handle, slot_id, layout.gate_bytes, layout.up_bytes, layout.down_bytes,
                                                       C.byref(g), C.byref(u), C.byref(d))
        if not ok:
            raise RedHipError(self._last_error())
        return int(g.value), int(u.value), int(d.value)

    def execute(self, slot_id, layout, ggml_type, hidden_size, ffn_size, output_row_start, output_row_count, input_values):
        x = np.ascontiguousarray(input_values, np.float32)
        if x.size != hidden_size:
            raise ValueError("input has %d values, expected %d" % (x.size, hidden_size))
        if not self._have_grids and {ggml_type & 255, (ggml_type >> 8) & 255} & {17, 29}:
            raise ValueError("IQ2_XS / IQ1_M experts need the pool created with iq2_xs_grid and iq1_m_grid")
        out = np.zeros(max(output_row_count, 1), np.float32)
        ms = C.c_double()
        ok = self.lib.redmetal_ffn_pool_execute_expert(self.handle, slot_id, int(ggml_type), layout.gate_bytes, layout.up_bytes,
                                                       layout.down_bytes, hidden_size, ffn_size, output_row_start, output_row_count,
                                                       x.ctypes.data, hidden_size, out.ctypes.data, output_row_count, C.byref(ms))
        if not ok:
            raise RedHipError(self._last_error())
        return out[:output_row_count], float(ms.value)

    def execute_noalloc(self, slot_id, layout, ggml_type, hidden_size, ffn_size, output_row_start, output_row_count, x_dev, out_dev, stream=None):
        """The same computation enqueued on `stream` (a hipStream_t value) with device pointers and no device allocation: x_dev / out_dev are
        device addresses (int) of float32 [hidden] / [output_row_count]. Returns once the two launches are enqueued."""
        ok = self.lib.redmetal_ffn_pool_execute_expert_noalloc(self.handle, slot_id, int(ggml_type), layout.gate_bytes, layout.up_bytes,
                                                               layout.down_bytes, hidden_size, ffn_size, output_row_start, output_row_count,
                                                               int(x_dev), hidden_size, int(out_dev), output_row_count, stream)
        if not ok:
            raise RedHipError(self._last_error())

    def telemetry(self):
        L, h = self.lib, self.handle
        return {"capacity": self.capacity, "slab_count": int(L.redmetal_ffn_pool_slab_count(h)),
                "allocated_bytes": int(L.redmetal_ffn_pool_allocated_bytes(h)), "bytes_read": int(L.redmetal_ffn_pool_bytes_read(h)),
                "read_calls": int(L.redmetal_ffn_pool_read_calls(h)), "read_ms": float(L.redmetal_ffn_pool_read_ms(h))}
