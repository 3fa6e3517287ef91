"""Resident MoE FFN layers (include/redhip_moe.h). torch owns the activation buffers and the stream; weights are
uploaded once and stay in HBM."""
import ctypes as C
import os

import numpy as np
import torch

from . import expert_type_word
from ._lib import MoeConfig, RedHipError, load


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, torch.Tensor):
        assert t.is_contiguous()
        return t.data_ptr()
    return np.ascontiguousarray(t).ctypes.data


def _stream():
    return torch.cuda.current_stream().cuda_stream


class ResidentMoe:
    def __init__(self, cfg, n_layer=1, max_tokens=1):
        """cfg: dict as produced by synth.layer_config (hidden, ffn, n_expert, top_k and the five type fields)."""
        self.lib = load()
        self.cfg = dict(cfg)
        self.n_layer, self.max_tokens = n_layer, max_tokens
        c = MoeConfig(cfg["hidden"], cfg["ffn"], cfg["n_expert"], cfg["top_k"], n_layer, max_tokens, cfg["router_type"],
                      expert_type_word(cfg["gate_up_type"], cfg["down_type"]),
                      expert_type_word(cfg["sh_gate_up_type"], cfg["sh_down_type"]), 0)
        torch.cuda.init()
        self.handle = self.lib.redhip_moe_create(C.byref(c))
        if not self.handle:
            raise RedHipError(self._err())

    @classmethod
    def from_gguf(cls, path, first_layer=0, n_layer=None, max_tokens=1):
        """Resident layers straight from a GGUF file: shapes, types and top_k come from the file."""
        cfg, in_file = gguf_moe_config(path, first_layer)
        n = in_file if n_layer is None else n_layer
        m = cls(cfg, n_layer=n, max_tokens=max_tokens)
        m.load_gguf(path, first_layer, n)
        return m

    def load_gguf(self, path, first_layer=0, n_layer=None):
        cfg = self.cfg
        c = MoeConfig(cfg["hidden"], cfg["ffn"], cfg["n_expert"], cfg["top_k"], self.n_layer, self.max_tokens, cfg["router_type"],
                      expert_type_word(cfg["gate_up_type"], cfg["down_type"]),
                      expert_type_word(cfg["sh_gate_up_type"], cfg["sh_down_type"]), 0)
        if not self.lib.redhip_moe_load_gguf(self.handle, os.fsencode(path), first_layer, self.n_layer if n_layer is None else n_layer, C.byref(c)):
            raise RedHipError(self.lib.redhip_gguf_last_error().decode("utf-8", errors="replace"))

    def _err(self):
        raw = self.lib.redhip_moe_last_error()
        return raw.decode("utf-8", errors="replace") if raw else "unknown redhip MoE error"

    def _check(self, ok):
        if not ok:
            raise RedHipError(self._err())

    def close(self):
        if self.handle:
            self.lib.redhip_moe_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def resident_bytes(self):
        return int(self.lib.redhip_moe_resident_bytes(self.handle))

    # ---- uploads (numpy arrays or torch tensors, host or device) ----
    def load_layer(self, layer, arrays):
        """arrays: dict with router, gate, up, down, sh_gate, sh_up, sh_down, sh_gate_inp (raw GGUF bytes)."""
        a = arrays
        nbytes = lambda t: t.numel() * t.element_size() if isinstance(t, torch.Tensor) else np.asarray(t).nbytes
        self._check(self.lib.redhip_moe_load_router(self.handle, layer, _ptr(a["router"]), nbytes(a["router"])))
        self._check(self.lib.redhip_moe_load_shared(self.handle, layer, _ptr(a["sh_gate_inp"]), _ptr(a["sh_gate"]), nbytes(a["sh_gate"]),
                                                    _ptr(a["sh_up"]), nbytes(a["sh_up"]), _ptr(a["sh_down"]), nbytes(a["sh_down"])))
        self.load_experts(layer, 0, self.cfg["n_expert"], a["gate"], a["up"], a["down"])

    def load_experts(self, layer, first, count, gate, up, down):
        self._check(self.lib.redhip_moe_load_experts(self.handle, layer, first, count, _ptr(gate), _ptr(up), _ptr(down)))

    # ---- execution (torch CUDA tensors, current stream) ----
    def forward(self, layer, x, out=None):
        x = x.reshape(-1, self.cfg["hidden"])
        assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()
        if out is None:
            out = torch.empty_like(x)
        self._check(self.lib.redhip_moe_forward(self.handle, layer, x.data_ptr(), x.shape[0], out.data_ptr(), _stream()))
        return out

    def forward_block(self, layer, x, branch, post_norm, eps=1e-6, out=None):
        """x_out = (x + branch) + layer(rmsnorm(x + branch) * post_norm): the layer with the residual steps around it."""
        x = x.reshape(-1, self.cfg["hidden"])
        branch = branch.reshape(-1, self.cfg["hidden"])
        for t in (x, branch, post_norm):
            assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
        assert branch.shape == x.shape and post_norm.numel() == self.cfg["hidden"]
        if out is None:
            out = torch.empty_like(x)
        self._check(self.lib.redhip_moe_forward_block(self.handle, layer, x.data_ptr(), branch.data_ptr(), post_norm.data_ptr(), float(eps),
                                                      x.shape[0], out.data_ptr(), _stream()))
        return out

    def route(self, layer, x):
        x = x.reshape(-1, self.cfg["hidden"])
        n, K, E = x.shape[0], self.cfg["top_k"], self.cfg["n_expert"]
        ids = torch.empty((n, K), dtype=torch.int32, device=x.device)
        w = torch.empty((n, K), dtype=torch.float32, device=x.device)
        logits = torch.empty((n, E), dtype=torch.float32, device=x.device)
        self._check(self.lib.redhip_moe_route(self.handle, layer, x.data_ptr(), n, ids.data_ptr(), w.data_ptr(), logits.data_ptr(), _stream()))
        return ids, w, logits

    def experts(self, layer, x, ids, weights, out=None):
        x = x.reshape(-1, self.cfg["hidden"])
        if out is None:
            out = torch.empty_like(x)
        self._check(self.lib.redhip_moe_experts(self.handle, layer, x.data_ptr(), x.shape[0], ids.data_ptr(), weights.data_ptr(),
                                                out.data_ptr(), _stream()))
        return out

    def last_route(self, ntok):
        K, E = self.cfg["top_k"], self.cfg["n_expert"]
        ids = np.empty((ntok, K), np.uint32)
        w = np.empty((ntok, K), np.float32)
        logits = np.empty((ntok, E), np.float32)
        self._check(self.lib.redhip_moe_last_route(self.handle, ntok, ids.ctypes.data, w.ctypes.data, logits.ctypes.data, _stream()))
        return ids, w, logits

    def group(self, ids, weights):
        n, K = ids.shape
        P, dev = n * K, ids.device
        U_cap = min(P, self.cfg["n_expert"])
        uid = torch.zeros(U_cap, dtype=torch.int32, device=dev)
        start = torch.zeros(U_cap + 1, dtype=torch.int32, device=dev)
        ptok = torch.zeros(P, dtype=torch.int32, device=dev)
        pw = torch.zeros(P, dtype=torch.float32, device=dev)
        tp = torch.zeros(P, dtype=torch.int32, device=dev)
        nu = torch.zeros(1, dtype=torch.int32, device=dev)
        self._check(self.lib.redhip_moe_group(self.handle, ids.data_ptr(), weights.data_ptr(), n, uid.data_ptr(), start.data_ptr(),
                                              ptok.data_ptr(), pw.data_ptr(), tp.data_ptr(), nu.data_ptr(), _stream()))
        U = int(nu.item())
        return uid[:U], start[:U + 1], ptok, pw, tp

    def dequant_resident(self, layer, expert, which):
        H, F, E = self.cfg["hidden"], self.cfg["ffn"], self.cfg["n_expert"]
        shape = (E, H) if which == 3 else ((F, H) if which < 2 else (H, F))      # which 4: the column-sliced copy of a down matrix
        out = torch.empty(shape, dtype=torch.float32, device="cuda")
        self._check(self.lib.redhip_moe_dequant_resident(self.handle, layer, expert, which, out.data_ptr(), _stream()))
        return out


def gguf_moe_config(path, first_layer=0):
    """(cfg dict as synth.layer_config gives it, number of consecutive MoE layers from first_layer) of a GGUF file. Host only."""
    lib = load()
    c = MoeConfig()
    if not lib.redhip_gguf_moe_config(os.fsencode(path), first_layer, C.byref(c)):
        raise RedHipError(lib.redhip_gguf_last_error().decode("utf-8", errors="replace"))
    gu, dn = c.expert_type_word & 255, (c.expert_type_word >> 8) or (c.expert_type_word & 255)
    sgu, sdn = c.shared_type_word & 255, (c.shared_type_word >> 8) or (c.shared_type_word & 255)
    cfg = dict(hidden=c.hidden, ffn=c.ffn, n_expert=c.n_expert, top_k=c.top_k, router_type=c.router_type, gate_up_type=gu, down_type=dn,
               sh_gate_up_type=sgu, sh_down_type=sdn)
    return cfg, c.n_layer


def gguf_expert_layout(path, n_expert, layer, expert):
    """dict of the reference's rl_expert_layout fields (native/redlite_native_gguf.h:47-59) for one routed expert of a GGUF file:
    quantisation types and the absolute byte ranges of its gate / up / down matrices. Host only."""
    from ._lib import GgufExpertLayout
    lib = load()
    out = GgufExpertLayout()
    if not lib.redhip_gguf_expert_layout(os.fsencode(path), n_expert, layer, expert, C.byref(out)):
        raise RedHipError(lib.redhip_gguf_last_error().decode("utf-8", errors="replace"))
    return {n: int(getattr(out, n)) for n, _ in GgufExpertLayout._fields_}


def set_codebooks(iq2_xs_grid=None, iq1_m_grid=None):
    """upload the int8 codebooks (512 x 8 and 2048 x 8 values) that IQ2_XS / IQ1_M rows decode through."""
    lib = load()
    a = np.ascontiguousarray(iq2_xs_grid, np.int8).ravel() if iq2_xs_grid is not None else None
    b = np.ascontiguousarray(iq1_m_grid, np.int8).ravel() if iq1_m_grid is not None else None
    if not lib.redhip_set_codebooks(a.ctypes.data if a is not None else None, a.size if a is not None else 0,
                                    b.ctypes.data if b is not None else None, b.size if b is not None else 0):
        raise RedHipError(lib.redhip_moe_last_error().decode())


def dequant_rows(ggml_type, rows, ncols):
    """rows: uint8 CUDA tensor [nrows, row_bytes] of raw GGUF blocks -> float32 [nrows, ncols]."""
    lib = load()
    rows = rows.contiguous()
    out = torch.empty((rows.shape[0], ncols), dtype=torch.float32, device=rows.device)
    if not lib.redhip_dequant_rows(ggml_type, rows.data_ptr(), rows.shape[0], ncols, out.data_ptr(), _stream()):
        raise RedHipError(lib.redhip_moe_last_error().decode())
    return out


def gemv_rows(ggml_type, matrix, ncols, x, row_start=0, row_count=None):
    lib = load()
    nrows = matrix.shape[0]
    if row_count is None:
        row_count = nrows - row_start
    out = torch.empty(row_count, dtype=torch.float32, device=x.device)
    if not lib.redhip_gemv_rows(ggml_type, matrix.data_ptr(), ncols, row_start, row_count, x.data_ptr(), out.data_ptr(), _stream()):
        raise RedHipError(lib.redhip_moe_last_error().decode())
    return out
