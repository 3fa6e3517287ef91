"""Seeded synthetic GGUF blocks, router matrices and activations.

Every bit pattern is a valid IQ2_XXS / IQ3_S / Q6_K block (8-bit grid indices, 7-bit signs, 4-bit scales; 9-bit
IQ3_S indices; int8 Q6_K scales), so a block is random bytes with its fp16 ``d`` field overwritten by a value drawn
uniformly from a realistic range. The same seed gives the same bytes on every machine (numpy PCG64).
"""
import numpy as np

TYPE_F32, TYPE_Q6_K, TYPE_IQ2_XXS, TYPE_IQ2_XS, TYPE_IQ3_S, TYPE_IQ1_M = 0, 14, 16, 17, 21, 29
BLOCK_BYTES = {TYPE_Q6_K: 210, TYPE_IQ2_XXS: 66, TYPE_IQ3_S: 110, TYPE_IQ2_XS: 74, TYPE_IQ1_M: 56}
D_OFFSET = {TYPE_Q6_K: 208, TYPE_IQ2_XXS: 0, TYPE_IQ3_S: 0, TYPE_IQ2_XS: 0}
# default fp16 scale ranges: IQ formats as in the benchmark definition; Q6_K smaller because its integer part
# (int8 scale x 6-bit quant) is ~70x larger
D_RANGE = {TYPE_IQ2_XXS: (1e-3, 2e-2), TYPE_IQ3_S: (1e-3, 2e-2), TYPE_Q6_K: (1e-4, 5e-4), TYPE_IQ2_XS: (1e-3, 2e-2), TYPE_IQ1_M: (1e-3, 2e-2)}


def row_bytes(t, ncols):
    if t == TYPE_F32:
        return 4 * ncols
    assert ncols % 256 == 0
    return BLOCK_BYTES[t] * (ncols // 256)


def quant_rows(rng, t, nrows, ncols, d_range=None):
    """uint8 [nrows, row_bytes]: random-valid blocks of type t."""
    bb = BLOCK_BYTES[t]
    nb = nrows * (ncols // 256)
    raw = rng.integers(0, 256, size=(nb, bb), dtype=np.uint8)
    lo, hi = d_range or D_RANGE[t]
    d = rng.uniform(lo, hi, size=nb).astype(np.float16).view(np.uint16)
    if t == TYPE_IQ1_M:          # d is spread over the top nibbles of the four 16-bit scale words (bytes 48..55)
        for i in range(4):
            raw[:, 49 + 2 * i] = (raw[:, 49 + 2 * i] & 0x0f) | ((((d >> (4 * i)) & 15) << 4).astype(np.uint8))
        return raw.reshape(nrows, -1)
    raw[:, D_OFFSET[t]] = (d & 255).astype(np.uint8)
    raw[:, D_OFFSET[t] + 1] = (d >> 8).astype(np.uint8)
    return raw.reshape(nrows, -1)


def normed_x(rng, ntok, hidden):
    """x ~ N(0,1), RMS-normalised with eps 1e-6 (float32 [ntok, hidden])."""
    x = rng.standard_normal((ntok, hidden)).astype(np.float32)
    x = x / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6)
    return x.astype(np.float32)


def layer_config(hidden=2048, ffn=512, n_expert=512, top_k=10, layout="iq2"):
    """layout 'iq2': everything IQ2_XXS, F32 router. layout 'f2': gate/up IQ2_XXS, down IQ3_S, shared expert
    and router Q6_K. layouts 'xs' / 'm': routed experts IQ2_XS / IQ1_M (what the reference's target file holds per
    layer), F32 router, Q6_K shared expert."""
    cfg = dict(hidden=hidden, ffn=ffn, n_expert=n_expert, top_k=top_k)
    if layout == "iq2":
        cfg.update(router_type=TYPE_F32, gate_up_type=TYPE_IQ2_XXS, down_type=TYPE_IQ2_XXS,
                   sh_gate_up_type=TYPE_IQ2_XXS, sh_down_type=TYPE_IQ2_XXS)
    elif layout == "f2":
        cfg.update(router_type=TYPE_Q6_K, gate_up_type=TYPE_IQ2_XXS, down_type=TYPE_IQ3_S,
                   sh_gate_up_type=TYPE_Q6_K, sh_down_type=TYPE_Q6_K)
    elif layout in ("xs", "m"):
        t = TYPE_IQ2_XS if layout == "xs" else TYPE_IQ1_M
        cfg.update(router_type=TYPE_F32, gate_up_type=t, down_type=t, sh_gate_up_type=TYPE_Q6_K, sh_down_type=TYPE_Q6_K)
    else:
        raise ValueError(layout)
    cfg["layout"] = layout
    return cfg


def make_layer(seed, cfg):
    """dict of numpy arrays holding one MoE layer in raw GGUF block layout (expert-major)."""
    rng = np.random.default_rng(seed)
    H, F, E = cfg["hidden"], cfg["ffn"], cfg["n_expert"]
    out = {}
    if cfg["router_type"] == TYPE_F32:
        out["router"] = (0.02 * rng.standard_normal((E, H))).astype(np.float32)
    else:
        # fp16-subnormal d keeps Q6_K router logits O(1); real files use subnormal d too
        out["router"] = quant_rows(rng, cfg["router_type"], E, H, d_range=(1e-5, 3e-5))
    out["gate"] = quant_rows(rng, cfg["gate_up_type"], E * F, H).reshape(E, -1)
    out["up"] = quant_rows(rng, cfg["gate_up_type"], E * F, H).reshape(E, -1)
    out["down"] = quant_rows(rng, cfg["down_type"], E * H, F).reshape(E, -1)
    out["sh_gate"] = quant_rows(rng, cfg["sh_gate_up_type"], F, H)
    out["sh_up"] = quant_rows(rng, cfg["sh_gate_up_type"], F, H)
    out["sh_down"] = quant_rows(rng, cfg["sh_down_type"], H, F)
    out["sh_gate_inp"] = (0.02 * rng.standard_normal(H)).astype(np.float32)
    return out


def hot_logits(rng, ntok, n_expert, n_hot=32, bias=2.0):
    """Router logits N(0,1) with a bias on a fixed set of hot experts (tokens overlap in their experts)."""
    l = rng.standard_normal((ntok, n_expert)).astype(np.float32)
    hot = (np.arange(n_hot) * 37) % n_expert
    l[:, hot] += np.float32(bias)
    return l


def zipf_topk(rng, ntok, n_expert, top_k, s=1.1):
    """Per token, top_k distinct experts drawn without replacement from a Zipf(s) popularity."""
    p = 1.0 / np.arange(1, n_expert + 1) ** s
    p /= p.sum()
    perm = rng.permutation(n_expert)
    ids = np.empty((ntok, top_k), np.uint32)
    for t in range(ntok):
        ids[t] = perm[rng.choice(n_expert, size=top_k, replace=False, p=p)]
    return ids


def make_layer_gpu(torch, gen, cfg):
    """The same construction as make_layer with torch's generator on the GPU (dict of CUDA tensors): random-valid blocks,
    d drawn from the format's range. For resident stacks too large to draw on the host in reasonable time."""
    def rows(t, nrows, ncols, d_range=None):
        bb = BLOCK_BYTES[t]
        nb = nrows * (ncols // 256)
        raw = torch.randint(0, 256, (nb, bb), dtype=torch.uint8, device="cuda", generator=gen)
        lo, hi = d_range or D_RANGE[t]
        d = (lo + (hi - lo) * torch.rand(nb, device="cuda", generator=gen)).to(torch.float16).view(torch.uint8).reshape(nb, 2)
        if t == TYPE_IQ1_M:          # d sits in the top nibbles of the four 16-bit scale words (bytes 48..55)
            for i in range(4):
                nib = (d[:, i // 2] >> (4 * (i % 2))) & 15
                raw[:, 49 + 2 * i] = (raw[:, 49 + 2 * i] & 0x0F) | (nib << 4)
        else:
            off = D_OFFSET[t]
            raw[:, off:off + 2] = d
        return raw.reshape(nrows, -1)

    H, F, E = cfg["hidden"], cfg["ffn"], cfg["n_expert"]
    a = {}
    if cfg["router_type"] == TYPE_F32:
        a["router"] = 0.02 * torch.randn((E, H), device="cuda", generator=gen)
    else:
        a["router"] = rows(cfg["router_type"], E, H, d_range=(1e-5, 3e-5))
    a["gate"] = rows(cfg["gate_up_type"], E * F, H).reshape(E, -1)
    a["up"] = rows(cfg["gate_up_type"], E * F, H).reshape(E, -1)
    a["down"] = rows(cfg["down_type"], E * H, F).reshape(E, -1)
    a["sh_gate"] = rows(cfg["sh_gate_up_type"], F, H)
    a["sh_up"] = rows(cfg["sh_gate_up_type"], F, H)
    a["sh_down"] = rows(cfg["sh_down_type"], H, F)
    a["sh_gate_inp"] = 0.02 * torch.randn(H, device="cuda", generator=gen)
    return a


def layer_to_host(a, cfg):
    """make_layer_gpu's tensors as the numpy arrays make_layer returns"""
    out = {k: v.cpu().numpy() for k, v in a.items()}
    if cfg["router_type"] != TYPE_F32:
        out["router"] = out["router"].view(np.uint8)
    return out
