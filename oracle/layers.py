"""PyTorch-CPU restatement of the E.T. encoder-layer mathematics (test oracle).

Everything is computed in fp32 on the CPU.  ``store`` selects the storage type
of activations: ``None`` keeps fp32 throughout (the plain mathematics);
``torch.float16`` rounds to fp16 exactly where the GPU engine writes fp16 to
memory (after each Linear incl. its fused bias/activation, after the attention
output, after each LayerNorm) and where it feeds fp16 operands to the matrix
cores (the un-normalised softmax probabilities).  ``LayerConfig.resid`` selects
the storage of the residual stream separately: with ``resid=torch.float32`` and
``store=torch.float16`` (the engine's mixed-precision mode) the outputs of the
two projections that feed a SkipLayerNorm and the SkipLayerNorm results stay
fp32, and fp16 rounding happens only where a value becomes a matrix-core
operand.

Weights are applied as masked dense ``[out, in]`` matrices; sparse containers
are expanded with ``oracle.formats.*_to_dense`` first.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import torch
import torch.nn.functional as F


def _store(x: torch.Tensor, store) -> torch.Tensor:
    return x if store is None else x.to(store).to(torch.float32)


# -- activations ---------------------------------------------------------------

def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """x*(0.5 + 0.5*tanh(x*(0.035677408*x^2 + 0.7978845608))) — Encoder/Encoder.cu:25-37."""
    return x * (0.5 + 0.5 * torch.tanh(x * (0.035677408136 * x * x + 0.7978845608028654)))


def relu(x: torch.Tensor) -> torch.Tensor:
    """Encoder/Encoder.h:29-33."""
    return torch.clamp_min(x, 0.0)


ACTS = {None: lambda x: x, "none": lambda x: x, "relu": relu, "gelu": gelu_tanh}


# -- Linear ----------------------------------------------------------------------

def linear(x, W, b=None, act=None, store=None):
    """y = act(x W^T + b), W the masked dense [out, in] matrix (Linear/Linear.h:11-15,
    operand orientation Linear/SPMM_tile.cu:275-308).  One rounding at the end:
    the engine applies bias and activation on the fp32 accumulator."""
    y = x.to(torch.float32) @ W.to(torch.float32).T
    if b is not None:
        y = y + b.to(torch.float32)
    return _store(ACTS[act](y), store)


def linear_rowpruned(x, rows, row_id, out, b=None, act=None, store=None):
    """Output-feature pruning (Linear/SPMM_row.cu:62-75): live columns of y get
    x.w + b, pruned columns get b alone (the reference leaves them stale)."""
    T = x.shape[0]
    y = torch.zeros(T, out, dtype=torch.float32)
    y[:, torch.as_tensor(row_id, dtype=torch.long)] = x.to(torch.float32) @ rows.to(torch.float32).T
    if b is not None:
        y = y + b.to(torch.float32)
    return _store(ACTS[act](y), store)


def linear_colpruned(x, cols, col_id, b=None, act=None, store=None):
    """Input-feature pruning (Linear/SPMM_col.cu:25-69): y = x[:, col_id] cols^T + b."""
    xg = x.to(torch.float32)[:, torch.as_tensor(col_id, dtype=torch.long)]
    y = xg @ cols.to(torch.float32).T
    if b is not None:
        y = y + b.to(torch.float32)
    return _store(ACTS[act](y), store)


# -- normalisation -------------------------------------------------------------

def layernorm(x, gamma, beta, eps=1e-5, store=None):
    """LayerNorm/LayerNorm.cu:9-35 with the intended variance E[(x-mean)^2]."""
    x = x.to(torch.float32)
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    y = (x - mean) / torch.sqrt(var + eps) * gamma.to(torch.float32) + beta.to(torch.float32)
    return _store(y, store)


def skip_layernorm(src, skip, gamma, beta, eps=1e-5, store=None):
    """out = LN(src + skip)*gamma + beta (SkipLayerNorm/SkipLayerNorm.cu:22-63);
    the sum is formed in fp32."""
    return layernorm(src.to(torch.float32) + skip.to(torch.float32), gamma, beta, eps, store)


# -- attention -------------------------------------------------------------------

def additive_mask(S: int, kind: str = "none") -> Optional[torch.Tensor]:
    """``causal`` is the mask every reference attention constructor builds
    (Attention/Attention.h:96-104): 0 where j <= i, -inf elsewhere."""
    if kind == "none":
        return None
    if kind == "causal":
        i = torch.arange(S)
        return torch.where(i[None, :] <= i[:, None], 0.0, float("-inf")).to(torch.float32)
    raise ValueError(kind)


def mha(q, k, v, nh: int, B: int = 1, scale: Optional[float] = None, mask=None, lens=None,
        causal: bool = False, store=None, return_probs: bool = False):
    """softmax(scale * Q_h K_h^T + mask) V_h per head and sequence.

    q, k, v: [B*S, nh*hd]; head h is the column slice [h*hd, (h+1)*hd)
    (Attention/OTFkernel_full.h:34,49,116,122).  mask: additive [S, S] shared by
    all heads/sequences (OTFkernel_full.h:69-78).  lens[b]: keys >= lens[b] get
    probability 0.  With ``store=float16`` the un-normalised probabilities
    exp(s - max) are rounded to fp16 before P*V and the row sum is taken over
    the rounded values, as the engine does.
    """
    T, width = q.shape
    S = T // B
    hd = width // nh
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    qh = q.to(torch.float32).reshape(B, S, nh, hd).permute(0, 2, 1, 3)
    kh = k.to(torch.float32).reshape(B, S, nh, hd).permute(0, 2, 1, 3)
    vh = v.to(torch.float32).reshape(B, S, nh, v.shape[1] // nh).permute(0, 2, 1, 3)
    s = (qh @ kh.transpose(-1, -2)) * scale  # [B, nh, S, S]
    if mask is not None:
        s = s + mask.to(torch.float32)
    if causal:
        s = s + additive_mask(S, "causal")
    if lens is not None:
        key = torch.arange(S)[None, None, None, :]
        ln = torch.as_tensor(lens).reshape(B, 1, 1, 1)
        s = torch.where(key < ln, s, torch.full_like(s, float("-inf")))
    m = s.max(-1, keepdim=True).values
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    p = torch.exp(s - m)
    p = _store(p, store)
    l = p.sum(-1, keepdim=True)
    o = (p @ vh) / torch.where(l > 0, l, torch.ones_like(l))
    o = torch.where(l > 0, o, torch.zeros_like(o))
    z = o.permute(0, 2, 1, 3).reshape(T, -1)
    z = _store(z, store)
    if return_probs:
        return z, p / torch.where(l > 0, l, torch.ones_like(l))
    return z


def fused_vo_attention(x_q, x_k, x_v, Wq, bq, Wk, bk, Wvo, bvo, bo, nh: int, B: int = 1,
                       scale=None, mask=None, lens=None, causal=False, store=None):
    """The pre-computed-VO attention (Fused_attention/Fused_attention.h:93-116):
    VO_h = X W_VO,h + b_VO,h  ([nh][S][H], Fused_attention/Linear_VO.h:39-58),
    out = sum_h P_h VO_h + b_O.  Wvo: [nh, H, N] row-major, bvo: [nh, N]."""
    T = x_q.shape[0]
    S = T // B
    q = linear(x_q, Wq, bq, store=store)
    k = linear(x_k, Wk, bk, store=store)
    hd = q.shape[1] // nh
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    N = Wvo.shape[2]
    out = torch.zeros(T, N, dtype=torch.float32)
    qh = q.reshape(B, S, nh, hd)
    kh = k.reshape(B, S, nh, hd)
    for h in range(nh):
        vo = _store(x_v.to(torch.float32) @ Wvo[h].to(torch.float32) + bvo[h].to(torch.float32), store)
        vo = vo.reshape(B, S, N)
        for b in range(B):
            s = (qh[b, :, h] @ kh[b, :, h].T) * scale
            if mask is not None:
                s = s + mask
            if causal:
                s = s + additive_mask(S, "causal")
            if lens is not None:
                s[:, int(lens[b]):] = float("-inf")
            m = s.max(-1, keepdim=True).values
            m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
            p = _store(torch.exp(s - m), store)
            l = p.sum(-1, keepdim=True)
            out[b * S:(b + 1) * S] += (p @ vo[b]) / torch.where(l > 0, l, torch.ones_like(l))
    out = out + bo.to(torch.float32)
    return _store(out, store)


# -- encoder layer -----------------------------------------------------------------

@dataclass
class LayerParams:
    """Masked dense weights of one encoder layer ([out, in] fp32 tensors)."""
    Wqkv: torch.Tensor  # [3H, H]: rows [0,H) = Q, [H,2H) = K, [2H,3H) = V (Attention/Attention.h:258-260)
    bqkv: torch.Tensor
    Wo: torch.Tensor
    bo: torch.Tensor
    W1: torch.Tensor  # [dimFF, H]
    b1: torch.Tensor
    W2: torch.Tensor  # [H, dimFF]
    b2: torch.Tensor
    g1: torch.Tensor
    be1: torch.Tensor
    g2: torch.Tensor
    be2: torch.Tensor


@dataclass
class LayerConfig:
    nh: int
    B: int = 1
    act: str = "gelu"
    eps: float = 1e-5
    causal: bool = False
    mask: Optional[torch.Tensor] = None
    lens: Optional[torch.Tensor] = None
    store: object = None
    resid: object = "same"  # storage of the residual stream; "same" = as ``store``
    fused_act: bool = True  # activation applied on the fp32 accumulator of linear1
    boundary: object = None  # storage of a layer's result where it is handed to the next layer (None: as the residual stream)
    extras: dict = field(default_factory=dict)


def _resid_store(cfg: LayerConfig):
    return cfg.store if isinstance(cfg.resid, str) else cfg.resid


def attention_block(x, P: LayerParams, cfg: LayerConfig):
    """One Linear H -> 3H, attention over column slices, output Linear
    (Attention/Attention.h:246-265).  x is rounded to the operand type on its
    way into the projection; the output projection is stored as the residual
    stream is."""
    H = P.Wo.shape[1]
    qkv = linear(_store(x, cfg.store), P.Wqkv, P.bqkv, store=cfg.store)
    q, k, v = qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:]
    z = mha(q, k, v, cfg.nh, cfg.B, mask=cfg.mask, lens=cfg.lens, causal=cfg.causal, store=cfg.store)
    return linear(z, P.Wo, P.bo, store=_resid_store(cfg))


def encoder_layer(x, P: LayerParams, cfg: LayerConfig):
    """attn -> SkipLN(attn, x) -> L1 -> act -> L2 -> SkipLN(L2, LN1)
    (Encoder/Encoder.h:81-96)."""
    rs = _resid_store(cfg)
    a = attention_block(x, P, cfg)
    y1 = skip_layernorm(a, x, P.g1, P.be1, cfg.eps, rs)
    y1_op = _store(y1, cfg.store)  # what linear1's matrix cores see
    if cfg.fused_act:
        f = linear(y1_op, P.W1, P.b1, act=cfg.act, store=cfg.store)
    else:
        f = _store(ACTS[cfg.act](linear(y1_op, P.W1, P.b1, store=cfg.store)), cfg.store)
    f2 = linear(f, P.W2, P.b2, store=rs)
    return skip_layernorm(f2, y1, P.g2, P.be2, cfg.eps, rs)


def encoder_stack(x, layers, cfg: LayerConfig):
    """Layer i feeds layer i+1 (example/main.cu:175-177)."""
    for P in layers:
        x = _store(encoder_layer(x, P, cfg), cfg.boundary)
    return x
