"""
Ops for layer stacks with sandwich norms and depth-weighted averaging, and for decayed linear attention, on the
``src/_Cmix`` HIP extension (``csrc/kernels/lin_mix.hip``):

* :func:`embed_pos` — token vector plus a learned position vector, into the fp32 residual;
* :func:`post_pre_norm` — ``resid += rms(y + bias) * w_post`` and the next sublayer's input ``rms(resid) * w_pre``
  in one launch (a norm after one sublayer and before the next);
* :func:`depth_avg_norm` — a layer's last post-norm, the learned weighted average over the results of all layers so
  far, and the next layer's first norm (or the model's final norm) in one launch;
* :func:`bias_relu2` — ``relu(z + b)^2``; :func:`tanh_cap` — ``cap * tanh(z / cap)`` into fp32 (capped logits);
* :func:`head_gate`, :func:`norm_sigmoid_gate` — sigmoid output gates, one per head or one per channel after an RMS
  norm over all heads;
* :func:`lightning_attn` — linear attention with a fixed decay per head and an fp32 matrix state per (sequence,
  head), for prompt portions and decode rows alike.

rms(v) = v / sqrt(mean(v^2) + eps). GPU tensors always run the HIP kernels (a missing extension raises); CPU tensors
run the plain-PyTorch semantics below, which lets the engine's control flow run in CPU-only tests.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from .mix import _kern
from .seq import Ragged


def _rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def embed_pos(ids: torch.Tensor, positions: torch.Tensor, embed: torch.Tensor, pos: torch.Tensor,
              out: torch.Tensor) -> torch.Tensor:
    """out [T, W] fp32 (written) = embed[ids] + pos[positions]."""
    if ids.is_cuda:
        _kern().embed_pos(out, embed, pos, ids, positions)
        return out
    out.copy_(embed[ids].float() + pos[positions].float())
    return out


def post_pre_norm(resid: torch.Tensor, y: torch.Tensor, ybias: Optional[torch.Tensor], w_post: torch.Tensor,
                  w_pre: Optional[torch.Tensor], eps: float, out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """resid [T, W] fp32, in place: += rms(y + ybias) * w_post. Returns rms(resid) * w_pre in ``out_dtype`` (None
    without ``w_pre``). Norm weights are fp32 [W]; ``ybias`` has y's dtype."""
    if resid.is_cuda:
        h = torch.empty(resid.shape, dtype=out_dtype, device=resid.device) if w_pre is not None else None
        _kern().post_pre_norm(resid, y, ybias, w_post, w_pre, h, eps)
        return h
    yf = y.float() if ybias is None else y.float() + ybias.float()
    resid.add_(_rms(yf, eps) * w_post)
    return None if w_pre is None else (_rms(resid, eps) * w_pre).to(out_dtype)


def depth_avg_norm(planes: torch.Tensor, n: int, dw: Optional[torch.Tensor], y: Optional[torch.Tensor],
                   ybias: Optional[torch.Tensor], w_post: Optional[torch.Tensor], w_pre: Optional[torch.Tensor],
                   eps: float, out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """planes [>= n + 1, T, W] fp32 hold X_0 .. X_(n-1) (the embedding output and the layer results so far; plane
    n - 1 is the running residual of the layer that just ended). With ``y``: planes[n - 1] += rms(y + ybias) * w_post
    first (the layer's last post-norm). Then planes[n] = sum_(j < n) dw[j] planes[j] (``dw`` None: a copy of plane
    n - 1), the next layer's input and running residual, and the return value is rms(planes[n]) * w_pre in
    ``out_dtype`` (None without ``w_pre``)."""
    if planes.is_cuda:
        h = torch.empty(planes.shape[1:], dtype=out_dtype, device=planes.device) if w_pre is not None else None
        _kern().depth_avg_norm(planes, n, dw, y, ybias, w_post, w_pre, h, eps)
        return h
    if y is not None:
        yf = y.float() if ybias is None else y.float() + ybias.float()
        planes[n - 1].add_(_rms(yf, eps) * w_post)
    if dw is None:
        planes[n].copy_(planes[n - 1])
    else:
        planes[n].copy_(torch.einsum("j,jtw->tw", dw, planes[:n]))
    return None if w_pre is None else (_rms(planes[n], eps) * w_pre).to(out_dtype)


def bias_relu2(z: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """relu(z + b)^2, [rows, n] in z's dtype."""
    if z.is_cuda:
        z = z.contiguous()
        out = torch.empty_like(z)
        _kern().bias_relu2(out, z, b)
        return out
    x = torch.relu((z.float() + b.float()).to(z.dtype).float())
    return (x * x).to(z.dtype)


def tanh_cap(z: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(z / cap) as fp32, any shape."""
    if z.is_cuda:
        z = z.contiguous()
        out = torch.empty(z.shape, dtype=torch.float32, device=z.device)
        _kern().tanh_cap(out, z, float(cap))
        return out
    return torch.tanh(z.float() / cap) * cap


def head_gate(o: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """o [H, T, v] head-major, g [T, H] (any row stride) -> [T, H * v]: o[h, t] * sigmoid(g[t, h])."""
    H, T, v = o.shape
    if o.is_cuda:
        out = torch.empty(T, H * v, dtype=o.dtype, device=o.device)
        _kern().head_gate(out, o.contiguous(), g)
        return out
    return (o.float().transpose(0, 1) * torch.sigmoid(g.float())[:, :, None]).reshape(T, H * v).to(o.dtype)


def norm_sigmoid_gate(o: torch.Tensor, g: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """rms(o) * w * sigmoid(g): o [T, n] fp32, g [T, n] (any row stride), result in g's dtype."""
    if o.is_cuda:
        out = torch.empty(o.shape, dtype=g.dtype, device=o.device)
        _kern().norm_sigmoid_gate(out, o, g, w, eps)
        return out
    return (_rms(o, eps) * w * torch.sigmoid(g.float())).to(g.dtype)


def lightning_attn(x: torch.Tensor, qoff: int, koff: int, voff: int, decay: torch.Tensor, state: torch.Tensor,
                   heads: int, dim: int, vdim: int, rag: Ragged) -> torch.Tensor:
    """x [T, *]: the q | k (heads * dim each) and v (heads * vdim) projections at column offsets qoff / koff / voff;
    SiLU is applied here. Per (sequence, head), token by token: S <- decay[h] S + k v^T, o = S^T q; the state S
    [dim, vdim] fp32 lives in ``state`` [slots, H, dim, vdim] and a sequence whose step starts at position 0 starts
    from zero. Returns o [T, H * vdim] fp32."""
    T = x.shape[0]
    out = torch.empty(T, heads * vdim, dtype=torch.float32, device=x.device)
    if x.is_cuda:
        _kern().lightning_attn(out, x, qoff, koff, voff, decay, state, heads, dim, vdim, rag.positions, rag.cu_q,
                               rag.state_slots)
        return out
    q = F.silu(x[:, qoff: qoff + heads * dim]).float().view(T, heads, dim)
    k = F.silu(x[:, koff: koff + heads * dim]).float().view(T, heads, dim)
    v = F.silu(x[:, voff: voff + heads * vdim]).float().view(T, heads, vdim)
    o = out.view(T, heads, vdim)
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(T):
        S = state[slot].clone() if pos[q0] > 0 else torch.zeros_like(state[slot])
        for t in range(q0, q0 + n):
            S = S * decay[:, None, None] + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S
    return out
