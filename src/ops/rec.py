"""
Ops for recurrent mixers whose state is a vector or matrix per channel or head, on the ``src/_Cmix`` HIP extension
(``csrc/kernels/rec_mix.hip``):

* :func:`embed_scaled` — token vectors times a constant, into the fp32 residual (and its activation copy);
* :func:`conv_silu`, :func:`conv_tail_update` — a short causal convolution per channel with bias and SiLU, the
  inputs before the step taken from the sequence's state slot; optionally also the per-head step size and decay
  ``(exp(-exp(A_log) * dt), dt)``, ``dt = softplus(raw + bias)``, of a scalar-decay state-space layer;
* :func:`selective_scan` — a diagonal state per channel with input-dependent step size, input map and output map
  (S <- exp(dt A) S + dt x B; y = S . C + D x), gated by SiLU(z);
* :func:`exp_gate_scan` — exponential input gate and sigmoid forget gate in log space with a running maximum:
  the per-token decay, input weight and normaliser floor of a matrix-memory LSTM;
* :func:`gated_linear_attn` — the matrix recurrence S <- a_t S + b_t k_t v_t^T, o_t = S^T q_t with one (a_t, b_t) per
  token and head, grouped q / k, and an optional normaliser vector n <- a_t n + b_t k_t read out as n . q;
* :func:`head_norm_gate` — the read-out divided by max(|n . q|, floor) + 1e-6, every head RMS-normed, weight,
  sigmoid gate;
* :func:`skip_gate_group_norm` — (o + D_h x) * SiLU(z), RMS norm in equal parts of the row, weight;
* :func:`pair_post_norm_residual` — two sublayer outputs, each RMS-normed over the row with its own weight,
  averaged, then the layer's norm on the result, times a constant, added into the fp32 residual: one launch.

A step is a ragged batch (:class:`src.ops.seq.Ragged`); a sequence whose first row of the step is at position 0
starts from zero state whatever its slot holds. GPU tensors always run the HIP kernels (a missing extension
raises); CPU tensors run the plain-PyTorch semantics below, which lets the engine's control flow run in CPU-only
tests.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from .mix import _kern
from .seq import Ragged


def _rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def embed_scaled(ids: torch.Tensor, embed: torch.Tensor, scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """(resid fp32 [T, W] = embed[ids] * scale, act = resid in embed's dtype; the same tensor for an fp32 table)."""
    T, W = ids.shape[0], embed.shape[1]
    resid = torch.empty(T, W, dtype=torch.float32, device=ids.device)
    act = resid if embed.dtype == torch.float32 else torch.empty(T, W, dtype=embed.dtype, device=ids.device)
    if ids.is_cuda:
        _kern().embed_scaled(resid, None if act is resid else act, embed, ids, float(scale))
        return resid, act
    resid.copy_(embed[ids].float() * scale)
    if act is not resid:
        act.copy_(resid)
    return resid, act


# ------------------------------------------------------------------------------------------------ convolution
def conv_silu(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], conv_state: torch.Tensor, rag: Ragged,
              wt: Optional[torch.Tensor] = None, dt: Optional[torch.Tensor] = None,
              dt_bias: Optional[torch.Tensor] = None, A_log: Optional[torch.Tensor] = None):
    """x [T, C] (any row stride): y[t, c] = silu(bias[c] + sum_j w[c, j] * x[t - (taps - 1 - j), c]) in x's dtype; rows
    before the step come from conv_state [slots, taps - 1, C] (fp32, the most recent last), rows before the
    sequence's start are zero. ``wt``: the same weights tap-major ([taps, C]) for 16-byte loads. With ``dt`` [T, H] (a
    slice of the same projection as x) also returns ab [T, H, 2] fp32 = (exp(-exp(A_log) * d), d) with
    d = softplus(dt + dt_bias). On the GPU a step with one row per sequence also moves the row's input into conv_state
    (:func:`conv_tail_update` then has nothing left to do)."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.empty(T, C, dtype=x.dtype, device=x.device)
    ab = None
    if dt is not None:
        ab = torch.empty(T, dt.shape[1], 2, dtype=torch.float32, device=x.device)
    if x.is_cuda:
        _kern().conv_silu(y, x, w, wt, bias, conv_state, dt, dt_bias, A_log, ab, rag.positions, rag.cu_q,
                          rag.state_slots)
        return (y, ab) if dt is not None else y
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(T):
        hist = conv_state[slot].clone() if pos[q0] > 0 else torch.zeros(taps - 1, C)
        if 0 < pos[q0] < taps - 1:
            hist[: taps - 1 - pos[q0]] = 0
        s = torch.cat([hist, x[q0:q0 + n].float()], 0)                 # [taps - 1 + n, C]
        acc = (s.unfold(0, taps, 1) * w[None]).sum(-1)
        if bias is not None:
            acc = acc + bias
        y[q0:q0 + n] = F.silu(acc.to(x.dtype).float()).to(x.dtype)
    if dt is not None:
        d = F.softplus(dt.float() + dt_bias, threshold=20.0)
        ab[..., 0] = torch.exp(-torch.exp(A_log) * d)
        ab[..., 1] = d
        return y, ab
    return y


def conv_tail_update(conv_state: torch.Tensor, x: torch.Tensor, rag: Ragged) -> None:
    """conv_state[slot] <- the sequence's last taps - 1 inputs after this step."""
    k = conv_state.shape[1]
    if k == 0:
        return
    if x.is_cuda:
        if rag.cu_q is not None:   # one row per sequence: conv_silu moved it
            _kern().conv_tail_update(conv_state, x, rag.positions, rag.cu_q, rag.state_slots)
        return
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(x.shape[0]):
        old = conv_state[slot] if pos[q0] > 0 else torch.zeros_like(conv_state[slot])
        conv_state[slot] = torch.cat([old, x[q0:q0 + n].float()], 0)[-k:]


# --------------------------------------------------------------------------------------------- selective scan
def selective_scan(x: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, bc: torch.Tensor, boff: int, coff: int,
                   A: torch.Tensor, D: torch.Tensor, z: torch.Tensor, state: torch.Tensor, rag: Ragged) -> torch.Tensor:
    """Per (sequence, channel c), token by token, with d = softplus(dt[t, c] + dt_bias[c]):
    S[c, :] <- exp(d * A[c, :]) * S[c, :] + d * x[t, c] * B_t;  y = S[c, :] . C_t + D[c] * x[t, c];  out = y * silu(z).
    x, dt, z [T, I] (any row stride); B_t, C_t = bc[t, boff: boff + N], bc[t, coff: coff + N]; A [I, N] fp32 (negative);
    state [slots, I, N] fp32. Returns [T, I] in x's dtype."""
    T, I = x.shape
    N = A.shape[1]
    out = torch.empty(T, I, dtype=x.dtype, device=x.device)
    if x.is_cuda:
        _kern().selective_scan(out, x, dt, dt_bias, bc, boff, coff, A, D, z, state, rag.positions, rag.cu_q,
                               rag.state_slots)
        return out
    d = F.softplus(dt.float() + dt_bias, threshold=20.0)
    xf, zf = x.float(), z.float()
    B, C = bc[:, boff: boff + N].float(), bc[:, coff: coff + N].float()
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(T):
        S = state[slot].clone() if pos[q0] > 0 else torch.zeros_like(state[slot])
        for t in range(q0, q0 + n):
            S = torch.exp(d[t][:, None] * A) * S + (d[t] * xf[t])[:, None] * B[t][None, :]
            out[t] = ((S @ C[t] + D * xf[t]) * F.silu(zf[t])).to(x.dtype)
        state[slot] = S
    return out


# ------------------------------------------------------------------------------------------ matrix recurrences
def exp_gate_scan(x: torch.Tensor, ioff: int, foff: int, i_bias: torch.Tensor, f_bias: torch.Tensor, cap: float,
                  m_state: torch.Tensor, heads: int, rag: Ragged) -> torch.Tensor:
    """x [T, *]: raw gate pre-activations of H heads at column offsets ioff / foff. Per token and head, in fp32:
    i = cap * tanh((x_i + i_bias) / cap), f = logsigmoid(cap * tanh((x_f + f_bias) / cap)); with the running maximum
    m (per sequence and head, in m_state [slots, H], 0 at a sequence's start) m_t = max(f + m_(t-1), i). Returns
    abe [T, H, 3] fp32 = (exp(f + m_(t-1) - m_t), exp(i - m_t), exp(-m_t))."""
    T = x.shape[0]
    abe = torch.empty(T, heads, 3, dtype=torch.float32, device=x.device)
    if x.is_cuda:
        _kern().exp_gate_scan(abe, x, ioff, foff, i_bias, f_bias, float(cap), m_state, heads, rag.positions, rag.cu_q,
                              rag.state_slots)
        return abe
    ig = cap * torch.tanh((x[:, ioff: ioff + heads].float() + i_bias) / cap)
    fg = F.logsigmoid(cap * torch.tanh((x[:, foff: foff + heads].float() + f_bias) / cap))
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(T):
        m = m_state[slot].clone() if pos[q0] > 0 else torch.zeros_like(m_state[slot])
        for t in range(q0, q0 + n):
            m_new = torch.maximum(fg[t] + m, ig[t])
            abe[t, :, 0] = torch.exp(fg[t] + m - m_new)
            abe[t, :, 1] = torch.exp(ig[t] - m_new)
            abe[t, :, 2] = torch.exp(-m_new)
            m = m_new
        m_state[slot] = m
    return abe


def gated_linear_attn(x: torch.Tensor, qoff: int, koff: int, voff: int, ab: torch.Tensor, state: torch.Tensor,
                      n_state: Optional[torch.Tensor], heads: int, groups: int, dim: int, vdim: int, qscale: float,
                      rag: Ragged) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """x [T, *]: q | k (groups * dim each; head h reads group h // (heads / groups)) and v (heads * vdim) at column
    offsets qoff / koff / voff. Per (sequence, head), token by token, with (a, b) = ab[t, h, :2]:
    S <- a S + b k v^T;  o = S^T (q * qscale), S [dim, vdim] fp32 in ``state`` [slots, H, dim, vdim]. With ``n_state``
    [slots, H, dim] also n <- a n + b k and nq = n . (q * qscale). Returns (o [T, H * vdim] fp32, nq [T, H] fp32 or
    None)."""
    T = x.shape[0]
    o = torch.empty(T, heads * vdim, dtype=torch.float32, device=x.device)
    nq = torch.empty(T, heads, dtype=torch.float32, device=x.device) if n_state is not None else None
    if x.is_cuda:
        _kern().gated_linear_attn(o, nq, x, qoff, koff, voff, ab, state, n_state, heads, groups, dim, vdim,
                                  float(qscale), rag.positions, rag.cu_q, rag.state_slots)
        return o, nq
    rep = heads // groups
    q = x[:, qoff: qoff + groups * dim].float().view(T, groups, dim).repeat_interleave(rep, 1) * qscale
    k = x[:, koff: koff + groups * dim].float().view(T, groups, dim).repeat_interleave(rep, 1)
    v = x[:, voff: voff + heads * vdim].float().view(T, heads, vdim)
    ov = o.view(T, heads, vdim)
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(T):
        fresh = pos[q0] <= 0
        S = torch.zeros_like(state[slot]) if fresh else state[slot].clone()
        nv = None
        if n_state is not None:
            nv = torch.zeros_like(n_state[slot]) if fresh else n_state[slot].clone()
        for t in range(q0, q0 + n):
            a, b = ab[t, :, 0], ab[t, :, 1]
            S = a[:, None, None] * S + (b[:, None] * k[t])[:, :, None] * v[t][:, None, :]
            ov[t] = torch.einsum("hdv,hd->hv", S, q[t])
            if nv is not None:
                nv = a[:, None] * nv + b[:, None] * k[t]
                nq[t] = (nv * q[t]).sum(-1)
        state[slot] = S
        if nv is not None:
            n_state[slot] = nv
    return o, nq


def head_norm_gate(o: torch.Tensor, nq: torch.Tensor, abe: torch.Tensor, g: torch.Tensor, w: torch.Tensor, heads: int,
                   vdim: int, eps: float) -> torch.Tensor:
    """o [T, H * vdim] fp32, nq [T, H], abe [T, H, 3] (its last entry the floor), g [T, H * vdim] (any row stride):
    u = o_h / (max(|nq_h|, floor_h) + 1e-6); out = rms(u) over each head * w * sigmoid(g), in g's dtype."""
    T = o.shape[0]
    out = torch.empty(T, heads * vdim, dtype=g.dtype, device=o.device)
    if o.is_cuda:
        _kern().head_norm_gate(out, o, nq, abe, g, w, heads, vdim, float(eps))
        return out
    den = torch.maximum(nq.abs(), abe[..., 2]) + 1e-6
    u = _rms(o.view(T, heads, vdim) / den[..., None], eps).reshape(T, heads * vdim)
    return (u * w * torch.sigmoid(g.float())).to(g.dtype)


def skip_gate_group_norm(o: torch.Tensor, x: torch.Tensor, D: torch.Tensor, z: torch.Tensor, w: torch.Tensor,
                         heads: int, vdim: int, parts: int, eps: float) -> torch.Tensor:
    """o [T, H * vdim] fp32; x, z [T, H * vdim] (any row stride): y = (o + D[h] * x) * silu(z); the row is RMS-normed
    in ``parts`` equal parts, times w; in z's dtype."""
    T, n = o.shape
    out = torch.empty(T, n, dtype=z.dtype, device=o.device)
    if o.is_cuda:
        _kern().skip_gate_group_norm(out, o, x, D, z, w, heads, vdim, parts, float(eps))
        return out
    y = (o + D.repeat_interleave(vdim)[None, :] * x.float()) * F.silu(z.float())
    return (_rms(y.view(T, parts, n // parts), eps).reshape(T, n) * w).to(z.dtype)


# ------------------------------------------------------------------------------------------------ residual
def pair_post_norm_residual(resid: torch.Tensor, act: Optional[torch.Tensor], y1: torch.Tensor, w1: torch.Tensor,
                            y2: torch.Tensor, w2: torch.Tensor, w: torch.Tensor, mult: float, eps: float) -> None:
    """resid (fp32 [T, W], in place) += mult * rms(u) * (1 + w) with u = (rms(y1) * w1 + rms(y2) * w2) / 2; w1, w2
    fp32 [W]; ``act`` (optional, the activation dtype) receives the new residual."""
    if resid.is_cuda:
        _kern().pair_post_norm_residual(resid, act, y1, w1, y2, w2, w, float(mult), float(eps))
        return
    u = 0.5 * (_rms(y1.float(), eps) * w1 + _rms(y2.float(), eps) * w2)
    resid.add_(mult * _rms(u, eps) * (1.0 + w.float()))
    if act is not None:
        act.copy_(resid)
