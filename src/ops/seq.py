"""
Ops for models that carry per-sequence state besides the paged KV cache, on the ``src/_Cmix`` HIP extension
(``csrc/kernels/seq_mix.hip``, ``csrc/kernels/sink_attn.hip``):

* :func:`embed_hash`, :func:`store_last_token` — token embedding plus a hashed bigram embedding; the previous
  token of a sequence is state;
* :func:`stream_mix_norm` — several fp32 residual streams with learned mixing (hyper-connections): the update of
  the streams by a sublayer's output and the next sublayer's normed input in one launch;
* :func:`poly_norm_act` — a polynomial of RMS-normalised powers as feed-forward activation;
* :func:`delta_prep`, :func:`conv_state_update`, :func:`gated_delta` — short causal convolutions and the gated
  delta rule with its fp32 matrix state per head;
* :func:`qkv_prep`, :func:`sink_attn` — grouped-query attention over a paged cache with a softmax sink, an
  optional sliding window, rotate-half rotary positions, whole-projection q/k norms, value norms or cross-layer
  value mixing, and a learned bias per (distance, head).

A step is a ragged batch (:class:`Ragged`): sequence s owns rows ``cu_q[s] .. cu_q[s + 1] - 1`` (``cu_q`` None: one
row per sequence). A sequence whose first row of the step is at position 0 starts from zero state.

GPU tensors always run the HIP kernels (a missing extension raises); CPU tensors run the plain-PyTorch semantics
below, which lets the engine's control flow run in CPU-only tests.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

from .mix import _kern


@dataclass
class Ragged:
    positions: torch.Tensor            # [T] int64
    cu_q: Optional[torch.Tensor]       # [S + 1] int32 or None (one row per sequence)
    state_slots: torch.Tensor          # [S] int32

    def spans(self, rows: int) -> List[Tuple[int, int, int]]:
        """(first row, rows, slot) per sequence — host-side, CPU path only."""
        slots = self.state_slots.tolist()
        if self.cu_q is None:
            return [(i, 1, slots[i]) for i in range(rows)]
        cu = self.cu_q.tolist()
        return [(cu[s], cu[s + 1] - cu[s], slots[s]) for s in range(len(cu) - 1) if cu[s + 1] > cu[s]]


def distance_bias_table(rel: torch.Tensor, bias_max: float, window: int = 0) -> torch.Tensor:
    """fp32 [rows, H]: the bias of a key at distance n is row min(n, rows - 1). ``rel`` [B, H] holds one row per
    bucket: distances below B // 2 have a bucket each, larger ones share buckets that grow logarithmically up to
    ``bias_max`` (the last bucket takes everything beyond). Bucket numbers are computed once, in float64."""
    B = rel.shape[0]
    half = B // 2
    top = int(math.ceil(bias_max)) + 1
    if window:
        top = min(top, window)
    top = max(top, half + 1, 1)
    idx = []
    for n in range(top + 1):
        if n < half or half == 0:
            idx.append(min(n, B - 1))
        elif bias_max <= half:   # no room for shared buckets: everything from B // 2 on takes the last one
            idx.append(B - 1)
        else:
            idx.append(min(B - 1, half + int(math.floor(math.log(n / half) / math.log(bias_max / half) * (B - half)))))
    return rel.float()[torch.tensor(idx, device=rel.device)].contiguous()


# -------------------------------------------------------------------------------------------------- embedding
def embed_hash(ids: torch.Tensor, embed: torch.Tensor, bigram: Optional[torch.Tensor], rag: Ragged,
               prev_tok: torch.Tensor, scale: float, buckets: int, mul_prev: int, mul_cur: int,
               streams: int) -> torch.Tensor:
    """fp32 [T, streams, W]: embed[id] * scale + bigram[(prev * mul_prev + id * mul_cur) mod buckets] (row
    ``buckets`` at position 0), copied into every stream. On the GPU a step with one row per sequence also stores
    the row's token as the new previous token (:func:`store_last_token` then has nothing left to do)."""
    T, W = ids.shape[0], embed.shape[1]
    out = torch.empty(T, streams, W, dtype=torch.float32, device=ids.device)
    if ids.is_cuda:
        _kern().embed_hash(out, embed, bigram, ids, rag.positions, rag.cu_q, rag.state_slots, prev_tok, scale, buckets,
                           mul_prev, mul_cur)
        return out
    x = embed[ids].float() * scale
    if bigram is not None:
        idl, pos = ids.tolist(), rag.positions.tolist()
        rows = []
        for q0, n, slot in rag.spans(T):
            for i in range(q0, q0 + n):
                if pos[i] <= 0:
                    rows.append(buckets)
                else:
                    prev = idl[i - 1] if i > q0 else int(prev_tok[slot])
                    rows.append((prev * mul_prev + idl[i] * mul_cur) % buckets)
        x = x + bigram[torch.tensor(rows)].float()
    out.copy_(x.unsqueeze(1).expand(T, streams, W))
    return out


def store_last_token(prev_tok: torch.Tensor, ids: torch.Tensor, rag: Ragged) -> None:
    if ids.is_cuda:
        if rag.cu_q is not None:   # one row per sequence: embed_hash stored it
            _kern().store_last_token(prev_tok, ids, rag.positions, rag.cu_q, rag.state_slots)
        return
    for q0, n, slot in rag.spans(ids.shape[0]):
        prev_tok[slot] = ids[q0 + n - 1]


# ---------------------------------------------------------------------------------------------- residual streams
def stream_mix_norm(streams: torch.Tensor, y1: Optional[torch.Tensor], y2: Optional[torch.Tensor], a1: float,
                    a2: float, mix: Optional[torch.Tensor], outw: Optional[torch.Tensor],
                    inw: Optional[torch.Tensor], gain: Optional[torch.Tensor], eps: float,
                    out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """streams [T, S, W] fp32, in place: x_t <- sum_s mix[s, t] x_s + outw[t] * (a1 y1 + a2 y2) (skipped without
    y1); returns h = rmsnorm(sum_t inw[t] x_t) * gain in ``out_dtype`` (None: no h). ``inw`` None: the plain sum;
    ``mix`` / ``outw`` None: identity / ones (one stream: the ordinary residual sum)."""
    T, S, W = streams.shape
    if streams.is_cuda:
        h = torch.empty(T, W, dtype=out_dtype, device=streams.device) if out_dtype is not None else None
        _kern().stream_mix_norm(streams, y1, y2, a1, a2, mix, outw, inw, gain, eps, h)
        return h
    if y1 is not None:
        y = a1 * y1.float()
        if y2 is not None:
            y = y + a2 * y2.float()
        m = mix if mix is not None else torch.eye(S)
        o = outw if outw is not None else torch.ones(S)
        streams.copy_(torch.einsum("sq,tsw->tqw", m, streams) + o[None, :, None] * y[:, None, :])
    if out_dtype is None:
        return None
    u = streams.sum(1) if inw is None else torch.einsum("s,tsw->tw", inw, streams)
    return (u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * gain).to(out_dtype)


def poly_norm_act(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3] per row, N(v) = v / sqrt(mean(v^2) + eps)."""
    if z.is_cuda:
        out = torch.empty(z.shape, dtype=z.dtype, device=z.device)
        _kern().poly_norm_act(out, z, coef, eps)
        return out
    x = z.float()

    def n(v):
        return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)

    return (coef[0] * n(x) + coef[1] * n(x * x) + coef[2] * n(x * x * x) + coef[3]).to(z.dtype)


# ---------------------------------------------------------------------------------------------- gated delta rule
def delta_prep(x: torch.Tensor, b: torch.Tensor, a: torch.Tensor, conv_w: torch.Tensor, conv_state: torch.Tensor,
               A_log: torch.Tensor, dt_bias: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int,
               rag: Ragged, conv_wt: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [T, C = 2 G dim + H vdim] = [q | k | v] channels: causal convolution over the sequence's last ``taps``
    inputs (those before the step from conv_state [slots, taps - 1, C]) + SiLU; q and k heads to unit length
    (q also times dim^-1/2). Returns (qkv32 [T, C] fp32, bg [T, 2 H] fp32 = [sigmoid(b) | exp(-exp(A_log) *
    softplus(a + dt_bias))]). On the GPU a step with one row per sequence also moves the row's input into
    conv_state (:func:`conv_state_update` then has nothing left to do). ``conv_wt``: the same weights tap-major,
    [taps, C] contiguous, which lets the kernel load them 16 bytes at a time in prompt-sized bf16 steps."""
    T, C = x.shape
    taps = conv_w.shape[1]
    qkv32 = torch.empty(T, C, dtype=torch.float32, device=x.device)
    bg = torch.empty(T, 2 * heads, dtype=torch.float32, device=x.device)
    if x.is_cuda:
        _kern().delta_prep(qkv32, bg, x, b, a, conv_w, conv_wt, conv_state, A_log, dt_bias, heads, kv_heads, dim, vdim,
                           rag.positions, rag.cu_q, rag.state_slots)
        return qkv32, bg
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(T):
        hist = conv_state[slot].clone() if pos[q0] > 0 else torch.zeros(taps - 1, C)
        if 0 < pos[q0] < taps - 1:
            hist[: taps - 1 - pos[q0]] = 0
        seq = torch.cat([hist, x[q0:q0 + n].float()], 0)            # [taps - 1 + n, C]
        win = seq.unfold(0, taps, 1)                                # [n, C, taps]
        y = (win * conv_w[None]).sum(-1).to(x.dtype)
        qkv32[q0:q0 + n] = F.silu(y).float()
    G = kv_heads
    qk = qkv32[:, : 2 * G * dim].view(T, 2 * G, dim)
    qk = qk / torch.sqrt((qk * qk).sum(-1, keepdim=True) + 1e-6)
    qk[:, :G] *= dim ** -0.5
    qkv32[:, : 2 * G * dim] = qk.reshape(T, 2 * G * dim)
    bg[:, :heads] = torch.sigmoid(b.float())
    bg[:, heads:] = torch.exp(-torch.exp(A_log) * F.softplus(a.float() + dt_bias))
    return qkv32, bg


def conv_state_update(conv_state: torch.Tensor, x: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int,
                      rag: Ragged) -> None:
    """conv_state[slot] <- the sequence's last taps - 1 inputs after this step."""
    if conv_state.shape[1] == 0:
        return
    if x.is_cuda:
        if rag.cu_q is not None:   # one row per sequence: delta_prep moved it
            _kern().conv_state_update(conv_state, x, heads, kv_heads, dim, vdim, rag.positions, rag.cu_q,
                                      rag.state_slots)
        return
    k = conv_state.shape[1]
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(x.shape[0]):
        old = conv_state[slot] if pos[q0] > 0 else torch.zeros_like(conv_state[slot])
        conv_state[slot] = torch.cat([old, x[q0:q0 + n].float()], 0)[-k:]


def gated_delta(qkv32: torch.Tensor, bg: torch.Tensor, gate: torch.Tensor, norm_w: torch.Tensor, eps: float,
                state: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, rag: Ragged) -> torch.Tensor:
    """Per (sequence, head), token by token: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q; the state S
    [dim, vdim] fp32 lives in ``state`` [slots, H, dim, vdim]. Returns o / rms(o) * norm_w * silu(gate),
    [T, H * vdim] in gate's dtype."""
    T = qkv32.shape[0]
    out = torch.empty(T, heads * vdim, dtype=gate.dtype, device=gate.device)
    if gate.is_cuda:
        _kern().gated_delta(out, qkv32, bg, gate, norm_w, eps, state, heads, kv_heads, dim, vdim, rag.positions,
                            rag.cu_q, rag.state_slots)
        return out
    G, rep = kv_heads, heads // kv_heads
    q = qkv32[:, : G * dim].view(T, G, dim).repeat_interleave(rep, 1)
    k = qkv32[:, G * dim: 2 * G * dim].view(T, G, dim).repeat_interleave(rep, 1)
    v = qkv32[:, 2 * G * dim:].view(T, heads, vdim)
    o = torch.empty(T, heads, vdim)
    pos = rag.positions.tolist()
    for q0, n, slot in rag.spans(T):
        S = state[slot].clone() if pos[q0] > 0 else torch.zeros_like(state[slot])      # [H, dim, vdim]
        for t in range(q0, q0 + n):
            S = S * bg[t, heads:, None, None]
            u = bg[t, :heads, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
            S = S + k[t][:, :, None] * u[:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * norm_w * F.silu(gate.float().view(T, heads, vdim))
    return o.reshape(T, heads * vdim).to(gate.dtype)


# ---------------------------------------------------------------------------------------------------- attention
def _head_major(cache: torch.Tensor, kv_heads: int) -> "_HeadMajorView":
    return _HeadMajorView(cache, kv_heads)


class _HeadMajorView:
    """Slot-indexed reads and writes (CPU path) of a cache [blocks, block_size, G * (dim + vdim)] whose blocks are
    laid out head-major inside, [G][block_size][K | V], so that what one key/value head reads from a block is
    contiguous: item [slots] is [n, G, dim + vdim]."""

    def __init__(self, cache: torch.Tensor, kv_heads: int):
        nb, bs, w = cache.shape
        self.v = cache.view(nb, kv_heads, bs, w // kv_heads)
        self.bs = bs

    def __getitem__(self, slots: torch.Tensor) -> torch.Tensor:
        return self.v[slots // self.bs, :, slots % self.bs]

    def __setitem__(self, slots: torch.Tensor, rows: torch.Tensor) -> None:
        self.v[slots // self.bs, :, slots % self.bs] = rows


def qkv_prep(q: torch.Tensor, k: torch.Tensor, v: Optional[torch.Tensor], cache: torch.Tensor, heads: int,
             kv_heads: int, dim: int, vdim: int, positions: torch.Tensor, slots: torch.Tensor, eps: float,
             q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None, rot_dims: int = 0,
             inv_freq: Optional[torch.Tensor] = None, v_unit: bool = False, v_lambda: Optional[torch.Tensor] = None,
             v_first: Optional[torch.Tensor] = None, head_norm: bool = False, q_temp_coef: float = 0.0,
             q_temp_every: int = 1, norm_after_rot: bool = False) -> torch.Tensor:
    """The step between the q/k/v projection and the attention, one launch: optional RMS norm of q and of k (plain
    weights) over the whole projection or, with ``head_norm``, of every head by itself with weights [dim] shared by
    the heads; optional query temperature, q times 1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1) after its
    norm; optional rotate-half rotary on the first ``rot_dims`` dims of every head (pair i, i + rot_dims / 2, angle
    position * inv_freq[i]) — with ``norm_after_rot`` (and ``head_norm``) the rotation comes first and the per-head
    norm acts on the rotated heads; values either divided by their per-head root mean square or blended as
    (1 - l) v + l v_first; ``v`` None: the values are the keys as projected, before norm and rotation. Writes the
    token's keys and values into the cache at slots[t] (< 0: skipped; a block's interior is head-major,
    [G][block_size][k | v]) and returns q [T, H * dim]."""
    T = q.shape[0]
    if q.is_cuda:
        q_out = torch.empty(T, heads * dim, dtype=q.dtype, device=q.device)
        _kern().qkv_prep(q_out, cache, q, k, v, heads, kv_heads, dim, vdim, q_norm, k_norm, rot_dims, inv_freq, v_unit,
                         v_lambda, v_first, eps, positions, slots, head_norm, float(q_temp_coef), int(q_temp_every),
                         bool(norm_after_rot))
        return q_out
    if v is None:
        v = k
    qf, kf, vf = q.float(), k.float(), v.float()
    if v_lambda is not None:
        vf = (1.0 - v_lambda) * vf + v_lambda * v_first.float()

    def rot(x, n):
        half = rot_dims // 2
        ang = positions.float()[:, None] * inv_freq[None, :]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        x = x.view(T, n, dim).clone()
        u, w = x[..., :half].clone(), x[..., half:rot_dims].clone()
        x[..., :half] = u * c - w * s
        x[..., half:rot_dims] = w * c + u * s
        return x.reshape(T, n * dim)

    if rot_dims and norm_after_rot:
        qf, kf = rot(qf, heads), rot(kf, kv_heads)
    if q_norm is not None and head_norm:
        qh, kh = qf.view(T, heads, dim), kf.view(T, kv_heads, dim)
        qf = (qh / torch.sqrt((qh * qh).mean(-1, keepdim=True) + eps) * q_norm).reshape(T, heads * dim)
        kf = (kh / torch.sqrt((kh * kh).mean(-1, keepdim=True) + eps) * k_norm).reshape(T, kv_heads * dim)
    elif q_norm is not None:
        qf = qf / torch.sqrt((qf * qf).mean(-1, keepdim=True) + eps) * q_norm
        kf = kf / torch.sqrt((kf * kf).mean(-1, keepdim=True) + eps) * k_norm
    if q_temp_coef:
        steps = torch.div(positions + 1, q_temp_every, rounding_mode="floor").float()
        qf = qf * (1.0 + q_temp_coef * torch.log(steps + 1.0))[:, None]
    if rot_dims and not norm_after_rot:
        qf, kf = rot(qf, heads), rot(kf, kv_heads)
    if v_unit:
        vh = vf.view(T, kv_heads, vdim)
        vf = (vh / torch.sqrt((vh * vh).mean(-1, keepdim=True) + eps)).reshape(T, kv_heads * vdim)
    ok = slots >= 0
    _head_major(cache, kv_heads)[slots[ok]] = torch.cat(
        [kf.view(T, kv_heads, dim), vf.view(T, kv_heads, vdim)], 2)[ok].to(cache.dtype)
    return qf.to(q.dtype)


def sink_attn(q: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor, cu_q: Optional[torch.Tensor],
              ctx_lens: torch.Tensor, positions: torch.Tensor, sink: Optional[torch.Tensor],
              bias: Optional[torch.Tensor], max_q: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int,
              scale: float, impl: int = 0, softcap: float = 0.0, slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Grouped-query attention over the cache that :func:`qkv_prep` writes. The query at position p sees the cached
    positions j <= p with p - j < window (0: all). Score: s = (q . k_j) * scale; with ``softcap`` > 0,
    s <- softcap * tanh(s / softcap); then - slopes[h] * (p - j) (``slopes`` [H] fp32, a linear distance penalty)
    and + bias[min(p - j, rows - 1), h]. The softmax denominator has one more term exp(sink[h]) when ``sink`` is
    given. Returns [T, H * vdim]. ``impl``: 0 = the matrix-core kernel where it applies, 1 = the FMA kernel, 2 = the
    matrix-core kernel or an error."""
    T = q.shape[0]
    if q.is_cuda:
        out = torch.empty(T, heads * vdim, dtype=q.dtype, device=q.device)
        _kern().sink_attn(out, q, cache, block_tables, cu_q, ctx_lens, positions, sink, bias, max_q, heads, kv_heads,
                          dim, vdim, window, scale, impl, float(softcap), slopes)
        return out
    bs = cache.shape[1]
    hm = _head_major(cache, kv_heads)
    out = torch.zeros(T, heads, vdim)
    qh = q.float().view(T, heads, dim)
    S = block_tables.shape[0]
    cu = cu_q.tolist() if cu_q is not None else list(range(S + 1))
    pos = positions.tolist()
    rep = heads // kv_heads
    for s in range(S):
        if cu[s + 1] <= cu[s]:
            continue
        n_ctx = int(ctx_lens[s])
        j = torch.arange(n_ctx)
        rows = hm[block_tables[s].long()[j // bs] * bs + j % bs].float()      # [n_ctx, G, dim + vdim]
        kk = rows[:, :, :dim].repeat_interleave(rep, 1)
        vv = rows[:, :, dim:].repeat_interleave(rep, 1)
        for t in range(cu[s], cu[s + 1]):
            n = pos[t] - j
            ok = (n >= 0) & ((n < window) if window > 0 else torch.ones_like(n, dtype=torch.bool))
            sc = torch.einsum("hd,jhd->hj", qh[t], kk) * scale
            if softcap:
                sc = softcap * torch.tanh(sc / softcap)
            if slopes is not None:
                sc = sc - slopes[:, None] * n[None, :].float()
            if bias is not None:
                sc = sc + bias[n.clamp(0, bias.shape[0] - 1)].T
            sc = sc.masked_fill(~ok[None, :], -math.inf)
            if sink is not None:
                sc = torch.cat([sc, sink[:, None]], 1)
            p = torch.softmax(sc, -1)[:, :n_ctx]
            out[t] = torch.einsum("hj,jhv->hv", p, vv)
    return out.reshape(T, heads * vdim).to(q.dtype)
