"""
Dtype-generic ops (bf16 or fp32 storage, fp32 arithmetic) on the ``src/_Cmix`` HIP extension:

* :func:`rms_norm_ext`, :func:`post_norm_residual` — RMS norms with a plain weight or a `1 + w` gain,
  the second one applied to a sublayer's OUTPUT and added into an fp32 residual stream;
* :func:`gated_act` — SiLU-gated, clamped sigmoid-gated and GELU-gated feed-forward activations;
* :func:`route_sigmoid_topk`, :func:`moe_input_scaled` — sigmoid-scored top-k routing whose weight scales
  the expert's input, with an optional always-on shared expert;
* :func:`route_softmax_topk`, :func:`moe_output_weighted` — softmax-scored top-k routing with a correction that
  enters the choice only, identity experts, renormalised weights on the experts' outputs and a gated shared expert;
* :func:`latent_kv_write`, :func:`latent_attn` — latent (compressed-KV) attention over a paged cache of
  [latent | rotated shared key] rows, with a sliding window and a per-head softmax sink.

GPU tensors always run the HIP kernels (a missing extension raises); CPU tensors run the plain-PyTorch
semantics in :mod:`src.ops.reference`, which lets the engine's control flow run in CPU-only tests.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import reference as ref

_Cmix = None
_CMIX_ERR: Optional[BaseException] = None
try:
    from src import _Cmix  # type: ignore  # noqa: F811
except Exception as e:  # pragma: no cover - depends on build state
    _CMIX_ERR = e


def _load():
    """Import the extension if it was not there when this module was first imported (built since, in place)."""
    global _Cmix, _CMIX_ERR
    if _Cmix is None:
        try:
            import importlib

            _Cmix = importlib.import_module("src._Cmix")
        except Exception as e:  # noqa: BLE001
            _CMIX_ERR = e
    return _Cmix


def mix_available() -> bool:
    return _load() is not None


def _kern():
    if _load() is None:
        raise RuntimeError(
            "HIP kernel extension src/_Cmix is not built or failed to load "
            f"({_CMIX_ERR!r}); run `python -m src._build --mix-only` (hipcc --offload-arch=gfx950)")
    return _Cmix


def rms_norm_ext(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, unit_offset: bool = False,
                 out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * g over the last dim of [rows, n] (any row stride); g = w, or 1 + w with
    ``unit_offset`` (the stored weight is an offset from one), or 1 without a weight."""
    out_dtype = out_dtype or x.dtype
    if not x.is_cuda:
        return ref.rms_norm_ext(x, w, eps, unit_offset, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    _kern().rms_norm_ext(out, x, w, unit_offset, eps)
    return out


def post_norm_residual(resid: torch.Tensor, y: torch.Tensor, w: torch.Tensor, eps: float, unit_offset: bool = True,
                       act: Optional[torch.Tensor] = None, mult: float = 1.0) -> torch.Tensor:
    """resid (fp32 [rows, n], in place) += mult * rmsnorm(y) * g — the norm sits on the sublayer's output, the
    residual sum is fp32. ``act`` (bf16, same shape): also receives the new residual, the next projection's input."""
    if not resid.is_cuda:
        resid.add_(ref.rms_norm_ext(y, w, eps, unit_offset, torch.float32), alpha=mult)
        if act is not None:
            act.copy_(resid)
        return resid
    _kern().post_norm_residual(resid, act, y, w, unit_offset, eps, float(mult))
    return resid


ACT_SILU, ACT_CLAMPED, ACT_GELU_TANH = 0, 1, 2


def gated_act(gu: torch.Tensor, kind: int = ACT_SILU, limit: float = 0.0, alpha: float = 1.0) -> torch.Tensor:
    """[rows, 2f] = [gate | up] -> [rows, f]. ACT_SILU: silu(g) * u. ACT_CLAMPED: g' = min(g, limit),
    u' = clamp(u, -limit, limit), g' * sigmoid(alpha * g') * (u' + 1). ACT_GELU_TANH: gelu(g) * u with the tanh
    form 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3)))."""
    if not gu.is_cuda:
        return ref.gated_act(gu, kind, limit, alpha)
    gu = gu.contiguous()
    out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
    _kern().gated_act(out, gu, kind, limit, alpha)
    return out


ROUTE_FUSED_MAX_T = 256  # up to here one fused launch computes the logits and selects (decode-sized steps)


def route_sigmoid_topk(x: torch.Tensor, router: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(w [T, k] fp32, ids [T, k] int32): the k experts with the largest sigmoid(x . router[e]) (fp32 logits) and
    those scores, not renormalised."""
    if not x.is_cuda:
        return ref.route_sigmoid_topk(x, router, k)
    t = x.shape[0]
    w = torch.empty(t, k, dtype=torch.float32, device=x.device)
    ids = torch.empty(t, k, dtype=torch.int32, device=x.device)
    if t > ROUTE_FUSED_MAX_T:
        # prompt-sized steps: the logits as one true-fp32 library GEMM, then the selection kernel
        _kern().topk_sigmoid(w, ids, F.linear(x.float(), router.float()))
    else:
        _kern().route_sigmoid_topk(w, ids, x, router.contiguous())
    return w, ids


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y = x @ w^T. bf16 steps of up to 128 rows go through :func:`src.ops.linear` (the weight-streaming decode
    GEMM where the shape tiles it) when the Llama-path extension is loaded; everything else is the library GEMM
    (fp32 inputs: true fp32)."""
    if x.is_cuda and x.dtype == torch.bfloat16 and 0 < x.shape[0] <= 128 and x.is_contiguous():
        from src import ops

        if ops.native_available():
            return ops.linear(x, w)
    return F.linear(x, w)


# (token, expert) rows up to which the experts' weights are gathered per row for two batched GEMMs (no host
# read, hipGraph-capturable: decode steps); above it each expert runs one library GEMM pair over its rows
MOE_BMM_MAX_ROWS = 64


def moe_input_scaled(x: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, w: torch.Tensor, ids: torch.Tensor,
                     extra: Optional[torch.Tensor] = None, post_norm=None) -> Optional[torch.Tensor]:
    """out[t] (fp32) = sum_j expert_{ids[t, j]}(w[t, j] * x[t]) (+ extra[t]); expert(z) = W2 (silu(W1 z) * (W3 z))
    with w13 [E, 2f, H] = [W1; W3] and w2 [E, H, f]. The routing weight multiplies the expert's INPUT.
    ``post_norm`` = (resid fp32 [T, H], norm weight, eps, unit_offset, act or None): instead of returning the sum,
    add its RMS-normalised form into ``resid`` (and refresh ``act``) in the same launch that forms it —
    :func:`post_norm_residual` fused with the expert sum; returns None."""
    if not x.is_cuda:
        out = ref.moe_input_scaled(x, w13, w2, w, ids, extra)
        if post_norm is None:
            return out
        resid, nw, eps, unit, act = post_norm
        post_norm_residual(resid, out, nw, eps, unit, act=act)
        return None
    kern = _kern()
    t, h = x.shape
    k = ids.shape[1]
    n = t * k
    e = w13.shape[0]
    x = x.contiguous()
    w = w.contiguous()
    xs = torch.empty(n, h, dtype=x.dtype, device=x.device)

    def finish(ys, pos):
        if post_norm is not None:
            resid, nw, eps, unit, act = post_norm
            kern.combine_post_norm(resid, act, ys, pos, extra, k, nw, unit, eps)
            return None
        out = torch.empty(t, h, dtype=torch.float32, device=x.device)
        kern.combine_sum(out, ys, pos, extra, k)
        return out

    if x.dtype == torch.bfloat16 and t <= 128:
        # decode-sized steps: the framework's expert-streaming grouped GEMM (every routed expert's weights
        # streamed once, SiLU * up fused; no host read, hipGraph-capturable) on the scaled, expert-sorted rows
        from src import ops

        tiles = ops._moe_decode_tiles(h, w13.shape[1] // 2, t) if ops.native_available() else None
        if tiles is not None:
            ck = ops._kern()
            (wr1, kc1), (wr2, kc2) = tiles
            offsets = torch.empty(e + 1, dtype=torch.int32, device=x.device)
            sorted_idx = torch.empty(n, dtype=torch.int32, device=x.device)
            pos = torch.empty(n, dtype=torch.int32, device=x.device)
            kern.moe_align(offsets, sorted_idx, pos, ids.reshape(-1).contiguous(), e)
            kern.gather_scaled(xs, x, sorted_idx, w, k)
            a = torch.empty(n, w13.shape[1] // 2, dtype=x.dtype, device=x.device)
            ys = torch.empty(n, h, dtype=x.dtype, device=x.device)
            none = ops._NO_ROWS(x.device)
            ck.gemm_decode_grouped(a, xs, w13, offsets, 1, wr1, kc1, none, 1, t, 1)
            ck.gemm_decode_grouped(ys, a, w2, offsets, 0, wr2, kc2, none, 1, t, 1)
            return finish(ys, pos)
    if n <= MOE_BMM_MAX_ROWS or torch.cuda.is_current_stream_capturing():
        kern.gather_scaled(xs, x, None, w, k)
        sel = ids.reshape(-1).long()
        g = torch.bmm(w13.index_select(0, sel), xs.unsqueeze(2)).squeeze(2)
        ys = torch.bmm(w2.index_select(0, sel), gated_act(g, ACT_SILU).unsqueeze(2)).squeeze(2).contiguous()
        return finish(ys, None)
    offsets = torch.empty(e + 1, dtype=torch.int32, device=x.device)
    sorted_idx = torch.empty(n, dtype=torch.int32, device=x.device)
    pos = torch.empty(n, dtype=torch.int32, device=x.device)
    kern.moe_align(offsets, sorted_idx, pos, ids.reshape(-1).contiguous(), e)
    kern.gather_scaled(xs, x, sorted_idx, w, k)
    ys = torch.empty(n, h, dtype=x.dtype, device=x.device)
    off = offsets.tolist()  # one host read per layer: the per-expert groups become library GEMMs
    for ei in range(e):
        a0, a1 = off[ei], off[ei + 1]
        if a1 > a0:
            F.linear(gated_act(F.linear(xs[a0:a1], w13[ei]), ACT_SILU), w2[ei], out=ys[a0:a1])
    return finish(ys, pos)


def route_softmax_topk(x: torch.Tensor, router: torch.Tensor, k: int, n_route: int,
                       correction: Optional[torch.Tensor] = None, gate_row: bool = False):
    """Softmax-scored routing over ``n_route`` choices (fp32 logits x . router[e], e < n_route): the k largest
    scores + correction (lowest index on ties) are chosen; their weights are the scores WITHOUT the correction,
    divided by their sum (+ 1e-20). With ``gate_row`` the router has one more row whose logit goes through a sigmoid
    (a per-token gate that rides in the same product). Returns (w [T, k] fp32, ids [T, k] int32, gate [T] fp32 or
    None)."""
    t = x.shape[0]
    rows = n_route + (1 if gate_row else 0)
    if not x.is_cuda:
        z = x.float() @ router[:rows].float().t()
        w, ids = ref.softmax_topk_corrected(z[:, :n_route], k, correction)
        return w, ids, (torch.sigmoid(z[:, n_route]).contiguous() if gate_row else None)
    w = torch.empty(t, k, dtype=torch.float32, device=x.device)
    ids = torch.empty(t, k, dtype=torch.int32, device=x.device)
    gate = torch.empty(t, dtype=torch.float32, device=x.device) if gate_row else None
    if t > ROUTE_FUSED_MAX_T:
        # prompt-sized steps: the logits as one true-fp32 library GEMM, then the selection kernel
        _kern().topk_softmax_corrected(w, ids, gate, F.linear(x.float(), router[:rows].float()), n_route, correction)
    else:
        _kern().route_softmax_topk(w, ids, gate, x, router.contiguous(), n_route, correction)
    return w, ids, gate


def moe_output_weighted(x: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, w: torch.Tensor, ids: torch.Tensor,
                        kind: int, limit: float, alpha: float, n_route: int = 0,
                        extra: Optional[torch.Tensor] = None, extra_gate: Optional[torch.Tensor] = None,
                        post_norm=None) -> Optional[torch.Tensor]:
    """out[t] (fp32) = sum_j w[t, j] * expert_{ids[t, j]}(x[t]) (+ extra_gate[t] * extra[t]); expert(z) =
    W2 act(W1 z, W3 z) with w13 [E, 2f, H] = [W1; W3], w2 [E, H, f] and ``act`` one of :func:`gated_act`'s kinds. An
    id in [E, n_route) names an identity expert, whose output is x[t] itself. The routing weight multiplies the expert's OUTPUT
    (in fp32, in the launch that sums). ``post_norm`` = (resid fp32 [T, H], norm weight, eps, unit_offset, act or
    None, mult): instead of returning the sum, add mult * its RMS-normalised form into ``resid`` (and refresh ``act``)
    in the same launch; returns None."""
    if not x.is_cuda:
        out = ref.moe_output_weighted(x, w13, w2, w, ids, kind, limit, alpha, extra, extra_gate)
        if post_norm is None:
            return out
        resid, nw, eps, unit, act, mult = post_norm
        post_norm_residual(resid, out, nw, eps, unit, act=act, mult=mult)
        return None
    kern = _kern()
    t, h = x.shape
    k = ids.shape[1]
    n = t * k
    e = w13.shape[0]
    x = x.contiguous()
    w = w.contiguous()

    def finish(ys, pos):
        if post_norm is not None:
            resid, nw, eps, unit, act, mult = post_norm
            kern.combine_weighted(None, resid, act, ys, pos, x, w, ids, e, extra, extra_gate, nw, unit, eps, float(mult))
            return None
        out = torch.empty(t, h, dtype=torch.float32, device=x.device)
        kern.combine_weighted(out, None, None, ys, pos, x, w, ids, e, extra, extra_gate, None, False, 0.0, 1.0)
        return out

    if e == 0:
        return finish(torch.empty(0, h, dtype=x.dtype, device=x.device), None)
    buckets = max(e, int(n_route))
    if x.dtype == torch.bfloat16 and t <= 128:
        # decode-sized steps: the framework's expert-streaming grouped GEMM (every routed expert's weights streamed
        # once; rows gathered in expert-sorted order by the kernel; no host read, hipGraph-capturable). Identity
        # entries sort behind the last real expert and run nothing.
        from src import ops

        tiles = None
        if ops.native_available() and h % 32 == 0 and w2.shape[2] % 32 == 0:
            try:
                b = ops._bucket(t)
                tiles = (ops._generic_tile(w13.shape[1], h, 0, b, max_sk=1)[:2],
                         ops._generic_tile(h, w2.shape[2], 0, b, max_sk=1)[:2])
            except ValueError:
                tiles = None
        if tiles is not None:
            ck = ops._kern()
            (wr1, kc1), (wr2, kc2) = tiles
            offsets = torch.empty(buckets + 1, dtype=torch.int32, device=x.device)
            sorted_idx = torch.empty(n, dtype=torch.int32, device=x.device)
            pos = torch.empty(n, dtype=torch.int32, device=x.device)
            kern.moe_align(offsets, sorted_idx, pos, ids.reshape(-1).contiguous(), buckets)
            g = torch.empty(n, w13.shape[1], dtype=x.dtype, device=x.device)
            ys = torch.empty(n, h, dtype=x.dtype, device=x.device)
            ck.gemm_decode_grouped(g, x, w13, offsets, 0, wr1, kc1, sorted_idx, k, t, 1)
            ck.gemm_decode_grouped(ys, gated_act(g, kind, limit, alpha), w2, offsets, 0, wr2, kc2,
                                   ops._NO_ROWS(x.device), 1, t, 1)
            return finish(ys, pos)
    if n <= MOE_BMM_MAX_ROWS or torch.cuda.is_current_stream_capturing():
        # decode-sized steps: the routed experts' weights gathered per row for two batched products (no host read,
        # hipGraph-capturable); an identity entry runs expert E - 1 and its product is ignored by the sum
        sel = ids.reshape(-1).long().clamp_(max=e - 1)
        xr = x.unsqueeze(1).expand(t, k, h).reshape(n, h, 1)
        g = torch.bmm(w13.index_select(0, sel), xr).squeeze(2)
        ys = torch.bmm(w2.index_select(0, sel), gated_act(g, kind, limit, alpha).unsqueeze(2)).squeeze(2).contiguous()
        return finish(ys, None)
    # prompt-sized steps: rows sorted by expert (identity entries sort last and run nothing), one library GEMM pair
    # per real expert over its rows
    offsets = torch.empty(buckets + 1, dtype=torch.int32, device=x.device)
    sorted_idx = torch.empty(n, dtype=torch.int32, device=x.device)
    pos = torch.empty(n, dtype=torch.int32, device=x.device)
    kern.moe_align(offsets, sorted_idx, pos, ids.reshape(-1).contiguous(), buckets)
    xs = torch.empty(n, h, dtype=x.dtype, device=x.device)
    kern.gather_scaled(xs, x, sorted_idx, None, k)
    ys = torch.empty(n, h, dtype=x.dtype, device=x.device)
    off = offsets.tolist()  # one host read per layer: the per-expert groups become library GEMMs
    for ei in range(e):
        a0, a1 = off[ei], off[ei + 1]
        if a1 > a0:
            F.linear(gated_act(F.linear(xs[a0:a1], w13[ei]), kind, limit, alpha), w2[ei], out=ys[a0:a1])
    return finish(ys, pos)


def rope_inv_freq(base: float, dims: int, device, scaling: Optional[Tuple[float, float, float, float]] = None) -> torch.Tensor:
    """fp32 [dims / 2]: base^(-2 i / dims), rounded once from float64. ``scaling`` = (factor, low, high, original)
    stretches long wavelengths: with l = 2 pi / f, f stays where l < original / high, becomes f / factor where
    l > original / low, and in between (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    if scaling is not None:
        factor, low, high, orig = (float(v) for v in scaling)
        wl = 2.0 * math.pi / f
        s = (orig / wl - low) / (high - low) if high != low else torch.ones_like(f)
        mid = (1.0 - s) * f / factor + s * f
        f = torch.where(wl < orig / high, f, torch.where(wl > orig / low, f / factor, mid))
    return f.float().to(device)


def latent_kv_write(cache: torch.Tensor, kv: torch.Tensor, w: torch.Tensor, positions: torch.Tensor,
                    slots: torch.Tensor, rank: int, rot_dim: int, inv_freq: torch.Tensor, eps: float) -> None:
    """cache [blocks, block_size, rank + rot_dim]: the row at slot slots[t] (< 0: skipped) becomes
    [rmsnorm(kv[t, :rank]) * w | kv[t, rank:] with its first 2 * len(inv_freq) dims rotated as interleaved
    pairs (2i, 2i + 1) by the angle positions[t] * inv_freq[i]]."""
    if not kv.is_cuda:
        ref.latent_kv_write(cache, kv, w, positions, slots, rank, rot_dim, inv_freq, eps)
        return
    _kern().latent_kv_write(cache, kv, w, positions, slots, rank, rot_dim, inv_freq, eps)


def latent_qkv_prep(p: torch.Tensor, q_rank: int, wq: torch.Tensor, wkv: torch.Tensor, cache: torch.Tensor,
                    positions: torch.Tensor, slots: torch.Tensor, rank: int, rot_dim: int, inv_freq: torch.Tensor,
                    eps: float) -> torch.Tensor:
    """Both consumers of the fused down-projection p [T, q_rank + rank + rot_dim] in one launch: returns
    cq = rmsnorm(p[:, :q_rank]) * wq (model dtype) and writes the cache rows from p[:, q_rank:] as
    :func:`latent_kv_write` does."""
    if not p.is_cuda:
        latent_kv_write(cache, p[:, q_rank:], wkv, positions, slots, rank, rot_dim, inv_freq, eps)
        return rms_norm_ext(p[:, :q_rank], wq, eps)
    cq = torch.empty(p.shape[0], q_rank, dtype=p.dtype, device=p.device)
    _kern().latent_qkv_prep(cq, cache, p, wq, wkv, positions, slots, rank, rot_dim, inv_freq, eps)
    return cq


def latent_attn(q_lat: torch.Tensor, q: torch.Tensor, rot_off: int, cache: torch.Tensor, block_tables: torch.Tensor,
                cu_q: Optional[torch.Tensor], ctx_lens: torch.Tensor, positions: torch.Tensor,
                sink: Optional[torch.Tensor], max_q: int, window: int, scale: float, rot_dim: int,
                inv_freq: torch.Tensor, impl: int = 0) -> torch.Tensor:
    """Absorbed latent attention. q_lat [H, T, rank]: the queries projected into the latent space; q [T, H * qh]:
    the full queries, head h's rotary part at [h * qh + rot_off, + rot_dim) (rotated here, by positions[t]).
    Row (t, h) scores the cache rows j of its sequence with 0 <= p - j < window (window 0: j <= p):
    (q_lat . latent_j + q_rot . krot_j) * scale, softmax with exp(sink[h]) added to the denominator, and
    returns the weighted sum of the latent rows, [H, T, rank]. cu_q None: one query row per sequence.
    ``impl`` (GPU): 0 = the matrix-core kernel where it applies (bf16, rank % 32 == 0, rank <= 256,
    rot_dim % 16 == 0), else the FMA kernel; 1 = the FMA kernel; 2 = the matrix-core kernel or an error;
    3 = as 2 but never its register-query variant (tests, A/B)."""
    if not q_lat.is_cuda:
        return ref.latent_attn(q_lat, q, rot_off, cache, block_tables, cu_q, ctx_lens, positions, sink, window, scale,
                               rot_dim, inv_freq)
    out = torch.empty_like(q_lat)
    _kern().latent_attn(out, q_lat, q, rot_off, cache, block_tables, cu_q, ctx_lens, positions, sink, max_q, window,
                        scale, rot_dim, inv_freq, impl)
    return out
