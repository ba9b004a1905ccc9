"""
Plain-PyTorch fp32 reference implementations of every custom op.

They define the semantics the gfx950 kernels must match (the numerics tests
compare kernel vs. these) and run the engine on CPU tensors for control-flow
tests. They are never used for GPU tensors: :mod:`src.ops` routes GPU tensors
to the HIP extension and raises if it is missing.
"""

from __future__ import annotations

import math
from typing import Optional

import torch


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    return (xf * torch.rsqrt(var + eps) * w.float()).to(x.dtype)


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor, eps: float):
    r = (x.float() + residual.float()).to(residual.dtype)
    return rms_norm(r, w, eps), r


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    i = x.shape[-1] // 2
    g, u = x[..., :i].float(), x[..., i:].float()
    return (torch.nn.functional.silu(g) * u).to(x.dtype)


def rope_cos_sin(max_pos: int, head_dim: int, theta: float, device=None, scaling: Optional[dict] = None) -> torch.Tensor:
    """[max_pos, head_dim] fp32 table: cos in the first half, sin in the second."""
    half = head_dim // 2
    inv = 1.0 / (theta ** (torch.arange(0, half, dtype=torch.float64) / half))
    if scaling and scaling.get("rope_type") == "llama3":
        factor = scaling["factor"]
        lo, hi = scaling.get("low_freq_factor", 1.0), scaling.get("high_freq_factor", 4.0)
        old = scaling.get("original_max_position_embeddings", 8192)
        wavelen = 2 * math.pi / inv
        lo_w, hi_w = old / lo, old / hi
        smooth = (old / wavelen - lo) / (hi - lo)
        scaled = torch.where(wavelen > lo_w, inv / factor, inv)
        mid = (wavelen <= lo_w) & (wavelen >= hi_w)
        inv = torch.where(mid, (1 - smooth) * inv / factor + smooth * inv, scaled)
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv)
    return torch.cat([f.cos(), f.sin()], dim=-1).float().to(device)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor) -> torch.Tensor:
    """x [T, H, D] neox-style rotation."""
    d = x.shape[-1]
    half = d // 2
    cs = cos_sin[positions.long()]
    cos, sin = cs[:, None, :half], cs[:, None, half:]
    xf = x.float()
    a, b = xf[..., :half], xf[..., half:]
    return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1).to(x.dtype)


def rope_and_cache(qkv, positions, cos_sin, slot_mapping, k_cache, v_cache, hq, hkv, head_dim):
    t = qkv.shape[0]
    q = qkv[:, : hq * head_dim].view(t, hq, head_dim)
    k = qkv[:, hq * head_dim:(hq + hkv) * head_dim].view(t, hkv, head_dim)
    v = qkv[:, (hq + hkv) * head_dim:(hq + 2 * hkv) * head_dim].view(t, hkv, head_dim)
    qr = apply_rope(q, positions, cos_sin)
    kr = apply_rope(k, positions, cos_sin)
    qkv[:, : hq * head_dim] = qr.reshape(t, -1)
    bs = k_cache.shape[2]
    for i in range(t):
        s = int(slot_mapping[i])
        if s < 0:
            continue
        k_cache[s // bs, :, s % bs] = kr[i]
        v_cache[s // bs, :, s % bs] = v[i]


def gather_kv(cache: torch.Tensor, block_table: torch.Tensor, n: int) -> torch.Tensor:
    """[n, hkv, D] rows 0..n-1 of one sequence from the paged cache."""
    bs = cache.shape[2]
    pos = torch.arange(n, device=cache.device)
    blocks = block_table[(pos // bs).long()].long()
    return cache[blocks, :, pos % bs]


def attention(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, hq, hkv, scale):
    """Causal paged attention; q [T, >=hq*D] (rows may be strided) → [T, hq, D]."""
    d = 128
    out = torch.empty(q.shape[0], hq, d, dtype=q.dtype, device=q.device)
    g = hq // hkv
    for s in range(ctx_lens.numel()):
        a, b = int(cu_q[s]), int(cu_q[s + 1])
        qlen, ctx = b - a, int(ctx_lens[s])
        if qlen == 0:
            continue
        qs = q[a:b, : hq * d].reshape(qlen, hq, d).float()
        k = gather_kv(k_cache, block_tables[s], ctx).float().repeat_interleave(g, dim=1)
        v = gather_kv(v_cache, block_tables[s], ctx).float().repeat_interleave(g, dim=1)
        sc = torch.einsum("qhd,khd->hqk", qs, k) * scale
        qpos = torch.arange(ctx - qlen, ctx, device=q.device)[:, None]
        kpos = torch.arange(ctx, device=q.device)[None, :]
        sc = sc.masked_fill((kpos > qpos)[None], float("-inf"))
        p = torch.softmax(sc, dim=-1)
        out[a:b] = torch.einsum("hqk,khd->qhd", p, v).to(q.dtype)
    return out


def sample(logits, temperature=None, top_k=None, top_p=None, seeds=None, steps=None):
    """Greedy where temperature==0; otherwise a (non-bit-exact) torch sampler
    with the same filtering semantics (top-k, then top-p on the renormalised set)."""
    out = torch.empty(logits.shape[0], dtype=torch.long, device=logits.device)
    for r in range(logits.shape[0]):
        row = logits[r].float()
        t = float(temperature[r]) if temperature is not None else 0.0
        k = int(top_k[r]) if top_k is not None else 0
        if t <= 0 or k == 1:
            out[r] = int(torch.argmax(row))
            continue
        z = row / t
        keep = torch.ones_like(z, dtype=torch.bool)
        if 0 < k < z.numel():
            kth = torch.topk(z, k).values[-1]
            keep &= z >= kth
        p = float(top_p[r]) if top_p is not None else 1.0
        if p < 1.0:
            zz = z.masked_fill(~keep, float("-inf"))
            probs = torch.softmax(zz, -1)
            sp, si = torch.sort(probs, descending=True)
            cum = torch.cumsum(sp, 0)
            cut = int(torch.searchsorted(cum, torch.tensor(p, device=cum.device))) + 1
            thr = sp[min(cut, sp.numel()) - 1]
            keep &= probs >= thr
        probs = torch.softmax(z.masked_fill(~keep, float("-inf")), -1)
        gen = torch.Generator(device="cpu")
        gen.manual_seed(int(seeds[r]) * 1000003 + int(steps[r]) if seeds is not None and steps is not None else 0)
        out[r] = int(torch.multinomial(probs.cpu(), 1, generator=gen))
    return out


def topk_softmax(gating: torch.Tensor, k: int, renorm: bool = True):
    p = torch.softmax(gating.float(), dim=-1)
    w, ids = torch.topk(p, k, dim=-1)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return w, ids.int()


def moe_forward(x, w13, w2, gating, k: int, renorm: bool = True):
    """Reference MoE FFN: x [T,H], w13 [E, 2I, H], w2 [E, H, I]."""
    w, ids = topk_softmax(gating, k, renorm)
    return moe_experts(x, w13, w2, w, ids)


def moe_experts(x, w13, w2, w, ids):
    """Experts' weighted sum for given routing (w [T,k], ids [T,k]); ids >= E are skipped."""
    out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
    inter = w2.shape[-1]
    for e in range(w13.shape[0]):
        tok, slot = (ids == e).nonzero(as_tuple=True)
        if tok.numel() == 0:
            continue
        h = x[tok].float() @ w13[e].float().t()
        a = torch.nn.functional.silu(h[:, :inter]) * h[:, inter:]
        y = a.to(x.dtype).float() @ w2[e].float().t()
        out.index_add_(0, tok, y * w[tok, slot][:, None])
    return out.to(x.dtype)


# ----------------------------------------------------------------- dtype-generic ops (src/ops/mix.py)
def rms_norm_ext(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, unit_offset: bool = False,
                 out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    xf = x.float()
    y = xf / torch.sqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if w is not None:
        y = y * (w.float() + 1.0 if unit_offset else w.float())
    return y.to(out_dtype or x.dtype)


def gated_act(gu: torch.Tensor, kind: int, limit: float, alpha: float) -> torch.Tensor:
    f = gu.shape[-1] // 2
    g, u = gu[..., :f].float(), gu[..., f:].float()
    if kind == 0:
        return (g * torch.sigmoid(g) * u).to(gu.dtype)
    if kind == 2:
        gg = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
        return (gg * u).to(gu.dtype)
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, -limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def route_sigmoid_topk(x: torch.Tensor, router: torch.Tensor, k: int):
    z = x.float() @ router.float().t()
    zs, ids = torch.sort(z, dim=-1, descending=True, stable=True)
    return torch.sigmoid(zs[:, :k]).contiguous(), ids[:, :k].to(torch.int32).contiguous()


def moe_input_scaled(x, w13, w2, w, ids, extra=None) -> torch.Tensor:
    t, h = x.shape
    out = torch.zeros(t, h, dtype=torch.float32) if extra is None else extra.float().clone()
    for j in range(ids.shape[1]):
        for e in ids[:, j].unique().tolist():
            rows = (ids[:, j] == e).nonzero().flatten()
            xs = (w[rows, j, None] * x[rows].float()).to(x.dtype)
            a = gated_act(torch.nn.functional.linear(xs, w13[e]), 0, 0.0, 1.0)
            out[rows] += torch.nn.functional.linear(a, w2[e]).float()
    return out


def softmax_topk_corrected(z: torch.Tensor, k: int, correction: Optional[torch.Tensor]):
    """z [T, E] fp32 logits: the k largest softmax(z) + correction (lowest index on ties); weights = the chosen
    scores without the correction, over their sum + 1e-20."""
    s = torch.softmax(z.float(), -1)
    c = s if correction is None else s + correction.float()
    ids = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :k]
    w = torch.gather(s, 1, ids)
    return (w / (w.sum(-1, keepdim=True) + 1e-20)).contiguous(), ids.to(torch.int32).contiguous()


def moe_output_weighted(x, w13, w2, w, ids, kind, limit, alpha, extra=None, extra_gate=None) -> torch.Tensor:
    t, h = x.shape
    e_real = w13.shape[0]
    out = torch.zeros(t, h, dtype=torch.float32)
    for j in range(ids.shape[1]):
        for e in ids[:, j].unique().tolist():
            rows = (ids[:, j] == e).nonzero().flatten()
            if e >= e_real:
                y = x[rows].float()
            else:
                a = gated_act(torch.nn.functional.linear(x[rows], w13[e]), kind, limit, alpha)
                y = torch.nn.functional.linear(a, w2[e]).float()
            out[rows] += w[rows, j, None] * y
    if extra is not None:
        out += extra.float() if extra_gate is None else extra_gate[:, None] * extra.float()
    return out


def _rotate_pairs(x: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """x [..., n] fp32 with a leading token dim: the first 2 * len(inv_freq) dims rotate as pairs (2i, 2i + 1)."""
    n = 2 * inv_freq.numel()
    ang = pos.float().reshape(-1, *([1] * (x.dim() - 1))) * inv_freq.float()
    cs, sn = ang.cos(), ang.sin()
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * cs - v * sn
    out[..., 1:n:2] = v * cs + u * sn
    return out


def latent_kv_write(cache, kv, w, positions, slots, rank, rot_dim, inv_freq, eps) -> None:
    t = kv.shape[0]
    c = rms_norm_ext(kv[:, :rank], w, eps).float()
    kr = _rotate_pairs(kv[:, rank:rank + rot_dim].float(), positions[:t], inv_freq)
    rows = torch.cat([c, kr], -1).to(cache.dtype)
    flat = cache.view(-1, cache.shape[-1])
    for i in range(t):
        s = int(slots[i])
        if s >= 0:
            flat[s] = rows[i]


def latent_attn(q_lat, q, rot_off, cache, block_tables, cu_q, ctx_lens, positions, sink, window, scale, rot_dim,
                inv_freq) -> torch.Tensor:
    heads, total, rank = q_lat.shape
    qh = q.shape[1] // heads
    qr = q.view(total, heads, qh)[:, :, rot_off:rot_off + rot_dim].float()
    qr = _rotate_pairs(qr, positions[:total], inv_freq)
    out = torch.zeros(heads, total, rank, dtype=torch.float32)
    bs = cache.shape[1]
    nseq = block_tables.shape[0]
    for s in range(nseq):
        a, b = (int(cu_q[s]), int(cu_q[s + 1])) if cu_q is not None else (s, s + 1)
        if b <= a:
            continue
        ctx = int(ctx_lens[s])
        idx = torch.arange(ctx)
        rows = cache[block_tables[s].long()[idx // bs], idx % bs].float()      # [ctx, rank + rot_dim]
        p = positions[a:b].long()
        sc = (torch.einsum("hqr,jr->hqj", q_lat[:, a:b].float(), rows[:, :rank])
              + torch.einsum("qhd,jd->hqj", qr[a:b], rows[:, rank:])) * scale
        d = p[:, None] - idx[None, :]
        ok = d >= 0
        if window > 0:
            ok = ok & (d < window)
        sc = sc.masked_fill(~ok[None], float("-inf"))
        mx = sc.max(-1).values
        if sink is not None:
            mx = torch.maximum(mx, sink.float()[:, None])
        mx = torch.where(torch.isfinite(mx), mx, torch.zeros_like(mx))
        e = torch.exp(sc - mx[..., None])
        den = e.sum(-1)
        if sink is not None:
            den = den + torch.exp(sink.float()[:, None] - mx)
        pr = e / den.clamp_min(1e-38)[..., None]
        out[:, a:b] = torch.einsum("hqj,jr->hqr", pr, rows[:, :rank])
    return out.to(q_lat.dtype)
