"""
A plain, slow implementation of the Kogerax design in float64, written from its equations: dense masks, explicit
loops over time, no cache, no batching, one function per mechanism. It shares no code with ``src/`` and is what
``tests/test_kogerax.py`` compares the engine with. It also makes the tests' configurations and random weights.

Notation: ``h`` [T, W] is a sublayer's input, weights are stored [out, in] and applied as ``h @ W.T``; positions count
from 0; rms(x) = x / sqrt(mean(x^2) + eps).
"""

from __future__ import annotations

import math
from typing import Any, Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def logsigmoid(x):
    return -softplus(-x)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------------------------------------- positions
def rotary_frequencies(rot: Dict[str, Any]) -> torch.Tensor:
    """f_i = base^(-2i/dims) for i < dims/2, then the wavelength-dependent rescaling: short wavelengths keep f, long
    ones use f / factor, those between are blended linearly in original / wavelength."""
    dims = int(rot["dims"])
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f
    factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = f.clone()
    for i in range(f.numel()):
        wl = 2.0 * math.pi / float(f[i])
        if wl < orig / high:
            continue
        if wl > orig / low:
            out[i] = f[i] / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[i] = (1.0 - s) * f[i] / factor + s * f[i]
    return out


def rotate(x: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """x [T, heads, dim]: dimension i is paired with i + n (n = len(freqs)) and the pair turns by position * f_i; the
    dimensions from 2n on pass unchanged."""
    T = x.shape[0]
    n = freqs.numel()
    ang = torch.arange(T, dtype=F64)[:, None] * freqs[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :n], x[..., n: 2 * n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], -1)


# ---------------------------------------------------------------------------------------------------- mixers
def window_attention(h, w: Dict[str, torch.Tensor], m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Grouped-query softmax attention: partial rotary positions, then q and k divided by their per-head root mean
    square, a sliding window, plain softmax."""
    T, H, D, V = h.shape[0], m["heads"], m["dim"], m["vdim"]
    G = m.get("kv_heads") or H
    q = (h @ w["q"].T).view(T, H, D)
    k = (h @ w["k"].T).view(T, G, D)
    v = (h @ w["v"].T).view(T, G, V)
    if m.get("rot"):
        fr = rotary_frequencies(m["rot"])
        q, k = rotate(q, fr), rotate(k, fr)
    q, k = rms(q, eps), rms(k, eps)
    win = (m.get("mask") or {}).get("size") or 0
    out = torch.zeros(T, H, V, dtype=F64)
    for i in range(T):
        lo = max(0, i - win + 1) if win else 0
        for hd in range(H):
            g = hd // (H // G)
            s = (k[lo: i + 1, g] @ q[i, hd]) * m["scale"]
            p = torch.softmax(s, 0)
            out[i, hd] = (p[:, None] * v[lo: i + 1, g]).sum(0)
    return out.reshape(T, H * V) @ w["o"].T


def causal_conv(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """x [T, C], w [C, taps] (last column: the current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], 0)
    out = b[None, :].expand(T, C).clone()
    for j in range(taps):
        out = out + pad[j: j + T] * w[:, j][None, :]
    return out


def selective_scan(h, w: Dict[str, torch.Tensor], m: Dict[str, Any]) -> torch.Tensor:
    """Mamba: a diagonal state per channel with input-dependent step size, input and output maps."""
    T = h.shape[0]
    I, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ w["in"].T
    x, z = xz[:, :I], xz[:, I:]
    x = silu(causal_conv(x, w["conv"], w["conv.b"]))
    p = x @ w["x"].T
    dt, B, C = p[:, :R], p[:, R: R + N], p[:, R + N: R + 2 * N]
    dt = softplus(dt @ w["dt"].T + w["dt.b"])                      # [T, I]
    A = -torch.exp(w["A_log"])                                     # [I, N]
    S = torch.zeros(I, N, dtype=F64)
    y = torch.zeros(T, I, dtype=F64)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + w["D"] * x[t]
    return (y * silu(z)) @ w["o"].T


def parallel(h, w: Dict[str, torch.Tensor], m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Attention and a selective scan on the same input; each output normed over the width with a plain weight;
    half their sum."""
    def side(prefix):
        return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}

    wl, wr = side("left."), side("right.")
    a = rms(window_attention(h, wl, m["left"], eps), eps) * wl["out"]
    b = rms(selective_scan(h, wr, m["right"]), eps) * wr["out"]
    return 0.5 * (a + b)


def mlstm(h, w: Dict[str, torch.Tensor], m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Matrix-memory LSTM: exponential input gate and sigmoid forget gate in log space, stabilised by a running
    maximum that starts at 0; a normaliser vector beside the matrix; per-head norm, output gate."""
    T, H, D, V = h.shape[0], m["heads"], m["dim"], m["vdim"]
    cap = float(m["gate_cap"])
    q = (h @ w["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, V)
    ig = cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap)                      # [T, H]
    fg = logsigmoid(cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap))
    o = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, V, dtype=F64)
        n = torch.zeros(D, dtype=F64)
        mx = torch.zeros((), dtype=F64)
        for t in range(T):
            m_new = torch.maximum(fg[t, hd] + mx, ig[t, hd])
            a, b = torch.exp(fg[t, hd] + mx - m_new), torch.exp(ig[t, hd] - m_new)
            S = a * S + b * torch.outer(k[t, hd], v[t, hd])
            n = a * n + b * k[t, hd]
            mx = m_new
            den = torch.maximum(torch.abs(n @ q[t, hd]), torch.exp(-mx)) + 1e-6
            o[t, hd] = (S.T @ q[t, hd]) / den
    o = rms(o, eps).reshape(T, H * V) * w["norm"] * sigmoid(h @ w["g"].T)
    return o @ w["o"].T


def mamba2(h, w: Dict[str, torch.Tensor], m: Dict[str, Any], eps: float) -> torch.Tensor:
    """State-space duality layer: a scalar decay per head and token, input and output maps shared by the heads of a
    group; gate, then a norm in equal parts."""
    T, H, V, N, G = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"]
    I = H * V
    p = h @ w["in"].T
    z, xbc, dt = p[:, :I], p[:, I: 2 * I + 2 * G * N], p[:, 2 * I + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w["conv"], w["conv.b"]))
    x = xbc[:, :I].view(T, H, V)
    B = xbc[:, I: I + G * N].view(T, G, N)
    C = xbc[:, I + G * N:].view(T, G, N)
    dt = softplus(dt + w["dt_bias"])                                            # [T, H]
    decay = torch.exp(-torch.exp(w["A_log"])[None, :] * dt)
    y = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, V, dtype=F64)
        for t in range(T):
            S = decay[t, hd] * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + w["D"][hd] * x[t, hd]
    y = y.reshape(T, I) * silu(z)
    parts = int(m.get("norm_groups") or 1)
    y = rms(y.view(T, parts, I // parts), eps).reshape(T, I) * w["norm"]
    return y @ w["o"].T


MIXERS = {"parallel": parallel, "mlstm": mlstm, "mamba2": lambda h, w, m, eps: mamba2(h, w, m, eps)}


# ---------------------------------------------------------------------------------------------- feed-forward
def dense_ff(h, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def expert(h, w: Dict[str, torch.Tensor], limit: float) -> torch.Tensor:
    g = torch.clamp(h @ w["gate"].T, max=limit)
    u = torch.clamp(h @ w["up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def route(h, w: Dict[str, torch.Tensor], f: Dict[str, Any]):
    """(chosen experts [T, top], their weights [T, top]): softmax scores over real + identity experts; the choice adds
    a correction to the scores, the weights are the chosen scores themselves, renormalised."""
    s = torch.softmax(h @ w["router"].T, -1)
    choice = s + w["correction"] if "correction" in w else s
    ids = torch.topk(choice, int(f["router"]["top"]), dim=-1).indices
    ws = torch.gather(s, 1, ids)
    return ids, ws / (ws.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, w: Dict[str, torch.Tensor], f: Dict[str, Any]) -> torch.Tensor:
    T = h.shape[0]
    E = int(f["router"]["experts"])
    ids, ws = route(h, w, f)
    out = torch.zeros_like(h)
    for t in range(T):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            if e >= E:                       # an identity expert: the input itself
                out[t] += ws[t, j] * h[t]
            else:
                we = {k[len(f"e{e}."):]: v for k, v in w.items() if k.startswith(f"e{e}.")}
                out[t] += ws[t, j] * expert(h[t: t + 1], we, float(f["expert"]["limit"]))[0]
    if f.get("shared"):
        wsh = {k[len("shared."):]: v for k, v in w.items() if k.startswith("shared.")}
        out = out + sigmoid(h @ wsh["sg"].T) * expert(h, wsh, float(f["shared"]["limit"]))
    return out


def feed_forward(h, w, f):
    return dense_ff(h, w) if f["kind"] == "dense" else moe_ff(h, w, f)


# ----------------------------------------------------------------------------------------------------- model
def forward(config: Dict[str, Any], weights: Dict[str, torch.Tensor], tokens: List[int], keep_layers: bool = False):
    """Logits [T, vocab] of one sequence (float64); with ``keep_layers`` also the stream after every layer."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    mult = float(config.get("residual_mult", 1.0))

    def sub(prefix):
        return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}

    x = W["embed"][torch.tensor(tokens)] * float((config.get("embedding") or {}).get("scale", 1.0))
    kept = []
    for i, lc in enumerate(config["layers"]):
        p = f"l{i}."
        y = MIXERS[lc["type"]](x, sub(p + "mix."), lc["mixer"], eps)
        x = x + mult * rms(y, eps) * (1.0 + W[p + "norm1"])
        if lc.get("mlp") is not None:
            y = feed_forward(x, sub(p + "mlp."), lc["mlp"])
            x = x + mult * rms(y, eps) * (1.0 + W[p + "norm2"])
        kept.append(x.clone())
    logits = (rms(x, eps) * (1.0 + W["final.norm"])) @ W["head"].T
    return (logits, torch.stack(kept)) if keep_layers else logits


# ---------------------------------------------------------------------------------- configurations + weights
def tensor_shapes(config: Dict[str, Any]) -> Dict[str, tuple]:
    Wd, out = int(config["width"]), {}
    out["embed"] = (int(config["vocab"]), Wd)
    for i, lc in enumerate(config["layers"]):
        p, m, t = f"l{i}.", lc["mixer"], lc["type"]
        out[p + "norm1"] = (Wd,)
        if t == "mlstm":
            H, D, V = m["heads"], m["dim"], m["vdim"]
            for nm, r in (("q", H * D), ("k", H * D), ("v", H * V), ("g", H * V), ("i", H), ("f", H)):
                out[p + "mix." + nm] = (r, Wd)
            out[p + "mix.i.b"], out[p + "mix.f.b"] = (H,), (H,)
            out[p + "mix.norm"], out[p + "mix.o"] = (H * V,), (Wd, H * V)
        elif t == "mamba2":
            H, V, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            I = H * V
            out[p + "mix.in"] = (2 * I + 2 * G * N + H, Wd)
            out[p + "mix.conv"], out[p + "mix.conv.b"] = (I + 2 * G * N, K), (I + 2 * G * N,)
            out[p + "mix.dt_bias"], out[p + "mix.A_log"], out[p + "mix.D"] = (H,), (H,), (H,)
            out[p + "mix.norm"], out[p + "mix.o"] = (I,), (Wd, I)
        elif t == "parallel":
            l, r = m["left"], m["right"]
            H, G, D, V = l["heads"], l.get("kv_heads") or l["heads"], l["dim"], l["vdim"]
            q = p + "mix.left."
            out[q + "q"], out[q + "k"], out[q + "v"] = (H * D, Wd), (G * D, Wd), (G * V, Wd)
            out[q + "o"], out[q + "out"] = (Wd, H * V), (Wd,)
            q = p + "mix.right."
            I, N, R, K = r["inner"], r["state"], r["dt_rank"], r["conv"]
            out[q + "in"], out[q + "conv"], out[q + "conv.b"] = (2 * I, Wd), (I, K), (I,)
            out[q + "x"], out[q + "dt"], out[q + "dt.b"] = (R + 2 * N, I), (I, R), (I,)
            out[q + "A_log"], out[q + "D"], out[q + "o"], out[q + "out"] = (I, N), (I,), (Wd, I), (Wd,)
        else:
            raise ValueError(t)
        f = lc.get("mlp")
        if f is None:
            continue
        out[p + "norm2"] = (Wd,)
        q = p + "mlp."
        if f["kind"] == "dense":
            out[q + "gate"], out[q + "up"], out[q + "down"] = (f["ff"], Wd), (f["ff"], Wd), (Wd, f["ff"])
        else:
            E, idn = f["router"]["experts"], int(f["router"].get("identity") or 0)
            for e in range(E):
                ff = f["expert"]["ff"]
                out[q + f"e{e}.gate"], out[q + f"e{e}.up"], out[q + f"e{e}.down"] = (ff, Wd), (ff, Wd), (Wd, ff)
            out[q + "router"], out[q + "correction"] = (E + idn, Wd), (E + idn,)
            if f.get("shared"):
                ff = f["shared"]["ff"]
                out[q + "shared.gate"], out[q + "shared.up"] = (ff, Wd), (ff, Wd)
                out[q + "shared.down"], out[q + "shared.sg"] = (Wd, ff), (1, Wd)
    out["final.norm"], out["head"] = (Wd,), (int(config["vocab"]), Wd)
    return out


def make_weights(config: Dict[str, Any], seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Random weights of sizes that keep every mechanism visible: gates neither saturated nor dead, decays that reach
    back tens of tokens, router scores with clear gaps. Values are rounded to bf16 so both dtypes load the same."""
    g = torch.Generator().manual_seed(seed)
    Wd = int(config["width"])
    out = {}
    for name, shape in tensor_shapes(config).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and name[1].isdigit() else name
        if name == "embed":
            t = torch.randn(shape, generator=g) * 0.5
        elif name == "head":
            t = torch.randn(shape, generator=g) * (2.0 / math.sqrt(Wd))
        elif leaf in ("norm1", "norm2") or name == "final.norm":
            t = torch.randn(shape, generator=g) * 0.1
        elif leaf.endswith(".out") or leaf == "mix.norm":
            t = 1.0 + torch.randn(shape, generator=g) * 0.1
        elif leaf.endswith("A_log"):
            t = torch.log(0.3 + 1.5 * torch.rand(shape, generator=g))
        elif leaf.endswith(".D"):
            t = 1.0 + torch.randn(shape, generator=g) * 0.2
        elif leaf.endswith("dt_bias") or leaf.endswith("dt.b"):
            t = torch.randn(shape, generator=g) * 0.5 - 1.5
        elif leaf.endswith("conv"):
            t = torch.randn(shape, generator=g) * 0.5
        elif leaf.endswith("conv.b") or leaf.endswith("i.b"):
            t = torch.randn(shape, generator=g) * 0.3
        elif leaf.endswith("f.b"):
            t = 2.0 + torch.randn(shape, generator=g)
        elif leaf.endswith("correction"):
            t = torch.randn(shape, generator=g) * 0.05
        elif leaf.endswith("router"):
            t = torch.randn(shape, generator=g) * (3.0 / math.sqrt(shape[1]))
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16).to(dtype)
    return out


def routing_margins(config: Dict[str, Any], weights: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """Per position: the smallest gap, over all mixture layers, between the last chosen and the first rejected choice
    score. A position whose gap is below the compared precision may legitimately route differently."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    mult = float(config.get("residual_mult", 1.0))

    def sub(prefix):
        return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}

    x = W["embed"][torch.tensor(tokens)] * float((config.get("embedding") or {}).get("scale", 1.0))
    gaps = torch.full((len(tokens),), math.inf, dtype=F64)
    for i, lc in enumerate(config["layers"]):
        p = f"l{i}."
        x = x + mult * rms(MIXERS[lc["type"]](x, sub(p + "mix."), lc["mixer"], eps), eps) * (1.0 + W[p + "norm1"])
        f = lc.get("mlp")
        if f is None:
            continue
        if f["kind"] == "moe":
            w = sub(p + "mlp.")
            s = torch.softmax(x @ w["router"].T, -1)
            c = torch.sort(s + w["correction"], -1, descending=True).values
            k = int(f["router"]["top"])
            if k < c.shape[1]:
                gaps = torch.minimum(gaps, c[:, k - 1] - c[:, k])
        x = x + mult * rms(feed_forward(x, sub(p + "mlp."), f), eps) * (1.0 + W[p + "norm2"])
    return gaps


# layer entries of a configuration
def dense(ff: int = 40) -> Dict[str, Any]:
    return {"kind": "dense", "ff": ff}


def moe(experts: int = 4, identity: int = 2, top: int = 3, ff: int = 24, limit: float = 1.5, shared_ff: int = 16,
        shared_limit: float = 2.5) -> Dict[str, Any]:
    f: Dict[str, Any] = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
                         "router": {"experts": experts, "identity": identity, "top": top}}
    if shared_ff:
        f["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return f


def mlstm_layer(heads=2, dim=8, vdim=12, gate_cap=10.0, mlp=None) -> Dict[str, Any]:
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}, "mlp": mlp}


def mamba2_layer(heads=4, vdim=6, state=8, groups=2, conv=4, norm_groups=2, mlp=None) -> Dict[str, Any]:
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": mlp}


def parallel_layer(heads=4, kv_heads=2, dim=16, vdim=8, window=9, rot_dims=8, rot_base=100.0, scaling=(8.0, 1.0, 4.0, 40),
                   scale=0.4, inner=24, state=6, dt_rank=3, conv=3, mlp=None) -> Dict[str, Any]:
    left: Dict[str, Any] = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        left["mask"] = {"size": window}
    if rot_dims:
        left["rot"] = {"base": rot_base, "dims": rot_dims}
        if scaling:
            left["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    right = {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def make_config(layers, vocab=67, width=32, eps=1e-5, embed_scale=3.0, residual_mult=0.4) -> Dict[str, Any]:
    return {"architecture": "Kogerax", "embedding": {"scale": embed_scale}, "layers": layers, "norm": {"eps": eps},
            "residual_mult": residual_mult, "vocab": vocab, "width": width}
