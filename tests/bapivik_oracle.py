"""
A plain, slow implementation of the Bapivik design in float64, written from its equations: dense masks, explicit
loops over time, no cache, no batching, one function per mechanism. It shares no code with ``src/`` and is what
``tests/test_bapivik.py`` compares the engine with. It also makes the tests' configurations and random weights.

Notation: ``h`` [T, W] is a sublayer's input, weights are stored [out, in] and applied as ``h @ W.T``; positions count
from 0; rms(x) = x / sqrt(mean(x^2) + eps).
"""

from __future__ import annotations

import math
from typing import Any, Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(x):
    return x / (1.0 + torch.exp(-x))


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def softcap(x, cap: float):
    return cap * torch.tanh(x / cap) if cap else x


def embedding(tok: List[int], embed: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
    """Token vector plus the learned vector of its position."""
    return embed[torch.tensor(tok)] + pos[: len(tok)]


def lightning(h, w: Dict[str, torch.Tensor], m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Linear attention with a fixed decay per head: S_t = d S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, from a zero state;
    all heads normed together, gated by sigmoid(W_g h), projected."""
    T, H, D, V = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).view(T, H, D)
    k = silu(h @ w["k"].T).view(T, H, D)
    v = silu(h @ w["v"].T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, V, dtype=F64)
        for t in range(T):
            S = m["decay"][hd] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    y = rms(o.reshape(T, H * V), w["norm"], eps) * sigmoid(h @ w["g"].T)
    return y @ w["o"].T


def latent(h: torch.Tensor, w: Dict[str, torch.Tensor], eps: float) -> torch.Tensor:
    """The normed low-rank key/value latent of every token."""
    return rms(h @ w["dkv"].T, w["dkv.norm"], eps)


def latent_attention(h, c, w: Dict[str, torch.Tensor], m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Causal softmax attention whose keys and values are expanded per head from the latent ``c`` (this layer's or
    another's); queries through a normed latent of their own; one output gate per head."""
    T, H, D, V = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = (rms(h @ w["dq"].T, w["dq.norm"], eps) @ w["uq"].T).view(T, H, D)
    k = (c @ w["uk"].T).view(T, H, D)
    v = (c @ w["uv"].T).view(T, H, V)
    g = sigmoid(h @ w["g"].T)                                     # [T, H]
    out = torch.zeros(T, H, V, dtype=F64)
    for i in range(T):
        for hd in range(H):
            s = (k[: i + 1, hd] @ q[i, hd]) * m["scale"]
            p = torch.softmax(s, 0)
            out[i, hd] = (p[:, None] * v[: i + 1, hd]).sum(0) * g[i, hd]
    return out.reshape(T, H * V) @ w["o"].T


def query_temperature(p: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log((p + 1) // every + 1)


def window_attention(h, w: Dict[str, torch.Tensor], m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Grouped-query softmax attention without rotation: the values are the un-normed keys; q and k normed per head;
    a query temperature that grows with the position; capped scores; a linear distance penalty per head; a window."""
    T, H, G, D = h.shape[0], m["heads"], m.get("kv_heads") or m["heads"], m["dim"]
    q = rms((h @ w["q"].T).view(T, H, D), w["q.norm"], eps)
    kraw = (h @ w["k"].T).view(T, G, D)
    k = rms(kraw, w["k.norm"], eps)
    qt = m.get("q_temp")
    win = (m.get("mask") or {}).get("size") or 0
    cap = m.get("softcap") or 0.0
    out = torch.zeros(T, H, D, dtype=F64)
    for i in range(T):
        lo = max(0, i - win + 1) if win else 0
        dist = torch.arange(i - lo, -1, -1, dtype=F64)            # i - j for j = lo .. i
        for hd in range(H):
            g = hd // (H // G)
            qq = q[i, hd] * (query_temperature(i, qt["coef"], qt["every"]) if qt else 1.0)
            s = softcap((k[lo: i + 1, g] @ qq) * m["scale"], cap) - 2.0 ** (-8.0 * (hd + 1) / H) * dist
            p = torch.softmax(s, 0)
            out[i, hd] = (p[:, None] * kraw[lo: i + 1, g]).sum(0)
    return out.reshape(T, H * D) @ w["o"].T


def feed_forward(h, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    z = torch.relu(h @ w["up"].T + w["up.b"])
    return (z * z) @ w["down"].T + w["down.b"]


def forward(config: Dict[str, Any], weights: Dict[str, torch.Tensor], tokens: List[int], keep_layers: bool = False):
    """Logits [T, vocab] of one sequence (float64); with ``keep_layers`` also the stream after every layer."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])

    def sub(prefix):
        return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}

    x = embedding(tokens, W["embed"], W["pos"])
    results = [x]                                                 # X_0 and every layer's own result
    latents: Dict[int, torch.Tensor] = {}
    streams = []
    for i, lc in enumerate(config["layers"]):
        p, m, mw = f"l{i}.", lc["mixer"], sub(f"l{i}.mix.")
        h = rms(x, W[p + "norm1"], eps)
        if lc["type"] == "lightning":
            y = lightning(h, mw, m, eps)
        elif lc["type"] == "latent_attention":
            if "kv_from" in m and m["kv_from"] is not None:
                c = latents[int(m["kv_from"])]
            else:
                c = latents[i] = latent(h, mw, eps)
            y = latent_attention(h, c, mw, m, eps)
        elif lc["type"] == "attention":
            y = window_attention(h, mw, m, eps)
        else:
            raise ValueError(lc["type"])
        x = x + rms(y, W[p + "norm1b"], eps)
        if lc.get("mlp") is not None:
            x = x + rms(feed_forward(rms(x, W[p + "norm2"], eps), sub(p + "mlp.")), W[p + "norm2b"], eps)
        results.append(x)
        a = W[p + "dwa"]
        x = sum(a[j] * results[j] for j in range(i + 2))
        streams.append(x)
    logits = softcap(rms(x, W["final.norm"], eps) @ W["embed"].T, float(config.get("logit_softcap") or 0.0))
    return (logits, torch.stack(streams)) if keep_layers else logits


# --------------------------------------------------------------------------------------- configurations, weights
def attn_layer(heads=4, kv_heads=2, dim=16, window=0, softcap=0.0, q_temp=None, scale=None, ff=48):
    m: Dict[str, Any] = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                         "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if softcap:
        m["softcap"] = softcap
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent_layer(heads=4, dim=16, vdim=24, kv_rank=32, q_rank=24, kv_from=None, scale=None, ff=48):
    m: Dict[str, Any] = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                         "scale": scale if scale is not None else dim ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def lightning_layer(heads=3, dim=16, vdim=16, decay=None, ff=0):
    decay = decay or [math.exp(-2.0 ** -(1 + 1.5 * i)) for i in range(heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers, vocab=96, width=48, max_positions=512, eps=1e-5, logit_softcap=20.0):
    return {"architecture": "Bapivik", "layers": layers, "logit_softcap": logit_softcap,
            "max_positions": max_positions, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def tensor_shapes(config) -> Dict[str, tuple]:
    Wd = config["width"]
    out: Dict[str, tuple] = {"embed": (config["vocab"], Wd), "pos": (config["max_positions"], Wd),
                             "final.norm": (Wd,)}
    for i, lc in enumerate(config["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (Wd,)
        out[p + "dwa"] = (i + 2,)
        if lc["type"] == "lightning":
            n, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out.update({p + "mix.q": (n, Wd), p + "mix.k": (n, Wd), p + "mix.v": (nv, Wd), p + "mix.g": (nv, Wd),
                        p + "mix.o": (Wd, nv), p + "mix.norm": (nv,)})
        elif lc["type"] == "latent_attention":
            H = m["heads"]
            out.update({p + "mix.dq": (m["q_rank"], Wd), p + "mix.dq.norm": (m["q_rank"],),
                        p + "mix.uq": (H * m["dim"], m["q_rank"]), p + "mix.uk": (H * m["dim"], m["kv_rank"]),
                        p + "mix.uv": (H * m["vdim"], m["kv_rank"]), p + "mix.g": (H, Wd),
                        p + "mix.o": (Wd, H * m["vdim"])})
            if m.get("kv_from") is None:
                out.update({p + "mix.dkv": (m["kv_rank"], Wd), p + "mix.dkv.norm": (m["kv_rank"],)})
        else:
            H, G, D = m["heads"], m.get("kv_heads") or m["heads"], m["dim"]
            out.update({p + "mix.q": (H * D, Wd), p + "mix.k": (G * D, Wd), p + "mix.q.norm": (D,),
                        p + "mix.k.norm": (D,), p + "mix.o": (Wd, H * D)})
        if lc.get("mlp") is not None:
            ff = lc["mlp"]["ff"]
            out[p + "norm2"] = out[p + "norm2b"] = (Wd,)
            out.update({p + "mlp.up": (ff, Wd), p + "mlp.up.b": (ff,), p + "mlp.down": (Wd, ff),
                        p + "mlp.down.b": (Wd,)})
    return out


def random_weights(config, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's names, rounded to ``dtype`` (so that every precision starts from the
    same numbers). Matrices ~ N(0, 1/in); norms near one; the depth weights near an average with a dominant last."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        if name.endswith("dwa"):
            t = torch.full(shape, 0.3 / max(1, shape[0] - 1)) + 0.05 * torch.randn(shape, generator=g)
            t[-1] = 0.7 + 0.05 * float(torch.randn((), generator=g))
        elif "norm" in name:
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif name in ("embed", "pos"):
            t = torch.randn(shape, generator=g) * (1.0 if name == "embed" else 0.5)
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(dtype)
    return out
