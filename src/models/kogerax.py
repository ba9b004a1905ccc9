"""
Kogerax: a decoder-only LM whose layers are listed in ``config.json``. Every sublayer reads the fp32 residual stream
itself (no norm in front); its output is RMS-normed with a ``1 + w`` gain, multiplied by a constant and added. Three
mixer types, all with per-sequence recurrent state:

* ``mlstm`` — matrix-memory LSTM (:class:`MLstmMixer`): exponential input gate and sigmoid forget gate in log space
  under a running maximum, a matrix and a normaliser vector per head, per-head norm and sigmoid output gate;
* ``mamba2`` — scalar-decay state-space layer (:class:`Mamba2Mixer`): short convolution over x | B | C, one decay and
  step size per head and token, gated and normed in equal parts of the row;
* ``parallel`` — windowed rotary grouped-query attention (:class:`src.models.fekolorn.SinkAttentionMixer` with
  stretched rotary wavelengths and a weightless per-head norm after the rotation, no sink) beside a selective scan
  (:class:`SelectiveScanMixer`), each output normed over the model width with its own weight, then averaged
  (:class:`NormedPairMixer`).

Feed-forward: dense GELU-gated, or a mixture of clamped sigmoid-gated experts with softmax routing (a correction added
for the choice only), identity experts that pass their input through, renormalised output weights and a shared
expert behind a per-token sigmoid gate.

Per layer (T tokens, residual r fp32, a = its copy in the activation dtype, m = ``residual_mult``):

    y = mixer(a);  r += m * rms(y) * (1 + norm1)        post_norm_residual / pair_post_norm_residual   HIP
    y = ff(a);     r += m * rms(y) * (1 + norm2)        post_norm_residual / combine_weighted          HIP

The model plugs into :class:`src.engine.llm_engine.LLMEngine` like the other families: paged cache rows per layer
from :class:`src.models.datatar.LayerRowPool` (none for layers without attention), state slots from
:class:`src.models.fekolorn.SeqStatePool`.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, replace
from typing import Any, Dict, List, Optional, Tuple

import torch

from src.models.datatar import MIXERS, LayerRowPool
from src.models.fekolorn import SeqStatePool, SinkAttentionMixer, SinkAttnSpec
from src.ops import mix, rec, seq
from src.parallel.tp import TPContext

# the experts' gate is g * sigmoid(EXPERT_GATE_ALPHA * g)
EXPERT_GATE_ALPHA = 1.702


# ------------------------------------------------------------------------------------------ configuration
@dataclass(frozen=True)
class MLstmSpec:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @property
    def cache_width(self) -> int:
        return 0

    def state_shapes(self) -> Dict[str, Tuple[tuple, torch.dtype]]:
        f32 = torch.float32
        return {"mem": ((self.heads, self.dim, self.vdim), f32), "nrm": ((self.heads, self.dim), f32),
                "max": ((self.heads,), f32)}

    def to_config(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class Mamba2Spec:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @property
    def dim(self) -> int:
        return self.state

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def cache_width(self) -> int:
        return 0

    def state_shapes(self) -> Dict[str, Tuple[tuple, torch.dtype]]:
        f32 = torch.float32
        return {"ssd": ((self.heads, self.state, self.vdim), f32), "conv": ((self.conv - 1, self.channels), f32)}

    def to_config(self) -> Dict[str, Any]:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class SelectiveScanSpec:
    inner: int
    state: int
    dt_rank: int
    conv: int

    heads = 1

    @property
    def cache_width(self) -> int:
        return 0

    def state_shapes(self) -> Dict[str, Tuple[tuple, torch.dtype]]:
        f32 = torch.float32
        return {"ssm": ((self.inner, self.state), f32), "conv": ((self.conv - 1, self.inner), f32)}

    def to_config(self) -> Dict[str, Any]:
        return {"inner": self.inner, "state": self.state, "dt_rank": self.dt_rank, "conv": self.conv}


@dataclass(frozen=True)
class NormedPairSpec:
    left: SinkAttnSpec
    right: SelectiveScanSpec

    @property
    def heads(self) -> int:
        return self.left.heads

    @property
    def cache_width(self) -> int:
        return self.left.cache_width

    def state_shapes(self):
        return self.right.state_shapes()

    def to_config(self) -> Dict[str, Any]:
        return {"left": self.left.to_config(), "right": self.right.to_config()}


@dataclass(frozen=True)
class GatedMlpSpec:
    kind: str                  # "dense" | "moe"
    ff: int = 0                # dense
    experts: int = 0           # moe: experts with weights
    identity: int = 0          #      experts that return their input
    top: int = 0
    expert_ff: int = 0
    expert_limit: float = 0.0
    shared_ff: int = 0         # 0: no shared expert
    shared_limit: float = 0.0

    @property
    def n_route(self) -> int:
        return self.experts + self.identity

    @staticmethod
    def from_config(m: Optional[Dict[str, Any]]) -> Optional["GatedMlpSpec"]:
        if m is None:
            return None
        kind = m["kind"]
        if kind == "dense":
            return GatedMlpSpec("dense", ff=int(m["ff"]))
        if kind == "moe":
            r, shared = m["router"], m.get("shared") or {}
            f = GatedMlpSpec("moe", experts=int(r["experts"]), identity=int(r.get("identity") or 0), top=int(r["top"]),
                             expert_ff=int(m["expert"]["ff"]), expert_limit=float(m["expert"]["limit"]),
                             shared_ff=int(shared.get("ff") or 0), shared_limit=float(shared.get("limit") or 0.0))
            if not 1 <= f.top <= f.n_route:
                raise ValueError("router.top must lie in 1 .. experts + identity")
            return f
        raise ValueError(f"unknown feed-forward kind {kind!r}")

    def to_config(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        c: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.expert_ff, "limit": self.expert_limit},
                             "router": {"experts": self.experts, "identity": self.identity, "top": self.top}}
        if self.shared_ff:
            c["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return c


def _mlstm_spec(m: Dict[str, Any]) -> MLstmSpec:
    return MLstmSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim") or m["dim"]),
                     gate_cap=float(m["gate_cap"]))


def _mamba2_spec(m: Dict[str, Any]) -> Mamba2Spec:
    s = Mamba2Spec(heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]), groups=int(m.get("groups") or 1),
                   conv=int(m.get("conv") or 1), norm_groups=int(m.get("norm_groups") or 1))
    if s.heads % s.groups or s.inner % s.norm_groups:
        raise ValueError("heads must be a multiple of groups, heads * vdim of norm_groups")
    return s


def _scan_spec(m: Dict[str, Any]) -> SelectiveScanSpec:
    return SelectiveScanSpec(inner=int(m["inner"]), state=int(m["state"]), dt_rank=int(m["dt_rank"]),
                             conv=int(m.get("conv") or 1))


def _attn_spec(m: Dict[str, Any]) -> SinkAttnSpec:
    rot, mask = m.get("rot") or {}, m.get("mask") or {}
    sc = rot.get("scaling")
    return SinkAttnSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=int(m["dim"]),
                        vdim=int(m.get("vdim") or m["dim"]), scale=float(m["scale"]), window=int(mask.get("size") or 0),
                        rot_dims=int(rot.get("dims") or 0), rot_base=float(rot.get("base", 10000.0)),
                        rot_scaling=None if not sc else (float(sc["factor"]), float(sc["low"]), float(sc["high"]),
                                                         float(sc["original"])),
                        qk_norm=True, head_norm=True, norm_after_rot=True, norm_weights=False, has_sink=False)


def _pair_spec(m: Dict[str, Any]) -> NormedPairSpec:
    return NormedPairSpec(left=_attn_spec(m["left"]), right=_scan_spec(m["right"]))


@dataclass(frozen=True)
class KogLayerSpec:
    type: str
    mixer: Any
    mlp: Optional[GatedMlpSpec]


@dataclass(frozen=True)
class KogeraxArch:
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    rms_eps: float = 1e-6
    embed_scale: float = 1.0
    residual_mult: float = 1.0
    max_position: int = 1 << 20   # positions are rotated from an inverse-frequency table: no position table

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(l.mlp is not None and l.mlp.kind == "moe" for l in self.layers)

    @property
    def num_heads(self) -> int:
        return max(l.mixer.heads for l in self.layers)

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(l.mixer.cache_width for l in self.layers) * dtype_bytes

    @staticmethod
    def from_config(c: Dict[str, Any], name: str = "kogerax") -> "KogeraxArch":
        layers = []
        for i, lc in enumerate(c["layers"]):
            t = lc["type"]
            if t not in KOGERAX_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {t!r} (known: {sorted(KOGERAX_MIXERS)})")
            layers.append(KogLayerSpec(t, KOGERAX_MIXERS[t][1](lc["mixer"]), GatedMlpSpec.from_config(lc.get("mlp"))))
        return KogeraxArch(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(layers),
                           rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                           embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                           residual_mult=float(c.get("residual_mult", 1.0)))

    def to_config(self) -> Dict[str, Any]:
        return {"architecture": "Kogerax", "embedding": {"scale": self.embed_scale},
                "layers": [{"type": l.type, "mixer": l.mixer.to_config(),
                            "mlp": None if l.mlp is None else l.mlp.to_config()} for l in self.layers],
                "norm": {"eps": self.rms_eps}, "residual_mult": self.residual_mult, "vocab": self.vocab_size,
                "width": self.hidden_size}


def kogerax_arch_from_dir(path: str, **overrides) -> KogeraxArch:
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    arch = KogeraxArch.from_config(c, name=os.path.basename(os.path.normpath(path)))
    return replace(arch, **overrides) if overrides else arch


# -------------------------------------------------------------------------------------------------- mixers
def _put(dst: torch.Tensor, src: torch.Tensor) -> bool:
    dst.copy_(src.to(dst.device, dst.dtype).reshape(dst.shape))
    return True


class _Base:
    def __init__(self, device, dtype, gen, std):
        self.device, self.dtype, self._gen, self._std = torch.device(device), dtype, gen, std

    def rnd(self, *shape, scale=None, dt=None, shift=0.0):
        t = torch.empty(*shape, dtype=dt or self.dtype, device=self.device)
        if self._gen is None:
            return t.zero_()
        t.normal_(0.0, self._std if scale is None else scale, generator=self._gen)
        return t.add_(shift) if shift else t

    def finalize(self) -> None:
        """Nothing is derived from the weights."""


class MLstmMixer(_Base):
    """Weights and forward of a matrix-memory LSTM. Per head, with log gates i (capped) and f (log-sigmoid of the
    capped pre-activation) and the running maximum m (0 at the start): m_t = max(f + m_(t-1), i);
    S <- e^(f + m_(t-1) - m_t) S + e^(i - m_t) k v^T, n likewise with k alone; o = S^T q / (max(|n . q|, e^(-m_t)) + 1e-6)
    with q scaled by dim^-1/2; every head's o RMS-normed, times a weight and sigmoid(W_g a), projected. S, n and m are
    per-sequence state (``state`` dict: "mem" [slots, H, dim, vdim], "nrm" [slots, H, dim], "max" [slots, H])."""

    type_name = "mlstm"

    @staticmethod
    def spec_from_config(m: Dict[str, Any]) -> MLstmSpec:
        return _mlstm_spec(m)

    def __init__(self, spec: MLstmSpec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        super().__init__(device, dtype, gen, std)
        s = self.spec = spec
        f32 = torch.float32
        self.nqk, self.nv = s.heads * s.dim, s.heads * s.vdim
        # one projection: [q | k | v | g | i | f] rows
        self.w_in = self.rnd(2 * self.nqk + 2 * self.nv + 2 * s.heads, hidden)
        self.i_b = self.rnd(s.heads, scale=0.3, dt=f32)
        self.f_b = self.rnd(s.heads, scale=0.5, dt=f32, shift=2.0)
        self.norm = self.rnd(self.nv, scale=0.1, dt=f32, shift=1.0)
        self.o = self.rnd(hidden, self.nv)

    def tensors(self) -> List[torch.Tensor]:
        return [self.w_in, self.i_b, self.f_b, self.norm, self.o]

    def _rows(self) -> Dict[str, Tuple[int, int]]:
        n, v, H = self.nqk, self.nv, self.spec.heads
        e = 2 * n + 2 * v
        return {"q": (0, n), "k": (n, 2 * n), "v": (2 * n, 2 * n + v), "g": (2 * n + v, e), "i": (e, e + H),
                "f": (e + H, e + 2 * H)}

    def load(self, name: str, t: torch.Tensor) -> bool:
        rows = self._rows()
        if name in rows:
            return _put(self.w_in[rows[name][0]: rows[name][1]], t)
        for nm, dst in (("i.b", self.i_b), ("f.b", self.f_b), ("norm", self.norm), ("o", self.o)):
            if name == nm:
                return _put(dst, t)
        return False

    def state(self) -> Dict[str, torch.Tensor]:
        out = {k: self.w_in[a:b] for k, (a, b) in self._rows().items()}
        out.update({"i.b": self.i_b, "f.b": self.f_b, "norm": self.norm, "o": self.o})
        return out

    def forward(self, a, positions, meta, cache, eps, state=None, rag=None, **_):
        s = self.spec
        rows = self._rows()
        p = mix.linear(a, self.w_in)
        abe = rec.exp_gate_scan(p, rows["i"][0], rows["f"][0], self.i_b, self.f_b, s.gate_cap, state["max"], s.heads,
                                rag)
        o, nq = rec.gated_linear_attn(p, 0, self.nqk, 2 * self.nqk, abe, state["mem"], state["nrm"], s.heads, s.heads,
                                      s.dim, s.vdim, s.dim ** -0.5, rag)
        g = p[:, rows["g"][0]: rows["g"][1]]
        return mix.linear(rec.head_norm_gate(o, nq, abe, g, self.norm, s.heads, s.vdim, eps), self.o)


class Mamba2Mixer(_Base):
    """Weights and forward of a scalar-decay state-space layer. One projection [z | x | B | C | dt]; x, B, C through a
    causal convolution with bias and SiLU; d = softplus(dt + dt_bias); per head (in group h // (heads / groups)):
    S <- exp(-exp(A_log_h) d) S + d B x^T (S is state x vdim), y = S^T C + D_h x; y * silu(z), RMS-normed in
    ``norm_groups`` equal parts, times a weight, projected. S and the convolution's last inputs are per-sequence state
    (``state`` dict: "ssd" [slots, H, state, vdim], "conv" [slots, taps - 1, channels])."""

    type_name = "mamba2"

    @staticmethod
    def spec_from_config(m: Dict[str, Any]) -> Mamba2Spec:
        return _mamba2_spec(m)

    def __init__(self, spec: Mamba2Spec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        super().__init__(device, dtype, gen, std)
        s = self.spec = spec
        f32 = torch.float32
        I, C, H = s.inner, s.channels, s.heads
        self.w_in = self.rnd(I + C + H, hidden)
        self.conv_w = self.rnd(C, s.conv, scale=0.5, dt=f32)
        self.conv_b = self.rnd(C, scale=0.3, dt=f32)
        self.dt_bias = self.rnd(H, scale=0.5, dt=f32, shift=-1.5)
        self.A_log = self.rnd(H, scale=0.5, dt=f32)
        self.D = self.rnd(H, scale=0.2, dt=f32, shift=1.0)
        self.norm = self.rnd(I, scale=0.1, dt=f32, shift=1.0)
        self.o = self.rnd(hidden, I)
        self.conv_wt = None
        self.finalize()

    def finalize(self) -> None:
        """Derived tensors, after the weights changed: the convolution weights tap-major for 16-byte loads."""
        self.conv_wt = self.conv_w.t().contiguous()

    def tensors(self) -> List[torch.Tensor]:
        return [self.w_in, self.conv_w, self.conv_b, self.dt_bias, self.A_log, self.D, self.norm, self.o]

    def _named(self) -> Dict[str, torch.Tensor]:
        return {"in": self.w_in, "conv": self.conv_w, "conv.b": self.conv_b, "dt_bias": self.dt_bias,
                "A_log": self.A_log, "D": self.D, "norm": self.norm, "o": self.o}

    def load(self, name: str, t: torch.Tensor) -> bool:
        dst = self._named().get(name)
        return dst is not None and _put(dst, t)

    def state(self) -> Dict[str, torch.Tensor]:
        return self._named()

    def forward(self, a, positions, meta, cache, eps, state=None, rag=None, **_):
        s = self.spec
        I, C, GN = s.inner, s.channels, s.groups * s.state
        p = mix.linear(a, self.w_in)
        xbc_in = p[:, I: I + C]
        xbc, ab = rec.conv_silu(xbc_in, self.conv_w, self.conv_b, state["conv"], rag, wt=self.conv_wt,
                                dt=p[:, I + C:], dt_bias=self.dt_bias, A_log=self.A_log)
        rec.conv_tail_update(state["conv"], xbc_in, rag)
        # the output map C plays the query's part, the input map B the key's, x the value's
        o, _ = rec.gated_linear_attn(xbc, I + GN, I, 0, ab, state["ssd"], None, s.heads, s.groups, s.state, s.vdim,
                                     1.0, rag)
        y = rec.skip_gate_group_norm(o, xbc[:, :I], self.D, p[:, :I], self.norm, s.heads, s.vdim, s.norm_groups, eps)
        return mix.linear(y, self.o)


class SelectiveScanMixer(_Base):
    """Weights and forward of a selective scan. W_in a = [x | z]; x through a causal convolution with bias and SiLU;
    W_x x = [dt | B | C]; d = softplus(W_dt dt + dt.b) per channel; S[c] <- exp(d_c A[c]) S[c] + d_c x_c B,
    y_c = S[c] . C + D_c x_c with A = -exp(A_log); y * silu(z), projected. S and the convolution's last inputs are
    per-sequence state (``state`` dict: "ssm" [slots, inner, state], "conv" [slots, taps - 1, inner])."""

    type_name = "selective_scan"

    @staticmethod
    def spec_from_config(m: Dict[str, Any]) -> SelectiveScanSpec:
        return _scan_spec(m)

    def __init__(self, spec: SelectiveScanSpec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        super().__init__(device, dtype, gen, std)
        s = self.spec = spec
        f32 = torch.float32
        I, N, R = s.inner, s.state, s.dt_rank
        self.w_in = self.rnd(2 * I, hidden)
        self.conv_w = self.rnd(I, s.conv, scale=0.5, dt=f32)
        self.conv_b = self.rnd(I, scale=0.3, dt=f32)
        self.w_x = self.rnd(R + 2 * N, I)
        self.w_dt = self.rnd(I, R, scale=0.3)
        self.dt_b = self.rnd(I, scale=0.5, dt=f32, shift=-1.5)
        self.A_log = self.rnd(I, N, scale=0.5, dt=f32)
        self.D = self.rnd(I, scale=0.2, dt=f32, shift=1.0)
        self.o = self.rnd(hidden, I)
        self.conv_wt = self.A = None
        self.finalize()

    def finalize(self) -> None:
        """Derived tensors, after the weights changed: tap-major convolution weights and A = -exp(A_log)."""
        self.conv_wt = self.conv_w.t().contiguous()
        self.A = (-torch.exp(self.A_log.double())).float().contiguous()

    def tensors(self) -> List[torch.Tensor]:
        return [self.w_in, self.conv_w, self.conv_b, self.w_x, self.w_dt, self.dt_b, self.A_log, self.D, self.o]

    def in_rows(self) -> int:
        return self.w_in.shape[0]

    def _named(self) -> Dict[str, torch.Tensor]:
        return {"in": self.w_in, "conv": self.conv_w, "conv.b": self.conv_b, "x": self.w_x, "dt": self.w_dt,
                "dt.b": self.dt_b, "A_log": self.A_log, "D": self.D, "o": self.o}

    def load(self, name: str, t: torch.Tensor) -> bool:
        dst = self._named().get(name)
        return dst is not None and _put(dst, t)

    def state(self) -> Dict[str, torch.Tensor]:
        return self._named()

    def recur(self, p: torch.Tensor, eps: float, state: Dict[str, torch.Tensor], rag: seq.Ragged) -> torch.Tensor:
        """p [T, 2 * inner]: this mixer's columns of a projection output. Returns W_o of the gated scan."""
        s = self.spec
        I, N, R = s.inner, s.state, s.dt_rank
        x_in, z = p[:, :I], p[:, I: 2 * I]
        x = rec.conv_silu(x_in, self.conv_w, self.conv_b, state["conv"], rag, wt=self.conv_wt)
        rec.conv_tail_update(state["conv"], x_in, rag)
        bc = mix.linear(x, self.w_x)
        dt = mix.linear(bc[:, :R].contiguous(), self.w_dt)
        y = rec.selective_scan(x, dt, self.dt_b, bc, R, R + N, self.A, self.D, z, state["ssm"], rag)
        return mix.linear(y, self.o)

    def forward(self, a, positions, meta, cache, eps, state=None, rag=None, **_):
        return self.recur(mix.linear(a, self.w_in), eps, state, rag)


class PairOut:
    """What a pair of side-by-side mixers hands to the layer: both outputs and their norm weights; the layer's
    residual update norms and averages them in its own launch (:func:`src.ops.rec.pair_post_norm_residual`)."""

    __slots__ = ("y1", "w1", "y2", "w2")

    def __init__(self, y1, w1, y2, w2):
        self.y1, self.w1, self.y2, self.w2 = y1, w1, y2, w2


class NormedPairMixer:
    """Softmax attention and a selective scan side by side on the same input (one fused input projection); the result
    is half the sum of the two outputs, each first RMS-normed over the model width with a plain weight."""

    type_name = "normed_pair"

    @staticmethod
    def spec_from_config(m: Dict[str, Any]) -> NormedPairSpec:
        return _pair_spec(m)

    def __init__(self, spec: NormedPairSpec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        self.spec = spec
        self.left = SinkAttentionMixer(spec.left, hidden, device, dtype, gen, std)
        self.right = SelectiveScanMixer(spec.right, hidden, device, dtype, gen, std)
        f32 = torch.float32
        self.out_l = torch.ones(hidden, dtype=f32, device=device)
        self.out_r = torch.ones(hidden, dtype=f32, device=device)
        if gen is not None:
            self.out_l.add_(torch.empty_like(self.out_l).normal_(0.0, 0.1, generator=gen))
            self.out_r.add_(torch.empty_like(self.out_r).normal_(0.0, 0.1, generator=gen))
        # both input projections as one weight; the halves stay views of it, so loading writes in place
        nl = self.left.in_rows()
        self.w_in = torch.cat([self.left.qkv, self.right.w_in], 0)
        self.left.qkv, self.right.w_in = self.w_in[:nl], self.w_in[nl:]

    def finalize(self) -> None:
        self.left.finalize()
        self.right.finalize()

    def tensors(self) -> List[torch.Tensor]:
        return [self.w_in] + self.left.tensors()[1:] + self.right.tensors()[1:]

    def load(self, name: str, t: torch.Tensor) -> bool:
        if name == "left.out":
            return _put(self.out_l, t)
        if name == "right.out":
            return _put(self.out_r, t)
        if name.startswith("left."):
            return self.left.load(name[5:], t)
        if name.startswith("right."):
            return self.right.load(name[6:], t)
        return False

    def state(self) -> Dict[str, torch.Tensor]:
        out = {"left." + k: v for k, v in self.left.state().items()}
        out.update({"right." + k: v for k, v in self.right.state().items()})
        out["left.out"], out["right.out"] = self.out_l, self.out_r
        return out

    def forward(self, a, positions, meta, cache, eps, state=None, rag=None, shared=None, **_):
        p = mix.linear(a, self.w_in)
        nl = self.left.in_rows()
        yl = self.left.attend(p[:, :nl], positions, meta, cache, eps, shared if shared is not None else {})
        yr = self.right.recur(p[:, nl:], eps, state, rag)
        return PairOut(yl, self.out_l, yr, self.out_r)


for _m in (MLstmMixer, Mamba2Mixer, SelectiveScanMixer, NormedPairMixer):
    MIXERS[_m.type_name] = _m

# this family's reading of the layer types: (mixer class, spec from the layer's "mixer" entry)
KOGERAX_MIXERS = {
    "mlstm": (MLstmMixer, _mlstm_spec),
    "mamba2": (Mamba2Mixer, _mamba2_spec),
    "parallel": (NormedPairMixer, _pair_spec),
}


class KogLayerWeights:
    __slots__ = ("norm1", "norm2", "mix", "gate_up", "down", "router", "correction", "w13", "w2", "shared_gate_up",
                 "shared_down")

    def __init__(self):
        for s in self.__slots__:
            setattr(self, s, None)


class KogeraxLM:
    """The model behind :class:`src.engine.llm_engine.LLMEngine` for ``architecture: Kogerax`` checkpoints (same
    interface as the other families: forward / compute_logits / load_state_dict, plus ``make_seq_state``)."""

    needs_decode_partials = False
    graph_capturable = True

    def __init__(self, arch: KogeraxArch, device, dtype=torch.bfloat16, tp: Optional[TPContext] = None, seed: int = 0,
                 init_std: float = 0.05, max_position: Optional[int] = None, random_init: bool = True, **_):
        if tp is not None and tp.enabled:
            raise ValueError("Kogerax runs on one GPU (no tensor-parallel layout is defined for its mixers)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Kogerax runs in bfloat16 or float32")
        self.arch, self.device, self.dtype = arch, torch.device(device), dtype
        self.tp = tp or TPContext()
        self.hq, self.hkv = arch.num_heads, 1
        self.max_position = max_position or arch.max_position
        # the engine gives every live sequence a state slot when a layer keeps recurrent state; a cached prefix holds
        # keys and values but not the state after it
        self.needs_seq_state = any(l.mixer.state_shapes() for l in arch.layers)
        self.supports_prefix_cache = not self.needs_seq_state
        gen = None
        if random_init:
            gen = torch.Generator(device=self.device)
            gen.manual_seed(seed)
        h = arch.hidden_size

        def rnd(*shape, scale=init_std, dt=dtype):
            t = torch.empty(*shape, dtype=dt, device=self.device)
            return t.normal_(0.0, scale, generator=gen) if gen is not None else t.zero_()

        self.embed = rnd(arch.vocab_size, h, scale=1.0)
        self.layers: List[KogLayerWeights] = []
        for spec in arch.layers:
            lw = KogLayerWeights()
            lw.norm1 = rnd(h, scale=0.1)
            lw.mix = KOGERAX_MIXERS[spec.type][0](spec.mixer, h, self.device, dtype, gen, init_std)
            f = spec.mlp
            if f is not None:
                lw.norm2 = rnd(h, scale=0.1)
                if f.kind == "dense":
                    lw.gate_up = rnd(2 * f.ff, h)
                    lw.down = rnd(h, f.ff)
                else:
                    # the shared expert's gate row rides below the router's rows: one product gives both
                    lw.router = rnd(f.n_route + (1 if f.shared_ff else 0), h, scale=init_std * 4)
                    lw.correction = torch.zeros(f.n_route, dtype=torch.float32, device=self.device)
                    lw.w13 = rnd(f.experts, 2 * f.expert_ff, h)
                    lw.w2 = rnd(f.experts, h, f.expert_ff)
                    if f.shared_ff:
                        lw.shared_gate_up = rnd(2 * f.shared_ff, h)
                        lw.shared_down = rnd(h, f.shared_ff)
            self.layers.append(lw)
        self.norm = rnd(h, scale=0.1)
        self.lm_head = rnd(arch.vocab_size, h)
        self.seq_state: Optional[SeqStatePool] = None

    # ------------------------------------------------------------------ weights
    def load_state_dict(self, tensors: Dict[str, torch.Tensor], fold: bool = True) -> int:
        """Tensors under the checkpoint's names: ``embed``, ``head``, ``final.norm`` and, for layer i,
        ``l<i>.norm1|norm2``, ``l<i>.mix.<name>`` (the mixer's own), ``l<i>.mlp.gate|up|down`` (dense) or
        ``l<i>.mlp.router|correction``, ``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.mlp.shared.gate|up|down|sg`` (moe)."""
        n = 0
        top = {"embed": self.embed, "head": self.lm_head, "final.norm": self.norm}
        for name, t in tensors.items():
            if name in top:
                n += _put(top[name], t)
                continue
            if not (name.startswith("l") and "." in name and name[1:name.index(".")].isdigit()):
                continue
            li, rest = int(name[1:name.index(".")]), name[name.index(".") + 1:]
            if li >= len(self.layers):
                continue
            lw, f = self.layers[li], self.arch.layers[li].mlp
            if rest == "norm1":
                n += _put(lw.norm1, t)
            elif rest == "norm2" and lw.norm2 is not None:
                n += _put(lw.norm2, t)
            elif rest.startswith("mix."):
                n += bool(lw.mix.load(rest[4:], t))
            elif rest.startswith("mlp.") and f is not None:
                parts = rest.split(".")[1:]
                if f.kind == "dense" and len(parts) == 1:
                    dst = {"gate": lw.gate_up[: f.ff], "up": lw.gate_up[f.ff:], "down": lw.down}.get(parts[0])
                    if dst is not None:
                        n += _put(dst, t)
                elif f.kind == "moe":
                    if parts == ["router"]:
                        n += _put(lw.router[: f.n_route], t)
                    elif parts == ["correction"]:
                        n += _put(lw.correction, t)
                    elif len(parts) == 2 and parts[0] == "shared" and lw.shared_gate_up is not None:
                        dst = {"gate": lw.shared_gate_up[: f.shared_ff], "up": lw.shared_gate_up[f.shared_ff:],
                               "down": lw.shared_down, "sg": lw.router[f.n_route:]}.get(parts[1])
                        if dst is not None:
                            n += _put(dst, t)
                    elif len(parts) == 2 and parts[0][0] == "e" and parts[0][1:].isdigit():
                        e = int(parts[0][1:])
                        if e < f.experts:
                            dst = {"gate": lw.w13[e, : f.expert_ff], "up": lw.w13[e, f.expert_ff:],
                                   "down": lw.w2[e]}.get(parts[1])
                            if dst is not None:
                                n += _put(dst, t)
        if fold:
            self.fold_norm_weights()
        return n

    def fold_norm_weights(self, layers=None) -> None:
        """Called once the weights are in: tensors derived from them (tap-major convolutions, A = -exp(A_log))."""
        for lw in self.layers:
            lw.mix.finalize()

    def state_dict(self) -> Dict[str, torch.Tensor]:
        out = {"embed": self.embed, "head": self.lm_head, "final.norm": self.norm}
        for i, (lw, spec) in enumerate(zip(self.layers, self.arch.layers)):
            p = f"l{i}."
            out[p + "norm1"] = lw.norm1
            for k, v in lw.mix.state().items():
                out[p + "mix." + k] = v
            f = spec.mlp
            if f is None:
                continue
            out[p + "norm2"] = lw.norm2
            q = p + "mlp."
            if f.kind == "dense":
                out[q + "gate"], out[q + "up"], out[q + "down"] = lw.gate_up[: f.ff], lw.gate_up[f.ff:], lw.down
                continue
            out[q + "router"], out[q + "correction"] = lw.router[: f.n_route], lw.correction
            for e in range(f.experts):
                out[q + f"e{e}.gate"], out[q + f"e{e}.up"] = lw.w13[e, : f.expert_ff], lw.w13[e, f.expert_ff:]
                out[q + f"e{e}.down"] = lw.w2[e]
            if f.shared_ff:
                out[q + "shared.gate"], out[q + "shared.up"] = lw.shared_gate_up[: f.shared_ff], lw.shared_gate_up[f.shared_ff:]
                out[q + "shared.down"], out[q + "shared.sg"] = lw.shared_down, lw.router[f.n_route:]
        return out

    def save(self, path: str) -> None:
        """``config.json`` + ``model.safetensors`` under the checkpoint names (tests, tooling)."""
        from safetensors.torch import save_file

        os.makedirs(path, exist_ok=True)
        with open(os.path.join(path, "config.json"), "w") as f:
            json.dump(self.arch.to_config(), f, indent=1)
        save_file({k: v.detach().to("cpu").contiguous() for k, v in self.state_dict().items()},
                  os.path.join(path, "model.safetensors"))

    def weight_bytes(self) -> int:
        tot = sum(t.numel() * t.element_size() for t in (self.embed, self.lm_head, self.norm))
        for lw in self.layers:
            tot += sum(t.numel() * t.element_size() for t in lw.mix.tensors())
            for s in KogLayerWeights.__slots__:
                t = getattr(lw, s)
                if isinstance(t, torch.Tensor):
                    tot += t.numel() * t.element_size()
        return tot

    # ------------------------------------------------------------ cache + state
    def kv_bytes_per_block(self, block_size: int) -> int:
        return max(1, self.arch.kv_bytes_per_token(self.embed.element_size())) * block_size

    def make_kv_pool(self, num_blocks: int, block_size: int) -> LayerRowPool:
        """One row per token and layer with attention; the recurrent layers cache nothing (width 0)."""
        return LayerRowPool([l.mixer.cache_width for l in self.arch.layers], num_blocks, block_size, self.device,
                            self.dtype)

    def make_seq_state(self, num_slots: int) -> SeqStatePool:
        self.seq_state = SeqStatePool([l.mixer.state_shapes() for l in self.arch.layers], num_slots, self.device)
        return self.seq_state

    def activation_bytes(self, tokens: int) -> int:
        a = self.arch
        widest = 0
        for l, lw in zip(a.layers, self.layers):
            w = 4 * lw.mix.w_in.shape[0]
            f = l.mlp
            if f is not None:
                w = max(w, 3 * f.ff if f.kind == "dense" else 4 * f.top * (a.hidden_size + f.expert_ff) + 3 * f.shared_ff)
            widest = max(widest, w)
        return tokens * (10 * a.hidden_size + 4 * widest) + (1 << 30)

    # ----------------------------------------------------------------- forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, meta, kv_pool,
                layer_hook=None) -> torch.Tensor:
        """Final-norm hidden states [T, W] in the model dtype. ``kv_pool``: one cache tensor per layer.
        ``meta.state_slots``: the state slot of every sequence of the step. ``layer_hook(i, residual)``: called after
        each layer with the fp32 residual."""
        a, eps, m = self.arch, self.arch.rms_eps, self.arch.residual_mult
        st_layers = rag = None
        if self.needs_seq_state:
            if self.seq_state is None or getattr(meta, "state_slots", None) is None:
                raise RuntimeError("Kogerax's recurrent layers need per-sequence state slots (LLMEngine provides them)")
            st_layers = self.seq_state.layers
            rag = seq.Ragged(positions, meta.cu_q if meta.is_prefill else None, meta.state_slots)
        resid, act = rec.embed_scaled(input_ids, self.embed, a.embed_scale)
        act_out = None if act is resid else act
        shared: Dict[str, Any] = {}
        for li, lw in enumerate(self.layers):
            y = lw.mix.forward(act, positions, meta, kv_pool[li], eps,
                               state=None if st_layers is None else st_layers[li], rag=rag, shared=shared)
            if isinstance(y, PairOut):
                rec.pair_post_norm_residual(resid, act_out, y.y1, y.w1, y.y2, y.w2, lw.norm1, m, eps)
            else:
                mix.post_norm_residual(resid, y, lw.norm1, eps, True, act=act_out, mult=m)
            if meta.kv_hook is not None:
                meta.kv_hook(li)
            f = a.layers[li].mlp
            if f is not None:
                y = self._mlp(lw, f, act, post_norm=(resid, lw.norm2, eps, True, act_out, m))
                if y is not None:
                    mix.post_norm_residual(resid, y, lw.norm2, eps, True, act=act_out, mult=m)
            if layer_hook is not None:
                layer_hook(li, resid)
        return mix.rms_norm_ext(resid, self.norm, eps, True, out_dtype=self.dtype)

    def _mlp(self, lw: KogLayerWeights, f: GatedMlpSpec, a: torch.Tensor, post_norm=None) -> Optional[torch.Tensor]:
        """The feed-forward's output, or None when it was already added into the residual (``post_norm``: the MoE's
        weighted expert sum and its post-norm are one launch)."""
        if f.kind == "dense":
            return mix.linear(mix.gated_act(mix.linear(a, lw.gate_up), mix.ACT_GELU_TANH), lw.down)
        w, ids, gate = mix.route_softmax_topk(a, lw.router, f.top, f.n_route, lw.correction,
                                              gate_row=lw.shared_gate_up is not None)
        shared = None
        if lw.shared_gate_up is not None:
            shared = mix.linear(mix.gated_act(mix.linear(a, lw.shared_gate_up), mix.ACT_CLAMPED, f.shared_limit,
                                              EXPERT_GATE_ALPHA), lw.shared_down)
        return mix.moe_output_weighted(a, lw.w13, lw.w2, w, ids, mix.ACT_CLAMPED, f.expert_limit, EXPERT_GATE_ALPHA,
                                       n_route=f.n_route, extra=shared, extra_gate=gate, post_norm=post_norm)

    def compute_logits(self, hidden: torch.Tensor, argmax_parts=None) -> torch.Tensor:
        """fp32 logits [rows, vocab] = head(hidden)."""
        if argmax_parts is not None:
            raise ValueError("this head writes no per-tile argmax candidates")
        return mix.linear(hidden, self.lm_head).float()
