"""
Fekolorn: a decoder-only LM whose layers are listed in ``config.json``, with several fp32 residual streams
(hyper-connections), scalar-gain pre-norms, a hashed bigram embedding, and two mixer types:

* ``attention`` — grouped-query attention without rotation: q and k RMS-normed over the whole projection, a learned
  bias per (distance bucket, head), a sliding window, a softmax sink, values blended with those of the first such
  layer (:class:`SinkAttentionMixer`);
* ``parallel`` — two mixers reading the same input, summed with fixed scales: rotary grouped-query attention with
  unit-RMS values and a sink (the same class, other switches), beside a gated delta rule with short convolutions
  (:class:`GatedDeltaMixer`), whose matrix state and convolution tail live in per-sequence state slots.

Feed-forward: ``W_down polynorm(W_up h)``. Per layer (T tokens, streams x_1 .. x_S fp32):

    h = rmsnorm(in1 . x) * g1            stream_mix_norm   HIP (fused with the previous sublayer's stream update)
    y = mixer(h)                         GEMMs + qkv_prep / sink_attn / delta_prep / gated_delta   HIP
    x_t <- mix1[:, t] . x + out1[t] y;   h = rmsnorm(in2 . x) * g2        stream_mix_norm   HIP, one launch
    y = W_down polynorm(W_up h)          GEMM + poly_norm_act HIP + GEMM
    x_t <- mix2[:, t] . x + out2[t] y;   h = the next layer's input (or the final norm of sum_t x_t)

The mixers register in :data:`src.models.datatar.MIXERS` beside the latent attention, with the same interface, and
the model plugs into :class:`src.engine.llm_engine.LLMEngine` like the other families (paged cache rows per layer
from :class:`src.models.datatar.LayerRowPool`, state slots from :class:`SeqStatePool`).
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, replace
from typing import Any, Dict, List, Optional, Tuple

import torch

from src.models.datatar import MIXERS, LayerRowPool
from src.ops import mix, seq
from src.parallel.tp import TPContext


# ------------------------------------------------------------------------------------------ configuration
@dataclass(frozen=True)
class SinkAttnSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0            # 0: every earlier position
    rot_dims: int = 0          # rotate-half rotary on the first rot_dims dims of each head (0: none)
    rot_base: float = 10000.0
    qk_norm: bool = False      # RMS norm of q and of k over the whole projection, plain weights
    v_unit: bool = False       # every value head divided by its root mean square
    v_mix: bool = False        # values blended with the first such layer's
    bias_max: float = 0.0      # > 0: learned bias per (distance bucket, head); the last bucket starts here
    has_sink: bool = True      # a per-head term exp(sink_h) in the softmax denominator
    head_norm: bool = False    # with qk_norm: every head normed by itself, weights [dim] shared by the heads
    v_from_k: bool = False     # no value projection: the values are the keys as projected, before their norm
    softcap: float = 0.0       # > 0: scaled scores pass through softcap * tanh(s / softcap)
    slope_exp: float = 0.0     # > 0: head h's score drops by 2^(-slope_exp (h + 1) / heads) per position of distance
    q_temp_coef: float = 0.0   # != 0: q times 1 + coef * ln(floor((p + 1) / q_temp_every) + 1) at position p
    q_temp_every: int = 1
    rot_scaling: Optional[Tuple[float, float, float, float]] = None   # (factor, low, high, original): long
    #                            wavelengths of the rotary frequencies stretched (src.ops.mix.rope_inv_freq)
    norm_after_rot: bool = False   # with head_norm: the per-head norm follows the rotation instead of preceding it
    norm_weights: bool = True      # False: the q / k norms have no weights (and the checkpoint no such tensors)

    @property
    def cache_width(self) -> int:
        return self.kv_heads * (self.dim + self.vdim)

    def state_shapes(self) -> Dict[str, Tuple[tuple, torch.dtype]]:
        return {}

    def to_config(self) -> Dict[str, Any]:
        c: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale}
        if self.window:
            c["mask"] = {"size": self.window}
        if self.rot_dims:
            c["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                c["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), self.rot_scaling))
        if self.bias_max:
            c["bias_max"] = self.bias_max
        if self.v_mix:
            c["v_mix"] = True
        return c


@dataclass(frozen=True)
class GatedDeltaSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                  # taps of the short convolution

    @property
    def cache_width(self) -> int:
        return 0

    @property
    def channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    def state_shapes(self) -> Dict[str, Tuple[tuple, torch.dtype]]:
        return {"delta": ((self.heads, self.dim, self.vdim), torch.float32),
                "conv": ((self.conv - 1, self.channels), torch.float32)}

    def to_config(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class ParallelSpec:
    left: SinkAttnSpec
    right: GatedDeltaSpec
    left_scale: float
    right_scale: float

    @property
    def heads(self) -> int:
        return max(self.left.heads, self.right.heads)

    @property
    def cache_width(self) -> int:
        return self.left.cache_width

    def state_shapes(self):
        return self.right.state_shapes()

    def to_config(self) -> Dict[str, Any]:
        return {"left": self.left.to_config(), "right": self.right.to_config(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class PolyMlpSpec:
    ff: int
    kind: str = "dense"

    @staticmethod
    def from_config(m: Optional[Dict[str, Any]]) -> Optional["PolyMlpSpec"]:
        if m is None:
            return None
        if m.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {m.get('kind')!r}")
        return PolyMlpSpec(ff=int(m["ff"]))


@dataclass(frozen=True)
class FekLayerSpec:
    type: str
    mixer: Any
    mlp: Optional[PolyMlpSpec]


@dataclass(frozen=True)
class FekolornArch:
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    streams: int = 0               # 0: one residual stream, no hyper-connection tensors
    rms_eps: float = 1e-6
    embed_scale: float = 1.0
    bigram_buckets: int = 0        # 0: no bigram embedding
    bigram_mul_prev: int = 0
    bigram_mul_cur: int = 0
    max_position: int = 1 << 20

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return False

    @property
    def num_heads(self) -> int:
        return max(l.mixer.heads for l in self.layers)

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(l.mixer.cache_width for l in self.layers) * dtype_bytes

    @staticmethod
    def from_config(c: Dict[str, Any], name: str = "fekolorn") -> "FekolornArch":
        layers = []
        for i, lc in enumerate(c["layers"]):
            t = lc["type"]
            if t not in MIXERS or not hasattr(MIXERS[t], "forward_streams"):
                raise ValueError(f"layer {i}: unknown mixer type {t!r}")
            layers.append(FekLayerSpec(t, MIXERS[t].spec_from_config(lc["mixer"]),
                                       PolyMlpSpec.from_config(lc.get("mlp"))))
        e = c.get("embedding") or {}
        bg = e.get("bigram") or {}
        return FekolornArch(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(layers),
                            streams=int(c.get("streams") or 0), rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                            embed_scale=float(e.get("scale", 1.0)), bigram_buckets=int(bg.get("buckets") or 0),
                            bigram_mul_prev=int(bg.get("mul_prev") or 0), bigram_mul_cur=int(bg.get("mul_cur") or 0))

    def to_config(self) -> Dict[str, Any]:
        emb: Dict[str, Any] = {"scale": self.embed_scale}
        if self.bigram_buckets:
            emb["bigram"] = {"buckets": self.bigram_buckets, "mul_prev": self.bigram_mul_prev,
                             "mul_cur": self.bigram_mul_cur}
        c = {"architecture": "Fekolorn", "embedding": emb, "norm": {"eps": self.rms_eps}, "vocab": self.vocab_size,
             "width": self.hidden_size,
             "layers": [{"type": l.type, "mixer": l.mixer.to_config(),
                         "mlp": None if l.mlp is None else {"kind": l.mlp.kind, "ff": l.mlp.ff}} for l in self.layers]}
        if self.streams:
            c["streams"] = self.streams
        return c


def fekolorn_arch_from_dir(path: str, **overrides) -> FekolornArch:
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    arch = FekolornArch.from_config(c, name=os.path.basename(os.path.normpath(path)))
    return replace(arch, **overrides) if overrides else arch


# -------------------------------------------------------------------------------------------------- mixers
def _put(dst: torch.Tensor, src: torch.Tensor) -> bool:
    dst.copy_(src.to(dst.device, dst.dtype).reshape(dst.shape))
    return True


class SinkAttentionMixer:
    """Weights and forward of grouped-query attention with a softmax sink over the paged cache; the switches of
    :class:`SinkAttnSpec` select rotary positions, q/k norms, value norm or mixing, window and distance bias."""

    type_name = "attention"

    @staticmethod
    def spec_from_config(m: Dict[str, Any], as_left: bool = False) -> SinkAttnSpec:
        rot = m.get("rot") or {}
        mask = m.get("mask") or {}
        common = dict(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=int(m["dim"]),
                      vdim=int(m.get("vdim") or m["dim"]), scale=float(m["scale"]), window=int(mask.get("size") or 0))
        if as_left:   # rotary, unit-RMS values
            return SinkAttnSpec(**common, rot_dims=int(rot.get("dims") or 0), rot_base=float(rot.get("base", 10000.0)),
                                v_unit=True)
        return SinkAttnSpec(**common, qk_norm=True, v_mix=bool(m.get("v_mix")), bias_max=float(m.get("bias_max") or 0))

    def __init__(self, spec: SinkAttnSpec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        s = self.spec = spec
        self.device, self.dtype = torch.device(device), dtype
        if s.heads % s.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if s.rot_dims % 2 or s.rot_dims > s.dim:
            raise ValueError("rot.dims must be even and at most dim")

        def rnd(*shape, scale=std, dt=dtype):
            t = torch.empty(*shape, dtype=dt, device=self.device)
            return t.normal_(0.0, scale, generator=gen) if gen is not None else t.zero_()

        if s.v_from_k and (s.vdim != s.dim or s.v_mix):
            raise ValueError("values taken from the keys: vdim must equal dim, and there is no value mixing")
        if s.head_norm and not s.qk_norm:
            raise ValueError("head_norm is a form of qk_norm")
        self.nq, self.nk = s.heads * s.dim, s.kv_heads * s.dim
        self.nv = 0 if s.v_from_k else s.kv_heads * s.vdim
        self.qkv = rnd(self.nq + self.nk + self.nv, hidden)
        self.o = rnd(hidden, s.heads * s.vdim)
        f32 = torch.float32
        self.sink = rnd(s.heads, scale=0.5, dt=f32) if s.has_sink else None
        if s.norm_after_rot and not s.head_norm:
            raise ValueError("norm_after_rot is a form of head_norm")
        nscale = 0.1 if s.norm_weights else 0.0   # weightless norms: ones that no checkpoint tensor replaces
        self.q_norm = (1.0 + rnd(s.dim if s.head_norm else self.nq, scale=nscale, dt=f32)) if s.qk_norm else None
        self.k_norm = (1.0 + rnd(s.dim if s.head_norm else self.nk, scale=nscale, dt=f32)) if s.qk_norm else None
        if s.qk_norm and not s.norm_weights:
            self.q_norm.fill_(1.0)
            self.k_norm.fill_(1.0)
        # the distance penalty per head, rounded once from float64
        self.slopes = None
        if s.slope_exp:
            hs = torch.arange(1, s.heads + 1, dtype=torch.float64)
            self.slopes = torch.pow(2.0, -float(s.slope_exp) * hs / s.heads).float().to(self.device)
        self.vmix = (0.3 + rnd(1, scale=0.05, dt=f32)) if s.v_mix else None
        # buckets of the distance bias: a checkpoint's tensor decides (load); a random model takes up to 32, half
        # of them below bias_max
        self.rel_rows = max(2, min(32, 2 * (math.ceil(s.bias_max) - 1)))
        self.rel = rnd(self.rel_rows, s.heads, scale=0.5, dt=f32) if s.bias_max else None
        self.bias = None
        self.inv_freq = mix.rope_inv_freq(s.rot_base, s.rot_dims, self.device, s.rot_scaling) if s.rot_dims else None
        self.finalize()

    def finalize(self) -> None:
        """Derived tensors, after the weights changed: the bias per distance from the bias per bucket."""
        if self.rel is not None:
            self.bias = seq.distance_bias_table(self.rel, self.spec.bias_max, self.spec.window)

    def tensors(self) -> List[torch.Tensor]:
        return [t for t in (self.qkv, self.o, self.sink, self.q_norm, self.k_norm, self.vmix, self.rel) if t is not None]

    def in_rows(self) -> int:
        return self.qkv.shape[0]

    def load(self, name: str, t: torch.Tensor) -> bool:
        if name == "q":
            return _put(self.qkv[: self.nq], t)
        if name == "k":
            return _put(self.qkv[self.nq: self.nq + self.nk], t)
        if name == "v" and self.nv:
            return _put(self.qkv[self.nq + self.nk:], t)
        if name == "o":
            return _put(self.o, t)
        if name == "sink" and self.sink is not None:
            return _put(self.sink, t)
        if name == "q.norm" and self.q_norm is not None and self.spec.norm_weights:
            return _put(self.q_norm, t)
        if name == "k.norm" and self.k_norm is not None and self.spec.norm_weights:
            return _put(self.k_norm, t)
        if name == "vmix" and self.vmix is not None:
            return _put(self.vmix, t)
        if name == "rel" and self.spec.bias_max:
            if t.shape != self.rel.shape:   # the number of buckets is the tensor's
                self.rel = torch.empty(t.shape, dtype=torch.float32, device=self.device)
            return _put(self.rel, t)
        return False

    def state(self) -> Dict[str, torch.Tensor]:
        out = {"q": self.qkv[: self.nq], "k": self.qkv[self.nq: self.nq + self.nk], "o": self.o}
        if self.nv:
            out["v"] = self.qkv[self.nq + self.nk:]
        if self.sink is not None:
            out["sink"] = self.sink
        if self.q_norm is not None and self.spec.norm_weights:
            out["q.norm"], out["k.norm"] = self.q_norm, self.k_norm
        if self.vmix is not None:
            out["vmix"] = self.vmix.reshape(())
        if self.rel is not None:
            out["rel"] = self.rel
        return out

    def attend(self, p: torch.Tensor, positions: torch.Tensor, meta, cache: torch.Tensor, eps: float,
               shared: Dict[str, Any]) -> torch.Tensor:
        """p [T, >= nq + nk + nv]: this mixer's q | k | v columns of a projection output. Returns W_o attn."""
        s = self.spec
        q, k = p[:, : self.nq], p[:, self.nq: self.nq + self.nk]
        v = p[:, self.nq + self.nk: self.nq + self.nk + self.nv] if self.nv else None
        v_first = lam = None
        if s.v_mix:
            if "v_first" in shared:
                v_first, lam = shared["v_first"], self.vmix
            else:
                shared["v_first"] = v   # a view: the projection output stays alive for the later layers
        qr = seq.qkv_prep(q, k, v, cache, s.heads, s.kv_heads, s.dim, s.vdim, positions, meta.slot_mapping, eps,
                          q_norm=self.q_norm, k_norm=self.k_norm, rot_dims=s.rot_dims, inv_freq=self.inv_freq,
                          v_unit=s.v_unit, v_lambda=lam, v_first=v_first, head_norm=s.head_norm,
                          q_temp_coef=s.q_temp_coef, q_temp_every=s.q_temp_every, norm_after_rot=s.norm_after_rot)
        o = seq.sink_attn(qr, cache, meta.block_tables, meta.cu_q if meta.is_prefill else None, meta.ctx_lens,
                          positions, self.sink, self.bias, meta.max_q_len if meta.is_prefill else 1, s.heads,
                          s.kv_heads, s.dim, s.vdim, s.window, s.scale, softcap=s.softcap, slopes=self.slopes)
        return mix.linear(o, self.o)

    def forward_streams(self, h, positions, meta, cache, eps, state, shared, rag):
        """(y1, y2, a1, a2): the mixer's output is a1 * y1 (+ a2 * y2)."""
        return self.attend(mix.linear(h, self.qkv), positions, meta, cache, eps, shared), None, 1.0, 1.0

    def forward(self, a, positions, meta, cache, eps, state=None, shared=None, **_):
        return self.attend(mix.linear(a, self.qkv), positions, meta, cache, eps, shared if shared is not None else {})


class GatedDeltaMixer:
    """Weights and forward of the gated delta rule: q / k / v through a short causal convolution and SiLU, unit q
    and k, a decay and a write strength per head, S <- g S + k (beta (v - S^T k))^T, read-out S^T q, RMS norm,
    output gate. The fp32 state S and the convolution's last inputs are per-sequence state (``state`` dict:
    "delta" [slots, H, dim, vdim], "conv" [slots, taps - 1, C])."""

    type_name = "gated_delta"

    @staticmethod
    def spec_from_config(m: Dict[str, Any]) -> GatedDeltaSpec:
        return GatedDeltaSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=int(m["dim"]),
                              vdim=int(m.get("vdim") or m["dim"]), conv=int(m.get("conv") or 1))

    def __init__(self, spec: GatedDeltaSpec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        s = self.spec = spec
        self.device, self.dtype = torch.device(device), dtype
        if s.heads % s.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")

        def rnd(*shape, scale=std, dt=dtype):
            t = torch.empty(*shape, dtype=dt, device=self.device)
            return t.normal_(0.0, scale, generator=gen) if gen is not None else t.zero_()

        f32 = torch.float32
        C, H = s.channels, s.heads
        self.nqk = s.kv_heads * s.dim
        # one projection: [q | k | v | b | a | g] rows
        self.w_in = rnd(C + 2 * H + H * s.vdim, hidden)
        self.conv_w = rnd(C, s.conv, scale=0.5, dt=f32)
        self.A_log = rnd(H, scale=0.5, dt=f32)
        self.dt_bias = rnd(H, scale=0.5, dt=f32)
        self.norm = 1.0 + rnd(s.vdim, scale=0.1, dt=f32)
        self.o = rnd(hidden, H * s.vdim)
        self.conv_wt = None
        self.finalize()

    def finalize(self) -> None:
        """Derived tensors, after the weights changed: the convolution weights tap-major for 16-byte loads."""
        self.conv_wt = self.conv_w.t().contiguous()

    def tensors(self) -> List[torch.Tensor]:
        return [self.w_in, self.conv_w, self.A_log, self.dt_bias, self.norm, self.o]

    def in_rows(self) -> int:
        return self.w_in.shape[0]

    def _rows(self) -> Dict[str, Tuple[int, int]]:
        s = self.spec
        C, H, n = s.channels, s.heads, self.nqk
        return {"q": (0, n), "k": (n, 2 * n), "v": (2 * n, C), "b": (C, C + H), "a": (C + H, C + 2 * H),
                "g": (C + 2 * H, C + 2 * H + H * s.vdim)}

    def load(self, name: str, t: torch.Tensor) -> bool:
        rows = self._rows()
        if name in rows:
            return _put(self.w_in[rows[name][0]: rows[name][1]], t)
        if name.endswith(".conv") and name[:-5] in ("q", "k", "v"):
            a, b = rows[name[:-5]]
            return _put(self.conv_w[a:b], t)
        for nm, dst in (("A_log", self.A_log), ("dt_bias", self.dt_bias), ("norm", self.norm), ("o", self.o)):
            if name == nm:
                return _put(dst, t)
        return False

    def state(self) -> Dict[str, torch.Tensor]:
        rows = self._rows()
        out = {k: self.w_in[a:b] for k, (a, b) in rows.items()}
        for k in ("q", "k", "v"):
            out[k + ".conv"] = self.conv_w[rows[k][0]: rows[k][1]]
        out.update({"A_log": self.A_log, "dt_bias": self.dt_bias, "norm": self.norm, "o": self.o})
        return out

    def recur(self, p: torch.Tensor, eps: float, state: Dict[str, torch.Tensor], rag: seq.Ragged) -> torch.Tensor:
        """p [T, in_rows]: this mixer's columns of a projection output. Returns W_o of the gated read-out."""
        s = self.spec
        C, H = s.channels, s.heads
        x, b, a, g = p[:, :C], p[:, C: C + H], p[:, C + H: C + 2 * H], p[:, C + 2 * H: C + 2 * H + H * s.vdim]
        qkv32, bg = seq.delta_prep(x, b, a, self.conv_w, state["conv"], self.A_log, self.dt_bias, H, s.kv_heads, s.dim,
                                   s.vdim, rag, conv_wt=self.conv_wt)
        seq.conv_state_update(state["conv"], x, H, s.kv_heads, s.dim, s.vdim, rag)
        o = seq.gated_delta(qkv32, bg, g, self.norm, eps, state["delta"], H, s.kv_heads, s.dim, s.vdim, rag)
        return mix.linear(o, self.o)

    def forward_streams(self, h, positions, meta, cache, eps, state, shared, rag):
        return self.recur(mix.linear(h, self.w_in), eps, state, rag), None, 1.0, 1.0


class ParallelMixer:
    """Softmax attention and a gated delta rule side by side on the same input (one fused input projection), summed
    with the config's two scales."""

    type_name = "parallel"

    @staticmethod
    def spec_from_config(m: Dict[str, Any]) -> ParallelSpec:
        return ParallelSpec(left=SinkAttentionMixer.spec_from_config(m["left"], as_left=True),
                            right=GatedDeltaMixer.spec_from_config(m["right"]),
                            left_scale=float(m.get("left_scale", 1.0)), right_scale=float(m.get("right_scale", 1.0)))

    def __init__(self, spec: ParallelSpec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        self.spec = spec
        self.left = SinkAttentionMixer(spec.left, hidden, device, dtype, gen, std)
        self.right = GatedDeltaMixer(spec.right, hidden, device, dtype, gen, std)
        self._fuse()

    def _fuse(self) -> None:
        # both input projections as one weight; the halves stay views of it, so loading writes in place
        nl = self.left.in_rows()
        self.w_in = torch.cat([self.left.qkv, self.right.w_in], 0)
        self.left.qkv, self.right.w_in = self.w_in[:nl], self.w_in[nl:]

    def finalize(self) -> None:
        self.left.finalize()
        self.right.finalize()

    def tensors(self) -> List[torch.Tensor]:
        return [self.w_in] + [t for t in self.left.tensors()[1:]] + [t for t in self.right.tensors()[1:]]

    def load(self, name: str, t: torch.Tensor) -> bool:
        if name.startswith("left."):
            return self.left.load(name[5:], t)
        if name.startswith("right."):
            return self.right.load(name[6:], t)
        return False

    def state(self) -> Dict[str, torch.Tensor]:
        out = {"left." + k: v for k, v in self.left.state().items()}
        out.update({"right." + k: v for k, v in self.right.state().items()})
        return out

    def forward_streams(self, h, positions, meta, cache, eps, state, shared, rag):
        p = mix.linear(h, self.w_in)
        nl = self.left.in_rows()
        yl = self.left.attend(p[:, :nl], positions, meta, cache, eps, shared)
        yr = self.right.recur(p[:, nl:], eps, state, rag)
        return yl, yr, self.spec.left_scale, self.spec.right_scale


for _m in (SinkAttentionMixer, GatedDeltaMixer, ParallelMixer):
    MIXERS[_m.type_name] = _m


# -------------------------------------------------------------------------------------------------- state
class SeqStatePool:
    """Per-sequence state besides the paged cache, one slot per live sequence: ``layers[i]`` maps a state name to
    a tensor [slots + 1, ...] (what the layer's mixer declares in ``state_shapes``), ``prev_tok`` [slots + 1] the
    last token seen. The last slot belongs to no sequence: padded rows of a captured decode step write there.
    Nothing is cleared when a slot changes hands: a sequence at position 0 starts from zero state by itself."""

    def __init__(self, layer_shapes: List[Dict[str, Tuple[tuple, torch.dtype]]], num_slots: int, device):
        self.num_slots = num_slots
        self.pad_slot = num_slots
        self.layers = [{k: torch.zeros((num_slots + 1,) + tuple(shape), dtype=dt, device=device)
                        for k, (shape, dt) in shapes.items()} for shapes in layer_shapes]
        self.prev_tok = torch.zeros(num_slots + 1, dtype=torch.int64, device=device)

    @property
    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for d in self.layers for t in d.values()) + self.prev_tok.numel() * 8


class FekLayerWeights:
    __slots__ = ("norm1", "norm2", "mix", "up", "down", "act", "hc1", "hc2")

    def __init__(self):
        for s in self.__slots__:
            setattr(self, s, None)


class FekolornLM:
    """The model behind :class:`src.engine.llm_engine.LLMEngine` for ``architecture: Fekolorn`` checkpoints (same
    interface as the other families: forward / compute_logits / load_state_dict, plus ``make_seq_state``)."""

    needs_decode_partials = False
    graph_capturable = True
    needs_seq_state = True          # the engine gives every live sequence a state slot (AttnMetadata.state_slots)
    supports_prefix_cache = False   # a cached prefix holds keys and values but not the recurrent state after it

    def __init__(self, arch: FekolornArch, device, dtype=torch.bfloat16, tp: Optional[TPContext] = None, seed: int = 0,
                 init_std: float = 0.05, max_position: Optional[int] = None, random_init: bool = True, **_):
        if tp is not None and tp.enabled:
            raise ValueError("Fekolorn runs on one GPU (no tensor-parallel layout is defined for its mixers)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Fekolorn runs in bfloat16 or float32")
        if arch.streams > 8:
            raise ValueError("at most 8 residual streams")
        self.arch, self.device, self.dtype = arch, torch.device(device), dtype
        self.tp = tp or TPContext()
        self.hq, self.hkv = arch.num_heads, 1
        self.max_position = max_position or arch.max_position
        self.S = max(1, arch.streams)
        gen = None
        if random_init:
            gen = torch.Generator(device=self.device)
            gen.manual_seed(seed)
        h, f32 = arch.hidden_size, torch.float32

        def rnd(*shape, scale=init_std, dt=dtype):
            t = torch.empty(*shape, dtype=dt, device=self.device)
            return t.normal_(0.0, scale, generator=gen) if gen is not None else t.zero_()

        def hc():
            if not arch.streams:
                return None
            S = arch.streams
            return {"in": 1.0 / S + rnd(S, scale=0.1, dt=f32), "out": 1.0 + rnd(S, scale=0.1, dt=f32),
                    "mix": torch.eye(S, dtype=f32, device=self.device) + rnd(S, S, scale=0.1, dt=f32)}

        self.embed = rnd(arch.vocab_size, h, scale=1.0)
        self.bigram = rnd(arch.bigram_buckets + 1, h, scale=1.0) if arch.bigram_buckets else None
        self.layers: List[FekLayerWeights] = []
        for spec in arch.layers:
            lw = FekLayerWeights()
            lw.norm1 = 1.0 + rnd(1, scale=0.1, dt=f32)
            lw.hc1 = hc()
            lw.mix = MIXERS[spec.type](spec.mixer, h, self.device, dtype, gen, init_std)
            if spec.mlp is not None:
                lw.norm2 = 1.0 + rnd(1, scale=0.1, dt=f32)
                lw.hc2 = hc()
                lw.up = rnd(spec.mlp.ff, h)
                lw.down = rnd(h, spec.mlp.ff)
                lw.act = rnd(4, scale=0.5, dt=f32)
            self.layers.append(lw)
        self.norm = 1.0 + rnd(1, scale=0.1, dt=f32)
        self.lm_head = rnd(arch.vocab_size, h)
        self.seq_state: Optional[SeqStatePool] = None

    # ------------------------------------------------------------------ weights
    def load_state_dict(self, tensors: Dict[str, torch.Tensor], fold: bool = True) -> int:
        """Tensors under the checkpoint's names: ``embed``, ``bigram``, ``head``, ``final.norm`` and, for layer i,
        ``l<i>.norm1|norm2``, ``l<i>.hc1|hc2.in|out|mix``, ``l<i>.mix.<name>`` (the mixer's own),
        ``l<i>.mlp.up|down|act``."""
        n = 0
        top = {"embed": self.embed, "bigram": self.bigram, "head": self.lm_head, "final.norm": self.norm}
        for name, t in tensors.items():
            if name in top:
                if top[name] is not None:
                    n += _put(top[name], t)
                continue
            if not (name.startswith("l") and "." in name and name[1:name.index(".")].isdigit()):
                continue
            li, rest = int(name[1:name.index(".")]), name[name.index(".") + 1:]
            if li >= len(self.layers):
                continue
            lw = self.layers[li]
            if rest == "norm1":
                n += _put(lw.norm1, t)
            elif rest == "norm2" and lw.norm2 is not None:
                n += _put(lw.norm2, t)
            elif rest.startswith("mix."):
                n += bool(lw.mix.load(rest[4:], t))
            elif rest.startswith("hc1.") and lw.hc1 is not None and rest[4:] in lw.hc1:
                n += _put(lw.hc1[rest[4:]], t)
            elif rest.startswith("hc2.") and lw.hc2 is not None and rest[4:] in lw.hc2:
                n += _put(lw.hc2[rest[4:]], t)
            elif rest.startswith("mlp.") and lw.up is not None:
                dst = {"up": lw.up, "down": lw.down, "act": lw.act}.get(rest[4:])
                if dst is not None:
                    n += _put(dst, t)
        if fold:
            self.fold_norm_weights()
        return n

    def fold_norm_weights(self, layers=None) -> None:
        """Called once the weights are in: tensors derived from them (the attention bias per distance)."""
        for lw in self.layers:
            lw.mix.finalize()

    def state_dict(self) -> Dict[str, torch.Tensor]:
        out = {"embed": self.embed, "head": self.lm_head, "final.norm": self.norm.reshape(())}
        if self.bigram is not None:
            out["bigram"] = self.bigram
        for i, lw in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = lw.norm1.reshape(())
            for k, v in lw.mix.state().items():
                out[p + "mix." + k] = v
            if lw.hc1 is not None:
                for k, v in lw.hc1.items():
                    out[p + "hc1." + k] = v
            if lw.up is not None:
                out[p + "norm2"] = lw.norm2.reshape(())
                out[p + "mlp.up"], out[p + "mlp.down"], out[p + "mlp.act"] = lw.up, lw.down, lw.act
                if lw.hc2 is not None:
                    for k, v in lw.hc2.items():
                        out[p + "hc2." + k] = v
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
        tot = sum(t.numel() * t.element_size() for t in (self.embed, self.lm_head) + (
            (self.bigram,) if self.bigram is not None else ()))
        for lw in self.layers:
            tot += sum(t.numel() * t.element_size() for t in lw.mix.tensors())
            tot += sum(t.numel() * t.element_size() for t in (lw.up, lw.down) if t is not None)
        return tot

    # ------------------------------------------------------------ cache + state
    def kv_bytes_per_block(self, block_size: int) -> int:
        return max(1, self.arch.kv_bytes_per_token(self.embed.element_size())) * block_size

    def make_kv_pool(self, num_blocks: int, block_size: int) -> LayerRowPool:
        return LayerRowPool([l.mixer.cache_width for l in self.arch.layers], num_blocks, block_size, self.device,
                            self.dtype)

    def make_seq_state(self, num_slots: int) -> SeqStatePool:
        self.seq_state = SeqStatePool([l.mixer.state_shapes() for l in self.arch.layers], num_slots, self.device)
        return self.seq_state

    def activation_bytes(self, tokens: int) -> int:
        a = self.arch
        widest = 0
        for l, lw in zip(a.layers, self.layers):
            w = 3 * lw.mix.w_in.shape[0] if hasattr(lw.mix, "w_in") else 3 * lw.mix.qkv.shape[0]
            if l.mlp is not None:
                w = max(w, 3 * l.mlp.ff)
            widest = max(widest, w)
        return tokens * (4 * self.S * a.hidden_size + 8 * a.hidden_size + 4 * widest) + (1 << 30)

    # ----------------------------------------------------------------- forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, meta, kv_pool,
                layer_hook=None) -> torch.Tensor:
        """Final-norm hidden states [T, W] in the model dtype. ``kv_pool``: one cache tensor per layer.
        ``meta.state_slots``: the state slot of every sequence of the step. ``layer_hook(i, residual)``: called
        after each layer with the fp32 sum of the streams."""
        if self.seq_state is None or getattr(meta, "state_slots", None) is None:
            raise RuntimeError("Fekolorn needs per-sequence state slots (LLMEngine provides them)")
        a, st, eps = self.arch, self.seq_state, self.arch.rms_eps
        rag = seq.Ragged(positions, meta.cu_q if meta.is_prefill else None, meta.state_slots)
        xs = seq.embed_hash(input_ids, self.embed, self.bigram, rag, st.prev_tok, a.embed_scale, a.bigram_buckets,
                            a.bigram_mul_prev, a.bigram_mul_cur, self.S)
        if self.bigram is not None:
            seq.store_last_token(st.prev_tok, input_ids, rag)

        def nxt(li: int, second: bool):
            """(in weights, gain) of the sublayer that follows sublayer (li, second)."""
            lw = self.layers[li]
            if not second and lw.up is not None:
                return (lw.hc2["in"] if lw.hc2 else None), lw.norm2
            if li + 1 < len(self.layers):
                n = self.layers[li + 1]
                return (n.hc1["in"] if n.hc1 else None), n.norm1
            return None, self.norm

        l0 = self.layers[0]
        h = seq.stream_mix_norm(xs, None, None, 1.0, 1.0, None, None, l0.hc1["in"] if l0.hc1 else None, l0.norm1, eps,
                                self.dtype)
        shared: Dict[str, Any] = {}
        for li, lw in enumerate(self.layers):
            y1, y2, a1, a2 = lw.mix.forward_streams(h, positions, meta, kv_pool[li], eps, st.layers[li], shared, rag)
            if meta.kv_hook is not None:
                meta.kv_hook(li)
            inw, gain = nxt(li, False)
            hc = lw.hc1 or {}
            h = seq.stream_mix_norm(xs, y1, y2, a1, a2, hc.get("mix"), hc.get("out"), inw, gain, eps, self.dtype)
            if lw.up is not None:
                y = mix.linear(seq.poly_norm_act(mix.linear(h, lw.up), lw.act, eps), lw.down)
                inw, gain = nxt(li, True)
                hc = lw.hc2 or {}
                h = seq.stream_mix_norm(xs, y, None, 1.0, 1.0, hc.get("mix"), hc.get("out"), inw, gain, eps, self.dtype)
            if layer_hook is not None:
                layer_hook(li, xs.sum(1))
        return h

    def compute_logits(self, hidden: torch.Tensor, argmax_parts=None) -> torch.Tensor:
        """fp32 logits [rows, vocab] = head(hidden)."""
        if argmax_parts is not None:
            raise ValueError("this head writes no per-tile argmax candidates")
        return mix.linear(hidden, self.lm_head).float()
