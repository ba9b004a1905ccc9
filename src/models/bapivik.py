"""
Bapivik: a decoder-only LM whose layers are listed in ``config.json``, with learned position vectors, a norm before
and after every sublayer, a learned weighted average over the results of all earlier layers after every layer, tied
input / output embeddings with capped logits, and three mixer types:

* ``lightning`` — linear attention with a fixed decay per head, SiLU feature maps, one RMS norm over all heads and a
  sigmoid output gate (:class:`LightningMixer`); its fp32 matrix state per head lives in per-sequence state slots;
* ``latent_attention`` — causal softmax attention whose keys and values are expanded from a cached low-rank latent,
  without positions, with one sigmoid output gate per head; a layer may attend over the latents that an earlier
  layer cached instead of making its own (:class:`src.models.datatar.LatentAttentionMixer` with ``out_gate``,
  ``kv_from``, no rotary part, no sink);
* ``attention`` — grouped-query softmax attention without rotation whose values are the un-normed keys, with q and k
  normed per head, a query temperature growing with the position, capped scores, a linear distance penalty per head
  and a sliding window (:class:`src.models.fekolorn.SinkAttentionMixer` with ``head_norm``, ``v_from_k``,
  ``softcap``, ``slope_exp``, ``q_temp_*``, no sink).

Feed-forward: ``W_down relu(W_up h + b_up)^2 + b_down``. Per layer i (T tokens; X_0 the embedding output, X_(i+1)
the layer's result, all fp32 planes of one buffer):

    x = X_(i+1) <- the averaged input (written by the previous boundary launch), h = rms(x) * norm1
    y = mixer(h);  x += rms(y) * norm1b;  h = rms(x) * norm2                      post_pre_norm     HIP, one launch
    y = ff(h);     x += rms(y + b_down) * norm2b                                  |
    next input = sum_(j <= i+1) dwa[j] X_j;  h = rms(next input) * next norm1     depth_avg_norm    HIP, one launch

The model plugs into :class:`src.engine.llm_engine.LLMEngine` like the other families: paged cache rows per layer
from :class:`src.models.datatar.LayerRowPool` (none for layers without a cache of their own), state slots from
:class:`src.models.fekolorn.SeqStatePool`.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, replace
from typing import Any, Dict, List, Optional, Tuple

import torch

from src.models.datatar import MIXERS, LatentAttentionMixer, LatentAttnSpec, LayerRowPool
from src.models.fekolorn import SeqStatePool, SinkAttentionMixer, SinkAttnSpec
from src.ops import lin, mix, seq
from src.parallel.tp import TPContext

# head h of the windowed attention loses 2^(-SLOPE_EXP (h + 1) / heads) per position of distance
SLOPE_EXP = 8.0


# ------------------------------------------------------------------------------------------ configuration
@dataclass(frozen=True)
class LightningSpec:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]   # one per head

    @property
    def cache_width(self) -> int:
        return 0

    def state_shapes(self) -> Dict[str, Tuple[tuple, torch.dtype]]:
        return {"lin": ((self.heads, self.dim, self.vdim), torch.float32)}


@dataclass(frozen=True)
class ReluSqMlpSpec:
    ff: int
    kind: str = "dense"

    @staticmethod
    def from_config(m: Optional[Dict[str, Any]]) -> Optional["ReluSqMlpSpec"]:
        if m is None:
            return None
        if m.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {m.get('kind')!r}")
        return ReluSqMlpSpec(ff=int(m["ff"]))


def _latent_spec(m: Dict[str, Any]) -> LatentAttnSpec:
    mask = m.get("mask") or {}
    kv_from = m.get("kv_from")
    return LatentAttnSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=0, vdim=int(m["vdim"]),
                          kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), scale=float(m["scale"]),
                          window=int(mask.get("size") or 0), rot_base=10000.0, rot_dims=0, has_sink=False,
                          out_gate=True, kv_from=None if kv_from is None else int(kv_from))


def _attn_spec(m: Dict[str, Any]) -> SinkAttnSpec:
    mask = m.get("mask") or {}
    qt = m.get("q_temp") or {}
    dim = int(m["dim"])
    if int(m.get("vdim") or dim) != dim:
        raise ValueError("the values are the keys: vdim must equal dim")
    return SinkAttnSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=dim, vdim=dim,
                        scale=float(m["scale"]), window=int(mask.get("size") or 0), qk_norm=True, has_sink=False,
                        head_norm=True, v_from_k=True, softcap=float(m.get("softcap") or 0.0), slope_exp=SLOPE_EXP,
                        q_temp_coef=float(qt.get("coef") or 0.0), q_temp_every=int(qt.get("every") or 1))


def _lightning_spec(m: Dict[str, Any]) -> LightningSpec:
    heads = int(m["heads"])
    decay = tuple(float(d) for d in m["decay"])
    if len(decay) != heads:
        raise ValueError("one decay per head")
    return LightningSpec(heads=heads, dim=int(m["dim"]), vdim=int(m.get("vdim") or m["dim"]), decay=decay)


@dataclass(frozen=True)
class BapLayerSpec:
    type: str
    mixer: Any
    mlp: Optional[ReluSqMlpSpec]


@dataclass(frozen=True)
class BapivikArch:
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    rms_eps: float = 1e-6
    logit_softcap: float = 0.0     # 0: logits as they are
    max_position: int = 2048       # rows of the position table

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
    def from_config(c: Dict[str, Any], name: str = "bapivik") -> "BapivikArch":
        layers = []
        for i, lc in enumerate(c["layers"]):
            t = lc["type"]
            if t not in BAPIVIK_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {t!r} (known: {sorted(BAPIVIK_MIXERS)})")
            spec = BAPIVIK_MIXERS[t][1](lc["mixer"])
            src = getattr(spec, "kv_from", None)
            if src is not None:
                ok = 0 <= src < i and layers[src].type == t and layers[src].mixer.kv_from is None and \
                    layers[src].mixer.kv_rank == spec.kv_rank
                if not ok:
                    raise ValueError(f"layer {i}: kv_from must name an earlier layer of the same type and latent "
                                     "width that makes its own latents")
            layers.append(BapLayerSpec(t, spec, ReluSqMlpSpec.from_config(lc.get("mlp"))))
        return BapivikArch(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(layers),
                           rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                           logit_softcap=float(c.get("logit_softcap") or 0.0),
                           max_position=int(c["max_positions"]))

    def to_config(self) -> Dict[str, Any]:
        out = []
        for l in self.layers:
            m = l.mixer
            if l.type == "lightning":
                mc: Dict[str, Any] = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "decay": list(m.decay)}
            elif l.type == "latent_attention":
                mc = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "q_rank": m.q_rank,
                      "scale": m.scale}
                if m.kv_from is not None:
                    mc["kv_from"] = m.kv_from
            else:
                mc = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
                if m.softcap:
                    mc["softcap"] = m.softcap
                if m.q_temp_coef:
                    mc["q_temp"] = {"coef": m.q_temp_coef, "every": m.q_temp_every}
            if l.type != "lightning" and m.window:
                mc["mask"] = {"size": m.window}
            out.append({"type": l.type, "mixer": mc,
                        "mlp": None if l.mlp is None else {"kind": l.mlp.kind, "ff": l.mlp.ff}})
        return {"architecture": "Bapivik", "layers": out, "logit_softcap": self.logit_softcap,
                "max_positions": self.max_position, "norm": {"eps": self.rms_eps}, "vocab": self.vocab_size,
                "width": self.hidden_size}


def bapivik_arch_from_dir(path: str, **overrides) -> BapivikArch:
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    arch = BapivikArch.from_config(c, name=os.path.basename(os.path.normpath(path)))
    return replace(arch, **overrides) if overrides else arch


# -------------------------------------------------------------------------------------------------- mixers
def _put(dst: torch.Tensor, src: torch.Tensor) -> bool:
    dst.copy_(src.to(dst.device, dst.dtype).reshape(dst.shape))
    return True


class LightningMixer:
    """Weights and forward of decayed linear attention: q, k, v = SiLU of their projections; per head
    S <- decay_h S + k v^T, o = S^T q; the heads' read-outs normed together (RMS, plain weight), times
    sigmoid(W_g h), projected. The fp32 state S is per-sequence state (``state`` dict: "lin" [slots, H, dim, vdim])."""

    type_name = "lightning"

    @staticmethod
    def spec_from_config(m: Dict[str, Any]) -> LightningSpec:
        return _lightning_spec(m)

    def __init__(self, spec: LightningSpec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        s = self.spec = spec
        self.device, self.dtype = torch.device(device), dtype

        def rnd(*shape, scale=std, dt=dtype):
            t = torch.empty(*shape, dtype=dt, device=self.device)
            return t.normal_(0.0, scale, generator=gen) if gen is not None else t.zero_()

        self.nqk, self.nv = s.heads * s.dim, s.heads * s.vdim
        self.w_in = rnd(2 * self.nqk + 2 * self.nv, hidden)            # one projection: [q | k | v | g] rows
        self.norm = 1.0 + rnd(self.nv, scale=0.1, dt=torch.float32)
        self.o = rnd(hidden, self.nv)
        self.decay = torch.tensor(s.decay, dtype=torch.float64).float().to(self.device)

    def finalize(self) -> None:
        """Nothing is derived from the weights."""

    def tensors(self) -> List[torch.Tensor]:
        return [self.w_in, self.norm, self.o]

    def _rows(self) -> Dict[str, Tuple[int, int]]:
        n, v = self.nqk, self.nv
        return {"q": (0, n), "k": (n, 2 * n), "v": (2 * n, 2 * n + v), "g": (2 * n + v, 2 * n + 2 * v)}

    def load(self, name: str, t: torch.Tensor) -> bool:
        rows = self._rows()
        if name in rows:
            return _put(self.w_in[rows[name][0]: rows[name][1]], t)
        if name == "norm":
            return _put(self.norm, t)
        if name == "o":
            return _put(self.o, t)
        return False

    def state(self) -> Dict[str, torch.Tensor]:
        out = {k: self.w_in[a:b] for k, (a, b) in self._rows().items()}
        out.update({"norm": self.norm, "o": self.o})
        return out

    def forward(self, a, positions, meta, cache, eps, state=None, rag=None, **_):
        s = self.spec
        p = mix.linear(a, self.w_in)
        o = lin.lightning_attn(p, 0, self.nqk, 2 * self.nqk, self.decay, state["lin"], s.heads, s.dim, s.vdim, rag)
        return mix.linear(lin.norm_sigmoid_gate(o, p[:, 2 * self.nqk + self.nv:], self.norm, eps), self.o)


MIXERS[LightningMixer.type_name] = LightningMixer

# this family's reading of the layer types: (mixer class, spec from the layer's "mixer" entry)
BAPIVIK_MIXERS = {
    "lightning": (LightningMixer, _lightning_spec),
    "latent_attention": (LatentAttentionMixer, _latent_spec),
    "attention": (SinkAttentionMixer, _attn_spec),
}


class BapLayerWeights:
    __slots__ = ("norm1", "norm1b", "norm2", "norm2b", "mix", "up", "up_b", "down", "down_b", "dwa")

    def __init__(self):
        for s in self.__slots__:
            setattr(self, s, None)


class BapivikLM:
    """The model behind :class:`src.engine.llm_engine.LLMEngine` for ``architecture: Bapivik`` checkpoints (same
    interface as the other families: forward / compute_logits / load_state_dict, plus ``make_seq_state`` when a
    layer carries recurrent state)."""

    needs_decode_partials = False
    graph_capturable = True

    def __init__(self, arch: BapivikArch, device, dtype=torch.bfloat16, tp: Optional[TPContext] = None, seed: int = 0,
                 init_std: float = 0.05, max_position: Optional[int] = None, random_init: bool = True, **_):
        if tp is not None and tp.enabled:
            raise ValueError("Bapivik runs on one GPU (no tensor-parallel layout is defined for its mixers)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Bapivik runs in bfloat16 or float32")
        if arch.num_layers + 1 > 128:
            raise ValueError("the depth average spans at most 128 planes")
        self.arch, self.device, self.dtype = arch, torch.device(device), dtype
        self.tp = tp or TPContext()
        self.hq, self.hkv = arch.num_heads, 1
        # positions index a learned table: nothing beyond it can be served
        self.max_position = arch.max_position
        # the engine gives every live sequence a state slot when a layer keeps recurrent state; a cached prefix holds
        # keys and values but not the state after it
        self.needs_seq_state = any(l.mixer.state_shapes() for l in arch.layers)
        self.supports_prefix_cache = not self.needs_seq_state
        gen = None
        if random_init:
            gen = torch.Generator(device=self.device)
            gen.manual_seed(seed)
        h, f32 = arch.hidden_size, torch.float32

        def rnd(*shape, scale=init_std, dt=dtype):
            t = torch.empty(*shape, dtype=dt, device=self.device)
            return t.normal_(0.0, scale, generator=gen) if gen is not None else t.zero_()

        def gain():
            return 1.0 + rnd(h, scale=0.1, dt=f32)

        self.embed = rnd(arch.vocab_size, h, scale=1.0)
        self.pos = rnd(arch.max_position, h, scale=0.5)
        self.layers: List[BapLayerWeights] = []
        for i, spec in enumerate(arch.layers):
            lw = BapLayerWeights()
            lw.norm1, lw.norm1b = gain(), gain()
            lw.mix = BAPIVIK_MIXERS[spec.type][0](spec.mixer, h, self.device, dtype, gen, init_std)
            if spec.mlp is not None:
                lw.norm2, lw.norm2b = gain(), gain()
                lw.up, lw.up_b = rnd(spec.mlp.ff, h), rnd(spec.mlp.ff, scale=0.1)
                lw.down, lw.down_b = rnd(h, spec.mlp.ff), rnd(h, scale=0.1)
            # the average starts as mostly the newest result
            lw.dwa = torch.full((i + 2,), 0.3 / (i + 1), dtype=f32, device=self.device)
            lw.dwa[-1] = 0.7
            self.layers.append(lw)
        self.norm = gain()
        self.seq_state: Optional[SeqStatePool] = None

    # ------------------------------------------------------------------ weights
    def load_state_dict(self, tensors: Dict[str, torch.Tensor], fold: bool = True) -> int:
        """Tensors under the checkpoint's names: ``embed``, ``pos``, ``final.norm`` and, for layer i,
        ``l<i>.norm1|norm1b|norm2|norm2b``, ``l<i>.dwa``, ``l<i>.mix.<name>`` (the mixer's own),
        ``l<i>.mlp.up|up.b|down|down.b``. The output projection is the embedding table."""
        n = 0
        top = {"embed": self.embed, "pos": self.pos, "final.norm": self.norm}
        for name, t in tensors.items():
            if name in top:
                if name == "pos" and t.shape[0] != self.pos.shape[0]:
                    raise ValueError("the position table's rows differ from max_positions")
                n += _put(top[name], t)
                continue
            if not (name.startswith("l") and "." in name and name[1:name.index(".")].isdigit()):
                continue
            li, rest = int(name[1:name.index(".")]), name[name.index(".") + 1:]
            if li >= len(self.layers):
                continue
            lw = self.layers[li]
            if rest in ("norm1", "norm1b", "dwa"):
                n += _put(getattr(lw, rest), t)
            elif rest in ("norm2", "norm2b") and lw.up is not None:
                n += _put(getattr(lw, rest), t)
            elif rest.startswith("mix."):
                n += bool(lw.mix.load(rest[4:], t))
            elif rest.startswith("mlp.") and lw.up is not None:
                dst = {"up": lw.up, "up.b": lw.up_b, "down": lw.down, "down.b": lw.down_b}.get(rest[4:])
                if dst is not None:
                    n += _put(dst, t)
        if fold:
            self.fold_norm_weights()
        return n

    def fold_norm_weights(self, layers=None) -> None:
        """Called once the weights are in: tensors derived from them."""
        for lw in self.layers:
            lw.mix.finalize()

    def state_dict(self) -> Dict[str, torch.Tensor]:
        out = {"embed": self.embed, "pos": self.pos, "final.norm": self.norm}
        for i, lw in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"], out[p + "norm1b"], out[p + "dwa"] = lw.norm1, lw.norm1b, lw.dwa
            for k, v in lw.mix.state().items():
                out[p + "mix." + k] = v
            if lw.up is not None:
                out[p + "norm2"], out[p + "norm2b"] = lw.norm2, lw.norm2b
                out[p + "mlp.up"], out[p + "mlp.up.b"] = lw.up, lw.up_b
                out[p + "mlp.down"], out[p + "mlp.down.b"] = lw.down, lw.down_b
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
        tot = sum(t.numel() * t.element_size() for t in (self.embed, self.pos))
        for lw in self.layers:
            tot += sum(t.numel() * t.element_size() for t in lw.mix.tensors())
            tot += sum(t.numel() * t.element_size() for t in (lw.up, lw.down) if t is not None)
        return tot

    # ------------------------------------------------------------ cache + state
    def kv_bytes_per_block(self, block_size: int) -> int:
        return max(1, self.arch.kv_bytes_per_token(self.embed.element_size())) * block_size

    def make_kv_pool(self, num_blocks: int, block_size: int) -> LayerRowPool:
        """One row per token and layer that caches something; a layer that shares another's latents, or keeps only
        recurrent state, has width 0."""
        return LayerRowPool([l.mixer.cache_width for l in self.arch.layers], num_blocks, block_size, self.device,
                            self.dtype)

    def make_seq_state(self, num_slots: int) -> SeqStatePool:
        self.seq_state = SeqStatePool([l.mixer.state_shapes() for l in self.arch.layers], num_slots, self.device)
        return self.seq_state

    def activation_bytes(self, tokens: int) -> int:
        a = self.arch
        widest = 0
        for l, lw in zip(a.layers, self.layers):
            first = lw.mix.tensors()[0].shape[0]
            w = 3 * first + 4 * l.mixer.heads * (getattr(l.mixer, "kv_rank", 0) + l.mixer.vdim)
            if l.mlp is not None:
                w = max(w, 3 * l.mlp.ff)
            widest = max(widest, w)
        return tokens * (4 * (a.num_layers + 2) * a.hidden_size + 8 * a.hidden_size + 4 * widest) + (1 << 30)

    # ----------------------------------------------------------------- forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, meta, kv_pool,
                layer_hook=None) -> torch.Tensor:
        """Final-norm hidden states [T, W] in the model dtype. ``kv_pool``: one cache tensor per layer.
        ``meta.state_slots``: the state slot of every sequence of the step (models with recurrent layers).
        ``layer_hook(i, x)``: called after each layer with the fp32 stream that goes on to the next one."""
        a, eps, dt = self.arch, self.arch.rms_eps, self.dtype
        st_layers = None
        rag = None
        if self.needs_seq_state:
            if self.seq_state is None or getattr(meta, "state_slots", None) is None:
                raise RuntimeError("Bapivik's recurrent layers need per-sequence state slots (LLMEngine provides them)")
            st_layers = self.seq_state.layers
            rag = seq.Ragged(positions, meta.cu_q if meta.is_prefill else None, meta.state_slots)
        T, L = input_ids.shape[0], len(self.layers)
        # planes 0 .. L: the embedding output and every layer's result; plane i + 1 starts as layer i's (averaged)
        # input and is updated in place; plane L + 1 takes the last average
        planes = torch.empty(L + 2, T, a.hidden_size, dtype=torch.float32, device=input_ids.device)
        lin.embed_pos(input_ids, positions, self.embed, self.pos, planes[0])
        h = lin.depth_avg_norm(planes, 1, None, None, None, None, self.layers[0].norm1, eps, dt)
        shared: Dict[str, Any] = {}
        for i, lw in enumerate(self.layers):
            spec = a.layers[i].mixer
            src = getattr(spec, "kv_from", None)
            y = lw.mix.forward(h, positions, meta, kv_pool[i if src is None else src], eps,
                               state=None if st_layers is None else st_layers[i], shared=shared, rag=rag)
            if meta.kv_hook is not None:
                meta.kv_hook(i)
            nxt = self.layers[i + 1].norm1 if i + 1 < L else self.norm
            if lw.up is not None:
                h = lin.post_pre_norm(planes[i + 1], y, None, lw.norm1b, lw.norm2, eps, dt)
                y = mix.linear(lin.bias_relu2(mix.linear(h, lw.up), lw.up_b), lw.down)
                h = lin.depth_avg_norm(planes, i + 2, lw.dwa, y, lw.down_b, lw.norm2b, nxt, eps, dt)
            else:
                h = lin.depth_avg_norm(planes, i + 2, lw.dwa, y, None, lw.norm1b, nxt, eps, dt)
            if layer_hook is not None:
                layer_hook(i, planes[i + 2])
        return h

    def compute_logits(self, hidden: torch.Tensor, argmax_parts=None) -> torch.Tensor:
        """fp32 logits [rows, vocab] = cap * tanh(embed . hidden / cap) (no cap: the products themselves)."""
        if argmax_parts is not None:
            raise ValueError("this head writes no per-tile argmax candidates")
        z = mix.linear(hidden, self.embed)
        cap = self.arch.logit_softcap
        return lin.tanh_cap(z, cap) if cap else z.float()
