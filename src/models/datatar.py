"""
Datatar: a decoder-only LM whose layers are read from ``config.json`` (one entry per layer: the mixer's type
and sizes, and its feed-forward or none), on the dtype-generic kernels of :mod:`src.ops.mix`.

Per layer (T tokens, residual stream r in fp32, a = its bf16 copy in bf16 mode, r itself in fp32 mode):

    y = mixer(a);  r += rmsnorm(y) * (1 + norm1)        post_norm_residual   HIP (norm on the sublayer OUTPUT)
    y = ff(a);     r += rmsnorm(y) * (1 + norm2)        post_norm_residual   HIP

Mixer ``latent_attention`` (H heads; per head `dim` unrotated + `rot_dim` rotary query dims, value size `vdim`;
the keys and values of all heads come from one latent of width `kv_rank`):

    p    = a @ [W_dq; W_dkv]^T                         one GEMM  [T, q_rank + kv_rank + rot_dim]
    q    = rmsnorm(p[:, :q_rank]) * dq_norm @ W_uq^T   HIP norm + GEMM  [T, H * (dim + rot_dim)]
    cache row = [rmsnorm(p[:, q_rank:q_rank + kv_rank]) * dkv_norm | rotate(p[:, -rot_dim:])]   latent_kv_write HIP
    q_lat[h] = q_nope[h] @ W_uk[h]                     batched GEMM: the query absorbed into the latent space
    o_lat = latent_attn(q_lat, rotate(q_rot), cache)   HIP: window, per-head sink, fp32 scores and weights
    y    = concat_h(o_lat[h] @ W_uv[h]^T) @ W_o^T      batched GEMM + GEMM

so only the latent and the shared rotary key (kv_rank + rot_dim numbers per token and layer) are cached, and
prompt chunks and decode tokens run the same kernel over the paged cache.

Feed-forward ``dense``: clamped sigmoid-gated (``gated_act`` ACT_CLAMPED). ``moe``: sigmoid-scored top-k
routing in fp32, the weight scaling the expert's input, plus an optional shared expert
(``route_sigmoid_topk`` + ``moe_input_scaled``).

Mixer types are looked up in :data:`MIXERS`, so another design's mixer can be added beside this one.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch
import torch.nn.functional as F

from src.ops import lin, mix
from src.parallel.tp import TPContext


# ------------------------------------------------------------------------------------------ configuration
@dataclass(frozen=True)
class LatentAttnSpec:
    heads: int
    dim: int          # unrotated query / key dims per head
    rot_dim: int      # rotary query dims per head = width of the shared rotary key
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    window: int       # 0: every earlier position
    rot_base: float
    rot_dims: int     # rotated dims (pairs 2i, 2i + 1) at the start of the rotary part
    has_sink: bool = True            # a per-head term exp(sink_h) in the softmax denominator
    out_gate: bool = False           # head h's output times sigmoid(W_g a)_h, W_g [heads, hidden]
    kv_from: Optional[int] = None    # no down-projection of its own: attends over that layer's cached latents

    @property
    def cache_width(self) -> int:
        return 0 if self.kv_from is not None else self.kv_rank + self.rot_dim

    def state_shapes(self) -> Dict[str, Any]:
        return {}

    @staticmethod
    def from_config(m: Dict[str, Any]) -> "LatentAttnSpec":
        rot = m.get("rot") or {}
        mask = m.get("mask") or {}
        rot_dim = int(m["rot_dim"])
        return LatentAttnSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim, vdim=int(m["vdim"]),
                              kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), scale=float(m["scale"]),
                              window=int(mask.get("size") or 0), rot_base=float(rot.get("base", 10000.0)),
                              rot_dims=int(rot.get("dims", rot_dim)))


@dataclass(frozen=True)
class MlpSpec:
    kind: str             # "dense" | "moe"
    ff: int = 0           # dense
    limit: float = 0.0    # dense: clamp of gate (above) and up (both sides)
    experts: int = 0      # moe
    top: int = 0
    expert_ff: int = 0
    shared_ff: int = 0    # 0: no shared expert

    @staticmethod
    def from_config(m: Optional[Dict[str, Any]]) -> Optional["MlpSpec"]:
        if m is None:
            return None
        kind = m["kind"]
        if kind == "dense":
            return MlpSpec("dense", ff=int(m["ff"]), limit=float(m["limit"]))
        if kind == "moe":
            shared = m.get("shared") or {}
            return MlpSpec("moe", experts=int(m["router"]["experts"]), top=int(m["router"]["top"]),
                           expert_ff=int(m["expert"]["ff"]), shared_ff=int(shared.get("ff") or 0))
        raise ValueError(f"unknown feed-forward kind {kind!r}")


@dataclass(frozen=True)
class LayerSpec:
    type: str
    mixer: Any
    mlp: Optional[MlpSpec]


@dataclass(frozen=True)
class DatatarArch:
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    rms_eps: float = 1e-6
    logit_scale: float = 1.0
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
    def from_config(c: Dict[str, Any], name: str = "datatar") -> "DatatarArch":
        layers = []
        for i, lc in enumerate(c["layers"]):
            t = lc["type"]
            if t not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {t!r} (known: {sorted(MIXERS)})")
            layers.append(LayerSpec(t, MIXERS[t].spec_from_config(lc["mixer"]), MlpSpec.from_config(lc.get("mlp"))))
        return DatatarArch(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=tuple(layers),
                           rms_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                           logit_scale=float(c.get("logit_scale", 1.0)))

    def to_config(self) -> Dict[str, Any]:
        out = []
        for l in self.layers:
            m = l.mixer
            mc = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                  "q_rank": m.q_rank, "scale": m.scale, "rot": {"base": m.rot_base, "dims": m.rot_dims}}
            if m.window:
                mc["mask"] = {"size": m.window}
            f = l.mlp
            if f is None:
                fc = None
            elif f.kind == "dense":
                fc = {"kind": "dense", "ff": f.ff, "limit": f.limit}
            else:
                fc = {"kind": "moe", "router": {"experts": f.experts, "top": f.top}, "expert": {"ff": f.expert_ff}}
                if f.shared_ff:
                    fc["shared"] = {"ff": f.shared_ff}
            out.append({"type": l.type, "mixer": mc, "mlp": fc})
        return {"architecture": "Datatar", "layers": out, "logit_scale": self.logit_scale,
                "norm": {"eps": self.rms_eps}, "vocab": self.vocab_size, "width": self.hidden_size}


def datatar_arch_from_dir(path: str, **overrides) -> DatatarArch:
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    arch = DatatarArch.from_config(c, name=os.path.basename(os.path.normpath(path)))
    if overrides:
        from dataclasses import replace

        arch = replace(arch, **overrides)
    return arch


# ------------------------------------------------------------------------------------------------ weights
class MixLayerWeights:
    __slots__ = ("norm1", "norm2", "mix", "gate_up", "down", "router", "w13", "w2", "shared_gate_up", "shared_down")

    def __init__(self):
        for s in self.__slots__:
            setattr(self, s, None)


class LatentAttentionMixer:
    """Weights and forward of one ``latent_attention`` mixer."""

    type_name = "latent_attention"

    @staticmethod
    def spec_from_config(m: Dict[str, Any]) -> LatentAttnSpec:
        return LatentAttnSpec.from_config(m)

    def __init__(self, spec: LatentAttnSpec, hidden: int, device, dtype, gen: Optional[torch.Generator], std: float):
        s = self.spec = spec

        def rnd(*shape, scale=std):
            t = torch.empty(*shape, dtype=dtype, device=device)
            return t.normal_(0.0, scale, generator=gen) if gen is not None else t.zero_()

        # one input projection: [W_dq; W_dkv (unless the latents are another layer's); W_g (with an output gate)]
        self.kvw = 0 if s.kv_from is not None else s.kv_rank + s.rot_dim
        self.dqkv = rnd(s.q_rank + self.kvw + (s.heads if s.out_gate else 0), hidden)
        self.dq_norm = torch.ones(s.q_rank, dtype=dtype, device=device)
        self.dkv_norm = torch.ones(s.kv_rank, dtype=dtype, device=device) if self.kvw else None
        self.uq = rnd(s.heads * (s.dim + s.rot_dim), s.q_rank, scale=std * 4)
        self.uk = rnd(s.heads, s.dim, s.kv_rank, scale=std * 4)            # W_uk, head by head: [H, dim, rank]
        self.uv_t = rnd(s.heads, s.kv_rank, s.vdim, scale=std * 4)         # W_uv^T head by head: [H, rank, vdim]
        self.sink = torch.zeros(s.heads, dtype=torch.float32, device=device) if s.has_sink else None
        self.o = rnd(hidden, s.heads * s.vdim)
        self.inv_freq = mix.rope_inv_freq(s.rot_base, s.rot_dims, device)

    def finalize(self) -> None:
        """Nothing is derived from the weights."""

    def tensors(self) -> List[torch.Tensor]:
        return [t for t in (self.dqkv, self.dq_norm, self.dkv_norm, self.uq, self.uk, self.uv_t, self.sink, self.o)
                if t is not None]

    def load(self, name: str, t: torch.Tensor) -> bool:
        """One checkpoint tensor ``<layer>.mix.<name>``; False if the name is not this mixer's."""
        s = self.spec

        def put(dst, src):
            dst.copy_(src.to(dst.device, dst.dtype))
            return True

        if name == "dq":
            return put(self.dqkv[: s.q_rank], t)
        if name == "dkv" and self.kvw:
            return put(self.dqkv[s.q_rank: s.q_rank + self.kvw], t)
        if name == "g" and s.out_gate:
            return put(self.dqkv[s.q_rank + self.kvw:], t)
        if name == "dq.norm":
            return put(self.dq_norm, t)
        if name == "dkv.norm" and self.kvw:
            return put(self.dkv_norm, t)
        if name == "uq":
            return put(self.uq, t)
        if name == "uk":
            return put(self.uk, t.view(s.heads, s.dim, s.kv_rank))
        if name == "uv":
            return put(self.uv_t, t.view(s.heads, s.vdim, s.kv_rank).transpose(1, 2))
        if name == "sink" and s.has_sink:
            return put(self.sink, t)
        if name == "o":
            return put(self.o, t)
        return False

    def state(self) -> Dict[str, torch.Tensor]:
        s = self.spec
        out = {"dq": self.dqkv[: s.q_rank], "dq.norm": self.dq_norm, "uq": self.uq,
               "uk": self.uk.reshape(s.heads * s.dim, s.kv_rank),
               "uv": self.uv_t.transpose(1, 2).reshape(s.heads * s.vdim, s.kv_rank), "o": self.o}
        if self.kvw:
            out["dkv"], out["dkv.norm"] = self.dqkv[s.q_rank: s.q_rank + self.kvw], self.dkv_norm
        if s.out_gate:
            out["g"] = self.dqkv[s.q_rank + self.kvw:]
        if s.has_sink:
            out["sink"] = self.sink
        return out

    def forward(self, a: torch.Tensor, positions: torch.Tensor, meta, cache: torch.Tensor, eps: float,
                **_) -> torch.Tensor:
        """``cache``: this layer's rows, or with ``kv_from`` the rows of the layer whose latents it shares (that
        layer ran earlier in the step, so this step's tokens are already there)."""
        s = self.spec
        t = a.shape[0]
        p = mix.linear(a, self.dqkv)
        nq = s.q_rank
        if self.kvw:
            cq = mix.latent_qkv_prep(p[:, : nq + self.kvw], nq, self.dq_norm, self.dkv_norm, cache, positions,
                                     meta.slot_mapping, s.kv_rank, s.rot_dim, self.inv_freq, eps)
        else:
            cq = mix.rms_norm_ext(p[:, :nq], self.dq_norm, eps)
        q = mix.linear(cq, self.uq)
        q_lat = torch.bmm(q.view(t, s.heads, s.dim + s.rot_dim)[:, :, : s.dim].transpose(0, 1), self.uk)
        o_lat = mix.latent_attn(q_lat, q, s.dim, cache, meta.block_tables, meta.cu_q if meta.is_prefill else None,
                                meta.ctx_lens, positions, self.sink, meta.max_q_len if meta.is_prefill else 1,
                                s.window, s.scale, s.rot_dim, self.inv_freq)
        o = torch.bmm(o_lat, self.uv_t)                                    # [H, T, vdim]
        if s.out_gate:
            o = lin.head_gate(o, p[:, nq + self.kvw:])
        else:
            o = o.transpose(0, 1).reshape(t, s.heads * s.vdim)
        return mix.linear(o, self.o)


MIXERS = {LatentAttentionMixer.type_name: LatentAttentionMixer}

GATE_ALPHA = 1.702   # the dense feed-forward's gate is g * sigmoid(GATE_ALPHA * g)


class LayerRowPool:
    """Paged cache with one row per token and layer: ``layers[i]`` is [num_blocks, block_size, width_i]. One
    block id addresses the same block in every layer (one block table per sequence). Zeroed once: a padded
    decode row reads block 0 before anything was written there."""

    def __init__(self, widths: List[int], num_blocks: int, block_size: int, device, dtype):
        self.num_blocks, self.block_size, self.widths = num_blocks, block_size, list(widths)
        self.uniform = len(set(widths)) == 1
        if self.uniform:
            self._flat = torch.zeros(len(widths), num_blocks, block_size, widths[0], dtype=dtype, device=device)
            self.layers = [self._flat[i] for i in range(len(widths))]
        else:
            self._flat = None
            self.layers = [torch.zeros(num_blocks, block_size, w, dtype=dtype, device=device) for w in widths]
        self.tensor = self.layers   # what the model's forward receives

    @property
    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.layers)

    def planes(self) -> torch.Tensor:
        """[layers, num_blocks, 1, block_size, width] for the block movers (layers of one width only)."""
        if self._flat is None:
            raise NotImplementedError("block movers need one row width in every layer")
        return self._flat.unsqueeze(2)


class DatatarLM:
    """The model behind :class:`src.engine.llm_engine.LLMEngine` for ``architecture: Datatar`` checkpoints
    (same interface as :class:`src.models.llama.CausalLM`: forward / compute_logits / load_state_dict)."""

    needs_decode_partials = False   # the runner's split-KV scratch of the GQA decode kernel is not used
    graph_capturable = True

    def __init__(self, arch: DatatarArch, device, dtype=torch.bfloat16, tp: Optional[TPContext] = None, seed: int = 0,
                 init_std: float = 0.05, max_position: Optional[int] = None, random_init: bool = True, **_):
        if tp is not None and tp.enabled:
            raise ValueError("Datatar runs on one GPU (no tensor-parallel layout is defined for its latent mixer)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Datatar runs in bfloat16 or float32")
        self.arch = arch
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp = tp or TPContext()
        self.hq, self.hkv = arch.num_heads, 1
        self.max_position = max_position or arch.max_position
        gen = None
        if random_init:
            gen = torch.Generator(device=self.device)
            gen.manual_seed(seed)
        h = arch.hidden_size

        def rnd(*shape, scale=init_std):
            t = torch.empty(*shape, dtype=dtype, device=self.device)
            return t.normal_(0.0, scale, generator=gen) if gen is not None else t.zero_()

        self.embed = rnd(arch.vocab_size, h, scale=1.0)
        self.layers: List[MixLayerWeights] = []
        for spec in arch.layers:
            lw = MixLayerWeights()
            lw.norm1 = rnd(h, scale=0.1)
            lw.mix = MIXERS[spec.type](spec.mixer, h, self.device, dtype, gen, init_std)
            f = spec.mlp
            if f is not None:
                lw.norm2 = rnd(h, scale=0.1)
                if f.kind == "dense":
                    lw.gate_up = rnd(2 * f.ff, h)
                    lw.down = rnd(h, f.ff)
                else:
                    lw.router = rnd(f.experts, h, scale=init_std * 4)
                    lw.w13 = rnd(f.experts, 2 * f.expert_ff, h)
                    lw.w2 = rnd(f.experts, h, f.expert_ff)
                    if f.shared_ff:
                        lw.shared_gate_up = rnd(2 * f.shared_ff, h)
                        lw.shared_down = rnd(h, f.shared_ff)
            self.layers.append(lw)
        self.norm = rnd(h, scale=0.1)
        self.lm_head = rnd(arch.vocab_size, h)

    # ------------------------------------------------------------------ weights
    def load_state_dict(self, tensors: Dict[str, torch.Tensor], fold: bool = True) -> int:
        """Tensors under the checkpoint's names: ``embed``, ``head``, ``final.norm`` and, for layer i,
        ``l<i>.norm1|norm2``, ``l<i>.mix.<name>`` (the mixer's own), ``l<i>.mlp.gate|up|down`` (dense) or
        ``l<i>.mlp.router``, ``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.mlp.shared.gate|up|down`` (moe)."""
        n = 0

        def put(dst, src):
            nonlocal n
            dst.copy_(src.to(dst.device, dst.dtype))
            n += 1

        for name, t in tensors.items():
            if name == "embed":
                put(self.embed, t)
            elif name == "head":
                put(self.lm_head, t)
            elif name == "final.norm":
                put(self.norm, t)
            elif name.startswith("l") and "." in name and name[1:name.index(".")].isdigit():
                li = int(name[1:name.index(".")])
                rest = name[name.index(".") + 1:]
                if li >= len(self.layers):
                    continue
                lw, f = self.layers[li], self.arch.layers[li].mlp
                if rest == "norm1":
                    put(lw.norm1, t)
                elif rest == "norm2" and lw.norm2 is not None:
                    put(lw.norm2, t)
                elif rest.startswith("mix."):
                    if lw.mix.load(rest[4:], t):
                        n += 1
                elif rest.startswith("mlp.") and f is not None:
                    parts = rest.split(".")[1:]
                    if f.kind == "dense" and len(parts) == 1:
                        if parts[0] == "gate":
                            put(lw.gate_up[: f.ff], t)
                        elif parts[0] == "up":
                            put(lw.gate_up[f.ff:], t)
                        elif parts[0] == "down":
                            put(lw.down, t)
                    elif f.kind == "moe":
                        if parts == ["router"]:
                            put(lw.router, t)
                        elif len(parts) == 2 and parts[0] == "shared" and lw.shared_gate_up is not None:
                            if parts[1] == "gate":
                                put(lw.shared_gate_up[: f.shared_ff], t)
                            elif parts[1] == "up":
                                put(lw.shared_gate_up[f.shared_ff:], t)
                            elif parts[1] == "down":
                                put(lw.shared_down, t)
                        elif len(parts) == 2 and parts[0][0] == "e" and parts[0][1:].isdigit():
                            e = int(parts[0][1:])
                            if e < f.experts:
                                if parts[1] == "gate":
                                    put(lw.w13[e, : f.expert_ff], t)
                                elif parts[1] == "up":
                                    put(lw.w13[e, f.expert_ff:], t)
                                elif parts[1] == "down":
                                    put(lw.w2[e], t)
        return n

    def fold_norm_weights(self, layers=None) -> None:
        """Nothing to fold: the norms sit on the sublayers' outputs."""

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
            if f.kind == "dense":
                out[p + "mlp.gate"], out[p + "mlp.up"], out[p + "mlp.down"] = lw.gate_up[: f.ff], lw.gate_up[f.ff:], lw.down
            else:
                out[p + "mlp.router"] = lw.router
                for e in range(f.experts):
                    q = p + f"mlp.e{e}."
                    out[q + "gate"], out[q + "up"], out[q + "down"] = lw.w13[e, : f.expert_ff], lw.w13[e, f.expert_ff:], lw.w2[e]
                if f.shared_ff:
                    q = p + "mlp.shared."
                    out[q + "gate"], out[q + "up"] = lw.shared_gate_up[: f.shared_ff], lw.shared_gate_up[f.shared_ff:]
                    out[q + "down"] = lw.shared_down
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
        tot = 0
        for lw in self.layers:
            for s in MixLayerWeights.__slots__:
                t = getattr(lw, s)
                if isinstance(t, torch.Tensor):
                    tot += t.numel() * t.element_size()
            tot += sum(t.numel() * t.element_size() for t in lw.mix.tensors())
        return tot + sum(t.numel() * t.element_size() for t in (self.embed, self.lm_head, self.norm))

    # ------------------------------------------------------------------- cache
    def kv_bytes_per_block(self, block_size: int) -> int:
        return self.arch.kv_bytes_per_token(self.embed.element_size()) * block_size

    def make_kv_pool(self, num_blocks: int, block_size: int) -> LayerRowPool:
        return LayerRowPool([l.mixer.cache_width for l in self.arch.layers], num_blocks, block_size, self.device,
                            self.dtype)

    def activation_bytes(self, tokens: int) -> int:
        """Rough peak of one step's activations (projections, expert rows, fp32 residual + logits slack)."""
        a = self.arch
        widest = 0
        for l in a.layers:
            m, f = l.mixer, l.mlp
            w = m.q_rank + m.cache_width + 2 * m.heads * (m.dim + m.rot_dim + m.kv_rank + m.vdim)
            if f is not None:
                w = max(w, 3 * f.ff if f.kind == "dense" else 4 * f.top * (a.hidden_size + f.expert_ff) + 3 * f.shared_ff)
            widest = max(widest, w)
        return tokens * (8 * a.hidden_size + 4 * widest) + (1 << 30)

    # ----------------------------------------------------------------- forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, meta, kv_pool,
                layer_hook=None) -> torch.Tensor:
        """Final-norm hidden states [T, H] in the model dtype. ``kv_pool``: one cache tensor per layer
        (:class:`LayerRowPool`). ``layer_hook(i, residual)``: called after each layer with the fp32 residual."""
        eps = self.arch.rms_eps
        x = F.embedding(input_ids, self.embed)
        if self.dtype == torch.float32:
            resid, act, act_out = x, x, None
        else:
            resid, act, act_out = x.float(), x, x
        for li, lw in enumerate(self.layers):
            y = lw.mix.forward(act, positions, meta, kv_pool[li], eps)
            mix.post_norm_residual(resid, y, lw.norm1, eps, True, act=act_out)
            if meta.kv_hook is not None:
                meta.kv_hook(li)
            f = self.arch.layers[li].mlp
            if f is not None:
                y = self._mlp(lw, f, act, post_norm=(resid, lw.norm2, eps, True, act_out))
                if y is not None:
                    mix.post_norm_residual(resid, y, lw.norm2, eps, True, act=act_out)
            if layer_hook is not None:
                layer_hook(li, resid)
        return mix.rms_norm_ext(resid, self.norm, eps, True, out_dtype=self.dtype)

    def _mlp(self, lw: MixLayerWeights, f: MlpSpec, a: torch.Tensor, post_norm=None) -> Optional[torch.Tensor]:
        """The feed-forward's output, or None when it was already added into the residual (``post_norm``: the MoE's
        expert sum and its post-norm are one launch)."""
        if f.kind == "dense":
            return mix.linear(mix.gated_act(mix.linear(a, lw.gate_up), mix.ACT_CLAMPED, f.limit, GATE_ALPHA), lw.down)
        w, ids = mix.route_sigmoid_topk(a, lw.router, f.top)
        shared = None
        if lw.shared_gate_up is not None:
            shared = mix.linear(mix.gated_act(mix.linear(a, lw.shared_gate_up), mix.ACT_SILU), lw.shared_down)
        return mix.moe_input_scaled(a, lw.w13, lw.w2, w, ids, extra=shared, post_norm=post_norm)

    def compute_logits(self, hidden: torch.Tensor, argmax_parts=None) -> torch.Tensor:
        """fp32 logits [rows, vocab] = head(hidden) * logit_scale."""
        if argmax_parts is not None:
            raise ValueError("this head writes no per-tile argmax candidates")
        return mix.linear(hidden, self.lm_head).float() * self.arch.logit_scale
