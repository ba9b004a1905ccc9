#!/usr/bin/env python3
"""
Bapivik beside the framework's closest existing model (Llama: dense feed-forward, paged GQA attention) at equal
size, random weights, one GPU (``python bench.py --bapivik-compare`` runs this; the default bench is unchanged).

Per size, for both models through the same engine (scheduler, paged cache, state slots, runner, hipGraph decode,
sampling):

* prefill throughput: ``batch`` prompts of ``prompt`` tokens, prompt tokens / s of the prefill steps;
* decode throughput: ``gen`` tokens per sequence, generated tokens / s of the decode steps;

and for the new design's kernels alone beside their like in the Llama path (events around the op, median of
``iters``), each as a fraction of the roofline that binds it:

* windowed attention with capped scores and distance slopes, and latent attention without a rotary part, prefill
  (matrix FLOP/s over the 2.5 PFLOP/s dense bf16 peak, FLOPs over the visible (query, key) pairs) and decode (cache
  bytes read / time over the 8 TB/s HBM3E peak), beside ``attn_prefill`` / ``attn_decode``;
* the sublayer-boundary and layer-boundary norm launches, the squared-ReLU activation, the q/k preparation and the
  output gates (memory-bound: bytes moved / time over the HBM peak), beside ``fused_add_rms_norm`` / ``silu_and_mul``;
* decayed linear attention (a sequential recurrence on the vector ALUs; at decode bound by the state's HBM traffic):
  FLOP/s over the 157 TFLOP/s fp32 vector peak, beside the framework's other recurrence, ``gated_delta``.

Prints one JSON line per measurement and a final summary line.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def _sibling(name):
    """A module of this folder by file (the folder shares its name with bench.py and is no package)."""
    import importlib.util

    spec = importlib.util.spec_from_file_location(name, os.path.join(ROOT, "bench", name + ".py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


_dc = _sibling("design_compare")
PEAK_BF16, PEAK_HBM, _time, serve = _dc.PEAK_BF16, _dc.PEAK_HBM, _dc._time, _dc.serve

PEAK_FP32_VALU = 157.3e12

# hidden, layers (latent, a layer on its latents, windowed attention, lightning: repeated), heads, head sizes, widths
SIZES = {
    "2k": dict(hidden=2048, layers=4, heads=16, kv_heads=4, dim=128, vdim=128, kv_rank=256, q_rank=768, ff=8192,
               llama_ff=5504, vocab=32000, window=1024),
    "4k": dict(hidden=4096, layers=4, heads=32, kv_heads=8, dim=128, vdim=128, kv_rank=256, q_rank=1536, ff=16384,
               llama_ff=11008, vocab=32000, window=1024),
}


def bapivik_arch(z):
    from src.models.bapivik import SLOPE_EXP, BapivikArch, BapLayerSpec, LightningSpec, ReluSqMlpSpec
    from src.models.datatar import LatentAttnSpec
    from src.models.fekolorn import SinkAttnSpec

    H, D = z["heads"], z["dim"]
    scale = 1.0 / math.sqrt(D)

    def latent(kv_from=None):
        return LatentAttnSpec(heads=H, dim=D, rot_dim=0, vdim=z["vdim"], kv_rank=z["kv_rank"], q_rank=z["q_rank"],
                              scale=scale, window=0, rot_base=10000.0, rot_dims=0, has_sink=False, out_gate=True,
                              kv_from=kv_from)

    att = SinkAttnSpec(heads=H, kv_heads=z["kv_heads"], dim=D, vdim=D, scale=scale, window=z["window"], qk_norm=True,
                       has_sink=False, head_norm=True, v_from_k=True, softcap=30.0, slope_exp=SLOPE_EXP,
                       q_temp_coef=0.2, q_temp_every=256)
    decay = tuple(math.exp(-2.0 ** -(2 + 6 * i / max(1, H - 1))) for i in range(H))
    li = LightningSpec(heads=H, dim=D, vdim=z["vdim"], decay=decay)
    mlp = ReluSqMlpSpec(z["ff"])
    layers = []
    for i in range(z["layers"]):
        k = i % 4
        if k == 0:
            layers.append(BapLayerSpec("latent_attention", latent(), mlp))
        elif k == 1:
            layers.append(BapLayerSpec("latent_attention", latent(kv_from=i - 1), mlp))
        elif k == 2:
            layers.append(BapLayerSpec("attention", att, mlp))
        else:
            layers.append(BapLayerSpec("lightning", li, mlp))
    return BapivikArch("bapivik-bench", z["vocab"], z["hidden"], tuple(layers), logit_softcap=30.0, max_position=2048)


def llama_arch(z):
    from src.models.presets import ArchConfig

    return ArchConfig("llama-bench", z["hidden"], z["layers"], z["heads"], z["kv_heads"], z["llama_ff"], z["vocab"],
                      rope_theta=1e6, max_position=8192)


def kernels(z, a, size):
    from src import ops
    from src.ops import lin, mix, seq

    dev, bf = "cuda", torch.bfloat16
    bs, S, L = 16, a.batch, a.prompt
    H, G, D, DV, W = z["heads"], z["kv_heads"], z["dim"], z["vdim"], z["hidden"]
    R = z["kv_rank"]
    win = min(z["window"], L)
    nb = S * (L // bs)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(S, L // bs)
    ctx = torch.full((S,), L, dtype=torch.int32, device=dev)
    cu = (torch.arange(S + 1, dtype=torch.int32, device=dev) * L)
    pairs = S * sum(min(i + 1, win) for i in range(L))
    res = []

    def emit(r):
        r.update(bench="kernel", size=size)
        res.append(r)
        print(json.dumps(r), flush=True)

    scale = 1.0 / math.sqrt(D)
    steps = (("prefill", S * L, torch.arange(L, device=dev).repeat(S), cu, L),
             ("decode", S, torch.full((S,), L - 1, device=dev), None, 1))
    # windowed attention: values = keys, capped scores, distance slopes
    cache = (torch.randn(nb, bs, G * 2 * D, device=dev) * 0.5).to(bf)
    slopes = torch.pow(2.0, -8.0 * torch.arange(1, H + 1, dtype=torch.float64) / H).float().to(dev)
    for mode, T, pos, cuq, mq in steps:
        q = (torch.randn(T, H * D, device=dev) * 0.1).to(bf)
        for label, cap, sl in (("sink_attn", 0.0, None), ("sink_attn+cap+slopes", 30.0, slopes)):
            t = _time(lambda: seq.sink_attn(q, cache, bt, cuq, ctx, pos, None, None, mq, H, G, D, D, win, scale,
                                            softcap=cap, slopes=sl), a.iters)
            r = {"design": "bapivik", "kernel": label, "mode": mode, "ms": round(t * 1e3, 4)}
            if mode == "prefill":
                r["flops_frac_of_peak"] = round(2 * pairs * H * 2 * D / t / PEAK_BF16, 4)
            else:
                r["hbm_frac_of_peak"] = round(S * win * G * 2 * D * 2 / t / PEAK_HBM, 4)
            emit(r)
    # latent attention in its absorbed form: score width and value width kv_rank, no rotary part, no sink
    lcache = (torch.randn(nb, bs, R, device=dev) * 0.5).to(bf)
    inv = mix.rope_inv_freq(10000.0, 0, dev)
    full_pairs = S * L * (L + 1) / 2
    for mode, T, pos, cuq, mq in steps:
        q_lat = (torch.randn(H, T, R, device=dev) * 0.1).to(bf)
        qd = (torch.randn(T, H * D, device=dev) * 0.1).to(bf)
        t = _time(lambda: mix.latent_attn(q_lat, qd, D, lcache, bt, cuq, ctx, pos, None, mq, 0, scale, 0, inv), a.iters)
        r = {"design": "bapivik", "kernel": "latent_attn", "mode": mode, "ms": round(t * 1e3, 4)}
        if mode == "prefill":
            r["flops_frac_of_peak"] = round(2 * full_pairs * H * 2 * R / t / PEAK_BF16, 4)
        else:
            r["hbm_frac_of_peak"] = round(S * L * R * 2 / t / PEAK_HBM, 4)
        emit(r)
    if ops.native_available() and D == 128:
        kc = (torch.randn(nb, G, bs, D, device=dev) * 0.5).to(bf)
        vc = (torch.randn(nb, G, bs, D, device=dev) * 0.5).to(bf)
        q = (torch.randn(S * L, H * D, device=dev) * 0.1).to(bf)
        t = _time(lambda: ops.attn_prefill(q, kc, vc, bt, cu, ctx, L, H, G, scale), a.iters)
        emit({"design": "llama", "kernel": "attn_prefill", "mode": "prefill", "ms": round(t * 1e3, 4),
              "flops_frac_of_peak": round(2 * full_pairs * H * 2 * D / t / PEAK_BF16, 4)})
        maxp = ops.decode_partials(L)
        part_o = torch.empty(S * H * maxp * 128, dtype=torch.float32, device=dev)
        part_ml = torch.empty(S * H * maxp * 2, dtype=torch.float32, device=dev)
        cnt = torch.zeros(S * G, dtype=torch.int32, device=dev)
        qd = (torch.randn(S, H * D, device=dev) * 0.1).to(bf)
        t = _time(lambda: ops.attn_decode(qd, kc, vc, bt, ctx, L, H, G, scale, part_o=part_o, part_ml=part_ml,
                                          counters=cnt), a.iters)
        emit({"design": "llama", "kernel": "attn_decode", "mode": "decode", "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(S * L * G * D * 2 * 2 / t / PEAK_HBM, 4)})

    # memory-bound row kernels at prompt size
    T = S * L
    n = z["layers"] + 1
    planes = torch.randn(n + 1, T, W, device=dev)
    y = torch.randn(T, W, device=dev).to(bf)
    yb = torch.randn(W, device=dev).to(bf)
    g1, g2 = torch.ones(W, device=dev), torch.ones(W, device=dev)
    t = _time(lambda: lin.post_pre_norm(planes[1], y, None, g1, g2, 1e-6, bf), a.iters)
    emit({"design": "bapivik", "kernel": "post_pre_norm", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * W * (2 + 8 + 2) / t / PEAK_HBM, 4)})
    dw = torch.full((n,), 1.0 / n, device=dev)
    t = _time(lambda: lin.depth_avg_norm(planes, n, dw, y, yb, g1, g2, 1e-6, bf), a.iters)
    emit({"design": "bapivik", "kernel": f"depth_avg_norm ({n} planes)", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * W * (2 + 4 * n + 4 + 4 + 2) / t / PEAK_HBM, 4)})
    if ops.native_available():
        r32 = torch.randn(T, W, device=dev).to(bf)
        wn = torch.ones(W, device=dev).to(bf)
        t = _time(lambda: ops.fused_add_rms_norm(y, r32, wn, 1e-6), a.iters)
        emit({"design": "llama", "kernel": "fused_add_rms_norm", "mode": "prefill", "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(T * W * 8 / t / PEAK_HBM, 4)})
    zf = torch.randn(T, z["ff"], device=dev).to(bf)
    bb = torch.randn(z["ff"], device=dev).to(bf)
    t = _time(lambda: lin.bias_relu2(zf, bb), a.iters)
    emit({"design": "bapivik", "kernel": "bias_relu2", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * z["ff"] * 4 / t / PEAK_HBM, 4)})
    if ops.native_available():
        gu = torch.randn(T, 2 * z["llama_ff"], device=dev).to(bf)
        t = _time(lambda: ops.silu_and_mul(gu), a.iters)
        emit({"design": "llama", "kernel": "silu_and_mul", "mode": "prefill", "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(T * z["llama_ff"] * 6 / t / PEAK_HBM, 4)})
    p = torch.randn(T, (H + G) * D, device=dev).to(bf)
    nq = H * D
    slots = torch.arange(T, device=dev)
    pos = torch.arange(L, device=dev).repeat(S)
    qn, kn = torch.ones(D, device=dev), torch.ones(D, device=dev)
    t = _time(lambda: seq.qkv_prep(p[:, :nq], p[:, nq:], None, cache, H, G, D, D, pos, slots, 1e-6, q_norm=qn,
                                   k_norm=kn, head_norm=True, q_temp_coef=0.2, q_temp_every=256), a.iters)
    emit({"design": "bapivik", "kernel": "qkv_prep (head norm, v = k)", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * ((H + G) * D * 2 + (H + 2 * G) * D * 2) / t / PEAK_HBM, 4)})
    oh = torch.randn(H, T, DV, device=dev).to(bf)
    gt = torch.randn(T, H, device=dev).to(bf)
    t = _time(lambda: lin.head_gate(oh, gt), a.iters)
    emit({"design": "bapivik", "kernel": "head_gate", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * H * DV * 4 / t / PEAK_HBM, 4)})
    o32 = torch.randn(T, H * DV, device=dev)
    gg = torch.randn(T, H * DV, device=dev).to(bf)
    nw = torch.ones(H * DV, device=dev)
    t = _time(lambda: lin.norm_sigmoid_gate(o32, gg, nw, 1e-6), a.iters)
    emit({"design": "bapivik", "kernel": "norm_sigmoid_gate", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * H * DV * 8 / t / PEAK_HBM, 4)})

    # the recurrences: decayed linear attention beside the gated delta rule
    state = torch.zeros(S + 1, H, D, DV, device=dev)
    sl = torch.arange(S, dtype=torch.int32, device=dev)
    decay = torch.full((H,), 0.97, device=dev)
    C = 2 * H * D + H * DV
    for mode, T2, rag in (("prefill", S * L, seq.Ragged(torch.arange(L, device=dev).repeat(S), cu, sl)),
                          ("decode", S, seq.Ragged(torch.full((S,), L - 1, device=dev), None, sl))):
        x = (torch.randn(T2, C, device=dev) * 0.5).to(bf)
        t = _time(lambda: lin.lightning_attn(x, 0, H * D, 2 * H * D, decay, state, H, D, DV, rag), a.iters)
        r = {"design": "bapivik", "kernel": "lightning_attn", "mode": mode, "ms": round(t * 1e3, 4),
             "valu_fp32_frac_of_peak": round(T2 * H * 4 * D * DV / t / PEAK_FP32_VALU, 4)}
        if mode == "decode":
            r["hbm_frac_of_peak"] = round(S * H * D * DV * 8 / t / PEAK_HBM, 4)
        emit(r)
        Cg = 2 * G * D + H * DV
        qkv32 = torch.randn(T2, Cg, device=dev) * 0.1
        bg = torch.rand(T2, 2 * H, device=dev)
        gate = torch.randn(T2, H * DV, device=dev).to(bf)
        nv = torch.ones(DV, device=dev)
        t = _time(lambda: seq.gated_delta(qkv32, bg, gate, nv, 1e-6, state, H, G, D, DV, rag), a.iters)
        r = {"design": "fekolorn", "kernel": "gated_delta", "mode": mode, "ms": round(t * 1e3, 4),
             "valu_fp32_frac_of_peak": round(T2 * H * 6 * D * DV / t / PEAK_FP32_VALU, 4)}
        if mode == "decode":
            r["hbm_frac_of_peak"] = round(S * H * D * DV * 8 / t / PEAK_HBM, 4)
        emit(r)
    return res


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--sizes", default=",".join(SIZES))
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--prompt", type=int, default=1024)
    ap.add_argument("--gen", type=int, default=64)
    ap.add_argument("--steps", type=int, default=2)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--skip-serving", action="store_true")
    ap.add_argument("--skip-kernels", action="store_true")
    ap.add_argument("--models", default="bapivik,llama", help="which models to serve")
    a = ap.parse_args(argv)
    assert torch.cuda.is_available(), "needs a GPU"
    from src.models.bapivik import BapivikLM
    from src.models.llama import CausalLM

    t0 = time.time()
    summary = []
    for size in a.sizes.split(","):
        z = SIZES[size]
        if not a.skip_kernels:
            summary += kernels(z, a, size)
        if a.skip_serving:
            continue
        if "bapivik" in a.models.split(","):
            summary.append(serve(BapivikLM(bapivik_arch(z), "cuda:0", seed=1, init_std=0.02), a, "bapivik", size))
        if "llama" in a.models.split(","):
            summary.append(serve(CausalLM(llama_arch(z), "cuda:0", seed=1), a, "llama", size))
    print(json.dumps({"bench": "bapivik_compare_summary", "seconds": round(time.time() - t0, 1), "rows": summary}),
          flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
