#!/usr/bin/env python3
"""
Kogerax beside the framework's closest existing models at equal size, random weights, one GPU
(``python bench.py --kogerax-compare`` runs this; the default bench is unchanged).

Served through the same engine (scheduler, paged cache, state slots, runner, hipGraph decode, sampling) beside
Fekolorn, the other family with recurrent state next to windowed attention:

* prefill throughput: ``batch`` prompts of ``prompt`` tokens, prompt tokens / s of the prefill steps;
* decode throughput: ``gen`` tokens per sequence, generated tokens / s of the decode steps;

and the new design's kernels alone beside their like in the other families (events around the op, median of
``iters``), each as a fraction of the roofline that binds it:

* the matrix recurrence with per-token decay (matrix-memory LSTM shape with its normaliser, scalar-decay state-space
  shape) and the selective scan: FLOP/s over the 157 TFLOP/s fp32 vector peak at prefill, state bytes / time over the
  8 TB/s HBM3E peak at decode, beside ``lightning_attn`` and ``gated_delta``;
* windowed rotary attention: matrix FLOP/s over the 2.5 PFLOP/s dense bf16 peak (prefill), cache bytes / time over the
  HBM peak (decode), beside ``attn_prefill`` / ``attn_decode``;
* the row kernels (residual updates behind a norm, pair update, weighted expert sum + norm, convolution, read-out
  epilogues, q/k preparation): bytes moved / time over the HBM peak, beside ``post_norm_residual``,
  ``combine_post_norm``, ``fused_add_rms_norm``, ``delta_prep``, ``norm_sigmoid_gate``.

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
_fc = _sibling("fekolorn_compare")
PEAK_BF16, PEAK_HBM, _time, serve = _dc.PEAK_BF16, _dc.PEAK_HBM, _dc._time, _dc.serve
PEAK_FP32_VALU = 157.3e12

# width; attention heads / key-value heads / head size; matrix-LSTM heads, key and value sizes; state-space heads, head
# size, state, groups; selective scan inner width, state, step-size rank; feed-forward widths; experts
SIZES = {
    "2k": dict(hidden=2048, layers=4, heads=16, kv_heads=4, dim=128, vdim=128, window=1024, conv=4,
               l_heads=16, l_dim=64, l_vdim=128, m_heads=64, m_vdim=64, m_state=128, m_groups=1,
               s_inner=4096, s_state=16, s_rank=128, ff=5504, experts=8, identity=2, top=2, expert_ff=2048,
               shared_ff=2048, vocab=32000, streams=4, llama_ff=5504),
    "4k": dict(hidden=4096, layers=4, heads=32, kv_heads=8, dim=128, vdim=128, window=1024, conv=4,
               l_heads=32, l_dim=64, l_vdim=128, m_heads=128, m_vdim=64, m_state=128, m_groups=1,
               s_inner=8192, s_state=16, s_rank=256, ff=11008, experts=8, identity=2, top=2, expert_ff=4096,
               shared_ff=4096, vocab=32000, streams=4, llama_ff=11008),
}


def kogerax_arch(z):
    from src.models.fekolorn import SinkAttnSpec
    from src.models.kogerax import (GatedMlpSpec, KogeraxArch, KogLayerSpec, MLstmSpec, Mamba2Spec, NormedPairSpec,
                                    SelectiveScanSpec)

    att = SinkAttnSpec(heads=z["heads"], kv_heads=z["kv_heads"], dim=z["dim"], vdim=z["vdim"],
                       scale=1.0 / math.sqrt(z["dim"]), window=z["window"], rot_dims=z["dim"] // 2, rot_base=1e6,
                       rot_scaling=(8.0, 1.0, 4.0, 8192.0), qk_norm=True, head_norm=True, norm_after_rot=True,
                       norm_weights=False, has_sink=False)
    scan = SelectiveScanSpec(inner=z["s_inner"], state=z["s_state"], dt_rank=z["s_rank"], conv=z["conv"])
    lstm = MLstmSpec(heads=z["l_heads"], dim=z["l_dim"], vdim=z["l_vdim"], gate_cap=12.0)
    ssd = Mamba2Spec(heads=z["m_heads"], vdim=z["m_vdim"], state=z["m_state"], groups=z["m_groups"], conv=z["conv"],
                     norm_groups=1)
    dense = GatedMlpSpec("dense", ff=z["ff"])
    moe = GatedMlpSpec("moe", experts=z["experts"], identity=z["identity"], top=z["top"], expert_ff=z["expert_ff"],
                       expert_limit=7.0, shared_ff=z["shared_ff"], shared_limit=7.0)
    kinds = [("mlstm", lstm, dense), ("mamba2", ssd, moe), ("parallel", NormedPairSpec(att, scan), moe),
             ("mlstm", lstm, moe)]
    layers = tuple(KogLayerSpec(*kinds[i % 4]) for i in range(z["layers"]))
    return KogeraxArch("kogerax-bench", z["vocab"], z["hidden"], layers, embed_scale=math.sqrt(z["hidden"]),
                       residual_mult=0.3)


def kernels(z, a, size):
    from src import ops
    from src.ops import lin, mix, rec, seq

    dev, bf = "cuda", torch.bfloat16
    bs, S, L = 16, a.batch, a.prompt
    W = z["hidden"]
    T = S * L
    cu = (torch.arange(S + 1, dtype=torch.int32, device=dev) * L)
    sl = torch.arange(S, dtype=torch.int32, device=dev)
    rags = (("prefill", T, seq.Ragged(torch.arange(L, device=dev).repeat(S), cu, sl)),
            ("decode", S, seq.Ragged(torch.full((S,), L - 1, device=dev), None, sl)))
    res = []

    def emit(r):
        r.update(bench="kernel", size=size)
        res.append(r)
        print(json.dumps(r), flush=True)

    # ---- the matrix recurrence at the two shapes it serves, beside lightning_attn and gated_delta at the first
    for label, H, G, D, V, norm in (("mlstm", z["l_heads"], z["l_heads"], z["l_dim"], z["l_vdim"], True),
                                    ("mamba2", z["m_heads"], z["m_groups"], z["m_state"], z["m_vdim"], False)):
        state = torch.zeros(S + 1, H, D, V, device=dev)
        nst = torch.zeros(S + 1, H, D, device=dev) if norm else None
        C = 2 * G * D + H * V
        for mode, T2, rag in rags:
            x = (torch.randn(T2, C, device=dev) * 0.3).to(bf)
            ab = torch.rand(T2, H, 3, device=dev) * 0.5 + 0.4
            t = _time(lambda: rec.gated_linear_attn(x, 0, G * D, 2 * G * D, ab, state, nst, H, G, D, V, 0.125, rag), a.iters)
            r = {"design": "kogerax", "kernel": f"gated_linear_attn ({label} shape)", "mode": mode, "ms": round(t * 1e3, 4),
                 "valu_fp32_frac_of_peak": round(T2 * H * 4 * D * (V + (1 if norm else 0)) / t / PEAK_FP32_VALU, 4)}
            if mode == "decode":
                r["hbm_frac_of_peak"] = round(S * H * D * V * 8 / t / PEAK_HBM, 4)
            emit(r)
            if label != "mlstm":
                continue
            decay = torch.full((H,), 0.97, device=dev)
            xl = (torch.randn(T2, 2 * H * D + H * V, device=dev) * 0.3).to(bf)
            t = _time(lambda: lin.lightning_attn(xl, 0, H * D, 2 * H * D, decay, state, H, D, V, rag), a.iters)
            r = {"design": "bapivik", "kernel": "lightning_attn", "mode": mode, "ms": round(t * 1e3, 4),
                 "valu_fp32_frac_of_peak": round(T2 * H * 4 * D * V / t / PEAK_FP32_VALU, 4)}
            if mode == "decode":
                r["hbm_frac_of_peak"] = round(S * H * D * V * 8 / t / PEAK_HBM, 4)
            emit(r)
            qkv32 = torch.randn(T2, 2 * H * D + H * V, device=dev) * 0.1
            bg = torch.rand(T2, 2 * H, device=dev)
            gate = torch.randn(T2, H * V, device=dev).to(bf)
            nv = torch.ones(V, device=dev)
            t = _time(lambda: seq.gated_delta(qkv32, bg, gate, nv, 1e-6, state, H, H, D, V, rag), a.iters)
            r = {"design": "fekolorn", "kernel": "gated_delta", "mode": mode, "ms": round(t * 1e3, 4),
                 "valu_fp32_frac_of_peak": round(T2 * H * 6 * D * V / t / PEAK_FP32_VALU, 4)}
            if mode == "decode":
                r["hbm_frac_of_peak"] = round(S * H * D * V * 8 / t / PEAK_HBM, 4)
            emit(r)
    # ---- gates of the matrix-memory LSTM
    H = z["l_heads"]
    mst = torch.zeros(S + 1, H, device=dev)
    ib, fb = torch.zeros(H, device=dev), torch.full((H,), 2.0, device=dev)
    for mode, T2, rag in rags:
        x = torch.randn(T2, 2 * H, device=dev).to(bf)
        t = _time(lambda: rec.exp_gate_scan(x, 0, H, ib, fb, 12.0, mst, H, rag), a.iters)
        emit({"design": "kogerax", "kernel": "exp_gate_scan", "mode": mode, "ms": round(t * 1e3, 4)})
    # ---- selective scan
    I, N, R = z["s_inner"], z["s_state"], z["s_rank"]
    sstate = torch.zeros(S + 1, I, N, device=dev)
    A = -torch.rand(I, N, device=dev) - 0.2
    Dv, dtb = torch.ones(I, device=dev), torch.full((I,), -1.5, device=dev)
    for mode, T2, rag in rags:
        x = (torch.randn(T2, I, device=dev) * 0.5).to(bf)
        dt = torch.randn(T2, I, device=dev).to(bf)
        zz = torch.randn(T2, I, device=dev).to(bf)
        bc = (torch.randn(T2, R + 2 * N, device=dev) * 0.5).to(bf)
        t = _time(lambda: rec.selective_scan(x, dt, dtb, bc, R, R + N, A, Dv, zz, sstate, rag), a.iters)
        r = {"design": "kogerax", "kernel": "selective_scan", "mode": mode, "ms": round(t * 1e3, 4),
             "valu_fp32_frac_of_peak": round(T2 * I * N * 7 / t / PEAK_FP32_VALU, 4)}
        if mode == "decode":
            r["hbm_frac_of_peak"] = round(S * I * N * 8 / t / PEAK_HBM, 4)
        else:
            r["hbm_frac_of_peak"] = round(T2 * I * 8 / t / PEAK_HBM, 4)
        emit(r)
    # ---- convolutions: the state-space layer's (with its step sizes) beside the gated delta rule's preparation
    Hm, C = z["m_heads"], z["m_heads"] * z["m_vdim"] + 2 * z["m_groups"] * z["m_state"]
    taps = z["conv"]
    cst = torch.zeros(S + 1, taps - 1, C, device=dev)
    cw, cb = torch.randn(C, taps, device=dev) * 0.3, torch.zeros(C, device=dev)
    cwt = cw.t().contiguous()
    dtb2, al = torch.zeros(Hm, device=dev), torch.zeros(Hm, device=dev)
    for mode, T2, rag in rags:
        p = torch.randn(T2, C + Hm, device=dev).to(bf)
        t = _time(lambda: rec.conv_silu(p[:, :C], cw, cb, cst, rag, wt=cwt, dt=p[:, C:], dt_bias=dtb2, A_log=al), a.iters)
        emit({"design": "kogerax", "kernel": "conv_silu (+ step sizes)", "mode": mode, "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(T2 * C * 4 / t / PEAK_HBM, 4)})
    Hf, Gf, Df = z["heads"], z["kv_heads"], z["dim"]
    Cf = 2 * Gf * Df + Hf * Df
    fst = torch.zeros(S + 1, taps - 1, Cf, device=dev)
    fw = torch.randn(Cf, taps, device=dev) * 0.3
    fwt = fw.t().contiguous()
    for mode, T2, rag in rags:
        p = torch.randn(T2, Cf + 2 * Hf, device=dev).to(bf)
        t = _time(lambda: seq.delta_prep(p[:, :Cf], p[:, Cf: Cf + Hf], p[:, Cf + Hf:], fw, fst, torch.zeros(Hf, device=dev),
                                         torch.zeros(Hf, device=dev), Hf, Gf, Df, Df, rag, conv_wt=fwt), a.iters)
        emit({"design": "fekolorn", "kernel": "delta_prep", "mode": mode, "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(T2 * Cf * 6 / t / PEAK_HBM, 4)})
    # ---- read-out epilogues beside norm_sigmoid_gate
    H, V = z["l_heads"], z["l_vdim"]
    o32 = torch.randn(T, H * V, device=dev)
    nq, abe = torch.randn(T, H, device=dev), torch.rand(T, H, 3, device=dev)
    gg = torch.randn(T, H * V, device=dev).to(bf)
    nw = torch.ones(H * V, device=dev)
    t = _time(lambda: rec.head_norm_gate(o32, nq, abe, gg, nw, H, V, 1e-6), a.iters)
    emit({"design": "kogerax", "kernel": "head_norm_gate", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * H * V * 8 / t / PEAK_HBM, 4)})
    t = _time(lambda: lin.norm_sigmoid_gate(o32, gg, nw, 1e-6), a.iters)
    emit({"design": "bapivik", "kernel": "norm_sigmoid_gate", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * H * V * 8 / t / PEAK_HBM, 4)})
    Hm, Vm = z["m_heads"], z["m_vdim"]
    om = torch.randn(T, Hm * Vm, device=dev)
    xm, zm = torch.randn(T, Hm * Vm, device=dev).to(bf), torch.randn(T, Hm * Vm, device=dev).to(bf)
    Dm, wm = torch.ones(Hm, device=dev), torch.ones(Hm * Vm, device=dev)
    t = _time(lambda: rec.skip_gate_group_norm(om, xm, Dm, zm, wm, Hm, Vm, 1, 1e-6), a.iters)
    emit({"design": "kogerax", "kernel": "skip_gate_group_norm", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * Hm * Vm * 10 / t / PEAK_HBM, 4)})
    # ---- residual updates
    resid = torch.randn(T, W, device=dev)
    act = torch.empty(T, W, device=dev, dtype=bf)
    y1, y2 = torch.randn(T, W, device=dev).to(bf), torch.randn(T, W, device=dev).to(bf)
    w1, w2 = torch.ones(W, device=dev), torch.ones(W, device=dev)
    wn = torch.zeros(W, device=dev).to(bf)
    t = _time(lambda: rec.pair_post_norm_residual(resid, act, y1, w1, y2, w2, wn, 0.3, 1e-6), a.iters)
    emit({"design": "kogerax", "kernel": "pair_post_norm_residual", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * W * (2 + 2 + 8 + 2) / t / PEAK_HBM, 4)})
    t = _time(lambda: mix.post_norm_residual(resid, y1, wn, 1e-6, True, act=act, mult=0.3), a.iters)
    emit({"design": "kogerax / datatar", "kernel": "post_norm_residual", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * W * (2 + 8 + 2) / t / PEAK_HBM, 4)})
    if ops.native_available():
        r16 = torch.randn(T, W, device=dev).to(bf)
        t = _time(lambda: ops.fused_add_rms_norm(y1, r16, wn, 1e-6), a.iters)
        emit({"design": "llama", "kernel": "fused_add_rms_norm", "mode": "prefill", "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(T * W * 8 / t / PEAK_HBM, 4)})
    K, E = z["top"], z["experts"]
    ys = torch.randn(T * K, W, device=dev).to(bf)
    xx = torch.randn(T, W, device=dev).to(bf)
    wk = torch.rand(T, K, device=dev)
    ids = torch.randint(0, E + z["identity"], (T, K), device=dev, dtype=torch.int32)
    extra, gate = torch.randn(T, W, device=dev).to(bf), torch.rand(T, device=dev)
    kern = mix._kern()
    t = _time(lambda: kern.combine_weighted(None, resid, act, ys, None, xx, wk, ids, E, extra, gate, wn, True, 1e-6, 0.3), a.iters)
    emit({"design": "kogerax", "kernel": "combine_weighted (+ norm + residual)", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * W * (2 * K + 2 + 8 + 2) / t / PEAK_HBM, 4)})
    t = _time(lambda: kern.combine_post_norm(resid, act, ys, None, extra, K, wn, True, 1e-6), a.iters)
    emit({"design": "datatar", "kernel": "combine_post_norm", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * W * (2 * K + 2 + 8 + 2) / t / PEAK_HBM, 4)})
    gu = torch.randn(T, 2 * z["ff"], device=dev).to(bf)
    t = _time(lambda: mix.gated_act(gu, mix.ACT_GELU_TANH), a.iters)
    emit({"design": "kogerax", "kernel": "gated_act (gelu)", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * z["ff"] * 6 / t / PEAK_HBM, 4)})
    t = _time(lambda: mix.gated_act(gu, mix.ACT_CLAMPED, 7.0, 1.702), a.iters)
    emit({"design": "datatar", "kernel": "gated_act (clamped)", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * z["ff"] * 6 / t / PEAK_HBM, 4)})
    # ---- attention: windowed, rotary, per-head norm after the rotation
    H, G, D = z["heads"], z["kv_heads"], z["dim"]
    win = min(z["window"], L)
    nb = S * (L // bs)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(S, L // bs)
    ctx = torch.full((S,), L, dtype=torch.int32, device=dev)
    cache = (torch.randn(nb, bs, G * 2 * D, device=dev) * 0.5).to(bf)
    pairs = S * sum(min(i + 1, win) for i in range(L))
    scale = 1.0 / math.sqrt(D)
    for mode, T2, rag in rags:
        q = (torch.randn(T2, H * D, device=dev) * 0.1).to(bf)
        cuq, mq = (cu, L) if mode == "prefill" else (None, 1)
        t = _time(lambda: seq.sink_attn(q, cache, bt, cuq, ctx, rag.positions, None, None, mq, H, G, D, D, win, scale), a.iters)
        r = {"design": "kogerax", "kernel": "sink_attn (window, no sink)", "mode": mode, "ms": round(t * 1e3, 4)}
        if mode == "prefill":
            r["flops_frac_of_peak"] = round(2 * pairs * H * 2 * D / t / PEAK_BF16, 4)
        else:
            r["hbm_frac_of_peak"] = round(S * win * G * 2 * D * 2 / t / PEAK_HBM, 4)
        emit(r)
    p = torch.randn(T, (H + 2 * G) * D, device=dev).to(bf)
    slots = torch.arange(T, device=dev)
    pos = torch.arange(L, device=dev).repeat(S)
    ones = torch.ones(D, device=dev)
    inv = mix.rope_inv_freq(1e6, D // 2, dev, (8.0, 1.0, 4.0, 8192.0))
    t = _time(lambda: seq.qkv_prep(p[:, : H * D], p[:, H * D: (H + G) * D], p[:, (H + G) * D:], cache, H, G, D, D, pos,
                                   slots, 1e-6, q_norm=ones, k_norm=ones, rot_dims=D // 2, inv_freq=inv, head_norm=True,
                                   norm_after_rot=True), a.iters)
    emit({"design": "kogerax", "kernel": "qkv_prep (rotary, then head norm)", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * ((H + 2 * G) * D * 2 + (H + 2 * G) * D * 2) / t / PEAK_HBM, 4)})
    t = _time(lambda: seq.qkv_prep(p[:, : H * D], p[:, H * D: (H + G) * D], p[:, (H + G) * D:], cache, H, G, D, D, pos,
                                   slots, 1e-6, rot_dims=D // 2, inv_freq=inv, v_unit=True), a.iters)
    emit({"design": "fekolorn", "kernel": "qkv_prep (rotary, unit values)", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * ((H + 2 * G) * D * 2 + (H + 2 * G) * D * 2) / t / PEAK_HBM, 4)})
    if ops.native_available() and D == 128:
        kc = (torch.randn(nb, G, bs, D, device=dev) * 0.5).to(bf)
        vc = (torch.randn(nb, G, bs, D, device=dev) * 0.5).to(bf)
        q = (torch.randn(T, H * D, device=dev) * 0.1).to(bf)
        full_pairs = S * L * (L + 1) / 2
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
    # ---- routing at decode size, both score functions
    xr = torch.randn(S, W, device=dev).to(bf)
    n_route = E + z["identity"]
    router = torch.randn(n_route + 1, W, device=dev).to(bf)
    corr = torch.zeros(n_route, device=dev)
    t = _time(lambda: mix.route_softmax_topk(xr, router, K, n_route, corr, gate_row=True), a.iters)
    emit({"design": "kogerax", "kernel": "route_softmax_topk", "mode": "decode", "ms": round(t * 1e3, 4)})
    t = _time(lambda: mix.route_sigmoid_topk(xr, router[:E].contiguous(), K), a.iters)
    emit({"design": "datatar", "kernel": "route_sigmoid_topk", "mode": "decode", "ms": round(t * 1e3, 4)})
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
    ap.add_argument("--models", default="kogerax,fekolorn", help="which models to serve")
    a = ap.parse_args(argv)
    assert torch.cuda.is_available(), "needs a GPU"
    from src.models.fekolorn import FekolornLM
    from src.models.kogerax import KogeraxLM

    t0 = time.time()
    summary = []
    for size in a.sizes.split(","):
        z = SIZES[size]
        if not a.skip_kernels:
            summary += kernels(z, a, size)
        if a.skip_serving:
            continue
        if "kogerax" in a.models.split(","):
            summary.append(serve(KogeraxLM(kogerax_arch(z), "cuda:0", seed=1, init_std=0.02), a, "kogerax", size))
        if "fekolorn" in a.models.split(","):
            zf = dict(_fc.SIZES["2k"], hidden=z["hidden"], layers=z["layers"], heads=z["heads"], kv_heads=z["kv_heads"],
                      ff=4 * z["hidden"])
            summary.append(serve(FekolornLM(_fc.fekolorn_arch(zf), "cuda:0", seed=1, init_std=0.02), a, "fekolorn", size))
    print(json.dumps({"bench": "kogerax_compare_summary", "seconds": round(time.time() - t0, 1), "rows": summary}),
          flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
