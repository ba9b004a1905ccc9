"""
Kogerax on the serving engine against the plain float64 oracle (tests/kogerax_oracle.py).

Every test makes its own small configuration and random weights, writes them as a checkpoint directory, loads it
through ``LLMEngine.from_pretrained`` (registry -> model class -> loader) and steps it with
``LLMEngine.replay_step`` (scheduler, block manager with state slots, runner, kernels). The CPU cases run the engine's
control flow on the plain-PyTorch op semantics; the ``gpu`` cases run the HIP kernels. Structural faults (a window
one token off, a lost state, a forgotten identity expert) are far above the fp32 tolerance, so those cases run in
fp32; bf16 cases check the served precision.
"""

import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import kogerax_oracle as orc  # noqa: E402

F64 = torch.float64
CPU = pytest.param("cpu", id="cpu")
GPU = pytest.param("cuda:0", marks=pytest.mark.gpu, id="gpu")
DEVICES = [CPU, GPU]
TOL = {torch.float32: 3e-4, torch.bfloat16: 6e-2}
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _need(device):
    if device != "cpu":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        from src.ops import mix

        assert mix.mix_available(), "HIP extension src/_Cmix not loaded"


def save_checkpoint(path, config, weights):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))


def make_engine(tmp_path, config, weights, device, dtype, max_tokens=512, max_seqs=4, block_size=16, name="ckpt",
                capture=False, **cfg_kw):
    from src.config import EngineConfig
    from src.engine import LLMEngine

    path = str(tmp_path / name)
    save_checkpoint(path, config, weights)
    nb = (max_tokens + block_size - 1) // block_size
    kw = dict(max_num_seqs=max_seqs, max_num_batched_tokens=nb * block_size, block_size=block_size, num_kv_blocks=nb,
              enable_prefix_caching=False, use_cuda_graph=False, preemption_mode="recompute", tuned_gemm_table=False,
              decode_window=1)
    kw.update(cfg_kw)
    return LLMEngine.from_pretrained(path, device=device, cfg=EngineConfig(**kw), max_model_len=nb * block_size,
                                     capture=capture, dtype=dtype)


def row_errs(got, want):
    """Per row: rms of the logit difference (mean taken off) over the rms of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-12)


def tokens_for(config, n, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, config["vocab"], (n,), generator=g).tolist()


def replay(eng, steps):
    """steps: list of lists of (request id, tokens, wanted places[, ends]). Returns {rid: {position: logits row}}."""
    got, at = {}, {}
    for step in steps:
        entries, end = [], []
        for e in step:
            rid, toks, want = e[:3]
            entries.append((rid, toks, want))
            if len(e) > 3 and e[3]:
                end.append(rid)
        logits = eng.replay_step(entries, end)
        r = 0
        for rid, toks, want in entries:
            base = at.get(rid, 0)
            for w in want:
                got.setdefault(rid, {})[base + w] = logits[r]
                r += 1
            at[rid] = base + len(toks)
        for rid in end:
            at.pop(rid, None)
        assert r == logits.shape[0]
    return got


def cut(rid, toks, sizes, end=True):
    """One request alone, cut into portions of the given sizes (the rest one token at a time)."""
    steps, lo = [], 0
    sizes = list(sizes)
    while lo < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - lo)
        hi = lo + n
        steps.append([(rid, toks[lo:hi], list(range(n)), end and hi == len(toks))])
        lo = hi
    return steps


def check_against_oracle(got, weights, config, toks, tol, want=None):
    want = orc.forward(config, weights, toks) if want is None else want
    pos = sorted(got)
    if tol >= 1e-2:
        # bf16: positions whose routing rests on a close call at that precision may take another expert
        gaps = orc.routing_margins(config, weights, toks)
        pos = [p for p in pos if float(gaps[p]) > 5e-3]
        assert len(pos) >= max(1, len(got) // 4)
    g = torch.stack([got[p] for p in pos])
    assert torch.isfinite(g).all()
    e = row_errs(g, want[pos])
    if tol >= 1e-2:
        # the typical row is held to the tolerance and no row may be far off (a structural fault moves rows by O(1))
        assert float(e.median()) < tol / 2 and float(e.max()) < 4 * tol, f"median {float(e.median()):.3e} max {float(e.max()):.3e}"
    else:
        assert float(e.max()) < tol, f"relative error {float(e.max()):.3e} >= {tol}"


CONFIGS = {
    # every mixer and both feed-forwards; a layer without feed-forward; groups, parts, key/value heads and dim / vdim
    # all unequal
    "std": lambda: orc.make_config(
        [orc.mlstm_layer(mlp=orc.dense()), orc.mamba2_layer(mlp=orc.moe()),
         orc.parallel_layer(mlp=orc.moe(experts=3, identity=0, top=2, shared_ff=0)), orc.mlstm_layer(heads=4, dim=4, vdim=6),
         orc.parallel_layer(heads=2, kv_heads=1, dim=8, vdim=12, window=21, rot_dims=8, scaling=None, inner=16, state=17,
                            dt_rank=1, conv=2, mlp=orc.dense(24))]),
    # odd sizes, one head, one tap, top 1, only identity experts beside one real one, no window, no rotation, no
    # scaling of the embedding or the residual update
    "odd": lambda: orc.make_config(
        [orc.mamba2_layer(heads=3, vdim=5, state=7, groups=1, conv=1, norm_groups=3, mlp=orc.moe(experts=1, identity=3, top=1, ff=10, shared_ff=6)),
         orc.parallel_layer(heads=3, kv_heads=3, dim=6, vdim=5, window=0, rot_dims=0, inner=9, state=3, dt_rank=2, conv=4,
                            mlp=orc.moe(experts=5, identity=1, top=6, ff=7, shared_ff=0)),
         orc.mlstm_layer(heads=1, dim=10, vdim=7, gate_cap=3.0, mlp=orc.dense(11)),
         orc.mamba2_layer(heads=2, vdim=4, state=5, groups=2, conv=3, norm_groups=1)],
        vocab=53, width=30, eps=1e-6, embed_scale=1.0, residual_mult=1.0),
    # matrix-core shapes: attention heads of 32 / 64, wider recurrent heads
    "mc": lambda: orc.make_config(
        [orc.parallel_layer(heads=4, kv_heads=2, dim=32, vdim=32, window=40, rot_dims=16, rot_base=10000.0,
                            scaling=(3.0, 1.0, 4.0, 64), scale=0.35, inner=64, state=16, dt_rank=4, conv=4, mlp=orc.moe(ff=32)),
         orc.mlstm_layer(heads=2, dim=32, vdim=64, mlp=orc.dense(96)),
         orc.mamba2_layer(heads=4, vdim=32, state=64, groups=1, conv=4, norm_groups=2, mlp=orc.moe(experts=6, identity=3, top=3, ff=32)),
         orc.parallel_layer(heads=2, kv_heads=1, dim=64, vdim=64, window=80, rot_dims=32, scaling=None, scale=0.25,
                            inner=128, state=20, dt_rank=8, conv=2)], vocab=128, width=64),
}


def weights_for(config, seed=0):
    return orc.make_weights(config, seed)


def _rag(device, pos, cu, slots):
    from src.ops import seq

    return seq.Ragged(torch.tensor(pos, device=device), None if cu is None else torch.tensor(cu, dtype=torch.int32, device=device),
                      torch.tensor(slots, dtype=torch.int32, device=device))


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("W", [48, 30, 1032])
def test_embedding_residual_updates_and_gelu(device, W):
    """embed_scaled, post_norm_residual with a multiplier, the pair update and the GELU-gated activation against the
    equations, on vector and scalar paths."""
    _need(device)
    from src.ops import mix, rec

    g = torch.Generator().manual_seed(W)
    T, eps, mult = 5, 1e-5, 0.3
    for dt in (torch.float32, torch.bfloat16):
        tol = 1e-5 if dt == torch.float32 else 2e-2
        d = lambda t: t.to(device)  # noqa: E731
        embed = torch.randn(17, W, generator=g).to(dt)
        ids = torch.randint(0, 17, (T,), generator=g)
        resid, act = rec.embed_scaled(d(ids), d(embed), 2.5)
        want = embed.to(F64)[ids] * 2.5
        assert torch.allclose(resid.cpu().double(), want, atol=1e-6)
        assert (act is resid) == (dt == torch.float32) and torch.allclose(act.cpu().double(), want, atol=tol, rtol=tol)
        y = torch.randn(T, W + 3, generator=g).to(dt)[:, :W]
        w = (0.2 * torch.randn(W, generator=g)).to(dt)
        r0 = torch.randn(T, W, generator=g)
        resid = d(r0.clone())
        a2 = d(torch.zeros(T, W, dtype=dt)) if dt == torch.bfloat16 else None
        mix.post_norm_residual(resid, d(y), d(w), eps, True, act=a2, mult=mult)
        want = r0.to(F64) + mult * orc.rms(y.to(F64), eps) * (1 + w.to(F64))
        assert torch.allclose(resid.cpu().double(), want, atol=1e-5)
        if a2 is not None:
            assert torch.allclose(a2.cpu().double(), want, atol=tol, rtol=tol)
        y2 = torch.randn(T, W + 5, generator=g).to(dt)[:, 5:]
        w1, w2 = 1 + 0.2 * torch.randn(W, generator=g), 1 + 0.2 * torch.randn(W, generator=g)
        resid = d(r0.clone())
        rec.pair_post_norm_residual(resid, a2, d(y), d(w1), d(y2), d(w2), d(w), mult, eps)
        u = 0.5 * (orc.rms(y.to(F64), eps) * w1.to(F64) + orc.rms(y2.to(F64), eps) * w2.to(F64))
        want = r0.to(F64) + mult * orc.rms(u, eps) * (1 + w.to(F64))
        assert torch.allclose(resid.cpu().double(), want, atol=1e-5)
        if a2 is not None:
            assert torch.allclose(a2.cpu().double(), want, atol=tol, rtol=tol)
        gu = (torch.randn(T, 2 * 24, generator=g) * 2).to(dt)
        got = mix.gated_act(d(gu), mix.ACT_GELU_TANH).cpu().double()
        assert torch.allclose(got, orc.gelu_tanh(gu.to(F64)[:, :24]) * gu.to(F64)[:, 24:], atol=tol, rtol=tol)


def _portions_through_mixer(device, mixer, state, xs, portions, slots, eps=1e-5):
    """Feed several sequences' inputs through one mixer in shared steps (``portions``: lists of (sequence, rows));
    returns each sequence's outputs in order."""
    from src.models.llama import AttnMetadata

    at, got = [0] * len(xs), [[] for _ in xs]
    for step in portions:
        rows, pos, cu, sl = [], [], [0], []
        for s, n in step:
            rows.append(xs[s][at[s]: at[s] + n])
            pos += list(range(at[s], at[s] + n))
            cu.append(cu[-1] + n)
            sl.append(slots[s])
        single = all(n == 1 for _, n in step)
        rag = _rag(device, pos, None if single else cu, sl)
        meta = AttnMetadata(is_prefill=not single, slot_mapping=None, block_tables=None, ctx_lens=None)
        y = mixer.forward(torch.cat(rows).to(device), rag.positions, meta, None, eps, state=state, rag=rag)
        y = y.cpu()
        for i, (s, n) in enumerate(step):
            got[s].append(y[cu[i]: cu[i + 1]])
            at[s] += n
    return [torch.cat(g).double() for g in got], at


PORTIONS = [[(0, 5), (1, 1)], [(0, 1)], [(0, 2), (1, 2)], [(1, 6)], [(0, 1), (1, 1)], [(0, 70)], [(1, 3), (0, 2)]]


def _mixer_case(device, kind, spec_cfg, dt=torch.float32, W=24, seed=0):
    """A recurrent mixer alone: two sequences in shared steps, portions down to one token and a portion longer than
    a 64-token trip, in state slots that hold stale content, against the oracle's loop over each whole sequence."""
    from src.models import kogerax as kg

    cls, spec_fn, ofn = {"mlstm": (kg.MLstmMixer, kg._mlstm_spec, orc.mlstm), "mamba2": (kg.Mamba2Mixer, kg._mamba2_spec, orc.mamba2),
                         "scan": (kg.SelectiveScanMixer, kg._scan_spec, lambda h, w, m, eps: orc.selective_scan(h, w, m))}[kind]
    layer = {"mlstm": orc.mlstm_layer, "mamba2": orc.mamba2_layer}.get(kind)
    cfg_layer = layer(**spec_cfg) if layer else {"type": "parallel", "mixer": {"left": orc.parallel_layer()["mixer"]["left"], "right": spec_cfg}, "mlp": None}
    config = orc.make_config([cfg_layer], width=W)
    weights = weights_for(config, seed)
    prefix = "l0.mix." + ("right." if kind == "scan" else "")
    w = {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}
    mcfg = cfg_layer["mixer"]["right"] if kind == "scan" else cfg_layer["mixer"]
    mixer = cls(spec_fn(mcfg), W, device, dt, None, 0.0)
    for k, v in w.items():
        assert mixer.load(k, v) or k == "out", k
    mixer.finalize()
    g = torch.Generator().manual_seed(seed + 5)
    xs = [(torch.randn(n, W, generator=g) * 1.5).to(dt) for n in (81, 14)]
    want = [ofn(x.to(F64), {k: v.to(F64) for k, v in w.items()}, mcfg, 1e-5) for x in xs]
    state = {k: torch.full((4,) + tuple(shape), 7.0, dtype=sdt, device=device) for k, (shape, sdt) in mixer.spec.state_shapes().items()}
    got, at = _portions_through_mixer(device, mixer, state, xs, PORTIONS, [2, 0])
    tol = 2e-4 if dt == torch.float32 else 5e-2
    for s in range(2):
        assert got[s].shape[0] == at[s]
        ref = want[s][: at[s]]
        if dt == torch.float32:
            assert float((got[s] - ref).abs().max()) < tol * float(ref.abs().max()), (kind, s)
        else:   # bf16: a norm over a narrow part of the row magnifies single rounding errors; the whole is held
            assert float((got[s] - ref).pow(2).mean().sqrt()) < tol * float(ref.pow(2).mean().sqrt()), (kind, s)
    for t in state.values():
        if t.numel() == 0:       # a one-tap convolution keeps no tail
            continue
        assert float(t[1].min()) == 7.0 and float(t[3].max()) == 7.0   # other slots untouched


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,V,cap", [(2, 5, 7, 4.0), (3, 16, 16, 15.0), (2, 64, 128, 10.0), (1, 128, 40, 10.0), (1, 24, 150, 8.0)])
def test_mlstm_in_portions(device, H, D, V, cap):
    _need(device)
    _mixer_case(device, "mlstm", dict(heads=H, dim=D, vdim=V, gate_cap=cap), seed=D)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,V,N,G,K,P", [(3, 5, 7, 1, 1, 3), (4, 8, 16, 2, 4, 1), (2, 64, 128, 1, 4, 2), (6, 16, 20, 3, 2, 6)])
def test_mamba2_in_portions(device, H, V, N, G, K, P):
    _need(device)
    _mixer_case(device, "mamba2", dict(heads=H, vdim=V, state=N, groups=G, conv=K, norm_groups=P), seed=N)
    if device != "cpu":
        _mixer_case(device, "mamba2", dict(heads=H, vdim=V, state=N, groups=G, conv=K, norm_groups=P), dt=torch.bfloat16, seed=N)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("I,N,R,K", [(9, 3, 2, 4), (24, 16, 3, 3), (40, 28, 5, 2), (300, 40, 4, 1), (16, 70, 2, 3), (8, 130, 1, 4)])
def test_selective_scan_in_portions(device, I, N, R, K):
    _need(device)
    _mixer_case(device, "scan", dict(inner=I, state=N, dt_rank=R, conv=K), seed=N)
    if device != "cpu":
        _mixer_case(device, "scan", dict(inner=I, state=N, dt_rank=R, conv=K), dt=torch.bfloat16, seed=N)


@pytest.mark.parametrize("device", DEVICES)
def test_gate_scan_keeps_its_maximum_over_long_steps(device):
    """The running maximum of the log gates over a 300-token step equals the token-by-token recursion, with forget
    gates near 0 and near the cap and input gates that overtake the maximum now and then."""
    _need(device)
    from src.ops import rec

    g = torch.Generator().manual_seed(4)
    T, H, cap = 300, 3, 6.0
    x = torch.randn(T, 2 * H + 1, generator=g) * 4
    x[::37, :H] += 9
    ib, fb = torch.randn(H, generator=g), torch.randn(H, generator=g) + 1
    ig = cap * torch.tanh((x[:, :H].to(F64) + ib.to(F64)) / cap)
    fg = orc.logsigmoid(cap * torch.tanh((x[:, H + 1:].to(F64) + fb.to(F64)) / cap))
    m = torch.full((H,), 0.25, dtype=F64)
    want = torch.zeros(T, H, 3, dtype=F64)
    for t in range(T):
        mn = torch.maximum(fg[t] + m, ig[t])
        want[t, :, 0], want[t, :, 1], want[t, :, 2] = torch.exp(fg[t] + m - mn), torch.exp(ig[t] - mn), torch.exp(-mn)
        m = mn
    st = torch.full((3, H), 0.25, device=device)
    rag = _rag(device, list(range(9, 9 + T)), [0, T], [1])
    got = rec.exp_gate_scan(x.to(device), 0, H + 1, ib.to(device), fb.to(device), cap, st, H, rag).cpu().double()
    assert float(((got - want).abs() / (1.0 + want.abs())).max()) < 1e-5
    assert torch.allclose(st[1].cpu().double(), m, atol=1e-5) and float(st[0].max()) == 0.25


def _attention_case(device, dt, impl, n_ctx, q_lo, standout, window, present=True, H=4, G=2, D=32, V=32, R=16, block=16):
    """One sequence of n_ctx tokens whose queries q_lo .. n_ctx - 1 run as one step over scattered pages. The last
    query and the key at ``standout`` carry their weight on the unrotated dimensions and point the same way, so that
    key's score stands far above the others when it is visible; its value is large. Returns (engine ops' output,
    oracle output) for the query rows."""
    from src.ops import mix, seq

    g = torch.Generator().manual_seed(n_ctx * 7 + standout)
    eps, scale = 1e-5, 0.5
    rot = {"base": 100.0, "dims": R, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 40}}
    p = torch.randn(n_ctx, (H + G) * D + G * V, generator=g)
    p[-1].view(-1)[: H * D].view(H, D)[:, R:] = 6.0
    if present:
        p[standout, H * D: (H + G) * D].view(G, D)[:, R:] = 6.0
        p[standout, (H + G) * D:] = 9.0
    p = p.to(dt)
    nb = (n_ctx + block - 1) // block
    perm = torch.randperm(nb + 3, generator=g)[:nb]
    cache = torch.zeros(nb + 3, block, G * (D + V), dtype=dt, device=device)
    pos = torch.arange(n_ctx)
    slots = perm[pos // block] * block + pos % block
    inv = mix.rope_inv_freq(rot["base"], R, device, (8.0, 1.0, 4.0, 40))
    assert torch.allclose(inv.cpu().double(), orc.rotary_frequencies(rot), rtol=1e-6)
    pd = p.to(device)
    ones = torch.ones(D, device=device)
    qr = seq.qkv_prep(pd[:, : H * D], pd[:, H * D: (H + G) * D], pd[:, (H + G) * D:], cache, H, G, D, V, pos.to(device),
                      slots.to(device), eps, q_norm=ones, k_norm=ones, rot_dims=R, inv_freq=inv, head_norm=True,
                      norm_after_rot=True)
    nq = n_ctx - q_lo
    single = nq == 1
    out = seq.sink_attn(qr[q_lo:].contiguous(), cache, perm[None].to(torch.int32).to(device),
                        None if single else torch.tensor([0, nq], dtype=torch.int32, device=device),
                        torch.tensor([n_ctx], dtype=torch.int32, device=device), pos[q_lo:].to(device), None, None,
                        nq, H, G, D, V, window, scale, impl=impl)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale, "rot": rot}
    if window:
        m["mask"] = {"size": window}
    eye = torch.eye(p.shape[1], dtype=F64)
    w = {"q": eye[: H * D], "k": eye[H * D: (H + G) * D], "v": eye[(H + G) * D:], "o": torch.eye(H * V, dtype=F64)}
    want = orc.window_attention(p.to(F64), w, m, eps)[q_lo:]
    return out.cpu().double(), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("where", ["inside", "outside", "far", "page", "first"])
@pytest.mark.parametrize("rows", ["portion", "decode"])
def test_attention_window_edges_and_far_keys(device, where, rows):
    """A key made to stand out just inside / just outside the window, far back without a window, on a page border
    and at position 0, for a prompt portion and for a decode row, over scattered pages; rotary with stretched
    wavelengths, the weightless per-head norm after it. Leaving the key out moves the oracle by much more than the
    tolerance, so a window one token off cannot pass."""
    _need(device)
    n_ctx, window = 300, 37
    standout, win = {"inside": (n_ctx - window, window), "outside": (n_ctx - window - 1, window), "far": (3, 0),
                     "page": (255, 0), "first": (0, 0)}[where]
    q_lo = n_ctx - 1 if rows == "decode" else n_ctx - 45
    cases = [(torch.float32, 1)] if device == "cpu" else [(torch.float32, 1), (torch.bfloat16, 0), (torch.bfloat16, 2)]
    for dt, impl in cases:
        got, want = _attention_case(device, dt, impl, n_ctx, q_lo, standout, win)
        tol = 3e-5 if dt == torch.float32 else 4e-2
        assert float((got - want).abs().max()) < tol * float(want.abs().max()), (dt, impl)
        _, without = _attention_case(device, dt, impl, n_ctx, q_lo, standout, win, present=False)
        moved = float((want[-1] - without[-1]).abs().max())
        if where == "outside":
            assert moved < 1e-9
        else:
            assert moved > 0.5 * float(want.abs().max())   # the key carries the last row's output


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T", [7, 300])
@pytest.mark.parametrize("E,I,K,shared", [(4, 2, 3, True), (1, 3, 1, True), (5, 0, 2, False), (3, 2, 5, False)])
def test_mixture_routing_and_weighted_sum(device, T, E, I, K, shared):
    """Softmax routing with a correction that changes the choice but not the weights, identity experts, the clamped
    expert activation, renormalised weights on the outputs and the gated shared expert, on the decode-sized and the
    prompt-sized paths, against the oracle."""
    _need(device)
    from src.ops import mix

    g = torch.Generator().manual_seed(T + E)
    W, ff, sff, limit = 24, 10, 6, 1.2
    f = orc.moe(experts=E, identity=I, top=K, ff=ff, limit=limit, shared_ff=sff if shared else 0, shared_limit=0.8)
    config = orc.make_config([orc.mlstm_layer(mlp=f)], width=W)
    wts = {k[len("l0.mlp."):]: v for k, v in weights_for(config, E).items() if k.startswith("l0.mlp.")}
    wts["correction"] = torch.randn(E + I, generator=g) * 0.3            # large enough to change choices
    x = torch.randn(T, W, generator=g)
    w64 = {k: v.to(F64) for k, v in wts.items()}
    ids_want, ws_want = orc.route(x.to(F64), w64, f)
    plain = torch.topk(torch.softmax(x.to(F64) @ w64["router"].T, -1), K).indices
    if E + I > K and T > 100:
        assert (ids_want.sort(-1).values != plain.sort(-1).values).any()     # the correction matters here
    want = orc.moe_ff(x.to(F64), w64, f)
    d = lambda t: t.to(device)  # noqa: E731
    router = torch.cat([wts["router"]] + ([wts["shared.sg"]] if shared else []), 0)
    w, ids, gate = mix.route_softmax_topk(d(x), d(router), K, E + I, d(wts["correction"]), gate_row=shared)
    assert torch.equal(ids.cpu().long().sort(-1).values, ids_want.sort(-1).values)
    order = ids.cpu().long().argsort(-1)
    assert torch.allclose(torch.gather(w.cpu().double(), 1, order), torch.gather(ws_want, 1, ids_want.argsort(-1)), atol=1e-5)
    w13 = torch.stack([torch.cat([wts[f"e{e}.gate"], wts[f"e{e}.up"]], 0) for e in range(E)])
    w2 = torch.stack([wts[f"e{e}.down"] for e in range(E)])
    extra = None
    if shared:
        assert torch.allclose(gate.cpu().double(), orc.sigmoid(x.to(F64) @ w64["shared.sg"].T)[:, 0], atol=1e-5)
        gu = torch.nn.functional.linear(d(x), d(torch.cat([wts["shared.gate"], wts["shared.up"]], 0)))
        extra = torch.nn.functional.linear(mix.gated_act(gu, mix.ACT_CLAMPED, 0.8, 1.702), d(wts["shared.down"]))
    out = mix.moe_output_weighted(d(x), d(w13), d(w2), w, ids, mix.ACT_CLAMPED, limit, 1.702, n_route=E + I, extra=extra,
                                  extra_gate=gate)
    assert float((out.cpu().double() - want).abs().max()) < 2e-5 * max(1.0, float(want.abs().max()))
    # the same sum added into a residual behind its norm, in one launch
    resid = d(torch.zeros(T, W))
    nw = d(torch.zeros(W))
    assert mix.moe_output_weighted(d(x), d(w13), d(w2), w, ids, mix.ACT_CLAMPED, limit, 1.702, n_route=E + I, extra=extra,
                                   extra_gate=gate, post_norm=(resid, nw, 1e-5, True, None, 0.5)) is None
    assert torch.allclose(resid.cpu().double(), 0.5 * orc.rms(want, 1e-5), atol=2e-5)


# -------------------------------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_whole_prompt_and_layer_streams(tmp_path, device, name, dtype):
    _need(device)
    config = CONFIGS[name]()
    weights = weights_for(config, 1)
    toks = tokens_for(config, 61, 2)
    eng = make_engine(tmp_path, config, weights, device, dtype)
    got = replay(eng, [[("a", toks, list(range(len(toks))), True)]])
    want, streams = orc.forward(config, weights, toks, keep_layers=True)
    check_against_oracle(got["a"], weights, config, toks, TOL[dtype], want=want)
    if dtype == torch.float32:
        # the residual after every layer, through the model's layer hook
        seen = {}
        orig = eng.model.forward
        eng.model.forward = lambda *a, **k: orig(
            *a, layer_hook=lambda i, x: seen.__setitem__(i, x.detach().cpu().clone()), **k)
        eng.replay_step([("c", toks, [])], ["c"])
        eng.model.forward = orig
        for i in range(len(config["layers"])):
            err = float((seen[i].double() - streams[i]).abs().max() / streams[i].abs().max())
            assert err < 1e-4, f"layer {i}: {err:.2e}"


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_single_token_request(tmp_path, device):
    _need(device)
    config = CONFIGS["std"]()
    weights = weights_for(config, 12)
    eng = make_engine(tmp_path, config, weights, device, torch.float32)
    toks = tokens_for(config, 4, 2)
    got = replay(eng, [[("one", toks[:1], [0], True)]] + cut("a", toks, [1, 1, 2]))
    check_against_oracle(got["one"], weights, config, toks[:1], TOL[torch.float32])
    check_against_oracle(got["a"], weights, config, toks, TOL[torch.float32])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["std", "odd"])
@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 2, 16, 2, 7], [1], [30, 2], [15, 16, 17]], ids=str)
def test_portions_then_token_by_token(tmp_path, device, name, sizes):
    """Prompt portions of several sizes down to two tokens, cut inside pages, windows and convolution tails, then
    single tokens, against the oracle's whole-sequence logits."""
    _need(device)
    config = CONFIGS[name]()
    weights = weights_for(config, 3)
    toks = tokens_for(config, 58, 5)
    eng = make_engine(tmp_path, config, weights, device, torch.float32)
    got = replay(eng, cut("a", toks, sizes))
    assert len(got["a"]) == len(toks)
    check_against_oracle(got["a"], weights, config, toks, TOL[torch.float32])


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_bf16_and_prefill_equals_decode(tmp_path, device):
    """A prompt then 100 single-token steps in bf16 (windows pass over decoded tokens, every recurrent state is
    carried 100 times), and the same positions from one whole-prompt step: both hold the oracle's logits."""
    _need(device)
    config = CONFIGS["mc" if device != "cpu" else "std"]()
    weights = weights_for(config, 4)
    toks = tokens_for(config, 130, 6)
    eng = make_engine(tmp_path, config, weights, device, torch.bfloat16)
    want = orc.forward(config, weights, toks)
    dec = replay(eng, cut("a", toks, [30]))
    check_against_oracle(dec["a"], weights, config, toks, TOL[torch.bfloat16], want=want)
    whole = replay(eng, [[("b", toks, list(range(len(toks))), True)]])
    check_against_oracle(whole["b"], weights, config, toks, TOL[torch.bfloat16], want=want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_unequal_requests_share_steps_pages_and_slots_reused(tmp_path, device, dtype):
    """Six unequal requests, at most four live, in a pool too small for all of them: portions beside single tokens,
    requests sitting out steps, finished requests' pages and state slots handed to later ones. Every request's logits
    equal those of the request alone (the oracle)."""
    _need(device)
    config = CONFIGS["std"]()
    weights = weights_for(config, 5)
    lens = {"a": 70, "b": 33, "c": 1, "d": 47, "e": 64, "f": 18}
    toks = {r: tokens_for(config, n, 10 + i) for i, (r, n) in enumerate(lens.items())}
    eng = make_engine(tmp_path, config, weights, device, dtype, max_tokens=208, max_seqs=4)

    def part(r, lo, hi):
        return (r, toks[r][lo:hi], list(range(hi - lo)), hi == lens[r])

    steps = [[part("a", 0, 17), part("b", 0, 2)], [part("a", 17, 18), part("b", 2, 33), part("c", 0, 1)],
             [part("a", 18, 50), part("d", 0, 16)], [part("d", 16, 17), part("a", 50, 51)],
             [part("a", 51, 52), part("d", 17, 18), part("e", 0, 3)], [part("e", 3, 40), part("d", 18, 47)],
             [part("a", 52, 70), part("e", 40, 41), part("f", 0, 2)], [part("f", 2, 3), part("e", 41, 42)],
             [part("f", 3, 18), part("e", 42, 64)]]
    used_slots, used_blocks = {}, {}
    got = {}
    at = {}
    for step in steps:
        entries = [(r, t, w) for r, t, w, _ in step]
        logits = eng.replay_step(entries, [])
        for r, _, _, _ in step:
            s = eng.seqs[r]
            used_slots[r] = s.state_slot
            used_blocks.setdefault(r, set()).update(s.block_table)
        k = 0
        for r, t, w, _ in step:
            for x in w:
                got.setdefault(r, {})[at.get(r, 0) + x] = logits[k]
                k += 1
            at[r] = at.get(r, 0) + len(t)
        eng.replay_step([], [r for r, _, _, e in step if e])
    assert len(set(used_slots.values())) <= 4 and len(used_slots) == 6      # slots were handed on
    assert used_blocks["e"] & (used_blocks["b"] | used_blocks["c"] | used_blocks["a"])   # and so were pages
    for r in lens:
        assert len(got[r]) == lens[r]
        check_against_oracle(got[r], weights, config, toks[r], TOL[dtype])


def test_oracle_sensitivity():
    """What the engine is checked against moves by far more than the tolerance when a mechanism is altered: the
    window by one token, the stretched wavelengths, where the per-head norm sits in magnitude, a gate cap, a decay, a
    tap, the identity experts, the correction, the shared expert's gate, the multiplier, the first tokens."""
    config = CONFIGS["std"]()
    weights = weights_for(config, 1)
    toks = tokens_for(config, 40, 2)
    base = orc.forward(config, weights, toks)

    def moved(cfg=None, w=None, t=None):
        e = row_errs(orc.forward(cfg or config, w or weights, t or toks), base)
        return float(e[-8:].max())

    def with_entry(i, path, value):
        c = copy.deepcopy(config)
        node = c["layers"][i]
        for k in path[:-1]:
            node = node[k]
        if value is None:
            node.pop(path[-1], None)
        else:
            node[path[-1]] = value
        return c

    floor = 30 * TOL[torch.float32]
    assert moved(with_entry(2, ["mixer", "left", "mask", "size"], 10)) > floor
    assert moved(with_entry(2, ["mixer", "left", "mask", "size"], 8)) > floor
    assert moved(with_entry(2, ["mixer", "left", "rot", "scaling"], None)) > floor
    assert moved(with_entry(2, ["mixer", "left", "scale"], 0.5)) > floor
    assert moved(with_entry(0, ["mixer", "gate_cap"], 2.0)) > floor
    assert moved(with_entry(1, ["mlp", "router", "top"], 2)) > floor
    c = copy.deepcopy(config)
    c["residual_mult"] = 0.5
    assert moved(c) > floor
    c = copy.deepcopy(config)
    c["embedding"]["scale"] = 2.0
    assert moved(c) > floor
    for name in ("l1.mix.A_log", "l1.mix.conv", "l2.mix.right.conv", "l2.mix.right.A_log", "l1.mlp.correction",
                 "l1.mlp.shared.sg", "l0.mix.f.b", "l2.mix.left.out", "l1.mix.D", "l3.mix.norm"):
        w = dict(weights)
        w[name] = torch.flip(weights[name], [-1]) if weights[name].shape[-1] > 1 and name.endswith(("conv", "correction", "out", "norm")) \
            else weights[name] + 1.0
        assert moved(w=w) > floor, name
    # the identity experts: routing their share to a real expert instead changes the result
    w = dict(weights)
    w["l1.mlp.router"] = weights["l1.mlp.router"].clone()
    w["l1.mlp.router"][4:] -= 50.0
    assert moved(w=w) > floor
    # the first tokens reach the last rows through the recurrent state
    assert moved(t=[(toks[0] + 1) % config["vocab"]] + toks[1:]) > floor


# ------------------------------------------------------------------------------------ generation, registry, CLI
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_engine(tmp_path, device):
    """LLMEngine.generate (scheduler, continuous batching on three slots, sampling) continues five prompts as the
    oracle's greedy choice does; on the GPU also from captured decode graphs."""
    _need(device)
    from src.preproc import SamplingParams

    config = CONFIGS["mc" if device != "cpu" else "std"]()
    weights = weights_for(config, 7)
    prompts = [tokens_for(config, n, 20 + n) for n in (5, 1, 19, 33, 8)]
    n_new = 6

    def is_greedy(prompt, out):
        """Every generated token is the oracle's argmax given the tokens before it, or ties with it at the sampler's
        precision (the GPU sampling kernel reads the logits as bf16)."""
        seq_ = list(prompt)
        for tok in out:
            lg = orc.forward(config, weights, seq_)[-1]
            slack = 1e-3 * float(lg.std()) if device == "cpu" else 2.0 ** -7 * float(lg.abs().max())
            if float(lg[tok]) < float(lg.max()) - slack:
                return False
            seq_.append(tok)
        return len(out) == n_new

    modes = [dict(capture=False)]
    if device != "cpu":
        modes.append(dict(capture=True, use_cuda_graph=True, graph_batch_sizes=[1, 2, 4], decode_window=4))
    for i, kw in enumerate(modes):
        eng = make_engine(tmp_path, config, weights, device, torch.float32, max_seqs=3, name=f"g{i}", **kw)
        eng.eos_token_id = None
        outs = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0))
        assert all(is_greedy(p, o) for p, o in zip(prompts, outs)), (kw, outs)


def test_registry_config_roundtrip(tmp_path):
    from src.models.kogerax import KogeraxArch, KogeraxLM
    from src.models.registry import family_of, resolve

    config = CONFIGS["std"]()
    path = str(tmp_path / "ckpt")
    save_checkpoint(path, config, weights_for(config))
    assert family_of(path) == "kogerax"
    name, arch, cls = resolve(path)
    assert cls is KogeraxLM and arch.num_layers == len(config["layers"])
    assert arch.to_config() == json.loads(json.dumps(config))
    model = cls(arch, "cpu", dtype=torch.float32)
    assert model.needs_seq_state and not model.supports_prefix_cache
    widths = [l.mixer.cache_width for l in arch.layers]
    assert widths == [0, 0, 2 * (16 + 8), 0, 1 * (8 + 12)]
    from safetensors.torch import load_file

    n = model.load_state_dict(load_file(os.path.join(path, "model.safetensors")))
    assert n == len(orc.tensor_shapes(config))
    model.save(str(tmp_path / "again"))
    again = load_file(str(tmp_path / "again" / "model.safetensors"))
    for k, v in weights_for(config).items():
        assert torch.equal(again[k].float().reshape(v.shape), v.float()), k
    for bad in (dict(type="lightning"), ):
        c = copy.deepcopy(config)
        c["layers"][0].update(bad)
        with pytest.raises(ValueError):
            KogeraxArch.from_config(c)
    c = copy.deepcopy(config)
    c["layers"][1]["mlp"]["router"]["top"] = 9
    with pytest.raises(ValueError):
        KogeraxArch.from_config(c)


@pytest.mark.parametrize("device", DEVICES)
def test_trace_runner_command_line(tmp_path, device):
    _need(device)
    config = CONFIGS["std"]()
    weights = weights_for(config, 9)
    path = str(tmp_path / "ckpt")
    save_checkpoint(path, config, weights)
    toks = tokens_for(config, 21, 1)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:12], "want": [0, 11]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[12:13], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[13:], "want": [7]}], "end": ["x"]}]
    out = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", out,
           "--max-tokens", "64", "--device", device]
    r = subprocess.run(cmd, input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=600, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np

    want = orc.forward(config, weights, toks)
    a = torch.from_numpy(np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(2, -1))
    b = torch.from_numpy(np.fromfile(os.path.join(out, "2.f32"), dtype="<f4").reshape(1, -1))
    assert not os.path.exists(os.path.join(out, "1.f32"))
    assert float(row_errs(torch.cat([a, b]), want[[0, 11, 20]]).max()) < TOL[torch.float32]
