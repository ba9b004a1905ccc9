"""
Bapivik on the serving engine against the plain float64 oracle (tests/bapivik_oracle.py).

Every test makes its own small configuration and random weights, writes them as a checkpoint directory, loads it
through ``LLMEngine.from_pretrained`` (registry -> model class -> loader) and steps it with
``LLMEngine.replay_step`` (scheduler, block manager with state slots, runner, kernels). The CPU cases run the engine's
control flow on the plain-PyTorch op semantics; the ``gpu`` cases run the HIP kernels. Structural faults (a window
one token off, a lost state, the wrong layer's latents) are far above the fp32 tolerance, so those cases run in fp32;
bf16 cases check the served precision.
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
import bapivik_oracle as orc  # noqa: E402

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
    g = torch.stack([got[p] for p in pos])
    assert torch.isfinite(g).all()
    e = row_errs(g, want[pos])
    if tol >= 1e-2:
        # bf16 on models this narrow: the typical row is held to the tolerance and no row may be far off (a
        # structural fault moves rows by O(1))
        assert float(e.median()) < tol / 2 and float(e.max()) < 4 * tol, f"median {float(e.median()):.3e} max {float(e.max()):.3e}"
    else:
        assert float(e.max()) < tol, f"relative error {float(e.max()):.3e} >= {tol}"


def std_layers():
    """latent, a layer on its latents, windowed attention, lightning without feed-forward, a second latent group whose
    follower is not adjacent."""
    return [orc.latent_layer(), orc.latent_layer(kv_from=0, heads=2, dim=8, vdim=16, q_rank=16),
            orc.attn_layer(window=9, softcap=6.0, q_temp=(0.4, 5)), orc.lightning_layer(),
            orc.latent_layer(kv_rank=16, heads=3, vdim=8), orc.attn_layer(heads=4, kv_heads=4, window=21, ff=0),
            orc.latent_layer(kv_from=4, kv_rank=16)]


CONFIGS = {
    "std": lambda: orc.make_config(std_layers()),
    # lightning first and with a feed-forward, one key/value head, one head, no cap / temperature / window, no logit
    # cap, a temperature step of one token, odd sizes
    "odd": lambda: orc.make_config(
        [orc.lightning_layer(heads=2, dim=5, vdim=7, decay=[1.0, 0.5], ff=20),
         orc.attn_layer(heads=3, kv_heads=1, dim=6, ff=0), orc.attn_layer(heads=1, kv_heads=1, dim=10, q_temp=(0.7, 1)),
         orc.latent_layer(heads=1, dim=6, vdim=5, kv_rank=7, q_rank=3, ff=0),
         orc.latent_layer(heads=5, dim=4, vdim=6, kv_rank=7, q_rank=9, kv_from=3)],
        vocab=53, width=30, logit_softcap=0.0, eps=1e-6),
    # matrix-core shapes: head sizes 32 / 64, latents of 64
    "mc": lambda: orc.make_config(
        [orc.attn_layer(heads=4, kv_heads=2, dim=32, window=40, softcap=10.0, q_temp=(0.3, 16), ff=96),
         orc.latent_layer(heads=4, dim=32, vdim=32, kv_rank=64, q_rank=32, ff=96),
         orc.lightning_layer(heads=2, dim=32, vdim=64),
         orc.latent_layer(heads=2, dim=16, vdim=64, kv_rank=64, q_rank=32, kv_from=1, ff=0),
         orc.attn_layer(heads=2, kv_heads=1, dim=64, ff=96)], vocab=128, width=64),
    "attn_only": lambda: orc.make_config([orc.attn_layer(window=7), orc.attn_layer(window=0, softcap=3.0)]),
}


def weights_for(config, seed=0):
    return orc.random_weights(config, seed)


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("W", [48, 30, 1030])
def test_embedding_and_boundary_norms(device, W):
    """embed_pos, post_pre_norm and depth_avg_norm against the equations, on vector and scalar paths, with and without
    a bias / a second norm / weights."""
    _need(device)
    from src.ops import lin

    g = torch.Generator().manual_seed(W)
    T, n, eps = 5, 4, 1e-5
    for dt in (torch.float32, torch.bfloat16):
        embed = torch.randn(17, W, generator=g).to(dt)
        pos = torch.randn(40, W, generator=g).to(dt)
        ids = torch.randint(0, 17, (T,), generator=g)
        pp = torch.tensor([0, 1, 39, 7, 7])
        planes = torch.zeros(n + 1, T, W)
        planes[: n - 1] = torch.randn(n - 1, T, W, generator=g)
        y = torch.randn(T, W + 3, generator=g).to(dt)[:, :W]            # a strided view
        yb = torch.randn(W, generator=g).to(dt)
        w_post, w_pre = 1 + 0.2 * torch.randn(W, generator=g), 1 + 0.2 * torch.randn(W, generator=g)
        dw = torch.randn(n, generator=g)
        tol = 1e-5 if dt == torch.float32 else 2e-2
        d = lambda t: t.to(device)  # noqa: E731
        out = torch.empty(T, W, device=device)
        lin.embed_pos(d(ids), d(pp), d(embed), d(pos), out)
        want0 = embed.to(F64)[ids] + pos.to(F64)[pp]
        assert torch.allclose(out.cpu().double(), want0, atol=1e-6)
        # a norm after one sublayer and before the next
        resid = d(planes[n - 2].clone())
        h = lin.post_pre_norm(resid, d(y), d(yb), d(w_post), d(w_pre), eps, dt)
        r_want = planes[n - 2].to(F64) + orc.rms(y.to(F64) + yb.to(F64), w_post.to(F64), eps)
        assert torch.allclose(resid.cpu().double(), r_want, atol=1e-5)
        assert torch.allclose(h.cpu().double(), orc.rms(r_want, w_pre.to(F64), eps), atol=tol, rtol=tol)
        resid2 = d(planes[n - 2].clone())
        assert lin.post_pre_norm(resid2, d(y), None, d(w_post), None, eps, None) is None
        assert torch.allclose(resid2.cpu().double(),
                              planes[n - 2].to(F64) + orc.rms(y.to(F64), w_post.to(F64), eps), atol=1e-5)
        # the layer boundary: last post-norm + weighted average + next norm
        pl = d(planes.clone())
        pl[n - 1] = d(planes[n - 2])
        h = lin.depth_avg_norm(pl, n, d(dw), d(y), d(yb), d(w_post), d(w_pre), eps, dt)
        assert torch.allclose(pl[n - 1].cpu().double(), r_want, atol=1e-5)
        avg = sum(dw[j].double() * (planes[j].to(F64) if j < n - 1 else r_want) for j in range(n))
        assert torch.allclose(pl[n].cpu().double(), avg, atol=1e-5)
        assert torch.allclose(h.cpu().double(), orc.rms(avg, w_pre.to(F64), eps), atol=tol, rtol=tol)
        # without a sublayer output and without weights: a copy and a norm
        pl = d(planes.clone())
        h = lin.depth_avg_norm(pl, 1, None, None, None, None, d(w_pre), eps, dt)
        assert torch.equal(pl[1], pl[0])
        assert torch.allclose(h.cpu().double(), orc.rms(planes[0].to(F64), w_pre.to(F64), eps), atol=tol, rtol=tol)


@pytest.mark.parametrize("device", DEVICES)
def test_activation_and_gates(device):
    _need(device)
    from src.ops import lin

    g = torch.Generator().manual_seed(3)
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        for n in (24, 13):
            z, b = torch.randn(7, n, generator=g).to(dt), torch.randn(n, generator=g).to(dt)
            got = lin.bias_relu2(z.to(device), b.to(device)).cpu().double()
            assert torch.allclose(got, torch.relu(z.to(F64) + b.to(F64)) ** 2, atol=tol, rtol=tol)
        z = (torch.randn(5, 19, generator=g) * 20).to(dt)
        got = lin.tanh_cap(z.to(device), 7.5).cpu()
        assert got.dtype == torch.float32
        assert torch.allclose(got.double(), 7.5 * torch.tanh(z.to(F64) / 7.5), atol=1e-5, rtol=1e-5)
        H, T, v = 3, 6, 5
        o = torch.randn(H, T, v, generator=g).to(dt)
        gt = torch.randn(T, H + 4, generator=g).to(dt)
        got = lin.head_gate(o.to(device), gt.to(device)[:, 2: 2 + H]).cpu().double()
        want = (o.to(F64).transpose(0, 1) * orc.sigmoid(gt.to(F64)[:, 2: 2 + H])[:, :, None]).reshape(T, H * v)
        assert torch.allclose(got, want, atol=tol, rtol=tol)
        o32 = torch.randn(T, 20, generator=g)
        gg = torch.randn(T, 31, generator=g).to(dt)
        w = 1 + 0.1 * torch.randn(20, generator=g)
        got = lin.norm_sigmoid_gate(o32.to(device), gg.to(device)[:, 11:], w.to(device), 1e-5).cpu().double()
        want = orc.rms(o32.to(F64), w.to(F64), 1e-5) * orc.sigmoid(gg.to(F64)[:, 11:])
        assert torch.allclose(got, want, atol=tol, rtol=tol)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,V", [(2, 5, 7), (3, 16, 16), (2, 64, 128), (1, 128, 64)])
def test_lightning_recurrence_in_portions(device, H, D, V):
    """The recurrence cut into portions down to one token, two sequences sharing steps in slots that hold stale
    content, against the oracle's loop over the whole sequences; decays of 1 and near 0 included."""
    _need(device)
    from src.ops import lin, seq

    g = torch.Generator().manual_seed(D)
    decay = [1.0, 0.05, 0.9][:H] if H <= 3 else [0.9] * H
    C = 2 * H * D + H * V
    lens = [23, 9]
    xs = [torch.randn(n, C + 3, generator=g) * 1.5 for n in lens]
    want = []
    for x in xs:
        q, k = orc.silu(x[:, :H * D].to(F64)).view(-1, H, D), orc.silu(x[:, H * D: 2 * H * D].to(F64)).view(-1, H, D)
        v = orc.silu(x[:, 2 * H * D: C].to(F64)).view(-1, H, V)
        o = torch.zeros(x.shape[0], H, V, dtype=F64)
        for h in range(H):
            S = torch.zeros(D, V, dtype=F64)
            for t in range(x.shape[0]):
                S = decay[h] * S + torch.outer(k[t, h], v[t, h])
                o[t, h] = S.T @ q[t, h]
        want.append(o.reshape(-1, H * V))
    state = torch.full((4, H, D, V), 7.0, device=device)       # stale content everywhere
    dec = torch.tensor(decay, dtype=torch.float32, device=device)
    slots = [2, 0]
    portions = [[(0, 5), (1, 1)], [(0, 1)], [(0, 2), (1, 2)], [(1, 6)], [(0, 15)]]
    at, got = [0, 0], [[], []]
    for step in portions:
        rows, pos, cu, sl = [], [], [0], []
        for s, n in step:
            rows.append(xs[s][at[s]: at[s] + n])
            pos += list(range(at[s], at[s] + n))
            cu.append(cu[-1] + n)
            sl.append(slots[s])
        x = torch.cat(rows).to(device)
        single = all(n == 1 for _, n in step)
        rag = seq.Ragged(torch.tensor(pos, device=device), None if single else torch.tensor(cu, dtype=torch.int32, device=device),
                         torch.tensor(sl, dtype=torch.int32, device=device))
        o = lin.lightning_attn(x, 0, H * D, 2 * H * D, dec, state, H, D, V, rag).cpu()
        for i, (s, n) in enumerate(step):
            got[s].append(o[cu[i]: cu[i + 1]])
            at[s] += n
    for s in range(2):
        gs = torch.cat(got[s]).double()
        assert gs.shape[0] == at[s]
        ref = want[s][: at[s]]
        assert float((gs - ref).abs().max()) < 1e-4 * float(ref.abs().max())
    assert float(state[1].min()) == 7.0 and float(state[3].max()) == 7.0   # other slots untouched


def _attention_case(device, dt, impl, n_ctx, q_lo, standout, window, H=4, G=2, D=32, softcap=30.0, block=16):
    """One sequence of n_ctx tokens whose queries q_lo .. n_ctx - 1 run as one step over scattered pages; the key at
    position ``standout`` and the last query are scaled so that their score dominates when the key is visible.
    Returns (engine ops' output, oracle output) for the query rows."""
    from src.ops import seq

    g = torch.Generator().manual_seed(n_ctx * 7 + standout)
    eps, scale, coef, every = 1e-5, D ** -0.5, 0.5, 8
    p = torch.randn(n_ctx, (H + G) * D, generator=g)
    qn, kn = 1 + 0.2 * torch.randn(D, generator=g), 1 + 0.2 * torch.randn(D, generator=g)
    qn[0], kn[0] = qn[0].abs(), kn[0].abs()
    # the last query and the standout key put their weight on each head's first dimension: that score is about 11,
    # every other one about N(0, 2), and the standout's value (its raw key) is large where the others' are not
    p[-1, : H * D: D] = 12.0
    p[standout, H * D:: D] = 12.0
    p = p.to(dt)
    nb = (n_ctx + block - 1) // block
    perm = torch.randperm(nb + 3, generator=g)[:nb]
    cache = torch.zeros(nb + 3, block, G * 2 * D, dtype=dt, device=device)
    pos = torch.arange(n_ctx)
    slots = perm[pos // block] * block + pos % block
    slopes = torch.pow(2.0, -8.0 * torch.arange(1, H + 1, dtype=F64) / H).float()
    pd = p.to(device)
    qr = seq.qkv_prep(pd[:, : H * D], pd[:, H * D:], None, cache, H, G, D, D, pos.to(device), slots.to(device), eps,
                      q_norm=qn.to(device), k_norm=kn.to(device), head_norm=True, q_temp_coef=coef, q_temp_every=every)
    nq = n_ctx - q_lo
    single = nq == 1
    out = seq.sink_attn(qr[q_lo:].contiguous(), cache, perm[None].to(torch.int32).to(device),
                        None if single else torch.tensor([0, nq], dtype=torch.int32, device=device),
                        torch.tensor([n_ctx], dtype=torch.int32, device=device), pos[q_lo:].to(device), None, None,
                        nq, H, G, D, D, window, scale, impl=impl, softcap=softcap, slopes=slopes.to(device))
    # oracle: the same mixer without its projections (identity weights)
    m = {"heads": H, "kv_heads": G, "dim": D, "scale": scale, "softcap": softcap, "q_temp": {"coef": coef, "every": every}}
    if window:
        m["mask"] = {"size": window}
    w = {"q": torch.eye(H * D, (H + G) * D, dtype=F64),
         "k": torch.cat([torch.zeros(G * D, H * D, dtype=F64), torch.eye(G * D, dtype=F64)], 1),
         "q.norm": qn.to(F64), "k.norm": kn.to(F64), "o": torch.eye(H * D, dtype=F64)}
    want = orc.window_attention(p.to(F64), w, m, eps)[q_lo:]
    return out.cpu().double(), want


IMPLS = [pytest.param("cpu", 0, id="cpu"), pytest.param("cuda:0", 1, marks=pytest.mark.gpu, id="gpu-fma"),
         pytest.param("cuda:0", 2, marks=pytest.mark.gpu, id="gpu-mfma"),
         pytest.param("cuda:0", 0, marks=pytest.mark.gpu, id="gpu-auto")]


@pytest.mark.parametrize("device,impl", IMPLS)
@pytest.mark.parametrize("where", ["in", "out", "far", "page", "first"])
@pytest.mark.parametrize("rows", ["portion", "decode"])
def test_attention_keys_at_the_windows_edges(device, impl, where, rows):
    """A key made to stand out just inside / just outside the window of the last query, far back without a window,
    on a page border, and at position 0 — in a prompt portion and for a single decode row."""
    _need(device)
    n_ctx, window = 150, 37
    if where == "in":
        standout = n_ctx - window            # i - j = window - 1: the oldest visible key
    elif where == "out":
        standout = n_ctx - window - 1        # one further back: hidden
    elif where == "far":
        standout, window = 3, 0
    elif where == "page":
        standout, window = 127, 0            # the last row of a page, the next key opens a new one
    else:
        standout, window = 0, 0
    q_lo = n_ctx - 1 if rows == "decode" else n_ctx - 41
    for dt in ((torch.float32,) if impl == 1 or device == "cpu" else (torch.bfloat16,)):
        if impl == 2 and dt != torch.bfloat16:
            continue
        got, want = _attention_case(device, dt, impl, n_ctx, q_lo, standout, window)
        tol = 2e-5 if dt == torch.float32 else 3e-2
        assert float((got - want).abs().max()) < tol * float(want.abs().max())
        if where != "out":
            # the standout key carries the last row: leaving it out changes the output by far more than the tolerance
            other, _ = _attention_case(device, dt, impl, n_ctx, q_lo, standout, (n_ctx - 1 - standout) if standout else 149)
            assert float((other[-1] - want[-1]).abs().max()) > 20 * tol * float(want.abs().max())


@pytest.mark.parametrize("device", DEVICES)
def test_attention_other_shapes(device):
    """Head counts and sizes that the matrix-core kernels do not take, one key/value head, no cap, heads == kv_heads."""
    _need(device)
    for H, G, D, cap, win in ((3, 1, 6, 0.0, 5), (2, 2, 20, 4.0, 0), (8, 2, 64, 20.0, 33), (5, 5, 8, 2.0, 1)):
        for q_lo in (0, 29):
            got, want = _attention_case(device, torch.float32, 0, 30, q_lo, 11, win, H=H, G=G, D=D, softcap=cap, block=4)
            assert float((got - want).abs().max()) < 2e-5 * float(want.abs().max())


def _latent_case(device, dt, n_ctx, q_lo, standout, present=True, block=16):
    """Two mixers of the engine: A caches its latents for n_ctx tokens; B (``kv_from``) runs the queries
    q_lo .. n_ctx - 1 over A's scattered pages. The input of token ``standout`` is chosen so that its latent lines up
    with head 0's last query in latent space (score about 16, every other one about N(0, 3)). Returns (B's output,
    the oracle's) for the query rows."""
    from src.models.bapivik import BAPIVIK_MIXERS
    from src.models.llama import AttnMetadata

    g = torch.Generator().manual_seed(n_ctx + 3 * standout)
    Wd, eps = 40, 1e-5
    la = orc.latent_layer(heads=2, dim=16, vdim=16, kv_rank=32, q_rank=24, ff=0)
    lb = orc.latent_layer(heads=3, dim=16, vdim=24, kv_rank=32, q_rank=16, kv_from=0, ff=0)
    config = orc.make_config([la, lb], width=Wd)
    w = {k: v.to(F64) for k, v in orc.random_weights(config, 4, dtype=dt).items()}
    wa = {k[7:]: v for k, v in w.items() if k.startswith("l0.mix.")}
    wb = {k[7:]: v for k, v in w.items() if k.startswith("l1.mix.")}
    ha = torch.randn(n_ctx, Wd, generator=g).to(dt).to(F64)
    hb = torch.randn(n_ctx, Wd, generator=g).to(dt).to(F64)
    mb = dict(lb["mixer"])
    # head 0's last query in latent space, and an input whose latent points that way
    q_last = (orc.rms(hb[-1:] @ wb["dq"].T, wb["dq.norm"], eps) @ wb["uq"].T)[0, :16]
    u = wb["uk"][:16].T @ q_last                                     # [kv_rank]
    if present:
        ha[standout] = (torch.linalg.pinv(wa["dkv"]) @ (u / wa["dkv.norm"])).to(dt).to(F64)
    c = orc.latent(ha, wa, eps)
    mb["scale"] = 16.0 / float(c[standout].norm() * u.norm()) if present else 16.0 / float(math.sqrt(32) * u.norm())
    want = orc.latent_attention(hb, c, wb, mb, eps)[q_lo:]
    # the engine's mixers on their own cache tensor
    spec_a, spec_b = BAPIVIK_MIXERS["latent_attention"][1](la["mixer"]), BAPIVIK_MIXERS["latent_attention"][1](mb)
    A = BAPIVIK_MIXERS["latent_attention"][0](spec_a, Wd, device, dt, None, 0.0)
    B = BAPIVIK_MIXERS["latent_attention"][0](spec_b, Wd, device, dt, None, 0.0)
    for mixer, ww in ((A, wa), (B, wb)):
        for name, t in ww.items():
            assert mixer.load(name, t.float()), name
    nb = (n_ctx + block - 1) // block
    perm = torch.randperm(nb + 2, generator=g)[:nb]
    cache = torch.zeros(nb + 2, block, 32, dtype=dt, device=device)
    pos = torch.arange(n_ctx)
    slots = (perm[pos // block] * block + pos % block).to(device)
    bt = perm[None].to(torch.int32).to(device)
    ctx = torch.tensor([n_ctx], dtype=torch.int32, device=device)

    def meta(lo):
        n = n_ctx - lo
        if n == 1:
            return AttnMetadata(is_prefill=False, slot_mapping=slots[lo:], block_tables=bt, ctx_lens=ctx)
        return AttnMetadata(is_prefill=True, slot_mapping=slots[lo:], block_tables=bt, ctx_lens=ctx,
                            cu_q=torch.tensor([0, n], dtype=torch.int32, device=device), max_q_len=n)

    A.forward(ha.to(dt).to(device), pos.to(device), meta(0), cache, eps)
    assert B.spec.cache_width == 0 and B.dkv_norm is None
    got = B.forward(hb[q_lo:].to(dt).to(device), pos[q_lo:].to(device), meta(q_lo), cache, eps)
    return got.cpu().double(), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("where", ["far", "page", "first"])
@pytest.mark.parametrize("rows", ["portion", "decode"])
def test_latent_attention_on_shared_latents_far_keys(device, where, rows):
    """A layer without latents of its own finds a key far back among 300, on a page border and at position 0 in the
    pages another layer wrote — in a prompt portion and for a single decode row; fp32 (FMA kernel) and, on the GPU,
    bf16 (matrix cores)."""
    _need(device)
    n_ctx = 300
    standout = {"far": 2, "page": 255, "first": 0}[where]
    q_lo = n_ctx - 1 if rows == "decode" else n_ctx - 45
    for dt in ((torch.float32,) if device == "cpu" else (torch.float32, torch.bfloat16)):
        got, want = _latent_case(device, dt, n_ctx, q_lo, standout)
        tol = 3e-5 if dt == torch.float32 else 4e-2
        assert float((got - want).abs().max()) < tol * float(want.abs().max())
        _, without = _latent_case(device, dt, n_ctx, q_lo, standout, present=False)
        # the engine's last row is much nearer to the oracle with that key than to the oracle without it
        near, away = float((got[-1] - want[-1]).abs().max()), float((got[-1] - without[-1]).abs().max())
        assert near < 0.15 * away, (near, away)


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
        # the stream after every layer, through the model's layer hook
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
@pytest.mark.parametrize("name", ["std", "odd"])
@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 2, 16, 2, 7], [1], [30, 2], [15, 16, 17]], ids=str)
def test_portions_then_token_by_token(tmp_path, device, name, sizes):
    """Prompt portions of several sizes, then single tokens, against the oracle's whole-sequence logits."""
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
    """A prompt then 100 single-token steps in bf16 (windows pass over decoded tokens, the recurrent state is carried
    100 times), and the same positions from one whole-prompt step: both hold the oracle's logits."""
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
    window by one token, the distance slopes, the score cap, the query temperature, a decay, whose latents a layer
    reads, the depth weights, an output gate, the position vectors, a bias."""
    config = CONFIGS["std"]()
    weights = weights_for(config, 1)
    toks = tokens_for(config, 40, 2)
    base = orc.forward(config, weights, toks)

    def moved(cfg=None, w=None):
        e = row_errs(orc.forward(cfg or config, w or weights, toks), base)
        return float(e[-8:].max())

    def with_mixer(i, **kw):
        c = copy.deepcopy(config)
        for k, v in kw.items():
            if v is None:
                c["layers"][i]["mixer"].pop(k, None)
            else:
                c["layers"][i]["mixer"][k] = v
        return c

    floor = 30 * TOL[torch.float32]
    assert moved(with_mixer(2, mask={"size": 10})) > floor
    assert moved(with_mixer(2, mask={"size": 8})) > floor
    assert moved(with_mixer(2, softcap=None)) > floor
    assert moved(with_mixer(2, q_temp=None)) > floor
    assert moved(with_mixer(2, q_temp={"coef": 0.4, "every": 6})) > floor
    assert moved(with_mixer(3, decay=[0.5, 0.5, 0.5])) > floor
    c = with_mixer(6, kv_from=None)
    w = dict(weights)
    w["l6.mix.dkv"], w["l6.mix.dkv.norm"] = weights["l4.mix.dkv"], weights["l4.mix.dkv.norm"]
    assert moved(c, w) > floor                         # its own latents from the same weights, not layer 4's
    for name in ("l3.dwa", "l0.mix.g", "pos", "l0.mlp.down.b", "l5.mix.k.norm"):
        w = dict(weights)
        w[name] = torch.flip(weights[name], [0]) if weights[name].dim() == 1 else weights[name] * 0.5
        assert moved(w=w) > floor, name


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
        """Every generated token is the oracle's argmax given the tokens before it (or within a rounding error of
        it: random weights with tied embeddings produce near-ties)."""
        seq_ = list(prompt)
        for tok in out:
            lg = orc.forward(config, weights, seq_)[-1]
            if float(lg[tok]) < float(lg.max()) - 1e-3 * float(lg.std()):
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


def test_registry_config_roundtrip_and_refusals(tmp_path):
    from src.models.bapivik import BapivikArch, BapivikLM
    from src.models.registry import family_of, resolve

    config = CONFIGS["std"]()
    path = str(tmp_path / "ckpt")
    save_checkpoint(path, config, weights_for(config))
    assert family_of(path) == "bapivik"
    name, arch, cls = resolve(path)
    assert cls is BapivikLM and arch.num_layers == len(config["layers"])
    assert arch.to_config() == json.loads(json.dumps(config))
    model = cls(arch, "cpu", dtype=torch.float32)
    assert model.needs_seq_state and not model.supports_prefix_cache
    widths = [l.mixer.cache_width for l in arch.layers]
    assert widths[1] == 0 and widths[3] == 0 and widths[6] == 0 and widths[0] == 32
    # saving and loading again gives the same tensors
    from safetensors.torch import load_file

    n = model.load_state_dict(load_file(os.path.join(path, "model.safetensors")))
    assert n == len(orc.tensor_shapes(config))
    model.save(str(tmp_path / "again"))
    again = load_file(str(tmp_path / "again" / "model.safetensors"))
    for k, v in weights_for(config).items():
        assert torch.equal(again[k].float().reshape(v.shape), v.float()), k
    # a follower must name an earlier layer that makes latents of the same width
    for bad in (dict(kv_from=1), dict(kv_from=2), dict(kv_from=5), dict(kv_from=4, kv_rank=32)):
        c = copy.deepcopy(config)
        c["layers"][6]["mixer"].update(bad)
        with pytest.raises(ValueError):
            BapivikArch.from_config(c)
    # no recurrent layer: no state slots, prefix cache allowed
    c2 = CONFIGS["attn_only"]()
    m2 = BapivikLM(BapivikArch.from_config(c2), "cpu", dtype=torch.float32)
    assert not m2.needs_seq_state and m2.supports_prefix_cache


def test_positions_beyond_the_table_are_refused(tmp_path):
    config = orc.make_config([orc.attn_layer()], max_positions=24)
    eng = make_engine(tmp_path, config, weights_for(config), "cpu", torch.float32, max_tokens=64)
    assert eng.max_model_len == 24


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
