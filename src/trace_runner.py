"""
Trace runner: feeds given token ids through a model on the serving engine, step by step, and writes logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

It samples nothing and owns no forward pass, cache or loader: every step is
:meth:`src.engine.llm_engine.LLMEngine.replay_step` — the engine's scheduler admits the requests and grows
their block tables in a KV pool made for ``--max-tokens`` tokens (each request's count rounded up to the block
size) with at most ``--max-seqs`` live requests, the model runner stages the ragged batch and the model's own
kernels run it from the cache that earlier steps left. The model class is chosen by ``config.json``
(:mod:`src.models.registry`).

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: each request's next tokens and the places among them whose logits are wanted; all entries of a step
run as one batch. ``end``: requests finished after the step. For a step with wanted places the logits are
written to ``<out>/<step>.f32`` (little-endian fp32, [wanted, vocab], in entry order); after every step a line
``done <step>`` is printed. The native extensions the model needs are compiled on first use.
"""

from __future__ import annotations

import argparse
import json
import os
import sys


def _ensure_built(need_full: bool) -> None:
    """Build (in-tree) what is missing: the host runtime and the dtype-generic kernel extension; the Llama-path
    kernels only when the model needs them."""
    from src import _build

    def missing(stem: str) -> bool:
        return not os.path.exists(os.path.join(_build.ROOT, "src", stem + _build.EXT_SUFFIX))

    if missing("_runtime"):
        print("building src/_runtime ...", file=sys.stderr, flush=True)
        _build.build_runtime()
    if missing("_Cmix"):
        print("building src/_Cmix ...", file=sys.stderr, flush=True)
        _build.build_mix()
    if need_full and missing("_C"):
        print("building src/_C ...", file=sys.stderr, flush=True)
        _build.build_kernels()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True, help="KV pool capacity in tokens")
    ap.add_argument("--max-seqs", type=int, default=4, help="most requests live at any time")
    ap.add_argument("--device", default=None, help="default: cuda:0 if there is a GPU, else cpu")
    a = ap.parse_args(argv)

    from src.models.registry import family_of

    family = family_of(a.model)
    generic = family in ("datatar", "fekolorn", "bapivik", "kogerax")   # families on the dtype-generic kernels (src/_Cmix) alone
    if not generic and a.dtype == "float32":
        print(f"the {family} kernels are bfloat16 only", file=sys.stderr)
        return 3
    _ensure_built(need_full=not generic)

    import numpy as np
    import torch

    from src.config import EngineConfig
    from src.engine import LLMEngine

    device = a.device or ("cuda:0" if torch.cuda.is_available() else "cpu")
    dtype = torch.bfloat16 if a.dtype == "bfloat16" else torch.float32
    if dtype == torch.float32:  # true fp32 matrix products
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
    block = EngineConfig.block_size
    n_blocks = (a.max_tokens + block - 1) // block
    cfg = EngineConfig(max_num_seqs=a.max_seqs, max_num_batched_tokens=n_blocks * block, block_size=block,
                       num_kv_blocks=n_blocks, enable_prefix_caching=False, use_cuda_graph=False,
                       preemption_mode="recompute", tuned_gemm_table=False, decode_window=1)
    eng = LLMEngine.from_pretrained(a.model, device=device, cfg=cfg, max_model_len=n_blocks * block, capture=False,
                                    dtype=dtype)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or []) for e in st["entries"]]
        logits = eng.replay_step(entries, st.get("end") or [])
        if logits.shape[0]:
            tmp = os.path.join(a.out, ".%s.part" % st["step"])
            np.ascontiguousarray(logits.numpy().astype("<f4")).tofile(tmp)
            os.replace(tmp, os.path.join(a.out, "%s.f32" % st["step"]))
        print("done %s" % st["step"], flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
