"""Trace runner: feeds given token ids through a model folder's model, step by step, on the
serving engine (:meth:`LLMEngine.replay_step`) and writes the logits of the places asked for.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: per request its next tokens and the places among them whose logits are wanted;
``end``: requests that are finished after the step (their pages and state slot are freed). All
entries of a step run as one batch. A step with wanted places writes ``DIR/<step>.f32`` (little-
endian fp32 [wanted, vocab], in the order of the entries); every step prints ``done <step>``.

The engine's page pool holds ``--max-tokens`` tokens (``N / 64`` pages) and ``--slots`` (4) state
slots / concurrent requests. The native extensions are built on first use when the checkout has
none. Nothing is sampled.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def _ensure_built() -> None:
    """Build the in-tree extensions when they are missing (a fresh checkout)."""
    try:
        from .. import _C, _rt  # noqa: F401
        return
    except ImportError:
        pass
    from .. import _build

    print("building the native extensions (first run in this checkout)", file=sys.stderr, flush=True)
    _build.build_all()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the page pool holds")
    ap.add_argument("--slots", type=int, default=4, help="state slots = requests live at once")
    ap.add_argument("--device", default="cuda", help="cuda (the HIP kernels); cpu runs the fp32 reference ops")
    ap.add_argument("--no-graphs", action="store_true", help="decode steps eagerly instead of from hipGraphs")
    a = ap.parse_args(argv)
    if a.device.startswith("cuda"):
        _ensure_built()
    import torch

    from ..engine.llm_engine import EngineConfig, LLMEngine
    from ..models.registry import read_config

    if a.device.startswith("cuda") and not torch.cuda.is_available():
        print("trace_run: no GPU visible (the product path is the HIP kernels; --device cpu runs the reference ops)",
              file=sys.stderr)
        return 2
    torch.backends.cuda.matmul.allow_tf32 = False
    mcfg, _ = read_config(a.model)
    pages = max(1, a.max_tokens // 64)
    # no request outgrows the pool, whatever the model's own limit
    max_len = min(int(getattr(mcfg, "max_position", 8192)), max(64, -(-a.max_tokens // 64) * 64))
    sizes = tuple(b for b in (1, 2, 4, 8, 16, 32) if b <= a.slots)
    eng = LLMEngine(EngineConfig(model=a.model, dtype=a.dtype, max_num_seqs=a.slots,
                                 max_batched_tokens=max(a.max_tokens, 64), max_model_len=max_len,
                                 kv_cache_blocks=pages, enable_prefix_caching=False, detokenize=False,
                                 use_graphs=not a.no_graphs, graph_batch_sizes=sizes, mixed_graphs=False,
                                 logits_tap=True, tuned_gemms=False, async_decode=False),
                    device=a.device)
    os.makedirs(a.out, exist_ok=True)
    names: dict = {}
    next_id = 0
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        rows = []
        for e in st.get("entries", []):
            if e["id"] not in names:
                next_id += 1
                names[e["id"]] = next_id
            rid = names[e["id"]]
            rows.append((rid, e["tokens"], e.get("want", [])))
        ended = [names[i] for i in st.get("end", []) if i in names]
        logits = eng.replay_step(rows, ended)
        for i in st.get("end", []):
            names.pop(i, None)
        if logits is not None:
            arr = logits.detach().float().cpu().numpy().astype("<f4")
            tmp = os.path.join(a.out, f".{st['step']}.part")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        elif eng.gpu:
            torch.cuda.synchronize()
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
