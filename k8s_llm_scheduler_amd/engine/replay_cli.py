"""Command-line front ends that work on token ids: ``replay`` (logits of dictated steps) and ``generate``.

    python -m k8s_llm_scheduler_amd replay --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N < steps.jsonl
    python -m k8s_llm_scheduler_amd generate --model DIR_OR_PRESET --prompt "5 17 3" --max-new 16

``replay`` reads one JSON object per line from standard input,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

runs the entries of a step as one engine batch (``LLMEngine.replay_step``), writes the wanted rows' logits to
``OUT/<step>.f32`` (little-endian fp32 [rows, vocab]; no file when nothing is wanted) and prints ``done <step>``.
The cache pool holds ``--max-tokens`` tokens (each live request's count rounded up to whole blocks) and
``--slots`` requests, so blocks and slots are reused as requests end.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
from typing import List, Optional


def _engine(model: str, dtype: str, max_tokens: int, slots: int, device: Optional[str], graphs: bool):
    from pathlib import Path

    from . import build_engine

    is_ckpt = Path(model).exists()
    block = 16
    blocks = max(1, math.ceil(max_tokens / 64) * 64 // block)
    return build_engine(preset=model, weights=model if is_ckpt else None, device=device, dtype=dtype, max_batch=slots,
                        block_size=block, num_blocks=blocks, max_model_len=blocks * block, prefix_caching=False,
                        cuda_graphs=graphs, capture=graphs, tokenizer="ids")


def cmd_replay(argv: List[str]) -> int:
    ap = argparse.ArgumentParser(prog="k8s_llm_scheduler_amd replay", description=__doc__.splitlines()[0])
    ap.add_argument("--model", required=True, help="checkpoint directory (config.json + *.safetensors) or a preset")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the cache pool holds")
    ap.add_argument("--slots", type=int, default=4, help="requests live at a time")
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)
    try:
        eng = _engine(a.model, a.dtype, a.max_tokens, a.slots, a.device, graphs=False)
    except ValueError as e:
        if a.dtype == "float32" and "not supported" in str(e):
            print(str(e), file=sys.stderr)
            return 3
        raise
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(str(e["id"]), [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
                   for e in st.get("entries", [])]
        rows = eng.replay_step(entries, [str(x) for x in st.get("end", [])])
        if rows.shape[0]:
            tmp = os.path.join(a.out, f".{st['step']}.part")
            rows.contiguous().numpy().astype("<f4").tofile(tmp)
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        print(f"done {st['step']}", flush=True)
    return 0


def cmd_generate(argv: List[str]) -> int:
    ap = argparse.ArgumentParser(prog="k8s_llm_scheduler_amd generate", description="Generate from token ids")
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prompt", action="append", required=True, help="whitespace-separated token ids (repeatable)")
    ap.add_argument("--max-new", type=int, default=16)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--max-tokens", type=int, default=4096, help="tokens the cache pool holds")
    ap.add_argument("--device", default=None)
    ap.add_argument("--no-graphs", action="store_true")
    a = ap.parse_args(argv)
    from .sampling import SamplingParams

    eng = _engine(a.model, a.dtype, a.max_tokens, max(4, len(a.prompt)), a.device, graphs=not a.no_graphs)
    sp = SamplingParams(max_tokens=a.max_new, temperature=a.temperature, ignore_eos=True, stop_on_json_close=False)
    for out in eng.generate([eng.tok.encode(p) for p in a.prompt], sp):
        print(json.dumps({"prompt_tokens": out.prompt_tokens, "token_ids": out.token_ids,
                          "finish_reason": out.finish_reason}))
    return 0
