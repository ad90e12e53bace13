"""Replay a recorded schedule of given tokens through the engine and write the logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

``DIR`` holds ``config.json`` + ``model.safetensors``; the model class is chosen from
``config.json`` (``models/registry.py``).  Standard input carries one JSON object per line,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}

All entries of a step run as one engine step (``LLMEngine.score_step``): portions of prompts as
prefill rows next to single next tokens as decode rows, through the scheduler's admission, the
paged KV cache, the state slots and the kernels that generation uses.  For a step that asks for
logits the file ``<out>/<step>.f32`` holds them as little-endian fp32 [asked, vocab], in the
order of the entries and of ``want``; after every step the line ``done <step>`` is printed.
``--max-tokens``: the most tokens live requests hold at any time (each rounded up to a whole
KV block of ``--block-size`` tokens); the KV pool gets that many and no more, and there are
``--max-seqs`` sequence (and state) slots.  Whatever native library the model's step needs is
built on first use.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def _ensure_built(need_sampler: bool) -> None:
    from minivllm_amd import build
    build.build_host(verbose=False)
    build.build_hip_group("hybrid", verbose=False)
    if need_sampler:
        build.build_hip(verbose=False)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--block-size", type=int, default=64)
    ap.add_argument("--max-seqs", type=int, default=4)
    ap.add_argument("--device", default="auto", choices=["auto", "cuda", "cpu"])
    ap.add_argument("--eager", action="store_true", help="no captured decode graphs")
    a = ap.parse_args(argv)

    import torch
    from minivllm_amd.models.registry import config_from_path
    model_cfg = config_from_path(a.model)
    dense = not hasattr(model_cfg, "validate_engine")
    device = a.device
    if device == "auto":
        device = "cuda" if torch.cuda.is_available() else "cpu"
    if device == "cuda":
        if dense and a.dtype == "float32":
            print("this model family has no 32-bit GPU kernels", file=sys.stderr)
            return 3
        _ensure_built(need_sampler=dense)
        torch.backends.cuda.matmul.allow_tf32 = False
    bs = a.block_size
    blocks = (a.max_tokens + bs - 1) // bs
    length = blocks * bs
    if getattr(model_cfg, "max_position", length) < length:
        model_cfg.max_position = length
    from minivllm_amd.engine.llm_engine import LLMEngine
    eng = LLMEngine(dict(model=model_cfg, checkpoint_path=a.model, model_name_or_path=None,
                         dtype=a.dtype, device=device, block_size=bs, max_cached_blocks=blocks,
                         max_num_sequences=a.max_seqs, max_model_length=length,
                         max_num_batched_tokens=max(length, bs), eos=-1, enforce_eager=a.eager,
                         graph_batch_sizes=sorted({1, 2, a.max_seqs}), tuned_gemms=dense,
                         tune_decode_gemms=dense, tune_prefill_gemms=dense, score_only=True))
    os.makedirs(a.out, exist_ok=True)
    try:
        for line in sys.stdin:
            line = line.strip()
            if not line:
                continue
            step = json.loads(line)
            got = eng.score_step(step.get("entries", []), step.get("end", []))
            rows = [got[e["id"]] for e in step.get("entries", []) if e.get("want")]
            if rows:
                data = torch.cat(rows, 0).to(torch.float32).contiguous().numpy().astype("<f4")
                tmp = os.path.join(a.out, f".{step['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(data.tobytes())
                os.replace(tmp, os.path.join(a.out, f"{step['step']}.f32"))
            print(f"done {step['step']}", flush=True)
    finally:
        eng.exit()
    return 0


if __name__ == "__main__":
    sys.exit(main())
