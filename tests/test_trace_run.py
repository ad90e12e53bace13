"""The schedule-replay entry point (``bin/trace_run``) as a user runs it: a checkpoint folder, JSON
steps on standard input, logits per step in files, ``done <step>`` lines; and ``score_step`` for
the dense family (portions of a text score like the whole text)."""
import json
import os
import subprocess
import sys

import numpy as np
import torch

import natilix_fixtures as fx
from natilix_oracle import Oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_replay_writes_the_oracles_logits(tmp_path):
    c = fx.default_config()
    w = fx.weights(c, 21)
    folder = fx.save_checkpoint(str(tmp_path / "m"), c, w)
    g = torch.Generator().manual_seed(22)
    a = torch.randint(0, c["vocab"], (70,), generator=g).tolist()
    b = torch.randint(0, c["vocab"], (9,), generator=g).tolist()
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[40:69], "want": []},
                                     {"id": "b", "tokens": b[:8], "want": [7]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[8:], "want": [0]},
                                     {"id": "a", "tokens": a[69:], "want": [0]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder,
                        "--dtype", "float32", "--out", str(out), "--max-tokens", "192",
                        "--block-size", "16", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = Oracle(c, w).feed(a).float().numpy(), Oracle(c, w).feed(b).float().numpy()
    V = c["vocab"]
    got = {n: np.fromfile(out / f"{n}.f32", "<f4").reshape(-1, V) for n in range(3)}
    np.testing.assert_allclose(got[0], la[[0, 39]], rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(got[1], lb[[7]], rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(got[2], np.stack([lb[8], la[69]]), rtol=2e-4, atol=2e-4)


def test_score_step_of_the_dense_family_does_not_depend_on_the_cut():
    from minivllm_amd.engine.llm_engine import LLMEngine
    eng = LLMEngine(dict(model_preset="qwen3-tiny", device="cpu", dtype="fp32", block_size=8,
                         max_cached_blocks=32, max_num_sequences=2, max_model_length=128,
                         max_num_batched_tokens=128, eos=-1))
    g = torch.Generator().manual_seed(3)
    toks = torch.randint(0, 512, (30,), generator=g).tolist()
    whole = eng.score_step([{"id": "w", "tokens": toks, "want": list(range(30))}], ["w"])["w"]
    parts = []
    at = 0
    for n in (5, 2, 1, 12, 1, 9):
        parts.append(eng.score_step([{"id": "p", "tokens": toks[at:at + n], "want": list(range(n))}],
                                    ["p"] if at + n == 30 else [])["p"])
        at += n
    torch.testing.assert_close(torch.cat(parts), whole, rtol=1e-4, atol=1e-4)
    eng.exit()
