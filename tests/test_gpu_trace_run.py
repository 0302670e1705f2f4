"""bin/trace_run as a user runs it: a subprocess fed JSON lines, files of float32 logits back."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import CONFIG_B, make_folder, peak_tokens, random_tokens, rel_err, trace_mixed
from plain import qwen2_plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-4), ("bfloat16", 3e-2)])
def test_replay_through_the_program(tmp_path, dtype, tol):
    folder = make_folder(tmp_path / "model", CONFIG_B, 1, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, weights = qwen2_plain.load_folder(folder)
    requests = {f"q{k}": random_tokens(CONFIG_B["vocab_size"], n, 500 + k) for k, n in enumerate((40, 23, 66, 9, 31))}
    steps = trace_mixed(requests, seed=3)
    steps.insert(2, {"step": 1000, "entries": [], "end": []})                      # a step with nothing in it
    steps[4]["entries"][0]["want"] = []                                            # a portion whose logits nobody wants
    out_dir = tmp_path / "out"
    process = subprocess.run([sys.executable, TRACE_RUN, "--model", folder, "--dtype", dtype, "--out", str(out_dir),
                              "--max-tokens", str(peak_tokens(steps))],
                             input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert process.returncode == 0, process.stderr
    assert process.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    want = {rid: qwen2_plain.forward(cfg, weights, toks) for rid, toks in requests.items()}
    at = {rid: 0 for rid in requests}
    vocab = CONFIG_B["vocab_size"]
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        path = out_dir / f"{s['step']}.f32"
        if wanted == 0:
            assert not path.exists()
        else:
            rows = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
            row = 0
            for e in s["entries"]:
                for w in e["want"]:
                    assert rel_err(rows[row], want[e["id"]][at[e["id"]] + w]) < tol
                    row += 1
        for e in s["entries"]:
            at[e["id"]] += len(e["tokens"])


def test_errors_are_reported_and_not_swallowed(tmp_path):
    folder = make_folder(tmp_path / "model", CONFIG_B, 1)
    base = [sys.executable, TRACE_RUN, "--model", folder, "--dtype", "float32", "--out", str(tmp_path / "o")]
    too_many = subprocess.run(base + ["--max-tokens", "64"], capture_output=True, text=True, timeout=300,
                              input=json.dumps({"step": 0, "entries": [{"id": "a", "tokens": list(range(100)), "want": [0]}],
                                                "end": []}) + "\n")
    assert too_many.returncode == 3 and "trace_run:" in too_many.stderr and "done 0" not in too_many.stdout
    bad_token = subprocess.run(base + ["--max-tokens", "64"], capture_output=True, text=True, timeout=300,
                               input=json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [1, 300], "want": [0]}],
                                                 "end": []}) + "\n")
    assert bad_token.returncode == 2 and "outside the vocabulary of 300" in bad_token.stderr
    missing = subprocess.run([sys.executable, TRACE_RUN, "--model", str(tmp_path / "none"), "--dtype", "float32",
                              "--out", str(tmp_path / "o"), "--max-tokens", "64"], capture_output=True, text=True,
                             timeout=300, input="")
    assert missing.returncode == 2 and "trace_run:" in missing.stderr
