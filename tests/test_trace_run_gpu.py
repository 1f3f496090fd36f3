"""bin/trace_run as a user runs it: a subprocess fed JSON lines, logits files out."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import cuttings
from engine_helpers import TOL, make_folder, plain_logits, random_sequences
from tiny_configs import tiny

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_trace(folder, dtype, steps, out_dir, max_tokens):
    proc = subprocess.Popen(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", out_dir, "--max-tokens", str(max_tokens)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:
        proc.stdin.write(json.dumps(st) + "\n")
        proc.stdin.flush()
        line = proc.stdout.readline().strip()      # the next step may come only after "done"
        assert line == f"done {st['step']}", line
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0


def collect(out_dir, steps, seqs, vocab):
    out = {rid: torch.full((len(t), vocab), float("nan")) for rid, t in seqs.items()}
    fed = {rid: 0 for rid in seqs}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        path = os.path.join(out_dir, f"{st['step']}.f32")
        if not wanted:
            assert not os.path.exists(path)
            arr = torch.empty(0, vocab)
        else:
            arr = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab).copy())
        row = 0
        for e in st["entries"]:
            for w in e["want"]:
                out[e["id"]][fed[e["id"]] + w] = arr[row]
                row += 1
            fed[e["id"]] += len(e["tokens"])
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_of_a_mixed_trace(tmp_path_factory, gpu_device, dtype):
    folder, _ = make_folder(tmp_path_factory, "B", seed=31)
    vocab = tiny("B")[0]["vocab_size"]
    seqs = random_sequences(vocab, [50, 90, 33, 120, 64, 70], seed=4)
    tdtype = torch.float32 if dtype == "float32" else torch.bfloat16
    want = plain_logits(folder, seqs, tdtype)
    steps = cuttings.mixed(seqs, seed=1, max_live=4)
    # some steps want nothing, some only a few places
    for i, st in enumerate(steps):
        if i % 5 == 3:
            for e in st["entries"]:
                e["want"] = []
        elif i % 5 == 4:
            for e in st["entries"]:
                e["want"] = e["want"][-1:]
    n = cuttings.max_live_tokens(steps)
    assert n < sum(-(-len(t) // 64) * 64 for t in seqs.values())      # pages must be used again
    out_dir = str(tmp_path_factory.mktemp("trace_out"))
    run_trace(folder, dtype, steps, out_dir, n)
    got = collect(out_dir, steps, seqs, vocab)
    for rid in seqs:
        have = ~torch.isnan(got[rid][:, 0])
        assert have.any()
        scale = float(want[rid].abs().max())
        err = (got[rid][have] - want[rid][have]).abs().max() / scale
        assert err < TOL[tdtype], (rid, float(err))
