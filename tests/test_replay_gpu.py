"""bin/trace_run as a user runs it: a subprocess fed JSON lines. The same requests
are replayed whole, with the last 32 tokens one by one, and in batches of unequal
lengths whose shorter requests end earlier while slots are used again, in 32-bit
and in bfloat16, and every logit row is compared with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests.conftest import ROOT, TINY
from tests.helpers import close, rand_ids
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def replay(model_dir, dtype, steps, out_dir, max_tokens):
    """Feeds the steps one by one, each only after 'done <step>' of the one before."""
    proc = subprocess.Popen([sys.executable, TRACE_RUN, "--model", model_dir, "--dtype", dtype,
                             "--out", out_dir, "--max-tokens", str(max_tokens)],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {st['step']}", line
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


def read_rows(out_dir, step, vocab):
    a = np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4")
    assert a.size % vocab == 0
    return torch.from_numpy(a.reshape(-1, vocab).copy())


def requests_for(name, plain_models):
    vocab = plain_models[name][0]["vocab_size"]
    lengths = [40, 97, 33, 150, 64, 35] if name == "C" else [40, 97, 33, 70, 64, 35]
    return {f"r{i}": rand_ids(vocab, n, 80 + i) for i, n in enumerate(lengths)}


def rounded(n):
    return (n + 63) // 64 * 64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_replay_three_ways(model_dirs, plain_models, tmp_path, name, dtype):
    cfg, w = plain_models[name]
    vocab = cfg["vocab_size"]
    reqs = requests_for(name, plain_models)
    want = {rid: P.forward(cfg, w, ids) for rid, ids in reqs.items()}

    # 1. each request alone and whole
    steps, where = [], {}
    for k, (rid, ids) in enumerate(reqs.items()):
        steps.append({"step": k, "entries": [{"id": rid, "tokens": ids, "want": list(range(len(ids)))}],
                      "end": [rid]})
        where[rid] = k
    out1 = str(tmp_path / "whole")
    replay(model_dirs[name], dtype, steps, out1, max(rounded(len(i)) for i in reqs.values()))
    whole = {rid: read_rows(out1, k, vocab) for rid, k in where.items()}
    for rid in reqs:
        close(whole[rid], want[rid], dtype)

    # 2. the last 32 tokens one by one
    steps, k, rows_at = [], 0, {}
    for rid, ids in reqs.items():
        n = len(ids)
        steps.append({"step": k, "entries": [{"id": rid, "tokens": ids[:n - 32], "want": []}], "end": []})
        k += 1
        rows_at[rid] = []
        for j in range(n - 32, n):
            steps.append({"step": k, "entries": [{"id": rid, "tokens": [ids[j]], "want": [0]}],
                          "end": [rid] if j == n - 1 else []})
            rows_at[rid].append(k)
            k += 1
    out2 = str(tmp_path / "tail")
    replay(model_dirs[name], dtype, steps, out2, max(rounded(len(i)) for i in reqs.values()))
    for rid, ids in reqs.items():
        assert not os.path.exists(os.path.join(out2, f"{rows_at[rid][0] - 1}.f32"))   # nothing wanted, no file
        dec = torch.cat([read_rows(out2, s, vocab) for s in rows_at[rid]])
        close(dec, want[rid][-32:], dtype)
        if dtype == "float32":
            assert torch.equal(dec, whole[rid][-32:])

    # 3. batches of unequal lengths; shorter requests end earlier; the next batch starts
    #    at once and takes the slots and pages that came back
    names = list(reqs)
    batches = [names[:3], names[3:5], names[5:]]
    steps, k = [], 0
    got = {rid: [] for rid in reqs}
    plan = []
    for batch in batches:
        fed = {rid: max(1, len(reqs[rid]) // 3) for rid in batch}
        ents = [{"id": rid, "tokens": reqs[rid][:fed[rid]], "want": list(range(fed[rid]))} for rid in batch]
        live = list(batch)
        while True:
            end = [rid for rid in live if fed[rid] == len(reqs[rid])]
            steps.append({"step": k, "entries": ents, "end": end})
            plan.append((k, [(e["id"], len(e["want"])) for e in ents]))
            k += 1
            live = [rid for rid in live if rid not in end]
            if not live:
                break
            ents = [{"id": rid, "tokens": [reqs[rid][fed[rid]]], "want": [0]} for rid in live]
            for rid in live:
                fed[rid] += 1
    peak = max(sum(rounded(len(reqs[r])) for r in b) for b in batches)
    out3 = str(tmp_path / "batches")
    replay(model_dirs[name], dtype, steps, out3, peak)
    for k, ents in plan:
        rows = read_rows(out3, k, vocab)
        r = 0
        for rid, n in ents:
            got[rid].append(rows[r:r + n])
            r += n
        assert r == rows.shape[0]
    for rid in reqs:
        close(torch.cat(got[rid]), want[rid], dtype)
        if dtype == "float32":
            assert torch.equal(torch.cat(got[rid]), whole[rid])


def test_trace_run_refuses_what_does_not_fit(model_dirs, tmp_path):
    """max-tokens sizes the cache: a request beyond it fails loudly, not silently."""
    proc = subprocess.run([sys.executable, TRACE_RUN, "--model", model_dirs["A"], "--dtype", "float32",
                           "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                          input=json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [1] * 65, "want": [0]}],
                                            "end": []}) + "\n",
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0 and "done 0" not in proc.stdout
    assert "exceed" in proc.stderr or "pages" in proc.stderr
