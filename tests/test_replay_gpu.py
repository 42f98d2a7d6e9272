"""bin/trace_run as a user runs it: the same requests whole, with the last 32 tokens one
by one, and in batches of unequal lengths, in float32 and bfloat16, against the plain
implementation."""
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from helpers import assert_close, make_folder, random_ids

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]
LENGTHS = {"A": [97, 40, 128], "B": [33, 150, 64, 256]}


def replay(folder, dtype, out_dir, max_tokens, steps):
    text = "".join(json.dumps(step) + "\n" for step in steps)
    run = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder),
                          "--dtype", dtype, "--out", str(out_dir), "--max-tokens",
                          str(max_tokens)], input=text, capture_output=True, text=True,
                         timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [line for line in run.stdout.split("\n") if line.startswith("done")] == \
        [f"done {step['step']}" for step in steps]

    def read(step, vocab):
        return torch.from_numpy(np.fromfile(str(out_dir / f"{step}.f32"), dtype="<f4")
                                .reshape(-1, vocab).astype(np.float32))
    return read


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_trace_replay(tmp_path, name, dtype):
    folder = make_folder(name, tmp_path)
    cfg, w = plain.read_folder(folder)
    vocab = cfg["vocab_size"]
    requests = [random_ids(vocab, n, 50 + i) for i, n in enumerate(LENGTHS[name])]
    refs = [plain.forward(w, cfg, ids) for ids in requests]
    rounded = sum((n + 63) // 64 * 64 for n in LENGTHS[name])

    # whole: each request alone, every position wanted
    steps = [{"step": i, "entries": [{"id": f"r{i}", "tokens": ids, "want": list(range(len(ids)))}],
              "end": [f"r{i}"]} for i, ids in enumerate(requests)]
    read = replay(folder, dtype, tmp_path / "whole", max(len(r) for r in requests), steps)
    for i, ref in enumerate(refs):
        assert_close(dtype, read(i, vocab), ref, f"whole {i}")

    # the last 32 tokens one by one
    steps, expect, number = [], [], 0
    for i, ids in enumerate(requests):
        cut = len(ids) - 32
        steps.append({"step": number, "entries": [{"id": f"t{i}", "tokens": ids[:cut], "want": [cut - 1]}],
                      "end": []})
        expect.append((number, refs[i][cut - 1:cut]))
        number += 1
        for t in range(cut, len(ids)):
            last = t == len(ids) - 1
            steps.append({"step": number, "entries": [{"id": f"t{i}", "tokens": [ids[t]], "want": [0]}],
                          "end": [f"t{i}"] if last else []})
            expect.append((number, refs[i][t:t + 1]))
            number += 1
    read = replay(folder, dtype, tmp_path / "tail", max(len(r) for r in requests), steps)
    for step, ref in expect:
        assert_close(dtype, read(step, vocab), ref, f"tail step {step}")

    # batches of unequal lengths, one after another, shorter requests end earlier;
    # a step in which nothing is wanted writes no file
    steps, expect, number = [], [], 0
    for batch in (list(range(len(requests))), list(reversed(range(len(requests))))):
        cuts = {r: len(requests[r]) - 32 for r in batch}
        tag = f"b{number}_"
        steps.append({"step": number, "entries": [
            {"id": tag + str(r), "tokens": requests[r][:cuts[r]], "want": [cuts[r] - 1]} for r in batch],
            "end": []})
        expect.append((number, torch.cat([refs[r][cuts[r] - 1:cuts[r]] for r in batch])))
        number += 1
        drop_at = {r: 32 - 3 * k for k, r in enumerate(batch)}      # 32, 29, 26, ... tokens
        for t in range(32):
            live = [r for r in batch if t < drop_at[r]]
            wanted = t % 5 != 4
            steps.append({"step": number, "entries": [
                {"id": tag + str(r), "tokens": [requests[r][cuts[r] + t]], "want": [0] if wanted else []}
                for r in live], "end": [tag + str(r) for r in live if t + 1 == drop_at[r]]})
            if wanted:
                expect.append((number, torch.cat([refs[r][cuts[r] + t:cuts[r] + t + 1] for r in live])))
            else:
                expect.append((number, None))
            number += 1
    read = replay(folder, dtype, tmp_path / "batched", rounded, steps)
    for step, ref in expect:
        if ref is None:
            assert not (tmp_path / "batched" / f"{step}.f32").exists()
        else:
            assert_close(dtype, read(step, vocab), ref, f"batched step {step}")
