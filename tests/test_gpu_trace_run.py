"""bin/trace_run as a user runs it: a subprocess fed JSON lines, logits read back from files."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import schedules
from tests.plain import qwen3_plain
from tests.util import TINY, make_model_dir, random_tokens, read_config, read_weights, tolerance

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def replay(folder, dtype_name, steps, out_dir, max_tokens, *flags):
    process = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype",
                                dtype_name, "--out", out_dir, "--max-tokens", str(max_tokens), *flags],
                               stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    outputs = {}
    vocab = read_config(folder)["vocab_size"]
    for s in steps:
        process.stdin.write(json.dumps(s) + "\n")
        process.stdin.flush()
        line = process.stdout.readline().strip()
        assert line == f"done {s['step']}", line
        wanted = sum(len(e["want"]) for e in s["entries"])
        path = os.path.join(out_dir, f"{s['step']}.f32")
        if wanted:
            outputs[s["step"]] = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        else:
            assert not os.path.exists(path)
    process.stdin.close()
    assert process.wait(timeout=60) == 0
    return outputs


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_modes_agree_with_plain(tmp_path, name, dtype_name):
    folder = make_model_dir(str(tmp_path / "model"), TINY[name], 31,
                            torch.float32 if dtype_name == "float32" else torch.bfloat16,
                            sharpen=2.0 if dtype_name == "float32" else 1.0)
    weights, config = read_weights(folder), read_config(folder)
    lengths = [150, 70, 40, 200, 97, 64] if name == "A" else [130, 260, 65, 33, 190]
    requests = {f"q{i}": random_tokens(500 + i, n, config["vocab_size"]) for i, n in enumerate(lengths)}
    expected = {rid: qwen3_plain.forward(weights, config, toks).numpy() for rid, toks in requests.items()}
    for mode in ("whole", "tail_decoded", "portions", "mixed"):
        steps = getattr(schedules, mode)(requests)
        if mode == "mixed":   # only some places wanted, some steps with none
            for s in steps:
                for e in s["entries"]:
                    e["want"] = [w for w in e["want"] if (w + s["step"]) % 3 != 0]
        out_dir = str(tmp_path / f"out_{mode}")
        outputs = replay(folder, dtype_name, steps, out_dir, schedules.max_live_tokens(steps, 64))
        at = {rid: 0 for rid in requests}
        for s in steps:
            row = 0
            for e in s["entries"]:
                for w in e["want"]:
                    have = outputs[s["step"]][row]
                    want = expected[e["id"]][at[e["id"]] + w]
                    err = float(np.abs(have - want).max())
                    assert np.isfinite(have).all() and err <= tolerance(dtype_name), \
                        f"{mode}: request {e['id']} position {at[e['id']] + w}: {err:.3e}"
                    row += 1
                at[e["id"]] += len(e["tokens"])


def test_sidecar_ties_the_logits_to_what_made_them(tmp_path):
    """--sidecar: model and build identity, the schedule and digests of input and outputs; --poison-freed: pages
    given back are filled with NaN and the logits of a run that reuses them are the same bits as without."""
    import hashlib
    folder = make_model_dir(str(tmp_path / "model"), TINY["A"], 33, torch.bfloat16)
    config = read_config(folder)
    requests = {f"q{i}": random_tokens(700 + i, n, config["vocab_size"]) for i, n in enumerate([90, 70, 40, 120, 64, 33])}
    steps = schedules.mixed(requests)
    room = schedules.max_live_tokens(steps, 64)
    plain_out, poisoned_out = str(tmp_path / "plain"), str(tmp_path / "poisoned")
    first = replay(folder, "bfloat16", steps, plain_out, room)
    second = replay(folder, "bfloat16", steps, poisoned_out, room, "--sidecar", "--poison-freed")
    assert not os.path.exists(os.path.join(plain_out, "sidecar.json"))
    for step, block in first.items():
        assert np.isfinite(block).all() and np.array_equal(block, second[step])
    with open(os.path.join(poisoned_out, "sidecar.json")) as handle:
        sidecar = json.load(handle)
    assert sidecar["schema"] == "leone-amd.trace.v1" and sidecar["dtype"] == "bfloat16" and sidecar["poison_freed"]
    assert sidecar["architecture"] == config["architectures"][0] and sidecar["vocab"] == config["vocab_size"]
    with open(os.path.join(folder, "config.json"), "rb") as handle:
        assert sidecar["config_sha256"] == hashlib.sha256(handle.read()).hexdigest()
    with open(os.path.join(folder, "model.safetensors"), "rb") as handle:
        assert sidecar["weights"] == [{"file": "model.safetensors", "bytes": os.path.getsize(handle.name),
                                       "header_sha256": sidecar["weights"][0]["header_sha256"],
                                       "sha256": hashlib.sha256(handle.read()).hexdigest()}]
    assert sidecar["input_sha256"] == hashlib.sha256("".join(json.dumps(s) + "\n" for s in steps).encode()).hexdigest()
    assert len(sidecar["build"]["kernels"]) == 16 and len(sidecar["build"]["host"]) == 16
    assert [s["step"] for s in sidecar["steps"]] == [s["step"] for s in steps]
    for noted, s in zip(sidecar["steps"], steps):
        assert noted["end"] == s["end"]
        assert noted["entries"] == [{"id": e["id"], "tokens": len(e["tokens"]), "want": e["want"]} for e in s["entries"]]
        if any(e["want"] for e in s["entries"]):
            with open(os.path.join(poisoned_out, noted["file"]), "rb") as handle:
                assert noted["sha256"] == hashlib.sha256(handle.read()).hexdigest()
            assert noted["rows"] == sum(len(e["want"]) for e in s["entries"])
        else:
            assert "file" not in noted
