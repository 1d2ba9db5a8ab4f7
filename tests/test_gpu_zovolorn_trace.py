"""bin/trace_run end to end on a Zovolorn directory of the test's own making: the command line picks the model class by config.json, replays steps (whole prompts,
prompt + decoded tokens, a batch of unequal requests decoded together, states given back and reused) and writes the logits asked for -- against the float64 oracle,
in both precisions."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import zovolorn_oracle as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def model(tmp_path):
    cfg = O.config(vocab=83, width=48, eps=3e-6, groups=4, taps=3, embed_scale=0.8, bigram=(101, 13, 29), logit_softcap=20.0, layers=[
        O.attention_layer(6, 3, 8, 16, rot_dims=4, rot_base=3000.0, scale=0.5, mlp=O.dense(24)),
        O.parallel_layer(3, 3, 16, 24, 12, 90.0, 4, 2, 8, 12, 4, rank=5, scale=0.2, left_scale=0.6, right_scale=0.9, mlp=None),
        O.parallel_layer(2, 1, 8, 40, 6, 50.0, 2, 2, 16, 8, 2, rank=3, left_scale=1.0, right_scale=0.7, mlp=O.dense(16)),
        O.attention_layer(2, 1, 24, 8, rot_dims=24, mlp=None),
    ])
    W = O.weights(cfg, 17)
    path = str(tmp_path / "model")
    O.write_model_dir(path, cfg, W)
    return cfg, {k: v.astype(np.float64) for k, v in W.items()}, path


def replay(path, dtype, steps, out):
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", dtype, "--out", out, "--max-tokens", "700"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    done = [l for l in p.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {s['step']}" for s in steps]
    return {s["step"]: np.fromfile(os.path.join(out, f"{s['step']}.f32"), dtype="<f4") for s in steps if any(e.get("want") for e in s["entries"])}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_whole_decode_and_together(tmp_path, dtype):
    cfg, W, path = model(tmp_path)
    V = cfg["vocab"]
    rng = np.random.default_rng(4)
    reqs = {name: [int(t) for t in rng.integers(0, V, size=n)] for name, n in (("a", 150), ("b", 1), ("c", 67), ("d", 40))}
    want = {k: O.forward(cfg, W, t)[0] for k, t in reqs.items()}
    steps, expect = [], {}
    # a: whole, every tenth position asked for; its state goes back and is taken by the next request
    steps.append({"step": 0, "entries": [{"id": "a", "tokens": reqs["a"], "want": list(range(0, 150, 10))}], "end": ["a"]})
    expect[0] = want["a"][0:150:10]
    # c: most of the prompt, then token by token across the chunks' edges
    steps.append({"step": 1, "entries": [{"id": "c", "tokens": reqs["c"][:39], "want": [38]}], "end": []})
    expect[1] = want["c"][38:39]
    for i in range(39, 67):
        steps.append({"step": len(steps), "entries": [{"id": "c", "tokens": [reqs["c"][i]], "want": [0] if i % 2 else []}], "end": ["c"] if i == 66 else []})
        if i % 2:
            expect[len(steps) - 1] = want["c"][i:i + 1]
    # b, d and a again (another name) together, unequal lengths; then decoded together, the short ones leaving first
    cut = {"b": 1, "d": 30, "e": 140}
    reqs["e"], want["e"] = reqs["a"], want["a"]
    steps.append({"step": len(steps), "entries": [{"id": k, "tokens": reqs[k][:cut[k]], "want": [cut[k] - 1]} for k in ("b", "d", "e")], "end": ["b"]})
    expect[len(steps) - 1] = np.stack([want[k][cut[k] - 1] for k in ("b", "d", "e")])
    for i in range(10):
        live = [k for k in ("d", "e") if cut[k] + i < len(reqs[k])]
        steps.append({"step": len(steps), "entries": [{"id": k, "tokens": [reqs[k][cut[k] + i]], "want": [0]} for k in live],
                      "end": [k for k in live if cut[k] + i == len(reqs[k]) - 1]})
        expect[len(steps) - 1] = np.stack([want[k][cut[k] + i] for k in live])
    got = replay(path, dtype, steps, str(tmp_path / "out"))
    assert sorted(got) == sorted(expect)
    errs = np.concatenate([O.logit_error(got[n].reshape(-1, V), np.asarray(expect[n]).reshape(-1, V)) for n in sorted(expect)])
    if dtype == "float32":
        assert errs.max() < 4e-5, errs.max()
    else:  # the rounding noise of bf16 products in a narrow stream: a row may stand out
        assert np.median(errs) < 3e-2 and np.mean(errs < 6e-2) >= 0.9, (np.median(errs), errs.max())
