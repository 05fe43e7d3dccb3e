"""bin/trace_run as a user runs it: a checkpoint folder on disk, steps on
standard input, logits files out — compared with the float64 oracle."""

import json
import os
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "tests"))
import kipirax_oracle as O  # noqa: E402

CFG = dict(architecture="Kipirax", vocab=30, width=16, max_positions=64,
           layers=[dict(type="channel_delta", mixer=dict(conv=3, dim=4, heads=2, kv_heads=1, vdim=6),
                        mlp=dict(kind="dense", ff=24)),
                   dict(type="parallel",
                        mixer=dict(left=dict(dim=4, heads=2, kv_heads=2, vdim=8, scale=0.5,
                                             mask=dict(size=5, keep_first=1)),
                                   right=dict(dim=4, heads=2, vdim=4)),
                        mlp=dict(kind="dense", ff=24))],
           norm=dict(eps=1e-5, groups=2), logit_softcap=5.0)


def test_replay_writes_the_oracles_logits(tmp_path):
    from safetensors.torch import save_file

    P = O.random_weights(CFG, seed=11)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(CFG))
    save_file({k: v.contiguous() for k, v in P.items()}, str(model_dir / "model.safetensors"))
    a = torch.randint(0, 30, (21,), generator=torch.Generator().manual_seed(0)).tolist()
    b = torch.randint(0, 30, (9,), generator=torch.Generator().manual_seed(1)).tolist()
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:8], "want": [7]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[8:9], "want": []}, {"id": "b", "tokens": b[:9], "want": [0, 8]}],
         "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[9:], "want": [11, 2]}, {"id": "c", "tokens": b[:2], "want": [1]}],
         "end": ["a", "c"]},
    ]
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dir), "--dtype", "float32",
                        "--out", str(out_dir), "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, env=env,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ya, yb = O.forward(CFG, P, a).float().numpy(), O.forward(CFG, P, b).float().numpy()
    got = {n: np.fromfile(out_dir / f"{n}.f32", dtype="<f4").reshape(-1, 30) for n in range(3)}
    np.testing.assert_allclose(got[0], ya[[7]], atol=2e-4)
    np.testing.assert_allclose(got[1], yb[[0, 8]], atol=2e-4)
    np.testing.assert_allclose(got[2], np.concatenate([ya[[20, 11]], yb[[1]]]), atol=2e-4)
