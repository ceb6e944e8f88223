"""bench.py's command-line contract that can be checked without a GPU."""
import os
import subprocess
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_headline_inputs_are_seeded_and_route_k_experts_per_token():
    sys.path.insert(0, ROOT)
    import bench
    a = bench.headline_inputs(64, 32, 16, 8, 2)
    b = bench.headline_inputs(64, 32, 16, 8, 2)
    for u, v in zip(a, b):
        assert torch.equal(u, v)
    x, W1, W2, mask, s, dy = a
    assert x.shape == (64, 32) and W1.shape == (8, 32, 32) and W2.shape == (8, 16, 32)
    assert mask.dtype == torch.int32 and torch.all(mask.sum(0) == 2)
    assert torch.allclose(s.sum(0), torch.ones(64), atol=1e-5) and torch.all(s[mask == 0] == 0)
