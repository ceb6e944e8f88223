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


def test_measured_traffic_is_what_the_committed_counter_summaries_say():
    # roofline.traffic must come from profiles/*_fetch_size.txt and *_write_size.txt, scaled by
    # the factors the calibration copy gave: read the two files here with a parser of our own
    # and compare with what bench.py derives from them, for every grouped GEMM.
    import re
    sys.path.insert(0, ROOT)
    import bench

    def table(path, counter):
        scale, rows = None, {}
        for line in open(os.path.join(ROOT, path)):
            m = re.match(r"== scale:\s*([0-9.]+)", line)
            if m:
                scale = float(m.group(1))
            m = re.match(r"(\S.*?)\s+%s\s+([0-9.]+)\s+\d+\s*$" % counter, line)
            if m:
                rows[m.group(1).strip()] = float(m.group(2))
        return scale, rows

    sf, fetch = table(bench.TRAFFIC_FILES["fetch"], "FETCH_SIZE")
    sw, write = table(bench.TRAFFIC_FILES["write"], "WRITE_SIZE")
    assert sf == 2.0 and sw == 1.0   # what a 256 MiB copy reads back through each counter
    gemms = set(bench.kernel_flops(2048, 1024, 65536))
    assert gemms <= set(bench.MEASURED_TRAFFIC_BYTES)
    alg = bench.gemm_algorithmic_bytes(8192, 2048, 1024, 128, 8)
    for prof_name, entry in bench.PROFILE_KERNELS.items():
        f = [v for k, v in fetch.items() if k.startswith(prof_name)]
        w = [v for k, v in write.items() if k.startswith(prof_name)]
        assert len(f) == 1 and len(w) == 1, prof_name
        want = (sf * f[0] + sw * w[0]) * 1024
        assert abs(bench.MEASURED_TRAFFIC_BYTES[entry] - want) <= 1, entry
        if entry in alg:   # a GEMM moves at least its operands and at most a few times that
            assert 1.0 <= want / alg[entry] < 3.0, (entry, want / alg[entry])
