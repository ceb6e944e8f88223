"""GPU: the routing-index entry point that allocates nothing (momoe_index_build_static) gives
bit-identical results to momoe_index_build, on consecutive calls that share the library's fixed
scratch array, the later ones with smaller inputs."""
import ctypes

import pytest
import torch

from helpers import make_routing

pytestmark = pytest.mark.gpu


def _both(mask, K):
    from momoe_amd import _hip
    d = mask.to("cuda:0")
    a = _hip.index_build(d, K, static_scratch=True)
    b = _hip.index_build(d, K)
    torch.cuda.synchronize()
    return a, b


def test_static_scratch_index_build_matches_on_consecutive_calls():
    # large, then smaller, then tiny, then large again: stale panel counts of an earlier call
    # must never leak into a later one
    for M, N, K, Ks, skew in [(8192, 128, 8, 0, None), (1000, 60, 6, 2, 1.8), (16, 128, 8, 0, None),
                              (65536, 64, 8, 0, None)]:
        mask, _ = make_routing(M, N, K, Ks, seed=M, skew=skew)
        a, b = _both(mask, K)
        for k in ("sizes_N", "cumsums_N", "idx_Msum", "which_Msum", "inv_MK", "violations"):
            assert torch.equal(a[k], b[k]), (k, M, N)
        used = 4 + 4 * int(a["tile_table"][0])  # the entries past the last row tile are not written
        assert torch.equal(a["tile_table"][:used], b["tile_table"][:used])
        assert a["violations"].item() == 0
        assert torch.equal(a["sizes_N"].cpu(), (mask != 0).sum(1))


def test_static_scratch_allocates_nothing_and_refuses_oversized_inputs():
    from momoe_amd import _hip
    M, N, K = 4096, 64, 4
    mask, _ = make_routing(M, N, K, seed=1)
    d = mask.to("cuda:0")
    _hip.index_build(d, K, static_scratch=True)  # first call on the device: address look-up
    torch.cuda.synchronize()
    out = {k: torch.empty_like(v) for k, v in _hip.index_build(d, K, recompute_table=True).items()}
    out["violations"].zero_()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    rc = _hip._lib.momoe_index_build_static(
        d.data_ptr(), d.stride(0), d.stride(1), M, N, K, out["sizes_N"].data_ptr(),
        out["cumsums_N"].data_ptr(), out["idx_Msum"].data_ptr(), out["which_Msum"].data_ptr(),
        out["inv_MK"].data_ptr(), out["tile_table"].data_ptr(), _hip.AUTO_TILE_ROWS,
        out["recompute_table"].data_ptr(), out["violations"].data_ptr(),
        torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert rc == 0 and free_after == free_before  # no device memory was taken from the driver
    ref = _hip.index_build(d, K, recompute_table=True)
    torch.cuda.synchronize()
    for k in ("sizes_N", "cumsums_N", "idx_Msum", "which_Msum", "inv_MK"):
        assert torch.equal(out[k], ref[k]), k
    for k in ("tile_table", "recompute_table"):
        used = 4 + 4 * int(ref[k][0])
        assert torch.equal(out[k][:used], ref[k][:used]), k
    # 65536 tokens x 256 experts needs 4.2 MiB of panel counts: more than the fixed array
    z = ctypes.c_void_p(0)
    i64 = ctypes.c_int64
    assert _hip._lib.momoe_index_workspace_bytes(65536, 256) > 4 * 2**20
    assert _hip._lib.momoe_index_build_static(z, i64(1), i64(1), i64(65536), i64(256), i64(8), z, z, z, z,
                                              z, z, 256, z, z, z) == 2
