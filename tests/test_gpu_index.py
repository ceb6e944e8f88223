"""GPU: routing index build through the C ABI, bit-exact against the oracle."""
import numpy as np
import pytest
import torch

import oracle
from helpers import make_routing

pytestmark = pytest.mark.gpu


def _run(mask, K):
    from momoe_amd import _hip
    out = _hip.index_build(mask.to("cuda:0"), K, recompute_table=True)
    torch.cuda.synchronize()
    return {k: v.cpu() for k, v in out.items()}


def _check_table(t, o, tile_rows):
    # tile table: every expert's rows are covered exactly once, in order
    nt, bm = int(t[0]), int(t[1])
    assert bm == tile_rows
    ent = t[4:4 + 4 * nt].reshape(nt, 4)
    expect = []
    for i, (c0, sz) in enumerate(zip(o["cumsums_N"][:-1], o["sizes_N"])):
        first = len(expect)
        for _ in range(-(-int(sz) // bm)):
            expect.append((i, first, int(c0), int(sz)))
    assert ent.tolist() == [list(e) for e in expect]


def _compare(mask, K, out):
    from momoe_amd import _hip
    o = oracle.index_build(mask)
    assert out["sizes_N"].dtype == torch.int64 and out["cumsums_N"].dtype == torch.int32
    for k in ("sizes_N", "cumsums_N", "idx_Msum", "which_Msum"):
        assert np.array_equal(out[k].numpy(), o[k]), k
    assert np.array_equal(out["inv_MK"].numpy(), o["inv_MK"])
    assert out["violations"].item() == 0
    # left to choose, the library takes the taller tiles when they save more than 4 % of
    # sum over the tiles of (rows + 256), the bytes a tile streams per k
    def cost(rows):
        return sum(int(v) + 256 * -(-int(v) // rows) for v in o["sizes_N"])
    tall = cost(_hip.TILE_ROWS) * 26 < cost(_hip.RECOMPUTE_TILE_ROWS) * 25
    _check_table(out["tile_table"].numpy(), o, _hip.TILE_ROWS if tall else _hip.RECOMPUTE_TILE_ROWS)
    # the recomputing GEMM's table, written by the same call when asked for
    if "recompute_table" in out:
        _check_table(out["recompute_table"].numpy(), o, _hip.RECOMPUTE_TILE_ROWS)
    # the table for another tile height, made from the prefix sums alone
    M = mask.shape[1]
    for rows in (_hip.RECOMPUTE_TILE_ROWS, _hip.TILE_ROWS, 32):
        t = _hip.tile_table_build(out["cumsums_N"].to("cuda:0"), M, K, rows)
        torch.cuda.synchronize()
        _check_table(t.cpu().numpy(), o, rows)


@pytest.mark.parametrize("M,N,K,Ks,skew", [
    (128, 8, 2, 0, None),       # the tiny CPU-reference configuration
    (8192, 128, 8, 0, None),    # headline routing
    (1000, 60, 6, 0, None),     # M not a multiple of the 256-token panel, N not of the 16-expert panel
    (16384, 64, 8, 4, 1.8),     # skewed routing + 4 shared experts (full rows)
    (16, 128, 8, 0, None),      # decode-sized
    (1, 4, 4, 0, None),
    (65536, 64, 8, 0, None),    # largest token count of the configurations
    (4096, 64, 4, 0, None),     # experts of about 256 rows: half of them need a second 256-row tile
    # one token panel (M <= 256)
    (256, 128, 8, 0, None),     # a full panel
    (200, 300, 7, 2, None),     # 19 expert groups, two shared experts
    (255, 1024, 6, 0, 1.8),     # many experts, few tokens
    (256, 1025, 3, 0, None),    # N one past a multiple of the 16-expert panel
    (77, 17, 17, 0, None),      # every token on every expert, N just over one group
    # at most 64 tokens and 256 experts: the kernel with one thread per expert
    (64, 256, 8, 0, None),      # its largest case
    (33, 17, 17, 0, None),      # every token on every expert
    (48, 200, 7, 2, None),      # two shared experts, experts in all four wavefronts
    (17, 255, 6, 0, 1.8),       # skewed, one token past a chunk of 16
    (64, 257, 4, 0, None),      # one expert too many for it: the one-panel kernel
    (65, 256, 4, 0, None),      # one token too many
    # a few token panels
    (1024, 128, 8, 0, None),
    (257, 1, 1, 0, None),       # a single expert: one 320-row tile, two of 256 rows for the recomputing GEMM
    (1024, 64, 8, 4, 1.8),      # experts of up to 1024 rows: tall tiles chosen on the device
    (700, 128, 8, 0, 1.8),
])
def test_index_bit_exact(M, N, K, Ks, skew):
    mask, _ = make_routing(M, N, K, Ks, seed=11, skew=skew)
    _compare(mask, K, _run(mask, K))


def test_index_with_a_given_tile_height():
    from momoe_amd import _hip
    mask, _ = make_routing(8192, 128, 8, seed=11)
    o = oracle.index_build(mask)
    for rows in (_hip.TILE_ROWS, _hip.RECOMPUTE_TILE_ROWS, 64):
        out = _hip.index_build(mask.to("cuda:0"), 8, tile_rows=rows)
        torch.cuda.synchronize()
        _check_table(out["tile_table"].cpu().numpy(), o, rows)


def test_tile_heights_no_kernel_takes_are_refused():
    from momoe_amd import _hip
    mask, _ = make_routing(300, 8, 2, seed=1)
    # the second table comes with the library's own choice of the height only
    with pytest.raises(RuntimeError):
        _hip.index_build(mask.to("cuda:0"), 2, tile_rows=_hip.RECOMPUTE_TILE_ROWS, recompute_table=True)
    with pytest.raises(RuntimeError):
        _hip.index_build(mask.to("cuda:0"), 2, tile_rows=_hip.TILE_ROWS + 32)
    ib = _hip.index_build(mask.to("cuda:0"), 2)
    # heights below one 32-row fragment row, or not a whole number of them, would give tiles
    # without rows: refused on the host, nothing is launched
    for rows in (1, 16, 31, 48, 250, _hip.TILE_ROWS + 1):
        with pytest.raises(RuntimeError):
            _hip.index_build(mask.to("cuda:0"), 2, tile_rows=rows)
        with pytest.raises(RuntimeError):
            _hip.tile_table_build(ib["cumsums_N"], 300, 2, rows)
    with pytest.raises(RuntimeError):
        _hip.tile_table_build(ib["cumsums_N"], 300, 2, 0)


def test_index_strided_mask():
    mask, _ = make_routing(777, 24, 3, seed=2)
    strided = mask.T.contiguous().to("cuda:0").T  # strides (1, N)
    from momoe_amd import _hip
    out = {k: v.cpu() for k, v in _hip.index_build(strided, 3).items()}
    _compare(mask, 3, out)


def test_violation_counter_and_no_out_of_bounds():
    mask, _ = make_routing(512, 16, 4, seed=3)
    bad = mask.clone()
    bad[:, 5] = 0          # token 5 has no expert
    bad[0:6, 9] = 1        # token 9 has more than K
    out = _run(bad, 4)
    assert out["violations"].item() >= 2
    # too many pairs in total: both tile tables are emptied
    out = _run(torch.ones(16, 512, dtype=torch.int32), 4)
    assert out["violations"].item() >= 1
    assert out["tile_table"][0].item() == 0 and out["recompute_table"][0].item() == 0
    assert out["recompute_table"][1].item() == 256


def test_violations_single_panel():
    mask, _ = make_routing(100, 40, 4, seed=4)
    bad = mask.clone()
    bad[:, 5] = 0          # token 5 has no expert
    bad[0:6, 9] = 1        # token 9 has more than K
    out = _run(bad, 4)
    assert out["violations"].item() >= 2
    # too many pairs in total: the tile table is emptied so that the GEMMs do nothing
    over = torch.ones(40, 100, dtype=torch.int32)
    out = _run(over, 4)
    assert out["violations"].item() >= 1 and out["tile_table"][0].item() == 0
    assert out["recompute_table"][0].item() == 0
    # a table made from those prefix sums is empty as well
    from momoe_amd import _hip
    t = _hip.tile_table_build(out["cumsums_N"].to("cuda:0"), 100, 4, _hip.RECOMPUTE_TILE_ROWS)
    assert t[0].item() == 0


def test_strided_mask_single_panel():
    mask, _ = make_routing(130, 24, 3, seed=2)
    strided = mask.T.contiguous().to("cuda:0").T  # strides (1, N)
    from momoe_amd import _hip
    out = {k: v.cpu() for k, v in _hip.index_build(strided, 3).items()}
    _compare(mask, 3, out)


def test_experts_without_tokens():
    mask = torch.zeros(8, 300, dtype=torch.int32)
    mask[1] = 1
    mask[6] = 1
    out = _run(mask, 2)
    _compare(mask, 2, out)
    assert out["sizes_N"].tolist() == [0, 300, 0, 0, 0, 0, 300, 0]


def test_routing_with_missing_pairs_leaves_nothing_undefined():
    # tokens with fewer than K experts: the sorted rows past the last pair get token 0 / slot 0
    # and the token's unused slots of inv_MK say "no row" (-1)
    M, N, K = 600, 20, 4
    mask, _ = make_routing(M, N, K, seed=8)
    short = mask.clone()
    short[:, 17] = 0
    for m in (3, 300, 599):
        short[int(torch.nonzero(short[:, m])[-1]), m] = 0
    out = _run(short, K)
    o = oracle.index_build(short)
    total = int(o["cumsums_N"][-1])
    assert total == M * K - K - 3 and out["violations"].item() == 4
    for k in ("sizes_N", "cumsums_N"):
        assert np.array_equal(out[k].numpy(), o[k]), k
    assert np.array_equal(out["idx_Msum"].numpy()[:total], o["idx_Msum"])
    assert np.array_equal(out["which_Msum"].numpy()[:total], o["which_Msum"])
    assert np.all(out["idx_Msum"].numpy()[total:] == 0) and np.all(out["which_Msum"].numpy()[total:] == 0)
    assert np.array_equal(out["inv_MK"].numpy(), o["inv_MK"])  # the oracle writes -1 for missing pairs


def test_violations_strides_and_missing_pairs_with_one_thread_per_expert():
    # the same checks at 64 tokens or fewer, where another kernel builds the index
    from momoe_amd import _hip
    M, N, K = 40, 130, 4
    mask, _ = make_routing(M, N, K, seed=5)
    strided = mask.T.contiguous().to("cuda:0").T  # strides (1, N)
    _compare(mask, K, {k: v.cpu() for k, v in _hip.index_build(strided, K).items()})
    # views into a wider matrix: rows that start 16 bytes / 4 bytes into a line (the kernel reads
    # aligned rows of a multiple of four tokens with 16-byte loads, anything else entry by entry)
    wide = torch.zeros(N, M + 8, dtype=torch.int32)
    for first in (4, 1):
        wide.zero_()
        wide[:, first:first + M] = mask
        view = wide.to("cuda:0")[:, first:first + M]
        assert not view.is_contiguous()
        _compare(mask, K, {k: v.cpu() for k, v in _hip.index_build(view, K).items()})
    bad = mask.clone()
    bad[:, 5] = 0          # token 5 has no expert
    bad[0:6, 9] = 1        # token 9 has more than K
    out = _run(bad, K)
    assert out["violations"].item() >= 2
    over = torch.ones(N, M, dtype=torch.int32)
    out = _run(over, K)
    assert out["violations"].item() >= 1 and out["tile_table"][0].item() == 0
    assert np.all(out["inv_MK"].numpy() == -1)
    short = mask.clone()
    short[:, 17] = 0
    for m in (3, 20, 39):
        short[int(torch.nonzero(short[:, m])[-1]), m] = 0
    out = _run(short, K)
    o = oracle.index_build(short)
    total = int(o["cumsums_N"][-1])
    assert total == M * K - K - 3 and out["violations"].item() == 4
    for k in ("sizes_N", "cumsums_N"):
        assert np.array_equal(out[k].numpy(), o[k]), k
    assert np.array_equal(out["idx_Msum"].numpy()[:total], o["idx_Msum"])
    assert np.array_equal(out["which_Msum"].numpy()[:total], o["which_Msum"])
    assert np.all(out["idx_Msum"].numpy()[total:] == 0) and np.all(out["which_Msum"].numpy()[total:] == 0)
    assert np.array_equal(out["inv_MK"].numpy(), o["inv_MK"])


def test_random_shapes_up_to_1024_tokens():
    # 60 seeded shapes: the single-launch kernels (one thread per expert up to 64 tokens, one per
    # token up to 256 tokens and 256 experts) and a few token panels, routed and shared experts
    # mixed, contiguous and transposed masks
    from momoe_amd import _hip
    rng = np.random.default_rng(17)
    for case in range(60):
        M = int(rng.integers(1, 65)) if case % 3 == 0 else int(rng.integers(65, 257)) if case % 3 == 1 else int(rng.integers(257, 1025))
        N = int(rng.integers(1, 257)) if M <= 256 else int(rng.integers(1, 129))
        K = int(rng.integers(1, min(N, 12) + 1))
        Ks = int(rng.integers(0, K)) if case % 5 == 0 else 0
        mask, _ = make_routing(M, N, K, Ks, seed=100 + case, skew=1.8 if case % 7 == 0 else None)
        dev = mask.to("cuda:0")
        if case % 4 == 0:
            dev = mask.T.contiguous().to("cuda:0").T
        out = {k: v.cpu() for k, v in _hip.index_build(dev, K, recompute_table=case % 4 != 1).items()}
        try:
            _compare(mask, K, out)
        except AssertionError as e:
            raise AssertionError(f"case {case}: M={M} N={N} K={K} Ks={Ks}: {e}") from e
