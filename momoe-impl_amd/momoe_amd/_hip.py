"""ctypes binding of libmomoe_hip.so (the C ABI declared in include/momoe_hip.h).

The library is the only compute path: if it is missing or fails to load, importing
this module raises, and every wrapper raises RuntimeError on a non-zero status.
torch must be imported first so that the HIP runtime already loaded by torch is the
one the library binds to (both use the SONAME libamdhip64.so.7).
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmomoe_hip.so")

TILE_ROWS = 320            # MOMOE_TILE_ROWS: the tallest row tile
RECOMPUTE_TILE_ROWS = 256  # MOMOE_RECOMPUTE_TILE_ROWS: what lin1_swiglu_bwd takes
AUTO_TILE_ROWS = 0         # index_build: the library picks one of the two from the routing
GS_BLOCK = 128

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} not found: build it with `python momoe-impl_amd/build.py` "
        "(there is no fallback compute path)")

_lib = ctypes.CDLL(LIB_PATH)

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int

_SIGNATURES = {
    "momoe_abi_version": (_int, []),
    "momoe_status_string": (ctypes.c_char_p, [_int]),
    "momoe_set_clock_trace": (_int, [_p]),
    "momoe_mfma_rate_probe": (_i64, [_p, _p, _int, _p, _p]),
    "momoe_hbm_stream_probe": (_i64, [_p, _i64, _i64, _i64, _p]),
    "momoe_tile_table_ints": (_i64, [_i64, _i64, _i64, _int]),
    "momoe_index_workspace_bytes": (_i64, [_i64, _i64]),
    "momoe_index_build": (_int, [_p, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p, _int,
                                 _p, _p, _i64, _p, _p]),
    "momoe_tile_table_build": (_int, [_p, _i64, _i64, _int, _p, _p]),
    "momoe_index_build_static": (_int, [_p, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p,
                                        _int, _p, _p, _p]),
    "momoe_lin1_swiglu_fwd": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64,
                                     _i64, _p]),
    "momoe_lin2_scale_fwd": (_int, [_p, _p, _p, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i64,
                                    _i64, _p]),
    "momoe_combine": (_int, [_p, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "momoe_dgrad_h": (_int, [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p]),
    "momoe_lin1_swiglu_bwd": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _i64, _p,
                                     _i64, _i64, _i64, _i64, _i64, _p]),
    "momoe_swiglu_bwd_saved": (_int, [_p, _p, _p, _i64, _i64, _p, _p, _i64, _p, _p, _i64, _p, _i64,
                                      _i64, _i64, _i64, _i64, _p]),
    "momoe_gs_scatter": (_int, [_p, _i64, _p, _p, _p, _i64, _i64, _i64, _p]),
    "momoe_dgrad_x": (_int, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p]),
    "momoe_wgrad_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "momoe_padded_rows": (_i64, [_i64, _i64]),
    "momoe_wgrad": (_int, [_p, _i64, _int, _p, _p, _i64, _int, _p, _p, _p, _i64, _i64, _i64, _i64,
                           _i64, _p, _i64, _p]),
    "momoe_router_fwd": (_int, [_p, _int, _p, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p]),
    "momoe_router_bwd": (_int, [_p, _i64, _i64, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p, _p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

for _name, (_res, _args) in _SIGNATURES.items():
    _fn = getattr(_lib, _name)  # AttributeError here = library/header mismatch
    _fn.restype = _res
    _fn.argtypes = _args


def status_string(code):
    return _lib.momoe_status_string(int(code)).decode()


_TIMINGS = None  # list of (entry point, start event, end event) while kernel_timer() is active


class kernel_timer:
    """Context manager: record a HIP event pair around every C-ABI call made inside it
    (on torch's current stream).  `durations_ms()` synchronises and returns
    [(entry point, milliseconds), ...] in call order."""

    def __enter__(self):
        global _TIMINGS
        self.records = _TIMINGS = []
        return self

    def __exit__(self, *exc):
        global _TIMINGS
        _TIMINGS = None
        return False

    def durations_ms(self):
        torch.cuda.synchronize()
        return [(name, a.elapsed_time(b)) for name, a, b in self.records]


class clock_trace:
    """Context manager: average shader clock (MHz) under the grouped-GEMM kernels launched
    inside it, from the in-kernel clock64() / wall_clock64() counters (momoe_set_clock_trace)."""

    def __enter__(self):
        self.ticks = torch.zeros(2, dtype=torch.int64, device="cuda")
        _lib.momoe_set_clock_trace(self.ticks.data_ptr())
        return self

    def __exit__(self, *exc):
        _lib.momoe_set_clock_trace(None)
        return False

    def mhz(self):
        torch.cuda.synchronize()
        c, w = self.ticks.tolist()
        return 100.0 * c / w if w else float("nan")


def mfma_rate_probe(kind="gaussian", iters=20000, launches=3):
    """Sustained rate of the GEMMs' MFMA on register operands (momoe_mfma_rate_probe): returns
    (TFLOP/s, shader clock in MHz).  kind: "gaussian" = N(0,1) activations against N(0,0.02)
    weights, the layer's kind of data; "zeros"."""
    dev = "cuda"
    ops = torch.zeros(4096 * 8, dtype=torch.bfloat16, device=dev)
    if kind == "gaussian":
        g = torch.Generator(device=dev).manual_seed(5)
        # row-side fragments come from the first half of the buffer, column-side ones from the second
        v = torch.randn(4096, 8, generator=g, device=dev)
        v[2048:] *= 0.02
        ops = v.reshape(-1).to(torch.bfloat16)
    elif kind != "zeros":
        raise ValueError(kind)
    sink = torch.zeros(512, dtype=torch.float32, device=dev)
    ticks = torch.zeros(2, dtype=torch.int64, device=dev)
    st = _stream()
    flops = _lib.momoe_mfma_rate_probe(ops.data_ptr(), sink.data_ptr(), iters, ticks.data_ptr(), st)
    if flops < 0:
        raise RuntimeError("momoe_mfma_rate_probe failed")
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(launches):
        _lib.momoe_mfma_rate_probe(ops.data_ptr(), sink.data_ptr(), iters, ticks.data_ptr(), st)
    b.record()
    torch.cuda.synchronize()
    c, w = ticks.tolist()
    return flops * launches / (a.elapsed_time(b) * 1e-3) / 1e12, (100.0 * c / w if w else float("nan"))


def hbm_stream_probe(weights_NKC, launches=5):
    """GB/s at which the weight stream of the grouped GEMMs alone reads the bf16 tensor
    [blocks, krows, ncol] (momoe_hbm_stream_probe); give it more than the last-level cache holds."""
    blocks, krows, ncol = weights_NKC.shape
    st = _stream()
    args = (weights_NKC.data_ptr(), blocks, krows, ncol, st)
    nbytes = _lib.momoe_hbm_stream_probe(*args)
    if nbytes < 0:
        raise RuntimeError("momoe_hbm_stream_probe failed")
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(launches):
        _lib.momoe_hbm_stream_probe(*args)
    b.record()
    torch.cuda.synchronize()
    return nbytes * launches / (a.elapsed_time(b) * 1e-3) / 1e9


def _call(name, *args):
    fn = getattr(_lib, name)
    if _TIMINGS is None:
        code = fn(*args)
    else:
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        code = fn(*args)
        b.record()
        _TIMINGS.append((name, a, b))
    if code != 0:
        raise RuntimeError(f"{name} failed: status {code} ({status_string(code)})")


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("momoe_amd kernels need device tensors (no CPU compute path exists)")


def abi_version():
    return _lib.momoe_abi_version()


# ---------------------------------------------------------------- index build
def index_build(mask_NM, K, static_scratch=False, tile_rows=AUTO_TILE_ROWS, recompute_table=False):
    """mask_NM int32 [N,M] (any strides) -> dict of device tensors.
    See momoe_index_build in include/momoe_hip.h.  static_scratch=True goes through
    momoe_index_build_static: no workspace is allocated, the library's fixed array is used.
    recompute_table=True (only with tile_rows=AUTO_TILE_ROWS) also returns "recompute_table", the
    table of RECOMPUTE_TILE_ROWS-row tiles that lin1_swiglu_bwd walks."""
    _need_cuda(mask_NM)
    assert mask_NM.dtype == torch.int32 and mask_NM.dim() == 2
    N, M = mask_NM.shape
    dev = mask_NM.device
    msum = M * K
    sizes = torch.empty(N, dtype=torch.int64, device=dev)
    cumsums = torch.empty(N + 1, dtype=torch.int32, device=dev)
    idx = torch.empty(msum, dtype=torch.int32, device=dev)
    which = torch.empty(msum, dtype=torch.int32, device=dev)
    inv = torch.empty(msum, dtype=torch.int32, device=dev)
    table = torch.empty(_lib.momoe_tile_table_ints(M, N, K, tile_rows), dtype=torch.int32, device=dev)
    table_rc = None
    if recompute_table:
        table_rc = torch.empty(_lib.momoe_tile_table_ints(M, N, K, RECOMPUTE_TILE_ROWS), dtype=torch.int32,
                               device=dev)
    violations = torch.zeros(1, dtype=torch.int32, device=dev)
    if static_scratch:
        _call("momoe_index_build_static", _ptr(mask_NM), mask_NM.stride(0), mask_NM.stride(1), M, N,
              K, _ptr(sizes), _ptr(cumsums), _ptr(idx), _ptr(which), _ptr(inv), _ptr(table),
              tile_rows, _ptr(table_rc), _ptr(violations), _stream())
    else:
        ws_bytes = _lib.momoe_index_workspace_bytes(M, N)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        _call("momoe_index_build", _ptr(mask_NM), mask_NM.stride(0), mask_NM.stride(1), M, N, K,
              _ptr(sizes), _ptr(cumsums), _ptr(idx), _ptr(which), _ptr(inv), _ptr(table),
              tile_rows, _ptr(table_rc), _ptr(ws), ws_bytes, _ptr(violations), _stream())
    out = {"sizes_N": sizes, "cumsums_N": cumsums, "idx_Msum": idx, "which_Msum": which,
           "inv_MK": inv.view(M, K), "tile_table": table, "violations": violations}
    if table_rc is not None:
        out["recompute_table"] = table_rc
    return out


def tile_table_build(cumsums_N1, M, K, tile_rows):
    """The tile table of a finished index build for another tile height (momoe_tile_table_build)."""
    _need_cuda(cumsums_N1)
    N = cumsums_N1.numel() - 1
    table = torch.empty(_lib.momoe_tile_table_ints(M, N, K, tile_rows), dtype=torch.int32,
                        device=cumsums_N1.device)
    _call("momoe_tile_table_build", _ptr(cumsums_N1), N, M * K, tile_rows, _ptr(table), _stream())
    return table


# ---------------------------------------------------------------- experts fwd
def lin1_swiglu_fwd(x_MD, Wl1_ND2H, idx, table, h, ab, ab_lo, ab_hi):
    _need_cuda(x_MD, Wl1_ND2H)
    M, D = x_MD.shape
    N, _, H2 = Wl1_ND2H.shape
    _call("momoe_lin1_swiglu_fwd", _ptr(x_MD), _ptr(Wl1_ND2H), _ptr(idx), _ptr(table), _ptr(h),
                                      _ptr(ab), ab_lo, ab_hi, M, D, H2 // 2, N, idx.numel(),
                                      _stream())


def lin2_scale_fwd(h, Wl2_NHD, s_NM, idx, table, ys, M):
    _need_cuda(h, Wl2_NHD, s_NM)
    N, H, D = Wl2_NHD.shape
    _call("momoe_lin2_scale_fwd", _ptr(h), _ptr(Wl2_NHD), _ptr(s_NM), s_NM.stride(0),
                                     s_NM.stride(1), _ptr(idx), _ptr(table), _ptr(ys), M, D, H, N,
                                     idx.numel(), _stream())


def combine(rows_MsumD, inv_MK, out_MD):
    M, K = inv_MK.shape
    D = rows_MsumD.shape[1]
    _call("momoe_combine", _ptr(rows_MsumD), _ptr(inv_MK), _ptr(out_MD), M, D, K,
                              rows_MsumD.shape[0], _stream())


# ---------------------------------------------------------------- experts bwd
def dgrad_h(Gy_MD, Wl2_NHD, idx, table, u):
    _need_cuda(Gy_MD, Wl2_NHD)
    M, D = Gy_MD.shape
    N, H, _ = Wl2_NHD.shape
    _call("momoe_dgrad_h", _ptr(Gy_MD), _ptr(Wl2_NHD), _ptr(idx), _ptr(table), _ptr(u), M, D, H, N,
                              idx.numel(), _stream())


def lin1_swiglu_bwd(x_MD, Wl1_ND2H, idx, table, u, s_NM, row_lo, gz, hsT, gs_part):
    _need_cuda(x_MD, Wl1_ND2H, u, s_NM)
    M, D = x_MD.shape
    N, _, H2 = Wl1_ND2H.shape
    _call("momoe_lin1_swiglu_bwd", _ptr(x_MD), _ptr(Wl1_ND2H), _ptr(idx), _ptr(table), _ptr(u),
          _ptr(s_NM), s_NM.stride(0), s_NM.stride(1), row_lo, _ptr(gz), _ptr(hsT), hsT.shape[1],
          _ptr(gs_part), M, D, H2 // 2, N, idx.numel(), _stream())


def swiglu_bwd_saved(ab_save, u, s_NM, idx, cumsums, Msave, gz, hsT, gs_part):
    _need_cuda(ab_save, u, s_NM)
    N, M = s_NM.shape
    H = u.shape[1]
    _call("momoe_swiglu_bwd_saved", _ptr(ab_save), _ptr(u), _ptr(s_NM), s_NM.stride(0),
          s_NM.stride(1), _ptr(idx), _ptr(cumsums), Msave, _ptr(gz), _ptr(hsT), hsT.shape[1],
          _ptr(gs_part), gs_part.shape[0], M, H, N, idx.numel(), _stream())


def gs_scatter(gs_part, idx, cumsums, Gs_NM):
    N, M = Gs_NM.shape
    _call("momoe_gs_scatter", _ptr(gs_part), gs_part.shape[0], _ptr(idx), _ptr(cumsums),
                                 _ptr(Gs_NM), M, N, idx.numel(), _stream())


def dgrad_x(gz, Wl1_ND2H, table, gxs, M):
    """gz k-blocked: [2H/32, Msum, 32]."""
    N, D, H2 = Wl1_ND2H.shape
    _call("momoe_dgrad_x", _ptr(gz), _ptr(Wl1_ND2H), _ptr(table), _ptr(gxs), M, D, H2 // 2, N,
                              gz.shape[1], _stream())


def wgrad_workspace_bytes(N, X, Y, Msum):
    return _lib.momoe_wgrad_workspace_bytes(N, X, Y, Msum)


def padded_rows(Msum, N):
    return _lib.momoe_padded_rows(Msum, N)


def wgrad(A, a_gather, B, b_gather, cumsums, GW_NXY, M, Msum, workspace_bytes=None,
          a_transposed=False, b_transposed=False, b_kblocked=False):
    """GW[i] = A_i^T . B_i over the sorted rows of expert i.  An operand is [row, feature]
    (optionally gathered) or, with *_transposed, [padded sorted row / 32, feature, 32] as written
    by the SwiGLU backward kernels; B may also be k-blocked, [feature / 32, row, 32] (gz).
    workspace_bytes: scratch for the partial tiles of experts with many rows; default = the
    most the library can use for this shape, 0 = never cut an expert."""
    N, X, Y = GW_NXY.shape
    if workspace_bytes is None:
        workspace_bytes = wgrad_workspace_bytes(N, X, Y, Msum)
    ws = torch.empty(workspace_bytes, device=GW_NXY.device, dtype=torch.uint8) if workspace_bytes else None
    lda = A.shape[1] if a_transposed else A.stride(0)
    ldb = B.shape[1] if (b_transposed or b_kblocked) else B.stride(0)
    _call("momoe_wgrad", _ptr(A), lda, int(a_transposed), _ptr(a_gather), _ptr(B),
          ldb, 2 if b_kblocked else int(b_transposed), _ptr(b_gather), _ptr(cumsums), _ptr(GW_NXY), M, N, X, Y,
          Msum, _ptr(ws), workspace_bytes, _stream())


# ---------------------------------------------------------------- router
def router_fwd(logits_MN, biases_N, K, Ks):
    _need_cuda(logits_MN, biases_N)
    M, N = logits_MN.shape
    dev = logits_MN.device
    assert logits_MN.is_contiguous() and logits_MN.dtype in (torch.bfloat16, torch.float32)
    mask = torch.empty((N, M), dtype=torch.int32, device=dev)
    s_MN = torch.empty((M, N), dtype=torch.float32, device=dev)
    p_sel = torch.empty((M, N), dtype=torch.float32, device=dev)
    Ng_M = torch.empty(M, dtype=torch.float32, device=dev)
    Ks_M = torch.empty(M, dtype=torch.float32, device=dev)
    _call("momoe_router_fwd", _ptr(logits_MN), int(logits_MN.dtype == torch.float32),
                                 _ptr(biases_N), M, N, K, Ks, _ptr(mask), _ptr(s_MN), _ptr(p_sel),
                                 _ptr(Ng_M), _ptr(Ks_M), _stream())
    return mask, s_MN, p_sel, Ng_M, Ks_M


def router_bwd(Gs_NM, p_sel_MN, s_MN, Ng_M, Ks_M, mask_NM, Ks):
    N, M = Gs_NM.shape
    out = torch.empty((M, N), dtype=torch.bfloat16, device=Gs_NM.device)
    _call("momoe_router_bwd", _ptr(Gs_NM), Gs_NM.stride(0), Gs_NM.stride(1), _ptr(p_sel_MN),
                                 _ptr(s_MN), _ptr(Ng_M), _ptr(Ks_M), _ptr(mask_NM), M, N, Ks,
                                 _ptr(out), _stream())
    return out
