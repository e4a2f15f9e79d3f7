"""ctypes binding of the C-ABI in include/fluxmi.h.

Thin on purpose: arguments are torch tensors (device memory + the current HIP stream come from
PyTorch-ROCm), every call goes straight to libfluxmi_kernels.so and a non-zero status becomes a
RuntimeError carrying fluxmi_last_error().  There is no fallback: a missing library raises on load.
"""
import ctypes
import os

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libfluxmi_kernels.so")
_lib = None

BF16 = 0
FP8_E4M3 = 1
FP16 = 2
_DTYPES = {torch.bfloat16: BF16, torch.float8_e4m3fn: FP8_E4M3, torch.float16: FP16}


def _half_out(in_dtype):
    """16-bit output type of an operand type: fp16 operands give fp16, bf16 and fp8 give bf16."""
    return torch.float16 if in_dtype == torch.float16 else torch.bfloat16


EXPORTS = (
    "fluxmi_version", "fluxmi_last_error", "fluxmi_device_cu_count",
    "fluxmi_moe_route_sort_workspace_bytes", "fluxmi_moe_route_sort", "fluxmi_moe_gather_index",
    "fluxmi_moe_route_sort_static_max_bytes", "fluxmi_moe_route_sort_static_init", "fluxmi_moe_route_sort_static",
    "fluxmi_grouped_gemm_workspace_bytes", "fluxmi_grouped_gemm", "fluxmi_grouped_gemm_kernel_kind",
    "fluxmi_grouped_gemm_multi", "fluxmi_grouped_gemm_topk_reduce_workspace_bytes",
    "fluxmi_grouped_gemm_topk_reduce", "fluxmi_grouped_gemm_blockscale",
    "fluxmi_topk_gather_reduce", "fluxmi_quant_e4m3_rowwise", "fluxmi_quant_e4m3_square",
    "fluxmi_quant_e4m3_block128", "fluxmi_calib_stream_sink_bytes", "fluxmi_calib_stream",
)


class GroupedGemmArgs(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32), ("nexperts", ctypes.c_int32), ("max_rows", ctypes.c_int32),
        ("n", ctypes.c_int32), ("k", ctypes.c_int32), ("a_rows", ctypes.c_int32),
        ("a", ctypes.c_void_p), ("b", ctypes.c_void_p), ("d", ctypes.c_void_p),
        ("splits", ctypes.c_void_p), ("gather_a", ctypes.c_void_p), ("scatter_d", ctypes.c_void_p),
        ("alpha", ctypes.c_void_p), ("row_scale", ctypes.c_void_p), ("col_scale", ctypes.c_void_p),
        ("scalar_scale", ctypes.c_float), ("d_fp32", ctypes.c_int32),
        ("scalar_scale_dev", ctypes.c_void_p),
        ("cu_margin", ctypes.c_int32), ("raster_rows", ctypes.c_int32), ("sched_flags", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


def lib_path():
    return _LIB_PATH


def load():
    """Load libfluxmi_kernels.so (after torch, so that both share one HIP runtime)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with `python -m flux_amd.build` (there is no fallback path)")
    lib = ctypes.CDLL(_LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    vp, i32, i64, f32, sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t
    lib.fluxmi_version.restype = ctypes.c_int
    lib.fluxmi_last_error.restype = ctypes.c_char_p
    lib.fluxmi_device_cu_count.restype = ctypes.c_int
    lib.fluxmi_moe_route_sort_workspace_bytes.restype = sz
    lib.fluxmi_moe_route_sort_workspace_bytes.argtypes = [i32, i32, i32]
    lib.fluxmi_moe_route_sort.argtypes = [vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, sz, vp]
    lib.fluxmi_moe_gather_index.argtypes = [vp, i32, i32, vp, vp, vp]
    lib.fluxmi_moe_route_sort_static_max_bytes.restype = sz
    lib.fluxmi_moe_route_sort_static.argtypes = [vp, i32, i32, i32, vp, vp, vp, vp, vp, vp]
    lib.fluxmi_grouped_gemm_workspace_bytes.restype = sz
    lib.fluxmi_grouped_gemm_workspace_bytes.argtypes = [ctypes.POINTER(GroupedGemmArgs)]
    lib.fluxmi_grouped_gemm.argtypes = [ctypes.POINTER(GroupedGemmArgs), vp, sz, vp]
    lib.fluxmi_grouped_gemm_kernel_kind.argtypes = [ctypes.POINTER(GroupedGemmArgs)]
    lib.fluxmi_grouped_gemm_topk_reduce_workspace_bytes.restype = sz
    lib.fluxmi_grouped_gemm_topk_reduce_workspace_bytes.argtypes = [i32, i32]
    lib.fluxmi_grouped_gemm_topk_reduce.argtypes = [ctypes.POINTER(GroupedGemmArgs), vp, i32, vp, vp, sz, vp]
    lib.fluxmi_grouped_gemm_blockscale.argtypes = [ctypes.POINTER(GroupedGemmArgs), vp, i32, vp, i32, vp]
    lib.fluxmi_grouped_gemm_multi.argtypes = [ctypes.POINTER(GroupedGemmArgs), i32, vp, vp, vp, vp, sz, vp]
    lib.fluxmi_topk_gather_reduce.argtypes = [ctypes.POINTER(vp), i32, i32, vp, vp, f32, i32, i32, i32, vp, vp]
    lib.fluxmi_quant_e4m3_rowwise.argtypes = [vp, i64, i64, i32, f32, vp, vp, i32, vp]
    lib.fluxmi_quant_e4m3_square.argtypes = [vp, i64, i64, i64, f32, vp, vp, vp, vp, vp]
    lib.fluxmi_quant_e4m3_block128.argtypes = [vp, i64, i64, f32, vp, vp, vp, vp, vp]
    lib.fluxmi_calib_stream_sink_bytes.restype = sz
    lib.fluxmi_calib_stream.argtypes = [vp, vp, sz, i32, vp]
    _lib = lib
    return lib


def _check(status, what):
    if status != 0:
        raise RuntimeError(f"{what} failed ({status}): {load().fluxmi_last_error().decode()}")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev_tensor(t, dtype, name):
    if t is None:
        return
    if not t.is_cuda or not t.is_contiguous() or t.dtype != dtype:
        raise ValueError(f"{name} must be a contiguous device tensor of {dtype}, got {t.dtype} on {t.device}")


def route_sort(choosed, nexperts, want_gather=True, want_topk_index=True):
    """-> (splits[E], offsets[E+1], scatter_index like choosed, gather_index[M], topk_index[M])."""
    lib = load()
    _dev_tensor(choosed, torch.int32, "choosed")
    ntokens, topk = choosed.shape
    dev = choosed.device
    m = ntokens * topk
    splits = torch.empty(nexperts, dtype=torch.int32, device=dev)
    offsets = torch.empty(nexperts + 1, dtype=torch.int32, device=dev)
    scatter = torch.empty_like(choosed)
    gather = torch.empty(m, dtype=torch.int32, device=dev) if want_gather else None
    tki = torch.empty(m, dtype=torch.int32, device=dev) if want_topk_index else None
    ws_bytes = lib.fluxmi_moe_route_sort_workspace_bytes(ntokens, topk, nexperts)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    _check(lib.fluxmi_moe_route_sort(_ptr(choosed), ntokens, topk, nexperts, _ptr(splits), _ptr(offsets),
                                     _ptr(scatter), _ptr(gather), _ptr(tki), _ptr(ws), ws_bytes, _stream()),
           "fluxmi_moe_route_sort")
    return splits, offsets, scatter, gather, tki


def route_sort_static(choosed, nexperts, out):
    """fluxmi_moe_route_sort_static into the caller's tensors `out` = (splits, offsets, scatter_index,
    gather_index, topk_index), the last two optional (None).  Allocates nothing, here or in the library."""
    lib = load()
    _dev_tensor(choosed, torch.int32, "choosed")
    ntokens, topk = choosed.shape
    splits, offsets, scatter, gather, tki = out
    for nm, t in (("splits", splits), ("offsets", offsets), ("scatter_index", scatter), ("gather_index", gather),
                  ("topk_index", tki)):
        _dev_tensor(t, torch.int32, nm)
    _check(lib.fluxmi_moe_route_sort_static(_ptr(choosed), ntokens, topk, nexperts, _ptr(splits), _ptr(offsets),
                                            _ptr(scatter), _ptr(gather), _ptr(tki), _stream()),
           "fluxmi_moe_route_sort_static")
    return out


def gather_index(scatter_index, topk):
    lib = load()
    _dev_tensor(scatter_index, torch.int32, "scatter_index")
    m = scatter_index.numel()
    gather = torch.empty(m, dtype=torch.int32, device=scatter_index.device)
    tki = torch.empty(m, dtype=torch.int32, device=scatter_index.device)
    _check(lib.fluxmi_moe_gather_index(_ptr(scatter_index), m, topk, _ptr(gather), _ptr(tki), _stream()),
           "fluxmi_moe_gather_index")
    return gather, tki


SCHED_WHOLE_TAIL_TILES = 1
SCHED_NO_HALF_TILES = 2
SCHED_NO_SKINNY_TAIL = 4
SCHED_FORCE_SKINNY_TAIL = 8
SCHED_HALF_LINE_FILLS = 16
SCHED_WHOLE_LINE_FILLS = 32


# Form of the MFMA kernel's ring fills for calls that name none themselves: 0 (the library's rule by shape),
# SCHED_HALF_LINE_FILLS or SCHED_WHOLE_LINE_FILLS.  Results are bit-identical either way.
default_fill_form = 0


def _gemm_args(a, b, splits, out, gather_a, scatter_d, alpha, row_scale, col_scale, scalar_scale, scalar_scale_dev,
               max_rows, out_dtype, cu_margin, raster_rows, sched_flags, need_out=True):
    if not sched_flags & (SCHED_HALF_LINE_FILLS | SCHED_WHOLE_LINE_FILLS):
        sched_flags |= default_fill_form
    dtype = _DTYPES.get(a.dtype)
    if dtype is None:
        raise ValueError(f"unsupported input dtype {a.dtype}")
    _dev_tensor(a, a.dtype, "a")
    _dev_tensor(b, a.dtype, "b")
    _dev_tensor(splits, torch.int32, "splits")
    _dev_tensor(gather_a, torch.int32, "gather_a")
    _dev_tensor(scatter_d, torch.int32, "scatter_d")
    for nm, t in (("alpha", alpha), ("row_scale", row_scale), ("col_scale", col_scale),
                  ("scalar_scale_dev", scalar_scale_dev)):
        _dev_tensor(t, torch.float32, nm)
    e, n, k = b.shape
    if a.shape[1] != k:
        raise ValueError(f"K mismatch: a {tuple(a.shape)} vs b {tuple(b.shape)}")
    if max_rows is None:
        max_rows = gather_a.numel() if gather_a is not None else a.shape[0]
    if need_out:
        if out is None:
            out = torch.empty(max_rows, n, dtype=out_dtype or _half_out(a.dtype), device=a.device)
        if out.dtype not in (_half_out(a.dtype), torch.float32):
            raise ValueError(f"out must be {_half_out(a.dtype)} or fp32, got {out.dtype}")
        _dev_tensor(out, out.dtype, "out")
        if out.shape[0] < max_rows or out.shape[1] != n:
            raise ValueError(f"out {tuple(out.shape)} too small for [{max_rows}, {n}]")
    args = GroupedGemmArgs(
        dtype=dtype, nexperts=e, max_rows=max_rows, n=n, k=k, a_rows=a.shape[0],
        a=a.data_ptr(), b=b.data_ptr(), d=out.data_ptr() if need_out else None, splits=splits.data_ptr(),
        gather_a=None if gather_a is None else gather_a.data_ptr(),
        scatter_d=None if scatter_d is None else scatter_d.data_ptr(),
        alpha=None if alpha is None else alpha.data_ptr(),
        row_scale=None if row_scale is None else row_scale.data_ptr(),
        col_scale=None if col_scale is None else col_scale.data_ptr(),
        scalar_scale=float(scalar_scale), d_fp32=int(need_out and out.dtype == torch.float32),
        scalar_scale_dev=None if scalar_scale_dev is None else scalar_scale_dev.data_ptr(),
        cu_margin=cu_margin, raster_rows=raster_rows, sched_flags=sched_flags)
    return args, out


def grouped_gemm(a, b, splits, out=None, gather_a=None, scatter_d=None, alpha=None, row_scale=None,
                 col_scale=None, scalar_scale=1.0, scalar_scale_dev=None, max_rows=None, out_dtype=None,
                 cu_margin=0, raster_rows=0, sched_flags=0, want_kind=False):
    """D = grouped GEMM of A [rows_a, K] with B [E, N, K]; see fluxmi_grouped_gemm in include/fluxmi.h.
    With `want_kind` the result is (D, kind): kind 1 = the MFMA kernel ran, 0 = the generic kernel."""
    lib = load()
    args, out = _gemm_args(a, b, splits, out, gather_a, scatter_d, alpha, row_scale, col_scale, scalar_scale,
                           scalar_scale_dev, max_rows, out_dtype, cu_margin, raster_rows, sched_flags)
    _check(lib.fluxmi_grouped_gemm(ctypes.byref(args), None, 0, _stream()), "fluxmi_grouped_gemm")
    if want_kind:
        return out, lib.fluxmi_grouped_gemm_kernel_kind(ctypes.byref(args))
    return out


ASCALE_BLOCK128, ASCALE_EXPERT_K_M = 0, 1
BSCALE_N_K, BSCALE_K_N = 0, 1


def grouped_gemm_blockscale(a, b, splits, a_scale, b_scale, a_scale_layout=ASCALE_BLOCK128, b_scale_layout=BSCALE_N_K,
                            out=None, gather_a=None, scatter_d=None, alpha=None, row_scale=None, col_scale=None,
                            scalar_scale=1.0, max_rows=None, out_dtype=None):
    """Block-scaled fp8 grouped GEMM (fluxmi_grouped_gemm_blockscale): a_scale per (row of A, 128 of K), b_scale
    per 128 x 128 block of each B[e]; layouts as in include/fluxmi.h."""
    lib = load()
    _dev_tensor(a_scale, torch.float32, "a_scale")
    _dev_tensor(b_scale, torch.float32, "b_scale")
    args, out = _gemm_args(a, b, splits, out, gather_a, scatter_d, alpha, row_scale, col_scale, scalar_scale, None,
                           max_rows, out_dtype, 0, 0, 0)
    _check(lib.fluxmi_grouped_gemm_blockscale(ctypes.byref(args), _ptr(a_scale), a_scale_layout, _ptr(b_scale),
                                              b_scale_layout, _stream()), "fluxmi_grouped_gemm_blockscale")
    return out


def grouped_gemm_topk_reduce(a, b, splits, token_of_row, ntokens, out=None, workspace=None, gather_a=None, alpha=None,
                             row_scale=None, col_scale=None, scalar_scale=1.0, scalar_scale_dev=None, max_rows=None):
    """out[t] = bf16(sum of the scaled GEMM rows r with token_of_row[r] == t): the top-k reduction fused into the
    grouped GEMM's epilogue (fluxmi_grouped_gemm_topk_reduce).  `workspace`: fp32 [ntokens, N] scratch."""
    lib = load()
    _dev_tensor(token_of_row, torch.int32, "token_of_row")
    args, _ = _gemm_args(a, b, splits, None, gather_a, None, alpha, row_scale, col_scale, scalar_scale,
                         scalar_scale_dev, max_rows, None, 0, 0, 0, need_out=False)
    n = b.shape[1]
    if out is None:
        out = torch.empty(ntokens, n, dtype=_half_out(a.dtype), device=a.device)
    _dev_tensor(out, _half_out(a.dtype), "out")
    ws_bytes = lib.fluxmi_grouped_gemm_topk_reduce_workspace_bytes(ntokens, n)
    if workspace is None:
        workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=a.device)
    _check(lib.fluxmi_grouped_gemm_topk_reduce(ctypes.byref(args), _ptr(token_of_row), ntokens, _ptr(out),
                                               _ptr(workspace), workspace.numel() * workspace.element_size(), _stream()),
           "fluxmi_grouped_gemm_topk_reduce")
    return out


def grouped_gemm_multi(a, bs, splits, outs=None, gather_a=None, alphas=None, row_scale=None, col_scale=None,
                       scalar_scale=1.0, max_rows=None, out_dtype=None, raster_rows=0, sched_flags=0):
    """[A @ B_g for B_g in bs] in one launch (fluxmi_grouped_gemm_multi): the same sorted rows times up to four
    weight tensors [E, N, K], each with its own output and optional per-expert alpha."""
    lib = load()
    dtype = _DTYPES.get(a.dtype)
    if dtype is None:
        raise ValueError(f"unsupported input dtype {a.dtype}")
    ng = len(bs)
    _dev_tensor(a, a.dtype, "a")
    for b in bs:
        _dev_tensor(b, a.dtype, "b")
        if b.shape != bs[0].shape:
            raise ValueError("all weight groups must have one shape")
    _dev_tensor(splits, torch.int32, "splits")
    _dev_tensor(gather_a, torch.int32, "gather_a")
    _dev_tensor(row_scale, torch.float32, "row_scale")
    _dev_tensor(col_scale, torch.float32, "col_scale")
    e, n, k = bs[0].shape
    if a.shape[1] != k:
        raise ValueError(f"K mismatch: a {tuple(a.shape)} vs b {tuple(bs[0].shape)}")
    if max_rows is None:
        max_rows = gather_a.numel() if gather_a is not None else a.shape[0]
    if outs is None:
        outs = [torch.empty(max_rows, n, dtype=out_dtype or _half_out(a.dtype), device=a.device) for _ in range(ng)]
    for o in outs:
        _dev_tensor(o, outs[0].dtype, "out")
        if o.dtype not in (_half_out(a.dtype), torch.float32) or o.shape[0] < max_rows or o.shape[1] != n:
            raise ValueError(f"out {tuple(o.shape)} {o.dtype} does not fit [{max_rows}, {n}] bf16/fp32")
    if len(outs) != ng or (alphas is not None and len(alphas) != ng):
        raise ValueError("outs / alphas need one entry per weight group")
    for al in alphas or ():
        _dev_tensor(al, torch.float32, "alpha")
    args = GroupedGemmArgs(
        dtype=dtype, nexperts=e, max_rows=max_rows, n=n, k=k, a_rows=a.shape[0], a=a.data_ptr(), b=None, d=None,
        splits=splits.data_ptr(), gather_a=None if gather_a is None else gather_a.data_ptr(), scatter_d=None,
        alpha=None, row_scale=None if row_scale is None else row_scale.data_ptr(),
        col_scale=None if col_scale is None else col_scale.data_ptr(), scalar_scale=float(scalar_scale),
        d_fp32=int(outs[0].dtype == torch.float32), scalar_scale_dev=None, raster_rows=raster_rows,
        sched_flags=sched_flags)
    vps = ctypes.c_void_p * ng
    b_arr = vps(*[b.data_ptr() for b in bs])
    d_arr = vps(*[o.data_ptr() for o in outs])
    al_arr = None if alphas is None else vps(*[None if al is None else al.data_ptr() for al in alphas])
    _check(lib.fluxmi_grouped_gemm_multi(ctypes.byref(args), ng, b_arr, d_arr, al_arr, None, 0, _stream()),
           "fluxmi_grouped_gemm_multi")
    return outs


def topk_gather_reduce(inputs, routing_idx, topk, row_weight=None, scale=1.0, out=None, out_dtype=None):
    """out[t] = bf16(scale * sum_g sum_j w[r] * inputs[g][r]), r = routing_idx[t*topk+j].  fp16 inputs give an fp16
    result; fp32 inputs give bf16 unless out / out_dtype say fp16."""
    lib = load()
    if isinstance(inputs, torch.Tensor):
        inputs = [inputs]
    in_dtype = inputs[0].dtype
    if in_dtype not in (torch.bfloat16, torch.float32, torch.float16):
        raise ValueError(f"inputs must be bf16, fp16 or fp32, got {in_dtype}")
    for g, t in enumerate(inputs):
        _dev_tensor(t, in_dtype, f"inputs[{g}]")
    _dev_tensor(routing_idx, torch.int32, "routing_idx")
    _dev_tensor(row_weight, torch.float32, "row_weight")
    m, n = inputs[0].shape
    if routing_idx.numel() % topk:
        raise ValueError("routing_idx length is not a multiple of topk")
    ntokens = routing_idx.numel() // topk
    if out is None:
        out = torch.empty(ntokens, n, dtype=out_dtype or _half_out(in_dtype), device=inputs[0].device)
    if out.dtype != (_half_out(in_dtype) if in_dtype != torch.float32 else out.dtype) or out.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError(f"out dtype {out.dtype} does not go with {in_dtype} inputs")
    io_format = int(in_dtype == torch.float32) | (2 if out.dtype == torch.float16 else 0)
    ptrs = (ctypes.c_void_p * len(inputs))(*[t.data_ptr() for t in inputs])
    _check(lib.fluxmi_topk_gather_reduce(ptrs, len(inputs), io_format, _ptr(routing_idx), _ptr(row_weight),
                                         float(scale), ntokens, topk, n, _ptr(out), _stream()),
           "fluxmi_topk_gather_reduce")
    return out


def quant_e4m3(x, block_cols=0, eps=0.0, permute_scale=False, out=None):
    """-> (q fp8_e4m3fn like x, scale_inv fp32).  block_cols 0 = one scale per row, 128 = 1x128 blocks.
    `out` = (q, scale_inv) of a previous call with the same arguments writes into those tensors."""
    lib = load()
    _dev_tensor(x, torch.bfloat16, "x")
    rows, cols = x.shape
    if out is not None:
        q, si = out
        if q.shape != x.shape or q.dtype != torch.float8_e4m3fn or si.dtype != torch.float32 or not (
                q.is_cuda and si.is_cuda and q.is_contiguous() and si.is_contiguous()):
            raise ValueError("out must be the (q, scale_inv) pair of a call with the same arguments")
        want = rows if block_cols == 0 else (
            (rows + 127) // 128 * 128 if permute_scale else rows) * ((cols + block_cols - 1) // block_cols)
        if si.numel() != want:
            raise ValueError(f"scale_inv has {si.numel()} entries, expected {want}")
    else:
        q = torch.empty(rows, cols, dtype=torch.float8_e4m3fn, device=x.device)
    if out is not None:
        pass
    elif block_cols == 0:
        si = torch.empty(rows, dtype=torch.float32, device=x.device)
    else:
        nb = (cols + block_cols - 1) // block_cols
        if permute_scale:
            si = torch.zeros((rows + 127) // 128, nb, 128, dtype=torch.float32, device=x.device)
        else:
            si = torch.empty(rows, nb, dtype=torch.float32, device=x.device)
    _check(lib.fluxmi_quant_e4m3_rowwise(_ptr(x), rows, cols, block_cols, float(eps), _ptr(q), _ptr(si),
                                         int(permute_scale), _stream()), "fluxmi_quant_e4m3_rowwise")
    return q, si


def quant_e4m3_square(x, eps=0.0, transpose=False):
    """x [rows, cols] or [batch, rows, cols] bf16 -> (q, scale_inv [.., rows/128, cols/128], q_t, scale_inv_t);
    the last two are None without `transpose`.  One scale per 128 x 128 block."""
    lib = load()
    _dev_tensor(x, torch.bfloat16, "x")
    lead = tuple(x.shape[:-2])
    if len(lead) > 1:
        raise ValueError("x must have 2 or 3 dimensions")
    batch = lead[0] if lead else 1
    rows, cols = x.shape[-2:]
    nby, nbx = (rows + 127) // 128, (cols + 127) // 128
    q = torch.empty(*lead, rows, cols, dtype=torch.float8_e4m3fn, device=x.device)
    si = torch.empty(*lead, nby, nbx, dtype=torch.float32, device=x.device)
    qt = sit = None
    if transpose:
        qt = torch.empty(*lead, cols, rows, dtype=torch.float8_e4m3fn, device=x.device)
        sit = torch.empty(*lead, nbx, nby, dtype=torch.float32, device=x.device)
    _check(lib.fluxmi_quant_e4m3_square(_ptr(x), batch, rows, cols, float(eps), _ptr(q), _ptr(si), _ptr(qt), _ptr(sit),
                                        _stream()), "fluxmi_quant_e4m3_square")
    return q, si, qt, sit


def quant_e4m3_block128(x, eps=0.0, transpose=False):
    """x [rows, cols] bf16 -> (q, scale_inv [rows/128, cols/128, 128], q_t [cols, rows], scale_inv_t
    [cols/128, rows/128, 128]); the last two are None without `transpose`.  One scale per (row, 128 columns);
    the transposed output has one per (column, 128 rows)."""
    lib = load()
    _dev_tensor(x, torch.bfloat16, "x")
    rows, cols = x.shape
    nby, nbx = (rows + 127) // 128, (cols + 127) // 128
    q = torch.empty(rows, cols, dtype=torch.float8_e4m3fn, device=x.device)
    alloc = lambda n, *shape: (torch.zeros if n % 128 else torch.empty)(*shape, dtype=torch.float32, device=x.device)
    si = alloc(rows, nby, nbx, 128)  # entries past the last row of the last block are not written
    qt = sit = None
    if transpose:
        qt = torch.empty(cols, rows, dtype=torch.float8_e4m3fn, device=x.device)
        sit = alloc(cols, nbx, nby, 128)
    _check(lib.fluxmi_quant_e4m3_block128(_ptr(x), rows, cols, float(eps), _ptr(q), _ptr(si), _ptr(qt), _ptr(sit),
                                          _stream()), "fluxmi_quant_e4m3_block128")
    return q, si, qt, sit


def calib_stream(src, dst, nbytes, copy=False):
    """fluxmi_calib_stream: a plain read stream of src[:nbytes] (copy=False; dst is a small sink of at least
    calib_stream_sink_bytes()) or a copy of it into dst."""
    lib = load()
    need = nbytes if copy else lib.fluxmi_calib_stream_sink_bytes()
    if src.numel() * src.element_size() < nbytes or dst.numel() * dst.element_size() < need:
        raise ValueError("calib_stream: buffers smaller than the stream")
    _check(lib.fluxmi_calib_stream(_ptr(src), _ptr(dst), nbytes, int(copy), _stream()), "fluxmi_calib_stream")
