"""Quantisation oracle: numpy restatement + loader of the C restatement (quant_ref.c)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libquant_ref.so")
_lib = None

E4M3_MAX = np.float32(448.0)
BF16_MAX = np.float32(float.fromhex("0x1.FEp127"))


def build():
    subprocess.run(["make", "-C", _HERE, "-B", "_build/libquant_ref.so"], check=True, stdout=subprocess.DEVNULL)
    return _SO


def clib():
    global _lib
    if _lib is None:
        src = os.path.join(_HERE, "quant_ref.c")
        if not os.path.exists(_SO) or (os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(_SO)):
            build()
        lib = ctypes.CDLL(_SO)
        lib.fluxref_compute_scale.restype = ctypes.c_float
        lib.fluxref_compute_scale.argtypes = [ctypes.c_float, ctypes.c_float]
        lib.fluxref_f32_to_e4m3.restype = ctypes.c_uint8
        lib.fluxref_f32_to_e4m3.argtypes = [ctypes.c_float]
        lib.fluxref_e4m3_to_f32.restype = ctypes.c_float
        lib.fluxref_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        lib.fluxref_quant_rows.restype = None
        lib.fluxref_quant_rows.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32,
                                           ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32]
        lib.fluxref_quant_square.restype = None
        lib.fluxref_quant_square.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_float,
                                             ctypes.c_void_p, ctypes.c_void_p]
        _lib = lib
    return _lib


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def compute_scale(amax, eps=0.0):
    """ComputeScale (src/quantization/quantization.cu:306-367), bf16 input type, no power-of-two rounding."""
    amax = np.asarray(amax, dtype=np.float32)
    a = np.fmax(amax, np.float32(eps))
    with np.errstate(divide="ignore", over="ignore"):
        s = np.where(a == 0, np.float32(1.0), E4M3_MAX / np.where(a == 0, np.float32(1.0), a)).astype(np.float32)
    s = np.where(np.isinf(s), BF16_MAX, s).astype(np.float32)
    return s


def e4m3_decode(codes):
    """All 256 e4m3fn codes -> float32 (0x7f / 0xff are NaN; no infinities)."""
    b = np.asarray(codes, dtype=np.uint8).astype(np.int32)
    sign = np.where(b & 0x80, -1.0, 1.0).astype(np.float32)
    e = (b >> 3) & 0xF
    m = b & 7
    sub = np.ldexp(m.astype(np.float32), -9)
    nor = np.ldexp((8 + m).astype(np.float32), e - 10)
    v = np.where(e == 0, sub, nor).astype(np.float32)
    v = np.where((e == 0xF) & (m == 7), np.float32(np.nan), v)
    return (sign * v).astype(np.float32)


def e4m3_encode(x):
    """float32 -> e4m3fn code, round to nearest even, saturate to +-448 (CUDA __nv_fp8_e4m3 semantics,
    src/quantization/quantization.cu:674-676), NaN -> 0x7f | sign."""
    x = np.asarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    sign = ((u >> 24) & 0x80).astype(np.uint8)
    a = np.abs(x)
    out = np.zeros(x.shape, dtype=np.uint8)
    nan = np.isnan(x)
    sat = (~nan) & (a >= 448.0)
    sub = (~nan) & (a < 2.0 ** -6)
    nor = (~nan) & ~sat & ~sub
    with np.errstate(invalid="ignore"):
        qs = np.rint(np.where(sub, a, 0) * np.float32(512.0)).astype(np.uint8)
    m, ex = np.frexp(np.where(nor, a, np.float32(1.0)))
    q = np.rint(m.astype(np.float32) * np.float32(16.0))
    carry = q == 16
    q = np.where(carry, 8, q).astype(np.int32)
    ex = ex + carry
    e = (ex - 1 + 7).astype(np.int32)
    qn = ((e << 3) | (q & 7)).astype(np.uint8)
    out = np.where(sub, qs, out)
    out = np.where(nor, qn, out)
    out = np.where(sat, np.uint8(0x7E), out)
    out = np.where(nan, np.uint8(0x7F), out)
    return (out | sign).astype(np.uint8)


def quant_rows(x_bits, block_cols=0, eps=0.0, permute=False):
    """numpy form of the per-(row, block) quantisation.  x_bits: uint16 bf16 bit patterns [rows, cols].
    Returns (q uint8 [rows, cols], scale_inv float32)."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    rows, cols = x_bits.shape
    x = bf16_bits_to_f32(x_bits)
    bc = cols if block_cols == 0 else block_cols
    nb = (cols + bc - 1) // bc if bc else 0
    pad = nb * bc - cols
    ax = np.abs(x)
    ax = np.where(np.isnan(ax), np.float32(0), ax)  # fmaxf ignores NaN
    if pad:
        ax = np.pad(ax, ((0, 0), (0, pad)))
    amax = ax.reshape(rows, nb, bc).max(axis=2) if nb else np.zeros((rows, 0), np.float32)
    scale = compute_scale(amax, eps)  # [rows, nb]
    inv = (1.0 / scale.astype(np.float64)).astype(np.float32)
    full = np.repeat(scale, bc, axis=1)[:, :cols]
    with np.errstate(over="ignore", invalid="ignore"):
        q = e4m3_encode((x * full).astype(np.float32))
    if block_cols == 0:
        return q, inv.reshape(rows)
    if permute:
        out = np.zeros(((rows + 127) // 128, nb, 128), dtype=np.float32)
        r = np.arange(rows)
        out[r // 128, :, r % 128] = inv
        return q, out
    return q, inv


def quant_rows_c(x_bits, block_cols=0, eps=0.0, permute=False):
    """Same through the C restatement."""
    lib = clib()
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    rows, cols = x_bits.shape
    q = np.zeros((rows, cols), dtype=np.uint8)
    bc = cols if block_cols == 0 else block_cols
    nb = (cols + bc - 1) // bc if bc else 0
    if block_cols == 0:
        inv = np.zeros(rows, dtype=np.float32)
    elif permute:
        inv = np.zeros(((rows + 127) // 128, nb, 128), dtype=np.float32)
    else:
        inv = np.zeros((rows, nb), dtype=np.float32)
    lib.fluxref_quant_rows(x_bits.ctypes.data, rows, cols, block_cols, eps, q.ctypes.data, inv.ctypes.data,
                           int(permute))
    return q, inv


def quant_square(x_bits, eps=0.0):
    """numpy form of the 128 x 128 block quantisation (src/quantization/quantization.cu:971-1183 ragged blocks,
    :1185-1380 full blocks): amax over the part of a block inside the matrix, scale_inv = 1.0f / scale.
    x_bits: uint16 bf16 bit patterns [rows, cols].  Returns (q uint8 [rows, cols], scale_inv float32
    [ceil(rows/128), ceil(cols/128)]); the transposed outputs of the reference are q.T and scale_inv.T."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    rows, cols = x_bits.shape
    x = bf16_bits_to_f32(x_bits)
    nby, nbx = (rows + 127) // 128, (cols + 127) // 128
    ax = np.abs(x)
    ax = np.where(np.isnan(ax), np.float32(0), ax)  # fmaxf ignores NaN
    ax = np.pad(ax, ((0, nby * 128 - rows), (0, nbx * 128 - cols)))
    amax = ax.reshape(nby, 128, nbx, 128).max(axis=(1, 3))
    scale = compute_scale(amax, eps)
    with np.errstate(divide="ignore"):
        inv = (np.float32(1.0) / scale).astype(np.float32)
    full = np.repeat(np.repeat(scale, 128, axis=0), 128, axis=1)[:rows, :cols]
    with np.errstate(over="ignore", invalid="ignore"):
        q = e4m3_encode((x * full).astype(np.float32))
    return q, inv


def quant_square_c(x_bits, eps=0.0):
    """Same through the C restatement."""
    lib = clib()
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    rows, cols = x_bits.shape
    q = np.zeros((rows, cols), dtype=np.uint8)
    inv = np.zeros(((rows + 127) // 128, (cols + 127) // 128), dtype=np.float32)
    lib.fluxref_quant_square(x_bits.ctypes.data, rows, cols, eps, q.ctypes.data, inv.ctypes.data)
    return q, inv
