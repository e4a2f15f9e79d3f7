"""Pins oracle.quant: three independent statements (numpy, C, torch's float8_e4m3fn cast) must agree
exhaustively, plus the ComputeScale special cases of src/quantization/quantization.cu:306-367."""
import numpy as np
import pytest
import torch

from oracle import quant


def test_decode_matches_torch_and_roundtrips():
    codes = np.arange(256, dtype=np.uint8)
    v = quant.e4m3_decode(codes)
    t = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(v), np.isnan(t))
    assert np.array_equal(v[~np.isnan(v)], t[~np.isnan(t)])
    assert np.nanmax(v) == 448.0 and np.nanmin(np.abs(v[v != 0])) == 2.0 ** -9
    enc = quant.e4m3_encode(v)
    keep = ~np.isnan(v)
    assert np.array_equal(enc[keep], codes[keep])
    lib = quant.clib()
    for c in codes[keep]:
        assert lib.fluxref_f32_to_e4m3(float(lib.fluxref_e4m3_to_f32(int(c)))) == c


@pytest.mark.parametrize("scale", [1.0, 0.37, 3.3, 448.0 / 7.3, 2.0 ** -20, 1e4])
def test_all_bf16_patterns_three_ways(scale):
    bits = np.arange(65536, dtype=np.uint16)
    with np.errstate(over="ignore", invalid="ignore"):
        y = (quant.bf16_bits_to_f32(bits) * np.float32(scale)).astype(np.float32)
    e_np = quant.e4m3_encode(y)
    lib = quant.clib()
    e_c = np.fromiter((lib.fluxref_f32_to_e4m3(float(a)) for a in y), dtype=np.uint8, count=y.size)
    assert np.array_equal(e_np, e_c)
    # torch's cast is round-to-nearest-even but does not saturate; it agrees wherever |y| <= 448
    inside = np.isfinite(y) & (np.abs(y) <= 448.0)
    e_t = torch.from_numpy(y).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(e_np[inside], e_t[inside])
    # saturation and NaN rules
    big = np.isfinite(y) & (np.abs(y) > 448.0)
    assert np.all((e_np[big] & 0x7F) == 0x7E)
    assert np.all((e_np[np.isnan(y)] & 0x7F) == 0x7F)
    assert np.all((e_np[np.isinf(y)] & 0x7F) == 0x7E)


def test_round_to_nearest_even_ties():
    # 17 -> 16, 19 -> 20, 18 exactly representable; 2^-10 (half the smallest subnormal) -> 0; 3*2^-10 -> 2^-8
    x = np.array([17.0, 19.0, 18.0, 2.0 ** -10, 3 * 2.0 ** -10, 464.0, 465.0, -17.0], dtype=np.float32)
    got = quant.e4m3_decode(quant.e4m3_encode(x))
    assert got.tolist() == [16.0, 20.0, 18.0, 0.0, 2.0 ** -8, 448.0, 448.0, -16.0]


def test_compute_scale_special_cases():
    lib = quant.clib()
    f = np.float32
    assert quant.compute_scale(f(0.0)) == 1.0 and lib.fluxref_compute_scale(0.0, 0.0) == 1.0
    assert quant.compute_scale(f(448.0)) == 1.0
    assert quant.compute_scale(f(1.0)) == 448.0
    assert quant.compute_scale(f(0.0), 0.5) == 896.0 and lib.fluxref_compute_scale(0.0, 0.5) == 896.0
    tiny = f(1e-38)  # 448 / tiny overflows -> bf16 max
    assert quant.compute_scale(tiny) == f(float.fromhex("0x1.FEp127"))
    assert lib.fluxref_compute_scale(float(tiny), 0.0) == float(f(float.fromhex("0x1.FEp127")))
    assert quant.compute_scale(f(np.inf)) == 0.0 and lib.fluxref_compute_scale(float("inf"), 0.0) == 0.0
    # fp32 division, not double: compare against the correctly rounded quotient
    for a in [3.0, 7.3, 0.001, 123.456]:
        assert quant.compute_scale(f(a)) == f(448.0) / f(a)
        assert lib.fluxref_compute_scale(float(f(a)), 0.0) == float(f(448.0) / f(a))


@pytest.mark.parametrize("rows,cols,block,permute", [(16, 256, 0, False), (16, 256, 128, False),
                                                      (130, 384, 128, True), (5, 200, 128, False),
                                                      (3, 8, 0, False), (129, 136, 128, True)])
def test_quant_rows_numpy_vs_c(rows, cols, block, permute):
    rng = np.random.default_rng(rows * 1000 + cols)
    x = (rng.standard_normal((rows, cols)) * rng.uniform(0.01, 30, size=(rows, 1))).astype(np.float32)
    x[0, :] = 0  # an all-zero row: scale 1, all-zero codes
    bits = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    q1, s1 = quant.quant_rows(bits, block, 0.0, permute)
    q2, s2 = quant.quant_rows_c(bits, block, 0.0, permute)
    assert np.array_equal(q1, q2)
    assert np.array_equal(s1, s2)
    assert np.all(q1[0] == 0)
    # the largest element of every block maps to +-448, dequantisation error is within half a grid step
    if block == 0:
        xb = quant.bf16_bits_to_f32(bits)
        deq = quant.e4m3_decode(q1) * s1[:, None]
        amax = np.abs(xb).max(1)
        assert np.all(np.abs(quant.e4m3_decode(q1)).max(1)[amax > 0] == 448.0)
        assert np.all(np.abs(deq - xb) <= amax[:, None] / 448.0 * 16.0 + 1e-30)
        assert s1[0] == 1.0


def test_quant_golden_fixture():
    """Committed fixture (tests/golden/quant_16x256.npz, written by tests/golden/make_golden.py)."""
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "quant_16x256.npz")
    z = np.load(path)
    q, s = quant.quant_rows(z["x_bits"], 0, 0.0, False)
    assert np.array_equal(q, z["q_row"]) and np.array_equal(s, z["scale_inv_row"])
    q, s = quant.quant_rows_c(z["x_bits"], 128, 0.0, True)
    assert np.array_equal(q, z["q_blk"]) and np.array_equal(s, z["scale_inv_blk_perm"])


def _bits(x):
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("rows,cols", [(128, 128), (256, 384), (130, 200), (5, 3), (1, 129), (257, 127)])
def test_quant_square_numpy_vs_c_vs_loops(rows, cols):
    """128 x 128 blocks: the numpy and the C restatement agree, and both agree with a per-block loop built from
    the already pinned scalar pieces (compute_scale, e4m3_encode)."""
    rng = np.random.default_rng(rows * 977 + cols)
    x = (rng.standard_normal((rows, cols)) * rng.uniform(0.01, 30, size=(rows, 1))).astype(np.float32)
    bits = _bits(x)
    q1, s1 = quant.quant_square(bits)
    q2, s2 = quant.quant_square_c(bits)
    assert np.array_equal(q1, q2) and np.array_equal(s1, s2)
    xf = quant.bf16_bits_to_f32(bits)
    for by in range((rows + 127) // 128):
        for bx in range((cols + 127) // 128):
            blk = xf[by * 128:(by + 1) * 128, bx * 128:(bx + 1) * 128]
            scale = quant.compute_scale(np.float32(np.abs(blk).max()))
            assert s1[by, bx] == np.float32(1.0) / scale
            assert np.array_equal(q1[by * 128:(by + 1) * 128, bx * 128:(bx + 1) * 128],
                                  quant.e4m3_encode((blk * scale).astype(np.float32)))
            assert np.abs(quant.e4m3_decode(q1[by * 128:(by + 1) * 128, bx * 128:(bx + 1) * 128])).max() == 448.0


def test_quant_square_against_row_blocks_and_special_blocks():
    """A block's scale is the smallest of its rows' 1 x 128 scales (scale_inv: the largest); an all-zero block
    gets scale 1 and zero codes; NaN is skipped by the amax and encoded as NaN; eps floors the amax."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((256, 256)) * rng.uniform(0.01, 30, size=(256, 1))).astype(np.float32)
    x[128:, :128] = 0
    x[3, 200] = np.nan
    bits = _bits(x)
    q, s = quant.quant_square(bits)
    qc, sc = quant.quant_square_c(bits)
    assert np.array_equal(q, qc) and np.array_equal(s, sc)
    _, srow = quant.quant_rows(bits, 128, 0.0, False)           # [256, 2]
    assert np.array_equal(s, srow.reshape(2, 128, 2).max(axis=1))
    assert s[1, 0] == 1.0 and np.all(q[128:, :128] == 0)
    assert q[3, 200] & 0x7F == 0x7F and np.isfinite(s).all()
    q_eps, s_eps = quant.quant_square(bits, eps=1e4)
    assert np.all(s_eps == np.float32(1.0) / (np.float32(448.0) / np.float32(1e4)))
    assert np.array_equal(q_eps, quant.quant_square_c(bits, eps=1e4)[0])
