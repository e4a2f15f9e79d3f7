"""GPU parity, fp8-e4m3 quantisation: codes and scales bit-exact against the CPU oracle."""
import os

import numpy as np
import pytest
import torch

from oracle import quant

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def to_bits(t_bf16):
    return t_bf16.view(torch.int16).cpu().numpy().view(np.uint16)


def run(bits, block=0, eps=0.0, permute=False):
    from flux_amd import capi
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).cuda()
    q, s = capi.quant_e4m3(x, block, eps, permute)
    torch.cuda.synchronize()
    return q.view(torch.uint8).cpu().numpy(), s.cpu().numpy()


def test_all_bf16_bit_patterns_per_row_scale():
    """Each row holds 256 consecutive bf16 bit patterns, so all 65536 patterns (NaN and inf included) go through
    the cast under 256 different scales."""
    bits = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    q, s = run(bits)
    rq, rs = quant.quant_rows_c(bits)
    finite_rows = np.isfinite(quant.bf16_bits_to_f32(bits)).all(1)
    assert np.array_equal(q[finite_rows], rq[finite_rows])
    assert np.array_equal(s[finite_rows], rs[finite_rows])
    # rows holding inf / NaN: amax = inf -> scale 0 -> finite elements become 0, inf * 0 = NaN.
    # The sign bit of a NaN code is not specified by IEEE arithmetic: compare NaN codes without it.
    canon = lambda a: np.where((a & 0x7F) == 0x7F, np.uint8(0x7F), a)
    assert np.array_equal(canon(q), canon(rq)) and np.array_equal(s.view(np.uint32), rs.view(np.uint32))


@pytest.mark.parametrize("scale", [1.0, 0.37, 3.3, 2.0 ** -12, 100.0])
def test_all_finite_patterns_fixed_scale(scale):
    """All finite bf16 patterns in one matrix whose rows share a known amax, so the cast sees x * (448/amax)."""
    bits = np.arange(65536, dtype=np.uint16)
    f = quant.bf16_bits_to_f32(bits)
    keep = np.isfinite(f) & (np.abs(f) <= scale)
    vals = bits[keep]
    cols = 512
    pad = (-len(vals)) % (cols - 8)
    vals = np.concatenate([vals, np.zeros(pad, np.uint16)]).reshape(-1, cols - 8)
    amax_bits = torch.tensor([scale], dtype=torch.float32).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    mat = np.concatenate([vals, np.broadcast_to(amax_bits, (vals.shape[0], 8))], axis=1)
    mat = np.ascontiguousarray(mat)
    q, s = run(mat)
    rq, rs = quant.quant_rows(mat)
    assert np.array_equal(q, rq) and np.array_equal(s, rs)


@pytest.mark.parametrize("rows,cols,block,permute,eps", [
    (16, 256, 0, False, 0.0), (16, 256, 128, True, 0.0), (130, 384, 128, True, 0.0), (5, 200, 128, False, 0.0),
    (3, 8, 0, False, 0.0), (129, 136, 128, True, 0.0), (257, 7168, 0, False, 0.0), (64, 2048, 0, False, 1e-3),
    (33, 1000, 0, False, 0.0), (9, 4104, 0, False, 0.0), (4, 16384, 0, False, 0.0), (3, 20000, 0, False, 0.0),
    (70, 1536, 128, False, 0.5), (7, 4096, 0, False, 0.0), (6, 3000, 0, False, 0.0), (11, 1024, 128, False, 0.0),
    (6, 7168, 128, False, 0.0), (2, 640, 128, False, 0.0)])
def test_shapes_against_oracle(rows, cols, block, permute, eps):
    print(f"[case] quant rows={rows} cols={cols} block={block} permute={permute} eps={eps}", flush=True)
    rng = np.random.default_rng(rows * 131 + cols)
    x = (rng.standard_normal((rows, cols)) * rng.uniform(1e-3, 50, size=(rows, 1))).astype(np.float32)
    x[0] = 0
    bits = to_bits(torch.from_numpy(x).to(torch.bfloat16))
    q, s = run(bits, block, eps, permute)
    rq, rs = quant.quant_rows_c(bits, block, eps, permute)
    assert np.array_equal(q, rq)
    assert np.array_equal(s, rs)


def test_golden_fixture():
    z = np.load(os.path.join(ROOT, "tests", "golden", "quant_16x256.npz"))
    q, s = run(z["x_bits"])
    assert np.array_equal(q, z["q_row"]) and np.array_equal(s, z["scale_inv_row"])
    q, s = run(z["x_bits"], 128, 0.0, True)
    assert np.array_equal(q, z["q_blk"]) and np.array_equal(s, z["scale_inv_blk_perm"])


@pytest.mark.parametrize("rows,cols", [(4096, 7168), (32768, 2048)])
def test_benchmark_shapes(rows, cols):
    """C5's two shapes: a 64-row sample bit-exact against the oracle; on the whole matrix the dequantisation
    error bound and 'row maximum maps to +-448'."""
    from flux_amd import capi
    print(f"[case] quant benchmark {rows}x{cols}", flush=True)
    gen = torch.Generator(device="cuda").manual_seed(rows)
    x = torch.randn(rows, cols, generator=gen, device="cuda").to(torch.bfloat16)
    q, s = capi.quant_e4m3(x)
    sample = torch.randperm(rows)[:64].cuda()
    rq, rs = quant.quant_rows_c(to_bits(x[sample]))
    assert np.array_equal(q[sample].view(torch.uint8).cpu().numpy(), rq)
    assert np.array_equal(s[sample].cpu().numpy(), rs)
    deq = q.float() * s[:, None]
    amax = x.float().abs().amax(1)
    assert bool((q.float().abs().amax(1) == 448.0).all())
    # half of the widest e4m3 step (32, between 256 and 448), in input units; ties reach it exactly, hence the slack
    assert bool(((deq - x.float()).abs() <= amax[:, None] / 448.0 * 16.0 * 1.001).all())
    assert torch.allclose(s * (448.0 / amax), torch.ones_like(s), rtol=1e-6)


def run_square(bits, eps=0.0, transpose=False):
    from flux_amd import capi
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).cuda()
    q, s, qt, st = capi.quant_e4m3_square(x, eps, transpose)
    torch.cuda.synchronize()
    u8 = lambda t: None if t is None else t.view(torch.uint8).cpu().numpy()
    return u8(q), s.cpu().numpy(), u8(qt), None if st is None else st.cpu().numpy()


@pytest.mark.parametrize("rows,cols,eps", [
    (128, 128, 0.0), (256, 384, 0.0), (130, 200, 0.0), (5, 3, 0.0), (1, 129, 0.0), (257, 127, 0.0),
    (384, 1024, 0.0), (100, 1032, 0.0), (144, 72, 0.0), (512, 256, 5.0), (129, 7168, 0.0)])
def test_square_blocks_against_oracle(rows, cols, eps):
    """128 x 128 block scales: bytes, scales and both transposed outputs bit-exact, whole, ragged and unaligned."""
    print(f"[case] quant square rows={rows} cols={cols} eps={eps}", flush=True)
    rng = np.random.default_rng(rows * 31 + cols)
    x = (rng.standard_normal((rows, cols)) * rng.uniform(1e-3, 50, size=(rows, 1))).astype(np.float32)
    x[: min(rows, 128), : min(cols, 128)] = 0
    if rows > 2 and cols > 2:
        x[2, 1] = np.nan
    bits = to_bits(torch.from_numpy(x).to(torch.bfloat16))
    rq, rs = quant.quant_square_c(bits, eps)
    q, s, qt, st = run_square(bits, eps, True)
    assert np.array_equal(q, rq) and np.array_equal(s, rs)
    assert np.array_equal(qt, rq.T) and np.array_equal(st, rs.T)
    q2, s2, none_q, none_s = run_square(bits, eps, False)
    assert none_q is None and none_s is None and np.array_equal(q2, rq) and np.array_equal(s2, rs)


def test_square_blocks_all_bit_patterns_and_batch():
    """All 65536 bf16 patterns through the block form (a batch of 2 x [128, 256]: four blocks, each with its own
    amax; inf and NaN included), and a batch equals its matrices one by one."""
    from flux_amd import capi
    bits = np.arange(65536, dtype=np.uint16).reshape(2, 128, 256)
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).cuda()
    q, s, qt, st = capi.quant_e4m3_square(x, 0.0, True)
    assert tuple(q.shape) == (2, 128, 256) and tuple(s.shape) == (2, 1, 2)
    assert tuple(qt.shape) == (2, 256, 128) and tuple(st.shape) == (2, 2, 1)
    # Blocks holding inf: amax = inf -> scale 0 -> inf * 0 = NaN, whose sign IEEE arithmetic leaves open:
    # NaN codes are compared without the sign bit.
    canon = lambda a: np.where((a & 0x7F) == 0x7F, np.uint8(0x7F), a)
    for b in range(2):
        rq, rs = quant.quant_square_c(bits[b])
        gq, gqt = q[b].view(torch.uint8).cpu().numpy(), qt[b].view(torch.uint8).cpu().numpy()
        assert np.array_equal(canon(gq), canon(rq))
        assert np.array_equal(gq[:, :128], rq[:, :128])  # the block without inf: exact, signs included
        assert np.array_equal(s[b].cpu().numpy(), rs)
        assert np.array_equal(gqt, gq.T)
        assert np.array_equal(st[b].cpu().numpy(), rs.T)


def test_square_blocks_weight_shapes():
    """C5's weights [32, 2048, 7168] as one batched call: a sample of blocks bit-exact against the oracle, on the
    whole tensor 'block maximum maps to +-448', the dequantisation bound and transposed = transpose."""
    from flux_amd import capi
    e, n, k = 32, 2048, 7168
    print(f"[case] quant square weights {e}x{n}x{k}", flush=True)
    gen = torch.Generator(device="cuda").manual_seed(77)
    w = (torch.randn(e, n, k, generator=gen, device="cuda") * 0.02).to(torch.bfloat16)
    q, s, qt, st = capi.quant_e4m3_square(w, 0.0, True)
    assert torch.equal(qt.view(torch.uint8), q.view(torch.uint8).transpose(1, 2))
    assert torch.equal(st, s.transpose(1, 2))
    rng = np.random.default_rng(3)
    for _ in range(6):
        b, by, bx = int(rng.integers(e)), int(rng.integers(n // 128)), int(rng.integers(k // 128))
        blk = w[b, by * 128:(by + 1) * 128, bx * 128:(bx + 1) * 128].contiguous()
        rq, rs = quant.quant_square_c(to_bits(blk))
        assert np.array_equal(q[b, by * 128:(by + 1) * 128, bx * 128:(bx + 1) * 128].view(torch.uint8).cpu().numpy(), rq)
        assert float(s[b, by, bx]) == float(rs[0, 0])
    amax = w.float().abs().view(e, n // 128, 128, k // 128, 128).amax(dim=(2, 4))
    qmax = q.float().abs().view(e, n // 128, 128, k // 128, 128).amax(dim=(2, 4))
    assert bool((qmax == 448.0).all())
    assert torch.allclose(s * (448.0 / amax), torch.ones_like(s), rtol=1e-6)


@pytest.mark.parametrize("rows,cols,eps", [
    (128, 128, 0.0), (256, 384, 0.0), (130, 200, 0.0), (5, 3, 0.0), (1, 129, 0.0), (257, 127, 0.0),
    (384, 1024, 0.0), (100, 1032, 0.0), (144, 72, 0.0), (512, 256, 5.0), (129, 7168, 0.0)])
def test_block128_with_transposed_output(rows, cols, eps):
    """1 x 128 scales plus the transposed matrix with 128 x 1 scales from one pass: both bit-exact against the
    oracle's row form applied to x and to x.T (permuted scale layouts), whole, ragged and unaligned shapes."""
    from flux_amd import capi
    print(f"[case] quant block128+transpose rows={rows} cols={cols} eps={eps}", flush=True)
    rng = np.random.default_rng(rows * 37 + cols)
    x = (rng.standard_normal((rows, cols)) * rng.uniform(1e-3, 50, size=(rows, 1))).astype(np.float32)
    x[0] = 0
    x[:, cols // 2] = 0
    if rows > 2 and cols > 2:
        x[2, 1] = np.nan
    bits = to_bits(torch.from_numpy(x).to(torch.bfloat16))
    xd = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).cuda()
    q, s, qt, st = capi.quant_e4m3_block128(xd, eps, True)
    rq, rs = quant.quant_rows_c(bits, 128, eps, True)
    rqt, rst = quant.quant_rows_c(np.ascontiguousarray(bits.T), 128, eps, True)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), rq) and np.array_equal(s.cpu().numpy(), rs)
    assert np.array_equal(qt.view(torch.uint8).cpu().numpy(), rqt) and np.array_equal(st.cpu().numpy(), rst)
    q2, s2, none_q, none_s = capi.quant_e4m3_block128(xd, eps, False)
    assert none_q is None and none_s is None
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2, s)
    # the older row-walking kernel behind fluxmi_quant_e4m3_rowwise gives the same bytes and scales
    if cols % 8 == 0:
        q3, s3 = capi.quant_e4m3(xd, 128, eps, True)
        assert torch.equal(q3.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s3, s)


def test_block128_all_bit_patterns_both_directions():
    """All 65536 bf16 patterns as a 256 x 256 matrix through the fused kernel: tiny amax (scale saturates at the
    bf16 maximum, scale_inv denormal), inf (scale 0) and NaN, along rows and along columns."""
    from flux_amd import capi
    bits = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    xd = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).cuda()
    q, s, qt, st = capi.quant_e4m3_block128(xd, 0.0, True)
    canon = lambda a: np.where((a & 0x7F) == 0x7F, np.uint8(0x7F), a)  # the sign of inf * 0 = NaN is open
    for got_q, got_s, src in ((q, s, bits), (qt, st, np.ascontiguousarray(bits.T))):
        rq, rs = quant.quant_rows_c(src, 128, 0.0, True)
        gq = got_q.view(torch.uint8).cpu().numpy()
        assert np.array_equal(canon(gq), canon(rq))
        f = quant.bf16_bits_to_f32(src).reshape(256, 2, 128)
        finite = np.repeat(np.isfinite(f).all(axis=2), 128, axis=1)  # per (row, block), spread over its columns
        assert np.array_equal(gq[finite], rq[finite])
        assert np.array_equal(got_s.cpu().numpy().view(np.uint32), rs.view(np.uint32))
