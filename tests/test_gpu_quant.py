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
    (70, 1536, 128, False, 0.5)])
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
