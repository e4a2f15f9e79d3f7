"""CPU oracle for the MoE hot path — TEST INFRASTRUCTURE ONLY.

A restatement, in plain numpy / PyTorch-CPU / C, of what bytedance/flux computes on the single-GPU MoE
path (routing sort, gathered grouped GEMM, top-k weighted gather-reduce, fp8 row quantisation).  Every
function cites the reference file:line it follows.  Only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this package, and only as the checker or the timed baseline; nothing under
flux_amd/ imports it and the product never falls back to it.

What pins each function (see tests/test_oracle_*.py):
  routing.*            closed forms + brute-force loops on small inputs + permutation invariants +
                       numpy's stable argsort (library routine) + the reference's own monotonicity check
  layers.grouped_gemm  per-expert float64 matmul on small inputs; E=1 reduces to one dense matmul
  layers.layer0/1      brute-force python loops on tiny inputs; weights==1 reduces to the loop form of
                       test/python/util/test_scatter_only.py:79-96; the closed-form `--debug` data of
                       test/python/moe_gather_rs/test_moe_gather_rs.py:502-518
  quant.*              exhaustive: all 256 e4m3 codes decode->encode; all 65536 bf16 bit patterns x several
                       scales against torch.float8_e4m3fn (library routine) and against the C restatement
                       (quant_ref.c); ComputeScale special cases (0, inf, overflow).  The reference holds no
                       golden vector for quantisation (test/python/quantization/test_quantization.py:61-63
                       compares the output with itself), so beyond these checks its parity is pinned by
                       the arithmetic definition only.
"""
