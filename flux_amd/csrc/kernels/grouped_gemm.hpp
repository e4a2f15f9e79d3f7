// Grouped GEMM over ragged per-expert row counts: D[r,:] = scale(r,:) * A[gather(r),:] @ B[e(r)]^T.
//
// Persistent kernel, one 256-thread workgroup (4 waves, one per SIMD) per CU, macro tile 256 rows x 256
// columns, k-step of 64 bytes per row (32 bf16 or 64 fp8).  Both operand tiles are staged in LDS by
// direct-to-LDS global loads (no register staging) in a ring of five 32 KiB stages; the row gather of A
// is folded into the per-lane global address of those loads.  Each wave owns a 128 x 128 quarter of the
// macro tile (bf16: 8x8 MFMA blocks of 16x16, fp8: 4x4 blocks of 32x32; 256 fp32 accumulator registers
// either way) and runs a software pipeline of its own: while the MFMAs of k-step s run on one set of
// fragment registers, the fragments of step s+1 are read from LDS into a second set and the ring fills of
// steps s+4 / s+5 are issued, all in a fixed interleaving (the 16 fragment reads spread evenly over the
// first half of the step's MFMAs, the 8 fills evenly over the whole step).  One workgroup barrier per
// k-step publishes the landed stage.
//
// A launch may carry up to four weight tensors ("groups") that multiply the same rows, each with its own
// output: their column tiles are numbered through one schedule (GemmParams::ngroups).
//
// Ring fills are issued in pairs of k-steps: the two 64-byte halves of a 128-byte line are requested
// back to back (they go to different stages), so the second request hits the line the first one
// brought into the vector L1 and L2 sees one request per line instead of two.
//
// The MFMA "A" operand is the weight fragment and the "B" operand the activation fragment, i.e. the
// hardware computes D^T blocks: a lane then holds, for one output row, four consecutive output columns
// per accumulator quad.  The epilogue passes each 64-row x 32-column block through a wave-private LDS
// window in fp32 and reads it back with eight lanes per row, so that one store instruction writes 64
// (bf16) or 128 (fp32) contiguous bytes of each row.
//
// Tile schedule: every wave walks the device-resident `splits` with scalar loads, in step with the
// increasing logical tile ids of its workgroup; ids are assigned so that the workgroups of one XCD
// (those with equal blockIdx % 8) take a run of consecutive tiles; tiles of an expert are ordered in
// groups of at most 8 row tiles, each group walked column-major over the weight panels, so an XCD's L2
// sees a few weight panels shared by the row tiles of a group.
#pragma once

#include <cstdlib>
#include <type_traits>

#include "common.hpp"

namespace fluxmi {


constexpr int BM = 256;                    // rows of a macro tile
constexpr int BN = 256;                    // columns of a macro tile
constexpr int KBYTES = 64;                 // bytes of K per row per k-step
constexpr int X_TILE_BYTES = BM * KBYTES;  // activation tile of one stage: 16 KiB
constexpr int W_TILE_BYTES = BN * KBYTES;
constexpr int STAGE_BYTES = X_TILE_BYTES + W_TILE_BYTES;
constexpr int STAGES = 5;                  // 160 KiB: the whole LDS of a CU
constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
constexpr int NTHREADS = 256;
constexpr int kMaxExperts = 1024;

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kMaxWeightGroups = 4;

// b / d / alpha: one entry per weight group of the launch (the same rows times several weight tensors).
struct GemmParams {
  const uint8_t *a;
  const uint8_t *b[kMaxWeightGroups];
  void *d[kMaxWeightGroups];
  const int32_t *splits;
  const int32_t *gather_a;
  const int32_t *scatter_d;
  const float *alpha[kMaxWeightGroups];
  const float *row_scale;
  const float *col_scale;
  const float *scalar_dev;
  float scalar;
  int32_t nexperts;
  int32_t max_rows;
  int32_t a_rows;
  int32_t n;
  int32_t k;
  int32_t d_fp32;
  int32_t ngroups;
  int32_t raster_rows;  // row tiles per raster group, >= 1
  int32_t sched_flags;  // FLUXMI_SCHED_*
  int32_t nt_stores;    // fp32 outputs are stored non-temporally
  int32_t accumulate;   // D is fp32 and every result is added to it atomically (rows meeting in one D row sum up)
  int32_t d_rows;       // rows of D: bound for scatter_d entries
  // Block-scaled fp8 (one scale per row of A and 128 of K, one per 128 x 128 block of B); null otherwise.
  const float *a_scale;
  const float *b_scale;
  int32_t a_scale_layout;  // FLUXMI_ASCALE_*
  int32_t b_scale_layout;  // FLUXMI_BSCALE_*
  int32_t half_is_f16;     // 2-byte operands and outputs are fp16, not bf16 (read by the generic kernel; the MFMA
                           // kernel is built once per 16-bit type)
};


// One launcher per element type, each in a translation unit of its own (the kernel is a long compile).
int launch_grouped_gemm_bf16(const GemmParams &p, int grid, hipStream_t s);
int launch_grouped_gemm_f16(const GemmParams &p, int grid, hipStream_t s);
int launch_grouped_gemm_fp8(const GemmParams &p, int grid, hipStream_t s);
int launch_grouped_gemm_fp8_blockscale(const GemmParams &p, int grid, hipStream_t s);
// The bf16 and fp8 kernels with whole-line ring fills (FLUXMI_SCHED_WHOLE_LINE_FILLS and the default rule in
// grouped_gemm.hip); fp16 has the half-line form only.
int launch_grouped_gemm_bf16_lines(const GemmParams &p, int grid, hipStream_t s);
int launch_grouped_gemm_fp8_lines(const GemmParams &p, int grid, hipStream_t s);

}  // namespace fluxmi
