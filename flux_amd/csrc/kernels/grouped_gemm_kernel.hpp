// Device code of the grouped GEMM MFMA kernel; included by one translation unit per element type.
#pragma once

#include "grouped_gemm.hpp"

namespace fluxmi {
namespace {

// Which form of ring fills whole, half-height, half-width and 64-row tiles use: 64-byte half lines, one k-step per ring
// stage (gemm_tile), or, if the including translation unit defines FLUXMI_LINE_FILLS, whole 128-byte lines, a pair of
// k-steps per ring unit (gemm_tile_lines).
#ifdef FLUXMI_LINE_FILLS
constexpr bool kLineFills = true;
#else
constexpr bool kLineFills = false;
#endif

// The device code below is compiled in the device pass only; the host pass sees the kernel's declaration with an empty
// body (all it needs for the launch stub).
#if defined(__HIP_DEVICE_COMPILE__)

#define FLUXMI_WAITCNT(vm, lgkm) \
  __builtin_amdgcn_s_waitcnt(((vm)&15) | (((vm) >> 4) << 14) | (7 << 4) | ((lgkm) << 8))

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *gbl_ptr_t;

// One wave-wide direct-to-LDS load: lane l fetches 16 bytes from `src` (per lane) and the hardware
// stores them at lds_base + 16*l (lds_base is wave-uniform).
__device__ __forceinline__ void load_to_lds16(const uint8_t *src, uint8_t *lds_base) {
  __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)lds_base, 16, 0, 0);
}

// Which 16-bit float the 2-byte instantiation computes in: bf16 unless the including translation unit defines
// FLUXMI_HALF_IS_F16 (the fp16 build of the same kernel: another MFMA opcode and another output cast, nothing else).
#ifdef FLUXMI_HALF_IS_F16
constexpr bool kHalfIsF16 = true;
#else
constexpr bool kHalfIsF16 = false;
#endif

// Two floats to the packed 16-bit output type (bf16: one v_cvt_pk_bf16_f32; fp16: two v_cvt_f16_f32 and a pack),
// round to nearest even.  fp8 inputs always produce bf16.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  if constexpr (kHalfIsF16) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f16x2 h = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    return __builtin_bit_cast(uint32_t, h);
  } else {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
}

// Source of the ring fills of a k-step past the end of K: every lane reads 16 zero bytes.
__device__ __attribute__((aligned(1024))) const uint8_t g_zero_page[1024] = {};

// MFMA geometry per element type.  bf16 uses v_mfma_f32_16x16x32_bf16: one instruction consumes a whole
// k-step (32 elements) of a 16-row block of each operand, i.e. one 16-byte fragment register set per
// block, and accumulates a 16x16 block in 4 registers.  At the same FLOP rate as the 32x32x16 form it
// moves half the accumulator bytes per FLOP through the register file, and measured under the board's
// power limit that is worth 18 % of sustained MFMA throughput.  fp8 uses the 32x32x64 f8f6f4 form: two
// 16-byte fragment chunks per 32-row block and k-step, 16 accumulator registers per block.
template <int ELT>
struct Geom {
  static constexpr int BLK = ELT == 2 ? 16 : 32;  // rows (columns) of an operand block
  static constexpr int NCH = ELT == 2 ? 1 : 2;    // 16-byte fragment chunks per block and k-step
  static constexpr int NACC = BLK * BLK / 64;     // accumulator registers per block
  typedef float Acc __attribute__((ext_vector_type(NACC)));
};

// MFMA number t of a k-step over MBK x NBK blocks: block row i = t / NBK, block column j = t % NBK.
template <int ELT, int MBK, int NBK>
__device__ __forceinline__ void mfma_slot(int t, const i32x4 (&xf)[MBK][Geom<ELT>::NCH], const i32x4 (&wf)[NBK][Geom<ELT>::NCH],
                                          typename Geom<ELT>::Acc (&acc)[MBK][NBK]) {
  const int i = t / NBK, j = t % NBK;
  if constexpr (ELT == 2) {
    // Written as asm to pin the accumulators to the accumulation registers: given the builtin, the
    // register allocator spreads the 64 four-register accumulators over both register files and shuffles
    // them at the loop's back edge.  Every accumulator is touched once per k-step, 63 MFMAs apart, and
    // the fragment operands come from LDS reads the compiler still tracks, so no hazard needs software
    // wait states here.
    if constexpr (kHalfIsF16)
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(wf[j][0]), "v"(xf[i][0]));
    else
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(wf[j][0]), "v"(xf[i][0]));
  } else {
    i32x8 wa, xa;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      wa[v] = wf[j][0][v];
      wa[4 + v] = wf[j][1][v];
      xa[v] = xf[i][0][v];
      xa[4 + v] = xf[i][1][v];
    }
    // cbsz = blgp = 0: both operands e4m3; zero scale operands select the unscaled form (scale 1).
    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wa, xa, acc[i][j], 0, 0, 0, 0, 0, 0);
  }
}

// Clamped row count of expert e: negative entries count as 0 and rows past max_rows do not exist.
__device__ __forceinline__ int expert_rows(const GemmParams &p, int e, int row_base) {
  int rows = p.splits[e];
  if (rows < 0) rows = 0;
  if (rows > p.max_rows - row_base) rows = p.max_rows - row_base;
  return rows;
}

// Per-lane constants shared by all tile shapes.
struct TileCtx {
  int wave, lane, wn, wm;
  int fill_row, fill_chunk;
  int frag_off[2];
  // The same for whole-line fills (one instruction covers 8 rows x 128 bytes, i.e. a pair of k-steps): the row of
  // the 8 this lane fetches, its byte offset inside the row's 128 bytes for fill instructions over even / odd
  // 8-row blocks, and its fragment offsets inside a 32 KiB operand unit.
  int lfill_row;
  int lfill_byte[2];
  int lfrag_off[2];
  int nk;           // k-steps of 64 bytes per row, a partial last one included
  int nkf;          // whole k-steps
  int tail_chunks;  // 16-byte chunks of the partial last k-step (0: K is a whole number of k-steps)
  int64_t kbytes;
  float scalar;
};

// The kernel's only argument, read again from the kernel argument segment where it is used.  A copy of
// all of it kept live in scalar registers through the main loop does not fit the register file; the
// empty asm keeps the compiler from hoisting these loads back to the top of the kernel.
typedef const __attribute__((address_space(4))) GemmParams *KernArgs;
__device__ __forceinline__ KernArgs kernel_args() {
  KernArgs k = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(k));
  return k;
}

// One accumulator element, moved out of its accumulation register at the point of use.  Left to itself
// the compiler copies all 256 of them into vector registers ahead of the epilogue's branches, which
// does not fit.
__device__ __forceinline__ float acc_read(float a) {
  float v;
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
  return v;
}

template <bool IN_VGPR>
__device__ __forceinline__ float sum_read(float a) {
  if constexpr (IN_VGPR) return a;
  else return acc_read(a);
}

// Compile-time loop: f(integral_constant<int, I>) for I in [0, N).
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// Epilogue of one wave: acc (32*MB rows x 32*NB columns, MFMA layout) -> scaled, cast, stored.
// Blocks of 32 rows x 32 columns go through the two 4 KiB halves of the wave's LDS window in fp32 (alternating, so
// the writes of a block do not wait for the reads of the one before) and come back with eight lanes per
// row (j below counts 32-column groups, ip 64-row groups).  FULL: every row and column of the wave's quarter exists and rows are stored where they are (no
// scatter), so no store is predicated.  OUT_F32 selects the output element type.  !SCALED: every scale
// factor is 1 and the multiplications are left out.
// SUMS_IN_VGPRS: the sums are ordinary vector-register values (the block-scaled kernel's promoted sums) and are
// read as they are.
template <int ELT, int MB, int NB, bool FULL, bool OUT_F32, bool SCALED, bool SUMS_IN_VGPRS = false>
__device__ __forceinline__ void store_tile(uint8_t *windows, const TileCtx &c, int g, int e, int row_base, int rows_e,
                                           int wrow0, int wcol0,
                                           const typename Geom<ELT>::Acc (&acc)[32 * MB / Geom<ELT>::BLK][32 * NB / Geom<ELT>::BLK]) {
  constexpr int BLK = Geom<ELT>::BLK;
  constexpr int MBK = 32 * MB / BLK;
  constexpr int ELT_OUT = OUT_F32 ? 4 : 2;
  const KernArgs p = kernel_args();
  const int lane = c.lane;
  const int h = lane >> 5;
  const int n = p->n;
  const float *alpha = p->alpha[g], *row_scale = p->row_scale, *col_scale = p->col_scale;
  const float tile_scale = c.scalar * (alpha ? alpha[e] : 1.f);
  float rs[MBK];  // scale of this lane's row in each block row
#pragma unroll
  for (int i = 0; i < MBK; ++i) {
    const int m = wrow0 + i * BLK + (lane & (BLK - 1));
    rs[i] = tile_scale * ((row_scale && (FULL || m < rows_e)) ? row_scale[row_base + m] : 1.f);
  }
  const int rr0 = lane >> 3;  // row of this lane within a group of 8 rows (store phase)
  const int cc = lane & 7;    // its 4-column chunk
  // Output address of (first row of the wave + rr0, first column of the wave + 4 * cc); blocks and row
  // groups add multiples of 32 columns and 8 rows.
  uint8_t *const d = static_cast<uint8_t *>(p->d[g]);
  uint8_t *dlane = d + (static_cast<int64_t>(row_base + wrow0 + rr0) * n + wcol0 + cc * 4) * ELT_OUT;
  const int64_t rowgroup_bytes = static_cast<int64_t>(8) * n * ELT_OUT;
  const int32_t *scatter = FULL ? nullptr : p->scatter_d;
  const int d_rows = p->d_rows;
  const bool nt_stores = p->nt_stores != 0;  // wave-uniform
  const bool accumulate = !FULL && p->accumulate != 0;
  if constexpr (ELT == 2 && !OUT_F32 && FULL && NB % 2 == 0 && MB % 2 == 0) {
    // bf16 rows of whole tiles leave as whole 128-byte lines: two 32-column blocks per pass, packed to bf16
    // before the pass, so that the window (64 rows x 128 bytes) comes back as eight lanes x 16 bytes per row.
    // In 64-byte pieces a line is written in two halves at different times and part of the lines reach HBM
    // twice.  Needs 16-byte aligned rows; other outputs take the 64-byte path below.  (The same form for the
    // 32 x 32 blocks of the fp8 kernel measured 3-5 % slower than the 64-byte path on the fp8 benchmark shapes.)
    if ((n & 7) == 0 && (reinterpret_cast<uintptr_t>(d) & 15u) == 0) {
      uint8_t *const wlane = d + (static_cast<int64_t>(row_base + wrow0 + rr0) * n + wcol0 + cc * 8) * 2;
#pragma unroll
      for (int j2 = 0; j2 < NB / 2; ++j2) {
#pragma unroll
        for (int ip = 0; ip < MB / 2; ++ip) {
          uint8_t *window = windows;
#pragma unroll
          for (int jq = 0; jq < 4; ++jq) {
            const int jb = j2 * 4 + jq;
            float4 cs = make_float4(1.f, 1.f, 1.f, 1.f);
            if constexpr (SCALED) {
              if (col_scale)
                cs = *reinterpret_cast<const float4 *>(col_scale + static_cast<int64_t>(e) * n + wcol0 + jb * 16 + 4 * (lane >> 4));
            }
#pragma unroll
            for (int ii = 0; ii < 4; ++ii) {
              const int i = ip * 4 + ii;
              const int r = ii * 16 + (lane & 15);
              float4 v = make_float4(sum_read<SUMS_IN_VGPRS>(acc[i][jb][0]), sum_read<SUMS_IN_VGPRS>(acc[i][jb][1]), sum_read<SUMS_IN_VGPRS>(acc[i][jb][2]),
                                     sum_read<SUMS_IN_VGPRS>(acc[i][jb][3]));
              if constexpr (SCALED) {
                v = make_float4(v.x * rs[i], v.y * rs[i], v.z * rs[i], v.w * rs[i]);
                v = make_float4(v.x * cs.x, v.y * cs.y, v.z * cs.z, v.w * cs.w);
              }
              u32x2 b;
              b[0] = pack_bf16x2(v.x, v.y);
              b[1] = pack_bf16x2(v.z, v.w);
              const int chunk = jq * 2 + (lane >> 5);  // 16-byte chunk of the 128-byte row; (lane >> 4) & 1: its half
              *reinterpret_cast<u32x2 *>(window + r * 128 + ((chunk ^ ((r >> 1) & 7)) << 4) + ((lane >> 4) & 1) * 8) = b;
            }
          }
          u32x4 v[8];
#pragma unroll
          for (int it = 0; it < 8; ++it) {
            const int rr = it * 8 + rr0;
            v[it] = *reinterpret_cast<const u32x4 *>(window + rr * 128 + ((cc ^ ((rr >> 1) & 7)) << 4));
          }
          uint8_t *dp = wlane + (static_cast<int64_t>(ip) * 8) * rowgroup_bytes + j2 * 128;
#pragma unroll
          for (int it = 0; it < 8; ++it, dp += rowgroup_bytes) *reinterpret_cast<u32x4 *>(dp) = v[it];
        }
      }
      return;
    }
  }
  // 64-byte (bf16) / 128-byte (fp32) pieces: passes of 32 rows x 32 columns through the two 4 KiB halves of the
  // window in fp32, software-pipelined: while the rows of pass p come back from LDS and are stored, the
  // accumulators of pass p + 1 are already being written to the other half, so that the LDS round trip of a pass
  // is not exposed.  Pass p = j * MB + g: column group j, 32-row group g of the wave's rows; passes alternate between
  // the two halves of the window.
  constexpr int NPASS = NB * MB;
  float4 csj[NB];  // column scales of this lane's 4-column chunk in every column group
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int col = wcol0 + j * 32 + cc * 4;
    csj[j] = make_float4(1.f, 1.f, 1.f, 1.f);
    if (col_scale && (FULL || col < n)) csj[j] = *reinterpret_cast<const float4 *>(col_scale + static_cast<int64_t>(e) * n + col);
  }
  // A lane holds one row of a block and groups of 4 consecutive columns of it: with 16x16 blocks one group,
  // columns 4 * (lane / 16); with 32x32 blocks four, columns 8q + 4 * (lane / 32).
  auto write_half = [&](auto PC) {
    constexpr int ps = decltype(PC)::value, hh = ps & 1, g32 = ps % MB, j = ps / MB;
    uint8_t *half = windows + hh * 4096;
#pragma unroll
    for (int i2 = 0; i2 < 32 / BLK; ++i2) {
      const int i = g32 * (32 / BLK) + i2;
      const int r = i2 * BLK + (lane & (BLK - 1));
#pragma unroll
      for (int jj = 0; jj < 32 / BLK; ++jj) {
        const int jb = j * (32 / BLK) + jj;
#pragma unroll
        for (int q = 0; q < Geom<ELT>::NACC / 4; ++q) {
          const int chunk = BLK == 32 ? 2 * q + h : jj * 4 + (lane >> 4);
          float4 v = make_float4(sum_read<SUMS_IN_VGPRS>(acc[i][jb][4 * q + 0]), sum_read<SUMS_IN_VGPRS>(acc[i][jb][4 * q + 1]),
                                 sum_read<SUMS_IN_VGPRS>(acc[i][jb][4 * q + 2]), sum_read<SUMS_IN_VGPRS>(acc[i][jb][4 * q + 3]));
          if constexpr (SCALED) v = make_float4(v.x * rs[i], v.y * rs[i], v.z * rs[i], v.w * rs[i]);
          *reinterpret_cast<float4 *>(half + r * 128 + ((chunk ^ ((r >> 1) & 7)) << 4)) = v;
        }
      }
    }
  };
  // 8 lanes per row, 8 rows per instruction
  auto read_half = [&](auto PC, float4 (&v)[4]) {
    constexpr int hh = decltype(PC)::value & 1;
    const uint8_t *half = windows + hh * 4096;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int rr = it * 8 + rr0;
      v[it] = *reinterpret_cast<const float4 *>(half + rr * 128 + ((cc ^ ((rr >> 1) & 7)) << 4));
    }
  };
  auto store_half = [&](auto PC, const float4 (&v)[4]) {
    constexpr int ps = decltype(PC)::value, g32 = ps % MB, j = ps / MB;
    const int col = wcol0 + j * 32 + cc * 4;
    const float4 cs = csj[j];
    uint8_t *dp = dlane + (static_cast<int64_t>(g32) * 4) * rowgroup_bytes + j * 32 * ELT_OUT;
#pragma unroll
    for (int it = 0; it < 4; ++it, dp += rowgroup_bytes) {
      uint8_t *dst = dp;
      if constexpr (!FULL) {
        const int m = wrow0 + g32 * 32 + it * 8 + rr0;
        if (m >= rows_e || col >= n) continue;  // n % 4 == 0: a chunk is all in or all out
        if (scatter) {
          const int64_t drow = scatter[row_base + m];
          if (drow < 0 || drow >= d_rows) continue;
          dst = d + (drow * n + col) * ELT_OUT;
        }
      }
      float4 o = v[it];
      if constexpr (SCALED) o = make_float4(o.x * cs.x, o.y * cs.y, o.z * cs.z, o.w * cs.w);
      if constexpr (OUT_F32) {
        if (nt_stores) {
          typedef float f32x4_t __attribute__((ext_vector_type(4)));
          const f32x4_t ov = {o.x, o.y, o.z, o.w};
          __builtin_nontemporal_store(ov, reinterpret_cast<f32x4_t *>(dst));
        } else {
          *reinterpret_cast<float4 *>(dst) = o;
        }
      } else {
        u32x2 b;
        b[0] = pack_bf16x2(o.x, o.y);
        b[1] = pack_bf16x2(o.z, o.w);
        *reinterpret_cast<u32x2 *>(dst) = b;
      }
    }
  };
  if constexpr (!FULL && OUT_F32) {
    if (accumulate) {
      // Top-k reduction in the epilogue: every result is added to row scatter[row] of the fp32 output with a hardware
      // float atomic (no return value).  The block comes back from the window with 32 lanes per row, one float each,
      // so that an atomic instruction covers two whole 128-byte lines (with the 8-lanes-per-row layout of the stores
      // it would touch eight lines for 32 bytes each: four times the line operations at the L2 atomic units).
      const int half_lane = lane >> 5, col_lane = lane & 31;
      float csl[NB];
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int col = wcol0 + j * 32 + col_lane;
        csl[j] = (col_scale && col < n) ? col_scale[static_cast<int64_t>(e) * n + col] : 1.f;
      }
      float *const df = reinterpret_cast<float *>(d);
      auto read_rows = [&](auto PC, float (&f)[16]) {
        constexpr int hh = decltype(PC)::value & 1;
        const uint8_t *half = windows + hh * 4096;
#pragma unroll
        for (int it = 0; it < 16; ++it) {
          const int rr = it * 2 + half_lane;
          f[it] = *reinterpret_cast<const float *>(half + rr * 128 + (((col_lane >> 2) ^ ((rr >> 1) & 7)) << 4) + (col_lane & 3) * 4);
        }
      };
      auto add_rows = [&](auto PC, const float (&f)[16]) {
        constexpr int ps = decltype(PC)::value, g32 = ps % MB, j = ps / MB;
        const int col = wcol0 + j * 32 + col_lane;
#pragma unroll
        for (int it = 0; it < 16; ++it) {
          const int m = wrow0 + g32 * 32 + it * 2 + half_lane;
          if (m >= rows_e || col >= n) continue;
          const int64_t drow = scatter ? static_cast<int64_t>(scatter[row_base + m]) : static_cast<int64_t>(row_base + m);
          if (drow < 0 || drow >= d_rows) continue;
          unsafeAtomicAdd(df + drow * n + col, f[it] * csl[j]);
        }
      };
      float fa[16], fb[16];
      write_half(std::integral_constant<int, 0>{});
      static_for<0, NPASS>([&](auto PC) {
        constexpr int ps = decltype(PC)::value;
        if constexpr ((ps & 1) == 0) read_rows(PC, fa);
        else read_rows(PC, fb);
        if constexpr (ps + 1 < NPASS) write_half(std::integral_constant<int, (ps + 1 < NPASS ? ps + 1 : 0)>{});
        if constexpr ((ps & 1) == 0) add_rows(PC, fa);
        else add_rows(PC, fb);
      });
      return;
    }
  }
  float4 va[4], vb[4];
  write_half(std::integral_constant<int, 0>{});
  static_for<0, NPASS>([&](auto PC) {
    constexpr int ps = decltype(PC)::value;
    if constexpr ((ps & 1) == 0) read_half(PC, va);
    else read_half(PC, vb);
    if constexpr (ps + 1 < NPASS) write_half(std::integral_constant<int, (ps + 1 < NPASS ? ps + 1 : 0)>{});
    if constexpr ((ps & 1) == 0) store_half(PC, va);
    else store_half(PC, vb);
  });
}

// Buffer resource over [base, base + bytes): loads past the end return zero instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const uint8_t *base, int64_t bytes) {
  const uint32_t n = bytes > 0xffffffffll ? 0xffffffffu : static_cast<uint32_t>(bytes < 0 ? 0 : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, static_cast<int>(n), 0x00020000);
}
// Where a work item lies.  kind: 0 a whole macro tile (4, 4); 1 the 128-row tile ending an expert (2, 4);
// 2 a 256x128 piece (4, 2); 3 a 128x128 piece (2, 2); 4 a 64x64 piece of an expert's last rows (1, 1); 5 the 64-row
// tile ending an expert (1, 4); -1 an item without work; -2 past the last item.
// n0 is a column of the launch's virtual output: weight group g (a launch may multiply the same rows by up
// to four weight tensors, each with an output of its own) occupies columns [g * npad, g * npad + n), npad =
// n rounded up to whole macro tiles.
struct TileDesc {
  int kind, e, row_base, rows_e, m0, n0;
};

// Virtual column -> weight group (returned) and column inside it (n0).
__device__ __forceinline__ int split_group(int &n0, int n, int ngroups) {
  int g = 0;
  if (ngroups > 1) {
    const int npad = ((n + BN - 1) / BN) * BN;
    while (n0 >= npad) {
      n0 -= npad;
      ++g;
    }
  }
  return g;
}

// Ring geometry per tile shape.  Whole and half tiles: five stages of 32 KiB, fills four k-steps ahead.  The
// 128x128 pieces of a last round need 16 KiB per stage and have short k-steps (16 MFMAs per wave), so four
// steps of look-ahead do not cover the memory latency: they run ten stages of 16 KiB, eight steps ahead.
// Both stage counts divide ten, the number of k-steps over which the loop is unrolled.
// The 64x64 pieces that the few last rows of an expert are cut into (one MFMA block row per wave and k-step) take
// 8 KiB per stage: twenty stages, sixteen steps ahead, unrolled over twenty k-steps.
template <int MB, int NB>
struct Ring {
  static_assert(MB != 1 || NB == 1 || NB == 4, "64-row tiles exist as 64x64 pieces and as 64x256 tiles");
  static constexpr bool tiny = MB == 1 && NB == 1;
  static constexpr bool deep = MB == 2 && NB == 2;
  static constexpr int STG = tiny ? 4 * STAGES : (deep ? 2 * STAGES : STAGES);
  static constexpr int XB = tiny ? X_TILE_BYTES / 4 : (deep ? X_TILE_BYTES / 2 : X_TILE_BYTES);  // X part of a stage
  static constexpr int SB = tiny ? STAGE_BYTES / 4 : (deep ? STAGE_BYTES / 2 : STAGE_BYTES);     // a stage
  static constexpr int LA = tiny ? 16 : (deep ? 8 : 4);                                          // look-ahead in k-steps (even)
  static constexpr int TRIP = tiny ? 20 : 10;  // k-steps after which ring slot and fragment set repeat
};

// Operand addressing of a tile: buffer resources and this lane's byte offsets of its fill instructions.
template <int XL, int WL>
struct TileOperands {
  __amdgpu_buffer_rsrc_t xrsrc, wrsrc;
  uint32_t xoff[XL], woff[WL];
};


// What a tile leaves behind for the next one when that is a whole macro tile: its operand addressing,
// with k-steps 0..3 already requested into ring slots 0..3 ahead of the epilogue, so that their latency
// passes while the epilogue runs.
struct TilePrefetch {
  bool valid;
  TileOperands<4, 4> op;
};

// Ring fills address global memory through buffer resources: a scalar base per operand, a loop-invariant
// 32-bit byte offset per lane and fill instruction, and the k offset as scalar offset.  Fill
// instruction q of a tile covers rows [16q, 16q+16); tail rows re-read the last valid row.
// The rows of A this lane's X fill instructions of tile t fetch (tail rows repeat the last valid row): the
// gather indices when A is gathered.  Split from setup_operands so that a tile can request the indices of the
// tile after it before its own main loop, and find them in registers when it sets that tile up.
template <int XL>
__device__ __forceinline__ void load_gather_rows(const GemmParams &p, const TileCtx &c, const TileDesc &t, int (&arow)[XL]) {
#pragma unroll
  for (int j = 0; j < XL; ++j) {
    int xr = t.m0 + (XL * c.wave + j) * 16 + c.fill_row;
    if (xr > t.rows_e - 1) xr = t.rows_e - 1;
    if (xr < 0) xr = 0;
    arow[j] = p.gather_a[t.row_base + xr];
  }
}

template <int XL, int WL>
__device__ __forceinline__ void setup_operands(const GemmParams &p, const TileCtx &c, const TileDesc &t,
                                               TileOperands<XL, WL> &op, const int *preloaded_rows = nullptr) {
  const bool gathered = p.gather_a != nullptr;
  const uint8_t *xbase = gathered ? p.a : p.a + static_cast<int64_t>(t.row_base + t.m0) * c.kbytes;
  const int64_t xrows = gathered ? p.a_rows : t.rows_e - t.m0;
  op.xrsrc = make_rsrc(xbase, xrows > 0 ? xrows * c.kbytes : 0xffffffffll);
  int n0 = t.n0;
  const int g = split_group(n0, p.n, p.ngroups);
  op.wrsrc = make_rsrc(kernel_args()->b[g] + (static_cast<int64_t>(t.e) * p.n + n0) * c.kbytes, static_cast<int64_t>(p.n - n0) * c.kbytes);
#pragma unroll
  for (int j = 0; j < XL; ++j) {
    int xr = t.m0 + (XL * c.wave + j) * 16 + c.fill_row;
    if (xr > t.rows_e - 1) xr = t.rows_e - 1;
    int64_t arow = xr - t.m0;
    if (gathered) {
      arow = preloaded_rows ? preloaded_rows[j] : p.gather_a[t.row_base + xr];
      if (p.a_rows > 0) arow = arow < 0 ? 0 : (arow >= p.a_rows ? p.a_rows - 1 : arow);
    }
    op.xoff[j] = static_cast<uint32_t>(arow * c.kbytes) + c.fill_chunk * 16;
  }
#pragma unroll
  for (int j = 0; j < WL; ++j) {
    int wr = n0 + (WL * c.wave + j) * 16 + c.fill_row;
    if (wr > p.n - 1) wr = p.n - 1;
    op.woff[j] = static_cast<uint32_t>((wr - n0) * c.kbytes) + c.fill_chunk * 16;
  }
}

// The partial last k-step of a K that is not a whole number of k-steps: lanes whose 16-byte chunk lies inside
// the row fetch it, the others write zeros to their LDS slot themselves (an out-of-range direct-to-LDS load
// writes nothing).  Still one vector-memory instruction per wave, so the fill counts of the waits hold; the
// LDS write is waited for on the spot (a rare path: once per operand row group and tile).
__device__ __forceinline__ void fill_partial(__amdgpu_buffer_rsrc_t rsrc, uint32_t off, int kbyte, uint8_t *dst,
                                             const TileCtx &c) {
  if (c.fill_chunk < c.tail_chunks) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)dst, 16, static_cast<int>(off), kbyte, 0, 0);
  } else {
    *reinterpret_cast<u32x4 *>(dst + c.lane * 16) = u32x4{0u, 0u, 0u, 0u};
  }
  FLUXMI_WAITCNT(63, 0);
}

// Fill instruction q (X rows first, then W rows) of k-step `kstep` of a tile into ring slot `slot`.  A
// k-step past the end of K (the phantom second half of the last pair of an odd K) is filled from the
// zero page.  The k offset travels as the scalar offset: an instruction immediate would also be added
// to the LDS address.
template <int XL, int WL>
__device__ __forceinline__ void fill_any(const TileOperands<XL, WL> &op, uint8_t *smem, const TileCtx &c, int q, int slot,
                                         int kstep) {
  const bool in = kstep < c.nkf;
  const int kbyte = in ? kstep * KBYTES : 0;
  const __amdgpu_buffer_rsrc_t zrsrc = make_rsrc(g_zero_page, 1024);
  const uint32_t zoff = c.lane * 16;
  uint8_t *const dst = q < XL ? smem + slot * Ring<XL, WL>::SB + (XL * c.wave + q) * 1024
                              : smem + slot * Ring<XL, WL>::SB + Ring<XL, WL>::XB + (WL * c.wave + (q - XL)) * 1024;
  if (kstep == c.nkf && c.tail_chunks != 0) {  // wave-uniform
    if (q < XL) fill_partial(op.xrsrc, op.xoff[q < XL ? q : 0], kstep * KBYTES, dst, c);
    else fill_partial(op.wrsrc, op.woff[q >= XL ? q - XL : 0], kstep * KBYTES, dst, c);
    return;
  }
  if (q < XL)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(in ? op.xrsrc : zrsrc, (lds_ptr_t)dst, 16,
                                             static_cast<int>(in ? op.xoff[q < XL ? q : 0] : zoff), kbyte, 0, 0);
  else
    __builtin_amdgcn_raw_ptr_buffer_load_lds(in ? op.wrsrc : zrsrc, (lds_ptr_t)dst, 16,
                                             static_cast<int>(in ? op.woff[q >= XL ? q - XL : 0] : zoff), kbyte, 0, 0);
}

// Requests the first LA k-steps of a tile pair by pair into ring slots 0..LA-1 (q is a constant after unrolling).
template <int XL, int WL>
__device__ __forceinline__ void issue_first_pairs(const TileOperands<XL, WL> &op, uint8_t *smem, const TileCtx &c) {
  if (c.nkf >= Ring<XL, WL>::LA) {
    // All of these k-steps are whole ones (every K of practical interest): the same fills without the per-fill
    // choice between operand, partial step and zero page; slots and k offsets are immediates.
#pragma unroll
    for (int s = 0; s < Ring<XL, WL>::LA; s += 2) {
#pragma unroll
      for (int q = 0; q < XL + WL; ++q) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          if (q < XL)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(op.xrsrc, (lds_ptr_t)(smem + (s + h) * Ring<XL, WL>::SB + (XL * c.wave + q) * 1024),
                                                     16, static_cast<int>(op.xoff[q < XL ? q : 0]), (s + h) * KBYTES, 0, 0);
          else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                op.wrsrc, (lds_ptr_t)(smem + (s + h) * Ring<XL, WL>::SB + Ring<XL, WL>::XB + (WL * c.wave + (q - XL)) * 1024), 16,
                static_cast<int>(op.woff[q >= XL ? q - XL : 0]), (s + h) * KBYTES, 0, 0);
        }
      }
    }
    return;
  }
#pragma unroll
  for (int s = 0; s < Ring<XL, WL>::LA; s += 2) {
#pragma unroll
    for (int q = 0; q < XL + WL; ++q) {
      fill_any<XL, WL>(op, smem, c, q, s, s);
      fill_any<XL, WL>(op, smem, c, q, s + 1, s + 1);
    }
  }
}

// ---- the same tile with whole-line ring fills ---------------------------------------------------------------
// The unit of the ring is one operand's share of a PAIR of k-steps: 64*NB (64*MB) rows x 128 bytes, at most 32 KiB,
// one of five ring slots; W of pair P is unit 2P, X of pair P unit 2P + 1, unit u lies in slot u % 5.  A fill
// instruction fetches 8 rows x 128 bytes, whole cache lines (the 64-byte form fetches the two halves of a line with
// two instructions: the second finds the line in L1, but the memory pipeline handles it twice — measured on fills
// alone 88 against 101 GB/s per compute unit).  During the even step of pair P the W unit of pair P + 2 is
// requested (into the slot X of pair P - 1 has left), during the odd step its X unit (into the slot of W of pair P,
// whose last fragment reads were issued during the even step).  A pair's units are read by both of its steps, so
// only odd steps wait and synchronise: one `s_waitcnt vmcnt` and one barrier per pair of k-steps.  A unit is requested
// two (X) to three (W) steps before its first read; the fills per step and the LDS banks of the fragment reads are
// those of the 64-byte ring.  What the form costs: a pair's 64 KiB stay in LDS for both of its steps, so between 32
// and 96 KiB of fills are in flight where the 64-byte ring keeps 64 to 96 — enough while the compute units that share
// operand panels run in step and share each L2 miss, too little for a unit that runs apart from the others (ragged
// row counts), which is why a launch picks its form by shape (grouped_gemm.hip).
template <int MB, int NB>
struct LineRing {
  static constexpr int XF = 2 * MB;  // fill instructions per wave and pair: X unit
  static constexpr int WF = 2 * NB;  // ... W unit
  static constexpr int UB = STAGE_BYTES;  // bytes of a ring slot
  static constexpr int ROWB = 2 * KBYTES;  // bytes of a row in a unit
};

template <int XF, int WF>
struct LineOperands {
  __amdgpu_buffer_rsrc_t xrsrc, wrsrc;
  uint32_t xoff[XF], woff[WF];
};

struct LinePrefetch {
  bool valid;
  LineOperands<8, 8> op;
};

template <int XF>
__device__ __forceinline__ void load_gather_rows_lines(const GemmParams &p, const TileCtx &c, const TileDesc &t, int (&arow)[XF]) {
#pragma unroll
  for (int j = 0; j < XF; ++j) {
    int xr = t.m0 + (XF * c.wave + j) * 8 + c.lfill_row;
    if (xr > t.rows_e - 1) xr = t.rows_e - 1;
    if (xr < 0) xr = 0;
    arow[j] = p.gather_a[t.row_base + xr];
  }
}

template <int XF, int WF>
__device__ __forceinline__ void setup_operands_lines(const GemmParams &p, const TileCtx &c, const TileDesc &t,
                                                     LineOperands<XF, WF> &op, const int *preloaded_rows = nullptr) {
  const bool gathered = p.gather_a != nullptr;
  const uint8_t *xbase = gathered ? p.a : p.a + static_cast<int64_t>(t.row_base + t.m0) * c.kbytes;
  const int64_t xrows = gathered ? p.a_rows : t.rows_e - t.m0;
  op.xrsrc = make_rsrc(xbase, xrows > 0 ? xrows * c.kbytes : 0xffffffffll);
  int n0 = t.n0;
  const int g = split_group(n0, p.n, p.ngroups);
  op.wrsrc = make_rsrc(kernel_args()->b[g] + (static_cast<int64_t>(t.e) * p.n + n0) * c.kbytes, static_cast<int64_t>(p.n - n0) * c.kbytes);
#pragma unroll
  for (int j = 0; j < XF; ++j) {
    int xr = t.m0 + (XF * c.wave + j) * 8 + c.lfill_row;
    if (xr > t.rows_e - 1) xr = t.rows_e - 1;
    int64_t arow = xr - t.m0;
    if (gathered) {
      arow = preloaded_rows ? preloaded_rows[j] : p.gather_a[t.row_base + xr];
      if (p.a_rows > 0) arow = arow < 0 ? 0 : (arow >= p.a_rows ? p.a_rows - 1 : arow);
    }
    op.xoff[j] = static_cast<uint32_t>(arow * c.kbytes) + c.lfill_byte[j & 1];
  }
#pragma unroll
  for (int j = 0; j < WF; ++j) {
    int wr = n0 + (WF * c.wave + j) * 8 + c.lfill_row;
    if (wr > p.n - 1) wr = p.n - 1;
    op.woff[j] = static_cast<uint32_t>((wr - n0) * c.kbytes) + c.lfill_byte[j & 1];
  }
}

// Fill instruction q of a unit (an operand's 128 bytes of K at byte offset kb of every row) into LDS at dst, whatever
// kb is: a whole unit, the last unit of a K that is not a multiple of 128 bytes (lanes whose 16 bytes lie inside the
// row fetch them, the others write zeros to their own LDS slot: an out-of-range direct-to-LDS load writes
// nothing), or a unit past the end of K (requested from a page of zeros, so that the fill counts of the waits
// hold).  `lane_byte` is the lane's byte offset inside the 128 bytes.
__device__ __forceinline__ void fill_unit_any(__amdgpu_buffer_rsrc_t rsrc, uint32_t off, int lane_byte, int64_t kb, uint8_t *dst,
                                              const TileCtx &c) {
  if (kb + 128 <= c.kbytes) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)dst, 16, static_cast<int>(off), static_cast<int>(kb), 0, 0);
  } else if (kb < c.kbytes) {  // wave-uniform
    if (lane_byte < static_cast<int>(c.kbytes - kb)) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)dst, 16, static_cast<int>(off), static_cast<int>(kb), 0, 0);
    } else {
      *reinterpret_cast<u32x4 *>(dst + c.lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
    FLUXMI_WAITCNT(63, 0);
  } else {
    const __amdgpu_buffer_rsrc_t zrsrc = make_rsrc(g_zero_page, 1024);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(zrsrc, (lds_ptr_t)dst, 16, c.lane * 16, 0, 0, 0);
  }
}

// Requests the first two pairs of a tile: units 0..3 (W0, X0, W1, X1) into ring slots 0..3.
template <int XF, int WF>
__device__ __forceinline__ void issue_first_units(const LineOperands<XF, WF> &op, uint8_t *smem, const TileCtx &c) {
  constexpr int UB = STAGE_BYTES;
  if (c.kbytes >= 256) {  // all four are whole units (every K of practical interest): no per-fill choices
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
#pragma unroll
      for (int q = 0; q < WF; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(op.wrsrc, (lds_ptr_t)(smem + (2 * pr) * UB + (WF * c.wave + q) * 1024), 16,
                                                 static_cast<int>(op.woff[q]), pr * 128, 0, 0);
#pragma unroll
      for (int q = 0; q < XF; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(op.xrsrc, (lds_ptr_t)(smem + (2 * pr + 1) * UB + (XF * c.wave + q) * 1024), 16,
                                                 static_cast<int>(op.xoff[q]), pr * 128, 0, 0);
    }
    return;
  }
#pragma unroll
  for (int pr = 0; pr < 2; ++pr) {
#pragma unroll
    for (int q = 0; q < WF; ++q)
      fill_unit_any(op.wrsrc, op.woff[q], c.lfill_byte[q & 1], pr * 128, smem + (2 * pr) * UB + (WF * c.wave + q) * 1024, c);
#pragma unroll
    for (int q = 0; q < XF; ++q)
      fill_unit_any(op.xrsrc, op.xoff[q], c.lfill_byte[q & 1], pr * 128, smem + (2 * pr + 1) * UB + (XF * c.wave + q) * 1024, c);
  }
}

// Operand addressing and first fills of the whole macro tile `next`, in the form its tile function expects.
__device__ __forceinline__ void prefetch_whole_tile(const GemmParams &p, uint8_t *smem, const TileCtx &c, const TileDesc &next,
                                                    TilePrefetch &pf, const int *rows) {
  setup_operands<4, 4>(p, c, next, pf.op, rows);
  issue_first_pairs<4, 4>(pf.op, smem, c);
  pf.valid = true;
}
__device__ __forceinline__ void prefetch_whole_tile(const GemmParams &p, uint8_t *smem, const TileCtx &c, const TileDesc &next,
                                                    LinePrefetch &pf, const int *rows) {
  setup_operands_lines<8, 8>(p, c, next, pf.op, rows);
  issue_first_units<8, 8>(pf.op, smem, c);
  pf.valid = true;
}

// One output tile of (64*MB) rows x (64*NB) columns at rows [m0, ..) of expert e, columns [n0, ..).
// (MB, NB) = (4, 4) is the macro tile, (2, 4) its upper half (for the last rows of an expert); (4, 2) and
// (2, 2) are the 256x128 and 128x128 pieces a tile of the last, partly filled round is cut into.  Waves
// are laid out 2 x 2.
template <int ELT, int MB, int NB, class PF>
__device__ __forceinline__ void gemm_tile(const GemmParams &p, uint8_t *smem, const TileCtx &c, const TileDesc &t,
                                          const TileDesc &next, PF &pf) {
  // PF = TilePrefetch: every tile shape of the launch runs this function.  PF = LinePrefetch: whole, half-height,
  // half-width and 64-row tiles run gemm_tile_lines, and a whole tile that follows one of this function's tiles
  // gets its first fills in that function's form.
  constexpr bool LINES_NEXT = std::is_same<PF, LinePrefetch>::value;
  static_assert(!LINES_NEXT || MB != 4 || NB != 4, "whole tiles of such a launch run gemm_tile_lines");
  constexpr int XLOADS = MB;           // direct-to-LDS instructions per wave per stage, X tile
  constexpr int WLOADS = NB;           // same, W tile
  constexpr int LOADS = XLOADS + WLOADS;
  constexpr int STG = Ring<MB, NB>::STG, SB = Ring<MB, NB>::SB, XB = Ring<MB, NB>::XB, LA = Ring<MB, NB>::LA;
  constexpr int BLK = Geom<ELT>::BLK, NCH = Geom<ELT>::NCH;
  constexpr int MBK = 32 * MB / BLK, NBK = 32 * NB / BLK;  // operand blocks of a wave
  constexpr int NR = (MBK + NBK) * NCH;  // fragment reads per k-step (16 bytes per lane each)
  constexpr int NM = MBK * NBK;          // MFMAs per k-step
  constexpr int RSPAN = NM / 2;        // MFMA slots over which the fragment reads of a step are spread
  constexpr int PAIR = 2 * LOADS;  // vector-memory instructions per wave and pair of k-steps
  constexpr int HALF = LOADS;      // ... of which the pair's first step issues this many
  constexpr int WAIT_EVEN = (LA - 2) / 2 * PAIR;  // outstanding fills allowed when an even step starts
  constexpr int WAIT_ODD = (LA - 4) / 2 * PAIR + HALF;
  // A fill's M0 write is set apart from its load (one MFMA slot ahead) only while every fill of a pair of steps has
  // an MFMA slot of its own; with more fills than slots (fp8 tiles 64 rows high) the whole fill stays in one place.
  constexpr bool SPLIT_M0 = LOADS <= NM;
  const int wave = c.wave, lane = c.lane, wm = c.wm, wn = c.wn, nk = c.nk;
  const int e = t.e, row_base = t.row_base, rows_e = t.rows_e, m0 = t.m0;

  // Operand addressing: prepared by the previous tile together with the first fills, or set up here.
  bool prefetched = false;
  TileOperands<XLOADS, WLOADS> op;
  if constexpr (MB == 4 && NB == 4 && !LINES_NEXT) {
    if (pf.valid) {
      prefetched = true;
      op = pf.op;
    }
  }
  if (!prefetched) setup_operands<XLOADS, WLOADS>(p, c, t, op);
  // The gather indices of the next tile (when it is a whole macro tile, whose first fills this tile requests
  // ahead of its epilogue): requested now, so that their latency passes under this tile's main loop.
  constexpr int NPRE = LINES_NEXT ? 8 : 4;  // row indices per lane of a whole tile's X fills
  int next_rows[NPRE] = {};
  const bool preload_next = next.kind == 0 && p.gather_a != nullptr;
  if (preload_next) {
    if constexpr (LINES_NEXT) load_gather_rows_lines<NPRE>(p, c, next, next_rows);
    else load_gather_rows<NPRE>(p, c, next, next_rows);
  }
  const __amdgpu_buffer_rsrc_t xrsrc = op.xrsrc, wrsrc = op.wrsrc;
  uint32_t xoff[XLOADS], woff[WLOADS];
#pragma unroll
  for (int j = 0; j < XLOADS; ++j) xoff[j] = op.xoff[j];
#pragma unroll
  for (int j = 0; j < WLOADS; ++j) woff[j] = op.woff[j];
  // LDS destinations of this wave's fill instructions inside a stage (X rows first, then W rows).
  uint8_t *xdst = smem + (XLOADS * wave) * 1024;
  uint8_t *wdst = smem + XB + (WLOADS * wave) * 1024;

  // Fill instruction Q of the k-step at byte offset kbyte of every row, into ring slot SLOT (compile-time
  // slot: the LDS address is an immediate).  The k offset travels as the scalar offset: an instruction
  // immediate would also be added to the LDS address.
  // The 64 x 64 pieces of a skinny tail read their weights once and from HBM (470 MB on the Mixtral shape, after
  // the launch's other tiles): those fills are marked non-temporal, so that they do not push the output the launch
  // has just written out of the Infinity Cache ahead of the kernel that reads it next.
  constexpr int W_AUX = Ring<MB, NB>::tiny ? 2 : 0;  // cache policy of the weight fills: 2 = nt
  auto fill_one = [&](auto SLOT, auto Q, int kbyte) {
    constexpr int slot = decltype(SLOT)::value, q = decltype(Q)::value;
    if constexpr (q < XLOADS)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, (lds_ptr_t)(xdst + slot * SB + q * 1024), 16,
                                               static_cast<int>(xoff[q]), kbyte, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(wrsrc, (lds_ptr_t)(wdst + slot * SB + (q - XLOADS) * 1024), 16,
                                               static_cast<int>(woff[q - XLOADS]), kbyte, 0, W_AUX);
  };
  // The same fill as two instructions placed by hand: the LDS destination goes into M0 one MFMA slot ahead
  // of the load.  The builtin emits s_mov m0 / s_nop / buffer_load as one cluster; every instruction between
  // two MFMAs costs about two cycles of the MFMA pipe, and set apart the pair needs no s_nop (+0.7 % end to
  // end).  Nothing else in the k loop uses M0.
  const uint32_t xdst32 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)xdst));
  const uint32_t wdst32 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)wdst));
  auto fill_m0 = [&](auto SLOT, auto Q) {
    constexpr int slot = decltype(SLOT)::value, q = decltype(Q)::value;
    const uint32_t dst = q < XLOADS ? xdst32 + slot * SB + q * 1024 : wdst32 + slot * SB + (q - XLOADS) * 1024;
    // M0 cannot be named in the clobber list (the compiler reserves it and warns that such a clobber is not
    // honoured), so nothing tells the compiler that M0 changes here.  It is safe while the compiler itself puts
    // no M0 use between this statement and the load that follows it (the schedule barriers around every MFMA slot
    // see to that) and re-initialises M0 before every fill it emits itself (it does: the builtin writes M0 each
    // time); the test that compares this variant bit for bit with the builtin-only fills guards both.
    asm volatile("s_mov_b32 m0, %0" : : "s"(dst) : "memory");
  };
  auto fill_go = [&](auto Q, int kbyte) {
    constexpr int q = decltype(Q)::value;
    if constexpr (q < XLOADS) {
      const uint32_t vo = xoff[q];
      __amdgpu_buffer_rsrc_t r = xrsrc;
      asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(vo), "s"(r), "s"(kbyte) : "memory");
    } else {
      const uint32_t vo = woff[q - XLOADS];
      __amdgpu_buffer_rsrc_t r = wrsrc;
      if constexpr (W_AUX == 2) asm volatile("buffer_load_dwordx4 %0, %1, %2 offen nt lds" : : "v"(vo), "s"(r), "s"(kbyte) : "memory");
      else asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(vo), "s"(r), "s"(kbyte) : "memory");
    }
  };
  typename Geom<ELT>::Acc acc[MBK][NBK];
#pragma unroll
  for (int i = 0; i < MBK; ++i)
#pragma unroll
    for (int j = 0; j < NBK; ++j)
#pragma unroll
      for (int v = 0; v < Geom<ELT>::NACC; ++v) acc[i][j][v] = 0.f;

  // Fragment addresses: per lane and 16-byte chunk s a base for each operand; a stage and block add a
  // compile-time offset.  LDS instructions carry 16 bits of offset, so three bases 64 KiB apart.
  const uint8_t *xfrag[3][NCH], *wfrag[3][NCH];
#pragma unroll
  for (int hi = 0; hi < 3; ++hi)
#pragma unroll
    for (int s = 0; s < NCH; ++s) {
      xfrag[hi][s] = smem + hi * 65536 + wm * (32 * MB) * KBYTES + c.frag_off[s];
      wfrag[hi][s] = smem + hi * 65536 + XB + wn * (32 * NB) * KBYTES + c.frag_off[s];
    }
  i32x4 xa[MBK][NCH], wa[NBK][NCH], xb[MBK][NCH], wb[NBK][NCH];
  // Fragment read R of the k-step in ring slot SLOT: chunk s = R / (MBK + NBK) of W block q (q < NBK) or of
  // X block q - NBK.
  auto read_one = [&](auto SLOT, auto R, i32x4 (&xf)[MBK][NCH], i32x4 (&wf)[NBK][NCH]) {
    constexpr int slot = decltype(SLOT)::value, r = decltype(R)::value;
    constexpr int s = r / (MBK + NBK), q = r % (MBK + NBK);
    constexpr int hi = (slot * SB) / 65536, lo = (slot * SB) % 65536;
    if constexpr (q < NBK) wf[q][s] = *reinterpret_cast<const i32x4 *>(wfrag[hi][s] + lo + q * BLK * KBYTES);
    else xf[q - NBK][s] = *reinterpret_cast<const i32x4 *>(xfrag[hi][s] + lo + (q - NBK) * BLK * KBYTES);
  };

  // One k-step, number U within a run of ten (ring of five slots x two fragment sets: after ten steps
  // every slot index and register role repeats, so all of them are compile-time constants here).
  // MFMAs run on `cur` (read during the previous step), the fragments of the next step go into `nxt`,
  // and half of the fills of the pair of steps (E+4, E+5), E = U rounded down to even, are issued:
  // that pair is requested over the two steps E and E+1, row group by row group, both k-steps of a row
  // group back to back (the second one hits the line the first one brought into L1).
  // GUARDED (the last steps of a tile; they start at a multiple of the trip length, so ring slots and fragment sets are
  // the trip's): a k-step the step requests may be the partial last one of a K that is not a multiple of 64 bytes, or
  // lie past the end of K.  Its fills go through flat addresses, per lane either its 16 bytes of the operand or, where
  // those lie past the end of the row, 16 bytes of a page of zeros: one vector-memory instruction per fill either
  // way, so the fill counts of the waits hold.  kb0 is the byte offset along K of step 0 of the trip, xbase / wbase
  // (guarded steps only) the operands' first bytes.
  auto step = [&](auto GUARDED, auto U, int64_t kb0, const uint8_t *xbase, const uint8_t *wbase, i32x4 (&xc)[MBK][NCH],
                  i32x4 (&wc)[NBK][NCH], i32x4 (&xn)[MBK][NCH], i32x4 (&wn_)[NBK][NCH]) {
    constexpr bool guarded = decltype(GUARDED)::value;
    constexpr int u = decltype(U)::value;
    constexpr bool even = (u & 1) == 0;
    constexpr int e0 = u & ~1;
    const int kbase = static_cast<int>(kb0);
    int valid[2] = {KBYTES, KBYTES};          // guarded: bytes of the two requested k-steps that lie inside K
    int64_t gk[2] = {0, 0};                   // ... and their byte offsets along K
    if constexpr (guarded) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int64_t kb = kb0 + (e0 + LA + h) * KBYTES;
        const int64_t rem = c.kbytes - kb;
        valid[h] = rem >= KBYTES ? KBYTES : (rem <= 0 ? 0 : static_cast<int>(rem));
        gk[h] = rem > 0 ? kb : 0;
      }
    }
    // Stage u+1 has landed once the pair it belongs to is complete; fills are counted in issue order.
    if constexpr (even) {
      FLUXMI_WAITCNT(WAIT_EVEN, 15);  // all but the pairs requested since the one stage u+1 is in
    } else {
      FLUXMI_WAITCNT(WAIT_ODD, 15);  // ... and the half pair requested during the last step
    }
    __builtin_amdgcn_s_barrier();     // ... for every wave's share; and everybody is done reading stage u
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NM>([&](auto T) {
      constexpr int t = decltype(T)::value;
      static_for<0, NR>([&](auto R) {
        constexpr int r = decltype(R)::value;
        if constexpr (r * RSPAN / NR == t) read_one(std::integral_constant<int, (u + 1) % STG>{}, R, xn, wn_);
      });
      // Loads of this slot first, M0 writes for the loads of the next slot after them: a whole fill placed
      // here (fill_one writes M0 itself) must not come between another fill's M0 write and its load.
      static_for<0, 2 * LOADS>([&](auto D) {
        constexpr int d = decltype(D)::value;
        constexpr int at = (d * (2 * NM) / (2 * LOADS) + 1) % (2 * NM);
        if constexpr (at == t + (even ? 0 : NM)) {
          if constexpr (guarded) {
            constexpr int q = d >> 1, h = d & 1, slot = (e0 + LA + h) % STG;
            const bool ok = c.fill_chunk * 16 < valid[h];
            if constexpr (q < XLOADS) {
              const uint8_t *src = ok ? xbase + gk[h] + xoff[q] : g_zero_page + lane * 16;
              __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)(xdst + slot * SB + q * 1024), 16, 0, 0);
            } else {
              const uint8_t *src = ok ? wbase + gk[h] + woff[q - XLOADS] : g_zero_page + lane * 16;
              __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)(wdst + slot * SB + (q - XLOADS) * 1024), 16, 0, W_AUX);
            }
          } else if constexpr (SPLIT_M0 && at % NM != 0)  // the slot before is in the same step: M0 was written there
            fill_go(std::integral_constant<int, (d >> 1)>{}, kbase + (e0 + LA + (d & 1)) * KBYTES);
          else
            fill_one(std::integral_constant<int, (e0 + LA + (d & 1)) % STG>{}, std::integral_constant<int, (d >> 1)>{},
                     kbase + (e0 + LA + (d & 1)) * KBYTES);
        }
      });
      static_for<0, 2 * LOADS>([&](auto D) {
        constexpr int d = decltype(D)::value;
        constexpr int at = (d * (2 * NM) / (2 * LOADS) + 1) % (2 * NM);
        if constexpr (!guarded && SPLIT_M0 && at % NM != 0 && at - 1 == t + (even ? 0 : NM))
          fill_m0(std::integral_constant<int, (e0 + LA + (d & 1)) % STG>{}, std::integral_constant<int, (d >> 1)>{});
      });
      mfma_slot<ELT, MBK, NBK>(t, xc, wc, acc);
      __builtin_amdgcn_sched_barrier(0);
    });
    FLUXMI_WAITCNT(63, 0);  // the fragments of the next step are in registers (requested long ago)
    __builtin_amdgcn_sched_barrier(0);
  };
  // ---- prologue: k-steps 0..3 requested as two pairs, here or by the previous tile ahead of its epilogue --
  FLUXMI_WAITCNT(0, 0);  // stores of the previous tile's epilogue (and, if it requested them, the first fills)
  if (!prefetched) issue_first_pairs<XLOADS, WLOADS>(op, smem, c);
  FLUXMI_WAITCNT(WAIT_EVEN, 15);
  __builtin_amdgcn_s_barrier();
  static_for<0, NR>([&](auto R) { read_one(std::integral_constant<int, 0>{}, R, xa, wa); });
  FLUXMI_WAITCNT(63, 0);  // in registers before the first step's barrier lets anyone refill that slot

  // ---- main loop ----------------------------------------------------------------------------------
  // Whole trips of TRIP k-steps while every k-step a trip requests (up to TRIP - 1 + LA past its first one) is a
  // whole one, then the remaining steps pair by pair with guarded fills.  An odd number of k-steps ends with a
  // phantom step on zero fragments.
  constexpr int TRIP = Ring<MB, NB>::TRIP;
  const int nkf = c.nkf;
  const int nfast = nkf >= TRIP + LA ? (nkf - (TRIP + LA)) / TRIP + 1 : 0;  // trips with TRIP * trip + TRIP - 1 + LA < nkf
  int kbase = 0;  // byte offset along K of step 0 of the current trip
  for (int trip = 0; trip < nfast; ++trip) {
    static_for<0, TRIP / 2>([&](auto H) {
      constexpr int u = 2 * decltype(H)::value;
      step(std::false_type{}, std::integral_constant<int, u>{}, kbase, nullptr, nullptr, xa, wa, xb, wb);
      step(std::false_type{}, std::integral_constant<int, u + 1>{}, kbase, nullptr, nullptr, xb, wb, xa, wa);
    });
    kbase += TRIP * KBYTES;
  }
  if (TRIP * nfast < nk) {
    const KernArgs pe = kernel_args();
    const uint8_t *xbase = pe->gather_a != nullptr ? pe->a : pe->a + static_cast<int64_t>(row_base + m0) * c.kbytes;
    int n0g = t.n0;
    const int gg = split_group(n0g, pe->n, pe->ngroups);
    const uint8_t *wbase = pe->b[gg] + (static_cast<int64_t>(e) * pe->n + n0g) * c.kbytes;
    int64_t kb = static_cast<int64_t>(kbase);
    for (int ks = TRIP * nfast; ks < nk; ks += TRIP, kb += TRIP * KBYTES) {
      static_for<0, TRIP / 2>([&](auto H) {
        constexpr int u = 2 * decltype(H)::value;
        if (ks + u < nk) {
          step(std::true_type{}, std::integral_constant<int, u>{}, kb, xbase, wbase, xa, wa, xb, wb);
          step(std::true_type{}, std::integral_constant<int, u + 1>{}, kb, xbase, wbase, xb, wb, xa, wa);
        }
      });
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------------
  FLUXMI_WAITCNT(0, 0);          // this wave's trailing ring fills have landed
  __builtin_amdgcn_s_barrier();  // ... and everybody else's; nobody reads the ring any more
  // A whole macro tile next: its first four k-steps are requested now, into ring slots 0..3; the
  // epilogue's LDS windows lie in slot 4.
  pf.valid = false;
  if (next.kind == 0) prefetch_whole_tile(p, smem, c, next, pf, preload_next ? next_rows : nullptr);
  uint8_t *windows = smem + 4 * STAGE_BYTES + wave * 8192;  // one 8 KiB window per wave
  const int wrow0 = m0 + wm * (32 * MB);
  {
    const KernArgs pe = kernel_args();
    int n0 = t.n0;
    const int g = split_group(n0, pe->n, pe->ngroups);
    const int wcol0 = n0 + wn * (32 * NB);
    const bool full = wrow0 + 32 * MB <= rows_e && wcol0 + 32 * NB <= pe->n && pe->scatter_d == nullptr &&
                      pe->accumulate == 0;
    const bool out_f32 = pe->d_fp32 != 0;
    const bool scaled = !(c.scalar == 1.f && pe->alpha[g] == nullptr && pe->row_scale == nullptr && pe->col_scale == nullptr);
    auto store = [&](const typename Geom<ELT>::Acc (&res)[MBK][NBK]) {
      if (full && !scaled) {
        if (out_f32) store_tile<ELT, MB, NB, true, true, false>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, res);
        else store_tile<ELT, MB, NB, true, false, false>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, res);
      } else if (full) {
        if (out_f32) store_tile<ELT, MB, NB, true, true, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, res);
        else store_tile<ELT, MB, NB, true, false, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, res);
      } else {
        if (out_f32) store_tile<ELT, MB, NB, false, true, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, res);
        else store_tile<ELT, MB, NB, false, false, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, res);
      }
    };
    store(acc);
  }
  __builtin_amdgcn_s_barrier();  // the LDS windows are free again before the next tile's fills start
}

template <int ELT, int MB, int NB>
__device__ __forceinline__ void gemm_tile_lines(const GemmParams &p, uint8_t *smem, const TileCtx &c, const TileDesc &t,
                                                const TileDesc &next, LinePrefetch &pf) {
  constexpr int XF = LineRing<MB, NB>::XF, WF = LineRing<MB, NB>::WF;
  constexpr int UB = LineRing<MB, NB>::UB, ROWB = LineRing<MB, NB>::ROWB;
  constexpr int BLK = Geom<ELT>::BLK, NCH = Geom<ELT>::NCH;
  constexpr int MBK = 32 * MB / BLK, NBK = 32 * NB / BLK;  // operand blocks of a wave
  constexpr int NR = (MBK + NBK) * NCH;                    // fragment reads per k-step (16 bytes per lane each)
  constexpr int NM = MBK * NBK;                            // MFMAs per k-step
  constexpr int RSPAN = NM / 2;                            // MFMA slots over which the fragment reads of a step are spread
  constexpr int TRIP = 10;                                 // k-steps after which ring slots and fragment sets repeat
  const int wave = c.wave, wm = c.wm, wn = c.wn, nk = c.nk;
  const int e = t.e, row_base = t.row_base, rows_e = t.rows_e, m0 = t.m0;

  bool prefetched = false;
  LineOperands<XF, WF> op;
  if constexpr (MB == 4 && NB == 4) {
    if (pf.valid) {
      prefetched = true;
      op = pf.op;
    }
  }
  if (!prefetched) setup_operands_lines<XF, WF>(p, c, t, op);
  int next_rows[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  const bool preload_next = next.kind == 0 && p.gather_a != nullptr;
  if (preload_next) load_gather_rows_lines<8>(p, c, next, next_rows);
  const __amdgpu_buffer_rsrc_t xrsrc = op.xrsrc, wrsrc = op.wrsrc;
  uint32_t xoff[XF], woff[WF];
#pragma unroll
  for (int j = 0; j < XF; ++j) xoff[j] = op.xoff[j];
#pragma unroll
  for (int j = 0; j < WF; ++j) woff[j] = op.woff[j];
  uint8_t *xdst = smem + (XF * wave) * 1024;  // this wave's first fill block inside an X unit
  uint8_t *wdst = smem + (WF * wave) * 1024;
  const uint32_t xdst32 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)xdst));
  const uint32_t wdst32 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)wdst));

  // Fill instruction Q of the X (IS_W: W) unit at byte offset kbyte of every row into ring slot SLOT, as one cluster
  // (the builtin writes M0 itself) ...
  auto fill_one = [&](auto IS_W, auto SLOT, auto Q, int kbyte) {
    constexpr int slot = decltype(SLOT)::value, q = decltype(Q)::value;
    if constexpr (!decltype(IS_W)::value)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, (lds_ptr_t)(xdst + slot * UB + q * 1024), 16, static_cast<int>(xoff[q]), kbyte, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(wrsrc, (lds_ptr_t)(wdst + slot * UB + q * 1024), 16, static_cast<int>(woff[q]), kbyte, 0, 0);
  };
  // ... or as two instructions placed by hand: the LDS destination goes into M0 one MFMA slot ahead of the load.
  // Nothing else in the k loop uses M0; the compiler is not told that M0 changes, which is safe while it puts no M0
  // use of its own between the two (the schedule barriers around every MFMA slot see to that).
  auto fill_m0 = [&](auto IS_W, auto SLOT, auto Q) {
    constexpr int slot = decltype(SLOT)::value, q = decltype(Q)::value;
    const uint32_t dst = (decltype(IS_W)::value ? wdst32 : xdst32) + slot * UB + q * 1024;
    asm volatile("s_mov_b32 m0, %0" : : "s"(dst) : "memory");
  };
  auto fill_go = [&](auto IS_W, auto Q, int kbyte) {
    constexpr int q = decltype(Q)::value;
    if constexpr (decltype(IS_W)::value) {
      const uint32_t vo = woff[q];
      __amdgpu_buffer_rsrc_t r = wrsrc;
      asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(vo), "s"(r), "s"(kbyte) : "memory");
    } else {
      const uint32_t vo = xoff[q];
      __amdgpu_buffer_rsrc_t r = xrsrc;
      asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(vo), "s"(r), "s"(kbyte) : "memory");
    }
  };

  typename Geom<ELT>::Acc acc[MBK][NBK];
#pragma unroll
  for (int i = 0; i < MBK; ++i)
#pragma unroll
    for (int j = 0; j < NBK; ++j)
#pragma unroll
      for (int v = 0; v < Geom<ELT>::NACC; ++v) acc[i][j][v] = 0.f;

  // Fragment addresses: per lane and 16-byte chunk s a base for each operand; slot, block and k-step parity add a
  // compile-time offset.  LDS instructions carry 16 bits of offset, so three bases 64 KiB apart.
  const uint8_t *xfrag[3][NCH], *wfrag[3][NCH];
#pragma unroll
  for (int hi = 0; hi < 3; ++hi)
#pragma unroll
    for (int s = 0; s < NCH; ++s) {
      xfrag[hi][s] = smem + hi * 65536 + wm * (32 * MB) * ROWB + c.lfrag_off[s];
      wfrag[hi][s] = smem + hi * 65536 + wn * (32 * NB) * ROWB + c.lfrag_off[s];
    }
  i32x4 xa[MBK][NCH], wa[NBK][NCH], xb[MBK][NCH], wb[NBK][NCH];
  // Fragment read R of k-step U (counted within a trip; step u is half u & 1 of pair u >> 1).
  auto read_one = [&](auto U, auto R, i32x4 (&xf)[MBK][NCH], i32x4 (&wf)[NBK][NCH]) {
    constexpr int u = decltype(U)::value % TRIP, r = decltype(R)::value;
    constexpr int ws = (2 * (u >> 1)) % 5, xs = (2 * (u >> 1) + 1) % 5, h = u & 1;
    constexpr int s = r / (MBK + NBK), q = r % (MBK + NBK);
    if constexpr (q < NBK)
      wf[q][s] = *reinterpret_cast<const i32x4 *>(wfrag[(ws * UB) / 65536][s] + (ws * UB) % 65536 + q * BLK * ROWB + h * 512);
    else
      xf[q - NBK][s] = *reinterpret_cast<const i32x4 *>(xfrag[(xs * UB) / 65536][s] + (xs * UB) % 65536 + (q - NBK) * BLK * ROWB + h * 512);
  };
  // One k-step, number U of a trip of ten: MFMAs on `cur`, the fragments of step U + 1 into `nxt`, and the fills of
  // one unit of pair U / 2 + 2 (even: X, odd: W), one fill per MFMA slot at most when there are slots enough.
  // GUARDED (the last steps of a tile, which run the same code with the same ring slots: they start at a multiple
  // of ten): the unit may be the last one of a K that is not a multiple of 128 bytes, or lie past the end of K.  Its
  // fills then go through flat addresses, per lane either its 16 bytes of the operand or, where those lie past the
  // end of the row, 16 bytes of a page of zeros; one vector-memory instruction per fill either way, so the fill
  // counts of the waits hold.  kb is the byte offset along K of step 0 of the trip; xbase / wbase (guarded steps
  // only) are the operands' first bytes.
  auto step = [&](auto GUARDED, auto U, int64_t kb, const uint8_t *xbase, const uint8_t *wbase, i32x4 (&xc)[MBK][NCH],
                  i32x4 (&wc)[NBK][NCH], i32x4 (&xn)[MBK][NCH], i32x4 (&wn_)[NBK][NCH]) {
    constexpr bool guarded = decltype(GUARDED)::value;
    constexpr int u = decltype(U)::value;
    constexpr bool even = (u & 1) == 0;
    constexpr int pr2 = (u >> 1) + 2;                      // pair whose unit this step requests
    constexpr int fslot = (2 * pr2 + (even ? 0 : 1)) % 5;  // ring slot of that unit
    constexpr int NF = even ? WF : XF;
    constexpr bool SPLIT = !guarded && NF < NM;  // every fill has an MFMA slot of its own, and the slot before it for its M0 write
    static_assert(!SPLIT || (NF - 1) * NM / NF + 1 < NM, "the last fill's load still lies inside the step");
    typedef std::integral_constant<bool, even> IsW;
    const int kbyte = static_cast<int>(kb) + pr2 * 128;
    int valid = 128;                 // guarded: bytes of the unit's 128 that lie inside K
    const uint8_t *gbase = nullptr;  // ... and the operand's first byte of the unit
    if constexpr (guarded) {
      const int64_t rem = c.kbytes - (kb + pr2 * 128);
      valid = rem >= 128 ? 128 : (rem <= 0 ? 0 : static_cast<int>(rem));
      gbase = (even ? wbase : xbase) + (rem > 0 ? kb + pr2 * 128 : 0);
    }
    if constexpr (!even) {
      FLUXMI_WAITCNT(WF, 15);        // everything but the W unit requested during the even step has landed: pair u/2 + 1
      __builtin_amdgcn_s_barrier();  // ... for every wave's share; and everybody is done reading W of this pair
    }
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NM>([&](auto T) {
      constexpr int t = decltype(T)::value;
      static_for<0, NR>([&](auto R) {
        constexpr int r = decltype(R)::value;
        if constexpr (r * RSPAN / NR == t) read_one(std::integral_constant<int, u + 1>{}, R, xn, wn_);
      });
      static_for<0, NF>([&](auto Q) {
        constexpr int q = decltype(Q)::value;
        if constexpr (guarded) {
          if constexpr (q * NM / NF == t) {
            uint32_t off;
            if constexpr (even) off = woff[q];
            else off = xoff[q];
            const uint8_t *src = c.lfill_byte[q & 1] < valid ? gbase + off : g_zero_page + c.lane * 16;
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)((even ? wdst : xdst) + fslot * UB + q * 1024), 16, 0, 0);
          }
        } else if constexpr (SPLIT) {
          if constexpr (q * NM / NF + 1 == t) fill_go(IsW{}, Q, kbyte);
        } else {
          if constexpr (q * NM / NF == t) fill_one(IsW{}, std::integral_constant<int, fslot>{}, Q, kbyte);
        }
      });
      static_for<0, NF>([&](auto Q) {
        constexpr int q = decltype(Q)::value;
        if constexpr (SPLIT && q * NM / NF == t) fill_m0(IsW{}, std::integral_constant<int, fslot>{}, Q);
      });
      mfma_slot<ELT, MBK, NBK>(t, xc, wc, acc);
      __builtin_amdgcn_sched_barrier(0);
    });
    FLUXMI_WAITCNT(63, 0);  // the fragments of the next step are in registers (requested long ago)
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- prologue: the first two pairs are requested here or by the previous tile ahead of its epilogue ----------
  FLUXMI_WAITCNT(0, 0);  // stores of the previous tile's epilogue (and, if it requested them, the first fills)
  if (!prefetched) issue_first_units<XF, WF>(op, smem, c);
  FLUXMI_WAITCNT(XF + WF, 15);  // pair 0 has landed
  __builtin_amdgcn_s_barrier();
  static_for<0, NR>([&](auto R) { read_one(std::integral_constant<int, 0>{}, R, xa, wa); });
  FLUXMI_WAITCNT(63, 0);

  // ---- main loop: whole trips while every unit a trip requests (up to pair 5 * trip + 6) is a whole one, then the
  // remaining 4 .. 13 steps pair by pair with guarded fills; an odd number of k-steps ends with a step on zeros -----
  const int nkf = c.nkf;
  const int nfast = nkf >= TRIP + 4 ? (nkf - (TRIP + 4)) / TRIP + 1 : 0;
  int kbase = 0;
  for (int trip = 0; trip < nfast; ++trip) {
    static_for<0, TRIP / 2>([&](auto H) {
      constexpr int u = 2 * decltype(H)::value;
      step(std::false_type{}, std::integral_constant<int, u>{}, kbase, nullptr, nullptr, xa, wa, xb, wb);
      step(std::false_type{}, std::integral_constant<int, u + 1>{}, kbase, nullptr, nullptr, xb, wb, xa, wa);
    });
    kbase += TRIP * KBYTES;
  }
  if (TRIP * nfast < nk) {
    const KernArgs pe = kernel_args();
    const uint8_t *xbase = pe->gather_a != nullptr ? pe->a : pe->a + static_cast<int64_t>(row_base + m0) * c.kbytes;
    int n0g = t.n0;
    const int gg = split_group(n0g, pe->n, pe->ngroups);
    const uint8_t *wbase = pe->b[gg] + (static_cast<int64_t>(e) * pe->n + n0g) * c.kbytes;
    int64_t kb = static_cast<int64_t>(kbase);
    for (int ks = TRIP * nfast; ks < nk; ks += TRIP, kb += TRIP * KBYTES) {
      static_for<0, TRIP / 2>([&](auto H) {
        constexpr int u = 2 * decltype(H)::value;
        if (ks + u < nk) {
          step(std::true_type{}, std::integral_constant<int, u>{}, kb, xbase, wbase, xa, wa, xb, wb);
          step(std::true_type{}, std::integral_constant<int, u + 1>{}, kb, xbase, wbase, xb, wb, xa, wa);
        }
      });
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------------
  FLUXMI_WAITCNT(0, 0);          // this wave's trailing ring fills have landed
  __builtin_amdgcn_s_barrier();  // ... and everybody else's; nobody reads the ring any more
  pf.valid = false;
  if (next.kind == 0) {
    setup_operands_lines(p, c, next, pf.op, preload_next ? next_rows : nullptr);
    issue_first_units(pf.op, smem, c);
    pf.valid = true;
  }
  uint8_t *windows = smem + 4 * STAGE_BYTES + wave * 8192;  // one 8 KiB window per wave, in ring slot 4
  const int wrow0 = m0 + wm * (32 * MB);
  {
    const KernArgs pe = kernel_args();
    int n0 = t.n0;
    const int g = split_group(n0, pe->n, pe->ngroups);
    const int wcol0 = n0 + wn * (32 * NB);
    const bool full = wrow0 + 32 * MB <= rows_e && wcol0 + 32 * NB <= pe->n && pe->scatter_d == nullptr &&
                      pe->accumulate == 0;
    const bool out_f32 = pe->d_fp32 != 0;
    const bool scaled = !(c.scalar == 1.f && pe->alpha[g] == nullptr && pe->row_scale == nullptr && pe->col_scale == nullptr);
    if (full && !scaled) {
      if (out_f32) store_tile<ELT, MB, NB, true, true, false>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, acc);
      else store_tile<ELT, MB, NB, true, false, false>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, acc);
    } else if (full) {
      if (out_f32) store_tile<ELT, MB, NB, true, true, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, acc);
      else store_tile<ELT, MB, NB, true, false, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, acc);
    } else {
      if (out_f32) store_tile<ELT, MB, NB, false, true, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, acc);
      else store_tile<ELT, MB, NB, false, false, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, acc);
    }
  }
  __builtin_amdgcn_s_barrier();  // the LDS windows are free again before the next tile's fills start
}

// Block-scaled fp8, one 256 x 128 piece: A carries one scale per row and 128 of K, B one per 128 x 128 block, and
// the products of every 128 of K are added to the result with a_scale[row] * b_scale (the promotion).
//
// The unit of the k loop is a pair of k-steps, i.e. one scale block: LDS rows hold 128 bytes of K, a ring stage is
// 256 X rows + 128 W rows + the 256 row scales of the pair (49 KiB; three stages).  A wave computes its 128 x 64
// quarter block by block: for each 32 x 32 block the two MFMAs of the pair (the first with C = 0), then
// main += block * scale — the block's sums live in vector registers for the length of three MFMAs and the promotion
// is one v_fmac per element (sums kept in accumulation registers across a whole k-step would cost a register read
// per element as well: with one wave per SIMD the vector ALU's time adds to the MFMA time).  Fragments of a whole
// pair are in registers, double-buffered: during pair kb the first half of the MFMA slots issues the fills of pair
// kb + 2 (stage (kb + 2) % 3), then one wait + barrier makes pair kb + 1 visible (requested during the first half
// of pair kb - 1), and the second half reads its fragments.  One barrier per 128 of K.
//
// A fill instruction covers 8 rows x 128 bytes (whole cache lines); chunk c of row r lies in 16-byte slot
// c ^ ((r >> 1) & 7) of the row, which makes the 32-row fragment reads free of bank conflicts.
__device__ __forceinline__ void gemm_tile_blockscaled(const GemmParams &p, uint8_t *smem, const TileCtx &c, const TileDesc &t) {
  constexpr int XROWS = 256, WROWS = 128, ROWB = 128;
  constexpr int XBYTES = XROWS * ROWB, WBYTES = WROWS * ROWB;  // 32 KiB, 16 KiB
  constexpr int SCALE_OFF = XBYTES + WBYTES;                   // 256 floats
  constexpr int PSB = SCALE_OFF + 1024;                        // bytes of a stage
  constexpr int NSTG = 3;
  static_assert(NSTG * PSB <= LDS_BYTES, "three stages fit the LDS");
  constexpr int XF = 8, WF = 4;          // fill instructions per wave and pair: X rows, W rows
  constexpr int PAIRF = XF + WF + 1;     // ... with the scale fill
  constexpr int MBK = 4, NBK = 2, NBLK = MBK * NBK;
  typedef Geom<1>::Acc Acc;
  const int wave = c.wave, lane = c.lane, wm = c.wm, wn = c.wn;
  const int e = t.e, row_base = t.row_base, rows_e = t.rows_e, m0 = t.m0;
  const int kblocks = c.nk >> 1;
  const KernArgs pe = kernel_args();

  // ---- operand addressing -------------------------------------------------------------------------------
  const bool gathered = p.gather_a != nullptr;
  const uint8_t *xbase = gathered ? p.a : p.a + static_cast<int64_t>(row_base + m0) * c.kbytes;
  const int64_t xrows = gathered ? p.a_rows : rows_e - m0;
  const __amdgpu_buffer_rsrc_t xrsrc = make_rsrc(xbase, xrows > 0 ? xrows * c.kbytes : 0xffffffffll);
  int n0 = t.n0;
  const int g = split_group(n0, p.n, p.ngroups);
  const __amdgpu_buffer_rsrc_t wrsrc =
      make_rsrc(pe->b[g] + (static_cast<int64_t>(e) * p.n + n0) * c.kbytes, static_cast<int64_t>(p.n - n0) * c.kbytes);
  const __amdgpu_buffer_rsrc_t zrsrc = make_rsrc(g_zero_page, 1024);
  const uint32_t zoff = (lane & 7) * 16;
  uint32_t xoff[XF], woff[WF];
#pragma unroll
  for (int j = 0; j < XF; ++j) {
    int xr = m0 + 64 * wave + 8 * j + (lane >> 3);
    if (xr > rows_e - 1) xr = rows_e - 1;
    if (xr < 0) xr = 0;
    int64_t arow = xr - m0;
    if (gathered) {
      arow = p.gather_a[row_base + xr];
      if (p.a_rows > 0) arow = arow < 0 ? 0 : (arow >= p.a_rows ? p.a_rows - 1 : arow);
    }
    const int chunk = (lane & 7) ^ ((4 * j + (lane >> 4)) & 7);
    xoff[j] = static_cast<uint32_t>(arow * c.kbytes) + chunk * 16;
  }
#pragma unroll
  for (int j = 0; j < WF; ++j) {
    int wr = n0 + 32 * wave + 8 * j + (lane >> 3);
    if (wr > p.n - 1) wr = p.n - 1;
    const int chunk = (lane & 7) ^ ((4 * j + (lane >> 4)) & 7);
    woff[j] = static_cast<uint32_t>((wr - n0) * c.kbytes) + chunk * 16;
  }
  // Scales: lane l of a wave fetches the scale of tile row 64 * wave + l.
  const __amdgpu_buffer_rsrc_t as_rsrc = make_rsrc(reinterpret_cast<const uint8_t *>(pe->a_scale), 0xffffffffll);
  uint32_t as_voff;
  int as_kstep, bs_base, bs_kstep;
  {
    int xr = m0 + 64 * wave + lane;
    if (xr > rows_e - 1) xr = rows_e - 1;
    int64_t arow = row_base + xr;
    if (gathered) {
      arow = p.gather_a[row_base + xr];
      if (p.a_rows > 0) arow = arow < 0 ? 0 : (arow >= p.a_rows ? p.a_rows - 1 : arow);
    }
    if (pe->a_scale_layout == FLUXMI_ASCALE_BLOCK128) {  // [ceil(rows/128), K/128, 128], row in block fastest
      as_voff = static_cast<uint32_t>(((arow >> 7) * kblocks * 128 + (arow & 127)) * 4);
      as_kstep = 128 * 4;
    } else {  // per expert [K/128, rows of the expert], experts back to back
      as_voff = static_cast<uint32_t>((static_cast<int64_t>(row_base) * kblocks + xr) * 4);
      as_kstep = rows_e * 4;
    }
    const int nb = n0 >> 7, nblocks = (pe->n + 127) >> 7;
    if (pe->b_scale_layout == FLUXMI_BSCALE_N_K) {  // [E, N/128, K/128]
      bs_base = (e * nblocks + nb) * kblocks;
      bs_kstep = 1;
    } else {  // [E, K/128, N/128]
      bs_base = e * kblocks * nblocks + nb;
      bs_kstep = nblocks;
    }
  }
  typedef const __attribute__((address_space(4))) float *ConstF32;
  const ConstF32 bscale = (ConstF32)(pe->b_scale);
  auto bscale_of = [&](int kb) { return bscale[__builtin_amdgcn_readfirstlane(bs_base + (kb < kblocks ? kb : 0) * bs_kstep)]; };

  // Fill instruction Q of pair kb into stage STAGE: the scale fill first, then X row groups, then W row groups.
  // Past the end of K the fills read the zero page (the fill counts of the waits must hold).
  uint8_t *const xdst = smem + (XF * wave) * 1024;
  uint8_t *const wdst = smem + XBYTES + (WF * wave) * 1024;
  auto fill = [&](auto STAGE, auto Q, int kb) {
    constexpr int stage = decltype(STAGE)::value, q = decltype(Q)::value;
    const bool in = kb < kblocks;
    if constexpr (q == 0)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(in ? as_rsrc : zrsrc, (lds_ptr_t)(smem + stage * PSB + SCALE_OFF + wave * 256), 4,
                                               static_cast<int>(in ? as_voff : static_cast<uint32_t>(lane * 4)),
                                               in ? kb * as_kstep : 0, 0, 0);
    else if constexpr (q <= XF)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(in ? xrsrc : zrsrc, (lds_ptr_t)(xdst + stage * PSB + (q - 1) * 1024), 16,
                                               static_cast<int>(in ? xoff[q - 1] : zoff), in ? kb * ROWB : 0, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(in ? wrsrc : zrsrc, (lds_ptr_t)(wdst + stage * PSB + (q - 1 - XF) * 1024), 16,
                                               static_cast<int>(in ? woff[q - 1 - XF] : zoff), in ? kb * ROWB : 0, 0, 0);
  };

  // Fragments of a pair: block b of an operand, k-step h of the pair, 16-byte chunk s (a 32x32x64 MFMA takes two).
  // Lane l reads row l & 31 of the block, logical chunk 4 h + 2 (l >> 5) + s.
  struct Frags {
    i32x4 x[MBK][2][2], w[NBK][2][2];
  };
  Frags fa, fb;
  float sa[MBK], sb[MBK];  // row scales of the pair, as read
  uint32_t roff[2][2];     // byte offset of (h, s) inside a 32-row block, this lane
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const int r = lane & 31, ch = 4 * h + 2 * (lane >> 5) + s2;
      roff[h][s2] = r * ROWB + ((ch ^ ((r >> 1) & 7)) << 4);
    }
  const uint8_t *const xread = smem + wm * 128 * ROWB;
  const uint8_t *const wread = smem + XBYTES + wn * 64 * ROWB;
  const float *const sread = reinterpret_cast<const float *>(smem + SCALE_OFF) + wm * 128 + (lane & 31);
  // Read number R (0 .. 25) of the pair in stage STAGE: 16 X chunks, 8 W chunks, then the row scales (2 x 2).
  auto read_one = [&](auto STAGE, auto R, Frags &f, float (&sc)[MBK]) {
    constexpr int stage = decltype(STAGE)::value, r = decltype(R)::value;
    if constexpr (r < 16) {
      constexpr int i = r >> 2, h = (r >> 1) & 1, s2 = r & 1;
      f.x[i][h][s2] = *reinterpret_cast<const i32x4 *>(xread + stage * PSB + i * 32 * ROWB + roff[h][s2]);
    } else if constexpr (r < 24) {
      constexpr int j = (r - 16) >> 2, h = ((r - 16) >> 1) & 1, s2 = (r - 16) & 1;
      f.w[j][h][s2] = *reinterpret_cast<const i32x4 *>(wread + stage * PSB + j * 32 * ROWB + roff[h][s2]);
    } else {
      constexpr int i0 = (r - 24) * 2;
      sc[i0] = sread[stage * (PSB / 4) + i0 * 32];
      sc[i0 + 1] = sread[stage * (PSB / 4) + (i0 + 1) * 32];
    }
  };
  constexpr int NREADS = 26;

  Acc main_acc[MBK][NBK];
#pragma unroll
  for (int i = 0; i < MBK; ++i)
#pragma unroll
    for (int j = 0; j < NBK; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) main_acc[i][j][v] = 0.f;

  auto mfma = [&](const Frags &f, int i, int j, int h, Acc cacc) {
    i32x8 wa, xa;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      wa[v] = f.w[j][h][0][v];
      wa[4 + v] = f.w[j][h][1][v];
      xa[v] = f.x[i][h][0][v];
      xa[4 + v] = f.x[i][h][1][v];
    }
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wa, xa, cacc, 0, 0, 0, 0, 0, 0);
  };

  // One pair of k-steps, number U within a run of six (three stages x two fragment sets): MFMAs on `cur`, the
  // fragments and scales of the next pair into `nxt`.  MFMA slot t: blocks two at a time, (b, k0) (b+1, k0) (b, k1)
  // (b+1, k1), so that the second MFMA of a block does not follow its first directly; block b is promoted two slots
  // after its second MFMA.
  float bsv_next = 0.f;
  auto pair_step = [&](auto U, int kb0, const Frags &cur, const float (&scur)[MBK], Frags &nxt, float (&snxt)[MBK], float bsv) {
    constexpr int u = decltype(U)::value;
    const int kb = kb0 + u;
    float psc[MBK];
#pragma unroll
    for (int i = 0; i < MBK; ++i) psc[i] = scur[i] * bsv;
    bsv_next = bscale_of(kb + 1);
    Acc blk[NBLK];
    static_for<0, 2 * NBLK>([&](auto T) {
      constexpr int tt = decltype(T)::value;
      constexpr int b = (tt >> 2) * 2 + (tt & 1), h = (tt >> 1) & 1;
      if constexpr (tt < NBLK) {
        // first half: the fills of pair kb + 2
        static_for<0, PAIRF>([&](auto Q) {
          constexpr int q = decltype(Q)::value;
          if constexpr (q * NBLK / PAIRF == tt) fill(std::integral_constant<int, (u + 2) % NSTG>{}, Q, kb + 2);
        });
      } else {
        if constexpr (tt == NBLK) {
          // pair kb + 1 has landed (everything but the fills just issued), for every wave's share
          FLUXMI_WAITCNT(PAIRF, 15);
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_sched_barrier(0);
        }
        static_for<0, NREADS>([&](auto R) {
          constexpr int r = decltype(R)::value;
          if constexpr (r * NBLK / NREADS == tt - NBLK) read_one(std::integral_constant<int, (u + 1) % NSTG>{}, R, nxt, snxt);
        });
      }
      if constexpr (h == 0) blk[b] = mfma(cur, b / NBK, b % NBK, 0, Acc{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f});
      else blk[b] = mfma(cur, b / NBK, b % NBK, 1, blk[b]);
      // promotion of the block whose second MFMA was issued two slots ago
      if constexpr (tt >= 4 && ((tt - 2) >> 1 & 1) == 1) {
        constexpr int pb = ((tt - 2) >> 2) * 2 + ((tt - 2) & 1);
#pragma unroll
        for (int v = 0; v < 16; ++v) main_acc[pb / NBK][pb % NBK][v] = fmaf(blk[pb][v], psc[pb / NBK], main_acc[pb / NBK][pb % NBK][v]);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    // the last two blocks
    static_for<NBLK - 2, NBLK>([&](auto B) {
      constexpr int pb = decltype(B)::value;
#pragma unroll
      for (int v = 0; v < 16; ++v) main_acc[pb / NBK][pb % NBK][v] = fmaf(blk[pb][v], psc[pb / NBK], main_acc[pb / NBK][pb % NBK][v]);
    });
    FLUXMI_WAITCNT(63, 0);  // the fragments of the next pair are in registers
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- prologue: pairs 0 and 1 requested, pair 0 read ---------------------------------------------------
  FLUXMI_WAITCNT(0, 0);  // stores of the previous tile's epilogue
  static_for<0, PAIRF>([&](auto Q) { fill(std::integral_constant<int, 0>{}, Q, 0); });
  static_for<0, PAIRF>([&](auto Q) { fill(std::integral_constant<int, 1>{}, Q, 1); });
  float bsv = bscale_of(0);
  FLUXMI_WAITCNT(PAIRF, 15);
  __builtin_amdgcn_s_barrier();
  static_for<0, NREADS>([&](auto R) { read_one(std::integral_constant<int, 0>{}, R, fa, sa); });
  FLUXMI_WAITCNT(63, 0);

  // ---- main loop: six pairs per trip, pairs past the end of K skipped ------------------------------------
  // (A skipped pair issues no fills either: the waits count the fills of executed pairs only, and those are the
  // same for every wave.)
  for (int kb0 = 0; kb0 < kblocks; kb0 += 6) {
    pair_step(std::integral_constant<int, 0>{}, kb0, fa, sa, fb, sb, bsv);
    bsv = bsv_next;
    if (kb0 + 1 < kblocks) { pair_step(std::integral_constant<int, 1>{}, kb0, fb, sb, fa, sa, bsv); bsv = bsv_next; }
    if (kb0 + 2 < kblocks) { pair_step(std::integral_constant<int, 2>{}, kb0, fa, sa, fb, sb, bsv); bsv = bsv_next; }
    if (kb0 + 3 < kblocks) { pair_step(std::integral_constant<int, 3>{}, kb0, fb, sb, fa, sa, bsv); bsv = bsv_next; }
    if (kb0 + 4 < kblocks) { pair_step(std::integral_constant<int, 4>{}, kb0, fa, sa, fb, sb, bsv); bsv = bsv_next; }
    if (kb0 + 5 < kblocks) { pair_step(std::integral_constant<int, 5>{}, kb0, fb, sb, fa, sa, bsv); bsv = bsv_next; }
  }

  // ---- epilogue -------------------------------------------------------------------------------------------
  FLUXMI_WAITCNT(0, 0);          // this wave's trailing fills have landed
  __builtin_amdgcn_s_barrier();  // ... and everybody else's; nobody reads the ring any more
  uint8_t *windows = smem + wave * 8192;  // one 8 KiB window per wave
  const int wrow0 = m0 + wm * 128;
  {
    const int wcol0 = n0 + wn * 64;
    const bool full = wrow0 + 128 <= rows_e && wcol0 + 64 <= pe->n && pe->scatter_d == nullptr && pe->accumulate == 0;
    const bool out_f32 = pe->d_fp32 != 0;
    const bool scaled = !(c.scalar == 1.f && pe->alpha[g] == nullptr && pe->row_scale == nullptr && pe->col_scale == nullptr);
    if (full && !scaled) {
      if (out_f32) store_tile<1, 4, 2, true, true, false, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, main_acc);
      else store_tile<1, 4, 2, true, false, false, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, main_acc);
    } else if (full) {
      if (out_f32) store_tile<1, 4, 2, true, true, true, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, main_acc);
      else store_tile<1, 4, 2, true, false, true, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, main_acc);
    } else {
      if (out_f32) store_tile<1, 4, 2, false, true, true, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, main_acc);
      else store_tile<1, 4, 2, false, false, true, true>(windows, c, g, e, row_base, rows_e, wrow0, wcol0, main_acc);
    }
  }
  __builtin_amdgcn_s_barrier();  // the LDS windows are free again before the next tile's fills start
}

#endif  // __HIP_DEVICE_COMPILE__

// LINE_FILLS is part of the kernel's name only (kLineFills decides the code): traces tell the two forms apart.
template <int ELT, bool BS = false, bool LINE_FILLS = kLineFills>
__global__ __launch_bounds__(NTHREADS) void grouped_gemm_mfma_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];  // STAGES x (X tile | W tile)

  TileCtx c;
  const int tid = threadIdx.x;
  c.wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: branches on it stay uniform
  c.lane = tid & 63;
  c.wn = c.wave & 1;   // column half
  c.wm = c.wave >> 1;  // row half
  const int lane = c.lane;
  const int tiles_n1 = (p.n + BN - 1) / BN;  // column tiles of one weight group
  const int tiles_n = tiles_n1 * p.ngroups;  // ... of the launch
  c.kbytes = static_cast<int64_t>(p.k) * ELT;
  c.nkf = static_cast<int>(c.kbytes / KBYTES);
  c.tail_chunks = static_cast<int>(c.kbytes % KBYTES) / 16;
  c.nk = c.nkf + (c.tail_chunks != 0 ? 1 : 0);

  // LDS tile layout: rows of 64 bytes = four 16-byte chunks; a direct-to-LDS fill instruction covers 16
  // rows = 1 KiB, lane l landing at byte 16 * l of it, so which (row, chunk) a slot holds is decided by the
  // address the lane fetches from.  The chunks of a row are permuted so that the fragment reads of the
  // element type run without bank conflicts (measured: ds_read_b128 at 235 B/clk/CU instead of 117):
  //   bf16 (a lane reads row l & 15, chunk l >> 4 of a 16-row block): row r at r * 64, chunk c in place
  //     c ^ ((r >> 1) & 3);
  //   fp8 (row l & 31, chunks 2 * (l >> 5) + s of a 32-row block): four rows per 256-byte line S = r >> 2,
  //     (row, chunk) in 16-byte slot ((r & 3) << 2) | (c ^ (S & 3)).
  // Either permutation conflicts for the other element type's read pattern.
  if (ELT == 2) {
    c.fill_row = lane >> 2;
    c.fill_chunk = (lane & 3) ^ ((lane >> 3) & 3);
    const int r = lane & 15, ch = lane >> 4;
    c.frag_off[0] = r * 64 + ((ch ^ ((r >> 1) & 3)) << 4);
    c.frag_off[1] = 0;
  } else {
    c.fill_row = lane >> 2;
    c.fill_chunk = (lane & 3) ^ ((lane >> 4) & 3);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int ch = 2 * (lane >> 5) + s;
      const int slot = ((lane & 3) << 2) | (ch ^ ((lane >> 2) & 3));
      c.frag_off[s] = ((lane & 31) >> 2) * 256 + slot * 16;
    }
  }
  // Whole-line fills: a 1 KiB block of LDS holds 8 rows x 128 bytes as two halves of 512 bytes (k-step parity),
  // each half laid out like 8 rows of the 64-byte layout above; lanes 0..31 of a fill instruction fetch the first
  // 64 bytes of the 8 rows, lanes 32..63 the second (the memory pipeline still sees whole 128-byte lines), and the
  // bank a fragment read touches is the same as in the 64-byte layout.
  c.lfill_row = (lane & 31) >> 2;
  if (ELT == 2) {
    c.lfill_byte[0] = c.lfill_byte[1] = (lane >> 5) * 64 + (((lane & 3) ^ ((lane >> 3) & 3)) << 4);
    const int r = lane & 15, ch = lane >> 4;
    c.lfrag_off[0] = (r >> 3) * 1024 + (r & 7) * 64 + ((ch ^ ((r >> 1) & 3)) << 4);
    c.lfrag_off[1] = 0;
  } else {
#pragma unroll
    for (int b = 0; b < 2; ++b)
      c.lfill_byte[b] = (lane >> 5) * 64 + (((lane & 3) ^ (((c.lfill_row >> 2) & 1) | (b << 1))) << 4);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int r = lane & 31, ch = 2 * (lane >> 5) + s;
      const int slot = ((lane & 3) << 2) | (ch ^ ((lane >> 2) & 3));
      c.lfrag_off[s] = (r >> 3) * 1024 + ((r >> 2) & 1) * 256 + slot * 16;
    }
  }
  c.scalar = p.scalar;
  if (p.scalar_dev) c.scalar *= p.scalar_dev[0];

  const int grid = gridDim.x;
  const int bid = blockIdx.x;
  // Workgroups are dealt to XCDs round-robin; give each XCD a run of consecutive logical work items.
  const int virt = (grid % 8 == 0) ? (bid & 7) * (grid >> 3) + (bid >> 3) : bid;

  // ---- tile counts (one wave-wide pass over splits) -> shape of the last round ------------------------
  // An expert whose last row tile holds 1 .. 64 rows is a candidate for a skinny tail: that row tile is then left
  // out of the expert's ordinary tiles and computed after all of them as 64 x 64 pieces (below).
  const bool cut_tail = (p.sched_flags & FLUXMI_SCHED_WHOLE_TAIL_TILES) == 0;
  const bool half_tiles = (p.sched_flags & FLUXMI_SCHED_NO_HALF_TILES) == 0;
  int total_tiles = 0, skinny_experts = 0;
  {
    int row_carry = 0, acc_tiles = 0, acc_cand = 0;
    for (int e0 = 0; e0 < p.nexperts; e0 += 64) {
      const int ee = e0 + lane;
      int rows = ee < p.nexperts ? p.splits[ee] : 0;
      if (rows < 0) rows = 0;
      const int incl = wave_inclusive_scan(rows);
      int begin = row_carry + incl - rows, end = row_carry + incl;
      if (begin > p.max_rows) begin = p.max_rows;
      if (end > p.max_rows) end = p.max_rows;
      int tiles = ((end - begin + BM - 1) / BM) * tiles_n;
      int cand = (end > begin && ((end - begin - 1) & (BM - 1)) < 64) ? 1 : 0;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        tiles += __shfl_xor(tiles, off, 64);
        cand += __shfl_xor(cand, off, 64);
      }
      acc_tiles += tiles;
      acc_cand += cand;
      row_carry += __shfl(incl, 63, 64);
    }
    total_tiles = __builtin_amdgcn_readfirstlane(acc_tiles);
    skinny_experts = __builtin_amdgcn_readfirstlane(acc_cand);
  }
  // Skinny tails.  A row tile with at most 64 rows costs a whole tile's weight traffic for a quarter of its MFMA
  // work, and as an ordinary work item it occupies one compute unit for that long while the static schedule gives
  // every unit the same number of items.  When such row tiles are few (their 64 x 64 pieces fill at most two
  // rounds: long K, few column tiles) they are numbered after all ordinary tiles and cut along N into 64-column
  // pieces, so that every unit streams an equal share of those experts' weights at the end; when they are many
  // (many column tiles) they already spread evenly as ordinary items and stay where they are, and so they do when K
  // is short (under 128 k-steps a piece is mostly its own start and end: measured 2-3 % slower on 64 experts at
  // K = 2048).
  const int skinny_tiles_all = skinny_experts * tiles_n;
  const bool skinny_on = !BS && half_tiles && (p.sched_flags & FLUXMI_SCHED_NO_SKINNY_TAIL) == 0 && skinny_tiles_all > 0 &&
                         ((p.sched_flags & FLUXMI_SCHED_FORCE_SKINNY_TAIL) != 0 || (skinny_tiles_all * 4 <= 2 * grid && c.nk >= 128));
  const int skinny_items = skinny_on ? skinny_tiles_all * 4 : 0;
  const int reg_tiles = total_tiles - (skinny_on ? skinny_tiles_all : 0);
  // Full rounds run whole macro tiles.  The tiles of the last, partly filled round are cut into
  // `pieces` parts (2 pieces of 256x128, or 4 of 128x128) when that still fits one round, so that the
  // chip does not idle while a fraction of the CUs finishes whole tiles.
  // Block-scaled launches run every tile as two 256 x 128 pieces (one column block of B's scales each).
  const int full_items = BS ? 0 : (reg_tiles / grid) * grid;
  const int rem_tiles = reg_tiles - full_items;
  const int pieces = BS ? 2 : (!cut_tail ? 1 : (rem_tiles * 4 <= grid ? 4 : (rem_tiles * 2 <= grid ? 2 : 1)));
  const int skinny_first = full_items + rem_tiles * pieces;  // first work item of the skinny pieces
  const int total_items = skinny_first + skinny_items;

  // ---- schedule: walk the experts once, in step with this workgroup's increasing tile ids ----------
  // All of it is wave-uniform scalar work on the device-resident splits (no LDS, no host round trip).
  // The walk is made twice: over the ordinary tiles, then (from work item skinny_first on) over the skinny pieces.
  int e = 0;
  int row_base = 0;   // sorted rows before expert e
  int tile_base = 0;  // ordinary tiles (second walk: skinny pieces) before expert e
  int rows_e = expert_rows(p, 0, 0);
  bool in_skinny = false;
  // Ordinary row tiles of an expert with `rows` rows / its skinny pieces.
  auto is_skinny = [&](int rows) { return skinny_on && rows > 0 && ((rows - 1) & (BM - 1)) < 64; };
  auto count_of = [&](int rows) {
    const int mt = (rows + BM - 1) / BM;
    if (in_skinny) return is_skinny(rows) ? tiles_n * 4 : 0;
    return (mt - (is_skinny(rows) ? 1 : 0)) * tiles_n;
  };
  int tiles_e = count_of(rows_e);

  // Work item -> tile (items must be asked for in increasing order).
  auto locate = [&](int item) {
    TileDesc t = {-2, 0, 0, 0, 0, 0};
    if (item >= total_items) return t;
    if (item >= skinny_first && !in_skinny) {  // restart the walk for the skinny pieces
      in_skinny = true;
      e = 0;
      row_base = 0;
      tile_base = 0;
      rows_e = expert_rows(p, 0, 0);
      tiles_e = count_of(rows_e);
    }
    int tile = item, piece = 0;
    if (in_skinny) {
      tile = item - skinny_first;
    } else if (item >= full_items) {
      tile = full_items + (item - full_items) / pieces;
      piece = (item - full_items) % pieces;
    }
    while (e < p.nexperts && tile >= tile_base + tiles_e) {
      tile_base += tiles_e;
      row_base += rows_e;
      ++e;
      if (e < p.nexperts) {
        rows_e = expert_rows(p, e, row_base);
        tiles_e = count_of(rows_e);
      }
    }
    if (e >= p.nexperts) return t;
    t.e = e;
    t.row_base = row_base;
    t.rows_e = rows_e;
    if (in_skinny) {
      // Piece `local` of the expert's last row tile: column tile local / 4 (over all weight groups), quarter local % 4.
      const int local = tile - tile_base;
      const int nt = local >> 2;
      const int g = p.ngroups > 1 ? nt / tiles_n1 : 0;
      t.m0 = ((rows_e - 1) / BM) * BM;
      t.n0 = (nt - g * tiles_n1) * BN + (local & 3) * 64;
      t.kind = t.n0 < p.n ? 4 : -1;
      t.n0 += g * tiles_n1 * BN;
      return t;
    }
    // Order inside an expert: row tiles are cut into groups of at most p.raster_rows (8 unless tuned); a group is walked
    // column-major over all weight panels before the next group starts.  32 consecutive tiles (one
    // XCD's share of a round) then cover about 8 row tiles x 4 panels: 12 distinct operand tiles per
    // k-step for 32 CUs.
    const int m_tiles = (rows_e + BM - 1) / BM - (is_skinny(rows_e) ? 1 : 0);
    const int ngroups_m = (m_tiles + p.raster_rows - 1) / p.raster_rows;
    const int gm = (m_tiles + ngroups_m - 1) / ngroups_m;  // group height, <= raster_rows
    const int local = tile - tile_base;
    const int group = local / (gm * tiles_n);
    const int group_first = group * gm;
    const int group_rows = m_tiles - group_first < gm ? m_tiles - group_first : gm;
    const int in_group = local - group * gm * tiles_n;
    const int nt = in_group / group_rows;
    const int mt = group_first + (in_group - nt * group_rows);
    t.m0 = mt * BM;
    const int g = p.ngroups > 1 ? nt / tiles_n1 : 0;
    const int gcol = g * tiles_n1 * BN;  // first virtual column of the weight group
    t.n0 = (nt - g * tiles_n1) * BN;
    if (item < full_items || pieces == 1) {
      // The last row tile of an expert is run 128 rows high when that covers its rows, the last column
      // tile 128 columns wide when that covers its columns (N = 1408: the sixth tile holds 128 columns).
      // With at most 64 rows left (and the skinny tail not in use for them) it runs 64 rows high.
      const bool low = half_tiles && rows_e - t.m0 <= 128;
      const bool narrow = half_tiles && p.n - t.n0 <= 128;
      t.kind = low ? (narrow ? 3 : (rows_e - t.m0 <= 64 ? 5 : 1)) : (narrow ? 2 : 0);
    } else if (pieces == 2) {
      t.n0 += piece * 128;
      t.kind = t.n0 < p.n ? 2 : -1;
    } else {
      t.m0 += (piece >> 1) * 128;
      t.n0 += (piece & 1) * 128;
      t.kind = (t.m0 < rows_e && t.n0 < p.n) ? 3 : -1;
    }
    t.n0 += gcol;
    return t;
  };

  typename std::conditional<kLineFills, LinePrefetch, TilePrefetch>::type pf;
  pf.valid = false;
  int item = virt;
  TileDesc cur = locate(item);
  while (cur.kind != -2) {
    item += grid;
    const TileDesc next = locate(item);
    if constexpr (BS) {
      if (cur.kind == 2) gemm_tile_blockscaled(p, smem, c, cur);
    } else if constexpr (kLineFills) {
      if (cur.kind == 0) gemm_tile_lines<ELT, 4, 4>(p, smem, c, cur, next, pf);
      else if (cur.kind == 1) gemm_tile_lines<ELT, 2, 4>(p, smem, c, cur, next, pf);
      else if (cur.kind == 2) gemm_tile_lines<ELT, 4, 2>(p, smem, c, cur, next, pf);
      else if (cur.kind == 3) gemm_tile<ELT, 2, 2>(p, smem, c, cur, next, pf);
      else if (cur.kind == 4) gemm_tile<ELT, 1, 1>(p, smem, c, cur, next, pf);
      else if (cur.kind == 5) gemm_tile_lines<ELT, 1, 4>(p, smem, c, cur, next, pf);
    } else {
      if (cur.kind == 0) gemm_tile<ELT, 4, 4>(p, smem, c, cur, next, pf);
      else if (cur.kind == 1) gemm_tile<ELT, 2, 4>(p, smem, c, cur, next, pf);
      else if (cur.kind == 2) gemm_tile<ELT, 4, 2>(p, smem, c, cur, next, pf);
      else if (cur.kind == 3) gemm_tile<ELT, 2, 2>(p, smem, c, cur, next, pf);
      else if (cur.kind == 4) gemm_tile<ELT, 1, 1>(p, smem, c, cur, next, pf);
      else if (cur.kind == 5) gemm_tile<ELT, 1, 4>(p, smem, c, cur, next, pf);
    }
    cur = next;
  }
#endif  // __HIP_DEVICE_COMPILE__
}

template <int ELT, bool BS = false>
int launch_mfma(const GemmParams &p, int grid, hipStream_t s) {
  static std::atomic<uint64_t> lds_done{0};
  const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(grouped_gemm_mfma_kernel<ELT, BS, kLineFills>), LDS_BYTES, lds_done);
  if (rc != FLUXMI_OK) return rc;
  hipLaunchKernelGGL((grouped_gemm_mfma_kernel<ELT, BS, kLineFills>), dim3(grid), dim3(NTHREADS), LDS_BYTES, s, p);
  return FLUXMI_OK;
}

}  // namespace
}  // namespace fluxmi
