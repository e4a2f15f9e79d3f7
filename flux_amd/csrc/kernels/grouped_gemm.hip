// Grouped GEMM over ragged per-expert row counts: D[r,:] = scale(r,:) * A[gather(r),:] @ B[e(r)]^T.
//
// Persistent kernel, one 512-thread workgroup (8 waves, 2 per SIMD) per CU, macro tile 256 rows x 256
// columns, k-step of 64 bytes per row (32 bf16 or 64 fp8).  Both operand tiles are staged in LDS by
// direct-to-LDS global loads (no register staging) in a 5-deep ring; the row gather of A is folded into
// the per-lane global address of those loads.  Each wave owns a 128x64 slice of the macro tile
// (4x2 MFMA blocks of 32x32, fp32 accumulators).  The two waves that share a SIMD run one phase apart
// ("ping-pong"): while one issues its LDS fragment reads and the next global loads, the other issues
// MFMAs, and workgroup barriers keep them alternating.
//
// The MFMA "A" operand is the weight fragment and the "B" operand the activation fragment, i.e. the
// hardware computes D^T blocks: a lane then holds, for one output row, four consecutive output columns
// per accumulator quad, which makes the epilogue's stores 8-byte packed bf16x4.
//
// Tile schedule: every wave walks the device-resident `splits` with scalar loads, in step with the
// increasing logical tile ids of its workgroup; ids are assigned so that the workgroups of one XCD
// (those with equal blockIdx % 8) take a run of consecutive tiles; tiles of an expert are ordered
// column-major (all row tiles of one weight panel first), so an XCD's L2 sees a few weight panels
// shared by all row tiles of the expert.
#include <cstdlib>

#include "common.hpp"

namespace fluxmi {
namespace {

constexpr int BM = 256;                    // rows of a macro tile
constexpr int KBYTES = 64;                 // bytes of K per row per k-step
constexpr int X_TILE_BYTES = BM * KBYTES;  // activation tile of one stage: 16 KiB

// Two macro tile widths.  NBMAX = number of 32-column MFMA blocks per wave (4 waves across):
//   NBMAX = 2: 256 x 256, stage 32 KiB, 5 stages;  NBMAX = 3: 256 x 384, stage 40 KiB, 4 stages.
// Both fill the 160 KiB LDS of a CU.  The wide tile moves 17 % fewer operand bytes per FLOP through
// L2, which is what bounds this kernel; its 192 accumulator registers leave room for the fragments of
// only half a k-step, so it runs its memory / MFMA phases per 32-byte half step (KSPLIT = 2).
template <int NBMAX>
struct TileCfg {
  static constexpr int BN = 128 * NBMAX;
  static constexpr int W_TILE_BYTES = BN * KBYTES;
  static constexpr int STAGE_BYTES = X_TILE_BYTES + W_TILE_BYTES;
  static constexpr int STAGES = NBMAX == 2 ? 5 : 4;
  static constexpr int DIST = STAGES - 1;  // prefetch distance in k-steps
  static constexpr int KSPLIT = NBMAX == 2 ? 1 : 2;
};
constexpr int NTHREADS = 512;
constexpr int kMaxExperts = 1024;

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct GemmParams {
  const uint8_t *a;
  const uint8_t *b;
  void *d;
  const int32_t *splits;
  const int32_t *gather_a;
  const int32_t *scatter_d;
  const float *alpha;
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
};

#define FLUXMI_WAITCNT(vm, lgkm) \
  __builtin_amdgcn_s_waitcnt(((vm)&15) | (((vm) >> 4) << 14) | (7 << 4) | ((lgkm) << 8))

typedef __attribute__((address_space(3))) void *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *gbl_ptr_t;

// One wave-wide direct-to-LDS load: lane l fetches 16 bytes from `src` (per lane) and the hardware
// stores them at lds_base + 16*l (lds_base is wave-uniform).
__device__ __forceinline__ void load_to_lds16(const uint8_t *src, uint8_t *lds_base) {
  __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)lds_base, 16, 0, 0);
}

template <int ELT>
__device__ __forceinline__ f32x16 mfma_step(const i32x4 (&w)[2], const i32x4 (&x)[2], f32x16 acc);

template <>
__device__ __forceinline__ f32x16 mfma_step<2>(const i32x4 (&w)[2], const i32x4 (&x)[2], f32x16 acc) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[0]),
                                                __builtin_bit_cast(bf16x8, x[0]), acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[1]),
                                                __builtin_bit_cast(bf16x8, x[1]), acc, 0, 0, 0);
  return acc;
}

// bf16 only: one 16-element half of a k-step.
__device__ __forceinline__ f32x16 mfma_half_bf16(const i32x4 &w, const i32x4 &x, f32x16 acc) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, x), acc,
                                                 0, 0, 0);
}

template <>
__device__ __forceinline__ f32x16 mfma_step<1>(const i32x4 (&w)[2], const i32x4 (&x)[2], f32x16 acc) {
  i32x8 wa, xa;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    wa[i] = w[0][i];
    wa[4 + i] = w[1][i];
    xa[i] = x[0][i];
    xa[4 + i] = x[1][i];
  }
  // cbsz = blgp = 0: both operands e4m3; zero scale operands select the unscaled form (scale 1).
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wa, xa, acc, 0, 0, 0, 0, 0, 0);
}

// Clamped row count of expert e: negative entries count as 0 and rows past max_rows do not exist.
__device__ __forceinline__ int expert_rows(const GemmParams &p, int e, int row_base) {
  int rows = p.splits[e];
  if (rows < 0) rows = 0;
  if (rows > p.max_rows - row_base) rows = p.max_rows - row_base;
  return rows;
}

// Per-lane constants and ring state shared by all tile shapes.
struct TileCtx {
  int wave, lane, wn, wm;
  int fill_row, fill_chunk;
  int frag_off[2];
  int fill_stage;  // ring slot the next issued k-step goes to
  int read_stage;  // ring slot of the k-step read next
  int nk;
  int64_t kbytes;
  float scalar;
};

// One output tile of (64*MB) rows x (128*NB) columns: MB x NB MFMA blocks of 32x32 per wave, waves laid
// out 2 (rows) x 4 (columns).  (MB, NB) = (4, NBMAX) is the macro tile; (4, 1) and (2, 1) are the 256x128
// and 128x128 pieces a tile of the last, partly filled round is cut into.  KSPLIT = 2 runs the
// memory / MFMA phase pair once per half k-step with half the fragment registers (bf16 only).
template <int ELT, int NBMAX, int MB, int NB, int KSPLIT>
__device__ __forceinline__ void gemm_tile(const GemmParams &p, uint8_t *smem, TileCtx &c, int e,
                                          int row_base, int rows_e, int m0, int n0) {
  using Cfg = TileCfg<NBMAX>;
  constexpr int STAGES = Cfg::STAGES, DIST = Cfg::DIST, STAGE_BYTES = Cfg::STAGE_BYTES;
  constexpr int XLOADS = MB / 2;             // direct-to-LDS instructions per wave per stage, X tile
  constexpr int WLOADS = NB;                 // same, W tile
  constexpr int LOADS = XLOADS + WLOADS;
  constexpr int NS = 2 / KSPLIT;             // 16-byte fragment chunks read per phase
  static_assert(KSPLIT == 1 || ELT == 2, "half k-steps exist for bf16 only");
  const int wave = c.wave, lane = c.lane, wm = c.wm, wn = c.wn, nk = c.nk;
  const int x_frag_base = wm * (32 * MB) * KBYTES;
  const int w_frag_base = X_TILE_BYTES + wn * (32 * NB) * KBYTES;

  // Global source pointers of this lane's fill instructions (k offset added per step).  Instruction q
  // of a tile covers rows [16q, 16q+16); tail rows re-read the last valid row.
  const uint8_t *xsrc[XLOADS];
  const uint8_t *wsrc[WLOADS];
#pragma unroll
  for (int j = 0; j < XLOADS; ++j) {
    int xr = m0 + (XLOADS * wave + j) * 16 + c.fill_row;
    if (xr > rows_e - 1) xr = rows_e - 1;
    int64_t arow = row_base + xr;
    if (p.gather_a) {
      arow = p.gather_a[arow];
      if (p.a_rows > 0) arow = arow < 0 ? 0 : (arow >= p.a_rows ? p.a_rows - 1 : arow);
    }
    xsrc[j] = p.a + arow * c.kbytes + c.fill_chunk * 16;
  }
#pragma unroll
  for (int j = 0; j < WLOADS; ++j) {
    int wr = n0 + (WLOADS * wave + j) * 16 + c.fill_row;
    if (wr > p.n - 1) wr = p.n - 1;
    wsrc[j] = p.b + (static_cast<int64_t>(e) * p.n + wr) * c.kbytes + c.fill_chunk * 16;
  }

  auto issue_stage = [&](int kstep) {
    uint8_t *stage = smem + c.fill_stage * STAGE_BYTES;
    c.fill_stage = c.fill_stage + 1 == STAGES ? 0 : c.fill_stage + 1;
    const int64_t koff = static_cast<int64_t>(kstep) * KBYTES;
#pragma unroll
    for (int j = 0; j < XLOADS; ++j) load_to_lds16(xsrc[j] + koff, stage + (XLOADS * wave + j) * 1024);
#pragma unroll
    for (int j = 0; j < WLOADS; ++j)
      load_to_lds16(wsrc[j] + koff, stage + X_TILE_BYTES + (WLOADS * wave + j) * 1024);
  };

  f32x16 acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // ---- prologue: fill DIST stages ---------------------------------------------------------------
  FLUXMI_WAITCNT(0, 0);  // stores of the previous tile's epilogue
#pragma unroll
  for (int s = 0; s < DIST; ++s)
    if (s < nk) issue_stage(s);
  if (nk >= DIST) {
    FLUXMI_WAITCNT((DIST - 1) * LOADS, 15);
  } else {
    FLUXMI_WAITCNT(0, 15);
  }
  __builtin_amdgcn_s_barrier();
  if (wm == 1) __builtin_amdgcn_s_barrier();  // group 1 runs one phase behind group 0

  for (int ks = 0; ks < nk; ++ks) {
    const uint8_t *stage = smem + c.read_stage * STAGE_BYTES;
    c.read_stage = c.read_stage + 1 == STAGES ? 0 : c.read_stage + 1;
    const bool more = ks + DIST < nk;
#pragma unroll
    for (int sub = 0; sub < KSPLIT; ++sub) {
      // ---- memory phase -------------------------------------------------------------------------
      i32x4 xf[MB][NS], wf[NB][NS];
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int s = 0; s < NS; ++s)
          wf[j][s] = *reinterpret_cast<const i32x4 *>(stage + w_frag_base + j * 32 * KBYTES +
                                                      c.frag_off[KSPLIT == 1 ? s : sub]);
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int s = 0; s < NS; ++s)
          xf[i][s] = *reinterpret_cast<const i32x4 *>(stage + x_frag_base + i * 32 * KBYTES +
                                                      c.frag_off[KSPLIT == 1 ? s : sub]);
      if (sub == 0 && more) issue_stage(ks + DIST);
      if (sub == KSPLIT - 1) {
        if (more) {
          FLUXMI_WAITCNT((DIST - 1) * LOADS, 0);  // stage ks+1 landed, fragments in registers
        } else {
          FLUXMI_WAITCNT(0, 0);
        }
      } else {
        FLUXMI_WAITCNT(63, 0);  // fragments in registers; global loads keep flying
      }
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      // ---- compute phase ------------------------------------------------------------------------
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          if constexpr (KSPLIT == 1) acc[i][j] = mfma_step<ELT>(wf[j], xf[i], acc[i][j]);
          else acc[i][j] = mfma_half_bf16(wf[j][0], xf[i][0], acc[i][j]);
        }
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (wm == 0) __builtin_amdgcn_s_barrier();  // re-align the two groups

  // ---- epilogue: scale, cast, packed stores -------------------------------------------------------
  const float tile_scale = c.scalar * (p.alpha ? p.alpha[e] : 1.f);
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int m = m0 + wm * (32 * MB) + i * 32 + (lane & 31);
    if (m >= rows_e) continue;
    const int64_t srow = row_base + m;
    const float rs = tile_scale * (p.row_scale ? p.row_scale[srow] : 1.f);
    int64_t drow = srow;
    if (p.scatter_d) {
      drow = p.scatter_d[srow];
      if (drow < 0 || drow >= p.max_rows) continue;
    }
    uint16_t *dptr = static_cast<uint16_t *>(p.d) + drow * p.n;
    float *dptr32 = static_cast<float *>(p.d) + drow * p.n;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * (32 * NB) + j * 32 + q * 8 + (lane >> 5) * 4;
        if (n >= p.n) continue;  // n % 4 == 0 is required, so a quad is all in or all out
        float v0 = acc[i][j][4 * q + 0] * rs;
        float v1 = acc[i][j][4 * q + 1] * rs;
        float v2 = acc[i][j][4 * q + 2] * rs;
        float v3 = acc[i][j][4 * q + 3] * rs;
        if (p.col_scale) {
          const float4 cs = *reinterpret_cast<const float4 *>(p.col_scale + static_cast<int64_t>(e) * p.n + n);
          v0 *= cs.x;
          v1 *= cs.y;
          v2 *= cs.z;
          v3 *= cs.w;
        }
        if (p.d_fp32) {
          *reinterpret_cast<float4 *>(dptr32 + n) = make_float4(v0, v1, v2, v3);
        } else {
          u32x2 o;
          o[0] = float_to_bf16_bits(v0) | (static_cast<uint32_t>(float_to_bf16_bits(v1)) << 16);
          o[1] = float_to_bf16_bits(v2) | (static_cast<uint32_t>(float_to_bf16_bits(v3)) << 16);
          *reinterpret_cast<u32x2 *>(dptr + n) = o;
        }
      }
    }
  }
}

template <int ELT, int NBMAX>
__global__ __launch_bounds__(NTHREADS) void grouped_gemm_mfma_kernel(const GemmParams p) {
  constexpr int BN = TileCfg<NBMAX>::BN;
  constexpr int KSPLIT = TileCfg<NBMAX>::KSPLIT;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];  // STAGES x (X tile | W tile)

  TileCtx c;
  const int tid = threadIdx.x;
  c.wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: branches on it stay uniform
  c.lane = tid & 63;
  c.wn = c.wave & 3;   // column slice
  c.wm = c.wave >> 2;  // row slice == ping-pong group
  const int lane = c.lane;
  const int tiles_n = (p.n + BN - 1) / BN;
  c.kbytes = static_cast<int64_t>(p.k) * ELT;
  c.nk = static_cast<int>(c.kbytes / KBYTES);

  // LDS tile layout: rows of 64 bytes, four rows per 256-byte "superline" S = r >> 2 (the LDS serves
  // 64 banks x 4 bytes per clock, 16 lanes of a 16-byte read at a time).  (row r, chunk c) sits in
  // 16-byte slot ((r & 3) << 2) | (c ^ (S & 3)) of its superline, so the 16 rows read together by a
  // quarter wave (same chunk) fall into 16 different slots.
  // Direct-to-LDS fill: instruction q of a tile covers rows [16q, 16q+16) = 1 KiB; lane l lands in
  // superline 4q + (l >> 4), slot l & 15, i.e. row 16q + (l >> 2), chunk (l & 3) ^ ((l >> 4) & 3).
  c.fill_row = lane >> 2;
  c.fill_chunk = (lane & 3) ^ ((lane >> 4) & 3);
  // Fragment reads: lane l reads row (l & 31) of a 32-row block, chunk c(s) for s = 0,1.
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const int ch = ELT == 2 ? 2 * s + (lane >> 5) : 2 * (lane >> 5) + s;
    const int slot = ((lane & 3) << 2) | (ch ^ ((lane >> 2) & 3));
    c.frag_off[s] = ((lane & 31) >> 2) * 256 + slot * 16;
  }
  c.scalar = p.scalar;
  if (p.scalar_dev) c.scalar *= p.scalar_dev[0];
  c.fill_stage = 0;
  c.read_stage = 0;

  const int grid = gridDim.x;
  const int bid = blockIdx.x;
  // Workgroups are dealt to XCDs round-robin; give each XCD a run of consecutive logical work items.
  const int virt = (grid % 8 == 0) ? (bid & 7) * (grid >> 3) + (bid >> 3) : bid;

  // ---- total tile count (one wave-wide pass over splits) -> shape of the last round -----------------
  int total_tiles = 0;
  {
    int row_carry = 0, acc_tiles = 0;
    for (int e0 = 0; e0 < p.nexperts; e0 += 64) {
      const int ee = e0 + lane;
      int rows = ee < p.nexperts ? p.splits[ee] : 0;
      if (rows < 0) rows = 0;
      const int incl = wave_inclusive_scan(rows);
      int begin = row_carry + incl - rows, end = row_carry + incl;
      if (begin > p.max_rows) begin = p.max_rows;
      if (end > p.max_rows) end = p.max_rows;
      int tiles = ((end - begin + BM - 1) / BM) * tiles_n;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) tiles += __shfl_xor(tiles, off, 64);
      acc_tiles += tiles;
      row_carry += __shfl(incl, 63, 64);
    }
    total_tiles = __builtin_amdgcn_readfirstlane(acc_tiles);
  }
  // Full rounds run whole macro tiles.  The tiles of the last, partly filled round are cut into
  // `pieces` parts (NBMAX pieces of 256x128, or 2*NBMAX of 128x128) when that still fits one round, so
  // that the chip does not idle while a fraction of the CUs finishes whole tiles.
  const int full_items = (total_tiles / grid) * grid;
  const int rem_tiles = total_tiles - full_items;
  const int pieces = rem_tiles * 2 * NBMAX <= grid ? 2 * NBMAX : (rem_tiles * NBMAX <= grid ? NBMAX : 1);
  const int total_items = full_items + rem_tiles * pieces;

  // ---- schedule: walk the experts once, in step with this workgroup's increasing tile ids ----------
  // All of it is wave-uniform scalar work on the device-resident splits (no LDS, no host round trip).
  int e = 0;
  int row_base = 0;   // sorted rows before expert e
  int tile_base = 0;  // tiles before expert e
  int rows_e = expert_rows(p, 0, 0);
  int tiles_e = ((rows_e + BM - 1) / BM) * tiles_n;

  for (int item = virt; item < total_items; item += grid) {
    int tile = item, piece = 0;
    if (item >= full_items) {
      tile = full_items + (item - full_items) / pieces;
      piece = (item - full_items) % pieces;
    }
    while (e < p.nexperts && tile >= tile_base + tiles_e) {
      tile_base += tiles_e;
      row_base += rows_e;
      ++e;
      if (e < p.nexperts) {
        rows_e = expert_rows(p, e, row_base);
        tiles_e = ((rows_e + BM - 1) / BM) * tiles_n;
      }
    }
    if (e >= p.nexperts) break;
    // Order inside an expert: row tiles are cut into groups of at most 8; a group is walked
    // column-major over all weight panels before the next group starts.  32 consecutive tiles (one
    // XCD's share of a round) then cover about 8 row tiles x 4 panels: 12 distinct operand tiles per
    // k-step for 32 CUs.
    const int m_tiles = (rows_e + BM - 1) / BM;
    const int ngroups_m = (m_tiles + 7) >> 3;
    const int gm = (m_tiles + ngroups_m - 1) / ngroups_m;  // group height, <= 8
    const int local = tile - tile_base;
    const int group = local / (gm * tiles_n);
    const int group_first = group * gm;
    const int group_rows = m_tiles - group_first < gm ? m_tiles - group_first : gm;
    const int in_group = local - group * gm * tiles_n;
    const int nt = in_group / group_rows;
    const int mt = group_first + (in_group - nt * group_rows);
    int m0 = mt * BM;
    int n0 = nt * BN;

    if (item < full_items || pieces == 1) {
      gemm_tile<ELT, NBMAX, 4, NBMAX, KSPLIT>(p, smem, c, e, row_base, rows_e, m0, n0);
    } else if (pieces == NBMAX) {
      n0 += piece * 128;
      if (n0 < p.n) gemm_tile<ELT, NBMAX, 4, 1, 1>(p, smem, c, e, row_base, rows_e, m0, n0);
    } else {
      m0 += (piece / NBMAX) * 128;
      n0 += (piece % NBMAX) * 128;
      if (m0 < rows_e && n0 < p.n) gemm_tile<ELT, NBMAX, 2, 1, 1>(p, smem, c, e, row_base, rows_e, m0, n0);
    }
  }
}

// ---- generic kernel: any K / N, no alignment demands beyond element size -------------------------
// One thread per output element, a wave covers 64 consecutive columns of one row.  Only used when the
// MFMA kernel's shape requirements do not hold.
__device__ __forceinline__ float e4m3_to_float(uint8_t b) {
  const uint32_t sign = (b & 0x80u) << 24;
  const uint32_t em = b & 0x7fu;
  if (em == 0x7fu) return __uint_as_float(sign | 0x7fc00000u);
  if (em < 8u) return __uint_as_float(sign) + (sign ? -1.f : 1.f) * static_cast<float>(em) * 0x1p-9f;
  return __uint_as_float(sign | ((em + (120u << 3)) << 20));
}

template <int ELT>
__global__ __launch_bounds__(256) void grouped_gemm_generic_kernel(const GemmParams p) {
  __shared__ int32_t s_row_off[kMaxExperts + 1];
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < p.nexperts; ++e) {
      s_row_off[e] = acc;
      const int v = p.splits[e];
      acc += v > 0 ? v : 0;
    }
    s_row_off[p.nexperts] = acc;
  }
  __syncthreads();
  const int total_rows = s_row_off[p.nexperts] < p.max_rows ? s_row_off[p.nexperts] : p.max_rows;
  float scalar = p.scalar;
  if (p.scalar_dev) scalar *= p.scalar_dev[0];
  const int ncol_blocks = (p.n + 255) / 256;
  for (int64_t item = blockIdx.x; item < static_cast<int64_t>(total_rows) * ncol_blocks;
       item += gridDim.x) {
    const int r = static_cast<int>(item / ncol_blocks);
    const int n = static_cast<int>(item % ncol_blocks) * 256 + threadIdx.x;
    int e = 0;
    while (r >= s_row_off[e + 1]) ++e;
    if (n >= p.n) continue;
    int64_t arow = r;
    if (p.gather_a) {
      arow = p.gather_a[r];
      if (p.a_rows > 0) arow = arow < 0 ? 0 : (arow >= p.a_rows ? p.a_rows - 1 : arow);
    }
    const uint8_t *ap = p.a + arow * p.k * ELT;
    const uint8_t *bp = p.b + (static_cast<int64_t>(e) * p.n + n) * p.k * ELT;
    float acc = 0.f;
    for (int kk = 0; kk < p.k; ++kk) {
      float av, bv;
      if (ELT == 2) {
        av = bf16_bits_to_float(reinterpret_cast<const uint16_t *>(ap)[kk]);
        bv = bf16_bits_to_float(reinterpret_cast<const uint16_t *>(bp)[kk]);
      } else {
        av = e4m3_to_float(ap[kk]);
        bv = e4m3_to_float(bp[kk]);
      }
      acc = fmaf(av, bv, acc);
    }
    float v = acc * scalar * (p.alpha ? p.alpha[e] : 1.f) * (p.row_scale ? p.row_scale[r] : 1.f);
    if (p.col_scale) v *= p.col_scale[static_cast<int64_t>(e) * p.n + n];
    int64_t drow = r;
    if (p.scatter_d) {
      drow = p.scatter_d[r];
      if (drow < 0 || drow >= p.max_rows) continue;
    }
    if (p.d_fp32) static_cast<float *>(p.d)[drow * p.n + n] = v;
    else static_cast<uint16_t *>(p.d)[drow * p.n + n] = float_to_bf16_bits(v);
  }
}

bool mfma_path_ok(const fluxmi_grouped_gemm_args *a) {
  const int elt = a->dtype == FLUXMI_BF16 ? 2 : 1;
  const int64_t kbytes = static_cast<int64_t>(a->k) * elt;
  return kbytes % KBYTES == 0 && kbytes >= KBYTES && a->n % 4 == 0 && aligned16(a->a) &&
         aligned16(a->b) && (reinterpret_cast<uintptr_t>(a->d) & (a->d_fp32 ? 15u : 7u)) == 0 &&
         (a->col_scale == nullptr || aligned16(a->col_scale));
}

template <int NBMAX>
constexpr size_t mfma_lds_bytes() {
  return static_cast<size_t>(TileCfg<NBMAX>::STAGES) * TileCfg<NBMAX>::STAGE_BYTES;
}

// Macro tile width: 384 columns (bf16 only) unless padding N up to a multiple of 384 wastes clearly
// more work than padding it to a multiple of 256.  FLUXMI_GEMM_TILE_N=256|384 overrides.
int pick_nbmax(const fluxmi_grouped_gemm_args *a) {
  if (a->dtype != FLUXMI_BF16) return 2;
  if (const char *env = getenv("FLUXMI_GEMM_TILE_N")) {
    if (atoi(env) == 256) return 2;
    if (atoi(env) == 384) return 3;
  }
  const int64_t pad2 = (static_cast<int64_t>(a->n) + 255) / 256 * 256;
  const int64_t pad3 = (static_cast<int64_t>(a->n) + 383) / 384 * 384;
  return pad3 * 100 <= pad2 * 104 ? 3 : 2;
}

template <int ELT, int NBMAX>
int launch_mfma(const GemmParams &p, int grid, hipStream_t s) {
  static std::atomic<uint64_t> lds_done{0};
  const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(grouped_gemm_mfma_kernel<ELT, NBMAX>), 160 * 1024,
                                    lds_done);
  if (rc != FLUXMI_OK) return rc;
  hipLaunchKernelGGL((grouped_gemm_mfma_kernel<ELT, NBMAX>), dim3(grid), dim3(NTHREADS), mfma_lds_bytes<NBMAX>(), s, p);
  return FLUXMI_OK;
}

}  // namespace
}  // namespace fluxmi

extern "C" size_t fluxmi_grouped_gemm_workspace_bytes(const fluxmi_grouped_gemm_args *) { return 0; }

extern "C" int fluxmi_grouped_gemm(const fluxmi_grouped_gemm_args *args, void *, size_t, void *stream) {
  using namespace fluxmi;
  FLUXMI_REQUIRE(args != nullptr, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: null args");
  FLUXMI_REQUIRE(args->dtype == FLUXMI_BF16 || args->dtype == FLUXMI_FP8_E4M3, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm: unknown dtype %d", args->dtype);
  FLUXMI_REQUIRE(args->d_fp32 == 0 || args->d_fp32 == 1, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm: d_fp32 must be 0 or 1");
  FLUXMI_REQUIRE(args->a_rows >= 0, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: negative a_rows");
  FLUXMI_REQUIRE(args->nexperts >= 1 && args->nexperts <= kMaxExperts, FLUXMI_ERR_UNSUPPORTED,
                 "grouped_gemm: nexperts=%d outside [1,%d]", args->nexperts, kMaxExperts);
  FLUXMI_REQUIRE(args->max_rows >= 0 && args->n >= 0 && args->k >= 0, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm: negative size (max_rows=%d, n=%d, k=%d)", args->max_rows, args->n,
                 args->k);
  if (args->max_rows == 0 || args->n == 0) return FLUXMI_OK;
  FLUXMI_REQUIRE(args->k >= 1, FLUXMI_ERR_UNSUPPORTED, "grouped_gemm: k must be positive");
  FLUXMI_REQUIRE(args->a && args->b && args->d && args->splits, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm: null a / b / d / splits");

  GemmParams p;
  p.a = static_cast<const uint8_t *>(args->a);
  p.b = static_cast<const uint8_t *>(args->b);
  p.d = args->d;
  p.splits = args->splits;
  p.gather_a = args->gather_a;
  p.scatter_d = args->scatter_d;
  p.alpha = args->alpha;
  p.row_scale = args->row_scale;
  p.col_scale = args->col_scale;
  p.scalar_dev = args->scalar_scale_dev;
  p.scalar = args->scalar_scale;
  p.nexperts = args->nexperts;
  p.max_rows = args->max_rows;
  p.a_rows = args->a_rows;
  p.n = args->n;
  p.k = args->k;
  p.d_fp32 = args->d_fp32;

  hipStream_t s = static_cast<hipStream_t>(stream);
  const int cus = fluxmi_device_cu_count();
  FLUXMI_REQUIRE(cus > 0, FLUXMI_ERR_HIP, "grouped_gemm: cannot query the device");

  if (mfma_path_ok(args)) {
    const int nbmax = pick_nbmax(args);
    // Upper bound of the tile count: never launch more workgroups than tiles.
    const int64_t tiles_n = (args->n + 128 * nbmax - 1) / (128 * nbmax);
    const int64_t max_tiles = (static_cast<int64_t>(args->max_rows) / BM + args->nexperts) * tiles_n;
    const int grid = static_cast<int>(max_tiles < cus ? max_tiles : cus);
    int rc;
    if (args->dtype == FLUXMI_BF16) rc = nbmax == 3 ? launch_mfma<2, 3>(p, grid, s) : launch_mfma<2, 2>(p, grid, s);
    else rc = launch_mfma<1, 2>(p, grid, s);
    if (rc != FLUXMI_OK) return rc;
  } else {
    const int grid = cus * 8;
    if (args->dtype == FLUXMI_BF16)
      hipLaunchKernelGGL(grouped_gemm_generic_kernel<2>, dim3(grid), dim3(256), 0, s, p);
    else
      hipLaunchKernelGGL(grouped_gemm_generic_kernel<1>, dim3(grid), dim3(256), 0, s, p);
  }
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}
