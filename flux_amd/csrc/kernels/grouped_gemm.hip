// Grouped GEMM over ragged per-expert row counts: D[r,:] = scale(r,:) * A[gather(r),:] @ B[e(r)]^T.
//
// Persistent kernel, one 256-thread workgroup (4 waves, one per SIMD) per CU, macro tile 256 rows x 256
// columns, k-step of 64 bytes per row (32 bf16 or 64 fp8).  Both operand tiles are staged in LDS by
// direct-to-LDS global loads (no register staging) in a ring of five 32 KiB stages; the row gather of A
// is folded into the per-lane global address of those loads.  Each wave owns a 128 x 128 quarter of the
// macro tile (4x4 MFMA blocks of 32x32, 256 fp32 accumulator registers) and runs a software pipeline
// of its own: while the MFMAs of k-step s run on one set of fragment registers, the fragments of step
// s+1 are read from LDS into a second set and the ring fills of steps s+4 / s+5 are issued, all in a
// fixed interleaving (one fragment read per MFMA over the first half of the step, one fill every
// fourth MFMA).  One workgroup barrier per k-step publishes the landed stage.
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
#include <cstdlib>

#include "common.hpp"

namespace fluxmi {
namespace {

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

// Two floats to packed bf16, round to nearest even (one v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// Source of the fills of a k-step past the end of K (odd number of k-steps): both operands read zeros.
__device__ __attribute__((aligned(1024))) const uint8_t g_zero_page[1024] = {};

// MFMA number t of a k-step.  bf16: 2 * MB * NB instructions of 32x32x16, the two 16-element halves of
// the step one after the other.  fp8: MB * NB instructions of 32x32x64 (both 16-byte chunks at once).
template <int ELT, int MB, int NB>
__device__ __forceinline__ void mfma_slot(int t, const i32x4 (&xf)[MB][2], const i32x4 (&wf)[NB][2],
                                          f32x16 (&acc)[MB][NB]) {
  if constexpr (ELT == 2) {
    const int s = t / (MB * NB), i = (t % (MB * NB)) / NB, j = t % NB;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wf[j][s]),
                                                        __builtin_bit_cast(bf16x8, xf[i][s]), acc[i][j], 0, 0, 0);
  } else {
    const int i = t / NB, j = t % NB;
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
  int nk;
  int64_t kbytes;
  float scalar;
};

// Epilogue of one wave: acc (32*MB rows x 32*NB columns, MFMA layout) -> scaled, cast, stored.
// FULL: every row and column of the wave's quarter exists and rows are stored where they are (no
// scatter), so no store is predicated.  OUT_F32 selects the output element type.
template <int MB, int NB, bool FULL, bool OUT_F32>
__device__ __forceinline__ void store_tile(const GemmParams &p, uint8_t *window, const TileCtx &c, int e, int row_base,
                                           int rows_e, int wrow0, int wcol0, const f32x16 (&acc)[MB][NB]) {
  static_assert(MB % 2 == 0, "the window holds two 32-row blocks");
  const int lane = c.lane;
  const int h = lane >> 5;
  const float tile_scale = c.scalar * (p.alpha ? p.alpha[e] : 1.f);
  float rs[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int m = wrow0 + i * 32 + (lane & 31);
    rs[i] = tile_scale * ((p.row_scale && (FULL || m < rows_e)) ? p.row_scale[row_base + m] : 1.f);
  }
  const int rr0 = lane >> 3;  // row of this lane within a group of 8 rows (store phase)
  const int cc = lane & 7;    // its 4-column chunk
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int col = wcol0 + j * 32 + cc * 4;
    float4 cs = make_float4(1.f, 1.f, 1.f, 1.f);
    if (p.col_scale && (FULL || col < p.n))
      cs = *reinterpret_cast<const float4 *>(p.col_scale + static_cast<int64_t>(e) * p.n + col);
#pragma unroll
    for (int ip = 0; ip < MB / 2; ++ip) {
      // write phase: lane holds row (ii*32 + lane%32), columns q*8 + h*4 .. +3 = 16-byte chunk 2q+h
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
        const int i = ip * 2 + ii;
        const int r = ii * 32 + (lane & 31);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 v = make_float4(acc[i][j][4 * q + 0] * rs[i], acc[i][j][4 * q + 1] * rs[i],
                                       acc[i][j][4 * q + 2] * rs[i], acc[i][j][4 * q + 3] * rs[i]);
          *reinterpret_cast<float4 *>(window + r * 128 + (((2 * q + h) ^ ((r >> 1) & 7)) << 4)) = v;
        }
      }
      // store phase: 8 lanes per row, 8 rows per instruction
      float4 v[8];
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int rr = it * 8 + rr0;
        v[it] = *reinterpret_cast<const float4 *>(window + rr * 128 + ((cc ^ ((rr >> 1) & 7)) << 4));
      }
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int m = wrow0 + ip * 64 + it * 8 + rr0;
        int64_t drow = row_base + m;
        if constexpr (!FULL) {
          if (m >= rows_e || col >= p.n) continue;  // n % 4 == 0: a chunk is all in or all out
          if (p.scatter_d) {
            drow = p.scatter_d[row_base + m];
            if (drow < 0 || drow >= p.max_rows) continue;
          }
        }
        const float4 o = make_float4(v[it].x * cs.x, v[it].y * cs.y, v[it].z * cs.z, v[it].w * cs.w);
        if constexpr (OUT_F32) {
          *reinterpret_cast<float4 *>(static_cast<float *>(p.d) + drow * p.n + col) = o;
        } else {
          u32x2 b;
          b[0] = pack_bf16x2(o.x, o.y);
          b[1] = pack_bf16x2(o.z, o.w);
          *reinterpret_cast<u32x2 *>(static_cast<uint16_t *>(p.d) + drow * p.n + col) = b;
        }
      }
    }
  }
}

// One output tile of (64*MB) rows x (64*NB) columns at rows [m0, ..) of expert e, columns [n0, ..).
// (MB, NB) = (4, 4) is the macro tile; (4, 2) and (2, 2) are the 256x128 and 128x128 pieces a tile of
// the last, partly filled round is cut into.  Waves are laid out 2 x 2.
template <int ELT, int MB, int NB>
__device__ __forceinline__ void gemm_tile(const GemmParams &p, uint8_t *smem, const TileCtx &c, int e, int row_base,
                                          int rows_e, int m0, int n0) {
  constexpr int XLOADS = MB;           // direct-to-LDS instructions per wave per stage, X tile
  constexpr int WLOADS = NB;           // same, W tile
  constexpr int LOADS = XLOADS + WLOADS;
  constexpr int NR = LOADS * 2;        // fragment reads per k-step
  constexpr int NM = MB * NB * (ELT == 2 ? 2 : 1);  // MFMAs per k-step
  constexpr int RSPAN = NM / 2;        // MFMA slots over which the fragment reads of a step are spread
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
  const uint8_t *zsrc = g_zero_page + lane * 16;

  // Fill instruction q (X rows first, then W rows) of k-step `kstep` into ring slot `slot`.  A k-step
  // past the end of K is clamped to the last one (never consumed) or, if it is the phantom second half
  // of the last pair of an odd K, filled with zeros.
  auto fill_one = [&](int slot, int kstep, int q) {
    uint8_t *stage = smem + slot * STAGE_BYTES;
    const bool zero = kstep == nk;
    const int64_t koff = static_cast<int64_t>(kstep < nk ? kstep : nk - 1) * KBYTES;
    if (q < XLOADS) load_to_lds16(zero ? zsrc : xsrc[q] + koff, stage + (XLOADS * wave + q) * 1024);
    else load_to_lds16(zero ? zsrc : wsrc[q - XLOADS] + koff, stage + X_TILE_BYTES + (WLOADS * wave + (q - XLOADS)) * 1024);
  };

  f32x16 acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  i32x4 xa[MB][2], wa[NB][2], xb[MB][2], wb[NB][2];
  // Fragment read r of a k-step: chunk s = r / LOADS of W block q (q < NB) or X block q - NB.
  auto read_one = [&](const uint8_t *stage, int r, i32x4 (&xf)[MB][2], i32x4 (&wf)[NB][2]) {
    const int s = r / LOADS, q = r % LOADS;
    if (q < NB) wf[q][s] = *reinterpret_cast<const i32x4 *>(stage + w_frag_base + q * 32 * KBYTES + c.frag_off[s]);
    else xf[q - NB][s] = *reinterpret_cast<const i32x4 *>(stage + x_frag_base + (q - NB) * 32 * KBYTES + c.frag_off[s]);
  };

  // Ring slots: k-step s lives in slot s % 5.  `rslot` is the slot of the step whose fragments are read
  // next, `fslot` the slot the next requested step goes to.
  int rslot = 0, fslot = 0;
  auto next_slot = [](int s) { return s + 1 == STAGES ? 0 : s + 1; };

  // One k-step `ks`: MFMAs on `cur` (read during the previous step), fragments of step ks+1 into `nxt`,
  // and half of the fills of the pair of steps (e+4, e+5), e = ks rounded down to even: that pair is
  // requested over the two steps e and e+1, X/W row group by row group, both k-steps of a row group
  // back to back.
  int pslot0 = 0, pslot1 = 0;
  auto step = [&](int ks, bool even, i32x4 (&xc)[MB][2], i32x4 (&wc)[NB][2], i32x4 (&xn)[MB][2], i32x4 (&wn_)[NB][2]) {
    // Stage ks+1 has landed once the pair it belongs to is complete; fills are counted in issue order.
    if (even) {
      FLUXMI_WAITCNT(2 * LOADS, 15);  // all but the pair requested during steps ks-2, ks-1
    } else {
      FLUXMI_WAITCNT(LOADS, 15);      // all but the half pair requested during step ks-1
    }
    __builtin_amdgcn_s_barrier();     // ... for every wave's share; and everybody is done reading stage ks
    __builtin_amdgcn_sched_barrier(0);
    const uint8_t *rstage = smem + rslot * STAGE_BYTES;
    rslot = next_slot(rslot);
    if (even) {
      pslot0 = fslot;
      pslot1 = next_slot(fslot);
      fslot = next_slot(pslot1);
    }
    const int e0 = even ? ks : ks - 1;
#pragma unroll
    for (int t = 0; t < NM; ++t) {
#pragma unroll
      for (int r = 0; r < NR; ++r)
        if (r * RSPAN / NR == t) read_one(rstage, r, xn, wn_);
#pragma unroll
      for (int d = 0; d < 2 * LOADS; ++d)
        if ((d * (2 * NM) / (2 * LOADS) + 1) % (2 * NM) == t + (even ? 0 : NM))
          fill_one((d & 1) ? pslot1 : pslot0, e0 + 4 + (d & 1), d >> 1);
      mfma_slot<ELT, MB, NB>(t, xc, wc, acc);
      __builtin_amdgcn_sched_barrier(0);
    }
    FLUXMI_WAITCNT(63, 0);  // the fragments of the next step are in registers (requested long ago)
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- prologue: request k-steps 0..3 as two pairs, wait for the first pair ------------------------
  FLUXMI_WAITCNT(0, 0);  // stores of the previous tile's epilogue
#pragma unroll
  for (int s = 0; s < 4; s += 2) {
    const int s0 = fslot, s1 = next_slot(fslot);
    fslot = next_slot(s1);
#pragma unroll
    for (int q = 0; q < LOADS; ++q) {
      fill_one(s0, s, q);
      fill_one(s1, s + 1, q);
    }
  }
  FLUXMI_WAITCNT(2 * LOADS, 15);
  __builtin_amdgcn_s_barrier();
  {
    const uint8_t *stage = smem + rslot * STAGE_BYTES;
    rslot = next_slot(rslot);
#pragma unroll
    for (int r = 0; r < NR; ++r) read_one(stage, r, xa, wa);
  }
  FLUXMI_WAITCNT(63, 0);  // in registers before the first step's barrier lets anyone refill that slot
  // An odd number of k-steps runs one phantom step on zero fragments.
  for (int ks = 0; ks < nk; ks += 2) {
    step(ks, true, xa, wa, xb, wb);
    step(ks + 1, false, xb, wb, xa, wa);
  }

  // ---- epilogue ---------------------------------------------------------------------------------
  FLUXMI_WAITCNT(0, 0);          // this wave's trailing ring fills have landed
  __builtin_amdgcn_s_barrier();  // ... and everybody else's; nobody reads the ring any more
  uint8_t *window = smem + wave * 8192;
  const int wrow0 = m0 + wm * (32 * MB);
  const int wcol0 = n0 + wn * (32 * NB);
  const bool full = wrow0 + 32 * MB <= rows_e && wcol0 + 32 * NB <= p.n && p.scatter_d == nullptr;
  if (full) {
    if (p.d_fp32) store_tile<MB, NB, true, true>(p, window, c, e, row_base, rows_e, wrow0, wcol0, acc);
    else store_tile<MB, NB, true, false>(p, window, c, e, row_base, rows_e, wrow0, wcol0, acc);
  } else {
    if (p.d_fp32) store_tile<MB, NB, false, true>(p, window, c, e, row_base, rows_e, wrow0, wcol0, acc);
    else store_tile<MB, NB, false, false>(p, window, c, e, row_base, rows_e, wrow0, wcol0, acc);
  }
  __builtin_amdgcn_s_barrier();  // the LDS windows are free again before the next tile's fills start
}

template <int ELT>
__global__ __launch_bounds__(NTHREADS) void grouped_gemm_mfma_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];  // STAGES x (X tile | W tile)

  TileCtx c;
  const int tid = threadIdx.x;
  c.wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: branches on it stay uniform
  c.lane = tid & 63;
  c.wn = c.wave & 1;   // column half
  c.wm = c.wave >> 1;  // row half
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
  // `pieces` parts (2 pieces of 256x128, or 4 of 128x128) when that still fits one round, so that the
  // chip does not idle while a fraction of the CUs finishes whole tiles.
  const int full_items = (total_tiles / grid) * grid;
  const int rem_tiles = total_tiles - full_items;
  const int pieces = rem_tiles * 4 <= grid ? 4 : (rem_tiles * 2 <= grid ? 2 : 1);
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
      gemm_tile<ELT, 4, 4>(p, smem, c, e, row_base, rows_e, m0, n0);
    } else if (pieces == 2) {
      n0 += piece * 128;
      if (n0 < p.n) gemm_tile<ELT, 4, 2>(p, smem, c, e, row_base, rows_e, m0, n0);
    } else {
      m0 += (piece >> 1) * 128;
      n0 += (piece & 1) * 128;
      if (m0 < rows_e && n0 < p.n) gemm_tile<ELT, 2, 2>(p, smem, c, e, row_base, rows_e, m0, n0);
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

template <int ELT>
int launch_mfma(const GemmParams &p, int grid, hipStream_t s) {
  static std::atomic<uint64_t> lds_done{0};
  const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(grouped_gemm_mfma_kernel<ELT>), LDS_BYTES, lds_done);
  if (rc != FLUXMI_OK) return rc;
  hipLaunchKernelGGL((grouped_gemm_mfma_kernel<ELT>), dim3(grid), dim3(NTHREADS), LDS_BYTES, s, p);
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
    // Upper bound of the tile count: never launch more workgroups than tiles.
    const int64_t tiles_n = (args->n + BN - 1) / BN;
    const int64_t max_tiles = (static_cast<int64_t>(args->max_rows) / BM + args->nexperts) * tiles_n;
    const int grid = static_cast<int>(max_tiles < cus ? max_tiles : cus);
    const int rc = args->dtype == FLUXMI_BF16 ? launch_mfma<2>(p, grid, s) : launch_mfma<1>(p, grid, s);
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
