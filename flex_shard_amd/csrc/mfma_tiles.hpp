// Shared pieces of the MFMA tile kernels (bf16 Newton-Schulz GEMM, FP8
// blockwise GEMM): launch parameters, the XCD-aware workgroup -> tile order,
// the LDS-staged epilogue, and the global->LDS load helpers.
#pragma once
#include "common.hpp"

#include <atomic>
#include <type_traits>

namespace fsh {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct GemmParams {
  const uint16_t* A;
  const uint16_t* B;
  const uint16_t* D;
  uint16_t* C;
  uint16_t* Ct;
  int64_t M, N, K;
  int64_t lda, ldb, ldd, ldc, ldct;
  int64_t sA, sB, sD, sC, sCt;
  float alpha, beta;
  float diag_add;         // added to C[i][i] before the rounding
  int32_t tiles_m, tiles_n;
  int32_t symmetric;      // only tiles with tm <= tn are computed; the others are mirrored
  int32_t k_major;        // A is [K, M] and B is [K, N]: the product is A^T B (large-tile kernel only)
  int32_t tiles_per_matrix;
  int64_t work_items;     // tiles_per_matrix * batch
  int64_t items_per_xcd;  // ceil(work_items / 8); the grid has 8 * items_per_xcd workgroups
  // Muon update fused into the epilogue (large-tile kernel only).  When
  // update_ptrs is not null, C and D are ignored: matrix b of the batch is the
  // separately allocated parameter at update_ptrs[b] (row stride ldc), and the
  // epilogue stores  p = bf16(bf16(p * decay) + neg_lr * d),  d = bf16(acc)
  // (d scaled by dir_scale and rounded first when that is not 1): the
  // product itself is never written.
  const int64_t* update_ptrs;
  float update_decay, update_neg_lr, update_dir_scale;
#ifdef FSH_TRACE
  uint64_t* trace;
#endif
};
#ifdef FSH_TRACE
#define FSH_STAMP(slot) do { if (p.trace && threadIdx.x == 0) p.trace[blockIdx.x * 16 + (slot)] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define FSH_STAMP(slot) do {} while (0)
#endif

// Several problems served by one launch of the large-tile kernel: problem i
// owns the workgroup ids [first_workgroup[i], first_workgroup[i+1]), each run
// a multiple of 8 long so that the id -> XCD mapping is the same for all.
// Workgroups are dispatched in id order, so the host lists the problem with
// the longest tiles first and the short ones fill the tail of the long ones.
constexpr int kMaxGemmProblems = 4;
struct GemmLaunch {
  GemmParams problem[kMaxGemmProblems];
  int32_t first_workgroup[kMaxGemmProblems];  // INT32_MAX past the last problem
  int32_t total_workgroups;
};

constexpr int kXcds = 8;         // accelerator dies, each with its own L2
constexpr int kGroupTilesM = 4;  // tile rows walked together

// Tile t of a (non-symmetric) matrix in the patch order described below.
__device__ inline void tile_in_order(const GemmParams& p, int t, int* tm, int* tn) {
  const int group_span = kGroupTilesM * p.tiles_n;
  const int first_m = (t / group_span) * kGroupTilesM;
  const int rows = min(p.tiles_m - first_m, kGroupTilesM);
  const int within = t % group_span;
  *tm = first_m + within % rows;
  *tn = within / rows;
}

// Workgroup id -> (batch, tile row, tile column).  Workgroups are handed to
// the 8 XCDs round-robin by id, and an XCD holds 32 of the large-tile
// workgroups at a time (one per CU), so XCD x is given the contiguous run
// [x, x+1) * items_per_xcd of an ordering in which 32 neighbours form a 4 x 8
// patch of tiles of one matrix: its L2 then serves 12 distinct operand panels
// per k-tile instead of 33.  Returns false for the padding ids at the end of
// an XCD's run.
__device__ inline bool tile_of_workgroup(const GemmParams& p, int64_t id, int64_t* batch, int* tm, int* tn) {
  const int64_t slot = id / kXcds;
  const int64_t item = (id % kXcds) * p.items_per_xcd + slot;
  if (item >= p.work_items) return false;
  const int tiles = p.tiles_per_matrix;
  *batch = item / tiles;
  int t = static_cast<int>(item % tiles);
  if (p.symmetric) {
    // Upper triangle row by row: row r holds columns r .. tiles_n-1.  One
    // matrix's triangle (36 tiles of a 2048^2 result) is about what an XCD
    // holds at a time, and it needs only the 8 row panels of the operand.
    int r = 0;
    for (int len = p.tiles_n; t >= len; --len) {
      t -= len;
      ++r;
    }
    *tm = r;
    *tn = r + t;
    return true;
  }
  tile_in_order(p, t, tm, tn);
  return true;
}

// Epilogue of the whole-tile kernels, staged through LDS (free once the last
// k-tile's barrier has passed; every wave uses a private region, but the
// phases are still separated by workgroup barriers).
//
// The accumulate is issued as mfma(B, A), so accumulator r of block (i, j)
// belongs to output row m = lane%32 and column n = 8*(r/4) + 4*(lane/32) + r%4
// of the block.  In that layout a store instruction would touch 32 rows with
// 16 bytes each, and the transposed output would leave as 2-byte stores.
// Instead:
//   1. D is loaded row-wise (16 bytes per lane) into the staging region; the
//      finals = bf16(alpha*acc + beta*D) are computed in registers and written
//      to LDS as [row][col], each over the D value it used;
//   2. the wave reads its region back row-wise and stores C as 16 bytes per
//      lane, 256 contiguous bytes per row;
//   3. for a transposed (or mirrored) output the finals are read back in
//      accumulator layout, written again as [col][row] and leave the same way.
// The LDS row pitch is the row plus 8 bytes: 8-byte writes of 16 lanes then
// cover all 32 banks, and so do the row-wise 8-byte reads of a half-wave.
template <typename Cfg>
struct WholeTileEpilogue {
  static constexpr int kPitch = Cfg::kWaveN * 2 + 8;   // bytes, [row][col] staging
  static constexpr int kPitchT = Cfg::kWaveM * 2 + 8;  // bytes, [col][row] staging
  static constexpr int kRegion =
      (Cfg::kWaveM * kPitch > Cfg::kWaveN * kPitchT) ? Cfg::kWaveM * kPitch : Cfg::kWaveN * kPitchT;
  static constexpr int kLdsBytes = Cfg::WM * Cfg::WN * kRegion;
};

// Values that are the same in every lane but that the compiler cannot prove
// so: moved to scalar registers.
__device__ __forceinline__ int uniform_i32(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v & 0xFFFFFFFFLL)));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v >> 32)));
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}
template <typename T>
__device__ __forceinline__ T* uniform_ptr(T* ptr) {
  return reinterpret_cast<T*>(uniform_i64(reinterpret_cast<int64_t>(ptr)));
}

// Stores a [rows][row_bytes] bf16 image held in LDS (pitch bytes apart) to
// global rows `ld` elements apart, 16 bytes per lane.  `dst` is the same in
// every lane: each store is a scalar base (advanced per pass) plus one 32-bit
// lane offset, so the passes share a single address register.
template <int kRows, int kRowBytes, int kPitch>
__device__ inline void store_staged_rows(const uint8_t* region, uint16_t* dst, int64_t ld, int lane) {
  constexpr int kLanesPerRow = kRowBytes / 16;
  constexpr int kRowsPerPass = 64 / kLanesPerRow;
  static_assert(kRowBytes % 16 == 0 && 64 % kLanesPerRow == 0 && kRows % kRowsPerPass == 0, "staged store shape");
  const int r0 = lane / kLanesPerRow, chunk = lane % kLanesPerRow;
  const uint32_t lane_off = static_cast<uint32_t>(r0) * static_cast<uint32_t>(ld * 2) + chunk * 16;
  uint8_t* base = uniform_ptr(reinterpret_cast<uint8_t*>(dst));
  const int64_t pass_bytes = uniform_i64(static_cast<int64_t>(kRowsPerPass) * ld * 2);
#pragma unroll
  for (int pass = 0; pass < kRows / kRowsPerPass; ++pass) {
    const int r = pass * kRowsPerPass + r0;
    const uint8_t* src = region + r * kPitch + chunk * 16;
    const u32x2 lo = *reinterpret_cast<const u32x2*>(src);
    const u32x2 hi = *reinterpret_cast<const u32x2*>(src + 8);
    *reinterpret_cast<u32x4*>(base + pass * pass_bytes + lane_off) = u32x4{lo.x, lo.y, hi.x, hi.y};
  }
}

// Two floats -> packed bf16 pair (low half = first), round to nearest even:
// one v_cvt_pk_bf16_f32 on gfx950.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Half of a wave's D tile (its upper or lower kWaveM/2 rows), loaded the way
// C leaves: 16 bytes per lane, 256 contiguous bytes per row (in accumulator
// layout a load instruction would touch 32 rows with 16 bytes each).  Both
// halves are requested when the epilogue starts; the lower one lands while
// the upper one is being used.  (Requesting a half before the last k-tile
// was tried: with 256 accumulators live the extra 64 registers spill.)
template <typename Cfg>
struct DRows {
  static constexpr int kLanesPerRow = Cfg::kWaveN * 2 / 16, kRowsPerPass = 64 / kLanesPerRow;
  static constexpr int kPasses = Cfg::kWaveM / 2 / kRowsPerPass;
  u32x4 t[kPasses];
};

// `d` is matrix `batch` of D (row stride ldd elements).
template <typename Cfg>
__device__ __forceinline__ void load_d_rows_from(const uint16_t* d, int64_t ldd, int64_t m0, int64_t n0, int wm, int wn,
                                                 int lane, int half, DRows<Cfg>& rows) {
  using R = DRows<Cfg>;
  const int r0 = lane / R::kLanesPerRow, chunk = lane % R::kLanesPerRow;
  const uint32_t lane_off = static_cast<uint32_t>(r0) * static_cast<uint32_t>(ldd * 2) + chunk * 16;
  const uint8_t* base = uniform_ptr(reinterpret_cast<const uint8_t*>(
      d + (m0 + wm * Cfg::kWaveM + half * (Cfg::kWaveM / 2)) * ldd + n0 + wn * Cfg::kWaveN));
  const int64_t pass_bytes = uniform_i64(static_cast<int64_t>(R::kRowsPerPass) * ldd * 2);
#pragma unroll
  for (int q = 0; q < R::kPasses; ++q) rows.t[q] = *reinterpret_cast<const u32x4*>(base + q * pass_bytes + lane_off);
}

template <typename Cfg>
__device__ __forceinline__ void load_d_rows(const GemmParams& p, int64_t batch, int64_t m0, int64_t n0, int wm, int wn,
                                            int lane, int half, DRows<Cfg>& rows) {
  load_d_rows_from<Cfg>(p.D + batch * p.sD, p.ldd, m0, n0, wm, wn, lane, half, rows);
}

template <typename Cfg, int kPitch>
__device__ __forceinline__ void stage_d_rows(uint8_t* region, int lane, int half, const DRows<Cfg>& rows) {
  using R = DRows<Cfg>;
  const int r0 = half * (Cfg::kWaveM / 2) + lane / R::kLanesPerRow, chunk = lane % R::kLanesPerRow;
  uint8_t* ddst = region + r0 * kPitch + chunk * 16;
#pragma unroll
  for (int q = 0; q < R::kPasses; ++q) {
    uint8_t* d = ddst + q * R::kRowsPerPass * kPitch;
    *reinterpret_cast<u32x2*>(d) = u32x2{rows.t[q].x, rows.t[q].y};
    *reinterpret_cast<u32x2*>(d + 8) = u32x2{rows.t[q].z, rows.t[q].w};
  }
}

template <typename Cfg>
__device__ inline void store_whole_tile(const GemmParams& p, int64_t batch, int64_t m0, int64_t n0, int wm, int wn,
                                        int lane, bool mirror, const f32x16 (&acc)[Cfg::TM][Cfg::TN],
                                        uint8_t* lds) {
  using Epi = WholeTileEpilogue<Cfg>;
  constexpr int TM = Cfg::TM, TN = Cfg::TN;
  static_assert(TM % 2 == 0, "the D tile is handled in two halves of TM/2 blocks");
  const bool has_d = p.D != nullptr;
  uint16_t* C = p.C + batch * p.sC;
  // A symmetric product mirrors its off-diagonal tiles into the lower triangle.
  uint16_t* Ct = mirror ? C : (p.Ct ? p.Ct + batch * p.sCt : nullptr);
  const int64_t ldct = mirror ? p.ldc : p.ldct;
  const int64_t wave_row = m0 + wm * Cfg::kWaveM, wave_col = n0 + wn * Cfg::kWaveN;
  uint8_t* region = lds + (wm * Cfg::WN + wn) * Epi::kRegion;
  const int r_lane = lane & 31, h = lane >> 5;

  // D goes to the wave's staging region row-wise and is read back in
  // accumulator layout; each final then replaces the D value it used.
  DRows<Cfg> upper, lower;
  if (has_d) {
    load_d_rows<Cfg>(p, batch, m0, n0, wm, wn, lane, 0, upper);
    load_d_rows<Cfg>(p, batch, m0, n0, wm, wn, lane, 1, lower);
    stage_d_rows<Cfg, Epi::kPitch>(region, lane, 0, upper);
  }
  FSH_STAMP(8);

  // finals = bf16(fma(beta, D, alpha*acc)): one rounding of the scaled
  // accumulator, one of the sum, as a BLAS epilogue does.
  const bool unit_alpha = p.alpha == 1.0f;
  // Block tiles and wave sub-tiles are square, so C's diagonal runs through
  // the (i, i) blocks of the diagonal sub-tiles of the diagonal tiles.
  const bool on_diagonal = p.diag_add != 0.0f && m0 == n0 && wm == wn;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (has_d && i == TM / 2) stage_d_rows<Cfg, Epi::kPitch>(region, lane, 1, lower);
    // All of a 32-row block's D reads are issued before its first write: the
    // compiler cannot move a read above a write to the same region.
    u32x2 dv[TN][4];
    if (has_d) {
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          dv[j][b] = *reinterpret_cast<const u32x2*>(region + (i * 32 + r_lane) * Epi::kPitch +
                                                     (j * 32 + 8 * b + 4 * h) * 2);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        float v[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) v[t] = unit_alpha ? acc[i][j][4 * b + t] : p.alpha * acc[i][j][4 * b + t];
        if (has_d) {
          v[0] = __builtin_fmaf(p.beta, u32_as_f32(dv[j][b].x << 16), v[0]);
          v[1] = __builtin_fmaf(p.beta, u32_as_f32(dv[j][b].x & 0xFFFF0000u), v[1]);
          v[2] = __builtin_fmaf(p.beta, u32_as_f32(dv[j][b].y << 16), v[2]);
          v[3] = __builtin_fmaf(p.beta, u32_as_f32(dv[j][b].y & 0xFFFF0000u), v[3]);
        }
        if (on_diagonal && i == j) {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (r_lane == 8 * b + 4 * h + t) v[t] += p.diag_add;
        }
        *reinterpret_cast<u32x2*>(region + (i * 32 + r_lane) * Epi::kPitch + (j * 32 + 8 * b + 4 * h) * 2) =
            u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
      }
  }
  FSH_STAMP(9);
  __syncthreads();
  store_staged_rows<Cfg::kWaveM, Cfg::kWaveN * 2, Epi::kPitch>(region, C + wave_row * p.ldc + wave_col, p.ldc, lane);
  FSH_STAMP(10);
  if (Ct == nullptr) return;  // uniform over the workgroup
  __syncthreads();
  FSH_STAMP(11);
  // The finals come back from the [row][col] image in accumulator layout
  // (all reads before the first write: the transposed image reuses the
  // region) and are written again as [col][row].
  u32x2 fin[TM][TN][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int b = 0; b < 4; ++b)
        fin[i][j][b] = *reinterpret_cast<const u32x2*>(region + (i * 32 + r_lane) * Epi::kPitch +
                                                       (j * 32 + 8 * b + 4 * h) * 2);
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t pair = (t >> 1) ? fin[i][j][b].y : fin[i][j][b].x;
          *reinterpret_cast<uint16_t*>(region + (j * 32 + 8 * b + 4 * h + t) * Epi::kPitchT + (i * 32 + r_lane) * 2) =
              static_cast<uint16_t>((t & 1) ? (pair >> 16) : pair);
        }
  FSH_STAMP(12);
  __syncthreads();
  store_staged_rows<Cfg::kWaveN, Cfg::kWaveM * 2, Epi::kPitchT>(region, Ct + wave_col * ldct + wave_row, ldct, lane);
}

// Orders the LDS traffic of one wave: lanes exchange data through the wave's
// private staging region, which the hardware serves in program order; this
// only keeps the compiler from moving a lane's reads above other lanes'
// writes.  No counter is waited for and no workgroup barrier is taken.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Epilogue of the large-tile kernel: the same steps as store_whole_tile, but
// on the upper and then the lower 64 rows of the wave's 128x128 sub-tile, in a
// staging region of 17 KB per wave that only the wave itself touches.  The
// region then fits beside one k-loop stage, which leaves the other stage free
// to receive the next tile's first operands while this runs, and no step
// needs a workgroup barrier (whose memory fence would wait for those loads).
template <typename Cfg>
struct HalfTileEpilogue {
  static constexpr int kRows = Cfg::kWaveM / 2;                 // 64
  static constexpr int kPitch = Cfg::kWaveN * 2 + 8;            // [row][col] image
  static constexpr int kPitchT = kRows * 2 + 8;                 // [col][row] image
  static constexpr int kRegion =
      (kRows * kPitch > Cfg::kWaveN * kPitchT) ? kRows * kPitch : Cfg::kWaveN * kPitchT;
  static constexpr int kLdsBytes = Cfg::WM * Cfg::WN * kRegion;
};

// kMode fixes the flags that every final depends on, so that the 256 finals
// of a lane are straight-line code (with the flags read at run time the
// compiler keeps a branch per group of four finals, and the waits at every
// join serialize the epilogue):
//   kEpiGeneric  any combination, flags read at run time
//   kEpiPlain    C = bf16(acc): no D, no diagonal term, alpha == 1
//   kEpiPoly     C = bf16(fma(beta, D, alpha * acc) + diag): D, alpha and the diagonal term
//   kEpiUpdate   Muon update of separately allocated parameters (see GemmParams::update_ptrs)
constexpr int kEpiGeneric = 0, kEpiPlain = 1, kEpiPoly = 2, kEpiUpdate = 3;

// (Always inlined: as a real call the accumulators and the launch's problem
// table would have to live in scratch memory.)
template <typename Cfg, int kMode>
__device__ __forceinline__ void store_tile_in_halves_as(const GemmParams& p, int64_t batch, int64_t m0, int64_t n0, int wm,
                                               int wn, int lane, bool mirror, const f32x16 (&acc)[Cfg::TM][Cfg::TN],
                                               uint8_t* staging) {
  using Epi = HalfTileEpilogue<Cfg>;
  using R = DRows<Cfg>;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, HM = TM / 2;
  static_assert(TM % 2 == 0 && Epi::kRows == HM * 32, "two halves of whole 32-row blocks");
  const bool has_d = kMode == kEpiPlain ? false : (kMode == kEpiPoly || kMode == kEpiUpdate) ? true : p.D != nullptr;
  // (a pointer loaded from a table is a per-lane value to the compiler: said to be uniform here)
  uint16_t* C = kMode == kEpiUpdate ? reinterpret_cast<uint16_t*>(uniform_i64(p.update_ptrs[batch])) : p.C + batch * p.sC;
  const uint16_t* D = kMode == kEpiUpdate ? C : p.D + batch * p.sD;
  const int64_t ldd = kMode == kEpiUpdate ? p.ldc : p.ldd;
  // A symmetric product mirrors its off-diagonal tiles into the lower triangle.
  uint16_t* Ct = mirror ? C : (p.Ct ? p.Ct + batch * p.sCt : nullptr);
  const int64_t ldct = mirror ? p.ldc : p.ldct;
  const int64_t wave_row = m0 + wm * Cfg::kWaveM, wave_col = n0 + wn * Cfg::kWaveN;
  uint8_t* region = staging + (wm * Cfg::WN + wn) * Epi::kRegion;
  const int r_lane = lane & 31, h = lane >> 5;
  const bool unit_alpha = (kMode == kEpiPlain || kMode == kEpiUpdate) ? true : kMode == kEpiPoly ? false : p.alpha == 1.0f;
  // Block tiles and wave sub-tiles are square, so C's diagonal runs through
  // the (i, i) blocks of the diagonal sub-tiles of the diagonal tiles.
  const bool on_diagonal = kMode != kEpiPlain && kMode != kEpiUpdate && p.diag_add != 0.0f && m0 == n0 && wm == wn;

  // The lower half of D is requested once the upper half has left its
  // registers for LDS, and lands while the upper half is worked on.
  DRows<Cfg> drows[2];
  if (has_d) load_d_rows_from<Cfg>(D, ldd, m0, n0, wm, wn, lane, 0, drows[0]);
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    if (has_d) {
      // stage_d_rows with the half's rows at the top of the region
      const int r0 = lane / R::kLanesPerRow, chunk = lane % R::kLanesPerRow;
#pragma unroll
      for (int q = 0; q < R::kPasses; ++q) {
        uint8_t* d = region + (r0 + q * R::kRowsPerPass) * Epi::kPitch + chunk * 16;
        *reinterpret_cast<u32x2*>(d) = u32x2{drows[hf].t[q].x, drows[hf].t[q].y};
        *reinterpret_cast<u32x2*>(d + 8) = u32x2{drows[hf].t[q].z, drows[hf].t[q].w};
      }
      if (hf == 0) load_d_rows_from<Cfg>(D, ldd, m0, n0, wm, wn, lane, 1, drows[1]);
      wave_lds_sync();
    }
#pragma unroll
    for (int ih = 0; ih < HM; ++ih) {
      u32x2 fin[TN][4];  // packed bf16 finals of this 32-row block, accumulator layout
      const int i = hf * HM + ih;
      u32x2 dv[TN][4];
      if (has_d) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int b = 0; b < 4; ++b)
            dv[j][b] = *reinterpret_cast<const u32x2*>(region + (ih * 32 + r_lane) * Epi::kPitch +
                                                       (j * 32 + 8 * b + 4 * h) * 2);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          float v[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) v[t] = unit_alpha ? acc[i][j][4 * b + t] : p.alpha * acc[i][j][4 * b + t];
          if (kMode == kEpiUpdate) {
            // The rounding sequence of the separate update kernel: direction
            // to bf16 (scaled and rounded again when the scale is not 1),
            // decayed parameter to bf16, then one multiply and one add.
            const uint32_t d01 = pack_bf16x2(v[0], v[1]), d23 = pack_bf16x2(v[2], v[3]);
            float d[4] = {u32_as_f32(d01 << 16), u32_as_f32(d01 & 0xFFFF0000u), u32_as_f32(d23 << 16),
                          u32_as_f32(d23 & 0xFFFF0000u)};
            if (p.update_dir_scale != 1.0f) {
              const uint32_t s01 = pack_bf16x2(d[0] * p.update_dir_scale, d[1] * p.update_dir_scale);
              const uint32_t s23 = pack_bf16x2(d[2] * p.update_dir_scale, d[3] * p.update_dir_scale);
              d[0] = u32_as_f32(s01 << 16); d[1] = u32_as_f32(s01 & 0xFFFF0000u);
              d[2] = u32_as_f32(s23 << 16); d[3] = u32_as_f32(s23 & 0xFFFF0000u);
            }
            const uint32_t p01 = pack_bf16x2(u32_as_f32(dv[j][b].x << 16) * p.update_decay,
                                             u32_as_f32(dv[j][b].x & 0xFFFF0000u) * p.update_decay);
            const uint32_t p23 = pack_bf16x2(u32_as_f32(dv[j][b].y << 16) * p.update_decay,
                                             u32_as_f32(dv[j][b].y & 0xFFFF0000u) * p.update_decay);
            v[0] = u32_as_f32(p01 << 16) + p.update_neg_lr * d[0];
            v[1] = u32_as_f32(p01 & 0xFFFF0000u) + p.update_neg_lr * d[1];
            v[2] = u32_as_f32(p23 << 16) + p.update_neg_lr * d[2];
            v[3] = u32_as_f32(p23 & 0xFFFF0000u) + p.update_neg_lr * d[3];
          } else if (has_d) {
            v[0] = __builtin_fmaf(p.beta, u32_as_f32(dv[j][b].x << 16), v[0]);
            v[1] = __builtin_fmaf(p.beta, u32_as_f32(dv[j][b].x & 0xFFFF0000u), v[1]);
            v[2] = __builtin_fmaf(p.beta, u32_as_f32(dv[j][b].y << 16), v[2]);
            v[3] = __builtin_fmaf(p.beta, u32_as_f32(dv[j][b].y & 0xFFFF0000u), v[3]);
          }
          if (kMode != kEpiPlain && kMode != kEpiUpdate && i == j) {
            // a select per final rather than a branch per block (adding zero
            // elsewhere would turn a -0 into +0)
#pragma unroll
            for (int t = 0; t < 4; ++t) v[t] = (on_diagonal && r_lane == 8 * b + 4 * h + t) ? v[t] + p.diag_add : v[t];
          }
          fin[j][b] = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        }
      // A lane's finals replace exactly the D values it read itself.
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          *reinterpret_cast<u32x2*>(region + (ih * 32 + r_lane) * Epi::kPitch + (j * 32 + 8 * b + 4 * h) * 2) =
              fin[j][b];
    }
    if (hf == 1) FSH_STAMP(9);
    wave_lds_sync();
    store_staged_rows<Epi::kRows, Cfg::kWaveN * 2, Epi::kPitch>(
        region, C + (wave_row + hf * Epi::kRows) * p.ldc + wave_col, p.ldc, lane);
    if (hf == 1) FSH_STAMP(10);
    if (Ct != nullptr) {  // uniform over the workgroup
      // The finals come back in accumulator layout (every read before the
      // first write: the transposed image reuses the region).
      u32x2 fin[HM][TN][4];
#pragma unroll
      for (int ih = 0; ih < HM; ++ih)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int b = 0; b < 4; ++b)
            fin[ih][j][b] = *reinterpret_cast<const u32x2*>(region + (ih * 32 + r_lane) * Epi::kPitch +
                                                            (j * 32 + 8 * b + 4 * h) * 2);
      wave_lds_sync();  // these reads and the row reads are done before the region is reused
#pragma unroll
      for (int ih = 0; ih < HM; ++ih)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const uint32_t pair = (t >> 1) ? fin[ih][j][b].y : fin[ih][j][b].x;
              *reinterpret_cast<uint16_t*>(region + (j * 32 + 8 * b + 4 * h + t) * Epi::kPitchT +
                                           (ih * 32 + r_lane) * 2) =
                  static_cast<uint16_t>((t & 1) ? (pair >> 16) : pair);
            }
      if (hf == 1) FSH_STAMP(12);
      wave_lds_sync();
      store_staged_rows<Cfg::kWaveN, Epi::kRows * 2, Epi::kPitchT>(
          region, Ct + wave_col * ldct + wave_row + hf * Epi::kRows, ldct, lane);
    }
    if (hf == 0) FSH_STAMP(8);
    if (hf == 0) wave_lds_sync();  // before the lower half overwrites the region
  }
}

template <typename Cfg>
__device__ __forceinline__ void store_tile_in_halves(const GemmParams& p, int64_t batch, int64_t m0, int64_t n0, int wm, int wn,
                                            int lane, bool mirror, const f32x16 (&acc)[Cfg::TM][Cfg::TN],
                                            uint8_t* staging) {
  // uniform over the launch's problem, so one branch per tile
  const bool has_d = p.D != nullptr, diag = p.diag_add != 0.0f, unit_alpha = p.alpha == 1.0f;
  if (p.update_ptrs != nullptr)
    store_tile_in_halves_as<Cfg, kEpiUpdate>(p, batch, m0, n0, wm, wn, lane, mirror, acc, staging);
  else if (!has_d && !diag && unit_alpha)
    store_tile_in_halves_as<Cfg, kEpiPlain>(p, batch, m0, n0, wm, wn, lane, mirror, acc, staging);
  else if (has_d && !unit_alpha)
    store_tile_in_halves_as<Cfg, kEpiPoly>(p, batch, m0, n0, wm, wn, lane, mirror, acc, staging);
  else
    store_tile_in_halves_as<Cfg, kEpiGeneric>(p, batch, m0, n0, wm, wn, lane, mirror, acc, staging);
}

// Scheduling-group masks of __builtin_amdgcn_sched_group_barrier.
constexpr int kSchedValu = 0x002, kSchedMfma = 0x008, kSchedVmemRead = 0x020, kSchedDsRead = 0x100, kSchedDsWrite = 0x200;

// gfx950 loads 16 bytes per lane from global memory straight into LDS: lane l
// of a wave writes LDS bytes [M0 + 16 l, M0 + 16 l + 16).  The address is a
// uniform 64-bit base plus a 32-bit per-lane offset.  Inline asm: the compiler
// neither reorders these against other memory operations nor counts them.
__device__ inline void dma_load_16(uint32_t voffset, const uint8_t* base, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voffset), "s"(base), "s"(lds_addr) : "memory");
}
__device__ inline void wait_for_dma_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// The 4-byte form: lane l writes LDS bytes [M0 + 4 l, M0 + 4 l + 4).
__device__ inline void dma_touch_4(uint32_t voffset, const uint8_t* base, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" ::"v"(voffset), "s"(base), "s"(lds_addr) : "memory");
}

constexpr int max_int(int a, int b) { return a > b ? a : b; }

template <typename Kernel>
int reserve_lds(Kernel kernel, int bytes) {
  if (bytes <= 64 * 1024) return FSH_OK;
  hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (err != hipSuccess) return fail(FSH_EHIP, "gemm: cannot reserve %d bytes of LDS: %s", bytes, hipGetErrorString(err));
  return FSH_OK;
}


// Compute units of the current device (0 when the query fails).
inline int64_t compute_units() {
  static int cached[64] = {0};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
  if (cached[device] == 0) {
    int count = 0;
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    cached[device] = count;
  }
  return cached[device];
}

// The attribute is per device and function, and sticky: it is set once per
// device and kernel, whichever host thread gets there first (setting it
// twice is harmless).
struct LdsReservation {
  std::atomic<uint64_t> devices{0};
};
template <typename Kernel>
int reserve_lds_once(LdsReservation& done, Kernel kernel, int bytes) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) device = 0;
  const uint64_t bit = (device >= 0 && device < 64) ? (1ull << device) : 0;
  if (bit && (done.devices.load(std::memory_order_acquire) & bit)) return FSH_OK;
  if (int rc = reserve_lds(kernel, bytes)) return rc;
  if (bit) done.devices.fetch_or(bit, std::memory_order_release);
  return FSH_OK;
}

}  // namespace
}  // namespace fsh
