// Newton-Schulz orthogonalization for Muon on gfx950 matrix cores.
//
// Everything is built from one batched "NT" GEMM, C = bf16(alpha*A*B^T +
// beta*D) with both operands k-contiguous, so every MFMA operand is one
// 16-byte LDS read.  To keep all three products of an iteration in that
// form the iterate is carried in both orientations, X [s, l] and X^T [l, s]
// (s <= l):
//   G  = X X^T                 A = X,  B = X
//   P  = b G + c G G           A = G,  B = G   (G symmetric, so G^T = G)
//   X' = a X + P X             A = P,  B = X^T; the epilogue writes X' in
//                              place and X'^T into the other X^T buffer.
// A tall input is its own X^T, so no transpose kernel is needed in either
// case, and the result lands in the caller's buffer without a copy.
//
// GEMM kernels: 256 threads (2x2 wavefronts) on v_mfma_f32_32x32x16_bf16, in
// two tile configurations (256x256x64 for large problems, 128x128x32 when
// there are too few tiles to fill the chip) and two bodies: a predicated one
// for any shape, and a predicate-free, software-pipelined one for problems
// whose dimensions are multiples of the tile.  Global->register->LDS double
// buffering with one barrier per k-tile; LDS rows padded by 16 bytes so the
// 64 lanes of a ds_read_b128 hit distinct banks.
#include "mfma_tiles.hpp"
#include "muon_elementwise.hpp"

namespace fsh {
namespace {

// Tile configuration of one GEMM kernel instantiation.
//   BM x BN block tile, BK k-tile, WM x WN wavefronts, each wave owns a
//   (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA tiles.
template <int BM_, int BN_, int BK_, int WM_, int WN_>
struct GemmCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int kThreads = WM * WN * 64;
  static constexpr int kWaveM = BM / WM, kWaveN = BN / WN;
  static constexpr int TM = kWaveM / 32, TN = kWaveN / 32;
  static constexpr int kLdsStride = BK + 8;  // bf16 per LDS row: 16 bytes of padding
  static constexpr int kStageElems = (BM + BN) * kLdsStride;
  static constexpr int kLdsBytes = 2 * kStageElems * 2;  // double buffered
  static constexpr int kChunksPerRow = BK / 8;
  static constexpr int kChunksA = BM * kChunksPerRow / kThreads;
  static constexpr int kChunksB = BN * kChunksPerRow / kThreads;
  static_assert(BM * kChunksPerRow % kThreads == 0 && BN * kChunksPerRow % kThreads == 0, "chunk split");
};

// Large problems: 256x256x64, four waves of 128x128 (256 fp32 accumulators per
// lane).  Per 16-wide k step a wave issues 8 ds_read_b128 for 16 MFMAs, so LDS
// traffic is half of what 64x64 wave tiles need, and a k-tile lasts ~2000
// cycles, long enough for the next tile's global loads to land.
using BigCfg = GemmCfg<256, 256, 64, 2, 2>;
// Small problems (few tiles): 128x128x32, four waves of 64x64.
using SmallCfg = GemmCfg<128, 128, 32, 2, 2>;

template <typename Cfg>
__global__ __launch_bounds__(Cfg::kThreads) void gemm_nt_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, TM = Cfg::TM, TN = Cfg::TN;
  constexpr int kLdsStride = Cfg::kLdsStride;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  int64_t batch;
  int tm, tn;
  if (!tile_of_workgroup(p, blockIdx.x, &batch, &tm, &tn)) return;  // whole workgroup, before any barrier
  const int64_t m0 = static_cast<int64_t>(tm) * BM;
  const int64_t n0 = static_cast<int64_t>(tn) * BN;

  const uint16_t* A = p.A + batch * p.sA;
  const uint16_t* B = p.B + batch * p.sB;

  // Global -> register staging in 16-byte chunks.
  u32x4 ra[Cfg::kChunksA], rb[Cfg::kChunksB];
  auto load_global = [&](int64_t k0) {
#pragma unroll
    for (int i = 0; i < Cfg::kChunksA; ++i) {
      const int c = tid + i * Cfg::kThreads;
      const int64_t row = m0 + c / Cfg::kChunksPerRow, gk = k0 + (c % Cfg::kChunksPerRow) * 8;
      ra[i] = u32x4{0, 0, 0, 0};
      if (row < p.M && gk < p.K) ra[i] = *reinterpret_cast<const u32x4*>(A + row * p.lda + gk);
    }
#pragma unroll
    for (int i = 0; i < Cfg::kChunksB; ++i) {
      const int c = tid + i * Cfg::kThreads;
      const int64_t row = n0 + c / Cfg::kChunksPerRow, gk = k0 + (c % Cfg::kChunksPerRow) * 8;
      rb[i] = u32x4{0, 0, 0, 0};
      if (row < p.N && gk < p.K) rb[i] = *reinterpret_cast<const u32x4*>(B + row * p.ldb + gk);
    }
  };
  auto store_lds = [&](int buf) {
    uint16_t* base = smem + buf * Cfg::kStageElems;
#pragma unroll
    for (int i = 0; i < Cfg::kChunksA; ++i) {
      const int c = tid + i * Cfg::kThreads;
      *reinterpret_cast<u32x4*>(&base[(c / Cfg::kChunksPerRow) * kLdsStride + (c % Cfg::kChunksPerRow) * 8]) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < Cfg::kChunksB; ++i) {
      const int c = tid + i * Cfg::kThreads;
      *reinterpret_cast<u32x4*>(&base[(BM + c / Cfg::kChunksPerRow) * kLdsStride + (c % Cfg::kChunksPerRow) * 8]) = rb[i];
    }
  };

  // acc[i][j] accumulates (B sub-tile j) x (A sub-tile i)^T, i.e. the
  // transposed 32x32 block: a lane then owns one output row (m) and runs of
  // four consecutive columns (n), which makes the epilogue's C stores 8 bytes
  // wide.
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;
  const int64_t ktiles = (p.K + BK - 1) / BK;

  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int64_t kt = 0; kt < ktiles; ++kt) {
    const int buf = static_cast<int>(kt & 1);
    if (kt + 1 < ktiles) load_global((kt + 1) * BK);
    const uint16_t* As = smem + buf * Cfg::kStageElems;
    const uint16_t* Bs = As + BM * kLdsStride;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const bf16x8*>(
            &As[(wm * Cfg::kWaveM + i * 32 + frag_row) * kLdsStride + ks * 16 + frag_k]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bf[j] = *reinterpret_cast<const bf16x8*>(
            &Bs[(wn * Cfg::kWaveN + j * 32 + frag_row) * kLdsStride + ks * 16 + frag_k]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[j], af[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < ktiles) store_lds(buf ^ 1);
    __syncthreads();
  }

  // Epilogue.  Accumulator r of block (i, j) belongs to output row
  // m = lane%32 and column n = 8*(r/4) + 4*(lane/32) + r%4 of the block.
  const uint16_t* D = p.D ? p.D + batch * p.sD : nullptr;
  uint16_t* C = p.C + batch * p.sC;
  // A symmetric product mirrors its off-diagonal tiles into the lower triangle.
  const bool mirror = p.symmetric && tm != tn;
  uint16_t* Ct = mirror ? C : (p.Ct ? p.Ct + batch * p.sCt : nullptr);
  const int64_t ldct = mirror ? p.ldc : p.ldct;
  const bool c_vec = (p.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7) == 0);
  const bool d_vec = D != nullptr && (p.ldd % 4 == 0) && ((reinterpret_cast<uintptr_t>(D) & 7) == 0);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int64_t row = m0 + wm * Cfg::kWaveM + i * 32 + (lane & 31);
    if (row >= p.M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int64_t col = n0 + wn * Cfg::kWaveN + j * 32 + 8 * b + 4 * (lane >> 5);
        if (col >= p.N) continue;
        const bool full = col + 3 < p.N;
        float dv[4] = {0.f, 0.f, 0.f, 0.f};
        if (D != nullptr) {
          if (full && d_vec) {
            const u32x2 raw = *reinterpret_cast<const u32x2*>(&D[row * p.ldd + col]);
            dv[0] = u32_as_f32(raw.x << 16);
            dv[1] = u32_as_f32(raw.x & 0xFFFF0000u);
            dv[2] = u32_as_f32(raw.y << 16);
            dv[3] = u32_as_f32(raw.y & 0xFFFF0000u);
          } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
              if (col + t < p.N) dv[t] = bf16_bits_to_f32(D[row * p.ldd + col + t]);
          }
        }
        uint32_t packed[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          float v = p.alpha * acc[i][j][4 * b + t];
          if (D != nullptr) v += p.beta * dv[t];
          if (row == col + t) v += p.diag_add;
          packed[t] = f32_to_bf16_bits(v);
        }
        if (full && c_vec) {
          *reinterpret_cast<u32x2*>(&C[row * p.ldc + col]) =
              u32x2{packed[0] | (packed[1] << 16), packed[2] | (packed[3] << 16)};
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (col + t < p.N) C[row * p.ldc + col + t] = static_cast<uint16_t>(packed[t]);
        }
        if (Ct != nullptr) {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (col + t < p.N) Ct[(col + t) * ldct + row] = static_cast<uint16_t>(packed[t]);
        }
      }
  }
}


// Interior fast path: M, N multiples of the block tile and K of BK, so there
// are no predicates, addresses are one per-thread 32-bit offset plus uniform
// terms, and the k loop is software pipelined by hand.  With 256 accumulators
// a SIMD holds a single wave, so nothing else hides latency: the fragments of
// k step s+1 are read from LDS while the MFMAs of step s issue, the next
// tile's global loads are spread over the first k step, and their LDS writes
// are interleaved with the MFMAs of the last one.
template <typename Cfg>
__global__ __launch_bounds__(Cfg::kThreads) void gemm_nt_interior_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, TM = Cfg::TM, TN = Cfg::TN;
  constexpr int kLdsStride = Cfg::kLdsStride, KS = BK / 16, CPR = Cfg::kChunksPerRow;
  constexpr int kRowsPerPass = Cfg::kThreads / CPR;  // tile rows covered by one chunk pass

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  int64_t batch;
  int tm, tn;
  if (!tile_of_workgroup(p, blockIdx.x, &batch, &tm, &tn)) return;  // whole workgroup, before any barrier
  const int64_t m0 = static_cast<int64_t>(tm) * BM;
  const int64_t n0 = static_cast<int64_t>(tn) * BN;

  // Uniform tile bases and one per-thread byte offset each for A and B.
  const uint8_t* Ab = reinterpret_cast<const uint8_t*>(p.A + batch * p.sA + m0 * p.lda);
  const uint8_t* Bb = reinterpret_cast<const uint8_t*>(p.B + batch * p.sB + n0 * p.ldb);
  const int trow = tid / CPR, tkc = tid % CPR;
  const uint32_t a_toff = static_cast<uint32_t>((trow * p.lda + tkc * 8) * 2);
  const uint32_t b_toff = static_cast<uint32_t>((trow * p.ldb + tkc * 8) * 2);
  const int64_t a_pass = static_cast<int64_t>(kRowsPerPass) * p.lda * 2;
  const int64_t b_pass = static_cast<int64_t>(kRowsPerPass) * p.ldb * 2;
  const int lds_toff = trow * kLdsStride + tkc * 8;  // elements

  u32x4 ra[Cfg::kChunksA], rb[Cfg::kChunksB];
  auto load_global = [&](int64_t kt) {
    const int64_t koff = kt * BK * 2;
#pragma unroll
    for (int i = 0; i < Cfg::kChunksA; ++i)
      ra[i] = *reinterpret_cast<const u32x4*>(Ab + (koff + i * a_pass) + a_toff);
#pragma unroll
    for (int i = 0; i < Cfg::kChunksB; ++i)
      rb[i] = *reinterpret_cast<const u32x4*>(Bb + (koff + i * b_pass) + b_toff);
  };
  auto store_lds = [&](int buf) {
    uint16_t* base = smem + buf * Cfg::kStageElems + lds_toff;
#pragma unroll
    for (int i = 0; i < Cfg::kChunksA; ++i)
      *reinterpret_cast<u32x4*>(&base[i * kRowsPerPass * kLdsStride]) = ra[i];
#pragma unroll
    for (int i = 0; i < Cfg::kChunksB; ++i)
      *reinterpret_cast<u32x4*>(&base[(BM + i * kRowsPerPass) * kLdsStride]) = rb[i];
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int a_frag = (wm * Cfg::kWaveM + (lane & 31)) * kLdsStride + (lane >> 5) * 8;
  const int b_frag = (BM + wn * Cfg::kWaveN + (lane & 31)) * kLdsStride + (lane >> 5) * 8;
  bf16x8 af[2][TM], bf[2][TN];
  auto load_frags = [&](int set, const uint16_t* stage, int ks) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
      af[set][i] = *reinterpret_cast<const bf16x8*>(&stage[a_frag + i * 32 * kLdsStride + ks * 16]);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      bf[set][j] = *reinterpret_cast<const bf16x8*>(&stage[b_frag + j * 32 * kLdsStride + ks * 16]);
  };
  auto mfma_step = [&](int set) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[set][j], af[set][i], acc[i][j], 0, 0, 0);
  };

  const int64_t ktiles = p.K / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  load_frags(0, smem, 0);

  constexpr int kMfmaPerStep = TM * TN;
  constexpr int kFragReads = TM + TN;
  constexpr int kGlobalLoads = Cfg::kChunksA + Cfg::kChunksB;
  // One k-tile.  `more` (a compile-time tag) says whether a next tile exists:
  // the last tile is peeled so that each variant is straight-line code the
  // scheduling hints can reorder freely.
  auto k_tile = [&](int64_t kt, auto more_tag) {
    constexpr bool more = decltype(more_tag)::value;
    const int buf = static_cast<int>(kt & 1);
    const uint16_t* stage = smem + buf * Cfg::kStageElems;
    if (more) load_global(kt + 1);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS) load_frags((ks + 1) & 1, stage, ks + 1);
      if (ks == KS - 1 && more) store_lds(buf ^ 1);
      mfma_step(ks & 1);
      if (ks == 0 && more) {
#pragma unroll
        for (int g = 0; g < kGlobalLoads; ++g) {
          __builtin_amdgcn_sched_group_barrier(kSchedVmemRead, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
          if (g < kFragReads) __builtin_amdgcn_sched_group_barrier(kSchedDsRead, 1, 0);
        }
      } else if (ks + 1 < KS) {
#pragma unroll
        for (int g = 0; g < kFragReads; ++g) {
          __builtin_amdgcn_sched_group_barrier(kSchedDsRead, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kSchedMfma, kMfmaPerStep / kFragReads, 0);
        }
      } else if (more) {
#pragma unroll
        for (int g = 0; g < kGlobalLoads; ++g) {
          __builtin_amdgcn_sched_group_barrier(kSchedDsWrite, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
        }
      }
    }
    __syncthreads();
    if (more) load_frags(0, smem + (buf ^ 1) * Cfg::kStageElems, 0);
  };
  for (int64_t kt = 0; kt + 1 < ktiles; ++kt) k_tile(kt, std::true_type{});
  k_tile(ktiles - 1, std::false_type{});

  store_whole_tile<Cfg>(p, batch, m0, n0, wm, wn, lane, p.symmetric && tm != tn, acc,
                        reinterpret_cast<uint8_t*>(smem));
}

// ---------------------------------------------------------------------------
// Large whole-tile problems: 256x256x64 tiles with global->LDS loads.
//
// gfx950 can load 16 bytes per lane from global memory straight into LDS
// (global_load_lds_dwordx4: lane l of a wave writes LDS bytes
// [M0 + 16 l, M0 + 16 l + 16)), so a k-tile needs no staging registers and
// no ds_write, and the loads of tile t+1 are waited for only at the end of
// tile t.  A wave-level load fills 1 KB of LDS = 8 tile rows of 128 bytes
// with no padding, so bank conflicts are avoided by an XOR swizzle instead:
// the 16-byte chunk c of row r is stored in slot c ^ ((r >> 1) & 7) of its
// row, done on the global side by letting the lane that fills slot s of row r
// fetch chunk s ^ ((r >> 1) & 7).  The LDS has 64 banks of 4 bytes and serves
// a 16-byte-per-lane read sixteen lanes at a time; rows are 128 bytes, so the
// sixteen rows of such a group alternate between the two halves of the bank
// window and, within a half, take eight different slots.  (XOR with r & 7
// spreads only eight lanes and costs a two-way conflict on every fragment
// read: 8 instead of 4 cycles by the bank-conflict counter.)
//
// These loads and their waits are inline asm, which the compiler neither
// reorders nor counts; everything else in the loop is compiler-visible and is
// pinned around them with sched_barrier.
//
// The part does not hold its peak clock under this kernel (1.5-1.6 GHz on
// random operands, 2.3 GHz on zeros, by the shader-clock counter against the
// 100 MHz one).  Cycle counters in the loop put under 5 % of a k-tile into the
// wait for operands and the barrier together; asking for every operand line
// once more, a few k-tiles ahead, to pull it into L2 (4-byte requests into a
// scrap area) made all three products 2-5 % slower and is gone.
struct DmaGemm {
  static constexpr int BM = 256, BN = 256, BK = 64, WM = 2, WN = 2, TM = 4, TN = 4;
  static constexpr int kThreads = 256, kWaveM = 128, kWaveN = 128, KS = BK / 16;
  static constexpr int kRowBytes = BK * 2;                   // 128
  static constexpr int kOperandBytes = BM * kRowBytes;       // 32 KB per operand and stage
  static constexpr int kStageBytes = 2 * kOperandBytes;      // 64 KB
  static constexpr int kLoopLdsBytes = 2 * kStageBytes;
  static constexpr int kLoadsPerOperand = BM / 8 / 4;        // wave-level 1 KB loads per wave: 8
};

// LDS of the kernel: two operand stages, the epilogue's staging region from
// stage 1 upward.
constexpr int kDmaGemmLdsBytes = DmaGemm::kStageBytes + max_int(DmaGemm::kStageBytes, HalfTileEpilogue<DmaGemm>::kLdsBytes);

// kPersistent: the grid is one workgroup per compute unit and workgroup g
// takes the ids g, g + gridDim.x, ... of the launch (the same XCD every time,
// and the 32 workgroups of an XCD stay on 32 neighbouring tiles).  While the
// epilogue of a tile runs, the first operands of the next one are already on
// their way into stage 0.  The schedule is static, so the host uses it only
// when all tiles of the launch are equally long; otherwise each id is its own
// workgroup and the hardware hands them out as compute units come free.
//
// kKMajor: both operands are given k-major, A as [K, M] and B as [K, N] (row
// strides lda / ldb), i.e. the product is A^T B.  A k-tile of an operand is
// then 64 rows of 512 bytes.  It lands in LDS as it is (chunk c of k-row r in
// slot c ^ 4 (r & 3)), and the fragments come out of it through the
// transposing LDS read of gfx950 (ds_read_b64_tr_b16): within 16 lanes, lane
// 4 j + q passes the address of four consecutive columns 4 q .. 4 q + 3 of
// k-row j, and lane t receives column t of k-rows 0 .. 3 -- four consecutive
// k of one output row, half of an MFMA operand.  The products and their order
// are those of the k-contiguous form on the transposed operands, so the
// results are bit-identical.
template <bool kPersistent, bool kKMajor>
__global__ __launch_bounds__(DmaGemm::kThreads) void gemm_nt_dma_kernel(const GemmLaunch launch) {
  using Cfg = DmaGemm;
#ifdef FSH_TRACE
  const GemmParams& p = launch.problem[0];  // the profiling build stamps into the first problem's buffer
#endif
  FSH_STAMP(0);
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds_bytes[];
  constexpr int TM = Cfg::TM, TN = Cfg::TN, KS = Cfg::KS;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;

  // Tile of launch id `id`: problem index, batch, tile row and column (all
  // uniform; moved to scalar registers explicitly).  False for padding ids.
  auto locate = [&](int64_t id, int& which, int64_t& batch, int& tm, int& tn) -> bool {
    int w = 0;
#pragma unroll
    for (int i = 1; i < kMaxGemmProblems; ++i) w += id >= launch.first_workgroup[i] ? 1 : 0;
    w = uniform_i32(w);
    int64_t b;
    int r, c;
    if (!tile_of_workgroup(launch.problem[w], id - launch.first_workgroup[w], &b, &r, &c)) return false;
    which = w;
    batch = uniform_i64(b);
    tm = uniform_i32(r);
    tn = uniform_i32(c);
    return true;
  };

  // Load side.  Wave-level load q (0..7) of this wave fills tile rows
  // [32 q + 8 wave, +8); lane l fills slot l & 7 of row l >> 3 there.
  // (k-major: load q fills k-rows [8 q + 2 wave, +2); lane l fills slot
  // l & 31 of row l >> 5 there.)
  // (The per-lane values of both sides are derived from the lane number again
  // at the start of every tile, see derive_lane_values below.)
  uint32_t fill_row0 = 0;
  int fill_chunk = 0;
  constexpr uint32_t kRowsPerLoadStep = kKMajor ? 8 : 32;
  // M0 takes the LDS byte address relative to the workgroup's allocation.
  typedef __attribute__((address_space(3))) uint8_t* lds_address;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_address)lds_bytes));
  const uint32_t fill_lds = lds_base + static_cast<uint32_t>(wave * 1024);  // + q * 4096 (+ operand, + stage)
  // Operand tile bases of (problem, batch, tile row / column), k-tile 0.
  auto a_base = [&](int which, int64_t batch, int tm) -> const uint8_t* {
    const GemmParams& q = launch.problem[which];
    return uniform_ptr(reinterpret_cast<const uint8_t*>(
        q.A + batch * q.sA + static_cast<int64_t>(tm) * Cfg::BM * (kKMajor ? 1 : q.lda)));
  };
  auto b_base = [&](int which, int64_t batch, int tn) -> const uint8_t* {
    const GemmParams& q = launch.problem[which];
    return uniform_ptr(reinterpret_cast<const uint8_t*>(
        q.B + batch * q.sB + static_cast<int64_t>(tn) * Cfg::BN * (kKMajor ? 1 : q.ldb)));
  };
  auto issue_tile_load = [&](const uint8_t* a_src, const uint8_t* b_src, uint32_t a_row_bytes, uint32_t b_row_bytes,
                             int stage_off, int q_first, int q_last) {
    // The part of the address that depends on q goes into the scalar base, so
    // that one lane offset per operand serves all eight loads.
    const uint32_t a_voff = fill_row0 * a_row_bytes + fill_chunk * 16, b_voff = fill_row0 * b_row_bytes + fill_chunk * 16;
#pragma unroll
    for (int q = q_first; q < q_last; ++q) {
      dma_load_16(a_voff, a_src + static_cast<uint64_t>(kRowsPerLoadStep * q) * a_row_bytes, stage_off + fill_lds + q * 4096);
      dma_load_16(b_voff, b_src + static_cast<uint64_t>(kRowsPerLoadStep * q) * b_row_bytes,
                  stage_off + Cfg::kOperandBytes + fill_lds + q * 4096);
    }
  };

  // Operand pointer of k-tile kt: 128 bytes along the rows, or 64 rows down.
  auto k_tile_ptr = [&](const uint8_t* base, uint32_t row_bytes, int64_t kt) -> const uint8_t* {
    return kKMajor ? base + kt * (static_cast<int64_t>(Cfg::BK) * row_bytes) : base + kt * Cfg::kRowBytes;
  };

  // Fragment side.  Lane l reads row l & 31 of a 32-row block, k chunk
  // 2 ks + (l >> 5); its slot is that chunk XOR ((row >> 1) & 7), i.e. the
  // ks = 0 address with bits 5..6 flipped by ks.
  uint32_t a_frag[KS], b_frag[KS];
  // k-major fragments: lane l = 16 g + t of a wave serves output row
  // 16 (g & 1) + t of a 32-row block and the k octet g >> 1 of a k step; it
  // passes the address of columns 4 (t & 3) .. + 3 of k-row (t >> 2) of its
  // octet's first half, then of its second half (4 rows = 2048 bytes down).
  // The block index enters the slot through the swizzle: i ^ (k-row & 3).
  uint32_t a_frag_km[TM], b_frag_km[TN];
  // All per-lane addresses of the k loop, from the lane number.  Called with
  // a lane number the compiler cannot see through at the start of every tile:
  // the values then live from there to the end of the k loop only.  Kept
  // across the epilogue (which needs every register it can get), the compiler
  // spilled some of them and reloaded them inside the k loop, and a reload is
  // a vector memory load: the wait for it also waited for every operand
  // request in flight.
  auto derive_lane_values = [&](int l) {
    const int fill_row = kKMajor ? l >> 5 : l >> 3;
    fill_row0 = static_cast<uint32_t>((kKMajor ? 2 : 8) * wave + fill_row);
    fill_chunk = kKMajor ? (l & 31) ^ (4 * static_cast<int>(fill_row0 & 3)) : (l & 7) ^ static_cast<int>((fill_row0 >> 1) & 7);
    const int frag_row = l & 31;
    const uint32_t frag_base = static_cast<uint32_t>(frag_row * Cfg::kRowBytes + (((l >> 5) ^ ((frag_row >> 1) & 7)) * 16));
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      a_frag[ks] = (frag_base ^ (ks * 32)) + wm * Cfg::kWaveM * Cfg::kRowBytes;
      b_frag[ks] = (frag_base ^ (ks * 32)) + Cfg::kOperandBytes + wn * Cfg::kWaveN * Cfg::kRowBytes;
    }
    const int t = l & 15, g = l >> 4;
    const uint32_t common = static_cast<uint32_t>(((g >> 1) * 8 + (t >> 2)) * 512 + (g & 1) * 32 + (t & 3) * 8);
#pragma unroll
    for (int i = 0; i < TM; ++i) a_frag_km[i] = common + wm * 256 + ((i ^ (t >> 2)) * 64);
#pragma unroll
    for (int j = 0; j < TN; ++j) b_frag_km[j] = Cfg::kOperandBytes + common + wn * 256 + ((j ^ (t >> 2)) * 64);
  };
  derive_lane_values(lane);

  f32x16 acc[TM][TN];
  bf16x8 af[2][TM], bf[2][TN];
  auto read_transposed = [&](uint32_t offset) -> bf16x8 {
    typedef short i16x4 __attribute__((__vector_size__(4 * sizeof(short))));
    typedef __attribute__((address_space(3))) i16x4* lds_i16x4;
    const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4)(lds_bytes + offset));
    const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4)(lds_bytes + offset + 2048));
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto read_a = [&](int set, int stage_off, int ks, int i) {
    if (kKMajor)
      af[set][i] = read_transposed(stage_off + a_frag_km[i] + ks * 8192);
    else
      af[set][i] = *reinterpret_cast<const bf16x8*>(lds_bytes + stage_off + a_frag[ks] + i * 32 * Cfg::kRowBytes);
  };
  auto read_b = [&](int set, int stage_off, int ks, int j) {
    if (kKMajor)
      bf[set][j] = read_transposed(stage_off + b_frag_km[j] + ks * 8192);
    else
      bf[set][j] = *reinterpret_cast<const bf16x8*>(lds_bytes + stage_off + b_frag[ks] + j * 32 * Cfg::kRowBytes);
  };
  auto read_frags = [&](int set, int stage_off, int ks) {
#pragma unroll
    for (int i = 0; i < TM; ++i) read_a(set, stage_off, ks, i);
#pragma unroll
    for (int j = 0; j < TN; ++j) read_b(set, stage_off, ks, j);
  };
  auto mfma = [&](int set, int i, int j) {
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[set][j], af[set][i], acc[i][j], 0, 0, 0);
  };
  // The first k step of a tile starts its accumulators from a zero operand
  // instead of from 256 cleared registers.
  auto mfma_from_zero = [&](int set, int i, int j) {
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[set][j], af[set][i], zero, 0, 0, 0);
  };

  // Current tile: plain scalars, reassigned per tile.
  int which = 0, tm = 0, tn = 0;
  int64_t batch = 0;
  int64_t id = blockIdx.x;
  const int64_t stride = gridDim.x;
  if (kPersistent) {
    while (id < launch.total_workgroups && !locate(id, which, batch, tm, tn)) id = uniform_i64(id + stride);
    if (id >= launch.total_workgroups) return;  // whole workgroup, before any barrier
  } else if (!locate(id, which, batch, tm, tn)) {
    return;  // whole workgroup, before any barrier
  }
  const uint8_t* Ab = a_base(which, batch, tm);
  const uint8_t* Bb = b_base(which, batch, tn);
  uint32_t a_row_bytes = static_cast<uint32_t>(launch.problem[which].lda * 2);
  uint32_t b_row_bytes = static_cast<uint32_t>(launch.problem[which].ldb * 2);
  FSH_STAMP(1);
  issue_tile_load(Ab, Bb, a_row_bytes, b_row_bytes, 0, 0, Cfg::kLoadsPerOperand);

  // One k-tile, rotated by a quarter: the barrier that hands over the next
  // tile's operands sits before the last k step, so that step's MFMAs cover
  // the first fragment reads of the next tile (otherwise exposed after every
  // barrier) and the requests for the tile after it (the stage they fill was
  // released by the same barrier: every wave holds its last fragments of it
  // in registers).
  //   entering:  set 0 holds the fragments of (kt, k step 0); the operands of
  //              kt + 1 are on their way
  //   k steps 0 .. KS-2: MFMAs while the next step's fragments are read
  //   wait for kt + 1, barrier
  //   k step KS-1: one MFMA, one fragment read of (kt + 1, 0), one pair of
  //              requests for kt + 2 at a time
#ifdef FSH_TRACE
  uint64_t trace_wait = 0, trace_barrier = 0, trace_ktiles = 0, trace_tile_wait = 0, trace_tile_barrier = 0, trace_tiles = 0, trace_kloop = 0, trace_epi = 0, trace_steps = 0, trace_last = 0, trace_mark = 0;
  const uint64_t trace_begin = __builtin_amdgcn_s_memtime();
#endif
  // Requests for a k-tile's operands.  A wave cannot issue anything else
  // while a request waits to be accepted, and with all four waves asking at
  // once each request takes about 80 cycles: cycle counters put the last k
  // step, when it carried all sixteen requests of a wave, at 1250 cycles
  // against 512 of matrix work.  The requests are therefore spread over two k
  // steps, one per two MFMAs: eight behind the barrier that released their
  // stage and eight in the first k step of the next k-tile, which still
  // leaves them two k steps to land.  (Spread over all four k steps, the late
  // ones were waited for.)
  constexpr int kFirstRequests = 8, kSecondRequests = 16 - kFirstRequests;  // 6 / 10, 10 / 6 and 12 / 4 measured the same or slower
  // request idx (0 .. 15) of a k-tile: operand A for even idx, B for odd, wave-level load idx / 2
  auto issue_one = [&](int idx, const uint8_t* a_src, const uint8_t* b_src, int stage) {
    const int q = idx >> 1;
    if (idx & 1)
      dma_load_16(fill_row0 * b_row_bytes + fill_chunk * 16, b_src + static_cast<uint64_t>(kRowsPerLoadStep * q) * b_row_bytes,
                  stage + Cfg::kOperandBytes + fill_lds + q * 4096);
    else
      dma_load_16(fill_row0 * a_row_bytes + fill_chunk * 16, a_src + static_cast<uint64_t>(kRowsPerLoadStep * q) * a_row_bytes,
                  stage + fill_lds + q * 4096);
  };
  auto k_tile = [&](int64_t kt, int64_t ktiles, auto more_tag, auto first_tag) {
    constexpr bool more = decltype(more_tag)::value;
    constexpr bool first = decltype(first_tag)::value;  // k-tile 0 of an output tile
    const int stage_off = static_cast<int>(kt & 1) * Cfg::kStageBytes;
    const int next_off = stage_off ^ Cfg::kStageBytes;
#pragma unroll
    for (int ks = 0; ks + 1 < KS; ++ks) {
      if (ks == 0 && more && !first) {
        // the second eight requests for k-tile kt + 1 (the first eight went out in the last k step of kt - 1)
        const uint8_t* a_cur = k_tile_ptr(Ab, a_row_bytes, kt + 1);
        const uint8_t* b_cur = k_tile_ptr(Bb, b_row_bytes, kt + 1);
#pragma unroll
        for (int g = 0; g < TM * TN; ++g) {
          mfma(0, g / TN, g % TN);
          if (g < TM) read_a(1, stage_off, 1, g);
          else if (g < TM + TN) read_b(1, stage_off, 1, g - TM);
          if ((g + 1) * kSecondRequests / 16 != g * kSecondRequests / 16)
            issue_one(kFirstRequests + g * kSecondRequests / 16, a_cur, b_cur, next_off);
          __builtin_amdgcn_sched_barrier(0);
        }
        continue;
      }
      read_frags((ks + 1) & 1, stage_off, ks + 1);
#pragma unroll
      for (int g = 0; g < TM * TN; ++g) {
        if (first && ks == 0) mfma_from_zero(0, g / TN, g % TN);
        else mfma(ks & 1, g / TN, g % TN);
      }
#pragma unroll
      for (int g = 0; g < TM + TN; ++g) {
        __builtin_amdgcn_sched_group_barrier(kSchedDsRead, kKMajor ? 2 : 1, 0);
        __builtin_amdgcn_sched_group_barrier(kSchedMfma, TM * TN / (TM + TN), 0);
      }
    }
#ifdef FSH_TRACE
    const uint64_t tr0 = __builtin_amdgcn_s_memtime();
    trace_steps += tr0 - trace_mark;
#endif
    if (more) {  // this wave's part of the next tile has landed
      wait_for_dma_loads();
    }
#ifdef FSH_TRACE
    const uint64_t tr1 = __builtin_amdgcn_s_memtime();
#endif
    __syncthreads();
#ifdef FSH_TRACE
    const uint64_t tr2 = __builtin_amdgcn_s_memtime();
    trace_wait += tr1 - tr0;
    trace_barrier += tr2 - tr1;
    trace_ktiles += 1;
#endif
    const bool more2 = more && kt + 2 < ktiles;
    const uint8_t* a_next = k_tile_ptr(Ab, a_row_bytes, kt + 2);
    const uint8_t* b_next = k_tile_ptr(Bb, b_row_bytes, kt + 2);
#pragma unroll
    for (int g = 0; g < TM * TN; ++g) {
      mfma((KS - 1) & 1, g / TN, g % TN);
      if (more) {
        if (g < TM) read_a(0, next_off, 0, g);
        else if (g < TM + TN) read_b(0, next_off, 0, g - TM);
      }
      if (more2 && (g + 1) * kFirstRequests / 16 != g * kFirstRequests / 16)
        issue_one(g * kFirstRequests / 16, a_next, b_next, stage_off);
      __builtin_amdgcn_sched_barrier(0);
    }
#ifdef FSH_TRACE
    trace_mark = __builtin_amdgcn_s_memtime();
    trace_last += trace_mark - tr2;
#endif
  };

  while (true) {
    const GemmParams& p = launch.problem[which];
    const int64_t ktiles = p.K / Cfg::BK;
    {
      int lane_again = lane;
      asm volatile("" : "+v"(lane_again));
      derive_lane_values(lane_again);
    }
    FSH_STAMP(6);
#ifdef FSH_TRACE
    const uint64_t ts0 = __builtin_amdgcn_s_memtime();
#endif
    wait_for_dma_loads();
    FSH_STAMP(7);
#ifdef FSH_TRACE
    const uint64_t ts1 = __builtin_amdgcn_s_memtime();
#endif
    __syncthreads();  // also: every wave has left the previous tile's epilogue
#ifdef FSH_TRACE
    trace_tile_wait += ts1 - ts0;
    trace_tile_barrier += __builtin_amdgcn_s_memtime() - ts1;
    trace_tiles += 1;
    const uint64_t tk0 = __builtin_amdgcn_s_memtime();
    trace_mark = tk0;
#endif
    read_frags(0, 0, 0);
    if (ktiles > 1)
      issue_tile_load(k_tile_ptr(Ab, a_row_bytes, 1), k_tile_ptr(Bb, b_row_bytes, 1), a_row_bytes, b_row_bytes,
                      Cfg::kStageBytes, 0, Cfg::kLoadsPerOperand);
    FSH_STAMP(2);

    if (ktiles > 1) {
      k_tile(0, ktiles, std::true_type{}, std::true_type{});
      for (int64_t kt = 1; kt + 1 < ktiles; ++kt) k_tile(kt, ktiles, std::true_type{}, std::false_type{});
      k_tile(ktiles - 1, ktiles, std::false_type{}, std::false_type{});
    } else {
      k_tile(0, ktiles, std::false_type{}, std::true_type{});
    }
    FSH_STAMP(3);
#ifdef FSH_TRACE
    trace_kloop += __builtin_amdgcn_s_memtime() - tk0;
#endif

    // Both stages are free now.  The next tile's first operands go to stage 0
    // while the epilogue stages its output beside it, from stage 1 upward.
    int next_which = 0, next_tm = 0, next_tn = 0;
    int64_t next_batch = 0;
    bool have_next = false;
    if (kPersistent) {
      id = uniform_i64(id + stride);
      while (id < launch.total_workgroups && !(have_next = locate(id, next_which, next_batch, next_tm, next_tn)))
        id = uniform_i64(id + stride);
      if (have_next) {
        Ab = a_base(next_which, next_batch, next_tm);
        Bb = b_base(next_which, next_batch, next_tn);
        a_row_bytes = static_cast<uint32_t>(launch.problem[next_which].lda * 2);
        b_row_bytes = static_cast<uint32_t>(launch.problem[next_which].ldb * 2);
        issue_tile_load(Ab, Bb, a_row_bytes, b_row_bytes, 0, 0, Cfg::kLoadsPerOperand);
      }
    }
#ifdef FSH_TRACE
    const uint64_t te0 = __builtin_amdgcn_s_memtime();
#endif
    store_tile_in_halves<Cfg>(p, batch, static_cast<int64_t>(tm) * Cfg::BM, static_cast<int64_t>(tn) * Cfg::BN, wm,
                              wn, lane, p.symmetric && tm != tn, acc, lds_bytes + Cfg::kStageBytes);
#ifdef FSH_TRACE
    trace_epi += __builtin_amdgcn_s_memtime() - te0;
#endif
    FSH_STAMP(4);
#if defined(FSH_TRACE) && !defined(FSH_TRACE_NODRAIN)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    FSH_STAMP(5);
#endif
#ifdef FSH_TRACE
    if (!have_next && p.trace && threadIdx.x == 0) {
      p.trace[blockIdx.x * 16 + 12] = __builtin_amdgcn_s_memtime() - trace_begin;
      p.trace[blockIdx.x * 16 + 13] = trace_wait;
      p.trace[blockIdx.x * 16 + 14] = trace_barrier;
      p.trace[blockIdx.x * 16 + 15] = trace_ktiles;
      p.trace[blockIdx.x * 16 + 8] = trace_tile_wait;
      p.trace[blockIdx.x * 16 + 9] = trace_tile_barrier;
      p.trace[blockIdx.x * 16 + 10] = trace_tiles;
      p.trace[blockIdx.x * 16 + 11] = trace_kloop;
      p.trace[blockIdx.x * 16 + 7] = trace_epi;
      p.trace[blockIdx.x * 16 + 5] = trace_steps;
      p.trace[blockIdx.x * 16 + 6] = trace_last;
    }
#endif
    if (!have_next) break;
    which = next_which;
    batch = next_batch;
    tm = next_tm;
    tn = next_tn;
  }
}

// A validated problem with its kernel chosen and its tile schedule filled in.
enum GemmKernelKind { kKernelDma, kKernelInteriorBig, kKernelInteriorSmall, kKernelEdgeBig, kKernelEdgeSmall };
struct PlannedGemm {
  GemmParams p;
  GemmKernelKind kind;
  int64_t workgroups;
};

template <typename Cfg>
int plan_gemm_cfg(PlannedGemm* plan, int64_t batch) {
  GemmParams& p = plan->p;
  p.tiles_m = static_cast<int32_t>(ceil_div(p.M, Cfg::BM));
  p.tiles_n = static_cast<int32_t>(ceil_div(p.N, Cfg::BN));
  const int64_t tiles = p.symmetric ? static_cast<int64_t>(p.tiles_n) * (p.tiles_n + 1) / 2
                                    : static_cast<int64_t>(p.tiles_m) * p.tiles_n;
  p.tiles_per_matrix = static_cast<int32_t>(tiles);
  p.work_items = tiles * batch;
  p.items_per_xcd = ceil_div(p.work_items, static_cast<int64_t>(kXcds));
  if (tiles > 0x3FFFFFFFLL || p.items_per_xcd * kXcds > 0x3FFFFFFFLL)
    return fail(FSH_ENOTSUP, "gemm: too many tiles");
  plan->workgroups = p.items_per_xcd * kXcds;
  constexpr bool big = std::is_same<Cfg, BigCfg>::value;
  // Interior path: whole tiles, 16-byte accesses in the epilogue, 32-bit tile spans.
  const bool interior =
      p.M % Cfg::BM == 0 && p.N % Cfg::BN == 0 && p.K % Cfg::BK == 0 && p.ldc % 8 == 0 &&
      (reinterpret_cast<uintptr_t>(p.C) & 15) == 0 && p.sC % 8 == 0 &&
      (p.Ct == nullptr || (p.ldct % 8 == 0 && (reinterpret_cast<uintptr_t>(p.Ct) & 15) == 0 && p.sCt % 8 == 0)) &&
      (p.D == nullptr || (p.ldd % 8 == 0 && (reinterpret_cast<uintptr_t>(p.D) & 15) == 0 && p.sD % 8 == 0)) &&
      static_cast<int64_t>(Cfg::BM) * p.lda * 2 < (1LL << 31) && static_cast<int64_t>(Cfg::BN) * p.ldb * 2 < (1LL << 31);
  if (interior)
    plan->kind = big ? kKernelDma : kKernelInteriorSmall;
  else
    plan->kind = big ? kKernelEdgeBig : kKernelEdgeSmall;
  if (p.k_major && plan->kind != kKernelDma)
    return fail(FSH_ENOTSUP,
                "gemm: k-major operands need whole 256 x 256 x 64 tiles and at least 192 of them (m %lld, n %lld, "
                "k %lld, batch %lld)", (long long)p.M, (long long)p.N, (long long)p.K, (long long)batch);
  return FSH_OK;
}

// The Muon update an epilogue applies instead of storing its product (see
// GemmParams::update_ptrs); ptrs == nullptr: an ordinary product.
struct GemmUpdate {
  const int64_t* ptrs;
  float decay, neg_lr, dir_scale;
};

int plan_gemm(const fsh_gemm_desc& d, PlannedGemm* plan, const GemmUpdate* update = nullptr) {
  if (d.m <= 0 || d.n <= 0 || d.k <= 0 || d.batch <= 0)
    return fail(FSH_EINVAL, "gemm: non-positive size (m %lld, n %lld, k %lld, batch %lld)", (long long)d.m,
                (long long)d.n, (long long)d.k, (long long)d.batch);
  if (!d.a_dev || !d.b_dev || !d.c_dev) return fail(FSH_EINVAL, "gemm: null operand");
  if (d.k % 8 || d.lda % 8 || d.ldb % 8 || d.stride_a % 8 || d.stride_b % 8 || !aligned(d.a_dev, 16) ||
      !aligned(d.b_dev, 16))
    return fail(FSH_ENOTSUP, "gemm: k, lda, ldb and batch strides must be multiples of 8 and A, B 16-byte aligned");
  // k-contiguous operands have rows of k elements; k-major ones rows of m and of n.
  if (d.lda < (d.k_major ? d.m : d.k) || d.ldb < (d.k_major ? d.n : d.k) || d.ldc < d.n || (d.d_dev && d.ldd < d.n) ||
      (d.ct_dev && d.ldct < d.m))
    return fail(FSH_EINVAL, "gemm: leading dimension smaller than the row length");
  if (d.symmetric && (d.m != d.n || d.ct_dev != nullptr))
    return fail(FSH_EINVAL, "gemm: a symmetric product needs m == n and no transposed output");
  GemmParams& p = plan->p;
  memset(&p, 0, sizeof(p));
  p.symmetric = d.symmetric ? 1 : 0;
  p.k_major = d.k_major ? 1 : 0;
  p.A = static_cast<const uint16_t*>(d.a_dev);
  p.B = static_cast<const uint16_t*>(d.b_dev);
  p.D = static_cast<const uint16_t*>(d.d_dev);
  p.C = static_cast<uint16_t*>(d.c_dev);
  p.Ct = static_cast<uint16_t*>(d.ct_dev);
  p.M = d.m; p.N = d.n; p.K = d.k;
  p.lda = d.lda; p.ldb = d.ldb; p.ldd = d.ldd; p.ldc = d.ldc; p.ldct = d.ldct;
  p.sA = d.stride_a; p.sB = d.stride_b; p.sD = d.stride_d; p.sC = d.stride_c; p.sCt = d.stride_ct;
  p.alpha = d.alpha; p.beta = d.beta;
  p.diag_add = d.diag_add;
  if (update != nullptr && update->ptrs != nullptr) {
    if (d.d_dev != nullptr || d.ct_dev != nullptr || d.symmetric || d.alpha != 1.0f || d.diag_add != 0.0f)
      return fail(FSH_EINVAL, "gemm: a fused update takes a plain product");
    p.update_ptrs = update->ptrs;
    p.update_decay = update->decay;
    p.update_neg_lr = update->neg_lr;
    p.update_dir_scale = update->dir_scale;
  }
#ifdef FSH_TRACE
  if (const char* e = getenv("FSH_GEMM_TRACE")) p.trace = reinterpret_cast<uint64_t*>(strtoull(e, nullptr, 0));
#endif
  // The big tile pays off once it fills the chip at least once.
  const int64_t big_n = ceil_div(d.n, BigCfg::BN);
  const int64_t big_tiles = (d.symmetric ? big_n * (big_n + 1) / 2 : ceil_div(d.m, BigCfg::BM) * big_n) * d.batch;
  const int rc = big_tiles >= 192 ? plan_gemm_cfg<BigCfg>(plan, d.batch) : plan_gemm_cfg<SmallCfg>(plan, d.batch);
  if (rc == FSH_OK && p.update_ptrs != nullptr && plan->kind != kKernelDma)
    return fail(FSH_ENOTSUP, "gemm: only the large-tile kernel applies a fused update");
  return rc;
}

// Whether `d` would run on the large-tile kernel (whose epilogue can apply a fused update).
bool takes_large_tile_kernel(const fsh_gemm_desc& d) {
  PlannedGemm plan;
  return plan_gemm(d, &plan) == FSH_OK && plan.kind == kKernelDma;
}

template <typename Kernel>
int launch_single(Kernel kernel, LdsReservation* reserved, int lds_bytes, int threads, const PlannedGemm& plan,
                  hipStream_t stream, const char* name) {
  if (int rc = reserve_lds_once(*reserved, kernel, lds_bytes)) return rc;
  hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(plan.workgroups)), dim3(threads), lds_bytes, stream, plan.p);
  return check_launch(name);
}

// Launches the planned problems in order.  Runs of problems that take the
// large-tile kernel share launches (up to kMaxGemmProblems each, longest k
// first): the short tiles of one problem then fill the partly empty last
// round of another instead of each launch paying its own tail.  The problems
// of one call must not depend on each other.
int launch_planned(PlannedGemm* plans, int count, hipStream_t stream) {
  static LdsReservation reserved_dma, reserved_persistent, reserved_dma_km, reserved_persistent_km, reserved_small,
      reserved_edge_big, reserved_edge_small;
  constexpr int kDmaLds = kDmaGemmLdsBytes;
  int i = 0;
  while (i < count) {
    if (plans[i].kind != kKernelDma) {
      int rc;
      if (plans[i].kind == kKernelInteriorSmall)
        rc = launch_single(&gemm_nt_interior_kernel<SmallCfg>, &reserved_small,
                           max_int(SmallCfg::kLdsBytes, WholeTileEpilogue<SmallCfg>::kLdsBytes), SmallCfg::kThreads,
                           plans[i], stream, "gemm_nt_interior_kernel");
      else if (plans[i].kind == kKernelEdgeBig)
        rc = launch_single(&gemm_nt_kernel<BigCfg>, &reserved_edge_big, BigCfg::kLdsBytes, BigCfg::kThreads, plans[i],
                           stream, "gemm_nt_kernel");
      else
        rc = launch_single(&gemm_nt_kernel<SmallCfg>, &reserved_edge_small, SmallCfg::kLdsBytes, SmallCfg::kThreads,
                           plans[i], stream, "gemm_nt_kernel");
      if (rc) return rc;
      ++i;
      continue;
    }
    int order[kMaxGemmProblems];
    int n = 0;
    int64_t total = 0;
    const int k_major = plans[i].p.k_major;  // one operand layout per launch
    while (i < count && n < kMaxGemmProblems && plans[i].kind == kKernelDma && plans[i].p.k_major == k_major &&
           total + plans[i].workgroups <= 0x3FFFFFFFLL) {
      total += plans[i].workgroups;
      order[n++] = i++;
    }
    for (int a = 1; a < n; ++a)  // insertion sort, longest k first, stable
      for (int b = a; b > 0 && plans[order[b]].p.K > plans[order[b - 1]].p.K; --b) {
        const int t = order[b];
        order[b] = order[b - 1];
        order[b - 1] = t;
      }
    GemmLaunch launch;
    memset(&launch, 0, sizeof(launch));
    int64_t first = 0;
    for (int k = 0; k < kMaxGemmProblems; ++k) {
      launch.first_workgroup[k] = k < n ? static_cast<int32_t>(first) : INT32_MAX;
      if (k < n) {
        launch.problem[k] = plans[order[k]].p;
        first += plans[order[k]].workgroups;
      }
    }
    launch.total_workgroups = static_cast<int32_t>(total);
    // Equally long tiles and more of them than compute units: one resident
    // workgroup per compute unit walks a static schedule.
    bool equal_k = true;
    for (int k = 1; k < n; ++k) equal_k = equal_k && plans[order[k]].p.K == plans[order[0]].p.K;
    const int64_t units = compute_units();
    const bool resident = equal_k && units >= kXcds && units % kXcds == 0 && total > units;
    const dim3 grid(static_cast<uint32_t>(resident ? units : total)), block(DmaGemm::kThreads);
    if (resident && k_major) {
      if (int rc = reserve_lds_once(reserved_persistent_km, &gemm_nt_dma_kernel<true, true>, kDmaLds)) return rc;
      hipLaunchKernelGGL((gemm_nt_dma_kernel<true, true>), grid, block, kDmaLds, stream, launch);
    } else if (resident) {
      if (int rc = reserve_lds_once(reserved_persistent, &gemm_nt_dma_kernel<true, false>, kDmaLds)) return rc;
      hipLaunchKernelGGL((gemm_nt_dma_kernel<true, false>), grid, block, kDmaLds, stream, launch);
    } else if (k_major) {
      if (int rc = reserve_lds_once(reserved_dma_km, &gemm_nt_dma_kernel<false, true>, kDmaLds)) return rc;
      hipLaunchKernelGGL((gemm_nt_dma_kernel<false, true>), grid, block, kDmaLds, stream, launch);
    } else {
      if (int rc = reserve_lds_once(reserved_dma, &gemm_nt_dma_kernel<false, false>, kDmaLds)) return rc;
      hipLaunchKernelGGL((gemm_nt_dma_kernel<false, false>), grid, block, kDmaLds, stream, launch);
    }
    if (int rc = check_launch("gemm_nt_dma_kernel")) return rc;
  }
  return FSH_OK;
}

int launch_gemms(const fsh_gemm_desc* descs, int count, hipStream_t stream, const GemmUpdate* updates = nullptr) {
  constexpr int kChunk = 16;
  PlannedGemm plans[kChunk];
  for (int begin = 0; begin < count; begin += kChunk) {
    const int n = count - begin < kChunk ? count - begin : kChunk;
    for (int i = 0; i < n; ++i)
      if (int rc = plan_gemm(descs[begin + i], &plans[i], updates ? &updates[begin + i] : nullptr)) return rc;
    if (int rc = launch_planned(plans, n, stream)) return rc;
  }
  return FSH_OK;
}

// ------------------------------------------------------- Frobenius normalize
constexpr int kNormThreads = 256;
constexpr int kNormBlocksPerMatrix = 64;

// s plus the squares of the eight bf16 values of v, added one after the
// other in element order.
__device__ __forceinline__ float add_squares8(float s, const u32x4 v) {
  const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float lo = u32_as_f32(d[j] << 16), hi = u32_as_f32(d[j] & 0xFFFF0000u);
    s += lo * lo;
    s += hi * hi;
  }
  return s;
}
// The workgroup's total in a fixed order: lanes by the wave reduction, then
// the four waves as (0 + 1) + (2 + 3).  All threads call it.
__device__ __forceinline__ void store_block_partial(float s, float* lds, float* slot) {
  s = wave_sum_f32(s);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) *slot = (lds[0] + lds[1]) + (lds[2] + lds[3]);
}

// partial[b][j] = sum of squares of slice j of matrix b in fp32.  The order
// is fixed: a thread walks its 8-element groups front to back, lanes are
// folded by the wave reduction, waves left to right.  numel is a multiple of
// 8 and every matrix starts 16-byte aligned.
__global__ __launch_bounds__(kNormThreads) void sumsq_partial_kernel(const uint16_t* __restrict__ x,
                                                                    int64_t numel, float* __restrict__ partial) {
  __shared__ float lds[kNormThreads / 64];
  const int64_t b = blockIdx.y;
  const uint16_t* m = x + b * numel;
  const int64_t groups = numel / 8;
  const int64_t per = ceil_div(groups, (int64_t)kNormBlocksPerMatrix);
  const int64_t begin = blockIdx.x * per;
  const int64_t end = (begin + per) < groups ? (begin + per) : groups;
  float s = 0.0f;
  for (int64_t g = begin + threadIdx.x; g < end; g += kNormThreads) s = add_squares8(s, load_stream_u32x4(m + g * 8));
  store_block_partial(s, lds, &partial[b * kNormBlocksPerMatrix + blockIdx.x]);
}

// The momentum step of Muon for a batch of separately allocated matrices,
// fused with the sum of squares of its output: for matrix b (blockIdx.y)
//   m = bf16(lerp(m, g, 1 - mu));  u = nesterov ? bf16(lerp(g, m, mu)) : m
// with u written to slot b of the contiguous batch buffer, and partial[b][j]
// = the sum of squares of slice j of u.  Slices, the walk of a thread through
// its slice and the order of the additions are those of sumsq_partial_kernel
// on the stored u, so the partials are the same bits and the orthogonalization
// that follows need not read u again to find its norm.
struct MuonPrepareBatch {
  const int64_t* momentum_ptrs;  // device table [batch]
  const int64_t* grad_ptrs;      // device table [batch]
  uint16_t* out;                 // [batch, numel]
  float* partial;                // [batch, kNormBlocksPerMatrix]
  int64_t numel;
  float one_minus_mu, mu;
  int32_t nesterov;
};
__global__ __launch_bounds__(kNormThreads) void muon_prepare_sumsq_kernel(const MuonPrepareBatch q) {
  __shared__ float lds[kNormThreads / 64];
  const int64_t b = blockIdx.y;
  uint16_t* mom = reinterpret_cast<uint16_t*>(q.momentum_ptrs[b]);
  const uint16_t* grad = reinterpret_cast<const uint16_t*>(q.grad_ptrs[b]);
  uint16_t* out = q.out + b * q.numel;
  const int64_t groups = q.numel / 8;
  const int64_t per = ceil_div(groups, (int64_t)kNormBlocksPerMatrix);
  const int64_t begin = blockIdx.x * per;
  const int64_t end = (begin + per) < groups ? (begin + per) : groups;
  float s = 0.0f;
  // Four 16-byte groups per pass, all eight loads issued before the first
  // store: the tables give the compiler no aliasing information, so a plain
  // loop would hold every load back behind the previous group's stores.  The
  // squares are still added group by group in walk order.
  constexpr int kUnroll = 4;
  int64_t g = begin + threadIdx.x;
  for (; g + (kUnroll - 1) * kNormThreads < end; g += kUnroll * kNormThreads) {
    u32x4 mraw[kUnroll], graw[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      mraw[k] = load_stream_u32x4(mom + (g + k * kNormThreads) * 8);
      graw[k] = load_stream_u32x4(grad + (g + k * kNormThreads) * 8);
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      float mv[8], gv[8];
      unpack8(mraw[k], mv);
      unpack8(graw[k], gv);
      uint32_t mb[8], ob[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) muon_prepare_one(mv[j], gv[j], q.one_minus_mu, q.mu, q.nesterov, &mb[j], &ob[j]);
      store_stream_u32x4(mom + (g + k * kNormThreads) * 8, pack8(mb));
      const u32x4 u = pack8(ob);
      store_stream_u32x4(out + (g + k * kNormThreads) * 8, u);
      s = add_squares8(s, u);
    }
  }
  for (; g < end; g += kNormThreads) {
    float mv[8], gv[8];
    unpack8(load_stream_u32x4(mom + g * 8), mv);
    unpack8(load_stream_u32x4(grad + g * 8), gv);
    uint32_t mb[8], ob[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) muon_prepare_one(mv[j], gv[j], q.one_minus_mu, q.mu, q.nesterov, &mb[j], &ob[j]);
    store_stream_u32x4(mom + g * 8, pack8(mb));
    const u32x4 u = pack8(ob);
    store_stream_u32x4(out + g * 8, u);
    s = add_squares8(s, u);
  }
  store_block_partial(s, lds, &q.partial[b * kNormBlocksPerMatrix + blockIdx.x]);
}

// The same for fp32 master state: momentum buffers and gradients are fp32,
//   m = lerp(m, g, 1 - mu) (fp32);  u = bf16(nesterov ? lerp(g, m, mu) : m).
__global__ __launch_bounds__(kNormThreads) void muon_prepare_sumsq_f32_kernel(const MuonPrepareBatch q) {
  __shared__ float lds[kNormThreads / 64];
  const int64_t b = blockIdx.y;
  float* mom = reinterpret_cast<float*>(q.momentum_ptrs[b]);
  const float* grad = reinterpret_cast<const float*>(q.grad_ptrs[b]);
  uint16_t* out = q.out + b * q.numel;
  const int64_t groups = q.numel / 8;
  const int64_t per = ceil_div(groups, (int64_t)kNormBlocksPerMatrix);
  const int64_t begin = blockIdx.x * per;
  const int64_t end = (begin + per) < groups ? (begin + per) : groups;
  float s = 0.0f;
  constexpr int kUnroll = 2;  // 2 x (32 + 32) bytes of loads per thread before the first store
  int64_t g = begin + threadIdx.x;
  for (; g + (kUnroll - 1) * kNormThreads < end; g += kUnroll * kNormThreads) {
    float mv[kUnroll][8], gv[kUnroll][8];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      load8_f32(mom + (g + k * kNormThreads) * 8, mv[k]);
      load8_f32(grad + (g + k * kNormThreads) * 8, gv[k]);
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      uint32_t ob[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        muon_prepare_one_f32(mv[k][j], gv[k][j], q.one_minus_mu, q.mu, q.nesterov, &mv[k][j], &ob[j]);
      store8_f32(mom + (g + k * kNormThreads) * 8, mv[k]);
      const u32x4 u = pack8(ob);
      store_stream_u32x4(out + (g + k * kNormThreads) * 8, u);
      s = add_squares8(s, u);
    }
  }
  for (; g < end; g += kNormThreads) {
    float mv[8], gv[8];
    load8_f32(mom + g * 8, mv);
    load8_f32(grad + g * 8, gv);
    uint32_t ob[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) muon_prepare_one_f32(mv[j], gv[j], q.one_minus_mu, q.mu, q.nesterov, &mv[j], &ob[j]);
    store8_f32(mom + g * 8, mv);
    const u32x4 u = pack8(ob);
    store_stream_u32x4(out + g * 8, u);
    s = add_squares8(s, u);
  }
  store_block_partial(s, lds, &q.partial[b * kNormBlocksPerMatrix + blockIdx.x]);
}

// The update of Muon for the same batch: parameter b (a separate allocation)
// takes the direction in slot b of the batch buffer,
//   p = bf16(p * decay);  p = bf16(p + neg_lr * d)   (d first scaled and rounded if scale != 1).
struct MuonApplyBatch {
  const int64_t* param_ptrs;  // device table [batch]
  const uint16_t* direction;  // [batch, numel]
  int64_t numel;
  float decay, neg_lr, dir_scale;
};
__global__ __launch_bounds__(kNormThreads) void muon_apply_batch_kernel(const MuonApplyBatch q) {
  const int64_t b = blockIdx.y;
  uint16_t* param = reinterpret_cast<uint16_t*>(q.param_ptrs[b]);
  const uint16_t* dir = q.direction + b * q.numel;
  const int64_t groups = q.numel / 8;
  // A block owns runs of four consecutive 4 KiB pieces; a thread's four
  // loads of the parameter and of the direction go out before its stores.
  constexpr int kUnroll = 4;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kNormThreads * kUnroll;
  for (int64_t g0 = static_cast<int64_t>(blockIdx.x) * kNormThreads * kUnroll + threadIdx.x; g0 < groups; g0 += stride) {
    u32x4 praw[kUnroll], draw[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int64_t g = g0 + k * kNormThreads;
      if (g < groups) {
        praw[k] = load_stream_u32x4(param + g * 8);
        draw[k] = load_stream_u32x4(dir + g * 8);
      }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int64_t g = g0 + k * kNormThreads;
      if (g < groups) {
        float pv[8], dv[8];
        unpack8(praw[k], pv);
        unpack8(draw[k], dv);
        uint32_t pb[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) pb[j] = muon_apply_one(pv[j], dv[j], q.decay, q.neg_lr, q.dir_scale);
        store_stream_u32x4(param + g * 8, pack8(pb));
      }
    }
  }
}

// The update on fp32 parameters: p = p * decay; p = p + neg_lr * d, d the bf16
// direction (times scale in fp32 if scale != 1).
__global__ __launch_bounds__(kNormThreads) void muon_apply_batch_f32_kernel(const MuonApplyBatch q) {
  const int64_t b = blockIdx.y;
  float* param = reinterpret_cast<float*>(q.param_ptrs[b]);
  const uint16_t* dir = q.direction + b * q.numel;
  const int64_t groups = q.numel / 8;
  constexpr int kUnroll = 2;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kNormThreads * kUnroll;
  for (int64_t g0 = static_cast<int64_t>(blockIdx.x) * kNormThreads * kUnroll + threadIdx.x; g0 < groups; g0 += stride) {
    float pv[kUnroll][8];
    u32x4 draw[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int64_t g = g0 + k * kNormThreads;
      if (g < groups) {
        load8_f32(param + g * 8, pv[k]);
        draw[k] = load_stream_u32x4(dir + g * 8);
      }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int64_t g = g0 + k * kNormThreads;
      if (g < groups) {
        float dv[8];
        unpack8(draw[k], dv);
#pragma unroll
        for (int j = 0; j < 8; ++j) pv[k][j] = muon_apply_one_f32(pv[k][j], dv[j], q.decay, q.neg_lr, q.dir_scale);
        store8_f32(param + g * 8, pv[k]);
      }
    }
  }
}

// Reads matrix b of `in` ([rows, cols]), divides by max(||.||_F, eps) as bf16
// tensor ops would (norm rounded to bf16, fp32 division, bf16 result), and
// writes the result to `out_same` ([rows, cols]) and `out_t` ([cols, rows]);
// either output may be null.
// A workgroup owns a 64x64 tile: 16-byte loads and stores of 8 elements along
// the rows, and for the transposed copy the tile goes through LDS and leaves
// as 16-byte stores of 8 elements along the columns.  rows and cols are
// multiples of 8, so an 8-element group is either whole or absent.
constexpr int kNormTile = 64;
constexpr int kNormPitch = kNormTile + 2;  // u16 per LDS row
__global__ __launch_bounds__(kNormThreads) void normalize_dual_kernel(const uint16_t* __restrict__ in,
                                                                     uint16_t* __restrict__ out_same,
                                                                     uint16_t* __restrict__ out_t, int64_t rows,
                                                                     int64_t cols, const float* __restrict__ partial,
                                                                     float eps_bf16) {
  __shared__ uint16_t tile[kNormTile * kNormPitch];
  const int64_t b = blockIdx.z;
  float total = 0.0f;
  for (int j = 0; j < kNormBlocksPerMatrix; ++j) total += partial[b * kNormBlocksPerMatrix + j];
  float norm = bf16_bits_to_f32(f32_to_bf16_bits(sqrtf(total)));
  norm = norm < eps_bf16 ? eps_bf16 : norm;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * kNormTile, c0 = static_cast<int64_t>(blockIdx.x) * kNormTile;
  const uint16_t* m = in + b * rows * cols;
  uint16_t* o = out_same ? out_same + b * rows * cols : nullptr;
  uint16_t* ot = out_t ? out_t + b * rows * cols : nullptr;
  const int q = threadIdx.x & 7, line = threadIdx.x >> 3;  // 8 groups of 8 elements per line, 32 lines per pass
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int lr = line + 32 * pass;
    const int64_t r = r0 + lr, c = c0 + 8 * q;
    if (r < rows && c < cols) {
      const u32x4 v = load_stream_u32x4(m + r * cols + c);
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};
      uint32_t bits[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        bits[2 * j] = f32_to_bf16_bits(u32_as_f32(d[j] << 16) / norm);
        bits[2 * j + 1] = f32_to_bf16_bits(u32_as_f32(d[j] & 0xFFFF0000u) / norm);
      }
      if (o != nullptr)
        store_stream_u32x4(o + r * cols + c, u32x4{bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16),
                                                     bits[4] | (bits[5] << 16), bits[6] | (bits[7] << 16)});
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *reinterpret_cast<uint32_t*>(&tile[lr * kNormPitch + 8 * q + 2 * j]) = bits[2 * j] | (bits[2 * j + 1] << 16);
    }
  }
  if (ot == nullptr) return;  // the same for the whole workgroup
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int lc = line + 32 * pass;  // tile column = row of the transposed output
    const int64_t c = c0 + lc, r = r0 + 8 * q;
    if (c < cols && r < rows) {
      uint32_t bits[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) bits[j] = tile[(8 * q + j) * kNormPitch + lc];
      store_stream_u32x4(ot + c * rows + r, u32x4{bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16),
                                                    bits[4] | (bits[5] << 16), bits[6] | (bits[7] << 16)});
    }
  }
}

float bf16_round_host(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  memcpy(&f, &u, 4);
  return f;
}

int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

}  // namespace
}  // namespace fsh

FSH_API int fsh_gemm_bf16_nt(const fsh_gemm_desc* desc, void* stream) {
  if (desc == nullptr) return fsh::fail(FSH_EINVAL, "fsh_gemm_bf16_nt: null descriptor");
  return fsh::launch_gemms(desc, 1, static_cast<hipStream_t>(stream));
}

FSH_API int fsh_gemm_bf16_nt_group(const fsh_gemm_desc* descs, int32_t count, void* stream) {
  if (count < 0 || (count > 0 && descs == nullptr))
    return fsh::fail(FSH_EINVAL, "fsh_gemm_bf16_nt_group: bad descriptor list");
  return fsh::launch_gemms(descs, count, static_cast<hipStream_t>(stream));
}

// Workspace layout (bytes, each region 256-aligned):
//   other orientation of the iterate [batch, s*l] bf16
//   second X^T buffer                [batch, s*l] bf16
//   G                                [batch, s*s] bf16
//   P                                [batch, s*s] bf16
//   norm partials                    [batch, 64] fp32
FSH_API int64_t fsh_newton_schulz_workspace_bytes(int64_t batch, int64_t rows, int64_t cols) {
  using namespace fsh;
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  const int64_t s = rows < cols ? rows : cols, l = rows < cols ? cols : rows;
  return 2 * align256(batch * s * l * 2) + 2 * align256(batch * s * s * 2) +
         align256(batch * kNormBlocksPerMatrix * 4);
}

namespace fsh {
namespace {

// One batch of equally shaped matrices on its way through the iteration.
// X is [s, l]; XT[0], XT[1] are the two [l, s] buffers.  The caller's buffer
// is X when the input is wide and XT[0] when it is tall.  The first X^T goes
// to XT[steps % 2] so that the last step leaves X^T in XT[0].
struct NsState {
  int64_t batch, s, l;
  uint16_t* X;
  uint16_t* XT[2];
  uint16_t* G;
  uint16_t* P;
  int cur;
  bool tall;    // the caller's matrix is X^T
  bool single;  // only X^T is carried from step to step (G = X X^T is then computed from its k-major rows)
};

// Workspace offset of the [batch, 64] norm partials.
int64_t ns_partial_offset(int64_t batch, int64_t rows, int64_t cols) {
  const int64_t s = rows < cols ? rows : cols, l = rows < cols ? cols : rows;
  return 2 * align256(batch * s * l * 2) + 2 * align256(batch * s * s * 2);
}

// `partials_ready`: the norm partials of x are in the workspace already (the
// fused momentum kernel wrote them), so x is not read for its norm.
int ns_begin(const fsh_ns_problem& q, int32_t steps, float eps, hipStream_t stream, NsState* st,
             bool partials_ready = false) {
  const int64_t batch = q.batch, rows = q.rows, cols = q.cols;
  if (batch <= 0 || rows <= 0 || cols <= 0)
    return fail(FSH_EINVAL, "newton_schulz: bad sizes (batch %lld, rows %lld, cols %lld)", (long long)batch,
                (long long)rows, (long long)cols);
  if (!q.x_dev || !q.workspace_dev) return fail(FSH_EINVAL, "newton_schulz: null pointer");
  if (rows % 8 || cols % 8)
    return fail(FSH_ENOTSUP, "newton_schulz: rows and cols must be multiples of 8, got %lld x %lld", (long long)rows,
                (long long)cols);
  if (!aligned(q.x_dev, 16) || !aligned(q.workspace_dev, 256))
    return fail(FSH_EINVAL, "newton_schulz: x must be 16-byte and workspace 256-byte aligned");
  if (batch > 65535) return fail(FSH_ENOTSUP, "newton_schulz: batch %lld exceeds 65535", (long long)batch);
  const int64_t need = fsh_newton_schulz_workspace_bytes(batch, rows, cols);
  if (q.workspace_nbytes < need)
    return fail(FSH_EINVAL, "newton_schulz: workspace of %lld bytes, need %lld", (long long)q.workspace_nbytes,
                (long long)need);
  const bool tall = rows > cols;
  const int64_t s = tall ? cols : rows, l = tall ? rows : cols;
  const int64_t sl = s * l, ss = s * s;
  uint8_t* ws = static_cast<uint8_t*>(q.workspace_dev);
  uint16_t* w0 = reinterpret_cast<uint16_t*>(ws);
  uint16_t* w1 = reinterpret_cast<uint16_t*>(ws + align256(batch * sl * 2));
  uint16_t* x = static_cast<uint16_t*>(q.x_dev);
  st->batch = batch;
  st->s = s;
  st->l = l;
  st->G = reinterpret_cast<uint16_t*>(ws + 2 * align256(batch * sl * 2));
  st->P = reinterpret_cast<uint16_t*>(ws + 2 * align256(batch * sl * 2) + align256(batch * ss * 2));
  float* partial = reinterpret_cast<float*>(ws + 2 * align256(batch * sl * 2) + 2 * align256(batch * ss * 2));
  // With whole 256 x 256 x 64 tiles, and enough of them for the large-tile
  // kernel, G = X X^T is computed from X^T as it lies (k-major operands), so
  // X itself is never written: a tall input alternates between the caller's
  // buffer and one workspace buffer, a wide one between the two workspace
  // buffers and its last step writes X' = P X into the caller's buffer.
  st->single = steps > 0 && s % 256 == 0 && l % 64 == 0 && (s / 256) * (s / 256 + 1) / 2 * batch >= 192;
  st->X = tall ? w0 : x;
  st->XT[0] = tall ? x : w0;
  st->XT[1] = (st->single && tall) ? w0 : w1;
  st->cur = steps & 1;
  st->tall = tall;

  if (!partials_ready) {
    hipLaunchKernelGGL(sumsq_partial_kernel, dim3(kNormBlocksPerMatrix, static_cast<uint32_t>(batch)),
                       dim3(kNormThreads), 0, stream, x, rows * cols, partial);
    if (int rc = check_launch("sumsq_partial_kernel")) return rc;
  }
  // Input is [rows, cols]; "same orientation" output is X for a wide input
  // and X^T for a tall one.
  uint16_t* same = tall ? st->XT[st->cur] : st->X;
  uint16_t* transposed = tall ? st->X : st->XT[st->cur];
  if (st->single) (tall ? transposed : same) = nullptr;
  const dim3 grid(static_cast<uint32_t>(ceil_div(cols, (int64_t)kNormTile)),
                  static_cast<uint32_t>(ceil_div(rows, (int64_t)kNormTile)), static_cast<uint32_t>(batch));
  if (grid.y > 65535) return fail(FSH_ENOTSUP, "newton_schulz: more than %d row tiles", 65535 * kNormTile);
  hipLaunchKernelGGL(normalize_dual_kernel, grid, dim3(kNormThreads), 0, stream, x, same, transposed, rows, cols,
                     partial, bf16_round_host(eps));
  return check_launch("normalize_dual_kernel");
}

// The three products of one iteration; `which` = 0: G = X X^T, 1: P = a I +
// b G + c G G (symmetric because G is), 2: X' = P X = a X + (b G + c G G) X,
// also written transposed into the other X^T buffer -- or, when only X^T is
// carried, X'^T = X^T P alone, with G read from the k-major rows of X^T and
// the last step of a wide input written as X' = P X.  Carrying `a` on P's
// diagonal (added in fp32 before P is rounded) spares the last product a
// read of X from HBM per output tile.  The last step of the iteration writes
// only the orientation the caller holds: X' for a wide input, and for a tall
// one X'^T = X^T P (P is symmetric) computed directly.
fsh_gemm_desc ns_product(const NsState& st, int which, float a, float b, float c, bool last_step) {
  const int64_t s = st.s, l = st.l, sl = s * l, ss = s * s;
  fsh_gemm_desc g;
  memset(&g, 0, sizeof(g));
  g.batch = st.batch;
  if (which == 0 && st.single) {
    g.a_dev = st.XT[st.cur]; g.b_dev = st.XT[st.cur]; g.c_dev = st.G;
    g.m = s; g.n = s; g.k = l; g.lda = s; g.ldb = s; g.ldc = s;
    g.stride_a = sl; g.stride_b = sl; g.stride_c = ss;
    g.alpha = 1.0f; g.beta = 0.0f;
    g.symmetric = 1;
    g.k_major = 1;
  } else if (which == 0) {
    g.a_dev = st.X; g.b_dev = st.X; g.c_dev = st.G;
    g.m = s; g.n = s; g.k = l; g.lda = l; g.ldb = l; g.ldc = s;
    g.stride_a = sl; g.stride_b = sl; g.stride_c = ss;
    g.alpha = 1.0f; g.beta = 0.0f;
    g.symmetric = 1;
  } else if (which == 1) {
    g.a_dev = st.G; g.b_dev = st.G; g.d_dev = st.G; g.c_dev = st.P;
    g.m = s; g.n = s; g.k = s; g.lda = s; g.ldb = s; g.ldd = s; g.ldc = s;
    g.stride_a = ss; g.stride_b = ss; g.stride_d = ss; g.stride_c = ss;
    g.alpha = c; g.beta = b;
    g.diag_add = a;
    g.symmetric = 1;
  } else if (st.single ? (st.tall || !last_step) : (last_step && st.tall)) {
    // X'^T = X^T P (P is symmetric), the orientation that is carried
    g.a_dev = st.XT[st.cur]; g.b_dev = st.P; g.c_dev = st.XT[st.cur ^ 1];
    g.m = l; g.n = s; g.k = s; g.lda = s; g.ldb = s; g.ldc = s;
    g.stride_a = sl; g.stride_b = ss; g.stride_c = sl;
    g.alpha = 1.0f; g.beta = 0.0f;
  } else {
    g.a_dev = st.P; g.b_dev = st.XT[st.cur]; g.c_dev = st.X;
    g.ct_dev = (last_step || st.single) ? nullptr : st.XT[st.cur ^ 1];
    g.m = s; g.n = l; g.k = s; g.lda = s; g.ldb = s; g.ldc = l; g.ldct = s;
    g.stride_a = ss; g.stride_b = sl; g.stride_c = sl; g.stride_ct = sl;
    g.alpha = 1.0f; g.beta = 0.0f;
  }
  return g;
}

// The iteration proper for `count` normalized problems.
// `last_updates` (one per problem, or null): the last product of a problem
// whose entry has ptrs set applies that update to the parameters instead of
// writing the orthogonalized matrix to the caller's buffer.
int ns_iterate(NsState* st, int count, float a, float b, float c, int32_t steps, hipStream_t stream,
               const GemmUpdate* last_updates = nullptr) {
  fsh_gemm_desc descs[FSH_MAX_NS_PROBLEMS];
  for (int step = 0; step < steps; ++step) {
    // The same product of every problem goes out together: problems are
    // independent of each other, the three products of one are not.
    for (int which = 0; which < 3; ++which) {
      const bool last = step + 1 == steps;
      for (int i = 0; i < count; ++i) descs[i] = ns_product(st[i], which, a, b, c, last);
      if (int rc = launch_gemms(descs, count, stream, last && which == 2 ? last_updates : nullptr)) return rc;
    }
    for (int i = 0; i < count; ++i) st[i].cur ^= 1;
  }
  // cur == 0 here: for a tall input the result X^T is in the caller's buffer;
  // for a wide input X was updated in place.
  return FSH_OK;
}

}  // namespace
}  // namespace fsh

FSH_API int fsh_newton_schulz_multi(const fsh_ns_problem* problems, int32_t count, float a, float b, float c,
                                    int32_t steps, float eps, void* stream_) {
  using namespace fsh;
  if (count < 0 || count > FSH_MAX_NS_PROBLEMS || (count > 0 && problems == nullptr))
    return fail(FSH_EINVAL, "fsh_newton_schulz_multi: count %d outside [0, %d] or null list", count,
                FSH_MAX_NS_PROBLEMS);
  if (steps < 0) return fail(FSH_EINVAL, "fsh_newton_schulz_multi: negative step count %d", steps);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  NsState st[FSH_MAX_NS_PROBLEMS];
  for (int i = 0; i < count; ++i)
    if (int rc = ns_begin(problems[i], steps, eps, stream, &st[i])) return rc;
  return ns_iterate(st, count, a, b, c, steps, stream);
}

FSH_API int fsh_newton_schulz(void* x_dev, int64_t batch, int64_t rows, int64_t cols, float a, float b,
                              float c, int32_t steps, float eps, void* workspace_dev,
                              int64_t workspace_nbytes, void* stream_) {
  fsh_ns_problem q;
  q.x_dev = x_dev;
  q.batch = batch;
  q.rows = rows;
  q.cols = cols;
  q.workspace_dev = workspace_dev;
  q.workspace_nbytes = workspace_nbytes;
  return fsh_newton_schulz_multi(&q, 1, a, b, c, steps, eps, stream_);
}

// One Muon step over whole matrices grouped by shape: momentum (fused with
// the sum of squares), Newton-Schulz over all groups together, update.
FSH_API int fsh_muon_step(const fsh_muon_group* groups, int32_t count, float lerp_weight, float nesterov_weight,
                          int32_t nesterov, float decay_factor, float a, float b, float c, int32_t steps, float eps,
                          void* stream_) {
  using namespace fsh;
  if (count < 0 || count > FSH_MAX_NS_PROBLEMS || (count > 0 && groups == nullptr))
    return fail(FSH_EINVAL, "fsh_muon_step: count %d outside [0, %d] or null list", count, FSH_MAX_NS_PROBLEMS);
  if (steps < 0) return fail(FSH_EINVAL, "fsh_muon_step: negative step count %d", steps);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  fsh_ns_problem problems[FSH_MAX_NS_PROBLEMS];
  for (int i = 0; i < count; ++i) {
    const fsh_muon_group& g = groups[i];
    if (g.batch <= 0 || g.batch > 65535 || g.rows <= 0 || g.cols <= 0 || g.rows % 8 || g.cols % 8)
      return fail(FSH_EINVAL, "fsh_muon_step: group %d has bad sizes (batch %lld, rows %lld, cols %lld; rows and cols "
                  "must be multiples of 8)", i, (long long)g.batch, (long long)g.rows, (long long)g.cols);
    if (!g.param_ptrs_dev || !g.grad_ptrs_dev || !g.momentum_ptrs_dev || !g.batch_dev || !g.workspace_dev)
      return fail(FSH_EINVAL, "fsh_muon_step: group %d has a null pointer", i);
    if (!aligned(g.batch_dev, 16) || !aligned(g.workspace_dev, 256))
      return fail(FSH_EINVAL, "fsh_muon_step: group %d: batch buffer must be 16-byte and workspace 256-byte aligned", i);
    if (g.master_dtype != FSH_DT_BF16 && g.master_dtype != FSH_DT_F32)
      return fail(FSH_EINVAL, "fsh_muon_step: group %d: master_dtype %d is neither FSH_DT_BF16 nor FSH_DT_F32", i,
                  g.master_dtype);
    if (g.workspace_nbytes < fsh_newton_schulz_workspace_bytes(g.batch, g.rows, g.cols))
      return fail(FSH_EINVAL, "fsh_muon_step: group %d: workspace of %lld bytes, need %lld", i,
                  (long long)g.workspace_nbytes, (long long)fsh_newton_schulz_workspace_bytes(g.batch, g.rows, g.cols));
    problems[i].x_dev = g.batch_dev;
    problems[i].batch = g.batch;
    problems[i].rows = g.rows;
    problems[i].cols = g.cols;
    problems[i].workspace_dev = g.workspace_dev;
    problems[i].workspace_nbytes = g.workspace_nbytes;
  }
  for (int i = 0; i < count; ++i) {
    const fsh_muon_group& g = groups[i];
    MuonPrepareBatch q;
    q.momentum_ptrs = g.momentum_ptrs_dev;
    q.grad_ptrs = g.grad_ptrs_dev;
    q.out = static_cast<uint16_t*>(g.batch_dev);
    q.partial = reinterpret_cast<float*>(static_cast<uint8_t*>(g.workspace_dev) +
                                         ns_partial_offset(g.batch, g.rows, g.cols));
    q.numel = g.rows * g.cols;
    q.one_minus_mu = lerp_weight;
    q.mu = nesterov_weight;
    q.nesterov = nesterov;
    if (g.master_dtype == FSH_DT_F32)
      hipLaunchKernelGGL(muon_prepare_sumsq_f32_kernel, dim3(kNormBlocksPerMatrix, static_cast<uint32_t>(g.batch)),
                         dim3(kNormThreads), 0, stream, q);
    else
      hipLaunchKernelGGL(muon_prepare_sumsq_kernel, dim3(kNormBlocksPerMatrix, static_cast<uint32_t>(g.batch)),
                         dim3(kNormThreads), 0, stream, q);
    if (int rc = check_launch("muon_prepare_sumsq_kernel")) return rc;
  }
  NsState st[FSH_MAX_NS_PROBLEMS];
  for (int i = 0; i < count; ++i)
    if (int rc = ns_begin(problems[i], steps, eps, stream, &st[i], /*partials_ready=*/true)) return rc;
  // A group whose last product runs on the large-tile kernel gets its update
  // from that product's epilogue: the direction is never written and read
  // back.  The other groups' directions land in their batch buffers and a
  // separate launch applies them.
  GemmUpdate updates[FSH_MAX_NS_PROBLEMS];
  for (int i = 0; i < count; ++i) {
    // (the epilogue writes bf16 parameters; fp32 masters take the separate launch)
    const bool fused = steps > 0 && groups[i].master_dtype == FSH_DT_BF16 &&
                       takes_large_tile_kernel(ns_product(st[i], 2, a, b, c, true));
    updates[i].ptrs = fused ? groups[i].param_ptrs_dev : nullptr;
    updates[i].decay = decay_factor;
    updates[i].neg_lr = groups[i].neg_adjusted_lr;
    updates[i].dir_scale = groups[i].direction_scale;
  }
  if (int rc = ns_iterate(st, count, a, b, c, steps, stream, updates)) return rc;
  for (int i = 0; i < count; ++i) {
    if (updates[i].ptrs != nullptr) continue;
    const fsh_muon_group& g = groups[i];
    MuonApplyBatch q;
    q.param_ptrs = g.param_ptrs_dev;
    q.direction = static_cast<const uint16_t*>(g.batch_dev);
    q.numel = g.rows * g.cols;
    q.decay = decay_factor;
    q.neg_lr = g.neg_adjusted_lr;
    q.dir_scale = g.direction_scale;
    const int64_t groups8 = q.numel / 8;
    const int64_t blocks = ceil_div(groups8, (int64_t)kNormThreads * 4);  // four 16-byte groups per thread
    const dim3 grid(static_cast<uint32_t>(blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks)),
                    static_cast<uint32_t>(g.batch));
    if (g.master_dtype == FSH_DT_F32)
      hipLaunchKernelGGL(muon_apply_batch_f32_kernel, grid, dim3(kNormThreads), 0, stream, q);
    else
      hipLaunchKernelGGL(muon_apply_batch_kernel, grid, dim3(kNormThreads), 0, stream, q);
    if (int rc = check_launch("muon_apply_batch_kernel")) return rc;
  }
  return FSH_OK;
}

// ------------------------------------------------------------------------
// Allocation-free variant: the workspace is a static device array.
//
// `scratch` is a host-side stand-in for the device array, not a device
// address: each GPU holds its own copy at its own address, resolved once per
// device with hipGetSymbolAddress while that device is current.  Everything
// below uses the resolved pointer, never the array's name.
namespace fsh {
namespace {

static __device__ __align__(256) uint8_t scratch[FSH_NS_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// The current device's copy of `scratch`.
int static_scratch(void** out) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return fail(FSH_EHIP, "fsh_newton_schulz_noalloc: hipGetDevice: %s", hipGetErrorString(err));
  if (device < 0 || device >= kMaxDevices)
    return fail(FSH_ENOTSUP, "fsh_newton_schulz_noalloc: device index %d outside [0, %d)", device, kMaxDevices);
  void* ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr)
      return fail(FSH_EHIP, "fsh_newton_schulz_noalloc: hipGetSymbolAddress(scratch) on device %d: %s", device,
                  hipGetErrorString(err));
    g_scratch_ptr[device].store(ptr, std::memory_order_release);  // every thread resolves the same address
  }
  *out = ptr;
  return FSH_OK;
}

}  // namespace
}  // namespace fsh

FSH_API int fsh_newton_schulz_noalloc(void* x_dev, int64_t batch, int64_t rows, int64_t cols, float a, float b,
                                      float c, int32_t steps, float eps, void* stream_) {
  using namespace fsh;
  if (batch <= 0 || rows <= 0 || cols <= 0)
    return fail(FSH_EINVAL, "fsh_newton_schulz_noalloc: bad sizes (batch %lld, rows %lld, cols %lld)", (long long)batch,
                (long long)rows, (long long)cols);
  // Checked in wide arithmetic before the byte count is formed: a huge request must not wrap around.
  const int64_t s = rows < cols ? rows : cols, l = rows < cols ? cols : rows;
  if (batch > 65535 || l > (1LL << 24) || s * l > FSH_NS_STATIC_SCRATCH_BYTES / 4 / batch)
    return fail(FSH_ENOTSUP,
                "fsh_newton_schulz_noalloc: batch %lld of %lld x %lld exceeds the %lld-byte static scratch; call "
                "fsh_newton_schulz with a workspace of fsh_newton_schulz_workspace_bytes()",
                (long long)batch, (long long)rows, (long long)cols, (long long)FSH_NS_STATIC_SCRATCH_BYTES);
  const int64_t need = fsh_newton_schulz_workspace_bytes(batch, rows, cols);
  if (need > FSH_NS_STATIC_SCRATCH_BYTES)
    return fail(FSH_ENOTSUP,
                "fsh_newton_schulz_noalloc: batch %lld of %lld x %lld needs %lld bytes of scratch, the static scratch "
                "holds %lld; call fsh_newton_schulz with a workspace of that size",
                (long long)batch, (long long)rows, (long long)cols, (long long)need,
                (long long)FSH_NS_STATIC_SCRATCH_BYTES);
  void* ptr = nullptr;
  if (int rc = static_scratch(&ptr)) return rc;
  // Every region of the workspace is written before it is read (norm
  // partials, both iterate buffers, G and P), so nothing has to be cleared
  // between calls.
  return fsh_newton_schulz(x_dev, batch, rows, cols, a, b, c, steps, eps, ptr, FSH_NS_STATIC_SCRATCH_BYTES, stream_);
}

