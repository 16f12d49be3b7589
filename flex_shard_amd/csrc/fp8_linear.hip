// Forward GEMM of a linear layer whose weight arrives already quantized
// (128x128 tiles, FP8 E4M3FN) from the bucket unpack: 1x128 quantization of
// the activation and the FP8 product with both sets of scales.
//
//   xq, xs = quantize each run of 128 consecutive elements of a row of x
//            (amax floored at 1e-12, scale = fp32(448 / fp64(amax)),
//            q = e4m3fn(fp32(x) * scale), stored scale = 1.0f / scale)
//   out[m][n] = bf16( sum over k-blocks kb of
//                     dot(xq[m][kb], wq[n][kb]) * (xs[kb][m] * ws[n / 128][kb]) )
//
// Matrix cores: v_mfma_f32_32x32x64_f8f6f4 (64 FP8 products per lane pair and
// instruction, twice the rate of the 32x32x16 FP8 form on gfx950).  A k-tile
// is one scale block (128 bytes of each row), so its partial products are
// accumulated from zero in a scratch accumulator and folded into the result
// with one fused multiply-add per element; the folds of one 32x32 block run
// on the vector ALU while the matrix core works on the next.
#include "mfma_tiles.hpp"

namespace fsh {
namespace {

// ------------------------------------------------------------ 1x128 quantize
// A workgroup owns 64 rows x 512 columns (4 scale blocks per row).  Sixteen
// lanes own one run of 128 elements (16 bytes each); a wavefront load covers
// four runs = 1 KB of one row.  All sixteen loads of a thread are issued
// before the first is used.  The maximum of a run stays inside its row of 16
// lanes (four DPP steps, no LDS, no barrier).  Scales go through LDS so that
// they leave as 256-byte runs of the [k-block][row] table.
constexpr int kActThreads = 256;
constexpr int kActRows = 64;
constexpr int kActBlocks = 4;  // 128-element runs per row and workgroup
constexpr int kActPasses = kActRows * kActBlocks * 16 / kActThreads;

struct ActQuantParams {
  const uint8_t* x;
  uint8_t* q;
  float* scales;
  int64_t rows, cols, ldx, ldq;  // elements; ldq = cols rounded up to 128
  int32_t col_groups;            // ceil(ceil(cols / 128) / 4)
  float eps;
};

__global__ __launch_bounds__(kActThreads) void act_quant_1x128_kernel(const ActQuantParams p) {
  __shared__ float lds_scales[kActBlocks * kActRows];
  const int tid = threadIdx.x;
  const int sub = tid & 15, run_lane = tid >> 4;
  const int64_t tile_r = blockIdx.x / p.col_groups, tile_c = blockIdx.x % p.col_groups;
  const int64_t row0 = tile_r * kActRows, kb0 = tile_c * kActBlocks;

  u32x4 v[kActPasses];
#pragma unroll
  for (int pass = 0; pass < kActPasses; ++pass) {
    const int run = pass * 16 + run_lane;  // 0..255 within the tile
    const int64_t row = row0 + run / kActBlocks;
    const int64_t col = (kb0 + run % kActBlocks) * 128 + sub * 8;
    v[pass] = u32x4{0, 0, 0, 0};
    if (row < p.rows && col < p.cols) v[pass] = load_stream_u32x4(p.x + (row * p.ldx + col) * 2);
  }
#pragma unroll
  for (int pass = 0; pass < kActPasses; ++pass) {
    const int run = pass * 16 + run_lane;
    const int64_t row = row0 + run / kActBlocks;
    const int64_t col = (kb0 + run % kActBlocks) * 128 + sub * 8;
    uint32_t m = pk_max_u16(v[pass].x & 0x7FFF7FFFu, v[pass].y & 0x7FFF7FFFu);
    m = pk_max_u16(m, v[pass].z & 0x7FFF7FFFu);
    m = pk_max_u16(m, v[pass].w & 0x7FFF7FFFu);
    const uint32_t lo = m & 0xFFFFu, hi = m >> 16;
    m = row16_max_u32(lo > hi ? lo : hi);
    float scale, recip;
    tile_scale(bf16_bits_to_f32(m), p.eps, scale, recip);
    if (sub == 0) lds_scales[(run % kActBlocks) * kActRows + run / kActBlocks] = recip;
    if (row < p.rows && col < p.ldq) {
      const uint32_t d[4] = {v[pass].x, v[pass].y, v[pass].z, v[pass].w};
      uint32_t w[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e0 = u32_as_f32(d[j] << 16) * scale;
        const float e1 = u32_as_f32(d[j] & 0xFFFF0000u) * scale;
        w[j >> 1] = cvt2_fp8(e0, e1, w[j >> 1], (j & 1) != 0);
      }
      store_stream_u32x2(p.q + row * p.ldq + col, w[0], w[1]);
    }
  }
  __syncthreads();
  {
    const int kbl = tid / kActRows, r = tid % kActRows;
    const int64_t kb = kb0 + kbl, row = row0 + r;
    if (row < p.rows && kb * 128 < p.ldq) p.scales[kb * p.rows + row] = lds_scales[tid];
  }
}

// ----------------------------------------------------------------- FP8 GEMM
// 256 x 256 output tile per workgroup (262 flop per operand byte, which is
// what keeps the request rate to L2 within reach at FP8 speed), eight waves of
// 64 x 128 (two by four 32x32 blocks).  A wave's 128 accumulators stay in
// architectural VGPRs, where the vector ALU folds into them, and two waves
// share a SIMD, so one wave's folds run under the other's MFMAs.  Operand
// tiles are 128 bytes per row and k-tile and travel global -> LDS directly,
// 16-byte chunk c of row r in slot c ^ ((r >> 1) & 7), into one of two 64 KB
// stages.  A lane feeds the matrix core bytes [32 h, 32 h + 32) of each half
// of its row (h = lane / 32), i.e. chunks 2h and 2h+1 of a 64-byte half.
//
// TM_ = 1 is the half tile (128 x 256, waves of 32 x 128) that the tiles of a
// last, at most half-full round are cut into; it keeps the LDS layout of the
// whole tile and fills the first half of the A area.
template <int TM_>
struct Fp8GemmCfg {
  static constexpr int BM = 128 * TM_, BN = 256, BK = 128, WM = 4, WN = 2, TM = TM_, TN = 4;
  static constexpr int kWaves = WM * WN, kThreads = 64 * kWaves, kWaveM = BM / WM, kWaveN = BN / WN;
  static constexpr int kRowBytes = 128;
  static constexpr int kABytes = 256 * kRowBytes;              // 32 KB (half of it used by the half tile)
  static constexpr int kStageBytes = (256 + BN) * kRowBytes;   // 64 KB
  static constexpr int kFillRows = 8 * kWaves;                 // tile rows per wave-level load of all waves
  static constexpr int kLoadsA = BM / kFillRows, kLoadsB = BN / kFillRows;  // per wave: 4 (2) and 4
  static constexpr int kPitch = kWaveN * 2 + 8;                // epilogue staging, bytes
  static constexpr int kRegion = kWaveM * kPitch;              // per wave
  static constexpr int kStages = 2;
  static constexpr int kScaleSlots = 64;                        // row scales per wave and stage (one 4-byte request per lane)
  static constexpr int kScaleStageBytes = kWaves * kScaleSlots * 4;
  static constexpr int kScaleOffset = kStages * kStageBytes;
  static constexpr int kWeightScaleOffset = kScaleOffset + kStages * kScaleStageBytes;  // [wave][256] block scales
  static constexpr int kMaxKTilesInLds = 256;  // window of weight block scales kept in LDS per wave (a power of two)
  static constexpr int kLdsBytes = max_int(kWeightScaleOffset + kWaves * kMaxKTilesInLds * 4, kWaves * kRegion);
  static_assert(kWaveM <= kScaleSlots, "one 4-byte scale request per lane covers the wave's rows");
};
using Fp8Gemm = Fp8GemmCfg<2>;
static_assert(Fp8GemmCfg<1>::kLdsBytes <= Fp8Gemm::kLdsBytes, "the half tile lives in the whole tile's LDS");

struct Fp8GemmParams {
  const uint8_t* xq;
  const float* xs;   // [k / 128][m]
  const uint8_t* wq;
  const float* ws;   // block scales: element (output-column block cb, k-block kb) at ws[cb * ws_cb + kb * ws_kb]
  const float* cs;   // per-column scales [k / 128][n] (the other kernel variant)
  uint16_t* out;
  int64_t m, n, k;
  int64_t ldxq, ldwq, ldo, ws_cb, ws_kb;
  GemmParams schedule;  // tile order; its work items are the tiles computed whole
  // Workgroups [whole_grid, ...) take the remaining tiles (in the same order)
  // as two half tiles each, half_items in all.
  int64_t whole_grid, half_items, half_items_per_xcd;
};

typedef int v8i32 __attribute__((ext_vector_type(8)));

// acc[n] += (product[n] * row_scale) * (column_scales of lane n of this lane's row of 16).
// The broadcast is the multiply-add's own operand modifier (the compiler keeps
// a separate move per element when given the builtin).  column_scales comes
// from LDS, not from the vector ALU, so the modifier's read needs no wait states.
template <int N = 0>
__device__ __forceinline__ void fold_with_row_broadcast(f32x16& acc, const f32x16& product, float row_scale,
                                                        float column_scales) {
  if constexpr (N < 16) {
    const float scaled = product[N] * row_scale;
    float sum = acc[N];
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
        : "+v"(sum)
        : "v"(column_scales), "v"(scaled), "n"(N));
    acc[N] = sum;
    fold_with_row_broadcast<N + 1>(acc, product, row_scale, column_scales);
  }
}

// One output tile (TM_ = 2) or half tile (TM_ = 1, rows [128 half, +128) of the tile).
// kLongK: the contraction is longer than one window of weight block scales
// (kMaxKTilesInLds k-tiles); the block-scale variant then refills the window
// inside the loop.  A separate instantiation: the refill's few instructions
// cost the loop 12 % of its rate, which the usual lengths should not pay.
template <bool kColumnScales, int TM_, bool kLongK>
__device__ __forceinline__ void fp8_gemm_tile(const Fp8GemmParams& p, uint8_t* lds_bytes, int tm, int tn, int half) {
  using Cfg = Fp8GemmCfg<TM_>;
  static_assert(Cfg::kStages == 2, "the loop below alternates between two stages");
  constexpr int TM = Cfg::TM, TN = Cfg::TN;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int64_t m0 = static_cast<int64_t>(tm) * Fp8Gemm::BM + static_cast<int64_t>(half) * Cfg::BM;
  const int64_t n0 = static_cast<int64_t>(tn) * Cfg::BN;
  if (m0 >= p.m) return;  // the second half of a tile that ends in its first (whole workgroup)
#ifdef FSH_TRACE
  const uint64_t t_entry = __builtin_amdgcn_s_memrealtime();
#endif
  const int64_t ktiles = p.k / Cfg::BK;

  // Load side: wave-level load q of a wave fills tile rows [64 q + 8 wave, +8);
  // lane l fills slot l & 7 of row l >> 3 there.  Rows past the matrix are
  // read from its last row (their products are never stored).
  const int fill_row = lane >> 3;
  const int fill_chunk = (lane & 7) ^ (((8 * wave + fill_row) >> 1) & 7);
  uint32_t a_voff[Cfg::kLoadsA], b_voff[Cfg::kLoadsB];
#pragma unroll
  for (int q = 0; q < Cfg::kLoadsA; ++q) {
    int64_t row = m0 + Cfg::kFillRows * q + 8 * wave + fill_row;
    row = row < p.m ? row : p.m - 1;
    a_voff[q] = static_cast<uint32_t>((row - m0) * p.ldxq + fill_chunk * 16);
  }
#pragma unroll
  for (int q = 0; q < Cfg::kLoadsB; ++q) {
    int64_t row = n0 + Cfg::kFillRows * q + 8 * wave + fill_row;
    row = row < p.n ? row : p.n - 1;
    b_voff[q] = static_cast<uint32_t>((row - n0) * p.ldwq + fill_chunk * 16);
  }
  const uint8_t* Ab = uniform_ptr(p.xq + m0 * p.ldxq);
  const uint8_t* Bb = uniform_ptr(p.wq + n0 * p.ldwq);
  typedef __attribute__((address_space(3))) uint8_t* lds_address;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_address)lds_bytes));
  const uint32_t fill_lds = lds_base + static_cast<uint32_t>(wave * 1024);
  auto issue_tile_load = [&](int64_t kt, int stage_off) {
    const uint8_t* a_src = Ab + kt * Cfg::kRowBytes;
    const uint8_t* b_src = Bb + kt * Cfg::kRowBytes;
#pragma unroll
    for (int q = 0; q < Cfg::kLoadsA; ++q)
      dma_load_16(a_voff[q], a_src, stage_off + fill_lds + q * Cfg::kFillRows * Cfg::kRowBytes);
#pragma unroll
    for (int q = 0; q < Cfg::kLoadsB; ++q)
      dma_load_16(b_voff[q], b_src, stage_off + Cfg::kABytes + fill_lds + q * Cfg::kFillRows * Cfg::kRowBytes);
  };

  // Fragment side: row = lane & 31 of a 32-row block; chunks 4 kh + 2 h and
  // 4 kh + 2 h + 1 of the row (kh = 64-byte half), each in slot chunk ^ ((row >> 1) & 7).
  const int frag_row = lane & 31, h = lane >> 5;
  uint32_t frag_off[2][2];
#pragma unroll
  for (int kh = 0; kh < 2; ++kh)
#pragma unroll
    for (int c = 0; c < 2; ++c)
      frag_off[kh][c] = static_cast<uint32_t>(frag_row * Cfg::kRowBytes + (((4 * kh + 2 * h + c) ^ ((frag_row >> 1) & 7)) * 16));
  auto read_frag = [&](int stage_off, int operand_off, int block, int kh) -> v8i32 {
    const uint8_t* base = lds_bytes + stage_off + operand_off + block * 32 * Cfg::kRowBytes;
    const u32x4 lo = *reinterpret_cast<const u32x4*>(base + frag_off[kh][0]);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(base + frag_off[kh][1]);
    return v8i32{static_cast<int>(lo.x), static_cast<int>(lo.y), static_cast<int>(lo.z), static_cast<int>(lo.w),
                 static_cast<int>(hi.x), static_cast<int>(hi.y), static_cast<int>(hi.z), static_cast<int>(hi.w)};
  };

  // Scales: a lane owns output row lane & 31 of each of its two 32-row blocks,
  // so it needs xs[kb][row] for two rows and the one weight scale of the
  // wave's 128 columns.
  const int64_t wcol = n0 + wn * Cfg::kWaveN;
  const int64_t wblock = (wcol < p.n ? wcol : p.n - 1) / 128;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Two stages: the operands of k-tile kt + 1 are in flight while kt is
  // multiplied.  The row scales ride the same global->LDS path (two 4-byte-
  // per-lane requests per wave and k-tile for the wave's 128 rows): a
  // compiler-visible load here would make the compiler wait for everything in
  // flight, the prefetched tile included.
  const uint32_t scale_lds0 = lds_base + static_cast<uint32_t>(Cfg::kScaleOffset + wave * Cfg::kScaleSlots * 4);
  const int64_t scale_row = m0 + wm * Cfg::kWaveM + (lane & (Cfg::kWaveM - 1));  // lanes past the wave's rows repeat them
  const uint32_t scale_voff = static_cast<uint32_t>((scale_row < p.m ? scale_row : p.m - 1) * 4);
  // Per-column scales of the workgroup's 256 columns take the same road, 64
  // columns per wave (the first four waves), into [stage][256] floats of the
  // block-scale area.
  const uint32_t cscale_lds0 = lds_base + static_cast<uint32_t>(Cfg::kWeightScaleOffset + wave * 256);
  const int64_t cscale_col0 = n0 + wave * 64 + lane;
  const uint32_t cscale_voff = static_cast<uint32_t>((cscale_col0 < p.n ? cscale_col0 : p.n - 1) * 4);
  auto issue_scale_loads = [&](int64_t kt, int stage) {
    const uint8_t* xs_row = reinterpret_cast<const uint8_t*>(p.xs + kt * p.m);
    dma_touch_4(scale_voff, xs_row, scale_lds0 + stage * Cfg::kScaleStageBytes);
    if (kColumnScales && wave < 4)
      dma_touch_4(cscale_voff, reinterpret_cast<const uint8_t*>(p.cs + kt * p.n), cscale_lds0 + stage * 1024);
  };
  auto issue_k_tile = [&](int64_t kt, int stage) {
    issue_tile_load(kt, stage * Cfg::kStageBytes);
    issue_scale_loads(kt, stage);
  };
  // One of the wave's requests for the next k-tile; they are issued a few at
  // a time behind the MFMAs of the first blocks rather than all at once, which
  // would hold up the wave's instruction issue while the matrix core runs dry.
  auto issue_k_tile_part = [&](int64_t kt, int stage, int part) {
    const int stage_off = stage * Cfg::kStageBytes;
    if (part >= Cfg::kLoadsA + Cfg::kLoadsB) return;
    if (part >= Cfg::kLoadsA) {
      const int q = part - Cfg::kLoadsA;
      dma_load_16(b_voff[q], Bb + kt * Cfg::kRowBytes,
                  stage_off + Cfg::kABytes + fill_lds + q * Cfg::kFillRows * Cfg::kRowBytes);
    } else {
      dma_load_16(a_voff[part], Ab + kt * Cfg::kRowBytes, stage_off + fill_lds + part * Cfg::kFillRows * Cfg::kRowBytes);
    }
    if (part == 0) issue_scale_loads(kt, stage);
  };
  // The first k-tile's requests go out before anything else that has to wait
  // for memory.  The block scales of the wave's 128 columns, one per k-tile,
  // are copied to LDS once, under those requests (a load from global memory
  // inside the loop would again wait for the prefetched tile).
  issue_k_tile(0, 0);
  float* ws_lds = reinterpret_cast<float*>(lds_bytes + Cfg::kWeightScaleOffset + wave * Cfg::kMaxKTilesInLds * 4);
  // ws_lds holds the scales of k-tiles [window, window + kMaxKTilesInLds).
  // For a contraction of at most one window they are copied once, under the
  // first k-tile's requests.  A longer one (kLongK) refills the window when
  // the loop reaches its last k-tile, and then the scales travel global -> LDS
  // like everything else the loop reads (four 4-byte-per-lane requests per
  // window): a load the compiler sees inside the loop makes it wait for all
  // memory traffic in flight on every iteration (measured: 20 % slower).
  const uint32_t ws_lds_addr = lds_base + static_cast<uint32_t>(Cfg::kWeightScaleOffset + wave * Cfg::kMaxKTilesInLds * 4);
  auto issue_weight_scale_window = [&](int64_t first_kt) {
    const uint8_t* ws_row = reinterpret_cast<const uint8_t*>(p.ws + wblock * p.ws_cb);
#pragma unroll
    for (int q = 0; q < Cfg::kMaxKTilesInLds / 64; ++q) {
      int64_t kt_of_lane = first_kt + q * 64 + lane;
      kt_of_lane = kt_of_lane < ktiles ? kt_of_lane : ktiles - 1;  // past the end: any valid entry, never read
      dma_touch_4(static_cast<uint32_t>(kt_of_lane * p.ws_kb * 4), ws_row, ws_lds_addr + q * 256);
    }
  };
  if (!kColumnScales) {
    if (kLongK) {
      issue_weight_scale_window(0);
    } else {
      const float* ws_row = p.ws + wblock * p.ws_cb;
      for (int64_t i = lane; i < ktiles; i += 64) ws_lds[i] = ws_row[i * p.ws_kb];  // ktiles <= kMaxKTilesInLds (host)
    }
  }
  wait_for_dma_loads();
  __syncthreads();

#ifdef FSH_TRACE
  // Time per phase of the k loop, summed over the k-tiles (10 ns ticks).
  uint64_t t_compute = 0, t_wait = 0, t_barrier = 0, t_mark = __builtin_amdgcn_s_memrealtime();
  const uint64_t t_begin = t_mark;
  auto lap = [&](uint64_t& sum) {
    const uint64_t now = __builtin_amdgcn_s_memrealtime();
    sum += now - t_mark;
    t_mark = now;
  };
#endif
  // The k loop is rotated by one block: the barrier that hands over k-tile
  // kt + 1 sits before the last 32x32 block of k-tile kt, and behind that
  // block's MFMAs the wave already reads what the first block of kt + 1 needs
  // (its first A and B fragments).  The first MFMAs after a
  // barrier thus never wait for an LDS read, which every wave of the
  // workgroup would otherwise do at the same moment.
  //   carried into a k-tile: afrag[0], bfrag[0]
  constexpr int kBSets = kColumnScales ? 1 : 2;  // the per-column variant has registers for one set of B fragments only
  constexpr int kBlocks = TM * TN;
  v8i32 afrag[TM][2], bfrag[kBSets][2];
  float s[TM], cs_rows[TN];
  // Row scales of the wave's rows for the k-tile in `stage`, times the weight
  // block's scale in the block-scale variant.
  auto read_row_scales = [&](float (&dst)[TM], int stage, int64_t kt) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
      dst[i] = *reinterpret_cast<const float*>(lds_bytes + Cfg::kScaleOffset + stage * Cfg::kScaleStageBytes +
                                               (wave * Cfg::kScaleSlots + i * 32 + frag_row) * 4);
    if (!kColumnScales) {
      const float ws_now = ws_lds[kLongK ? (kt & (Cfg::kMaxKTilesInLds - 1)) : kt];
#pragma unroll
      for (int i = 0; i < TM; ++i) dst[i] *= ws_now;
    }
  };
  // Per-column scales: register j holds, in every row of 16 lanes, the 16
  // scales of column block j that the lanes of that row fold with (lane n of
  // the row the scale of accumulator element n), so a fold takes element n's
  // scale from lane n of its own row through the data-parallel-primitive
  // broadcast of the multiply-add itself: no scale is read from LDS between a
  // product and its fold.
  auto read_column_scales = [&](float (&dst)[TN], int stage) {
    if (kColumnScales) {
      const uint8_t* cscale_lds = lds_bytes + Cfg::kWeightScaleOffset + stage * 1024 +
                                  (wn * Cfg::kWaveN + 8 * ((lane & 15) >> 2) + 4 * h + (lane & 3)) * 4;
#pragma unroll
      for (int j = 0; j < TN; ++j) dst[j] = *reinterpret_cast<const float*>(cscale_lds + j * 32 * 4);
    }
  };
  auto read_first_frags = [&](int stage_off) {
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) bfrag[0][kh] = read_frag(stage_off, Cfg::kABytes, wn * (Cfg::kWaveN / 32), kh);
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) afrag[0][kh] = read_frag(stage_off, 0, wm * (Cfg::kWaveM / 32), kh);
  };
  read_first_frags(0);

  int stage = 0;
  for (int64_t kt = 0; kt < ktiles; ++kt) {
    const int stage_off = stage * Cfg::kStageBytes;
    const bool more = kt + 1 < ktiles;  // the next k-tile's stage was released by the barrier inside kt - 1
    // The scales are first needed by the fold behind the second block's MFMAs.
    read_row_scales(s, stage, kt);
    read_column_scales(cs_rows, stage);
    if (kLongK && !kColumnScales && more && (kt & (Cfg::kMaxKTilesInLds - 1)) == Cfg::kMaxKTilesInLds - 1) {
      // Last k-tile of the window (once per 32 768 of k): its scale has just
      // been read; the next window is requested over it and lands before this
      // k-tile's hand-over barrier, like the operands of k-tile kt + 1.
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      issue_weight_scale_window(kt + 1);
    }
    // Fragments are read in the order the blocks need them: the other A row
    // blocks under the MFMAs of the first column block (they stay for the
    // whole k-tile), each further B column block while the previous one is
    // multiplied.
    // The wave's eight 32x32 blocks, column block by column block: two MFMAs, back
    // to back, give a block's partial product for this scale block.  It is
    // folded into the result (16 fused multiply-adds, or multiply + fused
    // multiply-add with per-column scales) one block later, behind that
    // block's MFMAs: a fold that reads the product of the MFMA issued just
    // before it waits for the matrix core to drain (measured: 122 against 100
    // time units per block for the arrangement used here).
    // Blocks between a product and its fold.  One: the other wave of the SIMD
    // keeps the matrix core busy while this one waits for its own product,
    // and the registers of a third product are needed elsewhere.
    constexpr int kLag = 1;
    f32x16 part[kLag + 1];
    auto fold = [&](int blk, const f32x16& product) {
      const int pi = blk % TM, pj = blk / TM;
      if (kColumnScales) {
        fold_with_row_broadcast(acc[pi][pj], product, s[pi], cs_rows[pj]);
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[pi][pj][r] = __builtin_fmaf(product[r], s[pi], acc[pi][pj][r]);
      }
      // An empty statement that "uses" the folded block keeps its arithmetic
      // on this side of the next scheduling barrier.
      asm volatile("" : "+v"(acc[pi][pj]));
    };
#pragma unroll
    for (int blk = 0; blk < kBlocks; ++blk) {
      const int i = blk % TM, j = blk / TM;
      const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (blk == kBlocks - 1) {
        // Every fragment of this k-tile is in registers: hand the stage over.
#ifdef FSH_TRACE
        lap(t_compute);
#endif
        if (more) wait_for_dma_loads();  // this wave's part of k-tile kt + 1 has landed
#ifdef FSH_TRACE
        lap(t_wait);
#endif
        __syncthreads();
#ifdef FSH_TRACE
        lap(t_barrier);
#endif
      }
      if (j == 0 && i + 1 < TM) {  // next row block's A fragments
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) afrag[i + 1][kh] = read_frag(stage_off, 0, wm * (Cfg::kWaveM / 32) + i + 1, kh);
      }
      if (kBSets == 2 && i == TM - 1 && j + 1 < TN) {  // next column block's B fragments, one block ahead
#pragma unroll
        for (int kh = 0; kh < 2; ++kh)
          bfrag[(j + 1) % kBSets][kh] = read_frag(stage_off, Cfg::kABytes, wn * (Cfg::kWaveN / 32) + j + 1, kh);
      }
      // Wave priority falls as the k-tile proceeds: of the two waves of a SIMD
      // the one that is behind wins the issue slot, so both reach the barrier
      // together (with equal priorities the older wave runs ahead and then
      // idles at the barrier while the other finishes alone, without a
      // partner to overlap its folds with).
      if (blk * 4 == 0 * kBlocks) __builtin_amdgcn_s_setprio(3);
      if (blk * 4 == 1 * kBlocks) __builtin_amdgcn_s_setprio(2);
      if (blk * 4 == 2 * kBlocks) __builtin_amdgcn_s_setprio(1);
      if (blk * 4 == 3 * kBlocks) __builtin_amdgcn_s_setprio(0);
      f32x16 product =
          __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bfrag[j % kBSets][0], afrag[i][0], zero, 0, 0, 0, 0, 0, 0);
      product =
          __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bfrag[j % kBSets][1], afrag[i][1], product, 0, 0, 0, 0, 0, 0);
      part[blk % (kLag + 1)] = product;
      __builtin_amdgcn_sched_barrier(0);
      if (kBSets == 1 && i == TM - 1 && j + 1 < TN) {  // behind the last MFMAs that read the current set
#pragma unroll
        for (int kh = 0; kh < 2; ++kh)
          bfrag[0][kh] = read_frag(stage_off, Cfg::kABytes, wn * (Cfg::kWaveN / 32) + j + 1, kh);
      }
      if (blk == kBlocks - 1 && more) {  // behind the last MFMAs of this k-tile: what the next one starts with
        read_first_frags(stage_off ^ Cfg::kStageBytes);
      }
      // The next k-tile's requests leave during the first half of this one, so
      // the data has the second half to arrive (spread over all blocks, the last
      // requests were still in flight at the hand-over: 0.15-0.35 us of every
      // 2 us k-tile went to waiting for them; moved one block earlier still,
      // behind the hand-over barrier of the previous k-tile, the per-column
      // variant ran out of registers).
      constexpr int kIssueBlocks = kBlocks / 2;
      constexpr int kPartsPerBlock = (Cfg::kLoadsA + Cfg::kLoadsB + kIssueBlocks - 1) / kIssueBlocks;
      if (more && blk < kIssueBlocks) {
#pragma unroll
        for (int part = 0; part < kPartsPerBlock; ++part) issue_k_tile_part(kt + 1, stage ^ 1, blk * kPartsPerBlock + part);
      }
      if (blk >= kLag) fold(blk - kLag, part[(blk - kLag) % (kLag + 1)]);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int blk = kBlocks - kLag; blk < kBlocks; ++blk) fold(blk, part[blk % (kLag + 1)]);
    stage ^= 1;
  }
#ifdef FSH_TRACE
  if (p.schedule.trace && lane == 0) {
    uint64_t* out = p.schedule.trace + (static_cast<int64_t>(blockIdx.x) * Cfg::kWaves + wave) * 8;
    out[0] = t_begin; out[1] = t_compute; out[2] = t_wait; out[3] = t_barrier; out[4] = t_mark; out[5] = t_entry;
  }
#endif

  // Epilogue: bf16 finals to the wave's staging region as [row][col], then
  // 16-byte row stores, rows and 8-column groups past the matrix skipped.
  uint8_t* region = lds_bytes + wave * Cfg::kRegion;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int b = 0; b < 4; ++b)
        *reinterpret_cast<u32x2*>(region + (i * 32 + frag_row) * Cfg::kPitch + (j * 32 + 8 * b + 4 * h) * 2) =
            u32x2{pack_bf16x2(acc[i][j][4 * b], acc[i][j][4 * b + 1]),
                  pack_bf16x2(acc[i][j][4 * b + 2], acc[i][j][4 * b + 3])};
  wave_lds_sync();
  {
    constexpr int kLanesPerRow = Cfg::kWaveN * 2 / 16, kRowsPerPass = 64 / kLanesPerRow;
    const int r0 = lane / kLanesPerRow, chunk = lane % kLanesPerRow;
    const int64_t wave_row = m0 + wm * Cfg::kWaveM, col = n0 + wn * Cfg::kWaveN + chunk * 8;
    const bool vec_ok = (p.ldo % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
    for (int pass = 0; pass < Cfg::kWaveM / kRowsPerPass; ++pass) {
      const int r = pass * kRowsPerPass + r0;
      const int64_t row = wave_row + r;
      if (row >= p.m || col >= p.n) continue;
      const uint8_t* src = region + r * Cfg::kPitch + chunk * 16;
      const u32x2 lo = *reinterpret_cast<const u32x2*>(src);
      const u32x2 hi = *reinterpret_cast<const u32x2*>(src + 8);
      uint16_t* dst = p.out + row * p.ldo + col;
      if (vec_ok && col + 8 <= p.n) {
        *reinterpret_cast<u32x4*>(dst) = u32x4{lo.x, lo.y, hi.x, hi.y};
      } else {
        const uint32_t w[4] = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < p.n) dst[e] = static_cast<uint16_t>(w[e >> 1] >> (16 * (e & 1)));
      }
    }
  }
#ifdef FSH_TRACE
  if (p.schedule.trace && lane == 0) {
    __builtin_amdgcn_s_waitcnt(0);
    p.schedule.trace[(static_cast<int64_t>(blockIdx.x) * Cfg::kWaves + wave) * 8 + 6] = __builtin_amdgcn_s_memrealtime();
    uint32_t hw_id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_id));
    uint32_t xcc_id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_id));
    p.schedule.trace[(static_cast<int64_t>(blockIdx.x) * Cfg::kWaves + wave) * 8 + 7] = (static_cast<uint64_t>(xcc_id) << 32) | hw_id;
  }
#endif
}

// kColumnScales = false: the second operand carries one scale per 128 x 128
// tile (a prequantized weight, either orientation).  true: one scale per
// output column and k-block (an operand quantized in 128 x 1 runs).
template <bool kColumnScales, bool kLongK = false>
__global__ __launch_bounds__(Fp8Gemm::kThreads) void fp8_gemm_blockwise_kernel(const Fp8GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds_bytes[];
  int64_t unused_batch;
  int tm, tn;
  if (static_cast<int64_t>(blockIdx.x) < p.whole_grid) {
    if (!tile_of_workgroup(p.schedule, blockIdx.x, &unused_batch, &tm, &tn)) return;  // whole workgroup
    fp8_gemm_tile<kColumnScales, 2, kLongK>(p, lds_bytes, uniform_i32(tm), uniform_i32(tn), 0);
  } else {
    // Same split over the XCDs as the whole tiles: the two halves of a tile are
    // neighbours in an XCD's run and share the tile's second operand in its L2.
    const int64_t id = static_cast<int64_t>(blockIdx.x) - p.whole_grid;
    const int64_t item = (id % kXcds) * p.half_items_per_xcd + id / kXcds;
    if (item >= p.half_items) return;
    tile_in_order(p.schedule, static_cast<int>(p.schedule.work_items + item / 2), &tm, &tn);
    fp8_gemm_tile<kColumnScales, 1, kLongK>(p, lds_bytes, uniform_i32(tm), uniform_i32(tn),
                                            uniform_i32(static_cast<int>(item & 1)));
  }
}

}  // namespace
}  // namespace fsh

FSH_API int fsh_act_quant_1x128(const void* x_dev, int64_t rows, int64_t cols, int64_t ldx, void* q_dev,
                                int64_t ldq, float* scales_dev, int32_t eps_mode, void* stream) {
  using namespace fsh;
  if (rows < 0 || cols < 0) return fail(FSH_EINVAL, "fsh_act_quant_1x128: negative shape");
  if (rows == 0 || cols == 0) return FSH_OK;
  if (!x_dev || !q_dev || !scales_dev) return fail(FSH_EINVAL, "fsh_act_quant_1x128: null pointer");
  if (eps_mode != FSH_EPS_INPUT_DTYPE && eps_mode != FSH_EPS_FP32)
    return fail(FSH_EINVAL, "fsh_act_quant_1x128: unknown eps_mode %d", eps_mode);
  const int64_t padded = ceil_div(cols, (int64_t)128) * 128;
  if (ldx < cols || ldq != padded)
    return fail(FSH_EINVAL, "fsh_act_quant_1x128: ldx %lld < cols %lld, or ldq %lld is not cols rounded up to 128 (%lld)",
                (long long)ldx, (long long)cols, (long long)ldq, (long long)padded);
  if (cols % 8 || ldx % 8 || !aligned(x_dev, 16) || !aligned(q_dev, 8) || !aligned(scales_dev, 4))
    return fail(FSH_ENOTSUP, "fsh_act_quant_1x128: cols and ldx must be multiples of 8, x 16-byte and q 8-byte aligned");
  ActQuantParams p;
  p.x = static_cast<const uint8_t*>(x_dev);
  p.q = static_cast<uint8_t*>(q_dev);
  p.scales = scales_dev;
  p.rows = rows;
  p.cols = cols;
  p.ldx = ldx;
  p.ldq = ldq;
  const int64_t col_groups = ceil_div(padded / 128, (int64_t)kActBlocks);
  p.col_groups = static_cast<int32_t>(col_groups);
  const float eps32 = 1e-12f;
  uint32_t bits;
  memcpy(&bits, &eps32, 4);
  bits = (bits + 0x7FFFu + ((bits >> 16) & 1u)) & 0xFFFF0000u;
  float eps_bf16;
  memcpy(&eps_bf16, &bits, 4);
  p.eps = eps_mode == FSH_EPS_FP32 ? eps32 : eps_bf16;
  const int64_t grid = ceil_div(rows, (int64_t)kActRows) * col_groups;
  if (grid > 0x7FFFFFFFLL || col_groups > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "fsh_act_quant_1x128: too many tiles");
  hipLaunchKernelGGL(act_quant_1x128_kernel, dim3(static_cast<uint32_t>(grid)), dim3(kActThreads), 0,
                     static_cast<hipStream_t>(stream), p);
  return check_launch("act_quant_1x128_kernel");
}

namespace fsh {
namespace {

// Shared checks and launch of the two FP8 GEMM variants.  `p` arrives with
// the operands, sizes and scale tables filled in.
int launch_fp8_gemm(Fp8GemmParams& p, bool column_scales, const char* who, void* stream) {
  if (p.m < 0 || p.n < 0 || p.k < 0) return fail(FSH_EINVAL, "%s: negative size", who);
  if (p.m == 0 || p.n == 0) return FSH_OK;
  if (!p.xq || !p.xs || !p.wq || !p.out || (column_scales ? !p.cs : !p.ws)) return fail(FSH_EINVAL, "%s: null pointer", who);
  if (p.k == 0 || p.k % 128)
    return fail(FSH_ENOTSUP, "%s: k must be a positive multiple of 128 (pad the operands), got %lld", who, (long long)p.k);
  if (p.k >= (1LL << 31)) return fail(FSH_ENOTSUP, "%s: k must be below 2^31, got %lld", who, (long long)p.k);
  if (!column_scales && (p.k / 128) * p.ws_kb * 4 >= (1LL << 31))
    return fail(FSH_ENOTSUP, "%s: a row of the weight scale table spans more than 2 GiB", who);
  if (p.ldxq < p.k || p.ldwq < p.k || p.ldo < p.n)
    return fail(FSH_EINVAL, "%s: a leading dimension is smaller than its row", who);
  if (p.ldxq % 16 || p.ldwq % 16 || !aligned(p.xq, 16) || !aligned(p.wq, 16) || !aligned(p.out, 2))
    return fail(FSH_ENOTSUP, "%s: operand rows must be 16-byte aligned", who);
  if (static_cast<int64_t>(Fp8Gemm::BN) * p.ldwq >= (1LL << 31) || static_cast<int64_t>(Fp8Gemm::BM) * p.ldxq >= (1LL << 31) ||
      p.m >= (1LL << 29) || p.n >= (1LL << 29))
    return fail(FSH_ENOTSUP, "%s: a tile spans more than 2 GiB", who);
  GemmParams& s = p.schedule;
  memset(&s, 0, sizeof(s));
#ifdef FSH_TRACE
  if (const char* e = getenv("FSH_GEMM_TRACE")) s.trace = reinterpret_cast<uint64_t*>(strtoull(e, nullptr, 0));
#endif
  s.tiles_m = static_cast<int32_t>(ceil_div(p.m, (int64_t)Fp8Gemm::BM));
  s.tiles_n = static_cast<int32_t>(ceil_div(p.n, (int64_t)Fp8Gemm::BN));
  const int64_t tiles = static_cast<int64_t>(s.tiles_m) * s.tiles_n;
  if (tiles > 0x3FFFFFFFLL) return fail(FSH_ENOTSUP, "%s: too many tiles", who);
  s.tiles_per_matrix = static_cast<int32_t>(tiles);
  // A workgroup holds a CU for a tile, so the tiles go through the chip in
  // rounds of one per CU.  A last round that is at most half full is cut into
  // half tiles, twice as many workgroups of half the length: e.g. the 896
  // tiles of a [14336, 4096] result take 3.5 rounds instead of 4.
  const int64_t units = compute_units();
  const int64_t tail = units > 0 ? tiles % units : 0;
  const int64_t cut = (tail > 0 && 2 * tail <= units) ? tail : 0;
  s.work_items = tiles - cut;
  s.items_per_xcd = ceil_div(s.work_items, static_cast<int64_t>(kXcds));
  p.whole_grid = s.items_per_xcd * kXcds;
  p.half_items = 2 * cut;
  p.half_items_per_xcd = ceil_div(p.half_items, static_cast<int64_t>(kXcds));
  // The block-scale variant keeps one window of weight scales in LDS; a longer
  // contraction takes the instantiation that refills it.
  const bool long_k = !column_scales && p.k / 128 > Fp8Gemm::kMaxKTilesInLds;
  static LdsReservation reserved_block_scales, reserved_block_scales_long, reserved_column_scales;
  if (int rc = column_scales
                   ? reserve_lds_once(reserved_column_scales, &fp8_gemm_blockwise_kernel<true>, Fp8Gemm::kLdsBytes)
               : long_k
                   ? reserve_lds_once(reserved_block_scales_long, &fp8_gemm_blockwise_kernel<false, true>, Fp8Gemm::kLdsBytes)
                   : reserve_lds_once(reserved_block_scales, &fp8_gemm_blockwise_kernel<false>, Fp8Gemm::kLdsBytes))
    return rc;
  const dim3 grid(static_cast<uint32_t>(p.whole_grid + p.half_items_per_xcd * kXcds)), block(Fp8Gemm::kThreads);
  if (column_scales)
    hipLaunchKernelGGL(fp8_gemm_blockwise_kernel<true>, grid, block, Fp8Gemm::kLdsBytes, static_cast<hipStream_t>(stream), p);
  else if (long_k)
    hipLaunchKernelGGL((fp8_gemm_blockwise_kernel<false, true>), grid, block, Fp8Gemm::kLdsBytes,
                       static_cast<hipStream_t>(stream), p);
  else
    hipLaunchKernelGGL(fp8_gemm_blockwise_kernel<false>, grid, block, Fp8Gemm::kLdsBytes, static_cast<hipStream_t>(stream), p);
  return check_launch("fp8_gemm_blockwise_kernel");
}

}  // namespace
}  // namespace fsh

FSH_API int fsh_fp8_gemm_1x128_128x128(const void* xq_dev, const float* xs_dev, const void* wq_dev,
                                       const float* ws_dev, void* out_dev, int64_t m, int64_t n, int64_t k,
                                       int64_t ldxq, int64_t ldwq, int64_t ldo, int64_t ws_cols, void* stream) {
  using namespace fsh;
  if (k > 0 && ws_cols < k / 128)
    return fail(FSH_EINVAL, "fsh_fp8_gemm_1x128_128x128: the weight scale table has %lld columns, k / 128 = %lld",
                (long long)ws_cols, (long long)(k / 128));
  Fp8GemmParams p;
  memset(&p, 0, sizeof(p));
  p.xq = static_cast<const uint8_t*>(xq_dev);
  p.xs = xs_dev;
  p.wq = static_cast<const uint8_t*>(wq_dev);
  p.ws = ws_dev;
  p.out = static_cast<uint16_t*>(out_dev);
  p.m = m; p.n = n; p.k = k;
  p.ldxq = ldxq; p.ldwq = ldwq; p.ldo = ldo;
  p.ws_cb = ws_cols; p.ws_kb = 1;
  return launch_fp8_gemm(p, false, "fsh_fp8_gemm_1x128_128x128", stream);
}

FSH_API int fsh_fp8_gemm_1x128_128x128_dgrad(const void* gq_dev, const float* gs_dev, const void* wtq_dev,
                                             const float* ws_dev, void* out_dev, int64_t m, int64_t in_dim,
                                             int64_t out_dim, int64_t ldgq, int64_t ldwt, int64_t ldo,
                                             int64_t ws_cols, void* stream) {
  using namespace fsh;
  if (in_dim > 0 && ws_cols < ceil_div(in_dim, (int64_t)128))
    return fail(FSH_EINVAL, "fsh_fp8_gemm_1x128_128x128_dgrad: the weight scale table has %lld columns, in_dim needs %lld",
                (long long)ws_cols, (long long)ceil_div(in_dim, (int64_t)128));
  Fp8GemmParams p;
  memset(&p, 0, sizeof(p));
  p.xq = static_cast<const uint8_t*>(gq_dev);
  p.xs = gs_dev;
  p.wq = static_cast<const uint8_t*>(wtq_dev);
  p.ws = ws_dev;
  p.out = static_cast<uint16_t*>(out_dev);
  p.m = m; p.n = in_dim; p.k = out_dim;
  p.ldxq = ldgq; p.ldwq = ldwt; p.ldo = ldo;
  p.ws_cb = 1; p.ws_kb = ws_cols;  // the weight's table read across: (input block, output block)
  return launch_fp8_gemm(p, false, "fsh_fp8_gemm_1x128_128x128_dgrad", stream);
}

FSH_API int fsh_fp8_gemm_1x128_128x1(const void* aq_dev, const float* as_dev, const void* bq_dev,
                                     const float* bs_dev, void* out_dev, int64_t m, int64_t n, int64_t k,
                                     int64_t ldaq, int64_t ldbq, int64_t ldo, void* stream) {
  using namespace fsh;
  Fp8GemmParams p;
  memset(&p, 0, sizeof(p));
  p.xq = static_cast<const uint8_t*>(aq_dev);
  p.xs = as_dev;
  p.wq = static_cast<const uint8_t*>(bq_dev);
  p.cs = bs_dev;
  p.out = static_cast<uint16_t*>(out_dev);
  p.m = m; p.n = n; p.k = k;
  p.ldxq = ldaq; p.ldwq = ldbq; p.ldo = ldo;
  return launch_fp8_gemm(p, true, "fsh_fp8_gemm_1x128_128x1", stream);
}
