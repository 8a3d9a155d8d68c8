// Scaled FP8 GEMMs for gfx950: c[m,n] = sum_kb sa(m,kb) * sb(n,kb) * (A_kb . B_kb^T).
//
// Layout of the work
//   * Both operands are K-contiguous E4M3 codes, so a 16-row x 128-byte slab of either is exactly
//     one operand of v_mfma_f32_16x16x128_f8f6f4: one matrix instruction consumes one whole
//     128-wide scaling block, and its fp32 result is promoted into the running accumulator with
//     one FMA per element (acc += partial * sa * sb).
//   * The weight-like operand b feeds the MFMA "A" port and the activation-like operand a the
//     "B" port: a lane then holds 4 consecutive n for one m, which makes the per-row scale
//     sa(m,kb) a per-lane constant.
//   * Workgroup tile 256(m) x 256(n) x 128(k), 8 waves as 4(m) x 2(n), wave tile 64 x 128
//     (128 fp32 accumulators per lane, 2 waves per SIMD so one wave's FMAs overlap the other's
//     MFMAs).  LDS holds two buffers for the a tile and three for the b tile (32 KB each); tiles
//     are DMA'd global -> LDS with 128-bit buffer loads (out-of-range rows read as zero), 16-byte
//     chunks XOR-swizzled by row so that both the DMA writes and the ds_read_b128 fragment reads
//     are bank-conflict free.
//   * The grid is persistent: one workgroup per CU walks a list of tiles, and the rounds of
//     consecutive tiles follow each other without a gap.  Each XCD (own L2) owns a contiguous run
//     of tile numbers.
//   * Results leave through the wave's own slice of a consumed LDS buffer, regrouped into whole rows of
//     256 bytes, as streaming stores through a buffer resource that ends with the tile's last valid row
//     (rows past the end of a ragged tile or of an expert are dropped by its range check); with
//     accumulate, c's old values are the accumulators' starting values, loaded before the tile's first round.
//   * One kernel template, by scale form: per tensor, 128x128 blocks of b (forward, dgrad), per-row
//     scales on both operands (wgrad), and the two blockwise forms again for scales that are powers of
//     two, which the matrix instruction applies itself (no promotion FMAs); dense, grouped by expert
//     along the rows (MoE forward and dgrad: an expert owns a range of rows of a and c and its own b), or
//     grouped along the contraction (MoE wgrad: an expert owns a range of k-blocks of both operands and
//     its own c); bf16 or fp32 output, optionally added onto what c holds.
#include <atomic>
#include <type_traits>

#include "hpfp8_device.h"
#include "hpfp8_host.h"

namespace hpfp8 {

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kGemmThreads = 512;
constexpr int kTileBytes = 256 * BK;          // one operand tile in LDS (32 KB)
// LDS: two buffers for the a tile, then kBStages buffers for the b tile.  The b operand is the one
// that streams from HBM (each weight panel is used by one XCD only), so where LDS allows it gets a
// third buffer and its transfers run two k-blocks ahead; a's re-reads come from the Infinity Cache.
__host__ __device__ constexpr int b_stages(int mode) { return (mode == 2 || mode == 4) /* per-row b scales: LDS also holds them */ ? 2 : 3; }
constexpr int kXcds = 8;
constexpr int kRectTiles = 32;              // tiles of the rectangle one XCD (32 CUs) works on at a time

// kScalePow2: scales laid out as for kScaleBlock but every one a power of two; the matrix instruction
// applies them itself (its E8M0 block-scale operands) and accumulates across k-blocks, so there is no
// promotion arithmetic at all.
// kScalePow2Row: the same with the scales laid out as for kScaleRow.
enum ScaleMode { kScaleTensor = 0, kScaleBlock = 1, kScaleRow = 2, kScalePow2 = 3, kScalePow2Row = 4 };

enum Grouping { kDense = 0, kGroupedRows = 1, kGroupedK = 2 };

struct GemmParams {
  const uint8_t* a;
  const uint8_t* b;
  const float* sa;
  const float* sb;
  int64_t sa_sm, sa_sk;   // element strides of sa over (row, k-block)
  int64_t sb_sn, sb_sk;   // element strides of sb over (row or 128-row block, k-block)
  int64_t sb_se;          // grouped by rows: stride of sb between experts
  int64_t b_se;           // grouped by rows: bytes from one expert's b to the next
  int64_t c_se;           // grouped along the contraction: elements from one expert's c to the next
  int sb_bytes;           // size of the sb array in bytes (block form)
  void* c;
  int64_t ldc;
  const uint16_t* bias;
  const int32_t* offs;    // grouped by rows: inclusive prefix sums of rows per expert
  const int32_t* layout;  // grouped along the contraction: the table of grouped.hip
  int experts;
  int64_t lda, ldb;       // row strides of a and b in bytes (>= K)
  int M, N, K;            // M = total rows of a; grouped along the contraction: K = the padded token axis
  int tiles;              // dense: number of output tiles; grouped along the contraction: per expert
  int accumulate;
  // SwiGLU epilogue: b = W_gate_up codes [2 * inter, K] (gate rows first), N = 2 * inter; c = codes of the
  // activation [M, inter] (row stride ldc bytes), q_scale (may be null) / q_scale_inv its 1x128 scales, [inter / 128, M]
  int inter;
  int pow2_out;
  float* q_scale;
  float* q_scale_inv;
};

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// XOR applied to the 16-byte chunk index of tile row r.  ds_read_b128 is served 16 lanes at a time
// and the 16 are not consecutive: per half-wave the lane quads {0,3,5,6} go together and {1,2,4,7}
// go together (measured with SQ_LDS_BANK_CONFLICT on pairs of active lanes).  With the fragment
// mapping lane -> (row = lane%16, k-chunk pair = lane/16) each such group holds all 16 rows once,
// rows 4..11 with one k-chunk and the other rows with the neighbouring one; shifting the usual
// (r/2)%8 pattern by 6 sends those two row sets to disjoint chunk ranges, so the 16 lanes hit 16
// different bank groups.
__device__ __forceinline__ int row_swizzle(int r) { return (((r >> 1) & 7) + 6) & 7; }

__device__ __forceinline__ v4i lds_read16(const uint8_t* p) {
  return *reinterpret_cast<const v4i*>(p);
}

__device__ __forceinline__ v8i frag_read(const uint8_t* row_base, int pc0) {
  v4i lo = lds_read16(row_base + pc0 * 16);
  v4i hi = lds_read16(row_base + (pc0 ^ 1) * 16);
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

// two floats -> two bf16 in one word (a low, b high): one v_cvt_pk_bf16_f32 (converted one by one, each
// value costs a conversion, a shift and an or)
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}

// Tile number -> (m tile, n tile).  Consecutive numbers (one XCD's CUs at any moment) cover
// gm x gn rectangles of tiles (gm * gn = 32), n fastest inside a rectangle, so the L2 of that XCD
// serves each activation / weight panel to several CUs.  A panel of a is fetched once per column
// of rectangles (tiles_n / gn times in all) and a panel of b once per row of rectangles: the longer
// side of the rectangle goes along the shorter side of the tile grid, so that the larger operand,
// the one the Infinity Cache cannot hold, is the one fetched fewer times.  Rectangles at the right
// and bottom edges shrink.
__device__ __forceinline__ void rect_map(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int gm = tiles_m > tiles_n ? 4 : 8, gn_full = kRectTiles / gm;
  const int per_ngroup = gn_full * tiles_m;
  const int ng = t / per_ngroup, rest = t % per_ngroup;
  const int gn = (tiles_n - ng * gn_full) < gn_full ? (tiles_n - ng * gn_full) : gn_full;
  const int mg = rest / (gm * gn);
  const int r3 = rest - mg * gm * gn;
  tm = mg * gm + r3 / gn;
  tn = ng * gn_full + r3 % gn;
}

// One output tile of a workgroup's list.  A tile with no rows (row0 == row_end, n0 >= N) stands for
// "past the end of the list": transfers addressed to it fetch nothing.
struct TileInfo {
  int row0, row_end;   // rows [row0, row_end) of a and c that exist (row_end - row0 may be < BM)
  int n0;              // first row of b / column of c
  int expert;
  int kb0, kbn;        // grouped along the contraction: first k-block of the tile's expert and how many (>= 1)
};

// Position `d` k-blocks after k-block kb of the current tile (which has k0 k-blocks, the next one k1, every
// tile at least one): how many tiles further (0..2, d <= 2) and which k-block there.
__device__ __forceinline__ int tiles_ahead(int kb, int d, int k0, int k1, int& kb_out) {
  int pos = kb + d, q = 0;
  if (pos >= k0) {
    pos -= k0;
    q = 1;
    if (pos >= k1) { pos -= k1; q = 2; }
  }
  kb_out = pos;
  return q;
}

__device__ __forceinline__ TileInfo pick_tile(int q, TileInfo t0, TileInfo t1, TileInfo t2) {
  TileInfo r;
  r.row0 = q == 2 ? t2.row0 : (q == 1 ? t1.row0 : t0.row0);
  r.row_end = q == 2 ? t2.row_end : (q == 1 ? t1.row_end : t0.row_end);
  r.n0 = q == 2 ? t2.n0 : (q == 1 ? t1.n0 : t0.n0);
  r.expert = q == 2 ? t2.expert : (q == 1 ? t1.expert : t0.expert);
  r.kb0 = q == 2 ? t2.kb0 : (q == 1 ? t1.kb0 : t0.kb0);
  r.kbn = q == 2 ? t2.kbn : (q == 1 ? t1.kbn : t0.kbn);
  return r;
}

// End row of an expert as the kernel uses it: offsets that decrease or run past the row count (a
// malformed table) are clamped, so that every address derived from them stays inside a.
__device__ __forceinline__ int expert_end(int off, int prev, int total_rows) {
  const int lo = off > prev ? off : prev;
  return lo < total_rows ? lo : total_rows;
}

// SA4: the activation scales have unit stride over rows (the k-block-major layout), so a lane's four
// of them are one 16-byte load.
// EPI: 0 = c is the GEMM's result; 1 / 2 = the gate/up projection of a SwiGLU MLP with the activation and its
// 1x128 quantization as the epilogue (1: exactly specified silu, 2: hardware exponential and reciprocal).  A tile's
// 256 columns are then the 128 gate columns and the 128 up columns of one scaling group of the activation: the b
// tile's upper 128 rows come from `inter` rows further down, the two waves that share 64 rows hold gate and up.
template <int MODE, int GROUPED, bool OUT_F32, bool ACC, bool SA4, int EPI = 0>
__global__ __launch_bounds__(kGemmThreads) void gemm_kernel(const GemmParams p) {
  static_assert(EPI == 0 || ((MODE == kScaleBlock || MODE == kScalePow2) && GROUPED == kDense && !OUT_F32 && !ACC),
                "SwiGLU epilogue: dense block-scaled forward");
  static_assert(!ACC || (OUT_F32 && MODE != kScaleTensor), "accumulating onto c: fp32 output, sums that start from c's values");
  static_assert(GROUPED != kGroupedK || (!ACC && (MODE == kScaleRow || MODE == kScalePow2Row)),
                "grouped along the contraction: the wgrad form");
  constexpr int kBStages = b_stages(MODE);
  constexpr bool kRowScales = MODE == kScaleRow || MODE == kScalePow2Row;   // per-row b scales, staged in LDS
  constexpr bool kPromote = MODE == kScaleBlock || MODE == kScaleRow;       // partial sums scaled by FMAs
  constexpr bool kHwScale = MODE == kScalePow2 || MODE == kScalePow2Row;    // scales applied by the MFMA
  constexpr int kBAhead = kBStages - 1;     // k-blocks between issuing a b transfer and using it
  // One LDS object for everything.  (With a second __shared__ array the compiler tells the two apart
  // with alias scopes, and from then on makes every LDS read wait for all transfers into the array it
  // reads, those to other buffers included: the transfers' latency would be paid in every round.)
  __shared__ __attribute__((aligned(1024))) uint8_t lds[(2 + kBStages) * kTileBytes + (kRowScales ? 3 * BN * 4 : 0)];
  // per-row scales of the b operand for one k-block (wgrad form), three stages of 256 floats: the
  // stage of k-block kb+1 is filled while slower waves may still read that of kb-1
  float* const sb_lds = reinterpret_cast<float*>(lds + (2 + kBStages) * kTileBytes);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = p.K, N = p.N;
  const int kblocks = K / BK;
  const int tiles_n = (N + BN - 1) / BN;

  // ---- the tile list of this workgroup.  The grid is persistent (one workgroup per CU); tiles are
  // numbered so that consecutive numbers cover rectangles of 32 tiles (rect_map), each XCD (workgroup ids
  // congruent mod 8, own L2) owns a contiguous run of numbers, and the workgroups of an XCD walk
  // through that run side by side, so at any moment they work on one rectangle.
  int total_tiles = p.tiles;
  if (GROUPED == kGroupedK) total_tiles = p.experts * p.tiles;
  if (GROUPED == kGroupedRows) {
    // tiles are numbered expert by expert; an expert with no rows has none
    int prev = 0, mt = 0;
    for (int e = 0; e < p.experts; ++e) {
      const int end = expert_end(p.offs[e], prev, p.M);
      mt += (end - prev + BM - 1) / BM;
      prev = end;
    }
    total_tiles = mt * tiles_n;
  }
  int my_tiles, t_first, t_step;
  {
    const int nwg = gridDim.x, pid = blockIdx.x;
    const int xu = nwg < kXcds ? nwg : kXcds;        // the host launches a multiple of 8 workgroups, or fewer than 8
    const int xcd = pid % xu, slot = pid / xu;
    t_step = nwg / xu;
    const int base = total_tiles / xu, big = total_tiles % xu;
    const int cnt = base + (xcd < big ? 1 : 0);
    t_first = xcd * base + (xcd < big ? xcd : big) + slot;
    my_tiles = slot < cnt ? (cnt - slot + t_step - 1) / t_step : 0;
    if (GROUPED == kGroupedK) {
      // Tiles differ in length (an expert's contraction is its own token count) and are numbered longest expert
      // first.  They are dealt out in rounds of one tile per workgroup -- the XCD with index x takes positions
      // [x * t_step, (x + 1) * t_step) of every round, consecutive tiles as before -- so that every workgroup
      // gets the same mix of lengths and only the shortest tiles are left for the last, incomplete round.
      t_first = xcd * t_step + slot;
      t_step = nwg;
      my_tiles = t_first < total_tiles ? (total_tiles - t_first + nwg - 1) / nwg : 0;
    }
  }
  if (my_tiles == 0) return;
  const int n_pad = tiles_n * BN;
  // grouped: forward-only search state (tile numbers are asked for in increasing order)
  int g_e = 0, g_prev = 0, g_first = 0;
  auto lookup = [&](int k, TileInfo& ti) {
    int row0 = p.M, row_end = p.M, n0 = n_pad, expert = 0, kb0 = 0, kbn = GROUPED == kGroupedK ? 1 : kblocks;
    if (k < my_tiles) {
      const int t = t_first + k * t_step;
      int tm, tn;
      if (GROUPED == kGroupedK) {
        const int i = t / p.tiles;
        expert = p.layout[4 * p.experts + i];
        kb0 = p.layout[4 * expert + 2];
        kbn = p.layout[4 * expert + 3];
        rect_map(t - i * p.tiles, (p.M + BM - 1) / BM, tiles_n, tm, tn);
        row0 = tm * BM;
        row_end = row0 + BM < p.M ? row0 + BM : p.M;
        n0 = tn * BN;
      } else if (GROUPED == kGroupedRows) {
        int end = 0, cnt = 0;
        while (g_e < p.experts) {
          end = expert_end(p.offs[g_e], g_prev, p.M);
          cnt = (end - g_prev + BM - 1) / BM;
          if (t < g_first + cnt * tiles_n) break;
          g_first += cnt * tiles_n;
          g_prev = end;
          ++g_e;
        }
        if (g_e < p.experts) {
          rect_map(t - g_first, cnt, tiles_n, tm, tn);
          expert = g_e;
          row0 = g_prev + tm * BM;
          row_end = end < p.M ? end : p.M;
          if (row0 + BM < row_end) row_end = row0 + BM;
          n0 = tn * BN;
        }
      } else {
        rect_map(t, (p.M + BM - 1) / BM, tiles_n, tm, tn);
        row0 = tm * BM;
        row_end = row0 + BM < p.M ? row0 + BM : p.M;
        n0 = tn * BN;
      }
    }
    // (values found through the expert search sit in vector registers; as scalars they keep the
    // buffer resources built from them scalar too)
    ti.row0 = __builtin_amdgcn_readfirstlane(row0);
    ti.row_end = __builtin_amdgcn_readfirstlane(row_end);
    ti.n0 = __builtin_amdgcn_readfirstlane(n0);
    ti.expert = __builtin_amdgcn_readfirstlane(expert);
    ti.kb0 = __builtin_amdgcn_readfirstlane(kb0);
    ti.kbn = __builtin_amdgcn_readfirstlane(kbn);
  };
  // T0 is the tile being accumulated; transfers and scale loads run up to two k-blocks ahead and
  // so reach into T1 (and into T2 when K is a single k-block).
  TileInfo T0, T1, T2;
  lookup(0, T0);
  lookup(1, T1);
  lookup(2, T2);
  // ---- global -> LDS tile DMA.  One wave instruction moves 8 rows x 128 B (lane i -> LDS slot
  // i); the lane picks the 16-byte global chunk whose swizzled home is its slot.  The buffer
  // resource of a transfer starts at the tile's first row and ends with the tensor, so lane
  // offsets do not depend on the tile and rows past the end of the tensor read as zero.
  // (The resource runs on to the end of the tensor rather than to the end of the tile: transfers
  // through a resource that only just covers the rows they touch were measured markedly slower.  Rows
  // of a between the end of a ragged tile and the end of the tensor are read but never stored.)
  auto span_bytes = [&](int64_t rows, int64_t ld) {     // up to the end of the last row's K codes
    const int64_t bytes = rows > 0 ? (rows - 1) * ld + K : 0;
    return (int)(bytes < (int64_t)0x7FFFF000 ? bytes : (int64_t)0x7FFFF000);   // 256 rows always fit (host check)
  };
  auto rsrc_a_of = [&](const TileInfo& ti) {
    const int rows = ti.row_end > ti.row0 ? p.M - ti.row0 : 0;
    return __builtin_amdgcn_make_buffer_rsrc((void*)(p.a + (int64_t)ti.row0 * p.lda), 0, span_bytes(rows, p.lda),
                                             0x00020000);
  };
  auto rsrc_b_of = [&](const TileInfo& ti) {
    // (SwiGLU epilogue: the tile's first b row is gate row n0 / 2; its up rows lie `inter` rows further down)
    const int brow0 = EPI ? ti.n0 >> 1 : ti.n0;
    const int rows = N - ti.n0 > 0 ? N - brow0 : 0;
    const uint8_t* base = p.b + (GROUPED == kGroupedRows ? (int64_t)ti.expert * p.b_se : 0) + (int64_t)(rows ? brow0 : 0) * p.ldb;
    return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, span_bytes(rows, p.ldb), 0x00020000);
  };
  uint32_t a_off[4], b_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = wave * 4 + i;                       // 8-row group inside the tile
    const int r = q * 8 + (lane >> 3);                // row inside the tile
    const int chunk = (lane & 7) ^ row_swizzle(r);    // logical 16-byte chunk of that row
    // The rows of the a tile are permuted on their way into LDS: LDS row 64 w + 16 j + l holds tile row
    // 64 w + 4 l + j.  The lane that owns LDS rows 16 j + l16 (j = 0..3) of its wave's 64 then owns four
    // consecutive rows of a, whose scales are one 16-byte load and whose results are four adjacent
    // rows of c.  (The b tile keeps its order.)
    const int ra = (r & ~63) + (r & 15) * 4 + ((r >> 4) & 3);
    a_off[i] = (uint32_t)ra * (uint32_t)p.lda + chunk * 16;
    b_off[i] = (uint32_t)(EPI && r >= 128 ? r - 128 + p.inter : r) * (uint32_t)p.ldb + chunk * 16;
  }
  // wgrad form: the 256 per-row scales of the b tile for one k-block are one more 1 KB transfer
  // (wave 0), possible because that scale array is k-block-major (unit stride over rows).
  const __amdgpu_buffer_rsrc_t rsrc_sb = __builtin_amdgcn_make_buffer_rsrc(
      (void*)p.sb, 0, kRowScales ? (int)((((int64_t)kblocks - 1) * p.sb_sk + N) * 4) : 0, 0x00020000);
  auto issue_sb_load = [&](const TileInfo& ti, int kb, int stage) {      // kb counted inside the tile's own contraction
    if (kRowScales && wave == 0)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_sb, (lds_ptr_t)(sb_lds + stage * BN), 16,
                                               (uint32_t)(ti.n0 + lane * 4) * 4u,
                                               (int)(((GROUPED == kGroupedK ? ti.kb0 : 0) + kb) * p.sb_sk * 4), 0, 0);
  };
  // One transfer = 8 rows x 128 B per wave; `sub` (0..3) selects which of the wave's four 8-row groups
  // of the 256-row tile.  The four transfers of one operand tile share one LDS base (M0) and differ
  // in the instruction's immediate offset, which the hardware adds to both the LDS and the memory
  // address; the memory side is compensated in the lane offset.
  auto issue_tile = [&](const __amdgpu_buffer_rsrc_t& rs, const uint32_t (&off)[4], int buf, int kb, int sub) {
    uint8_t* sbase = lds + wave * 4096 + buf * kTileBytes;
    const uint32_t voff = off[sub] - sub * 1024;
    switch (sub) {   // the immediate must be a literal; sub is a compile-time constant after unrolling
      case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)sbase, 16, voff, kb * BK, 0, 0); break;
      case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)sbase, 16, voff, kb * BK, 1024, 0); break;
      case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)sbase, 16, voff, kb * BK, 2048, 0); break;
      default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)sbase, 16, voff, kb * BK, 3072, 0); break;
    }
  };

  // ---- fragment addressing
  const int wn = wave & 1, wm = wave >> 1;
  const int l16 = lane & 15, g = lane >> 4;
  const int pc0 = (2 * g) ^ row_swizzle(l16);
  const int a_frag_off = (wm * 64 + l16) * BK;               // + j * 16 rows
  const int b_frag_off = (wn * 128 + l16) * BK;               // + i * 16 rows, inside a b buffer

  // ---- scales.  Raw values for one k-block are loaded at the top of the round before it and only
  // combined (sa * sb) at its end, so nothing waits on global memory in between.
  // Both scale arrays are read through buffer resources with 32-bit byte offsets (the host checks
  // that they span less than 2 GiB): the row part of an offset is per tile, the k-block part a
  // scalar, so a round spends no vector arithmetic on addresses.
  const __amdgpu_buffer_rsrc_t rsrc_sa = __builtin_amdgcn_make_buffer_rsrc(
      (void*)p.sa, 0, MODE == kScaleTensor ? 4 : (int)((((int64_t)p.M - 1) * p.sa_sm + ((int64_t)kblocks - 1) * p.sa_sk + 1) * 4),
      0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_sbb = __builtin_amdgcn_make_buffer_rsrc((void*)p.sb, 0, p.sb_bytes, 0x00020000);
  uint32_t sa_voff[4];         // byte offset of this lane's four rows in sa (SA4: [0] covers all four)
  int sb_soff = 0;             // block form: byte offset of the b tile's scale row
  const int sa_kstep = (int)p.sa_sk * 4, sb_kstep = (int)p.sb_sk * 4;
  auto scale_target = [&](const TileInfo& ti) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = ti.row0 + wm * 64 + l16 * 4 + j;
      // (SA4 does not clamp: words past the end of the array read as zero, and rows past M are never stored)
      sa_voff[j] = SA4 ? (uint32_t)r * 4u : (uint32_t)(r < p.M ? r : p.M - 1) * (uint32_t)((int)p.sa_sm * 4);
    }
    int nblk_idx = EPI ? (ti.n0 >> 8) + wn * (p.inter >> 7) : (ti.n0 + wn * 128) >> 7;
    if (nblk_idx > (N >> 7) - 1) nblk_idx = (N >> 7) - 1;
    sb_soff = ((GROUPED == kGroupedRows ? ti.expert * (int)p.sb_se : 0) + nblk_idx * (int)p.sb_sn) * 4;
  };
  auto load_scales = [&](int kb, float raw[5]) {
    if (MODE == kScaleBlock || MODE == kScalePow2)
      raw[4] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_sbb, 0, sb_soff + kb * sb_kstep, 0));
    if (MODE != kScaleTensor) {
      if (SA4) {
        const v4f four = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc_sa, sa_voff[0], kb * sa_kstep, 0));
#pragma unroll
        for (int j = 0; j < 4; ++j) raw[j] = four[j];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          raw[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_sa, sa_voff[j], kb * sa_kstep, 0));
      }
    }
  };
  // kScalePow2: the exponent fields of the scales of the current k-block, which are their E8M0 codes:
  // e_a[j] for the activation rows j * 16 + l16 of this lane, e_b for the weight block
  int e_a[4] = {127, 127, 127, 127}, e_b = 127;
  auto combine_scales = [&](const float raw[5], float s[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) s[j] = MODE == kScaleBlock ? raw[j] * raw[4] : raw[j];
    if (kHwScale) {
#pragma unroll
      for (int j = 0; j < 4; ++j) e_a[j] = (int)(__builtin_bit_cast(uint32_t, raw[j]) >> 23);
      if (MODE == kScalePow2) e_b = (int)(__builtin_bit_cast(uint32_t, raw[4]) >> 23);
    }
  };

  // ---- accumulators.  When the result is added onto c (ACC), a tile's accumulators do not start from
  // zero but from the tile's old values, loaded right before its first round in the order in which
  // that round touches them: they cost no registers and only the first of them is waited for.  A
  // lane's four sums of one 16 x 16 subtile are four consecutive columns of one row: one 16-byte
  // load.  The resource ends with the tensor: rows past it (and the tiles past the end of the list)
  // read as zero.
  auto rsrc_c_of = [&](const TileInfo& ti) {
    const int ncol = ti.n0 + wn * 128;
    const bool ok = ti.row_end > ti.row0 && ncol < N;
    int64_t bytes = ok ? (((int64_t)p.M - ti.row0 - 1) * p.ldc + N - ncol) * 4 : 0;
    if (bytes > (int64_t)0x7FFFF000) bytes = 0x7FFFF000;       // 256 rows always fit (host check)
    const float* base = reinterpret_cast<const float*>(p.c) + (ok ? (int64_t)ti.row0 * p.ldc + ncol : 0);
    return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)bytes, 0x00020000);
  };
  const int c_jstep = (int)p.ldc * 4;                          // bytes between the rows of subtiles j and j + 1
  auto old_values = [&](const __amdgpu_buffer_rsrc_t& rs, uint32_t lane_off, int i, int j) {
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rs, lane_off + i * 64, j * c_jstep, 0));
  };
  const v4f zero = {0.f, 0.f, 0.f, 0.f};
  v4f acc[8][4];
  auto load_old_values = [&](const TileInfo& ti) {
    int lane_c = lane;
    asm volatile("" : "+v"(lane_c));    // (keeps the lane offset out of the registers held through the rounds)
    const __amdgpu_buffer_rsrc_t rc = rsrc_c_of(ti);
    const uint32_t c_lane = ((uint32_t)(wm * 64 + (lane_c & 15) * 4) * (uint32_t)p.ldc + (lane_c >> 4) * 4) * 4u;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = old_values(rc, c_lane, i, j);
  };
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = zero;

  // ---- prologue: k-block 0 of both operands, k-block 1 of b where it has three buffers, and the
  // first half of k-block 1 of a (and of b where it has two buffers)
  float s_cur[4] = {1.f, 1.f, 1.f, 1.f}, s_raw[5] = {1.f, 1.f, 1.f, 1.f, 1.f};
  // (k-block numbers passed to transfers and scale loads are absolute: grouped along the contraction, a tile's
  // own k-blocks start at its expert's first block kb0; otherwise kb0 is 0)
  auto kfirst = [](const TileInfo& ti) { return GROUPED == kGroupedK ? ti.kb0 : 0; };
  auto kcount = [&](const TileInfo& ti) { return GROUPED == kGroupedK ? ti.kbn : kblocks; };
  scale_target(T0);
  load_scales(kfirst(T0), s_raw);
  combine_scales(s_raw, s_cur);
  {
    const __amdgpu_buffer_rsrc_t ra = rsrc_a_of(T0), rb = rsrc_b_of(T0);
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) issue_tile(ra, a_off, 0, kfirst(T0), sub);
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) issue_tile(rb, b_off, 2, kfirst(T0), sub);
    int kb1;
    const TileInfo t1 = pick_tile(tiles_ahead(0, 1, kcount(T0), kcount(T1), kb1), T0, T1, T2);
    kb1 += kfirst(t1);
    if (kBAhead == 2) {
      const __amdgpu_buffer_rsrc_t rb1 = rsrc_b_of(t1);
#pragma unroll
      for (int sub = 0; sub < 4; ++sub) issue_tile(rb1, b_off, 3, kb1, sub);
    }
    issue_sb_load(T0, 0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    const __amdgpu_buffer_rsrc_t ra1 = rsrc_a_of(t1);
    issue_tile(ra1, a_off, 1, kb1, 0);
    issue_tile(ra1, a_off, 1, kb1, 1);
    if (kBAhead == 1) {
      const __amdgpu_buffer_rsrc_t rb1 = rsrc_b_of(t1);
      issue_tile(rb1, b_off, 3, kb1, 0);
      issue_tile(rb1, b_off, 3, kb1, 1);
    }
  }

  // The synchronisation point of a round sits before its last two n-subtiles, not at its end: what
  // follows the barrier (the weight fragments of the next round's first two subtiles, and the
  // activation fragments re-read one by one as the last subtile releases their registers) is then
  // covered by the matrix instructions still to be issued, and no round starts with every wave
  // waiting on LDS at once.  Fragments that cross the round boundary are carried in registers.
  // Rounds follow each other without a gap across tiles: the last rounds of a tile already fetch
  // the first k-blocks of the next one, and its stores drain while the next tile computes.
  v8i xf[4], wf_n0, wf_n1;
  wf_n0 = frag_read(lds + 2 * kTileBytes + b_frag_off, pc0);
#pragma unroll
  for (int j = 0; j < 4; ++j) xf[j] = frag_read(lds + a_frag_off + j * 16 * BK, pc0);
  wf_n1 = frag_read(lds + 2 * kTileBytes + b_frag_off + 16 * BK, pc0);

  constexpr bool kCarry = MODE == kScaleBlock;   // promote subtile 7 inside the next round's first group
  v4f part_c[4] = {zero, zero, zero, zero};
  float s_old[4] = {0.f, 0.f, 0.f, 0.f};
  int stage = 0;                       // a buffer holding the current k-block
  int bbuf = 0;                        // b buffer holding the current k-block
  int sbuf = 0;                        // scale stage (wgrad form) holding the current k-block
  // transfer targets (ordinal in the tile list) and their buffer resources
  int ord_1 = 0, ord_2 = 0;
  TileInfo tile_1 = T0;
  int kofs_2 = kfirst(T0);             // first k-block of the tile the transfers two ahead go to
  __amdgpu_buffer_rsrc_t rs_a1 = rsrc_a_of(T0), rs_a2 = rs_a1, rs_b1 = rsrc_b_of(T0), rs_b2 = rs_b1;

  // per-tensor form: the one multiplier of the store phase, read once (inside the tile loop the loads
  // would be repeated for every tile and waited for)
  float tensor_scale = 1.f;
  if (MODE == kScaleTensor) tensor_scale = p.sa[0] * p.sb[0];

  for (int tile = 0; tile < my_tiles; ++tile) {
  if (ACC) load_old_values(T0);
  const int kbn0 = kcount(T0);         // k-blocks of this tile
  for (int kb = 0; kb < kbn0; ++kb) {
    // Where this round's transfers and scale loads go: one k-block ahead (scales, second half of
    // those tiles), two ahead (first half of those tiles, or the whole b tile when it has three
    // buffers).  Only in the last
    // two rounds of a tile does a target move on to the next tile of the list; its resource is
    // rebuilt then and stays valid when that tile becomes the current one.
    int kb1 = kb + 1, kb2 = kb + 2;
    if (kb2 >= kbn0) {
      const int o1 = tile + tiles_ahead(kb, 1, kbn0, kcount(T1), kb1);
      const int o2 = tile + tiles_ahead(kb, 2, kbn0, kcount(T1), kb2);
      if (o1 != ord_1) {
        ord_1 = o1;
        tile_1 = pick_tile(o1 - tile, T0, T1, T2);
        rs_a1 = rsrc_a_of(tile_1);
        if (kBAhead == 1) rs_b1 = rsrc_b_of(tile_1);
        scale_target(tile_1);
      }
      if (o2 != ord_2) {
        ord_2 = o2;
        const TileInfo t2 = pick_tile(o2 - tile, T0, T1, T2);
        rs_a2 = rsrc_a_of(t2);
        rs_b2 = rsrc_b_of(t2);
        kofs_2 = kfirst(t2);
      }
    }
    const int kb1_rel = kb1;             // inside tile_1's own contraction (what issue_sb_load counts in)
    kb1 += kfirst(tile_1);
    kb2 += kofs_2;
    load_scales(kb1, s_raw);
    const uint8_t* bcur = lds + (2 + bbuf) * kTileBytes;
    int bnext = bbuf + 1 == kBStages ? 0 : bbuf + 1;           // holds the next k-block
    int bbuf_issue = bbuf + kBAhead;                           // receives the k-block kBAhead ahead
    if (bbuf_issue >= kBStages) bbuf_issue -= kBStages;
    const uint8_t* bnxt = lds + (2 + bnext) * kTileBytes;
    const uint8_t* anxt = lds + (stage ^ 1) * kTileBytes;
    int snext = sbuf + 1 == 3 ? 0 : sbuf + 1;
    // Per round, with three b buffers: the rest of the next a tile at subtiles 0,1; the b tile two
    // rounds ahead at 2..5; after the barrier the first half of the a tile after next, into the
    // buffer whose fragments every wave has just left behind.  One transfer per subtile: a burst
    // would queue up in the texture path ahead of the LDS reads.
    // With two b buffers (wgrad form) the b tile has to land within one round like the a tile, so
    // both go out in the four subtiles that follow the barrier, one transfer of each per subtile.
    auto issue_slot = [&](int i) {
      if (kBAhead == 2) {
        if (i < 2) issue_tile(rs_a1, a_off, stage ^ 1, kb1, i + 2);
        else if (i < 6) issue_tile(rs_b2, b_off, 2 + bbuf_issue, kb2, i - 2);
        else issue_tile(rs_a2, a_off, stage, kb2, i - 6);
      } else if (i < 2) {
        issue_tile(rs_a1, a_off, stage ^ 1, kb1, i + 2);
        issue_tile(rs_b1, b_off, 2 + bnext, kb1, i + 2);
      } else if (i >= 6) {
        issue_tile(rs_a2, a_off, stage, kb2, i - 6);
        issue_tile(rs_b2, b_off, 2 + bbuf, kb2, i - 6);
      }
    };
    auto round_sync = [&]() {
      // Own transfers for the next round have landed and own LDS reads of this round's buffers are
      // done; then everyone's.  With three b buffers the four b transfers of this round (the
      // youngest vector-memory operations) are for the round after next and may stay in flight.
      if (kBAhead == 2) __builtin_amdgcn_s_waitcnt(0x0074);  // vmcnt(4) lgkmcnt(0)
      else __builtin_amdgcn_s_waitcnt(0x0070);               // vmcnt(0) lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
    };
    // weight fragment of subtile i + 2 (the first two of the next round once past the barrier)
    auto read_ahead = [&](int i) {
      return i + 2 < 8 ? frag_read(bcur + b_frag_off + (i + 2) * 16 * BK, pc0)
                       : frag_read(bnxt + b_frag_off + (i + 2 - 8) * 16 * BK, pc0);
    };
    if (kPromote) {
      // Software pipeline over the 8 n-subtiles: the matrix instructions of subtile i are issued
      // interleaved with the promotion FMAs of subtile i-1, whose partial sums left the matrix
      // pipe four instructions earlier, so neither pipe waits for the other.
      v4f part[2][4];
      v8i wf[3];
      wf[0] = wf_n0;
      wf[1] = wf_n1;
#pragma unroll
      for (int j = 0; j < 4; ++j) part[1][j] = part_c[j];
      // wgrad form: the four per-row b scales of subtile i for this lane's four n
      const float* sb_row = sb_lds + sbuf * BN + wn * 128 + g * 4;
      v4f sbv[2];
      if (MODE == kScaleRow) sbv[0] = *reinterpret_cast<const v4f*>(sb_row);
      if (MODE == kScaleRow) issue_sb_load(tile_1, kb1_rel, snext);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (i == 6) round_sync();
        wf[(i + 2) % 3] = read_ahead(i);
        if (MODE == kScaleRow && i > 0) sbv[i & 1] = *reinterpret_cast<const v4f*>(sb_row + i * 16);   // used by the FMAs of group i+1
        issue_slot(i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          part[i & 1][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[i % 3], xf[j], zero, 0, 0, 0, 0, 0, 0);
          if (i > 0 || kCarry) {
            const int ip = (i + 7) & 7;     // subtile being promoted; for i = 0 the last one of the previous round
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float pv = part[(i - 1) & 1][j][r];
              if (MODE == kScaleRow) pv *= sbv[(i - 1) & 1][r];
              acc[ip][j][r] = __builtin_fmaf(pv, i == 0 ? s_old[j] : s_cur[j], acc[ip][j][r]);
            }
          }
          if (i == 7) xf[j] = frag_read(anxt + a_frag_off + j * 16 * BK, pc0);
          __builtin_amdgcn_sched_barrier(0);   // keep this (MFMA, FMAs) group together, in this order
        }
      }
      if (kCarry) {
#pragma unroll
        for (int j = 0; j < 4; ++j) part_c[j] = part[1][j];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float pv = part[1][j][r];
            if (MODE == kScaleRow) pv *= sbv[1][r];
            acc[7][j][r] = __builtin_fmaf(pv, s_cur[j], acc[7][j][r]);
          }
      }
      wf_n0 = wf[8 % 3];
      wf_n1 = wf[9 % 3];
    } else {
      v8i wf[3];
      wf[0] = wf_n0;
      wf[1] = wf_n1;
      // per-row b scales: this lane's row of subtile i is row i * 16 + l16 of the wave's 128
      const float* sb_lane = sb_lds + sbuf * BN + wn * 128 + l16;
      int e_bi[2] = {127, 127};
      if (MODE == kScalePow2Row) e_bi[0] = (int)(__builtin_bit_cast(uint32_t, sb_lane[0]) >> 23);
      if (MODE == kScalePow2Row) issue_sb_load(tile_1, kb1_rel, snext);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (i == 6) round_sync();
        wf[(i + 2) % 3] = read_ahead(i);
        if (MODE == kScalePow2Row && i < 7) e_bi[(i + 1) & 1] = (int)(__builtin_bit_cast(uint32_t, sb_lane[(i + 1) * 16]) >> 23);
        issue_slot(i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // (weights on the A port, activations on the B port: a lane's own row is the one it supplies
          // the scale of)
          if (kHwScale)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[i % 3], xf[j], acc[i][j], 0, 0, 0,
                                                                        MODE == kScalePow2 ? e_b : e_bi[i & 1], 0, e_a[j]);
          else
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[i % 3], xf[j], acc[i][j], 0, 0, 0, 0, 0, 0);
          if (i == 7) xf[j] = frag_read(anxt + a_frag_off + j * 16 * BK, pc0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      wf_n0 = wf[8 % 3];
      wf_n1 = wf[9 % 3];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; ++j) s_old[j] = s_cur[j];
    combine_scales(s_raw, s_cur);
    stage ^= 1;
    bbuf = bnext;
    sbuf = snext;
  }
  // ---- the tile is complete: last promotion, then its stores
  if (kCarry) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[7][j][r] = __builtin_fmaf(part_c[j][r], s_old[j], acc[7][j][r]);
#pragma unroll
    for (int j = 0; j < 4; ++j) part_c[j] = zero;
  }
  // The wave's 64 x 128 results go out 16 rows at a time (pass j: rows 4 s + j, s = 0..15, of the wave's
  // 64, the a tile's rows being permuted in LDS) through its own 4 KB slice of the b buffer
  // whose k-block was consumed last (nothing is in flight to that buffer, and this wave alone
  // transfers into this slice later), so that a store instruction writes whole rows of 256 bytes
  // instead of 16 pieces of 8 bytes.  The slice holds 16 rows x 256 B, 16-byte chunks XOR-ed with
  // the row so that both the fragment-order writes and the row-order reads spread over all banks.
  const int row0 = T0.row0, row_end = T0.row_end, n0 = T0.n0;
  // Lane coordinates re-derived behind an opaque copy: store addresses built from them would
  // otherwise be hoisted out of the tile loop and held in registers through the main loop.
  int lane_e = lane;
  asm volatile("" : "+v"(lane_e));
  const int l16e = lane_e & 15, ge = lane_e >> 4;
  uint8_t* stg = lds + (2 + (bbuf == 0 ? kBStages - 1 : bbuf - 1)) * kTileBytes + wave * 4096;
  // With two b buffers the lower half of that slice already receives the next transfers: rows 0..7
  // then go to its upper half and rows 8..15 to the upper half of this wave's slice of the a buffer
  // that is being refilled (its upper half is filled after these stores).
  uint8_t* stg_hi = kBAhead == 1 ? lds + (stage ^ 1) * kTileBytes + wave * 4096 + 2048 : stg + 2048;
  if (kBAhead == 1) stg += 2048;
  auto stg_row = [&](int row) { return (row < 8 ? stg : stg_hi) + (row & 7) * 256; };   // (row = l16e: the write side)
  const int ncol = n0 + wn * 128;                 // first column of the wave tile
  const bool cols_ok = ncol < N;
  constexpr int kHalves = OUT_F32 ? 2 : 1;       // fp32 rows of 128 columns take two slices
  constexpr int kPerHalf = 8 / kHalves;           // n-subtiles per slice
  const uint32_t stg_w = (uint32_t)(uintptr_t)(lds_ptr_t)stg_row(l16e);   // LDS byte address of this lane's row
  // Rows leave through a buffer resource that starts at the wave tile's first element and ends with the
  // tile's last valid row: the lane part of a store address is one offset computed once per tile, the
  // rest scalar, and rows past the end of a ragged tile (or of an expert) are dropped by the range check.
  constexpr int kEsize = OUT_F32 ? 4 : 2;
  const int rows_valid = row_end - row0 < BM ? row_end - row0 : BM;
  const __amdgpu_buffer_rsrc_t rsrc_st = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(reinterpret_cast<uint8_t*>(p.c) +
              ((int64_t)row0 * p.ldc + ncol + (GROUPED == kGroupedK ? (int64_t)T0.expert * p.c_se : 0)) * kEsize), 0,
      cols_ok && rows_valid > 0 ? (int)((((int64_t)rows_valid - 1) * p.ldc + 128) * kEsize) : 0, 0x00020000);
  const uint32_t st_lane = (uint32_t)(((wm * 64 + ge * 4) * (int)p.ldc) * kEsize + l16e * 16);
  const int st_row = (int)p.ldc * kEsize;        // bytes from one row of c to the next
  auto store_tile = [&](auto with_bias) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int h = 0; h < kHalves; ++h) {
#pragma unroll
        for (int ii = 0; ii < kPerHalf; ++ii) {
          const int i = h * kPerHalf + ii;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            v[r] = acc[i][j][r];
            if (MODE == kScaleTensor) v[r] *= tensor_scale;
          }
          if (decltype(with_bias)::value) {
            const uint2 braw = *reinterpret_cast<const uint2*>(p.bias + ncol + i * 16 + ge * 4);
            v[0] += bf16lo(braw.x); v[1] += bf16hi(braw.x); v[2] += bf16lo(braw.y); v[3] += bf16hi(braw.y);
          }
          // The staging writes are issued as bare instructions: the compiler would otherwise make
          // every LDS store wait for the tile transfers in flight (to other buffers) to land.
          if (OUT_F32) {
            const v4f o = {v[0], v[1], v[2], v[3]};
            asm volatile("ds_write_b128 %0, %1" ::"v"(stg_w + (((ii * 4 + ge) ^ l16e) * 16)), "v"(o) : "memory");
          } else {
            u32x2 o;
            o[0] = pack_bf16x2(v[0], v[1]);
            o[1] = pack_bf16x2(v[2], v[3]);
            asm volatile("ds_write_b64 %0, %1" ::"v"(stg_w + (((ii * 2 + (ge >> 1)) ^ l16e) * 16) + (ge & 1) * 8), "v"(o)
                         : "memory");
          }
          acc[i][j] = zero;
        }
#pragma unroll
        for (int k2 = 0; k2 < 4; k2 += 2) {      // two rows per lane at a time (registers are scarce here)
          v4i val[2];
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            // staging row 4 (k2 + k) + ge; which half of the staging area it lies in does not depend on the lane
            const int row = 4 * (k2 + k) + ge;
            const uint8_t* half = (k2 + k) < 2 ? stg : stg_hi;
            val[k] = *reinterpret_cast<const v4i*>(half + (4 * ((k2 + k) & 1) + ge) * 256 + ((l16e ^ row) * 16));
          }
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            // staging row s of pass j is tile row 4 s + j (s = 4 (k2 + k) + ge: the ge part is in st_lane).
            // Streaming stores: the output is not read again here, and as ordinary stores a tile's
            // 128-256 KB would push operand panels out of the L2.
            __builtin_amdgcn_raw_buffer_store_b128(val[k], rsrc_st, st_lane, (16 * (k2 + k) + j) * st_row + h * 256, 2);
          }
        }
      }
    }
  };
  if constexpr (EPI != 0) {
    // SwiGLU epilogue.  Per pass j (16 of the wave's 64 rows) both waves of a pair write their bf16-rounded
    // results -- gate from the wave with wn = 0, up from its neighbour -- into their staging slices as for a plain
    // store; after a barrier each wave of the pair takes 8 of the 16 rows, reads gate and up of a row from the two
    // slices (16 lanes x 8 columns: one scaling group of the activation), and computes, quantizes and stores
    // the activation exactly as the stand-alone kernel does on a bf16 gate/up tensor.  A second barrier keeps the
    // next pass's writes (and, after the last pass, the next tile's transfers) off slices still being read.
    static_assert(kBStages == 3, "staging rows 0..15 of a wave are contiguous");
    const uint8_t* gate_s = stg - wave * 4096 + (wave & ~1) * 4096;
    const uint8_t* up_s = gate_s + 4096;
    const uint32_t stg_we = (uint32_t)(uintptr_t)(lds_ptr_t)(stg + l16e * 256);   // this lane's staging row
    const int gcol = n0 >> 1;                        // first activation column of the tile's scaling group
    const __amdgpu_buffer_rsrc_t rsrc_q = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(reinterpret_cast<uint8_t*>(p.c) + (int64_t)row0 * p.ldc + gcol), 0,
        rows_valid > 0 ? (int)(((int64_t)rows_valid - 1) * p.ldc + 128) : 0, 0x00020000);
    const int64_t s_first = (int64_t)(n0 >> 8) * p.M + row0;
    const __amdgpu_buffer_rsrc_t rsrc_si = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(p.q_scale_inv + s_first), 0, rows_valid > 0 ? rows_valid * 4 : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_sc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(p.q_scale ? p.q_scale + s_first : p.q_scale_inv), 0, p.q_scale && rows_valid > 0 ? rows_valid * 4 : 0,
        0x00020000);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int ii = 0; ii < 8; ++ii) {
        u32x2 o;
        o[0] = pack_bf16x2(acc[ii][j][0], acc[ii][j][1]);
        o[1] = pack_bf16x2(acc[ii][j][2], acc[ii][j][3]);
        asm volatile("ds_write_b64 %0, %1" ::"v"(stg_we + (((ii * 2 + (ge >> 1)) ^ l16e) * 16) + (ge & 1) * 8), "v"(o)
                     : "memory");
        acc[ii][j] = zero;
      }
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
      for (int it = 0; it < 2; ++it) {
        const int srow = 8 * wn + 4 * it + ge;                   // staging row: tile row wm * 64 + 4 * srow + j
        const int soff = srow * 256 + ((l16e ^ srow) * 16);
        const v4i gv = *reinterpret_cast<const v4i*>(gate_s + soff);
        const v4i uv = *reinterpret_cast<const v4i*>(up_s + soff);
        uint4 a;
        a.x = swiglu2<EPI == 2>((uint32_t)gv[0], (uint32_t)uv[0]);
        a.y = swiglu2<EPI == 2>((uint32_t)gv[1], (uint32_t)uv[1]);
        a.z = swiglu2<EPI == 2>((uint32_t)gv[2], (uint32_t)uv[2]);
        a.w = swiglu2<EPI == 2>((uint32_t)gv[3], (uint32_t)uv[3]);
        const uint32_t m = row16_max_u32(mag8(a));
        float sc, sci;
        scales_from_amax(__uint_as_float(m << 16), sc, sci, p.pow2_out);
        const uint2 codes = cvt8<false>(a, sc);
        const int trow = wm * 64 + 4 * srow + j;
        u32x2 cw = {codes.x, codes.y};
        __builtin_amdgcn_raw_buffer_store_b64(cw, rsrc_q, (uint32_t)trow * (uint32_t)p.ldc + l16e * 8, 0, 2);
        if (l16e == 0) {
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(sci), rsrc_si, trow * 4, 0, 0);
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(sc), rsrc_sc, trow * 4, 0, 0);
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
  } else if (cols_ok) {
    if (!p.bias) store_tile(std::false_type{});
    else store_tile(std::true_type{});
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i][j] = zero;
  }
  T0 = T1;
  T1 = T2;
  lookup(tile + 3, T2);
  }

  // Transfers issued past the end of the list (they fetch nothing) still target this workgroup's
  // LDS: drain them before the LDS can be handed to another workgroup.
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
}

// ---------------------------------------------------------------------------------------------
// small problems: fewer 256 x 256 tiles than compute units
// ---------------------------------------------------------------------------------------------
// One 128 x 128 output tile per workgroup of 4 waves (2 x 2, wave tile 64 x 64), no persistence: four times as
// many workgroups as the kernel above has tiles, each with a quarter of the matrix work per k-block.  Same
// operand layout in LDS (global -> LDS transfers, swizzle, fragment reads), five stages of one a tile and one b
// tile (16 KB each), transfers four k-blocks ahead, one barrier per k-block.  Same arithmetic in the same order as
// the kernel above (one matrix instruction per 16 x 16 subtile and k-block; block form: acc += partial * (sa * sb)),
// so the two give identical results.  Per-tensor and 128x128-block scale forms, dense, bf16 or fp32 output, bias.
constexpr int kSmallThreads = 256;
constexpr int kSmallTile = 128;
constexpr int kSmallStages = 5;

// TM: rows of the tile, 128 or 64.  With 64 (wave tile 32 x 64) a problem has twice as many workgroups: the form for
// problems whose 128 x 128 tiles would leave compute units idle (cfg 1: 128 tiles on 256 compute units).
template <int MODE, bool OUT_F32, int TM = 128>
__global__ __launch_bounds__(kSmallThreads) void gemm_small_kernel(const GemmParams p) {
  static_assert(MODE == kScaleTensor || MODE == kScaleBlock, "per-tensor or block scales");
  static_assert(TM == 128 || TM == 64, "tile rows");
  constexpr int kStageBytes = (TM + kSmallTile) * BK;     // a tile + b tile
  constexpr int NA = TM / 32;                             // a transfers per wave and k-block; also m-subtiles per wave
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kSmallStages * kStageBytes];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 1, wm = wave >> 1;
  const int l16 = lane & 15, g = lane >> 4;
  const int kblocks = p.K / BK;
  const int tiles_n = p.N / kSmallTile;
  const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
  const int row0 = tm * TM, n0 = tn * kSmallTile;
  const int rows_valid = p.M - row0 < TM ? p.M - row0 : TM;

  // transfers: as in gemm_kernel, a wave moves 8 rows x 128 B per instruction, four per operand tile and k-block;
  // the resources start at the tile's first row and end with the tensor (rows past it read as zero); k-blocks
  // past the end go through an empty resource and fetch nothing
  auto span = [&](int64_t rows, int64_t ld) {
    const int64_t bytes = rows > 0 ? (rows - 1) * ld + p.K : 0;
    return (int)(bytes < (int64_t)0x7FFFF000 ? bytes : (int64_t)0x7FFFF000);
  };
  const __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc((void*)(p.a + (int64_t)row0 * p.lda), 0,
                                                                      span(p.M - row0, p.lda), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc((void*)(p.b + (int64_t)n0 * p.ldb), 0,
                                                                      span(p.N - n0, p.ldb), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_none = __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, 0, 0x00020000);
  uint32_t a_off[4], b_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = (wave * 4 + i) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ row_swizzle(r);
    b_off[i] = (uint32_t)r * (uint32_t)p.ldb + chunk * 16 - i * 1024;
    const int ra = (wave * NA + (i < NA ? i : 0)) * 8 + (lane >> 3);
    const int chunk_a = (lane & 7) ^ row_swizzle(ra);
    a_off[i] = (uint32_t)ra * (uint32_t)p.lda + chunk_a * 16 - (i < NA ? i : 0) * 1024;
  }
  auto issue_stage = [&](int kb, int stage) {
    const bool ok = kb < kblocks;
    const __amdgpu_buffer_rsrc_t ra = ok ? rs_a : rs_none, rb = ok ? rs_b : rs_none;
    uint8_t* sa_base = lds + stage * kStageBytes + wave * (NA * 1024);
    uint8_t* sb_base = lds + stage * kStageBytes + TM * BK + wave * 4096;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)sa_base, 16, a_off[0], kb * BK, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)sa_base, 16, a_off[1], kb * BK, 1024, 0);
    if (NA == 4) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)sa_base, 16, a_off[2], kb * BK, 2048, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)sa_base, 16, a_off[3], kb * BK, 3072, 0);
    }
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)sb_base, 16, b_off[0], kb * BK, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)sb_base, 16, b_off[1], kb * BK, 1024, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)sb_base, 16, b_off[2], kb * BK, 2048, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)sb_base, 16, b_off[3], kb * BK, 3072, 0);
  };
  const int pc0 = (2 * g) ^ row_swizzle(l16);
  const int a_frag = (wm * (TM / 2) + l16) * BK, b_frag = TM * BK + (wn * 64 + l16) * BK;

  // scales of the block form: this lane's four rows of a (clamped: rows past M are never stored), the tile's
  // one 128-row block of b
  const float* sa_row[NA];
#pragma unroll
  for (int j = 0; j < NA; ++j) {
    const int r = row0 + wm * (TM / 2) + j * 16 + l16;
    sa_row[j] = p.sa + (int64_t)(r < p.M ? r : p.M - 1) * p.sa_sm;
  }
  const float* sb_blk = p.sb + (int64_t)(n0 >> 7) * p.sb_sn;

  const v4f zero = {0.f, 0.f, 0.f, 0.f};
  v4f acc[4][NA];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NA; ++j) acc[i][j] = zero;

  // Transfers run four k-blocks ahead (five stages); the block form's scales are fetched three k-blocks ahead
  // into a ring of registers, so that waiting for them never waits for a transfer that is not needed yet
  // (vector-memory operations complete in order).  Issue order per iteration i: wait + barrier, scale loads of
  // k-block i + 3, transfers of k-block i + 4.
  float s_ring[4][5];
  auto load_scales = [&](int kb, float raw[5]) {
    if (MODE == kScaleBlock) {
      const int kk = kb < kblocks ? kb : kblocks - 1;
      raw[4] = sb_blk[(int64_t)kk * p.sb_sk];
#pragma unroll
      for (int j = 0; j < NA; ++j) raw[j] = sa_row[j][(int64_t)kk * p.sa_sk];
    }
  };
  issue_stage(0, 0);
  load_scales(0, s_ring[0]);
  issue_stage(1, 1);
  load_scales(1, s_ring[1]);
  issue_stage(2, 2);
  load_scales(2, s_ring[2]);
  issue_stage(3, 3);
  int st = 0, st_issue = 4;
  // one k-block; Q = kb % 4 is the ring slot that holds its scales (static, so the ring needs no register moves:
  // a move would have to wait for the load it moves)
  auto k_block = [&](int kb, auto q_tag) {
    constexpr int Q = decltype(q_tag)::value;
    // all but the youngest transfers of three k-blocks (and, block form, the scale loads issued between them)
    // have landed: this k-block's tiles of this wave; after the barrier everyone's, and everyone has left the
    // stage that is refilled next
    // (in flight and allowed to stay so: the transfers of three k-blocks, NA + 4 each, and in the block form the scale
    // loads of two, NA + 1 each)
    if (MODE == kScaleBlock && NA == 4) asm volatile("s_waitcnt vmcnt(34)\n\ts_barrier" ::: "memory");
    else if (MODE == kScaleBlock) asm volatile("s_waitcnt vmcnt(24)\n\ts_barrier" ::: "memory");
    else if (NA == 4) asm volatile("s_waitcnt vmcnt(24)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(18)\n\ts_barrier" ::: "memory");
    load_scales(kb + 3, s_ring[(Q + 3) & 3]);
    asm volatile("" ::: "memory");       // (keeps the scale loads ahead of the transfers, as the wait above counts them)
    issue_stage(kb + 4, st_issue);
    const uint8_t* base = lds + st * kStageBytes;
    st = st == kSmallStages - 1 ? 0 : st + 1;
    st_issue = st_issue == kSmallStages - 1 ? 0 : st_issue + 1;
    v8i xf[NA], wf[4];
#pragma unroll
    for (int j = 0; j < NA; ++j) xf[j] = frag_read(base + a_frag + j * 16 * BK, pc0);
#pragma unroll
    for (int i = 0; i < 4; ++i) wf[i] = frag_read(base + b_frag + i * 16 * BK, pc0);
    if (MODE == kScaleTensor) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NA; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[i], xf[j], acc[i][j], 0, 0, 0, 0, 0, 0);
    } else {
      v4f part[4][NA];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NA; ++j)
          part[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[i], xf[j], zero, 0, 0, 0, 0, 0, 0);
      float s[NA];
#pragma unroll
      for (int j = 0; j < NA; ++j) s[j] = s_ring[Q][j] * s_ring[Q][4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NA; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][j][r] = __builtin_fmaf(part[i][j][r], s[j], acc[i][j][r]);
    }
  };
  for (int kb = 0; kb < kblocks; kb += 4) {
    k_block(kb, std::integral_constant<int, 0>{});
    if (kb + 1 < kblocks) k_block(kb + 1, std::integral_constant<int, 1>{});
    if (kb + 2 < kblocks) k_block(kb + 2, std::integral_constant<int, 2>{});
    if (kb + 3 < kblocks) k_block(kb + 3, std::integral_constant<int, 3>{});
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // the transfers past the last k-block (they fetch nothing) still target this LDS

  // store: a lane holds, per subtile, four consecutive columns of one row
  float tensor_scale = 1.f;
  if (MODE == kScaleTensor) tensor_scale = p.sa[0] * p.sb[0];
#pragma unroll
  for (int j = 0; j < NA; ++j) {
    const int r = wm * (TM / 2) + j * 16 + l16;
    if (r >= rows_valid) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = n0 + wn * 64 + i * 16 + g * 4;
      float v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        v[q] = acc[i][j][q];
        if (MODE == kScaleTensor) v[q] *= tensor_scale;
      }
      if (p.bias) {
        const uint2 braw = *reinterpret_cast<const uint2*>(p.bias + col);
        v[0] += bf16lo(braw.x); v[1] += bf16hi(braw.x); v[2] += bf16lo(braw.y); v[3] += bf16hi(braw.y);
      }
      const int64_t o = (int64_t)(row0 + r) * p.ldc + col;
      if (OUT_F32) {
        *reinterpret_cast<v4f*>(reinterpret_cast<float*>(p.c) + o) = v4f{v[0], v[1], v[2], v[3]};
      } else {
        u32x2 w2;
        w2[0] = pack_bf16x2(v[0], v[1]);
        w2[1] = pack_bf16x2(v[2], v[3]);
        *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(p.c) + o) = w2;
      }
    }
  }
}

// 0: the small-tile kernel serves problems with fewer 256 x 256 tiles than half the compute units (and more
// 128 x 128 tiles than that); 1: never; 2: whenever its forms allow (test hook)
static std::atomic<int> g_small_gemm_mode{0};   // (atomic: the test hook may be called from any thread)

// Workgroups to launch for `tiles` tiles: one per CU, a multiple of 8 (one share per XCD) unless
// there are fewer than 8 tiles.
static int persistent_grid(int64_t tiles) {
  static const int cus = [] {           // (initialised once, also when the first calls come from several threads)
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  int64_t g = tiles < cus ? tiles : cus;
  if (g >= kXcds) g -= g % kXcds;
  return (int)g;
}

static bool use_small_kernel(int64_t M, int64_t N) {
  const int mode = g_small_gemm_mode.load(std::memory_order_relaxed);
  if (mode == 1) return false;
  if (mode == 2) return true;
  const int64_t big = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  const int64_t small = ((M + kSmallTile - 1) / kSmallTile) * (N / kSmallTile);
  const int cus = persistent_grid((int64_t)1 << 40);
  return 2 * big < cus && small > big && small < (int64_t)0x7FFFFFFF;
}

template <int MODE>
static int launch_small(const GemmParams& p, int out_type, hipStream_t stream) {
  const int64_t tiles = (((int64_t)p.M + kSmallTile - 1) / kSmallTile) * (p.N / kSmallTile);
  dim3 block(kSmallThreads);
  // fewer 128 x 128 tiles than compute units: tiles of 64 rows, twice as many workgroups (the same results)
  if (tiles < persistent_grid((int64_t)1 << 40)) {
    dim3 grid((unsigned)((((int64_t)p.M + 63) / 64) * (p.N / kSmallTile)));
    if (out_type == HPFP8_OUT_F32) gemm_small_kernel<MODE, true, 64><<<grid, block, 0, stream>>>(p);
    else gemm_small_kernel<MODE, false, 64><<<grid, block, 0, stream>>>(p);
    return check_launch("gemm (small tiles)");
  }
  dim3 grid((unsigned)tiles);
  if (out_type == HPFP8_OUT_F32) gemm_small_kernel<MODE, true><<<grid, block, 0, stream>>>(p);
  else gemm_small_kernel<MODE, false><<<grid, block, 0, stream>>>(p);
  return check_launch("gemm (small tiles)");
}

template <int MODE, int GROUPED, bool SA4>
static int launch_sa(const GemmParams& p, int out_type, int64_t tiles, hipStream_t stream) {
  dim3 grid((unsigned)persistent_grid(tiles)), block(kGemmThreads);
  if (out_type == HPFP8_OUT_F32) {
    if constexpr (MODE != kScaleTensor && GROUPED == kDense) {   // (the per-tensor and grouped entry points have no accumulate)
      if (p.accumulate) {
        gemm_kernel<MODE, GROUPED, true, true, SA4><<<grid, block, 0, stream>>>(p);
        return check_launch("gemm");
      }
    }
    gemm_kernel<MODE, GROUPED, true, false, SA4><<<grid, block, 0, stream>>>(p);
  } else {
    gemm_kernel<MODE, GROUPED, false, false, SA4><<<grid, block, 0, stream>>>(p);
  }
  return check_launch("gemm");
}

template <int MODE, int GROUPED>
static int launch(const GemmParams& p, int out_type, int64_t tiles, hipStream_t stream) {
  if constexpr (MODE != kScaleTensor) {
    if (p.sa_sm == 1) return launch_sa<MODE, GROUPED, true>(p, out_type, tiles, stream);
  }
  return launch_sa<MODE, GROUPED, false>(p, out_type, tiles, stream);
}

static int check_common(const char* what, const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                        const float* sb, int64_t M, int64_t N, int64_t K, const void* bias, const void* c,
                        int64_t ldc, int out_type, int accumulate) {
  HPFP8_REQUIRE(M >= 0 && N >= 0 && K >= 0, HPFP8_ERR_SHAPE, "%s: negative shape", what);
  HPFP8_REQUIRE(K > 0 && K % BK == 0 && N % kBlock == 0, HPFP8_ERR_SHAPE,
                "%s: K=%lld must be a positive multiple of 128 and N=%lld a multiple of 128", what, (long long)K,
                (long long)N);
  HPFP8_REQUIRE(out_type == HPFP8_OUT_BF16 || out_type == HPFP8_OUT_F32, HPFP8_ERR_ARG, "%s: bad out_type", what);
  HPFP8_REQUIRE(!accumulate || out_type == HPFP8_OUT_F32, HPFP8_ERR_ARG, "%s: accumulate needs fp32 output", what);
  HPFP8_REQUIRE(lda >= K && ldb >= K && lda % 16 == 0 && ldb % 16 == 0, HPFP8_ERR_SHAPE,
                "%s: lda=%lld and ldb=%lld must be multiples of 16 and at least K=%lld", what, (long long)lda,
                (long long)ldb, (long long)K);
  HPFP8_REQUIRE(ldc >= N, HPFP8_ERR_SHAPE, "%s: ldc=%lld smaller than N=%lld", what, (long long)ldc, (long long)N);
  // rows of c are written in 16-byte pieces
  HPFP8_REQUIRE(ldc % (out_type == HPFP8_OUT_F32 ? 4 : 8) == 0, HPFP8_ERR_ALIGN,
                "%s: ldc must be a multiple of %d", what, out_type == HPFP8_OUT_F32 ? 4 : 8);
  if (M == 0 || N == 0) return HPFP8_OK;
  HPFP8_REQUIRE(a && b && sa && sb && c, HPFP8_ERR_ARG, "%s: null buffer", what);
  HPFP8_REQUIRE(aligned16(a) && aligned16(b) && aligned16(c) && (!bias || aligned16(bias)), HPFP8_ERR_ALIGN,
                "%s: buffers must be 16-byte aligned", what);
  // 32-bit byte offsets inside one tile's buffer resource (256 rows); the operands themselves may be
  // of any size
  HPFP8_REQUIRE(BM * lda < (int64_t)0x7FFFFFFF && BN * ldb < (int64_t)0x7FFFFFFF, HPFP8_ERR_SHAPE,
                "%s: a row stride of 8 MiB or more is not supported", what);
  HPFP8_REQUIRE(M < (int64_t)0x7FFFFF00 && N < (int64_t)0x7FFFFF00, HPFP8_ERR_SHAPE, "%s: M or N too large", what);
  // a tile's 256 rows of c are stored (and its old values read) with 32-bit byte offsets
  HPFP8_REQUIRE(BM * ldc * 4 < (int64_t)0x7FFFF000, HPFP8_ERR_SHAPE, "%s: the row stride of c must stay below 8 MiB", what);
  return 1;
}

// Scale arrays are addressed with 32-bit byte offsets inside the kernels.
static int check_scale_span(const char* what, int64_t rows, int64_t kblocks, int64_t stride_r, int64_t stride_k,
                            const char* name) {
  HPFP8_REQUIRE(stride_r >= 0 && stride_k >= 0, HPFP8_ERR_SHAPE, "%s: negative %s stride", what, name);
  if (rows == 0) return 1;
  HPFP8_REQUIRE(((rows - 1) * stride_r + (kblocks - 1) * stride_k + 1) * 4 < (int64_t)0x7FFFFFFF, HPFP8_ERR_SHAPE,
                "%s: the %s array spans 2 GiB or more", what, name);
  return 1;
}

}  // namespace hpfp8

using namespace hpfp8;

extern "C" {

static int gemm_blockwise_impl(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                               const void* b, int64_t ldb, const float* sb, int64_t sb_stride_n, int64_t sb_stride_k,
                               int sb_gran, int64_t M, int64_t N, int64_t K, const void* bias, void* c,
                               int64_t ldc, int out_type, int accumulate, bool pow2, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(sb_gran == 1 || sb_gran == 128, HPFP8_ERR_ARG, "gemm_blockwise: sb_gran must be 1 or 128");
  int rc = check_common("gemm_blockwise", a, lda, b, ldb, sa, sb, M, N, K, bias, c, ldc, out_type, accumulate);
  if (rc <= 0) return rc;
  GemmParams p{};
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.sa = sa; p.sb = sb; p.lda = lda; p.ldb = ldb;
  p.sa_sm = sa_stride_m; p.sa_sk = sa_stride_k; p.sb_sn = sb_stride_n; p.sb_sk = sb_stride_k;
  rc = check_scale_span("gemm_blockwise", M, K / BK, sa_stride_m, sa_stride_k, "sa");
  if (rc <= 0) return rc;
  rc = check_scale_span("gemm_blockwise", sb_gran == 128 ? N / kBlock : N, K / BK, sb_stride_n, sb_stride_k, "sb");
  if (rc <= 0) return rc;
  p.sb_bytes = (int)(((N / kBlock - 1) * sb_stride_n + (K / BK - 1) * sb_stride_k + 1) * 4);
  p.c = c; p.ldc = ldc; p.bias = (const uint16_t*)bias;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.accumulate = accumulate;
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  p.tiles = (int)tiles;
  if (sb_gran == 128) {
    if (pow2) return launch<kScalePow2, kDense>(p, out_type, tiles, (hipStream_t)stream);
    if (!accumulate && use_small_kernel(M, N)) return launch_small<kScaleBlock>(p, out_type, (hipStream_t)stream);
    return launch<kScaleBlock, kDense>(p, out_type, tiles, (hipStream_t)stream);
  }
  // per-row b scales travel to LDS as one contiguous 1 KB piece per k-block
  if (K == BK) sb_stride_k = N;     // a single k-block: the stride between k-blocks is never used
  p.sb_sk = sb_stride_k;
  HPFP8_REQUIRE(sb_stride_n == 1 && sb_stride_k >= N && sb_stride_k % 4 == 0 && aligned16(sb), HPFP8_ERR_SHAPE,
                "gemm_blockwise: with sb_gran=1 the b scales must be k-block-major (sb_stride_n = 1, sb_stride_k >= N, "
                "16-byte aligned rows)");
  HPFP8_REQUIRE(((K / BK - 1) * sb_stride_k + N) * 4 < (int64_t)0x7FFFFFFF, HPFP8_ERR_SHAPE,
                "gemm_blockwise: b scale array too large");
  if (pow2) return launch<kScalePow2Row, kDense>(p, out_type, tiles, (hipStream_t)stream);
  return launch<kScaleRow, kDense>(p, out_type, tiles, (hipStream_t)stream);
}

int hpfp8_gemm_blockwise(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                         const void* b, int64_t ldb, const float* sb, int64_t sb_stride_n, int64_t sb_stride_k,
                         int sb_gran, int64_t M, int64_t N, int64_t K, const void* bias, void* c,
                         int64_t ldc, int out_type, int accumulate, hpfp8_stream_t stream) {
  return gemm_blockwise_impl(a, lda, sa, sa_stride_m, sa_stride_k, b, ldb, sb, sb_stride_n, sb_stride_k, sb_gran, M, N, K,
                             bias, c, ldc, out_type, accumulate, false, stream);
}

int hpfp8_gemm_blockwise_pow2(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                              const void* b, int64_t ldb, const float* sb, int64_t sb_stride_n, int64_t sb_stride_k,
                              int sb_gran, int64_t M, int64_t N, int64_t K, const void* bias, void* c, int64_t ldc,
                              int out_type, int accumulate, hpfp8_stream_t stream) {
  return gemm_blockwise_impl(a, lda, sa, sa_stride_m, sa_stride_k, b, ldb, sb, sb_stride_n, sb_stride_k, sb_gran, M, N, K,
                             bias, c, ldc, out_type, accumulate, true, stream);
}

int hpfp8_gemm_blockwise_swiglu_quantize(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m,
                                         int64_t sa_stride_k, const void* b, int64_t ldb, const float* sb,
                                         int64_t sb_stride_n, int64_t sb_stride_k, int64_t M, int64_t inter, int64_t K,
                                         int fast, int pow2, int pow2_out, void* q, int64_t ldq, float* scale,
                                         float* scale_inv, hpfp8_stream_t stream) {
  const char* what = "gemm_blockwise_swiglu_quantize";
  HPFP8_REQUIRE((fast == 0 || fast == 1) && (pow2 == 0 || pow2 == 1) && (pow2_out == 0 || pow2_out == 1), HPFP8_ERR_ARG,
                "%s: fast, pow2 and pow2_out must be 0 or 1", what);
  HPFP8_REQUIRE(inter >= 0 && inter % kBlock == 0 && inter < (1 << 29), HPFP8_ERR_SHAPE,
                "%s: the activation's width %lld must be a multiple of 128", what, (long long)inter);
  HPFP8_REQUIRE(ldq >= inter && ldq % 16 == 0, HPFP8_ERR_SHAPE, "%s: ldq=%lld must be a multiple of 16 and at least the width",
                what, (long long)ldq);
  // (the common checks see the gate/up matrix this call does not write, [M, 2 * inter]; the code matrix it does
  // write is checked here: a tile's 256 rows are addressed with 32-bit byte offsets)
  HPFP8_REQUIRE(BM * ldq < (int64_t)0x7FFFF000, HPFP8_ERR_SHAPE, "%s: the row stride of q must stay below 8 MiB", what);
  int rc = check_common(what, a, lda, b, ldb, sa, sb, M, 2 * inter, K, nullptr, q, 2 * inter, HPFP8_OUT_F32, 0);
  if (rc <= 0) return rc;
  HPFP8_REQUIRE(scale_inv != nullptr, HPFP8_ERR_ARG, "%s: null scale_inv", what);
  // the up rows of a b tile are addressed `inter` rows past its gate rows, inside one buffer resource
  HPFP8_REQUIRE(2 * inter * ldb < (int64_t)0x7FFFF000, HPFP8_ERR_SHAPE, "%s: the weight's codes must span less than 2 GiB", what);
  GemmParams p{};
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.sa = sa; p.sb = sb; p.lda = lda; p.ldb = ldb;
  p.sa_sm = sa_stride_m; p.sa_sk = sa_stride_k; p.sb_sn = sb_stride_n; p.sb_sk = sb_stride_k;
  rc = check_scale_span(what, M, K / BK, sa_stride_m, sa_stride_k, "sa");
  if (rc <= 0) return rc;
  rc = check_scale_span(what, 2 * inter / kBlock, K / BK, sb_stride_n, sb_stride_k, "sb");
  if (rc <= 0) return rc;
  p.sb_bytes = (int)(((2 * inter / kBlock - 1) * sb_stride_n + (K / BK - 1) * sb_stride_k + 1) * 4);
  p.c = q; p.ldc = ldq;
  p.M = (int)M; p.N = (int)(2 * inter); p.K = (int)K;
  p.inter = (int)inter; p.pow2_out = pow2_out; p.q_scale = scale; p.q_scale_inv = scale_inv;
  const int64_t tiles = ((M + BM - 1) / BM) * (inter / kBlock);
  p.tiles = (int)tiles;
  dim3 grid((unsigned)persistent_grid(tiles)), block(kGemmThreads);
  hipStream_t st = (hipStream_t)stream;
  const bool sa4 = sa_stride_m == 1;
#define HPFP8_LAUNCH_EPI(MODE, SA4, EPI) gemm_kernel<MODE, kDense, false, false, SA4, EPI><<<grid, block, 0, st>>>(p)
  if (pow2) {
    if (sa4) { if (fast) HPFP8_LAUNCH_EPI(kScalePow2, true, 2); else HPFP8_LAUNCH_EPI(kScalePow2, true, 1); }
    else { if (fast) HPFP8_LAUNCH_EPI(kScalePow2, false, 2); else HPFP8_LAUNCH_EPI(kScalePow2, false, 1); }
  } else {
    if (sa4) { if (fast) HPFP8_LAUNCH_EPI(kScaleBlock, true, 2); else HPFP8_LAUNCH_EPI(kScaleBlock, true, 1); }
    else { if (fast) HPFP8_LAUNCH_EPI(kScaleBlock, false, 2); else HPFP8_LAUNCH_EPI(kScaleBlock, false, 1); }
  }
#undef HPFP8_LAUNCH_EPI
  return check_launch(what);
}

void hpfp8_debug_set_small_gemm(int mode) { g_small_gemm_mode.store(mode == 1 || mode == 2 ? mode : 0, std::memory_order_relaxed); }

int hpfp8_gemm_per_tensor(const void* a, int64_t lda, const float* sa_inv, const void* b, int64_t ldb,
                          const float* sb_inv, int64_t M, int64_t N, int64_t K, const void* bias, void* c,
                          int64_t ldc, int out_type, hpfp8_stream_t stream) {
  int rc = check_common("gemm_per_tensor", a, lda, b, ldb, sa_inv, sb_inv, M, N, K, bias, c, ldc, out_type, 0);
  if (rc <= 0) return rc;
  GemmParams p{};
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.sa = sa_inv; p.sb = sb_inv; p.lda = lda; p.ldb = ldb;
  p.c = c; p.ldc = ldc; p.bias = (const uint16_t*)bias;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  p.tiles = (int)tiles;
  if (use_small_kernel(M, N)) return launch_small<kScaleTensor>(p, out_type, (hipStream_t)stream);
  return launch<kScaleTensor, kDense>(p, out_type, tiles, (hipStream_t)stream);
}

static int gemm_grouped_impl(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                             const void* b, int64_t ldb, int64_t b_stride_e, const float* sb, int64_t sb_stride_e,
                             int64_t sb_stride_n, int64_t sb_stride_k, const int32_t* offs, int experts,
                             int64_t total_m, int64_t N, int64_t K, void* c, int64_t ldc, int out_type, bool pow2,
                             hpfp8_stream_t stream) {
  HPFP8_REQUIRE(experts >= 0 && experts <= 4096, HPFP8_ERR_SHAPE, "gemm_grouped: bad expert count %d", experts);
  int rc = check_common("gemm_grouped", a, lda, b, ldb, sa, sb, total_m, N, K, nullptr, c, ldc, out_type, 0);
  if (rc <= 0) return rc;
  if (experts == 0) return HPFP8_OK;
  HPFP8_REQUIRE(offs != nullptr, HPFP8_ERR_ARG, "gemm_grouped: null offs");
  HPFP8_REQUIRE(b_stride_e >= 0 && b_stride_e % 16 == 0, HPFP8_ERR_SHAPE,
                "gemm_grouped: the stride between experts' b matrices must be a non-negative multiple of 16 bytes");
  HPFP8_REQUIRE(sb_stride_e >= 0 && sb_stride_n >= 0 && sb_stride_k >= 0, HPFP8_ERR_SHAPE, "gemm_grouped: negative sb stride");
  GemmParams p{};
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.sa = sa; p.sb = sb; p.lda = lda; p.ldb = ldb; p.b_se = b_stride_e;
  p.sa_sm = sa_stride_m; p.sa_sk = sa_stride_k;
  p.sb_sn = sb_stride_n; p.sb_sk = sb_stride_k; p.sb_se = sb_stride_e;
  rc = check_scale_span("gemm_grouped", total_m, K / BK, sa_stride_m, sa_stride_k, "sa");
  if (rc <= 0) return rc;
  const int64_t sb_span = ((int64_t)(experts - 1) * sb_stride_e + (N / kBlock - 1) * sb_stride_n + (K / BK - 1) * sb_stride_k + 1) * 4;
  HPFP8_REQUIRE(sb_span < (int64_t)0x7FFFFFFF, HPFP8_ERR_SHAPE, "gemm_grouped: b scale array exceeds 2 GiB");
  p.sb_bytes = (int)sb_span;
  p.c = c; p.ldc = ldc; p.offs = offs; p.experts = experts;
  p.M = (int)total_m; p.N = (int)N; p.K = (int)K;
  // upper bound on row tiles: every expert may add one partial tile
  const int64_t tiles = (total_m / BM + experts) * ((N + BN - 1) / BN);
  if (pow2) return launch<kScalePow2, kGroupedRows>(p, out_type, tiles, (hipStream_t)stream);
  return launch<kScaleBlock, kGroupedRows>(p, out_type, tiles, (hipStream_t)stream);
}

int hpfp8_gemm_grouped_blockwise(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                                 const void* b, const float* sb, const int32_t* offs, int experts,
                                 int64_t total_m, int64_t N, int64_t K, void* c, int64_t ldc, int out_type,
                                 hpfp8_stream_t stream) {
  return gemm_grouped_impl(a, lda, sa, sa_stride_m, sa_stride_k, b, K, N * K, sb, (N / kBlock) * (K / BK), K / BK, 1, offs,
                           experts, total_m, N, K, c, ldc, out_type, false, stream);
}

int hpfp8_gemm_grouped_blockwise_pow2(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m,
                                      int64_t sa_stride_k, const void* b, const float* sb, const int32_t* offs,
                                      int experts, int64_t total_m, int64_t N, int64_t K, void* c, int64_t ldc,
                                      int out_type, hpfp8_stream_t stream) {
  return gemm_grouped_impl(a, lda, sa, sa_stride_m, sa_stride_k, b, K, N * K, sb, (N / kBlock) * (K / BK), K / BK, 1, offs,
                           experts, total_m, N, K, c, ldc, out_type, true, stream);
}

int hpfp8_gemm_grouped_blockwise_strided(const void* a, int64_t lda, const float* sa, int64_t sa_stride_m,
                                         int64_t sa_stride_k, const void* b, int64_t ldb, int64_t b_stride_e,
                                         const float* sb, int64_t sb_stride_e, int64_t sb_stride_n, int64_t sb_stride_k,
                                         const int32_t* offs, int experts, int64_t total_m, int64_t N, int64_t K,
                                         void* c, int64_t ldc, int out_type, int pow2, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(pow2 == 0 || pow2 == 1, HPFP8_ERR_ARG, "gemm_grouped: pow2 must be 0 or 1");
  return gemm_grouped_impl(a, lda, sa, sa_stride_m, sa_stride_k, b, ldb, b_stride_e, sb, sb_stride_e, sb_stride_n,
                           sb_stride_k, offs, experts, total_m, N, K, c, ldc, out_type, pow2 != 0, stream);
}

int hpfp8_gemm_grouped_wgrad(const void* a, int64_t lda, const float* sa, const void* b, int64_t ldb, const float* sb,
                             const int32_t* layout, int experts, int64_t total_m, int64_t N, int64_t K, void* c,
                             int out_type, hpfp8_stream_t stream) {
  const char* what = "gemm_grouped_wgrad";
  HPFP8_REQUIRE(experts >= 0 && experts <= 4096, HPFP8_ERR_SHAPE, "%s: bad expert count %d", what, experts);
  HPFP8_REQUIRE(total_m >= 0 && total_m < (int64_t)0x7FFFFF00, HPFP8_ERR_SHAPE, "%s: bad row count", what);
  HPFP8_REQUIRE(N >= 0 && K >= 0 && N % kBlock == 0 && K % kBlock == 0, HPFP8_ERR_SHAPE,
                "%s: N=%lld and K=%lld must be multiples of 128", what, (long long)N, (long long)K);
  if (experts == 0 || N == 0 || K == 0) return HPFP8_OK;
  // the GEMM behind it: rows = N (rows of grad_out^T), columns = K (rows of x^T), contraction = the padded token axis
  const int64_t padded = (total_m / kBlock + experts) * kBlock;
  int rc = check_common(what, a, lda, b, ldb, sa, sb, N, K, padded, nullptr, c, K, out_type, 0);
  if (rc <= 0) return rc;
  HPFP8_REQUIRE(layout != nullptr, HPFP8_ERR_ARG, "%s: null layout", what);
  HPFP8_REQUIRE(aligned16(sa) && aligned16(sb), HPFP8_ERR_ALIGN, "%s: scale arrays must be 16-byte aligned", what);
  HPFP8_REQUIRE((padded / BK) * (N > K ? N : K) * 4 < (int64_t)0x7FFFFFFF, HPFP8_ERR_SHAPE, "%s: a scale array spans 2 GiB or more", what);
  HPFP8_REQUIRE((int64_t)experts * (((N + BM - 1) / BM) * ((K + BN - 1) / BN)) < (int64_t)0x7FFFFFFF, HPFP8_ERR_SHAPE, "%s: too many tiles", what);
  GemmParams p{};
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.sa = sa; p.sb = sb; p.lda = lda; p.ldb = ldb;
  p.sa_sm = 1; p.sa_sk = N;          // [padded / 128, N]: block-major, as the grouped transposed quantizer writes them
  p.sb_sn = 1; p.sb_sk = K;          // [padded / 128, K]
  p.c = c; p.ldc = K; p.c_se = N * K; p.layout = layout; p.experts = experts;
  p.M = (int)N; p.N = (int)K; p.K = (int)padded;
  const int64_t per_expert = ((N + BM - 1) / BM) * ((K + BN - 1) / BN);
  p.tiles = (int)per_expert;
  return launch<kScaleRow, kGroupedK>(p, out_type, per_expert * experts, (hipStream_t)stream);
}

}  // extern "C"
