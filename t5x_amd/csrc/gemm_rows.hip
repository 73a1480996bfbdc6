// Dense layers over many rows (the encoder side: M = batch x encoder length).
//
// Unlike the decode-step GEMMs these are compute-bound.  A workgroup (4
// wavefronts, 2 x 2) owns a 256 x 128 output tile, each wavefront a 128 x 64
// sub-tile = 8 x 4 MFMA tiles (v_mfma_f32_16x16x32_bf16).  Per k-tile of 32 the
// workgroup needs 16 activation fragments (16 rows x 64 bytes each) and 8
// packed weight tiles, 1 KB apiece in MFMA operand layout; every wavefront
// fetches 6 of them from memory, parks them in LDS exactly as loaded (lane l
// at byte 16 l: conflict-free both ways), and after one barrier reads the 12
// it multiplies.  Global loads for k + 1 are in flight while k is multiplied;
// two LDS buffers, one barrier per k-tile.  Sharing through LDS cuts the
// operand traffic per matrix instruction to 3/8 of what loading every
// operand per wavefront costs, which is what bounds this shape.
// A packed weight tile has the same lane layout as either MFMA operand, so the
// product can be formed as C (activations as A) or as C^T (weights as A); C^T
// leaves every lane with 4 consecutive output COLUMNS of one row, C with 4
// consecutive ROWS of one column — whichever makes the 8-byte stores
// contiguous in the requested output layout.
#include "common.h"

namespace t5d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_r;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_r;

union FragR {
  uint4 u;
  bf16x8_r v;
};

__device__ __forceinline__ uint32_t i8x2_to_bf16x2(int a, int b) {
  // int8 values are exactly representable in bfloat16.
  return (__float_as_uint((float)a) >> 16) |
         (__float_as_uint((float)b) & 0xFFFF0000u);
}

// A packed weight tile as loaded (`Raw`) and widened to bfloat16 (`frag`).
template <typename WT> struct RowsWeightTile;
template <> struct RowsWeightTile<bf16_t> {
  static constexpr int kTileBytes = 1024;
  typedef uint4 Raw;
  __device__ static __forceinline__ Raw load(const char* tile, int lane) {
    return reinterpret_cast<const uint4*>(tile)[lane];
  }
  __device__ static __forceinline__ uint4 frag(const Raw& r) { return r; }
};
template <> struct RowsWeightTile<int8_t> {
  static constexpr int kTileBytes = 512;
  typedef uint2 Raw;
  __device__ static __forceinline__ Raw load(const char* tile, int lane) {
    return reinterpret_cast<const uint2*>(tile)[lane];
  }
  __device__ static __forceinline__ uint4 frag(const Raw& q) {
    uint4 f;
    f.x = i8x2_to_bf16x2((int8_t)(q.x), (int8_t)(q.x >> 8));
    f.y = i8x2_to_bf16x2((int8_t)(q.x >> 16), (int8_t)(q.x >> 24));
    f.z = i8x2_to_bf16x2((int8_t)(q.y), (int8_t)(q.y >> 8));
    f.w = i8x2_to_bf16x2((int8_t)(q.y >> 16), (int8_t)(q.y >> 24));
    return f;
  }
};

struct RowsGemmArgs {
  const bf16_t* A;         // [M, K]
  const char* W;           // packed tiles [N/16][K/32]
  const float* scales;     // [N] for int8 weights, else null
  const bf16_t* residual;  // [M, N] row-major, or null
  bf16_t* C;
  int M, K, N;
  int epilogue;            // T5D_EPI_*
  int layout;              // T5D_OUT_*
  int E, Ep, H;            // heads layouts: m = b * E + e, n = h * 64 + d
};

__device__ __forceinline__ uint2 pack4(float a, float b, float c, float d) {
  uint2 p;
  p.x = pack_bf16x2(a, b);
  p.y = pack_bf16x2(c, d);
  return p;
}

constexpr int kRowsBM = 256, kRowsBN = 128;  // workgroup tile
constexpr int kRowsMT = 8, kRowsNT = 4;        // MFMA tiles per wavefront

// What a wavefront does with its finished accumulator tiles (m0: its first
// row, nt0: its first 16-column tile) when the product was formed as C, for
// the value layout:
template <int NT>
__device__ __forceinline__ void rows_epilogue_values(
    const RowsGemmArgs& g, const f32x4_r (&acc)[kRowsMT][NT], int m0,
    int nt0, int n_tiles, int l16, int gq) {
  constexpr int MT = kRowsMT;
  // acc[mt][nt][i]: row m = m0 + 16 mt + 4 gq + i, column n = 16 (nt0 + nt) + l16
  // (values layout [B, H, Ep / 32, 64, 32]: 4 consecutive positions per store)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + 16 * mt + 4 * gq;
    if (m >= g.M) continue;
    const int b = m / g.E, e = m - b * g.E;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (nt0 + nt >= n_tiles) continue;
      const int n = 16 * (nt0 + nt) + l16;
      float s = g.scales ? g.scales[n] : 1.f;
      const int hh = n >> 6, d = n & 63;
      const size_t o =
          ((((size_t)b * g.H + hh) * (g.Ep >> 5) + (e >> 5)) * 64 + d) * 32 +
          (e & 31);
      *reinterpret_cast<uint2*>(g.C + o) =
          pack4(acc[mt][nt][0] * s, acc[mt][nt][1] * s, acc[mt][nt][2] * s,
                acc[mt][nt][3] * s);
    }
  }
}

// ... and when it was formed as C^T, with the stores made whole: a lane holds
// 4 consecutive columns of one row, so storing from the accumulators would
// write 16 rows x 8..32 bytes per instruction.  Each
// wavefront instead parks one 16-row slice at a time in a private piece of
// LDS (rounded to bfloat16, rows padded by 16 bytes) and reads it back with 4
// or 8 lanes per row, 16 bytes per lane: every store instruction then writes
// whole 64-byte (gated) or 128-byte rows, and the residual is read the same
// way.  LDS operations of one wavefront complete in order, so the slices
// follow one another through the same piece without a wait in between; the
// empty asm statements keep the compiler from moving one lane's read above
// another lane's write (to it they are accesses of unrelated addresses).
constexpr int kRowsStageBytes = 16 * 144;
template <int NT>
__device__ __forceinline__ void rows_epilogue_staged(
    const RowsGemmArgs& g, const f32x4_r (&acc)[kRowsMT][NT], int m0, int nt0,
    int n_tiles, int lane, char* stage) {
  static_assert(NT == 3 || NT == 4, "a wavefront's slice: 48 or 64 columns");
  constexpr int MT = kRowsMT;
  const int l16 = lane & 15, gq = lane >> 4;
  // int8 weights: the scale of each of this lane's 4 columns (1 otherwise)
  float4 sc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    sc[nt] = (g.scales && nt0 + nt < n_tiles)
                 ? *reinterpret_cast<const float4*>(g.scales +
                                                    16 * (nt0 + nt) + 4 * gq)
                 : make_float4(1.f, 1.f, 1.f, 1.f);
  if (g.epilogue == T5D_EPI_GEGLU) {
    // tile columns 0..7 are wi_0, 8..15 the matching wi_1 columns: the lanes
    // with gq >= 2 hold the gates of the lanes with gq - 2.  32 output columns.
    // Two v_permlane32_swap hand every lane two (value, gate) pairs — the
    // lower half of the wavefront keeps its values 2, 3 and receives their
    // gates, the upper half keeps its gates 0, 1 and receives their values —
    // so all 64 lanes evaluate GELU on values that are used.
    const int F = g.N >> 1;
    const int row = lane / NT, piece = lane % NT;  // NT 16-byte pieces per row
    const bool lower = gq < 2;
    const int col0 = 4 * (gq & 1) + (lower ? 2 : 0);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const auto a = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(acc[mt][nt][2] * sc[nt].z),
            __float_as_uint(acc[mt][nt][0] * sc[nt].x), false, false);
        const auto b = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(acc[mt][nt][3] * sc[nt].w),
            __float_as_uint(acc[mt][nt][1] * sc[nt].y), false, false);
        // [0]: the value (own in the lower half), [1]: its gate
        const float h0 =
            round_bf16(gelu_sigmoid_form(round_bf16(__uint_as_float(a[0])))) *
            round_bf16(__uint_as_float(a[1]));
        const float h1 =
            round_bf16(gelu_sigmoid_form(round_bf16(__uint_as_float(b[0])))) *
            round_bf16(__uint_as_float(b[1]));
        *reinterpret_cast<uint32_t*>(stage + l16 * 80 + (8 * nt + col0) * 2) =
            pack_bf16x2(h0, h1);
      }
      asm volatile("" ::: "memory");
      const uint4 q = *reinterpret_cast<const uint4*>(
          stage + min(row, 15) * 80 + piece * 16);
      asm volatile("" ::: "memory");
      const int m = m0 + 16 * mt + row;
      if (row < 16 && m < g.M && nt0 + piece < n_tiles)
        *reinterpret_cast<uint4*>(g.C + (size_t)m * F + 8 * (nt0 + piece)) = q;
    }
    return;
  }
  constexpr int PP = 2 * NT;    // 16-byte pieces per row of the slice
  constexpr int RPI = 64 / PP;  // rows per instruction (8, or 10 with 4 lanes idle)
  const int piece = lane % PP, prow = lane / PP;
  const int n = 16 * nt0 + 8 * piece;
  const bool n_ok = nt0 + (piece >> 1) < n_tiles;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      *reinterpret_cast<uint2*>(stage + l16 * 144 + (16 * nt + 4 * gq) * 2) =
          pack4(acc[mt][nt][0] * sc[nt].x, acc[mt][nt][1] * sc[nt].y,
                acc[mt][nt][2] * sc[nt].z, acc[mt][nt][3] * sc[nt].w);
    asm volatile("" ::: "memory");
    uint4 back[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
      back[j] = *reinterpret_cast<const uint4*>(
          stage + min(RPI * j + prow, 15) * 144 + piece * 16);
    asm volatile("" ::: "memory");
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = RPI * j + prow;
      if (prow >= RPI || row >= 16) continue;
      uint4 q = back[j];
      const int m = m0 + 16 * mt + row;
      if (m >= g.M || !n_ok) continue;
      size_t o;
      if (g.layout == T5D_OUT_HEADS_KEY) {
        // [B, H, 2, Ep, 32]: the two 32-wide halves of the head dim as planes
        const int b = m / g.E, e = m - b * g.E;
        const int hh = n >> 6, c = (n >> 5) & 1, jj = n & 31;
        o = ((((size_t)b * g.H + hh) * 2 + c) * g.Ep + e) * 32 + jj;
      } else {
        o = (size_t)m * g.N + n;
      }
      if (g.epilogue == T5D_EPI_RESIDUAL) {
        const uint4 r = *reinterpret_cast<const uint4*>(
            g.residual + (size_t)m * g.N + n);
        q.x = pack_bf16x2(bf16lo_to_f32(q.x) + bf16lo_to_f32(r.x),
                          bf16hi_to_f32(q.x) + bf16hi_to_f32(r.x));
        q.y = pack_bf16x2(bf16lo_to_f32(q.y) + bf16lo_to_f32(r.y),
                          bf16hi_to_f32(q.y) + bf16hi_to_f32(r.y));
        q.z = pack_bf16x2(bf16lo_to_f32(q.z) + bf16lo_to_f32(r.z),
                          bf16hi_to_f32(q.z) + bf16hi_to_f32(r.z));
        q.w = pack_bf16x2(bf16lo_to_f32(q.w) + bf16lo_to_f32(r.w),
                          bf16hi_to_f32(q.w) + bf16hi_to_f32(r.w));
      }
      *reinterpret_cast<uint4*>(g.C + o) = q;
    }
  }
}

// SWAP: weights are the MFMA A operand (C^T is formed).
template <typename WT, bool SWAP>
__global__ void __launch_bounds__(256, 2)
rows_gemm_kernel(RowsGemmArgs g) {
  constexpr int TB = RowsWeightTile<WT>::kTileBytes;
  constexpr int MT = kRowsMT, NT = kRowsNT;
  // [buffer][tile][lane]: tiles 0..15 activations (rows 16 t ..), 16..23 weights
  __shared__ uint4 s_t[2][24][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, gq = lane >> 4;
  const int m_blocks = (g.M + kRowsBM - 1) / kRowsBM;
  const int m_blk = blockIdx.x % m_blocks, n_blk = blockIdx.x / m_blocks;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = m_blk * kRowsBM + wm * (16 * MT);
  const int nt0 = n_blk * (kRowsBN / 16) + wn * NT;  // first 16-column tile
  const int KT = g.K >> 5, n_tiles = g.N >> 4;

  // The 6 tiles this wavefront fetches: activation tiles wave + 4 i (i < 4),
  // weight tiles wave + 4 i (i < 2).  Out-of-range rows / tiles are clamped
  // (their products are discarded in the epilogue).
  // An activation tile is fetched with lane l reading piece l % 4 (8 k) of row
  // l / 4, so that four neighbouring lanes read 64 contiguous bytes: fetched in
  // operand order (lane = row + 16 * piece) every lane of a quarter wavefront
  // touches another row, 64 separate requests per instruction, and the L1's
  // tag lookups, not the matrix cores, set the pace.  The piece lands in LDS at
  // its operand slot, XOR-swizzled so that neither the parking writes nor the
  // operand reads collide on banks.
  const int ld_row = lane >> 2, ld_piece = lane & 3;
  const int park_slot = (ld_piece * 16 + ld_row) ^ (ld_piece * 2);
  const int read_slot = lane ^ (gq * 2);
  const bf16_t* arow[4];
  const char* wtile[2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    arow[i] = g.A +
              (size_t)min(m_blk * kRowsBM + 16 * (wave + 4 * i) + ld_row, g.M - 1) *
                  g.K + 8 * ld_piece;
#pragma unroll
  for (int i = 0; i < 2; ++i)
    wtile[i] = g.W + (size_t)min(n_blk * (kRowsBN / 16) + wave + 4 * i,
                                 n_tiles - 1) * KT * TB;

  f32x4_r acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = (f32x4_r){0.f, 0.f, 0.f, 0.f};

  // Staging registers of the 6 tiles in flight (named, not an array: they
  // must stay in registers across the loop).
  typedef typename RowsWeightTile<WT>::Raw RawW;
  uint4 sa0, sa1, sa2, sa3;
  RawW sw0, sw1;
#define T5D_ROWS_FETCH(kt_)                                                    \
  do {                                                                         \
    sa0 = *reinterpret_cast<const uint4*>(arow[0] + 32 * (kt_));               \
    sa1 = *reinterpret_cast<const uint4*>(arow[1] + 32 * (kt_));               \
    sa2 = *reinterpret_cast<const uint4*>(arow[2] + 32 * (kt_));               \
    sa3 = *reinterpret_cast<const uint4*>(arow[3] + 32 * (kt_));               \
    sw0 = RowsWeightTile<WT>::load(wtile[0] + (size_t)(kt_) * TB, lane);       \
    sw1 = RowsWeightTile<WT>::load(wtile[1] + (size_t)(kt_) * TB, lane);       \
  } while (0)
#define T5D_ROWS_PARK(buf_)                                                    \
  do {                                                                         \
    s_t[buf_][wave][park_slot] = sa0;                                          \
    s_t[buf_][wave + 4][park_slot] = sa1;                                      \
    s_t[buf_][wave + 8][park_slot] = sa2;                                      \
    s_t[buf_][wave + 12][park_slot] = sa3;                                     \
    s_t[buf_][16 + wave][lane] = RowsWeightTile<WT>::frag(sw0);                \
    s_t[buf_][20 + wave][lane] = RowsWeightTile<WT>::frag(sw1);                \
  } while (0)
  T5D_ROWS_FETCH(0);
  T5D_ROWS_PARK(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) T5D_ROWS_FETCH(kt + 1);
    FragR wb[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) wb[nt].u = s_t[buf][16 + wn * NT + nt][lane];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      FragR xa;
      xa.u = s_t[buf][wm * MT + mt][read_slot];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        if (SWAP)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              wb[nt].v, xa.v, acc[mt][nt], 0, 0, 0);
        else
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              xa.v, wb[nt].v, acc[mt][nt], 0, 0, 0);
      }
    }
    if (kt + 1 < KT) T5D_ROWS_PARK(buf ^ 1);
    __syncthreads();
  }
#undef T5D_ROWS_FETCH
#undef T5D_ROWS_PARK

  if (SWAP) {
    // (the loop ends with a barrier: every wavefront is done with the tiles)
    static_assert(sizeof(s_t[0]) >= 4 * kRowsStageBytes, "stage too small");
    rows_epilogue_staged<NT>(
        g, acc, m0, nt0, n_tiles, lane,
        reinterpret_cast<char*>(&s_t[0][0][0]) + wave * kRowsStageBytes);
  } else {
    rows_epilogue_values<NT>(g, acc, m0, nt0, n_tiles, l16, gq);
  }
}

// ---- the same tile with operands loaded straight into LDS ---------------------
// rows_gemm_kernel keeps one k-tile of loads in flight per workgroup (staging
// registers), which covers a fifth of the memory latency; the matrix cores
// wait for the rest.  Here the 24 operand tiles of a k-tile go from memory
// into LDS without passing through registers (global_load_lds, 16 bytes per
// lane, lane l of an instruction landing at byte 16 l of the destination), in
// a ring of three stages, so two k-tiles are in flight while one is
// multiplied.  One barrier per k-tile, placed by hand together with the wait
// for "all but my newest six loads": the stages are three separate arrays and
// the K loop handles three k-tiles per round, so that the compiler can tell a
// read of one stage from a load into another and adds no wait of its own.
// An activation tile is fetched with lane 4 q + j reading row q, piece
// (j + q / 4) % 4 — four neighbouring lanes still read 64 contiguous bytes —
// which puts piece p of row r at slot 4 r + (p - r / 4) % 4, so that the 16
// lanes of a quarter wavefront read 16 slots that differ mod 16.  The LDS
// still counts bank conflicts for these reads (its rule for 16-byte reads is
// not the plain one; other rotations measured the same or worse), but the
// alternative without any — every lane fetching its own operand piece, 16
// rows per quarter wavefront — loses more in the fetch (185 us against 174).
// bfloat16 weights (int8 tiles must be widened on the way).
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* glb_ptr_t;

// WN: wavefront columns of the workgroup, 2 (256 x 128 tile, 4 wavefronts, two
// workgroups per CU) or 4 (256 x 256, 8 wavefronts, one per CU).
// Measured on the gated MLP input projection of the T5.1.1-base encoder
// (16384 x 768 x 4096): 182 -> 176 us per launch with the ring alone, 123 us
// with the epilogue below (the library tanh and the 8-byte stores were a
// third of the launch), 118 us with the 256 x 256 tile.  The same tile from 4
// wavefronts of 128 x 128 (accumulators in the accumulation registers) lasts
// 257 us: with one wavefront per SIMD nothing covers the operand reads from
// LDS.
template <bool SWAP, int NT, int WN>
__global__ void __launch_bounds__(128 * WN, WN == 2 ? 2 : 1)
rows_gemm_direct_kernel(RowsGemmArgs g) {
  constexpr int MT = kRowsMT;
  constexpr int WAVES = 2 * WN;         // 2 rows of WN wavefronts
  constexpr int BN = WN * NT * 16;      // columns of the workgroup tile
  constexpr int AL = 16 / WAVES;        // activation tiles a wavefront loads per stage
  constexpr int WTILES = WN * NT;       // weight tiles of a stage
  // weight tiles a wavefront loads per stage; when they do not divide evenly
  // some wavefronts load a tile a second time (same bytes to the same place)
  constexpr int WL = (WTILES + WAVES - 1) / WAVES;
  constexpr int TILES = 16 + WN * NT;
  // Before every barrier: all but my newest AL + WL loads have landed AND all
  // my reads of LDS have returned, s_waitcnt vmcnt(AL + WL) lgkmcnt(0).  The
  // second half matters: the barrier orders instructions that have been
  // issued, not LDS reads that have completed, and the compiler is free to
  // sink the last operand reads and matrix instructions of a k-tile below the
  // next barrier.  Without the wait a workgroup's fastest wavefront could
  // refill the stage while the slowest still had reads of it queued (seen as
  // one wrong 16-row slice in about one launch in ten at 16384 x 768).
  constexpr int kWaitStage = 0x070 | (AL + WL);
  constexpr int kWaitAll = 0x070;
  // [tile][lane]: tiles 0..15 activations (rows 16 t ..), then the weights
  __shared__ uint4 s_t0[TILES][64];
  __shared__ uint4 s_t1[TILES][64];
  __shared__ uint4 s_t2[TILES][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, gq = lane >> 4;
  const int m_blocks = (g.M + kRowsBM - 1) / kRowsBM;
  const int m_blk = blockIdx.x % m_blocks, n_blk = blockIdx.x / m_blocks;
  const int wm = wave / WN, wn = wave % WN;
  const int m0 = m_blk * kRowsBM + wm * (16 * MT);
  const int nt0 = n_blk * (BN / 16) + wn * NT;
  const int KT = g.K >> 5, n_tiles = g.N >> 4;

  const int ld_row = lane >> 2;
  const int ld_piece = ((lane & 3) + (ld_row >> 2)) & 3;
  const int read_slot = 4 * l16 + ((gq - (l16 >> 2)) & 3);
  // this wavefront's tiles of every stage: activation tiles wave + WAVES i,
  // weight tiles wave + WAVES i (rows / tiles past the edge clamped: their
  // products are discarded in the epilogue)
  const char* arow[AL];
  const char* wtile[WL];
#pragma unroll
  for (int i = 0; i < AL; ++i)
    arow[i] = reinterpret_cast<const char*>(
        g.A +
        (size_t)min(m_blk * kRowsBM + 16 * (wave + WAVES * i) + ld_row,
                    g.M - 1) *
            g.K + 8 * ld_piece);
#pragma unroll
  for (int i = 0; i < WL; ++i)
    wtile[i] = g.W + (size_t)min(n_blk * (BN / 16) +
                                     (wave + WAVES * i) % WTILES,
                                 n_tiles - 1) * KT * 1024 + lane * 16;

  f32x4_r acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = (f32x4_r){0.f, 0.f, 0.f, 0.f};

#define T5D_ROWS_ISSUE(kt_, S_)                                                \
  do {                                                                         \
    _Pragma("unroll") for (int i = 0; i < AL; ++i)                             \
      __builtin_amdgcn_global_load_lds((glb_ptr_t)(arow[i] + 64 * (kt_)),      \
                                       (lds_ptr_t)&S_[wave + WAVES * i][0],    \
                                       16, 0, 0);                              \
    _Pragma("unroll") for (int i = 0; i < WL; ++i)                             \
      __builtin_amdgcn_global_load_lds(                                        \
          (glb_ptr_t)(wtile[i] + (size_t)(kt_) * 1024),                        \
          (lds_ptr_t)&S_[16 + (wave + WAVES * i) % WTILES][0], 16, 0, 0);      \
  } while (0)
#define T5D_ROWS_MULTIPLY(S_)                                                  \
  do {                                                                         \
    FragR wb[NT];                                                              \
    _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                          \
      wb[nt].u = S_[16 + wn * NT + nt][lane];                                  \
    _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                        \
      FragR xa;                                                                \
      xa.u = S_[wm * MT + mt][read_slot];                                      \
      _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) {                      \
        if (SWAP)                                                              \
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(               \
              wb[nt].v, xa.v, acc[mt][nt], 0, 0, 0);                           \
        else                                                                   \
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(               \
              xa.v, wb[nt].v, acc[mt][nt], 0, 0, 0);                           \
      }                                                                        \
    }                                                                          \
  } while (0)
  // kWaitStage: all but this wavefront's newest loads have landed, i.e. its
  // share of the stage about to be multiplied, and its reads of the previous
  // stage have returned; after the barrier every wavefront's share has
  // landed, and every wavefront is done with the stage that the next loads
  // overwrite.
#define T5D_ROWS_STEP(kt_, CUR_, NEXT2_)                                       \
  do {                                                                         \
    __builtin_amdgcn_s_waitcnt(kWaitStage);                                    \
    __builtin_amdgcn_s_barrier();                                              \
    T5D_ROWS_ISSUE((kt_) + 2, NEXT2_);                                         \
    __builtin_amdgcn_sched_barrier(0);                                         \
    T5D_ROWS_MULTIPLY(CUR_);                                                   \
  } while (0)
#define T5D_ROWS_LAST(kt_, CUR_, NEXT2_)                                       \
  do {                                                                         \
    if ((kt_) + 1 < KT) __builtin_amdgcn_s_waitcnt(kWaitStage);                \
    else __builtin_amdgcn_s_waitcnt(kWaitAll);                                 \
    __builtin_amdgcn_s_barrier();                                              \
    if ((kt_) + 2 < KT) T5D_ROWS_ISSUE((kt_) + 2, NEXT2_);                     \
    __builtin_amdgcn_sched_barrier(0);                                         \
    T5D_ROWS_MULTIPLY(CUR_);                                                   \
  } while (0)
  T5D_ROWS_ISSUE(0, s_t0);
  T5D_ROWS_ISSUE(1, s_t1);  // KT >= 2 (checked by the caller)
  const int n_main = (KT - 2) / 3 * 3;
  int kt = 0;
  for (; kt < n_main; kt += 3) {
    T5D_ROWS_STEP(kt, s_t0, s_t2);
    T5D_ROWS_STEP(kt + 1, s_t1, s_t0);
    T5D_ROWS_STEP(kt + 2, s_t2, s_t1);
  }
  // the last 2 to 4 k-tiles
  T5D_ROWS_LAST(kt, s_t0, s_t2);
  T5D_ROWS_LAST(kt + 1, s_t1, s_t0);
  if (kt + 2 < KT) T5D_ROWS_LAST(kt + 2, s_t2, s_t1);
  if (kt + 3 < KT) T5D_ROWS_LAST(kt + 3, s_t0, s_t2);
#undef T5D_ROWS_ISSUE
#undef T5D_ROWS_MULTIPLY
#undef T5D_ROWS_STEP
#undef T5D_ROWS_LAST
  if (SWAP) {
    static_assert(sizeof(s_t0) >= WAVES * kRowsStageBytes, "stage too small");
    __syncthreads();  // every wavefront is done with the ring
    rows_epilogue_staged<NT>(
        g, acc, m0, nt0, n_tiles, lane,
        reinterpret_cast<char*>(&s_t0[0][0]) + wave * kRowsStageBytes);
  } else {
    rows_epilogue_values<NT>(g, acc, m0, nt0, n_tiles, l16, gq);
  }
}

}  // namespace t5d

using namespace t5d;

// Three workgroup tiles.  256 x 256 (8 wavefronts, one workgroup per CU)
// halves the operand bytes per flop of 256 x 128 (4 wavefronts, two per CU)
// and measures 3-11 % faster whenever its workgroups fill the 256 CUs
// evenly; 256 x 192 (8 wavefronts of 128 x 48) is for the shapes where
// neither does: N = 768 over 16384 rows is 192 tiles of 256 x 256 (a quarter
// of the chip idle) but exactly 256 of 256 x 192.  Picked by the cost of the
// rounds each tile needs, a last round that fills at most half of the CUs'
// two slots counting 0.6 for the 256 x 128 tile.
extern "C" int t5d_gemm_rows_tile(int w_dtype, int64_t M, int K, int N) {
  if (w_dtype != T5D_BF16 || K < 64 || M <= 0 || N <= 0) return 1;
  const auto rounds = [](int64_t wgs, int slots) {
    return (double)((wgs + slots - 1) / slots);
  };
  const int64_t m_blocks = (M + kRowsBM - 1) / kRowsBM;
  const int64_t wgs128 = m_blocks * ((N + 127) / 128),
                wgs192 = m_blocks * ((N + 191) / 192),
                wgs256 = m_blocks * ((N + 255) / 256);
  double c128 = rounds(wgs128, 512) * 2.0 * 128;
  if ((wgs128 - 1) % 512 < 256) c128 -= 0.4 * 2.0 * 128;
  const double c192 = rounds(wgs192, 256) * 192.0,
               c256 = rounds(wgs256, 256) * 256.0;
  int pick = 2;
  double best = c256;
  if (c192 < best) { best = c192; pick = 3; }
  if (c128 < 0.97 * best) pick = 1;
  return pick;
}

extern "C" int t5d_gemm_rows(void* stream, int w_dtype, const void* A,
                             const void* W, const float* scales,
                             const void* residual, void* C, int64_t M, int K,
                             int N, int epilogue, int out_layout, int E,
                             int Ep) {
  return t5d_gemm_rows_tiled(stream, w_dtype, A, W, scales, residual, C, M, K,
                             N, epilogue, out_layout, E, Ep, 0);
}

extern "C" int t5d_gemm_rows_tiled(void* stream, int w_dtype, const void* A,
                                   const void* W, const float* scales,
                                   const void* residual, void* C, int64_t M,
                                   int K, int N, int epilogue, int out_layout,
                                   int E, int Ep, int tile) {
  T5D_REQUIRE(A && W && C, T5D_EINVAL, "t5d_gemm_rows: null pointer");
  T5D_REQUIRE(tile >= 0 && tile <= 3, T5D_EINVAL,
              "t5d_gemm_rows_tiled: tile %d (0 chosen here, 1: 256 x 128, "
              "2: 256 x 256, 3: 256 x 192)", tile);
  T5D_REQUIRE(w_dtype == T5D_BF16 || w_dtype == T5D_I8, T5D_EINVAL,
              "t5d_gemm_rows: w_dtype %d (packed bfloat16 or int8)", w_dtype);
  T5D_REQUIRE(w_dtype != T5D_I8 || scales, T5D_EINVAL,
              "t5d_gemm_rows: int8 weights need scales");
  T5D_REQUIRE(M > 0 && M < (1 << 30) && K > 0 && K % 32 == 0 && N > 0 &&
                  N % 16 == 0,
              T5D_EINVAL, "t5d_gemm_rows: M=%lld K=%d N=%d (K %% 32, N %% 16)",
              (long long)M, K, N);
  T5D_REQUIRE(epilogue >= T5D_EPI_NONE && epilogue <= T5D_EPI_GEGLU, T5D_EINVAL,
              "t5d_gemm_rows: epilogue %d", epilogue);
  T5D_REQUIRE(epilogue != T5D_EPI_RESIDUAL || residual, T5D_EINVAL,
              "t5d_gemm_rows: residual epilogue without residual");
  T5D_REQUIRE(out_layout >= T5D_OUT_ROWS && out_layout <= T5D_OUT_HEADS_VALUE,
              T5D_EINVAL, "t5d_gemm_rows: out_layout %d", out_layout);
  T5D_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 &&
                  ((uintptr_t)C % 8) == 0 && ((uintptr_t)residual % 8) == 0,
              T5D_EINVAL, "t5d_gemm_rows: operand alignment");
  int H = 0;
  if (out_layout != T5D_OUT_ROWS) {
    T5D_REQUIRE(epilogue == T5D_EPI_NONE && N % 64 == 0 && E > 0 && Ep >= E &&
                    M % E == 0 && E % 4 == 0 && Ep % 32 == 0,
                T5D_EINVAL,
                "t5d_gemm_rows: heads layout needs epilogue none, N %% 64 == 0,"
                " M %% E == 0, E %% 4 == 0, Ep %% 32 == 0 (N=%d E=%d Ep=%d)", N,
                E, Ep);
    H = N / 64;
  }
  RowsGemmArgs g;
  g.A = (const bf16_t*)A; g.W = (const char*)W;
  g.scales = w_dtype == T5D_I8 ? scales : nullptr;
  g.residual = (const bf16_t*)residual; g.C = (bf16_t*)C;
  g.M = (int)M; g.K = K; g.N = N;
  g.epilogue = epilogue; g.layout = out_layout;
  g.E = E; g.Ep = Ep; g.H = H;
  const int m_blocks = ((int)M + kRowsBM - 1) / kRowsBM;
  const int n_blocks = (N + kRowsBN - 1) / kRowsBN;
  dim3 grid((unsigned)m_blocks * n_blocks), block(256);
  hipStream_t s = as_stream(stream);
  const bool swap = out_layout != T5D_OUT_HEADS_VALUE;
  const int pick = tile ? tile : t5d_gemm_rows_tile(w_dtype, M, K, N);
  const int wgs192 = m_blocks * ((N + 191) / 192),
            wgs256 = m_blocks * ((N + 255) / 256);
  if (w_dtype == T5D_BF16 && K >= 64 && pick == 3) {
    dim3 wgrid((unsigned)wgs192), wblock(512);
    if (swap)
      hipLaunchKernelGGL((rows_gemm_direct_kernel<true, 3, 4>), wgrid, wblock,
                         0, s, g);
    else
      hipLaunchKernelGGL((rows_gemm_direct_kernel<false, 3, 4>), wgrid, wblock,
                         0, s, g);
  } else if (w_dtype == T5D_BF16 && K >= 64 && pick == 2) {
    dim3 wgrid((unsigned)wgs256), wblock(512);
    if (swap)
      hipLaunchKernelGGL((rows_gemm_direct_kernel<true, kRowsNT, 4>), wgrid,
                         wblock, 0, s, g);
    else
      hipLaunchKernelGGL((rows_gemm_direct_kernel<false, kRowsNT, 4>), wgrid,
                         wblock, 0, s, g);
  } else if (w_dtype == T5D_BF16 && K >= 64) {
    if (swap)
      hipLaunchKernelGGL((rows_gemm_direct_kernel<true, kRowsNT, 2>), grid,
                         block, 0, s, g);
    else
      hipLaunchKernelGGL((rows_gemm_direct_kernel<false, kRowsNT, 2>), grid,
                         block, 0, s, g);
  } else if (w_dtype == T5D_BF16) {
    if (swap)
      hipLaunchKernelGGL((rows_gemm_kernel<bf16_t, true>), grid, block, 0, s, g);
    else
      hipLaunchKernelGGL((rows_gemm_kernel<bf16_t, false>), grid, block, 0, s, g);
  } else {
    if (swap)
      hipLaunchKernelGGL((rows_gemm_kernel<int8_t, true>), grid, block, 0, s, g);
    else
      hipLaunchKernelGGL((rows_gemm_kernel<int8_t, false>), grid, block, 0, s, g);
  }
  T5D_CHECK_LAUNCH("t5d_gemm_rows");
  return T5D_OK;
}
