// Weight-streaming dense layers for M <= 128 activation rows.
//
// At these row counts every GEMM of the decode step is bound by reading the
// weight matrix once, so the kernels are organised around the weight stream:
//   * bf16 / int8 weights are pre-packed into 32(k) x 16(n) MFMA B-operand
//     tiles stored lane-major, so one wavefront load instruction fetches one
//     whole tile as a single contiguous 1 KB (bf16) / 512 B (int8) burst
//     straight into the registers v_mfma_f32_16x16x32_bf16 consumes;
//   * a workgroup owns NT adjacent 16-column tiles and MP 16-row tiles; its 4
//     wavefronts split the K range in pairs of k-tiles (pair p goes to wave
//     p % 4), keep several pairs of weight tiles in flight ahead of the MFMAs,
//     and sum their 4 partial accumulators through LDS in a fixed order
//     (bitwise deterministic, no atomics, no cross-workgroup traffic);
//   * small-N layers get their parallelism from splitting M across
//     workgroups; the workgroups that share a weight slice are mapped to the
//     same XCD (consecutive block ids go round-robin over the 8 XCDs), so the
//     slice comes from HBM once and from that XCD's L2 afterwards.
// The activation operand is read from L2 in full 128-byte lines (a pair of
// k-tiles is 64 contiguous bf16 per row).
#include <cstdlib>
#include <cstring>

#include "common.h"
#include "gemm_tiles.h"

namespace t5d {

// NJ > 0: K is NJ * 256, every wavefront owns exactly NJ k-tile pairs and the K
// loop is straight-line code (see gemm_big_kernel).
template <int MP, int NT, typename WT, int NJ = 0>
__global__ void __launch_bounds__(256)
gemm_mfma_kernel(GemmArgs g) {
  constexpr int ACC = MP * NT;
  constexpr int TN = NT * 16;
  // k-tile pairs in flight per wavefront (an unrolled loop that requests all
  // 8 pairs of K = 2048 at once is slower: 4.8 -> 5.3 us, registers)
  constexpr int PF =
      ((NT >= 4) ? 2 : (NT == 2 ? 3 : 4)) * WeightTile<WT>::kDepth;
  static_assert(ACC <= 16, "accumulator tile budget");
  // Small tiles: every wavefront parks its partial sums and one barrier
  // suffices; large tiles: two buffers and a tree (LDS budget).
  constexpr bool FLAT = ACC <= 4;
  __shared__ float red[FLAT ? 4 : 2][ACC * 4][64];
  T5D_GATE_READ(g.gate);

  // XCD-aware block mapping: the m_parts workgroups of one column group get
  // block ids 8 apart, i.e. the same XCD and adjacent dispatch slots.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int n_group = (slot / g.m_parts) * 8 + xcd;
  const int m_part = slot % g.m_parts;
  const int n_tiles_total = g.N >> 4;
  const int nt0 = n_group * NT;
  if (nt0 >= n_tiles_total) return;
  const int m0 = m_part * MP * 16;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int KT = g.K >> 5;
  const int n_pairs = (KT + 1) >> 1;
  const int nj = (n_pairs - wave + 3) >> 2;  // pairs owned by this wave

  f32x4_v acc[ACC];
#pragma unroll
  for (int i = 0; i < ACC; ++i) acc[i] = (f32x4_v){0.f, 0.f, 0.f, 0.f};

  const OperandLanes ol(lane);
  const int arow = ol.ld_row;
  const int akoff = ol.ld_piece * 8;
  const char* wbase = reinterpret_cast<const char*>(g.W);
  constexpr int TB = WeightTile<WT>::kTileBytes;

  typename WeightTile<WT>::Raw bq[PF][2][NT];
  auto load_b = [&](int slot_, int j) {
    const int kt = (wave + 4 * j) * 2;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int nn = 0; nn < NT; ++nn) {
        const int nt = nt0 + nn;
        if (NJ > 0)  // every k-tile exists; tiles past the edge are never stored
          bq[slot_][h][nn] = WeightTile<WT>::load(
              wbase + ((size_t)min(nt, n_tiles_total - 1) * KT + kt + h) * TB,
              lane);
        else if (nt < n_tiles_total && kt + h < KT)
          bq[slot_][h][nn] = WeightTile<WT>::load(
              wbase + ((size_t)nt * KT + kt + h) * TB, lane);
        else
          bq[slot_][h][nn] = WeightTile<WT>::zero();
      }
  };
  // The activation rows of a pair travel with its weight tiles (requested
  // together, PF pairs ahead): requested only when a pair is due, they would be
  // the newest loads in flight, and since loads return in order, waiting for
  // them would drain the whole weight queue once per pair.
  // (at most 64 registers of them: fewer pairs ahead for tall tiles)
  // (a divisor of PF: pair j then sits in slot j % APF in every round)
  constexpr int APF_CAP = PF * MP <= 8 ? PF : (8 / MP > 0 ? 8 / MP : 1);
  constexpr int APF = PF % APF_CAP == 0 ? APF_CAP
                      : (PF % (APF_CAP - 1) == 0 ? APF_CAP - 1
                         : (APF_CAP > 2 && PF % (APF_CAP - 2) == 0 ? APF_CAP - 2 : 1));
  static_assert(PF % APF == 0, "activation ring out of phase with the weight ring");
  uint4 aq[APF][2][MP];
  auto load_a = [&](int slot_, int j) {
    const int kt = (wave + 4 * j) * 2;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int mt = 0; mt < MP; ++mt) {
        const int row = m0 + mt * 16 + arow;
        if (NJ > 0)  // rows past the edge are never stored
          aq[slot_][h][mt] = *reinterpret_cast<const uint4*>(
              g.A + (size_t)min(row, g.M - 1) * g.K + (kt + h) * 32 + akoff);
        else if (row < g.M && kt + h < KT)
          aq[slot_][h][mt] = *reinterpret_cast<const uint4*>(
              g.A + (size_t)row * g.K + (kt + h) * 32 + akoff);
        else
          aq[slot_][h][mt] = make_uint4(0, 0, 0, 0);
      }
  };
#pragma unroll
  for (int p = 0; p < PF; ++p)
    if (NJ > 0 ? p < NJ : p < nj) {
      load_b(p, p);
      if (p < APF) load_a(p, p);
    }
  // The residual elements this thread will need in the epilogue.
  float res[FLAT ? ACC : 1];
  if (FLAT && g.epilogue == T5D_EPI_RESIDUAL) {
#pragma unroll
    for (int p = 0; p < (FLAT ? ACC : 0); ++p) {
      const int e = threadIdx.x + 256 * p;
      const int m = m0 + e / TN, n = nt0 * 16 + e % TN;
      res[p] = (m < g.M && n < g.N)
                   ? bf16_to_f32(reinterpret_cast<const bf16_t*>(
                         g.residual)[(size_t)m * g.N + n])
                   : 0.f;
    }
  }
  T5D_GATE_TEST();

  auto consume = [&](int pb_, int pa_) {
    Frag a[2][MP];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int mt = 0; mt < MP; ++mt)
        a[h][mt].u = ol.to_operand(aq[pa_][h][mt]);
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int mt = 0; mt < MP; ++mt)
#pragma unroll
        for (int nn = 0; nn < NT; ++nn)
          acc[mt * NT + nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              a[h][mt].v, WeightTile<WT>::frag(bq[pb_][h][nn]).v,
              acc[mt * NT + nn], 0, 0, 0);
  };
  if constexpr (NJ > 0) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      __builtin_amdgcn_sched_barrier(0);
      consume(j % PF, j % APF);
      __builtin_amdgcn_sched_barrier(0);
      if (j + PF < NJ) load_b(j % PF, j + PF);
      if (j + APF < NJ) load_a(j % APF, j + APF);
    }
  } else {
    for (int j0 = 0; j0 < nj; j0 += PF) {
#pragma unroll
      for (int p = 0; p < PF; ++p) {
        const int j = j0 + p;
        if (j < nj) {
          consume(p, p % APF);
          if (j + PF < nj) load_b(p, j + PF);
          if (j + APF < nj) load_a(p % APF, j + APF);
        }
      }
    }
  }

  // Cross-wave reduction in a fixed order: (w0 + w2) + (w1 + w3).
  // Accumulator element i of tile (mt, nn) in lane l is
  // C[16*mt + 4*(l/16) + i][16*nn + l%16].
  if constexpr (FLAT) {
#pragma unroll
    for (int t = 0; t < ACC; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][t * 4 + i][lane] = acc[t][i];
    __syncthreads();
  } else {
    if (wave >= 2) {
#pragma unroll
      for (int t = 0; t < ACC; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave - 2][t * 4 + i][lane] = acc[t][i];
    }
    __syncthreads();
    if (wave < 2) {
#pragma unroll
      for (int t = 0; t < ACC; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[t][i] += red[wave][t * 4 + i][lane];
    }
    __syncthreads();
    if (wave == 1) {
#pragma unroll
      for (int t = 0; t < ACC; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[0][t * 4 + i][lane] = acc[t][i];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int t = 0; t < ACC; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          red[1][t * 4 + i][lane] = acc[t][i] + red[0][t * 4 + i][lane];
    }
    __syncthreads();
  }

  const bool geglu = g.epilogue == T5D_EPI_GEGLU;
  auto tile_sum = [&](int ml, int nl) -> float {
    const int mt = ml >> 4, i = ml & 3, c = (ml & 15) >> 2;
    const int nn = nl >> 4, l = c * 16 + (nl & 15);
    const int idx = (mt * NT + nn) * 4 + i;
    if constexpr (FLAT)
      return (red[0][idx][l] + red[2][idx][l]) +
             (red[1][idx][l] + red[3][idx][l]);
    else
      return red[1][idx][l];
  };
  auto finish = [&](int e, float r) {
    const int ml = e / TN, nl = e % TN;
    const int m = m0 + ml, n = nt0 * 16 + nl;
    if (m >= g.M || n >= g.N) return;
    if (geglu && (nl & 8)) return;
    float v = tile_sum(ml, nl);
    float vg = geglu ? tile_sum(ml, nl + 8) : 0.f;
    if (g.scales) {
      v *= g.scales[n];
      if (geglu) vg *= g.scales[n + 8];
    }
    store_result(g, m, n, v, vg, r);
  };
  if constexpr (FLAT) {
#pragma unroll
    for (int p = 0; p < ACC; ++p) finish(threadIdx.x + 256 * p, res[p]);
  } else {
    for (int e = threadIdx.x; e < MP * 16 * TN; e += 256) {
      float r = 0.f;
      if (g.epilogue == T5D_EPI_RESIDUAL) {
        const int m = m0 + e / TN, n = nt0 * 16 + e % TN;
        if (m < g.M && n < g.N)
          r = bf16_to_f32(reinterpret_cast<const bf16_t*>(
              g.residual)[(size_t)m * g.N + n]);
      }
      finish(e, r);
    }
  }
}

// ---- layer norm + dense in one kernel -------------------------------------------
// y = bf16(bf16(x / rms(x)) * scale) feeds the matrix cores directly.  A
// workgroup owns 16 rows and NT column tiles; its 4 wavefronts split K in
// k-tile pairs exactly like gemm_mfma_kernel (same accumulation and summation
// order) and hold ALL their operand fragments in registers (K <= 256 * NJ;
// int8 weight tiles stay raw until they are multiplied), so
// the row statistics come from the fragments already loaded for the product:
// one exchange through LDS, no second pass over x, and only 16 rows per
// workgroup to normalise.
template <int NT, int NJ, typename WT>
__global__ void __launch_bounds__(256)
norm_gemm_kernel(GemmArgs g) {
  constexpr int TB = WeightTile<WT>::kTileBytes;
  constexpr int TN = NT * 16;
  __shared__ float red[4][NT * 4][64];
  __shared__ float s_ss[4][16];
  T5D_GATE_READ(g.gate);
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int n_group = (slot / g.m_parts) * 8 + xcd;
  const int m_part = slot % g.m_parts;
  const int n_tiles_total = g.N >> 4;
  const int nt0 = n_group * NT;
  if (nt0 >= n_tiles_total) return;
  const int m0 = m_part * 16;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Rows are loaded, measured and normalised in the load layout (lane l: piece
  // l % 4 of row l / 4) and moved to operand order just before the products.
  const OperandLanes ol(lane);
  const int n16 = ol.ld_row, gq = ol.ld_piece;
  const int KT = g.K >> 5, n_pairs = KT >> 1;
  const int row = m0 + n16;
  const bool row_ok = row < g.M;

  Frag xa[NJ][2];
  typename WeightTile<WT>::Raw wt[NJ][2][NT];
  uint4 lnv[NJ][2];
  {
    // Rows first, then the norm scale, then the weight tiles: loads return in
    // the order they were issued, and the row statistics need only the rows —
    // issued between the weight tiles they would wait for most of those too.
    const bf16_t* xrow = g.A + (size_t)(row_ok ? row : g.M - 1) * g.K + 8 * gq;
    const char* wbase = reinterpret_cast<const char*>(g.W);
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int kt = min((wave + 4 * j) * 2 + hh, KT - 1);
        xa[j][hh].u = *reinterpret_cast<const uint4*>(xrow + 32 * kt);
      }
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int kt = min((wave + 4 * j) * 2 + hh, KT - 1);
        lnv[j][hh] =
            *reinterpret_cast<const uint4*>(g.norm_scale + 32 * kt + 8 * gq);
      }
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int kt = min((wave + 4 * j) * 2 + hh, KT - 1);
#pragma unroll
        for (int nn = 0; nn < NT; ++nn)
          wt[j][hh][nn] = WeightTile<WT>::load(
              wbase + ((size_t)min(nt0 + nn, n_tiles_total - 1) * KT + kt) * TB,
              lane);
      }
  }
  T5D_GATE_TEST();

  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    if (wave + 4 * j < n_pairs) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        float f[8];
        unpack16(xa[j][hh].u, f);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
      }
    }
  }
  ss += dpp_move<kDppXor1>(ss);  // over the 4 pieces of the row
  ss += dpp_move<kDppXor2>(ss);
  if (gq == 0) s_ss[wave][n16] = ss;
  __syncthreads();
  const float tot = (s_ss[0][n16] + s_ss[2][n16]) + (s_ss[1][n16] + s_ss[3][n16]);
  const float inv = 1.0f / sqrtf(tot / (float)g.K + g.eps);

  f32x4_v acc[NT];
#pragma unroll
  for (int nn = 0; nn < NT; ++nn) acc[nn] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    if (wave + 4 * j < n_pairs) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        float xf[8], sf[8];
        unpack16(xa[j][hh].u, xf);
        unpack16(lnv[j][hh], sf);
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float y0 = round_bf16(xf[2 * e] * inv);
          const float y1 = round_bf16(xf[2 * e + 1] * inv);
          o[e] = pack_bf16x2(y0 * sf[2 * e], y1 * sf[2 * e + 1]);
        }
        Frag an;
        an.u = ol.to_operand(row_ok ? make_uint4(o[0], o[1], o[2], o[3])
                                    : make_uint4(0, 0, 0, 0));
#pragma unroll
        for (int nn = 0; nn < NT; ++nn)
          acc[nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              an.v, WeightTile<WT>::frag(wt[j][hh][nn]).v, acc[nn], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][t * 4 + i][lane] = acc[t][i];
  __syncthreads();

  const bool geglu = g.epilogue == T5D_EPI_GEGLU;
  auto tile_sum = [&](int ml, int nl) -> float {
    const int i = ml & 3, c = (ml & 15) >> 2;
    const int nn = nl >> 4, l = c * 16 + (nl & 15);
    const int idx = nn * 4 + i;
    return (red[0][idx][l] + red[2][idx][l]) + (red[1][idx][l] + red[3][idx][l]);
  };
#pragma unroll
  for (int p = 0; p < NT; ++p) {
    const int e = threadIdx.x + 256 * p;
    const int ml = e / TN, nl = e % TN;
    const int m = m0 + ml, n = nt0 * 16 + nl;
    if (m >= g.M || n >= g.N) continue;
    if (geglu && (nl & 8)) continue;
    float v = tile_sum(ml, nl);
    float vg = geglu ? tile_sum(ml, nl + 8) : 0.f;
    if (g.scales) {
      v *= g.scales[n];
      if (geglu) vg *= g.scales[n + 8];
    }
    store_result(g, m, n, v, vg, 0.f);
  }
}

// ---- layer norm + dense for a very wide layer (the vocabulary projection) -------
// With tens of thousands of output columns the kernels above re-read the
// activation rows once per column group, and those re-reads, not the weights,
// are most of what enters the CUs.  Here the rows stay put: a workgroup
// normalises 64 rows once, parks them in LDS in matrix-core operand order
// ([m-tile][k-tile][lane], read back without bank conflicts) and then walks
// over column groups of 128 (groups g0, g0 + G, ...), so that only weights
// stream.  A wavefront owns 2 column tiles of the group over ALL of K — no
// sum across wavefronts — and every operand it reads from LDS feeds two
// products.  The weight tiles of a whole group are in flight at once, in
// chunks of 8 k-tiles; a chunk's registers are refilled with the same chunk of
// the next group as soon as it is consumed.  The rows and the norm scale are
// requested BEFORE the weights: loads return in the order they were issued,
// so the normalisation runs while the weight tiles are still on their way.
// The two row halves of a 128-row call work on the same groups from the same
// XCD (block ids 8 apart), so the second read of a weight tile is served by
// that XCD's L2.  The code is kept small on purpose (one copy of the chunk
// loop and of the stores): it runs once or twice per workgroup, so every
// instruction is an instruction-cache miss.
constexpr int kWideCT = 2;     // column tiles per wavefront
constexpr int kWideChunk = 8;  // k-tiles per chunk
constexpr int kWideMinN = 8192;  // columns from which the wide kernel is used


template <int KT>
__global__ void __launch_bounds__(256)
norm_gemm_wide_kernel(GemmArgs g, int G, int halves) {
  static_assert(KT % kWideChunk == 0 && KT <= 32, "K of the wide kernel");
  constexpr int CT = kWideCT, CH = kWideChunk;
  constexpr int CPG = KT / CH;  // chunks per column group
  __shared__ uint4 s_a[4 * KT * 64];
  __shared__ uint4 s_scale[KT * 4];
  T5D_GATE_READ(g.gate);
  const int xcd = blockIdx.x & 7, s = blockIdx.x >> 3;
  const int half = s % halves;
  const int g0 = (s / halves) * 8 + xcd;
  const int n_tiles_total = g.N >> 4;
  const int n_groups = (n_tiles_total + 4 * CT - 1) / (4 * CT);
  if (g0 >= n_groups) return;
  const int m0 = half * 64;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n16 = lane & 15, gq = lane >> 4;

  // Rows of m-tile `wave` and the norm scale first ...  Lane l fetches piece
  // l % 8 (8 k) of a pair of k-tiles for rows l / 8 and 8 + l / 8: eight
  // neighbouring lanes read one 128-byte line (fetched in operand order, each
  // lane of a quarter wavefront would touch another row and the L1 would look
  // up 64 lines per instruction instead of 8).
  const int ld_r8 = lane >> 3, oct = lane & 7;
  bool row_ok[2];
  uint4 xa[2][KT / 2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = m0 + wave * 16 + 8 * i + ld_r8;
    row_ok[i] = row < g.M;
    const bf16_t* xrow = g.A + (size_t)(row_ok[i] ? row : g.M - 1) * g.K + 8 * oct;
#pragma unroll
    for (int j = 0; j < KT / 2; ++j)
      xa[i][j] = *reinterpret_cast<const uint4*>(xrow + 64 * j);
  }
  uint4 scale_part = make_uint4(0, 0, 0, 0);
  if (threadIdx.x < KT * 4)
    scale_part = reinterpret_cast<const uint4*>(g.norm_scale)[threadIdx.x];
  T5D_GATE_TEST();

  // ... then the weight tiles of the first group.
  const uint4* wbase = reinterpret_cast<const uint4*>(g.W);
  uint4 wq[CPG][CH][CT];
  auto load_chunk = [&](int ci, int grp) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int nt = min((grp * 4 + wave) * CT + ct, n_tiles_total - 1);
      const uint4* p = wbase + ((size_t)nt * KT + ci * CH) * 64 + lane;
#pragma unroll
      for (int k = 0; k < CH; ++k) wq[ci][k][ct] = p[k * 64];
    }
  };
  // (at most three chunks now, the rest once the rows have left the registers)
  constexpr int PRE = CPG < 2 ? CPG : 2;
  constexpr int MID = CPG < 3 ? CPG : 3;
#pragma unroll
  for (int ci = 0; ci < PRE; ++ci) load_chunk(ci, g0);

  if (threadIdx.x < KT * 4) s_scale[threadIdx.x] = scale_part;
  float inv[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < KT / 2; ++j) {
      float f[8];
      unpack16(xa[i][j], f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
    }
    ss += dpp_move<kDppXor1>(ss);  // over the 8 lanes that share the row
    ss += dpp_move<kDppXor2>(ss);
    ss += lane_xor4(ss);
    inv[i] = 1.0f / sqrtf(ss / (float)g.K + g.eps);
  }
  __syncthreads();
  // the rows have arrived: a third chunk can follow without delaying them
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int ci = PRE; ci < MID; ++ci) load_chunk(ci, g0);
  __builtin_amdgcn_sched_barrier(0);
  // Normalised pieces go to their operand slot (lane = row + 16 * piece of
  // k-tile 2 j + oct / 4), XOR-swizzled so that neither these writes nor the
  // operand reads below collide on LDS banks.  Scale reads in batches: one LDS
  // latency per batch, not one per piece.
  const int kt_lo = oct >> 2, piece = oct & 3;
  constexpr int JB = 4;
#pragma unroll
  for (int jb = 0; jb < KT / 2; jb += JB) {
    uint4 sc[JB];
#pragma unroll
    for (int jj = 0; jj < JB; ++jj) sc[jj] = s_scale[8 * (jb + jj) + oct];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int jj = 0; jj < JB; ++jj) {
      const int j = jb + jj;
      float sf[8];
      unpack16(sc[jj], sf);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        float xf[8];
        unpack16(xa[i][j], xf);
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float y0 = round_bf16(xf[2 * e] * inv[i]);
          const float y1 = round_bf16(xf[2 * e + 1] * inv[i]);
          o[e] = pack_bf16x2(y0 * sf[2 * e], y1 * sf[2 * e + 1]);
        }
        const int slot = (piece * 16 + 8 * i + ld_r8) ^ (2 * piece + kt_lo);
        s_a[(wave * KT + 2 * j + kt_lo) * 64 + slot] =
            row_ok[i] ? make_uint4(o[0], o[1], o[2], o[3])
                      : make_uint4(0, 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int ci = MID; ci < CPG; ++ci) load_chunk(ci, g0);
  __syncthreads();

  for (int grp = g0; grp < n_groups; grp += G) {
    f32x4_v acc[4][CT];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) acc[mt][ct] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
    const bool more = grp + G < n_groups;
    // The row operands of k-tile kk + 1 are read from LDS while the products
    // of k-tile kk run (two register sets, pinned in this order: left alone,
    // the compiler reads one operand, waits, multiplies, and pays the LDS
    // latency 4 * KT times per group).
    Frag af[2][4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
      af[0][mt].u = s_a[(mt * KT) * 64 + (lane ^ (2 * gq))];
#pragma unroll
    for (int ci = 0; ci < CPG; ++ci) {
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int kk = ci * CH + k;
        __builtin_amdgcn_sched_barrier(0);
        if (kk + 1 < KT) {
#pragma unroll
          for (int mt = 0; mt < 4; ++mt)
            af[(kk + 1) & 1][mt].u =
                s_a[(mt * KT + kk + 1) * 64 + (lane ^ (2 * gq + ((kk + 1) & 1)))];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
          for (int ct = 0; ct < CT; ++ct) {
            Frag b;
            b.u = wq[ci][k][ct];
            acc[mt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                af[kk & 1][mt].v, b.v, acc[mt][ct], 0, 0, 0);
          }
        }
      }
      // keep the refill behind the products that read these registers
      __builtin_amdgcn_sched_barrier(0);
      if (more) load_chunk(ci, grp + G);
      __builtin_amdgcn_sched_barrier(0);
    }
    // Accumulator element i of tile (mt, ct) in lane l is
    // C[16*mt + 4*(l/16) + i][16*ct + l%16].
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int nt = (grp * 4 + wave) * CT + ct;
      if (nt >= n_tiles_total) continue;
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int m = m0 + mt * 16 + 4 * gq + i;
          if (m >= g.M) continue;
          const size_t o = (size_t)m * g.N + nt * 16 + n16;
          if (g.out_f32)
            reinterpret_cast<float*>(g.C)[o] = acc[mt][ct][i];
          else
            reinterpret_cast<bf16_t*>(g.C)[o] = f32_to_bf16(acc[mt][ct][i]);
        }
    }
  }
}

// ---- float32 path (activation dtype float32, unpacked [K, N] kernel) ---------
// A workgroup owns 8 rows x 16 output columns: with a handful of rows the
// kernel is a stream of the weight matrix, and narrow column tiles are what
// spreads that stream over enough CUs (N / 16 workgroups).  Lane (c, s) =
// (column c of 16, k-subrange s of 4): per pass of 32 k it multiplies the 8 k
// of subrange s, every load of the pass in flight at once; the WV wavefronts
// split K in contiguous ranges.  Sums: ascending k inside a lane, then over
// the 4 subranges (rows_sum), then over the wavefronts in a fixed tree, so
// the result does not depend on how many rows a call carries.
// With `norm_scale` the rows are RMS-normalised on the way (T5 LayerNorm in
// front of the dense layer): the scale g_k multiplies the weights w_kn as they
// are loaded, the sum of squares of the row rides along with the products, and
// 1/rms, which is common to the whole row, multiplies the finished sum.
constexpr int kF32Rows = 8, kF32Cols = 16;

template <int WV, bool NORMED>
__global__ void __launch_bounds__(64 * WV)
gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ W,
                const float* __restrict__ residual, float* __restrict__ C,
                int M, int K, int N, int epilogue, const int32_t* gate,
                const float* __restrict__ norm_scale, float eps) {
  static_assert(WV == 4 || WV == 16, "wavefronts per workgroup");
  constexpr int MB = kF32Rows;
  constexpr int RW = WV == 4 ? 4 : 8;  // partial sums held in LDS at once
  __shared__ float red[RW][3 * MB][kF32Cols];
  T5D_GATED(gate);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, sub = lane >> 4;
  const bool geglu = epilogue == T5D_EPI_GEGLU;
  const int F = N >> 1;
  const int ncols = geglu ? F : N;  // columns of work
  const int n = blockIdx.x * kF32Cols + c;
  const int m0 = blockIdx.y * MB;
  const bool active = n < ncols;
  float acc0[MB], acc1[MB], ssq[MB];
#pragma unroll
  for (int m = 0; m < MB; ++m) acc0[m] = acc1[m] = ssq[m] = 0.f;
  constexpr bool normed = NORMED;
  // contiguous K ranges, multiples of 32 so that the 32-wide passes apply
  const int kq = ((K + WV - 1) / WV + 31) & ~31;
  const int kb = min(K, wave * kq), ke = min(K, kb + kq);
  int k = kb;
  if ((K & 31) == 0 && ((uintptr_t)A & 15) == 0) {
    for (; k + 32 <= ke; k += 32) {
      const int kk = k + 8 * sub;
      float w0[8], w1[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        w0[u] = active ? W[(size_t)(kk + u) * N + n] : 0.f;
        w1[u] = (active && geglu) ? W[(size_t)(kk + u) * N + F + n] : 0.f;
      }
      float4 ax[MB], ay[MB];
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const int row = m0 + m;
        ax[m] = ay[m] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (row < M) {
          const float4* ap =
              reinterpret_cast<const float4*>(A + (size_t)row * K + kk);
          ax[m] = ap[0];
          ay[m] = ap[1];
        }
      }
      if constexpr (normed) {
        const float4* gp = reinterpret_cast<const float4*>(norm_scale + kk);
        const float4 x = gp[0], y = gp[1];
        const float g[8] = {x.x, x.y, x.z, x.w, y.x, y.y, y.z, y.w};
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          w0[u] *= g[u];
          w1[u] *= g[u];
        }
      }
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const float a[8] = {ax[m].x, ax[m].y, ax[m].z, ax[m].w,
                            ay[m].x, ay[m].y, ay[m].z, ay[m].w};
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if constexpr (normed) ssq[m] = fmaf(a[u], a[u], ssq[m]);
          acc0[m] = fmaf(a[u], w0[u], acc0[m]);
          acc1[m] = fmaf(a[u], w1[u], acc1[m]);
        }
      }
    }
  }
  for (k += sub; k < ke; k += 4) {  // any K: one k per lane subrange
    float w0 = active ? W[(size_t)k * N + n] : 0.f;
    float w1 = (active && geglu) ? W[(size_t)k * N + F + n] : 0.f;
    if constexpr (normed) {
      w0 *= norm_scale[k];
      w1 *= norm_scale[k];
    }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const int row = m0 + m;
      const float a = row < M ? A[(size_t)row * K + k] : 0.f;
      if constexpr (normed) ssq[m] = fmaf(a, a, ssq[m]);
      acc0[m] = fmaf(a, w0, acc0[m]);
      acc1[m] = fmaf(a, w1, acc1[m]);
    }
  }
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    acc0[m] = rows_sum(acc0[m]);
    acc1[m] = rows_sum(acc1[m]);
    if constexpr (normed) ssq[m] = rows_sum(ssq[m]);
  }
  if constexpr (WV == 16) {
    // wavefronts 8..15 hand their sums to 0..7 first
    if (wave >= 8 && sub == 0) {
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        red[wave - 8][m][c] = acc0[m];
        red[wave - 8][MB + m][c] = acc1[m];
        red[wave - 8][2 * MB + m][c] = ssq[m];
      }
    }
    __syncthreads();
    if (wave < 8) {
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        acc0[m] += red[wave][m][c];
        acc1[m] += red[wave][MB + m][c];
        ssq[m] += red[wave][2 * MB + m][c];
      }
    }
    __syncthreads();
  }
  if (wave < RW && sub == 0) {
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      red[wave][m][c] = acc0[m];
      red[wave][MB + m][c] = acc1[m];
      red[wave][2 * MB + m][c] = ssq[m];
    }
  }
  __syncthreads();
  auto total = [&](int i, int l) -> float {
    float v = (red[0][i][l] + red[1][i][l]) + (red[2][i][l] + red[3][i][l]);
    if constexpr (RW == 8)
      v += (red[4][i][l] + red[5][i][l]) + (red[6][i][l] + red[7][i][l]);
    return v;
  };
  for (int e = threadIdx.x; e < MB * kF32Cols; e += 64 * WV) {
    const int m = e / kF32Cols, l = e % kF32Cols;
    const int col = blockIdx.x * kF32Cols + l;
    const int row = m0 + m;
    if (row >= M || col >= ncols) continue;
    float v = total(m, l);
    // every lane subrange saw its own k of the row: the total is the row's
    const float inv =
        normed ? 1.0f / sqrtf(total(2 * MB + m, l) / (float)K + eps) : 1.f;
    v *= inv;
    if (geglu) {
      float vg = total(MB + m, l) * inv;
      C[(size_t)row * F + col] = gelu_tanh(v) * vg;
    } else {
      if (epilogue == T5D_EPI_RESIDUAL) v += residual[(size_t)row * N + col];
      C[(size_t)row * N + col] = v;
    }
  }
}

// ---- weight packing -----------------------------------------------------------
template <typename WT>
__global__ void pack_weight_kernel(const WT* __restrict__ src,
                                   const WT* __restrict__ src2,
                                   WT* __restrict__ dst, int K, int N,
                                   int geglu) {
  // One thread per packed element; N here is the packed column count.
  const int KT = K >> 5;
  const size_t total = (size_t)K * N;
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int j = idx & 7;
  const int lane = (idx >> 3) & 63;
  const size_t tile = idx >> 9;
  const int kt = tile % KT;
  const int nt = tile / KT;
  const int k = kt * 32 + (lane >> 4) * 8 + j;
  const int c = lane & 15;
  WT v;
  if (geglu) {
    const int Nsrc = N >> 1;
    const int f = nt * 8 + (c & 7);
    v = (c < 8) ? src[(size_t)k * Nsrc + f] : src2[(size_t)k * Nsrc + f];
  } else {
    v = src[(size_t)k * N + nt * 16 + c];
  }
  dst[idx] = v;
}

// Pick the workgroup tile.  Model: the workgroups run in rounds of as many
// as are resident at once (256 CUs x the tile's occupancy, which its register
// count sets); a round costs a fixed latency plus the time one workgroup needs
// to pull its A and B bytes; all bytes entering the CUs share one aggregate
// rate.  w_bytes: bytes per weight element.
static int tile_occupancy(int mp, int nt) {
  // workgroups per CU = wavefronts per SIMD of gemm_mfma_kernel<mp, nt>
  // (from the registers the compiler reports for the bfloat16 instances)
  const int acc = mp * nt;
  if (acc == 1) return 5;
  if (acc <= 4) return mp == 1 ? 4 : 3;
  return acc == 8 && mp == 2 ? 3 : 2;
}

constexpr int kMaxRows = 128;  // rows one launch of the MFMA kernels covers

static GemmPlan plan_gemm(int M, int K, int N, int w_bytes) {
  const int mt_total = (M + 15) / 16;
  const int n_tiles = N / 16;
  GemmPlan best = {1, 1, 1, 1, 1, false};
  double best_cost = 1e30;
  const int mps[4] = {1, 2, 4, 8};
  const int nts[3] = {1, 2, 4};
  for (int mi = 0; mi < 4; ++mi)
    for (int ni = 0; ni < 3; ++ni) {
      const int mp = mps[mi], nt = nts[ni];
      if (mp * nt > 16) continue;
      if (mp > mt_total && mp != 1 && (mp >> 1) >= mt_total) continue;
      const int m_parts = (mt_total + mp - 1) / mp;
      const int n_groups = (n_tiles + nt - 1) / nt;
      const double wgs = (double)m_parts * n_groups;
      const double slots = 256.0 * tile_occupancy(mp, nt);
      const double rounds = (double)(long)((wgs + slots - 1) / slots);
      const double bytes = (double)K * (2.0 * mp * 16 + (double)w_bytes * nt * 16);
      const double cost = rounds * (3.0 + bytes / 40e3) + wgs * bytes / 40e6;
      if (cost < best_cost) {
        best_cost = cost;
        best = {mp, nt, m_parts, n_groups, 1, false};
      }
    }
  return best;
}

// CUs of the current device (256 on MI355X).
static int cu_count() {
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) !=
            hipSuccess || v <= 0)
      v = 256;
    n_cu = v;
  }
  return n_cu;
}

// Layers whose weights are at least this many bytes are planned for
// gemm_big_kernel; smaller ones are bound by launch latency and keep the
// small tiles (measured: the large-tile kernel is slower on every layer of
// T5.1.1-large and on the 4-21 MB layers of T5.1.1-XL with int8 weights).
constexpr double kBigWeightBytes = 24e6;
constexpr double kCuBytesPerUs = 45e3;   // what one CU takes in from L2

// Microseconds of a large-tile launch: rounds of one workgroup per CU, each
// lasting the bytes that workgroup reads over a CU's intake rate; the larger
// the accumulator tile, the fewer registers are left for loads in flight and
// the further the kernel stays below that rate (fitted to measurements).  A
// split over K additionally costs the kernel that adds the parts.
static double big_cost(int M, int K, int N, int w_bytes, int mp, int nt,
                       int k_parts) {
  const int mt_total = (M + 15) / 16, n_tiles = N / 16;
  const int m_parts = (mt_total + mp - 1) / mp;
  const int n_groups = (n_tiles + nt - 1) / nt;
  const double wgs = (double)m_parts * n_groups * k_parts;
  const double rounds = (double)(long)((wgs + cu_count() - 1) / cu_count());
  const double bytes = (double)K / k_parts *
                       (2.0 * min(mp * 16, M) + (double)w_bytes * nt * 16);
  double t = 4.0 + rounds * bytes * (1.0 + 0.012 * mp * nt) / kCuBytesPerUs;
  if (k_parts > 1) t += 4.5 + 2.0 * k_parts * (double)M * N * 4.0 / 4e6;
  return t;
}

// Tiles measured best for the layer shapes of the benchmark models (rows up
// to M, K, N, bytes per weight); the cost model covers everything else.
struct TunedTile { int M, K, N, wb, mp, nt; };
static const TunedTile kTunedTiles[] = {
    {128, 4096, 4096, 2, 2, 4},    // XXL attention projections: 18 us
    {128, 4096, 12288, 2, 4, 6},   // XXL q, k, v: 33 us
    {128, 4096, 20480, 2, 8, 5},   // XXL MLP in: 55 us
    {128, 10240, 4096, 2, 2, 4},   // XXL MLP out: 36 us
    {128, 4096, 32128, 2, 8, 8},   // XXL vocabulary projection: 65 us
    {64, 2048, 32128, 1, 4, 4},    // XL int8 vocabulary projection: 24 us
};

// The plan never splits K by itself: at these shapes the split was measured
// equal at best once the kernel that adds the parts is counted
// (K = 10240, N = 4096: 39.3 + finish against 40.1 us); t5d_gemm_tiled runs
// it on request.
static bool plan_big(int M, int K, int N, int w_bytes, GemmPlan* out) {
  if ((double)K * N * w_bytes < kBigWeightBytes || M < 32 || K < 2048)
    return false;
  const int mt_total = (M + 15) / 16, n_tiles = N / 16;
  for (const TunedTile& t : kTunedTiles)
    if (M <= t.M && 2 * M > t.M && K == t.K && N == t.N && w_bytes == t.wb) {
      *out = {t.mp, t.nt, (mt_total + t.mp - 1) / t.mp,
              (n_tiles + t.nt - 1) / t.nt, 1, true};
      return true;
    }
  double best_cost = 1e30;
  bool found = false;
  for (int mp = 2; mp <= 8; mp *= 2)
    for (int nt = 3; nt <= 8; ++nt) {
      if (!gemm_big_has_tile(mp, nt)) continue;
      if (mp > mt_total && (mp >> 1) >= mt_total) continue;
      const double c = big_cost(M, K, N, w_bytes, mp, nt, 1);
      if (c < best_cost) {
        best_cost = c;
        *out = {mp, nt, (mt_total + mp - 1) / mp, (n_tiles + nt - 1) / nt, 1,
                true};
        found = true;
      }
    }
  return found;
}

template <typename WT>
static void launch_mfma(const GemmPlan& p, GemmArgs g, hipStream_t s) {
  g.m_parts = p.m_parts;
  const int groups8 = (p.n_groups + 7) / 8 * 8;
  dim3 grid(groups8 * p.m_parts), block(256);
  // K loops of the benchmark models' layers that need refills, unrolled
  const int nj = g.K % 256 == 0 ? g.K / 256 : 0;
#define T5D_GEMM_NJ(MT, NT_, NJ_)                                           \
  if (p.mp == MT && p.nt == NT_ && nj == NJ_) {                             \
    hipLaunchKernelGGL((gemm_mfma_kernel<MT, NT_, WT, NJ_>), grid, block, 0, \
                       s, g);                                               \
    return;                                                                 \
  }
  T5D_GEMM_NJ(1, 1, 3) T5D_GEMM_NJ(1, 1, 4)
  T5D_GEMM_NJ(1, 1, 8) T5D_GEMM_NJ(1, 1, 11) T5D_GEMM_NJ(1, 1, 20)
  T5D_GEMM_NJ(1, 2, 8) T5D_GEMM_NJ(1, 4, 8)
#undef T5D_GEMM_NJ
#define T5D_GEMM_CASE(MT, NT_)                                              \
  if (p.mp == MT && p.nt == NT_) {                                          \
    hipLaunchKernelGGL((gemm_mfma_kernel<MT, NT_, WT>), grid, block, 0, s, g); \
    return;                                                                 \
  }
  T5D_GEMM_CASE(1, 1) T5D_GEMM_CASE(1, 2) T5D_GEMM_CASE(1, 4)
  T5D_GEMM_CASE(2, 1) T5D_GEMM_CASE(2, 2) T5D_GEMM_CASE(2, 4)
  T5D_GEMM_CASE(4, 1) T5D_GEMM_CASE(4, 2) T5D_GEMM_CASE(4, 4)
  T5D_GEMM_CASE(8, 1) T5D_GEMM_CASE(8, 2)
#undef T5D_GEMM_CASE
}

}  // namespace t5d

using namespace t5d;

bool t5d::norm_gemm_is_wide(int w_dtype, int K, int N) {
  return w_dtype == T5D_BF16 && N >= kWideMinN && N % 16 == 0 &&
         (K == 512 || K == 768 || K == 1024);
}

// One kernel shape for every M (rows in groups of 8 along grid.y), so the
// summation order, and with it every bit of the result, does not depend on
// how many rows a call carries.
static void launch_gemm_f32(hipStream_t s, const float* A, const float* W,
                            const float* residual, float* C, int M, int K,
                            int N, int epilogue, const float* norm_scale,
                            float eps) {
  const int ncols = epilogue == T5D_EPI_GEGLU ? N / 2 : N;
  dim3 grid((ncols + kF32Cols - 1) / kF32Cols, (M + kF32Rows - 1) / kF32Rows);
#define T5D_F32_LAUNCH(WV_, NORMED_)                                          \
  hipLaunchKernelGGL((gemm_f32_kernel<WV_, NORMED_>), grid, dim3(64 * WV_), 0, \
                     s, A, W, residual, C, M, K, N, epilogue, tls_gate,       \
                     norm_scale, eps)
  if (K >= 128) {
    if (norm_scale) T5D_F32_LAUNCH(16, true);
    else T5D_F32_LAUNCH(16, false);
  } else {
    if (norm_scale) T5D_F32_LAUNCH(4, true);
    else T5D_F32_LAUNCH(4, false);
  }
#undef T5D_F32_LAUNCH
}

extern "C" int64_t t5d_packed_weight_bytes(int w_dtype, int K, int N) {
  if (K <= 0 || N <= 0 || K % 32 || N % 16) return -1;
  if (w_dtype == T5D_BF16) return (int64_t)K * N * 2;
  if (w_dtype == T5D_I8) return (int64_t)K * N;
  return -1;
}

extern "C" int t5d_pack_weight(void* stream, int w_dtype, const void* src,
                               const void* src2, void* dst, int K, int N,
                               int geglu) {
  T5D_REQUIRE(w_dtype == T5D_BF16 || w_dtype == T5D_I8, T5D_EINVAL,
              "t5d_pack_weight: w_dtype %d", w_dtype);
  T5D_REQUIRE(src && dst && (!geglu || src2), T5D_EINVAL,
              "t5d_pack_weight: null pointer");
  const int Np = geglu ? 2 * N : N;
  T5D_REQUIRE(K > 0 && N > 0 && K % 32 == 0 && Np % 16 == 0 &&
                  (!geglu || N % 8 == 0),
              T5D_EINVAL, "t5d_pack_weight: K=%d N=%d must tile 32x16", K, N);
  const size_t total = (size_t)K * Np;
  const int threads = 256;
  const unsigned blocks = (unsigned)((total + threads - 1) / threads);
  if (w_dtype == T5D_BF16)
    hipLaunchKernelGGL(pack_weight_kernel<bf16_t>, dim3(blocks), dim3(threads),
                       0, as_stream(stream), (const bf16_t*)src,
                       (const bf16_t*)src2, (bf16_t*)dst, K, Np, geglu);
  else
    hipLaunchKernelGGL(pack_weight_kernel<int8_t>, dim3(blocks), dim3(threads),
                       0, as_stream(stream), (const int8_t*)src,
                       (const int8_t*)src2, (int8_t*)dst, K, Np, geglu);
  T5D_CHECK_LAUNCH("t5d_pack_weight");
  return T5D_OK;
}

extern "C" int64_t t5d_gemm_workspace_bytes(int dtype, int w_dtype, int M,
                                            int K, int N) {
  (void)dtype; (void)w_dtype; (void)M; (void)K; (void)N;
  return 0;  // no plan needs scratch memory (see plan_big)
}

extern "C" int t5d_gemm(void* stream, int dtype, int w_dtype, int out_dtype,
                        const void* A, const void* W, const float* scales,
                        const void* residual, void* C, int M, int K, int N,
                        int epilogue, void* workspace, int32_t* counters) {
  T5D_REQUIRE(A && W && C, T5D_EINVAL, "t5d_gemm: null pointer");
  T5D_REQUIRE(M > 0 && K > 0 && N > 0, T5D_EINVAL, "t5d_gemm: M=%d K=%d N=%d",
              M, K, N);
  T5D_REQUIRE(epilogue >= T5D_EPI_NONE && epilogue <= T5D_EPI_GEGLU,
              T5D_EINVAL, "t5d_gemm: epilogue %d", epilogue);
  T5D_REQUIRE(epilogue != T5D_EPI_RESIDUAL || residual, T5D_EINVAL,
              "t5d_gemm: residual epilogue without residual");
  T5D_REQUIRE(epilogue != T5D_EPI_GEGLU || N % 2 == 0, T5D_EINVAL,
              "t5d_gemm: geglu needs even N");
  hipStream_t s = as_stream(stream);
  if (dtype == T5D_F32) {
    T5D_REQUIRE(w_dtype == T5D_F32 && out_dtype == T5D_F32, T5D_EINVAL,
                "t5d_gemm: float32 activations need float32 weights/outputs");
    launch_gemm_f32(s, (const float*)A, (const float*)W, (const float*)residual,
                    (float*)C, M, K, N, epilogue, nullptr, 0.f);
    T5D_CHECK_LAUNCH("t5d_gemm(f32)");
    return T5D_OK;
  }
  T5D_REQUIRE(dtype == T5D_BF16, T5D_EINVAL, "t5d_gemm: dtype %d", dtype);
  T5D_REQUIRE(w_dtype == T5D_BF16 || w_dtype == T5D_I8, T5D_EINVAL,
              "t5d_gemm: w_dtype %d", w_dtype);
  T5D_REQUIRE(w_dtype != T5D_I8 || scales, T5D_EINVAL,
              "t5d_gemm: int8 weights need scales");
  T5D_REQUIRE(out_dtype == T5D_BF16 ||
                  (out_dtype == T5D_F32 && epilogue == T5D_EPI_NONE),
              T5D_EINVAL, "t5d_gemm: out_dtype %d with epilogue %d", out_dtype,
              epilogue);
  T5D_REQUIRE(K % 32 == 0 && N % 16 == 0, T5D_EINVAL,
              "t5d_gemm: K=%d N=%d must tile 32x16", K, N);
  T5D_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, T5D_EINVAL,
              "t5d_gemm: A/W must be 16-byte aligned");
  (void)counters;
  // The kernels cover up to kMaxRows rows; more rows go through in chunks
  // (each streams the weights again: beyond a few hundred rows t5d_gemm_rows
  // is the kernel to use).
  const int n_out = epilogue == T5D_EPI_GEGLU ? N / 2 : N;
  const size_t out_elem = out_dtype == T5D_F32 ? 4 : 2;
  const int wb = w_dtype == T5D_I8 ? 1 : 2;
  (void)workspace;
  for (int m0 = 0; m0 < M; m0 += kMaxRows) {
    const int mc = min(kMaxRows, M - m0);
    GemmPlan p;
    if (!plan_big(mc, K, N, wb, &p)) p = plan_gemm(mc, K, N, wb);
    GemmArgs g;
    g.A = (const bf16_t*)A + (size_t)m0 * K;
    g.W = W;
    g.scales = w_dtype == T5D_I8 ? scales : nullptr;
    g.residual = residual ? (const char*)residual + (size_t)m0 * n_out * 2
                          : nullptr;
    g.C = (char*)C + (size_t)m0 * n_out * out_elem;
    g.M = mc; g.K = K; g.N = N;
    g.m_parts = 1;
    g.gate = tls_gate;
    g.epilogue = epilogue;
    g.out_f32 = out_dtype == T5D_F32;
    g.norm_scale = nullptr;
    g.eps = 0.f;
    if (p.big) {
      launch_gemm_big(w_dtype, p, g, nullptr, s);
    } else if (w_dtype == T5D_BF16) {
      launch_mfma<bf16_t>(p, g, s);
    } else {
      launch_mfma<int8_t>(p, g, s);
    }
    T5D_CHECK_LAUNCH("t5d_gemm");
  }
  return T5D_OK;
}

// Shared argument checks of the bfloat16 MFMA entry points.
static int check_mfma_args(const char* name, int dtype, int w_dtype,
                           const void* A, const void* W, const float* scales,
                           int M, int K, int N) {
  T5D_REQUIRE(dtype == T5D_BF16 && (w_dtype == T5D_BF16 || w_dtype == T5D_I8),
              T5D_EINVAL,
              "%s: bfloat16 activations with packed bfloat16 or int8 weights",
              name);
  T5D_REQUIRE(A && W, T5D_EINVAL, "%s: null pointer", name);
  T5D_REQUIRE(w_dtype != T5D_I8 || scales, T5D_EINVAL,
              "%s: int8 weights need scales", name);
  T5D_REQUIRE(M > 0 && M <= kMaxRows && K > 0 && N > 0 && K % 32 == 0 &&
                  N % 16 == 0,
              T5D_EINVAL, "%s: M=%d (1..%d), K=%d N=%d must tile 32x16", name,
              M, kMaxRows, K, N);
  T5D_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, T5D_EINVAL,
              "%s: A/W must be 16-byte aligned", name);
  return T5D_OK;
}

extern "C" int t5d_gemm_tiled(void* stream, int dtype, int w_dtype,
                              int out_dtype, const void* A, const void* W,
                              const float* scales, const void* residual,
                              void* C, int M, int K, int N, int epilogue,
                              void* workspace, int mp, int nt, int k_parts) {
  int rc = check_mfma_args("t5d_gemm_tiled", dtype, w_dtype, A, W, scales, M, K,
                           N);
  if (rc != T5D_OK) return rc;
  T5D_REQUIRE(C && epilogue >= T5D_EPI_NONE && epilogue <= T5D_EPI_GEGLU &&
                  (epilogue != T5D_EPI_RESIDUAL || residual) &&
                  (out_dtype == T5D_BF16 ||
                   (out_dtype == T5D_F32 && epilogue == T5D_EPI_NONE)),
              T5D_EINVAL, "t5d_gemm_tiled: epilogue %d, out_dtype %d", epilogue,
              out_dtype);
  T5D_REQUIRE(gemm_big_has_tile(mp, nt), T5D_EINVAL,
              "t5d_gemm_tiled: no kernel for a tile of %d x %d", mp * 16,
              nt * 16);
  T5D_REQUIRE(k_parts >= 1 && k_parts <= 16, T5D_EINVAL,
              "t5d_gemm_tiled: k_parts=%d", k_parts);
  T5D_REQUIRE(k_parts == 1 ||
                  (workspace && epilogue == T5D_EPI_RESIDUAL && N % 8 == 0 &&
                   N <= 16384 &&
                   ((uintptr_t)workspace | (uintptr_t)residual | (uintptr_t)C) %
                           16 == 0),
              T5D_EINVAL,
              "t5d_gemm_tiled: a split over K needs a workspace, the residual "
              "epilogue, 16-byte aligned rows and N <= 16384");
  const int mt_total = (M + 15) / 16, n_tiles = N / 16;
  GemmPlan p = {mp, nt, (mt_total + mp - 1) / mp, (n_tiles + nt - 1) / nt,
                k_parts, true};
  GemmArgs g;
  g.A = (const bf16_t*)A; g.W = W;
  g.scales = w_dtype == T5D_I8 ? scales : nullptr;
  g.residual = residual; g.C = C;
  g.M = M; g.K = K; g.N = N; g.m_parts = p.m_parts;
  g.gate = tls_gate; g.epilogue = epilogue;
  g.out_f32 = out_dtype == T5D_F32;
  g.norm_scale = nullptr; g.eps = 0.f;
  hipStream_t s = as_stream(stream);
  launch_gemm_big(w_dtype, p, g, k_parts > 1 ? (float*)workspace : nullptr, s);
  T5D_CHECK_LAUNCH("t5d_gemm_tiled");
  if (k_parts > 1) {
    rc = launch_splitk_finish(s, (const float*)workspace, k_parts, g.scales,
                              residual, C, nullptr, nullptr, M, N, 0.f);
    if (rc != T5D_OK) return rc;
    T5D_CHECK_LAUNCH("t5d_gemm_tiled(finish)");
  }
  return T5D_OK;
}

extern "C" int t5d_norm_gemm(void* stream, int dtype, int w_dtype,
                             int out_dtype, const void* A,
                             const void* norm_scale, float eps, const void* W,
                             const float* scales, void* C, int M, int K, int N,
                             int epilogue) {
  T5D_REQUIRE(A && norm_scale && W && C, T5D_EINVAL,
              "t5d_norm_gemm: null pointer");
  if (dtype == T5D_BF16 && M > kMaxRows) {
    // in chunks of the rows the kernels cover (rows are independent)
    T5D_REQUIRE(epilogue == T5D_EPI_NONE || epilogue == T5D_EPI_GEGLU,
                T5D_EINVAL, "t5d_norm_gemm: epilogue %d (none or geglu)",
                epilogue);
    const int n_out = epilogue == T5D_EPI_GEGLU ? N / 2 : N;
    const size_t out_elem = out_dtype == T5D_F32 ? 4 : 2;
    for (int m0 = 0; m0 < M; m0 += kMaxRows) {
      const int rc = t5d_norm_gemm(
          stream, dtype, w_dtype, out_dtype, (const char*)A + (size_t)m0 * K * 2,
          norm_scale, eps, W, scales, (char*)C + (size_t)m0 * n_out * out_elem,
          min(kMaxRows, M - m0), K, N, epilogue);
      if (rc != T5D_OK) return rc;
    }
    return T5D_OK;
  }
  if (dtype == T5D_F32) {
    T5D_REQUIRE(w_dtype == T5D_F32 && out_dtype == T5D_F32, T5D_EINVAL,
                "t5d_norm_gemm: float32 activations need float32 weights / "
                "outputs");
    T5D_REQUIRE(epilogue == T5D_EPI_NONE ||
                    (epilogue == T5D_EPI_GEGLU && N % 2 == 0),
                T5D_EINVAL, "t5d_norm_gemm: epilogue %d (none or geglu), N=%d",
                epilogue, N);
    T5D_REQUIRE(M > 0 && K > 0 && N > 0, T5D_EINVAL,
                "t5d_norm_gemm: M=%d K=%d N=%d", M, K, N);
    T5D_REQUIRE(K % 32 != 0 || ((uintptr_t)norm_scale % 16) == 0, T5D_EINVAL,
                "t5d_norm_gemm: norm_scale must be 16-byte aligned");
    launch_gemm_f32(as_stream(stream), (const float*)A, (const float*)W,
                    nullptr, (float*)C, M, K, N, epilogue,
                    (const float*)norm_scale, eps);
    T5D_CHECK_LAUNCH("t5d_norm_gemm(f32)");
    return T5D_OK;
  }
  T5D_REQUIRE(dtype == T5D_BF16 && (w_dtype == T5D_BF16 || w_dtype == T5D_I8),
              T5D_EINVAL,
              "t5d_norm_gemm: bfloat16 activations with packed bfloat16 or int8 "
              "weights, or float32 with float32");
  T5D_REQUIRE(w_dtype != T5D_I8 || scales, T5D_EINVAL,
              "t5d_norm_gemm: int8 weights need scales");
  T5D_REQUIRE(out_dtype == T5D_BF16 ||
                  (out_dtype == T5D_F32 && epilogue == T5D_EPI_NONE),
              T5D_EINVAL, "t5d_norm_gemm: out_dtype %d with epilogue %d",
              out_dtype, epilogue);
  T5D_REQUIRE(epilogue == T5D_EPI_NONE || epilogue == T5D_EPI_GEGLU, T5D_EINVAL,
              "t5d_norm_gemm: epilogue %d (none or geglu)", epilogue);
  T5D_REQUIRE(M > 0, T5D_EINVAL, "t5d_norm_gemm: M=%d", M);
  T5D_REQUIRE(K >= 64 && K % 64 == 0 && K <= 2048 && N > 0 && N % 16 == 0,
              T5D_ELIMIT,
              "t5d_norm_gemm: K=%d (multiple of 64, <= 2048), N=%d (multiple "
              "of 16)", K, N);
  T5D_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 &&
                  ((uintptr_t)norm_scale % 16) == 0,
              T5D_EINVAL, "t5d_norm_gemm: operands must be 16-byte aligned");
  GemmArgs g;
  g.A = (const bf16_t*)A; g.W = W;
  g.scales = w_dtype == T5D_I8 ? scales : nullptr;
  g.residual = nullptr;
  g.C = C; g.M = M; g.K = K; g.N = N;
  g.m_parts = (M + 15) / 16;
  g.gate = tls_gate;
  g.epilogue = epilogue;
  g.out_f32 = out_dtype == T5D_F32;
  g.norm_scale = (const bf16_t*)norm_scale;
  g.eps = eps;
  const int n_tiles = N / 16;
  hipStream_t s = as_stream(stream);
  // Very wide layers (the vocabulary projection): rows resident in LDS, only
  // the weights stream.
  if (epilogue == T5D_EPI_NONE && norm_gemm_is_wide(w_dtype, K, N)) {
    const int halves = (M + 63) / 64;
    const int n_groups = (n_tiles + 4 * kWideCT - 1) / (4 * kWideCT);
    const int G = min((n_groups + 7) / 8 * 8, 256 / halves);
    dim3 grid(G * halves), block(256);
    if (K == 512)
      hipLaunchKernelGGL(norm_gemm_wide_kernel<16>, grid, block, 0, s, g, G, halves);
    else if (K == 768)
      hipLaunchKernelGGL(norm_gemm_wide_kernel<24>, grid, block, 0, s, g, G, halves);
    else
      hipLaunchKernelGGL(norm_gemm_wide_kernel<32>, grid, block, 0, s, g, G, halves);
    T5D_CHECK_LAUNCH("t5d_norm_gemm(wide)");
    return T5D_OK;
  }
  const int nj = (K / 64 + 3) / 4;  // k-tile pairs per wavefront
  // 64-column tiles unless that leaves too few workgroups to fill the chip;
  // beyond K = 1024 the fragments of fewer column tiles fit the registers
  // (bfloat16 weights: one, int8: two).
  int nt = (n_tiles / 4) * g.m_parts >= 256 ? 4 : (n_tiles >= 64 ? 2 : 1);
  if (nj > 4) nt = min(nt, w_dtype == T5D_I8 ? 2 : 1);
  const int n_groups = (n_tiles + nt - 1) / nt;
  dim3 grid((n_groups + 7) / 8 * 8 * g.m_parts), block(256);
#define T5D_NG_LAUNCH(NT_, NJ_, WT_)                                          \
  hipLaunchKernelGGL((norm_gemm_kernel<NT_, NJ_, WT_>), grid, block, 0, s, g)
#define T5D_NG_CASE(NT_, WT_)                                                 \
  if (nt == NT_) {                                                            \
    if (nj <= 3) T5D_NG_LAUNCH(NT_, 3, WT_);                                  \
    else if (nj <= 4) T5D_NG_LAUNCH(NT_, 4, WT_);                             \
  }
  if (w_dtype == T5D_BF16) {
    if (nj > 4) T5D_NG_LAUNCH(1, 8, bf16_t);
    T5D_NG_CASE(1, bf16_t) T5D_NG_CASE(2, bf16_t) T5D_NG_CASE(4, bf16_t)
  } else {
    if (nj > 4 && nt == 1) T5D_NG_LAUNCH(1, 8, int8_t);
    if (nj > 4 && nt == 2) T5D_NG_LAUNCH(2, 8, int8_t);
    T5D_NG_CASE(1, int8_t) T5D_NG_CASE(2, int8_t) T5D_NG_CASE(4, int8_t)
  }
#undef T5D_NG_CASE
#undef T5D_NG_LAUNCH
  T5D_CHECK_LAUNCH("t5d_norm_gemm");
  return T5D_OK;
}
