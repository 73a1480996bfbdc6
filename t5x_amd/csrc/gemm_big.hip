// Dense layers of a few activation rows (M <= 128) with large workgroup tiles,
// and the consumer of their split-K parts.
#include "gemm_tiles.h"

namespace t5d {

// ---- large workgroup tiles ---------------------------------------------------
// What bounds a dense layer with thousands of columns AND thousands of input
// features at M <= 128 rows is not HBM but what a CU can take in: about 45
// bytes per ns from its XCD's L2, whatever the number of wavefronts (measured),
// so about 11.5 TB/s over the chip, and EVERY byte a workgroup reads counts —
// with a 32 x 64 tile the activation rows, re-read by every column group, are
// three times the weight bytes.  The time of a layer is therefore the bytes of
// its most loaded CU over that rate, and the tile to choose is the one that
// minimises 2 * K * rows + w * K * columns per workgroup with one workgroup on
// every CU.  This kernel is gemm_mfma_kernel with tiles of up to 128 rows x 128
// columns (one workgroup per CU, up to 512 registers per wavefront): the same
// split of K over the 4 wavefronts in k-tile pairs, the same accumulation and
// summation order — so the same bits — with the cross-wavefront sum going
// through LDS 8 accumulator tiles at a time.
//
// k_parts > 1 additionally splits K over workgroups: part z takes the k-tiles
// [z * kt_per, (z + 1) * kt_per) and writes its float32 sums, without scale or
// epilogue, to partials[z][M][N]; the kernel that consumes the layer's output
// (splitk_finish_kernel) adds the parts in ascending order.  No fences, no
// atomics: the hand-over is the kernel boundary.
template <int MP, int NT, typename WT, int NJ = 0>
__global__ void __launch_bounds__(256, 1)
gemm_big_kernel(GemmArgs g, int k_parts, float* __restrict__ partials) {
  constexpr int ACC = MP * NT;
  constexpr int CH = 8;  // accumulator tiles per reduction round
  constexpr int RAW = sizeof(typename WeightTile<WT>::Raw) / 4;
  // weight tiles in flight: 128 registers' worth, half that for the widest tile
  constexpr int PF0 = (NT >= 8 ? 64 : 128) / (2 * NT * RAW);
  constexpr int PF = PF0 < 1 ? 1 : (PF0 > 4 ? 4 : PF0);
  constexpr int APF0 = 64 / (2 * MP * 4);
  constexpr int APF = APF0 < 1 ? 1 : (APF0 > PF ? PF : APF0);
  static_assert(PF % APF == 0, "activation ring out of phase with the weight ring");
  __shared__ float red[4][CH * 4][64];
  T5D_GATE_READ(g.gate);

  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int per_group = g.m_parts * k_parts;
  const int n_group = (slot / per_group) * 8 + xcd;
  const int m_part = (slot % per_group) % g.m_parts;
  const int kz = (slot % per_group) / g.m_parts;
  const int n_tiles_total = g.N >> 4;
  const int nt0 = n_group * NT;
  if (nt0 >= n_tiles_total) return;
  const int m0 = m_part * MP * 16;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int KT = g.K >> 5;
  // k-tiles of this part (an even number per part, so pairs do not straddle)
  const int kt_per = (((KT + k_parts - 1) / k_parts) + 1) & ~1;
  const int kt_lo = kz * kt_per;
  const int kt_hi = min(KT, kt_lo + kt_per);
  const int n_pairs = kt_hi > kt_lo ? (kt_hi - kt_lo + 1) >> 1 : 0;
  const int nj = n_pairs > wave ? (n_pairs - wave + 3) >> 2 : 0;

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
    const int kt = kt_lo + (wave + 4 * j) * 2;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int nn = 0; nn < NT; ++nn) {
        const int nt = nt0 + nn;
        if (NJ > 0)  // every k-tile exists; tiles past the edge are never stored
          bq[slot_][h][nn] = WeightTile<WT>::load(
              wbase + ((size_t)min(nt, n_tiles_total - 1) * KT + kt + h) * TB,
              lane);
        else if (nt < n_tiles_total && kt + h < kt_hi)
          bq[slot_][h][nn] = WeightTile<WT>::load(
              wbase + ((size_t)nt * KT + kt + h) * TB, lane);
        else
          bq[slot_][h][nn] = WeightTile<WT>::zero();
      }
  };
  // (rings of whole k-tile pairs: single k-tiles as the unit, which would keep
  // more of a ring in flight, were measured 15-20 % slower: the wait the
  // compiler places per unit then drains the queue twice as often)
  uint4 aq[APF][2][MP];
  auto load_a = [&](int slot_, int j) {
    const int kt = kt_lo + (wave + 4 * j) * 2;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int mt = 0; mt < MP; ++mt) {
        const int row = m0 + mt * 16 + arow;
        if (NJ > 0)  // rows past the edge are never stored
          aq[slot_][h][mt] = *reinterpret_cast<const uint4*>(
              g.A + (size_t)min(row, g.M - 1) * g.K + (kt + h) * 32 + akoff);
        else if (row < g.M && kt + h < kt_hi)
          aq[slot_][h][mt] = *reinterpret_cast<const uint4*>(
              g.A + (size_t)row * g.K + (kt + h) * 32 + akoff);
        else
          aq[slot_][h][mt] = make_uint4(0, 0, 0, 0);
      }
  };
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
      for (int nn = 0; nn < NT; ++nn) {
        const Frag b = WeightTile<WT>::frag(bq[pb_][h][nn]);
#pragma unroll
        for (int mt = 0; mt < MP; ++mt)
          acc[mt * NT + nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              a[h][mt].v, b.v, acc[mt * NT + nn], 0, 0, 0);
      }
  };
  if constexpr (NJ > 0) {
    // Every wavefront has exactly NJ pairs: the whole K loop as straight-line
    // code, so the compiler counts the loads in flight exactly and waits for
    // the oldest pair only (a loop drains the queue at its head every round).
#pragma unroll
    for (int p = 0; p < PF; ++p)
      if (p < NJ) {
        load_b(p, p);
        if (p < APF) load_a(p, p);
      }
    T5D_GATE_TEST();
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      // (the fences keep the scheduler from sinking the refills down to their
      // use, which would leave one pair in flight)
      __builtin_amdgcn_sched_barrier(0);
      consume(j % PF, j % APF);
      __builtin_amdgcn_sched_barrier(0);
      if (j + PF < NJ) load_b(j % PF, j + PF);
      if (j + APF < NJ) load_a(j % APF, j + APF);
    }
  } else {
#pragma unroll
  for (int p = 0; p < PF; ++p)
    if (p < nj) {
      load_b(p, p);
      if (p < APF) load_a(p, p);
    }
  T5D_GATE_TEST();

  for (int j0 = 0; j0 < nj; j0 += PF) {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      const int j = j0 + p;
      if (j < nj) {
        Frag a[2][MP];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int mt = 0; mt < MP; ++mt)
            a[h][mt].u = ol.to_operand(aq[p % APF][h][mt]);
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int nn = 0; nn < NT; ++nn) {
            const Frag b = WeightTile<WT>::frag(bq[p][h][nn]);
#pragma unroll
            for (int mt = 0; mt < MP; ++mt)
              acc[mt * NT + nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  a[h][mt].v, b.v, acc[mt * NT + nn], 0, 0, 0);
          }
        if (j + PF < nj) load_b(p, j + PF);
        if (j + APF < nj) load_a(p % APF, j + APF);
      }
    }
  }
  }

  // Cross-wavefront sums, CH tiles per round: (w0 + w2) + (w1 + w3).  Thread
  // (ml, nl) = (tid / 16, tid % 16) finishes element (ml, nl) of every tile.
  const bool geglu = g.epilogue == T5D_EPI_GEGLU;
  const int ml = threadIdx.x >> 4, nl = threadIdx.x & 15;
  const int rl = ((ml >> 2) << 4) + nl, ri = ml & 3;
#pragma unroll
  for (int t0 = 0; t0 < ACC; t0 += CH) {
    if (t0 > 0) __syncthreads();
#pragma unroll
    for (int q = 0; q < CH; ++q)
      if (t0 + q < ACC) {
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][q * 4 + i][lane] = acc[t0 + q][i];
      }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      if (t0 + q >= ACC) continue;
      const int mt = (t0 + q) / NT, nn = (t0 + q) % NT;
      const int m = m0 + mt * 16 + ml, n = (nt0 + nn) * 16 + nl;
      if (m >= g.M || n >= g.N) continue;
      const int idx = q * 4 + ri;
      float v = (red[0][idx][rl] + red[2][idx][rl]) +
                (red[1][idx][rl] + red[3][idx][rl]);
      if (partials != nullptr) {
        partials[((size_t)kz * g.M + m) * g.N + n] = v;
        continue;
      }
      if (geglu && (nl & 8)) continue;
      float vg = geglu ? (red[0][idx][rl + 8] + red[2][idx][rl + 8]) +
                             (red[1][idx][rl + 8] + red[3][idx][rl + 8])
                       : 0.f;
      if (g.scales) {
        v *= g.scales[n];
        if (geglu) vg *= g.scales[n + 8];
      }
      float r = 0.f;
      if (g.epilogue == T5D_EPI_RESIDUAL)
        r = bf16_to_f32(
            reinterpret_cast<const bf16_t*>(g.residual)[(size_t)m * g.N + n]);
      store_result(g, m, n, v, vg, r);
    }
  }
}

// Consumer of gemm_big_kernel's split-K parts for a residual layer that is
// followed by a layer norm: y = bf16(sum of the parts [* scale]) + residual
// (the dense layer's epilogue), written to `out`, and the T5 RMS norm of y,
// written to `normed`, with the arithmetic of rmsnorm_vec_kernel<1> (so
// `normed` has the bits t5d_rmsnorm gives on `out`).  One workgroup per row;
// N a multiple of 8, at most 8 * 256 * VPT.  normed == nullptr: the sum and
// the epilogue only.
template <int VPT>
__global__ void __launch_bounds__(256)
splitk_finish_kernel(const float* __restrict__ partials, int k_parts,
                     const float* __restrict__ scales,
                     const bf16_t* __restrict__ residual,
                     bf16_t* __restrict__ out,
                     const bf16_t* __restrict__ norm_scale,
                     bf16_t* __restrict__ normed, int M, int N, float eps,
                     const int32_t* gate) {
  T5D_GATE_READ(gate);
  __shared__ float partial[4];
  const int r = blockIdx.x, t = threadIdx.x;
  const int chunks = N >> 3;
  float y[VPT][8];
  float ss = 0.f;
  T5D_GATE_TEST();
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
    const int c = t + 256 * u;
    if (c >= chunks) continue;
    float s[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) s[e] = 0.f;
    for (int z = 0; z < k_parts; ++z) {
      const float4* p = reinterpret_cast<const float4*>(
          partials + ((size_t)z * M + r) * N + 8 * c);
      const float4 a = p[0], b = p[1];
      s[0] += a.x; s[1] += a.y; s[2] += a.z; s[3] += a.w;
      s[4] += b.x; s[5] += b.y; s[6] += b.z; s[7] += b.w;
    }
    if (scales) {
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] *= scales[8 * c + e];
    }
    float res[8];
    unpack16(reinterpret_cast<const uint4*>(residual + (size_t)r * N)[c], res);
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      o[e] = pack_bf16x2(round_bf16(s[2 * e]) + res[2 * e],
                         round_bf16(s[2 * e + 1]) + res[2 * e + 1]);
    const uint4 ov = make_uint4(o[0], o[1], o[2], o[3]);
    reinterpret_cast<uint4*>(out + (size_t)r * N)[c] = ov;
    unpack16(ov, y[u]);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(y[u][e], y[u][e], ss);
  }
  if (normed == nullptr) return;
  ss = wave_sum(ss);
  if ((t & 63) == 0) partial[t >> 6] = ss;
  __syncthreads();
  ss = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float inv = 1.0f / sqrtf(ss / (float)N + eps);
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
    const int c = t + 256 * u;
    if (c >= chunks) continue;
    float sf[8];
    unpack16(reinterpret_cast<const uint4*>(norm_scale)[c], sf);
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      o[e] = pack_bf16x2(round_bf16(y[u][2 * e] * inv) * sf[2 * e],
                         round_bf16(y[u][2 * e + 1] * inv) * sf[2 * e + 1]);
    reinterpret_cast<uint4*>(normed + (size_t)r * N)[c] =
        make_uint4(o[0], o[1], o[2], o[3]);
  }
}


#define T5D_BIG_TILES(X) \
  X(2, 3) X(2, 4) X(2, 5) X(4, 4) X(4, 6) X(4, 8) X(8, 4) X(8, 5) X(8, 8)

bool gemm_big_has_tile(int mp, int nt) {
#define T5D_X(MP_, NT_) if (mp == MP_ && nt == NT_) return true;
  T5D_BIG_TILES(T5D_X)
#undef T5D_X
  return false;
}

void launch_gemm_big(int w_dtype, const GemmPlan& p, GemmArgs g,
                     float* partials, hipStream_t s) {
  g.m_parts = p.m_parts;
  const int groups8 = (p.n_groups + 7) / 8 * 8;
  const int kp = partials ? p.k_parts : 1;
  dim3 grid(groups8 * p.m_parts * kp), block(256);
  // Without a split and with K a multiple of 256 every wavefront has K / 256
  // k-tile pairs: the K loops of the benchmark models' widths are unrolled.
  const int nj = (kp == 1 && g.K % 256 == 0) ? g.K / 256 : 0;
#define T5D_X(MP_, NT_)                                                        \
  if (p.mp == MP_ && p.nt == NT_) {                                            \
    if (w_dtype != T5D_I8 && nj == 16) {                                       \
      hipLaunchKernelGGL((gemm_big_kernel<MP_, NT_, bf16_t, 16>), grid, block, \
                         0, s, g, kp, partials);                               \
      return;                                                                  \
    }                                                                          \
    if (w_dtype != T5D_I8 && nj == 40) {                                       \
      hipLaunchKernelGGL((gemm_big_kernel<MP_, NT_, bf16_t, 40>), grid, block, \
                         0, s, g, kp, partials);                               \
      return;                                                                  \
    }                                                                          \
  }
  T5D_BIG_TILES(T5D_X)
#undef T5D_X
  if (w_dtype == T5D_I8 && nj == 8 && p.mp == 4 && p.nt == 4) {
    hipLaunchKernelGGL((gemm_big_kernel<4, 4, int8_t, 8>), grid, block, 0, s, g,
                       kp, partials);
    return;
  }
#define T5D_X(MP_, NT_)                                                        \
  if (p.mp == MP_ && p.nt == NT_) {                                            \
    if (w_dtype == T5D_I8)                                                     \
      hipLaunchKernelGGL((gemm_big_kernel<MP_, NT_, int8_t>), grid, block, 0,  \
                         s, g, kp, partials);                                  \
    else                                                                       \
      hipLaunchKernelGGL((gemm_big_kernel<MP_, NT_, bf16_t>), grid, block, 0,  \
                         s, g, kp, partials);                                  \
    return;                                                                    \
  }
  T5D_BIG_TILES(T5D_X)
#undef T5D_X
}

int launch_splitk_finish(hipStream_t s, const float* partials, int k_parts,
                         const float* scales, const void* residual, void* out,
                         const void* norm_scale, void* normed, int M, int N,
                         float eps) {
  T5D_REQUIRE(N % 8 == 0 && N <= 8 * 256 * 8, T5D_ELIMIT,
              "split-K dense layer: N=%d (multiple of 8, <= 16384)", N);
  const int chunks = N / 8;
#define T5D_FIN(VPT_)                                                          \
  hipLaunchKernelGGL(splitk_finish_kernel<VPT_>, dim3(M), dim3(256), 0, s,     \
                     partials, k_parts, scales, (const bf16_t*)residual,       \
                     (bf16_t*)out, (const bf16_t*)norm_scale, (bf16_t*)normed, \
                     M, N, eps, tls_gate)
  if (chunks <= 256) T5D_FIN(1);
  else if (chunks <= 512) T5D_FIN(2);
  else if (chunks <= 1024) T5D_FIN(4);
  else T5D_FIN(8);
#undef T5D_FIN
  return T5D_OK;
}

}  // namespace t5d
