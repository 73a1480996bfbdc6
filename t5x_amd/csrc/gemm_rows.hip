// Dense layers over many rows (the encoder side: M = batch x encoder length).
//
// Unlike the decode-step GEMMs these are compute-bound.  A workgroup (4
// wavefronts, 2 x 2) owns a 128 x 128 output tile, each wavefront a 64 x 64
// sub-tile = 4 x 4 MFMA tiles (v_mfma_f32_16x16x32_bf16).  Both operands go
// straight from memory into MFMA operand registers, double-buffered over k:
// the weights are the same pre-packed 32 x 16 lane-major tiles the decode
// GEMMs use (one contiguous 1 KB load per tile), an activation fragment is 16
// rows x 64 contiguous bytes.  A packed weight tile has the same lane layout
// as either MFMA operand, so the product can be formed as C (activations as A)
// or as C^T (weights as A); C^T leaves every lane with 4 consecutive output
// COLUMNS of one row, C with 4 consecutive ROWS of one column — whichever makes
// the 8-byte stores contiguous in the requested output layout.
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

template <typename WT> struct RowsWeightTile;
template <> struct RowsWeightTile<bf16_t> {
  static constexpr int kTileBytes = 1024;
  __device__ static __forceinline__ FragR load(const char* tile, int lane) {
    FragR f;
    f.u = reinterpret_cast<const uint4*>(tile)[lane];
    return f;
  }
};
template <> struct RowsWeightTile<int8_t> {
  static constexpr int kTileBytes = 512;
  __device__ static __forceinline__ FragR load(const char* tile, int lane) {
    const uint2 q = reinterpret_cast<const uint2*>(tile)[lane];
    FragR f;
    f.u.x = i8x2_to_bf16x2((int8_t)(q.x), (int8_t)(q.x >> 8));
    f.u.y = i8x2_to_bf16x2((int8_t)(q.x >> 16), (int8_t)(q.x >> 24));
    f.u.z = i8x2_to_bf16x2((int8_t)(q.y), (int8_t)(q.y >> 8));
    f.u.w = i8x2_to_bf16x2((int8_t)(q.y >> 16), (int8_t)(q.y >> 24));
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

// SWAP: weights are the MFMA A operand (C^T is formed).
template <typename WT, bool SWAP>
__global__ void __launch_bounds__(256)
rows_gemm_kernel(RowsGemmArgs g) {
  constexpr int TB = RowsWeightTile<WT>::kTileBytes;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, gq = lane >> 4;
  const int m_blocks = (g.M + 127) >> 7;
  const int m_blk = blockIdx.x % m_blocks, n_blk = blockIdx.x / m_blocks;
  const int m0 = m_blk * 128 + (wave >> 1) * 64;
  const int nt0 = n_blk * 8 + (wave & 1) * 4;  // first 16-column tile
  const int KT = g.K >> 5, n_tiles = g.N >> 4;
  if (m0 >= g.M || nt0 >= n_tiles) return;

  const bf16_t* arow[4];
  const char* wtile[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    arow[t] = g.A + (size_t)min(m0 + 16 * t + l16, g.M - 1) * g.K + 8 * gq;
    wtile[t] = g.W + (size_t)min(nt0 + t, n_tiles - 1) * KT * TB;
  }
  f32x4_r acc[4][4];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = (f32x4_r){0.f, 0.f, 0.f, 0.f};

  FragR xa[2][4], wb[2][4];
  auto load = [&](int buf, int kt) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      xa[buf][t].u = *reinterpret_cast<const uint4*>(arow[t] + 32 * kt);
      wb[buf][t] = RowsWeightTile<WT>::load(wtile[t] + (size_t)kt * TB, lane);
    }
  };
  auto mma = [&](int buf) {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        if (SWAP)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              wb[buf][nt].v, xa[buf][mt].v, acc[mt][nt], 0, 0, 0);
        else
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              xa[buf][mt].v, wb[buf][nt].v, acc[mt][nt], 0, 0, 0);
      }
  };
  load(0, 0);
  for (int kt = 0; kt < KT; kt += 2) {
    if (kt + 1 < KT) load(1, kt + 1);
    mma(0);
    if (kt + 1 < KT) {
      if (kt + 2 < KT) load(0, kt + 2);
      mma(1);
    }
  }

  // ---- epilogue ---------------------------------------------------------------
  if (SWAP) {
    // acc[mt][nt][i]: row m = m0 + 16 mt + l16, column n = 16 (nt0 + nt) + 4 gq + i
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      const int m = m0 + 16 * mt + l16;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        if (nt0 + nt >= n_tiles) continue;
        const int n = 16 * (nt0 + nt) + 4 * gq;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = acc[mt][nt][i];
        if (g.scales) {
          const float4 sc = *reinterpret_cast<const float4*>(g.scales + n);
          v[0] *= sc.x; v[1] *= sc.y; v[2] *= sc.z; v[3] *= sc.w;
        }
        if (g.epilogue == T5D_EPI_GEGLU) {
          // tile columns 0..7 are wi_0, 8..15 the matching wi_1 columns: the
          // lanes with gq >= 2 hold the gates of the lanes with gq - 2.
          float gate[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) gate[i] = __shfl_xor(v[i], 32, 64);
          if (gq < 2 && m < g.M) {
            float h[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
              h[i] = round_bf16(round_bf16(gelu_tanh(round_bf16(v[i]))) *
                                round_bf16(gate[i]));
            const int F = g.N >> 1;
            *reinterpret_cast<uint2*>(g.C + (size_t)m * F + 8 * (nt0 + nt) +
                                      4 * gq) = pack4(h[0], h[1], h[2], h[3]);
          }
          continue;
        }
        if (m >= g.M) continue;
        size_t o;
        if (g.layout == T5D_OUT_HEADS_KEY) {
          const int b = m / g.E, e = m - b * g.E;
          const int hh = n >> 6, d = n & 63;
          o = (((size_t)b * g.H + hh) * g.Ep + e) * 64 + d;
        } else {
          o = (size_t)m * g.N + n;
        }
        if (g.epilogue == T5D_EPI_RESIDUAL) {
          const uint2 r = *reinterpret_cast<const uint2*>(
              g.residual + (size_t)m * g.N + n);
          v[0] = round_bf16(v[0]) + bf16lo_to_f32(r.x);
          v[1] = round_bf16(v[1]) + bf16hi_to_f32(r.x);
          v[2] = round_bf16(v[2]) + bf16lo_to_f32(r.y);
          v[3] = round_bf16(v[3]) + bf16hi_to_f32(r.y);
        }
        *reinterpret_cast<uint2*>(g.C + o) = pack4(v[0], v[1], v[2], v[3]);
      }
    }
  } else {
    // acc[mt][nt][i]: row m = m0 + 16 mt + 4 gq + i, column n = 16 (nt0 + nt) + l16
    // (values layout [B, H, 64, Ep]: 4 consecutive positions per store)
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      const int m = m0 + 16 * mt + 4 * gq;
      if (m >= g.M) continue;
      const int b = m / g.E, e = m - b * g.E;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        if (nt0 + nt >= n_tiles) continue;
        const int n = 16 * (nt0 + nt) + l16;
        float s = g.scales ? g.scales[n] : 1.f;
        const int hh = n >> 6, d = n & 63;
        const size_t o = (((size_t)b * g.H + hh) * 64 + d) * g.Ep + e;
        *reinterpret_cast<uint2*>(g.C + o) =
            pack4(acc[mt][nt][0] * s, acc[mt][nt][1] * s, acc[mt][nt][2] * s,
                  acc[mt][nt][3] * s);
      }
    }
  }
}

}  // namespace t5d

using namespace t5d;

extern "C" int t5d_gemm_rows(void* stream, int w_dtype, const void* A,
                             const void* W, const float* scales,
                             const void* residual, void* C, int64_t M, int K,
                             int N, int epilogue, int out_layout, int E,
                             int Ep) {
  T5D_REQUIRE(A && W && C, T5D_EINVAL, "t5d_gemm_rows: null pointer");
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
                    M % E == 0 && E % 4 == 0 && Ep % 4 == 0,
                T5D_EINVAL,
                "t5d_gemm_rows: heads layout needs epilogue none, N %% 64 == 0,"
                " M %% E == 0, E %% 4 == 0 (N=%d E=%d Ep=%d)", N, E, Ep);
    H = N / 64;
  }
  RowsGemmArgs g;
  g.A = (const bf16_t*)A; g.W = (const char*)W;
  g.scales = w_dtype == T5D_I8 ? scales : nullptr;
  g.residual = (const bf16_t*)residual; g.C = (bf16_t*)C;
  g.M = (int)M; g.K = K; g.N = N;
  g.epilogue = epilogue; g.layout = out_layout;
  g.E = E; g.Ep = Ep; g.H = H;
  const int m_blocks = ((int)M + 127) / 128, n_blocks = (N / 16 + 7) / 8;
  dim3 grid((unsigned)m_blocks * n_blocks), block(256);
  hipStream_t s = as_stream(stream);
  const bool swap = out_layout != T5D_OUT_HEADS_VALUE;
  if (w_dtype == T5D_BF16) {
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
