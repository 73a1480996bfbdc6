// What the dense kernels for a few activation rows share: the packed weight
// tile as it travels and as the matrix cores take it, the kernel arguments and
// the epilogue of one output element.
#ifndef T5D_GEMM_TILES_H_
#define T5D_GEMM_TILES_H_
#include "common.h"

namespace t5d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_v;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_v;

union Frag {
  uint4 u;
  bf16x8_v v;
};

__device__ __forceinline__ uint32_t pack_i8x2_to_bf16x2(int a, int b) {
  // int8 values are exactly representable in bfloat16.
  return pack_bf16x2((float)a, (float)b);
}

// A packed weight tile as it travels from memory (`Raw`, kept in registers
// while the load is in flight) and as the matrix cores take it (`Frag`).
// int8 tiles are half the bytes, so twice as many can be in flight (kDepth);
// they are widened only when consumed — converting at load time would put a
// wait for the load right behind it.
template <typename WT> struct WeightTile;
template <> struct WeightTile<bf16_t> {
  static constexpr int kTileBytes = 1024;
  static constexpr int kDepth = 1;
  typedef uint4 Raw;
  __device__ static __forceinline__ Raw load(const void* tile, int lane) {
    return reinterpret_cast<const uint4*>(tile)[lane];
  }
  __device__ static __forceinline__ Raw zero() { return make_uint4(0, 0, 0, 0); }
  __device__ static __forceinline__ Frag frag(const Raw& r) {
    Frag f;
    f.u = r;
    return f;
  }
};
template <> struct WeightTile<int8_t> {
  static constexpr int kTileBytes = 512;
  static constexpr int kDepth = 2;
  typedef uint2 Raw;
  __device__ static __forceinline__ Raw load(const void* tile, int lane) {
    return reinterpret_cast<const uint2*>(tile)[lane];
  }
  __device__ static __forceinline__ Raw zero() { return make_uint2(0, 0); }
  __device__ static __forceinline__ Frag frag(const Raw& q) {
    Frag f;
    f.u.x = pack_i8x2_to_bf16x2((int8_t)(q.x), (int8_t)(q.x >> 8));
    f.u.y = pack_i8x2_to_bf16x2((int8_t)(q.x >> 16), (int8_t)(q.x >> 24));
    f.u.z = pack_i8x2_to_bf16x2((int8_t)(q.y), (int8_t)(q.y >> 8));
    f.u.w = pack_i8x2_to_bf16x2((int8_t)(q.y >> 16), (int8_t)(q.y >> 24));
    return f;
  }
};

struct GemmArgs {
  const bf16_t* A;      // [M, K]
  const void* W;        // packed tiles
  const float* scales;  // [N] or null
  const void* residual; // [M, Nout] act dtype or null
  void* C;              // [M, Nout]
  int M, K, N;          // N = number of weight columns
  int m_parts;          // workgroups along M
  const int32_t* gate;  // optional device-side enable flag
  int epilogue;
  int out_f32;
  const bf16_t* norm_scale;  // norm_gemm_kernel: [K] layer-norm scale
  float eps;
};

// Apply scale + epilogue to one finished column (pair) of row m; `res` is the
// residual element (fetched early by the caller).
__device__ __forceinline__ void store_result(const GemmArgs& g, int m, int n,
                                             float v, float v_gate, float res) {
  if (g.epilogue == T5D_EPI_GEGLU) {
    const int f = (n >> 4) * 8 + (n & 7);
    const int F = g.N >> 1;
    float a0 = round_bf16(v), a1 = round_bf16(v_gate);
    float h = round_bf16(round_bf16(gelu_sigmoid_form(a0)) * a1);
    reinterpret_cast<bf16_t*>(g.C)[(size_t)m * F + f] = f32_to_bf16(h);
    return;
  }
  const size_t o = (size_t)m * g.N + n;
  if (g.out_f32) {
    reinterpret_cast<float*>(g.C)[o] = v;
    return;
  }
  if (g.epilogue == T5D_EPI_RESIDUAL) v = round_bf16(v) + res;
  reinterpret_cast<bf16_t*>(g.C)[o] = f32_to_bf16(v);
}


struct GemmPlan {
  int mp, nt, m_parts, n_groups;
  int k_parts;  // > 1: K split over workgroups (large tiles only)
  bool big;     // gemm_big_kernel instead of gemm_mfma_kernel
};

// Large-tile kernel (gemm_big.hip).  partials != nullptr: the float32 sums of
// the plan's k_parts parts go there, [k_parts][M][N], nothing else is written.
void launch_gemm_big(int w_dtype, const GemmPlan& p, GemmArgs g,
                     float* partials, hipStream_t s);
bool gemm_big_has_tile(int mp, int nt);
// Sum of split-K parts + scale + residual -> out, optional RMS norm -> normed.
int launch_splitk_finish(hipStream_t s, const float* partials, int k_parts,
                         const float* scales, const void* residual, void* out,
                         const void* norm_scale, void* normed, int M, int N,
                         float eps);

}  // namespace t5d
#endif  // T5D_GEMM_TILES_H_
