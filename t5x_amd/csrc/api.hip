// Error reporting, version, and the small element-wise kernels.
#include <stdarg.h>

#include "common.h"

namespace t5d {

static thread_local char g_error[512] = "";
thread_local const int32_t* tls_gate = nullptr;

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// ---- embedding gather --------------------------------------------------------
// One workgroup per row; 16-byte copies.
// ids == nullptr: the id of row r is seqs[r * S + *cur_index].
__global__ void embed_kernel(const uint4* __restrict__ table,
                             const int32_t* __restrict__ ids,
                             uint4* __restrict__ out, int vec_per_row, int V,
                             const int32_t* gate,
                             const int32_t* __restrict__ seqs,
                             const int32_t* __restrict__ cur_index, int S) {
  T5D_GATED(gate);
  const int r = blockIdx.x;
  int id = ids != nullptr ? ids[r] : seqs[(size_t)r * S + *cur_index];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  const uint4* src = table + (size_t)id * vec_per_row;
  uint4* dst = out + (size_t)r * vec_per_row;
  for (int i = threadIdx.x; i < vec_per_row; i += blockDim.x) dst[i] = src[i];
}

// ---- T5 RMS norm -------------------------------------------------------------
// One workgroup (256 threads) per row.  mean(x^2) in float32, two roundings to
// the activation dtype as in the reference.
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_kernel(const T* __restrict__ x, const T* __restrict__ scale,
               T* __restrict__ out, int d, float eps, const int32_t* gate) {
  T5D_GATE_READ(gate);
  __shared__ float partial[4];
  const int r = blockIdx.x;
  const T* xr = x + (size_t)r * d;
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += 256) {
    float v = Act<T>::load(xr + i);
    ss += v * v;
  }
  T5D_GATE_TEST();
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float total = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float inv = 1.0f / sqrtf(total / (float)d + eps);
  T* o = out + (size_t)r * d;
  for (int i = threadIdx.x; i < d; i += 256) {
    float y = Act<T>::round(Act<T>::load(xr + i) * inv);
    Act<T>::store(o + i, y * Act<T>::load(scale + i));
  }
}

// bfloat16 rows in 16-byte pieces: RPW rows per 256-thread workgroup, 256 / RPW
// threads per row (a wavefront per row when there are thousands of rows, the
// whole workgroup on one row when rows are few and long).  Same roundings as
// above; the row is read a second time for the output, from L1.
template <int RPW>
__global__ void __launch_bounds__(256)
rmsnorm_vec_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ scale,
                   bf16_t* __restrict__ out, int R, int d, float eps,
                   const int32_t* gate) {
  constexpr int TPR = 256 / RPW;  // threads per row
  static_assert(TPR == 64 || TPR == 256, "a wavefront or the workgroup per row");
  T5D_GATE_READ(gate);
  __shared__ float partial[4];
  const int t = threadIdx.x % TPR;
  const int r = blockIdx.x * RPW + threadIdx.x / TPR;
  const bool row_ok = r < R;  // uniform per wavefront
  const int chunks = d >> 3;
  const uint4* xr = reinterpret_cast<const uint4*>(x + (size_t)(row_ok ? r : 0) * d);
  float ss = 0.f;
  for (int c = t; c < chunks; c += TPR) {
    float f[8];
    unpack16(xr[c], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
  }
  T5D_GATE_TEST();
  ss = wave_sum(ss);
  if (TPR == 256) {
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  }
  if (!row_ok) return;
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  uint4* o = reinterpret_cast<uint4*>(out + (size_t)r * d);
  const uint4* sv = reinterpret_cast<const uint4*>(scale);
  for (int c = t; c < chunks; c += TPR) {
    float xf[8], sf[8];
    unpack16(xr[c], xf);
    unpack16(sv[c], sf);
    uint32_t y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      y[e] = pack_bf16x2(round_bf16(xf[2 * e] * inv) * sf[2 * e],
                         round_bf16(xf[2 * e + 1] * inv) * sf[2 * e + 1]);
    o[c] = make_uint4(y[0], y[1], y[2], y[3]);
  }
}

__global__ void add_i32_kernel(int32_t* x, int n, int delta,
                               const int32_t* gate) {
  T5D_GATED(gate);
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] += delta;
}

}  // namespace t5d

using namespace t5d;

extern "C" int t5d_version(void) { return 1; }
extern "C" const char* t5d_last_error(void) { return g_error; }

extern "C" int t5d_embed(void* stream, int dtype, const void* table,
                         const int32_t* ids, void* out, int R, int d, int V) {
  T5D_REQUIRE(dtype == T5D_F32 || dtype == T5D_BF16, T5D_EINVAL,
              "t5d_embed: dtype %d", dtype);
  T5D_REQUIRE(table && ids && out, T5D_EINVAL, "t5d_embed: null pointer");
  T5D_REQUIRE(R > 0 && d > 0 && V > 0, T5D_EINVAL, "t5d_embed: R=%d d=%d V=%d",
              R, d, V);
  const int esz = dtype == T5D_F32 ? 4 : 2;
  T5D_REQUIRE((d * esz) % 16 == 0, T5D_EINVAL,
              "t5d_embed: row bytes %d not a multiple of 16", d * esz);
  hipLaunchKernelGGL(embed_kernel, dim3(R), dim3(128), 0, as_stream(stream),
                     (const uint4*)table, ids, (uint4*)out, d * esz / 16, V,
                     tls_gate, nullptr, nullptr, 0);
  T5D_CHECK_LAUNCH("t5d_embed");
  return T5D_OK;
}

int t5d::launch_embed_from_seqs(hipStream_t s, int dtype, const void* table,
                                const int32_t* seqs, const int32_t* cur_index,
                                int S, void* out, int R, int d, int V) {
  T5D_REQUIRE(table && seqs && cur_index && out && R > 0 && S > 0, T5D_EINVAL,
              "embed(from sequences): null pointer or R=%d S=%d", R, S);
  const int esz = dtype == T5D_F32 ? 4 : 2;
  T5D_REQUIRE((d * esz) % 16 == 0, T5D_EINVAL,
              "embed: row bytes %d not a multiple of 16", d * esz);
  hipLaunchKernelGGL(embed_kernel, dim3(R), dim3(128), 0, s,
                     (const uint4*)table, (const int32_t*)nullptr, (uint4*)out,
                     d * esz / 16, V, tls_gate, seqs, cur_index, S);
  T5D_CHECK_LAUNCH("embed(from sequences)");
  return T5D_OK;
}

extern "C" int t5d_rmsnorm(void* stream, int dtype, const void* x,
                           const void* scale, void* out, int R, int d,
                           float eps) {
  T5D_REQUIRE(dtype == T5D_F32 || dtype == T5D_BF16, T5D_EINVAL,
              "t5d_rmsnorm: dtype %d", dtype);
  T5D_REQUIRE(x && scale && out, T5D_EINVAL, "t5d_rmsnorm: null pointer");
  T5D_REQUIRE(R > 0 && d > 0, T5D_EINVAL, "t5d_rmsnorm: R=%d d=%d", R, d);
  if (dtype == T5D_F32)
    hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(R), dim3(256), 0,
                       as_stream(stream), (const float*)x, (const float*)scale,
                       (float*)out, d, eps, tls_gate);
  else if (d % 8 == 0 && R >= 512 && ((uintptr_t)x | (uintptr_t)scale | (uintptr_t)out) % 16 == 0)
    hipLaunchKernelGGL(rmsnorm_vec_kernel<4>, dim3((R + 3) / 4), dim3(256), 0,
                       as_stream(stream), (const bf16_t*)x,
                       (const bf16_t*)scale, (bf16_t*)out, R, d, eps, tls_gate);
  else if (d % 8 == 0 && d >= 2048 && ((uintptr_t)x | (uintptr_t)scale | (uintptr_t)out) % 16 == 0)
    hipLaunchKernelGGL(rmsnorm_vec_kernel<1>, dim3(R), dim3(256), 0,
                       as_stream(stream), (const bf16_t*)x,
                       (const bf16_t*)scale, (bf16_t*)out, R, d, eps, tls_gate);
  else
    hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, dim3(R), dim3(256), 0,
                       as_stream(stream), (const bf16_t*)x,
                       (const bf16_t*)scale, (bf16_t*)out, d, eps, tls_gate);
  T5D_CHECK_LAUNCH("t5d_rmsnorm");
  return T5D_OK;
}

extern "C" int t5d_add_i32(void* stream, int32_t* x, int n, int delta) {
  T5D_REQUIRE(x && n > 0, T5D_EINVAL, "t5d_add_i32: x=%p n=%d", (void*)x, n);
  hipLaunchKernelGGL(add_i32_kernel, dim3((n + 63) / 64), dim3(64), 0,
                     as_stream(stream), x, n, delta, tls_gate);
  T5D_CHECK_LAUNCH("t5d_add_i32");
  return T5D_OK;
}
