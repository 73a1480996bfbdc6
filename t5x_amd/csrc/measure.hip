// Measurement aids declared in include/t5d_measure.h: plain streaming kernels
// of known size.  No product path launches them.
#include "common.h"
#include "../../include/t5d_measure.h"

namespace t5d {

__global__ void __launch_bounds__(256)
measure_fill_kernel(uint4* __restrict__ p, size_t n, uint32_t seed) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
    p[i] = make_uint4(seed + (uint32_t)i, 1u, 2u, 3u);
}

// TAG only gives the launches of one measurement their own name in a kernel
// trace.
template <int TAG>
__global__ void __launch_bounds__(256)
measure_read_kernel(const uint4* __restrict__ p, size_t n, int shift,
                    uint32_t* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * 256;
  const size_t b = (blockIdx.x + (unsigned)shift) % gridDim.x;
  uint32_t acc = 0;
#pragma unroll 8
  for (size_t i = b * 256 + threadIdx.x; i < n; i += stride) {
    const uint4 v = p[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  // (never true for a buffer written by measure_fill_kernel: word y is 1)
  if (acc == 0xffffffffu) *sink = acc;
}

}  // namespace t5d

extern "C" int t5d_measure_fill(void* stream, void* buffer, long long bytes,
                                unsigned seed, int blocks) {
  using namespace t5d;
  T5D_REQUIRE(buffer != nullptr && bytes > 0 && bytes % 16 == 0 && blocks > 0,
              T5D_EINVAL, "t5d_measure_fill: bytes=%lld blocks=%d", bytes,
              blocks);
  hipLaunchKernelGGL(measure_fill_kernel, dim3(blocks), dim3(256), 0,
                     as_stream(stream), (uint4*)buffer, (size_t)(bytes / 16),
                     seed);
  T5D_CHECK_LAUNCH("t5d_measure_fill");
  return T5D_OK;
}

extern "C" int t5d_measure_read(void* stream, const void* buffer,
                                long long bytes, int shift, int blocks,
                                void* sink, int tag) {
  using namespace t5d;
  T5D_REQUIRE(buffer != nullptr && sink != nullptr && bytes > 0 &&
                  bytes % 16 == 0 && blocks > 0 && shift >= 0 && tag >= 0 &&
                  tag < 6,
              T5D_EINVAL,
              "t5d_measure_read: bytes=%lld blocks=%d shift=%d tag=%d", bytes,
              blocks, shift, tag);
#define T5D_READ(TAG_)                                                        \
  if (tag == TAG_)                                                            \
    hipLaunchKernelGGL(measure_read_kernel<TAG_>, dim3(blocks), dim3(256), 0, \
                       as_stream(stream), (const uint4*)buffer,               \
                       (size_t)(bytes / 16), shift, (uint32_t*)sink)
  T5D_READ(0); T5D_READ(1); T5D_READ(2); T5D_READ(3); T5D_READ(4); T5D_READ(5);
#undef T5D_READ
  T5D_CHECK_LAUNCH("t5d_measure_read");
  return T5D_OK;
}
