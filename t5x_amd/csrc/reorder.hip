// In-place beam-axis gather of the self-attention caches.
//
// The caches are [B, beams, inner, L] with the beam axis second, so the gather
// is a permutation-with-repeats among the `beams` slices of one batch item.
// A thread owns one 16-byte column chunk of one (batch, inner-row) and moves
// it for all beams at once: every source is read into registers before any
// destination is written, which makes the in-place update safe without a
// second buffer.  Only chunks that intersect the valid prefix are touched, and
// batch items whose indices are the identity are skipped, so the traffic is
// the algorithmic 2 x valid-prefix bytes.
#include "common.h"

namespace t5d {

constexpr int kMaxGatherBeams = 8;

struct GatherArgs {
  char* cache;
  size_t tensor_stride;  // bytes
  const int32_t* idx;    // [B, beams]
  const int32_t* valid_len;
  int valid_off;
  int beams, inner, row_bytes, elem_bytes, L;
  const int32_t* gate;  // optional device-side enable flag
};

template <int BEAMS>
__global__ void __launch_bounds__(256)
cache_gather_kernel(GatherArgs a) {
  T5D_GATED(a.gate);
  const int b = blockIdx.y;
  int src[BEAMS];
  bool identity = true;
#pragma unroll
  for (int e = 0; e < BEAMS; ++e) {
    int s = a.idx[(size_t)b * BEAMS + e];
    s = s < 0 ? 0 : (s >= BEAMS ? BEAMS - 1 : s);
    src[e] = s;
    identity = identity && (s == e);
  }
  if (identity) return;
  int valid = a.L;
  if (a.valid_len) {
    valid = *a.valid_len + a.valid_off;
    valid = valid < 0 ? 0 : (valid > a.L ? a.L : valid);
  }
  const int chunks_valid = (valid * a.elem_bytes + 15) >> 4;
  const int chunks_row = a.row_bytes >> 4;
  const size_t total = (size_t)a.inner * chunks_valid;
  const size_t slice = (size_t)a.inner * a.row_bytes;  // one beam's bytes
  char* base = a.cache + (size_t)blockIdx.z * a.tensor_stride +
               (size_t)b * BEAMS * slice;
  for (size_t w = (size_t)blockIdx.x * 256 + threadIdx.x; w < total;
       w += (size_t)gridDim.x * 256) {
    const size_t row = w / chunks_valid;
    const int c = (int)(w % chunks_valid);
    const size_t off = (row * chunks_row + c) << 4;
    uint4 v[BEAMS];
#pragma unroll
    for (int e = 0; e < BEAMS; ++e)
      v[e] = *reinterpret_cast<const uint4*>(base + e * slice + off);
#pragma unroll
    for (int e = 0; e < BEAMS; ++e) {
      uint4 pick = v[0];
#pragma unroll
      for (int q = 1; q < BEAMS; ++q) pick = (src[e] == q) ? v[q] : pick;
      if (src[e] != e) *reinterpret_cast<uint4*>(base + e * slice + off) = pick;
    }
  }
}

}  // namespace t5d

using namespace t5d;

extern "C" int t5d_cache_gather_beams(void* stream, void* cache,
                                      int64_t tensor_stride_bytes,
                                      int n_tensors, int elem_bytes, int B,
                                      int beams, int inner, int L,
                                      const int32_t* beam_indices,
                                      const int32_t* valid_len,
                                      int valid_len_offset) {
  T5D_REQUIRE(cache && beam_indices, T5D_EINVAL,
              "t5d_cache_gather_beams: null pointer");
  T5D_REQUIRE(n_tensors > 0 && B > 0 && beams > 0 && inner > 0 && L > 0 &&
                  (elem_bytes == 2 || elem_bytes == 4),
              T5D_EINVAL,
              "t5d_cache_gather_beams: n=%d B=%d beams=%d inner=%d L=%d elem=%d",
              n_tensors, B, beams, inner, L, elem_bytes);
  T5D_REQUIRE(beams <= kMaxGatherBeams, T5D_ELIMIT,
              "t5d_cache_gather_beams: beams=%d > %d", beams, kMaxGatherBeams);
  T5D_REQUIRE((L * elem_bytes) % 16 == 0 && ((uintptr_t)cache % 16) == 0 &&
                  (tensor_stride_bytes % 16) == 0,
              T5D_EINVAL,
              "t5d_cache_gather_beams: rows must be 16-byte multiples/aligned");
  if (beams == 1) return T5D_OK;  // nothing to permute
  GatherArgs a;
  a.cache = (char*)cache;
  a.tensor_stride = (size_t)tensor_stride_bytes;
  a.idx = beam_indices;
  a.valid_len = valid_len;
  a.valid_off = valid_len_offset;
  a.beams = beams; a.inner = inner; a.row_bytes = L * elem_bytes;
  a.elem_bytes = elem_bytes; a.L = L;
  a.gate = tls_gate;
  const size_t work = (size_t)inner * (a.row_bytes / 16);
  int gx = (int)((work + 255) / 256);
  gx = gx < 1 ? 1 : (gx > 256 ? 256 : gx);
  dim3 grid(gx, B, n_tensors), block(256);
  hipStream_t s = as_stream(stream);
  switch (beams) {
#define T5D_GATHER_CASE(N)                                                   \
  case N:                                                                    \
    hipLaunchKernelGGL(cache_gather_kernel<N>, grid, block, 0, s, a);        \
    break;
    T5D_GATHER_CASE(2) T5D_GATHER_CASE(3) T5D_GATHER_CASE(4)
    T5D_GATHER_CASE(5) T5D_GATHER_CASE(6) T5D_GATHER_CASE(7)
    T5D_GATHER_CASE(8)
#undef T5D_GATHER_CASE
  }
  T5D_CHECK_LAUNCH("t5d_cache_gather_beams");
  return T5D_OK;
}
