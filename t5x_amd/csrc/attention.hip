// Single-query ("decode step") attention over K/V stored [.., heads, 64, len]
// with `len` contiguous — the reference's cache layout
// (t5x/examples/t5/layers.py:226-241).
//
// The step is bound by streaming K and V once.  One workgroup handles one
// (row-or-batch-item, head); wavefront w owns key positions
// [w*BJ, (w+1)*BJ) (BJ = 128 bf16 / 64 f32 positions).  Inside a wavefront,
// lane = (dg, jc): jc = lane % 16 selects a 16-byte chunk of consecutive key
// positions, dg = lane / 16 selects head-dim rows d = dg + 4*i, i = 0..15.
// Every load instruction therefore fetches 4 rows x 256 contiguous bytes and
// only chunks that start inside the valid prefix are requested at all.
//   scores : per-lane FMAs over its 16 rows, then 2 xor-shuffles across dg;
//   softmax: 4 xor-shuffles across jc (+ an LDS exchange when several
//            wavefronts share the key axis); probabilities are normalised and
//            rounded to the activation dtype BEFORE the value product, as the
//            reference does;
//   P·V    : per-lane partial dot products, then a 15-step shuffle
//            reduce-scatter across jc leaves lane (dg, jc) holding output
//            element d = dg + 4*jc.
// NQ queries share the K/V stream (the beams of one batch item in
// cross-attention; 1 for self-attention, where each beam has its own cache).
#include <math.h>

#include "common.h"

namespace t5d {

struct AttnArgs {
  const void* q;        // self: qkv [R, 3*HD]; cross: q [R, HD]
  void* k;              // [G, H, 64, S]
  void* v;              // [G, H, 64, S]
  const void* rel_bias; // self: [H, S] by distance; cross: null
  const int32_t* index; // self: cache_index scalar; cross: enc_len [G]
  void* out;            // [R, HD]
  int H, S, nq, q_stride;
  const int32_t* gate;  // optional device-side enable flag
};

constexpr int kD = 64;
constexpr int kMaxWaves = 16;

// WM = the most wavefronts a launch of this instance uses; it bounds the
// workgroup size so short key axes get the full register file.
template <typename T, int NQ, bool SELF, int WM>
__global__ void __launch_bounds__(64 * WM)
attn_step_kernel(AttnArgs a) {
  constexpr int EL = Act<T>::kElemsPer16B;  // key positions per 16-byte chunk
  constexpr int BJ = 16 * EL;               // key positions per wavefront
  __shared__ float s_red[WM][NQ];
  __shared__ float s_out[WM][NQ][kD];
  T5D_GATED(a.gate);

  const int h = blockIdx.x, g = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nwaves = blockDim.x >> 6;
  const int jc = lane & 15, dg = lane >> 4;
  const int HD = a.H * kD;

  int n, t = 0;
  bool uniform = false;  // no valid key: the masked softmax is uniform
  // A cache index outside [0, S) (a decode loop longer than its cache) must
  // not become an address: nothing is inserted then and all S columns are
  // attended with the bias row of the last position, which is what the
  // reference's one-hot insert and clamped slices do (layers.py:258-303).
  bool past_end = false;
  if (SELF) {
    t = *a.index;
    past_end = t < 0 || t >= a.S;
    if (past_end) t = a.S - 1;
    n = t + 1;
  } else {
    n = a.index[g];
    n = n < 0 ? 0 : (n > a.S ? a.S : n);
    if (n == 0) { uniform = true; n = a.S; }
  }

  const int j0 = wave * BJ + jc * EL;
  const bool live = j0 < n;
  const T* kbase = reinterpret_cast<const T*>(a.k) +
                   ((size_t)g * a.H + h) * kD * a.S;
  const T* vbase = reinterpret_cast<const T*>(a.v) +
                   ((size_t)g * a.H + h) * kD * a.S;
  const T* qbase = reinterpret_cast<const T*>(a.q);

  // Queries: lane needs q[d] for its 16 rows.
  float qv[NQ][16];
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) {
    const int row = SELF ? g : g * a.nq + qi;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      qv[qi][i] = (qi < a.nq)
                      ? Act<T>::load(qbase + (size_t)row * a.q_stride + h * kD +
                                     dg + 4 * i)
                      : 0.f;
    }
  }

  // Self-attention: the lane whose chunk contains column t carries the new
  // key/value, patches its registers and writes the column to the cache.
  const bool ins = SELF && !past_end && live && (t >= j0) && (t < j0 + EL);
  const int e_t = t - j0;

  float s[NQ][EL];
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi)
#pragma unroll
    for (int e = 0; e < EL; ++e) s[qi][e] = 0.f;

  if (live) {
    uint4 kc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
      kc[i] = *reinterpret_cast<const uint4*>(kbase + (size_t)(dg + 4 * i) * a.S + j0);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float kf[EL];
      unpack16(kc[i], kf);
      if (SELF && ins) {
        const int d = dg + 4 * i;
        const T knew = qbase[(size_t)g * a.q_stride + HD + h * kD + d];
        const float kn = Act<T>::load(&knew);
#pragma unroll
        for (int e = 0; e < EL; ++e) kf[e] = (e == e_t) ? kn : kf[e];
        reinterpret_cast<T*>(a.k)[((size_t)g * a.H + h) * kD * a.S +
                                  (size_t)d * a.S + t] = knew;
      }
#pragma unroll
      for (int qi = 0; qi < NQ; ++qi)
#pragma unroll
        for (int e = 0; e < EL; ++e) s[qi][e] = fmaf(qv[qi][i], kf[e], s[qi][e]);
    }
  }

  // Issue the value loads now; they do not depend on the softmax.
  uint4 vc[16];
  if (live) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      vc[i] = *reinterpret_cast<const uint4*>(vbase + (size_t)(dg + 4 * i) * a.S + j0);
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) vc[i] = make_uint4(0, 0, 0, 0);
  }

  // Sum the partial dot products of the 4 row groups.
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi)
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      float x = s[qi][e];
      x += __shfl_xor(x, 16, 64);
      x += __shfl_xor(x, 32, 64);
      s[qi][e] = x;
    }

  // Bias, mask, running max.
  float mx[NQ];
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) {
    float m = -INFINITY;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const int j = j0 + e;
      float x = Act<T>::round(s[qi][e]);
      if (SELF) {
        if (j < n) {
          const float b = Act<T>::load(reinterpret_cast<const T*>(a.rel_bias) +
                                       (size_t)h * a.S + (t - j));
          x = Act<T>::round(x + b);
        }
      }
      if (uniform) x = 0.f;
      x = (j < n) ? x : -INFINITY;
      s[qi][e] = x;
      m = fmaxf(m, x);
    }
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    mx[qi] = m;
  }
  if (nwaves > 1) {
    if (lane == 0) {
#pragma unroll
      for (int qi = 0; qi < NQ; ++qi) s_red[wave][qi] = mx[qi];
    }
    __syncthreads();
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) {
      float m = s_red[0][qi];
      for (int w = 1; w < nwaves; ++w) m = fmaxf(m, s_red[w][qi]);
      mx[qi] = m;
    }
    __syncthreads();
  }

  // exp, sum, normalise, round to the activation dtype.
  float p[NQ][EL];
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) {
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const float x = s[qi][e];
      const float ex = (x == -INFINITY) ? 0.f : expf(x - mx[qi]);
      p[qi][e] = ex;
      sum += ex;
    }
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) sum += __shfl_xor(sum, o, 64);
    if (nwaves > 1) {
      if (lane == 0) s_red[wave][qi] = sum;
    } else {
#pragma unroll
      for (int e = 0; e < EL; ++e) p[qi][e] = Act<T>::round(p[qi][e] / sum);
    }
  }
  if (nwaves > 1) {
    __syncthreads();
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) {
      float sum = s_red[0][qi];
      for (int w = 1; w < nwaves; ++w) sum += s_red[w][qi];
#pragma unroll
      for (int e = 0; e < EL; ++e) p[qi][e] = Act<T>::round(p[qi][e] / sum);
    }
  }

  // P·V partial sums for this lane's 16 rows.
  float o[NQ][16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    float vf[EL];
    unpack16(vc[i], vf);
    if (SELF && ins) {
      const int d = dg + 4 * i;
      const T vnew = qbase[(size_t)g * a.q_stride + 2 * HD + h * kD + d];
      const float vn = Act<T>::load(&vnew);
#pragma unroll
      for (int e = 0; e < EL; ++e) vf[e] = (e == e_t) ? vn : vf[e];
      reinterpret_cast<T*>(a.v)[((size_t)g * a.H + h) * kD * a.S +
                                (size_t)d * a.S + t] = vnew;
    }
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) {
      float acc = 0.f;
#pragma unroll
      for (int e = 0; e < EL; ++e) {
        // A zero probability must not pick up whatever lies past the prefix.
        const float pe = p[qi][e];
        acc = fmaf(pe, pe != 0.f ? vf[e] : 0.f, acc);
      }
      o[qi][i] = acc;
    }
  }

  // Reduce-scatter across the 16 chunk lanes: afterwards o[qi][0] in lane
  // (dg, jc) is the sum over jc' of row index i = jc, i.e. d = dg + 4*jc.
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) {
#pragma unroll
    for (int st = 8; st >= 1; st >>= 1) {
      const bool up = (jc & st) != 0;
#pragma unroll
      for (int k2 = 0; k2 < st; ++k2) {
        const float mine = up ? o[qi][k2 + st] : o[qi][k2];
        const float other = up ? o[qi][k2] : o[qi][k2 + st];
        o[qi][k2] = mine + __shfl_xor(other, st, 64);
      }
    }
  }
  const int d_out = dg + 4 * jc;
  T* outp = reinterpret_cast<T*>(a.out);
  if (nwaves == 1) {
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) {
      if (qi < a.nq) {
        const int row = SELF ? g : g * a.nq + qi;
        Act<T>::store(outp + (size_t)row * HD + h * kD + d_out, o[qi][0]);
      }
    }
    return;
  }
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) s_out[wave][qi][d_out] = o[qi][0];
  __syncthreads();
  for (int e = threadIdx.x; e < NQ * kD; e += blockDim.x) {
    const int qi = e / kD, d = e % kD;
    if (qi >= a.nq) continue;
    float acc = s_out[0][qi][d];
    for (int w = 1; w < nwaves; ++w) acc += s_out[w][qi][d];
    const int row = SELF ? g : g * a.nq + qi;
    Act<T>::store(outp + (size_t)row * HD + h * kD + d, acc);
  }
}

// ---- float32 cross-attention -------------------------------------------------
// K is [B, H, E, 64] (head dim contiguous), V is [B, H, 64, E].  Lane = key
// position for the scores (a lane reads its own 256-byte K row), lane = head
// dim for the value product.  Float32 activations only occur in the small
// CPU-comparable configuration; this kernel favours clarity.
template <int NQ>
__global__ void __launch_bounds__(1024)
cross_attn_f32_kernel(AttnArgs a) {
  __shared__ float s_q[NQ][kD];
  __shared__ float s_red[kMaxWaves][NQ];
  __shared__ float s_p[NQ][kMaxWaves * 64];
  __shared__ float s_out[kMaxWaves][NQ][kD];
  T5D_GATED(a.gate);
  const int h = blockIdx.x, b = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nwaves = blockDim.x >> 6;
  const int HD = a.H * kD;
  int n = a.index[b];
  n = n < 0 ? 0 : (n > a.S ? a.S : n);
  bool uniform = false;
  if (n == 0) { uniform = true; n = a.S; }
  const float* kbase = reinterpret_cast<const float*>(a.k) +
                       ((size_t)b * a.H + h) * (size_t)a.S * kD;
  const float* vbase = reinterpret_cast<const float*>(a.v) +
                       ((size_t)b * a.H + h) * (size_t)kD * a.S;
  const float* qbase = reinterpret_cast<const float*>(a.q);
  for (int e = threadIdx.x; e < NQ * kD; e += blockDim.x) {
    const int qi = e / kD, d = e % kD;
    s_q[qi][d] = qi < a.nq
                     ? qbase[(size_t)(b * a.nq + qi) * a.q_stride + h * kD + d]
                     : 0.f;
  }
  __syncthreads();
  const int j = wave * 64 + lane;
  float s[NQ];
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) s[qi] = 0.f;
  if (j < n) {
    const float4* row = reinterpret_cast<const float4*>(kbase + (size_t)j * kD);
#pragma unroll
    for (int c = 0; c < kD / 4; ++c) {
      const float4 kv = row[c];
#pragma unroll
      for (int qi = 0; qi < NQ; ++qi) {
        s[qi] = fmaf(s_q[qi][4 * c + 0], kv.x, s[qi]);
        s[qi] = fmaf(s_q[qi][4 * c + 1], kv.y, s[qi]);
        s[qi] = fmaf(s_q[qi][4 * c + 2], kv.z, s[qi]);
        s[qi] = fmaf(s_q[qi][4 * c + 3], kv.w, s[qi]);
      }
    }
  }
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) {
    float x = uniform ? 0.f : s[qi];
    x = (j < n) ? x : -INFINITY;
    s[qi] = x;
    const float m = wave_max(x);
    if (lane == 0) s_red[wave][qi] = m;
  }
  __syncthreads();
  float ex[NQ];
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) {
    float m = s_red[0][qi];
    for (int w = 1; w < nwaves; ++w) m = fmaxf(m, s_red[w][qi]);
    ex[qi] = (s[qi] == -INFINITY) ? 0.f : expf(s[qi] - m);
  }
  __syncthreads();
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) {
    const float t = wave_sum(ex[qi]);
    if (lane == 0) s_red[wave][qi] = t;
  }
  __syncthreads();
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) {
    float t = s_red[0][qi];
    for (int w = 1; w < nwaves; ++w) t += s_red[w][qi];
    s_p[qi][j] = ex[qi] / t;
  }
  __syncthreads();
  // value product: lane = head dim, this wavefront's 64 positions
  float o[NQ];
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) o[qi] = 0.f;
  const int jb = wave * 64, je = min(n, jb + 64);
  for (int jj = jb; jj < je; ++jj) {
    const float v = vbase[(size_t)lane * a.S + jj];
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) o[qi] = fmaf(s_p[qi][jj], v, o[qi]);
  }
#pragma unroll
  for (int qi = 0; qi < NQ; ++qi) s_out[wave][qi][lane] = o[qi];
  __syncthreads();
  for (int e = threadIdx.x; e < NQ * kD; e += blockDim.x) {
    const int qi = e / kD, d = e % kD;
    if (qi >= a.nq) continue;
    float acc = s_out[0][qi][d];
    for (int w = 1; w < nwaves; ++w) acc += s_out[w][qi][d];
    reinterpret_cast<float*>(a.out)[(size_t)(b * a.nq + qi) * HD + h * kD + d] =
        acc;
  }
}

template <typename T, int NQ, bool SELF>
static void launch_attn_nq(const AttnArgs& a, int groups, hipStream_t s) {
  constexpr int BJ = 16 * Act<T>::kElemsPer16B;
  const int waves = (a.S + BJ - 1) / BJ;
  dim3 grid(a.H, groups), block(64 * waves);
  if (waves <= 4)
    hipLaunchKernelGGL((attn_step_kernel<T, NQ, SELF, 4>), grid, block, 0, s, a);
  else if (waves <= 8)
    hipLaunchKernelGGL((attn_step_kernel<T, NQ, SELF, 8>), grid, block, 0, s, a);
  else
    hipLaunchKernelGGL((attn_step_kernel<T, NQ, SELF, 16>), grid, block, 0, s, a);
}

static void launch_cross_f32(const AttnArgs& a, int B, hipStream_t s) {
  const int waves = (a.S + 63) / 64;
  dim3 grid(a.H, B), block(64 * waves);
  if (a.nq == 1) hipLaunchKernelGGL(cross_attn_f32_kernel<1>, grid, block, 0, s, a);
  else if (a.nq == 2) hipLaunchKernelGGL(cross_attn_f32_kernel<2>, grid, block, 0, s, a);
  else if (a.nq <= 4) hipLaunchKernelGGL(cross_attn_f32_kernel<4>, grid, block, 0, s, a);
  else hipLaunchKernelGGL(cross_attn_f32_kernel<8>, grid, block, 0, s, a);
}

int launch_cross_attention_bf16(hipStream_t s, const void* q, const void* k,
                                const void* v, const int32_t* enc_len,
                                void* out, int B, int beams, int H, int E,
                                const void* x, const void* ln, const void* wq,
                                int d, float eps, const int32_t* units);
int launch_self_attention_bf16(hipStream_t s, const void* qkv, void* ck,
                               void* cv, const void* rel_bias,
                               const int32_t* cache_index, void* out, int R,
                               int H, int L, const int32_t* pending,
                               const int32_t* pending_dst, int beams,
                               int value_blocked);

static int check_common(const char* name, int dtype, int H, int S) {
  T5D_REQUIRE(dtype == T5D_F32 || dtype == T5D_BF16, T5D_EINVAL, "%s: dtype %d",
              name, dtype);
  const int el = dtype == T5D_F32 ? 4 : 8;
  T5D_REQUIRE(H > 0 && S > 0 && S % el == 0, T5D_EINVAL,
              "%s: H=%d, length %d must be a positive multiple of %d", name, H,
              S, el);
  T5D_REQUIRE(S <= kMaxWaves * 16 * el, T5D_ELIMIT,
              "%s: length %d beyond the %d positions one workgroup covers",
              name, S, kMaxWaves * 16 * el);
  return T5D_OK;
}

}  // namespace t5d

using namespace t5d;

extern "C" int t5d_self_attention_step(void* stream, int dtype, const void* qkv,
                                       void* cached_key, void* cached_value,
                                       const void* rel_bias,
                                       const int32_t* cache_index, void* out,
                                       int R, int H, int L) {
  int rc = check_common("t5d_self_attention_step", dtype, H, L);
  if (rc) return rc;
  T5D_REQUIRE(qkv && cached_key && cached_value && rel_bias && cache_index &&
                  out && R > 0,
              T5D_EINVAL, "t5d_self_attention_step: null pointer or R=%d", R);
  T5D_REQUIRE(((uintptr_t)cached_key % 16) == 0 &&
                  ((uintptr_t)cached_value % 16) == 0,
              T5D_EINVAL, "t5d_self_attention_step: cache not 16-byte aligned");
  AttnArgs a;
  a.q = qkv; a.k = cached_key; a.v = cached_value; a.rel_bias = rel_bias;
  a.index = cache_index; a.out = out;
  a.H = H; a.S = L; a.nq = 1; a.q_stride = 3 * H * kD;
  a.gate = tls_gate;
  if (dtype == T5D_F32)
    launch_attn_nq<float, 1, true>(a, R, as_stream(stream));
  else
    launch_self_attention_bf16(as_stream(stream), qkv, cached_key, cached_value,
                               rel_bias, cache_index, out, R, H, L, nullptr,
                               nullptr, 1, 0);
  T5D_CHECK_LAUNCH("t5d_self_attention_step");
  return T5D_OK;
}

extern "C" int t5d_self_attention_step_gather(
    void* stream, int dtype, const void* qkv, void* cached_key,
    void* cached_value, const void* rel_bias, const int32_t* cache_index,
    void* out, int B, int beams, int H, int L, const int32_t* pending_src,
    const int32_t* pending_dst, int value_blocked) {
  int rc = check_common("t5d_self_attention_step_gather", dtype, H, L);
  if (rc) return rc;
  T5D_REQUIRE(dtype == T5D_BF16, T5D_EINVAL,
              "t5d_self_attention_step_gather: bfloat16 caches only");
  T5D_REQUIRE(qkv && cached_key && cached_value && rel_bias && cache_index &&
                  out && B > 0 && beams > 0,
              T5D_EINVAL,
              "t5d_self_attention_step_gather: null pointer or B=%d beams=%d", B,
              beams);
  T5D_REQUIRE(pending_src == nullptr ||
                  beams * ((L + 127) / 128) <= kMaxWaves,
              T5D_ELIMIT,
              "t5d_self_attention_step_gather: beams=%d x L=%d needs more than "
              "%d wavefronts per workgroup", beams, L, kMaxWaves);
  T5D_REQUIRE(pending_dst == nullptr || pending_src != nullptr, T5D_EINVAL,
              "t5d_self_attention_step_gather: pending_dst without pending_src");
  T5D_REQUIRE(value_blocked >= 0 && value_blocked <= 3, T5D_EINVAL,
              "t5d_self_attention_step_gather: value_blocked=%d", value_blocked);
  const bool in_place = pending_src != nullptr && pending_dst == nullptr;
  T5D_REQUIRE(value_blocked != 3 || L <= (in_place ? 128 : 256), T5D_ELIMIT,
              "t5d_self_attention_step_gather: the tail layout covers L <= %d "
              "%s (L=%d)", in_place ? 128 : 256,
              in_place ? "for a gather without destination slots" : "", L);
  T5D_REQUIRE(value_blocked != 3 || beams <= 8, T5D_ELIMIT,
              "t5d_self_attention_step_gather: beams=%d (tail layout: 1..8)",
              beams);
  T5D_REQUIRE(!value_blocked || L % 32 == 0, T5D_EINVAL,
              "t5d_self_attention_step_gather: blocked caches need L %% 32 == 0 "
              "(L=%d)", L);
  T5D_REQUIRE(((uintptr_t)cached_key % 16) == 0 &&
                  ((uintptr_t)cached_value % 16) == 0,
              T5D_EINVAL,
              "t5d_self_attention_step_gather: cache not 16-byte aligned");
  launch_self_attention_bf16(as_stream(stream), qkv, cached_key, cached_value,
                             rel_bias, cache_index, out, B * beams, H, L,
                             pending_src, pending_dst, beams, value_blocked);
  T5D_CHECK_LAUNCH("t5d_self_attention_step_gather");
  return T5D_OK;
}

extern "C" int t5d_cross_attention_step(void* stream, int dtype, const void* q,
                                        const void* cross_key,
                                        const void* cross_value,
                                        const int32_t* enc_len, void* out,
                                        int B, int beams, int H, int E,
                                        const int32_t* units) {
  int rc = check_common("t5d_cross_attention_step", dtype, H, E);
  if (rc) return rc;
  T5D_REQUIRE(units == nullptr || dtype == T5D_BF16, T5D_EINVAL,
              "t5d_cross_attention_step: a work order is for bfloat16 only");
  T5D_REQUIRE(q && cross_key && cross_value && enc_len && out && B > 0,
              T5D_EINVAL, "t5d_cross_attention_step: null pointer or B=%d", B);
  T5D_REQUIRE(beams >= 1 && beams <= 8, T5D_ELIMIT,
              "t5d_cross_attention_step: beams=%d (supported: 1..8)", beams);
  T5D_REQUIRE(((uintptr_t)cross_key % 16) == 0 &&
                  ((uintptr_t)cross_value % 16) == 0,
              T5D_EINVAL, "t5d_cross_attention_step: K/V not 16-byte aligned");
  AttnArgs a;
  a.q = q; a.k = const_cast<void*>(cross_key);
  a.v = const_cast<void*>(cross_value); a.rel_bias = nullptr;
  a.index = enc_len; a.out = out;
  a.H = H; a.S = E; a.nq = beams; a.q_stride = H * kD;
  a.gate = tls_gate;
  if (dtype == T5D_F32) {
    T5D_REQUIRE(E <= kMaxWaves * 64, T5D_ELIMIT,
                "t5d_cross_attention_step: float32 covers at most %d positions",
                kMaxWaves * 64);
    launch_cross_f32(a, B, as_stream(stream));
  } else {
    T5D_REQUIRE(E % 32 == 0, T5D_EINVAL,
                "t5d_cross_attention_step: bfloat16 K/V are stored in blocks of "
                "32 positions, E=%d", E);
    launch_cross_attention_bf16(as_stream(stream), q, cross_key, cross_value,
                                enc_len, out, B, beams, H, E, nullptr, nullptr,
                                nullptr, 0, 0.f, units);
  }
  T5D_CHECK_LAUNCH("t5d_cross_attention_step");
  return T5D_OK;
}

// ---- work order of the cross-attention workgroups ---------------------------------
// A cross-attention launch has one workgroup per (item, head) whose work grows
// with the item's valid encoder length.  The dispatcher deals workgroups out
// round-robin (position p goes to XCD p % 8 and, there, to CU (p / 8) % 32), two
// to a CU at most, so with more workgroups than CUs position p shares its CU
// with position p + n_cu, and the launch lasts as long as its most loaded CU.
// This kernel writes the order that evens the CUs out: the heaviest units sit
// alone on a CU, the rest are paired heaviest with lightest; launches of more
// than two rounds get the units by falling length.  One workgroup; B <= 256.
__global__ void __launch_bounds__(256)
cross_units_kernel(const int32_t* __restrict__ enc_len, int B, int H, int E,
                   int n_cu, int32_t* __restrict__ units) {
  __shared__ int s_len[256];
  __shared__ int s_item[256];  // items by falling length (ties: lower index)
  const int tid = threadIdx.x;
  if (tid < B) {
    const int n = enc_len[tid];
    s_len[tid] = n < 0 ? 0 : (n > E ? E : n);
  }
  __syncthreads();
  if (tid < B) {
    const int mine = s_len[tid];
    int rank = 0;
    for (int o = 0; o < B; ++o) {
      const int other = s_len[o];
      rank += (other > mine || (other == mine && o < tid)) ? 1 : 0;
    }
    s_item[rank] = tid;
  }
  __syncthreads();
  const int n = B * H;
  const int pairs = n - n_cu, alone = 2 * n_cu - n;
  for (int r = tid; r < n; r += 256) {
    const int b = s_item[r / H], h = r % H;
    int p = r;
    if (n > n_cu && n <= 2 * n_cu) {
      const int rr = r - alone;
      p = r < alone ? pairs + r : (rr < pairs ? rr : n_cu + (2 * pairs - 1 - rr));
    }
    // an item without a valid key keeps 0: the kernel then attends uniformly
    units[p] = h | (b << 8) | (int)((uint32_t)s_len[b] << 16);
  }
}

extern "C" int t5d_cross_attention_units(void* stream, const int32_t* enc_len,
                                         int B, int H, int E, int32_t* units) {
  T5D_REQUIRE(enc_len && units, T5D_EINVAL,
              "t5d_cross_attention_units: null pointer");
  T5D_REQUIRE(B > 0 && B <= 256 && H > 0 && H <= 256 && E > 0 && E < 32768,
              T5D_ELIMIT,
              "t5d_cross_attention_units: B=%d H=%d (1..256 each), E=%d "
              "(below 32768)", B, H, E);
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) !=
            hipSuccess || v <= 0)
      v = 256;
    n_cu = v;
  }
  hipLaunchKernelGGL(cross_units_kernel, dim3(1), dim3(256), 0,
                     as_stream(stream), enc_len, B, H, E, n_cu, units);
  T5D_CHECK_LAUNCH("t5d_cross_attention_units");
  return T5D_OK;
}

extern "C" int t5d_cross_attention_step_norm_q(
    void* stream, int dtype, int w_dtype, const void* x, const void* ln_scale,
    float eps, const void* query_kernel, const void* cross_key,
    const void* cross_value, const int32_t* enc_len, void* out, int B,
    int beams, int H, int E, int d, const int32_t* units) {
  int rc = check_common("t5d_cross_attention_step_norm_q", dtype, H, E);
  if (rc) return rc;
  T5D_REQUIRE(dtype == T5D_BF16 && w_dtype == T5D_BF16, T5D_EINVAL,
              "t5d_cross_attention_step_norm_q: bfloat16 activations and "
              "weights only");
  T5D_REQUIRE(x && ln_scale && query_kernel && cross_key && cross_value &&
                  enc_len && out && B > 0,
              T5D_EINVAL,
              "t5d_cross_attention_step_norm_q: null pointer or B=%d", B);
  T5D_REQUIRE(beams >= 1 && beams <= 8, T5D_ELIMIT,
              "t5d_cross_attention_step_norm_q: beams=%d (supported: 1..8)",
              beams);
  T5D_REQUIRE(E <= 512 && E % 32 == 0 && d >= 64 && d % 64 == 0 && d <= 1024,
              T5D_ELIMIT,
              "t5d_cross_attention_step_norm_q: E=%d (multiple of 32, <= 512), "
              "d=%d (multiple of 64, <= 1024)", E, d);
  T5D_REQUIRE(((uintptr_t)cross_key % 16) == 0 &&
                  ((uintptr_t)cross_value % 16) == 0 &&
                  ((uintptr_t)x % 16) == 0 && ((uintptr_t)ln_scale % 16) == 0 &&
                  ((uintptr_t)query_kernel % 16) == 0,
              T5D_EINVAL,
              "t5d_cross_attention_step_norm_q: operands not 16-byte aligned");
  launch_cross_attention_bf16(as_stream(stream), nullptr, cross_key, cross_value,
                              enc_len, out, B, beams, H, E, x, ln_scale,
                              query_kernel, d, eps, units);
  T5D_CHECK_LAUNCH("t5d_cross_attention_step_norm_q");
  return T5D_OK;
}
