// Shared helpers for the t5d HIP kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/t5d.h"

namespace t5d {

// ---- error reporting --------------------------------------------------------
void set_error(const char* fmt, ...);

#define T5D_REQUIRE(cond, code, ...)      \
  do {                                    \
    if (!(cond)) {                        \
      ::t5d::set_error(__VA_ARGS__);      \
      return (code);                      \
    }                                     \
  } while (0)

#define T5D_CHECK_LAUNCH(name)                                            \
  do {                                                                    \
    hipError_t e_ = hipGetLastError();                                    \
    if (e_ != hipSuccess) {                                               \
      ::t5d::set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return T5D_EHIP;                                                    \
    }                                                                     \
  } while (0)

// ---- bfloat16 <-> float32 ---------------------------------------------------
typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}
__device__ __forceinline__ float bf16lo_to_f32(uint32_t packed) {
  return __uint_as_float(packed << 16);
}
__device__ __forceinline__ float bf16hi_to_f32(uint32_t packed) {
  return __uint_as_float(packed & 0xFFFF0000u);
}
// Round to nearest even with the hardware conversion (v_cvt_pk_bf16_f32).
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_v;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_v;
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float round_bf16(float f) {
  return __uint_as_float(((uint32_t)f32_to_bf16(f)) << 16);
}
// Two values rounded and packed (lo in bits 0..15) by one instruction.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_v v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_v));
}

// Activation-dtype traits: how a value is rounded / loaded / stored.
template <typename T> struct Act;
template <> struct Act<float> {
  static constexpr int kElemsPer16B = 4;
  __device__ static __forceinline__ float round(float v) { return v; }
  __device__ static __forceinline__ float load(const float* p) { return *p; }
  __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Act<bf16_t> {
  static constexpr int kElemsPer16B = 8;
  __device__ static __forceinline__ float round(float v) { return round_bf16(v); }
  __device__ static __forceinline__ float load(const bf16_t* p) {
    return bf16_to_f32(*p);
  }
  __device__ static __forceinline__ void store(bf16_t* p, float v) {
    *p = f32_to_bf16(v);
  }
};

// Unpack a 16-byte vector of activations into floats.
__device__ __forceinline__ void unpack16(const uint4& v, float (&f)[8]) {
  f[0] = bf16lo_to_f32(v.x); f[1] = bf16hi_to_f32(v.x);
  f[2] = bf16lo_to_f32(v.y); f[3] = bf16hi_to_f32(v.y);
  f[4] = bf16lo_to_f32(v.z); f[5] = bf16hi_to_f32(v.z);
  f[6] = bf16lo_to_f32(v.w); f[7] = bf16hi_to_f32(v.w);
}
__device__ __forceinline__ void unpack16(const uint4& v, float (&f)[4]) {
  f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
  f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
}

// ---- wavefront (64 lanes) reductions ---------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// T5 tanh-approximate GELU in float32.
__device__ __forceinline__ float gelu_tanh(float x) {
  const float c = 0.7978845608028654f;  // sqrt(2/pi)
  return x * (0.5f * (1.0f + tanhf(c * (x + 0.044715f * (x * x * x)))));
}

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Optional device-side gate.  While a fused multi-kernel entry point is
// enqueueing work it publishes a pointer to an int32 flag here; every kernel
// launched by this thread then receives it and returns immediately when the
// flag is 0.  This lets a decode loop run several steps per host
// synchronisation: once the loop condition turns false on the device, the
// remaining enqueued steps are no-ops.  Null outside fused entry points.
extern thread_local const int32_t* tls_gate;
#define T5D_GATED(gate) \
  if ((gate) != nullptr && *(gate) == 0) return
// Two-part form: read the flag first, test it after the kernel has issued its
// first (side-effect free) loads, so the flag's memory latency overlaps theirs.
#define T5D_GATE_READ(gate) \
  const int t5d_gate_open_ = (gate) != nullptr ? *(gate) : 1
#define T5D_GATE_TEST() \
  if (t5d_gate_open_ == 0) return

// ---- internal launches used by the fused step (not part of the C ABI) -------
// Embedding rows of the current tokens, read straight from the sequences:
// ids[r] = seqs[r, *cur_index] (t5d_gather_step_ids + t5d_embed in one kernel).
int launch_embed_from_seqs(hipStream_t s, int dtype, const void* table,
                           const int32_t* seqs, const int32_t* cur_index,
                           int S, void* out, int R, int d, int V);
// log_softmax + prefix add + per-row top-2K, then one kernel that merges the
// rows' candidates and does all the beam bookkeeping of the iteration
// (t5d_beam_topk + t5d_beam_update without the index advance).
int launch_beam_select(hipStream_t s, const float* logits,
                       const t5d_beam_state* st, float* topk_vals,
                       int32_t* topk_idx, float* row_max, float* row_lse,
                       void* scratch, const int32_t* inputs,
                       const int32_t* initial_index, const float* brevity,
                       int32_t* top_alive, int B, int K, int S, int Lin, int V,
                       int eos_id);
// End of a beam-search iteration in one single-workgroup kernel: advance
// *state.cur_index, add 1 to `counters[0..n_counters)` (the layers' cache
// indices), and, if do_cond, evaluate the loop condition into *keep_going.
int launch_beam_tail(hipStream_t s, const t5d_beam_state* state, int B, int K,
                     int S, float min_brevity, float min_log_prob,
                     int max_decode_step, int min_initial_index,
                     int32_t* keep_going, int do_cond, int32_t* counters,
                     int n_counters);

}  // namespace t5d
