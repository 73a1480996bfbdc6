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
// Loads of data that no later launch of the step finds cached anyway (cached
// keys and values by the hundred megabytes): marked non-temporal so that they
// do not push what is read again (code, kernel arguments, activation rows,
// weights shared by the batch lanes) out of the caches.
typedef uint32_t u32x4_v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_once(const uint4* p) {
  u32x4_v v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_v*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
template <bool ONCE>
__device__ __forceinline__ uint4 load_kv(const uint4* p) {
  if constexpr (ONCE) return load_once(p);
  return *p;
}

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
// All-reduce butterflies on the data-parallel-primitive path (no LDS round
// trips): lane^1 and lane^2 by quad permutes, then the mirror of each 8 and
// of each 16 lanes (the partner holds the other half's partial by then), then
// v_permlane16_swap / v_permlane32_swap of the value with itself, which hand
// every lane both 16-lane (32-lane) partials.  Every lane ends with the same
// bits: both partners of a step combine the same two operands.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(
      0, (int)__float_as_uint(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7 - i within 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15 - i within 16

constexpr int kDppReverse4 = 0x1B;    // quad_perm [3,2,1,0]
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v) {
  const uint64_t b = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(
      0, (int)(uint32_t)b, CTRL, 0xF, 0xF, true);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(
      0, (int)(uint32_t)(b >> 32), CTRL, 0xF, 0xF, true);
  return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}
// The exact lane ^ 4 and lane ^ 8 partners, two moves each.
__device__ __forceinline__ float lane_xor4(float v) {
  return dpp_move<kDppReverse4>(dpp_move<kDppHalfMirror>(v));
}
__device__ __forceinline__ float lane_xor8(float v) {
  return dpp_move<kDppMirror>(dpp_move<kDppHalfMirror>(v));
}

// Over the 16 lanes of a row (lanes 16 r .. 16 r + 15).
__device__ __forceinline__ float lanes16_max(float v) {
  v = fmaxf(v, dpp_move<kDppXor1>(v));
  v = fmaxf(v, dpp_move<kDppXor2>(v));
  v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
  return fmaxf(v, dpp_move<kDppMirror>(v));
}
template <typename T>
__device__ __forceinline__ T lanes16_sum(T v) {
  v += dpp_move<kDppXor1>(v);
  v += dpp_move<kDppXor2>(v);
  v += dpp_move<kDppHalfMirror>(v);
  return v + dpp_move<kDppMirror>(v);
}
// Over the 4 lanes lane % 16 + {0, 16, 32, 48}.
__device__ __forceinline__ float rows_max(float v) {
  auto w = __builtin_amdgcn_permlane16_swap(__float_as_uint(v),
                                            __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(w[0]), __uint_as_float(w[1]));
  w = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v),
                                       false, false);
  return fmaxf(__uint_as_float(w[0]), __uint_as_float(w[1]));
}
__device__ __forceinline__ float rows_sum(float v) {
  auto w = __builtin_amdgcn_permlane16_swap(__float_as_uint(v),
                                            __float_as_uint(v), false, false);
  v = __uint_as_float(w[0]) + __uint_as_float(w[1]);
  w = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v),
                                       false, false);
  return __uint_as_float(w[0]) + __uint_as_float(w[1]);
}
__device__ __forceinline__ double rows_sum(double v) {
  const uint64_t b = __builtin_bit_cast(uint64_t, v);
  uint32_t lo = (uint32_t)b, hi = (uint32_t)(b >> 32);
  auto wl = __builtin_amdgcn_permlane16_swap(lo, lo, false, false);
  auto wh = __builtin_amdgcn_permlane16_swap(hi, hi, false, false);
  v = __builtin_bit_cast(double, ((uint64_t)wh[0] << 32) | wl[0]) +
      __builtin_bit_cast(double, ((uint64_t)wh[1] << 32) | wl[1]);
  const uint64_t c = __builtin_bit_cast(uint64_t, v);
  lo = (uint32_t)c; hi = (uint32_t)(c >> 32);
  wl = __builtin_amdgcn_permlane32_swap(lo, lo, false, false);
  wh = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
  return __builtin_bit_cast(double, ((uint64_t)wh[0] << 32) | wl[0]) +
         __builtin_bit_cast(double, ((uint64_t)wh[1] << 32) | wl[1]);
}

__device__ __forceinline__ float wave_max(float v) { return rows_max(lanes16_max(v)); }
__device__ __forceinline__ float wave_sum(float v) { return rows_sum(lanes16_sum(v)); }
__device__ __forceinline__ double wave_sum(double v) { return rows_sum(lanes16_sum(v)); }

// The matrix cores want lane (m, g) = (lane % 16, lane / 16) to hold the 8
// values k = 8g .. 8g+7 of row m.  Loaded that way, the 16 lanes of a quarter
// wavefront touch 16 different rows: 64 separate 16-byte requests per load
// instruction, and the L1's tag lookups (one per request) become the
// bottleneck of a kernel that reads a few KB.  Instead lane l loads piece
// l % 4 of row l / 4 — four neighbouring lanes read 64 contiguous bytes — and
// the 16-byte pieces are moved to the lanes that need them through the LDS
// crossbar (ds_bpermute: no LDS memory involved).
struct OperandLanes {
  int ld_row, ld_piece;  // what this lane loads: row within the tile, 8-k piece
  int src_addr;          // ds_bpermute address of the lane that loaded my piece
  __device__ __forceinline__ explicit OperandLanes(int lane)
      : ld_row(lane >> 2), ld_piece(lane & 3),
        src_addr((((lane & 15) << 2) | (lane >> 4)) << 2) {}
  __device__ __forceinline__ uint4 to_operand(const uint4& loaded) const {
    uint4 r;
    r.x = (uint32_t)__builtin_amdgcn_ds_bpermute(src_addr, (int)loaded.x);
    r.y = (uint32_t)__builtin_amdgcn_ds_bpermute(src_addr, (int)loaded.y);
    r.z = (uint32_t)__builtin_amdgcn_ds_bpermute(src_addr, (int)loaded.z);
    r.w = (uint32_t)__builtin_amdgcn_ds_bpermute(src_addr, (int)loaded.w);
    return r;
  }
};

// T5 tanh-approximate GELU in float32.
__device__ __forceinline__ float gelu_tanh(float x) {
  const float c = 0.7978845608028654f;  // sqrt(2/pi)
  return x * (0.5f * (1.0f + tanhf(c * (x + 0.044715f * (x * x * x)))));
}

// The tanh form of GELU written as x * sigmoid(2 c (x + 0.044715 x^3)): one
// exponential and one reciprocal instead of the library tanh, whose ~50
// instructions per element made the gated epilogue of the many-row dense
// kernel a third of its launch.
// Relative error ~3e-7 before the rounding to bfloat16.
__device__ __forceinline__ float gelu_sigmoid_form(float x) {
  const float k = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  const float y = k * (x + 0.044715f * (x * x * x));
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(y));
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
// True when t5d_norm_gemm (bfloat16 activations, no epilogue) runs this shape on
// its kernel for very wide layers, which keeps the rows resident and streams
// only the weights.
bool norm_gemm_is_wide(int w_dtype, int K, int N);
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
                       int eos_id, int32_t* cache_slot, int32_t* cache_src,
                       int32_t* cache_dst);
// End of a beam-search iteration in one single-workgroup kernel: advance
// *state.cur_index, add 1 to `counters[0..n_counters)` (the layers' cache
// indices), and, if do_cond, evaluate the loop condition into *keep_going.
int launch_beam_tail(hipStream_t s, const t5d_beam_state* state, int B, int K,
                     int S, float min_brevity, float min_log_prob,
                     int max_decode_step, int min_initial_index,
                     int32_t* keep_going, int do_cond, int32_t* counters,
                     int n_counters);

// The two kernels of a temperature_sample iteration after the decoder step:
// token choice, then the bookkeeping, which also advances `counters` (the
// layers' cache indices) and the step count and sets the loop flag.
int launch_sample_step(hipStream_t s, const float* logits,
                       const t5d_sample_step* st, int R, int V,
                       int32_t* counters, int n_counters);

}  // namespace t5d
