// Encoder self-attention over whole sequences (bfloat16), once per batch:
// out = softmax(Q K^T + relative-position bias + padding mask) V per
// (batch item, head), t5x/examples/t5/layers.py:52-129 with the encoder's
// bidirectional bias (layers.py:560-677) and mask (network.py:325-328).
//
// A workgroup takes 64 queries of one (item, head), a wavefront 16 of them.
// Two passes over the keys, 16 at a time, both on the matrix cores:
//   pass 1: S^T = K Q^T (keys as MFMA rows, so a lane ends up with 4
//           consecutive keys of ONE query), scores rounded where the reference
//           rounds them, running max / sum per lane, combined at the end;
//   pass 2: S^T again, P = bf16(exp(s - max) / sum) written 4 keys at a time
//           into a small LDS tile, read back as the B operand of
//           out^T = V^T P^T, 32 keys per step.  V is given transposed in
//           32-key blocks ([B, H, Ep / 32, 64, 32], what t5d_gemm_rows' value
//           layout writes), so a fragment is one contiguous 1 KB.
// Masked keys get the reference's -1e10 (so a padded query attends uniformly,
// as it does there); keys beyond E do not exist and get -inf.
#include <math.h>

#include "common.h"

namespace t5d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_e;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_e;

union FragE {
  uint4 u;
  bf16x8_e v;
};

struct EncAttnArgs {
  const bf16_t* q;    // [B*E, q_stride]: head h at columns h*64 .. +64
  const bf16_t* k;    // same layout as q
  const bf16_t* vt;   // [B, H, Ep / 32, 64, 32]: 32-key blocks
  const bf16_t* bias; // [H, 2E-1]: by (key - query + E - 1)
  const int32_t* len; // [B] valid prefix length (with `valid`: last valid + 1)
  const uint32_t* valid;  // optional [B, (E + 31) / 32]: bit e = position e valid
  bf16_t* out;        // [B*E, H*64]
  int H, E, Ep, q_stride, k_stride;
};

constexpr int kMaxEncLen = 2048;

__global__ void __launch_bounds__(256)
enc_attn_kernel(EncAttnArgs a) {
  __shared__ __attribute__((aligned(16))) bf16_t s_p[4][16][32];
  __shared__ float s_bias[2 * kMaxEncLen];  // this head's bias by distance
  __shared__ uint32_t s_valid[kMaxEncLen / 32];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, gq = lane >> 4;
  const int h = blockIdx.y, b = blockIdx.z;
  const int q0 = blockIdx.x * 64 + wave * 16;
  const int E = a.E;
  for (int i = threadIdx.x; i < 2 * E - 1; i += 256)
    s_bias[i] = bf16_to_f32(a.bias[(size_t)h * (2 * E - 1) + i]);
  int n = a.len[b];
  n = n < 0 ? 0 : (n > E ? E : n);
  // Which positions are valid: the prefix [0, n), or the caller's bits (a
  // padding token inside the text: encoder_input_tokens > 0 element-wise).
  const int words = (E + 31) >> 5;
  for (int i = threadIdx.x; i < words; i += 256) {
    const int left = n - 32 * i;
    const uint32_t prefix =
        left >= 32 ? 0xffffffffu : (left <= 0 ? 0u : ((1u << left) - 1u));
    s_valid[i] = a.valid ? (a.valid[(size_t)b * words + i] & prefix) : prefix;
  }
  __syncthreads();
  if (q0 >= E) return;
  auto is_valid = [&](int pos) {
    return pos < E && ((s_valid[pos >> 5] >> (pos & 31)) & 1u) != 0;
  };
  const float kMasked = -9.9857e9f;  // bf16(-1e10), layers.py:309-311
  const size_t row0 = (size_t)b * E;

  // B operand of S^T: lane (col = query l16, g) holds Q[q][32c + 8g .. +8]
  const int qi = min(q0 + l16, E - 1);
  FragE qb[2];
#pragma unroll
  for (int c = 0; c < 2; ++c)
    qb[c].u = *reinterpret_cast<const uint4*>(
        a.q + (row0 + qi) * a.q_stride + h * 64 + 32 * c + 8 * gq);
  const bool q_valid = is_valid(q0 + l16);
  const float* bias_row = s_bias + (E - 1) - qi;

  // Keys past the valid length get -1e10, whose exp underflows to exactly 0
  // next to any valid key: when all 16 queries of this wavefront are valid,
  // the key tiles that hold only padding are skipped.  (A padded query attends
  // uniformly over ALL keys, so a wavefront with one walks them all.)
  const bool all_valid =
      q0 + 15 < E &&
      ((s_valid[q0 >> 5] >> (q0 & 31)) & 0xffffu) == 0xffffu;  // q0 % 16 == 0
  const int n_tiles = all_valid ? (n + 15) >> 4 : (E + 15) >> 4;

  // K tile kt as the A operand: lane (row = key l16, g) holds K[key][32c + 8g .. +8].
  // It is fetched with four neighbouring lanes on 64 contiguous bytes of one key
  // (16 requests per instruction instead of 64: this kernel walks every key
  // tile twice, and fetched in operand order the L1's tag lookups bound it) and
  // moved to operand order by `operand_k` when it is consumed.
  const OperandLanes ol(lane);
  auto load_k = [&](int kt, FragE (&ka)[2]) {
    const int key_row = min(16 * kt + ol.ld_row, E - 1);
#pragma unroll
    for (int c = 0; c < 2; ++c)
      ka[c].u = *reinterpret_cast<const uint4*>(
          a.k + (row0 + key_row) * a.k_stride + h * 64 + 32 * c + 8 * ol.ld_piece);
  };
  // scores of key tile kt for this lane: keys 16 kt + 4 g + i of query l16
  auto score_tile = [&](int kt, const FragE (&ka)[2], float (&s)[4]) {
    f32x4_e acc = (f32x4_e){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      FragE kop;
      kop.u = ol.to_operand(ka[c].u);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop.v, qb[c].v, acc, 0, 0, 0);
    }
    // validity of the tile's 16 keys: from the prefix length alone, or one
    // (broadcast) LDS word when the caller gave bits
    const int left = n - 16 * kt;
    const uint32_t tile_bits =
        a.valid ? (s_valid[kt >> 1] >> ((kt & 1) * 16)) & 0xffffu
                : (left >= 16 ? 0xffffu : (left <= 0 ? 0u : (1u << left) - 1u));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = 16 * kt + 4 * gq + i;
      float x = round_bf16(acc[i]);
      if (key < E) {
        const bool ok = q_valid && ((tile_bits >> (4 * gq + i)) & 1u) != 0;
        x = ok ? round_bf16(x + bias_row[key]) : kMasked;
      } else {
        x = -INFINITY;
      }
      s[i] = x;
    }
  };

  // The running maximum starts at a finite floor: a lane whose 4 keys of the
  // first tile all lie beyond E (E < 16) has only -inf scores, and
  // exp(-inf - (-inf)) would poison its sum.
  float m = -3.0e38f, l = 0.f;
  {
    FragE kcur[2], knext[2];
    load_k(0, kcur);
    for (int kt = 0; kt < n_tiles; ++kt) {
      if (kt + 1 < n_tiles) load_k(kt + 1, knext);  // in flight during this tile
      float s[4];
      score_tile(kt, kcur, s);
      const float tm = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
      const float nm = fmaxf(m, tm);
      float add = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) add += __expf(s[i] - nm);
      l = l * __expf(m - nm) + add;  // exp(-inf - finite) == 0 on the first tile
      m = nm;
      kcur[0] = knext[0];
      kcur[1] = knext[1];
    }
  }
  // combine the 4 lanes (g) that share a query
#pragma unroll
  for (int o = 16; o <= 32; o <<= 1) {
    const float om = __shfl_xor(m, o, 64), ol = __shfl_xor(l, o, 64);
    const float nm = fmaxf(m, om);
    l = l * __expf(m - nm) + ol * __expf(om - nm);
    m = nm;
  }
  const float inv = 1.0f / l;

  f32x4_e oc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) oc[dt] = (f32x4_e){0.f, 0.f, 0.f, 0.f};
  const bf16_t* vbase = a.vt + ((size_t)b * a.H + h) * 64 * (size_t)a.Ep;
  // V^T fragments of a 32-key step: lane (row = d l16, g) holds
  // V^T[16 dt + l16][32 (kb / 2) + 8 g .. +8], 1 KB contiguous per fragment
  auto load_v = [&](int kb, FragE (&va)[4]) {  // kb even: block kb / 2
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
      va[dt].u = *reinterpret_cast<const uint4*>(
          vbase + ((size_t)(kb >> 1) * 64 + 16 * dt + l16) * 32 + 8 * gq);
  };
  FragE kcur[2][2], knext[2][2], vcur[4], vnext[4];
  load_k(0, kcur[0]);
  if (1 < n_tiles) load_k(1, kcur[1]);
  load_v(0, vcur);
  for (int kb = 0; kb < n_tiles; kb += 2) {  // 32 keys per step
    if (kb + 2 < n_tiles) {
      load_k(kb + 2, knext[0]);
      if (kb + 3 < n_tiles) load_k(kb + 3, knext[1]);
      load_v(kb + 2, vnext);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      float s[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      if (kb + t < n_tiles) score_tile(kb + t, kcur[t], s);
      uint2 pk;
      pk.x = pack_bf16x2(__expf(s[0] - m) * inv, __expf(s[1] - m) * inv);
      pk.y = pack_bf16x2(__expf(s[2] - m) * inv, __expf(s[3] - m) * inv);
      *reinterpret_cast<uint2*>(&s_p[wave][l16][16 * t + 4 * gq]) = pk;
    }
    // LDS traffic stays inside the wavefront: its own writes are visible to it
    // once they have completed.
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    FragE pb;  // B: lane (col = query l16, g) holds P[q][8g .. +8] of the 32
    pb.u = *reinterpret_cast<const uint4*>(&s_p[wave][l16][8 * gq]);
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
      oc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vcur[dt].v, pb.v, oc[dt],
                                                       0, 0, 0);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      kcur[t][0] = knext[t][0];
      kcur[t][1] = knext[t][1];
    }
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) vcur[dt] = vnext[dt];
  }
  // oc[dt][i]: out[q = l16][d = 16 dt + 4 g + i]
  if (q0 + l16 < E) {
    bf16_t* o = a.out + (row0 + q0 + l16) * (size_t)(a.H * 64) + h * 64 + 4 * gq;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      uint2 pk;
      pk.x = pack_bf16x2(oc[dt][0], oc[dt][1]);
      pk.y = pack_bf16x2(oc[dt][2], oc[dt][3]);
      *reinterpret_cast<uint2*>(o + 16 * dt) = pk;
    }
  }
}

// ---- float32 -------------------------------------------------------------------
// The exactness-test dtype: plain vector arithmetic, one wavefront per query
// row.  Scores (lane = key, ascending head dim), bias and mask summed first and
// added to the score as the reference does (a masked pair ends at exactly
// -1e10, so a padded query attends uniformly), softmax over all E keys, then
// lane = head dim accumulates the normalised weights times V in ascending key
// order.  qkv rows hold q | k | v (H*64 columns each).
struct EncAttnF32Args {
  const float* qkv;   // [B*E, 3*H*64]
  const float* bias;  // [H, 2E-1], by (key - query + E - 1)
  const int32_t* len; // [B]
  const uint32_t* valid;  // optional [B, (E + 31) / 32], as EncAttnArgs
  float* out;         // [B*E, H*64]
  int H, E;
};

constexpr int kEncF32Rows = 4;  // query rows (wavefronts) per workgroup
constexpr int kHeadDim = 64;

__global__ void __launch_bounds__(64 * kEncF32Rows)
enc_attn_f32_kernel(EncAttnF32Args a) {
  __shared__ float s_w[kEncF32Rows][kMaxEncLen];
  __shared__ __attribute__((aligned(16))) float s_q[kEncF32Rows][kHeadDim];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int e = blockIdx.x * kEncF32Rows + wave;
  const int h = blockIdx.y, b = blockIdx.z;
  if (e >= a.E) return;  // whole wavefronts; no workgroup barrier below
  const int HD = a.H * kHeadDim, row_stride = 3 * HD;
  const int n = min(max(a.len[b], 0), a.E);
  const float* base = a.qkv + (size_t)b * a.E * row_stride + h * kHeadDim;
  s_q[wave][lane] = base[(size_t)e * row_stride + lane];
  const float* bias = a.bias + (size_t)h * (2 * a.E - 1) + (a.E - 1) - e;
  const int words = (a.E + 31) >> 5;
  auto is_valid = [&](int pos) {
    return pos < n &&
           (a.valid == nullptr ||
            ((a.valid[(size_t)b * words + (pos >> 5)] >> (pos & 31)) & 1u) != 0);
  };
  const bool q_valid = is_valid(e);

  float m = -INFINITY;
  for (int j = lane; j < a.E; j += 64) {
    const float4* kr =
        reinterpret_cast<const float4*>(base + (size_t)j * row_stride + HD);
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < kHeadDim / 4; ++c) {
      const float4 kv = kr[c];
      const float4 qv = *reinterpret_cast<const float4*>(&s_q[wave][4 * c]);
      s = fmaf(qv.x, kv.x, s);
      s = fmaf(qv.y, kv.y, s);
      s = fmaf(qv.z, kv.z, s);
      s = fmaf(qv.w, kv.w, s);
    }
    const float mask = (q_valid && is_valid(j)) ? 0.f : -1e10f;
    const float x = s + (mask + bias[j]);
    s_w[wave][j] = x;
    m = fmaxf(m, x);
  }
  m = wave_max(m);
  float sum = 0.f;
  for (int j = lane; j < a.E; j += 64) {
    const float p = expf(s_w[wave][j] - m);
    s_w[wave][j] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  // s_w[wave] is written and read by this wavefront only
  float acc = 0.f;
  const float* vr = base + 2 * HD + lane;
  for (int j = 0; j < a.E; ++j)
    acc = fmaf(s_w[wave][j] / sum, vr[(size_t)j * row_stride], acc);
  a.out[((size_t)b * a.E + e) * HD + h * kHeadDim + lane] = acc;
}

}  // namespace t5d

using namespace t5d;

extern "C" int t5d_encoder_attention(void* stream, const void* q, const void* k,
                                     const void* v_t, const void* rel_bias,
                                     const int32_t* enc_len,
                                     const uint32_t* valid_bits, void* out,
                                     int B, int H, int E, int Ep, int q_stride,
                                     int k_stride) {
  T5D_REQUIRE(q && k && v_t && rel_bias && enc_len && out, T5D_EINVAL,
              "t5d_encoder_attention: null pointer");
  T5D_REQUIRE(B > 0 && H > 0 && E > 0 && Ep >= E && Ep % 32 == 0,
              T5D_EINVAL, "t5d_encoder_attention: B=%d H=%d E=%d Ep=%d", B, H,
              E, Ep);
  T5D_REQUIRE(q_stride >= H * 64 && k_stride >= H * 64 && q_stride % 8 == 0 &&
                  k_stride % 8 == 0,
              T5D_EINVAL, "t5d_encoder_attention: row strides %d / %d", q_stride,
              k_stride);
  T5D_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 &&
                  ((uintptr_t)v_t % 16) == 0 && ((uintptr_t)out % 8) == 0,
              T5D_EINVAL, "t5d_encoder_attention: operand alignment");
  T5D_REQUIRE(E <= kMaxEncLen, T5D_ELIMIT,
              "t5d_encoder_attention: E=%d beyond %d", E, kMaxEncLen);
  T5D_REQUIRE(H <= 65535 && B <= 65535, T5D_ELIMIT,
              "t5d_encoder_attention: H=%d B=%d beyond the launch grid", H, B);
  EncAttnArgs a;
  a.q = (const bf16_t*)q; a.k = (const bf16_t*)k; a.vt = (const bf16_t*)v_t;
  a.bias = (const bf16_t*)rel_bias; a.len = enc_len; a.out = (bf16_t*)out;
  a.valid = valid_bits;
  a.H = H; a.E = E; a.Ep = Ep; a.q_stride = q_stride; a.k_stride = k_stride;
  dim3 grid((E + 63) / 64, H, B), block(256);
  hipLaunchKernelGGL(enc_attn_kernel, grid, block, 0, as_stream(stream), a);
  T5D_CHECK_LAUNCH("t5d_encoder_attention");
  return T5D_OK;
}

extern "C" int t5d_encoder_attention_f32(void* stream, const float* qkv,
                                         const float* rel_bias,
                                         const int32_t* enc_len,
                                         const uint32_t* valid_bits,
                                         float* out, int B, int H, int E) {
  T5D_REQUIRE(qkv && rel_bias && enc_len && out, T5D_EINVAL,
              "t5d_encoder_attention_f32: null pointer");
  T5D_REQUIRE(B > 0 && H > 0 && E > 0, T5D_EINVAL,
              "t5d_encoder_attention_f32: B=%d H=%d E=%d", B, H, E);
  T5D_REQUIRE(E <= kMaxEncLen, T5D_ELIMIT,
              "t5d_encoder_attention_f32: E=%d beyond %d", E, kMaxEncLen);
  T5D_REQUIRE(H <= 65535 && B <= 65535, T5D_ELIMIT,
              "t5d_encoder_attention_f32: H=%d B=%d beyond the launch grid", H,
              B);
  T5D_REQUIRE(((uintptr_t)qkv % 16) == 0, T5D_EINVAL,
              "t5d_encoder_attention_f32: qkv must be 16-byte aligned");
  EncAttnF32Args a;
  a.qkv = qkv; a.bias = rel_bias; a.len = enc_len; a.out = out;
  a.valid = valid_bits;
  a.H = H; a.E = E;
  dim3 grid((E + kEncF32Rows - 1) / kEncF32Rows, H, B);
  hipLaunchKernelGGL(enc_attn_f32_kernel, grid, dim3(64 * kEncF32Rows), 0,
                     as_stream(stream), a);
  T5D_CHECK_LAUNCH("t5d_encoder_attention_f32");
  return T5D_OK;
}
