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
  const float kMasked = -9999220736.0f;  // bf16(-1e10) exactly, layers.py:309-311
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
    // validity of the tile's 16 keys: one (broadcast) LDS word, which holds
    // the prefix when the caller gave no bits.  Deliberately without a branch
    // on a.valid here: with one between the matrix instructions above and the
    // first read of their result, the compiler's wait-state count followed
    // the fall-through side only and the taken side read the accumulator 6
    // issue slots after the v_mfma (9 are needed; at 4 a stale value comes
    // back).
    const uint32_t tile_bits = (s_valid[kt >> 1] >> ((kt & 1) * 16)) & 0xffffu;
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

// ---- the same attention for E <= 512, scores kept in registers ---------------
// enc_attn_kernel walks the keys twice and forms every score twice, each
// wavefront fetching K and V for itself.  For encoder lengths up to 512 the 16
// x E scores of a wavefront fit its registers as bfloat16 pairs (they ARE
// bfloat16 values at that point), so here
//   pass 1 forms the scores once, keeps them, and tracks max / sum as before;
//   pass 2 turns the kept scores into P in registers, already in the layout
//          of the matrix cores' B operand: a lane holds keys 4g .. 4g+3 of two
//          neighbouring 16-key tiles, and the V^T operand is read from LDS in
//          that same key order, so P never goes through LDS.
// K (pass 1) and V^T (pass 2) are fetched once per workgroup, 64 keys = 8 KB
// at a time, straight from memory into a ring of three LDS stages
// (global_load_lds: lane l of an instruction lands at byte 16 l, so the
// address each lane reads from picks the XOR swizzle that makes the operand
// reads spread over the banks); the four wavefronts read their operand
// fragments from there.  One barrier per 64 keys, placed by hand with the wait
// for "all but my newest two loads"; the stages are separate arrays and the
// loops are unrolled so that every stage is named at compile time.
// Scores, maxima, sums and probabilities have the bits of enc_attn_kernel's;
// the products of a 32-key step enter the matrix instruction in another key
// order, so an output can differ from enc_attn_kernel's in its last bit (1
// in 4000 measured).
typedef __attribute__((address_space(3))) void* enc_lds_ptr_t;
typedef __attribute__((address_space(1))) const void* enc_glb_ptr_t;

template <int MAXB>  // 64-key blocks: E <= 64 MAXB
__global__ void __launch_bounds__(256)
enc_attn_ring_kernel(EncAttnArgs a) {
  __shared__ uint4 s_r0[512];
  __shared__ uint4 s_r1[512];
  __shared__ uint4 s_r2[512];
  __shared__ float s_bias[128 * MAXB + 16];
  __shared__ uint32_t s_valid[2 * MAXB];
  // what a score is capped by, per key: [0] for a valid query (+inf for a
  // valid key, bf16(-1e10) for a masked one, -inf past E), [1] for a padded
  // query (bf16(-1e10) for every key that exists)
  __shared__ __attribute__((aligned(16))) float s_lim[2][64 * MAXB + 16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, gq = lane >> 4;
  const int h = blockIdx.y, b = blockIdx.z;
  const int E = a.E;
  for (int i = threadIdx.x; i < 2 * E - 1; i += 256)
    s_bias[i] = bf16_to_f32(a.bias[(size_t)h * (2 * E - 1) + i]);
  int n = a.len[b];
  n = n < 0 ? 0 : (n > E ? E : n);
  const int words = (E + 31) >> 5;
  for (int i = threadIdx.x; i < words; i += 256) {
    const int left = n - 32 * i;
    const uint32_t prefix =
        left >= 32 ? 0xffffffffu : (left <= 0 ? 0u : ((1u << left) - 1u));
    s_valid[i] = a.valid ? (a.valid[(size_t)b * words + i] & prefix) : prefix;
  }
  __syncthreads();
  const float kMasked = -9999220736.0f;  // bf16(-1e10) exactly, layers.py:309-311
  for (int i = threadIdx.x; i < 64 * MAXB + 16; i += 256) {
    const bool ok = i < E && ((s_valid[i >> 5] >> (i & 31)) & 1u) != 0;
    s_lim[0][i] = ok ? INFINITY : (i < E ? kMasked : -INFINITY);
    s_lim[1][i] = i < E ? kMasked : -INFINITY;
  }
  __syncthreads();
  // Key tiles each wavefront walks (as in enc_attn_kernel: the valid prefix
  // when all of its 16 queries are valid — the keys beyond add exact zeros —
  // else every key; none when its queries lie beyond E) and what the
  // workgroup as a whole must fetch, in 64-key blocks.
  const int all_tiles = (E + 15) >> 4;
  int my_tiles = 0, wg_tiles = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int qw = blockIdx.x * 64 + w * 16;
    int t = 0;
    if (qw < E) {
      const bool all_valid =
          qw + 15 < E &&
          ((s_valid[qw >> 5] >> (qw & 31)) & 0xffffu) == 0xffffu;
      t = all_valid ? (n + 15) >> 4 : all_tiles;
    }
    if (w == wave) my_tiles = t;
    wg_tiles = max(wg_tiles, t);
  }
  my_tiles = __builtin_amdgcn_readfirstlane(my_tiles);
  const int nb = __builtin_amdgcn_readfirstlane((wg_tiles + 3) >> 2);
  const int q0 = blockIdx.x * 64 + wave * 16;
  const size_t row0 = (size_t)b * E;

  const int qi = min(q0 + l16, E - 1);
  FragE qb[2];
#pragma unroll
  for (int c = 0; c < 2; ++c)
    qb[c].u = *reinterpret_cast<const uint4*>(
        a.q + (row0 + qi) * a.q_stride + h * 64 + 32 * c + 8 * gq);
  const bool q_valid =
      q0 + l16 < E &&
      ((s_valid[(q0 + l16) >> 5] >> ((q0 + l16) & 31)) & 1u) != 0;
  // this lane's 4 keys of key tile kt: bias and cap at [16 kt .. 16 kt + 3].
  // Masking is a minimum with the cap: a score never lies below -1e10, so
  // min(x, bf16(-1e10)) is the reference's masked value, min(x, -inf) removes
  // a key that does not exist, min(x, +inf) keeps x.
  const float* bias_g = s_bias + (E - 1) - qi + 4 * gq;
  const float* lim_g = s_lim[q_valid ? 0 : 1] + 4 * gq;

  // What this lane fetches of a 64-key block of K: chunks (8 keys, 1 KB)
  // wave and wave + 4; lane s lands at slot s & 7 of key s >> 3 and therefore
  // reads piece (s & 7) ^ (s >> 3) of that key.
  const int k_r = lane >> 3, k_piece = (lane & 7) ^ k_r;
  const char* kbase = reinterpret_cast<const char*>(a.k) +
                      (size_t)h * 128 + k_piece * 16;
  // ... and of a 64-key block of V^T (two [64 d][32 keys] blocks, 4 KB each):
  // chunks (16 rows d, 1 KB) wave and wave + 4; lane s lands at slot s & 3 of
  // row s >> 2 and reads piece (s & 3) ^ ((row >> 1) & 1): one swizzle bit, so
  // that the two pieces a lane needs in pass 2 (p and p + 2) stay 32 bytes
  // apart and come with one two-address read, already in operand order.
  const int v_r = lane >> 2, v_piece = (lane & 3) ^ ((v_r >> 1) & 1);
  const char* vbase = reinterpret_cast<const char*>(a.vt) +
                      ((size_t)b * a.H + h) * 128 * (size_t)a.Ep;
  const int v_blocks = a.Ep >> 5;
#define T5D_ENC_ISSUE_K(i_, S_)                                                \
  do {                                                                         \
    _Pragma("unroll") for (int u = 0; u < 2; ++u) {                            \
      const int c = wave + 4 * u;                                              \
      const int key = min(64 * (i_) + 8 * c + k_r, E - 1);                     \
      __builtin_amdgcn_global_load_lds(                                        \
          (enc_glb_ptr_t)(kbase + (row0 + key) * (size_t)a.k_stride * 2),      \
          (enc_lds_ptr_t)&S_[64 * c], 16, 0, 0);                               \
    }                                                                          \
  } while (0)
#define T5D_ENC_ISSUE_V(i_, S_)                                                \
  do {                                                                         \
    _Pragma("unroll") for (int u = 0; u < 2; ++u) {                            \
      const int c = wave + 4 * u;                                              \
      const int blk = min(2 * (i_) + (c >> 2), v_blocks - 1);                  \
      __builtin_amdgcn_global_load_lds(                                        \
          (enc_glb_ptr_t)(vbase + (size_t)blk * 4096 +                         \
                          (16 * (c & 3) + v_r) * 64 + v_piece * 16),           \
          (enc_lds_ptr_t)&S_[64 * c], 16, 0, 0);                               \
    }                                                                          \
  } while (0)
  // all but my newest two loads (the next block) have landed and my reads of
  // LDS have returned (vmcnt(2) lgkmcnt(0): a barrier orders issued
  // instructions, not completed LDS reads); after the barrier so have
  // everyone's, and everyone is done with the stage that the loads issued
  // next overwrite.  Nothing in a step is conditional — the loads past the
  // last block fetch clamped addresses into a stage nobody reads, every
  // wavefront forms all four key tiles of a block — and the only branch is
  // the loop exit in front of a step: where two paths meet between a load
  // into LDS and a read of LDS the compiler waits for every load in flight.
#define T5D_ENC_STEP(i_, CUR_, NEXT2_, ISSUE_, BODY_)                          \
  if ((i_) >= nb) break;                                                       \
  __builtin_amdgcn_s_waitcnt(0x070 | 2);                                       \
  __builtin_amdgcn_s_barrier();                                                \
  ISSUE_((i_) + 2, NEXT2_);                                                    \
  __builtin_amdgcn_sched_barrier(0);                                           \
  BODY_(i_, CUR_);

  // scores of key tile kt for this lane: keys 16 kt + 4 g + i of query l16
  constexpr int ROUNDS = (MAXB + 2) / 3;
  uint32_t sc[12 * ROUNDS][2];
#pragma unroll
  for (int t = 0; t < 12 * ROUNDS; ++t)
    sc[t][0] = sc[t][1] = 0xFF80FF80u;  // -inf
  float m = -3.0e38f, l = 0.f;
  const int swz = l16 & 7;
#define T5D_ENC_SCORES(i_, S_)                                                 \
  _Pragma("unroll") for (int t = 0; t < 4; ++t) {                              \
    const int kt = 4 * (i_) + t;                                               \
    /* two key tiles per test: their chains of dependent instructions (LDS   \
       read, matrix instruction, rounding, exp) interleave */                 \
    if ((kt & ~1) < my_tiles) {                                                \
      f32x4_e acc = (f32x4_e){0.f, 0.f, 0.f, 0.f};                             \
      _Pragma("unroll") for (int c = 0; c < 2; ++c) {                          \
        FragE kop;                                                             \
        kop.u = S_[(16 * t + l16) * 8 + ((4 * c + gq) ^ swz)];                 \
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop.v, qb[c].v, acc, 0,  \
                                                      0, 0);                   \
      }                                                                        \
      const float4 cap = *reinterpret_cast<const float4*>(lim_g + 16 * kt);    \
      /* two values per rounding instruction; the cap as a median with -inf   \
         (one instruction: fminf would first make both operands canonical) */ \
      const uint32_t r01 = pack_bf16x2(acc[0], acc[1]);                        \
      const uint32_t r23 = pack_bf16x2(acc[2], acc[3]);                        \
      const uint32_t x01 =                                                     \
          pack_bf16x2(bf16lo_to_f32(r01) + bias_g[16 * kt],                    \
                      bf16hi_to_f32(r01) + bias_g[16 * kt + 1]);               \
      const uint32_t x23 =                                                     \
          pack_bf16x2(bf16lo_to_f32(r23) + bias_g[16 * kt + 2],                \
                      bf16hi_to_f32(r23) + bias_g[16 * kt + 3]);               \
      float s[4];                                                              \
      s[0] = __builtin_amdgcn_fmed3f(bf16lo_to_f32(x01), cap.x, -INFINITY);    \
      s[1] = __builtin_amdgcn_fmed3f(bf16hi_to_f32(x01), cap.y, -INFINITY);    \
      s[2] = __builtin_amdgcn_fmed3f(bf16lo_to_f32(x23), cap.z, -INFINITY);    \
      s[3] = __builtin_amdgcn_fmed3f(bf16hi_to_f32(x23), cap.w, -INFINITY);    \
      const float tm = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));            \
      const float nm = fmaxf(m, tm);                                           \
      float add = 0.f;                                                         \
      _Pragma("unroll") for (int i = 0; i < 4; ++i) add += __expf(s[i] - nm);  \
      l = l * __expf(m - nm) + add;                                            \
      m = nm;                                                                  \
      sc[kt][0] = pack_bf16x2(s[0], s[1]);                                     \
      sc[kt][1] = pack_bf16x2(s[2], s[3]);                                     \
    }                                                                          \
  }

  T5D_ENC_ISSUE_K(0, s_r0);
  T5D_ENC_ISSUE_K(1, s_r1);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    T5D_ENC_STEP(3 * r, s_r0, s_r2, T5D_ENC_ISSUE_K, T5D_ENC_SCORES)
    T5D_ENC_STEP(3 * r + 1, s_r1, s_r0, T5D_ENC_ISSUE_K, T5D_ENC_SCORES)
    T5D_ENC_STEP(3 * r + 2, s_r2, s_r1, T5D_ENC_ISSUE_K, T5D_ENC_SCORES)
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
  // V^T operand of a 32-key step: row d = 16 dt + l16, the 8 bytes of keys
  // 4g .. 4g+3 and of keys 16+4g .. 16+4g+3 (pieces g / 2 and 2 + g / 2)
  const int v_swz = (l16 >> 1) & 1;
  const int v_off0 = l16 * 64 + (((gq >> 1) ^ v_swz) * 16) + (gq & 1) * 8;
  auto prob2 = [&](uint32_t packed) {
    return pack_bf16x2(__expf(bf16lo_to_f32(packed) - m) * inv,
                       __expf(bf16hi_to_f32(packed) - m) * inv);
  };
#define T5D_ENC_VALUES(i_, S_)                                                 \
  _Pragma("unroll") for (int hb = 0; hb < 2; ++hb) {                           \
    const int kt = 4 * (i_) + 2 * hb;                                          \
    {                                                                          \
      FragE pb;                                                                \
      pb.u.x = prob2(sc[kt][0]);                                               \
      pb.u.y = prob2(sc[kt][1]);                                               \
      pb.u.z = prob2(sc[kt + 1][0]);                                           \
      pb.u.w = prob2(sc[kt + 1][1]);                                           \
      const char* blk = reinterpret_cast<const char*>(&S_[0]) + hb * 4096;     \
      _Pragma("unroll") for (int dt = 0; dt < 4; ++dt) {                       \
        const uint2* vp =                                                      \
            reinterpret_cast<const uint2*>(blk + dt * 1024 + v_off0);          \
        const uint2 lo = vp[0], hi = vp[4];                                    \
        FragE va;                                                              \
        va.u = make_uint4(lo.x, lo.y, hi.x, hi.y);                             \
        oc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va.v, pb.v, oc[dt],   \
                                                         0, 0, 0);             \
      }                                                                        \
    }                                                                          \
  }
  __builtin_amdgcn_s_waitcnt(0x070);
  __builtin_amdgcn_s_barrier();  // every wavefront is done with the K stages
  T5D_ENC_ISSUE_V(0, s_r0);
  T5D_ENC_ISSUE_V(1, s_r1);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    T5D_ENC_STEP(3 * r, s_r0, s_r2, T5D_ENC_ISSUE_V, T5D_ENC_VALUES)
    T5D_ENC_STEP(3 * r + 1, s_r1, s_r0, T5D_ENC_ISSUE_V, T5D_ENC_VALUES)
    T5D_ENC_STEP(3 * r + 2, s_r2, s_r1, T5D_ENC_ISSUE_V, T5D_ENC_VALUES)
  }
  // the loads issued past the last block must land before this workgroup's
  // LDS can go to another
  __builtin_amdgcn_s_waitcnt(0x070);
#undef T5D_ENC_ISSUE_K
#undef T5D_ENC_ISSUE_V
#undef T5D_ENC_STEP
#undef T5D_ENC_SCORES
#undef T5D_ENC_VALUES
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
  return t5d_encoder_attention_variant(stream, q, k, v_t, rel_bias, enc_len,
                                       valid_bits, out, B, H, E, Ep, q_stride,
                                       k_stride, 0);
}

extern "C" int t5d_encoder_attention_variant(
    void* stream, const void* q, const void* k, const void* v_t,
    const void* rel_bias, const int32_t* enc_len, const uint32_t* valid_bits,
    void* out, int B, int H, int E, int Ep, int q_stride, int k_stride,
    int variant) {
  T5D_REQUIRE(variant >= 0 && variant <= 2 && (variant != 2 || E <= 512),
              T5D_EINVAL,
              "t5d_encoder_attention_variant: variant %d (0 chosen here, 1 "
              "scores formed twice, 2 scores kept in registers: E <= 512)",
              variant);
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
  if (variant == 1)
    hipLaunchKernelGGL(enc_attn_kernel, grid, block, 0, as_stream(stream), a);
  else if (E <= 128)
    hipLaunchKernelGGL(enc_attn_ring_kernel<2>, grid, block, 0,
                       as_stream(stream), a);
  else if (E <= 256)
    hipLaunchKernelGGL(enc_attn_ring_kernel<4>, grid, block, 0,
                       as_stream(stream), a);
  else if (E <= 512)
    hipLaunchKernelGGL(enc_attn_ring_kernel<8>, grid, block, 0,
                       as_stream(stream), a);
  else
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
