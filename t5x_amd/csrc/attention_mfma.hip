// bfloat16 decode-step attention on the matrix cores.
//
// A decode step streams K and V once; with VALU dot products the 64-wide
// wavefront spends more cycles converting and multiplying than the memory
// system needs to deliver the data.  Here every 16-byte chunk a lane loads is
// directly an MFMA operand (v_mfma_f32_16x16x32_bf16), so the vector ALU only
// runs the softmax.
//
//   cross-attention:  K is kept [B, H, E, 64] (head dim contiguous) and V
//     [B, H, 64, E] (positions contiguous) — both projected once per batch
//     item, layouts free to choose.  scores = Q·K^T uses K chunks as the B
//     operand (k = head dim), out = P·V uses V chunks as the B operand
//     (k = position).  The <= 8 queries of a batch item's beams are rows of
//     the A operand, so the K/V stream is shared by the beams.
//   self-attention:   the cache layout [R, H, 64, L] is fixed by the drop-in
//     contract (positions contiguous) for both K and V.  P·V maps onto MFMA as
//     above; Q·K^T would need the head dim contiguous, so with its single
//     query row it stays on the vector ALU (one FMA per loaded element).
//
// One workgroup per (row or batch item, head); wavefront w owns positions
// [128 w, 128 w + 128).  Probabilities are normalised with the workgroup-wide
// max / sum (exchanged through LDS), rounded to bf16, and only then multiplied
// with V, which is where the reference rounds them.
#include <math.h>

#include "common.h"

namespace t5d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_v;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_v;

union Frag16 {
  uint4 u;
  bf16x8_v v;
  bf16_t h[8];
};

struct AttnMfmaArgs {
  const bf16_t* q;      // self: qkv [R, 3*HD]; cross: q [R, HD]
  bf16_t* k;            // self: [R, H, 64, L]; cross: [B, H, E, 64]
  bf16_t* v;            // [.., H, 64, S]
  const bf16_t* rel_bias;  // self: [H, L]
  const int32_t* index;    // self: cache_index; cross: enc_len [B]
  bf16_t* out;             // [R, HD]
  int H, S, nq, q_stride;
  const int32_t* gate;
  // self-attention only
  const int32_t* pending;  // [B, beams] source beam per row, or null
  int beams, nblk;         // rows per workgroup, wavefronts per row
};

constexpr int kHeadDim = 64;
constexpr int kBlockJ = 128;  // positions per wavefront

// Phase timestamps for kernel tuning; compiled out unless T5D_PROBE is set.
#ifdef T5D_PROBE
__device__ long long t5d_probe_buf[64 * 16];
#define T5D_STAMP(i)                                                       \
  if (lane == 0 && wave == 0 && (blockIdx.x + blockIdx.y * gridDim.x) % 37 == 0 && \
      (blockIdx.x + blockIdx.y * gridDim.x) / 37 < 64)                      \
    t5d_probe_buf[((blockIdx.x + blockIdx.y * gridDim.x) / 37) * 16 + (i)] = \
        __builtin_readcyclecounter()
#else
#define T5D_STAMP(i)
#endif

// ---- cross-attention -----------------------------------------------------------
// NQP: query rows padded to a multiple of 4 (4, 8).  WM: max wavefronts.
template <int NQP, int WM>
__global__ void __launch_bounds__(64 * WM)
cross_attn_mfma_kernel(AttnMfmaArgs a) {
  __shared__ float s_red[WM][NQP];
  // s_p (probabilities, bf16) and s_out (partial outputs, f32) are used one
  // after the other and share storage.
  __shared__ __attribute__((aligned(16))) float s_raw[WM * NQP * kHeadDim];
  bf16_t (*s_p)[NQP][kBlockJ] =
      reinterpret_cast<bf16_t (*)[NQP][kBlockJ]>(s_raw);
  float (*s_out)[NQP][kHeadDim] =
      reinterpret_cast<float (*)[NQP][kHeadDim]>(s_raw);
  static_assert(sizeof(bf16_t) * kBlockJ <= sizeof(float) * kHeadDim, "alias");
  T5D_GATED(a.gate);

  const int h = blockIdx.x, b = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nwaves = blockDim.x >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int HD = a.H * kHeadDim;

  T5D_STAMP(0);
  int n = a.index[b];
  n = n < 0 ? 0 : (n > a.S ? a.S : n);
  bool uniform = false;  // no valid key: the masked softmax is uniform
  if (n == 0) { uniform = true; n = a.S; }
  T5D_STAMP(1);

  const int jw = wave * kBlockJ;          // first position of this wavefront
  const bool wave_live = jw < n;
  const bf16_t* kbase = a.k + ((size_t)b * a.H + h) * (size_t)a.S * kHeadDim;
  const bf16_t* vbase = a.v + ((size_t)b * a.H + h) * (size_t)kHeadDim * a.S;

  // A operand of Q·K^T: lane (m = n16, g) holds Q[m][32c + 8g .. +8].
  Frag16 qa[2];
  {
    const bool qrow = n16 < a.nq;
    const bf16_t* qp = a.q + (size_t)(b * a.nq + (qrow ? n16 : 0)) * a.q_stride +
                       h * kHeadDim + 8 * g;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (qrow) qa[c].u = *reinterpret_cast<const uint4*>(qp + 32 * c);
      else qa[c].u = make_uint4(0, 0, 0, 0);
    }
  }

  // Every K and V chunk this lane needs is requested up front, before any of
  // it is consumed, so one memory round trip covers the whole stream.
  //   K: B operand of Q·K^T, lane (n = j%16, g) holds K[j][32c + 8g .. +8];
  //   V: B operand of P·V,   lane (n = d%16, g) holds V[16dt + n16][32jb + 8g .. +8].
  Frag16 kb[8][2];
  Frag16 vb[4][4];
#pragma unroll
  for (int jt = 0; jt < 8; ++jt) {
    const int j = jw + 16 * jt + n16;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (j < n)  // rows beyond the valid prefix are never requested
        kb[jt][c].u = *reinterpret_cast<const uint4*>(
            kbase + (size_t)j * kHeadDim + 32 * c + 8 * g);
      else
        kb[jt][c].u = make_uint4(0, 0, 0, 0);
    }
  }
#pragma unroll
  for (int jb = 0; jb < 4; ++jb)
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      const int j0 = jw + 32 * jb + 8 * g;
      if (j0 < n)
        vb[jb][dt].u = *reinterpret_cast<const uint4*>(
            vbase + (size_t)(16 * dt + n16) * a.S + j0);
      else
        vb[jb][dt].u = make_uint4(0, 0, 0, 0);
    }

  // scores: tile jt covers positions jw + 16 jt .. +16; lane holds column
  // n16 of the tile and rows q = 4g + i.
  f32x4_v sc[8];
#pragma unroll
  for (int jt = 0; jt < 8; ++jt) sc[jt] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
  if (wave_live) {
#pragma unroll
    for (int jt = 0; jt < 8; ++jt)
#pragma unroll
      for (int c = 0; c < 2; ++c)
        sc[jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[c].v, kb[jt][c].v,
                                                         sc[jt], 0, 0, 0);
  }

  T5D_STAMP(2);
  // Softmax over all positions of the workgroup, per query row q = 4g + i.
  const bool rows_live = 4 * g < a.nq;
  float mx[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float m = -INFINITY;
#pragma unroll
    for (int jt = 0; jt < 8; ++jt) {
      const int j = jw + 16 * jt + n16;
      float x = round_bf16(sc[jt][i]);
      if (uniform) x = 0.f;
      x = (j < n && rows_live) ? x : -INFINITY;
      sc[jt][i] = x;
      m = fmaxf(m, x);
    }
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    mx[i] = m;
  }
  if (nwaves > 1) {
    if (n16 == 0 && 4 * g < NQP) {
#pragma unroll
      for (int i = 0; i < 4; ++i) s_red[wave][4 * g + i] = mx[i];
    }
    __syncthreads();
    if (4 * g < NQP) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float m = s_red[0][4 * g + i];
        for (int w = 1; w < nwaves; ++w) m = fmaxf(m, s_red[w][4 * g + i]);
        mx[i] = m;
      }
    }
    __syncthreads();
  }
  T5D_STAMP(3);
  float sum[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float s = 0.f;
#pragma unroll
    for (int jt = 0; jt < 8; ++jt) {
      const float x = sc[jt][i];
      const float ex = (x == -INFINITY) ? 0.f : __expf(x - mx[i]);
      sc[jt][i] = ex;
      s += ex;
    }
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) s += __shfl_xor(s, o, 64);
    sum[i] = s;
  }
  if (nwaves > 1) {
    if (n16 == 0 && 4 * g < NQP) {
#pragma unroll
      for (int i = 0; i < 4; ++i) s_red[wave][4 * g + i] = sum[i];
    }
    __syncthreads();
    if (4 * g < NQP) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float s = s_red[0][4 * g + i];
        for (int w = 1; w < nwaves; ++w) s += s_red[w][4 * g + i];
        sum[i] = s;
      }
    }
  }
  T5D_STAMP(4);
  // Normalise, round to bf16, hand to the P·V A-operand layout through LDS.
  if (4 * g < NQP) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float inv = rows_live ? 1.0f / sum[i] : 0.f;
#pragma unroll
      for (int jt = 0; jt < 8; ++jt)
        s_p[wave][4 * g + i][16 * jt + n16] = f32_to_bf16(sc[jt][i] * inv);
    }
  }
  __syncthreads();

  T5D_STAMP(5);
  // out[q][d] = sum_j P[q][j] V[d][j]; A lane (m = n16, g) holds
  // P[m][32 jb + 8g .. +8].
  f32x4_v oc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) oc[dt] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
  if (wave_live) {
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      Frag16 pa;
      if (n16 < NQP)
        pa.u = *reinterpret_cast<const uint4*>(&s_p[wave][n16][32 * jb + 8 * g]);
      else
        pa.u = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
        oc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa.v, vb[jb][dt].v,
                                                         oc[dt], 0, 0, 0);
    }
  }
  T5D_STAMP(6);
  // oc[dt][i] in lane (n16, g) is out[q = 4g + i][d = 16 dt + n16].
  if (nwaves == 1) {
    if (rows_live) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int q = 4 * g + i;
        if (q < a.nq) {
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
            a.out[(size_t)(b * a.nq + q) * HD + h * kHeadDim + 16 * dt + n16] =
                f32_to_bf16(oc[dt][i]);
        }
      }
    }
    return;
  }
  __syncthreads();  // every wavefront is done reading s_p
  if (4 * g < NQP) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
        s_out[wave][4 * g + i][16 * dt + n16] = oc[dt][i];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < a.nq * kHeadDim; e += blockDim.x) {
    const int q = e / kHeadDim, d = e % kHeadDim;
    float acc = s_out[0][q][d];
    for (int w = 1; w < nwaves; ++w) acc += s_out[w][q][d];
    a.out[(size_t)(b * a.nq + q) * HD + h * kHeadDim + d] = f32_to_bf16(acc);
  }
  T5D_STAMP(7);
}

// ---- self-attention ------------------------------------------------------------
// Optionally applies a pending beam gather on the fly: when `pending` is set,
// a workgroup handles the `beams` rows of one batch item (wavefront = beam x
// 128-position block), every wavefront reads the cache of its SOURCE beam
// pending[b, e], and — if the item's beams were actually permuted — writes what
// it read into its own slot after a workgroup barrier (all reads are in
// registers by then, so the in-place permutation is safe).  This replaces a
// separate read+write pass over every cache by the writes alone.
template <int WM>
__global__ void __launch_bounds__(64 * WM)
self_attn_mfma_kernel(AttnMfmaArgs a) {
  __shared__ float s_red[WM];
  __shared__ float s_out[WM][kHeadDim];
  __shared__ __attribute__((aligned(16))) bf16_t s_p[WM][kBlockJ];
  T5D_GATED(a.gate);

  const int h = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nblk = a.nblk;                 // wavefronts per row
  const int blk = wave % nblk;             // 128-position block of this wave
  const int wave0 = wave - blk;            // first wavefront of this row
  const int jc = lane & 15, dg = lane >> 4;  // score layout
  const int n16 = lane & 15, g = lane >> 4;  // MFMA layout
  const int HD = a.H * kHeadDim;
  const int S = a.S;

  int r, rs;             // own row (slot) and source row
  bool permuted = false; // does this batch item need its beams moved?
  if (a.pending != nullptr) {
    const int b = blockIdx.y, e = wave / nblk;
    r = b * a.beams + e;
    int src = a.pending[r];
    src = src < 0 ? 0 : (src >= a.beams ? a.beams - 1 : src);
    rs = b * a.beams + src;
    for (int q = 0; q < a.beams; ++q)
      permuted = permuted || (a.pending[b * a.beams + q] != q);
  } else {
    r = rs = blockIdx.y;
  }

  const int t = *a.index;
  const int n = t + 1;
  const int jw = blk * kBlockJ;
  const bool wave_live = jw < n;
  const bool wave_has_t = t >= jw && t < jw + kBlockJ;
  const size_t slot = (size_t)kHeadDim * S;
  const bf16_t* ksrc = a.k + ((size_t)rs * a.H + h) * slot;
  const bf16_t* vsrc = a.v + ((size_t)rs * a.H + h) * slot;
  bf16_t* kdst = a.k + ((size_t)r * a.H + h) * slot;
  bf16_t* vdst = a.v + ((size_t)r * a.H + h) * slot;
  const bf16_t* qrow = a.q + (size_t)r * a.q_stride + h * kHeadDim;

  // Query and (for the wavefront holding column t) new key, for this lane's
  // 16 head-dim rows d = dg + 4i; new value for its 4 MFMA rows 16 dt + n16.
  float qv[16], knew[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    qv[i] = bf16_to_f32(qrow[dg + 4 * i]);
    knew[i] = wave_has_t ? bf16_to_f32(qrow[HD + dg + 4 * i]) : 0.f;
  }
  bf16_t vnew[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
    vnew[dt] = wave_has_t ? qrow[2 * HD + 16 * dt + n16] : (bf16_t)0;

  // Scores on the vector ALU: lane (dg, jc) owns positions j0 .. j0 + 7.
  const int j0 = jw + 8 * jc;
  const bool live = j0 < n;
  const bool ins = wave_has_t && (t >= j0) && (t < j0 + 8);
  const int e_t = t - j0;
  const int jv = jw + 8 * g;  // + 32 jb: first position of a value chunk
  // All K and V chunks are requested before anything is consumed.
  uint4 kc[16];
  Frag16 vb[4][4];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if (live)
      kc[i] = *reinterpret_cast<const uint4*>(ksrc + (size_t)(dg + 4 * i) * S + j0);
    else
      kc[i] = make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int jb = 0; jb < 4; ++jb)
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      if (jv + 32 * jb < n)
        vb[jb][dt].u = *reinterpret_cast<const uint4*>(
            vsrc + (size_t)(16 * dt + n16) * S + jv + 32 * jb);
      else
        vb[jb][dt].u = make_uint4(0, 0, 0, 0);
    }
  float s[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) s[e] = 0.f;
  if (live) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float kf[8];
      unpack16(kc[i], kf);
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] = fmaf(qv[i], kf[e], s[e]);
    }
  }
  // Score of the position being written, from the new key (the cache column
  // itself still holds its old content in the registers above).
  float snew = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) snew = fmaf(qv[i], knew[i], snew);

  if (permuted) {
    // Every wavefront of the workgroup has its source data in registers (the
    // scores above consumed K; V is forced below) before any slot is written.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (r != rs) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (live)
          *reinterpret_cast<uint4*>(kdst + (size_t)(dg + 4 * i) * S + j0) = kc[i];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
          if (jv + 32 * jb < n)
            *reinterpret_cast<uint4*>(vdst + (size_t)(16 * dt + n16) * S + jv +
                                      32 * jb) = vb[jb][dt].u;
      // the column written below must land after the chunks that cover it
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
  }
  // The column being written: K by the 4 score lanes whose chunk holds t,
  // V by the 16 MFMA lanes whose chunk holds t.
  if (ins) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      kdst[(size_t)(dg + 4 * i) * S + t] = qrow[HD + dg + 4 * i];
  }
  const int tl = t - jw;  // position of column t inside this wavefront
  const int jb_t = tl >> 5, g_t = (tl & 31) >> 3, ev = tl & 7;
  if (wave_has_t && g == g_t) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
      vdst[(size_t)(16 * dt + n16) * S + t] = vnew[dt];
  }

  // Reduce the 4 row groups, add the relative-position bias, mask, softmax.
  snew += __shfl_xor(snew, 16, 64);
  snew += __shfl_xor(snew, 32, 64);
  float m = -INFINITY;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float x = s[e];
    x += __shfl_xor(x, 16, 64);
    x += __shfl_xor(x, 32, 64);
    x = (ins && e == e_t) ? snew : x;
    const int j = j0 + e;
    x = round_bf16(x);
    if (j < n) x = round_bf16(x + bf16_to_f32(a.rel_bias[(size_t)h * S + (t - j)]));
    x = (j < n) ? x : -INFINITY;
    s[e] = x;
    m = fmaxf(m, x);
  }
#pragma unroll
  for (int o = 8; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if (nblk > 1) {
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    m = s_red[wave0];
    for (int w = 1; w < nblk; ++w) m = fmaxf(m, s_red[wave0 + w]);
    __syncthreads();
  }
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float ex = (s[e] == -INFINITY) ? 0.f : __expf(s[e] - m);
    s[e] = ex;
    sum += ex;
  }
#pragma unroll
  for (int o = 8; o >= 1; o >>= 1) sum += __shfl_xor(sum, o, 64);
  if (nblk > 1) {
    if (lane == 0) s_red[wave] = sum;
    __syncthreads();
    sum = s_red[wave0];
    for (int w = 1; w < nblk; ++w) sum += s_red[wave0 + w];
  }
  if (dg == 0) {
    Frag16 pk;
    const float inv = 1.0f / sum;
#pragma unroll
    for (int e = 0; e < 8; ++e) pk.h[e] = f32_to_bf16(s[e] * inv);
    *reinterpret_cast<uint4*>(&s_p[wave][8 * jc]) = pk.u;
  }
  __syncthreads();

  // P·V on the matrix cores; only A row 0 (lanes with n16 == 0) is non-zero.
  // Column t is taken out of the matrix product (the V registers still hold
  // the column's old content) and added from the new value below.
  const float p_t = wave_has_t ? bf16_to_f32(s_p[wave][tl]) : 0.f;
  f32x4_v oc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) oc[dt] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
  if (wave_live) {
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      Frag16 pa;
      if (n16 == 0)
        pa.u = *reinterpret_cast<const uint4*>(&s_p[wave][32 * jb + 8 * g]);
      else
        pa.u = make_uint4(0, 0, 0, 0);
      if (wave_has_t && jb == jb_t && g == g_t) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (e == ev) pa.h[e] = 0;
      }
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
        oc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa.v, vb[jb][dt].v,
                                                         oc[dt], 0, 0, 0);
    }
  }
  // Row 0 of the result: lanes 0..15, element 0 -> out[d = 16 dt + lane].
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
    oc[dt][0] = fmaf(p_t, bf16_to_f32(vnew[dt]), oc[dt][0]);
  if (nblk == 1) {
    if (g == 0) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
        a.out[(size_t)r * HD + h * kHeadDim + 16 * dt + n16] =
            f32_to_bf16(oc[dt][0]);
    }
    return;
  }
  if (g == 0) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) s_out[wave][16 * dt + n16] = oc[dt][0];
  }
  __syncthreads();
  if (blk == 0 && lane < kHeadDim) {
    float acc = s_out[wave0][lane];
    for (int w = 1; w < nblk; ++w) acc += s_out[wave0 + w][lane];
    a.out[(size_t)r * HD + h * kHeadDim + lane] = f32_to_bf16(acc);
  }
}

// ---- dispatch -------------------------------------------------------------------
template <int NQP>
static void launch_cross(const AttnMfmaArgs& a, int B, hipStream_t s) {
  const int waves = (a.S + kBlockJ - 1) / kBlockJ;
  dim3 grid(a.H, B), block(64 * waves);
  if (waves <= 4)
    hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 4>), grid, block, 0, s, a);
  else if (waves <= 8)
    hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 8>), grid, block, 0, s, a);
  else
    hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 16>), grid, block, 0, s, a);
}

int launch_cross_attention_bf16(hipStream_t s, const void* q, const void* k,
                                const void* v, const int32_t* enc_len,
                                void* out, int B, int beams, int H, int E) {
  AttnMfmaArgs a;
  a.q = (const bf16_t*)q; a.k = (bf16_t*)k; a.v = (bf16_t*)v;
  a.rel_bias = nullptr; a.index = enc_len; a.out = (bf16_t*)out;
  a.H = H; a.S = E; a.nq = beams; a.q_stride = H * kHeadDim;
  a.gate = tls_gate;
  if (beams <= 4) launch_cross<4>(a, B, s);
  else launch_cross<8>(a, B, s);
  return 0;
}

int launch_self_attention_bf16(hipStream_t s, const void* qkv, void* ck,
                               void* cv, const void* rel_bias,
                               const int32_t* cache_index, void* out, int R,
                               int H, int L, const int32_t* pending,
                               int beams) {
  AttnMfmaArgs a;
  a.q = (const bf16_t*)qkv; a.k = (bf16_t*)ck; a.v = (bf16_t*)cv;
  a.rel_bias = (const bf16_t*)rel_bias; a.index = cache_index;
  a.out = (bf16_t*)out;
  a.H = H; a.S = L; a.nq = 1; a.q_stride = 3 * H * kHeadDim;
  a.gate = tls_gate;
  a.nblk = (L + kBlockJ - 1) / kBlockJ;
  a.pending = pending;
  a.beams = pending ? beams : 1;
  const int waves = a.nblk * a.beams;
  dim3 grid(H, pending ? R / beams : R), block(64 * waves);
  if (waves <= 4)
    hipLaunchKernelGGL((self_attn_mfma_kernel<4>), grid, block, 0, s, a);
  else if (waves <= 8)
    hipLaunchKernelGGL((self_attn_mfma_kernel<8>), grid, block, 0, s, a);
  else
    hipLaunchKernelGGL((self_attn_mfma_kernel<16>), grid, block, 0, s, a);
  return 0;
}

#ifdef T5D_PROBE
extern "C" int t5d_probe_read(long long* host) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(t5d_probe_buf),
                                  sizeof(long long) * 64 * 16);
}
#endif

}  // namespace t5d
