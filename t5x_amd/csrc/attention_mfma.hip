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
  const int32_t* pending;  // [B, beams] source slot per row, or null
  const int32_t* pending_dst;  // [B, beams] slot per row (null: row e, slot e)
  int beams, nblk;         // rows per workgroup, wavefronts per row
  int n_units;             // self_attn_rows_kernel: rows * heads
  // cross-attention with the query projection fused in (q == nullptr)
  const bf16_t* x;         // [R, d] residual stream
  const bf16_t* ln;        // [d] pre-attention layer-norm scale
  const void* wq;          // packed [d, H*64] query kernel (bf16 tiles)
  int d;
  float eps;
  int v_blocked;  // self-attention: value cache stored as [S/32][64][32] per head
  int k_blocked;  // self-attention: key cache stored the same way
  // cross-attention: optional work order, [B * H] entries
  // head | item << 8 | valid length << 16; workgroup (x, y) takes entry
  // y * H + x instead of (head x, item y, index[y])
  const int32_t* units;
};

constexpr int kHeadDim = 64;
constexpr int kBlockJ = 128;  // positions per wavefront


// ---- cross-attention -----------------------------------------------------------
// scores^T = K·Q^T with the K tile (16 positions x 32 dims) as the A operand
// and Q^T as the B operand whose 16 columns are the NQP (4 or 8) query rows
// repeated REP = 16 / NQP times.  The repeats cost nothing on the matrix
// cores and leave every score in REP lanes; copy s of a column keeps the
// tiles jt = s (mod REP), so the softmax runs on all 64 lanes with 32 / REP
// scores each instead of 32 scores in 16 lanes.  out^T = V·P^T likewise (V
// tile as A, P^T with repeated query columns as B).
//
// NJ > 0 fuses the pre-attention layer norm and the query projection in: the
// workgroup (4 wavefronts) normalises the item's NQP rows of the residual
// stream and multiplies them with the head's 64 columns of the query kernel
// while its K stream is in flight — same k-tile split over wavefronts, same
// accumulation and summation order as gemm_mfma_kernel, so q has the same
// bits as the stand-alone dense layer given the same row statistics.  NJ is
// the number of k-tile pairs per wavefront (d / 256, rounded up).
template <int NQP, int WM, int NJ, bool ONCE = false>
// fused, d <= 768: 2 workgroups per CU (256 registers hold both streams);
// not fused: V is requested once the scores have consumed K, so a wavefront
// needs under 128 registers and every workgroup of a launch of 64 x 16 or
// 16 x 32 (item, head) pairs is resident at once — the K and V streams of the
// whole launch then follow each other without a second round of workgroups
// (T5.1.1-large: 26.1 -> 24.5 us per launch, XL 15.4 -> 13.8, XXL 338 -> 329)
__global__ void __launch_bounds__(64 * WM, NJ > 0 ? (NJ <= 3 ? 2 : 1)
                                                  : (WM <= 8 ? 4 : 1))
cross_attn_mfma_kernel(AttnMfmaArgs a) {
  constexpr int REP = 16 / NQP;   // copies of each query column
  constexpr int TPL = 8 / REP;    // score tiles a lane keeps
  constexpr bool FQ = NJ > 0;
  static_assert(!FQ || WM == 4, "the fused projection splits K over 4 waves");
  __shared__ float s_red[2][WM][16];
  __shared__ float s_ss[FQ ? 4 : 1][16];
  __shared__ __attribute__((aligned(16))) float s_qp[FQ ? 4 : 1][NQP][kHeadDim];
  __shared__ __attribute__((aligned(16))) bf16_t s_qb[FQ ? NQP : 1][kHeadDim];
  __shared__ __attribute__((aligned(16))) bf16_t s_p[WM][NQP][kBlockJ];
  __shared__ __attribute__((aligned(16))) float s_out[WM][NQP][kHeadDim];
  T5D_GATE_READ(a.gate);

  int h = blockIdx.x, b = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nwaves = blockDim.x >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int q = n16 % NQP, rep = n16 / NQP;
  const int HD = a.H * kHeadDim;

  int n;
  if (a.units != nullptr) {
    const int u = a.units[b * a.H + h];
    T5D_GATE_TEST();  // after both scalar loads are in flight
    // (clamped: a table that does not belong to this launch must not become
    // an address)
    h = min(u & 0xff, a.H - 1);
    b = min((u >> 8) & 0xff, (int)gridDim.y - 1);
    n = (int)((uint32_t)u >> 16);
  } else {
    n = a.index[b];
    T5D_GATE_TEST();
  }
  n = n < 0 ? 0 : (n > a.S ? a.S : n);
  bool uniform = false;  // no valid key: the masked softmax is uniform
  if (n == 0) { uniform = true; n = a.S; }

  const int jw = wave * kBlockJ;  // first position of this wavefront
  // K [B, H, 2, S, 32] (the head dim's two halves as planes) and
  // V [B, H, S / 32, 64, 32] (32-position blocks): every fragment load of a
  // wavefront below is one contiguous 1 KB.
  const bf16_t* kbase = a.k + ((size_t)b * a.H + h) * (size_t)a.S * kHeadDim;
  const bf16_t* vbase = a.v + ((size_t)b * a.H + h) * (size_t)kHeadDim * a.S;
  const int nw = n - jw;  // valid positions of this wavefront (may be <= 0)

  // Every K and V chunk is requested up front (whole 16 / 32 position tiles,
  // skipped by wave-uniform branches beyond the valid length; inside a tile
  // the tail past the valid length is read and masked, it must be finite).
  //   K: A operand, lane (row = position n16, g) holds K[j][32c + 8g .. +8];
  //   V: A operand, lane (row = d n16, g) holds V[16dt + n16][32jb + 8g .. +8].
  // S is a multiple of 8 but not of the tile sizes: addresses are clamped to
  // the last row / last 8 positions (those positions are masked anyway).
  Frag16 kb[8][2];
  Frag16 vb[4][4];
  // Fused projection: this wavefront's k-tile pairs p = wave + 4 j.
  Frag16 xa[FQ ? NJ : 1][2];      // A: rows of x (row n16), k = 8g .. +8
  uint4 lnv[FQ ? NJ : 1][2];      // layer-norm scale for the same k
  Frag16 wt[FQ ? NJ : 1][2][4];   // B: query-kernel tiles of this head
  const int KT = FQ ? a.d >> 5 : 0;
  if constexpr (FQ) {
    const int xr = b * a.nq + (n16 < a.nq ? n16 : 0);
    const bf16_t* xrow = a.x + (size_t)xr * a.d + 8 * g;
    const char* wbase = reinterpret_cast<const char*>(a.wq);
    // Rows, then the norm scale, then the weight tiles: loads return in the
    // order they were issued, and the row statistics need only the rows.
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int kt = min((wave + 4 * j) * 2 + hh, KT - 1);
        xa[j][hh].u = *reinterpret_cast<const uint4*>(xrow + 32 * kt);
      }
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int kt = min((wave + 4 * j) * 2 + hh, KT - 1);
        lnv[j][hh] = *reinterpret_cast<const uint4*>(a.ln + 32 * kt + 8 * g);
      }
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int kt = min((wave + 4 * j) * 2 + hh, KT - 1);
#pragma unroll
        for (int nn = 0; nn < 4; ++nn)
          wt[j][hh][nn].u = reinterpret_cast<const uint4*>(
              wbase + ((size_t)(4 * h + nn) * KT + kt) * 1024)[lane];
      }
  }
#pragma unroll
  for (int jt = 0; jt < 8; ++jt) {
    if (16 * jt < nw) {
#pragma unroll
      for (int c = 0; c < 2; ++c)
        kb[jt][c].u = load_kv<ONCE>(reinterpret_cast<const uint4*>(
            kbase + ((size_t)c * a.S + min(jw + 16 * jt + n16, a.S - 1)) * 32 +
            8 * g));
    } else {
      kb[jt][0].u = kb[jt][1].u = make_uint4(0, 0, 0, 0);
    }
  }
  auto load_v = [&]() {
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      if (32 * jb < nw) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
          vb[jb][dt].u = load_kv<ONCE>(reinterpret_cast<const uint4*>(
              vbase + ((size_t)(wave * (kBlockJ / 32) + jb) * kHeadDim +
                       16 * dt + n16) * 32 + 8 * g));
      } else {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) vb[jb][dt].u = make_uint4(0, 0, 0, 0);
      }
    }
  };
  // B operand of K·Q^T: lane (col n16 -> query q, g) holds Q[q][32c + 8g .. +8].
  Frag16 qb[2];
  if constexpr (!FQ) {
    const bool qrow = q < a.nq;
    const bf16_t* qp = a.q + (size_t)(b * a.nq + (qrow ? q : 0)) * a.q_stride +
                       h * kHeadDim + 8 * g;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      qb[c].u = *reinterpret_cast<const uint4*>(qp + 32 * c);
      if (!qrow) qb[c].u = make_uint4(0, 0, 0, 0);
    }
  } else {
    // Row statistics: sum of squares of row n16 over this wavefront's k range.
    const int n_pairs = KT >> 1;
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      if (wave + 4 * j < n_pairs) {
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          float f[8];
          unpack16(xa[j][hh].u, f);
#pragma unroll
          for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
        }
      }
    }
    ss = rows_sum(ss);
    if (g == 0) s_ss[wave][n16] = n16 < a.nq ? ss : 0.f;
    __syncthreads();
    const float tot = (s_ss[0][n16] + s_ss[2][n16]) + (s_ss[1][n16] + s_ss[3][n16]);
    const float inv = 1.0f / sqrtf(tot / (float)a.d + a.eps);
    f32x4_v qacc[4];
#pragma unroll
    for (int nn = 0; nn < 4; ++nn) qacc[nn] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      if (wave + 4 * j < n_pairs) {
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          float xf[8], sf[8];
          unpack16(xa[j][hh].u, xf);
          unpack16(lnv[j][hh], sf);
          uint32_t o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float y0 = round_bf16(xf[2 * e] * inv);
            const float y1 = round_bf16(xf[2 * e + 1] * inv);
            o[e] = pack_bf16x2(y0 * sf[2 * e], y1 * sf[2 * e + 1]);
          }
          Frag16 an;
          an.u = n16 < a.nq ? make_uint4(o[0], o[1], o[2], o[3])
                            : make_uint4(0, 0, 0, 0);
#pragma unroll
          for (int nn = 0; nn < 4; ++nn)
            qacc[nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                an.v, wt[j][hh][nn].v, qacc[nn], 0, 0, 0);
        }
      }
    }
    // qacc[nn][i] in lane (n16, g) is the partial q[row 4g + i][16 nn + n16].
    if (4 * g < NQP) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int nn = 0; nn < 4; ++nn)
          s_qp[wave][4 * g + i][16 * nn + n16] = qacc[nn][i];
    }
    load_v();  // the V stream follows K while the projection is reduced
    __syncthreads();
    for (int e = threadIdx.x; e < NQP * kHeadDim; e += 64 * WM) {
      const int row = e / kHeadDim, col = e % kHeadDim;
      const float v = (s_qp[0][row][col] + s_qp[2][row][col]) +
                      (s_qp[1][row][col] + s_qp[3][row][col]);
      s_qb[row][col] = f32_to_bf16(v);
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 2; ++c)
      qb[c].u = *reinterpret_cast<const uint4*>(&s_qb[q][32 * c + 8 * g]);
  }

  // Tile jt: lane (n16, g) gets scores of positions 16 jt + 4g + i, query q.
  // It keeps the tiles with jt % REP == rep.
  float sc[TPL][4];
#pragma unroll
  for (int t = 0; t < TPL; ++t)
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      const int jt = t * REP + r;
      f32x4_v acc = (f32x4_v){0.f, 0.f, 0.f, 0.f};
      if (16 * jt < nw) {
#pragma unroll
        for (int c = 0; c < 2; ++c)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[jt][c].v, qb[c].v,
                                                        acc, 0, 0, 0);
      }
      if (REP == 1 || r == rep) {
#pragma unroll
        for (int i = 0; i < 4; ++i) sc[t][i] = acc[i];
      }
    }

  if constexpr (!FQ) load_v();  // K is consumed: its registers take V
  // Softmax over all positions of the workgroup for query q.  The 16 lanes
  // that share q differ in lane bits {2,3 (if REP == 4) | 3 (REP == 2)} and
  // in g (bits 4, 5).
  float m = -INFINITY;
#pragma unroll
  for (int t = 0; t < TPL; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = 16 * (t * REP + rep) + 4 * g + i;  // within the wavefront
      float x = uniform ? 0.f : round_bf16(sc[t][i]);
      x = j < nw ? x : -INFINITY;
      sc[t][i] = x;
      m = fmaxf(m, x);
    }
  if (NQP <= 4) m = fmaxf(m, lane_xor4(m));
  if (NQP <= 8) m = fmaxf(m, lane_xor8(m));
  m = rows_max(m);
  if (nwaves > 1) {
    if (lane < 16) s_red[0][wave][lane] = m;  // lanes 0..15: q = lane % NQP
    __syncthreads();
    m = s_red[0][0][n16];
    for (int w = 1; w < nwaves; ++w) m = fmaxf(m, s_red[0][w][n16]);
  }
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < TPL; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float ex = __expf(sc[t][i] - m);  // exp(-inf) == 0
      sc[t][i] = ex;
      sum += ex;
    }
  if (NQP <= 4) sum += lane_xor4(sum);
  if (NQP <= 8) sum += lane_xor8(sum);
  sum = rows_sum(sum);
  if (nwaves > 1) {
    if (lane < 16) s_red[1][wave][lane] = sum;
    __syncthreads();
    sum = s_red[1][0][n16];
    for (int w = 1; w < nwaves; ++w) sum += s_red[1][w][n16];
  }
  // Normalise, round to bf16 (where the reference rounds), hand over to the
  // B-operand layout of V·P^T through LDS: 4 consecutive positions per tile.
  {
    const float inv = 1.0f / sum;
#pragma unroll
    for (int t = 0; t < TPL; ++t) {
      uint2 pk;
      pk.x = pack_bf16x2(sc[t][0] * inv, sc[t][1] * inv);
      pk.y = pack_bf16x2(sc[t][2] * inv, sc[t][3] * inv);
      *reinterpret_cast<uint2*>(&s_p[wave][q][16 * (t * REP + rep) + 4 * g]) = pk;
    }
  }
  __syncthreads();

  // out^T[d][q] = sum_j V[d][j] P[q][j]; B lane (col n16 -> q, g) holds
  // P[q][32 jb + 8g .. +8].
  f32x4_v oc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) oc[dt] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int jb = 0; jb < 4; ++jb) {
    if (32 * jb < nw) {
      Frag16 pb;
      pb.u = *reinterpret_cast<const uint4*>(&s_p[wave][q][32 * jb + 8 * g]);
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
        oc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vb[jb][dt].v, pb.v,
                                                         oc[dt], 0, 0, 0);
    }
  }
  // oc[dt][i] in lane (n16, g) is out[q][d = 16 dt + 4g + i] (all REP copies).
  if (nwaves == 1) {
    if (rep == 0 && q < a.nq) {
      bf16_t* o = a.out + (size_t)(b * a.nq + q) * HD + h * kHeadDim + 4 * g;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        uint2 pk;
        pk.x = pack_bf16x2(oc[dt][0], oc[dt][1]);
        pk.y = pack_bf16x2(oc[dt][2], oc[dt][3]);
        *reinterpret_cast<uint2*>(o + 16 * dt) = pk;
      }
    }
    return;
  }
  if (rep == 0) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
      *reinterpret_cast<float4*>(&s_out[wave][q][16 * dt + 4 * g]) =
          make_float4(oc[dt][0], oc[dt][1], oc[dt][2], oc[dt][3]);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < a.nq * kHeadDim; e += blockDim.x) {
    const int qq = e / kHeadDim, d = e % kHeadDim;
    float acc = s_out[0][qq][d];
    for (int w = 1; w < nwaves; ++w) acc += s_out[w][qq][d];
    a.out[(size_t)(b * a.nq + qq) * HD + h * kHeadDim + d] = f32_to_bf16(acc);
  }
}

// ---- self-attention ------------------------------------------------------------
// Sum across the 4 row groups of a wavefront (lane bits 4 and 5) of 8 values,
// leaving each lane with 2 of the 8 totals (reduce-scatter): one
// v_permlane32_swap / v_permlane16_swap plus one add per pair of registers.
// Lane (bit5, bit4) ends with totals 4*bit5 + 2*bit4 + {0, 1}.
__device__ __forceinline__ void reduce_scatter_8(const float (&s)[8],
                                                 float (&out)[2]) {
  float r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    auto w = __builtin_amdgcn_permlane32_swap(__float_as_uint(s[e]),
                                              __float_as_uint(s[e + 4]), false,
                                              false);
    r[e] = __uint_as_float(w[0]) + __uint_as_float(w[1]);
  }
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    auto w = __builtin_amdgcn_permlane16_swap(__float_as_uint(r[e]),
                                              __float_as_uint(r[e + 2]), false,
                                              false);
    out[e] = __uint_as_float(w[0]) + __uint_as_float(w[1]);
  }
}

// One wavefront per (row, 128-position block).  Optionally applies a pending
// beam gather on the fly: when `pending` is set, a workgroup handles the
// `beams` rows of one batch item, every wavefront reads the cache of its
// SOURCE beam pending[b, e], and — if the item's beams were actually permuted —
// writes what it read into its own slot after a workgroup barrier (all reads
// are in registers by then, so the in-place permutation is safe).  This
// replaces a separate read+write pass over every cache by the writes alone.
// With `pending_dst` the row's own slot is pending_dst[b, e] rather than e: a
// caller that lets beams inherit their parents' slots writes only the rows
// of beams whose parent has another child.
//
//   scores: vector ALU.  Lane (dg = lane / 16, jc = lane % 16) multiplies head
//     dims 16 dg .. +16 of the query with positions 8 jc .. +8 of the key
//     cache (one 16-byte load per dim), the 4 dg partials are reduce-scattered
//     so each lane softmaxes 2 positions.
//   out^T = V·P^T on the matrix cores: V chunks are the A operand (rows = head
//     dim, k = position), P^T the B operand with the single query repeated in
//     all 16 columns, so every lane ends with 4 consecutive outputs per tile.
//   The column being written (position t) never goes through the cache: its
//   score comes from the new key, its output share from the new value.
constexpr int kMaxSelfLen = 2048;

template <int WM>
__global__ void __launch_bounds__(64 * WM)
self_attn_mfma_kernel(AttnMfmaArgs a) {
  __shared__ float s_red[2][WM];
  __shared__ float s_pt[WM];
  __shared__ __attribute__((aligned(16))) float s_out[WM][kHeadDim];
  __shared__ __attribute__((aligned(16))) bf16_t s_p[WM][kBlockJ];
  __shared__ float s_bias[kMaxSelfLen];
  T5D_GATE_READ(a.gate);

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

  int r, rs, rw;         // row of the step; cache slot it reads; its own slot
  bool permuted = false; // does this batch item need cache rows moved?
  if (a.pending != nullptr) {
    const int b = blockIdx.y, e = wave / nblk;
    auto in_range = [&](int v) { return v < 0 ? 0 : (v >= a.beams ? a.beams - 1 : v); };
    r = b * a.beams + e;
    rs = b * a.beams + in_range(a.pending[r]);
    rw = a.pending_dst ? b * a.beams + in_range(a.pending_dst[r]) : r;
    for (int q = 0; q < a.beams; ++q)
      permuted = permuted ||
                 (a.pending[b * a.beams + q] !=
                  (a.pending_dst ? a.pending_dst[b * a.beams + q] : q));
  } else {
    r = rs = rw = blockIdx.y;
  }

  const int t_in = *a.index;
  T5D_GATE_TEST();  // after the scalar loads above are in flight
  // A cache index outside [0, S) (a decode loop longer than its cache) must
  // not become an address: nothing is inserted then and all S columns are
  // attended with the bias row of the last position, which is what the
  // reference's one-hot insert and clamped slices do (layers.py:258-303).
  const bool past_end = t_in < 0 || t_in >= S;
  const int t = past_end ? S - 1 : t_in;
  const int n = t + 1;
  const int jw = blk * kBlockJ;
  const int nw = n - jw;  // positions of this wavefront in use (may be <= 0)
  const bool wave_has_t = !past_end && t >= jw && t < jw + kBlockJ;
  const size_t slot = (size_t)kHeadDim * S;
  const bf16_t* ksrc = a.k + ((size_t)rs * a.H + h) * slot;
  const bf16_t* vsrc = a.v + ((size_t)rs * a.H + h) * slot;
  bf16_t* kdst = a.k + ((size_t)rw * a.H + h) * slot;
  bf16_t* vdst = a.v + ((size_t)rw * a.H + h) * slot;
  const bf16_t* qrow = a.q + (size_t)r * a.q_stride + h * kHeadDim;

  // Relative-position bias of this head, by distance, for the softmax below.
  for (int i = threadIdx.x; i < n; i += blockDim.x)
    s_bias[i] = bf16_to_f32(a.rel_bias[(size_t)h * S + i]);

  // All K and V chunks are requested before anything is consumed.  K: lanes
  // whose 8 positions lie beyond the current length skip their loads (one
  // predicated region; what they compute is masked).  V: whole 32-position
  // groups are skipped by wave-uniform branches, together with their matrix
  // products.  Offsets are clamped to the row end when S is not a multiple of
  // the tile (those positions are masked).
  // K: head dim 16 dg + i, positions j0 .. j0 + 7.  Reference layout [64][S]:
  // a head dim's positions are contiguous, a lane's 16 chunks are S apart.
  // Blocked layout [S/32][64][32]: the chunk sits in block j0 / 32, the 16
  // chunks are 64 bytes apart and the cache of a head is read as whole 4 KB
  // blocks up to the current length instead of the first part of 64 rows.
  const int j0 = jw + 8 * jc;
  const bool live = j0 < n;
  const int j0c = min(j0, S - 8);
  const uint32_t koff =
      a.k_blocked
          ? (uint32_t)(((j0c >> 5) * kHeadDim + 16 * dg) * 32 + (j0c & 31)) * 2u
          : (uint32_t)(16 * dg * S + j0c) * 2u;
  const uint32_t kdim = (a.k_blocked ? 32u : (uint32_t)S) * 2u;  // next head dim
  uint4 kc[16];
  if (live) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      kc[i] = *reinterpret_cast<const uint4*>(
          reinterpret_cast<const char*>(ksrc) + i * kdim + koff);
  }
  // Byte offset of this lane's chunk of V tile (jb, dt) inside the head's
  // slot.  Reference layout [64][S]: row 16 dt + n16, positions 32 jb + 8 g ..;
  // blocked layout [S/32][64][32] (S a multiple of 32): the same chunk sits in
  // block blk * 4 + jb, and the 64 chunks of a tile are 1 KB of consecutive
  // memory instead of 16 separate half cache lines.
  uint32_t voff[4];
#pragma unroll
  for (int jb = 0; jb < 4; ++jb)
    voff[jb] = a.v_blocked
                   ? (uint32_t)(((blk * 4 + jb) * kHeadDim + n16) * 32 + 8 * g) * 2u
                   : (uint32_t)(n16 * S + min(jw + 32 * jb + 8 * g, S - 8)) * 2u;
  const uint32_t vdt = (a.v_blocked ? 16u * 32u : 16u * (uint32_t)S) * 2u;
  Frag16 vb[4][4];
#pragma unroll
  for (int jb = 0; jb < 4; ++jb) {
    if (32 * jb < nw) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
        vb[jb][dt].u = *reinterpret_cast<const uint4*>(
            reinterpret_cast<const char*>(vsrc) + dt * vdt + voff[jb]);
    }
  }
  // Query: this lane's 16 head dims.  New key / value / query element of
  // head dim `lane` for the column being written.
  float qv[16];
  {
    const uint4* qp = reinterpret_cast<const uint4*>(qrow + 16 * dg);
    float f[8];
    unpack16(qp[0], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[e] = f[e];
    unpack16(qp[1], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[8 + e] = f[e];
  }
  const bf16_t knew_d = qrow[HD + lane];
  const bf16_t vnew_d = qrow[2 * HD + lane];
  // Score of position t from the new key.
  float snew = wave_sum(bf16_to_f32(qrow[lane]) * bf16_to_f32(knew_d));

  float s8[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) s8[e] = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    float kf[8];
    unpack16(kc[i], kf);
#pragma unroll
    for (int e = 0; e < 8; ++e) s8[e] = fmaf(qv[i], kf[e], s8[e]);
  }

  if (permuted) {
    // Every wavefront of the workgroup has its source data in registers
    // before any slot is written.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (rw != rs) {
      if (live) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
          *reinterpret_cast<uint4*>(reinterpret_cast<char*>(kdst) + i * kdim +
                                    koff) = kc[i];
      }
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        if (32 * jb < nw) {
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
            *reinterpret_cast<uint4*>(reinterpret_cast<char*>(vdst) + dt * vdt +
                                      voff[jb]) = vb[jb][dt].u;
        }
      }
    }
  } else {
    __syncthreads();  // s_bias
  }
  // The column being written: lane d stores element d of the new key / value.
  // It must land after this wavefront's chunk stores above that cover it, so
  // it is issued last, when waiting for those stores costs nothing.
  auto store_column = [&]() {
    if (wave_has_t) {
      if (rw != rs) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      const size_t plain = (size_t)lane * S + t;
      const size_t blocked = ((size_t)(t >> 5) * kHeadDim + lane) * 32 + (t & 31);
      kdst[a.k_blocked ? blocked : plain] = knew_d;
      vdst[a.v_blocked ? blocked : plain] = vnew_d;
    }
  };

  // 2 positions per lane: bias, mask, softmax.
  float sc[2];
  reduce_scatter_8(s8, sc);
  const int jp = j0 + 4 * (dg >> 1) + 2 * (dg & 1);  // first of the 2 positions
  float m = -INFINITY;
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int j = jp + e;
    float x = (j == t && !past_end) ? snew : sc[e];
    x = round_bf16(x);
    if (j < n) x = round_bf16(x + s_bias[t - j]);
    else x = -INFINITY;
    sc[e] = x;
    m = fmaxf(m, x);
  }
  m = wave_max(m);
  if (nblk > 1) {
    if (lane == 0) s_red[0][wave] = m;
    __syncthreads();
    m = s_red[0][wave0];
    for (int w = 1; w < nblk; ++w) m = fmaxf(m, s_red[0][wave0 + w]);
  }
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    sc[e] = __expf(sc[e] - m);  // exp(-inf) == 0
    sum += sc[e];
  }
  sum = wave_sum(sum);
  if (nblk > 1) {
    if (lane == 0) s_red[1][wave] = sum;
    __syncthreads();
    sum = s_red[1][wave0];
    for (int w = 1; w < nblk; ++w) sum += s_red[1][wave0 + w];
  }
  {
    // Normalised probabilities, rounded to bf16 where the reference rounds.
    // Position t is kept out of the matrix product (the V registers hold the
    // column's old content): its probability goes to s_pt instead.
    const float inv = 1.0f / sum;
    float p0 = round_bf16(sc[0] * inv), p1 = round_bf16(sc[1] * inv);
    if (jp == t && !past_end) { s_pt[wave] = p0; p0 = 0.f; }
    if (jp + 1 == t && !past_end) { s_pt[wave] = p1; p1 = 0.f; }
    *reinterpret_cast<uint32_t*>(&s_p[wave][jp - jw]) = pack_bf16x2(p0, p1);
  }
  __syncthreads();

  // out^T tile dt: lane (n16, g) gets out[16 dt + 4g + i], i < 4, in every
  // column n16.  B lane (col, g) holds P[32 jb + 8g .. +8].
  f32x4_v oc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) oc[dt] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int jb = 0; jb < 4; ++jb) {
    if (32 * jb < nw) {
      Frag16 pb;
      pb.u = *reinterpret_cast<const uint4*>(&s_p[wave][32 * jb + 8 * g]);
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
        oc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vb[jb][dt].v, pb.v,
                                                         oc[dt], 0, 0, 0);
    }
  }
  if (wave_has_t) {
    const float p_t = s_pt[wave];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      const uint2 vn = *reinterpret_cast<const uint2*>(qrow + 2 * HD + 16 * dt +
                                                       4 * g);
      oc[dt][0] = fmaf(p_t, bf16lo_to_f32(vn.x), oc[dt][0]);
      oc[dt][1] = fmaf(p_t, bf16hi_to_f32(vn.x), oc[dt][1]);
      oc[dt][2] = fmaf(p_t, bf16lo_to_f32(vn.y), oc[dt][2]);
      oc[dt][3] = fmaf(p_t, bf16hi_to_f32(vn.y), oc[dt][3]);
    }
  }
  if (nblk == 1) {
    if (n16 == 0) {
      bf16_t* o = a.out + (size_t)r * HD + h * kHeadDim + 4 * g;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        uint2 pk;
        pk.x = pack_bf16x2(oc[dt][0], oc[dt][1]);
        pk.y = pack_bf16x2(oc[dt][2], oc[dt][3]);
        *reinterpret_cast<uint2*>(o + 16 * dt) = pk;
      }
    }
    store_column();
    return;
  }
  if (n16 == 0) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
      *reinterpret_cast<float4*>(&s_out[wave][16 * dt + 4 * g]) =
          make_float4(oc[dt][0], oc[dt][1], oc[dt][2], oc[dt][3]);
  }
  __syncthreads();
  if (blk == 0) {
    float acc = s_out[wave0][lane];
    for (int w = 1; w < nblk; ++w) acc += s_out[wave0 + w][lane];
    a.out[(size_t)r * HD + h * kHeadDim + lane] = f32_to_bf16(acc);
  }
  store_column();
}


// ---- self-attention on caches laid out for the decode loop -----------------------
// The column a step appends is 64 head dims of ONE position.  In the reference
// layout (and in the blocked ones above) those are 64 separate 2-byte stores
// into 64 different cache lines per (row, head) and cache: partial-line
// writes, which the memory system turns into read-modify-write cycles —
// measured at 2.1 us of a 13.8 us launch over 128 rows x 12 heads and 21 us
// of 73 us over 128 x 64, against nothing measurable for one 128-byte line.
// A loop that owns its caches therefore keeps them like this ("tail" layout,
// value_blocked == 3), per (row, head) slot of (L + 32) * 64 elements:
//   keys    [L + 32][64]: position-major, a new key is one full line.  The
//           score arithmetic does not care: lane (dg, jc) still multiplies
//           head dims 16 dg .. +16 with positions 8 jc .. +8 in the same
//           order, it just finds a position's 16 dims in two 16-byte loads
//           instead of a dim's 8 positions in one.
//   values  [L / 32 + 1][64][32]: blocks of 32 positions as before (the layout
//           the matrix cores take operands from), but a block is written
//           once, whole, when its 32nd position arrives.  Until then its
//           positions live in the slot's last block, the tail, as [32][64]
//           position-major (a new value is one full line); a step reads the
//           tail lane-linearly, turns it into the operand layout through LDS
//           and, on the block's last position, stores the operand registers
//           as the finished block (4 KB of consecutive memory).
// One wavefront does all of a (row, head) pair and walks its NC chunks of 128
// positions itself, so nothing is exchanged between wavefronts, and a
// workgroup is just WM consecutive pairs without any barrier.  That holds for
// rows that are never reordered (the sampling loops) and equally for a beam
// search's rows when every row has a slot of its own to keep its cache in
// (pending_dst): the slot rule — a new beam keeps the slot it read unless an
// earlier one does, and then takes one that no new beam reads — means no
// wavefront writes what another reads.  Pairs being independent, the launch
// is cut into workgroups of 4, 2 or 1 so that the CUs get equal shares (128
// rows x 12 heads as 768 workgroups of 2: 3 per CU, where workgroups of one
// batch item's 4 beams put 2 on half of the CUs and 1 on the others).
//   BARRIER: a gather WITHOUT destination slots permutes an item's rows in
//     place; a workgroup is then the item's `beams` rows, with the one
//     barrier of self_attn_mfma_kernel when the item's beams moved; NC == 1.
// Operation for operation the arithmetic is that of self_attn_mfma_kernel
// (per-chunk partial sums added by rising chunk), so the results have the
// same bits whatever the layout.
constexpr int kTailRow = 144;  // bytes per position of the tail tile in LDS
constexpr int kCUs = 256;       // compute units of the device (MI355X)

template <int NC, int WM, bool BARRIER>
__global__ void __launch_bounds__(64 * WM, BARRIER ? 1 : 2)
self_attn_tail_kernel(AttnMfmaArgs a) {
  static_assert(!BARRIER || NC == 1, "a row permuted in place is one chunk");
  __shared__ __attribute__((aligned(16))) bf16_t s_p[WM][NC * kBlockJ];
  __shared__ __attribute__((aligned(16))) unsigned char s_tail[WM][32 * kTailRow];
  __shared__ float s_pt[WM];
  T5D_GATE_READ(a.gate);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int jc = lane & 15, dg = lane >> 4;  // score layout
  const int n16 = lane & 15, g = lane >> 4;  // MFMA layout
  const int HD = a.H * kHeadDim;
  const int S = a.S;

  int r, h;              // row of the step, head
  if (BARRIER) {
    h = blockIdx.x;
    r = blockIdx.y * a.beams + wave;
  } else {
    const int unit = blockIdx.x * WM + wave;
    r = unit / a.H;
    h = unit - r * a.H;
    if (r >= a.n_units / a.H) return;  // no barrier on this path
  }
  int rs = r, rw = r;    // slot the row reads; slot it keeps
  bool permuted = false; // BARRIER: does this batch item need rows moved?
  if (a.pending != nullptr) {
    const int b0 = r / a.beams * a.beams;
    auto in_range = [&](int v) { return v < 0 ? 0 : (v >= a.beams ? a.beams - 1 : v); };
    rs = b0 + in_range(a.pending[r]);
    if (a.pending_dst) rw = b0 + in_range(a.pending_dst[r]);
    if (BARRIER)
      for (int q = 0; q < a.beams; ++q)
        permuted = permuted || a.pending[b0 + q] != q;
  }
  const int t_in = *a.index;
  T5D_GATE_TEST();  // after the scalar loads above are in flight
  const bool copy = rw != rs;  // what the row reads goes into its own slot

  // (self_attn_mfma_kernel explains the index outside [0, S).)  By then every
  // block is finished: nothing is in the tail.
  const bool past_end = t_in < 0 || t_in >= S;
  const int t = past_end ? S - 1 : t_in;
  const int n = t + 1;
  const int pb = past_end ? (S >> 5) : (t >> 5);  // the block still in the tail
  const int tl = past_end ? 0 : (t & 31);         // positions the tail holds
  const size_t slot = (size_t)kHeadDim * (S + 32) * 2;  // bytes
  const size_t tail_at = (size_t)(S >> 5) * 4096;
  const char* ksrc = reinterpret_cast<const char*>(a.k) + ((size_t)rs * a.H + h) * slot;
  const char* vsrc = reinterpret_cast<const char*>(a.v) + ((size_t)rs * a.H + h) * slot;
  char* kdst = reinterpret_cast<char*>(a.k) + ((size_t)rw * a.H + h) * slot;
  char* vdst = reinterpret_cast<char*>(a.v) + ((size_t)rw * a.H + h) * slot;
  const bf16_t* qrow = a.q + (size_t)r * a.q_stride + h * kHeadDim;

  // Keys of every chunk in use: lane (dg, jc) takes head dims 16 dg .. +16 of
  // positions 128 c + 8 jc .. +8, 32 bytes of each position's line.
  uint4 kr[NC][8][2];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int j0 = c * kBlockJ + 8 * jc;
    if (j0 < n) {
      const char* p = ksrc + ((size_t)j0 * kHeadDim + 16 * dg) * 2;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        kr[c][e][0] = *reinterpret_cast<const uint4*>(p + e * 128);
        kr[c][e][1] = *reinterpret_cast<const uint4*>(p + e * 128 + 16);
      }
    }
  }
  // The step's own row: query (this lane's 16 head dims for the scores, its
  // own element for the new column's score), new key / value elements.
  float qv[16];
  {
    const uint4* qp = reinterpret_cast<const uint4*>(qrow + 16 * dg);
    float f[8];
    unpack16(qp[0], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[e] = f[e];
    unpack16(qp[1], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[8 + e] = f[e];
  }
  const bf16_t q_d = qrow[lane];
  const bf16_t knew_d = qrow[HD + lane];
  const bf16_t vnew_d = qrow[2 * HD + lane];
  // (the new value again, as this lane's 4 outputs per tile need it: with two
  // chunks of keys in flight the registers are short, and it is asked for
  // after the scores instead, behind the softmax)
  uint2 vn[4];
  auto load_vn = [&]() {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
      vn[dt] = *reinterpret_cast<const uint2*>(qrow + 2 * HD + 16 * dt + 4 * g);
  };
  if (NC == 1) load_vn();
  // Relative-position bias of this lane's 2 positions per chunk, by distance.
  float bias[NC][2];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int jp = c * kBlockJ + 8 * jc + 4 * (dg >> 1) + 2 * (dg & 1);
#pragma unroll
    for (int e = 0; e < 2; ++e)
      bias[c][e] = jp + e < n
                       ? bf16_to_f32(a.rel_bias[(size_t)h * S + (t - jp - e)])
                       : 0.f;
  }
  // The tail: positions 32 pb .. t - 1, 128 bytes each, read lane-linearly
  // (lane l of load k has 8 head dims of position 8 k + l / 8).
  uint4 tr[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    tr[k] = make_uint4(0, 0, 0, 0);
    if (8 * k + (lane >> 3) < tl)
      tr[k] = *reinterpret_cast<const uint4*>(vsrc + tail_at + k * 1024 + lane * 16);
  }
  // Finished value blocks: whole 32-position groups (1 KB per tile).
  Frag16 vb[NC][4][4];
  auto load_values = [&](int c) {
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      if (c * 4 + jb < pb) {
        const char* p = vsrc + ((size_t)((c * 4 + jb) * kHeadDim + n16) * 32 + 8 * g) * 2;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
          vb[c][jb][dt].u = *reinterpret_cast<const uint4*>(p + dt * 1024);
      }
    }
  };
  // One chunk: keys and values in flight together.  Two: the registers hold
  // both chunks' keys or one chunk's keys and values, so a chunk's values are
  // requested when its scores have freed the registers of its keys.
  if (NC == 1) load_values(0);
  __builtin_amdgcn_sched_barrier(0);

  const float snew = wave_sum(bf16_to_f32(q_d) * bf16_to_f32(knew_d));
  float sc[NC][2];
  float m = -INFINITY;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    if (c * kBlockJ < n) {
      float s8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // position e of this lane: its 16 head dims in rising order
        float kf[8], acc = 0.f;
        unpack16(kr[c][e][0], kf);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = fmaf(qv[i], kf[i], acc);
        unpack16(kr[c][e][1], kf);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = fmaf(qv[8 + i], kf[i], acc);
        s8[e] = acc;
      }
      if (BARRIER && permuted) {
        // Every wavefront of the item has its source data in registers
        // before any slot is written.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
      }
      if (copy && c * kBlockJ + 8 * jc < n) {
        char* p = kdst + ((size_t)(c * kBlockJ + 8 * jc) * kHeadDim + 16 * dg) * 2;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          *reinterpret_cast<uint4*>(p + e * 128) = kr[c][e][0];
          *reinterpret_cast<uint4*>(p + e * 128 + 16) = kr[c][e][1];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (NC > 1) load_values(c);  // into the registers the keys have left
      __builtin_amdgcn_sched_barrier(0);
      reduce_scatter_8(s8, sc[c]);
      const int jp = c * kBlockJ + 8 * jc + 4 * (dg >> 1) + 2 * (dg & 1);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int j = jp + e;
        float x = (j == t && !past_end) ? snew : sc[c][e];
        x = round_bf16(x);
        if (j < n) x = round_bf16(x + bias[c][e]);
        else x = -INFINITY;
        sc[c][e] = x;
        m = fmaxf(m, x);
      }
    } else {
      sc[c][0] = sc[c][1] = -INFINITY;
    }
  }
  if (NC > 1) load_vn();
  // The tail into LDS, one position per row, the new value as position tl (it
  // takes part in the matrix product with probability 0, see below, and
  // completes the block when tl == 31); positions beyond are zero.
#pragma unroll
  for (int k = 0; k < 4; ++k)
    *reinterpret_cast<uint4*>(&s_tail[wave][(8 * k + (lane >> 3)) * kTailRow +
                                            (lane & 7) * 16]) = tr[k];
  if (copy) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (8 * k + (lane >> 3) < tl)
        *reinterpret_cast<uint4*>(vdst + tail_at + k * 1024 + lane * 16) = tr[k];
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  if (!past_end)
    *reinterpret_cast<bf16_t*>(&s_tail[wave][tl * kTailRow + lane * 2]) = vnew_d;

  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    float part = 0.f;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      sc[c][e] = __expf(sc[c][e] - m);  // exp(-inf) == 0
      part += sc[c][e];
    }
    part = wave_sum(part);
    sum = c == 0 ? part : sum + part;
  }
  {
    // Normalised probabilities, rounded to bf16 where the reference rounds.
    // Position t is kept out of the matrix product: its probability goes to
    // s_pt and its output share is added from the new value below.
    const float inv = 1.0f / sum;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int jp = c * kBlockJ + 8 * jc + 4 * (dg >> 1) + 2 * (dg & 1);
      float p0 = round_bf16(sc[c][0] * inv), p1 = round_bf16(sc[c][1] * inv);
      if (jp == t && !past_end) { s_pt[wave] = p0; p0 = 0.f; }
      if (jp + 1 == t && !past_end) { s_pt[wave] = p1; p1 = 0.f; }
      *reinterpret_cast<uint32_t*>(&s_p[wave][jp]) = pack_bf16x2(p0, p1);
    }
  }
  // The wavefront's own LDS writes above are read back below in another lane
  // order; no other wavefront is involved, so ordering within the wavefront
  // is all that is needed.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // The tail block as matrix operand: lane (n16, g) of tile dt holds head dim
  // 16 dt + n16 of positions 8 g .. +8.
  Frag16 vt[4];
  const bool tail_used = !past_end && tl > 0;
  if (tail_used) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int e = 0; e < 8; ++e)
        vt[dt].h[e] = *reinterpret_cast<const bf16_t*>(
            &s_tail[wave][(8 * g + e) * kTailRow + (16 * dt + n16) * 2]);
  }

  f32x4_v acc[4];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    f32x4_v oc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) oc[dt] = (f32x4_v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      const int gb = c * 4 + jb;
      if (gb < pb || (gb == pb && tail_used)) {
        Frag16 pb16;
        pb16.u = *reinterpret_cast<const uint4*>(
            &s_p[wave][c * kBlockJ + 32 * jb + 8 * g]);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
          Frag16 v;
          v.u = gb < pb ? vb[c][jb][dt].u : vt[dt].u;
          oc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v.v, pb16.v, oc[dt],
                                                           0, 0, 0);
        }
      }
    }
    if (copy) {
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        if (c * 4 + jb < pb) {
          char* p = vdst + ((size_t)((c * 4 + jb) * kHeadDim + n16) * 32 + 8 * g) * 2;
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
            *reinterpret_cast<uint4*>(p + dt * 1024) = vb[c][jb][dt].u;
        }
      }
    }
    if (!past_end && t >= c * kBlockJ && t < (c + 1) * kBlockJ) {
      const float p_t = s_pt[wave];
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        oc[dt][0] = fmaf(p_t, bf16lo_to_f32(vn[dt].x), oc[dt][0]);
        oc[dt][1] = fmaf(p_t, bf16hi_to_f32(vn[dt].x), oc[dt][1]);
        oc[dt][2] = fmaf(p_t, bf16lo_to_f32(vn[dt].y), oc[dt][2]);
        oc[dt][3] = fmaf(p_t, bf16hi_to_f32(vn[dt].y), oc[dt][3]);
      }
    }
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      if (c == 0) acc[dt] = oc[dt];
      else acc[dt] += oc[dt];
    }
  }
  if (n16 == 0) {
    bf16_t* o = a.out + (size_t)r * HD + h * kHeadDim + 4 * g;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      uint2 pk;
      pk.x = pack_bf16x2(acc[dt][0], acc[dt][1]);
      pk.y = pack_bf16x2(acc[dt][2], acc[dt][3]);
      *reinterpret_cast<uint2*>(o + 16 * dt) = pk;
    }
  }
  // The step's column: the key as one line of its cache; the value as one
  // line of the tail, or, when it is its block's last, the finished block.
  // The key line must land after the copy of the old line above.
  if (!past_end) {
    if (copy) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    *reinterpret_cast<bf16_t*>(kdst + ((size_t)t * kHeadDim + lane) * 2) = knew_d;
    if (tl == 31) {
      char* p = vdst + ((size_t)(pb * kHeadDim + n16) * 32 + 8 * g) * 2;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
        *reinterpret_cast<uint4*>(p + dt * 1024) = vt[dt].u;
    } else {
      *reinterpret_cast<bf16_t*>(vdst + tail_at + tl * 128 + lane * 2) = vnew_d;
    }
  }
}

// ---- dispatch -------------------------------------------------------------------
template <int NQP>
static void launch_cross(const AttnMfmaArgs& a, int B, hipStream_t s) {
  const int waves = (a.S + kBlockJ - 1) / kBlockJ;
  dim3 grid(a.H, B), block(64 * waves);
  if (a.q == nullptr) {  // fused query projection: always 4 wavefronts
    block = dim3(256);
    const int nj = (a.d / 64 + 3) / 4;
    if (nj <= 3)
      hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 4, 3>), grid, block, 0, s,
                         a);
    else
      hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 4, 4>), grid, block, 0, s,
                         a);
    return;
  }
  // A launch whose keys and values outgrow what the memory-side cache could
  // hand back to the next step reads them as streaming data (measured at
  // 67 MB to 2.1 GB per launch: 2-6 % shorter launches, and the step's other
  // kernels find more of their rows and code still cached); at 33 MB per
  // launch (400 MB over the layers of T5.1.1-base) ordinary loads are faster.
  const bool once =
      (size_t)B * a.H * a.S * kHeadDim * 4 >= ((size_t)48 << 20);
  if (waves <= 4) {
    if (once)
      hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 4, 0, true>), grid, block, 0, s, a);
    else
      hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 4, 0>), grid, block, 0, s, a);
  } else if (waves <= 8) {
    if (once)
      hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 8, 0, true>), grid, block, 0, s, a);
    else
      hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 8, 0>), grid, block, 0, s, a);
  } else {
    if (once)
      hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 16, 0, true>), grid, block, 0, s, a);
    else
      hipLaunchKernelGGL((cross_attn_mfma_kernel<NQP, 16, 0>), grid, block, 0, s, a);
  }
}

int launch_cross_attention_bf16(hipStream_t s, const void* q, const void* k,
                                const void* v, const int32_t* enc_len,
                                void* out, int B, int beams, int H, int E,
                                const void* x, const void* ln, const void* wq,
                                int d, float eps, const int32_t* units) {
  AttnMfmaArgs a;
  a.v_blocked = 0;
  a.k_blocked = 0;
  a.units = units;
  a.x = (const bf16_t*)x; a.ln = (const bf16_t*)ln; a.wq = wq;
  a.d = d; a.eps = eps;
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
                               const int32_t* pending_dst, int beams,
                               int value_blocked) {
  AttnMfmaArgs a;
  a.v_blocked = value_blocked != 0;
  a.k_blocked = value_blocked == 2;
  a.q = (const bf16_t*)qkv; a.k = (bf16_t*)ck; a.v = (bf16_t*)cv;
  a.rel_bias = (const bf16_t*)rel_bias; a.index = cache_index;
  a.out = (bf16_t*)out;
  a.H = H; a.S = L; a.nq = 1; a.q_stride = 3 * H * kHeadDim;
  a.gate = tls_gate;
  a.x = nullptr; a.ln = nullptr; a.wq = nullptr; a.d = 0; a.eps = 0.f;
  a.units = nullptr;
  a.nblk = (L + kBlockJ - 1) / kBlockJ;
  a.n_units = R * H;
  if (value_blocked == 3) {
    // caches in the decode loop's own layout (checked by the caller: one
    // chunk for a gather in place, two at most otherwise)
    a.v_blocked = a.k_blocked = 1;
    a.pending = pending;
    a.pending_dst = pending ? pending_dst : nullptr;
    a.beams = pending ? beams : 1;
    if (pending != nullptr && pending_dst == nullptr) {
      dim3 grid(H, R / beams), block(64 * beams);
      if (beams <= 4)
        hipLaunchKernelGGL((self_attn_tail_kernel<1, 4, true>), grid, block, 0, s, a);
      else
        hipLaunchKernelGGL((self_attn_tail_kernel<1, 8, true>), grid, block, 0, s, a);
      return 0;
    }
    // independent (row, head) pairs: workgroups of 4, 2 or 1 of them,
    // whichever leaves the most loaded CU the fewest wavefronts
    int wm = 4, worst = 1 << 30;
    for (int cand = 4; cand >= 1; cand >>= 1) {
      const int groups = (a.n_units + cand - 1) / cand;
      const int load = (groups + kCUs - 1) / kCUs * cand;
      if (load < worst) { worst = load; wm = cand; }
    }
    dim3 grid((a.n_units + wm - 1) / wm), block(64 * wm);
#define T5D_LAUNCH_TAIL(NC_, WM_)                                              \
  hipLaunchKernelGGL((self_attn_tail_kernel<NC_, WM_, false>), grid, block, 0, \
                     s, a)
    if (a.nblk == 1) {
      if (wm == 4) T5D_LAUNCH_TAIL(1, 4);
      else if (wm == 2) T5D_LAUNCH_TAIL(1, 2);
      else T5D_LAUNCH_TAIL(1, 1);
    } else {
      if (wm == 4) T5D_LAUNCH_TAIL(2, 4);
      else if (wm == 2) T5D_LAUNCH_TAIL(2, 2);
      else T5D_LAUNCH_TAIL(2, 1);
    }
#undef T5D_LAUNCH_TAIL
    return 0;
  }
  a.pending = pending;
  a.pending_dst = pending ? pending_dst : nullptr;
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

}  // namespace t5d
