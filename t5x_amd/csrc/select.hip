// Selection kernels of the decode loops: exact top-k, fused
// log_softmax + prefix add + top-2K over beam x vocab, beam bookkeeping, the
// loop condition, and the sampling step (greedy / top-k / top-p + Gumbel).
//
// All orderings are total: candidates compare by (value descending, index
// ascending), which is lax.top_k's tie rule and jnp.argmax's first-occurrence
// rule, so results do not depend on how the work is split over lanes.
#include <math.h>

#include <mutex>

#include "common.h"

namespace t5d {

constexpr float kNegInf = -1.0e7f;  // t5x/decoding.py:33

struct Cand {
  float v;
  int i;
};

__device__ __forceinline__ bool better(float va, int ia, float vb, int ib) {
  return va > vb || (va == vb && ia < ib);
}

__device__ __forceinline__ Cand wave_best(Cand c) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    float v = __shfl_xor(c.v, o, 64);
    int i = __shfl_xor(c.i, o, 64);
    if (better(v, i, c.v, c.i)) { c.v = v; c.i = i; }
  }
  return c;
}

// Best candidate of a workgroup (blockDim.x a multiple of 64, <= 1024).
// `scratch` holds one Cand per wavefront.  Result is returned to all threads.
__device__ __forceinline__ Cand block_best(Cand c, Cand* scratch) {
  c = wave_best(c);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[wave] = c;
  __syncthreads();
  Cand r = scratch[0];
  for (int w = 1; w < nw; ++w) {
    Cand o = scratch[w];
    if (better(o.v, o.i, r.v, r.i)) r = o;
  }
  return r;
}

__device__ __forceinline__ double block_sum_f64(double v, double* scratch) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  double r = 0.0;
  for (int w = 0; w < nw; ++w) r += scratch[w];
  return r;
}

__device__ __forceinline__ float block_max_f32(float v, float* scratch) {
  v = wave_max(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
  for (int w = 1; w < nw; ++w) r = fmaxf(r, scratch[w]);
  return r;
}

__device__ __forceinline__ int block_sum_i32(int v, int* scratch) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  int r = 0;
  for (int w = 0; w < nw; ++w) r += scratch[w];
  return r;
}

// ---- generic exact top-k -----------------------------------------------------
// One workgroup per row; k rounds, each finds the best element strictly after
// the previously selected one in the total order.
__global__ void __launch_bounds__(256)
top_k_kernel(const float* __restrict__ x, float* __restrict__ vals,
             int32_t* __restrict__ idx, int n, int k) {
  __shared__ Cand scratch[4];
  const float* row = x + (size_t)blockIdx.x * n;
  float pv = INFINITY;
  int pi = -1;
  for (int r = 0; r < k; ++r) {
    Cand best = {-INFINITY, 0x7FFFFFFF};
    for (int j = threadIdx.x; j < n; j += 256) {
      const float v = row[j];
      const bool after = better(pv, pi, v, j);  // (pv,pi) ranks before (v,j)
      if (after && better(v, j, best.v, best.i)) { best.v = v; best.i = j; }
    }
    best = block_best(best, scratch);
    if (threadIdx.x == 0) {
      vals[(size_t)blockIdx.x * k + r] = best.v;
      idx[(size_t)blockIdx.x * k + r] = best.i;
    }
    pv = best.v;
    pi = best.i;
  }
}

// ---- log_softmax + prefix add + per-row top-k --------------------------------
// One workgroup per (batch, beam) row.  max and log-sum-exp first (the sum is
// carried in double so the result does not depend on the reduction shape),
// then every thread keeps the best KMAX of its strided share of
//   f(j) = ((x[j] - max) - lse) + live_logprob
// and the workgroup merges the lists by k rounds of arg-best.
template <int KMAX>
__global__ void __launch_bounds__(256)
beam_row_topk_kernel(const float* __restrict__ logits,
                     const float* __restrict__ live_logprobs,
                     float* __restrict__ row_max, float* __restrict__ row_lse,
                     float* __restrict__ cand_vals, int32_t* __restrict__ cand_idx,
                     int V, int beams, int k, const int32_t* gate) {
  __shared__ Cand scratch[4];
  __shared__ float fscratch[4];
  __shared__ double dscratch[4];
  T5D_GATED(gate);
  const int r = blockIdx.x;
  const float* x = logits + (size_t)r * V;
  float m = -INFINITY;
  for (int j = threadIdx.x; j < V; j += 256) m = fmaxf(m, x[j]);
  m = block_max_f32(m, fscratch);
  double sum = 0.0;
  for (int j = threadIdx.x; j < V; j += 256) sum += (double)expf(x[j] - m);
  sum = block_sum_f64(sum, dscratch);
  const float lse = (float)log(sum);
  const float lp = live_logprobs[r];
  if (threadIdx.x == 0) {
    row_max[r] = m;
    row_lse[r] = lse;
  }
  const int base = (r % beams) * V;

  float lv[KMAX];
  int li[KMAX];
#pragma unroll
  for (int q = 0; q < KMAX; ++q) { lv[q] = -INFINITY; li[q] = 0x7FFFFFFF; }
  for (int j = threadIdx.x; j < V; j += 256) {
    const float f = ((x[j] - m) - lse) + lp;
    const int fi = base + j;
    if (better(f, fi, lv[KMAX - 1], li[KMAX - 1])) {
      // insertion keeping the list sorted best-first
      float cv = f;
      int ci = fi;
#pragma unroll
      for (int q = 0; q < KMAX; ++q) {
        if (better(cv, ci, lv[q], li[q])) {
          const float tv = lv[q]; const int ti = li[q];
          lv[q] = cv; li[q] = ci;
          cv = tv; ci = ti;
        }
      }
    }
  }
  for (int out = 0; out < k; ++out) {
    Cand head = {lv[0], li[0]};
    Cand best = block_best(head, scratch);
    if (head.i == best.i && head.v == best.v && best.i != 0x7FFFFFFF) {
      // pop (indices are unique, so exactly one thread matches)
#pragma unroll
      for (int q = 0; q + 1 < KMAX; ++q) { lv[q] = lv[q + 1]; li[q] = li[q + 1]; }
      lv[KMAX - 1] = -INFINITY; li[KMAX - 1] = 0x7FFFFFFF;
    }
    if (threadIdx.x == 0) {
      cand_vals[(size_t)r * k + out] = best.v;
      cand_idx[(size_t)r * k + out] = best.i;
    }
  }
}

// Fast path of the same computation for 16-byte aligned rows of at most 32768
// elements with V % 4 == 0: 1024 threads per row, the row lives in registers
// (8 float4 per thread, all loads issued at once), so logits are read from
// memory exactly once.  Selection is by threshold: f is monotone in x, so with
// t = the k-th largest of the 16 wavefront maxima at least k elements have
// f >= f(t) and nothing below f(t) can be among the k best.  The few elements
// that pass (about 16 (H_16 - H_(16-k)) of an exchangeable row: 11 for k = 8)
// are appended to a list in LDS and ranked there by counting.  A row with more
// than kTopkCap elements at or above the threshold (long runs of equal values)
// takes the slow path instead: every thread keeps the best two of its 32
// elements, each wavefront extracts its k best by k rounds of a 64-lane
// arg-best (a lane that runs out of candidates rescans its registers for the
// next two below the last one it gave away), and wavefront 0 merges the 16
// sorted lists the same way.
constexpr int kTopkCap = 512;
constexpr int kFastTopkVec = 8;

// exp(x) for x <= 0 to about 1 ulp with the hardware exp2: the rounding error
// of x * log2(e) is recovered with an fma and folded back in as a first-order
// correction.  Anything below -1e30 (padding, -inf logits) gives exactly 0.
__device__ __forceinline__ float exp_nonpositive(float x) {
  const float kL2eHi = 1.44269502162933349609375f;    // float(log2(e))
  const float kL2eLo = 1.92596299112661746e-8f;       // log2(e) - kL2eHi
  const float hi = x * kL2eHi;
  const float lo = fmaf(x, kL2eHi, -hi) + x * kL2eLo;
  const float e = __builtin_amdgcn_exp2f(hi);
  const float r = fmaf(e, lo * 0.693147180559945309f, e);
  return x < -1.0e30f ? 0.f : r;
}

__device__ __forceinline__ void top2_insert(float f, int fi, float& v0, int& i0,
                                            float& v1, int& i1) {
  // selects only: a branchy form makes the compiler index the pair in memory
  const bool b0 = better(f, fi, v0, i0);
  const bool b1 = better(f, fi, v1, i1);
  v1 = b0 ? v0 : (b1 ? f : v1);
  i1 = b0 ? i0 : (b1 ? fi : i1);
  v0 = b0 ? f : v0;
  i0 = b0 ? fi : i0;
}

__global__ void __launch_bounds__(1024)
beam_row_topk_fast_kernel(const float* __restrict__ logits,
                          const float* __restrict__ live_logprobs,
                          float* __restrict__ row_max,
                          float* __restrict__ row_lse,
                          float* __restrict__ cand_vals,
                          int32_t* __restrict__ cand_idx, int V, int beams,
                          int k, const int32_t* gate) {
  __shared__ float s_f[16];
  __shared__ double s_d[16];
  __shared__ float s_cv[16][16];
  __shared__ int s_ci[16][16];
  __shared__ float s_lv[kTopkCap];
  __shared__ int s_li[kTopkCap];
  __shared__ int s_count;
  T5D_GATED(gate);
  constexpr int kNone = 0x7FFFFFFF;
  const int r = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const float4* x4 = reinterpret_cast<const float4*>(logits + (size_t)r * V);
  const int nvec = V >> 2;
  float4 x[kFastTopkVec];
#pragma unroll
  for (int u = 0; u < kFastTopkVec; ++u) {
    const int vi = u * 1024 + tid;
    x[u] = vi < nvec ? x4[vi]
                     : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  }
  const float lp = live_logprobs[r];

  float m = -INFINITY;
#pragma unroll
  for (int u = 0; u < kFastTopkVec; ++u)
    m = fmaxf(fmaxf(m, fmaxf(x[u].x, x[u].y)), fmaxf(x[u].z, x[u].w));
  m = wave_max(m);
  if (lane == 0) s_f[wave] = m;
  if (tid == 0) s_count = 0;
  __syncthreads();
  const float wmax = s_f[lane & 15];
  m = lanes16_max(wmax);
  // k-th largest wavefront maximum (k <= 16; ties ordered by wavefront)
  int wrank = 0;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const float o = s_f[j];
    wrank += (o > wmax || (o == wmax && j < (lane & 15))) ? 1 : 0;
  }
  const unsigned long long whit = __builtin_amdgcn_ballot_w64(wrank == k - 1);
  const float tx = __shfl(wmax, (int)__builtin_ctzll(whit | (1ull << 63)), 64);

  double sum = 0.0;
#pragma unroll
  for (int u = 0; u < kFastTopkVec; ++u) {
    // exp(-inf) == 0 for the padding
    sum += (double)exp_nonpositive(x[u].x - m);
    sum += (double)exp_nonpositive(x[u].y - m);
    sum += (double)exp_nonpositive(x[u].z - m);
    sum += (double)exp_nonpositive(x[u].w - m);
  }
  sum = wave_sum(sum);
  if (lane == 0) s_d[wave] = sum;
  __syncthreads();
  sum = lanes16_sum(s_d[lane & 15]);
  const float lse = (float)log(sum);
  if (tid == 0) {
    row_max[r] = m;
    row_lse[r] = lse;
  }

  // f(j) = ((x[j] - max) - lse) + live_logprob, in place; elements at or
  // above the threshold go to the list.
  const int base = (r % beams) * V;
  const float tf = ((tx - m) - lse) + lp;
#pragma unroll
  for (int u = 0; u < kFastTopkVec; ++u) {
    const int vi = u * 1024 + tid;
    const int j = base + 4 * vi;
    x[u].x = ((x[u].x - m) - lse) + lp;
    x[u].y = ((x[u].y - m) - lse) + lp;
    x[u].z = ((x[u].z - m) - lse) + lp;
    x[u].w = ((x[u].w - m) - lse) + lp;
    const float top = fmaxf(fmaxf(x[u].x, x[u].y), fmaxf(x[u].z, x[u].w));
    if (vi < nvec && top >= tf) {
      const float e[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (e[c] >= tf) {
          const int p = atomicAdd(&s_count, 1);
          if (p < kTopkCap) { s_lv[p] = e[c]; s_li[p] = j + c; }
        }
      }
    }
  }
  __syncthreads();
  const int ncand = s_count;
  if (ncand <= kTopkCap) {
    // rank by counting; indices are unique, so ranks are too
    if (tid < ncand) {
      const float v = s_lv[tid];
      const int i = s_li[tid];
      int rank = 0;
      for (int c = 0; c < ncand; ++c)
        rank += better(s_lv[c], s_li[c], v, i) ? 1 : 0;
      if (rank < k) {
        cand_vals[(size_t)r * k + rank] = v;
        cand_idx[(size_t)r * k + rank] = i;
      }
    } else if (tid < k) {  // fewer than k elements in the row
      cand_vals[(size_t)r * k + tid] = -INFINITY;
      cand_idx[(size_t)r * k + tid] = kNone;
    }
    return;
  }

  // Slow path.
  float v0 = -INFINITY, v1 = -INFINITY;
  int i0 = kNone, i1 = kNone;
#pragma unroll
  for (int u = 0; u < kFastTopkVec; ++u) {
    const int vi = u * 1024 + tid;
    const int j = base + 4 * vi;
    if (vi < nvec) {
      top2_insert(x[u].x, j, v0, i0, v1, i1);
      top2_insert(x[u].y, j + 1, v0, i0, v1, i1);
      top2_insert(x[u].z, j + 2, v0, i0, v1, i1);
      top2_insert(x[u].w, j + 3, v0, i0, v1, i1);
    }
  }

  // k rounds per wavefront.  `have` counts the valid entries of (v0, v1);
  // (lv, li) is the last candidate this lane gave away.
  int have = 2;
  float lv = INFINITY;
  int li = -1;
  for (int out = 0; out < k; ++out) {
    if (__builtin_amdgcn_ballot_w64(have == 0) != 0) {
      if (have == 0) {  // rescan: best two strictly after (lv, li)
        v0 = v1 = -INFINITY;
        i0 = i1 = kNone;
#pragma unroll
        for (int u = 0; u < kFastTopkVec; ++u) {
          const int vi = u * 1024 + tid;
          const int j = base + 4 * vi;
          if (vi < nvec) {
            if (better(lv, li, x[u].x, j))
              top2_insert(x[u].x, j, v0, i0, v1, i1);
            if (better(lv, li, x[u].y, j + 1))
              top2_insert(x[u].y, j + 1, v0, i0, v1, i1);
            if (better(lv, li, x[u].z, j + 2))
              top2_insert(x[u].z, j + 2, v0, i0, v1, i1);
            if (better(lv, li, x[u].w, j + 3))
              top2_insert(x[u].w, j + 3, v0, i0, v1, i1);
          }
        }
        have = 2;  // entries may be (-inf, none): they lose every comparison
      }
    }
    Cand head = {v0, i0};
    Cand best = wave_best(head);
    if (head.i == best.i && best.i != kNone) {  // indices are unique
      lv = v0; li = i0;
      v0 = v1; i0 = i1;
      v1 = -INFINITY; i1 = kNone;
      --have;
    }
    if (lane == 0) {
      s_cv[wave][out] = best.v;
      s_ci[wave][out] = best.i;
    }
  }
  __syncthreads();
  if (wave != 0) return;
  // Merge the 16 best-first lists: lane w < 16 walks list w.
  int pos = 0;
  for (int out = 0; out < k; ++out) {
    Cand head = {-INFINITY, kNone};
    if (lane < 16 && pos < k) {
      head.v = s_cv[lane][pos];
      head.i = s_ci[lane][pos];
    }
    Cand best = head;
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) {
      float v = __shfl_xor(best.v, o, 64);
      int i = __shfl_xor(best.i, o, 64);
      if (better(v, i, best.v, best.i)) { best.v = v; best.i = i; }
    }
    if (lane < 16 && head.i == best.i && best.i != kNone) ++pos;
    if (lane == 0) {
      cand_vals[(size_t)r * k + out] = best.v;
      cand_idx[(size_t)r * k + out] = best.i;
    }
  }
}

// Merge the beams' per-row candidates of one batch item: one candidate per
// thread (beams*k <= 128), rank by counting better candidates.
__global__ void __launch_bounds__(128)
beam_merge_kernel(const float* __restrict__ cand_vals,
                  const int32_t* __restrict__ cand_idx,
                  float* __restrict__ topk_vals, int32_t* __restrict__ topk_idx,
                  int beams, int k, const int32_t* gate) {
  __shared__ float sv[128];
  __shared__ int si[128];
  T5D_GATED(gate);
  const int b = blockIdx.x, tid = threadIdx.x;
  const int n = beams * k;
  float v = -INFINITY;
  int i = 0x7FFFFFFF;
  if (tid < n) {
    v = cand_vals[(size_t)b * n + tid];
    i = cand_idx[(size_t)b * n + tid];
  }
  sv[tid] = v;
  si[tid] = i;
  __syncthreads();
  if (tid >= n) return;
  int rank = 0;
  for (int o = 0; o < n; ++o)
    if (better(sv[o], si[o], v, i)) ++rank;
  if (rank < k) {
    topk_vals[(size_t)b * k + rank] = v;
    topk_idx[(size_t)b * k + rank] = i;
  }
}

// ---- beam bookkeeping -------------------------------------------------------
constexpr int kMaxBeams = 8;

struct BeamUpdateArgs {
  t5d_beam_state cur, next;
  const float* topk_vals;
  const int32_t* topk_idx;
  const int32_t* inputs;
  const int32_t* initial_index;
  const float* brevity;
  int32_t* top_alive_indices;
  int B, K, S, Lin, V, eos_id;
  const int32_t* gate;
  // optional merge of per-row candidates [B, K, 2K] first (then topk_vals /
  // topk_idx above are not read; the merged top 2K goes to *_out)
  const float* cand_vals;
  const int32_t* cand_idx;
  float* topk_vals_out;
  int32_t* topk_idx_out;
  // optional bookkeeping of where each beam's cache rows live (all [B, K]):
  // cache_slot[b, e] is the slot of beam e (in: before, out: after this
  // iteration); cache_src / cache_dst (out) tell the next reader of the cache
  // where new beam e finds its parent's rows and where its own go.
  int32_t* cache_slot;
  int32_t* cache_src;
  int32_t* cache_dst;
};

// Slots for the K new beams of one item, given their parents' slots rd[0..K):
// the first child of a parent (lowest e) inherits the parent's slot, so a
// mere re-ranking of the beams moves no cache row at all; every further child
// takes the n-th slot that no new beam reads (n counted over such children in
// order of e), which it must fill with a copy.  The result is a permutation
// of 0..K-1 and no slot that is written is also read.
__device__ __forceinline__ int new_beam_slot(const int (&rd)[kMaxBeams], int K,
                                             int e) {
  unsigned seen = 0, all = 0;
  int later = 0;  // children before e that also need a free slot
#pragma unroll
  for (int o = 0; o < kMaxBeams; ++o) {
    if (o < K) {
      const unsigned bit = 1u << rd[o];
      if (o < e) {
        later += (seen & bit) ? 1 : 0;
        seen |= bit;
      }
      all |= bit;
    }
  }
  int mine = 0;
#pragma unroll
  for (int o = 0; o < kMaxBeams; ++o) mine = o == e ? rd[o] : mine;
  if (!(seen & (1u << mine))) return mine;
  int found = mine;  // K reads of fewer than K slots always leave one free
#pragma unroll
  for (int slot = kMaxBeams - 1; slot >= 0; --slot) {
    if (slot < K && !(all & (1u << slot))) {
      // free slots below `slot`: this is the later-th free slot if that count
      // equals `later`
      const unsigned below = ~all & ((1u << slot) - 1u);
      if (__popc(below) == later) found = slot;
    }
  }
  return found;
}

// Stable descending order of n values (ties keep index order).
__device__ __forceinline__ void stable_order_desc(const float* v, int n,
                                                  int* order) {
  for (int a = 0; a < n; ++a) {
    int rank = 0;
    for (int c = 0; c < n; ++c)
      if (better(v[c], c, v[a], a)) ++rank;
    order[rank] = a;
  }
}

// One workgroup per batch item.  Optionally first merges the
// beams' per-row candidates (cand_* != null) into the item's top 2K.  The
// order-sensitive bookkeeping is done in parallel, one candidate / pool entry
// per lane, ranks by counting under the total order (value descending, index
// ascending), which is what the reference's stable sorts produce.  Then every
// thread owns sequence COLUMNS: for a column it reads the item's K live and K
// finished entries into registers before writing any, so `cur` and `next`
// may be the same buffers.  Everything that does not depend on another load
// (candidates, the finished pool, the first column of every thread) is
// requested before the first wait, so the chain of cold misses is two deep
// (cur_index, then the forced token and the brevity penalty).
constexpr int kUpdateThreads = 256;
__global__ void __launch_bounds__(kUpdateThreads)
beam_update_kernel(BeamUpdateArgs a) {
  __shared__ int s_src_live[kMaxBeams];       // source live beam of new live e
  __shared__ int s_slot_of[kMaxBeams];        // cache slot of old beam e
  __shared__ int s_tok_live[kMaxBeams];
  __shared__ int s_fin_from[kMaxBeams];       // <K: old finished; else K+cand
  __shared__ int s_cand_beam[2 * kMaxBeams];
  __shared__ int s_cand_tok[2 * kMaxBeams];
  __shared__ float s_live_lp[kMaxBeams];
  __shared__ float s_fin_score[kMaxBeams];
  __shared__ int s_fin_flag[kMaxBeams];
  __shared__ float s_mv[128];                 // candidates being merged
  __shared__ int s_mi[128];
  __shared__ float s_top_v[2 * kMaxBeams];    // the item's top 2K
  __shared__ int s_top_i[2 * kMaxBeams];
  __shared__ float s_new_lp[2 * kMaxBeams], s_lp[2 * kMaxBeams];
  __shared__ int s_fin[2 * kMaxBeams];
  __shared__ float s_pool[3 * kMaxBeams];
  T5D_GATED(a.gate);
  const int b = blockIdx.x, lane = threadIdx.x;
  const int K = a.K, K2 = 2 * a.K, S = a.S;
  const size_t base = (size_t)b * K * S;
  int live[kMaxBeams], fin[kMaxBeams];
#pragma unroll
  for (int e = 0; e < kMaxBeams; ++e) {
    if (e < K && lane < S) {
      live[e] = a.cur.live_seqs[base + (size_t)e * S + lane];
      fin[e] = a.cur.finished_seqs[base + (size_t)e * S + lane];
    }
  }
  float old_score = 0.f;
  int old_flag = 0;
  int old_slot = 0;
  if (lane < K) {
    old_score = a.cur.finished_scores[(size_t)b * K + lane];
    old_flag = a.cur.finished_flags[(size_t)b * K + lane];
    if (a.cache_slot) old_slot = a.cache_slot[(size_t)b * K + lane];
  }
  const int first = a.initial_index[b];
  const int cur = *a.cur.cur_index;

  if (a.cand_vals != nullptr) {
    // top 2K of the K rows' 2K candidates each
    const int n = K * K2;
    if (lane < n) {
      s_mv[lane] = a.cand_vals[(size_t)b * n + lane];
      s_mi[lane] = a.cand_idx[(size_t)b * n + lane];
    }
    __syncthreads();
    if (lane < n) {
      const int c = lane;
      const float v = s_mv[c];
      const int i = s_mi[c];
      int rank = 0;
      for (int o = 0; o < n; ++o)
        if (better(s_mv[o], s_mi[o], v, i)) ++rank;
      if (rank < K2) {
        s_top_v[rank] = v;
        s_top_i[rank] = i;
        a.topk_vals_out[(size_t)b * K2 + rank] = v;
        a.topk_idx_out[(size_t)b * K2 + rank] = i;
      }
    }
  } else if (lane < K2) {
    s_top_v[lane] = a.topk_vals[(size_t)b * K2 + lane];
    s_top_i[lane] = a.topk_idx[(size_t)b * K2 + lane];
  }
  __syncthreads();

  const int col = min(cur + 1, a.Lin - 1);
  const int nxt = a.inputs[(size_t)b * a.Lin + col];
  const bool oop = nxt == 0;
  if (lane < K2) {
    const int c = lane;
    const float raw = s_top_v[c];
    const int fi = s_top_i[c];
    const int beam = fi / a.V;
    const int id = oop ? fi % a.V : nxt;
    const float lp = oop ? raw : (c == 0 ? 0.f : kNegInf);
    const bool fin = id == a.eos_id;
    s_cand_beam[c] = beam;
    s_cand_tok[c] = id;
    s_lp[c] = lp;
    s_fin[c] = fin;
    s_new_lp[c] = lp + (fin ? kNegInf : 0.f);
  }
  const int len = first + cur + 1;
  const float bp = a.brevity[len];
  __syncthreads();
  // finished pool: K old + 2K new, brevity-penalised
  if (lane < 3 * K) {
    s_pool[lane] = lane < K
        ? old_score
        : s_lp[lane - K] / bp + (s_fin[lane - K] ? 0.f : kNegInf);
  }
  __syncthreads();
  // live beams: top K of the 2K, ascending (lax.top_k then flip)
  if (lane < K2) {
    const float v = s_new_lp[lane];
    int rank = 0;
    for (int o = 0; o < K2; ++o)
      if (better(s_new_lp[o], o, v, lane)) ++rank;
    if (rank < K) {
      const int e = K - 1 - rank;
      s_live_lp[e] = v;
      s_src_live[e] = s_cand_beam[lane];
      s_tok_live[e] = s_cand_tok[lane];
    }
  }
  if (lane < 3 * K) {
    const float v = s_pool[lane];
    int rank = 0;
    for (int o = 0; o < 3 * K; ++o)
      if (better(s_pool[o], o, v, lane)) ++rank;
    if (rank < K) {
      const int e = K - 1 - rank;
      s_fin_from[e] = lane;
      s_fin_score[e] = v;
      s_fin_flag[e] = lane < K ? old_flag : s_fin[lane - K];
    }
  }
  __syncthreads();
  if (lane < K) {
    const int e = lane;
    a.next.live_logprobs[(size_t)b * K + e] = s_live_lp[e];
    a.top_alive_indices[(size_t)b * K + e] = s_src_live[e];
    a.next.finished_scores[(size_t)b * K + e] = s_fin_score[e];
    a.next.finished_flags[(size_t)b * K + e] = (uint8_t)s_fin_flag[e];
    s_slot_of[e] = old_slot < 0 ? 0 : (old_slot >= K ? K - 1 : old_slot);
  }
  __syncthreads();
  // (the last wavefront does this: it has the fewest sequence columns below)
  const int slot_lane = lane - (kUpdateThreads - 64);
  if (a.cache_slot && slot_lane >= 0 && slot_lane < K) {
    const int e = slot_lane;
    int rd[kMaxBeams];
#pragma unroll
    for (int o = 0; o < kMaxBeams; ++o)
      rd[o] = o < K ? s_slot_of[s_src_live[o]] : 0;
    const int dst = new_beam_slot(rd, K, e);
    a.cache_src[(size_t)b * K + e] = s_slot_of[s_src_live[e]];
    a.cache_dst[(size_t)b * K + e] = dst;
    a.cache_slot[(size_t)b * K + e] = dst;
  }

  for (int j = lane; j < S; j += kUpdateThreads) {
    if (j != lane) {
#pragma unroll
      for (int e = 0; e < kMaxBeams; ++e) {
        if (e < K) {
          live[e] = a.cur.live_seqs[base + (size_t)e * S + j];
          fin[e] = a.cur.finished_seqs[base + (size_t)e * S + j];
        }
      }
    }
    const bool tokcol = j == cur + 1;
#pragma unroll
    for (int e = 0; e < kMaxBeams; ++e) {
      if (e < K) {
        int lv = live[0], fv;
#pragma unroll
        for (int q = 1; q < kMaxBeams; ++q)
          lv = (s_src_live[e] == q) ? live[q] : lv;
        const int from = s_fin_from[e];
        if (from < K) {
          fv = fin[0];
#pragma unroll
          for (int q = 1; q < kMaxBeams; ++q) fv = (from == q) ? fin[q] : fv;
        } else {
          const int cb = s_cand_beam[from - K];
          fv = live[0];
#pragma unroll
          for (int q = 1; q < kMaxBeams; ++q) fv = (cb == q) ? live[q] : fv;
          if (tokcol) fv = s_cand_tok[from - K];
        }
        a.next.live_seqs[base + (size_t)e * S + j] =
            tokcol ? s_tok_live[e] : lv;
        a.next.finished_seqs[base + (size_t)e * S + j] = fv;
      }
    }
  }
  // cur_index is read by every workgroup at entry; a separate 1-thread kernel
  // advances it after this one.
}

__global__ void advance_index_kernel(const int32_t* cur, int32_t* next,
                                     const int32_t* gate) {
  T5D_GATED(gate);
  *next = *cur + 1;
}

// ids[r] = live_seqs[r, cur_index] (t5x/decoding.py:1308-1312).
__global__ void gather_ids_kernel(const int32_t* __restrict__ live_seqs,
                                  const int32_t* __restrict__ cur_index,
                                  int32_t* __restrict__ ids, int R, int S,
                                  const int32_t* gate) {
  T5D_GATED(gate);
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r < R) ids[r] = live_seqs[(size_t)r * S + *cur_index];
}

__global__ void __launch_bounds__(256)
beam_cond_kernel(t5d_beam_state st, int B, int K, int S, float min_brevity,
                 float min_log_prob, int max_decode_step, int min_initial_index,
                 int32_t* keep_going, const int32_t* gate, int advance,
                 int do_cond, int32_t* counters, int n_counters) {
  __shared__ int iscratch[4];
  T5D_GATED(gate);
  // advance: this launch also ends the iteration (cur_index and the layers'
  // cache indices move on before the condition looks at them).
  const int cur = *st.cur_index + (advance ? 1 : 0);
  if (advance) {
    __syncthreads();  // every thread has read the old value
    if (threadIdx.x == 0) *st.cur_index = cur;
    if ((int)threadIdx.x < n_counters) counters[threadIdx.x] += 1;
  }
  if (!do_cond) return;
  const float raw_min = min_log_prob / min_brevity;
  int not_terminated = 0, passes_min = 0;
  for (int b = threadIdx.x; b < B; b += 256) {
    const float best_live = st.live_logprobs[(size_t)b * K + K - 1] / min_brevity;
    float worst = INFINITY;
    for (int e = 0; e < K; ++e)
      worst = fminf(worst, st.finished_scores[(size_t)b * K + e]);
    bool term = true;
    for (int e = 0; e < K; ++e) {
      const float w = st.finished_flags[(size_t)b * K + e] ? worst : kNegInf;
      term = term && (w > best_live);
    }
    if (!term) ++not_terminated;
    if (!(best_live < raw_min)) ++passes_min;
  }
  not_terminated = block_sum_i32(not_terminated, iscratch);
  passes_min = block_sum_i32(passes_min, iscratch);
  if (threadIdx.x == 0) {
    const bool not_at_end = (cur + min_initial_index) < S - 1;
    const bool exceed = (max_decode_step > 0) && (cur >= max_decode_step);
    const bool search_terminated = not_terminated == 0;
    const bool none_pass = (passes_min == 0) && (cur > 0);
    *keep_going = (not_at_end && !search_terminated && !none_pass && !exceed) ? 1 : 0;
  }
}

// ---- sampling -----------------------------------------------------------------
__device__ __forceinline__ uint32_t order_key(float f) {
  // Monotone map float -> uint32 (t5x/binary_search.py:74-101 does the same
  // through int32).
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_to_float(uint32_t k) {
  const uint32_t u = (k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k;
  return __uint_as_float(u);
}

struct SampleArgs {
  const float* logits;
  const float* gumbel;       // [noise_ring, R, V]; slot *noise_step % noise_ring
  const float* temperature;
  int32_t* tokens;
  float* logprobs;
  int V, topk, rescale;
  float topp;
  const int32_t* noise_step; // null: slot 0
  int noise_ring, R;
  const int32_t* gate;
  // optional: the rows' top-k candidates found by sample_topk_parts_kernel
  // (sample_parts_* below), or null
  int32_t* parts;
};

// One workgroup per row.
__global__ void __launch_bounds__(256)
sample_tokens_kernel(SampleArgs a) {
  __shared__ Cand cscratch[4];
  __shared__ float fscratch[4];
  __shared__ double dscratch[4];
  __shared__ int iscratch[4];
  __shared__ unsigned hist[256];
  T5D_GATED(a.gate);
  const int r = blockIdx.x;
  const int V = a.V;
  const float* x = a.logits + (size_t)r * V;
  const float T = a.temperature[r];
  const int slot = a.noise_step ? *a.noise_step % a.noise_ring : 0;
  const float* noise = a.gumbel + ((size_t)slot * a.R + r) * V;
  const float kMinT = 1e-4f;

  if (!(T > kMinT)) {  // greedy (t5x/decoding.py:575-592)
    Cand best = {-INFINITY, 0x7FFFFFFF};
    for (int j = threadIdx.x; j < V; j += 256)
      if (better(x[j], j, best.v, best.i)) { best.v = x[j]; best.i = j; }
    best = block_best(best, cscratch);
    float lp = 0.f;
    if (!a.rescale) {
      double sum = 0.0;
      for (int j = threadIdx.x; j < V; j += 256) sum += (double)expf(x[j] - best.v);
      sum = block_sum_f64(sum, dscratch);
      lp = (best.v - best.v) - (float)log(sum);
    }
    if (threadIdx.x == 0) { a.tokens[r] = best.i; a.logprobs[r] = lp; }
    return;
  }

  const float Tm = fmaxf(T, kMinT);
  float cutoff = -INFINITY;  // keep scaled >= cutoff

  if (a.topk > 0 && a.topk < V) {
    // k-th largest of scaled logits by radix select on the order-preserving
    // key, most significant byte first.
    uint32_t prefix = 0, mask = 0;
    int want = a.topk;  // rank (1-based, from the top) within the current set
    for (int shift = 24; shift >= 0; shift -= 8) {
      hist[threadIdx.x] = 0;
      __syncthreads();
      for (int j = threadIdx.x; j < V; j += 256) {
        const uint32_t key = order_key(x[j] / Tm);
        if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 0xFF], 1u);
      }
      __syncthreads();
      if (threadIdx.x == 0) {
        int digit = 255, acc = 0;
        for (; digit > 0; --digit) {
          if (acc + (int)hist[digit] >= want) break;
          acc += hist[digit];
        }
        iscratch[0] = digit;
        iscratch[1] = want - acc;
      }
      __syncthreads();
      prefix |= ((uint32_t)iscratch[0]) << shift;
      mask |= 0xFFu << shift;
      want = iscratch[1];
      __syncthreads();
    }
    cutoff = key_to_float(prefix);
  }

  float pcut = -INFINITY;  // top-p: keep prob >= pcut
  float smax = 0.f, ssum = 1.f;
  if (a.topp > 0.f) {
    // t5x/binary_search.py:230-299 — largest threshold whose kept mass >= p,
    // found by the same 32-step search over float bit patterns.
    float m = -INFINITY;
    for (int j = threadIdx.x; j < V; j += 256) {
      float y = x[j] / Tm;
      y = (y >= cutoff) ? y : kNegInf;
      m = fmaxf(m, y);
    }
    m = block_max_f32(m, fscratch);
    double sum = 0.0;
    for (int j = threadIdx.x; j < V; j += 256) {
      float y = x[j] / Tm;
      y = (y >= cutoff) ? y : kNegInf;
      sum += (double)expf(y - m);
    }
    sum = block_sum_f64(sum, dscratch);
    smax = m;
    ssum = (float)sum;
    int32_t bits = 0;
    for (int it = 0; it < 32; ++it) {
      int32_t mid = it == 0 ? bits : (bits | (int32_t)(1u << (31 - it)));
      int32_t pat = mid ^ (mid < 0 ? 0x7FFFFFFF : 0);
      const bool finite = (pat & 0x7F800000) != 0x7F800000;
      bool pred;
      if (finite) {
        const float thr = __int_as_float(pat);
        double mass = 0.0;
        for (int j = threadIdx.x; j < V; j += 256) {
          float y = x[j] / Tm;
          y = (y >= cutoff) ? y : kNegInf;
          const float pr = expf(y - smax) / ssum;
          if (pr >= thr) mass += (double)pr;
        }
        mass = block_sum_f64(mass, dscratch);
        pred = (float)mass < a.topp;
      } else {
        pred = pat >= 0;
      }
      if (it == 0) {
        if (pred) bits |= (int32_t)0x80000000u;
      } else if (!pred) {
        bits |= (int32_t)(1u << (31 - it));
      }
    }
    const int32_t pat = bits ^ (bits < 0 ? 0x7FFFFFFF : 0);
    pcut = __int_as_float(pat);
  }

  // argmax(masked + gumbel), and log-softmax statistics of the masked row.
  Cand best = {-INFINITY, 0x7FFFFFFF};
  float m = -INFINITY;
  for (int j = threadIdx.x; j < V; j += 256) {
    float y = x[j] / Tm;
    y = (y >= cutoff) ? y : kNegInf;
    if (a.topp > 0.f) {
      const float pr = expf(y - smax) / ssum;
      y = (pr >= pcut) ? y : kNegInf;
    }
    const float z = y + noise[j];
    if (better(z, j, best.v, best.i)) { best.v = z; best.i = j; }
    m = fmaxf(m, a.rescale ? y : x[j]);
  }
  best = block_best(best, cscratch);
  m = block_max_f32(m, fscratch);
  double sum = 0.0;
  float ytok = 0.f;
  for (int j = threadIdx.x; j < V; j += 256) {
    float y = x[j] / Tm;
    y = (y >= cutoff) ? y : kNegInf;
    if (a.topp > 0.f) {
      const float pr = expf(y - smax) / ssum;
      y = (pr >= pcut) ? y : kNegInf;
    }
    const float w = a.rescale ? y : x[j];
    sum += (double)expf(w - m);
    if (j == best.i) ytok = w;
  }
  sum = block_sum_f64(sum, dscratch);
  // ytok lives in exactly one thread; broadcast through the float scratch.
  __syncthreads();
  if ((best.i & 255) == (int)threadIdx.x) fscratch[0] = ytok;
  __syncthreads();
  ytok = fscratch[0];
  if (threadIdx.x == 0) {
    a.tokens[r] = best.i;
    a.logprobs[r] = (ytok - m) - (float)log(sum);
  }
}

// Fast path of sample_tokens_kernel for 16-byte aligned rows of at most 32768
// elements with V % 4 == 0: 1024 threads per row, the scaled row lives in
// registers (8 float4 per thread), so logits and noise are read once.
// The top-k cutoff (the k-th largest scaled logit, ties kept) is found by
// threshold: with m = ceil(k / 16), the smallest over the 16 wavefronts of the
// m-th largest per-thread maximum of a wavefront is a bound that at least k
// elements reach; the few elements at or above it go to a list in LDS, where
// the k-th largest is read off by counting.  More than kTopkCap such elements
// (long runs of equal values) fall back to the radix select, on registers.
__device__ __forceinline__ float kth_largest_by_radix(const float4 (&y)[8],
                                                      int nvec, int tid, int k,
                                                      unsigned* hist,
                                                      int* iscratch) {
  uint32_t prefix = 0, mask = 0;
  int want = k;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (u * 1024 + tid < nvec) {
        const float e[4] = {y[u].x, y[u].y, y[u].z, y[u].w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint32_t key = order_key(e[c]);
          if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 0xFF], 1u);
        }
      }
    }
    __syncthreads();
    if (tid == 0) {
      int digit = 255, acc = 0;
      for (; digit > 0; --digit) {
        if (acc + (int)hist[digit] >= want) break;
        acc += hist[digit];
      }
      iscratch[0] = digit;
      iscratch[1] = want - acc;
    }
    __syncthreads();
    prefix |= ((uint32_t)iscratch[0]) << shift;
    mask |= 0xFFu << shift;
    want = iscratch[1];
    __syncthreads();
  }
  return key_to_float(prefix);
}

// ---- top-k sampling in two launches ------------------------------------------------
// A row per workgroup leaves three quarters of the device idle at 64 rows, and
// the workgroup spends its time in a dozen block-wide exchanges.  With a
// top-k mask only the k largest scaled logits (and their ties) can be chosen
// or enter the log-softmax — everything else is -1e7, whose exponential is
// exactly 0 next to them — so the row is first cut into kSampleParts parts,
// one small workgroup each (every CU gets some), which emit their own k
// largest, ties at the k-th included; the row's k largest are among those
// 4 k.  The row's workgroup then works on that list alone: the k-th largest
// overall, Gumbel noise gathered for the kept candidates only (the noise
// tensor is not read otherwise), argmax, log-softmax.  A part whose list
// overflows (long runs of equal values), a greedy row, logits so low that
// -1e7 is not far below them: the row is marked and its workgroup runs
// the one-launch algorithm on the whole row.
// Workspace (int32 words): counts [R][kSampleParts] (-1: marked), then values
// [R][kSampleParts][kSamplePartCap] (float bits), then indices of the same
// shape.
constexpr int kSampleParts = 4;
constexpr int kSamplePartCap = 64;   // candidates a part may emit
constexpr int kSamplePartList = 256; // elements at or above a part's bound
__host__ __device__ inline size_t sample_parts_words(int R) {
  return (size_t)R * kSampleParts * (1 + 2 * kSamplePartCap);
}
__device__ __forceinline__ int32_t* sample_parts_count(int32_t* ws, int r, int p) {
  return ws + (size_t)r * kSampleParts + p;
}
__device__ __forceinline__ int32_t* sample_parts_vals(int32_t* ws, int R, int r, int p) {
  return ws + (size_t)R * kSampleParts +
         ((size_t)r * kSampleParts + p) * kSamplePartCap;
}
__device__ __forceinline__ int32_t* sample_parts_idx(int32_t* ws, int R, int r, int p) {
  return ws + (size_t)R * kSampleParts * (1 + kSamplePartCap) +
         ((size_t)r * kSampleParts + p) * kSamplePartCap;
}

__global__ void __launch_bounds__(256)
sample_topk_parts_kernel(SampleArgs a) {
  __shared__ float s_wm[4];
  __shared__ float s_lv[kSamplePartList];
  __shared__ int s_li[kSamplePartList];
  __shared__ int s_count, s_out;
  __shared__ float s_cut;
  T5D_GATED(a.gate);
  const int p = blockIdx.x, r = blockIdx.y, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int V = a.V, nvec = V >> 2;
  const int chunk = (nvec + kSampleParts - 1) / kSampleParts;  // <= 2048
  const int v0 = p * chunk, v1 = min(nvec, v0 + chunk);
  const float4 kPad = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  const float4* x4 = reinterpret_cast<const float4*>(a.logits + (size_t)r * V);
  float4 y[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int vi = v0 + u * 256 + tid;
    y[u] = vi < v1 ? x4[vi] : kPad;
  }
  const float T = a.temperature[r];
  const float kMinT = 1e-4f;
  if (tid == 0) { s_count = 0; s_out = 0; }
  int32_t* count = sample_parts_count(a.parts, r, p);
  if (!(T > kMinT)) {  // greedy rows take the one-launch path
    if (tid == 0) *count = -1;
    return;
  }
  const float Tm = fmaxf(T, kMinT);
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    y[u].x /= Tm; y[u].y /= Tm; y[u].z /= Tm; y[u].w /= Tm;
  }
  // bound: the smallest over the 4 wavefronts of a wavefront's m-th largest
  // per-thread maximum, m = ceil(k / 4): at least k elements reach it
  const int m = (a.topk + 3) >> 2;
  float tmax = -INFINITY;
#pragma unroll
  for (int u = 0; u < 8; ++u)
    tmax = fmaxf(fmaxf(tmax, fmaxf(y[u].x, y[u].y)), fmaxf(y[u].z, y[u].w));
  float rest = tmax, wm = -INFINITY;
  for (int it = 0; it < m; ++it) {
    wm = wave_max(rest);
    const unsigned long long hit = __builtin_amdgcn_ballot_w64(rest == wm);
    if (lane == (int)__builtin_ctzll(hit | (1ull << 63))) rest = -INFINITY;
  }
  if (lane == 0) s_wm[wave] = wm;
  __syncthreads();
  const float bound = fminf(fminf(s_wm[0], s_wm[1]), fminf(s_wm[2], s_wm[3]));
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const float top = fmaxf(fmaxf(y[u].x, y[u].y), fmaxf(y[u].z, y[u].w));
    if (top >= bound) {  // (-inf pads never reach a finite bound)
      const float e[4] = {y[u].x, y[u].y, y[u].z, y[u].w};
      const int j = 4 * (v0 + u * 256 + tid);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (e[c] >= bound) {
          const int q = atomicAdd(&s_count, 1);
          if (q < kSamplePartList) { s_lv[q] = e[c]; s_li[q] = j + c; }
        }
      }
    }
  }
  __syncthreads();
  const int ncand = s_count;
  // fewer than k (a -inf bound: rows of -inf) or more than the list holds
  bool ok = ncand >= a.topk && ncand <= kSamplePartList && bound > -INFINITY;
  if (ok) {
    if (tid < ncand) {
      const float v = s_lv[tid];
      int gt = 0, ge = 0;
      for (int c = 0; c < ncand; ++c) {
        const float o = s_lv[c];
        gt += o > v ? 1 : 0;
        ge += o >= v ? 1 : 0;
      }
      if (gt < a.topk && a.topk <= ge) s_cut = v;  // equal candidates: same bits
    }
    __syncthreads();
    const float cut = s_cut;
    float* vals = reinterpret_cast<float*>(sample_parts_vals(a.parts, a.R, r, p));
    int32_t* idx = sample_parts_idx(a.parts, a.R, r, p);
    if (tid < ncand && s_lv[tid] >= cut) {
      const int q = atomicAdd(&s_out, 1);
      if (q < kSamplePartCap) { vals[q] = s_lv[tid]; idx[q] = s_li[tid]; }
    }
    __syncthreads();
    ok = s_out <= kSamplePartCap;
  }
  if (tid == 0) *count = ok ? s_out : -1;
}

__global__ void __launch_bounds__(1024)
sample_tokens_fast_kernel(SampleArgs a) {
  __shared__ Cand cscratch[16];
  __shared__ float fscratch[16];
  __shared__ double dscratch[16];
  __shared__ int iscratch[4];
  __shared__ unsigned hist[256];
  __shared__ float s_lv[kTopkCap];
  __shared__ int s_count;
  __shared__ float s_cut;
  T5D_GATED(a.gate);
  const int r = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int V = a.V, nvec = V >> 2;
  if (a.parts != nullptr) {
    // The row's candidates from sample_topk_parts_kernel: at most
    // kSampleParts * kSamplePartCap = 256 of them, one per thread.
    int n[kSampleParts], total = 0;
    bool usable = true;
#pragma unroll
    for (int p = 0; p < kSampleParts; ++p) {
      n[p] = *sample_parts_count(a.parts, r, p);
      usable = usable && n[p] >= 0;
      total += n[p];
    }
    if (usable) {
      float v = -INFINITY;
      int j = 0x7FFFFFFF;
      int base = 0;
#pragma unroll
      for (int p = 0; p < kSampleParts; ++p) {
        if (tid >= base && tid < base + n[p]) {
          v = reinterpret_cast<const float*>(
              sample_parts_vals(a.parts, a.R, r, p))[tid - base];
          j = sample_parts_idx(a.parts, a.R, r, p)[tid - base];
        }
        base += n[p];
      }
      if (tid < total) s_lv[tid] = v;
      __syncthreads();
      // the k-th largest of the row (ties kept): by counting
      int gt = 0, ge = 0;
      if (tid < total) {
        for (int c = 0; c < total; ++c) {
          const float o = s_lv[c];
          gt += o > v ? 1 : 0;
          ge += o >= v ? 1 : 0;
        }
        if (gt < a.topk && a.topk <= ge) s_cut = v;
      }
      const float mx = block_max_f32(v, fscratch);  // (a barrier: s_cut is set)
      const float cutoff = s_cut;
      // -1e7 must be so far below the kept values that its exponential is 0
      if (mx > kNegInf + 1000.f) {
        const bool kept = tid < total && v >= cutoff;
        const int slot = a.noise_step ? *a.noise_step % a.noise_ring : 0;
        Cand best = {-INFINITY, 0x7FFFFFFF};
        if (kept) {
          best.v = v + a.gumbel[((size_t)slot * a.R + r) * V + j];
          best.i = j;
        }
        best = block_best(best, cscratch);
        double sum = kept ? (double)expf(v - mx) : 0.0;
        sum = block_sum_f64(sum, dscratch);
        __syncthreads();
        if (kept && j == best.i) fscratch[0] = v;  // one thread holds the token
        __syncthreads();
        if (tid == 0) {
          a.tokens[r] = best.i;
          a.logprobs[r] = (fscratch[0] - mx) - (float)log(sum);
        }
        return;
      }
      __syncthreads();  // (everyone has read what the path below reuses)
    }
  }
  const float4 kPad = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  const float4* x4 = reinterpret_cast<const float4*>(a.logits + (size_t)r * V);
  float4 y[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int vi = u * 1024 + tid;
    y[u] = vi < nvec ? x4[vi] : kPad;
  }
  const float T = a.temperature[r];
  const float kMinT = 1e-4f;
  if (tid == 0) s_count = 0;

  if (!(T > kMinT)) {  // greedy (t5x/decoding.py:575-592)
    Cand best = {-INFINITY, 0x7FFFFFFF};
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int j = 4 * (u * 1024 + tid);  // ascending within the thread
      if (y[u].x > best.v) { best.v = y[u].x; best.i = j; }
      if (y[u].y > best.v) { best.v = y[u].y; best.i = j + 1; }
      if (y[u].z > best.v) { best.v = y[u].z; best.i = j + 2; }
      if (y[u].w > best.v) { best.v = y[u].w; best.i = j + 3; }
    }
    best = block_best(best, cscratch);
    float lp = 0.f;
    if (!a.rescale) {
      double sum = 0.0;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        sum += (double)expf(y[u].x - best.v);
        sum += (double)expf(y[u].y - best.v);
        sum += (double)expf(y[u].z - best.v);
        sum += (double)expf(y[u].w - best.v);
      }
      sum = block_sum_f64(sum, dscratch);
      lp = (best.v - best.v) - (float)log(sum);
    }
    if (tid == 0) { a.tokens[r] = best.i; a.logprobs[r] = lp; }
    return;
  }

  const float Tm = fmaxf(T, kMinT);
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    y[u].x /= Tm; y[u].y /= Tm; y[u].z /= Tm; y[u].w /= Tm;
  }

  float cutoff = -INFINITY;  // keep scaled >= cutoff
  if (a.topk > 0 && a.topk < V) {
    const int m = (a.topk + 15) >> 4;
    bool counted = false;
    if (m <= 8) {
      float tmax = -INFINITY;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        tmax = fmaxf(fmaxf(tmax, fmaxf(y[u].x, y[u].y)), fmaxf(y[u].z, y[u].w));
      // m-th largest per-thread maximum of this wavefront
      float rest = tmax, wm = -INFINITY;
      for (int it = 0; it < m; ++it) {
        wm = wave_max(rest);
        const unsigned long long hit = __builtin_amdgcn_ballot_w64(rest == wm);
        if (lane == (int)__builtin_ctzll(hit | (1ull << 63))) rest = -INFINITY;
      }
      if (lane == 0) fscratch[wave] = wm;
      __syncthreads();
      float bound = fscratch[0];
      for (int w = 1; w < 16; ++w) bound = fminf(bound, fscratch[w]);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float top = fmaxf(fmaxf(y[u].x, y[u].y), fmaxf(y[u].z, y[u].w));
        if (u * 1024 + tid < nvec && top >= bound) {
          const float e[4] = {y[u].x, y[u].y, y[u].z, y[u].w};
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            if (e[c] >= bound) {
              const int p = atomicAdd(&s_count, 1);
              if (p < kTopkCap) s_lv[p] = e[c];
            }
          }
        }
      }
      __syncthreads();
      const int ncand = s_count;
      if (ncand >= a.topk && ncand <= kTopkCap) {
        if (tid < ncand) {
          const float v = s_lv[tid];
          int gt = 0, ge = 0;
          for (int c = 0; c < ncand; ++c) {
            const float o = s_lv[c];
            gt += o > v ? 1 : 0;
            ge += o >= v ? 1 : 0;
          }
          // the k-th largest value; equal candidates all write the same bits
          if (gt < a.topk && a.topk <= ge) s_cut = v;
        }
        __syncthreads();
        cutoff = s_cut;
        counted = true;
      }
    }
    if (!counted)
      cutoff = kth_largest_by_radix(y, nvec, tid, a.topk, hist, iscratch);
  }
  // apply the top-k mask in place (t5x/decoding.py:556-562: others = -1e7)
  if (cutoff > -INFINITY) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (u * 1024 + tid < nvec) {
        y[u].x = y[u].x >= cutoff ? y[u].x : kNegInf;
        y[u].y = y[u].y >= cutoff ? y[u].y : kNegInf;
        y[u].z = y[u].z >= cutoff ? y[u].z : kNegInf;
        y[u].w = y[u].w >= cutoff ? y[u].w : kNegInf;
      }
    }
  }

  if (a.topp > 0.f) {
    // t5x/binary_search.py:230-299 — largest threshold whose kept mass >= p,
    // found by the same 32-step search over float bit patterns.
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < 8; ++u)
      mx = fmaxf(fmaxf(mx, fmaxf(y[u].x, y[u].y)), fmaxf(y[u].z, y[u].w));
    const float smax = block_max_f32(mx, fscratch);
    double sum = 0.0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      sum += (double)expf(y[u].x - smax);
      sum += (double)expf(y[u].y - smax);
      sum += (double)expf(y[u].z - smax);
      sum += (double)expf(y[u].w - smax);
    }
    const float ssum = (float)block_sum_f64(sum, dscratch);
    float4 pr[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      pr[u].x = expf(y[u].x - smax) / ssum;
      pr[u].y = expf(y[u].y - smax) / ssum;
      pr[u].z = expf(y[u].z - smax) / ssum;
      pr[u].w = expf(y[u].w - smax) / ssum;
    }
    int32_t bits = 0;
    for (int it = 0; it < 32; ++it) {
      const int32_t mid = it == 0 ? bits : (bits | (int32_t)(1u << (31 - it)));
      const int32_t pat = mid ^ (mid < 0 ? 0x7FFFFFFF : 0);
      const bool finite = (pat & 0x7F800000) != 0x7F800000;
      bool pred;
      if (finite) {
        const float thr = __int_as_float(pat);
        double mass = 0.0;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (pr[u].x >= thr) mass += (double)pr[u].x;
          if (pr[u].y >= thr) mass += (double)pr[u].y;
          if (pr[u].z >= thr) mass += (double)pr[u].z;
          if (pr[u].w >= thr) mass += (double)pr[u].w;
        }
        mass = block_sum_f64(mass, dscratch);
        pred = (float)mass < a.topp;
      } else {
        pred = pat >= 0;
      }
      if (it == 0) {
        if (pred) bits |= (int32_t)0x80000000u;
      } else if (!pred) {
        bits |= (int32_t)(1u << (31 - it));
      }
    }
    const int32_t pat = bits ^ (bits < 0 ? 0x7FFFFFFF : 0);
    const float pcut = __int_as_float(pat);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (u * 1024 + tid < nvec) {
        y[u].x = pr[u].x >= pcut ? y[u].x : kNegInf;
        y[u].y = pr[u].y >= pcut ? y[u].y : kNegInf;
        y[u].z = pr[u].z >= pcut ? y[u].z : kNegInf;
        y[u].w = pr[u].w >= pcut ? y[u].w : kNegInf;
      }
    }
  }

  // argmax(masked + gumbel), and log-softmax statistics of the masked row (or
  // of the raw logits when log-probs are not rescaled).
  const int slot = a.noise_step ? *a.noise_step % a.noise_ring : 0;
  const float4* g4 = reinterpret_cast<const float4*>(
      a.gumbel + ((size_t)slot * a.R + r) * V);
  Cand best = {-INFINITY, 0x7FFFFFFF};
  float mx = -INFINITY;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int vi = u * 1024 + tid;
    if (vi < nvec) {
      const float4 g = g4[vi];
      const int j = 4 * vi;
      const float z0 = y[u].x + g.x, z1 = y[u].y + g.y;
      const float z2 = y[u].z + g.z, z3 = y[u].w + g.w;
      if (z0 > best.v) { best.v = z0; best.i = j; }
      if (z1 > best.v) { best.v = z1; best.i = j + 1; }
      if (z2 > best.v) { best.v = z2; best.i = j + 2; }
      if (z3 > best.v) { best.v = z3; best.i = j + 3; }
    }
    // without rescaling the log-probs are those of the raw logits, read again
    const float4 w = a.rescale ? y[u] : (vi < nvec ? x4[vi] : kPad);
    mx = fmaxf(fmaxf(mx, fmaxf(w.x, w.y)), fmaxf(w.z, w.w));
  }
  best = block_best(best, cscratch);
  mx = block_max_f32(mx, fscratch);
  double sum = 0.0;
  float wtok = 0.f;
  bool mine = false;
  // After a top-k / top-p mask all but a few elements are -1e7, and with a
  // maximum this far above them exp(x - max) is exactly 0 in float32: chunks
  // that are masked throughout add nothing and skip the four exponentials.
  const bool far = mx > kNegInf + 1000.f;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const float4 w =
        a.rescale ? y[u] : (u * 1024 + tid < nvec ? x4[u * 1024 + tid] : kPad);
    const bool masked = far && w.x <= kNegInf && w.y <= kNegInf &&
                        w.z <= kNegInf && w.w <= kNegInf;
    if (!masked) {
      sum += (double)expf(w.x - mx);
      sum += (double)expf(w.y - mx);
      sum += (double)expf(w.z - mx);
      sum += (double)expf(w.w - mx);
    }
    const int j = 4 * (u * 1024 + tid);
    if (best.i == j) { wtok = w.x; mine = true; }
    if (best.i == j + 1) { wtok = w.y; mine = true; }
    if (best.i == j + 2) { wtok = w.z; mine = true; }
    if (best.i == j + 3) { wtok = w.w; mine = true; }
  }
  sum = block_sum_f64(sum, dscratch);
  __syncthreads();
  if (mine) fscratch[0] = wtok;  // exactly one thread holds the token
  __syncthreads();
  wtok = fscratch[0];
  if (tid == 0) {
    a.tokens[r] = best.i;
    a.logprobs[r] = (wtok - mx) - (float)log(sum);
  }
}

struct SampleUpdateArgs {
  const int32_t* tokens;
  const float* token_logprobs;
  int32_t* sequences;
  int32_t* cur_index;
  int32_t* cur_token;
  uint8_t* ended;
  float* log_prob;
  const int32_t* max_decode_len;
  const int32_t* initial_eos_count;
  int32_t* all_ended;
  int R, S, eos_id;
  // fused loop only: the loop flag (= !all_ended, also the gate of this
  // launch), the count of executed steps, and counters that advance with it
  // (the layers' cache indices)
  int32_t* keep_going;
  int32_t* step_count;
  int32_t* counters;
  int n_counters;
  const int32_t* gate;
};

// One workgroup; 8 lanes per row (128 rows per pass), which read the row's
// sequence once — counting its EOS tokens and picking up the forced token at
// position i + 1 on the way — so that every load of a row is asked for
// before the first one is waited for (with 16 lanes per row, 64 rows per pass,
// one row element per trip to the L2 and the loads chained index -> forced
// token -> row it took 13 us for 64 rows and 23 us for 128).
constexpr int kSampleUpdateThreads = 1024;
constexpr int kSampleUpdateLanes = 8;
__device__ __forceinline__ int lanes8_sum(int v) {
  v += dpp_move<kDppXor1>(v);
  v += dpp_move<kDppXor2>(v);
  return v + dpp_move<kDppHalfMirror>(v);
}

__global__ void __launch_bounds__(kSampleUpdateThreads)
sample_update_kernel(SampleUpdateArgs a) {
  __shared__ int iscratch[kSampleUpdateThreads / 64];
  T5D_GATED(a.gate);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int group = threadIdx.x / kSampleUpdateLanes;
  const int gl = threadIdx.x % kSampleUpdateLanes;
  int not_ended = 0;  // rows of this group still running (its lanes agree)
  for (int r0 = 0; r0 < a.R; r0 += kSampleUpdateThreads / kSampleUpdateLanes) {
    // whole wavefronts stay in the loop (the reductions below cross lanes);
    // groups past the last row work on row 0 and discard the result
    const bool real = r0 + group < a.R;
    const int r = real ? r0 + group : 0;
    int32_t* seq = a.sequences + (size_t)r * a.S;
    const int mdl = a.max_decode_len[r];
    const int ci = a.cur_index[r];
    const bool was_ended = a.ended[r] != 0;
    const int sampled = a.tokens[r];
    const float sampled_lp = a.token_logprobs[r];
    const float lp = a.log_prob[r];
    const int initial_eos = a.initial_eos_count[r];
    const int i = min(ci, mdl);
    // EOS count of the row without position i + 1, and that position's token
    // (12 loads in flight per lane and pass: a row of 258 takes three passes;
    // one load per pass would be one trip to the L2 per element)
    constexpr int kU = 12;
    int eos = 0, next_input = 0;
    for (int j0 = gl; j0 < a.S; j0 += kSampleUpdateLanes * kU) {
      int v[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int j = j0 + kSampleUpdateLanes * u;
        v[u] = j < a.S ? seq[j] : 0;
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int j = j0 + kSampleUpdateLanes * u;
        if (j == i + 1) next_input = v[u];
        else if (j < a.S) eos += (v[u] == a.eos_id) ? 1 : 0;
      }
    }
    eos = lanes8_sum(eos);
    next_input = lanes8_sum(next_input);  // one lane held it
    const bool oop = next_input == 0;
    const int tok = oop ? sampled : next_input;
    const int out_tok = was_ended ? 0 : tok;
    eos += (out_tok == a.eos_id) ? 1 : 0;
    const bool ended = was_ended || (eos > initial_eos) || (i >= mdl - 1);
    if (real && gl == 0) {
      if (oop && !was_ended) a.log_prob[r] = lp + sampled_lp;
      seq[i + 1] = out_tok;
      a.ended[r] = ended ? 1 : 0;
      a.cur_index[r] = i + 1;
      a.cur_token[r] = out_tok;
    }
    if (real && gl == 0 && !ended) ++not_ended;
  }
  // lanes 0, 8, .., 56 hold their groups' counts
  not_ended += __shfl_xor(not_ended, 8, 64);
  not_ended += __shfl_xor(not_ended, 16, 64);
  not_ended += __shfl_xor(not_ended, 32, 64);
  if (lane == 0) iscratch[wave] = not_ended;
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0;
    for (int w = 0; w < kSampleUpdateThreads / 64; ++w) total += iscratch[w];
    *a.all_ended = total == 0 ? 1 : 0;
    if (a.step_count) *a.step_count += 1;
    // the gate was read by every thread before the barrier above
    if (a.keep_going) *a.keep_going = total == 0 ? 0 : 1;
  }
  if ((int)threadIdx.x < a.n_counters) a.counters[threadIdx.x] += 1;
}

// ---- generic beam-axis gather (out of place) -----------------------------------
__global__ void gather_beams_kernel(const char* __restrict__ src,
                                    char* __restrict__ dst,
                                    const int32_t* __restrict__ idx,
                                    int old_beams, int new_beams,
                                    size_t inner_bytes) {
  const int be = blockIdx.x;  // b * new_beams + e
  const int b = be / new_beams;
  int s = idx[be];
  s = s < 0 ? 0 : (s >= old_beams ? old_beams - 1 : s);
  const char* p = src + ((size_t)b * old_beams + s) * inner_bytes;
  char* q = dst + (size_t)be * inner_bytes;
  if ((inner_bytes % 16) == 0 && (((uintptr_t)p | (uintptr_t)q) % 16) == 0) {
    const size_t n = inner_bytes / 16;
    for (size_t i = (size_t)blockIdx.y * blockDim.x + threadIdx.x; i < n;
         i += (size_t)gridDim.y * blockDim.x)
      reinterpret_cast<uint4*>(q)[i] = reinterpret_cast<const uint4*>(p)[i];
  } else {
    for (size_t i = (size_t)blockIdx.y * blockDim.x + threadIdx.x;
         i < inner_bytes; i += (size_t)gridDim.y * blockDim.x)
      q[i] = p[i];
  }
}

}  // namespace t5d

using namespace t5d;

extern "C" int t5d_top_k(void* stream, const float* x, float* vals,
                         int32_t* idx, int rows, int n, int k) {
  T5D_REQUIRE(x && vals && idx, T5D_EINVAL, "t5d_top_k: null pointer");
  T5D_REQUIRE(rows > 0 && n > 0 && k > 0 && k <= n, T5D_EINVAL,
              "t5d_top_k: rows=%d n=%d k=%d", rows, n, k);
  T5D_REQUIRE(k <= 64, T5D_ELIMIT, "t5d_top_k: k=%d > 64", k);
  hipLaunchKernelGGL(top_k_kernel, dim3(rows), dim3(256), 0, as_stream(stream),
                     x, vals, idx, n, k);
  T5D_CHECK_LAUNCH("t5d_top_k");
  return T5D_OK;
}

static int launch_row_topk(hipStream_t s, const float* logits,
                           const float* live_logprobs, float* row_max,
                           float* row_lse, float* cand_vals, int32_t* cand_idx,
                           int R, int V, int beams, int k) {
  if (V % 4 == 0 && V <= kFastTopkVec * 4096 && ((uintptr_t)logits % 16) == 0)
    hipLaunchKernelGGL(beam_row_topk_fast_kernel, dim3(R), dim3(1024), 0, s,
                       logits, live_logprobs, row_max, row_lse, cand_vals,
                       cand_idx, V, beams, k, tls_gate);
  else if (k <= 4)
    hipLaunchKernelGGL(beam_row_topk_kernel<4>, dim3(R), dim3(256), 0, s,
                       logits, live_logprobs, row_max, row_lse, cand_vals,
                       cand_idx, V, beams, k, tls_gate);
  else if (k <= 8)
    hipLaunchKernelGGL(beam_row_topk_kernel<8>, dim3(R), dim3(256), 0, s,
                       logits, live_logprobs, row_max, row_lse, cand_vals,
                       cand_idx, V, beams, k, tls_gate);
  else
    hipLaunchKernelGGL(beam_row_topk_kernel<16>, dim3(R), dim3(256), 0, s,
                       logits, live_logprobs, row_max, row_lse, cand_vals,
                       cand_idx, V, beams, k, tls_gate);
  T5D_CHECK_LAUNCH("beam top-k (rows)");
  return T5D_OK;
}

extern "C" int t5d_beam_topk(void* stream, const float* logits,
                             const float* live_logprobs, float* topk_vals,
                             int32_t* topk_idx, float* row_max, float* row_lse,
                             void* scratch, int B, int beams, int V, int k) {
  T5D_REQUIRE(logits && live_logprobs && topk_vals && topk_idx && row_max &&
                  row_lse && scratch,
              T5D_EINVAL, "t5d_beam_topk: null pointer");
  T5D_REQUIRE(B > 0 && beams > 0 && V > 0 && k > 0, T5D_EINVAL,
              "t5d_beam_topk: B=%d beams=%d V=%d k=%d", B, beams, V, k);
  T5D_REQUIRE(k <= 16 && beams * k <= 128, T5D_ELIMIT,
              "t5d_beam_topk: k=%d beams=%d (need k<=16, beams*k<=128)", k,
              beams);
  T5D_REQUIRE((long)beams * V < 0x7FFFFFFFL && k <= beams * V, T5D_EINVAL,
              "t5d_beam_topk: beams*V out of range");
  const int R = B * beams;
  float* cand_vals = (float*)scratch;
  int32_t* cand_idx = (int32_t*)((char*)scratch + (size_t)R * k * 4);
  hipStream_t s = as_stream(stream);
  int rc = launch_row_topk(s, logits, live_logprobs, row_max, row_lse, cand_vals,
                           cand_idx, R, V, beams, k);
  if (rc) return rc;
  hipLaunchKernelGGL(beam_merge_kernel, dim3(B), dim3(128), 0, s, cand_vals,
                     cand_idx, topk_vals, topk_idx, beams, k, tls_gate);
  T5D_CHECK_LAUNCH("t5d_beam_topk(merge)");
  return T5D_OK;
}

// ---- t5d_beam_topk for callers that cannot allocate ---------------------------
// The per-row candidates (what t5d_beam_topk keeps in its `scratch` argument)
// live in a file-scope device array instead.  Every GPU the library runs on
// holds its own copy of the array at its own address; the address is looked up
// once per device, with that device current, and kept.  The array's name is
// only a host-side handle: kernels get the looked-up pointer.
constexpr int kStaticCandPairs = 16384;  // rows * k candidates at most
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char
    g_topk_scratch[2 * kStaticCandPairs * 4];
static void* g_topk_scratch_ptr[kMaxDevices];
static std::mutex g_topk_scratch_mutex;

static int static_topk_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  T5D_REQUIRE(e == hipSuccess && dev >= 0 && dev < kMaxDevices, T5D_EHIP,
              "t5d_beam_topk_static: hipGetDevice: %s (device %d)",
              hipGetErrorString(e), dev);
  std::lock_guard<std::mutex> lock(g_topk_scratch_mutex);
  if (g_topk_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_topk_scratch));
    T5D_REQUIRE(e == hipSuccess && p != nullptr, T5D_EHIP,
                "t5d_beam_topk_static: hipGetSymbolAddress: %s",
                hipGetErrorString(e));
    g_topk_scratch_ptr[dev] = p;
  }
  *out = g_topk_scratch_ptr[dev];
  return T5D_OK;
}

extern "C" int t5d_beam_topk_static(void* stream, const float* logits,
                                    const float* live_logprobs,
                                    float* topk_vals, int32_t* topk_idx,
                                    float* row_max, float* row_lse, int B,
                                    int beams, int V, int k) {
  T5D_REQUIRE(B > 0 && beams > 0 && k > 0, T5D_EINVAL,
              "t5d_beam_topk_static: B=%d beams=%d k=%d", B, beams, k);
  T5D_REQUIRE((int64_t)B * beams * k <= kStaticCandPairs, T5D_ELIMIT,
              "t5d_beam_topk_static: B*beams*k = %lld candidates exceed the "
              "built-in workspace of %d; use t5d_beam_topk with a workspace of "
              "your own",
              (long long)B * beams * k, kStaticCandPairs);
  void* scratch = nullptr;
  int rc = static_topk_scratch(&scratch);
  if (rc) return rc;
  return t5d_beam_topk(stream, logits, live_logprobs, topk_vals, topk_idx,
                       row_max, row_lse, scratch, B, beams, V, k);
}

static int check_state(const char* name, const t5d_beam_state* st) {
  T5D_REQUIRE(st && st->cur_index && st->live_logprobs && st->finished_scores &&
                  st->live_seqs && st->finished_seqs && st->finished_flags,
              T5D_EINVAL, "%s: null beam state pointer", name);
  return T5D_OK;
}

extern "C" int t5d_beam_update(void* stream, const t5d_beam_state* cur,
                               const t5d_beam_state* next,
                               const float* topk_vals, const int32_t* topk_idx,
                               const int32_t* inputs,
                               const int32_t* initial_index,
                               const float* brevity,
                               int32_t* top_alive_indices, int B, int K, int S,
                               int Lin, int V, int eos_id) {
  int rc = check_state("t5d_beam_update", cur);
  if (rc) return rc;
  rc = check_state("t5d_beam_update", next);
  if (rc) return rc;
  T5D_REQUIRE(topk_vals && topk_idx && inputs && initial_index && brevity &&
                  top_alive_indices,
              T5D_EINVAL, "t5d_beam_update: null pointer");
  T5D_REQUIRE(B > 0 && K > 0 && S > 1 && Lin > 0 && V > 0, T5D_EINVAL,
              "t5d_beam_update: B=%d K=%d S=%d Lin=%d V=%d", B, K, S, Lin, V);
  T5D_REQUIRE(K <= kMaxBeams, T5D_ELIMIT, "t5d_beam_update: K=%d > %d", K,
              kMaxBeams);
  BeamUpdateArgs a;
  a.cur = *cur; a.next = *next;
  a.topk_vals = topk_vals; a.topk_idx = topk_idx; a.inputs = inputs;
  a.initial_index = initial_index; a.brevity = brevity;
  a.top_alive_indices = top_alive_indices;
  a.B = B; a.K = K; a.S = S; a.Lin = Lin; a.V = V; a.eos_id = eos_id;
  a.gate = tls_gate;
  a.cand_vals = nullptr; a.cand_idx = nullptr;
  a.topk_vals_out = nullptr; a.topk_idx_out = nullptr;
  a.cache_slot = a.cache_src = a.cache_dst = nullptr;
  hipLaunchKernelGGL(beam_update_kernel, dim3(B), dim3(kUpdateThreads), 0,
                     as_stream(stream), a);
  T5D_CHECK_LAUNCH("t5d_beam_update");
  hipLaunchKernelGGL(advance_index_kernel, dim3(1), dim3(1), 0,
                     as_stream(stream), cur->cur_index, next->cur_index,
                     tls_gate);
  T5D_CHECK_LAUNCH("t5d_beam_update(index)");
  return T5D_OK;
}

extern "C" int t5d_beam_cond(void* stream, const t5d_beam_state* state, int B,
                             int K, int S, float min_brevity,
                             float min_log_prob, int max_decode_step,
                             int min_initial_index, int32_t* keep_going) {
  int rc = check_state("t5d_beam_cond", state);
  if (rc) return rc;
  T5D_REQUIRE(keep_going && B > 0 && K > 0 && S > 1, T5D_EINVAL,
              "t5d_beam_cond: B=%d K=%d S=%d", B, K, S);
  hipLaunchKernelGGL(beam_cond_kernel, dim3(1), dim3(256), 0,
                     as_stream(stream), *state, B, K, S, min_brevity,
                     min_log_prob, max_decode_step, min_initial_index,
                     keep_going, tls_gate, 0, 1, nullptr, 0);
  T5D_CHECK_LAUNCH("t5d_beam_cond");
  return T5D_OK;
}

int t5d::launch_beam_select(hipStream_t s, const float* logits,
                            const t5d_beam_state* st, float* topk_vals,
                            int32_t* topk_idx, float* row_max, float* row_lse,
                            void* scratch, const int32_t* inputs,
                            const int32_t* initial_index, const float* brevity,
                            int32_t* top_alive, int B, int K, int S, int Lin,
                            int V, int eos_id, int32_t* cache_slot,
                            int32_t* cache_src, int32_t* cache_dst) {
  int rc = check_state("beam select", st);
  if (rc) return rc;
  T5D_REQUIRE(K <= kMaxBeams, T5D_ELIMIT, "beam select: K=%d > %d", K,
              kMaxBeams);
  const int k = 2 * K, R = B * K;
  float* cand_vals = (float*)scratch;
  int32_t* cand_idx = (int32_t*)((char*)scratch + (size_t)R * k * 4);
  rc = launch_row_topk(s, logits, st->live_logprobs, row_max, row_lse,
                       cand_vals, cand_idx, R, V, K, k);
  if (rc) return rc;
  BeamUpdateArgs a;
  a.cur = *st; a.next = *st;
  a.topk_vals = nullptr; a.topk_idx = nullptr; a.inputs = inputs;
  a.initial_index = initial_index; a.brevity = brevity;
  a.top_alive_indices = top_alive;
  a.B = B; a.K = K; a.S = S; a.Lin = Lin; a.V = V; a.eos_id = eos_id;
  a.gate = tls_gate;
  a.cand_vals = cand_vals; a.cand_idx = cand_idx;
  a.topk_vals_out = topk_vals; a.topk_idx_out = topk_idx;
  a.cache_slot = cache_slot; a.cache_src = cache_src; a.cache_dst = cache_dst;
  hipLaunchKernelGGL(beam_update_kernel, dim3(B), dim3(kUpdateThreads), 0, s, a);
  T5D_CHECK_LAUNCH("beam select");
  return T5D_OK;
}

int t5d::launch_beam_tail(hipStream_t s, const t5d_beam_state* state, int B,
                          int K, int S, float min_brevity, float min_log_prob,
                          int max_decode_step, int min_initial_index,
                          int32_t* keep_going, int do_cond, int32_t* counters,
                          int n_counters) {
  int rc = check_state("beam tail", state);
  if (rc) return rc;
  T5D_REQUIRE((keep_going || !do_cond) && B > 0 && K > 0 && S > 1 &&
                  n_counters >= 0 && n_counters <= 256 &&
                  (counters || n_counters == 0),
              T5D_EINVAL, "beam tail: B=%d K=%d S=%d counters=%d", B, K, S,
              n_counters);
  hipLaunchKernelGGL(beam_cond_kernel, dim3(1), dim3(256), 0, s, *state, B, K,
                     S, min_brevity, min_log_prob, max_decode_step,
                     min_initial_index, keep_going, tls_gate, 1, do_cond,
                     counters, n_counters);
  T5D_CHECK_LAUNCH("beam tail");
  return T5D_OK;
}

static void launch_sample_tokens(hipStream_t s, SampleArgs a, int R) {
  const bool aligned = ((uintptr_t)a.logits % 16) == 0 &&
                       (a.gumbel == nullptr || ((uintptr_t)a.gumbel % 16) == 0);
  const bool fast = a.V % 4 == 0 && a.V <= 32768 && aligned;
  // Two launches when the rows' candidates can be found by parts: a top-k
  // mask of at most kSamplePartCap, log-probs of the masked row, rows long
  // enough that every part holds k elements, few enough rows to leave CUs
  // idle otherwise.
  const bool by_parts = fast && a.parts != nullptr && a.gumbel != nullptr &&
                        a.topk > 0 && a.topk <= kSamplePartCap && a.rescale &&
                        !(a.topp > 0.f) && a.V >= 4096 && R <= 128;
  if (!by_parts) a.parts = nullptr;
  if (by_parts)
    hipLaunchKernelGGL(sample_topk_parts_kernel, dim3(kSampleParts, R),
                       dim3(256), 0, s, a);
  if (fast)
    hipLaunchKernelGGL(sample_tokens_fast_kernel, dim3(R), dim3(1024), 0, s, a);
  else
    hipLaunchKernelGGL(sample_tokens_kernel, dim3(R), dim3(256), 0, s, a);
}

extern "C" int64_t t5d_sample_tokens_workspace_bytes(int R) {
  return R > 0 ? (int64_t)(sample_parts_words(R) * sizeof(int32_t)) : 0;
}

extern "C" int t5d_sample_tokens(void* stream, const float* logits,
                                 const float* gumbel, const float* temperature,
                                 int32_t* tokens, float* logprobs, int R,
                                 int V, int topk, float topp, int rescale,
                                 void* workspace) {
  T5D_REQUIRE(logits && temperature && tokens && logprobs, T5D_EINVAL,
              "t5d_sample_tokens: null pointer");
  T5D_REQUIRE(R > 0 && V > 0 && topk >= 0 && topp >= 0.f, T5D_EINVAL,
              "t5d_sample_tokens: R=%d V=%d topk=%d topp=%f", R, V, topk,
              (double)topp);
  T5D_REQUIRE(!(topk > 0 && topp > 0.f), T5D_EINVAL,
              "At most one of `topp` or `topk` may be non-zero.");
  SampleArgs a;
  a.logits = logits; a.gumbel = gumbel; a.temperature = temperature;
  a.tokens = tokens; a.logprobs = logprobs;
  a.V = V; a.topk = topk; a.rescale = rescale; a.topp = topp;
  a.noise_step = nullptr; a.noise_ring = 1; a.R = R; a.gate = tls_gate;
  T5D_REQUIRE(((uintptr_t)workspace % 4) == 0, T5D_EINVAL,
              "t5d_sample_tokens: workspace alignment");
  a.parts = static_cast<int32_t*>(workspace);
  launch_sample_tokens(as_stream(stream), a, R);
  T5D_CHECK_LAUNCH("t5d_sample_tokens");
  return T5D_OK;
}

int t5d::launch_sample_step(hipStream_t s, const float* logits,
                            const t5d_sample_step* st, int R, int V,
                            int32_t* counters, int n_counters) {
  SampleArgs a;
  a.logits = logits; a.gumbel = st->gumbel; a.temperature = st->temperature;
  a.tokens = st->tokens; a.logprobs = st->token_logprobs;
  a.V = V; a.topk = st->topk; a.rescale = st->rescale; a.topp = st->topp;
  a.noise_step = st->step_count; a.noise_ring = st->noise_ring; a.R = R;
  a.gate = tls_gate;
  a.parts = static_cast<int32_t*>(st->workspace);
  launch_sample_tokens(s, a, R);
  T5D_CHECK_LAUNCH("sample step (tokens)");
  SampleUpdateArgs u;
  u.tokens = st->tokens; u.token_logprobs = st->token_logprobs;
  u.sequences = st->sequences; u.cur_index = st->cur_index;
  u.cur_token = st->cur_token; u.ended = st->ended; u.log_prob = st->log_prob;
  u.max_decode_len = st->max_decode_len;
  u.initial_eos_count = st->initial_eos_count; u.all_ended = st->all_ended;
  u.R = R; u.S = st->S; u.eos_id = st->eos_id;
  u.keep_going = st->keep_going; u.step_count = st->step_count;
  u.counters = counters; u.n_counters = n_counters; u.gate = tls_gate;
  hipLaunchKernelGGL(sample_update_kernel, dim3(1), dim3(kSampleUpdateThreads),
                     0, s, u);
  T5D_CHECK_LAUNCH("sample step (update)");
  return T5D_OK;
}

extern "C" int t5d_sample_update(void* stream, const int32_t* tokens,
                                 const float* token_logprobs,
                                 int32_t* sequences, int32_t* cur_index,
                                 int32_t* cur_token, uint8_t* ended,
                                 float* log_prob, const int32_t* max_decode_len,
                                 const int32_t* initial_eos_count,
                                 int32_t* all_ended, int R, int S, int eos_id) {
  T5D_REQUIRE(tokens && token_logprobs && sequences && cur_index && cur_token &&
                  ended && log_prob && max_decode_len && initial_eos_count &&
                  all_ended,
              T5D_EINVAL, "t5d_sample_update: null pointer");
  T5D_REQUIRE(R > 0 && S > 2, T5D_EINVAL, "t5d_sample_update: R=%d S=%d", R, S);
  SampleUpdateArgs a;
  a.tokens = tokens; a.token_logprobs = token_logprobs; a.sequences = sequences;
  a.cur_index = cur_index; a.cur_token = cur_token; a.ended = ended;
  a.log_prob = log_prob; a.max_decode_len = max_decode_len;
  a.initial_eos_count = initial_eos_count; a.all_ended = all_ended;
  a.R = R; a.S = S; a.eos_id = eos_id;
  a.keep_going = nullptr; a.step_count = nullptr; a.counters = nullptr;
  a.n_counters = 0; a.gate = tls_gate;
  hipLaunchKernelGGL(sample_update_kernel, dim3(1), dim3(kSampleUpdateThreads),
                     0, as_stream(stream), a);
  T5D_CHECK_LAUNCH("t5d_sample_update");
  return T5D_OK;
}

extern "C" int t5d_gather_beams(void* stream, const void* src, void* dst,
                                const int32_t* beam_indices, int B,
                                int old_beams, int new_beams,
                                int64_t inner_bytes) {
  T5D_REQUIRE(src && dst && beam_indices && src != dst, T5D_EINVAL,
              "t5d_gather_beams: null or aliased pointer");
  T5D_REQUIRE(B > 0 && old_beams > 0 && new_beams > 0 && inner_bytes > 0,
              T5D_EINVAL, "t5d_gather_beams: B=%d old=%d new=%d inner=%ld", B,
              old_beams, new_beams, (long)inner_bytes);
  int gy = (int)((inner_bytes / 16 + 255) / 256);
  gy = gy < 1 ? 1 : (gy > 64 ? 64 : gy);
  hipLaunchKernelGGL(gather_beams_kernel, dim3(B * new_beams, gy), dim3(256), 0,
                     as_stream(stream), (const char*)src, (char*)dst,
                     beam_indices, old_beams, new_beams, (size_t)inner_bytes);
  T5D_CHECK_LAUNCH("t5d_gather_beams");
  return T5D_OK;
}

extern "C" int t5d_gather_step_ids(void* stream, const int32_t* live_seqs,
                                   const int32_t* cur_index, int32_t* ids,
                                   int R, int S) {
  T5D_REQUIRE(live_seqs && cur_index && ids && R > 0 && S > 0, T5D_EINVAL,
              "t5d_gather_step_ids: null pointer or R=%d S=%d", R, S);
  hipLaunchKernelGGL(gather_ids_kernel, dim3((R + 63) / 64), dim3(64), 0,
                     as_stream(stream), live_seqs, cur_index, ids, R, S,
                     tls_gate);
  T5D_CHECK_LAUNCH("t5d_gather_step_ids");
  return T5D_OK;
}
