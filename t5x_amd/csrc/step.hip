// Fused host-side entry points: one call enqueues every kernel of a decoder
// step (and of a whole beam-search iteration) on the caller's stream, and a
// thin wrapper over HIP graph capture lets the caller record that call once
// and replay it every step.  Nothing here synchronises with the device.
#include <vector>

#include "common.h"
#include "../../include/t5d_measure.h"

using namespace t5d;

namespace {

// t5d_measure_leave_out: kernel families the calling thread's fused steps are
// enqueued without (a measurement aid, 0 in every product call).
thread_local int tls_leave_out = 0;

struct GateScope {
  explicit GateScope(const int32_t* g) { tls_gate = g; }
  ~GateScope() { tls_gate = nullptr; }
};

#define T5D_TRY(call)        \
  do {                       \
    int rc_ = (call);        \
    if (rc_ != T5D_OK) return rc_; \
  } while (0)

int check_model(const t5d_model_step* m) {
  T5D_REQUIRE(m && m->layers, T5D_EINVAL, "t5d step: null model description");
  T5D_REQUIRE(m->dtype == T5D_F32 || m->dtype == T5D_BF16, T5D_EINVAL,
              "t5d step: dtype %d", m->dtype);
  T5D_REQUIRE(m->d > 0 && m->H > 0 && m->F > 0 && m->V > 0 && m->L > 0 &&
                  m->E > 0 && m->NL > 0 && m->R > 0 && m->B > 0 &&
                  m->beams > 0 && m->R == m->B * m->beams,
              T5D_EINVAL,
              "t5d step: d=%d H=%d F=%d V=%d L=%d E=%d NL=%d R=%d B=%d beams=%d",
              m->d, m->H, m->F, m->V, m->L, m->E, m->NL, m->R, m->B, m->beams);
  T5D_REQUIRE(m->embedding && m->rel_bias && m->ln_final && m->logits_w &&
                  m->cache_index && m->enc_len && m->x && m->x1 && m->x2 &&
                  m->xn && m->qkv && m->q && m->ao && m->h && m->logits,
              T5D_EINVAL, "t5d step: null buffer");
  return T5D_OK;
}

}  // namespace

namespace {
// One decoder step.  ids == nullptr: the current tokens are read from
// seqs[r, *cur_index] inside the embedding kernel.  bump_index: add 1 to the
// layers' cache indices at the end (the beam-search step does that in its
// tail kernel instead).
int decoder_step_impl(void* stream, const t5d_model_step* m, const int32_t* ids,
                      const int32_t* seqs, const int32_t* cur_index, int S,
                      bool bump_index) {
  GateScope gate(m->gate);
  const int dt = m->dtype, wd = m->w_dtype;
  const int R = m->R, d = m->d, HD = m->H * 64, F = m->F;
  if (ids)
    T5D_TRY(t5d_embed(stream, dt, m->embedding, ids, m->x, R, d, m->V));
  else
    T5D_TRY(launch_embed_from_seqs(as_stream(stream), dt, m->embedding, seqs,
                                   cur_index, S, m->x, R, d, m->V));
  const void* x = m->x;
  // Layer norm + query projection ride inside the cross-attention kernel when
  // its limits allow (bfloat16 weights, E <= 512) and the model is narrow
  // enough for that to pay: every (item, head) workgroup re-reads the head's
  // slice of the query kernel, d * 128 bytes, next to at most E * 256 bytes of
  // K and V, and beyond d = 768 its registers no longer hold both streams
  // (measured at d = 1024: 56 us fused against 41 us for the three kernels).
  const bool fuse_cross_q = dt == T5D_BF16 && wd == T5D_BF16 && m->E <= 512 &&
                            d % 64 == 0 && d <= 768;
  // Likewise the pre-attention / pre-MLP norms ride inside their dense layers
  // where that was measured to pay: up to d = 1024 for every layer (all
  // fragments of a row tile fit the registers with room to spare); with int8
  // weights up to d = 2048 for a layer of at most 2048 columns (wider ones
  // lose more to the single resident workgroup per CU than the launch saves:
  // 23.8 us against 15.3 us for 6144 columns).
  // float32: always (the kernel carries the row statistics along for free).
  auto norm_rides = [&](int n_out) {
    if (dt == T5D_F32) return true;
    return dt == T5D_BF16 && d % 64 == 0 &&
           (d <= 1024 || (wd == T5D_I8 && d <= 2048 && n_out <= 2048));
  };
  for (int l = 0; l < m->NL; ++l) {
    const t5d_layer& w = m->layers[l];
    if (norm_rides(3 * HD)) {
      T5D_TRY(t5d_norm_gemm(stream, dt, wd, dt, x, w.ln_self, 1e-6f, w.qkv,
                            w.qkv_scales, m->qkv, R, d, 3 * HD, T5D_EPI_NONE));
    } else {
      T5D_TRY(t5d_rmsnorm(stream, dt, x, w.ln_self, m->xn, R, d, 1e-6f));
      T5D_TRY(t5d_gemm(stream, dt, wd, dt, m->xn, w.qkv, w.qkv_scales, nullptr,
                       m->qkv, R, d, 3 * HD, T5D_EPI_NONE, nullptr, nullptr));
    }
    if (tls_leave_out & T5D_LEAVE_OUT_SELF_ATTENTION) {
      // measurement aid: see t5d_measure_leave_out
    } else if (m->pending_src || m->value_blocked)
      T5D_TRY(t5d_self_attention_step_gather(
          stream, dt, m->qkv, w.cached_key, w.cached_value, m->rel_bias,
          m->cache_index + l, m->ao, m->B, m->beams, m->H, m->L,
          m->pending_src, m->pending_dst, m->value_blocked));
    else
      T5D_TRY(t5d_self_attention_step(stream, dt, m->qkv, w.cached_key,
                                      w.cached_value, m->rel_bias,
                                      m->cache_index + l, m->ao, R, m->H,
                                      m->L));
    T5D_TRY(t5d_gemm(stream, dt, wd, dt, m->ao, w.self_out, w.self_out_scales,
                     x, m->x1, R, HD, d, T5D_EPI_RESIDUAL, nullptr, nullptr));
    const bool no_cross = tls_leave_out & T5D_LEAVE_OUT_CROSS_ATTENTION;
    if (no_cross && fuse_cross_q) {
      // measurement aid: see t5d_measure_leave_out
    } else if (fuse_cross_q) {
      T5D_TRY(t5d_cross_attention_step_norm_q(
          stream, dt, wd, m->x1, w.ln_cross, 1e-6f, w.cross_q, w.cross_key,
          w.cross_value, m->enc_len, m->ao, m->B, m->beams, m->H, m->E, d,
          m->cross_units));
    } else {
      if (norm_rides(HD)) {
        T5D_TRY(t5d_norm_gemm(stream, dt, wd, dt, m->x1, w.ln_cross, 1e-6f,
                              w.cross_q, w.cross_q_scales, m->q, R, d, HD,
                              T5D_EPI_NONE));
      } else {
        T5D_TRY(t5d_rmsnorm(stream, dt, m->x1, w.ln_cross, m->xn, R, d, 1e-6f));
        T5D_TRY(t5d_gemm(stream, dt, wd, dt, m->xn, w.cross_q,
                         w.cross_q_scales, nullptr, m->q, R, d, HD,
                         T5D_EPI_NONE, nullptr, nullptr));
      }
      if (!no_cross)
        T5D_TRY(t5d_cross_attention_step(stream, dt, m->q, w.cross_key,
                                         w.cross_value, m->enc_len, m->ao,
                                         m->B, m->beams, m->H, m->E,
                                         dt == T5D_BF16 ? m->cross_units
                                                        : nullptr));
    }
    T5D_TRY(t5d_gemm(stream, dt, wd, dt, m->ao, w.cross_out,
                     w.cross_out_scales, m->x1, m->x2, R, HD, d,
                     T5D_EPI_RESIDUAL, nullptr, nullptr));
    if (norm_rides(2 * F)) {
      T5D_TRY(t5d_norm_gemm(stream, dt, wd, dt, m->x2, w.ln_mlp, 1e-6f, w.wi,
                            w.wi_scales, m->h, R, d, 2 * F, T5D_EPI_GEGLU));
    } else {
      T5D_TRY(t5d_rmsnorm(stream, dt, m->x2, w.ln_mlp, m->xn, R, d, 1e-6f));
      T5D_TRY(t5d_gemm(stream, dt, wd, dt, m->xn, w.wi, w.wi_scales, nullptr,
                       m->h, R, d, 2 * F, T5D_EPI_GEGLU, nullptr, nullptr));
    }
    T5D_TRY(t5d_gemm(stream, dt, wd, dt, m->h, w.wo, w.wo_scales, m->x2, m->x,
                     R, F, d, T5D_EPI_RESIDUAL, nullptr, nullptr));
    x = m->x;
  }
  // The final norm rides inside the vocabulary projection where the kernel
  // for very wide layers covers the shape (34 + 4.7 us as two kernels at
  // d = 768, V = 32128, 128 rows).
  if (dt == T5D_BF16 && norm_gemm_is_wide(wd, d, m->V)) {
    T5D_TRY(t5d_norm_gemm(stream, dt, wd, T5D_F32, x, m->ln_final, 1e-6f,
                          m->logits_w, nullptr, m->logits, R, d, m->V,
                          T5D_EPI_NONE));
  } else {
    T5D_TRY(t5d_rmsnorm(stream, dt, x, m->ln_final, m->xn, R, d, 1e-6f));
    T5D_TRY(t5d_gemm(stream, dt, wd, T5D_F32, m->xn, m->logits_w,
                     m->logits_scales, nullptr, m->logits, R, d, m->V,
                     T5D_EPI_NONE, nullptr, nullptr));
  }
  if (bump_index) T5D_TRY(t5d_add_i32(stream, m->cache_index, m->NL, 1));
  return T5D_OK;
}
}  // namespace

extern "C" int t5d_decoder_step(void* stream, const t5d_model_step* m,
                                const int32_t* ids) {
  T5D_TRY(check_model(m));
  T5D_REQUIRE(ids, T5D_EINVAL, "t5d_decoder_step: null ids");
  return decoder_step_impl(stream, m, ids, nullptr, nullptr, 0, true);
}

extern "C" int t5d_beam_search_step(void* stream, const t5d_model_step* m,
                                    const t5d_beam_step* b) {
  T5D_TRY(check_model(m));
  T5D_REQUIRE(b && b->ids && b->topk_vals && b->topk_idx && b->row_max &&
                  b->row_lse && b->scratch && b->top_alive && b->keep_going &&
                  b->inputs && b->initial_index && b->brevity && b->kv_base,
              T5D_EINVAL, "t5d_beam_search_step: null buffer");
  T5D_REQUIRE(m->gate == b->keep_going, T5D_EINVAL,
              "t5d_beam_search_step: the model gate must be the loop flag");
  const bool slots = b->cache_slot || b->cache_src || b->cache_dst;
  if (slots) {
    T5D_REQUIRE(b->cache_slot && b->cache_src && b->cache_dst, T5D_EINVAL,
                "t5d_beam_search_step: cache_slot / cache_src / cache_dst go "
                "together");
    T5D_REQUIRE(m->pending_src == b->cache_src && m->pending_dst == b->cache_dst,
                T5D_EINVAL,
                "t5d_beam_search_step: with cache slots the model's pending_src "
                "/ pending_dst must be cache_src / cache_dst");
  } else {
    T5D_REQUIRE(m->pending_dst == nullptr &&
                    (m->pending_src == nullptr || m->pending_src == b->top_alive),
                T5D_EINVAL,
                "t5d_beam_search_step: pending_src must be the top_alive buffer");
  }
  const int K = m->beams, B = m->B;
  T5D_TRY(decoder_step_impl(stream, m, nullptr, b->state.live_seqs,
                            b->state.cur_index, b->S, false));
  GateScope gate(b->keep_going);
  hipStream_t hs = as_stream(stream);
  T5D_TRY(launch_beam_select(hs, m->logits, &b->state, b->topk_vals,
                             b->topk_idx, b->row_max, b->row_lse, b->scratch,
                             b->inputs, b->initial_index, b->brevity,
                             b->top_alive, B, K, b->S, b->Lin, m->V,
                             b->eos_id, b->cache_slot, b->cache_src,
                             b->cache_dst));
  // When the model applies pending gathers inside its self-attention
  // (pending_src == top_alive) the reorder happens there, on the next step.
  // Otherwise reorder now: cur_index + 1 columns are valid.
  if (K > 1 && m->pending_src == nullptr)
    T5D_TRY(t5d_cache_gather_beams(
        stream, b->kv_base, b->kv_tensor_stride_bytes, b->n_kv_tensors,
        m->dtype == T5D_F32 ? 4 : 2, B, K, m->H * 64, m->L, b->top_alive,
        b->state.cur_index, 1));
  // The tail advances cur_index and the cache indices and evaluates the loop
  // condition.
  T5D_TRY(launch_beam_tail(hs, &b->state, B, K, b->S, b->min_brevity,
                           b->min_log_prob, b->max_decode_step,
                           b->min_initial_index, b->keep_going, !b->skip_cond,
                           m->cache_index, m->NL));
  return T5D_OK;
}

extern "C" int t5d_temperature_sample_step(void* stream,
                                           const t5d_model_step* m,
                                           const t5d_sample_step* s) {
  T5D_TRY(check_model(m));
  T5D_REQUIRE(s && s->sequences && s->cur_index && s->cur_token && s->ended &&
                  s->log_prob && s->max_decode_len && s->initial_eos_count &&
                  s->temperature && s->step_count && s->tokens &&
                  s->token_logprobs && s->all_ended && s->keep_going,
              T5D_EINVAL, "t5d_temperature_sample_step: null buffer");
  T5D_REQUIRE(m->gate == s->keep_going, T5D_EINVAL,
              "t5d_temperature_sample_step: the model gate must be the loop "
              "flag");
  T5D_REQUIRE(m->pending_src == nullptr, T5D_EINVAL,
              "t5d_temperature_sample_step: sampling rows are never reordered");
  T5D_REQUIRE(s->S > 2 && s->topk >= 0 && s->topp >= 0.f &&
                  (s->gumbel == nullptr || s->noise_ring > 0),
              T5D_EINVAL,
              "t5d_temperature_sample_step: S=%d topk=%d topp=%f ring=%d", s->S,
              s->topk, (double)s->topp, s->noise_ring);
  T5D_REQUIRE(!(s->topk > 0 && s->topp > 0.f), T5D_EINVAL,
              "At most one of `topp` or `topk` may be non-zero.");
  T5D_TRY(decoder_step_impl(stream, m, s->cur_token, nullptr, nullptr, 0,
                            false));
  GateScope gate(s->keep_going);
  return launch_sample_step(as_stream(stream), m->logits, s, m->R, m->V,
                            m->cache_index, m->NL);
}

extern "C" int t5d_measure_leave_out(int mask) {
  const int before = tls_leave_out;
  tls_leave_out = mask;
  return before;
}

// ---- HIP graph capture --------------------------------------------------------

extern "C" int t5d_graph_begin(void* stream) {
  hipError_t e = hipStreamBeginCapture(as_stream(stream),
                                       hipStreamCaptureModeThreadLocal);
  T5D_REQUIRE(e == hipSuccess, T5D_EHIP, "t5d_graph_begin: %s",
              hipGetErrorString(e));
  return T5D_OK;
}

extern "C" int t5d_graph_end(void* stream, void** graph_exec) {
  T5D_REQUIRE(graph_exec, T5D_EINVAL, "t5d_graph_end: null output");
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(as_stream(stream), &graph);
  T5D_REQUIRE(e == hipSuccess && graph, T5D_EHIP, "t5d_graph_end: %s",
              hipGetErrorString(e));
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  T5D_REQUIRE(e == hipSuccess && exec, T5D_EHIP,
              "t5d_graph_end: instantiate: %s", hipGetErrorString(e));
  *graph_exec = exec;
  return T5D_OK;
}

extern "C" int t5d_graph_launch(void* graph_exec, void* stream) {
  T5D_REQUIRE(graph_exec, T5D_EINVAL, "t5d_graph_launch: null graph");
  hipError_t e = hipGraphLaunch(reinterpret_cast<hipGraphExec_t>(graph_exec),
                                as_stream(stream));
  T5D_REQUIRE(e == hipSuccess, T5D_EHIP, "t5d_graph_launch: %s",
              hipGetErrorString(e));
  return T5D_OK;
}

extern "C" int t5d_graph_destroy(void* graph_exec) {
  if (!graph_exec) return T5D_OK;
  hipError_t e =
      hipGraphExecDestroy(reinterpret_cast<hipGraphExec_t>(graph_exec));
  T5D_REQUIRE(e == hipSuccess, T5D_EHIP, "t5d_graph_destroy: %s",
              hipGetErrorString(e));
  return T5D_OK;
}
