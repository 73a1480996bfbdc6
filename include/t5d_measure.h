/* Measurement aids of libt5d.so.  NOT part of the drop-in boundary
 * (include/t5d.h): nothing here has a counterpart in the reference and no
 * product code calls it; bench.py does, to time a kernel family where it
 * runs. */
#ifndef T5D_MEASURE_H_
#define T5D_MEASURE_H_

#ifdef __cplusplus
extern "C" {
#endif

enum {
  T5D_LEAVE_OUT_CROSS_ATTENTION = 1,  /* t5d_cross_attention_step[_norm_q] */
  T5D_LEAVE_OUT_SELF_ATTENTION = 2    /* t5d_self_attention_step[_gather] */
};

/* Sets, for the calling thread, a mask of T5D_LEAVE_OUT_* bits (0 restores the
 * normal behaviour) and returns the previous mask.  While a bit is set, the
 * fused entry points (t5d_decoder_step, t5d_beam_search_step,
 * t5d_temperature_sample_step) enqueue their step WITHOUT the launches of that
 * kernel family: its outputs keep whatever the buffers held, so the results
 * are meaningless.  The time a loop of such steps saves against the full loop
 * is what the family costs where it runs, between the step's other kernels. */
int t5d_measure_leave_out(int mask);

#ifdef __cplusplus
}
#endif
#endif  /* T5D_MEASURE_H_ */
