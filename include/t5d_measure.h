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

/* Two plain streaming kernels of known size, for what the memory system
 * gives a kernel that does nothing else (bench.py --stage memory; also the
 * copy of known size that counter readings are calibrated on).  `bytes` is a
 * multiple of 16; `blocks` workgroups of 256 threads walk the buffer with
 * 16-byte accesses, workgroup b taking the pieces b, b + blocks, ...
 *   t5d_measure_fill: writes the buffer.
 *   t5d_measure_read: reads it; workgroup b takes the pieces that workgroup
 *   (b + shift) % blocks of a fill or read with the same `blocks` took
 *   (workgroups are dealt to the XCDs in turn, so a shift that is not a
 *   multiple of 8 reads every piece through another XCD's L2 than wrote it).
 *   `sink` (4 bytes of device memory) keeps the loads alive; `tag` (0..5)
 *   picks one of six identical kernels, so that a kernel trace keeps the
 *   launches of different measurements apart.
 * Both return 0 or a negative T5D_E* code, like the boundary's calls. */
int t5d_measure_fill(void* stream, void* buffer, long long bytes,
                     unsigned seed, int blocks);
int t5d_measure_read(void* stream, const void* buffer, long long bytes,
                     int shift, int blocks, void* sink, int tag);

#ifdef __cplusplus
}
#endif
#endif  /* T5D_MEASURE_H_ */
