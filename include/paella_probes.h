/* C ABI of libpaella_probes.so: measurement probes of the device (launch floor, sustained matrix rate, vector/matrix
 * overlap, queue concurrency).  Loaded by the bench and the tests only; the operator and serving libraries do not link it.
 * No counterpart in the reference, which measures none of these. */
#ifndef PAELLA_PROBES_H
#define PAELLA_PROBES_H

#ifdef __cplusplus
extern "C" {
#endif

/* Duration of a kernel that does nothing (256 workgroups of 256 lanes), between the begin and end time stamps the
 * device records for it: the floor under every per-launch figure measured the same way.  Median of `iters` launches. */
int paella_empty_kernel_probe(int iters, double* median_us);

/* Sustained fp32 MFMA rate of the device (v_mfma_f32_32x32x2_f32, register-resident operands, every SIMD busy):
 * the measured denominator next to the published 157.3 TFLOP/s. */
int paella_mfma_peak_probe(double* tflops);

/* Whether vector-ALU work hides behind matrix instructions on this device.  A register-resident loop, eight waves per SIMD,
 * of four v_mfma_f32_32x32x2_f32 and `valu_per_four_mfma` independent multiply-adds per iteration (0, 8, 16, 32, 64 or 128),
 * 2000 iterations: *us_both is its duration, *us_valu_alone that of the same loop without the matrix instructions, *tflops the
 * matrix rate of the first.  On MI355X us_both equals the N = 0 duration plus us_valu_alone: the two do not overlap, whichever
 * waves of the SIMD they come from (what the conv kernel's reduction loop is built around). */
int paella_mfma_valu_overlap_probe(int valu_per_four_mfma, double* us_both, double* us_valu_alone, double* tflops);

/* How many kernels the device runs side by side, and what sharing a launch is worth.  `instances` independent copies of
 * the conv layer `desc` (32 x 32 tile; own input, output and workspace each, shared weights) are launched round-robin over
 * `queues` direct-dispatch queues (with the barrier bit when `ordered`), `per_launch` (1 .. PAELLA_CONV_GROUP_MAX) of them
 * in one grid, `reps` times over; *us_per_conv = elapsed / (reps x instances).  One unordered queue against four shows
 * whether a queue overlaps its kernels; per_launch 1 against 4 shows the gain of packing. */
struct paella_conv_desc;
int paella_queue_concurrency_probe(const struct paella_conv_desc* desc, int instances, int per_launch, int queues, int ordered, int reps,
                                   double* us_per_conv);

#ifdef __cplusplus
}
#endif
#endif
