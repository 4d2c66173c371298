/*
 * paella_ring.h -- C-ABI for exercising and timing the GPU->host notification channel on its own.
 *
 * The channel itself is the C++ type llis::ipc::Gpu2SchedChannel plus the device-side hooks in
 * llis/job/finished_block_notifier.h and llis/job/instrument.h; these entry points wrap them so that a
 * test or bench written in another language can (a) launch an instrumented kernel of a chosen grid and
 * collect the raw 64-bit messages, and (b) run the two latency probes the reference keeps as stand-alone
 * programs:
 *   paella_ring_bench_drain     N-workgroup kernel, every workgroup writes a start and an end message,
 *                               host drains 2*N messages per iteration
 *                               (reference tests/ipc/shm_channel/latency/shmpc_latency_gpu.cu:7-67)
 *   paella_ring_bench_pingpong  host clears a flag, a one-lane kernel sets it with a system-scope store,
 *                               host spins; compared with hipStreamSynchronize of an empty kernel
 *                               (reference tests/simple/cuda_sync_benchmark.cu:12-32)
 * Return value: 0 on success, hipError_t (>0) or -1 (bad argument / timeout) otherwise.
 */
#ifndef PAELLA_RING_H
#define PAELLA_RING_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct paella_ring paella_ring;

/* Workgroups covered by one aggregated message when nothing else is asked for
 * (llis::job::FinishedBlockNotifier::noti_batch_size; the reference's constant is 16,
 * reference include/llis/job/finished_block_notifier.h:118). */
unsigned paella_ring_batch_size(void);

/* A ring of `slots` 64-bit slots in coherent host memory plus `num_notifiers` device-resident notifiers. */
int paella_ring_create(size_t slots, unsigned num_notifiers, paella_ring** out);
/* The same with notifiers that send one message per `batch` workgroups (a power of two, at most 128; else -1). */
int paella_ring_create_batched(size_t slots, unsigned num_notifiers, unsigned batch, paella_ring** out);
int paella_ring_destroy(paella_ring* ring);
/* Device pointer to notifier `idx` (an llis::job::FinishedBlockNotifier*). */
void* paella_ring_notifier(paella_ring* ring, unsigned idx);
/* Pointer to the underlying llis::ipc::Gpu2SchedChannel (host object). */
void* paella_ring_channel(paella_ring* ring);

/* Launches a small vector-add kernel of grid (gx,gy,gz) x block threads on `stream`, instrumented with
 * the aggregated notifier hooks (hooks = 0) or the per-workgroup kernel_start/kernel_end hooks (hooks = 1). */
int paella_ring_probe_launch(paella_ring* ring, unsigned notifier_idx, unsigned gx, unsigned gy, unsigned gz,
                             unsigned block, uint32_t job_id, int hooks, void* stream);

/* Host consumer.  drain() reads exactly n messages (as raw slot values, ready byte cleared on return) or
 * gives up after timeout_s seconds; returns the number read. */
int paella_ring_can_read(paella_ring* ring);
size_t paella_ring_drain(paella_ring* ring, uint64_t* out, size_t n, double timeout_s);

/* Latency probes; results in microseconds. */
int paella_ring_bench_drain(paella_ring* ring, unsigned blocks, unsigned vec_len, int warmup, int iters,
                            double* us_per_iter);
int paella_ring_bench_pingpong(int warmup, int iters, double* flag_us, double* sync_us, double* flag_samples_us);

/* One-way notification latency without a kernel launch in the way (the reference has no counterpart; its probes
 * above include the launch).  A resident one-lane kernel answers warmup + iters host pings: for each, the host
 * raises a flag in host memory, the lane sees it, reads the device's realtime counter and sends one ring message.
 *   round_trip_us[i]  host flag store -> message readable on the host (upper bound of the notification latency)
 *   gpu_to_host_us[i] (may be NULL) host time at which the message became readable minus the lane's counter value
 *                     translated to the host's clock by the runtime; -1e30 where the translation is unavailable.
 * Both arrays hold `iters` doubles.  The lane's wait is bounded (20 s of device time) and ends early on error. */
int paella_ring_bench_echo(paella_ring* ring, int warmup, int iters, double* round_trip_us, double* gpu_to_host_us);

#ifdef __cplusplus
}
#endif
#endif
