/*
 * paella_ops.h -- C-ABI of the hand-written gfx950 operator kernels (fp32, NCHW, batch 1).
 *
 * These entry points replace the kernels that the reference obtains from its custom TVM build: in the
 * reference the only call site is `run_()` inside every job adapter (reference
 * jobs/tvm_mnist/tvm_mnist.cpp:24-33,41 and the ten sibling adapters), which executes one generated CUDA
 * kernel per scheduler stage.  Here each of those kernels is an explicit launch function.
 *
 * Conventions
 *   - all tensor pointers are DEVICE pointers to contiguous fp32 NCHW data with N == 1; a channel slice
 *     of a larger tensor is contiguous for N == 1, so "write into channels [off, off+K) of a concat
 *     buffer" is expressed by offsetting the pointer;
 *   - `stream` is a hipStream_t passed as void*;
 *   - `notifier` is a device pointer to an llis::job::FinishedBlockNotifier (or NULL for un-instrumented
 *     launches); when non-NULL every workgroup calls notifier->start(job_id) on entry and
 *     notifier->end(job_id) on exit (reference include/llis/job/finished_block_notifier.h:18-94);
 *   - every function returns 0 on success, a negative PAELLA_E* code for a rejected argument and a
 *     positive hipError_t for a runtime failure.  Nothing falls back to the CPU.
 */
#ifndef PAELLA_OPS_H
#define PAELLA_OPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* OR-ed into the job_id argument of a launch: the kernel reports only workgroup ENDS, not starts.  A scheduler
 * needs start messages only for kernels it admitted beyond the occupancy budget (to learn when they have
 * become fully resident); for every other kernel they are pure overhead.  Messages carry the id without the bit. */
#define PAELLA_JOB_ID_NO_START 0x80000000u
/* OR-ed into job_id by callers whose scheduler collects per-workgroup timing (second ring of the notifier):
 * the kernel samples the clock on entry and exit and reports the pair.  Off: the kernel never looks. */
#define PAELLA_JOB_ID_TIME_BLOCKS 0x40000000u
#define PAELLA_JOB_ID_FLAGS (PAELLA_JOB_ID_NO_START | PAELLA_JOB_ID_TIME_BLOCKS)

#define PAELLA_EINVAL (-1)   /* malformed descriptor */
#define PAELLA_ENOSUP (-2)   /* shape class not implemented (e.g. grouped conv that is not depthwise), or facility unavailable */
#define PAELLA_ETIMEDOUT (-3) /* a bounded wait expired */

enum paella_act { PAELLA_ACT_NONE = 0, PAELLA_ACT_RELU = 1, PAELLA_ACT_RELU6 = 2, PAELLA_ACT_PRELU = 3, PAELLA_ACT_CLIP = 4 };

/* Resources of one launch, in the units the block-level scheduler accounts in
 * (reference include/llis/job/job.h:62-76, src/server/sm_resources.cpp:36-66). */
typedef struct paella_launch_dims {
    unsigned grid;        /* number of workgroups */
    unsigned block;       /* threads per workgroup */
    unsigned lds_bytes;   /* LDS per workgroup: what the launch asks for (paella_conv_plan.dims) or, from the *_dims functions
                             that look at the loaded kernel, that plus the kernel's statically allocated LDS */
    unsigned vgprs;       /* vector registers per thread */
} paella_launch_dims;

/* ---------------------------------------------------------------- conv2d (O1 dense, O2 depthwise) */

typedef struct paella_conv_desc {
    int C, H, W;                 /* input */
    int K, R, S;                 /* output channels, kernel */
    int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
    int groups;                  /* 1 (implicit GEMM on MFMA) or C == K (depthwise) */
    int act;                     /* enum paella_act, applied after bias and residual */
    float act_lo, act_hi;        /* PAELLA_ACT_CLIP bounds */
} paella_conv_desc;

typedef struct paella_conv_plan {
    paella_conv_desc d;
    int P, Q;                    /* output extent */
    int kind;                    /* 0 = MFMA implicit GEMM, 1 = depthwise */
    int mi, ni, kw;              /* per-wave tile = (32*mi) x (32*ni) outputs, kw waves split the reduction */
    int splits;                  /* workgroups per output tile that split the reduction further (grid z) */
    int m_pad, k_pad;            /* padded GEMM dims of the packed weight blob */
    int k_order;                 /* reduction order of the blob: 0 = (c, r, s), 1 = (r, s, c) (chosen when C % 8 == 0) */
    int wg_order;                /* which workgroups share an XCD (and its L2): 1 = readers of the same weights, 0 = neighbouring pixel tiles, 2 = launch order */
    int fast_div;                /* 1: the kernel divides by multiply-high where its operands allow (0 only for tests of the plain path) */
    size_t blob_bytes;           /* size of the packed weight blob */
    size_t workspace_bytes;      /* per-request scratch for splits > 1 (0 otherwise); must start out zeroed */
    paella_launch_dims dims;
    double flops;                /* algorithmic: 2*K*(C/g)*R*S*P*Q */
    double bytes;                /* algorithmic: 4*(C*H*W + K*(C/g)*R*S + K + K*P*Q [+K*P*Q residual]) */
    int depth;                   /* chunks of operands a wave keeps in flight; 0 = the tile's default */
    int pair_taps;               /* 0, or 1 + the first of two filter columns whose chunks are interleaved in the blob: a stride-2
                                    3-wide filter reads them as neighbouring input pixels (see the kernel's operand fetch) */
} paella_conv_plan;

/* Pure host arithmetic: picks the kernel variant and launch shape.  tile_hint = 0 lets the library
 * choose; otherwise log2(splits)<<12 | mi<<8 | ni<<4 | log2(kw) forces a shape (tuning sweeps and tests). */
int paella_conv2d_plan(const paella_conv_desc* desc, int has_residual, int tile_hint, paella_conv_plan* plan);

/* Launch shape of paella_conv2d_launch for the scheduler: the plan's, with the register count and the static LDS of the
 * kernel that is actually launched (read from the loaded code object; the plan's own figures without a device). */
int paella_conv2d_dims(const paella_conv_plan* plan, paella_launch_dims* dims);

/* Re-lays out OIHW weights [K][C/g][R][S] into the blob the kernel reads (host memory to host memory). */
int paella_conv2d_pack(const paella_conv_plan* plan, const float* w_oihw, void* blob_host);

/* y = act(conv(x, w) + bias + residual); bias, residual, slope may be NULL (slope: PReLU, per channel).
 * workspace: device buffer of plan->workspace_bytes, private to the request (launches that share it must not
 * overlap), zero-filled once before its first use; NULL when workspace_bytes == 0. */
int paella_conv2d_launch(const paella_conv_plan* plan, const float* x, const void* blob_dev, const float* bias,
                         const float* residual, const float* slope, float* y, void* workspace,
                         void* stream, uint32_t job_id, void* notifier);

/* paella_conv2d_launch for callers that cannot allocate and have no workspace to bring (code under stream capture,
 * tight serving loops, harnesses that forbid hipMalloc): the split reduction's counters and partial tiles live in a
 * fixed array inside the library's device image (PAELLA_CONV_STATIC_WORKSPACE_BYTES per GPU, there from load to
 * process end) instead of a caller-supplied workspace.  No counterpart in the reference.  Same kernels, same results
 * bit for bit as paella_conv2d_launch.  Performs no device or host allocation.  Limits: plan->workspace_bytes must
 * not exceed PAELLA_CONV_STATIC_WORKSPACE_BYTES (PAELLA_ETOOBIG otherwise, nothing launched); `stream` must be a HIP
 * stream, not a direct-dispatch queue (PAELLA_ENOSUP); all calls on one GPU share the one array, so two calls that may
 * overlap in time on that GPU (different streams, no dependency between them) race -- serialise them.  Every call
 * first zeroes the counters it will use with a small fill kernel on `stream` (the array keeps whatever the last
 * call, or an interrupted one, left behind); arguments are checked before that kernel goes out, so a refused call launches
 * nothing.  The first use on a GPU looks up that GPU's copy of the array (a runtime call that may load the code object: not
 * for a stream under capture): call paella_conv2d_static_init() once per GPU, with that GPU current, before capturing, or
 * make the first paella_conv2d_launch_static call there outside capture.  paella_conv2d_static_workspace() hands out the
 * array's device address on the current GPU (diagnostics and tests: what is in it between calls is the library's). */
#define PAELLA_CONV_STATIC_WORKSPACE_BYTES (4u << 20)
#define PAELLA_ETOOBIG (-4)  /* the request exceeds a fixed capacity of the library */
int paella_conv2d_static_init(void);
int paella_conv2d_static_workspace(void** ptr);
int paella_conv2d_launch_static(const paella_conv_plan* plan, const float* x, const void* blob_dev, const float* bias,
                                const float* residual, const float* slope, float* y, void* stream, uint32_t job_id,
                                void* notifier);

/* The same conv on a transformed input: x' = in_act(x * in_scale[c] + in_shift[c]) per input channel c, with the
 * zero padding applied AFTER the transform (a padding tap contributes 0, not in_act(in_shift[c])); in_act is
 * PAELLA_ACT_NONE or PAELLA_ACT_RELU.  This is a batch-norm (+ ReLU) stage that stands in front of a conv and cannot
 * be folded into the producer's weights -- pre-activation dense layers, the leading norm of an ArcFace unit -- run
 * inside the conv's operand fetch instead of as a kernel of its own.  The reference's generated code gets the same
 * effect from TVM's operator fusion (the kernels behind reference jobs/tvm_arcfaceresnet100/tvm_arcfaceresnet100.cpp:41 and
 * jobs/tvm_densenet121/tvm_densenet121.cpp:41).  Only plans for which paella_conv2d_plan_takes_input_transform() returns 1
 * (MFMA plan, mi == ni == 1, C a multiple of 8); PAELLA_ENOSUP otherwise. */
int paella_conv2d_plan_takes_input_transform(const paella_conv_plan* plan);
/* Launch shape of that form: the plan's, with the register count of the kernel that is actually launched and the LDS of its
 * table of scales and shifts (64 bytes + 8 per input channel, on top of the plan's). */
int paella_conv2d_transformed_dims(const paella_conv_plan* plan, paella_launch_dims* dims);
int paella_conv2d_launch_transformed(const paella_conv_plan* plan, const float* x, const float* in_scale, const float* in_shift,
                                     int in_act, const void* blob_dev, const float* bias, const float* residual,
                                     const float* slope, float* y, void* workspace, void* stream, uint32_t job_id,
                                     void* notifier);

/* Two convs that do not depend on each other as ONE launch: the first problem's workgroups followed by the
 * second's, so that layers whose own grids are far below the 256 CUs (the 1x1 projection beside a residual block's
 * first 3x3 conv, parallel branches of an inception module) fill the device together and cost one dispatch.  No
 * counterpart in the reference, whose generated code launches every operator by itself.  Both plans must be MFMA
 * plans with mi == ni == 1 and the same kw and k_order (paella_conv2d_pair_dims returns PAELLA_ENOSUP otherwise; a
 * plan can be forced to that shape with tile_hint); neither conv may read or overwrite what the other writes, and
 * two split plans need separate workspaces.  The results are bit-identical to two paella_conv2d_launch calls.
 * The hooks report one kernel of dims->grid workgroups. */
typedef struct paella_conv_operands {
    const paella_conv_plan* plan;
    const float* x;
    const void* blob_dev;
    const float* bias;
    const float* residual;
    const float* slope;
    float* y;
    void* workspace;
} paella_conv_operands;

int paella_conv2d_pair_dims(const paella_conv_plan* first, const paella_conv_plan* second, paella_launch_dims* dims);
/* The same for 2 to PAELLA_CONV_GROUP_MAX convs, one problem's workgroups after the other's in the order given; every
 * pair of members must meet the conditions above. */
#define PAELLA_CONV_GROUP_MAX 4
/* Problems in one launch of the group kernel when the library packs several calls together (below). */
#define PAELLA_CONV_PACK_MAX 8
int paella_conv2d_group_dims(const paella_conv_plan* const* plans, int n, paella_launch_dims* dims);
int paella_conv2d_launch_group(const paella_conv_operands* members, int n, void* stream, uint32_t job_id, void* notifier);

/* Launch packing.  A hardware queue of this device runs one kernel at a time and four run side by side, so at batch 1 a
 * conv that fills a fifth of the compute units still occupies a queue for its whole latency.  After paella_pack_enable(1)
 * on a thread, that thread's paella_conv2d_launch / _launch_group / _launch_group_pool / _launch_transformed calls on the
 * 32 x 32 tile whose target is an UNORDERED direct-dispatch queue (the serving path: the scheduler orders a job's stages through the notification
 * ring) are held back and sent together, up to PAELLA_CONV_PACK_MAX problems of any jobs in one grid, every problem
 * reporting to its own job id and notifier exactly as if launched alone (convs with a fused input transform share launches
 * among themselves, the others among themselves); results are bit-identical.  Everything else
 * (HIP streams, ordered queues, other operators, larger tiles) is launched at once as before.  The thread must call
 * paella_pack_poll() from its loop: it sends what is held as soon as a queue of the shared set (paella_direct_queue_shared)
 * has no packet waiting, when a launch is full, or after 30 us at the latest, on the least loaded queue of that set, and
 * returns the number of launches made (negative: error).  paella_pack_flush() sends everything now;
 * paella_pack_enable(0) flushes and switches packing off.  paella_pack_stats: launches made by the packer and problems
 * they carried so far in this process; returns the number of calls the calling thread currently holds.  No counterpart in the reference
 * (its GPUs run kernels of one stream pool side by side without this limit). */
int paella_pack_enable(int on);
int paella_pack_poll(void);
int paella_pack_flush(void);
void paella_pack_poll_hook(void); /* paella_pack_poll with the signature of a serving-loop hook (llis::job::Context::add_poll_hook) */
int paella_pack_stats(uint64_t* launches, uint64_t* members);

/* The same for a job that issues several dependent launches at once on an ORDERED direct-dispatch queue (a model of
 * small kernels, one scheduler stage): between paella_pack_sequence_begin(key, queue) and paella_pack_sequence_end() the
 * calling thread's paella_conv2d_launch (32 x 32 tile), paella_pool2d_launch and paella_dense_launch calls on `queue` are
 * recorded instead of launched; _end holds the sequence, and sequences recorded under one `key` with the same operators
 * position by position (requests of one model) are later sent together: the k-th launches of up to
 * PAELLA_CONV_PACK_MAX sequences as one grid, position after position on one queue with the barrier bit set.  Any other
 * launch in between ends the recording: what was recorded goes to `queue` at once, the launch follows it, and _end does
 * nothing.  Results are bit-identical.  paella_pack_poll / _flush / _enable(0) send held sequences like held launches.
 * _begin returns PAELLA_ENOSUP when packing is off on the thread or `queue` is not an ordered direct-dispatch queue
 * (the caller then launches as usual). */
int paella_pack_sequence_begin(const void* key, void* queue);
int paella_pack_sequence_end(void);
int paella_conv2d_launch_pair(const paella_conv_operands* first, const paella_conv_operands* second,
                              void* stream, uint32_t job_id, void* notifier);

/* ---------------------------------------------------------------- dense (O3) */

/* y[o] = act(bias[o] + sum_i x[i] * w[o][i]); w is the plain [O][I] row-major matrix. */
int paella_dense_dims(int I, int O, paella_launch_dims* dims);
int paella_dense_launch(const float* x, const float* w, const float* bias, float* y, int I, int O, int act,
                        void* stream, uint32_t job_id, void* notifier);

/* ---------------------------------------------------------------- pooling (O4, O5) */

typedef struct paella_pool_desc {
    int C, H, W;
    int R, S, stride_h, stride_w, pad_h, pad_w;
    int ceil_mode;
    int is_avg;                  /* 0 = max (padding never selected), 1 = average */
    int count_include_pad;       /* average only */
} paella_pool_desc;

int paella_pool_out(int in, int k, int stride, int pad, int ceil_mode);
int paella_pool2d_dims(const paella_pool_desc* d, paella_launch_dims* dims);
int paella_pool2d_launch(const paella_pool_desc* d, const float* x, float* y,
                         void* stream, uint32_t job_id, void* notifier);

/* Up to three such convs (tap-major plans: C a multiple of 8) and one pooling operator in ONE launch: the conv
 * problems' workgroups followed by the pool's, one output element per thread.  An inception module starts with
 * three 1x1 convs and a 3x3 pool that all read the module's input; alone the pool is a launch shorter than the cost of
 * launching it.  No counterpart in the reference (one kernel per fused operator).  The pool must not read or
 * overwrite what a member writes, nor write what a member reads.  Results are bit-identical to separate launches. */
int paella_conv2d_group_pool_dims(const paella_conv_plan* const* plans, int n, const paella_pool_desc* pool, paella_launch_dims* dims);
int paella_conv2d_launch_group_pool(const paella_conv_operands* members, int n, const paella_pool_desc* pool, const float* pool_x,
                                    float* pool_y, void* stream, uint32_t job_id, void* notifier);

/* y[c] = mean over HW of x[c][:] */
int paella_global_avgpool_dims(int C, int HW, paella_launch_dims* dims);
int paella_global_avgpool_launch(const float* x, float* y, int C, int HW,
                                 void* stream, uint32_t job_id, void* notifier);

/* ---------------------------------------------------------------- elementwise (O6), copy (O7) */

/* y = act(a*scale[c] + shift[c] + b): b, scale, shift may be NULL.  Covers residual add(+ReLU),
 * standalone per-channel scale-shift(+ReLU), ReLU, clip and PReLU (slope per channel). */
int paella_eltwise_dims(int C, int HW, paella_launch_dims* dims);
int paella_eltwise_launch(const float* a, const float* b, const float* scale, const float* shift,
                          const float* slope, float* y, int C, int HW, int act, float lo, float hi,
                          void* stream, uint32_t job_id, void* notifier);

/* Plain device copy of n floats (only used where a concat cannot be elided). */
int paella_copy_dims(size_t n, paella_launch_dims* dims);
int paella_copy_launch(const float* x, float* y, size_t n, void* stream, uint32_t job_id, void* notifier);

/* ---------------------------------------------------------------- softmax, LRN (O8) */

int paella_softmax_dims(int rows, int cols, paella_launch_dims* dims);
int paella_softmax_launch(const float* x, float* y, int rows, int cols,
                          void* stream, uint32_t job_id, void* notifier);

int paella_lrn_dims(int C, int HW, paella_launch_dims* dims);
int paella_lrn_launch(const float* x, float* y, int C, int HW, int size, float alpha, float beta, float k,
                      void* stream, uint32_t job_id, void* notifier);

/* Vector registers per thread of a kernel, read from the loaded code object (needs a GPU).
 * family: "dense", "pool", "gap", "eltwise", "copy", "softmax", "lrn". */
int paella_kernel_vgprs(const char* family, unsigned* vgprs);
/* Same for a conv variant: kind 0 = MFMA implicit GEMM with tile (mi, ni, kw), kind 1 = depthwise. */
int paella_conv_kernel_vgprs(int kind, int mi, int ni, int kw, unsigned* vgprs);

/* Workgroups of a kernel that the runtime's occupancy calculator places on one compute unit, for a workgroup of
 * `block` threads with `lds_bytes` of dynamic LDS (needs a GPU).  What the block-level scheduler's resource model
 * (llis::server::SmResources::blocks_per_cu; the reference's counterpart is the budget arithmetic of
 * src/server/sm_resources.cpp:17-66) is checked against.  `form` of a conv: 0 = one conv, 1 = conv on a transformed
 * input, 2 = group of convs, 3 = group of convs with a pooling operator (forms 1 to 3: mi == ni == 1; 1 and 3: k_order 1). */
int paella_kernel_occupancy(const char* family, unsigned block, unsigned lds_bytes, int* blocks_per_cu);
/* Statically allocated LDS of a kernel family, read from the loaded code object (needs a GPU). */
int paella_kernel_static_lds(const char* family, unsigned* lds_bytes);
/* vgprs, static_lds (may be NULL): vector registers per thread and statically allocated LDS of that same kernel, read from
 * the loaded code object; lds_bytes is the dynamic LDS of the launch. */
int paella_conv_kernel_occupancy(int kind, int form, int mi, int ni, int kw, int k_order, unsigned lds_bytes, int* blocks_per_cu,
                                 unsigned* vgprs, unsigned* static_lds);

/*
 * Direct dispatch.  A queue created here is a user-mode hardware queue owned by this library; its handle can
 * be passed wherever a launch function of this header (or paella_exec_launch_stage / paella_exec_forward)
 * takes `void* stream`, and the kernel is then submitted as one AQL packet written by the calling thread
 * instead of going through the HIP launch path (a few hundred nanoseconds instead of 2.3 to 3.9 us of host
 * time).  Kernels submitted to one queue are NOT ordered with respect to each other or to HIP streams: the
 * caller orders dependent work itself, as the serving path does with the notification ring (or with
 * paella_direct_queue_wait).  One producer thread per queue.  Returns PAELLA_ENOSUP when the runtime cannot
 * provide such queues.  No counterpart in the reference: CUDA launches are cheap enough there.
 */
int paella_direct_queue_create(void** queue);
/* ordered != 0: every later kernel waits for all earlier ones of this queue (stream semantics). Default 0. */
int paella_direct_queue_set_ordered(void* queue, int ordered);
/* Blocks until every kernel submitted to the queue so far has finished (at most 10 s: PAELLA_ETIMEDOUT). */
int paella_direct_queue_wait(void* queue);
/* Next of a process-wide set of unordered queues (PAELLA_DIRECT_QUEUES of them, default 4), round-robin.  All
 * callers must be the same thread.  The set lives until the process ends. */
int paella_direct_queue_shared(void** queue);
int paella_direct_queue_destroy(void* queue);

/*
 * Copies `bytes` from src to dst (host memory both) on a helper thread of this library and then calls done(arg) on that
 * thread; returns at once.  For a job's copy of a request's input into its pinned staging buffer (the reference copies
 * straight from the client's pinned pool, reference jobs/tvm_mnist/tvm_mnist.cpp:38; here that pool cannot be pinned, so there
 * is a host-side copy, and on the serving thread it would stop the notification ring from being read for its duration).
 * The helper makes no GPU runtime call.  Copies are done in submission order; done() must be cheap and must not block.
 * Returns PAELLA_EBUSY, with nothing copied and done() not called, when the helper is asleep (it sleeps after half a
 * millisecond without a copy): the caller then copies by itself -- at such rates it has the time, and a wake-up through
 * the kernel would cost a lone request more than the hand-over saves -- and the helper is awake for the copies that follow.
 */
#define PAELLA_EBUSY (-5)  /* not taken now; do it yourself or try again */
int paella_host_copy_submit(void* dst, const void* src, size_t bytes, void (*done)(void*), void* arg);

/*
 * Measurement aid.  While a pair of events (llis_hip_event_create) is armed on the calling thread, every
 * operator launch made by that thread stamps them with the kernel's own begin and end time on the device, so
 * llis_hip_event_elapsed_ms(start, stop) after a stream synchronize is that launch's execution time, the same
 * quantity a kernel trace reports.  Pass NULL, NULL to disarm.  Not for concurrent use of one event pair.
 */
int paella_ops_time_launches(void* start_event, void* stop_event);

#ifdef __cplusplus
}
#endif
#endif
