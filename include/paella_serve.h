/*
 * paella_serve.h -- C-ABI for running the llis server and the load generator INSIDE the calling process.
 *
 * The product binaries are paella_amd/bin/llis_server and llis_app_client (same options as the reference's
 * llis_server and llis_app_client: reference src/server/server.cpp:203-235, app/client.cpp:246-330).  A
 * bench or test harness that has already touched the GPU must not spawn them, so these entry points run
 * exactly the same classes on threads of the caller:
 *   paella_server_start   = main() of llis_server on a new thread (server poll loop)
 *   paella_client_run     = main() of llis_app_client: register jobs, warm every instance, open-loop run
 *   paella_client_single  = closed loop with one instance (reference tests/client/client_single_latency.cpp:16-36)
 *                           that also carries real input bytes in and output bytes out
 * Client and server still talk through the shared-memory rings and the datagram socket.
 * Return value: 0 on success, -1 on error (message on stderr).
 */
#ifndef PAELLA_SERVE_H
#define PAELLA_SERVE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct paella_server paella_server;

typedef struct paella_server_options {
    const char* name;          /* --name */
    const char* sched;         /* --sched: fifo, fifo2, full3 */
    unsigned num_streams;      /* --num_streams */
    unsigned extra_kernels;    /* --extra_kernels */
    float unfair;              /* --unfair */
    unsigned sched_sleep;      /* --sched_sleep */
    int mem_marker;            /* 1: ring-marker kernel reports copy stages, 0: runtime host callback */
    int event_log;             /* 1: record the scheduler event log */
    int cpu;                   /* pin the serving thread to this CPU, -1 = do not pin */
    int measure_block_time;    /* 1: --measure_block_time (per-workgroup entry/exit clocks for the profiler) */
    unsigned noti_batch;       /* --noti_batch: workgroups per aggregated notification, a power of two <= 128; 0 = default (64);
                                  16 = the reference's constant (reference include/llis/job/finished_block_notifier.h:118) */
    int print_ipc_latency;     /* 1: --print_ipc_latency: LAUNCH_JOB carries its send time and the server reports the request ring's mean
                                  latency (the reference's PRINT_LAUNCH_JOB_IPC_LATENCY build, reference src/server/server.cpp:121-141).  The
                                  switch is process-wide: clients of this process send the time from then on; 0 leaves it as it is */
    int placement;             /* --placement: 0 = pooled occupancy budget (the reference's full3), 1 = per_cu: admission against the
                                  per-compute-unit model (include/llis/server/gpu_resources.h; the reference sketches it in
                                  include/llis/server/gpu_resources.h:10-58 and builds it into no scheduler it ships); full3 only */
} paella_server_options;

int paella_server_start(const paella_server_options* options, paella_server** out);
/* Stops the poll loop, joins the thread, destroys scheduler and rings. */
int paella_server_stop(paella_server* server);
/* Text of the event log recorded so far (call after paella_server_stop, or while the server is idle).
 * Copies at most cap bytes including the NUL; returns the full length. */
size_t paella_server_event_log(paella_server* server, char* buf, size_t cap);
/* With print_ipc_latency: mean client-to-server latency of LAUNCH_JOB in microseconds over `*count` requests (the first
 * LLIS_IPC_LATENCY_SKIP requests, 10 000 unless the environment says otherwise, are left out as in the reference).
 * Call while the server runs.  0 on success. */
int paella_server_ipc_latency(paella_server* server, double* mean_us, uint64_t* count);
/* Switches the send time in LAUNCH_JOB off again for this process (after the server that asked for it has stopped). */
void paella_ipc_latency_off(void);

#define PAELLA_MAX_JOB_TYPES 16

typedef struct paella_load_options {
    const char* server_name;
    int num_types;
    const char* job_paths[PAELLA_MAX_JOB_TYPES];
    float proportions[PAELLA_MAX_JOB_TYPES];
    unsigned max_outstanding[PAELLA_MAX_JOB_TYPES];
    double iat_us;             /* mean inter-arrival time; 0 = saturation */
    int dist_exp;              /* 1 exponential (Poisson arrivals), 0 log-normal */
    double ln_sigma;
    int concurrency;           /* global cap on outstanding requests */
    unsigned num_jobs;         /* measured requests */
    unsigned warmup_jobs;      /* served before the clock starts, beyond the one run per pooled instance */
    unsigned seed;
    int pin_threads;           /* pin monitor/submit threads to CPUs 0 and 2 like the reference client */
    const char* profile_prefix; /* non-NULL: server-side recording around the measured phase, saved to this prefix */
    const char* trace_path;    /* non-NULL: replay this "<type> <submit time us>" trace (paella_workload_pregen,
                                  llis_app_workload_pregen; reference tests/utils/workload_pregen.cpp:107) instead of drawing */
    int verify;                /* > 0: verify mode with this many seeded inputs per job type (paella_verify_input): the warm-up runs
                                  every pooled instance alone on the idle server and keeps the first output of every (type, input) pair;
                                  every later completion is compared with it byte for byte before its slot is reused (the reference's
                                  client, app/client.cpp:62-121, checks no output).  0 = off */
    void* verify_expected;     /* optional: receives those expected outputs, [type][input] one after the other */
    size_t verify_expected_bytes; /* capacity of verify_expected */
} paella_load_options;

typedef struct paella_latency_stats {
    double mean, p50, p90, p95, p99, max, sd;
    uint64_t count;
} paella_latency_stats;

typedef struct paella_load_result {
    double elapsed_us;         /* first submission to last completion of the measured requests */
    double throughput_rps;
    paella_latency_stats all;
    paella_latency_stats per_type[PAELLA_MAX_JOB_TYPES];
    unsigned queue_full_events, type_full_events;
    uint64_t verified_requests; /* verify mode: completions compared with their expectation (warm-up included) */
    uint64_t mismatches;        /* ... and how many differed */
} paella_load_result;

/* Element i of input `variant` of job type `type` under arrival seed `seed`, as verify mode writes it into a request slot:
 * floats in [-1, 1).  0 on success. */
int paella_verify_input(unsigned seed, unsigned type, unsigned variant, float* out, size_t n);

/* Writes an arrival trace with the draws of the live generator (type first, then the gap), in the file set of the
 * reference's tool (reference tests/utils/workload_pregen.cpp:72-115): <prefix>_iat<I>_lns<S>_n<N>_seed<K>.txt plus one
 * _job<t>.txt per type.  The combined file's path goes to path_out (capacity cap, NUL-terminated).  0 on success. */
int paella_workload_pregen(double iat_us, int dist_exp, double ln_sigma, unsigned num_jobs, unsigned seed, const char* prefix,
                           const float* proportions, int num_types, char* path_out, size_t cap);

/* latencies_us (optional) receives the measured latencies in completion order; capacity num_jobs. */
int paella_client_run(const paella_load_options* options, paella_load_result* result, double* latencies_us);

/* n closed-loop requests on one instance of job_path; the same input is sent every time and the output
 * of the last request is returned.  latencies_us (optional, capacity n) in microseconds. */
int paella_client_single(const char* server_name, const char* job_path, const void* input, size_t in_bytes, void* output,
                         size_t out_bytes, int n, double* latencies_us);

/*
 * Plain multi-stream serving with no server and no scheduler: `num_streams` HIP streams, each request's whole
 * forward pass (input copy, every kernel back to back, output copy) issued on one free stream by the submitting
 * thread, completion found by polling the streams.  The comparison arm the reference keeps as a stand-alone program
 * (reference tests/simple/tvm_direct_multistream.cpp:143-156,193-301; CUDA-SS with one stream, CUDA-MS with 141,
 * sosp23_artifact/gen_data_fig11_cuda.sh:34-44).  Same arrival process, caps and statistics as paella_client_run.
 */
typedef struct paella_direct_options {
    int num_types;
    const char* models[PAELLA_MAX_JOB_TYPES];     /* zoo model names (paella_models.h), e.g. "mnist", "inception_v3" */
    float proportions[PAELLA_MAX_JOB_TYPES];
    unsigned max_outstanding[PAELLA_MAX_JOB_TYPES]; /* pooled instances per model */
    uint64_t seed_weights;     /* seed of the models' weights (the adapters' LLIS_MODEL_SEED) */
    int num_streams;           /* streams = cap on requests in flight */
    double iat_us;             /* mean inter-arrival time; 0 = saturation */
    int dist_exp;              /* 1 exponential (Poisson arrivals), 0 log-normal */
    double ln_sigma;
    unsigned num_jobs;         /* measured requests */
    unsigned warmup_jobs;      /* served before the clock starts, beyond the one run per pooled instance */
    unsigned seed;             /* of the arrival process */
    int pin_threads;           /* pin monitor/submit threads to CPUs 0 and 2 like the reference */
} paella_direct_options;

int paella_direct_multistream_run(const paella_direct_options* options, paella_load_result* result);

#ifdef __cplusplus
}
#endif
#endif
