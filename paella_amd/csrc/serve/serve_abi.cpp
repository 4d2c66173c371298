// In-process server and load generator behind include/paella_serve.h.

#include "paella_serve.h"

#include "load_generator.h"
#include "workload_pregen.h"

#include <llis/ipc/defs.h>
#include <llis/server/scheduler.h>
#include <llis/server/server.h>

#include "paella_hip.h"

#include <pthread.h>

#include <cstdio>
#include <cstring>
#include <exception>
#include <memory>
#include <string>
#include <thread>

struct paella_server {
    std::unique_ptr<llis::server::Scheduler> scheduler;
    std::unique_ptr<llis::server::Server> server;
    std::thread thread;
    std::string log_text;
    bool stopped = false;
};

namespace {

void fill(paella_latency_stats* out, std::vector<double>& v) {
    const llis::loadgen::Stats s = llis::loadgen::summarize(v);
    out->mean = s.mean; out->p50 = s.p50; out->p90 = s.p90; out->p95 = s.p95; out->p99 = s.p99; out->max = s.max; out->sd = s.sd;
    out->count = v.size();
}

}  // namespace

extern "C" {

int paella_server_start(const paella_server_options* o, paella_server** out) {
    if (!o || !out || !o->name || !o->sched) return -1;
    try {
        llis::server::SchedulerOptions so;
        if (o->num_streams) so.num_streams = o->num_streams;
        so.extra_kernels = o->extra_kernels;
        if (o->unfair > 0) so.unfair = o->unfair;
        so.sched_sleep = o->sched_sleep;
        so.mem_marker = o->mem_marker != 0;
        so.measure_block_time = o->measure_block_time != 0;
        so.noti_batch = o->noti_batch;
        so.per_cu_placement = o->placement == 1;
        if (so.per_cu_placement && std::string(o->sched) != "full3") return -1;
        if (o->print_ipc_latency) llis::ipc::set_launch_timestamps(true);
        auto s = std::make_unique<paella_server>();
        s->scheduler = llis::server::SchedulerFactory::create(o->sched, so);
        s->server = std::make_unique<llis::server::Server>(o->name, s->scheduler.get());
        if (o->event_log) s->server->get_event_log()->enable(true);
        llis::server::Server* srv = s->server.get();
        s->thread = std::thread([srv] {
            try {
                srv->serve();
            } catch (const std::exception& e) {
                std::fprintf(stderr, "[llis] server thread died: %s\n", e.what());
            }
        });
        if (o->cpu >= 0) {
            cpu_set_t set;
            CPU_ZERO(&set);
            CPU_SET(o->cpu, &set);
            pthread_setaffinity_np(s->thread.native_handle(), sizeof(set), &set);
        }
        *out = s.release();
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "paella_server_start: %s\n", e.what());
        return -1;
    }
}

int paella_server_stop(paella_server* s) {
    if (!s) return -1;
    if (!s->stopped) {
        s->server->request_stop();
        if (s->thread.joinable()) s->thread.join();
        s->log_text = s->server->get_event_log()->to_text();
        s->server.reset();
        s->scheduler.reset();
        s->stopped = true;
    }
    return 0;
}

int paella_server_ipc_latency(paella_server* s, double* mean_us, uint64_t* count) {
    if (!s || s->stopped || !mean_us || !count) return -1;
    *mean_us = s->server->ipc_latency_mean_us();
    *count = s->server->ipc_latency_count();
    return 0;
}

void paella_ipc_latency_off(void) { llis::ipc::set_launch_timestamps(false); }

size_t paella_server_event_log(paella_server* s, char* buf, size_t cap) {
    if (!s) return 0;
    const std::string text = s->stopped ? s->log_text : s->server->get_event_log()->to_text();
    if (buf && cap) {
        const size_t n = text.size() < cap - 1 ? text.size() : cap - 1;
        std::memcpy(buf, text.data(), n);
        buf[n] = 0;
    }
    return text.size();
}

int paella_client_run(const paella_load_options* o, paella_load_result* result, double* latencies_us) {
    if (!o || !result || !o->server_name || o->num_types <= 0 || o->num_types > PAELLA_MAX_JOB_TYPES || o->concurrency <= 0 || o->num_jobs == 0)
        return -1;
    try {
        llis::loadgen::Options opt;
        opt.server_name = o->server_name;
        opt.iat = o->iat_us;
        opt.dist = o->dist_exp ? "exp" : "ln";
        opt.ln_sigma = o->ln_sigma;
        opt.concurrency = o->concurrency;
        opt.num_jobs = o->num_jobs;
        opt.warmup_jobs = o->warmup_jobs;
        opt.seed = o->seed;
        opt.pin_threads = o->pin_threads != 0;
        if (o->profile_prefix) opt.profile_prefix = o->profile_prefix;
        if (o->trace_path) opt.trace_path = o->trace_path;
        opt.verify_variants = o->verify > 0 ? (unsigned)o->verify : 0;

        std::vector<float> props_cum;
        std::vector<unsigned> max_outstanding;
        for (int t = 0; t < o->num_types; ++t) {
            props_cum.push_back(o->proportions[t] + (t ? props_cum.back() : 0.f));
            max_outstanding.push_back(o->max_outstanding[t]);
        }

        llis::client::Client client(o->server_name);
        std::vector<llis::client::JobRef> job_refs;
        job_refs.reserve((size_t)o->num_types);
        for (int t = 0; t < o->num_types; ++t) job_refs.push_back(client.register_job(o->job_paths[t]));

        llis::loadgen::LoadGenerator gen(&client, opt, props_cum, max_outstanding);
        gen.warm_up(job_refs);
        gen.run();

        std::memset(result, 0, sizeof(*result));
        result->elapsed_us = gen.elapsed_us();
        result->throughput_rps = o->num_jobs / result->elapsed_us * 1e6;
        result->queue_full_events = gen.queue_full_events();
        result->type_full_events = gen.type_full_events();
        result->verified_requests = gen.verified();
        result->mismatches = gen.mismatches();
        for (const llis::loadgen::Mismatch& m : gen.first_mismatches())
            std::fprintf(stderr, "paella_client_run: output mismatch at checked completion %llu: job type %u, input variant %u, first differing byte %zu\n",
                         (unsigned long long)m.request, m.type, m.variant, m.offset);
        if (o->verify > 0 && o->verify_expected) gen.copy_expected(o->verify_expected, o->verify_expected_bytes);
        if (latencies_us) std::copy(gen.latencies().begin(), gen.latencies().end(), latencies_us);
        fill(&result->all, gen.latencies());
        for (int t = 0; t < o->num_types; ++t) fill(&result->per_type[t], gen.latencies_per_type()[t]);
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "paella_client_run: %s\n", e.what());
        return -1;
    }
}

int paella_verify_input(unsigned seed, unsigned type, unsigned variant, float* out, size_t n) {
    if (!out) return -1;
    llis::loadgen::verify_input(seed, type, variant, out, n);
    return 0;
}

int paella_workload_pregen(double iat_us, int dist_exp, double ln_sigma, unsigned num_jobs, unsigned seed, const char* prefix,
                           const float* proportions, int num_types, char* path_out, size_t cap) {
    if (iat_us <= 0 || num_jobs == 0 || !prefix || !proportions || num_types <= 0 || !path_out || cap == 0) return -1;
    std::vector<float> props_cum;
    for (int t = 0; t < num_types; ++t) props_cum.push_back(proportions[t] + (t ? props_cum.back() : 0.f));
    const std::string path = llis::loadgen::write_pregen_trace(iat_us, dist_exp != 0, ln_sigma, num_jobs, seed, prefix, props_cum);
    if (path.empty() || path.size() + 1 > cap) return -1;
    std::memcpy(path_out, path.c_str(), path.size() + 1);
    return 0;
}

int paella_client_single(const char* server_name, const char* job_path, const void* input, size_t in_bytes, void* output, size_t out_bytes,
                         int n, double* latencies_us) {
    if (!server_name || !job_path || n <= 0) return -1;
    try {
        llis::client::Client client(server_name);
        llis::client::JobRef job = client.register_job(job_path);
        if (in_bytes > job.get_job()->get_input_size() || out_bytes > job.get_job()->get_output_size()) return -1;
        llis::client::JobInstanceRef* inst = job.create_instance();
        std::memset(inst->get_input_ptr(), 0, job.get_job()->get_input_size());
        if (input) std::memcpy(inst->get_input_ptr(), input, in_bytes);
        for (int i = 0; i < n; ++i) {
            const auto t0 = std::chrono::steady_clock::now();
            inst->launch();
            llis::client::JobInstanceRef* done = client.wait();
            const auto t1 = std::chrono::steady_clock::now();
            if (done != inst) return -1;
            if (latencies_us) latencies_us[i] = std::chrono::duration<double, std::micro>(t1 - t0).count();
        }
        if (output) std::memcpy(output, inst->get_output_ptr(), out_bytes);
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "paella_client_single: %s\n", e.what());
        return -1;
    }
}

}  // extern "C"
