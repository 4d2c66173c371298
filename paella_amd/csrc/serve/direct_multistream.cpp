// Plain multi-stream serving without any server or scheduler: N HIP streams, every request's whole forward pass
// (input copy, all kernels back to back, output copy) issued on one stream by the submitting thread, completion
// found by polling the streams.  The comparison arm the reference keeps as a stand-alone program
// (reference tests/simple/tvm_direct_multistream.cpp:143-156 launch_job, :193-247 monitor, :249-301 submit;
// sweep script sosp23_artifact/gen_data_fig11_cuda.sh:34-44), on the same kernels and the same arrival
// process as the served arms (load_generator.h).

#include "paella_serve.h"

#include "load_generator.h"

#include "paella_hip.h"
#include "paella_models.h"

#include <cstdio>
#include <cstring>
#include <deque>
#include <stdexcept>

namespace {

struct Module {  // one pooled request instance of one model
    unsigned type = 0;
    paella_exec* exec = nullptr;
    char* host_in = nullptr;   // pinned
    char* host_out = nullptr;  // pinned
    size_t in_bytes = 0, out_bytes = 0;
    double start_time = 0;
    void* stream = nullptr;    // non-null while in flight
};

void check(int rc, const char* what) {
    if (rc != 0) throw std::runtime_error(std::string(what) + " failed with code " + std::to_string(rc));
}

class DirectRunner {
  public:
    DirectRunner(const paella_direct_options* o) : o_(*o) {
        const int types = o->num_types;
        free_.resize(types);
        due_.resize(types);
        lat_per_type_.resize(types);
        for (int t = 0; t < types; ++t) {
            props_cum_.push_back(o->proportions[t] + (t ? props_cum_.back() : 0.f));
            paella_model* m = nullptr;
            check(paella_model_get(o->models[t], o->seed_weights, &m), "paella_model_get");
            size_t in_b = 0, out_b = 0;
            check(paella_model_io_bytes(o->models[t], &in_b, &out_b), "paella_model_io_bytes");
            for (unsigned i = 0; i < o->max_outstanding[t]; ++i) {
                modules_.emplace_back();
                Module& mod = modules_.back();
                mod.type = (unsigned)t;
                mod.in_bytes = in_b;
                mod.out_bytes = out_b;
                check(paella_exec_create(m, &mod.exec), "paella_exec_create");
                void* p = nullptr;
                check(llis_hip_host_alloc_pinned(&p, in_b + out_b), "llis_hip_host_alloc_pinned");
                mod.host_in = reinterpret_cast<char*>(p);
                mod.host_out = mod.host_in + in_b;
                std::memset(mod.host_in, 0, in_b);
            }
        }
        for (Module& m : modules_) free_[m.type].push_back(&m);  // after the vector stopped growing
        streams_.resize((size_t)o->num_streams);
        for (void*& s : streams_) check(llis_hip_stream_create(&s), "llis_hip_stream_create");
        unused_streams_ = streams_;
    }

    ~DirectRunner() {
        llis_hip_device_synchronize();
        for (void* s : streams_) llis_hip_stream_destroy(s);
        for (Module& m : modules_) {
            if (m.exec) paella_exec_destroy(m.exec);
            if (m.host_in) llis_hip_host_free(m.host_in);
        }
    }

    void run(paella_load_result* result) {
        // every pooled instance once, as the served arms do before the clock starts
        for (Module& m : modules_) {
            issue(&m, streams_[0]);
            check(llis_hip_stream_synchronize(streams_[0]), "warm-up");
            m.stream = nullptr;
        }
        if (o_.warmup_jobs) phase(o_.warmup_jobs, false);
        phase(o_.num_jobs, true);
        std::memset(result, 0, sizeof(*result));
        result->elapsed_us = std::chrono::duration<double, std::micro>(end_time_ - start_time_).count();
        result->throughput_rps = o_.num_jobs / result->elapsed_us * 1e6;
        result->queue_full_events = num_queue_full_;
        result->type_full_events = num_type_full_;
        fill(&result->all, lat_);
        for (size_t t = 0; t < lat_per_type_.size(); ++t) fill(&result->per_type[t], lat_per_type_[t]);
    }

  private:
    static void fill(paella_latency_stats* out, std::vector<double>& v) {
        const llis::loadgen::Stats s = llis::loadgen::summarize(v);
        out->mean = s.mean; out->p50 = s.p50; out->p90 = s.p90; out->p95 = s.p95; out->p99 = s.p99; out->max = s.max; out->sd = s.sd;
        out->count = v.size();
    }

    // The whole request on one stream; the caller holds mtx_ (or runs alone).
    void issue(Module* m, void* stream) {
        check(llis_hip_memcpy_async(paella_exec_input(m->exec), m->host_in, m->in_bytes, LLIS_HIP_H2D, stream), "input copy");
        check(paella_exec_forward(m->exec, stream), "paella_exec_forward");
        check(llis_hip_memcpy_async(m->host_out, paella_exec_output(m->exec), m->out_bytes, LLIS_HIP_D2H, stream), "output copy");
        // Published last: the monitor scans without the lock and takes "stream set and idle" for "request done".  Set before the
        // work is on the stream (where the reference sets it, reference tests/simple/tvm_direct_multistream.cpp:143-156) an idle
        // stream would pass for a finished request of no latency, and the instance would be handed out again while this thread
        // still issues onto it.
        __atomic_store_n(&m->stream, stream, __ATOMIC_RELEASE);
    }

    void launch(unsigned type, double scheduled_arrival_us) {
        Module* m = free_[type].back();
        free_[type].pop_back();
        void* s = unused_streams_.back();
        unused_streams_.pop_back();
        m->start_time = scheduled_arrival_us;
        issue(m, s);
    }

    void phase(unsigned num_jobs, bool record) {
        phase_jobs_ = num_jobs;
        phase_record_ = record;
        num_outstanding_.store(0);
        std::thread monitor_thr([this] { monitor(); });
        std::thread submit_thr([this] { submit(); });
        if (o_.pin_threads) {
            pin(monitor_thr, 0);
            pin(submit_thr, 2);
        }
        monitor_thr.join();
        submit_thr.join();
    }

    static void pin(std::thread& thr, int cpu) {
        cpu_set_t set;
        CPU_ZERO(&set);
        CPU_SET(cpu, &set);
        pthread_setaffinity_np(thr.native_handle(), sizeof(set), &set);
    }

    void monitor() {
        using llis::loadgen::Clock;
        for (unsigned done = 0; done < phase_jobs_; ++done) {
            Module* mod = nullptr;
            do {  // scan every instance in flight, as the reference's monitor does
                for (Module& m : modules_) {
                    void* s = __atomic_load_n(&m.stream, __ATOMIC_ACQUIRE);
                    if (s && llis_hip_stream_busy(s) == 0) {
                        mod = &m;
                        break;
                    }
                }
            } while (!mod);
            const double latency = llis::loadgen::us_since_epoch(Clock::now()) - mod->start_time;
            const unsigned type = mod->type;
            {
                std::lock_guard<std::mutex> lk(mtx_);
                free_[type].push_back(mod);
                unused_streams_.push_back(mod->stream);
                __atomic_store_n(&mod->stream, (void*)nullptr, __ATOMIC_RELEASE);
                num_outstanding_.fetch_sub(1, std::memory_order_release);
                while (!due_[type].empty() && !free_[type].empty() && !unused_streams_.empty()) {
                    launch(type, due_[type].front());
                    due_[type].pop();
                }
            }
            if (phase_record_) {
                lat_.push_back(latency);
                lat_per_type_[type].push_back(latency);
            }
        }
        end_time_ = Clock::now();
    }

    void submit() {
        using llis::loadgen::Clock;
        std::mt19937 gen(o_.seed);
        std::exponential_distribution<> d_exp(o_.iat_us > 0 ? 1. / o_.iat_us : 1.);
        const double mu = o_.iat_us > 0 ? std::log(o_.iat_us) - o_.ln_sigma * o_.ln_sigma / 2 : 0;
        std::lognormal_distribution<> d_ln(mu, o_.ln_sigma);
        std::uniform_real_distribution<float> d_type(0, 1);
        double next_submit = 0;
        start_time_ = Clock::now();
        const double start_us = llis::loadgen::us_since_epoch(start_time_);
        for (unsigned submitted = 0; submitted < phase_jobs_;) {
            const double elapsed = std::chrono::duration<double, std::micro>(Clock::now() - start_time_).count();
            if (elapsed < next_submit) continue;
            // one stream per request in flight: the stream count is the cap on outstanding requests
            if (num_outstanding_.load(std::memory_order_acquire) >= o_.num_streams) {
                ++num_queue_full_;
                while (num_outstanding_.load(std::memory_order_acquire) >= o_.num_streams) {
                }
            }
            const unsigned type = std::min<unsigned>((unsigned)(std::lower_bound(props_cum_.begin(), props_cum_.end(), d_type(gen)) - props_cum_.begin()),
                                                     (unsigned)props_cum_.size() - 1);
            {
                std::lock_guard<std::mutex> lk(mtx_);
                if (free_[type].empty()) {
                    ++num_type_full_;
                    due_[type].push(start_us + next_submit);
                } else {
                    launch(type, start_us + next_submit);
                }
            }
            num_outstanding_.fetch_add(1, std::memory_order_release);
            ++submitted;
            if (o_.iat_us > 0) next_submit += o_.dist_exp ? d_exp(gen) : d_ln(gen);
        }
    }

    const paella_direct_options o_;
    std::vector<float> props_cum_;
    std::deque<Module> modules_;
    std::vector<std::vector<Module*>> free_;
    std::vector<std::queue<double>> due_;
    std::vector<void*> streams_, unused_streams_;
    std::mutex mtx_;
    std::atomic<int> num_outstanding_{0};
    std::vector<double> lat_;
    std::vector<std::vector<double>> lat_per_type_;
    llis::loadgen::Clock::time_point start_time_, end_time_;
    unsigned num_queue_full_ = 0, num_type_full_ = 0, phase_jobs_ = 0;
    bool phase_record_ = true;
};

}  // namespace

extern "C" int paella_direct_multistream_run(const paella_direct_options* o, paella_load_result* result) {
    if (!o || !result || o->num_types <= 0 || o->num_types > PAELLA_MAX_JOB_TYPES || o->num_streams <= 0 || o->num_jobs == 0) return -1;
    for (int t = 0; t < o->num_types; ++t)
        if (!o->models[t] || o->max_outstanding[t] == 0) return -1;
    try {
        DirectRunner runner(o);
        runner.run(result);
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "paella_direct_multistream_run: %s\n", e.what());
        return -1;
    }
}
