#pragma once
// Open-loop load generator and latency statistics shared by llis_app_client and the in-process bench
// entry points.  Arrival and statistics arithmetic reproduce reference app/client.cpp:50-212:
//   * std::mt19937 seeded with `seed`; per request FIRST the job type is drawn
//     (std::uniform_real_distribution<float>(0,1), lower_bound on cumulative proportions), THEN the next
//     inter-arrival time (log-normal with mu = ln(mean) - sigma^2/2, or exponential with rate 1/mean);
//   * a request whose type has no free instance is queued with its DUE time and launched by the monitor
//     when an instance of that type returns; a global cap `concurrency` blocks the submitter;
//   * latency = completion time - scheduled arrival time; percentiles are sorted[size * q] (truncated).
// iat == 0 submits as fast as the caps allow (saturation).
//
// Verify mode (Options::verify_variants > 0; the reference's client checks no output at all): every pooled instance carries one
// of `verify_variants` seeded inputs of its job type (verify_input below), the warm-up runs the instances ONE AT A TIME on the
// otherwise idle server and keeps the first output of every (type, variant) as that pair's expectation, and from then on every
// completion -- warm-up, measured, whatever shared a launch with whatever -- is compared with its expectation byte for byte
// before its slot is handed out again; the slot's output area is overwritten with 0xFF bytes before each launch, so a request
// that was never answered cannot pass on its predecessor's bytes.

#include <llis/client/client.h>
#include <llis/client/job_instance_ref.h>
#include <llis/client/job_ref.h>

#include <pthread.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <mutex>
#include <queue>
#include <random>
#include <string>
#include <thread>
#include <vector>

namespace llis {
namespace loadgen {

using Clock = std::chrono::steady_clock;

inline double us_since_epoch(Clock::time_point t) { return std::chrono::duration<double, std::micro>(t.time_since_epoch()).count(); }

struct Stats {
    double mean = 0, p50 = 0, p90 = 0, p95 = 0, p99 = 0, max = 0, sd = 0;
};

inline Stats summarize(std::vector<double>& v) {
    Stats s;
    if (v.empty()) return s;
    std::sort(v.begin(), v.end());
    const double n = (double)v.size();
    double mean = 0, mean_sqr = 0;
    for (double x : v) {
        mean += x / n;
        mean_sqr += x * x / n;
    }
    s.mean = mean;
    s.sd = v.size() > 1 ? std::sqrt((mean_sqr - mean * mean) * (n / (n - 1))) : 0;
    s.p50 = v[v.size() / 2];
    s.p90 = v[(size_t)(n * 0.90)];
    s.p95 = v[(size_t)(n * 0.95)];
    s.p99 = v[(size_t)(n * 0.99)];
    s.max = v.back();
    return s;
}

// Element i of the seeded input of (seed, job type, variant): 24 bits of splitmix64's output function over a counter, mapped
// to [-1, 1).  paella_amd/serve.py restates it in numpy (tests compare the two bit for bit and derive the expected model outputs from it).
inline uint64_t verify_mix(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline void verify_input(unsigned seed, unsigned type, unsigned variant, float* out, size_t n) {
    const uint64_t base = ((uint64_t)seed << 40) ^ ((uint64_t)type << 32) ^ ((uint64_t)variant << 24);
    for (size_t i = 0; i < n; ++i) out[i] = (float)(verify_mix(base + i) >> 40) * (1.0f / 8388608.0f) - 1.0f;
}

struct Mismatch {
    unsigned type = 0, variant = 0;
    size_t offset = 0;        // first differing byte of the output
    uint64_t request = 0;     // how many completions had been checked before it
};

struct Options {
    std::string server_name, prefix = "llis_client", dist = "ln";
    double iat = -1, ln_sigma = 2.0, fairness = -1;
    int concurrency = -1;
    unsigned num_jobs = 0, start_record_num = 0, seed = 1, sched_sleep = 0;
    unsigned warmup_jobs = 0;  // extra requests served (same arrival process) before the measured ones
    bool pin_threads = true;
    std::string trace_path;      // non-empty: replay "<type> <submit time us>" lines (llis_app_workload_pregen) instead of drawing
    std::string profile_prefix;  // non-empty: the server records everything during the measured phase and saves to this prefix
    unsigned verify_variants = 0;  // > 0: verify mode with this many distinct inputs per job type
    // name-shaping switches (which parameters appear in the output file names, which one is the x column)
    bool n_iat = false, n_lns = false, n_con = false, n_n = false, n_srn = false, n_seed = false, n_fair = false, n_scheds = false;
    bool g_iat = false, g_lns = false, g_con = false, g_n = false, g_srn = false, g_seed = false, g_fair = false, g_scheds = false;
};

class LoadGenerator {
  public:
    LoadGenerator(llis::client::Client* client, const Options& opt, std::vector<float> props_cum, std::vector<unsigned> max_outstanding)
        : client_(client), opt_(opt), props_cum_(std::move(props_cum)), max_outstanding_(std::move(max_outstanding)) {
        const size_t types = props_cum_.size();
        free_instances_.resize(types);
        free_counts_ = std::vector<std::atomic<unsigned>>(types);
        due_.resize(types);
        outstanding_per_type_.assign(types, 0);
        latencies_per_type_.resize(types);
    }

    void add_instance(unsigned type, llis::client::JobInstanceRef* inst) {
        free_instances_[type].push_back(inst);
        // Job reference ids are handed out server-wide, so they equal the type index only for the first client of a
        // server (which is what reference app/client.cpp:77 relies on); keep the mapping instead.
        const unsigned ref = inst->get_job_ref_id();
        if (ref >= type_of_ref_.size()) type_of_ref_.resize(ref + 1, 0);
        type_of_ref_[ref] = type;
    }

    // Creates every pooled instance and runs it once before the clock starts (reference app/client.cpp:425-448 launches them
    // all and then waits).  In verify mode the runs go one at a time, so the first output of every (type, variant) is what an
    // idle server answers; the others of the same pair are already held against it.
    void warm_up(std::vector<llis::client::JobRef>& job_refs) {
        const unsigned variants = opt_.verify_variants;
        if (variants) {
            expected_.assign(job_refs.size(), std::vector<std::vector<char>>(variants));
            in_size_.clear();
            out_size_.clear();
            for (auto& ref : job_refs) {
                in_size_.push_back(ref.get_job()->get_input_size());
                out_size_.push_back(ref.get_job()->get_output_size());
            }
        }
        unsigned total = 0;
        for (unsigned t = 0; t < job_refs.size(); ++t) {
            for (unsigned i = 0; i < max_outstanding_[t]; ++i) {
                llis::client::JobInstanceRef* inst = job_refs[t].create_instance();
                const size_t in_bytes = job_refs[t].get_job()->get_input_size();
                std::memset(inst->get_input_ptr(), 0, in_bytes);
                add_instance(t, inst);
                if (!variants) {
                    inst->launch();
                    ++total;
                    continue;
                }
                const unsigned v = i % variants;
                variant_of_[inst] = v;
                verify_input(opt_.seed, t, v, static_cast<float*>(inst->get_input_ptr()), in_bytes / sizeof(float));
                std::memset(inst->get_output_ptr(), 0xFF, out_size_[t]);
                inst->launch();
                if (client_->wait() != inst) throw std::runtime_error("verify warm-up: a completion for another instance");
                std::vector<char>& want = expected_[t][v];
                if (want.empty() && out_size_[t]) {
                    want.assign(static_cast<char*>(inst->get_output_ptr()), static_cast<char*>(inst->get_output_ptr()) + out_size_[t]);
                } else {
                    check(inst, t);
                }
            }
        }
        for (unsigned i = 0; i < total; ++i) client_->wait();
        if (variants) {
            // ... and once more all at once, as the reference's warm-up does: the server builds a pooled job instance of its own
            // for every request in flight (device arena, workspace, weights on first use), which the one-at-a-time pass above
            // never made it do; left to the measured phase that would be allocations inside the timed region.
            std::vector<std::pair<llis::client::JobInstanceRef*, unsigned>> all;
            for (unsigned t = 0; t < free_instances_.size(); ++t)
                for (llis::client::JobInstanceRef* inst : free_instances_[t]) all.emplace_back(inst, t);
            for (auto& it : all) {
                if (out_size_[it.second]) std::memset(it.first->get_output_ptr(), 0xFF, out_size_[it.second]);
                it.first->launch();
            }
            for (size_t i = 0; i < all.size(); ++i) {
                llis::client::JobInstanceRef* inst = client_->wait();
                check(inst, type_of_ref_[inst->get_job_ref_id()]);
            }
        }
        publish_free_counts();
    }

    uint64_t verified() const { return verified_; }
    uint64_t mismatches() const { return mismatches_; }
    const std::vector<Mismatch>& first_mismatches() const { return first_mismatches_; }
    // Expected outputs, [type][variant] one after the other (each type's output size); returns the bytes written.
    size_t copy_expected(void* dst, size_t cap) const {
        size_t at = 0;
        for (const auto& type : expected_)
            for (const auto& e : type) {
                if (at + e.size() > cap) return at;
                std::memcpy(static_cast<char*>(dst) + at, e.data(), e.size());
                at += e.size();
            }
        return at;
    }

    void publish_free_counts() {
        for (size_t t = 0; t < free_instances_.size(); ++t) free_counts_[t].store((unsigned)free_instances_[t].size(), std::memory_order_release);
    }

    void run() {
        if (opt_.warmup_jobs) phase(opt_.warmup_jobs, false);
        // Server-side recording around the measured phase (the reference keeps these calls commented out in
        // its monitor thread, reference app/client.cpp:101-121).
        llis::client::ProfilerClient* prof = opt_.profile_prefix.empty() ? nullptr : client_->get_profiler_client();
        if (prof) {
            prof->set_record_kernel_info();
            prof->set_record_block_exec_time();
            prof->set_record_kernel_block_mis_alloc();
            prof->set_record_run_next_times();
            prof->set_record_job_events();
            prof->set_record_resource_events();
        }
        phase(opt_.num_jobs, true);
        if (prof) {
            prof->unset_record_kernel_info();
            prof->unset_record_block_exec_time();
            prof->unset_record_kernel_block_mis_alloc();
            prof->unset_record_run_next_times();
            prof->unset_record_job_events();
            prof->unset_record_resource_events();
            prof->save(opt_.profile_prefix);
        }
    }

    double elapsed_us() const { return std::chrono::duration<double, std::micro>(end_time_ - start_time_).count(); }
    std::vector<double>& latencies() { return latencies_; }
    std::vector<std::vector<double>>& latencies_per_type() { return latencies_per_type_; }
    const std::vector<unsigned>& timeline() const { return timeline_; }
    unsigned queue_full_events() const { return num_queue_full_; }
    unsigned type_full_events() const { return num_type_full_; }

  private:
    void phase(unsigned num_jobs, bool record) {
        phase_jobs_ = num_jobs;
        phase_record_ = record;
        std::thread monitor_thr([this] { monitor(); });
        std::thread submit_thr([this] { submit(); });
        if (opt_.pin_threads) {
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
        pthread_setaffinity_np(thr.native_handle(), sizeof(set), &set);  // best effort
    }

    void sample_timeline(double t) {
        timeline_.push_back((unsigned)t);
        for (unsigned n : outstanding_per_type_) timeline_.push_back(n);
    }

    // Caller holds mtx_.
    void launch(unsigned type, double scheduled_arrival_us) {
        free_counts_[type].fetch_sub(1, std::memory_order_release);
        llis::client::JobInstanceRef* inst = free_instances_[type].back();
        free_instances_[type].pop_back();
        ++outstanding_per_type_[type];
        inst->set_start_time(scheduled_arrival_us);
        if (opt_.verify_variants && out_size_[type]) std::memset(inst->get_output_ptr(), 0xFF, out_size_[type]);
        inst->launch();
    }

    // The monitor thread (or the warm-up) compares a completed instance's output with its expectation.
    void check(llis::client::JobInstanceRef* inst, unsigned type) {
        const std::vector<char>& want = expected_[type][variant_of_[inst]];
        ++verified_;
        if (want.empty() || std::memcmp(inst->get_output_ptr(), want.data(), want.size()) == 0) return;
        ++mismatches_;
        if (first_mismatches_.size() < 8) {
            Mismatch m;
            m.type = type;
            m.variant = variant_of_[inst];
            m.request = verified_ - 1;
            const char* got = static_cast<const char*>(inst->get_output_ptr());
            while (m.offset < want.size() && got[m.offset] == want[m.offset]) ++m.offset;
            first_mismatches_.push_back(m);
        }
    }

    void monitor() {
        const auto very_start = Clock::now();
        for (unsigned done = 0; done < phase_jobs_; ++done) {
            llis::client::JobInstanceRef* inst = client_->wait();
            const auto now = Clock::now();
            const double latency = us_since_epoch(now) - inst->get_start_time();
            const double t = std::chrono::duration<double, std::micro>(now - very_start).count();
            const unsigned type = type_of_ref_[inst->get_job_ref_id()];
            if (opt_.verify_variants) check(inst, type);
            {
                std::lock_guard<std::mutex> lk(mtx_);
                free_instances_[type].push_back(inst);
                free_counts_[type].fetch_add(1, std::memory_order_release);
                --outstanding_per_type_[type];
                sample_timeline(t);
                num_outstanding_.fetch_sub(1, std::memory_order_release);
                while (!due_[type].empty() && !free_instances_[type].empty()) {
                    launch(type, due_[type].front());
                    due_[type].pop();
                }
            }
            if (phase_record_ && done >= opt_.start_record_num) {
                latencies_.push_back(latency);
                latencies_per_type_[type].push_back(latency);
            }
        }
        end_time_ = Clock::now();
    }

    void submit() {
        std::mt19937 gen(opt_.seed);
        std::exponential_distribution<> d_exp(opt_.iat > 0 ? 1. / opt_.iat : 1.);
        const double mu = opt_.iat > 0 ? std::log(opt_.iat) - opt_.ln_sigma * opt_.ln_sigma / 2 : 0;
        std::lognormal_distribution<> d_ln(mu, opt_.ln_sigma);
        std::uniform_real_distribution<float> d_type(0, 1);
        const bool use_exp = opt_.dist == "exp";

        // A pre-generated trace replaces the draws: request i is of trace_[i].first and due at trace_[i].second.
        if (!opt_.trace_path.empty() && trace_.empty()) {
            if (FILE* fp = std::fopen(opt_.trace_path.c_str(), "r")) {
                unsigned type;
                double when;
                while (std::fscanf(fp, "%u %lf", &type, &when) == 2) trace_.emplace_back(type, when);
                std::fclose(fp);
            }
            if (trace_.empty()) throw std::runtime_error("cannot read arrival trace " + opt_.trace_path);
        }
        const bool replay = !trace_.empty();
        size_t trace_pos = 0;

        double next_submit = replay ? trace_[0].second : 0;
        start_time_ = Clock::now();
        const double start_us = us_since_epoch(start_time_);
        unsigned submitted = 0;

        while (submitted < phase_jobs_) {
            const double elapsed = std::chrono::duration<double, std::micro>(Clock::now() - start_time_).count();
            if (elapsed < next_submit) continue;

            if (num_outstanding_.load(std::memory_order_acquire) >= opt_.concurrency) {
                ++num_queue_full_;
                while (num_outstanding_.load(std::memory_order_acquire) >= opt_.concurrency) {
                }
            }
            const unsigned type = replay ? trace_[trace_pos % trace_.size()].first
                                         : (unsigned)(std::lower_bound(props_cum_.begin(), props_cum_.end(), d_type(gen)) - props_cum_.begin());
            const unsigned t = std::min<unsigned>(type, (unsigned)props_cum_.size() - 1);
            {
                std::lock_guard<std::mutex> lk(mtx_);
                if (free_counts_[t].load(std::memory_order_acquire) == 0) {
                    ++num_type_full_;
                    due_[t].push(start_us + next_submit);
                } else {
                    launch(t, start_us + next_submit);
                    sample_timeline(elapsed);
                }
            }
            num_outstanding_.fetch_add(1, std::memory_order_release);
            ++submitted;
            if (replay) {
                // the trace wraps around (shifted by its own span) when more requests are asked for than it holds
                ++trace_pos;
                const double span = trace_.back().second + (trace_.size() > 1 ? trace_.back().second / (double)(trace_.size() - 1) : 0);
                next_submit = trace_[trace_pos % trace_.size()].second + span * (double)(trace_pos / trace_.size());
            } else if (opt_.iat > 0) {
                next_submit += use_exp ? d_exp(gen) : d_ln(gen);
            }
        }
    }

    llis::client::Client* client_;
    const Options& opt_;
    std::vector<float> props_cum_;
    std::vector<unsigned> max_outstanding_;

    std::mutex mtx_;
    std::vector<std::vector<llis::client::JobInstanceRef*>> free_instances_;
    std::vector<std::atomic<unsigned>> free_counts_;
    std::vector<std::queue<double>> due_;
    std::vector<unsigned> outstanding_per_type_;
    std::atomic<int> num_outstanding_{0};

    std::vector<unsigned> type_of_ref_;
    std::vector<std::pair<unsigned, double>> trace_;
    std::vector<double> latencies_;
    std::vector<std::vector<double>> latencies_per_type_;
    std::vector<unsigned> timeline_;
    Clock::time_point start_time_, end_time_;
    unsigned num_queue_full_ = 0, num_type_full_ = 0;
    unsigned phase_jobs_ = 0;
    bool phase_record_ = true;

    // verify mode
    std::vector<std::vector<std::vector<char>>> expected_;  // [type][variant]
    std::vector<size_t> in_size_, out_size_;
    std::map<llis::client::JobInstanceRef*, unsigned> variant_of_;
    uint64_t verified_ = 0, mismatches_ = 0;
    std::vector<Mismatch> first_mismatches_;
};


}  // namespace loadgen
}  // namespace llis
