// llis_app_client -- open-loop load generator and latency recorder.
//
//   llis_app_client --server_name S --iat MEAN_US [--dist exp|ln] [--ln_sigma SIGMA] --concurrency C
//                   --num_jobs N [--start_record_num R] --seed SEED --prefix OUT
//                   job.so proportion max_outstanding [job.so proportion max_outstanding ...]
//
// Arrival and statistics arithmetic reproduce reference app/client.cpp:50-212 so runs are comparable:
//   * std::mt19937 seeded with --seed; per request FIRST the job type is drawn
//     (std::uniform_real_distribution<float>(0,1), lower_bound on cumulative proportions), THEN the next
//     inter-arrival time (log-normal with mu = ln(mean) - sigma^2/2, or exponential with rate 1/mean);
//   * a request whose type has no free instance is queued with its DUE time and launched by the monitor
//     when an instance of that type returns; a global cap --concurrency blocks the submitter;
//   * latency = completion time - scheduled arrival time; percentiles are sorted[size * q] (truncated);
//   * every pooled instance is run once as warm-up before the clock starts;
//   * <prefix>.txt gets one CSV row: x,num_jobs,elapsed_us, then mean,p50,p90,p95,p99,max,sd overall and
//     per type; <prefix>_raw.txt all latencies; <prefix>_timeline.txt outstanding-per-type samples.
// --iat 0 submits as fast as the caps allow (saturation).  A one-line JSON summary goes to stdout.

#include <llis/client/client.h>
#include <llis/client/job_instance_ref.h>
#include <llis/client/job_ref.h>

#include <getopt.h>
#include <pthread.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <queue>
#include <random>
#include <sstream>
#include <string>
#include <thread>
#include <vector>

namespace {

using Clock = std::chrono::steady_clock;

double us_since_epoch(Clock::time_point t) { return std::chrono::duration<double, std::micro>(t.time_since_epoch()).count(); }

struct Stats {
    double mean = 0, p50 = 0, p90 = 0, p95 = 0, p99 = 0, max = 0, sd = 0;
};

Stats summarize(std::vector<double>& v) {
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

struct Options {
    std::string server_name, prefix = "llis_client", dist = "ln";
    double iat = -1, ln_sigma = 2.0, fairness = -1;
    int concurrency = -1;
    unsigned num_jobs = 0, start_record_num = 0, seed = 1, sched_sleep = 0;
    bool pin_threads = true;
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

    void add_instance(unsigned type, llis::client::JobInstanceRef* inst) { free_instances_[type].push_back(inst); }

    void publish_free_counts() {
        for (size_t t = 0; t < free_instances_.size(); ++t) free_counts_[t].store((unsigned)free_instances_[t].size(), std::memory_order_release);
    }

    void run() {
        std::thread monitor_thr([this] { monitor(); });
        std::thread submit_thr([this] { submit(); });
        if (opt_.pin_threads) {
            pin(monitor_thr, 0);
            pin(submit_thr, 2);
        }
        monitor_thr.join();
        submit_thr.join();
    }

    double elapsed_us() const { return std::chrono::duration<double, std::micro>(end_time_ - start_time_).count(); }
    std::vector<double>& latencies() { return latencies_; }
    std::vector<std::vector<double>>& latencies_per_type() { return latencies_per_type_; }
    const std::vector<unsigned>& timeline() const { return timeline_; }
    unsigned queue_full_events() const { return num_queue_full_; }
    unsigned type_full_events() const { return num_type_full_; }

  private:
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
        inst->launch();
    }

    void monitor() {
        const auto very_start = Clock::now();
        for (unsigned done = 0; done < opt_.num_jobs; ++done) {
            llis::client::JobInstanceRef* inst = client_->wait();
            const auto now = Clock::now();
            const double latency = us_since_epoch(now) - inst->get_start_time();
            const double t = std::chrono::duration<double, std::micro>(now - very_start).count();
            const unsigned type = inst->get_job_ref_id();
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
            if (done >= opt_.start_record_num) {
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

        double next_submit = 0;
        start_time_ = Clock::now();
        const double start_us = us_since_epoch(start_time_);
        unsigned submitted = 0;

        while (submitted < opt_.num_jobs) {
            const double elapsed = std::chrono::duration<double, std::micro>(Clock::now() - start_time_).count();
            if (elapsed < next_submit) continue;

            if (num_outstanding_.load(std::memory_order_acquire) >= opt_.concurrency) {
                ++num_queue_full_;
                while (num_outstanding_.load(std::memory_order_acquire) >= opt_.concurrency) {
                }
            }
            const unsigned type = (unsigned)(std::lower_bound(props_cum_.begin(), props_cum_.end(), d_type(gen)) - props_cum_.begin());
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
            if (opt_.iat > 0) next_submit += use_exp ? d_exp(gen) : d_ln(gen);
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

    std::vector<double> latencies_;
    std::vector<std::vector<double>> latencies_per_type_;
    std::vector<unsigned> timeline_;
    Clock::time_point start_time_, end_time_;
    unsigned num_queue_full_ = 0, num_type_full_ = 0;
};

void append(std::ostringstream& os, bool named, bool grouped, bool want_grouped, const char* tag, double value) {
    if (named && grouped == want_grouped) os << tag << value;
}

}  // namespace

int main(int argc, char** argv) {
    Options opt;
    int flag_slot = 0;
    bool* flag_targets[] = {&opt.n_iat, &opt.n_lns, &opt.n_con, &opt.n_n, &opt.n_srn, &opt.n_seed, &opt.n_fair, &opt.n_scheds,
                            &opt.g_iat, &opt.g_lns, &opt.g_con, &opt.g_n, &opt.g_srn, &opt.g_seed, &opt.g_fair, &opt.g_scheds};
    static const char* flag_names[] = {"iat_n", "ln_sigma_n", "concurrency_n", "num_jobs_n", "start_record_num_n", "seed_n", "fairness_n", "sched_sleep_n",
                                       "iat_g", "ln_sigma_g", "concurrency_g", "num_jobs_g", "start_record_num_g", "seed_g", "fairness_g", "sched_sleep_g"};
    std::vector<option> long_opts = {{"server_name", required_argument, nullptr, 'm'}, {"iat", required_argument, nullptr, 'i'},
                                     {"ln_sigma", required_argument, nullptr, 'l'},    {"concurrency", required_argument, nullptr, 'c'},
                                     {"num_jobs", required_argument, nullptr, 'n'},    {"start_record_num", required_argument, nullptr, 'r'},
                                     {"seed", required_argument, nullptr, 's'},        {"prefix", required_argument, nullptr, 'p'},
                                     {"fairness", required_argument, nullptr, 'f'},    {"sched_sleep", required_argument, nullptr, 'h'},
                                     {"dist", required_argument, nullptr, 'd'},        {"no_pin", no_argument, nullptr, 'P'}};
    for (int i = 0; i < 16; ++i) long_opts.push_back(option{flag_names[i], no_argument, &flag_slot, i + 1});
    long_opts.push_back(option{nullptr, 0, nullptr, 0});

    for (int c; (c = getopt_long(argc, argv, "m:i:l:c:n:r:s:p:f:", long_opts.data(), nullptr)) != -1;) {
        switch (c) {
            case 0: if (flag_slot >= 1 && flag_slot <= 16) *flag_targets[flag_slot - 1] = true; break;
            case 'm': opt.server_name = optarg; break;
            case 'i': opt.iat = std::atof(optarg); break;
            case 'l': opt.ln_sigma = std::atof(optarg); break;
            case 'c': opt.concurrency = std::atoi(optarg); break;
            case 'n': opt.num_jobs = (unsigned)std::atoi(optarg); break;
            case 'r': opt.start_record_num = (unsigned)std::atoi(optarg); break;
            case 's': opt.seed = (unsigned)std::atoi(optarg); break;
            case 'p': opt.prefix = optarg; break;
            case 'f': opt.fairness = std::atof(optarg); break;
            case 'h': opt.sched_sleep = (unsigned)std::atoi(optarg); break;
            case 'd': opt.dist = optarg; break;
            case 'P': opt.pin_threads = false; break;
            default: return 2;
        }
    }
    if (opt.server_name.empty() || opt.iat < 0 || opt.concurrency <= 0 || opt.num_jobs == 0 || (argc - optind) < 3 || (argc - optind) % 3 != 0 ||
        (opt.dist != "exp" && opt.dist != "ln")) {
        std::fprintf(stderr, "usage: %s --server_name S --iat US [--dist exp|ln] [--ln_sigma X] --concurrency C --num_jobs N [--start_record_num R]\n"
                             "          [--seed S] [--prefix OUT] job.so proportion max_outstanding ...\n", argv[0]);
        return 2;
    }

    std::vector<std::string> job_paths;
    std::vector<float> props_cum;
    std::vector<unsigned> max_outstanding;
    for (int i = optind; i < argc; i += 3) {
        job_paths.push_back(argv[i]);
        const float p = std::stof(argv[i + 1]);
        props_cum.push_back(props_cum.empty() ? p : p + props_cum.back());
        max_outstanding.push_back((unsigned)std::atoi(argv[i + 2]));
    }

    // <prefix>[_param...] for the stats file: every named parameter except the grouped (x-axis) one;
    // the long prefix adds the grouped one too.
    std::ostringstream stats_prefix;
    stats_prefix << opt.prefix;
    append(stats_prefix, opt.n_iat, opt.g_iat, false, "_iat", opt.iat);
    append(stats_prefix, opt.n_lns, opt.g_lns, false, "_lns", opt.ln_sigma);
    append(stats_prefix, opt.n_con, opt.g_con, false, "_con", opt.concurrency);
    append(stats_prefix, opt.n_n, opt.g_n, false, "_n", opt.num_jobs);
    append(stats_prefix, opt.n_srn, opt.g_srn, false, "_srn", opt.start_record_num);
    append(stats_prefix, opt.n_seed, opt.g_seed, false, "_seed", opt.seed);
    append(stats_prefix, opt.n_fair, opt.g_fair, false, "_fair", opt.fairness);
    append(stats_prefix, opt.n_scheds, opt.g_scheds, false, "_scheds", opt.sched_sleep);
    std::ostringstream long_prefix;
    long_prefix << stats_prefix.str();
    append(long_prefix, opt.n_iat, opt.g_iat, true, "_iat", opt.iat);
    append(long_prefix, opt.n_lns, opt.g_lns, true, "_lns", opt.ln_sigma);
    append(long_prefix, opt.n_con, opt.g_con, true, "_con", opt.concurrency);
    append(long_prefix, opt.n_n, opt.g_n, true, "_n", opt.num_jobs);
    append(long_prefix, opt.n_srn, opt.g_srn, true, "_srn", opt.start_record_num);
    append(long_prefix, opt.n_seed, opt.g_seed, true, "_seed", opt.seed);
    append(long_prefix, opt.n_fair, opt.g_fair, true, "_fair", opt.fairness);
    append(long_prefix, opt.n_scheds, opt.g_scheds, true, "_scheds", opt.sched_sleep);

    llis::client::Client client(opt.server_name);
    std::vector<llis::client::JobRef> job_refs;
    job_refs.reserve(job_paths.size());
    for (const std::string& p : job_paths) job_refs.push_back(client.register_job(p));

    LoadGenerator gen(&client, opt, props_cum, max_outstanding);

    // Warm-up: create every pooled instance and run it once.
    const auto init_start = Clock::now();
    unsigned total_instances = 0;
    for (unsigned t = 0; t < job_refs.size(); ++t) {
        for (unsigned i = 0; i < max_outstanding[t]; ++i) {
            llis::client::JobInstanceRef* inst = job_refs[t].create_instance();
            gen.add_instance(t, inst);
            inst->launch();
            ++total_instances;
        }
    }
    for (unsigned i = 0; i < total_instances; ++i) client.wait();
    gen.publish_free_counts();
    const double init_us = std::chrono::duration<double, std::micro>(Clock::now() - init_start).count();

    gen.run();

    const double elapsed = gen.elapsed_us();
    Stats all = summarize(gen.latencies());
    std::vector<Stats> per_type;
    for (auto& v : gen.latencies_per_type()) per_type.push_back(summarize(v));

    if (FILE* fp = std::fopen((stats_prefix.str() + ".txt").c_str(), "a")) {
        if (opt.g_fair) std::fprintf(fp, "%f", opt.fairness);
        else if (opt.g_scheds) std::fprintf(fp, "%u", opt.sched_sleep);
        else std::fprintf(fp, "%d", (int)opt.iat);
        std::fprintf(fp, ",%u,%f", opt.num_jobs, elapsed);
        auto put = [fp](const Stats& s) { std::fprintf(fp, ",%f,%f,%f,%f,%f,%f,%f", s.mean, s.p50, s.p90, s.p95, s.p99, s.max, s.sd); };
        put(all);
        for (const Stats& s : per_type) put(s);
        std::fprintf(fp, "\n");
        std::fclose(fp);
    }
    if (FILE* fp = std::fopen((long_prefix.str() + "_raw.txt").c_str(), "w")) {
        for (double l : gen.latencies()) std::fprintf(fp, "%f\n", l);
        std::fclose(fp);
    }
    if (FILE* fp = std::fopen((long_prefix.str() + "_timeline.txt").c_str(), "w")) {
        const size_t row = props_cum.size() + 1;
        for (size_t i = 0; i < gen.timeline().size(); ++i) {
            if (i && i % row == 0) std::fprintf(fp, "\n");
            std::fprintf(fp, "%u ", gen.timeline()[i]);
        }
        std::fclose(fp);
    }

    std::printf("{\"num_jobs\": %u, \"elapsed_us\": %.3f, \"throughput_rps\": %.3f, \"mean_us\": %.3f, \"p50_us\": %.3f, \"p90_us\": %.3f, "
                "\"p95_us\": %.3f, \"p99_us\": %.3f, \"max_us\": %.3f, \"init_us\": %.1f, \"queue_full\": %u, \"type_full\": %u, \"per_type_p99_us\": [",
                opt.num_jobs, elapsed, opt.num_jobs / elapsed * 1e6, all.mean, all.p50, all.p90, all.p95, all.p99, all.max, init_us,
                gen.queue_full_events(), gen.type_full_events());
    for (size_t t = 0; t < per_type.size(); ++t) std::printf("%s%.3f", t ? ", " : "", per_type[t].p99);
    std::printf("], \"per_type_p50_us\": [");
    for (size_t t = 0; t < per_type.size(); ++t) std::printf("%s%.3f", t ? ", " : "", per_type[t].p50);
    std::printf("], \"per_type_count\": [");
    for (size_t t = 0; t < gen.latencies_per_type().size(); ++t) std::printf("%s%zu", t ? ", " : "", gen.latencies_per_type()[t].size());
    std::printf("]}\n");
    std::fflush(stdout);

    if (!std::getenv("LLIS_CLIENT_KEEP_SERVER")) client.kill_server();
    return 0;
}
