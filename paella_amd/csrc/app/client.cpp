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
// --print_ipc_latency: LAUNCH_JOB carries its send time (the reference's PRINT_LAUNCH_JOB_IPC_LATENCY build); the server must
// run with the same switch.
// --verify N (no counterpart in the reference, whose client checks no output): N seeded inputs per job type, expected outputs learnt
// from the idle server during the warm-up, every completion compared with its expectation byte for byte; exit code 3 on a mismatch.

#include <llis/client/client.h>
#include <llis/client/job_instance_ref.h>
#include <llis/client/job_ref.h>
#include <llis/ipc/defs.h>

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

#include "serve/load_generator.h"

using namespace llis::loadgen;

namespace {

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
                                     {"dist", required_argument, nullptr, 'd'},        {"warmup", required_argument, nullptr, 'w'},        {"no_pin", no_argument, nullptr, 'P'},
                                     {"profile", required_argument, nullptr, 'R'},
                                     {"trace", required_argument, nullptr, 'T'},
                                     {"verify", required_argument, nullptr, 'V'},
                                     {"print_ipc_latency", no_argument, nullptr, 'L'}};
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
            case 'w': opt.warmup_jobs = (unsigned)std::atoi(optarg); break;
            case 'P': opt.pin_threads = false; break;
            case 'R': opt.profile_prefix = optarg; break;
            case 'T': opt.trace_path = optarg; break;
            case 'V': opt.verify_variants = (unsigned)std::atoi(optarg); break;
            case 'L': llis::ipc::set_launch_timestamps(true); break;
            default: return 2;
        }
    }
    if (opt.server_name.empty() || opt.iat < 0 || opt.concurrency <= 0 || opt.num_jobs == 0 || (argc - optind) < 3 || (argc - optind) % 3 != 0 ||
        (opt.dist != "exp" && opt.dist != "ln")) {
        std::fprintf(stderr, "usage: %s --server_name S --iat US [--dist exp|ln] [--ln_sigma X] --concurrency C --num_jobs N [--start_record_num R]\n"
                             "          [--seed S] [--prefix OUT] [--warmup N] [--no_pin] [--profile PREFIX] [--trace FILE] [--verify INPUTS_PER_TYPE] [--print_ipc_latency] job.so proportion max_outstanding ...\n", argv[0]);
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

    // Warm-up: create every pooled instance and run it once (one at a time in verify mode, which also learns the expected outputs).
    const auto init_start = Clock::now();
    gen.warm_up(job_refs);
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
    std::printf("]");
    if (opt.verify_variants) std::printf(", \"verified_requests\": %llu, \"mismatches\": %llu", (unsigned long long)gen.verified(), (unsigned long long)gen.mismatches());
    std::printf("}\n");
    std::fflush(stdout);
    for (const Mismatch& m : gen.first_mismatches())
        std::fprintf(stderr, "llis_app_client: output mismatch at checked completion %llu: job type %u, input variant %u, first differing byte %zu\n",
                     (unsigned long long)m.request, m.type, m.variant, m.offset);

    if (!std::getenv("LLIS_CLIENT_KEEP_SERVER")) client.kill_server();
    if (gen.mismatches()) return 3;
    return 0;
}
