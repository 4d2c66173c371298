// llis_server --name NAME --sched {fifo,fifo2,full3} [--num_streams N] [--extra_kernels N] [--unfair X]
//             [--sched_sleep N] [--mem_notify {marker,hostfunc}] [--device N] [--measure_block_time] [--noti_batch N]
//             [--print_ipc_latency] [--placement {pooled,per_cu}]
// Same options and defaults as reference src/server/server.cpp:203-235; an unknown scheduler name is an
// error with the list of known ones instead of a null dereference.  --placement per_cu (full3 only, not in the
// reference) admits kernels against the per-compute-unit occupancy model instead of the pooled budget.

#include <llis/ipc/defs.h>
#include <llis/server/scheduler.h>
#include <llis/server/server.h>

#include "paella_hip.h"

#include <getopt.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <string>

static void usage(const char* argv0) {
    std::fprintf(stderr,
                 "usage: %s --name NAME --sched {fifo,fifo2,full3} [--num_streams 500] [--extra_kernels 2]\n"
                 "          [--unfair 1000000] [--sched_sleep 0] [--mem_notify marker|hostfunc] [--device 0] [--measure_block_time] [--noti_batch 64] [--print_ipc_latency]\n"
                 "          [--placement pooled|per_cu]\n",
                 argv0);
}

int main(int argc, char** argv) {
    std::string name, sched;
    llis::server::SchedulerOptions opts;
    int device = 0;

    static const option long_opts[] = {{"help", no_argument, nullptr, 'h'},          {"name", required_argument, nullptr, 'n'},
                                       {"sched", required_argument, nullptr, 's'},   {"num_streams", required_argument, nullptr, 't'},
                                       {"extra_kernels", required_argument, nullptr, 'e'}, {"unfair", required_argument, nullptr, 'u'},
                                       {"sched_sleep", required_argument, nullptr, 'p'},   {"mem_notify", required_argument, nullptr, 'm'},
                                       {"device", required_argument, nullptr, 'd'},  {"measure_block_time", no_argument, nullptr, 'B'},
                                       {"noti_batch", required_argument, nullptr, 'b'},  {"print_ipc_latency", no_argument, nullptr, 'L'},
                                       {"placement", required_argument, nullptr, 'P'},
                                       {nullptr, 0, nullptr, 0}};
    for (int c; (c = getopt_long(argc, argv, "h", long_opts, nullptr)) != -1;) {
        switch (c) {
            case 'n': name = optarg; break;
            case 's': sched = optarg; break;
            case 't': opts.num_streams = (unsigned)std::strtoul(optarg, nullptr, 10); break;
            case 'e': opts.extra_kernels = (unsigned)std::strtoul(optarg, nullptr, 10); break;
            case 'u': opts.unfair = std::strtof(optarg, nullptr); break;
            case 'p': opts.sched_sleep = (unsigned)std::strtoul(optarg, nullptr, 10); break;
            case 'm':
                if (!std::strcmp(optarg, "marker")) opts.mem_marker = true;
                else if (!std::strcmp(optarg, "hostfunc")) opts.mem_marker = false;
                else { usage(argv[0]); return 2; }
                break;
            case 'd': device = std::atoi(optarg); break;
            case 'B': opts.measure_block_time = true; break;
            case 'b': opts.noti_batch = (unsigned)std::strtoul(optarg, nullptr, 10); break;
            case 'L': llis::ipc::set_launch_timestamps(true); break;
            case 'P':
                if (!std::strcmp(optarg, "per_cu")) opts.per_cu_placement = true;
                else if (!std::strcmp(optarg, "pooled")) opts.per_cu_placement = false;
                else { usage(argv[0]); return 2; }
                break;
            default: usage(argv[0]); return c == 'h' ? 1 : 2;
        }
    }
    if (name.empty() || sched.empty() || opts.num_streams == 0) {
        usage(argv[0]);
        return 2;
    }
    if (opts.per_cu_placement && sched != "full3") {
        std::fprintf(stderr, "[llis] --placement per_cu needs --sched full3 (the other schedulers admit without an occupancy model)\n");
        return 2;
    }

    try {
        if (int rc = llis_hip_set_device(device)) {
            std::fprintf(stderr, "[llis] cannot select GPU %d: %s\n", device, llis_hip_error_string(rc));
            return 3;
        }
        std::unique_ptr<llis::server::Scheduler> scheduler = llis::server::SchedulerFactory::create(sched, opts);
        llis::server::Server server(name, scheduler.get());
        std::fprintf(stderr, "[llis] server '%s' up: sched=%s streams=%u\n", name.c_str(), sched.c_str(), opts.num_streams);
        server.serve();
        std::fprintf(stderr, "[llis] server '%s' exiting\n", name.c_str());
    } catch (const std::exception& e) {
        std::fprintf(stderr, "[llis] fatal: %s\n", e.what());
        return 4;
    }
    return 0;
}
