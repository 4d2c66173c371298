// llis_app_workload_pregen -- writes an arrival trace that llis_app_client --trace replays.
//
// Same draws, in the same order, as the live load generator (type first, then the gap to the next request) and
// the same files as the reference tool (reference tests/utils/workload_pregen.cpp:75-115):
//   <prefix>_iat<I>_lns<S>_n<N>_seed<K>.txt        one line "<type> <submit time us>" per request
//   <prefix>_iat<I>_lns<S>_n<N>_seed<K>_job<t>.txt  one line "0 <submit time us>" per request of type t
// --dist exp draws exponential gaps instead of log-normal ones (the reference picks at compile time).

#include "../serve/workload_pregen.h"

#include <getopt.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <sstream>
#include <string>
#include <vector>

int main(int argc, char** argv) {
    double iat = -1, ln_sigma = -1;
    unsigned num_jobs = 0, seed = 1;
    std::string prefix, dist = "ln";
    static const option long_opts[] = {{"iat", required_argument, nullptr, 'i'},      {"ln_sigma", required_argument, nullptr, 'l'},
                                       {"num_jobs", required_argument, nullptr, 'n'}, {"seed", required_argument, nullptr, 's'},
                                       {"pregen_prefix", required_argument, nullptr, 'g'}, {"dist", required_argument, nullptr, 'd'},
                                       {nullptr, 0, nullptr, 0}};
    for (int c; (c = getopt_long(argc, argv, "i:l:n:s:g:d:", long_opts, nullptr)) != -1;) {
        switch (c) {
            case 'i': iat = std::atof(optarg); break;
            case 'l': ln_sigma = std::atof(optarg); break;
            case 'n': num_jobs = (unsigned)std::atoi(optarg); break;
            case 's': seed = (unsigned)std::atoi(optarg); break;
            case 'g': prefix = optarg; break;
            case 'd': dist = optarg; break;
            default: return 2;
        }
    }
    std::vector<float> props_cum;
    for (int i = optind; i < argc; ++i) props_cum.push_back(std::stof(argv[i]) + (props_cum.empty() ? 0.f : props_cum.back()));
    if (iat <= 0 || num_jobs == 0 || prefix.empty() || props_cum.empty() || (dist != "ln" && dist != "exp") || (dist == "ln" && ln_sigma < 0)) {
        std::fprintf(stderr, "usage: %s --iat US [--dist ln|exp] --ln_sigma X --num_jobs N --seed S --pregen_prefix OUT proportion ...\n", argv[0]);
        return 2;
    }

    const std::string path = llis::loadgen::write_pregen_trace(iat, dist == "exp", ln_sigma, num_jobs, seed, prefix, props_cum);
    if (path.empty()) {
        std::perror("pregen output");
        return 1;
    }
    std::printf("%s\n", path.c_str());
    return 0;
}
