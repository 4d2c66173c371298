// llis_app_workload_pregen -- writes an arrival trace that llis_app_client --trace replays.
//
// Same draws, in the same order, as the live load generator (type first, then the gap to the next request) and
// the same files as the reference tool (reference tests/utils/workload_pregen.cpp:75-115):
//   <prefix>_iat<I>_lns<S>_n<N>_seed<K>.txt        one line "<type> <submit time us>" per request
//   <prefix>_iat<I>_lns<S>_n<N>_seed<K>_job<t>.txt  one line "0 <submit time us>" per request of type t
// --dist exp draws exponential gaps instead of log-normal ones (the reference picks at compile time).

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

    std::mt19937 gen(seed);
    std::uniform_real_distribution<float> d_type(0, 1);
    std::exponential_distribution<> d_exp(1. / iat);
    std::lognormal_distribution<> d_ln(std::log(iat) - ln_sigma * ln_sigma / 2, ln_sigma < 0 ? 1.0 : ln_sigma);

    std::ostringstream base;
    base << prefix << "_iat" << iat << "_lns" << ln_sigma << "_n" << num_jobs << "_seed" << seed;
    FILE* all = std::fopen((base.str() + ".txt").c_str(), "w");
    if (!all) {
        std::perror("pregen output");
        return 1;
    }
    std::vector<FILE*> per_type;
    for (size_t t = 0; t < props_cum.size(); ++t) per_type.push_back(std::fopen((base.str() + "_job" + std::to_string(t) + ".txt").c_str(), "w"));

    double next_submit = 0;
    for (unsigned i = 0; i < num_jobs; ++i) {
        unsigned type = (unsigned)(std::lower_bound(props_cum.begin(), props_cum.end(), d_type(gen)) - props_cum.begin());
        type = std::min<unsigned>(type, (unsigned)props_cum.size() - 1);
        const double gap = dist == "exp" ? d_exp(gen) : d_ln(gen);
        std::fprintf(all, "%u %f\n", type, next_submit);
        if (per_type[type]) std::fprintf(per_type[type], "0 %f\n", next_submit);
        next_submit += gap;
    }
    for (FILE* fp : per_type)
        if (fp) std::fclose(fp);
    std::fclose(all);
    std::printf("%s.txt\n", base.str().c_str());
    return 0;
}
