#pragma once
// Writes an arrival trace that the load generator replays: the same draws, in the same order, as the live generator
// (type first, then the gap to the next request) and the same files as the reference tool
// (reference tests/utils/workload_pregen.cpp:72-115):
//   <prefix>_iat<I>_lns<S>_n<N>_seed<K>.txt        one line "<type> <submit time us>" per request
//   <prefix>_iat<I>_lns<S>_n<N>_seed<K>_job<t>.txt  one line "0 <submit time us>" per request of type t
// dist "exp" draws exponential gaps instead of log-normal ones (the reference picks at compile time).
// Shared by llis_app_workload_pregen and paella_workload_pregen.

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <random>
#include <sstream>
#include <string>
#include <vector>

namespace llis {
namespace loadgen {

// Returns the path of the combined trace, or an empty string when a file cannot be written.
inline std::string write_pregen_trace(double iat, bool dist_exp, double ln_sigma, unsigned num_jobs, unsigned seed, const std::string& prefix,
                                      const std::vector<float>& props_cum) {
    std::mt19937 gen(seed);
    std::uniform_real_distribution<float> d_type(0, 1);
    std::exponential_distribution<> d_exp(1. / iat);
    std::lognormal_distribution<> d_ln(std::log(iat) - ln_sigma * ln_sigma / 2, ln_sigma < 0 ? 1.0 : ln_sigma);

    std::ostringstream base;
    base << prefix << "_iat" << iat << "_lns" << ln_sigma << "_n" << num_jobs << "_seed" << seed;
    FILE* all = std::fopen((base.str() + ".txt").c_str(), "w");
    if (!all) return std::string();
    std::vector<FILE*> per_type;
    for (size_t t = 0; t < props_cum.size(); ++t) per_type.push_back(std::fopen((base.str() + "_job" + std::to_string(t) + ".txt").c_str(), "w"));

    double next_submit = 0;
    for (unsigned i = 0; i < num_jobs; ++i) {
        unsigned type = (unsigned)(std::lower_bound(props_cum.begin(), props_cum.end(), d_type(gen)) - props_cum.begin());
        type = std::min<unsigned>(type, (unsigned)props_cum.size() - 1);
        const double gap = dist_exp ? d_exp(gen) : d_ln(gen);
        std::fprintf(all, "%u %f\n", type, next_submit);
        if (per_type[type]) std::fprintf(per_type[type], "0 %f\n", next_submit);
        next_submit += gap;
    }
    for (FILE* fp : per_type)
        if (fp) std::fclose(fp);
    std::fclose(all);
    return base.str() + ".txt";
}

}  // namespace loadgen
}  // namespace llis
