// llis_app_single_latency SERVER JOB.so N [--check-vec-add]
// Closed loop with one client and one instance: launch, wait, repeat; prints microseconds per request
// (pattern of reference tests/client/client_single_latency.cpp:16-36) and a JSON summary at the end.

#include <llis/client/client.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

int main(int argc, char** argv) {
    if (argc < 4) {
        std::fprintf(stderr, "usage: %s SERVER JOB.so N [--quiet] [--keep-server]\n", argv[0]);
        return 2;
    }
    bool quiet = false, keep = false;
    for (int i = 4; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--quiet")) quiet = true;
        if (!std::strcmp(argv[i], "--keep-server")) keep = true;
    }
    const int n = std::atoi(argv[3]);
    llis::client::Client client(argv[1]);
    llis::client::JobRef job_ref = client.register_job(argv[2]);
    llis::client::JobInstanceRef* inst = job_ref.create_instance();
    std::memset(inst->get_input_ptr(), 0, job_ref.get_job()->get_input_size());

    inst->launch();  // warm-up: first use of the instance builds the model on the server
    client.wait();

    std::vector<double> lat;
    lat.reserve(n);
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < n; ++i) {
        const auto a = std::chrono::steady_clock::now();
        inst->launch();
        client.wait();
        const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - a).count();
        lat.push_back(us);
        if (!quiet) std::printf("%f\n", us);
    }
    const double total = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    std::sort(lat.begin(), lat.end());
    std::printf("{\"num_jobs\": %d, \"elapsed_us\": %.3f, \"throughput_rps\": %.3f, \"p50_us\": %.3f, \"p99_us\": %.3f, \"min_us\": %.3f}\n", n, total,
                n / total * 1e6, lat[lat.size() / 2], lat[(size_t)(lat.size() * 0.99)], lat.front());
    if (!keep) client.kill_server();
    return 0;
}
