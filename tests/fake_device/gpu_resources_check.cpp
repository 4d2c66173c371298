// Command-driven exerciser of llis::server::GpuResources (tests only).  One command per line on stdin:
//   new CUS XCDS REGS SMEM THREADS BLOCKS      fresh model
//   job J BLOCKS THREADS SMEM REGS             declares the next stage of job J (created on first use)
//   fits J                                     -> "fits 0|1"
//   run J                                      stage becomes current, placement predicted -> "pred cu:n cu:n ..."
//   start J CU | finish J CU                   a workgroup reported that compute unit
//   reconcile J                                -> "wrong W C"
//   dump                                       -> "state full=F all_full=0|1 total_threads=T : t0/b0 t1/b1 ..." (free threads/slots)
#include <llis/server/gpu_resources.h>

#include <cstdio>
#include <iostream>
#include <map>
#include <memory>
#include <sstream>
#include <string>

namespace {
class PlainJob : public llis::job::Job {
  public:
    size_t get_input_size() override { return 0; }
    size_t get_output_size() override { return 0; }
    size_t get_param_size() override { return 0; }
    void full_init(void*) override {}
    void init(void*) override {}
    void run_next() override {}
    bool has_next() const override { return true; }
};
}  // namespace

int main() {
    std::unique_ptr<llis::server::GpuResources> g;
    std::map<int, std::unique_ptr<PlainJob>> jobs;
    std::string line;
    while (std::getline(std::cin, line)) {
        std::istringstream in(line);
        std::string cmd;
        in >> cmd;
        if (cmd == "new") {
            unsigned cus, xcds;
            long long r, s, t, b;
            in >> cus >> xcds >> r >> s >> t >> b;
            g = std::make_unique<llis::server::GpuResources>(cus, xcds, r, s, t, b);
            jobs.clear();
            continue;
        }
        if (cmd == "dump") {
            std::printf("state full=%u all_full=%d total_threads=%lld :", g->num_full_cus(), (int)g->is_full(), g->total().free_threads());
            for (unsigned c = 0; c < g->get_num_cus(); ++c) std::printf(" %lld/%lld", g->cu(c).free_threads(), g->cu(c).free_blocks());
            std::printf("\n");
            continue;
        }
        int j;
        in >> j;
        auto& job = jobs[j];
        if (!job) job = std::make_unique<PlainJob>();
        if (cmd == "job") {
            unsigned b, t, s, r;
            in >> b >> t >> s >> r;
            job->set_num_blocks(b);
            job->set_num_threads_per_block(t);
            job->set_smem_size_per_block(s);
            job->set_num_registers_per_thread(r);
        } else if (cmd == "fits") {
            std::printf("fits %d\n", (int)g->job_fits(job.get()));
        } else if (cmd == "run") {
            job->set_running(nullptr);
            g->choose_cus(job.get());
            std::printf("pred");
            const unsigned* p = job->get_predicted_smid_nums();
            for (unsigned c = 0; c < g->get_num_cus(); ++c)
                if (p[c]) std::printf(" %u:%u", c, p[c]);
            std::printf("\n");
        } else if (cmd == "start" || cmd == "finish") {
            unsigned cu;
            in >> cu;
            if (cmd == "start") g->observe_block_start(job.get(), cu);
            else g->observe_block_finish(job.get(), cu);
        } else if (cmd == "reconcile") {
            unsigned cus = 0;
            const unsigned wrong = g->reconcile(job.get(), &cus);
            std::printf("wrong %u %u\n", wrong, cus);
        } else {
            std::printf("ERROR unknown command %s\n", cmd.c_str());
            return 1;
        }
    }
    return 0;
}
