// Single-threaded scripted driver (tests only): the real Server + scheduler + rings on the scripted device,
// with the client side of the wire protocol written out by hand, message by message.  Reads commands on
// stdin, prints replies and finally the scheduler's event log on stdout.
//
//   sched NAME streams N [extra K] [unfair X] [mem marker|hostfunc] [budget REGS SMEM THREADS BLOCKS] [batch B]
//         [percu CUS XCDS REGS SMEM THREADS BLOCKS]   full3 with per-compute-unit placement over that topology
//   client                      register a client                      -> "client ID"
//   job PATH                    register a job type, grow its pool     -> "job TYPE"
//   launch TYPE [SLOT]          LAUNCH_JOB for slot SLOT of the pool
//   step [N]                    run the oldest device operation to completion, N times
//   start STREAM | finish STREAM   advance the head operation of a stream by one phase / to completion
//   sleep US                    let wall-clock time pass (stage lengths are measured)
//   drain                       step until the device is idle
//   put TYPE SLOT BYTE          fill the slot's input with BYTE;   get TYPE SLOT -> "out B0 B1 ..." (first 8 output bytes)
//   log                         print the event log so far (also printed at exit)

#include <llis/job/context.h>
#include <llis/ipc/name_format.h>
#include <llis/ipc/shm_channel.h>
#include <llis/ipc/unix_datagram_socket.h>
#include <llis/server/scheduler.h>
#include <llis/server/scheduler_full3.h>
#include <llis/server/server.h>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/socket.h>
#include <unistd.h>

#include <csignal>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

extern "C" int fake_hip_step_oldest(int full);
extern "C" int fake_hip_step_stream(unsigned index, int full);
extern "C" unsigned fake_hip_pending(void);
extern "C" void fake_hip_set_batch(unsigned batch);

using namespace llis;

namespace {

constexpr size_t kChunk = 30638080;

struct JobType {
    unsigned id;
    std::string shm_name;
    char* pool;
    size_t in_size, slot_size;
};

struct Harness {
    std::string server_name;
    std::unique_ptr<server::Scheduler> scheduler;
    std::unique_ptr<server::Server> server;
    std::unique_ptr<ipc::ShmChannelCpuWriter> c2s;
    std::unique_ptr<ipc::ShmChannelCpuReader> s2c;
    int sock = -1;
    ClientId client_id = 0;
    std::vector<JobType> types;
    unsigned completions = 0, wakeups = 0, launches = 0;
    unsigned long long polls = 0;

    void poll(bool drain = true) {
        int idle = 0;
        while (idle < 4) {
            const size_t before = server->get_event_log()->events().size();
            server->poll_once();
            ++polls;
            idle = server->get_event_log()->events().size() == before ? idle + 1 : 0;
            if (drain) drain_client();
        }
    }

    void drain_client() {
        if (sock != -1) {
            char b;
            while (recv(sock, &b, 1, MSG_DONTWAIT) == 1) ++wakeups;
        }
        while (s2c && s2c->can_read()) {
            void* cookie;
            s2c->read(&cookie);
            std::printf("done %llu\n", (unsigned long long)(uintptr_t)cookie);
            ++completions;
        }
    }
};

// Name of the request ring the server creates, kept for the exit paths that run no destructors.
char g_c2s_object[128];

void unlink_request_ring() {
    if (g_c2s_object[0]) shm_unlink(g_c2s_object);
}

void on_fatal_signal(int sig) {
    unlink_request_ring();
    _exit(128 + sig);
}

}  // namespace

static unsigned long long g_hook_calls = 0;
static void count_poll_hook() { ++g_hook_calls; }

int main() {
    llis::job::Context::add_poll_hook(&count_poll_hook);
    llis::job::Context::add_poll_hook(&count_poll_hook);
    // The script owns the device: a background thread that completes operations on its own (what the
    // in-process serving tests ask the scripted device for) would race every "step" of the script.
    if (const char* autorun = std::getenv("FAKE_HIP_AUTORUN"); autorun && *autorun == '1') {
        std::fprintf(stderr, "sched_harness: FAKE_HIP_AUTORUN=1 is set; the harness steps the device itself\n");
        return 4;
    }
    Harness h;
    h.server_name = "harness" + std::to_string(getpid());
    std::snprintf(g_c2s_object, sizeof(g_c2s_object), "llis:channel:%s", ipc::c2s_channel_name(h.server_name).c_str());
    std::atexit(unlink_request_ring);
    std::set_terminate([] { unlink_request_ring(); std::abort(); });
    for (int sig : {SIGTERM, SIGINT, SIGHUP, SIGSEGV, SIGABRT, SIGPIPE}) std::signal(sig, on_fatal_signal);
    std::string line;
    while (std::getline(std::cin, line)) {
        std::istringstream in(line);
        std::string cmd;
        if (!(in >> cmd) || cmd[0] == '#') continue;
        if (cmd == "sched") {
            std::string name, key;
            in >> name;
            server::SchedulerOptions opt;
            opt.ring_slots = 4096;
            bool have_budget = false, have_percu = false;
            long long b[4] = {0, 0, 0, 0}, pc[6] = {0, 0, 0, 0, 0, 0};
            while (in >> key) {
                if (key == "streams") in >> opt.num_streams;
                else if (key == "extra") in >> opt.extra_kernels;
                else if (key == "unfair") in >> opt.unfair;
                else if (key == "mem") { std::string m; in >> m; opt.mem_marker = (m == "marker"); }
                else if (key == "batch") { in >> opt.noti_batch; fake_hip_set_batch(opt.noti_batch); }
                else if (key == "budget") { in >> b[0] >> b[1] >> b[2] >> b[3]; have_budget = true; }
                else if (key == "percu") { in >> pc[0] >> pc[1] >> pc[2] >> pc[3] >> pc[4] >> pc[5]; have_percu = true; }
            }
            if (have_percu && name == "full3")
                h.scheduler = std::make_unique<server::SchedulerFull3>(
                    opt, std::make_unique<server::GpuResources>((unsigned)pc[0], (unsigned)pc[1], pc[2], pc[3], pc[4], pc[5]));
            else if (have_budget && name == "full3") h.scheduler = std::make_unique<server::SchedulerFull3>(opt, server::SmResources(b[0], b[1], b[2], b[3]));
            else h.scheduler = server::SchedulerFactory::create(name, opt);
            h.server = std::make_unique<server::Server>(h.server_name, h.scheduler.get());
            h.server->get_event_log()->enable(true);
            h.c2s = std::make_unique<ipc::ShmChannelCpuWriter>(ipc::c2s_channel_name(h.server_name));
        } else if (cmd == "client") {
            const ClientId tmp = 0xABCD0000u + (unsigned)getpid() % 1000;
            ipc::ShmChannelCpuReader reply(ipc::s2c_channel_name(h.server_name, tmp), 8);
            h.c2s->acquire_writer_lock();
            h.c2s->write(MsgType::REGISTER_CLIENT);
            h.c2s->write(tmp);
            h.c2s->release_writer_lock();
            h.poll();
            reply.read(&h.client_id);
            h.s2c = std::make_unique<ipc::ShmChannelCpuReader>(ipc::s2c_channel_name(h.server_name, h.client_id));
            h.sock = socket(AF_UNIX, SOCK_DGRAM, 0);
            sockaddr_un addr;
            std::memset(&addr, 0, sizeof(addr));
            addr.sun_family = AF_UNIX;
            const std::string sname = ipc::s2c_socket_name(h.server_name, h.client_id);
            std::memcpy(addr.sun_path + 1, sname.data(), sname.size());
            if (bind(h.sock, reinterpret_cast<sockaddr*>(&addr), sizeof(addr)) != 0) { std::perror("bind"); return 1; }
            std::printf("client %u\n", h.client_id);
        } else if (cmd == "job") {
            std::string path;
            in >> path;
            JobType t;
            t.shm_name = "llis:shm:" + std::to_string(h.client_id) + ":" + std::to_string(getpid() * 100 + (int)h.types.size());
            int fd = shm_open(t.shm_name.c_str(), O_CREAT | O_RDWR, 0600);
            if (fd < 0 || ftruncate(fd, kChunk) != 0) { std::perror("shm"); return 1; }
            t.pool = reinterpret_cast<char*>(mmap(nullptr, kChunk, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0));
            h.c2s->acquire_writer_lock();
            h.c2s->write(MsgType::REGISTER_JOB);
            h.c2s->write(h.client_id);
            h.c2s->write(path);
            h.c2s->write(t.shm_name);
            h.c2s->release_writer_lock();
            h.poll(false);  // the reply on the completion ring is a 4-byte id, not a completion
            h.s2c->read(&t.id);
            h.c2s->acquire_writer_lock();
            h.c2s->write(MsgType::GROW_POOL);
            h.c2s->write(t.id);
            h.c2s->write(kChunk);
            h.c2s->release_writer_lock();
            h.poll();
            shm_unlink(t.shm_name.c_str());
            t.in_size = 100;
            t.slot_size = 208;
            h.types.push_back(t);
            std::printf("job %u\n", t.id);
        } else if (cmd == "launch") {
            unsigned type, slot = 0;
            in >> type;
            in >> slot;
            h.c2s->acquire_writer_lock();
            h.c2s->write(MsgType::LAUNCH_JOB);
            h.c2s->write((JobRefId)type);
            h.c2s->write((int)0);
            h.c2s->write((size_t)slot * h.types[type].slot_size);
            h.c2s->write(reinterpret_cast<void*>((uintptr_t)(1000 * (type + 1) + slot)));
            h.c2s->release_writer_lock();
            ++h.launches;
            h.poll();
        } else if (cmd == "step") {
            int n = 1;
            in >> n;
            for (int i = 0; i < n; ++i) {
                if (!fake_hip_step_oldest(1)) break;
                h.poll();
            }
        } else if (cmd == "start" || cmd == "finish") {
            unsigned s;
            in >> s;
            fake_hip_step_stream(s, cmd == "finish");
            h.poll();
        } else if (cmd == "sleep") {
            unsigned us;
            in >> us;
            usleep(us);
        } else if (cmd == "drain") {
            while (fake_hip_pending()) {
                fake_hip_step_oldest(1);
                h.poll();
            }
        } else if (cmd == "put") {
            unsigned type, slot, byte;
            in >> type >> slot >> byte;
            std::memset(h.types[type].pool + slot * h.types[type].slot_size, (int)byte, h.types[type].in_size);
        } else if (cmd == "get") {
            unsigned type, slot;
            in >> type >> slot;
            const unsigned char* out = reinterpret_cast<unsigned char*>(h.types[type].pool + slot * h.types[type].slot_size + h.types[type].in_size);
            std::printf("out");
            for (int i = 0; i < 8; ++i) std::printf(" %u", out[i]);
            std::printf("\n");
        } else if (cmd == "log") {
            std::fputs(h.server->get_event_log()->to_text().c_str(), stdout);
        } else {
            std::fprintf(stderr, "unknown command: %s\n", cmd.c_str());
            return 2;
        }
    }
    std::printf("wakeups %u completions %u pending %u\n", h.wakeups, h.completions, fake_hip_pending());
    // the serving loop's per-turn hooks of job libraries (llis::job::Context::add_poll_hook): once per turn, registered twice
    std::printf("hooks %llu polls %llu\n", g_hook_calls, h.polls);
    std::printf("--- event log\n");
    std::fputs(h.server->get_event_log()->to_text().c_str(), stdout);
    if (fake_hip_pending() == 0 && h.completions != h.launches) {
        std::fprintf(stderr, "sched_harness: device idle, but %u completions for %u launches\n", h.completions, h.launches);
        return 3;
    }
    return 0;
}
