// Self-checking exerciser of the host IPC primitives (tests only).  Prints "OK ..." or "ERROR ..." per check.
//   threads                10 000 ints through an anonymous 64-byte ring, reader and writer threads
//                          (pattern of reference tests/ipc/shm_channel/shmc_read_write_same_proc.cpp:5-31)
//   reader NAME | writer NAME   the same between two processes over a named 64-byte ring
//                          (reference tests/ipc/shm_channel/shmc_read.cpp:3-13, shmc_write.cpp:3-8)
//   messages               strings, structs and ragged sizes across the wrap-around, reader/writer threads
//   multiwriter            two writer endpoints (separate objects, as two client processes have) alternate
//                          whole messages under the writer lock
//   pring                  CPU flavour of the fixed-slot ring: 4 producer threads, 1 consumer, slot reuse
//   hold NAME              create a named ring, write a known message, wait for a line on stdin (layout probe)
//   socket                 abstract-namespace datagram round trip incl. the non-blocking full-queue path

#include <llis/job/context.h>
#include <llis/ipc/defs.h>
#include <llis/ipc/name_format.h>
#include <llis/ipc/shm_channel.h>
#include <llis/ipc/shm_primitive_channel.h>
#include <llis/ipc/unix_datagram_socket.h>
#include <llis/server/client_connection.h>
#include <llis/job/instrument_info.h>

#include <unistd.h>

#include <atomic>
#include <cstdio>
#include <cstring>
#include <iostream>
#include <string>
#include <thread>
#include <vector>

using namespace llis::ipc;

static int read_ints(ShmChannelCpuReader* ch, int n) {
    for (int i = 0; i < n; ++i) {
        int v;
        ch->read(&v, sizeof(v));
        if (v != i) {
            std::printf("ERROR expected %d got %d\n", i, v);
            return 1;
        }
    }
    return 0;
}

int main(int argc, char** argv) {
    const std::string cmd = argc > 1 ? argv[1] : "";
    if (cmd == "threads") {
        ShmChannelCpuReader rd(64);
        ShmChannelCpuWriter wr = rd.fork();
        int rc = 1;
        std::thread t1([&] { rc = read_ints(&rd, 10000); });
        std::thread t2([&] { for (int i = 0; i < 10000; ++i) wr.write(i); });
        t1.join();
        t2.join();
        if (rc == 0) std::printf("OK threads\n");
        return rc;
    }
    if (cmd == "reader") {
        ShmChannelCpuReader rd(argv[2], 64);
        std::printf("READY\n");
        std::fflush(stdout);
        int rc = read_ints(&rd, 10000);
        if (rc == 0) std::printf("OK reader\n");
        return rc;
    }
    if (cmd == "writer") {
        ShmChannelCpuWriter wr(argv[2]);
        for (int i = 0; i < 10000; ++i) wr.write(&i, sizeof(i));
        std::printf("OK writer\n");
        return 0;
    }
    if (cmd == "messages") {
        ShmChannelCpuReader rd(37);  // odd capacity: every message straddles the end sooner or later
        ShmChannelCpuWriter wr = rd.fork();
        struct Rec { uint32_t a; double b; char c; };
        int bad = 0;
        std::thread t1([&] {
            for (int i = 0; i < 3000; ++i) {
                std::string s;
                rd.read(&s);
                Rec r;
                rd.read(&r);
                llis::MsgType t;
                rd.read(&t);
                if (s != std::string((size_t)(i % 23), (char)('a' + i % 26)) || r.a != (uint32_t)i || r.b != i * 0.5 || r.c != (char)(i % 100) ||
                    t != llis::MsgType::GROW_POOL)
                    ++bad;
            }
        });
        std::thread t2([&] {
            for (int i = 0; i < 3000; ++i) {
                wr.write(std::string((size_t)(i % 23), (char)('a' + i % 26)));
                Rec r{(uint32_t)i, i * 0.5, (char)(i % 100)};
                wr.write(r);
                wr.write(llis::MsgType::GROW_POOL);
            }
        });
        t1.join();
        t2.join();
        std::printf(bad ? "ERROR messages %d corrupted\n" : "OK messages\n", bad);
        return bad != 0;
    }
    if (cmd == "multiwriter") {
        ShmChannelCpuReader rd("mw" + std::to_string(getpid()), 256);
        ShmChannelCpuWriter w1("mw" + std::to_string(getpid())), w2("mw" + std::to_string(getpid()));
        std::atomic<int> bad{0};
        std::thread t0([&] {
            int seen[2] = {0, 0};
            for (int i = 0; i < 20000; ++i) {
                int who, seq, check;
                rd.read(&who);
                rd.read(&seq);
                rd.read(&check);
                if (who < 0 || who > 1 || seq != seen[who] || check != (who * 1000003 + seq)) { ++bad; break; }
                ++seen[who];
            }
        });
        auto producer = [&](ShmChannelCpuWriter* w, int who) {
            for (int i = 0; i < 10000; ++i) {
                w->acquire_writer_lock();
                w->write(who);
                w->write(i);
                w->write(who * 1000003 + i);
                w->release_writer_lock();
            }
        };
        std::thread t1(producer, &w1, 0), t2(producer, &w2, 1);
        t1.join();
        t2.join();
        t0.join();
        std::printf(bad ? "ERROR multiwriter\n" : "OK multiwriter\n");
        return bad != 0;
    }
    if (cmd == "pollhooks") {
        // the serving thread's per-turn hooks: a function registers once however often it is added, hooks run in order
        static int a = 0, b = 0;
        llis::job::Context::run_poll_hooks();  // none yet
        llis::job::Context::add_poll_hook(+[] { ++a; });
        auto fb = +[] { b += a; };
        llis::job::Context::add_poll_hook(fb);
        llis::job::Context::add_poll_hook(fb);
        llis::job::Context::add_poll_hook(nullptr);
        for (int i = 0; i < 3; ++i) llis::job::Context::run_poll_hooks();
        const bool ok = a == 3 && b == 1 + 2 + 3;
        std::printf(ok ? "OK pollhooks\n" : "ERROR pollhooks %d %d\n", a, b);
        return !ok;
    }
    if (cmd == "pring") {
        using Info = llis::job::InstrumentInfo;
        ShmPrimitiveChannel<uint64_t> ring(std::string(), 64);
        std::vector<std::thread> producers;
        const int per = 5000;
        std::atomic<int> consumed{0};
        // Producers must not lap the consumer (the ring has no full check): throttle on the consumed count.
        std::atomic<int> produced{0};
        for (int p = 0; p < 4; ++p)
            producers.emplace_back([&, p] {
                ShmPrimitiveChannel<uint64_t> w(&ring);
                for (int i = 0; i < per; ++i) {
                    while (produced.load() - consumed.load() >= 60) {
                    }
                    ++produced;
                    Info info;
                    info.is_start = (uint8_t)(i & 1);
                    info.num = (uint8_t)(p + 1);
                    info.job_id = (uint32_t)i;
                    w.write(info);
                }
            });
        int next[4] = {0, 0, 0, 0};
        int bad = 0;
        for (int n = 0; n < 4 * per; ++n) {
            Info info = ring.read<Info>();
            const int p = info.num - 1;
            if (p < 0 || p > 3 || (int)info.job_id != next[p] || info.is_start != (next[p] & 1) || info.can_read()) ++bad;
            else ++next[p];
            ++consumed;
        }
        for (auto& t : producers) t.join();
        if (ring.can_read<Info>()) ++bad;  // every slot was handed back
        std::printf(bad ? "ERROR pring %d\n" : "OK pring\n", bad);
        return bad != 0;
    }
    if (cmd == "hold") {
        ShmChannelCpuWriter wr(argv[2], 64);
        wr.write(llis::MsgType::REGISTER_JOB);
        wr.write((uint32_t)0xAABBCCDD);
        wr.write(std::string("hi"));
        std::printf("READY %s\n", c2s_channel_name("x").c_str());
        std::fflush(stdout);
        std::string line;
        std::getline(std::cin, line);
        return 0;
    }
    if (cmd == "socket") {
        const std::string name = s2c_socket_name("chk" + std::to_string(getpid()), 7);
        UnixDatagramSocket receiver(name);
        UnixDatagramSocket sender;
        UnixDatagramSocket peer = sender.connect(name);
        char b = 42;
        peer.write(&b, 1);
        char got = 0;
        receiver.read(&got, 1);
        int sent = 0, refused = 0;
        for (int i = 0; i < 200; ++i) (peer.try_write(&b, 1) ? sent : refused)++;
        int drained = 0;
        for (int i = 0; i < sent; ++i) { receiver.read(&got, 1); ++drained; }
        const bool ok = got == 42 && sent >= 1 && refused >= 1 && drained == sent && peer.try_write(&b, 1);
        std::printf(ok ? "OK socket sent=%d refused=%d\n" : "ERROR socket sent=%d refused=%d\n", sent, refused);
        return !ok;
    }
    if (cmd == "deadclient") {
        // A peer that refuses every wake-up is taken for dead after two seconds, gets completions only while its ring has
        // room (the serving thread never waits for it), and comes back when a wake-up gets through again.
        const std::string tag = "dead" + std::to_string(getpid());
        const std::string sock_name = s2c_socket_name(tag, 3);
        UnixDatagramSocket sender;
        llis::server::ClientConnection conn(3);
        ShmChannelCpuReader ring(s2c_channel_name(tag, 3), 64);   // the client's end; 63 usable bytes = 7 completions
        conn.use_s2c_channel(ShmChannelCpuWriter(s2c_channel_name(tag, 3)));
        conn.use_s2c_socket(sender.connect(sock_name));           // nobody is bound there yet
        int bad = 0;
        for (int i = 0; i < 5; ++i) bad += !conn.wake();          // all owed
        const auto t0 = std::chrono::steady_clock::now();
        while (!conn.is_dead() && std::chrono::steady_clock::now() - t0 < std::chrono::seconds(4)) {
            bad += conn.retry_wakeups() != 0;
            usleep(1000);
        }
        bad += !conn.is_dead();
        unsigned gave_back = 0;
        for (uintptr_t i = 1; i <= 10; ++i) gave_back += conn.post_completion(reinterpret_cast<void*>(i));   // returns at once, every time
        bad += conn.dropped_completions() != 3 || gave_back != 3;  // 7 fit; each dropped one takes an owed wake-up with it
        UnixDatagramSocket receiver(sock_name);                    // the "client" shows up after all
        usleep(250000);
        const unsigned settled = conn.retry_wakeups();
        bad += conn.is_dead() || settled != 2;
        char b;
        for (unsigned i = 0; i < settled; ++i) receiver.read(&b, 1);
        for (uintptr_t i = 1; i <= 7; ++i) {
            void* p = nullptr;
            ring.read(&p);
            bad += p != reinterpret_cast<void*>(i);
        }
        bad += ring.can_read();
        bad += conn.wake();   // goes straight out again
        std::printf(bad ? "ERROR deadclient %d\n" : "OK deadclient\n", bad);
        return bad != 0;
    }
    std::fprintf(stderr, "unknown check\n");
    return 2;
}
