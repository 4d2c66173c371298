#pragma once
// Identifier types and the client->server wire enums.  The numeric values are part of the IPC protocol: they
// equal those of reference include/llis/ipc/defs.h:7-37, so a reference-built client can talk to this server.

#include <cstdint>

namespace llis {

using ClientId = uint32_t;
using JobRefId = uint32_t;
using JobInstanceRefId = uint32_t;
using JobId = uint32_t;

// First word of every message on the client->server ring.
enum class MsgType : uint32_t {
    REGISTER_CLIENT = 0,      // {u32 temporary id}                         -> u32 client id on the temporary reply ring
    REGISTER_JOB = 1,         // {u32 client, str library path, str pool}   -> u32 job reference id
    LAUNCH_JOB = 2,           // {[u64 send time,] u32 job reference, i32 pool, size_t offset, void* client-side handle}
    GROW_POOL = 3,            // {u32 job reference, size_t bytes}
    CUDA_PROFILER_START = 4,  // (names kept from the reference; they switch the device profiler range on / off)
    CUDA_PROFILER_STOP = 5,
    PROFILER_CMD = 6,         // {u32 ProfilerMsgType [, str path]}
    EXIT_CMD = 7,
};

// Sub-command of PROFILER_CMD.  Every record kind has a "set" (even) and an "unset" (odd) value; SAVE comes last.
#define LLIS_PROFILER_RECORD_KINDS(X) \
    X(KERNEL_INFO, 0)                 \
    X(BLOCK_EXEC_TIME, 1)             \
    X(KERNEL_BLOCK_MIS_ALLOC, 2)      \
    X(RUN_NEXT_TIMES, 3)              \
    X(JOB_EVENTS, 4)                  \
    X(RESOURCE_EVENTS, 5)

enum class ProfilerMsgType : uint32_t {
#define LLIS_PROFILER_MSG(kind, index) SET_RECORD_##kind = 2 * (index), UNSET_RECORD_##kind = 2 * (index) + 1,
    LLIS_PROFILER_RECORD_KINDS(LLIS_PROFILER_MSG)
#undef LLIS_PROFILER_MSG
    SAVE = 12,
};

namespace ipc {
// Whether LAUNCH_JOB carries the client's send time (std::chrono::steady_clock ticks, a u64 right behind the message type)
// so that the server can report the mean client-to-server latency of the request ring.  The reference compiles this in or
// out on both sides with -DPRINT_LAUNCH_JOB_IPC_LATENCY (reference CMakeLists.txt:27-45, src/client/job_instance_ref.cpp:35-38,
// src/server/server.cpp:121-141); here it is a process-wide run-time switch with the same default rule -- on when this
// library was built with that macro, else the environment variable LLIS_PRINT_LAUNCH_JOB_IPC_LATENCY=1, else off -- which
// `llis_server --print_ipc_latency` and `llis_app_client --print_ipc_latency` set.  Client and server must agree (the two
// encodings cannot be told apart on the ring), exactly as two reference builds must.
bool launch_timestamps();
void set_launch_timestamps(bool on);
}  // namespace ipc

static_assert((uint32_t)ProfilerMsgType::UNSET_RECORD_RESOURCE_EVENTS == 11 && (uint32_t)ProfilerMsgType::SET_RECORD_RUN_NEXT_TIMES == 6,
              "profiler sub-commands are wire values");

}  // namespace llis
