#pragma once
// Launch packing across the operator library's translation units (the packer itself is in ops_conv.hip).
//
// While a thread records a job's ordered launch sequence (paella_pack_sequence_begin / _end), the launch functions of
// the operators that a packed launch can carry hand their arguments to the recorder instead of launching; any other
// launch on that thread ends the recording first (what was recorded goes out, in order, ahead of it).

namespace paella {

struct PoolArgs;
struct DenseArgs;

extern thread_local bool g_pack_recording;

// True when the launch was taken into the sequence being recorded on this thread.
bool pack_record_pool(const PoolArgs& a, void* stream);
bool pack_record_dense(const DenseArgs& a, void* stream);

// Sends what the current recording holds so far to the sequence's queue and stops recording.
void pack_sequence_break_slow();
inline void pack_sequence_break() {
    if (g_pack_recording) pack_sequence_break_slow();
}

}  // namespace paella
