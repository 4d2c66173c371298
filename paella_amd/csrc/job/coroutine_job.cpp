// Stackful coroutine under CoroutineJob: a callee-saved-register context switch for x86-64 System V.

#include <llis/job/coroutine_job.h>
#include <llis/utils/error.h>

#include <sys/mman.h>
#include <unistd.h>

#include <cstdint>
#include <cstdlib>

#if !defined(__x86_64__)
#error "the coroutine context switch is written for x86-64 System V"
#endif

// void llis_ctx_switch(void** save_sp, void* load_sp)
// Pushes the callee-saved registers, stores the stack pointer through save_sp, adopts load_sp and pops the
// registers that the other side pushed.  A fresh stack is laid out so that the final `ret` enters the trampoline.
asm(R"(
    .text
    .globl llis_ctx_switch
    .type llis_ctx_switch,@function
llis_ctx_switch:
    pushq %rbp
    pushq %rbx
    pushq %r12
    pushq %r13
    pushq %r14
    pushq %r15
    movq %rsp, (%rdi)
    movq %rsi, %rsp
    popq %r15
    popq %r14
    popq %r13
    popq %r12
    popq %rbx
    popq %rbp
    ret
    .size llis_ctx_switch,.-llis_ctx_switch
)");

extern "C" void llis_ctx_switch(void** save_sp, void* load_sp);

namespace llis {
namespace job {

namespace {
// The job whose body() is being entered for the first time (the server drives jobs from one thread, but
// keep it per thread so tests may drive independent jobs from several).
thread_local CoroutineJob* g_starting = nullptr;
}  // namespace

CoroutineJob::~CoroutineJob() {
    if (stack_base_) munmap(stack_base_, kStackBytes + (size_t)sysconf(_SC_PAGE_SIZE));
}

void CoroutineJob::entry_trampoline() {
    CoroutineJob* self = g_starting;
    g_starting = nullptr;
    self->body(self->io_ptr_);
    self->finished_ = true;
    // Leave for good: nobody resumes a finished coroutine.
    void* dead;
    llis_ctx_switch(&dead, self->caller_sp_);
    std::abort();
}

void CoroutineJob::init(void* io_ptr) {
    const size_t page = (size_t)sysconf(_SC_PAGE_SIZE);
    if (!stack_base_) {
        void* p = mmap(nullptr, kStackBytes + page, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_STACK, -1, 0);
        LLIS_CHECK_POSIX_PTR(p, MAP_FAILED);
        LLIS_CHECK_POSIX(mprotect(p, page, PROT_NONE));  // overflow faults instead of corrupting the heap
        stack_base_ = p;
    }
    io_ptr_ = io_ptr;
    finished_ = false;

    // Fresh frame, top down: [pad][&entry_trampoline][six zeroed callee-saved slots] <- sp.
    // After the switch pops six registers and returns, rsp % 16 == 8, as at any function entry.
    uintptr_t top = (reinterpret_cast<uintptr_t>(stack_base_) + page + kStackBytes) & ~(uintptr_t)15;
    void** sp = reinterpret_cast<void**>(top - 64);
    for (int i = 0; i < 6; ++i) sp[i] = nullptr;
    sp[6] = reinterpret_cast<void*>(&CoroutineJob::entry_trampoline);
    sp[7] = nullptr;
    coroutine_sp_ = sp;

    g_starting = this;
    llis_ctx_switch(&caller_sp_, coroutine_sp_);  // runs body() up to its first yield()
}

void CoroutineJob::resume() {
    if (finished_) return;
    llis_ctx_switch(&caller_sp_, coroutine_sp_);
}

void CoroutineJob::yield() { llis_ctx_switch(&coroutine_sp_, caller_sp_); }

}  // namespace job
}  // namespace llis
