// TEST INFRASTRUCTURE: the host side of the CPU execution model (see amdgcn_emu.hpp) -- device
// memory, kernel launches and the handful of HIP runtime calls the library's host code makes, so
// that the library's own source (workspace logic, launch geometry, heuristics, the C ABI) runs on
// the CPU as it is.
//
//   device memory   a shared anonymous mapping per allocation, between two inaccessible pages and
//                   ending at the upper one; the list of allocations is what emu_check consults
//   a launch        runs to completion before the call returns (every stream is synchronous): one
//                   forked process per workgroup, all alive together, 64 threads per wave
//   the device      EMU_CUS compute units (environment, default 3) with 160 KB of LDS each; the
//                   occupancy query divides that by a kernel's LDS and caps the result at 4
//   graph capture   one capture at a time, of every stream at once (emu_capture_begin / _end, for
//                   the test harness): launches are recorded with their arguments instead of run,
//                   and run in order at every replay; an allocation, a copy or a memset while a
//                   capture is under way ends the run with a report (the library must not make one)
//
// One translation unit of a program defines EMU_DEFINE_GLOBALS before including this.
#pragma once

#include <signal.h>
#include <stdio_ext.h>
#include <sys/mman.h>
#include <sys/prctl.h>
#include <sys/wait.h>
#include <unistd.h>

#include <functional>
#include <vector>

#include "amdgcn_emu.hpp"

// ---------------------------------------------------------------- device memory
const size_t emu_page = 4096;

// (the list is shared by the host threads of a program: ranks of a ring that allocate side by side)
extern pthread_mutex_t emu_alloc_lock;
struct emu_locked {
    pthread_mutex_t *m;
    explicit emu_locked(pthread_mutex_t *m_) : m(m_) { pthread_mutex_lock(m); }
    ~emu_locked() { pthread_mutex_unlock(m); }
};

// `bytes` of shared memory that end (rounded up to `align`) at an inaccessible page and start behind one
inline void *emu_device_alloc_named(size_t bytes, const char *name, size_t align = 256)
{
    const emu_locked lock(&emu_alloc_lock);
    if (emu_n_allocs >= (int)(sizeof emu_allocs / sizeof emu_allocs[0])) {
        fprintf(stderr, "EMU: too many allocations\n");
        abort();
    }
    const size_t room = (bytes + align - 1) / align * align + (bytes ? 0 : align);
    const size_t pages = (room + emu_page - 1) / emu_page * emu_page;
    uint8_t *m = (uint8_t *)mmap(nullptr, pages + 2 * emu_page, PROT_NONE, MAP_SHARED | MAP_ANONYMOUS, -1, 0);
    if (m == MAP_FAILED || mprotect(m + emu_page, pages, PROT_READ | PROT_WRITE) != 0) return nullptr;
    uint8_t *p = m + emu_page + pages - room;
    emu_allocs[emu_n_allocs++] = emu_alloc{(uintptr_t)p, (uintptr_t)p + room, name, (uintptr_t)m, pages + 2 * emu_page};
    return p;
}
inline bool emu_device_free(void *p)
{
    const emu_locked lock(&emu_alloc_lock);
    for (int i = 0; i < emu_n_allocs; ++i)
        if (emu_allocs[i].lo == (uintptr_t)p) {
            munmap((void *)emu_allocs[i].map, emu_allocs[i].map_bytes);
            emu_allocs[i] = emu_allocs[--emu_n_allocs];
            return true;
        }
    return false;
}

// ---------------------------------------------------------------- launches
// the section of the `__shared__` arrays of this program or library (absent if it has none)
extern "C" uint8_t __start_emu_lds[] __attribute__((weak, visibility("hidden"))), __stop_emu_lds[] __attribute__((weak, visibility("hidden")));

// A worker process runs the workgroups first, first + step, ... of a grid one after the other, with
// one thread per wave and one set of lane stacks for all of them.
struct emu_worker {
    const std::function<void()> *kernel;
    unsigned threads, first, step, blocks, grid_x;
};
struct emu_wave_start {
    const emu_worker *worker;
    unsigned index;   // of the wave in its workgroup
};
const size_t emu_lane_stack = 1 << 20;   // per lane; only the pages a lane touches exist

// where a lane starts, and where it ends up when it leaves the kernel
extern "C" inline void emu_lane_entry()
{
    emu_wave *w = emu_wave_of_thread;
#ifdef EMU_ASAN
    {   // first time on this stack; the wave's first lane learns the thread's own stack from it
        const void *from = nullptr;
        size_t from_bytes = 0;
        __sanitizer_finish_switch_fiber(nullptr, &from, &from_bytes);
        if (!w->main_stack) {
            w->main_stack = from;
            w->main_stack_bytes = from_bytes;
        }
    }
#endif
    (*(const std::function<void()> *)w->kernel)();
    emu_lane_ctx *me = emu_cur;
    me->done = true;
    w->live--;
    if (w->live == 0) {
        emu_switch_stacks(&me->sp, w->main_sp, w->main_stack, w->main_stack_bytes, true);   // the wave is through; does not come back
    }
    if (w->arrived == w->live) {                 // the others were waiting for this lane only
        emu_note_present(w, 0);
        emu_note_present(w, 1);
        emu_release(w);
    }
    emu_next_lane(w);                             // does not come back either
    abort();
}

inline void *emu_wave_main(void *arg)
{
    const emu_wave_start *s = (const emu_wave_start *)arg;
    const emu_worker *k = s->worker;
    emu_wave *w = new emu_wave;
    emu_wave_of_thread = w;
    w->kernel = k->kernel;
    w->stack_bytes = emu_lane_stack;
    w->count = k->threads - 64 * s->index < 64 ? k->threads - 64 * s->index : 64;
    uint8_t *stacks = (uint8_t *)mmap(nullptr, 64 * emu_lane_stack, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (stacks == MAP_FAILED) {
        perror("EMU: lane stacks");
        _exit(3);
    }
    for (unsigned l = 0; l < 64; ++l) mprotect(stacks + l * emu_lane_stack, emu_page, PROT_NONE);   // a lane that outgrows its stack faults
    w->stacks = stacks;
    for (unsigned i = k->first; i < k->blocks; i += k->step) {
        if (s->index == 0) {
            blockIdx.x = i % k->grid_x;
            blockIdx.y = i / k->grid_x;
            // LDS as the workgroup finds it: not zeros
            for (uint8_t *b = __start_emu_lds; b && b != __stop_emu_lds; ++b) *b = (uint8_t)(0xC3u ^ (uintptr_t)b * 37u ^ i * 11u);
        }
        for (unsigned l = 0; l < w->count; ++l) {
            emu_lane_ctx &c = w->lanes[l];
            c.tid = emu_dim3(64 * s->index + l);
            c.lane = (int)l;
            c.parity = 0;
            c.call_seq = 0;
            c.done = false;
            // the frame emu_switch pops: six callee-saved registers, then the address it returns to; the
            // stack pointer after that return is 8 below a multiple of 16, as at any function's entry
            uint64_t *top = (uint64_t *)(stacks + (l + 1) * emu_lane_stack);
            top[-2] = (uint64_t)(uintptr_t)&emu_lane_entry;
            for (int r = 3; r <= 8; ++r) top[-r] = 0;
            c.sp = top - 8;
        }
        w->live = w->count;
        w->arrived = 0;
        w->gen = 0;
        w->log.clear();
        w->n_guards = 0;
        if (s->index == 0) emu_dynamic_lds = nullptr;
        pthread_barrier_wait(&emu_block_barrier);
        emu_cur = &w->lanes[0];
        w->main_stack = nullptr;
        emu_switch_stacks(&w->main_sp, w->lanes[0].sp, stacks, emu_lane_stack);   // back here when the wave's last lane has left the kernel
        pthread_barrier_wait(&emu_block_barrier);
        // nothing was written behind a part of LDS that is this wave's own, by any wave (the pattern emu_guard_behind laid)
        for (unsigned g = 0; g < w->n_guards; ++g)
            for (unsigned b = 0; b < EMU_SLOT_GUARD; ++b)
                if (w->guards[g][b] != 0xD6u) {
                    fprintf(stderr, "EMU: block %u wrote beyond a part of LDS of wave %u (byte %u behind its end)\n", i, s->index, b);
                    if (getenv("EMU_TRACE")) {
                        fprintf(stderr, "EMU: guard %u of the wave, at %p:", g, (void *)w->guards[g]);
                        for (unsigned k = 0; k < 48; ++k) fprintf(stderr, " %02x", w->guards[g][k]);
                        fprintf(stderr, "\n");
                    }
                    _exit(5);
                }
        if (s->index == 0 && emu_dynamic_lds) {
            // nothing was written beyond the dynamic LDS the launch asked for (the pattern emu_note_dynamic_lds laid)
            uint8_t *const end = emu_dynamic_lds + emu_dynamic_lds_bytes + emu_dynamic_lds_extra;
            for (uint8_t *b = end; b != emu_dynamic_lds + EMU_DYN_LDS + emu_dynamic_lds_extra; ++b)
                if (*b != 0xD5u) {
                    fprintf(stderr, "EMU: block %u wrote %zu bytes beyond its %zu bytes of dynamic LDS\n", i,
                            (size_t)(b - end) + 1, emu_dynamic_lds_bytes);
                    _exit(5);
                }
        }
        pthread_barrier_wait(&emu_block_barrier);   // the next workgroup's LDS pattern is laid when every wave has looked at its guards
    }
    munmap(stacks, 64 * emu_lane_stack);
    delete w;
    return nullptr;
}

inline void emu_run_worker(emu_worker &k)
{
    const unsigned waves = (k.threads + 63) / 64;
    pthread_barrier_init(&emu_block_barrier, nullptr, waves);
    pthread_t *th = new pthread_t[waves];
    emu_wave_start *st = new emu_wave_start[waves];
    pthread_attr_t attr;
    pthread_attr_init(&attr);
    pthread_attr_setstacksize(&attr, 1 << 20);
    for (unsigned i = 0; i < waves; ++i) {
        st[i] = emu_wave_start{&k, i};
        if (pthread_create(&th[i], &attr, emu_wave_main, &st[i]) != 0) {
            perror("EMU: pthread_create");
            _exit(3);
        }
    }
    for (unsigned i = 0; i < waves; ++i) pthread_join(th[i], nullptr);
}

// A grid.  Up to emu_resident_limit() workgroups are alive at the same time, each in a process of
// its own (the kernels whose workgroups wait for one another size their grids far below that).
// The workgroups of a larger grid are dealt out to that many worker processes in turn, which run
// theirs in index order: the unfinished workgroup with the smallest index is always running, which
// is what a kernel may rely on (a workgroup only ever waits for workgroups with smaller indices).
// Returns false when a workgroup ended abnormally (an access beyond a buffer, an abort of the model).
extern pthread_mutex_t emu_launch_lock;
inline unsigned emu_resident_limit()
{
    const char *e = getenv("EMU_RESIDENT");
    const int v = e ? atoi(e) : 48;
    return v < 1 ? 1u : (unsigned)v;
}
inline bool emu_run_grid(const std::function<void()> &kernel, emu_dim3 grid, emu_dim3 block, size_t dyn_lds = EMU_DYN_LDS)
{
    const emu_locked lock(&emu_launch_lock);   // one launch at a time, whichever host thread makes it
    emu_dynamic_lds_bytes = dyn_lds;
    gridDim = grid;
    blockDim = block;
    const unsigned n = grid.x * grid.y * grid.z, limit = emu_resident_limit(), workers = n < limit ? n : limit;
    pid_t *kids = new pid_t[workers];
    const pid_t parent = getpid();
    if (getenv("EMU_TRACE")) fprintf(stderr, "EMU: a grid of %u workgroups of %u lanes, %u at a time\n", n, block.x, workers);
    unsigned started = 0;
    bool ok = true;
    fflush(nullptr);
    // the workers check accesses against the list of buffers as it is when they start: no other host
    // thread is half-way through changing it then (the workers never take this lock themselves)
    pthread_mutex_lock(&emu_alloc_lock);
    for (unsigned i = 0; i < workers; ++i) {
        const pid_t k = fork();
        if (k < 0) {
            perror("EMU: fork");
            ok = false;
            break;
        }
        if (k == 0) {
            // a worker does not outlive the program that launched it (one that was killed at a time limit, say)
            prctl(PR_SET_PDEATHSIG, SIGKILL);
            if (getppid() != parent) _exit(6);
            // The worker inherits a copy of every stdio buffer as it was at the fork, with whatever another
            // host thread had in it at that moment (the unwritten end of a file, half a line): none of that
            // is the worker's to write.  What the program's standard output held is dropped, the other
            // streams are never flushed here (_exit), and only what the kernel itself prints goes out.
            __fpurge(stdout);
            emu_worker w{&kernel, block.x, i, workers, n, grid.x};
            emu_run_worker(w);
            fflush(stdout);
            _exit(0);
        }
        kids[started++] = k;
    }
    pthread_mutex_unlock(&emu_alloc_lock);
    for (unsigned i = 0; i < started; ++i) {
        int status = 0;
        waitpid(kids[i], &status, 0);
        if (!WIFEXITED(status) || WEXITSTATUS(status) != 0) {
            fprintf(stderr, "EMU: a workgroup ended abnormally (status 0x%x%s)\n", status,
                    WIFSIGNALED(status) && WTERMSIG(status) == SIGSEGV ? ": segmentation fault, an access beyond a buffer" : "");
            ok = false;
        }
    }
    delete[] kids;
    return ok;
}

// ---------------------------------------------------------------- the HIP runtime calls of the library's host code
typedef int hipError_t;
typedef void *hipStream_t;
typedef void *hipEvent_t;
constexpr hipError_t hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2, hipErrorLaunchFailure = 719;
extern thread_local hipError_t emu_last_error;
inline const char *hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "an error of the emulated runtime"; }
inline hipError_t hipGetLastError()
{
    const hipError_t e = emu_last_error;
    emu_last_error = hipSuccess;
    return e;
}

// ---- graph capture
struct emu_graph {
    std::vector<std::function<bool()>> launches;
};
extern emu_graph *emu_capturing;            // the graph under construction, if any
extern unsigned long long emu_capture_id;   // of that capture (unique per capture)
inline void emu_not_while_capturing(const char *what)
{
    if (emu_capturing) {
        fprintf(stderr, "EMU: %s while a graph is being captured\n", what);
        abort();
    }
}
inline emu_graph *emu_capture_begin()
{
    emu_not_while_capturing("a second capture");
    ++emu_capture_id;
    return emu_capturing = new emu_graph;
}
inline emu_graph *emu_capture_end()
{
    emu_graph *g = emu_capturing;
    emu_capturing = nullptr;
    return g;
}
inline bool emu_graph_replay(emu_graph *g)
{
    for (const std::function<bool()> &launch : g->launches)
        if (!launch()) return false;
    return true;
}

// hipLaunchKernelGGL(kernel, grid, block, dynamic LDS, stream, arguments...)
template <typename K, typename... A>
inline void emu_launch(K kernel, emu_dim3 grid, emu_dim3 block, size_t dyn_lds, hipStream_t, A... args)
{
    if (dyn_lds > EMU_DYN_LDS || grid.x == 0 || block.x == 0 || block.x > 1024) {
        emu_last_error = hipErrorInvalidValue;
        return;
    }
    const std::function<void()> body = [=]() { kernel(args...); };
    if (emu_capturing) {
        emu_capturing->launches.push_back([=]() { return emu_run_grid(body, grid, block, dyn_lds); });
        return;
    }
    if (!emu_run_grid(body, grid, block, dyn_lds)) emu_last_error = hipErrorLaunchFailure;
}
#define hipLaunchKernelGGL(kernel, grid, block, dyn, stream, ...) emu_launch(kernel, grid, block, dyn, stream, __VA_ARGS__)

inline hipError_t hipMalloc(void **p, size_t bytes)
{
    emu_not_while_capturing("hipMalloc");
    *p = emu_device_alloc_named(bytes, "hipMalloc");
    if (*p) memset(*p, 0xB6, bytes);   // fresh device memory is not zero
    return *p ? hipSuccess : hipErrorOutOfMemory;
}
template <typename T>
inline hipError_t hipMalloc(T **p, size_t bytes)
{
    return hipMalloc((void **)p, bytes);
}
inline hipError_t hipFree(void *p) { return !p || emu_device_free(p) ? hipSuccess : hipErrorInvalidValue; }
constexpr unsigned hipHostMallocDefault = 0;
inline hipError_t hipHostMalloc(void **p, size_t bytes, unsigned)
{
    *p = emu_device_alloc_named(bytes, "hipHostMalloc");
    return *p ? hipSuccess : hipErrorOutOfMemory;
}
inline hipError_t hipHostFree(void *p) { return hipFree(p); }
inline hipError_t hipMemset(void *p, int v, size_t bytes)
{
    emu_not_while_capturing("a memset (a memset node in a graph has given wrong results on replays; the library fills with a kernel)");
    emu_check(p, bytes, "hipMemset");
    memset(p, v, bytes);
    return hipSuccess;
}
enum hipMemcpyKind { hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice, hipMemcpyDefault };
inline hipError_t hipMemcpy(void *dst, const void *src, size_t bytes, hipMemcpyKind kind)
{
    emu_not_while_capturing("a copy");
    // the side that is device memory must lie inside an allocation
    if (kind == hipMemcpyHostToDevice || kind == hipMemcpyDeviceToDevice) emu_check(dst, bytes, "hipMemcpy (destination)");
    if (kind == hipMemcpyDeviceToHost || kind == hipMemcpyDeviceToDevice) emu_check(src, bytes, "hipMemcpy (source)");
    memmove(dst, src, bytes);
    return hipSuccess;
}
inline hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind kind, hipStream_t) { return hipMemcpy(dst, src, bytes, kind); }
inline hipError_t hipMemsetAsync(void *p, int v, size_t bytes, hipStream_t) { return hipMemset(p, v, bytes); }
inline hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidValue; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
inline hipError_t hipDeviceSynchronize() { return hipSuccess; }
inline hipError_t hipGetDevice(int *d)
{
    *d = 0;
    return hipSuccess;
}
inline hipError_t hipGetDeviceCount(int *n)
{
    *n = 1;
    return hipSuccess;
}
struct hipDeviceProp_t {
    int multiProcessorCount;
};
inline int emu_compute_units()
{
    const char *e = getenv("EMU_CUS");
    const int v = e ? atoi(e) : 3;
    return v < 1 ? 1 : (v > 256 ? 256 : v);
}
inline hipError_t hipGetDeviceProperties(hipDeviceProp_t *prop, int)
{
    prop->multiProcessorCount = emu_compute_units();
    return hipSuccess;
}
constexpr unsigned hipEventDisableTiming = 2;
inline hipError_t hipEventCreateWithFlags(hipEvent_t *e, unsigned)
{
    *e = (hipEvent_t)(uintptr_t)1;
    return hipSuccess;
}
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
inline hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
enum hipStreamCaptureStatus { hipStreamCaptureStatusNone, hipStreamCaptureStatusActive, hipStreamCaptureStatusInvalidated };
inline hipError_t hipStreamGetCaptureInfo(hipStream_t, hipStreamCaptureStatus *status, unsigned long long *id)
{
    *status = emu_capturing ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone;
    if (id) *id = emu_capturing ? emu_capture_id : 0;
    return hipSuccess;
}
// A kernel's LDS is not known to this model: every kernel is taken to have the static LDS of the
// largest one of the library, which only makes the emulated grids a little smaller.
struct hipFuncAttributes {
    size_t sharedSizeBytes;
};
constexpr size_t emu_static_lds = 20480;
inline hipError_t hipFuncGetAttributes(hipFuncAttributes *fa, const void *)
{
    fa->sharedSizeBytes = emu_static_lds;
    return hipSuccess;
}
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize };
inline hipError_t hipFuncSetAttribute(const void *, hipFuncAttribute, int bytes) { return bytes <= EMU_DYN_LDS ? hipSuccess : hipErrorInvalidValue; }
template <typename K>
inline hipError_t hipOccupancyMaxActiveBlocksPerMultiprocessor(int *blocks, K, int, size_t dyn)
{
    const size_t per = emu_static_lds + dyn;
    *blocks = (int)(160u * 1024u / per);
    if (*blocks > 8) *blocks = 8;
    return hipSuccess;
}
// The address of a `__device__` array: the array itself lives in the program's private memory,
// which workgroups (processes) cannot share, so a shared mapping of its size stands in for it.
#define HIP_SYMBOL(x) (&(x)), sizeof(x)
inline hipError_t hipGetSymbolAddress(void **p, const void *symbol, size_t bytes)
{
    static const void *known[8];
    static void *mapped[8];
    for (int i = 0; i < 8; ++i)
        if (known[i] == symbol) {
            *p = mapped[i];
            return hipSuccess;
        }
    for (int i = 0; i < 8; ++i)
        if (!known[i]) {
            mapped[i] = emu_device_alloc_named(bytes, "__device__ array");
            if (!mapped[i]) return hipErrorOutOfMemory;
            memset(mapped[i], 0, bytes);   // static storage starts as zeros on the device as well
            known[i] = symbol;
            *p = mapped[i];
            return hipSuccess;
        }
    return hipErrorInvalidValue;
}

#ifdef EMU_DEFINE_GLOBALS
emu_dim3 blockIdx, gridDim, blockDim;
thread_local emu_wave *emu_wave_of_thread = nullptr;
thread_local emu_lane_ctx *emu_cur = nullptr;
pthread_barrier_t emu_block_barrier;
uint8_t *emu_dynamic_lds = nullptr;
size_t emu_dynamic_lds_bytes = 0;
size_t emu_dynamic_lds_extra = 0;
emu_graph *emu_capturing = nullptr;
unsigned long long emu_capture_id = 0;
emu_alloc emu_allocs[8192];
int emu_n_allocs = 0;
thread_local hipError_t emu_last_error = hipSuccess;
pthread_mutex_t emu_alloc_lock = PTHREAD_MUTEX_INITIALIZER, emu_launch_lock = PTHREAD_MUTEX_INITIALIZER;
// emu_switch(save_sp, load_sp), x86-64 System V: the registers a call preserves go onto the running
// lane's stack, its stack pointer into *save_sp; the other lane's are taken up the same way round
asm(R"(
    .text
    .globl emu_switch
    .type emu_switch,@function
emu_switch:
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
    .size emu_switch, .-emu_switch
)");
#endif
