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
//   graph capture   does not exist here: no stream is ever capturing
//
// One translation unit of a program defines EMU_DEFINE_GLOBALS before including this.
#pragma once

#include <sys/mman.h>
#include <sys/wait.h>
#include <unistd.h>

#include <functional>

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
// one set of lane threads for all of them (starting 256 threads per workgroup is what a large grid
// of small workgroups would otherwise spend its time on).
struct emu_worker {
    const std::function<void()> *kernel;
    emu_wave *waves;
    unsigned threads, first, step, blocks, grid_x;
};
struct emu_lane_start {
    const emu_worker *worker;
    int tid;
};
inline void *emu_lane_main(void *arg)
{
    const emu_lane_start *s = (const emu_lane_start *)arg;
    const emu_worker *w = s->worker;
    threadIdx.x = (unsigned)s->tid;
    emu_lane = s->tid & 63;
    emu_wave_of_thread = &w->waves[s->tid / 64];
    for (unsigned i = w->first; i < w->blocks; i += w->step) {
        if (s->tid == 0) {
            blockIdx.x = i % w->grid_x;
            blockIdx.y = i / w->grid_x;
            // LDS as the workgroup finds it: not zeros
            for (uint8_t *b = __start_emu_lds; b && b != __stop_emu_lds; ++b) *b = (uint8_t)(0xC3u ^ (uintptr_t)b * 37u ^ i * 11u);
        }
        emu_parity = 0;
        emu_call_seq = 0;
        emu_dirty = false;
        pthread_barrier_wait(&emu_block_barrier);
        (*w->kernel)();
        pthread_barrier_wait(&emu_block_barrier);
    }
    return nullptr;
}

inline void emu_run_worker(emu_worker &w)
{
    const unsigned threads = w.threads, waves = (threads + 63) / 64;
    w.waves = new emu_wave[waves];
    for (unsigned i = 0; i < waves; ++i) pthread_barrier_init(&w.waves[i].bar, nullptr, i + 1 < waves || threads % 64 == 0 ? 64 : threads % 64);
    pthread_barrier_init(&emu_block_barrier, nullptr, threads);
    pthread_t *th = new pthread_t[threads];
    emu_lane_start *st = new emu_lane_start[threads];
    pthread_attr_t attr;
    pthread_attr_init(&attr);
    pthread_attr_setstacksize(&attr, 1 << 20);
    for (unsigned t = 0; t < threads; ++t) {
        st[t] = emu_lane_start{&w, (int)t};
        if (pthread_create(&th[t], &attr, emu_lane_main, &st[t]) != 0) {
            perror("EMU: pthread_create");
            _exit(3);
        }
    }
    for (unsigned t = 0; t < threads; ++t) pthread_join(th[t], nullptr);
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
inline bool emu_run_grid(const std::function<void()> &kernel, emu_dim3 grid, emu_dim3 block)
{
    const emu_locked lock(&emu_launch_lock);   // one launch at a time, whichever host thread makes it
    gridDim = grid;
    blockDim = block;
    const unsigned n = grid.x * grid.y * grid.z, limit = emu_resident_limit(), workers = n < limit ? n : limit;
    pid_t *kids = new pid_t[workers];
    unsigned started = 0;
    bool ok = true;
    fflush(nullptr);
    for (unsigned i = 0; i < workers; ++i) {
        const pid_t k = fork();
        if (k < 0) {
            perror("EMU: fork");
            ok = false;
            break;
        }
        if (k == 0) {
            emu_worker w{&kernel, nullptr, block.x, i, workers, n, grid.x};
            emu_run_worker(w);
            fflush(nullptr);
            _exit(0);
        }
        kids[started++] = k;
    }
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

// hipLaunchKernelGGL(kernel, grid, block, dynamic LDS, stream, arguments...)
template <typename K, typename... A>
inline void emu_launch(K kernel, emu_dim3 grid, emu_dim3 block, size_t dyn_lds, hipStream_t, A... args)
{
    if (dyn_lds > EMU_DYN_LDS || grid.x == 0 || block.x == 0 || block.x > 1024) {
        emu_last_error = hipErrorInvalidValue;
        return;
    }
    const std::function<void()> body = [=]() { kernel(args...); };
    if (!emu_run_grid(body, grid, block)) emu_last_error = hipErrorLaunchFailure;
}
#define hipLaunchKernelGGL(kernel, grid, block, dyn, stream, ...) emu_launch(kernel, grid, block, dyn, stream, __VA_ARGS__)

inline hipError_t hipMalloc(void **p, size_t bytes)
{
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
    emu_check(p, bytes, "hipMemset");
    memset(p, v, bytes);
    return hipSuccess;
}
enum hipMemcpyKind { hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice, hipMemcpyDefault };
inline hipError_t hipMemcpy(void *dst, const void *src, size_t bytes, hipMemcpyKind kind)
{
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
    return v < 1 ? 1 : (v > 16 ? 16 : v);
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
    *status = hipStreamCaptureStatusNone;
    if (id) *id = 0;
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
thread_local emu_dim3 threadIdx;
emu_dim3 blockIdx, gridDim, blockDim;
thread_local emu_wave *emu_wave_of_thread = nullptr;
thread_local int emu_lane = 0;
thread_local unsigned emu_parity = 0;
thread_local uint32_t emu_call_seq = 0;
thread_local bool emu_dirty = false;
pthread_barrier_t emu_block_barrier;
emu_alloc emu_allocs[1024];
int emu_n_allocs = 0;
thread_local hipError_t emu_last_error = hipSuccess;
pthread_mutex_t emu_alloc_lock = PTHREAD_MUTEX_INITIALIZER, emu_launch_lock = PTHREAD_MUTEX_INITIALIZER;
#endif
