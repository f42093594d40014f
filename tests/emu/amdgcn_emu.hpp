// TEST INFRASTRUCTURE: a host-side execution model for the device code of the HomComp kernels.
//
// The kernels under tirocinio-triennale_amd/csrc are written against wave64 primitives (DPP lane
// permutations, ballots, readlane, byte permutes, range-checked buffer accesses, LDS shared by a
// workgroup, device-scope words other workgroups poll).  This header gives those primitives a
// plain C++ meaning so that the same source text runs on the CPU:
//
//   lane        a fiber (a stack and a saved stack pointer) of its wave's thread; a wave is one
//               OS thread that runs its 64 lanes in turn, a workgroup four such threads in one
//               process
//   workgroup   one process (forked by the driver): `__shared__` becomes `static`, so every
//               process has its own copy, like every workgroup its own LDS
//   device      memory: one shared anonymous mapping created before the fork, same addresses in
//               every process; device-scope atomics are host atomics on it
//   cross-lane  operations: the lanes of a wave meet -- each leaves its value and gives way to
//               the next lane until all that have not left the kernel are there -- exchange
//               through a slot array and go on.  All of them must be at the same place of the
//               program, as on the hardware all lanes must be active for DPP: a meeting of
//               lanes at different places ends the run with a report.  wave_lds_fence is such a
//               meeting too, because the lanes do not run in lockstep
//
// It models what the instruction set defines (lane sources of the DPP controls, byte selectors of
// v_perm, field extracts, saturating conversion, zero for loads and nothing for stores beyond a
// buffer descriptor's byte count).  It does not model timing, register allocation or the
// compiler: it checks the kernels' logic and their address arithmetic, not their code generation.
// Nothing under tirocinio-triennale_amd/ includes this file.
#pragma once

#include <pthread.h>
#include <sched.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <algorithm>
#include <cmath>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
// LDS: one copy per process, in a section of its own so that the driver can fill all of it with
// a pattern before a workgroup starts (the hardware hands a workgroup whatever the last one left)
#define __shared__ static __attribute__((section("emu_lds")))
#define __align__(n) __attribute__((aligned(n)))
#define amdgpu_waves_per_eu(n) unused

// ---------------------------------------------------------------- thread identity
struct emu_dim3 {
    unsigned x, y, z;
    emu_dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
typedef emu_dim3 dim3;
extern emu_dim3 blockIdx, gridDim, blockDim;   // one workgroup per process

// A byte store whose place in the wave's instruction stream matters (see emu_ordered_store8).
struct emu_store {
    uint8_t *addr;
    uint32_t seq;
    uint8_t value;
};
struct emu_lane_ctx {
    emu_dim3 tid;        // threadIdx
    int lane;
    unsigned parity;     // which of the two slot arrays its next meeting uses
    uint32_t call_seq;   // see emu_ordered_store8
    void *sp;            // its stack pointer while another lane runs
    bool done;           // has left the kernel
};
struct emu_wave {
    emu_lane_ctx lanes[64];
    unsigned count;            // lanes of the wave (64; fewer in the last wave of an odd workgroup)
    unsigned live;             // lanes that have not left the kernel
    unsigned arrived, gen;     // of the meeting under way; meetings so far
    unsigned site;             // the place in the program the meeting's first lane came from
    uint64_t slot[2][64];
    uint64_t present[2];       // the lanes that took part in the meeting whose values the slot array holds
    std::vector<emu_store> log;
    void *main_sp;             // the wave thread's own stack pointer while its lanes run
    const uint8_t *stacks;     // the lanes' stacks, one after the other, stack_bytes each
    size_t stack_bytes;
    const void *main_stack;    // the wave thread's own stack (known to a sanitizer build only)
    size_t main_stack_bytes;
    const void *kernel;        // std::function<void()> of the launch
    uint8_t *guards[16];       // behind the parts of LDS that are this wave's own, in the workgroup under way (emu_guard_behind)
    unsigned n_guards;
};
extern thread_local emu_wave *emu_wave_of_thread;
extern thread_local emu_lane_ctx *emu_cur;   // the lane that is running on this thread
#define threadIdx (emu_cur->tid)
#define emu_lane (emu_cur->lane)
extern pthread_barrier_t emu_block_barrier;   // of the workgroup's wave threads
// Dynamic LDS: the array that stands for it has the size of the largest launch; what lies beyond
// the size of the launch under way holds a pattern that must still be there when a workgroup ends.
extern uint8_t *emu_dynamic_lds;          // where the running kernel's array is (a kernel with one says so)
extern size_t emu_dynamic_lds_bytes;      // of the launch under way
extern size_t emu_dynamic_lds_extra;      // bytes the model adds between the parts of the array (emu_stage_slot); the array is that much longer
inline void emu_note_dynamic_lds(uint8_t *array, size_t extra = 0)
{
    // the first lane of the workgroup to come by lays the pattern (nothing has used the array yet)
    if (__sync_bool_compare_and_swap(&emu_dynamic_lds, (uint8_t *)nullptr, array)) {
        emu_dynamic_lds_extra = extra;
        memset(array + emu_dynamic_lds_bytes + extra, 0xD5, EMU_DYN_LDS - emu_dynamic_lds_bytes);
    }
}
// Guards inside LDS: EMU_SLOT_GUARD bytes of pattern behind a part of an array that belongs to one
// wave, laid at the wave's first mention of it and intact when the workgroup ends -- or a wave
// has written beyond its part, which the end of the whole array would not show.
#define EMU_SLOT_GUARD 256
inline void emu_guard_behind(uint8_t *end_of_part)
{
    emu_wave *w = emu_wave_of_thread;
    for (unsigned i = 0; i < w->n_guards; ++i)
        if (w->guards[i] == end_of_part) return;
    if (w->n_guards == sizeof w->guards / sizeof w->guards[0]) {
        fprintf(stderr, "EMU: a wave with more guarded parts of LDS than the model keeps track of\n");
        abort();
    }
    memset(end_of_part, 0xD6, EMU_SLOT_GUARD);   // the wave's first mention of the part: nothing is in it yet
    w->guards[w->n_guards++] = end_of_part;
}
// A kernel that cuts its dynamic LDS into slots (`slots` per wave, `slot_bytes` each) gets them
// with a guard behind each.
inline uint8_t *emu_stage_slot(uint8_t *array, uint32_t wave, uint32_t slot, uint32_t slots, uint32_t slot_bytes)
{
    uint8_t *at = array + (size_t)(wave * slots + slot) * ((size_t)slot_bytes + EMU_SLOT_GUARD);
    emu_guard_behind(at + slot_bytes);
    return at;
}

// Every access a kernel makes to "device memory" must fall into a registered allocation; the
// first one that does not is reported with its address and aborts the run.
struct emu_alloc {
    uintptr_t lo, hi;
    const char *name;
    uintptr_t map;      // the mapping around it (guard pages included), for its release
    size_t map_bytes;
};
extern emu_alloc emu_allocs[8192];
extern int emu_n_allocs;
inline void emu_check(const void *p, size_t bytes, const char *what)
{
    const uintptr_t a = (uintptr_t)p;
    for (int i = 0; i < emu_n_allocs; ++i)
        if (a >= emu_allocs[i].lo && a + bytes <= emu_allocs[i].hi) return;
    fprintf(stderr, "EMU: %s of %zu bytes at %p is outside every buffer (block %u thread %u)\n", what, bytes, p, blockIdx.x,
            threadIdx.x);
    for (int i = 0; i < emu_n_allocs; ++i)
        fprintf(stderr, "   %-12s [%p, %p)\n", emu_allocs[i].name, (void *)emu_allocs[i].lo, (void *)emu_allocs[i].hi);
    fflush(stderr);
    abort();
}

// Stores in instruction order.  On the hardware the lanes of a wave execute one instruction
// together, so of two stores to one address the one later in the program wins, whichever lanes
// issue them; the encoder's back end relies on that (a lane also writes bytes for planes its
// block does not have, and a later instruction of another lane overwrites them).  Lanes that run one
// after the other have no such order, so these stores are logged with their position in the program
// (`seq`: the count of calls of the storing function so far, which is the same in all lanes, and
// the store's index inside it) and carried out in that order at the wave's next meeting point.
inline void emu_ordered_enter() { emu_cur->call_seq += 64; }
inline void emu_ordered_store8(uint8_t *addr, uint8_t value, uint32_t index)
{
    emu_wave_of_thread->log.push_back(emu_store{addr, emu_cur->call_seq + index, value});
}
inline void emu_ordered_store(void *addr, const void *value, uint32_t bytes, uint32_t index)
{
    for (uint32_t i = 0; i < bytes; ++i) emu_ordered_store8((uint8_t *)addr + i, ((const uint8_t *)value)[i], index);
}
inline void emu_ordered_store32(void *addr, uint32_t value, uint32_t index) { emu_ordered_store(addr, &value, 4, index); }

// saves the callee-saved registers and the stack pointer of the running lane, takes up another's
extern "C" void emu_switch(void **save_sp, void *load_sp);
// The same with the notices an AddressSanitizer build of the model needs about stacks that change
// under it (`bottom`, `bytes`: the stack that is switched to; `leaving`: the running lane never comes back).
#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define EMU_ASAN 1
extern "C" void __sanitizer_start_switch_fiber(void **fake_stack_save, const void *bottom, size_t size);
extern "C" void __sanitizer_finish_switch_fiber(void *fake_stack_save, const void **bottom_old, size_t *size_old);
#endif
#endif
inline void emu_switch_stacks(void **save_sp, void *load_sp, const void *bottom, size_t bytes, bool leaving = false)
{
#ifdef EMU_ASAN
    void *fake = nullptr;
    __sanitizer_start_switch_fiber(leaving ? nullptr : &fake, bottom, bytes);
    emu_switch(save_sp, load_sp);
    __sanitizer_finish_switch_fiber(fake, nullptr, nullptr);
#else
    (void)bottom, (void)bytes, (void)leaving;
    emu_switch(save_sp, load_sp);
#endif
}
// gives way to the next lane of the wave that has not left the kernel
inline void emu_next_lane(emu_wave *w)
{
    emu_lane_ctx *me = emu_cur;
    unsigned i = (unsigned)me->lane;
    for (unsigned k = 0; k < w->count; ++k) {
        i = i + 1 == w->count ? 0 : i + 1;
        if (!w->lanes[i].done) break;
    }
    emu_lane_ctx *next = &w->lanes[i];
    if (next == me) {
        fprintf(stderr, "EMU: lane %d of block %u waits for lanes that have all left the kernel\n", me->lane, blockIdx.x);
        abort();
    }
    emu_cur = next;
    emu_switch_stacks(&me->sp, next->sp, w->stacks + (size_t)next->lane * w->stack_bytes, w->stack_bytes, me->done);
}
// the last lane to arrive lets the meeting go: the logged stores are carried out in program order first
inline void emu_release(emu_wave *w)
{
    if (!w->log.empty()) {
        std::stable_sort(w->log.begin(), w->log.end(), [](const emu_store &a, const emu_store &b) { return a.seq < b.seq; });
        for (const emu_store &st : w->log) *st.addr = st.value;
        w->log.clear();
    }
    w->arrived = 0;
    w->gen++;
}
// (for a meeting with values: who is there, noted by the lane that arrives last)
inline void emu_note_present(emu_wave *w, unsigned p)
{
    uint64_t m = 0;
    for (unsigned l = 0; l < w->count; ++l)
        if (!w->lanes[l].done) m |= 1ull << l;
    w->present[p] = m;
}
// All lanes of the wave that have not left the kernel meet; true in the one that arrived last.
inline bool emu_meet(unsigned site, int parity = -1)
{
    emu_wave *w = emu_wave_of_thread;
    if (w->arrived == 0) {
        w->site = site;
    } else if (w->site != site) {
        fprintf(stderr, "EMU: the lanes of a wave are at different places of the program (lines %u and %u, lane %d, block %u): "
                        "a cross-lane operation under a branch that is not uniform\n", w->site, site, emu_cur->lane, blockIdx.x);
        abort();
    }
    const unsigned my = w->gen;
    if (++w->arrived == w->live) {
        if (parity >= 0) emu_note_present(w, (unsigned)parity);
        emu_release(w);
        return true;
    }
    while (w->gen == my) emu_next_lane(w);
    return false;
}
// all lanes meet; each leaves a value and reads another lane's (src < 0: none, gives 0)
inline uint64_t emu_exchange(unsigned site, uint64_t mine, int src)
{
    emu_wave *w = emu_wave_of_thread;
    const unsigned p = emu_cur->parity++ & 1u;
    w->slot[p][emu_lane] = mine;
    emu_meet(site, (int)p);
    return src >= 0 ? w->slot[p][src] : 0;
}
// the same, every lane seeing all values (valid until the lane's next meeting but one); `present`: who took part
inline const uint64_t *emu_gather(unsigned site, uint64_t mine, uint64_t *present)
{
    emu_wave *w = emu_wave_of_thread;
    const unsigned p = emu_cur->parity++ & 1u;
    w->slot[p][emu_lane] = mine;
    emu_meet(site, (int)p);
    *present = w->present[p];
    return w->slot[p];
}

// the workgroup's barrier: the lanes of each wave meet, the last one to arrive waits for the other waves
inline void emu_syncthreads(unsigned site)
{
    if (emu_meet(site)) pthread_barrier_wait(&emu_block_barrier);
}
#define __syncthreads() emu_syncthreads(__LINE__)

// ---------------------------------------------------------------- cross-lane builtins
// v_mov_b32 with a DPP control (the controls the kernels use): the lane the value comes from,
// or -1 when the control names no lane for this one.
inline int emu_dpp_source(int lane, int ctrl)
{
    const int row = lane & ~15, in_row = lane & 15;
    if (ctrl >= 0x000 && ctrl <= 0x0ff) return (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);   // quad_perm
    if (ctrl >= 0x101 && ctrl <= 0x10f) return in_row + (ctrl & 15) <= 15 ? lane + (ctrl & 15) : -1;   // row_shl
    if (ctrl >= 0x111 && ctrl <= 0x11f) return in_row >= (ctrl & 15) ? lane - (ctrl & 15) : -1;        // row_shr
    if (ctrl == 0x140) return row | (15 - in_row);                                                    // row_mirror
    if (ctrl == 0x141) return (lane & ~7) | (7 - (lane & 7));                                         // row_half_mirror
    if (ctrl == 0x142) return lane >= 16 ? (row - 16) | 15 : -1;                                      // row_bcast:15
    if (ctrl == 0x143) return lane >= 32 ? 31 : -1;                                                   // row_bcast:31
    fprintf(stderr, "EMU: DPP control 0x%x is not modelled\n", ctrl);
    abort();
}
inline int emu_update_dpp(unsigned site, int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl)
{
    const int lane = emu_lane;
    const int from = emu_dpp_source(lane, ctrl);
    const uint64_t got = emu_exchange(site, (uint32_t)src, from);
    const bool enabled = ((row_mask >> (lane >> 4)) & 1) && ((bank_mask >> ((lane >> 2) & 3)) & 1);
    if (!enabled) return old;
    // row_bcast writes only the lanes it has a source for; the others keep `old`
    if (from < 0) return (bound_ctrl && ctrl != 0x142 && ctrl != 0x143) ? 0 : old;
    return (int)(uint32_t)got;
}
// (the first lane that is still in the kernel, as the hardware takes the first active one)
inline int emu_readfirstlane(unsigned site, int v)
{
    const emu_wave *w = emu_wave_of_thread;
    int first = 0;
    while (first < 63 && w->lanes[first].done) ++first;
    return (int)(uint32_t)emu_exchange(site, (uint32_t)v, first);
}
inline int emu_readlane(unsigned site, int v, int lane) { return (int)(uint32_t)emu_exchange(site, (uint32_t)v, lane & 63); }
inline uint64_t emu_ballot(unsigned site, bool pred)
{
    uint64_t present = 0;
    const uint64_t *all = emu_gather(site, pred ? 1u : 0u, &present);
    uint64_t m = 0;
    for (unsigned l = 0; l < 64; ++l)
        if ((present >> l) & 1u) m |= (all[l] & 1u) << l;
    return m;
}
template <typename T>
inline T emu_shfl_xor(unsigned site, T v, int mask, int /*width*/)
{
    static_assert(sizeof(T) <= 8, "values of up to 64 bits");
    uint64_t bits = 0;
    memcpy(&bits, &v, sizeof(T));
    const uint64_t got = emu_exchange(site, bits, (emu_lane ^ mask) & 63);
    T out;
    memcpy(&out, &got, sizeof(T));
    return out;
}
#define __shfl_xor(v, mask, width) emu_shfl_xor(__LINE__, v, mask, width)
inline void emu_wave_barrier(unsigned site) { (void)emu_meet(site); }

// ---------------------------------------------------------------- lane-local builtins
inline uint32_t emu_perm(uint32_t s0, uint32_t s1, uint32_t sel)
{
    // v_perm_b32: selector bytes 0-3 pick bytes of the second operand, 4-7 of the first, 0x0c gives 0x00, 0x0d and up 0xff
    const uint64_t both = ((uint64_t)s0 << 32) | s1;
    uint32_t out = 0;
    for (int i = 0; i < 4; ++i) {
        const uint32_t c = (sel >> (8 * i)) & 0xffu;
        uint32_t b;
        if (c <= 7) b = (uint32_t)(both >> (8 * c)) & 0xffu;
        else if (c == 0x0c) b = 0;
        else if (c >= 0x0d) b = 0xff;
        else {   // 8..11: the sign of a byte, replicated
            const uint32_t byte = (uint32_t)(both >> (8 * (2 * (c - 8) + 1))) & 0xffu;
            b = (byte & 0x80u) ? 0xffu : 0u;
        }
        out |= b << (8 * i);
    }
    return out;
}
inline uint32_t emu_alignbit(uint32_t hi, uint32_t lo, uint32_t sh) { return (uint32_t)((((uint64_t)hi << 32) | lo) >> (sh & 31u)); }
inline uint32_t emu_alignbyte(uint32_t hi, uint32_t lo, uint32_t sh) { return (uint32_t)((((uint64_t)hi << 32) | lo) >> (8u * (sh & 3u))); }
inline uint32_t emu_ubfe(uint32_t v, uint32_t off, uint32_t width)
{
    off &= 31u;
    width &= 31u;
    return width ? (v >> off) & ((1u << width) - 1u) : 0u;
}
inline int32_t emu_sbfe(int32_t v, uint32_t off, uint32_t width)
{
    off &= 31u;
    width &= 31u;
    if (!width) return 0;
    const uint32_t field = ((uint32_t)v >> off) & ((1u << width) - 1u);
    return (field >> (width - 1)) & 1u ? (int32_t)(field | ~((1u << width) - 1u)) : (int32_t)field;
}
inline uint32_t emu_sad_u8(uint32_t a, uint32_t b, uint32_t acc)
{
    for (int i = 0; i < 4; ++i) {
        const int x = (a >> (8 * i)) & 0xff, y = (b >> (8 * i)) & 0xff;
        acc += (uint32_t)(x > y ? x - y : y - x);
    }
    return acc;
}
// v_cvt_i32_f32: toward zero, saturating, NaN gives 0
inline int32_t emu_cvt_i32_f32(float t)
{
    if (std::isnan(t)) return 0;
    if (t >= 2147483648.0f) return INT32_MAX;
    if (t <= -2147483648.0f) return INT32_MIN;
    return (int32_t)t;
}
inline int __clz(int v) { return v ? __builtin_clz((unsigned)v) : 32; }
inline float __fmul_rn(float a, float b) { volatile float r = a * b; return r; }
inline float __fadd_rn(float a, float b) { volatile float r = a + b; return r; }

// ---------------------------------------------------------------- buffer descriptors
struct emu_rsrc {
    uint8_t *base;
    uint32_t bytes;
};
typedef unsigned int emu_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int emu_u32x2 __attribute__((ext_vector_type(2)));
inline emu_rsrc emu_make_rsrc(void *base, short /*stride*/, int bytes, int /*flags*/) { return emu_rsrc{(uint8_t *)base, (uint32_t)bytes}; }
// dword d of an access at `off` is in range when it ends within the descriptor's byte count.
// An aligned pair of dwords is moved as one 64-bit access, a dword as one 32-bit access: the
// hardware does not tear them, and the status words other workgroups poll rely on that.
template <int DWORDS>
inline void emu_buf_load(const emu_rsrc &rs, uint32_t voff, uint32_t soff, uint32_t *out)
{
    const uint64_t off = (uint64_t)voff + soff;
    for (int d = 0; d < DWORDS; ++d) {
        out[d] = 0;
        const uint8_t *at = rs.base + off + 4u * d;
        if (d + 1 < DWORDS && ((uintptr_t)at & 7u) == 0 && off + 4u * d + 8u <= rs.bytes) {
            emu_check(at, 8, "buffer load");
            const uint64_t v = __atomic_load_n((const uint64_t *)at, __ATOMIC_SEQ_CST);
            out[d] = (uint32_t)v;
            out[++d] = (uint32_t)(v >> 32);
        } else if (off + 4u * d + 4u <= rs.bytes) {
            emu_check(at, 4, "buffer load");
            if (((uintptr_t)at & 3u) == 0)
                out[d] = __atomic_load_n((const uint32_t *)at, __ATOMIC_SEQ_CST);
            else
                memcpy(&out[d], at, 4);
        }
        // (a dword that straddles the end is out of range as a whole, like one beyond it: the check is per dword)
    }
}
template <int DWORDS>
inline void emu_buf_store(const emu_rsrc &rs, uint32_t voff, uint32_t soff, const uint32_t *in)
{
    const uint64_t off = (uint64_t)voff + soff;
    for (int d = 0; d < DWORDS; ++d) {
        uint8_t *at = rs.base + off + 4u * d;
        if (d + 1 < DWORDS && ((uintptr_t)at & 7u) == 0 && off + 4u * d + 8u <= rs.bytes) {
            emu_check(at, 8, "buffer store");
            __atomic_store_n((uint64_t *)at, (uint64_t)in[d] | ((uint64_t)in[d + 1] << 32), __ATOMIC_SEQ_CST);
            ++d;
        } else if (off + 4u * d + 4u <= rs.bytes) {
            emu_check(at, 4, "buffer store");
            if (((uintptr_t)at & 3u) == 0)
                __atomic_store_n((uint32_t *)at, in[d], __ATOMIC_SEQ_CST);
            else
                memcpy(at, &in[d], 4);
        }
    }
}
inline emu_u32x4 emu_load_b128(emu_rsrc rs, int voff, int soff, int)
{
    uint32_t w[4];
    emu_buf_load<4>(rs, (uint32_t)voff, (uint32_t)soff, w);
    return emu_u32x4{w[0], w[1], w[2], w[3]};
}
inline emu_u32x2 emu_load_b64(emu_rsrc rs, int voff, int soff, int)
{
    uint32_t w[2];
    emu_buf_load<2>(rs, (uint32_t)voff, (uint32_t)soff, w);
    return emu_u32x2{w[0], w[1]};
}
inline uint32_t emu_load_b32(emu_rsrc rs, int voff, int soff, int)
{
    uint32_t w;
    emu_buf_load<1>(rs, (uint32_t)voff, (uint32_t)soff, &w);
    return w;
}
inline uint16_t emu_load_b16(emu_rsrc rs, int voff, int soff, int)
{
    const uint64_t off = (uint64_t)(uint32_t)voff + (uint32_t)soff;
    uint16_t v = 0;
    if (off + 2u <= rs.bytes) {
        emu_check(rs.base + off, 2, "buffer load");
        memcpy(&v, rs.base + off, 2);
    }
    return v;
}
inline void emu_store_b128(emu_u32x4 v, emu_rsrc rs, int voff, int soff, int)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    emu_buf_store<4>(rs, (uint32_t)voff, (uint32_t)soff, w);
}
inline void emu_store_b64(emu_u32x2 v, emu_rsrc rs, int voff, int soff, int)
{
    const uint32_t w[2] = {v.x, v.y};
    emu_buf_store<2>(rs, (uint32_t)voff, (uint32_t)soff, w);
}
inline void emu_store_b8(uint8_t v, emu_rsrc rs, int voff, int soff, int)
{
    const uint64_t off = (uint64_t)(uint32_t)voff + (uint32_t)soff;
    if (off + 1u <= rs.bytes) {
        emu_check(rs.base + off, 1, "buffer store");
        rs.base[off] = v;
    }
}

#define __amdgpu_buffer_rsrc_t emu_rsrc
#define __builtin_amdgcn_make_buffer_rsrc emu_make_rsrc
#define __builtin_amdgcn_raw_buffer_load_b128 emu_load_b128
#define __builtin_amdgcn_raw_buffer_load_b64 emu_load_b64
#define __builtin_amdgcn_raw_buffer_load_b32 emu_load_b32
#define __builtin_amdgcn_raw_buffer_load_b16 emu_load_b16
#define __builtin_amdgcn_raw_buffer_store_b128 emu_store_b128
#define __builtin_amdgcn_raw_buffer_store_b64 emu_store_b64
#define __builtin_amdgcn_raw_buffer_store_b8 emu_store_b8
#define __builtin_amdgcn_update_dpp(...) emu_update_dpp(__LINE__, __VA_ARGS__)
#define __builtin_amdgcn_readfirstlane(...) emu_readfirstlane(__LINE__, __VA_ARGS__)
#define __builtin_amdgcn_readlane(...) emu_readlane(__LINE__, __VA_ARGS__)
#define __builtin_amdgcn_ballot_w64(...) emu_ballot(__LINE__, __VA_ARGS__)
#define __builtin_amdgcn_perm emu_perm
#define __builtin_amdgcn_alignbit emu_alignbit
#define __builtin_amdgcn_alignbyte emu_alignbyte
#define __builtin_amdgcn_ubfe emu_ubfe
#define __builtin_amdgcn_sbfe emu_sbfe
#define __builtin_amdgcn_sad_u8 emu_sad_u8
// A lane that sleeps between two looks at a word another workgroup writes.  On the hardware the
// other lanes of its wave go on meanwhile; here they run on the same thread, so the lane gives
// way to them first (what it waits for may depend on a store one of them has not made yet), then
// the thread sleeps: the bounds on such waits count looks and are sized for a device on which
// every workgroup runs at once, while here a workgroup may have to wait for a processor.
inline void emu_sleep()
{
    emu_wave *w = emu_wave_of_thread;
    if (w && w->live > 1) emu_next_lane(w);
    const timespec t{0, 100000};
    nanosleep(&t, nullptr);
}
#define __builtin_amdgcn_s_sleep(n) emu_sleep()
#define __builtin_amdgcn_s_setprio(n) ((void)0)
#define __builtin_amdgcn_fence(order, scope) __atomic_thread_fence(__ATOMIC_SEQ_CST)
#define __builtin_amdgcn_wave_barrier() emu_wave_barrier(__LINE__)

// device-scope atomics: host atomics on the shared mapping
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __hip_atomic_load(p, order, scope) __atomic_load_n((p), __ATOMIC_SEQ_CST)
#define __hip_atomic_store(p, v, order, scope) __atomic_store_n((p), (v), __ATOMIC_SEQ_CST)
inline unsigned atomicOr(uint32_t *p, uint32_t v) { return __atomic_fetch_or(p, v, __ATOMIC_SEQ_CST); }

// ---------------------------------------------------------------- vector types of the HIP headers
struct float4 {
    float x, y, z, w;
};
struct int4 {
    int x, y, z, w;
};
inline int4 make_int4(int x, int y, int z, int w) { return int4{x, y, z, w}; }
