// TEST INFRASTRUCTURE: the CPU execution model checked against itself -- small kernels whose
// outcome is known from the instruction set's definitions, and kernels that do what the model is
// there to catch (each of those must end the run the way the model promises).
//
//   model_selftest semantics      DPP controls, readlane / readfirstlane, ballot, byte permute, field
//                                 extracts, alignbit / alignbyte, sad_u8, the saturating conversion,
//                                 buffer loads and stores at the end of a descriptor, lanes that leave early
//   model_selftest divergent      a cross-lane operation under a branch that is not uniform: reported
//   model_selftest beyond_buffer  a descriptor over memory no allocation holds: reported
//   model_selftest beyond_lds     a store behind the dynamic LDS the launch asked for: reported
//   model_selftest beyond_slot    a store behind one of the slots a kernel cuts its dynamic LDS into: reported
//   model_selftest guard_page     a plain store one byte behind an allocation: a fault of the workgroup
//   model_selftest host_threads FILE   launches from one host thread while another writes FILE through
//                                 stdio: the workgroups' processes add nothing to it, a kernel's printf arrives once
#define EMU_DYN_LDS 4096
#define EMU_DEFINE_GLOBALS
#include "hip/hip_runtime.h"

#include <atomic>
#include <string>
#include <thread>

namespace {

struct Out {
    uint32_t v[64][16];
    uint64_t ballot[4];
    uint32_t scalar[16];
};

constexpr int kShr1 = 0x111, kShr8 = 0x118, kShl2 = 0x102, kQuadBcast2 = 0xAA, kQuadXor1 = 0xB1, kMirror = 0x140, kHalfMirror = 0x141;

__global__ void k_semantics(Out *out, uint8_t *buf)
{
    const int lane = threadIdx.x;
    const uint32_t x = 1000u + (uint32_t)lane;
    uint32_t *o = out->v[lane];
    o[0] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kShr1, 0xF, 0xF, true);
    o[1] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kShr8, 0xF, 0xF, true);
    o[2] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kShl2, 0xF, 0xF, true);
    o[3] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kQuadBcast2, 0xF, 0xF, true);
    o[4] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kQuadXor1, 0xF, 0xF, true);
    o[5] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kMirror, 0xF, 0xF, true);
    o[6] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kHalfMirror, 0xF, 0xF, true);
    o[7] = (uint32_t)__builtin_amdgcn_update_dpp(7, (int)x, 0x142, 0xA, 0xF, false);   // row_bcast:15 into rows 1 and 3
    o[8] = (uint32_t)__builtin_amdgcn_update_dpp(7, (int)x, 0x143, 0xC, 0xF, false);   // row_bcast:31 into rows 2 and 3
    o[9] = (uint32_t)__builtin_amdgcn_update_dpp(7, (int)x, kShr1, 0x5, 0x3, true);    // rows 0 and 2, banks 0 and 1 only
    o[10] = (uint32_t)__builtin_amdgcn_readlane((int)x, 37);
    o[11] = (uint32_t)__builtin_amdgcn_readfirstlane((int)x);
    const uint64_t b = __builtin_amdgcn_ballot_w64((lane % 3) == 0);
    if (lane == 0) out->ballot[0] = b;
    // buffer accesses at the end of a descriptor of 10 bytes
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(buf, 0, 10, 0x00020000);
    if (lane == 0) {
        out->scalar[0] = __builtin_amdgcn_raw_buffer_load_b32(rs, 4, 0, 0);
        out->scalar[2] = __builtin_amdgcn_raw_buffer_load_b32(rs, 12, 0, 0);
        out->scalar[3] = __builtin_amdgcn_raw_buffer_load_b32(rs, 0, 4, 0);    // the scalar offset counts
        __builtin_amdgcn_raw_buffer_store_b8((uint8_t)0xEE, rs, 9, 0, 0);       // inside
        __builtin_amdgcn_raw_buffer_store_b8((uint8_t)0xEE, rs, 10, 0, 0);      // dropped
        __builtin_amdgcn_raw_buffer_store_b64(emu_u32x2{0x11223344u, 0x55667788u}, rs, 4, 0, 0);   // the second dword does not fit: dropped
        out->scalar[4] = __builtin_amdgcn_perm(0xA3A2A1A0u, 0xB3B2B1B0u, 0x0c070400u);
        out->scalar[5] = __builtin_amdgcn_perm(0x80000000u, 0x00008000u, 0x0d0b0908u);
        out->scalar[6] = __builtin_amdgcn_alignbit(0x12345678u, 0x9abcdef0u, 8);
        out->scalar[7] = __builtin_amdgcn_alignbyte(0x12345678u, 0x9abcdef0u, 3);
        out->scalar[8] = __builtin_amdgcn_ubfe(0xdeadbeefu, 8, 12);
        out->scalar[9] = (uint32_t)__builtin_amdgcn_sbfe((int)0x00000f00u, 8, 4);
        out->scalar[10] = __builtin_amdgcn_sad_u8(0x01ff1000u, 0x02000f10u, 5u);
        out->scalar[11] = (uint32_t)emu_cvt_i32_f32(3e9f);
        out->scalar[12] = (uint32_t)emu_cvt_i32_f32(-2.75f);
        out->scalar[13] = (uint32_t)emu_cvt_i32_f32(__builtin_nanf(""));
    }
    // lanes that leave the kernel no longer take part: the upper half is gone for what follows
    if (lane >= 32) return;
    const uint64_t b2 = __builtin_amdgcn_ballot_w64(true);
    o[12] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kShr1, 0xF, 0xF, true);
    if (lane == 0) out->ballot[1] = b2;
}

__global__ void k_divergent(Out *out)
{
    const int lane = threadIdx.x;
    uint32_t x = (uint32_t)lane;
    if (lane & 1) x = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kShr1, 0xF, 0xF, true);
    out->v[lane][0] = (uint32_t)__builtin_amdgcn_readlane((int)x, 0);
}

__global__ void k_beyond_buffer(uint8_t *stray)
{
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(stray, 0, 64, 0x00020000);
    (void)__builtin_amdgcn_raw_buffer_load_b32(rs, (int)threadIdx.x * 4 % 64, 0, 0);
}

__global__ void k_beyond_lds(int)
{
    static __attribute__((aligned(16), section("emu_lds"))) uint8_t s_dyn[EMU_DYN_LDS];
    emu_note_dynamic_lds(s_dyn);
    s_dyn[threadIdx.x] = 1;          // within the 64 bytes the launch asked for
    if (threadIdx.x == 5) s_dyn[64] = 1;
}

__global__ void k_beyond_slot(int)
{
    static __attribute__((aligned(16), section("emu_lds"))) uint8_t s_dyn[EMU_DYN_LDS + 16 * EMU_SLOT_GUARD];
    emu_note_dynamic_lds(s_dyn, 16 * EMU_SLOT_GUARD);
    // two slots of 64 bytes for the one wave; the first is filled to its last byte, the second one byte further
    uint8_t *first = emu_stage_slot(s_dyn, 0, 0, 2, 64), *second = emu_stage_slot(s_dyn, 0, 1, 2, 64);
    first[threadIdx.x] = 1;
    second[threadIdx.x] = 1;
    if (threadIdx.x == 9) second[64] = 1;
}

__global__ void k_guard_page(uint8_t *buf, size_t bytes)
{
    if (threadIdx.x == 0) buf[bytes] = 1;
}

__global__ void k_says_hello(uint32_t *count)
{
    if (threadIdx.x == 0) {
        count[blockIdx.x] += 1;
        if (blockIdx.x == 0 && count[0] == 1) printf("a kernel's line\n");
    }
}

int fail(const char *what)
{
    fprintf(stderr, "model_selftest: %s\n", what);
    return 1;
}

int semantics()
{
    Out *out = (Out *)emu_device_alloc_named(sizeof(Out), "out");
    uint8_t *buf = (uint8_t *)emu_device_alloc_named(16, "buf", 1);
    memset(out, 0, sizeof(Out));
    for (int i = 0; i < 16; ++i) buf[i] = (uint8_t)(0x10 + i);
    hipLaunchKernelGGL(k_semantics, dim3(1), dim3(64), 0, 0, out, buf);
    if (hipGetLastError() != hipSuccess) return fail("the launch");
    for (int l = 0; l < 64; ++l) {
        const uint32_t *o = out->v[l];
        const uint32_t x = 1000u + (uint32_t)l;
        const int in_row = l & 15;
        if (o[0] != (in_row >= 1 ? x - 1 : 0u)) return fail("row_shr:1");
        if (o[1] != (in_row >= 8 ? x - 8 : 0u)) return fail("row_shr:8");
        if (o[2] != (in_row <= 13 ? x + 2 : 0u)) return fail("row_shl:2");
        if (o[3] != 1000u + (uint32_t)((l & ~3) | 2)) return fail("quad_perm [2,2,2,2]");
        if (o[4] != 1000u + (uint32_t)(l ^ 1)) return fail("quad_perm [1,0,3,2]");
        if (o[5] != 1000u + (uint32_t)((l & ~15) | (15 - in_row))) return fail("row_mirror");
        if (o[6] != 1000u + (uint32_t)((l & ~7) | (7 - (l & 7)))) return fail("row_half_mirror");
        const int row = l >> 4;
        if (o[7] != ((row == 1 || row == 3) ? 1000u + (uint32_t)(16 * row - 1) : 7u)) return fail("row_bcast:15");
        if (o[8] != (row >= 2 ? 1031u : 7u)) return fail("row_bcast:31");
        const bool enabled = (row == 0 || row == 2) && ((l >> 2) & 3) < 2;
        if (o[9] != (enabled ? (in_row >= 1 ? x - 1 : 0u) : 7u)) return fail("row and bank masks");
        if (o[10] != 1037u) return fail("readlane");
        if (o[11] != 1000u) return fail("readfirstlane");
        if (l < 32 && o[12] != (in_row >= 1 ? x - 1 : 0u)) return fail("DPP after half the wave has left");
    }
    uint64_t want = 0;
    for (int l = 0; l < 64; ++l)
        if (l % 3 == 0) want |= 1ull << l;
    if (out->ballot[0] != want) return fail("ballot");
    if (out->ballot[1] != 0xffffffffull) return fail("ballot after half the wave has left");
    const uint32_t *s = out->scalar;
    if (s[0] != 0x17161514u) return fail("buffer load inside");
    if (s[2] != 0u) return fail("buffer load beyond the end");
    if (s[3] != 0x17161514u) return fail("scalar offset");
    if (buf[9] != 0xEE || buf[10] != 0x1A || buf[8] != 0x18 || buf[4] != 0x44 || buf[7] != 0x11) return fail("buffer stores at the end");
    if (s[4] != 0x00A3A0B0u) return fail("v_perm: bytes of both operands and 0x0c");
    if (s[5] != 0xffff00ffu) return fail("v_perm: sign bytes and 0x0d");
    if (s[6] != 0x789abcdeu) return fail("v_alignbit");
    if (s[7] != 0x3456789au) return fail("v_alignbyte");
    if (s[8] != 0xdbeu) return fail("v_bfe_u32");
    if (s[9] != 0xffffffffu) return fail("v_bfe_i32");
    if (s[10] != 5u + 1u + 255u + 1u + 16u) return fail("v_sad_u8");
    if (s[11] != 0x7fffffffu || s[12] != (uint32_t)-2 || s[13] != 0u) return fail("v_cvt_i32_f32");
    printf("semantics ok\n");
    return 0;
}

// A workgroup is a forked process: it starts with a copy of every stdio buffer of the program, as
// another host thread had filled it at that moment, and must not write any of that out.
int host_threads(const char *path)
{
    FILE *f = fopen(path, "wb");
    if (!f) return fail("the file");
    std::atomic<bool> stop{false};
    size_t records = 0;
    std::thread writer([&]() {
        char record[100];
        while (!stop.load()) {
            memset(record, 'a' + (int)(records % 26), sizeof(record));
            fwrite(record, 1, sizeof(record), f);     // stays in the stream's buffer most of the time
            ++records;
            usleep(20);
        }
    });
    uint32_t *count = (uint32_t *)emu_device_alloc_named(2 * sizeof(uint32_t), "count");
    count[0] = count[1] = 0;
    for (int i = 0; i < 150; ++i) hipLaunchKernelGGL(k_says_hello, dim3(2), dim3(64), 0, 0, count);
    stop.store(true);
    writer.join();
    fclose(f);
    if (hipGetLastError() != hipSuccess) return fail("a launch");
    if (count[0] != 150 || count[1] != 150) return fail("the launches' count");
    printf("records %zu\n", records);
    return 0;
}

}  // namespace

int main(int argc, char **argv)
{
    const std::string what = argc > 1 ? argv[1] : "";
    if (what == "semantics") return semantics();
    if (what == "host_threads" && argc > 2) return host_threads(argv[2]);
    Out *out = (Out *)emu_device_alloc_named(sizeof(Out), "out");
    if (what == "divergent") {
        hipLaunchKernelGGL(k_divergent, dim3(1), dim3(64), 0, 0, out);
    } else if (what == "beyond_buffer") {
        static uint8_t stray[64];
        hipLaunchKernelGGL(k_beyond_buffer, dim3(1), dim3(64), 0, 0, stray);
    } else if (what == "beyond_lds") {
        hipLaunchKernelGGL(k_beyond_lds, dim3(1), dim3(64), 64, 0, 0);
    } else if (what == "beyond_slot") {
        hipLaunchKernelGGL(k_beyond_slot, dim3(1), dim3(64), 128, 0, 0);
    } else if (what == "guard_page") {
        uint8_t *buf = (uint8_t *)emu_device_alloc_named(100, "buf", 1);
        hipLaunchKernelGGL(k_guard_page, dim3(1), dim3(64), 0, 0, buf, (size_t)100);
    } else {
        fprintf(stderr, "usage: %s semantics|divergent|beyond_buffer|beyond_lds|beyond_slot|guard_page|host_threads FILE\n", argv[0]);
        return 2;
    }
    // the kernels above must not get away with it
    const hipError_t e = hipGetLastError();
    printf("launch %s\n", e == hipSuccess ? "went through" : "failed");
    return e == hipSuccess ? 0 : 3;
}
