// Device-side building blocks of the HomComp codec for gfx950 (wave64).
//
// Work mapping (differs on purpose from the reference's one-thread-per-block, 32-thread layout,
// HomComp/include/GSZ.h:4-9): a 32-element block is owned by 4 adjacent lanes, 8 consecutive
// elements per lane.  One lane therefore produces exactly one byte of every bit plane (the
// stream stores plane p as 4 bytes, byte k covering elements 8k..8k+7 MSB first,
// HomComp/src/GSZ.cu:312-351), and an 8x8 bit-matrix transpose turns its eight magnitudes
// into eight plane bytes at once.  Cross-lane traffic is limited to quad-local DPP moves.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "homcomp_kernels.hpp"

#ifndef HC_POLL_SLEEP
#define HC_POLL_SLEEP 16
#endif
namespace hc {

constexpr int kWG = 256;                              // threads per workgroup (4 independent waves)
constexpr int kEPL = 8;                               // elements per lane per sub-step
constexpr int kTileBlocks = 128;                      // blocks per tile
constexpr int kTileElems = kTileBlocks * 32;          // 4096
constexpr int kChunkElems = 32768;                    // reference thread-block share
constexpr int kMaxBlockBytes = 132;                   // largest size a header byte can imply
constexpr int kOutBlockBytes = 128;                   // largest payload the encoder emits per block

// Native 16-byte vectors (the streaming load/store builtins take these, not HIP's float4).
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Every buffer is read or written exactly once per call, so loads and stores carry the
// non-temporal hint and do not displace the scan words from the caches.
template <typename V>
__device__ __forceinline__ V stream_load(const void *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
}
// Same from a device address computed as an integer: the global address space is stated, so
// the access is a global load, not a flat one (flat accesses count against both memory counters
// and keep the compiler from waiting for individual loads).
template <typename V>
__device__ __forceinline__ V stream_load_global(uintptr_t addr)
{
    return __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) V *>(addr));
}
template <typename V>
__device__ __forceinline__ void stream_store(void *p, V v)
{
    __builtin_nontemporal_store(v, reinterpret_cast<V *>(p));
}

// ---------------------------------------------------------------- cross-lane helpers

// Quad-local lane permutation through DPP; must run with all lanes of the wave active.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
constexpr int kDppXor1 = 0xB1;      // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;      // quad_perm [2,3,0,1]
constexpr int kDppBcast0 = 0x00;    // quad_perm [0,0,0,0]
constexpr int kDppBcast1 = 0x55;    // quad_perm [1,1,1,1]
constexpr int kDppBcast2 = 0xAA;    // quad_perm [2,2,2,2]
constexpr int kDppRowShr1 = 0x111;  // lane i reads lane i-1 inside its row of 16 (0 at row start)

__device__ __forceinline__ uint32_t quad_or(uint32_t v)
{
    v |= dpp_u32<kDppXor1>(v);
    v |= dpp_u32<kDppXor2>(v);
    return v;
}

constexpr int kDppRowHalfMirror = 0x141;  // lane i reads lane 7-i inside its group of 8
constexpr int kDppRowMirror = 0x140;      // lane i reads lane 15-i inside its row of 16

// Inclusive scan across the wave: Hillis-Steele with DPP row shifts inside each row of 16 lanes,
// then the row totals travel on with the two row-broadcast steps (lane 15 of a row into the next
// row, lane 31 into the upper half).  Must run with all lanes active.
__device__ __forceinline__ uint32_t wave_incl_scan_u32(uint32_t x, int /*lane*/)
{
    x += dpp_u32<0x111>(x);   // row_shr:1
    x += dpp_u32<0x112>(x);   // row_shr:2
    x += dpp_u32<0x114>(x);   // row_shr:4
    x += dpp_u32<0x118>(x);   // row_shr:8
    // row_bcast:15 into rows 1 and 3, row_bcast:31 into rows 2 and 3; other rows keep their value
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xA, 0xF, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xC, 0xF, false);
    return x;
}

// The same for a value that is equal in the four lanes of every quad: the inclusive sum over the
// quads up to the lane's own, with two row shifts less.
__device__ __forceinline__ uint32_t quad_incl_scan_u32(uint32_t x)
{
    x += dpp_u32<0x114>(x);   // row_shr:4
    x += dpp_u32<0x118>(x);   // row_shr:8
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xA, 0xF, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xC, 0xF, false);
    return x;
}

// ---------------------------------------------------------------- scalar arithmetic

// HomComp/src/GSZ.cu:6-25: fl(x*r), compare with -0.5, fl(.+0.5), convert toward zero
// (saturating, NaN -> 0, which v_cvt_i32_f32 does as PTX cvt.rzi.s32.f32 does), wrapping subtract.
__device__ __forceinline__ int32_t quantize(float x, float recip)
{
    float d = __fmul_rn(x, recip);
    uint32_t s = (d >= -0.5f) ? 0u : 1u;
    float t = __fadd_rn(d, 0.5f);
    int32_t r;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(t));
    return (int32_t)((uint32_t)r - s);
}

// HomComp/src/GSZ.cu:1437: currQuant * eb * 2, two float32 multiplications.
__device__ __forceinline__ float dequantize(int32_t q, float eb)
{
    return __fmul_rn(__fmul_rn((float)q, eb), 2.0f);
}

// HomComp/src/GSZ.cu:27-31
__device__ __forceinline__ uint32_t bit_num(uint32_t x) { return 32u - (uint32_t)__clz((int)x); }

// Plane count of a block maximum; the 5-bit header field caps it at 31.
__device__ __forceinline__ uint32_t planes_of(uint32_t m)
{
    uint32_t b = bit_num(m);
    return b > 31u ? 31u : b;
}

// HomComp/src/GSZ.cu:795-802: payload bytes implied by a header byte.  (The kernels use the
// byte-parallel forms below; this one is what they are checked against, at compile time.)
__device__ __forceinline__ constexpr uint32_t size_from_header(uint32_t h)
{
    uint32_t F = h & 0x1fu;
    uint32_t ob = ((h >> 5) & 3u) + 1u;
    return (h & 0x80u) ? 4u + 4u * F + ob : (F ? 4u + 4u * F : 0u);
}

// The same for four header bytes at once, added to acc: byte-parallel arithmetic (a size is at
// most 132, so nothing carries from byte to byte) and one sum-of-bytes instruction.
__device__ __forceinline__ uint32_t add_sizes_from_4_headers(uint32_t w, uint32_t acc)
{
    const uint32_t F = w & 0x1f1f1f1fu;
    const uint32_t sel = (w >> 7) & 0x01010101u;
    const uint32_t has_planes = ((F + 0x7f7f7f7fu) >> 7) & 0x01010101u;   // F != 0
    const uint32_t ob = (((w >> 5) & 0x03030303u) + 0x01010101u) & (sel * 0xffu);
    const uint32_t sizes = (F << 2) + ((has_planes | sel) << 2) + ob;
    return __builtin_amdgcn_sad_u8(sizes, 0u, acc);
}

// Transpose of an 8x8 bit matrix held row-per-byte in (lo, hi): result bit (8r+c) = input bit
// (8c+r).  Three rounds of delta swaps; the first two stay inside the 32-bit halves, only the last
// one moves nibbles between them, so everything is full-rate 32-bit arithmetic.
__device__ __forceinline__ void transpose8(uint32_t &lo, uint32_t &hi)
{
    uint32_t t;
    t = (lo ^ (lo >> 7)) & 0x00AA00AAu;
    lo ^= t ^ (t << 7);
    t = (hi ^ (hi >> 7)) & 0x00AA00AAu;
    hi ^= t ^ (t << 7);
    t = (lo ^ (lo >> 14)) & 0x0000CCCCu;
    lo ^= t ^ (t << 14);
    t = (hi ^ (hi >> 14)) & 0x0000CCCCu;
    hi ^= t ^ (t << 14);
    // x >> 28 of the 64-bit value, low word only (the mask 0x00000000F0F0F0F0 has no high bits)
    t = (lo ^ __builtin_amdgcn_alignbit(hi, lo, 28)) & 0xF0F0F0F0u;
    lo ^= t ^ (t << 28);
    hi ^= t >> 4;
}

// The same for blocks of at most four planes, in one register: eight 4-bit values as
// [4 bytes][2 nibbles][4 bits], byte r = value 7-r in the low and value 3-r in the high nibble.
// Swapping the byte index with the bit index inside the nibble (two delta swaps) leaves plane p in
// byte p with the bit of value m at position 7-m; the same two swaps lead back.
__device__ __forceinline__ uint32_t transpose4(uint32_t y)
{
    uint32_t t;
    t = (y ^ (y >> 7)) & 0x00AA00AAu;
    y ^= t ^ (t << 7);
    t = (y ^ (y >> 14)) & 0x0000CCCCu;
    y ^= t ^ (t << 14);
    return y;
}

// ---------------------------------------------------------------- per-lane block pieces

// Encoder front end for one lane's 8 signed deltas (HomComp/src/GSZ.cu:86-164): sign byte,
// magnitudes, block-wide bit widths through the quad, rate selection.  `k` is the lane's
// position in its quad.  hdr, size and a0 (|delta| of the block's element 0) come out identical
// in the four lanes of a quad.
// plain_only: the plain codec (HomComp/src/GSZ.cu:1578-1581), which knows no outlier mode.
__device__ __forceinline__ void analyse8(const int32_t v[8], int k, uint32_t a[8], uint32_t &sb,
                                         uint32_t &hdr, uint32_t &size, uint32_t &a0, bool plain_only = false)
{
    sb = 0;
    uint32_t rest = 0;
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        const uint32_t u = (uint32_t)v[m];
        const int32_t neg = (int32_t)(0u - u);
        a[m] = (uint32_t)(v[m] > neg ? v[m] : neg);        // |v| (0x80000000 stays, as in the reference)
        sb = __builtin_amdgcn_alignbit(sb, u, 31);        // shift in the sign bit: element 0 ends at bit 7
        if (m) rest |= a[m];
    }
    // bit width of a maximum equals the bit width of the OR
    uint32_t or1 = quad_or(rest | a[0]);                  // all 32 elements   (:152)
    uint32_t or2 = quad_or(rest | (k ? a[0] : 0u));       // elements 1..31    (:153)
    a0 = dpp_u32<kDppBcast0>(a[0]);                       // element 0         (:154)
    uint32_t fr1 = planes_of(or1);
    uint32_t fr2 = planes_of(or2);
    uint32_t ob = (bit_num(a0) + 7u) >> 3;
    uint32_t sz1 = fr1 ? 4u + 4u * fr1 : 0u;              // :156
    uint32_t sz2 = 4u + 4u * fr2 + ob;                    // :157
    if (plain_only || sz1 <= sz2) {                       // :158-160
        hdr = fr1;
        size = sz1;
    } else {                                              // :161-164
        hdr = fr2 | 0x80u | ((ob - 1u) << 5);
        size = sz2;
    }
}

// Encoder back end for one lane (HomComp/src/GSZ.cu:245-751): writes this lane's share of the
// block payload into the stage at `pos0` (the block's tile-relative offset).  Lane k contributes
// byte k of the sign word and of every plane, and byte k of the outlier.
//
// The code is kept free of per-plane branches: planes are written in whole groups of eight, so a
// lane also stores bytes for planes its block does not have.  Those land in the space of the
// blocks that follow (at most 35 bytes past the block's end) and are harmless because of the
// store order: planes from the highest to the lowest, then the sign bytes, then the outlier bytes.
// If a stray byte of block B and a valid plane byte of a later block X fall on one address, X's
// plane index is lower (X starts at least 4 bytes after B's first plane), so X's store is issued
// later and wins; sign and outlier bytes are issued after all plane stores.  Blocks without
// payload must not store at all (they share their position with the next block).  The stages
// keep 64 bytes of slack behind the last block.
//
// `stage` may carry an explicit address space (lds_bytes / global_bytes below) so that two calls
// with different destinations cannot be merged into one sequence of flat stores.
typedef __attribute__((address_space(3))) uint8_t *lds_bytes;
typedef __attribute__((address_space(1))) uint8_t *global_bytes;

template <int G, typename Bytes>
__device__ __forceinline__ void pack_group(Bytes stage, uint32_t base, const uint32_t a[8])
{
    // byte r of (lo, hi) = bits 8G..8G+7 of a[7-r]; after the transpose byte r is plane 8G+r
    constexpr uint32_t two = 0x0c0c0400u + 0x0101u * (uint32_t)G;   // byte G of the second, then of the first operand
    uint32_t lo = __builtin_amdgcn_perm(__builtin_amdgcn_perm(a[4], a[5], two),
                                        __builtin_amdgcn_perm(a[6], a[7], two), 0x05040100u);
    uint32_t hi = __builtin_amdgcn_perm(__builtin_amdgcn_perm(a[0], a[1], two),
                                        __builtin_amdgcn_perm(a[2], a[3], two), 0x05040100u);
    transpose8(lo, hi);
#pragma unroll
    for (int r = 7; r >= 0; --r)
        stage[base + 4u * (uint32_t)(8 * G + r)] = (uint8_t)((r < 4 ? lo : hi) >> (8 * (r & 3)));
}

// Planes 0-3 of a block whose values are all below 16.
template <typename Bytes>
__device__ __forceinline__ void pack_low4(Bytes stage, uint32_t base, const uint32_t a[8])
{
    constexpr uint32_t two = 0x0c0c0400u;
    const uint32_t lo = __builtin_amdgcn_perm(__builtin_amdgcn_perm(a[4], a[5], two),
                                              __builtin_amdgcn_perm(a[6], a[7], two), 0x05040100u);
    const uint32_t hi = __builtin_amdgcn_perm(__builtin_amdgcn_perm(a[0], a[1], two),
                                              __builtin_amdgcn_perm(a[2], a[3], two), 0x05040100u);
    const uint32_t y = transpose4(lo | (hi << 4));
#pragma unroll
    for (int r = 3; r >= 0; --r) stage[base + 4u * (uint32_t)r] = (uint8_t)(y >> (8 * r));
}

template <typename Bytes>
__device__ __forceinline__ void pack8(Bytes stage, uint32_t pos0, uint32_t hdr, int k,
                                      const uint32_t a_in[8], uint32_t sb, uint32_t a0)
{
    // no block of the wave has more than four planes (the usual case at moderate error bounds):
    // half the stores and a third of the transposition
    const bool low = __builtin_amdgcn_ballot_w64((hdr & 0x1fu) > 4u) == 0;
    if (hdr == 0) return;                                 // zero block (:287)
    const uint32_t sel = hdr >> 7;
    const uint32_t F = hdr & 0x1fu;
    const uint32_t ob = sel ? ((hdr >> 5) & 3u) + 1u : 0u;
    uint32_t a[8];
#pragma unroll
    for (int m = 1; m < 8; ++m) a[m] = a_in[m];
    a[0] = (sel && k == 0) ? 0u : a_in[0];                // element 0 leaves the planes (:274)
    const uint32_t base = pos0 + ob + 4u + (uint32_t)k;
    if (low) {
        pack_low4(stage, base, a);
    } else {
        if (F > 24u) pack_group<3>(stage, base, a);
        if (F > 16u) pack_group<2>(stage, base, a);
        if (F > 8u) pack_group<1>(stage, base, a);
        pack_group<0>(stage, base, a);
    }
    stage[pos0 + ob + (uint32_t)k] = (uint8_t)sb;         // sign word, MSB = element 0 (:292-295)
    if ((uint32_t)k < ob) stage[pos0 + (uint32_t)k] = (uint8_t)(a0 >> (8 * k));   // little-endian outlier (:271-275)
}

// Decoder for one lane (HomComp/src/GSZ.cu:883-1434 up to the signed deltas): reads this lane's
// bytes of the block payload at `pos0` in the LDS stage.  Inactive blocks (rate 0, or payload
// offset beyond the stated stream size, :908-911) give zero deltas.  Branch-free like pack8: the
// first eight plane bytes are always read (up to 35 bytes past the block's end, inside the
// stage's slack) and the planes the block does not have are cut off when the bits are extracted.
// Must run with all lanes of the wave active (the outlier bytes are gathered across the quad).
// Four bytes, each in a register of its own, as one word (byte 0 first): three byte permutes.
__device__ __forceinline__ uint32_t word_of_bytes(uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3)
{
    return __builtin_amdgcn_perm(__builtin_amdgcn_perm(b3, b2, 0x0c0c0400u), __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u),
                                 0x05040100u);
}

// Planes 8G..8G+7 of the lane's eight values: byte r of (lo, hi) = those planes of value 7-r.
template <int G>
__device__ __forceinline__ void load_group(const uint8_t *stage, uint32_t base, uint32_t &lo, uint32_t &hi)
{
    uint32_t b[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) b[r] = stage[base + 4u * (uint32_t)(8 * G + r)];
    lo = word_of_bytes(b[0], b[1], b[2], b[3]);
    hi = word_of_bytes(b[4], b[5], b[6], b[7]);
    transpose8(lo, hi);
}

// Planes 0-3 only, for a wave in which no block has more: four bytes, one register.
__device__ __forceinline__ void unpack_low4(const uint8_t *stage, uint32_t base, uint32_t width, uint32_t a[8])
{
    const uint32_t y = transpose4(word_of_bytes(stage[base], stage[base + 4u], stage[base + 8u], stage[base + 12u]));
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        a[7 - r] = __builtin_amdgcn_ubfe(y, 8 * r, width);
        a[3 - r] = __builtin_amdgcn_ubfe(y, 8 * r + 4, width);
    }
}

// Sizes (size_from_header) and digests (header_digest, below) of two header bytes at once, a
// byte each in the results: the same byte-parallel arithmetic as add_sizes_from_4_headers.
__device__ __forceinline__ constexpr void sizes_and_digests_of_2_headers(uint32_t w, uint32_t &sizes, uint32_t &digests)
{
    const uint32_t F = w & 0x1f1fu;
    const uint32_t sel = (w >> 7) & 0x0101u;
    const uint32_t has_planes = ((F + 0x7f7fu) >> 7) & 0x0101u;   // F != 0
    const uint32_t ob = (((w >> 5) & 0x0303u) + 0x0101u) & (sel * 0xffu);
    sizes = (F << 2) + ((has_planes | sel) << 2) + ob;
    digests = F | (ob << 5);
}

// What the decoder needs of a header byte, in one byte: bits 0-4 the plane count F, bits 5-7 the
// number of outlier bytes (0 in plain mode, 1-4 in outlier mode).  0 for a block without payload.
__device__ __forceinline__ constexpr uint32_t header_digest(uint32_t h)
{
    const uint32_t F = h & 0x1fu;
    const uint32_t ob = (h & 0x80u) ? ((h >> 5) & 3u) + 1u : 0u;
    return F | (ob << 5);
}

// every header byte, in either place of a pair, against the two definitions a byte at a time
__device__ __forceinline__ constexpr bool pairs_of_headers_agree_with_single_ones()
{
    for (uint32_t h = 0; h < 256u; ++h) {
        const uint32_t other = (h * 167u + 13u) & 0xffu;
        uint32_t sizes = 0, digests = 0;
        sizes_and_digests_of_2_headers(h | (other << 8), sizes, digests);
        if ((sizes & 0xffu) != size_from_header(h) || (sizes >> 8) != size_from_header(other)) return false;
        if ((digests & 0xffu) != header_digest(h) || (digests >> 8) != header_digest(other)) return false;
    }
    return true;
}
static_assert(pairs_of_headers_agree_with_single_ones(), "sizes_and_digests_of_2_headers");

// (a ^ b) + c in one instruction
__device__ __forceinline__ uint32_t xor_add(uint32_t a, uint32_t b, uint32_t c)
{
    uint32_t r;
    asm("v_xad_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Decodes the lane's eight deltas of a block and adds them to v[] (wrapping).  `digest` is
// header_digest() of the block's header byte, or 0 for a block that is not to be read.
__device__ __forceinline__ void unpack8_add(const uint8_t *stage, uint32_t pos0, uint32_t digest, int k, int32_t v[8])
{
    // sixteen blocks without payload (long runs of them make up streams of sparse data): nothing to add
    if (__builtin_amdgcn_ballot_w64(digest != 0u) == 0) return;
    const uint32_t F = digest & 0x1fu;
    const uint32_t ob = digest >> 5;
    const uint32_t base = pos0 + ob + 4u + (uint32_t)k;
    uint32_t a[8];
    if (__builtin_amdgcn_ballot_w64(F > 4u) == 0) {   // wave-uniform
        unpack_low4(stage, base, F, a);
    } else {
        // Groups of eight planes: a lane reads the groups its block has; the bytes of a value are
        // then put together for as many groups as the widest block of the wave has, and the
        // planes a block does not have (stray bytes, or the zeros of a group not read) are cut off
        // in one extract of F bits.
        uint32_t lo[4] = {0u, 0u, 0u, 0u}, hi[4] = {0u, 0u, 0u, 0u};
        load_group<0>(stage, base, lo[0], hi[0]);
        if (F > 8u) load_group<1>(stage, base, lo[1], hi[1]);
        if (F > 16u) load_group<2>(stage, base, lo[2], hi[2]);
        if (F > 24u) load_group<3>(stage, base, lo[3], hi[3]);
        const bool any8 = __builtin_amdgcn_ballot_w64(F > 8u) != 0;
        const bool any16 = __builtin_amdgcn_ballot_w64(F > 16u) != 0;
        const bool any24 = __builtin_amdgcn_ballot_w64(F > 24u) != 0;
        // byte j of the second, then of the first operand
        auto two = [](int j) { return 0x0c0c0400u + 0x0101u * (uint32_t)j; };
        auto sel = [](const uint32_t (&w)[4], const uint32_t (&v)[4], int g, int r) { return r < 4 ? w[g] : v[g]; };
        if (!any8) {
#pragma unroll
            for (int r = 0; r < 8; ++r) a[7 - r] = __builtin_amdgcn_ubfe(sel(lo, hi, 0, r), 8 * (r & 3), F);
        } else if (any24) {
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const uint32_t x01 = __builtin_amdgcn_perm(sel(lo, hi, 1, r), sel(lo, hi, 0, r), two(r & 3));
                const uint32_t x23 = __builtin_amdgcn_perm(sel(lo, hi, 3, r), sel(lo, hi, 2, r), two(r & 3));
                a[7 - r] = __builtin_amdgcn_ubfe(__builtin_amdgcn_perm(x23, x01, 0x05040100u), 0, F);
            }
        } else if (any16) {
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const uint32_t x01 = __builtin_amdgcn_perm(sel(lo, hi, 1, r), sel(lo, hi, 0, r), two(r & 3));
                const uint32_t x = __builtin_amdgcn_perm(sel(lo, hi, 2, r), x01, 0x0c000100u + ((uint32_t)(4 + (r & 3)) << 16));
                a[7 - r] = __builtin_amdgcn_ubfe(x, 0, F);
            }
        } else {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                a[7 - r] = __builtin_amdgcn_ubfe(__builtin_amdgcn_perm(sel(lo, hi, 1, r), sel(lo, hi, 0, r), two(r & 3)), 0, F);
        }
    }
    const uint32_t sb = digest ? stage[pos0 + ob + (uint32_t)k] : 0u;   // :921-924, :990-994
    // outlier: lane k reads byte k, the quad ORs the pieces together (:913-917, :986-987, :1005-1006)
    const uint32_t piece = (uint32_t)k < ob ? (uint32_t)stage[pos0 + (uint32_t)k] << (8 * k) : 0u;
    const uint32_t o = quad_or(piece);
    if (ob != 0u && k == 0) a[0] = o;
#pragma unroll
    for (int m = 0; m < 8; ++m) {                         // :1432-1434
        uint32_t mask = (uint32_t)__builtin_amdgcn_sbfe((int)sb, 7 - m, 1);   // 0 or ~0
        // v + ((a ^ mask) - mask): a subtraction and one xor-add.  (Where the compiler sees where
        // the mask comes from it extracts the bit a second time to add it instead.)
        asm("" : "+v"(mask));
        v[m] = (int32_t)xor_add(a[m], mask, (uint32_t)v[m] - mask);
    }
}

// ---------------------------------------------------------------- sums in the bit-plane domain
//
// A plane of a block is one 32-bit word of the stream, so with one lane per block a single
// instruction handles a plane of all 32 elements: stream (+) stream needs no transposition at
// all.  Blocks of at most kSlicedMaxF planes are read as words (outlier bytes, sign word,
// planes), turned into two's complement plane by plane (invert where the sign bit is set, ripple
// the +1), added with a ripple of full adders, and turned back into sign and magnitude; the
// result is at most kSlicedMaxF + 1 bits wide.  Element 0 is kept out of the planes and handled
// as a scalar: in outlier mode its magnitude is the outlier (HomComp/src/GSZ.cu:913-917,
// 1005-1006), which has up to 32 bits.  In a word of the stream, byte k bit 7-m is element
// 8k+m, so element 0 is bit 7; sums of deltas need no order of the elements, and the words go
// out as they came in.
constexpr int kSlicedOutPlanes = kSlicedMaxF + 2;   // plain mode can take element 0 one plane further
// The common streams have one to three planes per block: code for kFewPlanes serves waves none
// of whose blocks has more.  stream (+) local operand takes the bit-plane path for such tiles
// only, with the local deltas as kLocalFew two's-complement planes (sign plane included), so a
// sum has up to kLocalFew + 1 bits.
constexpr uint32_t kLocalFew = 4;
constexpr int kSlicedOutWords = kSlicedOutPlanes > (int)kLocalFew + 1 ? kSlicedOutPlanes : (int)kLocalFew + 1;

typedef uint32_t __attribute__((aligned(1))) u32_unaligned;
__device__ __forceinline__ uint32_t load_u32_any(const uint8_t *p) { return *reinterpret_cast<const u32_unaligned *>(p); }
__device__ __forceinline__ void store_u32_any(lds_bytes p, uint32_t v)
{
    *(__attribute__((address_space(3))) u32_unaligned *)p = v;
}

struct SlicedIn {
    uint32_t a0, sign, ob, pl[kSlicedMaxF];
};

// The lane's block of an incoming stream straight from memory, as unaligned 32-bit words through a
// range-checked buffer descriptor (`rs` starts at the tile's payload, `ofs` is the block's offset
// in it): outlier bytes, sign word, NP planes.  A block that is not to be read (digest 0) asks
// for words beyond every buffer and gets zeros without touching memory.  Request and use are
// separate so that the words travel while the wave does something else.
constexpr uint32_t kSlicedNoRead = 0xffffff00u;

struct SlicedRaw {
    uint32_t first, sign, pl[kSlicedMaxF];
};

template <uint32_t NP>   // planes that any block of the wave can have (the others are not asked for)
__device__ __forceinline__ void sliced_request(__amdgpu_buffer_rsrc_t rs, uint32_t ofs, uint32_t digest, SlicedRaw &w)
{
    const uint32_t ob = digest >> 5;
    const uint32_t at = digest ? ofs : kSlicedNoRead;
    w.first = __builtin_amdgcn_raw_buffer_load_b32(rs, (int)at, 0, 0);
    w.sign = __builtin_amdgcn_raw_buffer_load_b32(rs, (int)(at + ob), 0, 0);
#pragma unroll
    for (uint32_t q = 0; q < NP; ++q) w.pl[q] = __builtin_amdgcn_raw_buffer_load_b32(rs, (int)(at + ob), (int)(4u + 4u * q), 0);
#pragma unroll
    for (uint32_t q = NP; q < kSlicedMaxF; ++q) w.pl[q] = 0u;   // every word has a value on every path: the struct stays in registers
}

template <uint32_t NP>
__device__ __forceinline__ void sliced_take(const SlicedRaw &w, uint32_t digest, SlicedIn &b)
{
    const uint32_t F = digest & 0x1fu;
    b.ob = digest >> 5;
    const uint32_t low_bytes = ~(0xffffff00u << ((8u * (b.ob - 1u)) & 31u));   // ob = 1..4
    b.a0 = b.ob ? w.first & low_bytes : 0u;
    b.sign = w.sign;
#pragma unroll
    for (uint32_t q = 0; q < kSlicedMaxF; ++q) b.pl[q] = 0u;
#pragma unroll
    for (uint32_t q = 0; q < NP; ++q) b.pl[q] = q < F ? w.pl[q] : 0u;
}

struct SlicedOut {
    uint32_t hdr, size, ob, F, a0, sign, m[kSlicedOutWords];
};

// Rate selection of a block summed in the bit-plane domain (HomComp/src/GSZ.cu:151-167): `nz` has
// bit q set when magnitude plane q of elements 1..31 is not empty, s0 is the sum of element 0,
// `sign` the sign plane of elements 1..31; o.m[] holds the magnitude planes, o.a0 = |s0|.
template <uint32_t NW>   // words of o.m[] a block can need
__device__ __forceinline__ void sliced_select(uint32_t nz, uint32_t s0, uint32_t sign, SlicedOut &o)
{
    constexpr uint32_t E = 0x80u;   // element 0
    const uint32_t fr2 = bit_num(nz);                      // elements 1..31   (:153)
    const uint32_t b0 = bit_num(o.a0);
    uint32_t fr1 = b0 > fr2 ? b0 : fr2;                    // all 32 elements  (:152)
    if (fr1 > 31u) fr1 = 31u;
    const uint32_t ob = (b0 + 7u) >> 3;                    // :154
    const uint32_t sz1 = fr1 ? 4u + 4u * fr1 : 0u;         // :156
    const uint32_t sz2 = 4u + 4u * fr2 + ob;               // :157
    const bool plain = sz1 <= sz2;                         // :158-164
    o.hdr = plain ? fr1 : fr2 | 0x80u | ((ob - 1u) << 5);
    o.size = plain ? sz1 : sz2;
    o.F = plain ? fr1 : fr2;
    o.ob = plain ? 0u : ob;
    o.sign = sign | (((int32_t)s0 < 0) ? E : 0u);
    // plain mode: element 0 goes back into the planes (it has at most one plane more than the rest)
    const uint32_t ins = plain ? o.a0 : 0u;
    if (__builtin_amdgcn_ballot_w64(ins != 0u) != 0) {
#pragma unroll
        for (uint32_t q = 0; q < NW; ++q) o.m[q] |= ((ins >> q) & 1u) << 7;
    }
}

// delta_out = delta_A + delta_B for the lane's block, and the block's rate selection
// (HomComp/src/GSZ.cu:151-167).
template <uint32_t NP>   // planes that any of the wave's blocks of either stream can have; the sums have NP + 1
__device__ __forceinline__ void sliced_add(const SlicedIn &A, const SlicedIn &B, SlicedOut &o)
{
    constexpr uint32_t E = 0x80u;   // element 0
    // ---- element 0: plane bits in plain mode, the outlier in outlier mode
    uint32_t m0A = A.a0, m0B = B.a0;
    {
        uint32_t anyA = 0, anyB = 0;
#pragma unroll
        for (uint32_t q = 0; q < NP; ++q) {
            anyA |= A.pl[q];
            anyB |= B.pl[q];
        }
        const bool gatherA = A.ob == 0u && (anyA & E), gatherB = B.ob == 0u && (anyB & E);
        if (__builtin_amdgcn_ballot_w64(gatherA || gatherB) != 0) {   // wave-uniform; rare where outlier mode prevails
            uint32_t gA = 0, gB = 0;
#pragma unroll
            for (uint32_t q = 0; q < NP; ++q) {
                gA |= ((A.pl[q] >> 7) & 1u) << q;
                gB |= ((B.pl[q] >> 7) & 1u) << q;
            }
            if (A.ob == 0u) m0A = gA;
            if (B.ob == 0u) m0B = gB;
        }
    }
    const uint32_t v0A = (A.sign & E) ? 0u - m0A : m0A, v0B = (B.sign & E) ? 0u - m0B : m0B;
    const uint32_t s0 = v0A + v0B;   // wrapping, as the reference's int
    const int32_t s0neg = (int32_t)(0u - s0);
    o.a0 = (uint32_t)((int32_t)s0 > s0neg ? (int32_t)s0 : s0neg);   // |s0| (0x80000000 stays)
    // ---- elements 1..31, plane by plane
    const uint32_t SA = A.sign & ~E, SB = B.sign & ~E;
    uint32_t cA = SA, cB = SB, carry = 0, r[NP + 2];
#pragma unroll
    for (uint32_t q = 0; q < NP + 2; ++q) {
        const uint32_t tA = (q < NP ? A.pl[q] & ~E : 0u) ^ SA;
        const uint32_t tB = (q < NP ? B.pl[q] & ~E : 0u) ^ SB;
        const uint32_t xA = tA ^ cA, xB = tB ^ cB;
        cA &= tA;
        cB &= tB;
        r[q] = xA ^ xB ^ carry;
        carry = (xA & xB) | (carry & (xA ^ xB));
    }
    const uint32_t SR = r[NP + 1];   // the sign plane: the sums fit NP + 1 bits
    uint32_t c = SR, nz = 0;
#pragma unroll
    for (uint32_t q = 0; q < (uint32_t)kSlicedOutWords; ++q) o.m[q] = 0;
#pragma unroll
    for (uint32_t q = 0; q < NP + 1; ++q) {
        const uint32_t t = r[q] ^ SR;
        o.m[q] = t ^ c;
        c &= t;
        nz |= (o.m[q] ? 1u : 0u) << q;
    }
    sliced_select<NP + 2>(nz, s0, SR, o);
}

// delta_out = delta_A + delta_local for the lane's block: A from a stream (sign and magnitude
// planes, NPA of them), the local deltas as NPB two's-complement planes `plB` (the last one is the
// sign plane; element 0's bit is clear in all of them) with the delta of element 0 beside them
// in b0 (HomComp/src/homcomp.cu:3601-3660 computes the same sums value by value).
template <uint32_t NPA, uint32_t NPB>
__device__ __forceinline__ void sliced_add_local(const SlicedIn &A, const uint32_t (&plB)[NPB], uint32_t b0, SlicedOut &o)
{
    constexpr uint32_t E = 0x80u;   // element 0
    constexpr uint32_t W = (NPA + 1 > NPB ? NPA + 1 : NPB) + 1;   // bits of a sum, sign included
    static_assert(W <= (uint32_t)kSlicedOutWords, "the sums fit the output planes");
    // ---- element 0: plane bits in plain mode, the outlier in outlier mode
    uint32_t m0A = A.a0;
    {
        uint32_t anyA = 0;
#pragma unroll
        for (uint32_t q = 0; q < NPA; ++q) anyA |= A.pl[q];
        const bool gatherA = A.ob == 0u && (anyA & E);
        if (__builtin_amdgcn_ballot_w64(gatherA) != 0) {   // wave-uniform; rare where outlier mode prevails
            uint32_t gA = 0;
#pragma unroll
            for (uint32_t q = 0; q < NPA; ++q) gA |= ((A.pl[q] >> 7) & 1u) << q;
            if (A.ob == 0u) m0A = gA;
        }
    }
    const uint32_t v0A = (A.sign & E) ? 0u - m0A : m0A;
    const uint32_t s0 = v0A + b0;   // wrapping, as the reference's int
    const int32_t s0neg = (int32_t)(0u - s0);
    o.a0 = (uint32_t)((int32_t)s0 > s0neg ? (int32_t)s0 : s0neg);   // |s0| (0x80000000 stays)
    // ---- elements 1..31, plane by plane
    const uint32_t SA = A.sign & ~E;
    uint32_t cA = SA, carry = 0, r[W];
#pragma unroll
    for (uint32_t q = 0; q < W; ++q) {
        const uint32_t tA = (q < NPA ? A.pl[q] & ~E : 0u) ^ SA;
        const uint32_t xA = tA ^ cA;
        cA &= tA;
        const uint32_t xB = plB[q < NPB ? q : NPB - 1];
        r[q] = xA ^ xB ^ carry;
        carry = (xA & xB) | (carry & (xA ^ xB));
    }
    const uint32_t SR = r[W - 1];   // the sign plane
    uint32_t c = SR, nz = 0;
#pragma unroll
    for (uint32_t q = 0; q < (uint32_t)kSlicedOutWords; ++q) o.m[q] = 0;
#pragma unroll
    for (uint32_t q = 0; q < W - 1; ++q) {
        const uint32_t t = r[q] ^ SR;
        o.m[q] = t ^ c;
        c &= t;
        nz |= (o.m[q] ? 1u : 0u) << q;
    }
    sliced_select<W>(nz, s0, SR, o);
}

// The local operand of a sub-step (16 blocks, 8 deltas per lane, 4 lanes per block) as
// two's-complement planes: lane k of a quad ends up with the whole word of plane k of its block.  Plane bytes come out of the same bit-matrix transposition as in pack8 (a
// lane's byte of a plane covers its 8 elements, element 0 of the lane at the top bit); the four
// bytes of a word are then collected across the quad with two lane exchanges.
// sel1 / sel2: the lane's byte selectors of the two exchanges (quad_transpose_selectors).
__device__ __forceinline__ void quad_transpose_selectors(int k, uint32_t &sel1, uint32_t &sel2)
{
    sel1 = (k & 1) ? 0x03070105u : 0x06020400u;   // odd lanes keep bytes 1, 3 and take the partner's; even lanes bytes 0, 2
    sel2 = (k & 2) ? 0x03020706u : 0x05040100u;   // lanes 2, 3 keep the upper half word, lanes 0, 1 the lower
}

// y: byte p = the lane's byte (number k) of plane p's word.  Returns the word of plane k.
__device__ __forceinline__ uint32_t quad_transpose_bytes(uint32_t y, uint32_t sel1, uint32_t sel2)
{
    const uint32_t t = dpp_u32<kDppXor1>(y);
    const uint32_t u = __builtin_amdgcn_perm(t, y, sel1);
    const uint32_t t2 = dpp_u32<kDppXor2>(u);
    return __builtin_amdgcn_perm(t2, u, sel2);
}

// Four planes of deltas within -8 .. 7.
__device__ __forceinline__ uint32_t local_planes4(const int32_t v[8], uint32_t sel1, uint32_t sel2)
{
    constexpr uint32_t two = 0x0c0c0400u;
    const uint32_t lo = __builtin_amdgcn_perm(__builtin_amdgcn_perm((uint32_t)v[4], (uint32_t)v[5], two),
                                              __builtin_amdgcn_perm((uint32_t)v[6], (uint32_t)v[7], two), 0x05040100u);
    const uint32_t hi = __builtin_amdgcn_perm(__builtin_amdgcn_perm((uint32_t)v[0], (uint32_t)v[1], two),
                                              __builtin_amdgcn_perm((uint32_t)v[2], (uint32_t)v[3], two), 0x05040100u);
    // low nibbles of lo, low nibbles of hi moved up: (lo & 0x0f0f0f0f) | ((hi << 4) & 0xf0f0f0f0)
    const uint32_t y = transpose4((lo & 0x0f0f0f0fu) | ((hi << 4) & 0xf0f0f0f0u));
    return quad_transpose_bytes(y, sel1, sel2);
}

// The block's payload at `pos` of the stage: outlier bytes (a whole word is stored; what it
// writes beyond them is overwritten by the sign word), sign word, planes.
template <uint32_t NW>   // plane words a block of the wave can have
__device__ __forceinline__ void sliced_write(lds_bytes stage, uint32_t pos, const SlicedOut &o)
{
    if (o.hdr == 0u) return;
    if (o.ob) store_u32_any(stage + pos, o.a0);
    store_u32_any(stage + pos + o.ob, o.sign);
#pragma unroll
    for (uint32_t q = 0; q < NW; ++q)
        if (q < o.F) store_u32_any(stage + pos + o.ob + 4u + 4u * q, o.m[q]);
}

// ---------------------------------------------------------------- wide blocks in the bit-plane domain
//
// stream (+) stream for blocks of up to kWideMaxF planes, a block per lane as above, laid out
// for many planes.  A lane reads its block from the sign word on in 16-byte pieces (word 0 of a
// block's pieces is the sign word, word q + 1 is plane q; measured on MI355X, pieces at a
// multiple of four bytes -- every block of a stream without outlier-mode blocks -- come in at
// the rate of memory, words one by one at two thirds of it).  Only as many pieces as the widest
// block of the wave needs are asked for, summed and written (`chunks`, wave-uniform), and a piece
// is worked on as a whole: everything below is arranged by words of the block, not by planes.
//
// The sum works on sign and magnitude directly.  With d = sign_A ^ sign_B, a + (b ^ d) + d over
// W planes is a + b where the signs agree (it fits: both are below 2^(W-1)) and a - b + 2^W where
// they differ, whose carry out of plane W - 1 says a >= b; where it is missing the W planes are
// negated (invert, ripple the +1) and the sign is B's.  A sum of zero has no sign
// (HomComp/src/GSZ.cu:93: the sign bit is "delta < 0").
//
// Element 0 (bit 7 of every word) rides along like the others while both blocks are in plain
// mode.  With an outlier-mode block in the pair its sum is made as a scalar beside the planes, as
// in sliced_add, and bit 7 of the planes is left out.
constexpr uint32_t kWideChunks = 6;
constexpr uint32_t kWideWords = 4 * kWideChunks;      // the sign word and 23 planes
// `chunks` pieces cover W = 4 * chunks - 1 planes, and the blocks summed over them have at most W - 1
constexpr uint32_t kWideMaxF = kWideWords - 2;
constexpr uint32_t kWideOutWords = kWideWords + 4;    // a sum has one plane more, and plain mode can take element 0 one plane further
constexpr uint32_t kWideOutBytes = 8 + 4 * (kWideMaxF + 2);   // outlier bytes, sign word, planes

// pieces from the sign word on that blocks of up to F planes are summed over
__device__ __forceinline__ constexpr uint32_t wide_chunks_for(uint32_t F) { return (F + 1u) / 4u + 1u; }

struct WideIn {
    uint32_t first;           // the word at the block's start (the outlier bytes of an outlier-mode block)
    uint32_t w[kWideWords];   // from the sign word on
};

struct WideOut {
    uint32_t hdr, size, ob, F, a0, w[kWideOutWords];   // w[]: from the sign word on
};

// `rs` starts at the tile's payload and reaches 16 bytes beyond the last block that is read.
// Only the lanes whose block has the piece take part in its load: a lane that asks for words
// beyond the buffer gets zeros without a memory access, but costs the load unit as much as
// one that reads (measured: the cache's access count was 2.4 times that of the words needed).
__device__ __forceinline__ void wide_request(__amdgpu_buffer_rsrc_t rs, uint32_t ofs, uint32_t digest, uint32_t chunks, WideIn &x)
{
    const uint32_t F = digest & 0x1fu, ob = digest >> 5;
    x.first = 0u;
    if (ob) x.first = __builtin_amdgcn_raw_buffer_load_b32(rs, (int)ofs, 0, 0);
#pragma unroll
    for (uint32_t j = 0; j < kWideChunks; ++j) {
        u32x4 v = {0u, 0u, 0u, 0u};
        if (j < chunks) {   // wave-uniform
            // word 4j is there when the block has 4j planes or more (a block that is not to be read has digest 0)
            if (digest != 0u && 4u * j <= F) v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(ofs + ob), (int)(16u * j), 0);
        }
        x.w[4 * j] = v.x;
        x.w[4 * j + 1] = v.y;
        x.w[4 * j + 2] = v.z;
        x.w[4 * j + 3] = v.w;
    }
}

// What the first part of a sum leaves for the second.
struct WideSum {
    uint32_t r[kWideWords];   // r[w], w >= 1: plane w - 1 of a + (b ^ d) + d
    uint32_t neg;             // elements whose planes are still to be negated
    uint32_t sign_a;          // A's sign word
    uint32_t v0;              // blocks whose element 0 is summed beside the planes: that sum
    uint32_t chunks;          // pieces the sum was made over (wave-uniform)
    bool scalar0;
};

// delta_out = delta_A + delta_B for the lane's block, first part: the planes' sum.
__device__ __forceinline__ void wide_sum(const WideIn &A, uint32_t digA, const WideIn &B, uint32_t digB, uint32_t chunks, WideSum &s)
{
    constexpr uint32_t E = 0x80u;   // element 0
    const uint32_t FA = digA & 0x1fu, FB = digB & 0x1fu, obA = digA >> 5, obB = digB >> 5;
    s.chunks = chunks;
    s.scalar0 = (obA | obB) != 0u;   // element 0 is summed beside the planes
    const uint32_t SA = A.w[0], SB = B.w[0];
    s.sign_a = SA;
    const uint32_t d = SA ^ SB;
    uint32_t carry = d;
#pragma unroll
    for (uint32_t j = 0; j < kWideChunks; ++j) {
        if (j < chunks) {   // wave-uniform
#pragma unroll
            for (uint32_t w = 4 * j ? 4 * j : 1; w < 4 * j + 4; ++w) {
                // a word beyond the block's planes belongs to the next block
                const uint32_t pa = w <= FA ? A.w[w] : 0u;
                const uint32_t pb = w <= FB ? B.w[w] : 0u;
                const uint32_t y = pb ^ d;
                const uint32_t x = pa ^ y;
                s.r[w] = x ^ carry;
                carry = (x & carry) | (~x & pa);   // the majority of pa, y and carry
            }
        }
    }
    // (The carry is hidden from the compiler here.  The same sum written for the few-plane path
    // came out wrong with hipcc 7.2 -- sums of zeros were 2^NP: the last plane, whose operands are
    // constants, was folded into the three-input bit operations that follow -- and right with
    // this empty statement in place, which costs nothing.)
    asm("" : "+v"(carry));
    s.neg = d & ~carry;   // signs differ and a < b
    // ---- element 0 beside the planes
    s.v0 = 0u;
    if (__builtin_amdgcn_ballot_w64(s.scalar0) != 0) {   // wave-uniform
        // the magnitude of a plain-mode block's element 0 lies in its planes, an outlier-mode
        // block's in the outlier (HomComp/src/GSZ.cu:913-917, 1005-1006)
        uint32_t gA = 0, gB = 0;
        if (__builtin_amdgcn_ballot_w64(s.scalar0 && (obA == 0u || obB == 0u)) != 0) {
#pragma unroll
            for (uint32_t j = 0; j < kWideChunks; ++j) {
                if (j < chunks) {
#pragma unroll
                    for (uint32_t w = 4 * j ? 4 * j : 1; w < 4 * j + 4; ++w) {
                        gA |= (w <= FA ? (A.w[w] >> 7) & 1u : 0u) << (w - 1);
                        gB |= (w <= FB ? (B.w[w] >> 7) & 1u : 0u) << (w - 1);
                    }
                }
            }
        }
        const uint32_t lowA = ~(0xffffff00u << ((8u * (obA - 1u)) & 31u)), lowB = ~(0xffffff00u << ((8u * (obB - 1u)) & 31u));
        const uint32_t m0A = obA ? A.first & lowA : gA, m0B = obB ? B.first & lowB : gB;
        const uint32_t v0A = (SA & E) ? 0u - m0A : m0A, v0B = (SB & E) ? 0u - m0B : m0B;
        s.v0 = v0A + v0B;   // wrapping, as the reference's int
    }
}

// Second part: magnitudes and signs of the sums, and the block's rate selection
// (HomComp/src/GSZ.cu:151-167).
__device__ __forceinline__ void wide_finish(const WideSum &s, WideOut &o)
{
    constexpr uint32_t E = 0x80u;   // element 0
    const uint32_t chunks = s.chunks, neg = s.neg;
    // ---- magnitudes, the planes in use, element 0's bits
    uint32_t c = neg, any = 0, fr2 = 0, g = 0;
#pragma unroll
    for (uint32_t j = 0; j <= kWideChunks; ++j) {
        if (j < chunks) {   // wave-uniform
#pragma unroll
            for (uint32_t w = 4 * j ? 4 * j : 1; w < 4 * j + 4; ++w) {
                const uint32_t t = s.r[w] ^ neg;
                const uint32_t m = t ^ c;
                c &= t;
                o.w[w] = m;
                any |= m;
                fr2 = (m & ~E) ? w : fr2;           // elements 1..31   (:153)
                g |= ((m >> 7) & 1u) << (w - 1);
            }
        } else {
            o.w[4 * j] = o.w[4 * j + 1] = o.w[4 * j + 2] = o.w[4 * j + 3] = 0u;
        }
    }
    uint32_t sign = (s.sign_a ^ neg) & any;
    // ---- element 0
    uint32_t s0neg = sign & E;   // nonzero: the sum of element 0 is negative
    o.a0 = g;
    if (s.scalar0) {
        const int32_t minus = (int32_t)(0u - s.v0);
        o.a0 = (uint32_t)((int32_t)s.v0 > minus ? (int32_t)s.v0 : minus);   // |sum| (0x80000000 stays)
        s0neg = (int32_t)s.v0 < 0 ? E : 0u;
    }
    o.w[0] = (sign & ~E) | s0neg;
    // ---- rate selection
    const uint32_t b0 = bit_num(o.a0);
    uint32_t fr1 = b0 > fr2 ? b0 : fr2;                    // all 32 elements  (:152)
    if (fr1 > 31u) fr1 = 31u;
    const uint32_t ob = (b0 + 7u) >> 3;                    // :154
    const uint32_t sz1 = fr1 ? 4u + 4u * fr1 : 0u;         // :156
    const uint32_t sz2 = 4u + 4u * fr2 + ob;               // :157
    const bool plain = sz1 <= sz2;                         // :158-164
    o.hdr = plain ? fr1 : fr2 | 0x80u | ((ob - 1u) << 5);
    o.size = plain ? sz1 : sz2;
    o.F = plain ? fr1 : fr2;
    o.ob = plain ? 0u : ob;
    // bit 7 of the planes: element 0's bits in plain mode, clear in outlier mode.  They are in
    // place where element 0 rode along; after a sum beside the planes they are put in.
    const uint32_t keep = plain && !s.scalar0 ? ~0u : ~E;
    if (__builtin_amdgcn_ballot_w64(keep != ~0u) != 0) {   // wave-uniform
#pragma unroll
        for (uint32_t j = 0; j < kWideChunks; ++j) {
            if (j < chunks) {
#pragma unroll
                for (uint32_t w = 4 * j ? 4 * j : 1; w < 4 * j + 4; ++w) o.w[w] &= keep;
            }
        }
    }
    const uint32_t ins = plain && s.scalar0 ? o.a0 : 0u;
    if (__builtin_amdgcn_ballot_w64(ins != 0u) != 0) {   // wave-uniform
#pragma unroll
        for (uint32_t j = 0; j <= kWideChunks; ++j) {
            if (j <= chunks) {
#pragma unroll
                for (uint32_t w = 4 * j ? 4 * j : 1; w < 4 * j + 4; ++w) o.w[w] |= ((ins >> (w - 1)) & 1u) << 7;
            }
        }
    }
}

typedef u32x4 __attribute__((aligned(1))) u32x4_unaligned;

// The block's payload at `pos` of the stage: outlier bytes (a whole word is stored; what it
// writes beyond them is overwritten by the sign word), sign word, planes.  The blocks of the
// lanes that write together follow each other in the stage, and the words from the fourth on go
// out in pieces of four, highest first: a block's last piece may reach up to 12 bytes into what
// follows it, where the first words of the next blocks belong, and those are written after it
// (by the last instructions here, or by the group of lanes that writes next).
__device__ __forceinline__ void wide_write(lds_bytes stage, uint32_t pos, const WideOut &o, uint32_t chunks)
{
    if (o.hdr == 0u) return;
    const lds_bytes at = stage + pos + o.ob;
#pragma unroll
    for (uint32_t j = kWideChunks; j >= 1; --j) {
        if (j <= chunks) {   // wave-uniform
            if (4u * j <= o.F)
                *(__attribute__((address_space(3))) u32x4_unaligned *)(at + 16u * j) =
                    u32x4{o.w[4 * j], o.w[4 * j + 1], o.w[4 * j + 2], o.w[4 * j + 3]};
        }
    }
    if (o.ob) store_u32_any(stage + pos, o.a0);
    store_u32_any(at, o.w[0]);
#pragma unroll
    for (uint32_t w = 1; w < 4; ++w)
        if (w <= o.F) store_u32_any(at + 4u * w, o.w[w]);
}

// ---------------------------------------------------------------- output-offset scan
//
// The byte offset of a tile's payload in the outgoing stream is an exclusive prefix sum over
// all earlier tiles (HomComp/src/GSZ.cu:170-239).  It is resolved in a single pass by a division
// of labour between the data waves (one tile per wave and round) and one scan-server workgroup of
// the same launch:
//
//   data wave, round i          publishes the tile's byte total in the tile's total word and keeps
//                               the payload (in LDS, or in its spill area when it does not fit)
//   scan server                 sweeps the total words in tile order, up to 1024 tiles per step,
//                               waits until they are all there, scans them and writes every
//                               tile's exclusive prefix into the tile's prefix word
//   data wave, round i+D-1      issues the load of the prefix word (D = 2..4 payloads kept)
//   data wave, round i+D        uses it: the payload goes to its place in the stream
//
// so a data wave never waits for another data wave, only the server waits, and every word is
// written by one wave and read by one.  (Measured on MI355X: read-modify-write atomics on one
// 128-byte line are serialised at about 11 ns each, and plain loads of a line that is being
// updated atomically by other compute units are about as slow -- a ticket counter or shared
// accumulators that thousands of waves touch cost more than the codec.)
//
// A word carries an epoch tag: bits 63-62 state (0 empty, 1 total, 2 exclusive prefix), bits
// 61-40 the call's epoch, bits 39-0 a byte count; a word of another epoch reads as empty, so the
// arrays are never cleared between calls (the host clears them when the 22-bit epoch wraps).
//
// All workgroups of the launch are resident at the same time (the grid is sized to fit the
// device), so every word waited for is on its way.  As a guard against a launch that could not
// become fully resident the waits are bounded: after `spin_limit` unsuccessful re-reads a wave
// raises *err and goes on with what it has, so the kernel always terminates.

constexpr uint64_t kValueMask = (1ull << 40) - 1;
constexpr uint32_t kEpochMask = (1u << 22) - 1;

__device__ __forceinline__ uint64_t status_word(uint32_t epoch, uint32_t state, uint64_t value)
{
    return ((uint64_t)state << 62) | ((uint64_t)(epoch & kEpochMask) << 40) | (value & kValueMask);
}

__device__ __forceinline__ uint64_t status_load(const uint64_t *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void status_store(uint64_t *p, uint64_t w)
{
    __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// state of a word under the current epoch (0 when the word belongs to an earlier call)
__device__ __forceinline__ uint32_t status_state(uint64_t w, uint32_t epoch)
{
    return (((uint32_t)(w >> 40)) & kEpochMask) == (epoch & kEpochMask) ? (uint32_t)(w >> 62) : 0u;
}

struct ScanCtx {
    uint64_t *totals;     // tile total words, written by the data workgroups
    uint64_t *prefixes;   // tile prefix words, written by the scan server
    uint32_t n_tiles;
    uint32_t epoch;
    uint32_t spin_limit;
    uint32_t *err;
};

template <int SLEEP = 1>
__device__ __forceinline__ bool scan_give_up(const ScanCtx &c, uint32_t &spins)
{
    if (++spins > c.spin_limit) {
        atomicOr(c.err, 1u);
        return true;
    }
    __builtin_amdgcn_s_sleep(SLEEP);
    return false;
}

// data side ---------------------------------------------------------------------------------

__device__ __forceinline__ void scan_publish(const ScanCtx &c, uint32_t tile, uint32_t total)
{
    status_store(&c.totals[tile], status_word(c.epoch, 1, total));
}

__device__ __forceinline__ uint64_t scan_probe(const ScanCtx &c, uint32_t tile)
{
    return status_load(&c.prefixes[tile]);
}

// Exclusive prefix of `tile` from an earlier scan_probe(tile).  `ok` is false when the wait ran
// into its bound: the word read last is not this call's prefix and must not be used as an offset.
__device__ __forceinline__ uint64_t scan_resolve(const ScanCtx &c, uint32_t tile, uint64_t w, bool &ok)
{
    uint32_t spins = 0;
    ok = true;
    // Thousands of waves may wait here at the same time, for words that share a few cache lines
    // with the words the scan server is writing: the pause between two looks keeps them from
    // crowding the server out of those lines (HC_POLL_SLEEP x 64 clocks; between 8 and 128 the
    // time of a 1 GiB call does not depend on it, short calls gain a few percent from short pauses).
    while (status_state(w, c.epoch) != 2u) {
        if (scan_give_up<HC_POLL_SLEEP>(c, spins)) {
            ok = false;
            break;
        }
        w = scan_probe(c, tile);
    }
    return w & kValueMask;
}

}  // namespace hc
