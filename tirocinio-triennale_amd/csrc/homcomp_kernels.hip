// HomComp kernels for gfx950.
//
// k_wave<NIN, LOCAL, OUT> is one persistent, single-pass kernel template that covers compress,
// decompress and the three homomorphic sums (NIN incoming streams, a local operand of float32
// values / int32 deltas / nothing, stream or float32 output).  A tile is 4096 elements = 128
// blocks and belongs to one wave; the scan-server workgroup of the same launch turns the tiles'
// byte totals into their offsets in the outgoing stream.  Small streaming kernels cover the
// incoming-stream offsets, the Lorenzo pre-pass and the value range.
#include "homcomp_device.hpp"
#include "homcomp_kernels.hpp"

#ifndef HC_LOAD_POLICY
#define HC_LOAD_POLICY 0
#endif
#ifndef HC_DEPTH_ENC
#define HC_DEPTH_ENC 2
#endif
namespace hc {

// Coalesced copy of a packed tile payload from LDS to its (arbitrarily aligned) place in the
// stream: bytes up to the first 16-byte boundary, aligned 16-byte stores assembled from
// unaligned LDS words with v_alignbyte, then the remaining bytes.
template <int LANES>
__device__ __forceinline__ void copy_out(const uint8_t *stage, uint8_t *g, uint32_t tot, int tid)
{
    const uint32_t mis = (uint32_t)((uintptr_t)g & 15u);
    uint32_t head = (16u - mis) & 15u;
    if (head > tot) head = tot;
    const uint32_t body = tot - head;
    const uint32_t nch = body >> 4;
    const uint32_t tail = body & 15u;
    if ((uint32_t)tid < head) g[tid] = stage[tid];
    const uint32_t *sw = reinterpret_cast<const uint32_t *>(stage);
    for (uint32_t c = tid; c < nch; c += LANES) {
        const uint32_t s = head + 16u * c;
        const uint32_t w0 = s >> 2, sh = s & 3u;
        const uint32_t x0 = sw[w0], x1 = sw[w0 + 1], x2 = sw[w0 + 2], x3 = sw[w0 + 3], x4 = sw[w0 + 4];
        u32x4 o;
        o.x = __builtin_amdgcn_alignbyte(x1, x0, sh);
        o.y = __builtin_amdgcn_alignbyte(x2, x1, sh);
        o.z = __builtin_amdgcn_alignbyte(x3, x2, sh);
        o.w = __builtin_amdgcn_alignbyte(x4, x3, sh);
        stream_store<u32x4>(g + s, o);
    }
    if ((uint32_t)tid < tail) g[head + 16u * nch + tid] = stage[head + 16u * nch + tid];
}

// Buffer addressing: the descriptor (base, byte count) lives in scalar registers, a lane adds a
// constant offset, and the hardware checks every dword against the byte count: loads beyond it
// return 0 and stores beyond it are dropped.  So the ends of the buffers need no branches, a
// request is a fixed number of memory operations (which lets the compiler wait for exactly the
// request it needs), and no per-lane address arithmetic is left.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const void *base, uint64_t bytes)
{
    const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}
constexpr int kBufNt = 2;   // cache policy bits of the buffer builtins: non-temporal (operands and results, touched once)
constexpr int kBufCached = 0;   // incoming payload: neighbouring sub-steps share cache lines, so these loads stay cached

// The scan server: one workgroup of the launch that turns the tile totals the data waves publish
// into exclusive prefixes (HomComp/src/GSZ.cu:170-239).  It sweeps the tiles in index order in
// steps: wait for the step's totals, scan them, write the prefixes, go on.  The data waves
// publish a whole round (G consecutive tiles, G = number of data waves) at about the same time,
// so a step rarely waits long.  Also writes the stream length once the last tile is in.
//
// Step size and progress: a data wave uses the prefix of its round-r tile two or more rounds
// later, before it publishes that round's tile.  A step must therefore never contain both a tile
// and the tile 2G after it (the step could not complete before the wave that waits for it has
// published), i.e. a step covers at most 2G tiles: 1024 tiles (4 per lane) when G >= 512,
// otherwise one tile per lane on min(256, 2G) lanes.
//
// Pace: a step is wave-scan arithmetic plus four memory instructions per lane, about 1.2 us next
// to a full grid of data waves (time stamps of the four server waves), as long as no wait in it
// covers more than the step's own request: with a wait for all outstanding operations in the
// look, every step cost a full memory round trip under load (3.7 us) and the server, not the
// data, set the pace of the stream-producing kernels.

// Status words through buffer addressing: a request or a write-back is a fixed number of memory
// instructions without a branch around them (lanes beyond the arrays read zeros, their stores
// are dropped), so the compiler can wait for exactly the request a step needs.  Device scope,
// like the atomic accesses of the data waves; issue_order() keeps the groups in program order.
constexpr int kBufStatus = 16;   // sc1

__device__ __forceinline__ void issue_order() { asm volatile("" ::: "memory"); }

template <uint32_t PER>
__device__ __forceinline__ void scan_server_steps(const TileParams &p, const ScanCtx &c, uint32_t lanes)
{
    __shared__ uint32_t s_wave[2][kWG / 64];   // by step parity: one barrier per step
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const uint32_t step = PER * lanes;
    // lane's place inside a step's words; lanes that take no part point beyond every array
    const uint32_t voff = (uint32_t)tid < lanes ? (uint32_t)tid * PER * 8u : 0xffffff00u;
    uint64_t base = 0;
    uint32_t over = 0;   // the lane's tiles with more payload than p.probe_bytes
    auto words_from = [&](const uint64_t *arr, uint32_t t0) {
        // a window from the step's first word; capped below the offset of the lanes that stay out
        uint64_t left = t0 < c.n_tiles ? (uint64_t)(c.n_tiles - t0) * 8u : 0u;
        if (left > 0x10000000u) left = 0x10000000u;
        return buffer_of(arr + (t0 < c.n_tiles ? t0 : 0u), left);
    };
    // The totals of a step are requested two steps ahead, into two register sets used
    // alternately: in the steady state they were published a round ago, so the server runs at the
    // pace of its arithmetic instead of one memory round trip per step.
    auto request = [&](uint32_t t0, uint64_t (&dst)[PER]) __attribute__((always_inline)) {
        const __amdgpu_buffer_rsrc_t rs = words_from(c.totals, t0);
        if constexpr (PER == 4) {   // two words per instruction: the step's cost is its memory instructions
            const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)voff, 0, kBufStatus);
            const u32x4 b = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(voff + 16u), 0, kBufStatus);
            dst[0] = ((uint64_t)a.y << 32) | a.x; dst[1] = ((uint64_t)a.w << 32) | a.z;
            dst[2] = ((uint64_t)b.y << 32) | b.x; dst[3] = ((uint64_t)b.w << 32) | b.z;
        } else {
#pragma unroll
            for (uint32_t j = 0; j < PER; ++j) {
                const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(rs, (int)(voff + 8u * j), 0, kBufStatus);
                dst[j] = ((uint64_t)w.y << 32) | w.x;
            }
        }
        issue_order();
    };
    auto process = [&](uint32_t t0, uint32_t parity, uint64_t (&w)[PER]) __attribute__((always_inline)) {
        const uint32_t idx = t0 + (uint32_t)tid * PER;   // n_tiles is a multiple of PER when PER > 1
        const bool in = (uint32_t)tid < lanes && t0 < c.n_tiles && idx < c.n_tiles;   // t0 beyond the end: an empty step
        auto all_there = [&]() {
            uint32_t ok = 1u;
#pragma unroll
            for (uint32_t j = 0; j < PER; ++j) ok &= (uint32_t)(status_state(w[j], c.epoch) == 1u);
            return ok != 0u;
        };
        // The first look is straight-line code, for every lane: the wait in front of it covers
        // this step's request only and leaves the later requests and the write-backs in flight.
        // (A look inside a retry loop, or behind a branch, makes the compiler wait for every
        // outstanding operation, the newest request included: a memory round trip per step.)
        const bool there = all_there();
        if (in && !there) {
            uint32_t spins = 0;
            do {
                if (scan_give_up(c, spins)) break;
                uint64_t again[PER];
#pragma unroll
                for (uint32_t j = 0; j < PER; ++j) again[j] = status_load(&c.totals[idx + j]);
#pragma unroll
                for (uint32_t j = 0; j < PER; ++j) w[j] = again[j];
            } while (!all_there());
        }
        uint32_t v[PER], mine = 0;
#pragma unroll
        for (uint32_t j = 0; j < PER; ++j) {
            // a tile total is at most kTileBlocks * kOutBlockBytes; the cap keeps every prefix within
            // the caller's buffer even when a wait gave up and a word of an earlier call is summed
            const uint32_t t = (uint32_t)(w[j] & 0xffffffffu);
            v[j] = in ? (t < (uint32_t)(kTileBlocks * kOutBlockBytes) ? t : (uint32_t)(kTileBlocks * kOutBlockBytes)) : 0u;
            mine += v[j];
        }
        const uint32_t incl = wave_incl_scan_u32(mine, lane);
        if (lane == 63) s_wave[parity][wave] = incl;
        __syncthreads();
        uint32_t before = 0, step_total = 0;
#pragma unroll
        for (int q = 0; q < kWG / 64; ++q) {
            const uint32_t t = s_wave[parity][q];
            if (q < wave) before += t;
            step_total += t;
        }
        const __amdgpu_buffer_rsrc_t rp = words_from(c.prefixes, t0);
        uint64_t run = base + before + (incl - mine);
        uint64_t o[PER];
#pragma unroll
        for (uint32_t j = 0; j < PER; ++j) {
            o[j] = status_word(c.epoch, 2, run);
            run += v[j];
        }
        if constexpr (PER == 4) {
            __builtin_amdgcn_raw_buffer_store_b128(
                u32x4{(uint32_t)o[0], (uint32_t)(o[0] >> 32), (uint32_t)o[1], (uint32_t)(o[1] >> 32)}, rp, (int)voff, 0, kBufStatus);
            __builtin_amdgcn_raw_buffer_store_b128(
                u32x4{(uint32_t)o[2], (uint32_t)(o[2] >> 32), (uint32_t)o[3], (uint32_t)(o[3] >> 32)}, rp, (int)(voff + 16u), 0,
                kBufStatus);
        } else {
#pragma unroll
            for (uint32_t j = 0; j < PER; ++j)
                __builtin_amdgcn_raw_buffer_store_b64(u32x2{(uint32_t)o[j], (uint32_t)(o[j] >> 32)}, rp, (int)(voff + 8u * j), 0,
                                                      kBufStatus);
        }
        issue_order();
        // (what follows comes after the prefixes have gone out: the data waves wait for them)
        {
            // The same offsets as plain words for the caller: absolute, header bytes included.
            // Unconditional like every memory operation of a step (the number of operations between
            // a request and its look must not depend on the path); without a destination the
            // window is empty and the stores are dropped.
            __amdgpu_buffer_rsrc_t ru = words_from(p.tile_ofs_out ? p.tile_ofs_out : c.prefixes, t0);
            if (!p.tile_ofs_out) ru = buffer_of(c.prefixes, 0);
            uint64_t at = p.hdr_bytes + base + before + (incl - mine);
            uint64_t u[PER];
#pragma unroll
            for (uint32_t j = 0; j < PER; ++j) {
                u[j] = at;
                at += v[j];
            }
            if constexpr (PER == 4) {
                __builtin_amdgcn_raw_buffer_store_b128(
                    u32x4{(uint32_t)u[0], (uint32_t)(u[0] >> 32), (uint32_t)u[1], (uint32_t)(u[1] >> 32)}, ru, (int)voff, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b128(
                    u32x4{(uint32_t)u[2], (uint32_t)(u[2] >> 32), (uint32_t)u[3], (uint32_t)(u[3] >> 32)}, ru, (int)(voff + 16u), 0, 0);
            } else {
#pragma unroll
                for (uint32_t j = 0; j < PER; ++j)
                    __builtin_amdgcn_raw_buffer_store_b64(u32x2{(uint32_t)u[j], (uint32_t)(u[j] >> 32)}, ru, (int)(voff + 8u * j), 0, 0);
            }
            issue_order();
        }
        base += step_total;
        if (p.probe_bytes != 0u) {
#pragma unroll
            for (uint32_t j = 0; j < PER; ++j) over += v[j] > p.probe_bytes ? 1u : 0u;
        }
    };
    // One loop shape for filling the pipeline and for the steady state: the first pass processes
    // two empty steps (a window beyond the end: no lane takes part) and issues the first two
    // requests.  Every path into a look then carries the same number of later operations, which
    // is what lets the compiler count instead of waiting for all of them.
    uint64_t wa[PER], wb[PER];
#pragma unroll
    for (uint32_t j = 0; j < PER; ++j) wa[j] = wb[j] = 0;
    const uint32_t none = 0xffffffffu;
    const uint64_t end = (uint64_t)c.n_tiles;
    process(none, 0, wa);
    request(0, wa);
    process(none, 1, wb);
    request(step, wb);
    for (uint64_t t0 = 0; t0 < end; t0 += 2ull * step) {
        auto at = [&](uint64_t t) { return t < end ? (uint32_t)t : none; };
        process(at(t0), 0, wa);
        request(at(t0 + 2ull * step), wa);
        process(at(t0 + step), 1, wb);
        request(at(t0 + 3ull * step), wb);
    }
    // how many tiles were larger than the slot size the host asks about
    __syncthreads();
    const uint32_t over_wave = wave_incl_scan_u32(over, lane);
    if (lane == 63) s_wave[0][wave] = over_wave;
    __syncthreads();
    if (tid == 0) {
        const uint64_t len = p.hdr_bytes + base;   // HomComp/src/GSZ.cu:752-755
        *p.total = len;
        if (p.user_total) *p.user_total = len;
        // for the host's choice of the next launch's LDS budget
        if (p.host_total) {
            uint32_t over_all = 0;
#pragma unroll
            for (int q = 0; q < kWG / 64; ++q) over_all += s_wave[0][q];
            const uint64_t share = p.probe_bytes ? (uint64_t)over_all * 256u / c.n_tiles : 0u;
            *p.host_total = ((base / c.n_tiles) & 0xffffffffu) | ((uint64_t)(p.probe_bytes / 64u) << 32) | (share << 48);
        }
    }
}

__device__ __forceinline__ void scan_server(const TileParams &p, const ScanCtx &c, uint32_t G)
{
    if (G >= 512u)
        scan_server_steps<4>(p, c, (uint32_t)kWG);
    else
        scan_server_steps<1>(p, c, 2u * G < (uint32_t)kWG ? 2u * G : (uint32_t)kWG);
}

// ---------------------------------------------------------------- wave-autonomous kernels
//
// k_wave<NIN, LOCAL, OUT>: all five operations with one tile per WAVE and no workgroup barrier
// anywhere.  A workgroup is four independent waves that share nothing but the launch; each wave
// walks its tiles (tile = wave index, += number of data waves) and handles a tile as kSub
// sub-steps of 16 blocks (512 elements, 8 per lane, 4 lanes per block).  Everything a sub-step
// consumes from memory was requested two sub-steps earlier into registers (two register sets
// used alternately), across tile boundaries as well:
//   local operand      2 x 16 bytes per lane
//   incoming payload   the 16 blocks of a sub-step are one contiguous byte range of the stream;
//                      lane l holds its l-th aligned 16-byte chunk (ranges beyond 1 KiB fetch the
//                      rest on the spot), which goes through a small LDS stage to the byte-wise
//                      decoder
//   incoming headers   the 128 header bytes of the next tile are fetched a tile ahead; before the
//                      first payload request of that tile they are turned into block offsets
//                      (in-wave scan) and kept in LDS, double-buffered by tile parity
// Stream output: rate selection, an in-wave DPP scan of the 16 block sizes, pack at the running
// offset into the wave's LDS stage.  The tile's place in the stream comes from the scan server
// (HomComp/src/GSZ.cu:170-239): total published when the tile is packed, prefix requested a
// round later, payload copied out two rounds later.  The LDS stage of a wave is sized by the launch
// (a budget chosen from the expected compressed size: smaller stages let more waves share a
// compute unit); a tile that outgrows its slot continues in the wave's slot of a global spill
// area and is copied out from there.
constexpr int kSub = kTileBlocks / 16;
constexpr int kInStage = 16 * kMaxBlockBytes + 96;   // one sub-step's payload range, alignment shift, read-ahead slack

template <int LOCAL>
struct SubRegs {
    f32x4 f[2];
    i32x4 i[2];
};

// Operand of one sub-step of the tile whose elements start at `tile_elem0` (beyond n: zeros).
template <int LOCAL>
__device__ __forceinline__ void load_sub(SubRegs<LOCAL> &r, const void *local, uint64_t n, uint64_t tile_elem0,
                                         bool valid, int s, int lane)
{
    if constexpr (LOCAL == kLocalNone) return;
    const uint64_t left = valid && tile_elem0 < n ? (n - tile_elem0) * 4u : 0u;
    const __amdgpu_buffer_rsrc_t rs = buffer_of((const uint8_t *)local + (valid ? tile_elem0 * 4u : 0u), left);
    const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 32, s * 2048, HC_LOAD_POLICY);
    const u32x4 b = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 32 + 16, s * 2048, HC_LOAD_POLICY);
    if constexpr (LOCAL == kLocalF32) {
        r.f[0] = __builtin_bit_cast(f32x4, a);
        r.f[1] = __builtin_bit_cast(f32x4, b);
    } else {
        r.i[0] = __builtin_bit_cast(i32x4, a);
        r.i[1] = __builtin_bit_cast(i32x4, b);
    }
}

// Orders the LDS traffic of the lanes of one wave: LDS operations of a wave execute in program
// order, so no instruction is needed, only a point the compiler does not move them across.
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Whole 16-byte pieces from the front of a wave's LDS slot to its spill slot (both 16-byte aligned).
__device__ __forceinline__ void spill_pieces(const uint8_t *stage, uint8_t *slot_at, uint32_t bytes, int lane)
{
    for (uint32_t i = 16u * (uint32_t)lane; i < bytes; i += 1024u)
        *reinterpret_cast<u32x4 *>(slot_at + i) = *reinterpret_cast<const u32x4 *>(stage + i);
}

// Copy of a spilled tile from the wave's slot of the spill area to its place in the stream: like
// copy_out, bytes up to the first 16-byte boundary of the destination, aligned 16-byte stores put
// together from two aligned 16-byte pieces of the slot, then the remaining bytes.  The slot is
// read with device-scope loads (it was written by this wave, but an older copy of a line may sit
// in the vector cache from the slot's previous use).
__device__ __forceinline__ void copy_out_spill(const uint8_t *slot, uint8_t *g, uint32_t tot, int lane)
{
    const uint32_t mis = (uint32_t)((uintptr_t)g & 15u);
    uint32_t head = (16u - mis) & 15u;
    if (head > tot) head = tot;
    const uint32_t body = tot - head;
    const uint32_t nch = body >> 4;
    const uint32_t tail = body & 15u;
    const uint32_t *sw = reinterpret_cast<const uint32_t *>(slot);
    auto byte_at = [&](uint32_t i) {
        return (uint8_t)(__hip_atomic_load(sw + (i >> 2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> (8u * (i & 3u)));
    };
    if ((uint32_t)lane < head) g[lane] = byte_at((uint32_t)lane);
    const __amdgpu_buffer_rsrc_t rs = buffer_of(slot, kSpillSlotBytes);
    const uint32_t ws = head >> 2, bs = head & 3u;   // source word and byte shift, the same for every piece
    for (uint32_t c = lane; c < nch; c += 64) {
        const uint32_t s = head + 16u * c;
        const u32x4 A = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(s & ~15u), 0, kBufStatus);
        const u32x4 B = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(s & ~15u) + 16, 0, kBufStatus);
        uint32_t w0, w1, w2, w3, w4;
        switch (ws) {
        case 0: w0 = A.x; w1 = A.y; w2 = A.z; w3 = A.w; w4 = B.x; break;
        case 1: w0 = A.y; w1 = A.z; w2 = A.w; w3 = B.x; w4 = B.y; break;
        case 2: w0 = A.z; w1 = A.w; w2 = B.x; w3 = B.y; w4 = B.z; break;
        default: w0 = A.w; w1 = B.x; w2 = B.y; w3 = B.z; w4 = B.w; break;
        }
        u32x4 o;
        o.x = __builtin_amdgcn_alignbyte(w1, w0, bs);
        o.y = __builtin_amdgcn_alignbyte(w2, w1, bs);
        o.z = __builtin_amdgcn_alignbyte(w3, w2, bs);
        o.w = __builtin_amdgcn_alignbyte(w4, w3, bs);
        stream_store<u32x4>(g + s, o);
    }
    if ((uint32_t)lane < tail) g[head + 16u * nch + lane] = byte_at(head + 16u * nch + (uint32_t)lane);
}

// Tile and round indices inside a launch.  32-bit arithmetic keeps the comparisons against the
// tile count scalar, which the kernels with incoming streams (short of scalar registers) gain 1-3 %
// from; compress, which has registers to spare, came out 1.7 % slower with it and keeps 64 bits.
template <int NIN> struct TileIndex { typedef int32_t type; };
template <> struct TileIndex<0> { typedef int64_t type; };

// Registers of one incoming stream that travel ahead of the computation.
struct InRegs {
    u32x4 chunk;   // the lane's 16-byte chunk of a sub-step's payload range
};

// BITPLANE: the kernel's bit-plane path (kPlanesNone: none).  stream (+) local operand comes with
// and without the path for tiles of few planes: the host launches the kind without where the
// incoming streams are too wide for it anyway, because the general path alone is the faster code
// for such data (fewer registers in use; a tile of the general path costs about 8 % more in the
// kernel that has both).  stream (+) stream comes with the path for few planes or with the one
// for wide blocks.
enum : int { kPlanesNone = 0, kPlanesFew = 1, kPlanesWide = 2 };
template <int NIN, int LOCAL, int OUT, int BITPLANE>
__global__ __launch_bounds__(kWG) __attribute__((amdgpu_waves_per_eu(4))) void k_wave(const TileParams p)
{
    constexpr bool kEnc = OUT == kOutStream;
    constexpr int kW = kWG / 64;
    constexpr int kIn = NIN > 0 ? NIN : 1;
    // Sub-steps between a request and its use.  A wave's memory operations complete in order, so
    // waiting for a load also waits for every store issued before it: the decoder, which stores
    // 2 KiB per sub-step, looks further ahead to keep more of its stores in flight.
    constexpr int kDepth = HC_DEPTH_ENC > 0 && kEnc ? HC_DEPTH_ENC : 4;
    static_assert(kSub % kDepth == 0, "the register sets rotate with the sub-steps of a tile");
    // stage of the packed tiles that wait for their stream offset: p.stage_bytes per wave, sized by
    // the launch (dynamic LDS), see TileParams
    extern __shared__ __align__(16) uint8_t s_dyn[];
    __shared__ __align__(4) uint8_t s_hdr_out[kW][kEnc ? kTileBlocks : 4];
    // one stage per wave: the incoming streams of a sub-step are decoded one after the other
    // stream (+) stream as a sum in the bit-plane domain, tile by tile where the tiles allow it
    constexpr bool kSliced = BITPLANE == kPlanesFew && kEnc && NIN == 2 && LOCAL == kLocalNone;
    // the same for blocks of many planes
    constexpr bool kWide = BITPLANE == kPlanesWide && kEnc && NIN == 2 && LOCAL == kLocalNone;
    // stream (+) local operand likewise, the local deltas turned into bit planes on the way
    constexpr bool kSlicedLocal = BITPLANE == kPlanesFew && kEnc && NIN == 1 && LOCAL != kLocalNone;
    constexpr bool kAnySliced = kSliced || kSlicedLocal;   // the paths that keep a half tile's words in registers ahead of their use
    constexpr bool kAnyPlanes = kAnySliced || kWide;
    // the planes of the local operand of half a tile, a row of 64 words per plane and one for the
    // deltas of the blocks' first elements; they share the wave's stage of incoming payload
    constexpr int kLocalRows = (int)kLocalFew + 1;
    constexpr int kInBytes = kSlicedLocal && kLocalRows * 256 > kInStage ? kLocalRows * 256 : kInStage;
    __shared__ __align__(16) uint8_t s_in[kW][NIN > 0 ? kInBytes : 16];
    __shared__ __align__(4) uint16_t s_ofs_in[kW][kIn][2][NIN > 0 ? kTileBlocks : 2];
    __shared__ __align__(4) uint8_t s_hdr_in[kW][kIn][2][NIN > 0 ? kTileBlocks : 4];
    __shared__ __align__(16) float s_tr[kW][kEnc ? 4 : 512];     // decoder: exchange of the lanes' output pieces
    __shared__ uint32_t s_rel[kW][kIn][2][NIN > 0 ? kSub + 1 : 1];   // tile-relative start of every sub-step's range

    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));   // wave-uniform, kept in a scalar register
    const int lane = threadIdx.x & 63;
    const int k = lane & 3;
    const int quad = lane >> 2;
    // tile indices are 32-bit: a launch has fewer than 2^31 - 2^15 tiles (the host checks), so
    // tile + D * waves stays below 2^31 and the comparisons are scalar instructions
    typedef typename TileIndex<NIN>::type tidx;
    const tidx n_tiles = (tidx)p.n_tiles;
    const ScanCtx scan{p.tile_totals, p.tile_prefixes, p.n_tiles, p.epoch, p.spin_limit, p.error};
    // on the encoder the last workgroup of the grid is the scan server
    const tidx G = kEnc ? (tidx)gridDim.x - 1 : (tidx)gridDim.x;
    const tidx GW = G * kW;   // data waves
    if constexpr (kEnc) {
        if ((tidx)blockIdx.x == G) {
            scan_server(p, scan, (uint32_t)GW);
            return;
        }
    }
    const tidx wid = (tidx)blockIdx.x * kW + wave;
    if (wid >= n_tiles) return;   // no barrier in this kernel: a wave without work just leaves

    auto tile_of = [&](tidx r) { return wid + r * GW; };

    // ---- incoming streams: per-tile context
    uint32_t hdr_next[kIn];     // header bytes of blocks 2*lane, 2*lane+1 of the next tile
    uint64_t start_next[kIn];   // absolute payload offset of the next tile
    uint64_t start_ctx0[kIn], start_ctx1[kIn];   // of the tiles in the two context buffers (tile parity)
    // bytes of the stream from the tile's payload start to its stated end, saturated to 32 bits:
    // everything inside a tile is 32-bit arithmetic against these
    uint32_t room_ctx0[kIn], room_ctx1[kIn];
    uint32_t end_ctx0[kIn], end_ctx1[kIn];   // payload bytes of those tiles
    uint32_t few_ctx = 0;   // bit-plane paths: bit b set = the blocks of the tile in context b (any stream) have few enough planes for them
    auto fetch_headers = [&](tidx r) __attribute__((always_inline)) {
        if constexpr (NIN > 0) {
            tidx t = tile_of(r);
            if (t >= n_tiles) t = 0;   // loads are issued unconditionally; the values are not used then
#pragma unroll
            for (int c = 0; c < NIN; ++c) {
                if constexpr (kSlicedLocal) {
                    // Through a descriptor of the tile's header bytes: the address is the tile's, in
                    // scalar registers, plus the lane.  These kernels use every vector register, and
                    // the per-lane pointer the plain form keeps across the rounds was spilled to
                    // scratch memory; fetching it back waits for every load under way (4 % of a call).
                    const __amdgpu_buffer_rsrc_t hb = buffer_of(p.in[c] + (uint64_t)t * kTileBlocks, kTileBlocks);
                    hdr_next[c] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(hb, 2 * lane, 0, 0);
                } else {
                    const uint8_t *h = p.in[c] + (uint64_t)t * kTileBlocks + 2 * lane;
                    hdr_next[c] = (uint32_t)h[0] | ((uint32_t)h[1] << 8);
                }
                const uint64_t st = p.in_ofs[c][t];
                start_next[c] = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(st >> 32)) << 32) |
                                (uint32_t)__builtin_amdgcn_readfirstlane((int)st);
            }
        }
    };
    // header bytes -> block offsets of tile r in context buffer r & 1 (HomComp/src/GSZ.cu:790-874)
    auto prepare = [&](tidx r, int b) __attribute__((always_inline)) {
        if constexpr (NIN > 0) {
            if (tile_of(r) < n_tiles) {
#pragma unroll
                for (int c = 0; c < NIN; ++c) {
                    uint32_t sizes, digests;
                    sizes_and_digests_of_2_headers(hdr_next[c], sizes, digests);
                    const uint32_t z0 = sizes & 0xffu, z1 = sizes >> 8;
                    const uint32_t incl = wave_incl_scan_u32(z0 + z1, lane);
                    const uint32_t o0 = incl - z0 - z1, o1 = o0 + z0;
                    *reinterpret_cast<uint32_t *>(&s_ofs_in[wave][c][b][2 * lane]) = o0 | (o1 << 16);
                    if ((lane & 7) == 0) s_rel[wave][c][b][lane >> 3] = o0;
                    if (lane == 63) s_rel[wave][c][b][kSub] = incl;
                    const uint64_t room64 = p.in_size[c] > start_next[c] ? p.in_size[c] - start_next[c] : 0u;
                    const uint32_t room = room64 > 0xffff0000ull ? 0xffff0000u : (uint32_t)room64;
                    // what the sub-steps need of the header bytes; a block without payload, or one
                    // that starts at or beyond the stated size (out-of-bound rule of
                    // HomComp/src/GSZ.cu:908-911 on the absolute payload offset), is not read
                    const uint32_t d0 = z0 != 0u && o0 < room ? digests & 0xffu : 0u;
                    const uint32_t d1 = z1 != 0u && o1 < room ? digests >> 8 : 0u;
                    *reinterpret_cast<uint16_t *>(&s_hdr_in[wave][c][b][2 * lane]) = (uint16_t)(d0 | (d1 << 8));
                    if constexpr (kAnyPlanes) {
                        // stream (+) stream takes tiles of up to kSlicedMaxF or kWideMaxF planes, stream (+) local operand of up to kFewPlanes
                        constexpr uint32_t most = kWide ? kWideMaxF : (kSliced ? kSlicedMaxF : kFewPlanes);
                        const bool few = __builtin_amdgcn_ballot_w64((d0 & 0x1fu) > most || (d1 & 0x1fu) > most) == 0;
                        const uint32_t bit = 1u << b;
                        if (c == 0) few_ctx |= bit;
                        if (!few) few_ctx &= ~bit;
                    }
                    const uint32_t tile_end = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
                    if (b) {
                        start_ctx1[c] = start_next[c];
                        room_ctx1[c] = room;
                        end_ctx1[c] = tile_end;
                    } else {
                        start_ctx0[c] = start_next[c];
                        room_ctx0[c] = room;
                        end_ctx0[c] = tile_end;
                    }
                }
                wave_lds_fence();
            }
        }
    };

    // ---- requests kDepth sub-steps ahead, into kDepth register sets used in rotation
    SubRegs<LOCAL> loc[kDepth];
    InRegs in[kDepth][kIn];
    // byte range of sub-step s of the tile in context b: aligned base address, bytes from there
    auto range_of = [&](int c, int b, int s, uintptr_t &ga, uint32_t &shift, uint32_t &nbytes, uint32_t &rel0)
                        __attribute__((always_inline)) {
        rel0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_rel[wave][c][b][s]);
        const uint32_t rel1 = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_rel[wave][c][b][s + 1]);
        const uint64_t start = b ? start_ctx1[c] : start_ctx0[c];
        // a block that starts below the stated size is read in full (HomComp/src/GSZ.cu:908-911),
        // nothing further out is touched
        const uint32_t room = b ? room_ctx1[c] : room_ctx0[c];
        const uint32_t lim = room ? room + (kMaxBlockBytes - 1) : 0u;
        const uint32_t end = rel1 < lim ? rel1 : lim;
        const uintptr_t g0 = (uintptr_t)p.in[c] + start + rel0;
        ga = g0 & ~(uintptr_t)15;
        shift = (uint32_t)(g0 - ga);
        nbytes = end > rel0 ? shift + (end - rel0) : 0u;
    };
    // The registers of a set are free again as soon as the sub-step has converted the operand /
    // staged the chunk, and the request for the sub-step after the next one is issued right there:
    // as early as possible, and ahead of the sub-step's own stores (a wave's memory operations
    // complete in order, so a load is only as fast as the stores issued before it).
    auto request_local = [&](tidx r, int s, SubRegs<LOCAL> &loc) __attribute__((always_inline)) {
        const tidx t = tile_of(r);
        load_sub<LOCAL>(loc, p.local, p.n, (uint64_t)t * kTileElems, t < n_tiles, s, lane);
    };
    // (`wanted` false: nothing is read, the registers are only given a value)
    auto request_in = [&](int c, tidx r, int b, int s, InRegs (&in)[kIn], bool wanted = true) __attribute__((always_inline)) {
        if constexpr (kSliced || kWide) {
            if (!wanted) {   // wave-uniform; cheaper here than a request that fetches nothing
                in[c].chunk = u32x4{0u, 0u, 0u, 0u};
                return;
            }
        }
        uintptr_t ga;
        uint32_t shift, nbytes, rel0;
        range_of(c, b, s, ga, shift, nbytes, rel0);
        // whole 16-byte pieces; lanes beyond the range get zeros without touching memory
        const __amdgpu_buffer_rsrc_t rs =
            buffer_of(reinterpret_cast<const void *>(ga), wanted && tile_of(r) < n_tiles ? (nbytes + 15u) & ~15u : 0u);
        in[c].chunk = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16, 0, kBufCached);
    };
    auto request = [&](tidx r, int b, int s, SubRegs<LOCAL> &loc, InRegs (&in)[kIn], bool wanted = true) __attribute__((always_inline)) {
        request_local(r, s, loc);
        if constexpr (NIN > 0) {
#pragma unroll
            for (int c = 0; c < NIN; ++c) request_in(c, r, b, s, in, wanted);
        }
    };

    // ---- stream (+) stream in the bit-plane domain (tiles none of whose blocks has more than
    //      kSlicedMaxF planes): a lane reads the words of its block (outlier bytes, sign word,
    //      planes) straight from the stream, unaligned, through a descriptor of the tile's
    //      payload.  The words of half a tile (64 blocks) are asked for while the half before is
    //      summed, the first half of a tile at the end of the tile before, so they travel while
    //      the wave copies the finished tile out.
    // Most streams this path sees have one to three planes per block: a wave none of whose blocks
    // (of the half, either stream) has more takes the code for three.
    constexpr uint32_t kFewer = kFewPlanes;
    SlicedRaw sl_raw[kIn];
    uint32_t sl_dig[kIn];
    bool sl_fewer = false;
    // (`wanted` false: nothing is read, the registers are only given a value, so that they are not
    // kept alive through a tile of the general path)
    auto sliced_request_half = [&](int b, int half, bool wanted) __attribute__((always_inline)) {
        if constexpr (kAnySliced) {
            // (stream (+) local operand, see fetch_headers: the lane number taken anew, because the
            // addresses made from it once and kept across the rounds were spilled to scratch memory)
            int fresh_lane = lane;
            if constexpr (kSlicedLocal) asm volatile("" : "+v"(fresh_lane));
            const int blk = half * 64 + fresh_lane;
            bool more = false;
#pragma unroll
            for (int c = 0; c < NIN; ++c) {
                sl_dig[c] = wanted ? (uint32_t)s_hdr_in[wave][c][b][blk] : 0u;
                more = more || (sl_dig[c] & 0x1fu) > kFewer;
            }
            sl_fewer = __builtin_amdgcn_ballot_w64(more) == 0;
#pragma unroll
            for (int c = 0; c < NIN; ++c) {
                const uint32_t ofs = s_ofs_in[wave][c][b][blk];
                const uint32_t room = b ? room_ctx1[c] : room_ctx0[c];
                const uint32_t rel_end = b ? end_ctx1[c] : end_ctx0[c];
                // a block that starts below the stated size is read in full (HomComp/src/GSZ.cu:908-911);
                // the words asked for beyond a block's last plane end at most `reach` bytes into the tile
                uint32_t lim = room ? room + (kMaxBlockBytes - 1) : 0u;
                const uint32_t reach = rel_end + 8u + 4u * kSlicedMaxF;
                if (lim > reach) lim = reach;
                const __amdgpu_buffer_rsrc_t pay = buffer_of(p.in[c] + (b ? start_ctx1[c] : start_ctx0[c]), lim);
                if (sl_fewer)
                    sliced_request<kFewer>(pay, ofs, sl_dig[c], sl_raw[c]);
                else
                    sliced_request<kSlicedMaxF>(pay, ofs, sl_dig[c], sl_raw[c]);
            }
        }
    };
    // the blocks written at once (outlier bytes, sign word, planes: 32 blocks, 16 wide ones) must fit an empty slot
    constexpr uint32_t kSlicedWords = kSlicedLocal ? kLocalFew + 1u : (uint32_t)kSlicedOutPlanes;
    constexpr uint32_t kSlicedAtOnce = kWide ? 16u : 32u;
    const bool sliced_ok = kAnyPlanes && p.sliced &&
                           ((p.stage_bytes / p.out_slots) & ~15u) - 64u >= kSlicedAtOnce * (kWide ? kWideOutBytes : 8u + 4u * kSlicedWords) + 16u;
    // The local operand is only known to fit its planes (deltas within -8 .. 7) once it has been
    // quantised.  A tile goes down the bit-plane path when its incoming blocks have few planes
    // and the tile before gave no reason for doubt: a half tile whose local deltas did not fit is
    // redone by the general path and withdraws the trust, a tile of the general path whose sums
    // all have few planes restores it.
    bool sl_trust = true;
    uint32_t planes_seen = 0;   // general path: the largest plane count among the lane's output blocks of the tile
    // does the tile in context b take the bit-plane path?
    auto sliced_ctx = [&](int b) __attribute__((always_inline)) { return sliced_ok && sl_trust && ((few_ctx >> b) & 1u) != 0; };
    uint32_t sel1 = 0, sel2 = 0;
    if constexpr (kSlicedLocal) quad_transpose_selectors(k, sel1, sel2);

    fetch_headers(0);
    prepare(0, 0);
    sliced_request_half(0, 0, sliced_ctx(0));
    if constexpr (!kWide) {
#pragma unroll
        for (int j = 0; j < kDepth; ++j) request(0, 0, j, loc[j], in[j], !sliced_ctx(0));
    }

    // Deferred tiles: a tile packed in round r is copied out in round r + D (D = p.out_slots, 2 to
    // 4): its total is published when it is packed, the prefix word is requested in round
    // r + D - 1 and used at the start of round r + D.  The wave's LDS stage is cut into D slots;
    // more, smaller slots give the scan more time to come back (the words travel through memory,
    // several microseconds each way under load) at the price of spilling tiles beyond a slot.
    // Measured on MI355X: two slots are enough, three or four are not faster.
    const int D = (int)p.out_slots;
    const uint32_t slot_bytes = (p.stage_bytes / (uint32_t)D) & ~15u;
    const uint32_t slot_cap = slot_bytes - 64u;
    uint32_t tot[4] = {0, 0, 0, 0};     // byte totals of the tiles of the previous rounds, newest first
    uint32_t spl[4] = {0, 0, 0, 0};     // how many of their first bytes lie in the spill slot (the rest in the LDS slot)
    uint64_t probe = 0;                // prefix word of the oldest one, requested a round ago

    for (tidx r = 0;; ++r) {
        const tidx t0 = tile_of(r);
        const tidx tp = t0 - (tidx)(D - 1) * GW;   // its prefix is requested at the end of this round
        const tidx td = t0 - (tidx)D * GW;         // copied out at the start of this round
        const bool v0 = t0 < n_tiles;
        const bool vp = kEnc && r >= D - 1 && tp < n_tiles;
        const bool vd = kEnc && r >= D && td < n_tiles;
        if (!v0 && (!kEnc || td >= n_tiles)) break;
        const int buf = (int)(r & 1);
        const int obuf = (int)(r % D);
        uint8_t *stage = s_dyn + (uint32_t)wave * p.stage_bytes + (uint32_t)obuf * slot_bytes;
        uint8_t *slot = kEnc ? p.spill + ((uint64_t)wid * (uint64_t)D + (uint64_t)obuf) * kSpillSlotBytes : nullptr;

        // ---- the tile packed D rounds ago goes to its place in the stream
        if constexpr (kEnc) {
            if (vd) {
                const uint32_t total_d = D == 2 ? tot[1] : (D == 3 ? tot[2] : tot[3]);
                const uint32_t spilled_d = D == 2 ? spl[1] : (D == 3 ? spl[2] : spl[3]);
                // the prefix word travels in lane 0 only: a device-scope load is executed per
                // lane, so 64 lanes asking for the same word would be 64 requests
                uint64_t excl = 0;
                {
                    // Every wave of a round has to publish before the round's last prefixes
                    // exist, so the launch moves at the pace of its slowest waves (the hardware
                    // favours the oldest waves of a SIMD: the workgroup that arrived last on a
                    // compute unit ran 60 % slower per tile than the first).  A wave whose
                    // prefix is already there runs behind the scan and takes the higher issue
                    // priority for this round; one that has to wait runs ahead and yields.
                    const int behind = __builtin_amdgcn_readfirstlane((int)(status_state(probe, scan.epoch) == 2u));
                    if (behind)
                        __builtin_amdgcn_s_setprio(1);
                    else
                        __builtin_amdgcn_s_setprio(0);
                }
                bool got = true;
                if (lane == 0) excl = scan_resolve(scan, (uint32_t)td, probe, got);
                excl = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(excl >> 32)) << 32) |
                       (uint32_t)__builtin_amdgcn_readfirstlane((int)excl);
                // A wait that ran into its bound leaves no offset: the tile is dropped (the call
                // is reported as failed).  An offset is also only taken when the tiles before
                // this one can add up to it (each emits at most kTileBlocks * kOutBlockBytes
                // bytes), so nothing is ever written beyond the capacity the caller provides,
                // whatever the scan words hold after a failed call.
                const bool usable = __builtin_amdgcn_readfirstlane((int)got) != 0 &&
                                    excl <= (uint64_t)td * (uint64_t)(kTileBlocks * kOutBlockBytes);
                if (!usable && lane == 0) atomicOr(scan.err, 1u);
                uint8_t *dst = p.out_cmp + p.hdr_bytes + excl;
                // the pieces that went to the spill slot, then what stayed in LDS (behind them in the
                // slot's numbering: LDS position 0 is the tile's byte `spilled_d`)
                if (usable && spilled_d) copy_out_spill(slot, dst, spilled_d, lane);
                if (usable && total_d > spilled_d) copy_out<64>(stage, dst + spilled_d, total_d - spilled_d, lane);
            }
        }

        // ---- this round's tile
        uint32_t run = 0;
        // The prefix word of the tile to be copied out next round is asked for late in the round,
        // when the scan server has had its time; on the bit-plane path of stream (+) local operand
        // ahead of the requests for the next tile, which are the last thing such a tile does
        // (measured: 3 % of the call).
        bool probed = false;
        auto probe_next = [&]() __attribute__((always_inline)) {
            if constexpr (kEnc) {
                if (vp && lane == 0) probe = scan_probe(scan, (uint32_t)tp);
                probed = true;
            }
        };
        // A tile that outgrows its LDS slot goes to the wave's slot of the spill area piece by
        // piece: whenever the next sub-step would not fit, the whole 16-byte pieces packed so far
        // are flushed with wide stores and packing goes on at the front of the LDS slot
        // (`flushed` = tile bytes already in the spill slot, a multiple of 16); what is in LDS at
        // the end of the tile stays there until the tile is copied out.  Only a sub-step
        // that does not fit an empty LDS slot (tiny slots, incompressible data) is packed into
        // the spill slot directly, byte by byte, and so is the rest of its tile.
        bool direct0 = false;
        uint32_t flushed = 0;
        if (v0) {
            fetch_headers(r + 1);
            const uint64_t tile_elem0 = (uint64_t)t0 * kTileElems;
            // room in the LDS slot for the next `bytes` of the tile (see above); false: they are to
            // be packed into the spill slot in place
            auto make_room = [&](uint32_t bytes) __attribute__((always_inline)) {
                if (!direct0 && run - flushed + bytes > slot_cap) {
                    const uint32_t local = run - flushed, whole = local & ~15u, rest = local & 15u;
                    spill_pieces(stage, slot + flushed, whole, lane);
                    if (rest + bytes > slot_cap) {
                        // not even an empty slot holds this much: the rest of the tile is packed in place
                        if ((uint32_t)lane < rest) slot[flushed + whole + (uint32_t)lane] = stage[whole + (uint32_t)lane];
                        direct0 = true;
                    } else {
                        // the bytes beyond the last whole piece move to the front of the slot
                        const uint8_t moved = (uint32_t)lane < rest ? stage[whole + (uint32_t)lane] : (uint8_t)0;
                        wave_lds_fence();
                        if ((uint32_t)lane < rest) stage[lane] = moved;
                        wave_lds_fence();
                        flushed += whole;
                    }
                }
                return !direct0;
            };
            // sub-step s of this tile; (r2, b2, s2) is the sub-step the freed registers are requested for
            // the lane's eight local deltas of a sub-step from its operand registers;
            // elements beyond the end arrive as zeros (0.0f quantises to 0), as the reference pads
            auto local_deltas = [&](const SubRegs<LOCAL> &loc, int32_t (&v)[8]) __attribute__((always_inline)) {
                if constexpr (LOCAL == kLocalF32) {
                    // HomComp/src/GSZ.cu:82-149: quantise, Lorenzo with prevQuant = 0 at block start
                    const float x[8] = {loc.f[0].x, loc.f[0].y, loc.f[0].z, loc.f[0].w,
                                        loc.f[1].x, loc.f[1].y, loc.f[1].z, loc.f[1].w};
                    int32_t q[8];
#pragma unroll
                    for (int m = 0; m < 8; ++m) q[m] = quantize(x[m], p.recip);
                    uint32_t prev = dpp_u32<kDppRowShr1>((uint32_t)q[7]);
                    if (k == 0) prev = 0;
                    v[0] = (int32_t)((uint32_t)q[0] - prev);
#pragma unroll
                    for (int m = 1; m < 8; ++m) v[m] = (int32_t)((uint32_t)q[m] - (uint32_t)q[m - 1]);
                } else if constexpr (LOCAL == kLocalI32) {
                    // HomComp/src/homcomp.cu:2252-2268: precomputed deltas
                    v[0] = loc.i[0].x; v[1] = loc.i[0].y; v[2] = loc.i[0].z; v[3] = loc.i[0].w;
                    v[4] = loc.i[1].x; v[5] = loc.i[1].y; v[6] = loc.i[1].z; v[7] = loc.i[1].w;
                } else {
#pragma unroll
                    for (int m = 0; m < 8; ++m) v[m] = 0;
                }
            };
            // `ahead` false: the registers are not sent out again (a sub-step run out of turn)
            auto sub = [&](int s, SubRegs<LOCAL> &loc, InRegs (&in)[kIn], tidx r2, int b2, int s2, bool ahead = true)
                           __attribute__((always_inline)) {
                // the blocks' digests and offsets first: nothing in the sub-step writes them, and
                // read here they are on their way while the wave waits for its operands
                uint32_t digest[kIn], ofs[kIn];
                if constexpr (NIN > 0) {
#pragma unroll
                    for (int c = 0; c < NIN; ++c) {
                        digest[c] = s_hdr_in[wave][c][buf][s * 16 + quad];
                        ofs[c] = s_ofs_in[wave][c][buf][s * 16 + quad];
                    }
                }
                int32_t v[8];
                local_deltas(loc, v);
                if (ahead) request_local(r2, s2, loc);
                if constexpr (NIN > 0) {
#pragma unroll
                    for (int c = 0; c < NIN; ++c) {
                        // ---- the sub-step's payload range: registers -> LDS stage
                        uintptr_t ga;
                        uint32_t shift, nbytes, rel0;
                        range_of(c, buf, s, ga, shift, nbytes, rel0);
                        uint8_t *st = s_in[wave];
                        if (16u * (uint32_t)lane < nbytes)
                            *reinterpret_cast<u32x4 *>(st + 16u * lane) = in[c].chunk;
                        if (nbytes > 1024u) {   // a range of more than 64 pieces: the rest is fetched now
                            const __amdgpu_buffer_rsrc_t rs =
                                buffer_of(reinterpret_cast<const void *>(ga), (nbytes + 15u) & ~15u);
                            for (uint32_t i = (uint32_t)lane + 64u; 16u * i < nbytes; i += 64u)
                                *reinterpret_cast<u32x4 *>(st + 16u * i) =
                                    __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(16u * i), 0, kBufCached);
                        }
                        if (ahead) request_in(c, r2, b2, s2, in);
                        wave_lds_fence();
                        // ---- decode (HomComp/src/GSZ.cu:883-1434)
                        unpack8_add(st, shift + ofs[c] - rel0, digest[c], k, v);
                        wave_lds_fence();   // the stage is rewritten by the next stream and the next sub-step
                    }
                }
                if constexpr (!kEnc) {
                    // ---- HomComp/src/GSZ.cu:1426-1468: running sum inside the block, dequantise, store
                    uint32_t q[8];
                    q[0] = (uint32_t)v[0];
#pragma unroll
                    for (int m = 1; m < 8; ++m) q[m] = q[m - 1] + (uint32_t)v[m];
                    const uint32_t s0 = dpp_u32<kDppBcast0>(q[7]);
                    const uint32_t s1 = dpp_u32<kDppBcast1>(q[7]);
                    const uint32_t s2 = dpp_u32<kDppBcast2>(q[7]);
                    const uint32_t off = (k > 0 ? s0 : 0u) + (k > 1 ? s1 : 0u) + (k > 2 ? s2 : 0u);
                    float y[8];
#pragma unroll
                    for (int m = 0; m < 8; ++m) y[m] = dequantize((int32_t)(q[m] + off), p.eb);
                    // The lanes' 32-byte pieces are exchanged through LDS so that each store
                    // instruction writes 1 KiB of consecutive bytes (full cache lines): stores of
                    // 16 bytes at a 32-byte stride reach only a fraction of the write bandwidth.
                    // 16-byte piece P of the 2 KiB lives at piece P ^ x(P), x = bit 3 ^ bit 4 of P:
                    // a lane writes pieces 2 * lane and 2 * lane + 1 and reads pieces lane and
                    // 64 + lane, and with the swap the lanes that access the LDS in the same
                    // cycle (8 or 16 neighbours) hit different banks both ways.
                    float *tr = s_tr[wave];
                    const int xw = ((lane >> 2) ^ (lane >> 3)) & 1, xr = ((lane >> 3) ^ (lane >> 4)) & 1;
                    *reinterpret_cast<f32x4 *>(tr + 4 * (2 * lane + xw)) = f32x4{y[0], y[1], y[2], y[3]};
                    *reinterpret_cast<f32x4 *>(tr + 4 * (2 * lane + 1 - xw)) = f32x4{y[4], y[5], y[6], y[7]};
                    wave_lds_fence();
                    const f32x4 lo = *reinterpret_cast<const f32x4 *>(tr + 4 * (lane ^ xr));
                    const f32x4 hi = *reinterpret_cast<const f32x4 *>(tr + 256 + 4 * (lane ^ xr));
                    wave_lds_fence();
                    const __amdgpu_buffer_rsrc_t ro =
                        buffer_of(p.out_f32 + tile_elem0, tile_elem0 < p.n ? (p.n - tile_elem0) * 4u : 0u);
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, lo), ro, lane * 16, s * 2048, kBufNt);
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, hi), ro, lane * 16 + 1024, s * 2048, kBufNt);
                } else {
                    // ---- rate selection (HomComp/src/GSZ.cu:151-167) and the block's offset: the
                    //      sizes are equal in the four lanes of a quad, so a scan over the quads
                    //      minus the own size is the exclusive prefix in every lane
                    uint32_t a[8], sb, hd, size, a0;
                    analyse8(v, k, a, sb, hd, size, a0, NIN == 0 && p.plain != 0);
                    const uint32_t incl = quad_incl_scan_u32(size);
                    const uint32_t sub_total = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
                    if (k == 0) s_hdr_out[wave][s * 16 + quad] = (uint8_t)hd;
                    if constexpr (kSlicedLocal) planes_seen = planes_seen > (hd & 0x1fu) ? planes_seen : (hd & 0x1fu);
                    make_room(sub_total);
                    if (direct0)
                        pack8((global_bytes)slot, run + incl - size, hd, k, a, sb, a0);
                    else
                        pack8((lds_bytes)stage, run - flushed + incl - size, hd, k, a, sb, a0);
                    run += sub_total;
                }
            };
            const bool sliced_tile = sliced_ctx(buf);
            if (sliced_tile) {
                if constexpr (kSliced) {
                    // ---- the whole tile in the bit-plane domain, 64 blocks (a block per lane) at a time
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        SlicedIn A, B;
                        SlicedOut out;
                        const bool fewer = sl_fewer;
                        if (fewer) {
                            sliced_take<kFewer>(sl_raw[0], sl_dig[0], A);
                            sliced_take<kFewer>(sl_raw[1], sl_dig[1], B);
                        } else {
                            sliced_take<kSlicedMaxF>(sl_raw[0], sl_dig[0], A);
                            sliced_take<kSlicedMaxF>(sl_raw[1], sl_dig[1], B);
                        }
                        if (half == 0) sliced_request_half(buf, 1, true);   // on its way while the first half is summed
                        if (fewer)
                            sliced_add<kFewer>(A, B, out);
                        else
                            sliced_add<kSlicedMaxF>(A, B, out);
                        s_hdr_out[wave][half * 64 + lane] = (uint8_t)out.hdr;
                        const uint32_t incl = wave_incl_scan_u32(out.size, lane);
                        const uint32_t first32 = (uint32_t)__builtin_amdgcn_readlane((int)incl, 31);
                        const uint32_t all64 = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
                        // two writes of 32 blocks each, so that what is written at once fits an empty slot
#pragma unroll
                        for (int q = 0; q < 2; ++q) {
                            const uint32_t bytes = q ? all64 - first32 : first32;
                            make_room(bytes);   // always true here: 32 blocks fit an empty slot
                            const uint32_t pos = run - flushed + (incl - out.size) - (q ? first32 : 0u);
                            if ((lane >> 5) == q) {
                                if (fewer)
                                    sliced_write<kFewer + 2>((lds_bytes)stage, pos, out);
                                else
                                    sliced_write<kSlicedMaxF + 2>((lds_bytes)stage, pos, out);
                            }
                            run += bytes;
                        }
                    }
                    wave_lds_fence();
                    // the next tile's block offsets and first requests: of its first half on this
                    // path, else as the sub-steps below leave them
                    prepare(r + 1, buf ^ 1);
                    const bool next_sliced = tile_of(r + 1) < n_tiles && sliced_ctx(buf ^ 1);
                    sliced_request_half(buf ^ 1, 0, next_sliced);
#pragma unroll
                    for (int j = 0; j < kDepth; ++j) request(r + 1, buf ^ 1, j, loc[j], in[j], !next_sliced);
                }
                if constexpr (kWide) {
                    // ---- the whole tile in the bit-plane domain, 64 blocks (a block per lane) at a
                    //      time: the blocks' words are asked for, in 16-byte pieces from the sign
                    //      word on, as many as the widest block of the wave has; summed; written.
                    //      Nothing travels ahead of its use here (the other waves of the SIMD
                    //      fill the wait; registers for a half tile ahead are not to be had).
#pragma unroll 1
                    for (int half = 0; half < 2; ++half) {
                        const int blk = half * 64 + lane;
                        uint32_t dig[kIn], ofs[kIn];
                        uint32_t widest = 0;
#pragma unroll
                        for (int c = 0; c < NIN; ++c) {
                            dig[c] = (uint32_t)s_hdr_in[wave][c][buf][blk];
                            ofs[c] = s_ofs_in[wave][c][buf][blk];
                            widest = widest > (dig[c] & 0x1fu) ? widest : (dig[c] & 0x1fu);
                        }
                        uint32_t chunks = 1;
#pragma unroll
                        for (uint32_t j = 1; j < kWideChunks; ++j)
                            if (__builtin_amdgcn_ballot_w64(wide_chunks_for(widest) > j) != 0) chunks = j + 1u;
                        WideIn AB[kIn];
#pragma unroll
                        for (int c = 0; c < NIN; ++c) {
                            const uint32_t room = buf ? room_ctx1[c] : room_ctx0[c];
                            const uint32_t rel_end = buf ? end_ctx1[c] : end_ctx0[c];
                            // a block that starts below the stated size is read in full (HomComp/src/GSZ.cu:908-911);
                            // a block's last piece ends at most 12 bytes beyond the block
                            uint32_t lim = room ? room + (kMaxBlockBytes - 1) + 16u : 0u;
                            const uint32_t reach = rel_end + 16u;
                            if (lim > reach) lim = reach;
                            const __amdgpu_buffer_rsrc_t pay = buffer_of(p.in[c] + (buf ? start_ctx1[c] : start_ctx0[c]), lim);
                            wide_request(pay, ofs[c], dig[c], chunks, AB[c]);
                        }
                        WideOut out;
                        {
                            WideSum sum;
                            wide_sum(AB[0], dig[0], AB[kIn - 1], dig[kIn - 1], chunks, sum);
                            wide_finish(sum, out);
                        }
                        s_hdr_out[wave][blk] = (uint8_t)out.hdr;
                        const uint32_t incl = wave_incl_scan_u32(out.size, lane);
                        // four writes of 16 blocks each, so that what is written at once fits an empty slot
                        uint32_t before = 0;
#pragma unroll 1
                        for (int q = 0; q < 4; ++q) {
                            const uint32_t upto = (uint32_t)__builtin_amdgcn_readlane((int)incl, 16 * q + 15);
                            const uint32_t bytes = upto - before;
                            make_room(bytes);   // always true here: 16 blocks fit an empty slot
                            const uint32_t pos = run - flushed + (incl - out.size) - before;
                            if ((lane >> 4) == q) wide_write((lds_bytes)stage, pos, out, chunks);
                            run += bytes;
                            before = upto;
                        }
                    }
                    wave_lds_fence();
                    prepare(r + 1, buf ^ 1);   // the next tile's block offsets
                }
                if constexpr (kSlicedLocal) {
                    // ---- stream (+) local operand in the bit-plane domain, half a tile at a time:
                    //      four sub-steps turn the local values into deltas (as the general path
                    //      does) and the deltas into two's-complement planes, a row of words per
                    //      plane in LDS; then a lane takes a block: the incoming block's words from
                    //      its registers, the local block's planes from the rows, sum, rate selection,
                    //      payload words into the stage.
                    uint32_t *rows = reinterpret_cast<uint32_t *>(s_in[wave]);
                    bool fell_back = false;
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        bool all4 = true;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int s = 4 * half + j;
                            SubRegs<LOCAL> &L = loc[s % kDepth];
                            int32_t v[8];
                            local_deltas(L, v);
                            {   // the freed registers go out for the sub-step kDepth further on (the next tile's at the end)
                                const int wrap = s + kDepth >= kSub ? 1 : 0;
                                request_local(r + wrap, s + kDepth - wrap * kSub, L);
                            }
                            // element 0 of a block stays out of the planes (its delta is the value itself)
                            const uint32_t b0 = (uint32_t)v[0];
                            if (k == 0) v[0] = 0;
                            int32_t mx = v[0] > v[1] ? v[0] : v[1], mn = v[0] < v[1] ? v[0] : v[1];
#pragma unroll
                            for (int m = 2; m < 8; ++m) {
                                mx = mx > v[m] ? mx : v[m];
                                mn = mn < v[m] ? mn : v[m];
                            }
                            const int32_t z = mx > ~mn ? mx : ~mn;   // deltas within -(z + 1) .. z
                            all4 = all4 && __builtin_amdgcn_ballot_w64(z > 7) == 0;
                            const uint32_t at = (uint32_t)(j * 16 + quad);   // the block's lane in the second phase
                            rows[(uint32_t)k * 64u + at] = local_planes4(v, sel1, sel2);   // plane k
                            if (k == 0) rows[kLocalFew * 64u + at] = b0;
                        }
                        wave_lds_fence();
                        SlicedIn A;
                        sliced_take<kFewer>(sl_raw[0], sl_dig[0], A);
                        if (half == 0) sliced_request_half(buf, 1, true);   // on its way while the first half is summed
                        if (all4) {
                            SlicedOut out;
                            const uint32_t b0 = rows[kLocalFew * 64u + (uint32_t)lane];
                            uint32_t plB[kLocalFew];
#pragma unroll
                            for (uint32_t q = 0; q < kLocalFew; ++q) plB[q] = rows[q * 64u + (uint32_t)lane];
                            sliced_add_local<kFewer, kLocalFew>(A, plB, b0, out);
                            wave_lds_fence();   // the rows are rewritten by the next half
                            s_hdr_out[wave][half * 64 + lane] = (uint8_t)out.hdr;
                            const uint32_t incl = wave_incl_scan_u32(out.size, lane);
                            const uint32_t first32 = (uint32_t)__builtin_amdgcn_readlane((int)incl, 31);
                            const uint32_t all64 = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
                            // two writes of 32 blocks each, so that what is written at once fits an empty slot
#pragma unroll
                            for (int q = 0; q < 2; ++q) {
                                const uint32_t bytes = q ? all64 - first32 : first32;
                                make_room(bytes);   // always true here: 32 blocks fit an empty slot
                                const uint32_t pos = run - flushed + (incl - out.size) - (q ? first32 : 0u);
                                if ((lane >> 5) == q) sliced_write<kLocalFew + 1>((lds_bytes)stage, pos, out);
                                run += bytes;
                            }
                        } else {
                            // local deltas beyond the planes: these four sub-steps go down the general
                            // path after all, their operands fetched again on the spot
                            fell_back = true;
#pragma unroll 1
                            for (int s = 4 * half; s < 4 * half + 4; ++s) {
                                SubRegs<LOCAL> again;
                                InRegs again_in[kIn];
                                request_local(r, s, again);
                                request_in(0, r, buf, s, again_in);
                                sub(s, again, again_in, r, buf, s, false);
                            }
                        }
                    }
                    wave_lds_fence();
                    if (fell_back) sl_trust = false;
                    probe_next();
                    prepare(r + 1, buf ^ 1);
                    const bool next_sliced = tile_of(r + 1) < n_tiles && sliced_ctx(buf ^ 1);
                    sliced_request_half(buf ^ 1, 0, next_sliced);
#pragma unroll
                    for (int j = 0; j < kDepth; ++j) request_in(0, r + 1, buf ^ 1, j, in[j], !next_sliced);
                }
            } else if constexpr (kWide) {
                // A tile with a block beyond the bit-plane path: the general path, its operands
                // fetched on the spot.  (The host launches this kernel for streams whose tiles
                // rarely come here, and nothing is kept in registers for them.)
#pragma unroll 1
                for (int s = 0; s < kSub; ++s) {
                    SubRegs<LOCAL> now;
                    InRegs now_in[kIn];
                    request(r, buf, s, now, now_in);
                    sub(s, now, now_in, r, buf, s, false);
                }
                prepare(r + 1, buf ^ 1);
            } else {
            planes_seen = 0;
#pragma unroll 1
            for (int s = 0; s < kSub; s += kDepth) {
                // the requests of the last kDepth sub-steps are the next tile's, whose block offsets
                // must be in place before
                const int wrap = s + kDepth >= kSub ? 1 : 0;
                if (wrap) prepare(r + 1, buf ^ 1);
                const int s2 = s + kDepth - wrap * kSub;
#pragma unroll
                for (int j = 0; j < kDepth; ++j) sub(s + j, loc[j], in[j], r + wrap, buf ^ wrap, s2 + j);
            }
            if constexpr (kSlicedLocal) sl_trust = __builtin_amdgcn_ballot_w64(planes_seen > kFewPlanes) == 0;
            if constexpr (kAnySliced) sliced_request_half(buf ^ 1, 0, tile_of(r + 1) < n_tiles && sliced_ctx(buf ^ 1));
            }
            if constexpr (kEnc) {
                wave_lds_fence();
                // header bytes of the tile (HomComp/src/GSZ.cu:166)
                if constexpr (kSlicedLocal) {   // (as for the incoming header bytes)
                    const __amdgpu_buffer_rsrc_t ho = buffer_of(p.out_cmp + (uint64_t)t0 * kTileBlocks, kTileBlocks);
#pragma unroll
                    for (int i = lane; i < kTileBlocks; i += 64)
                        __builtin_amdgcn_raw_buffer_store_b8(s_hdr_out[wave][i], ho, i, 0, 0);
                } else {
#pragma unroll
                    for (int i = lane; i < kTileBlocks; i += 64)
                        p.out_cmp[(uint64_t)t0 * kTileBlocks + i] = s_hdr_out[wave][i];
                }
                if (lane == 0) scan_publish(scan, (uint32_t)t0, run);
            }
        }
        if constexpr (kEnc) {
            if (!probed) probe_next();
            tot[3] = tot[2]; tot[2] = tot[1]; tot[1] = tot[0]; tot[0] = run;
            spl[3] = spl[2]; spl[2] = spl[1]; spl[1] = spl[0]; spl[0] = direct0 ? run : flushed;
        }
    }
}

// ---------------------------------------------------------------- incoming-stream offsets
//
// The payload offset of a tile of an incoming stream depends on the header bytes only
// (HomComp/src/GSZ.cu:790-874), so it is computed ahead of the tile kernel, in one launch over
// blocks of 256 tiles: a workgroup sums the block sizes of each of its tiles (16 header bytes
// per lane), publishes the block's total in the block's word, scans its 256 totals, adds up
// the totals of the earlier blocks as they appear and writes the tiles' absolute offsets
// (`base` = header length).  A workgroup only ever waits for workgroups with smaller indices,
// which the hardware starts first, and every one of them publishes before it waits, so the
// waits end whatever else runs on the device; they are bounded all the same (a wait that runs
// into its bound raises the error flag, and the offsets it leaves are only ever used to read
// within the stream's stated size).  The words carry the launch's epoch like the scan words of
// the tile kernels, so they are never cleared between calls.

constexpr uint32_t kOfsBlockTiles = 256;
constexpr uint32_t kBlockSumBits = 23;

__device__ __forceinline__ uint32_t wg_reduce_u32(uint32_t v, uint32_t *s_tmp)
{
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    v += __shfl_xor(v, 8, 64);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    if ((threadIdx.x & 63) == 0) s_tmp[threadIdx.x >> 6] = v;
    __syncthreads();
    uint32_t t = 0;
    for (uint32_t w = 0; w < blockDim.x / 64; ++w) t += s_tmp[w];
    __syncthreads();
    return t;
}

// One launch serves up to two streams (blockIdx.y), each with its own arrays.
__global__ __launch_bounds__(256) void k_in_offsets(const InOffsetsArgs a, uint32_t n_tiles, uint64_t base,
                                                    uint32_t epoch, uint32_t spin_limit)
{
    const uint8_t *__restrict__ hdr = a.hdr[blockIdx.y];
    uint64_t *__restrict__ words = a.block_words[blockIdx.y];
    uint64_t *__restrict__ ofs = a.ofs[blockIdx.y];
    __shared__ uint32_t s_tmp[4];
    __shared__ uint32_t s_tot[kOfsBlockTiles];
    uint32_t acc = 0, few_tiles = 0;
    constexpr uint32_t kPieces = kTileBlocks / 16;            // 16-byte header pieces (lanes) per tile
    constexpr uint32_t kPasses = kOfsBlockTiles * kPieces / 256;
    // all pieces of the thread are requested before the first is used: the kernel is a handful of
    // dependent memory round trips otherwise (9 us for any stream length)
    u32x4 q[kPasses];
    const bool aligned = ((uintptr_t)hdr & 15u) == 0;
#pragma unroll
    for (uint32_t it = 0; it < kPasses; ++it) {
        const uint32_t t = (blockIdx.x * kPasses + it) * 256u + threadIdx.x;   // piece index
        q[it] = u32x4{0u, 0u, 0u, 0u};   // zero header bytes: blocks of size 0
        if (t / kPieces < n_tiles) {
            const uint8_t *src = hdr + (uint64_t)t * 16u;
            if (aligned) {
                q[it] = *reinterpret_cast<const u32x4 *>(src);
            } else {
                uint32_t w[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    w[i] = (uint32_t)src[4 * i] | ((uint32_t)src[4 * i + 1] << 8) |
                           ((uint32_t)src[4 * i + 2] << 16) | ((uint32_t)src[4 * i + 3] << 24);
                q[it] = u32x4{w[0], w[1], w[2], w[3]};
            }
        }
    }
#pragma unroll
    for (uint32_t it = 0; it < kPasses; ++it) {
        const uint32_t t = (blockIdx.x * kPasses + it) * 256u + threadIdx.x;
        const uint32_t tile = t / kPieces;
        uint32_t sum = add_sizes_from_4_headers(q[it].x, 0u);
        sum = add_sizes_from_4_headers(q[it].y, sum);
        sum = add_sizes_from_4_headers(q[it].z, sum);
        sum = add_sizes_from_4_headers(q[it].w, sum);
        acc += sum;
        // the eight pieces of a tile sit in eight neighbouring lanes
        static_assert(kPieces == 8, "reduction over groups of eight lanes");
        sum += dpp_u32<kDppXor1>(sum);
        sum += dpp_u32<kDppXor2>(sum);
        sum += dpp_u32<kDppRowHalfMirror>(sum);   // the other quad of the eight
        // does any block of the tile have more than a.few_limit planes?  Byte-parallel: F + (127 -
        // limit) reaches bit 7 of its byte exactly then (nothing carries from byte to byte)
        const uint32_t slack = 0x7f7f7f7fu - a.few_limit * 0x01010101u;
        uint32_t wider = (((q[it].x & 0x1f1f1f1fu) + slack) | ((q[it].y & 0x1f1f1f1fu) + slack) |
                          ((q[it].z & 0x1f1f1f1fu) + slack) | ((q[it].w & 0x1f1f1f1fu) + slack)) & 0x80808080u;
        wider |= dpp_u32<kDppXor1>(wider);
        wider |= dpp_u32<kDppXor2>(wider);
        wider |= dpp_u32<kDppRowHalfMirror>(wider);
        if ((threadIdx.x & (kPieces - 1)) == 0) {
            if (tile < n_tiles) few_tiles += wider == 0u ? 1u : 0u;
            s_tot[tile % kOfsBlockTiles] = sum;   // 0 beyond the last tile
        }
    }
    // a block's bytes stay below 2^23 (256 tiles of at most 128 * 132 bytes): its count of tiles
    // with few planes (at most 256) travels in the bits above, through the reduction as well
    static_assert(kOfsBlockTiles * kTileBlocks * kMaxBlockBytes < (1u << kBlockSumBits), "packing of the block totals");
    const uint32_t block_packed = wg_reduce_u32(acc | (few_tiles << kBlockSumBits), s_tmp);   // with a barrier: s_tot is complete
    const uint32_t block_few = block_packed >> kBlockSumBits;
    if (threadIdx.x == 0) status_store(&words[blockIdx.x], status_word(epoch, 2u, block_packed));
    // a first look at the words of the blocks before this one, on its way during the scan below
    uint64_t first_look = 0;
    if (threadIdx.x < blockIdx.x) first_look = status_load(&words[threadIdx.x]);

    // the block's own tiles
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t mine = s_tot[threadIdx.x];
    const uint32_t incl = wave_incl_scan_u32(mine, lane);
    if (lane == 63) s_tmp[wave] = incl;
    __syncthreads();
    uint32_t earlier = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w)
        if (w < wave) earlier += s_tmp[w];
    __syncthreads();

    // the blocks before it, 256 at a time
    const bool last = (blockIdx.x + 1) * kOfsBlockTiles >= n_tiles;   // this block also reports the count of tiles with few planes
    uint64_t before = 0;
    uint32_t few_before = block_few;
    bool ok = true;
    for (uint32_t q0 = 0; q0 < blockIdx.x; q0 += 256) {
        const uint32_t b = q0 + threadIdx.x;
        uint32_t packed = 0;
        if (b < blockIdx.x) {
            uint64_t w = q0 == 0 ? first_look : status_load(&words[b]);
            uint32_t spins = 0;
            while (ok && status_state(w, epoch) != 2u) {
                if (++spins > spin_limit) {
                    ok = false;   // and no further waiting in this launch
                } else {
                    __builtin_amdgcn_s_sleep(2);
                    w = status_load(&words[b]);
                }
            }
            packed = ok ? (uint32_t)w : 0u;
        }
        // 256 values below 2^23 each: the sum fits 32 bits (the counts are summed apart: the byte
        // totals of 256 blocks would carry into them)
        before += wg_reduce_u32(packed & ((1u << kBlockSumBits) - 1u), s_tmp);
        if (last) few_before += wg_reduce_u32(packed >> kBlockSumBits, s_tmp);
    }
    if (!ok) atomicOr(a.error, 1u);
    const uint32_t tile = blockIdx.x * kOfsBlockTiles + threadIdx.x;
    if (tile < n_tiles) ofs[tile] = base + before + earlier + (incl - mine);
    if (threadIdx.x == 0 && last && a.few_report[blockIdx.y])
        *a.few_report[blockIdx.y] = ((uint64_t)n_tiles << 32) | few_before;
}

// HomComp/src/homcomp.cu:1553-1602: Lorenzo deltas of the quantised values as int32.
__global__ __launch_bounds__(kWG) void k_quant_predict(const float *__restrict__ x,
                                                       int32_t *__restrict__ out, uint64_t n,
                                                       float recip)
{
    const int k = threadIdx.x & 3;
    const uint64_t e0 = ((uint64_t)blockIdx.x * kWG + threadIdx.x) * kEPL;
    float xv[8];
    const bool full = e0 + kEPL <= n;
    if (full) {
        const float4 *src = reinterpret_cast<const float4 *>(x + e0);
        const float4 f0 = src[0], f1 = src[1];
        xv[0] = f0.x; xv[1] = f0.y; xv[2] = f0.z; xv[3] = f0.w;
        xv[4] = f1.x; xv[5] = f1.y; xv[6] = f1.z; xv[7] = f1.w;
    } else {
#pragma unroll
        for (int m = 0; m < 8; ++m) xv[m] = e0 + m < n ? x[e0 + m] : 0.0f;
    }
    int32_t q[8], d[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) q[m] = quantize(xv[m], recip);
    uint32_t prev = dpp_u32<kDppRowShr1>((uint32_t)q[7]);
    if (k == 0) prev = 0;
    d[0] = (int32_t)((uint32_t)q[0] - prev);
#pragma unroll
    for (int m = 1; m < 8; ++m) d[m] = (int32_t)((uint32_t)q[m] - (uint32_t)q[m - 1]);
    if (full) {
        int4 *dst = reinterpret_cast<int4 *>(out + e0);
        dst[0] = make_int4(d[0], d[1], d[2], d[3]);
        dst[1] = make_int4(d[4], d[5], d[6], d[7]);
    } else {
#pragma unroll
        for (int m = 0; m < 8; ++m)
            if (e0 + m < n) out[e0 + m] = d[m];
    }
}

// HomComp/src/homcomp_eval.cu:156-163: float32 minimum and maximum.  Comparisons as in the
// reference, so NaN elements never replace a bound.  Stage 1 leaves one (min,max) pair per
// workgroup, stage 2 folds the pairs.
__device__ __forceinline__ void minmax_fold(float &lo, float &hi, float a, float b)
{
    if (a < lo) lo = a;
    if (b > hi) hi = b;
}

__device__ __forceinline__ void wg_minmax(float &lo, float &hi)
{
    __shared__ float s_lo[kWG / 64], s_hi[kWG / 64];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const float a = __shfl_xor(lo, d, 64), b = __shfl_xor(hi, d, 64);
        minmax_fold(lo, hi, a, b);
    }
    if ((threadIdx.x & 63) == 0) {
        s_lo[threadIdx.x >> 6] = lo;
        s_hi[threadIdx.x >> 6] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kWG / 64; ++w) minmax_fold(lo, hi, s_lo[w], s_hi[w]);
    }
}

__global__ __launch_bounds__(kWG) void k_range_partial(const float *__restrict__ x, uint64_t n,
                                                       float *__restrict__ partial)
{
    const float first = x[0];
    float lo = first, hi = first;
    const uint64_t n4 = n / 4;
    const uint64_t stride = (uint64_t)gridDim.x * kWG;
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    for (uint64_t i = (uint64_t)blockIdx.x * kWG + threadIdx.x; i < n4; i += stride) {
        const float4 f = x4[i];
        minmax_fold(lo, hi, f.x, f.x);
        minmax_fold(lo, hi, f.y, f.y);
        minmax_fold(lo, hi, f.z, f.z);
        minmax_fold(lo, hi, f.w, f.w);
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const float f = x[n4 * 4 + threadIdx.x];
        minmax_fold(lo, hi, f, f);
    }
    wg_minmax(lo, hi);
    if (threadIdx.x == 0) {
        partial[2 * blockIdx.x] = lo;
        partial[2 * blockIdx.x + 1] = hi;
    }
}

__global__ __launch_bounds__(kWG) void k_range_final(const float *__restrict__ partial, uint32_t np,
                                                     float *__restrict__ out)
{
    float lo = partial[0], hi = partial[1];
    for (uint32_t i = threadIdx.x; i < np; i += kWG) minmax_fold(lo, hi, partial[2 * i], partial[2 * i + 1]);
    wg_minmax(lo, hi);
    if (threadIdx.x == 0) {
        out[0] = lo;
        out[1] = hi;
    }
}

// Zero fill used where a captured graph must not contain a memset node.
__global__ void k_fill_u64(uint64_t *p, uint64_t n)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// ---------------------------------------------------------------- launchers

template <int NIN, int LOCAL, int OUT, int BITPLANE>
static hipError_t launch_wave(const TileParams &p, uint32_t max_grid, hipStream_t s)
{
    // data workgroups of four waves (one tile per wave and round), on the encoder + the scan server
    const uint32_t extra = OUT == kOutStream ? 1u : 0u;
    uint32_t grid = (p.n_tiles + 3u) / 4u + extra;
    if (grid > max_grid) grid = max_grid;
    if (grid < 1u + extra) grid = 1u + extra;
    const uint32_t dyn = OUT == kOutStream ? (kWG / 64) * p.stage_bytes : 0u;
    hipLaunchKernelGGL((k_wave<NIN, LOCAL, OUT, BITPLANE>), dim3(grid), dim3(kWG), dyn, s, p);
    return hipGetLastError();
}

template <int NIN, int LOCAL, int OUT, int BITPLANE>
static hipError_t wave_resident_blocks(int *blocks_per_cu, uint32_t stage_bytes, uint32_t max_stage_bytes)
{
    const size_t dyn = OUT == kOutStream ? (size_t)(kWG / 64) * stage_bytes : 0;
    const size_t max_dyn = OUT == kOutStream ? (size_t)(kWG / 64) * max_stage_bytes : 0;
    const void *fn = reinterpret_cast<const void *>(&k_wave<NIN, LOCAL, OUT, BITPLANE>);
    // The limit on the kernel's dynamic LDS belongs to the function, not to a launch: it is only
    // ever set to the largest budget, because another host thread may be launching the kernel
    // with any budget at this moment (a limit lowered for the query made such a launch fail).
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)max_dyn);
    if (e != hipSuccess) return e;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(blocks_per_cu, k_wave<NIN, LOCAL, OUT, BITPLANE>, kWG, dyn);
    // The stream-producing kernels need every workgroup of the grid resident at the same time
    // (the scan's waits).  Near the LDS limit the runtime's answer was one workgroup too many on
    // MI355X (5 x 32 688 bytes reported to fit 160 KiB; the fifth was not resident and the waits
    // ran into their bound), so the grid stays within what a 2 KiB allocation unit leaves room
    // for and within four workgroups per compute unit.
    if (e == hipSuccess && OUT == kOutStream) {
        hipFuncAttributes fa;
        e = hipFuncGetAttributes(&fa, fn);
        if (e != hipSuccess) return e;
        const size_t unit = 2048, per_wg = (fa.sharedSizeBytes + dyn + unit - 1) / unit * unit;
        const int by_lds = (int)((160u * 1024u - unit) / per_wg);
        if (*blocks_per_cu > by_lds) *blocks_per_cu = by_lds;
        if (*blocks_per_cu > 4) *blocks_per_cu = 4;
    }
    return e;
}

// both kinds of a kernel: the smaller of the two answers
template <int NIN, int LOCAL, int OUT, int A, int B>
static hipError_t both_resident_blocks(int *blocks_per_cu, uint32_t stage_bytes, uint32_t max_stage_bytes)
{
    int with = 0, without = 0;
    hipError_t e = wave_resident_blocks<NIN, LOCAL, OUT, A>(&with, stage_bytes, max_stage_bytes);
    if (e == hipSuccess) e = wave_resident_blocks<NIN, LOCAL, OUT, B>(&without, stage_bytes, max_stage_bytes);
    *blocks_per_cu = with < without ? with : without;
    return e;
}

hipError_t op_kernel_residency(int op, uint32_t stage_bytes, uint32_t max_stage_bytes, int *blocks_per_cu)
{
    if (stage_bytes > max_stage_bytes) return hipErrorInvalidValue;
    switch (op) {
    case kOpCompress: return wave_resident_blocks<0, kLocalF32, kOutStream, kPlanesNone>(blocks_per_cu, stage_bytes, max_stage_bytes);
    case kOpDecompress: return wave_resident_blocks<1, kLocalNone, kOutF32, kPlanesNone>(blocks_per_cu, stage_bytes, max_stage_bytes);
    case kOpHomSumF32: return both_resident_blocks<1, kLocalF32, kOutStream, kPlanesFew, kPlanesNone>(blocks_per_cu, stage_bytes, max_stage_bytes);
    case kOpHomSumI32: return both_resident_blocks<1, kLocalI32, kOutStream, kPlanesFew, kPlanesNone>(blocks_per_cu, stage_bytes, max_stage_bytes);
    case kOpHomAdd: return both_resident_blocks<2, kLocalNone, kOutStream, kPlanesFew, kPlanesWide>(blocks_per_cu, stage_bytes, max_stage_bytes);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_op(int op, const TileParams &p, uint32_t max_grid, hipStream_t s)
{
    switch (op) {
    case kOpCompress: return launch_wave<0, kLocalF32, kOutStream, kPlanesNone>(p, max_grid, s);
    case kOpDecompress: return launch_wave<1, kLocalNone, kOutF32, kPlanesNone>(p, max_grid, s);
    case kOpHomSumF32:
        return p.sliced ? launch_wave<1, kLocalF32, kOutStream, kPlanesFew>(p, max_grid, s)
                        : launch_wave<1, kLocalF32, kOutStream, kPlanesNone>(p, max_grid, s);
    case kOpHomSumI32:
        return p.sliced ? launch_wave<1, kLocalI32, kOutStream, kPlanesFew>(p, max_grid, s)
                        : launch_wave<1, kLocalI32, kOutStream, kPlanesNone>(p, max_grid, s);
    case kOpHomAdd:
        return p.sliced == 2u ? launch_wave<2, kLocalNone, kOutStream, kPlanesWide>(p, max_grid, s)
                              : launch_wave<2, kLocalNone, kOutStream, kPlanesFew>(p, max_grid, s);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_in_offsets(const InOffsetsArgs &a, int n_streams, uint32_t n_tiles, uint64_t base, uint32_t epoch,
                             uint32_t spin_limit, hipStream_t s)
{
    const uint32_t blocks = (n_tiles + kOfsBlockTiles - 1) / kOfsBlockTiles;
    hipLaunchKernelGGL(k_in_offsets, dim3(blocks, n_streams), dim3(256), 0, s, a, n_tiles, base, epoch, spin_limit);
    return hipGetLastError();
}

hipError_t launch_quant_predict(const float *x, int32_t *out, uint64_t n, float recip, hipStream_t s)
{
    const uint64_t lanes = (n + kEPL - 1) / kEPL;
    const uint32_t grid = (uint32_t)((lanes + kWG - 1) / kWG);
    hipLaunchKernelGGL(k_quant_predict, dim3(grid), dim3(kWG), 0, s, x, out, n, recip);
    return hipGetLastError();
}

hipError_t launch_range(const float *x, uint64_t n, float *partial, uint32_t max_partials,
                        float *out, hipStream_t s)
{
    uint64_t want = (n / 4 + kWG - 1) / kWG;
    if (want < 1) want = 1;
    const uint32_t grid = (uint32_t)(want < max_partials ? want : max_partials);
    hipLaunchKernelGGL(k_range_partial, dim3(grid), dim3(kWG), 0, s, x, n, partial);
    hipLaunchKernelGGL(k_range_final, dim3(1), dim3(kWG), 0, s, partial, grid, out);
    return hipGetLastError();
}

hipError_t launch_fill_u64(uint64_t *p, uint64_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill_u64, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, s, p, n);
    return hipGetLastError();
}

}  // namespace hc
