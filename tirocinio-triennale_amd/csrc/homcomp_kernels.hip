// HomComp kernels for gfx950: one tiled, single-pass kernel template covers compress,
// decompress and the three homomorphic sums; two small streaming kernels cover the Lorenzo
// pre-pass and the value range.
//
// A tile is 4096 elements = 128 blocks, processed by one 256-thread workgroup in two
// iterations of 8 elements per lane.  Phases of the tile kernel:
//   1. take a tile index from the ticket counter; start the loads of the local operand
//   2. per incoming stream: header bytes -> block sizes -> tile-local scan -> look-back for the
//      tile's payload offset -> coalesced 16-byte copy of the payload into LDS -> per-lane decode
//   3. combine: delta_out = delta_local + sum of decoded deltas (HomComp/src/homcomp.cu:3611-3616)
//   4a. stream output: rate selection, header bytes, tile-local scan, look-back on the output
//       chain (overlapped with packing into LDS), coalesced 16-byte copy to the stream
//   4b. float output: in-block running sum, dequantise, two float4 stores per lane
#include "homcomp_device.hpp"
#include "homcomp_kernels.hpp"

namespace hc {

// Tile-local exclusive scan of the 128 block sizes, run by wave 0; returns the tile total in
// every lane.
__device__ __forceinline__ uint32_t tile_scan(const uint32_t *s_size, uint32_t *s_ofs, int lane)
{
    const uint32_t s0 = s_size[2 * lane], s1 = s_size[2 * lane + 1];
    const uint32_t incl = wave_incl_scan_u32(s0 + s1, lane);
    const uint32_t excl = incl - (s0 + s1);
    s_ofs[2 * lane] = excl;
    s_ofs[2 * lane + 1] = excl + s0;
    return __shfl(incl, 63, 64);
}

template <int NIN, int LOCAL, int OUT>
__global__ __launch_bounds__(kWG) void k_tile(const TileParams p)
{
    constexpr int kStages = NIN > 1 ? NIN : 1;
    __shared__ __align__(16) uint8_t s_stage[kStages][kStageBytes];
    __shared__ uint32_t s_size[kTileBlocks];
    __shared__ uint32_t s_ofs[kStages][kTileBlocks];
    __shared__ uint8_t s_hdr[kStages][kTileBlocks];
    __shared__ uint64_t s_base[kStages];
    __shared__ uint32_t s_total[kStages];
    __shared__ uint32_t s_tile;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int k = tid & 3;
    const int quad = tid >> 2;

    if (tid == 0) s_tile = atomicAdd(p.ticket, 1u) - p.ticket_base;
    __syncthreads();
    const uint32_t tile = s_tile;
    const uint64_t tile_elem0 = (uint64_t)tile * kTileElems;

    // ---- local operand: issue the loads first so they fly during the stream bookkeeping
    float4 lf[kIter][2];
    int4 li[kIter][2];
    if constexpr (LOCAL != kLocalNone) {
#pragma unroll
        for (int it = 0; it < kIter; ++it) {
            const uint64_t e0 = tile_elem0 + (uint64_t)it * (kWG * kEPL) + (uint64_t)tid * kEPL;
            if (e0 + kEPL <= p.n) {
                if constexpr (LOCAL == kLocalF32) {
                    const float4 *src = reinterpret_cast<const float4 *>((const float *)p.local + e0);
                    lf[it][0] = src[0];
                    lf[it][1] = src[1];
                } else {
                    const int4 *src = reinterpret_cast<const int4 *>((const int32_t *)p.local + e0);
                    li[it][0] = src[0];
                    li[it][1] = src[1];
                }
            } else {
                float tf[8];
                int32_t ti[8];
#pragma unroll
                for (int m = 0; m < 8; ++m) {
                    const bool in = e0 + m < p.n;
                    if constexpr (LOCAL == kLocalF32)
                        tf[m] = in ? ((const float *)p.local)[e0 + m] : 0.0f;
                    else
                        ti[m] = in ? ((const int32_t *)p.local)[e0 + m] : 0;
                }
                if constexpr (LOCAL == kLocalF32) {
                    lf[it][0] = make_float4(tf[0], tf[1], tf[2], tf[3]);
                    lf[it][1] = make_float4(tf[4], tf[5], tf[6], tf[7]);
                } else {
                    li[it][0] = make_int4(ti[0], ti[1], ti[2], ti[3]);
                    li[it][1] = make_int4(ti[4], ti[5], ti[6], ti[7]);
                }
            }
        }
    }

    // ---- incoming streams: sizes, offsets, payload into LDS
    uint32_t in_shift[kStages];
#pragma unroll
    for (int c = 0; c < NIN; ++c) {
        if (tid < kTileBlocks) {
            const uint32_t h = p.in[c][(uint64_t)tile * kTileBlocks + tid];
            s_hdr[c][tid] = (uint8_t)h;
            s_size[tid] = size_from_header(h);
        }
        __syncthreads();
        if (wave == 0) {
            const uint32_t total = tile_scan(s_size, s_ofs[c], lane);
            const uint64_t excl = lookback(p.status[c], tile, p.epoch, total, lane);
            if (lane == 0) {
                s_base[c] = p.hdr_bytes + excl;
                s_total[c] = total;
            }
        }
        __syncthreads();
        const uint64_t start = s_base[c];
        const uint32_t total = s_total[c];
        const uintptr_t g0 = (uintptr_t)p.in[c] + start;
        const uintptr_t ga = g0 & ~(uintptr_t)15;
        const uint32_t shift = (uint32_t)(g0 - ga);
        in_shift[c] = shift;
        const uint32_t nbytes = total ? shift + total : 0u;
        const uint32_t nchunks = (nbytes + 15u) >> 4;
        for (uint32_t i = tid; i < nchunks; i += kWG) {
            if (16u * (i + 1u) <= nbytes) {
                *reinterpret_cast<uint4 *>(&s_stage[c][16u * i]) =
                    *reinterpret_cast<const uint4 *>(ga + 16u * (uintptr_t)i);
            } else {
                for (uint32_t j = 16u * i; j < nbytes; ++j)
                    s_stage[c][j] = *reinterpret_cast<const uint8_t *>(ga + j);
            }
        }
        __syncthreads();
    }

    // ---- per iteration: local deltas + decoded deltas
    int32_t v[kIter][8];
#pragma unroll
    for (int it = 0; it < kIter; ++it) {
        const int blk = it * kBlocksPerIter + quad;
        if constexpr (LOCAL == kLocalF32) {
            // HomComp/src/GSZ.cu:82-149: quantise, then Lorenzo with prevQuant = 0 at block start
            const float x[8] = {lf[it][0].x, lf[it][0].y, lf[it][0].z, lf[it][0].w,
                                lf[it][1].x, lf[it][1].y, lf[it][1].z, lf[it][1].w};
            int32_t q[8];
#pragma unroll
            for (int m = 0; m < 8; ++m) q[m] = quantize(x[m], p.recip);
            uint32_t prev = dpp_u32<kDppRowShr1>((uint32_t)q[7]);
            if (k == 0) prev = 0;
            v[it][0] = (int32_t)((uint32_t)q[0] - prev);
#pragma unroll
            for (int m = 1; m < 8; ++m) v[it][m] = (int32_t)((uint32_t)q[m] - (uint32_t)q[m - 1]);
        } else if constexpr (LOCAL == kLocalI32) {
            // HomComp/src/homcomp.cu:2252-2268: precomputed deltas
            v[it][0] = li[it][0].x; v[it][1] = li[it][0].y; v[it][2] = li[it][0].z; v[it][3] = li[it][0].w;
            v[it][4] = li[it][1].x; v[it][5] = li[it][1].y; v[it][6] = li[it][1].z; v[it][7] = li[it][1].w;
        } else {
#pragma unroll
            for (int m = 0; m < 8; ++m) v[it][m] = 0;
        }
#pragma unroll
        for (int c = 0; c < NIN; ++c) {
            const uint32_t h = s_hdr[c][blk];
            const uint32_t ofs = s_ofs[c][blk];
            // out-of-bound rule of HomComp/src/GSZ.cu:908-911 on the absolute payload offset
            const bool active = size_from_header(h) != 0u && s_base[c] + ofs < p.in_size[c];
            int32_t d[8];
            unpack8(s_stage[c], in_shift[c] + ofs, h, active, k, d);
#pragma unroll
            for (int m = 0; m < 8; ++m) v[it][m] = (int32_t)((uint32_t)v[it][m] + (uint32_t)d[m]);
        }
    }

    if constexpr (OUT == kOutF32) {
        // ---- HomComp/src/GSZ.cu:1426-1468: running sum inside the block, dequantise, store
#pragma unroll
        for (int it = 0; it < kIter; ++it) {
            uint32_t q[8];
            q[0] = (uint32_t)v[it][0];
#pragma unroll
            for (int m = 1; m < 8; ++m) q[m] = q[m - 1] + (uint32_t)v[it][m];
            const uint32_t t0 = dpp_u32<kDppBcast0>(q[7]);
            const uint32_t t1 = dpp_u32<kDppBcast1>(q[7]);
            const uint32_t t2 = dpp_u32<kDppBcast2>(q[7]);
            const uint32_t off = (k > 0 ? t0 : 0u) + (k > 1 ? t1 : 0u) + (k > 2 ? t2 : 0u);
            float y[8];
#pragma unroll
            for (int m = 0; m < 8; ++m) y[m] = dequantize((int32_t)(q[m] + off), p.eb);
            const uint64_t e0 = tile_elem0 + (uint64_t)it * (kWG * kEPL) + (uint64_t)tid * kEPL;
            if (e0 + kEPL <= p.n) {
                float4 *dst = reinterpret_cast<float4 *>(p.out_f32 + e0);
                dst[0] = make_float4(y[0], y[1], y[2], y[3]);
                dst[1] = make_float4(y[4], y[5], y[6], y[7]);
            } else {
#pragma unroll
                for (int m = 0; m < 8; ++m)
                    if (e0 + m < p.n) p.out_f32[e0 + m] = y[m];
            }
        }
    } else {
        // ---- rate selection and header bytes (HomComp/src/GSZ.cu:151-167)
        uint32_t a[kIter][8], sb[kIter], hd[kIter];
        __syncthreads();  // every wave is done reading s_stage / s_size of the input side
#pragma unroll
        for (int it = 0; it < kIter; ++it) {
            uint32_t size;
            analyse8(v[it], k, a[it], sb[it], hd[it], size);
            if (k == 0) {
                const int blk = it * kBlocksPerIter + quad;
                s_size[blk] = size;
                s_hdr[0][blk] = (uint8_t)hd[it];
            }
        }
        __syncthreads();
        if (tid < kTileBlocks) p.out_cmp[(uint64_t)tile * kTileBlocks + tid] = s_hdr[0][tid];
        uint32_t total = 0;
        if (wave == 0) total = tile_scan(s_size, s_ofs[0], lane);
        __syncthreads();
        // ---- wave 0 resolves the global offset while the others pack (HomComp/src/GSZ.cu:170-239)
        if (wave == 0) {
            const uint64_t excl = lookback(p.status[kOutChain], tile, p.epoch, total, lane);
            if (lane == 0) {
                s_base[0] = p.hdr_bytes + excl;
                s_total[0] = total;
            }
        }
#pragma unroll
        for (int it = 0; it < kIter; ++it) {
            const int blk = it * kBlocksPerIter + quad;
            pack8(s_stage[0], s_ofs[0][blk], hd[it], k, a[it], sb[it]);
        }
        __syncthreads();
        // ---- coalesced copy of the tile payload to its place in the stream
        const uint64_t gofs = s_base[0];
        const uint32_t tot = s_total[0];
        uint8_t *g = p.out_cmp + gofs;
        const uint32_t mis = (uint32_t)((uintptr_t)g & 15u);
        uint32_t head = (16u - mis) & 15u;
        if (head > tot) head = tot;
        const uint32_t body = tot - head;
        const uint32_t nch = body >> 4;
        const uint32_t tail = body & 15u;
        if ((uint32_t)tid < head) g[tid] = s_stage[0][tid];
        const uint32_t *sw = reinterpret_cast<const uint32_t *>(s_stage[0]);
        for (uint32_t c = tid; c < nch; c += kWG) {
            const uint32_t s = head + 16u * c;
            const uint32_t w0 = s >> 2, sh = s & 3u;
            const uint32_t x0 = sw[w0], x1 = sw[w0 + 1], x2 = sw[w0 + 2], x3 = sw[w0 + 3], x4 = sw[w0 + 4];
            uint4 o;
            o.x = __builtin_amdgcn_alignbyte(x1, x0, sh);
            o.y = __builtin_amdgcn_alignbyte(x2, x1, sh);
            o.z = __builtin_amdgcn_alignbyte(x3, x2, sh);
            o.w = __builtin_amdgcn_alignbyte(x4, x3, sh);
            *reinterpret_cast<uint4 *>(g + s) = o;
        }
        if ((uint32_t)tid < tail) g[head + 16u * nch + tid] = s_stage[0][head + 16u * nch + tid];
        // ---- true stream length = absolute end offset of the last tile (HomComp/src/GSZ.cu:752-755)
        if (tile == p.n_tiles - 1 && tid == 0) {
            const uint64_t len = gofs + tot;
            *p.total = len;
            if (p.user_total) *p.user_total = len;
        }
    }
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

template <int NIN, int LOCAL, int OUT>
static hipError_t launch_tile(const TileParams &p, hipStream_t s)
{
    hipLaunchKernelGGL((k_tile<NIN, LOCAL, OUT>), dim3(p.n_tiles), dim3(kWG), 0, s, p);
    return hipGetLastError();
}

hipError_t launch_compress(const TileParams &p, hipStream_t s) { return launch_tile<0, kLocalF32, kOutStream>(p, s); }
hipError_t launch_decompress(const TileParams &p, hipStream_t s) { return launch_tile<1, kLocalNone, kOutF32>(p, s); }
hipError_t launch_hom_sum_f32(const TileParams &p, hipStream_t s) { return launch_tile<1, kLocalF32, kOutStream>(p, s); }
hipError_t launch_hom_sum_i32(const TileParams &p, hipStream_t s) { return launch_tile<1, kLocalI32, kOutStream>(p, s); }
hipError_t launch_hom_add(const TileParams &p, hipStream_t s) { return launch_tile<2, kLocalNone, kOutStream>(p, s); }

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
