// Host-visible launch interface of the HomComp kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hc {

enum : int { kLocalNone = 0, kLocalF32 = 1, kLocalI32 = 2 };   // local operand of the combine stage
enum : int { kOutStream = 0, kOutF32 = 1 };                    // what a tile produces
constexpr int kOutChain = 2;                                    // status chain of the output stream

// Geometry shared with the host (must match homcomp_device.hpp).
constexpr uint32_t kHostTileElems = 4096;
constexpr uint32_t kHostTileBlocks = 128;
constexpr uint32_t kHostChunkElems = 32768;

struct TileParams {
    const uint8_t *in[2];     // incoming streams (header + payload)
    uint64_t in_size[2];      // their stated sizes (out-of-bound rule)
    const void *local;        // float32 values or int32 deltas, n elements, 16-byte aligned
    uint8_t *out_cmp;         // outgoing stream
    float *out_f32;           // decompressed values
    uint64_t n;               // elements
    uint64_t hdr_bytes;       // header region = one byte per block of the 32768-padded length
    uint32_t n_tiles;         // padded length / 4096
    float eb;
    float recip;              // fl(0.5f / eb), rounded on the host
    uint64_t *status[3];      // tile status words: incoming 0, incoming 1, outgoing
    uint32_t *ticket;         // tile index dispenser
    uint32_t ticket_base;     // dispenser value when this launch starts
    uint32_t epoch;           // tag that makes this launch's status words distinguishable
    uint64_t *total;          // receives the stream length
    uint64_t *user_total;     // optional second destination for the stream length
};

hipError_t launch_compress(const TileParams &p, hipStream_t s);
hipError_t launch_decompress(const TileParams &p, hipStream_t s);
hipError_t launch_hom_sum_f32(const TileParams &p, hipStream_t s);
hipError_t launch_hom_sum_i32(const TileParams &p, hipStream_t s);
hipError_t launch_hom_add(const TileParams &p, hipStream_t s);
hipError_t launch_quant_predict(const float *x, int32_t *out, uint64_t n, float recip, hipStream_t s);
hipError_t launch_range(const float *x, uint64_t n, float *partial, uint32_t max_partials,
                        float *out, hipStream_t s);
hipError_t launch_fill_u64(uint64_t *p, uint64_t n, hipStream_t s);

}  // namespace hc
