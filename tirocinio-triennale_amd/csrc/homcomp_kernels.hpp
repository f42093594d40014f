// Host-visible launch interface of the HomComp kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hc {

enum : int { kLocalNone = 0, kLocalF32 = 1, kLocalI32 = 2 };   // local operand of the combine stage
enum : int { kOutStream = 0, kOutF32 = 1 };                    // what a tile produces
enum : int { kOpCompress = 0, kOpDecompress, kOpHomSumF32, kOpHomSumI32, kOpHomAdd, kOpCount };

// Tile geometry, shared by host and device: a tile is 128 blocks of 32 elements; a wave handles
// it in 8 sub-steps of 16 blocks (8 elements per lane, 4 lanes per block).
constexpr uint32_t kHostTileElems = 4096;
constexpr uint32_t kHostTileBlocks = kHostTileElems / 32u;
constexpr uint32_t kHostChunkElems = 32768;
// Plane counts the bit-plane paths of the sums take: stream (+) stream tiles none of whose blocks
// has more than kSlicedMaxF (the kernel for few planes), stream (+) local operand kFewPlanes.
constexpr uint32_t kSlicedMaxF = 6, kFewPlanes = 3;

struct TileParams {
    const uint8_t *in[2];       // incoming streams (header + payload)
    uint64_t in_size[2];        // their stated sizes (out-of-bound rule)
    const uint64_t *in_ofs[2];  // per stream: absolute payload offset of every tile
    const void *local;          // float32 values or int32 deltas, n elements, 16-byte aligned
    uint8_t *out_cmp;           // outgoing stream
    float *out_f32;             // decompressed values
    uint64_t n;                 // elements
    uint64_t hdr_bytes;         // header region = one byte per block of the 32768-padded length
    uint32_t n_tiles;           // padded length / 4096
    float eb;
    float recip;                // fl(0.5f / eb), rounded on the host
    uint64_t *tile_totals;      // output-offset scan: per tile the byte total (data workgroups)
    uint64_t *tile_prefixes;    // and the exclusive prefix (scan server)
    uint32_t epoch;             // tag that makes this launch's status words distinguishable
    uint32_t spin_limit;        // bound on unsuccessful scan probes before *error is raised
    uint32_t *error;            // sticky error flags (bit 0: scan wait gave up)
    uint64_t *total;            // receives the stream length
    uint64_t *user_total;       // optional second destination for the stream length
    uint64_t *tile_ofs_out;     // optional: receives, per tile of the outgoing stream, the absolute byte offset of the tile's
                                // payload (what in_ofs holds for an incoming stream), n_tiles plain words
    uint8_t *spill;             // out_slots slots of kSpillSlotBytes per data wave, for tiles that outgrow their LDS slot
    uint32_t out_slots;         // rounds a packed tile waits in LDS for its stream offset: 2 to 4
    uint32_t sliced;            // the sums' bit-plane paths.  0: no tile takes one (stream (+) local operand then runs the
                                // kernel without); 1: the kernel with the path for tiles of few planes; 2, stream (+)
                                // stream only: the kernel with the path for wide blocks
    uint32_t plain;             // compress: the plain codec, every block in plain mode (0: the outlier codec)
    uint32_t stage_bytes;       // LDS bytes per data wave for those tiles (a multiple of 64); cut into out_slots slots
    uint64_t *host_total;       // optional pinned host word for the host's choice of the next launch's LDS budget: mean payload
                                // bytes per tile (bits 0-31), probe_bytes / 64 (bits 32-47), and how many of 256 tiles had more
                                // payload than probe_bytes (bits 48-63)
    uint32_t probe_bytes;       // a slot size the host would like to know that share for (0: none)
};

// Bytes per slot of the spill area (TileParams::spill): a whole worst-case tile.
constexpr uint32_t kSpillSlotBytes = kHostTileBlocks * 128u + 128u;
// Resident workgroups per compute unit of the kernel behind an operation with `stage_bytes` of
// LDS stage per data wave (sizes the persistent grid).  `max_stage_bytes`: the largest stage any
// launch of the operation uses; the kernel's limit on dynamic LDS is set to that.
hipError_t op_kernel_residency(int op, uint32_t stage_bytes, uint32_t max_stage_bytes, int *blocks_per_cu);
hipError_t launch_op(int op, const TileParams &p, uint32_t max_grid, hipStream_t s);
// Tile payload offsets of one or two incoming streams (of the same length) from their header
// bytes, in one launch.
struct InOffsetsArgs {
    const uint8_t *hdr[2];      // the streams' header bytes
    uint64_t *block_words[2];   // per stream and block of 256 tiles: a word tagged with the launch's epoch, n_tiles / 256 + 1 of them
    uint64_t *ofs[2];           // result: absolute payload offset of every tile
    uint64_t *few_report[2];    // optional (host-visible) word per stream: n_tiles << 32 | tiles none of whose blocks has more than few_limit planes
    uint32_t few_limit;
    uint32_t *error;            // sticky error flags (bit 0: a bounded wait gave up)
};
// `epoch`: as TileParams::epoch, any value the block words have not seen since they were last cleared.
hipError_t launch_in_offsets(const InOffsetsArgs &a, int n_streams, uint32_t n_tiles, uint64_t base, uint32_t epoch,
                             uint32_t spin_limit, hipStream_t s);
hipError_t launch_quant_predict(const float *x, int32_t *out, uint64_t n, float recip, hipStream_t s);
hipError_t launch_range(const float *x, uint64_t n, float *partial, uint32_t max_partials,
                        float *out, hipStream_t s);
hipError_t launch_fill_u64(uint64_t *p, uint64_t n, hipStream_t s);

}  // namespace hc
