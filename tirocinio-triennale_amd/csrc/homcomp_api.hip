// C ABI of libhomcomp_amd.so: argument checking, workspace management and launch geometry.
// The interface is documented in include/homcomp.h.
#include "../../include/homcomp.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "homcomp_kernels.hpp"

namespace {

thread_local int g_last_hip_error = 0;

// Epochs 1 .. kMaxEpoch go to eager launches in turn.  The epochs above them are kept for launches
// recorded into a graph, which are replayed with the epoch they were captured with: the first
// launch a capture records on a workspace is preceded by kernels that clear the workspace's tagged
// words, the launches of that capture take the graph epochs in turn (the clears are recorded again
// when they run out), so a replay starts from cleared words and no call inside it meets the words
// of another, and an eager call is never handed an epoch whose words a replay left behind.
constexpr uint32_t kGraphEpochLast = (1u << 22) - 1;
constexpr uint32_t kGraphEpochFirst = kGraphEpochLast - 4095;
constexpr uint32_t kMaxEpoch = kGraphEpochFirst - 1;
// Unsuccessful scan re-reads before a wave gives up (each costs a memory round trip, so this is
// some tens of milliseconds): long enough for any delay of a resident workgroup, short enough
// that a launch which could not become resident ends with an error instead of stalling for minutes.
constexpr uint32_t kSpinLimit = 1u << 16;
constexpr uint32_t kRangePartials = 2048;

inline bool hip_ok(hipError_t e)
{
    if (e == hipSuccess) return true;
    g_last_hip_error = (int)e;
    return false;
}

inline size_t chunks_of(size_t n) { return (n + hc::kHostChunkElems - 1) / hc::kHostChunkElems; }
inline size_t padded_len(size_t n) { return chunks_of(n) * hc::kHostChunkElems; }
inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }
inline bool eb_ok(float eb) { return std::isfinite(eb) && eb > 0.0f; }

}  // namespace

struct homcomp_workspace {
    int device;
    size_t max_n;
    uint32_t max_tiles;
    void *d_block;            // one allocation holding everything below
    uint64_t *d_tile_totals;   // [max_tiles]  output-offset scan: tile totals
    uint64_t *d_tile_prefixes; // [max_tiles]  output-offset scan: tile prefixes (adjacent to the totals)
    uint64_t *d_in_ofs[2];    // [max_tiles+1] tile payload offsets of the incoming streams
    uint64_t *d_in_blocks[2]; // [max_tiles/256 + 1]  words of the offsets pre-pass, per stream: totals of blocks of 256 tiles, tagged with the epoch
    uint64_t *d_total;        // stream length of the last stream-producing call
    uint32_t *d_error;        // sticky error flags, next to d_total
    float *d_partial;         // min/max partials
    uint64_t *h_total;        // pinned host words (length, error) for the blocking read-back
    uint32_t epoch;           // last epoch handed out (1..kMaxEpoch)
    unsigned long long capture_id;   // the stream capture whose launches take graph epochs at the moment (0: none yet)
    uint32_t graph_epoch;     // the next of them
    // Tile offsets handed over for the next call (homcomp_workspace_tile_offsets), cleared by it
    const uint64_t *next_in_ofs[2];
    uint64_t *next_out_ofs;
    uint32_t max_grid[hc::kOpCount][3];  // persistent grid of each operation's kernel, per LDS budget (small, medium, large)
    uint32_t full_grid[hc::kOpCount][3]; // the same at 100 percent (HOMCOMP_OPT_GRID_PERCENT scales it)
    uint64_t *h_mean_tile;    // pinned host words, one per operation, left by its last finished call: mean payload bytes per
                              // tile and the share of tiles beyond a slot size asked about (TileParams::host_total)
    uint64_t *h_few;          // pinned host words, left by the offsets pre-pass of the last sum that got that far, n_tiles << 32 |
                              // tiles that can take the bit-plane path for few planes: [0] stream (+) local operand (none of
                              // the tile's blocks has more than three planes), [1] and [2] the two streams of stream (+)
                              // stream (six)
    uint32_t spin_limit;      // bound on unsuccessful scan re-reads (HOMCOMP_SPIN_LIMIT overrides)
    uint32_t out_slots;       // deferral depth of packed tiles (2..4); the device's spill area has this many slots per data wave
    bool holds_spill;         // counted among the users of the device's spill area
    uint32_t sliced;          // bit-plane paths of the sums: HOMCOMP_SLICED=0 switches them off; 1: chosen per call; 2: the
                              // kernels with the path for few planes whatever the streams look like; 3: stream (+) stream
                              // runs the kernel for wide blocks whatever the streams look like
    int stage_class;          // -1: chosen per call; 0 / 1 / 2: HOMCOMP_STAGE=small / medium / large forces one LDS budget
    int last_kind, last_budget;   // what the last stream-producing call was launched with (homcomp_workspace_last_launch)
};

namespace {

// The tile offsets handed over for a call are that call's only, however it ends.
struct HandOver {
    homcomp_workspace *ws;
    explicit HandOver(homcomp_workspace *w) : ws(w) {}
    ~HandOver()
    {
        if (!ws) return;
        ws->next_out_ofs = nullptr;
        ws->next_in_ofs[0] = ws->next_in_ofs[1] = nullptr;
    }
};

int check_ws(const homcomp_workspace *ws, size_t n)
{
    if (!ws) return HOMCOMP_ERR_INVALID_ARG;
    if (n > ws->max_n) return HOMCOMP_ERR_TOO_LARGE;
    int dev = -1;
    if (!hip_ok(hipGetDevice(&dev))) return HOMCOMP_ERR_HIP;
    if (dev != ws->device) return HOMCOMP_ERR_INVALID_ARG;
    return HOMCOMP_OK;
}

// `id`: the capture's identifier (unique per capture), 0 outside a capture.
bool stream_is_capturing(hipStream_t s, unsigned long long *id = nullptr)
{
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    unsigned long long cid = 0;
    if (hipStreamGetCaptureInfo(s, &cap, &cid) != hipSuccess) {
        (void)hipGetLastError();
        cap = hipStreamCaptureStatusInvalidated;   // treated like a capture: nothing is executed eagerly on such a stream
        cid = ~0ull;
    }
    if (id) *id = cap != hipStreamCaptureStatusNone ? (cid ? cid : ~0ull) : 0;
    return cap != hipStreamCaptureStatusNone;
}

// One fill over everything between the first scan word and the last pre-pass word (the tile offsets
// of the incoming streams lie between them; they are rewritten by every call that uses them).
int clear_tagged_words(homcomp_workspace *ws, hipStream_t s)
{
    const uint64_t blocks = (uint64_t)ws->max_tiles / 256 + 1;
    const uint64_t words = (uint64_t)((ws->d_in_blocks[1] + blocks) - ws->d_tile_totals);
    return hip_ok(hc::launch_fill_u64(ws->d_tile_totals, words, s)) ? HOMCOMP_OK : HOMCOMP_ERR_HIP;
}

// Fresh epoch for one launch; clears the scan words (the two arrays are adjacent) and the block
// words of the offsets pre-pass when the 22-bit tag wraps.  A launch that is being recorded into a
// graph takes no epoch of the eager sequence (clears issued for it are recorded, not executed, so
// the eager counter must not start over on their account): it takes the next graph epoch, and the
// first launch of a capture on this workspace records the clears ahead of itself.  (With one epoch
// for all recorded launches every one of them had to clear its words first: three small kernels
// per call, which made a recorded ring schedule slower than the eager one.)
int next_epoch(homcomp_workspace *ws, hipStream_t s, uint32_t *epoch)
{
    unsigned long long capture = 0;
    if (stream_is_capturing(s, &capture)) {
        if (capture != ws->capture_id || ws->graph_epoch > kGraphEpochLast) {
            const int rc = clear_tagged_words(ws, s);
            if (rc) return rc;
            ws->capture_id = capture;
            ws->graph_epoch = kGraphEpochFirst;
        }
        *epoch = ws->graph_epoch++;
        return HOMCOMP_OK;
    }
    if (ws->epoch >= kMaxEpoch) {
        const int rc = clear_tagged_words(ws, s);
        if (rc) return rc;
        ws->epoch = 0;
    }
    *epoch = ++ws->epoch;
    return HOMCOMP_OK;
}

int fill_params(homcomp_workspace *ws, size_t n, hipStream_t s, hc::TileParams *p)
{
    std::memset(p, 0, sizeof *p);
    p->n = n;
    p->hdr_bytes = homcomp_header_bytes(n);
    p->n_tiles = (uint32_t)(padded_len(n) / hc::kHostTileElems);
    p->tile_totals = ws->d_tile_totals;
    p->tile_prefixes = ws->d_tile_prefixes;
    p->spin_limit = ws->spin_limit;
    p->error = ws->d_error;
    p->total = ws->d_total;
    // tile offsets handed over for this call (one call only)
    p->tile_ofs_out = ws->next_out_ofs;
    p->in_ofs[0] = ws->next_in_ofs[0];
    p->in_ofs[1] = ws->next_in_ofs[1];
    return next_epoch(ws, s, &p->epoch);
}

// Offsets pre-pass of the incoming streams (header bytes -> payload offset of every tile): one
// launch for all of them, under the epoch of the call's tile kernel.  Streams whose offsets the
// caller handed over (homcomp_workspace_tile_offsets) need none; the launch is left out when that
// holds for all of them.
int in_offsets(homcomp_workspace *ws, int n_streams, hc::TileParams *p, hipStream_t s)
{
    const uint64_t *given[2] = {p->in_ofs[0], p->in_ofs[1]};
    bool all_given = true;
    for (int c = 0; c < n_streams; ++c) all_given = all_given && given[c] != nullptr;
    if (all_given) return HOMCOMP_OK;
    hc::InOffsetsArgs a;
    std::memset(&a, 0, sizeof a);
    a.error = ws->d_error;
    const uint32_t epoch = p->epoch;
    for (int c = 0; c < n_streams; ++c) {
        p->in_ofs[c] = given[c] ? given[c] : ws->d_in_ofs[c];
        a.hdr[c] = p->in[c];
        a.block_words[c] = ws->d_in_blocks[c];
        a.ofs[c] = ws->d_in_ofs[c];
    }
    // the sums: how many tiles could take the bit-plane path for few planes (see run_tile_op)
    if (p->local) {
        a.few_report[0] = ws->h_few;
        a.few_limit = hc::kFewPlanes;
    } else if (n_streams == 2) {
        a.few_report[0] = ws->h_few + 1;
        a.few_report[1] = ws->h_few + 2;
        a.few_limit = hc::kSlicedMaxF;
    }
    return hip_ok(hc::launch_in_offsets(a, n_streams, p->n_tiles, p->hdr_bytes, epoch, ws->spin_limit, s)) ? HOMCOMP_OK
                                                                                                            : HOMCOMP_ERR_HIP;
}

// LDS stage per data wave (two deferred tiles by default), in three budgets that let 4, 3 and 2
// workgroups share a compute unit (with the LDS the kernels hold besides: 0.6 KiB for compress,
// 12.5 KiB with one incoming stream, 19.4 KiB with two).  The slots hold tiles of streams
// compressed about 4.6x / 2.9x / 2x or better for compress, 6x / 3.7x / 2x for the sums with one
// incoming stream and 9x / 4.5x / 2.5x with two.  A tile beyond its slot still works (it goes
// through the spill area), so the choice below is a performance heuristic, never a correctness
// matter.  (With the full 8 KiB slots only one workgroup of the two-stream kernel
// fits a compute unit, which is slower than spilling: its largest slots are 7.3 KiB.)
constexpr int kStageClasses = 3;
constexpr uint64_t kBitplaneTileBytes = hc::kHostTileBlocks * 20u;
constexpr uint64_t kWideTileBytes = hc::kHostTileBlocks * 30u;   // blocks of six planes: 4 + 4 * 6 bytes and an outlier byte or two
constexpr uint32_t kStage[kStageClasses][hc::kOpCount] = {
    {2 * (4096 + 64), 0, 2 * (3072 + 64), 2 * (3072 + 64), 2 * (2048 + 64)},
    {2 * (6464 + 64), 0, 2 * (4992 + 64), 2 * (4992 + 64), 2 * (4112 + 64)},
    {2 * (8192 + 64), 0, 2 * (8192 + 64), 2 * (8192 + 64), 2 * (7440 + 64)}};

// Per-device state shared by all workspaces of the process.
//
// Launch chain.  The stream-producing kernels of this process never overlap on a device.  Each of
// them needs its whole grid resident (the scan's waits), and two such grids from different
// streams can each end up half resident, every wave waiting for workgroups that cannot start:
// both calls would run into the bound of their waits.  So a launch on another stream than the
// device's previous one first waits (on the GPU, not on the host) for an event recorded on that
// stream.  A stream under capture is left alone: its graph orders the launches it contains.
//
// Spill area.  A tile that outgrows its LDS slot waits for its stream offset in global memory:
// one slot of a worst-case tile per deferred tile and data wave.  Because the kernels that use it
// never overlap, one area per device serves every workspace; it is allocated with the first
// workspace, grows to the largest grid x deferral depth asked for, and is freed with the last
// workspace.  An area that has been outgrown stays allocated until then (a recorded graph may
// still name it).
struct DeviceState {
    std::mutex mu;
    hipEvent_t done = nullptr;
    hipStream_t last = nullptr;
    bool any = false;
    uint8_t *spill = nullptr;
    size_t spill_bytes = 0;
    int spill_users = 0;
    std::vector<void *> retired;
    // persistent grid of each operation's kernel per LDS budget, at 100 percent; worked out once
    bool grids_ready = false;
    uint32_t full_grid[hc::kOpCount][kStageClasses];
};
constexpr int kMaxDevices = 64;
DeviceState g_dev[kMaxDevices];

// Resident grid of every operation and LDS budget on `device` (the current device), computed once
// per process: the occupancy queries set a limit that belongs to the kernel function, which must
// not change while other host threads launch.
int device_grids(int device, const uint32_t (**grids)[kStageClasses])
{
    DeviceState &d = g_dev[device];
    std::lock_guard<std::mutex> lock(d.mu);
    *grids = d.full_grid;
    if (d.grids_ready) return HOMCOMP_OK;
    hipDeviceProp_t prop;
    if (!hip_ok(hipGetDeviceProperties(&prop, device))) return HOMCOMP_ERR_HIP;
    // one compute unit's worth of workgroups is left free: the persistent grid must be fully
    // resident, and an estimate that is off by a single workgroup would stall the launch
    const int cus = prop.multiProcessorCount > 1 ? prop.multiProcessorCount - 1 : 1;
    for (int op = 0; op < hc::kOpCount; ++op) {
        for (int cls = 0; cls < kStageClasses; ++cls) {
            int per_cu = 0;
            const uint32_t stage = op == hc::kOpDecompress ? 0u : kStage[cls][op];
            const uint32_t largest = op == hc::kOpDecompress ? 0u : kStage[kStageClasses - 1][op];
            if (!hip_ok(hc::op_kernel_residency(op, stage, largest, &per_cu))) return HOMCOMP_ERR_HIP;
            if (per_cu < 1) per_cu = 1;
            d.full_grid[op][cls] = (uint32_t)per_cu * (uint32_t)cus;
        }
    }
    d.grids_ready = true;
    return HOMCOMP_OK;
}

int spill_acquire(homcomp_workspace *ws, size_t bytes)
{
    DeviceState &d = g_dev[ws->device];
    std::lock_guard<std::mutex> lock(d.mu);
    if (bytes > d.spill_bytes) {
        void *area = nullptr;
        if (!hip_ok(hipMalloc(&area, bytes))) return HOMCOMP_ERR_HIP;
        if (d.spill) d.retired.push_back(d.spill);
        d.spill = (uint8_t *)area;
        d.spill_bytes = bytes;
    }
    ++d.spill_users;
    ws->holds_spill = true;
    return HOMCOMP_OK;
}

// after the device has been synchronised
int spill_release(homcomp_workspace *ws)
{
    if (!ws->holds_spill) return HOMCOMP_OK;
    DeviceState &d = g_dev[ws->device];
    std::lock_guard<std::mutex> lock(d.mu);
    ws->holds_spill = false;
    if (--d.spill_users > 0) return HOMCOMP_OK;
    int rc = HOMCOMP_OK;
    if (d.spill && !hip_ok(hipFree(d.spill))) rc = HOMCOMP_ERR_HIP;
    for (void *area : d.retired)
        if (!hip_ok(hipFree(area))) rc = HOMCOMP_ERR_HIP;
    d.retired.clear();
    d.spill = nullptr;
    d.spill_bytes = 0;
    return rc;
}

// p.spill == nullptr: the device's spill area is used.
int chained_launch(int device, int op, hc::TileParams p, uint32_t max_grid, hipStream_t s)
{
    const bool capturing = stream_is_capturing(s);
    DeviceState &c = g_dev[device];
    std::lock_guard<std::mutex> lock(c.mu);
    if (!p.spill) p.spill = c.spill;
    // a stream under capture is left alone: its graph orders the launches it contains
    if (capturing) return hip_ok(hc::launch_op(op, p, max_grid, s)) ? HOMCOMP_OK : HOMCOMP_ERR_HIP;
    if (c.any && c.last != s) {
        // The event is recorded only now, on the stream of the previous launch (a call that stays
        // on one stream pays nothing): it covers that launch and whatever followed it there.
        if (!c.done && !hip_ok(hipEventCreateWithFlags(&c.done, hipEventDisableTiming))) return HOMCOMP_ERR_HIP;
        if (hipEventRecord(c.done, c.last) == hipSuccess) {
            if (!hip_ok(hipStreamWaitEvent(s, c.done, 0))) return HOMCOMP_ERR_HIP;
        } else {
            // the previous stream is gone: wait for the device instead
            (void)hipGetLastError();
            if (!hip_ok(hipDeviceSynchronize())) return HOMCOMP_ERR_HIP;
        }
    }
    if (!hip_ok(hc::launch_op(op, p, max_grid, s))) return HOMCOMP_ERR_HIP;
    c.last = s;
    c.any = true;
    return HOMCOMP_OK;
}

// LDS budget of a stream-producing call from the payload bytes per tile it is expected to
// produce (0: unknown, the large budget).
int choose_stage_class(int op, uint64_t expected_tile_bytes, uint32_t out_slots)
{
    if (expected_tile_bytes == 0) return kStageClasses - 1;
    // the smallest budget whose slots hold the expected tile with an eighth to spare
    int holds = -1;
    for (int c = kStageClasses - 1; c >= 0; --c) {
        const uint64_t slot_cap = kStage[c][op] / out_slots - 64u;
        if (expected_tile_bytes + expected_tile_bytes / 8 + 64u <= slot_cap) holds = c;
    }
    // The sums are bound by instruction issue and gain more from a third and fourth
    // workgroup per compute unit than they lose by spilling, so they never take the large
    // budget by themselves; compress is bound by memory and avoids the spill traffic
    // where it can, and where no budget holds the tiles the medium one is its best
    // balance between waves and spilled bytes.  (Measured on MI355X at 1 GiB, compression
    // ratios 1.6 to 4.4.)
    if (op == hc::kOpCompress) return holds < 0 ? 1 : holds;
    return holds < 0 || holds == kStageClasses - 1 ? 0 : holds;
}

// Grid of the decoder.  The decoder is bound by its stores (2 KiB per wave and sub-step, each
// wave waiting for its own), and with every wave slot of the device taken they queue up behind
// each other: measured on MI355X at 64M and 256M elements over three data families and five
// bounds, streams of up to about 2.5 KB per tile (compressed 6.5 times and better, payload in most
// blocks) decode 9-13 % faster on 44 % of the resident grid (five waves per compute unit in two,
// 199 against 229 us for 1 GiB), streams of 2.5-4.2 KB per tile 8 % faster on half of it; longer
// tiles need every wave for their loads, and streams of almost empty tiles (below 300 bytes) do
// not care.  Calls of less than two rounds of the full grid keep it.  A heuristic for speed only:
// any grid gives the same values.
uint32_t decoder_grid(uint32_t full, uint32_t n_tiles, uint64_t tile_bytes)
{
    if ((uint64_t)n_tiles < 2ull * 4u * full) return full;
    uint32_t percent = 100;
    if (tile_bytes >= 300u && tile_bytes <= 2560u) percent = 44;
    else if (tile_bytes > 2560u && tile_bytes <= 4200u) percent = 50;
    const uint32_t g = (uint32_t)((uint64_t)full * percent / 100u);
    return g ? g : 1u;
}

// expected_tile_bytes: payload bytes per tile the call is expected to produce (the decoder: to read), 0 if unknown
int run_tile_op(homcomp_workspace *ws, int op, hc::TileParams &p, uint64_t expected_tile_bytes, hipStream_t s)
{
    p.out_slots = ws->out_slots;
    p.sliced = ws->sliced == 3u ? 1u : ws->sliced;
    if (op == hc::kOpDecompress) {
        p.stage_bytes = 0u;
        return hip_ok(hc::launch_op(op, p, decoder_grid(ws->max_grid[op][0], p.n_tiles, expected_tile_bytes), s)) ? HOMCOMP_OK
                                                                                                                    : HOMCOMP_ERR_HIP;
    }
    // Nothing known about the incoming tiles (the size was stated as the buffer's capacity): the
    // mean tile the operation's last finished call on this workspace produced stands in for them
    // (a ring step's partial sums resemble those of the step before).
    const uint64_t seen = *(volatile const uint64_t *)&ws->h_mean_tile[op];   // 0 until a call has finished
    if (expected_tile_bytes == 0) expected_tile_bytes = seen & 0xffffffffu;
    // stream (+) local operand: the kernel with the bit-plane path where most incoming tiles can
    // take it, else the one without.  The offsets pre-pass counts the tiles of few planes and
    // leaves the count in host-visible memory; it arrives too late for the launch it belongs to,
    // so the choice follows the previous call of the same length (a ring step sums chunk after
    // chunk of similar data), and the incoming stream's size where there is none (blocks of at
    // most three planes are at most 4 + 4 * 3 + 4 bytes).  Either kernel produces the same bytes.
    if ((op == hc::kOpHomSumF32 || op == hc::kOpHomSumI32) && p.sliced == 1u) {
        const uint64_t seen = *(volatile const uint64_t *)ws->h_few;
        if (seen >> 32 == p.n_tiles)
            p.sliced = (seen & 0xffffffffu) * 4u >= (uint64_t)p.n_tiles * 3u;
        else
            p.sliced = expected_tile_bytes <= kBitplaneTileBytes;
    }
    // stream (+) stream: the kernel for few planes (blocks of up to six go down its bit-plane
    // path) or the one for wide blocks (up to 22): the first where most tiles can take its path
    if (op == hc::kOpHomAdd) {
        if (ws->sliced == 1u) {
            // as above: by the previous call of the same length where there was one
            const uint64_t seen_a = *(volatile const uint64_t *)(ws->h_few + 1), seen_b = *(volatile const uint64_t *)(ws->h_few + 2);
            if (seen_a >> 32 == p.n_tiles && seen_b >> 32 == p.n_tiles) {
                const uint64_t few = (seen_a & 0xffffffffu) < (seen_b & 0xffffffffu) ? (seen_a & 0xffffffffu) : (seen_b & 0xffffffffu);
                p.sliced = few * 4u >= (uint64_t)p.n_tiles * 3u ? 1u : 2u;
            } else {
                p.sliced = expected_tile_bytes <= kWideTileBytes ? 1u : 2u;
            }
        } else if (ws->sliced != 0u)
            p.sliced = ws->sliced == 3u ? 2u : 1u;
    }
    int cls = choose_stage_class(op, expected_tile_bytes, ws->out_slots);
    // compress: the budget above holds the mean tile with an eighth to spare.  Tiles that vary
    // (spikes in the data) do not need that: with half of them a little beyond the slots of the
    // next smaller budget, that budget's extra workgroup per compute unit still wins (0.290
    // against 0.314 ms on 1 GiB whose tiles average 6.4 KB, in 6.4 KB slots); with all of them
    // beyond, it loses (0.394 against 0.308 ms).  So the kernel counts the tiles beyond that
    // slot size, and the next call takes the smaller budget while they stay below 55 %.
    if (op == hc::kOpCompress && cls > 0) {
        const uint32_t smaller = kStage[cls - 1][op] / ws->out_slots - 64u;
        p.probe_bytes = smaller & ~63u;
        if (((seen >> 32) & 0xffffu) * 64u == p.probe_bytes && (seen >> 48) <= 140u) cls -= 1;
    }
    if (ws->stage_class >= 0) cls = ws->stage_class;
    p.host_total = &ws->h_mean_tile[op];
    p.stage_bytes = kStage[cls][op];
    ws->last_budget = cls;
    if (op == hc::kOpCompress || p.sliced == 0u)
        ws->last_kind = HOMCOMP_KERNEL_GENERAL;
    else
        ws->last_kind = op == hc::kOpHomAdd && p.sliced == 2u ? HOMCOMP_KERNEL_WIDE_PLANES : HOMCOMP_KERNEL_FEW_PLANES;
    return chained_launch(ws->device, op, p, ws->max_grid[op][cls], s);
}

// payload bytes per tile of an incoming stream; 0 (unknown) when the stated size is no length but
// a capacity
uint64_t tile_bytes_of(const hc::TileParams &p, size_t stream_size)
{
    if (stream_size >= homcomp_max_stream_bytes(p.n)) return 0u;
    return stream_size > p.hdr_bytes ? (stream_size - p.hdr_bytes) / p.n_tiles : 1u;
}

// n == 0: the stream is empty; only the length words are written.
int empty_stream(homcomp_workspace *ws, uint64_t *d_stream_len, hipStream_t s)
{
    if (!hip_ok(hc::launch_fill_u64(ws->d_total, 1, s))) return HOMCOMP_ERR_HIP;
    if (d_stream_len && !hip_ok(hc::launch_fill_u64(d_stream_len, 1, s))) return HOMCOMP_ERR_HIP;
    return HOMCOMP_OK;
}

// ---------------------------------------------------------------- allocation-free entry point
//
// homcomp_hom_sum_f32_static keeps everything a workspace would hold in one device array of the
// library: scan words, the incoming stream's tile offsets and the scratch of their pre-pass, and
// a spill area for a grid of kStaticDataGroups data workgroups.  Layout (byte offsets):
constexpr size_t kStaticMaxElems = HOMCOMP_STATIC_MAX_ELEMENTS;
constexpr uint32_t kStaticMaxTiles = (uint32_t)(kStaticMaxElems / hc::kHostTileElems);
constexpr uint32_t kStaticDataGroups = 224;   // data workgroups of four waves
constexpr uint32_t kStaticSlots = 2;          // deferral depth
constexpr size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
constexpr size_t kStaticOfsScan = 0;                                                                   // 2 x tiles words
constexpr size_t kStaticOfsIn = kStaticOfsScan + align256(2 * (size_t)kStaticMaxTiles * 8);            // tiles offsets
constexpr size_t kStaticOfsBlocks = kStaticOfsIn + align256((size_t)kStaticMaxTiles * 8);              // words of blocks of 256 tiles
constexpr size_t kStaticOfsSpill = kStaticOfsBlocks + align256(((size_t)kStaticMaxTiles / 256 + 1) * 8);
constexpr size_t kStaticBytes =
    kStaticOfsSpill + (size_t)kStaticDataGroups * 4 * kStaticSlots * hc::kSpillSlotBytes;   // about 28.3 MiB

}  // namespace

// Every GPU the library runs on holds its own copy of this array, at its own address, until the
// process ends.  In host code the name is only a handle for hipGetSymbolAddress: the address a
// kernel can use is looked up once per device (static_state below) and passed as an argument.
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

namespace {

struct StaticState {
    std::mutex mu;
    bool ready = false;
    uint8_t *base = nullptr;                 // device address of `scratch` on this device
    uint32_t grid[kStageClasses] = {0, 0, 0};  // persistent grid of hom_sum_f32 per LDS budget, scan server included
};
StaticState g_static[kMaxDevices];

// First call on a device: the address of the device's copy of `scratch`, the resident grid, and
// the event of the launch chain, so that later calls create nothing.
int static_setup(int device, StaticState **out)
{
    StaticState &st = g_static[device];
    std::lock_guard<std::mutex> lock(st.mu);
    *out = &st;
    if (st.ready) return HOMCOMP_OK;
    void *ptr = nullptr;
    if (!hip_ok(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))) || !ptr) return HOMCOMP_ERR_HIP;
    const uint32_t (*grids)[kStageClasses] = nullptr;
    if (device_grids(device, &grids) != HOMCOMP_OK) return HOMCOMP_ERR_HIP;
    for (int cls = 0; cls < kStageClasses; ++cls) {
        uint32_t g = grids[hc::kOpHomSumF32][cls];
        if (g > kStaticDataGroups + 1) g = kStaticDataGroups + 1;   // the spill area holds this many groups
        if (g < 2) g = 2;
        st.grid[cls] = g;
    }
    {
        DeviceState &c = g_dev[device];
        std::lock_guard<std::mutex> chain(c.mu);
        if (!c.done && !hip_ok(hipEventCreateWithFlags(&c.done, hipEventDisableTiming))) return HOMCOMP_ERR_HIP;
    }
    st.base = (uint8_t *)ptr;
    st.ready = true;
    return HOMCOMP_OK;
}

}  // namespace

extern "C" {

const char *homcomp_status_string(int status)
{
    switch (status) {
    case HOMCOMP_OK: return "ok";
    case HOMCOMP_ERR_INVALID_ARG: return "invalid argument";
    case HOMCOMP_ERR_ALIGNMENT: return "float/int32 buffer not 16-byte aligned";
    case HOMCOMP_ERR_TOO_LARGE: return "nbEle exceeds the workspace capacity";
    case HOMCOMP_ERR_HIP: return "HIP runtime error";
    case HOMCOMP_ERR_NO_DEVICE: return "no usable GPU";
    case HOMCOMP_ERR_SCAN_TIMEOUT: return "offset scan gave up waiting (grid not fully resident?); output invalid";
    default: return "unknown status";
    }
}

int homcomp_last_hip_error(void) { return g_last_hip_error; }

size_t homcomp_header_bytes(size_t nbEle) { return chunks_of(nbEle) * (hc::kHostChunkElems / 32); }

size_t homcomp_max_stream_bytes(size_t nbEle)
{
    const size_t blocks = homcomp_header_bytes(nbEle);
    return blocks + blocks * 128u;
}

size_t homcomp_ref_cmpsize(size_t stream_len, size_t nbEle) { return stream_len + homcomp_header_bytes(nbEle); }

float homcomp_rel_to_abs(float rel, float vmin, float vmax)
{
    volatile float range = vmax - vmin;
    volatile float eb = rel * range;
    return eb;
}

int homcomp_workspace_create(homcomp_workspace **out, size_t max_nbEle)
{
    if (!out) return HOMCOMP_ERR_INVALID_ARG;
    *out = nullptr;
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) {
        (void)hipGetLastError();
        return HOMCOMP_ERR_NO_DEVICE;
    }
    const size_t tiles = padded_len(max_nbEle) / hc::kHostTileElems;
    // the kernels count tiles in 32 bits, with room for a few rounds of the grid beyond the last tile
    if (tiles >= (1ull << 31) - (1ull << 16)) return HOMCOMP_ERR_TOO_LARGE;
    homcomp_workspace *ws = new (std::nothrow) homcomp_workspace();
    if (!ws) return HOMCOMP_ERR_INVALID_ARG;
    std::memset(ws, 0, sizeof *ws);
    ws->max_n = max_nbEle;
    ws->max_tiles = (uint32_t)(tiles ? tiles : 1);
    if (!hip_ok(hipGetDevice(&ws->device))) {
        delete ws;
        return HOMCOMP_ERR_HIP;
    }
    if (ws->device < 0 || ws->device >= kMaxDevices) {
        delete ws;
        return HOMCOMP_ERR_NO_DEVICE;
    }
    const size_t t = ws->max_tiles;
    size_t off = 0;
    auto take = [&off](size_t bytes) { size_t o = off; off = (off + bytes + 255) & ~(size_t)255; return o; };
    const size_t o_status = take(2 * t * sizeof(uint64_t));
    const size_t o_in0 = take(t * sizeof(uint64_t));
    const size_t o_in1 = take(t * sizeof(uint64_t));
    const size_t o_blk0 = take((t / 256 + 1) * sizeof(uint64_t));
    const size_t o_blk1 = take((t / 256 + 1) * sizeof(uint64_t));
    const size_t o_total = take(64);
    const size_t o_partial = take(kRangePartials * 2 * sizeof(float));
    const size_t bytes = off;
    const uint32_t (*grids)[kStageClasses] = nullptr;
    bool ok = device_grids(ws->device, &grids) == HOMCOMP_OK;
    uint32_t widest = 0;
    for (int op = 0; ok && op < hc::kOpCount; ++op) {
        for (int cls = 0; cls < kStageClasses; ++cls) {
            const uint32_t g = grids[op][cls];
            ws->full_grid[op][cls] = g;
            if (op != hc::kOpDecompress && g > widest) widest = g;
        }
    }
    ws->out_slots = 2;
    if (const char *e = std::getenv("HOMCOMP_SLOTS")) {
        const long v = std::strtol(e, nullptr, 10);
        if (v >= 2 && v <= 4) ws->out_slots = (uint32_t)v;
    }
    if (ok) {
        // HOMCOMP_GRID_PERCENT (1..100): the initial value of HOMCOMP_OPT_GRID_PERCENT
        long pct = 100;
        if (const char *e = std::getenv("HOMCOMP_GRID_PERCENT")) {
            const long v = std::strtol(e, nullptr, 10);
            if (v >= 1 && v <= 100) pct = v;
        }
        homcomp_workspace_set_option(ws, HOMCOMP_OPT_GRID_PERCENT, pct);
        // a spill slot per deferred tile and data wave of the widest encoder grid, no more waves than tiles
        size_t waves = (size_t)(widest > 1 ? widest - 1 : 1) * 4;
        if (waves > ws->max_tiles) waves = ws->max_tiles;
        ok = spill_acquire(ws, waves * ws->out_slots * hc::kSpillSlotBytes) == HOMCOMP_OK;
    }
    ws->last_kind = ws->last_budget = -1;
    ws->stage_class = -1;
    if (const char *e = std::getenv("HOMCOMP_STAGE")) {
        if (std::strcmp(e, "small") == 0) ws->stage_class = 0;
        if (std::strcmp(e, "medium") == 0) ws->stage_class = 1;
        if (std::strcmp(e, "large") == 0) ws->stage_class = 2;
    }
    ws->sliced = 1;
    if (const char *e = std::getenv("HOMCOMP_SLICED")) {
        const long v = std::strtol(e, nullptr, 10);
        ws->sliced = v < 0 ? 0 : (v > 3 ? 3 : (int)v);
    }
    ws->spin_limit = kSpinLimit;
    if (const char *e = std::getenv("HOMCOMP_SPIN_LIMIT")) {
        const long v = std::strtol(e, nullptr, 10);
        if (v >= 0 && v <= (1l << 30)) ws->spin_limit = (uint32_t)v;
    }
    // HOMCOMP_EPOCH_START: the epoch handed out last before the first call (tests cross the wrap with it)
    if (const char *e = std::getenv("HOMCOMP_EPOCH_START")) {
        const long v = std::strtol(e, nullptr, 10);
        if (v >= 0 && v <= (long)kMaxEpoch) ws->epoch = (uint32_t)v;
    }
    if (!ok || !hip_ok(hipMalloc(&ws->d_block, bytes)) || !hip_ok(hipMemset(ws->d_block, 0, bytes)) ||
        !hip_ok(hipHostMalloc((void **)&ws->h_total, (5 + hc::kOpCount) * sizeof(uint64_t), hipHostMallocDefault))) {
        if (ws->d_block) (void)hipFree(ws->d_block);
        (void)spill_release(ws);
        delete ws;
        return HOMCOMP_ERR_HIP;
    }
    std::memset(ws->h_total, 0, (5 + hc::kOpCount) * sizeof(uint64_t));
    ws->h_mean_tile = ws->h_total + 2;
    ws->h_few = ws->h_mean_tile + hc::kOpCount;
    uint8_t *base = (uint8_t *)ws->d_block;
    ws->d_tile_totals = (uint64_t *)(base + o_status);
    ws->d_tile_prefixes = ws->d_tile_totals + t;
    ws->d_in_ofs[0] = (uint64_t *)(base + o_in0);
    ws->d_in_ofs[1] = (uint64_t *)(base + o_in1);
    ws->d_in_blocks[0] = (uint64_t *)(base + o_blk0);
    ws->d_in_blocks[1] = (uint64_t *)(base + o_blk1);
    ws->d_total = (uint64_t *)(base + o_total);
    ws->d_error = (uint32_t *)(base + o_total + 8);
    ws->d_partial = (float *)(base + o_partial);
    *out = ws;
    return HOMCOMP_OK;
}

int homcomp_workspace_set_option(homcomp_workspace *ws, int option, long value)
{
    if (!ws) return HOMCOMP_ERR_INVALID_ARG;
    switch (option) {
    case HOMCOMP_OPT_GRID_PERCENT:
        if (value < 1 || value > 100) return HOMCOMP_ERR_INVALID_ARG;
        for (int op = 0; op < hc::kOpCount; ++op) {
            for (int cls = 0; cls < kStageClasses; ++cls) {
                uint32_t g = (uint32_t)((uint64_t)ws->full_grid[op][cls] * (uint64_t)value / 100u);
                if (g < 2) g = 2;   // an encoder needs a data workgroup and the scan server
                ws->max_grid[op][cls] = g;
            }
        }
        return HOMCOMP_OK;
    case HOMCOMP_OPT_SPIN_LIMIT:
        if (value < 0 || value > (1l << 30)) return HOMCOMP_ERR_INVALID_ARG;
        ws->spin_limit = (uint32_t)value;
        return HOMCOMP_OK;
    case HOMCOMP_OPT_LDS_BUDGET:
        if (value < -1 || value >= kStageClasses) return HOMCOMP_ERR_INVALID_ARG;
        ws->stage_class = (int)value;
        return HOMCOMP_OK;
    case HOMCOMP_OPT_PLANE_PATHS:
        if (value < 0 || value > 3) return HOMCOMP_ERR_INVALID_ARG;
        ws->sliced = (uint32_t)value;
        return HOMCOMP_OK;
    default:
        return HOMCOMP_ERR_INVALID_ARG;
    }
}

int homcomp_workspace_last_launch(const homcomp_workspace *ws, int *kernel_kind, int *lds_budget)
{
    if (!ws) return HOMCOMP_ERR_INVALID_ARG;
    if (kernel_kind) *kernel_kind = ws->last_kind;
    if (lds_budget) *lds_budget = ws->last_budget;
    return HOMCOMP_OK;
}

size_t homcomp_tile_offsets_count(size_t nbEle) { return padded_len(nbEle) / hc::kHostTileElems; }

int homcomp_workspace_tile_offsets(homcomp_workspace *ws, const uint64_t *d_in_a, const uint64_t *d_in_b, uint64_t *d_out)
{
    if (!ws) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_in_a) || !aligned16(d_in_b) || !aligned16(d_out)) return HOMCOMP_ERR_ALIGNMENT;
    ws->next_in_ofs[0] = d_in_a;
    ws->next_in_ofs[1] = d_in_b;
    ws->next_out_ofs = d_out;
    return HOMCOMP_OK;
}

int homcomp_workspace_destroy(homcomp_workspace *ws)
{
    if (!ws) return HOMCOMP_OK;
    int rc = HOMCOMP_OK;
    if (!hip_ok(hipDeviceSynchronize())) rc = HOMCOMP_ERR_HIP;
    if (!hip_ok(hipFree(ws->d_block))) rc = HOMCOMP_ERR_HIP;
    if (spill_release(ws) != HOMCOMP_OK) rc = HOMCOMP_ERR_HIP;
    if (!hip_ok(hipHostFree(ws->h_total))) rc = HOMCOMP_ERR_HIP;
    delete ws;
    return rc;
}

int homcomp_compress_f32(homcomp_workspace *ws, const float *d_data, size_t nbEle, float eb,
                         unsigned char *d_cmp, uint64_t *d_stream_len, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    const HandOver hand_over(ws);
    int rc = check_ws(ws, nbEle);
    if (rc) return rc;
    if (!eb_ok(eb)) return HOMCOMP_ERR_INVALID_ARG;
    if (nbEle == 0) return empty_stream(ws, d_stream_len, s);
    if (!d_data || !d_cmp) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_data)) return HOMCOMP_ERR_ALIGNMENT;
    hc::TileParams p;
    if ((rc = fill_params(ws, nbEle, s, &p))) return rc;
    p.local = d_data;
    p.out_cmp = d_cmp;
    p.eb = eb;
    p.recip = 0.5f / eb;
    p.user_total = d_stream_len;
    return run_tile_op(ws, hc::kOpCompress, p, 0, s);
}

int homcomp_compress_plain_f32(homcomp_workspace *ws, const float *d_data, size_t nbEle, float eb,
                               unsigned char *d_cmp, uint64_t *d_stream_len, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    const HandOver hand_over(ws);
    int rc = check_ws(ws, nbEle);
    if (rc) return rc;
    if (!eb_ok(eb)) return HOMCOMP_ERR_INVALID_ARG;
    if (nbEle == 0) return empty_stream(ws, d_stream_len, s);
    if (!d_data || !d_cmp) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_data)) return HOMCOMP_ERR_ALIGNMENT;
    hc::TileParams p;
    if ((rc = fill_params(ws, nbEle, s, &p))) return rc;
    p.local = d_data;
    p.out_cmp = d_cmp;
    p.eb = eb;
    p.recip = 0.5f / eb;
    p.user_total = d_stream_len;
    p.plain = 1;
    return run_tile_op(ws, hc::kOpCompress, p, 0, s);
}

int homcomp_decompress_plain_f32(homcomp_workspace *ws, const unsigned char *d_cmp, size_t nbEle, float eb,
                                 float *d_out, void *stream)
{
    // A plain stream is a stream of the outlier codec in which every block is in plain mode, so
    // the one decoder reads both.  The plain decoder of the reference knows no stated size:
    // every block is read.
    return homcomp_decompress_f32(ws, d_cmp, homcomp_max_stream_bytes(nbEle), nbEle, eb, d_out, stream);
}

int homcomp_decompress_f32(homcomp_workspace *ws, const unsigned char *d_cmp, size_t cmp_size,
                           size_t nbEle, float eb, float *d_out, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    const HandOver hand_over(ws);
    int rc = check_ws(ws, nbEle);
    if (rc) return rc;
    if (!eb_ok(eb)) return HOMCOMP_ERR_INVALID_ARG;
    if (nbEle == 0) return HOMCOMP_OK;
    if (!d_cmp || !d_out) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_out)) return HOMCOMP_ERR_ALIGNMENT;
    hc::TileParams p;
    if ((rc = fill_params(ws, nbEle, s, &p))) return rc;
    p.in[0] = d_cmp;
    p.in_size[0] = cmp_size;
    p.out_f32 = d_out;
    p.eb = eb;
    p.recip = 0.5f / eb;
    if ((rc = in_offsets(ws, 1, &p, s))) return rc;
    return run_tile_op(ws, hc::kOpDecompress, p, tile_bytes_of(p, cmp_size), s);
}

int homcomp_hom_sum_f32(homcomp_workspace *ws, const unsigned char *d_cmp_in, size_t cmp_in_size,
                        const float *d_local, size_t nbEle, float eb, unsigned char *d_cmp_out,
                        uint64_t *d_stream_len, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    const HandOver hand_over(ws);
    int rc = check_ws(ws, nbEle);
    if (rc) return rc;
    if (!eb_ok(eb)) return HOMCOMP_ERR_INVALID_ARG;
    if (nbEle == 0) return empty_stream(ws, d_stream_len, s);
    if (!d_cmp_in || !d_local || !d_cmp_out) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_local)) return HOMCOMP_ERR_ALIGNMENT;
    hc::TileParams p;
    if ((rc = fill_params(ws, nbEle, s, &p))) return rc;
    p.in[0] = d_cmp_in;
    p.in_size[0] = cmp_in_size;
    p.local = d_local;
    p.out_cmp = d_cmp_out;
    p.eb = eb;
    p.recip = 0.5f / eb;
    p.user_total = d_stream_len;
    if ((rc = in_offsets(ws, 1, &p, s))) return rc;
    return run_tile_op(ws, hc::kOpHomSumF32, p, tile_bytes_of(p, cmp_in_size), s);
}

int homcomp_hom_sum_i32(homcomp_workspace *ws, const unsigned char *d_cmp_in, size_t cmp_in_size,
                        const int32_t *d_local_delta, size_t nbEle, unsigned char *d_cmp_out,
                        uint64_t *d_stream_len, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    const HandOver hand_over(ws);
    int rc = check_ws(ws, nbEle);
    if (rc) return rc;
    if (nbEle == 0) return empty_stream(ws, d_stream_len, s);
    if (!d_cmp_in || !d_local_delta || !d_cmp_out) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_local_delta)) return HOMCOMP_ERR_ALIGNMENT;
    // no stream of nbEle elements is longer than the first term, and callers of the reference state
    // the length plus the header bytes (homcomp_ref_cmpsize); see the note at the declaration
    if (cmp_in_size > homcomp_max_stream_bytes(nbEle) + homcomp_header_bytes(nbEle)) return HOMCOMP_ERR_INVALID_ARG;
    hc::TileParams p;
    if ((rc = fill_params(ws, nbEle, s, &p))) return rc;
    p.in[0] = d_cmp_in;
    p.in_size[0] = cmp_in_size;
    p.local = d_local_delta;
    p.out_cmp = d_cmp_out;
    p.user_total = d_stream_len;
    if ((rc = in_offsets(ws, 1, &p, s))) return rc;
    return run_tile_op(ws, hc::kOpHomSumI32, p, tile_bytes_of(p, cmp_in_size), s);
}

int homcomp_hom_add(homcomp_workspace *ws, const unsigned char *d_cmp_a, size_t size_a,
                    const unsigned char *d_cmp_b, size_t size_b, size_t nbEle,
                    unsigned char *d_cmp_out, uint64_t *d_stream_len, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    const HandOver hand_over(ws);
    int rc = check_ws(ws, nbEle);
    if (rc) return rc;
    if (nbEle == 0) return empty_stream(ws, d_stream_len, s);
    if (!d_cmp_a || !d_cmp_b || !d_cmp_out) return HOMCOMP_ERR_INVALID_ARG;
    hc::TileParams p;
    if ((rc = fill_params(ws, nbEle, s, &p))) return rc;
    p.in[0] = d_cmp_a;
    p.in_size[0] = size_a;
    p.in[1] = d_cmp_b;
    p.in_size[1] = size_b;
    p.out_cmp = d_cmp_out;
    p.user_total = d_stream_len;
    if ((rc = in_offsets(ws, 2, &p, s))) return rc;
    const uint64_t ta = tile_bytes_of(p, size_a), tb = tile_bytes_of(p, size_b);
    return run_tile_op(ws, hc::kOpHomAdd, p, ta > tb ? ta : tb, s);
}

int homcomp_hom_sum_f32_static(const unsigned char *d_cmp_in, size_t cmp_in_size, const float *d_local,
                               size_t nbEle, float eb, unsigned char *d_cmp_out, uint64_t *d_result,
                               void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    if (!d_result || !eb_ok(eb)) return HOMCOMP_ERR_INVALID_ARG;
    if (nbEle > kStaticMaxElems) return HOMCOMP_ERR_TOO_LARGE;
    // d_result[0] = stream length, d_result[1] = non-zero if a wave gave up waiting in the scan
    if (!hip_ok(hc::launch_fill_u64(d_result, 2, s))) return HOMCOMP_ERR_HIP;
    if (nbEle == 0) return HOMCOMP_OK;
    if (!d_cmp_in || !d_local || !d_cmp_out) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_local)) return HOMCOMP_ERR_ALIGNMENT;
    int device = -1;
    if (!hip_ok(hipGetDevice(&device))) return HOMCOMP_ERR_HIP;
    if (device < 0 || device >= kMaxDevices) return HOMCOMP_ERR_NO_DEVICE;
    StaticState *st = nullptr;
    int rc = static_setup(device, &st);
    if (rc) return rc;
    uint8_t *base = st->base;
    hc::TileParams p;
    std::memset(&p, 0, sizeof p);
    p.n = nbEle;
    p.hdr_bytes = homcomp_header_bytes(nbEle);
    p.n_tiles = (uint32_t)(padded_len(nbEle) / hc::kHostTileElems);
    p.tile_totals = (uint64_t *)(base + kStaticOfsScan);
    p.tile_prefixes = p.tile_totals + kStaticMaxTiles;
    p.spin_limit = kSpinLimit;
    p.total = d_result;
    p.error = (uint32_t *)(d_result + 1);
    p.epoch = 1;   // the scan words of the tiles in use are cleared by every call, so one tag serves
    p.in[0] = d_cmp_in;
    p.in_size[0] = cmp_in_size;
    p.in_ofs[0] = (uint64_t *)(base + kStaticOfsIn);
    p.local = d_local;
    p.out_cmp = d_cmp_out;
    p.eb = eb;
    p.recip = 0.5f / eb;
    p.spill = base + kStaticOfsSpill;
    p.out_slots = kStaticSlots;
    p.sliced = tile_bytes_of(p, cmp_in_size) <= kBitplaneTileBytes;
    const int cls = choose_stage_class(hc::kOpHomSumF32, tile_bytes_of(p, cmp_in_size), kStaticSlots);
    p.stage_bytes = kStage[cls][hc::kOpHomSumF32];
    // totals and prefixes of the tiles this call uses and the block words of its pre-pass (the
    // arrays keep the last call's words)
    hc::InOffsetsArgs a;
    std::memset(&a, 0, sizeof a);
    a.hdr[0] = d_cmp_in;
    a.block_words[0] = (uint64_t *)(base + kStaticOfsBlocks);
    a.ofs[0] = (uint64_t *)(base + kStaticOfsIn);
    a.error = p.error;
    if (!hip_ok(hc::launch_fill_u64(p.tile_totals, p.n_tiles, s)) ||
        !hip_ok(hc::launch_fill_u64(p.tile_prefixes, p.n_tiles, s)) ||
        !hip_ok(hc::launch_fill_u64(a.block_words[0], (uint64_t)p.n_tiles / 256 + 1, s)))
        return HOMCOMP_ERR_HIP;
    if (!hip_ok(hc::launch_in_offsets(a, 1, p.n_tiles, p.hdr_bytes, p.epoch, p.spin_limit, s))) return HOMCOMP_ERR_HIP;
    return chained_launch(device, hc::kOpHomSumF32, p, st->grid[cls], s);
}

int homcomp_quant_predict_f32(const float *d_data, size_t nbEle, float eb, int32_t *d_delta,
                              void *stream)
{
    if (!eb_ok(eb)) return HOMCOMP_ERR_INVALID_ARG;
    if (nbEle == 0) return HOMCOMP_OK;
    if (!d_data || !d_delta) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_data) || !aligned16(d_delta)) return HOMCOMP_ERR_ALIGNMENT;
    return hip_ok(hc::launch_quant_predict(d_data, d_delta, nbEle, 0.5f / eb, (hipStream_t)stream))
               ? HOMCOMP_OK
               : HOMCOMP_ERR_HIP;
}

int homcomp_range_f32(homcomp_workspace *ws, const float *d_data, size_t nbEle, float *d_minmax,
                      void *stream)
{
    int rc = check_ws(ws, 0);
    if (rc) return rc;
    if (!d_data || !d_minmax || nbEle == 0) return HOMCOMP_ERR_INVALID_ARG;
    if (!aligned16(d_data)) return HOMCOMP_ERR_ALIGNMENT;
    return hip_ok(hc::launch_range(d_data, nbEle, ws->d_partial, kRangePartials, d_minmax,
                                   (hipStream_t)stream))
               ? HOMCOMP_OK
               : HOMCOMP_ERR_HIP;
}

int homcomp_last_size(homcomp_workspace *ws, size_t *stream_len, void *stream)
{
    if (!ws || !stream_len) return HOMCOMP_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (!hip_ok(hipMemcpyAsync(ws->h_total, ws->d_total, 2 * sizeof(uint64_t), hipMemcpyDeviceToHost, s)) ||
        !hip_ok(hipStreamSynchronize(s)))
        return HOMCOMP_ERR_HIP;
    *stream_len = (size_t)ws->h_total[0];
    if ((uint32_t)ws->h_total[1] == 0) return HOMCOMP_OK;
    // reported once: the flag is cleared (on the same stream) so that the workspace can go on
    if (!hip_ok(hc::launch_fill_u64(ws->d_total + 1, 1, s))) return HOMCOMP_ERR_HIP;
    return HOMCOMP_ERR_SCAN_TIMEOUT;
}

}  // extern "C"
