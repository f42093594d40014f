// The ring all-reduce that calls the homomorphic compressor (HomComp/src/cuda_awareallreduce.cu:
// allreduce_ring_comprs_hom_sum :43-163, _hom_sum_F :166-265, _hom_sum_seg :268-433,
// _hom_sum_F_seg :436-585), on top of the C ABI of include/homcomp.h.
//
// Same names, argument order and schedule as the reference; the MPI communicator is replaced by
// the small interface RingComm, which has exactly the four MPI calls the reference makes on
// device buffers (MPI_Irecv / MPI_Send / MPI_Wait + MPI_Get_count / MPI_Sendrecv), so a
// maintainer implements it once over MPI or RCCL, and tests run it over the in-process
// communicator of loopback_comm.hpp (several ranks as host threads on one GPU).
//
// Per rank and call (size = R ranks, block b = the b-th piece of the array):
//   reduce-scatter  compress own block `rank`, send; R-2 times: receive a stream, add the local
//                   copy of that block in the compressed domain (homomorphic sum), send on; the
//                   last received stream (block rank+1) is summed and decompressed in place
//   all-gather      R-1 times: pass the reduced stream on, receive the neighbour's, decompress it
// Differences from the reference, none of which changes the reduced values:
//   * stream buffers hold homcomp_max_stream_bytes(block) bytes (the reference's 4 * block_count
//     is only enough for compressible data, and it sends its over-reported cmpSize, N/32 bytes
//     more than the stream); the true stream length is sent;
//   * the padding of the temporary array is zero-filled (the reference reduces whatever
//     cudaMalloc left there; it is never copied out);
//   * where the padding of the segmented variants pushes the start of the last block beyond
//     the array (count far below its multiple of 32768) the reference's block count goes
//     negative; here that block is empty and the blocks before it carry the padding;
//   * buffers and the workspace can be kept between calls (RingBuffers), which is what the
//     reference's _opt variant does by hand (:745-760);
//   * a message is the stream preceded by its tile offsets (8 bytes per 4096 elements of the
//     block, homcomp_workspace_tile_offsets): the call that produced the stream leaves them in
//     front of it, and the receiving rank's call takes them from there instead of scanning the
//     header bytes first (a launch of its own, a third of a ring step's call).
// Returns 0, or the first non-zero status (HOMCOMP_ERR_* or the communicator's).
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <vector>

#include "../../include/homcomp.h"

namespace homcomp {

class RingComm {
public:
    virtual ~RingComm() = default;
    virtual int rank() const = 0;
    virtual int size() const = 0;
    // MPI_Irecv(d_buf, capacity, MPI_BYTE, from, 0, comm, &reqs[request]); request is 0 or 1
    virtual int irecv(void *d_buf, size_t capacity, int from, int request) = 0;
    // MPI_Send(d_buf, bytes, MPI_BYTE, to, 0, comm); the data is complete on the device
    virtual int send(const void *d_buf, size_t bytes, int to) = 0;
    // MPI_Wait(&reqs[request], &status); MPI_Get_count(&status, MPI_BYTE, bytes)
    virtual int wait(int request, size_t *bytes) = 0;
    // MPI_Sendrecv(d_send, send_bytes, ..., to, d_recv, capacity, ..., from) + MPI_Get_count
    virtual int sendrecv(const void *d_send, size_t send_bytes, int to, void *d_recv, size_t capacity, int from,
                         size_t *bytes) = 0;
};

// Block b of the array: elements [offset[b], offset[b] + count[b]) of the padded temporary.
struct RingBlocks {
    std::vector<size_t> offset, count;
    size_t max_count = 0;   // largest block
    size_t padded = 0;      // elements of the temporary array
};

// HomComp/src/cuda_awareallreduce.cu:189-190: equal blocks of ceil(count / size), padded to 32768.
inline RingBlocks ring_blocks_equal(size_t count, int size)
{
    RingBlocks b;
    size_t block = (count + (size_t)size - 1) / (size_t)size;
    block = (block + 32768 - 1) / 32768 * 32768;
    for (int i = 0; i < size; ++i) {
        b.offset.push_back(block * (size_t)i);
        b.count.push_back(block);
    }
    b.max_count = block;
    b.padded = block * (size_t)size;
    return b;
}

// HomComp/src/cuda_awareallreduce.cu:455-489 (COLL_BASE_COMPUTE_BLOCKCOUNT on the count padded to
// 32768, block counts rounded up to multiples of 4, the last block ends with the array).
inline RingBlocks ring_blocks_seg(size_t count, int size)
{
    RingBlocks b;
    const size_t pad = (count + 32768 - 1) / 32768 * 32768;
    size_t early = pad / (size_t)size, late = early;
    const size_t split = pad % (size_t)size;
    if (split != 0) early += 1;
    early += (4 - early % 4) % 4;
    late += (4 - late % 4) % 4;
    for (int i = 0; i < size; ++i) {
        const size_t r = (size_t)i;
        const size_t off = r < split ? r * early : split * early + (r - split) * late;
        size_t cnt = r < split ? early : late;
        if (i == size - 1) cnt = count > off ? count - off : 0;
        b.offset.push_back(off);
        b.count.push_back(cnt);
    }
    b.max_count = early;
    b.padded = early * split + late * ((size_t)size - split);
    if (b.padded < count) b.padded = count;
    return b;
}

// Device buffers and workspace of one rank; grows on demand, freed with the object.
class RingBuffers {
public:
    RingBuffers() = default;
    RingBuffers(const RingBuffers &) = delete;
    RingBuffers &operator=(const RingBuffers &) = delete;
    ~RingBuffers() { release(); }

    int reserve(size_t padded, size_t max_block, bool int_deltas)
    {
        if (padded <= cap_padded_ && max_block <= cap_block_ && (!int_deltas || d_quant)) return HOMCOMP_OK;
        release();
        // a message: the tile offsets of the block's stream, then the stream
        stream_cap = homcomp_tile_offsets_count(max_block) * sizeof(uint64_t) + homcomp_max_stream_bytes(max_block);
        bool ok = hipMalloc((void **)&d_rtmpbuf, (padded ? padded : 1) * sizeof(float)) == hipSuccess;
        ok = ok && hipMalloc((void **)&d_cmpReduceBytes, stream_cap + HOMCOMP_STREAM_SLACK) == hipSuccess;
        ok = ok && hipMalloc((void **)&d_inbuf[0], stream_cap + HOMCOMP_STREAM_SLACK) == hipSuccess;
        ok = ok && hipMalloc((void **)&d_inbuf[1], stream_cap + HOMCOMP_STREAM_SLACK) == hipSuccess;
        if (int_deltas) ok = ok && hipMalloc((void **)&d_quant, (max_block ? max_block : 1) * sizeof(int)) == hipSuccess;
        if (!ok) {
            release();
            return HOMCOMP_ERR_HIP;
        }
        const int rc = homcomp_workspace_create(&ws, max_block);
        if (rc != HOMCOMP_OK) {
            release();
            return rc;
        }
        cap_padded_ = padded;
        cap_block_ = max_block;
        return HOMCOMP_OK;
    }

    float *d_rtmpbuf = nullptr;
    unsigned char *d_cmpReduceBytes = nullptr;
    unsigned char *d_inbuf[2] = {nullptr, nullptr};
    int *d_quant = nullptr;
    homcomp_workspace *ws = nullptr;
    size_t stream_cap = 0;   // capacity of a message buffer

private:
    void release()
    {
        if (ws) homcomp_workspace_destroy(ws);
        if (d_rtmpbuf) (void)hipFree(d_rtmpbuf);
        if (d_cmpReduceBytes) (void)hipFree(d_cmpReduceBytes);
        if (d_inbuf[0]) (void)hipFree(d_inbuf[0]);
        if (d_inbuf[1]) (void)hipFree(d_inbuf[1]);
        if (d_quant) (void)hipFree(d_quant);
        ws = nullptr;
        d_rtmpbuf = nullptr;
        d_cmpReduceBytes = d_inbuf[0] = d_inbuf[1] = nullptr;
        d_quant = nullptr;
        cap_padded_ = cap_block_ = 0;
    }
    size_t cap_padded_ = 0, cap_block_ = 0;
};

namespace detail {

struct RingCall {
    RingBuffers &buf;
    float eb;
    bool int_deltas;
    hipStream_t stream;

    // A stream-producing call and its size read-back (blocking, as the reference's wrappers).  A
    // call that ended in HOMCOMP_ERR_SCAN_TIMEOUT (kernels of the transport held compute units,
    // so its grid was not resident as a whole) is repeated once with half the grid, which the
    // workspace then keeps.
    template <typename Launch>
    int sized(Launch launch, size_t *len) const
    {
        int rc = launch();
        if (rc == HOMCOMP_OK) rc = homcomp_last_size(buf.ws, len, stream);
        if (rc != HOMCOMP_ERR_SCAN_TIMEOUT) return rc;
        homcomp_workspace_set_option(buf.ws, HOMCOMP_OPT_GRID_PERCENT, 50);
        rc = launch();
        return rc != HOMCOMP_OK ? rc : homcomp_last_size(buf.ws, len, stream);
    }
    // A message buffer holds the tile offsets of the block's stream, then the stream.
    static size_t ofs_bytes(size_t n) { return homcomp_tile_offsets_count(n) * sizeof(uint64_t); }
    static uint64_t *ofs_of(unsigned char *d_msg) { return reinterpret_cast<uint64_t *>(d_msg); }
    static const uint64_t *ofs_of(const unsigned char *d_msg) { return reinterpret_cast<const uint64_t *>(d_msg); }
    // A stream-producing call into the message buffer d_out, reading the message d_in (or none);
    // *msg_len = offsets + stream.  (The hand-over of the offsets is one call's: it is made again
    // when a timed-out call is repeated.)
    template <typename Launch>
    int produce(Launch launch, size_t n, const unsigned char *d_in, unsigned char *d_out, size_t *msg_len) const
    {
        size_t len = 0;
        const int rc = sized(
            [&] {
                const int ro = homcomp_workspace_tile_offsets(buf.ws, n && d_in ? ofs_of(d_in) : nullptr, nullptr,
                                                              n ? ofs_of(d_out) : nullptr);
                return ro != HOMCOMP_OK ? ro : launch(d_out + ofs_bytes(n));
            },
            &len);
        *msg_len = ofs_bytes(n) + len;
        return rc;
    }
    // GSZ_compress_deviceptr_outlier
    int compress(const float *d_block, size_t n, unsigned char *d_out, size_t *msg_len) const
    {
        return produce([&](unsigned char *d_cmp) { return homcomp_compress_f32(buf.ws, d_block, n, eb, d_cmp, nullptr, stream); }, n,
                       nullptr, d_out, msg_len);
    }
    // homomorphic_sum_F, or kernel_quant_prediction + homomorphic_sum (:61-72), on a received message
    int hom_sum(const unsigned char *d_in, size_t in_msg_len, const float *d_block, size_t n, unsigned char *d_out,
                size_t *msg_len) const
    {
        if (in_msg_len < ofs_bytes(n)) return HOMCOMP_ERR_INVALID_ARG;
        const unsigned char *d_cmp_in = d_in + ofs_bytes(n);
        const size_t in_len = in_msg_len - ofs_bytes(n);
        if (int_deltas) {
            const int rc = homcomp_quant_predict_f32(d_block, n, eb, buf.d_quant, stream);
            if (rc != HOMCOMP_OK) return rc;
        }
        return produce(
            [&](unsigned char *d_cmp) {
                return int_deltas ? homcomp_hom_sum_i32(buf.ws, d_cmp_in, in_len, buf.d_quant, n, d_cmp, nullptr, stream)
                                  : homcomp_hom_sum_f32(buf.ws, d_cmp_in, in_len, d_block, n, eb, d_cmp, nullptr, stream);
            },
            n, d_in, d_out, msg_len);
    }
    int decompress(const unsigned char *d_in, size_t in_msg_len, float *d_block, size_t n) const
    {
        if (in_msg_len < ofs_bytes(n)) return HOMCOMP_ERR_INVALID_ARG;
        int rc = homcomp_workspace_tile_offsets(buf.ws, n ? ofs_of(d_in) : nullptr, nullptr, nullptr);
        if (rc == HOMCOMP_OK)
            rc = homcomp_decompress_f32(buf.ws, d_in + ofs_bytes(n), in_msg_len - ofs_bytes(n), n, eb, d_block, stream);
        if (rc != HOMCOMP_OK) return rc;
        return hipStreamSynchronize(stream) == hipSuccess ? HOMCOMP_OK : HOMCOMP_ERR_HIP;
    }
};

#define HOMCOMP_RING_TRY(expr)          \
    do {                                \
        const int rc_ = (expr);         \
        if (rc_ != 0) return rc_;       \
    } while (0)

inline int ring(const float *d_sbuf, float *d_rbuf, size_t count, RingComm &comm, float eb, const RingBlocks &blk,
                bool int_deltas, RingBuffers &buf, hipStream_t stream)
{
    const int rank = comm.rank(), size = comm.size();
    if (size == 1) return 0;   // as the reference: nothing is done, d_rbuf is not written
    HOMCOMP_RING_TRY(buf.reserve(blk.padded, blk.max_count, int_deltas));
    const RingCall op{buf, eb, int_deltas, stream};
    float *tmp = buf.d_rtmpbuf;
    if (hipMemsetAsync(tmp, 0, blk.padded * sizeof(float), stream) != hipSuccess) return HOMCOMP_ERR_HIP;
    if (hipMemcpyAsync(tmp, d_sbuf, count * sizeof(float), hipMemcpyDeviceToDevice, stream) != hipSuccess)
        return HOMCOMP_ERR_HIP;

    int send_to = (rank + 1) % size;
    int recv_from = (rank + size - 1) % size;
    size_t cmpSize = 0, cmpSize2 = 0;
    int inbi = 0;

    // ---- reduce-scatter (:196-243)
    HOMCOMP_RING_TRY(op.compress(tmp + blk.offset[rank], blk.count[rank], buf.d_cmpReduceBytes, &cmpSize));
    HOMCOMP_RING_TRY(comm.irecv(buf.d_inbuf[inbi], buf.stream_cap, recv_from, inbi));
    HOMCOMP_RING_TRY(comm.send(buf.d_cmpReduceBytes, cmpSize, send_to));
    for (int k = 2; k < size; ++k) {
        const int prevblock = (rank + size - k + 1) % size;
        inbi ^= 1;
        HOMCOMP_RING_TRY(comm.irecv(buf.d_inbuf[inbi], buf.stream_cap, recv_from, inbi));
        HOMCOMP_RING_TRY(comm.wait(inbi ^ 1, &cmpSize2));
        HOMCOMP_RING_TRY(op.hom_sum(buf.d_inbuf[inbi ^ 1], cmpSize2, tmp + blk.offset[prevblock], blk.count[prevblock],
                                    buf.d_cmpReduceBytes, &cmpSize));
        HOMCOMP_RING_TRY(comm.send(buf.d_cmpReduceBytes, cmpSize, send_to));
    }
    const int last = (rank + 1) % size;
    HOMCOMP_RING_TRY(comm.wait(inbi, &cmpSize2));
    HOMCOMP_RING_TRY(op.hom_sum(buf.d_inbuf[inbi], cmpSize2, tmp + blk.offset[last], blk.count[last],
                                buf.d_inbuf[inbi ^ 1], &cmpSize));
    HOMCOMP_RING_TRY(op.decompress(buf.d_inbuf[inbi ^ 1], cmpSize, tmp + blk.offset[last], blk.count[last]));

    // ---- all-gather of the reduced streams (:244-257)
    for (int k = 0; k < size - 1; ++k) {
        inbi ^= 1;
        const int recv_data_from = (rank + size - k) % size;
        HOMCOMP_RING_TRY(comm.sendrecv(buf.d_inbuf[inbi], cmpSize, send_to, buf.d_inbuf[inbi ^ 1], buf.stream_cap,
                                       recv_from, &cmpSize));
        HOMCOMP_RING_TRY(op.decompress(buf.d_inbuf[inbi ^ 1], cmpSize, tmp + blk.offset[recv_data_from],
                                       blk.count[recv_data_from]));
    }
    if (hipMemcpyAsync(d_rbuf, tmp, count * sizeof(float), hipMemcpyDeviceToDevice, stream) != hipSuccess)
        return HOMCOMP_ERR_HIP;
    return hipStreamSynchronize(stream) == hipSuccess ? 0 : HOMCOMP_ERR_HIP;
}

#undef HOMCOMP_RING_TRY

inline RingBuffers &thread_buffers()
{
    thread_local RingBuffers buffers;
    return buffers;
}

}  // namespace detail
}  // namespace homcomp

// HomComp/include/cuda_awareallreduce.cuh:4-11 with MPI_Comm -> homcomp::RingComm&.  The optional
// arguments keep the buffers between calls (default: one set per host thread) and name the stream.

inline int allreduce_ring_comprs_hom_sum(const float *d_sbuf, float *d_rbuf, size_t count, homcomp::RingComm &comm,
                                         float eb, homcomp::RingBuffers *buffers = nullptr, hipStream_t stream = 0)
{
    return homcomp::detail::ring(d_sbuf, d_rbuf, count, comm, eb, homcomp::ring_blocks_equal(count, comm.size()), true,
                                 buffers ? *buffers : homcomp::detail::thread_buffers(), stream);
}

inline int allreduce_ring_comprs_hom_sum_F(const float *d_sbuf, float *d_rbuf, size_t count, homcomp::RingComm &comm,
                                           float eb, homcomp::RingBuffers *buffers = nullptr, hipStream_t stream = 0)
{
    return homcomp::detail::ring(d_sbuf, d_rbuf, count, comm, eb, homcomp::ring_blocks_equal(count, comm.size()), false,
                                 buffers ? *buffers : homcomp::detail::thread_buffers(), stream);
}

inline int allreduce_ring_comprs_hom_sum_seg(const float *d_sbuf, float *d_rbuf, size_t count, homcomp::RingComm &comm,
                                             float eb, homcomp::RingBuffers *buffers = nullptr, hipStream_t stream = 0)
{
    return homcomp::detail::ring(d_sbuf, d_rbuf, count, comm, eb, homcomp::ring_blocks_seg(count, comm.size()), true,
                                 buffers ? *buffers : homcomp::detail::thread_buffers(), stream);
}

inline int allreduce_ring_comprs_hom_sum_F_seg(const float *d_sbuf, float *d_rbuf, size_t count,
                                               homcomp::RingComm &comm, float eb,
                                               homcomp::RingBuffers *buffers = nullptr, hipStream_t stream = 0)
{
    return homcomp::detail::ring(d_sbuf, d_rbuf, count, comm, eb, homcomp::ring_blocks_seg(count, comm.size()), false,
                                 buffers ? *buffers : homcomp::detail::thread_buffers(), stream);
}

// The reference's _opt variant (:711-893) is _hom_sum_F with the kernels launched directly on
// scratch arrays that are allocated once per call instead of once per step; here every variant
// keeps its scratch (workspace, RingBuffers), so it is the same function.
inline int allreduce_ring_comprs_hom_sum_F_opt(const float *d_sbuf, float *d_rbuf, size_t count,
                                               homcomp::RingComm &comm, float eb,
                                               homcomp::RingBuffers *buffers = nullptr, hipStream_t stream = 0)
{
    return allreduce_ring_comprs_hom_sum_F(d_sbuf, d_rbuf, count, comm, eb, buffers, stream);
}
