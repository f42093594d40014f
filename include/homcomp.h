/*
 * homcomp.h -- C ABI of the MI355X HomComp library (libhomcomp_amd.so).
 *
 * HomComp is an error-bounded lossy codec for float32 with a homomorphic sum: two compressed
 * streams (or a stream and raw data) are added in the quantised-integer domain and re-encoded
 * without dequantising.  Each entry point names the reference interface it replaces (paths are
 * relative to the reference repository's HomComp/ directory).
 *
 * Conventions
 *   - All data pointers are device pointers on the device that was current when the workspace
 *     was created.  float / int32 buffers must be 16-byte aligned; stream buffers may have any
 *     alignment.  Input and output buffers must not overlap.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Work is enqueued
 *     asynchronously; nothing blocks except homcomp_last_size().
 *   - `eb` is always an ABSOLUTE error bound (> 0).  Value-range-relative bounds are turned into
 *     absolute ones with homcomp_range_f32() + homcomp_rel_to_abs().
 *   - A stream of nbEle elements is  header[homcomp_header_bytes(nbEle)] || payload  and can take
 *     up to homcomp_max_stream_bytes(nbEle) bytes; every output stream buffer needs that
 *     capacity.  nbEle may be any count; elements past nbEle up to the next multiple of 32768
 *     are encoded as zeros (what the reference sees in a zero-padded buffer).
 *   - Sizes reported are TRUE stream lengths L.  The reference's wrappers report L +
 *     header_bytes (src/GSZ_entry.cu:291-295 adds the header twice); homcomp_ref_cmpsize()
 *     gives that number.
 *   - A workspace holds the scan state of one call at a time: calls sharing a workspace must be
 *     ordered on one stream (or otherwise serialised).  Use one workspace per concurrent stream.
 *   - An INPUT stream buffer must be readable up to cmp_size + 160 bytes (or up to
 *     homcomp_max_stream_bytes(nbEle), whichever is smaller): a block whose payload starts below
 *     the stated size is fetched in full (the out-of-bound rule of src/GSZ.cu:908-911 looks at the
 *     block's start only), in whole 16-byte pieces.  Buffers of homcomp_max_stream_bytes(nbEle) +
 *     HOMCOMP_STREAM_SLACK bytes always do.
 *   - Stream-producing kernels keep their whole grid resident and wait for each other's scan
 *     words, so the library orders such launches of one process on a device, also across
 *     streams.  Launches recorded into a HIP graph are outside that order: a replay must not
 *     run at the same time as another stream-producing call or replay on the device (order them
 *     on one stream or with events), and must end before its workspace is destroyed.
 *   - Every function returns HOMCOMP_OK (0) or a negative HOMCOMP_ERR_* code; no call aborts.
 */
#ifndef HOMCOMP_H
#define HOMCOMP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HOMCOMP_OK 0
#define HOMCOMP_ERR_INVALID_ARG (-1)  /* NULL pointer, eb <= 0 or not finite                   */
#define HOMCOMP_ERR_ALIGNMENT (-2)    /* float / int32 buffer not 16-byte aligned               */
#define HOMCOMP_ERR_TOO_LARGE (-3)    /* nbEle exceeds the workspace's max_nbEle                */
#define HOMCOMP_ERR_HIP (-4)          /* a HIP runtime call failed; see homcomp_last_hip_error  */
#define HOMCOMP_ERR_NO_DEVICE (-5)    /* no usable GPU                                           */
#define HOMCOMP_ERR_SCAN_TIMEOUT (-6) /* a kernel gave up waiting in the offset scan; reported    */
                                      /* by homcomp_last_size, which also clears it: the streams */
                                      /* produced on the workspace since the previous            */
                                      /* homcomp_last_size are invalid, later calls are not      */

typedef struct homcomp_workspace homcomp_workspace;

const char *homcomp_status_string(int status);
/* hipError_t of the most recent failing HIP call on this thread (0 if none). */
int homcomp_last_hip_error(void);

/* rate_ofs of src/GSZ.cu:48-50: one header byte per 32-element block of the padded length. */
size_t homcomp_header_bytes(size_t nbEle);
/* Worst-case stream length: header + 128 payload bytes per block.  (The reference allocates
 * only 4*nbEle, src/homcomp_eval.cu:176, which incompressible input can overrun.) */
size_t homcomp_max_stream_bytes(size_t nbEle);
/* Bytes an INPUT stream buffer must be readable beyond the stream's stated size (see the
 * conventions above); allocate stream buffers that will be read as
 * homcomp_max_stream_bytes(nbEle) + HOMCOMP_STREAM_SLACK. */
#define HOMCOMP_STREAM_SLACK 160
/* The value the reference's wrappers store in *cmpSize for a stream of true length L. */
size_t homcomp_ref_cmpsize(size_t stream_len, size_t nbEle);

/* Replaces the per-call cudaMalloc/cudaMemset/cudaFree of three (codec) or six (homomorphic
 * sum) scratch arrays in src/GSZ_entry.cu:275-280,519-530 -- the shape
 * allreduce_ring_comprs_hom_sum_F_opt hoists out of its loop (src/cuda_awareallreduce.cu:745-760).
 * max_nbEle below about 8.79e12 (2^31 - 2^16 tiles of 4096 elements), else HOMCOMP_ERR_TOO_LARGE. */
int homcomp_workspace_create(homcomp_workspace **ws, size_t max_nbEle);
int homcomp_workspace_destroy(homcomp_workspace *ws);
/* Tuning of a workspace; no counterpart in the reference, whose one-warp thread blocks wait for
 * their predecessors without a bound (src/GSZ.cu:196-223).
 *   HOMCOMP_OPT_GRID_PERCENT  share of the device a stream-producing launch of ws occupies, 1..100
 *       percent of the resident grid (default 100, or the environment variable
 *       HOMCOMP_GRID_PERCENT at creation).  The launch needs all its workgroups resident at once;
 *       where other kernels hold compute units for longer than the bounded waits (tens of
 *       milliseconds) a full grid ends in HOMCOMP_ERR_SCAN_TIMEOUT, a smaller one fits beside them.
 *   HOMCOMP_OPT_SPIN_LIMIT    unsuccessful re-reads of a scan word before a wave gives up, 0..2^30
 *       (default 65536, or HOMCOMP_SPIN_LIMIT at creation).
 *   HOMCOMP_OPT_LDS_BUDGET    LDS stage per data wave of the stream-producing kernels: -1 (default) chosen
 *       per call from the size of the tiles the workspace has seen (so the time of a call can depend
 *       on the calls before it, never its bytes), 0 / 1 / 2 = always the small / medium / large one
 *       (4 / 3 / 2 workgroups per compute unit; HOMCOMP_STAGE=small|medium|large at creation).
 *   HOMCOMP_OPT_PLANE_PATHS   which kernel kind the homomorphic sums run: 1 (default) chosen per call
 *       from the plane counts of the streams the workspace has seen, 0 = the general path only, 2 =
 *       always the kernels with the path for blocks of few planes, 3 = stream (+) stream always the
 *       kernel for wide blocks (HOMCOMP_SLICED=0..3 at creation).  Every kind gives the same bytes.
 * Fixing the last two makes timings independent of the workspace's history. */
#define HOMCOMP_OPT_GRID_PERCENT 1
#define HOMCOMP_OPT_SPIN_LIMIT 2
#define HOMCOMP_OPT_LDS_BUDGET 3
#define HOMCOMP_OPT_PLANE_PATHS 4
int homcomp_workspace_set_option(homcomp_workspace *ws, int option, long value);
/* What the last stream-producing call on ws was launched with: the kernel kind and the LDS budget
 * (0 small, 1 medium, 2 large); -1 before the first such call.  Either pointer may be NULL. */
#define HOMCOMP_KERNEL_GENERAL 0
#define HOMCOMP_KERNEL_FEW_PLANES 1
#define HOMCOMP_KERNEL_WIDE_PLANES 2
int homcomp_workspace_last_launch(const homcomp_workspace *ws, int *kernel_kind, int *lds_budget);

/* Tile offsets: a side array that spares the call that reads a stream its pass over the header
 * bytes.  The payload position of a block follows from the header bytes of all blocks before it
 * (src/GSZ.cu:790-874 sums them per 32768-element chunk and scans the sums in the same kernel); a
 * call here does that in a launch of its own ahead of the tile kernel, about 5 us for a stream of
 * any length up to 4M elements -- a third of a ring step's call.  The call that PRODUCES a stream
 * knows the offsets already, so it can leave them in a caller buffer, and the call that reads the
 * stream can take them from there:
 *   entry t (uint64, t < homcomp_tile_offsets_count(nbEle)) = byte offset, from the start of the
 *   stream, of the payload of elements 4096 t .. 4096 t + 4095 (header bytes included; entry 0 is
 *   homcomp_header_bytes(nbEle)).
 * The array is a function of the stream's header bytes alone.  In a ring it travels with the
 * chunk (8 bytes per 4096 elements: 8 KB beside a 4M-element chunk).
 * homcomp_workspace_tile_offsets hands arrays over for the NEXT call on ws that reads or produces
 * a stream, and that call only: d_in_a / d_in_b for its first / second incoming stream (NULL: the
 * call computes them as usual), d_out (NULL: none) receives the offsets of the stream it produces.
 * Device pointers, 16-byte aligned, homcomp_tile_offsets_count(nbEle) entries.  Offsets that do not
 * belong to the stream give wrong values, never accesses beyond the stream's stated size.  No
 * counterpart in the reference. */
size_t homcomp_tile_offsets_count(size_t nbEle);
int homcomp_workspace_tile_offsets(homcomp_workspace *ws, const uint64_t *d_in_a, const uint64_t *d_in_b, uint64_t *d_out);

/* GSZ_compress_deviceptr_outlier (include/GSZ_entry.h:14-16, src/GSZ_entry.cu:263-301).
 * d_stream_len (optional, device uint64) receives L when the kernel finishes. */
int homcomp_compress_f32(homcomp_workspace *ws, const float *d_data, size_t nbEle, float eb,
                         unsigned char *d_cmp, uint64_t *d_stream_len, void *stream);

/* GSZ_decompress_deviceptr_outlier (include/GSZ_entry.h:17-20, src/GSZ_entry.cu:317-350).
 * Blocks whose payload starts at or beyond cmp_size are skipped (src/GSZ.cu:908-911).  Skipped
 * and rate-0 blocks are written as 0.0f (the reference leaves them untouched; identical on a
 * pre-zeroed buffer). */
int homcomp_decompress_f32(homcomp_workspace *ws, const unsigned char *d_cmp, size_t cmp_size,
                           size_t nbEle, float eb, float *d_out, void *stream);

/* GSZ_compress_deviceptr_plain / GSZ_decompress_deviceptr_plain (include/GSZ_entry.h:8-13,
 * src/GSZ_entry.cu:150-228, kernels src/GSZ.cu:1475-1991): the plain codec, without the outlier
 * mode.  A block's header byte is the bit width of its largest |delta| (capped at 31, as in the
 * outlier codec), its payload the sign word and that many planes.  A plain stream is a stream
 * of the outlier codec whose blocks are all in plain mode: homcomp_decompress_f32 and the
 * homomorphic sums read it too.  The plain decoder has no out-of-bound rule (the reference's
 * kernel never looks at cmpSize): every block the header bytes describe is read, so the buffer
 * must hold the whole stream and be readable up to the 16-byte address boundary at or after its
 * last byte (payload is fetched in aligned 16-byte pieces; nothing further out is touched, and the
 * general rule about cmp_size + 160 above does not apply to this entry).  The reference's
 * wrapper reports a cmpSize that leaves out the payload of the last 32768-element chunk
 * (src/GSZ_entry.cu:176-180 reads the exclusive offset of the last thread block); the length
 * reported here is the true one. */
int homcomp_compress_plain_f32(homcomp_workspace *ws, const float *d_data, size_t nbEle, float eb,
                               unsigned char *d_cmp, uint64_t *d_stream_len, void *stream);
int homcomp_decompress_plain_f32(homcomp_workspace *ws, const unsigned char *d_cmp, size_t nbEle, float eb,
                                 float *d_out, void *stream);

/* homomorphic_sum_F (include/GSZ_entry.h:33-36, src/GSZ_entry.cu:504-550): out = encode(
 * deltas(in) + Lorenzo(quantise(local))). */
int homcomp_hom_sum_f32(homcomp_workspace *ws, const unsigned char *d_cmp_in, size_t cmp_in_size,
                        const float *d_local, size_t nbEle, float eb, unsigned char *d_cmp_out,
                        uint64_t *d_stream_len, void *stream);

/* homomorphic_sum (include/GSZ_entry.h:29-32, src/GSZ_entry.cu:456-502): the local operand is the
 * int32 output of homcomp_quant_predict_f32.  cmp_in_size is at most
 * homcomp_ref_cmpsize(homcomp_max_stream_bytes(nbEle), nbEle), the largest value the reference's
 * convention can state (HOMCOMP_ERR_INVALID_ARG beyond): a size stated as the capacity of a
 * buffer laid out for a larger element count is not supported by this entry. */
int homcomp_hom_sum_i32(homcomp_workspace *ws, const unsigned char *d_cmp_in, size_t cmp_in_size,
                        const int32_t *d_local_delta, size_t nbEle, unsigned char *d_cmp_out,
                        uint64_t *d_stream_len, void *stream);

/* Stream (+) stream: the combine stage of src/homcomp.cu:3611-3616 with both operands decoded
 * from streams.  Equals homcomp_hom_sum_f32(a, x) when b = compress(x) with the same eb. */
int homcomp_hom_add(homcomp_workspace *ws, const unsigned char *d_cmp_a, size_t size_a,
                    const unsigned char *d_cmp_b, size_t size_b, size_t nbEle,
                    unsigned char *d_cmp_out, uint64_t *d_stream_len, void *stream);

/* homcomp_hom_sum_f32 for callers that cannot allocate: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
 * wrapper allocates, zeroes and frees six arrays per call, src/GSZ_entry.cu:519-548).  No
 * workspace: the scan words, the incoming stream's tile offsets and the spill area live in one
 * array of about 28.3 MiB inside the library, which every GPU the library runs on holds until
 * the process ends.  The call allocates and frees nothing (the first call on a device looks up
 * the array's address and the kernel's resident grid; make it outside a capture).
 *   - nbEle is at most HOMCOMP_STATIC_MAX_ELEMENTS, else HOMCOMP_ERR_TOO_LARGE.
 *   - d_result (required, device uint64[2]): [0] receives the stream length L, [1] is non-zero
 *     when a wave gave up waiting in the offset scan (the output is then invalid).
 *   - The array is shared by all calls on a GPU and keeps the last call's contents (the call
 *     clears what it needs): two calls that overlap on one GPU race, so issue them on one stream
 *     or order them with events.  Results equal homcomp_hom_sum_f32's byte for byte; the grid is
 *     capped at 224 data workgroups, so calls beyond about 3.6 M elements run below its speed. */
#define HOMCOMP_STATIC_MAX_ELEMENTS ((size_t)1 << 24)
int homcomp_hom_sum_f32_static(const unsigned char *d_cmp_in, size_t cmp_in_size, const float *d_local,
                               size_t nbEle, float eb, unsigned char *d_cmp_out, uint64_t *d_result,
                               void *stream);

/* kernel_quant_prediction (include/homcomp.cuh:2-5, src/homcomp.cu:1553-1602), which callers of
 * the reference launch directly.  Writes nbEle int32 deltas. */
int homcomp_quant_predict_f32(const float *d_data, size_t nbEle, float eb, int32_t *d_delta,
                              void *stream);

/* The min/max scan of src/homcomp_eval.cu:156-163, on the device.  d_minmax: device float[2]. */
int homcomp_range_f32(homcomp_workspace *ws, const float *d_data, size_t nbEle, float *d_minmax,
                      void *stream);
/* src/homcomp_eval.cu:165: eb_abs = fl(rel * fl(max - min)) in float32 (host arithmetic). */
float homcomp_rel_to_abs(float rel, float vmin, float vmax);

/* The blocking read-back of src/GSZ_entry.cu:291 (cudaMemcpy of cmpOffset[gsize-1]): waits for
 * `stream` and returns the length L produced by the last stream-producing call on ws.  Returns
 * HOMCOMP_ERR_SCAN_TIMEOUT if a kernel on ws had to abandon its bounded wait since the previous
 * homcomp_last_size (the output of those calls is incomplete, nothing was written outside the
 * output buffers) and clears that state, so the calls can be repeated on the same workspace. */
int homcomp_last_size(homcomp_workspace *ws, size_t *stream_len, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HOMCOMP_H */
