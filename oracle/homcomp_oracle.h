/*
 * homcomp_oracle.h -- CPU restatement of the HomComp codec (TEST INFRASTRUCTURE ONLY).
 *
 * This is the checker, not the product: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may link or call it.  The shipped library never does.
 *
 * Every function cites the reference lines (relative to /root/reference/HomComp) it
 * restates.  The wire format is independent of the reference's thread mapping
 * (thread-block w, iteration j, lane l  <=>  block index b = w*1024 + j*32 + l), so the
 * restatement walks blocks in ascending b.
 *
 * Pinning status (what fixes each function besides this file itself):
 *   hco_quantize        KATs from the thesis (x=42.683, eb=0.01 -> q=2134), half-way cases,
 *                       float-add round-up case, PTX cvt.rzi semantics; bound invariant.
 *   hco_bit_num         closed form 32-clz, brute force.
 *   block select/pack   thesis block KAT {1,4,0,12,4,3,1,1} -> F=4; hand-derived literal byte
 *                       vectors (tests/golden/handbuilt_blocks.json); exhaustive (fr1,fr2,ob)
 *                       selection against an independent numpy model; decode(encode)=id.
 *   stream scan         exclusive prefix sum vs numpy cumsum of the independent model's sizes.
 *   decompress          decode(encode)=id on ints, dequantisation closed form.
 *   hom sums            integer homomorphism q(A)+q(B), independent numpy model.
 *   plain codec         the hand-derived blocks re-derived without the outlier arm; equals the
 *                       outlier codec's stream wherever no block selects outlier mode and its
 *                       plain arm block by block; independent numpy model; decode(encode)=id.
 * The reference holds no golden vectors and cannot be built here (CUDA + inline PTX, no nvcc),
 * so nothing is pinned by an execution of the reference itself.
 */
#ifndef HOMCOMP_ORACLE_H
#define HOMCOMP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HCO_BLOCK 32u      /* elements per encoded block (src/GSZ.cu:70,82 literals)          */
#define HCO_CHUNK 32768u   /* elements per reference thread-block (include/GSZ.h:4-9: 32*1024) */

/* OpenMP thread control for the CPU-baseline timing (0 = leave the runtime default). */
void hco_set_threads(int n);
int  hco_get_threads(void);

/* src/GSZ.cu:6-25 (C form :1993-1998).  recip = fl(0.5f/eb) (src/GSZ.cu:51). */
int32_t hco_quantize(float x, float recip);
/* src/GSZ.cu:27-31 */
int hco_bit_num(uint32_t x);
/* rate_ofs, src/GSZ.cu:48-50: one header byte per block of the 32768-padded length. */
size_t hco_header_bytes(size_t n);
/* Largest stream any input of n elements can produce: header + 128 B per block. */
size_t hco_max_stream_bytes(size_t n);

/* src/homcomp_eval.cu:156-166: float32 min/max scan and eb_abs = fl(rel * fl(max-min)). */
void  hco_range(const float *x, size_t n, float *mn, float *mx);
float hco_rel_to_abs(float rel, float mn, float mx);

/* Block level (exported for the hand-built vector tests).
 * hco_block_select: src/GSZ.cu:151-164 -> header byte, *size = payload bytes.
 * hco_block_encode: src/GSZ.cu:245-751 -> writes payload, returns its size.
 * hco_block_decode: src/GSZ.cu:883-1424 (without prefix sum / dequantisation). */
uint8_t hco_block_select(const int32_t delta[32], uint32_t *size);
size_t  hco_block_encode(const int32_t delta[32], uint8_t *out, uint8_t *hdr);
uint32_t hco_block_size_from_header(uint8_t hdr);
void    hco_block_decode(uint8_t hdr, const uint8_t *payload, int32_t delta[32]);

/* src/homcomp.cu:1553-1602: Lorenzo deltas of the quantised values, int32.  Elements past n
 * (up to the 32768-padded length) are read as 0.0f; delta must hold the padded length when
 * padded != 0, else n. */
void hco_quant_predict(const float *x, size_t n, float eb, int32_t *delta, int padded);
/* Quantised values only (no Lorenzo), length n. */
void hco_quantize_array(const float *x, size_t n, float eb, int32_t *q);

/* src/GSZ.cu:33-756 + src/GSZ_entry.cu:263-301.  *stream_len = true length L (header
 * included).  block_ofs (optional, padded_blocks+1 entries, uint64) receives the absolute
 * byte offset of every block's payload. Returns 0 on success. */
int hco_compress(const float *x, size_t n, float eb, uint8_t *cmp, size_t *stream_len,
                 uint64_t *block_ofs);
/* The plain codec (no outlier mode): src/GSZ.cu:1475-1748 (compress) and :1750-1991 (decompress),
 * wrappers src/GSZ_entry.cu:150-228.  The header byte of a block is the bit width of its largest
 * |delta|; the payload is the sign word and that many planes, or nothing for a zero block.  The
 * reference's wrapper reports cmpOffset[gsize-1] + header bytes as cmpSize, which leaves out the
 * payload of the last 32768-element chunk; *stream_len here is the true length. */
int hco_compress_plain(const float *x, size_t n, float eb, uint8_t *cmp, size_t *stream_len);
int hco_decompress_plain(const uint8_t *cmp, size_t n, float eb, float *out);
size_t hco_block_encode_plain(const int32_t delta[32], uint8_t *out, uint8_t *hdr);
/* Same back end fed with ready-made deltas (length n, zero padded). */
int hco_encode_deltas(const int32_t *delta, size_t n, uint8_t *cmp, size_t *stream_len);

/* src/GSZ.cu:758-1473 + src/GSZ_entry.cu:317-350.  Blocks whose payload offset is >= cmp_size
 * are skipped (src/GSZ.cu:908-911); skipped and rate-0 blocks come out as 0.0f, which is what
 * the reference leaves in a pre-zeroed output buffer. */
int hco_decompress(const uint8_t *cmp, size_t cmp_size, size_t n, float eb, float *out);
/* Decoded signed deltas / quantised values (length n). */
int hco_decode_deltas(const uint8_t *cmp, size_t cmp_size, size_t n, int32_t *delta);
int hco_decode_quants(const uint8_t *cmp, size_t cmp_size, size_t n, int32_t *q);

/* src/homcomp.cu:2923-4311 + src/GSZ_entry.cu:504-550: stream (+) local floats. */
int hco_hom_sum_f32(const uint8_t *cmp_in, size_t cmp_in_size, const float *local, size_t n,
                    float eb, uint8_t *cmp_out, size_t *stream_len);
/* src/homcomp.cu:1604-2921 + src/GSZ_entry.cu:456-502: stream (+) precomputed int deltas. */
int hco_hom_sum_i32(const uint8_t *cmp_in, size_t cmp_in_size, const int32_t *local_delta,
                    size_t n, uint8_t *cmp_out, size_t *stream_len);
/* stream (+) stream: the same combine stage with the local deltas decoded from a second
 * stream instead of quantised from floats. */
int hco_hom_add(const uint8_t *cmp_a, size_t size_a, const uint8_t *cmp_b, size_t size_b,
                size_t n, uint8_t *cmp_out, size_t *stream_len);

#ifdef __cplusplus
}
#endif
#endif
