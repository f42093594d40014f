/*
 * homcomp_oracle.c -- CPU restatement of the HomComp codec (TEST INFRASTRUCTURE ONLY).
 *
 * See homcomp_oracle.h for scope, citations and the pinning status of each function.
 * Build: gcc -O3 -ffp-contract=off -fopenmp -shared -fPIC (FMA contraction must stay off:
 * the reference quantiser rounds the product and the sum separately, src/GSZ.cu:13,17).
 *
 * Structure: every stream-producing entry point runs the same two passes over
 * 32768-element chunks (the reference thread-block's share, include/GSZ.h:4-9):
 *   pass 1  produce each block's 32 signed deltas -> rate selection -> header byte, byte total
 *   scan    exclusive prefix sum of the chunk totals (src/GSZ.cu:170-239)
 *   pass 2  produce the deltas again and bit-plane pack them at the scanned offsets
 * Only the delta producer differs between compress and the homomorphic sums.
 */
#include "homcomp_oracle.h"

#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define BLOCKS_PER_CHUNK (HCO_CHUNK / HCO_BLOCK) /* 1024 */

static int g_threads = 0;

void hco_set_threads(int n) { g_threads = n; }

int hco_get_threads(void)
{
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

#ifdef _OPENMP
#define HCO_PARALLEL_FOR _Pragma("omp parallel for schedule(static) num_threads(hco_get_threads())")
#else
#define HCO_PARALLEL_FOR
#endif

/* ------------------------------------------------------------------ scalars */

/* src/GSZ.cu:6-25.  mul.f32, setp.ge, add.f32, cvt.rzi.s32.f32 (saturating, NaN -> 0), sub.s32. */
int32_t hco_quantize(float x, float recip)
{
    volatile float d = x * recip;       /* :13, rounded to float32 */
    int s = (d >= -0.5f) ? 0 : 1;       /* :14-16, NaN compares false -> s = 1 */
    volatile float t = d + 0.5f;        /* :17, second rounding */
    int32_t r;
    if (t != t)
        r = 0;                          /* :18, cvt of NaN gives 0 */
    else if (t >= 2147483648.0f)
        r = INT32_MAX;                  /* saturation */
    else if (t <= -2147483648.0f)
        r = INT32_MIN;
    else
        r = (int32_t)t;                 /* round toward zero */
    return (int32_t)((uint32_t)r - (uint32_t)s); /* :20, wrapping subtract */
}

/* src/GSZ.cu:27-31: 32 - clz(x), 0 for x == 0. */
int hco_bit_num(uint32_t x)
{
    int n = 0;
    while (x) {
        n++;
        x >>= 1;
    }
    return n;
}

static size_t chunks_of(size_t n) { return (n + HCO_CHUNK - 1) / HCO_CHUNK; }

/* src/GSZ.cu:48-50 */
size_t hco_header_bytes(size_t n) { return chunks_of(n) * BLOCKS_PER_CHUNK; }

size_t hco_max_stream_bytes(size_t n)
{
    size_t blocks = hco_header_bytes(n);
    return blocks + blocks * 128u;
}

/* src/homcomp_eval.cu:156-163 */
void hco_range(const float *x, size_t n, float *mn, float *mx)
{
    float lo = n ? x[0] : 0.0f, hi = lo;
    for (size_t i = 0; i < n; i++) {
        if (x[i] > hi)
            hi = x[i];
        else if (x[i] < lo)
            lo = x[i];
    }
    *mn = lo;
    *mx = hi;
}

/* src/homcomp_eval.cu:165: eb = eb * (max_val - min_val), all float32. */
float hco_rel_to_abs(float rel, float mn, float mx)
{
    volatile float range = mx - mn;
    volatile float eb = rel * range;
    return eb;
}

/* ------------------------------------------------------------------ one block */

typedef struct {
    uint32_t a[32];   /* |delta| */
    uint32_t sign;    /* bit (31-i) = delta_i < 0, src/GSZ.cu:93 */
    int outlier_mode; /* header bit 7 */
    int F;            /* planes, header bits 0-4 */
    int ob;           /* outlier bytes, header bits 5-6 hold ob-1 */
    uint32_t size;    /* payload bytes */
    uint8_t hdr;
} hco_blk;

/* Bit widths are capped at 31: the 5-bit header field cannot hold 32.  |delta| = 2^31 only
 * arises from saturated quantisation (outside the codec's domain); the cap keeps the stream
 * self-consistent there. */
static int planes_of(uint32_t m)
{
    int b = hco_bit_num(m);
    return b > 31 ? 31 : b;
}

/* src/GSZ.cu:86-164: sign map, absolute values, the two maxima, rate selection.
 * plain != 0: the plain codec of src/GSZ.cu:1475-1748, whose only rate is the bit width of the
 * block maximum (:1578-1581) -- the first arm below, always. */
static void blk_analyse(const int32_t d[32], hco_blk *k, int plain)
{
    uint32_t max1 = 0, max2 = 0;
    k->sign = 0;
    for (int i = 0; i < 32; i++) {
        uint32_t neg = d[i] < 0;
        uint32_t a = neg ? (uint32_t)0 - (uint32_t)d[i] : (uint32_t)d[i];
        k->sign |= neg << (31 - i);
        k->a[i] = a;
        if (a > max1)
            max1 = a;
        if (i && a > max2)
            max2 = a;
    }
    int fr1 = planes_of(max1);                      /* :152 */
    int fr2 = planes_of(max2);                      /* :153 */
    int ob = (hco_bit_num(k->a[0]) + 7) / 8;        /* :154 */
    uint32_t sz1 = fr1 ? 4u + 4u * (uint32_t)fr1 : 0u;   /* :156 */
    uint32_t sz2 = 4u + 4u * (uint32_t)fr2 + (uint32_t)ob; /* :157, both arms */
    if (plain || sz1 <= sz2) {                      /* :158-160; plain codec: :1578-1581 */
        k->outlier_mode = 0;
        k->F = fr1;
        k->ob = 0;
        k->size = sz1;
        k->hdr = (uint8_t)fr1;
    } else {                                        /* :161-164 */
        k->outlier_mode = 1;
        k->F = fr2;
        k->ob = ob;
        k->size = sz2;
        k->hdr = (uint8_t)(fr2 | 0x80 | ((ob - 1) << 5));
    }
}

/* src/GSZ.cu:245-751.  The four alignment cases there (vec_ofs 0..3) emit the same byte
 * sequence; it is produced here byte by byte. */
static size_t blk_pack(const hco_blk *k, uint8_t *out)
{
    size_t n = 0;
    if (k->outlier_mode) {
        uint32_t a0 = k->a[0];
        for (int i = 0; i < k->ob; i++) {           /* :271-275, little-endian */
            out[n++] = (uint8_t)(a0 & 0xff);
            a0 >>= 8;
        }
    } else if (k->F == 0) {
        return 0;                                   /* :287 zero block */
    }
    out[n++] = (uint8_t)(k->sign >> 24);            /* :292-295 / :279-282 */
    out[n++] = (uint8_t)(k->sign >> 16);
    out[n++] = (uint8_t)(k->sign >> 8);
    out[n++] = (uint8_t)(k->sign);
    for (int p = 0; p < k->F; p++) {                /* :301-357, plane p = bit p */
        for (int byte = 0; byte < 4; byte++) {
            uint32_t v = 0;
            for (int m = 0; m < 8; m++) {
                int e = byte * 8 + m;
                uint32_t bit = (k->a[e] >> p) & 1u;
                if (e == 0 && k->outlier_mode)
                    bit = 0;                        /* :274 leaves a0 = 0; :311-313 */
                v |= bit << (7 - m);
            }
            out[n++] = (uint8_t)v;
        }
    }
    return n;
}

uint32_t hco_block_size_from_header(uint8_t hdr)
{
    /* src/GSZ.cu:795-802 */
    int sel = hdr >> 7;
    uint32_t ob = ((hdr & 0x60u) >> 5) + 1u;
    uint32_t F = hdr & 0x1fu;
    if (!sel)
        return F ? 4u + 4u * F : 0u;
    return 4u + 4u * F + ob;
}

uint8_t hco_block_select(const int32_t delta[32], uint32_t *size)
{
    hco_blk k;
    blk_analyse(delta, &k, 0);
    if (size)
        *size = k.size;
    return k.hdr;
}

size_t hco_block_encode(const int32_t delta[32], uint8_t *out, uint8_t *hdr)
{
    hco_blk k;
    blk_analyse(delta, &k, 0);
    if (hdr)
        *hdr = k.hdr;
    return blk_pack(&k, out);
}

size_t hco_block_encode_plain(const int32_t delta[32], uint8_t *out, uint8_t *hdr)
{
    hco_blk k;
    blk_analyse(delta, &k, 1);
    if (hdr)
        *hdr = k.hdr;
    return blk_pack(&k, out);
}

/* src/GSZ.cu:883-1424 up to the signed deltas (lorenQuant), i.e. without the running sum and
 * the dequantisation of :1426-1468. */
void hco_block_decode(uint8_t hdr, const uint8_t *in, int32_t delta[32])
{
    int sel = hdr >> 7;
    int ob = ((hdr & 0x60) >> 5) + 1;
    int F = hdr & 0x1f;
    uint32_t a[32];
    memset(a, 0, sizeof a);
    if (!sel && F == 0) {
        memset(delta, 0, 32 * sizeof(int32_t));
        return;
    }
    size_t n = 0;
    uint32_t outlier = 0;
    if (sel)
        for (int i = 0; i < ob; i++)                /* :913-917 */
            outlier |= (uint32_t)in[n++] << (8 * i);
    uint32_t sign = ((uint32_t)in[n] << 24) | ((uint32_t)in[n + 1] << 16) |
                    ((uint32_t)in[n + 2] << 8) | (uint32_t)in[n + 3]; /* :921-924, :990-994 */
    n += 4;
    for (int p = 0; p < F; p++) {                   /* :998-1044 */
        for (int byte = 0; byte < 4; byte++) {
            uint32_t v = in[n++];
            for (int m = 0; m < 8; m++) {
                int e = byte * 8 + m;
                if (e == 0 && sel)
                    continue;                       /* :1005-1006 */
                a[e] |= ((v >> (7 - m)) & 1u) << p;
            }
        }
    }
    if (sel)
        a[0] = outlier;                             /* :986-987 */
    for (int i = 0; i < 32; i++) {                  /* :1432-1434 */
        uint32_t neg = (sign >> (31 - i)) & 1u;
        delta[i] = (int32_t)(neg ? (uint32_t)0 - a[i] : a[i]);
    }
}

/* ------------------------------------------------------------------ delta producers */

typedef struct {
    uint64_t *chunk_ofs; /* absolute payload offset of each chunk's first block */
    const uint8_t *cmp;
    size_t cmp_size;
} hco_instream;

typedef struct {
    const float *x;      /* local floats, quantised on the fly (hom_sum_F, compress) */
    const int32_t *d;    /* or ready-made deltas (hom_sum, encode_deltas)            */
    size_t n;
    float recip;
    int n_in;            /* incoming streams to decode and add (0, 1 or 2)           */
    int plain;           /* encode with the plain codec (no outlier mode)            */
    hco_instream in[2];
} hco_src;

/* src/GSZ.cu:170-239 on the decoder side (:790-874): per-chunk totals from the header bytes,
 * then an exclusive scan; chunk 0 starts right after the header (excl_sum = 0 there). */
static int instream_open(hco_instream *s, const uint8_t *cmp, size_t cmp_size, size_t n)
{
    size_t nc = chunks_of(n);
    s->cmp = cmp;
    s->cmp_size = cmp_size;
    s->chunk_ofs = (uint64_t *)malloc((nc + 1) * sizeof(uint64_t));
    if (!s->chunk_ofs)
        return -1;
    HCO_PARALLEL_FOR
    for (size_t c = 0; c < nc; c++) {
        uint64_t t = 0;
        for (size_t b = 0; b < BLOCKS_PER_CHUNK; b++)
            t += hco_block_size_from_header(cmp[c * BLOCKS_PER_CHUNK + b]);
        s->chunk_ofs[c + 1] = t;
    }
    s->chunk_ofs[0] = hco_header_bytes(n);
    for (size_t c = 0; c < nc; c++)
        s->chunk_ofs[c + 1] += s->chunk_ofs[c];
    return 0;
}

static void instream_close(hco_instream *s)
{
    free(s->chunk_ofs);
    s->chunk_ofs = NULL;
}

/* Decode block b of an incoming stream whose payload sits at *ofs; advances *ofs.
 * Out-of-bound rule: src/GSZ.cu:908-911 / src/homcomp.cu:3081-3084.  A zero header or a
 * skipped block contributes zero deltas (the intended meaning; the reference leaves stale
 * registers there, src/homcomp.cu:3086,3149). */
static void instream_block(const hco_instream *s, size_t b, uint64_t *ofs, int32_t d[32])
{
    uint8_t hdr = s->cmp[b];
    uint32_t sz = hco_block_size_from_header(hdr);
    if (sz == 0 || *ofs >= s->cmp_size)
        memset(d, 0, 32 * sizeof(int32_t));
    else
        hco_block_decode(hdr, s->cmp + *ofs, d);
    *ofs += sz;
}

/* Local contribution of block b: src/GSZ.cu:82-149 (quantise + Lorenzo with prevQuant = 0 at
 * the block start) or the stored deltas of src/homcomp.cu:2252-2268.  Elements past n read
 * as 0.0f / 0 (what the reference sees in a zero-padded buffer). */
static void local_block(const hco_src *s, size_t b, int32_t d[32])
{
    size_t base = b * HCO_BLOCK;
    if (s->x) {
        int32_t prev = 0;
        for (int i = 0; i < 32; i++) {
            size_t e = base + (size_t)i;
            float v = e < s->n ? s->x[e] : 0.0f;
            int32_t q = hco_quantize(v, s->recip);
            d[i] = (int32_t)((uint32_t)q - (uint32_t)prev);
            prev = q;
        }
    } else if (s->d) {
        for (int i = 0; i < 32; i++) {
            size_t e = base + (size_t)i;
            d[i] = e < s->n ? s->d[e] : 0;
        }
    } else {
        memset(d, 0, 32 * sizeof(int32_t));
    }
}

/* src/homcomp.cu:3611-3616 (and :2252-2268): delta_out = delta_in + delta_local. */
static void produce_block(const hco_src *s, size_t b, uint64_t ofs[2], int32_t d[32])
{
    local_block(s, b, d);
    for (int k = 0; k < s->n_in; k++) {
        int32_t t[32];
        instream_block(&s->in[k], b, &ofs[k], t);
        for (int i = 0; i < 32; i++)
            d[i] = (int32_t)((uint32_t)d[i] + (uint32_t)t[i]);
    }
}

/* ------------------------------------------------------------------ the two passes */

static int run_encode(const hco_src *s, size_t n, uint8_t *cmp, size_t *stream_len,
                      uint64_t *block_ofs)
{
    size_t nc = chunks_of(n);
    size_t hdr_bytes = hco_header_bytes(n);
    if (nc == 0) {
        *stream_len = 0;
        if (block_ofs)
            block_ofs[0] = 0;
        return 0;
    }
    uint64_t *excl = (uint64_t *)malloc((nc + 1) * sizeof(uint64_t));
    if (!excl)
        return -1;

    /* pass 1: src/GSZ.cu:68-169 */
    HCO_PARALLEL_FOR
    for (size_t c = 0; c < nc; c++) {
        uint64_t ofs[2] = {0, 0};
        for (int k = 0; k < s->n_in; k++)
            ofs[k] = s->in[k].chunk_ofs[c];
        uint64_t total = 0;
        for (size_t j = 0; j < BLOCKS_PER_CHUNK; j++) {
            size_t b = c * BLOCKS_PER_CHUNK + j;
            int32_t d[32];
            hco_blk k;
            produce_block(s, b, ofs, d);
            blk_analyse(d, &k, s->plain);
            cmp[b] = k.hdr;                         /* :167 */
            total += k.size;
        }
        excl[c + 1] = total;
    }
    /* scan: src/GSZ.cu:170-239; chunk 0's exclusive prefix is 0 */
    excl[0] = hdr_bytes;                            /* :238 base_idx = excl_sum + rate_ofs */
    for (size_t c = 0; c < nc; c++)
        excl[c + 1] += excl[c];

    /* pass 2: src/GSZ.cu:241-751 */
    HCO_PARALLEL_FOR
    for (size_t c = 0; c < nc; c++) {
        uint64_t ofs[2] = {0, 0};
        for (int k = 0; k < s->n_in; k++)
            ofs[k] = s->in[k].chunk_ofs[c];
        uint64_t o = excl[c];
        for (size_t j = 0; j < BLOCKS_PER_CHUNK; j++) {
            size_t b = c * BLOCKS_PER_CHUNK + j;
            int32_t d[32];
            hco_blk k;
            produce_block(s, b, ofs, d);
            blk_analyse(d, &k, s->plain);
            if (block_ofs)
                block_ofs[b] = o;
            o += blk_pack(&k, cmp + o);
        }
    }
    *stream_len = (size_t)excl[nc];                 /* :752-755, the absolute end offset */
    if (block_ofs)
        block_ofs[nc * BLOCKS_PER_CHUNK] = excl[nc];
    free(excl);
    return 0;
}

/* ------------------------------------------------------------------ entry points */

static float recip_of(float eb)
{
    volatile float r = 0.5f / eb;                   /* src/GSZ.cu:51 */
    return r;
}

void hco_quantize_array(const float *x, size_t n, float eb, int32_t *q)
{
    float r = recip_of(eb);
    HCO_PARALLEL_FOR
    for (size_t i = 0; i < n; i++)
        q[i] = hco_quantize(x[i], r);
}

void hco_quant_predict(const float *x, size_t n, float eb, int32_t *delta, int padded)
{
    hco_src s;
    memset(&s, 0, sizeof s);
    s.x = x;
    s.n = n;
    s.recip = recip_of(eb);
    size_t total = padded ? chunks_of(n) * HCO_CHUNK : n;
    size_t blocks = (total + HCO_BLOCK - 1) / HCO_BLOCK;
    HCO_PARALLEL_FOR
    for (size_t b = 0; b < blocks; b++) {
        int32_t d[32];
        local_block(&s, b, d);
        for (int i = 0; i < 32; i++)
            if (b * HCO_BLOCK + (size_t)i < total)
                delta[b * HCO_BLOCK + (size_t)i] = d[i];
    }
}

int hco_compress(const float *x, size_t n, float eb, uint8_t *cmp, size_t *stream_len,
                 uint64_t *block_ofs)
{
    hco_src s;
    memset(&s, 0, sizeof s);
    s.x = x;
    s.n = n;
    s.recip = recip_of(eb);
    return run_encode(&s, n, cmp, stream_len, block_ofs);
}

/* src/GSZ.cu:1475-1748 + src/GSZ_entry.cu:150-190: the plain codec. */
int hco_compress_plain(const float *x, size_t n, float eb, uint8_t *cmp, size_t *stream_len)
{
    hco_src s;
    memset(&s, 0, sizeof s);
    s.x = x;
    s.n = n;
    s.recip = recip_of(eb);
    s.plain = 1;
    return run_encode(&s, n, cmp, stream_len, NULL);
}

int hco_encode_deltas(const int32_t *delta, size_t n, uint8_t *cmp, size_t *stream_len)
{
    hco_src s;
    memset(&s, 0, sizeof s);
    s.d = delta;
    s.n = n;
    return run_encode(&s, n, cmp, stream_len, NULL);
}

int hco_hom_sum_f32(const uint8_t *cmp_in, size_t cmp_in_size, const float *local, size_t n,
                    float eb, uint8_t *cmp_out, size_t *stream_len)
{
    hco_src s;
    memset(&s, 0, sizeof s);
    s.x = local;
    s.n = n;
    s.recip = recip_of(eb);
    s.n_in = 1;
    if (instream_open(&s.in[0], cmp_in, cmp_in_size, n))
        return -1;
    int rc = run_encode(&s, n, cmp_out, stream_len, NULL);
    instream_close(&s.in[0]);
    return rc;
}

int hco_hom_sum_i32(const uint8_t *cmp_in, size_t cmp_in_size, const int32_t *local_delta,
                    size_t n, uint8_t *cmp_out, size_t *stream_len)
{
    hco_src s;
    memset(&s, 0, sizeof s);
    s.d = local_delta;
    s.n = n;
    s.n_in = 1;
    if (instream_open(&s.in[0], cmp_in, cmp_in_size, n))
        return -1;
    int rc = run_encode(&s, n, cmp_out, stream_len, NULL);
    instream_close(&s.in[0]);
    return rc;
}

int hco_hom_add(const uint8_t *cmp_a, size_t size_a, const uint8_t *cmp_b, size_t size_b,
                size_t n, uint8_t *cmp_out, size_t *stream_len)
{
    hco_src s;
    memset(&s, 0, sizeof s);
    s.n = n;
    s.n_in = 2;
    if (instream_open(&s.in[0], cmp_a, size_a, n))
        return -1;
    if (instream_open(&s.in[1], cmp_b, size_b, n)) {
        instream_close(&s.in[0]);
        return -1;
    }
    int rc = run_encode(&s, n, cmp_out, stream_len, NULL);
    instream_close(&s.in[0]);
    instream_close(&s.in[1]);
    return rc;
}

/* mode 0: signed deltas, 1: quantised values (running sum, src/GSZ.cu:1435-1436),
 * 2: floats x' = fl(fl((float)q * eb) * 2) (src/GSZ.cu:1437). */
static int run_decode(const uint8_t *cmp, size_t cmp_size, size_t n, float eb, int mode,
                      void *out)
{
    hco_instream in;
    size_t nc = chunks_of(n);
    if (nc == 0)
        return 0;
    if (instream_open(&in, cmp, cmp_size, n))
        return -1;
    HCO_PARALLEL_FOR
    for (size_t c = 0; c < nc; c++) {
        uint64_t ofs = in.chunk_ofs[c];
        for (size_t j = 0; j < BLOCKS_PER_CHUNK; j++) {
            size_t b = c * BLOCKS_PER_CHUNK + j;
            int32_t d[32];
            instream_block(&in, b, &ofs, d);
            int32_t q = 0;
            for (int i = 0; i < 32; i++) {
                size_t e = b * HCO_BLOCK + (size_t)i;
                q = (int32_t)((uint32_t)q + (uint32_t)d[i]);
                if (e >= n)
                    break;
                if (mode == 0) {
                    ((int32_t *)out)[e] = d[i];
                } else if (mode == 1) {
                    ((int32_t *)out)[e] = q;
                } else {
                    volatile float t = (float)q * eb;
                    volatile float v = t * 2.0f;
                    ((float *)out)[e] = v;
                }
            }
        }
    }
    instream_close(&in);
    return 0;
}

int hco_decompress(const uint8_t *cmp, size_t cmp_size, size_t n, float eb, float *out)
{
    return run_decode(cmp, cmp_size, n, eb, 2, out);
}

int hco_decode_deltas(const uint8_t *cmp, size_t cmp_size, size_t n, int32_t *delta)
{
    return run_decode(cmp, cmp_size, n, 0.0f, 0, delta);
}

int hco_decode_quants(const uint8_t *cmp, size_t cmp_size, size_t n, int32_t *q)
{
    return run_decode(cmp, cmp_size, n, 0.0f, 1, q);
}

/* src/GSZ.cu:1750-1991 + src/GSZ_entry.cu:192-228: the plain decoder.  A header byte is a plane
 * count and nothing else (:1783-1784); offsets are the prefix sums of 4 + 4 * F per non-empty
 * block (:1784, :1867-1880); there is no out-of-bound rule; a block is the sign word (:1887-1891)
 * and F planes (:1897-1960), then the running sum and the dequantisation (:1963-1986).  Rate-0
 * blocks come out as 0.0f (the reference leaves them unwritten). */
int hco_decompress_plain(const uint8_t *cmp, size_t n, float eb, float *out)
{
    size_t nc = chunks_of(n);
    if (nc == 0)
        return 0;
    uint64_t *excl = (uint64_t *)malloc((nc + 1) * sizeof(uint64_t));
    if (!excl)
        return -1;
    HCO_PARALLEL_FOR
    for (size_t c = 0; c < nc; c++) {
        uint64_t total = 0;
        for (size_t j = 0; j < BLOCKS_PER_CHUNK; j++) {
            uint32_t F = cmp[c * BLOCKS_PER_CHUNK + j];
            total += F ? 4u + 4u * F : 0u;
        }
        excl[c + 1] = total;
    }
    excl[0] = hco_header_bytes(n);
    for (size_t c = 0; c < nc; c++)
        excl[c + 1] += excl[c];
    HCO_PARALLEL_FOR
    for (size_t c = 0; c < nc; c++) {
        uint64_t o = excl[c];
        for (size_t j = 0; j < BLOCKS_PER_CHUNK; j++) {
            size_t b = c * BLOCKS_PER_CHUNK + j;
            uint32_t F = cmp[b];
            uint32_t a[32];
            uint32_t sign = 0;
            memset(a, 0, sizeof a);
            if (F) {
                const uint8_t *in = cmp + o;
                sign = ((uint32_t)in[0] << 24) | ((uint32_t)in[1] << 16) | ((uint32_t)in[2] << 8) | (uint32_t)in[3];
                for (uint32_t p = 0; p < F; p++)
                    for (int byte = 0; byte < 4; byte++) {
                        uint32_t v = in[4 + 4 * p + (uint32_t)byte];
                        for (int m = 0; m < 8; m++)
                            if (p < 32)
                                a[byte * 8 + m] |= ((v >> (7 - m)) & 1u) << p;
                    }
                o += 4u + 4u * F;
            }
            int32_t q = 0;
            for (int i = 0; i < 32; i++) {
                size_t e = b * HCO_BLOCK + (size_t)i;
                uint32_t d = (sign >> (31 - i)) & 1u ? (uint32_t)0 - a[i] : a[i];
                q = (int32_t)((uint32_t)q + d);
                if (e >= n)
                    break;
                volatile float t = (float)q * eb;
                volatile float v = t * 2.0f;
                out[e] = v;
            }
        }
    }
    free(excl);
    return 0;
}
