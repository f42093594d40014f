// TEST INFRASTRUCTURE: runs the HomComp kernels' source on the CPU (execution model in
// amdgcn_emu.hpp) on small inputs, so that their logic and address arithmetic can be compared
// with the oracle without a GPU.  One run = one operation:
//
//   emu_main OP N EB DATA_GROUPS BUDGET KIND SLOTS PLAIN IN_A IN_B OUT [OFS_OUT [STATED_A [STATED_B]]]
//
//   OP           compress | decompress | hom_sum_f32 | hom_sum_i32 | hom_add | quant_predict | value_range
//                (the last two take the float32 values in IN_A and use N and, quant_predict, EB only;
//                DATA_GROUPS is value_range's grid)
//   N, EB        element count, absolute error bound
//   DATA_GROUPS  data workgroups of four waves (the persistent grid; the scan server is added)
//   BUDGET       LDS bytes per data wave for packed tiles (cut into SLOTS slots)
//   KIND         0 general path only, 1 kernel with the few-plane path, 2 stream (+) stream kernel for wide blocks
//   IN_A, IN_B   raw files: float32 values / stream bytes / int32 deltas as the operation takes them ("-" where none);
//                a stream's stated size is its file size unless STATED_A/B says otherwise
//   OUT          raw file: the stream (its true length), the float32 values, the int32 deltas, or minimum and maximum
//   OFS_OUT      optional raw file: the tile offsets the producing call leaves (uint64 each)
//   STATED_A/B   optional: the size stated for an incoming stream where it is less than its file's (the file is what the
//                buffer holds: blocks that start below the stated size are read in full)
//
// Memory lives in shared mappings created before the workgroups are forked, each buffer between
// two inaccessible pages and ending at the upper one, so a plain access beyond a buffer is a
// segmentation fault of the run, and every buffer-descriptor access is checked against the list
// of buffers (emu_check).
#include <string>
#include <vector>

#define EMU_DYN_LDS (4 * 2 * (8192 + 64))
#define EMU_DEFINE_GLOBALS
#include "hip/hip_runtime.h"

#include "_gen/homcomp_device.hpp"
#include "_gen/homcomp_kernels.inc"

namespace {

uint8_t *device_alloc(size_t bytes, const char *name, size_t align = 256)
{
    uint8_t *p = (uint8_t *)emu_device_alloc_named(bytes, name, align);
    if (!p) {
        perror("mmap");
        exit(2);
    }
    memset(p, 0, bytes);
    return p;
}

std::vector<uint8_t> read_file(const char *path)
{
    std::vector<uint8_t> v;
    if (std::string(path) == "-") return v;
    FILE *f = fopen(path, "rb");
    if (!f) {
        perror(path);
        exit(2);
    }
    fseek(f, 0, SEEK_END);
    v.resize((size_t)ftell(f));
    rewind(f);
    if (!v.empty() && fread(v.data(), 1, v.size(), f) != v.size()) exit(2);
    fclose(f);
    return v;
}

void write_file(const char *path, const void *p, size_t bytes)
{
    FILE *f = fopen(path, "wb");
    if (!f || (bytes && fwrite(p, 1, bytes, f) != bytes)) {
        perror(path);
        exit(2);
    }
    fclose(f);
}

struct Launch {
    void (*kernel)(const void *);
    const void *args;
};

void run_grid(const Launch &l, unsigned gx, unsigned gy, unsigned threads, size_t dyn_lds = 0)
{
    const std::function<void()> body = [=]() { l.kernel(l.args); };
    if (!emu_run_grid(body, emu_dim3(gx, gy), emu_dim3(threads), dyn_lds)) exit(4);
}

template <int NIN, int LOCAL, int OUT, int BITPLANE>
void wave_kernel(const void *a)
{
    hc::k_wave<NIN, LOCAL, OUT, BITPLANE>(*(const hc::TileParams *)a);
}

struct OffsetsCall {
    hc::InOffsetsArgs a;
    uint32_t n_tiles;
    uint64_t base;
    uint32_t epoch, spin_limit;
};
void offsets_kernel(const void *p)
{
    const OffsetsCall *c = (const OffsetsCall *)p;
    hc::k_in_offsets(c->a, c->n_tiles, c->base, c->epoch, c->spin_limit);
}

struct QuantCall {
    const float *x;
    int32_t *out;
    uint64_t n;
    float recip;
};
void quant_kernel(const void *p)
{
    const QuantCall *c = (const QuantCall *)p;
    hc::k_quant_predict(c->x, c->out, c->n, c->recip);
}
struct RangeCall {
    const float *x;
    uint64_t n;
    float *partial;
    uint32_t partials;
    float *out;
};
void range_partial_kernel(const void *p)
{
    const RangeCall *c = (const RangeCall *)p;
    hc::k_range_partial(c->x, c->n, c->partial);
}
void range_final_kernel(const void *p)
{
    const RangeCall *c = (const RangeCall *)p;
    hc::k_range_final(c->partial, c->partials, c->out);
}

size_t header_bytes(size_t n) { return (n + 32767) / 32768 * 1024; }

// the two kernels that work on plain arrays
int run_array_op(const std::string &op, size_t n, float eb, unsigned groups, const std::vector<uint8_t> &in, const char *out_path)
{
    if (in.size() != n * 4) {
        fprintf(stderr, "values: %zu bytes for %zu elements\n", in.size(), n);
        return 1;
    }
    float *x = (float *)device_alloc(n * 4, "values", 16);
    memcpy(x, in.data(), n * 4);
    if (op == "quant_predict") {
        QuantCall c{x, (int32_t *)device_alloc(n * 4, "deltas", 16), n, 0.5f / eb};
        for (size_t i = 0; i < n; ++i) c.out[i] = 12345;
        const uint64_t lanes = (n + 7) / 8;
        run_grid(Launch{quant_kernel, &c}, (unsigned)((lanes + 255) / 256), 1, 256);
        write_file(out_path, c.out, n * 4);
        return 0;
    }
    uint64_t want = (n / 4 + 255) / 256;
    if (want < 1) want = 1;
    const unsigned grid = (unsigned)(want < groups ? want : groups);
    RangeCall c{x, n, (float *)device_alloc((size_t)grid * 8, "partials", 8), grid, (float *)device_alloc(8, "range", 8)};
    run_grid(Launch{range_partial_kernel, &c}, grid, 1, 256);
    run_grid(Launch{range_final_kernel, &c}, 1, 1, 256);
    write_file(out_path, c.out, 8);
    return 0;
}

}  // namespace

int main(int argc, char **argv)
{
    if (argc < 12) {
        fprintf(stderr, "usage: %s OP N EB DATA_GROUPS BUDGET KIND SLOTS PLAIN IN_A IN_B OUT [OFS_OUT [STATED_A [STATED_B]]]\n", argv[0]);
        return 1;
    }
    const std::string op = argv[1];
    const size_t n = strtoull(argv[2], nullptr, 10);
    const float eb = strtof(argv[3], nullptr);
    const unsigned groups = (unsigned)atoi(argv[4]);
    const unsigned budget = (unsigned)atoi(argv[5]);
    const unsigned kind = (unsigned)atoi(argv[6]);
    const unsigned slots = (unsigned)atoi(argv[7]);
    const unsigned plain = (unsigned)atoi(argv[8]);
    const std::vector<uint8_t> in_a = read_file(argv[9]), in_b = read_file(argv[10]);
    const char *out_path = argv[11];
    const char *ofs_path = argc > 12 && std::string(argv[12]) != "-" ? argv[12] : nullptr;
    const size_t stated[2] = {argc > 13 ? strtoull(argv[13], nullptr, 10) : in_a.size(), argc > 14 ? strtoull(argv[14], nullptr, 10) : in_b.size()};

    if (op == "quant_predict" || op == "value_range") return n && groups ? run_array_op(op, n, eb, groups, in_a, out_path) : 1;

    const size_t hdr = header_bytes(n);
    const size_t padded = hdr * 32;
    const uint32_t n_tiles = (uint32_t)(padded / 4096);
    const size_t cap = hdr + hdr * 132 + 64;   // the plain codec's largest block has 4 + 4 * 32 bytes
    const bool enc = op != "decompress";
    const int n_in = op == "hom_add" ? 2 : (op == "compress" ? 0 : 1);
    if (!n || !groups || slots < 2 || slots > 4 || budget % 64 || budget > 2 * (8192 + 64)) return 1;

    hc::TileParams p;
    memset(&p, 0, sizeof p);
    p.n = n;
    p.hdr_bytes = hdr;
    p.n_tiles = n_tiles;
    p.eb = eb;
    p.recip = 0.5f / eb;
    p.epoch = 7;
    p.spin_limit = 1u << 30;
    if (const char *e = getenv("EMU_SPIN_LIMIT")) p.spin_limit = (uint32_t)strtoul(e, nullptr, 10);   // looks a wait may take (a test of the bounded waits)
    p.out_slots = slots;
    p.sliced = kind;
    p.plain = plain;
    p.stage_bytes = budget;
    // What an earlier call on the same workspace leaves behind: status words of the epoch before
    // (totals and prefixes that look finished but are not this call's), a used spill area, old offsets.
    auto stale_words = [](uint64_t *w, size_t count, uint32_t epoch) {
        for (size_t i = 0; i < count; ++i) w[i] = hc::status_word(epoch, 1u + (uint32_t)(i & 1u), 0x123456789ull * (i + 1));
    };
    uint64_t *words = (uint64_t *)device_alloc(2 * (size_t)n_tiles * 8, "scan words");
    stale_words(words, 2 * (size_t)n_tiles, p.epoch - 1);
    p.tile_totals = words;
    p.tile_prefixes = words + n_tiles;
    uint64_t *misc = (uint64_t *)device_alloc(64, "length+error");
    p.total = misc;
    p.error = (uint32_t *)(misc + 1);
    if (enc) {
        p.spill = device_alloc((size_t)groups * 4 * slots * hc::kSpillSlotBytes, "spill area");
        memset(p.spill, 0xD7, (size_t)groups * 4 * slots * hc::kSpillSlotBytes);
        p.out_cmp = device_alloc(cap, "out stream", 1);
        memset(p.out_cmp, 0xA5, cap);
        if (ofs_path) {
            p.tile_ofs_out = (uint64_t *)device_alloc((size_t)n_tiles * 8, "offsets out");
            memset(p.tile_ofs_out, 0xEE, (size_t)n_tiles * 8);
        }
    } else {
        p.out_f32 = (float *)device_alloc(n * 4, "out floats", 16);
        for (size_t i = 0; i < n; ++i) p.out_f32[i] = 7.0f;
    }
    // operands: streams are readable up to their stated size + 160 bytes, as the library asks
    const std::vector<uint8_t> *streams[2] = {&in_a, &in_b};
    const std::vector<uint8_t> *local = nullptr;
    if (op == "compress") local = &in_a;
    if (op == "hom_sum_f32" || op == "hom_sum_i32") local = &in_b;
    for (int c = 0; c < n_in; ++c) {
        uint8_t *d = device_alloc(streams[c]->size() + 160, c ? "stream b" : "stream a", 1);
        memset(d, 0x5A, streams[c]->size() + 160);
        // the buffer ends 160 bytes behind the stated size; put the stream at its start
        memcpy(d, streams[c]->data(), streams[c]->size());
        p.in[c] = d;
        p.in_size[c] = stated[c] < streams[c]->size() ? stated[c] : streams[c]->size();
    }
    if (local) {
        if (local->size() != n * 4) {
            fprintf(stderr, "local operand: %zu bytes for %zu elements\n", local->size(), n);
            return 1;
        }
        uint8_t *d = device_alloc(n * 4, "local operand", 16);
        memcpy(d, local->data(), n * 4);
        p.local = d;
    }
    // ---- offsets pre-pass of the incoming streams
    if (n_in) {
        OffsetsCall oc;
        memset(&oc, 0, sizeof oc);
        const uint32_t blocks = (n_tiles + 255) / 256;
        for (int c = 0; c < n_in; ++c) {
            oc.a.hdr[c] = p.in[c];
            oc.a.block_words[c] = (uint64_t *)device_alloc((size_t)(n_tiles / 256 + 1) * 8, "pre-pass words");
            stale_words(oc.a.block_words[c], n_tiles / 256 + 1, p.epoch - 1);
            oc.a.ofs[c] = (uint64_t *)device_alloc((size_t)n_tiles * 8, "tile offsets in");
            memset(oc.a.ofs[c], 0xEE, (size_t)n_tiles * 8);
            p.in_ofs[c] = oc.a.ofs[c];
        }
        oc.a.few_limit = local ? hc::kFewPlanes : hc::kSlicedMaxF;
        oc.a.error = p.error;
        oc.n_tiles = n_tiles;
        oc.base = hdr;
        oc.epoch = p.epoch;
        oc.spin_limit = p.spin_limit;
        const Launch l{offsets_kernel, &oc};
        run_grid(l, blocks, (unsigned)n_in, 256);
    }
    // ---- the tile kernel
    Launch l{nullptr, &p};
    if (op == "compress") l.kernel = wave_kernel<0, hc::kLocalF32, hc::kOutStream, hc::kPlanesNone>;
    else if (op == "decompress") l.kernel = wave_kernel<1, hc::kLocalNone, hc::kOutF32, hc::kPlanesNone>;
    else if (op == "hom_sum_f32")
        l.kernel = kind ? wave_kernel<1, hc::kLocalF32, hc::kOutStream, hc::kPlanesFew> : wave_kernel<1, hc::kLocalF32, hc::kOutStream, hc::kPlanesNone>;
    else if (op == "hom_sum_i32")
        l.kernel = kind ? wave_kernel<1, hc::kLocalI32, hc::kOutStream, hc::kPlanesFew> : wave_kernel<1, hc::kLocalI32, hc::kOutStream, hc::kPlanesNone>;
    else if (op == "hom_add")
        l.kernel = kind == 2 ? wave_kernel<2, hc::kLocalNone, hc::kOutStream, hc::kPlanesWide> : wave_kernel<2, hc::kLocalNone, hc::kOutStream, hc::kPlanesFew>;
    else
        return 1;
    run_grid(l, groups + (enc ? 1u : 0u), 1, 256, enc ? 4u * (size_t)budget : 0u);   // as launch_wave asks for it
    if (*p.error) {
        fprintf(stderr, "EMU: the kernels raised the error word (0x%x)\n", *p.error);
        return 5;
    }
    if (enc) {
        const uint64_t len = *p.total;
        if (len > cap) {
            fprintf(stderr, "EMU: stream length %llu beyond the capacity %zu\n", (unsigned long long)len, cap);
            return 5;
        }
        write_file(out_path, p.out_cmp, len);
        if (ofs_path) write_file(ofs_path, p.tile_ofs_out, (size_t)n_tiles * 8);
    } else {
        write_file(out_path, p.out_f32, n * 4);
    }
    return 0;
}
