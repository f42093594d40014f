// The sums of the bit-plane paths (tirocinio-triennale_amd/csrc/homcomp_device.hpp), run alone on the
// GPU, a block per lane as in the kernels, and checked element by element against integer
// addition of the deltas the blocks encode (HomComp/src/homcomp.cu:2252-2268, 3611-3616: the
// sums the reference makes value by value).  Random blocks of every plane count the paths take,
// plain and outlier mode on either side, both signs, zeros; 64 lanes x 400 rounds per case.
// Prints one line per case and "units ok" at the end; exit status 1 on a mismatch.
#include "../../tirocinio-triennale_amd/csrc/homcomp_device.hpp"

#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

using namespace hc;

namespace {

// what the kernels hand the sums: the block's words from the sign word on, the word at its start, the digest of its header byte
struct Block {
    uint32_t first, digest, w[kWideWords];
};

// a block's result in one form for both paths
struct Result {
    uint32_t hdr, size, ob, F, a0, sign, m[kWideOutWords];
};

template <uint32_t NP>
__global__ void k_few(const Block *A, const Block *B, Result *R)
{
    SlicedIn a, b;
    auto take = [](const Block &x, SlicedIn &s) {
        const uint32_t F = x.digest & 0x1fu;
        s.ob = x.digest >> 5;
        s.a0 = s.ob ? x.first & ~(0xffffff00u << ((8u * (s.ob - 1u)) & 31u)) : 0u;   // the outlier bytes of the word
        s.sign = x.w[0];
        for (uint32_t q = 0; q < kSlicedMaxF; ++q) s.pl[q] = q < F ? x.w[q + 1] : 0u;
    };
    take(A[threadIdx.x], a);
    take(B[threadIdx.x], b);
    SlicedOut o;
    sliced_add<NP>(a, b, o);
    Result r = {};
    r.hdr = o.hdr; r.size = o.size; r.ob = o.ob; r.F = o.F; r.a0 = o.a0; r.sign = o.sign;
    for (uint32_t q = 0; q < (uint32_t)kSlicedOutWords; ++q) r.m[q] = o.m[q];
    R[threadIdx.x] = r;
}

// stream (+) local operand: B carries the local deltas as kLocalFew two's-complement planes in w[1..], the delta of element 0 in `first`
__global__ void k_local(const Block *A, const Block *B, Result *R)
{
    SlicedIn a;
    const Block &x = A[threadIdx.x];
    const uint32_t F = x.digest & 0x1fu;
    a.ob = x.digest >> 5;
    a.a0 = a.ob ? x.first & ~(0xffffff00u << ((8u * (a.ob - 1u)) & 31u)) : 0u;
    a.sign = x.w[0];
    for (uint32_t q = 0; q < kSlicedMaxF; ++q) a.pl[q] = q < F ? x.w[q + 1] : 0u;
    uint32_t plB[kLocalFew];
    for (uint32_t q = 0; q < kLocalFew; ++q) plB[q] = B[threadIdx.x].w[q + 1];
    SlicedOut o;
    sliced_add_local<kFewPlanes, kLocalFew>(a, plB, B[threadIdx.x].first, o);
    Result r = {};
    r.hdr = o.hdr; r.size = o.size; r.ob = o.ob; r.F = o.F; r.a0 = o.a0; r.sign = o.sign;
    for (uint32_t q = 0; q < (uint32_t)kSlicedOutWords; ++q) r.m[q] = o.m[q];
    R[threadIdx.x] = r;
}

__global__ void k_wide(const Block *A, const Block *B, Result *R, uint32_t chunks)
{
    WideIn a, b;
    auto take = [](const Block &x, WideIn &s) {
        s.first = x.first;
        for (uint32_t q = 0; q < kWideWords; ++q) s.w[q] = x.w[q];
    };
    take(A[threadIdx.x], a);
    take(B[threadIdx.x], b);
    WideSum sum;
    wide_sum(a, A[threadIdx.x].digest, b, B[threadIdx.x].digest, chunks, sum);
    WideOut o;
    wide_finish(sum, o);
    Result r = {};
    r.hdr = o.hdr; r.size = o.size; r.ob = o.ob; r.F = o.F; r.a0 = o.a0; r.sign = o.w[0];
    for (uint32_t q = 0; q + 1 < kWideOutWords; ++q) r.m[q] = o.w[q + 1];
    R[threadIdx.x] = r;
}

uint32_t bits(uint32_t x) { return x ? 32u - (uint32_t)__builtin_clz(x) : 0u; }

// element i of a block sits at bit 8 * (i / 8) + 7 - i % 8 of every word (HomComp/src/GSZ.cu:312-351)
uint32_t bit_of(int i) { return 1u << (8 * (i / 8) + 7 - i % 8); }

// a random block of at most `planes` planes: its deltas, and its words as the stream holds them
void make_block(std::mt19937 &rng, uint32_t planes, int *v, Block &x)
{
    const bool outlier = rng() % 2;
    const uint32_t top = planes ? 1u + rng() % planes : 0u;   // the block's own plane count
    for (int i = 0; i < 32; ++i) {
        int m = top ? (int)(rng() % (1u << top)) : 0;
        if (rng() % 4 == 0) m = 0;
        v[i] = (rng() & 1) ? -m : m;
    }
    if (outlier) {
        const uint32_t width = 1u + rng() % 30;   // (the sum of two stays within an int, as the comparison below assumes)
        v[0] = (int)(1u + rng() % ((1u << width) - 1u));
        if (rng() & 1) v[0] = -v[0];
    }
    uint32_t F = 0;
    for (int i = outlier ? 1 : 0; i < 32; ++i) F = F > bits((uint32_t)abs(v[i])) ? F : bits((uint32_t)abs(v[i]));
    x = Block{};
    for (int i = 0; i < 32; ++i) {
        if (v[i] < 0) x.w[0] |= bit_of(i);
        if (outlier && i == 0) continue;
        for (uint32_t q = 0; q < F; ++q)
            if (((uint32_t)abs(v[i]) >> q) & 1u) x.w[q + 1] |= bit_of(i);
    }
    uint32_t ob = 0;
    if (outlier) {
        ob = (bits((uint32_t)abs(v[0])) + 7) / 8;
        const uint32_t keep = ob < 4 ? (1u << 8 * ob) - 1u : ~0u;
        x.first = ((uint32_t)abs(v[0]) & keep) | ((uint32_t)rng() & ~keep);   // the bytes beyond the outlier belong to the sign word: anything
    }
    x.digest = (ob << 5) | F;
    if (ob == 0 && F == 0) x.digest = 0, x.w[0] = 0;   // an empty block has no sign word either
    for (uint32_t w = F + 1; w < kWideWords; ++w) x.w[w] = (uint32_t)rng();   // what follows a block's planes is the next block: anything
}

int check(const char *what, const std::vector<int> &va, const std::vector<int> &vb, const std::vector<Result> &R, int &shown)
{
    int bad = 0;
    for (int l = 0; l < 64; ++l) {
        const Result &o = R[l];
        for (int i = 0; i < 32; ++i) {
            long mag = 0;
            for (uint32_t q = 0; q < o.F; ++q)
                if (o.m[q] & bit_of(i)) mag |= 1l << q;
            if (i == 0 && o.ob) mag = o.a0;
            const long val = (o.sign & bit_of(i)) ? -mag : mag;
            const long want = (long)va[l * 32 + i] + vb[l * 32 + i];
            if (val != want) {
                if (shown++ < 5) printf("%s: lane %d element %d: got %ld, want %ld (header %02x)\n", what, l, i, val, want, o.hdr);
                ++bad;
            }
        }
        // the header byte and the size follow from the sums (HomComp/src/GSZ.cu:151-167)
        uint32_t fr1 = 0, fr2 = 0;
        for (int i = 0; i < 32; ++i) {
            const uint32_t b = bits((uint32_t)labs((long)va[l * 32 + i] + vb[l * 32 + i]));
            fr1 = fr1 > b ? fr1 : b;
            if (i) fr2 = fr2 > b ? fr2 : b;
        }
        if (fr1 > 31) fr1 = 31;
        const uint32_t ob = (bits((uint32_t)labs((long)va[l * 32] + vb[l * 32])) + 7) / 8;
        const uint32_t sz1 = fr1 ? 4 + 4 * fr1 : 0, sz2 = 4 + 4 * fr2 + ob;
        const uint32_t hdr = sz1 <= sz2 ? fr1 : (fr2 | 0x80u | ((ob - 1) << 5));
        if (o.hdr != hdr || o.size != (sz1 <= sz2 ? sz1 : sz2)) {
            if (shown++ < 5) printf("%s: lane %d: header %02x size %u, want %02x %u\n", what, l, o.hdr, o.size, hdr, sz1 <= sz2 ? sz1 : sz2);
            ++bad;
        }
    }
    return bad;
}

}  // namespace

int main()
{
    std::mt19937 rng(20240607);
    Block *dA, *dB;
    Result *dR;
    if (hipMalloc(&dA, 64 * sizeof(Block)) != hipSuccess || hipMalloc(&dB, 64 * sizeof(Block)) != hipSuccess ||
        hipMalloc(&dR, 64 * sizeof(Result)) != hipSuccess) {
        printf("hipMalloc failed\n");
        return 2;
    }
    std::vector<Block> hA(64), hB(64);
    std::vector<Result> hR(64);
    std::vector<int> va(64 * 32), vb(64 * 32);
    int total_bad = 0;
    auto run_case = [&](const char *what, uint32_t planes, auto launch) {
        int bad = 0, shown = 0;
        for (int round = 0; round < 400; ++round) {
            for (int l = 0; l < 64; ++l) {
                make_block(rng, planes, &va[l * 32], hA[l]);
                make_block(rng, rng() % 3 ? planes : 1u + rng() % planes, &vb[l * 32], hB[l]);
                if (round % 7 == 3) {   // blocks that cancel, whole or in their first element
                    for (int i = l % 2 ? 0 : 1; i < 32; ++i) vb[l * 32 + i] = -va[l * 32 + i];
                    if (l % 2 == 0) vb[l * 32] = va[l * 32];
                    hB[l] = hA[l];
                    hB[l].w[0] = ~hA[l].w[0];
                    if (l % 2 == 0) hB[l].w[0] ^= bit_of(0);
                    for (int i = 0; i < 32; ++i)   // no sign on a zero (as the reference writes them); it must not matter either
                        if (vb[l * 32 + i] == 0 && (rng() & 1)) hB[l].w[0] &= ~bit_of(i);
                }
            }
            if (hipMemcpy(dA, hA.data(), 64 * sizeof(Block), hipMemcpyHostToDevice) != hipSuccess ||
                hipMemcpy(dB, hB.data(), 64 * sizeof(Block), hipMemcpyHostToDevice) != hipSuccess) return;
            launch();
            if (hipMemcpy(hR.data(), dR, 64 * sizeof(Result), hipMemcpyDeviceToHost) != hipSuccess) { bad = 1 << 20; break; }
            bad += check(what, va, vb, hR, shown);
        }
        printf("%-40s %s (%d mismatches)\n", what, bad ? "FAILED" : "ok", bad);
        total_bad += bad;
    };
    run_case("few planes, up to 3", kFewPlanes, [&] { hipLaunchKernelGGL(k_few<kFewPlanes>, dim3(1), dim3(64), 0, 0, dA, dB, dR); });
    run_case("few planes, up to 6", kSlicedMaxF, [&] { hipLaunchKernelGGL(k_few<kSlicedMaxF>, dim3(1), dim3(64), 0, 0, dA, dB, dR); });
    for (uint32_t chunks = 1; chunks <= kWideChunks; ++chunks) {
        char what[64];
        const uint32_t planes = 4 * chunks - 2;   // the widest blocks that `chunks` pieces are summed over
        snprintf(what, sizeof what, "wide blocks, %u pieces (up to %u planes)", chunks, planes);
        run_case(what, planes, [&] { hipLaunchKernelGGL(k_wide, dim3(1), dim3(64), 0, 0, dA, dB, dR, chunks); });
    }
    {   // stream (+) local operand: incoming blocks of up to three planes, local deltas within -8 .. 7, any first delta
        int bad = 0, shown = 0;
        for (int round = 0; round < 400; ++round) {
            for (int l = 0; l < 64; ++l) {
                make_block(rng, kFewPlanes, &va[l * 32], hA[l]);
                hB[l] = Block{};
                for (int i = 0; i < 32; ++i) {
                    int v = (int)(rng() % 16) - 8;
                    if (round % 5 == 2 && i) v = va[l * 32 + i] > 7 || va[l * 32 + i] < -7 ? v : -va[l * 32 + i];   // sums of zero
                    if (i == 0) v = (int)(rng() % (1u << (1 + rng() % 30))) * ((rng() & 1) ? -1 : 1);
                    vb[l * 32 + i] = v;
                    if (i == 0) { hB[l].first = (uint32_t)v; continue; }
                    for (uint32_t q = 0; q < kLocalFew; ++q)
                        if (((uint32_t)v >> q) & 1u) hB[l].w[q + 1] |= bit_of(i);
                }
            }
            if (hipMemcpy(dA, hA.data(), 64 * sizeof(Block), hipMemcpyHostToDevice) != hipSuccess ||
                hipMemcpy(dB, hB.data(), 64 * sizeof(Block), hipMemcpyHostToDevice) != hipSuccess) { bad = 1 << 20; break; }
            hipLaunchKernelGGL(k_local, dim3(1), dim3(64), 0, 0, dA, dB, dR);
            if (hipMemcpy(hR.data(), dR, 64 * sizeof(Result), hipMemcpyDeviceToHost) != hipSuccess) { bad = 1 << 20; break; }
            bad += check("stream (+) local operand", va, vb, hR, shown);
        }
        printf("%-40s %s (%d mismatches)\n", "stream (+) local operand, up to 3 planes", bad ? "FAILED" : "ok", bad);
        total_bad += bad;
    }
    if (hipDeviceSynchronize() != hipSuccess) total_bad += 1;
    printf(total_bad ? "units FAILED\n" : "units ok\n");
    return total_bad ? 1 : 0;
}
