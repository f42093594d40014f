// Exercises the GSZ_entry.hpp drop-in the way the reference's evaluator does
// (HomComp/src/homcomp_eval.cu:182-212): compress, homomorphic_sum_F with a second operand,
// homomorphic_sum with its Lorenzo pre-pass, decompress.  Reads two raw float32 files, writes the
// two streams and the decompressed sum as raw files for the Python test to compare.
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "../../tirocinio-triennale_amd/host/GSZ_entry.hpp"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 2; } } while (0)
#define CHECK_HC() do { if (homcomp::last_status() != HOMCOMP_OK) { std::fprintf(stderr, "homcomp: %s at line %d\n", homcomp_status_string(homcomp::last_status()), __LINE__); return 3; } } while (0)

static std::vector<float> read_floats(const char *path)
{
    std::vector<float> v;
    if (FILE *f = std::fopen(path, "rb")) {
        std::fseek(f, 0, SEEK_END);
        const long bytes = std::ftell(f);
        std::fseek(f, 0, SEEK_SET);
        v.resize((size_t)bytes / sizeof(float));
        if (std::fread(v.data(), sizeof(float), v.size(), f) != v.size()) v.clear();
        std::fclose(f);
    }
    return v;
}

static bool write_bytes(const char *path, const void *p, size_t n)
{
    FILE *f = std::fopen(path, "wb");
    if (!f) return false;
    const bool ok = std::fwrite(p, 1, n, f) == n;
    std::fclose(f);
    return ok;
}

int main(int argc, char **argv)
{
    if (argc != 5) {
        std::fprintf(stderr, "usage: %s a.f32 b.f32 eb out_prefix\n", argv[0]);
        return 1;
    }
    const std::vector<float> a = read_floats(argv[1]), b = read_floats(argv[2]);
    const float eb = (float)std::atof(argv[3]);
    const std::string prefix = argv[4];
    if (a.empty() || a.size() != b.size()) return 1;
    const size_t n = a.size(), cap = homcomp_max_stream_bytes(n);
    float *d_a, *d_b, *d_dec;
    int *d_pred;
    unsigned char *d_cmp, *d_sum, *d_sum_i;
    CHECK_HIP(hipMalloc(&d_a, n * 4));
    CHECK_HIP(hipMalloc(&d_b, n * 4));
    CHECK_HIP(hipMalloc(&d_dec, n * 4));
    CHECK_HIP(hipMalloc(&d_pred, n * 4));
    CHECK_HIP(hipMalloc(&d_cmp, cap));
    CHECK_HIP(hipMalloc(&d_sum, cap));
    CHECK_HIP(hipMalloc(&d_sum_i, cap));
    CHECK_HIP(hipMemcpy(d_a, a.data(), n * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_b, b.data(), n * 4, hipMemcpyHostToDevice));

    size_t cmpSize = 0, sumSize = 0, sumSizeI = 0;
    GSZ_compress_deviceptr_outlier(d_a, d_cmp, n, &cmpSize, eb);
    CHECK_HC();
    homomorphic_sum_F(d_cmp, d_b, d_sum, n, eb, &sumSize, cmpSize);
    CHECK_HC();
    kernel_quant_prediction(d_b, d_pred, eb, n);
    CHECK_HC();
    homomorphic_sum(d_cmp, d_pred, d_sum_i, n, eb, &sumSizeI, cmpSize);
    CHECK_HC();
    GSZ_decompress_deviceptr_outlier(d_dec, d_sum, n, sumSize, eb);
    CHECK_HC();

    // sizes follow the reference's convention: true length = reported - header bytes
    const size_t hdr = homcomp_header_bytes(n);
    std::vector<unsigned char> h_cmp(cmpSize - hdr), h_sum(sumSize - hdr), h_sum_i(sumSizeI - hdr);
    std::vector<float> h_dec(n);
    CHECK_HIP(hipMemcpy(h_cmp.data(), d_cmp, h_cmp.size(), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(h_sum.data(), d_sum, h_sum.size(), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(h_sum_i.data(), d_sum_i, h_sum_i.size(), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(h_dec.data(), d_dec, n * 4, hipMemcpyDeviceToHost));
    if (!write_bytes((prefix + ".cmp").c_str(), h_cmp.data(), h_cmp.size()) ||
        !write_bytes((prefix + ".sum").c_str(), h_sum.data(), h_sum.size()) ||
        !write_bytes((prefix + ".sum_i").c_str(), h_sum_i.data(), h_sum_i.size()) ||
        !write_bytes((prefix + ".dec").c_str(), h_dec.data(), n * 4))
        return 4;
    std::printf("n=%zu cmpSize=%zu sumSize=%zu sumSizeI=%zu header=%zu\n", n, cmpSize, sumSize, sumSizeI, hdr);

    // the plain codec: device pointers, then the same through the host-pointer entries
    size_t plainSize = 0, hostSize = 0;
    GSZ_compress_deviceptr_plain(d_a, d_cmp, n, &plainSize, eb);
    CHECK_HC();
    GSZ_decompress_deviceptr_plain(d_dec, d_cmp, n, plainSize, eb);
    CHECK_HC();
    std::vector<unsigned char> h_plain(plainSize), h_host(cap);
    std::vector<float> h_pdec(n), h_hdec(n, -1.0f);
    CHECK_HIP(hipMemcpy(h_plain.data(), d_cmp, plainSize, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(h_pdec.data(), d_dec, n * 4, hipMemcpyDeviceToHost));
    std::vector<float> a_copy(a);
    GSZ_compress_hostptr(a_copy.data(), h_host.data(), n, &hostSize, eb);
    CHECK_HC();
    GSZ_decompress_hostptr(h_hdec.data(), h_host.data(), n, hostSize, eb);
    CHECK_HC();
    if (!write_bytes((prefix + ".plain").c_str(), h_plain.data(), plainSize) ||
        !write_bytes((prefix + ".plain_host").c_str(), h_host.data(), hostSize) ||
        !write_bytes((prefix + ".plain_dec").c_str(), h_pdec.data(), n * 4) ||
        !write_bytes((prefix + ".plain_host_dec").c_str(), h_hdec.data(), n * 4))
        return 4;
    std::printf("plainSize=%zu hostSize=%zu\n", plainSize, hostSize);
    return 0;
}
