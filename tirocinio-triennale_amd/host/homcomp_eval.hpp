// The reference's single-GPU evaluator (HomComp/src/homcomp_eval.cu) on top of the GSZ_entry.hpp
// drop-in: the raw float32 reader of HomComp/include/readFile.h:4-34, the element-wise addition the
// "operation" of the decompress-operate-compress workflow uses (sum2arrays, :47-55), the error
// measures of error_evaluation (:72-133) computed on the GPU, and the protocol of main (:135-236):
// compress, the timed decompress + add + compress workflow, the timed homomorphic_sum_F on the same
// operands, decompress, error measures of the reduced values against twice the input.
//
// Compile with hipcc (the header holds three small kernels; they have internal linkage, so the
// header can be included in several translation units of a program).
#pragma once

#include <hip/hip_runtime.h>

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "GSZ_entry.hpp"

namespace homcomp {

// HomComp/include/readFile.h:4-34: the whole file as float32 values (a trailing partial value is
// dropped).  Empty on failure.
inline std::vector<float> read_binary_floats(const char *filename)
{
    std::vector<float> buffer;
    FILE *file = std::fopen(filename, "rb");
    if (!file) {
        std::perror("Cannot open file");
        return buffer;
    }
    std::fseek(file, 0, SEEK_END);
    const long filesize = std::ftell(file);
    std::rewind(file);
    const size_t count = filesize > 0 ? (size_t)filesize / sizeof(float) : 0;
    buffer.resize(count);
    if (std::fread(buffer.data(), sizeof(float), count, file) != count) {
        std::perror("Error reading file");
        buffer.clear();
    }
    std::fclose(file);
    return buffer;
}

// HomComp/src/homcomp_eval.cu:47-55
static __global__ void sum2arrays(float *__restrict__ a, const float *b, size_t count)
{
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)blockDim.x * gridDim.x;
    for (size_t i = tid; i < count; i += stride) a[i] += b[i];
}

// What error_evaluation prints (HomComp/src/homcomp_eval.cu:126-132), as numbers.
struct ErrorStats {
    float min = 0, max = 0;          // of the original values
    double range = 0;                // max - min
    float max_abs_err = 0;           // diffMax
    double max_rel_err = 0;          // diffMax / (max - min)
    double max_pw_rel_err = 0;       // :95-102: err / ori where |ori| > 1, err where 0 < |ori| <= 1, skipped where ori == 0
    double psnr = 0, nrmse = 0;      // 20 log10(range) - 10 log10(mse), sqrt(mse) / range
    double correlation = 0;          // acEff: covariance / (std of the original * std of the reconstruction)
    double compression_ratio = 0;    // nbEle * 4 / cmpSize
};

namespace detail {

constexpr int kEvalThreads = 256;
constexpr int kEvalBlocks = 1024;

struct EvalPartial {
    double sum_ori, sum_dec, sum_err2, max_pw;
    float mn, mx, diff;
    float pad;
};

struct EvalMoments {
    double prod, dev_ori2, dev_dec2;
};

template <typename T, typename F>
__device__ inline T block_fold(T v, F f, T *scratch)
{
    for (int d = 32; d >= 1; d >>= 1) v = f(v, __shfl_xor(v, d, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    T r = scratch[0];
    for (int w = 1; w < kEvalThreads / 64; ++w) r = f(r, scratch[w]);
    return r;
}

// The original value the reconstruction is compared with, in float32: ori[i] * scale (the
// evaluator doubles its input, vec[i] *= 2, :214-215), or ori[i] + ori_b[i] when a second operand
// is given (the same number where the operands coincide).
__device__ inline float eval_original(const float *ori, const float *ori_b, size_t i, float scale)
{
    return ori_b ? ori[i] + ori_b[i] : ori[i] * scale;
}

static __global__ __launch_bounds__(kEvalThreads) void k_eval_first(const float *ori, const float *ori_b, const float *dec, size_t n,
                                                                    float scale, EvalPartial *out)
{
    __shared__ double s_d[kEvalThreads / 64];
    __shared__ float s_f[kEvalThreads / 64];
    const float first = eval_original(ori, ori_b, 0, scale);
    double sum_ori = 0, sum_dec = 0, sum_err2 = 0, max_pw = 0;
    float mn = first, mx = first, diff = 0;
    for (size_t i = (size_t)blockIdx.x * kEvalThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kEvalThreads) {
        const float o = eval_original(ori, ori_b, i, scale), d = dec[i];
        sum_ori += o;
        sum_dec += d;
        if (mx < o) mx = o;
        if (mn > o) mn = o;
        const float err = fabsf(d - o);
        if (o != 0) {
            // as the reference: divided by the value itself, not by its magnitude
            const double rel = fabsf(o) > 1 ? (double)(err / o) : (double)err;
            if (max_pw < rel) max_pw = rel;
        }
        if (diff < err) diff = err;
        sum_err2 += (double)(err * err);   // squared in float32, then widened (:112: `sum += err * err` with a float err)
    }
    auto add = [](double a, double b) { return a + b; };
    auto dmax = [](double a, double b) { return a > b ? a : b; };
    auto fmin_ = [](float a, float b) { return a < b ? a : b; };
    auto fmax_ = [](float a, float b) { return a > b ? a : b; };
    EvalPartial p;
    p.sum_ori = block_fold(sum_ori, add, s_d);
    p.sum_dec = block_fold(sum_dec, add, s_d);
    p.sum_err2 = block_fold(sum_err2, add, s_d);
    p.max_pw = block_fold(max_pw, dmax, s_d);
    p.mn = block_fold(mn, fmin_, s_f);
    p.mx = block_fold(mx, fmax_, s_f);
    p.diff = block_fold(diff, fmax_, s_f);
    p.pad = 0;
    if (threadIdx.x == 0) out[blockIdx.x] = p;
}

static __global__ __launch_bounds__(kEvalThreads) void k_eval_second(const float *ori, const float *ori_b, const float *dec, size_t n,
                                                                     float scale, double mean_ori, double mean_dec, EvalMoments *out)
{
    __shared__ double s_d[kEvalThreads / 64];
    double prod = 0, a2 = 0, b2 = 0;
    for (size_t i = (size_t)blockIdx.x * kEvalThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kEvalThreads) {
        const double a = (double)eval_original(ori, ori_b, i, scale) - mean_ori, b = (double)dec[i] - mean_dec;
        prod += a * b;
        a2 += a * a;
        b2 += b * b;
    }
    auto add = [](double a, double b) { return a + b; };
    EvalMoments m;
    m.prod = block_fold(prod, add, s_d);
    m.dev_ori2 = block_fold(a2, add, s_d);
    m.dev_dec2 = block_fold(b2, add, s_d);
    if (threadIdx.x == 0) out[blockIdx.x] = m;
}

}  // namespace detail

// HomComp/src/homcomp_eval.cu:72-133 on device buffers: the original values are d_ori[i] * scale
// (float32), or d_ori[i] + d_ori_b[i] when d_ori_b is given; the reconstruction is d_dec; cmpSize
// as the reference's wrappers report it.  Two passes as in the reference (means first, then the
// centred moments), accumulated in double; the squared error is formed in float32 as the
// reference forms it.  Returns false when a HIP call fails.
inline bool error_evaluation(const float *d_ori, const float *d_dec, size_t nbEle, size_t cmpSize, ErrorStats *out,
                             float scale = 1.0f, hipStream_t stream = 0, const float *d_ori_b = nullptr)
{
    using namespace detail;
    if (nbEle == 0) return false;
    void *d_part = nullptr;
    const size_t bytes = kEvalBlocks * (sizeof(EvalPartial) > sizeof(EvalMoments) ? sizeof(EvalPartial) : sizeof(EvalMoments));
    if (hipMalloc(&d_part, bytes) != hipSuccess) return false;
    std::vector<EvalPartial> part(kEvalBlocks);
    std::vector<EvalMoments> mom(kEvalBlocks);
    const int blocks = (int)((nbEle + kEvalThreads - 1) / kEvalThreads < (size_t)kEvalBlocks ? (nbEle + kEvalThreads - 1) / kEvalThreads
                                                                                            : (size_t)kEvalBlocks);
    bool ok = true;
    hipLaunchKernelGGL(k_eval_first, dim3(blocks), dim3(kEvalThreads), 0, stream, d_ori, d_ori_b, d_dec, nbEle, scale, (EvalPartial *)d_part);
    ok = hipGetLastError() == hipSuccess;
    ok = ok && hipMemcpyAsync(part.data(), d_part, blocks * sizeof(EvalPartial), hipMemcpyDeviceToHost, stream) == hipSuccess &&
         hipStreamSynchronize(stream) == hipSuccess;
    double sum_ori = 0, sum_dec = 0, sum_err2 = 0, max_pw = 0;
    float mn = part[0].mn, mx = part[0].mx, diff = 0;
    for (int b = 0; ok && b < blocks; ++b) {
        sum_ori += part[b].sum_ori;
        sum_dec += part[b].sum_dec;
        sum_err2 += part[b].sum_err2;
        if (max_pw < part[b].max_pw) max_pw = part[b].max_pw;
        if (mn > part[b].mn) mn = part[b].mn;
        if (mx < part[b].mx) mx = part[b].mx;
        if (diff < part[b].diff) diff = part[b].diff;
    }
    const double mean_ori = sum_ori / (double)nbEle, mean_dec = sum_dec / (double)nbEle;
    if (ok) {
        hipLaunchKernelGGL(k_eval_second, dim3(blocks), dim3(kEvalThreads), 0, stream, d_ori, d_ori_b, d_dec, nbEle, scale, mean_ori, mean_dec,
                           (EvalMoments *)d_part);
        ok = hipGetLastError() == hipSuccess && hipMemcpyAsync(mom.data(), d_part, blocks * sizeof(EvalMoments), hipMemcpyDeviceToHost, stream) == hipSuccess &&
             hipStreamSynchronize(stream) == hipSuccess;
    }
    (void)hipFree(d_part);
    if (!ok) return false;
    double prod = 0, a2 = 0, b2 = 0;
    for (int b = 0; b < blocks; ++b) {
        prod += mom[b].prod;
        a2 += mom[b].dev_ori2;
        b2 += mom[b].dev_dec2;
    }
    const double std1 = std::sqrt(a2 / (double)nbEle), std2 = std::sqrt(b2 / (double)nbEle);
    const double mse = sum_err2 / (double)nbEle;
    const double range = (double)(mx - mn);   // a float32 difference, as in the reference
    out->min = mn;
    out->max = mx;
    out->range = range;
    out->max_abs_err = diff;
    out->max_rel_err = (double)(diff / (mx - mn));
    out->max_pw_rel_err = max_pw;
    out->psnr = 20 * std::log10(range) - 10 * std::log10(mse);
    out->nrmse = std::sqrt(mse) / range;
    out->correlation = prod / (double)nbEle / std1 / std2;
    out->compression_ratio = 1.0 * (double)nbEle * sizeof(float) / (double)cmpSize;
    return true;
}

// The reference's printout (HomComp/src/homcomp_eval.cu:126-132), same wording.
inline void print_error_stats(const ErrorStats &s)
{
    std::printf("Min=%.20G, Max=%.20G, range=%.20G\n", s.min, s.max, s.range);
    std::printf("Max absolute error = %.10f\n", s.max_abs_err);
    std::printf("Max relative error = %f\n", s.max_rel_err);
    std::printf("Max pw relative error = %f\n", s.max_pw_rel_err);
    std::printf("PSNR = %.3f, NRMSE= %.5G\n", s.psnr, s.nrmse);
    std::printf("acEff=%f\n", s.correlation);
    std::printf("Compression Ratio = %f\n", s.compression_ratio);
}

struct EvalResult {
    float eb_abs = 0;
    size_t nbEle = 0, cmpSize = 0, cmpSizeSum = 0;   // reference convention (stream length + header bytes)
    double decompress_s = 0, operation_s = 0, compress_s = 0, hom_s = 0;   // wall clock around the blocking calls
    ErrorStats stats;
    int status = HOMCOMP_OK;
};

// HomComp/src/homcomp_eval.cu:135-236 with both operands given (the reference reads the same file
// twice).  rel: eb is relative to the value range of `vec` (:156-166; float32 arithmetic, done on
// the device here).  The reduced values are scored against vec[i] + vec_local[i] in float32, which
// is the reference's vec[i] * 2 (:214-215) where the operands coincide.  The reduced values are
// left in d_dec_out when it is not null (nbEle floats).
inline EvalResult evaluate(const std::vector<float> &vec, const std::vector<float> &vec_local, float eb, bool rel,
                           float *d_dec_out = nullptr)
{
    using clock = std::chrono::steady_clock;
    EvalResult res;
    const size_t nbEle = vec.size();
    res.nbEle = nbEle;
    if (nbEle == 0 || vec_local.size() != nbEle) {
        res.status = HOMCOMP_ERR_INVALID_ARG;
        return res;
    }
    const size_t cap = homcomp_max_stream_bytes(nbEle);
    float *d_vec = nullptr, *d_local = nullptr, *d_dec = nullptr, *d_minmax = nullptr;
    unsigned char *d_cmp = nullptr, *d_out = nullptr;
    auto release = [&] {
        for (void *p : {(void *)d_vec, (void *)d_local, (void *)d_dec, (void *)d_minmax, (void *)d_cmp, (void *)d_out})
            if (p) (void)hipFree(p);
    };
    bool ok = hipMalloc((void **)&d_vec, nbEle * sizeof(float)) == hipSuccess &&
              hipMalloc((void **)&d_local, nbEle * sizeof(float)) == hipSuccess &&
              hipMalloc((void **)&d_dec, nbEle * sizeof(float)) == hipSuccess &&
              hipMalloc((void **)&d_minmax, 2 * sizeof(float)) == hipSuccess && hipMalloc((void **)&d_cmp, cap + HOMCOMP_STREAM_SLACK) == hipSuccess &&
              hipMalloc((void **)&d_out, cap + HOMCOMP_STREAM_SLACK) == hipSuccess &&
              hipMemcpy(d_vec, vec.data(), nbEle * sizeof(float), hipMemcpyHostToDevice) == hipSuccess &&
              hipMemcpy(d_local, vec_local.data(), nbEle * sizeof(float), hipMemcpyHostToDevice) == hipSuccess;
    if (!ok) {
        release();
        res.status = HOMCOMP_ERR_HIP;
        return res;
    }
    auto failed = [&](int rc) {
        res.status = rc;
        release();
        return res;
    };
    if (rel) {
        homcomp_workspace *ws = detail::workspace(nbEle);
        if (!ws) return failed(last_status());
        float mm[2];
        const int rc = homcomp_range_f32(ws, d_vec, nbEle, d_minmax, 0);
        if (rc != HOMCOMP_OK) return failed(rc);
        if (hipMemcpy(mm, d_minmax, sizeof mm, hipMemcpyDeviceToHost) != hipSuccess) return failed(HOMCOMP_ERR_HIP);
        eb = homcomp_rel_to_abs(eb, mm[0], mm[1]);
    }
    res.eb_abs = eb;
    auto seconds = [](clock::time_point a, clock::time_point b) { return std::chrono::duration<double>(b - a).count(); };
    size_t cmpSize = 0, cmpSize2 = 0;
    GSZ_compress_deviceptr_outlier(d_vec, d_cmp, nbEle, &cmpSize, eb);   // :182 (also warms everything up)
    if (last_status() != HOMCOMP_OK) return failed(last_status());
    // ---- the workflow the homomorphic sum replaces: decompress, operate, compress (:189-203)
    auto t0 = clock::now();
    GSZ_decompress_deviceptr_outlier(d_dec, d_cmp, nbEle, cmpSize, eb);
    auto t1 = clock::now();
    hipLaunchKernelGGL(sum2arrays, dim3(4096), dim3(256), 0, 0, d_dec, d_dec, nbEle);
    if (hipDeviceSynchronize() != hipSuccess) return failed(HOMCOMP_ERR_HIP);
    auto t2 = clock::now();
    GSZ_compress_deviceptr_outlier(d_dec, d_out, nbEle, &cmpSize2, eb);
    auto t3 = clock::now();
    if (last_status() != HOMCOMP_OK) return failed(last_status());
    res.decompress_s = seconds(t0, t1);
    res.operation_s = seconds(t1, t2);
    res.compress_s = seconds(t2, t3);
    // ---- the homomorphic sum on the same operands (:205-209)
    GSZ_compress_deviceptr_outlier(d_vec, d_cmp, nbEle, &cmpSize, eb);
    if (last_status() != HOMCOMP_OK) return failed(last_status());
    t0 = clock::now();
    homomorphic_sum_F(d_cmp, d_local, d_out, nbEle, eb, &cmpSize2, cmpSize);
    t1 = clock::now();
    if (last_status() != HOMCOMP_OK) return failed(last_status());
    res.hom_s = seconds(t0, t1);
    GSZ_decompress_deviceptr_outlier(d_dec, d_out, nbEle, cmpSize2, eb);   // :210-211
    if (last_status() != HOMCOMP_OK) return failed(last_status());
    res.cmpSize = cmpSize;
    res.cmpSizeSum = cmpSize2;
    // :214-217: the reduced values against the sum of the operands (twice the input in the
    // reference, whose operands are one file), CR from the sum's cmpSize
    if (!error_evaluation(d_vec, d_dec, nbEle, cmpSize2, &res.stats, 1.0f, 0, d_local)) return failed(HOMCOMP_ERR_HIP);
    if (d_dec_out && hipMemcpy(d_dec_out, d_dec, nbEle * sizeof(float), hipMemcpyDeviceToDevice) != hipSuccess)
        return failed(HOMCOMP_ERR_HIP);
    release();
    return res;
}

// The closing lines of the reference's main (:220-225).
inline void print_performance(const EvalResult &r)
{
    const double normal_cost = r.operation_s + r.compress_s + r.decompress_s;
    const double bytes = (double)r.nbEle * sizeof(float);
    std::printf("Traditional DOC workflow (decompression+operation+compression) performance: time: %f s, throughput: %f GBps\n",
                normal_cost, bytes / normal_cost / 1000 / 1000 / 1000);
    std::printf("HomComp_F performance: time: %f s, throughput: %f GBps\n", r.hom_s, bytes / r.hom_s / 1000 / 1000 / 1000);
    std::printf("HomComp_F speedup: %0.2fX\n", normal_cost / r.hom_s);
}

}  // namespace homcomp
