// The reference's evaluator as a program (HomComp/src/homcomp_eval.cu:135-236) on top of
// host/homcomp_eval.hpp: reads raw float32 files, runs compress, the decompress + add + compress
// workflow and homomorphic_sum_F, prints the reference's report and, for the test that drives it,
// the same numbers in full precision on one line.
//   homcomp_eval data.f32 local.f32 eb rel(0|1) [reduced_out.f32]
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../tirocinio-triennale_amd/host/homcomp_eval.hpp"

int main(int argc, char **argv)
{
    if (argc < 5) {
        std::fprintf(stderr, "usage: %s data.f32 local.f32 eb rel(0|1) [reduced_out.f32]\n", argv[0]);
        return 1;
    }
    const std::vector<float> vec = homcomp::read_binary_floats(argv[1]);
    const std::vector<float> vec_local = homcomp::read_binary_floats(argv[2]);
    const float eb = (float)std::atof(argv[3]);
    const bool rel = std::atoi(argv[4]) != 0;
    if (vec.empty() || vec.size() != vec_local.size()) return 1;
    float *d_dec = nullptr;
    if (hipMalloc((void **)&d_dec, vec.size() * sizeof(float)) != hipSuccess) return 2;
    const homcomp::EvalResult r = homcomp::evaluate(vec, vec_local, eb, rel, d_dec);
    if (r.status != HOMCOMP_OK) {
        std::fprintf(stderr, "homcomp: %s\n", homcomp_status_string(r.status));
        return 3;
    }
    homcomp::print_error_stats(r.stats);
    homcomp::print_performance(r);
    const homcomp::ErrorStats &s = r.stats;
    std::printf("KV nbEle=%zu eb_abs=%.9g cmpSize=%zu cmpSizeSum=%zu min=%.9g max=%.9g range=%.17g max_abs_err=%.9g "
                "max_rel_err=%.17g max_pw_rel_err=%.17g psnr=%.17g nrmse=%.17g correlation=%.17g compression_ratio=%.17g "
                "doc_s=%.9g hom_s=%.9g\n",
                r.nbEle, r.eb_abs, r.cmpSize, r.cmpSizeSum, s.min, s.max, s.range, s.max_abs_err, s.max_rel_err, s.max_pw_rel_err,
                s.psnr, s.nrmse, s.correlation, s.compression_ratio, r.decompress_s + r.operation_s + r.compress_s, r.hom_s);
    if (argc > 5) {
        std::vector<float> h(vec.size());
        if (hipMemcpy(h.data(), d_dec, h.size() * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess) return 2;
        FILE *f = std::fopen(argv[5], "wb");
        if (!f || std::fwrite(h.data(), sizeof(float), h.size(), f) != h.size()) return 4;
        std::fclose(f);
    }
    (void)hipFree(d_dec);
    return 0;
}
