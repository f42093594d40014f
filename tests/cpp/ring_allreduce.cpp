// Runs one of the ring all-reduce variants of tirocinio-triennale_amd/host/allreduce_ring.hpp with
// R ranks as host threads on one GPU (loopback_comm.hpp), the way the reference's benchmark drives
// them over MPI (HomComp/src/cuda_awareallreduce.cu).
//   ring_allreduce <F|I|Fseg|Iseg|Fopt> <ranks> <count> <eb> <in_prefix> <out_prefix> [repeats]
// reads <in_prefix>.r<k>.f32 (count floats per rank), writes <out_prefix>.r<k>.f32, prints status=<rc> and
// the wall time per call of rank 0 (calls after the first, which allocates).
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <thread>
#include <vector>

#include "../../tirocinio-triennale_amd/host/loopback_comm.hpp"

static bool read_file(const std::string &path, std::vector<float> &v)
{
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) return false;
    const size_t got = std::fread(v.data(), sizeof(float), v.size(), f);
    std::fclose(f);
    return got == v.size();
}

static bool write_file(const std::string &path, const std::vector<float> &v)
{
    FILE *f = std::fopen(path.c_str(), "wb");
    if (!f) return false;
    const size_t put = std::fwrite(v.data(), sizeof(float), v.size(), f);
    std::fclose(f);
    return put == v.size();
}

int main(int argc, char **argv)
{
    if (argc < 7) {
        std::fprintf(stderr, "usage: %s <F|I|Fseg|Iseg|Fopt> <ranks> <count> <eb> <in_prefix> <out_prefix> [repeats]\n", argv[0]);
        return 2;
    }
    const std::string variant = argv[1];
    const int ranks = std::atoi(argv[2]);
    const size_t count = std::strtoull(argv[3], nullptr, 10);
    const float eb = std::strtof(argv[4], nullptr);
    const std::string in = argv[5], out = argv[6];
    const int repeats = argc > 7 ? std::atoi(argv[7]) : 1;
    if (ranks < 1 || ranks > 16 || count == 0) return 2;

    homcomp::LoopbackWorld world(ranks);
    std::vector<int> status((size_t)ranks, -1);
    std::chrono::steady_clock::time_point t_second;
    double ms_per_call = 0.0;
    std::vector<std::thread> threads;
    for (int r = 0; r < ranks; ++r) {
        threads.emplace_back([&, r] {
            int rc = 0;
            std::vector<float> host(count);
            float *d_sbuf = nullptr, *d_rbuf = nullptr;
            if (hipSetDevice(0) != hipSuccess || !read_file(in + ".r" + std::to_string(r) + ".f32", host)) rc = 100;
            if (!rc && (hipMalloc((void **)&d_sbuf, count * sizeof(float)) != hipSuccess ||
                        hipMalloc((void **)&d_rbuf, count * sizeof(float)) != hipSuccess))
                rc = 101;
            if (!rc && hipMemcpy(d_sbuf, host.data(), count * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) rc = 102;
            // a rank that failed before the ring still has to take part in it, or the others would wait
            homcomp::RingComm &comm = world.comm(r);
            const auto t_begin = std::chrono::steady_clock::now();
            for (int it = 0; it < repeats && !rc; ++it) {
                if (it == 1 && r == 0) t_second = std::chrono::steady_clock::now();   // the first call allocates
                if (variant == "F") rc = allreduce_ring_comprs_hom_sum_F(d_sbuf, d_rbuf, count, comm, eb);
                else if (variant == "I") rc = allreduce_ring_comprs_hom_sum(d_sbuf, d_rbuf, count, comm, eb);
                else if (variant == "Fseg") rc = allreduce_ring_comprs_hom_sum_F_seg(d_sbuf, d_rbuf, count, comm, eb);
                else if (variant == "Iseg") rc = allreduce_ring_comprs_hom_sum_seg(d_sbuf, d_rbuf, count, comm, eb);
                else if (variant == "Fopt") rc = allreduce_ring_comprs_hom_sum_F_opt(d_sbuf, d_rbuf, count, comm, eb);
                else rc = 2;
            }
            if (r == 0) {
                const auto t_end = std::chrono::steady_clock::now();
                const auto from = repeats > 1 ? t_second : t_begin;
                ms_per_call = std::chrono::duration<double, std::milli>(t_end - from).count() / (repeats > 1 ? repeats - 1 : 1);
            }
            if (!rc && hipMemcpy(host.data(), d_rbuf, count * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess) rc = 103;
            if (!rc && !write_file(out + ".r" + std::to_string(r) + ".f32", host)) rc = 104;
            if (d_sbuf) (void)hipFree(d_sbuf);
            if (d_rbuf) (void)hipFree(d_rbuf);
            status[(size_t)r] = rc;
        });
    }
    for (auto &t : threads) t.join();
    int worst = 0;
    for (int rc : status)
        if (rc != 0) worst = rc;
    std::printf("status=%d ms_per_call=%.3f\n", worst, ms_per_call);
    return worst == 0 ? 0 : 1;
}
