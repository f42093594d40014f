// Drop-in for the reference's host API (HomComp/include/GSZ_entry.h:4-37, without the abandoned
// _outlier_vec pair, and the directly
// launched kernel of HomComp/include/homcomp.cuh:2-5) on top of the C ABI of include/homcomp.h.
//
// Same names, argument order and meaning as the reference, with cudaStream_t -> hipStream_t:
//   * errorBound is an absolute bound;
//   * every call is synchronous with respect to the host, as in the reference (its wrappers
//     end in a blocking cudaMemcpy / cudaFree): the size is read back before returning;
//   * *cmpSize receives what the reference's wrappers report, L + nbEle_padded/32
//     (HomComp/src/GSZ_entry.cu:291-295 adds the header length a second time); define
//     HOMCOMP_TRUE_CMPSIZE to receive the true stream length L instead;
//   * like the reference, the functions return void; failures are reported through
//     homcomp::last_status() (0 = ok), which a caller can poll where the reference polls
//     cudaGetLastError() (HomComp/src/cuda_awareallreduce.cu:207).
// The scratch arrays the reference allocates and frees on every call live in a per-thread
// workspace that grows on demand.  d_cmpBytes needs homcomp_max_stream_bytes(nbEle) bytes.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

#include "../../include/homcomp.h"

namespace homcomp {

inline int &last_status()
{
    thread_local int status = HOMCOMP_OK;
    return status;
}

namespace detail {

struct Cache {
    homcomp_workspace *ws = nullptr;
    size_t capacity = 0;
    ~Cache() { if (ws) homcomp_workspace_destroy(ws); }
};

inline homcomp_workspace *workspace(size_t nbEle)
{
    thread_local Cache cache;
    if (!cache.ws || cache.capacity < nbEle) {
        if (cache.ws) homcomp_workspace_destroy(cache.ws);
        cache.ws = nullptr;
        cache.capacity = 0;
        const int rc = homcomp_workspace_create(&cache.ws, nbEle);
        if (rc != HOMCOMP_OK) {
            last_status() = rc;
            return nullptr;
        }
        cache.capacity = nbEle;
    }
    return cache.ws;
}

// Runs a stream-producing call and reads its size back.  A call that ended in
// HOMCOMP_ERR_SCAN_TIMEOUT (other kernels held compute units, so its grid was not resident as a
// whole) is repeated once with half the grid, which the workspace then keeps.
template <typename Launch>
inline void run_and_report(homcomp_workspace *ws, Launch launch, size_t nbEle, size_t *cmpSize, hipStream_t stream)
{
    size_t len = 0;
    int rc = launch();
    if (rc == HOMCOMP_OK) rc = homcomp_last_size(ws, &len, stream);
    if (rc == HOMCOMP_ERR_SCAN_TIMEOUT) {
        homcomp_workspace_set_option(ws, HOMCOMP_OPT_GRID_PERCENT, 50);
        rc = launch();
        if (rc == HOMCOMP_OK) rc = homcomp_last_size(ws, &len, stream);
    }
    last_status() = rc;
#ifdef HOMCOMP_TRUE_CMPSIZE
    *cmpSize = len;
    (void)nbEle;
#else
    *cmpSize = homcomp_ref_cmpsize(len, nbEle);
#endif
}

}  // namespace detail
}  // namespace homcomp

// HomComp/include/GSZ_entry.h:14-16
inline void GSZ_compress_deviceptr_outlier(float *d_oriData, unsigned char *d_cmpBytes, size_t nbEle,
                                           size_t *cmpSize, float errorBound, hipStream_t stream = 0)
{
    homcomp_workspace *ws = homcomp::detail::workspace(nbEle);
    if (!ws) return;
    homcomp::detail::run_and_report(
        ws, [&] { return homcomp_compress_f32(ws, d_oriData, nbEle, errorBound, d_cmpBytes, nullptr, stream); }, nbEle,
        cmpSize, stream);
}

// HomComp/include/GSZ_entry.h:17-20.  cmpSize may be either convention: blocks are only skipped
// when their payload starts at or beyond it (HomComp/src/GSZ.cu:908-911).
inline void GSZ_decompress_deviceptr_outlier(float *d_decData, unsigned char *d_cmpBytes, size_t nbEle,
                                             size_t cmpSize, float errorBound, hipStream_t stream = 0)
{
    homcomp_workspace *ws = homcomp::detail::workspace(nbEle);
    if (!ws) return;
    int rc = homcomp_decompress_f32(ws, d_cmpBytes, cmpSize, nbEle, errorBound, d_decData, stream);
    if (rc == HOMCOMP_OK && hipStreamSynchronize(stream) != hipSuccess) rc = HOMCOMP_ERR_HIP;
    homcomp::last_status() = rc;
}

// HomComp/include/GSZ_entry.h:8-10: the plain codec (no outlier mode).  *cmpSize receives the true
// stream length: the reference's wrapper (HomComp/src/GSZ_entry.cu:176-180) reports the exclusive
// offset of the last 32768-element chunk plus the header bytes, i.e. it leaves that chunk's
// payload out, and no caller could decode from that many bytes.
inline void GSZ_compress_deviceptr_plain(float *d_oriData, unsigned char *d_cmpBytes, size_t nbEle, size_t *cmpSize,
                                         float errorBound, hipStream_t stream = 0)
{
    homcomp_workspace *ws = homcomp::detail::workspace(nbEle);
    if (!ws) return;
    size_t len = 0;
    auto launch = [&] { return homcomp_compress_plain_f32(ws, d_oriData, nbEle, errorBound, d_cmpBytes, nullptr, stream); };
    int rc = launch();
    if (rc == HOMCOMP_OK) rc = homcomp_last_size(ws, &len, stream);
    if (rc == HOMCOMP_ERR_SCAN_TIMEOUT) {
        homcomp_workspace_set_option(ws, HOMCOMP_OPT_GRID_PERCENT, 50);
        rc = launch();
        if (rc == HOMCOMP_OK) rc = homcomp_last_size(ws, &len, stream);
    }
    homcomp::last_status() = rc;
    *cmpSize = len;
}

// HomComp/include/GSZ_entry.h:11-13.  cmpSize is not used, as in the reference's kernel
// (HomComp/src/GSZ.cu:1750-1991 never reads it): the buffer holds the whole stream.
inline void GSZ_decompress_deviceptr_plain(float *d_decData, unsigned char *d_cmpBytes, size_t nbEle, size_t cmpSize,
                                           float errorBound, hipStream_t stream = 0)
{
    (void)cmpSize;
    homcomp_workspace *ws = homcomp::detail::workspace(nbEle);
    if (!ws) return;
    int rc = homcomp_decompress_plain_f32(ws, d_cmpBytes, nbEle, errorBound, d_decData, stream);
    if (rc == HOMCOMP_OK && hipStreamSynchronize(stream) != hipSuccess) rc = HOMCOMP_ERR_HIP;
    homcomp::last_status() = rc;
}

// HomComp/include/GSZ_entry.h:4-5, HomComp/src/GSZ_entry.cu:28-83: plain codec on host buffers.
// Device buffers are allocated and freed inside the call, as in the reference.  Differences:
// nbEle floats are read from oriData and the padding up to a multiple of 32768 is zero-filled on
// the device (the reference copies the padded count from the host buffer, reading beyond nbEle);
// *cmpSize is the true stream length and that many bytes are copied to cmpBytes (the reference
// reports and copies a length that leaves out the last chunk's payload, :76-77), so cmpBytes needs
// homcomp_max_stream_bytes(nbEle) bytes in the worst case.
inline void GSZ_compress_hostptr(float *oriData, unsigned char *cmpBytes, size_t nbEle, size_t *cmpSize,
                                 float errorBound)
{
    *cmpSize = 0;
    float *d_ori = nullptr;
    unsigned char *d_cmp = nullptr;
    const size_t cap = homcomp_max_stream_bytes(nbEle);
    int rc = HOMCOMP_OK;
    if (hipMalloc((void **)&d_ori, (nbEle ? nbEle : 1) * sizeof(float)) != hipSuccess ||
        hipMalloc((void **)&d_cmp, cap + HOMCOMP_STREAM_SLACK) != hipSuccess ||
        hipMemcpy(d_ori, oriData, nbEle * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
        rc = HOMCOMP_ERR_HIP;
    if (rc == HOMCOMP_OK) {
        GSZ_compress_deviceptr_plain(d_ori, d_cmp, nbEle, cmpSize, errorBound, 0);
        rc = homcomp::last_status();
    }
    if (rc == HOMCOMP_OK && hipMemcpy(cmpBytes, d_cmp, *cmpSize, hipMemcpyDeviceToHost) != hipSuccess) rc = HOMCOMP_ERR_HIP;
    if (d_ori) (void)hipFree(d_ori);
    if (d_cmp) (void)hipFree(d_cmp);
    homcomp::last_status() = rc;
}

// HomComp/include/GSZ_entry.h:6-7, HomComp/src/GSZ_entry.cu:97-147.  cmpSize bytes of cmpBytes are
// copied to the device (it must cover the whole stream); nbEle floats are written to decData (the
// reference writes the count padded to a multiple of 32768).
inline void GSZ_decompress_hostptr(float *decData, unsigned char *cmpBytes, size_t nbEle, size_t cmpSize, float errorBound)
{
    float *d_dec = nullptr;
    unsigned char *d_cmp = nullptr;
    const size_t cap = homcomp_max_stream_bytes(nbEle);
    int rc = HOMCOMP_OK;
    if (cmpSize > cap) cmpSize = cap;
    if (hipMalloc((void **)&d_dec, (nbEle ? nbEle : 1) * sizeof(float)) != hipSuccess ||
        hipMalloc((void **)&d_cmp, cap + HOMCOMP_STREAM_SLACK) != hipSuccess ||
        hipMemset(d_cmp, 0, cap) != hipSuccess ||
        hipMemcpy(d_cmp, cmpBytes, cmpSize, hipMemcpyHostToDevice) != hipSuccess)
        rc = HOMCOMP_ERR_HIP;
    if (rc == HOMCOMP_OK) {
        GSZ_decompress_deviceptr_plain(d_dec, d_cmp, nbEle, cmpSize, errorBound, 0);
        rc = homcomp::last_status();
    }
    if (rc == HOMCOMP_OK && hipMemcpy(decData, d_dec, nbEle * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
        rc = HOMCOMP_ERR_HIP;
    if (d_dec) (void)hipFree(d_dec);
    if (d_cmp) (void)hipFree(d_cmp);
    homcomp::last_status() = rc;
}

// HomComp/include/GSZ_entry.h:29-32
inline void homomorphic_sum(unsigned char *d_cmpBytesIn, int *d_quantPredLoc, unsigned char *d_cmpByteOut,
                            size_t nbEle, float errorBound, size_t *cmpSize, size_t cmpSizeCmpBlock,
                            hipStream_t stream = 0)
{
    (void)errorBound;  // the integer path does not quantise
    homcomp_workspace *ws = homcomp::detail::workspace(nbEle);
    if (!ws) return;
    homcomp::detail::run_and_report(
        ws,
        [&] { return homcomp_hom_sum_i32(ws, d_cmpBytesIn, cmpSizeCmpBlock, d_quantPredLoc, nbEle, d_cmpByteOut, nullptr, stream); },
        nbEle, cmpSize, stream);
}

// HomComp/include/GSZ_entry.h:33-36
inline void homomorphic_sum_F(unsigned char *d_cmpBytesIn, float *d_localChunk, unsigned char *d_cmpByteOut,
                              size_t nbEle, float errorBound, size_t *cmpSize, size_t cmpSizeCmpBlock,
                              hipStream_t stream = 0)
{
    homcomp_workspace *ws = homcomp::detail::workspace(nbEle);
    if (!ws) return;
    homcomp::detail::run_and_report(
        ws,
        [&] {
            return homcomp_hom_sum_f32(ws, d_cmpBytesIn, cmpSizeCmpBlock, d_localChunk, nbEle, errorBound, d_cmpByteOut,
                                       nullptr, stream);
        },
        nbEle, cmpSize, stream);
}

// Callers of the reference launch kernel_quant_prediction<<<grid, 32, 0, stream>>>(...) directly
// (HomComp/src/cuda_awareallreduce.cu:103); this is the same operation as a function.
inline void kernel_quant_prediction(const float *d_localData, int *d_quantPredData, float errorBound,
                                    size_t nbEle, hipStream_t stream = 0)
{
    homcomp::last_status() = homcomp_quant_predict_f32(d_localData, nbEle, errorBound, d_quantPredData, stream);
}
