// Status codes and device plumbing of the luminal_hip C ABI.
#include "common.h"

namespace lhip {

static thread_local int g_last_hip_error = 0;

lhip_status hip_failed(hipError_t e) {
    g_last_hip_error = static_cast<int>(e);
    // Clear the sticky "last error" so the next call starts clean.
    (void)hipGetLastError();
    return LHIP_ERR_HIP;
}

lhip_status moe_static_setup();  // mxfp4_moe.hip

}  // namespace lhip

extern "C" {

const char *lhip_status_string(lhip_status s) {
    switch (s) {
        case LHIP_OK: return "LHIP_OK";
        case LHIP_ERR_NULL_PTR: return "LHIP_ERR_NULL_PTR";
        case LHIP_ERR_INVALID_SHAPE: return "LHIP_ERR_INVALID_SHAPE";
        case LHIP_ERR_MISALIGNED: return "LHIP_ERR_MISALIGNED";
        case LHIP_ERR_HIP: return "LHIP_ERR_HIP";
        case LHIP_ERR_UNSUPPORTED: return "LHIP_ERR_UNSUPPORTED";
        default: return "LHIP_ERR_UNKNOWN";
    }
}

int lhip_last_hip_error(void) { return lhip::g_last_hip_error; }

const char *lhip_version(void) { return "0.1.0"; }

lhip_status lhip_init(int device) {
    int count = 0;
    LHIP_HIP_TRY(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return LHIP_ERR_INVALID_SHAPE;
    LHIP_HIP_TRY(hipSetDevice(device));
    return lhip::moe_static_setup();  // the address of the per-device scratch array behind lhip_mxfp4_moe_bf16_static
}

lhip_status lhip_malloc(void **dptr, size_t nbytes) {
    if (!dptr) return LHIP_ERR_NULL_PTR;
    *dptr = nullptr;
    if (nbytes == 0) return LHIP_ERR_INVALID_SHAPE;
    LHIP_HIP_TRY(hipMalloc(dptr, nbytes));
    return LHIP_OK;
}

lhip_status lhip_free(void *dptr) {
    if (!dptr) return LHIP_OK;
    LHIP_HIP_TRY(hipFree(dptr));
    return LHIP_OK;
}

lhip_status lhip_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes, void *stream) {
    if (!dst_dev || !src_host) return LHIP_ERR_NULL_PTR;
    if (nbytes == 0) return LHIP_OK;
    hipStream_t s = lhip::as_stream(stream);
    LHIP_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, nbytes, hipMemcpyHostToDevice, s));
    LHIP_HIP_TRY(hipStreamSynchronize(s));
    return LHIP_OK;
}

lhip_status lhip_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes, void *stream) {
    if (!dst_host || !src_dev) return LHIP_ERR_NULL_PTR;
    if (nbytes == 0) return LHIP_OK;
    hipStream_t s = lhip::as_stream(stream);
    LHIP_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, s));
    LHIP_HIP_TRY(hipStreamSynchronize(s));
    return LHIP_OK;
}

lhip_status lhip_stream_sync(void *stream) {
    LHIP_HIP_TRY(hipStreamSynchronize(lhip::as_stream(stream)));
    return LHIP_OK;
}

}  // extern "C"
