// The one entry point of the library that allocates nothing: Kernel::forward / forward_batched of a Q8_0
// weight on device pointers (quantize_q8_0_into, then the x86-64-order GEMV, src/ops/kernel/trait_.rs:59-109),
// with the quantized activation -- the only memory these two kernels need beyond the caller's input and
// output -- in a fixed array of the code object instead of the per-thread staging buffers that
// rmi_hip_q8_0_forward_batched grows with hipMalloc.  For callers that cannot allocate: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.
#include "rmi_internal.h"

namespace {

// n_tokens * n_in of one call; the array holds that many int8 quants followed by one f32 scale per 32 of them
constexpr size_t kNoAllocMaxElems = RMI_HIP_NOALLOC_MAX_ELEMS;
constexpr size_t kScratchBytes = kNoAllocMaxElems + kNoAllocMaxElems / 32 * 4;  // 288 KiB

// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.
// The name is a host-side stand-in only: host code uses the address hipGetSymbolAddress returned for the device.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
unsigned char *g_scratch_ptr[kMaxDevices] = {};

}  // namespace

// Called by rmi_hip_init with `device` current: the device address of this device's copy of the array.
int rmi_noalloc_setup(int device) {
    if (device < 0 || device >= kMaxDevices)
        return rmi_fail(RMI_HIP_E_INVALID, "device %d: the no-allocation entry point knows devices 0..%d", device, kMaxDevices - 1);
    if (g_scratch_ptr[device]) return RMI_HIP_OK;
    void *p = nullptr;
    RMI_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return rmi_fail(RMI_HIP_E_RUNTIME, "hipGetSymbolAddress gave no address for the scratch array");
    g_scratch_ptr[device] = static_cast<unsigned char *>(p);
    return RMI_HIP_OK;
}

extern "C" {

int rmi_hip_q8_0_forward_noalloc_dev(const rmi_hip_weight *w, const float *x, float *y, uint32_t n_tokens,
                                     uint32_t y_stride, int rounding, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    if (!x || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(y) & 3) != 0)
        return rmi_fail(RMI_HIP_E_INVALID, "the input must be 16-byte aligned, the output 4-byte aligned");
    if (y_stride < w->n_out && n_tokens > 1) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < n_out=%u", y_stride, w->n_out);
    const uint64_t n_x = uint64_t(n_tokens) * w->n_in;
    if (n_x > kNoAllocMaxElems)
        return rmi_fail(RMI_HIP_E_INVALID,
                        "%u tokens x %u elements = %llu exceed the fixed scratch of %zu elements; use "
                        "rmi_hip_q8_0_forward_batched or split the batch",
                        n_tokens, w->n_in, (unsigned long long)n_x, kNoAllocMaxElems);
    // checked here, before the quantizer is enqueued: a refused call leaves the shared array as it was
    if (!rmi_gemv_q8_0_tokens_fits(w)) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u is too long for the GEMV staging", w->n_in);
    int device = -1;
    RMI_HIP_CHECK(hipGetDevice(&device));
    if (device != rmi_device())
        return rmi_fail(RMI_HIP_E_INVALID, "the calling thread's current device is %d, the library runs on %d", device, rmi_device());
    unsigned char *base = g_scratch_ptr[device];
    if (!base) return rmi_fail(RMI_HIP_E_NOT_INIT, "no scratch address for device %d", device);
    // every byte the GEMV reads is written by the quantizer of this call: nothing has to start at zero
    int8_t *q8 = reinterpret_cast<int8_t *>(base);
    float *scales = reinterpret_cast<float *>(base + kNoAllocMaxElems);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc = rmi_launch_quantize_q8_0(x, q8, scales, n_tokens, w->n_in, rounding, s);
    if (rc != RMI_HIP_OK) return rc;
    return rmi_gemv_q8_0_tokens(w, q8, scales, y, n_tokens, y_stride, 0, w->n_out, s);
}

}  // extern "C"
