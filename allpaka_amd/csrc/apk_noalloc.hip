// The one entry point of libapk_hip.so that allocates nothing: apk_argmax_rows_noalloc.
//
// Callers under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc cannot use an entry that
// grows a context buffer on demand.  The split-row argmax needs 128 bytes of device scratch per row (the running
// best and the arrival count of a row's workgroups); here that scratch is a static device array of this translation
// unit, APK_NOALLOC_MAX_ROWS rows = 256 KiB per GPU, held from the moment the library is loaded until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress: its device address is looked up
// once per device (apk_noalloc_setup, called by apk_init with that device current) and only that address is ever
// handed to a kernel.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two contexts,
// two host threads) race.  This file is built by hipcc (the array is device code); the kernels stay in the
// embedded code object and take the address as an argument, exactly as they take the context's buffer in
// apk_argmax_rows.
#include <hip/hip_runtime.h>

#include <mutex>

#include "apk_internal.h"

#define APK_NOALLOC_MAX_ROWS 2048

static __device__ __align__(256) unsigned long long scratch[APK_NOALLOC_MAX_ROWS * 16];  // 16 x 8 bytes per row

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_mu;
void* g_ptr[kMaxDevices] = {};   // device address of `scratch` on each device, once looked up
int g_status[kMaxDevices] = {};  // 0: not looked up yet; 1: ok; < 0: -(hipError_t) of the failed lookup
}  // namespace

int apk_noalloc_setup(int device) {
    if (device < 0 || device >= kMaxDevices) return apk_fail(APK_DECLINE_NO_DEVICE, "apk_noalloc_setup: device %d", device);
    std::lock_guard<std::mutex> lock(g_mu);
    if (g_status[device] == 0) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // the current device's copy of the array
        if (e != hipSuccess || !p) {
            g_status[device] = -(int)(e != hipSuccess ? e : hipErrorInvalidSymbol);
            return apk_fail(g_status[device], "hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(e));
        }
        g_ptr[device] = p;
        g_status[device] = 1;
    }
    return g_status[device] == 1 ? APK_OK : g_status[device];
}

extern "C" __attribute__((visibility("default"))) int apk_argmax_rows_noalloc(apk_ctx* ctx, const float* logits, size_t rows,
                                                                              size_t n, uint32_t* out) {
    if (!ctx) return apk_fail(APK_DECLINE_NULL, "apk_argmax_rows_noalloc: ctx is NULL");
    const int device = apk_ctx_device(ctx);
    if (rows > APK_NOALLOC_MAX_ROWS)
        return apk_fail(APK_DECLINE_SHAPE, "apk_argmax_rows_noalloc: %zu rows, the static scratch holds %d (use apk_argmax_rows)", rows,
                        APK_NOALLOC_MAX_ROWS);
    if (device < 0 || device >= kMaxDevices) return apk_fail(APK_DECLINE_NO_DEVICE, "apk_argmax_rows_noalloc: device %d", device);
    void* p;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        p = g_status[device] == 1 ? g_ptr[device] : nullptr;
    }
    if (!p) return apk_fail(APK_DECLINE_NO_DEVICE, "apk_argmax_rows_noalloc: no scratch address for device %d (apk_init looks it up)", device);
    // the array keeps whatever the last call left (nothing, unless that call was cut short): the rows' lines are
    // cleared by a fill kernel ahead of the launch, on the same stream
    return apk_argmax_launch(ctx, logits, rows, n, out, p, true);
}
