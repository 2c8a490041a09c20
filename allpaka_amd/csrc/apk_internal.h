// Internal to libapk_hip.so (not installed, not part of the C ABI): what the translation units of the library share.
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "apk_hip.h"

// apk_noalloc.hip: looks up, for the current device, the address of the library's static device scratch array
// (once per device; later calls return the stored result).  0 or -(hipError_t).
int apk_noalloc_setup(int device);

// apk_host.cpp: the argmax launch both apk_argmax_rows entries share.  scratch: 128 bytes per row, device memory.
// clear_first: zero the rows' scratch lines with a fill kernel on the context's stream before the launch.
int apk_argmax_launch(apk_ctx* c, const float* logits, size_t rows, size_t n, uint32_t* out, void* scratch, bool clear_first);
// apk_host.cpp: the device a context was created on.
int apk_ctx_device(apk_ctx* c);
// apk_host.cpp: sets the calling thread's apk_last_error text and returns status.
int apk_fail(int status, const char* fmt, ...);
