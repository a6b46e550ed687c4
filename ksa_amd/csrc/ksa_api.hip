// Library-level entry points of libksa_hip.so.
#include <hip/hip_runtime.h>

#include "ksa_api_internal.h"

extern "C" int ksa_version(void) { return 102; }

extern "C" const char* ksa_error_string(int code) {
    switch (code) {
        case KSA_OK: return "ok";
        case KSA_ERR_INVALID: return "invalid size or flag argument";
        case KSA_ERR_NULL: return "required pointer is null";
        case KSA_ERR_UNSUPPORTED: return "dtype or head_dim not supported (bf16/fp16; attention: head_dim 64, 128 or 256; pre-attention: 64 or 128)";
        case KSA_ERR_WORKSPACE: return "workspace missing or too small";
        case KSA_ERR_LAUNCH: return "HIP kernel launch failed";
        case KSA_ERR_ALIGN: return "pointers must be 16-byte aligned and strides multiples of 8 elements";
        default: return "unknown error";
    }
}

// Number of compute units of the current device (0 if no device is usable).
extern "C" int ksa_device_cu_count(void) {
    return ksa_cu_count_or(0);
}
