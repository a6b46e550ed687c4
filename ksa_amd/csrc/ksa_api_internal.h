// Internal helpers shared by the translation units of libksa_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// status codes returned by every extern "C" entry point (0 = success)
enum {
    KSA_OK = 0,
    KSA_ERR_INVALID = -1,      // a size / flag argument is out of range
    KSA_ERR_NULL = -2,         // a required pointer is null
    KSA_ERR_UNSUPPORTED = -3,  // dtype / head_dim not compiled in
    KSA_ERR_WORKSPACE = -4,    // workspace too small
    KSA_ERR_LAUNCH = -5,       // the HIP runtime refused the launch
    KSA_ERR_ALIGN = -6,        // pointer or stride not 16-byte aligned
};

enum { KSA_DTYPE_BF16 = 0, KSA_DTYPE_F16 = 1 };

// value of a weight matrix's row stride that names the streaming layout instead (include/ksa_hip.h, KSA_W_TILED)
constexpr long long kWTiled = -1;

// most rows of x that the few-rows GEMM (ksa_gemm_rows) and the consumers of its K-split partial sums take
constexpr int kMaxPartialRows = 128;

// size of the fixed device array behind ksa_decode_fwd_noalloc (32 MiB; include/ksa_hip.h states it too)
#define KSA_DECODE_NOALLOC_SCRATCH_BYTES (32u << 20)

static inline int ksa_check_launch() {
    return hipGetLastError() == hipSuccess ? KSA_OK : KSA_ERR_LAUNCH;
}

// Compute units of the current device, or `fallback` when no device can be asked (host-only use
// of the heuristics).
static inline int ksa_cu_count_or(int fallback) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fallback;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return fallback;
    return n;
}
