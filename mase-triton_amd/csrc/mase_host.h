// Host-side helpers shared by the C-ABI entry points: error reporting and argument checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <algorithm>
#include <atomic>
#include <string>

#include "mase_device.h"

namespace mase {

enum Status : int { OK = 0, ERR_INVALID = -1, ERR_UNSUPPORTED = -2, ERR_RUNTIME = -3 };

std::string& last_error();  // thread-local message of the most recent failure

inline int fail(int code, const std::string& msg) {
    last_error() = msg;
    return code;
}

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(ERR_RUNTIME, std::string(what) + ": " + hipGetErrorString(e));
    return OK;
}

// A kernel that uses more than 64 KB of dynamic LDS has to be given the limit once on every device it runs on (the
// attribute belongs to the function as loaded on the current device).  `done` is the call site's record: bit d = set on
// device d; devices past 63 set it on every launch.  Safe from several threads (setting it twice is harmless).
inline int allow_dynamic_lds(const void* kern, int bytes, std::atomic<uint64_t>& done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(ERR_RUNTIME, std::string("hipGetDevice: ") + hipGetErrorString(e));
    const uint64_t bit = dev >= 0 && dev < 64 ? uint64_t(1) << dev : 0;
    if (bit && (done.load(std::memory_order_relaxed) & bit)) return OK;
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail(ERR_RUNTIME, std::string("hipFuncSetAttribute: ") + hipGetErrorString(e));
    done.fetch_or(bit, std::memory_order_relaxed);
    return OK;
}

// compute units of the current device (at least 8), or -1
inline int device_cu_count() {
    static std::atomic<int> cus[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return -1;
    const bool cached = dev >= 0 && dev < 64;
    int n = cached ? cus[dev].load(std::memory_order_relaxed) : 0;
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -1;
        n = n > 8 ? n : 8;
        if (cached) cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

inline int check_minifloat_fmt(int E, int M, int rm) {
    if (E < 1 || M < 1 || E + M >= 16) return fail(ERR_INVALID, "minifloat format needs exp_bits >= 1, frac_bits >= 1, exp_bits + frac_bits < 16");
    if (rm < RN || rm > RZ) return fail(ERR_INVALID, "round_mode must be 0 (rn), 1 (ru), 2 (rd) or 3 (rz)");
    return OK;
}

inline int check_mxfp_fmt(int E, int M, int rm, int64_t n, int block) {
    const bool legal = (E == 4 && M == 3) || (E == 5 && M == 2) || (E == 2 && M == 3) || (E == 3 && M == 2) ||
                       (E == 2 && M == 1);
    if (!legal) return fail(ERR_INVALID, "MXFP element (exp_bits, frac_bits) must be one of (4,3) (5,2) (2,3) (3,2) (2,1)");
    if (rm < RN || rm > RZ) return fail(ERR_INVALID, "round_mode must be 0 (rn), 1 (ru), 2 (rd) or 3 (rz)");
    if (block < 1) return fail(ERR_INVALID, "block_size must be positive");
    if (n < 0 || n % block != 0) return fail(ERR_INVALID, "element count must be a non-negative multiple of block_size");
    return OK;
}

inline int check_dtype(int dt, const char* which) {
    if (dt != F32 && dt != F16 && dt != BF16) return fail(ERR_INVALID, std::string(which) + " dtype must be 0 (f32), 1 (f16) or 2 (bf16)");
    return OK;
}

inline int dtype_size(int dt) { return dt == F32 ? 4 : 2; }

// Calls fn(format object): a compile-time format for the five round-to-nearest finite
// presets, the run-time one otherwise.
template <class Fn>
inline int dispatch_fmt(int E, int M, int fin, int rm, Fn&& fn) {
    if (fin && rm == RN) {
        if (E == 4 && M == 3) return fn(SFmt<4, 3>{});
        if (E == 5 && M == 2) return fn(SFmt<5, 2>{});
        if (E == 2 && M == 3) return fn(SFmt<2, 3>{});
        if (E == 3 && M == 2) return fn(SFmt<3, 2>{});
        if (E == 2 && M == 1) return fn(SFmt<2, 1>{});
    }
    return fn(DFmt{E, M, fin, rm});
}

template <int V> struct IntC { static constexpr int value = V; };

template <class Fn>
inline int dispatch_dtype(int dt, Fn&& fn) {
    switch (dt) {
        case F32: return fn(IntC<F32>{});
        case F16: return fn(IntC<F16>{});
        default: return fn(IntC<BF16>{});
    }
}

}  // namespace mase
