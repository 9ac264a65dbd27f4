// Shared host-side helpers of libmoye_hip: status/error text, dtype table, tensor validation.
#pragma once
#include <algorithm>

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/moye_hip.h"

namespace moye {

// Thread-local text of the last failure; every C entry point funnels through fail().
std::string& last_error();
int32_t fail(moye_status st, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define MOYE_HIP_CHECK(expr)                                                              \
    do {                                                                                  \
        hipError_t _e = (expr);                                                           \
        if (_e != hipSuccess)                                                             \
            return ::moye::fail(MOYE_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

// A kernel that needs more dynamic LDS than the default cap has the cap raised once per device.  The call is
// idempotent, so two host threads that launch for the first time may both make it; the flag only saves later calls.
struct LdsCap {
    std::atomic<uint64_t> raised{0};  // bit d: done on device d
};
inline int32_t raise_lds_cap(LdsCap& cap, const void* kernel, int bytes) {
    int dev = 0;
    MOYE_HIP_CHECK(hipGetDevice(&dev));
    const uint64_t bit = 1ull << (dev & 63);
    if (cap.raised.load(std::memory_order_acquire) & bit) return MOYE_OK;
    MOYE_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    cap.raised.fetch_or(bit, std::memory_order_release);
    return MOYE_OK;
}

// Kernels that give every lane one piece and do not loop.  A launch holds fewer than 2^32 work-items per grid dimension,
// so from 2^22 workgroups of 256 on (16 GiB of 16-byte pieces) the rest of the workgroups go into the grid's second
// dimension; the lanes past the last piece of the last row of workgroups find nothing to do.
constexpr unsigned kFlatGridX = 1u << 22;
inline dim3 flat_grid(int64_t pieces) {
    const int64_t blocks = pieces > 0 ? (pieces + 255) / 256 : 1;
    if (blocks <= (int64_t)kFlatGridX) return dim3((unsigned)blocks);
    return dim3(kFlatGridX, (unsigned)((blocks + kFlatGridX - 1) / kFlatGridX));
}
#if defined(__HIPCC__)
__device__ __forceinline__ int64_t flat_piece() { return ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * 256 + threadIdx.x; }
#endif
// Kernels whose lanes walk the pieces with a stride of the whole grid: as many workgroups as pieces, up to 2^22.
inline dim3 strided_grid(int64_t pieces) {
    return dim3((unsigned)std::min<int64_t>(std::max<int64_t>(1, (pieces + 255) / 256), (int64_t)kFlatGridX));
}

inline int dtype_bytes(int32_t dt) {
    switch (dt) {
        case MOYE_F32: case MOYE_U32: return 4;
        case MOYE_F16: case MOYE_BF16: case MOYE_U16: return 2;
        case MOYE_F8E4M3: case MOYE_U8: return 1;
        case MOYE_F64: case MOYE_U64: return 8;
        case MOYE_U128: return 16;
        default: return 0;
    }
}

inline const char* dtype_name(int32_t dt) {
    static const char* n[] = {"f32", "f16", "bf16", "f8e4m3", "f64", "u8", "u16", "u32", "u64", "u128"};
    return (dt >= 0 && dt <= MOYE_U128) ? n[dt] : "?";
}

inline bool is_float_dtype(int32_t dt) { return dt >= MOYE_F32 && dt <= MOYE_F64; }

inline int64_t tensor_size(const moye_tensor& t) {
    int64_t n = 1;
    for (int i = 0; i < t.rank; ++i) n *= t.shape[i];
    return n;
}

// Largest element offset + 1 the layout can reach (cosize for non-negative strides).
inline int64_t tensor_cosize(const moye_tensor& t) {
    int64_t n = 1;
    for (int i = 0; i < t.rank; ++i) n += (t.shape[i] - 1) * t.stride[i];
    return n;
}

// Common checks on a tensor argument; `what` names it in the message.
int32_t check_tensor(const moye_tensor* t, const char* what);

// A rank-2 view (rows, cols) of a tensor: modes 0 and 1.
struct Mat {
    char* ptr;
    int64_t rows, cols, rs, cs;  // sizes and element strides
    int32_t dtype;
};
int32_t as_matrix(const moye_tensor* t, const char* what, Mat* m);

// An elementwise operation over arrays of one shape, mode by mode, takes coordinate c of every operand: the order in
// which the coordinates are visited is free.  Visit them along the smallest strides of the first layout (the
// destination), then of the second, so that neighbouring lanes touch neighbouring memory whatever the order the caller
// wrote the modes in (a row-major array handed over as shape (rows, cols), strides (pitch, 1) has its unit stride on
// the last mode).  L has rank, shape[], stride[]; the same permutation is applied to every layout; returns false, and
// changes nothing, when ranks or shapes differ.
template <class L>
inline bool order_modes_by_stride(L* const* layouts, int count) {
    const L& first = *layouts[0];
    const int r = first.rank;
    for (int q = 1; q < count; ++q) {
        if (layouts[q]->rank != r) return false;
        for (int m = 0; m < r; ++m)
            if (layouts[q]->shape[m] != first.shape[m]) return false;
    }
    int perm[MOYE_MAX_RANK];
    for (int m = 0; m < r; ++m) perm[m] = m;
    std::stable_sort(perm, perm + r, [&](int a, int b) {
        const bool one_a = first.shape[a] == 1, one_b = first.shape[b] == 1;  // modes of one element go last
        if (one_a != one_b) return one_b;
        for (int q = 0; q < count; ++q)
            if (layouts[q]->stride[a] != layouts[q]->stride[b]) return layouts[q]->stride[a] < layouts[q]->stride[b];
        return false;
    });
    for (int q = 0; q < count; ++q) {
        const L old = *layouts[q];
        for (int m = 0; m < r; ++m) {
            layouts[q]->shape[m] = old.shape[perm[m]];
            layouts[q]->stride[m] = old.stride[perm[m]];
        }
    }
    return true;
}

}  // namespace moye
