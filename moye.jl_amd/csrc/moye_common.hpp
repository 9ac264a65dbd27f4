// Shared host-side helpers of libmoye_hip: status/error text, dtype table, tensor validation.
#pragma once

#include <hip/hip_runtime.h>

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

}  // namespace moye
