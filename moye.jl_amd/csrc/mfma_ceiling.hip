// What the matrix pipe of this part sustains with nothing else going on: every wave of every CU
// issues independent MFMAs on register operands in a loop, no memory traffic at all.  The rate
// depends on the operand bits (dense random operands draw more power than zeros and the clock
// drops), so the probe reports both the TFLOP/s and the clock the loop actually ran at (cycle
// counter over wall time).  It is the yardstick the GEMM kernels' MFMA-roofline fractions are read
// against; it computes nothing a caller could use.
#include <algorithm>
#include <vector>

#include "mfma_common.hpp"

namespace moye {

template <typename In>
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(const u32x4* __restrict__ in, float* __restrict__ out,
                                                           unsigned long long* __restrict__ ticks, int iters) {
    const u32x4 a = in[threadIdx.x], b = in[threadIdx.x + 512];
    f32x4 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) In::mma(a, b, acc[i]);
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    f32x4 s = acc[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) s += acc[i];
    out[(size_t)blockIdx.x * 512 + threadIdx.x] = s.x + s.y + s.z + s.w;
    if ((threadIdx.x & 63) == 0) {  // per wave: the older wave of a SIMD wins the pipe and finishes first
        ticks[((size_t)blockIdx.x * 8 + threadIdx.x / 64) * 2] = t0;
        ticks[((size_t)blockIdx.x * 8 + threadIdx.x / 64) * 2 + 1] = t1;
    }
}

template <typename In>
static void launch_ceiling(int blocks, const u32x4* in, float* out, unsigned long long* ticks, int iters, hipStream_t st) {
    mfma_ceiling_kernel<In><<<blocks, 512, 0, st>>>(in, out, ticks, iters);
}

// flops of one In::mma call per wave (16 x 16 x K, two flops per multiply-add)
static double flops_per_mma(int32_t in_dt) {
    switch (in_dt) {
        case MOYE_F8E4M3: return 2.0 * 16 * 16 * 64;  // two 16x16x32 instructions per 16-byte chunk pair
        case MOYE_F32: return 2.0 * 16 * 16 * 16;     // four 16x16x4
        default: return 2.0 * 16 * 16 * 32;
    }
}

int32_t mfma_ceiling(int32_t in_dt, int32_t random_operands, float seconds, float* tflops, float* clock_ghz, hipStream_t st) {
    if (!tflops || !clock_ghz) return fail(MOYE_ERR_ARG, "moye_mfma_ceiling: null output");
    if (!(seconds > 0.f) || seconds > 5.f) return fail(MOYE_ERR_ARG, "moye_mfma_ceiling: duration must be in (0, 5] seconds");
    int dev = 0, cus = 0;
    MOYE_HIP_CHECK(hipGetDevice(&dev));
    MOYE_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int blocks = cus;  // one workgroup of 8 waves per CU: two waves per SIMD, like the GEMM kernels
    u32x4* in = nullptr;
    float* out = nullptr;
    unsigned long long* ticks = nullptr;
    MOYE_HIP_CHECK(hipMalloc(&in, 1024 * sizeof(u32x4)));
    MOYE_HIP_CHECK(hipMalloc(&out, (size_t)blocks * 512 * sizeof(float)));
    MOYE_HIP_CHECK(hipMalloc(&ticks, (size_t)blocks * 16 * sizeof(unsigned long long)));
    {
        // operands: zeros, or pseudo-random finite values of the input type with mixed signs and a
        // spread of exponents (16-bit types: sign, 4 exponent bits around 1/64..1/4, full mantissa)
        std::vector<uint32_t> h(4096, 0u);
        if (random_operands) {
            uint32_t x = 12345u;
            for (auto& w : h) {
                uint32_t bits = 0;
                if (in_dt == MOYE_F32) {
                    x = x * 1664525u + 1013904223u;
                    bits = 0x3c000000u | (x & 0x83ffffffu);
                } else if (in_dt == MOYE_F8E4M3) {
                    for (int k = 0; k < 4; ++k) {
                        x = x * 1664525u + 1013904223u;
                        bits |= (uint32_t)(0x20u | ((x >> 16) & 0x9fu)) << (8 * k);
                    }
                } else {
                    for (int k = 0; k < 2; ++k) {
                        x = x * 1664525u + 1013904223u;
                        const uint32_t hbits = in_dt == MOYE_F16 ? (0x2000u | ((x >> 16) & 0x83ffu)) : (0x3c00u | ((x >> 16) & 0x81ffu));
                        bits |= hbits << (16 * k);
                    }
                }
                w = bits;
            }
        }
        MOYE_HIP_CHECK(hipMemcpy(in, h.data(), h.size() * 4, hipMemcpyHostToDevice));
    }
    auto launch = [&](int iters) {
        switch (in_dt) {
            case MOYE_F16: launch_ceiling<InF16>(blocks, in, out, ticks, iters, st); break;
            case MOYE_BF16: launch_ceiling<InBF16>(blocks, in, out, ticks, iters, st); break;
            case MOYE_F8E4M3: launch_ceiling<InFP8>(blocks, in, out, ticks, iters, st); break;
            default: launch_ceiling<InF32>(blocks, in, out, ticks, iters, st); break;
        }
    };
    int32_t rc = MOYE_OK;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) rc = fail(MOYE_ERR_HIP, "moye_mfma_ceiling: event creation failed");
    if (!rc && (in_dt != MOYE_F16 && in_dt != MOYE_BF16 && in_dt != MOYE_F8E4M3 && in_dt != MOYE_F32))
        rc = fail(MOYE_ERR_UNSUPPORTED, "moye_mfma_ceiling: no MFMA atom for %s inputs", dtype_name(in_dt));
    if (!rc) {
        // launches of about 2 ms each until `seconds` have passed; the last one is the measurement
        const int iters = in_dt == MOYE_F32 ? 500 : 4000;
        float ms = 0.f, total = 0.f;
        do {
            (void)hipEventRecord(e0, st);
            launch(iters);
            (void)hipEventRecord(e1, st);
            if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) {
                rc = fail(MOYE_ERR_HIP, "moye_mfma_ceiling: launch failed");
                break;
            }
            total += ms;
        } while (total < seconds * 1e3f);
        if (!rc) {
            std::vector<unsigned long long> h((size_t)blocks * 16);
            if (hipMemcpy(h.data(), ticks, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost) != hipSuccess) {
                rc = fail(MOYE_ERR_HIP, "moye_mfma_ceiling: read-back failed");
            } else {
                double avg = 0;  // per workgroup: first wave in to last wave out
                for (int b = 0; b < blocks; ++b) {
                    unsigned long long lo = ~0ull, hi = 0;
                    for (int w = 0; w < 8; ++w) {
                        lo = std::min(lo, h[((size_t)b * 8 + w) * 2]);
                        hi = std::max(hi, h[((size_t)b * 8 + w) * 2 + 1]);
                    }
                    avg += (double)(hi - lo);
                }
                avg /= blocks;
                *clock_ghz = (float)(avg / (ms * 1e6));
                *tflops = (float)((double)blocks * 8 * iters * 16 * flops_per_mma(in_dt) / (ms * 1e9));
            }
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(in);
    (void)hipFree(out);
    (void)hipFree(ticks);
    return rc;
}

}  // namespace moye
