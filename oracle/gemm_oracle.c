/*
 * CPU restatement of MoYe's `gemm!` with the UniversalFMA atom over host arrays, and of the
 * element loop of `copyto!`.  TEST INFRASTRUCTURE ONLY: tests, the smoke check and the
 * cpu_baseline leg of bench.py load this; the shipped library never does.
 *
 * Follows (YichengDWu/MoYe.jl v4.0.1):
 *   src/algorithm/blas.jl:39-88   dispatch tower: k outermost ascending, then n, then m serpentine
 *   src/arch/mma/mma.jl:64        fma!: d = a * b + c, product rounded in promote_type(TA,TB),
 *                                 the add in the accumulator type, never fused
 *   test/device/matmul.jl:40-49   k-tile loop around gemm! (tiles of bM x bN x bK)
 *   src/algorithm/copy.jl:4-12    copyto!: logical element i -> logical element i
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (see build.py).  Contraction must stay
 * off or the compiler fuses the multiply and the add.
 *
 * Pinned by tests/test_oracle_c.py against the numpy restatement (bit-exact), hand-built
 * rounding cases, and numpy's own float16 conversion.
 */
#include <stdint.h>
#include <string.h>

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> nearest fp16 (ties to even) -> fp32 */
float moye_ref_round_f16(float f) {
    uint32_t u = f2u(f), sign = u & 0x80000000u, a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return f;                         /* inf / nan */
    if (a >= 0x477ff000u) return u2f(sign | 0x7f800000u);   /* >= 65520 rounds to inf */
    if (a < 0x38800000u) {                                  /* below 2^-14: fp16 subnormal grid 2^-24 */
        const float mag = u2f(a);
        const float magic = 0.5f;                           /* ulp of [0.5,1) is 2^-24 */
        const float t = (mag + magic) - magic;              /* mag rounded to a multiple of 2^-24, RNE */
        return u2f(sign | f2u(t));
    }
    a += 0xfffu + ((a >> 13) & 1u);                         /* RNE at 10 mantissa bits */
    a &= 0xffffe000u;
    return u2f(sign | a);
}

/* fp32 -> nearest bf16 (ties to even) -> fp32 */
float moye_ref_round_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return f;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u2f(u & 0xffff0000u);
}

static inline float round_prod(float p, int prod_type) {
    return prod_type == 1 ? moye_ref_round_f16(p) : prod_type == 2 ? moye_ref_round_bf16(p) : p;
}

/*
 * C(M,N) = A(M,K) * B(N,K)' + C, all operands fp32 storage with element strides; values of A and B
 * are representable in the operand type named by prod_type (0 fp32, 1 fp16, 2 bf16).
 * bm/bn/bk: CTA-style tiling of the loop nest (e.g. 32,32,8); threads > 1 splits C tiles over
 * OpenMP threads (each C element is still produced by one thread in the same order).
 */
void moye_ref_gemm(int M, int N, int K, const float* A, long sa_m, long sa_k, const float* B, long sb_n,
                   long sb_k, float* C, long sc_m, long sc_n, int prod_type, int bm, int bn, int bk,
                   int threads) {
    const int tm = (M + bm - 1) / bm, tn = (N + bn - 1) / bn;
#pragma omp parallel for collapse(2) schedule(static) num_threads(threads) if (threads > 1)
    for (int bi = 0; bi < tm; ++bi)
        for (int bj = 0; bj < tn; ++bj) {
            const int m0 = bi * bm, n0 = bj * bn;
            const int m1 = m0 + bm < M ? m0 + bm : M, n1 = n0 + bn < N ? n0 + bn : N;
            for (int k0 = 0; k0 < K; k0 += bk) {
                const int k1 = k0 + bk < K ? k0 + bk : K;
                for (int k = k0; k < k1; ++k)                   /* blas.jl:83-85 */
                    for (int n = n0; n < n1; ++n)               /* blas.jl:63 */
                        for (int i = m0; i < m1; ++i) {         /* blas.jl:64-65, serpentine */
                            const int m = ((n - n0) & 1) ? (m1 - 1 - (i - m0)) : i;
                            const float p = round_prod(A[m * sa_m + k * sa_k] * B[n * sb_n + k * sb_k], prod_type);
                            float* c = C + m * sc_m + n * sc_n;
                            *c = p + *c;                        /* mma.jl:64 */
                        }
            }
        }
}

/* copyto!(dst, src): flattened layouts of equal size, elements of `bytes` bytes */
void moye_ref_copy(int rank_d, const long* shape_d, const long* stride_d, int rank_s, const long* shape_s,
                   const long* stride_s, char* dst, const char* src, long n, int bytes) {
    for (long i = 0; i < n; ++i) {
        long r = i, od = 0, os = 0;
        for (int m = 0; m < rank_d; ++m) { od += (r % shape_d[m]) * stride_d[m]; r /= shape_d[m]; }
        r = i;
        for (int m = 0; m < rank_s; ++m) { os += (r % shape_s[m]) * stride_s[m]; r /= shape_s[m]; }
        memcpy(dst + od * bytes, src + os * bytes, (size_t)bytes);
    }
}
