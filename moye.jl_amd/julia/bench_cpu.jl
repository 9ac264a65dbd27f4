# Times the reference's own CPU path (MoYe.jl `gemm!` with UniversalFMA over host arrays, tiled
# as in test/host/tiling_matmul.jl) so that it can be quoted beside the GPU numbers when a Julia
# runtime with MoYe.jl installed is available.  Not executed in this repository's environment.
#
#   julia -t 16 bench_cpu.jl [n]      # n defaults to 512; prints JSON
using MoYe, LinearAlgebra

function tiled_matmul!(C, A, B, bM, bN, bK)
    M, N, K = size(A, 1), size(B, 1), size(A, 2)
    mA, mB, mC = MoYeArray(A), MoYeArray(B), MoYeArray(C)
    Threads.@threads :static for t in 0:(cld(M, bM) * cld(N, bN) - 1)
        i, j = t % cld(M, bM) + 1, t ÷ cld(M, bM) + 1
        gC = @tile mC (bM, bN) (i, j)
        for k in 1:cld(K, bK)
            gA = @tile mA (bM, bK) (i, k)
            gB = @tile mB (bN, bK) (j, k)
            MoYe.gemm!(gA, gB, gC)
        end
    end
    C
end

n = length(ARGS) >= 1 ? parse(Int, ARGS[1]) : 512
A = Float32.(Float16.(randn(Float32, n, n) ./ 64))
B = Float32.(Float16.(randn(Float32, n, n) ./ 64))
C = zeros(Float32, n, n)
tiled_matmul!(C, A, B, static(32), static(32), static(8))            # compile
fill!(C, 0)
t = @elapsed tiled_matmul!(C, A, B, static(32), static(32), static(8))
@assert C ≈ A * B'
println("{\"kind\": \"reference\", \"n\": $n, \"threads\": $(Threads.nthreads()), \"seconds\": $t, ",
        "\"tflops\": $(2.0 * n^3 / t / 1e12)}")
