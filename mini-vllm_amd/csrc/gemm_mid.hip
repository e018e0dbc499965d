// Matrix product for a few dozen rows against a large weight (decode steps of 17 to 64 sequences
// on models whose weights take tens of megabytes per matrix):
//     C[M, N] = A[M, K] * W[N, K]^T (+ bias)      or      C[M, I] = silu(A Wg^T) * (A Wu^T),
// M <= 64, bf16 inputs, float accumulation, on the MFMA units of gfx950.
//
// Each weight is still read from HBM exactly once, but here the activation rows, which every
// weight tile needs, weigh as much as the weights themselves. So a workgroup (4 waves) takes
// 64 * R weight rows and a slice of K, stages the activation rows of that slice through LDS once
// for all its waves (chunks of 128 columns, double-buffered, written in the order the MFMA operands
// are read), and every wave multiplies its R tiles of 16 weight rows, loaded straight from global
// memory one chunk ahead, with all token tiles. K is split over `F` workgroups so that the
// chip is filled although there are few weight tiles; with F > 1 the partial sums go to a float
// work area [F][M][N] and a second kernel adds them in a fixed order (no atomics: a row's result
// does not depend on what else runs), applies bias or the gated activation, and rounds.
#include "dispatch.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    uint16_t s[8];
    bf16x8_t v;
};

#define GM_WAVES 4
#define GM_THREADS (64 * GM_WAVES)
#ifndef GM_KC
#define GM_KC 128          // columns of a chunk
#endif
#define GM_KS (GM_KC / 32)  // MFMA steps of a chunk
#define GM_COMPUTE_UNITS 256

// R: tiles of 16 weight rows per wave; TM: tiles of 16 tokens (M <= 16 * TM).
template <int R, int TM>
__global__ void __launch_bounds__(GM_THREADS)
gemm_mid_kernel(const bf16* __restrict__ A, long lda, const bf16* __restrict__ W, float* __restrict__ part, int M,
                int N, int K, int F, int chunks_per_split) {
    __shared__ uint4 sA[2][TM * GM_KS * 64];  // [buffer][(token tile * GM_KS + k-step) * 64 + operand lane]
    const int tid = threadIdx.x;
    const int wave = tid / MV_WAVE;
    const int lane = tid % MV_WAVE;
    const int i = lane % 16;
    const int g = lane / 16;
    const int f = blockIdx.x % F;            // neighbouring workgroups take the splits of one row block
    const int nblock = blockIdx.x / F;
    const int n_base = (nblock * GM_WAVES + wave) * R * 16;
    const int chunks_total = K / GM_KC;
    const int c0 = f * chunks_per_split;
    int c1 = c0 + chunks_per_split;
    if (c1 > chunks_total) c1 = chunks_total;

    const uint4* wrow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int row = n_base + 16 * r + i;
        if (row > N - 1) row = N - 1;        // rows past the end are loaded again and never stored
        wrow[r] = reinterpret_cast<const uint4*>(W + (size_t)row * K) + g;
    }
    // which chunks of the activation tile this thread copies (its place in LDS follows its id)
    constexpr int AREP = TM * GM_KS * 64 / GM_THREADS;
    const uint4* asrc[AREP];
    bool avalid[AREP];
#pragma unroll
    for (int rep = 0; rep < AREP; ++rep) {
        const int L = tid + GM_THREADS * rep;          // (token tile * GM_KS + k-step) * 64 + operand lane
        const int ol = L % 64, ks = (L / 64) % GM_KS, t = L / (64 * GM_KS);
        const int tok = 16 * t + ol % 16;
        avalid[rep] = tok < M;
        asrc[rep] = reinterpret_cast<const uint4*>(A + (size_t)(avalid[rep] ? tok : 0) * lda + 32 * ks) + ol / 16;
    }

    floatx4_t acc[R][TM];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < TM; ++t) acc[r][t] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    struct Stage {
        Frag w[GM_KS][R];
        uint4 a[AREP];
    };
    auto fetch = [&](int c, Stage& st) {
        if (c >= c1) return;
        const size_t k16 = (size_t)c * (GM_KC / 8);    // offset of the chunk in 16-byte units
#pragma unroll
        for (int ks = 0; ks < GM_KS; ++ks)
#pragma unroll
            for (int r = 0; r < R; ++r) st.w[ks][r].u = wrow[r][k16 + 4 * ks];
#pragma unroll
        for (int rep = 0; rep < AREP; ++rep) st.a[rep] = avalid[rep] ? asrc[rep][k16] : uint4{0u, 0u, 0u, 0u};
    };
    auto stash = [&](int c, const Stage& st) {
        if (c >= c1) return;
#pragma unroll
        for (int rep = 0; rep < AREP; ++rep) sA[(c - c0) & 1][tid + GM_THREADS * rep] = st.a[rep];
    };
    auto multiply = [&](int c, const Stage& st) {
        const uint4* a = sA[(c - c0) & 1];
#pragma unroll
        for (int ks = 0; ks < GM_KS; ++ks) {
            Frag af[TM];
#pragma unroll
            for (int t = 0; t < TM; ++t) af[t].u = a[(t * GM_KS + ks) * 64 + lane];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < TM; ++t)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.w[ks][r].v, af[t].v, acc[r][t], 0, 0, 0);
        }
    };

    // chunk c is multiplied from LDS and `s0` while the weights and activations of chunk c + 1 are
    // on their way into `s1`
    Stage s0, s1;
    fetch(c0, s0);
    stash(c0, s0);
    __syncthreads();
    for (int c = c0; c < c1; c += 2) {
        fetch(c + 1, s1);
        multiply(c, s0);
        stash(c + 1, s1);
        __syncthreads();
        if (c + 1 >= c1) break;
        fetch(c + 2, s0);
        multiply(c + 1, s1);
        stash(c + 2, s0);
        __syncthreads();
    }

    // lane l holds C[token 16 t + l%16][n_base + 16 r + 4 (l/16) + 0..3]
    float* dst = part + (size_t)f * M * N;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const int tok = 16 * t + i;
            const int col = n_base + 16 * r + 4 * g;
            if (tok >= M || col >= N) continue;
            float* p = dst + (size_t)tok * N + col;
            if (col + 3 < N && (N & 3) == 0) {
                *reinterpret_cast<float4*>(p) = float4{acc[r][t][0], acc[r][t][1], acc[r][t][2], acc[r][t][3]};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < N) p[e] = acc[r][t][e];
            }
        }
}

// out[m][n] = sum_f part[f][m][n] (+ bias[n]), or with `swiglu` out[m][i] = silu(gate) * up with
// gate = sum_f part[f][m][i], up = sum_f part[f][m][I + i], N = 2 I.
template <typename TC>
__global__ void gemm_mid_reduce_kernel(const float* __restrict__ part, const bf16* __restrict__ bias,
                                       TC* __restrict__ C, long ldc, int M, int N, int F, int swiglu) {
    const int n_out = swiglu ? N / 2 : N;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)M * n_out) return;
    const int m = (int)(idx / n_out), n = (int)(idx % n_out);
    const size_t plane = (size_t)M * N;
    float a = 0.f, b = 0.f;
    for (int f = 0; f < F; ++f) {
        a += part[f * plane + (size_t)m * N + n];
        if (swiglu) b += part[f * plane + (size_t)m * N + n_out + n];
    }
    float v;
    if (swiglu) {
        v = a / (1.f + expf(-a)) * b;
    } else {
        v = a;
        if (bias) v += to_f(bias[n]);
    }
    C[(size_t)m * ldc + n] = from_f<TC>(v);
}

struct MidPlan {
    int R, F, chunks_per_split, blocks;
};

// Rows per workgroup and splits of K: enough workgroups for every compute unit to hold two, as few
// splits as that allows (their partial sums cost traffic), and at least two chunks per split.
static MidPlan mid_plan(int N, int K) {
    const int chunks = K / GM_KC;
    // 64 weight rows per workgroup (measured on MI355X against 128: faster at every shape tried),
    // and as many splits of K as bring about two workgroups to every compute unit
    const int R = 1;
    const int nblocks = (N + 64 * R - 1) / (64 * R);
    int F = (2 * GM_COMPUTE_UNITS + nblocks - 1) / nblocks;
    if (F > chunks / 2) F = chunks / 2;
    if (F < 1) F = 1;
    if (F > 32) F = 32;
    const int cps = (chunks + F - 1) / F;
    F = (chunks + cps - 1) / cps;
    MidPlan best{R, F, cps, nblocks};
    return best;
}

// Floats of work area a product of this shape needs (the partial sums [F][M][N]).
extern "C" long mv_gemm_mid_workspace(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % GM_KC) return 0;
    const MidPlan p = mid_plan(N, K);
    return (long)p.F * M * N;
}

// c_dtype: MV_BF16 or MV_F32. With `swiglu`, W is the packed gate/up weight [N = 2 I, K] and C is
// [M, I]. `work` holds at least mv_gemm_mid_workspace(M, N, K) floats.
extern "C" int mv_gemm_mid(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int c_dtype,
                           int M, int N, int K, int swiglu, float* work, long work_floats, hipStream_t stream) {
    MV_REQUIRE(M > 0 && M <= 64, "gemm_mid: takes 1 to 64 rows, got M=%d", M);
    MV_REQUIRE(N > 0 && K > 0 && K % GM_KC == 0, "gemm_mid: K=%d must be a positive multiple of %d (N=%d)", K, GM_KC, N);
    MV_REQUIRE(lda >= K && lda % 8 == 0, "gemm_mid: lda=%ld must be a multiple of 8 and at least K=%d", lda, K);
    MV_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_mid: operands must be 16-byte aligned");
    MV_REQUIRE(!swiglu || (N % 2 == 0 && bias == nullptr), "gemm_mid: the gated form takes an even N and no bias");
    MV_REQUIRE(ldc >= (swiglu ? N / 2 : N), "gemm_mid: ldc=%ld too small for N=%d", ldc, N);
    MV_REQUIRE(c_dtype == MV_F32 || c_dtype == MV_BF16, "gemm_mid: bad output dtype %d", c_dtype);
    const MidPlan p = mid_plan(N, K);
    MV_REQUIRE(work != nullptr && ((uintptr_t)work % 16) == 0 && work_floats >= (long)p.F * M * N,
               "gemm_mid: the work area holds %ld floats, %ld are needed", work_floats, (long)p.F * M * N);
    const dim3 grid((unsigned)(p.blocks * p.F));
    const int TM = (M + 15) / 16;
#define GM_LAUNCH(RR, TT)                                                                                          \
    hipLaunchKernelGGL((gemm_mid_kernel<RR, TT>), grid, dim3(GM_THREADS), 0, stream, (const bf16*)A, lda,           \
                       (const bf16*)W, work, M, N, K, p.F, p.chunks_per_split)
    if (p.R == 2) {
        if (TM == 1) GM_LAUNCH(2, 1);
        else if (TM == 2) GM_LAUNCH(2, 2);
        else if (TM == 3) GM_LAUNCH(2, 3);
        else GM_LAUNCH(2, 4);
    } else {
        if (TM == 1) GM_LAUNCH(1, 1);
        else if (TM == 2) GM_LAUNCH(1, 2);
        else if (TM == 3) GM_LAUNCH(1, 3);
        else GM_LAUNCH(1, 4);
    }
#undef GM_LAUNCH
    if (int rc = mv_check_launch("gemm_mid")) return rc;
    const long total = (long)M * (swiglu ? N / 2 : N);
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (c_dtype == MV_F32)
        hipLaunchKernelGGL(gemm_mid_reduce_kernel<float>, dim3(blocks), dim3(256), 0, stream, work, (const bf16*)bias,
                           (float*)C, ldc, M, N, p.F, swiglu);
    else
        hipLaunchKernelGGL(gemm_mid_reduce_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, work, (const bf16*)bias,
                           (bf16*)C, ldc, M, N, p.F, swiglu);
    return mv_check_launch("gemm_mid (reduce)");
}
