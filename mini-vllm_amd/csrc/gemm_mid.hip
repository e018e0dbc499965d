// Matrix product for up to 64 rows against a large weight (decode steps on models whose weights
// take tens or hundreds of megabytes per matrix, the output head):
//     C[M, N] = A[M, K] * W[N, K]^T (+ bias)      or      C[M, I] = silu(A Wg^T) * (A Wu^T),
// M <= 64, bf16 inputs, float accumulation, on the MFMA units of gfx950.
//
// Each weight is still read from HBM exactly once, but with dozens of rows the activation rows,
// which every weight tile needs, weigh as much as the weights themselves. So a workgroup (8 waves)
// takes 128 or 256 weight rows and a slice of K and stages the activation rows of that slice in
// LDS once for all its waves: in chunks of 128 columns, one chunk ahead, straight from global
// memory (global_load_lds) in the order the MFMA operands are read. Every wave multiplies its one
// or two tiles of 16 weight rows, loaded into registers one chunk ahead, with all token tiles. K
// is split over `F` workgroups so that the chip is filled although there are few weight tiles
// (that also makes it the faster kernel for a single row against the largest weights); the partial
// sums go to a float work area [F][M][N] and a second kernel adds them in a fixed order (no
// atomics: a row's result does not depend on what else runs), applies bias or the gated
// activation, and rounds.
#include "dispatch.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    uint16_t s[8];
    bf16x8_t v;
};

#define GM_WAVES 8
#ifndef GM_KC
#define GM_KC 128          // columns of a chunk
#endif
#define GM_KS (GM_KC / 32)  // MFMA steps of a chunk
#define GM_COMPUTE_UNITS mv_compute_units()

#define GM_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(0x0f70 | ((N) & 15) | (((N) >> 4) << 14))

// One load instruction that takes 16 bytes per lane from global memory straight into LDS: lane l's
// bytes land at lds_base + 16 * l (lds_base the same for the whole wave). It is written as assembly,
// not as the compiler's builtin, on purpose: the compiler then neither counts it nor guards it, and
// the waits for it are the explicit ones at the places marked below. (With the builtin the compiler
// puts a wait for all loads in flight in front of the first LDS read after a loop's head, which
// undoes the prefetch.) Counting it itself, the compiler could only wait longer, never too short:
// the vector memory counter retires in order.
__device__ __forceinline__ void load_to_lds_16(const void* src, __attribute__((address_space(3))) void* lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(src), "s"(lds_base)
                 : "memory", "m0");
}

// WAVES waves to a workgroup, R tiles of 16 weight rows each; TM: tiles of 16 tokens (M <= 16 * TM).
// The activation chunks land in one of two LDS arrays in turn.
template <int WAVES, int R, int TM>
__global__ void __launch_bounds__(64 * WAVES)
gemm_mid_kernel(const bf16* __restrict__ A, long lda, const bf16* __restrict__ W, float* __restrict__ part, int M,
                     int N, int K, int F, int chunks_per_split) {
    constexpr int PAIRS = TM * GM_KS;                       // (token tile, k-step) pairs of a chunk: 64 LDS chunks each
    constexpr int AREP = (PAIRS + WAVES - 1) / WAVES;       // load instructions a wave issues per chunk
    // a wave with fewer pairs than AREP loads its last one again into a spare slot: every wave has
    // the same number of loads in flight, which the waits below count
    __shared__ uint4 ring0[(PAIRS + 1) * 64];
    __shared__ uint4 ring1[(PAIRS + 1) * 64];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / MV_WAVE);
    const int lane = tid % MV_WAVE;
    const int i = lane % 16;
    const int g = lane / 16;
    const int f = blockIdx.x % F;            // neighbouring workgroups take the splits of one row block
    const int nblock = blockIdx.x / F;
    const int n_base = (nblock * WAVES + wave) * 16 * R;
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

    const char* asrc[AREP];
    int aslot[AREP];
#pragma unroll
    for (int rep = 0; rep < AREP; ++rep) {
        int pair = wave + WAVES * rep;
        aslot[rep] = pair < PAIRS ? pair : PAIRS;
        pair = pair < PAIRS ? pair : PAIRS - 1;
        const int t = pair / GM_KS, ks = pair % GM_KS;
        int tok = 16 * t + i;
        tok = tok < M ? tok : M - 1;         // rows past the end: some row; their products are never stored
        asrc[rep] = reinterpret_cast<const char*>(A + (size_t)tok * lda + 32 * ks + 8 * g);
    }

    floatx4_t acc[R][TM];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < TM; ++t) acc[r][t] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    struct Weights {
        Frag w[GM_KS][R];
    };
    auto fetch_w = [&](int c, Weights& st) {
        const size_t k16 = (size_t)c * (GM_KC / 8);    // offset of the chunk in 16-byte units
#pragma unroll
        for (int ks = 0; ks < GM_KS; ++ks)
#pragma unroll
            for (int r = 0; r < R; ++r) st.w[ks][r].u = wrow[r][k16 + 4 * ks];
    };
    auto fetch_a = [&](int c, uint4* ring) {
#pragma unroll
        for (int rep = 0; rep < AREP; ++rep)
            load_to_lds_16(asrc[rep] + (size_t)c * (GM_KC * sizeof(bf16)),
                           (__attribute__((address_space(3))) void*)(ring + aslot[rep] * 64));
    };
    auto multiply = [&](const Weights& st, const uint4* ring) {
#pragma unroll
        for (int ks = 0; ks < GM_KS; ++ks) {
            Frag af[TM];
#pragma unroll
            for (int t = 0; t < TM; ++t) af[t].u = ring[(t * GM_KS + ks) * 64 + lane];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < TM; ++t)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.w[ks][r].v, af[t].v, acc[r][t], 0, 0, 0);
        }
    };
    // One chunk that has a successor: ask for the activations and the weights of the next one,
    // multiply this one, make sure the next activations have landed (the weights that were asked
    // for after them may still be on their way), meet. The barrier also orders this chunk's operand
    // reads before the load that refills their array a chunk later. The body is straight-line code:
    // where two paths with different loads in flight meet, the compiler's one wait has to assume
    // the worse of them.
    auto step = [&](int c, const Weights& cur, Weights& nxt, const uint4* ring_cur, uint4* ring_nxt) {
        fetch_a(c + 1, ring_nxt);
        fetch_w(c + 1, nxt);
        multiply(cur, ring_cur);
        GM_WAIT_VMCNT(GM_KS * R);         // explicit wait: the activations of chunk c + 1 are in LDS
        __builtin_amdgcn_s_barrier();
    };
    Weights s0, s1;
    fetch_a(c0, ring0);
    fetch_w(c0, s0);
    GM_WAIT_VMCNT(GM_KS * R);             // explicit wait: the activations of the first chunk are in LDS
    __builtin_amdgcn_s_barrier();
    int c = c0;
    for (; c + 2 < c1; c += 2) {
        step(c, s0, s1, ring0, ring1);
        step(c + 1, s1, s0, ring1, ring0);
    }
    if (c + 1 < c1) {                     // two chunks left
        step(c, s0, s1, ring0, ring1);
        multiply(s1, ring1);
    } else if (c < c1) {
        multiply(s0, ring0);
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

// Splits of K. The weights are dealt out to blocks * F workgroups, which the chip takes in rounds
// of one per compute unit (the product is bound by memory, so one workgroup keeps a unit's share
// of the bandwidth busy): the time goes with rounds / F, and with the traffic, which every split
// raises by its float partial sums, written and read once, 4 F M / K of the weights. At least two
// chunks per split. The choice does not look at the number of rows (the traffic is priced at 32
// of them): a row's sum is then split the same way whatever else is in the step.
static MidPlan mid_plan(int N, int K) {
    const int chunks = K / GM_KC;
    // two tiles of weight rows per wave where that still leaves many workgroups: the activation
    // rows a workgroup stages then serve 256 weight rows (measured on MI355X: faster from about
    // ten thousand weight rows on, slower below)
    const int R = N >= 10240 ? 2 : 1;
    const int blocks = (N + 16 * GM_WAVES * R - 1) / (16 * GM_WAVES * R);
    MidPlan best{R, 1, chunks, blocks};
    double best_cost = -1.0;
    for (int cps = chunks; cps >= 2 || cps == chunks; --cps) {
        const int F = (chunks + cps - 1) / cps;
        if (F > 32) break;
        const long wgs = (long)blocks * F;
        const long rounds = (wgs + GM_COMPUTE_UNITS - 1) / GM_COMPUTE_UNITS;
        const double cost = (double)rounds / F * (1.0 + 4.0 * F * 32 / K);
        if (best_cost < 0.0 || cost < best_cost) {
            best_cost = cost;
            best = MidPlan{R, F, cps, blocks};
        }
        if (cps == 1) break;
    }
    return best;
}

// Floats of work area a product of this shape needs (the partial sums [F][M][N]).
extern "C" long mv_gemm_mid_workspace(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % GM_KC) return 0;
    const MidPlan p = mid_plan(N, K);
    return (long)p.F * M * N;
}

// The number of partial sums a product with an [N, K] weight is split into.
extern "C" int mv_gemm_mid_splits(int N, int K) {
    if (N <= 0 || K <= 0 || K % GM_KC) return 0;
    return mid_plan(N, K).F;
}

// The first half alone: the partial sums work[f][m][n], f < mv_gemm_mid_splits(N, K), of
// A[M, K] * W[N, K]^T. `work` holds at least mv_gemm_mid_workspace(M, N, K) floats.
extern "C" int mv_gemm_mid_sums(const void* A, long lda, const void* W, int M, int N, int K, float* work,
                                long work_floats, hipStream_t stream) {
    MV_REQUIRE(M > 0 && M <= 64, "gemm_mid: takes 1 to 64 rows, got M=%d", M);
    MV_REQUIRE(N > 0 && K > 0 && K % GM_KC == 0, "gemm_mid: K=%d must be a positive multiple of %d (N=%d)", K, GM_KC, N);
    MV_REQUIRE(lda >= K && lda % 8 == 0, "gemm_mid: lda=%ld must be a multiple of 8 and at least K=%d", lda, K);
    MV_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_mid: operands must be 16-byte aligned");
    const MidPlan p = mid_plan(N, K);
    MV_REQUIRE(work != nullptr && ((uintptr_t)work % 16) == 0 && work_floats >= (long)p.F * M * N,
               "gemm_mid: the work area holds %ld floats, %ld are needed", work_floats, (long)p.F * M * N);
    const dim3 grid((unsigned)(p.blocks * p.F));
    const int TM = (M + 15) / 16;
#define GM_LAUNCH(RR, TT)                                                                                          \
    hipLaunchKernelGGL((gemm_mid_kernel<GM_WAVES, RR, TT>), grid, dim3(64 * GM_WAVES), 0, stream, (const bf16*)A,  \
                       lda, (const bf16*)W, work, M, N, K, p.F, p.chunks_per_split)
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
    return mv_check_launch("gemm_mid");
}

// The second half alone: C = sum over f < F of work[f] (+ bias), or the gated activation of the two
// halves of the sum. c_dtype: MV_BF16 or MV_F32.
extern "C" int mv_gemm_mid_reduce(const float* work, const void* bias, void* C, long ldc, int c_dtype, int M, int N,
                                  int F, int swiglu, hipStream_t stream) {
    MV_REQUIRE(M > 0 && N > 0 && F > 0 && work != nullptr && C != nullptr, "gemm_mid: bad sizes M=%d N=%d F=%d", M, N, F);
    MV_REQUIRE(!swiglu || (N % 2 == 0 && bias == nullptr), "gemm_mid: the gated form takes an even N and no bias");
    MV_REQUIRE(ldc >= (swiglu ? N / 2 : N), "gemm_mid: ldc=%ld too small for N=%d", ldc, N);
    MV_REQUIRE(c_dtype == MV_F32 || c_dtype == MV_BF16, "gemm_mid: bad output dtype %d", c_dtype);
    const long total = (long)M * (swiglu ? N / 2 : N);
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (c_dtype == MV_F32)
        hipLaunchKernelGGL(gemm_mid_reduce_kernel<float>, dim3(blocks), dim3(256), 0, stream, work, (const bf16*)bias,
                           (float*)C, ldc, M, N, F, swiglu);
    else
        hipLaunchKernelGGL(gemm_mid_reduce_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, work, (const bf16*)bias,
                           (bf16*)C, ldc, M, N, F, swiglu);
    return mv_check_launch("gemm_mid (reduce)");
}

// Both halves. With `swiglu`, W is the packed gate/up weight [N = 2 I, K] and C is [M, I].
extern "C" int mv_gemm_mid(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int c_dtype,
                           int M, int N, int K, int swiglu, float* work, long work_floats, hipStream_t stream) {
    if (int rc = mv_gemm_mid_sums(A, lda, W, M, N, K, work, work_floats, stream)) return rc;
    return mv_gemm_mid_reduce(work, bias, C, ldc, c_dtype, M, N, mid_plan(N, K).F, swiglu, stream);
}
