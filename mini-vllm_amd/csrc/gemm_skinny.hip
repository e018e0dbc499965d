// Weight-streaming matrix product for few rows (decode steps, the output head):
//     C[M, N] = A[M, K] * W[N, K]^T (+ bias),   M <= 64, bf16 inputs, float accumulation,
// on the MFMA units of gfx950 (v_mfma_f32_16x16x32_bf16). Each weight is read from HBM exactly
// once; the few activation rows come from cache.
//
// Work split: a workgroup owns R tiles of 16 weight rows; its S waves split K between them and
// add their partial tiles through LDS in a fixed order (no atomics, so a row's result does not
// depend on what else runs). The weight rows are the MFMA's A operand (16 rows x 32 k per
// instruction: lane l holds row l%16, k-slots 8*(l/16)..+7, one 16-byte load), the activation
// rows its B operand (lane l holds token l%16, the same k-slots). The result tile has weight
// rows along i and tokens along j: lane l holds C[token l%16][n0 + 4*(l/16) + 0..3].
//
// A fused variant computes the gated activation of a feed-forward in the same pass:
//     out[M, I] = silu(A Wg^T) * (A Wu^T)  with Wg = W[0:I], Wu = W[I:2I].
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    bf16x8_t v;
};

#define SK_MAX_WAVES 8

template <typename TC> __device__ __forceinline__ void store_c(TC* p, float v);
template <> __device__ __forceinline__ void store_c<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_c<bf16>(bf16* p, float v) { *p = from_f<bf16>(v); }

// R: 16-row weight tiles per workgroup; TM: 16-token tiles (M <= 16 * TM); SWIGLU: R == 2 and
// the two tiles are the gate rows and the up rows of the same output columns.
template <int R, int TM, bool SWIGLU, typename TC>
__global__ void __launch_bounds__(64 * SK_MAX_WAVES)
gemm_skinny_kernel(const bf16* __restrict__ A, long lda, const bf16* __restrict__ W, const bf16* __restrict__ bias,
                   TC* __restrict__ C, long ldc, int M, int N, int K) {
    extern __shared__ float red[];  // [S - 1][R * TM][64][4]
    const int S = blockDim.x / MV_WAVE;
    const int wave = threadIdx.x / MV_WAVE;
    const int lane = threadIdx.x % MV_WAVE;
    const int i = lane % 16;
    const int g = lane / 16;
    // output columns of this workgroup: SWIGLU -> 16 columns of I = N; else 16 * R columns of N
    const int n_base = SWIGLU ? blockIdx.x * 16 : blockIdx.x * 16 * R;

    const int ksteps = K / 32;
    const int per = ksteps / S, rem = ksteps % S;
    const int ks0 = wave * per + (wave < rem ? wave : rem);
    const int ks1 = ks0 + per + (wave < rem ? 1 : 0);

    const uint4* wrow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int row;
        if (SWIGLU) {
            int col = n_base + i;
            if (col > N - 1) col = N - 1;
            row = r == 0 ? col : N + col;  // gate rows [0, N), up rows [N, 2N)
        } else {
            row = n_base + 16 * r + i;
            if (row > N - 1) row = N - 1;  // rows past the end are loaded again and never stored
        }
        wrow[r] = reinterpret_cast<const uint4*>(W + (size_t)row * K) + g;
    }
    const uint4* arow[TM];
    bool avalid[TM];
#pragma unroll
    for (int t = 0; t < TM; ++t) {
        const int tok = 16 * t + i;
        avalid[t] = tok < M;
        arow[t] = reinterpret_cast<const uint4*>(A + (size_t)(avalid[t] ? tok : 0) * lda) + g;
    }

    floatx4_t acc[R][TM];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < TM; ++t) acc[r][t] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // four k-steps per iteration: all loads are issued before the first MFMA needs its operands
    constexpr int U = 4;
    int ks = ks0;
    for (; ks + U <= ks1; ks += U) {
        Frag a[U][TM], w[U][R];
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int r = 0; r < R; ++r) w[u][r].u = wrow[r][(size_t)(ks + u) * 4];
#pragma unroll
            for (int t = 0; t < TM; ++t)
                a[u][t].u = avalid[t] ? arow[t][(size_t)(ks + u) * 4] : uint4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < TM; ++t)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][r].v, a[u][t].v, acc[r][t], 0, 0, 0);
    }
    for (; ks < ks1; ++ks) {
        Frag a[TM], w[R];
#pragma unroll
        for (int r = 0; r < R; ++r) w[r].u = wrow[r][(size_t)ks * 4];
#pragma unroll
        for (int t = 0; t < TM; ++t) a[t].u = avalid[t] ? arow[t][(size_t)ks * 4] : uint4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < TM; ++t)
                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[r].v, a[t].v, acc[r][t], 0, 0, 0);
    }

    // partial tiles of waves 1 .. S-1 go through LDS; wave 0 adds them in order
    if (wave > 0) {
        float* dst = red + ((size_t)(wave - 1) * R * TM) * 256;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[(r * TM + t) * 256 + e * 64 + lane] = acc[r][t][e];
    }
    __syncthreads();
    if (wave != 0) return;
    for (int w = 1; w < S; ++w) {
        const float* src = red + ((size_t)(w - 1) * R * TM) * 256;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[r][t][e] += src[(r * TM + t) * 256 + e * 64 + lane];
    }

    if (SWIGLU) {
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const int tok = 16 * t + i;
            if (tok >= M) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = n_base + 4 * g + e;
                if (col >= N) continue;
                const float gate = acc[0][t][e], up = acc[R - 1][t][e];
                store_c<TC>(C + (size_t)tok * ldc + col, gate / (1.f + expf(-gate)) * up);
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const int tok = 16 * t + i;
                if (tok >= M) continue;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int col = n_base + 16 * r + 4 * g + e;
                    if (col >= N) continue;
                    float v = acc[r][t][e];
                    if (bias) v += to_f(bias[col]);
                    store_c<TC>(C + (size_t)tok * ldc + col, v);
                }
            }
    }
}

template <int R, int TM, bool SWIGLU, typename TC>
static void launch_skinny(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int M, int N,
                          int K, int S, hipStream_t stream) {
    const int tiles = (N + 15) / 16;
    const int blocks = SWIGLU ? tiles : (tiles + R - 1) / R;
    const size_t lds = (size_t)(S - 1) * R * TM * 256 * sizeof(float);
    hipLaunchKernelGGL((gemm_skinny_kernel<R, TM, SWIGLU, TC>), dim3(blocks), dim3(64 * S), lds, stream,
                       (const bf16*)A, lda, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N, K);
}

static int pick_waves(int K) {
    int s = K / 128;  // at least four MFMA steps per wave
    if (s < 1) s = 1;
    if (s > SK_MAX_WAVES) s = SK_MAX_WAVES;
    return s;
}

template <int R, bool SWIGLU, typename TC>
static int dispatch_tm(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int M, int N, int K,
                       int S, hipStream_t stream) {
    if (M <= 16) launch_skinny<R, 1, SWIGLU, TC>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
    else if (M <= 32) launch_skinny<R, 2, SWIGLU, TC>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
    else if (M <= 48) launch_skinny<R, 3, SWIGLU, TC>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
    else launch_skinny<R, 4, SWIGLU, TC>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
    return 0;
}

static int check_skinny(const char* what, const void* A, long lda, const void* W, long ldc, int M, int N, int K) {
    MV_REQUIRE(M >= 0 && M <= 64, "%s: takes at most 64 rows, got M=%d", what, M);
    MV_REQUIRE(N > 0 && K > 0 && K % 32 == 0, "%s: K=%d must be a positive multiple of 32 (N=%d)", what, K, N);
    MV_REQUIRE(lda >= K && lda % 8 == 0, "%s: lda=%ld must be a multiple of 8 and at least K=%d", what, lda, K);
    MV_REQUIRE(ldc >= N, "%s: ldc=%ld smaller than N=%d", what, ldc, N);
    MV_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "%s: operands must be 16-byte aligned", what);
    return 0;
}

// c_dtype: MV_BF16 or MV_F32.
extern "C" int mv_gemm_skinny(const void* A, long lda, const void* W, long ldw, const void* bias, void* C, long ldc,
                              int c_dtype, int M, int N, int K, hipStream_t stream) {
    if (int rc = check_skinny("gemm_skinny", A, lda, W, ldc, M, N, K)) return rc;
    MV_REQUIRE(ldw == K, "gemm_skinny: the weight must be contiguous (ldw=%ld, K=%d)", ldw, K);
    MV_REQUIRE(c_dtype == MV_F32 || c_dtype == MV_BF16, "gemm_skinny: bad output dtype %d", c_dtype);
    if (M == 0) return 0;
    const int S = pick_waves(K);
    const int tiles = (N + 15) / 16;
    const int TM = (M + 15) / 16;
    // more row tiles per workgroup reuse the activation registers; keep at least ~512 workgroups
    // and the partial tiles of the waves within 56 KiB of LDS
    int R = tiles >= 2048 ? 4 : (tiles >= 1024 ? 2 : 1);
    while (R > 1 && (size_t)(S - 1) * R * TM * 1024 > 56 * 1024) R /= 2;
    int rc = 0;
    if (c_dtype == MV_F32) {
        if (R == 4) rc = dispatch_tm<4, false, float>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
        else if (R == 2) rc = dispatch_tm<2, false, float>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
        else rc = dispatch_tm<1, false, float>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
    } else {
        if (R == 4) rc = dispatch_tm<4, false, bf16>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
        else if (R == 2) rc = dispatch_tm<2, false, bf16>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
        else rc = dispatch_tm<1, false, bf16>(A, lda, W, bias, C, ldc, M, N, K, S, stream);
    }
    if (rc) return rc;
    return mv_check_launch("gemm_skinny");
}

// out[M, I] = silu(A Wgu[0:I]^T) * (A Wgu[I:2I]^T), bf16 in and out.
extern "C" int mv_gemm_skinny_swiglu(const void* A, long lda, const void* Wgu, void* out, long ldo, int M, int I,
                                     int K, hipStream_t stream) {
    if (int rc = check_skinny("gemm_skinny_swiglu", A, lda, Wgu, ldo, M, I, K)) return rc;
    if (M == 0) return 0;
    const int S = pick_waves(K);
    int rc = dispatch_tm<2, true, bf16>(A, lda, Wgu, nullptr, out, ldo, M, I, K, S, stream);
    if (rc) return rc;
    return mv_check_launch("gemm_skinny_swiglu");
}
