// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) with float accumulation in a fixed order.
//
// This is the exact matrix product of the engine: every output element is the fused
// multiply-add chain over k = 0 .. K-1, whatever M is and wherever the row lies in the
// batch, so a row's result never depends on what else is in the step. It serves the
// float32 path entirely, and the bfloat16 path wherever a weight is stored in float or
// no faster kernel takes the shape. Inputs are converted to float on load (exact for
// bf16); there is no reduced-precision mode.
#include "dispatch.h"

#define RB_M 64
#define RB_N 64
#define RB_K 16

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_nt_kernel(const TA* __restrict__ A, long lda, const TW* __restrict__ W, long ldw, const TW* __restrict__ bias,
               TC* __restrict__ C, long ldc, int M, int N, int K) {
    __shared__ float As[RB_K][RB_M + 1];
    __shared__ float Ws[RB_K][RB_N + 1];
    const int tid = threadIdx.x;
    const int tx = tid % 16;  // column direction
    const int ty = tid / 16;  // row direction
    const int m0 = blockIdx.y * RB_M;
    const int n0 = blockIdx.x * RB_N;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += RB_K) {
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const int idx = tid + 256 * l;
            const int r = idx / RB_K;
            const int k = idx % RB_K;
            const int gm = m0 + r, gn = n0 + r, gk = k0 + k;
            As[k][r] = (gm < M && gk < K) ? to_f(A[(size_t)gm * lda + gk]) : 0.f;
            Ws[k][r] = (gn < N && gk < K) ? to_f(W[(size_t)gn * ldw + gk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < RB_K; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + ty + 16 * i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx + 16 * j;
            if (gn >= N) continue;
            float v = acc[i][j];
            if (bias) v += to_f(bias[gn]);
            C[(size_t)gm * ldc + gn] = from_f<TC>(v);
        }
    }
}

template <typename TA, typename TW, typename TC>
static void launch_gemm(const void* A, long lda, const void* W, long ldw, const void* bias, void* C, long ldc,
                        int M, int N, int K, hipStream_t stream) {
    dim3 grid((N + RB_N - 1) / RB_N, (M + RB_M - 1) / RB_M);
    hipLaunchKernelGGL((gemm_nt_kernel<TA, TW, TC>), grid, dim3(256), 0, stream, (const TA*)A, lda, (const TW*)W,
                       ldw, (const TW*)bias, (TC*)C, ldc, M, N, K);
}

// a_dtype: activations; w_dtype: weight and bias as stored; c_dtype: a_dtype or float.
extern "C" int mv_gemm_ref(const void* A, long lda, int a_dtype, const void* W, long ldw, int w_dtype,
                           const void* bias, void* C, long ldc, int c_dtype, int M, int N, int K,
                           hipStream_t stream) {
    MV_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    MV_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: leading dimensions lda=%ld ldw=%ld ldc=%ld too small for "
               "M=%d N=%d K=%d", lda, ldw, ldc, M, N, K);
    MV_REQUIRE(mv_valid_dtype(w_dtype), "gemm: bad weight dtype %d", w_dtype);
    MV_REQUIRE(c_dtype == a_dtype || c_dtype == MV_F32, "gemm: output dtype %d must be the activation dtype %d "
               "or float", c_dtype, a_dtype);
    if (M == 0) return 0;
    MV_REQUIRE((M + RB_M - 1) / RB_M <= 65535, "gemm: M=%d too large for one launch", M);
    MV_DISPATCH_T(a_dtype, "gemm", {
        if (w_dtype == MV_F32) {
            if (c_dtype == MV_F32) launch_gemm<T, float, float>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream);
            else launch_gemm<T, float, T>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream);
        } else {
            if (c_dtype == MV_F32) launch_gemm<T, bf16, float>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream);
            else launch_gemm<T, bf16, T>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream);
        }
    });
    return mv_check_launch("gemm");
}
