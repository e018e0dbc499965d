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
#include "dispatch.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    uint16_t s[8];
    bf16x8_t v;
};

#define SK_MAX_WAVES 8

template <typename TC> __device__ __forceinline__ void store_c(TC* p, float v);
template <> __device__ __forceinline__ void store_c<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_c<bf16>(bf16* p, float v) { *p = from_f<bf16>(v); }

// What the NORM variant computes in front of the product (see below).
struct NormInput {
    const float* resid_in;   // [M, K] float
    const bf16* delta;       // [M, K] or null
    float* resid_out;        // [M, K] float, or null when delta is null
    WeightPtr weight;        // [K]
    float eps;
    int unit_offset;
};

// R: 16-row weight tiles per workgroup; TM: 16-token tiles (M <= 16 * TM); SWIGLU: R == 2 and
// the two tiles are the gate rows and the up rows of the same output columns.
// NORM (TM == 1): the activations are not read from A but made here:
//     x = resid_in + delta;  A[m][k] = bf16(x[m][k] * rsqrt(mean_k x[m]^2 + eps) * weight[k])
// Every workgroup normalises the (few) rows for itself into LDS, which costs less than a kernel
// launch; workgroup 0 also writes x to resid_out (a buffer other than resid_in: the other
// workgroups still read that one).
template <int R, int TM, bool SWIGLU, bool NORM, typename TC>
__global__ void __launch_bounds__(64 * SK_MAX_WAVES)
gemm_skinny_kernel(const bf16* __restrict__ A, long lda, const bf16* __restrict__ W, const bf16* __restrict__ bias,
                   TC* __restrict__ C, long ldc, int M, int N, int K, NormInput norm) {
    extern __shared__ float red[];  // [S - 1][R * TM][64][4], then (NORM) bf16 [M][K + 8]
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
    if (NORM) {
        bf16* sA = reinterpret_cast<bf16*>(red + (size_t)(S - 1) * R * TM * 256);
        const int lds_ld = K + 8;  // row pitch in elements: the 16 rows an operand load touches fall into different banks
        // A row is held in registers between the sum of squares and the scaling (up to 2048
        // columns: 4 chunks of 8 per lane), so that the kernel waits for memory once.
        constexpr int MAXJ = 4;
        const int nj = (K + 511) / 512;
        for (int m = wave; m < M; m += S) {
            const float* xr = norm.resid_in + (size_t)m * K;
            const bf16* dr = norm.delta ? norm.delta + (size_t)m * K : nullptr;
            float x[MAXJ][8];
            float ss = 0.f;
            if (nj <= MAXJ) {
                float4 r0[MAXJ], r1[MAXJ];
                Frag d[MAXJ];
#pragma unroll
                for (int j = 0; j < MAXJ; ++j) {
                    const int c = lane * 8 + 512 * j;
                    if (j < nj && c < K) {
                        r0[j] = *reinterpret_cast<const float4*>(xr + c);
                        r1[j] = *reinterpret_cast<const float4*>(xr + c + 4);
                        d[j].u = dr ? *reinterpret_cast<const uint4*>(dr + c) : uint4{0u, 0u, 0u, 0u};
                    }
                }
#pragma unroll
                for (int j = 0; j < MAXJ; ++j) {
                    const int c = lane * 8 + 512 * j;
                    if (j < nj && c < K) {
                        x[j][0] = r0[j].x; x[j][1] = r0[j].y; x[j][2] = r0[j].z; x[j][3] = r0[j].w;
                        x[j][4] = r1[j].x; x[j][5] = r1[j].y; x[j][6] = r1[j].z; x[j][7] = r1[j].w;
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            x[j][e] += (float)d[j].v[e];      // a missing delta was loaded as zeros
                            ss += x[j][e] * x[j][e];
                        }
                    }
                }
            } else {
                for (int c = lane * 8; c < K; c += 512) {
                    const float4 q0 = *reinterpret_cast<const float4*>(xr + c);
                    const float4 q1 = *reinterpret_cast<const float4*>(xr + c + 4);
                    float y[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
                    if (dr) {
                        Frag dd;
                        dd.u = *reinterpret_cast<const uint4*>(dr + c);
#pragma unroll
                        for (int e = 0; e < 8; ++e) y[e] += (float)dd.v[e];
                    }
#pragma unroll
                    for (int e = 0; e < 8; ++e) ss += y[e] * y[e];
                }
            }
            ss = wave_sum(ss);
            const float rinv = rsqrtf(ss / (float)K + norm.eps);
            // scales eight values, rounds them, and puts them where the MFMA operand loads expect
            // them; workgroup 0 also stores the new residual sum
            auto emit = [&](int c, const float* y) {
                if (dr && blockIdx.x == 0) {
                    float* yr = norm.resid_out + (size_t)m * K + c;
                    *reinterpret_cast<float4*>(yr) = float4{y[0], y[1], y[2], y[3]};
                    *reinterpret_cast<float4*>(yr + 4) = float4{y[4], y[5], y[6], y[7]};
                }
                Frag o;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float wt = norm.weight.at(c + e);
                    if (norm.unit_offset) wt += 1.f;
                    o.s[e] = f32_to_bf16_bits(y[e] * rinv * wt);
                }
                *reinterpret_cast<uint4*>(sA + (size_t)m * lds_ld + c) = o.u;
            };
            if (nj <= MAXJ) {
#pragma unroll
                for (int j = 0; j < MAXJ; ++j) {
                    const int c = lane * 8 + 512 * j;
                    if (j < nj && c < K) emit(c, x[j]);
                }
            } else {
                for (int c = lane * 8; c < K; c += 512) {
                    const float4 q0 = *reinterpret_cast<const float4*>(xr + c);
                    const float4 q1 = *reinterpret_cast<const float4*>(xr + c + 4);
                    float y[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
                    if (dr) {
                        Frag dd;
                        dd.u = *reinterpret_cast<const uint4*>(dr + c);
#pragma unroll
                        for (int e = 0; e < 8; ++e) y[e] += (float)dd.v[e];
                    }
                    emit(c, y);
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const int tok = 16 * t + i;
            avalid[t] = tok < M;
            arow[t] = reinterpret_cast<const uint4*>(sA + (size_t)(avalid[t] ? tok : 0) * lds_ld) + g;
        }
    } else {
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const int tok = 16 * t + i;
            avalid[t] = tok < M;
            arow[t] = reinterpret_cast<const uint4*>(A + (size_t)(avalid[t] ? tok : 0) * lda) + g;
        }
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

static size_t skinny_lds_bytes(int S, int R, int TM, bool with_norm, int M, int K) {
    size_t lds = (size_t)(S - 1) * R * TM * 256 * sizeof(float);
    if (with_norm) lds += (size_t)M * (K + 8) * sizeof(uint16_t);
    return lds;
}

template <int R, int TM, bool SWIGLU, typename TC>
static void launch_skinny(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int M, int N,
                          int K, int S, hipStream_t stream) {
    const int tiles = (N + 15) / 16;
    const int blocks = SWIGLU ? tiles : (tiles + R - 1) / R;
    const size_t lds = skinny_lds_bytes(S, R, TM, false, M, K);
    hipLaunchKernelGGL((gemm_skinny_kernel<R, TM, SWIGLU, false, TC>), dim3(blocks), dim3(64 * S), lds, stream,
                       (const bf16*)A, lda, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N, K, NormInput{});
}

template <int R, bool SWIGLU, typename TC>
static void launch_skinny_norm(const NormInput& norm, const void* W, const void* bias, void* C, long ldc, int M, int N,
                               int K, int S, hipStream_t stream) {
    const int tiles = (N + 15) / 16;
    const int blocks = SWIGLU ? tiles : (tiles + R - 1) / R;
    const size_t lds = skinny_lds_bytes(S, R, 1, true, M, K);
    hipLaunchKernelGGL((gemm_skinny_kernel<R, 1, SWIGLU, true, TC>), dim3(blocks), dim3(64 * S), lds, stream,
                       (const bf16*)nullptr, (long)K, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N, K, norm);
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

// The product (or the gated pair with `swiglu`) with the residual add and RMSNorm in front:
//     x = resid_in + delta (delta may be null); resid_out = x (written when delta is given);
//     A = bf16(rmsnorm(x) * weight);  C = A W^T (+ bias)   or   C = silu(A Wg^T) * (A Wu^T).
// At most 16 rows, K a multiple of 64, and the rows must fit LDS beside the partial tiles; returns
// 2 (and sets the error text) when the shape is not taken, so that the caller can run the two
// steps separately.
extern "C" int mv_gemm_skinny_norm(const float* resid_in, const void* delta, float* resid_out, const void* norm_weight,
                                   int norm_weight_dtype, float eps, int unit_offset, const void* W, const void* bias,
                                   void* C, long ldc, int c_dtype, int M, int N, int K, int swiglu,
                                   hipStream_t stream) {
    MV_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_skinny_norm: bad sizes M=%d N=%d K=%d", M, N, K);
    MV_REQUIRE(mv_valid_dtype(norm_weight_dtype) && norm_weight != nullptr, "gemm_skinny_norm: bad norm weight");
    MV_REQUIRE(delta == nullptr || (resid_out != nullptr && resid_out != resid_in),
               "gemm_skinny_norm: the updated residual needs a buffer of its own");
    MV_REQUIRE(eps > 0.f, "gemm_skinny_norm: eps must be positive");
    MV_REQUIRE(ldc >= N, "gemm_skinny_norm: ldc=%ld smaller than N=%d", ldc, N);
    MV_REQUIRE(c_dtype == MV_BF16 || (c_dtype == MV_F32 && !swiglu), "gemm_skinny_norm: bad output dtype %d", c_dtype);
    if (M == 0) return 0;
    const int S = pick_waves(K);
    const int R = swiglu ? 2 : 1;
    if (M > 16 || K % 64 != 0 || skinny_lds_bytes(S, R, 1, true, M, K) > 60 * 1024) {
        mv_fail("gemm_skinny_norm: M=%d K=%d is not taken by the fused kernel", M, K);
        return 2;
    }
    NormInput norm{resid_in, (const bf16*)delta, resid_out, WeightPtr{norm_weight, norm_weight_dtype}, eps, unit_offset};
    if (swiglu) launch_skinny_norm<2, true, bf16>(norm, W, nullptr, C, ldc, M, N, K, S, stream);
    else if (c_dtype == MV_F32) launch_skinny_norm<1, false, float>(norm, W, bias, C, ldc, M, N, K, S, stream);
    else launch_skinny_norm<1, false, bf16>(norm, W, bias, C, ldc, M, N, K, S, stream);
    return mv_check_launch("gemm_skinny_norm");
}
