// Weight-streaming matrix product for few rows (decode steps, the output head):
//     C[M, N] = A[M, K] * W[N, K]^T (+ bias),   M <= 512, bf16 inputs, float accumulation,
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
// PAIRED (weights of 16 MB and more, up to 16 rows): the loads of the layout above touch sixteen
// 128-byte lines an instruction and use half of each, and it is the number of lines a compute unit
// asks its cache for, not the bytes, that bounds the kernel (loading the activations of one row
// instead of eight, for the measurement, took an 8B-sized gate/up product from 45.6 to 40.7 us). Here
// a load takes whole lines: lane l holds piece 2 (l / 16) + (l % 16) / 8 of row (l % 16) % 8 of eight
// rows, 128 bytes of each. As an MFMA operand that is sixteen "rows" of which the first eight hold the
// even 16-byte pieces of the real rows and the last eight the odd ones: multiplied with the tokens'
// even pieces the first eight result rows are half of the dot products, multiplied with their odd
// pieces the last eight are the other half. Two MFMAs a load instead of one (the matrix unit is idle
// anyway), two accumulators, added across the lane halves once behind the loop, which also restores
// the usual result layout. 8B-sized gate/up at 8 rows: 45.6 -> 39.4 us, down 27.4 -> 25.1.
// PAIRED == 2 (up to 8 rows): the tokens' loads take whole lines the same way — lane l holds piece
// 2 (l / 16) + (l % 16) / 8 of token (l % 16) % 8 — and one MFMA a load is enough: its result rows
// 0-7 x columns 0-7 are the dot products' even halves, rows 8-15 x columns 8-15 the odd halves of
// the same (weight row, token) pairs, the other two quarters are not used.
//
// A fused variant computes the gated activation of a feed-forward in the same pass:
//     out[M, I] = silu(A Wg^T) * (A Wu^T)  with Wg = W[0:I], Wu = W[I:2I].
//
// Two more variants take a residual add and an RMSNorm between two products apart, for steps
// with too many rows to normalise them in every workgroup of the second product. The product in
// front of the norm (FOLD) owns each element of its output once, so it adds it to the residual
// there, leaves x * weight (rounded to bf16, not yet divided by the row's root mean square) and
// the sum of x^2 over its own columns; the product behind the norm (SCALED) multiplies with
// those rows and divides each output row by the root mean square, which it gets from the
// partial sums: (x w / rms) W^T = (x w) W^T / rms.
#include "gemm_skinny_shape.h"

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
template <int R, int TM, bool SWIGLU, bool NORM, typename TC, int EPI = EPI_NONE, int PAIRED = 0>
__global__ void __launch_bounds__(64 * SK_MAX_WAVES)
gemm_skinny_kernel(const bf16* __restrict__ A, long lda, const bf16* __restrict__ W, const bf16* __restrict__ bias,
                   TC* __restrict__ C, long ldc, int M, int N, int K, int groups, int blocks, int rows,
                   NormInput norm, RowsInput fold) {
    extern __shared__ float red[];  // [S - 1][R * TM][64][4], then (NORM) bf16 [M][K + 8], or (SCALED) float [16 * TM]
    // The tokens may be dealt out to `groups` workgroups per weight tile (16 * TM tokens each): with
    // few weight tiles that fills more compute units, and each unit pulls fewer activation rows.
    // Workgroups go to the chip's eight dies in turn, so the groups of one tile are given ids that
    // are 8 apart: they share a die's L2 and the tile's weights are fetched from memory once.
    int block = blockIdx.x;
    if (groups > 1) {
        const int within = blockIdx.x % (8 * groups);
        const int tg = within / 8;
        block = (blockIdx.x / (8 * groups)) * 8 + within % 8;
        if (block >= blocks) return;
        A += (size_t)tg * 16 * TM * lda;
        C += (size_t)tg * 16 * TM * ldc;
        if (EPI == EPI_FOLD) {
            fold.resid += (size_t)tg * 16 * TM * fold.ldr;
            fold.weighted += (size_t)tg * 16 * TM * fold.ldw;
        }
        if (EPI != EPI_NONE) fold.partial += (size_t)tg * 16 * TM * fold.P;
        M -= tg * 16 * TM;
        if (M <= 0) return;
        if (M > 16 * TM) M = 16 * TM;
    }
    const int S = blockDim.x / MV_WAVE;
    const int wave = threadIdx.x / MV_WAVE;
    const int lane = threadIdx.x % MV_WAVE;
    const int i = lane % 16;
    const int g = lane / 16;
    // output columns of this workgroup (SWIGLU: of I = N, at most 16): `rows` of them (at most 16 * R; fewer where that makes the
    // workgroups a whole number of rounds of the chip: the rows of a tile beyond them are loaded
    // again from the last one and never stored)
    // (The variant with the norm in front keeps whole tiles: more workgroups would each pay its
    // prologue, and the extra registers would cost it a wave per SIMD.)
    const int own = NORM ? (SWIGLU ? 16 : 16 * R) : rows;
    const int n_base = block * own;
    const int n_end = n_base + own < N ? n_base + own : N;

    // (PAIRED: the waves share K in chunks of 64 columns, two k-steps; ks0 and ks1 count k-steps either way)
    const int ksteps = PAIRED ? K / 64 : K / 32;
    const int per = ksteps / S, rem = ksteps % S;
    const int ks0 = (wave * per + (wave < rem ? wave : rem)) * (PAIRED ? 2 : 1);
    const int ks1 = ks0 + (per + (wave < rem ? 1 : 0)) * (PAIRED ? 2 : 1);

    // wrow[r][x]: where this lane's 16 bytes of k-step 0 lie. Not PAIRED: row i of tile r, piece g
    // (x unused). PAIRED: row i % 8 of half x of tile r, piece 2 g + i / 8 of the 128-byte chunk.
    const uint4* wrow[R][PAIRED ? 2 : 1];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int x = 0; x < (PAIRED ? 2 : 1); ++x) {
            const int in_tile = PAIRED ? 8 * x + i % 8 : i;
            int row;
            if (SWIGLU) {
                int col = n_base + in_tile;
                if (col > n_end - 1) col = n_end - 1;
                row = r == 0 ? col : N + col;  // gate rows [0, N), up rows [N, 2N)
            } else {
                row = n_base + 16 * r + in_tile;
                if (row > n_end - 1) row = n_end - 1;  // rows past the end are loaded again and never stored
            }
            wrow[r][x] = reinterpret_cast<const uint4*>(W + (size_t)row * K) + (PAIRED ? 2 * g + i / 8 : g);
        }
    // operand u (0 .. U-1, U even when PAIRED) of the stage that starts at k-step k
    auto w_at = [&](int r, int k, int u) -> uint4 {
        if constexpr (PAIRED != 0) return wrow[r][u & 1][(size_t)(k + (u & ~1)) * 4];
        else return wrow[r][0][(size_t)(k + u) * 4];
    };
    // k-steps per register stage of the main loop (see there)
    // (the fused-norm variants serve small steps, where a deeper first stage pays and registers are free)
    constexpr int FRAGS = NORM ? SK_STAGE_FRAGS + SK_STAGE_FRAGS / 2 : SK_STAGE_FRAGS;
    constexpr int U = FRAGS / (R + TM) >= 8 ? 8 : (FRAGS / (R + TM) >= 4 ? 4 : (FRAGS / (R + TM) >= 2 || PAIRED ? 2 : 1));
    const int nfull = (ks1 - ks0) / U;
    // NORM: the first stage's weights are asked for before the rows are normalised, so that their
    // way from memory overlaps the prologue
    Frag wfirst[NORM ? U : 1][R];
    if (NORM && nfull > 0) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r) wfirst[u][r].u = w_at(r, ks0, u);
    }
    const uint4* arow[TM];
    bool avalid[TM];
    if (NORM) {
        bf16* sA = reinterpret_cast<bf16*>(red + (size_t)(S - 1) * R * TM * 256);
        const int lds_ld = K + 8;  // row pitch in elements: the 16 rows an operand load touches fall into different banks
        // The rows are cut into chunks of 512 columns (8 per lane); wave w takes the chunks
        // w * cpw .. (w + 1) * cpw - 1 and holds them in registers between the sum of squares and
        // the scaling, so the kernel waits for memory once. Where a wave's chunks are whole rows
        // the sums stay in the wave; otherwise they are exchanged through LDS. The launcher takes
        // only shapes with at most SK_NORM_CHUNKS chunks a wave.
        float* part = reinterpret_cast<float*>(sA + (size_t)M * lds_ld);   // [chunks] sums of squares
        const int cpr = (K + 511) / 512;       // chunks per row
        const int nq = M * cpr;
        const int cpw = (nq + S - 1) / S;      // chunks per wave
        const bool whole = cpw % cpr == 0;
        float x[SK_NORM_CHUNKS][8], ss[SK_NORM_CHUNKS];
        {
            float4 r0[SK_NORM_CHUNKS], r1[SK_NORM_CHUNKS];
            Frag d[SK_NORM_CHUNKS];
#pragma unroll
            for (int qi = 0; qi < SK_NORM_CHUNKS; ++qi) {
                const int q = wave * cpw + qi;
                const int m = q / cpr, c = (q % cpr) * 512 + lane * 8;
                r0[qi] = r1[qi] = float4{0.f, 0.f, 0.f, 0.f};
                d[qi].u = uint4{0u, 0u, 0u, 0u};
                if (qi < cpw && q < nq && c < K) {
                    const float* xr = norm.resid_in + (size_t)m * K + c;
                    r0[qi] = *reinterpret_cast<const float4*>(xr);
                    r1[qi] = *reinterpret_cast<const float4*>(xr + 4);
                    if (norm.delta) d[qi].u = *reinterpret_cast<const uint4*>(norm.delta + (size_t)m * K + c);
                }
            }
#pragma unroll
            for (int qi = 0; qi < SK_NORM_CHUNKS; ++qi) {
                x[qi][0] = r0[qi].x; x[qi][1] = r0[qi].y; x[qi][2] = r0[qi].z; x[qi][3] = r0[qi].w;
                x[qi][4] = r1[qi].x; x[qi][5] = r1[qi].y; x[qi][6] = r1[qi].z; x[qi][7] = r1[qi].w;
                float t = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[qi][e] += (float)d[qi].v[e];      // a missing delta was loaded as zeros
                    t += x[qi][e] * x[qi][e];
                }
                ss[qi] = wave_sum(t);
            }
        }
        if (!whole) {
#pragma unroll
            for (int qi = 0; qi < SK_NORM_CHUNKS; ++qi) {
                const int q = wave * cpw + qi;
                if (qi < cpw && q < nq && lane == 0) part[q] = ss[qi];
            }
            __syncthreads();
        }
#pragma unroll
        for (int qi = 0; qi < SK_NORM_CHUNKS; ++qi) {
            const int q = wave * cpw + qi;
            const int m = q / cpr, c = (q % cpr) * 512 + lane * 8;
            if (qi >= cpw || q >= nq || c >= K) continue;
            float tot = 0.f;
            if (whole) {
#pragma unroll
                for (int qj = 0; qj < SK_NORM_CHUNKS; ++qj)
                    if (qj < cpw && qj / cpr == qi / cpr) tot += ss[qj];   // the chunks of this row, in order
            } else {
                for (int j = 0; j < cpr; ++j) tot += part[m * cpr + j];    // the same order in every workgroup
            }
            const float rinv = rsqrtf(tot / (float)K + norm.eps);
            if (norm.delta && blockIdx.x == 0) {   // workgroup 0 stores the new residual sum
                float* yr = norm.resid_out + (size_t)m * K + c;
                *reinterpret_cast<float4*>(yr) = float4{x[qi][0], x[qi][1], x[qi][2], x[qi][3]};
                *reinterpret_cast<float4*>(yr + 4) = float4{x[qi][4], x[qi][5], x[qi][6], x[qi][7]};
            }
            float wt[8];
            norm.weight.at8(c, wt);
            Frag o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o.s[e] = f32_to_bf16_bits(x[qi][e] * rinv * (norm.unit_offset ? wt[e] + 1.f : wt[e]));
            *reinterpret_cast<uint4*>(sA + (size_t)m * lds_ld + c) = o.u;
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const int tok = 16 * t + i;
            if (PAIRED == 2) {
                avalid[t] = i % 8 < M;
                arow[t] = reinterpret_cast<const uint4*>(sA + (size_t)(avalid[t] ? i % 8 : 0) * lds_ld) + (2 * g + i / 8);
            } else {
                avalid[t] = tok < M;
                arow[t] = reinterpret_cast<const uint4*>(sA + (size_t)(avalid[t] ? tok : 0) * lds_ld) + (PAIRED ? 2 * g : g);
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const int tok = 16 * t + i;
            if (PAIRED == 2) {
                avalid[t] = i % 8 < M;
                arow[t] = reinterpret_cast<const uint4*>(A + (size_t)(avalid[t] ? i % 8 : 0) * lda) + (2 * g + i / 8);
            } else {
                avalid[t] = tok < M;
                arow[t] = reinterpret_cast<const uint4*>(A + (size_t)(avalid[t] ? tok : 0) * lda) + (PAIRED ? 2 * g : g);
            }
        }
    }
    // (PAIRED: operand u of a stage is piece 2 g + u % 2 of chunk u / 2; PAIRED == 2: one operand a chunk, the even u)
    auto a_at = [&](int t, int k, int u) -> uint4 {
        if (!avalid[t] || (PAIRED == 2 && (u & 1))) return uint4{0u, 0u, 0u, 0u};
        if constexpr (PAIRED == 2) return arow[t][(size_t)(k + u) * 4];
        else if constexpr (PAIRED == 1) return arow[t][(size_t)(k + (u & ~1)) * 4 + (u & 1)];
        else return arow[t][(size_t)(k + u) * 4];
    };

    floatx4_t acc[R][TM];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < TM; ++t) acc[r][t] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // SCALED: one over the root mean square of each of the workgroup's rows, from the partial sums
    // the product in front left; a wave takes every S-th row and adds a row's partial sums in a
    // fixed order (the same in every workgroup). Read after the barrier behind the main loop.
    float* sh_rinv = red + (size_t)(S - 1) * R * TM * 256;
    // The sums of a row are added in an order that depends on nothing but their number P. Up to 64
    // of them: eight lanes a row, lane j of them adds the sums j, j + 8, ... in order, then the eight
    // are added pairwise; a thread's first row is asked for here and added up behind the main loop,
    // so that neither the sums nor the weights wait for each other. More than 64: a wave takes every
    // S-th row, lane j adds the sums j, j + 64, ..., then the lanes are added pairwise; the first
    // eight loads of a wave are asked for here.
    const bool scaled_narrow = EPI == EPI_SCALED && fold.P <= 64;
    const int scaled_chunks = EPI == EPI_SCALED ? (fold.P + MV_WAVE - 1) / MV_WAVE : 1;
    float scaled_first[EPI == EPI_SCALED ? 8 : 1];
    if (EPI == EPI_SCALED) {
        if (scaled_narrow) {
            const int m = threadIdx.x / 8;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int p = threadIdx.x % 8 + 8 * u;
                scaled_first[u] = (m < M && p < fold.P) ? fold.partial[(size_t)m * fold.P + p] : 0.f;
            }
        } else {
            int m = wave, c = 0;                   // (no division: it would stand in front of the first weight load)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int p = lane + MV_WAVE * c;
                scaled_first[u] = (m < M && p < fold.P) ? fold.partial[(size_t)m * fold.P + p] : 0.f;
                if (++c == scaled_chunks) {
                    c = 0;
                    m += S;
                }
            }
        }
    }
    // FOLD: the residual and the norm's weights of the elements this workgroup will own are asked
    // for now (by the wave that stores them), not after the product
    float4 fold_resid[EPI == EPI_FOLD ? R : 1][EPI == EPI_FOLD ? TM : 1];
    float fold_w[EPI == EPI_FOLD ? R : 1][4];
    if (EPI == EPI_FOLD && wave == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int col0 = n_base + 16 * r + 4 * g;
            const bool live = col0 < n_end;      // N, the workgroup's columns and col0 are multiples of four
            if (live) fold.weight.at_few<4>(col0, fold_w[r]);
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const int tok = 16 * t + i;
                fold_resid[r][t] = (live && tok < M)
                                       ? *reinterpret_cast<const float4*>(fold.resid + (size_t)tok * fold.ldr + col0)
                                       : float4{0.f, 0.f, 0.f, 0.f};
            }
        }
    }

    // Two register stages of U k-steps each: while the MFMAs of one stage run, the loads of the
    // next are in flight, so a wave always has a stage's worth of weight bytes on the way.
    struct Stage {
        Frag w[U][R], a[U][TM];
    };
    // PAIRED: accp[r][t][h][q] = weight operand of half h times the tokens' pieces of parity q
    floatx4_t accp[PAIRED ? R : 1][PAIRED ? TM : 1][2][2];
    if constexpr (PAIRED != 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int q = 0; q < 2; ++q) accp[r][t][h][q] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    }
    auto fetch = [&](Stage& st, int k0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int r = 0; r < R; ++r) st.w[u][r].u = w_at(r, k0, u);
#pragma unroll
            for (int t = 0; t < TM; ++t) st.a[u][t].u = a_at(t, k0, u);
        }
    };
    auto multiply = [&](const Stage& st) {
        if constexpr (PAIRED != 0) {
#pragma unroll
            for (int c = 0; c < U / 2; ++c)
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int t = 0; t < TM; ++t)
#pragma unroll
                        for (int h = 0; h < 2; ++h)
#pragma unroll
                            for (int q = 0; q < (PAIRED == 2 ? 1 : 2); ++q)
                                accp[r][t][h][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                    st.w[2 * c + h][r].v, st.a[2 * c + q][t].v, accp[r][t][h][q], 0, 0, 0);
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int t = 0; t < TM; ++t)
                        acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.w[u][r].v, st.a[u][t].v, acc[r][t], 0, 0, 0);
        }
    };
    int ks = ks0 + nfull * U;
    if (nfull > 0) {
        Stage s0, s1;
        if (NORM) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int r = 0; r < R; ++r) s0.w[u][r] = wfirst[u][r];
#pragma unroll
                for (int t = 0; t < TM; ++t) s0.a[u][t].u = a_at(t, ks0, u);
            }
        } else {
            fetch(s0, ks0);
        }
        int it = 0;
        for (; it + 2 <= nfull; it += 2) {
            fetch(s1, ks0 + (it + 1) * U);
            multiply(s0);
            if (it + 2 < nfull) fetch(s0, ks0 + (it + 2) * U);
            multiply(s1);
        }
        if (it < nfull) multiply(s0);
    }
    // what is left of the wave's share: one k-step at a time (PAIRED: one chunk of two)
    for (; ks < ks1; ks += PAIRED ? 2 : 1) {
        Frag a[PAIRED ? 2 : 1][TM], w[PAIRED ? 2 : 1][R];
#pragma unroll
        for (int x = 0; x < (PAIRED ? 2 : 1); ++x) {
#pragma unroll
            for (int r = 0; r < R; ++r) w[x][r].u = w_at(r, ks, x);
#pragma unroll
            for (int t = 0; t < TM; ++t) a[x][t].u = a_at(t, ks, x);
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                if constexpr (PAIRED != 0) {
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int q = 0; q < (PAIRED == 2 ? 1 : 2); ++q)
                            accp[r][t][h][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[h][r].v, a[q][t].v, accp[r][t][h][q], 0, 0, 0);
                } else {
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[0][r].v, a[0][t].v, acc[r][t], 0, 0, 0);
                }
            }
    }
    if constexpr (PAIRED != 0) {
        // Result rows 0-7 of a tile: the first half's products with the even pieces (they sit in lane
        // groups 0 and 1, where rows 0-7 belong) plus its products with the odd pieces (result rows
        // 8-15 of that MFMA: lane groups 2 and 3). Rows 8-15: the second half's products with the odd
        // pieces (groups 2 and 3, where rows 8-15 belong) plus those with the even pieces (groups 0
        // and 1). One exchange between the lane halves each, and the usual layout is back.
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < TM; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if constexpr (PAIRED == 2) {
                        // (token j < 8, lane group G): rows 0-7 of the first half = its even halves here plus its
                        // odd halves at (j + 8, G + 2); rows 8-15 = the second half's even halves at (j, G - 2)
                        // plus its odd halves at (j + 8, G). Lanes of tokens 8-15 hold nothing that is stored.
                        const float odd_of_first = __shfl_xor(accp[r][t][0][0][e], 40, MV_WAVE);
                        const float even_of_second = __shfl_xor(accp[r][t][1][0][e], 32, MV_WAVE);
                        const float odd_of_second = __shfl_xor(accp[r][t][1][0][e], 8, MV_WAVE);
                        acc[r][t][e] = g < 2 ? accp[r][t][0][0][e] + odd_of_first : even_of_second + odd_of_second;
                    } else {
                        const float odd_of_first = __shfl_xor(accp[r][t][0][1][e], 32, MV_WAVE);
                        const float even_of_second = __shfl_xor(accp[r][t][1][0][e], 32, MV_WAVE);
                        acc[r][t][e] = g < 2 ? accp[r][t][0][0][e] + odd_of_first : accp[r][t][1][1][e] + even_of_second;
                    }
                }
    }

    if (EPI == EPI_SCALED && scaled_narrow) {
        for (int m = threadIdx.x / 8; m < M; m += blockDim.x / 8) {
            float t = 0.f;
            if (m == (int)threadIdx.x / 8) {
#pragma unroll
                for (int u = 0; u < 8; ++u) t += scaled_first[u];
            } else {
                for (int p = threadIdx.x % 8; p < fold.P; p += 8) t += fold.partial[(size_t)m * fold.P + p];
            }
            t += __shfl_xor(t, 1, MV_WAVE);
            t += __shfl_xor(t, 2, MV_WAVE);
            t += __shfl_xor(t, 4, MV_WAVE);
            if (threadIdx.x % 8 == 0) sh_rinv[m] = rsqrtf(t / (float)fold.width + fold.eps);
        }
    } else if (EPI == EPI_SCALED) {
        int item = 0;
        for (int m = wave; m < M; m += S) {
            float t = 0.f;
            for (int c = 0; c < scaled_chunks; ++c, ++item) {
                float v;
                if (item < 8) {
                    v = scaled_first[0];
#pragma unroll
                    for (int u = 1; u < 8; ++u) v = item == u ? scaled_first[u] : v;
                } else {
                    const int p = lane + MV_WAVE * c;
                    v = p < fold.P ? fold.partial[(size_t)m * fold.P + p] : 0.f;
                }
                t += v;
            }
            t = wave_sum(t);
            if (lane == 0) sh_rinv[m] = rsqrtf(t / (float)fold.width + fold.eps);
        }
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

    if (EPI == EPI_SCALED) {
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const float rinv = 16 * t + i < M ? sh_rinv[16 * t + i] : 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r][t] *= rinv;
        }
    }
    if (EPI == EPI_FOLD) {
        // x = resid + bf16(product (+ bias)) (the sum the stand-alone add makes from the rounded
        // product); resid = x; weighted = bf16(x * w); partial[tok][block] = sum of x^2 over this
        // workgroup's columns (the four lane groups of a token, then its R tiles, in a fixed order)
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const int tok = 16 * t + i;
            float ssq = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int col0 = n_base + 16 * r + 4 * g;
                if (tok < M && col0 < n_end) {
                    const float old4[4] = {fold_resid[r][t].x, fold_resid[r][t].y, fold_resid[r][t].z, fold_resid[r][t].w};
                    float x[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float v = acc[r][t][e];
                        if (bias) v += to_f(bias[col0 + e]);
                        x[e] = old4[e] + __uint_as_float((uint32_t)f32_to_bf16_bits(v) << 16);
                        ssq += x[e] * x[e];
                    }
                    *reinterpret_cast<float4*>(fold.resid + (size_t)tok * fold.ldr + col0) = float4{x[0], x[1], x[2], x[3]};
                    const float off = fold.unit_offset ? 1.f : 0.f;
                    uint2 packed;
                    packed.x = f32x2_to_bf16x2_bits(x[0] * (fold_w[r][0] + off), x[1] * (fold_w[r][1] + off));
                    packed.y = f32x2_to_bf16x2_bits(x[2] * (fold_w[r][2] + off), x[3] * (fold_w[r][3] + off));
                    *reinterpret_cast<uint2*>(fold.weighted + (size_t)tok * fold.ldw + col0) = packed;
                }
            }
            ssq += __shfl_xor(ssq, 16, MV_WAVE);
            ssq += __shfl_xor(ssq, 32, MV_WAVE);
            if (g == 0 && tok < M) fold.partial[(size_t)tok * fold.P + block] = ssq;
        }
        return;
    }
    if (SWIGLU) {
#pragma unroll
        for (int t = 0; t < TM; ++t) {
            const int tok = 16 * t + i;
            if (tok >= M) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = n_base + 4 * g + e;
                if (col >= n_end) continue;
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
                    if (col >= n_end) continue;
                    float v = acc[r][t][e];
                    if (bias) v += to_f(bias[col]);
                    store_c<TC>(C + (size_t)tok * ldc + col, v);
                }
            }
    }
}

static size_t skinny_lds_bytes(int S, int R, int TM, bool with_norm, int M, int K, bool scaled = false) {
    size_t lds = (size_t)(S - 1) * R * TM * 256 * sizeof(float);
    if (with_norm) lds += (size_t)M * (K + 8) * sizeof(uint16_t) + (size_t)M * ((K + 511) / 512) * sizeof(float);
    if (scaled) lds += (size_t)16 * TM * sizeof(float);
    return lds;
}

// Whether a product takes the loads of whole lines (PAIRED, see the top of the file): one tile of
// tokens, K in chunks of 64, and a weight large enough for the stream to matter more than the
// longer tail (below 16 MB the kernels are 0.1-0.2 us slower with it).
static bool skinny_paired(int M, long weight_rows, int K) {
    return M <= 16 && K % 64 == 0 && weight_rows * K * 2 >= 16L * 1024 * 1024;
}

template <int R, int TM, bool SWIGLU, typename TC, int EPI = EPI_NONE>
static void launch_skinny(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int M, int N,
                          int K, int S, int rows, hipStream_t stream, const RowsInput& fold = RowsInput{}) {
    const int blocks = skinny_blocks(N, rows);
    const int groups = (M + 16 * TM - 1) / (16 * TM);
    const int grid = groups > 1 ? (blocks + 7) / 8 * 8 * groups : blocks;
    const size_t lds = skinny_lds_bytes(S, R, TM, false, M, K, EPI == EPI_SCALED);
    if constexpr (TM == 1 && R <= 2) {
        if (skinny_paired(M, SWIGLU ? 2L * N : N, K)) {
            if (M <= 8)
                hipLaunchKernelGGL((gemm_skinny_kernel<R, TM, SWIGLU, false, TC, EPI, 2>), dim3(grid), dim3(64 * S), lds,
                                   stream, (const bf16*)A, lda, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N, K,
                                   groups, blocks, rows, NormInput{}, fold);
            else
                hipLaunchKernelGGL((gemm_skinny_kernel<R, TM, SWIGLU, false, TC, EPI, 1>), dim3(grid), dim3(64 * S), lds,
                                   stream, (const bf16*)A, lda, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N, K,
                                   groups, blocks, rows, NormInput{}, fold);
            return;
        }
    }
    hipLaunchKernelGGL((gemm_skinny_kernel<R, TM, SWIGLU, false, TC, EPI>), dim3(grid), dim3(64 * S), lds, stream,
                       (const bf16*)A, lda, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N, K, groups, blocks,
                       rows, NormInput{}, fold);
}

template <int R, bool SWIGLU, typename TC>
static void launch_skinny_norm(const NormInput& norm, const void* W, const void* bias, void* C, long ldc, int M, int N,
                               int K, int S, hipStream_t stream) {
    const int rows = SWIGLU ? 16 : 16 * R;
    const int blocks = skinny_blocks(N, rows);
    const size_t lds = skinny_lds_bytes(S, R, 1, true, M, K);
    if (skinny_paired(M, SWIGLU ? 2L * N : N, K)) {
        if (M <= 8)
            hipLaunchKernelGGL((gemm_skinny_kernel<R, 1, SWIGLU, true, TC, EPI_NONE, 2>), dim3(blocks), dim3(64 * S), lds,
                               stream, (const bf16*)nullptr, (long)K, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N,
                               K, 1, blocks, rows, norm, RowsInput{});
        else
            hipLaunchKernelGGL((gemm_skinny_kernel<R, 1, SWIGLU, true, TC, EPI_NONE, 1>), dim3(blocks), dim3(64 * S), lds,
                               stream, (const bf16*)nullptr, (long)K, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N,
                               K, 1, blocks, rows, norm, RowsInput{});
        return;
    }
    hipLaunchKernelGGL((gemm_skinny_kernel<R, 1, SWIGLU, true, TC>), dim3(blocks), dim3(64 * S), lds, stream,
                       (const bf16*)nullptr, (long)K, (const bf16*)W, (const bf16*)bias, (TC*)C, ldc, M, N, K, 1, blocks,
                       rows, norm, RowsInput{});
}

template <int R, bool SWIGLU, typename TC, int EPI = EPI_NONE>
static int dispatch_tm(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int M, int N, int K,
                       int S, int rows, hipStream_t stream, const RowsInput& fold = RowsInput{}) {
    // Token tiles per workgroup: all of them (the weights pass each compute unit once), or fewer
    // with the tokens dealt out to several workgroups per weight tile. A compute unit pulls
    // R + TM operand rows of 16 per workgroup it runs; the choice with the least per unit wins.
    const int tiles_m = (M + 15) / 16;
    const int blocks = skinny_blocks(N, rows);
    int best_tm = tiles_m < 4 ? tiles_m : 4;
    long best_cost = -1;
    for (int tm = best_tm; tm >= 1; --tm) {
        if (tm == 3 && tiles_m % 3 == 1) continue;   // a last group of one tile wastes a workgroup
        const int groups = (tiles_m + tm - 1) / tm;
        const long cost = (((long)blocks * groups + SK_COMPUTE_UNITS - 1) / SK_COMPUTE_UNITS) * (R + tm);
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best_tm = tm;
        }
    }
    if (best_tm == 1) launch_skinny<R, 1, SWIGLU, TC, EPI>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream, fold);
    else if (best_tm == 2) launch_skinny<R, 2, SWIGLU, TC, EPI>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream, fold);
    else if (best_tm == 3) launch_skinny<R, 3, SWIGLU, TC, EPI>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream, fold);
    else launch_skinny<R, 4, SWIGLU, TC, EPI>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream, fold);
    return 0;
}

// c_dtype: MV_BF16 or MV_F32.
extern "C" int mv_gemm_skinny(const void* A, long lda, const void* W, long ldw, const void* bias, void* C, long ldc,
                              int c_dtype, int M, int N, int K, hipStream_t stream) {
    if (int rc = check_skinny("gemm_skinny", A, lda, W, ldc, M, N, K)) return rc;
    MV_REQUIRE(ldw == K, "gemm_skinny: the weight must be contiguous (ldw=%ld, K=%d)", ldw, K);
    MV_REQUIRE(c_dtype == MV_F32 || c_dtype == MV_BF16, "gemm_skinny: bad output dtype %d", c_dtype);
    if (M == 0) return 0;
    int S, R, rows;
    skinny_shape(M, N, K, S, R, rows);
    int rc = 0;
    if (c_dtype == MV_F32) {
        if (R == 4) rc = dispatch_tm<4, false, float>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream);
        else if (R == 2) rc = dispatch_tm<2, false, float>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream);
        else rc = dispatch_tm<1, false, float>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream);
    } else {
        if (R == 4) rc = dispatch_tm<4, false, bf16>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream);
        else if (R == 2) rc = dispatch_tm<2, false, bf16>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream);
        else rc = dispatch_tm<1, false, bf16>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream);
    }
    if (rc) return rc;
    return mv_check_launch("gemm_skinny");
}

// The product in front of a residual add and an RMSNorm, with both folded into it (see the top of
// the file): resid[M, N] (float) += bf16(A W^T (+ bias)); weighted[M, N] = bf16(resid * norm_weight
// (+ 1 with unit_offset)); partial[M, P] = sums of resid^2 over the columns of each of the P
// workgroups along N, P = mv_gemm_skinny_fold_parts(M, N, K). The product behind the norm
// (mv_gemm_skinny_scaled), or mv_scale_rows, turns `weighted` and `partial` into normalised rows.
extern "C" int mv_gemm_skinny_fold_parts(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    int S, R, rows;
    skinny_shape(M, N, K, S, R, rows);
    return skinny_blocks(N, rows);
}

extern "C" int mv_gemm_skinny_fold(const void* A, long lda, const void* W, const void* bias, float* resid, long ldr,
                                   const void* norm_weight, int norm_weight_dtype, int unit_offset, void* weighted,
                                   long ldw, float* partial, int P, int M, int N, int K, hipStream_t stream) {
    if (int rc = check_skinny("gemm_skinny_fold", A, lda, W, ldw, M, N, K)) return rc;
    MV_REQUIRE(resid != nullptr && weighted != nullptr && partial != nullptr && ldr >= N,
               "gemm_skinny_fold: the residual, the weighted rows or the partial sums are missing (ldr=%ld)", ldr);
    MV_REQUIRE(mv_valid_dtype(norm_weight_dtype) && norm_weight != nullptr && ((uintptr_t)norm_weight % 16) == 0,
               "gemm_skinny_fold: the norm weight is missing, of an unknown type or not 16-byte aligned");
    MV_REQUIRE(N % 4 == 0 && ldr % 4 == 0 && ldw % 4 == 0 && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)weighted % 8) == 0,
               "gemm_skinny_fold: N=%d and the row pitches %ld / %ld must be multiples of four, the rows aligned", N, ldr, ldw);
    if (M == 0) return 0;
    int S, R, rows;
    skinny_shape(M, N, K, S, R, rows);
    MV_REQUIRE(P == skinny_blocks(N, rows), "gemm_skinny_fold: %d partial sums a row, the launch makes %d", P,
               skinny_blocks(N, rows));
    RowsInput fold{resid, ldr, WeightPtr{norm_weight, norm_weight_dtype}, unit_offset, (bf16*)weighted, ldw, partial,
                   P, 0.f, 0};
    int rc = 0;
    if (R == 4) rc = dispatch_tm<4, false, bf16, EPI_FOLD>(A, lda, W, bias, nullptr, 0, M, N, K, S, rows, stream, fold);
    else if (R == 2) rc = dispatch_tm<2, false, bf16, EPI_FOLD>(A, lda, W, bias, nullptr, 0, M, N, K, S, rows, stream, fold);
    else rc = dispatch_tm<1, false, bf16, EPI_FOLD>(A, lda, W, bias, nullptr, 0, M, N, K, S, rows, stream, fold);
    if (rc) return rc;
    return mv_check_launch("gemm_skinny_fold");
}

// The product behind such a norm: C = (A W^T) / rms (+ bias), or the gated pair
// silu(g / rms) * (u / rms), where A = the weighted rows [M, K] and rms[m] =
// sqrt(sum_p partial[m][p] / K + eps). bf16 out.
extern "C" int mv_gemm_skinny_scaled(const void* A, long lda, const void* W, const void* bias, void* C, long ldc,
                                     const float* partial, int P, float eps, int M, int N, int K, int swiglu,
                                     hipStream_t stream) {
    if (int rc = check_skinny("gemm_skinny_scaled", A, lda, W, ldc, M, N, K)) return rc;
    MV_REQUIRE(partial != nullptr && P > 0 && eps > 0.f, "gemm_skinny_scaled: bad partial sums (P=%d) or eps", P);
    if (M == 0) return 0;
    RowsInput fold{nullptr, 0, WeightPtr{nullptr, MV_BF16}, 0, nullptr, 0, const_cast<float*>(partial), P, eps, K};
    int rc = 0;
    if (swiglu) {
        const int S = pick_waves(K);
        rc = dispatch_tm<2, true, bf16, EPI_SCALED>(A, lda, W, nullptr, C, ldc, M, N, K, S,
                                                    M <= 16 ? pick_rows(N, 16) : 16, stream, fold);
    } else {
        int S, R, rows;
        skinny_shape(M, N, K, S, R, rows);
        if (R == 4) rc = dispatch_tm<4, false, bf16, EPI_SCALED>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream, fold);
        else if (R == 2) rc = dispatch_tm<2, false, bf16, EPI_SCALED>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream, fold);
        else rc = dispatch_tm<1, false, bf16, EPI_SCALED>(A, lda, W, bias, C, ldc, M, N, K, S, rows, stream, fold);
    }
    if (rc) return rc;
    return mv_check_launch("gemm_skinny_scaled");
}

// out[M, I] = silu(A Wgu[0:I]^T) * (A Wgu[I:2I]^T), bf16 in and out.
extern "C" int mv_gemm_skinny_swiglu(const void* A, long lda, const void* Wgu, void* out, long ldo, int M, int I,
                                     int K, hipStream_t stream) {
    if (int rc = check_skinny("gemm_skinny_swiglu", A, lda, Wgu, ldo, M, I, K)) return rc;
    if (M == 0) return 0;
    const int S = pick_waves(K);
    int rc = dispatch_tm<2, true, bf16>(A, lda, Wgu, nullptr, out, ldo, M, I, K, S, M <= 16 ? pick_rows(I, 16) : 16, stream);
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
    MV_REQUIRE(mv_valid_dtype(norm_weight_dtype) && norm_weight != nullptr && ((uintptr_t)norm_weight % 16) == 0,
               "gemm_skinny_norm: the norm weight is missing, of an unknown type or not 16-byte aligned");
    MV_REQUIRE(delta == nullptr || (resid_out != nullptr && resid_out != resid_in),
               "gemm_skinny_norm: the updated residual needs a buffer of its own");
    MV_REQUIRE(eps > 0.f, "gemm_skinny_norm: eps must be positive");
    MV_REQUIRE(ldc >= N, "gemm_skinny_norm: ldc=%ld smaller than N=%d", ldc, N);
    MV_REQUIRE(c_dtype == MV_BF16 || (c_dtype == MV_F32 && !swiglu), "gemm_skinny_norm: bad output dtype %d", c_dtype);
    if (M == 0) return 0;
    // enough waves to hold the rows in registers during the prologue, also where K alone asks for fewer
    const int chunks = M * ((K + 511) / 512);
    int S = pick_waves(K);
    if (S * SK_NORM_CHUNKS < chunks) S = (chunks + SK_NORM_CHUNKS - 1) / SK_NORM_CHUNKS;
    const int R = swiglu ? 2 : 1;
    if (M > 16 || K % 64 != 0 || S > SK_MAX_WAVES || skinny_lds_bytes(S, R, 1, true, M, K) > 60 * 1024) {
        mv_fail("gemm_skinny_norm: M=%d K=%d is not taken by the fused kernel", M, K);
        return 2;
    }
    NormInput norm{resid_in, (const bf16*)delta, resid_out, WeightPtr{norm_weight, norm_weight_dtype}, eps, unit_offset};
    if (swiglu) launch_skinny_norm<2, true, bf16>(norm, W, nullptr, C, ldc, M, N, K, S, stream);
    else if (c_dtype == MV_F32) launch_skinny_norm<1, false, float>(norm, W, bias, C, ldc, M, N, K, S, stream);
    else launch_skinny_norm<1, false, bf16>(norm, W, bias, C, ldc, M, N, K, S, stream);
    return mv_check_launch("gemm_skinny_norm");
}
