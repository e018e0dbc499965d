// Matrix product for the steps between a few rows and thousands (decode steps of 9 sequences and
// more against large weights, of 32 and more against small ones, prompt portions of up to 1,536
// tokens; the caller's rules say which):
//     C[M, N] = A[M, K] * W[N, K]^T (+ bias)      or      C[M, I] = silu(A Wg^T) * (A Wu^T),
// bf16 inputs, float accumulation, on the MFMA units of gfx950 (v_mfma_f32_16x16x32_bf16).
//
// A workgroup of four waves (2 x 2) owns a tile of BM = 32 WM tokens by BN = 32 WN weight rows
// and a slice of K; a wave owns 16 WM x 16 WN of it. K is walked in chunks of 64 columns. A
// chunk's rows of A and of W go from global memory straight into LDS (global_load_lds, no
// registers in between), STAGES - 1 chunks ahead of the computation, into a ring of stages: a chunk
// is multiplied in a fraction of the time it takes to arrive, so several are on their way at once.
//
// Global side: one load instruction takes 8 rows of 128 bytes (whole cache lines; lane l reads
// row l / 8). LDS side: the same instruction writes 1 KB lane after lane, so a row's eight 16-byte
// pieces sit side by side, rows 128 bytes apart, and sixteen lanes reading one piece of sixteen
// rows would meet in the same banks. So the pieces of row r are stored rotated: slot p of the row
// holds piece p ^ (r & 7) (the lane that fills slot p asks global memory for that piece), and the
// lane that needs piece c of row r reads slot c ^ (r & 7): eight neighbouring rows use eight
// different slots.
//
//   C^T tile = W A^T     A operand: 16 weight rows x 32 k, B operand: 32 k x 16 tokens;
//                        lane l ends up with C[token l%16][weight rows 4 (l/16) .. + 3]: four
//                        neighbours of a row of C, one 8- or 16-byte store.
//
// With few tiles K is split over F workgroups a tile; the float partial sums go to a work area
// [F][M][N] and a second kernel (gemm_mid's) adds them in a fixed order, applies bias or the gated
// activation and rounds: a row's result never depends on the other rows of the step. Workgroup
// ids are dealt to the eight XCDs in turn, so the tile of a workgroup is chosen such that an XCD
// walks a band of weight rows: a weight tile is read into one L2 only.
#include "dispatch.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union TFrag {
    uint4 u;
    bf16x8_t v;
};

#define GT_KC 64                    // columns of a chunk: 128 bytes a row
#define GT_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(0x0f70 | ((N) & 15) | (((N) >> 4) << 14))
#define GT_XCDS 8

// 16 bytes per lane from global memory straight into LDS: lane l's bytes land at lds_base + 16 l.
// Written as assembly so that the compiler neither counts nor guards it: the waits are the
// explicit ones below (the vector memory counter retires in order).
__device__ __forceinline__ void gt_load_to_lds(const void* src, __attribute__((address_space(3))) void* lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(src), "s"(lds_base)
                 : "memory", "m0");
}

struct TileArgs {
    const bf16* A;
    long lda;
    const bf16* W;
    const bf16* bias;
    void* C;
    long ldc;
    int c_f32;
    float* part;          // [F][M][N] when F > 1
    int M, N, K;
    int F, chunks_per_split;
    int tiles_m, tiles_n;
    int I;                // GATED: the gate rows are W[0, I), the up rows W[I, 2 I); N = 2 I
    // rows of A that a product in front left without the division of their norm: row m of the result
    // is divided by sqrt(sum_p partial[m][p] / K + eps) (before the bias, before the gate). Null: as is.
    const float* partial;
    int P;
    float eps;
};

template <int WM, int WN, bool GATED, int STAGES, int OCC>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
gemm_tile_kernel(TileArgs a) {
    constexpr int BM = 32 * WM, BN = 32 * WN;
    constexpr int ROWS = BM + BN;              // rows of a stage: the tile's tokens, then its weight rows
    constexpr int INSTR = ROWS / 8;            // load instructions of a chunk
    constexpr int REPS = INSTR / 4;            // ... of one wave
    static_assert(INSTR % 4 == 0, "the rows of a stage do not divide the four waves");
    static_assert(!GATED || WN % 2 == 0, "a wave's weight tiles are half gate, half up");
    constexpr int STAGE = ROWS * 8;            // uint4 units of a stage
    static_assert(STAGES >= 2 && STAGES <= 8 && (STAGES - 2) * REPS <= 63, "the ring does not fit the wait counter");
    __shared__ uint4 ring[STAGES * STAGE];
    __shared__ float sh_rinv[BM];
    __shared__ float sh_part[256 / BM >= 1 ? 256 / BM : 1][BM];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / MV_WAVE);
    const int lane = tid % MV_WAVE;
    const int i = lane % 16, g = lane / 16;
    const int wm = wave / 2, wn = wave % 2;

    // ---- which tile, which slice of K
    int id = blockIdx.x;
    const int total = gridDim.x;
    if (total % GT_XCDS == 0) id = (id % GT_XCDS) * (total / GT_XCDS) + id / GT_XCDS;
    const int f = id % a.F;
    const int tile = id / a.F;
    const int tm = tile % a.tiles_m, tn = tile / a.tiles_m;
    const int m0 = tm * BM;
    const int n0 = tn * (GATED ? BN / 2 : BN);      // GATED: first gate column of the tile
    const int chunks_total = a.K / GT_KC;
    const int c0 = f * a.chunks_per_split;
    int c1 = c0 + a.chunks_per_split;
    if (c1 > chunks_total) c1 = chunks_total;

    // ---- this lane's share of the loads: row 8 j + l / 8 of the stage, piece (l % 8) ^ (l / 8)
    const int lrow = lane / 8;
    const int piece = (lane % 8) ^ lrow;
    const char* src[REPS];
    int slot[REPS];
#pragma unroll
    for (int rep = 0; rep < REPS; ++rep) {
        const int j = wave + 4 * rep;
        const int row = 8 * j + lrow;
        slot[rep] = j * 64;
        if (row < BM) {
            int tok = m0 + row;
            tok = tok < a.M ? tok : a.M - 1;        // rows past the end: some row; their products are never stored
            src[rep] = reinterpret_cast<const char*>(a.A + (size_t)tok * a.lda + 8 * piece);
        } else {
            const int r = row - BM;
            int n;
            if (GATED) n = r < BN / 2 ? n0 + r : a.I + n0 + (r - BN / 2);
            else n = n0 + r;
            const int last = GATED ? (r < BN / 2 ? a.I - 1 : 2 * a.I - 1) : a.N - 1;
            n = n < last ? n : last;
            src[rep] = reinterpret_cast<const char*>(a.W + (size_t)n * a.K + 8 * piece);
        }
    }
    auto fetch = [&](int c, uint4* stage) {
#pragma unroll
        for (int rep = 0; rep < REPS; ++rep)
            gt_load_to_lds(src[rep] + (size_t)c * (GT_KC * sizeof(bf16)),
                           (__attribute__((address_space(3))) void*)(stage + slot[rep]));
    };

    // ---- operand reads: piece 4 ks + g of row (16 t + i), at slot (4 ks + g) ^ (i & 7)
    int a_off[WM], w_off[WN];      // in uint4 units, for ks = 0
#pragma unroll
    for (int t = 0; t < WM; ++t) a_off[t] = (16 * (WM * wm + t) + i) * 8;
#pragma unroll
    for (int t = 0; t < WN; ++t) {
        int group;                 // which sixteen rows of the stage's weight part
        if (GATED) group = t < WN / 2 ? (WN / 2) * wn + t : WN + (WN / 2) * wn + (t - WN / 2);
        else group = WN * wn + t;
        w_off[t] = (BM + 16 * group + i) * 8;
    }
    const int sw0 = g ^ (i & 7), sw1 = (4 + g) ^ (i & 7);

    floatx4_t acc[WN][WM];
#pragma unroll
    for (int t = 0; t < WN; ++t)
#pragma unroll
        for (int u = 0; u < WM; ++u) acc[t][u] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    auto multiply = [&](const uint4* stage) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int sw = ks ? sw1 : sw0;
            TFrag af[WM], wf[WN];
#pragma unroll
            for (int u = 0; u < WM; ++u) af[u].u = stage[a_off[u] + sw];
#pragma unroll
            for (int t = 0; t < WN; ++t) wf[t].u = stage[w_off[t] + sw];
#pragma unroll
            for (int t = 0; t < WN; ++t)
#pragma unroll
                for (int u = 0; u < WM; ++u)
                    acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[t].v, af[u].v, acc[t][u], 0, 0, 0);
        }
    };
    // Chunk k of this workgroup's n chunks lives in stage k % STAGES. Before it is multiplied: wait
    // until this wave's loads of it have landed (the loads of later chunks, at most STAGES - 2 of
    // them, may still be on their way: the counter retires in order), meet the other waves (their
    // loads have landed too, and everybody is done reading the stage of chunk k - 1), then ask for
    // chunk k + STAGES - 1, which goes into that stage.
    const int n = c1 - c0;
#pragma unroll
    for (int k = 0; k < STAGES - 1; ++k)
        if (k < n) fetch(c0 + k, ring + k * STAGE);
    // One over the root mean square of the tile's rows, from the sums the product in front left: 256 / BM
    // threads share a row (each adds every (256 / BM)-th sum, all loads of a thread in flight at once),
    // their sums are added in the order of the threads. It runs while the first chunks are on their way.
    if (a.partial != nullptr) {
        constexpr int Q = 256 / BM >= 1 ? 256 / BM : 1;
        const int row = tid % BM, q = tid / BM;
        const int tok = m0 + row;
        float ss = 0.f;
        if (q < Q && tok < a.M) {
            const float* src = a.partial + (size_t)tok * a.P;
            for (int p = q; p < a.P; p += 8 * Q) {
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = p + e * Q < a.P ? src[p + e * Q] : 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) ss += v[e];
            }
        }
        if (q < Q) sh_part[q][row] = ss;
        __syncthreads();
        if (tid < BM) {
            float t = 0.f;
#pragma unroll
            for (int e = 0; e < Q; ++e) t += sh_part[e][tid];
            sh_rinv[tid] = rsqrtf(t / (float)a.K + a.eps);
        }
    }

    int st = 0, st_fetch = STAGES - 1;
    for (int k = 0; k < n; ++k) {
        const int later = n - k - 1 < STAGES - 2 ? n - k - 1 : STAGES - 2;   // chunks that may stay in flight
        switch (later) {                                                    // (the wait takes an immediate)
            case 0: GT_WAIT_VMCNT(0); break;
            case 1: GT_WAIT_VMCNT(REPS); break;
            case 2: GT_WAIT_VMCNT(2 * REPS); break;
            case 3: GT_WAIT_VMCNT(3 * REPS); break;
            case 4: GT_WAIT_VMCNT(4 * REPS); break;
            case 5: GT_WAIT_VMCNT(5 * REPS); break;
            default: GT_WAIT_VMCNT(6 * REPS); break;
        }
        __builtin_amdgcn_s_barrier();
        if (k + STAGES - 1 < n) fetch(c0 + k + STAGES - 1, ring + st_fetch * STAGE);
        multiply(ring + st * STAGE);
        st = st + 1 == STAGES ? 0 : st + 1;
        st_fetch = st_fetch + 1 == STAGES ? 0 : st_fetch + 1;
    }

    // ---- lane l holds C[token 16 u + l%16][weight row of tile t + 4 (l/16) + 0..3]
    const int m_base = m0 + 16 * WM * wm;
    if (a.F > 1) {
        float* dst = a.part + (size_t)f * a.M * a.N;
#pragma unroll
        for (int t = 0; t < WN; ++t) {
            int col;
            if (GATED) col = (t < WN / 2 ? n0 + 16 * ((WN / 2) * wn + t) : a.I + n0 + 16 * ((WN / 2) * wn + t - WN / 2)) + 4 * g;
            else col = n0 + 16 * (WN * wn + t) + 4 * g;
            const int lim = GATED ? (t < WN / 2 ? a.I : 2 * a.I) : a.N;
#pragma unroll
            for (int u = 0; u < WM; ++u) {
                const int tok = m_base + 16 * u + i;
                if (tok >= a.M || col >= lim) continue;
                float* p = dst + (size_t)tok * a.N + col;
                if (col + 3 < lim && (a.N & 3) == 0 && (!GATED || (a.I & 3) == 0)) {
                    *reinterpret_cast<float4*>(p) = float4{acc[t][u][0], acc[t][u][1], acc[t][u][2], acc[t][u][3]};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < lim) p[e] = acc[t][u][e];
                }
            }
        }
        return;
    }
    constexpr int TOUT = GATED ? WN / 2 : WN;
    const int n_out = GATED ? a.I : a.N;
#pragma unroll
    for (int t = 0; t < TOUT; ++t) {
        const int col = n0 + 16 * ((GATED ? WN / 2 : WN) * wn + t) + 4 * g;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (!GATED && a.bias != nullptr) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < n_out) bv[e] = to_f(a.bias[col + e]);
        }
#pragma unroll
        for (int u = 0; u < WM; ++u) {
            const int tok = m_base + 16 * u + i;
            if (tok >= a.M || col >= n_out) continue;
            const float rinv = a.partial != nullptr ? sh_rinv[16 * (WM * wm + u) + i] : 1.f;
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (GATED) {
                    const float gt = acc[t][u][e] * rinv, up = acc[t + WN / 2][u][e] * rinv;
                    v[e] = gt / (1.f + expf(-gt)) * up;
                } else {
                    v[e] = acc[t][u][e] * rinv + bv[e];
                }
            }
            const bool whole = col + 3 < n_out;
            if (a.c_f32) {
                float* p = reinterpret_cast<float*>(a.C) + (size_t)tok * a.ldc + col;
                if (whole && (a.ldc & 3) == 0) {
                    *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < n_out) p[e] = v[e];
                }
            } else {
                bf16* p = reinterpret_cast<bf16*>(a.C) + (size_t)tok * a.ldc + col;
                if (whole && (a.ldc & 3) == 0) {
                    uint2 packed;
                    packed.x = f32x2_to_bf16x2_bits(v[0], v[1]);
                    packed.y = f32x2_to_bf16x2_bits(v[2], v[3]);
                    *reinterpret_cast<uint2*>(p) = packed;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < n_out) p[e] = from_f<bf16>(v[e]);
                }
            }
        }
    }
}

struct TilePlan {
    int wm, wn;            // wave tile in units of 16: the workgroup's tile is 32 wm x 32 wn
    int deep;              // the 128 x 128 tile with a ring of four stages, one workgroup a compute unit
    int F, chunks_per_split;
    int tiles_m, tiles_n;
};

#define GT_COMPUTE_UNITS mv_compute_units()

// The tile and the number of splits of K, by rules read off measurements on MI355X (weights of 4 MB to
// 500 MB, 33 to 2,048 rows). Weights below 16 MB: the largest tile no taller than the rows need that
// still makes about 192 workgroups (one for most compute units; more, smaller ones lose to their own
// barriers), else the smallest; K is split only where there are fewer than 64 tiles (at most four
// ways, at least eight chunks a split: the second kernel that adds the sums costs as much as eight
// chunks). Weights of 16 MB and more are bound by the memory and by how long one workgroup walks a
// row: the largest tile that makes 64 workgroups, K split so that tiles x splits comes as close to
// the 256 compute units as it can from below (a fifth quarter-round costs a whole one: 80 tiles are
// best split three ways, not four). The choice looks at sizes only: for a given (M, N, K) a row's sum
// is always split the same way. `n_out`: columns
// of the result (gated: of each half). `force` is for measurements: (wm, wn, F) packed as
// wm * 10000 + wn * 100 + F, wm + 10 for the deep ring; 0 lets the rule choose.
static TilePlan tile_plan(int M, int n_out, int K, bool gated, int force) {
    const int chunks = K / GT_KC;
    auto make = [&](int wm, int wn, int F, bool deep) {
        TilePlan p;
        p.deep = deep;
        p.wm = wm;
        p.wn = wn;
        const int cols = gated ? 16 * wn : 32 * wn;     // gated: a tile holds as many up columns again
        p.tiles_m = (M + 32 * wm - 1) / (32 * wm);
        p.tiles_n = (n_out + cols - 1) / cols;
        if (F < 1) F = 1;
        if (F > chunks) F = chunks;
        p.chunks_per_split = (chunks + F - 1) / F;
        p.F = (chunks + p.chunks_per_split - 1) / p.chunks_per_split;
        return p;
    };
    if (force > 0) return make((force / 10000) % 10, (force / 100) % 100, force % 100, force / 10000 >= 10);
    const bool big = (double)(gated ? 2 : 1) * n_out * K * 2 >= 16.0 * 1024 * 1024;
    const int m_cap = (M + 63) / 64 * 64;
    // (a gated pair is never split, so the tiles alone have to fill the chip: up to 48 rows the 64-row
    // tile's 384 workgroups beat the 128-row tile's 192 on 8B-sized pairs, 41.5 against 46.5 us at 12 rows;
    // at 64 rows the larger tile is ahead again, 45.9 against 47.6)
    const int need = big ? (gated && M <= 48 ? 256 : 64) : 192;
    const int shapes[4][2] = {{4, 4}, {4, 2}, {2, 4}, {2, 2}};
    TilePlan pick = make(2, 2, 1, false);
    for (int s = 0; s < 4; ++s) {
        const int wm = shapes[s][0], wn = shapes[s][1];
        if (32 * wm > m_cap || (gated && wm == 4 && wn == 2)) continue;
        const TilePlan p = make(wm, wn, 1, false);
        if ((long)p.tiles_m * p.tiles_n >= need) {
            pick = p;
            break;
        }
    }
    const long tiles = (long)pick.tiles_m * pick.tiles_n;
    int F = 1;
    if (big) {
        F = tiles >= GT_COMPUTE_UNITS ? 1 : (int)(GT_COMPUTE_UNITS / tiles);
        if (F > 8) F = 8;
        if (F > chunks / 8) F = chunks / 8;
    } else if (tiles < 64) {
        F = 4;
        if (F > chunks / 8) F = chunks / 8;
        if (F > GT_COMPUTE_UNITS / tiles) F = (int)(GT_COMPUTE_UNITS / tiles);
    }
    if (F < 1 || gated) F = 1;      // (the gated pair is never split here: its activation stays in the epilogue)
    pick = make(pick.wm, pick.wn, F, false);
    // one workgroup a compute unit at most: the 128 x 128 tile then takes the deeper ring
    pick.deep = pick.wm == 4 && pick.wn == 4 && tiles * pick.F <= GT_COMPUTE_UNITS;
    return pick;
}

static bool tile_shape_served(const TilePlan& p, bool gated) {
    if (p.deep && !(p.wm == 4 && p.wn == 4)) return false;
    return (p.wm == 4 && p.wn == 4) || (p.wm == 2 && p.wn == 4) || (p.wm == 2 && p.wn == 2) ||
           (p.wm == 4 && p.wn == 2 && !gated);
}

// Floats of work area (partial sums [F][M][N]) a product of this shape needs; 0 when K is not split.
extern "C" long mv_gemm_tile_workspace(int M, int N, int K, int gated, int force) {
    if (M <= 0 || N <= 0 || K <= 0 || K % GT_KC) return -1;
    const TilePlan p = tile_plan(M, gated ? N / 2 : N, K, gated != 0, force);
    return p.F > 1 ? (long)p.F * M * N : 0;
}

extern "C" int mv_gemm_tile_splits(int M, int N, int K, int gated, int force) {
    if (M <= 0 || N <= 0 || K <= 0 || K % GT_KC) return 0;
    return tile_plan(M, gated ? N / 2 : N, K, gated != 0, force).F;
}

// (gemm_mid.hip) C = sum over f < F of work[f] (+ bias), or the gated activation of the two halves of the sum
extern "C" int mv_gemm_mid_reduce(const float* work, const void* bias, void* C, long ldc, int c_dtype, int M, int N,
                                  int F, int swiglu, hipStream_t stream);

// C[M, N] = A W^T (+ bias), or with `gated` C[M, N / 2] = silu(A Wg^T) * (A Wu^T) for the packed weight
// [N = 2 I, K]. bf16 A (row stride lda) and W (contiguous rows of K), C bf16 or float (c_dtype).
// K a multiple of 64. `work`: the float area mv_gemm_tile_workspace asks for (may be null when it
// asks for none).
static int tile_launch(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int c_dtype, int M,
                       int N, int K, int gated, float* work, long work_floats, int force, bool reduce,
                       const float* partial, int P, float eps, hipStream_t stream) {
    MV_REQUIRE(M > 0 && N > 0 && K > 0 && K % GT_KC == 0, "gemm_tile: K=%d must be a positive multiple of %d (M=%d, N=%d)",
               K, GT_KC, M, N);
    MV_REQUIRE(lda >= K && lda % 8 == 0, "gemm_tile: lda=%ld must be a multiple of 8 and at least K=%d", lda, K);
    MV_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_tile: operands must be 16-byte aligned");
    MV_REQUIRE(c_dtype == MV_F32 || c_dtype == MV_BF16, "gemm_tile: bad output dtype %d", c_dtype);
    MV_REQUIRE(!gated || (N % 2 == 0 && bias == nullptr), "gemm_tile: the gated form takes an even N and no bias");
    MV_REQUIRE(ldc >= (gated ? N / 2 : N), "gemm_tile: ldc=%ld too small for N=%d", ldc, N);
    MV_REQUIRE((long)M * N < (1L << 31), "gemm_tile: %d x %d outputs exceed the index range", M, N);
    const TilePlan p = tile_plan(M, gated ? N / 2 : N, K, gated != 0, force);
    MV_REQUIRE(tile_shape_served(p, gated != 0), "gemm_tile: no kernel for wave tiles %d x %d%s", p.wm, p.wn,
               p.deep ? " with the deep ring" : "");
    MV_REQUIRE(p.F == 1 || (work != nullptr && ((uintptr_t)work % 16) == 0 && work_floats >= (long)p.F * M * N),
               "gemm_tile: the work area holds %ld floats, %ld are needed", work_floats, (long)p.F * M * N);
    MV_REQUIRE(partial == nullptr || (p.F == 1 && P > 0 && eps > 0.f),
               "gemm_tile: rows without their norm's division need an unsplit K (F=%d), their sums (P=%d) and eps", p.F, P);
    TileArgs a{(const bf16*)A, lda, (const bf16*)W, (const bf16*)bias, C, ldc, c_dtype == MV_F32, p.F > 1 ? work : nullptr,
               M, N, K, p.F, p.chunks_per_split, p.tiles_m, p.tiles_n, gated ? N / 2 : 0, partial, P, eps};
    const dim3 grid((unsigned)((long)p.tiles_m * p.tiles_n * p.F));
    // rings: 128 x 128 tiles 2 stages of 32 KB with two workgroups a compute unit, or 4 with one;
    // 64 x 128 and 128 x 64 3 stages of 24 KB, 64 x 64 4 stages of 16 KB, two workgroups a unit
#define GT_LAUNCH(WMV, WNV, GV, SV, OV) \
    hipLaunchKernelGGL((gemm_tile_kernel<WMV, WNV, GV, SV, OV>), grid, dim3(256), 0, stream, a)
    if (gated) {
        if (p.wm == 4 && p.wn == 4 && p.deep) GT_LAUNCH(4, 4, true, 4, 1);
        else if (p.wm == 4 && p.wn == 4) GT_LAUNCH(4, 4, true, 2, 2);
        else if (p.wm == 2 && p.wn == 4) GT_LAUNCH(2, 4, true, 3, 2);
        else GT_LAUNCH(2, 2, true, 4, 2);
    } else {
        if (p.wm == 4 && p.wn == 4 && p.deep) GT_LAUNCH(4, 4, false, 4, 1);
        else if (p.wm == 4 && p.wn == 4) GT_LAUNCH(4, 4, false, 2, 2);
        else if (p.wm == 2 && p.wn == 4) GT_LAUNCH(2, 4, false, 3, 2);
        else if (p.wm == 4 && p.wn == 2) GT_LAUNCH(4, 2, false, 3, 2);
        else GT_LAUNCH(2, 2, false, 4, 2);
    }
#undef GT_LAUNCH
    if (int rc = mv_check_launch("gemm_tile")) return rc;
    if (p.F > 1 && reduce) return mv_gemm_mid_reduce(work, bias, C, ldc, c_dtype, M, N, p.F, gated, stream);
    return 0;
}

extern "C" int mv_gemm_tile(const void* A, long lda, const void* W, const void* bias, void* C, long ldc, int c_dtype,
                            int M, int N, int K, int gated, float* work, long work_floats, int force,
                            hipStream_t stream) {
    return tile_launch(A, lda, W, bias, C, ldc, c_dtype, M, N, K, gated, work, work_floats, force, true, nullptr, 0, 0.f,
                       stream);
}

// The same for rows that a product in front left weighted but not yet divided by their root mean
// square (see mv_gemm_skinny_fold): output row m is divided by sqrt(sum_p partial[m][p] / K + eps).
// Only for shapes whose K is not split (mv_gemm_tile_splits == 1).
extern "C" int mv_gemm_tile_scaled(const void* A, long lda, const void* W, const void* bias, void* C, long ldc,
                                   int c_dtype, int M, int N, int K, int gated, const float* partial, int P, float eps,
                                   hipStream_t stream) {
    MV_REQUIRE(partial != nullptr, "gemm_tile_scaled: the partial sums are missing");
    return tile_launch(A, lda, W, bias, C, ldc, c_dtype, M, N, K, gated, nullptr, 0, 0, true, partial, P, eps, stream);
}

// The partial sums alone, for a shape whose K is split (mv_gemm_tile_splits > 1): work[f][m][n] =
// the sum over split f, to be added up (with the bias) by whoever uses the result.
extern "C" int mv_gemm_tile_sums(const void* A, long lda, const void* W, int M, int N, int K, float* work,
                                 long work_floats, int force, hipStream_t stream) {
    MV_REQUIRE(mv_gemm_tile_splits(M, N, K, 0, force) > 1, "gemm_tile_sums: K is not split for M=%d N=%d K=%d", M, N, K);
    return tile_launch(A, lda, W, nullptr, work, N, MV_F32, M, N, K, 0, work, work_floats, force, false, nullptr, 0, 0.f,
                       stream);
}
