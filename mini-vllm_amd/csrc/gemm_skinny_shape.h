// The shapes of the weight-streaming product (gemm_skinny.hip), apart from its kernel: operand
// fragments, the inputs of the variants that take a norm apart, and the launch rules (waves,
// weight tiles and output columns per workgroup).
#pragma once
#include "dispatch.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    uint16_t s[8];
    bf16x8_t v;
};

#define SK_MAX_WAVES 8
#define SK_MAX_ROWS 512      // up to 64 rows per workgroup, more rows are dealt out to groups of workgroups
#define SK_COMPUTE_UNITS mv_compute_units()
#ifndef SK_STAGE_FRAGS
#define SK_STAGE_FRAGS 8    // 16-byte operand loads per lane in one register stage of the main loop
#endif
#define SK_NORM_CHUNKS 4   // chunks of 512 columns a wave holds in the fused norm's prologue
#ifndef SK_MIN_ROWS
#define SK_MIN_ROWS 4      // fewest output columns of a workgroup
#endif
#ifndef SK_WAVE_K
#define SK_WAVE_K 128      // fewest K elements of a wave
#endif

// What the FOLD and SCALED variants need beside the product (EPI below).
struct RowsInput {
    float* resid;            // FOLD: [M, N] float, updated in place: resid += bf16(product)
    long ldr;
    WeightPtr weight;        // FOLD: [N], the weight of the norm that follows
    int unit_offset;
    bf16* weighted;          // FOLD: [M, N] out: bf16(resid * weight)
    long ldw;
    float* partial;          // FOLD: [M, P] out, P = workgroups along N: sums of resid^2 over a workgroup's columns
                             // SCALED: the same array, read: row m of the input is to be divided by
                             //         sqrt(sum_p partial[m][p] / width + eps)
    int P;
    float eps;               // SCALED
    int width;               // SCALED: elements of an input row (the norm's size)
};

enum { EPI_NONE = 0, EPI_FOLD = 1, EPI_SCALED = 2 };

static inline int skinny_blocks(int N, int rows) { return (N + rows - 1) / rows; }

// Output columns per workgroup when there are few tiles and few tokens. The chip takes the
// workgroups in rounds of one per compute unit, and a last round that is not full costs as much as
// a full one (320 tiles on 256 units: two rounds for the work of 1.25). So a workgroup takes 8 to
// `most` columns, not a whole number of tiles, such that the rounds are as few and as full as
// possible: rounds * columns is what a unit streams. (The rows of a tile beyond the workgroup's
// own are loaded again from its last row.) Of equal choices the largest: fewer workgroups read
// the tokens.
static inline int pick_rows(int N, int most) {
    int rows = most;
    long best = -1;
    for (int p = most; p >= SK_MIN_ROWS; p -= 4) {
        const long wgs = (N + p - 1) / p;
        const long cost = ((wgs + SK_COMPUTE_UNITS - 1) / SK_COMPUTE_UNITS) * p;
        if (best < 0 || cost < best) {
            best = cost;
            rows = p;
        }
    }
    return rows;
}

static inline int pick_waves(int K) {
    int s = K / SK_WAVE_K;  // at least four MFMA steps per wave
    if (s < 1) s = 1;
    if (s > SK_MAX_WAVES) s = SK_MAX_WAVES;
    return s;
}

static inline int check_skinny(const char* what, const void* A, long lda, const void* W, long ldc, int M, int N, int K) {
    MV_REQUIRE(M >= 0 && M <= SK_MAX_ROWS, "%s: takes at most %d rows, got M=%d", what, SK_MAX_ROWS, M);
    MV_REQUIRE(N > 0 && K > 0 && K % 32 == 0, "%s: K=%d must be a positive multiple of 32 (N=%d)", what, K, N);
    MV_REQUIRE(lda >= K && lda % 8 == 0, "%s: lda=%ld must be a multiple of 8 and at least K=%d", what, lda, K);
    MV_REQUIRE(ldc >= N, "%s: ldc=%ld smaller than N=%d", what, ldc, N);
    MV_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "%s: operands must be 16-byte aligned", what);
    return 0;
}

// Waves per workgroup, weight tiles per workgroup and output columns per workgroup of the plain product.
static inline void skinny_shape(int M, int N, int K, int& S, int& R, int& rows) {
    S = pick_waves(K);
    const int tiles = (N + 15) / 16;
    const int TM = (M + 15) / 16;
    // more row tiles per workgroup reuse the activation registers; keep at least ~512 workgroups
    // and the partial tiles of the waves within 56 KiB of LDS
    R = tiles >= 2048 ? 4 : (tiles >= 1024 ? 2 : 1);
    // with three or four token tiles a workgroup of two weight tiles and two token tiles pulls less
    // from L2 than one of one and four, for the same number of workgroups (0.6B sizes, a step of 64
    // sequences: 1 % faster)
    if (R == 1 && TM >= 3 && tiles >= 256) R = 2;
    while (R > 1 && (size_t)(S - 1) * R * TM * 1024 > 56 * 1024) R /= 2;
    rows = 16 * R;
    if (R == 1 && M <= 16) {
        rows = pick_rows(N, 32);
        R = rows > 16 ? 2 : 1;
    }
}

