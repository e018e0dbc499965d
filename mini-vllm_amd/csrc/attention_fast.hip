// Paged attention for decode steps (one query token per sequence) on the MFMA units of gfx950,
// bf16 in and out, float inside.
//
// A workgroup serves one key/value head of one sequence; the query heads of the group are the
// columns of the problem (at most 16), so the keys and values are read once for the whole group.
//
//   scores^T = K Q^T     A operand: 16 keys x 32 d of the key page (one 16-byte load per lane),
//                        B operand: 32 d x 16 columns of the queries (kept in registers);
//                        result: lane l holds column l%16, keys 4*(l/16)+0..3 of the tile.
//   out^T    = V^T P^T   A operand: 16 d x 32 keys of the transposed value page,
//                        B operand: 32 keys x 16 columns of the probabilities.
// The probabilities a lane needs for the second product are exactly the scores it holds after
// the first: its eight k-slots are bound to the keys {4g..4g+3} of two neighbouring 16-key
// tiles (g = l/16), and the value operand is loaded for the same keys, so nothing is shuffled.
// Each column keeps its own running maximum and sum (online softmax, base 2).
//
// The W waves of a workgroup (4 or 8) take the 32-key blocks in turn, each with the K operands
// of its next block already in flight, and their partial results are merged through LDS. With
// nsplit > 1 several workgroups split a sequence's keys further and a second kernel merges
// their partial results.
//
// Layouts: K[page][kv_head][slot][d], V[page][kv_head][d][slot]; the page size is a multiple of
// 16. Keys outside the range (above the query's position, or more than `window` below it) get
// probability zero; value slots that were never written are read as zero.
#include "dispatch.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    uint2 h[2];
    uint16_t s[8];
    bf16x8_t v;
};

#define LOG2E 1.4426950408889634f
#define AF_MAX_CACHED_PAGES 1024

__device__ __forceinline__ int wave_max_i(int v) {
#pragma unroll
    for (int o = MV_WAVE / 2; o > 0; o >>= 1) {
        const int t = __shfl_xor(v, o, MV_WAVE);
        v = t > v ? t : v;
    }
    return v;
}

__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
    for (int o = MV_WAVE / 2; o > 0; o >>= 1) {
        const int t = __shfl_xor(v, o, MV_WAVE);
        v = t < v ? t : v;
    }
    return v;
}

// What the FUSED variant does itself instead of reading finished queries and a finished cache:
// the rows of the step's [q | k | v] product are normalised per head (RMSNorm, when weights are
// given) and rotated (half-split pairs, table row = cat(cos, sin) of the position, when a table
// is given) on the way into the registers; with `store` the new key and value also go to their
// page slot, and the wave that meets that slot among its keys uses the registers, not the page.
struct FusedInput {
    const bf16* qkv;        // [tokens, stride]
    long stride;
    int q_off, k_off, v_off;
    WeightPtr qw, kw;       // [D] each
    int has_norm;
    float eps;
    int unit_offset;
    const float* table;     // [positions, D] or null
    int store;
    const int* token_seq;   // rows that belong to no sequence (< 0) are left alone
};

// A head's raw elements (DS groups of eight a lane, d = 32 s + 8 g + e; the four lane groups g
// hold a head between them) are normalised (weights w[D], or null), rotated (cs = cat(cos, sin) of
// the position, or null; element d pairs with d + D/2: the same lane, DS/2 groups further) and
// rounded to the operand type. w and cs lie in LDS.
template <int DS>
__device__ __forceinline__ void norm_rotate(const Frag (&raw)[DS], int g, const float* w, float eps, const float* cs,
                                            int D, Frag (&dst)[DS]) {
    float x[DS][8];
#pragma unroll
    for (int s = 0; s < DS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) x[s][e] = (float)raw[s].v[e];
    if (w != nullptr) {
        float ss = 0.f;
#pragma unroll
        for (int s = 0; s < DS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += x[s][e] * x[s][e];
        ss += __shfl_xor(ss, 16, MV_WAVE);
        ss += __shfl_xor(ss, 32, MV_WAVE);
        const float rinv = rsqrtf(ss / (float)D + eps);
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            const float4 w0 = *reinterpret_cast<const float4*>(w + 32 * s + 8 * g);
            const float4 w1 = *reinterpret_cast<const float4*>(w + 32 * s + 8 * g + 4);
            const float wt[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) x[s][e] = x[s][e] * rinv * wt[e];
        }
    }
    if (cs != nullptr) {
        constexpr int HS = DS / 2;
#pragma unroll
        for (int s = 0; s < HS; ++s) {
            const float4 c0 = *reinterpret_cast<const float4*>(cs + 32 * s + 8 * g);
            const float4 c1 = *reinterpret_cast<const float4*>(cs + 32 * s + 8 * g + 4);
            const float4 s0 = *reinterpret_cast<const float4*>(cs + D / 2 + 32 * s + 8 * g);
            const float4 s1 = *reinterpret_cast<const float4*>(cs + D / 2 + 32 * s + 8 * g + 4);
            const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
            const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float a = x[s][e], b = x[s + HS][e];
                x[s][e] = a * c[e] - b * sn[e];
                x[s + HS][e] = b * c[e] + a * sn[e];
            }
        }
    }
#pragma unroll
    for (int s = 0; s < DS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[s].s[e] = f32_to_bf16_bits(x[s][e]);
}

// OCC workgroups are to share a compute unit (W / 4 waves of each on every SIMD): the register budget.
template <int D, int W, bool FUSED, int OCC>
__global__ void __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(OCC * W / 4, OCC * W / 4)))
attention_decode_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                      const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                      const int* __restrict__ block_table, int bt_width, int page_size,
                      const int* __restrict__ positions, const int* __restrict__ cu_seqlens, int n_seqs,
                      int H, int Hkv, float scale, int window, float* __restrict__ partials,
                      int nsplit, FusedInput fz) {
    constexpr int DS = D / 32;
    constexpr int DT = D / 16;
    constexpr int NT = 1;      // column tiles of a wave (the group's heads fit one tile)
    constexpr int COLS = 16;   // columns of a workgroup
    const int G = H / Hkv;
    const int kvh = blockIdx.y;
    const int split = blockIdx.z;
    const int wave = threadIdx.x / MV_WAVE;
    const int lane = threadIdx.x % MV_WAVE;
    const int i = lane % 16;
    const int g = lane / 16;
    const int tpu = COLS / G;  // tokens of a unit (the host made sure it is >= 1)

    __shared__ int sh_unit[3];
    int seq, t0, nt;
    if (FUSED) {
        // a decode step: row t of the step is the one token of sequence t (or padding)
        seq = blockIdx.x;
        t0 = seq;
        nt = fz.token_seq[t0] >= 0 ? 1 : 0;
    } else {
        if (threadIdx.x == 0) {
            const int s0 = blockIdx.x;
            const int first = cu_seqlens[s0];
            int count = cu_seqlens[s0 + 1] - first;
            if (count > tpu) count = tpu;
            sh_unit[0] = s0;
            sh_unit[1] = first;
            sh_unit[2] = count;
        }
        __syncthreads();
        seq = sh_unit[0];
        t0 = sh_unit[1];
        nt = sh_unit[2];
    }
    if (seq < 0 || nt <= 0) return;
    const int ncols = nt * G;
    const int* bt = block_table + (size_t)seq * bt_width;

    // ---- this lane's columns
    int col_tok[NT], col_head[NT], col_pos[NT], col_lo[NT];
    bool col_ok[NT];
    Frag qop[NT][DS];
    int hi_w = -1, lo_w = 0x7fffffff;
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        const int col = ct * 16 + i;
        col_ok[ct] = col < ncols;
        col_tok[ct] = t0 + (col_ok[ct] ? col / G : 0);
        col_head[ct] = kvh * G + (col_ok[ct] ? col % G : 0);
        col_pos[ct] = col_ok[ct] ? positions[FUSED ? t0 : col_tok[ct]] : -1;   // FUSED: one token, one position
        col_lo[ct] = (window >= 0 && col_pos[ct] - window > 0) ? col_pos[ct] - window : 0;
        if (col_ok[ct]) {
            hi_w = col_pos[ct] > hi_w ? col_pos[ct] : hi_w;
            lo_w = col_lo[ct] < lo_w ? col_lo[ct] : lo_w;
        }
        // the query rows: finished, or (FUSED) raw, to be normalised and rotated further down while
        // the first keys are on their way
        const bf16* qrow = FUSED ? fz.qkv + (size_t)col_tok[ct] * fz.stride + fz.q_off + (size_t)col_head[ct] * D + 8 * g
                                 : q + (size_t)col_tok[ct] * q_stride + (size_t)col_head[ct] * D + 8 * g;
#pragma unroll
        for (int s = 0; s < DS; ++s)
            qop[ct][s].u = col_ok[ct] ? *reinterpret_cast<const uint4*>(qrow + 32 * s) : uint4{0u, 0u, 0u, 0u};
    }
    if (FUSED) {   // known without asking the other lanes
        hi_w = positions[t0];
        lo_w = (window >= 0 && hi_w - window > 0) ? hi_w - window : 0;
    } else {
        hi_w = wave_max_i(hi_w);
        lo_w = wave_min_i(lo_w);
    }

    float m_run[NT], l_run[NT];
    floatx4_t acc_o[NT][DT];
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        m_run[ct] = -INFINITY;
        l_run[ct] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc_o[ct][dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    }

    // ---- the 32-key blocks of this wave
    int b_begin = 0, b_end = 0, b_step = 1;
    if (hi_w >= 0) {
        const int b0 = lo_w / 32, b1 = hi_w / 32;
        const int nblocks = b1 - b0 + 1;
        const int per = (nblocks + nsplit - 1) / nsplit;
        b_begin = b0 + split * per + wave;
        b_end = b0 + (split + 1) * per;
        if (b_end > b1 + 1) b_end = b1 + 1;
        b_step = W;
    }
    const float sc_mul = scale * LOG2E;

    // (FUSED) the norm weights and the table row of the position go to LDS with the page ids; the
    // wave that will meet the newest position among its keys asks for the raw key and value now
    __shared__ __attribute__((aligned(16))) float sh_const[FUSED ? 3 : 1][FUSED ? D : 1];
    const int b_new = hi_w >= 0 ? hi_w / 32 : -1;
    const bool owns_new = FUSED && fz.store && b_new >= b_begin && b_new < b_end && (b_new - b_begin) % b_step == 0;
    Frag knew[DS], kraw[DS];
    uint16_t vnew[DT];
    if (FUSED) {
        for (int d = threadIdx.x; d < D; d += blockDim.x) {
            if (fz.has_norm) {
                sh_const[0][d] = fz.qw.at(d) + (fz.unit_offset ? 1.f : 0.f);
                if (fz.kw.p != nullptr) sh_const[1][d] = fz.kw.at(d) + (fz.unit_offset ? 1.f : 0.f);
            }
            if (fz.table != nullptr) sh_const[2][d] = fz.table[(size_t)(hi_w >= 0 ? hi_w : 0) * D + d];
        }
#pragma unroll
        for (int s = 0; s < DS; ++s) knew[s].u = kraw[s].u = uint4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vnew[dt] = 0;
        if (owns_new) {
            const bf16* row = fz.qkv + (size_t)t0 * fz.stride;
            const bf16* krow = row + fz.k_off + (size_t)kvh * D + 8 * g;
#pragma unroll
            for (int s = 0; s < DS; ++s) kraw[s].u = *reinterpret_cast<const uint4*>(krow + 32 * s);
            const uint16_t* vrow = reinterpret_cast<const uint16_t*>(row + fz.v_off + (size_t)kvh * D);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vnew[dt] = vrow[16 * dt + i];
        }
    }

    // The page ids of this workgroup's key range go to LDS first (one round trip instead of one
    // per block); K and V operands are fetched one block ahead of their use.
    __shared__ int sh_pages[AF_MAX_CACHED_PAGES];
    const int first_block = hi_w >= 0 ? b_begin - wave : 0;          // of this workgroup's share of the keys
    const int p_first = (32 * first_block) / page_size;
    {
        int last_key = 32 * b_end - 1;
        if (last_key > hi_w) last_key = hi_w;
        const int p_last = (hi_w >= 0 && b_end > first_block) ? last_key / page_size : -1;
        for (int p = p_first + (int)threadIdx.x; p <= p_last && p - p_first < AF_MAX_CACHED_PAGES; p += blockDim.x)
            sh_pages[p - p_first] = p < bt_width ? bt[p] : -1;
    }
    __syncthreads();
    auto page_of = [&](int pidx) -> int {
        if (pidx >= bt_width) return -1;
        const int rel = pidx - p_first;
        return rel < AF_MAX_CACHED_PAGES ? sh_pages[rel] : bt[pidx];
    };
    struct Operands {
        int page[2];
        Frag k[2][DS];
        Frag v[DT];
    };
    auto fetch = [&](int b, Operands& op) {
        int slot0[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key0 = 32 * b + 16 * t;
            const int pidx = key0 / page_size;
            op.page[t] = (b < b_end && key0 <= hi_w) ? page_of(pidx) : -1;
            slot0[t] = key0 - pidx * page_size;
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (op.page[t] >= 0) {
                const size_t head = (size_t)op.page[t] * Hkv + kvh;
                const bf16* kptr = k_pages + ((head * page_size + slot0[t] + i) * D + 8 * g);
#pragma unroll
                for (int s = 0; s < DS; ++s) op.k[t][s].u = *reinterpret_cast<const uint4*>(kptr + 32 * s);
                const bf16* vptr = v_pages + (head * D + i) * page_size + slot0[t] + 4 * g;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    op.v[dt].h[t] = *reinterpret_cast<const uint2*>(vptr + (size_t)16 * dt * page_size);
            } else {
#pragma unroll
                for (int s = 0; s < DS; ++s) op.k[t][s].u = uint4{0u, 0u, 0u, 0u};
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) op.v[dt].h[t] = uint2{0u, 0u};
            }
        }
    };
    auto compute = [&](int b, Operands& op) {
        const int base = 32 * b;
        if (FUSED && owns_new && b == b_new) {   // the newest key and value come from the registers
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                if (base + 16 * t + i == hi_w) {
#pragma unroll
                    for (int s = 0; s < DS; ++s) op.k[t][s] = knew[s];
                }
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (base + 16 * t + 4 * g + r == hi_w) {
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) op.v[dt].s[t * 4 + r] = vnew[dt];
                    }
            }
        }
        // scores^T for two tiles of 16 keys
        float p[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            floatx4_t sacc = floatx4_t{0.f, 0.f, 0.f, 0.f};
            if (op.page[t] >= 0) {
#pragma unroll
                for (int s = 0; s < DS; ++s)
                    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(op.k[t][s].v, qop[0][s].v, sacc, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = base + 16 * t + 4 * g + r;
                const bool ok = op.page[t] >= 0 && col_ok[0] && key <= col_pos[0] && key >= col_lo[0];
                p[t][r] = ok ? sacc[r] * sc_mul : -INFINITY;
            }
        }
        // online softmax per column
        Frag pop;
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) mx = fmaxf(mx, p[t][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 16, MV_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, MV_WAVE));
        const float m_new = fmaxf(m_run[0], mx);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m_run[0] - m_safe);   // exp2(-inf) = 0
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(p[t][r] - m_safe);
                psum += e;
                pop.v[t * 4 + r] = (__bf16)e;
            }
        l_run[0] = l_run[0] * corr + psum;
        m_run[0] = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc_o[0][dt] *= corr;
        // out^T += V^T P^T
        if (base + 31 > hi_w) {  // slots above the newest key were never written
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (base + 16 * t + 4 * g + r > hi_w) op.v[dt].s[t * 4 + r] = 0;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            acc_o[0][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(op.v[dt].v, pop.v, acc_o[0][dt], 0, 0, 0);
    };

    Operands oa, ob;
    fetch(b_begin, oa);
    if (FUSED) {   // while those loads are in flight
        const float* cs = fz.table != nullptr ? sh_const[2] : nullptr;
        norm_rotate<DS>(qop[0], g, fz.has_norm ? sh_const[0] : nullptr, fz.eps, cs, D, qop[0]);
        if (owns_new) {
            norm_rotate<DS>(kraw, g, fz.has_norm ? sh_const[1] : nullptr, fz.eps, cs, D, knew);
            const int page = page_of(hi_w / page_size);
            if (page >= 0) {
                const int slot = hi_w % page_size;
                const size_t head = (size_t)page * Hkv + kvh;
                if (i == 0) {
                    bf16* kdst = const_cast<bf16*>(k_pages) + ((head * page_size + slot) * D + 8 * g);
#pragma unroll
                    for (int s = 0; s < DS; ++s) *reinterpret_cast<uint4*>(kdst + 32 * s) = knew[s].u;
                }
                if (g == 0) {
                    uint16_t* vdst = reinterpret_cast<uint16_t*>(const_cast<bf16*>(v_pages)) + (head * D + i) * page_size + slot;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) vdst[(size_t)16 * dt * page_size] = vnew[dt];
                }
            }
        }
    }
    for (int b = b_begin; b < b_end; b += 2 * b_step) {
        fetch(b + b_step, ob);
        compute(b, oa);
        if (b + b_step >= b_end) break;
        fetch(b + 2 * b_step, oa);
        compute(b + b_step, ob);
    }

    // the sum of a column is spread over the four lane groups
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        l_run[ct] += __shfl_xor(l_run[ct], 16, MV_WAVE);
        l_run[ct] += __shfl_xor(l_run[ct], 32, MV_WAVE);
    }

    // ---- merge the waves' partial results (same columns, disjoint keys) through LDS, half of the
    // d tiles at a time
    constexpr int HALF = DT / 2;
    __shared__ float sm_m[W][16];
    __shared__ float sm_l[W][16];
    __shared__ float sm_o[W][HALF][4][MV_WAVE];
    if (g == 0) {
        sm_m[wave][i] = m_run[0];
        sm_l[wave][i] = l_run[0];
    }
    __syncthreads();
    float m_fin = -INFINITY;
#pragma unroll
    for (int w = 0; w < W; ++w) m_fin = fmaxf(m_fin, sm_m[w][i]);
    float f[W], l_fin = 0.f;
#pragma unroll
    for (int w = 0; w < W; ++w) {
        const float mw = sm_m[w][i];
        f[w] = (mw == -INFINITY) ? 0.f : exp2f(mw - m_fin);
        l_fin += f[w] * sm_l[w][i];
    }
    float* prow = nullptr;
    bf16* orow = nullptr;
    if (col_ok[0]) {
        prow = partials ? partials + (((size_t)col_tok[0] * H + col_head[0]) * nsplit + split) * (D + 2) : nullptr;
        orow = out + (size_t)col_tok[0] * out_stride + (size_t)col_head[0] * D;
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        if (half) __syncthreads();
#pragma unroll
        for (int dt = 0; dt < HALF; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) sm_o[wave][dt][r][lane] = acc_o[0][half * HALF + dt][r];
        __syncthreads();
        if (col_ok[0]) {
            // the d tiles of this half are dealt out to the waves
            for (int dt = wave; dt < HALF; dt += W) {
                float o[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float a = 0.f;
#pragma unroll
                    for (int w = 0; w < W; ++w) a += f[w] * sm_o[w][dt][r][lane];
                    o[r] = a;
                }
                const int d0 = 16 * (half * HALF + dt) + 4 * g;
                if (nsplit == 1) {
                    const float inv = 1.f / l_fin;
                    uint2 packed;
                    packed.x = f32x2_to_bf16x2_bits(o[0] * inv, o[1] * inv);
                    packed.y = f32x2_to_bf16x2_bits(o[2] * inv, o[3] * inv);
                    *reinterpret_cast<uint2*>(orow + d0) = packed;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) prow[d0 + r] = o[r];
                }
            }
        }
    }
    if (nsplit > 1 && wave == 0 && g == 0 && col_ok[0]) {
        prow[D] = m_fin;
        prow[D + 1] = l_fin;
    }
}

// ---------------------------------------------------------------------------------------
// The one-wave variant, for steps whose grid is small (few sequences): a workgroup is a single
// wave that takes a fixed chunk of 32 * BPW keys of one (sequence, kv head) pair, asks for all of
// its keys and values at once and never meets a barrier or another wave. It is written for few
// instructions on the wave's path (a wave issues one instruction in about four cycles, so a
// thousand instructions are two microseconds whatever the memory does):
//   * which keys a chunk holds does not depend on the sequence's length, so the page ids are
//     asked for together with the position, not after it;
//   * the scores of the whole chunk are made first, one maximum is taken over them, and the
//     values are added up under that maximum: no rescaling between blocks;
//   * tiles wholly inside the visible range skip the masks; the tile of the newest key takes the
//     mask, the clearing of slots that were never written and (fused) the new key and value;
//   * the query is scaled by scale * log2(e) once, where it is normalised (fused);
//   * lanes whose column is no head of the group work on a copy of the last head and store nothing.
// Chunks above the newest key (or below the window) end at once. The last chunk also takes
// whatever lies above it (contexts longer than the launch was planned for), chunk after chunk with
// the usual rescaling. Each chunk leaves (o, m, l) in partials[token][head][chunk];
// attention_merge_range_kernel adds up the chunks a sequence really has. A sequence that has one
// chunk only gets its finished output row here. One token a sequence; the page size is a power of two.
// ---------------------------------------------------------------------------------------
template <int DS>
__device__ __forceinline__ void prepare_head(const Frag (&raw)[DS], int g, const WeightPtr& w, int has_norm, int unit_offset,
                                             float eps, const float* cs, float post_scale, int D, Frag (&dst)[DS]) {
    // the lane's 8 * DS elements of a head (d = 32 s + 8 g + e): RMSNorm over the head (the four lane
    // groups hold it between them), rotation by the table row cs = cat(cos, sin) (pairs d, d + D/2: the
    // same lane, DS/2 groups further), a scale, and rounding to the operand type. `w` and
    // `post_scale` may differ from lane to lane (a column that holds a key beside the query heads).
    // The norm's factor and the scale are one number per lane; it goes into the cosines and sines
    // where there is a rotation (which is linear), else into the weights.
    float x[DS][8];
#pragma unroll
    for (int s = 0; s < DS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) x[s][e] = (float)raw[s].v[e];
    float factor = post_scale;
    if (has_norm) {
        float ss = 0.f;
#pragma unroll
        for (int s = 0; s < DS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += x[s][e] * x[s][e];
        ss += __shfl_xor(ss, 16, MV_WAVE);
        ss += __shfl_xor(ss, 32, MV_WAVE);
        factor *= rsqrtf(ss / (float)D + eps);
        const float uo = unit_offset ? 1.f : 0.f;
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            float wt[8];
            w.at8(32 * s + 8 * g, wt);
            if (cs != nullptr) {
#pragma unroll
                for (int e = 0; e < 8; ++e) x[s][e] *= wt[e] + uo;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) x[s][e] *= (wt[e] + uo) * factor;
            }
        }
    }
    if (cs != nullptr) {
        constexpr int HS = DS / 2;
#pragma unroll
        for (int s = 0; s < HS; ++s) {
            const float4 c0 = *reinterpret_cast<const float4*>(cs + 32 * s + 8 * g);
            const float4 c1 = *reinterpret_cast<const float4*>(cs + 32 * s + 8 * g + 4);
            const float4 s0 = *reinterpret_cast<const float4*>(cs + D / 2 + 32 * s + 8 * g);
            const float4 s1 = *reinterpret_cast<const float4*>(cs + D / 2 + 32 * s + 8 * g + 4);
            const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
            const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float cc = c[e] * factor, sc = sn[e] * factor;
                const float a = x[s][e], b = x[s + HS][e];
                x[s][e] = a * cc - b * sc;
                x[s + HS][e] = b * cc + a * sc;
            }
        }
    } else if (!has_norm && post_scale != 1.f) {
#pragma unroll
        for (int s = 0; s < DS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) x[s][e] *= post_scale;
    }
#pragma unroll
    for (int s = 0; s < DS; ++s) {
        dst[s].u.x = f32x2_to_bf16x2_bits(x[s][0], x[s][1]);
        dst[s].u.y = f32x2_to_bf16x2_bits(x[s][2], x[s][3]);
        dst[s].u.z = f32x2_to_bf16x2_bits(x[s][4], x[s][5]);
        dst[s].u.w = f32x2_to_bf16x2_bits(x[s][6], x[s][7]);
    }
}

// Rows of the two 16-key score tiles of a 32-key block are bound to keys so that a lane ends up
// with eight neighbouring keys: tile tt, row rho  <->  key 8 * (rho / 4) + 4 * tt + rho % 4 of the
// block. After the first product lane (column, g) holds the scores of keys 8g .. 8g+7 (tile 0:
// 8g .. 8g+3, tile 1: 8g+4 .. 8g+7), which are the eight k-slots of its operand in the second
// product, and the value operand of a lane is one 16-byte load from the transposed page.
//
// What a wave does with its chunk. EDGE: the chunk touches an end of the visible range (it holds the
// newest key, or keys below a window's lower end, or it is the last chunk of a plan that is shorter
// than the sequence); only then are there masks, slots to clear, the new key and value, and more
// rounds than one. Chunks wholly inside the range take the other instantiation, which has none of
// that code. The order of the phases is pinned (keys asked for, query finished, values asked for,
// scores, sum): it keeps the registers in use below what a lane has, and the query's arithmetic
// runs while the keys are on their way.
struct WaveChunk {
    const bf16* k_pages;
    const bf16* v_pages;
    const int* bt;
    int bt_width, page_size, page_shift, Hkv, kvh, z, nchunks, pos, lo, b_hi;
    int i, g;
    float sc_mul;
    bool owns_new;
    int kcol;          // the query operand's column in which the new key rides (16: none)
    int t0;
    const float* cs;
};

template <int D, bool FUSED, int BPW, bool PS16, bool EDGE>
__device__ __forceinline__ void wave_chunk(const WaveChunk& c, const FusedInput& fz, Frag (&qop)[D / 32], int (&pga)[BPW],
                                           int (&pgb)[BPW], float& m_run, float& l_run,
                                           floatx4_t (&acc_o)[D / 16]) {
    constexpr int DS = D / 32;
    constexpr int DT = D / 16;
    const int page_size = PS16 ? 16 : c.page_size;
    const int page_shift = PS16 ? 4 : c.page_shift;
    const int slot_mask = page_size - 1;
    const int i = c.i, g = c.g, pos = c.pos, lo = c.lo;
    const size_t page_elems = (size_t)c.Hkv * page_size * D;      // elements of one page of keys (or values)
    // this lane's key rows of a block: tile tt, row i is key 8 * (i / 4) + 4 * tt + i % 4 of the block
    const int krow0 = 8 * (i >> 2) + (i & 3);
    const bf16* kbase = c.k_pages + (size_t)c.kvh * page_size * D + 8 * g;
    const bf16* vbase = c.v_pages + ((size_t)c.kvh * D + i) * page_size;
    const bool last_chunk = c.z == c.nchunks - 1;
    // with the new key and value coming from the registers, their slot in the page counts as unwritten
    const int pos_read = (EDGE && c.owns_new) ? pos - 1 : pos;

    // The new key (EDGE, fused, the wave that meets the new position among its keys): its raw row has
    // been loaded into the query operand's column `kcol`, a column that holds no query head, and is
    // normalised and rotated there together with the queries, with the key's weights and no scale.
    // (With sixteen query heads to a kv head there is no such column: the key is prepared by itself.)
    const bool rides = EDGE && FUSED && c.owns_new && c.kcol < 16 && (!fz.has_norm || fz.kw.p != nullptr);
    Frag knew[DS];
    uint16_t vnew[DT];
    if (EDGE && FUSED && c.owns_new) {   // the raw value of the new position (and the key, where it does not ride)
        const bf16* row = fz.qkv + (size_t)c.t0 * fz.stride;
        if (!rides) {
            const bf16* krow = row + fz.k_off + (size_t)c.kvh * D + 8 * g;
#pragma unroll
            for (int s = 0; s < DS; ++s) knew[s].u = *reinterpret_cast<const uint4*>(krow + 32 * s);
        }
        const uint16_t* vrow = reinterpret_cast<const uint16_t*>(row + fz.v_off + (size_t)c.kvh * D);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vnew[dt] = vrow[16 * dt + i];
    }

    bool first = true;
    for (int blk0 = BPW * c.z;; blk0 += BPW) {                 // one round, but for the last chunk of a short plan
        if (EDGE && !first) {
#pragma unroll
            for (int j = 0; j < BPW; ++j) {
                const int ia = (32 * (blk0 + j)) >> page_shift, ib = (32 * (blk0 + j) + 16) >> page_shift;
                pga[j] = ia < c.bt_width ? c.bt[ia] : -1;
                pgb[j] = ib < c.bt_width ? c.bt[ib] : -1;
            }
        }
        // ---- the keys of the chunk are asked for at once
        bool valid[BPW];
        int pa[BPW], pb[BPW];
        Frag kop[BPW][2][DS];
#pragma unroll
        for (int j = 0; j < BPW; ++j) {
            const int key0 = 32 * (blk0 + j);
            // a page that is not there (above the newest key, or given back by a window) holds only keys
            // that are masked below: the lanes that would read it read the block's other page instead
            pa[j] = (!EDGE || pga[j] >= 0) ? pga[j] : pgb[j];
            pb[j] = (!EDGE || pgb[j] >= 0) ? pgb[j] : pga[j];
            valid[j] = !EDGE || (pa[j] >= 0 && key0 <= pos && key0 + 31 >= lo);
            if (valid[j]) {
                const int pk = (PS16 && (i & 8)) ? pb[j] : pa[j];      // rows 8..15 of a tile are keys 16..31 of the block
                const bf16* kptr = kbase + (size_t)pk * page_elems + (size_t)((key0 + krow0) & slot_mask) * D;
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                    for (int s = 0; s < DS; ++s)
                        kop[j][tt][s].u = *reinterpret_cast<const uint4*>(kptr + (size_t)4 * tt * D + 32 * s);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (first && FUSED) {   // while the keys are on their way: the query (and the new key) are finished
            if (rides) {
                WeightPtr wl = fz.qw;
                if (i == c.kcol && fz.kw.p != nullptr) wl.p = fz.kw.p;
                prepare_head<DS>(qop, g, wl, fz.has_norm, fz.unit_offset, fz.eps, c.cs, i == c.kcol ? 1.f : c.sc_mul, D, qop);
#pragma unroll
                for (int s = 0; s < DS; ++s) {       // every lane of a group takes the key from the group's lane of column kcol
                    knew[s].u.x = __shfl(qop[s].u.x, 16 * g + c.kcol, MV_WAVE);
                    knew[s].u.y = __shfl(qop[s].u.y, 16 * g + c.kcol, MV_WAVE);
                    knew[s].u.z = __shfl(qop[s].u.z, 16 * g + c.kcol, MV_WAVE);
                    knew[s].u.w = __shfl(qop[s].u.w, 16 * g + c.kcol, MV_WAVE);
                }
            } else {
                prepare_head<DS>(qop, g, fz.qw, fz.has_norm, fz.unit_offset, fz.eps, c.cs, c.sc_mul, D, qop);
            }
            if (EDGE && c.owns_new) {
                if (!rides)
                    prepare_head<DS>(knew, g, fz.kw, fz.has_norm && fz.kw.p != nullptr, fz.unit_offset, fz.eps, c.cs, 1.f, D, knew);
                const int pidx = pos >> page_shift;
                const int page = pidx < c.bt_width ? c.bt[pidx] : -1;
                if (page >= 0) {
                    const int slot = pos & slot_mask;
                    if (i == 0) {
                        bf16* kdst = const_cast<bf16*>(c.k_pages) + (size_t)page * page_elems +
                                     ((size_t)c.kvh * page_size + slot) * D + 8 * g;
#pragma unroll
                        for (int s = 0; s < DS; ++s) *reinterpret_cast<uint4*>(kdst + 32 * s) = knew[s].u;
                    }
                    if (g == 0) {
                        uint16_t* vdst = reinterpret_cast<uint16_t*>(const_cast<bf16*>(c.v_pages)) + (size_t)page * page_elems +
                                         ((size_t)c.kvh * D + i) * page_size + slot;
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) vdst[(size_t)16 * dt * page_size] = vnew[dt];
                    }
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- the values of the chunk
        Frag vop[BPW][DT];
#pragma unroll
        for (int j = 0; j < BPW; ++j) {
            if (valid[j]) {
                const int pv = (PS16 && (g & 2)) ? pb[j] : pa[j];      // keys 8g .. 8g+7 of the block
                const bf16* vptr = vbase + (size_t)pv * page_elems + ((32 * (blk0 + j) + 8 * g) & slot_mask);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    vop[j][dt].u = *reinterpret_cast<const uint4*>(vptr + (size_t)16 * dt * page_size);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- scores^T of every block (in units of log2: the query carries scale * log2 e when fused)
        float sc[BPW][8];                                  // this lane's keys 8g .. 8g+7 of each block
#pragma unroll
        for (int j = 0; j < BPW; ++j) {
            if (valid[j]) {
                const int key0 = 32 * (blk0 + j);
                const bool new_here = EDGE && FUSED && c.owns_new && blk0 + j == c.b_hi;
                if (new_here) {                            // the newest key comes from the registers
                    const int rel = pos & 31;
                    const bool mine = i == (((rel >> 3) << 2) | (rel & 3));
                    const bool second = (rel >> 2) & 1;
#pragma unroll
                    for (int s = 0; s < DS; ++s) {
                        if (mine && !second) kop[j][0][s] = knew[s];
                        if (mine && second) kop[j][1][s] = knew[s];
                    }
                }
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    floatx4_t sacc = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < DS; ++s)
                        sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[j][tt][s].v, qop[s].v, sacc, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) sc[j][4 * tt + r] = FUSED ? sacc[r] : sacc[r] * c.sc_mul;
                }
                if (EDGE && (key0 + 31 > pos_read || key0 < lo)) {   // a block at an edge of the visible range
                    const int k0 = key0 + 8 * g;           // this lane's first key
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (k0 + e > pos || k0 + e < lo) sc[j][e] = -INFINITY;
                    // value slots above the newest key were never written, the newest key's own slot is not
                    // written yet where its value comes from the registers, and a page below a window may be
                    // another page's copy: everything outside [lo, pos_read] is cleared
                    uint32_t keep[4];
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const bool a0 = k0 + 2 * w >= lo && k0 + 2 * w <= pos_read;
                        const bool a1 = k0 + 2 * w + 1 >= lo && k0 + 2 * w + 1 <= pos_read;
                        keep[w] = (a0 ? 0x0000ffffu : 0u) | (a1 ? 0xffff0000u : 0u);
                    }
                    if (new_here && g == ((pos & 31) >> 3)) {
                        // (the cleared slot of the new position takes the value from the registers)
                        const int e = pos & 7;
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) {
                            const uint32_t v = (uint32_t)vnew[dt] << (16 * (e & 1));
                            vop[j][dt].u.x = (vop[j][dt].u.x & keep[0]) | ((e >> 1) == 0 ? v : 0u);
                            vop[j][dt].u.y = (vop[j][dt].u.y & keep[1]) | ((e >> 1) == 1 ? v : 0u);
                            vop[j][dt].u.z = (vop[j][dt].u.z & keep[2]) | ((e >> 1) == 2 ? v : 0u);
                            vop[j][dt].u.w = (vop[j][dt].u.w & keep[3]) | ((e >> 1) == 3 ? v : 0u);
                        }
                    } else {
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) {
                            vop[j][dt].u.x &= keep[0];
                            vop[j][dt].u.y &= keep[1];
                            vop[j][dt].u.z &= keep[2];
                            vop[j][dt].u.w &= keep[3];
                        }
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) sc[j][e] = -INFINITY;
            }
        }
        // ---- one maximum over the chunk, per column
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < BPW; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) mx = fmaxf(mx, sc[j][e]);
        mx = fmaxf(mx, __shfl_xor(mx, 16, MV_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, MV_WAVE));
        const float m_new = (!EDGE || first) ? mx : fmaxf(m_run, mx);
        const float m_safe = (EDGE && m_new == -INFINITY) ? 0.f : m_new;
        if (EDGE && !first) {
            const float corr = __builtin_amdgcn_exp2f(m_run - m_safe);
            l_run *= corr;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) acc_o[dt] *= corr;
        }
        m_run = m_new;
        // ---- out^T += V^T P^T, block by block
        float psum = 0.f;
#pragma unroll
        for (int j = 0; j < BPW; ++j) {
            if (!valid[j]) continue;
            float e[8];
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                e[x] = __builtin_amdgcn_exp2f(sc[j][x] - m_safe);
                psum += e[x];
            }
            Frag pop;
            pop.u.x = f32x2_to_bf16x2_bits(e[0], e[1]);
            pop.u.y = f32x2_to_bf16x2_bits(e[2], e[3]);
            pop.u.z = f32x2_to_bf16x2_bits(e[4], e[5]);
            pop.u.w = f32x2_to_bf16x2_bits(e[6], e[7]);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                acc_o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[j][dt].v, pop.v, acc_o[dt], 0, 0, 0);
        }
        l_run += psum;
        first = false;
        if (!EDGE || !last_chunk || 32 * (blk0 + BPW) > pos) break;
    }
}

template <int D, bool FUSED, int BPW, bool PS16>
__global__ void __launch_bounds__(64)
attention_decode_wave_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                             const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                             const int* __restrict__ block_table, int bt_width, int page_size_rt, int page_shift_rt,
                             const int* __restrict__ positions, const int* __restrict__ cu_seqlens, int n_seqs,
                             int H, int Hkv, float scale, int window, float* __restrict__ partials,
                             int nchunks, FusedInput fz) {
    constexpr int DS = D / 32;
    constexpr int DT = D / 16;
    const int page_shift = PS16 ? 4 : page_shift_rt;
    const int G = H / Hkv;
    const int seq = blockIdx.x, kvh = blockIdx.y, z = blockIdx.z;
    const int lane = threadIdx.x;
    const int i = lane & 15;
    const int g = lane >> 4;

    int t0;                                  // the sequence's one token
    if (FUSED) {
        t0 = seq;
        if (fz.token_seq[t0] < 0) return;
    } else {
        t0 = cu_seqlens[seq];
        if (cu_seqlens[seq + 1] - t0 <= 0) return;
    }
    const int* bt = block_table + (size_t)seq * bt_width;
    // the page ids of this chunk's blocks (two a block: keys 0..15 and 16..31 of it, the same page
    // where pages are larger): asked for before anything is known about the length
    int pga[BPW], pgb[BPW];
#pragma unroll
    for (int j = 0; j < BPW; ++j) {
        const int ia = (32 * (BPW * z + j)) >> page_shift, ib = (32 * (BPW * z + j) + 16) >> page_shift;
        pga[j] = ia < bt_width ? bt[ia] : -1;
        pgb[j] = ib < bt_width ? bt[ib] : -1;
    }
    const int pos = positions[t0];
    // the query head of this lane's column (lanes beyond the group copy its last head and store nothing;
    // fused with a cache write, the first column beyond the group holds the raw key of the new position,
    // which only the wave that meets the new position makes use of)
    const int head = kvh * G + (i < G ? i : G - 1);
    const int kcol = (FUSED && fz.store && G < 16) ? G : 16;
    Frag qop[DS];
    {
        const bf16* qrow = FUSED ? fz.qkv + (size_t)t0 * fz.stride + (i == kcol ? fz.k_off + (size_t)kvh * D
                                                                                  : fz.q_off + (size_t)head * D) + 8 * g
                                 : q + (size_t)t0 * q_stride + (size_t)head * D + 8 * g;
#pragma unroll
        for (int s = 0; s < DS; ++s) qop[s].u = *reinterpret_cast<const uint4*>(qrow + 32 * s);
    }
    if (pos < 0) return;
    const int lo = (window >= 0 && pos - window > 0) ? pos - window : 0;
    const int b_lo = lo >> 5, b_hi = pos >> 5;            // the 32-key blocks the sequence has
    const bool last_chunk = z == nchunks - 1;
    int b_stop = last_chunk ? b_hi + 1 : BPW * z + BPW;    // the last chunk takes what lies above it too
    if (b_stop > b_hi + 1) b_stop = b_hi + 1;
    if ((BPW * z > b_lo ? BPW * z : b_lo) >= b_stop) return;   // no key of the sequence in this chunk
    int z_lo = b_lo / BPW, z_hi = b_hi / BPW;
    if (z_lo > nchunks - 1) z_lo = nchunks - 1;
    if (z_hi > nchunks - 1) z_hi = nchunks - 1;
    const bool alone = z_lo == z_hi;                       // the sequence's only chunk: finish the row here

    WaveChunk c;
    c.k_pages = k_pages; c.v_pages = v_pages; c.bt = bt; c.bt_width = bt_width;
    c.page_size = page_size_rt; c.page_shift = page_shift_rt; c.Hkv = Hkv; c.kvh = kvh; c.z = z; c.nchunks = nchunks;
    c.pos = pos; c.lo = lo; c.b_hi = b_hi; c.i = i; c.g = g; c.sc_mul = scale * LOG2E; c.t0 = t0;
    c.owns_new = FUSED && fz.store && b_hi >= BPW * z && (last_chunk || b_hi < BPW * z + BPW);
    c.cs = (FUSED && fz.table != nullptr) ? fz.table + (size_t)pos * D : nullptr;
    c.kcol = kcol;

    float m_run = -INFINITY, l_run = 0.f;
    floatx4_t acc_o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc_o[dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    // a chunk wholly inside the visible range (and not the one that may have to go on above itself)
    const bool inside = 32 * BPW * z >= lo && 32 * BPW * (z + 1) - 1 < pos && !last_chunk;
    if (inside) wave_chunk<D, FUSED, BPW, PS16, false>(c, fz, qop, pga, pgb, m_run, l_run, acc_o);
    else wave_chunk<D, FUSED, BPW, PS16, true>(c, fz, qop, pga, pgb, m_run, l_run, acc_o);

    l_run += __shfl_xor(l_run, 16, MV_WAVE);
    l_run += __shfl_xor(l_run, 32, MV_WAVE);
    if (i >= G) return;
    if (alone) {
        bf16* orow = out + (size_t)t0 * out_stride + (size_t)head * D + 4 * g;
        const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            uint2 packed;
            packed.x = f32x2_to_bf16x2_bits(acc_o[dt][0] * inv, acc_o[dt][1] * inv);
            packed.y = f32x2_to_bf16x2_bits(acc_o[dt][2] * inv, acc_o[dt][3] * inv);
            *reinterpret_cast<uint2*>(orow + 16 * dt) = packed;
        }
        return;
    }
    float* prow = partials + (((size_t)t0 * H + head) * nchunks + z) * (D + 2);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        *reinterpret_cast<float4*>(prow + 16 * dt + 4 * g) = float4{acc_o[dt][0], acc_o[dt][1], acc_o[dt][2], acc_o[dt][3]};
    if (g == 0) {
        prow[D] = m_run;
        prow[D + 1] = l_run;
    }
}

// Adds up the chunks that attention_decode_wave_kernel left for a token: those between the chunk
// of the first key its query sees and the chunk of its own position. A token with a single chunk
// has its row already. One workgroup of D threads per (token, head).
template <int BPW>
__global__ void attention_merge_range_kernel(const float* __restrict__ partials, bf16* __restrict__ out, long out_stride,
                                             const int* __restrict__ token_seq, const int* __restrict__ positions,
                                             const int* __restrict__ cu_seqlens, int fused,
                                             int window, int H, int D, int nchunks) {
    __shared__ float sh_m[64], sh_l[64];
    const int head = blockIdx.y;
    const int d = threadIdx.x;            // blockDim.x == D
    // the sequence's token: row blockIdx.x of a step of one token a sequence (fused: padding rows
    // are rows too and get zeros), else the first token of sequence blockIdx.x, if it has one
    int tok = blockIdx.x;
    if (!fused) {
        tok = cu_seqlens[blockIdx.x];
        if (cu_seqlens[blockIdx.x + 1] - tok <= 0) return;
    }
    bf16* orow = out + (size_t)tok * out_stride + (size_t)head * D;
    if (token_seq[tok] < 0) {
        orow[d] = from_f<bf16>(0.f);
        return;
    }
    const int hi = positions[tok];
    const int lo = (window >= 0 && hi - window > 0) ? hi - window : 0;
    int z_lo = (lo / 32) / BPW, z_hi = (hi / 32) / BPW;
    if (z_lo > nchunks - 1) z_lo = nchunks - 1;
    if (z_hi > nchunks - 1) z_hi = nchunks - 1;
    if (z_lo == z_hi) return;             // the attention kernel finished this row itself
    const int nz = z_hi - z_lo + 1;
    const float* base = partials + (((size_t)tok * H + head) * nchunks + z_lo) * (D + 2);
    float m_run = -INFINITY, l_run = 0.f, a = 0.f;
    for (int z0 = 0; z0 < nz; z0 += 64) {             // batches of 64 chunks, merged as they come
        const int n = nz - z0 < 64 ? nz - z0 : 64;
        const float* bz = base + (size_t)z0 * (D + 2);
        float pre[8];                                  // asked for before the weights are known
#pragma unroll
        for (int j = 0; j < 8; ++j) pre[j] = j < n ? bz[(size_t)j * (D + 2) + d] : 0.f;
        __syncthreads();
        if (d < n) {
            sh_m[d] = bz[(size_t)d * (D + 2) + D];
            sh_l[d] = bz[(size_t)d * (D + 2) + D + 1];
        }
        __syncthreads();
        float mb = -INFINITY;
        for (int j = 0; j < n; ++j) mb = fmaxf(mb, sh_m[j]);
        const float m_new = fmaxf(m_run, mb);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = exp2f(m_run - m_safe);     // exp2(-inf) = 0
        a *= corr;
        l_run *= corr;
        m_run = m_new;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (j < n) {
                const float w = exp2f(sh_m[j] - m_safe);
                l_run += w * sh_l[j];
                a += w * pre[j];
            }
#pragma unroll 4
        for (int j = 8; j < n; ++j) {
            const float w = exp2f(sh_m[j] - m_safe);
            l_run += w * sh_l[j];
            a += w * bz[(size_t)j * (D + 2) + d];
        }
    }
    orow[d] = from_f<bf16>(l_run > 0.f ? a / l_run : 0.f);
}

// Merges the partial results of the key splits: out[token][head] = sum_z o_z 2^(m_z - m) / l.
#define AF_MAX_SPLITS 64
__global__ void attention_merge_kernel(const float* __restrict__ partials, bf16* __restrict__ out, long out_stride,
                                       const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens, int fused,
                                       int H, int D, int nsplit) {
    __shared__ float sh_m[AF_MAX_SPLITS], sh_w[AF_MAX_SPLITS];
    const int head = blockIdx.y;
    int tok = blockIdx.x;        // fused: row blockIdx.x of a step of one token a sequence; else the sequence's token
    if (!fused) {
        tok = cu_seqlens[blockIdx.x];
        if (cu_seqlens[blockIdx.x + 1] - tok <= 0) return;
    }
    bf16* orow = out + (size_t)tok * out_stride + (size_t)head * D;
    if (token_seq[tok] < 0) {
        for (int d = threadIdx.x; d < D; d += blockDim.x) orow[d] = from_f<bf16>(0.f);
        return;
    }
    const float* base = partials + ((size_t)tok * H + head) * nsplit * (D + 2);
    if ((int)threadIdx.x < nsplit) {
        sh_m[threadIdx.x] = base[(size_t)threadIdx.x * (D + 2) + D];
        sh_w[threadIdx.x] = base[(size_t)threadIdx.x * (D + 2) + D + 1];
    }
    __syncthreads();
    float m = -INFINITY;
    for (int z = 0; z < nsplit; ++z) m = fmaxf(m, sh_m[z]);
    float l = 0.f;
    for (int z = 0; z < nsplit; ++z)
        if (sh_m[z] != -INFINITY) l += exp2f(sh_m[z] - m) * sh_w[z];
    __syncthreads();
    if ((int)threadIdx.x < nsplit)
        sh_w[threadIdx.x] = (sh_m[threadIdx.x] == -INFINITY) ? 0.f : exp2f(sh_m[threadIdx.x] - m) / l;
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float a = 0.f;
#pragma unroll 8
        for (int z = 0; z < nsplit; ++z) a += sh_w[z] * base[(size_t)z * (D + 2) + d];
        orow[d] = from_f<bf16>(a);
    }
}

template <int D, int W, bool FUSED, int OCC>
static void launch_decode(dim3 grid, hipStream_t stream, const void* q, long q_stride, void* out, long out_stride,
                          const void* k_pages, const void* v_pages, const int* block_table, int bt_width,
                          int page_size, const int* positions, const int* cu_seqlens, int n_seqs, int H, int Hkv,
                          float scale, int window, float* partials, int nsplit, const FusedInput& fz) {
    hipLaunchKernelGGL((attention_decode_kernel<D, W, FUSED, OCC>), grid, dim3(64 * W), 0, stream, (const bf16*)q, q_stride,
                       (bf16*)out, out_stride, (const bf16*)k_pages, (const bf16*)v_pages, block_table, bt_width,
                       page_size, positions, cu_seqlens, n_seqs, H, Hkv, scale, window, partials, nsplit, fz);
}

static int check_common(const char* what, long q_stride, long out_stride, int page_size, int bt_width, int H, int Hkv,
                        int D) {
    MV_REQUIRE(H > 0 && Hkv > 0 && H % Hkv == 0, "%s: %d heads are not a multiple of %d kv heads", what, H, Hkv);
    MV_REQUIRE(D == 64 || D == 128, "%s: head_dim %d is not served by the MFMA kernel (64 or 128)", what, D);
    MV_REQUIRE(page_size > 0 && page_size % 16 == 0, "%s: page size %d must be a multiple of 16", what, page_size);
    MV_REQUIRE(bt_width > 0, "%s: empty block table", what);
    MV_REQUIRE(q_stride >= (long)H * D && q_stride % 8 == 0 && out_stride >= (long)H * D && out_stride % 4 == 0,
               "%s: row strides %ld / %ld do not fit %d heads of %d", what, q_stride, out_stride, H, D);
    MV_REQUIRE(Hkv <= 65535, "%s: too many kv heads", what);
    return 0;
}

static int decode_common(bool fused, const FusedInput& fz, const void* q, long q_stride, void* out, long out_stride,
                         const void* k_pages, const void* v_pages, const int* block_table, int bt_width,
                         int page_size, const int* positions, const int* cu_seqlens, int n_seqs, int H, int Hkv, int D,
                         float scale, int window, float* partials, int nsplit, int waves, int chunk_keys,
                         const int* token_seq, hipStream_t stream) {
    MV_REQUIRE(H / Hkv <= 16, "attention_decode: %d query heads per kv head exceed 16", H / Hkv);
    if (chunk_keys != 0) {
        // one wave per chunk of chunk_keys keys; nsplit chunks are planned for every sequence
        MV_REQUIRE(chunk_keys == 64 || chunk_keys == 128, "attention_decode: chunks of %d keys (64 or 128)", chunk_keys);
        MV_REQUIRE(nsplit >= 1 && nsplit <= 65535 && (nsplit == 1 || partials != nullptr),
                   "attention_decode: bad chunk count %d or missing work area", nsplit);
        MV_REQUIRE((page_size & (page_size - 1)) == 0, "attention_decode: the one-wave kernel takes pages of a power of "
                   "two slots, got %d", page_size);
        if (n_seqs <= 0) return 0;
        int page_shift = 0;
        while ((1 << page_shift) < page_size) ++page_shift;
        dim3 grid(n_seqs, Hkv, nsplit);
#define AF_WAVE(DD, FF, BB)                                                                                          \
        do {                                                                                                          \
            if (page_size == 16)                                                                                      \
                hipLaunchKernelGGL((attention_decode_wave_kernel<DD, FF, BB, true>), grid, dim3(64), 0, stream,        \
                                   (const bf16*)q, q_stride, (bf16*)out, out_stride, (const bf16*)k_pages,            \
                                   (const bf16*)v_pages, block_table, bt_width, page_size, page_shift, positions,     \
                                   cu_seqlens, n_seqs, H, Hkv, scale, window, partials, nsplit, fz);                  \
            else                                                                                                      \
                hipLaunchKernelGGL((attention_decode_wave_kernel<DD, FF, BB, false>), grid, dim3(64), 0, stream,       \
                                   (const bf16*)q, q_stride, (bf16*)out, out_stride, (const bf16*)k_pages,            \
                                   (const bf16*)v_pages, block_table, bt_width, page_size, page_shift, positions,     \
                                   cu_seqlens, n_seqs, H, Hkv, scale, window, partials, nsplit, fz);                  \
        } while (0)
        if (D == 128 && fused && chunk_keys == 64) AF_WAVE(128, true, 2);
        else if (D == 128 && fused) AF_WAVE(128, true, 4);
        else if (D == 128 && chunk_keys == 64) AF_WAVE(128, false, 2);
        else if (D == 128) AF_WAVE(128, false, 4);
        else if (fused && chunk_keys == 64) AF_WAVE(64, true, 2);
        else if (fused) AF_WAVE(64, true, 4);
        else if (chunk_keys == 64) AF_WAVE(64, false, 2);
        else AF_WAVE(64, false, 4);
#undef AF_WAVE
        if (int rc = mv_check_launch("attention_decode (one wave a chunk)")) return rc;
        if (nsplit > 1) {
            if (chunk_keys == 64)
                hipLaunchKernelGGL(attention_merge_range_kernel<2>, dim3(n_seqs, H), dim3(D), 0, stream, partials, (bf16*)out,
                                   out_stride, token_seq, positions, cu_seqlens, fused ? 1 : 0, window, H, D, nsplit);
            else
                hipLaunchKernelGGL(attention_merge_range_kernel<4>, dim3(n_seqs, H), dim3(D), 0, stream, partials, (bf16*)out,
                                   out_stride, token_seq, positions, cu_seqlens, fused ? 1 : 0, window, H, D, nsplit);
            return mv_check_launch("attention_merge (chunks)");
        }
        return 0;
    }
    MV_REQUIRE(nsplit >= 1 && nsplit <= AF_MAX_SPLITS && (nsplit == 1 || partials != nullptr),
               "attention_decode: bad split count %d or missing work area", nsplit);
    MV_REQUIRE(waves == 4 || waves == 8, "attention_decode: %d waves per workgroup (4 or 8)", waves);
    if (n_seqs <= 0) return 0;
    dim3 grid(n_seqs, Hkv, nsplit);
    float* part = nsplit > 1 ? partials : nullptr;
    // With more workgroups than compute units, two of them share a unit (the kernel is then held to
    // 256 registers a lane, which costs it three spilled ones at head size 128): one's set-up and
    // tail overlap the other's stream of keys, 4-6 % on a step of 64 to 256 sequences. A grid that
    // fits the chip at once keeps all registers.
    const int occ = (long)n_seqs * Hkv * nsplit > 256 ? 2 : 1;
#define AF_LAUNCH(DD, WW, FF)                                                                                     \
    do {                                                                                                          \
        if constexpr (WW == 4) {                                                                                  \
            if (occ == 2) {                                                                                       \
                launch_decode<DD, WW, FF, 2>(grid, stream, q, q_stride, out, out_stride, k_pages, v_pages,        \
                                             block_table, bt_width, page_size, positions, cu_seqlens, n_seqs, H,  \
                                             Hkv, scale, window, part, nsplit, fz);                               \
                break;                                                                                            \
            }                                                                                                     \
        }                                                                                                         \
        launch_decode<DD, WW, FF, 1>(grid, stream, q, q_stride, out, out_stride, k_pages, v_pages, block_table,   \
                                     bt_width, page_size, positions, cu_seqlens, n_seqs, H, Hkv, scale, window,   \
                                     part, nsplit, fz);                                                           \
    } while (0)
    if (fused) {
        MV_REQUIRE(waves == 4, "attention_decode_fused: %d waves per workgroup (4 only)", waves);
        if (D == 128) AF_LAUNCH(128, 4, true);
        else AF_LAUNCH(64, 4, true);
    } else {
        if (D == 128 && waves == 8) AF_LAUNCH(128, 8, false);
        else if (D == 128) AF_LAUNCH(128, 4, false);
        else if (waves == 8) AF_LAUNCH(64, 8, false);
        else AF_LAUNCH(64, 4, false);
    }
#undef AF_LAUNCH
    if (int rc = mv_check_launch("attention_decode")) return rc;
    if (nsplit > 1) {
        hipLaunchKernelGGL(attention_merge_kernel, dim3(n_seqs, H), dim3(D >= 128 ? 128 : 64), 0, stream, partials,
                           (bf16*)out, out_stride, token_seq, cu_seqlens, fused ? 1 : 0, H, D, nsplit);
        return mv_check_launch("attention_merge");
    }
    return 0;
}

// Decode steps: every sequence brings one token. grid = (sequences, kv heads, nsplit); `waves` (4
// or 8) per workgroup. partials: float [n_seqs * H * nsplit * (D + 2)], needed when nsplit > 1.
// chunk_keys != 0 (64 or 128) selects the one-wave variant for small grids instead: a wave per
// chunk of that many keys, nsplit chunks planned per sequence (nsplit * chunk_keys should cover the
// longest context; the last chunk takes what lies above), `waves` is ignored; `positions` must then
// hold, for a step of one token a sequence, token t's position at index t.
extern "C" int mv_attention_decode(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
                                   const void* v_pages, const int* block_table, int bt_width, int page_size,
                                   const int* positions, const int* cu_seqlens, int n_seqs, int H, int Hkv, int D,
                                   float scale, int window, float* partials, int nsplit, int waves, int chunk_keys,
                                   const int* token_seq, hipStream_t stream) {
    if (int rc = check_common("attention_decode", q_stride, out_stride, page_size, bt_width, H, Hkv, D)) return rc;
    return decode_common(false, FusedInput{}, q, q_stride, out, out_stride, k_pages, v_pages, block_table, bt_width,
                         page_size, positions, cu_seqlens, n_seqs, H, Hkv, D, scale, window, partials, nsplit, waves,
                         chunk_keys, token_seq, stream);
}

// The same for a decode step whose queries, keys and values are still the raw rows of the
// [q | k | v] product (one token a sequence; row t of qkv belongs to sequence t): per-head RMSNorm
// (q_weight / k_weight, or null for none) and rotation by the table row of the position
// (half-split pairs over the whole head, or null for none) happen on the way into the kernel;
// with store_kv the new key and value are written to their page slot as well.
extern "C" int mv_attention_decode_fused(const void* qkv, long qkv_stride, int q_off, int k_off, int v_off, void* out,
                                         long out_stride, void* k_pages, void* v_pages, const int* block_table,
                                         int bt_width, int page_size, const int* positions, const int* cu_seqlens,
                                         int n_seqs, int H, int Hkv, int D, float scale, int window,
                                         const void* q_weight, const void* k_weight, int weight_dtype, float eps,
                                         int unit_offset, const float* table, int store_kv, float* partials,
                                         int nsplit, int waves, int chunk_keys, const int* token_seq,
                                         hipStream_t stream) {
    if (int rc = check_common("attention_decode_fused", qkv_stride, out_stride, page_size, bt_width, H, Hkv, D))
        return rc;
    MV_REQUIRE(qkv != nullptr && ((uintptr_t)qkv % 16) == 0 && q_off % 8 == 0 && k_off % 8 == 0 && v_off >= 0,
               "attention_decode_fused: the qkv rows must be 16-byte aligned (offsets %d / %d / %d)", q_off, k_off, v_off);
    MV_REQUIRE(qkv_stride >= (long)q_off + (long)H * D, "attention_decode_fused: row stride %ld too small", qkv_stride);
    MV_REQUIRE(token_seq != nullptr, "attention_decode_fused: token_seq is missing");
    MV_REQUIRE(!store_kv || qkv_stride >= (long)(k_off > v_off ? k_off : v_off) + (long)Hkv * D,
               "attention_decode_fused: row stride %ld does not hold the key and value heads", qkv_stride);
    const int has_norm = q_weight != nullptr;
    MV_REQUIRE(!has_norm || ((k_weight != nullptr || !store_kv) && eps > 0.f && mv_valid_dtype(weight_dtype) &&
                             ((uintptr_t)q_weight % 16) == 0 && ((uintptr_t)k_weight % 16) == 0),
               "attention_decode_fused: bad norm weights (missing, unknown type or not 16-byte aligned) or eps");
    MV_REQUIRE(table == nullptr || ((uintptr_t)table % 16) == 0, "attention_decode_fused: the table is not 16-byte aligned");
    FusedInput fz{(const bf16*)qkv, qkv_stride, q_off, k_off, v_off, WeightPtr{q_weight, weight_dtype},
                  WeightPtr{k_weight, weight_dtype}, has_norm, eps, unit_offset, table, store_kv ? 1 : 0, token_seq};
    return decode_common(true, fz, nullptr, 0, out, out_stride, k_pages, v_pages, block_table, bt_width, page_size,
                         positions, cu_seqlens, n_seqs, H, Hkv, D, scale, window, partials, nsplit, waves, chunk_keys,
                         token_seq, stream);
}
