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
// the first: the rows of the two score tiles of a 32-key block interleave in groups of four keys
// (row 4g+r of tile t is key 8g+4t+r, g = l/16), so lane group g ends up with the keys 8g..8g+7,
// eight neighbours of a value row: one 16-byte load per value operand, and nothing is shuffled.
// Each column keeps its own running maximum and sum (online softmax, base 2).
//
// The W waves of a workgroup (4 or 8) take the 32-key blocks in turn, each with the K operands
// of its next block already in flight, and their partial results are merged through LDS. With
// nsplit > 1 several workgroups split a sequence's keys further; the one that finishes last adds
// their partial results up.
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
    const float* rows;      // [tokens, D] = the table rows of the step's positions, gathered once a step, or null
    int store;
    const int* token_seq;   // rows that belong to no sequence (< 0) are left alone
};

// A head's raw elements are prepared by half a wave, E = D / 32 elements a lane (d = E j + e for
// lane j of the half): RMSNorm over the head (weights w, already with their unit offset), rotation
// by the table row of the position (c and sn: this lane's cosines and sines; pairs d, d + D/2 are
// lane j and lane j ^ 16), rounding to the operand type. Every lane of the half wave must call it
// (the lanes exchange values).
template <int D>
__device__ __forceinline__ void prepare_head_spread(const uint16_t* raw, int j, bool has_norm, const float* w, float eps,
                                                    bool rotate, const float* c, const float* sn, uint16_t* dst) {
    constexpr int E = D / 32;
    float x[E];
#pragma unroll
    for (int e = 0; e < E; ++e) x[e] = __uint_as_float((uint32_t)raw[e] << 16);
    if (has_norm) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) ss += x[e] * x[e];
#pragma unroll
        for (int o = 1; o < 32; o <<= 1) ss += __shfl_xor(ss, o, MV_WAVE);
        const float rinv = rsqrtf(ss / (float)D + eps);
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = x[e] * rinv * w[e];
    }
    if (rotate) {
        const float sign = (j & 16) ? 1.f : -1.f;          // the upper half of the head adds, the lower subtracts
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float other = __shfl_xor(x[e], 16, MV_WAVE);
            x[e] = x[e] * c[e] + sign * other * sn[e];
        }
    }
#pragma unroll
    for (int e = 0; e < E; ++e) dst[e] = f32_to_bf16_bits(x[e]);
}

#define AF_MAX_SPLITS 64

// OCC workgroups are to share a compute unit (W / 4 waves of each on every SIMD): the register budget.
// OCC 2 is for grids larger than the chip, which do not split the keys (nsplit 1): that variant
// leaves the code of the splits out and keeps its registers for the stream of keys.
//
// The 32-key blocks are dealt out in turn: block b belongs to wave b % W of split (b / W) % nsplit,
// so which blocks a workgroup may meet does not depend on the sequence's length and the page ids
// can be asked for together with the position. A split whose blocks all lie outside the sequence's
// keys ends at once; the others leave their partial results and count themselves in, and the one
// that counts last adds the partial results up (see the end of the kernel).
template <int D, int W, bool FUSED, int OCC>
__global__ void __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(OCC * W / 4, OCC * W / 4)))
attention_decode_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                      const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                      const int* __restrict__ block_table, int bt_width, int page_size,
                      const int* __restrict__ positions, const int* __restrict__ cu_seqlens, int n_seqs,
                      int H, int Hkv, float scale, int window, float* __restrict__ partials,
                      int* __restrict__ counters, int nsplit, int max_pages, FusedInput fz) {
    constexpr int DS = D / 32;
    constexpr int DT = D / 16;
    constexpr int NT = 1;      // column tiles of a wave (the group's heads fit one tile)
    constexpr int COLS = 16;   // columns of a workgroup
    constexpr int E = D / 32;  // elements of a head that a lane prepares (FUSED)
    constexpr int HW = 2 * W;  // half waves of a workgroup
    constexpr int ROUNDS = (COLS + 1 + HW - 1) / HW;   // up to 16 query heads and the new key
    if (OCC != 1) nsplit = 1;
    const int G = H / Hkv;
    const int kvh = blockIdx.y;
    const int split = blockIdx.z;
    const int wave = threadIdx.x / MV_WAVE;
    const int lane = threadIdx.x % MV_WAVE;
    const int i = lane % 16;
    const int g = lane / 16;
    const int tpu = COLS / G;  // tokens of a unit (the host made sure it is >= 1)

    __shared__ int sh_unit[3];
    __shared__ int sh_pages[AF_MAX_CACHED_PAGES];
    __shared__ __attribute__((aligned(16))) uint16_t sh_heads[FUSED ? COLS + 1 : 1][FUSED ? D : 8];
    int seq, t0, nt;
    int pos0 = -1;
    union RawHead {
        uint16_t s[E];
        uint32_t u[E / 2];
    } raw[ROUNDS];
    const int hw = threadIdx.x / 32, hj = threadIdx.x % 32;   // (FUSED) this lane's half wave and place in it
    float head_w[ROUNDS][E], rot_c[E], rot_s[E];
    int first_a0 = -1, first_a1 = -1, first_b0 = -1, first_b1 = -1;   // page ids of the halves of the wave's first two blocks
    if (FUSED) {
        // a decode step: row t of the step is the one token of sequence t (or padding). Everything
        // that does not depend on the position is asked for before the position is looked at.
        seq = blockIdx.x;
        t0 = seq;
        const int tseq = fz.token_seq[t0];
        pos0 = positions[t0];
        const bf16* row = fz.qkv + (size_t)t0 * fz.stride;
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            if (r * HW > G) break;                 // no head left for any half wave (the same for the whole workgroup)
            const int h = hw + r * HW;
            const bf16* src = h < G ? row + fz.q_off + (size_t)(kvh * G + h) * D + E * hj
                                    : (h == G && fz.store ? row + fz.k_off + (size_t)kvh * D + E * hj : nullptr);
#pragma unroll
            for (int e = 0; e < E / 2; ++e)
                raw[r].u[e] = src != nullptr ? reinterpret_cast<const uint32_t*>(src)[e] : 0u;
            if (fz.has_norm && src != nullptr) {
                if (h < G) fz.qw.at_few<E>(E * hj, head_w[r]);
                else fz.kw.at_few<E>(E * hj, head_w[r]);
                if (fz.unit_offset) {
#pragma unroll
                    for (int e = 0; e < E; ++e) head_w[r][e] += 1.f;
                }
            }
        }
        if (fz.rows != nullptr) {   // the step's rotation rows: no need to know the position first
            const float* cs = fz.rows + (size_t)t0 * D + (E * hj) % (D / 2);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                rot_c[e] = cs[e];
                rot_s[e] = cs[D / 2 + e];
            }
        }
        if (window < 0) {
            // Without a window a wave's blocks are split * W + wave, + nsplit * W, ...: whatever the
            // sequence's length. The page ids of its first two blocks come straight from the block
            // table (uniform over the wave: scalar loads), so that their keys and values can be asked
            // for as soon as the position is known; the ids of all later blocks go to LDS meanwhile.
            const int* bt0 = block_table + (size_t)seq * bt_width;
            int n = bt_width < max_pages ? bt_width : max_pages;
            const int wv = __builtin_amdgcn_readfirstlane(wave);
            auto lookup = [&](int key0) -> int {     // (any page of the table, also beyond the planned context)
                const int pidx = key0 / page_size;
                return pidx < bt_width ? bt0[pidx] : -1;
            };
            const int key_a = 32 * (split * W + wv), key_b = key_a + 32 * nsplit * W;
            first_a0 = lookup(key_a);
            first_a1 = lookup(key_a + 16);
            first_b0 = lookup(key_b);
            first_b1 = lookup(key_b + 16);
            if (n > AF_MAX_CACHED_PAGES) n = AF_MAX_CACHED_PAGES;
            for (int p = threadIdx.x; p < n; p += blockDim.x) sh_pages[p] = bt0[p];
        }
        nt = tseq >= 0 ? 1 : 0;
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
        col_pos[ct] = col_ok[ct] ? (FUSED ? pos0 : positions[col_tok[ct]]) : -1;   // FUSED: one token, one position
        col_lo[ct] = (window >= 0 && col_pos[ct] - window > 0) ? col_pos[ct] - window : 0;
        if (col_ok[ct]) {
            hi_w = col_pos[ct] > hi_w ? col_pos[ct] : hi_w;
            lo_w = col_lo[ct] < lo_w ? col_lo[ct] : lo_w;
        }
        if (!FUSED) {   // finished query rows
            const bf16* qrow = q + (size_t)col_tok[ct] * q_stride + (size_t)col_head[ct] * D + 8 * g;
#pragma unroll
            for (int s = 0; s < DS; ++s)
                qop[ct][s].u = col_ok[ct] ? *reinterpret_cast<const uint4*>(qrow + 32 * s) : uint4{0u, 0u, 0u, 0u};
        }
    }
    if (FUSED) {   // known without asking the other lanes
        hi_w = pos0;
        lo_w = (window >= 0 && hi_w - window > 0) ? hi_w - window : 0;
        if (fz.table != nullptr && fz.rows == nullptr) {   // asked for before the keys, so that preparing the heads does not wait for keys
            const float* cs = fz.table + (size_t)(hi_w >= 0 ? hi_w : 0) * D + (E * hj) % (D / 2);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                rot_c[e] = cs[e];
                rot_s[e] = cs[D / 2 + e];
            }
        }
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

    // ---- the 32-key blocks of this wave: b_begin, b_begin + b_step, ... below b_end
    const int b0 = hi_w >= 0 ? lo_w / 32 : 0, b1 = hi_w >= 0 ? hi_w / 32 : -1;
    const int b_step = nsplit * W;
    const int b_end = b1 + 1;
    int b_begin = split * W + wave;
    if (b_begin < b0) b_begin += ((b0 - b_begin + b_step - 1) / b_step) * b_step;
    // the splits that hold a block of this sequence: n_active of them, from split z_first on in turn
    const int g0 = b0 / W, g1 = b1 / W;
    const int z_first = g0 % nsplit;
    const int n_active = hi_w < 0 ? 0 : (g1 - g0 + 1 < nsplit ? g1 - g0 + 1 : nsplit);
    if (nsplit > 1 && (split - z_first + nsplit) % nsplit >= n_active) return;
    const float sc_mul = scale * LOG2E;

    // (FUSED) the wave that meets the newest position among its keys takes the new key and value
    // from the step's rows, not from the page
    const int b_new = b1;
    const bool owns_new = FUSED && fz.store && b_new >= b_begin && b_new < b_end && (b_new - b_begin) % b_step == 0;
    const bool wg_owns_new = FUSED && fz.store && b_new >= 0 && (b_new / W) % nsplit == split;
    Frag knew[DS];
    uint16_t vnew[DT];
    if (FUSED) {
#pragma unroll
        for (int s = 0; s < DS; ++s) knew[s].u = uint4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vnew[dt] = 0;
        if (owns_new) {
            const uint16_t* vrow = reinterpret_cast<const uint16_t*>(fz.qkv + (size_t)t0 * fz.stride + fz.v_off + (size_t)kvh * D);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vnew[dt] = vrow[16 * dt + i];
        }
    }

    // The page ids are in LDS before the first block is asked for (one round trip instead of one
    // per block): all of the planned context when no window cuts the keys (asked for above), else
    // those from the window's first key on; pages beyond what LDS holds are looked up in place.
    // K and V operands are fetched one block ahead of their use.
    int p_first = 0, n_cached;
    if (FUSED && window < 0) {
        n_cached = bt_width < max_pages ? bt_width : max_pages;
        if (n_cached > AF_MAX_CACHED_PAGES) n_cached = AF_MAX_CACHED_PAGES;
    } else {
        p_first = (32 * b0) / page_size;
        const int p_last = hi_w >= 0 ? hi_w / page_size : -1;
        n_cached = p_last - p_first + 1;
        if (n_cached > AF_MAX_CACHED_PAGES) n_cached = AF_MAX_CACHED_PAGES;
        for (int r = threadIdx.x; r < n_cached; r += blockDim.x)
            sh_pages[r] = p_first + r < bt_width ? bt[p_first + r] : -1;
        __syncthreads();
    }
    // (FUSED without a window: the ids in LDS are first used behind the barrier of the head preparation)
    auto page_of = [&](int pidx) -> int {
        if (pidx >= bt_width) return -1;
        const int rel = pidx - p_first;
        return rel < n_cached ? sh_pages[rel] : bt[pidx];
    };
    // Which keys a lane's operand slots hold: row rho of score tile t is key 8 (rho / 4) + 4 t + rho % 4 of
    // the block, so that after the first product lane group g holds the probabilities of keys 8 g ..
    // 8 g + 7 (slot 4 t + r is key 8 g + 4 t + r) — eight neighbours in a value row, one 16-byte load
    // per operand, and still nothing is shuffled between the products. The block's two halves of 16
    // keys may lie in different pages: a key row of either tile lies in half rho / 8, a lane group's
    // values in half g / 2.
    struct Operands {
        int page[2];   // of the block's halves
        Frag k[2][DS];
        Frag v[DT];
    };
    const int k_half = i / 8, v_half = g / 2;
    // given: the caller has the page ids of the block's halves already (pg0, pg1); else they are looked up
    auto fetch = [&](int b, Operands& op, bool given, int pg0, int pg1) {
        int slot0[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int key0 = 32 * b + 16 * h;
            const int pidx = key0 / page_size;
            op.page[h] = (b < b_end && key0 <= hi_w) ? (given ? (h ? pg1 : pg0) : page_of(pidx)) : -1;
            slot0[h] = key0 - pidx * page_size;
        }
        const int kpage = k_half ? op.page[1] : op.page[0];
        const int vpage = v_half ? op.page[1] : op.page[0];
        if (kpage >= 0) {
            const size_t head = (size_t)kpage * Hkv + kvh;
            const int slot = (k_half ? slot0[1] : slot0[0]) + 8 * ((i / 4) % 2) + i % 4;   // of tile 0; tile 1 four on
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const bf16* kptr = k_pages + ((head * page_size + slot + 4 * t) * D + 8 * g);
#pragma unroll
                for (int s = 0; s < DS; ++s) op.k[t][s].u = *reinterpret_cast<const uint4*>(kptr + 32 * s);
            }
        } else {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int s = 0; s < DS; ++s) op.k[t][s].u = uint4{0u, 0u, 0u, 0u};
        }
        if (vpage >= 0) {
            const size_t head = (size_t)vpage * Hkv + kvh;
            const bf16* vptr = v_pages + (head * D + i) * page_size + (v_half ? slot0[1] : slot0[0]) + 8 * (g % 2);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) op.v[dt].u = *reinterpret_cast<const uint4*>(vptr + (size_t)16 * dt * page_size);
        } else {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) op.v[dt].u = uint4{0u, 0u, 0u, 0u};
        }
    };
    auto compute = [&](int b, Operands& op) {
        const int base = 32 * b;
        if (FUSED && owns_new && b == b_new) {   // the newest key and value come from the registers
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                if (base + 8 * (i / 4) + 4 * t + i % 4 == hi_w) {
#pragma unroll
                    for (int s = 0; s < DS; ++s) op.k[t][s] = knew[s];
                }
            }
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (base + 8 * g + e == hi_w) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) op.v[dt].s[e] = vnew[dt];
                }
        }
        const bool v_live = (v_half ? op.page[1] : op.page[0]) >= 0;     // the half of this lane's probabilities
        // scores^T for two tiles of 16 keys
        float p[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            floatx4_t sacc = floatx4_t{0.f, 0.f, 0.f, 0.f};
            if (op.page[0] >= 0 || op.page[1] >= 0) {
#pragma unroll
                for (int s = 0; s < DS; ++s)
                    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(op.k[t][s].v, qop[0][s].v, sacc, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = base + 8 * g + 4 * t + r;
                const bool ok = v_live && col_ok[0] && key <= col_pos[0] && key >= col_lo[0];
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
                for (int e = 0; e < 8; ++e)
                    if (base + 8 * g + e > hi_w) op.v[dt].s[e] = 0;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            acc_o[0][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(op.v[dt].v, pop.v, acc_o[0][dt], 0, 0, 0);
    };

    // two blocks are on their way before anything else is done with the position
    Operands oa, ob;
    const bool direct = FUSED && window < 0;
    fetch(b_begin, oa, direct, first_a0, first_a1);
    if (b_begin + b_step < b_end) fetch(b_begin + b_step, ob, direct, first_b0, first_b1);
    if (FUSED) {
        // while those loads are in flight: the group's query heads (and the new key, in the workgroup
        // that will meet it) are prepared by half a wave each and handed round through LDS
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            if (r * HW > G) break;
            const int h = hw + r * HW;
            if (h < G || (h == G && wg_owns_new))          // uniform over the half wave, and the exchange stays inside it
                prepare_head_spread<D>(raw[r].s, hj, fz.has_norm != 0, head_w[r], fz.eps,
                                       fz.table != nullptr || fz.rows != nullptr, rot_c, rot_s, &sh_heads[h][E * hj]);
        }
        __syncthreads();
#pragma unroll
        for (int s = 0; s < DS; ++s)
            qop[0][s].u = col_ok[0] ? *reinterpret_cast<const uint4*>(&sh_heads[i][32 * s + 8 * g]) : uint4{0u, 0u, 0u, 0u};
        if (owns_new) {
#pragma unroll
            for (int s = 0; s < DS; ++s) knew[s].u = *reinterpret_cast<const uint4*>(&sh_heads[G][32 * s + 8 * g]);
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
        compute(b, oa);
        if (b + b_step >= b_end) break;
        // Beyond the last block a fetch loads nothing and clears the registers. A wave of a grid that
        // fits the chip has two or three blocks and skips that; in the long loops of crowded grids the
        // straight line is faster (the branch costs the compiler its exact wait counts).
        if (OCC != 1 || b + 2 * b_step < b_end) fetch(b + 2 * b_step, oa, false, -1, -1);
        compute(b + b_step, ob);
        if (OCC != 1 || b + 3 * b_step < b_end) fetch(b + 3 * b_step, ob, false, -1, -1);
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
                if (OCC != 1 || nsplit == 1) {
                    const float inv = 1.f / l_fin;
                    uint2 packed;
                    packed.x = f32x2_to_bf16x2_bits(o[0] * inv, o[1] * inv);
                    packed.y = f32x2_to_bf16x2_bits(o[2] * inv, o[3] * inv);
                    *reinterpret_cast<uint2*>(orow + d0) = packed;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) __hip_atomic_store(prow + d0 + r, o[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
    }
    if (OCC != 1 || nsplit == 1) return;
    if (wave == 0 && g == 0 && col_ok[0]) {
        __hip_atomic_store(prow + D, m_fin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(prow + D + 1, l_fin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // ---- the workgroup that finishes last among the splits of this (sequence, kv head) adds their
    // partial results up. The splits run on compute units that share no cache, so the rows above
    // were stored at device scope (written through to memory) and are read back the same way; no
    // cache is flushed or invalidated, which costs more than a second kernel would (measured). A
    // wave's stores have arrived when its counter of outstanding memory operations is at zero;
    // after the barrier that holds for the whole workgroup, and only then it counts itself in. The
    // workgroup that counts last therefore finds every row. It also puts the counter back to zero:
    // the next launch finds it clean, and no memset is needed between launches.
    __shared__ int sh_last;
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {
        int* counter = counters + (size_t)blockIdx.x * Hkv + kvh;
        const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sh_last = before == n_active - 1;
        if (sh_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!sh_last) return;
#define AF_PEEK(p) __hip_atomic_load((p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
    // each thread adds up one element of one column; the rows of up to sixteen splits, with their
    // maxima and sums, are in flight at once (one round trip for the usual split counts)
    constexpr int MB = 16;
    for (int idx = threadIdx.x; idx < ncols * D; idx += blockDim.x) {
        const int col = idx / D, d = idx - col * D;
        const int tok = t0 + col / G, head = kvh * G + col % G;
        const float* base = partials + ((size_t)tok * H + head) * nsplit * (D + 2);
        float m = -INFINITY, l = 0.f, a = 0.f;
        for (int j0 = 0; j0 < n_active; j0 += MB) {
            float v[MB], mz[MB], lz[MB];
#pragma unroll
            for (int u = 0; u < MB; ++u) {
                int z = z_first + j0 + u;
                if (z >= nsplit) z -= nsplit;
                const float* row = base + (size_t)z * (D + 2);
                const bool live = j0 + u < n_active;
                v[u] = live ? AF_PEEK(row + d) : 0.f;
                mz[u] = live ? AF_PEEK(row + D) : -INFINITY;
                lz[u] = live ? AF_PEEK(row + D + 1) : 0.f;
            }
            float mb = m;
#pragma unroll
            for (int u = 0; u < MB; ++u) mb = fmaxf(mb, mz[u]);
            const float m_safe = (mb == -INFINITY) ? 0.f : mb;
            const float corr = exp2f(m - m_safe);     // exp2(-inf) = 0
            l *= corr;
            a *= corr;
            m = mb;
#pragma unroll
            for (int u = 0; u < MB; ++u) {
                const float w = exp2f(mz[u] - m_safe);
                l += w * lz[u];
                a += w * v[u];
            }
        }
        out[(size_t)tok * out_stride + (size_t)head * D + d] = from_f<bf16>(l > 0.f ? a / l : 0.f);
    }
#undef AF_PEEK
}

template <int D, int W, bool FUSED, int OCC>
static void launch_decode(dim3 grid, hipStream_t stream, const void* q, long q_stride, void* out, long out_stride,
                          const void* k_pages, const void* v_pages, const int* block_table, int bt_width,
                          int page_size, const int* positions, const int* cu_seqlens, int n_seqs, int H, int Hkv,
                          float scale, int window, float* partials, int* counters, int nsplit, int max_pages,
                          const FusedInput& fz) {
    hipLaunchKernelGGL((attention_decode_kernel<D, W, FUSED, OCC>), grid, dim3(64 * W), 0, stream, (const bf16*)q, q_stride,
                       (bf16*)out, out_stride, (const bf16*)k_pages, (const bf16*)v_pages, block_table, bt_width,
                       page_size, positions, cu_seqlens, n_seqs, H, Hkv, scale, window, partials, counters, nsplit, max_pages,
                       fz);
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
                         float scale, int window, float* partials, int* counters, int nsplit, int max_pages, int waves,
                         const int* token_seq, hipStream_t stream) {
    MV_REQUIRE(H / Hkv <= 16, "attention_decode: %d query heads per kv head exceed 16", H / Hkv);
    MV_REQUIRE(nsplit >= 1 && nsplit <= AF_MAX_SPLITS && (nsplit == 1 || (partials != nullptr && counters != nullptr)),
               "attention_decode: bad split count %d or missing work area or counters", nsplit);
    MV_REQUIRE(waves == 4 || waves == 8, "attention_decode: %d waves per workgroup (4 or 8)", waves);
    if (n_seqs <= 0) return 0;
    if (max_pages <= 0 || max_pages > bt_width) max_pages = bt_width;
    dim3 grid(n_seqs, Hkv, nsplit);
    float* part = nsplit > 1 ? partials : nullptr;
    // With more workgroups than compute units, two of them share a unit (the kernel is then held to
    // 256 registers a lane, which costs it three spilled ones at head size 128): one's set-up and
    // tail overlap the other's stream of keys, 4-6 % on a step of 64 to 256 sequences. A grid that
    // fits the chip at once keeps all registers.
    const int occ = ((long)n_seqs * Hkv > mv_compute_units() && nsplit == 1) ? 2 : 1;
#define AF_LAUNCH(DD, WW, FF)                                                                                     \
    do {                                                                                                          \
        if constexpr (WW == 4) {                                                                                  \
            if (occ == 2) {                                                                                       \
                launch_decode<DD, WW, FF, 2>(grid, stream, q, q_stride, out, out_stride, k_pages, v_pages,        \
                                             block_table, bt_width, page_size, positions, cu_seqlens, n_seqs, H,  \
                                             Hkv, scale, window, part, counters, nsplit, max_pages, fz);          \
                break;                                                                                            \
            }                                                                                                     \
        }                                                                                                         \
        launch_decode<DD, WW, FF, 1>(grid, stream, q, q_stride, out, out_stride, k_pages, v_pages, block_table,   \
                                     bt_width, page_size, positions, cu_seqlens, n_seqs, H, Hkv, scale, window,   \
                                     part, counters, nsplit, max_pages, fz);                                      \
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
    return mv_check_launch("attention_decode");
}

// Decode steps: every sequence brings one token (a sequence may bring up to 16 / (H / Hkv)).
// grid = (sequences, kv heads, nsplit); `waves` (4 or 8) per workgroup. With nsplit > 1 the keys of
// a sequence are dealt out over nsplit workgroups, which need partials: float [tokens * H * nsplit *
// (D + 2)] and counters: int [n_seqs * Hkv], zero before the first launch (every launch leaves them
// zero); launches that share the counters must not overlap. max_pages: the pages of the block table
// that the longest context of the step may fill (0: all), asked for before a sequence's length is
// known.
extern "C" int mv_attention_decode(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
                                   const void* v_pages, const int* block_table, int bt_width, int page_size,
                                   const int* positions, const int* cu_seqlens, int n_seqs, int H, int Hkv, int D,
                                   float scale, int window, float* partials, int* counters, int nsplit,
                                   int max_pages, int waves, const int* token_seq, hipStream_t stream) {
    if (int rc = check_common("attention_decode", q_stride, out_stride, page_size, bt_width, H, Hkv, D)) return rc;
    return decode_common(false, FusedInput{}, q, q_stride, out, out_stride, k_pages, v_pages, block_table, bt_width,
                         page_size, positions, cu_seqlens, n_seqs, H, Hkv, D, scale, window, partials, counters, nsplit,
                         max_pages, waves, token_seq, stream);
}

// The same for a decode step whose queries, keys and values are still the raw rows of the
// [q | k | v] product (one token a sequence; row t of qkv belongs to sequence t): per-head RMSNorm
// (q_weight / k_weight, or null for none) and rotation by the table row of the position
// (half-split pairs over the whole head, or null for none) happen on the way into the kernel;
// `rows` [tokens, D], when given, holds the table's rows of the step's positions (row t for token t),
// gathered once a step, so that no layer has to wait for the position before it can ask for the angles;
// with store_kv the new key and value are written to their page slot as well.
extern "C" int mv_attention_decode_fused(const void* qkv, long qkv_stride, int q_off, int k_off, int v_off, void* out,
                                         long out_stride, void* k_pages, void* v_pages, const int* block_table,
                                         int bt_width, int page_size, const int* positions, const int* cu_seqlens,
                                         int n_seqs, int H, int Hkv, int D, float scale, int window,
                                         const void* q_weight, const void* k_weight, int weight_dtype, float eps,
                                         int unit_offset, const float* table, const float* rows, int store_kv,
                                         float* partials,
                                         int* counters, int nsplit, int max_pages, int waves, const int* token_seq,
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
    MV_REQUIRE(rows == nullptr || (table != nullptr && ((uintptr_t)rows % 16) == 0),
               "attention_decode_fused: rotation rows come with their table and are 16-byte aligned");
    FusedInput fz{(const bf16*)qkv, qkv_stride, q_off, k_off, v_off, WeightPtr{q_weight, weight_dtype},
                  WeightPtr{k_weight, weight_dtype}, has_norm, eps, unit_offset, table, rows, store_kv ? 1 : 0, token_seq};
    return decode_common(true, fz, nullptr, 0, out, out_stride, k_pages, v_pages, block_table, bt_width, page_size,
                         positions, cu_seqlens, n_seqs, H, Hkv, D, scale, window, partials, counters, nsplit, max_pages,
                         waves, token_seq, stream);
}
