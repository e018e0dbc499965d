// Paged causal attention for prompt portions and mixed steps on the MFMA units of gfx950,
// bf16 in and out, float inside.
//
// A workgroup of four waves serves one key/value head of one unit: up to 64*NT columns, a column
// being a (query token, query head of the group) pair of a run of consecutive tokens of one
// sequence. Each wave owns 16*NT columns. The workgroup walks the keys the unit may see in blocks
// of 32; every block's K tile [32 keys x D] and transposed V tile [D x 32 keys] are copied from
// the cache pages into LDS once, in the order the MFMA operands are read (so the reads are
// conflict-free 16-byte loads), double-buffered: the copy of block b+1 is in flight while block
// b is computed, with one barrier per block.
//
//   scores^T = K Q^T     A operand: 16 keys x 32 d from LDS, B operand: the wave's queries (registers);
//                        result: lane l holds column l%16, keys 4*(l/16)+0..3 of the 16-key tile.
//   out^T    = V^T P^T   A operand: 16 d x 32 keys from LDS, B operand: the probabilities the lane
//                        already holds: its eight k-slots are bound to keys {4g..4g+3} of the two
//                        16-key tiles of the block (g = l/16), and V is stored in LDS for exactly
//                        those keys, so nothing is shuffled between the two products.
// Online softmax (base 2) per column. A wave skips blocks that lie outside the range of all its
// columns. Value slots above the unit's newest key were never written and are copied as zero.
//
// With KW = 2 the workgroup has eight waves: two groups of four that serve the same columns and
// take the key blocks in turn (group 0 the even ones of the unit's range, group 1 the odd ones),
// each with LDS tiles of its own, and merge their partial results through LDS at the end. The
// walk of a unit with many keys takes half as many rounds.
//
// Layouts: K[page][kv_head][slot][d], V[page][kv_head][d][slot]; page size a multiple of 16.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    uint2 h[2];
    uint16_t s[8];
    bf16x8_t v;
};

#define AP_WAVES 4
#define AP_THREADS (64 * AP_WAVES)
#define LOG2E 1.4426950408889634f

// Two workgroups share a compute unit (LDS and latency hiding are sized for that), so a wave may
// use half of a SIMD's registers: the accumulators stay in the vector registers and the operand
// reads from LDS run ahead of the MFMAs.
template <int D, int NT, int KW>
__global__ void __launch_bounds__(AP_THREADS * KW) __attribute__((amdgpu_waves_per_eu(2, 2)))
attention_prefill_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                         const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                         const int* __restrict__ block_table, int bt_width, int page_size, int page_shift,
                         const int* __restrict__ positions, const int* __restrict__ cu_seqlens, int n_seqs, int H,
                         int Hkv, float scale, int window, int fold) {
    constexpr int DS = D / 32;                 // k-steps of the score product
    constexpr int DT = D / 16;                 // d tiles of the output product
    constexpr int COLS = 16 * AP_WAVES * NT;   // columns of a workgroup
    constexpr int KCHUNKS = 2 * DS * 64;       // 16-byte chunks of a K tile
    constexpr int VCHUNKS = DT * 64;           // 16-byte chunks of a V tile (two 8-byte halves each)
    constexpr int KREP = KCHUNKS / AP_THREADS;
    constexpr int VREP = 2 * VCHUNKS / AP_THREADS;      // 8-byte chunks of a V tile pair per thread
    static_assert(KCHUNKS % AP_THREADS == 0 && (D * 2 * 2) % AP_THREADS == 0, "tile does not divide the workgroup");

    // [buffer][key group] tiles: K as 16-byte chunks, then V as 8-byte chunks
    extern __shared__ uint4 lds_tiles[];
    uint4* const sK_all = lds_tiles;
    uint2* const sV_all = reinterpret_cast<uint2*>(lds_tiles + 2 * KW * KCHUNKS);
    __shared__ int sh_unit[3];
    __shared__ int sh_range[2][AP_WAVES * KW];

    const int G = H / Hkv;
    // the key/value head is the fastest grid dimension: workgroups are dealt to the eight XCDs in
    // turn, so all units of a head land on the same XCD and share its L2
    const int kvh = blockIdx.x;
    const int tid = threadIdx.x;
    const int wave = tid / MV_WAVE;
    const int lane = tid % MV_WAVE;
    const int cw = wave % AP_WAVES;            // which columns of the unit
    const int kg = wave / AP_WAVES;            // which of the KW key groups
    const int gtid = tid % AP_THREADS;         // thread within its key group
    const int i = lane % 16;
    const int g = lane / 16;
    const int tpu = COLS / G;  // tokens of a unit (the host made sure it is >= 1)

    if (tid == 0) {
        int seq = -1, t0 = 0, nt = 0;
        // Units with the most keys start first. When the whole grid is resident at once (two
        // workgroups a compute unit, dealt out in order), the second half of the grid runs from
        // the lightest unit upwards instead, so that the two workgroups that share a compute unit
        // bring about the same number of key blocks together.
        const int n_all = gridDim.y, half = (n_all + 1) / 2;
        int u = (!fold || (int)blockIdx.y < half) ? n_all - 1 - (int)blockIdx.y : (int)blockIdx.y - half;
        for (int s = 0; s < n_seqs; ++s) {
            const int ql = cu_seqlens[s + 1] - cu_seqlens[s];
            const int nu = (ql + tpu - 1) / tpu;
            if (u < nu) {
                seq = s;
                t0 = cu_seqlens[s] + u * tpu;
                nt = ql - u * tpu;
                if (nt > tpu) nt = tpu;
                break;
            }
            u -= nu;
        }
        sh_unit[0] = seq;
        sh_unit[1] = t0;
        sh_unit[2] = nt;
    }
    __syncthreads();
    const int seq = sh_unit[0], t0 = sh_unit[1], nt = sh_unit[2];
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
        const int col = (cw * NT + ct) * 16 + i;
        col_ok[ct] = col < ncols;
        col_tok[ct] = t0 + (col_ok[ct] ? col / G : 0);
        col_head[ct] = kvh * G + (col_ok[ct] ? col % G : 0);
        col_pos[ct] = col_ok[ct] ? positions[col_tok[ct]] : -1;
        col_lo[ct] = (window >= 0 && col_pos[ct] - window > 0) ? col_pos[ct] - window : 0;
        if (col_ok[ct]) {
            hi_w = col_pos[ct] > hi_w ? col_pos[ct] : hi_w;
            lo_w = col_lo[ct] < lo_w ? col_lo[ct] : lo_w;
        }
        const bf16* qrow = q + (size_t)col_tok[ct] * q_stride + (size_t)col_head[ct] * D + 8 * g;
#pragma unroll
        for (int s = 0; s < DS; ++s)
            qop[ct][s].u = col_ok[ct] ? *reinterpret_cast<const uint4*>(qrow + 32 * s) : uint4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int o = MV_WAVE / 2; o > 0; o >>= 1) {
        const int a = __shfl_xor(hi_w, o, MV_WAVE), b = __shfl_xor(lo_w, o, MV_WAVE);
        hi_w = a > hi_w ? a : hi_w;
        lo_w = b < lo_w ? b : lo_w;
    }
    if (lane == 0) {
        sh_range[0][wave] = hi_w;
        sh_range[1][wave] = lo_w;
    }
    __syncthreads();
    int hi_g = -1, lo_g = 0x7fffffff;
#pragma unroll
    for (int w = 0; w < AP_WAVES * KW; ++w) {
        hi_g = sh_range[0][w] > hi_g ? sh_range[0][w] : hi_g;
        lo_g = sh_range[1][w] < lo_g ? sh_range[1][w] : lo_g;
    }
    if (hi_g < 0) return;
    const int b0 = lo_g / 32, b1 = hi_g / 32;

    float m_run[NT], l_run[NT];
    floatx4_t acc_o[NT][DT];
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        m_run[ct] = -INFINITY;
        l_run[ct] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc_o[ct][dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    }
    const float sc_mul = scale * LOG2E;

    // ---- copy of a block from the pages: global -> registers -> LDS.
    // Two blocks are in flight: while block b is computed, block b+1 waits in one register set
    // and block b+2 is being loaded into the other. Everything that does not depend on the block
    // (which chunk of the tile a thread copies, where it goes in LDS) is worked out once.
    // A thread copies the chunks whose place in LDS follows its id, so that the LDS writes of a wave
    // are consecutive (no bank conflicts); the matching global reads touch, per instruction, 64
    // contiguous bytes of 16 key rows (K) or the contiguous slots of a page's rows (V).
    struct Staged {
        uint4 k[KREP];
        uint2 v[VREP];
    };
    int k_tile[KREP], k_off[KREP], k_lds[KREP];
#pragma unroll
    for (int rep = 0; rep < KREP; ++rep) {
        const int L = gtid + AP_THREADS * rep;         // LDS chunk: ((tile * DS + s) * 64 + operand lane)
        const int ol = L % 64;
        k_tile[rep] = L / (DS * 64);
        k_off[rep] = (ol % 16) * D + 32 * ((L / 64) % DS) + 8 * (ol / 16);
        k_lds[rep] = L;
    }
    int v_tile[VREP], v_off[VREP], v_lds[VREP], v_key[VREP];
#pragma unroll
    for (int rep = 0; rep < VREP; ++rep) {
        const int L = gtid + AP_THREADS * rep;         // LDS chunk: ((d tile * 64 + operand lane) * 2 + key tile)
        const int ol = (L / 2) % 64;
        v_tile[rep] = L % 2;
        v_off[rep] = (16 * (L / 128) + ol % 16) * page_size + 4 * (ol / 16);
        v_key[rep] = 16 * v_tile[rep] + 4 * (ol / 16);
        v_lds[rep] = L;
    }
    const int page_mask = page_size - 1;
    auto fetch = [&](int b, Staged& st) {
        if (b > b1) {   // past the unit's range: nothing to read (the block is not computed either)
#pragma unroll
            for (int rep = 0; rep < KREP; ++rep) st.k[rep] = uint4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int rep = 0; rep < VREP; ++rep) st.v[rep] = uint2{0u, 0u};
            return;
        }
        const bf16* kbase[2];
        const bf16* vbase[2];
        bool gone[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key0 = 32 * b + 16 * t;
            int pidx = key0 >> page_shift;
            pidx = pidx < bt_width ? pidx : bt_width - 1;
            int pg = bt[pidx];
            gone[t] = pg < 0;      // a page that was given back (it lies below every column's range):
            pg = gone[t] ? 0 : pg; // read some page, then put zeros in its place
            const int slot0 = key0 & page_mask;
            const size_t head = (size_t)pg * Hkv + kvh;
            kbase[t] = k_pages + (head * page_size + slot0) * D;
            vbase[t] = v_pages + head * D * page_size + slot0;
        }
#pragma unroll
        for (int rep = 0; rep < KREP; ++rep)
            st.k[rep] = *reinterpret_cast<const uint4*>((k_tile[rep] ? kbase[1] : kbase[0]) + k_off[rep]);
#pragma unroll
        for (int rep = 0; rep < VREP; ++rep)
            st.v[rep] = *reinterpret_cast<const uint2*>((v_tile[rep] ? vbase[1] : vbase[0]) + v_off[rep]);
        if (gone[0] || gone[1]) {
#pragma unroll
            for (int rep = 0; rep < KREP; ++rep)
                if (gone[k_tile[rep]]) st.k[rep] = uint4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int rep = 0; rep < VREP; ++rep)
                if (gone[v_tile[rep]]) st.v[rep] = uint2{0u, 0u};
        }
    };
    // round j of the walk: key group kg has block b0 + j * KW + kg, in the tiles [j & 1][kg]
    auto block_of = [&](int j) { return b0 + j * KW + kg; };
    auto stash = [&](int j, const Staged& st) {
        const int b = block_of(j);
        uint4* sK = sK_all + ((j & 1) * KW + kg) * KCHUNKS;
        uint2* sV = sV_all + ((j & 1) * KW + kg) * (VCHUNKS * 2);
#pragma unroll
        for (int rep = 0; rep < KREP; ++rep) sK[k_lds[rep]] = st.k[rep];
        const bool tail = 32 * b + 31 > hi_g;  // slots above the newest key were never written
#pragma unroll
        for (int rep = 0; rep < VREP; ++rep) {
            uint2 f = st.v[rep];
            if (tail) {
                const int key = 32 * b + v_key[rep];
                if (key > hi_g) f.x = 0;
                else if (key + 1 > hi_g) f.x &= 0xffffu;
                if (key + 2 > hi_g) f.y = 0;
                else if (key + 3 > hi_g) f.y &= 0xffffu;
            }
            sV[v_lds[rep]] = f;
        }
    };

    // keys at or below `full_hi` and at or above `full_lo` are visible to every column of the wave:
    // blocks inside need no mask
    int full_hi = 0x7fffffff, full_lo = 0;
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        const int ph = col_ok[ct] ? col_pos[ct] : 0x7fffffff;
        const int pl = col_ok[ct] ? col_lo[ct] : 0;
        full_hi = ph < full_hi ? ph : full_hi;
        full_lo = pl > full_lo ? pl : full_lo;
    }
#pragma unroll
    for (int o = MV_WAVE / 2; o > 0; o >>= 1) {
        const int a = __shfl_xor(full_hi, o, MV_WAVE), c = __shfl_xor(full_lo, o, MV_WAVE);
        full_hi = a < full_hi ? a : full_hi;
        full_lo = c > full_lo ? c : full_lo;
    }
    bool all_cols = true;
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) all_cols = all_cols && col_ok[ct];
    const bool wave_full = __all(all_cols);

    auto compute = [&](int j) {
        const int b = block_of(j);
        const uint4* sK = sK_all + ((j & 1) * KW + kg) * KCHUNKS;
        const uint2* sV = sV_all + ((j & 1) * KW + kg) * (VCHUNKS * 2);
        const int base = 32 * b;
        if (b > b1 || !(base <= hi_w && base + 31 >= lo_w)) return;
        const bool masked = !(wave_full && base + 31 <= full_hi && base >= full_lo);
        // scores^T for the two 16-key tiles
        float p[NT][2][4];
        Frag kop[2][DS];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < DS; ++s) kop[t][s].u = sK[(t * DS + s) * 64 + lane];
        // the value operands are asked for now and arrive while the softmax is worked out
        Frag vop[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            vop[dt].h[0] = sV[(dt * 64 + lane) * 2];
            vop[dt].h[1] = sV[(dt * 64 + lane) * 2 + 1];
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) {
                floatx4_t sacc = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < DS; ++s)
                    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[t][s].v, qop[ct][s].v, sacc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) p[ct][t][r] = sacc[r];
            }
        }
        if (masked) {
#pragma unroll
            for (int ct = 0; ct < NT; ++ct)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = base + 16 * t + 4 * g + r;
                        const bool ok = col_ok[ct] && key <= col_pos[ct] && key >= col_lo[ct];
                        p[ct][t][r] = ok ? p[ct][t][r] : -INFINITY;
                    }
        }
        // online softmax per column
        Frag pop[NT];
#pragma unroll
        for (int ct = 0; ct < NT; ++ct) {
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) mx = fmaxf(mx, p[ct][t][r]);
            // The reference point of the exponentials (kept in the scaled, base-2 domain; the scale
            // is positive) only follows the maximum when it has been overtaken by more than 2^8:
            // until then the terms stay below 2^8 and nothing is rescaled. A column's maximum is
            // spread over four lanes, but it exceeds the bound exactly when one lane's share does,
            // so the lanes are only brought together (two shuffles) when a vote says so.
            const bool stale = mx * sc_mul > m_run[ct] + 8.f;
            if (__any(stale)) {
                mx = fmaxf(mx, __shfl_xor(mx, 16, MV_WAVE));
                mx = fmaxf(mx, __shfl_xor(mx, 32, MV_WAVE));
                const float mx_s = mx * sc_mul;
                const float m_new = fmaxf(m_run[ct], mx_s);
                const float m_ref = (m_new == -INFINITY) ? 0.f : m_new;
                const float corr = __builtin_amdgcn_exp2f(m_run[ct] - m_ref);   // exp2(-inf) = 0
                l_run[ct] *= corr;
                m_run[ct] = m_new;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) acc_o[ct][dt] *= corr;
            }
            const float m_safe = (m_run[ct] == -INFINITY) ? 0.f : m_run[ct];
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float e = __builtin_amdgcn_exp2f(fmaf(p[ct][t][r], sc_mul, -m_safe));
                    psum += e;
                    pop[ct].v[t * 4 + r] = (__bf16)e;
                }
            l_run[ct] += psum;
        }
        // out^T += V^T P^T
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int ct = 0; ct < NT; ++ct)
                acc_o[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[dt].v, pop[ct].v, acc_o[ct][dt], 0, 0, 0);
    };

    const int rounds = (b1 - b0 + KW) / KW;    // the same for every wave: they meet at the barriers
    Staged sa, sb;
    fetch(block_of(0), sa);
    fetch(block_of(1), sb);
    stash(0, sa);
    __syncthreads();
    // invariant at the top: LDS holds round j, `sb` holds round j+1 (or zeros past the end)
    for (int j = 0; j < rounds; j += 2) {
        fetch(block_of(j + 2), sa);
        compute(j);
        if (j + 1 < rounds) stash(j + 1, sb);
        __syncthreads();
        if (j + 1 >= rounds) break;
        fetch(block_of(j + 3), sb);
        compute(j + 1);
        if (j + 2 < rounds) stash(j + 2, sa);
        __syncthreads();
    }

    // the sum of a column is spread over the four lane groups
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        l_run[ct] += __shfl_xor(l_run[ct], 16, MV_WAVE);
        l_run[ct] += __shfl_xor(l_run[ct], 32, MV_WAVE);
    }

    if (KW > 1) {
        // ---- key group 1 hands its partial results to group 0 through LDS (the tiles are no
        // longer needed: every wave has passed the last barrier of the walk), one column tile at a time
        float* xo = reinterpret_cast<float*>(lds_tiles);                 // [AP_WAVES][DT][4][64]
        float* xm = xo + AP_WAVES * DT * 4 * MV_WAVE;                    // [AP_WAVES][16] maxima, then sums
        float* xl = xm + AP_WAVES * 16;
#pragma unroll
        for (int ct = 0; ct < NT; ++ct) {
            if (ct) __syncthreads();
            if (kg == 1) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) xo[((cw * DT + dt) * 4 + r) * MV_WAVE + lane] = acc_o[ct][dt][r];
                if (g == 0) {
                    xm[cw * 16 + i] = m_run[ct];
                    xl[cw * 16 + i] = l_run[ct];
                }
            }
            __syncthreads();
            if (kg == 0) {
                const float m1 = xm[cw * 16 + i], l1 = xl[cw * 16 + i];
                const float m_fin = fmaxf(m_run[ct], m1);
                const float f0 = (m_run[ct] == -INFINITY) ? 0.f : exp2f(m_run[ct] - m_fin);
                const float f1 = (m1 == -INFINITY) ? 0.f : exp2f(m1 - m_fin);
                l_run[ct] = f0 * l_run[ct] + f1 * l1;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        acc_o[ct][dt][r] = f0 * acc_o[ct][dt][r] + f1 * xo[((cw * DT + dt) * 4 + r) * MV_WAVE + lane];
            }
        }
        if (kg != 0) return;
    }

#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        if (!col_ok[ct]) continue;
        const float inv = 1.f / l_run[ct];
        bf16* orow = out + (size_t)col_tok[ct] * out_stride + (size_t)col_head[ct] * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            uint2 packed;
            packed.x = (uint32_t)f32_to_bf16_bits(acc_o[ct][dt][0] * inv) |
                       ((uint32_t)f32_to_bf16_bits(acc_o[ct][dt][1] * inv) << 16);
            packed.y = (uint32_t)f32_to_bf16_bits(acc_o[ct][dt][2] * inv) |
                       ((uint32_t)f32_to_bf16_bits(acc_o[ct][dt][3] * inv) << 16);
            *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * g) = packed;
        }
    }
}

extern "C" int mv_attention_prefill_unit_tokens(int group, int nt) {
    if (nt != 1 && nt != 2) return 0;
    const int cols = 16 * AP_WAVES * nt;
    return group > 0 && group <= cols ? cols / group : 0;
}

template <int D, int NT, int KW>
static int launch_prefill(dim3 grid, hipStream_t stream, const void* q, long q_stride, void* out, long out_stride,
                          const void* k_pages, const void* v_pages, const int* block_table, int bt_width,
                          int page_size, int page_shift, const int* positions, const int* cu_seqlens, int n_seqs,
                          int H, int Hkv, float scale, int window, int fold) {
    // K and V tiles of 32 keys, double-buffered, one set per key group
    const size_t lds = (size_t)2 * KW * (2 * (D / 32) * 64 * 16 + (D / 16) * 64 * 16);
    static bool allowed = false;   // more than 64 KiB of LDS has to be asked for, once per kernel
    if (!allowed && lds > 48 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_kernel<D, NT, KW>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return mv_fail("attention_prefill: %zu bytes of LDS were refused: %s", lds, hipGetErrorString(e));
        allowed = true;
    }
    hipLaunchKernelGGL((attention_prefill_kernel<D, NT, KW>), grid, dim3(AP_THREADS * KW), lds, stream, (const bf16*)q,
                       q_stride, (bf16*)out, out_stride, (const bf16*)k_pages, (const bf16*)v_pages, block_table,
                       bt_width, page_size, page_shift, positions, cu_seqlens, n_seqs, H, Hkv, scale, window, fold);
    return 0;
}

// nt: column tiles per wave (2 = 128 columns per workgroup, for long prompts; 1 = 64 columns, twice
// the workgroups, for steps too small to fill the chip otherwise).
// kw: key groups per workgroup (2: eight waves, the walk over a unit's keys takes half as many rounds).
// n_units = sum over sequences of ceil(q_len / unit tokens(group, nt)). grid = (kv heads, units).
extern "C" int mv_attention_prefill(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
                                    const void* v_pages, const int* block_table, int bt_width, int page_size,
                                    const int* positions, const int* cu_seqlens, int n_seqs, int n_units, int nt,
                                    int kw, int H, int Hkv, int D, float scale, int window, hipStream_t stream) {
    MV_REQUIRE(kw == 1 || kw == 2, "attention_prefill: %d key groups per workgroup (1 or 2)", kw);
    MV_REQUIRE(H > 0 && Hkv > 0 && H % Hkv == 0, "attention_prefill: %d heads are not a multiple of %d kv heads", H,
               Hkv);
    MV_REQUIRE(D == 64 || D == 128, "attention_prefill: head_dim %d is not served by the MFMA kernel (64 or 128)", D);
    MV_REQUIRE(page_size >= 16 && (page_size & (page_size - 1)) == 0,
               "attention_prefill: page size %d must be a power of two, at least 16", page_size);
    MV_REQUIRE(bt_width > 0, "attention_prefill: empty block table");
    MV_REQUIRE(q_stride >= (long)H * D && q_stride % 8 == 0 && out_stride >= (long)H * D && out_stride % 4 == 0,
               "attention_prefill: row strides %ld / %ld do not fit %d heads of %d", q_stride, out_stride, H, D);
    MV_REQUIRE(n_units <= 65535, "attention_prefill: %d units exceed one launch", n_units);
    MV_REQUIRE(mv_attention_prefill_unit_tokens(H / Hkv, nt) > 0, "attention_prefill: %d query heads per kv head "
               "with %d column tiles per wave are not served", H / Hkv, nt);
    if (n_seqs <= 0 || n_units <= 0) return 0;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    dim3 grid(Hkv, n_units, 1);
    // everything resident at once: two workgroups for each of the device's compute units
    int cus = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        cus = 256;
    const int fold = (kw == 1 && (long)Hkv * n_units <= 2L * cus) ? 1 : 0;
    int rc = 0;
#define AP_LAUNCH(DD, NN, KK)                                                                                      \
    rc = launch_prefill<DD, NN, KK>(grid, stream, q, q_stride, out, out_stride, k_pages, v_pages, block_table,       \
                                    bt_width, page_size, page_shift, positions, cu_seqlens, n_seqs, H, Hkv, scale,  \
                                    window, fold)
    if (kw == 2) {
        if (D == 128 && nt == 2) AP_LAUNCH(128, 2, 2);
        else if (D == 128) AP_LAUNCH(128, 1, 2);
        else if (nt == 2) AP_LAUNCH(64, 2, 2);
        else AP_LAUNCH(64, 1, 2);
    } else {
        if (D == 128 && nt == 2) AP_LAUNCH(128, 2, 1);
        else if (D == 128) AP_LAUNCH(128, 1, 1);
        else if (nt == 2) AP_LAUNCH(64, 2, 1);
        else AP_LAUNCH(64, 1, 1);
    }
#undef AP_LAUNCH
    if (rc) return rc;
    return mv_check_launch("attention_prefill");
}
