// Paged causal attention for prompt portions and mixed steps on the MFMA units of gfx950,
// bf16 in and out, float inside.
//
// A workgroup of four waves serves one key/value head of one unit: up to 64*NT columns, a column
// being a (query token, query head of the group) pair of a run of consecutive tokens of one
// sequence. Each wave owns 16*NT columns. The workgroup walks the keys the unit may see in blocks
// of 32. Every block's K tile [32 keys x D] and V tile [D x 32 keys] go from the cache pages
// straight into LDS (global_load_lds: no registers in between, no LDS store instructions), in the
// order the MFMA operands are read (so the reads are conflict-free 16-byte loads), into four stages
// in two pairs that are filled ahead of the computation: two blocks are computed to a barrier while
// the next two land in the other pair. With four waves the barrier stands between the two blocks
// of a pair and a block's operands come from LDS while the block before is computed (keys a block
// ahead, values behind the score product); with eight waves both blocks are read and computed
// between two barriers.
//
//   scores^T = K Q^T     A operand: 16 keys x 32 d from LDS, B operand: the wave's queries (registers);
//                        result: lane l holds column l%16 and rows 4*(l/16)+0..3 of the tile.
//   out^T    = V^T P^T   A operand: 16 d x 32 keys from LDS, B operand: the probabilities the lane
//                        already holds. Its eight k-slots must be eight keys that lie side by side
//                        in a page's V rows (one 16-byte load per operand), so row 4g+r of score tile
//                        t is bound to key 8g + 4t + r of the block (g = l/16): the two score tiles
//                        interleave in groups of four keys, and nothing is shuffled between the two
//                        products.
// Online softmax (base 2) per column. A wave skips blocks that lie outside the range of all its
// columns. Value slots above the unit's newest key were never written and may hold anything; the
// lane that brought them in clears them in LDS before the block is used (keys above a column's
// position get probability zero, and zero times a stray NaN would not be zero).
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
    uint16_t s[8];
    bf16x8_t v;
};

typedef __attribute__((address_space(1))) const void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// s_waitcnt that only bounds the vector memory counter (N outstanding loads may remain)
#define AP_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(0x0f70 | ((N) & 15) | (((N) >> 4) << 14))
// s_waitcnt that only waits for the LDS (and scalar memory) counter
#define AP_WAIT_LDS() __builtin_amdgcn_s_waitcnt(0xc07f)

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
    constexpr int VCHUNKS = DT * 64;           // 16-byte chunks of a V tile
    constexpr int TILE = KCHUNKS + VCHUNKS;    // chunks of a block: its K tile, then its V tile
    constexpr int KREP = 2 * DS / AP_WAVES;    // load instructions a wave issues for a K tile (64 chunks each)
    constexpr int VREP = DT / AP_WAVES;        // ... and for a V tile
    static_assert((2 * DS) % AP_WAVES == 0 && DT % AP_WAVES == 0, "tile does not divide the workgroup");

    // Four LDS stages of [key group] blocks in two pairs: the blocks of one pair are computed while
    // those of the other are landing. They are separate arrays, not one, so that the compiler can
    // tell a load into one stage from the operand reads of another and does not make the reads wait
    // for the loads in flight.
    __shared__ uint4 stage0[KW * TILE];
    __shared__ uint4 stage1[KW * TILE];
    __shared__ uint4 stage2[KW * TILE];
    __shared__ uint4 stage3[KW * TILE];
    __shared__ int sh_unit[3];
    __shared__ int sh_range[2][AP_WAVES * KW];

    const int G = H / Hkv;
    // the key/value head is the fastest grid dimension: workgroups are dealt to the eight XCDs in
    // turn, so all units of a head land on the same XCD and share its L2
    const int kvh = blockIdx.x;
    const int tid = threadIdx.x;
    const int wave = tid / MV_WAVE;
    const int lane = tid % MV_WAVE;
    const int cw = __builtin_amdgcn_readfirstlane(wave % AP_WAVES);   // which columns of the unit
    // which of the KW key groups; the same for a whole wave, and said so: everything that follows
    // from it (block numbers, page ids, tile addresses) then lives in scalar registers
    const int kg = __builtin_amdgcn_readfirstlane(wave / AP_WAVES);
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
    const int seq = __builtin_amdgcn_readfirstlane(sh_unit[0]);
    const int t0 = __builtin_amdgcn_readfirstlane(sh_unit[1]);
    const int nt = __builtin_amdgcn_readfirstlane(sh_unit[2]);
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
    hi_w = __builtin_amdgcn_readfirstlane(hi_w);
    lo_w = __builtin_amdgcn_readfirstlane(lo_w);
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
    hi_g = __builtin_amdgcn_readfirstlane(hi_g);
    lo_g = __builtin_amdgcn_readfirstlane(lo_g);
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

    // ---- a block's way from the pages into LDS.
    // A load instruction of a wave fills 64 consecutive 16-byte chunks of LDS, one per lane, from
    // addresses the lanes choose: the chunks of one (score tile, k-step) pair of K, or of one d tile
    // of V. A lane's chunk is the operand that lane will read back: 8 d of one key (K), or 8 keys of
    // one d row (V). Everything that does not depend on the block is worked out once. The block
    // number is the same for a wave, so its page ids are scalar loads, asked for a round before they
    // are used.
    // The page ids of a block are per-lane loads: a lane brings in keys of one half of the block and
    // values of one half (the halves differ), so it asks for exactly the two ids it needs, a round
    // before they are used, and nothing of the addressing lives in scalar registers.
    struct PageIds {
        int k, v;     // the pages of the lane's key half and value half
    };
    const int rho = lane % 16;
    // K: row rho of score tile t is key 8*(rho/4) + 4t + rho%4; the half of the block it lies in
    // does not depend on t
    const int k_half = rho / 8;
    const int v_half = g / 2;
    const int page_mask = page_size - 1;
    // a page's bytes per tensor, and where this key/value head starts in it (K [slot][d] and V [d][slot]
    // have the same size)
    const unsigned page_bytes = (unsigned)Hkv * page_size * D * sizeof(bf16);
    const char* const k_head = reinterpret_cast<const char*>(k_pages) + (size_t)kvh * page_size * D * sizeof(bf16);
    const char* const v_head = reinterpret_cast<const char*>(v_pages) + (size_t)kvh * page_size * D * sizeof(bf16);
    // what of a lane's addresses does not depend on the block: head, the slot of its half within a
    // page (pages of 16: none), its chunk of the first load
    const char* k_lane;
    const char* v_lane;
    unsigned k_step[KREP], v_step[VREP];   // further loads: constant distances from the first
    {
        const int hk = (16 * k_half) & page_mask, hv = (16 * v_half) & page_mask;
        unsigned k_off[KREP], v_off[VREP];
#pragma unroll
        for (int rep = 0; rep < KREP; ++rep) {
            const int pair = cw + AP_WAVES * rep;   // (score tile, k-step): LDS chunks pair * 64 ...
            const int t = pair / DS, ks = pair % DS;
            const int slot = 8 * ((rho / 4) % 2) + 4 * t + rho % 4;    // within its half
            k_off[rep] = (unsigned)((slot * D + 32 * ks + 8 * g) * sizeof(bf16));
            k_step[rep] = k_off[rep] - k_off[0];
        }
        // V: lane group g holds keys 8g .. 8g+7 of d row 16*dt + rho
#pragma unroll
        for (int rep = 0; rep < VREP; ++rep) {
            const int dt = cw + AP_WAVES * rep;
            v_off[rep] = (unsigned)(((16 * dt + rho) * page_size + 8 * (g % 2)) * sizeof(bf16));
            v_step[rep] = v_off[rep] - v_off[0];
        }
        k_lane = k_head + (size_t)hk * D * sizeof(bf16) + k_off[0];
        v_lane = v_head + (size_t)hv * sizeof(bf16) + v_off[0];
    }
    // round j of the walk: key group kg has block b0 + j * KW + kg
    auto block_of = [&](int j) { return b0 + j * KW + kg; };
    auto page_ids = [&](int j) {
        int b = block_of(j);
        b = b < b1 ? b : b1;    // past the unit's range: some valid entry (the block is not fetched)
        PageIds ids;
        int pk = (32 * b + 16 * k_half) >> page_shift, pv = (32 * b + 16 * v_half) >> page_shift;
        pk = pk < bt_width ? pk : bt_width - 1;
        pv = pv < bt_width ? pv : bt_width - 1;
        ids.k = bt[pk];
        ids.v = bt[pv];
        return ids;
    };
    // Asks for the block of round j (at most the unit's last one: the same block again does no harm).
    // A page that was given back (its keys lie below every column's range) has a negative id: some
    // page is read in its place and the values are cleared when they have landed.
    auto fetch = [&](int j, const PageIds& ids, uint4* stage) {
        int b = block_of(j);
        b = b < b1 ? b : b1;
        const unsigned sb = (unsigned)((32 * b) & page_mask);     // the block's first slot within its page
        const unsigned pgk = ids.k < 0 ? 0u : (unsigned)ids.k, pgv = ids.v < 0 ? 0u : (unsigned)ids.v;
        const char* kb = k_lane + (size_t)pgk * page_bytes + sb * (unsigned)(D * sizeof(bf16));
        const char* vb = v_lane + (size_t)pgv * page_bytes + sb * (unsigned)sizeof(bf16);
        uint4* tile = stage + kg * TILE;
#pragma unroll
        for (int rep = 0; rep < KREP; ++rep)
            __builtin_amdgcn_global_load_lds((global_ptr_t)(kb + k_step[rep]),
                                             (lds_ptr_t)(tile + (cw + AP_WAVES * rep) * 64), 16, 0, 0);
#pragma unroll
        for (int rep = 0; rep < VREP; ++rep)
            __builtin_amdgcn_global_load_lds((global_ptr_t)(vb + v_step[rep]),
                                             (lds_ptr_t)(tile + KCHUNKS + (cw + AP_WAVES * rep) * 64), 16, 0, 0);
        return ids.v < 0;
    };
    // After the wave's own loads of round j have landed: clears the values of keys that were never
    // written (above the unit's newest key) or whose page was given back. Each lane mends the chunks
    // it brought in, so no other wave is involved before the barrier.
    auto mend = [&](int j, bool gone, uint4* stage) {
        const int b = block_of(j);
        const bool tail = 32 * b + 31 > hi_g;
        if (!tail && !(window >= 0 && __any(gone))) return;
        uint4* sV = stage + kg * TILE + KCHUNKS;
#pragma unroll
        for (int rep = 0; rep < VREP; ++rep) {
            const int idx = (cw + AP_WAVES * rep) * 64 + lane;
            Frag f;
            f.u = sV[idx];
            if (gone) {
                f.u = uint4{0u, 0u, 0u, 0u};
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (32 * b + 8 * g + e > hi_g) f.s[e] = 0;
            }
            sV[idx] = f.u;
        }
        AP_WAIT_LDS();
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
    full_hi = __builtin_amdgcn_readfirstlane(full_hi);
    full_lo = __builtin_amdgcn_readfirstlane(full_lo);
    bool all_cols = true;
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) all_cols = all_cols && col_ok[ct];
    const bool wave_full = __all(all_cols);

    // the blocks the wave has anything to do with, and those of them that need no mask
    const int bw_hi = (hi_w >> 5) < b1 ? (hi_w >> 5) : b1, bw_lo = lo_w >> 5;
    auto wanted = [&](int j) {
        const int b = block_of(j);
        return b <= bw_hi && b >= bw_lo;
    };
    const int bm_hi = (wave_full && full_hi >= 31) ? (full_hi - 31) >> 5 : -1, bm_lo = (full_lo + 31) >> 5;
    // The operands of a block come from LDS in two parts (keys, values). The walk of four waves asks
    // for them a phase before they are used: the keys of block b + 1 and the values of block b behind
    // block b's score product; the walk of eight waves reads both in front of the block.
    struct KOps {
        Frag kop[2][DS];
    };
    struct VOps {
        Frag vop[DT];
    };
    auto read_k = [&](const uint4* stage, KOps& op) {
        const uint4* sK = stage + kg * TILE;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < DS; ++s) op.kop[t][s].u = sK[(t * DS + s) * 64 + lane];
    };
    auto read_v = [&](const uint4* stage, VOps& op) {
        const uint4* sV = stage + kg * TILE + KCHUNKS;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) op.vop[dt].u = sV[dt * 64 + lane];
    };
    // The two products with the softmax between them. ask_k / ask_v: behind the score product, ask
    // for the keys of the next block (from k_next into op_next) and for this block's values (from
    // v_now into vo_w, which is `vo`).
    auto compute = [&](int j, const KOps& op, const VOps& vo, const uint4* k_next, KOps& op_next, const uint4* v_now, VOps& vo_w, const bool ask_k, const bool ask_v) {
        const int base = 32 * block_of(j);
        const bool masked = block_of(j) > bm_hi || block_of(j) < bm_lo;
        // scores^T for the two 16-key tiles
        float p[NT][2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) {
                floatx4_t sacc = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < DS; ++s)
                    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(op.kop[t][s].v, qop[ct][s].v, sacc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) p[ct][t][r] = sacc[r];
            }
        }
        // (behind the score products, not in front: there the wait for this block's keys could not
        // leave sixteen younger reads in flight, the counter of LDS reads has four bits)
        __builtin_amdgcn_sched_barrier(0);
        if (ask_v) read_v(v_now, vo_w);
        if (ask_k) read_k(k_next, op_next);
        __builtin_amdgcn_sched_barrier(0);
        if (masked) {
#pragma unroll
            for (int ct = 0; ct < NT; ++ct)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = base + 8 * g + 4 * t + r;
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
                acc_o[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vo.vop[dt].v, pop[ct].v, acc_o[ct][dt], 0, 0, 0);
    };

    const int rounds = (b1 - b0 + KW) / KW;    // the same for every wave: they meet at the barriers
    PageIds ids_a, ids_b;
    KOps k_even, k_odd;
    VOps vals;
    if constexpr (KW == 1) {
        // Two rounds to a barrier, the barrier between the two: with blocks j and j + 1 in one pair of
        // stages and j + 2, j + 3 landing in the other,
        //   block j is computed (its values and the keys of j + 1 come from LDS behind its score product);
        //   values of j + 1 are asked for; the wave's loads of the other pair have landed, its reads of
        //   this pair are back: the workgroup meets;
        //   blocks j + 4 and j + 5 are asked for into this pair (nobody reads it any more); block j + 1 is
        //   computed from registers, the keys of j + 2 come from the other pair behind its score product.
        // So the reads from LDS run while a block is computed, and the loads from the pages have two
        // blocks' computation to land. (A block the wave has nothing to do with is computed all the
        // same: every key of it is masked; the walk has no branches around the reads and the products.)
        bool gone_a = false, gone_b = false;
        auto two_rounds = [&](int j, uint4* cur0, uint4* cur1, uint4* nxt0, uint4* nxt1) {
            compute(j, k_even, vals, cur1, k_odd, cur0, vals, true, true);
            read_v(cur1, vals);
            // (asked for here and not a block earlier: 32 columns a wave have no registers to spare
            // for them during the block, and the wait that follows is for the loads of two blocks)
            const PageIds nid_a = page_ids(j + 6), nid_b = page_ids(j + 7);
            AP_WAIT_VMCNT(0);
            if (j + 2 < rounds) {
                mend(j + 2, gone_a, nxt0);
                mend(j + 3, gone_b, nxt1);      // past the walk's end too: the block is computed
            }
            AP_WAIT_LDS();
            __builtin_amdgcn_s_barrier();
            if (j + 4 < rounds) {
                gone_a = fetch(j + 4, ids_a, cur0);
                gone_b = fetch(j + 5, ids_b, cur1);
            }
            ids_a = nid_a;
            ids_b = nid_b;
            compute(j + 1, k_odd, vals, nxt0, k_even, nxt0, vals, true, false);
        };
        {
            const PageIds i0 = page_ids(0), i1 = page_ids(1);
            AP_WAIT_VMCNT(0);
            const bool gone0 = fetch(0, i0, stage0);
            const bool gone1 = fetch(1, i1, stage1);
            ids_a = page_ids(2);
            ids_b = page_ids(3);
            AP_WAIT_VMCNT(0);
            mend(0, gone0, stage0);
            mend(1, gone1, stage1);
            __builtin_amdgcn_s_barrier();
            if (rounds > 2) {
                gone_a = fetch(2, ids_a, stage2);
                gone_b = fetch(3, ids_b, stage3);
            }
            ids_a = page_ids(4);
            ids_b = page_ids(5);
            AP_WAIT_LDS();
            read_k(stage0, k_even);
        }
        for (int j = 0; j < rounds; j += 4) {
            two_rounds(j, stage0, stage1, stage2, stage3);
            if (j + 2 >= rounds) break;
            two_rounds(j + 2, stage2, stage3, stage0, stage1);
        }
        AP_WAIT_VMCNT(0);
        __builtin_amdgcn_s_barrier();
    } else {
        // Two rounds to a barrier: read the operands of round j, ask for rounds j+2 and j+3 (into the
        // pair of stages that was computed last time), compute rounds j and j+1, make sure the loads
        // have landed, meet. The barrier orders the operand reads of a pair before the loads that
        // refill it, and makes every wave's loads visible to the others (each wave has waited for its
        // own). With two blocks between barriers the waves drift apart and one wave's products overlap
        // another's softmax (measured on MI355X against one block per barrier: up to a quarter faster
        // with four waves to a workgroup, the same with eight).
        auto two_rounds = [&](int j, uint4* cur0, uint4* cur1, uint4* nxt0, uint4* nxt1) {
            const bool more = j + 2 < rounds;
            const bool busy0 = wanted(j), busy1 = wanted(j + 1);
            bool gone_a = false, gone_b = false;
            if (busy0) {
                read_k(cur0, k_even);
                read_v(cur0, vals);
            }
            if (more) {
                gone_a = fetch(j + 2, ids_a, nxt0);
                gone_b = fetch(j + 3, ids_b, nxt1);
                ids_a = page_ids(j + 4);
                ids_b = page_ids(j + 5);
            }
            if (busy0) compute(j, k_even, vals, cur0, k_even, cur0, vals, false, false);
            if (busy1) {
                read_k(cur1, k_even);
                read_v(cur1, vals);
                compute(j + 1, k_even, vals, cur1, k_even, cur1, vals, false, false);
            }
            AP_WAIT_VMCNT(0);
            if (more) {
                mend(j + 2, gone_a, nxt0);
                if (j + 3 < rounds) mend(j + 3, gone_b, nxt1);
            }
            __builtin_amdgcn_s_barrier();
        };
        {
            const PageIds i0 = page_ids(0), i1 = page_ids(1);
            const bool gone0 = fetch(0, i0, stage0);
            const bool gone1 = fetch(1, i1, stage1);
            ids_a = page_ids(2);
            ids_b = page_ids(3);
            AP_WAIT_VMCNT(0);
            mend(0, gone0, stage0);
            if (rounds > 1) mend(1, gone1, stage1);
            __builtin_amdgcn_s_barrier();
        }
        for (int j = 0; j < rounds; j += 4) {
            two_rounds(j, stage0, stage1, stage2, stage3);
            if (j + 2 >= rounds) break;
            two_rounds(j + 2, stage2, stage3, stage0, stage1);
        }
    }
    // nothing is in flight any more

    // the sum of a column is spread over the four lane groups
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        l_run[ct] += __shfl_xor(l_run[ct], 16, MV_WAVE);
        l_run[ct] += __shfl_xor(l_run[ct], 32, MV_WAVE);
    }

    if constexpr (KW > 1) {
        // ---- the other key groups hand their partial results to group 0 through LDS, one after the
        // other and one column tile at a time (the tiles are no longer needed: every wave has passed
        // the last barrier of the walk, and nothing is in flight)
        static_assert(sizeof(stage0) >= AP_WAVES * DT * 4 * MV_WAVE * sizeof(float) && sizeof(stage1) >= 2 * AP_WAVES * 16 * sizeof(float),
                      "the stages are too small for the exchange");
        float* xo = reinterpret_cast<float*>(stage0);                    // [AP_WAVES][DT][4][64]
        float* xm = reinterpret_cast<float*>(stage1);                    // [AP_WAVES][16] maxima, then sums
        float* xl = xm + AP_WAVES * 16;
#pragma unroll
        for (int src = 1; src < KW; ++src) {
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) {
                if (src > 1 || ct > 0) __syncthreads();
                if (kg == src) {
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
                    m_run[ct] = m_fin;
                    l_run[ct] = f0 * l_run[ct] + f1 * l1;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            acc_o[ct][dt][r] = f0 * acc_o[ct][dt][r] + f1 * xo[((cw * DT + dt) * 4 + r) * MV_WAVE + lane];
                }
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
            packed.x = f32x2_to_bf16x2_bits(acc_o[ct][dt][0] * inv, acc_o[ct][dt][1] * inv);
            packed.y = f32x2_to_bf16x2_bits(acc_o[ct][dt][2] * inv, acc_o[ct][dt][3] * inv);
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
    // the stages of K and V tiles are static LDS (four of 16 KiB per key group with D = 128)
    hipLaunchKernelGGL((attention_prefill_kernel<D, NT, KW>), grid, dim3(AP_THREADS * KW), 0, stream, (const bf16*)q,
                       q_stride, (bf16*)out, out_stride, (const bf16*)k_pages, (const bf16*)v_pages, block_table,
                       bt_width, page_size, page_shift, positions, cu_seqlens, n_seqs, H, Hkv, scale, window, fold);
    return 0;
}

// nt: column tiles per wave (2 = 128 columns per workgroup, for long prompts; 1 = 64 columns, twice
// the workgroups, for steps too small to fill the chip otherwise).
// kw: key groups per workgroup (2: eight waves, the walk over a unit's keys takes half as many rounds).
// n_units = sum over sequences of ceil(q_len / unit tokens(group, nt)), or an upper bound of it (units
// beyond the step's own end at once); n_busy = the units that hold tokens, as far as the caller knows
// (n_units if it knows no better): it decides how the units are dealt out. grid = (kv heads, units).
extern "C" int mv_attention_prefill(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
                                    const void* v_pages, const int* block_table, int bt_width, int page_size,
                                    const int* positions, const int* cu_seqlens, int n_seqs, int n_units, int n_busy,
                                    int nt, int kw, int H, int Hkv, int D, float scale, int window, hipStream_t stream) {
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
    if (n_busy <= 0 || n_busy > n_units) n_busy = n_units;
    const int fold = (kw == 1 && (long)Hkv * n_busy <= 2L * cus) ? 1 : 0;
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
