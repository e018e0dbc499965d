// Paged causal attention on the MFMA units of gfx950, bf16 in and out, float inside.
//
// A workgroup serves one key/value head of one "unit": a run of consecutive query tokens of one
// sequence. The unit's (token, query head of the group) pairs are the columns of the problem;
// with grouped heads the keys and values are read once for the whole group.
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
// Two ways to share the work inside a workgroup of four waves:
//   SPLIT_KEYS   (decode: at most 16*NT columns) the waves take the 32-key blocks in turn and
//                their partial results are merged through LDS; with nsplit > 1 several
//                workgroups split the keys further and a second kernel merges their partials.
//   otherwise    (prompt portions) each wave owns 16*NT columns and walks all their keys.
//
// Layouts: K[page][kv_head][slot][d], V[page][kv_head][d][slot]; the page size is a multiple of
// 16. Keys outside a column's range (above its position, or more than `window` below it) get
// probability zero; value slots that were never written are read as zero.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    uint2 h[2];
    uint16_t s[8];
    bf16x8_t v;
};

#define AF_WAVES 4
#define LOG2E 1.4426950408889634f

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

template <int D, int NT, bool SPLIT_KEYS>
__global__ void __launch_bounds__(64 * AF_WAVES)
attention_mfma_kernel(const bf16* __restrict__ q, long q_stride, bf16* __restrict__ out, long out_stride,
                      const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                      const int* __restrict__ block_table, int bt_width, int page_size,
                      const int* __restrict__ positions, const int* __restrict__ cu_seqlens, int n_seqs,
                      int decode_only, int H, int Hkv, float scale, int window, float* __restrict__ partials,
                      int nsplit) {
    constexpr int DS = D / 32;
    constexpr int DT = D / 16;
    constexpr int COLS = (SPLIT_KEYS ? 16 : 16 * AF_WAVES) * NT;  // columns of a workgroup
    const int G = H / Hkv;
    const int kvh = blockIdx.y;
    const int split = blockIdx.z;
    const int wave = threadIdx.x / MV_WAVE;
    const int lane = threadIdx.x % MV_WAVE;
    const int i = lane % 16;
    const int g = lane / 16;
    const int tpu = COLS / G;  // tokens of a unit (the host made sure it is >= 1)

    __shared__ int sh_unit[3];
    if (threadIdx.x == 0) {
        int seq = -1, t0 = 0, nt = 0;
        if (decode_only) {
            seq = blockIdx.x;
            t0 = cu_seqlens[seq];
            nt = cu_seqlens[seq + 1] - t0;
            if (nt > tpu) nt = tpu;
        } else {
            int u = blockIdx.x;
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
        const int col = ((SPLIT_KEYS ? 0 : wave * NT) + ct) * 16 + i;
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
    hi_w = wave_max_i(hi_w);
    lo_w = wave_min_i(lo_w);

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
        if (SPLIT_KEYS) {
            const int nblocks = b1 - b0 + 1;
            const int per = (nblocks + nsplit - 1) / nsplit;
            b_begin = b0 + split * per + wave;
            b_end = b0 + (split + 1) * per;
            if (b_end > b1 + 1) b_end = b1 + 1;
            b_step = AF_WAVES;
        } else {
            b_begin = b0;
            b_end = b1 + 1;
        }
    }
    const float sc_mul = scale * LOG2E;

    // Pages and operands of a block. K operands are fetched one block ahead and V operands
    // before the scores are computed, so that their latency hides behind the MFMA work.
    auto block_pages = [&](int b, int* page, int* slot0) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key0 = 32 * b + 16 * t;
            const int pidx = key0 / page_size;
            page[t] = (b < b_end && key0 <= hi_w && pidx < bt_width) ? bt[pidx] : -1;
            slot0[t] = key0 % page_size;
        }
    };
    auto load_k = [&](const int* page, const int* slot0, Frag (*kop)[DS]) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (page[t] >= 0) {
                const bf16* kptr =
                    k_pages + (((size_t)page[t] * Hkv + kvh) * page_size + slot0[t] + i) * D + 8 * g;
#pragma unroll
                for (int s = 0; s < DS; ++s) kop[t][s].u = *reinterpret_cast<const uint4*>(kptr + 32 * s);
            } else {
#pragma unroll
                for (int s = 0; s < DS; ++s) kop[t][s].u = uint4{0u, 0u, 0u, 0u};
            }
        }
    };

    int page[2], slot0[2];
    Frag kop[2][DS];
    block_pages(b_begin, page, slot0);
    load_k(page, slot0, kop);

    for (int b = b_begin; b < b_end; b += b_step) {
        const int base = 32 * b;
        // V^T operands of this block
        Frag vop[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                if (page[t] >= 0) {
                    const bf16* vptr = v_pages + (((size_t)page[t] * Hkv + kvh) * D + 16 * dt + i) * page_size +
                                       slot0[t] + 4 * g;
                    vop[dt].h[t] = *reinterpret_cast<const uint2*>(vptr);
                } else {
                    vop[dt].h[t] = uint2{0u, 0u};
                }
            }
        }
        // K operands of the next block
        int npage[2], nslot0[2];
        Frag knext[2][DS];
        block_pages(b + b_step, npage, nslot0);
        load_k(npage, nslot0, knext);

        // scores^T for two tiles of 16 keys
        float p[NT][2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            floatx4_t sacc[NT];
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) sacc[ct] = floatx4_t{0.f, 0.f, 0.f, 0.f};
            if (page[t] >= 0) {
#pragma unroll
                for (int ct = 0; ct < NT; ++ct)
#pragma unroll
                    for (int s = 0; s < DS; ++s)
                        sacc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[t][s].v, qop[ct][s].v, sacc[ct], 0, 0, 0);
            }
#pragma unroll
            for (int ct = 0; ct < NT; ++ct)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = base + 16 * t + 4 * g + r;
                    const bool ok = page[t] >= 0 && col_ok[ct] && key <= col_pos[ct] && key >= col_lo[ct];
                    p[ct][t][r] = ok ? sacc[ct][r] * sc_mul : -INFINITY;
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
            mx = fmaxf(mx, __shfl_xor(mx, 16, MV_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, MV_WAVE));
            const float m_new = fmaxf(m_run[ct], mx);
            const float corr = (m_new == -INFINITY) ? 1.f : exp2f(m_run[ct] - m_new);
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float e = (p[ct][t][r] == -INFINITY) ? 0.f : exp2f(p[ct][t][r] - m_new);
                    psum += e;
                    pop[ct].v[t * 4 + r] = (__bf16)e;
                }
            l_run[ct] = l_run[ct] * corr + psum;
            m_run[ct] = m_new;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) acc_o[ct][dt] *= corr;
        }
        // out^T += V^T P^T
        if (base + 31 > hi_w) {  // slots above the newest key were never written
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (base + 16 * t + 4 * g + r > hi_w) vop[dt].s[t * 4 + r] = 0;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int ct = 0; ct < NT; ++ct)
                acc_o[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[dt].v, pop[ct].v, acc_o[ct][dt], 0, 0, 0);
        // the prefetched block becomes the current one
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            page[t] = npage[t];
            slot0[t] = nslot0[t];
#pragma unroll
            for (int s = 0; s < DS; ++s) kop[t][s] = knext[t][s];
        }
    }

    // the sum of a column is spread over the four lane groups
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        l_run[ct] += __shfl_xor(l_run[ct], 16, MV_WAVE);
        l_run[ct] += __shfl_xor(l_run[ct], 32, MV_WAVE);
    }

    if (!SPLIT_KEYS) {
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
        return;
    }

    // ---- merge the four waves' partial results (same columns, disjoint keys)
    __shared__ float sm_m[AF_WAVES][NT][16];
    __shared__ float sm_l[AF_WAVES][NT][16];
    __shared__ float sm_o[AF_WAVES][NT][DT][4][MV_WAVE];
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        if (g == 0) {
            sm_m[wave][ct][i] = m_run[ct];
            sm_l[wave][ct][i] = l_run[ct];
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) sm_o[wave][ct][dt][r][lane] = acc_o[ct][dt][r];
    }
    __syncthreads();
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        float m_fin = -INFINITY;
#pragma unroll
        for (int w = 0; w < AF_WAVES; ++w) m_fin = fmaxf(m_fin, sm_m[w][ct][i]);
        float f[AF_WAVES], l_fin = 0.f;
#pragma unroll
        for (int w = 0; w < AF_WAVES; ++w) {
            const float mw = sm_m[w][ct][i];
            f[w] = (mw == -INFINITY) ? 0.f : exp2f(mw - m_fin);
            l_fin += f[w] * sm_l[w][ct][i];
        }
        if (!col_ok[ct]) continue;
        // the d tiles are dealt out to the waves
        for (int dt = wave; dt < DT; dt += AF_WAVES) {
            float o[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float a = 0.f;
#pragma unroll
                for (int w = 0; w < AF_WAVES; ++w) a += f[w] * sm_o[w][ct][dt][r][lane];
                o[r] = a;
            }
            if (nsplit == 1) {
                const float inv = 1.f / l_fin;
                bf16* orow = out + (size_t)col_tok[ct] * out_stride + (size_t)col_head[ct] * D;
                uint2 packed;
                packed.x = (uint32_t)f32_to_bf16_bits(o[0] * inv) | ((uint32_t)f32_to_bf16_bits(o[1] * inv) << 16);
                packed.y = (uint32_t)f32_to_bf16_bits(o[2] * inv) | ((uint32_t)f32_to_bf16_bits(o[3] * inv) << 16);
                *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * g) = packed;
            } else {
                float* prow = partials + (((size_t)col_tok[ct] * H + col_head[ct]) * nsplit + split) * (D + 2);
#pragma unroll
                for (int r = 0; r < 4; ++r) prow[16 * dt + 4 * g + r] = o[r];
            }
        }
        if (nsplit > 1 && wave == 0 && g == 0) {
            float* prow = partials + (((size_t)col_tok[ct] * H + col_head[ct]) * nsplit + split) * (D + 2);
            prow[D] = m_fin;
            prow[D + 1] = l_fin;
        }
    }
}

// Merges the partial results of the key splits: out[token][head] = sum_z o_z 2^(m_z - m) / l.
#define AF_MAX_SPLITS 64
__global__ void attention_merge_kernel(const float* __restrict__ partials, bf16* __restrict__ out, long out_stride,
                                       const int* __restrict__ token_seq, int H, int D, int nsplit) {
    __shared__ float sh_m[AF_MAX_SPLITS], sh_w[AF_MAX_SPLITS];
    const int tok = blockIdx.x, head = blockIdx.y;
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

template <int D, int NT, bool SPLIT_KEYS>
static void launch_attention(dim3 grid, hipStream_t stream, const void* q, long q_stride, void* out, long out_stride,
                             const void* k_pages, const void* v_pages, const int* block_table, int bt_width,
                             int page_size, const int* positions, const int* cu_seqlens, int n_seqs, int decode_only,
                             int H, int Hkv, float scale, int window, float* partials, int nsplit) {
    hipLaunchKernelGGL((attention_mfma_kernel<D, NT, SPLIT_KEYS>), grid, dim3(64 * AF_WAVES), 0, stream,
                       (const bf16*)q, q_stride, (bf16*)out, out_stride, (const bf16*)k_pages, (const bf16*)v_pages,
                       block_table, bt_width, page_size, positions, cu_seqlens, n_seqs, decode_only, H, Hkv, scale,
                       window, partials, nsplit);
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

// Decode steps: every sequence brings one token. grid = (sequences, kv heads, nsplit).
// partials: float [n_seqs * H * nsplit * (D + 2)], needed when nsplit > 1.
extern "C" int mv_attention_decode(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
                                   const void* v_pages, const int* block_table, int bt_width, int page_size,
                                   const int* positions, const int* cu_seqlens, int n_seqs, int H, int Hkv, int D,
                                   float scale, int window, float* partials, int nsplit, const int* token_seq,
                                   hipStream_t stream) {
    if (int rc = check_common("attention_decode", q_stride, out_stride, page_size, bt_width, H, Hkv, D)) return rc;
    MV_REQUIRE(H / Hkv <= 16, "attention_decode: %d query heads per kv head exceed 16", H / Hkv);
    MV_REQUIRE(nsplit >= 1 && nsplit <= AF_MAX_SPLITS && (nsplit == 1 || partials != nullptr),
               "attention_decode: bad split count %d or missing work area", nsplit);
    if (n_seqs <= 0) return 0;
    dim3 grid(n_seqs, Hkv, nsplit);
    if (D == 128)
        launch_attention<128, 1, true>(grid, stream, q, q_stride, out, out_stride, k_pages, v_pages, block_table,
                                       bt_width, page_size, positions, cu_seqlens, n_seqs, 1, H, Hkv, scale, window,
                                       partials, nsplit);
    else
        launch_attention<64, 1, true>(grid, stream, q, q_stride, out, out_stride, k_pages, v_pages, block_table,
                                      bt_width, page_size, positions, cu_seqlens, n_seqs, 1, H, Hkv, scale, window,
                                      partials, nsplit);
    if (int rc = mv_check_launch("attention_decode")) return rc;
    if (nsplit > 1) {
        hipLaunchKernelGGL(attention_merge_kernel, dim3(n_seqs, H), dim3(D >= 128 ? 128 : 64), 0, stream, partials,
                           (bf16*)out, out_stride, token_seq, H, D, nsplit);
        return mv_check_launch("attention_merge");
    }
    return 0;
}

