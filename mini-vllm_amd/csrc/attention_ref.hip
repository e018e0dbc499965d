// Paged causal attention for any mix of query portions, one workgroup per (token, head).
//
// The query at absolute position p of a request sees the keys of that request at
// positions max(0, p - window) .. p (window < 0: all of them), read from the cache pages
// through the request's block table; the step's own keys are already in the cache when
// this runs. Scores, maximum, sum and the output accumulator are float; keys are visited
// in tiles of 128 starting at the first visible key, so the order of additions depends
// only on the query's position and the window, never on how the step was batched.
//
// Layouts:  K[page][kv_head][slot][d]   V[page][kv_head][d][slot]
// This kernel takes every head size up to 512 and every page size; it is the float32
// path's attention and the fall-back of the bfloat16 path.
#include "dispatch.h"

#define AR_THREADS 128
#define AR_MAX_D 512

template <typename T>
__global__ void __launch_bounds__(AR_THREADS)
attention_ref_kernel(const T* __restrict__ q, long q_stride, T* __restrict__ out, long out_stride,
                     const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                     const int* __restrict__ block_table, int bt_width, int page_size,
                     const int* __restrict__ positions, const int* __restrict__ token_seq, int H, int Hkv, int D,
                     float scale, int window) {
    __shared__ float qs[AR_MAX_D];
    __shared__ float ps[AR_THREADS];
    __shared__ long voff[AR_THREADS];
    __shared__ float scratch[17];

    const int tok = blockIdx.x;
    const int head = blockIdx.y;
    const int tid = threadIdx.x;
    const int seq = token_seq[tok];
    T* o = out + (size_t)tok * out_stride + (size_t)head * D;
    if (seq < 0) {
        for (int d = tid; d < D; d += AR_THREADS) o[d] = from_f<T>(0.f);
        return;
    }
    const int pos = positions[tok];
    const int kvh = head / (H / Hkv);
    const int lo = (window >= 0 && pos - window > 0) ? pos - window : 0;
    const int hi = pos;
    const int* bt = block_table + (size_t)seq * bt_width;

    const T* qrow = q + (size_t)tok * q_stride + (size_t)head * D;
    for (int d = tid; d < D; d += AR_THREADS) qs[d] = to_f(qrow[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[AR_MAX_D / AR_THREADS];
#pragma unroll
    for (int i = 0; i < AR_MAX_D / AR_THREADS; ++i) acc[i] = 0.f;

    for (int base = lo; base <= hi; base += AR_THREADS) {
        const int j = base + tid;
        const bool valid = j <= hi;
        float s = -INFINITY;
        long vo = 0;
        if (valid) {
            const int page = bt[j / page_size];
            const int slot = j % page_size;
            const T* krow = k_pages + (((size_t)page * Hkv + kvh) * page_size + slot) * D;
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f(krow[d]), dot);
            s = dot * scale;
            vo = (long)(((size_t)page * Hkv + kvh) * D) * page_size + slot;
        }
        const float tmax = block_max(s, scratch);
        const float m_new = fmaxf(m, tmax);
        const float p = valid ? expf(s - m_new) : 0.f;
        ps[tid] = p;
        voff[tid] = vo;
        const float tsum = block_sum(p, scratch);  // its barriers also publish ps and voff
        const float corr = expf(m - m_new);        // first tile: exp(-inf) = 0
        l = l * corr + tsum;
        m = m_new;
        const int cnt = (hi - base + 1) < AR_THREADS ? (hi - base + 1) : AR_THREADS;
#pragma unroll
        for (int i = 0; i < AR_MAX_D / AR_THREADS; ++i) {
            const int d = tid + i * AR_THREADS;
            if (d < D) {
                float a = acc[i] * corr;
                for (int jj = 0; jj < cnt; ++jj)
                    a = fmaf(ps[jj], to_f(v_pages[voff[jj] + (long)d * page_size]), a);
                acc[i] = a;
            }
        }
        __syncthreads();
    }
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < AR_MAX_D / AR_THREADS; ++i) {
        const int d = tid + i * AR_THREADS;
        if (d < D) o[d] = from_f<T>(acc[i] * inv);
    }
}

extern "C" int mv_attention_ref(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
                                const void* v_pages, const int* block_table, int bt_width, int page_size,
                                const int* positions, const int* token_seq, int n, int H, int Hkv, int D,
                                float scale, int window, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && Hkv > 0 && D > 0, "attention: bad sizes n=%d H=%d Hkv=%d D=%d", n, H, Hkv, D);
    MV_REQUIRE(H % Hkv == 0, "attention: %d query heads are not a multiple of %d key/value heads", H, Hkv);
    MV_REQUIRE(D <= AR_MAX_D, "attention: head_dim %d exceeds the supported maximum %d", D, AR_MAX_D);
    MV_REQUIRE(page_size > 0 && bt_width > 0, "attention: bad page size %d or block table width %d", page_size,
               bt_width);
    MV_REQUIRE(q_stride >= (long)H * D && out_stride >= (long)H * D, "attention: row strides too small");
    MV_REQUIRE(H <= 65535, "attention: too many heads %d", H);
    if (n == 0) return 0;
    MV_DISPATCH_T(dtype, "attention",
                  hipLaunchKernelGGL(attention_ref_kernel<T>, dim3(n, H), dim3(AR_THREADS), 0, stream, (const T*)q,
                                     q_stride, (T*)out, out_stride, (const T*)k_pages, (const T*)v_pages,
                                     block_table, bt_width, page_size, positions, token_seq, H, Hkv, D, scale,
                                     window));
    return mv_check_launch("attention");
}
