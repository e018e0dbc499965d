// Row-wise kernels of the decoder: embedding gather, residual add fused with RMS
// normalisation, rotary table, per-head q/k norm + rotary embedding + cache write, SwiGLU.
// All arithmetic is float; T is the storage type of activations and cache pages. The
// residual stream is always float.
#include "dispatch.h"

// ---------------------------------------------------------------------------------------
// Embedding: resid[n, :] = table[ids[n], :] * scale        (float residual stream)
// ---------------------------------------------------------------------------------------
__global__ void embedding_kernel(const int* __restrict__ ids, WeightPtr table, float* __restrict__ resid,
                                 int h, int vocab, float scale) {
    const int row = blockIdx.x;
    const int id = ids[row];
    const bool valid = id >= 0 && id < vocab;
    float* dst = resid + (size_t)row * h;
    const size_t base = (size_t)(valid ? id : 0) * h;
    for (int d = threadIdx.x; d < h; d += blockDim.x) dst[d] = valid ? table.at(base + d) * scale : 0.f;
}

extern "C" int mv_embedding(const int* ids, const void* table, int table_dtype, float* resid, int n, int h,
                            int vocab, float scale, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && h > 0 && vocab > 0, "embedding: bad sizes n=%d h=%d vocab=%d", n, h, vocab);
    MV_REQUIRE(mv_valid_dtype(table_dtype), "embedding: bad table dtype %d", table_dtype);
    if (n == 0) return 0;
    WeightPtr w{table, table_dtype};
    hipLaunchKernelGGL(embedding_kernel, dim3(n), dim3(256), 0, stream, ids, w, resid, h, vocab, scale);
    return mv_check_launch("embedding");
}

// The embedding and, in the same launch, a second gather of float rows: out2[n, :] = table2[ids2[n], :]
// (the rows of a position table at the step's positions, say). The first kernel of a step carries it,
// so that it costs no launch of its own.
__global__ void embedding_gather_kernel(const int* __restrict__ ids, WeightPtr table, float* __restrict__ resid, int h,
                                        int vocab, float scale, const int* __restrict__ ids2,
                                        const float* __restrict__ table2, float* __restrict__ out2, int h2, int rows2) {
    const int row = blockIdx.x;
    if (blockIdx.y == 0) {
        const int id = ids[row];
        const bool valid = id >= 0 && id < vocab;
        float* dst = resid + (size_t)row * h;
        const size_t base = (size_t)(valid ? id : 0) * h;
        for (int d = threadIdx.x; d < h; d += blockDim.x) dst[d] = valid ? table.at(base + d) * scale : 0.f;
    } else {
        const int id = ids2[row];
        const bool valid = id >= 0 && id < rows2;
        const float* src = table2 + (size_t)(valid ? id : 0) * h2;
        float* dst = out2 + (size_t)row * h2;
        for (int d = threadIdx.x; d < h2; d += blockDim.x) dst[d] = valid ? src[d] : 0.f;
    }
}

extern "C" int mv_embedding_gather(const int* ids, const void* table, int table_dtype, float* resid, int n, int h,
                                   int vocab, float scale, const int* ids2, const float* table2, float* out2, int h2,
                                   int rows2, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && h > 0 && vocab > 0, "embedding: bad sizes n=%d h=%d vocab=%d", n, h, vocab);
    MV_REQUIRE(mv_valid_dtype(table_dtype), "embedding: bad table dtype %d", table_dtype);
    MV_REQUIRE(ids2 != nullptr && table2 != nullptr && out2 != nullptr && h2 > 0 && rows2 > 0,
               "embedding: the second gather needs ids, a table of %d rows of %d and an output", rows2, h2);
    if (n == 0) return 0;
    WeightPtr w{table, table_dtype};
    hipLaunchKernelGGL(embedding_gather_kernel, dim3(n, 2), dim3(256), 0, stream, ids, w, resid, h, vocab, scale, ids2,
                       table2, out2, h2, rows2);
    return mv_check_launch("embedding_gather");
}

// Eight consecutive elements, read and written 16 bytes (bf16) or 32 bytes (float) at a time.
template <typename T> struct Vec8;
template <> struct Vec8<bf16> {
    static __device__ __forceinline__ void load(const bf16* p, float (&x)[8]) {
        const uint4 u = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x[2 * e] = __uint_as_float(w[e] << 16);
            x[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void store(bf16* p, const float (&x)[8]) {
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            w[e] = f32x2_to_bf16x2_bits(x[2 * e], x[2 * e + 1]);
        *reinterpret_cast<uint4*>(p) = uint4{w[0], w[1], w[2], w[3]};
    }
};
template <> struct Vec8<float> {
    static __device__ __forceinline__ void load(const float* p, float (&x)[8]) {
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&x)[8]) {
        *reinterpret_cast<float4*>(p) = float4{x[0], x[1], x[2], x[3]};
        *reinterpret_cast<float4*>(p + 4) = float4{x[4], x[5], x[6], x[7]};
    }
};

// ---------------------------------------------------------------------------------------
// Residual add + RMSNorm.
//   rows == null : for every row r: v = resid[r] + delta[r]; resid[r] = v; out[r] = norm(v) * w
//   rows != null : for i < n_out, r = rows[i]: v = resid[r] + delta[r]; out[i] = norm(v) * w
//                  (resid is left as it is; a negative row gives zeros)
//   delta == null: nothing is added.  out == null: only the add is done.
//   norm(v) = v / sqrt(mean(v^2) + eps);  weight is w, or 1 + w with unit_offset.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const T* __restrict__ delta, WeightPtr w, float eps,
                                   int unit_offset, T* __restrict__ out, const int* __restrict__ rows, int h) {
    __shared__ float scratch[17];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    if (r < 0) {
        if (out)
            for (int d = threadIdx.x; d < h; d += blockDim.x) out[(size_t)i * h + d] = from_f<T>(0.f);
        return;
    }
    float* x = resid + (size_t)r * h;
    const T* dl = delta ? delta + (size_t)r * h : nullptr;
    float ss = 0.f;
    if (out) {
        for (int d = threadIdx.x; d < h; d += blockDim.x) {
            float v = x[d];
            if (dl) v += to_f(dl[d]);
            ss += v * v;
        }
        ss = block_sum(ss, scratch);
    }
    const float rinv = out ? rsqrtf(ss / (float)h + eps) : 0.f;
    const bool write_back = (rows == nullptr) && (dl != nullptr);
    for (int d = threadIdx.x; d < h; d += blockDim.x) {
        float v = x[d];
        if (dl) v += to_f(dl[d]);
        if (write_back) x[d] = v;
        if (out) {
            float wt = w.at(d);
            if (unit_offset) wt += 1.f;
            out[(size_t)i * h + d] = from_f<T>(v * rinv * wt);
        }
    }
}

// The same with rows of a multiple of 8 columns, at most 8192: TPR threads share a row (a block
// of 256 serves 256 / TPR rows), each keeps its chunks of eight columns in registers between the
// sum of squares and the scaling, so a row is read once.
#define ARN_MAX_CHUNKS 4
// A delta that is still the partial sums of a product whose K was split over workgroups:
// delta[m][n] = round_T(sum over f < F of part[f * plane + m * h + n] (+ bias[n])), the sum taken
// in that order and rounded to the activation type as the kernel that adds them up would.
struct SplitDelta {
    const float* part;
    int F;
    long plane;
    const bf16* bias;
};

// SPLIT: the delta is given as `split` (then `delta` is null); a variant of its own, so that the
// plain one keeps its few registers.
template <typename T, bool SPLIT>
__global__ void __launch_bounds__(256)
add_rmsnorm_vec_kernel(float* __restrict__ resid, const T* __restrict__ delta, SplitDelta split, WeightPtr w,
                       float eps, int unit_offset, T* __restrict__ out, const int* __restrict__ rows, int n_out, int h,
                       int tpr) {
    __shared__ float part[256 / MV_WAVE];
    const int rpb = 256 / tpr;                        // rows of this block
    const int sub = threadIdx.x / tpr, t = threadIdx.x % tpr;
    const int i = blockIdx.x * rpb + sub;
    const bool live = i < n_out;
    const int r = live ? (rows ? rows[i] : i) : -1;
    float x[ARN_MAX_CHUNKS][8];
    float ss = 0.f;
    // the partial sums of a split product first: four planes of all the thread's chunks are asked
    // for at a time (the loads of one plane after the other would each wait for the last), and
    // added in the order of the planes
    float sum[SPLIT ? ARN_MAX_CHUNKS : 1][8];
    if (SPLIT && r >= 0) {
#pragma unroll
        for (int c = 0; c < ARN_MAX_CHUNKS; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) sum[c][e] = 0.f;
        const float* pr = split.part + (size_t)r * h;
        for (int f0 = 0; f0 < split.F; f0 += 4) {
            float dv[4][ARN_MAX_CHUNKS][8];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int c = 0; c < ARN_MAX_CHUNKS; ++c) {
                    const int d = (c * tpr + t) * 8;
                    if (d < h && f0 + u < split.F) {
                        Vec8<float>::load(pr + (size_t)(f0 + u) * split.plane + d, dv[u][c]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) dv[u][c][e] = 0.f;   // (adding +0 changes nothing)
                    }
                }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int c = 0; c < ARN_MAX_CHUNKS; ++c)
#pragma unroll
                    for (int e = 0; e < 8; ++e) sum[c][e] += dv[u][c][e];
        }
    }
    if (r >= 0) {
        float* xr = resid + (size_t)r * h;
        const T* dl = delta ? delta + (size_t)r * h : nullptr;
#pragma unroll
        for (int c = 0; c < ARN_MAX_CHUNKS; ++c) {
            const int d = (c * tpr + t) * 8;
            if (d < h) {
                Vec8<float>::load(xr + d, x[c]);
                if (dl) {
                    float dv[8];
                    Vec8<T>::load(dl + d, dv);
#pragma unroll
                    for (int e = 0; e < 8; ++e) x[c][e] += dv[e];
                } else if (SPLIT) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        float v = sum[SPLIT ? c : 0][e];
                        if (split.bias) v += to_f(split.bias[d + e]);
                        x[c][e] += to_f(from_f<T>(v));
                    }
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) ss += x[c][e] * x[c][e];
            }
        }
    }
    ss = wave_sum(ss);
    if (tpr > MV_WAVE) {                              // a row spans several waves
        if (threadIdx.x % MV_WAVE == 0) part[threadIdx.x / MV_WAVE] = ss;
        __syncthreads();
        const int w0 = sub * (tpr / MV_WAVE);
        ss = 0.f;
        for (int k = 0; k < tpr / MV_WAVE; ++k) ss += part[w0 + k];
    }
    if (!live) return;
    if (r < 0) {
        if (out) {
            const float zero[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int d = t * 8; d < h; d += tpr * 8) Vec8<T>::store(out + (size_t)i * h + d, zero);
        }
        return;
    }
    const float rinv = rsqrtf(ss / (float)h + eps);
    const bool write_back = rows == nullptr && (delta != nullptr || SPLIT);
#pragma unroll
    for (int c = 0; c < ARN_MAX_CHUNKS; ++c) {
        const int d = (c * tpr + t) * 8;
        if (d < h) {
            if (write_back) Vec8<float>::store(resid + (size_t)r * h + d, x[c]);
            if (out) {
                float wt[8], y[8];
                w.at8(d, wt);
#pragma unroll
                for (int e = 0; e < 8; ++e) y[e] = x[c][e] * rinv * (unit_offset ? wt[e] + 1.f : wt[e]);
                Vec8<T>::store(out + (size_t)i * h + d, y);
            }
        }
    }
}

extern "C" int mv_add_rmsnorm(float* resid, const void* delta, const void* weight, int weight_dtype, float eps,
                              int unit_offset, void* out, const int* rows, int n_out, int h, int dtype,
                              hipStream_t stream) {
    MV_REQUIRE(n_out >= 0 && h > 0, "add_rmsnorm: bad sizes n=%d h=%d", n_out, h);
    MV_REQUIRE(out == nullptr || weight != nullptr, "add_rmsnorm: norm asked without a weight");
    MV_REQUIRE(mv_valid_dtype(weight_dtype), "add_rmsnorm: bad weight dtype %d", weight_dtype);
    MV_REQUIRE(eps > 0.f || out == nullptr, "add_rmsnorm: eps must be positive");
    if (n_out == 0) return 0;
    WeightPtr w{weight, weight_dtype};
    if (out != nullptr && h % 8 == 0 && h <= 8 * 256 * ARN_MAX_CHUNKS && ((uintptr_t)resid % 16) == 0 &&
        ((uintptr_t)delta % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)weight % 16) == 0) {
        // threads per row: a power of two of at least 64 that covers the row in ARN_MAX_CHUNKS chunks or fewer
        int tpr = 64;
        while (tpr < 256 && tpr * 8 * 2 <= h) tpr *= 2;
        const int rpb = 256 / tpr;
        MV_DISPATCH_T(dtype, "add_rmsnorm",
                      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, false>), dim3((n_out + rpb - 1) / rpb), dim3(256), 0, stream,
                                         resid, (const T*)delta, SplitDelta{nullptr, 0, 0, nullptr}, w, eps, unit_offset,
                                         (T*)out, rows, n_out, h, tpr));
        return mv_check_launch("add_rmsnorm");
    }
    MV_DISPATCH_T(dtype, "add_rmsnorm",
                  hipLaunchKernelGGL(add_rmsnorm_kernel<T>, dim3(n_out), dim3(256), 0, stream, resid,
                                     (const T*)delta, w, eps, unit_offset, (T*)out, rows, h));
    return mv_check_launch("add_rmsnorm");
}

// The same with a delta that is still the F partial sums of a product (see SplitDelta): the kernel
// that would add them up and round is saved. Returns 2 (and sets the error text) when the sizes
// are not served by the vector kernel; the caller then adds the sums up first.
extern "C" int mv_add_rmsnorm_split(float* resid, const float* part, int F, long plane, const void* bias,
                                    const void* weight, int weight_dtype, float eps, int unit_offset, void* out,
                                    const int* rows, int n_out, int h, int dtype, hipStream_t stream) {
    MV_REQUIRE(n_out >= 0 && h > 0 && F > 0 && part != nullptr && plane >= (long)h,
               "add_rmsnorm_split: bad sizes n=%d h=%d F=%d", n_out, h, F);
    MV_REQUIRE(out != nullptr && weight != nullptr, "add_rmsnorm_split: the norm's output and weight are needed");
    MV_REQUIRE(mv_valid_dtype(weight_dtype), "add_rmsnorm_split: bad weight dtype %d", weight_dtype);
    MV_REQUIRE(eps > 0.f, "add_rmsnorm_split: eps must be positive");
    if (n_out == 0) return 0;
    if (!(h % 8 == 0 && h <= 8 * 256 * ARN_MAX_CHUNKS && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)part % 16) == 0 &&
          (plane * sizeof(float)) % 16 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)weight % 16) == 0)) {
        mv_fail("add_rmsnorm_split: rows of %d are not served", h);
        return 2;
    }
    WeightPtr w{weight, weight_dtype};
    int tpr = 64;
    while (tpr < 256 && tpr * 8 * 2 <= h) tpr *= 2;
    const int rpb = 256 / tpr;
    const SplitDelta split{part, F, plane, (const bf16*)bias};
    MV_DISPATCH_T(dtype, "add_rmsnorm_split",
                  hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, true>), dim3((n_out + rpb - 1) / rpb), dim3(256), 0, stream,
                                     resid, (const T*)nullptr, split, w, eps, unit_offset, (T*)out, rows, n_out, h,
                                     tpr));
    return mv_check_launch("add_rmsnorm_split");
}

// Plain RMSNorm over the last dimension of a strided [n, h] view.
template <typename T>
__global__ void rmsnorm_kernel(const T* __restrict__ in, long in_stride, WeightPtr w, float eps, int unit_offset,
                               T* __restrict__ out, long out_stride, int h) {
    __shared__ float scratch[17];
    const T* x = in + (size_t)blockIdx.x * in_stride;
    T* y = out + (size_t)blockIdx.x * out_stride;
    float ss = 0.f;
    for (int d = threadIdx.x; d < h; d += blockDim.x) {
        float v = to_f(x[d]);
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float rinv = rsqrtf(ss / (float)h + eps);
    for (int d = threadIdx.x; d < h; d += blockDim.x) {
        float wt = w.at(d);
        if (unit_offset) wt += 1.f;
        y[d] = from_f<T>(to_f(x[d]) * rinv * wt);
    }
}

extern "C" int mv_rmsnorm(const void* in, long in_stride, const void* weight, int weight_dtype, float eps,
                          int unit_offset, void* out, long out_stride, int n, int h, int dtype,
                          hipStream_t stream) {
    MV_REQUIRE(n >= 0 && h > 0, "rmsnorm: bad sizes n=%d h=%d", n, h);
    MV_REQUIRE(in_stride >= h && out_stride >= h, "rmsnorm: row strides %ld/%ld shorter than h=%d", in_stride,
               out_stride, h);
    MV_REQUIRE(mv_valid_dtype(weight_dtype), "rmsnorm: bad weight dtype %d", weight_dtype);
    MV_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive");
    if (n == 0) return 0;
    WeightPtr w{weight, weight_dtype};
    const int threads = h >= 256 ? 256 : 64;
    MV_DISPATCH_T(dtype, "rmsnorm",
                  hipLaunchKernelGGL(rmsnorm_kernel<T>, dim3(n), dim3(threads), 0, stream, (const T*)in, in_stride,
                                     w, eps, unit_offset, (T*)out, out_stride, h));
    return mv_check_launch("rmsnorm");
}

// ---------------------------------------------------------------------------------------
// Rows that a product left weighted but not yet normalised (gemm_skinny.hip, the FOLD variant):
//   out[m][k] = weighted[m][k] / sqrt(sum_p partial[m][p] / width + eps).
// For whatever comes behind such a norm and does not divide its own output rows. The partial
// sums are added in the order the SCALED product adds them (it depends on their number alone).
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void scale_rows_kernel(const T* __restrict__ weighted, long ldw, const float* __restrict__ partial, int P,
                                  float eps, T* __restrict__ out, long ldo, int width) {
    __shared__ float sh_rinv;
    const int m = blockIdx.x;
    if (threadIdx.x < MV_WAVE) {
        float t = 0.f;
        if (P <= 64) {
            if (threadIdx.x < 8)
                for (int p = threadIdx.x; p < P; p += 8) t += partial[(size_t)m * P + p];
            t += __shfl_xor(t, 1, MV_WAVE);
            t += __shfl_xor(t, 2, MV_WAVE);
            t += __shfl_xor(t, 4, MV_WAVE);
        } else {
            for (int p = threadIdx.x; p < P; p += MV_WAVE) t += partial[(size_t)m * P + p];
            t = wave_sum(t);
        }
        if (threadIdx.x == 0) sh_rinv = rsqrtf(t / (float)width + eps);
    }
    __syncthreads();
    const float rinv = sh_rinv;
    for (int k = threadIdx.x; k < width; k += blockDim.x)
        out[(size_t)m * ldo + k] = from_f<T>(to_f(weighted[(size_t)m * ldw + k]) * rinv);
}

extern "C" int mv_scale_rows(const void* weighted, long ldw, const float* partial, int P, float eps, void* out, long ldo,
                             int dtype, int M, int width, hipStream_t stream) {
    MV_REQUIRE(M >= 0 && width > 0 && P > 0 && eps > 0.f && ldw >= width && ldo >= width,
               "scale_rows: bad sizes M=%d width=%d P=%d", M, width, P);
    MV_REQUIRE(weighted != nullptr && partial != nullptr && out != nullptr, "scale_rows: null argument");
    if (M == 0) return 0;
    MV_DISPATCH_T(dtype, "scale_rows",
                    hipLaunchKernelGGL(scale_rows_kernel<T>, dim3(M), dim3(256), 0, stream, (const T*)weighted, ldw,
                                       partial, P, eps, (T*)out, ldo, width));
    return mv_check_launch("scale_rows");
}

// ---------------------------------------------------------------------------------------
// Rotary table: table[pos, 0:R/2] = cos(pos * inv_freq), table[pos, R/2:R] = sin(...).
// The angle is the float product of the float position and the float inverse frequency.
// ---------------------------------------------------------------------------------------
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, float* __restrict__ table, int max_pos,
                                  int half) {
    const int pos = blockIdx.x;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        const float ang = (float)pos * inv_freq[i];
        table[(size_t)pos * 2 * half + i] = cosf(ang);
        table[(size_t)pos * 2 * half + half + i] = sinf(ang);
    }
}

extern "C" int mv_rope_table(const float* inv_freq, float* table, int max_pos, int rot_dim, hipStream_t stream) {
    MV_REQUIRE(max_pos > 0 && rot_dim > 0 && rot_dim % 2 == 0, "rope_table: bad sizes max_pos=%d rot_dim=%d",
               max_pos, rot_dim);
    hipLaunchKernelGGL(rope_table_kernel, dim3(max_pos), dim3(64), 0, stream, inv_freq, table, max_pos,
                       rot_dim / 2);
    return mv_check_launch("rope_table");
}

// ---------------------------------------------------------------------------------------
// Per-head q/k RMSNorm + rotary embedding + cache write, one wave per (token, head).
//   q heads: normalised and rotated in place in the qkv rows.
//   k heads: normalised, rotated, written to the key page   K[page][kv_head][slot][d].
//   v heads: copied to the value page (transposed)            V[page][kv_head][d][slot].
// page = block_table[seq, pos / page_size], slot = pos % page_size. Rows of padding
// (token_seq < 0) and unmapped pages (< 0) are skipped.
// Rotation pairs: half-split (p, p + R/2) or interleaved (2p, 2p + 1), p < R/2; elements
// at or beyond R pass through.
// ---------------------------------------------------------------------------------------
#define MV_MAX_HEAD_DIM 512

template <typename T>
__global__ void qk_norm_rope_store_kernel(T* __restrict__ qkv, long row_stride, int q_off, int k_off, int v_off,
                                          const int* __restrict__ positions, const int* __restrict__ token_seq,
                                          const int* __restrict__ block_table, int bt_width, int page_size,
                                          T* __restrict__ k_pages, T* __restrict__ v_pages, int H, int Hkv, int D,
                                          WeightPtr qw, WeightPtr kw, int has_norm, float eps, int unit_offset,
                                          const float* __restrict__ table, int rot_dim, int interleaved,
                                          int store_kv) {
    __shared__ float sh[4][MV_MAX_HEAD_DIM];
    const int tok = blockIdx.x;
    const int wave = threadIdx.x / MV_WAVE;
    const int lane = threadIdx.x % MV_WAVE;
    const int head = blockIdx.y * 4 + wave;
    const int total = H + (store_kv == 1 ? 2 * Hkv : (store_kv == 2 ? Hkv : 0));
    const int seq = token_seq[tok];
    const int pos = positions[tok];
    const bool active = head < total && seq >= 0;
    int kind = 0, hh = head;  // 0 q, 1 k, 2 v
    if (head >= H + Hkv) {
        kind = 2;
        hh = head - H - Hkv;
    } else if (head >= H) {
        kind = 1;
        hh = head - H;
    }
    T* row = qkv + (size_t)tok * row_stride;
    T* src = row + (kind == 0 ? q_off : (kind == 1 ? k_off : v_off)) + (size_t)hh * D;
    float* x = sh[wave];

    float ss = 0.f;
    if (active) {
        for (int d = lane; d < D; d += MV_WAVE) {
            const float v = to_f(src[d]);
            x[d] = v;
            ss += v * v;
        }
    }
    ss = wave_sum(ss);
    __syncthreads();
    if (active && kind != 2 && has_norm) {
        const float rinv = rsqrtf(ss / (float)D + eps);
        const WeightPtr& w = kind == 0 ? qw : kw;
        for (int d = lane; d < D; d += MV_WAVE) {
            float wt = w.at(d);
            if (unit_offset) wt += 1.f;
            x[d] = x[d] * rinv * wt;
        }
    }
    __syncthreads();
    if (active && kind != 2 && table != nullptr) {
        const int half = rot_dim / 2;
        const float* cs = table + (size_t)pos * rot_dim;
        for (int p = lane; p < half; p += MV_WAVE) {
            const int i1 = interleaved ? 2 * p : p;
            const int i2 = interleaved ? 2 * p + 1 : p + half;
            const float c = cs[p], s = cs[half + p];
            const float a = x[i1], b = x[i2];
            x[i1] = a * c - b * s;
            x[i2] = b * c + a * s;
        }
    }
    __syncthreads();
    if (!active) return;
    if (kind == 0) {
        for (int d = lane; d < D; d += MV_WAVE) src[d] = from_f<T>(x[d]);
        return;
    }
    const int page = block_table[(size_t)seq * bt_width + pos / page_size];
    if (page < 0) return;
    const int slot = pos % page_size;
    if (kind == 1) {
        T* dst = k_pages + (((size_t)page * Hkv + hh) * page_size + slot) * D;
        for (int d = lane; d < D; d += MV_WAVE) dst[d] = from_f<T>(x[d]);
    } else {
        T* dst = v_pages + ((size_t)page * Hkv + hh) * D * page_size + slot;
        for (int d = lane; d < D; d += MV_WAVE) dst[(size_t)d * page_size] = from_f<T>(x[d]);
    }
}

// The same for the common case (rotation over the whole head in half-split pairs, head size 64,
// 128, 256 or 512): a head is spread over L = D / 8 neighbouring lanes, eight elements each, read
// and written 16 bytes (bf16) at a time; sums and rotation partners travel by lane shuffles, so
// nothing goes through LDS and a wave serves 64 / L heads.
template <typename T, int L, int HP>
__device__ __forceinline__ void
qk_norm_rope_store_vec(long block, T* __restrict__ qkv, long row_stride, int q_off, int k_off, int v_off,
                       const int* __restrict__ positions, const int* __restrict__ token_seq,
                       const int* __restrict__ block_table, int bt_width, int page_size,
                       T* __restrict__ k_pages, T* __restrict__ v_pages, int n, int H, int Hkv,
                       WeightPtr qw, WeightPtr kw, int has_norm, float eps, int unit_offset,
                       const float* __restrict__ table, int store_kv) {
    // A group of L lanes takes HP heads of one token in turn: the token's angles (twice a head's
    // bytes when the table is float) and the norm weights are read once for all of them.
    constexpr int D = 8 * L;
    const int heads = H + (store_kv == 1 ? 2 * Hkv : (store_kv == 2 ? Hkv : 0));
    const int groups = (heads + HP - 1) / HP;    // lane groups of a token
    const long gid = block * blockDim.x + threadIdx.x;
    const long hidx = gid / L;
    const int j = (int)(gid % L);            // this lane's eight elements start at d0 = 8 j
    const int tok = (int)(hidx / groups), head0 = (int)(hidx % groups) * HP;
    const int seq = tok < n ? token_seq[tok] : -1;
    const bool active = tok < n && seq >= 0;
    const int pos = active ? positions[tok] : 0;
    float c[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, sn[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (table != nullptr) {
        const float* cs = table + (size_t)pos * D + 8 * (j % (L / 2));
        const float4 c0 = *reinterpret_cast<const float4*>(cs), c1 = *reinterpret_cast<const float4*>(cs + 4);
        const float4 s0 = *reinterpret_cast<const float4*>(cs + D / 2);
        const float4 s1 = *reinterpret_cast<const float4*>(cs + D / 2 + 4);
        c[0] = c0.x; c[1] = c0.y; c[2] = c0.z; c[3] = c0.w; c[4] = c1.x; c[5] = c1.y; c[6] = c1.z; c[7] = c1.w;
        sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
    }
    float wq[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, wk[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (has_norm) {
        qw.at8(8 * j, wq);
        if (head0 + HP > H) kw.at8(8 * j, wk);   // (a query-only launch may come without key weights)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            wq[e] = unit_offset ? wq[e] + 1.f : wq[e];
            wk[e] = unit_offset ? wk[e] + 1.f : wk[e];
        }
    }
    const bool low = j < L / 2;              // holds d < D/2; its partner d + D/2 sits L/2 lanes on
    int page = -2;                           // the token's page, looked up when the first key or value comes
#pragma unroll
    for (int hp = 0; hp < HP; ++hp) {
        const int head = head0 + hp;
        if (head >= heads) break;            // the same for the whole lane group
        int kind = 0, hh = head;             // 0 q, 1 k, 2 v
        if (head >= H + Hkv) {
            kind = 2;
            hh = head - H - Hkv;
        } else if (head >= H) {
            kind = 1;
            hh = head - H;
        }
        T* src = qkv + (size_t)(active ? tok : 0) * row_stride + (kind == 0 ? q_off : (kind == 1 ? k_off : v_off)) +
                 (size_t)hh * D + 8 * j;
        float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (active) Vec8<T>::load(src, x);
        if (kind != 2) {
            if (has_norm) {
                float ss = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
#pragma unroll
                for (int o = L / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, MV_WAVE);
                const float rinv = rsqrtf(ss / (float)D + eps);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = x[e] * rinv * (kind == 0 ? wq[e] : wk[e]);
            }
            if (table != nullptr) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float other = __shfl_xor(x[e], L / 2, MV_WAVE);
                    x[e] = low ? x[e] * c[e] - other * sn[e] : x[e] * c[e] + other * sn[e];
                }
            }
        }
        if (!active) continue;
        if (kind == 0) {
            Vec8<T>::store(src, x);
            continue;
        }
        if (page == -2) page = block_table[(size_t)seq * bt_width + pos / page_size];
        if (page < 0) continue;
        const int slot = pos % page_size;
        if (kind == 1) {
            Vec8<T>::store(k_pages + (((size_t)page * Hkv + hh) * page_size + slot) * D + 8 * j, x);
        } else {
            T* dst = v_pages + (((size_t)page * Hkv + hh) * D + 8 * j) * page_size + slot;
#pragma unroll
            for (int e = 0; e < 8; ++e) dst[(size_t)e * page_size] = from_f<T>(x[e]);
        }
    }
}

template <typename T, int L, int HP>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_vec_kernel(T* __restrict__ qkv, long row_stride, int q_off, int k_off, int v_off,
                              const int* __restrict__ positions, const int* __restrict__ token_seq,
                              const int* __restrict__ block_table, int bt_width, int page_size,
                              T* __restrict__ k_pages, T* __restrict__ v_pages, int n, int H, int Hkv,
                              WeightPtr qw, WeightPtr kw, int has_norm, float eps, int unit_offset,
                              const float* __restrict__ table, int store_kv) {
    qk_norm_rope_store_vec<T, L, HP>(blockIdx.x, qkv, row_stride, q_off, k_off, v_off, positions, token_seq, block_table,
                                     bt_width, page_size, k_pages, v_pages, n, H, Hkv, qw, kw, has_norm, eps, unit_offset,
                                 table, store_kv);
}

// Value rows of 16 consecutive tokens of the step and one kv head into the transposed value pages
// V[page][kv_head][d][slot]: the rows are staged in LDS and written with the token index running
// fastest over the lanes, so that tokens that follow each other in a sequence fill neighbouring
// slots and the two-byte stores of a wave merge into 32-byte segments (a store per token and
// head scatters them 2 bytes at a time). `tile` has a row pitch of W >= D + 1 floats.
// VEC (the caller vouches for 16-byte aligned rows, D a multiple of 8): the rows come in with one
// 16-byte load a lane, and where eight tokens in a row fill eight neighbouring slots from a slot
// that is a multiple of eight (the usual case inside a prompt) a lane writes those eight values of
// one d with one store instead of eight.
template <typename T, int W, bool VEC = false>
__device__ __forceinline__ void
store_v_tile(int tok0, int kvh, const T* __restrict__ qkv, long row_stride, int v_off,
             const int* __restrict__ positions, const int* __restrict__ token_seq,
             const int* __restrict__ block_table, int bt_width, int page_size, T* __restrict__ v_pages, int n,
             int Hkv, int D, float (*tile)[W], long* dst_base) {
    const int tid = threadIdx.x;
    if (tid < 16) {
        const int tok = tok0 + tid;
        long base = -1;
        if (tok < n) {
            const int seq = token_seq[tok];
            if (seq >= 0) {
                const int pos = positions[tok];
                const int page = block_table[(size_t)seq * bt_width + pos / page_size];
                if (page >= 0) base = ((long)page * Hkv + kvh) * D * page_size + pos % page_size;
            }
        }
        dst_base[tid] = base;
    }
    if (VEC) {
        const int pieces = D / 8;
        for (int idx = tid; idx < 16 * pieces; idx += 256) {
            const int j = idx / pieces, d0 = (idx % pieces) * 8;
            const int tok = tok0 + j;
            float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (tok < n) Vec8<T>::load(qkv + (size_t)tok * row_stride + v_off + (size_t)kvh * D + d0, x);
#pragma unroll
            for (int e = 0; e < 8; ++e) tile[j][d0 + e] = x[e];
        }
    } else {
        for (int idx = tid; idx < 16 * D; idx += 256) {
            const int j = idx / D, d = idx % D;
            const int tok = tok0 + j;
            tile[j][d] = tok < n ? to_f(qkv[(size_t)tok * row_stride + v_off + (size_t)kvh * D + d]) : 0.f;
        }
    }
    __syncthreads();
    if (VEC) {
        // lane (d, h): the eight tokens 8 h .. 8 h + 7 of the tile at this d
        for (int idx = tid; idx < 2 * D; idx += 256) {
            const int d = idx / 2, h = idx % 2;
            const long b0 = dst_base[8 * h];
            bool run = b0 >= 0 && page_size % 8 == 0;
#pragma unroll
            for (int e = 1; e < 8; ++e) run = run && dst_base[8 * h + e] == b0 + e;
            T* dst = v_pages + b0 + (long)d * page_size;
            if (run && ((uintptr_t)dst % (8 * sizeof(T))) == 0) {
                float x[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = tile[8 * h + e][d];
                Vec8<T>::store(dst, x);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const long base = dst_base[8 * h + e];
                    if (base >= 0) v_pages[base + (long)d * page_size] = from_f<T>(tile[8 * h + e][d]);
                }
            }
        }
        return;
    }
    const int j = tid % 16;
    const long base = dst_base[j];
    if (base < 0) return;
    for (int d = tid / 16; d < D; d += 16) v_pages[base + (long)d * page_size] = from_f<T>(tile[j][d]);
}

// Prompt portions: queries and keys as above (store_kv == 2) in the first `qk_blocks` workgroups,
// the value rows tile by tile in the others, in one launch.
template <typename T, int L, int HP>
__global__ void __launch_bounds__(256)
qkv_prompt_vec_kernel(T* __restrict__ qkv, long row_stride, int q_off, int k_off, int v_off,
                      const int* __restrict__ positions, const int* __restrict__ token_seq,
                      const int* __restrict__ block_table, int bt_width, int page_size, T* __restrict__ k_pages,
                      T* __restrict__ v_pages, int n, int H, int Hkv, WeightPtr qw, WeightPtr kw, int has_norm,
                      float eps, int unit_offset, const float* __restrict__ table, int qk_blocks) {
    if ((int)blockIdx.x < qk_blocks) {
        qk_norm_rope_store_vec<T, L, HP>(blockIdx.x, qkv, row_stride, q_off, k_off, v_off, positions, token_seq,
                                     block_table, bt_width, page_size, k_pages, v_pages, n, H, Hkv, qw, kw, has_norm,
                                     eps, unit_offset, table, 2);
        return;
    }
    __shared__ float tile[16][8 * L + 1];
    __shared__ long dst_base[16];
    const int vb = (int)blockIdx.x - qk_blocks;
    store_v_tile<T, 8 * L + 1, true>((vb / Hkv) * 16, vb % Hkv, qkv, row_stride, v_off, positions, token_seq,
                                     block_table, bt_width, page_size, v_pages, n, Hkv, 8 * L, tile, dst_base);
}

template <typename T>
static bool launch_qk_vec(T* qkv, long row_stride, int q_off, int k_off, int v_off, const int* positions,
                          const int* token_seq, const int* block_table, int bt_width, int page_size, T* k_pages,
                          T* v_pages, int n, int H, int Hkv, int D, WeightPtr qw, WeightPtr kw, int has_norm, float eps,
                          int unit_offset, const float* table, int store_kv, hipStream_t stream) {
    const bool v_tiles = store_kv == 3;     // keys per head here, values tile by tile in the same launch
    if (v_tiles) store_kv = 2;
    const int heads = H + (store_kv == 1 ? 2 * Hkv : (store_kv == 2 ? Hkv : 0));
    // four heads to a lane group in steps of many tokens (the angles are read once for them); one
    // head each otherwise: smaller steps need the lanes more than the bytes (measured on MI355X:
    // even at 2048 tokens of 24 heads, faster at 8192)
    const int hp = (long)n * heads >= 65536 ? 4 : 1;
    const long lanes = (long)n * ((heads + hp - 1) / hp) * (D / 8);
    const unsigned qk_blocks = (unsigned)((lanes + 255) / 256);
    const dim3 grid(qk_blocks + (v_tiles ? (unsigned)((n + 15) / 16) * Hkv : 0u));
#define QK_VEC_HP(LL, PP)                                                                                          \
    if (v_tiles)                                                                                                   \
        hipLaunchKernelGGL((qkv_prompt_vec_kernel<T, LL, PP>), grid, dim3(256), 0, stream, qkv, row_stride, q_off, \
                           k_off, v_off, positions, token_seq, block_table, bt_width, page_size, k_pages, v_pages, \
                           n, H, Hkv, qw, kw, has_norm, eps, unit_offset, table, (int)qk_blocks);                  \
    else                                                                                                           \
        hipLaunchKernelGGL((qk_norm_rope_store_vec_kernel<T, LL, PP>), grid, dim3(256), 0, stream, qkv,            \
                           row_stride, q_off, k_off, v_off, positions, token_seq, block_table, bt_width,           \
                           page_size, k_pages, v_pages, n, H, Hkv, qw, kw, has_norm, eps, unit_offset, table,      \
                           store_kv)
#define QK_VEC(LL)                                                                                                 \
    do {                                                                                                           \
        if (hp == 4) { QK_VEC_HP(LL, 4); } else { QK_VEC_HP(LL, 1); }                                              \
    } while (0)
    if (D == 64) QK_VEC(8);
    else if (D == 128) QK_VEC(16);
    else if (D == 256) QK_VEC(32);
    else if (D == 512) QK_VEC(64);
    else return false;
#undef QK_VEC
#undef QK_VEC_HP
    return true;
}

extern "C" int mv_store_v_pages(const void* qkv, long row_stride, int v_off, const int* positions,
                                const int* token_seq, const int* block_table, int bt_width, int page_size,
                                void* v_pages, int n, int Hkv, int D, int dtype, hipStream_t stream);

// store_kv: 0 nothing goes to the cache; 1 keys and values, a store per token and head; 2 keys only;
// 3 keys per token and head, values tile by tile (16 tokens of a kv head at a time, for steps of
// many tokens), in the same launch where the vector kernel serves the shape.
extern "C" int mv_qk_norm_rope_store(void* qkv, long row_stride, int q_off, int k_off, int v_off,
                                     const int* positions, const int* token_seq, const int* block_table,
                                     int bt_width, int page_size, void* k_pages, void* v_pages, int n, int H,
                                     int Hkv, int D, const void* q_weight, const void* k_weight, int weight_dtype,
                                     float eps, int unit_offset, const float* table, int rot_dim, int interleaved,
                                     int store_kv, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && Hkv >= 0 && D > 0, "qk_norm_rope_store: bad sizes n=%d H=%d Hkv=%d D=%d", n, H,
               Hkv, D);
    MV_REQUIRE(D <= MV_MAX_HEAD_DIM, "qk_norm_rope_store: head_dim %d exceeds the supported maximum %d", D,
               MV_MAX_HEAD_DIM);
    MV_REQUIRE(table == nullptr || (rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= D),
               "qk_norm_rope_store: rotary dim %d must be even and at most head_dim %d", rot_dim, D);
    MV_REQUIRE(!store_kv || (block_table && k_pages && v_pages && page_size > 0 && bt_width > 0),
               "qk_norm_rope_store: cache write asked without pages or block table");
    const int has_norm = q_weight != nullptr;
    MV_REQUIRE(!has_norm || (k_weight != nullptr || !store_kv), "qk_norm_rope_store: q norm without k norm");
    MV_REQUIRE(!has_norm || eps > 0.f, "qk_norm_rope_store: eps must be positive");
    MV_REQUIRE(mv_valid_dtype(weight_dtype), "qk_norm_rope_store: bad weight dtype %d", weight_dtype);
    MV_REQUIRE(store_kv >= 0 && store_kv <= 3, "qk_norm_rope_store: bad cache mode %d", store_kv);
    if (n == 0) return 0;
    const int heads = H + (store_kv == 1 ? 2 * Hkv : (store_kv >= 2 ? Hkv : 0));
    WeightPtr qw{q_weight, weight_dtype}, kw{k_weight, weight_dtype};
    // the vector kernel: rotation over the whole head in half-split pairs, everything 16-byte aligned
    const size_t esz = dtype == MV_F32 ? 4 : 2;
    const bool aligned = ((uintptr_t)qkv % 16) == 0 && (row_stride * esz) % 16 == 0 && (q_off * esz) % 16 == 0 &&
                         (k_off * esz) % 16 == 0 && (v_off * esz) % 16 == 0 && ((uintptr_t)k_pages % 16) == 0 &&
                         ((uintptr_t)q_weight % 16) == 0 && ((uintptr_t)k_weight % 16) == 0 &&
                         ((uintptr_t)table % 16) == 0;
    if (aligned && (D == 64 || D == 128 || D == 256 || D == 512) && (table == nullptr || (rot_dim == D && !interleaved)) &&
        (long)n * heads * (D / 8) < (1L << 31)) {
        bool took = false;
        MV_DISPATCH_T(dtype, "qk_norm_rope_store",
                      took = launch_qk_vec<T>((T*)qkv, row_stride, q_off, k_off, v_off, positions, token_seq,
                                              block_table, bt_width, page_size, (T*)k_pages, (T*)v_pages, n, H, Hkv, D,
                                              qw, kw, has_norm, eps, unit_offset, table, store_kv, stream));
        if (took) return mv_check_launch("qk_norm_rope_store");
    }
    dim3 grid(n, (heads + 3) / 4);
    MV_DISPATCH_T(dtype, "qk_norm_rope_store",
                  hipLaunchKernelGGL(qk_norm_rope_store_kernel<T>, grid, dim3(256), 0, stream, (T*)qkv, row_stride,
                                     q_off, k_off, v_off, positions, token_seq, block_table, bt_width, page_size,
                                     (T*)k_pages, (T*)v_pages, H, Hkv, D, qw, kw, has_norm, eps, unit_offset, table,
                                     rot_dim, interleaved, store_kv == 3 ? 2 : store_kv));
    if (int rc = mv_check_launch("qk_norm_rope_store")) return rc;
    if (store_kv == 3)
        return mv_store_v_pages(qkv, row_stride, v_off, positions, token_seq, block_table, bt_width, page_size, v_pages,
                                n, Hkv, D, dtype, stream);
    return 0;
}

// The value rows of a step as a launch of their own (one workgroup per 16 tokens and kv head).
template <typename T>
__global__ void __launch_bounds__(256)
store_v_pages_kernel(const T* __restrict__ qkv, long row_stride, int v_off, const int* __restrict__ positions,
                     const int* __restrict__ token_seq, const int* __restrict__ block_table, int bt_width,
                     int page_size, T* __restrict__ v_pages, int n, int Hkv, int D) {
    __shared__ float tile[16][MV_MAX_HEAD_DIM + 1];
    __shared__ long dst_base[16];
    store_v_tile<T, MV_MAX_HEAD_DIM + 1>(blockIdx.x * 16, blockIdx.y, qkv, row_stride, v_off, positions, token_seq,
                                         block_table, bt_width, page_size, v_pages, n, Hkv, D, tile, dst_base);
}

extern "C" int mv_store_v_pages(const void* qkv, long row_stride, int v_off, const int* positions,
                                const int* token_seq, const int* block_table, int bt_width, int page_size,
                                void* v_pages, int n, int Hkv, int D, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && Hkv > 0 && D > 0 && D <= MV_MAX_HEAD_DIM, "store_v_pages: bad sizes n=%d Hkv=%d D=%d", n, Hkv,
               D);
    MV_REQUIRE(block_table && v_pages && page_size > 0 && bt_width > 0, "store_v_pages: missing pages or block table");
    MV_REQUIRE(Hkv <= 65535, "store_v_pages: too many kv heads");
    if (n == 0) return 0;
    dim3 grid((n + 15) / 16, Hkv);
    MV_DISPATCH_T(dtype, "store_v_pages",
                  hipLaunchKernelGGL(store_v_pages_kernel<T>, grid, dim3(256), 0, stream, (const T*)qkv, row_stride,
                                     v_off, positions, token_seq, block_table, bt_width, page_size, (T*)v_pages, n,
                                     Hkv, D));
    return mv_check_launch("store_v_pages");
}

// ---------------------------------------------------------------------------------------
// SwiGLU: out[n, i] = silu(gu[n, i]) * gu[n, I + i],  silu(z) = z / (1 + exp(-z))
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, long total, int I) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const long row = idx / I;
    const int col = (int)(idx - row * I);
    const float g = to_f(gu[row * 2 * I + col]);
    const float u = to_f(gu[row * 2 * I + I + col]);
    out[idx] = from_f<T>(g / (1.f + expf(-g)) * u);
}

template <typename T>
__global__ void swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, long total8, int I8) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;   // eight columns each
    if (idx >= total8) return;
    const long row = idx / I8;
    const int col = (int)(idx - row * I8) * 8;
    const int I = I8 * 8;
    float g[8], u[8], y[8];
    Vec8<T>::load(gu + row * 2 * I + col, g);
    Vec8<T>::load(gu + row * 2 * I + I + col, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = g[e] / (1.f + expf(-g[e])) * u[e];
    Vec8<T>::store(out + row * I + col, y);
}

extern "C" int mv_swiglu(const void* gate_up, void* out, int n, int I, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && I > 0, "swiglu: bad sizes n=%d I=%d", n, I);
    if (n == 0) return 0;
    if (I % 8 == 0 && ((uintptr_t)gate_up % 16) == 0 && ((uintptr_t)out % 16) == 0) {
        const long total8 = (long)n * (I / 8);
        MV_DISPATCH_T(dtype, "swiglu",
                      hipLaunchKernelGGL(swiglu_vec_kernel<T>, dim3((unsigned)((total8 + 255) / 256)), dim3(256), 0,
                                         stream, (const T*)gate_up, (T*)out, total8, I / 8));
        return mv_check_launch("swiglu");
    }
    const long total = (long)n * I;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    MV_DISPATCH_T(dtype, "swiglu",
                  hipLaunchKernelGGL(swiglu_kernel<T>, dim3(blocks), dim3(256), 0, stream, (const T*)gate_up,
                                     (T*)out, total, I));
    return mv_check_launch("swiglu");
}
