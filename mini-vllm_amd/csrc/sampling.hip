// Token sampling over float logits [M, V], one workgroup per row.
//
//   temperature == 0 : arg-max, ties to the lowest id.
//   temperature  > 0 : z = logit / temperature; optional top-k (keep every z >= the k-th
//                      largest), then optional top-p over the kept set (keep every z >= t,
//                      t the largest value whose upper set has at least p of the kept
//                      probability mass); then one draw from softmax(z) over the kept set by
//                      the Gumbel-max rule: argmax_i z_i - log(-log(u_i)), ties to the lowest
//                      id. u_i comes from a counter-based generator keyed by (seed, counter,
//                      i), so a row's draw does not depend on the rest of the batch.
// Thresholds are found by radix descent over the order-preserving integer image of z.
#include "common.h"

#define SP_THREADS 1024

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
    x ^= x >> 30;
    x *= 0xBF58476D1CE4E5B9ull;
    x ^= x >> 27;
    x *= 0x94D049BB133111EBull;
    x ^= x >> 31;
    return x;
}

// Uniform in (0, 1) with 23 bits, from (seed, counter, index): (n + 0.5) / 2^23 is exact in float.
__device__ __forceinline__ float uniform23(uint64_t seed, uint64_t counter, uint32_t index) {
    uint64_t x = mix64(seed + 0x9E3779B97F4A7C15ull * (counter + 1));
    x = mix64(x ^ (0xD1B54A32D192ED03ull * ((uint64_t)index + 1)));
    return ((float)(uint32_t)(x >> 41) + 0.5f) * (1.0f / 8388608.0f);
}

struct Best {
    float v;
    int i;
};

__device__ __forceinline__ Best better(Best a, Best b) {
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}

__device__ Best block_argmax(Best b, Best* sh) {
#pragma unroll
    for (int o = MV_WAVE / 2; o > 0; o >>= 1) {
        Best other;
        other.v = __shfl_xor(b.v, o, MV_WAVE);
        other.i = __shfl_xor(b.i, o, MV_WAVE);
        b = better(b, other);
    }
    const int lane = threadIdx.x % MV_WAVE, wave = threadIdx.x / MV_WAVE;
    __syncthreads();
    if (lane == 0) sh[wave] = b;
    __syncthreads();
    if (threadIdx.x == 0) {
        Best t = sh[0];
        for (int w = 1; w < SP_THREADS / MV_WAVE; ++w) t = better(t, sh[w]);
        sh[16] = t;
    }
    __syncthreads();
    return sh[16];
}

__global__ void __launch_bounds__(SP_THREADS)
sample_kernel(const float* __restrict__ logits, long ld, int V, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const unsigned long long* __restrict__ rng, int* __restrict__ out) {
    __shared__ Best shb[17];
    __shared__ float scratch[17];
    __shared__ int hcount[256];
    __shared__ float hmass[256];
    __shared__ uint32_t sh_prefix;
    __shared__ float sh_remaining;
    __shared__ int sh_kremaining;

    const int row = blockIdx.x;
    const int tid = threadIdx.x;
    const float* x = logits + (size_t)row * ld;
    const float T = temperature ? temperature[row] : 0.f;
    const int NEG_I = 0x7fffffff;

    if (!(T > 0.f)) {
        Best b{-INFINITY, NEG_I};
        for (int i = tid; i < V; i += SP_THREADS) b = better(b, Best{x[i], i});
        b = block_argmax(b, shb);
        if (tid == 0) out[row] = b.i;
        return;
    }

    uint32_t thr = 0;  // keep keys >= thr
    const int k = top_k ? top_k[row] : 0;
    if (k > 0 && k < V) {
        if (tid == 0) {
            sh_prefix = 0;
            sh_kremaining = k;
        }
        for (int byte = 3; byte >= 0; --byte) {
            for (int b = tid; b < 256; b += SP_THREADS) hcount[b] = 0;
            __syncthreads();
            const uint32_t prefix = sh_prefix;
            const uint32_t himask = byte == 3 ? 0u : (0xffffffffu << (8 * (byte + 1)));
            for (int i = tid; i < V; i += SP_THREADS) {
                const uint32_t key = order_key(x[i] / T);
                if ((key & himask) == prefix) atomicAdd(&hcount[(key >> (8 * byte)) & 0xff], 1);
            }
            __syncthreads();
            if (tid == 0) {
                int need = sh_kremaining, b = 255;
                for (; b > 0; --b) {
                    if (hcount[b] >= need) break;
                    need -= hcount[b];
                }
                sh_kremaining = need;
                sh_prefix = prefix | ((uint32_t)b << (8 * byte));
            }
            __syncthreads();
        }
        thr = sh_prefix;
    }

    const float p = top_p ? top_p[row] : 1.f;
    if (p < 1.f) {
        float zm = -INFINITY;
        for (int i = tid; i < V; i += SP_THREADS) {
            const float z = x[i] / T;
            if (order_key(z) >= thr) zm = fmaxf(zm, z);
        }
        zm = block_max(zm, scratch);
        float part = 0.f;
        for (int i = tid; i < V; i += SP_THREADS) {
            const float z = x[i] / T;
            if (order_key(z) >= thr) part += expf(z - zm);
        }
        const float total = block_sum(part, scratch);
        if (tid == 0) {
            sh_prefix = 0;
            sh_remaining = p * total;
        }
        for (int byte = 3; byte >= 0; --byte) {
            for (int b = tid; b < 256; b += SP_THREADS) hmass[b] = 0.f;
            __syncthreads();
            const uint32_t prefix = sh_prefix;
            const uint32_t himask = byte == 3 ? 0u : (0xffffffffu << (8 * (byte + 1)));
            for (int i = tid; i < V; i += SP_THREADS) {
                const float z = x[i] / T;
                const uint32_t key = order_key(z);
                if (key >= thr && (key & himask) == prefix)
                    atomicAdd(&hmass[(key >> (8 * byte)) & 0xff], expf(z - zm));
            }
            __syncthreads();
            if (tid == 0) {
                float need = sh_remaining;
                int b = 255, last_nonempty = -1;
                for (; b >= 0; --b) {
                    if (hmass[b] > 0.f) last_nonempty = b;
                    if (hmass[b] > 0.f && hmass[b] >= need) break;
                    need -= hmass[b];
                }
                if (b < 0) {  // rounding kept the sum just below the target: take everything
                    b = last_nonempty < 0 ? 0 : last_nonempty;
                    need = 0.f;
                }
                sh_remaining = need;
                sh_prefix = prefix | ((uint32_t)b << (8 * byte));
            }
            __syncthreads();
        }
        if (sh_prefix > thr) thr = sh_prefix;
    }

    const uint64_t seed = rng[2 * (size_t)row], counter = rng[2 * (size_t)row + 1];
    Best best{-INFINITY, NEG_I};
    for (int i = tid; i < V; i += SP_THREADS) {
        const float z = x[i] / T;
        if (order_key(z) < thr) continue;
        const float u = uniform23(seed, counter, (uint32_t)i);
        const float g = -logf(-logf(u));
        best = better(best, Best{z + g, i});
    }
    best = block_argmax(best, shb);
    if (tid == 0) out[row] = best.i;
}

// temperature, top_k, top_p: per row, or null for 0 / off / off. rng: [M][2] = (seed, counter).
extern "C" int mv_sample(const float* logits, long ld, int M, int V, const float* temperature, const int* top_k,
                         const float* top_p, const unsigned long long* rng, int* out, hipStream_t stream) {
    MV_REQUIRE(M >= 0 && V > 0 && ld >= V, "sample: bad sizes M=%d V=%d ld=%ld", M, V, ld);
    MV_REQUIRE(temperature == nullptr || rng != nullptr, "sample: temperatures given without random keys");
    if (M == 0) return 0;
    hipLaunchKernelGGL(sample_kernel, dim3(M), dim3(SP_THREADS), 0, stream, logits, ld, V, temperature, top_k,
                       top_p, rng, out);
    return mv_check_launch("sample");
}
