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
#include "mv_noalloc.h"
#include <mutex>

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

// A row needs no threshold when nothing is cut away: its token is one arg-max over the row (of the
// logits, or of z + Gumbel noise), which many workgroups can share.
__device__ __forceinline__ bool row_is_simple(int row, int V, float T, const int* top_k, const float* top_p) {
    if (!(T > 0.f)) return true;
    const int k = top_k ? top_k[row] : 0;
    const float p = top_p ? top_p[row] : 1.f;
    return !(k > 0 && k < V) && !(p < 1.f);
}

#define SP_PART_THREADS 256

// First of two passes for simple rows: workgroup (row, chunk) finds the best of its chunk of the
// vocabulary and leaves it in partial[row][chunk]. Rows that need thresholds are left to the
// second pass alone.
__global__ void __launch_bounds__(SP_PART_THREADS)
sample_partial_kernel(const float* __restrict__ logits, long ld, int V, const float* __restrict__ temperature,
                      const int* __restrict__ top_k, const float* __restrict__ top_p,
                      const unsigned long long* __restrict__ rng, Best* __restrict__ partial, int chunks) {
    __shared__ Best sh[SP_PART_THREADS / MV_WAVE];
    const int row = blockIdx.x, chunk = blockIdx.y;
    const float T = temperature ? temperature[row] : 0.f;
    if (!row_is_simple(row, V, T, top_k, top_p)) return;
    const float* x = logits + (size_t)row * ld;
    const int per = ((V + chunks - 1) / chunks + 3) & ~3;
    const int lo = chunk * per, hi = lo + per < V ? lo + per : V;
    const bool greedy = !(T > 0.f);
    uint64_t seed = 0, counter = 0;
    if (!greedy) {
        seed = rng[2 * (size_t)row];
        counter = rng[2 * (size_t)row + 1];
    }
    Best b{-INFINITY, 0x7fffffff};
    auto take = [&](float v, int i) {
        if (!greedy) v = v / T - logf(-logf(uniform23(seed, counter, (uint32_t)i)));
        b = better(b, Best{v, i});
    };
    if ((ld & 3) == 0 && (((uintptr_t)logits) & 15) == 0) {
        for (int i = lo + 4 * (int)threadIdx.x; i < hi; i += 4 * SP_PART_THREADS) {
            if (i + 3 < hi) {
                const float4 v = *reinterpret_cast<const float4*>(x + i);
                take(v.x, i); take(v.y, i + 1); take(v.z, i + 2); take(v.w, i + 3);
            } else {
                for (int j = i; j < hi; ++j) take(x[j], j);
            }
        }
    } else {
        for (int i = lo + (int)threadIdx.x; i < hi; i += SP_PART_THREADS) take(x[i], i);
    }
#pragma unroll
    for (int o = MV_WAVE / 2; o > 0; o >>= 1) {
        Best other;
        other.v = __shfl_xor(b.v, o, MV_WAVE);
        other.i = __shfl_xor(b.i, o, MV_WAVE);
        b = better(b, other);
    }
    if (threadIdx.x % MV_WAVE == 0) sh[threadIdx.x / MV_WAVE] = b;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < SP_PART_THREADS / MV_WAVE; ++w) b = better(b, sh[w]);
        partial[(size_t)row * chunks + chunk] = b;
    }
}

// What a row's drawn token is written to. Besides the output, a decode step that runs again at
// once on the device takes the token as its next input: ``next_ids[row]`` receives it, the row's
// position and context length move on by one and its random stream's counter by one. Null
// pointers leave all that out.
struct Advance {
    int* next_ids;
    int* positions;
    int* context_lens;
    unsigned long long* rng;
};

__device__ __forceinline__ void deliver(int row, int token, int* out, const Advance& adv) {
    out[row] = token;
    if (adv.next_ids != nullptr) {
        adv.next_ids[row] = token;
        adv.positions[row] += 1;
        adv.context_lens[row] += 1;
        if (adv.rng != nullptr) adv.rng[2 * (size_t)row + 1] += 1;
    }
}

__global__ void __launch_bounds__(SP_THREADS)
sample_kernel(const float* __restrict__ logits, long ld, int V, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const unsigned long long* rng, int* __restrict__ out,
              const Best* __restrict__ partial, int chunks, Advance adv) {
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

    if (partial != nullptr && row_is_simple(row, V, T, top_k, top_p)) {   // the first pass did the work
        Best b{-INFINITY, NEG_I};
        for (int c = tid; c < chunks; c += SP_THREADS) b = better(b, partial[(size_t)row * chunks + c]);
        b = block_argmax(b, shb);
        if (tid == 0) deliver(row, b.i, out, adv);
        return;
    }
    if (!(T > 0.f)) {
        Best b{-INFINITY, NEG_I};
        for (int i = tid; i < V; i += SP_THREADS) b = better(b, Best{x[i], i});
        b = block_argmax(b, shb);
        if (tid == 0) deliver(row, b.i, out, adv);
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
    best = block_argmax(best, shb);        // (its barriers lie between every lane's read of the counter and the write)
    if (tid == 0) deliver(row, best.i, out, adv);
}

// temperature, top_k, top_p: per row, or null for 0 / off / off. rng: [M][2] = (seed, counter).
// work: 8 * M * chunks bytes of scratch, or null. With it, rows that need no threshold (greedy
// rows, and drawn rows without top-k and top-p) are served by two short launches in which
// `chunks` workgroups share a row; the drawn token is the same either way.
static int sample_launch(const float* logits, long ld, int M, int V, const float* temperature, const int* top_k,
                         const float* top_p, const unsigned long long* rng, int* out, void* work, int chunks,
                         Advance adv, hipStream_t stream) {
    MV_REQUIRE(M >= 0 && V > 0 && ld >= V, "sample: bad sizes M=%d V=%d ld=%ld", M, V, ld);
    MV_REQUIRE(temperature == nullptr || rng != nullptr, "sample: temperatures given without random keys");
    MV_REQUIRE(work == nullptr || (chunks >= 1 && chunks <= 65535), "sample: bad chunk count %d", chunks);
    if (M == 0) return 0;
    if (work != nullptr) {
        hipLaunchKernelGGL(sample_partial_kernel, dim3(M, chunks), dim3(SP_PART_THREADS), 0, stream, logits, ld, V,
                           temperature, top_k, top_p, rng, (Best*)work, chunks);
        if (int rc = mv_check_launch("sample (first pass)")) return rc;
    }
    hipLaunchKernelGGL(sample_kernel, dim3(M), dim3(SP_THREADS), 0, stream, logits, ld, V, temperature, top_k,
                       top_p, rng, out, (const Best*)work, chunks, adv);
    return mv_check_launch("sample");
}

extern "C" int mv_sample(const float* logits, long ld, int M, int V, const float* temperature, const int* top_k,
                         const float* top_p, const unsigned long long* rng, int* out, void* work, int chunks,
                         hipStream_t stream) {
    return sample_launch(logits, ld, M, V, temperature, top_k, top_p, rng, out, work, chunks,
                         Advance{nullptr, nullptr, nullptr, nullptr}, stream);
}

// The same, for a decode step that runs again on the device with the drawn tokens: row m's token also
// goes to next_ids[m], positions[m] and context_lens[m] move on by one, and so does the counter of
// the row's random stream (rng is written here).
extern "C" int mv_sample_advance(const float* logits, long ld, int M, int V, const float* temperature,
                                 const int* top_k, const float* top_p, unsigned long long* rng, int* out, void* work,
                                 int chunks, int* next_ids, int* positions, int* context_lens, hipStream_t stream) {
    MV_REQUIRE(next_ids != nullptr && positions != nullptr && context_lens != nullptr,
               "sample_advance: the next step's token ids, positions and context lengths are needed");
    return sample_launch(logits, ld, M, V, temperature, top_k, top_p, rng, out, work, chunks,
                         Advance{next_ids, positions, context_lens, rng}, stream);
}


// ---------------------------------------------------------------------------------------
// The variant that allocates nothing (see mv_noalloc.h): the first pass's partial results go
// through this array instead of a workspace of the caller's.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[MV_NOALLOC_SCRATCH_BYTES];

#define MV_NOALLOC_MAX_DEVICES 64
static std::mutex g_scratch_lock;
static void* g_scratch_ptr[MV_NOALLOC_MAX_DEVICES] = {nullptr};

// The array's address on the current device, looked up once per device (every GPU holds a copy of
// its own at an address of its own; the name `scratch` itself means nothing to host code).
static int scratch_on_current_device(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return mv_fail("sample_noalloc: hipGetDevice: %s", hipGetErrorString(e));
    MV_REQUIRE(dev >= 0 && dev < MV_NOALLOC_MAX_DEVICES, "sample_noalloc: device %d is beyond the %d this build knows",
               dev, MV_NOALLOC_MAX_DEVICES);
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr)
            return mv_fail("sample_noalloc: hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

extern "C" int mv_sample_noalloc(const float* logits, long ld, int M, int V, const float* temperature,
                                 const int* top_k, const float* top_p, const unsigned long long* rng, int* out,
                                 hipStream_t stream) {
    static_assert(sizeof(Best) == 8, "a partial result is 8 bytes");
    MV_REQUIRE(M <= MV_NOALLOC_MAX_ROWS, "sample_noalloc: %d rows exceed the %d rows the library's own scratch "
               "array holds; split the call, or use mv_sample with a workspace", M, MV_NOALLOC_MAX_ROWS);
    MV_REQUIRE(logits != nullptr && out != nullptr, "sample_noalloc: logits and output are needed");
    void* ptr = nullptr;
    if (int rc = scratch_on_current_device(&ptr)) return rc;
    return sample_launch(logits, ld, M, V, temperature, top_k, top_p, rng, out, ptr, MV_NOALLOC_CHUNKS,
                         Advance{nullptr, nullptr, nullptr, nullptr}, stream);
}
