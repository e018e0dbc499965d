// Host-side support of the C entry points: the error channel and a few queries.
#include "common.h"
#include <stdlib.h>
#include <string.h>

static thread_local char g_error[512] = "";

extern "C" const char* mv_last_error() { return g_error; }

int mv_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return 1;
}

int mv_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mv_fail("%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// Bit mask of the activation types this library was built for (bit 0 float, bit 1 bf16).
extern "C" int mv_built_dtypes() {
    int m = 0;
#ifdef MV_WITH_F32
    m |= 1;
#endif
#ifdef MV_WITH_BF16
    m |= 2;
#endif
    return m;
}

extern "C" int mv_abi_version() { return 1; }

// Compute units of the current device, asked once (the launch rules size their grids in rounds of
// one workgroup a compute unit); 256 if the device does not say. MV_COMPUTE_UNITS overrides it,
// for a process that is confined to part of the chip.
int mv_compute_units() {
    static int units = 0;
    if (units > 0) return units;
    int n = 0;
    const char* env = getenv("MV_COMPUTE_UNITS");
    if (env != nullptr) n = atoi(env);
    if (n <= 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            n = prop.multiProcessorCount;
    }
    units = n > 0 ? n : 256;
    return units;
}

extern "C" int mv_device_compute_units() { return mv_compute_units(); }

// A kernel that does nothing: a graph of these, each depending on the one before, shows what a
// dependent launch costs on the device whatever it computes (the floor of a decode step that is a
// chain of small kernels).
__global__ void empty_kernel(const void* unused) {}

extern "C" int mv_launch_empty(int grid, int block, const void* arg, hipStream_t stream) {
    MV_REQUIRE(grid > 0 && block > 0 && block <= 1024, "launch_empty: bad launch %d x %d", grid, block);
    hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), 0, stream, arg);
    return mv_check_launch("launch_empty");
}

// What a captured graph holds, by kind of node: out[0] kernels, out[1] memsets, out[2] copies,
// out[3] anything else. The engine admits no memset node in a graph it replays (such nodes have
// given wrong results on replays after the first); a library call that records one is found here.
extern "C" int mv_graph_census(void* graph, int* out) {
    MV_REQUIRE(graph != nullptr && out != nullptr, "mv_graph_census: null argument");
    size_t n = 0;
    hipError_t e = hipGraphGetNodes((hipGraph_t)graph, nullptr, &n);
    if (e != hipSuccess) return mv_fail("mv_graph_census: hipGraphGetNodes: %s", hipGetErrorString(e));
    out[0] = out[1] = out[2] = out[3] = 0;
    if (n == 0) return 0;
    hipGraphNode_t* nodes = (hipGraphNode_t*)malloc(n * sizeof(hipGraphNode_t));
    MV_REQUIRE(nodes != nullptr, "mv_graph_census: out of host memory");
    e = hipGraphGetNodes((hipGraph_t)graph, nodes, &n);
    if (e != hipSuccess) {
        free(nodes);
        return mv_fail("mv_graph_census: hipGraphGetNodes: %s", hipGetErrorString(e));
    }
    for (size_t i = 0; i < n; ++i) {
        hipGraphNodeType t;
        e = hipGraphNodeGetType(nodes[i], &t);
        if (e != hipSuccess) {
            free(nodes);
            return mv_fail("mv_graph_census: hipGraphNodeGetType: %s", hipGetErrorString(e));
        }
        if (t == hipGraphNodeTypeKernel) out[0]++;
        else if (t == hipGraphNodeTypeMemset) out[1]++;
        else if (t == hipGraphNodeTypeMemcpy) out[2]++;
        else out[3]++;
    }
    free(nodes);
    return 0;
}
