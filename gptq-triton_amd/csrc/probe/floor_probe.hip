// Floor probe: what one launch costs on this GPU before it computes anything, and how fast a launch of a given
// size can read memory at all.  Stand-alone program (no library code); bench.py --floor-probe runs it and puts
// the figures beside the decode kernels' times.
//   1. launch floor: N back-to-back launches of an empty kernel, replayed as one HIP graph, in the launch shapes
//      the decode kernels use (one workgroup per CU with a large LDS request, and many small workgroups);
//   2. plain read: every lane loads 16 bytes per instruction, `sizes` bytes per launch, each launch from its own
//      region of a pool larger than the 256 MB last-level cache (so every launch reads HBM), graph replay; the
//      best (grid, loads in flight) combination per size is reported, together with the same launch on a region
//      that is read over and over (served by the cache).
// Output: one line per figure, "name value unit", parsed by bench.py.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("error %s at line %d\n", hipGetErrorString(e_), __LINE__);          \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

__global__ void empty_kernel(unsigned *out) {
    extern __shared__ unsigned lds[];
    if (threadIdx.x == 0xFFFFFF) out[0] = lds[0];
}

template <int UNROLL>
__global__ __launch_bounds__(256) void read_kernel(const uint4 *__restrict__ src, size_t n16, unsigned *__restrict__ out) {
    // each workgroup owns one contiguous share; UNROLL independent 16-byte loads in flight per lane
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t b = (size_t)blockIdx.x * per, e = b + per < n16 ? b + per : n16;
    unsigned acc = 0;
    size_t i = b + threadIdx.x;
    for (; i + (UNROLL - 1) * 256 < e; i += UNROLL * 256) {
        uint4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = src[i + u * 256];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < e; i += 256) {
        const uint4 v = src[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x12345678u) out[0] = acc;
}

struct Timer {
    hipEvent_t e0, e1;
    hipStream_t s;
};

// median time of one replay of a graph of `n` launches made by `enqueue`, per launch, in microseconds
template <typename F>
static int graph_us(Timer &t, int n, F enqueue, double *us) {
    hipGraph_t g;
    hipGraphExec_t ge;
    CK(hipStreamBeginCapture(t.s, hipStreamCaptureModeGlobal));
    for (int i = 0; i < n; ++i) enqueue(i);
    CK(hipStreamEndCapture(t.s, &g));
    CK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
    for (int r = 0; r < 3; ++r) CK(hipGraphLaunch(ge, t.s));
    CK(hipStreamSynchronize(t.s));
    std::vector<float> ms(9);
    for (auto &m : ms) {
        CK(hipEventRecord(t.e0, t.s));
        CK(hipGraphLaunch(ge, t.s));
        CK(hipEventRecord(t.e1, t.s));
        CK(hipEventSynchronize(t.e1));
        CK(hipEventElapsedTime(&m, t.e0, t.e1));
    }
    std::sort(ms.begin(), ms.end());
    *us = ms[ms.size() / 2] * 1e3 / n;
    CK(hipGraphExecDestroy(ge));
    CK(hipGraphDestroy(g));
    return 0;
}

int main(int argc, char **argv) {
    Timer t;
    CK(hipStreamCreate(&t.s));
    CK(hipEventCreate(&t.e0));
    CK(hipEventCreate(&t.e1));
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    printf("device_cus %d count\n", cus);
    unsigned *out;
    CK(hipMalloc(&out, 256));
    CK(hipFuncSetAttribute(reinterpret_cast<const void *>(&empty_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 512));

    // ---- 1. launch floor
    struct Shape {
        const char *name;
        int grid, block, lds;
    } shapes[] = {{"launch_floor_1wg_per_cu_512t_81k", cus, 512, 81 * 1024},
                  {"launch_floor_1wg_per_cu_1024t_81k", cus, 1024, 81 * 1024},
                  {"launch_floor_2wg_per_cu_256t_64k", 2 * cus, 256, 64 * 1024},
                  {"launch_floor_8wg_per_cu_256t", 8 * cus, 256, 0}};
    for (const Shape &sh : shapes) {
        double us = 0;
        if (graph_us(t, 128, [&](int) { hipLaunchKernelGGL(empty_kernel, dim3(sh.grid), dim3(sh.block), sh.lds, t.s, out); }, &us)) return 1;
        printf("%s %.3f us\n", sh.name, us);
    }

    // ---- 2. plain read
    const size_t pool = (size_t)3 << 29;  // 1.5 GiB
    char *buf;
    CK(hipMalloc(&buf, pool));
    CK(hipMemset(buf, 1, pool));
    const size_t sizes[] = {8716288, 23425024, 26148864, 46850048};  // o_proj, down_proj, QKV, gate + up of LLaMA-7B, groupsize 128
    const char *names[] = {"8.7MB", "23.4MB", "26.1MB", "46.9MB"};
    for (int si = 0; si < 4; ++si) {
        const size_t sz = sizes[si] & ~(size_t)4095;
        const size_t stride = (sz + 4095) & ~(size_t)4095;
        const int regions = (int)(pool / stride) < 64 ? (int)(pool / stride) : 64;
        double best = 1e30, best_hot = 1e30;
        int best_grid = 0, best_unroll = 0;
        for (int wg_per_cu : {2, 4, 8, 16}) {
            for (int unroll : {2, 4, 8}) {
                const int grid = wg_per_cu * cus;
                auto launch = [&](const char *base) {
                    const uint4 *s = reinterpret_cast<const uint4 *>(base);
                    if (unroll == 2) hipLaunchKernelGGL(read_kernel<2>, dim3(grid), dim3(256), 0, t.s, s, sz / 16, out);
                    if (unroll == 4) hipLaunchKernelGGL(read_kernel<4>, dim3(grid), dim3(256), 0, t.s, s, sz / 16, out);
                    if (unroll == 8) hipLaunchKernelGGL(read_kernel<8>, dim3(grid), dim3(256), 0, t.s, s, sz / 16, out);
                };
                double us = 0, hot = 0;
                if (graph_us(t, regions, [&](int i) { launch(buf + (size_t)i * stride); }, &us)) return 1;
                if (graph_us(t, regions, [&](int) { launch(buf); }, &hot)) return 1;
                if (us < best) best = us, best_grid = grid, best_unroll = unroll;
                if (hot < best_hot) best_hot = hot;
            }
        }
        printf("plain_read_%s %.3f us\n", names[si], best);
        printf("plain_read_%s_rate %.1f GB/s\n", names[si], sz / best / 1e3);
        printf("plain_read_%s_grid %d workgroups\n", names[si], best_grid);
        printf("plain_read_%s_in_flight %d loads\n", names[si], best_unroll);
        printf("plain_read_%s_cached %.3f us\n", names[si], best_hot);
    }
    return 0;
}
