// The last step of a greedy decode token: logits = x . W^T with the fp16 lm_head weight W [V, K] and the index of the
// largest logit per row, in one launch.  (The reference's scripts call the model's lm_head - a dense fp16 linear -
// and take the argmax of its output, generate.py; the vendor's GEMV plus torch's argmax are 59 + 15 us of a 1.6 ms
// LLaMA-7B step.)  A memory-bound stream over V x K x 2 bytes: the rows of W are dealt to the workgroups in contiguous
// ranges, inside a workgroup to the waves one by one; a wave has the next row's loads in flight while it multiplies
// one (64 lanes x KCH 16-byte chunks, the x rows out of LDS), rounds the sum to fp16 as the linear layer's output
// would be, and keeps the best (value, index) per x row - the lower index among equal values, as torch.argmax does.
// Workgroup bests go through the workspace; the last workgroup to arrive picks the winners.
#include "../../include/gptq4.h"
#include "gptq4_internal.h"

namespace {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
constexpr int HEAD_WAVES = 8;
constexpr int HEAD_MAX_B = 16;

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

template <int KCH>
__global__ __launch_bounds__(64 * HEAD_WAVES) void gptq4_head_argmax_kernel(const half_t *__restrict__ x, const half_t *__restrict__ w,
                                                                            long long *__restrict__ out, float *part, int *counters,
                                                                            int B, int V, int rows_per_wg) {
    constexpr int K = KCH * 512;
    constexpr int CHUNKS = K / 8;
    extern __shared__ uint4 head_xs[];  // [B][CHUNKS]
    __shared__ float s_val[HEAD_WAVES][HEAD_MAX_B];
    __shared__ int s_idx[HEAD_WAVES][HEAD_MAX_B];
    __shared__ int s_last;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (int c = tid; c < B * CHUNKS; c += 64 * HEAD_WAVES) head_xs[c] = reinterpret_cast<const uint4 *>(x)[c];
    if (lane < HEAD_MAX_B) {
        s_val[wave][lane] = -INFINITY;
        s_idx[wave][lane] = 0x7fffffff;
    }
    __syncthreads();

    const int r0 = blockIdx.x * rows_per_wg, r1 = min(r0 + rows_per_wg, V);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(w), 0, (int)0x7FFFFFF0, 0x00020000);
    u32x4_t cur[KCH], nxt[KCH];
    auto fetch = [&](u32x4_t (&dst)[KCH], int row) {
        // (rows past the range: a lane offset the buffer rejects - zeros, no memory touched)
        const uint32_t off = row < r1 ? (uint32_t)lane * 16u : 0x80000000u;
#pragma unroll
        for (int j = 0; j < KCH; ++j) dst[j] = __builtin_amdgcn_raw_buffer_load_b128(rs, off, (uint32_t)row * (uint32_t)(K * 2) + 1024u * j, 0);
    };
    fetch(cur, r0 + wave);
    for (int row = r0 + wave; row < r1; row += HEAD_WAVES) {
        fetch(nxt, row + HEAD_WAVES);
        for (int b = 0; b < B; ++b) {
            const uint4 *xb = head_xs + b * CHUNKS + lane;
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < KCH; ++j) {
                const uint4 xv = xb[64 * j];
                acc = __builtin_amdgcn_fdot2(as_h2(cur[j].x), as_h2(xv.x), acc, false);
                acc = __builtin_amdgcn_fdot2(as_h2(cur[j].y), as_h2(xv.y), acc, false);
                acc = __builtin_amdgcn_fdot2(as_h2(cur[j].z), as_h2(xv.z), acc, false);
                acc = __builtin_amdgcn_fdot2(as_h2(cur[j].w), as_h2(xv.w), acc, false);
            }
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) acc += __shfl_xor(acc, o);
            const float v = (float)(half_t)acc;  // the linear layer's fp16 output
            if (lane == 0 && better(v, row, s_val[wave][b], s_idx[wave][b])) {
                s_val[wave][b] = v;
                s_idx[wave][b] = row;
            }
        }
#pragma unroll
        for (int j = 0; j < KCH; ++j) cur[j] = nxt[j];
    }
    __syncthreads();

    // ---- the workgroup's best per x row -> workspace; the last workgroup to arrive reduces them
    const int nwg = gridDim.x;
    if (tid < B) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int wv = 0; wv < HEAD_WAVES; ++wv)
            if (better(s_val[wv][tid], s_idx[wv][tid], bv, bi)) bv = s_val[wv][tid], bi = s_idx[wv][tid];
        float *dst = part + ((size_t)blockIdx.x * HEAD_MAX_B + tid) * 2;
        __hip_atomic_store(dst, bv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(reinterpret_cast<int *>(dst) + 1, bi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const int old = __hip_atomic_fetch_add(&counters[0], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == nwg - 1);
    }
    __syncthreads();
    if (!s_last) return;
    if (tid == 0) __hip_atomic_store(&counters[0], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int b = 0; b < B; ++b) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int g = tid; g < nwg; g += 64 * HEAD_WAVES) {
            const float *src = part + ((size_t)g * HEAD_MAX_B + b) * 2;
            const float v = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int i = __hip_atomic_load(reinterpret_cast<const int *>(src) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (better(v, i, bv, bi)) bv = v, bi = i;
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) {
            const float ov = __shfl_xor(bv, o);
            const int oi = __shfl_xor(bi, o);
            if (better(ov, oi, bv, bi)) bv = ov, bi = oi;
        }
        __syncthreads();  // (the slots of the row before have been read)
        if (lane == 0) {
            s_val[wave][0] = bv;
            s_idx[wave][0] = bi;
        }
        __syncthreads();
        if (tid == 0) {
#pragma unroll
            for (int wv = 1; wv < HEAD_WAVES; ++wv)
                if (better(s_val[wv][0], s_idx[wv][0], bv, bi)) bv = s_val[wv][0], bi = s_idx[wv][0];
            out[b] = (long long)bi;
        }
    }
}

template <int KCH>
int launch_kch(const half_t *x, const half_t *w, long long *out, float *part, int *counters, int B, int V, hipStream_t stream) {
    const int cus = device_shape().cus;
    const int nwg = V < cus ? V : cus;
    const int rows_per_wg = (V + nwg - 1) / nwg;
    const int grid = (V + rows_per_wg - 1) / rows_per_wg;
    const size_t lds = (size_t)B * KCH * 512 * sizeof(half_t);
    if (lds > 48 * 1024) {
        static bool allowed = false;
        if (!allowed) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gptq4_head_argmax_kernel<KCH>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 2048);
            if (e != hipSuccess) return (int)e;
            allowed = true;
        }
    }
    hipLaunchKernelGGL((gptq4_head_argmax_kernel<KCH>), dim3((unsigned)grid), dim3(64 * HEAD_WAVES), lds, stream, x, w, out, part, counters, B, V,
                       rows_per_wg);
    return (int)hipGetLastError();
}

}  // namespace

size_t head_argmax_partial_bytes() { return (size_t)device_shape().cus * HEAD_MAX_B * 2 * sizeof(float); }

// -GPTQ4_E_SHAPE for row lengths without an instantiation
int launch_head_argmax(const half_t *x, const half_t *w, long long *out, float *part, int *counters, int B, int K, int V, hipStream_t stream) {
    if (B < 1 || B > HEAD_MAX_B || V < 1 || (size_t)V * K * 2 >= 0x7FFFFFF0ull || (size_t)B * K * 2 > 160 * 1024 - 2048) return -GPTQ4_E_SHAPE;
    switch (K) {
        case 4096: return launch_kch<8>(x, w, out, part, counters, B, V, stream);
        case 5120: return launch_kch<10>(x, w, out, part, counters, B, V, stream);
        case 6656: return launch_kch<13>(x, w, out, part, counters, B, V, stream);
        case 8192: return launch_kch<16>(x, w, out, part, counters, B, V, stream);
        default: return -GPTQ4_E_SHAPE;
    }
}
