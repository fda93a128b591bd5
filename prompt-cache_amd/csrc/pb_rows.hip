// Row-wise building blocks: embedding rows into the fp32 residual stream, the weighted sum of residual streams fused with the
// RMS norms that read it, the polynomial-of-normalised-powers activation, the sigmoid top-k router and the bookkeeping of a
// mixture of experts (bucketing pairs by expert, summing the pairs' results back into the stream).  All reductions fp32.
#include <string.h>

#include "pb_common.h"

static thread_local char g_err[512] = "";

void pcb_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

PCB_EXPORT int pcb_version(void) { return PCB_ABI_VERSION; }
PCB_EXPORT const char* pcb_last_error_string(void) { return g_err; }

namespace {
using namespace pcb;

// block-wide sum of NV values per thread; every thread gets the totals.  red: [waves * NV]
template <int NV>
__device__ __forceinline__ void block_sum(float (&v)[NV], float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = wave_sum(v[i]);
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < NV; ++i) red[wave * NV + i] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        float t = 0.0f;
        for (int w = 0; w < waves; ++w) t += red[w * NV + i];
        v[i] = t;
    }
}

template <typename E>
__global__ __launch_bounds__(256) void embed_rows_kernel(const E* __restrict__ table, const int32_t* __restrict__ ids,
                                                         float* __restrict__ out, int width, int vocab) {
    const int r = blockIdx.x;
    int id = ids[r];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const E* src = table + (int64_t)id * width;
    for (int c = threadIdx.x; c < width; c += 256) out[(int64_t)r * width + c] = to_f32(src[c]);
}

// one workgroup per output row; the row is held in LDS between the sum and the norms (width * 4 bytes of dynamic LDS)
template <typename E>
__global__ __launch_bounds__(1024) void mix_norm_kernel(pcb_mix_norm_args a) {
    extern __shared__ float row[];
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int64_t src = a.rows ? a.rows[r] : r;
    const int W = a.width;
    float ss[1] = {0.0f};
    // (streams and coefficients are read through restrict-qualified pointers: the stores to x_out must not fence the loads)
    const float* __restrict__ hist = a.hist + src * W;
    const float* __restrict__ coef = a.coef;
    float* __restrict__ xo = a.x_out ? a.x_out + (int64_t)r * W : nullptr;
    const int nt = a.n_terms;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float x = nt > 0 ? 0.0f : hist[c];
        for (int j = 0; j < nt; ++j) x += coef[j] * hist[j * a.hist_stride + c];
        row[c] = x;
        if (xo) xo[c] = x;
        ss[0] += x * x;
    }
    block_sum<1>(ss, red);
    const float inv = 1.0f / sqrtf(ss[0] / (float)W + a.eps);
    E* o1 = (E*)a.out1;
    E* o2 = (E*)a.out2;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float x = row[c] * inv;
        if (o1) o1[(int64_t)r * W + c] = from_f32<E>(x * a.gain1[c]);
        if (o2) o2[(int64_t)r * W + c] = from_f32<E>(x * a.gain2[c]);
    }
}

template <typename E>
__global__ __launch_bounds__(1024) void polynorm_kernel(const float* __restrict__ z, const float* __restrict__ coef, E* __restrict__ out,
                                                       float eps, int ff) {
    __shared__ float red[48];
    const int64_t r = blockIdx.x;
    const float* zr = z + r * ff;
    float s[3] = {0.0f, 0.0f, 0.0f};
    for (int c = threadIdx.x; c < ff; c += blockDim.x) {
        const float v = zr[c], v2 = v * v, v3 = v2 * v;
        s[0] += v2;
        s[1] += v2 * v2;
        s[2] += v3 * v3;
    }
    block_sum<3>(s, red);
    const float i1 = coef[0] / sqrtf(s[0] / (float)ff + eps);
    const float i2 = coef[1] / sqrtf(s[1] / (float)ff + eps);
    const float i3 = coef[2] / sqrtf(s[2] / (float)ff + eps);
    const float c3 = coef[3];
    for (int c = threadIdx.x; c < ff; c += blockDim.x) {
        const float v = zr[c], v2 = v * v;
        out[r * ff + c] = from_f32<E>(i1 * v + i2 * v2 + i3 * (v2 * v) + c3);
    }
}

// one wave per row of router logits: sigmoid scores in LDS, `top` rounds of a wave-wide arg-max
__global__ __launch_bounds__(256) void router_topk_kernel(const float* __restrict__ logits, int n_rows, int n_experts, int top,
                                                          int32_t* __restrict__ expert, float* __restrict__ weight) {
    extern __shared__ float sc[];          // [4][n_experts]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = blockIdx.x * 4 + wave;
    if (r >= n_rows) return;
    float* s = sc + wave * n_experts;
    for (int e = lane; e < n_experts; e += 64) s[e] = 1.0f / (1.0f + expf(-logits[(int64_t)r * n_experts + e]));
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int k = 0; k < top; ++k) {
        float best = -1.0f;
        int bi = 0x7fffffff;
        for (int e = lane; e < n_experts; e += 64) {
            const float v = s[e];
            if (v > best) best = v, bi = e;        // ascending e: the first of equal scores stays
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ov > best || (ov == best && oi < bi)) best = ov, bi = oi;
        }
        if (lane == 0) {
            expert[(int64_t)r * top + k] = bi;
            weight[(int64_t)r * top + k] = best;
            s[bi] = -2.0f;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t* __restrict__ expert, const float* __restrict__ weight, int n_pairs,
                                                        int top, int n_experts, int32_t* __restrict__ group_off,
                                                        int32_t* __restrict__ row_src, int32_t* __restrict__ row_dst,
                                                        float* __restrict__ row_scale) {
    extern __shared__ int cnt[];           // [n_experts] counts, then [n_experts] cursors
    int* cur = cnt + n_experts;
    for (int e = threadIdx.x; e < n_experts; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += 1024) atomicAdd(&cnt[expert[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int off = 0;
        for (int e = 0; e < n_experts; ++e) {
            group_off[e] = off;
            cur[e] = off;
            off += cnt[e];
        }
        group_off[n_experts] = off;
    }
    __syncthreads();
    // (which row of its bucket a pair lands in does not enter any result: rows of a bucket are independent)
    for (int p = threadIdx.x; p < n_pairs; p += 1024) {
        const int at = atomicAdd(&cur[expert[p]], 1);
        row_src[at] = p / top;
        row_dst[at] = p;
        row_scale[at] = weight[p];
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ pair_out, const float* __restrict__ col_scale,
                                                          float* __restrict__ y, int width, int top) {
    const int64_t r = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += 256) {
        float s = 0.0f;
        for (int k = 0; k < top; ++k) s += pair_out[(r * top + k) * width + c];
        y[r * width + c] += col_scale[c] * s;
    }
}

}  // namespace

#define PCB_DTYPE_OK(d) ((d) == PCB_BF16 || (d) == PCB_F32)

PCB_EXPORT int pcb_embed_rows(const void* table, int32_t dtype, const int32_t* ids, float* out, int32_t n_rows, int32_t width,
                              int32_t vocab, void* stream) {
    PCB_REQUIRE(PCB_DTYPE_OK(dtype) && n_rows >= 0 && width > 0 && vocab > 0, PCB_ERR_ARG, "pcb_embed_rows: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(table && ids && out, PCB_ERR_ARG, "pcb_embed_rows: null pointer");
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(embed_rows_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)table, ids, out,
                           width, vocab);
    else
        hipLaunchKernelGGL(embed_rows_kernel<float>, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, (const float*)table, ids, out,
                           width, vocab);
    return pcb_check_launch("embed_rows_kernel");
}

PCB_EXPORT int pcb_mix_norm(const pcb_mix_norm_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_mix_norm_args), PCB_ERR_ARG, "pcb_mix_norm: struct size mismatch");
    PCB_REQUIRE(PCB_DTYPE_OK(a->dtype) && a->n_rows >= 0 && a->width > 0 && a->width <= 16384 && a->n_terms >= 0, PCB_ERR_ARG,
                "pcb_mix_norm: bad sizes (width <= 16384)");
    if (a->n_rows == 0) return PCB_OK;
    PCB_REQUIRE(a->hist && (a->n_terms == 0 || a->coef) && (!a->out1 || a->gain1) && (!a->out2 || a->gain2), PCB_ERR_ARG,
                "pcb_mix_norm: null pointer");
    const size_t lds = (size_t)a->width * sizeof(float);
    // few rows: a row's columns are spread over up to 1024 threads (the loads of a thread's columns are a dependent chain)
    const dim3 threads(a->n_rows <= 512 && a->width > 1024 ? 1024 : 256);
    if (a->dtype == PCB_BF16)
        hipLaunchKernelGGL(mix_norm_kernel<bf16_t>, dim3(a->n_rows), threads, lds, (hipStream_t)stream, *a);
    else
        hipLaunchKernelGGL(mix_norm_kernel<float>, dim3(a->n_rows), threads, lds, (hipStream_t)stream, *a);
    return pcb_check_launch("mix_norm_kernel");
}

PCB_EXPORT int pcb_polynorm(const float* z, const float* coef, void* out, int32_t dtype, float eps, int32_t n_rows, int32_t ff,
                            void* stream) {
    PCB_REQUIRE(PCB_DTYPE_OK(dtype) && n_rows >= 0 && ff > 0, PCB_ERR_ARG, "pcb_polynorm: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(z && coef && out, PCB_ERR_ARG, "pcb_polynorm: null pointer");
    const dim3 threads(n_rows <= 512 && ff > 1024 ? 1024 : 256);
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(polynorm_kernel<bf16_t>, dim3(n_rows), threads, 0, (hipStream_t)stream, z, coef, (bf16_t*)out, eps, ff);
    else
        hipLaunchKernelGGL(polynorm_kernel<float>, dim3(n_rows), threads, 0, (hipStream_t)stream, z, coef, (float*)out, eps, ff);
    return pcb_check_launch("polynorm_kernel");
}

PCB_EXPORT int pcb_router_topk(const float* logits, int32_t n_rows, int32_t n_experts, int32_t top, int32_t* expert, float* weight,
                               void* stream) {
    PCB_REQUIRE(n_rows >= 0 && n_experts > 0 && n_experts <= 2048 && top > 0 && top <= n_experts, PCB_ERR_ARG,
                "pcb_router_topk: bad sizes (1 <= top <= n_experts <= 2048)");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(logits && expert && weight, PCB_ERR_ARG, "pcb_router_topk: null pointer");
    hipLaunchKernelGGL(router_topk_kernel, dim3(pcb_ceil_div(n_rows, 4)), dim3(256), (size_t)4 * n_experts * sizeof(float),
                       (hipStream_t)stream, logits, n_rows, n_experts, top, expert, weight);
    return pcb_check_launch("router_topk_kernel");
}

PCB_EXPORT int pcb_moe_plan(const int32_t* expert, const float* weight, int32_t n_pairs, int32_t top, int32_t n_experts,
                            int32_t* group_off, int32_t* row_src, int32_t* row_dst, float* row_scale, void* stream) {
    PCB_REQUIRE(n_pairs >= 0 && n_pairs <= (1 << 20) && top > 0 && n_experts > 0 && n_experts <= 2048, PCB_ERR_ARG,
                "pcb_moe_plan: bad sizes");
    PCB_REQUIRE(expert && weight && group_off && row_src && row_dst && row_scale, PCB_ERR_ARG, "pcb_moe_plan: null pointer");
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), (size_t)2 * n_experts * sizeof(int), (hipStream_t)stream, expert, weight,
                       n_pairs, top, n_experts, group_off, row_src, row_dst, row_scale);
    return pcb_check_launch("moe_plan_kernel");
}

PCB_EXPORT int pcb_moe_combine(const float* pair_out, const float* col_scale, float* y, int32_t n_rows, int32_t width, int32_t top,
                               void* stream) {
    PCB_REQUIRE(n_rows >= 0 && width > 0 && top > 0, PCB_ERR_ARG, "pcb_moe_combine: bad sizes");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(pair_out && col_scale && y, PCB_ERR_ARG, "pcb_moe_combine: null pointer");
    hipLaunchKernelGGL(moe_combine_kernel, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, pair_out, col_scale, y, width, top);
    return pcb_check_launch("moe_combine_kernel");
}
