// Mixers that carry a state from token to token instead of a key cache: linear attention with a scalar decay per head
// (pcb_decay_attn), the short causal convolution (pcb_causal_conv, pcb_conv_state_update) and the selective scan
// (pcb_selective_scan).  States, decays, step sizes and every product that feeds a state are fp32.
#include "pb_common.h"

namespace {
using namespace pcb;

__device__ __forceinline__ f4 mma4(float a, float b, f4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

// decay^n for a small non-negative integer n, fp32
__device__ __forceinline__ float decay_pow(float log2_decay, int n) { return n <= 0 ? 1.0f : exp2f((float)n * log2_decay); }

// ---- linear attention with decay ----------------------------------------------------------------------------------------------
// One wave = (request, head, 16 value columns); it walks the request's tokens in chunks of up to 16 and keeps its [dim][16] slice of
// the state in registers as NB result tiles (tile b: rows = key columns 16 b + 4 (l >> 4) + r, column = value column l & 15).
// Per chunk (t, j = token indices inside it, n tokens, L = decay):
//   W^T  = K Q^T                       [j][t]   then  w(t, j) = L^(t-j) q_t.k_j for j <= t, else 0
//   O^T  = L^(t+1) S^T Q^T + V^T W^T   [value column][t]
//   S   <- L^n S + sum_j L^(n-1-j) k_j v_j^T
// all on the fp32 matrix cores (v_mfma_f32_16x16x4_f32), elements of E widened exactly.  The state tiles ARE the operand
// fragments of S^T Q^T: the k index of that product runs over the key columns in the order (l >> 4, e) -> 16 (e >> 2) + 4 (l >> 4) +
// (e & 3) inside a 32-column step, which the query operand follows.
template <typename E, int NB>
__global__ __launch_bounds__(64) void decay_attn_kernel(pcb_decay_attn_args a) {
    const int lane = threadIdx.x, g = lane >> 4, c = lane & 15;
    const int32_t* rq = a.reqs + 4 * blockIdx.x;
    const int slot = rq[0], pos0 = rq[1], count = rq[2], row0 = rq[3];
    const int h = blockIdx.y, vcol = blockIdx.z * 16 + c;
    const int dim = a.dim, vdim = a.vdim;
    const bool v_ok = vcol < vdim;
    const float lam = a.decay[h];
    const float lg = lam > 0.0f ? log2f(lam) : -__builtin_inff();
    float* st = a.state + (int64_t)slot * a.slot_stride + (int64_t)h * dim * vdim;

    f4 S[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int d = 16 * b + 4 * g + r;
            S[b][r] = (pos0 > 0 && d < dim && v_ok) ? st[(int64_t)d * vdim + vcol] : 0.0f;
        }
    }
    const E* Q = (const E*)a.q + (int64_t)h * dim;
    const E* K = (const E*)a.k + (int64_t)h * dim;
    const E* V = (const E*)a.v + (int64_t)h * vdim;

    for (int c0 = 0; c0 < count; c0 += 16) {
        const int n = count - c0 < 16 ? count - c0 : 16;
        const int64_t r0 = row0 + c0;
        // operands with the token in the lane's row (l & 15): q as the B side, k as the A side, k index = key column
        const bool t_ok = c < n;
        const E* qrow = Q + (r0 + c) * a.ldq;
        const E* krow = K + (r0 + c) * a.ldk;
        f4 wt = f4{0.f, 0.f, 0.f, 0.f}, ot = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < NB / 2; ++ks) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int d = 32 * ks + 16 * (e >> 2) + 4 * g + (e & 3);
                const bool ok = t_ok && d < dim;
                const float qv = ok ? to_f32(qrow[d]) : 0.0f;
                const float kv = ok ? to_f32(krow[d]) : 0.0f;
                wt = mma4(kv, qv, wt);
                ot = mma4(S[2 * ks + (e >> 2)][e & 3], qv, ot);
            }
        }
        // wt: column t = c, rows j = 4 g + r;  ot: column t = c, rows = value columns 4 g + r
        const float lt1 = decay_pow(lg, c + 1);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int j = 4 * g + r;
            wt[r] = (j <= c && j < n) ? wt[r] * decay_pow(lg, c - j) : 0.0f;
            ot[r] *= lt1;
        }
        // values with the token in the k index: element e of lane group g is token 4 g + e
        float vv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j = 4 * g + e;
            vv[e] = (j < n && v_ok) ? to_f32(V[(r0 + j) * a.ldv + vcol]) : 0.0f;
            ot = mma4(vv[e], wt[e], ot);
        }
        if (t_ok && a.out) {
            float* op = a.out + (r0 + c) * a.ldo + (int64_t)h * vdim + blockIdx.z * 16;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (blockIdx.z * 16 + 4 * g + r < vdim) op[4 * g + r] = ot[r];
        }
        // the state moves behind the chunk
        const float ln = decay_pow(lg, n);
        float kd[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) kd[e] = 4 * g + e < n ? decay_pow(lg, n - 1 - (4 * g + e)) : 0.0f;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            f4 s = S[b];
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] *= ln;
            const int d = 16 * b + c;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = 4 * g + e;
                const float kv = (j < n && d < dim) ? to_f32(K[(r0 + j) * a.ldk + d]) * kd[e] : 0.0f;
                s = mma4(kv, vv[e], s);
            }
            S[b] = s;
        }
    }
    if (!v_ok) return;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int d = 16 * b + 4 * g + r;
            if (d < dim) st[(int64_t)d * vdim + vcol] = S[b][r];
        }
}

template <typename E>
int launch_decay(const pcb_decay_attn_args& a, hipStream_t stream) {
    const dim3 grid(a.n_reqs, a.H, pcb_ceil_div(a.vdim, 16));
    if (a.dim <= 32)
        hipLaunchKernelGGL((decay_attn_kernel<E, 2>), grid, dim3(64), 0, stream, a);
    else if (a.dim <= 64)
        hipLaunchKernelGGL((decay_attn_kernel<E, 4>), grid, dim3(64), 0, stream, a);
    else if (a.dim <= 128)
        hipLaunchKernelGGL((decay_attn_kernel<E, 8>), grid, dim3(64), 0, stream, a);
    else
        hipLaunchKernelGGL((decay_attn_kernel<E, 16>), grid, dim3(64), 0, stream, a);
    return pcb_check_launch("decay_attn_kernel");
}

// ---- short causal convolution -----------------------------------------------------------------------------------------------------
constexpr int MAX_TAPS = 16;

template <typename E>
__global__ __launch_bounds__(256) void causal_conv_kernel(const E* __restrict__ x, int64_t ldx, const E* __restrict__ w,
                                                          const E* __restrict__ bias, int silu, const int32_t* __restrict__ meta,
                                                          const E* __restrict__ state, int64_t slot_stride, E* __restrict__ out,
                                                          int64_t ldo, int C, int taps) {
    const int64_t r = blockIdx.x;
    const int ch = blockIdx.y * 256 + threadIdx.x;
    if (ch >= C) return;
    const int slot = meta[4 * r], pos = meta[4 * r + 1], idx = meta[4 * r + 2];
    float acc = bias ? to_f32(bias[ch]) : 0.0f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;                     // how many tokens before this one
        float v = 0.0f;
        if (back <= idx)
            v = to_f32(x[(r - back) * ldx + ch]);
        else if (pos - back >= 0)
            v = to_f32(state[(int64_t)slot * slot_stride + (int64_t)(taps - 1 - (back - idx)) * C + ch]);
        acc += to_f32(w[(int64_t)ch * taps + j]) * v;
    }
    if (silu) acc = acc / (1.0f + expf(-acc));
    out[r * ldo + ch] = from_f32<E>(acc);
}

template <typename E>
__global__ __launch_bounds__(256) void conv_state_kernel(const E* __restrict__ x, int64_t ldx, const int32_t* __restrict__ reqs,
                                                         E* __restrict__ state, int64_t slot_stride, int C, int taps) {
    const int32_t* rq = reqs + 4 * blockIdx.x;
    const int slot = rq[0], pos0 = rq[1], count = rq[2], row0 = rq[3];
    const int ch = blockIdx.y * 256 + threadIdx.x;
    if (ch >= C) return;
    E* st = state + (int64_t)slot * slot_stride;
    E keep[MAX_TAPS];
    const int m1 = taps - 1;
#pragma unroll
    for (int m = 0; m < MAX_TAPS; ++m) {
        if (m >= m1) break;
        const int p = pos0 + count - m1 + m;              // the position state row m holds after the step
        E v = from_f32<E>(0.0f);
        if (p >= pos0)
            v = x[(int64_t)(row0 + p - pos0) * ldx + ch];
        else if (p >= 0)
            v = st[(int64_t)(m + count) * C + ch];
        keep[m] = v;
    }
#pragma unroll
    for (int m = 0; m < MAX_TAPS; ++m) {
        if (m >= m1) break;
        st[(int64_t)m * C + ch] = keep[m];
    }
}

// ---- selective scan ---------------------------------------------------------------------------------------------------------------
// Four lanes share a channel: lane `sub` owns states sub, sub + 4, ... (NPL of them at most); a workgroup holds 64 channels of one
// request and walks its tokens in order, the next token's operands requested before the current one's arithmetic.
template <typename E, int NPL>
__global__ __launch_bounds__(256) void selective_scan_kernel(pcb_selective_scan_args a) {
    const int32_t* rq = a.reqs + 4 * blockIdx.x;
    const int slot = rq[0], pos0 = rq[1], count = rq[2], row0 = rq[3];
    const int sub = threadIdx.x & 3, ch = blockIdx.y * 64 + (threadIdx.x >> 2);
    const int C = a.C, N = a.N;
    const bool ok = ch < C;
    const int chc = ok ? ch : C - 1;
    float* st = a.state + (int64_t)slot * a.slot_stride + (int64_t)chc * N;
    float S[NPL], A[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int n = sub + 4 * i;
        A[i] = n < N ? a.A[(int64_t)chc * N + n] : 0.0f;
        S[i] = (pos0 > 0 && n < N) ? st[n] : 0.0f;
    }
    const float Dv = a.D ? a.D[chc] : 0.0f;
    const E* x = (const E*)a.x;
    const E* z = (const E*)a.z;
    E* out = (E*)a.out;

    float dt_n = 0.f, x_n = 0.f, z_n = 0.f, B_n[NPL], C_n[NPL];
    auto fetch = [&](int t) {
        const int64_t r = row0 + t;
        dt_n = a.dt[r * a.lddt + chc];
        x_n = to_f32(x[r * a.ldx + chc]);
        z_n = z ? to_f32(z[r * a.ldz + chc]) : 0.0f;
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
            const int n = sub + 4 * i;
            B_n[i] = n < N ? a.B[r * a.ldbc + n] : 0.0f;
            C_n[i] = n < N ? a.Cm[r * a.ldbc + n] : 0.0f;
        }
    };
    if (count > 0) fetch(0);
    float dsum = 0.0f;
    for (int t = 0; t < count; ++t) {
        const float dt = dt_n, xv = x_n, zv = z_n;
        dsum += dt;
        float Bc[NPL], Cc[NPL];
#pragma unroll
        for (int i = 0; i < NPL; ++i) Bc[i] = B_n[i], Cc[i] = C_n[i];
        if (t + 1 < count) fetch(t + 1);
        const float dx = dt * xv;
        float y = 0.0f;
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
            S[i] = expf(dt * A[i]) * S[i] + dx * Bc[i];
            y += S[i] * Cc[i];
        }
        y += __shfl_xor(y, 1, 64);
        y += __shfl_xor(y, 2, 64);
        if (sub == 0 && ok && out) {
            y += Dv * xv;
            if (z) y *= zv / (1.0f + expf(-zv));
            out[(int64_t)(row0 + t) * a.ldo + ch] = from_f32<E>(y);
        }
    }
    if (!ok) return;
    if (a.dt_sum && sub == 0) a.dt_sum[(int64_t)blockIdx.x * C + ch] = dsum;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int n = sub + 4 * i;
        if (n < N) st[n] = S[i];
    }
}

// ---- chaining the segments of a long prefill ----------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void state_chain_kernel(const float* __restrict__ local, float* __restrict__ start, float* __restrict__ state,
                                                          int64_t slot_stride, const int32_t* __restrict__ chains,
                                                          const float* __restrict__ coef, const float* __restrict__ x, int elems, int group) {
    const int32_t* ch = chains + 4 * blockIdx.x;
    const int slot = ch[0], pos0 = ch[1], g0 = ch[2], ng = ch[3];
    const int e = blockIdx.y * 256 + threadIdx.x;
    if (e >= elems) return;
    const int groups = elems / group;
    float* st = state + (int64_t)slot * slot_stride + e;
    float s = pos0 > 0 ? *st : 0.0f;
    const float cf = coef[e];
    for (int g = g0; g < g0 + ng; ++g) {
        start[(int64_t)g * elems + e] = s;
        s = expf(cf * x[(int64_t)g * groups + e / group]) * s + local[(int64_t)g * elems + e];
    }
    *st = s;
}

template <typename E>
int launch_scan(const pcb_selective_scan_args& a, hipStream_t stream) {
    const dim3 grid(a.n_reqs, pcb_ceil_div(a.C, 64));
    if (a.N <= 16)
        hipLaunchKernelGGL((selective_scan_kernel<E, 4>), grid, dim3(256), 0, stream, a);
    else if (a.N <= 32)
        hipLaunchKernelGGL((selective_scan_kernel<E, 8>), grid, dim3(256), 0, stream, a);
    else if (a.N <= 64)
        hipLaunchKernelGGL((selective_scan_kernel<E, 16>), grid, dim3(256), 0, stream, a);
    else
        hipLaunchKernelGGL((selective_scan_kernel<E, 64>), grid, dim3(256), 0, stream, a);
    return pcb_check_launch("selective_scan_kernel");
}

}  // namespace

PCB_EXPORT int pcb_decay_attn(const pcb_decay_attn_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_decay_attn_args), PCB_ERR_ARG, "pcb_decay_attn: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_decay_attn: unknown dtype");
    PCB_REQUIRE(a->n_reqs >= 0 && a->H > 0 && a->dim > 0 && a->dim <= 256 && a->vdim > 0 && a->ldq >= (int64_t)a->H * a->dim &&
                    a->ldk >= (int64_t)a->H * a->dim && a->ldv >= (int64_t)a->H * a->vdim && (!a->out || a->ldo >= (int64_t)a->H * a->vdim) &&
                    a->slot_stride >= (int64_t)a->H * a->dim * a->vdim && pcb_ceil_div(a->vdim, 16) <= 65535 && a->H <= 65535,
                PCB_ERR_ARG, "pcb_decay_attn: bad sizes (key size up to 256)");
    if (a->n_reqs == 0) return PCB_OK;
    PCB_REQUIRE(a->q && a->k && a->v && a->reqs && a->state && a->decay, PCB_ERR_ARG, "pcb_decay_attn: null pointer");
    return a->dtype == PCB_BF16 ? launch_decay<pcb::bf16_t>(*a, (hipStream_t)stream) : launch_decay<float>(*a, (hipStream_t)stream);
}

PCB_EXPORT int pcb_causal_conv(const void* x, int64_t ldx, const void* w, const void* bias, int32_t dtype, int32_t silu,
                               const int32_t* row_meta, const void* state, int64_t slot_stride, void* out, int64_t ldo, int32_t n_rows,
                               int32_t C, int32_t taps, void* stream) {
    PCB_REQUIRE((dtype == PCB_BF16 || dtype == PCB_F32) && n_rows >= 0 && C > 0 && taps >= 1 && taps <= MAX_TAPS && ldx >= C && ldo >= C &&
                    slot_stride >= (int64_t)(taps - 1) * C,
                PCB_ERR_ARG, "pcb_causal_conv: bad sizes (1 <= taps <= 16)");
    if (n_rows == 0) return PCB_OK;
    PCB_REQUIRE(x && w && row_meta && out && (taps == 1 || state), PCB_ERR_ARG, "pcb_causal_conv: null pointer");
    const dim3 grid(n_rows, pcb_ceil_div(C, 256));
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(causal_conv_kernel<pcb::bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const pcb::bf16_t*)x, ldx,
                           (const pcb::bf16_t*)w, (const pcb::bf16_t*)bias, silu, row_meta, (const pcb::bf16_t*)state, slot_stride,
                           (pcb::bf16_t*)out, ldo, C, taps);
    else
        hipLaunchKernelGGL(causal_conv_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)x, ldx, (const float*)w,
                           (const float*)bias, silu, row_meta, (const float*)state, slot_stride, (float*)out, ldo, C, taps);
    return pcb_check_launch("causal_conv_kernel");
}

PCB_EXPORT int pcb_conv_state_update(const void* x, int64_t ldx, int32_t dtype, const int32_t* reqs, int32_t n_reqs, void* state,
                                     int64_t slot_stride, int32_t C, int32_t taps, void* stream) {
    PCB_REQUIRE((dtype == PCB_BF16 || dtype == PCB_F32) && n_reqs >= 0 && C > 0 && taps >= 1 && taps <= MAX_TAPS && ldx >= C &&
                    slot_stride >= (int64_t)(taps - 1) * C,
                PCB_ERR_ARG, "pcb_conv_state_update: bad sizes (1 <= taps <= 16)");
    if (n_reqs == 0 || taps == 1) return PCB_OK;
    PCB_REQUIRE(x && reqs && state, PCB_ERR_ARG, "pcb_conv_state_update: null pointer");
    const dim3 grid(n_reqs, pcb_ceil_div(C, 256));
    if (dtype == PCB_BF16)
        hipLaunchKernelGGL(conv_state_kernel<pcb::bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const pcb::bf16_t*)x, ldx, reqs,
                           (pcb::bf16_t*)state, slot_stride, C, taps);
    else
        hipLaunchKernelGGL(conv_state_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)x, ldx, reqs, (float*)state,
                           slot_stride, C, taps);
    return pcb_check_launch("conv_state_kernel");
}

PCB_EXPORT int pcb_selective_scan(const pcb_selective_scan_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_selective_scan_args), PCB_ERR_ARG, "pcb_selective_scan: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_selective_scan: unknown dtype");
    PCB_REQUIRE(a->n_reqs >= 0 && a->C > 0 && a->N > 0 && a->N <= 256 && a->ldx >= a->C && a->lddt >= a->C && a->ldbc >= a->N &&
                    (!a->out || a->ldo >= a->C) && (!a->z || a->ldz >= a->C) && a->slot_stride >= (int64_t)a->C * a->N,
                PCB_ERR_ARG, "pcb_selective_scan: bad sizes (up to 256 states per channel)");
    if (a->n_reqs == 0) return PCB_OK;
    PCB_REQUIRE(a->x && a->dt && a->B && a->Cm && a->A && a->reqs && a->state, PCB_ERR_ARG, "pcb_selective_scan: null pointer");
    return a->dtype == PCB_BF16 ? launch_scan<pcb::bf16_t>(*a, (hipStream_t)stream) : launch_scan<float>(*a, (hipStream_t)stream);
}

PCB_EXPORT int pcb_state_chain(const float* local, float* start, float* state, int64_t slot_stride, const int32_t* chains, int32_t n_chains,
                               const float* coef, const float* x, int32_t elems, int32_t group, void* stream) {
    PCB_REQUIRE(n_chains >= 0 && elems > 0 && group > 0 && elems % group == 0 && slot_stride >= elems && pcb_ceil_div(elems, 256) <= 65535,
                PCB_ERR_ARG, "pcb_state_chain: bad sizes");
    if (n_chains == 0) return PCB_OK;
    PCB_REQUIRE(local && start && state && chains && coef && x, PCB_ERR_ARG, "pcb_state_chain: null pointer");
    hipLaunchKernelGGL(state_chain_kernel, dim3(n_chains, pcb_ceil_div(elems, 256)), dim3(256), 0, (hipStream_t)stream, local, start, state,
                       slot_stride, chains, coef, x, elems, group);
    return pcb_check_launch("state_chain_kernel");
}
