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
// fragments of S^T Q^T: the k index of that product runs over the key columns in the order (l >> 4, 4 i + u) -> 16 i + 4 (l >> 4) + u,
// which the query operand follows.
// four consecutive elements of a row as floats; `valid` of them exist (<= 0: none); `vec`: one 8- or 16-byte load is allowed
__device__ __forceinline__ void load4(const bf16_t* p, bool vec, int valid, float (&o)[4]) {
    if (vec && valid >= 4) {
        const uint2 w = *reinterpret_cast<const uint2*>(p);
        o[0] = __uint_as_float(w.x << 16), o[1] = __uint_as_float(w.x & 0xffff0000u);
        o[2] = __uint_as_float(w.y << 16), o[3] = __uint_as_float(w.y & 0xffff0000u);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = i < valid ? to_f32(p[i]) : 0.0f;
    }
}
__device__ __forceinline__ void load4(const float* p, bool vec, int valid, float (&o)[4]) {
    if (vec && valid >= 4) {
        const float4 w = *reinterpret_cast<const float4*>(p);
        o[0] = w.x, o[1] = w.y, o[2] = w.z, o[3] = w.w;
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = i < valid ? p[i] : 0.0f;
    }
}

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
    constexpr int A4 = 4 * sizeof(E);
    const bool vec = dim % 4 == 0 && a.ldq % 4 == 0 && a.ldk % 4 == 0 && (uintptr_t)a.q % A4 == 0 && (uintptr_t)a.k % A4 == 0;

    // operands with the token in the lane's row (l & 15): q as the B side, k as the A side; element 4 i + u of lane group g is key
    // column 16 i + 4 g + u -- four consecutive columns per load.  The next chunk's are requested while this chunk computes.
    float qn[NB][4] = {}, kn[NB][4] = {};
    auto fetch_rows = [&](int c0) {
        const int n = count - c0 < 16 ? count - c0 : 16;
        const E* qrow = Q + (row0 + c0 + c) * a.ldq;
        const E* krow = K + (row0 + c0 + c) * a.ldk;
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int d0 = 16 * i + 4 * g;
            const int valid = c < n ? dim - d0 : 0;
            load4(qrow + d0, vec, valid, qn[i]);
            load4(krow + d0, vec, valid, kn[i]);
        }
    };
    if (count > 0 && a.out) fetch_rows(0);

    for (int c0 = 0; c0 < count; c0 += 16) {
        const int n = count - c0 < 16 ? count - c0 : 16;
        const int64_t r0 = row0 + c0;
        const bool t_ok = c < n;
        float qc[NB][4], kc[NB][4];
#pragma unroll
        for (int i = 0; i < NB; ++i)
#pragma unroll
            for (int u = 0; u < 4; ++u) qc[i][u] = qn[i][u], kc[i][u] = kn[i][u];
        // this chunk's operands with the token in the k index (element e of lane group g is token 4 g + e), then the next chunk's rows
        float vv[4], kt[NB][4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j = 4 * g + e;
            vv[e] = (j < n && v_ok) ? to_f32(V[(r0 + j) * a.ldv + vcol]) : 0.0f;
#pragma unroll
            for (int b = 0; b < NB; ++b) kt[b][e] = (j < n && 16 * b + c < dim) ? to_f32(K[(r0 + j) * a.ldk + 16 * b + c]) : 0.0f;
        }
        if (c0 + 16 < count && a.out) fetch_rows(c0 + 16);

        if (a.out) {                                        // (a states-only pass skips the scores and the outputs)
            f4 wt = f4{0.f, 0.f, 0.f, 0.f}, ot = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    wt = mma4(kc[i][u], qc[i][u], wt);
                    ot = mma4(S[i][u], qc[i][u], ot);
                }
            // wt: column t = c, rows j = 4 g + r;  ot: column t = c, rows = value columns 4 g + r
            const float lt1 = decay_pow(lg, c + 1);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = 4 * g + r;
                wt[r] = (j <= c && j < n) ? wt[r] * decay_pow(lg, c - j) : 0.0f;
                ot[r] *= lt1;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) ot = mma4(vv[e], wt[e], ot);
            if (t_ok) {
                float* op = a.out + (r0 + c) * a.ldo + (int64_t)h * vdim + blockIdx.z * 16;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (blockIdx.z * 16 + 4 * g + r < vdim) op[4 * g + r] = ot[r];
            }
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
#pragma unroll
            for (int e = 0; e < 4; ++e) s = mma4(kt[b][e] * kd[e], vv[e], s);
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
// LPC lanes share a channel: lane `sub` owns states sub, sub + LPC, ... (NPL of them at most); a workgroup holds 256 / LPC channels
// of one request and walks its tokens in order, later tokens' operands requested before the current one's arithmetic.  LPC = 1
// (up to 32 states): a lane owns its channel's whole state, B and C of a token are the same for every lane (scalar loads), and
// nothing is reduced across lanes; LPC = 4 spreads larger states over four lanes.
template <typename E, int NPL, int LPC>
__global__ __launch_bounds__(256) void selective_scan_kernel(pcb_selective_scan_args a) {
    const int32_t* rq = a.reqs + 4 * blockIdx.x;
    const int slot = rq[0], pos0 = rq[1], count = rq[2], row0 = rq[3];
    const int sub = threadIdx.x % LPC, ch = blockIdx.y * (256 / LPC) + threadIdx.x / LPC;
    const int C = a.C, N = a.N;
    const bool ok = ch < C;
    const int chc = ok ? ch : C - 1;
    float* st = a.state + (int64_t)slot * a.slot_stride + (int64_t)chc * N;
    float S[NPL], A[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int n = sub + LPC * i;
        A[i] = n < N ? a.A[(int64_t)chc * N + n] * 1.44269504088896f : 0.0f;     // exp(dt A) = exp2(dt A log2(e))
        S[i] = (pos0 > 0 && n < N) ? st[n] : 0.0f;
    }
    const float Dv = a.D ? a.D[chc] : 0.0f;
    const E* x = (const E*)a.x;
    const E* z = (const E*)a.z;
    E* out = (E*)a.out;

    // a ring of PF tokens' operands: token t waits in slot t % PF and is replaced by token t + PF once it has been used, so PF
    // tokens' loads are in flight while one token's arithmetic runs.  Row pointers advance by their strides (no 64-bit products
    // in the loop); state columns past N read column N - 1 and are masked out of the sums.
    constexpr int PF = NPL <= 4 ? 4 : (NPL <= 8 ? 2 : 1);
    constexpr bool RING_BC = NPL <= 16;                     // (large states read B and C where they are used: registers go to the state)
    float dt_r[PF], x_r[PF], z_r[PF], B_r[PF][RING_BC ? NPL : 1], C_r[PF][RING_BC ? NPL : 1];
    constexpr bool TAB = NPL <= 16;                         // (large states: recomputed in place, the registers go to the state)
    int ncol[TAB ? NPL : 1];
    float keep[TAB ? NPL : 1];
#pragma unroll
    for (int i = 0; i < (TAB ? NPL : 1); ++i) {
        const int n = sub + LPC * i;
        ncol[i] = n < N ? n : N - 1;
        keep[i] = n < N ? 1.0f : 0.0f;
    }
    auto col = [&](int i) { return TAB ? ncol[TAB ? i : 0] : (sub + LPC * i < N ? sub + LPC * i : N - 1); };
    auto kept = [&](int i) { return TAB ? keep[TAB ? i : 0] : (sub + LPC * i < N ? 1.0f : 0.0f); };
    const bool with_out = out != nullptr, with_z = z != nullptr && with_out;
    const float* dtp = a.dt + (int64_t)row0 * a.lddt + chc;
    const E* xp = x + (int64_t)row0 * a.ldx + chc;
    const E* zp = with_z ? z + (int64_t)row0 * a.ldz + chc : nullptr;
    const float* bp = a.B + (int64_t)row0 * a.ldbc;
    const float* cp = a.Cm + (int64_t)row0 * a.ldbc;
    auto fetch = [&](int u) {                               // the next row the pointers stand at, into slot u
        dt_r[u] = *dtp;
        x_r[u] = to_f32(*xp);
        z_r[u] = with_z ? to_f32(*zp) : 0.0f;
#pragma unroll
        for (int i = 0; i < (RING_BC ? NPL : 0); ++i) {
            B_r[u][i] = bp[col(i)];
            C_r[u][i] = with_out ? cp[col(i)] : 0.0f;
        }
        dtp += a.lddt, xp += a.ldx, bp += a.ldbc, cp += a.ldbc;
        if (with_z) zp += a.ldz;
    };
#pragma unroll
    for (int u = 0; u < PF; ++u)
        if (u < count) fetch(u);
    float dsum = 0.0f;
    E* op = with_out ? out + (int64_t)row0 * a.ldo + ch : nullptr;
    const float* bq = a.B + (int64_t)row0 * a.ldbc;         // (the current token's B and C rows, for the states that do not ring)
    const float* cq = a.Cm + (int64_t)row0 * a.ldbc;
    for (int t0 = 0; t0 < count; t0 += PF) {
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            const int t = t0 + u;
            if (t >= count) break;
            const float dt = dt_r[u], xv = x_r[u], zv = z_r[u];
            float Bc[RING_BC ? NPL : 1], Cc[RING_BC ? NPL : 1];
#pragma unroll
            for (int i = 0; i < (RING_BC ? NPL : 0); ++i) Bc[i] = B_r[u][i], Cc[i] = C_r[u][i];
            if (t + PF < count) fetch(u);
            dsum += dt;
            const float dx = dt * xv;
            float y = 0.0f;
#pragma unroll
            for (int i = 0; i < NPL; ++i) {
                const float b = RING_BC ? Bc[RING_BC ? i : 0] : bq[col(i)];
                S[i] = __builtin_amdgcn_exp2f(dt * A[i]) * S[i] + dx * b;            // (dt A <= 0: no overflow; tiny results flush to 0)
                if (with_out) y += kept(i) * S[i] * (RING_BC ? Cc[RING_BC ? i : 0] : cq[col(i)]);
            }
            bq += a.ldbc, cq += a.ldbc;
            if (!with_out) continue;                        // (a states-only pass)
            if (LPC == 4) {
                y += __shfl_xor(y, 1, 64);
                y += __shfl_xor(y, 2, 64);
            }
            if (sub == 0 && ok) {
                y += Dv * xv;
                if (with_z) y *= zv * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896f * zv));
                *op = from_f32<E>(y);
            }
            op += a.ldo;
        }
    }
    if (!ok) return;
    if (a.dt_sum && sub == 0) a.dt_sum[(int64_t)blockIdx.x * C + ch] = dsum;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int n = sub + LPC * i;
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
    // (one lane per channel -- LPC = 1, scalar B / C loads, no reduction -- was measured at 16 states: 220 us against 125 us per
    // pass for 2 048 tokens x 4 096 channels, and 11.5 against 5.5 us at decode: a quarter of the waves, each four times as long)
    const dim3 four(a.n_reqs, pcb_ceil_div(a.C, 64));
    if (a.N <= 16)
        hipLaunchKernelGGL((selective_scan_kernel<E, 4, 4>), four, dim3(256), 0, stream, a);
    else if (a.N <= 32)
        hipLaunchKernelGGL((selective_scan_kernel<E, 8, 4>), four, dim3(256), 0, stream, a);
    else if (a.N <= 64)
        hipLaunchKernelGGL((selective_scan_kernel<E, 16, 4>), four, dim3(256), 0, stream, a);
    else
        hipLaunchKernelGGL((selective_scan_kernel<E, 64, 4>), four, dim3(256), 0, stream, a);
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
