// pcb_attn_talk: causal attention whose heads exchange their scores before the softmax ("talking heads"), over a key cache that
// doubles as the value cache, with a linear distance bias, a sliding window and an optional value-less sink in the denominator.
//
// Mixing couples all heads of one (query, key) pair, so the work is cut differently from per-head flash attention:
//   1. talk_scores_kernel: one wave owns a 16-query x 16-key tile and computes it for EVERY head on the matrix cores; with the
//      MFMA result layout a lane then holds the same four (query, key) pairs of all heads, so bias, mixing
//      (H x H fp32 multiply-adds per pair) and the window test are lane-local.  The mixed scores go to an fp32 band
//      [row][head][distance i - j] -- no softmax state, hence no coupling between key tiles: the grid runs over key blocks too.
//   2. talk_values_kernel: per (query tile, head): row maximum and denominator from the band (the sink enters as a score of 0),
//      then P V on the matrix cores with the keys as values; bf16 runs P as a hi + lo pair so the fp32 weights are not rounded.
#include "pb_common.h"

namespace {
using namespace pcb;

struct TileRec {
    int32_t slot, q0, nq, row0;
};

template <typename E, int HMAX>
__global__ __launch_bounds__(256) void talk_scores_kernel(pcb_attn_talk_args a, int band) {
    __shared__ float talk[HMAX * HMAX];
    __shared__ float slope[HMAX];
    const int H = a.H, D = a.head_dim, rep = H / a.Hkv;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, group = lane >> 4, l15 = lane & 15;
    const TileRec t = reinterpret_cast<const TileRec*>(a.tiles)[blockIdx.x];
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_last = t.q0 + t.nq - 1;
    const int j_min = t.q0 - window + 1 > 0 ? t.q0 - window + 1 : 0;
    const int j0 = j_min + 64 * blockIdx.y + 16 * wave;          // this wave's 16 keys
    if (j_min + 64 * (int)blockIdx.y > i_last) return;            // (uniform over the workgroup)
    for (int e = tid; e < H * H; e += 256) talk[e] = a.talk ? a.talk[e] : ((e / H == e % H) ? 1.0f : 0.0f);
    for (int e = tid; e < H; e += 256) slope[e] = a.slopes ? a.slopes[e] : 0.0f;
    __syncthreads();
    if (j0 > i_last) return;

    const E* Q = (const E*)a.q;
    const E* C = (const E*)a.cache + (int64_t)t.slot * a.slot_stride;
    const bool vec = sizeof(E) == 2 && D % 8 == 0 && a.ldq % 8 == 0 && a.head_stride % 8 == 0 && a.slot_stride % 8 == 0 &&
                     (((uintptr_t)Q | (uintptr_t)a.cache) % 16 == 0);
    const int jk = j0 + l15;                                      // the key this lane loads (as a B-operand row)
    const bool key_ok = jk <= i_last;
    const bool q_ok = l15 < t.nq;

    float s[HMAX][4];
#pragma unroll
    for (int h = 0; h < HMAX; ++h) {
        if (h < H) {
            const E* qrow = Q + (int64_t)(t.row0 + l15) * a.ldq + h * D;
            const E* krow = C + (int64_t)(h / rep) * a.head_stride + (int64_t)jk * D;
            f4 acc = f4{0.f, 0.f, 0.f, 0.f};
            for (int k0 = 0; k0 < D; k0 += 32) {
                const Frag<E> fq = load_frag(qrow + k0, group, q_ok ? D - k0 : 0, vec);
                const Frag<E> fk = load_frag(krow + k0, group, key_ok ? D - k0 : 0, vec);
                acc = mma(fq, fk, acc);
            }
            // lane: key column l15 (j = j0 + l15), query rows 4 * group + r
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int dist = t.q0 + 4 * group + r - jk;
                s[h][r] = acc[r] * a.scale - slope[h] * (float)dist;
            }
        }
    }
    const bool mix = a.talk != nullptr;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int qr = 4 * group + r;
        const int dist = t.q0 + qr - jk;
        const bool ok = qr < t.nq && dist >= 0 && dist < window && jk >= 0;
        if (!ok) continue;
        float* dst = a.scratch + ((int64_t)(t.row0 + qr) * H) * band + dist;
#pragma unroll
        for (int h = 0; h < HMAX; ++h) {
            if (h < H) {
                float v = s[h][r];
                if (mix) {
                    v = 0.0f;
#pragma unroll
                    for (int g2 = 0; g2 < HMAX; ++g2)
                        if (g2 < H) v += talk[h * H + g2] * s[g2][r];
                }
                dst[(int64_t)h * band] = v;
            }
        }
    }
}

template <typename E>
__global__ __launch_bounds__(256) void talk_values_kernel(pcb_attn_talk_args a, int band) {
    constexpr bool SPLIT = sizeof(E) == 2;           // bf16: P as hi + lo
    constexpr int LD = 32 + 16 / sizeof(E);
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    __shared__ float row_m[16], row_inv[16];
    __shared__ __attribute__((aligned(16))) E Ph[16 * LD];
    __shared__ __attribute__((aligned(16))) E Pl[SPLIT ? 16 * LD : 1];
    E* Vt = reinterpret_cast<E*>(lds_raw);           // [D16][LD]: Vt[d][key]
    const int H = a.H, D = a.head_dim, rep = H / a.Hkv;
    const int D16 = (D + 15) / 16 * 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, group = lane >> 4, l15 = lane & 15;
    const TileRec t = reinterpret_cast<const TileRec*>(a.tiles)[blockIdx.x];
    const int h = blockIdx.y;
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_last = t.q0 + t.nq - 1;
    const int j_min = t.q0 - window + 1 > 0 ? t.q0 - window + 1 : 0;
    const float* S = a.scratch + ((int64_t)t.row0 * H + h) * band;         // row r of the tile: + r * H * band
    const int64_t s_row = (int64_t)H * band;

    // row statistics: wave w takes rows w, w + 4, ...
    for (int r = wave; r < t.nq; r += 4) {
        const int i = t.q0 + r;
        const int n = i + 1 < window ? i + 1 : window;
        const float* sr = S + r * s_row;
        float m = a.sink ? 0.0f : -INFINITY;
        for (int d = lane; d < n; d += 64) m = fmaxf(m, sr[d]);
        m = wave_max(m);
        float l = 0.0f;
        for (int d = lane; d < n; d += 64) l += expf(sr[d] - m);
        l = wave_sum(l);
        if (a.sink) l += expf(-m);
        if (lane == 0) row_m[r] = m, row_inv[r] = 1.0f / l;
    }
    __syncthreads();

    const E* V = (const E*)a.cache + (int64_t)t.slot * a.slot_stride + (int64_t)(h / rep) * a.head_stride;
    f4 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};
    const int n_dt = D16 / 16;

    for (int j0 = j_min; j0 <= i_last; j0 += 32) {
        // weights of 16 rows x 32 keys
        for (int e = tid; e < 16 * 32; e += 256) {
            const int r = e >> 5, kk = e & 31;
            const int j = j0 + kk, dist = t.q0 + r - j;
            float p = 0.0f;
            if (r < t.nq && dist >= 0 && dist < window) p = expf(S[r * s_row + dist] - row_m[r]) * row_inv[r];
            if (SPLIT) {
                const E hi = from_f32<E>(p);
                Ph[r * LD + kk] = hi;
                Pl[r * LD + kk] = from_f32<E>(p - to_f32(hi));
            } else {
                Ph[r * LD + kk] = from_f32<E>(p);
            }
        }
        // the keys as values, transposed: Vt[d][kk]
        for (int e = tid; e < 32 * D16; e += 256) {
            const int kk = e / D16, d = e % D16;
            const int j = j0 + kk;
            Vt[d * LD + kk] = (j <= i_last && d < D) ? V[(int64_t)j * D + d] : from_f32<E>(0.0f);
        }
        __syncthreads();
        const Frag<E> ph = load_frag(&Ph[l15 * LD], group, 32, true);
        Frag<E> pl;
        if (SPLIT) pl = load_frag(&Pl[l15 * LD], group, 32, true);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int dt = wave + 4 * i;
            if (dt < n_dt) {
                const Frag<E> fv = load_frag(&Vt[(dt * 16 + l15) * LD], group, 32, true);
                acc[i] = mma(ph, fv, acc[i]);
                if (SPLIT) acc[i] = mma(pl, fv, acc[i]);
            }
        }
        __syncthreads();
    }
    E* O = (E*)a.out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int d = (wave + 4 * i) * 16 + l15;
        if (wave + 4 * i < n_dt && d < D) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int qr = 4 * group + r;
                if (qr < t.nq) O[(int64_t)(t.row0 + qr) * a.ldo + h * D + d] = from_f32<E>(acc[i][r]);
            }
        }
    }
}

template <typename E>
int run(const pcb_attn_talk_args& a, int band, hipStream_t stream) {
    const int H = a.H;
    const int key_blocks = pcb_ceil_div(band + 15, 64);
    const dim3 g1(a.n_tiles, key_blocks);
    if (H <= 4)
        hipLaunchKernelGGL((talk_scores_kernel<E, 4>), g1, dim3(256), 0, stream, a, band);
    else if (H <= 8)
        hipLaunchKernelGGL((talk_scores_kernel<E, 8>), g1, dim3(256), 0, stream, a, band);
    else if (H <= 16)
        hipLaunchKernelGGL((talk_scores_kernel<E, 16>), g1, dim3(256), 0, stream, a, band);
    else
        hipLaunchKernelGGL((talk_scores_kernel<E, 32>), g1, dim3(256), 0, stream, a, band);
    int rc = pcb_check_launch("talk_scores_kernel");
    if (rc != PCB_OK) return rc;
    const int D16 = (a.head_dim + 15) / 16 * 16;
    const size_t lds = (size_t)D16 * (32 + 16 / sizeof(E)) * sizeof(E);
    hipLaunchKernelGGL((talk_values_kernel<E>), dim3(a.n_tiles, H), dim3(256), lds, stream, a, band);
    return pcb_check_launch("talk_values_kernel");
}

}  // namespace

PCB_EXPORT int32_t pcb_attn_talk_band(int32_t window, int32_t max_kv_len) {
    const int b = (window > 0 && window < max_kv_len) ? window : max_kv_len;
    return b < 1 ? 1 : b;
}

PCB_EXPORT int pcb_attn_talk(const pcb_attn_talk_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_attn_talk_args), PCB_ERR_ARG, "pcb_attn_talk: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_attn_talk: unknown dtype");
    PCB_REQUIRE(a->H > 0 && a->H <= 32 && a->Hkv > 0 && a->H % a->Hkv == 0 && a->head_dim > 0 && a->head_dim <= 256, PCB_ERR_ARG,
                "pcb_attn_talk: heads <= 32, kv heads | heads, head_dim <= 256");
    PCB_REQUIRE(a->n_tiles >= 0 && a->max_kv_len > 0, PCB_ERR_ARG, "pcb_attn_talk: bad sizes");
    if (a->n_tiles == 0) return PCB_OK;
    PCB_REQUIRE(a->q && a->tiles && a->cache && a->scratch && a->out, PCB_ERR_ARG, "pcb_attn_talk: null pointer");
    PCB_REQUIRE(a->ldq >= (int64_t)a->H * a->head_dim && a->ldo >= (int64_t)a->H * a->head_dim, PCB_ERR_ARG,
                "pcb_attn_talk: row strides shorter than heads * head_dim");
    const int band = pcb_attn_talk_band(a->window, a->max_kv_len);
    PCB_REQUIRE(a->scratch_floats >= (int64_t)a->n_tiles * 16 * a->H * band, PCB_ERR_ARG,
                "pcb_attn_talk: scratch holds %lld floats, %lld needed", (long long)a->scratch_floats,
                (long long)a->n_tiles * 16 * a->H * band);
    return a->dtype == PCB_BF16 ? run<pcb::bf16_t>(*a, band, (hipStream_t)stream) : run<float>(*a, band, (hipStream_t)stream);
}
