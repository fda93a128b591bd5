// pcb_attn_talk: causal attention whose heads exchange their scores before the softmax ("talking heads"), over a key cache that
// doubles as the value cache, with a linear distance bias, a sliding window and an optional value-less sink in the denominator.
//
// Mixing couples all heads of one (query, key) pair, so the work is cut differently from per-head flash attention:
//   1. talk_scores_kernel: one wave owns a 16-query x 16-key tile and computes it for EVERY head on the matrix cores; with the
//      MFMA result layout a lane then holds the same four (query, key) pairs of all heads, so bias, mixing
//      (H x H fp32 multiply-adds per pair) and the window test are lane-local.  The mixed scores go to an fp32 band
//      [row][head][distance i - j] -- no softmax state, hence no coupling between key tiles: the grid runs over key blocks too.
//   2. talk_values_kernel: per (up to 64 queries, head): one sweep over the band with a running maximum and denominator per row
//      (the sink enters as a score of 0), P V on the matrix cores with the keys as values; bf16 runs P as a hi + lo pair so the
//      fp32 weights are not rounded.  Tiles of at most 4 rows (decoding) take talk_values_few_kernel: fp32 multiply-adds over
//      coalesced key rows, no matrix cores.
#include "pb_common.h"

namespace {
using namespace pcb;

struct TileRec {
    int32_t slot, q0, nq, row0;
};

// ---- 1. scores ---------------------------------------------------------------------------------------------------------------
// Workgroup = one 16-query tile x KC keys (128, or 64 when the launch has few tiles: decoding); a wave owns 16-key subtiles of
// them, one after the other.  The tile's queries (all
// heads) wait in LDS when they fit (q_lds), so the per-subtile traffic is the keys alone; a key fragment is loaded once per key
// head and used by every query head of its group.

template <typename E, int HMAX, int NST, int PG>
__global__ __launch_bounds__(256) void talk_scores_kernel(pcb_attn_talk_args a, int band, int q_lds, int qld, int KC) {
    extern __shared__ __attribute__((aligned(16))) unsigned char dyn[];
    __shared__ __attribute__((aligned(16))) float talk[HMAX * HMAX];      // [h][g], rows padded with zeros
    __shared__ float slope[HMAX];
    const int H = a.H, D = a.head_dim, rep = H / a.Hkv, HD = H * D;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, group = lane >> 4, l15 = lane & 15;
    const TileRec t = reinterpret_cast<const TileRec*>(a.tiles)[blockIdx.x];
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_last = t.q0 + t.nq - 1;
    const int j_min = t.q0 - window + 1 > 0 ? t.q0 - window + 1 : 0;
    const int j_blk = j_min + KC * blockIdx.y;
    if (j_blk > i_last) return;                                   // (uniform over the workgroup)
    const E* Q = (const E*)a.q;
    const E* C = (const E*)a.cache + (int64_t)t.slot * a.slot_stride;
    const bool vec = sizeof(E) == 2 && D % 8 == 0 && a.ldq % 8 == 0 && a.head_stride % 8 == 0 && a.slot_stride % 8 == 0 &&
                     (((uintptr_t)Q | (uintptr_t)a.cache) % 16 == 0);
    for (int e = tid; e < HMAX * HMAX; e += 256) {
        const int h = e / HMAX, g2 = e % HMAX;
        talk[e] = (h < H && g2 < H) ? (a.talk ? a.talk[h * H + g2] : (h == g2 ? 1.0f : 0.0f)) : 0.0f;
    }
    for (int e = tid; e < HMAX; e += 256) slope[e] = (e < H && a.slopes) ? a.slopes[e] : 0.0f;
    E* Qs = reinterpret_cast<E*>(dyn);
    if (q_lds) {
        if (vec) {
            const int cpr = HD / 8, total = 16 * cpr;
            for (int e0 = tid; e0 < total; e0 += 256 * 8) {       // eight loads in flight per thread, then their LDS stores
                u32x4 v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int e = e0 + 256 * u, r = e / cpr, c = (e % cpr) * 8;
                    v[u] = u32x4{0u, 0u, 0u, 0u};
                    if (e < total && r < t.nq) v[u] = *reinterpret_cast<const u32x4*>(Q + (int64_t)(t.row0 + r) * a.ldq + c);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int e = e0 + 256 * u, r = e / cpr, c = (e % cpr) * 8;
                    if (e < total) *reinterpret_cast<u32x4*>(Qs + r * qld + c) = v[u];
                }
            }
        } else {
            for (int e = tid; e < 16 * HD; e += 256) {
                const int r = e / HD, c = e % HD;
                Qs[r * qld + c] = r < t.nq ? Q[(int64_t)(t.row0 + r) * a.ldq + c] : from_f32<E>(0.0f);
            }
        }
    }
    __syncthreads();
    const E* qrow0 = q_lds ? Qs + l15 * qld : Q + (int64_t)(t.row0 + l15) * a.ldq;
    const bool q_ok = q_lds ? true : l15 < t.nq;
    const bool mix = a.talk != nullptr;
    const int nsteps = (D + 31) / 32;

    for (int sub = 0; sub < KC / 64; ++sub) {
        const int j0 = j_blk + 64 * sub + 16 * wave;              // this wave's 16 keys
        if (j0 > i_last) break;
        const int jk = j0 + l15;                                  // the key this lane loads (as a B-operand row)
        const bool key_ok = jk <= i_last;
        float s[HMAX][4];
#pragma unroll
        for (int h = 0; h < HMAX; ++h) s[h][0] = s[h][1] = s[h][2] = s[h][3] = 0.0f;
        // the key fragments of PG key heads are requested together (one memory round trip per PG heads, not per head)
        for (int c0 = 0; c0 < a.Hkv; c0 += PG) {
            Frag<E> fk[PG][NST];
#pragma unroll
            for (int u = 0; u < PG; ++u) {
                const bool ok = key_ok && c0 + u < a.Hkv;
                const E* krow = C + (int64_t)(ok ? c0 + u : 0) * a.head_stride + (int64_t)(ok ? jk : 0) * D;
#pragma unroll
                for (int st = 0; st < NST; ++st)
                    if (st < nsteps) fk[u][st] = load_frag(krow + 32 * st, group, ok ? D - 32 * st : 0, vec);
            }
#pragma unroll
            for (int h = 0; h < HMAX; ++h) {
                const int c = h / rep;
                if (h < H && c >= c0 && c < c0 + PG) {
                    f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int u = 0; u < PG; ++u)
                        if (c - c0 == u) {
#pragma unroll
                            for (int st = 0; st < NST; ++st)
                                if (st < nsteps) {
                                    const Frag<E> fq = load_frag(qrow0 + h * D + 32 * st, group, q_ok ? D - 32 * st : 0, vec);
                                    acc = mma(fq, fk[u][st], acc);
                                }
                        }
                    // lane: key column l15 (j = j0 + l15), query rows 4 * group + r
#pragma unroll
                    for (int r = 0; r < 4; ++r) s[h][r] = acc[r] * a.scale - slope[h] * (float)(t.q0 + 4 * group + r - jk);
                    // (a head's query fragments come from LDS and die here: keep the scheduler from hoisting all heads' reads to the
                    // top of the unrolled loop, which costs the registers of every head at once)
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int qr = 4 * group + r;
            const int dist = t.q0 + qr - jk;
            if (!(qr < t.nq && dist >= 0 && dist < window)) continue;
            float* dst = a.scratch + ((int64_t)(t.row0 + qr) * H) * band + dist;
#pragma unroll
            for (int h = 0; h < HMAX; ++h) {
                if (h < H) {
                    float v = s[h][r];
                    if (mix) {
                        v = 0.0f;
#pragma unroll
                        for (int g4 = 0; g4 < HMAX; g4 += 4) {
                            const f4 tw = *reinterpret_cast<const f4*>(&talk[h * HMAX + g4]);
                            v += tw[0] * s[g4][r] + tw[1] * s[g4 + 1][r] + tw[2] * s[g4 + 2][r] + tw[3] * s[g4 + 3][r];
                        }
                    }
                    dst[(int64_t)h * band] = v;
                }
            }
        }
    }
}

// ---- 2. values ---------------------------------------------------------------------------------------------------------------
// Workgroup = up to 64 consecutive queries of one sequence (a tile of the second table) x one head.  Per 32 keys: the rows'
// unnormalised weights into LDS (hi + lo for bf16) with a running maximum / denominator per row, the keys transposed into LDS
// once for all rows, and the (16-row subtile, 16-column subtile) products dealt round-robin to the four waves.
template <typename E, int NP>
__global__ __launch_bounds__(256) void talk_values_kernel(pcb_attn_talk_args a, int band, const int32_t* tiles) {
    constexpr bool SPLIT = sizeof(E) == 2;           // bf16: P as hi + lo
    constexpr int CE = 16 / sizeof(E), LD = 32 + CE;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    __shared__ float row_alpha[64], row_inv[64];
    __shared__ __attribute__((aligned(16))) E Ph[64 * LD];
    __shared__ __attribute__((aligned(16))) E Pl[SPLIT ? 64 * LD : 1];
    E* Vt = reinterpret_cast<E*>(lds_raw);           // [D16][LD]: Vt[d][key]
    const int H = a.H, D = a.head_dim, rep = H / a.Hkv;
    const int D16 = (D + 15) / 16 * 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, group = lane >> 4, l15 = lane & 15;
    const TileRec t = reinterpret_cast<const TileRec*>(tiles)[blockIdx.x];
    const int h = blockIdx.y;
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_last = t.q0 + t.nq - 1;
    const int j_min = t.q0 - window + 1 > 0 ? t.q0 - window + 1 : 0;
    const float* S = a.scratch + ((int64_t)t.row0 * H + h) * band;         // row r of the tile: + r * H * band
    const int64_t s_row = (int64_t)H * band;
    const int n_sub = (t.nq + 15) / 16, n_dt = D16 / 16, n_pairs = n_sub * n_dt;

    const E* V = (const E*)a.cache + (int64_t)t.slot * a.slot_stride + (int64_t)(h / rep) * a.head_stride;
    const bool vec = D % CE == 0 && a.head_stride % CE == 0 && a.slot_stride % CE == 0 && ((uintptr_t)a.cache % 16 == 0);
    f4 acc[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};

    // Software pipeline over 32-key steps: the band values and key chunks of step n + 1 are requested before the MFMAs of step n
    // and turned into LDS operands after them, so a step costs its arithmetic and two barriers, not a memory round trip.
    // A thread owns 4 consecutive keys of a row (twice: rows r and r + 32) and the same 16-byte column chunk of 2 consecutive
    // keys, so its LDS operands go out as 8- and 4-byte stores (4 + 8 per step and thread) instead of one per element.
    constexpr int SP = 8;                             // band values per thread and step: 64 rows x 32 keys / 256 threads
    constexpr int VC = NP * (int)sizeof(E) / 8 < 2 ? 2 : NP * (int)sizeof(E) / 8;     // 16-byte key chunks per thread and step (in pairs)
    const int cpk = D / CE;
    float sv[SP];
    u32x4 vv[VC];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int u = 0; u < SP / 4; ++u) {
            const int e = tid + 256 * u, r = e >> 3, kq = (e & 7) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dist = t.q0 + r - (j0 + kq + i);
                sv[4 * u + i] = -INFINITY;
                if (r < n_sub * 16 && r < t.nq && dist >= 0 && dist < window) sv[4 * u + i] = S[r * s_row + dist];
            }
        }
        if (vec) {
#pragma unroll
            for (int u = 0; u < VC; ++u) {
                // chunk index within the step: pair p of keys (2p, 2p + 1), column chunk c; u even: key 2p, u odd: key 2p + 1
                const int pe = tid + 256 * (u >> 1), kk = (pe & 15) * 2 + (u & 1), c = (pe >> 4) * CE;
                vv[u] = u32x4{0u, 0u, 0u, 0u};
                if (pe < 16 * cpk && j0 + kk <= i_last) vv[u] = *reinterpret_cast<const u32x4*>(V + (int64_t)(j0 + kk) * D + c);
            }
        }
    };
    // Online softmax: the 8 lanes that own a row's 32 keys of a step keep its running maximum and denominator (the sink enters
    // as maximum 0, denominator 1), publish the factor that rescales what the row has accumulated so far, and write unnormalised
    // weights; the division by the denominator happens once, at the end.  The band is read exactly once.
    float rm[SP / 4], rl[SP / 4];
#pragma unroll
    for (int u = 0; u < SP / 4; ++u) rm[u] = a.sink ? 0.0f : -INFINITY, rl[u] = a.sink ? 1.0f : 0.0f;
    fetch(j_min);
    for (int j0 = j_min; j0 <= i_last; j0 += 32) {
#pragma unroll
        for (int u = 0; u < SP / 4; ++u) {
            const int e = tid + 256 * u, r = e >> 3, kq = (e & 7) * 4;
            float tmax = fmaxf(fmaxf(sv[4 * u], sv[4 * u + 1]), fmaxf(sv[4 * u + 2], sv[4 * u + 3]));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 1, 64));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 2, 64));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 4, 64));
            const float m_new = fmaxf(rm[u], tmax);
            const float alpha = m_new == -INFINITY ? 1.0f : expf(rm[u] - m_new);
            float pv[4], psum = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pv[i] = sv[4 * u + i] == -INFINITY ? 0.0f : expf(sv[4 * u + i] - m_new);
                psum += pv[i];
            }
            psum += __shfl_xor(psum, 1, 64);
            psum += __shfl_xor(psum, 2, 64);
            psum += __shfl_xor(psum, 4, 64);
            rl[u] = rl[u] * alpha + psum;
            rm[u] = m_new;
            if (r < n_sub * 16) {
                if ((lane & 7) == 0) row_alpha[r] = alpha;
                __attribute__((aligned(16))) E hi[4];
                __attribute__((aligned(16))) E lo[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    hi[i] = from_f32<E>(pv[i]);
                    if (SPLIT) lo[i] = from_f32<E>(pv[i] - to_f32(hi[i]));
                }
                if (SPLIT) {
                    *reinterpret_cast<uint64_t*>(&Ph[r * LD + kq]) = *reinterpret_cast<const uint64_t*>(hi);
                    *reinterpret_cast<uint64_t*>(&Pl[r * LD + kq]) = *reinterpret_cast<const uint64_t*>(lo);
                } else {
                    *reinterpret_cast<u32x4*>(&Ph[r * LD + kq]) = *reinterpret_cast<const u32x4*>(hi);
                }
            }
        }
        if (vec) {
#pragma unroll
            for (int u = 0; u < VC; u += 2) {
                const int pe = tid + 256 * (u >> 1), kk = (pe & 15) * 2, c = (pe >> 4) * CE;
                if (pe < 16 * cpk) {
                    __attribute__((aligned(16))) E t0[CE];
                    __attribute__((aligned(16))) E t1[CE];
                    *reinterpret_cast<u32x4*>(t0) = vv[u];
                    *reinterpret_cast<u32x4*>(t1) = vv[u + 1];
#pragma unroll
                    for (int i = 0; i < CE; ++i) {
                        __attribute__((aligned(8))) E pr[2] = {t0[i], t1[i]};
                        if (sizeof(E) == 2)
                            *reinterpret_cast<uint32_t*>(&Vt[(c + i) * LD + kk]) = *reinterpret_cast<const uint32_t*>(pr);
                        else
                            *reinterpret_cast<uint64_t*>(&Vt[(c + i) * LD + kk]) = *reinterpret_cast<const uint64_t*>(pr);
                    }
                }
            }
            for (int e = tid; e < 32 * (D16 - D); e += 256) Vt[(D + e / 32) * LD + (e & 31)] = from_f32<E>(0.0f);
        } else {
            for (int e = tid; e < 32 * D16; e += 256) {
                const int kk = e / D16, d = e % D16;
                const int j = j0 + kk;
                Vt[d * LD + kk] = (j <= i_last && d < D) ? V[(int64_t)j * D + d] : from_f32<E>(0.0f);
            }
        }
        __syncthreads();
        if (j0 + 32 <= i_last) fetch(j0 + 32);
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int p = wave + 4 * i;
            if (p < n_pairs) {
                const int sub = p % n_sub, dt = p / n_sub;
                const Frag<E> ph = load_frag(&Ph[(sub * 16 + l15) * LD], group, 32, true);
                const Frag<E> fv = load_frag(&Vt[(dt * 16 + l15) * LD], group, 32, true);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][r] *= row_alpha[sub * 16 + 4 * group + r];
                acc[i] = mma(ph, fv, acc[i]);
                if (SPLIT) {
                    const Frag<E> pl = load_frag(&Pl[(sub * 16 + l15) * LD], group, 32, true);
                    acc[i] = mma(pl, fv, acc[i]);
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int u = 0; u < SP / 4; ++u) {
        const int r = (tid + 256 * u) >> 3;
        if ((lane & 7) == 0) row_inv[r] = 1.0f / rl[u];
    }
    __syncthreads();
    E* O = (E*)a.out;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int p = wave + 4 * i;
        if (p < n_pairs) {
            const int sub = p % n_sub, d = (p / n_sub) * 16 + l15;
            if (d < D) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int qr = sub * 16 + 4 * group + r;
                    if (qr < t.nq) O[(int64_t)(t.row0 + qr) * a.ldo + h * D + d] = from_f32<E>(acc[i][r] * row_inv[qr]);
                }
            }
        }
    }
}

// ---- 2b. values for tiles of at most 4 rows (decoding) -------------------------------------------------------------------------
// A row's output is a weighted sum of key rows: no matrix core needed, and nothing to transpose.  Thread = (column d, key slice);
// it walks its slice's keys with coalesced loads (a key row is contiguous over d), multiplies by the rows' weights from LDS
// (fp32, not rounded) and the slices meet in LDS at the end.
constexpr int FEW_ROWS = 4, FEW_KEYS = 1024;

template <typename E>
__global__ __launch_bounds__(256) void talk_values_few_kernel(pcb_attn_talk_args a, int band, const int32_t* tiles) {
    __shared__ float row_m[FEW_ROWS], row_inv[FEW_ROWS];
    __shared__ float P[FEW_ROWS][FEW_KEYS];
    __shared__ float red[FEW_ROWS][256];
    const int H = a.H, D = a.head_dim, rep = H / a.Hkv;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const TileRec t = reinterpret_cast<const TileRec*>(tiles)[blockIdx.x];
    const int h = blockIdx.y;
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_last = t.q0 + t.nq - 1;
    const int j_min = t.q0 - window + 1 > 0 ? t.q0 - window + 1 : 0;
    const float* __restrict__ S = a.scratch + ((int64_t)t.row0 * H + h) * band;
    const int64_t s_row = (int64_t)H * band;
    // row statistics in one pass, all threads on one row at a time: a thread folds its share of the row into a (max, sum) pair
    // -- every load of the row is in flight at once -- and the pairs meet in LDS
    for (int r = 0; r < t.nq; ++r) {
        const int i = t.q0 + r;
        const int n = i + 1 < window ? i + 1 : window;
        const float* sr = S + r * s_row;
        float m = -INFINITY, l = 0.0f;
        for (int d = tid; d < n; d += 256) {
            const float v = sr[d];
            const float m2 = fmaxf(m, v);
            l = l * expf(m - m2) + expf(v - m2);
            m = m2;
        }
        const float wm = wave_max(m);
        l = wave_sum(m == -INFINITY ? 0.0f : l * expf(m - wm));
        if (lane == 0) red[0][wave] = wm, red[1][wave] = l;
        __syncthreads();
        if (tid == 0) {
            float bm = a.sink ? 0.0f : -INFINITY;
            for (int w = 0; w < 4; ++w) bm = fmaxf(bm, red[0][w]);
            float bl = a.sink ? expf(-bm) : 0.0f;
            for (int w = 0; w < 4; ++w)
                if (red[0][w] != -INFINITY) bl += red[1][w] * expf(red[0][w] - bm);
            row_m[r] = bm;
            row_inv[r] = 1.0f / bl;
        }
        __syncthreads();
    }
    for (int e = tid; e < FEW_ROWS * FEW_KEYS; e += 256) (&P[0][0])[e] = 0.0f;      // rows the tile does not have stay zero
    __syncthreads();
    const E* __restrict__ V = (const E*)a.cache + (int64_t)t.slot * a.slot_stride + (int64_t)(h / rep) * a.head_stride;
    // wide form: a thread owns one 16-byte chunk of the key rows (CE columns) and every (256 / chunks)-th key
    constexpr int CE = 16 / sizeof(E);
    const bool wide = D % CE == 0 && D / CE <= 256 && a.head_stride % CE == 0 && a.slot_stride % CE == 0 && ((uintptr_t)a.cache % 16 == 0);
    const int cols = wide ? D / CE : D;               // thread columns; D <= 256
    const int n_slices = 256 / cols;
    const int dcol = tid % cols, slice = tid / cols;
    const bool active = slice < n_slices;
    float acc[FEW_ROWS][CE];
#pragma unroll
    for (int r = 0; r < FEW_ROWS; ++r)
#pragma unroll
        for (int i = 0; i < CE; ++i) acc[r][i] = 0.0f;
    for (int j0 = j_min; j0 <= i_last; j0 += FEW_KEYS) {
        const int n = i_last - j0 + 1 < FEW_KEYS ? i_last - j0 + 1 : FEW_KEYS;
        for (int e = tid; e < t.nq * FEW_KEYS; e += 256) {
            const int r = e / FEW_KEYS, kk = e % FEW_KEYS;
            const int dist = t.q0 + r - (j0 + kk);
            float p = 0.0f;
            if (kk < n && dist >= 0 && dist < window) p = expf(S[r * s_row + dist] - row_m[r]) * row_inv[r];
            P[r][kk] = p;
        }
        __syncthreads();
        if (active && wide) {
#pragma unroll 16
            for (int kk = slice; kk < n; kk += n_slices) {
                __attribute__((aligned(16))) E tmp[CE];
                *reinterpret_cast<u32x4*>(tmp) = *reinterpret_cast<const u32x4*>(V + (int64_t)(j0 + kk) * D + dcol * CE);
#pragma unroll
                for (int r = 0; r < FEW_ROWS; ++r) {
                    const float p = P[r][kk];
#pragma unroll
                    for (int i = 0; i < CE; ++i) acc[r][i] += p * to_f32(tmp[i]);
                }
            }
        } else if (active) {
#pragma unroll 4
            for (int kk = slice; kk < n; kk += n_slices) {
                const float v = to_f32(V[(int64_t)(j0 + kk) * D + dcol]);
#pragma unroll
                for (int r = 0; r < FEW_ROWS; ++r) acc[r][0] += P[r][kk] * v;
            }
        }
        __syncthreads();
    }
    // the slices meet in LDS, one column chunk element at a time (red is [rows][256])
    E* O = (E*)a.out;
    const int per = wide ? CE : 1;
    for (int i = 0; i < per; ++i) {
#pragma unroll
        for (int r = 0; r < FEW_ROWS; ++r) {
            float v = 0.0f;
#pragma unroll
            for (int i2 = 0; i2 < CE; ++i2)
                if (i2 == i) v = acc[r][i2];
            red[r][tid] = active ? v : 0.0f;
        }
        __syncthreads();
        if (tid < cols) {
            for (int r = 0; r < t.nq; ++r) {
                float v = 0.0f;
                for (int sl = 0; sl < n_slices; ++sl) v += red[r][sl * cols + tid];
                O[(int64_t)(t.row0 + r) * a.ldo + h * D + tid * per + i] = from_f32<E>(v);
            }
        }
        __syncthreads();
    }
}

template <typename E, int HMAX>
void launch_scores(const pcb_attn_talk_args& a, int band, hipStream_t stream) {
    // the tile's queries wait in LDS when 16 rows of all heads fit beside the kernel's own tables (160 KiB per workgroup)
    const int ce = 16 / (int)sizeof(E);
    const int qld = a.H * a.head_dim + ce;
    const size_t q_bytes = (size_t)16 * qld * sizeof(E);
    const bool aligned = (a.H * a.head_dim) % ce == 0;
    const int q_lds = aligned && q_bytes + sizeof(float) * (HMAX * HMAX + HMAX) <= 150 * 1024;
    // NST = k-steps of a head (head_dim / 32, rounded up) the kernel is built for, PG = key heads fetched together
    constexpr int PG = (HMAX <= 16 && sizeof(E) == 2) ? 4 : 2;
    auto kern = a.head_dim <= 128 ? talk_scores_kernel<E, HMAX, 4, PG> : talk_scores_kernel<E, HMAX, 8, (PG > 2 ? 2 : PG)>;
    static bool raised[2] = {false, false};
    bool& up = raised[a.head_dim <= 128 ? 0 : 1];
    if (q_lds && q_bytes > 48 * 1024 && !up) {
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
        up = true;
    }
    const int KC = a.n_tiles >= 64 ? 128 : 64;
    const dim3 grid(a.n_tiles, pcb_ceil_div(band, KC));
    hipLaunchKernelGGL(kern, grid, dim3(256), q_lds ? q_bytes : 0, stream, a, band, q_lds, qld, KC);
}

template <typename E>
int run(const pcb_attn_talk_args& a, int band, hipStream_t stream) {
    const int H = a.H;
    if (H <= 4)
        launch_scores<E, 4>(a, band, stream);
    else if (H <= 8)
        launch_scores<E, 8>(a, band, stream);
    else if (H <= 16)
        launch_scores<E, 16>(a, band, stream);
    else
        launch_scores<E, 32>(a, band, stream);
    int rc = pcb_check_launch("talk_scores_kernel");
    if (rc != PCB_OK) return rc;
    const int D16 = (a.head_dim + 15) / 16 * 16;
    const size_t lds = (size_t)D16 * (32 + 16 / sizeof(E)) * sizeof(E);
    const int32_t* tiles = a.tiles64 ? a.tiles64 : a.tiles;
    const dim3 grid(a.tiles64 ? a.n_tiles64 : a.n_tiles, H);
    if (a.max_tile_rows > 0 && a.max_tile_rows <= FEW_ROWS) {
        hipLaunchKernelGGL((talk_values_few_kernel<E>), grid, dim3(256), 0, stream, a, band, tiles);
        return pcb_check_launch("talk_values_few_kernel");
    }
    if (D16 <= 64)
        hipLaunchKernelGGL((talk_values_kernel<E, 4>), grid, dim3(256), lds, stream, a, band, tiles);
    else if (D16 <= 128)
        hipLaunchKernelGGL((talk_values_kernel<E, 8>), grid, dim3(256), lds, stream, a, band, tiles);
    else
        hipLaunchKernelGGL((talk_values_kernel<E, 16>), grid, dim3(256), lds, stream, a, band, tiles);
    return pcb_check_launch("talk_values_kernel");
}

}  // namespace

PCB_EXPORT int32_t pcb_attn_talk_band(int32_t window, int32_t max_kv_len) {
    // rounded up to 16 floats plus 16 more: consecutive heads and rows of the band must not sit a power of two apart (their
    // stores would crowd into a few memory channels)
    const int b = (window > 0 && window < max_kv_len) ? window : max_kv_len;
    return ((b < 1 ? 1 : b) + 15) / 16 * 16 + 16;
}

PCB_EXPORT int pcb_attn_talk(const pcb_attn_talk_args* a, void* stream) {
    PCB_REQUIRE(a && a->struct_bytes == sizeof(pcb_attn_talk_args), PCB_ERR_ARG, "pcb_attn_talk: struct size mismatch");
    PCB_REQUIRE(a->dtype == PCB_BF16 || a->dtype == PCB_F32, PCB_ERR_ARG, "pcb_attn_talk: unknown dtype");
    PCB_REQUIRE(a->H > 0 && a->H <= 32 && a->Hkv > 0 && a->H % a->Hkv == 0 && a->head_dim > 0 && a->head_dim <= 256, PCB_ERR_ARG,
                "pcb_attn_talk: heads <= 32, kv heads | heads, head_dim <= 256");
    PCB_REQUIRE(a->n_tiles >= 0 && a->max_kv_len > 0, PCB_ERR_ARG, "pcb_attn_talk: bad sizes");
    if (a->n_tiles == 0) return PCB_OK;
    PCB_REQUIRE(a->q && a->tiles && a->cache && a->scratch && a->out, PCB_ERR_ARG, "pcb_attn_talk: null pointer");
    PCB_REQUIRE(!a->tiles64 || a->n_tiles64 > 0, PCB_ERR_ARG, "pcb_attn_talk: the second tile table is empty");
    PCB_REQUIRE(a->ldq >= (int64_t)a->H * a->head_dim && a->ldo >= (int64_t)a->H * a->head_dim, PCB_ERR_ARG,
                "pcb_attn_talk: row strides shorter than heads * head_dim");
    const int band = pcb_attn_talk_band(a->window, a->max_kv_len);
    PCB_REQUIRE(a->scratch_floats >= (int64_t)a->n_tiles * 16 * a->H * band, PCB_ERR_ARG,
                "pcb_attn_talk: scratch holds %lld floats, %lld needed", (long long)a->scratch_floats,
                (long long)a->n_tiles * 16 * a->H * band);
    return a->dtype == PCB_BF16 ? run<pcb::bf16_t>(*a, band, (hipStream_t)stream) : run<float>(*a, band, (hipStream_t)stream);
}
