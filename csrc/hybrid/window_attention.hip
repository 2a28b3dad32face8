// window_attention.hip — grouped-query softmax attention over paged keys and values through a sliding window that
// also keeps each sequence's first tokens, with a learned sink per head in the softmax denominator.
//
//   window_prep       per token: per-head RMS norm (float; skipped when no norm weights are given) and rotation
//                     (cos / sin from a float table made in double precision) of the query heads (in place) and key
//                     heads; the values optionally mixed with the same token's values of an earlier layer,
//                     (1 - lam) v + lam v_first, optionally rotated by the token's position over all Dv columns;
//                     keys and values written to the token's page and slot of kc [NB, BS, G, D] / vc [NB, BS, G, Dv].
//                     The values are read from column v_off of the projection's row (the column after the keys, or
//                     for instance the keys' own columns: values = keys as projected).
//   pool_blocks       per sequence and block of `pool` positions whose last position is among the step's tokens: the
//                     float means of the block's cached keys and values, written to kp / vp [NB, EP, G, .] (block e
//                     in row e % EP of the sequence's page e / EP, EP = ceil(BS / pool)).
//   window_attention  the general kernel (vector ALUs, float or bfloat16, any sizes): a workgroup takes one sequence,
//                     one key/value head and up to 16 consecutive query tokens with all the query heads of that
//                     group (at most 64 (token, head) rows, fewer when the LDS asks for it); 64-key tiles of the
//                     cache are staged in LDS; lanes are keys for the scores (float
//                     accumulation, online softmax in float) and value columns for the output.  The key range of a
//                     tile of queries is [0, keep_first) and [first query - window + 1, last query]; tiles of keys
//                     between the two are never touched, and each row masks by its own position:
//                         visible(i, j) = j <= i and (window == 0 or i - j < window or j < keep_first)
//                                         and (chunk == 0 or j >= floor(i / chunk) * chunk).
//                     With chunk > 0 a query sees only the keys of its own chunk of positions (counted from the
//                     sequence's position 0, wherever a prompt was cut); the tile walk starts at the first query's
//                     chunk start.
//                     With pool > 0 (and a window) the walk begins with tiles of POOLED pairs: the row at position i
//                     sees block e when e pool + pool - 1 <= i - window, so a token that has left the window is seen
//                     again only once its whole block has; tokens and blocks share the one softmax.
//                     After the last key the sink joins the denominator: l += exp(sink_h - m) (no value), and the
//                     row is multiplied by sigmoid(gate) when a gate is given.
// Prompt portions, decode rows and mixed steps are one code path (a decode row is a tile of one token).
#include <algorithm>

#include "hybrid_common.h"

namespace chronos {
namespace hy {

// LDS: one float row of D per wave.
template <typename T>
__global__ void __launch_bounds__(256) window_prep_kernel(
        T* __restrict__ qkv, int ldq, int H, int G, int D, int Dv, const T* __restrict__ v_first,
        const float* __restrict__ lam, const int32_t* __restrict__ pos, const int32_t* __restrict__ tok_seq,
        const int32_t* __restrict__ block_table, int max_blocks, const float* __restrict__ q_norm,
        const float* __restrict__ k_norm, float eps, const float* __restrict__ cos_sin, int dims, T* __restrict__ kc,
        T* __restrict__ vc, int BS, T* __restrict__ v_out, int v_off, const float* __restrict__ v_cos_sin) {
    extern __shared__ float wp_smem[];
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    float* row = wp_smem + wv * D;
    const int p = pos[t];
    const int64_t slot = (int64_t)block_table[(int64_t)tok_seq[t] * max_blocks + p / BS] * BS + p % BS;
    const int half = dims / 2;
    const float* cs = cos_sin != nullptr ? cos_sin + (int64_t)p * dims : nullptr;
    T* base = qkv + t * ldq;
    for (int j = wv; j < H + G; j += 4) {  // heads 0..H-1: queries (in place); H..H+G-1: keys (to the cache)
        const T* src = base + (int64_t)j * D;
        const float* nw = j < H ? q_norm : k_norm;
        if (nw == nullptr && dims == 0 && j < H) continue;  // plain queries stay as the projection wrote them
        float ss = 0.f;
        for (int i = lane; i < D; i += 64) {
            const float v = ld<T>(src + i);
            row[i] = v;
            ss += v * v;
        }
        const float inv = nw != nullptr ? 1.f / sqrtf(wave_sum(ss) / (float)D + eps) : 1.f;
        T* dst = j < H ? base + (int64_t)j * D : kc + (slot * G + (j - H)) * D;
        // (wave-private LDS row: the wave's own writes above are visible to its reads below without a barrier,
        // the compiler orders LDS accesses of one wave)
        for (int i = lane; i < D; i += 64) {
            auto nrm = [&](int c) { return nw != nullptr ? row[c] * inv * nw[c] : row[c]; };
            float v = nrm(i);
            if (i < half) v = v * cs[i] - nrm(i + half) * cs[half + i];
            else if (i < dims) v = v * cs[i - half] + nrm(i - half) * cs[i];
            st<T>(dst + i, v);
        }
    }
    const float l = v_first != nullptr ? lam[0] : 0.f;
    const T* vsrc = base + v_off;
    auto value = [&](int i) {
        float v = ld<T>(vsrc + i);
        if (v_first != nullptr) v = (1.f - l) * v + l * ld<T>(v_first + t * G * Dv + i);
        return v;
    };
    if (v_cos_sin != nullptr) {   // thread = (head, pair m): columns m and m + Dv / 2 turn by p * f_m
        const int vh = Dv / 2;
        const float* vcs = v_cos_sin + (int64_t)p * Dv;
        for (int it = threadIdx.x; it < G * vh; it += 256) {
            const int a = it / vh * Dv + it % vh, b = a + vh;
            const float u = value(a), v = value(b), c = vcs[it % vh], sn = vcs[vh + it % vh];
            if (v_out != nullptr) {
                st<T>(v_out + t * G * Dv + a, ld<T>(vsrc + a));
                st<T>(v_out + t * G * Dv + b, ld<T>(vsrc + b));
            }
            st<T>(vc + slot * G * Dv + a, u * c - v * sn);
            st<T>(vc + slot * G * Dv + b, v * c + u * sn);
        }
        return;
    }
    for (int i = threadIdx.x; i < G * Dv; i += 256) {
        if (v_out != nullptr) st<T>(v_out + t * G * Dv + i, ld<T>(vsrc + i));
        st<T>(vc + slot * G * Dv + i, value(i));
    }
}

// grid (blocks per sequence at most, B): workgroup = one block of `pool` positions that the step completes.
template <typename T>
__global__ void __launch_bounds__(256) pool_blocks_kernel(const T* __restrict__ kc, const T* __restrict__ vc,
                                                          T* __restrict__ kp, T* __restrict__ vp,
                                                          const int32_t* __restrict__ block_table, int max_blocks,
                                                          const int32_t* __restrict__ q_start,
                                                          const int32_t* __restrict__ pos0, int pool, int BS, int EP,
                                                          int GD, int GDv) {
    const int b = blockIdx.y;
    const int n = q_start[b + 1] - q_start[b];
    if (n <= 0) return;
    const int p0 = pos0[b];
    const int e = p0 / pool + blockIdx.x;          // blocks [p0 / pool, (p0 + n) / pool) end inside this step
    if (e >= (p0 + n) / pool) return;
    const int32_t* bt = block_table + (int64_t)b * max_blocks;
    const int64_t dst = (int64_t)bt[e / EP] * EP + e % EP;
    const float inv = 1.f / (float)pool;
    for (int c = threadIdx.x; c < GD + GDv; c += 256) {
        const bool isk = c < GD;
        const T* src = isk ? kc : vc;
        const int w = isk ? GD : GDv, cc = isk ? c : c - GD;
        float acc = 0.f;
        for (int r = 0; r < pool; ++r) {
            const int j = e * pool + r;
            acc += ld<T>(src + ((int64_t)bt[j / BS] * BS + j % BS) * w + cc);
        }
        st<T>((isk ? kp : vp) + dst * w + cc, acc * inv);
    }
}

// The same for widths that are multiples of 8 columns: grid (blocks per sequence at most, B, 512-column slabs of the
// keys then of the values).  A wave sums every fourth position of the block, a lane 8 neighbouring columns (16- or
// 32-byte loads); the four waves' partial sums meet in LDS and are added in a fixed order.
template <typename T>
__global__ void __launch_bounds__(256) pool_blocks_vec_kernel(const T* __restrict__ kc, const T* __restrict__ vc,
                                                              T* __restrict__ kp, T* __restrict__ vp,
                                                              const int32_t* __restrict__ block_table, int max_blocks,
                                                              const int32_t* __restrict__ q_start,
                                                              const int32_t* __restrict__ pos0, int pool, int BS, int EP,
                                                              int GD, int GDv, int nzk) {
    __shared__ float part[4][512];
    const int b = blockIdx.y;
    const int n = q_start[b + 1] - q_start[b];
    if (n <= 0) return;
    const int p0 = pos0[b];
    const int e = p0 / pool + blockIdx.x;
    if (e >= (p0 + n) / pool) return;
    const bool isk = (int)blockIdx.z < nzk;
    const T* src = isk ? kc : vc;
    const int w = isk ? GD : GDv;
    const int c0 = (isk ? blockIdx.z : blockIdx.z - nzk) * 512;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int32_t* bt = block_table + (int64_t)b * max_blocks;
    const int col = c0 + lane * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (col < w) {
        for (int r = wv; r < pool; r += 4) {
            const int j = e * pool + r;
            const T* p = src + ((int64_t)bt[j / BS] * BS + j % BS) * w + col;
            if constexpr (sizeof(T) == 2) {
                const u16x8 v = *reinterpret_cast<const u16x8*>(p);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] += bf2f(v[i]);
            } else {
                const f32x4 a = *reinterpret_cast<const f32x4*>(p), c = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[i] += a[i];
                    acc[4 + i] += c[i];
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[wv][lane * 8 + i] = acc[i];
    __syncthreads();
    const int64_t dst = (int64_t)bt[e / EP] * EP + e % EP;
    const float inv = 1.f / (float)pool;
    for (int c = threadIdx.x; c < 512 && c0 + c < w; c += 256)
        st<T>((isk ? kp : vp) + dst * w + c0 + c, ((part[0][c] + part[1][c]) + (part[2][c] + part[3][c])) * inv);
}

constexpr int kWaQT = 16;   // query tokens per workgroup at most (fewer when the group has more than 4 heads)
constexpr int kWaRows = 64; // (token, head) rows per workgroup at most
constexpr int kWaKT = 64;   // keys per tile
constexpr int kWaRB = 4;    // rows a wave carries through a tile together

template <typename T> struct WaPad { static constexpr int V = 2; };
template <> struct WaPad<float> { static constexpr int V = 1; };

// rows = query tokens x R heads of the group.  LDS: K tile [64][D + pad] T | V tile [64][Dv + pad] T |
// q rows [QT R][D] float | per wave: weights [RB][64] float.
template <typename T>
__global__ void __launch_bounds__(256) window_attention_kernel(
        const T* __restrict__ qkv, int ldq, const T* __restrict__ kc, const T* __restrict__ vc,
        const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ q_start,
        const int32_t* __restrict__ pos, const float* __restrict__ sink, const float* __restrict__ gate,
        T* __restrict__ out, int H, int G, int D, int Dv, int BS, float scale, int window, int keep, int chunk, int QT,
        int rows_cap, int pool, int EP, const T* __restrict__ kp, const T* __restrict__ vp) {
    extern __shared__ __attribute__((aligned(16))) unsigned char wa_smem[];
    constexpr int PAD = WaPad<T>::V;
    const int R = H / G;
    const int b = blockIdx.x, g = blockIdx.z;
    const int t0 = q_start[b] + blockIdx.y * QT;
    const int t1 = min(q_start[b + 1], t0 + QT);
    if (t1 <= t0) return;
    const int nq = t1 - t0, rows = nq * R;
    const int ldk = D + PAD, ldv = Dv + PAD;
    T* Ks = reinterpret_cast<T*>(wa_smem);
    T* Vs = Ks + kWaKT * ldk;
    float* Qs = reinterpret_cast<float*>(wa_smem + (((size_t)kWaKT * (ldk + ldv) * sizeof(T) + 15) & ~(size_t)15));
    float* Ps = Qs + (size_t)rows_cap * D;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    float* Pw = Ps + wv * kWaRB * kWaKT;
    for (int i = threadIdx.x; i < rows * D; i += 256) {
        const int r = i / D, d = i % D;
        Qs[i] = ld<T>(qkv + (int64_t)(t0 + r / R) * ldq + (g * R + r % R) * D + d);
    }
    const int p_lo = pos[t0], p_hi = pos[t1 - 1];
    // tokens of a range sit at consecutive positions, so the tile's queries are p_lo .. p_hi
    // the first key any row of the tile may see (the bounds of both masks grow with the position)
    const int w_lo = max(window > 0 ? max(0, p_lo - window + 1) : 0, chunk > 0 ? p_lo / chunk * chunk : 0);
    const int w_start = w_lo / kWaKT * kWaKT;
    // kept first tokens below the window's first tile: keys [0, k_end) (those from w_start on pass the window tiles'
    // own test), so no key is ever counted twice
    const int k_end = window > 0 ? min(keep, w_start) : 0;
    const int n_keep_tiles = (k_end + kWaKT - 1) / kWaKT;
    const int n_win_tiles = (p_hi - w_start) / kWaKT + 1;
    // pooled blocks any row of the tile may see: block e with (e + 1) pool - 1 + window <= p_hi
    const int n_pool = (pool > 0 && window > 0) ? max(0, p_hi - window + 1) / pool : 0;
    const int n_pool_tiles = (n_pool + kWaKT - 1) / kWaKT;
    const int NC = (Dv + 63) / 64;
    // every wave carries its row groups through all tiles: group q of wave wv = rows (q * 4 + wv) * RB ..
    const int ngroups = (rows + kWaRB - 1) / kWaRB;
    const int my_groups = (ngroups - wv + 3) / 4;
    constexpr int MAXG = kWaRows / kWaRB / 4;
    float m_[MAXG][kWaRB], l_[MAXG][kWaRB], o_[MAXG][kWaRB][4];
#pragma unroll
    for (int q = 0; q < MAXG; ++q)
#pragma unroll
        for (int r = 0; r < kWaRB; ++r) {
            m_[q][r] = -INFINITY;
            l_[q][r] = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) o_[q][r][c] = 0.f;
        }
    for (int tz = 0; tz < n_pool_tiles + n_keep_tiles + n_win_tiles; ++tz) {
        const bool pooled = tz < n_pool_tiles;   // a tile of pooled pairs: "key" j is block j
        const int ti = tz - n_pool_tiles;
        const int j0 = pooled ? tz * kWaKT : ti < n_keep_tiles ? ti * kWaKT : w_start + (ti - n_keep_tiles) * kWaKT;
        const int j_end = pooled ? min(n_pool, j0 + kWaKT)
                                 : ti < n_keep_tiles ? min(k_end, j0 + kWaKT) : min(p_hi + 1, j0 + kWaKT);  // keys [j0, j_end)
        const T* ksrc = pooled ? kp : kc;
        const T* vsrc = pooled ? vp : vc;
        const int per = pooled ? EP : BS;        // rows of a page in the source
        __syncthreads();
        for (int i = threadIdx.x; i < kWaKT * D; i += 256) {
            const int kk = i / D, d = i % D, j = j0 + kk;
            T v;
            st<T>(&v, 0.f);
            if (j < j_end) v = ksrc[(((int64_t)block_table[(int64_t)b * max_blocks + j / per] * per + j % per) * G + g) * D + d];
            Ks[kk * ldk + d] = v;
        }
        for (int i = threadIdx.x; i < kWaKT * Dv; i += 256) {
            const int kk = i / Dv, d = i % Dv, j = j0 + kk;
            T v;
            st<T>(&v, 0.f);
            if (j < j_end) v = vsrc[(((int64_t)block_table[(int64_t)b * max_blocks + j / per] * per + j % per) * G + g) * Dv + d];
            Vs[kk * ldv + d] = v;
        }
        __syncthreads();
        const int j = j0 + lane;
#pragma unroll
        for (int q = 0; q < MAXG; ++q) {
            if (q >= my_groups) break;
            const int r0 = (q * 4 + wv) * kWaRB;
            float s[kWaRB] = {0.f, 0.f, 0.f, 0.f};
            const T* krow = Ks + lane * ldk;
            for (int d = 0; d < D; ++d) {
                const float kv = ld<T>(krow + d);
#pragma unroll
                for (int r = 0; r < kWaRB; ++r) s[r] += Qs[min(r0 + r, rows - 1) * D + d] * kv;
            }
#pragma unroll
            for (int r = 0; r < kWaRB; ++r) {
                const int rr = min(r0 + r, rows - 1);
                const int pi = p_lo + rr / R;
                const bool vis = pooled ? (j < j_end && (j + 1) * pool - 1 + window <= pi)
                                        : (j < j_end && j <= pi && (window <= 0 || pi - j < window || j < keep) &&
                                           (chunk <= 0 || j >= pi / chunk * chunk));
                const float sv = vis ? s[r] * scale : -INFINITY;
                const float mn = fmaxf(m_[q][r], wave_max(sv));
                const float pw = mn == -INFINITY ? 0.f : expf(sv - mn);
                const float corr = m_[q][r] == -INFINITY ? 0.f : expf(m_[q][r] - mn);
                l_[q][r] = l_[q][r] * corr + wave_sum(pw);
                m_[q][r] = mn;
#pragma unroll
                for (int c = 0; c < 4; ++c) o_[q][r][c] *= corr;
                Pw[r * kWaKT + lane] = pw;
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int col = c * 64 + lane;
                if (c < NC && col < Dv) {
                    float a[kWaRB] = {0.f, 0.f, 0.f, 0.f};
                    for (int kk = 0; kk < kWaKT; ++kk) {
                        const float vv = ld<T>(Vs + kk * ldv + col);
#pragma unroll
                        for (int r = 0; r < kWaRB; ++r) a[r] += Pw[r * kWaKT + kk] * vv;
                    }
#pragma unroll
                    for (int r = 0; r < kWaRB; ++r) o_[q][r][c] += a[r];
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < MAXG; ++q) {
        if (q >= my_groups) break;
        const int r0 = (q * 4 + wv) * kWaRB;
#pragma unroll
        for (int r = 0; r < kWaRB; ++r) {
            const int rr = r0 + r;
            if (rr >= rows) continue;
            const int64_t t = t0 + rr / R;
            const int hd = g * R + rr % R;
            float m = m_[q][r], l = l_[q][r];
            if (sink != nullptr) {
                const float sk = sink[hd];
                const float mn = fmaxf(m, sk);
                const float corr = m == -INFINITY ? 0.f : expf(m - mn);
                l = l * corr + expf(sk - mn);
#pragma unroll
                for (int c = 0; c < 4; ++c) o_[q][r][c] *= corr;
            }
            float f = l > 0.f ? 1.f / l : 0.f;
            if (gate != nullptr) f *= sigmoidf_(gate[t * H + hd]);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int col = c * 64 + lane;
                if (c < NC && col < Dv) st<T>(out + (t * H + hd) * Dv + col, o_[q][r][c] * f);
            }
        }
    }
}

}  // namespace hy

void launch_hy_window_prep(void* qkv, int ld, int H, int G, int D, int Dv, const void* v_first, const float* lam,
                           const int32_t* pos, const int32_t* tok_seq, const int32_t* block_table, int max_blocks,
                           const float* q_norm, const float* k_norm, float eps, const float* cos_sin, int dims, void* kc,
                           void* vc, int BS, void* v_out, int v_off, const float* v_cos_sin, int T, bool f32,
                           hipStream_t s) {
    if (T == 0) return;
    const int bytes = 4 * D * 4;
    if (v_off < 0) v_off = (H + G) * D;
    if (f32) hy::window_prep_kernel<float><<<T, 256, bytes, s>>>((float*)qkv, ld, H, G, D, Dv, (const float*)v_first, lam, pos, tok_seq, block_table, max_blocks, q_norm, k_norm, eps, cos_sin, dims, (float*)kc, (float*)vc, BS, (float*)v_out, v_off, v_cos_sin);
    else hy::window_prep_kernel<uint16_t><<<T, 256, bytes, s>>>((uint16_t*)qkv, ld, H, G, D, Dv, (const uint16_t*)v_first, lam, pos, tok_seq, block_table, max_blocks, q_norm, k_norm, eps, cos_sin, dims, (uint16_t*)kc, (uint16_t*)vc, BS, (uint16_t*)v_out, v_off, v_cos_sin);
}

// max_q: the most tokens a sequence brings in this step; a sequence completes at most max_q / pool + 1 blocks
void launch_hy_pool_blocks(const void* kc, const void* vc, void* kp, void* vp, const int32_t* block_table, int max_blocks,
                           const int32_t* q_start, const int32_t* pos0, int pool, int BS, int EP, int GD, int GDv, int B,
                           int max_q, bool f32, hipStream_t s) {
    if (B == 0 || max_q == 0) return;
    if (GD % 8 == 0 && GDv % 8 == 0) {
        const int nzk = (GD + 511) / 512;
        const dim3 grid(max_q / pool + 1, B, nzk + (GDv + 511) / 512);
        if (f32) hy::pool_blocks_vec_kernel<float><<<grid, 256, 0, s>>>((const float*)kc, (const float*)vc, (float*)kp, (float*)vp, block_table, max_blocks, q_start, pos0, pool, BS, EP, GD, GDv, nzk);
        else hy::pool_blocks_vec_kernel<uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)kc, (const uint16_t*)vc, (uint16_t*)kp, (uint16_t*)vp, block_table, max_blocks, q_start, pos0, pool, BS, EP, GD, GDv, nzk);
        return;
    }
    const dim3 grid(max_q / pool + 1, B);
    if (f32) hy::pool_blocks_kernel<float><<<grid, 256, 0, s>>>((const float*)kc, (const float*)vc, (float*)kp, (float*)vp, block_table, max_blocks, q_start, pos0, pool, BS, EP, GD, GDv);
    else hy::pool_blocks_kernel<uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)kc, (const uint16_t*)vc, (uint16_t*)kp, (uint16_t*)vp, block_table, max_blocks, q_start, pos0, pool, BS, EP, GD, GDv);
}

// LDS bytes of the general kernel with room for `rows` (token, head) query rows.
static size_t window_attention_lds(int rows, int D, int Dv, bool f32) {
    const size_t e = f32 ? 4 : 2, pad = f32 ? 1 : 2;
    const size_t tiles = ((size_t)hy::kWaKT * (D + pad + Dv + pad) * e + 15) & ~(size_t)15;
    return tiles + ((size_t)rows * D + 4 * hy::kWaRB * hy::kWaKT) * 4;
}

// Query rows per workgroup of the general kernel: the most (64 at most, a power of two, at least the R heads of a
// group) whose float copies fit the 160 KB of a CU beside a key tile; 0: these sizes do not fit at all.
int hy_window_rows_cap(int R, int D, int Dv, bool f32) {
    for (int rows = hy::kWaRows; rows >= 1 && rows >= R; rows >>= 1)
        if (window_attention_lds(rows, D, Dv, f32) <= 160 * 1024) return rows;
    return 0;
}

bool launch_hy_window_attention_mfma(const uint16_t*, int, const uint16_t*, const uint16_t*, const int32_t*, int,
                                     const int32_t*, const int32_t*, const float*, const float*, uint16_t*, int, int, int,
                                     int, int, int, int, float, int, int, int, int, float*, float*, int64_t, int, int,
                                     const uint16_t*, const uint16_t*, const float*, int, hipStream_t);
void launch_hy_unrotate_gate(const void*, const int32_t*, const float*, const void*, int, int, void*, int, int, int, bool,
                             hipStream_t);

// bfloat16 at matrix-core sizes runs window_attention_mfma.hip; float32 and every other size the general kernel.
// vcs (may be nullptr): a rotation table [P, Dv] by which every head's output is turned back at the query's position;
// g_off >= 0: the output is multiplied by sigmoid of the columns g_off .. g_off + H Dv of the query's row of qkv.
// The matrix-core kernel does both in its epilogue (Dv % 32 == 0); otherwise a pass over the output follows.
void launch_hy_window_attention(const void* qkv, int ld, const void* kc, const void* vc, const int32_t* block_table,
                                int max_blocks, const int32_t* q_start, const int32_t* pos, const float* sink,
                                const float* gate, void* out, int B, int max_q, int H, int G, int D, int Dv, int BS,
                                float scale, int window, int keep, int chunk, bool f32, int nsplit, float* part_o,
                                float* part_ml, int64_t total_rows, int pool, int EP, const void* kp, const void* vp,
                                const float* vcs, int g_off, hipStream_t s) {
    if (B == 0 || max_q == 0) return;
    const bool post = vcs != nullptr || g_off >= 0;
    const bool fused = post && (vcs == nullptr || Dv % 32 == 0);   // the matrix-core epilogue can do it
    const int T = (int)(total_rows / H);
    if (!f32 && launch_hy_window_attention_mfma((const uint16_t*)qkv, ld, (const uint16_t*)kc, (const uint16_t*)vc,
                                                block_table, max_blocks, q_start, pos, sink, gate, (uint16_t*)out, B,
                                                max_q, H, G, D, Dv, BS, scale, window, keep, chunk, nsplit, part_o,
                                                part_ml, total_rows, pool, EP, (const uint16_t*)kp,
                                                (const uint16_t*)vp, fused ? vcs : nullptr, fused ? g_off : -1, s)) {
        if (post && !fused) launch_hy_unrotate_gate(out, pos, vcs, g_off >= 0 ? qkv : nullptr, ld, g_off, out, T, H, Dv, false, s);
        return;
    }
    const int R = H / G;   // the caller has checked R <= 64, Dv <= 256 and that hy_window_rows_cap is not 0
    const int rows_cap = hy_window_rows_cap(R, D, Dv, f32);
    const int bytes = (int)window_attention_lds(rows_cap, D, Dv, f32);
    const int QT = std::max(1, std::min(hy::kWaQT, rows_cap / R));
    const dim3 grid(B, (max_q + QT - 1) / QT, G);
    if (f32) {
        auto kern = hy::window_attention_kernel<float>;
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        kern<<<grid, 256, bytes, s>>>((const float*)qkv, ld, (const float*)kc, (const float*)vc, block_table, max_blocks, q_start, pos, sink, gate, (float*)out, H, G, D, Dv, BS, scale, window, keep, chunk, QT, rows_cap, pool, EP, (const float*)kp, (const float*)vp);
    } else {
        auto kern = hy::window_attention_kernel<uint16_t>;
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        kern<<<grid, 256, bytes, s>>>((const uint16_t*)qkv, ld, (const uint16_t*)kc, (const uint16_t*)vc, block_table, max_blocks, q_start, pos, sink, gate, (uint16_t*)out, H, G, D, Dv, BS, scale, window, keep, chunk, QT, rows_cap, pool, EP, (const uint16_t*)kp, (const uint16_t*)vp);
    }
    if (post) launch_hy_unrotate_gate(out, pos, vcs, g_off >= 0 ? qkv : nullptr, ld, g_off, out, T, H, Dv, f32, s);
}

}  // namespace chronos
