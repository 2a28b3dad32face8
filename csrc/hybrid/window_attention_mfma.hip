// window_attention_mfma.hip — the bfloat16 windowed sink attention on the matrix cores (see window_attention.hip for
// the math and the visible set).
//
// One workgroup takes one sequence, one key/value head and 16 NW (token, head-of-the-group) rows — 16 per wave; rows
// are (token * R + head within the group), so any group size tiles the same way — and walks the keys it can see 64
// at a time: first (with pooled blocks) the pooled pairs of the blocks that lie wholly before a row's window, then the
// kept first tokens that lie below the window's first tile, then the tiles from the window's first key to the last
// query.  Per tile:
//   * the keys are staged row-major [64][D] and the values transposed [Dv][64] in LDS (both MFMA operands want 8
//     consecutive k-values per lane: dims for the scores, KEYS for the sum); the transposed image is written as
//     32-bit words holding two neighbouring keys;
//   * scores  S^T = K Q^T : 16x16x32 MFMAs, key rows as A operand, the wave's 16 query rows (in registers for the
//     whole kernel) as B operand: a lane ends up with 4 keys x 1 query row per 16-key tile;
//   * softmax in float per query row (lane & 15): each row masks by its own position (causal, window, kept tokens),
//     running maximum and sum, reductions over the 4 lane groups by two shuffles;
//   * sum  O^T = V^T P^T : the lane's 8 weights of two neighbouring 16-key tiles ARE a B operand (the k index is a
//     fixed permutation of the 32 keys, the same one the transposed value image is read with); each weight enters
//     as two bfloat16 terms (rounded value + remainder), which keeps the float softmax weights nearly exact.
// After the last tile the head's sink joins the denominator and the row is scaled by sigmoid(gate).  Two more steps
// may follow in the same epilogue: with a rotation table for the values, the head's output row is turned BACK by the
// query's position (column m pairs with m + Dv / 2; a lane holds both when Dv % 32 == 0: accumulator tile c and tile
// c + Dv / 32), and with a gate per output column the row is multiplied by sigmoid of the gate columns of the
// query's own projection row.  Launches of few
// rows (decode) deal a row block's key tiles to several workgroups and merge the float partials in a second kernel.
// With chunk > 0 a row also hides the keys below its own chunk of positions (key >= floor(pos / chunk) * chunk).
// Sizes: D % 32 == 0, Dv % 16 == 0, D <= 256, Dv <= 256.  Everything else takes the general kernel.
#include <algorithm>

#include "hybrid_common.h"

namespace chronos {
namespace hy {

constexpr int WKT = 64;  // keys per tile

template <int NS, int NCT, int NW>
__global__ void __launch_bounds__(64 * NW) window_attention_mfma_kernel(
        const uint16_t* __restrict__ qkv, int ldq, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
        const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ q_start,
        const int32_t* __restrict__ pos, const float* __restrict__ sink, const float* __restrict__ gate,
        uint16_t* __restrict__ out, int H, int G, int D, int Dv, int BS, float scale, int window, int keep, int chunk,
        int nsplit, float* __restrict__ part_o, float* __restrict__ part_ml, int pool, int EP,
        const uint16_t* __restrict__ kp, const uint16_t* __restrict__ vp, const float* __restrict__ vcs, int g_off) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int KT = WKT, NT = 64 * NW, RPB = 16 * NW, PP = KT / 2;
    const int R = H / G;
    const int b = blockIdx.x, kvh = blockIdx.z;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    const int rows_total = (t1 - t0) * R;
    const int split = blockIdx.y % nsplit;   // key tiles are dealt round-robin to the nsplit workgroups of a row block
    const int rb0 = blockIdx.y / nsplit * RPB;
    if (rb0 >= rows_total) return;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, g4 = lane >> 4, qi = lane & 15;
    const int ns = D / 32, nct = Dv / 16;
    const int krs = D * 2 + 16;          // row-major key image: bytes per key row
    constexpr int vts = KT * 2 + 8;      // transposed value image: bytes per value column
    __shared__ int krow[KT];             // cache row (page * page size + slot) of each key of the tile
    unsigned char* kimg = smem;
    unsigned char* vimg = smem + KT * krs;
    const int r = rb0 + wv * 16 + qi;
    const bool rok = r < rows_total;
    const int rc = rok ? r : rows_total - 1;
    const int64_t tok = t0 + rc / R;
    const int head = kvh * R + rc % R;
    const int prow = rok ? pos[tok] : -1;
    const int last_row = min(rows_total, rb0 + RPB) - 1;
    const int pmin = pos[t0 + rb0 / R], pmax = pos[t0 + last_row / R];  // positions grow along the sequence
    bf16x8 qf[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
        if (s < ns) qf[s] = *reinterpret_cast<const bf16x8*>(qkv + tok * ldq + head * D + 32 * s + 8 * g4);
    f32x4 O[NCT];
#pragma unroll
    for (int c = 0; c < NCT; ++c) O[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mrow = -INFINITY, lrow = 0.f;
    const float scale2 = scale * 1.4426950408889634f;
    const int32_t* bt = block_table + (int64_t)b * max_blocks;
    const int kchunks = D / 8, vchunks = Dv / 8;
    // the first key any row of the block may see: the window's or the chunk's lower bound of the first row
    const int w_lo = max(window > 0 ? max(0, pmin - window + 1) : 0, chunk > 0 ? pmin / chunk * chunk : 0);
    const int w_start = w_lo / KT * KT;
    const int c_lo = chunk > 0 ? prow / chunk * chunk : 0;        // this row's chunk starts here
    const int c_lo_max = chunk > 0 ? pmax / chunk * chunk : 0;    // the last row's
    // kept first tokens below the window's first tile are keys [0, k_end); those from w_start on pass the window
    // tiles' own test, so no key is counted twice
    const int k_end = window > 0 ? min(keep, w_start) : 0;
    const int n_keep_tiles = (k_end + KT - 1) / KT;
    // pooled blocks any row of the block may see: block e with (e + 1) pool - 1 + window <= pmax
    const int n_pool = (pool > 0 && window > 0) ? max(0, pmax - window + 1) / pool : 0;
    const int n_pool_tiles = (n_pool + KT - 1) / KT;
    const int n_tiles = n_pool_tiles + n_keep_tiles + (pmax - w_start) / KT + 1;
    for (int tz = split; tz < n_tiles; tz += nsplit) {
        const bool pooled = tz < n_pool_tiles;   // a tile of pooled pairs: "key" e is block e
        const int ti = tz - n_pool_tiles;
        const bool kept = !pooled && ti < n_keep_tiles;
        const int k0 = pooled ? tz * KT : kept ? ti * KT : w_start + (ti - n_keep_tiles) * KT;
        const int k_last = pooled ? n_pool - 1 : kept ? k_end - 1 : pmax;  // last real key this tile may hold
        const uint16_t* ksrc = pooled ? kp : kc;
        const uint16_t* vsrc = pooled ? vp : vc;
        __syncthreads();
        if (threadIdx.x < KT) {
            const int key = min(k0 + (int)threadIdx.x, k_last);  // past the end: a real row, masked below
            const int per = pooled ? EP : BS;
            krow[threadIdx.x] = (bt[key / per] * per + key % per) * G + kvh;
        }
        __syncthreads();
        // ---- stage: work item = (key pair jp, 8-element chunk dc); lanes of a wave take consecutive key pairs
        for (int it = threadIdx.x; it < PP * kchunks; it += NT) {
            const int jp = it & (PP - 1), dc = it / PP;
            const u16x8 va = *reinterpret_cast<const u16x8*>(ksrc + (int64_t)krow[2 * jp] * D + dc * 8);
            const u16x8 vb = *reinterpret_cast<const u16x8*>(ksrc + (int64_t)krow[2 * jp + 1] * D + dc * 8);
            *reinterpret_cast<u16x8*>(kimg + (2 * jp) * krs + dc * 16) = va;
            *reinterpret_cast<u16x8*>(kimg + (2 * jp + 1) * krs + dc * 16) = vb;
        }
        for (int it = threadIdx.x; it < PP * vchunks; it += NT) {
            const int jp = it & (PP - 1), dc = it / PP;
            const u16x8 va = *reinterpret_cast<const u16x8*>(vsrc + (int64_t)krow[2 * jp] * Dv + dc * 8);
            const u16x8 vb = *reinterpret_cast<const u16x8*>(vsrc + (int64_t)krow[2 * jp + 1] * Dv + dc * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                *reinterpret_cast<uint32_t*>(vimg + (dc * 8 + e) * vts + jp * 4) = (uint32_t)va[e] | ((uint32_t)vb[e] << 16);
        }
        __syncthreads();
        // ---- scores: 4 key tiles of 16; lane gets keys 16 kt + 4 g4 + i of query row qi
        constexpr int NKT = KT / 16;
        f32x4 S[NKT];
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            S[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
            const unsigned char* arow = kimg + (16 * kt + qi) * krs + g4 * 16;
#pragma unroll
            for (int s = 0; s < NS; ++s)
                if (s < ns)
                    S[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(arow + s * 64), qf[s],
                                                                    S[kt], 0, 0, 0);
        }
        // scores, maxima and sums live in the base-2 domain (score * scale * log2 e): one multiply and one
        // subtraction in front of the hardware's exp2.  A tile that every row of the block sees whole (the common case
        // inside a window) skips the per-key visibility tests.
        const bool whole = pooled ? (k0 + KT - 1 <= k_last && (k0 + KT) * pool - 1 + window <= pmin)
                                  : (k0 + KT - 1 <= min(k_last, pmin) && (window <= 0 || kept || pmax - k0 < window) &&
                                     k0 >= c_lo_max);
        float mx = -INFINITY;
        if (whole) {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    S[kt][i] *= scale2;
                    mx = fmaxf(mx, S[kt][i]);
                }
        } else {
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = k0 + 16 * kt + 4 * g4 + i;
                    const bool vis = pooled ? (key <= k_last && (key + 1) * pool - 1 + window <= prow)
                                            : (key <= k_last && key <= prow &&
                                               (window <= 0 || prow - key < window || key < keep) && key >= c_lo);
                    const float sv = vis ? S[kt][i] * scale2 : -INFINITY;
                    S[kt][i] = sv;
                    mx = fmaxf(mx, sv);
                }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(mrow, mx);
        const float corr = (mn == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(mrow - mn);
        const float mref = (mn == -INFINITY) ? 0.f : mn;  // (all masked: every exponent is -inf, every weight 0)
        float sum = 0.f;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = __builtin_amdgcn_exp2f(S[kt][i] - mref);
                S[kt][i] = p;
                sum += p;
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        lrow = lrow * corr + sum;
        mrow = mn;
        // ---- weighted sum of the values: k index of step u = [tile 2u keys 4g4..4g4+3 | tile 2u+1 keys 4g4..4g4+3]
        constexpr int NU = KT / 32;
        // the float weights enter the MFMA as a sum of two bfloat16 terms (the rounded weight and the rounding's
        // remainder), so the weighted sum sees them to about 2^-17 instead of 2^-9
        bf16x8 pf[NU], pl[NU];
#pragma unroll
        for (int u = 0; u < NU; ++u) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float w = S[2 * u + (e >> 2)][e & 3];
                const __bf16 hi = (__bf16)w;
                pf[u][e] = hi;
                pl[u][e] = (__bf16)(w - (float)hi);
            }
        }
#pragma unroll
        for (int c = 0; c < NCT; ++c) {
            if (c < nct) {
                O[c] *= corr;
                const unsigned char* vrow = vimg + (16 * c + qi) * vts + g4 * 8;
#pragma unroll
                for (int u = 0; u < NU; ++u) {
                    const bf16x4 lo = *reinterpret_cast<const bf16x4*>(vrow + u * 64);
                    const bf16x4 hi = *reinterpret_cast<const bf16x4*>(vrow + u * 64 + 32);
                    const bf16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    O[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[u], O[c], 0, 0, 0);
                    O[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl[u], O[c], 0, 0, 0);
                }
            }
        }
    }
    if (!rok) return;
    if (nsplit > 1) {  // unnormalised partial: the combine kernel merges the splits and adds sink and gate
        const int64_t pr = (tok * H + head) * nsplit + split;
        if (g4 == 0) {
            part_ml[pr * 2] = mrow;
            part_ml[pr * 2 + 1] = lrow;
        }
#pragma unroll
        for (int c = 0; c < NCT; ++c)
            if (c < nct) *reinterpret_cast<f32x4*>(part_o + pr * Dv + 16 * c + 4 * g4) = O[c];
        return;
    }
    float oc = 1.f;
    if (sink != nullptr) {
        const float sk = sink[head] * 1.4426950408889634f;   // into the base-2 domain of mrow
        const float mn = fmaxf(mrow, sk);
        oc = mrow == -INFINITY ? 0.f : exp2f(mrow - mn);
        lrow = lrow * oc + exp2f(sk - mn);
    }
    float f = lrow > 0.f ? oc / lrow : 0.f;
    if (gate != nullptr) f *= sigmoidf_(gate[tok * H + head]);
    // lane holds O^T[col = 16 c + 4 g4 + i][query row qi]
    const uint16_t* gsrc = g_off >= 0 ? qkv + tok * ldq + g_off + head * Dv : nullptr;
    auto emit = [&](int c, f32x4 v) {   // the final values of columns 16 c + 4 g4 .. + 3
        if (gsrc != nullptr) {
            const u16x4 gv = *reinterpret_cast<const u16x4*>(gsrc + 16 * c + 4 * g4);
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] *= sigmoidf_(bf2f(gv[i]));
        }
        *reinterpret_cast<u16x4*>(out + (tok * H + head) * Dv + 16 * c + 4 * g4) =
            u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
    };
    if (vcs == nullptr) {
#pragma unroll
        for (int c = 0; c < NCT; ++c)
            if (c < nct) emit(c, O[c] * f);
        return;
    }
    // turn the row back by the query's position: (a, b) -> (a cos + b sin, b cos - a sin) for the column pairs
    // (m, m + Dv / 2); tile c pairs with tile c + nct / 2 (every index below is a compile-time constant)
    const float* cs = vcs + (int64_t)prow * Dv;
    const int hh = nct / 2;
#pragma unroll
    for (int c = 0; c < NCT / 2; ++c)
#pragma unroll
        for (int h2 = 1; h2 <= NCT / 2; ++h2)
            if (h2 == hh && c < hh) {
                const f32x4 a = O[c] * f, b = O[c + h2] * f;
                const f32x4 co = *reinterpret_cast<const f32x4*>(cs + 16 * c + 4 * g4);
                const f32x4 si = *reinterpret_cast<const f32x4*>(cs + Dv / 2 + 16 * c + 4 * g4);
                emit(c, a * co + b * si);
                emit(c + h2, b * co - a * si);
            }
}

// one wave per (token, head) row: out = sum_z 2^(m_z - m) O_z / (sum_z 2^(m_z - m) l_z + 2^(sink log2 e - m)) * sigmoid(gate),
// then (with a table) turned back by the row's position and (with gate columns) times sigmoid of them
__global__ void __launch_bounds__(256) window_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                             const float* __restrict__ sink, const float* __restrict__ gate,
                                                             uint16_t* __restrict__ out, int64_t rows, int H, int Dv,
                                                             int nsplit, const float* __restrict__ vcs,
                                                             const int32_t* __restrict__ pos, const uint16_t* __restrict__ qkv,
                                                             int ldq, int g_off) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    // (the partial maxima are in the base-2 domain: score * scale * log2 e)
    const float sk = sink != nullptr ? sink[r % H] * 1.4426950408889634f : -INFINITY;
    float m = sk;
    for (int z = 0; z < nsplit; ++z) m = fmaxf(m, part_ml[(r * nsplit + z) * 2]);
    float l = sink != nullptr ? exp2f(sk - m) : 0.f;
    for (int z = 0; z < nsplit; ++z) {
        const float mz = part_ml[(r * nsplit + z) * 2];
        if (mz != -INFINITY) l += exp2f(mz - m) * part_ml[(r * nsplit + z) * 2 + 1];
    }
    float f = l > 0.f ? 1.f / l : 0.f;
    if (gate != nullptr) f *= sigmoidf_(gate[r]);
    auto col = [&](int c) {
        float acc = 0.f;
        for (int z = 0; z < nsplit; ++z) {
            const float mz = part_ml[(r * nsplit + z) * 2];
            if (mz != -INFINITY) acc += exp2f(mz - m) * part_o[(r * nsplit + z) * Dv + c];
        }
        return acc * f;
    };
    const uint16_t* gsrc = g_off >= 0 ? qkv + (r / H) * ldq + g_off + (r % H) * Dv : nullptr;
    auto wide = [&](int c) { return gsrc != nullptr ? sigmoidf_(bf2f(gsrc[c])) : 1.f; };
    if (vcs == nullptr) {
        for (int c = lane; c < Dv; c += 64) out[r * Dv + c] = f2bf(col(c) * wide(c));
        return;
    }
    const int half = Dv / 2;
    const float* cs = vcs + (int64_t)pos[r / H] * Dv;
    for (int c = lane; c < half; c += 64) {
        const float a = col(c), b = col(c + half), co = cs[c], si = cs[half + c];
        out[r * Dv + c] = f2bf((a * co + b * si) * wide(c));
        out[r * Dv + c + half] = f2bf((b * co - a * si) * wide(c + half));
    }
}

}  // namespace hy

template <int NS, int NCT, int NW>
static void wa_mfma_launch(const uint16_t* qkv, int ldq, const uint16_t* kc, const uint16_t* vc, const int32_t* bt,
                           int max_blocks, const int32_t* q_start, const int32_t* pos, const float* sink,
                           const float* gate, uint16_t* out, int B, int max_q, int H, int G, int D, int Dv, int BS,
                           float scale, int window, int keep, int chunk, int nsplit, float* part_o, float* part_ml,
                           int pool, int EP, const uint16_t* kp, const uint16_t* vp, const float* vcs, int g_off,
                           hipStream_t s) {
    auto kern = hy::window_attention_mfma_kernel<NS, NCT, NW>;
    const int bytes = hy::WKT * (D * 2 + 16) + Dv * (hy::WKT * 2 + 8);
    static int set_bytes = 0;
    if (bytes > set_bytes) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        set_bytes = bytes;
    }
    const dim3 grid(B, (max_q * (H / G) + 16 * NW - 1) / (16 * NW) * nsplit, G);
    kern<<<grid, 64 * NW, bytes, s>>>(qkv, ldq, kc, vc, bt, max_blocks, q_start, pos, sink, gate, out, H, G, D, Dv, BS, scale,
                                      window, keep, chunk, nsplit, part_o, part_ml, pool, EP, kp, vp, vcs, g_off);
}

bool hy_window_mfma_ok(int ldq, int D, int Dv) { return !(D % 32 || Dv % 16 || D > 256 || Dv > 256 || ldq % 8); }

// Splits of a row block's key tiles over workgroups (merged by a combine kernel) for launches that would leave most
// of the chip idle — decode rows, a lone short portion: enough workgroups to cover the CUs four times, at least 2 key
// tiles per split, at most 16.  The tile count follows from sizes the host knows (the window, or the block table's
// width when there is none).  1 for float32 and sizes the matrix-core kernel does not serve.
int hy_window_nsplit(bool f32, int ldq, int B, int max_q, int H, int G, int D, int Dv, int window, int keep, int chunk,
                     int max_ctx, int pool) {
    if (f32 || !hy_window_mfma_ok(ldq, D, Dv) || B <= 0) return 1;
    const int rows = max_q * (H / G);
    const int wgs = B * ((rows + (rows > 64 ? 127 : 63)) / (rows > 64 ? 128 : 64)) * G;
    if (wgs >= 512) return 1;
    int span = window > 0 ? std::min(max_ctx, window + max_q) : max_ctx;
    if (chunk > 0) span = std::min(span, chunk + max_q);   // a row block's keys start in its first row's chunk
    const int tiles = span / hy::WKT + 1 + (window > 0 ? (std::min(keep, max_ctx) + hy::WKT - 1) / hy::WKT : 0) +
                      (window > 0 && pool > 0 ? (max_ctx / pool + hy::WKT - 1) / hy::WKT : 0);
    int want = (1024 + wgs - 1) / wgs;
    want = std::min(want, std::min(16, tiles / 2));
    return want < 1 ? 1 : want;
}

// false: these sizes are not served here (the caller takes the general kernel).  vcs (a rotation table [P, Dv] for
// turning the outputs back; needs Dv % 32 == 0) and g_off (>= 0: the column of qkv where a gate per output column
// starts) are applied in the epilogue.  nsplit > 1: part_o float
// [T * H * nsplit, Dv] and part_ml float [T * H * nsplit, 2] scratch.
bool launch_hy_window_attention_mfma(const uint16_t* qkv, int ldq, const uint16_t* kc, const uint16_t* vc,
                                     const int32_t* bt, int max_blocks, const int32_t* q_start, const int32_t* pos,
                                     const float* sink, const float* gate, uint16_t* out, int B, int max_q, int H, int G,
                                     int D, int Dv, int BS, float scale, int window, int keep, int chunk, int nsplit,
                                     float* part_o, float* part_ml, int64_t total_rows, int pool, int EP,
                                     const uint16_t* kp, const uint16_t* vp, const float* vcs, int g_off, hipStream_t s) {
    if (!hy_window_mfma_ok(ldq, D, Dv)) return false;
    if (B == 0 || max_q == 0) return true;
#define HY_WAM(NS, NCT, NW) wa_mfma_launch<NS, NCT, NW>(qkv, ldq, kc, vc, bt, max_blocks, q_start, pos, sink, gate, out, B, max_q, H, G, D, Dv, BS, scale, window, keep, chunk, nsplit, part_o, part_ml, pool, EP, kp, vp, vcs, g_off, s)
    // 8 waves per workgroup when a sequence brings more than 64 rows per key/value head: a staged tile then serves
    // 128 rows and every SIMD holds two waves
    const bool nw8 = max_q * (H / G) > 64;
    if (D <= 128 && Dv <= 128) { if (nw8) HY_WAM(4, 8, 8); else HY_WAM(4, 8, 4); }
    else { if (nw8) HY_WAM(8, 16, 8); else HY_WAM(8, 16, 4); }
#undef HY_WAM
    if (nsplit > 1)
        hy::window_combine_kernel<<<(unsigned)((total_rows + 3) / 4), 256, 0, s>>>(part_o, part_ml, sink, gate, out, total_rows, H, Dv, nsplit, vcs, pos, qkv, ldq, g_off);
    return true;
}

}  // namespace chronos
