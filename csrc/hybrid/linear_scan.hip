// linear_scan.hip — recurrent mixers whose per-head state is a D x Dv matrix updated by rank-one writes: the gated
// delta rule and gated linear attention, plus the short causal convolution and the per-token scalars that feed them.
//
//   short_conv    y[t, c] = act(bias[c] + sum_i w[c, i] x[t - (K-1) + i, c]) over each sequence's own tokens (the
//                 bias is optional); inputs before the step's first token come from the sequence's history rows (its
//                 last K-1 inputs, by state slot), or are zero when the step starts at position 0.  A second launch
//                 then rewrites the history.
//   delta_prep    per token: 1 / |q|, 1 / |k| per query/key head (float), decay = exp(-exp(A) softplus(a)) and
//                 beta = sigmoid(b) per value head.
//   linear_scan   per (sequence, value head, 64 value columns): the state lives in registers (a wave owns 16 columns,
//                 a lane one column's quarter of the D rows), tokens are staged 16 at a time in LDS (q and k rows in
//                 float, the decays, the values) with the next stage's loads in flight, and every token does
//                     S <- decay * S;  u = v - S^T k (times beta; delta rule only, else u = v);  S <- S + k u^T;
//                     o = S^T q
//                 with two 2-step cross-lane sums (S^T k and S^T q over the four row groups).  decay is one number per
//                 head or one per state row.  The same kernel
//                 serves prompt portions of any length and decode rows (a range of one token); a range that starts at
//                 position 0 starts from the zero state, so a reused slot needs no clearing.
#include "hybrid_common.h"

namespace chronos {
namespace hy {

template <typename T>
__global__ void __launch_bounds__(256) short_conv_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ w,
                                                         const int32_t* __restrict__ tok_seq,
                                                         const int32_t* __restrict__ q_start,
                                                         const int32_t* __restrict__ pos0,
                                                         const int32_t* __restrict__ slots, const T* __restrict__ hist,
                                                         T* __restrict__ y, int C, int K, int silu,
                                                         const float* __restrict__ bias) {
    const int64_t t = blockIdx.x;
    const int b = tok_seq[t];
    const int t0 = q_start[b];
    const bool past = pos0[b] > 0;
    const T* hrow = hist + (int64_t)slots[b] * (K - 1) * C;
    for (int c = threadIdx.x; c < C; c += 256) {
        float acc = bias != nullptr ? bias[c] : 0.f;
        for (int i = 0; i < K; ++i) {
            const int64_t s = t - (K - 1) + i;
            float v = 0.f;
            if (s >= t0) v = ld<T>(x + s * ldx + c);
            else if (past) v = ld<T>(hrow + (int64_t)((K - 1) + (s - t0)) * C + c);
            acc += w[c * K + i] * v;
        }
        if (silu) acc = acc * sigmoidf_(acc);
        st<T>(y + t * C + c, acc);
    }
}

// hist[slot][i] <- the input K-1-i tokens before the sequence's new end.  Entry i reads either this step's tokens or
// an OLDER entry i + n (n >= 1 new tokens), so ascending i in place never reads what it has written.
template <typename T>
__global__ void __launch_bounds__(256) conv_hist_kernel(const T* __restrict__ x, int ldx,
                                                        const int32_t* __restrict__ q_start,
                                                        const int32_t* __restrict__ pos0,
                                                        const int32_t* __restrict__ slots, T* __restrict__ hist, int C,
                                                        int K) {
    const int b = blockIdx.x;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    if (t1 <= t0) return;
    const bool past = pos0[b] > 0;
    T* hrow = hist + (int64_t)slots[b] * (K - 1) * C;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
        for (int i = 0; i < K - 1; ++i) {
            const int64_t s = (int64_t)t1 - (K - 1) + i;
            T v;
            if (s >= t0) v = x[s * ldx + c];
            else if (past) v = hrow[(int64_t)((K - 1) + (s - t0)) * C + c];
            else st<T>(&v, 0.f);
            hrow[(int64_t)i * C + c] = v;
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(256) delta_prep_kernel(const T* __restrict__ y, int ldy, const float* __restrict__ ab,
                                                         const float* __restrict__ a_log, float* __restrict__ qscale,
                                                         float* __restrict__ kscale, float* __restrict__ decay,
                                                         float* __restrict__ beta, int HK, int H, int D, float q_mul) {
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int j = wv; j < 2 * HK; j += 4) {
        const T* row = y + t * ldy + (int64_t)j * D;
        float ss = 0.f;
        for (int i = lane; i < D; i += 64) {
            const float v = ld<T>(row + i);
            ss += v * v;
        }
        const float inv = 1.f / sqrtf(wave_sum(ss) + 1e-6f);
        if (lane == 0) {
            if (j < HK) qscale[t * HK + j] = inv * q_mul;
            else kscale[t * HK + (j - HK)] = inv;
        }
    }
    for (int h = threadIdx.x; h < H; h += 256) {
        const float a = ab[t * 2 * H + h];
        const float sp = a > 20.f ? a : log1pf(expf(a));
        decay[t * H + h] = expf(-expf(a_log[h]) * sp);
        beta[t * H + h] = sigmoidf_(ab[t * 2 * H + H + h]);
    }
}

constexpr int kScanTC = 16;  // tokens per LDS stage
// row groups per wave: a lane holds DP / RG rows of one of the wave's 64 / RG columns.  4 for decode rows (16
// columns = 64-byte runs of the state per row), 8 for prompt portions (half the per-token chain per wave, twice the
// waves)
constexpr int kScanRGDecode = 4, kScanRGPrefill = 8;

template <typename T> __device__ __forceinline__ T zero_of();
template <> __device__ __forceinline__ float zero_of<float>() { return 0.f; }
template <> __device__ __forceinline__ uint16_t zero_of<uint16_t>() { return 0; }

// 256 threads: wave w owns 64 / RG value columns of the workgroup's 4 x 64 / RG; a lane holds DP / RG rows of one
// column.  LDS (floats): q [TC][DP] | k [TC][DP] | (CHD: decay rows [TC][DP]) | v [TC][64] | per token: decay, beta,
// q scale, k scale (times the value's per-head scale when one is given).  The next stage's global loads are issued
// before the current stage's tokens are processed and
// land in LDS afterwards, so the token loop never waits on global memory; the scales of q and k are folded into
// per-token scalars (S^T k_hat = s_k S^T k, k_hat u^T = k (s_k u)^T, S^T q_hat = s_q S^T q).
// PIPE: the one-pass token loops with LDS rows prefetched (more registers: for launches with prompt portions);
// without it the plain order of operations, whose lower register count suits launches of single decode rows, which
// are bound by the state's bytes.
template <typename T, int DP, bool DELTA, bool CHD, bool PIPE>
__global__ void __launch_bounds__(256) linear_scan_kernel(
        const T* __restrict__ proj, int ldp, int q_off, int k_off, int v_off, const float* __restrict__ qscale,
        const float* __restrict__ kscale, float q_mul, const float* __restrict__ decay, int dts, const float* __restrict__ beta,
        const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0, const int32_t* __restrict__ slots,
        float* __restrict__ S, float* __restrict__ o, int HK, int H, int D, int Dv, const float* __restrict__ vscale) {
    constexpr int TC = kScanTC, RG = PIPE ? kScanRGPrefill : kScanRGDecode, CW = 64 / RG, RL = DP / RG;
    constexpr int NE = TC * DP / 256, WC = 4 * CW;  // WC: value columns of the workgroup
    __shared__ __attribute__((aligned(16))) float qs[TC * DP];
    __shared__ __attribute__((aligned(16))) float ks[TC * DP];
    __shared__ __attribute__((aligned(16))) float ds[CHD ? TC * DP : 4];
    __shared__ float vs[TC * WC];
    __shared__ float gs[TC], bs[TC], qsc[TC], ksc[TC];
    const int b = blockIdx.x, hd = blockIdx.y;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    if (t1 <= t0) return;
    const int hk = hd / (H / HK);
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, rg = lane / CW, c = lane % CW;
    const int col0 = blockIdx.z * WC;
    const int col = col0 + wv * CW + c;
    const bool live = col < Dv;
    float* Sp = S + (((int64_t)slots[b] * H + hd) * D) * Dv + col;
    float st_[RL];
    if (pos0[b] > 0 && live) {
#pragma unroll
        for (int i = 0; i < RL; ++i) st_[i] = rg * RL + i < D ? Sp[(int64_t)(rg * RL + i) * Dv] : 0.f;
    } else {
#pragma unroll
        for (int i = 0; i < RL; ++i) st_[i] = 0.f;
    }
    // staging registers of one stage: element e of thread x is (token e' = (x + 256 e) / DP, row (x + 256 e) % DP)
    constexpr int NV = (TC * WC + 255) / 256;
    T qraw[NE], kraw[NE], vraw[NV];
    float draw[CHD ? NE : 1], sraw[4];
    auto fetch = [&](int tb) {
        const int nt = min(TC, t1 - tb);
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const int i = threadIdx.x + 256 * e, tt = i / DP, r = i % DP;
            const bool ok = tt < nt && r < D;
            const int64_t t = tb + tt;
            qraw[e] = ok ? proj[t * ldp + q_off + hk * D + r] : zero_of<T>();
            kraw[e] = ok ? proj[t * ldp + k_off + hk * D + r] : zero_of<T>();
            if constexpr (CHD) draw[e] = ok ? decay[(t * H + hd) * D + r] : 0.f;
        }
#pragma unroll
        for (int e = 0; e < NV; ++e) {
            const int i = threadIdx.x + 256 * e, tt = i / WC, cc = col0 + i % WC;
            vraw[e] = (tt < nt && cc < Dv) ? proj[(int64_t)(tb + tt) * ldp + v_off + hd * Dv + cc] : zero_of<T>();
        }
        if (threadIdx.x < TC) {
            const bool ok = (int)threadIdx.x < nt;
            const int64_t t = tb + threadIdx.x;
            sraw[0] = (!CHD && ok) ? decay[t * dts + hd] : 1.f;   // dts = 0: the same decays for every token
            sraw[1] = (DELTA && ok) ? beta[t * H + hd] : 0.f;
            sraw[2] = (qscale != nullptr && ok) ? qscale[t * HK + hk] : q_mul;
            sraw[3] = (kscale != nullptr && ok) ? kscale[t * HK + hk] : 1.f;
            // a per-head factor on the written value u = v: k (s u)^T is all it enters (no delta correction then)
            if (!DELTA && vscale != nullptr && ok) sraw[3] *= vscale[t * H + hd];
        }
    };
    auto land = [&]() {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const int i = threadIdx.x + 256 * e;
            qs[i] = ld<T>(&qraw[e]);
            ks[i] = ld<T>(&kraw[e]);
            if constexpr (CHD) ds[i] = draw[e];
        }
#pragma unroll
        for (int e = 0; e < NV; ++e)
            if (threadIdx.x + 256 * e < TC * WC) vs[threadIdx.x + 256 * e] = ld<T>(&vraw[e]);
        if (threadIdx.x < TC) {
            gs[threadIdx.x] = sraw[0];
            bs[threadIdx.x] = sraw[1];
            qsc[threadIdx.x] = sraw[2];
            ksc[threadIdx.x] = sraw[3];
        }
    };
    fetch(t0);
    for (int tb = t0; tb < t1; tb += TC) {
        const int nt = min(TC, t1 - tb);
        __syncthreads();  // the previous stage has been consumed
        land();
        __syncthreads();
        if (tb + TC < t1) fetch(tb + TC);
        // a lane's RL rows of token tt's staged row, as registers (one batch of 16-byte LDS reads)
        auto ldrow = [&](const float* base, int tt, float (&dst)[RL]) {
            const f32x4* p4 = reinterpret_cast<const f32x4*>(base + tt * DP + rg * RL);
#pragma unroll
            for (int i = 0; i < RL; i += 4) {
                const f32x4 v = p4[i >> 2];
                dst[i] = v[0]; dst[i + 1] = v[1]; dst[i + 2] = v[2]; dst[i + 3] = v[3];
            }
        };
        auto rsum = [&](float x) {   // over the row groups
#pragma unroll
            for (int o = CW; o < 64; o <<= 1) x += __shfl_xor(x, o, 64);
            return x;
        };
        if constexpr (PIPE && DELTA && !CHD) {
            // The delta rule with one decay per head, one pass over the state per token: the pass that writes token
            // t and reads it out also forms S^T k of token t + 1 (its decay is a scalar factor applied afterwards),
            // so the two cross-lane sums of a token run side by side and the next token's k rows are read from LDS
            // while the current token is computed.  Two register sets of k rows alternate.
            float ka[RL], kb[RL], qc[RL];
            ldrow(ks, 0, ka);
            float p;
            {
                float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
                for (int i = 0; i < RL; i += 4) {
                    p0 += st_[i] * ka[i]; p1 += st_[i + 1] * ka[i + 1]; p2 += st_[i + 2] * ka[i + 2]; p3 += st_[i + 3] * ka[i + 3];
                }
                p = rsum((p0 + p1) + (p2 + p3));
            }
            auto step = [&](int tt, float (&kc)[RL], float (&kn)[RL]) {
                ldrow(qs, tt, qc);
                if (tt + 1 < nt) ldrow(ks, tt + 1, kn);   // (else kn keeps old rows: the sum below is not used)
                const float g = gs[tt], sk = ksc[tt];
                const float u = bs[tt] * (vs[tt * WC + wv * CW + c] - g * sk * p);
                const float uk = u * sk;
                float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f, n0 = 0.f, n1 = 0.f, n2 = 0.f, n3 = 0.f;
#pragma unroll
                for (int i = 0; i < RL; i += 4) {
                    st_[i] = g * st_[i] + kc[i] * uk;
                    st_[i + 1] = g * st_[i + 1] + kc[i + 1] * uk;
                    st_[i + 2] = g * st_[i + 2] + kc[i + 2] * uk;
                    st_[i + 3] = g * st_[i + 3] + kc[i + 3] * uk;
                    a0 += st_[i] * qc[i]; a1 += st_[i + 1] * qc[i + 1]; a2 += st_[i + 2] * qc[i + 2]; a3 += st_[i + 3] * qc[i + 3];
                    n0 += st_[i] * kn[i]; n1 += st_[i + 1] * kn[i + 1]; n2 += st_[i + 2] * kn[i + 2]; n3 += st_[i + 3] * kn[i + 3];
                }
                const float a = rsum((a0 + a1) + (a2 + a3));
                p = rsum((n0 + n1) + (n2 + n3));
                if (live && rg == 0) o[((int64_t)(tb + tt) * H + hd) * Dv + col] = a * qsc[tt];
            };
            for (int tt = 0; tt < nt; tt += 2) {
                step(tt, ka, kb);
                if (tt + 1 < nt) step(tt + 1, kb, ka);
            }
        } else if constexpr (PIPE && !DELTA && CHD) {
            // Per-row decays without the delta correction (gated linear attention): one fused pass per token,
            // S <- d S + k v^T and o = S^T q; the next token's rows are read from LDS during the current pass.
            float da[RL], ka[RL], qa[RL], db[RL], kb[RL], qb[RL];
            ldrow(ds, 0, da); ldrow(ks, 0, ka); ldrow(qs, 0, qa);
            auto step = [&](int tt, float (&dc)[RL], float (&kc)[RL], float (&qc)[RL], float (&dn)[RL], float (&kn)[RL], float (&qn)[RL]) {
                if (tt + 1 < nt) { ldrow(ds, tt + 1, dn); ldrow(ks, tt + 1, kn); ldrow(qs, tt + 1, qn); }
                const float uk = vs[tt * WC + wv * CW + c] * ksc[tt];
                float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
                for (int i = 0; i < RL; i += 4) {
                    st_[i] = dc[i] * st_[i] + kc[i] * uk;
                    st_[i + 1] = dc[i + 1] * st_[i + 1] + kc[i + 1] * uk;
                    st_[i + 2] = dc[i + 2] * st_[i + 2] + kc[i + 2] * uk;
                    st_[i + 3] = dc[i + 3] * st_[i + 3] + kc[i + 3] * uk;
                    a0 += st_[i] * qc[i]; a1 += st_[i + 1] * qc[i + 1]; a2 += st_[i + 2] * qc[i + 2]; a3 += st_[i + 3] * qc[i + 3];
                }
                const float a = rsum((a0 + a1) + (a2 + a3));
                if (live && rg == 0) o[((int64_t)(tb + tt) * H + hd) * Dv + col] = a * qsc[tt];
            };
            for (int tt = 0; tt < nt; tt += 2) {
                step(tt, da, ka, qa, db, kb, qb);
                if (tt + 1 < nt) step(tt + 1, db, kb, qb, da, ka, qa);
            }
        } else if constexpr (PIPE && !DELTA && !CHD) {
            // One decay per head without the delta correction (the state-space form): one fused pass per token,
            // S <- g S + k (s v)^T and o = S^T q; the next token's rows are read from LDS during the current pass.
            float ka[RL], qa[RL], kb[RL], qb[RL];
            ldrow(ks, 0, ka); ldrow(qs, 0, qa);
            auto step = [&](int tt, float (&kc)[RL], float (&qc)[RL], float (&kn)[RL], float (&qn)[RL]) {
                if (tt + 1 < nt) { ldrow(ks, tt + 1, kn); ldrow(qs, tt + 1, qn); }
                const float g = gs[tt];
                const float uk = vs[tt * WC + wv * CW + c] * ksc[tt];
                float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
                for (int i = 0; i < RL; i += 4) {
                    st_[i] = g * st_[i] + kc[i] * uk;
                    st_[i + 1] = g * st_[i + 1] + kc[i + 1] * uk;
                    st_[i + 2] = g * st_[i + 2] + kc[i + 2] * uk;
                    st_[i + 3] = g * st_[i + 3] + kc[i + 3] * uk;
                    a0 += st_[i] * qc[i]; a1 += st_[i + 1] * qc[i + 1]; a2 += st_[i + 2] * qc[i + 2]; a3 += st_[i + 3] * qc[i + 3];
                }
                const float a = rsum((a0 + a1) + (a2 + a3));
                if (live && rg == 0) o[((int64_t)(tb + tt) * H + hd) * Dv + col] = a * qsc[tt];
            };
            for (int tt = 0; tt < nt; tt += 2) {
                step(tt, ka, qa, kb, qb);
                if (tt + 1 < nt) step(tt + 1, kb, qb, ka, qa);
            }
        } else {
            // the plain order of operations
            for (int tt = 0; tt < nt; ++tt) {
                float kc[RL], qc[RL];
                ldrow(ks, tt, kc); ldrow(qs, tt, qc);
                float g = 1.f;
                if constexpr (CHD) {
                    float dc[RL];
                    ldrow(ds, tt, dc);
#pragma unroll
                    for (int i = 0; i < RL; ++i) st_[i] *= dc[i];
                } else {
                    g = gs[tt];
                }
                const float sk = ksc[tt];
                float u = vs[tt * WC + wv * CW + c];
                if constexpr (DELTA) {
                    float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
                    for (int i = 0; i < RL; i += 4) {
                        p0 += st_[i] * kc[i]; p1 += st_[i + 1] * kc[i + 1]; p2 += st_[i + 2] * kc[i + 2]; p3 += st_[i + 3] * kc[i + 3];
                    }
                    u = bs[tt] * (u - g * sk * rsum((p0 + p1) + (p2 + p3)));
                }
                const float uk = u * sk;
                float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
                for (int i = 0; i < RL; i += 4) {
                    st_[i] = g * st_[i] + kc[i] * uk;
                    st_[i + 1] = g * st_[i + 1] + kc[i + 1] * uk;
                    st_[i + 2] = g * st_[i + 2] + kc[i + 2] * uk;
                    st_[i + 3] = g * st_[i + 3] + kc[i + 3] * uk;
                    a0 += st_[i] * qc[i]; a1 += st_[i + 1] * qc[i + 1]; a2 += st_[i + 2] * qc[i + 2]; a3 += st_[i + 3] * qc[i + 3];
                }
                const float a = rsum((a0 + a1) + (a2 + a3));
                if (live && rg == 0) o[((int64_t)(tb + tt) * H + hd) * Dv + col] = a * qsc[tt];
            }
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < RL; ++i)
            if (rg * RL + i < D) Sp[(int64_t)(rg * RL + i) * Dv] = st_[i];
    }
}

}  // namespace hy

// x points at the first convolved column of the first row (rows ldx apart); bias may be nullptr
void launch_hy_short_conv(const void* x, int ldx, const float* w, const float* bias, const int32_t* tok_seq,
                          const int32_t* q_start, const int32_t* pos0, const int32_t* slots, void* hist, void* y, int T,
                          int B, int C, int K, bool silu, bool f32, hipStream_t s) {
    if (T == 0 || C == 0) return;
    const dim3 hg(B, (C + 255) / 256);
    if (f32) {
        hy::short_conv_kernel<float><<<T, 256, 0, s>>>((const float*)x, ldx, w, tok_seq, q_start, pos0, slots, (const float*)hist, (float*)y, C, K, silu, bias);
        if (K > 1) hy::conv_hist_kernel<float><<<hg, 256, 0, s>>>((const float*)x, ldx, q_start, pos0, slots, (float*)hist, C, K);
    } else {
        hy::short_conv_kernel<uint16_t><<<T, 256, 0, s>>>((const uint16_t*)x, ldx, w, tok_seq, q_start, pos0, slots, (const uint16_t*)hist, (uint16_t*)y, C, K, silu, bias);
        if (K > 1) hy::conv_hist_kernel<uint16_t><<<hg, 256, 0, s>>>((const uint16_t*)x, ldx, q_start, pos0, slots, (uint16_t*)hist, C, K);
    }
}

void launch_hy_delta_prep(const void* y, int ldy, const float* ab, const float* a_log, float* qscale, float* kscale,
                          float* decay, float* beta, int T, int HK, int H, int D, float q_mul, bool f32, hipStream_t s) {
    if (T == 0) return;
    if (f32) hy::delta_prep_kernel<float><<<T, 256, 0, s>>>((const float*)y, ldy, ab, a_log, qscale, kscale, decay, beta, HK, H, D, q_mul);
    else hy::delta_prep_kernel<uint16_t><<<T, 256, 0, s>>>((const uint16_t*)y, ldy, ab, a_log, qscale, kscale, decay, beta, HK, H, D, q_mul);
}

template <typename T, int DP, bool DELTA, bool CHD>
static void linear_scan_launch(bool pipe, const T* proj, int ldp, int q_off, int k_off, int v_off, const float* qscale,
                               const float* kscale, float q_mul, const float* decay, int dts, const float* beta,
                               const int32_t* q_start, const int32_t* pos0, const int32_t* slots, float* S, float* o, int B,
                               int HK, int H, int D, int Dv, const float* vscale, hipStream_t s) {
    constexpr bool HAS_PIPE = !(DELTA && CHD);   // the combinations with a pipelined token loop
    if constexpr (HAS_PIPE) {
        const int zp = (Dv + 4 * (64 / hy::kScanRGPrefill) - 1) / (4 * (64 / hy::kScanRGPrefill));
        // The head-decay form without the delta correction serves layers of many narrow heads: once its pipelined
        // launch (twice the workgroups) no longer fits on the chip at once, the plain loop with half the
        // workgroups is faster (measured at 128 heads of 64 columns: 1.71 ms pipelined, 1.10 ms plain; at 32 heads
        // 0.81 against 0.93 ms).
        if constexpr (!DELTA && !CHD) pipe = pipe && (int64_t)B * H * zp <= 512;
        if (pipe) {
            const dim3 grid(B, H, zp);
            hy::linear_scan_kernel<T, DP, DELTA, CHD, true><<<grid, 256, 0, s>>>(proj, ldp, q_off, k_off, v_off, qscale, kscale, q_mul, decay, dts,
                                                                                beta, q_start, pos0, slots, S, o, HK, H, D, Dv, vscale);
            return;
        }
    }
    const dim3 grid(B, H, (Dv + 4 * (64 / hy::kScanRGDecode) - 1) / (4 * (64 / hy::kScanRGDecode)));
    hy::linear_scan_kernel<T, DP, DELTA, CHD, false><<<grid, 256, 0, s>>>(proj, ldp, q_off, k_off, v_off, qscale, kscale, q_mul, decay, dts,
                                                                         beta, q_start, pos0, slots, S, o, HK, H, D, Dv, vscale);
}

template <typename T, bool DELTA, bool CHD>
static bool linear_scan_d(bool pipe, const T* proj, int ldp, int q_off, int k_off, int v_off, const float* qscale,
                          const float* kscale, float q_mul, const float* decay, int dts, const float* beta, const int32_t* q_start,
                          const int32_t* pos0, const int32_t* slots, float* S, float* o, int B, int HK, int H, int D,
                          int Dv, const float* vscale, hipStream_t s) {
#define HY_LS(DP)                                                                                                     \
    linear_scan_launch<T, DP, DELTA, CHD>(pipe, proj, ldp, q_off, k_off, v_off, qscale, kscale, q_mul, decay, dts, beta, q_start, \
                                          pos0, slots, S, o, B, HK, H, D, Dv, vscale, s)
    if (D <= 32) HY_LS(32);
    else if (D <= 64) HY_LS(64);
    else if (D <= 128) HY_LS(128);
    else if (D <= 256) HY_LS(256);
    else return false;
#undef HY_LS
    return true;
}

// delta: beta != nullptr.  vscale (float [T, H], may be nullptr; without delta only): a factor on the written value.
// chd: decay holds one number per state row ([T, H, D]) instead of one per head ([T, H]).
// fixed (not with chd): decay holds one number per head for all tokens ([H]).
// Returns false when D has no instantiation (D > 256).
bool launch_hy_linear_scan(const void* proj, int ldp, int q_off, int k_off, int v_off, const float* qscale,
                           const float* kscale, float q_mul, const float* decay, bool chd, bool fixed, const float* beta,
                           const int32_t* q_start, const int32_t* pos0, const int32_t* slots, float* S, float* o, int T,
                           int B, int HK, int H, int D, int Dv, const float* vscale, bool f32, hipStream_t s) {
    if (B == 0) return true;
    const bool pipe = T > B;   // some sequence brings more than one token
    const bool delta = beta != nullptr;
    const int dts = fixed ? 0 : H;
#define HY_LSD(T, DELTA, CHD)                                                                                        \
    return linear_scan_d<T, DELTA, CHD>(pipe, (const T*)proj, ldp, q_off, k_off, v_off, qscale, kscale, q_mul, decay, dts, beta, \
                                        q_start, pos0, slots, S, o, B, HK, H, D, Dv, vscale, s)
    if (f32) {
        if (delta && chd) HY_LSD(float, true, true);
        if (delta) HY_LSD(float, true, false);
        if (chd) HY_LSD(float, false, true);
        HY_LSD(float, false, false);
    } else {
        if (delta && chd) HY_LSD(uint16_t, true, true);
        if (delta) HY_LSD(uint16_t, true, false);
        if (chd) HY_LSD(uint16_t, false, true);
        HY_LSD(uint16_t, false, false);
    }
#undef HY_LSD
}

}  // namespace chronos
