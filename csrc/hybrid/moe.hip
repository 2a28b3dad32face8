// moe.hip — mixture-of-experts feed-forward of the hybrid decoders.
//
//   route   per token: float router logits (N = experts + identity outputs; the few-row projection of
//           hybrid_elementwise.hip), then one wave per token: softmax over all N, the `top` largest
//           of score + correction chosen (the correction steers the choice only), weights = the chosen outputs' plain
//           scores, not renormalised.  Ties go to the lower index.
//   route_group  sigmoid scores; the outputs form equal groups of neighbours, a group scores its top two
//           scores added up, only the best `keep` groups stay eligible, the `top` largest eligible scores are chosen and
//           weighted by score / (sum of the chosen + 1e-20) * scale.
//   ffn     per token: sum over its chosen experts of weight * W_down act(W_up h); an index >= E is an identity
//           expert (weight * h).  Token-parallel form: one workgroup per token streams the chosen experts' weights
//           (the decode regime: few tokens, every expert matrix read about once; float accumulation throughout).
//
// No step of either kernel depends on the host knowing the routing: both capture into a graph.
#include "hybrid_common.h"

namespace chronos {
namespace hy {

// router outputs N <= 256 (4 per lane)
// One wave per token: z [T, N] float router logits -> the chosen outputs and their weights.
__global__ void __launch_bounds__(256) moe_select_kernel(const float* __restrict__ z, const float* __restrict__ corr,
                                                         int32_t* __restrict__ idx, float* __restrict__ wt, int rows,
                                                         int N, int top) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= rows) return;
    float s[4], c[4];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        s[j] = e < N ? z[t * N + e] : -INFINITY;
        mx = fmaxf(mx, s[j]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s[j] = (lane + 64 * j < N) ? expf(s[j] - mx) : 0.f;
        sum += s[j];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        s[j] = s[j] / sum;
        c[j] = e < N ? s[j] + corr[e] : -INFINITY;
    }
    for (int k = 0; k < top; ++k) {
        // the wave's best (value, lowest index): a lane's own candidates first, then across lanes
        float bv = -INFINITY, bs = 0.f;
        int be = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + 64 * j;
            if (c[j] > bv || (c[j] == bv && e < be && c[j] != -INFINITY)) {
                bv = c[j]; be = e; bs = s[j];
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64), os = __shfl_xor(bs, o, 64);
            const int oe = __shfl_xor(be, o, 64);
            if (ov > bv || (ov == bv && oe < be)) {
                bv = ov; be = oe; bs = os;
            }
        }
        if (lane == 0) {
            idx[t * top + k] = be;
            wt[t * top + k] = bs;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (lane + 64 * j == be) c[j] = -INFINITY;
    }
}

// LDS: h row (d floats) | z (F floats) | out (d floats).
template <typename T>
__global__ void __launch_bounds__(256) moe_ffn_token_kernel(const T* __restrict__ h, const int32_t* __restrict__ idx,
                                                            const float* __restrict__ wt, const T* __restrict__ w_up,
                                                            const T* __restrict__ w_down, T* __restrict__ out, int d,
                                                            int F, int E, int top, int act) {
    extern __shared__ float sm[];
    float* hs = sm;
    float* zs = hs + d;
    float* os = zs + F;
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < d; i += 256) {
        hs[i] = ld<T>(h + t * d + i);
        os[i] = 0.f;
    }
    __syncthreads();
    for (int k = 0; k < top; ++k) {
        const int e = idx[t * top + k];
        const float g = wt[t * top + k];
        if (e >= E) {  // identity expert (uniform over the workgroup)
            for (int i = threadIdx.x; i < d; i += 256) os[i] += g * hs[i];
            __syncthreads();
            continue;
        }
        const T* wu = w_up + (int64_t)e * F * d;
        for (int f = wv; f < F; f += 4) {
            const T* wr = wu + (int64_t)f * d;
            float acc = 0.f;
            for (int i = lane; i < d; i += 64) acc += ld<T>(wr + i) * hs[i];
            acc = wave_sum(acc);
            if (lane == 0) zs[f] = act_apply(rnd<T>(acc), act);
        }
        __syncthreads();
        const T* wd = w_down + (int64_t)e * d * F;
        for (int r = wv; r < d; r += 4) {
            const T* wr = wd + (int64_t)r * F;
            float acc = 0.f;
            for (int i = lane; i < F; i += 64) acc += ld<T>(wr + i) * zs[i];
            acc = wave_sum(acc);
            if (lane == 0) os[r] += g * acc;
        }
        __syncthreads();
    }
    for (int i = threadIdx.x; i < d; i += 256) st<T>(out + t * d + i, os[i]);
}

// One wave per token: the `top` largest of z [T, N] (ties: the lower index), weighted by the softmax over the chosen
// logits only.  top <= 64 (lane k keeps the k-th choice).
__global__ void __launch_bounds__(256) moe_select_topk_kernel(const float* __restrict__ z, int32_t* __restrict__ idx,
                                                              float* __restrict__ wt, int rows, int N, int top) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= rows) return;
    float c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        c[j] = e < N ? z[t * N + e] : -INFINITY;
    }
    float first = 0.f, sum = 0.f, mine = 0.f;  // lane k keeps the k-th chosen logit's exponential
    for (int k = 0; k < top; ++k) {
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + 64 * j;
            if (e < N && (c[j] > bv || (c[j] == bv && e < be))) {
                bv = c[j]; be = e;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64);
            const int oe = __shfl_xor(be, o, 64);
            if (ov > bv || (ov == bv && oe < be)) {
                bv = ov; be = oe;
            }
        }
        if (k == 0) first = bv;  // the largest logit: the softmax's reference point
        const float ex = expf(bv - first);
        sum += ex;
        if (k == lane) {
            mine = ex;
            idx[t * top + k] = be;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (lane + 64 * j == be) c[j] = -INFINITY;
    }
    if (lane < top) wt[t * top + lane] = mine / sum;
}

// One wave per token: sigmoid scores of z [T, N], the choice limited to the best groups (ng groups of N / ng
// neighbouring outputs, a group's score = its top two scores added up, the `keep` best stay; ties: the lower
// index), then the `top` largest eligible scores (ties: the lower index), weights = score / (their sum + 1e-20) * scale.
// ng <= 64 (lane g ranks group g), top <= 64 (lane k keeps the k-th choice).  LDS per wave: N scores, ng flags.
__global__ void __launch_bounds__(256) moe_select_group_kernel(const float* __restrict__ z, int32_t* __restrict__ idx,
                                                               float* __restrict__ wt, int rows, int N, int top, int ng,
                                                               int keep, float scale) {
    __shared__ float sc[4][256];
    __shared__ int okg[4][64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t t = (int64_t)blockIdx.x * 4 + wv;
    if (t >= rows) return;   // (a whole wave leaves; the waves of a block share no barrier)
    const int per = N / ng;
    float s[4], c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        s[j] = e < N ? sigmoidf_(z[t * N + e]) : 0.f;
        if (e < N) sc[wv][e] = s[j];
    }
    // (wave-private LDS rows: a wave's own writes are visible to its later reads)
    if (keep < ng) {
        float gsc = -INFINITY;
        if (lane < ng) {
            float a = -INFINITY, b = -INFINITY;   // the group's two largest
            for (int i = 0; i < per; ++i) {
                const float v = sc[wv][lane * per + i];
                if (v > a) { b = a; a = v; }
                else if (v > b) b = v;
            }
            gsc = per > 1 ? a + b : a;
        }
        int rank = 0;   // groups that come before this one
        for (int g = 0; g < ng; ++g) {
            const float o = __shfl(gsc, g, 64);
            rank += (o > gsc || (o == gsc && g < lane)) ? 1 : 0;
        }
        if (lane < ng) okg[wv][lane] = rank < keep ? 1 : 0;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        c[j] = (e < N && (keep >= ng || okg[wv][e / per])) ? s[j] : -INFINITY;
    }
    float sum = 0.f, mine = 0.f;
    for (int k = 0; k < top; ++k) {
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + 64 * j;
            if (e < N && (c[j] > bv || (c[j] == bv && e < be && c[j] != -INFINITY))) {
                bv = c[j]; be = e;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64);
            const int oe = __shfl_xor(be, o, 64);
            if (ov > bv || (ov == bv && oe < be)) {
                bv = ov; be = oe;
            }
        }
        sum += bv;
        if (k == lane) {
            mine = bv;
            idx[t * top + k] = be;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (lane + 64 * j == be) c[j] = -INFINITY;
    }
    if (lane < top) wt[t * top + lane] = mine / (sum + 1e-20f) * scale;
}

// Gated experts: per token sum_k weight_k * W_down,e ( g sigmoid(slope g) (u + shift) ), g = min(W_gate,e h, limit),
// u = clamp(W_up,e h, +-limit).  w_gu [E, 2F, d]: gate rows then up rows, or (tiled) in the grouped path's tile order.
// LDS: h (d) | gate, up (2F) | out (d).
template <typename T>
__global__ void __launch_bounds__(256) moe_glu_token_kernel(const T* __restrict__ h, const int32_t* __restrict__ idx,
                                                            const float* __restrict__ wt, const T* __restrict__ w_gu,
                                                            const T* __restrict__ w_down, T* __restrict__ out, int d,
                                                            int F, int E, int top, float limit, float slope,
                                                            float shift, int tiled) {
    extern __shared__ float sm[];
    float* hs = sm;
    float* zs = hs + d;
    float* os = zs + 2 * F;
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < d; i += 256) {
        hs[i] = ld<T>(h + t * d + i);
        os[i] = 0.f;
    }
    __syncthreads();
    for (int k = 0; k < top; ++k) {
        const int e = idx[t * top + k];
        const float g = wt[t * top + k];
        if (e < 0 || e >= E) continue;  // (uniform over the workgroup)
        const T* wu = w_gu + (int64_t)e * 2 * F * d;
        for (int f = wv; f < 2 * F; f += 4) {
            int row = f;
            if (tiled) {  // the grouped path's row order: per 128-row tile and 64-row half, 32 gate rows then their up rows
                const int c = f < F ? f : f - F;
                row = (c >> 6) * 128 + ((c >> 5) & 1) * 64 + (c & 31) + (f < F ? 0 : 32);
            }
            const T* wr = wu + (int64_t)row * d;
            float acc = 0.f;
            for (int i = lane; i < d; i += 64) acc += ld<T>(wr + i) * hs[i];
            acc = wave_sum(acc);
            if (lane == 0) zs[f] = rnd<T>(acc);
        }
        __syncthreads();
        for (int f = threadIdx.x; f < F; f += 256) {
            const float a = fminf(zs[f], limit), u = fminf(fmaxf(zs[F + f], -limit), limit);
            zs[f] = rnd<T>(a * sigmoidf_(slope * a) * (u + shift));
        }
        __syncthreads();
        const T* wd = w_down + (int64_t)e * d * F;
        for (int r = wv; r < d; r += 4) {
            const T* wr = wd + (int64_t)r * F;
            float acc = 0.f;
            for (int i = lane; i < F; i += 64) acc += ld<T>(wr + i) * zs[i];
            acc = wave_sum(acc);
            if (lane == 0) os[r] += g * rnd<T>(acc);
        }
        __syncthreads();
    }
    for (int i = threadIdx.x; i < d; i += 256) st<T>(out + t * d + i, os[i]);
}

}  // namespace hy

void launch_hy_rowdot(const void*, const void*, const float*, float*, int, int, int, bool, hipStream_t);

// z: float [T, N] scratch for the router logits (the few-row float32-output projection, then the selection)
void launch_hy_moe_route(const void* h, const void* w, const float* corr, float* z, int32_t* idx, float* wt, int T, int d,
                         int N, int top, bool f32, hipStream_t s) {
    if (T == 0) return;
    launch_hy_rowdot(h, w, nullptr, z, T, d, N, f32, s);
    hy::moe_select_kernel<<<(T + 3) / 4, 256, 0, s>>>(z, corr, idx, wt, T, N, top);
}

void launch_hy_moe_ffn_token(const void* h, const int32_t* idx, const float* wt, const void* w_up, const void* w_down,
                             void* out, int T, int d, int F, int E, int top, int act, bool f32, hipStream_t s) {
    if (T == 0) return;
    const int bytes = (2 * d + F) * 4;
    if (f32) {
        auto kern = hy::moe_ffn_token_kernel<float>;
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        kern<<<T, 256, bytes, s>>>((const float*)h, idx, wt, (const float*)w_up, (const float*)w_down, (float*)out, d, F, E, top, act);
    } else {
        auto kern = hy::moe_ffn_token_kernel<uint16_t>;
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        kern<<<T, 256, bytes, s>>>((const uint16_t*)h, idx, wt, (const uint16_t*)w_up, (const uint16_t*)w_down, (uint16_t*)out, d, F, E, top, act);
    }
}

// z: float [T, N] scratch for the router logits (bias added by the projection), N <= 256
void launch_hy_moe_route_topk(const void* h, const void* w, const float* bias, float* z, int32_t* idx, float* wt, int T,
                              int d, int N, int top, bool f32, hipStream_t s) {
    if (T == 0) return;
    launch_hy_rowdot(h, w, bias, z, T, d, N, f32, s);
    hy::moe_select_topk_kernel<<<(T + 3) / 4, 256, 0, s>>>(z, idx, wt, T, N, top);
}

// z: float [T, N] scratch for the router logits, N <= 256, groups <= 64, top <= 64
void launch_hy_moe_route_group(const void* h, const void* w, float* z, int32_t* idx, float* wt, int T, int d, int N,
                               int top, int ng, int keep, float scale, bool f32, hipStream_t s) {
    if (T == 0) return;
    launch_hy_rowdot(h, w, nullptr, z, T, d, N, f32, s);
    hy::moe_select_group_kernel<<<(T + 3) / 4, 256, 0, s>>>(z, idx, wt, T, N, top, ng, keep, scale);
}

void launch_hy_moe_glu_token(const void* h, const int32_t* idx, const float* wt, const void* w_gu, const void* w_down,
                             void* out, int T, int d, int F, int E, int top, float limit, float slope, float shift,
                             bool tiled, bool f32, hipStream_t s) {
    if (T == 0) return;
    const int bytes = (2 * d + 2 * F) * 4;
    if (f32) {
        auto kern = hy::moe_glu_token_kernel<float>;
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        kern<<<T, 256, bytes, s>>>((const float*)h, idx, wt, (const float*)w_gu, (const float*)w_down, (float*)out, d, F, E, top, limit, slope, shift, tiled);
    } else {
        auto kern = hy::moe_glu_token_kernel<uint16_t>;
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        kern<<<T, 256, bytes, s>>>((const uint16_t*)h, idx, wt, (const uint16_t*)w_gu, (const uint16_t*)w_down, (uint16_t*)out, d, F, E, top, limit, slope, shift, tiled);
    }
}

}  // namespace chronos
