// pre_norm.hip — the float32 residual stream of pre-norm hybrid decoders, the per-layer token input's gate, and the
// element-wise parts of the state-space and gated linear recurrent mixers.
//
//   add_rms_norm      the stream's join, one workgroup per row:
//                         v = y (+ sigmoid(g2) y2);   [w_y:]  v <- v / sqrt(mean(v^2) + eps) * w_y;   x <- x + v
//                     and what the next sublayer reads, in the activation type: rms_norm(x) * w_out, or x itself
//                     (the token input's gate projects the stream, not a norm of it), or nothing.  All arithmetic in
//                     float; x is float and updated in place.  Rows up to 4096 wide are read once.
//   token_gate        out = gelu_tanh(a) * table[id, col0 : col0 + n]
//   ssm_prep          dt = softplus(dt_pre),  decay = exp(-exp(A) dt)          per token and head, float
//   gated_group_norm  y = (o + D_h x) silu(z), then RMS norm in equal groups of columns, times a weight
//   rglru_scan        per channel  S <- a S + sqrt(1 - a^2) i u,  a = exp(-c sigmoid(r) softplus(lam)), out = S gelu(y).
//                     A thread owns one channel of one chunk of 64 tokens of one sequence.  Sequences longer than a
//                     chunk run in two launches: the first forms every chunk's (product of a, end state from zero),
//                     the second folds the earlier chunks' pairs into the chunk's starting state and walks the chunk;
//                     the per-token arithmetic inside a chunk is that of the token-by-token form.  Loads of four
//                     tokens are issued together ahead of their four dependent updates.
#include "hybrid_common.h"

namespace chronos {
namespace hy {

template <typename T> __device__ __forceinline__ f32x4 pn_ld4(const T* p);
template <> __device__ __forceinline__ f32x4 pn_ld4<float>(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
template <> __device__ __forceinline__ f32x4 pn_ld4<uint16_t>(const uint16_t* p) {
    const u16x4 v = *reinterpret_cast<const u16x4*>(p);
    return f32x4{bf2f(v[0]), bf2f(v[1]), bf2f(v[2]), bf2f(v[3])};
}
template <typename T> __device__ __forceinline__ void pn_st4(T* p, const f32x4& v);
template <> __device__ __forceinline__ void pn_st4<float>(float* p, const f32x4& v) { *reinterpret_cast<f32x4*>(p) = v; }
template <> __device__ __forceinline__ void pn_st4<uint16_t>(uint16_t* p, const f32x4& v) {
    *reinterpret_cast<u16x4*>(p) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
}

__device__ __forceinline__ float gelu_tanhf_(float z) {
    return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
// The scan's per-token math on the hardware's exp2 and reciprocal (each good to about one unit in the last place):
// a token costs a wave two sigmoids, an exponential, 1 - exp(x), a root and a tanh, and the library forms of these
// (range reduction, IEEE division) made the scan ALU-bound.
__device__ __forceinline__ float fast_exp_(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float fast_sigmoid_(float x) { return __builtin_amdgcn_rcpf(1.f + fast_exp_(-x)); }
// 1 - exp(x) for x <= 0: the series near zero (where the subtraction would cancel), the exponential elsewhere
__device__ __forceinline__ float one_minus_exp_(float x) {
    const float p = -x * (1.f + x * (0.5f + x * (1.f / 6.f + x * (1.f / 24.f + x * (1.f / 120.f + x * (1.f / 720.f))))));
    return x > -0.25f ? p : 1.f - fast_exp_(x);
}
__device__ __forceinline__ float fast_gelu_tanh_(float z) {
    const float t = 0.7978845608028654f * (z + 0.044715f * z * z * z);   // tanh(t) = 1 - 2 / (exp(2t) + 1)
    return 0.5f * z * (2.f - 2.f * __builtin_amdgcn_rcpf(fast_exp_(2.f * t) + 1.f));
}
__device__ __forceinline__ float softplusf_(float z) { return z > 30.f ? z : log1pf(expf(z)); }

// emit: 0 nothing, 1 the updated row, 2 its RMS norm times w_out.  VEC: d % 4 == 0 (16-byte accesses).
template <typename T, bool VEC>
__global__ void __launch_bounds__(256) add_rms_norm_kernel(const T* __restrict__ y, const T* __restrict__ y2,
                                                           const float* __restrict__ g2, const float* __restrict__ w_y,
                                                           float* __restrict__ x, const float* __restrict__ w_out,
                                                           T* __restrict__ h, int d, float eps, int emit) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float* xr = x + row * d;
    const T* yr = y + row * d;
    const T* y2r = y2 != nullptr ? y2 + row * d : nullptr;
    const float s2 = y2 != nullptr ? sigmoidf_(g2[row]) : 0.f;
    T* hr = h != nullptr ? h + row * d : nullptr;
    if constexpr (VEC) {
        auto val = [&](int i) {
            f32x4 v = pn_ld4<T>(yr + i);
            if (y2r != nullptr) v = v + pn_ld4<T>(y2r + i) * s2;
            return v;
        };
        f32x4 c[4];
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = (threadIdx.x + 256 * j) * 4;
            c[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (i < d) {
                c[j] = val(i);
                ss += c[j][0] * c[j][0] + c[j][1] * c[j][1] + c[j][2] * c[j][2] + c[j][3] * c[j][3];
            }
        }
        float rs = 1.f;
        if (w_y != nullptr) {
            for (int i = (threadIdx.x + 1024) * 4; i < d; i += 1024) {
                const f32x4 v = val(i);
                ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
            }
            rs = 1.f / sqrtf(block_sum(ss, red) / (float)d + eps);
        }
        ss = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = (threadIdx.x + 256 * j) * 4;
            if (i < d) {
                f32x4 v = c[j];
                if (w_y != nullptr) v = v * rs * *reinterpret_cast<const f32x4*>(w_y + i);
                v = v + *reinterpret_cast<const f32x4*>(xr + i);
                *reinterpret_cast<f32x4*>(xr + i) = v;
                c[j] = v;
                ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
            }
        }
        for (int i = (threadIdx.x + 1024) * 4; i < d; i += 1024) {
            f32x4 v = val(i);
            if (w_y != nullptr) v = v * rs * *reinterpret_cast<const f32x4*>(w_y + i);
            v = v + *reinterpret_cast<const f32x4*>(xr + i);
            *reinterpret_cast<f32x4*>(xr + i) = v;
            ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
        }
        if (emit == 0 || hr == nullptr) return;
        const float rstd = emit == 2 ? 1.f / sqrtf(block_sum(ss, red) / (float)d + eps) : 1.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = (threadIdx.x + 256 * j) * 4;
            if (i < d) pn_st4<T>(hr + i, emit == 2 ? c[j] * rstd * *reinterpret_cast<const f32x4*>(w_out + i) : c[j]);
        }
        for (int i = (threadIdx.x + 1024) * 4; i < d; i += 1024) {  // (a thread re-reads what it wrote itself)
            const f32x4 v = *reinterpret_cast<const f32x4*>(xr + i);
            pn_st4<T>(hr + i, emit == 2 ? v * rstd * *reinterpret_cast<const f32x4*>(w_out + i) : v);
        }
    } else {
        auto val = [&](int i) {
            float v = ld<T>(yr + i);
            if (y2r != nullptr) v += ld<T>(y2r + i) * s2;
            return v;
        };
        float rs = 1.f;
        if (w_y != nullptr) {
            float ss = 0.f;
            for (int i = threadIdx.x; i < d; i += 256) {
                const float v = val(i);
                ss += v * v;
            }
            rs = 1.f / sqrtf(block_sum(ss, red) / (float)d + eps);
        }
        float ss = 0.f;
        for (int i = threadIdx.x; i < d; i += 256) {
            float v = val(i);
            if (w_y != nullptr) v = v * rs * w_y[i];
            v += xr[i];
            xr[i] = v;
            ss += v * v;
        }
        if (emit == 0 || hr == nullptr) return;
        const float rstd = emit == 2 ? 1.f / sqrtf(block_sum(ss, red) / (float)d + eps) : 1.f;
        for (int i = threadIdx.x; i < d; i += 256) st<T>(hr + i, emit == 2 ? xr[i] * rstd * w_out[i] : xr[i]);
    }
}

template <typename T>
__global__ void __launch_bounds__(256) token_gate_kernel(const T* __restrict__ a, const int32_t* __restrict__ ids,
                                                         const T* __restrict__ table, int ldt, int col0,
                                                         T* __restrict__ out, int64_t total, int n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int64_t t = i / n;
    const int c = (int)(i % n);
    st<T>(out + i, gelu_tanhf_(ld<T>(a + i)) * ld<T>(table + (int64_t)ids[t] * ldt + col0 + c));
}

__global__ void __launch_bounds__(256) ssm_prep_kernel(const float* __restrict__ dt_pre, const float* __restrict__ a_log,
                                                       float* __restrict__ decay, float* __restrict__ dt, int64_t total,
                                                       int H) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const float s = softplusf_(dt_pre[i]);
    dt[i] = s;
    decay[i] = expf(-expf(a_log[i % H]) * s);
}

// one workgroup per (token, group of gs columns); NT threads
template <typename T>
__global__ void gated_group_norm_kernel(const float* __restrict__ o, const T* __restrict__ xs, int ldx, int x_off,
                                        const float* __restrict__ skip, const T* __restrict__ zs, int ldz, int z_off,
                                        const float* __restrict__ w, T* __restrict__ y, int n, int gs, int Dv,
                                        float eps) {
    __shared__ float red[16];
    const int groups = n / gs;
    const int64_t t = blockIdx.x / groups;
    const int c0 = (int)(blockIdx.x % groups) * gs;
    auto val = [&](int c) {
        const float z = ld<T>(zs + t * ldz + z_off + c);
        return (o[t * n + c] + skip[c / Dv] * ld<T>(xs + t * ldx + x_off + c)) * (z * sigmoidf_(z));
    };
    float ss = 0.f;
    for (int i = threadIdx.x; i < gs; i += blockDim.x) {
        const float v = val(c0 + i);
        ss += v * v;
    }
    const float rstd = 1.f / sqrtf(block_sum(ss, red) / (float)gs + eps);
    for (int i = threadIdx.x; i < gs; i += blockDim.x) st<T>(y + t * n + c0 + i, val(c0 + i) * rstd * w[c0 + i]);
}

constexpr int kLruChunk = 64;  // tokens per chunk

// PHASE 1: per (sequence, chunk but the last, channel) the chunk's product of a and its end state from zero -> pq
// [B, NCH, 2, W]; chunk 0 also copies the sequence's starting state (its slot's row, or zero at position 0) to init
// [B, W].  PHASE 2: fold the earlier chunks into the starting state, walk the chunk, write the outputs; the last
// chunk writes the slot's row.  With one chunk per sequence at most (NCH == 1) only PHASE 2 runs and reads the
// slot's row itself.
template <typename T, int PHASE>
__global__ void __launch_bounds__(256) rglru_scan_kernel(const T* __restrict__ u, const float* __restrict__ gates,
                                                         const float* __restrict__ sp, float cc, const T* __restrict__ ys,
                                                         int ldy, int y_off, const int32_t* __restrict__ q_start,
                                                         const int32_t* __restrict__ pos0, const int32_t* __restrict__ slots,
                                                         float* __restrict__ S, float* __restrict__ pq,
                                                         float* __restrict__ init, T* __restrict__ out, int Ttot, int W,
                                                         int bw, int NCH) {
    const int b = blockIdx.x, k = blockIdx.z;
    const int c = blockIdx.y * 256 + threadIdx.x;
    const int s0 = q_start[b], s1 = q_start[b + 1];
    const int t0 = s0 + k * kLruChunk;
    if (c >= W || t0 >= s1) return;
    const int t1 = min(s1, t0 + kLruChunk);
    const bool last = t1 == s1;
    float* Srow = S + (int64_t)slots[b] * W;
    if (PHASE == 1) {
        if (k == 0) init[(int64_t)b * W + c] = pos0[b] > 0 ? Srow[c] : 0.f;
        if (last) return;
    }
    const float spc = sp[c];
    const float* gr = gates + ((int64_t)(c / bw) * Ttot) * 2 * bw + c % bw;   // + t * 2 bw (+ bw for the input gate)
    float s = 0.f, P = 1.f;
    if (PHASE == 2) {
        if (NCH == 1) s = pos0[b] > 0 ? Srow[c] : 0.f;
        else {
            s = init[(int64_t)b * W + c];
            const float* p = pq + ((int64_t)b * NCH) * 2 * W + c;
            for (int j = 0; j < k; ++j) s = p[(int64_t)j * 2 * W] * s + p[(int64_t)j * 2 * W + W];
        }
    }
    for (int tb = t0; tb < t1; tb += 4) {
        float a[4], m[4], g[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int t = min(tb + e, t1 - 1);
            const float r = fast_sigmoid_(gr[(int64_t)t * 2 * bw]);
            const float ig = fast_sigmoid_(gr[(int64_t)t * 2 * bw + bw]);
            const float la = -cc * r * spc;
            a[e] = fast_exp_(la);
            m[e] = __builtin_amdgcn_sqrtf(one_minus_exp_(2.f * la)) * ig * ld<T>(u + (int64_t)t * W + c);
            if (PHASE == 2) g[e] = fast_gelu_tanh_(ld<T>(ys + (int64_t)t * ldy + y_off + c));
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (tb + e < t1) {
                s = a[e] * s + m[e];
                if (PHASE == 1) P *= a[e];
                else st<T>(out + (int64_t)(tb + e) * W + c, s * g[e]);
            }
        }
    }
    if (PHASE == 1) {
        float* p = pq + (((int64_t)b * NCH + k) * 2) * W + c;
        p[0] = P;
        p[W] = s;
    } else if (last) {
        Srow[c] = s;
    }
}

}  // namespace hy

// y2 / g2 / w_y may be nullptr; h may be nullptr when emit == 0 (or for float activations reading the stream itself).
void launch_hy_add_rms_norm(const void* y, const void* y2, const float* g2, const float* w_y, float* x, const float* w_out,
                            void* h, int rows, int d, float eps, int emit, bool f32, hipStream_t s) {
    if (rows == 0) return;
    const bool vec = d % 4 == 0;
#define HY_ARN(T, VEC) hy::add_rms_norm_kernel<T, VEC><<<rows, 256, 0, s>>>((const T*)y, (const T*)y2, g2, w_y, x, w_out, (T*)h, d, eps, emit)
    if (f32) { if (vec) HY_ARN(float, true); else HY_ARN(float, false); }
    else { if (vec) HY_ARN(uint16_t, true); else HY_ARN(uint16_t, false); }
#undef HY_ARN
}

void launch_hy_token_gate(const void* a, const int32_t* ids, const void* table, int ldt, int col0, void* out, int T, int n,
                          bool f32, hipStream_t s) {
    const int64_t total = (int64_t)T * n;
    if (total == 0) return;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (f32) hy::token_gate_kernel<float><<<blocks, 256, 0, s>>>((const float*)a, ids, (const float*)table, ldt, col0, (float*)out, total, n);
    else hy::token_gate_kernel<uint16_t><<<blocks, 256, 0, s>>>((const uint16_t*)a, ids, (const uint16_t*)table, ldt, col0, (uint16_t*)out, total, n);
}

void launch_hy_ssm_prep(const float* dt_pre, const float* a_log, float* decay, float* dt, int T, int H, hipStream_t s) {
    const int64_t total = (int64_t)T * H;
    if (total == 0) return;
    hy::ssm_prep_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(dt_pre, a_log, decay, dt, total, H);
}

void launch_hy_gated_group_norm(const float* o, const void* xs, int ldx, int x_off, const float* skip, const void* zs,
                                int ldz, int z_off, const float* w, void* y, int T, int n, int groups, int Dv, float eps,
                                bool f32, hipStream_t s) {
    if (T == 0 || n == 0) return;
    const int gs = n / groups;
    const int nt = gs <= 512 ? 64 : 256;
    const unsigned blocks = (unsigned)((int64_t)T * groups);
    if (f32) hy::gated_group_norm_kernel<float><<<blocks, nt, 0, s>>>(o, (const float*)xs, ldx, x_off, skip, (const float*)zs, ldz, z_off, w, (float*)y, n, gs, Dv, eps);
    else hy::gated_group_norm_kernel<uint16_t><<<blocks, nt, 0, s>>>(o, (const uint16_t*)xs, ldx, x_off, skip, (const uint16_t*)zs, ldz, z_off, w, (uint16_t*)y, n, gs, Dv, eps);
}

int hy_rglru_chunks(int max_q) { return (max_q + hy::kLruChunk - 1) / hy::kLruChunk; }

// nch = hy_rglru_chunks(most tokens of any sequence); nch > 1: pq float [B, nch, 2, W] and init float [B, W] scratch.
void launch_hy_rglru_scan(const void* u, const float* gates, const float* sp, float c, const void* ys, int ldy, int y_off,
                          const int32_t* q_start, const int32_t* pos0, const int32_t* slots, float* S, float* pq,
                          float* init, void* out, int T, int B, int W, int bw, int nch, bool f32, hipStream_t s) {
    if (T == 0 || B == 0 || nch == 0) return;
    const dim3 grid(B, (W + 255) / 256, nch);
#define HY_LRU(T_, PH) hy::rglru_scan_kernel<T_, PH><<<grid, 256, 0, s>>>((const T_*)u, gates, sp, c, (const T_*)ys, ldy, y_off, q_start, pos0, slots, S, pq, init, (T_*)out, T, W, bw, nch)
    if (f32) { if (nch > 1) HY_LRU(float, 1); HY_LRU(float, 2); }
    else { if (nch > 1) HY_LRU(uint16_t, 1); HY_LRU(uint16_t, 2); }
#undef HY_LRU
}

}  // namespace chronos
