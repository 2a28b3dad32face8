// hybrid_elementwise.hip — the float32 residual stream of the hybrid decoders: embedding rows, layer norm (weight, no
// bias) with the residual add fused, the few-row float32-output projections, activations.
//
// The sublayers' outputs are normalised and ADDED to the stream (x <- x + norm(y)), so the norm kernel reads the
// sublayer output in the activation type, does all its arithmetic in float, updates the float stream in place and
// emits the stream's copy in the activation type for the next sublayer's GEMMs (one pass, nothing re-read from HBM).
#include "hybrid_common.h"

namespace chronos {
namespace hy {

template <typename T>
__global__ void __launch_bounds__(256) embed_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                                                    float* __restrict__ x, int d, float scale) {
    const int64_t t = blockIdx.x;
    const T* src = table + (int64_t)ids[t] * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) x[t * d + i] = ld<T>(src + i) * scale;
}

__global__ void __launch_bounds__(256) cast_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y, int64_t n) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 3 < n) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(x + i);
        *reinterpret_cast<u16x4*>(y + i) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
    } else {
        for (int64_t j = i; j < n; ++j) y[j] = f2bf(x[j]);
    }
}

// y [rows, d] (activation type, or float for the plain norm of the stream itself) -> float statistics in two passes
// (mean, then the mean of squared deviations), then
//   ADD:   x[row] += (y - mean) * rstd * w;   h[row] = T(x[row])   (h == nullptr: not written)
//   plain: h[row] = T((y - mean) * rstd * w)
template <typename TY, typename TH, bool ADD>
__global__ void __launch_bounds__(256) layer_norm_kernel(const TY* __restrict__ y, float* __restrict__ x,
                                                         const float* __restrict__ w, TH* __restrict__ h, int d,
                                                         float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    const TY* yr = y + row * d;
    float s = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) s += ld<TY>(yr + i);
    const float mean = block_sum(s, red) / (float)d;
    float q = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) {
        const float c = ld<TY>(yr + i) - mean;
        q += c * c;
    }
    const float rstd = 1.f / sqrtf(block_sum(q, red) / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += 256) {
        float v = (ld<TY>(yr + i) - mean) * rstd * w[i];
        if constexpr (ADD) {
            v += x[row * d + i];
            x[row * d + i] = v;
        }
        if (h != nullptr) st<TH>(h + row * d + i, v);
    }
}

// out[t, n] = sum_k h[t, k] * w[n, k] (+ bias[n]) in float.  A workgroup takes TB tokens (their rows sit in LDS) and
// 4 output rows, one per wave: a weight row is read ONCE for all TB tokens, 16 bytes per lane when the row length
// allows (VEC), and the grid's second axis spreads the output rows over workgroups so a handful of decode rows still
// fills many CUs.
template <typename T> struct Vec16 { static constexpr int E = 16 / (int)sizeof(T); };
template <typename T> __device__ __forceinline__ void unpack16(const uint4& v, float* f);
template <> __device__ __forceinline__ void unpack16<uint16_t>(const uint4& v, float* f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float(w[i] << 16);
        f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
template <> __device__ __forceinline__ void unpack16<float>(const uint4& v, float* f) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
}

template <typename T, int TB, bool VEC>
__global__ void __launch_bounds__(256) rowdot_kernel(const T* __restrict__ h, const T* __restrict__ w,
                                                     const float* __restrict__ bias, float* __restrict__ out, int rows,
                                                     int d, int n) {
    extern __shared__ __attribute__((aligned(16))) unsigned char rd_smem[];
    T* hs = reinterpret_cast<T*>(rd_smem);
    constexpr int E = Vec16<T>::E;
    const int64_t t0 = (int64_t)blockIdx.x * TB;
    const int nt = (int)min((int64_t)TB, rows - t0);
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if constexpr (VEC) {
        const uint4* src = reinterpret_cast<const uint4*>(h + t0 * d);
        for (int i = threadIdx.x; i < nt * d / E; i += 256) reinterpret_cast<uint4*>(hs)[i] = src[i];
    } else {
        for (int i = threadIdx.x; i < nt * d; i += 256) hs[i] = h[t0 * d + i];
    }
    __syncthreads();
    const int r = blockIdx.y * 4 + wv;
    if (r >= n) return;
    const T* wr = w + (int64_t)r * d;
    float acc[TB];
#pragma unroll
    for (int u = 0; u < TB; ++u) acc[u] = 0.f;
    if constexpr (VEC) {
        for (int k = lane * E; k < d; k += 64 * E) {
            float wf[E];
            unpack16<T>(*reinterpret_cast<const uint4*>(wr + k), wf);
#pragma unroll
            for (int u = 0; u < TB; ++u)
                if (u < nt) {
                    float hf[E];
                    unpack16<T>(*reinterpret_cast<const uint4*>(hs + u * d + k), hf);
#pragma unroll
                    for (int i = 0; i < E; ++i) acc[u] += hf[i] * wf[i];
                }
        }
    } else {
        for (int k = lane; k < d; k += 64) {
            const float wk = ld<T>(wr + k);
#pragma unroll
            for (int u = 0; u < TB; ++u)
                if (u < nt) acc[u] += ld<T>(hs + u * d + k) * wk;
        }
    }
#pragma unroll
    for (int u = 0; u < TB; ++u) {
        const float v = wave_sum(acc[u]);
        if (lane == 0 && u < nt) out[(t0 + u) * n + r] = v + (bias != nullptr ? bias[r] : 0.f);
    }
}

template <typename T>
__global__ void __launch_bounds__(256) act_kernel(T* __restrict__ x, int64_t n, int kind) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) st<T>(x + i, act_apply(ld<T>(x + i), kind));
}

}  // namespace hy

void launch_hy_embed(const int32_t* ids, const void* table, float* x, int T, int d, float scale, bool f32, hipStream_t s) {
    if (T == 0) return;
    if (f32) hy::embed_kernel<float><<<T, 256, 0, s>>>(ids, (const float*)table, x, d, scale);
    else hy::embed_kernel<uint16_t><<<T, 256, 0, s>>>(ids, (const uint16_t*)table, x, d, scale);
}
void launch_hy_cast_bf16(const float* x, uint16_t* y, int64_t n, hipStream_t s) {
    if (n == 0) return;
    const int64_t blocks = (n + 1023) / 1024;
    hy::cast_bf16_kernel<<<(unsigned)blocks, 256, 0, s>>>(x, y, n);
}
// y_f32: the input is float (the plain norm of the stream); out_f32: h is float.  x == nullptr: plain norm.
void launch_hy_layer_norm(const void* y, bool y_f32, float* x, const float* w, void* h, bool out_f32, int rows, int d,
                          float eps, hipStream_t s) {
    if (rows == 0) return;
    if (x != nullptr) {
        if (y_f32) hy::layer_norm_kernel<float, float, true><<<rows, 256, 0, s>>>((const float*)y, x, w, (float*)h, d, eps);
        else hy::layer_norm_kernel<uint16_t, uint16_t, true><<<rows, 256, 0, s>>>((const uint16_t*)y, x, w, (uint16_t*)h, d, eps);
    } else {
        if (out_f32) hy::layer_norm_kernel<float, float, false><<<rows, 256, 0, s>>>((const float*)y, nullptr, w, (float*)h, d, eps);
        else hy::layer_norm_kernel<float, uint16_t, false><<<rows, 256, 0, s>>>((const float*)y, nullptr, w, (uint16_t*)h, d, eps);
    }
}
template <typename T>
static void rowdot_t(const T* h, const T* w, const float* bias, float* out, int rows, int d, int n, hipStream_t s) {
    // tokens per workgroup: as many (up to 8) as keep the staged rows within 48 KB
    const int fit = (48 * 1024) / (d * (int)sizeof(T));
    const bool vec = d % hy::Vec16<T>::E == 0;
    const int ny = (n + 3) / 4;
#define HY_RD(TB)                                                                                                  \
    do {                                                                                                           \
        const dim3 grid((rows + TB - 1) / TB, ny);                                                                 \
        if (vec) hy::rowdot_kernel<T, TB, true><<<grid, 256, TB * d * sizeof(T), s>>>(h, w, bias, out, rows, d, n); \
        else hy::rowdot_kernel<T, TB, false><<<grid, 256, TB * d * sizeof(T), s>>>(h, w, bias, out, rows, d, n);    \
    } while (0)
    if (fit >= 8 && rows >= 8) HY_RD(8);
    else if (fit >= 4 && rows >= 4) HY_RD(4);
    else if (fit >= 2 && rows >= 2) HY_RD(2);
    else {
        auto kern = hy::rowdot_kernel<T, 1, false>;
        const int bytes = d * (int)sizeof(T);
        if (bytes > 48 * 1024)
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        kern<<<dim3(rows, ny), 256, bytes, s>>>(h, w, bias, out, rows, d, n);
    }
#undef HY_RD
}

void launch_hy_rowdot(const void* h, const void* w, const float* bias, float* out, int T, int d, int n, bool f32,
                      hipStream_t s) {
    if (T == 0 || n == 0) return;
    if (f32) rowdot_t<float>((const float*)h, (const float*)w, bias, out, T, d, n, s);
    else rowdot_t<uint16_t>((const uint16_t*)h, (const uint16_t*)w, bias, out, T, d, n, s);
}
void launch_hy_act(void* x, int64_t n, int kind, bool f32, hipStream_t s) {
    if (n == 0) return;
    const int64_t blocks = (n + 255) / 256;
    if (f32) hy::act_kernel<float><<<(unsigned)blocks, 256, 0, s>>>((float*)x, n, kind);
    else hy::act_kernel<uint16_t><<<(unsigned)blocks, 256, 0, s>>>((uint16_t*)x, n, kind);
}

}  // namespace chronos
