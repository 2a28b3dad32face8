// sandwich.hip — the float32 residual stream of sandwich-norm hybrid decoders (a norm before AND after every
// sublayer, each an RMS norm over equal parts of the row), and the rotations of the retention and rotated-value
// attention mixers.
//
//   sandwich_join   one workgroup per row:
//                       v = y (+ y2)                                              the sublayer's output(s), or
//                       v = (y / rms(y) * w_a + y2 / rms(y2) * w_b) / 2           two mixers side by side;
//                       v <- v / rms_g(v) * w_y     per group g of d / groups consecutive columns;
//                       x <- x + v                  float, in place;
//                       h  = x / rms_g(x) * w_out   what the next sublayer reads, in the activation type.
//                   Without y the kernel is the plain grouped norm of x.  rms(.) = sqrt(mean(.^2) + eps).  All
//                   arithmetic in float.  Rows up to 4096 wide whose groups are multiples of 4 columns are read once
//                   (16-byte accesses, values kept in registers between the statistics and the write passes): up to
//                   1024 columns a wave owns a row (no barrier), above that a workgroup does, with a group's sum
//                   formed per wave for every group in turn and added up over the waves in a fixed order.  A row's
//                   result does not depend on anything else in the launch.
//   rotate_qk       in place on a projection's rows: the first `dims` columns of every query and key head turn by the
//                   token's position (column i pairs with i + dims / 2), then the head is multiplied by q_mul / k_mul.
//   unrotate_gate   every head's output row turns BACK by the token's position over all its columns, then is
//                   multiplied element by element with sigmoid of a gate read from the projection's columns.
#include "hybrid_common.h"

namespace chronos {
namespace hy {

constexpr int kSwMaxGroups = 16;   // of the register paths; more groups take the per-wave kernel

template <typename T> __device__ __forceinline__ f32x4 sw_ld4(const T* p);
template <> __device__ __forceinline__ f32x4 sw_ld4<float>(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
template <> __device__ __forceinline__ f32x4 sw_ld4<uint16_t>(const uint16_t* p) {
    const u16x4 v = *reinterpret_cast<const u16x4*>(p);
    return f32x4{bf2f(v[0]), bf2f(v[1]), bf2f(v[2]), bf2f(v[3])};
}
template <typename T> __device__ __forceinline__ void sw_st4(T* p, const f32x4& v);
template <> __device__ __forceinline__ void sw_st4<float>(float* p, const f32x4& v) { *reinterpret_cast<f32x4*>(p) = v; }
template <> __device__ __forceinline__ void sw_st4<uint16_t>(uint16_t* p, const f32x4& v) {
    *reinterpret_cast<u16x4*>(p) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
}
__device__ __forceinline__ float sw_sq(const f32x4& v) { return v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3]; }

// Sums of squares per group over the whole workgroup: ss[j] belongs to the thread's j-th chunk (group gidx[j], or -1
// for no chunk).  Returns nothing; afterwards sw_total(red, g) is group g's total for every thread (the four waves'
// partials added in a fixed order).  One barrier: every reduction of a kernel has a scratch area of its own (`red`
// points at 4 * kSwMaxGroups floats), so a call never overwrites what a slower wave still reads from the call before.
template <int NJ>
__device__ __forceinline__ void sw_group_sums(const float (&ss)[NJ], const int (&gidx)[NJ], int groups, float* red) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int g = 0; g < groups; ++g) {
        float v = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) v += gidx[j] == g ? ss[j] : 0.f;
        v = wave_sum(v);
        if (lane == 0) red[wv * kSwMaxGroups + g] = v;
    }
    __syncthreads();
}
__device__ __forceinline__ float sw_total(const float* red, int g) {
    return (red[g] + red[kSwMaxGroups + g]) + (red[2 * kSwMaxGroups + g] + red[3 * kSwMaxGroups + g]);
}

// VEC: d <= 4096, d / groups % 4 == 0: every thread owns up to 4 chunks of 4 columns, read once.
// TY: the sublayer outputs' type; TH: the emitted type.
template <typename TY, typename TH>
__global__ void __launch_bounds__(256) sandwich_join_vec_kernel(const TY* __restrict__ y, const TY* __restrict__ y2,
                                                                float* __restrict__ x, const float* __restrict__ w_y,
                                                                const float* __restrict__ w_out,
                                                                const float* __restrict__ w_a, const float* __restrict__ w_b,
                                                                TH* __restrict__ h, int d, int groups, float eps) {
    __shared__ float red3[3][4 * kSwMaxGroups];   // one scratch area per reduction of the kernel
    const int64_t row = blockIdx.x;
    const int gsz = d / groups;
    float* xr = x + row * d;
    int gidx[4];
    f32x4 v[4];
    float ss[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = (threadIdx.x + 256 * j) * 4;
        gidx[j] = i < d ? i / gsz : -1;
        v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const float inv_g = 1.f / (float)gsz;
    if (y != nullptr) {
        const TY* yr = y + row * d;
        if (w_a != nullptr) {   // two outputs, each normed over the whole row, averaged
            const TY* y2r = y2 + row * d;
            f32x4 u[4];
            float sa = 0.f, sb = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = (threadIdx.x + 256 * j) * 4;
                u[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (i < d) {
                    v[j] = sw_ld4<TY>(yr + i);
                    u[j] = sw_ld4<TY>(y2r + i);
                    sa += sw_sq(v[j]);
                    sb += sw_sq(u[j]);
                }
            }
            {
                const float s2[2] = {sa, sb};
                const int g2[2] = {0, 1};
                sw_group_sums<2>(s2, g2, 2, red3[0]);
            }
            const float ra = 0.5f / sqrtf(sw_total(red3[0], 0) / (float)d + eps);
            const float rb = 0.5f / sqrtf(sw_total(red3[0], 1) / (float)d + eps);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = (threadIdx.x + 256 * j) * 4;
                if (i < d) v[j] = v[j] * ra * *reinterpret_cast<const f32x4*>(w_a + i) + u[j] * rb * *reinterpret_cast<const f32x4*>(w_b + i);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = (threadIdx.x + 256 * j) * 4;
                if (i < d) {
                    v[j] = sw_ld4<TY>(yr + i);
                    if (y2 != nullptr) v[j] = v[j] + sw_ld4<TY>(y2 + row * d + i);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) ss[j] = sw_sq(v[j]);
        sw_group_sums<4>(ss, gidx, groups, red3[1]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = (threadIdx.x + 256 * j) * 4;
            if (i < d) {
                const float r = 1.f / sqrtf(sw_total(red3[1], gidx[j]) * inv_g + eps);
                v[j] = v[j] * r * *reinterpret_cast<const f32x4*>(w_y + i) + *reinterpret_cast<const f32x4*>(xr + i);
                *reinterpret_cast<f32x4*>(xr + i) = v[j];
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = (threadIdx.x + 256 * j) * 4;
            if (i < d) v[j] = *reinterpret_cast<const f32x4*>(xr + i);
        }
    }
    if (h == nullptr) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) ss[j] = sw_sq(v[j]);
    sw_group_sums<4>(ss, gidx, groups, red3[2]);
    TH* hr = h + row * d;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = (threadIdx.x + 256 * j) * 4;
        if (i < d) {
            const float r = 1.f / sqrtf(sw_total(red3[2], gidx[j]) * inv_g + eps);
            sw_st4<TH>(hr + i, v[j] * r * *reinterpret_cast<const f32x4*>(w_out + i));
        }
    }
}

// Rows up to 1024 wide (d / groups % 4 == 0): a wave owns a row — NJ chunks of 4 columns per lane, read once — so the
// group sums are wave reductions and the kernel has no barrier at all; a workgroup takes 4 rows.
template <typename TY, typename TH, int NJ>
__global__ void __launch_bounds__(256) sandwich_join_wave_kernel(const TY* __restrict__ y, const TY* __restrict__ y2,
                                                                 float* __restrict__ x, const float* __restrict__ w_y,
                                                                 const float* __restrict__ w_out,
                                                                 const float* __restrict__ w_a, const float* __restrict__ w_b,
                                                                 TH* __restrict__ h, int rows, int d, int groups, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int gsz = d / groups;
    const float inv_g = 1.f / (float)gsz;
    float* xr = x + row * d;
    int gidx[NJ];
    f32x4 v[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int i = (lane + 64 * j) * 4;
        gidx[j] = i < d ? i / gsz : -1;
        v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // rs[j] <- 1 / rms of chunk j's group, from the chunks' sums of squares
    auto group_scales = [&](float (&rs)[NJ]) {
        float ss[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            ss[j] = sw_sq(v[j]);
            rs[j] = 0.f;
        }
        for (int g = 0; g < groups; ++g) {
            float t = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j) t += gidx[j] == g ? ss[j] : 0.f;
            const float r = 1.f / sqrtf(wave_sum(t) * inv_g + eps);
#pragma unroll
            for (int j = 0; j < NJ; ++j) rs[j] = gidx[j] == g ? r : rs[j];
        }
    };
    float rs[NJ];
    if (y != nullptr) {
        const TY* yr = y + row * d;
        if (w_a != nullptr) {
            const TY* y2r = y2 + row * d;
            f32x4 u[NJ];
            float sa = 0.f, sb = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int i = (lane + 64 * j) * 4;
                u[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (i < d) {
                    v[j] = sw_ld4<TY>(yr + i);
                    u[j] = sw_ld4<TY>(y2r + i);
                    sa += sw_sq(v[j]);
                    sb += sw_sq(u[j]);
                }
            }
            const float ra = 0.5f / sqrtf(wave_sum(sa) / (float)d + eps), rb = 0.5f / sqrtf(wave_sum(sb) / (float)d + eps);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int i = (lane + 64 * j) * 4;
                if (i < d) v[j] = v[j] * ra * *reinterpret_cast<const f32x4*>(w_a + i) + u[j] * rb * *reinterpret_cast<const f32x4*>(w_b + i);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int i = (lane + 64 * j) * 4;
                if (i < d) {
                    v[j] = sw_ld4<TY>(yr + i);
                    if (y2 != nullptr) v[j] = v[j] + sw_ld4<TY>(y2 + row * d + i);
                }
            }
        }
        group_scales(rs);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int i = (lane + 64 * j) * 4;
            if (i < d) {
                v[j] = v[j] * rs[j] * *reinterpret_cast<const f32x4*>(w_y + i) + *reinterpret_cast<const f32x4*>(xr + i);
                *reinterpret_cast<f32x4*>(xr + i) = v[j];
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int i = (lane + 64 * j) * 4;
            if (i < d) v[j] = *reinterpret_cast<const f32x4*>(xr + i);
        }
    }
    if (h == nullptr) return;
    group_scales(rs);
    TH* hr = h + row * d;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int i = (lane + 64 * j) * 4;
        if (i < d) sw_st4<TH>(hr + i, v[j] * rs[j] * *reinterpret_cast<const f32x4*>(w_out + i));
    }
}

// Any width and group size: a wave takes whole groups (group g goes to wave g % 4) and walks each three times.
template <typename TY, typename TH>
__global__ void __launch_bounds__(256) sandwich_join_any_kernel(const TY* __restrict__ y, const TY* __restrict__ y2,
                                                                float* __restrict__ x, const float* __restrict__ w_y,
                                                                const float* __restrict__ w_out,
                                                                const float* __restrict__ w_a, const float* __restrict__ w_b,
                                                                TH* __restrict__ h, int d, int groups, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    const int gsz = d / groups;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    float* xr = x + row * d;
    float ra = 0.f, rb = 0.f;
    if (y != nullptr && w_a != nullptr) {
        float sa = 0.f, sb = 0.f;
        for (int i = threadIdx.x; i < d; i += 256) {
            const float a = ld<TY>(y + row * d + i), b = ld<TY>(y2 + row * d + i);
            sa += a * a;
            sb += b * b;
        }
        ra = 0.5f / sqrtf(block_sum(sa, red) / (float)d + eps);
        rb = 0.5f / sqrtf(block_sum(sb, red) / (float)d + eps);
    }
    auto val = [&](int i) {
        float v = ld<TY>(y + row * d + i);
        if (w_a != nullptr) v = v * ra * w_a[i] + ld<TY>(y2 + row * d + i) * rb * w_b[i];
        else if (y2 != nullptr) v += ld<TY>(y2 + row * d + i);
        return v;
    };
    for (int g = wv; g < groups; g += 4) {
        const int c0 = g * gsz;
        if (y != nullptr) {
            float ss = 0.f;
            for (int i = lane; i < gsz; i += 64) {
                const float v = val(c0 + i);
                ss += v * v;
            }
            const float r = 1.f / sqrtf(wave_sum(ss) / (float)gsz + eps);
            for (int i = lane; i < gsz; i += 64) xr[c0 + i] += val(c0 + i) * r * w_y[c0 + i];
        }
        if (h == nullptr) continue;
        float ss = 0.f;
        for (int i = lane; i < gsz; i += 64) {   // (a lane re-reads what it wrote itself)
            const float v = xr[c0 + i];
            ss += v * v;
        }
        const float r = 1.f / sqrtf(wave_sum(ss) / (float)gsz + eps);
        for (int i = lane; i < gsz; i += 64) st<TH>(h + row * d + c0 + i, xr[c0 + i] * r * w_out[c0 + i]);
    }
}

// one workgroup per token; thread = (head, pair) of the query heads, then of the key heads
template <typename T>
__global__ void __launch_bounds__(256) rotate_qk_kernel(T* __restrict__ proj, int ldp, int q_off, int k_off, int HQ, int HK,
                                                        int D, int dims, const float* __restrict__ cos_sin,
                                                        const int32_t* __restrict__ pos, float q_mul, float k_mul) {
    const int64_t t = blockIdx.x;
    const int half = dims / 2;
    const float* cs = cos_sin != nullptr ? cos_sin + (int64_t)pos[t] * dims : nullptr;
    T* row = proj + t * ldp;
    const int per = D - half;   // work items of a head: `half` pairs, then the D - dims columns that only scale
    for (int it = threadIdx.x; it < (HQ + HK) * per; it += 256) {
        const int hd = it / per, i = it % per;
        const float mul = hd < HQ ? q_mul : k_mul;
        T* p = row + (hd < HQ ? q_off + hd * D : k_off + (hd - HQ) * D);
        if (i < half) {
            const float u = ld<T>(p + i), v = ld<T>(p + i + half), c = cs[i], s = cs[half + i];
            st<T>(p + i, (u * c - v * s) * mul);
            st<T>(p + i + half, (v * c + u * s) * mul);
        } else if (mul != 1.f) {
            st<T>(p + i + half, ld<T>(p + i + half) * mul);
        }
    }
}

// one workgroup per token; thread = (head, pair m of Dv / 2).  out may be o itself: a thread reads the two values it
// writes before it writes them.
template <typename T>
__global__ void __launch_bounds__(256) unrotate_gate_kernel(const T* o, const int32_t* __restrict__ pos,
                                                            const float* __restrict__ cos_sin, const T* __restrict__ gsrc,
                                                            int ldg, int g_off, T* out, int H, int Dv) {
    const int64_t t = blockIdx.x;
    const int half = Dv / 2;
    const float* cs = cos_sin != nullptr ? cos_sin + (int64_t)pos[t] * Dv : nullptr;
    const T* orow = o + t * H * Dv;
    const T* grow = gsrc != nullptr ? gsrc + t * ldg + g_off : nullptr;
    T* dst = out + t * H * Dv;
    if (cs == nullptr) {
        for (int i = threadIdx.x; i < H * Dv; i += 256) st<T>(dst + i, ld<T>(orow + i) * sigmoidf_(ld<T>(grow + i)));
        return;
    }
    for (int it = threadIdx.x; it < H * half; it += 256) {
        const int hd = it / half, m = it % half;
        const int a = hd * Dv + m, b = a + half;
        const float u = ld<T>(orow + a), v = ld<T>(orow + b), c = cs[m], s = cs[half + m];
        float ra = u * c + v * s, rb = v * c - u * s;
        if (grow != nullptr) {
            ra *= sigmoidf_(ld<T>(grow + a));
            rb *= sigmoidf_(ld<T>(grow + b));
        }
        st<T>(dst + a, ra);
        st<T>(dst + b, rb);
    }
}

}  // namespace hy

bool hy_sandwich_groups_ok(int d, int groups) { return groups >= 1 && d % groups == 0; }

// y == nullptr: the plain grouped norm of x (x untouched).  h == nullptr: nothing is emitted.  y_f32: y and y2 are
// float (else bfloat16); out_f32: h is float (else bfloat16).  w_a != nullptr: the pair form (y2 and w_b given).
void launch_hy_sandwich_join(const void* y, const void* y2, float* x, const float* w_y, const float* w_out,
                             const float* w_a, const float* w_b, void* h, int rows, int d, int groups, float eps,
                             bool y_f32, bool out_f32, hipStream_t s) {
    if (rows == 0) return;
    const bool vec = d <= 4096 && (d / groups) % 4 == 0 && groups <= hy::kSwMaxGroups;
    const int wg4 = (rows + 3) / 4;
#define HY_SW(TY, TH)                                                                                                      \
    do {                                                                                                                   \
        if (vec && d <= 1024) hy::sandwich_join_wave_kernel<TY, TH, 4><<<wg4, 256, 0, s>>>((const TY*)y, (const TY*)y2, x, w_y, w_out, w_a, w_b, (TH*)h, rows, d, groups, eps); \
        else if (vec) hy::sandwich_join_vec_kernel<TY, TH><<<rows, 256, 0, s>>>((const TY*)y, (const TY*)y2, x, w_y, w_out, w_a, w_b, (TH*)h, d, groups, eps); \
        else hy::sandwich_join_any_kernel<TY, TH><<<rows, 256, 0, s>>>((const TY*)y, (const TY*)y2, x, w_y, w_out, w_a, w_b, (TH*)h, d, groups, eps); \
    } while (0)
    if (y_f32 && out_f32) HY_SW(float, float);
    else if (y_f32) HY_SW(float, uint16_t);
    else if (out_f32) HY_SW(uint16_t, float);
    else HY_SW(uint16_t, uint16_t);
#undef HY_SW
}

void launch_hy_rotate_qk(void* proj, int ldp, int q_off, int k_off, int HQ, int HK, int D, int dims, const float* cos_sin,
                         const int32_t* pos, float q_mul, float k_mul, int T, bool f32, hipStream_t s) {
    if (T == 0) return;
    if (f32) hy::rotate_qk_kernel<float><<<T, 256, 0, s>>>((float*)proj, ldp, q_off, k_off, HQ, HK, D, dims, cos_sin, pos, q_mul, k_mul);
    else hy::rotate_qk_kernel<uint16_t><<<T, 256, 0, s>>>((uint16_t*)proj, ldp, q_off, k_off, HQ, HK, D, dims, cos_sin, pos, q_mul, k_mul);
}

void launch_hy_unrotate_gate(const void* o, const int32_t* pos, const float* cos_sin, const void* gsrc, int ldg, int g_off,
                             void* out, int T, int H, int Dv, bool f32, hipStream_t s) {
    if (T == 0) return;
    if (f32) hy::unrotate_gate_kernel<float><<<T, 256, 0, s>>>((const float*)o, pos, cos_sin, (const float*)gsrc, ldg, g_off, (float*)out, H, Dv);
    else hy::unrotate_gate_kernel<uint16_t><<<T, 256, 0, s>>>((const uint16_t*)o, pos, cos_sin, (const uint16_t*)gsrc, ldg, g_off, (uint16_t*)out, H, Dv);
}

}  // namespace chronos
