// Row-wise kernels around a fp32 residual stream for decoders with parallel sublayers and grouped
// norms: token row + sinusoidal position vector, RMS norm in groups, the fused residual update +
// next norm, the mean of several RMS-normalised branches added to the stream, unit-RMS q / k with
// the cache write, the routed gated activation, and the tanh soft cap.  One workgroup per token
// row unless noted; every reduction and every transcendental in fp32.
#include "hybrid_common.h"

using namespace hyb;

// x[t, 2i] = table[ids[t], 2i] + sin(p f_i);  x[t, 2i+1] = table[ids[t], 2i+1] + cos(p f_i)
template <typename T>
__global__ void embed_sinusoid_kernel(const int* __restrict__ ids, const int* __restrict__ positions,
                                      const T* __restrict__ table, const float* __restrict__ inv_freq,
                                      float* __restrict__ x, int W) {
    const long t = blockIdx.x;
    const T* a = table + (long)ids[t] * W;
    const float p = (float)positions[t];
    for (int i = threadIdx.x; i < W / 2; i += blockDim.x) {
        const float ang = p * inv_freq[i];
        float sn, cs;
        sincosf(ang, &sn, &cs);
        x[t * W + 2 * i] = ld(a + 2 * i) + sn;
        x[t * W + 2 * i + 1] = ld(a + 2 * i + 1) + cs;
    }
}

// x (+= y1 + y2);  h = x / rms_group(x) * w      (y1, y2, h optional)
template <typename T>
__global__ void residual_group_norm_kernel(float* __restrict__ x, const T* __restrict__ y1,
                                           long y1_stride, const T* __restrict__ y2, long y2_stride,
                                           const float* __restrict__ w, T* __restrict__ h, int W,
                                           int groups, float eps) {
    extern __shared__ float sm[];            // [groups] + 16
    float* gs = sm;
    float* red = sm + groups;
    const long t = blockIdx.x;
    float* xr = x + t * W;
    const int part = W / groups;
    for (int g = threadIdx.x; g < groups; g += blockDim.x) gs[g] = 0.f;
    // every group is a run of `part` columns; a thread's columns of one group are summed privately
    for (int g = 0; g < groups; ++g) {
        float s = 0.f;
        for (int c = g * part + threadIdx.x; c < (g + 1) * part; c += blockDim.x) {
            float v = xr[c];
            if (y1) v += ld(y1 + t * y1_stride + c);
            if (y2) v += ld(y2 + t * y2_stride + c);
            if (y1 || y2) xr[c] = v;
            s += v * v;
        }
        if (h) {
            const float tot = block_sum(s, red);
            if (threadIdx.x == 0) gs[g] = rsqrtf(tot / (float)part + eps);
        }
    }
    if (!h) return;
    __syncthreads();
    for (int c = threadIdx.x; c < W; c += blockDim.x)
        st(h + t * W + c, xr[c] * gs[c / part] * w[c]);
}

// x += (y1 / rms(y1) * w1 + y2 / rms(y2) * w2) / n     (y2 optional; rms over the whole row)
template <typename T>
__global__ void add_normed_mean_kernel(float* __restrict__ x, const T* __restrict__ y1,
                                       long y1_stride, const float* __restrict__ w1,
                                       const T* __restrict__ y2, long y2_stride,
                                       const float* __restrict__ w2, int W, float eps) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    float s1 = 0.f, s2 = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float a = ld(y1 + t * y1_stride + c);
        s1 += a * a;
        if (y2) { const float b = ld(y2 + t * y2_stride + c); s2 += b * b; }
    }
    const float r1 = rsqrtf(block_sum(s1, red) / (float)W + eps);
    const float r2 = y2 ? rsqrtf(block_sum(s2, red) / (float)W + eps) : 0.f;
    const float f = y2 ? 0.5f : 1.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float v = ld(y1 + t * y1_stride + c) * r1 * w1[c];
        if (y2) v += ld(y2 + t * y2_stride + c) * r2 * w2[c];
        x[t * W + c] += v * f;
    }
}

// Per token: every q head divided by its root mean square in place; the key row goes into the
// V cache as it is and, divided by its root mean square per head, into the K cache.  One wave per
// head (q heads first, then k heads); caches contiguous [slot, G, D].
template <typename T>
__global__ void unit_norm_store_kernel(T* __restrict__ q, const T* __restrict__ k, long row_stride,
                                       float eps, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                       const int* __restrict__ slot_mapping, int H, int G, int D) {
    const long t = blockIdx.x;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), nw = blockDim.x / kWave;
    const long slot = slot_mapping ? slot_mapping[t] : -1;
    for (int hd = wave; hd < H + G; hd += nw) {
        if (hd < H) {
            T* p = q + t * row_stride + (long)hd * D;
            float s = 0.f;
            for (int d = lane; d < D; d += kWave) { const float v = ld(p + d); s += v * v; }
            const float r = rsqrtf(wave_sum(s) / (float)D + eps);
            for (int d = lane; d < D; d += kWave) st(p + d, ld(p + d) * r);
        } else if (slot >= 0 && k_cache) {
            const int g = hd - H;
            const T* p = k + t * row_stride + (long)g * D;
            float s = 0.f;
            for (int d = lane; d < D; d += kWave) { const float v = ld(p + d); s += v * v; }
            const float r = rsqrtf(wave_sum(s) / (float)D + eps);
            T* kc = k_cache + (slot * G + g) * (long)D;
            T* vc = v_cache + (slot * G + g) * (long)D;
            for (int d = lane; d < D; d += kWave) {
                const float v = ld(p + d);
                st(kc + d, v * r);
                st(vc + d, v);
            }
        }
    }
}

// gu row = [gate columns C | up columns C], C = NE * ff + sff.  act[t, c] = silu(w g) * (w u) with
// w = dense[t, c / ff] for routed columns, 1 for the shared ones; exactly zero where w is (those
// columns' inputs are not even read).  VEC consecutive columns per thread (one expert lookup per
// run; VEC divides ff, sff and the row strides).
template <typename T, int VEC>
__global__ void swiglu_route_scale_kernel(const T* __restrict__ gu, long gu_stride,
                                          const float* __restrict__ dense, T* __restrict__ act,
                                          int NE, int ff, int C) {
    const long t = blockIdx.y;
    const T* g = gu + t * gu_stride;
    const T* u = g + C;
    const int routed = NE * ff;
    for (int c = (blockIdx.x * blockDim.x + threadIdx.x) * VEC; c < C; c += gridDim.x * blockDim.x * VEC) {
        const float w = (dense && c < routed) ? dense[t * NE + c / ff] : 1.f;
        float gv[VEC], uv[VEC];
        if (w != 0.f) {
            if constexpr (VEC == 1) { gv[0] = ld(g + c); uv[0] = ld(u + c); }
            else { load_run<T, VEC>(g + c, gv); load_run<T, VEC>(u + c, uv); }
#pragma unroll
            for (int j = 0; j < VEC; ++j) gv[j] = siluf_(gv[j] * w) * (uv[j] * w);
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) gv[j] = 0.f;
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) st(act + t * (long)C + c + j, gv[j]);
    }
}

template <typename T>
__global__ void tanh_cap_kernel(T* __restrict__ z, long n, float cap) {
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        st(z + i, cap * tanhf(ld(z + i) / cap));
}

static inline int threads_for(int n) { return n >= 1024 ? 512 : n >= 256 ? 256 : n > 64 ? 128 : 64; }

extern "C" {

int hyb_embed_sinusoid(const void* ids, const void* positions, const void* table,
                       const void* inv_freq, void* x, long T_, int W, int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    if (W & 1) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(embed_sinusoid_kernel<T>, dim3(T_), dim3(threads_for(W / 2)),
                                        0, s, (const int*)ids, (const int*)positions, (const T*)table,
                                        (const float*)inv_freq, (float*)x, W));
    return HYB_LAUNCH_OK();
}

// x [T, W] fp32 (updated in place when y1 / y2 are given); h [T, W] of the activation type, or null
int hyb_residual_group_norm(void* x, const void* y1, long y1_stride, const void* y2, long y2_stride,
                            const void* w, void* h, long T_, int W, int groups, float eps, int dt,
                            hipStream_t s) {
    if (T_ <= 0) return 0;
    if (groups < 1 || W % groups || groups > 1024 || (h && !w)) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(residual_group_norm_kernel<T>, dim3(T_),
                                        dim3(threads_for(W / groups)), (groups + 16) * sizeof(float), s,
                                        (float*)x, (const T*)y1, y1_stride, (const T*)y2, y2_stride,
                                        (const float*)w, (T*)h, W, groups, eps));
    return HYB_LAUNCH_OK();
}

int hyb_add_normed_mean(void* x, const void* y1, long y1_stride, const void* w1, const void* y2,
                        long y2_stride, const void* w2, long T_, int W, float eps, int dt,
                        hipStream_t s) {
    if (T_ <= 0) return 0;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(add_normed_mean_kernel<T>, dim3(T_), dim3(threads_for(W)), 0, s,
                                        (float*)x, (const T*)y1, y1_stride, (const float*)w1,
                                        (const T*)y2, y2_stride, (const float*)w2, W, eps));
    return HYB_LAUNCH_OK();
}

int hyb_unit_norm_store(void* q, const void* k, long row_stride, float eps, void* k_cache,
                        void* v_cache, const void* slot_mapping, long T_, int H, int G, int D, int dt,
                        hipStream_t s) {
    if (T_ <= 0) return 0;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(unit_norm_store_kernel<T>, dim3(T_), dim3(256), 0, s, (T*)q,
                                        (const T*)k, row_stride, eps, (T*)k_cache, (T*)v_cache,
                                        (const int*)slot_mapping, H, G, D));
    return HYB_LAUNCH_OK();
}

int hyb_swiglu_route_scale(const void* gu, long gu_stride, const void* dense, void* act, long T_,
                           int NE, int ff, int sff, int dt, hipStream_t s) {
    const int C = NE * ff + sff;
    if (T_ <= 0 || C <= 0) return 0;
    const int esize = dt == 0 ? 2 : 4;
    // eight columns per thread when every run of eight is one expert's and 16-byte addressable
    const bool vec = (NE == 0 || ff % 8 == 0) && sff % 8 == 0 && gu_stride % 8 == 0 &&
                     (size_t)gu % (4 * esize) == 0 && (C * (size_t)esize) % (4 * esize) == 0;
    const int per = vec ? 8 : 1;
    const int need = (C / per + 255) / 256;
    const int bx = need > 64 ? 64 : (need < 1 ? 1 : need);
    for (long t0 = 0; t0 < T_; t0 += 65535) {          // blockIdx.y holds at most 65535 rows
        const long n = T_ - t0 < 65535 ? T_ - t0 : 65535;
#define SWI(VEC)                                                                                  \
        HYB_DISPATCH(dt, hipLaunchKernelGGL((swiglu_route_scale_kernel<T, VEC>), dim3(bx, n),      \
                                            dim3(256), 0, s, (const T*)gu + t0 * gu_stride,       \
                                            gu_stride,                                            \
                                            dense ? (const float*)dense + t0 * NE : nullptr,      \
                                            (T*)act + t0 * (long)C, NE, ff, C))
        if (vec) SWI(8); else SWI(1);
#undef SWI
    }
    return HYB_LAUNCH_OK();
}

int hyb_tanh_cap(void* z, long n, float cap, int dt, hipStream_t s) {
    if (n <= 0) return 0;
    const int blocks = (int)((n + 255) / 256 > 8192 ? 8192 : (n + 255) / 256);
    HYB_DISPATCH(dt, hipLaunchKernelGGL(tanh_cap_kernel<T>, dim3(blocks), dim3(256), 0, s, (T*)z, n, cap));
    return HYB_LAUNCH_OK();
}

}  // extern "C"
