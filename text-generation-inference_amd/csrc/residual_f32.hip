// Kernels around an fp32 residual stream: scaled embedding lookup, the "sandwich" RMS norm (norm after a sublayer, add,
// norm before the next one, in one launch) and gated-unit activations with optional clamping.
//
// Models that keep their residual stream in the model dtype use norm.hip; a design that asks for a 32-bit residual sum and
// norms on both sides of every sublayer uses these.  Activations handed to / taken from the matrix products are T = bf16,
// f16 or float; statistics, gains and the residual itself are always float.
#include <type_traits>
#include "common.h"

namespace {

template <typename T> struct Elem;
template <> struct Elem<f16> { static __device__ __forceinline__ float ld(const f16* p) { return (float)*p; } };
template <> struct Elem<bf16> { static __device__ __forceinline__ float ld(const bf16* p) { return (float)*p; } };
template <> struct Elem<float> { static __device__ __forceinline__ float ld(const float* p) { return *p; } };
template <typename T> __device__ __forceinline__ T cvt_out(float v) { return (T)v; }

__device__ __forceinline__ float block_sum(float v, float* red) {
    // every thread of the block calls this; red holds one float per wave (<= 16)
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();  // red may still be read from a previous call
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    return s;
}

template <typename T>
__global__ void embedding_scaled_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out,
                                        int64_t E, int64_t vocab, float scale) {
    const int64_t t = blockIdx.x;
    const int64_t id = ids[t];
    const bool ok = id >= 0 && id < vocab;
    for (int64_t c = threadIdx.x; c < E; c += blockDim.x)
        out[t * E + c] = ok ? Elem<T>::ld(table + id * E + c) * scale : 0.f;
}

// One workgroup per row.
//   delta and post_w:     x_out = x + post_scale * delta / sqrt(mean(delta^2) + eps) * (post_w + post_add)
//   delta, post_w null:   x_out = x + post_scale * delta                     (a pre-norm design's plain residual sum)
//   pre_w != null:        y = x_out / sqrt(mean(x_out^2) + eps) * (pre_w + pre_add)
//   pre_w null, y given:  y = x_out rounded to TY                             (an operand for a projection of x itself)
// x_out may alias x.  TD: dtype of delta, TY: dtype of y.
template <typename TD, typename TY>
__global__ __launch_bounds__(256) void sandwich_norm_kernel(const float* x, const TD* __restrict__ delta,
                                                            int64_t ld_delta, const float* __restrict__ post_w, float post_add, float post_scale,
                                                            float* x_out, const float* __restrict__ pre_w,
                                                            float pre_add, TY* __restrict__ y, int64_t E, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    const float* xr = x + row * E;
    float* xo = x_out + row * E;
    float rinv_d = post_scale;
    if (delta && post_w) {
        const TD* dr = delta + row * ld_delta;
        float ss = 0.f;
        for (int64_t c = threadIdx.x; c < E; c += blockDim.x) {
            float d = Elem<TD>::ld(dr + c);
            ss += d * d;
        }
        ss = block_sum(ss, red);
        rinv_d = post_scale / sqrtf(ss / (float)E + eps);
    }
    float ss2 = 0.f;
    for (int64_t c = threadIdx.x; c < E; c += blockDim.x) {
        float v = xr[c];
        if (delta) {
            v += Elem<TD>::ld(delta + row * ld_delta + c) * rinv_d * (post_w ? post_w[c] + post_add : 1.f);
            xo[c] = v;
        } else if (xo != xr) {
            xo[c] = v;
        }
        ss2 += v * v;
    }
    if (!pre_w && !y) return;
    float rinv = 1.f;
    if (pre_w) {
        ss2 = block_sum(ss2, red);
        rinv = 1.0f / sqrtf(ss2 / (float)E + eps);
    }
    for (int64_t c = threadIdx.x; c < E; c += blockDim.x) {
        // the same thread wrote xo[c] above
        float v = (delta || xo != xr) ? xo[c] : xr[c];
        y[row * E + c] = cvt_out<TY>(v * rinv * (pre_w ? pre_w[c] + pre_add : 1.f));
    }
}


// The same, for E <= 256 * NPT: a row lives in registers, every global load is issued before the first reduction (one
// round trip instead of three), and nothing is read twice.
template <typename TD, typename TY, int NPT>
__global__ __launch_bounds__(256) void sandwich_norm_reg_kernel(const float* x, const TD* __restrict__ delta,
                                                                int64_t ld_delta, const float* __restrict__ post_w, float post_add, float post_scale,
                                                                float* x_out, const float* __restrict__ pre_w,
                                                                float pre_add, TY* __restrict__ y, int64_t E, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float xv[NPT], dv[NPT], pw[NPT], qw[NPT];
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int64_t c = threadIdx.x + 256 * i;
        const bool in = c < E;
        xv[i] = in ? x[row * E + c] : 0.f;
        dv[i] = (in && delta) ? Elem<TD>::ld(delta + row * ld_delta + c) : 0.f;
        pw[i] = (in && delta) ? (post_w ? post_w[c] + post_add : 1.f) : 0.f;
        qw[i] = in ? (pre_w ? pre_w[c] + pre_add : 1.f) : 0.f;
    }
    if (delta) {
        float rinv_d = post_scale;
        if (post_w) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < NPT; ++i) ss += dv[i] * dv[i];
            ss = block_sum(ss, red);
            rinv_d = post_scale / sqrtf(ss / (float)E + eps);
        }
#pragma unroll
        for (int i = 0; i < NPT; ++i) xv[i] += dv[i] * rinv_d * pw[i];
    }
    if (delta || x_out != x) {
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            const int64_t c = threadIdx.x + 256 * i;
            if (c < E) x_out[row * E + c] = xv[i];
        }
    }
    if (!pre_w && !y) return;
    float rinv = 1.f;
    if (pre_w) {
        float ss2 = 0.f;
#pragma unroll
        for (int i = 0; i < NPT; ++i) ss2 += xv[i] * xv[i];
        ss2 = block_sum(ss2, red);
        rinv = 1.0f / sqrtf(ss2 / (float)E + eps);
    }
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int64_t c = threadIdx.x + 256 * i;
        if (c < E) y[row * E + c] = cvt_out<TY>(xv[i] * rinv * qw[i]);
    }
}


// The same again for E % 4 == 0 and E <= 512 * 4 * NV: 512 threads, 16-byte loads and stores (a thread owns NV groups of four
// consecutive elements).  This is the form decode-sized steps run: few rows, so the launch is a chain of round trips and the
// number of memory instructions in it is what counts.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
    static __device__ __forceinline__ f32x4 ld(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
    static __device__ __forceinline__ void st(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
};
template <> struct Vec4<bf16> {
    static __device__ __forceinline__ f32x4 ld(const bf16* p) {
        bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
        return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    }
    static __device__ __forceinline__ void st(bf16* p, f32x4 v) {
        *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
    }
};
template <> struct Vec4<f16> {
    static __device__ __forceinline__ f32x4 ld(const f16* p) {
        f16x4 v = *reinterpret_cast<const f16x4*>(p);
        return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    }
    static __device__ __forceinline__ void st(f16* p, f32x4 v) {
        *reinterpret_cast<f16x4*>(p) = f16x4{(f16)v[0], (f16)v[1], (f16)v[2], (f16)v[3]};
    }
};


// four elements per thread (I % 4 == 0, rows 8- / 16-byte aligned)
template <typename T>
__global__ void glu_vec_kernel(const T* __restrict__ in, int64_t ld_in, T* __restrict__ out, int64_t ld_out, int64_t rows, int64_t I,
                               int mode, float alpha, float limit) {
    const int64_t I4 = I >> 2, n = rows * I4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = idx / I4, i = (idx - t * I4) * 4;
        f32x4 g = Vec4<T>::ld(in + t * ld_in + i);
        f32x4 u = Vec4<T>::ld(in + t * ld_in + I + i);
        f32x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (mode == 0) {
                r[e] = g[e] / (1.f + expf(-g[e])) * u[e];
            } else {
                const float ge = fminf(g[e], limit), ue = fminf(fmaxf(u[e], -limit), limit);
                r[e] = ge / (1.f + expf(-alpha * ge)) * (ue + 1.f);
            }
        }
        Vec4<T>::st(out + t * ld_out + i, r);
    }
}

// delta may also arrive as the S fp32 split-K slabs of the GEMM that produced it ([row / 32][S][32][slab_ld], TD = float,
// `delta` then points at the slabs): their sum is taken here instead of by a reduce launch of its own.
template <typename TD, typename TY, int NV>
__global__ __launch_bounds__(512) void sandwich_norm_vec_kernel(const float* x, const TD* __restrict__ delta, int64_t ld_delta,
                                                                const float* __restrict__ post_w, float post_add, float post_scale, float* x_out,
                                                                const float* __restrict__ pre_w, float pre_add,
                                                                TY* __restrict__ y, int64_t E, float eps, int S) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    f32x4 xv[NV], dv[NV], pw[NV], qw[NV];
    if (S > 0) {  // slabs: ld_delta is the slab row stride
        const float* sp = reinterpret_cast<const float*>(delta) + ((row >> 5) * S * 32 + (row & 31)) * ld_delta;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
            f32x4 acc = {};
            if (c < E)
                for (int sidx = 0; sidx < S; ++sidx) acc += Vec4<float>::ld(sp + (int64_t)sidx * 32 * ld_delta + c);
            dv[i] = acc;
        }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
        const bool in = c < E;
        xv[i] = in ? Vec4<float>::ld(x + row * E + c) : f32x4{};
        if (S == 0) dv[i] = (in && delta) ? Vec4<TD>::ld(delta + row * ld_delta + c) : f32x4{};
        pw[i] = (in && delta) ? (post_w ? Vec4<float>::ld(post_w + c) + post_add : f32x4{1.f, 1.f, 1.f, 1.f}) : f32x4{};
        qw[i] = in ? (pre_w ? Vec4<float>::ld(pre_w + c) + pre_add : f32x4{1.f, 1.f, 1.f, 1.f}) : f32x4{};
    }
    if (delta) {
        float rinv_d = post_scale;
        if (post_w) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < NV; ++i) ss += dv[i][0] * dv[i][0] + dv[i][1] * dv[i][1] + dv[i][2] * dv[i][2] + dv[i][3] * dv[i][3];
            ss = block_sum(ss, red);
            rinv_d = post_scale / sqrtf(ss / (float)E + eps);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) xv[i] += dv[i] * rinv_d * pw[i];
    }
    if (delta || x_out != x) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
            if (c < E) Vec4<float>::st(x_out + row * E + c, xv[i]);
        }
    }
    if (!pre_w && !y) return;
    float rinv = 1.f;
    if (pre_w) {
        float ss2 = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) ss2 += xv[i][0] * xv[i][0] + xv[i][1] * xv[i][1] + xv[i][2] * xv[i][2] + xv[i][3] * xv[i][3];
        ss2 = block_sum(ss2, red);
        rinv = 1.0f / sqrtf(ss2 / (float)E + eps);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
        if (c < E) Vec4<TY>::st(y + row * E + c, xv[i] * rinv * qw[i]);
    }
}

// out[t, i] = act(gate) * up' with gate = in[t, i], up = in[t, I + i]
//   mode 0: silu(gate) * up
//   mode 1: g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha * g) * (u + 1)
template <typename T>
__global__ void glu_kernel(const T* __restrict__ in, int64_t ld_in, T* __restrict__ out, int64_t ld_out, int64_t rows, int64_t I,
                           int mode, float alpha, float limit) {
    const int64_t n = rows * I;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = idx / I, i = idx - t * I;
        float g = Elem<T>::ld(in + t * ld_in + i);
        float u = Elem<T>::ld(in + t * ld_in + I + i);
        float r;
        if (mode == 0) {
            r = g / (1.f + expf(-g)) * u;
        } else {
            g = fminf(g, limit);
            u = fminf(fmaxf(u, -limit), limit);
            r = g / (1.f + expf(-alpha * g)) * (u + 1.f);
        }
        out[t * ld_out + i] = cvt_out<T>(r);
    }
}

template <typename TD, typename TY>
int launch_sandwich(const float* x, const void* delta, int64_t ld_delta, const float* post_w, float post_add, float post_scale, float* x_out,
                    const float* pre_w, float pre_add, void* y, int64_t rows, int64_t E, float eps, hipStream_t st, int num_slabs) {
#define TGIS_SANDWICH_REG(NPT)                                                                                                  \
    hipLaunchKernelGGL((sandwich_norm_reg_kernel<TD, TY, NPT>), dim3((unsigned)rows), dim3(256), 0, st, x, (const TD*)delta, ld_delta, \
                       post_w, post_add, post_scale, x_out, pre_w, pre_add, (TY*)y, E, eps)
#define TGIS_SANDWICH_VEC(NV)                                                                                                  \
    hipLaunchKernelGGL((sandwich_norm_vec_kernel<TD, TY, NV>), dim3((unsigned)rows), dim3(512), 0, st, x, (const TD*)delta, ld_delta, \
                       post_w, post_add, post_scale, x_out, pre_w, pre_add, (TY*)y, E, eps, num_slabs)
    const bool vec_ok = E % 4 == 0 && (!delta || ld_delta % 4 == 0) && ((uintptr_t)x % 16 == 0) && ((uintptr_t)x_out % 16 == 0) &&
                        ((uintptr_t)delta % 16 == 0) && ((uintptr_t)y % 16 == 0) && ((uintptr_t)post_w % 16 == 0) &&
                        ((uintptr_t)pre_w % 16 == 0);
    if (num_slabs > 0 && !(vec_ok && E <= 512 * 16)) return -1;  // slabs are taken by the 16-byte form only
    if (vec_ok && E <= 512 * 4)
        TGIS_SANDWICH_VEC(1);
    else if (vec_ok && E <= 512 * 8)
        TGIS_SANDWICH_VEC(2);
    else if (vec_ok && E <= 512 * 16)
        TGIS_SANDWICH_VEC(4);
    else if (E <= 256 * 4)
        TGIS_SANDWICH_REG(4);
    else if (E <= 256 * 8)
        TGIS_SANDWICH_REG(8);
    else if (E <= 256 * 16)
        TGIS_SANDWICH_REG(16);
    else if (E <= 256 * 32)
        TGIS_SANDWICH_REG(32);
    else
        hipLaunchKernelGGL((sandwich_norm_kernel<TD, TY>), dim3((unsigned)rows), dim3(256), 0, st, x, (const TD*)delta, ld_delta,
                           post_w, post_add, post_scale, x_out, pre_w, pre_add, (TY*)y, E, eps);
#undef TGIS_SANDWICH_REG
#undef TGIS_SANDWICH_VEC
    return 0;
}

template <typename TD>
int dispatch_y(int y_dtype, const float* x, const void* delta, int64_t ld_delta, const float* post_w, float post_add, float post_scale,
               float* x_out, const float* pre_w, float pre_add, void* y, int64_t rows, int64_t E, float eps, hipStream_t st,
               int num_slabs = 0) {
    switch (y_dtype) {
        case TGIS_F16: return launch_sandwich<TD, f16>(x, delta, ld_delta, post_w, post_add, post_scale, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
        case TGIS_BF16: return launch_sandwich<TD, bf16>(x, delta, ld_delta, post_w, post_add, post_scale, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
        default: return launch_sandwich<TD, float>(x, delta, ld_delta, post_w, post_add, post_scale, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
    }
}


// ---- elementwise pieces of pre-norm designs with a residual multiplier -------------------------------------------------
// xIELU with the two coefficients already through their softplus (ap = softplus(p), an = 1/2 + softplus(q)):
//   z > 0:  ap z^2 + z / 2        z <= 0:  an (exp(z) - 1 - z) + z / 2
__device__ __forceinline__ float xielu_f32(float z, float ap, float an) {
    return z > 0.f ? ap * z * z + 0.5f * z : an * (expm1f(z) - z) + 0.5f * z;
}

// act 0: xIELU(in)   act 1: in * sigmoid(other)   act 2: cap * tanh(in / cap) (p0 = cap)
template <typename T, typename TO>
__global__ void unary_rows_kernel(const T* __restrict__ in, int64_t ld_in, const T* __restrict__ other, int64_t ld_other,
                                  TO* __restrict__ out, int64_t ld_out, int64_t rows, int64_t C, int act, float p0, float p1) {
    const int64_t n = rows * C;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = idx / C, c = idx - t * C;
        const float z = Elem<T>::ld(in + t * ld_in + c);
        float r;
        if (act == 0) {
            r = xielu_f32(z, p0, p1);
        } else if (act == 1) {
            r = z / (1.f + expf(-Elem<T>::ld(other + t * ld_other + c)));
        } else {
            r = p0 * tanhf(z / p0);
        }
        out[t * ld_out + c] = cvt_out<TO>(r);
    }
}

// four elements per thread (C % 4 == 0, rows 8- / 16-byte aligned); T in and out
template <typename T>
__global__ void unary_rows_vec_kernel(const T* __restrict__ in, int64_t ld_in, const T* __restrict__ other, int64_t ld_other,
                                      T* __restrict__ out, int64_t ld_out, int64_t rows, int64_t C, int act, float p0, float p1) {
    const int64_t C4 = C >> 2, n = rows * C4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = idx / C4, c = (idx - t * C4) * 4;
        const f32x4 z = Vec4<T>::ld(in + t * ld_in + c);
        f32x4 r;
        if (act == 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = xielu_f32(z[e], p0, p1);
        } else if (act == 1) {
            const f32x4 g = Vec4<T>::ld(other + t * ld_other + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = z[e] / (1.f + expf(-g[e]));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = p0 * tanhf(z[e] / p0);
        }
        Vec4<T>::st(out + t * ld_out + c, r);
    }
}

// out[t][c] = gelu_tanh(gate[t][c]) * table[ids[t]][col0 + c]: a slice of a second token embedding, gated
template <typename T>
__global__ void gelu_gated_lookup_kernel(const T* __restrict__ gate, int64_t ld_gate, const int64_t* __restrict__ ids,
                                         const T* __restrict__ table, int64_t ld_table, int64_t col0, int64_t vocab,
                                         T* __restrict__ out, int64_t ld_out, int64_t rows, int64_t C) {
    const int64_t n = rows * C;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t t = idx / C, c = idx - t * C;
        const int64_t id = ids[t];
        const float e = (id >= 0 && id < vocab) ? Elem<T>::ld(table + id * ld_table + col0 + c) : 0.f;
        const float z = Elem<T>::ld(gate + t * ld_gate + c);
        const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
        out[t * ld_out + c] = cvt_out<T>(0.5f * z * (1.f + tanhf(inner)) * e);
    }
}

// y[t][c] = x[t][c] / sqrt(mean_c x^2 + eps) * w[c] for narrow rows (latents): a wave per row, fp32 statistics
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_rows_kernel(const T* __restrict__ x, int64_t ld_x, const float* __restrict__ w,
                                                            T* __restrict__ y, int64_t ld_y, int64_t rows, int C, float eps) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= rows) return;
    const T* xr = x + row * ld_x;
    float ss = 0.f;
    for (int c = lane; c < C; c += 64) {
        const float v = Elem<T>::ld(xr + c);
        ss += v * v;
    }
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)C + eps);
    for (int c = lane; c < C; c += 64) y[row * ld_y + c] = cvt_out<T>(Elem<T>::ld(xr + c) * rinv * w[c]);
}

template <typename T, typename TO>
void launch_unary(const void* in, int64_t ld_in, const void* other, int64_t ld_other, void* out, int64_t ld_out, int64_t rows,
                  int64_t C, int act, float p0, float p1, hipStream_t st) {
    const size_t al = 4 * sizeof(T);
    if (std::is_same<T, TO>::value && C % 4 == 0 && ld_in % 4 == 0 && ld_out % 4 == 0 && (uintptr_t)in % al == 0 && (uintptr_t)out % al == 0 &&
        (!other || (ld_other % 4 == 0 && (uintptr_t)other % al == 0))) {
        const int64_t n4 = rows * (C / 4);
        dim3 grid4((unsigned)(cdiv64(n4, 256) < 16384 ? cdiv64(n4, 256) : 16384));
        hipLaunchKernelGGL(unary_rows_vec_kernel<T>, grid4, dim3(256), 0, st, (const T*)in, ld_in, (const T*)other, ld_other, (T*)out, ld_out,
                           rows, C, act, p0, p1);
        return;
    }
    const int64_t n = rows * C;
    dim3 grid((unsigned)(cdiv64(n, 256) < 16384 ? cdiv64(n, 256) : 16384));
    hipLaunchKernelGGL((unary_rows_kernel<T, TO>), grid, dim3(256), 0, st, (const T*)in, ld_in, (const T*)other, ld_other, (TO*)out,
                       ld_out, rows, C, act, p0, p1);
}

}  // namespace

// ---- parallel layers with gated residuals and a learned mix over depth ------------------------------------------------
// One sublayer's result and the gate it passes before it joins the residual stream: delta is a [rows, ld] tensor of TD or the
// fp32 split-K slabs of the projection that produced it (slabs > 0, ld = their row stride); bias [E] TD is added to it;
// gate [rows, ld_gate] TD holds logits, gate_bias [E] TD is added to them, and the delta is multiplied by their sigmoid.
struct GatedDelta {
    const void* delta;
    int64_t ld;
    int slabs;
    const void* bias;
    const void* gate;
    int64_t ld_gate;
    const void* gate_bias;
};

template <typename T, int V> struct LdV;
template <typename T> struct LdV<T, 1> {
    static __device__ __forceinline__ f32x4 ld(const T* p) { return f32x4{Elem<T>::ld(p), 0.f, 0.f, 0.f}; }
    static __device__ __forceinline__ void st(T* p, f32x4 v) { *p = cvt_out<T>(v[0]); }
};
template <typename T> struct LdV<T, 4> {
    static __device__ __forceinline__ f32x4 ld(const T* p) { return Vec4<T>::ld(p); }
    static __device__ __forceinline__ void st(T* p, f32x4 v) { Vec4<T>::st(p, v); }
};

template <typename TD, int V>
__device__ __forceinline__ f32x4 gated_delta_at(const GatedDelta& d, int64_t row, int64_t c) {
    f32x4 v = {};
    if (d.slabs > 0) {
        const float* sp = reinterpret_cast<const float*>(d.delta) + ((row >> 5) * d.slabs * 32 + (row & 31)) * d.ld + c;
        for (int s2 = 0; s2 < d.slabs; ++s2) v += LdV<float, V>::ld(sp + (int64_t)s2 * 32 * d.ld);
    } else {
        v = LdV<TD, V>::ld(reinterpret_cast<const TD*>(d.delta) + row * d.ld + c);
    }
    if (d.bias) v += LdV<TD, V>::ld(reinterpret_cast<const TD*>(d.bias) + c);
    if (d.gate) {
        f32x4 z = LdV<TD, V>::ld(reinterpret_cast<const TD*>(d.gate) + row * d.ld_gate + c);
        if (d.gate_bias) z += LdV<TD, V>::ld(reinterpret_cast<const TD*>(d.gate_bias) + c);
#pragma unroll
        for (int u = 0; u < V; ++u) v[u] *= 1.f / (1.f + expf(-z[u]));
    }
    return v;
}

// One workgroup per row:
//     v = x + gate_a * a + gate_b * b                       (b optional)
//     hist[n_prev] = v;   x_out = sum_{j < n_prev} coef[j] hist[j] + coef[n_prev] v        (hist null: x_out = v)
//     y = x_out / sqrt(mean(x_out^2) + eps) * (pre_w + pre_add)                             (pre_w null: no y)
// hist entries are hist_stride floats apart.  x_out may alias x (not a hist entry that is still read).
template <typename TD, typename TY, int V>
__global__ __launch_bounds__(256) void parallel_residual_kernel(const float* x, GatedDelta a, GatedDelta b, float* hist, int n_prev,
                                                                int64_t hist_stride, const float* __restrict__ coef, float* x_out,
                                                                const float* __restrict__ pre_w, float pre_add, TY* __restrict__ y,
                                                                int64_t E, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float ss = 0.f;
    for (int64_t c = (int64_t)threadIdx.x * V; c < E; c += 256 * V) {
        f32x4 v = LdV<float, V>::ld(x + row * E + c) + gated_delta_at<TD, V>(a, row, c);
        if (b.delta) v += gated_delta_at<TD, V>(b, row, c);
        f32x4 xn = v;
        if (hist) {
            LdV<float, V>::st(hist + (int64_t)n_prev * hist_stride + row * E + c, v);
            xn = v * coef[n_prev];
            for (int j = 0; j < n_prev; ++j) xn += LdV<float, V>::ld(hist + (int64_t)j * hist_stride + row * E + c) * coef[j];
        }
        LdV<float, V>::st(x_out + row * E + c, xn);
#pragma unroll
        for (int u = 0; u < V; ++u) ss += xn[u] * xn[u];
    }
    if (!pre_w) return;
    ss = block_sum(ss, red);
    const float rinv = 1.0f / sqrtf(ss / (float)E + eps);
    for (int64_t c = (int64_t)threadIdx.x * V; c < E; c += 256 * V) {
        // the same thread wrote x_out[c .. c + V) above
        const f32x4 xn = LdV<float, V>::ld(x_out + row * E + c);
        f32x4 w = LdV<float, V>::ld(pre_w + c);
#pragma unroll
        for (int u = 0; u < V; ++u) w[u] = xn[u] * rinv * (w[u] + pre_add);
        LdV<TY, V>::st(y + row * E + c, w);
    }
}

// The same for E % 4 == 0, E <= 512 * 4 * NV and 16-byte aligned operands: 512 threads, a thread owns NV groups of four
// consecutive elements and keeps them in registers (nothing is read twice), and the entries of the depth mix are fetched four
// at a time before they are summed — a decode-sized step is a few rows, so the launch is a chain of round trips to memory and
// their number is what counts.
template <typename TD, typename TY, int NV>
__global__ __launch_bounds__(512) void parallel_residual_vec_kernel(const float* x, GatedDelta a, GatedDelta b, float* hist, int n_prev,
                                                                    int64_t hist_stride, const float* __restrict__ coef, float* x_out,
                                                                    const float* __restrict__ pre_w, float pre_add, TY* __restrict__ y,
                                                                    int64_t E, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    f32x4 v[NV], xn[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
        v[i] = f32x4{};
        if (c < E) {
            v[i] = Vec4<float>::ld(x + row * E + c) + gated_delta_at<TD, 4>(a, row, c);
            if (b.delta) v[i] += gated_delta_at<TD, 4>(b, row, c);
        }
        xn[i] = v[i];
    }
    if (hist) {
        const float* hrow = hist + row * E;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
            if (c < E) Vec4<float>::st(hist + (int64_t)n_prev * hist_stride + row * E + c, v[i]);
            xn[i] = v[i] * coef[n_prev];
        }
        int j = 0;
        for (; j + 4 <= n_prev; j += 4) {
            f32x4 t[4][NV];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
                    t[u][i] = c < E ? Vec4<float>::ld(hrow + (int64_t)(j + u) * hist_stride + c) : f32x4{};
                }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int i = 0; i < NV; ++i) xn[i] += t[u][i] * coef[j + u];
        }
        for (; j < n_prev; ++j)
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
                if (c < E) xn[i] += Vec4<float>::ld(hrow + (int64_t)j * hist_stride + c) * coef[j];
            }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
        if (c < E) Vec4<float>::st(x_out + row * E + c, xn[i]);
        ss += xn[i][0] * xn[i][0] + xn[i][1] * xn[i][1] + xn[i][2] * xn[i][2] + xn[i][3] * xn[i][3];
    }
    if (!pre_w) return;
    ss = block_sum(ss, red);
    const float rinv = 1.0f / sqrtf(ss / (float)E + eps);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t c = ((int64_t)threadIdx.x + 512 * i) * 4;
        if (c < E) Vec4<TY>::st(y + row * E + c, xn[i] * rinv * (Vec4<float>::ld(pre_w + c) + pre_add));
    }
}

template <typename TD, typename TY>
void launch_parallel_residual(const float* x, const GatedDelta& a, const GatedDelta& b, float* hist, int n_prev, int64_t hist_stride,
                              const float* coef, float* x_out, const float* pre_w, float pre_add, void* y, int64_t rows, int64_t E,
                              float eps, hipStream_t st) {
    auto al = [](const void* p, int n) { return ((uintptr_t)p % n) == 0; };
    auto ok = [&](const GatedDelta& d) {
        if (!d.delta) return true;
        const int esz = d.slabs > 0 ? 4 : (int)sizeof(TD);
        return d.ld % 4 == 0 && al(d.delta, 4 * esz) && al(d.bias, 4 * sizeof(TD)) && al(d.gate, 4 * sizeof(TD)) &&
               al(d.gate_bias, 4 * sizeof(TD)) && (!d.gate || d.ld_gate % 4 == 0);
    };
    const bool vec = E % 4 == 0 && ok(a) && ok(b) && al(x, 16) && al(x_out, 16) && al(hist, 16) && hist_stride % 4 == 0 && al(pre_w, 16) &&
                     al(y, 4 * sizeof(TY));
#define TGIS_PAR_VEC(NV)                                                                                                                 \
    hipLaunchKernelGGL((parallel_residual_vec_kernel<TD, TY, NV>), dim3((unsigned)rows), dim3(512), 0, st, x, a, b, hist, n_prev, hist_stride, \
                       coef, x_out, pre_w, pre_add, (TY*)y, E, eps)
    if (vec && E <= 512 * 4)
        TGIS_PAR_VEC(1);
    else if (vec && E <= 512 * 8)
        TGIS_PAR_VEC(2);
    else if (vec && E <= 512 * 16)
        TGIS_PAR_VEC(4);
    else if (vec)
        hipLaunchKernelGGL((parallel_residual_kernel<TD, TY, 4>), dim3((unsigned)rows), dim3(256), 0, st, x, a, b, hist, n_prev, hist_stride,
                           coef, x_out, pre_w, pre_add, (TY*)y, E, eps);
#undef TGIS_PAR_VEC
    else
        hipLaunchKernelGGL((parallel_residual_kernel<TD, TY, 1>), dim3((unsigned)rows), dim3(256), 0, st, x, a, b, hist, n_prev, hist_stride,
                           coef, x_out, pre_w, pre_add, (TY*)y, E, eps);
}

static bool dtype3(int d) { return d == TGIS_F16 || d == TGIS_BF16 || d == TGIS_F32; }

extern "C" int tgis_embedding_scaled_f32(const int64_t* ids, const void* table, float* out, int64_t T, int64_t E, int64_t vocab,
                                         float scale, int dtype, void* stream) {
    TGIS_CHECK_ARG(ids && table && out && E > 0 && vocab > 0, "tgis_embedding_scaled_f32: bad arguments");
    TGIS_CHECK_ARG(dtype3(dtype), "tgis_embedding_scaled_f32: bad dtype");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == TGIS_F16)
        hipLaunchKernelGGL(embedding_scaled_kernel<f16>, dim3((unsigned)T), dim3(256), 0, st, ids, (const f16*)table, out, E, vocab, scale);
    else if (dtype == TGIS_BF16)
        hipLaunchKernelGGL(embedding_scaled_kernel<bf16>, dim3((unsigned)T), dim3(256), 0, st, ids, (const bf16*)table, out, E, vocab, scale);
    else
        hipLaunchKernelGGL(embedding_scaled_kernel<float>, dim3((unsigned)T), dim3(256), 0, st, ids, (const float*)table, out, E, vocab, scale);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_sandwich_norm_f32(const float* x, const void* delta, int64_t ld_delta, int delta_dtype, const float* post_w,
                                      float post_add, float* x_out, const float* pre_w, float pre_add, void* y, int y_dtype,
                                      int64_t rows, int64_t E, float eps, void* stream) {
    TGIS_CHECK_ARG(x && x_out && E > 0 && rows >= 0, "tgis_sandwich_norm_f32: bad arguments");
    TGIS_CHECK_ARG(!delta || (post_w && ld_delta >= E && dtype3(delta_dtype)), "tgis_sandwich_norm_f32: delta needs its gain, a row stride and a dtype");
    TGIS_CHECK_ARG(!pre_w || (y && dtype3(y_dtype)), "tgis_sandwich_norm_f32: the normed output needs a buffer and a dtype");
    TGIS_CHECK_ARG(delta || pre_w || x_out != x, "tgis_sandwich_norm_f32: nothing to do");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    const int dd = delta ? delta_dtype : TGIS_F32;
    if (dd == TGIS_F16)
        dispatch_y<f16>(y_dtype, x, delta, ld_delta, post_w, post_add, 1.f, x_out, pre_w, pre_add, y, rows, E, eps, st);
    else if (dd == TGIS_BF16)
        dispatch_y<bf16>(y_dtype, x, delta, ld_delta, post_w, post_add, 1.f, x_out, pre_w, pre_add, y, rows, E, eps, st);
    else
        dispatch_y<float>(y_dtype, x, delta, ld_delta, post_w, post_add, 1.f, x_out, pre_w, pre_add, y, rows, E, eps, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_glu(const void* in, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int64_t I, int mode, float alpha,
                        float limit, int dtype, void* stream) {
    TGIS_CHECK_ARG(in && out && I > 0 && ld_in >= 2 * I && ld_out >= I, "tgis_glu: bad arguments");
    TGIS_CHECK_ARG(mode == 0 || mode == 1, "tgis_glu: mode 0 (silu(gate) * up) or 1 (clamped, sigmoid(alpha g), up + 1)");
    TGIS_CHECK_ARG(dtype3(dtype), "tgis_glu: bad dtype");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ACT, st);
    const int esz = dtype == TGIS_F32 ? 4 : 2;
    const bool vec = I % 4 == 0 && ld_in % 4 == 0 && ld_out % 4 == 0 && ((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                     (I * esz) % 8 == 0;
    const int64_t n = vec ? rows * (I / 4) : rows * I;
    dim3 grid((unsigned)(cdiv64(n, 256) < 16384 ? cdiv64(n, 256) : 16384));
#define TGIS_GLU(KERNEL, TT) \
    hipLaunchKernelGGL(KERNEL<TT>, grid, dim3(256), 0, st, (const TT*)in, ld_in, (TT*)out, ld_out, rows, I, mode, alpha, limit)
    if (dtype == TGIS_F16) {
        if (vec) TGIS_GLU(glu_vec_kernel, f16); else TGIS_GLU(glu_kernel, f16);
    } else if (dtype == TGIS_BF16) {
        if (vec) TGIS_GLU(glu_vec_kernel, bf16); else TGIS_GLU(glu_kernel, bf16);
    } else {
        if (vec) TGIS_GLU(glu_vec_kernel, float); else TGIS_GLU(glu_kernel, float);
    }
#undef TGIS_GLU
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_sandwich_norm_f32_partial(const float* x, const float* slabs, int num_slabs, int64_t slab_ld, const float* post_w,
                                              float post_add, float* x_out, const float* pre_w, float pre_add, void* y, int y_dtype,
                                              int64_t rows, int64_t E, float eps, void* stream) {
    TGIS_CHECK_ARG(x && x_out && slabs && post_w && E > 0 && rows >= 0, "tgis_sandwich_norm_f32_partial: bad arguments");
    TGIS_CHECK_ARG(num_slabs >= 1 && slab_ld >= E && slab_ld % 4 == 0, "tgis_sandwich_norm_f32_partial: bad slab geometry");
    TGIS_CHECK_ARG(!pre_w || (y && dtype3(y_dtype)), "tgis_sandwich_norm_f32_partial: the normed output needs a buffer and a dtype");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    const int rc = dispatch_y<float>(y_dtype, x, slabs, slab_ld, post_w, post_add, 1.f, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
    TGIS_CHECK_ARG(rc == 0, "tgis_sandwich_norm_f32_partial: needs E %% 4 == 0, E <= 8192 and 16-byte aligned operands");
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}


// The residual update of pre- and post-norm designs in one launch (see sandwich_norm_kernel): post_w null adds the scaled
// delta as it is; pre_w null with y given leaves x_out rounded to the activation dtype in y.
extern "C" int tgis_residual_update_f32(const float* x, const void* delta, int64_t ld_delta, int delta_dtype, const float* post_w,
                                        float post_add, float post_scale, float* x_out, const float* pre_w, float pre_add, void* y,
                                        int y_dtype, int64_t rows, int64_t E, float eps, void* stream) {
    TGIS_CHECK_ARG(x && x_out && E > 0 && rows >= 0, "tgis_residual_update_f32: bad arguments");
    TGIS_CHECK_ARG(!delta || (ld_delta >= E && dtype3(delta_dtype)), "tgis_residual_update_f32: delta needs a row stride and a dtype");
    TGIS_CHECK_ARG(!(pre_w || y) || (y && dtype3(y_dtype)), "tgis_residual_update_f32: the output needs a buffer and a dtype");
    TGIS_CHECK_ARG(delta || y || x_out != x, "tgis_residual_update_f32: nothing to do");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    const int dd = delta ? delta_dtype : TGIS_F32;
    if (dd == TGIS_F16)
        dispatch_y<f16>(y_dtype, x, delta, ld_delta, post_w, post_add, post_scale, x_out, pre_w, pre_add, y, rows, E, eps, st);
    else if (dd == TGIS_BF16)
        dispatch_y<bf16>(y_dtype, x, delta, ld_delta, post_w, post_add, post_scale, x_out, pre_w, pre_add, y, rows, E, eps, st);
    else
        dispatch_y<float>(y_dtype, x, delta, ld_delta, post_w, post_add, post_scale, x_out, pre_w, pre_add, y, rows, E, eps, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_residual_update_f32_partial(const float* x, const float* slabs, int num_slabs, int64_t slab_ld, const float* post_w,
                                                float post_add, float post_scale, float* x_out, const float* pre_w, float pre_add,
                                                void* y, int y_dtype, int64_t rows, int64_t E, float eps, void* stream) {
    TGIS_CHECK_ARG(x && x_out && slabs && E > 0 && rows >= 0, "tgis_residual_update_f32_partial: bad arguments");
    TGIS_CHECK_ARG(num_slabs >= 1 && slab_ld >= E && slab_ld % 4 == 0, "tgis_residual_update_f32_partial: bad slab geometry");
    TGIS_CHECK_ARG(!(pre_w || y) || (y && dtype3(y_dtype)), "tgis_residual_update_f32_partial: the output needs a buffer and a dtype");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    const int rc = dispatch_y<float>(y_dtype, x, slabs, slab_ld, post_w, post_add, post_scale, x_out, pre_w, pre_add, y, rows, E, eps, st, num_slabs);
    TGIS_CHECK_ARG(rc == 0, "tgis_residual_update_f32_partial: needs E %% 4 == 0, E <= 8192 and 16-byte aligned operands");
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

#define TGIS_BY_DTYPE(dtype, ...)                                    \
    do {                                                             \
        if ((dtype) == TGIS_F16) { using TT = f16; __VA_ARGS__; }        \
        else if ((dtype) == TGIS_BF16) { using TT = bf16; __VA_ARGS__; } \
        else { using TT = float; __VA_ARGS__; }                      \
    } while (0)

// out = xIELU(in) with ap = softplus(p), an = 1/2 + softplus(q) (the caller folds the learned scalars once)
extern "C" int tgis_xielu(const void* in, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int64_t C, float ap, float an,
                          int dtype, void* stream) {
    TGIS_CHECK_ARG(in && out && C > 0 && ld_in >= C && ld_out >= C && dtype3(dtype), "tgis_xielu: bad arguments");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ACT, st);
    TGIS_BY_DTYPE(dtype, launch_unary<TT, TT>(in, ld_in, nullptr, 0, out, ld_out, rows, C, 0, ap, an, st));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// out = in * sigmoid(gate): the output gate of a mixer (out may alias in)
extern "C" int tgis_sigmoid_gate_mul(const void* in, int64_t ld_in, const void* gate, int64_t ld_gate, void* out, int64_t ld_out,
                                     int64_t rows, int64_t C, int dtype, void* stream) {
    TGIS_CHECK_ARG(in && gate && out && C > 0 && ld_in >= C && ld_gate >= C && ld_out >= C && dtype3(dtype), "tgis_sigmoid_gate_mul: bad arguments");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ACT, st);
    TGIS_BY_DTYPE(dtype, launch_unary<TT, TT>(in, ld_in, gate, ld_gate, out, ld_out, rows, C, 1, 0.f, 0.f, st));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// logits <- cap * tanh(logits / cap), in place, fp32
extern "C" int tgis_logit_softcap(float* logits, int64_t ld, int64_t rows, int64_t V, float cap, void* stream) {
    TGIS_CHECK_ARG(logits && V > 0 && ld >= V && cap > 0.f, "tgis_logit_softcap: bad arguments");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    launch_unary<float, float>(logits, ld, nullptr, 0, logits, ld, rows, V, 2, cap, 0.f, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// out[t][c] = gelu_tanh(gate[t][c]) * table[ids[t]][col0 + c], c < C
extern "C" int tgis_gelu_gated_lookup(const void* gate, int64_t ld_gate, const int64_t* ids, const void* table, int64_t ld_table,
                                      int64_t col0, int64_t vocab, void* out, int64_t ld_out, int64_t rows, int64_t C, int dtype,
                                      void* stream) {
    TGIS_CHECK_ARG(gate && ids && table && out && C > 0 && ld_gate >= C && ld_out >= C && col0 >= 0 && ld_table >= col0 + C && vocab > 0 && dtype3(dtype),
                   "tgis_gelu_gated_lookup: bad arguments");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ACT, st);
    const int64_t n = rows * C;
    dim3 grid((unsigned)(cdiv64(n, 256) < 16384 ? cdiv64(n, 256) : 16384));
    TGIS_BY_DTYPE(dtype, hipLaunchKernelGGL(gelu_gated_lookup_kernel<TT>, grid, dim3(256), 0, st, (const TT*)gate, ld_gate, ids,
                                             (const TT*)table, ld_table, col0, vocab, (TT*)out, ld_out, rows, C));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// y = x / sqrt(mean x^2 + eps) * w over rows of C channels (y may alias x)
extern "C" int tgis_rms_norm_rows(const void* x, int64_t ld_x, const float* w, void* y, int64_t ld_y, int64_t rows, int64_t C,
                                  float eps, int dtype, void* stream) {
    TGIS_CHECK_ARG(x && w && y && C > 0 && C <= (1 << 30) && ld_x >= C && ld_y >= C && dtype3(dtype), "tgis_rms_norm_rows: bad arguments");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    TGIS_BY_DTYPE(dtype, hipLaunchKernelGGL(rms_norm_rows_kernel<TT>, dim3((unsigned)cdiv64(rows, 4)), dim3(256), 0, st, (const TT*)x,
                                             ld_x, w, (TT*)y, ld_y, rows, (int)C, eps));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// The residual update of a PARALLEL layer (one norm, mixer and feed-forward side by side) with gated residuals and a learned
// mix over depth, and the next layer's norm, in one launch:
//     v = x + sigmoid(gate_a + gate_bias_a) * (a + bias_a) + sigmoid(gate_b + gate_bias_b) * (b + bias_b)
//     hist[n_prev] = v;   x_out = sum_{j <= n_prev} mix[j] hist[j]            (hist NULL: x_out = v)
//     y = x_out / sqrt(mean(x_out^2) + eps) * (pre_w + pre_add)               (pre_w NULL: none)
// a / b: [rows, ld] tensors of `dtype`, or (slabs_x > 0) the fp32 split-K slabs of tgis_dense_gemm_partial with ld_x their row
// stride; b may be NULL (a layer without a feed-forward); biases [E] and gate logits [rows, ld_gate] / gate biases [E] are of
// `dtype`, each may be NULL.  hist: n_prev + 1 entries of [rows, E] fp32, hist_stride floats apart; mix [n_prev + 1] fp32.
extern "C" int tgis_parallel_residual_f32(const float* x, const void* a, int64_t ld_a, int slabs_a, const void* bias_a, const void* gate_a,
                                          int64_t ld_gate_a, const void* gate_bias_a, const void* b, int64_t ld_b, int slabs_b,
                                          const void* bias_b, const void* gate_b, int64_t ld_gate_b, const void* gate_bias_b, int dtype,
                                          float* hist, int n_prev, int64_t hist_stride, const float* mix, float* x_out, const float* pre_w,
                                          float pre_add, void* y, int y_dtype, int64_t rows, int64_t E, float eps, void* stream) {
    TGIS_CHECK_ARG(x && a && x_out && E > 0 && rows >= 0 && dtype3(dtype), "tgis_parallel_residual_f32: bad arguments");
    TGIS_CHECK_ARG(ld_a >= E && (!b || ld_b >= E) && (!gate_a || ld_gate_a >= E) && (!gate_b || ld_gate_b >= E) && slabs_a >= 0 && slabs_b >= 0,
                   "tgis_parallel_residual_f32: bad strides");
    TGIS_CHECK_ARG(!hist || (mix && n_prev >= 0 && hist_stride >= rows * E), "tgis_parallel_residual_f32: the depth mix needs coefficients and a stride");
    TGIS_CHECK_ARG(!pre_w || (y && dtype3(y_dtype)), "tgis_parallel_residual_f32: the normed output needs a buffer and a dtype");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    const GatedDelta da{a, ld_a, slabs_a, bias_a, gate_a, ld_gate_a, gate_bias_a};
    const GatedDelta db{b, ld_b, slabs_b, bias_b, gate_b, ld_gate_b, gate_bias_b};
#define TGIS_PAR_Y(TD)                                                                                                                  \
    do {                                                                                                                                \
        if (y_dtype == TGIS_F16) launch_parallel_residual<TD, f16>(x, da, db, hist, n_prev, hist_stride, mix, x_out, pre_w, pre_add, y, rows, E, eps, st);        \
        else if (y_dtype == TGIS_BF16) launch_parallel_residual<TD, bf16>(x, da, db, hist, n_prev, hist_stride, mix, x_out, pre_w, pre_add, y, rows, E, eps, st); \
        else launch_parallel_residual<TD, float>(x, da, db, hist, n_prev, hist_stride, mix, x_out, pre_w, pre_add, y, rows, E, eps, st);                          \
    } while (0)
    if (dtype == TGIS_F16) TGIS_PAR_Y(f16);
    else if (dtype == TGIS_BF16) TGIS_PAR_Y(bf16);
    else TGIS_PAR_Y(float);
#undef TGIS_PAR_Y
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
