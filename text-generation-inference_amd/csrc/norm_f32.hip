// Row kernels over an fp32 residual stream for layers with per-channel scales on their sublayers and a mean-free norm:
//
//   tgis_scaled_residual_norm   x <- x + s1 * a + s2 * b + v;   h = norm(x) * w        (norm: layer norm without bias, or RMS);
//                               a may be the average of two normed rows, c (a / rms(a) * wa + a2 / rms(a2) * wa2), made on the way
//   tgis_rms_pair_mean          y = ca * a / rms(a) * wa + cb * b / rms(b) * wb         (two mixers' results, normed, averaged)
//   tgis_poly_norm              y = c1 z / rms(z) + c2 z^2 / rms(z^2) + c3 z^3 / rms(z^3) + c0   over a row of feed-forward values
//
// Statistics, the stream and the normed rows are fp32; a and b arrive in the activation dtype or in fp32.  One workgroup of 256
// per row; the row waits in LDS between the passes (the variance is taken around the mean, not from the raw second moment).
#include "common.h"

namespace {

__device__ __forceinline__ float block_sum(float v, float* part) {
    v = wave_sum(v);
    __syncthreads();  // part may still be read from the sum before
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    return part[0] + part[1] + part[2] + part[3];
}

template <typename T> __device__ __forceinline__ float ld_as(const void* p, int64_t i, int f32) {
    return f32 ? reinterpret_cast<const float*>(p)[i] : (float)reinterpret_cast<const T*>(p)[i];
}

template <typename T, bool PAIR>
__global__ __launch_bounds__(256) void scaled_residual_norm_kernel(const float* x_in, float* x_out, const void* a,
                                                                   int64_t ld_a, int a_f32, const float* __restrict__ s1, const void* b,
                                                                   int64_t ld_b, int b_f32, const float* __restrict__ s2,
                                                                   const float* __restrict__ v, const float* __restrict__ w, void* h,
                                                                   int h_f32, int W, float eps, int mean_free, const void* a2,
                                                                   int64_t ld_a2, int a2_f32, const float* __restrict__ wa,
                                                                   const float* __restrict__ wa2, float pair_coef) {
    extern __shared__ float row[];
    __shared__ float part[4];
    const int64_t t = blockIdx.x;
    float ra = 1.f, ra2 = 0.f;
    if (PAIR) {  // a is a pair of rows, each divided by its root mean square
        float qa = 0.f, qb = 0.f;
        for (int c = threadIdx.x; c < W; c += 256) {
            const float u = ld_as<T>(a, t * ld_a + c, a_f32), u2 = ld_as<T>(a2, t * ld_a2 + c, a2_f32);
            qa += u * u;
            qb += u2 * u2;
        }
        ra = pair_coef / sqrtf(block_sum(qa, part) / (float)W + eps);
        ra2 = pair_coef / sqrtf(block_sum(qb, part) / (float)W + eps);
    }
    float sum = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float val = x_in ? x_in[t * W + c] : 0.f;
        if (PAIR) val = fmaf(s1 ? s1[c] : 1.f, ld_as<T>(a, t * ld_a + c, a_f32) * ra * wa[c] + ld_as<T>(a2, t * ld_a2 + c, a2_f32) * ra2 * wa2[c], val);
        else if (a) val = fmaf(s1 ? s1[c] : 1.f, ld_as<T>(a, t * ld_a + c, a_f32), val);
        if (b) val = fmaf(s2 ? s2[c] : 1.f, ld_as<T>(b, t * ld_b + c, b_f32), val);
        if (v) val += v[c];
        row[c] = val;
        if (x_out) x_out[t * W + c] = val;
        sum += val;
    }
    if (!w) return;
    const float mean = mean_free ? block_sum(sum, part) / (float)W : 0.f;
    float sq = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float d = row[c] - mean;
        sq += d * d;
    }
    const float rinv = 1.f / sqrtf(block_sum(sq, part) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) {
        const float y = (row[c] - mean) * rinv * w[c];
        if (h_f32) reinterpret_cast<float*>(h)[t * W + c] = y;
        else reinterpret_cast<T*>(h)[t * W + c] = (T)y;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void rms_pair_mean_kernel(const void* a, int64_t ld_a, int a_f32, const float* __restrict__ wa, float ca,
                                                            const void* b, int64_t ld_b, int b_f32, const float* __restrict__ wb, float cb,
                                                            float* __restrict__ y, int W, float eps) {
    __shared__ float part[4];
    const int64_t t = blockIdx.x;
    float sa = 0.f, sb = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float u = ld_as<T>(a, t * ld_a + c, a_f32), v = ld_as<T>(b, t * ld_b + c, b_f32);
        sa += u * u;
        sb += v * v;
    }
    const float ra = ca / sqrtf(block_sum(sa, part) / (float)W + eps);
    const float rb = cb / sqrtf(block_sum(sb, part) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256)
        y[t * W + c] = ld_as<T>(a, t * ld_a + c, a_f32) * ra * wa[c] + ld_as<T>(b, t * ld_b + c, b_f32) * rb * wb[c];
}

template <typename T>
__global__ __launch_bounds__(256) void poly_norm_kernel(const T* __restrict__ z, int64_t ld_z, T* __restrict__ y, int64_t ld_y, int F,
                                                        float c1, float c2, float c3, float c0, float eps) {
    __shared__ float part[4];
    const int64_t t = blockIdx.x;
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
    for (int c = threadIdx.x; c < F; c += 256) {
        const float v = (float)z[t * ld_z + c], v2 = v * v;
        s2 += v2;
        s4 += v2 * v2;
        s6 += v2 * v2 * v2;
    }
    const float r1 = c1 / sqrtf(block_sum(s2, part) / (float)F + eps);
    const float r2 = c2 / sqrtf(block_sum(s4, part) / (float)F + eps);
    const float r3 = c3 / sqrtf(block_sum(s6, part) / (float)F + eps);
    for (int c = threadIdx.x; c < F; c += 256) {
        const float v = (float)z[t * ld_z + c];
        y[t * ld_y + c] = (T)(v * (r1 + v * (r2 + v * r3)) + c0);
    }
}

bool dtype_ok(int d) { return d == TGIS_F16 || d == TGIS_BF16 || d == TGIS_F32; }

}  // namespace

#define BY_DTYPE(dtype, ...)                          \
    do {                                              \
        if (dtype == TGIS_F16) {                      \
            using TT = f16;                           \
            __VA_ARGS__;                              \
        } else if (dtype == TGIS_BF16) {              \
            using TT = bf16;                          \
            __VA_ARGS__;                              \
        } else {                                      \
            using TT = float;                         \
            __VA_ARGS__;                              \
        }                                             \
    } while (0)

extern "C" int tgis_scaled_residual_norm(const float* x_in, float* x_out, const void* a, int64_t ld_a, int a_f32, const float* s1,
                                         const void* b, int64_t ld_b, int b_f32, const float* s2, const float* v, const float* w,
                                         void* h, int h_f32, int64_t rows, int64_t W, float eps, int mean_free, const void* a2,
                                         int64_t ld_a2, int a2_f32, const float* wa, const float* wa2, float pair_coef, int dtype,
                                         void* stream) {
    TGIS_CHECK_ARG(!a2 || (a && wa && wa2 && ld_a2 >= W), "tgis_scaled_residual_norm: a pair needs both rows and both gains");
    TGIS_CHECK_ARG((x_in || a || b) && (x_out || (w && h)) && (!w || h), "tgis_scaled_residual_norm: nothing to do");
    TGIS_CHECK_ARG(W >= 1 && W * 4 <= 64 * 1024 && (!a || ld_a >= W) && (!b || ld_b >= W) && dtype_ok(dtype),
                   "tgis_scaled_residual_norm: rows of up to 16384 channels (got %ld)", (long)W);
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    if (a2)
        BY_DTYPE(dtype, hipLaunchKernelGGL((scaled_residual_norm_kernel<TT, true>), dim3((unsigned)rows), dim3(256), (size_t)W * 4, st, x_in, x_out, a,
                                           ld_a, a_f32, s1, b, ld_b, b_f32, s2, v, w, h, h_f32, (int)W, eps, mean_free, a2, ld_a2, a2_f32, wa, wa2,
                                           pair_coef));
    else
        BY_DTYPE(dtype, hipLaunchKernelGGL((scaled_residual_norm_kernel<TT, false>), dim3((unsigned)rows), dim3(256), (size_t)W * 4, st, x_in, x_out, a,
                                           ld_a, a_f32, s1, b, ld_b, b_f32, s2, v, w, h, h_f32, (int)W, eps, mean_free, a2, ld_a2, a2_f32, wa, wa2,
                                           pair_coef));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_rms_pair_mean(const void* a, int64_t ld_a, int a_f32, const float* wa, float ca, const void* b, int64_t ld_b, int b_f32,
                                  const float* wb, float cb, float* y, int64_t rows, int64_t W, float eps, int dtype, void* stream) {
    TGIS_CHECK_ARG(a && b && wa && wb && y && W >= 1 && ld_a >= W && ld_b >= W && dtype_ok(dtype), "tgis_rms_pair_mean: bad arguments");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_NORM, st);
    BY_DTYPE(dtype, hipLaunchKernelGGL(rms_pair_mean_kernel<TT>, dim3((unsigned)rows), dim3(256), 0, st, a, ld_a, a_f32, wa, ca, b, ld_b, b_f32,
                                       wb, cb, y, (int)W, eps));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_poly_norm(const void* z, int64_t ld_z, void* y, int64_t ld_y, int64_t rows, int64_t F, float c1, float c2, float c3,
                              float c0, float eps, int dtype, void* stream) {
    TGIS_CHECK_ARG(z && y && F >= 1 && ld_z >= F && ld_y >= F && dtype_ok(dtype), "tgis_poly_norm: bad arguments");
    if (rows == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ACT, st);
    BY_DTYPE(dtype, hipLaunchKernelGGL(poly_norm_kernel<TT>, dim3((unsigned)rows), dim3(256), 0, st, (const TT*)z, ld_z, (TT*)y, ld_y, (int)F, c1,
                                       c2, c3, c0, eps));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
