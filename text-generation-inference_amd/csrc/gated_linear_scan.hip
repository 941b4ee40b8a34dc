// Gated linear recurrence whose forget gate also decides what is written (HGRN2-style linear attention):
//
//     S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T          o_t = S_t^T q_t          per head, S [dk, dv] in fp32
//     f_t = l + (1 - l) sigmoid(z_t + b)                  a forget gate bounded below by l (per head and key channel)
//     q_t = silu(projection)  (or the projection as it is)
//     out_t = o_t / sqrt(mean(o_t^2) + eps) * gain * out_scale      (RMS norm over the head's dv channels, one gain for all heads)
//
// The state lives in a slot of the recurrent state cache ([slots][H][dk][dv] fp32, row-major) and is carried from step to step; a
// step that starts at position 0 starts from zeros whatever the slot holds.  Gates, (1 - f), the state and the read-out are
// fp32 whatever the activation dtype T of the projections is.
//
// Workgroup = (sequence, head) = dv_pad x 4 threads: a quad of neighbouring lanes shares column j of S, lane q of the quad
// keeps rows q RPL .. q RPL + RPL - 1 in registers.  Tokens go through LDS in stages of TS: the stage's q and f rows (activated,
// fp32, one padded segment per row group so that the four groups' 16-byte reads fall into different banks) and v rows; per token
// a lane does RPL fused updates s = v + f (s - v) and RPL products for the read-out, the quad adds up by two lane exchanges, and
// the stage's outputs wait in LDS for the norm, which a wave does per token once the stage is through.
#include "common.h"

namespace {

constexpr int TS = 16;   // tokens per stage
constexpr int SEG_PAD = 4;  // floats between the row groups' segments

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

template <typename T, int RPL>
__global__ __launch_bounds__(1024) void gated_linear_scan_kernel(
    const T* __restrict__ proj, int64_t ld, int64_t q_col0, int64_t f_col0, int64_t v_col0, const float* __restrict__ f_bias,
    const float* __restrict__ lower, const float* __restrict__ gain, float* __restrict__ state, const int32_t* __restrict__ state_slots,
    const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions, T* __restrict__ out, int64_t ld_out, float out_scale, int H,
    int dk, int dv, int dv_pad, float eps, int q_act) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    constexpr int SEG = RPL + SEG_PAD, ROW = 4 * SEG;
    float* qs = smem;                       // [TS][ROW]
    float* fs = qs + TS * ROW;              // [TS][ROW]
    float* vs = fs + TS * ROW;              // [TS][dv_pad]
    float* os = vs + TS * dv_pad;           // [TS][dv_pad]
    const int b = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, j = tid >> 2, qd = tid & 3;
    const int t0 = cu_q[b], qlen = cu_q[b + 1] - t0;
    if (qlen <= 0) return;
    const bool fresh = positions[t0] == 0;
    float* S = state + ((int64_t)state_slots[b] * H + h) * (int64_t)dk * dv;
    float s[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        const int i = qd * RPL + r;
        s[r] = (!fresh && i < dk && j < dv) ? S[(int64_t)i * dv + j] : 0.f;
    }
    const int nthreads = blockDim.x, wave = tid >> 6, lane = tid & 63, nw = nthreads >> 6;
    for (int base = 0; base < qlen; base += TS) {
        const int n = min(TS, qlen - base);
        __syncthreads();  // the stage before is consumed (its outputs normed)
        for (int e = tid; e < n * 4 * RPL; e += nthreads) {
            const int tt = e / (4 * RPL), i = e - tt * (4 * RPL);
            float qv = 0.f, fv = 1.f;  // rows past dk: the state stays zero and is never read
            if (i < dk) {
                const T* row = proj + (int64_t)(t0 + base + tt) * ld;
                qv = ldf(row + q_col0 + (int64_t)h * dk + i);
                if (q_act) qv = qv * sigmoid_f(qv);
                const float z = ldf(row + f_col0 + (int64_t)h * dk + i) + (f_bias ? f_bias[h * dk + i] : 0.f);
                const float lo = lower ? lower[h * dk + i] : 0.f;
                fv = lo + (1.f - lo) * sigmoid_f(z);
            }
            const int at = tt * ROW + (i / RPL) * SEG + (i % RPL);
            qs[at] = qv;
            fs[at] = fv;
        }
        for (int e = tid; e < n * dv_pad; e += nthreads) {
            const int tt = e / dv_pad, c = e - tt * dv_pad;
            vs[e] = c < dv ? ldf(proj + (int64_t)(t0 + base + tt) * ld + v_col0 + (int64_t)h * dv + c) : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < n; ++tt) {
            const float vj = vs[tt * dv_pad + j];
            const float* qrow = qs + tt * ROW + qd * SEG;
            const float* frow = fs + tt * ROW + qd * SEG;
            float acc = 0.f;
#pragma unroll
            for (int r4 = 0; r4 < RPL; r4 += 4) {
                const f32x4 f4 = *reinterpret_cast<const f32x4*>(frow + r4);
                const f32x4 q4 = *reinterpret_cast<const f32x4*>(qrow + r4);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    // f s + (1 - f) v
                    s[r4 + u] = f4[u] * s[r4 + u] + (1.f - f4[u]) * vj;
                    acc += s[r4 + u] * q4[u];
                }
            }
            acc += __shfl_xor(acc, 1, 64);
            acc += __shfl_xor(acc, 2, 64);
            if (qd == 0) os[tt * dv_pad + j] = acc;
        }
        __syncthreads();
        for (int tt = wave; tt < n; tt += nw) {
            float ss = 0.f;
            for (int c = lane; c < dv; c += 64) {
                const float o = os[tt * dv_pad + c];
                ss += o * o;
            }
            ss = wave_sum(ss);
            const float rinv = out_scale / sqrtf(ss / (float)dv + eps);
            T* orow = out + (int64_t)(t0 + base + tt) * ld_out + (int64_t)h * dv;
            for (int c = lane; c < dv; c += 64) orow[c] = (T)(os[tt * dv_pad + c] * rinv * gain[c]);
        }
    }
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        const int i = qd * RPL + r;
        if (i < dk && j < dv) S[(int64_t)i * dv + j] = s[r];
    }
}

template <typename T, int RPL>
void launch_scan(const void* proj, int64_t ld, int64_t q_col0, int64_t f_col0, int64_t v_col0, const float* f_bias, const float* lower,
                 const float* gain, float* state, const int32_t* state_slots, const int32_t* cu_q, const int32_t* positions, void* out,
                 int64_t ld_out, float out_scale, int64_t B, int H, int dk, int dv, float eps, int q_act, hipStream_t st) {
    const int dv_pad = (dv + 15) / 16 * 16;
    const size_t lds = ((size_t)2 * TS * 4 * (RPL + SEG_PAD) + (size_t)2 * TS * dv_pad) * sizeof(float);
    if (lds > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)gated_linear_scan_kernel<T, RPL>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((gated_linear_scan_kernel<T, RPL>), dim3((unsigned)B, (unsigned)H), dim3(4 * dv_pad), lds, st, (const T*)proj, ld,
                       q_col0, f_col0, v_col0, f_bias, lower, gain, state, state_slots, cu_q, positions, (T*)out, ld_out, out_scale, H, dk,
                       dv, dv_pad, eps, q_act);
}

template <typename T>
void launch_scan_rows(int dk, const void* proj, int64_t ld, int64_t q_col0, int64_t f_col0, int64_t v_col0, const float* f_bias,
                      const float* lower, const float* gain, float* state, const int32_t* state_slots, const int32_t* cu_q,
                      const int32_t* positions, void* out, int64_t ld_out, float out_scale, int64_t B, int H, int dv, float eps, int q_act,
                      hipStream_t st) {
#define TGIS_SCAN(RPL) \
    launch_scan<T, RPL>(proj, ld, q_col0, f_col0, v_col0, f_bias, lower, gain, state, state_slots, cu_q, positions, out, ld_out, out_scale, B, H, dk, dv, eps, q_act, st)
    if (dk <= 16) TGIS_SCAN(4);
    else if (dk <= 32) TGIS_SCAN(8);
    else if (dk <= 64) TGIS_SCAN(16);
    else if (dk <= 128) TGIS_SCAN(32);
    else TGIS_SCAN(64);
#undef TGIS_SCAN
}

}  // namespace

extern "C" int tgis_gated_linear_scan(const void* proj, int64_t ld, int64_t q_col0, int64_t f_col0, int64_t v_col0, const float* f_bias,
                                      const float* lower, const float* gain, float* state, const int32_t* state_slots,
                                      const int32_t* cu_seqlens_q, const int32_t* positions, void* out, int64_t ld_out, float out_scale,
                                      int64_t B, int H, int dk, int dv, float eps, int q_act, int dtype, void* stream) {
    TGIS_CHECK_ARG(proj && gain && state && state_slots && cu_seqlens_q && positions && out, "tgis_gated_linear_scan: null tensor");
    TGIS_CHECK_ARG(H >= 1 && H <= 65535 && dk >= 1 && dk <= 256 && dv >= 1 && dv <= 256, "tgis_gated_linear_scan: heads of up to 256 x 256 (got %d x %d)", dk, dv);
    TGIS_CHECK_ARG(q_col0 >= 0 && f_col0 >= 0 && v_col0 >= 0 && ld >= q_col0 + (int64_t)H * dk && ld >= f_col0 + (int64_t)H * dk &&
                       ld >= v_col0 + (int64_t)H * dv && ld_out >= (int64_t)H * dv,
                   "tgis_gated_linear_scan: bad strides");
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_gated_linear_scan: bad dtype");
    if (B == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_SCAN, st);
    if (dtype == TGIS_F16)
        launch_scan_rows<f16>(dk, proj, ld, q_col0, f_col0, v_col0, f_bias, lower, gain, state, state_slots, cu_seqlens_q, positions, out, ld_out, out_scale, B, H, dv, eps, q_act, st);
    else if (dtype == TGIS_BF16)
        launch_scan_rows<bf16>(dk, proj, ld, q_col0, f_col0, v_col0, f_bias, lower, gain, state, state_slots, cu_seqlens_q, positions, out, ld_out, out_scale, B, H, dv, eps, q_act, st);
    else
        launch_scan_rows<float>(dk, proj, ld, q_col0, f_col0, v_col0, f_bias, lower, gain, state, state_slots, cu_seqlens_q, positions, out, ld_out, out_scale, B, H, dv, eps, q_act, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
