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
// Workgroup = (sequence, head) = dv_pad x 4 / CPL threads: a quad of neighbouring lanes shares column j of S (and, with CPL = 2,
// column j + dv_pad / 2), lane q of the quad keeps rows q RPL .. q RPL + RPL - 1 of its columns in registers.  Tokens go through LDS in stages of `ts`: the stage's q and f rows (activated,
// fp32, one padded segment per row group so that the four groups' 16-byte reads fall into different banks) and v rows, in two
// buffers.  A thread asks for its share of the NEXT stage's projections before it works through the current one (per token RPL
// updates s = f s + (1 - f) v and RPL products for the read-out; the quad adds up by two data-parallel-primitive moves), and activates and
// stores them afterwards: the trip to memory is hidden behind the arithmetic.  The stage's outputs wait in LDS for the norm,
// which a wave does per token once the stage is through.
#include <algorithm>
#include "common.h"

namespace {

constexpr int SEG_PAD = 4;  // floats between the row groups' segments
constexpr int PFQ = 2;      // (q, f) pairs and
constexpr int PFV = 4;      // values of the next stage that a thread holds in registers: ts dk <= PFQ threads, ts dv <= PFV threads

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

struct ScanArgs {
    const void* proj;
    int64_t ld, q_col0, f_col0, v_col0;
    const float* f_bias;
    const float* lower;
    const float* gain;
    float* state;
    const int32_t* state_slots;
    const int32_t* cu_q;
    const int32_t* positions;
    void* out;
    int64_t ld_out;
    float out_scale;
    int H, dk, dv, dv_pad, ts;
    float eps;
    int q_act;
};

template <typename T, int RPL, int CPL, int MAXT>
__global__ __launch_bounds__(MAXT) void gated_linear_scan_kernel(ScanArgs a) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    constexpr int SEG = RPL + SEG_PAD, ROW = 4 * SEG;
    const int ts = a.ts, dk = a.dk, dv = a.dv, dv_pad = a.dv_pad;
    float* qs = smem;                        // [2][ts][ROW]
    float* fs = qs + 2 * ts * ROW;           // [2][ts][ROW]
    float* vs = fs + 2 * ts * ROW;           // [2][ts][dv_pad]
    float* os = vs + 2 * ts * dv_pad;        // [ts][dv_pad]
    const int b = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, j = tid >> 2, qd = tid & 3;
    const int t0 = a.cu_q[b], qlen = a.cu_q[b + 1] - t0;
    if (qlen <= 0) return;
    const int nthreads = blockDim.x;
    const bool fresh = a.positions[t0] == 0;
    const T* proj = reinterpret_cast<const T*>(a.proj);
    float* S = a.state + ((int64_t)a.state_slots[b] * a.H + h) * (int64_t)dk * dv;
    // a lane's CPL columns are dv_pad / CPL apart
    const int jstep = dv_pad / CPL;
    float s[CPL][RPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            const int i = qd * RPL + r, jc = j + c * jstep;
            s[c][r] = (!fresh && i < dk && jc < dv) ? S[(int64_t)i * dv + jc] : 0.f;
        }
    // rows past dk and columns past dv of both buffers: f = 1, q = 0, v = 0 (their state stays zero and is never read)
    for (int e = tid; e < 2 * ts * ROW; e += nthreads) {
        qs[e] = 0.f;
        fs[e] = 1.f;
    }
    for (int e = tid; e < 2 * ts * dv_pad; e += nthreads) vs[e] = 0.f;
    T qr[PFQ], fr[PFQ], vr[PFV];
    // tokens [first, first + n) of the sequence: this thread's share of their projections, as they are
    auto fetch = [&](int first, int n) {
#pragma unroll
        for (int u = 0; u < PFQ; ++u) {
            const int e = tid + u * nthreads;
            if (e < n * dk) {
                const int tt = e / dk, i = e - tt * dk;
                const T* row = proj + (int64_t)(t0 + first + tt) * a.ld + (int64_t)h * dk + i;
                qr[u] = row[a.q_col0];
                fr[u] = row[a.f_col0];
            }
        }
#pragma unroll
        for (int u = 0; u < PFV; ++u) {
            const int e = tid + u * nthreads;
            if (e < n * dv) {
                const int tt = e / dv, c = e - tt * dv;
                vr[u] = proj[(int64_t)(t0 + first + tt) * a.ld + a.v_col0 + (int64_t)h * dv + c];
            }
        }
    };
    // ... activated and stored into one stage buffer
    auto commit = [&](int n, float* qb, float* fb, float* vb) {
#pragma unroll
        for (int u = 0; u < PFQ; ++u) {
            const int e = tid + u * nthreads;
            if (e < n * dk) {
                const int tt = e / dk, i = e - tt * dk;
                float qv = (float)qr[u];
                if (a.q_act) qv = qv * sigmoid_f(qv);
                const float z = (float)fr[u] + (a.f_bias ? a.f_bias[h * dk + i] : 0.f);
                const float lo = a.lower ? a.lower[h * dk + i] : 0.f;
                const int at = tt * ROW + (i / RPL) * SEG + (i % RPL);
                qb[at] = qv;
                fb[at] = lo + (1.f - lo) * sigmoid_f(z);
            }
        }
#pragma unroll
        for (int u = 0; u < PFV; ++u) {
            const int e = tid + u * nthreads;
            if (e < n * dv) {
                const int tt = e / dv, c = e - tt * dv;
                vb[tt * dv_pad + c] = (float)vr[u];
            }
        }
    };
    fetch(0, min(ts, qlen));
    __syncthreads();  // the buffers are filled with their neutral values
    commit(min(ts, qlen), qs, fs, vs);
    __syncthreads();
    const int wave = tid >> 6, lane = tid & 63, nw = nthreads >> 6;
    T* out = reinterpret_cast<T*>(a.out);
    int buf = 0;
    for (int base = 0; base < qlen; base += ts, buf ^= 1) {
        const int n = min(ts, qlen - base);
        const int n_next = min(ts, qlen - base - ts);
        if (n_next > 0) fetch(base + ts, n_next);
        const float* qb = qs + buf * ts * ROW + qd * SEG;
        const float* fb = fs + buf * ts * ROW + qd * SEG;
        const float* vb = vs + buf * ts * dv_pad + j;
#pragma unroll 1
        for (int tt = 0; tt < n; ++tt) {
            float vj[CPL], acc[CPL];
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                vj[c] = vb[tt * dv_pad + c * jstep];
                acc[c] = 0.f;
            }
#pragma unroll
            for (int r4 = 0; r4 < RPL; r4 += 4) {
                const f32x4 f4 = *reinterpret_cast<const f32x4*>(fb + tt * ROW + r4);
                const f32x4 q4 = *reinterpret_cast<const f32x4*>(qb + tt * ROW + r4);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const float g = 1.f - f4[u];
#pragma unroll
                    for (int c = 0; c < CPL; ++c) {
                        s[c][r4 + u] = fmaf(f4[u], s[c][r4 + u], g * vj[c]);
                        acc[c] = fmaf(s[c][r4 + u], q4[u], acc[c]);
                    }
                }
            }
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                // the quad's sum, by data-parallel-primitive moves (no trip through LDS)
                float t = acc[c];
                t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0xB1, 0xF, 0xF, true));  // lane ^ 1
                t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x4E, 0xF, 0xF, true));  // lane ^ 2
                if (qd == 0) os[tt * dv_pad + j + c * jstep] = t;
            }
        }
        __syncthreads();
        for (int tt = wave; tt < n; tt += nw) {
            float ss = 0.f;
            for (int c = lane; c < dv; c += 64) {
                const float o = os[tt * dv_pad + c];
                ss += o * o;
            }
            ss = wave_sum(ss);
            const float rinv = a.out_scale / sqrtf(ss / (float)dv + a.eps);
            T* orow = out + (int64_t)(t0 + base + tt) * a.ld_out + (int64_t)h * dv;
            for (int c = lane; c < dv; c += 64) orow[c] = (T)(os[tt * dv_pad + c] * rinv * a.gain[c]);
        }
        if (n_next > 0) commit(n_next, qs + (buf ^ 1) * ts * ROW, fs + (buf ^ 1) * ts * ROW, vs + (buf ^ 1) * ts * dv_pad);
        __syncthreads();  // the outputs are out, the next stage is in
    }
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            const int i = qd * RPL + r, jc = j + c * jstep;
            if (i < dk && jc < dv) S[(int64_t)i * dv + jc] = s[c][r];
        }
}

template <typename T, int RPL, int CPL, int MAXT>
void launch_scan_as(ScanArgs a, int64_t B, int64_t max_q_len, hipStream_t st) {
    a.dv_pad = (a.dv + 16 * CPL - 1) / (16 * CPL) * (16 * CPL);
    const int threads = 4 * a.dv_pad / CPL;
    // tokens per stage: a power of two up to 32 that a thread's registers can prefetch, that 140 KiB of LDS hold (two input
    // buffers and the outputs), and no more than the longest run needs
    auto bytes = [&](int ts) { return ((size_t)4 * ts * 4 * (RPL + SEG_PAD) + (size_t)3 * ts * a.dv_pad) * sizeof(float); };
    int ts = 32;
    while (ts > 1 && (bytes(ts) > 140 * 1024 || ts >= 2 * max_q_len || ts * a.dk > PFQ * threads || ts * a.dv > PFV * threads)) ts >>= 1;
    a.ts = ts;
    const size_t lds = bytes(ts);
    if (lds > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)gated_linear_scan_kernel<T, RPL, CPL, MAXT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((gated_linear_scan_kernel<T, RPL, CPL, MAXT>), dim3((unsigned)B, (unsigned)a.H), dim3(threads), lds, st, a);
}

// The shape of the workgroup.  Long runs are a chain of dependent tokens, and what a token costs is the length of a lane's
// own work (its rows' updates and their LDS reads): one column per lane and as many waves as the value width gives (measured
// at dk 64 / dv 128, 4 x 1024 tokens: 0.46 ms per layer against 0.74 with two columns per lane).  A decode step is one token per
// sequence and mostly the state's trip from and to memory: there two columns per lane (half the waves, each read of the q / f
// rows serves two columns) measured 5 % faster, so steps of one or two tokens take that form from 64 value channels on.
template <typename T, int RPL>
void launch_scan(const ScanArgs& a, int64_t B, int64_t max_q_len, hipStream_t st) {
    if constexpr (RPL <= 32) {
        if (a.dv >= 64 && max_q_len <= 2) return launch_scan_as<T, RPL, 2, 512>(a, B, max_q_len, st);
    }
    if constexpr (RPL >= 16) {
        if (4 * ((a.dv + 15) / 16 * 16) <= 512) return launch_scan_as<T, RPL, 1, 512>(a, B, max_q_len, st);
    }
    launch_scan_as<T, RPL, 1, 1024>(a, B, max_q_len, st);
}

template <typename T>
void launch_scan_rows(const ScanArgs& a, int64_t B, int64_t max_q_len, hipStream_t st) {
    if (a.dk <= 16) launch_scan<T, 4>(a, B, max_q_len, st);
    else if (a.dk <= 32) launch_scan<T, 8>(a, B, max_q_len, st);
    else if (a.dk <= 64) launch_scan<T, 16>(a, B, max_q_len, st);
    else if (a.dk <= 128) launch_scan<T, 32>(a, B, max_q_len, st);
    else launch_scan<T, 64>(a, B, max_q_len, st);
}

}  // namespace

extern "C" int tgis_gated_linear_scan(const void* proj, int64_t ld, int64_t q_col0, int64_t f_col0, int64_t v_col0, const float* f_bias,
                                      const float* lower, const float* gain, float* state, const int32_t* state_slots,
                                      const int32_t* cu_seqlens_q, const int32_t* positions, void* out, int64_t ld_out, float out_scale,
                                      int64_t B, int64_t max_q_len, int H, int dk, int dv, float eps, int q_act, int dtype, void* stream) {
    TGIS_CHECK_ARG(proj && gain && state && state_slots && cu_seqlens_q && positions && out, "tgis_gated_linear_scan: null tensor");
    TGIS_CHECK_ARG(H >= 1 && H <= 65535 && dk >= 1 && dk <= 256 && dv >= 1 && dv <= 256, "tgis_gated_linear_scan: heads of up to 256 x 256 (got %d x %d)", dk, dv);
    TGIS_CHECK_ARG(q_col0 >= 0 && f_col0 >= 0 && v_col0 >= 0 && ld >= q_col0 + (int64_t)H * dk && ld >= f_col0 + (int64_t)H * dk &&
                       ld >= v_col0 + (int64_t)H * dv && ld_out >= (int64_t)H * dv && max_q_len >= 1,
                   "tgis_gated_linear_scan: bad strides");
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_gated_linear_scan: bad dtype");
    if (B == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_SCAN, st);
    const ScanArgs a{proj, ld, q_col0, f_col0, v_col0, f_bias, lower, gain, state, state_slots, cu_seqlens_q, positions, out, ld_out, out_scale,
                     H, dk, dv, 0, 0, eps, q_act};
    if (dtype == TGIS_F16) launch_scan_rows<f16>(a, B, max_q_len, st);
    else if (dtype == TGIS_BF16) launch_scan_rows<bf16>(a, B, max_q_len, st);
    else launch_scan_rows<float>(a, B, max_q_len, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
