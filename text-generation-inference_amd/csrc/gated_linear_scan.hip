// Linear attention with a decay per key channel, carried as a matrix state per head:
//
//     S_t = diag(a_t) S_(t-1) + k_t v_t^T                o_t = S_t^T q_t          per head, S [dk, dv] in fp32
//
// in the forms that differ in where a_t and k_t come from (tgis_linear_scan): a bounded sigmoid gate, a sigmoid gate to the power
// 1 / tau, or one constant per head; k a projection of its own (optionally through SiLU) or 1 - a_t; q and v as projected or
// through SiLU, q times a constant; the read-out normed per head or over all heads of a token, times a sigmoid / SiLU gate.
// The first of them, a gated linear recurrence whose forget gate also decides what is written (HGRN2-style):
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
// Workgroup = (sequence, head) = dv_pad x LPC / CPL threads: LPC = 4 or 8 neighbouring lanes share column j of S (and, with
// CPL = 2, column j + dv_pad / 2), lane q of them keeps rows q RPL .. q RPL + RPL - 1 of its columns in registers.  Tokens go through LDS in stages of `ts`: the stage's q and f rows (activated,
// fp32, one padded segment per row group so that the groups' 16-byte reads fall into different banks) and v rows, in two
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
// The logistic function in fp32: with the library's exponential and an IEEE division where the model is served in fp32, with the
// hardware's exponential and reciprocal (a few units in the last place) where the projections it is applied to were rounded to
// two bytes.
template <typename T> __device__ __forceinline__ float sigmoid_as(float z) {
    if (sizeof(T) == 4) return 1.f / (1.f + expf(-z));
    return __builtin_amdgcn_rcpf(1.f + __expf(-z));
}

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
    // with several workgroups per head (grid.z > 1) a workgroup owns dv_pad of the head's value columns and leaves its read-outs
    // unnormed in raw [T][H dv] for head_norm_kernel (a head's norm runs over all its columns)
    float* raw;
    // the general forms: keys of their own at k_col0 (< 0: k = 1 - a); decay_mode 0: a = lower + (1 - lower) sigmoid(f + b),
    // 1: a = sigmoid(f + b)^inv_tau, 2: a = head_decay[h] (no f columns); SiLU on k / v; q times q_scale; an output gate
    // (gate_act 1: sigmoid, 2: SiLU) on columns h dv + c of gate; norm_rows: the norm runs over all heads of a token (raw is set)
    int64_t k_col0 = -1;
    int decay_mode = 0;
    float inv_tau = 1.f;
    const float* head_decay = nullptr;
    int k_act = 0, v_act = 0;
    float q_scale = 1.f;
    const void* gate = nullptr;
    int64_t ld_gate = 0;
    int gate_act = 0;
    int norm_rows = 0;
};

template <typename T> __device__ __forceinline__ float gate_value(const ScanArgs& a, int64_t t, int col) {
    if (!a.gate_act) return 1.f;
    const float g = (float)reinterpret_cast<const T*>(a.gate)[t * a.ld_gate + col];
    const float sg = 1.f / (1.f + expf(-g));
    return a.gate_act == 2 ? g * sg : sg;
}
// ln(sigmoid(z)) without cancellation at either end
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename T, int RPL, int CPL, int LPC, int MAXT, bool KEYS>
__global__ __launch_bounds__(MAXT) void gated_linear_scan_kernel(ScanArgs a) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    constexpr int SEG = RPL + SEG_PAD, ROW = LPC * SEG;
    const int ts = a.ts, dk = a.dk, dv = a.dv, dv_pad = a.dv_pad;
    float* qs = smem;                        // [2][ts][ROW]
    float* fs = qs + 2 * ts * ROW;           // [2][ts][ROW]
    float* vs = fs + 2 * ts * ROW;           // [2][ts][dv_pad]
    float* os = vs + 2 * ts * dv_pad;        // [ts][dv_pad]
    float* ks = os + ts * dv_pad;            // [2][ts][ROW], keys of their own only
    const int b = blockIdx.x, h = blockIdx.y;
    const int col0 = blockIdx.z * dv_pad;  // this workgroup's first value column
    const int tid = threadIdx.x, j = tid / LPC, qd = tid % LPC;  // LPC neighbouring lanes share a column
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
            const int i = qd * RPL + r, jc = col0 + j + c * jstep;
            s[c][r] = (!fresh && i < dk && jc < dv) ? S[(int64_t)i * dv + jc] : 0.f;
        }
    // rows past dk and columns past dv of both buffers: f = 1, q = 0, v = 0 (their state stays zero and is never read)
    for (int e = tid; e < 2 * ts * ROW; e += nthreads) {
        qs[e] = 0.f;
        fs[e] = 1.f;
        if (KEYS) ks[e] = 0.f;
    }
    for (int e = tid; e < 2 * ts * dv_pad; e += nthreads) vs[e] = 0.f;
    // A thread's share of a stage is the same in every stage — elements tid + u nthreads of the stage's [token][channel] grids — so
    // where they come from and go to is worked out once: token within the stage, offsets into the projections and the buffers,
    // the gate's bias and lower bound.
    T qr[PFQ], fr[PFQ], vr[PFV], kr[PFQ];
    int q_tt[PFQ], q_src[PFQ], q_dst[PFQ], v_tt[PFV], v_src[PFV];
    float q_fb[PFQ], q_lo[PFQ];
#pragma unroll
    for (int u = 0; u < PFQ; ++u) {
        const int e = tid + u * nthreads;
        const int tt = e / dk, i = e - tt * dk;
        q_tt[u] = tt;
        q_src[u] = tt * (int)a.ld + h * dk + i;
        q_dst[u] = tt * ROW + (i / RPL) * SEG + (i % RPL);
        q_fb[u] = a.f_bias ? a.f_bias[h * dk + i] : 0.f;
        q_lo[u] = a.lower ? a.lower[h * dk + i] : 0.f;
        if (a.decay_mode == 2) q_lo[u] = a.head_decay[h];
    }
#pragma unroll
    for (int u = 0; u < PFV; ++u) {
        const int e = tid + u * nthreads;
        const int tt = e / dv_pad, c = col0 + e - tt * dv_pad;
        v_tt[u] = c < dv ? tt : 1 << 30;  // a column past the head's width is never fetched (its buffer entry stays zero)
        v_src[u] = tt * (int)a.ld + h * dv + c;
    }
    // tokens [first, first + n) of the sequence: this thread's share of their projections, as they are
    auto fetch = [&](int first, int n) {
        const T* base = proj + (int64_t)(t0 + first) * a.ld;
#pragma unroll
        for (int u = 0; u < PFQ; ++u)
            if (q_tt[u] < n) {
                qr[u] = base[a.q_col0 + q_src[u]];
                if (a.decay_mode != 2) fr[u] = base[a.f_col0 + q_src[u]];
                if (KEYS) kr[u] = base[a.k_col0 + q_src[u]];
            }
#pragma unroll
        for (int u = 0; u < PFV; ++u)
            if (v_tt[u] < n) vr[u] = base[a.v_col0 + v_src[u]];
    };
    // ... activated and stored into one stage buffer
    auto commit = [&](int n, float* qb, float* fb, float* vb, float* kb) {
#pragma unroll
        for (int u = 0; u < PFQ; ++u)
            if (q_tt[u] < n) {
                float qv = (float)qr[u];
                if (a.q_act) qv = qv * sigmoid_as<T>(qv);
                qb[q_dst[u]] = qv * a.q_scale;
                if (a.decay_mode == 0) fb[q_dst[u]] = q_lo[u] + (1.f - q_lo[u]) * sigmoid_as<T>((float)fr[u] + q_fb[u]);
                else if (a.decay_mode == 1) fb[q_dst[u]] = expf(a.inv_tau * log_sigmoid((float)fr[u] + q_fb[u]));
                else fb[q_dst[u]] = q_lo[u];
                if (KEYS) {
                    float kv = (float)kr[u];
                    if (a.k_act) kv = kv * sigmoid_as<T>(kv);
                    kb[q_dst[u]] = kv;
                }
            }
#pragma unroll
        for (int u = 0; u < PFV; ++u)
            if (v_tt[u] < n) {
                float vv = (float)vr[u];
                if (a.v_act) vv = vv * sigmoid_as<T>(vv);
                vb[tid + u * nthreads] = vv;
            }
    };
    fetch(0, min(ts, qlen));
    __syncthreads();  // the buffers are filled with their neutral values
    commit(min(ts, qlen), qs, fs, vs, ks);
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
        const float* kb = ks + buf * ts * ROW + qd * SEG;
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
                f32x4 k4;
                if (KEYS) k4 = *reinterpret_cast<const f32x4*>(kb + tt * ROW + r4);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const float g = KEYS ? k4[u] : 1.f - f4[u];
#pragma unroll
                    for (int c = 0; c < CPL; ++c) {
                        s[c][r4 + u] = fmaf(f4[u], s[c][r4 + u], g * vj[c]);
                        acc[c] = fmaf(s[c][r4 + u], q4[u], acc[c]);
                    }
                }
            }
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                // the sum over the column's lanes, by data-parallel-primitive moves (no trip through LDS)
                float t = acc[c];
                t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0xB1, 0xF, 0xF, true));  // lane ^ 1
                t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x4E, 0xF, 0xF, true));  // lane ^ 2
                if (LPC == 8)  // the other quad of the eight: lane 7 - i of the half row holds its total
                    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x141, 0xF, 0xF, true));
                if (qd == 0) os[tt * dv_pad + j + c * jstep] = t;
            }
        }
        __syncthreads();
        for (int tt = wave; tt < n; tt += nw) {
            if (a.raw) {
                float* rrow = a.raw + ((int64_t)(t0 + base + tt) * a.H + h) * dv + col0;
                for (int c = lane; c < dv_pad && col0 + c < dv; c += 64) rrow[c] = os[tt * dv_pad + c];
                continue;
            }
            float ss = 0.f;
            for (int c = lane; c < dv; c += 64) {
                const float o = os[tt * dv_pad + c];
                ss += o * o;
            }
            ss = wave_sum(ss);
            const float rinv = a.out_scale / sqrtf(ss / (float)dv + a.eps);
            T* orow = out + (int64_t)(t0 + base + tt) * a.ld_out + (int64_t)h * dv;
            for (int c = lane; c < dv; c += 64)
                orow[c] = (T)(os[tt * dv_pad + c] * rinv * a.gain[c] * gate_value<T>(a, t0 + base + tt, h * dv + c));
        }
        if (n_next > 0)
            commit(n_next, qs + (buf ^ 1) * ts * ROW, fs + (buf ^ 1) * ts * ROW, vs + (buf ^ 1) * ts * dv_pad, ks + (buf ^ 1) * ts * ROW);
        __syncthreads();  // the outputs are out, the next stage is in
    }
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            const int i = qd * RPL + r, jc = col0 + j + c * jstep;
            if (i < dk && jc < dv) S[(int64_t)i * dv + jc] = s[c][r];
        }
}

// out[t][h][:] = raw[t][h][:] / sqrt(mean(raw[t][h]^2) + eps) * gain * out_scale: the heads' norm after a scan whose workgroups each
// held a part of a head's columns.  grid (token, ceil(H / 4)): a wave per head.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_kernel(const float* __restrict__ raw, const float* __restrict__ gain, T* __restrict__ out,
                                                        int64_t ld_out, float out_scale, int H, int dv, float eps, ScanArgs a) {
    const int64_t t = blockIdx.x;
    const int h = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (h >= H) return;
    const float* r = raw + (t * H + h) * dv;
    float v[4], ss = 0.f;  // dv <= 256
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[i] = lane + 64 * i < dv ? r[lane + 64 * i] : 0.f;
        ss += v[i] * v[i];
    }
    ss = wave_sum(ss);
    const float rinv = out_scale / sqrtf(ss / (float)dv + eps);
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (lane + 64 * i < dv)
            out[t * ld_out + (int64_t)h * dv + lane + 64 * i] = (T)(v[i] * rinv * gain[lane + 64 * i] * gate_value<T>(a, t, h * dv + lane + 64 * i));
}

// out[t][:] = raw[t][:] / sqrt(mean over all H dv channels of raw[t]^2 + eps) * gain[H dv] * gate * out_scale: the norm of designs
// that norm a token's heads together.  grid (token): the row is walked twice (it is in the cache the second time).
template <typename T>
__global__ __launch_bounds__(256) void row_norm_kernel(const float* __restrict__ raw, const float* __restrict__ gain, T* __restrict__ out,
                                                       int64_t ld_out, float out_scale, int C, float eps, ScanArgs a) {
    __shared__ float part[4];
    const int64_t t = blockIdx.x;
    const float* r = raw + t * C;
    float ss = 0.f;
    for (int c = threadIdx.x; c < C; c += 256) ss += r[c] * r[c];
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = part[0] + part[1] + part[2] + part[3];
    const float rinv = out_scale / sqrtf(ss / (float)C + eps);
    for (int c = threadIdx.x; c < C; c += 256) out[t * ld_out + c] = (T)(r[c] * rinv * gain[c] * gate_value<T>(a, t, c));
}

// cols: value columns per workgroup (a multiple of 16 CPL; the head's padded width when a workgroup holds the whole head)
template <typename T, int RPL, int CPL, int LPC, int MAXT, bool KEYS>
void launch_scan_keys(ScanArgs a, int64_t B, int64_t max_q_len, int cols, int col_split, int64_t T_total, hipStream_t st) {
    a.dv_pad = cols;
    if (col_split <= 1 && !a.norm_rows) a.raw = nullptr;
    const int threads = LPC * a.dv_pad / CPL;
    // tokens per stage: a power of two up to 32 that a thread's registers can prefetch, that 140 KiB of LDS hold (two input
    // buffers and the outputs), and no more than the longest run needs
    auto bytes = [&](int ts) { return ((size_t)(KEYS ? 6 : 4) * ts * LPC * (RPL + SEG_PAD) + (size_t)3 * ts * a.dv_pad) * sizeof(float); };
    int ts = 32;
    while (ts > 1 && (bytes(ts) > 140 * 1024 || ts >= 2 * max_q_len || ts * a.dk > PFQ * threads || ts * a.dv_pad > PFV * threads)) ts >>= 1;
    a.ts = ts;
    const size_t lds = bytes(ts);
    if (lds > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)gated_linear_scan_kernel<T, RPL, CPL, LPC, MAXT, KEYS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((gated_linear_scan_kernel<T, RPL, CPL, LPC, MAXT, KEYS>), dim3((unsigned)B, (unsigned)a.H, (unsigned)std::max(col_split, 1)),
                       dim3(threads), lds, st, a);
    if (a.raw && a.norm_rows)
        hipLaunchKernelGGL(row_norm_kernel<T>, dim3((unsigned)T_total), dim3(256), 0, st, a.raw, a.gain, (T*)a.out, a.ld_out, a.out_scale,
                           a.H * a.dv, a.eps, a);
    else if (a.raw)
        hipLaunchKernelGGL(head_norm_kernel<T>, dim3((unsigned)T_total, (unsigned)((a.H + 3) / 4)), dim3(256), 0, st, a.raw, a.gain, (T*)a.out,
                           a.ld_out, a.out_scale, a.H, a.dv, a.eps, a);
}

template <typename T, int RPL, int CPL, int LPC, int MAXT>
void launch_scan_as(const ScanArgs& a, int64_t B, int64_t max_q_len, int cols, int col_split, int64_t T_total, hipStream_t st) {
    if (a.k_col0 >= 0) launch_scan_keys<T, RPL, CPL, LPC, MAXT, true>(a, B, max_q_len, cols, col_split, T_total, st);
    else launch_scan_keys<T, RPL, CPL, LPC, MAXT, false>(a, B, max_q_len, cols, col_split, T_total, st);
}

// The shape of the workgroup.  Long runs are a chain of dependent tokens; what a token costs is a wave's instructions for its
// share of the dk dv updates (four cycles each on a 16-lane SIMD) plus its share of activating the stage.  So runs of more than
// two tokens spread a column over EIGHT lanes where the value width leaves room for it (8 dv <= 1024 threads), else over four;
// and when the caller gave scratch memory, value heads wider than 64 are dealt to workgroups of 64 columns — columns are
// independent until the head's norm, which then runs as a pass of its own over the unnormed read-outs.  Measured at dk 64 /
// dv 128, 4 x 1024 tokens, per layer: 0.46 ms with four lanes per column, 0.38 with eight, 0.24 with eight and two workgroups
// of 64 columns (0.28 with four of 32: every workgroup activates the whole head's q and f rows).  A decode step is one token
// per sequence and mostly the state's trip from and to memory: there four lanes per column with two columns per lane (half the
// waves, each read of the q / f rows serves two columns) measured 5 % faster, so steps of one or two tokens take that form from
// 64 value channels on.
// R4: rows per lane with four lanes per column (a multiple of four, >= dk / 4); eight lanes take half of that.
template <typename T, int R4>
void launch_scan(const ScanArgs& a, int64_t B, int64_t max_q_len, int64_t T_total, hipStream_t st) {
    const int pad16 = (a.dv + 15) / 16 * 16;
    if constexpr (R4 <= 32) {
        if (a.dv >= 64 && max_q_len <= 2) return launch_scan_as<T, R4, 2, 4, 512>(a, B, max_q_len, (a.dv + 31) / 32 * 32, 1, T_total, st);
    }
    if constexpr (R4 >= 8) {
        if (max_q_len > 2 && a.raw && a.dv > 64 && B * a.H * ((a.dv + 63) / 64) <= 512)
            return launch_scan_as<T, R4 / 2, 1, 8, 1024>(a, B, max_q_len, 64, (a.dv + 63) / 64, T_total, st);
        if (max_q_len > 2 && 8 * pad16 <= 1024) return launch_scan_as<T, R4 / 2, 1, 8, 1024>(a, B, max_q_len, pad16, 1, T_total, st);
    }
    if constexpr (R4 >= 16) {
        if (4 * pad16 <= 512) return launch_scan_as<T, R4, 1, 4, 512>(a, B, max_q_len, pad16, 1, T_total, st);
    }
    launch_scan_as<T, R4, 1, 4, 1024>(a, B, max_q_len, pad16, 1, T_total, st);
}

template <typename T>
void launch_scan_rows(const ScanArgs& a, int64_t B, int64_t max_q_len, int64_t T_total, hipStream_t st) {
    if (a.dk <= 16) launch_scan<T, 4>(a, B, max_q_len, T_total, st);
    else if (a.dk <= 32) launch_scan<T, 8>(a, B, max_q_len, T_total, st);
    else if (a.dk <= 64) launch_scan<T, 16>(a, B, max_q_len, T_total, st);
    else if (a.dk <= 128) launch_scan<T, 32>(a, B, max_q_len, T_total, st);
    else launch_scan<T, 64>(a, B, max_q_len, T_total, st);
}

}  // namespace

extern "C" int tgis_gated_linear_scan(const void* proj, int64_t ld, int64_t q_col0, int64_t f_col0, int64_t v_col0, const float* f_bias,
                                      const float* lower, const float* gain, float* state, const int32_t* state_slots,
                                      const int32_t* cu_seqlens_q, const int32_t* positions, void* out, int64_t ld_out, float out_scale,
                                      int64_t B, int64_t T, int64_t max_q_len, int H, int dk, int dv, float eps, int q_act, float* scratch,
                                      int dtype, void* stream) {
    TGIS_CHECK_ARG(proj && gain && state && state_slots && cu_seqlens_q && positions && out, "tgis_gated_linear_scan: null tensor");
    TGIS_CHECK_ARG(H >= 1 && H <= 65535 && dk >= 1 && dk <= 256 && dv >= 1 && dv <= 256, "tgis_gated_linear_scan: heads of up to 256 x 256 (got %d x %d)", dk, dv);
    TGIS_CHECK_ARG(q_col0 >= 0 && f_col0 >= 0 && v_col0 >= 0 && ld >= q_col0 + (int64_t)H * dk && ld >= f_col0 + (int64_t)H * dk &&
                       ld >= v_col0 + (int64_t)H * dv && ld_out >= (int64_t)H * dv && max_q_len >= 1 && T >= 0,
                   "tgis_gated_linear_scan: bad strides");
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_gated_linear_scan: bad dtype");
    if (B == 0 || T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_SCAN, st);
    const ScanArgs a{proj, ld, q_col0, f_col0, v_col0, f_bias, lower, gain, state, state_slots, cu_seqlens_q, positions, out, ld_out, out_scale,
                     H, dk, dv, 0, 0, eps, q_act, scratch};
    if (dtype == TGIS_F16) launch_scan_rows<f16>(a, B, max_q_len, T, st);
    else if (dtype == TGIS_BF16) launch_scan_rows<bf16>(a, B, max_q_len, T, st);
    else launch_scan_rows<float>(a, B, max_q_len, T, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// The general forms (see the head of this file).  decay_mode 0 / 1 read gate pre-activations at f_col0 (+ f_bias), 2 takes
// head_decay [H]; k_col0 < 0: k = 1 - a.  norm_rows != 0: gain is [H dv] and the norm runs over all heads of a token (scratch
// [T][H dv] floats is then required); else gain is [dv], shared by the heads.  gate (optional): [T][>= H dv] in the activation
// dtype, gate_act 1: sigmoid, 2: SiLU.
extern "C" int tgis_linear_scan(const void* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t f_col0, int64_t v_col0,
                                const float* f_bias, const float* lower, const float* head_decay, int decay_mode, float inv_tau,
                                int q_act, int k_act, int v_act, float q_scale, const float* gain, int norm_rows, const void* gate,
                                int64_t ld_gate, int gate_act, float* state, const int32_t* state_slots, const int32_t* cu_seqlens_q,
                                const int32_t* positions, void* out, int64_t ld_out, float out_scale, int64_t B, int64_t T,
                                int64_t max_q_len, int H, int dk, int dv, float eps, float* scratch, int dtype, void* stream) {
    TGIS_CHECK_ARG(proj && gain && state && state_slots && cu_seqlens_q && positions && out, "tgis_linear_scan: null tensor");
    TGIS_CHECK_ARG(H >= 1 && H <= 65535 && dk >= 1 && dk <= 256 && dv >= 1 && dv <= 256, "tgis_linear_scan: heads of up to 256 x 256 (got %d x %d)", dk, dv);
    TGIS_CHECK_ARG(decay_mode >= 0 && decay_mode <= 2 && (decay_mode != 2 || head_decay) && (decay_mode == 2 || f_col0 >= 0),
                   "tgis_linear_scan: decay mode %d without its operand", decay_mode);
    TGIS_CHECK_ARG(q_col0 >= 0 && v_col0 >= 0 && ld >= q_col0 + (int64_t)H * dk && (decay_mode == 2 || ld >= f_col0 + (int64_t)H * dk) &&
                       (k_col0 < 0 || ld >= k_col0 + (int64_t)H * dk) && ld >= v_col0 + (int64_t)H * dv && ld_out >= (int64_t)H * dv &&
                       max_q_len >= 1 && T >= 0,
                   "tgis_linear_scan: bad strides");
    TGIS_CHECK_ARG(!gate_act || (gate && ld_gate >= (int64_t)H * dv && gate_act <= 2), "tgis_linear_scan: bad gate");
    TGIS_CHECK_ARG(!norm_rows || scratch, "tgis_linear_scan: a norm over all heads needs scratch memory");
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_linear_scan: bad dtype");
    if (B == 0 || T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_SCAN, st);
    ScanArgs a{proj, ld, q_col0, f_col0, v_col0, f_bias, lower, gain, state, state_slots, cu_seqlens_q, positions, out, ld_out, out_scale,
               H, dk, dv, 0, 0, eps, q_act, scratch};
    a.k_col0 = k_col0;
    a.decay_mode = decay_mode;
    a.inv_tau = inv_tau;
    a.head_decay = head_decay;
    a.k_act = k_act;
    a.v_act = v_act;
    a.q_scale = q_scale;
    a.gate = gate_act ? gate : nullptr;
    a.ld_gate = ld_gate;
    a.gate_act = gate_act;
    a.norm_rows = norm_rows;
    if (dtype == TGIS_F16) launch_scan_rows<f16>(a, B, max_q_len, T, st);
    else if (dtype == TGIS_BF16) launch_scan_rows<bf16>(a, B, max_q_len, T, st);
    else launch_scan_rows<float>(a, B, max_q_len, T, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
