// Selective state-space scan (Mamba's recurrence) for ragged steps.  Per sequence, channel c and state n, tokens in order:
//
//     dt_c  = softplus(dtp[t][c] + dt_bias[c])                          step size, fp32
//     S[c][n] <- exp(dt_c A[c][n]) S[c][n] + dt_c x[t][c] B[t][n]       A = -exp(A_log), fp32 state
//     y[t][c] = sum_n S[c][n] C[t][n] + D[c] x[t][c];    out[t][c] = y silu(z[t][c])
//
// x is the activated output of the channel convolution, B and C one row per token shared by all channels, dtp the step-size
// projection before its bias.  The state [inner][N] of a sequence lives in a slot (fp32), is read when the step does not start
// at position 0 and written back.
//
// Workgroup = (sequence, CW = threads / L channels; 64 .. 256 threads, fewer when the step has few sequences): L neighbouring
// lanes share a channel, lane l of them keeps states l SPT .. l SPT + SPT - 1 in registers (L a power of two, SPT = 1, 2, 4 or 8:
// as few states per lane as it takes to give every SIMD several waves).  Tokens go through LDS in stages of TS: the
// stage's B | C rows and the channels' step sizes and inputs (softplus applied once per (token, channel), not per state), then a
// sequential walk over the stage (stages of 16 .. 64 tokens by the longest run) with the read-out summed over the channel's lanes by shuffles; the stage's outputs leave
// together, gated, with neighbouring lanes on neighbouring channels.
#include "common.h"

namespace {

constexpr int MAX_SPT = 8;  // states a lane keeps at most

struct SelArgs {
    const void* x;
    int64_t ld_x;
    const void* dtp;
    int64_t ld_dt;
    int dt_f32;
    const float* dt_bias;
    const void* bc;
    int64_t ld_bc, b_col0, c_col0;
    const void* z;
    int64_t ld_z;
    const float* A_log;
    const float* D;
    float* state;
    const int32_t* state_slots;
    const int32_t* cu_q;
    const int32_t* positions;
    void* out;
    int64_t ld_out;
    int inner, N, L, ts, log_cw, log_np;
};

__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }
// e^(d a) per state and token is what the walk spends its time on: where the model is served in two bytes it is the hardware's
// base-two exponential (a few units in the last place of fp32) on a transition that was scaled by log2(e) once; fp32 serving
// takes the library's.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <typename T> __device__ __forceinline__ float decay_of(float d, float a) {
    if (sizeof(T) == 4) return expf(d * a);
    return __builtin_amdgcn_exp2f(d * a);
}

// SPT: states per lane (1, 2, 4 or 8); L = the channel's lanes, a power of two with L SPT >= N
template <typename T, int SPT>
__global__ __launch_bounds__(256) void selective_scan_kernel(SelArgs a) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int N = a.N, L = a.L, NT = blockDim.x, CW = NT / L, TS = a.ts;
    const int Np = L * SPT;
    float* Bs = smem;                 // [TS][Np]
    float* Cs = Bs + TS * Np;         // [TS][Np]
    float* dts = Cs + TS * Np;        // [TS][CW]
    float* xs = dts + TS * CW;        // [TS][CW]
    float* ys = xs + TS * CW;         // [TS][CW]
    const int b = blockIdx.x, tid = threadIdx.x;
    const int ch = tid / L, l = tid % L;
    const int c = blockIdx.y * CW + ch;
    const int t0 = a.cu_q[b], qlen = a.cu_q[b + 1] - t0;
    if (qlen <= 0) return;
    const bool fresh = a.positions[t0] == 0;
    const bool live = c < a.inner;
    float* S = a.state + ((int64_t)a.state_slots[b] * a.inner + (live ? c : 0)) * N;
    float s[SPT], A[SPT];
#pragma unroll
    for (int r = 0; r < SPT; ++r) {
        const int n = l * SPT + r;
        const bool ok = live && n < N;
        s[r] = (ok && !fresh) ? S[n] : 0.f;
        A[r] = ok ? -expf(a.A_log[(int64_t)c * N + n]) * (sizeof(T) == 4 ? 1.f : 1.4426950408889634f) : 0.f;
    }
    const float Dc = live ? a.D[c] : 0.f;
    const T* x = reinterpret_cast<const T*>(a.x);
    const T* bc = reinterpret_cast<const T*>(a.bc);
    const T* z = reinterpret_cast<const T*>(a.z);
    T* out = reinterpret_cast<T*>(a.out);
    for (int base = 0; base < qlen; base += TS) {
        const int n_t = min(TS, qlen - base);
        for (int e = tid; e < n_t * Np; e += NT) {
            const int tt = e >> a.log_np, n = e & (Np - 1);
            const T* row = bc + (int64_t)(t0 + base + tt) * a.ld_bc;
            Bs[e] = n < N ? (float)row[a.b_col0 + n] : 0.f;
            Cs[e] = n < N ? (float)row[a.c_col0 + n] : 0.f;
        }
        for (int e = tid; e < n_t * CW; e += NT) {
            const int tt = e >> a.log_cw, cc = blockIdx.y * CW + (e & (CW - 1));
            float d = 0.f, xv = 0.f;
            if (cc < a.inner) {
                const int64_t t = t0 + base + tt;
                const float pre = a.dt_f32 ? reinterpret_cast<const float*>(a.dtp)[t * a.ld_dt + cc] : (float)reinterpret_cast<const T*>(a.dtp)[t * a.ld_dt + cc];
                d = softplus_f32(pre + a.dt_bias[cc]);
                xv = (float)x[t * a.ld_x + cc];
            }
            dts[e] = d;
            xs[e] = xv;
        }
        __syncthreads();
        for (int tt = 0; tt < n_t; ++tt) {
            const float d = dts[tt * CW + ch], xv = xs[tt * CW + ch];
            const float dx = d * xv;
            const float* Br = Bs + tt * Np + l * SPT;
            const float* Cr = Cs + tt * Np + l * SPT;
            float y = 0.f;
            if constexpr (SPT % 4 == 0) {
#pragma unroll
                for (int r4 = 0; r4 < SPT; r4 += 4) {
                    const f32x4 b4 = *reinterpret_cast<const f32x4*>(Br + r4);
                    const f32x4 c4 = *reinterpret_cast<const f32x4*>(Cr + r4);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        s[r4 + u] = fmaf(decay_of<T>(d, A[r4 + u]), s[r4 + u], dx * b4[u]);
                        y = fmaf(s[r4 + u], c4[u], y);
                    }
                }
            } else {
#pragma unroll
                for (int r = 0; r < SPT; ++r) {
                    s[r] = fmaf(decay_of<T>(d, A[r]), s[r], dx * Br[r]);
                    y = fmaf(s[r], Cr[r], y);
                }
            }
            // the channel's lanes add up: neighbours, pairs, the other quad of eight and the other half of sixteen by
            // data-parallel-primitive moves (no trip through LDS), wider groups by shuffles
            if (L >= 2) y += dpp_move<0xB1>(y);
            if (L >= 4) y += dpp_move<0x4E>(y);
            if (L >= 8) y += dpp_move<0x141>(y);
            if (L >= 16) y += dpp_move<0x140>(y);
            for (int o = 16; o < L; o <<= 1) y += __shfl_xor(y, o, 64);
            if (l == 0) ys[tt * CW + ch] = fmaf(Dc, xv, y);
        }
        __syncthreads();
        for (int e = tid; e < n_t * CW; e += NT) {
            const int tt = e >> a.log_cw, cc = blockIdx.y * CW + (e & (CW - 1));
            if (cc < a.inner) {
                const int64_t t = t0 + base + tt;
                const float g = (float)z[t * a.ld_z + cc];
                out[t * a.ld_out + cc] = (T)(ys[e] * g / (1.f + expf(-g)));
            }
        }
        __syncthreads();
    }
    if (live)
#pragma unroll
        for (int r = 0; r < SPT; ++r) {
            const int n = l * SPT + r;
            if (n < N) S[n] = s[r];
        }
}

}  // namespace

extern "C" int tgis_selective_scan(const void* x, int64_t ld_x, const void* dt, int64_t ld_dt, int dt_f32, const float* dt_bias,
                                   const void* bc, int64_t ld_bc, int64_t b_col0, int64_t c_col0, const void* z, int64_t ld_z,
                                   const float* A_log, const float* D, float* state, const int32_t* state_slots,
                                   const int32_t* cu_seqlens_q, const int32_t* positions, void* out, int64_t ld_out, int64_t B,
                                   int64_t max_q_len, int64_t inner, int N, int dtype, void* stream) {
    TGIS_CHECK_ARG(x && dt && dt_bias && bc && z && A_log && D && state && state_slots && cu_seqlens_q && positions && out,
                   "tgis_selective_scan: null tensor");
    TGIS_CHECK_ARG(inner >= 1 && N >= 1 && N <= 16 * MAX_SPT && ld_x >= inner && ld_dt >= inner && ld_z >= inner && ld_out >= inner &&
                       b_col0 >= 0 && c_col0 >= 0 && ld_bc >= b_col0 + N && ld_bc >= c_col0 + N,
                   "tgis_selective_scan: bad arguments (inner %ld, states %d: up to %d)", (long)inner, N, 16 * MAX_SPT);
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_selective_scan: bad dtype");
    if (B == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_SCAN, st);
    // Lanes per channel.  A step's parallelism is sequences x channels x lanes per channel; a lane's walk is a chain of
    // dependent instructions, so a lane keeps 8 states only when that still leaves every SIMD several waves, and fewer (down to
    // one state per lane, 16 .. 64 lanes per channel reduced by shuffles) otherwise.
    auto lanes_for = [&](int spt) {
        int L = 1;
        while (L * spt < N) L <<= 1;
        return L;
    };
    int spt = MAX_SPT;
    while (spt > 1 && lanes_for(spt) < 64 && B * inner * lanes_for(spt) < (int64_t)8192 * 64) spt >>= 1;
    if (lanes_for(spt) > 64) spt = (N + 63) / 64 <= 2 ? 2 : ((N + 63) / 64 <= 4 ? 4 : 8);
    const int L = lanes_for(spt);
    int threads = 256;
    while (threads > 64 && threads / 2 >= L && B * cdiv64(inner, threads / L) < 512) threads >>= 1;
    const int CW = threads / L;
    int log_cw = 0, log_np = 0;
    while ((1 << log_cw) < CW) ++log_cw;
    while ((1 << log_np) < L * spt) ++log_np;
    // tokens per stage: every stage costs its trips to memory whatever it holds
    int TS = 32;
    while (TS > 16 && TS >= 2 * max_q_len) TS >>= 1;
    const SelArgs a{x, ld_x, dt, ld_dt, dt_f32, dt_bias, bc, ld_bc, b_col0, c_col0, z, ld_z, A_log, D, state, state_slots, cu_seqlens_q,
                    positions, out, ld_out, (int)inner, N, L, TS, log_cw, log_np};
    const size_t lds = ((size_t)2 * TS * L * spt + (size_t)3 * TS * CW) * sizeof(float);
    const dim3 grid((unsigned)B, (unsigned)cdiv64(inner, CW));
#define LAUNCH_SPT(TT)                                                                                        \
    do {                                                                                                      \
        if (spt == 8) hipLaunchKernelGGL((selective_scan_kernel<TT, 8>), grid, dim3(threads), lds, st, a);      \
        else if (spt == 4) hipLaunchKernelGGL((selective_scan_kernel<TT, 4>), grid, dim3(threads), lds, st, a); \
        else if (spt == 2) hipLaunchKernelGGL((selective_scan_kernel<TT, 2>), grid, dim3(threads), lds, st, a); \
        else hipLaunchKernelGGL((selective_scan_kernel<TT, 1>), grid, dim3(threads), lds, st, a);               \
    } while (0)
    if (dtype == TGIS_F16) LAUNCH_SPT(f16);
    else if (dtype == TGIS_BF16) LAUNCH_SPT(bf16);
    else LAUNCH_SPT(float);
#undef LAUNCH_SPT
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
