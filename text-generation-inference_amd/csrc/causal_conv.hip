// Short causal convolutions over time, one filter per channel, for ragged steps:
//
//     y[t][c] = act( bias[c] + sum_{j < taps} w[c][j] x[t - (taps - 1 - j)][c] )  (+ x[t][c] when `residual`)
//
// The last column of w meets the current token.  Inputs before a step's first token come from the sequence's tail
// ([taps - 1][C] fp32 in a state slot: the inputs at the positions just before the step), zeros when the step starts at
// position 0.  Up to two filter sets read the same input in one launch (two sublayers that each see the input through a
// convolution of their own); the tail is the input's, so they share it.  The launch also moves the tail on: the thread that
// reads a channel's old tail (the one that owns the run's first tokens) is the one that writes its new tail, after it has read.
//
// grid (sequence, run of RUN tokens, 256 channels): a thread walks its run in order with the last taps - 1 inputs in registers,
// so every input is loaded once per set of taps and neighbouring lanes read neighbouring channels.
#include "common.h"

namespace {

constexpr int RUN = 16;

struct ConvArgs {
    const void* x;
    int64_t ld_x;
    const float* w;     // [sets][C][taps]
    const float* bias;  // [sets][C] or null
    float* tail;        // slot s at tail + s * tail_stride: [taps - 1][C]
    int64_t tail_stride;
    const int32_t* state_slots;
    const int32_t* cu_q;
    const int32_t* positions;
    void* out;          // set s at out + s * set_stride (elements)
    int64_t ld_out, set_stride;
    int C, taps, sets, act, residual;
};

// XT: input type, OT: output type, MT: taps - 1 rounded up (registers for the lags), SETS: filter sets
template <typename XT, typename OT, int MT, int SETS>
__global__ __launch_bounds__(256) void causal_conv_kernel(ConvArgs a) {
    const int b = blockIdx.x, c = blockIdx.z * 256 + threadIdx.x;
    const int t0 = a.cu_q[b], n = a.cu_q[b + 1] - t0;
    const int first = blockIdx.y * RUN;
    if (c >= a.C || first >= n) return;
    const int cnt = min(RUN, n - first), taps = a.taps, C = a.C;
    const bool fresh = a.positions[t0] == 0;
    const XT* x = reinterpret_cast<const XT*>(a.x) + (int64_t)t0 * a.ld_x + c;
    float* tail = a.tail + (int64_t)a.state_slots[b] * a.tail_stride + c;
    // lag[k]: the input k + 1 tokens before the current one; wl[s][k] its weight
    float lag[MT], wl[SETS][MT], w0[SETS], bs[SETS];
#pragma unroll
    for (int k = 0; k < MT; ++k) {
        const int idx = first - 1 - k;
        lag[k] = 0.f;
        if (k < taps - 1) {
            if (idx >= 0) lag[k] = (float)x[(int64_t)idx * a.ld_x];
            else if (!fresh) lag[k] = tail[(int64_t)(taps - 1 + idx) * C];
        }
#pragma unroll
        for (int s = 0; s < SETS; ++s) wl[s][k] = k < taps - 1 ? a.w[((int64_t)s * C + c) * taps + taps - 2 - k] : 0.f;
    }
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
        w0[s] = a.w[((int64_t)s * C + c) * taps + taps - 1];
        bs[s] = a.bias ? a.bias[(int64_t)s * C + c] : 0.f;
    }
    if (first == 0) {
        // the new tail: inputs at the step's last taps - 1 positions; those before the step are rows of the old tail (row n + r
        // moves to row r: ascending r never overwrites a row that is still to be read)
        for (int r = 0; r < taps - 1; ++r) {
            const int idx = n - (taps - 1) + r;
            float v = 0.f;
            if (idx >= 0) v = (float)x[(int64_t)idx * a.ld_x];
            else if (!fresh) v = tail[(int64_t)(n + r) * C];
            tail[(int64_t)r * C] = v;
        }
    }
    OT* out = reinterpret_cast<OT*>(a.out) + (int64_t)(t0 + first) * a.ld_out + c;
    for (int i = 0; i < cnt; ++i) {
        const float cur = (float)x[(int64_t)(first + i) * a.ld_x];
#pragma unroll
        for (int s = 0; s < SETS; ++s) {
            float y = fmaf(w0[s], cur, bs[s]);
#pragma unroll
            for (int k = 0; k < MT; ++k) y = fmaf(wl[s][k], lag[k], y);
            if (a.act) y = y / (1.f + expf(-y));
            if (a.residual) y += cur;
            out[(int64_t)s * a.set_stride + (int64_t)i * a.ld_out] = (OT)y;
        }
#pragma unroll
        for (int k = MT - 1; k > 0; --k) lag[k] = lag[k - 1];
        if (MT > 0) lag[0] = cur;
    }
}

template <typename XT, typename OT, int MT>
void launch_sets(const ConvArgs& a, dim3 grid, hipStream_t st) {
    if (a.sets == 1) hipLaunchKernelGGL((causal_conv_kernel<XT, OT, MT, 1>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((causal_conv_kernel<XT, OT, MT, 2>), grid, dim3(256), 0, st, a);
}

template <typename XT, typename OT>
void launch_taps(const ConvArgs& a, dim3 grid, hipStream_t st) {
    if (a.taps <= 4) launch_sets<XT, OT, 3>(a, grid, st);
    else if (a.taps <= 8) launch_sets<XT, OT, 7>(a, grid, st);
    else launch_sets<XT, OT, 15>(a, grid, st);
}

template <typename OT>
void launch_in(const ConvArgs& a, int x_f32, dim3 grid, hipStream_t st) {
    if (x_f32) launch_taps<float, OT>(a, grid, st);
    else launch_taps<OT, OT>(a, grid, st);
}

}  // namespace

extern "C" int tgis_causal_conv(const void* x, int64_t ld_x, int x_f32, const float* w, const float* bias, int sets, float* tail,
                                int64_t tail_stride, const int32_t* state_slots, const int32_t* cu_seqlens_q, const int32_t* positions,
                                int64_t B, void* out, int64_t ld_out, int64_t set_stride, int64_t max_q_len, int64_t C, int taps, int act,
                                int residual, int dtype, void* stream) {
    TGIS_CHECK_ARG(x && w && state_slots && cu_seqlens_q && positions && out && (tail || taps == 1), "tgis_causal_conv: null tensor");
    TGIS_CHECK_ARG(taps >= 1 && taps <= 16 && (sets == 1 || sets == 2) && C >= 1 && ld_x >= C && ld_out >= C && max_q_len >= 1 &&
                       tail_stride >= (int64_t)(taps - 1) * C,
                   "tgis_causal_conv: bad arguments (taps %d, sets %d, C %ld)", taps, sets, (long)C);
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_causal_conv: bad dtype");
    if (B == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    const ConvArgs a{x, ld_x, w, bias, tail, tail_stride, state_slots, cu_seqlens_q, positions, out, ld_out, set_stride, (int)C, taps, sets, act, residual};
    const dim3 grid((unsigned)B, (unsigned)cdiv64(max_q_len, RUN), (unsigned)cdiv64(C, 256));
    TGIS_CHECK_ARG(grid.y <= 65535 && grid.z <= 65535, "tgis_causal_conv: step too long for one grid");
    if (dtype == TGIS_F16) launch_in<f16>(a, x_f32, grid, st);
    else if (dtype == TGIS_BF16) launch_in<bf16>(a, x_f32, grid, st);
    else launch_in<float>(a, x_f32, grid, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
