// Mixture of experts without a host round trip: router (fp32 logits, sigmoid or softmax scores, top-k), a one-workgroup
// sort of the (token, choice) pairs by expert into 32-row tiles, a grouped GEMM over those tiles on the matrix cores, and
// the combine that sums a token's rows (plus an optional gated shared expert).
//
//   route    logits = W_r h (fp32);  score = sigmoid(logit);  the k largest -> idx[T][k], weight[T][k]
//   align    pairs p = t * k + j sorted by expert; every expert's run padded to a multiple of 32 rows:
//            sorted[pos] = p or -1, tile_expert[pos / 32], pos_of_pair[p] = pos, n_tiles
//   gemm     out[pos][n] = sum_c A[row(pos)][c] * s(pos) * W[expert(pos)][n][c]        (s = 1 or the routing weight, applied
//            to the INPUT row and rounded to T like any other GEMM operand), optionally silu(gate) * up over a stacked
//            [gate | up] weight
//   combine  y[t] = sum_j rows[pos_of_pair[t k + j]] * (w[t][j] or 1) + g[t] * shared[t]
//
// The number of tiles is data dependent; the grid is sized for the worst case (T k + E * 31 rows) and tiles past n_tiles
// leave at once.
#include "common.h"

namespace {

constexpr int TM = 32;  // rows per tile = one 32x32 MFMA block

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)*p; }

// ---- router -----------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ h, int64_t ld_h, const float* __restrict__ wr,
                                                        const float* __restrict__ wg, int32_t* __restrict__ idx,
                                                        float* __restrict__ weight, float* __restrict__ shared_gate, int W, int E,
                                                        int k, const float* __restrict__ router_b, int softmax_top,
                                                        const float* __restrict__ correction, int n_groups, int keep_groups,
                                                        float renorm_eps) {
    extern __shared__ float sm[];
    float* hs = sm;          // [W]
    float* logit = sm + W;   // [E + 1]
    float* choice = logit + E + 1;  // [E] (softmax_top 2 only)
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    for (int c = threadIdx.x; c < W; c += blockDim.x) hs[c] = ldf(h + t * ld_h + c);
    __syncthreads();
    const int rows = E + (wg ? 1 : 0);
    for (int e = wave; e < rows; e += nw) {
        const float* w = e < E ? wr + (int64_t)e * W : wg;
        float s = 0.f;
        if ((W & 3) == 0) {  // 16-byte loads, several in flight
#pragma unroll 4
            for (int c = lane * 4; c < W; c += 256) {
                const f32x4 wv = *reinterpret_cast<const f32x4*>(w + c);
                const f32x4 hv = *reinterpret_cast<const f32x4*>(hs + c);
                s += wv[0] * hv[0] + wv[1] * hv[1] + wv[2] * hv[2] + wv[3] * hv[3];
            }
        } else {
            for (int c = lane; c < W; c += 64) s += hs[c] * w[c];
        }
        s = wave_sum(s);
        if (lane == 0) logit[e] = s + ((router_b && e < E) ? router_b[e] : 0.f);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (wg) shared_gate[t] = 1.f / (1.f + expf(-logit[E]));
        if (softmax_top == 2) {
            // scores = softmax over ALL experts; experts are chosen by score + correction among the keep_groups groups of
            // neighbours whose best choice score is largest (the others count as -inf); weights = the chosen scores / their sum
            float top = -INFINITY, sum = 0.f;
            for (int e = 0; e < E; ++e) top = fmaxf(top, logit[e]);
            for (int e = 0; e < E; ++e) sum += (logit[e] = expf(logit[e] - top));
            for (int e = 0; e < E; ++e) {
                logit[e] /= sum;
                choice[e] = logit[e] + (correction ? correction[e] : 0.f);
            }
            if (n_groups > 1 && keep_groups < n_groups) {
                const int per = E / n_groups;
                // a group is dropped when at least keep_groups others beat it (ties go to the lower index)
                for (int g = 0; g < n_groups; ++g) {
                    float best = -INFINITY;
                    for (int e = g * per; e < (g + 1) * per; ++e) best = fmaxf(best, choice[e]);
                    hs[g] = best;  // the row is no longer needed
                }
                for (int g = 0; g < n_groups; ++g) {
                    int ahead = 0;
                    for (int o = 0; o < n_groups; ++o) ahead += (hs[o] > hs[g] || (hs[o] == hs[g] && o < g)) ? 1 : 0;
                    if (ahead >= keep_groups)
                        for (int e = g * per; e < (g + 1) * per; ++e) choice[e] = -INFINITY;
                }
            }
            float wsum = 0.f;
            for (int j = 0; j < k; ++j) {
                int best = -1;
                float bv = -INFINITY;
                for (int e = 0; e < E; ++e)
                    if (choice[e] > bv) {
                        bv = choice[e];
                        best = e;
                    }
                if (best < 0) {  // fewer allowed experts than k, or NaN scores: the first index not taken yet
                    best = 0;
                    for (int e = E - 1; e >= 0; --e) {
                        bool taken = false;
                        for (int i = 0; i < j; ++i) taken |= idx[t * k + i] == e;
                        if (!taken) best = e;
                    }
                }
                idx[t * k + j] = best;
                weight[t * k + j] = logit[best];
                wsum += logit[best];
                choice[best] = -INFINITY;
            }
            for (int j = 0; j < k; ++j) weight[t * k + j] /= (wsum + renorm_eps);
            return;
        }
        // k passes of selection; ties go to the lower index
        for (int j = 0; j < k; ++j) {
            int best = -1;
            float bv = -INFINITY;
            for (int e = 0; e < E; ++e) {
                const float v = logit[e];
                if (v > bv) {
                    bv = v;
                    best = e;
                }
            }
            if (best < 0) best = 0;  // NaN logits: still a valid index
            idx[t * k + j] = best;
            // softmax_top: the chosen logits are softmaxed among themselves below (the first one is the largest)
            weight[t * k + j] = softmax_top ? bv : 1.f / (1.f + expf(-bv));
            logit[best] = -INFINITY;
        }
        if (softmax_top) {
            const float top = weight[t * k];
            float sum = 0.f;
            for (int j = 0; j < k; ++j) sum += expf(weight[t * k + j] - top);
            for (int j = 0; j < k; ++j) weight[t * k + j] = expf(weight[t * k + j] - top) / sum;
        }
    }
}

// ---- align: one workgroup ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void moe_align_kernel(const int32_t* __restrict__ idx, int64_t n_pairs, int E,
                                                         int32_t* __restrict__ sorted, int64_t cap, int32_t* __restrict__ tile_expert,
                                                         int32_t* __restrict__ pos_of_pair, int32_t* __restrict__ n_tiles) {
    extern __shared__ int32_t si[];
    int32_t* count = si;            // [E]
    int32_t* start = si + E;        // [E + 1]
    int32_t* cursor = si + 2 * E + 1;  // [E]
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = cursor[e] = 0;
    for (int64_t i = threadIdx.x; i < cap; i += blockDim.x) sorted[i] = -1;
    __syncthreads();
    for (int64_t p = threadIdx.x; p < n_pairs; p += blockDim.x) atomicAdd(&count[idx[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int32_t at = 0;
        for (int e = 0; e < E; ++e) {
            start[e] = at;
            at += (count[e] + TM - 1) / TM * TM;
        }
        start[E] = at;
        *n_tiles = at / TM;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x)
        for (int32_t tl = start[e] / TM; tl < start[e + 1] / TM; ++tl) tile_expert[tl] = e;
    // arrival order within an expert: the rows of a tile are independent of each other, so the order changes no result
    for (int64_t p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = idx[p];
        const int32_t pos = start[e] + atomicAdd(&cursor[e], 1);
        sorted[pos] = (int32_t)p;
        pos_of_pair[p] = pos;
    }
}

// ---- grouped GEMM -----------------------------------------------------------------------------------------------------
// Workgroup = 4 waves = one 32-row tile x 128 output columns; a wave owns 32 columns (GLU: 32 gate + the 32 matching up
// columns).  Operands come straight from global memory / L2 in MFMA fragment order: lane l holds row (l % 32) and 8 (bf16)
// or 4 (fp32) consecutive k at offset (l / 32) * that — a 16-byte load for A and for B ([out, in] weights are k-contiguous).
template <typename T> struct Frag;
template <> struct Frag<bf16> {
    static constexpr int KSTEP = 16, PER = 8;
    using V = bf16x8;
    static __device__ __forceinline__ V zero() { return V{}; }
    static __device__ __forceinline__ V scaled(V a, float s) {
        V r;
#pragma unroll
        for (int i = 0; i < 8; ++i) r[i] = (bf16)((float)a[i] * s);
        return r;
    }
    static __device__ __forceinline__ void mma(V a, V b, f32x16& c) { c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Frag<f16> {
    static constexpr int KSTEP = 16, PER = 8;
    using V = f16x8;
    static __device__ __forceinline__ V zero() { return V{}; }
    static __device__ __forceinline__ V scaled(V a, float s) {
        V r;
#pragma unroll
        for (int i = 0; i < 8; ++i) r[i] = (f16)((float)a[i] * s);
        return r;
    }
    static __device__ __forceinline__ void mma(V a, V b, f32x16& c) { c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct Frag<float> {
    static constexpr int KSTEP = 8, PER = 4;
    using V = f32x4;
    static __device__ __forceinline__ V zero() { return V{}; }
    static __device__ __forceinline__ V scaled(V a, float s) { return a * s; }
    // four 32x32x2 fp32 products: the k index a lane contributes to product i is (l / 32) * 4 + i, for A and B alike
    static __device__ __forceinline__ void mma(V a, V b, f32x16& c) {
#pragma unroll
        for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[i], c, 0, 0, 0);
    }
};

// Two shapes of workgroup (4 waves):
//   many tiles (prompts): wave w owns row tile 4 y + w and 64 output columns (GLU: 64 gate + the 64 matching up columns).  The
//     four waves walk the same weight rows at the same time, so an expert's weights come from L2 once per four row tiles
//     instead of once per tile, and a wave's A fragment feeds two (GLU: four) products;
//   few tiles (decode, KSPLIT): the four waves split K for ONE 32-row x 32-column block and meet in LDS, so that a launch with a
//     handful of tiles still has enough waves in flight to stream the expert weights.
template <typename T, bool GLU, bool KSPLIT>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const T* __restrict__ A, int64_t ld_a, const int32_t* __restrict__ sorted,
                                                       int pair_div, const float* __restrict__ pair_scale,
                                                       const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ n_tiles,
                                                       const T* __restrict__ Wt, int64_t expert_stride, int64_t N, int64_t K,
                                                       T* __restrict__ out, int64_t ld_out) {
    using F = Frag<T>;
    using V = typename F::V;
    constexpr int NB = KSPLIT ? 1 : 2;  // 32-column blocks per wave
    __shared__ float part[KSPLIT ? 4 * (GLU ? 2 : 1) * 16 * 64 : 1];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int tile = KSPLIT ? blockIdx.y : blockIdx.y * 4 + wave;
    if (tile >= *n_tiles) return;  // KSPLIT: the whole workgroup
    const int row = lane & 31, half = lane >> 5;
    const int64_t n0 = (int64_t)blockIdx.x * 32 * NB;
    const int64_t pos = (int64_t)tile * TM + row;
    const T* W = Wt + (int64_t)tile_expert[tile] * expert_stride;
    // A row of this lane
    int64_t arow = pos;
    float scale = 1.f;
    if (sorted) {
        const int32_t p = sorted[pos];
        const bool live = p >= 0;
        arow = live ? p / pair_div : 0;
        if (pair_scale) scale = live ? pair_scale[p] : 0.f;
    }
    const T* ap = A + arow * ld_a + half * F::PER;
    const T* bp[NB];
    const T* bp2[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int64_t n = n0 + nb * 32 + row;
        const int64_t ncol = n < N ? n : N - 1;  // clamped: columns past N are computed and dropped
        bp[nb] = W + ncol * K + half * F::PER;
        bp2[nb] = GLU ? W + (N + ncol) * K + half * F::PER : nullptr;
    }
    f32x16 acc[NB], acc2[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = acc2[nb] = f32x16{};
    // this wave's k range, in whole steps
    const int64_t steps = (K + F::KSTEP - 1) / F::KSTEP;
    const int64_t s0 = KSPLIT ? steps * wave / 4 : 0, s1 = KSPLIT ? steps * (wave + 1) / 4 : steps;
#pragma unroll 2
    for (int64_t kk = s0 * F::KSTEP; kk < s1 * F::KSTEP; kk += F::KSTEP) {
        const bool in = kk + half * F::PER + F::PER <= K;  // K is a multiple of PER: a fragment is whole or absent
        V a = in ? *reinterpret_cast<const V*>(ap + kk) : F::zero();
        if (pair_scale) a = F::scaled(a, scale);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            V b = in ? *reinterpret_cast<const V*>(bp[nb] + kk) : F::zero();
            F::mma(a, b, acc[nb]);
            if (GLU) {
                V b2 = in ? *reinterpret_cast<const V*>(bp2[nb] + kk) : F::zero();
                F::mma(a, b2, acc2[nb]);
            }
        }
    }
    // accumulator i of lane l: A row (i / 4) * 8 + (l / 32) * 4 + i % 4, B row (= output column) l % 32
    if (KSPLIT) {
        constexpr int NA = GLU ? 2 : 1;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            part[((wave * NA + 0) * 16 + i) * 64 + lane] = acc[0][i];
            if (GLU) part[((wave * NA + 1) * 16 + i) * 64 + lane] = acc2[0][i];
        }
        __syncthreads();
        if (n0 + row >= N) return;
        // wave w finishes accumulators 4 w .. 4 w + 3
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int i = wave * 4 + q;
            float v = 0.f, v2 = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                v += part[((w * NA + 0) * 16 + i) * 64 + lane];
                if (GLU) v2 += part[((w * NA + 1) * 16 + i) * 64 + lane];
            }
            if (GLU) v = v / (1.f + expf(-v)) * v2;
            const int m = (i >> 2) * 8 + half * 4 + (i & 3);
            out[((int64_t)tile * TM + m) * ld_out + n0 + row] = (T)v;
        }
        return;
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int64_t n = n0 + nb * 32 + row;
        if (n < N) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int m = (i >> 2) * 8 + half * 4 + (i & 3);
                float v = acc[nb][i];
                if (GLU) v = v / (1.f + expf(-v)) * acc2[nb][i];
                out[((int64_t)tile * TM + m) * ld_out + n] = (T)v;
            }
        }
    }
}

// ---- combine: one workgroup per token -----------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const T* __restrict__ rows, int64_t ld_rows, const int32_t* __restrict__ pos_of_pair,
                                                          const float* __restrict__ pair_weight, int k, const T* __restrict__ shared,
                                                          int64_t ld_shared, const float* __restrict__ shared_gate, T* __restrict__ out,
                                                          int64_t ld_out, int64_t W) {
    const int64_t t = blockIdx.x;
    const float g = shared ? (shared_gate ? shared_gate[t] : 1.f) : 0.f;
    const int64_t c = (int64_t)blockIdx.y * blockDim.x + threadIdx.x;  // grid (token, 256-column block)
    if (c >= W) return;
    float s = 0.f;
    for (int j = 0; j < k; ++j) {
        const float w = pair_weight ? pair_weight[t * k + j] : 1.f;
        s += w * ldf(rows + (int64_t)pos_of_pair[t * k + j] * ld_rows + c);
    }
    if (shared) s += g * ldf(shared + t * ld_shared + c);
    out[t * ld_out + c] = (T)s;
}

template <typename T>
void launch_gemm(bool glu, const void* A, int64_t ld_a, const int32_t* sorted, int pair_div, const float* pair_scale,
                 const int32_t* tile_expert, const int32_t* n_tiles, const void* Wt, int64_t expert_stride, int64_t N, int64_t K,
                 void* out, int64_t ld_out, int64_t max_tiles, hipStream_t st) {
    const bool ksplit = max_tiles * cdiv64(N, 128) < 1024;
    dim3 grid((unsigned)(ksplit ? cdiv64(N, 32) : cdiv64(N, 64)), (unsigned)(ksplit ? max_tiles : cdiv64(max_tiles, 4)));
#define TGIS_MOE_LAUNCH(GLU, KS)                                                                                              \
    hipLaunchKernelGGL((moe_gemm_kernel<T, GLU, KS>), grid, dim3(256), 0, st, (const T*)A, ld_a, sorted, pair_div, pair_scale, \
                       tile_expert, n_tiles, (const T*)Wt, expert_stride, N, K, (T*)out, ld_out)
    if (glu && ksplit)
        TGIS_MOE_LAUNCH(true, true);
    else if (glu)
        TGIS_MOE_LAUNCH(true, false);
    else if (ksplit)
        TGIS_MOE_LAUNCH(false, true);
    else
        TGIS_MOE_LAUNCH(false, false);
#undef TGIS_MOE_LAUNCH
}

}  // namespace

static bool dtype3(int d) { return d == TGIS_F16 || d == TGIS_BF16 || d == TGIS_F32; }

extern "C" int64_t tgis_moe_row_capacity(int64_t n_pairs, int64_t E) { return (n_pairs + E * (TM - 1) + TM - 1) / TM * TM; }

static int moe_route_impl(const void* h, int64_t ld_h, const float* router_w, const float* shared_gate_w, int32_t* idx,
                          float* weight, float* shared_gate, int64_t T, int64_t W, int E, int k, int dtype, void* stream,
                          const float* router_b, int softmax_top, const float* correction = nullptr, int n_groups = 1,
                          int keep_groups = 1, float renorm_eps = 0.f) {
    TGIS_CHECK_ARG(h && router_w && idx && weight && (!shared_gate_w || shared_gate), "tgis_moe_route: null tensor");
    TGIS_CHECK_ARG(n_groups >= 1 && keep_groups >= 1 && keep_groups <= n_groups && E % n_groups == 0 && n_groups <= W,
                   "tgis_moe_route: %d experts do not form %d equal groups", E, n_groups);
    TGIS_CHECK_ARG(E >= 1 && k >= 1 && k <= E && W >= 1 && ld_h >= W && dtype3(dtype), "tgis_moe_route: bad arguments");
    const size_t lds = ((size_t)W + 2 * E + 1) * sizeof(float);
    TGIS_CHECK_ARG(lds <= 64 * 1024, "tgis_moe_route: width + experts need %ld bytes of LDS", (long)lds);
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == TGIS_F16)
        hipLaunchKernelGGL(moe_route_kernel<f16>, dim3((unsigned)T), dim3(256), lds, st, (const f16*)h, ld_h, router_w, shared_gate_w, idx, weight, shared_gate, (int)W, E, k, router_b, softmax_top, correction, n_groups, keep_groups, renorm_eps);
    else if (dtype == TGIS_BF16)
        hipLaunchKernelGGL(moe_route_kernel<bf16>, dim3((unsigned)T), dim3(256), lds, st, (const bf16*)h, ld_h, router_w, shared_gate_w, idx, weight, shared_gate, (int)W, E, k, router_b, softmax_top, correction, n_groups, keep_groups, renorm_eps);
    else
        hipLaunchKernelGGL(moe_route_kernel<float>, dim3((unsigned)T), dim3(256), lds, st, (const float*)h, ld_h, router_w, shared_gate_w, idx, weight, shared_gate, (int)W, E, k, router_b, softmax_top, correction, n_groups, keep_groups, renorm_eps);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_moe_route(const void* h, int64_t ld_h, const float* router_w, const float* shared_gate_w, int32_t* idx,
                              float* weight, float* shared_gate, int64_t T, int64_t W, int E, int k, int dtype, void* stream) {
    return moe_route_impl(h, ld_h, router_w, shared_gate_w, idx, weight, shared_gate, T, W, E, k, dtype, stream, nullptr, 0);
}

// The same with a bias on the router logits (router_b [E] fp32 or NULL) and a choice of weights: softmax_top 0: the sigmoid of
// each chosen logit; 1: the softmax over the chosen logits only.
extern "C" int tgis_moe_route_ext(const void* h, int64_t ld_h, const float* router_w, const float* router_b, const float* shared_gate_w,
                                  int softmax_top, int32_t* idx, float* weight, float* shared_gate, int64_t T, int64_t W, int E, int k,
                                  int dtype, void* stream) {
    return moe_route_impl(h, ld_h, router_w, shared_gate_w, idx, weight, shared_gate, T, W, E, k, dtype, stream, router_b, softmax_top ? 1 : 0);
}

// Softmax scores over all experts; choice by score + correction [E] (fp32 or NULL) among the keep_groups best of n_groups equal
// groups of neighbouring experts (a group's rank is its largest choice score); weights = chosen scores / (their sum + renorm_eps).
extern "C" int tgis_moe_route_grouped(const void* h, int64_t ld_h, const float* router_w, const float* correction, int n_groups,
                                      int keep_groups, float renorm_eps, int32_t* idx, float* weight, int64_t T, int64_t W, int E, int k,
                                      int dtype, void* stream) {
    return moe_route_impl(h, ld_h, router_w, nullptr, idx, weight, nullptr, T, W, E, k, dtype, stream, nullptr, 2, correction, n_groups,
                          keep_groups, renorm_eps);
}

extern "C" int tgis_moe_align(const int32_t* idx, int64_t n_pairs, int E, int32_t* sorted, int64_t capacity, int32_t* tile_expert,
                              int32_t* pos_of_pair, int32_t* n_tiles, void* stream) {
    TGIS_CHECK_ARG(idx && sorted && tile_expert && pos_of_pair && n_tiles, "tgis_moe_align: null tensor");
    TGIS_CHECK_ARG(E >= 1 && E <= 4096 && n_pairs >= 0 && capacity >= tgis_moe_row_capacity(n_pairs, E),
                   "tgis_moe_align: capacity %ld below tgis_moe_row_capacity", (long)capacity);
    hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (size_t)(3 * E + 1) * sizeof(int32_t), (hipStream_t)stream, idx, n_pairs,
                       E, sorted, capacity, tile_expert, pos_of_pair, n_tiles);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_moe_gemm(const void* A, int64_t ld_a, const int32_t* sorted, int pair_div, const float* pair_scale,
                             const int32_t* tile_expert, const int32_t* n_tiles, const void* weights, int64_t expert_stride, int64_t N,
                             int64_t K, int glu, void* out, int64_t ld_out, int64_t capacity, int dtype, void* stream) {
    TGIS_CHECK_ARG(A && tile_expert && n_tiles && weights && out, "tgis_moe_gemm: null tensor");
    TGIS_CHECK_ARG(dtype3(dtype), "tgis_moe_gemm: bad dtype");
    const int per = dtype == TGIS_F32 ? 4 : 8;
    TGIS_CHECK_ARG(N >= 1 && K >= per && K % per == 0 && ld_a % per == 0 && ld_a >= K && ld_out >= N && capacity % TM == 0,
                   "tgis_moe_gemm: K (%ld) and the A row stride (%ld) must be multiples of %d", (long)K, (long)ld_a, per);
    TGIS_CHECK_ARG((((uintptr_t)A) & 15) == 0 && (((uintptr_t)weights) & 15) == 0 && (expert_stride * (dtype == TGIS_F32 ? 4 : 2)) % 16 == 0,
                   "tgis_moe_gemm: operands must be 16-byte aligned");
    TGIS_CHECK_ARG(!sorted || pair_div >= 1, "tgis_moe_gemm: gathered rows need pair_div >= 1");
    TGIS_CHECK_ARG(!pair_scale || sorted, "tgis_moe_gemm: a per-pair scale needs the sorted pair list");
    if (capacity == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_MOE_GEMM, st);
    const int64_t tiles = capacity / TM;
    TGIS_CHECK_ARG(tiles <= 65535, "tgis_moe_gemm: %ld tiles exceed one grid", (long)tiles);
    if (dtype == TGIS_F16)
        launch_gemm<f16>(glu != 0, A, ld_a, sorted, pair_div, pair_scale, tile_expert, n_tiles, weights, expert_stride, N, K, out, ld_out, tiles, st);
    else if (dtype == TGIS_BF16)
        launch_gemm<bf16>(glu != 0, A, ld_a, sorted, pair_div, pair_scale, tile_expert, n_tiles, weights, expert_stride, N, K, out, ld_out, tiles, st);
    else
        launch_gemm<float>(glu != 0, A, ld_a, sorted, pair_div, pair_scale, tile_expert, n_tiles, weights, expert_stride, N, K, out, ld_out, tiles, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_moe_combine(const void* rows, int64_t ld_rows, const int32_t* pos_of_pair, const float* pair_weight, int k,
                                const void* shared, int64_t ld_shared, const float* shared_gate, void* out, int64_t ld_out, int64_t T,
                                int64_t W, int dtype, void* stream) {
    TGIS_CHECK_ARG(rows && pos_of_pair && out && k >= 1 && W >= 1 && ld_rows >= W && ld_out >= W && (!shared || ld_shared >= W),
                   "tgis_moe_combine: bad arguments");
    TGIS_CHECK_ARG(dtype3(dtype), "tgis_moe_combine: bad dtype");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == TGIS_F16)
        hipLaunchKernelGGL(moe_combine_kernel<f16>, dim3((unsigned)T, (unsigned)cdiv64(W, 256)), dim3(256), 0, st, (const f16*)rows, ld_rows, pos_of_pair, pair_weight, k, (const f16*)shared, ld_shared, shared_gate, (f16*)out, ld_out, W);
    else if (dtype == TGIS_BF16)
        hipLaunchKernelGGL(moe_combine_kernel<bf16>, dim3((unsigned)T, (unsigned)cdiv64(W, 256)), dim3(256), 0, st, (const bf16*)rows, ld_rows, pos_of_pair, pair_weight, k, (const bf16*)shared, ld_shared, shared_gate, (bf16*)out, ld_out, W);
    else
        hipLaunchKernelGGL(moe_combine_kernel<float>, dim3((unsigned)T, (unsigned)cdiv64(W, 256)), dim3(256), 0, st, (const float*)rows, ld_rows, pos_of_pair, pair_weight, k, (const float*)shared, ld_shared, shared_gate, (float*)out, ld_out, W);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
