// Paged softmax attention for ragged steps (prompt portions beside single decoded tokens) with separate key and value
// widths, fp32 scores and weights, and the per-head preparation that goes with it: RMS norm of q and k, a query gain that
// depends on the position, value blending, and the cache write.
//
// Cache pages ("rows" layout, TGIS_KV_PAGE_TOKENS tokens per page, T = bf16 / f16 / float):
//   keys    k_pool[page][kv head][token in page][dk]      a (page, head) block is PAGE x dk, token-major
//   values  v_pool[page][kv head][dv][token in page]      a (page, head) block is dv x PAGE, channel-major (transposed):
//                                                          one lane streams one channel's tokens contiguously
// slot = page * PAGE + token in page, as everywhere in this library.
//
// A token t of sequence b sits at position ctx_lens[b] - (cu_q[b + 1] - t): the step's tokens are the LAST tokens of their
// sequences, whatever was cached before; token t sees keys 0 .. its own position.
#include <stdlib.h>
#include <algorithm>
#include <type_traits>
#include "common.h"

namespace {

constexpr int PAGE = TGIS_KV_PAGE_TOKENS;

// What a design may add to plain causal softmax attention (all off when zero / null):
//   chunk > 0:  a query at position i sees key j only if floor(i / chunk) == floor(j / chunk) (blocks counted from position 0)
//   r1, r2:     per query head, the score loses r1[h] * ln(1 + r2[h] * (i - j)) with the distance
//   gate:       out[t][h][c] is multiplied by sigmoid(gate[t][h dv + c]) where it is written (activation dtype, row stride ld_gate)
struct AttnExt {
    const float* r1;
    const float* r2;
    int chunk;
    const void* gate;
    int64_t ld_gate;
    // launch shaping of the matrix-core decode form (set by the launcher): with few (sequence, cached head) pairs — MQA, a
    // latent cache — the pages of a sequence are dealt to key_splits workgroups, which leave unnormalised partial results
    // ([split][token][head][m, l, dv sums], fp32) for attn_combine_splits_kernel
    int key_splits;
    float* partial;
    int64_t partial_tokens;  // tokens of the step (the partial results' second extent)
    //   window > 0: a query at position i sees key j <= i only if i - j < window or j < keep_first (a sliding window that
    //               also keeps the first positions of the sequence, at their true positions); not combined with chunk
    //   sink:       per query head, exp(sink[h]) joins the softmax denominator: a slot without key or value, not scaled
    //   gate_per_head: the gate holds ONE number per (token, head), gate[t][h], instead of one per output channel
    //   out_scale:  the output is multiplied by this where it is written
    int window = 0;
    int keep_first = 0;
    const float* sink = nullptr;
    int gate_per_head = 0;
    float out_scale = 1.f;
};
__device__ __forceinline__ float sigmoid_f32(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ int first_visible(const AttnExt& e, int pos) {
    if (e.window > 0) return max(pos - e.window + 1, 0);
    return e.chunk > 0 && pos > 0 ? pos / e.chunk * e.chunk : 0;
}
// key j of a query at position pos whose window / block starts at lo
__device__ __forceinline__ bool key_visible(const AttnExt& e, int key, int pos, int lo) { return key <= pos && (key >= lo || key < e.keep_first); }
// The pages (or 64-key chunks) a walk visits: the first `nkeep` units hold kept first positions, then it continues at unit `u0`.
__device__ __forceinline__ int kept_units(const AttnExt& e, int u0, int unit) { return min((e.keep_first + unit - 1) / unit, u0); }
__device__ __forceinline__ int walk_unit(int i, int nkeep, int u0) { return i < nkeep ? i : u0 + (i - nkeep); }
// Softmax statistics (m, l) of a finished column take the sink in: returns the factor for the unnormalised sums, l becomes the
// full denominator.  m is finite (a query always sees its own key).
__device__ __forceinline__ float fold_sink(const AttnExt& e, int head, float m, float& l) {
    if (!e.sink) return 1.f;
    const float sk = e.sink[head];
    const float mm = fmaxf(m, sk);
    const float f = expf(m - mm);
    l = l * f + expf(sk - mm);
    return f;
}
// what multiplies head `head` of token t where it is written (the per-head gate and the output scale)
template <typename T> __device__ __forceinline__ float head_out_factor(const AttnExt& e, int64_t t, int head) {
    float f = e.out_scale;
    if (e.gate && e.gate_per_head) f *= sigmoid_f32((float)reinterpret_cast<const T*>(e.gate)[t * e.ld_gate + head]);
    return f;
}

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)*p; }

__device__ __forceinline__ int seq_of_token(const int32_t* __restrict__ cu_q, int B, int t) {
    int lo = 0, hi = B;  // cu_q[lo] <= t < cu_q[hi]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (cu_q[mid] <= t) lo = mid; else hi = mid;
    }
    return lo;
}

// ---- preparation: grid (token, head group): a wave per q / k head -------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_kv_write_kernel(
    T* __restrict__ qkv, int64_t ld, const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps, float gain_coef, int gain_every,
    const T* __restrict__ v_first, int64_t ld_vf, const float* __restrict__ lambda_ptr, T* __restrict__ k_pool,
    T* __restrict__ v_pool, int H, int G, int dk, int dv, int v_inline) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    const int slot = slots[t];
    const int64_t page = slot / PAGE;
    const int off = slot % PAGE;
    T* row = qkv + t * ld;
    const int head_blocks = (H + G + nw - 1) / nw;
    if (v_inline && (int)blockIdx.y >= head_blocks) {
        // small steps (decode): the values go out from here, a few more workgroups per token (1024 values each) instead of
        // one more launch
        const float lam = (v_first && lambda_ptr) ? *lambda_ptr : 0.f;
        const T* vrow = row + (int64_t)(H + G) * dk;
        const int i0 = ((int)blockIdx.y - head_blocks) * 1024;
        const int i1 = min(i0 + 1024, G * dv);
        for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x) {
            float v = ldf(vrow + i);
            if (v_first) v = (1.f - lam) * v + lam * ldf(v_first + t * ld_vf + i);
            const int g = i / dv, c = i - g * dv;
            v_pool[((page * G + g) * dv + c) * PAGE + off] = (T)v;
        }
        return;
    }
    const int h = blockIdx.y * nw + wave;
    if (h >= H + G) return;
    const bool is_q = h < H;
    T* p = row + (int64_t)h * dk;  // k heads follow the q heads with the same width
    float gain = 1.f;
    if (is_q && gain_every > 0) gain = 1.f + gain_coef * logf((float)((positions[t] + 1) / gain_every) + 1.f);
    T* dst = is_q ? p : k_pool + ((page * G + (h - H)) * PAGE + off) * dk;
    const float* w = is_q ? qw : kw;
    if (sizeof(T) == 2 && dk <= 256 && (dk & 1) == 0 && (ld & 1) == 0) {
        // two-byte dtypes, heads of up to 256: a lane holds two pairs of neighbouring channels, read once
        using T2 = typename std::conditional<sizeof(T) == 2, T, bf16>::type;
        using V2 = typename VecT<T2>::x2;
        float v[4];
        float ss = 0.f;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int d = lane * 2 + it * 128;
            V2 x = d < dk ? *reinterpret_cast<const V2*>(reinterpret_cast<const T2*>(p) + d) : V2{};
            v[it * 2] = (float)x[0];
            v[it * 2 + 1] = (float)x[1];
            ss += v[it * 2] * v[it * 2] + v[it * 2 + 1] * v[it * 2 + 1];
        }
        ss = wave_sum(ss);
        const float rinv = 1.0f / sqrtf(ss / (float)dk + eps) * gain;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int d = lane * 2 + it * 128;
            if (d < dk) {
                V2 y;
                y[0] = (T2)(v[it * 2] * rinv * w[d]);
                y[1] = (T2)(v[it * 2 + 1] * rinv * w[d + 1]);
                *reinterpret_cast<V2*>(reinterpret_cast<T2*>(dst) + d) = y;
            }
        }
        return;
    }
    float ss = 0.f;
    for (int d = lane; d < dk; d += 64) {
        float v = ldf(p + d);
        ss += v * v;
    }
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)dk + eps) * gain;
    for (int d = lane; d < dk; d += 64) dst[d] = (T)(ldf(p + d) * rinv * w[d]);
}

// Values: blended if asked, then written channel-major.  A workgroup takes 32 consecutive step tokens x 64 value columns
// through LDS: rows are read as they lie in the projection's output (a token's columns are contiguous), and written with
// the tokens of a page side by side — a 16-byte store per (column, 8 tokens) wherever 8 neighbours of the step are 8
// neighbours in a page (prompt portions), single elements otherwise (decoded tokens of different sequences).
template <typename T>
__global__ __launch_bounds__(256) void v_write_kernel(const T* __restrict__ qkv, int64_t ld, int64_t v_col0, const int32_t* __restrict__ slots,
                                                      const T* __restrict__ v_first, int64_t ld_vf, const float* __restrict__ lambda_ptr,
                                                      T* __restrict__ v_pool, int64_t Ttot, int G, int dv) {
    __shared__ float tile[32][65];
    __shared__ int32_t sl[32];
    const int64_t t0 = (int64_t)blockIdx.x * 32;
    const int c0 = blockIdx.y * 64, C = G * dv;
    const int tid = threadIdx.x;
    if (tid < 32) sl[tid] = t0 + tid < Ttot ? slots[t0 + tid] : -1;
    const float lam = (v_first && lambda_ptr) ? *lambda_ptr : 0.f;
    for (int e = tid; e < 32 * 64; e += 256) {
        const int tt = e >> 6, cc = e & 63;
        float v = 0.f;
        if (t0 + tt < Ttot && c0 + cc < C) {
            v = ldf(qkv + (t0 + tt) * ld + v_col0 + c0 + cc);
            if (v_first) v = (1.f - lam) * v + lam * ldf(v_first + (t0 + tt) * ld_vf + c0 + cc);
        }
        tile[tt][cc] = v;
    }
    __syncthreads();
    // thread = (column, group of 8 tokens)
    const int cc = tid >> 2, tg = (tid & 3) * 8;
    const int col = c0 + cc;
    if (col >= C) return;
    const int g = col / dv, ch = col - g * dv;
    const int s0 = sl[tg];
    bool run = s0 >= 0 && (s0 % PAGE) % 8 == 0 && sizeof(T) == 2;
#pragma unroll
    for (int j = 1; j < 8; ++j) run = run && sl[tg + j] == s0 + j;
    if (run) {
        using V8 = typename VecT<typename std::conditional<sizeof(T) == 2, T, bf16>::type>::x8;
        V8 pack;
#pragma unroll
        for (int j = 0; j < 8; ++j) pack[j] = (typename std::conditional<sizeof(T) == 2, T, bf16>::type)tile[tg + j][cc];
        const int64_t page = s0 / PAGE;
        *reinterpret_cast<V8*>(v_pool + ((page * G + g) * dv + ch) * PAGE + (s0 % PAGE)) = pack;
        return;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int s = sl[tg + j];
        if (s < 0) continue;
        const int64_t page = s / PAGE;
        v_pool[((page * G + g) * dv + ch) * PAGE + (s % PAGE)] = (T)tile[tg + j][cc];
    }
}

// ---- attention, general form -----------------------------------------------------------------------------------------
// One workgroup per (token, kv head): R = H / G query heads x S key splits waves.  A wave walks its 64-key chunks: a lane
// owns one key for the scores (q . k with q staged in LDS as fp32, already scaled), then one value channel (per 64) for
// the weighted sum, with the weights handed from lane to lane by readlane.  Softmax statistics are kept per wave and the
// splits of a head meet in LDS at the end.
template <typename T> __device__ __forceinline__ float dot_row(const float* __restrict__ qs, const T* __restrict__ kp, int dk);

template <> __device__ __forceinline__ float dot_row<float>(const float* __restrict__ qs, const float* __restrict__ kp, int dk) {
    float s = 0.f;
    if ((dk & 3) == 0) {
        for (int d = 0; d < dk; d += 4) {
            f32x4 kv = *reinterpret_cast<const f32x4*>(kp + d);
            f32x4 qv = *reinterpret_cast<const f32x4*>(qs + d);
            s += qv[0] * kv[0] + qv[1] * kv[1] + qv[2] * kv[2] + qv[3] * kv[3];
        }
    } else {
        for (int d = 0; d < dk; ++d) s += qs[d] * kp[d];
    }
    return s;
}
template <typename T> __device__ __forceinline__ float dot_row(const float* __restrict__ qs, const T* __restrict__ kp, int dk) {
    using V8 = typename VecT<T>::x8;
    float s = 0.f;
    if ((dk & 7) == 0) {
        for (int d = 0; d < dk; d += 8) {
            V8 kv = *reinterpret_cast<const V8*>(kp + d);
            f32x4 q0 = *reinterpret_cast<const f32x4*>(qs + d);
            f32x4 q1 = *reinterpret_cast<const f32x4*>(qs + d + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) s += q0[i] * (float)kv[i];
#pragma unroll
            for (int i = 0; i < 4; ++i) s += q1[i] * (float)kv[4 + i];
        }
    } else {
        for (int d = 0; d < dk; ++d) s += qs[d] * (float)kp[d];
    }
    return s;
}

constexpr int DV_PER_LANE = 4;  // value channels per lane: dv <= 256

template <typename T>
__global__ __launch_bounds__(1024) void attn_varlen_kernel(
    const T* __restrict__ q, int64_t ldq, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int32_t* __restrict__ bt, int64_t bt_ld, const int32_t* __restrict__ ctx_lens, const int32_t* __restrict__ cu_q, int B,
    T* __restrict__ out, int64_t ld_out, int H, int G, int dk, int dv, float scale, int S, AttnExt ext) {
    extern __shared__ float smem[];
    // blockIdx.y = kv head * sub-blocks + sub-block; a sub-block is up to 16 query heads of the group
    const int Rall = H / G, nsub = (Rall + 15) / 16;
    const int t = blockIdx.x, g = blockIdx.y / nsub, r0 = (blockIdx.y % nsub) * 16;
    const int R = min(16, Rall - r0);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (wave >= R * S) return;  // the last sub-block may have fewer heads (no workgroup barrier precedes this)
    const int r = wave % R, sp = wave / R;
    const int b = seq_of_token(cu_q, B, t);
    const int pos = ctx_lens[b] - (cu_q[b + 1] - t);
    const int nkeys = pos + 1;
    const int lo = first_visible(ext, pos);
    const float r1h = ext.r1 ? ext.r1[g * Rall + r0 + r] : 0.f, r2h = ext.r1 ? ext.r2[g * Rall + r0 + r] : 0.f;
    float* qs = smem;                              // [R][dk]
    float* merge = smem + (int64_t)R * dk;          // [R * S][2 + dv]
    for (int i = threadIdx.x; i < R * dk; i += R * S * 64) qs[i] = ldf(q + (int64_t)t * ldq + (int64_t)(g * Rall + r0) * dk + i) * scale;
    __syncthreads();  // waves that left above no longer count at a barrier
    const float* myq = qs + r * dk;
    const int32_t* table = bt + (int64_t)b * bt_ld;
    float m = -INFINITY, l = 0.f;
    float o[DV_PER_LANE];
#pragma unroll
    for (int c = 0; c < DV_PER_LANE; ++c) o[c] = 0.f;
    const int c0 = lo / 64, nkc = kept_units(ext, c0, 64), nchunks = nkc + (nkeys + 63) / 64 - c0;
    for (int ci = sp; ci < nchunks; ci += S) {
        const int base = walk_unit(ci, nkc, c0) * 64;
        const int j = base + lane;
        float s = -INFINITY;
        if (key_visible(ext, j, pos, lo)) {
            const int64_t page = table[j / PAGE];
            s = dot_row<T>(myq, k_pool + ((page * G + g) * PAGE + (j % PAGE)) * dk, dk);
            if (ext.r1) s -= r1h * log1pf(r2h * (float)(pos - j));
        }
        const float mn = fmaxf(m, wave_max(s));  // finite: key `base` is visible
        const float corr = expf(m - mn);         // exp(-inf) = 0 on the first chunk
        const float p = key_visible(ext, j, pos, lo) ? expf(s - mn) : 0.f;
        l = l * corr + wave_sum(p);
        m = mn;
#pragma unroll
        for (int c = 0; c < DV_PER_LANE; ++c) o[c] *= corr;
        for (int half = 0; half < 64 / PAGE; ++half) {
            const int first = base + half * PAGE;
            if (first >= nkeys) break;
            if (first + PAGE <= lo && first >= ext.keep_first) continue;  // a page before the query's block: all its weights are zero
            const int n = min(PAGE, nkeys - first);
            const int64_t page = table[first / PAGE];
#pragma unroll
            for (int c = 0; c < DV_PER_LANE; ++c) {
                const int ch = lane + 64 * c;
                if (ch < dv) {
                    const T* vp = v_pool + ((page * G + g) * dv + ch) * PAGE;
                    float acc = 0.f;
                    for (int jj = 0; jj < n; ++jj) {
                        const float pj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p), half * PAGE + jj));
                        acc += pj * ldf(vp + jj);
                    }
                    o[c] += acc;
                }
            }
        }
    }
    // meet the splits of a head
    float* mine = merge + (int64_t)(r * S + sp) * (2 + dv);
    if (S > 1) {
        if (lane == 0) {
            mine[0] = m;
            mine[1] = l;
        }
#pragma unroll
        for (int c = 0; c < DV_PER_LANE; ++c)
            if (lane + 64 * c < dv) mine[2 + lane + 64 * c] = o[c];
    }
    __syncthreads();
    if (sp != 0) return;
    if (S > 1) {
        float mm = m;
        for (int s2 = 1; s2 < S; ++s2) mm = fmaxf(mm, merge[(int64_t)(r * S + s2) * (2 + dv)]);
        float ll = 0.f;
        float acc[DV_PER_LANE];
#pragma unroll
        for (int c = 0; c < DV_PER_LANE; ++c) acc[c] = 0.f;
        for (int s2 = 0; s2 < S; ++s2) {
            const float* other = merge + (int64_t)(r * S + s2) * (2 + dv);
            const float om = other[0];
            const float w = om == -INFINITY ? 0.f : expf(om - mm);
            ll += other[1] * w;
#pragma unroll
            for (int c = 0; c < DV_PER_LANE; ++c)
                if (lane + 64 * c < dv) acc[c] += other[2 + lane + 64 * c] * w;
        }
        l = ll;
        m = mm;
#pragma unroll
        for (int c = 0; c < DV_PER_LANE; ++c) o[c] = acc[c];
    }
    const float sink_f = fold_sink(ext, g * Rall + r0 + r, m, l);
    const float inv = sink_f / l * head_out_factor<T>(ext, t, g * Rall + r0 + r);
    T* orow = out + (int64_t)t * ld_out + (int64_t)(g * Rall + r0 + r) * dv;
    const T* grow = (ext.gate && !ext.gate_per_head) ? reinterpret_cast<const T*>(ext.gate) + (int64_t)t * ext.ld_gate + (int64_t)(g * Rall + r0 + r) * dv : nullptr;
#pragma unroll
    for (int c = 0; c < DV_PER_LANE; ++c)
        if (lane + 64 * c < dv) orow[lane + 64 * c] = (T)(o[c] * inv * (grow ? sigmoid_f32(ldf(grow + lane + 64 * c)) : 1.f));
}


// ---- attention on the matrix cores (two-byte dtypes, dk % 16 == 0, dv % 32 == 0) ----------------------------------------
// Columns of a sequence = (step token, query head of the kv group): col = tq * R + r.  A wave owns a 32-column tile and
// walks pages of 32 keys:   S^T = K Q^T  (A = the K page, 16-byte fragment loads; B = Q^T, held in registers),
// fp32 online softmax per column (a column lives in lanes c and c + 32), then  O^T += V^T P^T  with P rounded to T and taken
// as the B operand straight from the S^T accumulators: accumulator i of lane half h is key (i / 4) * 8 + h * 4 + i % 4, so
// the V^T fragment that matches k-slot order is two 8-byte loads of the channel-major V page.
//   mode 0 (a step with long runs):   the NW waves of a workgroup own NW neighbouring column tiles and all their keys;
//   mode 1 (runs * R <= 32, decode):  the NW waves split the pages of ONE tile and meet in LDS.
template <typename T, int DK16, int DVT>
__global__ __launch_bounds__(512) void attn_varlen_mfma_kernel(
    const T* __restrict__ q, int64_t ldq, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int32_t* __restrict__ bt, int64_t bt_ld, const int32_t* __restrict__ ctx_lens, const int32_t* __restrict__ cu_q,
    T* __restrict__ out, int64_t ld_out, int H, int G, int dk, int dv, float scale, int split, AttnExt ext) {
    using V8 = typename VecT<T>::x8;
    using V4 = typename VecT<T>::x4;
    extern __shared__ float smem[];
    const int b = blockIdx.z, g = blockIdx.y;
    const int R = H / G;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    const int c = lane & 31, h = lane >> 5;
    const int t0 = cu_q[b], qlen = cu_q[b + 1] - t0;
    const int ncols = qlen * R;
    const int tile = split ? 0 : blockIdx.x * nw + wave;
    if (tile * 32 >= ncols) return;  // split mode: uniform for the workgroup
    const int ctx = ctx_lens[b];
    const int col = tile * 32 + c;
    const bool live = col < ncols;
    const int tq = live ? col / R : 0, r = live ? col % R : 0;
    const int pos = live ? ctx - qlen + tq : -1;  // keys 0 .. pos are visible
    const int last_col = min(tile * 32 + 31, ncols - 1);
    const int max_pos = ctx - qlen + last_col / R;
    const int npages = max_pos / PAGE + 1;
    const int nks = dk >> 4, nvt = dv >> 5;
    // blocks: positions grow with the columns, so the tile's first column has the earliest first visible key
    const int lo = first_visible(ext, pos);
    const int page0 = first_visible(ext, ctx - qlen + tile * 32 / R) / PAGE;
    // the walk: pages with kept first positions that lie before the window, then the window's pages
    const int nkeep = kept_units(ext, page0, PAGE), nvis = nkeep + npages - page0;
    const float r1h = ext.r1 ? ext.r1[g * R + r] : 0.f, r2h = ext.r1 ? ext.r2[g * R + r] : 0.f;
    // Q^T fragments: lane (column c, half h) holds 8 consecutive channels of its column's query per 16-channel step
    V8 qf[DK16];
    const T* qrow = q + (int64_t)(t0 + tq) * ldq + (int64_t)(g * R + r) * dk + h * 8;
#pragma unroll
    for (int s = 0; s < DK16; ++s) qf[s] = (live && s < nks) ? *reinterpret_cast<const V8*>(qrow + s * 16) : V8{};
    f32x16 O[DVT];
#pragma unroll
    for (int t = 0; t < DVT; ++t) O[t] = f32x16{};
    float m = -INFINITY, lsum = 0.f;
    const int32_t* table = bt + (int64_t)b * bt_ld;
    const int nsplit = (split && ext.key_splits > 1) ? ext.key_splits : 1;
    const int pstep = split ? nw * nsplit : 1;
    // the K fragments of a page are asked for one page ahead: a page costs its arithmetic, not a round trip to memory
    V8 kf[DK16];
    int64_t page = 0;
    const int pstart = split ? (int)blockIdx.x * nw + wave : 0;
    if (pstart < nvis) {
        page = table[walk_unit(pstart, nkeep, page0)];
        const T* kp = k_pool + ((page * G + g) * PAGE + c) * dk + h * 8;
#pragma unroll
        for (int s = 0; s < DK16; ++s) kf[s] = s < nks ? *reinterpret_cast<const V8*>(kp + s * 16) : V8{};
    }
    for (int pi = pstart; pi < nvis; pi += pstep) {
        const int p = walk_unit(pi, nkeep, page0);
        f32x16 S = {};
#pragma unroll
        for (int s = 0; s < DK16; ++s)
            if (s < nks) S = mfma32(kf[s], qf[s], S);
        const int64_t this_page = page;
        if (pi + pstep < nvis) {
            page = table[walk_unit(pi + pstep, nkeep, page0)];
            const T* kp = k_pool + ((page * G + g) * PAGE + c) * dk + h * 8;
#pragma unroll
            for (int s = 0; s < DK16; ++s) kf[s] = s < nks ? *reinterpret_cast<const V8*>(kp + s * 16) : V8{};
        }
        // the V fragments of this page are independent of the softmax: ask for them now
        const T* vp = v_pool + ((this_page * G + g) * dv + c) * PAGE + h * 4;
        constexpr int VPRE = DVT <= 2 ? DVT : 1;  // wide values: fetched tile by tile below (registers)
        V4 vf[VPRE][4];
        if (DVT <= 2) {
#pragma unroll
            for (int t = 0; t < VPRE; ++t)
                if (t < nvt) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) vf[t][j] = *reinterpret_cast<const V4*>(vp + (int64_t)t * 32 * PAGE + j * 8);
                }
        }
        const int base = p * PAGE + h * 4;
        float mx = -INFINITY;
        if (ext.r1) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = base + (i >> 2) * 8 + (i & 3);
                S[i] = key_visible(ext, key, pos, lo) ? S[i] * scale - r1h * __logf(1.f + r2h * (float)(pos - key)) : -INFINITY;
                mx = fmaxf(mx, S[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = base + (i >> 2) * 8 + (i & 3);
                S[i] = key_visible(ext, key, pos, lo) ? S[i] * scale : -INFINITY;
                mx = fmaxf(mx, S[i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m, mx);
        float corr = 1.f;
        if (mn == -INFINITY) {
#pragma unroll
            for (int i = 0; i < 16; ++i) S[i] = 0.f;
        } else {
            corr = expf(m - mn);
#pragma unroll
            for (int i = 0; i < 16; ++i) S[i] = expf(S[i] - mn);
        }
        m = mn;
        float ps = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) ps += S[i];
        lsum = lsum * corr + ps;
        V8 pb[2];
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
            for (int i = 0; i < 8; ++i) pb[c2][i] = (T)S[c2 * 8 + i];
#pragma unroll
        for (int t = 0; t < DVT; ++t)
            if (t < nvt) {
                if (corr != 1.f) O[t] *= corr;
                V4 vt[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    vt[j] = DVT <= 2 ? vf[t < VPRE ? t : 0][j] : *reinterpret_cast<const V4*>(vp + (int64_t)t * 32 * PAGE + j * 8);
#pragma unroll
                for (int c2 = 0; c2 < 2; ++c2) {
                    V8 a;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        a[i] = vt[c2 * 2][i];
                        a[4 + i] = vt[c2 * 2 + 1][i];
                    }
                    O[t] = mfma32(a, pb[c2], O[t]);
                }
            }
    }
    lsum += __shfl_xor(lsum, 32, 64);
    if (split) {
        // [wave][64 lanes] m and l, then [wave][DVT * 4 groups][4][64] partial O^T; the waves share the merge by groups of
        // four accumulators (= four consecutive output channels of a lane's column)
        float* ml = smem;
        float* os = smem + nw * 128;
        ml[wave * 128 + lane] = m;
        ml[wave * 128 + 64 + lane] = lsum;
#pragma unroll
        for (int t = 0; t < DVT; ++t)
            if (t < nvt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) os[((wave * DVT + t) * 16 + i) * 64 + lane] = O[t][i];
            }
        __syncthreads();
        float mm = -INFINITY;
        for (int w = 0; w < nw; ++w) mm = fmaxf(mm, ml[w * 128 + lane]);
        float ll = 0.f;
        for (int w = 0; w < nw; ++w) {
            const float om = ml[w * 128 + lane];
            ll += om == -INFINITY ? 0.f : ml[w * 128 + 64 + lane] * expf(om - mm);
        }
        if (!live) return;
        if (nsplit > 1) {
            // this workgroup saw only its share of the pages: leave (m, l, unnormalised sums) for the combine pass
            float* prow = ext.partial + (((int64_t)blockIdx.x * ext.partial_tokens + (t0 + tq)) * H + (g * R + r)) * (int64_t)(dv + 2);
            if (wave == 0 && h == 0) {
                prow[0] = mm;
                prow[1] = ll;
            }
            for (int grp = wave; grp < nvt * 4; grp += nw) {
                const int t = grp >> 2, j = grp & 3;
                float acc[4] = {0.f, 0.f, 0.f, 0.f};
                for (int w = 0; w < nw; ++w) {
                    const float om = ml[w * 128 + lane];
                    const float wgt = om == -INFINITY ? 0.f : expf(om - mm);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[i] += os[((w * DVT + t) * 16 + j * 4 + i) * 64 + lane] * wgt;
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) prow[2 + h * 4 + t * 32 + j * 8 + i] = acc[i];
            }
            return;
        }
        const float sink_f = fold_sink(ext, g * R + r, mm, ll);
        const float inv = sink_f / ll * head_out_factor<T>(ext, t0 + tq, g * R + r);
        T* orow = out + (int64_t)(t0 + tq) * ld_out + (int64_t)(g * R + r) * dv + h * 4;
        const T* grow = (ext.gate && !ext.gate_per_head) ? reinterpret_cast<const T*>(ext.gate) + (int64_t)(t0 + tq) * ext.ld_gate + (int64_t)(g * R + r) * dv + h * 4 : nullptr;
        for (int grp = wave; grp < nvt * 4; grp += nw) {
            const int t = grp >> 2, j = grp & 3;
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            for (int w = 0; w < nw; ++w) {
                const float om = ml[w * 128 + lane];
                const float wgt = om == -INFINITY ? 0.f : expf(om - mm);
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[i] += os[((w * DVT + t) * 16 + j * 4 + i) * 64 + lane] * wgt;
            }
            V4 o4, g4 = {};
            if (grow) g4 = *reinterpret_cast<const V4*>(grow + t * 32 + j * 8);
#pragma unroll
            for (int i = 0; i < 4; ++i) o4[i] = (T)(acc[i] * inv * (grow ? sigmoid_f32((float)g4[i]) : 1.f));
            *reinterpret_cast<V4*>(orow + t * 32 + j * 8) = o4;
        }
        return;
    }
    if (!live) return;
    const float sink_f = fold_sink(ext, g * R + r, m, lsum);
    const float inv = sink_f / lsum * head_out_factor<T>(ext, t0 + tq, g * R + r);
    T* orow = out + (int64_t)(t0 + tq) * ld_out + (int64_t)(g * R + r) * dv + h * 4;
    const T* grow = (ext.gate && !ext.gate_per_head) ? reinterpret_cast<const T*>(ext.gate) + (int64_t)(t0 + tq) * ext.ld_gate + (int64_t)(g * R + r) * dv + h * 4 : nullptr;
#pragma unroll
    for (int t = 0; t < DVT; ++t)
        if (t < nvt) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                V4 o4, g4 = {};
                if (grow) g4 = *reinterpret_cast<const V4*>(grow + t * 32 + j * 8);
#pragma unroll
                for (int i = 0; i < 4; ++i) o4[i] = (T)(O[t][j * 4 + i] * inv * (grow ? sigmoid_f32((float)g4[i]) : 1.f));
                *reinterpret_cast<V4*>(orow + t * 32 + j * 8) = o4;
            }
        }
}


// One wave per (token, head): the key splits' partial results meet — out = sum_x e^(m_x - m) sums_x / sum_x e^(m_x - m) l_x.
template <typename T>
__global__ __launch_bounds__(64) void attn_combine_splits_kernel(const float* __restrict__ partial, int X, int64_t Ttot, int H, int dv,
                                                                 T* __restrict__ out, int64_t ld_out, AttnExt ext) {
    __shared__ float wx[64];  // X <= 64: the weight of every split, e^(m_x - m) / sum
    const int64_t t = blockIdx.x;
    const int head = blockIdx.y, lane = threadIdx.x;
    const int64_t stride = Ttot * H * (int64_t)(dv + 2);
    const float* p0 = partial + (t * H + head) * (int64_t)(dv + 2);
    const float om = lane < X ? p0[lane * stride] : -INFINITY;
    const float ol = lane < X ? p0[lane * stride + 1] : 0.f;
    const float mm = wave_max(om);
    const float e = om == -INFINITY ? 0.f : expf(om - mm);
    float ll = wave_sum(ol * e);
    const float sink_f = fold_sink(ext, head, mm, ll);
    wx[lane] = e * sink_f / ll * head_out_factor<T>(ext, t, head);
    __syncthreads();
    const T* grow = (ext.gate && !ext.gate_per_head) ? reinterpret_cast<const T*>(ext.gate) + t * ext.ld_gate + (int64_t)head * dv : nullptr;
    for (int c = lane; c < dv; c += 64) {
        float acc = 0.f;
        for (int x = 0; x < X; ++x) acc += p0[x * stride + 2 + c] * wx[x];
        out[t * ld_out + (int64_t)head * dv + c] = (T)(acc * (grow ? sigmoid_f32(ldf(grow + c)) : 1.f));
    }
}

// The same for steps with long runs (prompts and their portions): the four waves of a workgroup own four neighbouring
// column tiles of one sequence and kv head and walk the SAME pages, so a page is brought in once for all of them — global
// memory -> registers (one page ahead, in flight during the arithmetic) -> LDS (rows padded by 16 bytes for K, 8 for V, so
// that the fragment reads of a wave spread over the banks) -> fragments.  A wave whose tile ends earlier (causality) or does
// not exist keeps helping with the copies and skips the arithmetic.
template <typename T, int DK16, int DVT>
__global__ __launch_bounds__(256) void attn_varlen_staged_kernel(
    const T* __restrict__ q, int64_t ldq, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int32_t* __restrict__ bt, int64_t bt_ld, const int32_t* __restrict__ ctx_lens, const int32_t* __restrict__ cu_q,
    T* __restrict__ out, int64_t ld_out, int H, int G, int dk, int dv, float scale, AttnExt ext) {
    using V8 = typename VecT<T>::x8;
    using V4 = typename VecT<T>::x4;
    constexpr int KROW = DK16 * 16 + 8;       // LDS row of a key: its channels + 16 bytes
    constexpr int VROW = PAGE + 4;            // LDS row of a value channel: its 32 tokens + 8 bytes
    constexpr int KL = DK16 >= 4 ? DK16 / 4 : 1;  // 16-byte pieces of a K page per thread (256 threads)
    constexpr int VL = DVT >= 2 ? DVT / 2 : 1;
    __shared__ __attribute__((aligned(16))) T ks[PAGE * KROW];
    __shared__ __attribute__((aligned(16))) T vs[DVT * 32 * VROW];
    const int b = blockIdx.z, g = blockIdx.y;
    const int R = H / G;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int c = lane & 31, h = lane >> 5;
    const int t0 = cu_q[b], qlen = cu_q[b + 1] - t0;
    const int ncols = qlen * R;
    if ((int)blockIdx.x * 4 * 32 >= ncols) return;  // the whole workgroup
    const int tile = blockIdx.x * 4 + wave;
    const bool tile_live = tile * 32 < ncols;
    const int ctx = ctx_lens[b];
    const int col = tile * 32 + c;
    const bool live = col < ncols;
    const int tq = live ? col / R : 0, r = live ? col % R : 0;
    const int pos = live ? ctx - qlen + tq : -1;
    const int my_pages = tile_live ? (ctx - qlen + min(tile * 32 + 31, ncols - 1) / R) / PAGE + 1 : 0;
    const int wg_last_col = min((int)blockIdx.x * 128 + 127, ncols - 1);
    const int wg_pages = (ctx - qlen + wg_last_col / R) / PAGE + 1;
    const int nks = dk >> 4, nvt = dv >> 5;
    const int lo = first_visible(ext, pos);
    const int wg_page0 = first_visible(ext, ctx - qlen + (int)blockIdx.x * 128 / R) / PAGE;
    const int my_page0 = tile_live ? first_visible(ext, ctx - qlen + tile * 32 / R) / PAGE : 0;
    // the workgroup's walk: pages with kept first positions that lie before its window pages, then those
    const int wg_nkeep = kept_units(ext, wg_page0, PAGE), wg_nvis = wg_nkeep + wg_pages - wg_page0;
    const float r1h = ext.r1 ? ext.r1[g * R + r] : 0.f, r2h = ext.r1 ? ext.r2[g * R + r] : 0.f;
    V8 qf[DK16];
    const T* qrow = q + (int64_t)(t0 + tq) * ldq + (int64_t)(g * R + r) * dk + h * 8;
#pragma unroll
    for (int s = 0; s < DK16; ++s) qf[s] = (live && s < nks) ? *reinterpret_cast<const V8*>(qrow + s * 16) : V8{};
    f32x16 O[DVT];
#pragma unroll
    for (int t = 0; t < DVT; ++t) O[t] = f32x16{};
    float m = -INFINITY, lsum = 0.f;
    const int32_t* table = bt + (int64_t)b * bt_ld;
    const int kelems = PAGE * dk, velems = dv * PAGE;
    V8 kreg[KL], vreg[VL];
    auto fetch = [&](int p) {
        const int64_t page = table[p];
        const T* kp = k_pool + (page * G + g) * (int64_t)kelems;
        const T* vp = v_pool + (page * G + g) * (int64_t)velems;
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int e = (tid + i * 256) * 8;
            kreg[i] = e < kelems ? *reinterpret_cast<const V8*>(kp + e) : V8{};
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int e = (tid + i * 256) * 8;
            vreg[i] = e < velems ? *reinterpret_cast<const V8*>(vp + e) : V8{};
        }
    };
    fetch(walk_unit(0, wg_nkeep, wg_page0));
    for (int pi = 0; pi < wg_nvis; ++pi) {
        const int p = walk_unit(pi, wg_nkeep, wg_page0);
        __syncthreads();  // the page before is consumed
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int e = (tid + i * 256) * 8;
            if (e < kelems) *reinterpret_cast<V8*>(ks + (e / dk) * KROW + (e % dk)) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int e = (tid + i * 256) * 8;
            if (e < velems) {
                T* dst = vs + (e / PAGE) * VROW + (e % PAGE);  // 8-byte aligned: two stores
                V4 lo, hi;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    lo[j] = vreg[i][j];
                    hi[j] = vreg[i][4 + j];
                }
                *reinterpret_cast<V4*>(dst) = lo;
                *reinterpret_cast<V4*>(dst + 4) = hi;
            }
        }
        __syncthreads();
        if (pi + 1 < wg_nvis) fetch(walk_unit(pi + 1, wg_nkeep, wg_page0));
        if (p >= my_pages || (p < my_page0 && p * PAGE >= ext.keep_first)) continue;
        f32x16 S = {};
#pragma unroll
        for (int s = 0; s < DK16; ++s)
            if (s < nks) S = mfma32(*reinterpret_cast<const V8*>(ks + c * KROW + s * 16 + h * 8), qf[s], S);
        const int base = p * PAGE + h * 4;
        float mx = -INFINITY;
        if (ext.r1) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = base + (i >> 2) * 8 + (i & 3);
                S[i] = key_visible(ext, key, pos, lo) ? S[i] * scale - r1h * __logf(1.f + r2h * (float)(pos - key)) : -INFINITY;
                mx = fmaxf(mx, S[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = base + (i >> 2) * 8 + (i & 3);
                S[i] = key_visible(ext, key, pos, lo) ? S[i] * scale : -INFINITY;
                mx = fmaxf(mx, S[i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m, mx);
        float corr = 1.f;
        if (mn == -INFINITY) {
#pragma unroll
            for (int i = 0; i < 16; ++i) S[i] = 0.f;
        } else {
            corr = expf(m - mn);
#pragma unroll
            for (int i = 0; i < 16; ++i) S[i] = expf(S[i] - mn);
        }
        m = mn;
        float ps = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) ps += S[i];
        lsum = lsum * corr + ps;
        V8 pb[2];
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
            for (int i = 0; i < 8; ++i) pb[c2][i] = (T)S[c2 * 8 + i];
#pragma unroll
        for (int t = 0; t < DVT; ++t)
            if (t < nvt) {
                if (corr != 1.f) O[t] *= corr;
                const T* vrow = vs + (t * 32 + c) * VROW + h * 4;
#pragma unroll
                for (int c2 = 0; c2 < 2; ++c2) {
                    const V4 v0 = *reinterpret_cast<const V4*>(vrow + c2 * 16);
                    const V4 v1 = *reinterpret_cast<const V4*>(vrow + c2 * 16 + 8);
                    V8 a;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        a[i] = v0[i];
                        a[4 + i] = v1[i];
                    }
                    O[t] = mfma32(a, pb[c2], O[t]);
                }
            }
    }
    lsum += __shfl_xor(lsum, 32, 64);
    if (!live) return;
    const float sink_f = fold_sink(ext, g * R + r, m, lsum);
    const float inv = sink_f / lsum * head_out_factor<T>(ext, t0 + tq, g * R + r);
    T* orow = out + (int64_t)(t0 + tq) * ld_out + (int64_t)(g * R + r) * dv + h * 4;
    const T* grow = (ext.gate && !ext.gate_per_head) ? reinterpret_cast<const T*>(ext.gate) + (int64_t)(t0 + tq) * ext.ld_gate + (int64_t)(g * R + r) * dv + h * 4 : nullptr;
#pragma unroll
    for (int t = 0; t < DVT; ++t)
        if (t < nvt) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                V4 o4, g4 = {};
                if (grow) g4 = *reinterpret_cast<const V4*>(grow + t * 32 + j * 8);
#pragma unroll
                for (int i = 0; i < 4; ++i) o4[i] = (T)(O[t][j * 4 + i] * inv * (grow ? sigmoid_f32((float)g4[i]) : 1.f));
                *reinterpret_cast<V4*>(orow + t * 32 + j * 8) = o4;
            }
        }
}


// ---- cache writes of designs that do not norm q and k ----------------------------------------------------------------
// grid (token, ceil(2 G / 4)): a wave per kv head.  Keys go to their page slot as they are; a value head is divided by its
// root mean square (v_norm, no gain) and written channel-major (v_inline: short steps) or back in place, for the transposing
// writer (v_write_kernel) of long steps.
template <typename T>
__global__ __launch_bounds__(256) void kv_norm_write_kernel(T* __restrict__ qkv, int64_t ld, int64_t k_col0, int64_t v_col0,
                                                            const int32_t* __restrict__ slots, T* __restrict__ k_pool,
                                                            T* __restrict__ v_pool, int G, int dk, int dv, int v_norm, float eps,
                                                            int v_inline) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int h = blockIdx.y * 4 + wave;
    if (h >= 2 * G) return;
    const int slot = slots[t];
    const int64_t page = slot / PAGE;
    const int off = slot % PAGE;
    T* row = qkv + t * ld;
    if (h < G) {
        const T* src = row + k_col0 + (int64_t)h * dk;
        T* dst = k_pool + ((page * G + h) * PAGE + off) * dk;
        for (int d = lane; d < dk; d += 64) dst[d] = src[d];
        return;
    }
    const int g = h - G;
    T* src = row + v_col0 + (int64_t)g * dv;
    float v[DV_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < DV_PER_LANE; ++c) {
        const int ch = lane + 64 * c;
        v[c] = ch < dv ? ldf(src + ch) : 0.f;
        ss += v[c] * v[c];
    }
    ss = wave_sum(ss);
    const float rinv = v_norm ? 1.0f / sqrtf(ss / (float)dv + eps) : 1.f;
#pragma unroll
    for (int c = 0; c < DV_PER_LANE; ++c) {
        const int ch = lane + 64 * c;
        if (ch < dv) {
            if (v_inline)
                v_pool[((page * G + g) * dv + ch) * PAGE + off] = (T)(v[c] * rinv);
            else
                src[ch] = (T)(v[c] * rinv);
        }
    }
}

// Latent attention: what a token leaves in the cache is its normed latent c (kv_rank channels) and one rotated key part shared
// by all heads (dr channels): the K page row is [c | rotated part] (one kv head of width kv_rank + dr), the V page is c,
// channel-major.  Queries arrive as [H][dn unrotated | dr to rotate]; their rotated part goes to columns kv_rank .. of the
// head's row of q_abs (the unrotated part is carried into latent space by a matrix product of the caller).
// Rotation: pair (2i, 2i + 1) of the first `rdims` channels turns by pos * inv_freq[i]; the rest pass unchanged.
// grid (token, 1 + ceil(H / 4)): block row 0 = the cache row (wave 0 the latent, wave 1 the rotated key), then a wave per head.
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(const T* __restrict__ q, int64_t ldq, T* __restrict__ ckv, int64_t ld_ckv,
                                                              const float* __restrict__ cw, const float* __restrict__ inv_freq,
                                                              const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                                                              T* __restrict__ q_abs, int64_t ld_qa, T* __restrict__ k_pool,
                                                              T* __restrict__ v_pool, int H, int dn, int dr, int rk, int rdims, float eps,
                                                              int v_inline) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const float pos = (float)positions[t];
    const int dkc = rk + dr;
    if (blockIdx.y == 0) {
        const int slot = slots[t];
        const int64_t page = slot / PAGE;
        const int off = slot % PAGE;
        T* krow = k_pool + (page * PAGE + off) * (int64_t)dkc;
        T* src = ckv + t * ld_ckv;
        if (wave == 0) {
            float ss = 0.f;
            for (int c = lane; c < rk; c += 64) {
                const float v = ldf(src + c);
                ss += v * v;
            }
            ss = wave_sum(ss);
            const float rinv = 1.0f / sqrtf(ss / (float)rk + eps);
            for (int c = lane; c < rk; c += 64) {
                const T y = (T)(ldf(src + c) * rinv * cw[c]);
                krow[c] = y;
                if (v_inline)
                    v_pool[(page * rk + c) * PAGE + off] = y;
                else
                    src[c] = y;
            }
        } else if (wave == 1) {
            const T* rsrc = src + rk;
            for (int i = lane; i < dr / 2; i += 64) {
                const float u = ldf(rsrc + 2 * i), v = ldf(rsrc + 2 * i + 1);
                float cs = 1.f, sn = 0.f;
                if (2 * i < rdims) sincosf(pos * inv_freq[i], &sn, &cs);
                krow[rk + 2 * i] = (T)(u * cs - v * sn);
                krow[rk + 2 * i + 1] = (T)(v * cs + u * sn);
            }
            if ((dr & 1) && lane == 0) krow[rk + dr - 1] = rsrc[dr - 1];
        }
        return;
    }
    const int h = (blockIdx.y - 1) * 4 + wave;
    if (h >= H) return;
    const T* qr = q + t * ldq + (int64_t)h * (dn + dr) + dn;
    T* dst = q_abs + t * ld_qa + (int64_t)h * dkc + rk;
    for (int i = lane; i < dr / 2; i += 64) {
        const float u = ldf(qr + 2 * i), v = ldf(qr + 2 * i + 1);
        float cs = 1.f, sn = 0.f;
        if (2 * i < rdims) sincosf(pos * inv_freq[i], &sn, &cs);
        dst[2 * i] = (T)(u * cs - v * sn);
        dst[2 * i + 1] = (T)(v * cs + u * sn);
    }
    if ((dr & 1) && lane == 0) dst[dr - 1] = qr[dr - 1];
}

// Rotation and cache write of designs that rotate q and k: pair (2i, 2i + 1) of the first `rdims` channels of every q and k
// head turns by position * inv_freq[i] (angle and sin / cos in fp32), the rest pass.  q is rotated in place, k goes to its
// page slot rotated, v to its slot as projected (v_inline) or stays for the transposing writer.
// grid (token, ceil((H + G) / 4) [+ value blocks]): a wave per q / k head.
template <typename T>
__global__ __launch_bounds__(256) void rope_rows_kv_write_kernel(T* __restrict__ qkv, int64_t ld, int64_t q_col0, int64_t k_col0,
                                                                 int64_t v_col0, const float* __restrict__ inv_freq,
                                                                 const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                                                                 T* __restrict__ k_pool, T* __restrict__ v_pool, int H, int G, int dk,
                                                                 int dv, int rdims, int v_inline, float unit_eps) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int slot = slots[t];
    const int64_t page = slot / PAGE;
    const int off = slot % PAGE;
    T* row = qkv + t * ld;
    const int head_blocks = (H + G + 3) / 4;
    if ((int)blockIdx.y >= head_blocks) {
        const T* vrow = row + v_col0;
        const int i0 = ((int)blockIdx.y - head_blocks) * 1024;
        const int i1 = min(i0 + 1024, G * dv);
        for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x) {
            const int g = i / dv, c = i - g * dv;
            v_pool[((page * G + g) * dv + c) * PAGE + off] = vrow[i];
        }
        return;
    }
    const int h = blockIdx.y * 4 + wave;
    if (h >= H + G) return;
    const bool is_q = h < H;
    T* src = is_q ? row + q_col0 + (int64_t)h * dk : row + k_col0 + (int64_t)(h - H) * dk;
    T* dst = is_q ? src : k_pool + ((page * G + (h - H)) * PAGE + off) * dk;
    const float pos = (float)positions[t];
    if (unit_eps >= 0.f) {
        // rotated, then divided by the head's root mean square (no gain): the rotated pairs wait in registers for the sum
        float u[2], v[2], ss = 0.f;  // dk <= 256: two pairs per lane
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int i = lane + 64 * r, d = 2 * i;
            u[r] = v[r] = 0.f;
            if (d < dk) {
                u[r] = ldf(src + d);
                v[r] = d + 1 < dk ? ldf(src + d + 1) : 0.f;
                if (d + 1 < rdims) {
                    float sn, cs;
                    sincosf(pos * inv_freq[i], &sn, &cs);
                    const float a = u[r] * cs - v[r] * sn, b2 = v[r] * cs + u[r] * sn;
                    u[r] = a;
                    v[r] = b2;
                }
                ss += u[r] * u[r] + v[r] * v[r];
            }
        }
        ss = wave_sum(ss);
        const float rinv = 1.f / sqrtf(ss / (float)dk + unit_eps);
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int d = 2 * (lane + 64 * r);
            if (d < dk) dst[d] = (T)(u[r] * rinv);
            if (d + 1 < dk) dst[d + 1] = (T)(v[r] * rinv);
        }
        return;
    }
    for (int i = lane; 2 * i < dk; i += 64) {
        const int d = 2 * i;
        if (d + 1 >= dk) {  // an odd width's last channel has no partner
            dst[d] = src[d];
            continue;
        }
        const float u = ldf(src + d), v = ldf(src + d + 1);
        if (d + 1 < rdims) {
            float sn, cs;
            sincosf(pos * inv_freq[i], &sn, &cs);
            dst[d] = (T)(u * cs - v * sn);
            dst[d + 1] = (T)(v * cs + u * sn);
        } else if (!is_q) {
            dst[d] = src[d];
            dst[d + 1] = src[d + 1];
        }
    }
}

template <typename T, int DK16, int DVT>
void launch_mfma_one(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* bt, int64_t bt_ld,
                     const int32_t* ctx_lens, const int32_t* cu_q, int B, void* out, int64_t ld_out, int64_t max_q_len, int H, int G,
                     int dk, int dv, float scale, int64_t max_ctx, AttnExt ext, hipStream_t st) {
    const int R = H / G;
    const bool split = max_q_len * R <= 32;
    // a windowed query walks its window's pages and the kept first ones, whatever the context
    if (ext.window > 0) max_ctx = std::min<int64_t>(max_ctx, (int64_t)ext.window + ext.keep_first + 2 * PAGE);
    int nw = 4;
    size_t lds = 0;
    unsigned gx = 1;
    int key_splits = 1;
    if (split && ext.partial && (int64_t)B * G < 128) {
        // few (sequence, cached head) pairs: deal a sequence's pages to several workgroups of four waves, a page or two
        // per wave at least, about one workgroup per compute unit in all
        const int64_t pages = cdiv64(max_ctx, PAGE);
        int64_t want = 256 / ((int64_t)B * G);
        if (want > cdiv64(pages, 4)) want = cdiv64(pages, 4);
        const int64_t fits = ext.partial_tokens > 0 ? ext.key_splits : 1;  // on entry: the splits the caller's buffer holds
        if (want > fits) want = fits;
        if (want > 1) key_splits = (int)want;
    }
    ext.key_splits = key_splits;
    if (split) {
        gx = (unsigned)key_splits;
        const size_t per_wave = (128 + (size_t)DVT * 16 * 64) * sizeof(float);
        // eight waves share a tile's pages when the contexts are long or the grid alone would leave most of the chip idle
        nw = (key_splits == 1 && (max_ctx > 2048 || (int64_t)B * G < 512) && max_ctx > 4 * PAGE && 8 * per_wave <= 150 * 1024) ? 8 : 4;
        lds = nw * per_wave;
        if (lds > 48 * 1024)
            (void)hipFuncSetAttribute((const void*)attn_varlen_mfma_kernel<T, DK16, DVT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    } else {
        gx = (unsigned)cdiv64(cdiv64(max_q_len * R, 32), nw);
        // Measured (4 x 1024-token prompts): staging wins for narrow heads (dk 64 / dv 64, R 8: 2.96 ms against 3.20 for 22 layers)
        // and loses for wide ones (dk 128 / dv 128, MHA: 10.4 against 8.4 ms for 32 layers: two barriers per page and one LDS
        // buffer cost more than the second trip to L1 saves), so wide heads keep taking their fragments straight from L2 / L1.
        static const bool direct = getenv("TGIS_ATTN_VARLEN_DIRECT") != nullptr;  // A/B switch
        if (!direct && DK16 <= 4 && DVT <= 2) {
            hipLaunchKernelGGL((attn_varlen_staged_kernel<T, DK16, DVT>), dim3(gx, (unsigned)G, (unsigned)B), dim3(256), 0, st,
                               (const T*)q, ldq, (const T*)k_pool, (const T*)v_pool, bt, bt_ld, ctx_lens, cu_q, (T*)out, ld_out, H, G,
                               dk, dv, scale, ext);
            return;
        }
    }
    hipLaunchKernelGGL((attn_varlen_mfma_kernel<T, DK16, DVT>), dim3(gx, (unsigned)G, (unsigned)B), dim3(64 * nw), lds, st,
                       (const T*)q, ldq, (const T*)k_pool, (const T*)v_pool, bt, bt_ld, ctx_lens, cu_q, (T*)out, ld_out, H, G, dk, dv,
                       scale, split ? 1 : 0, ext);
    if (key_splits > 1)
        hipLaunchKernelGGL(attn_combine_splits_kernel<T>, dim3((unsigned)ext.partial_tokens, (unsigned)H), dim3(64), 0, st, ext.partial,
                           key_splits, ext.partial_tokens, H, dv, (T*)out, ld_out, ext);
}

template <typename T, int DK16>
void launch_mfma_dv(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* bt, int64_t bt_ld,
                    const int32_t* ctx_lens, const int32_t* cu_q, int B, void* out, int64_t ld_out, int64_t max_q_len, int H, int G,
                    int dk, int dv, float scale, int64_t max_ctx, AttnExt ext, hipStream_t st) {
    const int nvt = dv / 32;
    if (nvt <= 1)
        launch_mfma_one<T, DK16, 1>(q, ldq, k_pool, v_pool, bt, bt_ld, ctx_lens, cu_q, B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
    else if (nvt <= 2)
        launch_mfma_one<T, DK16, 2>(q, ldq, k_pool, v_pool, bt, bt_ld, ctx_lens, cu_q, B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
    else if (nvt <= 4)
        launch_mfma_one<T, DK16, 4>(q, ldq, k_pool, v_pool, bt, bt_ld, ctx_lens, cu_q, B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
    else
        launch_mfma_one<T, DK16, 8>(q, ldq, k_pool, v_pool, bt, bt_ld, ctx_lens, cu_q, B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
}

template <typename T>
void launch_mfma(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* bt, int64_t bt_ld,
                 const int32_t* ctx_lens, const int32_t* cu_q, int B, void* out, int64_t ld_out, int64_t max_q_len, int H, int G, int dk,
                 int dv, float scale, int64_t max_ctx, AttnExt ext, hipStream_t st) {
    if (dk <= 64)
        launch_mfma_dv<T, 4>(q, ldq, k_pool, v_pool, bt, bt_ld, ctx_lens, cu_q, B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
    else if (dk <= 128)
        launch_mfma_dv<T, 8>(q, ldq, k_pool, v_pool, bt, bt_ld, ctx_lens, cu_q, B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
    else
        launch_mfma_dv<T, 16>(q, ldq, k_pool, v_pool, bt, bt_ld, ctx_lens, cu_q, B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
}

template <typename T>
int launch_prep(void* qkv, int64_t ld, const int32_t* positions, const int32_t* slots, const float* qw, const float* kw, float eps,
                float gain_coef, int gain_every, const void* v_first, int64_t ld_vf, const float* lam, void* k_pool, void* v_pool,
                int64_t T_, int H, int G, int dk, int dv, hipStream_t st) {
    // steps of a few hundred tokens at most (decode, small mixes): values leave from the q / k launch; longer ones (prompt
    // portions) take the transposing writer, whose stores are whole page rows
    const int v_inline = T_ < 512 ? 1 : 0;
    const int v_blocks = v_inline ? (int)cdiv64((int64_t)G * dv, 1024) : 0;
    hipLaunchKernelGGL(qk_norm_kv_write_kernel<T>, dim3((unsigned)T_, (unsigned)((H + G + 3) / 4 + v_blocks)), dim3(256), 0, st, (T*)qkv, ld,
                       positions, slots, qw, kw, eps, gain_coef, gain_every, (const T*)v_first, ld_vf, lam, (T*)k_pool, (T*)v_pool, H, G, dk,
                       dv, v_inline);
    if (!v_inline)
        hipLaunchKernelGGL(v_write_kernel<T>, dim3((unsigned)cdiv64(T_, 32), (unsigned)cdiv64((int64_t)G * dv, 64)), dim3(256), 0, st,
                           (const T*)qkv, ld, (int64_t)(H + G) * dk, slots, (const T*)v_first, ld_vf, lam, (T*)v_pool, T_, G, dv);
    return 0;
}

template <typename T>
int launch_attn(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* bt, int64_t bt_ld,
                const int32_t* ctx_lens, const int32_t* cu_q, int B, void* out, int64_t ld_out, int64_t Tq, int H, int G, int dk,
                int dv, float scale, int S, AttnExt ext, hipStream_t st) {
    const int Rall = H / G, R = Rall < 16 ? Rall : 16, nsub = (Rall + 15) / 16;
    const size_t lds = ((size_t)R * dk + (size_t)R * S * (2 + dv)) * sizeof(float);
    hipLaunchKernelGGL(attn_varlen_kernel<T>, dim3((unsigned)Tq, (unsigned)(G * nsub)), dim3(64 * R * S), lds, st, (const T*)q, ldq,
                       (const T*)k_pool, (const T*)v_pool, bt, bt_ld, ctx_lens, cu_q, B, (T*)out, ld_out, H, G, dk, dv, scale, S, ext);
    return 0;
}

}  // namespace

extern "C" int tgis_qk_norm_kv_write(void* qkv, int64_t ld, const int32_t* positions, const int32_t* slots, const float* q_gain,
                                     const float* k_gain, float eps, float gain_coef, int gain_every, const void* v_first,
                                     int64_t ld_v_first, const float* v_lambda, void* k_pool, void* v_pool, int64_t T, int H, int G,
                                     int dk, int dv, int dtype, void* stream) {
    TGIS_CHECK_ARG(qkv && positions && slots && q_gain && k_gain && k_pool && v_pool, "tgis_qk_norm_kv_write: null tensor");
    TGIS_CHECK_ARG(H >= 1 && G >= 1 && H % G == 0 && dk >= 1 && dv >= 1 && ld >= (int64_t)(H + G) * dk + (int64_t)G * dv,
                   "tgis_qk_norm_kv_write: bad head geometry (H %d, G %d, dk %d, dv %d, ld %ld)", H, G, dk, dv, (long)ld);
    TGIS_CHECK_ARG(!v_first || (v_lambda && ld_v_first >= (int64_t)G * dv), "tgis_qk_norm_kv_write: blending needs lambda and a row stride");
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_qk_norm_kv_write: bad dtype");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ROPE_KV, st);
    if (dtype == TGIS_F16)
        launch_prep<f16>(qkv, ld, positions, slots, q_gain, k_gain, eps, gain_coef, gain_every, v_first, ld_v_first, v_lambda, k_pool, v_pool, T, H, G, dk, dv, st);
    else if (dtype == TGIS_BF16)
        launch_prep<bf16>(qkv, ld, positions, slots, q_gain, k_gain, eps, gain_coef, gain_every, v_first, ld_v_first, v_lambda, k_pool, v_pool, T, H, G, dk, dv, st);
    else
        launch_prep<float>(qkv, ld, positions, slots, q_gain, k_gain, eps, gain_coef, gain_every, v_first, ld_v_first, v_lambda, k_pool, v_pool, T, H, G, dk, dv, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

static int attn_varlen_impl(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                            int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B, void* out,
                            int64_t ld_out, int64_t total_q, int64_t max_q_len, int64_t max_ctx, int H, int G, int dk, int dv,
                            float scale, int impl, int dtype, AttnExt ext, void* stream) {
    TGIS_CHECK_ARG(q && k_pool && v_pool && block_tables && ctx_lens && cu_seqlens_q && out, "tgis_attn_varlen: null tensor");
    TGIS_CHECK_ARG(H >= 1 && G >= 1 && H % G == 0, "tgis_attn_varlen: needs H a multiple of G");
    TGIS_CHECK_ARG(dk >= 1 && dv >= 1 && dv <= 64 * DV_PER_LANE, "tgis_attn_varlen: value width %d exceeds %d", dv, 64 * DV_PER_LANE);
    TGIS_CHECK_ARG(ldq >= (int64_t)H * dk && ld_out >= (int64_t)H * dv && max_pages > 0 && B >= 1, "tgis_attn_varlen: bad strides");
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_attn_varlen: bad dtype");
    TGIS_CHECK_ARG(dtype == TGIS_F32 ? ((dk & 3) != 0 || (((uintptr_t)k_pool) & 15) == 0) : ((dk & 7) != 0 || (((uintptr_t)k_pool) & 15) == 0),
                   "tgis_attn_varlen: the key pool must be 16-byte aligned");
    TGIS_CHECK_ARG(impl >= 0 && impl <= 2 && max_q_len >= 1 && max_ctx >= 1, "tgis_attn_varlen: impl 0 (auto), 1 (general), 2 (matrix cores); max_q_len, max_ctx >= 1");
    if (total_q == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ATTN, st);
    const bool mfma_ok = dtype != TGIS_F32 && dk % 16 == 0 && dv % 32 == 0 && dk <= 256 && dv <= 256 && ldq % 8 == 0 &&
                         (((uintptr_t)q | (uintptr_t)k_pool | (uintptr_t)v_pool | (uintptr_t)out) & 15) == 0 && ld_out % 4 == 0 &&
                         B <= 65535 && G <= 65535;
    TGIS_CHECK_ARG(impl != 2 || mfma_ok, "tgis_attn_varlen: the matrix-core kernel needs a two-byte dtype, dk %% 16 == 0, dv %% 32 == 0, both <= 256, aligned operands");
    if (mfma_ok && impl != 1) {
        if (dtype == TGIS_F16)
            launch_mfma<f16>(q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, (int)B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
        else
            launch_mfma<bf16>(q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, (int)B, out, ld_out, max_q_len, H, G, dk, dv, scale, max_ctx, ext, st);
        TGIS_CHECK_LAUNCH();
        return TGIS_OK;
    }
    const int R = H / G < 16 ? H / G : 16;  // query heads per workgroup (larger groups take several workgroups)
    int S = 16 / R;  // waves per workgroup: R * S <= 16
    if (S > 4) S = 4;
    if (S < 1) S = 1;
    const size_t lds = ((size_t)R * dk + (size_t)R * S * (2 + dv)) * sizeof(float);
    TGIS_CHECK_ARG(lds <= 64 * 1024, "tgis_attn_varlen: head geometry needs %ld bytes of LDS", (long)lds);
    if (dtype == TGIS_F16)
        launch_attn<f16>(q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, (int)B, out, ld_out, total_q, H, G, dk, dv, scale, S, ext, st);
    else if (dtype == TGIS_BF16)
        launch_attn<bf16>(q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, (int)B, out, ld_out, total_q, H, G, dk, dv, scale, S, ext, st);
    else
        launch_attn<float>(q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, (int)B, out, ld_out, total_q, H, G, dk, dv, scale, S, ext, st);
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_attn_varlen(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                                int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B, void* out,
                                int64_t ld_out, int64_t total_q, int64_t max_q_len, int64_t max_ctx, int H, int G, int dk, int dv,
                                float scale, int impl, int dtype, void* stream) {
    return attn_varlen_impl(q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, B, out, ld_out, total_q, max_q_len,
                            max_ctx, H, G, dk, dv, scale, impl, dtype, AttnExt{nullptr, nullptr, 0, nullptr, 0, 0, nullptr, 0}, stream);
}

// The same with a block mask (chunk > 0: a query sees its own block of `chunk` positions only), a distance bias per query
// head (r1, r2 [H] fp32, both or neither: the score loses r1 ln(1 + r2 (i - j))) and / or a sigmoid output gate
// (gate [T, >= H dv] in the activation dtype: out *= sigmoid(gate), applied where the output is written).
// workspace (optional, 16-byte aligned): scratch for the partial results of decode steps whose pages are dealt to several
// workgroups (few sequences x cached heads); splits * total_q * H * (dv + 2) * 4 bytes are used, as many splits as fit.
extern "C" int tgis_attn_varlen_ext(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                                    int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B, void* out,
                                    int64_t ld_out, int64_t total_q, int64_t max_q_len, int64_t max_ctx, int H, int G, int dk, int dv,
                                    float scale, const float* r1, const float* r2, int chunk, const void* gate, int64_t ld_gate,
                                    void* workspace, int64_t workspace_bytes, int impl, int dtype, void* stream) {
    TGIS_CHECK_ARG((r1 == nullptr) == (r2 == nullptr) && chunk >= 0, "tgis_attn_varlen_ext: r1 and r2 come together; chunk >= 0");
    TGIS_CHECK_ARG(!gate || (ld_gate >= (int64_t)H * dv && (dtype == TGIS_F32 || (ld_gate % 4 == 0 && ((uintptr_t)gate & 7) == 0))),
                   "tgis_attn_varlen_ext: the gate needs a row stride >= H dv and 8-byte aligned rows");
    return attn_varlen_impl(q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, B, out, ld_out, total_q, max_q_len,
                            max_ctx, H, G, dk, dv, scale, impl, dtype, AttnExt{r1, r2, chunk, gate, ld_gate,
                                    // how many key splits of this step the caller's scratch buffer can hold (the launcher decides)
                                    (int)std::min<int64_t>(64, workspace && ((uintptr_t)workspace & 15) == 0 ? workspace_bytes / std::max<int64_t>(1, total_q * H * (int64_t)(dv + 2) * 4) : 0),
                                    (float*)workspace, total_q},
                            stream);
}

#define TGIS_ATTN_BY_DTYPE(dtype, ...)                               \
    do {                                                             \
        if ((dtype) == TGIS_F16) { using TT = f16; __VA_ARGS__; }        \
        else if ((dtype) == TGIS_BF16) { using TT = bf16; __VA_ARGS__; } \
        else { using TT = float; __VA_ARGS__; }                      \
    } while (0)

// Keys (as projected) and values (v_norm: each head divided by its root mean square, eps inside the root, no gain) of a step
// into their page slots.  qkv [T, ld]: keys at columns k_col0 + g dk, values at v_col0 + g dv; values are normed in place when
// the step is long enough for the transposing writer.
extern "C" int tgis_kv_norm_write(void* qkv, int64_t ld, int64_t k_col0, int64_t v_col0, const int32_t* slots, void* k_pool,
                                  void* v_pool, int64_t T, int G, int dk, int dv, int v_norm, float eps, int dtype, void* stream) {
    TGIS_CHECK_ARG(qkv && slots && k_pool && v_pool, "tgis_kv_norm_write: null tensor");
    TGIS_CHECK_ARG(G >= 1 && dk >= 1 && dv >= 1 && dv <= 64 * DV_PER_LANE && k_col0 >= 0 && v_col0 >= 0 &&
                       ld >= k_col0 + (int64_t)G * dk && ld >= v_col0 + (int64_t)G * dv,
                   "tgis_kv_norm_write: bad geometry (G %d, dk %d, dv %d <= %d, ld %ld)", G, dk, dv, 64 * DV_PER_LANE, (long)ld);
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_kv_norm_write: bad dtype");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ROPE_KV, st);
    const int v_inline = T < 512 ? 1 : 0;
    TGIS_ATTN_BY_DTYPE(dtype, hipLaunchKernelGGL(kv_norm_write_kernel<TT>, dim3((unsigned)T, (unsigned)((2 * G + 3) / 4)), dim3(256), 0, st,
                                                 (TT*)qkv, ld, k_col0, v_col0, slots, (TT*)k_pool, (TT*)v_pool, G, dk, dv, v_norm, eps, v_inline));
    if (!v_inline)
        TGIS_ATTN_BY_DTYPE(dtype, hipLaunchKernelGGL(v_write_kernel<TT>, dim3((unsigned)cdiv64(T, 32), (unsigned)cdiv64((int64_t)G * dv, 64)),
                                                     dim3(256), 0, st, (const TT*)qkv, ld, v_col0, slots, (const TT*)nullptr, (int64_t)0,
                                                     (const float*)nullptr, (TT*)v_pool, T, G, dv));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// The cache row and the rotated query parts of a latent-attention step (see latent_kv_write_kernel).  ckv [T, >= kv_rank + dr]
// is the down-projection (its first kv_rank columns are normed in place on long steps); q [T, H (dn + dr)];
// q_abs [T, H (kv_rank + dr)] receives the rotated parts; the pools are those of ONE kv head with key width kv_rank + dr and
// value width kv_rank.
extern "C" int tgis_latent_kv_write(const void* q, int64_t ldq, void* ckv, int64_t ld_ckv, const float* c_gain, const float* inv_freq,
                                    const int32_t* positions, const int32_t* slots, void* q_abs, int64_t ld_q_abs, void* k_pool,
                                    void* v_pool, int64_t T, int H, int dn, int dr, int kv_rank, int rot_dims, float eps, int dtype,
                                    void* stream) {
    TGIS_CHECK_ARG(q && ckv && c_gain && inv_freq && positions && slots && q_abs && k_pool && v_pool, "tgis_latent_kv_write: null tensor");
    TGIS_CHECK_ARG(H >= 1 && dn >= 0 && dr >= 0 && kv_rank >= 1 && rot_dims >= 0 && rot_dims <= dr && rot_dims % 2 == 0 &&
                       ldq >= (int64_t)H * (dn + dr) && ld_ckv >= kv_rank + dr && ld_q_abs >= (int64_t)H * (kv_rank + dr),
                   "tgis_latent_kv_write: bad geometry (H %d, dn %d, dr %d, kv_rank %d, rot_dims %d)", H, dn, dr, kv_rank, rot_dims);
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_latent_kv_write: bad dtype");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ROPE_KV, st);
    const int v_inline = T < 512 ? 1 : 0;
    TGIS_ATTN_BY_DTYPE(dtype, hipLaunchKernelGGL(latent_kv_write_kernel<TT>, dim3((unsigned)T, (unsigned)(1 + (H + 3) / 4)), dim3(256), 0, st,
                                                 (const TT*)q, ldq, (TT*)ckv, ld_ckv, c_gain, inv_freq, positions, slots, (TT*)q_abs, ld_q_abs,
                                                 (TT*)k_pool, (TT*)v_pool, H, dn, dr, kv_rank, rot_dims, eps, v_inline));
    if (!v_inline)
        TGIS_ATTN_BY_DTYPE(dtype, hipLaunchKernelGGL(v_write_kernel<TT>, dim3((unsigned)cdiv64(T, 32), (unsigned)cdiv64((int64_t)kv_rank, 64)),
                                                     dim3(256), 0, st, (const TT*)ckv, ld_ckv, (int64_t)0, slots, (const TT*)nullptr, (int64_t)0,
                                                     (const float*)nullptr, (TT*)v_pool, T, 1, kv_rank));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

// Interleaved-pair rotation of q (in place) and k (into its page slot) and the value write of a step, for the "rows" page
// layout of tgis_attn_varlen.  proj [T, ld] holds q at columns q_col0 + h dk, k at k_col0 + g dk, v at v_col0 + g dv; pair
// (2i, 2i + 1) of the first rot_dims channels of every head turns by positions[t] * inv_freq[i] (fp32 angle), the rest pass.
static int rope_rows_impl(void* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, const float* inv_freq,
                          const int32_t* positions, const int32_t* slots, void* k_pool, void* v_pool, int64_t T, int H,
                          int G, int dk, int dv, int rot_dims, float unit_eps, int dtype, void* stream) {
    TGIS_CHECK_ARG(proj && positions && slots && k_pool && v_pool && (inv_freq || rot_dims == 0), "tgis_rope_rows_kv_write: null tensor");
    TGIS_CHECK_ARG(H >= 1 && G >= 1 && dk >= 1 && dv >= 1 && rot_dims >= 0 && rot_dims <= dk && rot_dims % 2 == 0 && q_col0 >= 0 &&
                       k_col0 >= 0 && v_col0 >= 0 && ld >= q_col0 + (int64_t)H * dk && ld >= k_col0 + (int64_t)G * dk &&
                       ld >= v_col0 + (int64_t)G * dv,
                   "tgis_rope_rows_kv_write: bad geometry (H %d, G %d, dk %d, dv %d, rot_dims %d, ld %ld)", H, G, dk, dv, rot_dims, (long)ld);
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_rope_rows_kv_write: bad dtype");
    if (T == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ROPE_KV, st);
    const int v_inline = T < 512 ? 1 : 0;
    const int v_blocks = v_inline ? (int)cdiv64((int64_t)G * dv, 1024) : 0;
    TGIS_ATTN_BY_DTYPE(dtype, hipLaunchKernelGGL(rope_rows_kv_write_kernel<TT>, dim3((unsigned)T, (unsigned)((H + G + 3) / 4 + v_blocks)), dim3(256),
                                                 0, st, (TT*)proj, ld, q_col0, k_col0, v_col0, inv_freq, positions, slots, (TT*)k_pool,
                                                 (TT*)v_pool, H, G, dk, dv, rot_dims, v_inline, unit_eps));
    if (!v_inline)
        TGIS_ATTN_BY_DTYPE(dtype, hipLaunchKernelGGL(v_write_kernel<TT>, dim3((unsigned)cdiv64(T, 32), (unsigned)cdiv64((int64_t)G * dv, 64)),
                                                     dim3(256), 0, st, (const TT*)proj, ld, v_col0, slots, (const TT*)nullptr, (int64_t)0,
                                                     (const float*)nullptr, (TT*)v_pool, T, G, dv));
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}

extern "C" int tgis_rope_rows_kv_write(void* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, const float* inv_freq,
                                       const int32_t* positions, const int32_t* slots, void* k_pool, void* v_pool, int64_t T, int H,
                                       int G, int dk, int dv, int rot_dims, int dtype, void* stream) {
    return rope_rows_impl(proj, ld, q_col0, k_col0, v_col0, inv_freq, positions, slots, k_pool, v_pool, T, H, G, dk, dv, rot_dims, -1.f, dtype, stream);
}

// The same, and every q and k head is divided by its root mean square (sqrt(mean(x^2) + unit_eps), no gain) after the rotation.
extern "C" int tgis_rope_rows_unit_kv_write(void* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, const float* inv_freq,
                                            const int32_t* positions, const int32_t* slots, void* k_pool, void* v_pool, int64_t T, int H,
                                            int G, int dk, int dv, int rot_dims, float unit_eps, int dtype, void* stream) {
    TGIS_CHECK_ARG(unit_eps >= 0.f && dk <= 256, "tgis_rope_rows_unit_kv_write: heads of up to 256 channels, eps >= 0");
    return rope_rows_impl(proj, ld, q_col0, k_col0, v_col0, inv_freq, positions, slots, k_pool, v_pool, T, H, G, dk, dv, rot_dims, unit_eps, dtype, stream);
}

// tgis_attn_varlen with a sliding window that also keeps the first positions (window > 0: position i sees j <= i only if
// i - j < window or j < keep_first; pages between the kept ones and the window are never touched), a sink logit per query head
// in the softmax denominator (sink [H] fp32 or NULL), a sigmoid output gate (gate_per_head: one number per (token, head),
// gate [T, >= H]; else one per channel, gate [T, >= H dv]) and a constant factor on the output.  out may be a column range of
// a wider buffer (ld_out).  workspace: as for tgis_attn_varlen_ext.
extern "C" int tgis_attn_varlen_win(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                                    int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B, void* out,
                                    int64_t ld_out, int64_t total_q, int64_t max_q_len, int64_t max_ctx, int H, int G, int dk, int dv,
                                    float scale, int window, int keep_first, const float* sink, const void* gate, int64_t ld_gate,
                                    int gate_per_head, float out_scale, void* workspace, int64_t workspace_bytes, int impl, int dtype,
                                    void* stream) {
    TGIS_CHECK_ARG(window >= 0 && keep_first >= 0 && (window > 0 || keep_first == 0), "tgis_attn_varlen_win: kept first positions need a window");
    TGIS_CHECK_ARG(!gate || (gate_per_head ? ld_gate >= H
                                           : (ld_gate >= (int64_t)H * dv && (dtype == TGIS_F32 || (ld_gate % 4 == 0 && ((uintptr_t)gate & 7) == 0)))),
                   "tgis_attn_varlen_win: the gate needs a row stride >= H (per head) or >= H dv with 8-byte aligned rows");
    AttnExt ext{nullptr, nullptr, 0, gate, ld_gate,
                (int)std::min<int64_t>(64, workspace && ((uintptr_t)workspace & 15) == 0 ? workspace_bytes / std::max<int64_t>(1, total_q * H * (int64_t)(dv + 2) * 4) : 0),
                (float*)workspace, total_q};
    ext.window = window;
    ext.keep_first = keep_first;
    ext.sink = sink;
    ext.gate_per_head = gate_per_head ? 1 : 0;
    ext.out_scale = out_scale;
    return attn_varlen_impl(q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, B, out, ld_out, total_q, max_q_len,
                            max_ctx, H, G, dk, dv, scale, impl, dtype, ext, stream);
}
