// Paged softmax attention whose scores are mixed over the query heads BEFORE the softmax ("talking heads"):
//
//     s_g(i, j) = scale * q_g(i) . k_kv(g)(j)                 raw score of head g (kv head floor(g / (H / G)))
//     s'_h(i, j) = sum_g M[h][g] s_g(i, j)                     M [H, H] fp32
//     p_h(i, .) = softmax over the visible j of s'_h(i, .)     j <= i, and i - j < window when window > 0
//     o_h(i) = sum_j p_h(i, j) v_kv(h)(j)                      times sigmoid(gate[i][h dv + c]) when a gate is given
//
// A weight of head h needs the raw scores of ALL heads for its (query, key) pair, so a workgroup owns every head of a tile of
// QT consecutive query tokens of one sequence and walks the pages the tile can see (the window's, not the context's).  Per page
// of 32 keys: the raw scores [H][QT][32] (a thread per (head, key), the tile's queries from LDS, the key row from the page, fp32
// sums), the mix (a thread per (head, key) again, M's row against the column of raw scores in LDS), an online softmax per
// (head, query) over the half wave that holds its 32 keys, and the products with the values (a thread per (head, value channel):
// the page's value rows are channel-major, 32 tokens contiguous).  Scores, weights, statistics and sums are fp32 whatever the
// cache dtype T is.  The same kernel serves prompt portions (QT up to 8) and decode steps (QT = 1).
//
// Cache pages: the "rows" layout of tgis_attn_varlen — k_pool[page][kv head][token][dk], v_pool[page][kv head][dv][token].
#include <stdlib.h>
#include <algorithm>
#include "common.h"

namespace {

constexpr int PAGE = TGIS_KV_PAGE_TOKENS;
constexpr int THREADS = 256;

struct MixArgs {
    const void* q;
    int64_t ldq;
    const void* k_pool;
    const void* v_pool;
    const int32_t* bt;
    int64_t bt_ld;
    const int32_t* ctx_lens;
    const int32_t* cu_q;
    const float* mix;  // [H][H]
    const void* gate;
    int64_t ld_gate;
    void* out;
    int64_t ld_out;
    int H, G, dk, dv, window;
    float scale;
};

template <typename T> struct Vec16;
template <> struct Vec16<float> { static constexpr int N = 4; typedef f32x4 type; };
template <> struct Vec16<bf16> { static constexpr int N = 8; typedef bf16x8 type; };
template <> struct Vec16<f16> { static constexpr int N = 8; typedef f16x8 type; };

// OPT: output (head, channel) pairs a thread accumulates (H dv <= OPT * THREADS)
template <typename T, int QT, int OPT>
__global__ __launch_bounds__(THREADS) void attn_mixed_heads_kernel(MixArgs a) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int H = a.H, G = a.G, dk = a.dk, dv = a.dv, R = H / G;
    const int b = blockIdx.y;
    const int t0 = a.cu_q[b], qlen = a.cu_q[b + 1] - t0;
    const int first = blockIdx.x * QT;
    if (first >= qlen) return;
    const int nq = min(QT, qlen - first);
    const int ctx = a.ctx_lens[b];
    const int pos0 = ctx - qlen + first;  // position of the tile's first query
    const int tid = threadIdx.x;
    const int dkp = (dk + 3) & ~3;
    float* qs = smem;                           // [QT][H][dkp]
    float* raw = qs + QT * H * dkp;             // [H][QT][PAGE]
    float* pw = raw + H * QT * PAGE;            // [H][QT][PAGE] weights of the page
    float* fac = pw + H * QT * PAGE;            // [H][QT] what the sums so far are multiplied by
    float* lsum = fac + H * QT;                 // [H][QT] final denominators
    const T* q = reinterpret_cast<const T*>(a.q);
    for (int e = tid; e < QT * H * dkp; e += THREADS) {
        const int qi = e / (H * dkp), r = e - qi * H * dkp, h = r / dkp, d = r - h * dkp;
        qs[e] = (qi < nq && d < dk) ? (float)q[(int64_t)(t0 + first + qi) * a.ldq + (int64_t)h * dk + d] * a.scale : 0.f;
    }
    // a pair (head, key of the page) per thread and trip: keys are the fast index, so a half wave holds one head's 32 keys
    const int pairs = H * PAGE;
    const int trips = (pairs + THREADS - 1) / THREADS;
    // running statistics of (head, query): read by the half wave that holds the head's keys, written by its first lane
    float* mrun = lsum + H * QT;                // [H][QT]
    float* lrun = mrun + H * QT;                // [H][QT]
    float* mixs = lrun + H * QT;                // [H][H] the mixing matrix
    for (int e = tid; e < H * QT; e += THREADS) {
        mrun[e] = -INFINITY;
        lrun[e] = 0.f;
    }
    for (int e = tid; e < H * H; e += THREADS) mixs[e] = a.mix[e];
    // heads a thread mixes for its key: with many heads a column of raw scores is read once for HB of them
    const int HB = H % 4 == 0 && H >= 32 ? 4 : (H % 2 == 0 && H >= 16 ? 2 : 1);
    float acc[OPT][QT];
#pragma unroll
    for (int o = 0; o < OPT; ++o)
#pragma unroll
        for (int qi = 0; qi < QT; ++qi) acc[o][qi] = 0.f;
    const int lo_first = a.window > 0 ? max(pos0 - a.window + 1, 0) : 0;
    const int last_pos = pos0 + nq - 1;
    const T* kp = reinterpret_cast<const T*>(a.k_pool);
    const T* vp = reinterpret_cast<const T*>(a.v_pool);
    constexpr int VN = Vec16<T>::N;
    typedef typename Vec16<T>::type VT;
    const bool k_vec = dk % VN == 0;
    __syncthreads();
    for (int pg = lo_first / PAGE; pg <= last_pos / PAGE; ++pg) {
        const int64_t page = a.bt[(int64_t)b * a.bt_ld + pg];
        const int key0 = pg * PAGE;
        // ---- raw scores ----
        for (int tr = 0; tr < trips; ++tr) {
            const int pr = tid + tr * THREADS;
            if (pr >= pairs) break;
            const int h = pr / PAGE, j = pr % PAGE;
            const T* krow = kp + ((page * G + h / R) * PAGE + j) * (int64_t)dk;
            float s[QT];
#pragma unroll
            for (int qi = 0; qi < QT; ++qi) s[qi] = 0.f;
            if (key0 + j <= last_pos) {
                if (k_vec) {
                    for (int d = 0; d < dk; d += VN) {
                        const VT kv = *reinterpret_cast<const VT*>(krow + d);
#pragma unroll
                        for (int qi = 0; qi < QT; ++qi) {
                            const float* qq = qs + (qi * H + h) * dkp + d;
#pragma unroll
                            for (int u = 0; u < VN; u += 4) {
                                const f32x4 q4 = *reinterpret_cast<const f32x4*>(qq + u);
                                s[qi] = fmaf((float)kv[u], q4[0], s[qi]);
                                s[qi] = fmaf((float)kv[u + 1], q4[1], s[qi]);
                                s[qi] = fmaf((float)kv[u + 2], q4[2], s[qi]);
                                s[qi] = fmaf((float)kv[u + 3], q4[3], s[qi]);
                            }
                        }
                    }
                } else {
                    for (int d = 0; d < dk; ++d) {
                        const float kf = (float)krow[d];
#pragma unroll
                        for (int qi = 0; qi < QT; ++qi) s[qi] = fmaf(kf, qs[(qi * H + h) * dkp + d], s[qi]);
                    }
                }
            }
#pragma unroll
            for (int qi = 0; qi < QT; ++qi) raw[(h * QT + qi) * PAGE + j] = s[qi];
        }
        __syncthreads();
        // ---- mix over heads, mask, online softmax ----
        for (int pr = tid; pr < (H / HB) * PAGE; pr += THREADS) {  // whole half waves leave together
            const int h0 = pr / PAGE * HB, j = pr % PAGE;
            float s[4][QT];
#pragma unroll
            for (int hb = 0; hb < 4; ++hb)
#pragma unroll
                for (int qi = 0; qi < QT; ++qi) s[hb][qi] = 0.f;
            for (int g = 0; g < H; ++g) {
                float r[QT];
#pragma unroll
                for (int qi = 0; qi < QT; ++qi) r[qi] = raw[(g * QT + qi) * PAGE + j];
#pragma unroll
                for (int hb = 0; hb < 4; ++hb)
                    if (hb < HB) {
                        const float m = mixs[(h0 + hb) * H + g];
#pragma unroll
                        for (int qi = 0; qi < QT; ++qi) s[hb][qi] = fmaf(m, r[qi], s[hb][qi]);
                    }
            }
            const int key = key0 + j;
#pragma unroll
            for (int hb = 0; hb < 4; ++hb) {
                if (hb >= HB) break;
                const int h = h0 + hb;
#pragma unroll
                for (int qi = 0; qi < QT; ++qi) {
                    const int pos = pos0 + qi;
                    const bool vis = qi < nq && key <= pos && (a.window <= 0 || pos - key < a.window);
                    float v = vis ? s[hb][qi] : -INFINITY;
                    float mx = v;
#pragma unroll
                    for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
                    const float m_old = mrun[h * QT + qi];
                    const float m_new = fmaxf(m_old, mx);
                    const float p = vis ? expf(v - m_new) : 0.f;
                    float ps = p;
#pragma unroll
                    for (int o = 16; o > 0; o >>= 1) ps += __shfl_xor(ps, o, 64);
                    const float f = m_new == -INFINITY ? 1.f : expf(m_old - m_new);  // m_old = -inf: 0 (nothing summed yet)
                    pw[(h * QT + qi) * PAGE + j] = p;
                    if (j == 0) {
                        fac[h * QT + qi] = f;
                        lrun[h * QT + qi] = lrun[h * QT + qi] * f + ps;
                        mrun[h * QT + qi] = m_new;
                    }
                }
            }
        }
        __syncthreads();
        // ---- weights x values ----
#pragma unroll
        for (int o = 0; o < OPT; ++o) {
            const int oc = tid + o * THREADS;
            if (oc < H * dv) {
                const int h = oc / dv, c = oc - h * dv;
                const T* vrow = vp + ((page * G + h / R) * dv + c) * (int64_t)PAGE;
                float vv[PAGE];
#pragma unroll
                for (int u = 0; u < PAGE; u += VN) {
                    const VT v8 = *reinterpret_cast<const VT*>(vrow + u);
#pragma unroll
                    for (int w = 0; w < VN; ++w) vv[u + w] = (float)v8[w];
                }
#pragma unroll
                for (int qi = 0; qi < QT; ++qi) {
                    const float* pp = pw + (h * QT + qi) * PAGE;
                    float s = 0.f;
#pragma unroll
                    for (int u = 0; u < PAGE; u += 4) {
                        const f32x4 p4 = *reinterpret_cast<const f32x4*>(pp + u);
                        // masked keys have weight zero; what a page holds is always finite (utils/kv_cache.py)
                        s += p4[0] * vv[u] + p4[1] * vv[u + 1] + p4[2] * vv[u + 2] + p4[3] * vv[u + 3];
                    }
                    acc[o][qi] = acc[o][qi] * fac[h * QT + qi] + s;
                }
            }
        }
        __syncthreads();
    }
    T* out = reinterpret_cast<T*>(a.out);
    const T* gate = reinterpret_cast<const T*>(a.gate);
#pragma unroll
    for (int o = 0; o < OPT; ++o) {
        const int oc = tid + o * THREADS;
        if (oc < H * dv) {
            const int h = oc / dv;
#pragma unroll
            for (int qi = 0; qi < QT; ++qi)
                if (qi < nq) {
                    const int64_t t = t0 + first + qi;
                    float v = acc[o][qi] / lrun[h * QT + qi];
                    if (gate) v *= 1.f / (1.f + expf(-(float)gate[t * a.ld_gate + oc]));
                    out[t * a.ld_out + oc] = (T)v;
                }
        }
    }
}

// ---- decode steps: one query token per sequence -------------------------------------------------------------------------------
// A sequence's visible pages are dealt to `splits` workgroups (grid.x), so that a small batch still fills the chip; each leaves
// unnormalised sums and softmax statistics of its pages in `part` ([split][token][H][dv + 2] fp32: sums, m, l) and
// attn_mixed_combine_kernel merges them.  The R = H / G query heads that share a cached head are served together: a thread
// that holds a key row (or a value channel's 32 tokens) uses it for all R of them, so a page is read once per workgroup.
// MAXIT: (cached head, value channel) pairs a thread accumulates, R x MAXIT = 16.
template <typename T, int R, int MAXIT>
__global__ __launch_bounds__(THREADS) void attn_mixed_decode_kernel(MixArgs a, float* __restrict__ part, int splits, int64_t T_total) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int H = a.H, G = a.G, dk = a.dk, dv = a.dv;
    const int b = blockIdx.y, sp = blockIdx.x, tid = threadIdx.x;
    const int t = a.cu_q[b];
    if (a.cu_q[b + 1] - t <= 0) return;
    const int pos = a.ctx_lens[b] - 1;
    const int lo = a.window > 0 ? max(pos - a.window + 1, 0) : 0;
    const int p_lo = lo / PAGE, p_hi = pos / PAGE;
    const int per = (p_hi - p_lo + splits) / splits;
    const int pg0 = p_lo + sp * per, pg1 = min(pg0 + per - 1, p_hi);
    const int dkp = (dk + 3) & ~3;
    float* qs = smem;                 // [H][dkp]
    float* raw = qs + H * dkp;        // [H][PAGE]
    float* pw = raw + H * PAGE;       // [H][PAGE]
    float* fac = pw + H * PAGE;       // [H]
    float* mrun = fac + H;            // [H]
    float* lrun = mrun + H;           // [H]
    float* mixs = lrun + H;           // [H][H]
    for (int e = tid; e < H * H; e += THREADS) mixs[e] = a.mix[e];
    const T* q = reinterpret_cast<const T*>(a.q) + (int64_t)t * a.ldq;
    for (int e = tid; e < H * dkp; e += THREADS) {
        const int h = e / dkp, d = e - h * dkp;
        qs[e] = d < dk ? (float)q[(int64_t)h * dk + d] * a.scale : 0.f;
    }
    for (int e = tid; e < H; e += THREADS) {
        mrun[e] = -INFINITY;
        lrun[e] = 0.f;
    }
    float acc[MAXIT][R];
#pragma unroll
    for (int i = 0; i < MAXIT; ++i)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[i][r] = 0.f;
    const T* kp = reinterpret_cast<const T*>(a.k_pool);
    const T* vp = reinterpret_cast<const T*>(a.v_pool);
    constexpr int VN = Vec16<T>::N;
    typedef typename Vec16<T>::type VT;
    const bool k_vec = dk % VN == 0;
    const int items = G * dv;
    // heads per thread in the raw-score phase: R, or fewer (a power of two) while that gives more threads a key row
    int RT = R;
    while (RT > 1 && G * (R / RT) * PAGE * 2 <= THREADS) RT >>= 1;
    __syncthreads();
    for (int pg = pg0; pg <= pg1; ++pg) {
        const int64_t page = a.bt[(int64_t)b * a.bt_ld + pg];
        const int key0 = pg * PAGE;
        // raw scores of a cached head's R query heads against one key row; with few cached heads the R heads are dealt to
        // R / RT threads of RT heads each, so that the workgroup's threads all have a row
        for (int pr = tid; pr < G * (R / RT) * PAGE; pr += THREADS) {
            const int cs = pr / PAGE, j = pr % PAGE;
            const int c = cs / (R / RT), h0 = c * R + (cs % (R / RT)) * RT;
            const T* krow = kp + ((page * G + c) * PAGE + j) * (int64_t)dk;
            float s[R];
#pragma unroll
            for (int r = 0; r < R; ++r) s[r] = 0.f;
            if (key0 + j <= pos) {
                if (k_vec) {
                    // eight 16-byte pieces of the key row are asked for together (a piece at a time would cost a trip to memory each)
                    for (int d0 = 0; d0 < dk; d0 += 8 * VN) {
                        VT kv[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (d0 + e * VN < dk) kv[e] = *reinterpret_cast<const VT*>(krow + d0 + e * VN);
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (d0 + e * VN < dk) {
#pragma unroll
                                for (int r = 0; r < R; ++r)
                                    if (r < RT) {
                                        const float* qq = qs + (h0 + r) * dkp + d0 + e * VN;
#pragma unroll
                                        for (int u = 0; u < VN; u += 4) {
                                            const f32x4 q4 = *reinterpret_cast<const f32x4*>(qq + u);
                                            s[r] = fmaf((float)kv[e][u], q4[0], s[r]);
                                            s[r] = fmaf((float)kv[e][u + 1], q4[1], s[r]);
                                            s[r] = fmaf((float)kv[e][u + 2], q4[2], s[r]);
                                            s[r] = fmaf((float)kv[e][u + 3], q4[3], s[r]);
                                        }
                                    }
                            }
                    }
                } else {
                    for (int d = 0; d < dk; ++d) {
                        const float kf = (float)krow[d];
#pragma unroll
                        for (int r = 0; r < R; ++r)
                            if (r < RT) s[r] = fmaf(kf, qs[(h0 + r) * dkp + d], s[r]);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (r < RT) raw[(h0 + r) * PAGE + j] = s[r];
        }
        __syncthreads();
        for (int pr = tid; pr < H * PAGE; pr += THREADS) {
            const int h = pr / PAGE, j = pr % PAGE;
            float s = 0.f;
            for (int g = 0; g < H; ++g) s = fmaf(mixs[h * H + g], raw[g * PAGE + j], s);
            const int key = key0 + j;
            const bool vis = key <= pos && key >= lo;
            const float v = vis ? s : -INFINITY;
            float mx = v;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
            const float m_old = mrun[h];
            const float m_new = fmaxf(m_old, mx);
            const float p = vis ? expf(v - m_new) : 0.f;
            float ps = p;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) ps += __shfl_xor(ps, o, 64);
            pw[h * PAGE + j] = p;
            if (j == 0) {
                const float f = m_new == -INFINITY ? 1.f : expf(m_old - m_new);
                fac[h] = f;
                lrun[h] = lrun[h] * f + ps;
                mrun[h] = m_new;
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < MAXIT; ++i) {
            const int it = tid + i * THREADS;
            if (it < items) {
                const int c = it / dv, col = it - c * dv;
                const T* vrow = vp + ((page * G + c) * dv + col) * (int64_t)PAGE;
                float vv[PAGE];
#pragma unroll
                for (int u = 0; u < PAGE; u += VN) {
                    const VT v8 = *reinterpret_cast<const VT*>(vrow + u);
#pragma unroll
                    for (int w = 0; w < VN; ++w) vv[u + w] = (float)v8[w];
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float* pp = pw + (c * R + r) * PAGE;
                    float s = 0.f;
#pragma unroll
                    for (int u = 0; u < PAGE; u += 4) {
                        const f32x4 p4 = *reinterpret_cast<const f32x4*>(pp + u);
                        s += p4[0] * vv[u] + p4[1] * vv[u + 1] + p4[2] * vv[u + 2] + p4[3] * vv[u + 3];
                    }
                    acc[i][r] = acc[i][r] * fac[c * R + r] + s;
                }
            }
        }
        __syncthreads();
    }
    float* prow = part + ((int64_t)sp * T_total + t) * H * (dv + 2);
#pragma unroll
    for (int i = 0; i < MAXIT; ++i) {
        const int it = tid + i * THREADS;
        if (it < items) {
            const int c = it / dv, col = it - c * dv;
#pragma unroll
            for (int r = 0; r < R; ++r) prow[(int64_t)(c * R + r) * (dv + 2) + col] = acc[i][r];
        }
    }
    for (int h = tid; h < H; h += THREADS) {
        prow[(int64_t)h * (dv + 2) + dv] = mrun[h];
        prow[(int64_t)h * (dv + 2) + dv + 1] = lrun[h];
    }
}

// out[t][h dv + c] = sum_s acc_s e^(m_s - m) / sum_s l_s e^(m_s - m), m = max_s m_s, times the gate.  grid (token, ceil(H / 4)): a
// wave per head, its lanes over the splits for the statistics and over the value channels for the sums.
template <typename T>
__global__ __launch_bounds__(THREADS) void attn_mixed_combine_kernel(const float* __restrict__ part, int splits, int64_t T_total, MixArgs a) {
    const int64_t t = blockIdx.x;
    const int H = a.H, dv = a.dv;
    const int h = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (h >= H) return;
    const int64_t stride = T_total * H * (int64_t)(dv + 2);
    const float* p0 = part + (t * H + h) * (int64_t)(dv + 2);
    float m = -INFINITY;
    for (int s = lane; s < splits; s += 64) m = fmaxf(m, p0[s * stride + dv]);
    m = wave_max(m);
    float den = 0.f;
    for (int s = lane; s < splits; s += 64) {
        const float ms = p0[s * stride + dv];
        den += ms == -INFINITY ? 0.f : p0[s * stride + dv + 1] * expf(ms - m);
    }
    den = wave_sum(den);
    T* out = reinterpret_cast<T*>(a.out);
    const T* gate = reinterpret_cast<const T*>(a.gate);
    for (int c = lane; c < dv; c += 64) {
        float num = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float ms = p0[s * stride + dv];
            if (ms != -INFINITY) num = fmaf(p0[s * stride + c], expf(ms - m), num);
        }
        float v = num / den;
        const int oc = h * dv + c;
        if (gate) v *= 1.f / (1.f + expf(-(float)gate[t * a.ld_gate + oc]));
        out[t * a.ld_out + oc] = (T)v;
    }
}

template <typename T, int R>
void launch_decode(const MixArgs& a, int64_t B, int64_t T_total, int splits, float* part, hipStream_t st) {
    constexpr int MAXIT = 16 / R;
    const int dkp = (a.dk + 3) & ~3;
    const size_t lds = ((size_t)a.H * dkp + (size_t)2 * a.H * PAGE + (size_t)3 * a.H + (size_t)a.H * a.H) * sizeof(float);
    if (lds > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)attn_mixed_decode_kernel<T, R, MAXIT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((attn_mixed_decode_kernel<T, R, MAXIT>), dim3((unsigned)splits, (unsigned)B), dim3(THREADS), lds, st, a, part, splits, T_total);
    hipLaunchKernelGGL(attn_mixed_combine_kernel<T>, dim3((unsigned)T_total, (unsigned)((a.H + 3) / 4)), dim3(THREADS), 0, st, part, splits, T_total, a);
}

template <typename T>
bool try_decode(const MixArgs& a, int64_t B, int64_t T_total, int64_t max_ctx, void* ws, int64_t ws_bytes, hipStream_t st) {
    const int R = a.H / a.G;
    if (!ws || (R != 1 && R != 2 && R != 4 && R != 8 && R != 16)) return false;
    const int64_t keys = a.window > 0 ? std::min<int64_t>(max_ctx, (int64_t)a.window + PAGE) : max_ctx;
    const int pages = (int)cdiv64(std::max<int64_t>(keys, 1), PAGE) + (a.window > 0 ? 1 : 0);
    static const int64_t target_wgs = getenv("TGIS_MIXED_DECODE_WGS") ? atoll(getenv("TGIS_MIXED_DECODE_WGS")) : 512;
    int splits = (int)std::max<int64_t>(1, std::min<int64_t>(pages, target_wgs / std::max<int64_t>(B, 1)));
    const int64_t per_split = T_total * a.H * (a.dv + 2) * (int64_t)sizeof(float);
    splits = (int)std::min<int64_t>(splits, ws_bytes / std::max<int64_t>(per_split, 1));
    if (splits < 1) return false;
    float* part = reinterpret_cast<float*>(ws);
    if (R == 1) launch_decode<T, 1>(a, B, T_total, splits, part, st);
    else if (R == 2) launch_decode<T, 2>(a, B, T_total, splits, part, st);
    else if (R == 4) launch_decode<T, 4>(a, B, T_total, splits, part, st);
    else if (R == 8) launch_decode<T, 8>(a, B, T_total, splits, part, st);
    else launch_decode<T, 16>(a, B, T_total, splits, part, st);
    return true;
}

// ---- prompt portions on the matrix cores (two-byte dtypes, dk % 16 == 0, dv % 16 == 0) ------------------------------------------
// Workgroup = 16 consecutive query tokens of a sequence x all heads, NW waves; wave w owns heads w, w + NW, ...  Per page of 32
// keys: raw scores S_g = Q_g K^T by 16x16x32 products (A = the query rows, B = the page's key rows, both 16-byte fragment loads
// from memory; a lane of the accumulator holds key l % 16 of queries 4 (l / 16) .. + 3) into LDS in fp32; after a barrier every
// wave mixes the H raw tiles into its own heads' tiles (a raw value read from LDS serves all of the wave's heads), masks, and
// keeps the online softmax of its (head, query) rows in registers — a row's 32 keys live in 16 neighbouring lanes; the
// weights go to LDS rounded to T as the A operand of O += P V, whose B operand is the channel-major value page (16 bytes = 8
// tokens of a channel).  Scores, the mix, weights and statistics are fp32; only P is rounded for the last product.
constexpr int RAW_ROW = 20;   // floats per KEY row of a raw tile (16 queries + 4: a lane's four queries are one 16-byte access)
constexpr int P_ROW = 40;     // T elements per query row of a weight tile (80 bytes: 16-byte aligned, staggered)

// the value of the lane N places further on in its row of 16 lanes (a data-parallel-primitive move: no trip through LDS); four of
// them with N = 8, 4, 2, 1 leave a row's sum or maximum in all of its lanes
// e^x by the hardware's base-two exponential (fp32, a few units in the last place): this form serves two-byte models, whose
// weights are rounded to two bytes for the last product anyway
__device__ __forceinline__ float exp_hw(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
template <int N> __device__ __forceinline__ float row_ror(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xF, 0xF, true));
}

template <typename T, int HW, int DVT>
__global__ __launch_bounds__(512) void attn_mixed_mfma_kernel(MixArgs a) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    typedef typename Vec16<T>::type V8;
    const int H = a.H, G = a.G, dk = a.dk, dv = a.dv, R = H / G;
    const int NW = blockDim.x >> 6, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int lr = lane & 15, lg = lane >> 4;  // fragment row / column, and the group of 8 k-slots (or of 4 accumulator rows)
    const int b = blockIdx.y;
    const int t0 = a.cu_q[b], qlen = a.cu_q[b + 1] - t0;
    const int first = blockIdx.x * 16;
    if (first >= qlen) return;
    const int nq = min(16, qlen - first);
    const int pos0 = a.ctx_lens[b] - qlen + first;
    float* raw = smem;                                          // [H][32 keys][RAW_ROW]
    float* mixs = raw + H * 32 * RAW_ROW;                       // [H][H]
    T* pb = reinterpret_cast<T*>(mixs + H * H);                 // [H][16][P_ROW]
    for (int e = threadIdx.x; e < H * H; e += blockDim.x) mixs[e] = a.mix[e];
    const int nvt = dv / 16;
    f32x4 O[HW][DVT];
    float mrun[HW][4], lrun[HW][4];
#pragma unroll
    for (int i = 0; i < HW; ++i) {
#pragma unroll
        for (int t = 0; t < DVT; ++t) O[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            mrun[i][u] = -INFINITY;
            lrun[i][u] = 0.f;
        }
    }
    const T* q = reinterpret_cast<const T*>(a.q) + (int64_t)(t0 + first + min(lr, nq - 1)) * a.ldq;  // rows past the tile repeat its last one
    const T* kp = reinterpret_cast<const T*>(a.k_pool);
    const T* vp = reinterpret_cast<const T*>(a.v_pool);
    const int lo_first = a.window > 0 ? max(pos0 - a.window + 1, 0) : 0;
    const int last_pos = pos0 + nq - 1;
    __syncthreads();
    for (int pg = lo_first / PAGE; pg <= last_pos / PAGE; ++pg) {
        const int64_t page = a.bt[(int64_t)b * a.bt_ld + pg];
        const int key0 = pg * PAGE;
        // ---- raw scores of this wave's heads: per 32 key channels the fragments of all its heads are asked for together ----
        f32x4 s0[HW], s1[HW];
#pragma unroll
        for (int i = 0; i < HW; ++i) s0[i] = s1[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int d0 = 0; d0 < dk; d0 += 32) {
            const int d = d0 + lg * 8;
            V8 qa[HW], k0[HW], k1[HW];
#pragma unroll
            for (int i = 0; i < HW; ++i) {
                const int h = min(wave + NW * i, H - 1);
                const T* krow = kp + ((page * G + h / R) * PAGE + lr) * (int64_t)dk;
                qa[i] = k0[i] = k1[i] = V8{};
                if (d < dk) {
                    qa[i] = *reinterpret_cast<const V8*>(q + (int64_t)h * dk + d);
                    k0[i] = *reinterpret_cast<const V8*>(krow + d);
                    k1[i] = *reinterpret_cast<const V8*>(krow + (int64_t)16 * dk + d);
                }
            }
#pragma unroll
            for (int i = 0; i < HW; ++i) {
                s0[i] = mfma16(qa[i], k0[i], s0[i]);
                s1[i] = mfma16(qa[i], k1[i], s1[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < HW; ++i) {
            const int h = wave + NW * i;
            if (h < H) {
                float* rt = raw + (h * 32 + lr) * RAW_ROW + lg * 4;  // key lr (and lr + 16), queries 4 lg .. + 3
                *reinterpret_cast<f32x4*>(rt) = s0[i] * a.scale;
                *reinterpret_cast<f32x4*>(rt + 16 * RAW_ROW) = s1[i] * a.scale;
            }
        }
        __syncthreads();
        // ---- mix, mask, online softmax of this wave's (head, query) rows ----
        float sm[HW][8];
#pragma unroll
        for (int i = 0; i < HW; ++i)
#pragma unroll
            for (int u = 0; u < 8; ++u) sm[i][u] = 0.f;
        for (int g = 0; g < H; ++g) {
            const float* rt = raw + (g * 32 + lr) * RAW_ROW + lg * 4;
            const f32x4 ra = *reinterpret_cast<const f32x4*>(rt), rb = *reinterpret_cast<const f32x4*>(rt + 16 * RAW_ROW);
            const float r[8] = {ra[0], ra[1], ra[2], ra[3], rb[0], rb[1], rb[2], rb[3]};
#pragma unroll
            for (int i = 0; i < HW; ++i) {
                const int h = min(wave + NW * i, H - 1);
                const float m = mixs[h * H + g];
#pragma unroll
                for (int u = 0; u < 8; ++u) sm[i][u] = fmaf(m, r[u], sm[i][u]);
            }
        }
#pragma unroll
        for (int i = 0; i < HW; ++i) {
            const int h = wave + NW * i;
            if (h < H) {
                T* pt = pb + (h * 16 + lg * 4) * P_ROW + lr;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int qi = lg * 4 + u, pos = pos0 + qi;
                    const int ka = key0 + lr, kb2 = ka + 16;
                    const bool va = qi < nq && ka <= pos && (a.window <= 0 || pos - ka < a.window);
                    const bool vb = qi < nq && kb2 <= pos && (a.window <= 0 || pos - kb2 < a.window);
                    const float xa = va ? sm[i][u] : -INFINITY, xb = vb ? sm[i][4 + u] : -INFINITY;
                    float mx = fmaxf(xa, xb);
                    mx = fmaxf(mx, row_ror<8>(mx));
                    mx = fmaxf(mx, row_ror<4>(mx));
                    mx = fmaxf(mx, row_ror<2>(mx));
                    mx = fmaxf(mx, row_ror<1>(mx));
                    const float m_new = fmaxf(mrun[i][u], mx);
                    const float pa = va ? exp_hw(xa - m_new) : 0.f, pb2 = vb ? exp_hw(xb - m_new) : 0.f;
                    float ps = pa + pb2;
                    ps += row_ror<8>(ps);
                    ps += row_ror<4>(ps);
                    ps += row_ror<2>(ps);
                    ps += row_ror<1>(ps);
                    const float f = m_new == -INFINITY ? 1.f : exp_hw(mrun[i][u] - m_new);
                    lrun[i][u] = lrun[i][u] * f + ps;
                    mrun[i][u] = m_new;
                    if (f != 1.f) {
#pragma unroll
                        for (int t = 0; t < DVT; ++t) O[i][t][u] *= f;
                    }
                    pt[u * P_ROW] = (T)pa;
                    pt[u * P_ROW + 16] = (T)pb2;
                }
            }
        }
        __syncthreads();
        // ---- weights x values ----
#pragma unroll
        for (int i = 0; i < HW; ++i) {
            const int h = wave + NW * i;
            if (h < H) {
                const V8 pa = *reinterpret_cast<const V8*>(pb + (h * 16 + lr) * P_ROW + lg * 8);
                const T* vrow = vp + ((page * G + h / R) * dv + lr) * (int64_t)PAGE + lg * 8;
#pragma unroll
                for (int t = 0; t < DVT; ++t)
                    if (t < nvt) O[i][t] = mfma16(pa, *reinterpret_cast<const V8*>(vrow + (int64_t)t * 16 * PAGE), O[i][t]);
            }
        }
    }
    T* out = reinterpret_cast<T*>(a.out);
    const T* gate = reinterpret_cast<const T*>(a.gate);
#pragma unroll
    for (int i = 0; i < HW; ++i) {
        const int h = wave + NW * i;
        if (h < H) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int qi = lg * 4 + u;
                if (qi < nq) {
                    const int64_t t = t0 + first + qi;
                    const float inv = 1.f / lrun[i][u];
#pragma unroll
                    for (int tl = 0; tl < DVT; ++tl)
                        if (tl < nvt) {
                            const int oc = h * dv + tl * 16 + lr;
                            float v = O[i][tl][u] * inv;
                            if (gate) v *= 1.f / (1.f + expf(-(float)gate[t * a.ld_gate + oc]));
                            out[t * a.ld_out + oc] = (T)v;
                        }
                }
            }
        }
    }
}

template <typename T, int HW, int DVT>
void launch_mfma_as(const MixArgs& a, int64_t B, int64_t max_q_len, int nw, hipStream_t st) {
    const size_t lds = ((size_t)a.H * 32 * RAW_ROW + (size_t)a.H * a.H) * sizeof(float) + (size_t)a.H * 16 * P_ROW * sizeof(T);
    if (lds > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)attn_mixed_mfma_kernel<T, HW, DVT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((attn_mixed_mfma_kernel<T, HW, DVT>), dim3((unsigned)cdiv64(max_q_len, 16), (unsigned)B), dim3(64 * nw), lds, st, a);
}

template <typename T, int HW>
bool launch_mfma_hw(const MixArgs& a, int64_t B, int64_t max_q_len, int nw, hipStream_t st) {
    const int nvt = a.dv / 16;
    if (nvt <= 2) launch_mfma_as<T, HW, 2>(a, B, max_q_len, nw, st);
    else if (nvt <= 4) launch_mfma_as<T, HW, 4>(a, B, max_q_len, nw, st);
    else if (nvt <= 8) launch_mfma_as<T, HW, 8>(a, B, max_q_len, nw, st);
    else if (nvt <= 16 && HW <= 2) launch_mfma_as<T, HW, (HW <= 2 ? 16 : 2)>(a, B, max_q_len, nw, st);
    else return false;
    return true;
}

// up to 8 heads: four waves of up to two heads; up to 32: eight waves of up to four (a wave's accumulators stay within 32
// tiles of 16 x 16); false if the geometry is not served
template <typename T>
bool try_mfma(const MixArgs& a, int64_t B, int64_t max_q_len, hipStream_t st) {
    if (a.dk % 16 || a.dv % 16 || a.dv > 256 || a.ldq % 8 || a.H > 32) return false;
    if ((((uintptr_t)a.q) & 15) || (((uintptr_t)a.k_pool) & 15) || (((uintptr_t)a.v_pool) & 15)) return false;
    const size_t lds = ((size_t)a.H * 32 * RAW_ROW + (size_t)a.H * a.H) * sizeof(float) + (size_t)a.H * 16 * P_ROW * sizeof(T);
    if (lds > 150 * 1024) return false;
    const int nw = a.H > 8 ? 8 : 4;
    const int hw = (a.H + nw - 1) / nw;
    if (hw <= 1) return launch_mfma_hw<T, 1>(a, B, max_q_len, nw, st);
    if (hw <= 2) return launch_mfma_hw<T, 2>(a, B, max_q_len, nw, st);
    return launch_mfma_hw<T, 4>(a, B, max_q_len, nw, st);
}

size_t lds_bytes(int QT, int H, int dk) {
    const int dkp = (dk + 3) & ~3;
    return ((size_t)QT * H * dkp + (size_t)2 * H * QT * PAGE + (size_t)4 * H * QT + (size_t)H * H) * sizeof(float);
}

template <typename T, int QT, int OPT>
void launch_as(const MixArgs& a, int64_t B, int64_t max_q_len, hipStream_t st) {
    const size_t lds = lds_bytes(QT, a.H, a.dk);
    if (lds > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)attn_mixed_heads_kernel<T, QT, OPT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((attn_mixed_heads_kernel<T, QT, OPT>), dim3((unsigned)cdiv64(max_q_len, QT), (unsigned)B), dim3(THREADS), lds, st, a);
}

template <typename T, int QT>
void launch_qt(const MixArgs& a, int64_t B, int64_t max_q_len, hipStream_t st) {
    const int per = (a.H * a.dv + THREADS - 1) / THREADS;
    if (per <= 2) launch_as<T, QT, 2>(a, B, max_q_len, st);
    else if (per <= 4) launch_as<T, QT, 4>(a, B, max_q_len, st);
    else if (per <= 8) launch_as<T, QT, 8>(a, B, max_q_len, st);
    else launch_as<T, QT, 16>(a, B, max_q_len, st);
}

template <typename T>
void launch(const MixArgs& a, int64_t B, int64_t max_q_len, hipStream_t st) {
    // the widest tile of queries that the step has use for, that 96 KiB of LDS hold and that keeps the accumulators in registers
    const int per = (a.H * a.dv + THREADS - 1) / THREADS;
    int qt = 8;
    while (qt > 1 && (qt >= 2 * max_q_len || lds_bytes(qt, a.H, a.dk) > 96 * 1024 || per * qt > 64)) qt >>= 1;
    if (qt == 8) launch_qt<T, 8>(a, B, max_q_len, st);
    else if (qt == 4) launch_qt<T, 4>(a, B, max_q_len, st);
    else if (qt == 2) launch_qt<T, 2>(a, B, max_q_len, st);
    else launch_qt<T, 1>(a, B, max_q_len, st);
}

}  // namespace

extern "C" int tgis_attn_mixed_heads(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                                     int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B,
                                     const float* mix, const void* gate, int64_t ld_gate, void* out, int64_t ld_out,
                                     int64_t total_q, int64_t max_q_len, int64_t max_ctx, int H, int G, int dk, int dv, float scale,
                                     int window, void* workspace, int64_t workspace_bytes, int impl, int dtype, void* stream) {
    TGIS_CHECK_ARG(q && k_pool && v_pool && block_tables && ctx_lens && cu_seqlens_q && mix && out, "tgis_attn_mixed_heads: null tensor");
    TGIS_CHECK_ARG(H >= 1 && G >= 1 && H % G == 0 && dk >= 1 && dv >= 1 && ldq >= (int64_t)H * dk && ld_out >= (int64_t)H * dv &&
                       (!gate || ld_gate >= (int64_t)H * dv) && window >= 0 && max_q_len >= 1 && max_ctx >= 1 && total_q >= 0,
                   "tgis_attn_mixed_heads: bad geometry (H %d, G %d, dk %d, dv %d)", H, G, dk, dv);
    TGIS_CHECK_ARG((int64_t)H * dv <= 16 * THREADS, "tgis_attn_mixed_heads: heads x value width up to %d (got %d x %d)", 16 * THREADS, H, dv);
    TGIS_CHECK_ARG(lds_bytes(1, H, dk) <= 150 * 1024, "tgis_attn_mixed_heads: heads x key width too large for one workgroup (%d x %d)", H, dk);
    TGIS_CHECK_ARG(dtype == TGIS_F16 || dtype == TGIS_BF16 || dtype == TGIS_F32, "tgis_attn_mixed_heads: bad dtype");
    if (B == 0) return TGIS_OK;
    hipStream_t st = (hipStream_t)stream;
    TgisTimedScope timed(TGIS_OP_ATTN, st);
    const MixArgs a{q, ldq, k_pool, v_pool, block_tables, max_pages, ctx_lens, cu_seqlens_q, mix, gate, ld_gate, out, ld_out, H, G, dk, dv,
                    window, scale};
    // steps of single tokens (total_q <= B says so whatever max_q_len's bound is): the key-split form when the geometry allows
    bool done = false;
    if (max_q_len == 1 && total_q <= B) {
        if (dtype == TGIS_F16) done = try_decode<f16>(a, B, total_q, max_ctx, workspace, workspace_bytes, st);
        else if (dtype == TGIS_BF16) done = try_decode<bf16>(a, B, total_q, max_ctx, workspace, workspace_bytes, st);
        else done = try_decode<float>(a, B, total_q, max_ctx, workspace, workspace_bytes, st);
    }
    // prompt portions of two-byte models: the matrix-core form (impl 1 keeps the general kernel for comparisons)
    if (!done && max_q_len > 2 && impl != 1) {
        if (dtype == TGIS_F16) done = try_mfma<f16>(a, B, max_q_len, st);
        else if (dtype == TGIS_BF16) done = try_mfma<bf16>(a, B, max_q_len, st);
    }
    if (!done) {
        if (dtype == TGIS_F16) launch<f16>(a, B, max_q_len, st);
        else if (dtype == TGIS_BF16) launch<bf16>(a, B, max_q_len, st);
        else launch<float>(a, B, max_q_len, st);
    }
    TGIS_CHECK_LAUNCH();
    return TGIS_OK;
}
