/*
 * tgis_hip.h — C ABI of libtgis_hip.so, the MI355X (gfx950) native-kernel library that sits
 * where the reference's CUDA extension modules sit on the batched-decode hot path.
 *
 * Boundary: SURVEY.md §8(b) row #5.  The reference calls pybind/torch-extension functions with
 * at::Tensor arguments (flash_attn_2_cuda, dropout_layer_norm, rotary_emb, exllamav2_kernels);
 * this library exposes the same operations behind a plain C ABI: raw device pointers, int64
 * sizes/strides, float scalars and a hipStream_t passed as void*.  No torch types, no allocation
 * inside any call (callers pass workspaces; *_workspace_bytes queries say how large), no implicit
 * synchronisation.  Every function returns 0 on success or a negative TGIS_E* code;
 * tgis_last_error() returns a thread-local message for the last failure.
 *
 * dtype codes: TGIS_F16 (IEEE half) and TGIS_BF16.  All "T*" pointers below are 2-byte elements
 * of that dtype.  All pointers are device pointers unless the comment says host.
 *
 * Reference citations are relative to /root/reference/server/text_generation_server/.
 */
#ifndef TGIS_HIP_H
#define TGIS_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TGIS_OK 0
#define TGIS_EINVAL (-1)   /* bad argument (shape, alignment, dtype) */
#define TGIS_EHIP (-2)     /* a HIP runtime call failed */
#define TGIS_EUNSUPPORTED (-3)
#define TGIS_ENOMEM (-4)

#define TGIS_F16 0
#define TGIS_BF16 1
#define TGIS_F32 2 /* only where an entry point says so (the fp32-residual / ragged-step family at the end) */

/* KV page geometry: 32 tokens per page; per (page, k|v, kv_head) one
 * 32*head_dim element block in an MFMA-fragment-ready order. */
#define TGIS_KV_PAGE_TOKENS 32

/* ---- library info ------------------------------------------------------------------------- */
const char* tgis_version(void);          /* "tgis_hip x.y (gfx950)" */
const char* tgis_arch(void);             /* offload arch the kernels were compiled for */
const char* tgis_last_error(void);       /* thread-local, never NULL */
/* Forget the last failure, including the HIP runtime's sticky per-thread error: every launch in this library ends with
 * hipGetLastError(), so an error left behind by someone else's aborted stream capture would otherwise be reported by
 * the next, unrelated call. */
void tgis_clear_error(void);
int tgis_device_info(int device, int* num_cus, int64_t* hbm_bytes, char* name, int name_len);

/* Optional per-op device timing with HIP events recorded on the op's own stream.
 * tgis_timing_enable(1) makes every timed op (see TGIS_OP_*) bracket its kernel launch(es) with an
 * event pair; tgis_timing_read() synchronises those events and returns count and total
 * milliseconds since the last tgis_timing_reset().  Disabled by default (no events, no cost). */
#define TGIS_OP_GPTQ_GEMM 0
#define TGIS_OP_ATTN 1
#define TGIS_OP_DENSE_GEMM 2
#define TGIS_OP_NORM 3
#define TGIS_OP_ROPE_KV 4
#define TGIS_OP_ACT 5
#define TGIS_OP_SAMPLE 6
#define TGIS_OP_DECODE_TAIL 7
#define TGIS_OP_SCAN 8      /* recurrent scans (tgis_wkv_scan, tgis_delta_scan) */
#define TGIS_OP_MOE_GEMM 9  /* grouped expert GEMMs (tgis_moe_gemm) */
#define TGIS_OP_COUNT 10
int tgis_timing_enable(int on);
int tgis_timing_reset(void);
int tgis_timing_read(int op, int64_t* count, double* total_ms);

/* ---- GPTQ int4 linear (replaces exllamav2_kernels.make_q_matrix / gemm_half_q_half,
 *      utils/gptq/exllamav2.py:14-62,100-144; normative arithmetic utils/gptq/quant_linear.py:130-192) */

/* Bytes of the prepared (repacked) weight image for a [K,N] 4-bit matrix with `groups` groups. */
int64_t tgis_gptq_prepared_bytes(int64_t K, int64_t N, int64_t groups);

/* Repack GPTQ tensors into the kernel layout.  One-time, at load
 * (the reference does this in Ex4bitLinearV2.post_init, exllamav2.py:124-137).
 *   qweight [K/8, N] int32, qzeros [groups, N/8] int32, scales [groups, N] f16,
 *   g_idx [K] int32 or NULL (NULL = trivial k / groupsize), perm_out [K] int32 or NULL:
 *   when g_idx is not the trivial map (act-order) perm_out receives the row permutation that the
 *   activation must be gathered with (x'[:,k'] = x[:,perm[k']]); groupsize = K / groups.
 *   prepared: caller-owned buffer of tgis_gptq_prepared_bytes().  Requires K%32==0, N%32==0
 *   (same asserts as exllamav2.py:118-119) and (K/groups)%8==0.
 *   flags bit 0 (TGIS_GPTQ_GATE_UP): the matrix is a fused [gate | up] projection (N = 2 I); columns are
 *   interleaved in the image so that tgis_gptq_gemm_f16(act=2) can apply SiLU(gate)*up in its epilogue. */
#define TGIS_GPTQ_GATE_UP 1
int tgis_gptq_prepare(const int32_t* qweight, const int32_t* qzeros, const void* scales,
                      const int32_t* g_idx_host, int32_t* perm_out, int64_t K, int64_t N,
                      int64_t groups, int flags, void* prepared, void* stream);

/* Workspace for split-K partial sums + arrival counters of one gemm call. The counter region
 * (first 4096 bytes) must be zero before the first call; the kernel leaves it zero. */
/* Largest M for which tgis_gptq_gemm_f16 is a fused dequantise + MFMA kernel worth calling (above it the caller
 * dequantises once with tgis_gptq_dequant_f16 and uses a library GEMM, exllamav2.py:87 "M > 50"): M <= 64 streams the
 * weights once per pass, 64 < M <= 256 in 64-row passes, and — for K % 64 == 0, group size 64 * 2^n, no act-order, act != 1 —
 * a tall kernel (one dequantisation per 128 rows, 700-900 TFLOP/s, no scratch copy of W) takes over up to a few thousand
 * rows. */
int64_t tgis_gptq_gemm_fused_rows(int64_t K, int64_t groups, int act_order, int act);
int64_t tgis_gptq_gemm_workspace_bytes(int64_t M, int64_t K, int64_t N);

/* Activation layout between the decode step's own kernels (round 4).  A leading dimension of TGIS_LD_FRAGMENTS says that a
 * [M <= 64, K] f16 activation (K % 64 == 0; the buffer holds ceil(M / 32) * 32 * K elements) is stored in the order the MFMA
 * reads it — [row block m/32][k64-step][i = k/8 % 4][lane = 32 (k/32 % 2) + m % 32][k % 8], i.e. element (m, k) at
 * (m/32) * 32 K + ((k/64 * 4 + k/8 % 4) * 64 + 32 (k/32 % 2) + m % 32) * 8 + k % 8 — instead of row-major.  Producers that can write it:
 * tgis_rmsnorm_residual[_partial] (ldy), tgis_attn_paged (ld_out), tgis_gptq_gemm_f16 with act = 2 (ldo).  Consumers:
 * tgis_gptq_gemm_f16, tgis_gptq_gemm_f16_partial, tgis_gptq_gemm_rope_f16 (ldx), which then run the kernel of
 * csrc/gptq_wide_body.h: each k64-step of the activation is four contiguous KiB straight into the A operand, no LDS staging
 * (7B shapes, 32 rows: qkv + rope 16.9 -> 12 us, o 6.0 -> 5.3, gate_up 16.8 -> 14.4, down 10.5 -> 9.2).  Same arithmetic as
 * the row-major path ((q - z) * s rounded to f16 once, fp32 accumulation); only the summation order over k differs.
 * tgis_gptq_fragments_ok: 1 if the GEMM (act 0, 2, or 3 = the rope epilogue) takes such an activation and is expected to be
 * faster with it (1 <= M <= 64, no act-order, groups of 64 * 2^n rows; act 2 / 3 additionally >= 128 workgroups). */
#define TGIS_LD_FRAGMENTS ((int64_t)-32)
int tgis_gptq_fragments_ok(int64_t M, int64_t K, int64_t N, int64_t groups, int act_order, int act);

/* out[M,N] f16 = x[M,K] f16 @ dequant(W)[K,N] (+ bias[N] f16 if non-NULL); fp32 accumulate.
 * Fused int4-dequant MFMA kernel for any M (rows are processed in slabs of 32).
 * x row stride ldx, out row stride ldo (elements).  perm (int32 [K] or NULL) gathers x columns
 * for act-order matrices.  act: 0 = none; 1 = x is [M,2K] and the kernel consumes silu(x[:, :K]) * x[:, K:]
 * while staging it; 2 = the image was prepared with TGIS_GPTQ_GATE_UP and out is [M, N/2] =
 * silu(gate) * up applied in the epilogue (both fuse LlamaMLP's activation, flash_llama_modeling.py:332-335). */
int tgis_gptq_gemm_f16(const void* x, int64_t ldx, const void* prepared, const void* bias,
                       const int32_t* perm, void* out, int64_t ldo, int64_t M, int64_t K, int64_t N,
                       int64_t groups, int act, void* workspace, int64_t workspace_bytes, void* stream);

/* Deferred-reduce variant: instead of the f16 result, the S split-K partial sums are left in
 * `slabs` as fp32 [ceil(M/32)][S][32][ld] (ld = N rounded up to 32, returned in *slab_ld; S in *num_slabs, >= 1) for a
 * consumer that sums them in its prologue (tgis_rmsnorm_residual_partial / tgis_rope_kv_write_partial), which
 * removes the reduce launch.  The consumer rounds the sum (+bias) to f16 first, so results are bit-identical to
 * tgis_gptq_gemm_f16 followed by the plain consumer.  slabs must hold tgis_gptq_gemm_partial_bytes(M,K,N) bytes. */
int64_t tgis_gptq_gemm_partial_bytes(int64_t M, int64_t K, int64_t N);
int tgis_gptq_gemm_f16_partial(const void* x, int64_t ldx, const void* prepared, const int32_t* perm, int64_t M,
                               int64_t K, int64_t N, int64_t groups, int act, float* slabs, int64_t slabs_bytes,
                               int* num_slabs, int64_t* slab_ld, void* stream);

/* ---- fused qkv projection + rotary embedding + cache write (decode, round 3) ------------------------------------------
 * One launch for `qkv = query_key_value(x)`, `rotary_emb(q, k, cos, sin)` and `layer_past[slot] = (k, v)`
 * (flash_llama_modeling.py:251-268,282) at decode sizes: the GEMM keeps the whole k range in a block (no split-K slabs)
 * and its epilogue rounds the sum (+ bias) to f16, rotates q / k heads in fp32 (the arithmetic of tgis_rope_kv_write) and
 * stores q to q_out[M, ldq] and k / v into the cache pages of slots[m] (page layouts of tgis_rope_kv_write).
 * `prepared` is a SECOND image of the qkv weight made with flags = TGIS_GPTQ_ROPE_IMAGE(D, H + Hkv): inside each rotated
 * head a 32-column tile holds 16 dims and their 16 rotation partners, so every wave owns complete rotation pairs.
 * Full rotary span only (rot_dim == D).  tgis_gptq_rope_ok: whether the launch exists for the shape (1 <= M <= 64, groups
 * of 64 * 2^n rows, no act-order, D % 32 == 0) AND is expected to beat the two launches it replaces (its unsplit plan
 * still covers the chip: >= 128 workgroups); the entry point itself only checks the former. */
#define TGIS_GPTQ_ROPE_IMAGE(D, rotated_heads) (2 | ((int)(D) << 8) | ((int)(rotated_heads) << 20))
int tgis_gptq_rope_ok(int64_t M, int64_t K, int64_t N, int64_t groups, int act_order, int64_t D);
int tgis_gptq_gemm_rope_f16(const void* x, int64_t ldx, const void* prepared, const void* bias, const int32_t* positions,
                            const int32_t* slots, const void* cos, const void* sin, void* q_out, int64_t ldq,
                            void* k_pool, void* v_pool, int64_t M, int64_t K, int64_t N, int64_t groups, int64_t H,
                            int64_t Hkv, int64_t D, void* stream);

/* The same launch for dense (f16 / bf16) qkv weights: `prepared` from tgis_dense_prepare with
 * flags = TGIS_GPTQ_ROPE_IMAGE(D, H + Hkv); cos / sin in the model dtype; 1 <= M <= 64. */
int tgis_dense_rope_ok(int64_t M, int64_t K, int64_t N, int64_t D);
int tgis_dense_gemm_rope(const void* x, int64_t ldx, const void* prepared, const void* bias, const int32_t* positions,
                         const int32_t* slots, const void* cos, const void* sin, void* q_out, int64_t ldq, void* k_pool,
                         void* v_pool, int64_t M, int64_t K, int64_t N, int64_t H, int64_t Hkv, int64_t D, int dtype,
                         void* stream);

/* Full dequantisation to a dense f16 [K,N] matrix (row-major), the "temp_dq" path the reference
 * uses for M > 50 before a library GEMM (exllamav2.py:65-66,87). */
int tgis_gptq_dequant_f16(const void* prepared, void* w_out, int64_t K, int64_t N, int64_t groups,
                          int flags, void* stream);

/* ---- dense skinny GEMM (replaces F.linear / torch.mm at decode sizes, utils/layers.py:110-111,
 *      lm_head utils/layers.py:261) -------------------------------------------------------------- */
int64_t tgis_dense_prepared_bytes(int64_t N, int64_t K);
/* Repack a torch-Linear weight W[N,K] (row-major, dtype) into 32-column MFMA tiles.
 * flags bit 0: W is the Llama MLP's [gate rows | up rows] (N = 2 I, I a multiple of 16): tile t then holds gate rows
 * 16 t .. 16 t + 15 and the matching up rows, for the act = 2 epilogue of tgis_dense_gemm. */
int tgis_dense_prepare(const void* w, int64_t N, int64_t K, int dtype, int flags, void* prepared, void* stream);
int64_t tgis_dense_gemm_workspace_bytes(int64_t M, int64_t K, int64_t N);
/* out[M,N] = x[M,K] @ W^T (+bias).  out_f32 != 0 writes float32 output (logits).
 * act 0: plain.  act 1: x is [M, 2K] (gate | up) and the operand is silu(gate) * up, formed while it is staged
 * (down_proj after an un-fused gate_up).  act 2: the image has flags bit 0 and out is [M, N/2] =
 * silu(x @ Wgate^T) * (x @ Wup^T), each factor rounded to the model dtype as the reference's eager ops do
 * (flash_llama_modeling.py:332-335); the down projection then runs with act 0.
 * act 4 / 5: out = gelu(T(x @ W^T + bias)) in the model dtype, exact erf form / tanh approximation — the `self.act(...)`
 * behind `c_fc` (flash_santacoder_modeling.py:284-306) applied to the rounded output where it is finished (the epilogue of an
 * unsplit plan, the split-K reduce otherwise): bit-identical to tgis_dense_gemm(act 0) followed by tgis_gelu. */
int tgis_dense_gemm(const void* x, int64_t ldx, const void* prepared, const void* bias, void* out,
                    int64_t ldo, int64_t M, int64_t K, int64_t N, int dtype, int out_f32, int act,
                    void* workspace, int64_t workspace_bytes, void* stream);
/* Deferred split-K, as tgis_gptq_gemm_f16_partial: the fp32 partial sums [ceil(M/32)][num_slabs][32][slab_ld] are
 * left for the consumer kernel (tgis_rmsnorm_residual_partial / tgis_rope_kv_write_partial), which adds the bias. */
int64_t tgis_dense_gemm_partial_bytes(int64_t M, int64_t K, int64_t N);
int tgis_dense_gemm_partial(const void* x, int64_t ldx, const void* prepared, int64_t M, int64_t K, int64_t N,
                            int dtype, int act, float* slabs, int64_t slabs_bytes, int* num_slabs,
                            int64_t* slab_ld, void* stream);

/* ---- fused residual-add + RMSNorm / LayerNorm (replaces dropout_layer_norm.dropout_add_ln_fwd,
 *      custom_modeling/flash_llama_modeling.py:132-152, utils/layers.py:376-396) ---------------- */
/* res_out = x (+ residual); y = res_out * rsqrt(mean(res_out^2) + eps) * weight.
 * residual may be NULL (first layer).  res_out may alias residual or x.  fp32 statistics.
 * ldy: 0 or hidden (y row-major), or TGIS_LD_FRAGMENTS (rows <= 64, hidden % 64 == 0: y feeds an int4 GEMM of the decode
 * step, see TGIS_LD_FRAGMENTS above). */
int tgis_rmsnorm_residual(const void* x, const void* residual, const void* weight, void* y, int64_t ldy,
                          void* res_out, int64_t rows, int64_t hidden, float eps, int dtype,
                          void* stream);
/* Same as tgis_rmsnorm_residual with x given as split-K partial sums: x = f16(sum_s slabs[s][row][:] (+ bias)).
 * rows <= 32. */
int tgis_rmsnorm_residual_partial(const float* slabs, int num_slabs, int64_t slab_ld, const void* bias,
                                  const void* residual, const void* weight, void* y, int64_t ldy, void* res_out,
                                  int64_t rows, int64_t hidden, float eps, int dtype, void* stream);
int tgis_layernorm_residual(const void* x, const void* residual, const void* weight, const void* bias,
                            void* y, void* res_out, int64_t rows, int64_t hidden, float eps,
                            int dtype, void* stream);
/* tgis_layernorm_residual with x given as split-K partial sums (see tgis_rmsnorm_residual_partial): x = model-dtype
 * rounding of sum_s slabs[s][row][:] (+ xbias, the producing linear's bias).  Removes the reduce launch after the
 * c_proj linears of flash_santacoder_modeling.py:255-307. */
int tgis_layernorm_residual_partial(const float* slabs, int num_slabs, int64_t slab_ld, const void* xbias,
                                    const void* residual, const void* weight, const void* bias, void* y,
                                    void* res_out, int64_t rows, int64_t hidden, float eps, int dtype,
                                    void* stream);

/* ---- RoPE + KV-cache write (replaces rotary_emb.apply_rotary + the index_put at
 *      flash_llama_modeling.py:262-268,282; utils/layers.py:466-472) ---------------------------- */
/* qkv [T, (H + 2*Hkv)*D] (row stride ld_qkv): rotates q heads and k heads in place with the
 * half-split (NeoX) rotation using cos/sin tables [max_pos, rot_dim/2] of the model dtype gathered by
 * positions[T] (int32), then writes k and v of token t into KV page slot slots[t]
 * (= page_id*32 + offset).  cos == NULL skips the rotation (learned-position models).
 * k_pool / v_pool: this layer's K and V page pools, [num_pages][Hkv][32*D] each.  Inside a (page, kv head) block of
 * 32 tokens x D: K as [token >> 4][D / 8][16 tokens][8], V as [4 column groups][D][8] with token t in column
 * (i >> 2) * 8 + (t >> 4) * 4 + (i & 3), i = t & 15 (csrc/kv_layout.h, DESIGN.md section 3: the orders in which the
 * attention kernels' MFMA fragments are whole cache lines).  The pools are opaque to callers; oracle/ops_ref.py's
 * kv_page_unpack reads them back for tests. */
int tgis_rope_kv_write(void* qkv, int64_t ld_qkv, const void* cos, const void* sin,
                       const int32_t* positions, const int32_t* slots, void* k_pool, void* v_pool,
                       int64_t T, int H, int Hkv, int D, int rot_dim, int dtype, void* stream);

/* Same with the qkv activation given as split-K partial sums: qkv_out[T, ld_qkv] receives
 * f16(sum_s slabs[s] (+ bias)) with q,k rotated; k,v go to the cache. */
int tgis_rope_kv_write_partial(const float* slabs, int num_slabs, int64_t slab_ld, const void* bias, void* qkv_out,
                               int64_t ld_qkv, const void* cos, const void* sin, const int32_t* positions,
                               const int32_t* slots, void* k_pool, void* v_pool, int64_t T, int H, int Hkv, int D,
                               int rot_dim, int dtype, void* stream);

/* Prefill form of tgis_rope_kv_write for fresh sequences (token i of sequence b is cache position i): q is rotated in
 * place; k (rotated) and v go to the cache page by page — full 16-byte runs of the page layouts instead of the
 * per-token scatter — with the slots of a last partial page zeroed.  k/v inside `qkv` are left as they came.
 *   cu_seqlens [B+1]: token offsets; block_tables [B, max_pages]; T = total tokens; max_len = longest sequence. */
int tgis_rope_kv_write_prefill(void* qkv, int64_t ld_qkv, const void* cos, const void* sin, const int32_t* positions,
                               const int32_t* cu_seqlens, const int32_t* block_tables, int64_t max_pages, void* k_pool,
                               void* v_pool, int64_t B, int64_t T, int64_t max_len, int H, int Hkv, int D, int rot_dim,
                               int dtype, void* stream);

/* ---- paged attention, prefill and decode (replaces flash_attn_2_cuda.varlen_fwd,
 *      utils/flash_attn.py:43-78) ---------------------------------------------------------------- */
/* Number of key-range splits the launcher will use for this shape (so callers can size workspace). */
int tgis_attn_num_splits(int64_t B, int Hkv, int H, int64_t max_q_len, int64_t max_ctx);
int64_t tgis_attn_workspace_bytes(int64_t total_q_tokens, int H, int Hkv, int D, int num_splits);
/* Causal softmax(q k^T * scale) v over the paged cache.
 *   q: [total_q, H, D] with token stride ld_q (elements); out: [total_q, H*D] contiguous (ld_out = 0 or
 *   H*D), or — decode, B <= 64 — in fragment order for the o_proj GEMM (ld_out = TGIS_LD_FRAGMENTS).
 *   cu_seqlens_q [B+1] int32: q token offsets per sequence (decode: arange).
 *   ctx_lens [B] int32: tokens of each sequence present in the cache INCLUDING the q tokens.
 *   block_tables [B, max_pages] int32: page ids.  q token i of sequence b sits at position
 *   ctx_lens[b] - q_len_b + i and attends to cache positions <= its own.
 *   max_q_len / max_ctx are launch-shape bounds (host ints). */
int tgis_attn_paged(const void* q, int64_t ld_q, const void* k_pool, const void* v_pool,
                    const int32_t* block_tables, int64_t max_pages, const int32_t* ctx_lens,
                    const int32_t* cu_seqlens_q, void* out, int64_t ld_out, int64_t B, int H, int Hkv, int D,
                    int64_t max_q_len, int64_t max_ctx, float scale, int dtype, int num_splits,
                    void* workspace, int64_t workspace_bytes, void* stream);

/* ---- elementwise --------------------------------------------------------------------------------- */
/* out[T,I] = act(gate_up[T,0:I]) * gate_up[T,I:2I]; act 1 = SiLU (flash_llama_modeling.py:332-335). */
int tgis_act_mul(const void* gate_up, void* out, int64_t T, int64_t I, int act, int dtype, void* stream);
/* out[T,I] = gelu(x) ; approx 1 = tanh (flash_santacoder_modeling.py:303-307). */
int tgis_gelu(const void* x, void* out, int64_t n, int tanh_approx, int dtype, void* stream);
/* out[T,E] = table[ids[T]] (+ pos_table[positions[T]] if non-NULL); ids int64. Out-of-range id -> 0 row
 * (TensorParallelEmbedding's null row, utils/layers.py:325-357); ids are offset by -id_offset first. */
int tgis_embedding(const int64_t* ids, const void* table, const int32_t* positions,
                   const void* pos_table, void* out, int64_t T, int64_t E, int64_t vocab_rows,
                   int64_t id_offset, int dtype, void* stream);
/* Decode-step bookkeeping in one launch (flash_causal_lm.py:457-458,499 on device):
 * positions[b] (int32) -> slots[b] = block_tables[b][pos/32]*32 + pos%32 ; ctx_lens[b] = pos+1. */
int tgis_decode_slots(const int32_t* positions, const int32_t* block_tables, int64_t max_pages,
                      int32_t* slots, int32_t* ctx_lens, int64_t B, void* stream);
/* What follows a decode step on the device, in one launch (flash_causal_lm.py:457 `cu_seqlens.add_(cu_seqlens_q)`, :499
 * `position_ids += 1`, :533-535 `all_input_ids_tensor.scatter_(1, position_ids, next ids)`): position_ids int64 [B] += 1;
 * all_input_ids[b][position_ids[b]] = ids[b] (row stride ld_all, NULL: skip); ids_copy [B] = ids (NULL: skip; the caller's
 * next `input_ids`, since `ids` is a buffer the next step overwrites); cu_seqlens int32 [B + 1] += cu_seqlens_q (NULL:
 * skip); stage_ids int64 [B] / stage_positions int32 [B]: the same new ids / positions once more, e.g. into the static
 * input buffers of a captured decode step (NULL: skip). */
int tgis_decode_advance(const int64_t* ids, int64_t* ids_copy, int64_t* position_ids, int64_t* all_input_ids,
                        int64_t ld_all, int32_t* cu_seqlens, const int32_t* cu_seqlens_q, int64_t* stage_ids,
                        int32_t* stage_positions, int64_t B, void* stream);

/* ---- greedy sampling (Greedy + log_softmax + gather, utils/tokens.py:44-46,238-271,388-397) ------ */
/* Per row: token = argmax (lowest id on ties), logprob = logit[token] - logsumexp(row).
 * logits [B,V] f32 (logits_f32 != 0) or model dtype. ids_out int64 [B], logprob_out f32 [B].
 * scratch (may be NULL): tgis_argmax_scratch_bytes(B) bytes of device memory the call may use until it completes; with it
 * a small batch's rows are split over several workgroups each (two launches; same ids, logprobs within summation order). */
int64_t tgis_argmax_scratch_bytes(int64_t B);
int tgis_argmax_logprob(const void* logits, int64_t ld, int64_t B, int64_t V, int logits_f32, int dtype,
                        int64_t* ids_out, float* logprob_out, void* scratch, int64_t scratch_bytes, void* stream);

/* ---- next-token chooser for a heterogeneous batch -------------------------------------------------
 * One launch for what HeterogeneousNextTokenChooser.__call__ (utils/tokens.py:242-270) does with the
 * Heterogeneous* processors (utils/logits_process.py:93-402) and Sampling / HeterogeneousSampling
 * (utils/tokens.py:32-41,336-385), in the reference's order: EOS mask or length penalty, repetition
 * penalty, temperature, top-k, top-p, typical-p, then argmax (greedy rows) or a categorical draw.
 *   logits  [B,V] f32 (read only);  scores [B,V] f32 out: the warped scores, -inf where filtered — the
 *           tensor get_token_info (utils/tokens.py:388-425) takes top-n tokens and ranks from.
 *   Per-row parameter arrays, each may be NULL (= processor not instantiated): temperature; top_k
 *   (0 = off); top_p_cut = 1 - top_p as the host rounded it (<= 0 = off); typical_p (>= 1 = off);
 *   rep_penalty (1 = off) with input_ids [B,L] int64 (row stride ld_ids; padding included, as the
 *   reference passes it) and exclude_id (the id the penalty leaves alone, -1 = none);
 *   eos_adjust [B,2] = (mode, factor): mode 1 sets scores[eos_id] = -inf (min_new_tokens), mode 2
 *   scores[eos_id] += |scores[eos_id]| * factor (length penalty); do_sample [B] (NULL = all greedy).
 *   rng [B,2] uint64 (seed, offset): the request's Philox4x32-10 stream; offset += 1 per draw.
 * Outputs: next_ids int64 [B]; next_logprob f32 [B] = log_softmax(scores)[id]; lse f32 [B] =
 * logsumexp(scores) (log_softmax of a row = scores - lse). */
int tgis_warp_sample(const float* logits, int64_t ld_logits, float* scores, int64_t ld_scores, int64_t B,
                     int64_t V, const float* temperature, const int* top_k, const float* top_p_cut,
                     const float* typical_p, const float* rep_penalty, const int64_t* input_ids,
                     int64_t ld_ids, int64_t L, int64_t exclude_id, const float* eos_adjust, int64_t eos_id,
                     const int* do_sample, uint64_t* rng, int64_t* next_ids, float* next_logprob, float* lse,
                     void* stream);

/* ==== fp32-residual / ragged-step family ==============================================================
 * For decoders that keep the residual stream in fp32, put norms on both sides of every sublayer, run
 * ragged steps (portions of prompts beside single decoded tokens) and mix attention with recurrent layers.
 * Activations ("T*") are TGIS_F16, TGIS_BF16 or TGIS_F32; gains, statistics, states and the residual
 * are float.  Ragged steps are described as everywhere in this library: cu_seqlens_q [B + 1] (the step's
 * tokens, concatenated by sequence), ctx_lens [B] (tokens per sequence including the step's), positions
 * and slots per token.  A step's tokens are the last tokens of their sequences. */

/* out[t][:] = table[ids[t]][:] * scale as float; ids outside [0, vocab) give zeros. */
int tgis_embedding_scaled_f32(const int64_t* ids, const void* table, float* out, int64_t T, int64_t E, int64_t vocab,
                              float scale, int dtype, void* stream);
/* RMS norm on both sides of a residual add, one launch per row set:
 *   delta != NULL:  x_out = x + delta / sqrt(mean(delta^2) + eps) * (post_w + post_add)      (else x_out = x)
 *   pre_w != NULL:  y     = x_out / sqrt(mean(x_out^2) + eps) * (pre_w + pre_add)            (dtype y_dtype)
 * post_add / pre_add = 1 for gains stored around zero, 0 for plain gains.  x_out may be x. */
int tgis_sandwich_norm_f32(const float* x, const void* delta, int64_t ld_delta, int delta_dtype, const float* post_w,
                           float post_add, float* x_out, const float* pre_w, float pre_add, void* y, int y_dtype,
                           int64_t rows, int64_t E, float eps, void* stream);
/* The same with delta given as the num_slabs fp32 split-K slabs of the GEMM before it ([row / 32][S][32][slab_ld], as
 * tgis_dense_gemm_partial leaves them): the sum is taken here.  E % 4 == 0, E <= 8192. */
int tgis_sandwich_norm_f32_partial(const float* x, const float* slabs, int num_slabs, int64_t slab_ld, const float* post_w,
                                   float post_add, float* x_out, const float* pre_w, float pre_add, void* y, int y_dtype,
                                   int64_t rows, int64_t E, float eps, void* stream);
/* tgis_dense_gemm(act = 2) on a gate | up image, with the clamped unit of tgis_glu (mode 1) in the epilogue, computed
 * from the fp32 sums: out [M, N / 2] in the model dtype (TGIS_F16 / TGIS_BF16). */
int tgis_dense_gemm_clamped_glu(const void* x, int64_t ldx, const void* prepared, void* out, int64_t ldo, int64_t M, int64_t K,
                                int64_t N, int dtype, float alpha, float limit, void* workspace, int64_t workspace_bytes,
                                void* stream);
/* out[t][i] = act(in[t][i]) * in[t][I + i].  mode 0: silu(gate) * up.  mode 1: g = min(gate, limit),
 * u = clamp(up, -limit, limit), g * sigmoid(alpha g) * (u + 1). */
int tgis_glu(const void* in, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int64_t I, int mode, float alpha,
             float limit, int dtype, void* stream);

/* "Rows" cache pages (TGIS_KV_PAGE_TOKENS tokens): k_pool[page][G][token][dk], v_pool[page][G][dv][token].
 * qkv [T, H dk | G dk | G dv]: q heads are RMS-normed (gain q_gain[dk], eps inside the root), multiplied by
 * 1 + gain_coef * ln(floor((position + 1) / gain_every) + 1) (gain_every <= 0: no position gain) and written back in
 * place; k heads are RMS-normed (k_gain) and written to the token's slot; v is written to its slot, blended first as
 * (1 - *v_lambda) v + *v_lambda v_first[t] when v_first != NULL (v_first [T, G dv], row stride ld_v_first). */
int tgis_qk_norm_kv_write(void* qkv, int64_t ld, const int32_t* positions, const int32_t* slots, const float* q_gain,
                          const float* k_gain, float eps, float gain_coef, int gain_every, const void* v_first,
                          int64_t ld_v_first, const float* v_lambda, void* k_pool, void* v_pool, int64_t T, int H, int G,
                          int dk, int dv, int dtype, void* stream);
/* out[t][h][:] = softmax_j(scale q[t][h] . k[j]) v[j] over keys j <= the token's position, fp32 scores and weights;
 * query head h reads kv head h / (H / G).  max_q_len / max_ctx: upper bounds of a sequence's run in this step and of
 * ctx_lens (launch shaping only).  impl 0: the matrix-core kernel where it applies (two-byte dtype, dk % 16 == 0,
 * dv % 32 == 0, both <= 256; the weights are rounded to T for the P V product), else the general one (any widths, dv <= 256,
 * fp32 throughout); 1 / 2 force one of them. */
int tgis_attn_varlen(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                     int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B, void* out,
                     int64_t ld_out, int64_t total_q, int64_t max_q_len, int64_t max_ctx, int H, int G, int dk, int dv,
                     float scale, int impl, int dtype, void* stream);

/* Token shift: out[s][t][:] = h[t] + (h[t - 1] - h[t]) * mu[s], s < num_mixes; h[t - 1] of a sequence's first token in
 * the step is shift_state[state_slots[b]], or zero when that token is at position 0. */
int tgis_token_shift_mix(const float* h, const float* shift_state, const int32_t* state_slots, const int32_t* cu_seqlens_q,
                         const int32_t* positions, int64_t B, const float* mu, int num_mixes, void* out, int64_t T,
                         int64_t W, int dtype, void* stream);
/* logw[t][c] = -exp(w0[c] + sum_r tanh(a[t][r]) * w2t[r][c]) : the logarithm of a per-channel decay in (0, 1). */
int tgis_wkv_decay(const void* a, int64_t ld_a, const float* w2t, const float* w0, float* logw, int64_t T, int rank,
                   int64_t C, int dtype, void* stream);
/* Per (sequence, head), tokens in order:  o = (S + diag(u) k v^T)^T r;  S <- diag(exp(logw)) S + k v^T;
 * out = o / sqrt(mean(o^2) + eps) * gain * silu(gate).  state [slots][H][d][d] (key channel, value channel) and
 * shift_state [slots][W] are read (unless the step starts at position 0: zeros) and written back; shift_state gets the
 * last row of h [T, W].  d <= 128. */
int tgis_wkv_scan(const void* r, const void* k, const void* v, const void* gate, int64_t ld, const float* logw,
                  const float* u, const float* gain, float* state, float* shift_state, const float* h, int64_t W,
                  const int32_t* state_slots, const int32_t* cu_seqlens_q, const int32_t* positions, void* out,
                  int64_t ld_out, int64_t B, int H, int d, float eps, int dtype, void* stream);

/* Mixture of experts, no host round trip.  Pairs p = t * k + j.  Rows of the grouped GEMMs live in 32-row tiles, one
 * expert per tile; tgis_moe_row_capacity(n_pairs, E) rows always suffice. */
int64_t tgis_moe_row_capacity(int64_t n_pairs, int64_t E);
/* idx / weight [T][k]: the k experts with the largest router_w[e] . h[t] (fp32) and sigmoid of that logit;
 * shared_gate[t] = sigmoid(shared_gate_w . h[t]) when shared_gate_w != NULL. */
int tgis_moe_route(const void* h, int64_t ld_h, const float* router_w, const float* shared_gate_w, int32_t* idx,
                   float* weight, float* shared_gate, int64_t T, int64_t W, int E, int k, int dtype, void* stream);
/* sorted [capacity] = pair per row (-1: padding), tile_expert [capacity / 32], pos_of_pair [n_pairs], n_tiles [1]. */
int tgis_moe_align(const int32_t* idx, int64_t n_pairs, int E, int32_t* sorted, int64_t capacity, int32_t* tile_expert,
                   int32_t* pos_of_pair, int32_t* n_tiles, void* stream);
/* out[row][n] = sum_c a(row)[c] * W[tile_expert[row / 32]][n][c], weights [E][N (glu: 2 N)][K] k-contiguous.
 * a(row) = A[sorted[row] / pair_div] * pair_scale[sorted[row]] (rounded to T) when sorted != NULL, else A[row].
 * glu: out = silu(gate) * up with gate rows [0, N) and up rows [N, 2 N) of each expert. */
int tgis_moe_gemm(const void* A, int64_t ld_a, const int32_t* sorted, int pair_div, const float* pair_scale,
                  const int32_t* tile_expert, const int32_t* n_tiles, const void* weights, int64_t expert_stride, int64_t N,
                  int64_t K, int glu, void* out, int64_t ld_out, int64_t capacity, int dtype, void* stream);
/* out[t] = sum_j rows[pos_of_pair[t k + j]] * (pair_weight[t k + j] or 1) + (shared_gate[t] or 1) * shared[t]. */
int tgis_moe_combine(const void* rows, int64_t ld_rows, const int32_t* pos_of_pair, const float* pair_weight, int k,
                     const void* shared, int64_t ld_shared, const float* shared_gate, void* out, int64_t ld_out, int64_t T,
                     int64_t W, int dtype, void* stream);

/* ---- pre-norm hybrid decoders with a residual multiplier (Senadra): residual update, activations, cache writes,
 *      masked / biased attention and the gated delta rule.  T = TGIS_F16 / TGIS_BF16 / TGIS_F32 as above. */

/* The residual update in one launch, generalising tgis_sandwich_norm_f32:
 *   delta, post_w:      x_out = x + post_scale * delta / sqrt(mean(delta^2) + eps) * (post_w + post_add)
 *   delta, post_w NULL: x_out = x + post_scale * delta
 *   pre_w:              y = x_out / sqrt(mean(x_out^2) + eps) * (pre_w + pre_add)
 *   pre_w NULL, y:      y = x_out rounded to y_dtype
 * The _partial form takes delta as the fp32 split-K slabs of tgis_dense_gemm_partial. */
int tgis_residual_update_f32(const float* x, const void* delta, int64_t ld_delta, int delta_dtype, const float* post_w,
                             float post_add, float post_scale, float* x_out, const float* pre_w, float pre_add, void* y,
                             int y_dtype, int64_t rows, int64_t E, float eps, void* stream);
int tgis_residual_update_f32_partial(const float* x, const float* slabs, int num_slabs, int64_t slab_ld, const float* post_w,
                                     float post_add, float post_scale, float* x_out, const float* pre_w, float pre_add, void* y,
                                     int y_dtype, int64_t rows, int64_t E, float eps, void* stream);
/* out = xIELU(in):  z > 0: ap z^2 + z / 2;  z <= 0: an (exp(z) - 1 - z) + z / 2   (ap, an: the folded coefficients). */
int tgis_xielu(const void* in, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int64_t C, float ap, float an,
               int dtype, void* stream);
/* tgis_dense_gemm (no bias, model-dtype output) with xIELU applied where the output is finished: one launch for the
 * up-projection of W_down xielu(W_up h) at decode sizes; the same bits as tgis_dense_gemm followed by tgis_xielu. */
int tgis_dense_gemm_xielu(const void* x, int64_t ldx, const void* prepared, void* out, int64_t ldo, int64_t M, int64_t K,
                          int64_t N, int dtype, float ap, float an, void* workspace, int64_t workspace_bytes, void* stream);
/* tgis_dense_gemm (no bias, model-dtype output) whose finished sums become gelu_tanh(sum) * table[ids[m]][col0 + n]: the
 * gate projection and the gated lookup of a per-layer token input in one launch at decode sizes; the same bits as
 * tgis_dense_gemm followed by tgis_gelu_gated_lookup. */
int tgis_dense_gemm_gelu_lookup(const void* x, int64_t ldx, const void* prepared, const int64_t* ids, const void* table,
                                int64_t ld_table, int64_t col0, int64_t vocab, void* out, int64_t ldo, int64_t M, int64_t K,
                                int64_t N, int dtype, void* workspace, int64_t workspace_bytes, void* stream);
/* out = in * sigmoid(gate); out may alias in. */
int tgis_sigmoid_gate_mul(const void* in, int64_t ld_in, const void* gate, int64_t ld_gate, void* out, int64_t ld_out,
                          int64_t rows, int64_t C, int dtype, void* stream);
/* logits <- cap * tanh(logits / cap), in place. */
int tgis_logit_softcap(float* logits, int64_t ld, int64_t rows, int64_t V, float cap, void* stream);
/* out[t][c] = gelu_tanh(gate[t][c]) * table[ids[t]][col0 + c], c < C: a gated slice of a second token embedding. */
int tgis_gelu_gated_lookup(const void* gate, int64_t ld_gate, const int64_t* ids, const void* table, int64_t ld_table,
                           int64_t col0, int64_t vocab, void* out, int64_t ld_out, int64_t rows, int64_t C, int dtype,
                           void* stream);
/* y = x / sqrt(mean(x^2) + eps) * w over rows of C channels (latents); y may alias x. */
int tgis_rms_norm_rows(const void* x, int64_t ld_x, const float* w, void* y, int64_t ld_y, int64_t rows, int64_t C,
                       float eps, int dtype, void* stream);
/* Keys (as projected) and values (v_norm: each head / its root mean square, no gain) of a step into their page slots
 * ("rows" layout of tgis_attn_varlen).  Keys at columns k_col0 + g dk of qkv, values at v_col0 + g dv. */
int tgis_kv_norm_write(void* qkv, int64_t ld, int64_t k_col0, int64_t v_col0, const int32_t* slots, void* k_pool,
                       void* v_pool, int64_t T, int G, int dk, int dv, int v_norm, float eps, int dtype, void* stream);
/* Latent attention: cache row [normed latent (kv_rank) | rotated shared key part (dr)] as the K page of one kv head, the
 * latent again as its V page; rotated query parts into columns kv_rank.. of each head's row of q_abs [T, H (kv_rank + dr)].
 * Pair (2i, 2i + 1) of the first rot_dims channels turns by position * inv_freq[i]. */
int tgis_latent_kv_write(const void* q, int64_t ldq, void* ckv, int64_t ld_ckv, const float* c_gain, const float* inv_freq,
                         const int32_t* positions, const int32_t* slots, void* q_abs, int64_t ld_q_abs, void* k_pool,
                         void* v_pool, int64_t T, int H, int dn, int dr, int kv_rank, int rot_dims, float eps, int dtype,
                         void* stream);
/* tgis_attn_varlen with a block mask (chunk > 0: position i sees j <= i only if i / chunk == j / chunk), a distance
 * bias per query head (r1, r2 [H]: the score loses r1 ln(1 + r2 (i - j))) and / or a sigmoid output gate
 * (gate [T, >= H dv], activation dtype: out *= sigmoid(gate) where the output is written).  workspace (optional): scratch for
 * decode steps with few sequences x cached heads, whose pages are then dealt to several workgroups and combined. */
int tgis_attn_varlen_ext(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                         int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B, void* out,
                         int64_t ld_out, int64_t total_q, int64_t max_q_len, int64_t max_ctx, int H, int G, int dk, int dv,
                         float scale, const float* r1, const float* r2, int chunk, const void* gate, int64_t ld_gate,
                         void* workspace, int64_t workspace_bytes, int impl, int dtype, void* stream);
/* Causal per-channel convolution over time and SiLU: out[t][c] = silu(sum_j w[c][j] x[t - (taps - 1 - j)][c]); inputs before a
 * step's first token come from tail[state_slots[b]] ([taps - 1][C] fp32), zeros when the step starts at position 0. */
int tgis_short_conv_silu(const void* x, int64_t ld_x, const float* w, const float* tail, const int32_t* state_slots,
                         const int32_t* cu_seqlens_q, const int32_t* positions, int64_t B, float* out, int64_t T,
                         int64_t C, int taps, int dtype, void* stream);
/* floats of one head's matrix state in a slot, as tgis_delta_scan keeps it (-1: unsupported widths). */
int64_t tgis_delta_state_floats(int dk, int dv);
/* Gated delta rule per (sequence, head), tokens in order, on conv = the activated q | k | v of tgis_short_conv_silu:
 *   q, k unit vectors (q * q_scale);  beta = sigmoid(b);  g = exp(-exp(A_log[h]) softplus(a + dt_bias))  per key channel;
 *   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;  out = o / rms(o) * gain * sigmoid(gate).
 * state and tail are read (zeros when the step starts at position 0) and written back; tail gets the last taps - 1 rows of
 * proj (the projection before the convolution).  Query / key head of value head h: h / (H / G). */
int tgis_delta_scan(const float* conv, int64_t C, const void* a, int64_t ld_a, const void* b, int64_t ld_b, const void* gate,
                    int64_t ld_gate, const float* A_log, const float* dt_bias, const float* gain, float* state, float* tail,
                    const void* proj, int64_t ld_proj, const int32_t* state_slots, const int32_t* cu_seqlens_q,
                    const int32_t* positions, void* out, int64_t ld_out, int64_t B, int H, int G, int dk, int dv, int taps,
                    float eps, float unit_eps, float q_scale, int dtype, void* stream);

/* ---- parallel-layer decoders with gated residuals (Mananex): windowed attention with a sink, rotation in the "rows" page
 *      layout, a gated linear recurrence, the parallel residual update with a mix over depth.  T as above. */

/* Interleaved-pair rotation of q (in place) and k (into its page slot), and the value write, of a step.  proj [T, ld] holds q
 * at columns q_col0 + h dk, k at k_col0 + g dk, v at v_col0 + g dv.  Pair (2i, 2i + 1) of the first rot_dims channels of every
 * q and k head turns by positions[t] * inv_freq[i] (angle, sine and cosine in fp32); the other channels pass. */
int tgis_rope_rows_kv_write(void* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, const float* inv_freq,
                            const int32_t* positions, const int32_t* slots, void* k_pool, void* v_pool, int64_t T, int H, int G,
                            int dk, int dv, int rot_dims, int dtype, void* stream);
/* tgis_attn_varlen with a sliding window that keeps the first positions (window > 0: position i sees j <= i only if
 * i - j < window or j < keep_first; kept keys stay at their positions; pages between them and the window are not read), a sink
 * logit per query head in the softmax denominator (sink [H] fp32 or NULL: exp(sink[h]) is added once, unscaled, with no value),
 * a sigmoid output gate (gate_per_head != 0: gate [T, >= H], one logit per (token, head); else gate [T, >= H dv]) and a constant
 * factor out_scale on the output.  out may be a column range of a wider buffer (ld_out).  workspace as in tgis_attn_varlen_ext. */
int tgis_attn_varlen_win(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                         int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B, void* out,
                         int64_t ld_out, int64_t total_q, int64_t max_q_len, int64_t max_ctx, int H, int G, int dk, int dv,
                         float scale, int window, int keep_first, const float* sink, const void* gate, int64_t ld_gate,
                         int gate_per_head, float out_scale, void* workspace, int64_t workspace_bytes, int impl, int dtype,
                         void* stream);
/* Gated linear recurrence per (sequence, head), tokens in order, on columns of proj [T, ld]:
 *   q = proj[q_col0 + h dk ..] (q_act 1: silu of it);  f = lower + (1 - lower) sigmoid(proj[f_col0 + h dk ..] + f_bias)  (fp32;
 *   lower, f_bias [H dk] fp32 or NULL = 0);  v = proj[v_col0 + h dv ..];
 *   S <- diag(f) S + (1 - f) v^T;  o = S^T q (the new state);  out = o / sqrt(mean(o^2) + eps) * gain[dv] * out_scale.
 * state [slots][H][dk][dv] fp32 is read (zeros when the step starts at position 0) and written back.  dk, dv <= 256;
 * T: tokens of the step; max_q_len: an upper bound of a sequence's run in it (launch shaping only); scratch (optional): T * H * dv
 * floats that let a long step of few sequences deal a head's value columns to several workgroups (the norm then runs as a
 * pass of its own over the unnormed read-outs left there). */
int tgis_gated_linear_scan(const void* proj, int64_t ld, int64_t q_col0, int64_t f_col0, int64_t v_col0, const float* f_bias,
                           const float* lower, const float* gain, float* state, const int32_t* state_slots,
                           const int32_t* cu_seqlens_q, const int32_t* positions, void* out, int64_t ld_out, float out_scale,
                           int64_t B, int64_t T, int64_t max_q_len, int H, int dk, int dv, float eps, int q_act, float* scratch,
                           int dtype, void* stream);
/* tgis_moe_route with a bias on the router logits (router_b [E] fp32 or NULL) and, with softmax_top != 0, weights that are the
 * softmax over the chosen logits only (0: the sigmoid of each chosen logit). */
int tgis_moe_route_ext(const void* h, int64_t ld_h, const float* router_w, const float* router_b, const float* shared_gate_w,
                       int softmax_top, int32_t* idx, float* weight, float* shared_gate, int64_t T, int64_t W, int E, int k,
                       int dtype, void* stream);
/* The residual update of a parallel layer (mixer a and feed-forward b read the same normed input) with gated residuals and a
 * learned mix over depth, and the next norm, in one launch:
 *   v = x + sigmoid(gate_a + gate_bias_a) (a + bias_a) + sigmoid(gate_b + gate_bias_b) (b + bias_b)
 *   hist[n_prev] = v;  x_out = sum_{j <= n_prev} mix[j] hist[j]  (hist NULL: x_out = v);
 *   y = x_out / sqrt(mean(x_out^2) + eps) * (pre_w + pre_add)  (pre_w NULL: none)
 * a / b: [rows, ld] of `dtype`, or with slabs_x > 0 the fp32 split-K slabs of tgis_dense_gemm_partial (ld_x = their row
 * stride); b, the biases [E], gate logits [rows, ld_gate] and gate biases [E] (all of `dtype`) may be NULL.
 * hist: n_prev + 1 entries [rows, E] fp32, hist_stride floats apart; mix [n_prev + 1] fp32.  x_out may alias x. */
int tgis_parallel_residual_f32(const float* x, const void* a, int64_t ld_a, int slabs_a, const void* bias_a, const void* gate_a,
                               int64_t ld_gate_a, const void* gate_bias_a, const void* b, int64_t ld_b, int slabs_b,
                               const void* bias_b, const void* gate_b, int64_t ld_gate_b, const void* gate_bias_b, int dtype,
                               float* hist, int n_prev, int64_t hist_stride, const float* mix, float* x_out, const float* pre_w,
                               float pre_add, void* y, int y_dtype, int64_t rows, int64_t E, float eps, void* stream);

/* ---- parallel layers with per-channel sublayer scales, input convolutions, a selective scan, attention with scores mixed over
 * heads, and the general linear-attention scan -------------------------------------------------------------------------- */
/* tgis_rope_rows_kv_write, and every q and k head is divided by sqrt(mean(x^2) + unit_eps) after the rotation (no gain). */
int tgis_rope_rows_unit_kv_write(void* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, const float* inv_freq,
                                 const int32_t* positions, const int32_t* slots, void* k_pool, void* v_pool, int64_t T, int H,
                                 int G, int dk, int dv, int rot_dims, float unit_eps, int dtype, void* stream);
/* Paged softmax attention ("rows" page layout) whose scaled scores are mixed over the query heads before the softmax:
 * s'_h = sum_g mix[h][g] s_g, mix [H][H] fp32; a query at position i sees keys j <= i with i - j < window (window 0: all);
 * out[t][h dv + c] is multiplied by sigmoid(gate[t][h dv + c]) when gate is given.  H dv <= 4096.  total_q: tokens of the step;
 * max_q_len, max_ctx: upper bounds (launch shaping only).  workspace (optional): scratch for the key-split form of steps of
 * single tokens (splits * total_q * H * (dv + 2) floats are used, as many splits as fit).  impl 0: the launcher chooses
 * (matrix-core form for prompt portions of two-byte models with dk % 16 == 0 and dv % 16 == 0); 1: the general kernel. */
int tgis_attn_mixed_heads(const void* q, int64_t ldq, const void* k_pool, const void* v_pool, const int32_t* block_tables,
                          int64_t max_pages, const int32_t* ctx_lens, const int32_t* cu_seqlens_q, int64_t B, const float* mix,
                          const void* gate, int64_t ld_gate, void* out, int64_t ld_out, int64_t total_q, int64_t max_q_len,
                          int64_t max_ctx, int H, int G, int dk, int dv, float scale, int window, void* workspace,
                          int64_t workspace_bytes, int impl, int dtype, void* stream);
/* Linear attention S <- diag(a) S + k v^T, o = S^T q per (sequence, head) on columns of proj [T, ld]:
 *   decay_mode 0: a = lower + (1 - lower) sigmoid(f + f_bias);  1: a = sigmoid(f + f_bias)^inv_tau;  2: a = head_decay[h];
 *   k at k_col0 (k_col0 < 0: k = 1 - a);  q_act / k_act / v_act != 0: SiLU on the projection;  q times q_scale;
 *   norm_rows 0: out = o / rms(o over the head) * gain[dv];  != 0: out = o / rms(o over all heads) * gain[H dv] (needs scratch);
 *   gate_act 1: times sigmoid(gate[t][h dv + c]);  2: times SiLU of it.
 * state [slots][H][dk][dv] fp32 as in tgis_gated_linear_scan; scratch: T * H * dv floats or NULL. */
int tgis_linear_scan(const void* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t f_col0, int64_t v_col0,
                     const float* f_bias, const float* lower, const float* head_decay, int decay_mode, float inv_tau, int q_act,
                     int k_act, int v_act, float q_scale, const float* gain, int norm_rows, const void* gate, int64_t ld_gate,
                     int gate_act, float* state, const int32_t* state_slots, const int32_t* cu_seqlens_q,
                     const int32_t* positions, void* out, int64_t ld_out, float out_scale, int64_t B, int64_t T,
                     int64_t max_q_len, int H, int dk, int dv, float eps, float* scratch, int dtype, void* stream);
/* Causal per-channel convolution over time for ragged steps, `sets` (1 or 2) filter sets on the same input:
 *   out_s[t][c] = act(bias_s[c] + sum_j w_s[c][j] x[t - (taps - 1 - j)][c]) (+ x[t][c] if residual);  act 1: SiLU.
 * x [T, ld_x] fp32 (x_f32) or `dtype`; w [sets][C][taps], bias [sets][C] or NULL (fp32); out_s = out + s * set_stride elements,
 * rows ld_out apart, `dtype`.  tail: slot s at tail + s * tail_stride floats holds [taps - 1][C], the inputs just before the
 * step (zeros when the step starts at position 0); it is moved on to the step's end by the same launch. */
int tgis_causal_conv(const void* x, int64_t ld_x, int x_f32, const float* w, const float* bias, int sets, float* tail,
                     int64_t tail_stride, const int32_t* state_slots, const int32_t* cu_seqlens_q, const int32_t* positions,
                     int64_t B, void* out, int64_t ld_out, int64_t set_stride, int64_t max_q_len, int64_t C, int taps, int act,
                     int residual, int dtype, void* stream);
/* Selective state-space scan per (sequence, channel c, state n), tokens in order:
 *   d = softplus(dt[t][c] + dt_bias[c]);  S[c][n] <- exp(-d exp(A_log[c][n])) S[c][n] + d x[t][c] B[t][n];
 *   out[t][c] = (sum_n S[c][n] C[t][n] + D[c] x[t][c]) silu(z[t][c]).
 * x, z, out [T, >= inner] and bc [T, ld_bc] (B at b_col0, C at c_col0, N columns each) of `dtype`; dt fp32 (dt_f32) or `dtype`;
 * state [slots][inner][N] fp32, read unless the step starts at position 0, written back.  N <= 128.  max_q_len: an upper bound
 * of a sequence's run in the step (launch shaping only). */
int tgis_selective_scan(const void* x, int64_t ld_x, const void* dt, int64_t ld_dt, int dt_f32, const float* dt_bias,
                        const void* bc, int64_t ld_bc, int64_t b_col0, int64_t c_col0, const void* z, int64_t ld_z,
                        const float* A_log, const float* D, float* state, const int32_t* state_slots,
                        const int32_t* cu_seqlens_q, const int32_t* positions, void* out, int64_t ld_out, int64_t B,
                        int64_t max_q_len, int64_t inner, int N, int dtype, void* stream);
/* x_out = x_in + s1 * a + s2 * b + v  (each term optional; s1, s2, v [W] fp32; a, b [rows, ld] fp32 or `dtype`), and
 * h = norm(x_out) * w with norm the mean-free layer norm (mean_free) or the RMS norm, eps inside the root; h fp32 (h_f32) or
 * `dtype`; w NULL: no norm.  x_out may alias x_in.  With a2 (optional) the first term is the average of two normed rows,
 * pair_coef * (a / rms(a) * wa + a2 / rms(a2) * wa2), instead of a (what tgis_rms_pair_mean makes, without its launch). */
int tgis_scaled_residual_norm(const float* x_in, float* x_out, const void* a, int64_t ld_a, int a_f32, const float* s1,
                              const void* b, int64_t ld_b, int b_f32, const float* s2, const float* v, const float* w, void* h,
                              int h_f32, int64_t rows, int64_t W, float eps, int mean_free, const void* a2, int64_t ld_a2,
                              int a2_f32, const float* wa, const float* wa2, float pair_coef, int dtype, void* stream);
/* y = ca * a / rms(a) * wa + cb * b / rms(b) * wb over rows of W channels; a, b fp32 or `dtype`; y fp32. */
int tgis_rms_pair_mean(const void* a, int64_t ld_a, int a_f32, const float* wa, float ca, const void* b, int64_t ld_b, int b_f32,
                       const float* wb, float cb, float* y, int64_t rows, int64_t W, float eps, int dtype, void* stream);
/* y = c1 z / rms(z) + c2 z^2 / rms(z^2) + c3 z^3 / rms(z^3) + c0 over rows of F values (powers element by element). */
int tgis_poly_norm(const void* z, int64_t ld_z, void* y, int64_t ld_y, int64_t rows, int64_t F, float c1, float c2, float c3,
                   float c0, float eps, int dtype, void* stream);
/* Router with softmax scores over all experts: experts are chosen by score + correction[e] (fp32 [E] or NULL) among the
 * keep_groups best of n_groups equal groups of neighbouring experts (a group ranks by its largest choice score; the other
 * groups count as -inf); weights = the chosen experts' scores / (their sum + renorm_eps). */
int tgis_moe_route_grouped(const void* h, int64_t ld_h, const float* router_w, const float* correction, int n_groups,
                           int keep_groups, float renorm_eps, int32_t* idx, float* weight, int64_t T, int64_t W, int E, int k,
                           int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TGIS_HIP_H */
