"""Sequence mixers and feed-forward blocks for decoders with an fp32 residual stream, built on the ragged-step kernels of
libtgis_hip.so (csrc/residual_f32.hip, attn_varlen.hip, wkv.hip, moe.hip).  Every constant of a mechanism is a constructor
argument, so that a model file only maps its config keys and tensor names onto them.

  NormedQKAttention   softmax attention without a rotation: per-head RMS norm of q and k, optional position-dependent query
                      gain, optional blending of the values with another layer's, separate key / value widths, GQA
  WkvMixer            RWKV-style linear recurrence: token shift, low-rank data-dependent decay, bonus for the current token,
                      per-head unit norm, output gate; state in a RecurrentStateCache slot
  GatedUnit           W_down(act(W_gate h) * W_up h) with the plain SiLU form or the clamped sigmoid(alpha g) * (u + 1) form
  RoutedExperts       sigmoid-scored top-k mixture of GatedUnit experts whose routing weight scales the expert input, plus an
                      optional shared expert behind a sigmoid gate
  BlockBiasedAttention  softmax attention without a rotation whose queries see only their own block of positions and whose
                      scores fall with the logarithm of the distance; unit-RMS values; sigmoid output gate; may read the keys
                      and values another layer cached
  LatentAttention     queries and keys / values through normed low-rank latents, one rotated key part shared by the heads;
                      the cache holds the latent and the rotated part, the heads' key / value maps are applied to the query
                      and to the attention output instead of to every cached token
  DeltaRuleMixer      gated delta rule with a decay per head and key channel, short convolutions in front of q, k and v,
                      low-rank decay and output-gate projections; state in a RecurrentStateCache slot
  WindowSinkAttention rotated (interleaved pairs, partial) GQA softmax attention with a sliding window that keeps the first
                      positions, a learned sink logit per head in the denominator and a sigmoid gate per head
  GatedLinearRecurrence  HGRN2-style linear attention: S <- diag(f) S + (1 - f) v^T with a forget gate bounded below,
                      o = S^T silu(q), per-head RMS norm; state in a RecurrentStateCache slot
  SideBySideMixers    several mixers reading the same input through ONE stacked projection, their weighted results through
                      ONE stacked output projection
  InputConvolutions   h + conv(h): short causal per-channel convolutions in front of sublayers that read the same input
  SelectiveScanMixer  Mamba-style selective state-space scan behind a channel convolution, gated by SiLU(z)
  MixedHeadAttention  rotated, unit-RMS q and k; the heads' scores mixed by a matrix before the softmax; sliding window;
                      per-channel sigmoid output gate
  DecayedLinearAttention  S <- diag(a) S + k v^T with a per-head constant or a learned per-channel decay; per-head or
                      whole-row norm; sigmoid or SiLU output gate
  NormedPairMixers    two mixers on ONE stacked projection whose results are RMS-normed over the width and averaged
  PowerNormMLP        W_down P(W_up h), P a polynomial of the unit-RMS powers z, z^2, z^3
  ActivatedMLP        W_down act(W_up h) with the xIELU activation
  TokenSideInput      a slice of a second token embedding, gated by a GELU of a projection of the residual stream itself

Activations between kernels are in the serving dtype (bfloat16 or float32); what has to be 32-bit (norm statistics, scores,
softmax weights, router logits, decays, recurrent state) is 32-bit inside the kernels whatever the serving dtype.
All of them run ragged steps: a step's tokens are concatenated by sequence and described by a `StepArgs`-like object with
`cu_seqlens_q`, `ctx_lens`, `slots`, `block_tables`, `state_slots`, `cache`, `state` (models.custom_modeling KVArgs)."""
from typing import Optional

import torch

from tgis_amd import native
from tgis_amd.utils.layers import SKINNY_MAX_M, FastLinear, workspace

# rows up to which the clamped gated unit runs in the epilogue of the weight-streaming GEMM
CLAMPED_EPILOGUE_MAX_M = SKINNY_MAX_M


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


def can_defer(lin: FastLinear) -> bool:
    """May this projection leave its split-K sum to the sandwich norm behind it (decode-sized steps)?  The norm takes the
    slabs with 16-byte loads: widths that are multiples of 4, up to 8192."""
    return lin.streams and lin.out_features % 4 == 0 and lin.out_features <= 8192


def load_linear(weights, name: str) -> FastLinear:
    return FastLinear(weights.get_tensor(name).contiguous(), None)


def load_stacked_linear(weights, names, pad_rows_to: int = 1) -> FastLinear:
    """Several [out_i, in] weights that read the same input, as one GEMM.  pad_rows_to: zero rows are appended until the
    output width is a multiple of it (so that an output row starts on 16 bytes and column slices can feed the next GEMM)."""
    w = torch.cat([weights.get_tensor(n) for n in names], dim=0)
    extra = -w.shape[0] % pad_rows_to
    if extra:
        w = torch.cat([w, w.new_zeros((extra, w.shape[1]))], dim=0)
    return FastLinear(w.contiguous(), None)


class NormedQKAttention:
    def __init__(self, weights, prefix: str, layer_id: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 eps: float, gain_coef: float = 0.0, gain_every: int = 0, blend: bool = False):
        self.layer_id = layer_id
        self.H, self.G, self.dk, self.dv = heads, kv_heads, dim, vdim
        self.scale, self.eps = float(scale), float(eps)
        self.gain_coef, self.gain_every = float(gain_coef), int(gain_every)
        self.qkv = load_stacked_linear(weights, [f"{prefix}.q", f"{prefix}.k", f"{prefix}.v"])
        self.o = load_linear(weights, f"{prefix}.o")
        self.q_gain = _f32(weights.get_tensor(f"{prefix}.q.norm"))
        self.k_gain = _f32(weights.get_tensor(f"{prefix}.k.norm"))
        # blend: v <- (1 - lambda) v + lambda v_other, lambda a learned scalar kept on the device
        self.v_lambda = _f32(weights.get_tensor(f"{prefix}.vmix")).reshape(1) if blend else None
        self.defer = can_defer(self.o)

    def values_of(self, qkv: torch.Tensor) -> torch.Tensor:
        """The value columns of a projected step (what another layer blends with)."""
        return qkv[:, (self.H + self.G) * self.dk:]

    def forward(self, h: torch.Tensor, position_ids, step, v_other: Optional[torch.Tensor] = None):
        """h [T, W] -> (out [T, W], qkv [T, H dk + G dk + G dv] with q normed in place)."""
        qkv = self.qkv(h)
        cache = step.cache
        k_pool, v_pool = cache.k_pool(self.layer_id), cache.v_pool(self.layer_id)
        native.qk_norm_kv_write(qkv, position_ids, step.slots, self.q_gain, self.k_gain, self.eps, self.gain_coef,
                                self.gain_every, v_other if self.v_lambda is not None else None, self.v_lambda, k_pool, v_pool,
                                self.H, self.G, self.dk, self.dv)
        att = native.attn_varlen(qkv, k_pool, v_pool, step.block_tables, step.ctx_lens, step.cu_seqlens_q, self.H, self.G,
                                 self.dk, self.dv, self.scale, max_q_len=step.max_q_len, max_ctx=step.max_ctx)
        return self.o(att, partial=self.defer), qkv


class WkvMixer:
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, weights, prefix: str, layer_id: int, heads: int, dim: int, eps: float):
        self.layer_id = layer_id
        self.H, self.d, self.eps = heads, dim, float(eps)
        self.mu = torch.stack([_f32(weights.get_tensor(f"{prefix}.mu.{s}")) for s in self.MIXES]).contiguous()
        self.proj = [load_linear(weights, f"{prefix}.{s}") for s in ("r", "k", "v", "g")]
        self.w1 = load_linear(weights, f"{prefix}.w1")
        self.w2t = _f32(weights.get_tensor(f"{prefix}.w2")).t().contiguous()  # [rank, H d]
        self.w0 = _f32(weights.get_tensor(f"{prefix}.w0"))
        self.u = _f32(weights.get_tensor(f"{prefix}.u")).reshape(-1)
        self.gain = _f32(weights.get_tensor(f"{prefix}.norm"))
        self.o = load_linear(weights, f"{prefix}.o")
        self.defer = can_defer(self.o)

    def forward(self, h32: torch.Tensor, position_ids, step, dtype):
        """h32 [T, W] fp32 (the normed mixer input, kept in fp32 because it is also the shift state)."""
        st = step.state
        state, shift = st.state[self.layer_id], st.shift[self.layer_id]
        mixes = native.token_shift_mix(h32, shift, step.state_slots, step.cu_seqlens_q, position_ids, self.mu, dtype)
        T = h32.shape[0]
        HD = self.H * self.d
        rkvg = torch.empty((4, T, HD), dtype=dtype, device=h32.device)
        for i, lin in enumerate(self.proj):
            lin(mixes[i], out=rkvg[i])
        logw = native.wkv_decay(self.w1(mixes[4]), self.w2t, self.w0)
        out = native.wkv_scan(rkvg[0], rkvg[1], rkvg[2], rkvg[3], logw, self.u, self.gain, state, shift, h32, step.state_slots,
                              step.cu_seqlens_q, position_ids, self.H, self.d, self.eps)
        return self.o(out, partial=self.defer)


class GatedUnit:
    """mode "silu": silu(g) * u.  mode "clamped": g = min(g, limit), u = clamp(u, +-limit), g * sigmoid(alpha g) * (u + 1)."""

    def __init__(self, weights, prefix: str, mode: str = "silu", alpha: float = 1.0, limit: float = 0.0, bias: bool = False):
        """bias: the three projections have biases (`<name>.b`)."""
        self.gate_up = load_stacked_linear(weights, [f"{prefix}.gate", f"{prefix}.up"])
        self.down = load_linear(weights, f"{prefix}.down")
        if bias:
            self.gate_up.bias = torch.cat([weights.get_tensor(f"{prefix}.gate.b"), weights.get_tensor(f"{prefix}.up.b")]).contiguous()
            self.down.bias = weights.get_tensor(f"{prefix}.down.b").contiguous()
        self.ff = self.gate_up.out_features // 2
        self.mode = {"silu": 0, "clamped": 1}[mode]
        self.alpha, self.limit = float(alpha), float(limit)
        # the plain SiLU form is the epilogue the weight-streaming kernel already has for the Llama MLP (act 2 on a
        # gate | up image); the clamped form is a launch of its own
        self.fused = self.mode == 0 and self.gate_up.streams and self.ff % 16 == 0
        if self.fused:
            self.gate_up.gate_up = True
        # the clamped form at decode sizes: the same gate | up image with the clamped unit in the epilogue (a second image
        # of the weight; longer steps take the library GEMM on the checkpoint layout and the activation launch)
        self.clamped_image = None
        if self.mode == 1 and self.gate_up.streams and self.ff % 16 == 0 and self.limit > 0:
            self.clamped_image = native.DenseWeight(self.gate_up.weight, gate_up=True)

    def forward(self, h: torch.Tensor, partial: bool = False):
        """partial: the consumer is a sandwich norm, which can finish the down projection's split-K sum itself."""
        partial = partial and can_defer(self.down)
        if self.fused:
            return self.down(self.gate_up(h), partial=partial)
        if self.clamped_image is not None and h.shape[0] <= CLAMPED_EPILOGUE_MAX_M:
            act = native.dense_gemm_clamped_glu(h, self.clamped_image, workspace(h.device), self.alpha, self.limit)
            return self.down(act, partial=partial)
        return self.down(native.glu(self.gate_up(h), self.ff, self.mode, self.alpha, self.limit), partial=partial)

    __call__ = forward


class RoutedExperts:
    def __init__(self, weights, prefix: str, experts: int, top: int, shared: bool, router_bias: bool = False,
                 softmax_top: bool = False, weight_on_input: bool = True, grouped_softmax: bool = False, groups: int = 1,
                 keep_groups: int = 1, renorm_eps: float = 0.0):
        """softmax_top: the routing weights are the softmax over the chosen logits (else the sigmoid of each);
        weight_on_input: the weight scales the expert's input (else its output); router_bias: `<prefix>.router.b`.
        grouped_softmax: scores are the softmax over ALL experts; experts are chosen by score + `<prefix>.correction` among the
        `keep_groups` best of `groups` equal groups of neighbours; weights = chosen scores / (their sum + renorm_eps)."""
        self.E, self.k = experts, top
        self.grouped_softmax, self.groups, self.keep_groups, self.renorm_eps = bool(grouped_softmax), int(groups), int(keep_groups), float(renorm_eps)
        if grouped_softmax and (experts % self.groups or not 1 <= self.keep_groups <= self.groups):
            raise ValueError(f"{prefix}: {experts} experts in {groups} groups, {keep_groups} kept")
        self.correction = _f32(weights.get_tensor(f"{prefix}.correction")) if grouped_softmax and weights.has(f"{prefix}.correction") else None
        self.softmax_top, self.weight_on_input = bool(softmax_top), bool(weight_on_input)
        self.router = _f32(weights.get_tensor(f"{prefix}.router"))
        self.router_b = _f32(weights.get_tensor(f"{prefix}.router.b")) if router_bias else None
        pad8 = lambda n: (n + 7) // 8 * 8
        gate = [weights.get_tensor(f"{prefix}.e{e}.gate") for e in range(experts)]
        ff, W = gate[0].shape
        # the grouped GEMM reads 16-byte fragments along its inner dimension: widths that are not multiples of 8 are padded
        # with zero rows / columns once, here (silu(0) * 0 = 0 keeps a padded hidden channel out of the result)
        self.W, self.Wp, self.ff = W, pad8(W), pad8(ff)
        pad = lambda t, rows, cols: torch.nn.functional.pad(t, (0, cols - t.shape[1], 0, rows - t.shape[0]))
        # [E, 2 ff, W] (gate rows, then up rows) and [E, W, ff]
        self.w_gate_up = torch.stack([torch.cat([pad(gate[e], self.ff, self.Wp),
                                                 pad(weights.get_tensor(f"{prefix}.e{e}.up"), self.ff, self.Wp)], 0)
                                      for e in range(experts)]).contiguous()
        self.w_down = torch.stack([pad(weights.get_tensor(f"{prefix}.e{e}.down"), W, self.ff) for e in range(experts)]).contiguous()
        self.shared = GatedUnit(weights, f"{prefix}.shared") if shared else None
        self.shared_gate = _f32(weights.get_tensor(f"{prefix}.shared.sg")).reshape(-1) if shared else None

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        T, W = h.shape
        if self.grouped_softmax:
            idx, weight = native.moe_route_grouped(h, self.router, self.correction, self.k, self.groups, self.keep_groups, self.renorm_eps)
            sg = None
        else:
            idx, weight, sg = native.moe_route(h, self.router, self.shared_gate, self.k, self.router_b, self.softmax_top)
        sorted_, tile_expert, pos, n_tiles = native.moe_align(idx, self.E)
        cap = sorted_.shape[0]
        hp = h if self.Wp == W else torch.nn.functional.pad(h, (0, self.Wp - W))
        act = native.moe_gemm(hp, self.w_gate_up, self.ff, tile_expert, n_tiles, cap, sorted_=sorted_, pair_div=self.k,
                              pair_scale=weight.view(-1) if self.weight_on_input else None, glu_act=True)
        rows = native.moe_gemm(act, self.w_down, W, tile_expert, n_tiles, cap)
        shared = self.shared(h) if self.shared is not None else None
        return native.moe_combine(rows, pos, self.k, T, pair_weight=None if self.weight_on_input else weight.view(-1),
                                  shared=shared, shared_gate=sg)

    __call__ = forward


def _view_for_gemm(x: torch.Tensor) -> torch.Tensor:
    """A column slice of a projection's output as the next projection's input: the weight-streaming kernel takes rows that
    start on 16 bytes; anything else is copied."""
    if x.shape[0] == 1 and x.stride(1) == 1 and x.data_ptr() % 16 == 0:
        return x.as_strided(x.shape, (x.shape[1], 1))  # one row: its stride is free
    if x.stride(1) != 1 or (x.data_ptr() % 16) or (x.stride(0) * x.element_size()) % 16:
        return torch.empty(x.shape, dtype=x.dtype, device=x.device).copy_(x)
    return x


def _widths_ok_for_pages(*widths) -> None:
    for w in widths:
        if w > 256:
            raise NotImplementedError(f"attention widths above 256 per head are not served by the ragged-step kernels (got {w})")


class BlockBiasedAttention:
    """scores = q . k * scale - r1[h] ln(1 + r2[h] (i - j)), visible iff j <= i and floor(i / chunk) == floor(j / chunk)
    (chunk 0: plain causal).  kv_source: the layer whose cached keys and values this one reads (then it has none of its own)."""

    def __init__(self, weights, prefix: str, layer_id: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 eps: float, chunk: int = 0, kv_source: Optional[int] = None, value_norm: bool = True):
        self.layer_id, self.kv_layer = layer_id, layer_id if kv_source is None else int(kv_source)
        self.H, self.G, self.dk, self.dv = heads, kv_heads, dim, vdim
        _widths_ok_for_pages(dim, vdim)
        self.scale, self.eps, self.chunk, self.value_norm = float(scale), float(eps), int(chunk), bool(value_norm)
        self.own_kv = kv_source is None
        names = ["q", "k", "v", "g"] if self.own_kv else ["q", "g"]
        self.proj = load_stacked_linear(weights, [f"{prefix}.{n}" for n in names])
        self.k_col = heads * dim
        self.v_col = self.k_col + kv_heads * dim
        self.g_col = (self.v_col + kv_heads * vdim) if self.own_kv else self.k_col
        has_bias = weights.has(f"{prefix}.r1")
        self.r1 = _f32(weights.get_tensor(f"{prefix}.r1")) if has_bias else None
        self.r2 = _f32(weights.get_tensor(f"{prefix}.r2")) if has_bias else None
        self.o = load_linear(weights, f"{prefix}.o")
        self.defer = can_defer(self.o)

    def forward(self, h: torch.Tensor, position_ids, step):
        proj = self.proj(h)
        cache = step.cache
        k_pool, v_pool = cache.k_pool(self.kv_layer), cache.v_pool(self.kv_layer)
        if self.own_kv:
            native.kv_norm_write(proj, self.k_col, self.v_col, step.slots, k_pool, v_pool, self.G, self.dk, self.dv, self.value_norm,
                                 self.eps)
        gate = proj[:, self.g_col:self.g_col + self.H * self.dv]
        fused = gate.data_ptr() % 8 == 0 and proj.stride(0) % 4 == 0  # the gate rides in the attention kernel's epilogue
        att = native.attn_varlen_ext(proj, k_pool, v_pool, step.block_tables, step.ctx_lens, step.cu_seqlens_q, self.H, self.G,
                                     self.dk, self.dv, self.scale, self.r1, self.r2, self.chunk, gate if fused else None,
                                     max_q_len=step.max_q_len, max_ctx=step.max_ctx, ws=workspace(h.device))
        if not fused:
            native.sigmoid_gate_mul(att, gate, out=att)
        return self.o(att, partial=self.defer)


def rotary_inverse_frequencies(base: float, dims: int, device) -> torch.Tensor:
    """base^(-2i / dims), i < dims / 2, evaluated in float64 and rounded once."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / dims)).to(torch.float32).to(device)


class LatentAttention:
    """c_q = N(W_dq h), q = W_uq c_q = [H][dn | dr];  [c | r] = W_dkv h with c = N(first kv_rank rows);  per head
    k = [W_uk c | rot(r)], v = W_uv c;  causal softmax;  sigmoid output gate.  Only (c, rot(r)) is cached: a page row is
    [c | rot(r)] for ONE kv head, so the score of head h is (W_uk,h^T q_n,h) . c + rot(q_r,h) . rot(r) and its output
    W_uv,h (sum_j p_j c_j) — two batched products per step instead of two per cached token."""

    def __init__(self, weights, prefix: str, layer_id: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 scale: float, eps: float, rot_base: float, rot_dims: int):
        self.layer_id = layer_id
        self.H, self.dn, self.dr, self.dv, self.rk = heads, dim, rot_dim, vdim, kv_rank
        _widths_ok_for_pages(kv_rank + rot_dim, kv_rank)
        self.scale, self.eps, self.rot_dims = float(scale), float(eps), int(rot_dims)
        self.q_rank = weights.get_shape(f"{prefix}.dq")[0]
        self.down = load_stacked_linear(weights, [f"{prefix}.dq", f"{prefix}.dkv", f"{prefix}.g"])
        self.c_col = self.q_rank
        self.g_col = self.q_rank + kv_rank + rot_dim
        self.q_gain = _f32(weights.get_tensor(f"{prefix}.dq.norm"))
        self.c_gain = _f32(weights.get_tensor(f"{prefix}.dkv.norm"))
        self.uq = load_linear(weights, f"{prefix}.uq")
        # [H, dn, kv_rank]: head h's keys are W_uk,h c, so its query meets the latent as W_uk,h^T q_n
        self.uk = weights.get_tensor(f"{prefix}.uk").view(heads, dim, kv_rank).contiguous()
        # [H, kv_rank, dv]: W_uv,h^T, applied to the attention output in latent space
        self.uv_t = weights.get_tensor(f"{prefix}.uv").view(heads, vdim, kv_rank).transpose(1, 2).contiguous()
        self.inv_freq = rotary_inverse_frequencies(rot_base, self.rot_dims, self.uk.device) if self.rot_dims else \
            torch.zeros(1, dtype=torch.float32, device=self.uk.device)
        self.o = load_linear(weights, f"{prefix}.o")
        self.defer = can_defer(self.o)
        # cache geometry of this layer: one kv head
        self.kv_shape = (1, kv_rank + rot_dim, kv_rank)

    def forward(self, h: torch.Tensor, position_ids, step):
        T = h.shape[0]
        H, dn, dr, rk, dv = self.H, self.dn, self.dr, self.rk, self.dv
        down = self.down(h)
        cq = native.rms_norm_rows(down[:, :self.q_rank], self.q_gain, self.eps)
        q = self.uq(cq)
        cache = step.cache
        k_pool, v_pool = cache.k_pool(self.layer_id), cache.v_pool(self.layer_id)
        q_abs = torch.empty((T, H * (rk + dr)), dtype=q.dtype, device=q.device)
        native.latent_kv_write(q, down[:, self.c_col:self.c_col + rk + dr], self.c_gain, self.inv_freq, position_ids, step.slots,
                               q_abs, k_pool, v_pool, H, dn, dr, rk, self.rot_dims, self.eps)
        # the unrotated query parts in latent space: [H, T, dn] x [H, dn, rk] (library batched product)
        qn = q.view(T, H, dn + dr)[:, :, :dn].transpose(0, 1)
        q_abs.view(T, H, rk + dr)[:, :, :rk].copy_(torch.bmm(qn, self.uk).transpose(0, 1))
        lat = native.attn_varlen_ext(q_abs, k_pool, v_pool, step.block_tables, step.ctx_lens, step.cu_seqlens_q, H, 1, rk + dr, rk,
                                     self.scale, max_q_len=step.max_q_len, max_ctx=step.max_ctx, ws=workspace(h.device))
        att = torch.bmm(lat.view(T, H, rk).transpose(0, 1), self.uv_t).transpose(0, 1).reshape(T, H * dv)
        native.sigmoid_gate_mul(att, down[:, self.g_col:self.g_col + H * dv], out=att)
        return self.o(att, partial=self.defer)


class DeltaRuleMixer:
    """Per value head (query / key head h // (H / G)):  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q,
    with q, k, v behind a causal convolution of `taps` taps and SiLU, q and k unit vectors (q * dim^-1/2), beta = sigmoid(W_b h),
    g = exp(-exp(A_log) softplus(W_a2 W_a1 h + dt_bias)) per key channel, and o / rms(o) * gain * sigmoid(W_g2 W_g1 h)."""

    def __init__(self, weights, prefix: str, layer_id: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int,
                 eps: float, unit_eps: float = 1e-6):
        self.layer_id = layer_id
        self.H, self.G, self.dk, self.dv, self.taps = heads, kv_heads, dim, vdim, int(taps)
        self.eps, self.unit_eps = float(eps), float(unit_eps)
        self.C = 2 * kv_heads * dim + heads * vdim
        self.ra = weights.get_shape(f"{prefix}.a1")[0]
        self.rg = weights.get_shape(f"{prefix}.g1")[0]
        # one projection for everything that reads h; the low-rank pairs continue from its columns
        self.proj = load_stacked_linear(weights, [f"{prefix}.{n}" for n in ("q", "k", "v", "a1", "g1", "b")], pad_rows_to=8)
        self.a2 = load_linear(weights, f"{prefix}.a2")
        self.g2 = load_linear(weights, f"{prefix}.g2")
        self.conv_w = torch.cat([_f32(weights.get_tensor(f"{prefix}.{n}.conv")) for n in ("q", "k", "v")], 0).contiguous()
        assert self.conv_w.shape == (self.C, self.taps)
        self.A_log = _f32(weights.get_tensor(f"{prefix}.A_log"))
        self.dt_bias = _f32(weights.get_tensor(f"{prefix}.dt_bias"))
        self.gain = _f32(weights.get_tensor(f"{prefix}.norm"))
        self.o = load_linear(weights, f"{prefix}.o")
        self.defer = can_defer(self.o)
        # what a slot holds for this layer: the heads' matrices in the scan kernel's order, and the convolution's tail
        # (one tap: nothing to remember; a row is kept so that the tensor is not empty)
        self.state_shape = {"matrix": (heads, native.delta_state_floats(dim, vdim)), "memory": (max(self.taps - 1, 1), self.C)}

    def forward(self, h: torch.Tensor, position_ids, step):
        st = step.state
        state, tail = st.state[self.layer_id], st.shift[self.layer_id]
        C, ra, rg = self.C, self.ra, self.rg
        proj = self.proj(h)
        a = self.a2(_view_for_gemm(proj[:, C:C + ra]))
        gate = self.g2(_view_for_gemm(proj[:, C + ra:C + ra + rg]))
        conv = native.short_conv_silu(proj, self.conv_w, tail, step.state_slots, step.cu_seqlens_q, position_ids, C)
        out = native.delta_scan(conv, a, proj[:, C + ra + rg:C + ra + rg + self.H], gate, self.A_log, self.dt_bias, self.gain, state, tail, proj,
                                step.state_slots, step.cu_seqlens_q, position_ids, self.H, self.G, self.dk, self.dv, self.taps,
                                self.eps, self.unit_eps, self.dk ** -0.5)
        return self.o(out, partial=self.defer)


def load_stacked_blocks(weights, names, align: int = 8):
    """Several [out_i, in] weights that read the same input as one GEMM whose every block starts on a multiple of `align`
    output columns (zero rows between them) and whose width is one too: (FastLinear, [first column of each block])."""
    parts, cols, at = [], [], 0
    for n in names:
        w = weights.get_tensor(n)
        cols.append(at)
        pad = -w.shape[0] % align
        parts.append(w)
        if pad:
            parts.append(w.new_zeros((pad, w.shape[1])))
        at += w.shape[0] + pad
    return FastLinear(torch.cat(parts, dim=0).contiguous(), None), cols


class WindowSinkAttention:
    """GQA softmax attention: q, k rotated in interleaved pairs (2i, 2i + 1) over their first rot_dims channels by
    position * rot_base^(-2i / rot_dims); position i sees j <= i iff i - j < window or j < keep_first (window 0: plain causal);
    the denominator of head h also holds exp(sink[h]) (`<prefix>.sink`, optional); head h's output is multiplied by
    sigmoid(W_g h)[h] (`<prefix>.g`, optional).  The mixer reads columns of a projection its owner made (`in_names` are the
    weights to stack, in this order) and writes its heads into the owner's buffer."""

    def __init__(self, weights, prefix: str, layer_id: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int = 0, keep_first: int = 0, rot_base: float = 10000.0, rot_dims: int = 0):
        self.layer_id = layer_id
        self.H, self.G, self.dk, self.dv = heads, kv_heads, dim, vdim
        _widths_ok_for_pages(dim, vdim)
        if heads % kv_heads or rot_dims % 2 or rot_dims > dim:
            raise ValueError(f"{prefix}: {heads} heads on {kv_heads} kv heads, {rot_dims} rotated of {dim} channels")
        self.scale, self.window, self.keep_first = float(scale), int(window), int(keep_first) if window else 0
        self.rot_dims = int(rot_dims)
        self.has_gate = weights.has(f"{prefix}.g")
        self.in_names = [f"{prefix}.{n}" for n in (("q", "k", "v", "g") if self.has_gate else ("q", "k", "v"))]
        self.out_name, self.out_width = f"{prefix}.o", heads * vdim
        self.sink = _f32(weights.get_tensor(f"{prefix}.sink")) if weights.has(f"{prefix}.sink") else None
        dev = weights.device
        self.inv_freq = rotary_inverse_frequencies(rot_base, self.rot_dims, dev) if self.rot_dims else None
        self.kv_shape = (kv_heads, dim, vdim)
        self.state_shape = None

    def run(self, proj: torch.Tensor, cols, position_ids, step, out: torch.Tensor, out_scale: float = 1.0):
        """proj [T, ld] with this mixer's blocks at columns `cols` (one per in_name); out [T, H dv] (a view)."""
        cache = step.cache
        k_pool, v_pool = cache.k_pool(self.layer_id), cache.v_pool(self.layer_id)
        native.rope_rows_kv_write(proj, cols[0], cols[1], cols[2], self.inv_freq, position_ids, step.slots, k_pool, v_pool, self.H,
                                  self.G, self.dk, self.dv, self.rot_dims)
        gate = proj[:, cols[3]:cols[3] + self.H] if self.has_gate else None
        native.attn_varlen_win(proj[:, cols[0]:cols[0] + self.H * self.dk], k_pool, v_pool, step.block_tables, step.ctx_lens,
                               step.cu_seqlens_q, self.H, self.G, self.dk, self.dv, self.scale, window=self.window,
                               keep_first=self.keep_first, sink=self.sink, gate=gate, gate_per_head=True, out_scale=out_scale, out=out,
                               max_q_len=step.max_q_len, max_ctx=step.max_ctx, ws=workspace(proj.device))


class GatedLinearRecurrence:
    """Per head S <- diag(f) S + (1 - f) v^T, o = S^T q with q = silu(W_q h), v = W_v h and the forget gate
    f = l + (1 - l) sigmoid(W_f h + b) bounded below by l (`.lower`), one per head and key channel; o is RMS-normed per head
    with one gain for all heads (`.norm`).  Gates, state and read-out are fp32.  Reads columns of its owner's projection."""

    def __init__(self, weights, prefix: str, layer_id: int, heads: int, dim: int, vdim: int, eps: float):
        self.layer_id = layer_id
        self.H, self.dk, self.dv, self.eps = heads, dim, vdim, float(eps)
        if dim > 256 or vdim > 256:
            raise NotImplementedError(f"the gated linear scan serves heads of up to 256 x 256 (got {dim} x {vdim})")
        self.in_names = [f"{prefix}.{n}" for n in ("q", "f", "v")]
        self.out_name, self.out_width = f"{prefix}.o", heads * vdim
        self.f_bias = _f32(weights.get_tensor(f"{prefix}.f.b")) if weights.has(f"{prefix}.f.b") else None
        self.lower = _f32(weights.get_tensor(f"{prefix}.lower")) if weights.has(f"{prefix}.lower") else None
        self.gain = _f32(weights.get_tensor(f"{prefix}.norm"))
        self.kv_shape = None
        # a slot holds the heads' matrices [H, dk, dv]; nothing else is remembered (a one-float placeholder)
        self.state_shape = {"matrix": (heads, dim, vdim), "memory": (1,)}

    def run(self, proj: torch.Tensor, cols, position_ids, step, out: torch.Tensor, out_scale: float = 1.0):
        native.gated_linear_scan(proj, cols[0], cols[1], cols[2], self.f_bias, self.lower, self.gain, step.state.state[self.layer_id],
                                 step.state_slots, step.cu_seqlens_q, position_ids, self.H, self.dk, self.dv, self.eps, q_act=True,
                                 out_scale=out_scale, out=out, max_q_len=step.max_q_len)


class SideBySideMixers:
    """Mixers that read the same input and whose results are added with fixed weights: y = sum_m scale_m W_o,m mixer_m(h).
    Everything that reads h — the mixers' input projections and whatever else the owner names (`extra_in`: gates of the
    residual, ...) — is ONE stacked GEMM; the mixers write their heads, already scaled, side by side into one buffer, and the
    output projections are ONE GEMM over it (its split-K sum may be left to the residual update behind it)."""

    def __init__(self, weights, mixers, scales, extra_in=()):
        self.mixers, self.scales = list(mixers), [float(s) for s in scales]
        names = [n for m in self.mixers for n in m.in_names] + list(extra_in)
        self.proj, cols = load_stacked_blocks(weights, names, align=8)
        self.cols, at = [], 0
        for m in self.mixers:
            self.cols.append(cols[at:at + len(m.in_names)])
            at += len(m.in_names)
        self.extra_cols = dict(zip(extra_in, cols[at:]))
        # heads side by side, every mixer's block on a multiple of 8 columns; the output weight gets zero columns there
        self.out_cols, parts, at = [], [], 0
        for m in self.mixers:
            w = weights.get_tensor(m.out_name)
            pad = -w.shape[1] % 8
            self.out_cols.append(at)
            parts.append(w)
            if pad:
                parts.append(w.new_zeros((w.shape[0], pad)))
            at += w.shape[1] + pad
        self.out_width = at
        self.padded = any(m.out_width % 8 for m in self.mixers)
        self.o = FastLinear(torch.cat(parts, dim=1).contiguous(), None)
        self.defer = can_defer(self.o)

    def forward(self, h: torch.Tensor, position_ids, step):
        """(y [T, W] or its split-K slabs, proj): proj holds the extra blocks at self.extra_cols[name]."""
        proj = self.proj(h)
        T = h.shape[0]
        alloc = torch.zeros if self.padded else torch.empty
        heads = alloc((T, self.out_width), dtype=h.dtype, device=h.device)
        for m, cols, c0, sc in zip(self.mixers, self.cols, self.out_cols, self.scales):
            m.run(proj, cols, position_ids, step, heads[:, c0:c0 + m.out_width], out_scale=sc)
        return self.o(heads, partial=self.defer), proj


class InputConvolutions:
    """out_s = h + conv_s(h) for the sublayers s that read the same normed input h: per channel,
    conv_s(h)_t = sum_j w_s[:, j] h_(t - taps + 1 + j), zeros before the sequence's start.  The last taps - 1 inputs of a
    sequence wait in `floats` fp32 numbers of its state slot (one tail for all sets: it is the input's)."""

    def __init__(self, weights, names, width: int, taps: int):
        self.taps, self.width = int(taps), int(width)
        self.w = torch.stack([_f32(weights.get_tensor(n)) for n in names]).contiguous()  # [sets, width, taps]
        if self.w.shape[1:] != (self.width, self.taps) or not 1 <= self.taps <= 16:
            raise ValueError(f"{names[0]}: filters {tuple(self.w.shape[1:])} for width {width}, {taps} taps (1 .. 16)")
        self.floats = (self.taps - 1) * self.width

    def forward(self, h: torch.Tensor, tail: Optional[torch.Tensor], position_ids, step, dtype):
        """h [T, width] fp32 or `dtype`; tail: the slots' [*, floats] view -> [sets, T, width] in `dtype`."""
        return native.causal_conv(h, self.w, None, tail, step.state_slots, step.cu_seqlens_q, position_ids, dtype, residual=True,
                                  max_q_len=step.max_q_len)

    __call__ = forward


def _stack_rows_aligned(parts, align: int = 8):
    """Row blocks of one weight as a stacked weight whose blocks start on multiples of `align` output columns."""
    out, cols, at = [], [], 0
    for w in parts:
        cols.append(at)
        out.append(w)
        pad = -w.shape[0] % align
        if pad:
            out.append(w.new_zeros((pad, w.shape[1])))
        at += w.shape[0] + pad
    return torch.cat(out, 0).contiguous(), cols


class SelectiveScanMixer:
    """[x | z] = W_in h;  x <- silu(conv(x) + b) over `taps` taps;  [dt | B | C] = W_x x;  d = softplus(W_dt dt + b_dt);
    S[c, n] <- exp(-d_c exp(A_log[c, n])) S[c, n] + d_c x_c B_n;  y_c = sum_n S[c, n] C_n + D_c x_c;  W_o (y * silu(z)).
    A slot holds S [inner, state] (fp32) and the convolution's last taps - 1 inputs."""

    def __init__(self, weights, prefix: str, inner: int, state: int, dt_rank: int, taps: int):
        self.inner, self.N, self.R, self.taps = int(inner), int(state), int(dt_rank), int(taps)
        if self.N > 128:
            raise NotImplementedError(f"{prefix}: the selective scan keeps up to 128 states per channel (got {self.N})")
        self.in_proj = load_linear(weights, f"{prefix}.in")
        self.conv_w = _f32(weights.get_tensor(f"{prefix}.conv")).reshape(1, self.inner, self.taps).contiguous()
        self.conv_b = _f32(weights.get_tensor(f"{prefix}.conv.b")).reshape(1, self.inner).contiguous()
        wx = weights.get_tensor(f"{prefix}.x")
        R, N = self.R, self.N
        stacked, (self.dt_col, self.b_col, self.c_col) = _stack_rows_aligned([wx[:R], wx[R:R + N], wx[R + N:R + 2 * N]])
        self.x_proj = FastLinear(stacked, None)
        self.dt_proj = load_linear(weights, f"{prefix}.dt")
        self.dt_bias = _f32(weights.get_tensor(f"{prefix}.dt.b"))
        self.A_log = _f32(weights.get_tensor(f"{prefix}.A_log"))
        self.D = _f32(weights.get_tensor(f"{prefix}.D"))
        self.o = load_linear(weights, f"{prefix}.o")
        self.kv_shape = None
        self.state_matrix = (self.inner, self.N)
        self.memory_floats = (self.taps - 1) * self.inner

    def forward(self, h: torch.Tensor, position_ids, step, state: torch.Tensor, tail: Optional[torch.Tensor]):
        """state: the slots' [*, inner, N]; tail: the slots' [*, memory_floats] view."""
        xz = self.in_proj(h)
        x = native.causal_conv(xz[:, :self.inner], self.conv_w, self.conv_b, tail, step.state_slots, step.cu_seqlens_q, position_ids,
                               h.dtype, act=True, max_q_len=step.max_q_len)[0]
        low = self.x_proj(x)
        dt = self.dt_proj(_view_for_gemm(low[:, self.dt_col:self.dt_col + self.R]), out_f32=True)
        y = native.selective_scan(x, dt, self.dt_bias, low, self.b_col, self.c_col, xz[:, self.inner:], self.A_log, self.D, state,
                                  step.state_slots, step.cu_seqlens_q, position_ids, self.N, max_q_len=step.max_q_len)
        return self.o(y, out_f32=True)


class MixedHeadAttention:
    """GQA softmax attention: q, k, v (and the output projection) with biases; q and k rotated in interleaved pairs over their
    first rot_dims channels, then divided by their root mean square per head (no gain); the scaled scores of the H heads are
    mixed by `<prefix>.talk` [H, H] before the softmax; position i sees j <= i with i - j < window (0: all); the heads'
    outputs are multiplied channel by channel by sigmoid(W_g h).  Reads columns of its owner's projection."""

    def __init__(self, weights, prefix: str, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float,
                 window: int = 0, rot_base: float = 10000.0, rot_dims: int = 0):
        self.H, self.G, self.dk, self.dv = heads, kv_heads, dim, vdim
        _widths_ok_for_pages(dim, vdim)
        if heads % kv_heads or rot_dims % 2 or rot_dims > dim or heads * vdim > 4096:
            raise ValueError(f"{prefix}: {heads} heads of {dim} / {vdim} on {kv_heads} kv heads, {rot_dims} rotated channels")
        self.scale, self.eps, self.window, self.rot_dims = float(scale), float(eps), int(window), int(rot_dims)
        self.has_gate = weights.has(f"{prefix}.g")
        self.in_names = [f"{prefix}.{n}" for n in (("q", "k", "v", "g") if self.has_gate else ("q", "k", "v"))]
        self.out_name, self.out_width = f"{prefix}.o", heads * vdim
        self.talk = _f32(weights.get_tensor(f"{prefix}.talk")) if weights.has(f"{prefix}.talk") else \
            torch.eye(heads, dtype=torch.float32, device=weights.device)
        self.inv_freq = rotary_inverse_frequencies(rot_base, self.rot_dims, weights.device) if self.rot_dims else None
        self.kv_shape = (kv_heads, dim, vdim)
        self.state_matrix, self.memory_floats = None, 0

    def run(self, proj: torch.Tensor, cols, position_ids, step, cache_id: int, state=None) -> torch.Tensor:
        cache = step.cache
        k_pool, v_pool = cache.k_pool(cache_id), cache.v_pool(cache_id)
        native.rope_rows_unit_kv_write(proj, cols[0], cols[1], cols[2], self.inv_freq, position_ids, step.slots, k_pool, v_pool,
                                       self.H, self.G, self.dk, self.dv, self.rot_dims, self.eps)
        gate = proj[:, cols[3]:cols[3] + self.H * self.dv] if self.has_gate else None
        return native.attn_mixed_heads(proj[:, cols[0]:cols[0] + self.H * self.dk], k_pool, v_pool, step.block_tables, step.ctx_lens,
                                       step.cu_seqlens_q, self.talk, self.H, self.G, self.dk, self.dv, self.scale, window=self.window,
                                       gate=gate, max_q_len=step.max_q_len, max_ctx=step.max_ctx, ws=workspace(proj.device))


class DecayedLinearAttention:
    """Per head S <- diag(a) S + k v^T, o = S^T q (the new state is read), S fp32 in a state slot.
      decay "head":     a = one constant per head (`head_decay`)
      decay "channel":  a = sigmoid(W_a2 W_a1 h + b)^(1 / tau) per head and key channel (a low-rank pair `.a1`, `.a2`, `.a2.b`)
    act: SiLU on q, k and v;  q_scale: a factor on q;  norm "head": o / rms(o) * gain[dv] per head, "row": the heads of a token
    normed together with gain [H dv];  gate "sigmoid" / "silu": times that of W_g h.  Reads columns of its owner's projection."""

    def __init__(self, weights, prefix: str, heads: int, dim: int, vdim: int, eps: float, decay: str, head_decay=None,
                 tau: float = 1.0, act: bool = False, q_scale: float = 1.0, norm: str = "head", gate: str = "sigmoid"):
        self.H, self.dk, self.dv, self.eps = heads, dim, vdim, float(eps)
        if dim > 256 or vdim > 256:
            raise NotImplementedError(f"{prefix}: the linear scan serves heads of up to 256 x 256 (got {dim} x {vdim})")
        self.channel_decay = {"head": False, "channel": True}[decay]
        self.act, self.q_scale, self.inv_tau = bool(act), float(q_scale), 1.0 / float(tau)
        self.norm_rows = {"head": False, "row": True}[norm]
        self.gate_act = {"sigmoid": 1, "silu": 2}[gate]
        names = ["q", "k", "v", "g"] + (["a1"] if self.channel_decay else [])
        self.in_names = [f"{prefix}.{n}" for n in names]
        self.out_name, self.out_width = f"{prefix}.o", heads * vdim
        self.gain = _f32(weights.get_tensor(f"{prefix}.norm"))
        if self.gain.shape[0] != (heads * vdim if self.norm_rows else vdim):
            raise ValueError(f"{prefix}.norm: {self.gain.shape[0]} gains for a {norm} norm of {heads} x {vdim}")
        self.head_decay = self.a2 = self.a_bias = None
        if self.channel_decay:
            self.rank = weights.get_shape(f"{prefix}.a1")[0]
            self.a2 = load_linear(weights, f"{prefix}.a2")
            self.a_bias = _f32(weights.get_tensor(f"{prefix}.a2.b"))
        else:
            d = torch.tensor([float(x) for x in head_decay], dtype=torch.float32)
            if d.shape[0] != heads:
                raise ValueError(f"{prefix}: {d.shape[0]} decays for {heads} heads")
            self.head_decay = d.to(weights.device)
        self.kv_shape = None
        self.state_matrix, self.memory_floats = (heads, dim, vdim), 0
        # columns the mixer needs behind its owner's projection (the decay's pre-activations)
        self.extra_cols = heads * dim if self.channel_decay else 0

    def run(self, proj: torch.Tensor, cols, position_ids, step, cache_id: int, state: torch.Tensor, extra_col: int = -1) -> torch.Tensor:
        """state: the slots' [*, H, dk, dv]; extra_col: first of this mixer's extra_cols columns of proj (channel decay)."""
        f_col = -1
        if self.channel_decay:
            f_col = extra_col
            self.a2(_view_for_gemm(proj[:, cols[4]:cols[4] + self.rank]), out=proj[:, f_col:f_col + self.H * self.dk])
        gate = proj[:, cols[3]:cols[3] + self.H * self.dv]
        return native.linear_scan(proj, cols[0], cols[1], f_col, cols[2], state, step.state_slots, step.cu_seqlens_q, position_ids,
                                  self.H, self.dk, self.dv, self.eps, self.gain, decay_mode=1 if self.channel_decay else 2,
                                  f_bias=self.a_bias, head_decay=self.head_decay, inv_tau=self.inv_tau, q_act=self.act, k_act=self.act,
                                  v_act=self.act, q_scale=self.q_scale, norm_rows=self.norm_rows, gate=gate, gate_act=self.gate_act,
                                  max_q_len=step.max_q_len)


class StackedInput:
    """Everything that reads the same input as ONE GEMM (blocks on multiples of 8 columns, biases where the names have them,
    `extra` more columns behind the blocks for what a mixer computes from them)."""

    def __init__(self, weights, names, extra: int = 0):
        self.proj, self.cols = load_stacked_blocks(weights, names, align=8)
        self.width = self.proj.out_features
        self.extra_col, self.extra = self.width, int(extra)
        if any(weights.has(n + ".b") for n in names):
            bias = torch.zeros(self.width, dtype=self.proj.weight.dtype, device=self.proj.weight.device)
            for n, c in zip(names, self.cols):
                if weights.has(n + ".b"):
                    b = weights.get_tensor(n + ".b")
                    bias[c:c + b.shape[0]] = b
            self.proj.bias = bias

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        if not self.extra:
            return self.proj(h)
        assert self.proj.bias is None
        buf = torch.empty((h.shape[0], self.width + (self.extra + 7) // 8 * 8), dtype=h.dtype, device=h.device)
        self.proj(h, out=buf[:, :self.width])
        return buf

    __call__ = forward


class NormedPairMixers:
    """Two mixers that read the same input through one stacked projection; each result goes through its own output projection
    (a bias where `<out>.b` exists) and an RMS norm over the model width with a gain of its own; y = c (N(a) wa + N(b) wb)."""

    def __init__(self, weights, left, right, left_gain: str, right_gain: str, eps: float, coef: float = 0.5):
        self.left, self.right, self.eps, self.coef = left, right, float(eps), float(coef)
        self.stack = StackedInput(weights, left.in_names + right.in_names)
        n = len(left.in_names)
        self.cols = (self.stack.cols[:n], self.stack.cols[n:])
        self.o = []
        for m in (left, right):
            lin = load_linear(weights, m.out_name)
            if weights.has(m.out_name + ".b"):
                lin.bias = weights.get_tensor(m.out_name + ".b").contiguous()
            self.o.append(lin)
        self.gains = (_f32(weights.get_tensor(left_gain)), _f32(weights.get_tensor(right_gain)))

    def forward(self, h: torch.Tensor, position_ids, step, cache_id: int, state, defer: bool = False):
        """defer: hand the two projected rows on as (a, (b, gain a, gain b, coef)) for a residual update that norms and
        averages them on the way (native.scaled_residual_norm(pair=)); else the averaged row."""
        proj = self.stack(h)
        a = self.o[0](self.left.run(proj, self.cols[0], position_ids, step, cache_id, state), out_f32=True)
        b = self.o[1](self.right.run(proj, self.cols[1], position_ids, step, cache_id, state), out_f32=True)
        if defer:
            return a, (b, self.gains[0], self.gains[1], self.coef)
        return native.rms_pair_mean(a, self.gains[0], self.coef, b, self.gains[1], self.coef, self.eps, h.dtype)


class SingleMixer:
    """One column-reading mixer behind its stacked projection and in front of its output projection."""

    def __init__(self, weights, mixer):
        self.mixer = mixer
        self.stack = StackedInput(weights, mixer.in_names, extra=getattr(mixer, "extra_cols", 0))
        self.o = load_linear(weights, mixer.out_name)

    def forward(self, h: torch.Tensor, position_ids, step, cache_id: int, state) -> torch.Tensor:
        proj = self.stack(h)
        return self.o(self.mixer.run(proj, self.stack.cols, position_ids, step, cache_id, state, extra_col=self.stack.extra_col), out_f32=True)


class PowerNormMLP:
    """W_down (c1 N(z) + c2 N(z^2) + c3 N(z^3) + c0), z = W_up h, powers element by element, N(u) = u / sqrt(mean(u^2) + eps) over a
    token's feed-forward values; the four numbers are `<prefix>.act` = (c1, c2, c3, c0)."""

    def __init__(self, weights, prefix: str, eps: float):
        self.up = load_linear(weights, f"{prefix}.up")
        self.down = load_linear(weights, f"{prefix}.down")
        self.c1, self.c2, self.c3, self.c0 = weights.get_tensor(f"{prefix}.act").float().tolist()
        self.eps = float(eps)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(native.poly_norm(self.up(h), self.c1, self.c2, self.c3, self.c0, self.eps), out_f32=True)

    __call__ = forward


def _softplus(z: float) -> float:
    import math

    return z if z > 30 else math.log1p(math.exp(z))


class ActivatedMLP:
    """W_down xielu(W_up h);  xielu(z) = ap z^2 + z / 2 for z > 0, an (exp(z) - 1 - z) + z / 2 otherwise, with
    ap = softplus(p), an = 1/2 + softplus(q) from the layer's two learned numbers."""

    def __init__(self, weights, prefix: str):
        self.up = load_linear(weights, f"{prefix}.up")
        self.down = load_linear(weights, f"{prefix}.down")
        p, q = weights.get_tensor(f"{prefix}.act").float().tolist()
        self.ap, self.an = _softplus(p), 0.5 + _softplus(q)

    def forward(self, h: torch.Tensor, partial: bool = False):
        partial = partial and can_defer(self.down)
        if self.up.streams and h.shape[0] <= SKINNY_MAX_M:
            # decode-sized steps: the activation where the weight-streaming GEMM finishes its output
            act = native.dense_gemm_xielu(h, self.up.prepared, workspace(h.device), self.ap, self.an)
        else:
            act = native.xielu(self.up(h), self.ap, self.an)
        return self.down(act, partial=partial)

    __call__ = forward


class TokenSideInput:
    """y = W_proj (gelu_tanh(W_gate x) * e) where e is this layer's slice of a second embedding of the token; the caller
    norms y and adds it to the residual stream."""

    def __init__(self, weights, prefix: str, layer_id: int, table: torch.Tensor, dim: int):
        self.gate = load_linear(weights, f"{prefix}.gate")
        self.proj = load_linear(weights, f"{prefix}.proj")
        self.gain = _f32(weights.get_tensor(f"{prefix}.norm"))
        self.table, self.col0, self.dim = table, layer_id * dim, dim
        self.defer = can_defer(self.proj)

    def forward(self, x_act: torch.Tensor, input_ids: torch.Tensor):
        """x_act: the residual stream rounded to the activation dtype."""
        if self.gate.streams and x_act.shape[0] <= SKINNY_MAX_M:
            # decode-sized steps: activation and lookup where the weight-streaming GEMM finishes the gate projection
            g = native.dense_gemm_gelu_lookup(x_act, self.gate.prepared, workspace(x_act.device), input_ids, self.table, self.col0)
        else:
            g = native.gelu_gated_lookup(self.gate(x_act), input_ids, self.table, self.col0)
        return self.proj(g, partial=self.defer)

    __call__ = forward
