"""GPU: the Mananex family on the kernels (FlashCausalLM + utils/mixers.py + csrc/residual_f32, attn_varlen, gated_linear_scan,
moe) against the plain float64 restatement in oracle/mananex_ref.py, on small seeded checkpoints of their own sizes.

float32 serving is compared tightly (it differs from the oracle by accumulation order only); bfloat16 serving against a
bound that scales with bf16 rounding.  Schedules (whole prompts, token by token, portions down to two tokens, mixed batches,
pages and slots that change hands) are compared with the oracle run whole, where only rounding may differ."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import mananex_ref as ref
from oracle import mananex_tiny as tiny

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-4, torch.bfloat16: 0.15}
DTYPES = [torch.float32, torch.bfloat16]


def build_lm(cfg, tensors, dtype, pages=64, slots=4, tokenizer=None):
    from tgis_amd.inference_engine.synthetic import InferenceEngine
    from tgis_amd.models.custom_modeling.flash_mananex_modeling import MananexConfig
    from tgis_amd.models.flash_causal_lm import FlashCausalLM

    eng = InferenceEngine({k: v.clone() for k, v in tensors.items()}, MananexConfig(**cfg), dtype, None, tokenizer=tokenizer)
    return FlashCausalLM("synthetic", None, "synthetic", dtype, None, engine=eng, kv_cache_pages=pages, state_slots=slots)


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row: rms of the centred difference over the rms of the centred reference row."""
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def rel_err(got, want) -> float:
    return float(row_errors(got, want).max())


def close(got, want, dtype) -> bool:
    return rel_err(got, want) <= TOL[dtype]


_PROMPTS = {}


def rand_tokens(n, cfg, tensors, seed):
    """Random tokens for which no router of the checkpoint is near a tie and no read-out of a recurrence cancels before its
    norm (drawn again until so): a bfloat16 run then differs from the float64 restatement by rounding, not by a token that
    went to other experts or a division by almost nothing."""
    key = (json.dumps(cfg, sort_keys=True), n, seed)
    if key not in _PROMPTS:
        _PROMPTS[key] = ref.clear_cut_tokens(cfg, tensors, n, seed)
    return _PROMPTS[key]


@pytest.fixture(scope="module")
def std():
    cfg = tiny.make_config(tiny.standard_layers())
    return cfg, tiny.make_tensors(cfg, seed=3)


# ---- whole model -----------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [75, 300])
def test_whole_prompt_matches_oracle_layer_by_layer(gpu_device, std, dtype, n):
    """75 tokens: the decode-sized GEMM path (split-K sums finished by the residual update behind them); 300: the library
    GEMMs.  Both are longer than every window of the configuration."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(n, cfg, tensors, 1)
    want_trace = []
    want = ref.forward(cfg, tensors, toks, want_trace)
    with lm.context_manager():
        seq = lm.open_sequence()
        trace = []
        got = lm.step_sequences([(seq, toks)], None, residual_trace=trace)
    assert len(trace) == len(want_trace)
    for i, (g, w) in enumerate(zip(trace, want_trace)):
        assert close(g, w, dtype), f"layer {i}"
    assert close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_by_token_and_portions_equal_whole(gpu_device, std, dtype):
    """Prefill against decoding one token at a time, and portions of several sizes down to two tokens, some of them ending or
    starting on a page border (32) or where a window (24, 33, 40) begins to cut."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(101, cfg, tensors, 2)
    want = ref.forward(cfg, tensors, toks)
    with lm.context_manager():
        for cuts in ([1] * 101, [2] * 50 + [1], [31, 1, 2, 30, 3, 29, 5], [32, 32, 32, 5], [24, 9, 7, 61], [23, 2, 15, 1, 60], [7, 57, 37]):
            assert sum(cuts) == 101
            seq = lm.open_sequence()
            at, outs = 0, []
            for n in cuts:
                outs.append(lm.step_sequences([(seq, toks[at:at + n])], None))
                at += n
            assert close(torch.cat(outs), want, dtype), cuts
            lm.close_sequence(seq)


@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batches_reuse_pages_and_slots(gpu_device, std, dtype):
    """Up to four live requests of unequal length, portions of some beside single tokens of others, in a pool that is too
    small to hold all requests at once: pages and slots go back and are handed out again, to other requests."""
    cfg, tensors = std
    lens = [70, 33, 95, 5, 64, 40, 1]
    prompts = [rand_tokens(n, cfg, tensors, 10 + i) for i, n in enumerate(lens)]
    want = [ref.forward(cfg, tensors, p) for p in prompts]
    lm = build_lm(cfg, tensors, dtype, pages=9, slots=4)  # 9 pages = 288 tokens < sum(lens)
    rng = np.random.default_rng(0)
    got = [[] for _ in prompts]
    done = [0] * len(prompts)
    live, waiting = {}, list(range(len(prompts)))
    with lm.context_manager():
        while waiting or live:
            while waiting and len(live) < 4:
                i = waiting[0]
                if sum((lens[j] + 31) // 32 for j in live) + (lens[i] + 31) // 32 > 9:
                    break
                live[waiting.pop(0)] = lm.open_sequence()
            entries, who = [], []
            for i, seq in live.items():
                left = lens[i] - done[i]
                n = 1 if (left == 1 or rng.random() < 0.4) else int(rng.integers(2, min(left, 40) + 1))
                entries.append((seq, prompts[i][done[i]:done[i] + n]))
                who.append((i, n))
            logits = lm.step_sequences(entries, None)
            at = 0
            for i, n in who:
                got[i].append(logits[at:at + n])
                at += n
                done[i] += n
                if done[i] == lens[i]:
                    lm.close_sequence(live.pop(i))
    assert lm.kv_cache.free_pages == 9 and lm.state_cache.free_slots == 4
    for i in range(len(prompts)):
        assert close(torch.cat(got[i]), want[i], dtype), i


def test_stale_slot_and_pages_do_not_leak(gpu_device, std):
    """A request that takes over a slot and pages still holding another request's state and keys computes what it computes in
    a fresh pool; also its first tokens (position 0: zero state)."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, torch.float32, pages=4, slots=1)
    a, b = rand_tokens(120, cfg, tensors, 5), rand_tokens(50, cfg, tensors, 6)
    with lm.context_manager():
        s = lm.open_sequence()
        lm.step_sequences([(s, a)], None)
        lm.close_sequence(s)
        s = lm.open_sequence()
        got = torch.cat([lm.step_sequences([(s, b[:1])], None), lm.step_sequences([(s, b[1:3])], None),
                         lm.step_sequences([(s, b[3:])], None)])
    assert rel_err(got, ref.forward(cfg, tensors, b)) <= TOL[torch.float32]


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(gpu_device, std, dtype):
    """200 decoded tokens: every window passes over decoded tokens, the kept first positions stay."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(40 + 200, cfg, tensors, 8)
    want = ref.forward(cfg, tensors, toks)
    with lm.context_manager():
        s = lm.open_sequence()
        outs = [lm.step_sequences([(s, toks[:40])], None)]
        for t in toks[40:]:
            outs.append(lm.step_sequences([(s, [t])], None))
    assert close(torch.cat(outs), want, dtype)


OTHER_SHAPES = {
    # odd widths everywhere (the general attention kernel, library GEMMs, padded experts), no rotation / all channels rotated,
    # more kept positions than the window is wide, a window of one, every expert chosen
    "odd": dict(layers=[tiny.layer(left=tiny.attention_part(heads=3, kv_heads=1, dim=12, vdim=20, scale=0.3, window=5, keep_first=9, rot_dims=0),
                                   right=tiny.recurrent_part(heads=2, dim=20, vdim=12), mlp=tiny.moe_mlp(experts=3, top=3, ff=30)),
                        tiny.layer(left=tiny.attention_part(heads=3, kv_heads=3, dim=10, vdim=6, scale=0.4, window=1, keep_first=0, rot_dims=10),
                                   right=tiny.recurrent_part(heads=3, dim=5, vdim=7), left_scale=1.0, right_scale=1.0, mlp=tiny.dense_mlp(50)),
                        tiny.layer(left=tiny.attention_part(heads=2, kv_heads=2, dim=14, vdim=14, scale=0.3, window=70, keep_first=2, rot_dims=6),
                                   right=tiny.recurrent_part(heads=1, dim=3, vdim=33), mlp=None)],
                width=36, vocab=50),
    # matrix-core shapes: wide heads, MQA, a window of two pages with kept positions beyond the first page, wide recurrent heads
    "wide": dict(layers=[tiny.layer(left=tiny.attention_part(heads=8, kv_heads=1, dim=128, vdim=128, scale=0.09, window=64, keep_first=40, rot_dims=64),
                                    right=tiny.recurrent_part(heads=2, dim=128, vdim=64), mlp=tiny.moe_mlp(experts=8, top=2, ff=64)),
                         tiny.layer(left=tiny.attention_part(heads=4, kv_heads=2, dim=64, vdim=96, scale=0.12, window=32, keep_first=1, rot_dims=32),
                                    right=tiny.recurrent_part(heads=1, dim=256, vdim=128), mlp=tiny.dense_mlp(256)),
                         tiny.layer(left=tiny.attention_part(heads=2, kv_heads=2, dim=256, vdim=64, scale=0.06, window=50, keep_first=33, rot_dims=2),
                                    right=tiny.recurrent_part(heads=4, dim=64, vdim=256), mlp=None)],
                 width=128, vocab=120),
    # one layer, every count equal to one
    "ones": dict(layers=[tiny.layer(left=tiny.attention_part(heads=1, kv_heads=1, dim=16, vdim=32, window=7, keep_first=1, rot_dims=2),
                                    right=tiny.recurrent_part(heads=1, dim=8, vdim=8), mlp=tiny.moe_mlp(experts=1, top=1, ff=16))],
                 width=32, vocab=40),
    "plain": dict(layers=[tiny.layer(left=tiny.attention_part(window=None, rot_dims=0), mlp=None)], width=32, vocab=40),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(OTHER_SHAPES))
def test_other_sizes_and_layer_orders(gpu_device, dtype, shape):
    """Whole, then in portions with single tokens, for configurations that share no size with the standard one."""
    cfg = tiny.make_config(**OTHER_SHAPES[shape])
    tensors = tiny.make_tensors(cfg, seed=21)
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(90, cfg, tensors, 4)
    want = ref.forward(cfg, tensors, toks)
    with lm.context_manager():
        for cuts in ([90], [33, 1, 1, 2, 30, 23]):
            seq = lm.open_sequence()
            at, outs = 0, []
            for n in cuts:
                outs.append(lm.step_sequences([(seq, toks[at:at + n])], None))
                at += n
            assert close(torch.cat(outs), want, dtype), cuts
            lm.close_sequence(seq)


# ---- attention: keys that must or must not be seen -------------------------------------------------------------------------
def _planted(dtype, key_pos, n_ctx, q_chunks, window, keep, H, G, dk, dv, impl=0):
    """q of the LAST token and k of token `key_pos` are made parallel and large, v of that token is a marker: the last
    token's output is the marker iff the kernel sees that key.  Returns (output of the last token, marker per head)."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(key_pos * 1000 + n_ctx)
    qkv = torch.randn(n_ctx, (H + G) * dk + G * dv, generator=g) * 0.1
    direction = torch.nn.functional.normalize(torch.randn(dk, generator=g), dim=0) * 6
    for h in range(H):
        qkv[n_ctx - 1, h * dk:(h + 1) * dk] = direction
    for gg in range(G):
        qkv[key_pos, (H + gg) * dk:(H + gg + 1) * dk] = direction
    marker = torch.arange(1, G * dv + 1, dtype=torch.float32) * 0.25 + 50
    qkv[key_pos, (H + G) * dk:] = marker
    cache = PagedKVCache(1, G, dk, 40, dtype, dev, layer_shapes=[(G, dk, dv)])
    pages = cache.alloc((n_ctx + PAGE - 1) // PAGE)
    np.random.default_rng(1).shuffle(pages)  # pages of a sequence are scattered over the pool
    bt = torch.tensor([pages], dtype=torch.int32, device=dev)
    sink = torch.full((H,), -2.0, device=dev)
    out_last, at = None, 0
    for n in q_chunks:
        pos = torch.arange(at, at + n)
        slots = (torch.tensor(pages, dtype=torch.int64)[pos // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev)
        x = qkv[at:at + n].to(dtype).to(dev).contiguous()
        native.rope_rows_kv_write(x, 0, H * dk, (H + G) * dk, None, pos.to(torch.int32).to(dev), slots, cache.k_pool(0), cache.v_pool(0),
                                  H, G, dk, dv, 0)
        ctx = torch.tensor([at + n], dtype=torch.int32, device=dev)
        cu = torch.tensor([0, n], dtype=torch.int32, device=dev)
        o = native.attn_varlen_win(x, cache.k_pool(0), cache.v_pool(0), bt, ctx, cu, H, G, dk, dv, 1.0, window=window, keep_first=keep,
                                   sink=sink, max_q_len=n, max_ctx=at + n, impl=impl)
        out_last = o[-1]
        at += n
    torch.cuda.synchronize()
    return out_last.float().cpu(), marker.view(G, dv).repeat_interleave(H // G, 0).reshape(-1)


# (H, G, dk, dv): the general kernel (odd widths) and the matrix-core kernel's shapes under bf16 (narrow: staged; wide: direct)
GEOMETRIES = [(4, 2, 12, 8), (8, 2, 64, 64), (4, 4, 128, 64), (8, 1, 32, 96)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", GEOMETRIES)
@pytest.mark.parametrize("window,keep", [(0, 0), (224, 6), (96, 40), (50, 0), (33, 64), (1, 1)])
def test_attention_sees_its_window_and_the_kept_first_positions(gpu_device, dtype, geom, window, keep):
    """700 tokens; the query is the last one (position 699).  Keys inside its window — its first position, page borders, the
    query's neighbour — and the kept first positions must be found; the key just before the window, the first position that is
    not kept, far keys in between must not (without a window all are found).  In a prompt run whole, cut into portions (one of
    two tokens), and with the last token decoded alone."""
    n = 700
    start = n - window if window else 0
    inside = {p for p in (start, start + 1, n - 2, n - 1, start + 31, start + 32, 671, 672) if start <= p < n}
    inside |= set(range(0, keep, max(1, keep // 3))) | ({keep - 1} if keep else set()) | ({33, 255, 256} if not window else set())
    outside = set() if not window else {p for p in (keep, keep + 1, start - 1, start - 2, start - 33, 300, 31, 32, 63, 64) if keep <= p < start}
    for chunks in ([n], [300, 2, 397, 1], [n - 1, 1]):
        for key_pos in sorted(inside):
            got, want = _planted(dtype, key_pos, n, chunks, window, keep, *geom)
            assert torch.allclose(got, want, atol=0.3 if dtype == torch.bfloat16 else 1e-2, rtol=0.01), (chunks, key_pos, got[:3], want[:3])
        for key_pos in sorted(outside):
            got, _ = _planted(dtype, key_pos, n, chunks, window, keep, *geom)
            assert float(got.abs().max()) < 5.0, (chunks, key_pos, got[:3])


def _plain_window_attention(q, k, v, scale, H, G, window, keep, sink):
    n_q, n = q.shape[0], k.shape[0]
    out = torch.zeros(n_q, H, v.shape[2], dtype=torch.float64)
    ok = ref.visible(torch.arange(n_q) + n - n_q, n, window, keep)
    for h in range(H):
        s = ((q[:, h] @ k[:, h // (H // G)].T) * scale).masked_fill(~ok, float("-inf"))
        w = ref.sink_softmax(s, sink[h]) if sink is not None else torch.softmax(s, -1)
        out[:, h] = w @ v[:, h // (H // G)]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", GEOMETRIES + [(16, 1, 64, 128), (2, 2, 256, 256), (34, 2, 32, 32), (3, 1, 48, 72)])
@pytest.mark.parametrize("window,keep", [(0, 0), (77, 5), (300, 70)])
def test_attention_ragged_batch_against_plain_softmax(gpu_device, dtype, geom, window, keep):
    """A step of unequal sequences — whole prompts, a portion that continues a long context, single decoded tokens, one of
    them behind 3000 cached keys — through both kernels (where the matrix-core one applies) against plain softmax with the
    window, the kept positions, the sink, the per-head gate and the output factor; the output lands in a wider buffer."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache

    H, G, dk, dv = geom
    dev = torch.device("cuda:0")
    cached = [0, 200, 3000, 31, 0, 64]
    new = [70, 45, 1, 1, 1, 33]
    g = torch.Generator().manual_seed(H * 1000 + dk)
    cache = PagedKVCache(1, G, dk, 130, dtype, dev, layer_shapes=[(G, dk, dv)])
    sink = torch.randn(H, generator=g) + 1.0
    kcol, vcol = H * dk, (H + G) * dk
    full, pages = [], []

    def write(x, pg, lo, hi):
        pos = torch.arange(lo, hi)
        slots = (torch.tensor(pg)[pos // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev)
        native.rope_rows_kv_write(x, 0, kcol, vcol, None, pos.to(torch.int32).to(dev), slots, cache.k_pool(0), cache.v_pool(0), H, G, dk, dv, 0)

    for c, n in zip(cached, new):
        x = (torch.randn(c + n, (H + G) * dk + G * dv, generator=g) * (2.0 / dk ** 0.25)).to(dtype)
        pg = cache.alloc((c + n + PAGE - 1) // PAGE)
        if c:  # what earlier steps left in the cache (c >= 512 goes through the transposing value writer)
            write(x[:c].to(dev).contiguous(), pg, 0, c)
        full.append(x)
        pages.append(pg)
    step = torch.cat([x[c:] for x, c in zip(full, cached)]).to(dev).contiguous()
    at = 0
    for x, pg, c, n in zip(full, pages, cached, new):
        write(step[at:at + n], pg, c, c + n)
        at += n
    bt = torch.zeros(len(pages), max(len(p) for p in pages), dtype=torch.int32)
    for i, p in enumerate(pages):
        bt[i, :len(p)] = torch.tensor(p)
    ctx = torch.tensor([c + n for c, n in zip(cached, new)], dtype=torch.int32, device=dev)
    cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32, device=dev)
    want = []
    for x, c, n in zip(full, cached, new):
        xd = x.double()
        want.append(_plain_window_attention(xd[c:, :kcol].view(n, H, dk), xd[:, kcol:vcol].view(c + n, G, dk), xd[:, vcol:].view(c + n, G, dv),
                                            0.5, H, G, window, keep, sink.double()))
    want = torch.cat(want)
    gate = torch.randn(want.shape[0], H + 3, generator=g).to(dtype)
    want_gated = (want * torch.sigmoid(gate[:, 1:H + 1].double())[:, :, None] * 1.7).reshape(want.shape[0], -1)
    want = want.reshape(want.shape[0], -1)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    impls = [1] + ([2] if dtype == torch.bfloat16 and dk % 16 == 0 and dv % 32 == 0 else [])
    gd = gate.to(dev)
    for impl in impls:
        got = native.attn_varlen_win(step, cache.k_pool(0), cache.v_pool(0), bt.to(dev), ctx, cu, H, G, dk, dv, 0.5, window=window,
                                     keep_first=keep, sink=sink.to(dev), max_q_len=max(new), max_ctx=3001, impl=impl)
        assert float((got.double().cpu() - want).abs().max() / want.abs().max()) <= tol, impl
        wide = torch.zeros(want.shape[0], H * dv + 16, dtype=dtype, device=dev)
        native.attn_varlen_win(step, cache.k_pool(0), cache.v_pool(0), bt.to(dev), ctx, cu, H, G, dk, dv, 0.5, window=window,
                               keep_first=keep, sink=sink.to(dev), gate=gd[:, 1:H + 1], gate_per_head=True, out_scale=1.7,
                               out=wide[:, 8:8 + H * dv], max_q_len=max(new), max_ctx=3001, impl=impl)
        assert float((wide[:, 8:8 + H * dv].double().cpu() - want_gated).abs().max() / want_gated.abs().max()) <= tol, ("gated", impl)
        assert float(wide[:, :8].abs().max()) == 0 and float(wide[:, 8 + H * dv:].abs().max()) == 0
    if 2 in impls:  # decode-only steps take the key-split form of the matrix-core kernel
        sel = [i for i, n in enumerate(new) if n == 1]
        rows = [int(cu[i]) for i in sel]
        args = (step[rows].contiguous(), cache.k_pool(0), cache.v_pool(0), bt[sel].contiguous().to(dev), ctx[sel].contiguous(),
                torch.arange(len(sel) + 1, dtype=torch.int32, device=dev), H, G, dk, dv, 0.5)
        kw = dict(window=window, keep_first=keep, sink=sink.to(dev), gate=gd[rows][:, 1:H + 1], gate_per_head=True, out_scale=1.7,
                  max_q_len=1, max_ctx=3001, impl=2)
        got = native.attn_varlen_win(*args, **kw)
        assert float((got.double().cpu() - want_gated[rows]).abs().max() / want_gated.abs().max()) <= tol
        # with scratch memory the pages of these few sequences are dealt to several workgroups and combined afterwards
        ws = native.Workspace(8 << 20, dev)
        got2 = native.attn_varlen_win(*args, ws=ws, **kw)
        assert float((got2.double().cpu() - want_gated[rows]).abs().max() / want_gated.abs().max()) <= tol, "key splits"
        assert torch.all(ws.buf[:4096] == 0)  # the GEMMs' arrival counters are not scratch


def test_sink_takes_its_share(gpu_device):
    """One key, score 0: the weight of the value is 1 / (1 + exp(sink)); a sink far below the scores changes nothing."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PagedKVCache

    dev = torch.device("cuda:0")
    H, dk, dv = 2, 16, 32
    for dtype in DTYPES:
        cache = PagedKVCache(1, H, dk, 2, dtype, dev, layer_shapes=[(H, dk, dv)])
        x = torch.zeros(1, 2 * H * dk + H * dv, dtype=dtype, device=dev)
        x[:, 2 * H * dk:] = 1.0
        z = torch.zeros(1, dtype=torch.int32, device=dev)
        native.rope_rows_kv_write(x, 0, H * dk, 2 * H * dk, None, z, z, cache.k_pool(0), cache.v_pool(0), H, H, dk, dv, 0)
        sink = torch.tensor([1.0, -40.0], device=dev)
        o = native.attn_varlen_win(x, cache.k_pool(0), cache.v_pool(0), torch.zeros(1, 1, dtype=torch.int32, device=dev),
                                   torch.ones(1, dtype=torch.int32, device=dev), torch.tensor([0, 1], dtype=torch.int32, device=dev),
                                   H, H, dk, dv, 1.0, sink=sink).float().cpu().view(H, dv)
        assert torch.allclose(o[0], torch.full((dv,), 1 / (1 + np.e)), atol=5e-3) and torch.allclose(o[1], torch.ones(dv), atol=5e-3)


# ---- mechanisms alone ------------------------------------------------------------------------------------------------------
def _dict_weights(tensors, dtype):
    from tgis_amd.utils.dist import FakeGroup
    from tgis_amd.utils.weights import DictWeights

    return DictWeights(tensors, device=torch.device("cuda:0"), dtype=dtype, process_group=FakeGroup(0, 1))


def _f64(tensors, prefix):
    return {k[len(prefix):]: v.double() for k, v in tensors.items() if k.startswith(prefix)}


def _kv_step(cache, pages, at, m, state=None, slot=None):
    from tgis_amd.models.custom_modeling.flash_llama_modeling import KVArgs
    from tgis_amd.utils.kv_cache import PAGE

    dev = torch.device("cuda:0")
    pos = torch.arange(at, at + m)
    return KVArgs(cache=cache, block_tables=torch.tensor([pages], dtype=torch.int32, device=dev) if pages else None,
                  ctx_lens=torch.tensor([at + m], dtype=torch.int32, device=dev),
                  slots=(torch.tensor(pages)[pos // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev) if pages else None,
                  max_q_len=m, max_ctx=at + m, cu_seqlens_q=torch.tensor([0, m], dtype=torch.int32, device=dev), state=state,
                  state_slots=torch.tensor([slot], dtype=torch.int32, device=dev) if slot is not None else None), pos.to(torch.int32).to(dev)


@pytest.mark.parametrize("dtype", DTYPES)
def test_parallel_residual_update(gpu_device, dtype):
    """v = x + sigmoid(ga + ba) a + sigmoid(gb + bb) b; the mix over depth; the next norm — with tensors, without a second
    sublayer, without a mix, from split-K slabs with a bias."""
    from tgis_amd import native
    from tgis_amd.utils.layers import FastLinear

    g = torch.Generator().manual_seed(0)
    sig = torch.sigmoid
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=1e-2)
    for E in (8, 36, 257, 1024):
        rows, depth = 5, 3
        r = lambda *s: torch.randn(*s, generator=g)
        hist = r(depth + 2, rows, E)
        x = r(rows, E)
        a, b = (r(rows, E) * 2).to(dtype), (r(rows, E) * 2).to(dtype)
        gates = r(rows, 2 * E + 8).to(dtype)  # the gates are columns of a wider projection
        ba, bb = r(E).to(dtype), r(E).to(dtype)
        mix, w = r(depth + 1), r(E) * 0.1
        v = x.double() + sig(gates[:, :E].double() + ba.double()) * a.double() + sig(gates[:, E + 8:].double() + bb.double()) * b.double()
        want_x = (hist[:depth].double() * mix[:depth].double()[:, None, None]).sum(0) + mix[depth].double() * v
        hd, xo, gd = hist.cuda(), torch.empty(rows, E, device="cuda"), gates.cuda()
        y = native.parallel_residual_f32(x.cuda(), a.cuda(), gd[:, :E], ba.cuda(), b.cuda(), gd[:, E + 8:], bb.cuda(), dtype, hd, depth,
                                         mix.cuda(), xo, w.cuda(), 1e-3, dtype, pre_add=1.0)
        assert torch.allclose(hd[depth].cpu().double(), v, atol=1e-5, rtol=1e-5) and torch.equal(hd[depth + 1].cpu(), hist[depth + 1])
        assert torch.allclose(xo.cpu().double(), want_x, atol=1e-5, rtol=1e-5)
        assert torch.allclose(y.cpu().double(), ref.offset_norm(want_x, w.double(), 1e-3), **tol)
        # one sublayer, no gate bias, no mix, in place, no norm
        xd = x.cuda()
        assert native.parallel_residual_f32(xd, a.cuda(), gd[:, :E], None, None, None, None, dtype, None, 0, None, xd, None, 1e-3, dtype) is None
        assert torch.allclose(xd.cpu().double(), x.double() + sig(gates[:, :E].double()) * a.double(), atol=1e-5, rtol=1e-5)
    if dtype == torch.bfloat16:
        for M, K, N in ((1, 512, 256), (33, 2048, 512)):
            wt = (torch.randn(N, K, generator=g) * K ** -0.5).to(dtype).cuda()
            bias = torch.randn(N, generator=g).to(dtype).cuda()
            act = torch.randn(M, K, generator=g).to(dtype).cuda()
            x = torch.randn(M, N, generator=g).cuda()
            gates = torch.randn(M, N, generator=g).to(dtype).cuda()
            hist = torch.randn(2, M, N, generator=g).cuda()
            mix, wn = torch.tensor([0.3, 0.8]).cuda(), torch.randn(N, generator=g).cuda()
            part = FastLinear(wt, bias)(act, partial=True)
            assert isinstance(part, native.Partial) and part.bias is not None
            other = torch.randn(M, N, generator=g).to(dtype).cuda()
            v = x.double().cpu() + sig(gates.double().cpu()) * (act.double().cpu() @ wt.double().cpu().T + bias.double().cpu()) + other.double().cpu()
            want_x = 0.3 * hist[0].double().cpu() + 0.8 * v
            xo = torch.empty_like(x)
            y = native.parallel_residual_f32(x, part, gates, None, other, None, None, dtype, hist, 1, mix, xo, wn, 1e-5, torch.float32)
            assert torch.allclose(xo.double().cpu(), want_x, atol=3e-3, rtol=1e-3)
            assert torch.allclose(y.double().cpu(), ref.rms_unit(want_x, 1e-5) * wn.double().cpu(), atol=3e-3, rtol=1e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotation_and_cache_write(gpu_device, dtype):
    """q in place and k in its page rotated over the first channels only (none, some, all; an odd width), v in its page; a short
    step (values from the same launch) and a long one (the transposing writer)."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache
    from tgis_amd.utils.mixers import rotary_inverse_frequencies

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(1)
    for (H, G, dk, dv, rd), T in (((4, 2, 32, 16, 8), 40), ((3, 3, 11, 7, 10), 40), ((2, 1, 16, 64, 16), 600), ((2, 2, 8, 8, 0), 5)):
        cache = PagedKVCache(1, G, dk, 24, dtype, dev, layer_shapes=[(G, dk, dv)])
        pages = cache.alloc((1000 + T + PAGE - 1) // PAGE - 1000 // PAGE)
        pos = torch.arange(1000, 1000 + T)
        rel = pos - 1000 // PAGE * PAGE
        slots = (torch.tensor(pages)[rel // PAGE] * PAGE + rel % PAGE).to(torch.int32).to(dev)
        x = torch.randn(T, 8 + (H + G) * dk + G * dv, generator=g).to(dtype)
        xd = x.to(dev).clone()
        inv = rotary_inverse_frequencies(777.0, rd, dev) if rd else None
        native.rope_rows_kv_write(xd, 8, 8 + H * dk, 8 + (H + G) * dk, inv, pos.to(torch.int32).to(dev), slots, cache.k_pool(0), cache.v_pool(0),
                                  H, G, dk, dv, rd)
        q_want = ref.rotate_pairs(x[:, 8:8 + H * dk].double().view(T, H, dk), pos, 777.0, rd)
        k_want = ref.rotate_pairs(x[:, 8 + H * dk:8 + (H + G) * dk].double().view(T, G, dk), pos, 777.0, rd)
        # positions 1000 .. 1600: an angle of that size carries 1e-4 of fp32 rounding
        tol = dict(atol=1e-3, rtol=1e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=1e-2)
        assert torch.allclose(xd[:, 8:8 + H * dk].cpu().double().view(T, H, dk), q_want, **tol)
        assert torch.equal(xd[:, :8].cpu(), x[:, :8]) and torch.equal(xd[:, 8 + H * dk:].cpu(), x[:, 8 + H * dk:])
        kp = cache.k_pool(0).view(-1, G, PAGE, dk)[slots.long() // PAGE, :, slots.long() % PAGE]  # [T, G, dk]
        vp = cache.v_pool(0).view(-1, G, dv, PAGE)[slots.long() // PAGE, :, :, slots.long() % PAGE]  # [T, G, dv]
        assert torch.allclose(kp.cpu().double(), k_want, **tol)
        assert torch.equal(vp.cpu().reshape(T, G * dv), x[:, 8 + (H + G) * dk:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim", [(3, 16, 32), (2, 40, 64), (1, 3, 33), (2, 20, 12), (2, 128, 64), (1, 256, 128), (2, 64, 256), (3, 24, 96)])
def test_gated_linear_recurrence_and_its_state(gpu_device, dtype, heads, dim, vdim):
    """The recurrence through a slot that held another sequence, whole and in portions down to one token; the state the slot
    holds afterwards; the output scaled and written into a wider buffer.  Value heads wider than 64 are dealt to several
    workgroups in the long steps (96: the last one holds half its columns), decode-sized steps give a lane two columns."""
    from tgis_amd import native
    from tgis_amd.utils.state_cache import RecurrentStateCache

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(heads * 100 + dim)
    T = 75
    C = heads * (2 * dim + vdim)
    proj = (torch.randn(T, C + 8, generator=g) * 1.5).to(dtype)
    fb, lower, gain = torch.randn(heads * dim, generator=g), torch.rand(heads * dim, generator=g) * 0.95, 1 + 0.2 * torch.randn(vdim, generator=g)
    pd = proj.double()
    q = ref.silu(pd[:, 8:8 + heads * dim]).view(T, heads, dim)
    f = ref.forget_gate(pd[:, 8 + heads * dim:8 + 2 * heads * dim] + fb.double(), lower.double()).view(T, heads, dim)
    v = pd[:, 8 + 2 * heads * dim:].view(T, heads, vdim)
    o, S = ref.gated_linear_recurrence(q, f, v, torch.zeros(heads, dim, vdim, dtype=torch.float64))
    want = (ref.rms_unit(o, 1e-4) * gain.double() * 0.7).reshape(T, heads * vdim)
    st = RecurrentStateCache([{"matrix": (heads, dim, vdim), "memory": (1,)}], 8, 3, dev)
    st.state[0].normal_()  # whatever the slot's last owner left
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for cuts in ([T], [1, 2, 16, 17, 32, 7], [1] * 20 + [55]):
        at, outs = 0, []
        for n in cuts:
            wide = torch.zeros(n, heads * vdim + 8, dtype=dtype, device=dev)
            native.gated_linear_scan(proj[at:at + n].to(dev).contiguous(), 8, 8 + heads * dim, 8 + 2 * heads * dim, fb.to(dev), lower.to(dev),
                                     gain.to(dev), st.state[0], torch.tensor([1], dtype=torch.int32, device=dev),
                                     torch.tensor([0, n], dtype=torch.int32, device=dev), torch.arange(at, at + n, dtype=torch.int32, device=dev),
                                     heads, dim, vdim, 1e-4, q_act=True, out_scale=0.7, out=wide[:, 8:])
            assert float(wide[:, :8].abs().max()) == 0
            outs.append(wide[:, 8:])
            at += n
        got = torch.cat(outs).double().cpu()
        assert float((got - want).abs().max() / want.abs().max()) <= tol, cuts
        assert float((st.state[0][1].double().cpu() - S).abs().max() / S.abs().max()) <= (1e-5 if dtype == torch.float32 else 1e-2), cuts


def test_recurrence_keeps_a_far_write(gpu_device):
    """A channel whose forget gate stays at its lower bound of almost one keeps what token 5 wrote for 600 tokens; a channel
    with a small bound has lost it.  Read back by a query on that channel alone."""
    from tgis_amd import native

    dev = torch.device("cuda:0")
    T, dk, dv = 600, 16, 32
    proj = torch.zeros(T, 2 * dk + dv)
    proj[:, dk:2 * dk] = -30.0           # sigmoid -> 0: f = lower
    proj[5, dk:2 * dk] = -30.0
    proj[:, 2 * dk:] = 0.01
    proj[5, 2 * dk:] = torch.arange(dv) + 10.0
    proj[T - 1, 0] = 4.0                 # the last query reads channel 0 ...
    lower = torch.full((dk,), 0.2)
    lower[0] = 0.9999                    # ... which forgets almost nothing
    # the write of token 5 enters with weight 1 - f = 1e-4 and decays by f^(T - 6); against a background of 0.01 it dominates
    st = torch.zeros(2, 1, dk, dv, device=dev)
    out = native.gated_linear_scan(proj.to(dev), 0, dk, 2 * dk, None, lower.to(dev), torch.ones(dv, device=dev), st,
                                   torch.zeros(1, dtype=torch.int32, device=dev), torch.tensor([0, T], dtype=torch.int32, device=dev),
                                   torch.arange(T, dtype=torch.int32, device=dev), 1, dk, dv, 1e-12, q_act=False)
    f0 = 0.9999
    s = torch.zeros(dv, dtype=torch.float64)
    for t in range(T):
        s = f0 * s + (1 - f0) * proj[t, 2 * dk:].double()
    want = ref.rms_unit((4.0 * s)[None], 1e-12)[0]
    assert torch.allclose(out[-1].double().cpu(), want, atol=1e-4)
    assert float(want[-1] / want[0]) > 1.5  # the ramp token 5 wrote is still there


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [37, 300])
def test_feed_forwards(gpu_device, dtype, T):
    """The gated unit with biases (activation in the projection's epilogue on short steps) and the expert mixture whose chosen
    logits are softmaxed among themselves (router with a bias, weights on the experts' outputs)."""
    from tgis_amd.utils.mixers import GatedUnit, RoutedExperts

    cfg = tiny.make_config([tiny.layer(mlp=tiny.dense_mlp(80)), tiny.layer(mlp=tiny.moe_mlp(experts=7, top=3, ff=24))], width=48)
    tensors = tiny.make_tensors(cfg, seed=5)
    w = _dict_weights(tensors, dtype)
    h = torch.randn(T, 48, generator=torch.Generator().manual_seed(T)).to(dtype)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    got = GatedUnit(w, "l0.mlp", mode="silu", bias=True)(h.cuda())
    want = ref.gated_unit(h.double(), _f64(tensors, "l0.mlp."))
    assert float((got.double().cpu() - want).abs().max() / want.abs().max()) <= tol
    moe = RoutedExperts(w, "l1.mlp", experts=7, top=3, shared=False, router_bias=True, softmax_top=True, weight_on_input=False)
    from tgis_amd import native

    idx, weight, _ = native.moe_route(h.cuda(), moe.router, None, 3, moe.router_b, True)
    want_idx, want_w = ref.route_top_softmax(h.double(), _f64(tensors, "l1.mlp."), 3)
    same = (idx.cpu().long() == want_idx).all(-1)
    assert float(same.double().mean()) >= (1.0 if dtype == torch.float32 else 0.95)
    assert torch.allclose(weight.cpu().double()[same], want_w[same], atol=1e-5 if dtype == torch.float32 else 1e-5)
    got = moe(h.cuda())
    want = ref.expert_mixture(h.double(), _f64(tensors, "l1.mlp."), cfg["layers"][1]["mlp"])
    err = (got.double().cpu() - want).abs().amax(-1) / want.abs().max()
    assert float(err[same].max()) <= tol


# ---- generation through the serving entry points -----------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [0, 16])
def test_greedy_generation_through_batches(gpu_device, std, dtype, chunk, monkeypatch):
    """from_pb -> generate_token(first) -> decode steps (captured graphs) with a second batch prefilled, concatenated and
    one request pruned on the way; prompts prefilled whole or in portions of 16.  Token ids against the oracle's greedy
    continuation, teacher-forced where bf16 may flip a near tie."""
    from tgis_amd.testing import SyntheticTokenizer, make_batch_pb

    cfg, tensors = std
    monkeypatch.setenv("TGIS_PREFILL_CHUNK", str(chunk))
    tok = SyntheticTokenizer(cfg["vocab"])
    lm = build_lm(cfg, tensors, dtype, pages=40, slots=6, tokenizer=tok)
    steps = 12
    with lm.context_manager():
        b1, errs = lm.batch_type.from_pb(make_batch_pb([37, 5, 50], steps, batch_id=0), tok, lm.dtype, lm.device, None, None, True)
        assert not errs
        prompts = {r.id: b1.all_input_ids_tensor[i, :l].tolist() for i, (r, l) in enumerate(zip(b1.requests, b1.input_lengths))}
        out = {r.id: [] for r in b1.requests}
        for t in lm.generate_token(b1, first=True)[0]:
            out[t.request_id].append(t.token_id)
        for _ in range(3):
            for t in lm.generate_token(b1)[0]:
                out[t.request_id].append(t.token_id)
        b2, _ = lm.batch_type.from_pb(make_batch_pb([20, 33], steps, batch_id=1, first_request_id=3), tok, lm.dtype, lm.device, None, None, True)
        for i, (r, l) in enumerate(zip(b2.requests, b2.input_lengths)):
            prompts[r.id] = b2.all_input_ids_tensor[i, :l].tolist()
            out[r.id] = []
        for t in lm.generate_token(b2, first=True)[0]:
            out[t.request_id].append(t.token_id)
        batch = lm.batch_type.concatenate([b1, b2])
        for _ in range(3):
            for t in lm.generate_token(batch)[0]:
                out[t.request_id].append(t.token_id)
        batch = lm.batch_type.prune(batch, [1])
        assert lm.state_cache.free_slots == 6 - 4
        for _ in range(4):
            for t in lm.generate_token(batch)[0]:
                out[t.request_id].append(t.token_id)
        batch.release()
    assert lm.kv_cache.free_pages == 40 and lm.state_cache.free_slots == 6
    for rid, ids in out.items():
        # the oracle, fed the engine's own tokens: at every step the engine's choice must be the oracle's argmax, or a
        # near tie of it under bf16
        st = ref.new_state(cfg)
        logits = ref.advance(cfg, tensors, prompts[rid], st)[-1]
        for k, t in enumerate(ids):
            best = int(logits.argmax())
            if t != best:
                gap = float(logits[best] - logits[t])
                assert dtype == torch.bfloat16 and gap < 0.05 * float(logits.std()), (rid, k, t, best, gap)
            logits = ref.advance(cfg, tensors, [t], st)[-1]


# ---- the trace runner, as a user starts it ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_replays_a_schedule(gpu_device, tmp_path, dtype):
    """A checkpoint folder of its own shape written to disk and replayed by bin/trace_run in a child process: requests admitted
    at different steps, portions beside single tokens, a request that sits a step out, a pool of 6 pages for 3 live requests,
    slots and pages handed on to later requests."""
    from safetensors.torch import save_file

    layers = [tiny.layer(left=tiny.attention_part(heads=8, kv_heads=2, dim=16, vdim=32, scale=0.25, window=20, keep_first=2, rot_dims=4),
                         right=tiny.recurrent_part(heads=4, dim=8, vdim=16), mlp=tiny.moe_mlp(experts=4, top=2, ff=32)),
              tiny.layer(left=tiny.attention_part(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.2, window=35, keep_first=5, rot_dims=32),
                         right=tiny.recurrent_part(heads=2, dim=32, vdim=32), mlp=tiny.dense_mlp(48)),
              tiny.layer(mlp=None)]
    cfg = tiny.make_config(layers, width=64, vocab=70, eps=1e-6)
    tensors = tiny.make_tensors(cfg, seed=11)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(model_dir / "model.safetensors"))
    prompts = {"a": rand_tokens(60, cfg, tensors, 1), "b": rand_tokens(33, cfg, tensors, 2), "c": rand_tokens(64, cfg, tensors, 3), "d": rand_tokens(40, cfg, tensors, 4)}
    want = {k: ref.forward(cfg, tensors, v) for k, v in prompts.items()}
    schedule = [[("a", 31)], [("a", 2), ("b", 30)], [("a", 1), ("b", 1), ("c", 33)], [("a", 26), ("c", 1)], [("b", 2), ("c", 30)],
                [("d", 2)], [("d", 37), ("c", 0)], [("d", 1)]]
    done = {k: 0 for k in prompts}
    lines, expect = [], []
    for n, step in enumerate(schedule):
        entries, rows, end = [], [], []
        for rid, cnt in step:
            if cnt == 0:
                continue
            lo = done[rid]
            entries.append({"id": rid, "tokens": prompts[rid][lo:lo + cnt], "want": list(range(cnt))})
            rows.append(want[rid][lo:lo + cnt])
            done[rid] += cnt
            if done[rid] == len(prompts[rid]):
                end.append(rid)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
        expect.append(torch.cat(rows))
    out_dir = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(out_dir), "--max-tokens", "192", "--slots", "3"],
                       input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=280)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {n}" for n in range(len(schedule))]
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    for n, e in enumerate(expect):
        got = torch.from_numpy(np.fromfile(out_dir / f"{n}.f32", dtype="<f4").reshape(e.shape).copy())
        assert close(got, e, dt), n
