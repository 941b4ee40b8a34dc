"""GPU: the Tatevik family on the kernels (FlashCausalLM + utils/mixers.py + csrc/norm_f32, causal_conv, selective_scan,
attn_mixed_heads, gated_linear_scan, moe) against the plain float64 restatement in oracle/tatevik_ref.py, on small seeded
checkpoints of their own sizes.

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

from oracle import tatevik_ref as ref
from oracle import tatevik_tiny as tiny

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-4, torch.bfloat16: 0.15}
DTYPES = [torch.float32, torch.bfloat16]
D = torch.float64


def build_lm(cfg, tensors, dtype, pages=64, slots=4, tokenizer=None):
    from tgis_amd.inference_engine.synthetic import InferenceEngine
    from tgis_amd.models.custom_modeling.flash_tatevik_modeling import TatevikConfig
    from tgis_amd.models.flash_causal_lm import FlashCausalLM

    eng = InferenceEngine({k: v.clone() for k, v in tensors.items()}, TatevikConfig(**cfg), dtype, None, tokenizer=tokenizer)
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
    """Random tokens for which no router of the checkpoint is near a tie and no read-out of a linear attention cancels before
    its norm (drawn again until so): a bfloat16 run then differs from the float64 restatement by rounding, not by a decision."""
    key = (json.dumps(cfg, sort_keys=True), n, seed)
    if key not in _PROMPTS:
        _PROMPTS[key] = ref.clear_cut_tokens(cfg, tensors, n, seed)
    return _PROMPTS[key]


STD_LOOP = {"start": 1, "stop": 3, "times": 3}


@pytest.fixture(scope="module")
def std():
    cfg = tiny.make_config(tiny.standard_layers(), loop=STD_LOOP)
    return cfg, tiny.make_tensors(cfg, seed=3)


# ---- whole model -----------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [75, 300])
def test_whole_prompt_matches_oracle_layer_by_layer(gpu_device, std, dtype, n):
    """75 tokens: the decode-sized GEMM path; 300: the library GEMMs.  Both are longer than every window of the configuration."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(n, cfg, tensors, 1)
    want_trace = []
    want = ref.TatevikRef(cfg, tensors).forward(toks, want_trace)
    with lm.context_manager():
        seq, trace = lm.open_sequence(), []
        got = lm.step_sequences([(seq, toks)], residual_trace=trace)
        lm.close_sequence(seq)
    assert len(trace) == len(want_trace) == 10  # six layers, two of them three times
    for r, (g, w) in enumerate(zip(trace, want_trace)):
        scale = float(w.abs().max())
        assert float((g.double().cpu() - w).abs().max()) <= (1e-4 if dtype == torch.float32 else 0.08) * scale, r
    assert close(got, want, dtype), rel_err(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_by_token_and_portions_equal_whole(gpu_device, std, dtype):
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(150, cfg, tensors, 2)
    want = ref.TatevikRef(cfg, tensors).forward(toks)
    for cuts in ([1] * 150, [2] * 75, [3, 2, 31, 33, 1, 2, 64, 5, 9], [97, 2, 2, 2, 47], [149, 1]):
        with lm.context_manager():
            seq, outs, at = lm.open_sequence(), [], 0
            for c in cuts:
                outs.append(lm.step_sequences([(seq, toks[at:at + c])]))
                at += c
            lm.close_sequence(seq)
        assert close(torch.cat(outs), want, dtype), (cuts[:4], rel_err(torch.cat(outs), want))


@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batches_reuse_pages_and_slots(gpu_device, std, dtype):
    """Five requests through a pool of 9 pages and 3 slots: portions of some beside single tokens of others, a request that
    sits steps out, pages and slots handed on to later requests with whatever their last owner left in them."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype, pages=9, slots=3)
    model = ref.TatevikRef(cfg, tensors)
    prompts = {k: rand_tokens(n, cfg, tensors, 10 + i) for i, (k, n) in enumerate({"a": 70, "b": 33, "c": 96, "d": 45, "e": 64}.items())}
    want = {k: model.forward(v) for k, v in prompts.items()}
    schedule = [[("a", 31), ("b", 2)], [("a", 1), ("b", 30)], [("a", 2), ("b", 1), ("c", 40)], [("a", 36), ("c", 1)], [("c", 23)],
                [("c", 2), ("d", 44)], [("c", 30), ("d", 1), ("e", 3)], [("e", 60)], [("e", 1)]]
    done, live, got = {k: 0 for k in prompts}, {}, {k: [] for k in prompts}
    with lm.context_manager():
        for step in schedule:
            entries = []
            for rid, cnt in step:
                if rid not in live:
                    live[rid] = lm.open_sequence()
                entries.append((live[rid], prompts[rid][done[rid]:done[rid] + cnt]))
            out = lm.step_sequences(entries)
            at = 0
            for rid, cnt in step:
                got[rid].append(out[at:at + cnt])
                at += cnt
                done[rid] += cnt
                if done[rid] == len(prompts[rid]):
                    lm.close_sequence(live.pop(rid))
    assert not live and lm.kv_cache.free_pages == 9 and lm.state_cache.free_slots == 3
    for rid in prompts:
        assert close(torch.cat(got[rid]), want[rid], dtype), (rid, rel_err(torch.cat(got[rid]), want[rid]))


def test_stale_slot_and_pages_do_not_leak(gpu_device, std):
    """Every state tensor and page filled with large numbers before a request starts: a sequence begins from zeros."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, torch.float32, pages=8, slots=1)
    for t in lm.state_cache.state + lm.state_cache.shift:
        t.fill_(37.0)
    for r in range(lm.num_layers):
        if lm.kv_cache.layer_shapes[r] is not None:
            lm.kv_cache.k_pool(r).fill_(19.0)
            lm.kv_cache.v_pool(r).fill_(-23.0)
    toks = rand_tokens(50, cfg, tensors, 4)
    want = ref.TatevikRef(cfg, tensors).forward(toks)
    with lm.context_manager():
        seq = lm.open_sequence()
        got = torch.cat([lm.step_sequences([(seq, toks[:2])]), lm.step_sequences([(seq, toks[2:])])])
        lm.close_sequence(seq)
    assert close(got, want, torch.float32), rel_err(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(gpu_device, std, dtype):
    """220 single-token steps behind a short prompt: windows pass over decoded tokens, states are carried all the way."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(240, cfg, tensors, 5)
    want = ref.TatevikRef(cfg, tensors).forward(toks)
    with lm.context_manager():
        seq = lm.open_sequence()
        outs = [lm.step_sequences([(seq, toks[:20])])] + [lm.step_sequences([(seq, [t])]) for t in toks[20:]]
        lm.close_sequence(seq)
    assert close(torch.cat(outs), want, dtype), rel_err(torch.cat(outs), want)


# sizes that the standard configuration happens to make equal, one, or a multiple of eight; other layer orders and loops
OTHER_SHAPES = {
    "no_loop_no_conv": dict(layers=[tiny.pair_layer(mlp=tiny.dense_mlp(40)), tiny.scan_layer(inner=48, state=3, dt_rank=1, conv=1)],
                            width=40, vocab=50, taps=0, loop=None),
    "loop_over_everything": dict(layers=[tiny.channel_decay_layer(heads=1, dim=8, vdim=8, tau=1.0, rank=8, mlp=tiny.moe_mlp(experts=2, top=2, ff=16, groups=2, keep=2)),
                                         tiny.pair_layer(left=tiny.attention_part(heads=2, kv_heads=1, dim=12, vdim=20, window=1, rot_dims=4),
                                                         right=tiny.fixed_decay_part(heads=1, dim=8, vdim=8, decay=(0.9,)))],
                                 width=24, vocab=33, taps=2, loop={"start": 0, "stop": 2, "times": 2}),
    "one_pass_one_tap": dict(layers=[tiny.scan_layer(inner=40, state=20, dt_rank=12, conv=3, mlp=tiny.moe_mlp(experts=9, top=4, ff=24, groups=3, keep=2)),
                                     tiny.channel_decay_layer(heads=5, dim=12, vdim=20, tau=12.0, rank=4, mlp=tiny.dense_mlp(30)),
                                     tiny.pair_layer(left=tiny.attention_part(heads=8, kv_heads=4, dim=24, vdim=8, window=33, rot_dims=0),
                                                     right=tiny.fixed_decay_part(heads=4, dim=16, vdim=12, decay=(0.3, 0.8, 0.97, 1.0)))],
                             width=56, vocab=64, taps=1, loop={"start": 1, "stop": 3, "times": 1}),
    "odd_widths": dict(layers=[tiny.pair_layer(left=tiny.attention_part(heads=3, kv_heads=3, dim=10, vdim=6, window=64, rot_dims=6),
                                               right=tiny.fixed_decay_part(heads=2, dim=6, vdim=10, decay=(0.6, 0.9)), mlp=tiny.moe_mlp(experts=3, top=1, ff=20, groups=1, keep=1)),
                               tiny.scan_layer(inner=30, state=5, dt_rank=3, conv=5, mlp=tiny.dense_mlp(22)),
                               tiny.channel_decay_layer(heads=2, dim=6, vdim=10, tau=2.5, rank=3)],
                       width=36, vocab=41, taps=5, loop={"start": 2, "stop": 3, "times": 4}),
    "wide_heads": dict(layers=[tiny.pair_layer(left=tiny.attention_part(heads=4, kv_heads=2, dim=128, vdim=64, scale=0.08, window=70, rot_dims=64),
                                               right=tiny.fixed_decay_part(heads=2, dim=128, vdim=64, decay=(0.9, 0.99)), mlp=tiny.dense_mlp(128)),
                               tiny.channel_decay_layer(heads=2, dim=64, vdim=128, tau=10.0, rank=16),
                               tiny.scan_layer(inner=256, state=64, dt_rank=8, conv=4)],
                       width=128, vocab=80, taps=3, loop={"start": 0, "stop": 1, "times": 2}),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(OTHER_SHAPES))
def test_other_sizes_and_layer_orders(gpu_device, dtype, shape):
    cfg = tiny.make_config(**OTHER_SHAPES[shape])
    tensors = tiny.make_tensors(cfg, seed=21)
    lm = build_lm(cfg, tensors, dtype, pages=12)
    toks = rand_tokens(90, cfg, tensors, 6)
    want = ref.TatevikRef(cfg, tensors).forward(toks)
    with lm.context_manager():
        seq = lm.open_sequence()
        whole = lm.step_sequences([(seq, toks)])
        lm.close_sequence(seq)
        seq = lm.open_sequence()
        cuts, outs, at = [40, 2, 3, 30] + [1] * 15, [], 0
        for c in cuts:
            outs.append(lm.step_sequences([(seq, toks[at:at + c])]))
            at += c
        lm.close_sequence(seq)
    assert close(whole, want, dtype), rel_err(whole, want)
    assert close(torch.cat(outs), want, dtype), rel_err(torch.cat(outs), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(16))
def test_configurations_drawn_at_random(gpu_device, seed, dtype):
    """Layer kinds, orders, loops, taps and sizes drawn from the design's whole space: a whole prompt, portions with single
    tokens, and two requests of unequal length in one batch."""
    cfg = tiny.random_config(seed)
    tensors = tiny.make_tensors(cfg, seed=100 + seed)
    lm = build_lm(cfg, tensors, dtype, pages=16)
    model = ref.TatevikRef(cfg, tensors)
    a, b = rand_tokens(120, cfg, tensors, 7), rand_tokens(45, cfg, tensors, 8)
    want_a, want_b = model.forward(a), model.forward(b)
    with lm.context_manager():
        seq = lm.open_sequence()
        whole = lm.step_sequences([(seq, a)])
        lm.close_sequence(seq)
        sa, sb = lm.open_sequence(), lm.open_sequence()
        got_a = [lm.step_sequences([(sa, a[:70])])]
        out = lm.step_sequences([(sa, a[70:72]), (sb, b[:40])])
        got_a.append(out[:2])
        got_b = [out[2:]]
        for i in range(5):
            out = lm.step_sequences([(sa, [a[72 + i]]), (sb, [b[40 + i]])])
            got_a.append(out[:1])
            got_b.append(out[1:])
        got_a.append(lm.step_sequences([(sa, a[77:])]))
        lm.close_sequence(sa)
        lm.close_sequence(sb)
    assert close(whole, want_a, dtype), (cfg, rel_err(whole, want_a))
    assert close(torch.cat(got_a), want_a, dtype), (cfg, rel_err(torch.cat(got_a), want_a))
    assert close(torch.cat(got_b), want_b, dtype), (cfg, rel_err(torch.cat(got_b), want_b))


# ---- mechanisms alone ------------------------------------------------------------------------------------------------------
class _Step:
    """What a mixer kernel needs to know about a ragged step of sequences that hold `cached` tokens and bring `new` more."""

    def __init__(self, cached, new, slots, dev):
        self.cu = torch.tensor(np.concatenate([[0], np.cumsum(new)]), dtype=torch.int32, device=dev)
        self.pos = torch.tensor(np.concatenate([np.arange(c, c + n) for c, n in zip(cached, new)]), dtype=torch.int32, device=dev)
        self.slots = torch.tensor(slots, dtype=torch.int32, device=dev)
        self.max_q = max(new)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,sets,act", [(3, 2, False), (4, 1, True), (1, 2, False), (9, 1, False), (2, 2, True)])
def test_causal_convolution_through_its_tail(gpu_device, dtype, taps, sets, act):
    """Two sequences in one launch, in portions of 1, 2, taps - 1 and more tokens, in slots with stale contents: filters, bias,
    SiLU, the residual form, and the tail carried from portion to portion."""
    from tgis_amd import native

    g = torch.Generator().manual_seed(taps)
    C, dev = 70, gpu_device
    lens = [41, 23]
    # the residual form reads the fp32 normed stream, the activated one a projection in the serving dtype
    xs = [torch.randn(n, C, generator=g) for n in lens]
    if act:
        xs = [x.to(dtype).float() for x in xs]
    w = torch.randn(sets, C, taps, generator=g) * 0.5
    bias = torch.randn(sets, C, generator=g) * 0.3 if act else None
    want = []
    for x in xs:
        per = []
        for s in range(sets):
            y, _ = ref.causal_conv(x.double(), w[s].double(), torch.zeros(taps - 1, C, dtype=D), None if bias is None else bias[s].double())
            per.append(ref.silu(y) if act else y + x.double())
        want.append(torch.stack(per))
    tail = torch.full((3, 5 + (taps - 1) * C), 99.0, device=dev)
    view = tail[:, 5:] if taps > 1 else None
    cuts = [[1, 2, max(taps - 1, 1), 20, 1, 41], [2, 1, 1, 1, 18, 23]]
    got, at = [[], []], [0, 0]
    while at[0] < lens[0] or at[1] < lens[1]:
        new, cached, slots, rows = [], [], [], []
        for b in range(2):
            if at[b] < lens[b]:
                c = min(cuts[b].pop(0), lens[b] - at[b])
                new.append(c), cached.append(at[b]), slots.append(2 * b), rows.append((b, at[b], c))
        st = _Step(cached, new, slots, dev)
        x_in = torch.cat([xs[b][a:a + c] for b, a, c in rows]).to(dev)
        x_in = x_in if not act else x_in.to(dtype)
        out = native.causal_conv(x_in, w.to(dev), None if bias is None else bias.to(dev), view, st.slots, st.cu, st.pos, dtype,
                                 act=act, residual=not act, max_q_len=st.max_q)
        o = 0
        for b, a, c in rows:
            got[b].append(out[:, o:o + c])
            o += c
            at[b] += c
    for b in range(2):
        g_ = torch.cat(got[b], 1).double().cpu()
        tol = 1e-5 if dtype == torch.float32 else 0.03
        assert float((g_ - want[b]).abs().max()) <= tol * float(want[b].abs().max()), b
    assert float(tail[:, :5].min()) == 99.0 and float(tail[1].min()) == 99.0  # nothing outside the two slots' tails was written


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inner,N", [(96, 12), (40, 1), (300, 16), (64, 20), (33, 128), (70, 9)])
def test_selective_scan_and_its_state(gpu_device, dtype, inner, N):
    from tgis_amd import native

    g = torch.Generator().manual_seed(inner + N)
    dev, n = gpu_device, 75
    rnd = lambda *s: torch.randn(*s, generator=g)
    x, z, dtp = rnd(n, inner).to(dtype), rnd(n, inner).to(dtype), rnd(n, inner)
    bc = (rnd(n, 2 * N + 3) * N ** -0.5).to(dtype)
    dt_bias, A_log, Dv = rnd(inner) - 1.0, torch.log(torch.rand(inner, N, generator=g) * 4 + 0.05), rnd(inner)
    d = ref.softplus(dtp.double() + dt_bias.double())
    S = torch.zeros(inner, N, dtype=D)
    want = []
    for t in range(n):
        S = torch.exp(d[t][:, None] * -torch.exp(A_log.double())) * S + (d[t] * x[t].double())[:, None] * bc[t, 3:3 + N].double()[None]
        want.append((S @ bc[t, 3 + N:].double() + Dv.double() * x[t].double()) * ref.silu(z[t].double()))
    want = torch.stack(want)
    state = torch.full((3, inner, N), 55.0, device=dev)
    outs, at = [], 0
    for c in (1, 2, 30, 17, 25):
        st = _Step([at], [c], [1], dev)
        outs.append(native.selective_scan(x[at:at + c].to(dev), dtp[at:at + c].to(dev), dt_bias.to(dev), bc[at:at + c].to(dev), 3, 3 + N,
                                          z[at:at + c].to(dev), A_log.to(dev), Dv.to(dev), state, st.slots, st.cu, st.pos, N))
        at += c
    got = torch.cat(outs).double().cpu()
    tol = 2e-5 if dtype == torch.float32 else 0.02
    assert float((got - want).abs().max()) <= tol * float(want.abs().max())
    assert float((state[1].double().cpu() - S).abs().max()) <= 2e-5 * float(S.abs().max()) and float(state[0].min()) == 55.0


GEOMETRIES = [(6, 3, 32, 24), (8, 2, 80, 48), (4, 4, 16, 64), (2, 1, 128, 128), (3, 1, 10, 6), (32, 8, 64, 64)]


def _write_and_attend(native, dev, dtype, q, k, v, talk, scale, window, rot, pieces, eps=1e-5, gate=None, impl=0):
    """q [n, H, dk], k [n, G, dk], v [n, G, dv] of one sequence go through rotation, unit norm and cache write, then
    attention, in the given portions; pages are dealt in a scrambled order.  Returns [n, H dv]."""
    n, H, dk = q.shape
    G, dv = k.shape[1], v.shape[2]
    pages = (n + 31) // 32
    kp = torch.zeros((pages + 3, G, 32 * dk), dtype=dtype, device=dev)
    vp = torch.zeros((pages + 3, G, dv * 32), dtype=dtype, device=dev)
    order = torch.randperm(pages + 2, generator=torch.Generator().manual_seed(n))[:pages].to(torch.int32)
    bt = order.view(1, -1).to(dev)
    from tgis_amd.utils.layers import workspace

    inv = torch.tensor([rot[0] ** (-2.0 * i / rot[1]) for i in range(rot[1] // 2)], dtype=torch.float32, device=dev) if rot[1] else None
    proj = torch.cat([q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)], 1).to(dtype).to(dev)
    outs, at = [], 0
    for c in pieces:
        pos = torch.arange(at, at + c, dtype=torch.int32, device=dev)
        slots = (bt[0, (pos // 32).long()] * 32 + pos % 32).to(torch.int32)
        part = proj[at:at + c].clone()
        native.rope_rows_unit_kv_write(part, 0, H * dk, (H + G) * dk, inv, pos, slots, kp, vp, H, G, dk, dv, rot[1], eps)
        outs.append(native.attn_mixed_heads(part[:, :H * dk], kp, vp, bt, torch.tensor([at + c], dtype=torch.int32, device=dev),
                                            torch.tensor([0, c], dtype=torch.int32, device=dev), talk.to(dev), H, G, dk, dv, scale,
                                            window=window, gate=None if gate is None else gate[at:at + c].to(dtype).to(dev), max_q_len=c,
                                            max_ctx=at + c, ws=workspace(dev), impl=impl))  # single tokens take the key-split form
        at += c
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", GEOMETRIES)
@pytest.mark.parametrize("window", [0, 1, 33, 70, 200])
def test_mixed_head_attention_against_plain_softmax(gpu_device, dtype, geom, window):
    """Rotation, unit norm, cache write and attention with mixed heads, a window and a gate, in prompt portions and single
    tokens over scrambled pages, against the plain form."""
    from tgis_amd import native

    H, G, dk, dv = geom
    g = torch.Generator().manual_seed(H * dk + window)
    n = 230
    q, k, v = torch.randn(n, H, dk, generator=g), torch.randn(n, G, dk, generator=g), torch.randn(n, G, dv, generator=g)
    gate = torch.randn(n, H * dv, generator=g)
    talk = torch.eye(H) + torch.randn(H, H, generator=g) * 0.3
    rot = (700.0, dk // 2 * 2 if H % 2 else (dk // 4) * 2)
    r16 = lambda t: t.to(dtype).double()
    pos = torch.arange(n)
    qn = ref.rms_unit(ref.rotate_pairs(r16(q), pos, *rot), 1e-5)
    kn = ref.rms_unit(ref.rotate_pairs(r16(k), pos, *rot), 1e-5)
    want = ref.attend_mixed(qn, kn, r16(v), pos, talk.double(), 0.5, window).reshape(n, H * dv) * torch.sigmoid(r16(gate))
    tol = 2e-5 if dtype == torch.float32 else 0.03
    for impl in (0, 1):  # the launcher's choice (matrix cores for portions of two-byte models), and the general kernel
        got = _write_and_attend(native, gpu_device, dtype, q, k, v, talk, 0.5, window, rot, [100, 2, 31, 33, 1, 1, 3, 40] + [1] * 19, gate=gate, impl=impl)
        assert float((got.double().cpu() - want).abs().max()) <= tol * float(want.abs().max()), impl


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(6, 3, 32, 24), (8, 2, 80, 48)])
@pytest.mark.parametrize("window", [40, 64, 97])
def test_attention_finds_a_planted_key_inside_its_window_only(gpu_device, dtype, geom, window):
    """One key among 700 points where every query points, and its value is far from all others: a query sees it iff it lies in
    its window — at the window's first position yes, one further back no — in a prompt, in portions that end at page borders
    and in single decoded tokens."""
    from tgis_amd import native

    H, G, dk, dv = geom
    g = torch.Generator().manual_seed(window)
    n, planted = 700, 411
    u = torch.randn(G, dk, generator=g)
    q = u.repeat_interleave(H // G, 0)[None] + 0.05 * torch.randn(n, H, dk, generator=g)
    k, v = torch.randn(n, G, dk, generator=g), torch.randn(n, G, dv, generator=g)
    k[planted] = u
    v[planted] = 50.0
    talk = torch.eye(H) + torch.randn(H, H, generator=g).abs() * 0.05
    for pieces in ([700], [planted + window - 1, 1, 1, 1] + [n - planted - window - 2], [416, 32, 32, 220], [planted + 1] + [1] * (n - planted - 1)):
        got = _write_and_attend(native, gpu_device, dtype, q, k, v, talk, 1.0, window, (0.0, 0), pieces).double().cpu().view(n, H, dv)
        share = got.mean(-1) / 50.0  # the planted value's weight, about
        inside = (torch.arange(n) >= planted) & (torch.arange(n) - planted < window)
        assert float(share[inside].min()) > 0.9, (pieces[:3], float(share[inside].min()))
        assert float(share[~inside].abs().max()) < 0.1, (pieces[:3], float(share[~inside].abs().max()))
        assert float(share[planted + window - 1].min()) > 0.9 and float(share[planted + window].abs().max()) < 0.1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim", [(3, 24, 40), (2, 40, 64), (1, 3, 33), (4, 64, 32), (2, 128, 64), (1, 256, 128), (2, 48, 96)])
@pytest.mark.parametrize("form", ["head", "channel"])
def test_linear_attention_scan_and_its_state(gpu_device, dtype, heads, dim, vdim, form):
    """Both forms of the decay on columns of one projection: SiLU on q, k, v and a norm over all heads of a token with a sigmoid
    gate (decay per head), or a scaled q, a norm per head and a SiLU gate (decay per channel, sigmoid^(1 / tau)); portions of
    1, 2 and more tokens through a slot with stale contents; the final state."""
    from tgis_amd import native

    g = torch.Generator().manual_seed(heads * dim + vdim)
    dev, n, H, dk, dv = gpu_device, 90, heads, dim, vdim
    cols = [5, 5 + H * dk + 3, 5 + 2 * H * dk + 8, 5 + 2 * H * dk + H * dv + 11, 5 + 2 * H * dk + 2 * H * dv + 16]  # q k v g f
    ld = cols[4] + H * dk + 2
    proj = (torch.randn(n, ld, generator=g) * (1.5 if form == "channel" else 1.0)).to(dtype)
    P = proj.double()
    q, k = P[:, cols[0]:cols[0] + H * dk].view(n, H, dk), P[:, cols[1]:cols[1] + H * dk].view(n, H, dk)
    v, gt = P[:, cols[2]:cols[2] + H * dv].view(n, H, dv), P[:, cols[3]:cols[3] + H * dv]
    S0 = torch.zeros(H, dk, dv, dtype=D)
    if form == "head":
        decay = torch.linspace(0.6, 0.995, H)
        gain = 1 + 0.2 * torch.randn(H * dv, generator=g)
        o, S = ref.linear_attention(ref.silu(q), ref.silu(k), ref.silu(v), decay.double().view(1, H, 1).expand(n, H, dk), S0)
        want = ref.rms_unit(o.reshape(n, H * dv), 1e-5) * gain.double() * torch.sigmoid(gt)
        kw = dict(decay_mode=2, head_decay=decay.to(dev), q_act=True, k_act=True, v_act=True, norm_rows=True, gate_act=1)
        f_col = -1
    else:
        tau, bias = 7.0, torch.randn(H * dk, generator=g) + 2.0
        gain = 1 + 0.2 * torch.randn(dv, generator=g)
        a = torch.exp(torch.nn.functional.logsigmoid(P[:, cols[4]:cols[4] + H * dk] + bias.double()) / tau).view(n, H, dk)
        o, S = ref.linear_attention(q * dk ** -0.5, k, v, a, S0)
        want = (ref.rms_unit(o, 1e-5) * gain.double()).reshape(n, H * dv) * ref.silu(gt)
        kw = dict(decay_mode=1, f_bias=bias.to(dev), inv_tau=1 / tau, q_scale=dk ** -0.5, norm_rows=False, gate_act=2)
        f_col = cols[4]
    state = torch.full((3, H, dk, dv), -41.0, device=dev)
    pd = proj.to(dev)
    outs, at = [], 0
    for c in (1, 2, 40, 1, 30, 16):
        st = _Step([at], [c], [2], dev)
        part = pd[at:at + c]
        outs.append(native.linear_scan(part, cols[0], cols[1], f_col, cols[2], state, st.slots, st.cu, st.pos, H, dk, dv, 1e-5, gain.to(dev),
                                       gate=part[:, cols[3]:cols[3] + H * dv], max_q_len=c, **kw))
        at += c
    got = torch.cat(outs).double().cpu()
    tol = 3e-5 if dtype == torch.float32 else 0.03
    assert float((got - want).abs().max()) <= tol * float(want.abs().max())
    assert float((state[2].double().cpu() - S).abs().max()) <= (3e-5 if dtype == torch.float32 else 0.02) * float(S.abs().max())
    assert float(state[0].max()) == -41.0


def test_linear_attention_keeps_a_far_write(gpu_device):
    """A key written at the first position and read 600 tokens later through a decay of 0.998 per step, among small writes."""
    from tgis_amd import native

    dev, n, dk, dv = gpu_device, 601, 16, 16
    q, k, v = torch.zeros(n, dk), torch.full((n, dk), -20.0), torch.zeros(n, dv)   # silu(-20) ~ 0: nothing is written ...
    k[0, 3], v[0, 5] = 10.0, 10.0                                                      # ... but one entry at the start
    q[n - 1, 3] = 10.0
    proj = torch.cat([q, k, v, torch.zeros(n, dv)], 1).to(dev)
    state = torch.zeros(1, 1, dk, dv, device=dev)
    st = _Step([0], [n], [0], dev)
    scratch_free = native.linear_scan(proj, 0, dk, -1, 2 * dk, state, st.slots, st.cu, st.pos, 1, dk, dv, 1e-12, torch.ones(dv, device=dev) * dv ** -0.5,
                                      decay_mode=2, head_decay=torch.tensor([0.998], device=dev), q_act=True, k_act=True, v_act=True,
                                      norm_rows=True, gate=proj[:, 2 * dk + dv:], gate_act=1, max_q_len=n)
    assert abs(float(state[0, 0, 3, 5]) / (10.0 * 10.0 * 0.998 ** 600) - 1) < 1e-3
    assert abs(float(scratch_free[n - 1, 5]) - 0.5) < 1e-3  # the row's only entry, normed to one, times sigmoid(0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [37, 300])
def test_feed_forwards_and_row_kernels(gpu_device, dtype, T):
    """The polynomial of unit-RMS powers, the grouped router with its correction, the residual update with both norms, and the
    average of two normed rows — each against its definition."""
    from tgis_amd import native

    g = torch.Generator().manual_seed(T)
    dev, W, F = gpu_device, 72, 104
    z = torch.randn(T, F, generator=g).to(dtype)
    c = (0.9, 0.4, -0.2, 0.1)
    u = z.double()
    want = c[0] * ref.rms_unit(u, 1e-5) + c[1] * ref.rms_unit(u * u, 1e-5) + c[2] * ref.rms_unit(u ** 3, 1e-5) + c[3]
    got = native.poly_norm(z.to(dev), *c, 1e-5).double().cpu()
    assert float((got - want).abs().max()) <= (1e-5 if dtype == torch.float32 else 0.02) * float(want.abs().max())
    # router: 12 experts in 4 groups, 2 kept, 3 chosen
    h = torch.randn(T, W, generator=g).to(dtype)
    p = {"router": torch.randn(12, W, generator=g) * 0.4, "correction": torch.randn(12, generator=g) * 0.1}
    r = {"experts": 12, "top": 3, "groups": {"count": 4, "keep": 2}}
    idx, wt, s, choice = ref.route(h.double(), {k_: v_.double() for k_, v_ in p.items()}, r)
    gi, gw = native.moe_route_grouped(h.to(dev), p["router"].to(dev), p["correction"].to(dev), 3, 4, 2, 1e-20)
    for t in range(T):
        b = choice[t].sort(descending=True).values
        if float(b[2] - b[3]) < 1e-4:
            continue  # a near tie: either choice is right
        assert sorted(gi[t].tolist()) == sorted(idx[t].tolist()), t
        order = {e: j for j, e in enumerate(gi[t].tolist())}
        for j, e in enumerate(idx[t].tolist()):
            assert abs(float(gw[t, order[e]]) - float(wt[t, j])) < 1e-5
    # residual update + norm, and the average of two normed rows
    x, a, b2 = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g).to(dtype), torch.randn(T, W, generator=g)
    s1, s2, vec, w = (torch.randn(W, generator=g) for _ in range(4))
    xs = x.double() + s1.double() * a.double() + s2.double() * b2.double() + vec.double()
    for mean_free in (True, False):
        xo, hn = native.scaled_residual_norm(x.to(dev), a.to(dev), s1.to(dev), b2.to(dev), s2.to(dev), vec.to(dev), w.to(dev), 1e-5, dtype,
                                             mean_free=mean_free)
        wn = ref.layer_norm(xs, w.double(), 1e-5) if mean_free else ref.rms_unit(xs, 1e-5) * w.double()
        assert float((xo.double().cpu() - xs).abs().max()) < 1e-5 and float((hn.double().cpu() - wn).abs().max()) < 1e-4
    y = native.rms_pair_mean(a.to(dev), s1.to(dev), 0.5, b2.to(dev), s2.to(dev), 0.5, 1e-5, dtype)
    wy = 0.5 * (ref.rms_unit(a.double(), 1e-5) * s1.double() + ref.rms_unit(b2.double(), 1e-5) * s2.double())
    assert float((y.double().cpu() - wy).abs().max()) < 1e-4
    # ... and the same average made inside the residual update
    xo, hn = native.scaled_residual_norm(x.to(dev), a.to(dev), vec.to(dev), None, None, None, w.to(dev), 1e-5, dtype,
                                         pair=(b2.to(dev), s1.to(dev), s2.to(dev), 0.5))
    xs = x.double() + vec.double() * wy
    assert float((xo.double().cpu() - xs).abs().max()) < 1e-4
    assert float((hn.double().cpu() - ref.layer_norm(xs, w.double(), 1e-5)).abs().max()) < 1e-4


# ---- generation through the serving entry points ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [0, 16])
def test_greedy_generation_through_batches(gpu_device, std, dtype, chunk, monkeypatch):
    """from_pb -> generate_token(first) -> decode steps (captured graphs) with a second batch prefilled, concatenated and
    one request pruned on the way; prompts prefilled whole or in portions of 16.  Token ids against a teacher-forced greedy
    continuation."""
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
    # float32: the oracle, fed the engine's own tokens — at every step the engine's choice must be the oracle's argmax.
    # bfloat16: the prompts here are not drawn to keep routers away from ties, so the yardstick is the same checkpoint stepped
    # sequence by sequence through step_sequences in bfloat16 (no batches, no captured graphs, no pruning); a choice may differ
    # only within the bf16 bound on a row.
    model = ref.TatevikRef(cfg, tensors)
    plain = build_lm(cfg, tensors, dtype, pages=40, slots=2) if dtype == torch.bfloat16 else None
    for rid, ids in out.items():
        if plain is None:
            st = model.new_state()
            step = lambda toks: model.advance(st, toks)[-1]
        else:
            seq = plain.open_sequence()
            step = lambda toks: plain.step_sequences([(seq, toks)])[-1].double().cpu()
        with (plain.context_manager() if plain is not None else torch.no_grad()):
            logits = step(prompts[rid])
            for k, t in enumerate(ids):
                best = int(logits.argmax())
                if t != best:
                    gap = float(logits[best] - logits[t])
                    assert dtype == torch.bfloat16 and gap < TOL[dtype] * float(logits.std()), (rid, k, t, best, gap)
                logits = step([t])
        if plain is not None:
            plain.close_sequence(seq)


# ---- the trace runner, as a user starts it ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_replays_a_schedule(gpu_device, tmp_path, dtype):
    """A checkpoint folder of its own shape written to disk and replayed by bin/trace_run in a child process: requests admitted
    at different steps, portions beside single tokens, a request that sits a step out, a pool of 6 pages for 3 live requests,
    slots and pages handed on to later requests."""
    from safetensors.torch import save_file

    layers = [tiny.pair_layer(left=tiny.attention_part(heads=8, kv_heads=4, dim=16, vdim=32, scale=0.25, window=20, rot_dims=4),
                              right=tiny.fixed_decay_part(heads=4, dim=8, vdim=16, decay=(0.5, 0.8, 0.95, 0.99)), mlp=tiny.moe_mlp(experts=4, top=2, ff=32, groups=2, keep=1)),
              tiny.scan_layer(inner=64, state=8, dt_rank=4, conv=3, mlp=tiny.dense_mlp(48)),
              tiny.channel_decay_layer(heads=2, dim=16, vdim=32, tau=4.0, rank=8, mlp=None)]
    cfg = tiny.make_config(layers, width=64, vocab=70, eps=1e-6, taps=2, loop={"start": 0, "stop": 2, "times": 2})
    tensors = tiny.make_tensors(cfg, seed=11)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(model_dir / "model.safetensors"))
    prompts = {"a": rand_tokens(60, cfg, tensors, 1), "b": rand_tokens(33, cfg, tensors, 2), "c": rand_tokens(64, cfg, tensors, 3), "d": rand_tokens(40, cfg, tensors, 4)}
    model = ref.TatevikRef(cfg, tensors)
    want = {k: model.forward(v) for k, v in prompts.items()}
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
