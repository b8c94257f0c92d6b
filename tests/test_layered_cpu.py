"""CPU: configuration reading and weight packing of layer-list designs, and the plain
restatement's own consistency (no GPU here)."""
import numpy as np
import pytest

import sinulorn_cases as C
import sinulorn_ref as R
from yalm_amd import layered as Ly
from yalm_amd import models as M


def test_config_reads_every_size_and_constant():
    c = Ly.sinulorn_config(C.MIXED, max_tokens=300)
    assert (c.width, c.vocab, c.embed_scale, c.norm_eps, c.max_tokens) == (96, 211, 7.0, 1e-5, 300)
    l0, l1, l2, l3, l4, l5 = c.layers
    assert (l0.mixer, l0.heads, l0.kv_heads, l0.dim, l0.vdim, l0.conv, l0.ff_kind, l0.ff) == (
        Ly.MIX_DELTA, 4, 2, 24, 40, 4, Ly.FF_DENSE, 72)
    assert (l1.mixer, l1.kv_from, l1.kv_rank, l1.q_rank, l1.attn_scale) == (Ly.MIX_LATENT, -1, 40, 56, 0.3)
    assert (l1.experts, l1.top, l1.groups, l1.groups_keep, l1.router_scale, l1.limit, l1.shared_ff, l1.shared_limit) == (
        8, 2, 4, 2, 1.75, 1.5, 40, 0.75)
    assert (l2.mixer, l2.rec_width, l2.blocks, l2.conv, l2.ff_kind) == (Ly.MIX_RGLRU, 80, 5, 3, Ly.FF_NONE)
    assert l3.kv_from == 1 and l3.in_rows == l3.q_rank
    assert l4.shared_ff == 0 and l4.top == 1
    assert l0.in_rows == 2 * 2 * 24 + 2 * 4 * 40 + 2 * 4


def test_unknown_names_are_refused():
    bad = C.config([("sliding", {}, None)])
    with pytest.raises(ValueError):
        Ly.sinulorn_config(bad)


def test_pack_concatenates_transposes_and_stacks():
    cfg = C.MIXED
    t = Ly.sinulorn_random_tensors(cfg, seed=3)
    for wdt in (M.F32, M.BF16):
        c = Ly.sinulorn_config(cfg, weight_dtype=wdt)
        p = Ly.sinulorn_pack(c, t)
        f = (lambda a: a) if wdt == M.F32 else Ly.bf16_to_f32
        d0 = p["layers"][0]
        got = f(d0["w_in"])
        want = np.concatenate([t["l0.mix." + n] for n in ("q", "k", "v", "g", "b", "a")])
        assert np.array_equal(got, want)
        d1, l1 = p["layers"][1], c.layers[1]
        ukt = f(d1["w_ukt"])
        uk = t["l1.mix.uk"].reshape(l1.heads, l1.dim, l1.kv_rank)
        assert np.array_equal(ukt, uk.transpose(0, 2, 1))
        assert np.array_equal(f(d1["w_in"]), np.concatenate([t["l1.mix.dq"], t["l1.mix.dkv"]]))
        assert np.array_equal(f(d1["w_gate"])[5], t["l1.mlp.e5.gate"])
        assert np.array_equal(f(p["layers"][3]["w_in"]), t["l3.mix.dq"]) and "kv_norm" not in p["layers"][3]
        assert d1["router"].dtype == np.float32 and np.array_equal(d1["router"], t["l1.mlp.router"])
        d2 = p["layers"][2]
        assert np.array_equal(d2["in_bias"], np.concatenate([t["l2.mix.y.b"], t["l2.mix.x.b"]]))
        for l, d in zip(c.layers, p["layers"]):
            assert set(d) == set(Ly.packed_shapes(c, l))


def test_bf16_round_trip_is_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.1415927, 1e-30], np.float32)
    b = Ly.f32_to_bf16(x)
    assert np.array_equal(Ly.bf16_to_f32(b)[:3], np.array([1.0, 1.0, 1.015625], np.float32))
    assert np.all(np.abs(Ly.bf16_to_f32(b) - x) <= np.abs(x) * 2.0**-8)


@pytest.mark.parametrize("cfg", [C.MIXED, C.ODD], ids=["mixed", "odd"])
def test_restatement_is_causal(cfg):
    """Position t of the plain restatement depends on positions 0..t only."""
    w = {k: v.astype(np.float64) for k, v in Ly.sinulorn_random_tensors(cfg, seed=1).items()}
    tok = C.tokens(cfg, 21)
    full = R.forward(cfg, w, tok)
    part = R.forward(cfg, w, tok[:9])
    assert np.allclose(full[:9], part, rtol=0, atol=1e-10)


def test_restatement_router_respects_groups():
    """An expert outside the kept groups is never chosen, however large its score."""
    rng = np.random.default_rng(0)
    E, G, keep, top, Wd = 8, 4, 1, 2, 12
    w = {"r.router": rng.standard_normal((E, Wd))}
    h = rng.standard_normal((50, Wd))
    idx, wt = R.route(w, "r.", h, {"experts": E, "top": top, "scale": 2.0, "groups": {"count": G, "keep": keep}})
    assert np.all(idx[:, 0] // (E // G) == idx[:, 1] // (E // G))
    z = h @ w["r.router"].T
    s = np.exp(z - z.max(1, keepdims=True))
    s /= s.sum(1, keepdims=True)
    assert np.array_equal(idx[:, 0], s.argmax(1))
    assert np.allclose(wt[:, 0], 2.0 * s.max(1))


# ------------------------------------------------------------------ Lenuzen
def test_lenuzen_config_reads_every_size_and_constant():
    import lenuzen_cases as LC

    c = Ly.lenuzen_config(LC.MIXED, max_tokens=300)
    assert (c.arch, c.width, c.vocab, c.embed_scale, c.norm_eps, c.max_tokens, c.logit_scale) == (
        "Lenuzen", 96, 211, 5.0, 1e-5, 300, 0.75)
    assert (c.norm_kind, c.pre_norm, c.pos_embed, c.tied_head) == (Ly.NORM_LAYER, False, False, True)
    l0, l1, l2, l3, l4, l5 = c.layers
    assert (l0.mixer, l0.heads, l0.kv_heads, l0.dim, l0.vdim, l0.mask_kind, l0.mask_size, l0.attn_scale) == (
        Ly.MIX_ATTN, 3, 1, 32, 16, Ly.MASK_CHUNK, 7, 0.17)
    assert (l0.qk_norm, l0.v_norm, l0.sink, l0.out_gate, l0.talking, l0.in_biased, l0.head_temps) == (
        Ly.QK_WHOLE, 0, 1, 0, True, False, False)
    assert (l0.rot_dims, l0.rot_base, l0.rot_factor, l0.rot_orig, l0.rot_fast, l0.rot_slow) == (32, 10000.0, 2.0, 64, 8.0, 2.0)
    assert (l1.mask_kind, l1.mask_size, l1.qk_norm, l1.v_norm, l1.sink, l1.out_gate, l1.in_biased, l1.head_temps) == (
        Ly.MASK_WINDOW, 9, Ly.QK_HEAD_UNIT, 1, 0, 1, True, True)
    assert (l1.ff_kind, l1.ff, l2.ff_kind) == (Ly.FF_PLAIN, 40, Ly.FF_NONE)
    assert l2.rot_factor == 0.0 and l3.rot_base == 500.0 and (l5.rot_factor, l5.rot_orig) == (8.0, 16)
    assert l0.in_rows == 3 * 32 + 1 * (32 + 16) and l1.in_rows == 4 * 24 + 2 * (24 + 40) + 4
    assert l1.mix_out == 4 * 40


def test_lenuzen_unknown_names_are_refused():
    import lenuzen_cases as LC

    with pytest.raises(ValueError):
        Ly.lenuzen_config(LC.config([("attention_3", LC.window(), None)]))
    with pytest.raises(ValueError):
        Ly.lenuzen_config(LC.config([("attention", LC.window(), {"kind": "moe", "ff": 8})]))


def test_lenuzen_pack_concatenates_and_ties_the_head():
    import lenuzen_cases as LC

    cfg = LC.MIXED
    t = Ly.lenuzen_random_tensors(cfg, seed=3)
    assert set(t) == set(Ly.lenuzen_tensor_shapes(cfg))
    for wdt in (M.F32, M.BF16):
        c = Ly.lenuzen_config(cfg, weight_dtype=wdt)
        p = Ly.lenuzen_pack(c, t)
        f = (lambda a: a) if wdt == M.F32 else Ly.bf16_to_f32
        assert p["head"] is p["embed"]
        d1, l1 = p["layers"][1], c.layers[1]
        assert np.array_equal(f(d1["w_in"]), np.concatenate([t["l1.mix." + n] for n in ("q", "k", "v", "g")]))
        nb = l1.in_rows - l1.heads
        assert np.array_equal(d1["in_bias"][:nb], np.concatenate([t["l1.mix." + n + ".b"] for n in ("q", "k", "v")]))
        assert not d1["in_bias"][nb:].any()
        assert np.array_equal(d1["head_temp"], t["l1.mix.temp"]) and np.array_equal(d1["norm1b"], t["l1.norm1"])
        d0 = p["layers"][0]
        assert np.array_equal(f(d0["w_in"]), np.concatenate([t["l0.mix." + n] for n in ("q", "k", "v")]))
        assert np.array_equal(d0["talk"], t["l0.mix.talk"]) and np.array_equal(d0["q_norm"], t["l0.mix.q.norm"])
        assert np.array_equal(f(d0["w_up"]), t["l0.mlp.up"]) and "norm2b" not in p["layers"][2]
        for l, d in zip(c.layers, p["layers"]):
            assert set(d) == set(Ly.packed_shapes(c, l))


def test_lenuzen_restatement_is_causal_and_masks_hold():
    """The restatement itself: logits at t do not depend on later tokens; a one-layer window
    model's logits at t do not depend on tokens the window has left behind."""
    import lenuzen_cases as LC
    import lenuzen_ref as LR

    cfg = LC.MIXED
    w = {k: v.astype(np.float64) for k, v in Ly.lenuzen_random_tensors(cfg, seed=4).items()}
    a = LC.tokens(cfg, 40, 1)
    b = list(a)
    b[30] = (b[30] + 1) % cfg["vocab"]
    ra, rb = LR.forward(cfg, w, a), LR.forward(cfg, w, b)
    assert np.array_equal(ra[:30], rb[:30]) and not np.allclose(ra[30], rb[30])
    one = LC.ONLY_WINDOW
    size = one["layers"][0]["mixer"]["mask"]["size"]
    w1 = {k: v.astype(np.float64) for k, v in Ly.lenuzen_random_tensors(one, seed=5).items()}
    a = LC.tokens(one, 30, 2)
    b = list(a)
    b[10] = (b[10] + 1) % one["vocab"]
    ra, rb = LR.forward(one, w1, a), LR.forward(one, w1, b)
    assert not np.allclose(ra[10 + size - 1], rb[10 + size - 1]) and np.allclose(ra[10 + size:], rb[10 + size:], atol=1e-12)
    m = LR.visible("chunk", 4, 10)
    assert m[5, 4] and not m[4, 3] and m[7, 4] and not m[8, 7] and not m[3, 4]
    p = LR.softmax_rows(np.zeros((1, 3)), np.array([[True, True, False]]), True)
    assert np.allclose(p, [[1 / 3, 1 / 3, 0.0]])


# ------------------------------------------------------------------ Mirorax
def test_mirorax_config_reads_every_size_and_constant():
    import mirorax_cases as MC

    c = Ly.mirorax_config(MC.MIXED, max_tokens=300)
    assert (c.arch, c.width, c.vocab, c.embed_scale, c.norm_eps, c.max_tokens, c.logit_scale) == (
        "Mirorax", 96, 211, 1.0, 1e-5, 300, 1.0)
    assert (c.norm_kind, c.pre_norm, c.pos_embed, c.tied_head, c.block_kind) == (
        Ly.NORM_RMS, True, False, False, Ly.BLOCK_PARALLEL)
    # layers 1..3 are walked twice: 6 layers, 9 runs; the repeated runs share their first pass
    assert [l.shares for l in c.layers] == [-1, -1, -1, -1, 1, 2, 3, -1, -1]
    assert [l.pre_added for l in c.layers] == [False, True, False, False, True, False, False, False, False]
    a0, l1, a2, l3 = c.layers[:4]
    assert (a0.mixer, a0.heads, a0.kv_heads, a0.dim, a0.vdim, a0.attn_scale, a0.mask_kind, a0.out_gate, a0.sink) == (
        Ly.MIX_ATTN, 4, 2, 24, 40, 0.21, Ly.MASK_CAUSAL, Ly.GATE_ELEMENT, 0)
    assert (a0.in_biased, a0.o_biased, a0.rot_dims, a0.ff_kind, a0.ff, a0.limit, a0.ff_act) == (
        True, True, 0, Ly.FF_DENSE, 72, 1.25, Ly.ACT_CLAMP)
    assert a0.in_rows == 4 * 24 + 2 * (24 + 40) + 4 * 40
    assert (l1.mixer, l1.heads, l1.dim, l1.rot_dim, l1.vdim, l1.kv_rank, l1.q_rank, l1.mask_kind, l1.mask_size) == (
        Ly.MIX_LATENT, 3, 24, 8, 40, 32, 0, Ly.MASK_WINDOW, 9)
    assert (l1.sink, l1.sink_learned, l1.rot_dims, l1.rot_base, l1.attn_scale) == (1, True, 8, 10000.0, 0.19)
    assert l1.in_rows == 3 * (24 + 8) + 32 + 8 and l1.mix_out == 3 * 40
    assert (l1.ff_kind, l1.ff, l1.experts, l1.top, l1.shared_ff, l1.shared_gated, l1.ff_act, l1.router_kind,
            l1.router_biased) == (Ly.FF_MOE, 40, 6, 2, 24, False, Ly.ACT_SILU, Ly.ROUTER_TOP_SOFTMAX, True)
    assert (a2.top, a2.shared_ff, a2.kv_heads) == (1, 0, 6)
    assert (l3.rot_dim, l3.rot_dims, l3.rot_base, l3.mask_size, l3.ff_kind) == (16, 8, 500.0, 1, Ly.FF_NONE)
    assert c.layers[7].limit == 0.75 and c.layers[8].top == 5


def test_mirorax_loops_unroll():
    assert Ly.unroll_loop([0] * 3, None) == [(0, None), (1, None), (2, None)]
    assert Ly.unroll_loop([0] * 3, {"start": 0, "stop": 3, "times": 1}) == [(0, 0), (1, None), (2, None)]
    assert Ly.unroll_loop([0] * 4, {"start": 1, "stop": 3, "times": 3}) == [
        (0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None)]
    assert Ly.unroll_loop([0] * 2, {"start": 1, "stop": 2, "times": 2}) == [(0, None), (1, 0), (1, 1)]
    with pytest.raises(ValueError):
        Ly.unroll_loop([0] * 2, {"start": 1, "stop": 3, "times": 2})
    import mirorax_cases as MC
    import mirorax_ref as MR

    for cfg in MC.ALL.values():
        assert MR.layer_runs(cfg) == Ly.unroll_loop(cfg["layers"], cfg.get("loop"))


def test_mirorax_unknown_names_are_refused():
    import mirorax_cases as MC

    with pytest.raises(ValueError):
        Ly.mirorax_config(MC.config([("attention_2", MC.attn(), None)]))
    with pytest.raises(ValueError):
        Ly.mirorax_config(MC.config([("attention", MC.attn(), {"kind": "plain", "ff": 8})]))


def test_mirorax_pack_concatenates_and_shares_repeated_runs():
    import mirorax_cases as MC

    cfg = MC.MIXED
    t = Ly.mirorax_random_tensors(cfg, seed=3)
    assert set(t) == set(Ly.mirorax_tensor_shapes(cfg))
    for wdt in (M.F32, M.BF16):
        c = Ly.mirorax_config(cfg, weight_dtype=wdt)
        p = Ly.mirorax_pack(c, t, cfg)
        f = (lambda a: a) if wdt == M.F32 else Ly.bf16_to_f32
        assert len(p["layers"]) == 9 and p["head"] is not p["embed"]
        d0, l0 = p["layers"][0], c.layers[0]
        assert np.array_equal(f(d0["w_in"]), np.concatenate([t["l0.mix." + n] for n in ("q", "k", "v", "g")]))
        nb = l0.in_rows - l0.heads * l0.vdim
        assert np.array_equal(d0["in_bias"][:nb], np.concatenate([t["l0.mix." + n + ".b"] for n in ("q", "k", "v")]))
        assert not d0["in_bias"][nb:].any() and np.array_equal(d0["o_bias"], t["l0.mix.o.b"])
        assert np.array_equal(d0["ls1"], t["l0.ls1"]) and np.array_equal(d0["ls2"], t["l0.ls2"]) and "pre_add" not in d0
        d1, l1 = p["layers"][1], c.layers[1]
        assert np.array_equal(f(d1["w_in"]), np.concatenate([t["l1.mix.q"], t["l1.mix.dkv"]]))
        uk = t["l1.mix.uk"].reshape(l1.heads, l1.dim, l1.kv_rank)
        assert np.array_equal(f(d1["w_ukt"]), uk.transpose(0, 2, 1))
        assert np.array_equal(f(d1["w_ukv"]), np.concatenate([t["l1.mix.uk"], t["l1.mix.uv"]])) and "w_uv" not in d1
        assert np.array_equal(d1["sink_w"], t["l1.mix.sink"]) and np.array_equal(d1["router_bias"], t["l1.mlp.router.b"])
        assert np.array_equal(f(d1["w_gate"][4]), t["l1.mlp.e4.gate"]) and "shared_sg" not in d1
        # the loop: pass t of layers 1..3 adds step[t] before layer 1; later passes hold the first pass's arrays
        assert np.array_equal(d1["pre_add"], t["loop.step"][0]) and np.array_equal(p["layers"][4]["pre_add"], t["loop.step"][1])
        for r, first in ((4, 1), (5, 2), (6, 3)):
            for k, a in p["layers"][r].items():
                assert k == "pre_add" or a is p["layers"][first][k]
        assert "pre_add" not in p["layers"][5] and "ls2" not in p["layers"][3]
        for l, d in zip(c.layers, p["layers"]):
            own = set(Ly.packed_shapes(c, l))
            assert own <= set(d) and (l.shares >= 0 or own == set(d))


def test_mirorax_restatement_is_causal_and_its_window_and_sink_hold():
    """The restatement itself: logits at t do not depend on later tokens; a one-layer latent
    model's logits at t do not depend on tokens its window has left behind; the sink takes
    its share of the softmax."""
    import mirorax_cases as MC
    import mirorax_ref as MR

    cfg = MC.MIXED
    w = {k: v.astype(np.float64) for k, v in Ly.mirorax_random_tensors(cfg, seed=4).items()}
    a = MC.tokens(cfg, 40, 1)
    b = list(a)
    b[30] = (b[30] + 1) % cfg["vocab"]
    ra, rb = MR.forward(cfg, w, a), MR.forward(cfg, w, b)
    assert np.array_equal(ra[:30], rb[:30]) and not np.allclose(ra[30], rb[30])
    one = MC.ONLY_LATENT
    size = one["layers"][0]["mixer"]["mask"]["size"]
    w1 = {k: v.astype(np.float64) for k, v in Ly.mirorax_random_tensors(one, seed=5).items()}
    a = MC.tokens(one, 30, 2)
    b = list(a)
    b[10] = (b[10] + 1) % one["vocab"]
    ra, rb = MR.forward(one, w1, a), MR.forward(one, w1, b)
    assert not np.allclose(ra[10 + size - 1], rb[10 + size - 1]) and np.allclose(ra[10 + size:], rb[10 + size:], atol=1e-12)
    m = MR.visible(3, 6)
    assert m[5, 3] and not m[5, 2] and m[2, 0] and not m[2, 3]
    p = MR.softmax_rows(np.zeros((1, 1, 3)), np.array([[[True, True, False]]]), sink=np.array([np.log(2.0)]))
    assert np.allclose(p, [[[0.25, 0.25, 0.0]]])
    idx, wt = MR.route({"r.router": np.eye(4), "r.router.b": np.array([0.0, 0.0, 5.0, 0.0])}, "r.",
                       np.array([[3.0, 1.0, 0.0, 2.0]]), 2)
    assert idx.tolist() == [[2, 0]] and np.allclose(wt, [[np.exp(2) / (1 + np.exp(2)), 1 / (1 + np.exp(2))]])


def test_bench_stacks_are_valid_layer_list_configurations():
    """The stacks bench.py --layered times: every layer's packed tensor set is well formed at
    every benchmarked width, and mixed-score layers keep their key row within the MFMA
    attention kernel's key size."""
    import bench

    for width in (1024, 2048, 4096):
        for make in (bench.layered_stack, bench.lenuzen_stack, bench.mirorax_stack, bench.lifenex_stack):
            c = make(Ly, M, width, 2112)
            assert c.width == width and len(c.layers) == 6
            for l in c.layers:
                shapes = Ly.packed_shapes(c, l)
                if l.shares >= 0:  # a repeated run of a loop owns its pre_add only
                    assert set(shapes) <= {"pre_add"} and c.layers[l.shares].mixer == l.mixer
                    continue
                assert shapes["w_in"][0] == (l.in_rows, width) and shapes["w_o"][0] == (width, l.mix_out)
                if l.side is not None:
                    side = Ly.packed_shapes(c, l.side, side=True)
                    assert side["w_in"][0] == (l.side.in_rows, width) and "norm1" not in side and "join_w" in shapes
                if l.mixer == Ly.MIX_ATTN:
                    assert l.heads % l.kv_heads == 0 and l.rot_dims <= l.dim
                    if l.talking:
                        assert l.kv_heads * l.dim <= 512 and "talk" in shapes
    c = bench.lenuzen_stack(Ly, M, 2048, 2112)
    assert (c.norm_kind, c.pre_norm, c.pos_embed, c.tied_head) == (Ly.NORM_LAYER, False, False, True)


# ------------------------------------------------------------------ Lifenex
def test_lifenex_config_reads_every_size_and_constant():
    import lifenex_cases as LC

    cfg = LC.MIXED
    t = Ly.lifenex_random_tensors(cfg, seed=1, **LC.sizes(cfg))
    c = Ly.lifenex_config(cfg, max_tokens=99, weight_dtype=M.F32, shapes={k: v.shape for k, v in t.items()})
    assert (c.arch, c.width, c.vocab, c.max_tokens, c.weight_dtype) == ("Lifenex", 96, 211, 99, M.F32)
    assert (c.block_kind, c.pre_norm, c.pos_embed, c.tied_head, c.embed_normed) == (Ly.BLOCK_PARALLEL, True, False, True, True)
    assert c.logit_scale == 0.5 and c.norm_eps == 1e-5 and c.norm_kind == Ly.NORM_RMS
    s0, m0 = c.layers[0], cfg["layers"][0]["mixer"]
    assert (s0.mixer, s0.heads, s0.vdim, s0.ssm_state, s0.ssm_groups, s0.norm_groups, s0.conv) == (
        Ly.MIX_SSM, m0["heads"], m0["vdim"], m0["state"], m0["groups"], m0["norm_groups"], m0["conv"])
    assert (s0.ff_kind, s0.ff, s0.ff_act, s0.ff_normed, s0.layer_scaled) == (Ly.FF_PLAIN, 72, Ly.ACT_RELU2, True, False)
    s2, m2 = c.layers[2], cfg["layers"][2]["mixer"]
    a, d = m2["left"], m2["right"]
    assert (s2.mixer, s2.heads, s2.kv_heads, s2.dim, s2.vdim, s2.attn_scale) == (Ly.MIX_ATTN, 6, 6, 16, 16, a["scale"])
    assert (s2.qk_norm, s2.sink, s2.sink_learned, s2.mask_kind, s2.rot_dims) == (Ly.QK_HEAD_W, 1, True, Ly.MASK_CAUSAL, 0)
    assert (s2.q_temp_coef, s2.q_temp_every, s2.rel_max, s2.rel_rows, s2.join_scale) == (0.4, 1, 9.0, 8, 0.5)
    sd = s2.side
    assert (sd.mixer, sd.heads, sd.kv_heads, sd.dim, sd.vdim, sd.conv) == (Ly.MIX_DELTA, d["heads"], d["kv_heads"], d["dim"],
                                                                          d["vdim"], d["conv"])
    assert (sd.decay_rank, sd.gate_rank, sd.gate_act, sd.ff_kind) == (5, 12, Ly.DELTA_GATE_SIGMOID, Ly.FF_NONE)
    assert (s2.ff_kind, s2.experts, s2.top, s2.groups, s2.groups_keep, s2.shared_ff) == (Ly.FF_MOE, 4, 1, 1, 1, 0)
    s5 = c.layers[5]
    assert (s5.router_kind, s5.router_biased, s5.groups, s5.groups_keep, s5.shared_ff, s5.shared_gated, s5.ff_act) == (
        Ly.ROUTER_SIGMOID_GROUPS, True, 4, 2, 8, True, Ly.ACT_SILU)
    assert c.layers[3].ff_kind == Ly.FF_NONE and c.layers[3].side is None
    # rows of the concatenated input projections
    assert s0.in_rows == 2 * 3 * 16 + 2 * 1 * 24 + 3
    assert sd.in_rows == 2 * 2 * 24 + 2 * 8 + 12 + 2 + 5


def test_lifenex_unknown_names_are_refused():
    import lifenex_cases as LC

    bad = {**LC.ONLY_SSM, "layers": [{"type": "mamba3", "mixer": LC.ssm(), "mlp": None}]}
    with pytest.raises(ValueError):
        Ly.lifenex_config(bad)
    bad = {**LC.ONLY_DENSE, "layers": [{"type": "mamba2", "mixer": LC.ssm(), "mlp": {"kind": "glu", "ff": 8}}]}
    with pytest.raises(ValueError):
        Ly.lifenex_config(bad)
    with pytest.raises(ValueError):  # a pair's table and ranks are the tensors' own sizes
        Ly.lifenex_config(LC.ONLY_PAIR)


def test_lifenex_pack_concatenates_and_nests_the_second_mixer():
    import lifenex_cases as LC

    cfg = LC.MIXED
    t = Ly.lifenex_random_tensors(cfg, seed=3, **LC.sizes(cfg))
    assert set(t) == set(Ly.lifenex_tensor_shapes(cfg, **LC.sizes(cfg)))
    for wdt in (M.F32, M.BF16):
        c = Ly.lifenex_config(cfg, weight_dtype=wdt, shapes={k: v.shape for k, v in t.items()})
        p = Ly.lifenex_pack(c, t)
        f = (lambda a: a) if wdt == M.F32 else Ly.bf16_to_f32
        assert p["head"] is p["embed"] and np.array_equal(p["embed_norm"], t["embed.norm"])
        d0 = p["layers"][0]
        assert np.array_equal(f(d0["w_in"]), t["l0.mix.in"]) and np.array_equal(d0["d_skip"], t["l0.mix.D"])
        assert np.array_equal(d0["conv_b"], t["l0.mix.conv.b"]) and np.array_equal(d0["norm2"], t["l0.norm2"])
        assert "ls1" not in d0 and "side" not in d0 and "w_gate" not in d0
        d1 = p["layers"][1]
        assert np.array_equal(f(d1["w_in"]), np.concatenate([t["l1.mix.left." + n] for n in ("q", "k", "v")]))
        assert np.array_equal(d1["rel"], t["l1.mix.left.rel"]) and np.array_equal(d1["sink_w"], t["l1.mix.left.sink"])
        assert np.array_equal(d1["join_w"], t["l1.mix.left.out"]) and np.array_equal(d1["side_join_w"], t["l1.mix.right.out"])
        assert np.array_equal(d1["router_bias"], t["l1.mlp.correction"]) and d1["shared_sg"].shape == (cfg["width"],)
        assert np.array_equal(f(d1["w_up"][4]), t["l1.mlp.e4.up"])
        sd = d1["side"]
        assert np.array_equal(f(sd["w_in"]), np.concatenate([t["l1.mix.right." + n] for n in ("q", "k", "v", "g1", "b", "a1")]))
        assert np.array_equal(sd["conv_w"], np.concatenate([t["l1.mix.right." + n + ".conv"] for n in ("q", "k", "v")]))
        assert np.array_equal(f(sd["w_a2"]), t["l1.mix.right.a2"]) and np.array_equal(f(sd["w_g2"]), t["l1.mix.right.g2"])
        assert "norm1" not in sd and "norm2" not in p["layers"][3]
        for l, d in zip(c.layers, p["layers"]):
            assert set(Ly.packed_shapes(c, l)) == set(d) - {"side"}
            if l.side is not None:
                assert set(Ly.packed_shapes(c, l.side, side=True)) == set(d["side"])


def test_lifenex_restatement_mechanisms():
    """The restatement itself: causality; the distance buckets; the temperature's blocks; the sink's
    share; the router's groups (ranked by their two best, forbidden experts behind every allowed
    one even when all choice scores are negative), its correction and its weights."""
    import lifenex_cases as LC
    import lifenex_ref as LR

    cfg = LC.MIXED
    w = {k: v.astype(np.float64) for k, v in Ly.lifenex_random_tensors(cfg, seed=4, **LC.sizes(cfg)).items()}
    a = LC.tokens(cfg, 40, 1)
    b = list(a)
    b[30] = (b[30] + 1) % cfg["vocab"]
    ra, rb = LR.forward(cfg, w, a), LR.forward(cfg, w, b)
    assert np.array_equal(ra[:30], rb[:30]) and not np.allclose(ra[30], rb[30])
    assert not np.allclose(ra[39], rb[39])  # and the change is carried on (states, keys)
    # 8 rows reaching 64 back: exact below 4, then 4 logarithmic rows up to 64, the last row beyond
    bk = LR.distance_bucket(np.arange(200), 8, 64.0)
    assert bk[:4].tolist() == [0, 1, 2, 3] and bk[4] == 4 and bk[7] == 4 and bk[8] == 5 and bk[15] == 5 and bk[16] == 6
    assert bk[31] == 6 and bk[32] == 7 and bk[63] == 7 and bk[64] == 7 and bk[199] == 7 and (np.diff(bk) >= 0).all()
    tq = LR.query_temperature(np.array([0, 6, 7, 14, 20]), 0.5, 7)
    assert np.allclose(tq, [1.0, 1.0 + 0.5 * np.log(2), 1.0 + 0.5 * np.log(2), 1.0 + 0.5 * np.log(3), 1.0 + 0.5 * np.log(4)])
    p = LR.softmax_sink(np.array([[0.0, 0.0, -np.inf]]), np.log(2.0))
    assert np.allclose(p, [[0.25, 0.25, 0.0]])
    # two groups of three: group 1 wins by the sum of its two best although group 0 holds the best expert
    z = np.array([3.0, -9.0, -9.0, 2.0, 2.0, -9.0])
    idx, wt = LR.route(z, np.zeros(6), 2, 2, 1)
    assert sorted(idx.tolist()) == [3, 4] and np.allclose(wt, LR.sigmoid(2.0))
    # the correction moves the choice, not the weights; negative choice scores keep forbidden experts out
    idx, wt = LR.route(z, np.array([0.0, 0.0, 0.0, 0.0, -5.0, 1.2]) - 10.0, 2, 2, 1)
    assert idx.tolist() == [5, 3] and np.allclose(wt, [LR.sigmoid(-9.0), LR.sigmoid(2.0)])
    g = LR.grouped_rms(np.array([[3.0, 4.0, 0.0, 5.0]]), 2, np.ones(4), 0.0)
    assert np.allclose(g, [[3 / np.sqrt(12.5), 4 / np.sqrt(12.5), 0.0, np.sqrt(2.0)]])
    y = LR.causal_conv(np.array([[1.0], [2.0], [3.0]]), np.array([[10.0, 1.0]]), np.array([0.5]))
    assert np.allclose(y[:, 0], [1.5, 12.5, 23.5])
