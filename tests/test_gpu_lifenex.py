"""MI355X: the layer-list engine serving Lifenex models against the plain float64 restatement
in tests/lifenex_ref.py, on small random models made here.

Errors are per position: || got - ref || / || ref || over the vocabulary. With f32 matrices
the engine differs from the restatement by f32 rounding only (F32_TOL); with bf16 matrices by
the rounding of the products' inputs and of the cached keys and values (BF16_TOL; a model with
routed experts may miss it at a few positions where that rounding flips a router near-tie). A
lost key, a distance bucket or temperature block one position off, a missing sink, a state that
is not carried or a token one place off moves the logits by orders of magnitude more than
F32_TOL; the edge tests show that on their own models before they trust it.
"""
import copy
import dataclasses
import json
import os
import subprocess

import numpy as np
import pytest

import lifenex_cases as C
import lifenex_ref as R

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_TOL, BF16_TOL = 2e-4, 6e-2


@pytest.fixture(scope="module")
def rt():
    from yalm_amd import runtime

    runtime.check(runtime.lib.yalm_set_device(0))
    return runtime


def make(cfg, seed=0, tensors=None, sizes=None):
    from yalm_amd import layered as Ly

    return tensors if tensors is not None else Ly.lifenex_random_tensors(cfg, seed=seed, **(sizes or C.sizes(cfg)))


def build(rt, cfg, wdt, seed=0, max_tokens=512, tensors=None, sizes=None):
    from yalm_amd import layered as Ly

    t = make(cfg, seed, tensors, sizes)
    c = Ly.lifenex_config(cfg, max_tokens=max_tokens, weight_dtype=wdt, shapes={k: v.shape for k, v in t.items()})
    model = rt.SeqModel.from_packed(c, Ly.lifenex_pack(c, t))
    return model, rt.SeqDecoder(model), {k: v.astype(np.float64) for k, v in t.items()}


def rel_err(got, ref):
    return np.linalg.norm(got - ref, axis=-1) / np.linalg.norm(ref, axis=-1)


def wdt_of(dtype):
    from yalm_amd import models as M

    return M.F32 if dtype == "f32" else M.BF16


def routed(cfg):
    return any((e.get("mlp") or {}).get("kind") == "moe" for e in cfg["layers"])


def agrees(got, ref, dtype, cfg):
    e = rel_err(got, ref)
    if dtype == "f32":
        return e.max() < F32_TOL
    if routed(cfg):  # a flipped near-tie of a router: a few positions, never the bulk
        return np.mean(e > BF16_TOL) <= 0.1 and np.median(e) < BF16_TOL / 3
    return e.max() < BF16_TOL


def run_portions(dec, tok, sizes):
    """Feed tok in portions of the given sizes (the last one takes the rest), asking for
    every position's logits."""
    out, at = [], 0
    for s in list(sizes) + [len(tok)]:
        s = min(s, len(tok) - at)
        if s <= 0:
            break
        out.append(dec.step(tok[at:at + s], list(range(s))))
        at += s
    return np.concatenate(out)


ALONE = {k: C.ALL[k] for k in ("only_ssm", "only_pair", "only_dense", "only_moe")}


@pytest.mark.parametrize("name", sorted(ALONE))
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_each_layer_kind_alone(rt, name, dtype):
    cfg = ALONE[name]
    model, dec, w = build(rt, cfg, wdt_of(dtype), seed=1)
    try:
        tok = C.tokens(cfg, 70, 1)
        ref = R.forward(cfg, w, tok)
        assert agrees(dec.step(tok, list(range(len(tok)))), ref, dtype, cfg)
        dec.reset()
        assert agrees(run_portions(dec, tok, [30] + [1] * 40), ref, dtype, cfg)
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("which", ["left", "right"])
def test_each_mixer_of_a_pair_alone(rt, which):
    """The two mixers of a pair are ordinary mixers of the engine: a one-layer stack put together
    by hand with the attention alone, or the delta rule alone (no second mixer, no join), against
    that mechanism's restatement."""
    from yalm_amd import layered as Ly
    from yalm_amd import models as M

    cfg = C.ONLY_PAIR
    t = make(cfg, 31)
    w = {k: v.astype(np.float64) for k, v in t.items()}
    c = Ly.lifenex_config(cfg, max_tokens=256, weight_dtype=M.F32, shapes={k: v.shape for k, v in t.items()})
    p = Ly.lifenex_pack(c, t)
    d, l = p["layers"][0], c.layers[0]
    if which == "left":
        spec = dataclasses.replace(l, side=None)
        pd = {k: v for k, v in d.items() if k not in ("side", "join_w", "side_join_w")}
    else:
        spec = dataclasses.replace(l.side, ff_normed=True, layer_scaled=False)
        pd = dict(d["side"], norm1=d["norm1"])
    c1 = c.with_(layers=[spec])
    assert set(pd) == set(Ly.packed_shapes(c1, spec))
    model = rt.SeqModel.from_packed(c1, dict(p, layers=[pd]))
    dec = rt.SeqDecoder(model)
    try:
        tok = C.tokens(cfg, 90, 31)
        eps, m = cfg["norm"]["eps"], cfg["layers"][0]["mixer"]
        x = R.rms_norm(w["embed"][tok], w["embed.norm"], eps)
        h = R.rms_norm(x, w["l0.norm1"], eps)
        x = x + (R.mixer_attention(cfg, w, "l0.mix.left.", h, m["left"]) if which == "left"
                 else R.mixer_delta(cfg, w, "l0.mix.right.", h, m["right"]))
        ref = R.rms_norm(x, w["final.norm"], eps) @ w["embed"].T * cfg["logit_scale"]
        for sizes in ([90], [40] + [1] * 50, [2, 9, 3, 8, 33]):
            dec.reset()
            assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_pair_in_serial_blocks(rt):
    """Two mixers side by side are a mechanism of the engine, not of one design: the same pair in
    the OTHER envelope (serial blocks, a closing norm after the sublayer), put together by hand;
    the join is then a launch of its own instead of a part of the parallel block's seam."""
    from yalm_amd import layered as Ly
    from yalm_amd import models as M

    cfg = C.ONLY_PAIR
    t = make(cfg, 33)
    w = {k: v.astype(np.float64) for k, v in t.items()}
    c = Ly.lifenex_config(cfg, max_tokens=256, weight_dtype=M.F32, shapes={k: v.shape for k, v in t.items()})
    p = Ly.lifenex_pack(c, t)
    closing = (1.0 + 0.1 * np.arange(cfg["width"]) / cfg["width"]).astype(np.float32)
    spec = dataclasses.replace(c.layers[0], ff_normed=False)
    c1 = c.with_(layers=[spec], block_kind=Ly.BLOCK_SERIAL)
    pd = dict(p["layers"][0], norm1b=closing)
    assert set(pd) - {"side"} == set(Ly.packed_shapes(c1, spec))
    model = rt.SeqModel.from_packed(c1, dict(p, layers=[pd]))
    dec = rt.SeqDecoder(model)
    try:
        tok = C.tokens(cfg, 80, 33)
        eps = cfg["norm"]["eps"]
        x = R.rms_norm(w["embed"][tok], w["embed.norm"], eps)
        y = R.mixer_pair(cfg, w, "l0.mix.", R.rms_norm(x, w["l0.norm1"], eps), cfg["layers"][0]["mixer"])
        x = x + R.rms_norm(y, closing.astype(np.float64), eps)
        ref = R.rms_norm(x, w["final.norm"], eps) @ w["embed"].T * cfg["logit_scale"]
        for sizes in ([80], [30] + [1] * 50, [2, 9, 3, 8, 33]):
            dec.reset()
            assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("name", ["mixed", "odd", "wide", "dense_only"])
def test_residual_stream_after_every_layer(rt, name):
    from yalm_amd import models as M

    cfg = C.ALL[name]
    model, dec, w = build(rt, cfg, M.F32, seed=2)
    try:
        tok = C.tokens(cfg, 57, 2)
        layers = []
        R.forward(cfg, w, tok, layers_out=layers)
        assert len(layers) == len(model.cfg.layers) == len(cfg["layers"])
        dec.layer_dump(True)
        dec.step(tok)
        got = dec.get_layers(len(tok))
        for i, ref in enumerate(layers):
            e = np.abs(got[i] - ref).max() / np.abs(ref).max()
            assert e < 1e-4, f"layer {i}: {e}"
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("name", ["mixed", "odd", "wide", "dense_only"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prefill_then_token_by_token(rt, name, dtype):
    """A prompt in one step, then single tokens through the caches and states: temperature blocks
    and distance buckets pass over decoded tokens, long prompts take the portion kernels."""
    cfg = C.ALL[name]
    model, dec, w = build(rt, cfg, wdt_of(dtype), seed=3, max_tokens=700)
    try:
        n = 420 if name in ("wide", "dense_only") else 150
        tok = C.tokens(cfg, n, 3)
        ref = R.forward(cfg, w, tok)
        assert agrees(run_portions(dec, tok, [n - 60] + [1] * 60), ref, dtype, cfg)
        dec.reset()
        assert agrees(dec.step(tok, list(range(n))), ref, dtype, cfg)
    finally:
        dec.close()
        model.close()


PORTIONS = [[2] * 30, [3, 2, 9, 8, 2, 64, 65], [1, 2, 3, 4, 5, 6, 7, 8, 9, 10], [128, 2, 2, 1, 40], [7, 200]]


@pytest.mark.parametrize("name", ["mixed", "odd", "wide"])
@pytest.mark.parametrize("sizes", PORTIONS, ids=[str(i) for i in range(len(PORTIONS))])
def test_portions_of_any_size(rt, name, sizes):
    """Portions cut anywhere (inside convolution windows, recurrence chunks and temperature
    blocks, down to two tokens) against the whole sequence; the GEMV / tile switch (8 | 9 tokens)
    and tile edges (64 | 65) included."""
    from yalm_amd import models as M

    cfg = C.ALL[name]
    model, dec, w = build(rt, cfg, M.F32, seed=4)
    try:
        tok = C.tokens(cfg, 260, 4)
        ref = R.forward(cfg, w, tok)
        assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_portions_bf16_differ_by_rounding_only(rt):
    from yalm_amd import models as M

    cfg = C.DENSE_ONLY
    model, dec, w = build(rt, cfg, M.BF16, seed=5, max_tokens=700)
    try:
        tok = C.tokens(cfg, 600, 5)
        ref = R.forward(cfg, w, tok)
        for sizes in ([600], [300, 2, 170, 1, 1, 1], [64] * 9):
            dec.reset()
            assert rel_err(run_portions(dec, tok, sizes), ref).max() < BF16_TOL
    finally:
        dec.close()
        model.close()


def test_decoder_reused_after_reset(rt):
    """States and cache rows of an ended sequence must not leak into the next one: the second
    sequence on a reused decoder equals the same sequence on a fresh decoder bit for bit."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=8)
    fresh = rt.SeqDecoder(model)
    try:
        a, b = C.tokens(cfg, 90, 6), C.tokens(cfg, 41, 7)
        run_portions(dec, a, [50, 1, 1, 38])
        dec.reset()
        assert dec.pos == 0
        got = run_portions(dec, b, [20, 1, 20])
        want = run_portions(fresh, b, [20, 1, 20])
        assert np.array_equal(got, want)
        assert rel_err(got, R.forward(cfg, w, b)).max() < F32_TOL
    finally:
        dec.close()
        fresh.close()
        model.close()


def test_two_live_sequences_do_not_mix(rt):
    """Two decoders on one model, unequal requests, their steps interleaved: each equals its
    sequence alone."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, d1, w = build(rt, cfg, M.F32, seed=20)
    d2 = rt.SeqDecoder(model)
    try:
        a, b = C.tokens(cfg, 60, 20), C.tokens(cfg, 45, 21)
        ga, gb, ia, ib = [], [], 0, 0
        for sa, sb in ((20, 3), (1, 30), (9, 1), (30, 11)):
            ga.append(d1.step(a[ia:ia + sa], list(range(sa))))
            gb.append(d2.step(b[ib:ib + sb], list(range(sb))))
            ia, ib = ia + sa, ib + sb
        assert rel_err(np.concatenate(ga), R.forward(cfg, w, a)).max() < F32_TOL
        assert rel_err(np.concatenate(gb), R.forward(cfg, w, b)).max() < F32_TOL
    finally:
        d1.close()
        d2.close()
        model.close()


def _peaked(cfg, tensors, scale=6.0):
    """Queries of the pair's attention scaled up so that single keys decide positions."""
    t = dict(tensors)
    t["l0.mix.left.q.norm"] = t["l0.mix.left.q.norm"] * scale
    return t


EDGE = C.config(
    [(C.P, C.pair(C.attn(heads=2, kv_heads=1, dim=16, vdim=24, scale=0.4, bias_max=48, coef=0.9, every=11),
                  C.delta(heads=2, kv_heads=1, dim=8, vdim=8, conv=2)), None)],
    width=64, vocab=101, sizes={"rel_rows": 10, "decay_rank": 4, "gate_rank": 4})
FAR = C.config(
    [(C.P, C.pair(C.attn(heads=2, kv_heads=1, dim=16, vdim=24, scale=0.4, bias_max=900, coef=0.2, every=100),
                  C.delta(heads=2, kv_heads=1, dim=8, vdim=8, conv=2)), None)],
    width=64, vocab=101, sizes={"rel_rows": 10, "decay_rank": 4, "gate_rank": 4})


@pytest.mark.parametrize("what", ["bucket", "block"])
def test_edges_of_distance_buckets_and_temperature_blocks(rt, what):
    """The restatement with the distance table's far end (which moves every logarithmic bucket's
    edge) or the temperature's block length one position off names the positions where the key
    just inside / just outside a bucket, or the first token of a block, decides the logits (they
    differ there by far more than the tolerance); the engine must agree with the true constants
    at all of them, with the query in a prompt's portion and decoded alone."""
    from yalm_amd import models as M

    cfg = EDGE
    t = make(cfg, 9)
    t["l0.mix.left.rel"] = t["l0.mix.left.rel"] * 4.0  # neighbouring buckets far apart
    t = _peaked(cfg, t, 3.0)
    model, dec, w = build(rt, cfg, M.F32, tensors=t)
    try:
        tok = C.tokens(cfg, 240, 8)
        ref = R.forward(cfg, w, tok)
        for delta in (-1, +1):
            off = copy.deepcopy(cfg)
            left = off["layers"][0]["mixer"]["left"]
            if what == "bucket":
                left["bias_max"] += 3 * delta
            else:
                left["q_temp"]["every"] += delta
            assert (rel_err(R.forward(off, w, tok), ref) > 100 * F32_TOL).sum() >= 5
        for sizes in ([240], [100] + [1] * 140, [61, 2, 50, 2, 2, 93]):
            dec.reset()
            assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_far_keys_decide_the_output(rt):
    """The restatement's own softmax weights name late queries whose winning key lies more than
    250 positions back; changing THAT token must move the query's logits, and the engine must
    follow, in a prompt's portion and decoded alone."""
    from yalm_amd import models as M

    cfg = FAR
    t = _peaked(cfg, make(cfg, 10), 8.0)
    model, dec, w = build(rt, cfg, M.F32, max_tokens=600, tensors=t)
    try:
        a = C.tokens(cfg, 500, 9)
        P = []
        ra = R.forward(cfg, w, a, weights_out=P)
        far = [(P[h][t_].max(), t_, int(P[h][t_].argmax())) for h in range(2) for t_ in range(340, 500)
               if t_ - int(P[h][t_].argmax()) >= 250]
        assert far, "no late query with a far winning key: pick another seed"
        weight, tq, j = max(far)
        assert weight > 0.3
        b = list(a)
        b[j] = (b[j] + 17) % cfg["vocab"]
        rb = R.forward(cfg, w, b)
        assert rel_err(ra[tq], rb[tq]) > 100 * F32_TOL
        for tok, ref in ((a, ra), (b, rb)):
            for sizes in ([490], [tq] + [1] * 5):
                dec.reset()
                assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_recurrent_states_carry_far(rt):
    """A token hundreds of positions back still shows in the logits through the recurrent states
    (slow decays), across portion cuts and single-token steps."""
    from yalm_amd import models as M

    cfg = C.config([(C.S, C.ssm(heads=2, vdim=8, state=16, groups=1, norm_groups=1, conv=2), None),
                    (C.P, C.pair(C.attn(heads=1, kv_heads=1, dim=8, vdim=8, scale=0.3, bias_max=20, every=50),
                                 C.delta(heads=2, kv_heads=1, dim=16, vdim=8, conv=2)), None)], width=32, vocab=53)
    t = make(cfg, 12)
    t["l0.mix.A_log"] = np.full_like(t["l0.mix.A_log"], -6.0)          # decays close to one
    t["l1.mix.right.A_log"] = np.full_like(t["l1.mix.right.A_log"], -7.0)
    t["l1.mix.left.v"] = np.zeros_like(t["l1.mix.left.v"])             # the attention carries nothing
    model, dec, w = build(rt, cfg, M.F32, max_tokens=400, tensors=t)
    try:
        a = C.tokens(cfg, 330, 12)
        b = list(a)
        b[3] = (b[3] + 5) % cfg["vocab"]
        ra, rb = R.forward(cfg, w, a), R.forward(cfg, w, b)
        assert rel_err(ra[300:], rb[300:]).min() > 20 * F32_TOL
        for tok, ref in ((a, ra), (b, rb)):
            for sizes in ([330], [2, 100, 17, 150] + [1] * 61):
                dec.reset()
                assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_every_mechanism_shows_in_the_logits(rt):
    """Taking one mechanism out of the restatement moves it far beyond the tolerance: the engine
    agreeing with the whole restatement means it computes each."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=11)
    try:
        tok = C.tokens(cfg, 40, 10)
        ref = R.forward(cfg, w, tok)

        def without(**changed):
            return rel_err(R.forward(cfg, {**w, **changed}, tok), ref).max()

        def other(path, value):
            c = copy.deepcopy(cfg)
            node = c
            for k in path[:-1]:
                node = node[k]
            node[path[-1]] = value
            return rel_err(R.forward(c, w, tok), ref).max()

        big = 100 * F32_TOL
        for name in ("embed.norm", "l1.norm2", "l1.mix.left.out", "l1.mix.right.out", "l1.mix.left.q.norm",
                     "l1.mix.left.k.norm", "l0.mix.norm", "l1.mix.right.norm"):
            assert without(**{name: np.ones_like(w[name])}) > big, name
        for name in ("l1.mix.left.rel", "l1.mlp.correction", "l0.mix.conv.b", "l0.mix.D", "l1.mix.right.a2",
                     "l1.mix.right.g2", "l1.mix.right.b", "l1.mlp.shared.sg", "l0.mix.dt_bias", "l1.mix.right.dt_bias"):
            assert without(**{name: np.zeros_like(w[name])}) > big, name
        assert without(**{"l1.mix.left.sink": w["l1.mix.left.sink"] - 30.0}) > big
        assert without(**{"l0.mix.A_log": w["l0.mix.A_log"] + 1.0}) > big
        assert without(**{"l1.mix.right.A_log": w["l1.mix.right.A_log"] + 1.0}) > big
        assert other(["layers", 1, "mixer", "left", "q_temp", "coef"], 0.0) > big
        assert other(["layers", 0, "mixer", "norm_groups"], 1) > big
        assert other(["layers", 5, "mlp", "router", "groups"], {"count": 1, "keep": 1}) > big
        assert other(["logit_scale"], 1.0) > big
        keep = R.mixer_pair
        try:  # the halving of the pair's sum
            R.mixer_pair = lambda *a, **k: 2.0 * keep(*a, **k)
            assert rel_err(R.forward(cfg, w, tok), ref).max() > big
        finally:
            R.mixer_pair = keep
        assert rel_err(dec.step(tok, list(range(40))), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_routed_experts_follow_the_restatement(rt):
    """Every token's chosen experts and weights, through the logits: a one-layer model whose
    feed-forward is all the model does beyond a tiny mixer; groups that forbid the best single
    expert, negative choice scores, top = 1, top = all experts, no shared expert."""
    from yalm_amd import models as M

    for k, mlp in enumerate((C.moe(), C.moe(experts=5, top=1, ff=24, shared=0, count=1, keep=1),
                             C.moe(experts=4, top=4, ff=16, shared=8, count=2, keep=2),
                             C.moe(experts=12, top=3, ff=8, shared=0, count=4, keep=1))):
        cfg = C.config([(C.S, C.TINY, mlp)], width=48, vocab=77)
        t = make(cfg, 21 + k)
        if k == 3:  # every choice score below zero: a forbidden expert must stay behind them all
            t["l0.mlp.correction"] = t["l0.mlp.correction"] - 3.0
        model, dec, w = build(rt, cfg, M.F32, tensors=t)
        try:
            tok = C.tokens(cfg, 50, 21)
            picks = []
            ref = R.forward(cfg, w, tok, choice_out=picks)
            assert len({tuple(sorted(i.tolist())) for i, _ in picks}) > 1 or mlp["router"]["top"] == mlp["router"]["experts"]
            if k == 3:  # the groups matter: without them other experts would have won somewhere
                free = copy.deepcopy(cfg)
                free["layers"][0]["mlp"]["router"]["groups"] = {"count": 1, "keep": 1}
                assert rel_err(R.forward(free, w, tok), ref).max() > 100 * F32_TOL
            assert rel_err(run_portions(dec, tok, [20, 5, 1, 1]), ref).max() < F32_TOL
        finally:
            dec.close()
            model.close()


@pytest.mark.parametrize("n", [1, 2, 3, 5])
def test_first_tokens(rt, n):
    """Sequences shorter than the convolutions, the first temperature block, distance 0 only."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=12)
    try:
        tok = C.tokens(cfg, n, 9)
        ref = R.forward(cfg, w, tok)
        assert rel_err(dec.step(tok, list(range(n))), ref).max() < F32_TOL
        dec.reset()
        assert rel_err(run_portions(dec, tok, [1] * n), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("name", ["odd", "mixed"])
def test_long_decoding(rt, name):
    """200 single tokens: every temperature block and distance bucket of the model passes over
    decoded tokens, the states are carried through 200 steps."""
    from yalm_amd import models as M

    cfg = C.ALL[name]
    model, dec, w = build(rt, cfg, M.F32, seed=13)
    try:
        tok = C.tokens(cfg, 5 + 200, 10)
        got = run_portions(dec, tok, [5] + [1] * 200)
        assert rel_err(got, R.forward(cfg, w, tok)).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_greedy_generation(rt):
    """The device greedy loop (no host round trip) picks the restatement's tokens, and the
    sequence can be continued by ordinary steps afterwards."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=14)
    try:
        prompt = C.tokens(cfg, 12, 11)
        dec.step(prompt[:-1])
        gen = dec.generate_greedy(prompt[-1], 40)
        seq = list(prompt)
        for g in gen:
            lg = R.forward(cfg, w, seq)[-1]
            top2 = np.sort(lg)[-2:]
            assert top2[1] - top2[0] > 1e-3, "the test's model has a near tie; pick another seed"
            assert int(np.argmax(lg)) == g
            seq.append(g)
        assert dec.pos == len(prompt) - 1 + len(gen)
        nxt = dec.step([gen[-1]], [0])
        assert rel_err(nxt, R.forward(cfg, w, seq)[-1:]).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_greedy_graph_replays_match_eager_steps(rt):
    """The greedy loop replays one captured token graph. Several generate calls with ordinary
    (eager) steps and synchronisations between them: every replayed token equals the argmax of
    an eager step of a second decoder fed the same tokens."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.BF16, seed=15)
    eager = rt.SeqDecoder(model)
    try:
        prompt = C.tokens(cfg, 9, 16)
        dec.step(prompt[:-1])
        eager.step(prompt[:-1])
        tok = prompt[-1]
        for n in (3, 1, 6, 2):
            gen = dec.generate_greedy(tok, n)
            for g in gen:
                lg = eager.step([tok], [0])[0]
                assert int(np.argmax(lg)) == g
                tok = g
            extra = C.tokens(cfg, 2, 17 + n)
            a = dec.step(extra, [1])
            b = eager.step(extra, [1])
            assert np.array_equal(a, b)
            tok = int(np.argmax(a[0]))
        assert dec.pos == eager.pos
    finally:
        dec.close()
        eager.close()
        model.close()


_LONG_REF = {}


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prompt_longer_than_one_internal_portion(rt, dtype):
    """A step of more tokens than the engine's work buffers hold (4096) is cut inside the engine,
    in the middle of a convolution window, a recurrence chunk and a temperature block; asked rows
    on both sides of the cut come back in order."""
    cfg = C.config([(C.S, C.ssm(heads=2, vdim=8, state=8, groups=1, norm_groups=2, conv=4), None),
                    (C.P, C.pair(C.attn(heads=2, kv_heads=1, dim=8, vdim=8, scale=0.35, bias_max=3000, every=777),
                                 C.delta(heads=2, kv_heads=2, dim=8, vdim=8, conv=3)), None)], width=32, vocab=53)
    model, dec, w = build(rt, cfg, wdt_of(dtype), seed=16, max_tokens=4300)
    try:
        tok = C.tokens(cfg, 4200, 15)
        want = [0, 5, 3999, 4000, 4094, 4095, 4096, 4097, 4150, 4199]
        got = dec.step(tok, want)
        assert dec.pos == len(tok)
        if "ref" not in _LONG_REF:  # the same weights and tokens for both matrix types
            _LONG_REF["ref"] = R.forward(cfg, w, tok)[want]
        assert rel_err(got, _LONG_REF["ref"]).max() < (F32_TOL if dtype == "f32" else BF16_TOL)
    finally:
        dec.close()
        model.close()


LARGE = {
    # the largest head sizes the kernels take: a state of 256 rows, keys of 256 entries
    "state256": [(C.S, C.ssm(heads=2, vdim=64, state=256, groups=1, norm_groups=2, conv=4), C.dense(ff=64))],
    "dim256": [(C.P, C.pair(C.attn(heads=4, kv_heads=2, dim=256, vdim=128, scale=0.06, bias_max=200, every=64),
                            C.delta(heads=2, kv_heads=1, dim=256, vdim=64, conv=4)), C.dense(ff=64))],
}


@pytest.mark.parametrize("name", sorted(LARGE))
def test_large_head_sizes(rt, name):
    cfg = C.config(LARGE[name], width=128, vocab=101, sizes={"rel_rows": 32, "decay_rank": 16, "gate_rank": 16})
    for dtype in ("f32", "bf16"):
        model, dec, w = build(rt, cfg, wdt_of(dtype), seed=22, max_tokens=400)
        try:
            tok = C.tokens(cfg, 330, 22)
            ref = R.forward(cfg, w, tok)
            assert agrees(run_portions(dec, tok, [270, 5, 2, 20, 9] + [1] * 24), ref, dtype, cfg)
        finally:
            dec.close()
            model.close()


def test_stream_wider_than_the_register_seam(rt):
    """A width above 4096 takes the seam kernel that keeps the row in LDS (join of the pair, experts'
    combine, both opening norms) and the embedding / norm kernels' strided loops."""
    from yalm_amd import models as M

    cfg = C.config([(C.P, C.pair(C.attn(heads=2, kv_heads=1, dim=16, vdim=8, scale=0.25, bias_max=20, every=8),
                                 C.delta(heads=2, kv_heads=1, dim=8, vdim=8, conv=2)), C.moe(experts=4, top=2, ff=8, shared=8, count=2, keep=1)),
                    (C.S, C.ssm(heads=2, vdim=8, state=8, groups=1, norm_groups=2, conv=2), C.dense(ff=16))],
                   width=4104, vocab=41, sizes={"rel_rows": 6, "decay_rank": 2, "gate_rank": 2})
    model, dec, w = build(rt, cfg, M.F32, seed=23, max_tokens=64)
    try:
        tok = C.tokens(cfg, 40, 23)
        ref = R.forward(cfg, w, tok)
        assert rel_err(run_portions(dec, tok, [12, 3, 9] + [1] * 16), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_sequence_cannot_pass_max_tokens(rt):
    from yalm_amd import models as M

    model, dec, _ = build(rt, C.ONLY_PAIR, M.F32, seed=13, max_tokens=16)
    try:
        dec.step(C.tokens(C.ONLY_PAIR, 16, 0))
        with pytest.raises(rt.YalmError):
            dec.step([1])
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner(rt, tmp_path, dtype):
    """bin/trace_run on a checkpoint folder written here: two requests one after the other,
    in portions, the second on the decoder the first gave back."""
    from yalm_amd import layered as Ly
    from yalm_amd.yalmfile import write_yalm

    cfg = C.DENSE_ONLY if dtype == "bfloat16" else C.MIXED
    t = make(cfg, 16)
    mdir = tmp_path / "model"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    write_yalm(str(mdir / "model.safetensors"), {k: Ly.f32_to_bf16(v).reshape(v.shape) for k, v in t.items()}, {},
               {k: "BF16" for k in t})
    a, b = C.tokens(cfg, 30, 12), C.tokens(cfg, 19, 13)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": [19, 0, 7]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[20:22], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[22:], "want": [7]}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b[:18], "want": [17]}], "end": []},
        {"step": 4, "entries": [{"id": "b", "tokens": b[18:], "want": [0]}], "end": ["b"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "64"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done %d" % i for i in range(5)]
    assert not (out / "1.f32").exists()
    w = {k: v.astype(np.float64) for k, v in t.items()}
    ra, rb = R.forward(cfg, w, a), R.forward(cfg, w, b)
    lim = F32_TOL if dtype == "float32" else BF16_TOL
    V = cfg["vocab"]
    assert rel_err(np.fromfile(out / "0.f32", "<f4").reshape(-1, V), ra[[19, 0, 7]]).max() < lim
    assert rel_err(np.fromfile(out / "2.f32", "<f4").reshape(-1, V), ra[[29]]).max() < lim
    assert rel_err(np.fromfile(out / "3.f32", "<f4").reshape(-1, V), rb[[17]]).max() < lim
    assert rel_err(np.fromfile(out / "4.f32", "<f4").reshape(-1, V), rb[[18]]).max() < lim
