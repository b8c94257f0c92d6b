"""MI355X: the layer-list engine serving Mirorax models against the plain float64 restatement
in tests/mirorax_ref.py, on small random models made here.

Errors are per position: || got - ref || / || ref || over the vocabulary. With f32 matrices
the engine differs from the restatement by f32 rounding only (F32_TOL); with bf16 matrices by
the rounding of the products' inputs and of the cached latents, keys and values (BF16_TOL; a
model with routed experts may miss it at a few positions where that rounding flips a router
near-tie). A lost key, a window one token off, a missing sink, a pass reading another pass's
cache or a token one place off moves the logits by orders of magnitude more than F32_TOL; the
edge tests show that on their own models before they trust it.
"""
import copy
import json
import os
import subprocess

import numpy as np
import pytest

import mirorax_cases as C
import mirorax_ref as R

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_TOL, BF16_TOL = 2e-4, 6e-2


@pytest.fixture(scope="module")
def rt():
    from yalm_amd import runtime

    runtime.check(runtime.lib.yalm_set_device(0))
    return runtime


def build(rt, cfg, wdt, seed=0, max_tokens=512, tensors=None):
    from yalm_amd import layered as Ly

    t = tensors if tensors is not None else Ly.mirorax_random_tensors(cfg, seed=seed)
    c = Ly.mirorax_config(cfg, max_tokens=max_tokens, weight_dtype=wdt)
    model = rt.SeqModel.from_packed(c, Ly.mirorax_pack(c, t, cfg))
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


ALONE = {k: C.ALL[k] for k in ("only_attn", "only_latent", "only_dense", "only_moe", "only_loop", "loop_once")}


@pytest.mark.parametrize("name", sorted(ALONE))
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_each_mechanism_alone(rt, name, dtype):
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


@pytest.mark.parametrize("name", ["mixed", "odd", "wide", "dense_only"])
def test_residual_stream_after_every_layer_run(rt, name):
    from yalm_amd import models as M

    cfg = C.ALL[name]
    model, dec, w = build(rt, cfg, M.F32, seed=2)
    try:
        tok = C.tokens(cfg, 57, 2)
        layers = []
        R.forward(cfg, w, tok, layers_out=layers)
        assert len(layers) == len(model.cfg.layers) > len(cfg["layers"])
        dec.layer_dump(True)
        dec.step(tok)
        got = dec.get_layers(len(tok))
        for i, ref in enumerate(layers):
            e = np.abs(got[i] - ref).max() / np.abs(ref).max()
            assert e < 1e-4, f"layer run {i}: {e}"
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("name", ["mixed", "odd", "wide", "dense_only"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prefill_then_token_by_token(rt, name, dtype):
    """A prompt in one step, then single tokens through the caches of every pass: the windows
    pass over decoded tokens, long prompts take the portion kernels."""
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
    """Portions cut anywhere (inside windows, down to two tokens) against the whole sequence;
    the GEMV / tile switch (8 | 9 tokens) and tile edges (64 | 65) included."""
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
    """Cache rows of an ended sequence (of any pass of the loop) must not leak into the next
    one: the second sequence on a reused decoder equals the same sequence on a fresh decoder
    bit for bit."""
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


def _resized(cfg, delta):
    c = copy.deepcopy(cfg)
    c["layers"][0]["mixer"]["mask"]["size"] += delta
    return c


EDGE = {
    # peaked attention (large score scale) in one layer: single keys decide positions
    "window": C.config([(C.L, C.latent(heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=24, size=37, scale=2.5), None)],
                       width=64, vocab=101),
    # the same inside a loop: every pass has its own window over its own cache
    "looped": C.config([(C.L, C.latent(heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=24, size=29, scale=2.0), None)],
                       width=64, vocab=101, loop=(0, 1, 2)),
    # a window longer than several key tiles: winning keys hundreds of positions back
    "far": C.config([(C.L, C.latent(heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=24, size=333, scale=2.5), None)],
                    width=64, vocab=101),
    # no window at all: the causal mixer's winning keys anywhere in the prompt
    "causal": C.config([(C.A, C.attn(heads=2, kv_heads=1, dim=16, vdim=24, scale=2.5), None)], width=64, vocab=101),
}


@pytest.mark.parametrize("name", ["window", "looped"])
def test_keys_just_inside_and_just_outside_the_window(rt, name):
    """The restatement with the window one position shorter / longer names the positions where
    the key just inside / just outside the edge decides the logits (they differ there by far
    more than the tolerance); the engine must agree with the true size at all of them, with
    the query in a prompt's portion and decoded alone."""
    from yalm_amd import models as M

    cfg = EDGE[name]
    model, dec, w = build(rt, cfg, M.F32, seed=9)
    try:
        tok = C.tokens(cfg, 240, 8)
        ref = R.forward(cfg, w, tok)
        inside = rel_err(R.forward(_resized(cfg, -1), w, tok), ref)   # the edge key taken away
        outside = rel_err(R.forward(_resized(cfg, +1), w, tok), ref)  # the next key let in
        assert (inside > 100 * F32_TOL).sum() >= 5 and (outside > 100 * F32_TOL).sum() >= 5
        for sizes in ([240], [100] + [1] * 140, [61, 2, 50, 2, 2, 93]):
            dec.reset()
            assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("name", ["far", "causal"])
def test_far_keys_decide_the_output(rt, name):
    """The restatement's own softmax weights name late queries whose winning key lies more
    than 250 positions back; changing THAT token must move the query's logits, and the engine
    must follow, in a prompt's portion and decoded alone."""
    from yalm_amd import models as M

    cfg = EDGE[name]
    model, dec, w = build(rt, cfg, M.F32, seed=10, max_tokens=600)
    try:
        a = C.tokens(cfg, 500, 9)
        P = []
        ra = R.forward(cfg, w, a, weights_out=P)
        P = P[0]
        far = [(P[h, t].max(), t, int(P[h, t].argmax())) for h in range(2) for t in range(340, 500)
               if t - int(P[h, t].argmax()) >= 250]
        assert far, "no late query with a far winning key: pick another seed"
        weight, t, j = max(far)
        assert weight > 0.3
        b = list(a)
        b[j] = (b[j] + 17) % cfg["vocab"]
        rb = R.forward(cfg, w, b)
        assert rel_err(ra[t], rb[t]) > 100 * F32_TOL
        for tok, ref in ((a, ra), (b, rb)):
            for sizes in ([490], [t] + [1] * 5):
                dec.reset()
                assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_every_mechanism_shows_in_the_logits(rt):
    """Taking one mechanism out of the restatement (the sink, the rotation, the loop's vectors,
    a layer scale, the output gate, the router's bias, a projection's bias) moves it far beyond
    the tolerance: the engine agreeing with the whole restatement means it computes each."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=11)
    try:
        tok = C.tokens(cfg, 40, 10)
        ref = R.forward(cfg, w, tok)

        def without(**changed):
            return rel_err(R.forward(cfg, {**w, **changed}, tok), ref).max()

        assert without(**{"l1.mix.sink": w["l1.mix.sink"] - 30.0}) > 100 * F32_TOL
        assert without(**{"loop.step": np.zeros_like(w["loop.step"])}) > 100 * F32_TOL
        assert without(**{"loop.step": w["loop.step"][::-1]}) > 100 * F32_TOL
        assert without(**{"l0.ls1": np.ones_like(w["l0.ls1"])}) > 100 * F32_TOL
        assert without(**{"l0.ls2": np.ones_like(w["l0.ls2"])}) > 100 * F32_TOL
        assert without(**{"l0.mix.g": np.zeros_like(w["l0.mix.g"])}) > 100 * F32_TOL
        assert without(**{"l1.mlp.router.b": np.zeros_like(w["l1.mlp.router.b"])}) > 100 * F32_TOL
        assert without(**{"l5.mix.o.b": np.zeros_like(w["l5.mix.o.b"])}) > 100 * F32_TOL
        # (a key bias shifts every score of a row alike and cancels in the softmax)
        assert without(**{"l0.mix.q.b": np.zeros_like(w["l0.mix.q.b"])}) > 100 * F32_TOL
        assert without(**{"l0.mix.v.b": np.zeros_like(w["l0.mix.v.b"])}) > 100 * F32_TOL
        keep = R.rotate
        try:
            R.rotate = lambda x, dims, base, positions: x
            assert rel_err(R.forward(cfg, w, tok), ref).max() > 100 * F32_TOL
        finally:
            R.rotate = keep
        assert rel_err(dec.step(tok, list(range(40))), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_routed_experts_follow_the_restatement(rt):
    """Every token's chosen experts and weights, through the logits: a one-layer model whose
    feed-forward is all the model does beyond a tiny mixer; the shared expert and each
    expert count (top = 1, top = all experts, no shared expert)."""
    from yalm_amd import models as M

    for mlp in (C.moe(), C.moe(experts=5, top=1, ff=24, shared=0), C.moe(experts=4, top=4, ff=16, shared=8)):
        cfg = C.config([(C.A, C.attn(heads=1, kv_heads=1, dim=8, vdim=8), mlp)], width=48, vocab=77)
        model, dec, w = build(rt, cfg, M.F32, seed=21)
        try:
            tok = C.tokens(cfg, 50, 21)
            picks = []
            ref = R.forward(cfg, w, tok, choice_out=picks)
            assert len({tuple(r) for r in picks[0][0].tolist()}) > 1 or mlp["router"]["top"] == mlp["router"]["experts"]
            assert rel_err(run_portions(dec, tok, [20, 5, 1, 1]), ref).max() < F32_TOL
        finally:
            dec.close()
            model.close()


@pytest.mark.parametrize("n", [1, 2, 3, 5])
def test_first_tokens(rt, n):
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
    """200 single tokens: every window of the model passes over decoded tokens several times."""
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


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_new_options_combine_freely(rt, dtype):
    """The options this design brought are parameters of the engine, not of one design: a
    stack put together by hand in the OTHER envelope (serial blocks with closing norms):
    latent attention with directly projected queries and a rotated key part but a full causal
    mask and no sink, followed by a gelu-gated dense feed-forward; then softmax attention with
    an elementwise output gate, an output bias, a zero-score sink and a window."""
    from yalm_amd import layered as Ly

    W, Vc, T = 48, 67, 90
    H, D, Rd, Vd, rank = 2, 8, 4, 12, 16
    H2, G2, D2, V2 = 4, 2, 8, 12
    rng = np.random.default_rng(5)

    def rnd(*shape, s=None):
        a = rng.standard_normal(shape) * (s if s is not None else 1.0 / np.sqrt(shape[-1]))
        return Ly.bf16_to_f32(Ly.f32_to_bf16(a.astype(np.float32))).reshape(shape)

    t = {"embed": rnd(Vc, W, s=0.5), "head": rnd(Vc, W), "final": 1 + rnd(W, s=0.2)}
    for i in (0, 1):
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            t[f"{n}.{i}"] = 1 + rnd(W, s=0.2)
    t.update(q0=rnd(H * (D + Rd), W), dkv0=rnd(rank + Rd, W), kvn0=1 + rnd(rank, s=0.2), uk0=rnd(H * D, rank),
             uv0=rnd(H * Vd, rank), o0=rnd(W, H * Vd), gate0=rnd(40, W), up0=rnd(40, W), down0=rnd(W, 40),
             q1=rnd(H2 * D2, W), k1=rnd(G2 * D2, W), v1=rnd(G2 * V2, W), g1=rnd(H2 * V2, W), o1=rnd(W, H2 * V2),
             ob1=rnd(W, s=0.3))
    s0 = Ly.LayerSpec(Ly.MIX_LATENT, heads=H, dim=D, vdim=Vd, kv_rank=rank, q_rank=0, rot_dim=Rd, rot_dims=Rd, rot_base=100.0,
                      attn_scale=0.4, mask_kind=Ly.MASK_CAUSAL, ff_kind=Ly.FF_DENSE, ff=40)
    s1 = Ly.LayerSpec(Ly.MIX_ATTN, heads=H2, kv_heads=G2, dim=D2, vdim=V2, attn_scale=0.5, mask_kind=Ly.MASK_WINDOW,
                      mask_size=11, sink=1, out_gate=Ly.GATE_ELEMENT, o_biased=True)
    c = Ly.LayeredConfig("by hand", W, Vc, [s0, s1], embed_scale=1.0, norm_eps=1e-5, max_tokens=128,
                         weight_dtype=wdt_of(dtype), norm_kind=Ly.NORM_RMS, pre_norm=True, pos_embed=False)
    as_w = (lambda a: np.ascontiguousarray(a, np.float32)) if dtype == "f32" else Ly.f32_to_bf16
    l0 = {"norm1": t["norm1.0"], "norm1b": t["norm1b.0"], "norm2": t["norm2.0"], "norm2b": t["norm2b.0"],
          "w_in": as_w(np.concatenate([t["q0"], t["dkv0"]])), "kv_norm": t["kvn0"],
          "w_ukt": as_w(np.ascontiguousarray(t["uk0"].reshape(H, D, rank).transpose(0, 2, 1))), "w_ukv": as_w(np.concatenate([t["uk0"], t["uv0"]])),
          "w_o": as_w(t["o0"]), "w_gate": as_w(t["gate0"]), "w_up": as_w(t["up0"]), "w_down": as_w(t["down0"])}
    l1 = {"norm1": t["norm1.1"], "norm1b": t["norm1b.1"], "w_in": as_w(np.concatenate([t["q1"], t["k1"], t["v1"], t["g1"]])),
          "w_o": as_w(t["o1"]), "o_bias": t["ob1"]}
    assert set(l0) == set(Ly.packed_shapes(c, s0)) and set(l1) == set(Ly.packed_shapes(c, s1))
    model = rt.SeqModel.from_packed(c, {"embed": as_w(t["embed"]), "final_norm": t["final"], "head": as_w(t["head"]),
                                        "layers": [l0, l1]})
    dec = rt.SeqDecoder(model)
    try:
        w = {k: v.astype(np.float64) for k, v in t.items()}
        tok = rng.integers(0, Vc, T).tolist()
        eps, pos = 1e-5, np.arange(T)
        x = w["embed"][tok]
        h = R.rms_norm(x, w["norm1.0"], eps)
        q = (h @ w["q0"].T).reshape(T, H, D + Rd)
        dkv = h @ w["dkv0"].T
        cl = R.rms_norm(dkv[:, :rank], w["kvn0"], eps)
        kr, qr = R.rotate(dkv[:, rank:], Rd, 100.0, pos), R.rotate(q[:, :, D:], Rd, 100.0, pos)
        kp, vv = (cl @ w["uk0"].T).reshape(T, H, D), (cl @ w["uv0"].T).reshape(T, H, Vd)
        s = np.stack([q[:, i, :D] @ kp[:, i].T + qr[:, i] @ kr.T for i in range(H)]) * 0.4
        p = R.softmax_rows(s, R.visible(None, T)[None])
        o = np.stack([p[i] @ vv[:, i] for i in range(H)], axis=1).reshape(T, H * Vd) @ w["o0"].T
        x = x + R.rms_norm(o, w["norm1b.0"], eps)
        h = R.rms_norm(x, w["norm2.0"], eps)
        x = x + R.rms_norm((R.gelu_tanh(h @ w["gate0"].T) * (h @ w["up0"].T)) @ w["down0"].T, w["norm2b.0"], eps)
        h = R.rms_norm(x, w["norm1.1"], eps)
        q = (h @ w["q1"].T).reshape(T, H2, D2)
        k = (h @ w["k1"].T).reshape(T, G2, D2)
        v = (h @ w["v1"].T).reshape(T, G2, V2)
        s = np.stack([q[:, i] @ k[:, i // 2].T for i in range(H2)]) * 0.5
        p = R.softmax_rows(s, R.visible(11, T)[None], sink=np.zeros(H2))
        o = np.stack([p[i] @ v[:, i // 2] for i in range(H2)], axis=1).reshape(T, H2 * V2) * R.sigmoid(h @ w["g1"].T)
        x = x + R.rms_norm(o @ w["o1"].T + w["ob1"], w["norm1b.1"], eps)
        ref = R.rms_norm(x, w["final"], eps) @ w["head"].T
        lim = F32_TOL if dtype == "f32" else BF16_TOL
        assert rel_err(dec.step(tok, list(range(T))), ref).max() < lim
        dec.reset()
        assert rel_err(run_portions(dec, tok, [40, 2, 9] + [1] * 39), ref).max() < lim
    finally:
        dec.close()
        model.close()


_LONG_REF = {}


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prompt_longer_than_one_internal_portion(rt, dtype):
    """A step of more tokens than the engine's work buffers hold (4096) is cut inside the
    engine, in the middle of a window; asked rows on both sides of the cut come back in order."""
    cfg = C.config([(C.L, C.latent(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=8, size=150, scale=0.35), None),
                    (C.A, C.attn(heads=2, kv_heads=2, dim=8, vdim=8, scale=0.35), None)], width=32, vocab=53, loop=(0, 1, 2))
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
    # key rows of more than 256 entries: long portions expand the latents into per-head keys and
    # values, short ones and single tokens attend over the latent rows (f32 tiles, key splits)
    "rank256": C.latent(heads=16, dim=32, rot_dim=64, vdim=32, kv_rank=256, size=200, scale=0.08, rot_dims=64),
    # latent rows too long for the f32 tiles: every portion of two tokens or more expands; single
    # tokens take blocks of 16 of the 24 heads per workgroup
    "rank512": C.latent(heads=24, dim=16, rot_dim=64, vdim=24, kv_rank=512, size=150, scale=0.06, rot_dims=32),
}


@pytest.mark.parametrize("name", sorted(LARGE))
def test_large_latent_sizes(rt, name):
    cfg = C.config([(C.L, LARGE[name], C.dense(ff=64))], width=128, vocab=101)
    for dtype in ("f32", "bf16"):
        model, dec, w = build(rt, cfg, wdt_of(dtype), seed=22, max_tokens=400)
        try:
            tok = C.tokens(cfg, 330, 22)
            ref = R.forward(cfg, w, tok)
            assert agrees(run_portions(dec, tok, [270, 5, 2, 20, 9] + [1] * 24), ref, dtype, cfg)
        finally:
            dec.close()
            model.close()


def test_sequence_cannot_pass_max_tokens(rt):
    from yalm_amd import models as M

    model, dec, _ = build(rt, C.ONLY_LATENT, M.F32, seed=13, max_tokens=16)
    try:
        dec.step(C.tokens(C.ONLY_LATENT, 16, 0))
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
    t = Ly.mirorax_random_tensors(cfg, seed=16)
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
