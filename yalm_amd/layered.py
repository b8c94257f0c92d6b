"""Layer-list model designs: configuration, checkpoint reading and weight packing.

A layer-list design gives every layer its own token mixer and feed-forward
(include/yalm_hip.h, "layer-list models"). ``LayeredConfig`` is the engine-facing
description; a design registers a reader that turns its ``config.json`` into one and
a packer that turns its checkpoint tensors into the engine's per-layer tensors
(concatenated input projections, per-head transposed key up-projections, stacked
experts). ``Sinulorn`` (latent attention, recurrences, routed experts), ``Lenuzen``
(windowed / chunked softmax attention, plain feed-forwards), ``Mirorax`` (parallel
blocks with layer scales, a looped run of layers, gated attention, latent attention with a
rotated key part, a window and a learned sink) and ``Lifenex`` (parallel blocks with a norm
per sublayer, a selective state-space mixer, attention with a distance bias beside a delta
rule with per-channel decays, grouped sigmoid routing) are such designs.

Checkpoints are folders with ``config.json`` and ``model.safetensors`` (bf16
matrices; read with yalmfile.read_yalm, the same container the .yalm files use).
"""

from __future__ import annotations

import dataclasses
import json
import os

import numpy as np

from . import models as M

MIX_LATENT, MIX_RGLRU, MIX_DELTA, MIX_ATTN, MIX_SSM = 0, 1, 2, 3, 4
FF_NONE, FF_DENSE, FF_MOE, FF_PLAIN = 0, 1, 2, 3
NORM_RMS, NORM_LAYER = 0, 1
MASK_CAUSAL, MASK_WINDOW, MASK_CHUNK = 0, 1, 2
QK_NONE, QK_HEAD_UNIT, QK_WHOLE, QK_HEAD_W = 0, 1, 2, 3
BLOCK_SERIAL, BLOCK_PARALLEL = 0, 1
ACT_DEFAULT, ACT_GELU, ACT_CLAMP, ACT_SILU, ACT_RELU2 = 0, 1, 2, 3, 4
ROUTER_SOFTMAX_TOP, ROUTER_TOP_SOFTMAX, ROUTER_SIGMOID_GROUPS = 0, 1, 2
DELTA_GATE_SILU, DELTA_GATE_SIGMOID = 0, 1
GATE_NONE, GATE_HEAD, GATE_ELEMENT = 0, 1, 2


@dataclasses.dataclass
class LayerSpec:
    mixer: int
    heads: int = 0
    kv_heads: int = 0
    dim: int = 0
    vdim: int = 0
    kv_rank: int = 0
    q_rank: int = 0
    kv_from: int = -1
    attn_scale: float = 0.0
    rec_width: int = 0
    blocks: int = 0
    conv: int = 0
    ff_kind: int = FF_NONE
    ff: int = 0
    experts: int = 0
    top: int = 0
    groups: int = 1
    groups_keep: int = 1
    router_scale: float = 1.0
    limit: float = 0.0
    shared_ff: int = 0
    shared_limit: float = 0.0
    # softmax attention over cached keys and values
    mask_kind: int = MASK_CAUSAL
    mask_size: int = 0
    qk_norm: int = QK_NONE
    v_norm: int = 0
    sink: int = 0
    out_gate: int = 0
    rot_dims: int = 0
    rot_orig: int = 0
    rot_base: float = 10000.0
    rot_factor: float = 0.0
    rot_fast: float = 0.0
    rot_slow: float = 0.0
    in_biased: bool = False
    head_temps: bool = False
    talking: bool = False
    # latent attention with directly projected queries (q_rank 0): the rotated part of a
    # query head and of the one key part all heads share
    rot_dim: int = 0
    sink_learned: bool = False  # the sink's score is a tensor (sink_w) instead of 0
    o_biased: bool = False
    # gated feed-forwards and routers
    ff_act: int = ACT_DEFAULT
    router_kind: int = ROUTER_SOFTMAX_TOP
    router_biased: bool = False
    shared_gated: bool = True   # the shared expert is scaled by sigmoid(shared_sg . x)
    # layer runs
    pre_added: bool = False     # a vector joins the stream before this run's opening norm
    shares: int = -1            # >= 0: this run uses the tensors of that (earlier) run, all but pre_add
    # selective state-space mixer: heads x vdim channels, a state of ssm_state x vdim per head
    ssm_state: int = 0
    ssm_groups: int = 1
    norm_groups: int = 1
    # delta rule: low-rank decay per head and key channel / low-rank output gate (0: the plain forms)
    decay_rank: int = 0
    gate_rank: int = 0
    gate_act: int = DELTA_GATE_SILU
    # softmax attention: query temperature by position, learned bias per head and bucketed distance
    q_temp_coef: float = 0.0
    q_temp_every: int = 0
    rel_rows: int = 0
    rel_max: float = 0.0
    # a second mixer beside this one (a LayerSpec whose mixer fields alone are used); the two
    # results are rms-normed with join_w / side_join_w, summed and scaled by join_scale
    side: "LayerSpec" = None
    join_scale: float = 1.0
    # parallel blocks: the feed-forward reads its own norm (norm2) of the stream; no layer scales
    ff_normed: bool = False
    layer_scaled: bool = True

    @property
    def in_rows(self) -> int:
        """Rows of the concatenated input projection w_in."""
        if self.mixer == MIX_LATENT:
            if self.q_rank == 0:
                return self.heads * (self.dim + self.rot_dim) + self.kv_rank + self.rot_dim
            return self.q_rank + (self.kv_rank if self.kv_from < 0 else 0)
        if self.mixer == MIX_RGLRU:
            return 2 * self.rec_width
        if self.mixer == MIX_ATTN:
            gate = {GATE_NONE: 0, GATE_HEAD: self.heads, GATE_ELEMENT: self.heads * self.vdim}[self.out_gate]
            return self.heads * self.dim + self.kv_heads * (self.dim + self.vdim) + gate
        if self.mixer == MIX_SSM:
            return 2 * self.heads * self.vdim + 2 * self.ssm_groups * self.ssm_state + self.heads
        return (2 * self.kv_heads * self.dim + self.heads * self.vdim + (self.gate_rank or self.heads * self.vdim)
                + self.heads + (self.decay_rank or self.heads))

    @property
    def mix_out(self) -> int:
        """Columns of the mixer's output projection."""
        return self.rec_width if self.mixer == MIX_RGLRU else self.heads * self.vdim


@dataclasses.dataclass
class LayeredConfig:
    arch: str
    width: int
    vocab: int
    layers: list
    embed_scale: float = 1.0
    norm_eps: float = 1e-5
    max_tokens: int = 4096
    weight_dtype: int = M.BF16
    norm_kind: int = NORM_RMS
    pre_norm: bool = True     # False: a sublayer reads the stream itself; only the closing norms exist
    pos_embed: bool = True    # the sin / cos position vector added to the embedding
    logit_scale: float = 1.0
    tied_head: bool = False   # the logits read the embedding table
    block_kind: int = BLOCK_SERIAL  # BLOCK_PARALLEL: x += ls1 * mixer(norm1(x)) + ls2 * ff(norm1(x))
    embed_normed: bool = False  # the embedding row is rms-normed (weight embed_norm) before it becomes the stream

    def with_(self, **kw) -> "LayeredConfig":
        return dataclasses.replace(self, **kw)


def packed_shapes(c: LayeredConfig, l: LayerSpec, side: bool = False) -> dict:
    """field -> (shape, kind) of one layer's engine tensors; kind "w": a matrix of the
    model's weight dtype, "f": f32. side: l is a layer's second mixer (its mixer tensors only)."""
    W = c.width
    out = {}
    if l.pre_added:
        out["pre_add"] = ((W,), "f")
    if l.shares >= 0:
        return out
    if side:
        pass
    elif c.block_kind == BLOCK_PARALLEL:
        out["norm1"] = ((W,), "f")
        if l.layer_scaled:
            out["ls1"] = ((W,), "f")
        if l.ff_kind != FF_NONE:
            if l.layer_scaled:
                out["ls2"] = ((W,), "f")
            if l.ff_normed:
                out["norm2"] = ((W,), "f")
    else:
        out["norm1b"] = ((W,), "f")
        if c.pre_norm:
            out["norm1"] = ((W,), "f")
        if l.ff_kind != FF_NONE:
            out["norm2b"] = ((W,), "f")
            if c.pre_norm:
                out["norm2"] = ((W,), "f")
    if l.side is not None:
        out["join_w"] = out["side_join_w"] = ((W,), "f")
    out["w_in"] = ((l.in_rows, W), "w")
    out["w_o"] = ((W, l.mix_out), "w")
    if l.o_biased:
        out["o_bias"] = ((W,), "f")
    if l.sink_learned:
        out["sink_w"] = ((l.heads,), "f")
    if l.mixer == MIX_LATENT:
        if l.q_rank:
            out["q_norm"] = ((l.q_rank,), "f")
            out["w_uq"] = ((l.heads * l.dim, l.q_rank), "w")
        if l.kv_from < 0:
            out["kv_norm"] = ((l.kv_rank,), "f")
        out["w_ukt"] = ((l.heads, l.kv_rank, l.dim), "w")
        if l.q_rank:
            out["w_uv"] = ((l.heads * l.vdim, l.kv_rank), "w")
        else:  # key and value up-projections stacked; the value rows serve as w_uv
            out["w_ukv"] = ((l.heads * (l.dim + l.vdim), l.kv_rank), "w")
    elif l.mixer == MIX_RGLRU:
        bs = l.rec_width // l.blocks
        out.update(
            in_bias=((2 * l.rec_width,), "f"), conv_w=((l.rec_width, l.conv), "f"), conv_b=((l.rec_width,), "f"),
            gate_a=((l.blocks, bs, bs), "f"), gate_a_b=((l.rec_width,), "f"),
            gate_i=((l.blocks, bs, bs), "f"), gate_i_b=((l.rec_width,), "f"), lam=((l.rec_width,), "f"),
        )
    elif l.mixer == MIX_ATTN:
        if l.in_biased:
            out["in_bias"] = ((l.in_rows,), "f")
        if l.qk_norm == QK_WHOLE:
            out.update(q_norm=((l.heads * l.dim,), "f"), kv_norm=((l.kv_heads * l.dim,), "f"))
        if l.head_temps:
            out["head_temp"] = ((l.heads,), "f")
        if l.talking:
            out["talk"] = ((l.heads, l.heads), "f")
        if l.qk_norm == QK_HEAD_W:
            out.update(q_norm=((l.dim,), "f"), kv_norm=((l.dim,), "f"))
        if l.rel_rows:
            out["rel"] = ((l.rel_rows, l.heads), "f")
    elif l.mixer == MIX_SSM:
        inner, cc = l.heads * l.vdim, l.heads * l.vdim + 2 * l.ssm_groups * l.ssm_state
        out.update(conv_w=((cc, l.conv), "f"), conv_b=((cc,), "f"), a_log=((l.heads,), "f"), dt_bias=((l.heads,), "f"),
                   d_skip=((l.heads,), "f"), out_norm=((inner,), "f"))
    else:
        cc = 2 * l.kv_heads * l.dim + l.heads * l.vdim
        out.update(conv_w=((cc, l.conv), "f"), a_log=((l.heads,), "f"),
                   dt_bias=((l.heads * l.dim if l.decay_rank else l.heads,), "f"), out_norm=((l.vdim,), "f"))
        if l.decay_rank:
            out["w_a2"] = ((l.heads * l.dim, l.decay_rank), "w")
        if l.gate_rank:
            out["w_g2"] = ((l.heads * l.vdim, l.gate_rank), "w")
    if l.ff_kind == FF_PLAIN:
        out.update(w_up=((l.ff, W), "w"), w_down=((W, l.ff), "w"))
    if l.ff_kind == FF_DENSE:
        out.update(w_gate=((l.ff, W), "w"), w_up=((l.ff, W), "w"), w_down=((W, l.ff), "w"))
    elif l.ff_kind == FF_MOE:
        out.update(router=((l.experts, W), "f"), w_gate=((l.experts, l.ff, W), "w"),
                   w_up=((l.experts, l.ff, W), "w"), w_down=((l.experts, W, l.ff), "w"))
        if l.router_biased:
            out["router_bias"] = ((l.experts,), "f")
        if l.shared_ff:
            out.update(ws_gate=((l.shared_ff, W), "w"), ws_up=((l.shared_ff, W), "w"),
                       ws_down=((W, l.shared_ff), "w"))
            if l.shared_gated:
                out["shared_sg"] = ((W,), "f")
    return out


# ------------------------------------------------------------------ bf16 <-> f32 on the host
def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round to nearest even on the f32 bits."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _as_f32(a: np.ndarray) -> np.ndarray:
    return bf16_to_f32(a) if a.dtype == np.uint16 else np.asarray(a, np.float32)


def _as_weight(a: np.ndarray, dtype: int) -> np.ndarray:
    """A matrix in the engine's storage: bf16 bits (uint16) or f32."""
    if dtype == M.F32:
        return np.ascontiguousarray(_as_f32(a))
    if dtype != M.BF16:
        raise ValueError("layer-list models run with bf16 or f32 matrices")
    return np.ascontiguousarray(a if a.dtype == np.uint16 else f32_to_bf16(a))


# ------------------------------------------------------------------ Sinulorn
SINULORN_MIXERS = {"latent_attention": MIX_LATENT, "rglru": MIX_RGLRU, "delta": MIX_DELTA}


def sinulorn_config(cfg: dict, max_tokens: int = 4096, weight_dtype: int = M.BF16) -> LayeredConfig:
    """config.json of a Sinulorn checkpoint -> LayeredConfig. Every size and every
    constant that can differ between models of the design is read from cfg."""
    layers = []
    for e in cfg["layers"]:
        m = e["mixer"]
        kind = SINULORN_MIXERS.get(e["type"])
        if kind is None:
            raise ValueError(f"unknown mixer type {e['type']!r}")
        if kind == MIX_LATENT:
            s = LayerSpec(kind, heads=m["heads"], dim=m["dim"], vdim=m["vdim"], kv_rank=m["kv_rank"],
                          q_rank=m["q_rank"], kv_from=m.get("kv_from", -1) if m.get("kv_from") is not None else -1,
                          attn_scale=float(m["scale"]))
        elif kind == MIX_RGLRU:
            s = LayerSpec(kind, rec_width=m["width"], blocks=m["blocks"], conv=m["conv"])
        else:
            s = LayerSpec(kind, heads=m["heads"], kv_heads=m.get("kv_heads", m["heads"]), dim=m["dim"], vdim=m["vdim"],
                          conv=m["conv"])
        mlp = e.get("mlp")
        if mlp:
            if mlp["kind"] == "dense":
                s.ff_kind, s.ff = FF_DENSE, mlp["ff"]
            elif mlp["kind"] == "moe":
                r = mlp["router"]
                g = r.get("groups") or {"count": 1, "keep": 1}
                s.ff_kind, s.ff, s.limit = FF_MOE, mlp["expert"]["ff"], float(mlp["expert"]["limit"])
                s.experts, s.top, s.router_scale = r["experts"], r["top"], float(r.get("scale", 1.0))
                s.groups, s.groups_keep = g["count"], g["keep"]
                sh = mlp.get("shared")
                if sh:
                    s.shared_ff, s.shared_limit = sh["ff"], float(sh["limit"])
            else:
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
        layers.append(s)
    return LayeredConfig(
        arch="Sinulorn", width=cfg["width"], vocab=cfg["vocab"], layers=layers,
        embed_scale=float(cfg["embedding"]["scale"]), norm_eps=float(cfg["norm"]["eps"]),
        max_tokens=max_tokens, weight_dtype=weight_dtype,
    )


def sinulorn_tensor_shapes(cfg: dict) -> dict:
    """Checkpoint tensor name -> shape for a Sinulorn config.json."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,), "head": (cfg["vocab"], W)}
    for i, e in enumerate(cfg["layers"]):
        p, m = f"l{i}.", e["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (W,)
        x = p + "mix."
        if e["type"] == "latent_attention":
            H, D, V = m["heads"], m["dim"], m["vdim"]
            out[x + "dq"], out[x + "dq.norm"], out[x + "uq"] = (m["q_rank"], W), (m["q_rank"],), (H * D, m["q_rank"])
            if m.get("kv_from") is None:
                out[x + "dkv"], out[x + "dkv.norm"] = (m["kv_rank"], W), (m["kv_rank"],)
            out[x + "uk"], out[x + "uv"], out[x + "o"] = (H * D, m["kv_rank"]), (H * V, m["kv_rank"]), (W, H * V)
        elif e["type"] == "rglru":
            R, B = m["width"], m["blocks"]
            for n in ("y", "x"):
                out[x + n], out[x + n + ".b"] = (R, W), (R,)
            out[x + "conv"], out[x + "conv.b"] = (R, m["conv"]), (R,)
            for n in ("ra", "ri"):
                out[x + n], out[x + n + ".b"] = (B, R // B, R // B), (B, R // B)
            out[x + "lam"], out[x + "o"] = (R,), (W, R)
        else:
            H, KH, D, V = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
            for n, rows in (("q", KH * D), ("k", KH * D), ("v", H * V)):
                out[x + n], out[x + n + ".conv"] = (rows, W), (rows, m["conv"])
            out[x + "b"] = out[x + "a"] = (H, W)
            out[x + "A_log"] = out[x + "dt_bias"] = (H,)
            out[x + "norm"], out[x + "g"], out[x + "o"] = (V,), (H * V, W), (W, H * V)
        mlp = e.get("mlp")
        if not mlp:
            continue
        out[p + "norm2"] = out[p + "norm2b"] = (W,)
        f = p + "mlp."
        if mlp["kind"] == "dense":
            out[f + "gate"] = out[f + "up"] = (mlp["ff"], W)
            out[f + "down"] = (W, mlp["ff"])
        else:
            ff = mlp["expert"]["ff"]
            for k in range(mlp["router"]["experts"]):
                out[f"{f}e{k}.gate"] = out[f"{f}e{k}.up"] = (ff, W)
                out[f"{f}e{k}.down"] = (W, ff)
            out[f + "router"] = (mlp["router"]["experts"], W)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                out[f + "shared.gate"] = out[f + "shared.up"] = (sf, W)
                out[f + "shared.down"], out[f + "shared.sg"] = (W, sf), (1, W)
    return out


def sinulorn_pack(c: LayeredConfig, t: dict) -> dict:
    """Checkpoint tensors (name -> array, bf16 bits as uint16 or floats, checkpoint shapes)
    -> the engine's tensors: {"embed", "final_norm", "head", "layers": [field -> array]}."""
    dt = c.weight_dtype

    def w(*names):
        parts = [_as_weight(t[n], dt) for n in names]
        return parts[0] if len(parts) == 1 else np.ascontiguousarray(np.concatenate(parts, axis=0))

    def f(*names):
        parts = [_as_f32(t[n]).reshape(-1) if len(names) > 1 else _as_f32(t[n]) for n in names]
        return np.ascontiguousarray(parts[0] if len(parts) == 1 else np.concatenate(parts))

    layers = []
    for i, l in enumerate(c.layers):
        p, x, m = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        d = {"norm1": f(p + "norm1"), "norm1b": f(p + "norm1b")}
        if l.ff_kind != FF_NONE:
            d.update(norm2=f(p + "norm2"), norm2b=f(p + "norm2b"))
        if l.mixer == MIX_LATENT:
            d["w_in"] = w(x + "dq", x + "dkv") if l.kv_from < 0 else w(x + "dq")
            d["q_norm"] = f(x + "dq.norm")
            if l.kv_from < 0:
                d["kv_norm"] = f(x + "dkv.norm")
            d["w_uq"] = w(x + "uq")
            uk = _as_weight(t[x + "uk"], dt).reshape(l.heads, l.dim, l.kv_rank)
            d["w_ukt"] = np.ascontiguousarray(uk.transpose(0, 2, 1))
            d["w_uv"] = w(x + "uv")
        elif l.mixer == MIX_RGLRU:
            d["w_in"] = w(x + "y", x + "x")
            d["in_bias"] = f(x + "y.b", x + "x.b")
            d.update(conv_w=f(x + "conv"), conv_b=f(x + "conv.b"), gate_a=f(x + "ra"), gate_a_b=f(x + "ra.b").reshape(-1),
                     gate_i=f(x + "ri"), gate_i_b=f(x + "ri.b").reshape(-1), lam=f(x + "lam"))
        else:
            d["w_in"] = w(x + "q", x + "k", x + "v", x + "g", x + "b", x + "a")
            d["conv_w"] = np.ascontiguousarray(
                np.concatenate([_as_f32(t[x + n + ".conv"]) for n in ("q", "k", "v")], axis=0))
            d.update(a_log=f(x + "A_log"), dt_bias=f(x + "dt_bias"), out_norm=f(x + "norm"))
        d["w_o"] = w(x + "o")
        if l.ff_kind == FF_DENSE:
            d.update(w_gate=w(m + "gate"), w_up=w(m + "up"), w_down=w(m + "down"))
        elif l.ff_kind == FF_MOE:
            d["router"] = f(m + "router")
            for k in ("gate", "up", "down"):
                d["w_" + k] = np.ascontiguousarray(
                    np.stack([_as_weight(t[f"{m}e{e}.{k}"], dt) for e in range(l.experts)]))
            if l.shared_ff:
                d.update(shared_sg=f(m + "shared.sg").reshape(-1), ws_gate=w(m + "shared.gate"),
                         ws_up=w(m + "shared.up"), ws_down=w(m + "shared.down"))
        want = packed_shapes(c, l)
        for k, (shape, _) in want.items():
            if tuple(d[k].shape) != tuple(shape):
                raise ValueError(f"layer {i}: tensor {k} has shape {d[k].shape}, the configuration gives {shape}")
        layers.append(d)
    return {"embed": w("embed"), "final_norm": f("final.norm"), "head": w("head"), "layers": layers}


def sinulorn_random_tensors(cfg: dict, seed: int = 0, gain: float = 1.0) -> dict:
    """Random checkpoint tensors for a Sinulorn config.json, as float32 arrays already
    rounded to bf16 values (so the f32 and bf16 engines and a float64 restatement see the
    same weights). Scales keep activations of order one through deep stacks."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in sinulorn_tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2", "norm1b", "norm2b") or name.endswith((".norm", "final.norm")):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "b" and len(shape) == 1 or name.endswith((".y.b", ".x.b", "conv.b", "ra.b", "ri.b")):
            a = 0.3 * rng.standard_normal(shape)
        elif leaf == "conv":
            a = 0.5 * rng.standard_normal(shape)
        elif leaf == "lam":
            a = rng.uniform(-4.0, 1.0, shape)
        elif leaf == "A_log":
            a = rng.uniform(-3.0, 0.5, shape)
        elif leaf == "dt_bias":
            a = rng.uniform(-2.0, 1.0, shape)
        elif leaf == "embed":
            a = 0.1 * rng.standard_normal(shape)
        else:
            a = gain * rng.standard_normal(shape) / np.sqrt(shape[-1])
        out[name] = bf16_to_f32(f32_to_bf16(a.astype(np.float32))).reshape(shape)
    return out


# ------------------------------------------------------------------ Lenuzen
# Every layer: x += layer_norm(mixer(x)), then x += layer_norm(ff(x)); the sublayers read
# the stream itself. Two mixers, both softmax attention over cached keys and values with
# grouped key/value heads and partial interleaved rotary positions with rescaled frequencies:
#   "attention":   biased projections, queries / keys / values divided by their per-head rms
#                  (queries and keys after the rotation), a per-head score temperature, a
#                  sliding window, a per-head sigmoid output gate;
#   "attention_2": weighted rms norm of the whole query and key projections before the
#                  rotation, scores mixed across heads by a [heads, heads] matrix, a chunked
#                  mask, a softmax with a zero-score sink.
# Feed-forward: w_down gelu(w_up x). Logits: the embedding table on the final norm, times
# logit_scale.
LENUZEN_MIXERS = ("attention", "attention_2")


def lenuzen_config(cfg: dict, max_tokens: int = 4096, weight_dtype: int = M.BF16) -> LayeredConfig:
    """config.json of a Lenuzen checkpoint -> LayeredConfig. Every size and every constant
    that can differ between models of the design is read from cfg."""
    layers = []
    for e in cfg["layers"]:
        m = e["mixer"]
        if e["type"] not in LENUZEN_MIXERS:
            raise ValueError(f"unknown mixer type {e['type']!r}")
        rot = m["rot"]
        sc = rot.get("scaling") or {}
        s = LayerSpec(MIX_ATTN, heads=m["heads"], kv_heads=m.get("kv_heads", m["heads"]), dim=m["dim"], vdim=m["vdim"],
                      attn_scale=float(m["scale"]), mask_size=int(m["mask"]["size"]), rot_dims=int(rot["dims"]),
                      rot_base=float(rot["base"]), rot_factor=float(sc.get("factor", 0.0)),
                      rot_orig=int(sc.get("original", 0)), rot_fast=float(sc.get("fast", 0.0)),
                      rot_slow=float(sc.get("slow", 0.0)))
        if e["type"] == "attention":
            s.mask_kind, s.qk_norm, s.v_norm, s.out_gate = MASK_WINDOW, QK_HEAD_UNIT, 1, 1
            s.in_biased = s.head_temps = True
        else:
            s.mask_kind, s.qk_norm, s.sink, s.talking = MASK_CHUNK, QK_WHOLE, 1, True
        mlp = e.get("mlp")
        if mlp:
            if mlp["kind"] != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            s.ff_kind, s.ff = FF_PLAIN, mlp["ff"]
        layers.append(s)
    return LayeredConfig(
        arch="Lenuzen", width=cfg["width"], vocab=cfg["vocab"], layers=layers,
        embed_scale=float(cfg["embedding"]["scale"]), norm_eps=float(cfg["norm"]["eps"]),
        max_tokens=max_tokens, weight_dtype=weight_dtype, norm_kind=NORM_LAYER, pre_norm=False, pos_embed=False,
        logit_scale=float(cfg.get("logit_scale", 1.0)), tied_head=True,
    )


def lenuzen_tensor_shapes(cfg: dict) -> dict:
    """Checkpoint tensor name -> shape for a Lenuzen config.json."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,)}
    for i, e in enumerate(cfg["layers"]):
        p, m = f"l{i}.", e["mixer"]
        x = p + "mix."
        H, G, D, V = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
        out[p + "norm1"] = (W,)
        out[x + "q"], out[x + "k"], out[x + "v"], out[x + "o"] = (H * D, W), (G * D, W), (G * V, W), (W, H * V)
        if e["type"] == "attention":
            out[x + "q.b"], out[x + "k.b"], out[x + "v.b"] = (H * D,), (G * D,), (G * V,)
            out[x + "temp"], out[x + "g"] = (H,), (H, W)
        else:
            out[x + "q.norm"], out[x + "k.norm"], out[x + "talk"] = (H * D,), (G * D,), (H, H)
        if e.get("mlp"):
            out[p + "norm2"] = (W,)
            out[p + "mlp.up"], out[p + "mlp.down"] = (e["mlp"]["ff"], W), (W, e["mlp"]["ff"])
    return out


def lenuzen_pack(c: LayeredConfig, t: dict) -> dict:
    """Checkpoint tensors -> the engine's tensors (see sinulorn_pack): q | k | v | gate rows
    concatenated into w_in with one bias vector over all of them (zeros for the gate rows)."""
    dt = c.weight_dtype

    def w(*names):
        parts = [_as_weight(t[n], dt) for n in names]
        return parts[0] if len(parts) == 1 else np.ascontiguousarray(np.concatenate(parts, axis=0))

    def f(name):
        return np.ascontiguousarray(_as_f32(t[name]))

    layers = []
    for i, l in enumerate(c.layers):
        p, x, m = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        d = {"norm1b": f(p + "norm1")}
        if l.out_gate:
            d["w_in"] = w(x + "q", x + "k", x + "v", x + "g")
        else:
            d["w_in"] = w(x + "q", x + "k", x + "v")
        if l.in_biased:
            b = np.zeros(l.in_rows, np.float32)
            nb = l.heads * l.dim + l.kv_heads * (l.dim + l.vdim)
            b[:nb] = np.concatenate([f(x + "q.b"), f(x + "k.b"), f(x + "v.b")])
            d["in_bias"] = b
        if l.qk_norm == QK_WHOLE:
            d.update(q_norm=f(x + "q.norm"), kv_norm=f(x + "k.norm"))
        if l.head_temps:
            d["head_temp"] = f(x + "temp")
        if l.talking:
            d["talk"] = f(x + "talk")
        d["w_o"] = w(x + "o")
        if l.ff_kind == FF_PLAIN:
            d.update(norm2b=f(p + "norm2"), w_up=w(m + "up"), w_down=w(m + "down"))
        want = packed_shapes(c, l)
        if set(want) != set(d):
            raise ValueError(f"layer {i}: packed tensors {sorted(d)} do not match the configuration's {sorted(want)}")
        for k, (shape, _) in want.items():
            if tuple(d[k].shape) != tuple(shape):
                raise ValueError(f"layer {i}: tensor {k} has shape {d[k].shape}, the configuration gives {shape}")
        layers.append(d)
    emb = w("embed")
    return {"embed": emb, "final_norm": f("final.norm"), "head": emb, "layers": layers}


def lenuzen_random_tensors(cfg: dict, seed: int = 0, gain: float = 1.0) -> dict:
    """Random checkpoint tensors for a Lenuzen config.json, as float32 arrays already rounded
    to bf16 values (the f32 and bf16 engines and a float64 restatement see the same weights)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in lenuzen_tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2") or name.endswith(".norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif leaf == "temp":
            a = rng.uniform(0.6, 1.6, shape)
        elif leaf == "talk":
            a = np.eye(shape[0]) + 0.25 * rng.standard_normal(shape)
        elif leaf == "embed":
            a = 0.1 * rng.standard_normal(shape)
        else:
            a = gain * rng.standard_normal(shape) / np.sqrt(shape[-1])
        out[name] = bf16_to_f32(f32_to_bf16(a.astype(np.float32))).reshape(shape)
    return out


# ------------------------------------------------------------------ Mirorax
# Every layer is a parallel block: h = rms(x) w1, x += ls1 * mixer(h) + ls2 * ff(h). A run of
# layers [start, stop) is walked `times` times with the same weights; pass t first adds row t of
# the tensor loop.step to the stream; every pass has caches of its own. Two mixers:
#   "attention":        grouped key/value heads, biased q / k / v / o projections, no positions,
#                       causal, plain softmax, the concatenated heads times sigmoid(W_g h);
#   "latent_attention": queries [dim plain | rot_dim rotated] per head from the input directly,
#                       a cached rms-normed latent (per-head plain keys and values are its
#                       up-projections) and one cached rotated key part shared by all heads,
#                       a sliding window, a learned per-head sink in the softmax's denominator.
# Feed-forwards: "dense" W_d (g' sigmoid(1.702 g') (u' + 1)) with g' = min(W_g h, limit), u' =
# clamp(W_u h, +-limit); "moe": silu-gated experts, the top logits of a biased router win and
# their weights are the softmax over the chosen logits, plus an ungated shared expert.
MIRORAX_MIXERS = ("attention", "latent_attention")


def unroll_loop(layers: list, loop) -> list:
    """The order the layers run in: [(layer index, pass number or None)], the pass number
    given for the first layer of every pass of the looped run [start, stop)."""
    n = len(layers)
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    if not (0 <= a < b <= n and times >= 1):
        raise ValueError(f"bad loop {loop!r} over {n} layers")
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def _mirorax_layer(e: dict) -> LayerSpec:
    m = e["mixer"]
    if e["type"] == "attention":
        s = LayerSpec(MIX_ATTN, heads=m["heads"], kv_heads=m.get("kv_heads", m["heads"]), dim=m["dim"], vdim=m["vdim"],
                      attn_scale=float(m["scale"]), mask_kind=MASK_CAUSAL, out_gate=GATE_ELEMENT, in_biased=True,
                      o_biased=True)
    elif e["type"] == "latent_attention":
        rot = m["rot"]
        s = LayerSpec(MIX_LATENT, heads=m["heads"], dim=m["dim"], vdim=m["vdim"], kv_rank=m["kv_rank"], q_rank=0,
                      rot_dim=int(m["rot_dim"]), attn_scale=float(m["scale"]), mask_kind=MASK_WINDOW,
                      mask_size=int(m["mask"]["size"]), rot_dims=int(rot["dims"]), rot_base=float(rot["base"]),
                      sink=1, sink_learned=True)
    else:
        raise ValueError(f"unknown mixer type {e['type']!r}")
    mlp = e.get("mlp")
    if mlp:
        if mlp["kind"] == "dense":
            s.ff_kind, s.ff, s.limit, s.ff_act = FF_DENSE, mlp["ff"], float(mlp["limit"]), ACT_CLAMP
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            s.ff_kind, s.ff, s.ff_act = FF_MOE, mlp["expert"]["ff"], ACT_SILU
            s.experts, s.top = r["experts"], r["top"]
            s.router_kind, s.router_biased = ROUTER_TOP_SOFTMAX, True
            if mlp.get("shared"):
                s.shared_ff, s.shared_gated = mlp["shared"]["ff"], False
        else:
            raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
    return s


def mirorax_config(cfg: dict, max_tokens: int = 4096, weight_dtype: int = M.BF16) -> LayeredConfig:
    """config.json of a Mirorax checkpoint -> LayeredConfig whose layers are the layer RUNS (the
    looped run unrolled; a repeated run shares the tensors of its first pass). Every size and
    every constant that can differ between models of the design is read from cfg."""
    first = {}
    runs = []
    for i, step in unroll_loop(cfg["layers"], cfg.get("loop")):
        s = _mirorax_layer(cfg["layers"][i])
        s.pre_added = step is not None
        s.shares = first.get(i, -1)
        first.setdefault(i, len(runs))
        runs.append(s)
    return LayeredConfig(
        arch="Mirorax", width=cfg["width"], vocab=cfg["vocab"], layers=runs, embed_scale=1.0,
        norm_eps=float(cfg["norm"]["eps"]), max_tokens=max_tokens, weight_dtype=weight_dtype, norm_kind=NORM_RMS,
        pre_norm=True, pos_embed=False, block_kind=BLOCK_PARALLEL,
    )


def mirorax_tensor_shapes(cfg: dict) -> dict:
    """Checkpoint tensor name -> shape for a Mirorax config.json."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,), "head": (cfg["vocab"], W)}
    if cfg.get("loop"):
        out["loop.step"] = (cfg["loop"]["times"], W)
    for i, e in enumerate(cfg["layers"]):
        p, m = f"l{i}.", e["mixer"]
        x = p + "mix."
        out[p + "norm1"] = out[p + "ls1"] = (W,)
        H, D, V = m["heads"], m["dim"], m["vdim"]
        if e["type"] == "attention":
            G = m.get("kv_heads", H)
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                out[x + n], out[x + n + ".b"] = (rows, W), (rows,)
            out[x + "g"], out[x + "o"], out[x + "o.b"] = (H * V, W), (W, H * V), (W,)
        else:
            R, rank = m["rot_dim"], m["kv_rank"]
            out[x + "q"], out[x + "dkv"], out[x + "dkv.norm"] = (H * (D + R), W), (rank + R, W), (rank,)
            out[x + "uk"], out[x + "uv"], out[x + "sink"], out[x + "o"] = (H * D, rank), (H * V, rank), (H,), (W, H * V)
        mlp = e.get("mlp")
        if not mlp:
            continue
        out[p + "ls2"] = (W,)
        f = p + "mlp."
        if mlp["kind"] == "dense":
            out[f + "gate"] = out[f + "up"] = (mlp["ff"], W)
            out[f + "down"] = (W, mlp["ff"])
        else:
            ff, E = mlp["expert"]["ff"], mlp["router"]["experts"]
            for k in range(E):
                out[f"{f}e{k}.gate"] = out[f"{f}e{k}.up"] = (ff, W)
                out[f"{f}e{k}.down"] = (W, ff)
            out[f + "router"], out[f + "router.b"] = (E, W), (E,)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                out[f + "shared.gate"] = out[f + "shared.up"] = (sf, W)
                out[f + "shared.down"] = (W, sf)
    return out


def mirorax_pack(c: LayeredConfig, t: dict, cfg: dict = None) -> dict:
    """Checkpoint tensors -> the engine's tensors (see sinulorn_pack), one dict per layer run;
    a repeated run holds the very arrays of its first pass (uploaded once) and its own pre_add."""
    dt = c.weight_dtype
    order = unroll_loop(cfg["layers"], cfg.get("loop"))

    def w(*names):
        parts = [_as_weight(t[n], dt) for n in names]
        return parts[0] if len(parts) == 1 else np.ascontiguousarray(np.concatenate(parts, axis=0))

    def f(name):
        return np.ascontiguousarray(_as_f32(t[name]))

    runs = []
    for r, (l, (i, step)) in enumerate(zip(c.layers, order)):
        own = {}
        if step is not None:
            own["pre_add"] = np.ascontiguousarray(f("loop.step")[step])
        if l.shares >= 0:
            d = {k: v for k, v in runs[l.shares].items() if k != "pre_add"}
            d.update(own)
            runs.append(d)
            continue
        p, x, m = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        d = dict(own, norm1=f(p + "norm1"), ls1=f(p + "ls1"))
        if l.mixer == MIX_ATTN:
            d["w_in"] = w(x + "q", x + "k", x + "v", x + "g")
            b = np.zeros(l.in_rows, np.float32)  # the gate rows have no bias
            qkv = np.concatenate([f(x + "q.b"), f(x + "k.b"), f(x + "v.b")])
            b[:qkv.size] = qkv
            d.update(in_bias=b, o_bias=f(x + "o.b"))
        else:
            d["w_in"] = w(x + "q", x + "dkv")
            d.update(kv_norm=f(x + "dkv.norm"), sink_w=f(x + "sink"), w_ukv=w(x + "uk", x + "uv"))
            uk = _as_weight(t[x + "uk"], dt).reshape(l.heads, l.dim, l.kv_rank)
            d["w_ukt"] = np.ascontiguousarray(uk.transpose(0, 2, 1))
        d["w_o"] = w(x + "o")
        if l.ff_kind != FF_NONE:
            d["ls2"] = f(p + "ls2")
        if l.ff_kind == FF_DENSE:
            d.update(w_gate=w(m + "gate"), w_up=w(m + "up"), w_down=w(m + "down"))
        elif l.ff_kind == FF_MOE:
            d.update(router=f(m + "router"), router_bias=f(m + "router.b"))
            for k in ("gate", "up", "down"):
                d["w_" + k] = np.ascontiguousarray(
                    np.stack([_as_weight(t[f"{m}e{e}.{k}"], dt) for e in range(l.experts)]))
            if l.shared_ff:
                d.update(ws_gate=w(m + "shared.gate"), ws_up=w(m + "shared.up"), ws_down=w(m + "shared.down"))
        want = packed_shapes(c, l)
        if set(want) != set(d):
            raise ValueError(f"layer {i}: packed tensors {sorted(d)} do not match the configuration's {sorted(want)}")
        for k, (shape, _) in want.items():
            if tuple(d[k].shape) != tuple(shape):
                raise ValueError(f"layer {i}: tensor {k} has shape {d[k].shape}, the configuration gives {shape}")
        runs.append(d)
    return {"embed": w("embed"), "final_norm": f("final.norm"), "head": w("head"), "layers": runs}


def mirorax_random_tensors(cfg: dict, seed: int = 0, gain: float = 1.0) -> dict:
    """Random checkpoint tensors for a Mirorax config.json, as float32 arrays already rounded
    to bf16 values (the f32 and bf16 engines and a float64 restatement see the same weights)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in mirorax_tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf == "norm1" or name.endswith(".norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf in ("ls1", "ls2"):
            a = rng.uniform(0.3, 1.1, shape) * rng.choice([-1.0, 1.0], shape)
        elif leaf == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif leaf == "sink":
            a = rng.uniform(-1.0, 2.0, shape)
        elif leaf == "step":
            a = 0.3 * rng.standard_normal(shape)
        elif leaf == "embed":
            a = 0.5 * rng.standard_normal(shape)
        else:
            a = gain * rng.standard_normal(shape) / np.sqrt(shape[-1])
        out[name] = bf16_to_f32(f32_to_bf16(a.astype(np.float32))).reshape(shape)
    return out


# ------------------------------------------------------------------ Lifenex
# x = rms(E[token]) w_e. Every layer is a parallel block with a norm per sublayer: x += mixer(rms(x)
# w1) + ff(rms(x) w2). Two mixers:
#   "mamba2":   a selective state-space layer: W_in h = [gate | x | B | C | step]; x | B | C pass a
#               biased causal convolution and silu; per head dt = softplus(step + dt_bias), S <-
#               exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x; y silu(gate) rms-normed in norm_groups
#               equal parts; W_o;
#   "parallel": two mixers on the same input, result = (rms(left) w_l + rms(right) w_r) / 2:
#               left, softmax attention without rotation (per-head weighted rms norm of queries and
#               keys, query temperature 1 + coef ln(floor((p + 1) / every) + 1), a learned bias per
#               head and bucketed distance added to the scaled score, a learned sink in the
#               denominator); right, a gated delta rule with one decay per head and key channel
#               (low-rank decay and gate projections, sigmoid output gate).
# Feed-forwards: "dense" W_d relu(W_u h)^2; "moe": silu-gated experts, scores sigmoid(W_r h), the
# choice by score + correction within the best groups (a group's rank: the sum of its two best),
# weights the plain scores, plus a shared expert times sigmoid(w_sg . h). Logits: the embedding
# table on the final norm, times logit_scale.
LIFENEX_MIXERS = ("mamba2", "parallel")


def _lifenex_layer(e: dict) -> LayerSpec:
    m = e["mixer"]
    if e["type"] == "mamba2":
        s = LayerSpec(MIX_SSM, heads=m["heads"], vdim=m["vdim"], ssm_state=m["state"], ssm_groups=m.get("groups", 1),
                      norm_groups=m.get("norm_groups", 1), conv=m["conv"])
    elif e["type"] == "parallel":
        a, d = m["left"], m["right"]
        qt = a.get("q_temp") or {}
        s = LayerSpec(MIX_ATTN, heads=a["heads"], kv_heads=a.get("kv_heads", a["heads"]), dim=a["dim"], vdim=a["vdim"],
                      attn_scale=float(a["scale"]), mask_kind=MASK_CAUSAL, qk_norm=QK_HEAD_W, sink=1, sink_learned=True,
                      q_temp_coef=float(qt.get("coef", 0.0)), q_temp_every=int(qt.get("every", 0)),
                      rel_max=float(a["bias_max"]), rel_rows=-1, join_scale=0.5)
        s.side = LayerSpec(MIX_DELTA, heads=d["heads"], kv_heads=d.get("kv_heads", d["heads"]), dim=d["dim"],
                           vdim=d["vdim"], conv=d["conv"], decay_rank=-1, gate_rank=-1, gate_act=DELTA_GATE_SIGMOID)
    else:
        raise ValueError(f"unknown mixer type {e['type']!r}")
    s.ff_normed, s.layer_scaled = True, False
    mlp = e.get("mlp")
    if mlp:
        if mlp["kind"] == "dense":
            s.ff_kind, s.ff, s.ff_act = FF_PLAIN, mlp["ff"], ACT_RELU2
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            s.ff_kind, s.ff, s.ff_act = FF_MOE, mlp["expert"]["ff"], ACT_SILU
            s.experts, s.top, s.groups, s.groups_keep = r["experts"], r["top"], g["count"], g["keep"]
            s.router_kind, s.router_biased, s.router_scale = ROUTER_SIGMOID_GROUPS, True, 1.0
            if mlp.get("shared"):
                s.shared_ff, s.shared_gated = mlp["shared"]["ff"], True
        else:
            raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
    return s


def lifenex_config(cfg: dict, max_tokens: int = 4096, weight_dtype: int = M.BF16, shapes: dict = None) -> LayeredConfig:
    """config.json of a Lifenex checkpoint -> LayeredConfig. Every size and every constant that
    can differ between models of the design is read from cfg; the sizes config.json does not
    name (rows of the distance-bias table, ranks of the low-rank decay and gate) are the
    checkpoint tensors' own: shapes maps tensor names to shapes."""
    layers = []
    for i, e in enumerate(cfg["layers"]):
        s = _lifenex_layer(e)
        if s.side is not None:
            if shapes is None:
                raise ValueError("a Lifenex 'parallel' layer takes sizes from the checkpoint's tensor shapes")
            s.rel_rows = int(shapes[f"l{i}.mix.left.rel"][0])
            s.side.decay_rank = int(shapes[f"l{i}.mix.right.a1"][0])
            s.side.gate_rank = int(shapes[f"l{i}.mix.right.g1"][0])
        layers.append(s)
    return LayeredConfig(
        arch="Lifenex", width=cfg["width"], vocab=cfg["vocab"], layers=layers, embed_scale=1.0,
        norm_eps=float(cfg["norm"]["eps"]), max_tokens=max_tokens, weight_dtype=weight_dtype, norm_kind=NORM_RMS,
        pre_norm=True, pos_embed=False, logit_scale=float(cfg.get("logit_scale", 1.0)), tied_head=True,
        block_kind=BLOCK_PARALLEL, embed_normed=True,
    )


def lifenex_tensor_shapes(cfg: dict, rel_rows: int = 16, decay_rank: int = 8, gate_rank: int = 8) -> dict:
    """Checkpoint tensor name -> shape for a Lifenex config.json; the three sizes config.json
    does not name are arguments."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "embed.norm": (W,), "final.norm": (W,)}
    for i, e in enumerate(cfg["layers"]):
        p, m = f"l{i}.", e["mixer"]
        x = p + "mix."
        out[p + "norm1"] = (W,)
        if e["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m.get("groups", 1)
            inner, cc = H * P, H * P + 2 * G * N
            out[x + "in"], out[x + "conv"], out[x + "conv.b"] = (2 * inner + 2 * G * N + H, W), (cc, m["conv"]), (cc,)
            out[x + "dt_bias"] = out[x + "A_log"] = out[x + "D"] = (H,)
            out[x + "norm"], out[x + "o"] = (inner,), (W, inner)
        else:
            a, d = m["left"], m["right"]
            H, G, D, V = a["heads"], a.get("kv_heads", a["heads"]), a["dim"], a["vdim"]
            y = x + "left."
            out[y + "q"], out[y + "k"], out[y + "v"], out[y + "o"] = (H * D, W), (G * D, W), (G * V, W), (W, H * V)
            out[y + "q.norm"] = out[y + "k.norm"] = (D,)
            out[y + "rel"], out[y + "sink"] = (rel_rows, H), (H,)
            H, KH, D, V = d["heads"], d.get("kv_heads", d["heads"]), d["dim"], d["vdim"]
            y = x + "right."
            for n, rows in (("q", KH * D), ("k", KH * D), ("v", H * V)):
                out[y + n], out[y + n + ".conv"] = (rows, W), (rows, d["conv"])
            out[y + "b"], out[y + "A_log"], out[y + "norm"] = (H, W), (H,), (V,)
            out[y + "a1"], out[y + "a2"], out[y + "dt_bias"] = (decay_rank, W), (H * D, decay_rank), (H * D,)
            out[y + "g1"], out[y + "g2"], out[y + "o"] = (gate_rank, W), (H * V, gate_rank), (W, H * V)
            out[x + "left.out"] = out[x + "right.out"] = (W,)
        mlp = e.get("mlp")
        if not mlp:
            continue
        out[p + "norm2"] = (W,)
        f = p + "mlp."
        if mlp["kind"] == "dense":
            out[f + "up"], out[f + "down"] = (mlp["ff"], W), (W, mlp["ff"])
        else:
            ff, E = mlp["expert"]["ff"], mlp["router"]["experts"]
            for k in range(E):
                out[f"{f}e{k}.gate"] = out[f"{f}e{k}.up"] = (ff, W)
                out[f"{f}e{k}.down"] = (W, ff)
            out[f + "router"], out[f + "correction"] = (E, W), (E,)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                out[f + "shared.gate"] = out[f + "shared.up"] = (sf, W)
                out[f + "shared.down"], out[f + "shared.sg"] = (W, sf), (1, W)
    return out


def _check_packed(where: str, want: dict, d: dict) -> None:
    if set(want) != set(d):
        raise ValueError(f"{where}: packed tensors {sorted(d)} do not match the configuration's {sorted(want)}")
    for k, (shape, _) in want.items():
        if tuple(d[k].shape) != tuple(shape):
            raise ValueError(f"{where}: tensor {k} has shape {d[k].shape}, the configuration gives {shape}")


def lifenex_pack(c: LayeredConfig, t: dict) -> dict:
    """Checkpoint tensors -> the engine's tensors (see sinulorn_pack). The input projections of a
    mixer become one w_in (attention: q | k | v; delta rule: q | k | v | gate down | beta | decay
    down); a layer's second mixer is the nested dict "side"."""
    dt = c.weight_dtype

    def w(*names):
        parts = [_as_weight(t[n], dt) for n in names]
        return parts[0] if len(parts) == 1 else np.ascontiguousarray(np.concatenate(parts, axis=0))

    def f(name):
        return np.ascontiguousarray(_as_f32(t[name]))

    layers = []
    for i, l in enumerate(c.layers):
        p, x, m = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        d = {"norm1": f(p + "norm1")}
        if l.mixer == MIX_SSM:
            d.update(w_in=w(x + "in"), conv_w=f(x + "conv"), conv_b=f(x + "conv.b"), a_log=f(x + "A_log"),
                     dt_bias=f(x + "dt_bias"), d_skip=f(x + "D"), out_norm=f(x + "norm"), w_o=w(x + "o"))
        else:
            y = x + "left."
            d.update(w_in=w(y + "q", y + "k", y + "v"), q_norm=f(y + "q.norm"), kv_norm=f(y + "k.norm"),
                     rel=f(y + "rel"), sink_w=f(y + "sink"), w_o=w(y + "o"), join_w=f(x + "left.out"),
                     side_join_w=f(x + "right.out"))
            y = x + "right."
            sd = {"w_in": w(y + "q", y + "k", y + "v", y + "g1", y + "b", y + "a1"),
                  "conv_w": np.ascontiguousarray(np.concatenate([f(y + n + ".conv") for n in ("q", "k", "v")], axis=0)),
                  "a_log": f(y + "A_log"), "dt_bias": f(y + "dt_bias"), "out_norm": f(y + "norm"),
                  "w_a2": w(y + "a2"), "w_g2": w(y + "g2"), "w_o": w(y + "o")}
            _check_packed(f"layer {i}, second mixer", packed_shapes(c, l.side, side=True), sd)
        if l.ff_kind != FF_NONE:
            d["norm2"] = f(p + "norm2")
        if l.ff_kind == FF_PLAIN:
            d.update(w_up=w(m + "up"), w_down=w(m + "down"))
        elif l.ff_kind == FF_MOE:
            d.update(router=f(m + "router"), router_bias=f(m + "correction"))
            for k in ("gate", "up", "down"):
                d["w_" + k] = np.ascontiguousarray(
                    np.stack([_as_weight(t[f"{m}e{e}.{k}"], dt) for e in range(l.experts)]))
            if l.shared_ff:
                d.update(ws_gate=w(m + "shared.gate"), ws_up=w(m + "shared.up"), ws_down=w(m + "shared.down"),
                         shared_sg=f(m + "shared.sg").reshape(-1))
        _check_packed(f"layer {i}", packed_shapes(c, l), d)
        if l.side is not None:
            d["side"] = sd
        layers.append(d)
    emb = w("embed")
    return {"embed": emb, "embed_norm": f("embed.norm"), "final_norm": f("final.norm"), "head": emb, "layers": layers}


def lifenex_random_tensors(cfg: dict, seed: int = 0, gain: float = 1.0, **sizes) -> dict:
    """Random checkpoint tensors for a Lifenex config.json, as float32 arrays already rounded to
    bf16 values (the f32 and bf16 engines and a float64 restatement see the same weights)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in lifenex_tensor_shapes(cfg, **sizes).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2", "out") or name.endswith(".norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "b" and len(shape) == 1:
            a = 0.3 * rng.standard_normal(shape)
        elif leaf == "conv":
            a = 0.5 * rng.standard_normal(shape)
        elif leaf == "A_log":
            a = rng.uniform(-3.0, 0.5, shape)
        elif leaf == "dt_bias":
            a = rng.uniform(-2.0, 1.0, shape)
        elif leaf == "D":
            a = rng.uniform(0.5, 1.5, shape)
        elif leaf == "rel":
            a = 0.7 * rng.standard_normal(shape)
        elif leaf == "sink":
            a = rng.uniform(-1.0, 2.0, shape)
        elif leaf == "correction":
            a = 0.2 * rng.standard_normal(shape)
        elif leaf == "embed":
            a = 0.5 * rng.standard_normal(shape)
        else:
            a = gain * rng.standard_normal(shape) / np.sqrt(shape[-1])
        out[name] = bf16_to_f32(f32_to_bf16(a.astype(np.float32))).reshape(shape)
    return out


# ------------------------------------------------------------------ registry
# design name (config.json "architecture") -> (config reader, weight packer)
DESIGNS = {"Sinulorn": (sinulorn_config, sinulorn_pack), "Lenuzen": (lenuzen_config, lenuzen_pack),
           "Mirorax": (mirorax_config, lambda c, t, cfg=None: mirorax_pack(c, t, cfg)),
           "Lifenex": (lifenex_config, lifenex_pack)}


def read_checkpoint(path: str, max_tokens: int = 4096, weight_dtype: int = M.BF16):
    """A checkpoint folder -> (LayeredConfig, packed engine tensors). The design is
    chosen by config.json's "architecture"."""
    from .yalmfile import read_yalm

    with open(os.path.join(path, "config.json")) as fh:
        cfg = json.load(fh)
    arch = cfg.get("architecture")
    if arch not in DESIGNS:
        raise ValueError(f"architecture {arch!r} is not a layer-list design this engine knows ({sorted(DESIGNS)})")
    reader, packer = DESIGNS[arch]
    yd = read_yalm(os.path.join(path, "model.safetensors"))
    try:
        if arch == "Lifenex":  # some sizes are the tensors' own
            c = reader(cfg, max_tokens, weight_dtype, {k: tuple(v.shape) for k, v in yd.tensors.items()})
        else:
            c = reader(cfg, max_tokens, weight_dtype)
        t = {k: np.asarray(v.data).reshape(v.shape) for k, v in yd.tensors.items()}
        return c, (packer(c, t, cfg) if arch == "Mirorax" else packer(c, t))
    finally:
        yd.close()
