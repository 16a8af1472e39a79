"""Layer-list models on the HIP backend (include/ps_hip.h, "layer-list models"): configuration, weight loading and the model object.

A model directory holds config.json and model.safetensors.  config.json names the architecture; ARCHITECTURES maps it to the function that
turns the configuration and the tensors into layer descriptors.  Every size and constant comes from config.json or a tensor's shape.

Ranutar: a list of layers, each  x += norm_b(mixer(conv(norm(x))))  and, where it has one,  x += norm_b(ff(conv(norm(x)))), the mixer one of
  wkv               per-channel decayed outer-product state with token-shift mixes and a bonus for the current token
  delta             gated delta rule with short convolutions on q / k / v
  latent_attention  attention over a low-rank latent + one shared rotated key part, sliding window
the norms RMS norms whose stored weight is the deviation from one, the feed-forward two dense matrices around the xIELU activation.

Vobisun: PARALLEL layers,  h = norm(x); x += mixer(h + conv(h)) + ff(h), plain norm weights, a scaled embedding, a SiLU-gated feed-forward, a stretch
of layers that runs several times with the same weights (config 'loop'; every pass has its own state), and the mixer type
  parallel          two mixers side by side on the same input, their outputs added with a scale each:
                    left  = grouped-query attention over a sliding window plus one mean key / value per block of 'pool' tokens wholly before the window,
                            a sink in the soft-max denominator, a temperature per head, RMS norms over the whole q / k projections, rotary on neighbouring
                            pairs of the first rot.dims numbers of a head with linearly scaled positions, a sigmoid gate per head;
                    right = gated linear attention (a decay per key channel from a two-matrix projection).

Zusolix: PARALLEL layers with two norms of the same vector,  y = x + r * (mix(n1(x)) + mlp(n2(x))), RMS norms taken over 'norm.groups' equal parts of
the vector, no input filter, a scaled embedding; what a layer hands on is a weighted average over the embedding and ALL layers' results so far (the layer's
'dwa' weights).  Mixers:
  attention         grouped-query soft-max attention over everything before the token, biases on q / k / v, no rotation; the query grows with the position
                    (1 + coef ln(floor((p + 1) / every) + 1)), scores pass scale, then softcap * tanh(. / softcap)
  mingru            an element-wise gated recurrence: z = sigmoid(W_z h + b), c = u + 1/2 (u >= 0) or sigmoid(u) with u = W_x h + b, S <- (1 - z) S + z c,
                    output W_o (S * silu(W_g h))
Feed-forward: SiLU-gated dense, or a mixture of such experts -- sigmoid router in fp32, the 'top' largest scores, a chosen expert's score multiplies its INPUT,
plus a shared expert for every token times sigmoid of a one-row projection.

Pokatar: PRE-NORM layers,  x += mix(ln1(x)); x += mlp(ln2(x)), the norms layer norms (mean taken off, a weight, no bias), logits against the embedding table itself.
Mixers:
  attention         grouped-query causal soft-max attention without positions: per-head RMS norms of q and k (one weight vector shared by the heads), every head's
                    value a unit-rms vector, a sink of score 0 in the denominator, sigmoid(W_g h) element by element on the concatenated heads
  latent_attention  queries straight from the input, keys / values through one normed latent plus one rotated key part shared by the heads; rotate-half rotary whose
                    frequencies are scaled by wavelength (slow pairs divided by a factor, a ramp between, cos and sin stretched); causal; a sigmoid gate per head
Feed-forward: relu-gated dense with biases, or a mixture of squared-relu experts -- soft-max router in fp32 over experts AND identity experts (output = input), a
correction added to the scores for the choice only, the choice limited to the best groups of neighbouring router rows, the chosen scores (not renormalised) on the
experts' outputs, plus a shared expert for every token.
"""
from __future__ import annotations

import ctypes as C
import json
import os

import numpy as np

from . import hip
from .safetensors_io import SafeTensors

MIX_WKV, MIX_DELTA, MIX_LATENT, MIX_WINATTN, MIX_GLA, MIX_MINGRU = 1, 2, 3, 4, 5, 6
FF_NONE, FF_DENSE_XIELU, FF_DENSE_SWIGLU, FF_MOE_SWIGLU, FF_DENSE_RELU_GLU, FF_MOE_RELU2 = 0, 1, 2, 3, 4, 5
LAYER_SEQUENTIAL, LAYER_PARALLEL, LAYER_PRENORM = 0, 1, 2
ROT_HALVES, ROT_NEIGHBOURS = 0, 1


class ConfigError(ValueError):
    pass


def _ranutar_layers(cfg: dict, st: SafeTensors, up) -> tuple[list, dict]:
    """-> (list of hip.SeqLayer, top-level fields).  up.vec(array) / up.mat(bits) put a tensor on the device and return its handle."""
    width = int(cfg["width"])
    taps = int(cfg["canon"]["taps"])
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        p, mc, kind = f"l{i}.", lc["mixer"], lc["type"]
        L = hip.SeqLayer()
        for n in ("norm1", "norm1b"):
            setattr(L, n, up.vec(st.f32(p + n)))
        L.canon1 = up.vec(_expect(st, p + "canon1", (width, taps)))
        mlp = lc.get("mlp")
        if mlp:
            if mlp.get("kind") != "dense":
                raise ConfigError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not known")
            L.ff_kind, L.ff = FF_DENSE_XIELU, int(mlp["ff"])
            for n in ("norm2", "norm2b"):
                setattr(L, n, up.vec(st.f32(p + n)))
            L.canon2 = up.vec(_expect(st, p + "canon2", (width, taps)))
            act = st.f32(p + "mlp.act")
            L.ff_act_p, L.ff_act_q = float(act[0]), float(act[1])
            L.ff_up, L.ff_down = up.mat(st.bf16_bits(p + "mlp.up")), up.mat(st.bf16_bits(p + "mlp.down"))
        m = p + "mix."
        L.heads, L.dim = int(mc["heads"]), int(mc["dim"])
        if kind == "wkv":
            L.kind, L.vdim = MIX_WKV, L.dim
            L.decay_rank = st.shape(m + "w1")[0]
            L.in_r, L.in_k, L.in_v, L.in_g = (up.mat(st.bf16_bits(m + n)) for n in ("r", "k", "v", "g"))
            L.decay1, L.decay2, L.out = up.mat(st.bf16_bits(m + "w1")), up.mat(st.bf16_bits(m + "w2")), up.mat(st.bf16_bits(m + "o"))
            L.mu = up.vec(np.stack([st.f32(m + "mu." + n) for n in ("r", "k", "v", "g", "w")]))
            L.decay0, L.bonus, L.onorm = up.vec(st.f32(m + "w0")), up.vec(st.f32(m + "u").reshape(-1)), up.vec(st.f32(m + "norm"))
        elif kind == "delta":
            L.kind, L.kv_heads, L.vdim, L.conv_taps = MIX_DELTA, int(mc["kv_heads"]), int(mc["vdim"]), int(mc["conv"])
            L.in_cat = up.mat(np.concatenate([st.bf16_bits(m + n) for n in ("q", "k", "v", "g", "b", "a")], axis=0))
            L.conv = up.vec(np.concatenate([_expect(st, m + n + ".conv", (st.shape(m + n)[0], L.conv_taps)) for n in ("q", "k", "v")], axis=0))
            L.a_log, L.dt_bias, L.onorm = up.vec(st.f32(m + "A_log")), up.vec(st.f32(m + "dt_bias")), up.vec(st.f32(m + "norm"))
            L.out = up.mat(st.bf16_bits(m + "o"))
        elif kind == "latent_attention":
            L.kind, L.vdim = MIX_LATENT, int(mc["vdim"])
            L.q_rank, L.kv_rank, L.rot_dim = int(mc["q_rank"]), int(mc["kv_rank"]), int(mc["rot_dim"])
            L.rot_dims, L.rot_base = int(mc["rot"]["dims"]), float(mc["rot"]["base"])
            L.window, L.scale = int(mc["mask"]["size"]), float(mc["scale"])
            L.in_cat = up.mat(np.concatenate([st.bf16_bits(m + "dq"), st.bf16_bits(m + "dkv")], axis=0))
            L.uq = up.mat(st.bf16_bits(m + "uq"))
            L.ukv = up.mat(np.concatenate([st.bf16_bits(m + "uk"), st.bf16_bits(m + "uv")], axis=0))
            L.out = up.mat(st.bf16_bits(m + "o"))
            L.qnorm, L.kvnorm = up.vec(st.f32(m + "dq.norm")), up.vec(st.f32(m + "dkv.norm"))
        else:
            raise ConfigError(f"layer {i}: mixer type {kind!r} is not known")
        L.form, L.mix_scale = LAYER_SEQUENTIAL, 1.0
        layers.append(L)
    top = dict(width=width, vocab=int(cfg["vocab"]), canon_taps=taps, norm_eps=float(cfg["norm"]["eps"]), norm_offset=1.0,
               logit_scale=float(cfg["logit_scale"]), embed=up.mat(st.bf16_bits("embed")), head=up.mat(st.bf16_bits("head")),
               final_norm=up.vec(st.f32("final.norm")))
    return layers, top


def _expect(st: SafeTensors, name: str, shape: tuple) -> np.ndarray:
    if st.shape(name) != tuple(shape):
        raise ConfigError(f"tensor {name}: shape {st.shape(name)}, the configuration gives {tuple(shape)}")
    return st.f32(name)


def _stack(st: SafeTensors, names: list) -> np.ndarray:
    return np.concatenate([st.bf16_bits(n) for n in names], axis=0)


def window_attention_mixer(L, st: SafeTensors, up, m: str, mc: dict, where: str):
    """Fill descriptor L with a windowed-attention mixer (MIX_WINATTN) from the tensors under prefix m and its configuration mc.  Whatever the
    configuration or the file does not have does not exist: no bias, no norm, no temperature, no sink, no gate, no rotation, no pooled blocks."""
    L.kind = MIX_WINATTN
    L.heads, L.dim = int(mc["heads"]), int(mc["dim"])
    L.kv_heads, L.vdim = int(mc.get("kv_heads") or L.heads), int(mc.get("vdim") or L.dim)
    if L.heads % L.kv_heads:
        raise ConfigError(f"{where}: {L.heads} heads over {L.kv_heads} key / value heads")
    mask, rot = mc.get("mask") or {}, mc.get("rot") or {}
    L.window, L.pool = int(mask.get("size") or 0), int(mask.get("pool") or 0)
    L.rot_dims, L.rot_base, L.rot_pairing = int(rot.get("dims") or 0), float(rot.get("base") or 10000.0), ROT_NEIGHBOURS
    L.rot_factor = float((rot.get("scaling") or {}).get("factor") or 1.0)
    L.scale = float(mc["scale"]) if mc.get("scale") is not None else L.dim ** -0.5
    L.softcap = float(mc.get("softcap") or 0.0)
    qt = mc.get("q_temp") or {}
    L.qtemp_coef, L.qtemp_every = float(qt.get("coef") or 0.0), int(qt.get("every") or 0)
    rows = [(m + "q", L.heads * L.dim), (m + "k", L.kv_heads * L.dim), (m + "v", L.kv_heads * L.vdim)]
    L.gated = int(m + "g" in st)
    if L.gated:
        rows.append((m + "g", L.heads))
    for n, r in rows:
        if st.shape(n)[0] != r:
            raise ConfigError(f"tensor {n}: {st.shape(n)[0]} rows, the configuration gives {r}")
    L.in_cat = up.mat(_stack(st, [n for n, _ in rows]))
    if any(n + ".b" in st for n, _ in rows):
        L.in_bias = up.vec(np.concatenate([_expect(st, n + ".b", (r,)) if n + ".b" in st else np.zeros(r, np.float32) for n, r in rows]))
    if m + "q.norm" in st:
        L.qnorm = up.vec(_expect(st, m + "q.norm", (L.heads * L.dim,)))
    if m + "k.norm" in st:
        L.knorm = up.vec(_expect(st, m + "k.norm", (L.kv_heads * L.dim,)))
    if m + "temp" in st:
        L.temp = up.vec(_expect(st, m + "temp", (L.heads,)))
    if m + "sink" in st:
        L.sink = up.vec(_expect(st, m + "sink", (L.heads,)))
    L.out = up.mat(st.bf16_bits(m + "o"))


def gated_linear_mixer(L, st: SafeTensors, up, m: str, mc: dict, where: str):
    """Fill descriptor L with a gated-linear-attention mixer (MIX_GLA)."""
    L.kind = MIX_GLA
    L.heads, L.dim = int(mc["heads"]), int(mc["dim"])
    L.vdim, L.tau = int(mc.get("vdim") or L.dim), float(mc.get("tau") or 1.0)
    L.decay_rank = st.shape(m + "a1")[0]
    for n, r in (("q", L.heads * L.dim), ("k", L.heads * L.dim), ("v", L.heads * L.vdim), ("g", L.heads * L.vdim)):
        if st.shape(m + n)[0] != r:
            raise ConfigError(f"tensor {m + n}: {st.shape(m + n)[0]} rows, the configuration gives {r}")
    L.in_cat = up.mat(_stack(st, [m + n for n in ("q", "k", "v", "g", "a1")]))
    L.decay2 = up.mat(st.bf16_bits(m + "a2"))
    L.decay0 = up.vec(_expect(st, m + "a2.b", (L.heads * L.dim,)) if m + "a2.b" in st else np.zeros(L.heads * L.dim, np.float32))
    L.onorm = up.vec(_expect(st, m + "norm", (L.vdim,)))
    L.out = up.mat(st.bf16_bits(m + "o"))


def gated_recurrence_mixer(L, st: SafeTensors, up, m: str, mc: dict, where: str):
    """Fill descriptor L with an element-wise gated recurrence (MIX_MINGRU): z | x | g stacked with one bias vector (zeros where a projection has none)."""
    L.kind, L.heads = MIX_MINGRU, 1
    L.dim = L.vdim = int(mc["width"])
    for n in ("z", "x", "g"):
        if st.shape(m + n)[0] != L.dim:
            raise ConfigError(f"tensor {m + n}: {st.shape(m + n)[0]} rows, the configuration gives {L.dim} ({where})")
    L.in_cat = up.mat(_stack(st, [m + n for n in ("z", "x", "g")]))
    if any(m + n + ".b" in st for n in ("z", "x", "g")):
        L.in_bias = up.vec(np.concatenate([_expect(st, m + n + ".b", (L.dim,)) if m + n + ".b" in st else np.zeros(L.dim, np.float32) for n in ("z", "x", "g")]))
    L.out = up.mat(st.bf16_bits(m + "o"))


def _gate_up(st: SafeTensors, p: str, ff: int, width: int, where: str) -> np.ndarray:
    """rows gate_0, up_0, gate_1, ... of the feed-forward under prefix p: the pair meets in one epilogue"""
    gate, upw = st.bf16_bits(p + "gate"), st.bf16_bits(p + "up")
    if gate.shape != (ff, width) or upw.shape != (ff, width) or st.shape(p + "down") != (width, ff):
        raise ConfigError(f"{where}: feed-forward shapes {gate.shape} / {upw.shape} / {st.shape(p + 'down')}, the configuration gives {(ff, width)}")
    return np.stack([gate, upw], axis=1).reshape(2 * ff, width)


def gated_feed_forward(L, st: SafeTensors, up, p: str, mlp: dict, width: int, where: str):
    """Fill descriptor L's feed-forward from the tensors under prefix p: 'dense' (SiLU-gated) or 'moe' (experts e0, e1, ... of that form stacked into one
    matrix each way, an fp32 router, an optional shared expert with an optional one-row gate)."""
    kind = mlp.get("kind")
    if kind == "dense":
        L.ff_kind, L.ff = FF_DENSE_SWIGLU, int(mlp["ff"])
        L.ff_up, L.ff_down = up.mat(_gate_up(st, p, L.ff, width, where)), up.mat(st.bf16_bits(p + "down"))
    elif kind == "moe":
        r = mlp["router"]
        L.ff_kind, L.ff, L.experts, L.top = FF_MOE_SWIGLU, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"])
        if not 0 < L.top <= L.experts:
            raise ConfigError(f"{where}: top {L.top} of {L.experts} experts")
        L.ff_up = up.mat(np.concatenate([_gate_up(st, f"{p}e{e}.", L.ff, width, where) for e in range(L.experts)], axis=0))
        L.ff_down = up.mat(np.concatenate([st.bf16_bits(f"{p}e{e}.down") for e in range(L.experts)], axis=0))
        L.router = up.vec(_expect(st, p + "router", (L.experts, width)))
        if mlp.get("shared"):
            L.shared_ff = int(mlp["shared"]["ff"])
            L.shared_up, L.shared_down = up.mat(_gate_up(st, p + "shared.", L.shared_ff, width, where)), up.mat(st.bf16_bits(p + "shared.down"))
            if p + "shared.sg" in st:
                L.shared_gate = up.vec(_expect(st, p + "shared.sg", (1, width)).reshape(-1))
    else:
        raise ConfigError(f"{where}: feed-forward kind {kind!r} is not known")


def _zusolix_layers(cfg: dict, st: SafeTensors, up) -> tuple[list, dict]:
    width = int(cfg["width"])
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        p, mc, kind = f"l{i}.", lc["mixer"], lc["type"]
        L = hip.SeqLayer()
        L.form, L.mix_scale, L.res_scale = LAYER_PARALLEL, 1.0, float(cfg.get("residual_mult") or 1.0)
        L.norm1 = up.vec(_expect(st, p + "norm1", (width,)))
        if kind == "attention":
            window_attention_mixer(L, st, up, p + "mix.", mc, f"layer {i}")
        elif kind == "mingru":
            gated_recurrence_mixer(L, st, up, p + "mix.", mc, f"layer {i}")
        else:
            raise ConfigError(f"layer {i}: mixer type {kind!r} is not known")
        if lc.get("mlp"):
            L.norm2 = up.vec(_expect(st, p + "norm2", (width,)))
            gated_feed_forward(L, st, up, p + "mlp.", lc["mlp"], width, f"layer {i}")
        if p + "dwa" in st:
            L.depth_mix = up.vec(_expect(st, p + "dwa", (i + 2,)))
        layers.append(L)
    norm = cfg.get("norm") or {}
    top = dict(width=width, vocab=int(cfg["vocab"]), canon_taps=1, norm_eps=float(norm["eps"]), norm_groups=int(norm.get("groups") or 1), norm_offset=0.0,
               logit_scale=1.0, embed_scale=float((cfg.get("embedding") or {}).get("scale") or 1.0), embed=up.mat(st.bf16_bits("embed")),
               head=up.mat(st.bf16_bits("head")), final_norm=up.vec(_expect(st, "final.norm", (width,))))
    return layers, top


def sink_attention_mixer(L, st: SafeTensors, up, m: str, mc: dict, where: str):
    """Fill descriptor L with grouped-query causal attention whose q / k norms are taken per head (one weight vector of `dim`), whose values are unit-rms
    vectors, whose soft-max has a sink of score 0, and whose gate has a row per output element: MIX_WINATTN with those switches on.  What the file does not
    have does not exist (no norm, no gate)."""
    L.kind = MIX_WINATTN
    L.heads, L.dim = int(mc["heads"]), int(mc["dim"])
    L.kv_heads, L.vdim = int(mc.get("kv_heads") or L.heads), int(mc.get("vdim") or L.dim)
    if L.heads % L.kv_heads:
        raise ConfigError(f"{where}: {L.heads} heads over {L.kv_heads} key / value heads")
    L.window, L.pool, L.rot_dims, L.rot_base, L.rot_pairing = int((mc.get("mask") or {}).get("size") or 0), 0, 0, 10000.0, ROT_HALVES
    L.scale = float(mc["scale"]) if mc.get("scale") is not None else L.dim ** -0.5
    L.head_norm, L.v_unit = 1, 1
    rows = [(m + "q", L.heads * L.dim), (m + "k", L.kv_heads * L.dim), (m + "v", L.kv_heads * L.vdim)]
    if m + "g" in st:
        L.gated = 2
        rows.append((m + "g", L.heads * L.vdim))
    for n, r in rows:
        if st.shape(n)[0] != r:
            raise ConfigError(f"tensor {n}: {st.shape(n)[0]} rows, the configuration gives {r}")
    L.in_cat = up.mat(_stack(st, [n for n, _ in rows]))
    if m + "q.norm" in st:
        L.qnorm = up.vec(_expect(st, m + "q.norm", (L.dim,)))
    if m + "k.norm" in st:
        L.knorm = up.vec(_expect(st, m + "k.norm", (L.dim,)))
    L.sink = up.vec(np.zeros(L.heads, np.float32))  # exp(0) = 1 joins every head's denominator
    L.out = up.mat(st.bf16_bits(m + "o"))


def shared_key_latent_mixer(L, st: SafeTensors, up, m: str, mc: dict, where: str):
    """Fill descriptor L with latent attention whose queries come straight from the input (MIX_LATENT with q_rank 0): q | dkv | g stacked, uk | uv stacked,
    causal (window 0) unless the configuration has a mask, frequency scaling from rot.scaling, a gate row per head where the file has one."""
    L.kind, L.q_rank = MIX_LATENT, 0
    L.heads, L.dim, L.vdim = int(mc["heads"]), int(mc["dim"]), int(mc.get("vdim") or mc["dim"])
    L.kv_rank, L.rot_dim = int(mc["kv_rank"]), int(mc["rot_dim"])
    rot = mc.get("rot") or {}
    L.rot_dims, L.rot_base = int(rot.get("dims") or 0), float(rot.get("base") or 10000.0)
    sc = rot.get("scaling") or {}
    if sc:
        L.yarn_factor, L.yarn_fast, L.yarn_slow, L.yarn_original = float(sc["factor"]), float(sc["fast"]), float(sc["slow"]), int(sc["original"])
    L.window, L.scale = int((mc.get("mask") or {}).get("size") or 0), float(mc["scale"])
    rows = [(m + "q", L.heads * (L.dim + L.rot_dim)), (m + "dkv", L.kv_rank + L.rot_dim)]
    if m + "g" in st:
        L.gated = 1
        rows.append((m + "g", L.heads))
    for n, r in rows + [(m + "uk", L.heads * L.dim), (m + "uv", L.heads * L.vdim)]:
        if st.shape(n)[0] != r:
            raise ConfigError(f"tensor {n}: {st.shape(n)[0]} rows, the configuration gives {r} ({where})")
    L.in_cat = up.mat(_stack(st, [n for n, _ in rows]))
    L.ukv = up.mat(_stack(st, [m + "uk", m + "uv"]))
    L.kvnorm = up.vec(_expect(st, m + "dkv.norm", (L.kv_rank,)))
    L.out = up.mat(st.bf16_bits(m + "o"))


def relu_feed_forward(L, st: SafeTensors, up, p: str, mlp: dict, width: int, where: str):
    """Fill descriptor L's feed-forward: 'dense' = relu-gated with optional biases (gate / up rows and their biases interleaved), 'moe' = squared-relu experts
    e0, e1, ... stacked into one matrix each way, an fp32 router over experts + identity experts with an optional correction and group limit, the scores on the
    experts' outputs, an optional shared expert."""
    kind = mlp.get("kind")
    if kind == "dense":
        L.ff_kind, L.ff = FF_DENSE_RELU_GLU, int(mlp["ff"])
        L.ff_up, L.ff_down = up.mat(_gate_up(st, p, L.ff, width, where)), up.mat(st.bf16_bits(p + "down"))
        if p + "gate.b" in st or p + "up.b" in st:
            b = [_expect(st, p + n + ".b", (L.ff,)) if p + n + ".b" in st else np.zeros(L.ff, np.float32) for n in ("gate", "up")]
            L.ff_up_bias = up.vec(np.stack(b, axis=1).reshape(-1))
        if p + "down.b" in st:
            L.ff_down_bias = up.vec(_expect(st, p + "down.b", (width,)))
    elif kind == "moe":
        r = mlp["router"]
        L.ff_kind, L.ff, L.experts, L.top = FF_MOE_RELU2, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"])
        L.moe_identity, L.moe_softmax, L.moe_weight_output = int(r.get("identity") or 0), 1, 1
        rows = L.experts + L.moe_identity
        gr = r.get("groups") or {}
        L.moe_groups, L.moe_keep = int(gr.get("count") or 0), int(gr.get("keep") or 0)
        if not 0 < L.top <= rows or (L.moe_groups and (rows % L.moe_groups or not 0 < L.moe_keep <= L.moe_groups or L.top > L.moe_keep * (rows // L.moe_groups))):
            raise ConfigError(f"{where}: top {L.top} of {rows} router rows in {L.moe_groups} groups of which {L.moe_keep} stay")
        for e in range(L.experts):
            if st.shape(f"{p}e{e}.up") != (L.ff, width) or st.shape(f"{p}e{e}.down") != (width, L.ff):
                raise ConfigError(f"{where}: expert {e} shapes {st.shape(f'{p}e{e}.up')} / {st.shape(f'{p}e{e}.down')}, the configuration gives {(L.ff, width)}")
        L.ff_up = up.mat(_stack(st, [f"{p}e{e}.up" for e in range(L.experts)]))
        L.ff_down = up.mat(_stack(st, [f"{p}e{e}.down" for e in range(L.experts)]))
        L.router = up.vec(_expect(st, p + "router", (rows, width)))
        if p + "correction" in st:
            L.moe_correction = up.vec(_expect(st, p + "correction", (rows,)))
        if mlp.get("shared"):
            L.shared_ff = int(mlp["shared"]["ff"])
            if st.shape(p + "shared.up") != (L.shared_ff, width) or st.shape(p + "shared.down") != (width, L.shared_ff):
                raise ConfigError(f"{where}: shared expert shapes, the configuration gives {(L.shared_ff, width)}")
            L.shared_up, L.shared_down = up.mat(st.bf16_bits(p + "shared.up")), up.mat(st.bf16_bits(p + "shared.down"))
    else:
        raise ConfigError(f"{where}: feed-forward kind {kind!r} is not known")


def _pokatar_layers(cfg: dict, st: SafeTensors, up) -> tuple[list, dict]:
    width = int(cfg["width"])
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        p, mc, kind = f"l{i}.", lc["mixer"], lc["type"]
        L = hip.SeqLayer()
        L.form, L.mix_scale = LAYER_PRENORM, 1.0
        L.norm1 = up.vec(_expect(st, p + "norm1", (width,)))
        if kind == "attention":
            sink_attention_mixer(L, st, up, p + "mix.", mc, f"layer {i}")
        elif kind == "latent_attention":
            shared_key_latent_mixer(L, st, up, p + "mix.", mc, f"layer {i}")
        else:
            raise ConfigError(f"layer {i}: mixer type {kind!r} is not known")
        if lc.get("mlp"):
            L.norm2 = up.vec(_expect(st, p + "norm2", (width,)))
            relu_feed_forward(L, st, up, p + "mlp.", lc["mlp"], width, f"layer {i}")
        layers.append(L)
    embed = up.mat(st.bf16_bits("embed"))
    top = dict(width=width, vocab=int(cfg["vocab"]), canon_taps=1, norm_eps=float(cfg["norm"]["eps"]), norm_offset=0.0, norm_center=1, logit_scale=1.0,
               embed=embed, head=embed, final_norm=up.vec(_expect(st, "final.norm", (width,))))
    return layers, top


def _vobisun_layers(cfg: dict, st: SafeTensors, up) -> tuple[list, dict]:
    width = int(cfg["width"])
    taps = int((cfg.get("canon") or {}).get("taps") or 1)
    layers, keep = [], []
    for i, lc in enumerate(cfg["layers"]):
        p, mc, kind = f"l{i}.", lc["mixer"], lc["type"]
        L = hip.SeqLayer()
        L.form = LAYER_PARALLEL
        L.norm1 = up.vec(_expect(st, p + "norm1", (width,)))
        L.canon1 = up.vec(_expect(st, p + "canon1", (width, taps)) if p + "canon1" in st else np.zeros((width, taps), np.float32))
        mlp = lc.get("mlp")
        if mlp:
            if mlp.get("kind") != "dense":
                raise ConfigError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not known")
            L.ff_kind, L.ff = FF_DENSE_SWIGLU, int(mlp["ff"])
            gate, upw = st.bf16_bits(p + "mlp.gate"), st.bf16_bits(p + "mlp.up")
            if gate.shape != (L.ff, width) or upw.shape != (L.ff, width):
                raise ConfigError(f"layer {i}: feed-forward shapes {gate.shape} / {upw.shape}, the configuration gives {(L.ff, width)}")
            L.ff_up = up.mat(np.stack([gate, upw], axis=1).reshape(2 * L.ff, width))  # rows gate_0, up_0, gate_1, ...: the pair meets in one epilogue
            L.ff_down = up.mat(st.bf16_bits(p + "mlp.down"))
        if kind == "parallel":
            window_attention_mixer(L, st, up, p + "mix.left.", mc["left"], f"layer {i} (left)")
            L.mix_scale = float(mc.get("left_scale", 1.0))
            R = hip.SeqLayer()
            gated_linear_mixer(R, st, up, p + "mix.right.", mc["right"], f"layer {i} (right)")
            R.mix_scale = float(mc.get("right_scale", 1.0))
            keep.append(R)
            L.beside = C.pointer(R)
        else:
            raise ConfigError(f"layer {i}: mixer type {kind!r} is not known")
        layers.append(L)
    loop = cfg.get("loop") or {}
    top = dict(width=width, vocab=int(cfg["vocab"]), canon_taps=taps, norm_eps=float(cfg["norm"]["eps"]), norm_offset=0.0, logit_scale=1.0,
               embed_scale=float((cfg.get("embedding") or {}).get("scale") or 1.0), loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
               loop_times=int(loop.get("times", 1)) if loop else 1, embed=up.mat(st.bf16_bits("embed")), head=up.mat(st.bf16_bits("head")),
               final_norm=up.vec(_expect(st, "final.norm", (width,))), _keep=keep)
    return layers, top


ARCHITECTURES = {"Ranutar": _ranutar_layers, "Vobisun": _vobisun_layers, "Zusolix": _zusolix_layers, "Pokatar": _pokatar_layers}


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    if cfg.get("architecture") not in ARCHITECTURES:
        raise ConfigError(f"unknown architecture {cfg.get('architecture')!r} (known: {sorted(ARCHITECTURES)})")
    return cfg


class _Uploader:
    def __init__(self, ctx: hip.Ctx, as_f32: bool):
        self.ctx, self.as_f32, self.vecs, self.mats = ctx, as_f32, [], []

    def vec(self, a: np.ndarray) -> int:
        d = self.ctx.to_device(np.ascontiguousarray(a, dtype=np.float32))
        self.vecs.append(d)
        return d.ptr

    def mat(self, bits: np.ndarray) -> int:
        bits = np.ascontiguousarray(bits, dtype=np.uint16)
        h = C.c_void_p()
        self.ctx.check(self.ctx.L.ps_hip_dense_upload(self.ctx.h, bits.ctypes.data_as(C.c_void_p), bits.shape[0], bits.shape[1], int(self.as_f32), C.byref(h)))
        self.mats.append(h.value)
        return h.value


class SeqModel:
    """ps_hip_seq over a model directory.  dtype "bfloat16": matrix products on bfloat16 operands, fp32 accumulation; "float32": fp32
    throughout.  Sequences live in slots (acquire / release); forward() is the step function, generate() the greedy / sampled loop."""

    def __init__(self, ctx: hip.Ctx, model_dir: str, dtype: str = "bfloat16", max_batch: int = 256, n_slots: int = 2, max_context: int = 0):
        if dtype not in ("bfloat16", "float32"):
            raise ConfigError(f"dtype {dtype!r}: bfloat16 or float32")
        self.ctx, self.dtype = ctx, dtype
        self.cfg = read_config(model_dir)
        self.arch = self.cfg["architecture"]
        st = SafeTensors(os.path.join(model_dir, "model.safetensors"))
        self._up = _Uploader(ctx, dtype == "float32")
        layers, top = ARCHITECTURES[self.arch](self.cfg, st, self._up)
        self._layers = (hip.SeqLayer * len(layers))(*layers)
        d = hip.SeqDesc()
        d.n_layers, d.max_batch, d.n_slots, d.compute = len(layers), int(max_batch), int(n_slots), int(dtype == "float32")
        d.max_context = int(max_context)  # most tokens of one sequence, for the memory that grows with it (0: the library's default)
        self._keep = top.pop("_keep", None)  # descriptors of second mixers, pointed to from the layers
        for k, v in top.items():
            setattr(d, k, v)
        d.layers = self._layers
        self.vocab, self.width, self.n_layers, self.max_batch = d.vocab, d.width, d.n_layers, int(max_batch)
        h = C.c_void_p()
        ctx.check(ctx.L.ps_hip_seq_create(ctx.h, C.byref(d), C.byref(h)))
        self.h = h
        self.n_runs = int(ctx.L.ps_hip_seq_layer_runs(h))  # executions of a layer per forward (a looped stretch counts every time)
        self._dbg = None

    def close(self):
        if getattr(self, "h", None):
            self.ctx.L.ps_hip_seq_destroy(self.h)
            self.h = None
            for m in self._up.mats:
                self.ctx.L.ps_hip_dense_free(self.ctx.h, m)
            for v in self._up.vecs:
                v.free()
            if self._dbg is not None:
                self._dbg.free()

    # ---- state manager
    def acquire(self) -> int:
        s = C.c_int(-1)
        self.ctx.check(self.ctx.L.ps_hip_seq_acquire(self.h, C.byref(s)))
        return s.value

    def release(self, slot: int):
        self.ctx.check(self.ctx.L.ps_hip_seq_release(self.h, int(slot)))

    def position(self, slot: int) -> int:
        return int(self.ctx.L.ps_hip_seq_position(self.h, int(slot)))

    @property
    def slot_bytes(self) -> int:
        return int(self.ctx.L.ps_hip_seq_slot_bytes(self.h))

    @property
    def weight_bytes_per_token(self) -> int:
        return int(self.ctx.L.ps_hip_seq_weight_bytes_per_token(self.h))

    def set_mode(self, mode: int):
        self.ctx.L.ps_hip_seq_set_mode(self.h, int(mode))

    # ---- step function
    def forward(self, slot: int, tokens, want=None, argmax: bool = False):
        """The next tokens of the sequence in `slot`; want: ascending indices into them.  -> logits [len(want), vocab] (or their arg-max ids)."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        want = np.ascontiguousarray(want if want is not None else [], dtype=np.int32)
        out = np.empty((want.size, self.vocab), dtype=np.float32) if not argmax else None
        ids = np.empty(want.size, dtype=np.int32) if argmax else None
        self.ctx.check(self.ctx.L.ps_hip_seq_forward(self.h, int(slot), hip._ptr(tokens), tokens.size, hip._ptr(want) if want.size else None, want.size,
                                                     hip._ptr(out) if out is not None and want.size else None, hip._ptr(ids) if ids is not None and want.size else None))
        return ids if argmax else out

    def decode_greedy(self, slot: int, token: int, steps: int) -> np.ndarray:
        out = np.empty(steps, dtype=np.int32)
        self.ctx.check(self.ctx.L.ps_hip_seq_decode_greedy(self.h, int(slot), int(token), int(steps), hip._ptr(out)))
        return out

    def generate(self, prompt, steps: int, sampler=None) -> np.ndarray:
        """Prefill all but the last prompt token without logits, then `steps` tokens: greedy on the device (sampler None), or each step's logits
        through `sampler` (a callable logits -> token id, e.g. host.Sampler.sample)."""
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        slot = self.acquire()
        try:
            if prompt.size > 1:
                self.forward(slot, prompt[:-1])
            if sampler is None:
                return self.decode_greedy(slot, int(prompt[-1]), steps)
            out, tok = [], int(prompt[-1])
            for _ in range(steps):
                tok = int(sampler(self.forward(slot, [tok], want=[0])[0]))
                out.append(tok)
            return np.asarray(out, dtype=np.int32)
        finally:
            self.release(slot)

    # ---- diagnostics
    def capture_layers(self, on: bool = True):
        """Keep the residual stream after every layer run of the next forwards (each at most max_batch tokens)."""
        if on and self._dbg is None:
            self._dbg = self.ctx.empty((self.n_runs, self.max_batch, self.width), np.float32)
        self.ctx.check(self.ctx.L.ps_hip_seq_debug_layers(self.h, self._dbg.ptr if on else None))

    def layers(self, n_tokens: int) -> np.ndarray:
        self.ctx.sync()
        return self._dbg.numpy()[:, :n_tokens]


def is_seq_model_dir(model_dir: str) -> bool:
    return os.path.exists(os.path.join(model_dir, "config.json")) and os.path.exists(os.path.join(model_dir, "model.safetensors"))


def load_model(ctx: hip.Ctx, model_dir: str, **kw):
    """The registry's front door: config.json + model.safetensors -> SeqModel (by its architecture), model.json + ggml/weights.gguf -> hip.Model."""
    if is_seq_model_dir(model_dir):
        return SeqModel(ctx, model_dir, **kw)
    if os.path.exists(os.path.join(model_dir, "model.json")):
        kw.pop("dtype", None)
        kw.pop("n_slots", None)
        kw.pop("max_context", None)
        return hip.Model(ctx, model_dir, **kw)
    raise ConfigError(f"{model_dir}: neither config.json + model.safetensors nor model.json + ggml/weights.gguf")


class RequestScheduler:
    """Requests by id over a model's slots: a request's first tokens take a slot, later portions continue it, finish() gives the slot back.
    Requests are served one portion at a time in the order they are handed in."""

    def __init__(self, model: SeqModel):
        self.model, self.slots = model, {}

    def feed(self, rid, tokens, want=None) -> np.ndarray:
        if rid not in self.slots:
            self.slots[rid] = self.model.acquire()
        if len(tokens) == 0:
            return np.empty((0, self.model.vocab), dtype=np.float32)
        return self.model.forward(self.slots[rid], tokens, want)

    def finish(self, rid):
        s = self.slots.pop(rid, None)
        if s is not None:
            self.model.release(s)

    def live_tokens(self) -> int:
        return sum(self.model.position(s) for s in self.slots.values())
