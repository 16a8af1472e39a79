"""Host side of the layer-list models, no GPU: the safetensors reader, the configuration reader's mapping onto layer descriptors, the ctypes
mirror of the descriptors against the C header, and the plain statement's own invariances."""
import ctypes as C
import json
import os
import subprocess

import numpy as np
import pytest

import seq_oracle
from powerserve_amd import hip, safetensors_io, seqmodel, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
L = synth.seq_layer
CFG = synth.seq_config(24, 30, [L("delta", 20, heads=4, kv_heads=2, dim=6, vdim=10, conv=4), L("wkv", None, heads=3, dim=8),
                                L("latent_attention", 16, heads=2, dim=6, vdim=10, q_rank=7, kv_rank=9, rot_dim=4, rot={"base": 77.0, "dims": 4},
                                  mask={"size": 5}, scale=0.25)], taps=2, eps=1e-5, logit_scale=0.75)


def test_safetensors_round_trip_and_rounding(tmp_path):
    a = np.array([1.0, 1.00390625, 1.01171875, -3.0e-5, 65504.0, 0.0], dtype=np.float32)  # 1 + 2^-8 ties to even (down), 1 + 3 * 2^-8 ties up
    bits = safetensors_io.f32_to_bf16_bits(a)
    back = (bits.astype(np.uint32) << 16).view(np.float32)
    assert back[1] == 1.0 and back[2] == np.float32(1.015625) and back[0] == 1.0 and back[5] == 0.0
    t = {"w": np.arange(12, dtype=np.float32).reshape(3, 4), "idx": np.arange(5, dtype=np.int32)}
    p = str(tmp_path / "x.safetensors")
    safetensors_io.write(p, t)
    st = safetensors_io.SafeTensors(p)
    assert st.dtype("w") == "BF16" and st.dtype("idx") == "I32" and st.shape("w") == (3, 4)
    assert np.array_equal(st.f32("w"), t["w"]) and np.array_equal(st.raw("idx"), t["idx"])
    with pytest.raises(ValueError):
        st.bf16_bits("idx")


class FakeUp:
    def __init__(self):
        self.vecs, self.mats = [], []

    def vec(self, a):
        self.vecs.append(np.array(a))
        return len(self.vecs)

    def mat(self, bits):
        self.mats.append(np.array(bits))
        return 1000 + len(self.mats)


def test_configuration_maps_onto_layer_descriptors(tmp_path):
    t = synth.write_seq_model_dir(str(tmp_path), CFG, 1)
    cfg = seqmodel.read_config(str(tmp_path))
    up = FakeUp()
    layers, top = seqmodel.ARCHITECTURES[cfg["architecture"]](cfg, safetensors_io.SafeTensors(str(tmp_path / "model.safetensors")), up)
    assert (top["width"], top["vocab"], top["canon_taps"], top["norm_offset"]) == (24, 30, 2, 1.0)
    assert abs(top["norm_eps"] - 1e-5) < 1e-12 and top["logit_scale"] == 0.75
    d, w, a = layers
    assert (d.kind, d.heads, d.kv_heads, d.dim, d.vdim, d.conv_taps, d.ff_kind, d.ff) == (seqmodel.MIX_DELTA, 4, 2, 6, 10, 4, seqmodel.FF_DENSE_XIELU, 20)
    assert (w.kind, w.heads, w.dim, w.vdim, w.decay_rank, w.ff_kind) == (seqmodel.MIX_WKV, 3, 8, 8, 8, seqmodel.FF_NONE)
    assert (a.kind, a.q_rank, a.kv_rank, a.rot_dim, a.rot_dims, a.window) == (seqmodel.MIX_LATENT, 7, 9, 4, 4, 5)
    assert abs(a.rot_base - 77.0) < 1e-6 and abs(a.scale - 0.25) < 1e-9
    # the fused input projection of the delta mixer: rows q | k | v | g | b | a
    cat = up.mats[d.in_cat - 1001]
    assert cat.shape == (2 * 2 * 6 + 2 * 4 * 10 + 2 * 4, 24)
    want = np.concatenate([safetensors_io.f32_to_bf16_bits(t["l0.mix." + n]) for n in ("q", "k", "v", "g", "b", "a")])
    assert np.array_equal(cat, want)
    assert up.mats[a.ukv - 1001].shape == (2 * 6 + 2 * 10, 9) and up.mats[a.in_cat - 1001].shape == (7 + 9 + 4, 24)
    assert up.vecs[w.mu - 1].shape == (5, 24)


def test_unknown_names_are_refused(tmp_path):
    bad = dict(CFG, architecture="Somethingelse")
    synth.write_seq_model_dir(str(tmp_path), bad, 1, tensors=synth.seq_tensors(CFG, 1))
    with pytest.raises(seqmodel.ConfigError):
        seqmodel.read_config(str(tmp_path))
    bad = json.loads(json.dumps(CFG))
    bad["layers"][1]["type"] = "conveyor"
    with open(tmp_path / "config.json", "w") as f:
        json.dump(bad, f)
    with pytest.raises(seqmodel.ConfigError):
        seqmodel.ARCHITECTURES["Ranutar"](bad, safetensors_io.SafeTensors(str(tmp_path / "model.safetensors")), FakeUp())
    bad = json.loads(json.dumps(CFG))
    bad["canon"]["taps"] = 3  # the file's tensors have two taps
    with pytest.raises(seqmodel.ConfigError):
        seqmodel.ARCHITECTURES["Ranutar"](bad, safetensors_io.SafeTensors(str(tmp_path / "model.safetensors")), FakeUp())


def test_ctypes_descriptors_match_the_header(tmp_path):
    src = tmp_path / "sz.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "ps_hip.h"\nint main(void){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\\n", sizeof(ps_seq_layer), '
                   'offsetof(ps_seq_layer, norm1), offsetof(ps_seq_layer, kvnorm), sizeof(ps_seq_desc), offsetof(ps_seq_desc, embed), offsetof(ps_seq_desc, layers), '
                   'offsetof(ps_seq_layer, beside), offsetof(ps_seq_layer, in_bias), offsetof(ps_seq_layer, tau), offsetof(ps_seq_desc, embed_scale), '
                   'offsetof(ps_seq_desc, max_context));'
                   'printf("%zu %zu %zu %zu %zu %zu %zu\\n", offsetof(ps_seq_layer, res_scale), offsetof(ps_seq_layer, depth_mix), offsetof(ps_seq_layer, softcap), '
                   'offsetof(ps_seq_layer, qtemp_every), offsetof(ps_seq_layer, experts), offsetof(ps_seq_layer, shared_down), offsetof(ps_seq_desc, norm_groups));'
                   'printf("%zu %zu %zu %zu %zu %zu %zu\\n", offsetof(ps_seq_layer, head_norm), offsetof(ps_seq_layer, yarn_factor), offsetof(ps_seq_layer, yarn_original), '
                   'offsetof(ps_seq_layer, ff_up_bias), offsetof(ps_seq_layer, moe_identity), offsetof(ps_seq_layer, moe_correction), offsetof(ps_seq_desc, norm_center));return 0;}\n')
    exe = str(tmp_path / "sz")
    subprocess.run(["gcc", "-I" + os.path.join(ROOT, "include"), str(src), "-o", exe], check=True)
    got = [int(x) for x in subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()]
    assert got == [C.sizeof(hip.SeqLayer), hip.SeqLayer.norm1.offset, hip.SeqLayer.kvnorm.offset, C.sizeof(hip.SeqDesc), hip.SeqDesc.embed.offset,
                   hip.SeqDesc.layers.offset, hip.SeqLayer.beside.offset, hip.SeqLayer.in_bias.offset, hip.SeqLayer.tau.offset, hip.SeqDesc.embed_scale.offset,
                   hip.SeqDesc.max_context.offset,
                   hip.SeqLayer.res_scale.offset, hip.SeqLayer.depth_mix.offset, hip.SeqLayer.softcap.offset, hip.SeqLayer.qtemp_every.offset, hip.SeqLayer.experts.offset,
                   hip.SeqLayer.shared_down.offset, hip.SeqDesc.norm_groups.offset,
                   hip.SeqLayer.head_norm.offset, hip.SeqLayer.yarn_factor.offset, hip.SeqLayer.yarn_original.offset, hip.SeqLayer.ff_up_bias.offset,
                   hip.SeqLayer.moe_identity.offset, hip.SeqLayer.moe_correction.offset, hip.SeqDesc.norm_center.offset]


def test_plain_statement_is_causal_and_windowed():
    """what a later token is does not change earlier logits; a token outside every window and with the recurrent layers cut out does not matter"""
    t = synth.seq_tensors(CFG, 2)
    rng = np.random.default_rng(0)
    a = rng.integers(0, 30, 20)
    b = a.copy()
    b[12] = (b[12] + 1) % 30
    la, lb = seq_oracle.run(CFG, t, a), seq_oracle.run(CFG, t, b)
    assert np.array_equal(la[:12], lb[:12]) and np.abs(la[12:] - lb[12:]).max() > 1e-3
    only = synth.seq_config(24, 30, [CFG["layers"][2]], taps=2)
    t2 = synth.seq_tensors(only, 2)
    la, lb = seq_oracle.run(only, t2, a), seq_oracle.run(only, t2, b)
    # window 5 and a 2-tap input filter in front of the mixer and of the feed-forward: token 12 reaches positions 12 .. 12 + 4 + 1 + 1
    assert np.abs(la[19:] - lb[19:]).max() < 1e-12 and np.abs(la[12:19] - lb[12:19]).max() > 1e-6


PCFG = synth.parallel_config(24, 30, [
    synth.parallel_layer(20, dict(heads=4, kv_heads=2, dim=6, vdim=10, mask={"size": 5, "pool": 3}, rot={"base": 77.0, "dims": 4, "scaling": {"factor": 2.0}}, scale=0.25),
                         dict(heads=3, dim=8, vdim=4, tau=5.0), 1.25, 0.5),
    synth.parallel_layer(None, dict(heads=2, kv_heads=2, dim=6, vdim=6, mask={"size": 4, "pool": 2}, rot={"base": 9.0, "dims": 6}, scale=0.5),
                         dict(heads=1, dim=5, vdim=7, tau=1.0))], taps=2, eps=1e-5, embed_scale=3.0, loop=(0, 1, 2))


def test_parallel_configuration_maps_onto_layer_descriptors(tmp_path):
    t = synth.write_seq_model_dir(str(tmp_path), PCFG, 1)
    cfg = seqmodel.read_config(str(tmp_path))
    up = FakeUp()
    layers, top = seqmodel.ARCHITECTURES[cfg["architecture"]](cfg, safetensors_io.SafeTensors(str(tmp_path / "model.safetensors")), up)
    assert (top["width"], top["vocab"], top["canon_taps"], top["norm_offset"], top["embed_scale"]) == (24, 30, 2, 0.0, 3.0)
    assert (top["loop_start"], top["loop_stop"], top["loop_times"]) == (0, 1, 2)
    a, b = layers
    assert (a.form, a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.pool, a.rot_dims, a.rot_pairing, a.gated) == \
        (seqmodel.LAYER_PARALLEL, seqmodel.MIX_WINATTN, 4, 2, 6, 10, 5, 3, 4, seqmodel.ROT_NEIGHBOURS, 1)
    assert abs(a.rot_base - 77.0) < 1e-6 and a.rot_factor == 2.0 and a.scale == 0.25 and a.mix_scale == 1.25 and b.rot_factor == 1.0
    r = a.beside.contents
    assert (r.kind, r.heads, r.dim, r.vdim, r.decay_rank, r.tau, r.mix_scale) == (seqmodel.MIX_GLA, 3, 8, 4, 8, 5.0, 0.5)
    assert (a.ff_kind, a.ff, b.ff_kind) == (seqmodel.FF_DENSE_SWIGLU, 20, seqmodel.FF_NONE)
    # stacked input projections: q | k | v | gate with their biases (the gate has none), and q | k | v | g | a1
    cat = up.mats[a.in_cat - 1001]
    assert cat.shape == (4 * 6 + 2 * 6 + 2 * 10 + 4, 24)
    assert np.array_equal(cat, np.concatenate([safetensors_io.f32_to_bf16_bits(t["l0.mix.left." + n]) for n in ("q", "k", "v", "g")]))
    bias = up.vecs[a.in_bias - 1]
    assert bias.shape == (60,) and np.array_equal(bias[:24], t["l0.mix.left.q.b"]) and not bias[56:].any()
    assert up.mats[r.in_cat - 1001].shape == (2 * 3 * 8 + 2 * 3 * 4 + 8, 24)
    # the feed-forward's gate and up rows alternate
    both = up.mats[a.ff_up - 1001]
    assert both.shape == (40, 24)
    assert np.array_equal(both[0::2], safetensors_io.f32_to_bf16_bits(t["l0.mlp.gate"])) and np.array_equal(both[1::2], safetensors_io.f32_to_bf16_bits(t["l0.mlp.up"]))
    # what the file does not have does not exist
    st = safetensors_io.SafeTensors(str(tmp_path / "model.safetensors"))
    less = {n: st.f32(n) for n in st.names() if not n.endswith((".b", "temp", "sink", "q.norm", "left.g"))}
    cfg2 = json.loads(json.dumps(PCFG))
    del cfg2["loop"], cfg2["layers"][0]["mixer"]["left"]["rot"]
    synth.write_seq_model_dir(str(tmp_path / "less"), cfg2, 1, tensors=less)
    layers, top = seqmodel.ARCHITECTURES["Vobisun"](cfg2, safetensors_io.SafeTensors(str(tmp_path / "less" / "model.safetensors")), FakeUp())
    a = layers[0]
    assert (a.gated, a.in_bias, a.temp, a.sink, a.qnorm, a.rot_dims, top["loop_times"]) == (0, None, None, None, None, 0, 1) and a.knorm is not None
    bad = json.loads(json.dumps(PCFG))
    bad["layers"][0]["mixer"]["left"]["heads"] = 5
    with pytest.raises(seqmodel.ConfigError):
        seqmodel.ARCHITECTURES["Vobisun"](bad, st, FakeUp())


def test_plain_parallel_statement_reach():
    """causal; with the recurrent mixer switched off, a token reaches exactly as far as its window, then only through its block's mean; the layers of a loop run in order"""
    assert seq_oracle.layer_runs(PCFG) == [0, 0, 1] and seq_oracle.layer_runs({"layers": [0, 0, 0, 0], "loop": {"start": 1, "stop": 3, "times": 3}}) == [0, 1, 2, 1, 2, 1, 2, 3]
    assert list(seq_oracle.visible_tokens(9, 4)) == [6, 7, 8, 9] and list(seq_oracle.visible_blocks(9, 4, 3)) == [0, 1] and list(seq_oracle.visible_blocks(8, 4, 3)) == [0]
    assert list(seq_oracle.visible_blocks(3, 4, 3)) == [] and list(seq_oracle.visible_tokens(2, 4)) == [0, 1, 2]
    one = synth.parallel_config(24, 30, [synth.parallel_layer(None, PCFG["layers"][0]["mixer"]["left"], PCFG["layers"][0]["mixer"]["right"], 1.0, 0.0)], taps=1)
    t = synth.seq_tensors(one, 2)
    rng = np.random.default_rng(0)
    a = rng.integers(0, 30, 24)
    b = a.copy()
    b[7] = (b[7] + 1) % 30
    la, lb = seq_oracle.run_parallel(one, t, a), seq_oracle.run_parallel(one, t, b)
    changed = [i for i in range(24) if np.abs(la[i] - lb[i]).max() > 1e-9]
    # window 5: positions 7 .. 11 see token 7 itself; its block 6 .. 8 is seen from 8 + 5 = 13 on; 12 sees neither
    assert changed == [7, 8, 9, 10, 11] + list(range(13, 24))
    la, lb = seq_oracle.run_parallel(one, t, a, pool=0), seq_oracle.run_parallel(one, t, b, pool=0)
    assert [i for i in range(24) if np.abs(la[i] - lb[i]).max() > 1e-9] == [7, 8, 9, 10, 11]


ZCFG = synth.zusolix_config(24, 30, [
    synth.zusolix_layer("attention", synth.zusolix_attention(4, 2, 6, 10, 0.25, 7.0, (0.3, 9)), moe=(3, 2, 8), shared=5),
    synth.zusolix_layer("mingru", {"width": 14}, ff=20),
    synth.zusolix_layer("attention", synth.zusolix_attention(2, 2, 6, 6, 0.5))], groups=3, eps=1e-5, embed_scale=3.0, residual_mult=0.4)


def test_zusolix_configuration_maps_onto_layer_descriptors(tmp_path):
    t = synth.write_seq_model_dir(str(tmp_path), ZCFG, 1)
    cfg = seqmodel.read_config(str(tmp_path))
    up = FakeUp()
    st = safetensors_io.SafeTensors(str(tmp_path / "model.safetensors"))
    layers, top = seqmodel.ARCHITECTURES[cfg["architecture"]](cfg, st, up)
    bits = safetensors_io.f32_to_bf16_bits
    assert (top["width"], top["vocab"], top["canon_taps"], top["norm_offset"], top["embed_scale"], top["norm_groups"]) == (24, 30, 1, 0.0, 3.0, 3)
    a, g, c = layers
    assert all(abs(x.res_scale - 0.4) < 1e-7 and x.form == seqmodel.LAYER_PARALLEL and x.canon1 is None for x in layers)
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.pool, a.rot_dims, a.gated, a.qtemp_every) == (seqmodel.MIX_WINATTN, 4, 2, 6, 10, 0, 0, 0, 0, 9)
    assert abs(a.softcap - 7.0) < 1e-6 and abs(a.qtemp_coef - 0.3) < 1e-6 and a.scale == 0.25 and (c.softcap, c.qtemp_every, c.qtemp_coef) == (0.0, 0, 0.0)
    assert (a.qnorm, a.knorm, a.temp, a.sink) == (None, None, None, None)
    bias = up.vecs[a.in_bias - 1]
    assert bias.shape == (24 + 12 + 20,) and np.array_equal(bias[24:36], t["l0.mix.k.b"])
    # the depth average's weights: one more per layer
    assert [up.vecs[x.depth_mix - 1].shape for x in layers] == [(2,), (3,), (4,)] and a.norm2 is not None and c.norm2 is None and c.ff_kind == seqmodel.FF_NONE
    # the recurrence: z | x | g stacked, one bias vector (g has none)
    assert (g.kind, g.heads, g.dim, g.ff_kind, g.ff) == (seqmodel.MIX_MINGRU, 1, 14, seqmodel.FF_DENSE_SWIGLU, 20)
    assert np.array_equal(up.mats[g.in_cat - 1001], np.concatenate([bits(t["l1.mix." + n]) for n in ("z", "x", "g")]))
    gb = up.vecs[g.in_bias - 1]
    assert gb.shape == (42,) and np.array_equal(gb[14:28], t["l1.mix.x.b"]) and not gb[28:].any()
    # the experts: one matrix each way, expert after expert, gate / up rows alternating inside an expert; the router and the shared gate stay fp32 vectors
    assert (a.ff_kind, a.ff, a.experts, a.top, a.shared_ff, a.moe_norm_top) == (seqmodel.FF_MOE_SWIGLU, 8, 3, 2, 5, 0)
    ups, downs = up.mats[a.ff_up - 1001], up.mats[a.ff_down - 1001]
    assert ups.shape == (3 * 16, 24) and downs.shape == (3 * 24, 8)
    assert np.array_equal(ups[16:32:2], bits(t["l0.mlp.e1.gate"])) and np.array_equal(ups[33:48:2], bits(t["l0.mlp.e2.up"])) and np.array_equal(downs[24:48], bits(t["l0.mlp.e1.down"]))
    assert up.vecs[a.router - 1].shape == (3, 24) and up.vecs[a.shared_gate - 1].shape == (24,) and up.mats[a.shared_up - 1001].shape == (10, 24)
    # what the file and the configuration do not have does not exist
    less = {n: st.f32(n) for n in st.names() if not n.endswith((".b", "dwa", "shared.sg"))}
    cfg2 = json.loads(json.dumps(ZCFG))
    del cfg2["layers"][0]["mixer"]["softcap"], cfg2["layers"][0]["mixer"]["q_temp"], cfg2["norm"]["groups"]
    synth.write_seq_model_dir(str(tmp_path / "less"), cfg2, 1, tensors=less)
    layers, top = seqmodel.ARCHITECTURES["Zusolix"](cfg2, safetensors_io.SafeTensors(str(tmp_path / "less" / "model.safetensors")), FakeUp())
    a, g, _ = layers
    assert (a.in_bias, g.in_bias, a.depth_mix, a.shared_gate, a.softcap, a.qtemp_every, top["norm_groups"]) == (None, None, None, None, 0.0, 0, 1) and a.shared_up is not None
    for key, val in (("type", "conveyor"), ("mlp", {"kind": "sparse", "ff": 8})):
        bad = json.loads(json.dumps(ZCFG))
        bad["layers"][1][key] = val
        with pytest.raises(seqmodel.ConfigError):
            seqmodel.ARCHITECTURES["Zusolix"](bad, st, FakeUp())
    bad = json.loads(json.dumps(ZCFG))
    bad["layers"][0]["mlp"]["router"]["top"] = 4
    with pytest.raises(seqmodel.ConfigError):
        seqmodel.ARCHITECTURES["Zusolix"](bad, st, FakeUp())


def test_plain_zusolix_statement_reach_and_pieces():
    """causal, and every later token sees a changed one (nothing limits the reach); the norm's groups are on their own; the temperature steps where it should;
    the largest scores are the ones chosen"""
    t = synth.seq_tensors(ZCFG, 2)
    rng = np.random.default_rng(0)
    a = rng.integers(0, 30, 20)
    b = a.copy()
    b[6] = (b[6] + 1) % 30
    la, lb = seq_oracle.run_zusolix(ZCFG, t, a), seq_oracle.run_zusolix(ZCFG, t, b)
    assert np.array_equal(la[:6], lb[:6]) and min(np.abs(la[i] - lb[i]).max() for i in range(6, 20)) > 1e-6
    x = rng.standard_normal((4, 12))
    y = x.copy()
    y[:, 4:8] *= 7.0  # scaling one part changes nothing (up to eps), inside or outside it
    assert np.abs(seq_oracle.grouped_norm(x, np.ones(12), 3, 0.0) - seq_oracle.grouped_norm(y, np.ones(12), 3, 0.0)).max() < 1e-12
    assert np.abs(seq_oracle.grouped_norm(x, np.ones(12), 1, 0.0) - seq_oracle.grouped_norm(y, np.ones(12), 1, 0.0)).max() > 0.1
    assert [round(float(seq_oracle.query_temperature(p, 1.0, 4)), 6) for p in (0, 2, 3, 6, 7)] == [1.0, 1.0, round(1 + np.log(2), 6), round(1 + np.log(2), 6), round(1 + np.log(3), 6)]
    W = {k: np.asarray(v, np.float64) for k, v in t.items()}
    h = rng.standard_normal((5, 24))
    mlp = ZCFG["layers"][0]["mlp"]
    full = seq_oracle.expert_mixture(W, "l0.mlp.", h, mlp, use_shared=False)
    for i in range(5):
        s = seq_oracle.sigmoid(W["l0.mlp.router"] @ h[i])
        keep = np.argsort(-s)[:2]
        assert np.allclose(full[i], sum(seq_oracle.one_expert(W, "l0.mlp.e%d." % e, s[e] * h[i]) for e in keep))


KCFG = synth.pokatar_config(24, 30, [
    synth.pokatar_layer("attention", synth.pokatar_attention(4, 2, 6, 10, 0.25), moe=(3, 2, 8, 2, 5, 2), shared=5),
    synth.pokatar_layer("latent_attention", synth.pokatar_latent(3, 6, 4, 5, 7, 0.3, 77.0, (3.0, 40, 8.0, 0.5)), ff=20),
    synth.pokatar_layer("latent_attention", synth.pokatar_latent(2, 4, 6, 4, 9, 0.5, 9.0))], eps=1e-5)


def test_pokatar_configuration_maps_onto_layer_descriptors(tmp_path):
    t = synth.write_seq_model_dir(str(tmp_path), KCFG, 1)
    cfg = seqmodel.read_config(str(tmp_path))
    up = FakeUp()
    st = safetensors_io.SafeTensors(str(tmp_path / "model.safetensors"))
    layers, top = seqmodel.ARCHITECTURES[cfg["architecture"]](cfg, st, up)
    bits = safetensors_io.f32_to_bf16_bits
    assert (top["width"], top["vocab"], top["canon_taps"], top["norm_offset"], top["norm_center"], top["logit_scale"]) == (24, 30, 1, 0.0, 1, 1.0)
    assert top["head"] == top["embed"]  # the logits are taken against the embedding table
    a, b, c = layers
    assert all(x.form == seqmodel.LAYER_PRENORM and x.canon1 is None and x.norm1b is None and x.depth_mix is None for x in layers)
    # attention: q | k | v | g stacked, a gate row per output element, norms per head with [dim] weights, unit values, a sink of zeros
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.pool, a.rot_dims, a.gated, a.head_norm, a.v_unit) == (seqmodel.MIX_WINATTN, 4, 2, 6, 10, 0, 0, 0, 2, 1, 1)
    assert up.mats[a.in_cat - 1001].shape == (24 + 12 + 20 + 40, 24) and np.array_equal(up.mats[a.in_cat - 1001][56:], bits(t["l0.mix.g"]))
    assert up.vecs[a.qnorm - 1].shape == (6,) and up.vecs[a.knorm - 1].shape == (6,) and not up.vecs[a.sink - 1].any() and up.vecs[a.sink - 1].shape == (4,) and a.in_bias is None
    # latent attention: q | dkv | g stacked, no query latent, everything before the token, the scaling constants
    assert (b.kind, b.heads, b.dim, b.vdim, b.q_rank, b.kv_rank, b.rot_dim, b.rot_dims, b.window, b.gated) == (seqmodel.MIX_LATENT, 3, 6, 5, 0, 7, 4, 4, 0, 1)
    assert (b.yarn_factor, b.yarn_original, b.yarn_fast, b.yarn_slow, b.rot_base) == (3.0, 40, 8.0, 0.5, 77.0) and (c.yarn_factor, c.yarn_original) == (0.0, 0)
    assert np.array_equal(up.mats[b.in_cat - 1001], np.concatenate([bits(t["l1.mix." + n]) for n in ("q", "dkv", "g")])) and up.mats[b.in_cat - 1001].shape == (30 + 11 + 3, 24)
    assert np.array_equal(up.mats[b.ukv - 1001], np.concatenate([bits(t["l1.mix.uk"]), bits(t["l1.mix.uv"])])) and b.uq is None and b.qnorm is None
    # the dense feed-forward: gate / up rows alternating, their biases alike, a bias on the way down
    assert (b.ff_kind, b.ff, c.ff_kind) == (seqmodel.FF_DENSE_RELU_GLU, 20, seqmodel.FF_NONE)
    ub = up.vecs[b.ff_up_bias - 1]
    assert ub.shape == (40,) and np.array_equal(ub[0::2], t["l1.mlp.gate.b"]) and np.array_equal(ub[1::2], t["l1.mlp.up.b"]) and np.array_equal(up.vecs[b.ff_down_bias - 1], t["l1.mlp.down.b"])
    assert np.array_equal(up.mats[b.ff_up - 1001][1::2], bits(t["l1.mlp.up"]))
    # the experts: one matrix each way; the router has rows for the identity experts too; groups over all of them
    assert (a.ff_kind, a.ff, a.experts, a.top, a.shared_ff, a.moe_identity, a.moe_softmax, a.moe_groups, a.moe_keep, a.moe_weight_output) == (seqmodel.FF_MOE_RELU2, 8, 3, 2, 5, 2, 1, 5, 2, 1)
    assert up.mats[a.ff_up - 1001].shape == (3 * 8, 24) and up.mats[a.ff_down - 1001].shape == (3 * 24, 8) and np.array_equal(up.mats[a.ff_up - 1001][8:16], bits(t["l0.mlp.e1.up"]))
    assert up.vecs[a.router - 1].shape == (5, 24) and up.vecs[a.moe_correction - 1].shape == (5,) and up.mats[a.shared_up - 1001].shape == (5, 24) and a.shared_gate is None
    # what the file and the configuration do not have does not exist
    less = {n: st.f32(n) for n in st.names() if not n.endswith((".b", "correction", ".g", "q.norm"))}
    cfg2 = json.loads(json.dumps(KCFG))
    del cfg2["layers"][0]["mlp"]["router"]["groups"], cfg2["layers"][0]["mlp"]["router"]["identity"], cfg2["layers"][0]["mlp"]["shared"], cfg2["layers"][1]["mixer"]["rot"]["scaling"]
    less["l0.mlp.router"] = less["l0.mlp.router"][:3]
    synth.write_seq_model_dir(str(tmp_path / "less"), cfg2, 1, tensors=less)
    layers, _ = seqmodel.ARCHITECTURES["Pokatar"](cfg2, safetensors_io.SafeTensors(str(tmp_path / "less" / "model.safetensors")), FakeUp())
    a, b, _ = layers
    assert (a.gated, b.gated, a.qnorm, a.moe_correction, a.moe_groups, a.moe_identity, a.shared_up, b.ff_up_bias, b.ff_down_bias, b.yarn_factor) == (0, 0, None, None, 0, 0, None, None, None, 0.0)
    assert a.knorm is not None
    for key, val in (("type", "conveyor"), ("mlp", {"kind": "sparse", "ff": 8})):
        bad = json.loads(json.dumps(KCFG))
        bad["layers"][1][key] = val
        with pytest.raises(seqmodel.ConfigError):
            seqmodel.ARCHITECTURES["Pokatar"](bad, st, FakeUp())
    for key, val in (("top", 6), ("groups", {"count": 2, "keep": 1}), ("groups", {"count": 5, "keep": 1})):  # more than the router has; groups that do not divide; top beyond what stays
        bad = json.loads(json.dumps(KCFG))
        bad["layers"][0]["mlp"]["router"][key] = val
        with pytest.raises(seqmodel.ConfigError):
            seqmodel.ARCHITECTURES["Pokatar"](bad, st, FakeUp())


def test_plain_pokatar_statement_reach_and_pieces():
    """causal, and every later token sees a changed one; the layer norm ignores a shift; the sink takes its share; the frequency ramp ends where it should; the
    router's choice stays inside the best groups and an identity expert hands its input on"""
    t = synth.seq_tensors(KCFG, 2)
    rng = np.random.default_rng(0)
    a = rng.integers(0, 30, 20)
    b = a.copy()
    b[6] = (b[6] + 1) % 30
    la, lb = seq_oracle.run_pokatar(KCFG, t, a), seq_oracle.run_pokatar(KCFG, t, b)
    assert np.array_equal(la[:6], lb[:6]) and min(np.abs(la[i] - lb[i]).max() for i in range(6, 20)) > 1e-6
    x = rng.standard_normal((4, 12))
    assert np.abs(seq_oracle.centred_norm(x, np.ones(12), 0.0) - seq_oracle.centred_norm(x + 5.0, np.ones(12), 0.0)).max() < 1e-12
    assert abs(np.mean(seq_oracle.centred_norm(x, np.ones(12), 1e-5))) < 1e-12
    p = seq_oracle.sink_softmax(np.array([0.0, 0.0, 0.0]))
    assert np.allclose(p, 0.25) and np.allclose(seq_oracle.sink_softmax(np.array([50.0])), 1.0) and np.allclose(seq_oracle.sink_softmax(np.array([-50.0])), 0.0, atol=1e-20)
    # base 100, 8 dims: f = 1, 100^-1/4, 100^-1/2, 100^-3/4; original 40: pairs turning more than 8 times in 40 positions keep their frequency, fewer than 1/2 are divided
    f, mag = seq_oracle.yarn_frequencies({"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 40, "fast": 8.0, "slow": 0.5}})
    plain = 100.0 ** (-np.arange(4) / 4.0)
    lo, hi = max(np.floor(8 * np.log(40 / (2 * np.pi * 8.0)) / (2 * np.log(100.0))), 0), min(np.ceil(8 * np.log(40 / (2 * np.pi * 0.5)) / (2 * np.log(100.0))), 7)
    assert (lo, hi) == (0, 3) and np.allclose(f, plain * (1 - np.arange(4) / 3) + plain / 4 * np.arange(4) / 3) and abs(mag - (0.1 * np.log(4.0) + 1)) < 1e-12
    assert np.allclose(seq_oracle.yarn_frequencies({"dims": 8, "base": 100.0})[0], plain)
    v = rng.standard_normal(8)
    r = seq_oracle.rotate_halves(v, 3, plain, 1.0)
    assert np.allclose(np.hypot(r[:4], r[4:]), np.hypot(v[:4], v[4:])) and np.allclose(seq_oracle.rotate_halves(v, 0, plain, 1.5), 1.5 * v)
    # five router rows in five groups of one of which two stay: exactly the two best corrected scores; with one group of five the same two
    s, corr = np.array([0.1, 0.3, 0.15, 0.25, 0.2]), np.array([0.0, -0.2, 0.0, 0.0, 0.2])
    assert seq_oracle.grouped_choice(s, corr, {"top": 2, "groups": {"count": 5, "keep": 2}}) == [4, 3]
    assert seq_oracle.grouped_choice(s, 0.0, {"top": 2}) == [1, 3]
    # six rows in three pairs, one pair stays: the best single row decides the pair, the second choice is its neighbour however small
    s6 = np.array([0.05, 0.3, 0.25, 0.2, 0.1, 0.1])
    assert seq_oracle.grouped_choice(s6, 0.0, {"top": 2, "groups": {"count": 3, "keep": 1}}) == [1, 0]
    W = {k: np.asarray(v, np.float64) for k, v in t.items()}
    h = rng.standard_normal((6, 24))
    mlp = KCFG["layers"][0]["mlp"]
    full = seq_oracle.routed_experts(W, "l0.mlp.", h, mlp, use_shared=False)
    for i in range(6):
        z = W["l0.mlp.router"] @ h[i]
        sc = np.exp(z) / np.exp(z).sum()
        keep = np.argsort(-(sc + W["l0.mlp.correction"]))[:2]  # (five groups of one, two stay: the group limit changes nothing here)
        assert np.allclose(full[i], sum(sc[e] * (seq_oracle.squared_relu_expert(W, "l0.mlp.e%d." % e, h[i]) if e < 3 else h[i]) for e in keep))


def test_the_small_library_exports_what_its_models_need():
    if not os.path.exists(hip.SEQ_LIB_PATH):
        pytest.skip("lib/libps_hip_seq.so not built")
    lib = C.CDLL(hip.SEQ_LIB_PATH)
    assert not [n for n in hip.SEQ_EXPORTS if not hasattr(lib, n)]
