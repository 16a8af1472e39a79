"""Pokatar (pre-norm layers with layer norms; grouped-query attention with per-head q / k norms, unit-rms values, a zero-score sink and an element-wise
gate; latent attention with direct queries, a shared rotated key part with wavelength-scaled frequencies and a gate per head; a relu-gated dense feed-forward
with biases; squared-relu experts behind a soft-max router with a choice correction, a group limit and identity experts) on the GPU against the plain
float64 statement in tests/seq_oracle.py: small configurations and weights made here, each mechanism alone, every schedule (whole prompts, token by
token, portions down to two tokens, interleaved requests, reused slots, long decoding, greedy generation), and hand-made models in which one far key
decides the logits, so that a lost key shows."""
import numpy as np
import pytest

import seq_oracle
from powerserve_amd import hip, host, seqmodel, synth
from powerserve_amd.safetensors_io import f32_to_bf16_bits

pytestmark = pytest.mark.gpu

PL, PA, PLA, PC = synth.pokatar_layer, synth.pokatar_attention, synth.pokatar_latent, synth.pokatar_config

CONFIGS = {
    # sizes that are multiples of nothing (per-key attention, 64 x 64 mat-mul, the expanded single-token latent step), one key / value head and kv_heads == heads,
    # dim != vdim, a layer without feed-forward, top 2 of 5 + 2 identity experts without groups, top 3 of 6 in 3 groups of which 2 stay, no frequency scaling
    "odd": PC(40, 50, [PL("attention", PA(3, 1, 10, 6, 0.3), moe=(5, 2, 12, 2, 0, 0), shared=20),
                       PL("latent_attention", PLA(3, 10, 6, 7, 12, 0.25, 1000.0, (3.0, 48, 6.0, 1.0)), ff=28),
                       PL("attention", PA(4, 4, 6, 10, 0.4)),
                       PL("latent_attention", PLA(2, 5, 4, 9, 10, 0.3, 50.0), moe=(5, 3, 8, 1, 3, 2))], eps=1e-5),
    # sizes the matrix-core kernels take (wide mat-mul: inputs that are multiples of 64; absorbed single-token latent step), top 1, top == what the groups leave,
    # no identity experts, one group
    "aligned": PC(128, 96, [PL("latent_attention", PLA(4, 48, 32, 16, 48, 0.15, 10000.0, (4.0, 128, 16.0, 2.0)), moe=(8, 1, 64, 0, 2, 1), shared=64),
                            PL("attention", PA(4, 2, 32, 16, 0.2), ff=192),
                            PL("attention", PA(8, 2, 16, 32, 0.25), moe=(6, 3, 64, 2, 4, 2)),
                            PL("latent_attention", PLA(2, 16, 32, 64, 32, 0.2, 500000.0, (8.0, 64, 32.0, 1.0)), moe=(4, 2, 128, 0, 1, 1))], eps=1e-6),
    # more heads in a key / value group than a tile of the single-token kernel has rows; a single expert beside three identity experts
    "manyheads": PC(64, 40, [PL("attention", PA(20, 1, 16, 8, 0.3), moe=(1, 2, 16, 3, 2, 1), shared=16), PL("latent_attention", PLA(18, 16, 16, 8, 32, 0.2, 100.0), ff=32)]),
    # 128 value columns per head, a latent wider than the model
    "wide": PC(96, 40, [PL("attention", PA(2, 2, 48, 128, 0.15), ff=40), PL("latent_attention", PLA(3, 48, 16, 128, 160, 0.1, 10000.0, (2.0, 32, 4.0, 0.5)), moe=(4, 2, 32, 4, 4, 3))]),
}
TOL = {"float32": 2e-4, "bfloat16": 1e-1}  # fp32: a few ulps of fp32 sums; bfloat16: 8-bit mantissas in models this narrow


def err(got, want):
    """centred rms of the difference over the rms of the logits, worst row"""
    d = np.asarray(got, dtype=np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    s = np.sqrt(np.mean((want - want.mean(-1, keepdims=True)) ** 2))
    return float(np.sqrt(np.mean(d * d, -1)).max() / s)


def rows(got, want, which):
    return [err(got[i:i + 1], want[i:i + 1]) for i in which]


def close(got, want, dtype):
    """float32: every row within TOL.  bfloat16: nine rows in ten within TOL and none beyond the logits' own spread -- where two choice scores of a router
    are closer than 8-bit mantissas resolve, the choice may go the other way and the rows behind it move; the same schedules are held to 2e-4 in float32."""
    if dtype == "float32":
        return err(got, want) < TOL[dtype]
    r = rows(got, want, range(len(want)))
    return float(np.quantile(r, 0.9)) < TOL[dtype] and max(r) < 1.0


@pytest.fixture(scope="module")
def made(ctx, tmp_path_factory):
    cache = {}

    def get(name, dtype="float32", max_batch=16, cfg=None, tensors=None, max_context=600):
        key = (name, dtype, max_batch, max_context)
        if key not in cache:
            c = cfg or CONFIGS[name]
            d = str(tmp_path_factory.mktemp("p"))
            t = synth.write_seq_model_dir(d, c, 0, tensors)
            cache[key] = (seqmodel.load_model(ctx, d, dtype=dtype, max_batch=max_batch, n_slots=3, max_context=max_context), c, t)
        return cache[key]

    yield get
    for m, _, _ in cache.values():
        m.close()


def tokens_for(cfg, n, seed=1, lo=0):
    return np.random.default_rng(seed).integers(lo, cfg["vocab"], n).astype(np.int32)


def run_portions(m, toks, sizes):
    s, out, at, i = m.acquire(), [], 0, 0
    while at < len(toks):
        n = min(sizes[i % len(sizes)], len(toks) - at)
        out.append(m.forward(s, toks[at:at + n], np.arange(n)))
        at, i = at + n, i + 1
    m.release(s)
    return np.concatenate(out)


def bf16(t):
    return {k: (f32_to_bf16_bits(np.asarray(v, np.float32)).astype(np.uint32) << 16).view(np.float32).reshape(np.shape(v)) for k, v in t.items()}


def first_layer_adds(m, toks, x0):
    m.capture_layers(True)
    s = m.acquire()
    m.forward(s, toks)
    got = m.layers(len(toks))[0].astype(np.float64) - x0
    m.release(s)
    m.capture_layers(False)
    return got


# ---------------------------------------------------------------------------------------------------------------- mechanisms, one at a time
MIXTURES = {"mixture": (6, 2, 14, 2, 4, 2), "mixture_aligned": (6, 3, 64, 2, 2, 1), "mixture_top1": (5, 1, 12, 1, 0, 0)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["attention", "attention_mfma", "latent", "latent_mfma", "dense", "mixture", "mixture_aligned", "mixture_top1"])
def test_each_mechanism_alone(made, which, dtype):
    """one layer in which only one sublayer contributes (the mixer's output matrix is zero, or there is no feed-forward): what it adds to the embedding
    against that mechanism's own plain function of the layer norm"""
    big = which in ("attention_mfma", "latent_mfma", "mixture_aligned")
    a = PA(4, 2, 16, 8, 0.3) if big else PA(3, 1, 10, 6, 0.3)
    la = PLA(4, 16, 16, 8, 32, 0.2, 10000.0, (4.0, 16, 8.0, 1.0)) if big else PLA(3, 10, 6, 7, 12, 0.25, 100.0, (3.0, 24, 4.0, 1.0))
    W_ = 64 if big else 40
    if which.startswith("attention"):
        layer = PL("attention", a)
    elif which.startswith("latent"):
        layer = PL("latent_attention", la)
    elif which == "dense":
        layer = PL("attention", a, ff=36)
    else:
        layer = PL("attention", a, moe=MIXTURES[which], shared=None if which == "mixture_top1" else (64 if big else 10))
    cfg = PC(W_, 32, [layer], eps=1e-5)
    t = synth.seq_tensors(cfg, 3)
    if layer["mlp"]:
        t["l0.mix.o"] = np.zeros_like(t["l0.mix.o"])
    m, _, _ = made("alone_" + which, dtype, max_batch=32, cfg=cfg, tensors=t)
    toks = tokens_for(cfg, 30, seed=3)
    W = {k: np.asarray(v, np.float64) for k, v in t.items()}
    x0 = W["embed"][toks]
    if layer["mlp"] and layer["mlp"]["kind"] == "dense":
        want = seq_oracle.relu_gated_feed_forward(W, "l0.mlp.", seq_oracle.centred_norm(x0, W["l0.norm2"], 1e-5))
    elif layer["mlp"]:
        want = seq_oracle.routed_experts(W, "l0.mlp.", seq_oracle.centred_norm(x0, W["l0.norm2"], 1e-5), layer["mlp"])
    elif layer["type"] == "attention":
        want = seq_oracle.sink_gated_attention(W, "l0.mix.", seq_oracle.centred_norm(x0, W["l0.norm1"], 1e-5), a, 1e-5)
    else:
        want = seq_oracle.shared_key_latent_attention(W, "l0.mix.", seq_oracle.centred_norm(x0, W["l0.norm1"], 1e-5), la, 1e-5)
    got = first_layer_adds(m, toks, x0)
    assert np.abs(got - want).max() < (2e-4 if dtype == "float32" else 6e-2) * np.abs(want).max()


def test_what_the_plain_statement_is_sensitive_to(made):
    """every mechanism of the design left out of the plain statement in turn moves its logits far from the right ones; the library agrees with the right ones"""
    m, cfg, t = made("odd", "float32", max_batch=32)
    toks = tokens_for(cfg, 30, seed=8)
    want = seq_oracle.run_pokatar(cfg, t, toks)
    for kw in ({"attn_kw": {"use_sink": False}}, {"attn_kw": {"norm_values": False}}, {"attn_kw": {"gate_per_element": False}}, {"latent_kw": {"use_scaling": False}},
               {"latent_kw": {"use_gate": False}}, {"moe_kw": {"use_identity": False}}, {"moe_kw": {"use_shared": False}}, {"moe_kw": {"use_groups": False}},
               {"moe_kw": {"use_correction": False}}):
        assert err(seq_oracle.run_pokatar(cfg, t, toks, **kw), want) > 5e-3, kw
    assert err(run_portions(m, toks, [30]), want) < TOL["float32"]
    assert err(run_portions(m, toks, [1]), want) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "aligned", "manyheads", "wide"])
def test_whole_prompt_against_the_plain_statement(made, name, dtype):
    m, cfg, t = made(name, dtype, max_batch=64)
    toks = tokens_for(cfg, 70)
    want = seq_oracle.run_pokatar(cfg, t, toks)
    s = m.acquire()
    got = m.forward(s, toks, np.arange(len(toks)))
    m.release(s)
    assert close(got, want, dtype)


@pytest.mark.parametrize("name", ["odd", "aligned", "wide"])
def test_the_residual_stream_after_every_layer(made, name):
    m, cfg, t = made(name, "float32", max_batch=64)
    toks = tokens_for(cfg, 45, seed=5)
    per = []
    seq_oracle.run_pokatar(cfg, t, toks, per_layer=per)
    assert m.n_runs == len(per) == len(cfg["layers"])
    m.capture_layers(True)
    s = m.acquire()
    m.forward(s, toks)
    got = m.layers(len(toks))
    m.release(s)
    m.capture_layers(False)
    for i, want in enumerate(per):
        assert np.abs(got[i] - want).max() < 2e-4 * np.abs(want).max(), i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "aligned", "manyheads", "wide"])
def test_token_by_token_and_portions_give_the_whole_prompts_logits(made, name, dtype):
    m, cfg, t = made(name, dtype, max_batch=16)  # 16: a 50-token portion is also cut inside the library
    toks = tokens_for(cfg, 90, seed=2)
    want = seq_oracle.run_pokatar(cfg, t, toks)
    for sizes in ([1], [2], [3, 1, 7, 2], [50, 2, 23], [16, 17, 15], [9, 8, 10]):  # (9 and 10 tokens: the smallest tiled mixtures, 8: the widest mat-vec)
        assert close(run_portions(m, toks, sizes), want, dtype), sizes


def test_first_tokens_of_a_sequence(made):
    """a first token's attention is its own value times e^s / (1 + e^s): the sink is half of the denominator or more"""
    m, cfg, t = made("aligned", "float32")
    for n in (1, 2, 3, 5):
        toks = tokens_for(cfg, n, seed=10 + n)
        want = seq_oracle.run_pokatar(cfg, t, toks)
        assert err(seq_oracle.run_pokatar(cfg, t, toks, attn_kw={"use_sink": False}), want) > 1e-2
        assert err(run_portions(m, toks, [n]), want) < TOL["float32"]
        assert err(run_portions(m, toks, [1]), want) < TOL["float32"]


def test_interleaved_requests_and_reused_slots(made):
    """requests of unequal length fed in turns through the scheduler against each alone; then every slot is used again and must start from nothing"""
    m, cfg, t = made("aligned", "float32", max_batch=16)
    seqs = [tokens_for(cfg, n, seed=20 + n) for n in (61, 9, 88)]
    want = [seq_oracle.run_pokatar(cfg, t, s) for s in seqs]
    sched = seqmodel.RequestScheduler(m)
    got, at = [[] for _ in seqs], [0, 0, 0]
    steps, i = [5, 2, 11, 1, 3], 0
    while any(a < len(s) for a, s in zip(at, seqs)):
        r = i % 3
        if at[r] < len(seqs[r]):
            n = min(steps[i % len(steps)], len(seqs[r]) - at[r])
            got[r].append(sched.feed("req%d" % r, seqs[r][at[r]:at[r] + n], np.arange(n)))
            at[r] += n
            if at[r] == len(seqs[r]):
                sched.finish("req%d" % r)
        i += 1
    for g, w in zip(got, want):
        assert err(np.concatenate(g), w) < TOL["float32"]
    for r in range(4):  # a short request after a long one in the same slot: what the long one left in the cache must not be seen
        which = 2 if r % 2 == 0 else 1
        assert err(sched.feed("again", seqs[which], np.arange(len(seqs[which]))), want[which]) < TOL["float32"]
        sched.finish("again")
    with pytest.raises(hip.PSHipError):
        [m.acquire() for _ in range(4)]
    for s in range(3):
        m.release(s)


# ---------------------------------------------------------------------------------------------------------------- weights made so that a fault shows
def marked_model(aligned, seed=0, moe=True):
    """Token 0 is a MARK: its embedding alone has feature 0; feature 1 is the same constant for every token (all norm weights one, so the layer norm keeps both
    apart from the noise in the other features).  Layer 0, attention: every key reads feature 0 into the last channel of its head and every query reads
    feature 1 into that channel, so after the per-head norms a query's score for a mark is about `dim` x scale, far above all others; every value channel
    reads feature 0.  Layer 1, latent attention: the latent's channel 0 reads feature 0, the key expansion sends it to the last plain channel of every head,
    where the query has read feature 1; the value expansion spreads it over the head.  Both output matrices are large, so what the attention finds decides
    the logits.  (moe False: dense feed-forwards -- in bfloat16 a router's close call may go the other way, which is no fault of the mechanism under test.)"""
    rng = np.random.default_rng(seed)
    W, V = (64, 24) if aligned else (30, 24)
    H, G, d, dv = (4, 2, 16, 8) if aligned else (3, 1, 10, 6)
    a = PA(H, G, d, dv, 1.0)
    la = PLA(H, d, 16 if aligned else 6, dv, 16 if aligned else 9, 0.9, 10000.0, (4.0, 64, 16.0, 1.0))
    ffs = [dict(moe=(4, 2, 12, 1, 0, 0), shared=8), dict(moe=(3, 1, 10, 2, 0, 0))] if moe else [dict(ff=24), dict(ff=20)]
    cfg = PC(W, V, [PL("attention", a, **ffs[0]), PL("latent_attention", la, **ffs[1])], eps=1e-5)
    t = synth.seq_tensors(cfg, seed)
    e = rng.standard_normal((V, W)).astype(np.float32) * 0.5
    e[:, 0], e[:, 1] = 0.0, 4.0
    e[0, 0] = 8.0
    t["embed"], t["l0.norm1"], t["l1.norm1"] = e, np.ones(W, np.float32), np.ones(W, np.float32)
    c = d - 1
    k = rng.standard_normal((G * d, W)).astype(np.float32) * 0.05
    q = rng.standard_normal((H * d, W)).astype(np.float32) * 0.05
    k[:, :2], q[:, :2] = 0.0, 0.0
    for g in range(G):
        k[g * d + c, 0] = 2.0
    for h in range(H):
        q[h * d + c, 1] = 2.0
    v = rng.standard_normal((G * dv, W)).astype(np.float32) * 0.2
    v[:, 0] = 1.5
    p = "l0.mix."
    t[p + "q"], t[p + "k"], t[p + "v"], t[p + "q.norm"], t[p + "k.norm"] = q, k, v, np.ones(d, np.float32), np.ones(d, np.float32)
    t[p + "o"] = t[p + "o"] * 1.5
    R, dr = la["kv_rank"], la["rot_dim"]
    p = "l1.mix."
    dkv = rng.standard_normal((R + dr, W)).astype(np.float32) * 0.1
    dkv[:, :2] = 0.0
    dkv[0, 0] = 3.0
    q1 = rng.standard_normal((H * (d + dr), W)).astype(np.float32) * 0.1
    q1[:, :2] = 0.0
    uk = rng.standard_normal((H * d, R)).astype(np.float32) * 0.1
    uv = rng.standard_normal((H * dv, R)).astype(np.float32) * 0.2
    uk[:, 0] = 0.0
    uv[:, 0] = 1.5
    for h in range(H):
        q1[h * (d + dr) + c, 1] = 1.0
        uk[h * d + c, 0] = 2.0
    t[p + "q"], t[p + "dkv"], t[p + "uk"], t[p + "uv"], t[p + "dkv.norm"] = q1, dkv, uk, uv, np.ones(R, np.float32)
    t[p + "o"] = t[p + "o"] * 1.5
    return cfg, bf16(t)


def marked_tokens(cfg, n, marks, seed):
    toks = tokens_for(cfg, n, seed, lo=1)
    toks[list(marks)] = 0
    return toks


@pytest.mark.parametrize("aligned", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_in_prompts_and_in_decoding(made, dtype, aligned):
    """One mark at position 4, 470 tokens: every later query of either attention must still find it.  The plain statement in which the queries of one of
    them see only their last 64 / 256 / 300 positions is far off on every row behind that reach (and exact before it); the library agrees with the right
    one in a prompt cut into portions of 64 (keys across portion and tile borders), and on 170 tokens decoded one by one behind a 300-token prompt."""
    cfg, t = marked_model(aligned, moe=dtype == "float32")
    m, _, _ = made("marked%d" % aligned, dtype, max_batch=64, cfg=cfg, tensors=t)
    toks = marked_tokens(cfg, 470, (4,), seed=3)
    want = seq_oracle.run_pokatar(cfg, t, toks)
    for which in ("attn_kw", "latent_kw"):
        for reach in (64, 256, 300):
            wrong = seq_oracle.run_pokatar(cfg, t, toks, **{which: {"reach": reach}})
            assert np.median(rows(wrong, want, range(4 + reach, 470))) > 0.03, (which, reach)
            assert max(rows(wrong, want, range(0, reach))) < 1e-9  # (up to there such a query still sees everything)
    tol = 1e-3 if dtype == "float32" else TOL[dtype]
    s = m.acquire()
    got = [m.forward(s, toks[:300], np.arange(300))] + [m.forward(s, toks[i:i + 1], [0]) for i in range(300, 470)]
    m.release(s)
    assert max(rows(np.concatenate(got), want, range(len(toks)))) < tol
    for sizes in ([470], [64], [61, 2, 100]):
        assert max(rows(run_portions(m, toks, sizes), want, range(len(toks)))) < tol, sizes


@pytest.mark.parametrize("aligned", [False, True])
def test_rotation_far_from_the_start(made, aligned):
    """a latent layer whose rotated parts carry the scores (their projections enlarged), 400 tokens: the plain statement with unscaled frequencies or
    unstretched cos / sin is off; the library agrees with the right one in portions, across their borders and token by token"""
    la = PLA(4, 16, 32, 8, 32, 0.15, 10000.0, (4.0, 32, 8.0, 0.5)) if aligned else PLA(3, 6, 10, 7, 12, 0.3, 200.0, (6.0, 40, 5.0, 1.0))
    cfg = PC(64 if aligned else 40, 32, [PL("latent_attention", la, ff=48)], eps=1e-5)
    t = synth.seq_tensors(cfg, 5)
    H, d, dr, R = la["heads"], la["dim"], la["rot_dim"], la["kv_rank"]
    q = t["l0.mix.q"].reshape(H, d + dr, -1).copy()
    q[:, d:] *= 3.0
    t["l0.mix.q"] = q.reshape(H * (d + dr), -1)
    t["l0.mix.dkv"] = t["l0.mix.dkv"].copy()
    t["l0.mix.dkv"][R:] *= 3.0
    t = bf16(t)
    m, _, _ = made("rot%d" % aligned, "float32", max_batch=64, cfg=cfg, tensors=t)
    toks = tokens_for(cfg, 400, seed=4)
    want = seq_oracle.run_pokatar(cfg, t, toks)
    assert err(seq_oracle.run_pokatar(cfg, t, toks, latent_kw={"use_scaling": False}), want) > 0.05
    for sizes in ([64], [1], [61, 2, 100, 1, 1]):
        assert max(rows(run_portions(m, toks, sizes), want, range(len(toks)))) < 1e-3, sizes


def test_long_decoding_keeps_the_caches(made):
    m, cfg, t = made("aligned", "float32", max_batch=16)
    toks = tokens_for(cfg, 260, seed=6)
    want = seq_oracle.run_pokatar(cfg, t, toks)
    assert err(run_portions(m, toks, [13, 1, 1, 1, 1, 1, 1, 1]), want) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["aligned", "odd"])
def test_greedy_generation_through_the_entry_point(made, name, dtype):
    """SeqModel.generate (prefill, then the captured single-token step feeding its own arg-max) picks, at every step, a token whose logit in the
    plain statement is the largest up to rounding; eager launches and a host sampler set to top-1 give the same ids."""
    m, cfg, t = made(name, dtype, max_batch=16)
    prompt = tokens_for(cfg, 29, seed=7)
    ids = m.generate(prompt, 40)
    assert ids.shape == (40,)
    full = np.concatenate([prompt, ids])
    want = seq_oracle.run_pokatar(cfg, t, full[:-1])
    spread = want.max() - want.min()
    for i, tok in enumerate(ids):
        row = want[len(prompt) - 1 + i]
        assert row.max() - row[tok] < (1e-4 if dtype == "float32" else 3e-2) * spread, i
    m.set_mode(1)
    assert np.array_equal(m.generate(prompt, 40), ids)
    m.set_mode(0)
    assert np.array_equal(m.generate(prompt, 40), ids)  # the captured sequence replayed on a slot that was used before
    sm = host.Sampler(host.SamplerCfg.make(cfg["vocab"], seed=1, temperature=1.0, top_p=1.0, top_k=1))
    assert np.array_equal(m.generate(prompt, 40, sampler=sm.sample), ids)
    sm.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["aligned", "manyheads", "wide"])
def test_matrix_core_forms_agree_with_the_plain_kernels(made, name, dtype):
    """mode bit 1 keeps the per-key attention, the expanded single-token latent step and the 64 x 64 mat-mul (also for the experts' grouped products): the
    wide mat-mul, the mat-vecs and the matrix-core attention of a portion and of a single token must give the same logits (fp32: up to the order of sums)"""
    m, cfg, t = made(name, dtype, max_batch=64)
    toks = tokens_for(cfg, 150, seed=9)
    fast = [run_portions(m, toks, sizes) for sizes in ([64], [1], [40, 1, 1, 1, 9])]
    m.set_mode(2)
    plain = [run_portions(m, toks, sizes) for sizes in ([64], [1], [40, 1, 1, 1, 9])]
    m.set_mode(0)
    want = seq_oracle.run_pokatar(cfg, t, toks)
    for a, b in zip(fast, plain):
        assert err(a, b) < 1e-4 if dtype == "float32" else close(a, b.astype(np.float64), dtype)
        assert close(a, want, dtype)


def test_host_facade_loads_and_generates_the_same(made, tmp_path):
    m, cfg, t = made("aligned", "float32", max_batch=16)
    synth.write_seq_model_dir(str(tmp_path), cfg, 0, t)
    hm = host.HostSeqModel(str(tmp_path), dtype="float32", max_batch=16, n_slots=2, max_context=600)
    prompt = tokens_for(cfg, 19, seed=7)
    ids = m.generate(prompt, 12)
    assert np.array_equal(hm.generate(prompt, 12), ids)
    s, s2 = hm.acquire(), m.acquire()
    a, b = hm.forward(s, prompt, [0, 5, 18]), m.forward(s2, prompt, [0, 5, 18])
    hm.release(s)
    m.release(s2)
    assert np.array_equal(a, b)
    hm.close()


def test_a_sequence_fills_its_context_and_no_more(ctx, tmp_path):
    cfg = CONFIGS["odd"]
    t = synth.write_seq_model_dir(str(tmp_path), cfg, 0)
    m = seqmodel.load_model(ctx, str(tmp_path), dtype="float32", max_batch=8, n_slots=1, max_context=20)
    toks = tokens_for(cfg, 20)
    s = m.acquire()
    got = [m.forward(s, toks[:18], np.arange(18))]
    with pytest.raises(hip.PSHipError):
        m.forward(s, [1, 2, 3])
    got.append(m.forward(s, toks[18:], [0, 1]))
    m.release(s)
    assert err(np.concatenate(got), seq_oracle.run_pokatar(cfg, t, toks)) < TOL["float32"]
    m.close()
