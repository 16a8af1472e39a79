"""Zusolix (two-norm parallel layers with a depth average; soft-capped attention with a query temperature; an element-wise gated recurrence;
dense and mixture-of-experts feed-forwards) on the GPU against the plain float64 statement in tests/seq_oracle.py: small configurations and
weights made here, each mechanism alone, every schedule (whole prompts, token by token, portions down to two tokens, interleaved requests,
reused slots, long decoding, greedy generation), and hand-made models in which one far key, the soft cap, a temperature step or the carried
state decides the logits, so that a lost key, a missing cap, a step one token off or a dropped state shows."""
import numpy as np
import pytest

import seq_oracle
from powerserve_amd import hip, host, seqmodel, synth
from powerserve_amd.safetensors_io import f32_to_bf16_bits

pytestmark = pytest.mark.gpu

ZL, ZA, ZC = synth.zusolix_layer, synth.zusolix_attention, synth.zusolix_config

CONFIGS = {
    # sizes that are multiples of nothing (per-key attention, 64 x 64 mat-mul), kv_heads == heads and one key / value head, dim != vdim, a layer without
    # feed-forward, a recurrence first, top 2 of 5 with a shared expert, top == experts without one, a temperature that steps at every token
    "odd": ZC(40, 50, [ZL("mingru", {"width": 36}, moe=(5, 2, 12), shared=20),
                       ZL("attention", ZA(3, 1, 10, 6, 0.3, 5.0, (0.4, 7)), ff=28),
                       ZL("attention", ZA(4, 4, 6, 10, 0.25, None, (0.2, 1))),
                       ZL("mingru", {"width": 70}, moe=(3, 3, 8))], groups=5, eps=1e-5, embed_scale=2.0, residual_mult=0.7),
    # sizes the matrix-core kernels take (wide mat-mul: inputs that are multiples of 64), one norm group, top 1 and top 3 of 8
    "aligned": ZC(128, 96, [ZL("attention", ZA(4, 2, 32, 16, 0.2, 8.0, (0.3, 16)), moe=(8, 1, 64), shared=64),
                            ZL("mingru", {"width": 192}, ff=192),
                            ZL("attention", ZA(2, 2, 16, 64, 0.3), moe=(8, 3, 64)),
                            ZL("attention", ZA(8, 2, 16, 32, 0.25, 30.0), ff=64)], groups=1, embed_scale=4.0, residual_mult=0.5),
    # more heads in a key / value group than a tile of the single-token kernel has rows; a single expert
    "manyheads": ZC(64, 40, [ZL("attention", ZA(20, 1, 16, 8, 0.3, 6.0, (0.5, 3)), moe=(1, 1, 16), shared=16)], groups=4),
    # 128 value columns per head, a recurrence wider than the model
    "wide": ZC(96, 40, [ZL("attention", ZA(2, 2, 48, 128, 0.15, 10.0)), ZL("mingru", {"width": 200}, moe=(4, 2, 32))], groups=3, residual_mult=1.5),
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


@pytest.fixture(scope="module")
def made(ctx, tmp_path_factory):
    cache = {}

    def get(name, dtype="float32", max_batch=16, cfg=None, tensors=None, max_context=600):
        key = (name, dtype, max_batch, max_context)
        if key not in cache:
            c = cfg or CONFIGS[name]
            d = str(tmp_path_factory.mktemp("z"))
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
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["attention", "attention_mfma", "recurrence", "dense", "mixture", "mixture_aligned"])
def test_each_mechanism_alone(made, which, dtype):
    """one layer that hands on its own result, in which only one sublayer contributes (the other's output matrix is zero or it is absent): what it adds to
    the embedding against that mechanism's own plain function of the grouped norm"""
    a = ZA(4, 2, 16, 8, 0.3, 4.0, (0.5, 5)) if which == "attention_mfma" else ZA(3, 1, 10, 6, 0.3, 4.0, (0.5, 5))
    W_, groups, mult = (64, 2, 0.8) if which in ("attention_mfma", "mixture_aligned") else (40, 5, 0.8)
    layer = {"attention": lambda: ZL("attention", a), "attention_mfma": lambda: ZL("attention", a), "recurrence": lambda: ZL("mingru", {"width": 52}),
             "dense": lambda: ZL("attention", a, ff=36), "mixture": lambda: ZL("attention", a, moe=(6, 2, 14), shared=10),
             "mixture_aligned": lambda: ZL("attention", a, moe=(4, 3, 64), shared=64)}[which]()
    cfg = ZC(W_, 32, [layer], groups=groups, eps=1e-5, embed_scale=1.5, residual_mult=mult)
    t = synth.seq_tensors(cfg, 3)
    t["l0.dwa"] = np.array([0.0, 1.0], np.float32)
    if layer["mlp"]:
        t["l0.mix.o"] = np.zeros_like(t["l0.mix.o"])
    m, _, _ = made("alone_" + which, dtype, max_batch=32, cfg=cfg, tensors=t)
    toks = tokens_for(cfg, 30, seed=3)
    W = {k: np.asarray(v, np.float64) for k, v in t.items()}
    x0 = W["embed"][toks] * 1.5
    if layer["mlp"]:
        want = seq_oracle.zusolix_feed_forward(W, "l0.mlp.", seq_oracle.grouped_norm(x0, W["l0.norm2"], groups, 1e-5), layer["mlp"])
    elif layer["type"] == "attention":
        want = seq_oracle.capped_attention(W, "l0.mix.", seq_oracle.grouped_norm(x0, W["l0.norm1"], groups, 1e-5), a)
    else:
        want = seq_oracle.min_gru(W, "l0.mix.", seq_oracle.grouped_norm(x0, W["l0.norm1"], groups, 1e-5), layer["mixer"])
    got = first_layer_adds(m, toks, x0)
    assert np.abs(got - mult * want).max() < (2e-4 if dtype == "float32" else 6e-2) * np.abs(mult * want).max()


def test_the_weight_of_an_expert_is_on_its_input(made):
    """the plain statement with the router's score on the expert's OUTPUT is far from the right one (the experts are not linear); the library agrees with the right one"""
    m, cfg, t = made("odd", "float32", max_batch=32)
    toks = tokens_for(cfg, 30, seed=8)
    want = seq_oracle.run_zusolix(cfg, t, toks)
    assert err(seq_oracle.run_zusolix(cfg, t, toks, moe_kw={"weight_on_output": True}), want) > 0.02
    assert err(seq_oracle.run_zusolix(cfg, t, toks, moe_kw={"use_shared": False}), want) > 0.02
    assert err(seq_oracle.run_zusolix(cfg, t, toks, use_depth=False), want) > 0.05
    assert err(run_portions(m, toks, [30]), want) < TOL["float32"]
    assert err(run_portions(m, toks, [1]), want) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "aligned", "manyheads", "wide"])
def test_whole_prompt_against_the_plain_statement(made, name, dtype):
    m, cfg, t = made(name, dtype, max_batch=64)
    toks = tokens_for(cfg, 70)
    want = seq_oracle.run_zusolix(cfg, t, toks)
    s = m.acquire()
    got = m.forward(s, toks, np.arange(len(toks)))
    m.release(s)
    assert err(got, want) < TOL[dtype]


@pytest.mark.parametrize("name", ["odd", "aligned", "wide"])
def test_what_every_layer_hands_on(made, name):
    """the depth average over the embedding and all results so far, layer by layer"""
    m, cfg, t = made(name, "float32", max_batch=64)
    toks = tokens_for(cfg, 45, seed=5)
    per = []
    seq_oracle.run_zusolix(cfg, t, toks, per_layer=per)
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
    want = seq_oracle.run_zusolix(cfg, t, toks)
    for sizes in ([1], [2], [3, 1, 7, 2], [50, 2, 23], [16, 17, 15], [9, 8, 10]):  # (9 and 10 tokens: the smallest tiled mixtures, 8: the widest mat-vec)
        assert err(run_portions(m, toks, sizes), want) < TOL[dtype], sizes


def test_first_tokens_of_a_sequence(made):
    m, cfg, t = made("aligned", "float32")
    for n in (1, 2, 3, 5):
        toks = tokens_for(cfg, n, seed=10 + n)
        want = seq_oracle.run_zusolix(cfg, t, toks)
        assert err(run_portions(m, toks, [n]), want) < TOL["float32"]
        assert err(run_portions(m, toks, [1]), want) < TOL["float32"]


def test_interleaved_requests_and_reused_slots(made):
    """requests of unequal length fed in turns through the scheduler against each alone; then every slot is used again and must start from nothing"""
    m, cfg, t = made("aligned", "float32", max_batch=16)
    seqs = [tokens_for(cfg, n, seed=20 + n) for n in (61, 9, 88)]
    want = [seq_oracle.run_zusolix(cfg, t, s) for s in seqs]
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
    for r in range(4):  # a short request after a long one in the same slot: what the long one left in the cache and the state must not be seen
        which = 2 if r % 2 == 0 else 1
        assert err(sched.feed("again", seqs[which], np.arange(len(seqs[which]))), want[which]) < TOL["float32"]
        sched.finish("again")
    with pytest.raises(hip.PSHipError):
        [m.acquire() for _ in range(4)]
    for s in range(3):
        m.release(s)


# ---------------------------------------------------------------------------------------------------------------- weights made so that a fault shows
def marked_model(aligned, cap, every, seed=0, moe=True):
    """Token 0 is a MARK: its embedding alone has feature 0 (norm weights one, so the grouped norm keeps it apart); every key reads feature 0 into one
    channel of its head and every query has a constant there (a bias), so a query's score for a mark is far above all others -- held down only by the
    soft cap -- and every value channel reads feature 0 too.  The first layer's output matrix is large, so what the attention finds decides the logits.
    A second layer is an element-wise recurrence whose gate is nearly shut: the state it carries holds what the first tokens put in.  (moe False: its
    feed-forward is dense -- in bfloat16 a router's close call may go the other way, which is no fault of the mechanism under test.)"""
    rng = np.random.default_rng(seed)
    W, V = (64, 24) if aligned else (30, 24)
    H, G, d, dv = (4, 2, 16, 8) if aligned else (3, 1, 10, 6)
    a = ZA(H, G, d, dv, 1.0, cap, (0.6, every))
    second = ZL("mingru", {"width": 20}, moe=(4, 2, 12), shared=8) if moe else ZL("mingru", {"width": 20}, ff=24)
    cfg = ZC(W, V, [ZL("attention", a), second], groups=2, eps=1e-5, embed_scale=1.0, residual_mult=0.9)
    t = synth.seq_tensors(cfg, seed)
    e = rng.standard_normal((V, W)).astype(np.float32)
    e[:, 0] = 0.0
    e[0, 0] = 6.0
    t["embed"], t["l0.norm1"] = e, np.ones(W, np.float32)
    c = d - 1
    k = rng.standard_normal((G * d, W)).astype(np.float32) * 0.1
    k[:, 0] = 0.0
    q = rng.standard_normal((H * d, W)).astype(np.float32) * 0.1
    qb = np.zeros(H * d, np.float32)
    for g in range(G):
        k[g * d + c, 0] = 2.0
    for h in range(H):
        qb[h * d + c] = 1.5
    v = rng.standard_normal((G * dv, W)).astype(np.float32) * 0.2
    v[:, 0] = 1.5
    p = "l0.mix."
    t[p + "q"], t[p + "q.b"], t[p + "k"], t[p + "k.b"], t[p + "v"], t[p + "v.b"] = q, qb, k, np.zeros(G * d, np.float32), v, np.zeros(G * dv, np.float32)
    t["l1.mix.z.b"] = np.full(20, -4.0, np.float32)  # z = sigmoid(-4 + ...) is small: the state forgets slowly
    return cfg, bf16(t)


def marked_tokens(cfg, n, marks, seed):
    toks = tokens_for(cfg, n, seed, lo=1)
    toks[list(marks)] = 0
    return toks


@pytest.mark.parametrize("aligned", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_in_prompts_and_in_decoding(made, dtype, aligned):
    """One mark at position 4, 470 tokens: every later query must still find it.  The plain statement in which a query sees only its last 256 (or 300, or 64)
    positions is far off on every row behind that reach; the library agrees with the right one in a prompt cut into portions of 64 (keys across portion
    and tile borders), and on 170 tokens decoded one by one behind a 300-token prompt."""
    cfg, t = marked_model(aligned, 9.0, 50, moe=dtype == "float32")
    m, _, _ = made("marked%d" % aligned, dtype, max_batch=64, cfg=cfg, tensors=t)
    toks = marked_tokens(cfg, 470, (4,), seed=3)
    want = seq_oracle.run_zusolix(cfg, t, toks)
    for reach in (64, 256, 300):
        wrong = seq_oracle.run_zusolix(cfg, t, toks, attn_kw={"reach": reach})
        assert min(rows(wrong, want, [4 + reach, 4 + reach + 1, 469])) > 0.1, reach
        assert max(rows(wrong, want, range(0, reach))) < 1e-9  # (up to there such a query still sees everything)
    tol = 1e-3 if dtype == "float32" else TOL[dtype]
    s = m.acquire()
    got = [m.forward(s, toks[:300], np.arange(300))] + [m.forward(s, toks[i:i + 1], [0]) for i in range(300, 470)]
    m.release(s)
    assert max(rows(np.concatenate(got), want, range(len(toks)))) < tol
    for sizes in ([470], [64], [61, 2, 100]):
        assert max(rows(run_portions(m, toks, sizes), want, range(len(toks)))) < tol, sizes


@pytest.mark.parametrize("aligned", [False, True])
def test_soft_cap_and_temperature_steps_at_their_edges(made, aligned):
    """The mark's score is about 10 x the temperature and the cap 4: without the cap the mark takes all the weight, with it a share.  The temperature
    steps at positions 10, 21, 32, ... (floor((p + 1) / 11) changes): the plain statement without it, or stepping one token early or late, is off from
    exactly those rows on; the library agrees with the right one with an edge inside a prompt, at a portion's border and on decoded tokens."""
    every = 11
    cfg, t = marked_model(aligned, 4.0, every, seed=1)
    m, _, _ = made("edges%d" % aligned, "float32", max_batch=8, cfg=cfg, tensors=t)
    toks = marked_tokens(cfg, 60, (2,), seed=4)
    want = seq_oracle.run_zusolix(cfg, t, toks)
    assert min(rows(seq_oracle.run_zusolix(cfg, t, toks, attn_kw={"use_cap": False}), want, range(3, 60))) > 0.02
    no_temp = seq_oracle.run_zusolix(cfg, t, toks, attn_kw={"use_temperature": False})
    assert max(rows(no_temp, want, range(0, every - 1))) < 1e-9 and min(rows(no_temp, want, range(every - 1, 60))) > 1e-3
    for shift in (-1, 1):  # the step one token early / late: the rows at the edges differ
        wrong = seq_oracle.run_zusolix(cfg, t, toks, attn_kw={"temperature_shift": shift})
        edge = [p for p in range(3, 60) if seq_oracle.query_temperature(max(0, p - shift), 0.6, every) != seq_oracle.query_temperature(p, 0.6, every)]
        assert len(edge) == 5 and all((p + 1) % every in (0, every - 1) for p in edge)
        assert min(rows(wrong, want, edge)) > 1e-3
    for sizes in ([60], [1], [2], [8], [10, 1, 1, 9], [9, 2, 10, 1], [21, 1, 1, 10]):
        got = run_portions(m, toks, sizes)
        assert max(rows(got, want, range(len(toks)))) < 1e-3, sizes


def test_the_recurrence_carries_its_state_through_long_decoding(made):
    """a gate that is nearly shut: without the carried state (the plain statement with the state dropped at every token) every row is far off; the library
    agrees with the right one over 400 tokens, decoded singly and in portions that cut the scan's chunks anywhere"""
    cfg, t = marked_model(False, 9.0, 50, seed=2)
    m, _, _ = made("carry", "float32", max_batch=64, cfg=cfg, tensors=t)
    toks = marked_tokens(cfg, 400, (7,), seed=5)
    want = seq_oracle.run_zusolix(cfg, t, toks)
    assert min(rows(seq_oracle.run_zusolix(cfg, t, toks, gru_kw={"carry": False}), want, range(1, 400))) > 1e-3
    for sizes in ([13, 1, 1, 1, 1, 1, 1, 1], [64], [17, 33, 2, 64, 5]):
        assert max(rows(run_portions(m, toks, sizes), want, range(len(toks)))) < 1e-3, sizes


def test_long_decoding_keeps_the_states(made):
    m, cfg, t = made("aligned", "float32", max_batch=16)
    toks = tokens_for(cfg, 260, seed=6)
    want = seq_oracle.run_zusolix(cfg, t, toks)
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
    want = seq_oracle.run_zusolix(cfg, t, full[:-1])
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
    """mode bit 1 keeps the per-key attention and the 64 x 64 mat-mul (also for the experts' grouped products): the wide mat-mul, the mat-vecs and the
    matrix-core attention of a portion and of a single token must give the same logits (fp32: up to the order of sums)"""
    m, cfg, t = made(name, dtype, max_batch=64)
    toks = tokens_for(cfg, 150, seed=9)
    fast = [run_portions(m, toks, sizes) for sizes in ([64], [1], [40, 1, 1, 1, 9])]
    m.set_mode(2)
    plain = [run_portions(m, toks, sizes) for sizes in ([64], [1], [40, 1, 1, 1, 9])]
    m.set_mode(0)
    want = seq_oracle.run_zusolix(cfg, t, toks)
    for a, b in zip(fast, plain):
        assert err(a, b) < (1e-4 if dtype == "float32" else TOL[dtype])
        assert err(a, want) < TOL[dtype]


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
    assert err(np.concatenate(got), seq_oracle.run_zusolix(cfg, t, toks)) < TOL["float32"]
    m.close()
