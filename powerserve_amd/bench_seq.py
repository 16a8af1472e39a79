"""Throughput of a layer-list model at layer sizes of real models (random weights), beside the quantized Llama path at equal width, depth
and feed-forward size.  Used by bench.py --layer-list; prints nothing itself."""
from __future__ import annotations

import ctypes as C
import tempfile
import time

import numpy as np

from . import gguf, hip, seqmodel, synth

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0

# name: (width, feed-forward, heads, head size, q_rank, kv_rank, rot_dim, window, layers, the Llama preset of the same width / depth class)
SIZES = {
    "2048x6": dict(width=2048, ff=8192, heads=16, dim=128, q_rank=768, kv_rank=512, rot_dim=64, window=1024, layers=6, llama="llama-1b-dims-2l"),
    "4096x3": dict(width=4096, ff=14336, heads=32, dim=128, q_rank=1536, kv_rank=512, rot_dim=64, window=1024, layers=3, llama="llama-8b-dims-4l"),
    # Vobisun (parallel layers: windowed attention with pooled blocks beside gated linear attention, SiLU-gated feed-forward) at the same widths, feed-forward
    # sizes, head counts and numbers of layer RUNS; `beside` names the layer-list model it is measured next to
    "v2048x6": dict(design="Vobisun", width=2048, ff=8192, heads=16, kv_heads=4, dim=128, window=1024, pool=64, rot_dims=64, lin_heads=16, lin_dim=64, lin_vdim=128,
                    layers=4, loop=(1, 3, 2), beside="2048x6"),
    "v4096x3": dict(design="Vobisun", width=4096, ff=14336, heads=32, kv_heads=8, dim=128, window=1024, pool=64, rot_dims=64, lin_heads=32, lin_dim=64, lin_vdim=128,
                    layers=3, loop=None, beside="4096x3"),
    # Zusolix (two-norm parallel layers with a depth average; causal attention with a soft cap and a query temperature, or an element-wise gated recurrence;
    # the first layer's feed-forward dense, the others 8 experts of which a token uses 2, plus a shared one: 2 x ff/4 + ff/2 = ff active rows) beside the
    # Vobisun model of equal width, feed-forward size, head counts and layer runs
    "z2048x6": dict(design="Zusolix", width=2048, ff=8192, heads=16, kv_heads=4, dim=128, gru=3072, experts=8, top=2, order="aagaag", layers=6, beside="v2048x6"),
    "z4096x3": dict(design="Zusolix", width=4096, ff=14336, heads=32, kv_heads=8, dim=128, gru=6144, experts=8, top=2, order="aga", layers=3, beside="v4096x3"),
    # Pokatar (pre-norm layers with layer norms; causal attention with a sink, per-head norms and an element-wise gate, or latent attention with a shared rotated
    # key part; the first layer's feed-forward relu-gated dense, the others 8 squared-relu experts + 2 identity experts in 5 groups of which three stay, top 2, plus
    # a shared expert -- two matrices per expert instead of three, so an inner size of 3/2 x ff/4 and 3/2 x ff/2 holds the Zusolix experts' weights) beside the
    # Zusolix model of equal width, feed-forward size, head counts and layers
    "p2048x6": dict(design="Pokatar", width=2048, ff=8192, heads=16, kv_heads=4, dim=128, kv_rank=512, rot_dim=64, experts=8, identity=2, groups=(5, 3), top=2,
                    order="aalaal", layers=6, beside="z2048x6"),
    "p4096x3": dict(design="Pokatar", width=4096, ff=14336, heads=32, kv_heads=8, dim=128, kv_rank=512, rot_dim=64, experts=8, identity=2, groups=(5, 3), top=2,
                    order="ala", layers=3, beside="z4096x3"),
}


def config(z: dict, vocab: int = 4096) -> dict:
    H, d = z["heads"], z["dim"]
    if z.get("design") == "Pokatar":
        att = synth.pokatar_attention(H, z["kv_heads"], d, d, float(d ** -0.5))
        lat = synth.pokatar_latent(H, d, z["rot_dim"], d, z["kv_rank"], float((d + z["rot_dim"]) ** -0.5), 5e5, (8.0, 4096, 16.0, 2.0))
        layers = []
        for i, k in enumerate(z["order"]):
            mixer = ("attention", att) if k == "a" else ("latent_attention", lat)
            layers.append(synth.pokatar_layer(*mixer, ff=z["ff"]) if i == 0 else
                          synth.pokatar_layer(*mixer, moe=(z["experts"], z["top"], z["ff"] * 3 // 8, z["identity"], *z["groups"]), shared=z["ff"] * 3 // 4))
        return synth.pokatar_config(z["width"], vocab, layers)
    if z.get("design") == "Zusolix":
        att = synth.zusolix_attention(H, z["kv_heads"], d, d, float(d ** -0.5), 30.0, (0.1, 1024))
        layers = []
        for i, k in enumerate(z["order"]):
            mixer = ("attention", att) if k == "a" else ("mingru", {"width": z["gru"]})
            layers.append(synth.zusolix_layer(*mixer, ff=z["ff"]) if i == 0 else
                          synth.zusolix_layer(*mixer, moe=(z["experts"], z["top"], z["ff"] // 4), shared=z["ff"] // 2))
        return synth.zusolix_config(z["width"], vocab, layers, groups=4, embed_scale=float(z["width"] ** 0.5), residual_mult=0.5)
    if z.get("design") == "Vobisun":
        left = dict(heads=H, kv_heads=z["kv_heads"], dim=d, vdim=d, mask={"size": z["window"], "pool": z["pool"]},
                    rot={"base": 1e6, "dims": z["rot_dims"], "scaling": {"factor": 4.0}}, scale=float(d ** -0.5))
        right = dict(heads=z["lin_heads"], dim=z["lin_dim"], vdim=z["lin_vdim"], tau=16.0)
        return synth.parallel_config(z["width"], vocab, [synth.parallel_layer(z["ff"], left, right, 1.0, 1.0) for _ in range(z["layers"])], taps=4,
                                     embed_scale=float(z["width"] ** 0.5), loop=z["loop"])
    kinds = {
        "delta": dict(heads=H, kv_heads=max(1, H // 2), dim=d, vdim=d, conv=4),
        "latent_attention": dict(heads=H, dim=d, vdim=d, q_rank=z["q_rank"], kv_rank=z["kv_rank"], rot_dim=z["rot_dim"],
                                 rot={"base": 1e6, "dims": z["rot_dim"]}, mask={"size": z["window"]}, scale=float((d + z["rot_dim"]) ** -0.5)),
        "wkv": dict(heads=H, dim=d),
    }
    order = ["delta", "latent_attention", "wkv"]
    layers = [synth.seq_layer(order[i % 3], z["ff"], **kinds[order[i % 3]]) for i in range(z["layers"])]
    return synth.seq_config(z["width"], vocab, layers, taps=4)


def _timed(ctx, fn):
    ctx.sync()
    t0 = time.perf_counter()
    fn()
    ctx.sync()
    return time.perf_counter() - t0


def _kernel(ctx, m, which, T, reps):
    us, by, fl = C.c_double(), C.c_double(), C.c_double()
    ctx.check(ctx.L.ps_hip_seq_bench_kernel(m.h, which, T, reps, C.byref(us), C.byref(by), C.byref(fl)))
    return us.value, by.value, fl.value


def run_size(ctx, name: str, prompt_len: int, steps: int, max_batch: int, seed: int = 0, with_llama: bool = True, with_beside: bool = True) -> dict:
    z = SIZES[name]
    cfg = config(z)
    out = {"size": name, "config": {k: v for k, v in z.items() if k not in ("llama", "beside")}, "prompt_len": prompt_len, "decode_steps": steps, "portion": max_batch}
    with tempfile.TemporaryDirectory() as d:
        t0 = time.time()
        synth.write_seq_model_dir(d, cfg, seed)
        m = seqmodel.SeqModel(ctx, d, dtype="bfloat16", max_batch=max_batch, n_slots=1, max_context=prompt_len + steps + 64)
        out["make_and_load_s"] = round(time.time() - t0, 1)
    out["layer_runs"] = m.n_runs
    prompt = np.random.default_rng(1).integers(0, cfg["vocab"], prompt_len).astype(np.int32)
    s = m.acquire()
    m.forward(s, prompt[:max_batch])  # untimed: first use of every kernel
    m.release(s)
    s = m.acquire()
    pre = _timed(ctx, lambda: m.forward(s, prompt[:-1]))
    m.decode_greedy(s, int(prompt[-1]), 4)
    dec = _timed(ctx, lambda: m.decode_greedy(s, 7, steps))
    m.release(s)
    out["prefill_tok_s"] = (prompt_len - 1) / pre
    out["decode_tok_s"] = steps / dec
    out["weight_bytes_per_token"] = m.weight_bytes_per_token
    out["decode_hbm_frac"] = m.weight_bytes_per_token * steps / dec / 1e9 / HBM_PEAK_GBS
    flops_tok = 2.0 * (m.weight_bytes_per_token / 2 - cfg["vocab"] * cfg["width"])
    out["prefill_mfma_frac"] = flops_tok * (prompt_len - 1) / pre / 1e12 / MFMA_BF16_PEAK_TFLOPS
    us, by, fl = _kernel(ctx, m, 0, 1, 20)
    out["ff_up_matvec"] = {"us": us, "GBs": by / us / 1e3, "hbm_frac": by / us / 1e3 / HBM_PEAK_GBS}
    us, by, fl = _kernel(ctx, m, 0, max_batch, 5)
    out["ff_up_matmul"] = {"tokens": max_batch, "us": us, "TFLOPs": fl / us / 1e6, "mfma_frac": fl / us / 1e6 / MFMA_BF16_PEAK_TFLOPS}
    if z.get("experts"):  # the experts' grouped products: up (gate / up rows, SiLU pair) and down, a single token and a portion
        for which, key in ((2, "moe_up"), (3, "moe_down")):
            us, by, fl = _kernel(ctx, m, which, 1, 20)
            out[key + "_matvec"] = {"us": us, "GBs": by / us / 1e3, "hbm_frac": by / us / 1e3 / HBM_PEAK_GBS}
            us, by, fl = _kernel(ctx, m, which, max_batch, 5)
            out[key + "_matmul"] = {"tokens": max_batch, "us": us, "TFLOPs": fl / us / 1e6, "mfma_frac": fl / us / 1e6 / MFMA_BF16_PEAK_TFLOPS}
    m.close()
    if with_beside and z.get("beside"):  # the closest existing model at equal size, same workload
        out["beside"] = run_size(ctx, z["beside"], prompt_len, steps, max_batch, seed, with_llama=False, with_beside=False)
    if with_llama and z.get("llama"):
        with tempfile.TemporaryDirectory() as d:
            synth.write_model_dir(d, z["llama"], gguf.Q4_K, n_ctx=prompt_len + steps + 64, seed=seed)
            lm = hip.Model(ctx, d, max_batch=512, n_ctx=prompt_len + steps + 64)
            lm.prefill(prompt[:128], 128)
            lm.reset()
            pre = _timed(ctx, lambda: lm.prefill(prompt[:-1], 128))
            lm.decode_greedy(int(prompt[-1]), 4)
            dec = _timed(ctx, lambda: lm.decode_greedy(7, steps))
            out["llama_q4k"] = {"preset": z["llama"], "n_layers": lm.cfg.n_layers, "prefill_tok_s": (prompt_len - 1) / pre, "decode_tok_s": steps / dec,
                                "weight_bytes_per_token": lm.weight_bytes_per_token,
                                "decode_hbm_frac": lm.weight_bytes_per_token * steps / dec / 1e9 / HBM_PEAK_GBS}
            lm.close()
    return out


def run(sizes, prompt_len=2048, steps=64, max_batch=512, device=0, with_llama=True) -> dict:
    ctx = hip.Ctx(device)
    res = {"metric": "layer_list_throughput", "dtype": "bf16", "data": "synthetic", "device": ctx.name(), "sizes": []}
    for name in sizes:
        res["sizes"].append(run_size(ctx, name, prompt_len, steps, max_batch, with_llama=with_llama))
    ctx.close()
    return res
