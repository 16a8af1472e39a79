"""Plain, slow float64 statement of the layer-list design (checker only: it shares no code with powerserve_amd).

Everything is computed for a whole sequence at once with explicit loops over time; one function per mechanism.  W maps tensor names to
float arrays, cfg is the parsed config.json.  Notation: x residual stream [T, width]; h what a sublayer reads; S a recurrent state.
"""
import numpy as np


def unit_rms(a, eps):
    return a / np.sqrt(np.mean(a * a, axis=-1, keepdims=True) + eps)


def offset_norm(a, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return unit_rms(a, eps) * (1.0 + w)


def silu(a):
    return a / (1.0 + np.exp(-a))


def softplus(a):
    return np.logaddexp(0.0, a)


def time_conv(a, w):
    """Per-channel causal filter: out[t] = sum_j w[:, j] * a[t - (taps - 1) + j], nothing before t = 0.  a [T, C], w [C, taps]."""
    T, taps = a.shape[0], w.shape[1]
    out = np.zeros_like(a)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                out[t] += w[:, j] * a[s]
    return out


def xielu(z, p, q):
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (np.expm1(np.minimum(z, 0.0)) - z) + 0.5 * z
    return np.where(z > 0, pos, neg)


def wkv_mixer(W, pre, h, mc, eps):
    T, width = h.shape
    H, d = mc["heads"], mc["dim"]
    out = np.zeros((T, H * d))
    S = np.zeros((H, d, d))
    prev = np.zeros(width)
    bonus = W[pre + "u"]
    for t in range(T):
        mixed = {s: h[t] + (prev - h[t]) * W[pre + "mu." + s] for s in "rkvgw"}
        r = (W[pre + "r"] @ mixed["r"]).reshape(H, d)
        k = (W[pre + "k"] @ mixed["k"]).reshape(H, d)
        v = (W[pre + "v"] @ mixed["v"]).reshape(H, d)
        gate = silu(W[pre + "g"] @ mixed["g"])
        decay = np.exp(-np.exp(W[pre + "w2"] @ np.tanh(W[pre + "w1"] @ mixed["w"]) + W[pre + "w0"])).reshape(H, d)
        o = np.zeros((H, d))
        for hd in range(H):
            kv = np.outer(k[hd], v[hd])
            o[hd] = (S[hd] + bonus[hd][:, None] * kv).T @ r[hd]
            S[hd] = decay[hd][:, None] * S[hd] + kv
        out[t] = unit_rms(o, eps).reshape(-1) * W[pre + "norm"] * gate
        prev = h[t]
    return out @ W[pre + "o"].T


def delta_mixer(W, pre, h, mc, eps):
    T = h.shape[0]
    H, KH, d, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]

    def branch(name):
        return silu(time_conv(h @ W[pre + name].T, W[pre + name + ".conv"]))

    q, k, v = branch("q").reshape(T, KH, d), branch("k").reshape(T, KH, d), branch("v").reshape(T, H, dv)
    q = q / np.sqrt(np.sum(q * q, -1, keepdims=True) + 1e-6) / np.sqrt(d)
    k = k / np.sqrt(np.sum(k * k, -1, keepdims=True) + 1e-6)
    beta = 1.0 / (1.0 + np.exp(-(h @ W[pre + "b"].T)))
    keep = np.exp(-np.exp(W[pre + "A_log"]) * softplus(h @ W[pre + "a"].T + W[pre + "dt_bias"]))
    gate = silu(h @ W[pre + "g"].T).reshape(T, H, dv)
    S = np.zeros((H, d, dv))
    out = np.zeros((T, H, dv))
    for t in range(T):
        for hd in range(H):
            g = hd // (H // KH)
            S[hd] *= keep[t, hd]
            write = beta[t, hd] * (v[t, hd] - S[hd].T @ k[t, g])
            S[hd] += np.outer(k[t, g], write)
            out[t, hd] = S[hd].T @ q[t, g]
    out = unit_rms(out, eps) * W[pre + "norm"] * gate
    return out.reshape(T, H * dv) @ W[pre + "o"].T


def rotate(vec, pos, base, dims):
    """First `dims` numbers of vec turn in pairs (i, i + dims/2) by pos * base^(-2i/dims); the rest is kept."""
    out = np.array(vec, dtype=np.float64)
    half = dims // 2
    for i in range(half):
        ang = pos * base ** (-2.0 * i / dims)
        a, b = vec[..., i], vec[..., i + half]
        out[..., i] = a * np.cos(ang) - b * np.sin(ang)
        out[..., i + half] = b * np.cos(ang) + a * np.sin(ang)
    return out


def latent_mixer(W, pre, h, mc, eps, window=None):
    T = h.shape[0]
    H, d, dr, dv, R = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    window = mc["mask"]["size"] if window is None else window
    base, dims = mc["rot"]["base"], mc["rot"]["dims"]
    out = np.zeros((T, H * dv))
    lat, shared = [], []
    for t in range(T):
        both = W[pre + "dkv"] @ h[t]
        lat.append(unit_rms(both[:R], eps) * W[pre + "dkv.norm"])
        shared.append(rotate(both[R:], t, base, dims))
        cq = unit_rms(W[pre + "dq"] @ h[t], eps) * W[pre + "dq.norm"]
        q = (W[pre + "uq"] @ cq).reshape(H, d + dr)
        o = np.zeros((H, dv))
        seen = range(max(0, t - window + 1), t + 1)
        for hd in range(H):
            q_plain, q_rot = q[hd, :d], rotate(q[hd, d:], t, base, dims)
            sc = np.array([(q_plain @ (W[pre + "uk"][hd * d:(hd + 1) * d] @ lat[s]) + q_rot @ shared[s]) * mc["scale"] for s in seen])
            p = np.exp(sc - sc.max())
            p /= p.sum()
            o[hd] = sum(p[n] * (W[pre + "uv"][hd * dv:(hd + 1) * dv] @ lat[s]) for n, s in enumerate(seen))
        out[t] = o.reshape(-1)
    return out @ W[pre + "o"].T


MIXERS = {"wkv": wkv_mixer, "delta": delta_mixer, "latent_attention": latent_mixer}


def feed_forward(W, pre, h):
    a = W[pre + "act"]
    return xielu(h @ W[pre + "up"].T, a[0], a[1]) @ W[pre + "down"].T


def run(cfg, W, tokens, per_layer=None, window_override=None):
    """Logits [T, vocab] of a whole sequence.  window_override: {layer index: window} to state a WRONG model on purpose (sensitivity checks)."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)]
    for i, lc in enumerate(cfg["layers"]):
        p = "l%d." % i
        h = offset_norm(x, W[p + "norm1"], eps)
        h = h + time_conv(h, W[p + "canon1"])
        if lc["type"] == "latent_attention" and window_override and i in window_override:
            y = latent_mixer(W, p + "mix.", h, lc["mixer"], eps, window_override[i])
        else:
            y = MIXERS[lc["type"]](W, p + "mix.", h, lc["mixer"], eps)
        x = x + offset_norm(y, W[p + "norm1b"], eps)
        if lc.get("mlp"):
            h = offset_norm(x, W[p + "norm2"], eps)
            h = h + time_conv(h, W[p + "canon2"])
            x = x + offset_norm(feed_forward(W, p + "mlp.", h), W[p + "norm2b"], eps)
        if per_layer is not None:
            per_layer.append(x.copy())
    return offset_norm(x, W["final.norm"], eps) @ W["head"].T * cfg["logit_scale"]


# ---------------------------------------------------------------------------------------------------------------------------------
# Vobisun: parallel layers (one norm; mixer and feed-forward read it, only the mixer's copy passes the input filter), a mixer made of two
# mixers side by side -- windowed attention with pooled blocks behind the window and a sink, and gated linear attention -- a SiLU-gated
# feed-forward, plain norm weights, a scaled embedding, and a run of layers that is repeated with the same weights.

def plain_norm(a, w, eps):
    return unit_rms(a, eps) * w


def rotate_pairs(vec, pos, base, dims, factor=1.0):
    """Neighbours (2i, 2i+1), i < dims/2, turn by pos * base^(-2i/dims) / factor; the rest of vec is kept."""
    out = np.array(vec, dtype=np.float64)
    for i in range(dims // 2):
        ang = pos * (base ** (-2.0 * i / dims) / factor)
        a, b = vec[..., 2 * i], vec[..., 2 * i + 1]
        out[..., 2 * i] = a * np.cos(ang) - b * np.sin(ang)
        out[..., 2 * i + 1] = b * np.cos(ang) + a * np.sin(ang)
    return out


def visible_tokens(i, size):
    """Positions a query at i sees directly."""
    return range(max(0, i - size + 1), i + 1)


def visible_blocks(i, size, pool):
    """Blocks of `pool` positions that lie wholly before the window of a query at i."""
    if not pool:
        return range(0)
    return range(max(0, (i - size + 1) // pool)) if i - size + 1 > 0 else range(0)


def pooled_window_attention(W, pre, h, mc, eps, size=None, pool=None, use_sink=True):
    """Soft-max attention over the last `size` tokens plus one mean key / value per block of `pool` tokens wholly before them, a sink in
    the denominator, a per-head temperature, norms over the whole q and k projections, neighbour-pair rotary, a sigmoid gate per head."""
    T = h.shape[0]
    H, G, d, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    mask = mc.get("mask") or {}
    size = (mask.get("size") or T + 1) if size is None else size
    pool = mask.get("pool", 0) if pool is None else pool
    rot = mc.get("rot") or {}
    dims, base = rot.get("dims", 0), rot.get("base", 10000.0)
    factor = (rot.get("scaling") or {}).get("factor", 1.0)

    def proj(n):
        y = h @ W[pre + n].T
        return y + W[pre + n + ".b"] if pre + n + ".b" in W else y

    q, k, v = proj("q"), proj("k"), proj("v").reshape(T, G, dv)
    if pre + "q.norm" in W:
        q = plain_norm(q, W[pre + "q.norm"], eps)
    if pre + "k.norm" in W:
        k = plain_norm(k, W[pre + "k.norm"], eps)
    q, k = q.reshape(T, H, d), k.reshape(T, G, d)
    for t in range(T):
        q[t], k[t] = rotate_pairs(q[t], t, base, dims, factor), rotate_pairs(k[t], t, base, dims, factor)
    gate = 1.0 / (1.0 + np.exp(-(h @ W[pre + "g"].T))) if pre + "g" in W else np.ones((T, H))
    temp = W[pre + "temp"] if pre + "temp" in W else np.ones(H)
    out = np.zeros((T, H, dv))
    for t in range(T):
        toks, blocks = list(visible_tokens(t, size)), list(visible_blocks(t, size, pool))
        for hd in range(H):
            g = hd // (H // G)
            keys = [k[b * pool:(b + 1) * pool, g].mean(axis=0) for b in blocks] + [k[s, g] for s in toks]
            vals = [v[b * pool:(b + 1) * pool, g].mean(axis=0) for b in blocks] + [v[s, g] for s in toks]
            sc = np.array([q[t, hd] @ kk for kk in keys]) * mc["scale"] * temp[hd]
            top = max(sc.max(), W[pre + "sink"][hd]) if use_sink and pre + "sink" in W else sc.max()
            e = np.exp(sc - top)
            den = e.sum() + (np.exp(W[pre + "sink"][hd] - top) if use_sink and pre + "sink" in W else 0.0)
            out[t, hd] = sum(e[n] * vals[n] for n in range(len(keys))) / den * gate[t, hd]
    return out.reshape(T, H * dv) @ W[pre + "o"].T


def gated_linear_attention(W, pre, h, mc, eps):
    """S <- diag(alpha) S + k v^T,  o = S^T q  per head, alpha = sigmoid(z)^(1/tau) per key channel from a two-matrix projection."""
    T = h.shape[0]
    H, d, dv, tau = mc["heads"], mc["dim"], mc["vdim"], mc["tau"]
    q = (h @ W[pre + "q"].T * d ** -0.5).reshape(T, H, d)
    k = (h @ W[pre + "k"].T).reshape(T, H, d)
    v = (h @ W[pre + "v"].T).reshape(T, H, dv)
    z = (h @ W[pre + "a1"].T) @ W[pre + "a2"].T + W[pre + "a2.b"]
    alpha = np.exp(-softplus(-z) / tau).reshape(T, H, d)
    S = np.zeros((H, d, dv))
    o = np.zeros((T, H, dv))
    for t in range(T):
        for hd in range(H):
            S[hd] = alpha[t, hd][:, None] * S[hd] + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S[hd].T @ q[t, hd]
    o = plain_norm(o, W[pre + "norm"], eps).reshape(T, H * dv) * silu(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def side_by_side_mixer(W, pre, h, mc, eps, **kw):
    return mc["left_scale"] * pooled_window_attention(W, pre + "left.", h, mc["left"], eps, **kw) + \
        mc["right_scale"] * gated_linear_attention(W, pre + "right.", h, mc["right"], eps)


def gated_feed_forward(W, pre, h):
    return (silu(h @ W[pre + "gate"].T) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def layer_runs(cfg):
    """Indices of the layers in the order they run: the looped stretch `times` times in a row."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b = loop["start"], loop["stop"]
    return list(range(a)) + list(range(a, b)) * loop["times"] + list(range(b, n))


def run_parallel(cfg, W, tokens, per_layer=None, **kw):
    """Logits [T, vocab] of a whole sequence of the parallel-layer design; kw overrides the attention's size / pool / use_sink on purpose
    (a WRONG model for sensitivity checks)."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    for i in layer_runs(cfg):
        lc, p = cfg["layers"][i], "l%d." % i
        h = plain_norm(x, W[p + "norm1"], eps)
        hm = h + time_conv(h, W[p + "canon1"]) if p + "canon1" in W else h
        if lc["type"] != "parallel":
            raise ValueError(lc["type"])
        y = side_by_side_mixer(W, p + "mix.", hm, lc["mixer"], eps, **kw)
        if lc.get("mlp"):
            y = y + gated_feed_forward(W, p + "mlp.", h)
        x = x + y
        if per_layer is not None:
            per_layer.append(x.copy())
    return plain_norm(x, W["final.norm"], eps) @ W["head"].T


# ---------------------------------------------------------------------------------------------------------------- Zusolix
# Parallel layers with two norms of the same vector,  X_(i+1) = x_i + m (mixer(norm1(x_i)) + ff(norm2(x_i))), where x_i, the input of layer i, is a
# weighted average over the embedding X_0 and all earlier results X_1 .. X_i (x_0 = X_0); norms in groups; attention without rotation whose queries
# grow with the position and whose scores are soft-capped; an element-wise gated recurrence; dense or mixture-of-experts feed-forwards.
def sigmoid(a):
    return 1.0 / (1.0 + np.exp(-a))


def grouped_norm(a, w, groups, eps):
    """the vector in `groups` equal consecutive parts, each divided by the root of (its own mean square + eps); then the weight"""
    n = a.shape[-1] // groups
    out = np.empty_like(a)
    for g in range(groups):
        part = a[..., g * n:(g + 1) * n]
        out[..., g * n:(g + 1) * n] = part / np.sqrt(np.mean(part * part, axis=-1, keepdims=True) + eps)
    return out * w


def query_temperature(p, coef, every):
    return 1.0 + coef * np.log(np.floor((p + 1) / every) + 1.0)


def capped_attention(W, pre, h, mc, reach=None, use_cap=True, use_temperature=True, temperature_shift=0):
    """Causal grouped-query soft-max attention, biases on q / k / v, no rotation.  reach: a WRONG model on purpose, in which a query sees only the last
    `reach` positions; use_cap / use_temperature False: wrong models without the soft cap / the query temperature; temperature_shift: a wrong model whose
    temperature steps that many tokens late (negative: early)."""
    T = h.shape[0]
    H, G, d, dv = mc["heads"], mc.get("kv_heads", mc["heads"]), mc["dim"], mc.get("vdim", mc["dim"])
    out = np.zeros((T, H * dv))
    keys, values = [], []
    cap, qt = mc.get("softcap"), mc.get("q_temp")
    for t in range(T):
        q = (W[pre + "q"] @ h[t] + W[pre + "q.b"]).reshape(H, d)
        keys.append((W[pre + "k"] @ h[t] + W[pre + "k.b"]).reshape(G, d))
        values.append((W[pre + "v"] @ h[t] + W[pre + "v.b"]).reshape(G, dv))
        if qt and use_temperature:
            q = q * query_temperature(max(0, t - temperature_shift), qt["coef"], qt["every"])
        first = 0 if reach is None else max(0, t - reach + 1)
        for hd in range(H):
            g = hd // (H // G)
            s = np.array([q[hd] @ keys[j][g] for j in range(first, t + 1)]) * mc["scale"]
            if cap and use_cap:
                s = cap * np.tanh(s / cap)
            e = np.exp(s - s.max())
            a = e / e.sum()
            out[t, hd * dv:(hd + 1) * dv] = sum(a[j - first] * values[j][g] for j in range(first, t + 1))
    return out @ W[pre + "o"].T


def min_gru(W, pre, h, mc, carry=True):
    """carry False: a WRONG model in which the state is lost at every token"""
    C = mc["width"]
    S = np.zeros(C)
    out = np.zeros((h.shape[0], C))
    for t in range(h.shape[0]):
        z = sigmoid(W[pre + "z"] @ h[t] + W[pre + "z.b"])
        u = W[pre + "x"] @ h[t] + W[pre + "x.b"]
        cand = np.where(u >= 0, u + 0.5, sigmoid(u))
        S = (1.0 - z) * (S if carry else 0.0) + z * cand
        out[t] = S * silu(W[pre + "g"] @ h[t])
    return out @ W[pre + "o"].T


def one_expert(W, pre, a):
    return W[pre + "down"] @ (silu(W[pre + "gate"] @ a) * (W[pre + "up"] @ a))


def expert_mixture(W, pre, h, mlp, weight_on_output=False, use_shared=True):
    """Scores sigmoid(router h); the `top` largest (the lower index on a tie); a chosen expert sees score * h.  weight_on_output: a WRONG model in which
    the score multiplies the expert's result instead."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        s = sigmoid(W[pre + "router"] @ h[t])
        left = list(range(E))
        for _ in range(top):
            e = max(left, key=lambda i: (s[i], -i))
            left.remove(e)
            out[t] += s[e] * one_expert(W, f"{pre}e{e}.", h[t]) if weight_on_output else one_expert(W, f"{pre}e{e}.", s[e] * h[t])
        if mlp.get("shared") and use_shared:
            gate = sigmoid(W[pre + "shared.sg"] @ h[t])[0] if pre + "shared.sg" in W else 1.0
            out[t] += gate * one_expert(W, pre + "shared.", h[t])
    return out


def zusolix_feed_forward(W, pre, h, mlp, **kw):
    if mlp["kind"] == "dense":
        return np.stack([one_expert(W, pre, h[t]) for t in range(h.shape[0])])
    return expert_mixture(W, pre, h, mlp, **kw)


def depth_average(w, streams):
    return sum(w[j] * streams[j] for j in range(len(streams)))


def run_zusolix(cfg, W, tokens, per_layer=None, use_depth=True, attn_kw=None, gru_kw=None, moe_kw=None):
    """-> logits [T, vocab]; per_layer (a list) receives what every layer hands on.  use_depth False: a WRONG model without the depth average."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps, groups, m = cfg["norm"]["eps"], cfg["norm"].get("groups", 1), cfg.get("residual_mult", 1.0)
    x = W["embed"][np.asarray(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    streams = [x]
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h1 = grouped_norm(x, W[p + "norm1"], groups, eps)
        if lc["type"] == "attention":
            y = capped_attention(W, p + "mix.", h1, lc["mixer"], **(attn_kw or {}))
        else:
            y = min_gru(W, p + "mix.", h1, lc["mixer"], **(gru_kw or {}))
        if lc.get("mlp"):
            kw = (moe_kw or {}) if lc["mlp"]["kind"] == "moe" else {}
            y = y + zusolix_feed_forward(W, p + "mlp.", grouped_norm(x, W[p + "norm2"], groups, eps), lc["mlp"], **kw)
        streams.append(x + m * y)
        x = depth_average(W[p + "dwa"], streams) if use_depth and p + "dwa" in W else streams[-1]
        if per_layer is not None:
            per_layer.append(x)
    return grouped_norm(x, W["final.norm"], groups, eps) @ W["head"].T


# ------------------------------------------------------------------------------------------------ Pokatar
# Sequential pre-norm layers,  x += mixer(ln1(x)); x += ff(ln2(x)),  with mean-centred layer norms (a weight, no bias), two kinds of causal
# attention (grouped-query with per-head q / k norms, unit-rms values, a zero-score sink and an element-wise output gate; latent attention with a
# direct query projection, YaRN-scaled rotate-half rotary on a shared key part and a per-head output gate), a relu-gated dense feed-forward with
# biases, and a mixture of squared-relu experts behind a soft-max router with a selection correction, group-limited choice and identity experts.
# The logits are the final layer norm against the embedding table itself.


def centred_norm(a, w, eps):
    """(a - mean) / sqrt(var + eps) * w, var the mean of the squared deviations."""
    dev = a - np.mean(a, axis=-1, keepdims=True)
    return dev / np.sqrt(np.mean(dev * dev, axis=-1, keepdims=True) + eps) * w


def sink_softmax(scores, use_sink=True):
    """exp(s_j) / (1 + sum exp(s)): one more term of score 0 that carries no value."""
    m = max(np.max(scores), 0.0) if use_sink else np.max(scores)
    e = np.exp(scores - m)
    return e / (e.sum() + (np.exp(-m) if use_sink else 0.0))


def sink_gated_attention(W, pre, h, mc, eps, reach=None, use_sink=True, norm_values=True, gate_per_element=True):
    """Grouped-query causal attention: per-head RMS norms of q and k (one weight vector of `dim` shared by the heads), values divided by their
    own root mean square, no positions, the sink soft-max, sigmoid(W_g h) element by element on the concatenated heads."""
    T = h.shape[0]
    H, G, d, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = (h @ W[pre + "q"].T).reshape(T, H, d)
    k = (h @ W[pre + "k"].T).reshape(T, G, d)
    v = (h @ W[pre + "v"].T).reshape(T, G, dv)
    q = unit_rms(q, eps) * W[pre + "q.norm"]
    k = unit_rms(k, eps) * W[pre + "k.norm"]
    if norm_values:
        v = unit_rms(v, eps)
    gate = sigmoid(h @ W[pre + "g"].T)
    out = np.zeros((T, H, dv))
    for i in range(T):
        lo = 0 if reach is None else max(0, i - reach + 1)
        for hd in range(H):
            g = hd // (H // G)
            s = np.array([q[i, hd] @ k[j, g] for j in range(lo, i + 1)]) * mc["scale"]
            p = sink_softmax(s, use_sink)
            out[i, hd] = p @ v[lo:i + 1, g]
    out = out.reshape(T, H * dv)
    out = out * gate if gate_per_element else out
    return out @ W[pre + "o"].T


def yarn_frequencies(rot):
    """f_i = base^(-2i/dims) blended with f_i / factor by a ramp over the pair index; -> (frequencies, the factor on cos and sin)."""
    dims, base, sc = rot["dims"], rot["base"], rot.get("scaling")
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not sc:
        return f, 1.0
    def turn_index(t):
        return dims * np.log(sc["original"] / (2.0 * np.pi * t)) / (2.0 * np.log(base))
    lo = max(np.floor(turn_index(sc["fast"])), 0)
    hi = min(np.ceil(turn_index(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * np.log(sc["factor"]) + 1.0


def rotate_halves(vec, pos, freqs, mag):
    """Pairs (i, i + n) of the first 2n numbers, n = len(freqs), turned by pos * freqs[i]; cos and sin both times mag."""
    n = len(freqs)
    out = np.array(vec, dtype=np.float64)
    a = pos * freqs
    c, s = np.cos(a) * mag, np.sin(a) * mag
    u, v = vec[..., :n], vec[..., n:2 * n]
    out[..., :n] = u * c - v * s
    out[..., n:2 * n] = v * c + u * s
    return out


def shared_key_latent_attention(W, pre, h, mc, eps, reach=None, use_scaling=True, use_gate=True):
    """q straight from the input, laid out per head as [dim plain | rot_dim rotated]; keys and values from one normed latent per token plus one
    rotated key part shared by the heads; ordinary soft-max; each head's output times sigmoid of its row of W_g."""
    T = h.shape[0]
    H, d, dr, dv, R = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    rot = dict(mc["rot"])
    if not use_scaling:
        rot.pop("scaling", None)
    freqs, mag = yarn_frequencies(rot)
    q = (h @ W[pre + "q"].T).reshape(T, H, d + dr)
    down = h @ W[pre + "dkv"].T
    c = unit_rms(down[:, :R], eps) * W[pre + "dkv.norm"]
    kr = np.stack([rotate_halves(down[t, R:], t, freqs, mag) for t in range(T)])
    kp = (c @ W[pre + "uk"].T).reshape(T, H, d)
    v = (c @ W[pre + "uv"].T).reshape(T, H, dv)
    gate = sigmoid(h @ W[pre + "g"].T) if use_gate else np.ones((T, H))
    out = np.zeros((T, H, dv))
    for i in range(T):
        lo = 0 if reach is None else max(0, i - reach + 1)
        for hd in range(H):
            qr = rotate_halves(q[i, hd, d:], i, freqs, mag)
            s = np.array([q[i, hd, :d] @ kp[j, hd] + qr @ kr[j] for j in range(lo, i + 1)]) * mc["scale"]
            p = np.exp(s - s.max())
            out[i, hd] = (p / p.sum()) @ v[lo:i + 1, hd] * gate[i, hd]
    return out.reshape(T, H * dv) @ W[pre + "o"].T


def relu_gated_feed_forward(W, pre, h):
    gate = np.maximum(h @ W[pre + "gate"].T + W[pre + "gate.b"], 0.0)
    return (gate * (h @ W[pre + "up"].T + W[pre + "up.b"])) @ W[pre + "down"].T + W[pre + "down.b"]


def squared_relu_expert(W, pre, a):
    return (np.maximum(a @ W[pre + "up"].T, 0.0) ** 2) @ W[pre + "down"].T


def grouped_choice(s, correction, router, use_correction=True, use_groups=True):
    """Which of the router's outputs one token uses: scores plus the correction decide, only inside the `keep` groups of neighbours whose best such
    score is largest.  -> chosen indices (largest first)."""
    n = len(s)
    choice = s + (correction if use_correction else 0.0)
    gr = router.get("groups")
    if gr and use_groups:
        size = n // gr["count"]
        best = np.array([choice[g * size:(g + 1) * size].max() for g in range(gr["count"])])
        kept = np.argsort(-best, kind="stable")[:gr["keep"]]
        masked = np.full(n, -np.inf)
        for g in kept:
            masked[g * size:(g + 1) * size] = choice[g * size:(g + 1) * size]
        choice = masked
    return [int(e) for e in np.argsort(-choice, kind="stable")[:router["top"]]]


def routed_experts(W, pre, h, mlp, use_identity=True, use_shared=True, **choice_kw):
    """Soft-max router over experts + identity experts; the chosen ones' soft-max scores (as they are) weigh their outputs; an identity expert hands
    its input on; a shared expert runs for every token."""
    r = mlp["router"]
    E, ident = r["experts"], r.get("identity", 0)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        z = W[pre + "router"] @ h[t]
        s = np.exp(z - z.max())
        s /= s.sum()
        for e in grouped_choice(s, W[pre + "correction"] if pre + "correction" in W else 0.0, r, **choice_kw):
            if e < E:
                out[t] += s[e] * squared_relu_expert(W, f"{pre}e{e}.", h[t])
            elif use_identity:
                out[t] += s[e] * h[t]
    if mlp.get("shared") and use_shared:
        out += squared_relu_expert(W, pre + "shared.", h)
    return out


def run_pokatar(cfg, W, tokens, per_layer=None, attn_kw=None, latent_kw=None, moe_kw=None):
    """-> logits [T, vocab]; per_layer (a list) receives the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)].astype(np.float64)
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = centred_norm(x, W[p + "norm1"], eps)
        if lc["type"] == "attention":
            x = x + sink_gated_attention(W, p + "mix.", h, lc["mixer"], eps, **(attn_kw or {}))
        elif lc["type"] == "latent_attention":
            x = x + shared_key_latent_attention(W, p + "mix.", h, lc["mixer"], eps, **(latent_kw or {}))
        else:
            raise ValueError(lc["type"])
        mlp = lc.get("mlp")
        if mlp:
            h = centred_norm(x, W[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                x = x + relu_gated_feed_forward(W, p + "mlp.", h)
            else:
                x = x + routed_experts(W, p + "mlp.", h, mlp, **(moe_kw or {}))
        if per_layer is not None:
            per_layer.append(x.copy())
    return centred_norm(x, W["final.norm"], eps) @ W["embed"].T
