#include "seq_model.hpp"

#include <cmath>
#include <cstring>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace powerserve {

// ---------------------------------------------------------------- safetensors
SafeTensorsFile::SafeTensorsFile(const std::string &path) : m_path(path) {
    int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) POWERSERVE_ABORT("cannot open " + path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 8) { close(fd); POWERSERVE_ABORT(path + ": not a safetensors file"); }
    m_size = (size_t)st.st_size;
    m_map = mmap(nullptr, m_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (m_map == MAP_FAILED) { m_map = nullptr; POWERSERVE_ABORT("mmap failed: " + path); }
    uint64_t n = 0;
    memcpy(&n, m_map, 8);
    if (n > m_size - 8) POWERSERVE_ABORT(path + ": header longer than the file");
    try {
        const JsonValue j = JsonValue::parse_text(std::string((const char *)m_map + 8, (size_t)n));
        const char *base = (const char *)m_map + 8 + n;
        const size_t room = m_size - 8 - (size_t)n;
        for (const auto &[name, v] : j.obj) {
            if (name == "__metadata__") continue;
            SafeTensor t;
            t.dtype = v.at("dtype").str;
            for (const auto &s : v.at("shape").arr) t.shape.push_back((int64_t)s.num);
            const auto &off = v.at("data_offsets").arr;
            const size_t a = (size_t)off.at(0).num, b = (size_t)off.at(1).num;
            const size_t es = t.dtype == "BF16" || t.dtype == "F16" ? 2 : (t.dtype == "F32" || t.dtype == "I32" ? 4 : 0);
            if (!es) throw std::runtime_error("tensor " + name + ": unsupported dtype " + t.dtype);
            if (b < a || b > room || b - a != (size_t)t.numel() * es) throw std::runtime_error("tensor " + name + ": data_offsets do not fit its shape");
            t.data = base + a;
            t.nbytes = b - a;
            tensors[name] = t;
        }
    } catch (const std::exception &e) { POWERSERVE_ABORT(path + ": " + e.what()); }
}
SafeTensorsFile::~SafeTensorsFile() { if (m_map) munmap(m_map, m_size); }
const SafeTensor &SafeTensorsFile::at(const std::string &name) const {
    auto it = tensors.find(name);
    if (it == tensors.end()) POWERSERVE_ABORT(m_path + ": tensor " + name + " is missing");
    return it->second;
}
std::vector<float> SafeTensorsFile::f32(const std::string &name) const {
    const SafeTensor &t = at(name);
    std::vector<float> out((size_t)t.numel());
    if (t.dtype == "F32") memcpy(out.data(), t.data, t.nbytes);
    else if (t.dtype == "BF16") {
        const uint16_t *b = (const uint16_t *)t.data;
        for (size_t i = 0; i < out.size(); i++) { const uint32_t u = (uint32_t)b[i] << 16; memcpy(&out[i], &u, 4); }
    } else POWERSERVE_ABORT("tensor " + name + ": " + t.dtype + " where a float tensor is expected");
    return out;
}
std::vector<uint16_t> SafeTensorsFile::bf16_bits(const std::string &name) const {
    const SafeTensor &t = at(name);
    if (t.dtype != "BF16") POWERSERVE_ABORT("tensor " + name + " is " + t.dtype + ": the dense path takes bfloat16 matrices");
    const uint16_t *b = (const uint16_t *)t.data;
    return std::vector<uint16_t>(b, b + t.numel());
}

// ---------------------------------------------------------------- device copies
static void hip_ok(ps_hip_ctx *c, int rc, const char *what) {
    if (rc != 0) POWERSERVE_ABORT(std::string(what) + ": " + ps_hip_last_error(c));
}
const float *SeqUploader::vec(const std::vector<float> &a) {
    void *p = nullptr;
    hip_ok(ctx, ps_hip_malloc(ctx, std::max<size_t>(a.size(), 4) * 4, &p), "ps_hip_malloc");
    vecs.push_back(p);
    hip_ok(ctx, ps_hip_memcpy_h2d(ctx, p, a.data(), a.size() * 4), "ps_hip_memcpy_h2d");
    return (const float *)p;
}
const ps_dense *SeqUploader::mat(const std::vector<uint16_t> &bits, int64_t rows, int64_t cols) {
    POWERSERVE_ASSERT((int64_t)bits.size() == rows * cols);
    ps_dense *w = nullptr;
    hip_ok(ctx, ps_hip_dense_upload(ctx, bits.data(), rows, cols, as_f32 ? 1 : 0, &w), "ps_hip_dense_upload");
    mats.push_back(w);
    return w;
}
void SeqUploader::free_all() {
    for (auto *w : mats) ps_hip_dense_free(ctx, w);
    for (auto *p : vecs) ps_hip_free(ctx, p);
    mats.clear();
    vecs.clear();
}

// ---------------------------------------------------------------- Ranutar: configuration + tensors -> layer descriptors
namespace {
int64_t rows_of(const SafeTensorsFile &st, const std::string &n) { return st.at(n).shape.at(0); }
int64_t cols_of(const SafeTensorsFile &st, const std::string &n) { return st.at(n).shape.at(1); }
const ps_dense *mat1(const SafeTensorsFile &st, SeqUploader &up, const std::string &n) { return up.mat(st.bf16_bits(n), rows_of(st, n), cols_of(st, n)); }
const ps_dense *mat_rows(const SafeTensorsFile &st, SeqUploader &up, const std::vector<std::string> &names) { // the matrices stacked by rows
    std::vector<uint16_t> all;
    int64_t rows = 0;
    const int64_t cols = cols_of(st, names[0]);
    for (const auto &n : names) {
        if (cols_of(st, n) != cols) POWERSERVE_ABORT("tensor " + n + ": input size differs from " + names[0]);
        auto b = st.bf16_bits(n);
        all.insert(all.end(), b.begin(), b.end());
        rows += rows_of(st, n);
    }
    return up.mat(all, rows, cols);
}
std::vector<float> expect(const SafeTensorsFile &st, const std::string &n, int64_t r, int64_t c) {
    const auto &t = st.at(n);
    if (t.shape.size() != 2 || t.shape[0] != r || t.shape[1] != c) POWERSERVE_ABORT("tensor " + n + ": its shape is not what the configuration gives");
    return st.f32(n);
}

void ranutar(const JsonValue &cfg, const SafeTensorsFile &st, SeqUploader &up, std::vector<ps_seq_layer> &layers, ps_seq_desc &d) {
    d.width = (int32_t)cfg.at("width").num;
    d.vocab = (int32_t)cfg.at("vocab").num;
    d.canon_taps = (int32_t)cfg.at("canon").at("taps").num;
    d.norm_eps = (float)cfg.at("norm").at("eps").num;
    d.norm_offset = 1.0f;
    d.logit_scale = (float)cfg.at("logit_scale").num;
    d.embed = mat1(st, up, "embed");
    d.head = mat1(st, up, "head");
    d.final_norm = up.vec(st.f32("final.norm"));
    const auto &ls = cfg.at("layers").arr;
    for (size_t i = 0; i < ls.size(); i++) {
        const JsonValue &lc = ls[i], &mc = lc.at("mixer");
        const std::string p = "l" + std::to_string(i) + ".", m = p + "mix.", kind = lc.at("type").str;
        ps_seq_layer L{};
        L.form = PS_LAYER_SEQUENTIAL;
        L.mix_scale = 1.0f;
        L.norm1 = up.vec(st.f32(p + "norm1"));
        L.norm1b = up.vec(st.f32(p + "norm1b"));
        L.canon1 = up.vec(expect(st, p + "canon1", d.width, d.canon_taps));
        if (lc.contains("mlp") && lc.at("mlp").kind == JsonValue::OBJ) {
            const JsonValue &f = lc.at("mlp");
            if (f.at("kind").str != "dense") POWERSERVE_ABORT("layer " + std::to_string(i) + ": feed-forward kind " + f.at("kind").str + " is not known");
            L.ff_kind = PS_FF_DENSE_XIELU;
            L.ff = (int32_t)f.at("ff").num;
            L.norm2 = up.vec(st.f32(p + "norm2"));
            L.norm2b = up.vec(st.f32(p + "norm2b"));
            L.canon2 = up.vec(expect(st, p + "canon2", d.width, d.canon_taps));
            const auto act = st.f32(p + "mlp.act");
            L.ff_act_p = act.at(0);
            L.ff_act_q = act.at(1);
            L.ff_up = mat1(st, up, p + "mlp.up");
            L.ff_down = mat1(st, up, p + "mlp.down");
        }
        L.heads = (int32_t)mc.at("heads").num;
        L.dim = (int32_t)mc.at("dim").num;
        if (kind == "wkv") {
            L.kind = PS_MIX_WKV;
            L.vdim = L.dim;
            L.decay_rank = (int32_t)rows_of(st, m + "w1");
            L.in_r = mat1(st, up, m + "r"); L.in_k = mat1(st, up, m + "k"); L.in_v = mat1(st, up, m + "v"); L.in_g = mat1(st, up, m + "g");
            L.decay1 = mat1(st, up, m + "w1"); L.decay2 = mat1(st, up, m + "w2"); L.out = mat1(st, up, m + "o");
            std::vector<float> mu;
            for (const char *s : {"r", "k", "v", "g", "w"}) { auto a = st.f32(m + "mu." + s); mu.insert(mu.end(), a.begin(), a.end()); }
            L.mu = up.vec(mu);
            L.decay0 = up.vec(st.f32(m + "w0")); L.bonus = up.vec(st.f32(m + "u")); L.onorm = up.vec(st.f32(m + "norm"));
        } else if (kind == "delta") {
            L.kind = PS_MIX_DELTA;
            L.kv_heads = (int32_t)mc.at("kv_heads").num; L.vdim = (int32_t)mc.at("vdim").num; L.conv_taps = (int32_t)mc.at("conv").num;
            L.in_cat = mat_rows(st, up, {m + "q", m + "k", m + "v", m + "g", m + "b", m + "a"});
            std::vector<float> cw;
            for (const char *s : {"q", "k", "v"}) { auto a = expect(st, m + s + ".conv", rows_of(st, m + s), L.conv_taps); cw.insert(cw.end(), a.begin(), a.end()); }
            L.conv = up.vec(cw);
            L.a_log = up.vec(st.f32(m + "A_log")); L.dt_bias = up.vec(st.f32(m + "dt_bias")); L.onorm = up.vec(st.f32(m + "norm"));
            L.out = mat1(st, up, m + "o");
        } else if (kind == "latent_attention") {
            L.kind = PS_MIX_LATENT;
            L.vdim = (int32_t)mc.at("vdim").num; L.q_rank = (int32_t)mc.at("q_rank").num; L.kv_rank = (int32_t)mc.at("kv_rank").num;
            L.rot_dim = (int32_t)mc.at("rot_dim").num; L.rot_dims = (int32_t)mc.at("rot").at("dims").num; L.rot_base = (float)mc.at("rot").at("base").num;
            L.window = (int32_t)mc.at("mask").at("size").num; L.scale = (float)mc.at("scale").num;
            L.in_cat = mat_rows(st, up, {m + "dq", m + "dkv"});
            L.uq = mat1(st, up, m + "uq");
            L.ukv = mat_rows(st, up, {m + "uk", m + "uv"});
            L.out = mat1(st, up, m + "o");
            L.qnorm = up.vec(st.f32(m + "dq.norm")); L.kvnorm = up.vec(st.f32(m + "dkv.norm"));
        } else {
            POWERSERVE_ABORT("layer " + std::to_string(i) + ": mixer type " + kind + " is not known");
        }
        layers.push_back(L);
    }
}

// ---------------------------------------------------------------- Vobisun: parallel layers, two mixers side by side, a looped stretch of layers
double num_or(const JsonValue &o, const std::string &key, double fallback) {
    return o.kind == JsonValue::OBJ && o.contains(key) && o.at(key).kind == JsonValue::NUM ? o.at(key).num : fallback;
}
const JsonValue *obj_or_null(const JsonValue &o, const std::string &key) {
    return o.kind == JsonValue::OBJ && o.contains(key) && o.at(key).kind == JsonValue::OBJ ? &o.at(key) : nullptr;
}
std::vector<float> expect1(const SafeTensorsFile &st, const std::string &n, int64_t r) {
    const auto &t = st.at(n);
    if (t.shape.size() != 1 || t.shape[0] != r) POWERSERVE_ABORT("tensor " + n + ": its shape is not what the configuration gives");
    return st.f32(n);
}
// windowed attention with pooled blocks: whatever the configuration or the file does not have does not exist
void window_attention_mixer(ps_seq_layer &L, const SafeTensorsFile &st, SeqUploader &up, const std::string &m, const JsonValue &mc) {
    L.kind = PS_MIX_WINATTN;
    L.heads = (int32_t)mc.at("heads").num;
    L.dim = (int32_t)mc.at("dim").num;
    L.kv_heads = (int32_t)num_or(mc, "kv_heads", L.heads);
    L.vdim = (int32_t)num_or(mc, "vdim", L.dim);
    if (L.kv_heads <= 0 || L.heads % L.kv_heads) POWERSERVE_ABORT(m + ": heads must be a multiple of kv_heads");
    if (const JsonValue *mask = obj_or_null(mc, "mask")) { L.window = (int32_t)num_or(*mask, "size", 0); L.pool = (int32_t)num_or(*mask, "pool", 0); }
    L.rot_pairing = PS_ROT_NEIGHBOURS;
    L.rot_base = 10000.f;
    L.rot_factor = 1.f;
    if (const JsonValue *rot = obj_or_null(mc, "rot")) {
        L.rot_dims = (int32_t)num_or(*rot, "dims", 0);
        L.rot_base = (float)num_or(*rot, "base", 10000.0);
        if (const JsonValue *sc = obj_or_null(*rot, "scaling")) L.rot_factor = (float)num_or(*sc, "factor", 1.0);
    }
    L.scale = (float)num_or(mc, "scale", 1.0 / std::sqrt((double)L.dim));
    L.softcap = (float)num_or(mc, "softcap", 0.0);
    if (const JsonValue *qt = obj_or_null(mc, "q_temp")) { L.qtemp_coef = (float)num_or(*qt, "coef", 0.0); L.qtemp_every = (int32_t)num_or(*qt, "every", 0); }
    L.gated = st.contains(m + "g") ? 1 : 0;
    std::vector<std::pair<std::string, int64_t>> rows = {{m + "q", (int64_t)L.heads * L.dim}, {m + "k", (int64_t)L.kv_heads * L.dim}, {m + "v", (int64_t)L.kv_heads * L.vdim}};
    if (L.gated) rows.push_back({m + "g", L.heads});
    std::vector<std::string> names;
    std::vector<float> bias;
    bool any_bias = false;
    for (const auto &[n, r] : rows) {
        if (rows_of(st, n) != r) POWERSERVE_ABORT("tensor " + n + ": its rows are not what the configuration gives");
        names.push_back(n);
        if (st.contains(n + ".b")) { auto b = expect1(st, n + ".b", r); bias.insert(bias.end(), b.begin(), b.end()); any_bias = true; }
        else bias.insert(bias.end(), (size_t)r, 0.f);
    }
    L.in_cat = mat_rows(st, up, names);
    if (any_bias) L.in_bias = up.vec(bias);
    if (st.contains(m + "q.norm")) L.qnorm = up.vec(expect1(st, m + "q.norm", (int64_t)L.heads * L.dim));
    if (st.contains(m + "k.norm")) L.knorm = up.vec(expect1(st, m + "k.norm", (int64_t)L.kv_heads * L.dim));
    if (st.contains(m + "temp")) L.temp = up.vec(expect1(st, m + "temp", L.heads));
    if (st.contains(m + "sink")) L.sink = up.vec(expect1(st, m + "sink", L.heads));
    L.out = mat1(st, up, m + "o");
}
void gated_linear_mixer(ps_seq_layer &L, const SafeTensorsFile &st, SeqUploader &up, const std::string &m, const JsonValue &mc) {
    L.kind = PS_MIX_GLA;
    L.heads = (int32_t)mc.at("heads").num;
    L.dim = (int32_t)mc.at("dim").num;
    L.vdim = (int32_t)num_or(mc, "vdim", L.dim);
    L.tau = (float)num_or(mc, "tau", 1.0);
    L.decay_rank = (int32_t)rows_of(st, m + "a1");
    const int64_t Hd = (int64_t)L.heads * L.dim, Hv = (int64_t)L.heads * L.vdim;
    if (rows_of(st, m + "q") != Hd || rows_of(st, m + "k") != Hd || rows_of(st, m + "v") != Hv || rows_of(st, m + "g") != Hv)
        POWERSERVE_ABORT(m + ": the projections' rows are not what the configuration gives");
    L.in_cat = mat_rows(st, up, {m + "q", m + "k", m + "v", m + "g", m + "a1"});
    L.decay2 = mat1(st, up, m + "a2");
    L.decay0 = up.vec(st.contains(m + "a2.b") ? expect1(st, m + "a2.b", Hd) : std::vector<float>((size_t)Hd, 0.f));
    L.onorm = up.vec(expect1(st, m + "norm", L.vdim));
    L.out = mat1(st, up, m + "o");
}

void vobisun(const JsonValue &cfg, const SafeTensorsFile &st, SeqUploader &up, std::vector<ps_seq_layer> &layers, ps_seq_desc &d) {
    d.width = (int32_t)cfg.at("width").num;
    d.vocab = (int32_t)cfg.at("vocab").num;
    const JsonValue *canon = obj_or_null(cfg, "canon");
    d.canon_taps = canon ? (int32_t)num_or(*canon, "taps", 1) : 1;
    d.norm_eps = (float)cfg.at("norm").at("eps").num;
    d.norm_offset = 0.0f;
    d.logit_scale = 1.0f;
    const JsonValue *emb = obj_or_null(cfg, "embedding");
    d.embed_scale = emb ? (float)num_or(*emb, "scale", 1.0) : 1.0f;
    d.loop_times = 1;
    if (const JsonValue *loop = obj_or_null(cfg, "loop")) {
        d.loop_start = (int32_t)num_or(*loop, "start", 0);
        d.loop_stop = (int32_t)num_or(*loop, "stop", 0);
        d.loop_times = (int32_t)num_or(*loop, "times", 1);
    }
    d.embed = mat1(st, up, "embed");
    d.head = mat1(st, up, "head");
    d.final_norm = up.vec(expect1(st, "final.norm", d.width));
    const auto &ls = cfg.at("layers").arr;
    for (size_t i = 0; i < ls.size(); i++) {
        const JsonValue &lc = ls[i], &mc = lc.at("mixer");
        const std::string p = "l" + std::to_string(i) + ".", kind = lc.at("type").str;
        ps_seq_layer L{};
        L.form = PS_LAYER_PARALLEL;
        L.norm1 = up.vec(expect1(st, p + "norm1", d.width));
        L.canon1 = up.vec(st.contains(p + "canon1") ? expect(st, p + "canon1", d.width, d.canon_taps) : std::vector<float>((size_t)d.width * d.canon_taps, 0.f));
        if (lc.contains("mlp") && lc.at("mlp").kind == JsonValue::OBJ) {
            const JsonValue &f = lc.at("mlp");
            if (f.at("kind").str != "dense") POWERSERVE_ABORT("layer " + std::to_string(i) + ": feed-forward kind " + f.at("kind").str + " is not known");
            L.ff_kind = PS_FF_DENSE_SWIGLU;
            L.ff = (int32_t)f.at("ff").num;
            const auto g = st.bf16_bits(p + "mlp.gate"), u = st.bf16_bits(p + "mlp.up");
            const size_t W = (size_t)d.width;
            if (g.size() != (size_t)L.ff * W || u.size() != g.size()) POWERSERVE_ABORT("layer " + std::to_string(i) + ": feed-forward shapes");
            std::vector<uint16_t> both(2 * g.size()); // rows gate_0, up_0, gate_1, ...: the pair meets in one epilogue
            for (size_t r = 0; r < (size_t)L.ff; r++) {
                memcpy(&both[(2 * r) * W], &g[r * W], W * 2);
                memcpy(&both[(2 * r + 1) * W], &u[r * W], W * 2);
            }
            L.ff_up = up.mat(both, 2 * (int64_t)L.ff, d.width);
            L.ff_down = mat1(st, up, p + "mlp.down");
        }
        if (kind != "parallel") POWERSERVE_ABORT("layer " + std::to_string(i) + ": mixer type " + kind + " is not known");
        window_attention_mixer(L, st, up, p + "mix.left.", mc.at("left"));
        L.mix_scale = (float)num_or(mc, "left_scale", 1.0);
        ps_seq_layer R{};
        gated_linear_mixer(R, st, up, p + "mix.right.", mc.at("right"));
        R.mix_scale = (float)num_or(mc, "right_scale", 1.0);
        up.beside.push_back(R);
        L.beside = &up.beside.back();
        layers.push_back(L);
    }
}

// ---------------------------------------------------------------- Zusolix: two-norm parallel layers, depth average, attention / gated recurrence, dense / expert feed-forwards
void gated_recurrence_mixer(ps_seq_layer &L, const SafeTensorsFile &st, SeqUploader &up, const std::string &m, const JsonValue &mc) {
    L.kind = PS_MIX_MINGRU;
    L.heads = 1;
    L.dim = L.vdim = (int32_t)mc.at("width").num;
    std::vector<std::string> names;
    std::vector<float> bias;
    bool any_bias = false;
    for (const char *n : {"z", "x", "g"}) {
        if (rows_of(st, m + n) != L.dim) POWERSERVE_ABORT("tensor " + m + n + ": its rows are not what the configuration gives");
        names.push_back(m + n);
        if (st.contains(m + n + ".b")) { auto b = expect1(st, m + n + ".b", L.dim); bias.insert(bias.end(), b.begin(), b.end()); any_bias = true; }
        else bias.insert(bias.end(), (size_t)L.dim, 0.f);
    }
    L.in_cat = mat_rows(st, up, names);
    if (any_bias) L.in_bias = up.vec(bias);
    L.out = mat1(st, up, m + "o");
}
// rows gate_0, up_0, gate_1, ... of the feed-forward under prefix p appended to `all`: the pair meets in one epilogue
void append_gate_up(const SafeTensorsFile &st, const std::string &p, int64_t ff, int64_t W, std::vector<uint16_t> &all) {
    const auto g = st.bf16_bits(p + "gate"), u = st.bf16_bits(p + "up");
    if ((int64_t)g.size() != ff * W || u.size() != g.size() || rows_of(st, p + "down") != W || cols_of(st, p + "down") != ff) POWERSERVE_ABORT(p + ": feed-forward shapes");
    const size_t at = all.size();
    all.resize(at + 2 * g.size());
    for (int64_t r = 0; r < ff; r++) {
        memcpy(&all[at + (size_t)(2 * r) * W], &g[(size_t)r * W], (size_t)W * 2);
        memcpy(&all[at + (size_t)(2 * r + 1) * W], &u[(size_t)r * W], (size_t)W * 2);
    }
}
void gated_feed_forward(ps_seq_layer &L, const SafeTensorsFile &st, SeqUploader &up, const std::string &p, const JsonValue &f, int64_t W) {
    const std::string kind = f.at("kind").str;
    if (kind == "dense") {
        L.ff_kind = PS_FF_DENSE_SWIGLU;
        L.ff = (int32_t)f.at("ff").num;
        std::vector<uint16_t> both;
        append_gate_up(st, p, L.ff, W, both);
        L.ff_up = up.mat(both, 2 * (int64_t)L.ff, W);
        L.ff_down = mat1(st, up, p + "down");
    } else if (kind == "moe") {
        L.ff_kind = PS_FF_MOE_SWIGLU;
        L.ff = (int32_t)f.at("expert").at("ff").num;
        L.experts = (int32_t)f.at("router").at("experts").num;
        L.top = (int32_t)f.at("router").at("top").num;
        if (L.experts <= 0 || L.top <= 0 || L.top > L.experts) POWERSERVE_ABORT(p + ": top / experts");
        std::vector<uint16_t> ups, downs;
        for (int e = 0; e < L.experts; e++) {
            const std::string pe = p + "e" + std::to_string(e) + ".";
            append_gate_up(st, pe, L.ff, W, ups);
            const auto dn = st.bf16_bits(pe + "down");
            downs.insert(downs.end(), dn.begin(), dn.end());
        }
        L.ff_up = up.mat(ups, (int64_t)L.experts * 2 * L.ff, W);
        L.ff_down = up.mat(downs, (int64_t)L.experts * W, L.ff);
        L.router = up.vec(expect(st, p + "router", L.experts, W));
        if (const JsonValue *sh = obj_or_null(f, "shared")) {
            L.shared_ff = (int32_t)sh->at("ff").num;
            std::vector<uint16_t> both;
            append_gate_up(st, p + "shared.", L.shared_ff, W, both);
            L.shared_up = up.mat(both, 2 * (int64_t)L.shared_ff, W);
            L.shared_down = mat1(st, up, p + "shared.down");
            if (st.contains(p + "shared.sg")) L.shared_gate = up.vec(expect(st, p + "shared.sg", 1, W));
        }
    } else {
        POWERSERVE_ABORT(p + ": feed-forward kind " + kind + " is not known");
    }
}
void zusolix(const JsonValue &cfg, const SafeTensorsFile &st, SeqUploader &up, std::vector<ps_seq_layer> &layers, ps_seq_desc &d) {
    d.width = (int32_t)cfg.at("width").num;
    d.vocab = (int32_t)cfg.at("vocab").num;
    d.canon_taps = 1;
    d.norm_eps = (float)cfg.at("norm").at("eps").num;
    d.norm_groups = (int32_t)num_or(cfg.at("norm"), "groups", 1);
    d.norm_offset = 0.0f;
    d.logit_scale = 1.0f;
    d.loop_times = 1;
    const JsonValue *emb = obj_or_null(cfg, "embedding");
    d.embed_scale = emb ? (float)num_or(*emb, "scale", 1.0) : 1.0f;
    const float res = (float)num_or(cfg, "residual_mult", 1.0);
    d.embed = mat1(st, up, "embed");
    d.head = mat1(st, up, "head");
    d.final_norm = up.vec(expect1(st, "final.norm", d.width));
    const auto &ls = cfg.at("layers").arr;
    for (size_t i = 0; i < ls.size(); i++) {
        const JsonValue &lc = ls[i], &mc = lc.at("mixer");
        const std::string p = "l" + std::to_string(i) + ".", kind = lc.at("type").str;
        ps_seq_layer L{};
        L.form = PS_LAYER_PARALLEL;
        L.mix_scale = 1.f;
        L.res_scale = res;
        L.norm1 = up.vec(expect1(st, p + "norm1", d.width));
        if (kind == "attention") window_attention_mixer(L, st, up, p + "mix.", mc);
        else if (kind == "mingru") gated_recurrence_mixer(L, st, up, p + "mix.", mc);
        else POWERSERVE_ABORT("layer " + std::to_string(i) + ": mixer type " + kind + " is not known");
        if (lc.contains("mlp") && lc.at("mlp").kind == JsonValue::OBJ) {
            L.norm2 = up.vec(expect1(st, p + "norm2", d.width));
            gated_feed_forward(L, st, up, p + "mlp.", lc.at("mlp"), d.width);
        }
        if (st.contains(p + "dwa")) L.depth_mix = up.vec(expect1(st, p + "dwa", (int64_t)i + 2));
        layers.push_back(L);
    }
}
// ---------------------------------------------------------------- Pokatar: pre-norm layers with layer norms, sink attention / shared-key latent attention, relu-gated dense / squared-relu expert feed-forwards
void check_rows(const SafeTensorsFile &st, const std::string &n, int64_t rows) {
    if (rows_of(st, n) != rows) POWERSERVE_ABORT("tensor " + n + ": its rows are not what the configuration gives");
}
void sink_attention_mixer(ps_seq_layer &L, const SafeTensorsFile &st, SeqUploader &up, const std::string &m, const JsonValue &mc) {
    L.kind = PS_MIX_WINATTN;
    L.heads = (int32_t)mc.at("heads").num;
    L.dim = (int32_t)mc.at("dim").num;
    L.kv_heads = (int32_t)num_or(mc, "kv_heads", L.heads);
    L.vdim = (int32_t)num_or(mc, "vdim", L.dim);
    if (L.kv_heads <= 0 || L.heads % L.kv_heads) POWERSERVE_ABORT(m + ": heads over key / value heads");
    if (const JsonValue *mask = obj_or_null(mc, "mask")) L.window = (int32_t)num_or(*mask, "size", 0);
    L.rot_pairing = PS_ROT_HALVES;
    L.rot_base = 10000.f;
    L.scale = (float)num_or(mc, "scale", 1.0 / std::sqrt((double)L.dim));
    L.head_norm = 1; // q / k norms per head, one weight vector of `dim`
    L.v_unit = 1;    // every head's value a unit-rms vector
    std::vector<std::string> names = {m + "q", m + "k", m + "v"};
    check_rows(st, m + "q", (int64_t)L.heads * L.dim);
    check_rows(st, m + "k", (int64_t)L.kv_heads * L.dim);
    check_rows(st, m + "v", (int64_t)L.kv_heads * L.vdim);
    if (st.contains(m + "g")) {
        check_rows(st, m + "g", (int64_t)L.heads * L.vdim);
        L.gated = 2; // a gate row per output element
        names.push_back(m + "g");
    }
    L.in_cat = mat_rows(st, up, names);
    if (st.contains(m + "q.norm")) L.qnorm = up.vec(expect1(st, m + "q.norm", L.dim));
    if (st.contains(m + "k.norm")) L.knorm = up.vec(expect1(st, m + "k.norm", L.dim));
    L.sink = up.vec(std::vector<float>((size_t)L.heads, 0.f)); // exp(0) = 1 joins every head's denominator
    L.out = mat1(st, up, m + "o");
}
void shared_key_latent_mixer(ps_seq_layer &L, const SafeTensorsFile &st, SeqUploader &up, const std::string &m, const JsonValue &mc) {
    L.kind = PS_MIX_LATENT;
    L.q_rank = 0; // the queries come straight from the input
    L.heads = (int32_t)mc.at("heads").num;
    L.dim = (int32_t)mc.at("dim").num;
    L.vdim = (int32_t)num_or(mc, "vdim", L.dim);
    L.kv_rank = (int32_t)mc.at("kv_rank").num;
    L.rot_dim = (int32_t)mc.at("rot_dim").num;
    L.rot_base = 10000.f;
    if (const JsonValue *rot = obj_or_null(mc, "rot")) {
        L.rot_dims = (int32_t)num_or(*rot, "dims", 0);
        L.rot_base = (float)num_or(*rot, "base", 10000.0);
        if (const JsonValue *sc = obj_or_null(*rot, "scaling")) {
            L.yarn_factor = (float)sc->at("factor").num;
            L.yarn_fast = (float)sc->at("fast").num;
            L.yarn_slow = (float)sc->at("slow").num;
            L.yarn_original = (int32_t)sc->at("original").num;
        }
    }
    if (const JsonValue *mask = obj_or_null(mc, "mask")) L.window = (int32_t)num_or(*mask, "size", 0);
    L.scale = (float)mc.at("scale").num;
    std::vector<std::string> names = {m + "q", m + "dkv"};
    check_rows(st, m + "q", (int64_t)L.heads * (L.dim + L.rot_dim));
    check_rows(st, m + "dkv", (int64_t)L.kv_rank + L.rot_dim);
    check_rows(st, m + "uk", (int64_t)L.heads * L.dim);
    check_rows(st, m + "uv", (int64_t)L.heads * L.vdim);
    if (st.contains(m + "g")) {
        check_rows(st, m + "g", L.heads);
        L.gated = 1;
        names.push_back(m + "g");
    }
    L.in_cat = mat_rows(st, up, names);
    L.ukv = mat_rows(st, up, {m + "uk", m + "uv"});
    L.kvnorm = up.vec(expect1(st, m + "dkv.norm", L.kv_rank));
    L.out = mat1(st, up, m + "o");
}
void relu_feed_forward(ps_seq_layer &L, const SafeTensorsFile &st, SeqUploader &up, const std::string &p, const JsonValue &f, int64_t W) {
    const std::string kind = f.at("kind").str;
    if (kind == "dense") {
        L.ff_kind = PS_FF_DENSE_RELU_GLU;
        L.ff = (int32_t)f.at("ff").num;
        std::vector<uint16_t> both;
        append_gate_up(st, p, L.ff, W, both);
        L.ff_up = up.mat(both, 2 * (int64_t)L.ff, W);
        L.ff_down = mat1(st, up, p + "down");
        if (st.contains(p + "gate.b") || st.contains(p + "up.b")) {
            const std::vector<float> zero((size_t)L.ff, 0.f);
            const auto g = st.contains(p + "gate.b") ? expect1(st, p + "gate.b", L.ff) : zero, u = st.contains(p + "up.b") ? expect1(st, p + "up.b", L.ff) : zero;
            std::vector<float> b(2 * (size_t)L.ff);
            for (int64_t r = 0; r < L.ff; r++) { b[2 * r] = g[r]; b[2 * r + 1] = u[r]; }
            L.ff_up_bias = up.vec(b);
        }
        if (st.contains(p + "down.b")) L.ff_down_bias = up.vec(expect1(st, p + "down.b", W));
    } else if (kind == "moe") {
        const JsonValue &r = f.at("router");
        L.ff_kind = PS_FF_MOE_RELU2;
        L.ff = (int32_t)f.at("expert").at("ff").num;
        L.experts = (int32_t)r.at("experts").num;
        L.top = (int32_t)r.at("top").num;
        L.moe_identity = (int32_t)num_or(r, "identity", 0);
        L.moe_softmax = 1;
        L.moe_weight_output = 1;
        if (const JsonValue *gr = obj_or_null(r, "groups")) { L.moe_groups = (int32_t)num_or(*gr, "count", 0); L.moe_keep = (int32_t)num_or(*gr, "keep", 0); }
        const int rows = L.experts + L.moe_identity;
        if (L.experts <= 0 || L.top <= 0 || L.top > rows) POWERSERVE_ABORT(p + ": top / experts");
        std::vector<std::string> ups, downs;
        for (int e = 0; e < L.experts; e++) {
            const std::string pe = p + "e" + std::to_string(e) + ".";
            if (rows_of(st, pe + "up") != L.ff || cols_of(st, pe + "up") != W || rows_of(st, pe + "down") != W || cols_of(st, pe + "down") != L.ff) POWERSERVE_ABORT(pe + ": expert shapes");
            ups.push_back(pe + "up");
            downs.push_back(pe + "down");
        }
        L.ff_up = mat_rows(st, up, ups);
        L.ff_down = mat_rows(st, up, downs);
        L.router = up.vec(expect(st, p + "router", rows, W));
        if (st.contains(p + "correction")) L.moe_correction = up.vec(expect1(st, p + "correction", rows));
        if (const JsonValue *sh = obj_or_null(f, "shared")) {
            L.shared_ff = (int32_t)sh->at("ff").num;
            if (rows_of(st, p + "shared.up") != L.shared_ff || rows_of(st, p + "shared.down") != W) POWERSERVE_ABORT(p + "shared: expert shapes");
            L.shared_up = mat1(st, up, p + "shared.up");
            L.shared_down = mat1(st, up, p + "shared.down");
        }
    } else {
        POWERSERVE_ABORT(p + ": feed-forward kind " + kind + " is not known");
    }
}
void pokatar(const JsonValue &cfg, const SafeTensorsFile &st, SeqUploader &up, std::vector<ps_seq_layer> &layers, ps_seq_desc &d) {
    d.width = (int32_t)cfg.at("width").num;
    d.vocab = (int32_t)cfg.at("vocab").num;
    d.canon_taps = 1;
    d.norm_eps = (float)cfg.at("norm").at("eps").num;
    d.norm_offset = 0.0f;
    d.norm_center = 1;
    d.logit_scale = 1.0f;
    d.loop_times = 1;
    d.embed = mat1(st, up, "embed");
    d.head = d.embed; // the logits are taken against the embedding table itself
    d.final_norm = up.vec(expect1(st, "final.norm", d.width));
    const auto &ls = cfg.at("layers").arr;
    for (size_t i = 0; i < ls.size(); i++) {
        const JsonValue &lc = ls[i], &mc = lc.at("mixer");
        const std::string p = "l" + std::to_string(i) + ".", kind = lc.at("type").str;
        ps_seq_layer L{};
        L.form = PS_LAYER_PRENORM;
        L.mix_scale = 1.f;
        L.norm1 = up.vec(expect1(st, p + "norm1", d.width));
        if (kind == "attention") sink_attention_mixer(L, st, up, p + "mix.", mc);
        else if (kind == "latent_attention") shared_key_latent_mixer(L, st, up, p + "mix.", mc);
        else POWERSERVE_ABORT("layer " + std::to_string(i) + ": mixer type " + kind + " is not known");
        if (lc.contains("mlp") && lc.at("mlp").kind == JsonValue::OBJ) {
            L.norm2 = up.vec(expect1(st, p + "norm2", d.width));
            relu_feed_forward(L, st, up, p + "mlp.", lc.at("mlp"), d.width);
        }
        layers.push_back(L);
    }
}
} // namespace

const std::map<std::string, SeqArchitecture> &seq_architectures() {
    static const std::map<std::string, SeqArchitecture> reg = {{"Ranutar", ranutar}, {"Vobisun", vobisun}, {"Zusolix", zusolix}, {"Pokatar", pokatar}};
    return reg;
}
bool is_seq_model_dir(const std::string &dir) {
    struct stat a, b;
    return stat((dir + "/config.json").c_str(), &a) == 0 && stat((dir + "/model.safetensors").c_str(), &b) == 0;
}

// ---------------------------------------------------------------- the model
SeqModel::SeqModel(const std::string &model_dir, const std::string &dtype, int device, size_t max_batch, int n_slots, int max_context) {
    if (dtype != "bfloat16" && dtype != "float32") POWERSERVE_ABORT("dtype " + dtype + ": bfloat16 or float32");
    JsonValue cfg;
    try { cfg = JsonValue::parse_file(model_dir + "/config.json"); } catch (const std::exception &e) { POWERSERVE_ABORT(std::string("config.json: ") + e.what()); }
    if (!cfg.contains("architecture") || !seq_architectures().count(cfg.at("architecture").str))
        POWERSERVE_ABORT("unknown model type: " + (cfg.contains("architecture") ? cfg.at("architecture").str : std::string("(config.json names no architecture)")));
    arch = cfg.at("architecture").str;
    SafeTensorsFile st(model_dir + "/model.safetensors");
    if (ps_hip_create(device, &m_ctx) != 0) POWERSERVE_ABORT("no HIP device: the MI355X backend cannot run (there is no CPU fallback)");
    m_up = SeqUploader{m_ctx, dtype == "float32", {}, {}, {}};
    std::vector<ps_seq_layer> layers;
    ps_seq_desc d{};
    try {
        seq_architectures().at(arch)(cfg, st, m_up, layers, d);
    } catch (const std::out_of_range &) { POWERSERVE_ABORT("config.json: a tensor has fewer dimensions than its use needs"); }
    d.n_layers = (int32_t)layers.size();
    d.max_batch = (int32_t)max_batch;
    d.n_slots = n_slots;
    d.compute = dtype == "float32";
    d.max_context = max_context;
    d.layers = layers.data();
    hip_ok(m_ctx, ps_hip_seq_create(m_ctx, &d, &m_h), "ps_hip_seq_create");
    vocab = (uint32_t)d.vocab; width = (uint32_t)d.width; n_layers = (uint32_t)d.n_layers;
}
SeqModel::~SeqModel() {
    if (m_h) ps_hip_seq_destroy(m_h);
    if (m_ctx) { m_up.free_all(); ps_hip_destroy(m_ctx); }
}
int SeqModel::acquire() { int s = -1; hip_ok(m_ctx, ps_hip_seq_acquire(m_h, &s), "ps_hip_seq_acquire"); return s; }
void SeqModel::release(int slot) { hip_ok(m_ctx, ps_hip_seq_release(m_h, slot), "ps_hip_seq_release"); }
int64_t SeqModel::position(int slot) const { return ps_hip_seq_position(m_h, slot); }
std::vector<float> SeqModel::forward(int slot, const std::vector<Token> &tokens, const std::vector<int> &want) {
    std::vector<float> out(want.size() * (size_t)vocab);
    hip_ok(m_ctx, ps_hip_seq_forward(m_h, slot, tokens.data(), (int)tokens.size(), want.empty() ? nullptr : want.data(), (int)want.size(),
                                     want.empty() ? nullptr : out.data(), nullptr), "ps_hip_seq_forward");
    return out;
}
std::vector<Token> SeqModel::generate(const std::vector<Token> &prompt, int steps) {
    POWERSERVE_ASSERT(!prompt.empty());
    const int slot = acquire();
    std::vector<Token> out((size_t)std::max(steps, 0));
    try {
        if (prompt.size() > 1) forward(slot, std::vector<Token>(prompt.begin(), prompt.end() - 1), {});
        hip_ok(m_ctx, ps_hip_seq_decode_greedy(m_h, slot, prompt.back(), steps, out.data()), "ps_hip_seq_decode_greedy");
    } catch (...) { release(slot); throw; }
    release(slot);
    return out;
}
std::vector<Token> SeqModel::generate(const std::vector<Token> &prompt, int steps, SamplerChain &sampler) {
    POWERSERVE_ASSERT(!prompt.empty());
    const int slot = acquire();
    std::vector<Token> out;
    try {
        if (prompt.size() > 1) forward(slot, std::vector<Token>(prompt.begin(), prompt.end() - 1), {});
        Token tok = prompt.back();
        for (int i = 0; i < steps; i++) {
            auto lg = forward(slot, {tok}, {0});
            tok = sampler.sample(std::span<const float>(lg.data(), lg.size()));
            out.push_back(tok);
        }
    } catch (...) { release(slot); throw; }
    release(slot);
    return out;
}
auto load_seq_model(const std::string &model_dir, const std::string &dtype, int device, size_t max_batch, int n_slots, int max_context) -> std::shared_ptr<SeqModel> {
    if (!is_seq_model_dir(model_dir)) POWERSERVE_ABORT(model_dir + ": config.json + model.safetensors expected");
    return std::make_shared<SeqModel>(model_dir, dtype, device, max_batch, n_slots, max_context);
}

} // namespace powerserve

// ---------------------------------------------------------------- C driver API
using namespace powerserve;
extern "C" {
void psh_set_error(const char *msg);
void *psh_sampler_create(const void *cfg);
void psh_sampler_free(void *s);
int psh_is_seq_model_dir(const char *dir) { return is_seq_model_dir(dir) ? 1 : 0; }
void *psh_seq_load(const char *model_dir, const char *dtype, int device, int max_batch, int n_slots, int max_context) {
    try { return new std::shared_ptr<SeqModel>(load_seq_model(model_dir, dtype, device, (size_t)max_batch, n_slots, max_context)); } catch (const std::exception &e) { psh_set_error(e.what()); return nullptr; }
}
void psh_seq_free(void *h) { delete (std::shared_ptr<SeqModel> *)h; }
uint32_t psh_seq_vocab(void *h) { return (*(std::shared_ptr<SeqModel> *)h)->vocab; }
int psh_seq_generate(void *h, const int32_t *prompt, int n_prompt, int steps, int32_t *out) {
    try {
        auto r = (*(std::shared_ptr<SeqModel> *)h)->generate(std::vector<Token>(prompt, prompt + n_prompt), steps);
        memcpy(out, r.data(), r.size() * 4);
        return 0;
    } catch (const std::exception &e) { psh_set_error(e.what()); return 1; }
}
int psh_seq_generate_sampled(void *h, const int32_t *prompt, int n_prompt, int steps, const void *sampler_cfg, int32_t *out) {
    void *s = psh_sampler_create(sampler_cfg);
    if (!s) return 1;
    int rc = 0;
    try {
        auto r = (*(std::shared_ptr<SeqModel> *)h)->generate(std::vector<Token>(prompt, prompt + n_prompt), steps, *(SamplerChain *)s);
        memcpy(out, r.data(), r.size() * 4);
    } catch (const std::exception &e) { psh_set_error(e.what()); rc = 1; }
    psh_sampler_free(s);
    return rc;
}
int psh_seq_forward(void *h, int slot, const int32_t *tokens, int n, const int32_t *want, int n_want, float *logits_out) {
    try {
        auto &m = *(std::shared_ptr<SeqModel> *)h;
        auto r = m->forward(slot, std::vector<Token>(tokens, tokens + n), std::vector<int>(want, want + n_want));
        if (n_want) memcpy(logits_out, r.data(), r.size() * 4);
        return 0;
    } catch (const std::exception &e) { psh_set_error(e.what()); return 1; }
}
int psh_seq_acquire(void *h) { try { return (*(std::shared_ptr<SeqModel> *)h)->acquire(); } catch (const std::exception &e) { psh_set_error(e.what()); return -1; } }
int psh_seq_release(void *h, int slot) { try { (*(std::shared_ptr<SeqModel> *)h)->release(slot); return 0; } catch (const std::exception &e) { psh_set_error(e.what()); return 1; } }
}
