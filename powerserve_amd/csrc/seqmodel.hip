// Layer-list models (include/ps_hip.h, "layer-list models"): the model object, its pool of sequence states and the step function.
//
// A step takes the next n tokens of ONE sequence from the state earlier steps left in its slot.  The residual stream is fp32; a
// layer is either SEQUENTIAL,  x += norm_b(mixer(conv(norm(x))))  then, where it has a feed-forward,  x += norm_b(ff(conv(norm(x)))),
// or PARALLEL,  h = norm(x); x += mixer(conv(h)) + ff(h).  A layer's mixer may have a second one beside it that reads the same input
// (their outputs are added, each times its scale), and a stretch of layers may run several times in a row with the same weights: the
// unit that owns state is the layer RUN.  What a sequence carries: per run the tails of the input convolutions, and per mixer kind a
// token-shift row + the wkv state, the short convolutions' tail + the delta-rule state, the gated-linear-attention state, the element-wise
// recurrence's state, the ring of latents, or the ring of keys and values + the block means -- one fp32 block per slot, rings and means last,
// the rest zeroed when the slot is handed out.
// A parallel layer may go without the input filter, take its two sublayers' inputs from two norms of the same vector, scale the sublayers' sum, and
// hand on a weighted average of ALL earlier layers' results instead of its own (depth_mix): the results X_0 .. X_runs of a portion then live side by
// side (`hist`), a layer's sublayers add into its own X, and the average, the next layer's norms and their group statistics are one launch (psk_front).
// The feed-forward may be a mixture of experts: the router (fp32) picks per token, the experts' products are grouped launches of the dense kernels.
// A PRE-NORM layer is  x += mixer(norm1(x)); x += ff(norm2(x)):  no filter, nothing normed behind a sublayer, the second norm reads what the mixer left; its norms
// (and the final one) may be layer norms (norm_center).
#include "ps_seq.h"

#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace {
struct LayerPlan { // one layer RUN (and, as `side`, the second mixer of one)
    ps_seq_layer d;
    int layer = 0; // index into the descriptor's layers (runs of a looped layer share it, and its weights)
    int64_t off_canon1 = 0, off_canon2 = 0, off_shift = 0, off_conv = 0, off_S = 0, off_ring = 0, off_pool = 0;
    int cap = 0;          // latent / windowed attention: ring rows
    int64_t pool_rows = 0; // windowed attention: block means held
    float *freq = nullptr; // rot_dims / 2 angular frequencies (shared by the runs of a layer)
    float act_p = 0.f, act_q = 0.f;
    float rot_mag = 1.f; // latent: the factor on cos and sin that comes with frequency scaling by wavelength
    int64_t ncat = 0, cqkv = 0;
    // two mixers side by side whose first step is one stacked projection of the same input: the rows of both are ONE matrix (joint, with joint_bias), its
    // result has in_ld columns and this mixer's part starts at column in_off (in_ld == 0: the mixer multiplies by its own in_cat)
    const ps_dense *joint = nullptr;
    const float *joint_bias = nullptr;
    int64_t in_ld = 0, in_off = 0;
    std::shared_ptr<LayerPlan> side;
};
} // namespace

struct ps_hip_seq {
    ps_hip_ctx *ctx = nullptr;
    ps_seq_desc d;
    std::vector<LayerPlan> L; // layer runs in execution order
    int64_t max_context = 0;
    bool needs_context = false; // some mixer's memory grows with the sequence: a sequence may hold at most max_context tokens
    float embed_scale = 1.f;
    int64_t state_floats = 0, zero_floats = 0;
    std::vector<float *> slot_state;
    std::vector<int64_t> slot_pos; // -1: free
    ps_seq_step *step = nullptr;   // device
    float *x = nullptr, *hn = nullptr, *h = nullptr, *y = nullptr, *t1 = nullptr, *t2 = nullptr, *t3 = nullptr, *t4 = nullptr, *kvx = nullptr, *xn = nullptr,
          *logits = nullptr;
    int32_t *tokens = nullptr, *want = nullptr, *amax = nullptr, *ids = nullptr;
    float *hist = nullptr;        // depth_mix: [runs + 1][max_batch][width], X_0 = the embedding, run i writes X_(i+1)
    int groups = 1;               // parts of every RMS norm over the width
    int32_t *moe_sel = nullptr, *moe_seg = nullptr, *moe_list = nullptr; // mixture of experts: expert per slot, the slots sorted by expert
    float *moe_wgt = nullptr, *moe_sg = nullptr, *moe_y = nullptr;       // weight per slot, the shared expert's gate per token, per-slot results (top > 1)
    float *win_scratch = nullptr; // the windowed attention's single-token partials
    float *abs_scratch = nullptr; // the absorbed single-token attention's folded queries, attended latents and per-tile partials
    void *pack = nullptr; // the wide mat-mul's bfloat16 operand copy
    size_t pack_bytes = 0;
    int ids_cap = 0;
    int64_t n_t2q = 0; // t2: [max_batch][q_rank max] then the queries
    float *dbg_layers = nullptr;
    int mode = 0;
    std::map<int, hipGraphExec_t> graphs; // single-token greedy step, per slot
    uint64_t weight_bytes = 0;
    std::vector<void *> owned;
    std::vector<ps_dense *> joints;
};

__global__ void seq_set_step_kernel(ps_seq_step *s, long long pos0, int n, int slot, float *state, int token0) {
    s->pos0 = pos0; s->n = n; s->slot = slot; s->state = state; s->token0 = token0; s->_pad = 0;
}
// behind a greedy single-token step: the arg-max becomes the next token, the position moves on, the id is kept at ids[_pad++]
__global__ void seq_advance_kernel(ps_seq_step *s, const int32_t *amax, int32_t *ids) {
    const int32_t id = amax[0];
    ids[s->_pad] = id;
    s->_pad += 1;
    s->token0 = id;
    s->pos0 += 1;
}

static int seq_fail(ps_hip_ctx *c, const std::string &msg) { c->err = msg; return 2; }

static uint64_t dense_bytes(const ps_dense *w) { return w ? (uint64_t)w->N * w->K * (w->dtype == PS_BF16 ? 2 : 4) : 0; }

extern "C" {

int ps_hip_seq_create(ps_hip_ctx *c, const ps_seq_desc *desc, ps_hip_seq **out) {
    *out = nullptr;
    if (!desc || desc->n_layers <= 0 || desc->width <= 0 || desc->vocab <= 0 || desc->max_batch <= 0 || desc->n_slots <= 0 || desc->canon_taps < 1)
        return seq_fail(c, "seq_create: bad descriptor");
    if (!desc->embed || !desc->head || !desc->final_norm) return seq_fail(c, "seq_create: embed / head / final_norm missing");
    if (desc->embed->K != desc->width || desc->head->K != desc->width || desc->head->N != desc->vocab) return seq_fail(c, "seq_create: embed / head shape");
    PS_CHECK(c, hipSetDevice(c->device));
    auto m = new ps_hip_seq();
    m->ctx = c;
    m->d = *desc;
    const int64_t W = desc->width, B = desc->max_batch;
    int64_t off = 0, n1 = 0, n2 = 0, n3 = 0, n4 = 0, nkv = 0, nq = 0;
    auto fail = [&](const std::string &msg) { ps_hip_seq_destroy(m); return seq_fail(c, "seq_create: " + msg); };
    auto shape = [](const ps_dense *w, int64_t N, int64_t K) { return w && w->N == N && w->K == K; };
    m->max_context = desc->max_context > 0 ? desc->max_context : 65536;
    m->embed_scale = desc->embed_scale != 0.f ? desc->embed_scale : 1.f;
    m->groups = desc->norm_groups > 0 ? desc->norm_groups : 1;
    if (W % m->groups) return fail("norm_groups does not divide the width");
    int64_t moe_slots = 0, moe_experts = 0, moe_top = 1;
    bool depth = false;
    std::vector<int> order; // layer index of every run
    {
        const bool loop = desc->loop_times > 1;
        if (loop && (desc->loop_start < 0 || desc->loop_stop > desc->n_layers || desc->loop_start >= desc->loop_stop)) return fail("loop_start / loop_stop");
        for (int i = 0; i < desc->n_layers; i++) {
            if (loop && i == desc->loop_start) {
                for (int r = 0; r < desc->loop_times; r++)
                    for (int j = desc->loop_start; j < desc->loop_stop; j++) order.push_back(j);
                i = desc->loop_stop - 1;
            } else {
                order.push_back(i);
            }
        }
    }
    m->weight_bytes = dense_bytes(desc->head);
    // a mixer's sizes, its tensors' shapes, its zeroed state and its scratch needs (rings and block means are placed afterwards)
    auto plan_mixer = [&](LayerPlan &P, const std::string &at) -> std::string {
        const ps_seq_layer &l = P.d;
        const int64_t H = l.heads, d = l.dim, dv = l.vdim;
        if (H <= 0 || d <= 0 || !l.out) return at + "heads / dim / out";
        if (l.kind == PS_MIX_WKV) {
            const int64_t Hd = H * d;
            if (d > 256) return at + "wkv: dim > 256 is not supported by the scan kernel";
            if (!shape(l.in_r, Hd, W) || !shape(l.in_k, Hd, W) || !shape(l.in_v, Hd, W) || !shape(l.in_g, Hd, W) || !shape(l.decay1, l.decay_rank, W) ||
                !shape(l.decay2, Hd, l.decay_rank) || !shape(l.out, W, Hd) || !l.mu || !l.decay0 || !l.bonus || !l.onorm)
                return at + "wkv tensors";
            P.off_shift = off; off += W;
            P.off_S = off; off += Hd * d;
            n1 = std::max(n1, 5 * Hd);
            n2 = std::max<int64_t>(n2, l.decay_rank);
            n3 = std::max(n3, Hd);
            m->weight_bytes += dense_bytes(l.in_r) * 4 + dense_bytes(l.decay1) + dense_bytes(l.decay2) + dense_bytes(l.out);
        } else if (l.kind == PS_MIX_DELTA) {
            if (d > 256) return at + "delta: dim > 256 is not supported by the scan kernel";
            if (l.kv_heads <= 0 || H % l.kv_heads || dv <= 0 || l.conv_taps < 1) return at + "delta sizes";
            P.cqkv = 2 * (int64_t)l.kv_heads * d + H * dv;
            P.ncat = P.cqkv + H * dv + 2 * H;
            if (!shape(l.in_cat, P.ncat, W) || !shape(l.out, W, H * dv) || !l.conv || !l.a_log || !l.dt_bias || !l.onorm) return at + "delta tensors";
            P.off_conv = off; off += (int64_t)(l.conv_taps - 1) * P.cqkv;
            P.off_S = off; off += H * d * dv;
            n1 = std::max(n1, P.ncat);
            n2 = std::max(n2, P.cqkv);
            n3 = std::max(n3, H * dv);
            m->weight_bytes += dense_bytes(l.in_cat) + dense_bytes(l.out);
        } else if (l.kind == PS_MIX_LATENT) {
            if (dv <= 0 || dv > 256 || l.q_rank < 0 || l.kv_rank <= 0 || l.rot_dim < 0 || l.rot_dims < 0 || l.rot_dims > l.rot_dim || (l.rot_dims & 1) || l.window < 0)
                return at + "latent sizes (vdim <= 256, even rot_dims <= rot_dim)";
            // q_rank 0: the queries come straight from the input, in_cat = q | dkv | gate
            P.ncat = (l.q_rank > 0 ? (int64_t)l.q_rank : H * (d + l.rot_dim)) + l.kv_rank + l.rot_dim + (l.gated ? H : 0);
            if (!shape(l.in_cat, P.ncat, W) || (l.q_rank > 0 && !shape(l.uq, H * (d + l.rot_dim), l.q_rank)) || !shape(l.ukv, H * d + H * dv, l.kv_rank) ||
                !shape(l.out, W, H * dv) || (l.q_rank > 0 && !l.qnorm) || !l.kvnorm || (l.gated && l.gated != 1))
                return at + "latent tensors";
            if (l.yarn_factor != 0.f && (!(l.yarn_factor > 0.f) || l.yarn_original <= 0 || !(l.yarn_fast > 0.f) || !(l.yarn_slow > 0.f) || !(l.rot_base > 1.f)))
                return at + "latent: frequency scaling constants";
            if (l.window <= 0 || l.window > m->max_context) m->needs_context = true; // (window 0: everything before the token)
            const int64_t window = l.window > 0 ? std::min<int64_t>(l.window, m->max_context) : m->max_context;
            P.d.window = (int32_t)window;
            P.cap = (int)(window - 1 + B);
            P.rot_mag = l.yarn_factor > 0.f ? (float)(0.1 * log((double)l.yarn_factor) + 1.0) : 1.f;
            n1 = std::max(n1, P.ncat);
            if (l.q_rank > 0) {
                nq = std::max(nq, H * (d + l.rot_dim));
                m->n_t2q = std::max<int64_t>(m->n_t2q, l.q_rank);
            }
            n3 = std::max(n3, H * dv);
            nkv = std::max(nkv, (int64_t)(window - 1 + B) * (H * d + H * dv));
            m->weight_bytes += dense_bytes(l.in_cat) + dense_bytes(l.uq) + dense_bytes(l.ukv) + dense_bytes(l.out);
        } else if (l.kind == PS_MIX_WINATTN) {
            const int64_t G = l.kv_heads;
            if (G <= 0 || H % G || dv <= 0 || dv > 256 || l.rot_dims < 0 || l.rot_dims > d || (l.rot_dims & 1) || l.window < 0 || l.pool < 0)
                return at + "windowed attention sizes (heads a multiple of kv_heads, vdim <= 256, even rot_dims <= dim)";
            if (l.rot_pairing != PS_ROT_HALVES && l.rot_pairing != PS_ROT_NEIGHBOURS) return at + "rot_pairing";
            if (l.gated < 0 || l.gated > 2) return at + "gated: 0 (none), 1 (a row per head) or 2 (a row per output element)";
            P.ncat = H * d + G * d + G * dv + (l.gated == 2 ? H * dv : l.gated ? H : 0);
            if (!shape(l.in_cat, P.ncat, W) || !shape(l.out, W, H * dv)) return at + "windowed attention tensors";
            if (l.pool > 0 || l.window <= 0 || l.window > m->max_context) m->needs_context = true;
            const int64_t window = l.window > 0 ? std::min<int64_t>(l.window, m->max_context) : m->max_context;
            P.d.window = (int32_t)window;
            P.cap = (int)(window - 1 + B);
            P.pool_rows = l.pool > 0 ? m->max_context / l.pool + 1 : 0;
            n1 = std::max(n1, P.ncat);
            n2 = std::max(n2, H * d);
            n3 = std::max(n3, H * dv);
            m->weight_bytes += dense_bytes(l.in_cat) + dense_bytes(l.out);
        } else if (l.kind == PS_MIX_GLA) {
            if (d > 256) return at + "gated linear attention: dim > 256 is not supported by the scan kernel";
            if (dv <= 0 || l.decay_rank <= 0 || !(l.tau > 0.f)) return at + "gated linear attention sizes";
            P.ncat = 2 * H * d + 2 * H * dv + l.decay_rank;
            if (!shape(l.in_cat, P.ncat, W) || !shape(l.decay2, H * d, l.decay_rank) || !shape(l.out, W, H * dv) || !l.decay0 || !l.onorm)
                return at + "gated linear attention tensors";
            P.off_S = off; off += H * d * dv;
            n1 = std::max(n1, P.ncat);
            n2 = std::max(n2, H * d);
            n3 = std::max(n3, H * dv);
            m->weight_bytes += dense_bytes(l.in_cat) + dense_bytes(l.decay2) + dense_bytes(l.out);
        } else if (l.kind == PS_MIX_MINGRU) {
            P.ncat = 3 * d;
            if (!shape(l.in_cat, P.ncat, W) || !shape(l.out, W, d)) return at + "gated recurrence tensors";
            P.off_S = off; off += d;
            n1 = std::max(n1, P.ncat);
            n3 = std::max(n3, d);
            m->weight_bytes += dense_bytes(l.in_cat) + dense_bytes(l.out);
        } else {
            return at + "unknown mixer kind";
        }
        return "";
    };
    m->L.resize(order.size());
    for (size_t ri = 0; ri < order.size(); ri++) {
        LayerPlan &P = m->L[ri];
        P.layer = order[ri];
        P.d = desc->layers[P.layer];
        const ps_seq_layer &l = P.d;
        const std::string at = "layer " + std::to_string(P.layer) + ": ";
        if (l.form != PS_LAYER_SEQUENTIAL && l.form != PS_LAYER_PARALLEL && l.form != PS_LAYER_PRENORM) return fail(at + "unknown layer form");
        if (l.form == PS_LAYER_PRENORM && (l.canon1 || l.canon2 || l.norm1b || l.norm2b || l.depth_mix)) return fail(at + "a pre-norm layer has no input filter, no norm behind a sublayer and no depth average");
        if (l.form != PS_LAYER_PRENORM && desc->norm_center) return fail(at + "layer norms (norm_center) are built for pre-norm layers");
        if (!l.norm1 || (l.form == PS_LAYER_SEQUENTIAL && !l.norm1b) || (l.form == PS_LAYER_SEQUENTIAL && !l.canon1)) return fail(at + "norm / canon missing");
        if (l.canon1) { P.off_canon1 = off; off += (int64_t)(desc->canon_taps - 1) * W; }
        if (l.canon1 && (l.norm2 && l.form == PS_LAYER_PARALLEL)) return fail(at + "a parallel layer with an input filter has one norm");
        if (l.depth_mix) {
            if (l.form != PS_LAYER_PARALLEL || l.canon1 || desc->loop_times > 1) return fail(at + "depth_mix needs parallel layers without an input filter and no loop");
            depth = true;
        }
        if (l.ff_kind != PS_FF_NONE) {
            if (l.ff_kind != PS_FF_DENSE_XIELU && l.ff_kind != PS_FF_DENSE_SWIGLU && l.ff_kind != PS_FF_MOE_SWIGLU && l.ff_kind != PS_FF_DENSE_RELU_GLU &&
                l.ff_kind != PS_FF_MOE_RELU2)
                return fail(at + "unknown feed-forward kind");
            const bool moe = l.ff_kind == PS_FF_MOE_SWIGLU || l.ff_kind == PS_FF_MOE_RELU2;
            const int64_t pair = l.ff_kind == PS_FF_MOE_RELU2 ? 1 : 2; // rows of the up matrix per inner unit (a gate and its partner, or one)
            if (moe) {
                if ((l.form != PS_LAYER_PARALLEL && l.form != PS_LAYER_PRENORM) || l.canon1)
                    return fail(at + "a mixture of experts needs a parallel or pre-norm layer without an input filter");
                const int rows = l.experts + l.moe_identity; // what the router puts out
                if (l.experts <= 0 || l.moe_identity < 0 || l.top <= 0 || l.top > rows || l.ff <= 0 || !l.router) return fail(at + "mixture-of-experts sizes / router");
                if (l.moe_groups > 0 && (rows % l.moe_groups || l.moe_keep <= 0 || l.moe_keep > l.moe_groups || l.top > (int64_t)l.moe_keep * (rows / l.moe_groups)))
                    return fail(at + "mixture-of-experts groups (equal groups over all router rows, top <= keep * group size)");
                if (!shape(l.ff_up, (int64_t)l.experts * pair * l.ff, W) || !shape(l.ff_down, (int64_t)l.experts * W, l.ff)) return fail(at + "expert tensors");
                if (l.shared_up || l.shared_down) {
                    if (l.shared_ff <= 0 || !shape(l.shared_up, pair * (int64_t)l.shared_ff, W) || !shape(l.shared_down, W, l.shared_ff)) return fail(at + "shared expert tensors");
                    m->weight_bytes += dense_bytes(l.shared_up) + dense_bytes(l.shared_down);
                }
                moe_slots = std::max(moe_slots, B * l.top);
                moe_experts = std::max<int64_t>(moe_experts, rows);
                moe_top = std::max<int64_t>(moe_top, l.top);
                n4 = std::max<int64_t>({n4, (int64_t)l.top * l.ff, (int64_t)l.shared_ff});
                m->weight_bytes += (dense_bytes(l.ff_up) + dense_bytes(l.ff_down)) / l.experts * std::min(l.top, l.experts) + (uint64_t)rows * W * 4;
            }
            const int64_t up_rows = l.ff_kind == PS_FF_DENSE_SWIGLU || l.ff_kind == PS_FF_DENSE_RELU_GLU ? 2 * (int64_t)l.ff : l.ff;
            if (!moe && (!shape(l.ff_up, up_rows, W) || !shape(l.ff_down, W, l.ff))) return fail(at + "feed-forward tensors");
            if (l.form == PS_LAYER_PRENORM && !l.norm2) return fail(at + "feed-forward norm missing");
            if (l.form == PS_LAYER_SEQUENTIAL) {
                if (!l.norm2 || !l.norm2b || !l.canon2) return fail(at + "feed-forward norm / canon missing");
                P.off_canon2 = off; off += (int64_t)(desc->canon_taps - 1) * W;
            }
            const double sp = log1p(exp((double)l.ff_act_p)), sq = log1p(exp((double)l.ff_act_q));
            P.act_p = (float)sp; P.act_q = (float)(0.5 + sq);
            n4 = std::max<int64_t>(n4, l.ff);
            if (!moe) m->weight_bytes += dense_bytes(l.ff_up) + dense_bytes(l.ff_down);
        }
        std::string e = plan_mixer(P, at);
        if (!e.empty()) return fail(e);
        if (l.beside) {
            P.side = std::make_shared<LayerPlan>();
            P.side->layer = P.layer;
            P.side->d = *l.beside;
            if (P.side->d.beside) return fail(at + "a mixer beside another has none beside itself");
            e = plan_mixer(*P.side, at + "second mixer: ");
            if (!e.empty()) return fail(e);
        }
    }
    n2 = std::max(n2, m->n_t2q + nq);
    if (depth)
        for (auto &P : m->L)
            if (P.d.form != PS_LAYER_PARALLEL || P.d.canon1) return fail("depth_mix needs every layer parallel and without an input filter");
    m->zero_floats = off;
    auto mixers = [&](auto &&f) { // every mixer plan, second ones included
        for (auto &P : m->L) { f(P); if (P.side) f(*P.side); }
    };
    mixers([&](LayerPlan &P) {
        if (P.d.kind == PS_MIX_LATENT) { off = (off + 3) / 4 * 4; P.off_ring = off; off += (int64_t)P.cap * (P.d.kv_rank + P.d.rot_dim); } // (16-byte rows for the matrix-core kernels)
        if (P.d.kind == PS_MIX_WINATTN) {
            const int64_t rs = (int64_t)P.d.kv_heads * (P.d.dim + P.d.vdim);
            off = (off + 3) / 4 * 4; P.off_ring = off; off += (int64_t)P.cap * rs;
            off = (off + 3) / 4 * 4; P.off_pool = off; off += P.pool_rows * rs;
        }
    });
    m->state_floats = off;
    auto alloc = [&](void **p, size_t bytes) {
        if (ps_dev_malloc(p, bytes + 256) != hipSuccess) return false;
        m->owned.push_back(*p);
        return true;
    };
    bool ok = true;
    std::map<const void *, float *> freq_of; // one table per layer (keyed by its output matrix), shared by its runs
    mixers([&](LayerPlan &P) {
        const bool lat = P.d.kind == PS_MIX_LATENT, win = P.d.kind == PS_MIX_WINATTN;
        if (!(lat || win) || P.d.rot_dims <= 0 || !ok) return;
        auto it = freq_of.find(P.d.out);
        if (it != freq_of.end()) { P.freq = it->second; return; }
        const int half = P.d.rot_dims / 2;
        const double factor = win && P.d.rot_factor != 0.f ? (double)P.d.rot_factor : 1.0;
        std::vector<float> f(half);
        for (int i = 0; i < half; i++) f[i] = (float)(pow((double)P.d.rot_base, -2.0 * i / (double)P.d.rot_dims) / factor);
        if (lat && P.d.yarn_factor > 0.f) {
            // frequency scaling by wavelength: pairs that turn often within the original context keep their frequency, slow ones are divided by the factor, a ramp between
            const double dims = P.d.rot_dims, base = P.d.rot_base, pi = 3.14159265358979323846;
            auto turn_index = [&](double turns) { return dims * log((double)P.d.yarn_original / (2.0 * pi * turns)) / (2.0 * log(base)); };
            const double lo = std::max(floor(turn_index(P.d.yarn_fast)), 0.0), hi = std::min(ceil(turn_index(P.d.yarn_slow)), dims - 1.0);
            for (int i = 0; i < half; i++) {
                const double fi = pow(base, -2.0 * i / dims), ramp = std::min(std::max((i - lo) / std::max(hi - lo, 0.001), 0.0), 1.0);
                f[i] = (float)(fi / (double)P.d.yarn_factor * ramp + fi * (1.0 - ramp));
            }
        }
        ok = ok && alloc((void **)&P.freq, half * 4);
        if (ok) ok = hipMemcpyAsync(P.freq, f.data(), half * 4, hipMemcpyHostToDevice, c->stream) == hipSuccess && hipStreamSynchronize(c->stream) == hipSuccess;
        freq_of[P.d.out] = P.freq;
    });
    {
        // the stacked input projections of two mixers side by side, joined once per layer (its runs share the copy)
        auto stacked = [](int kind) { return kind == PS_MIX_WINATTN || kind == PS_MIX_GLA || kind == PS_MIX_DELTA || kind == PS_MIX_MINGRU; };
        std::map<int, std::pair<const ps_dense *, const float *>> joint_of;
        for (auto &P : m->L) {
            if (!ok || !P.side || !stacked(P.d.kind) || !stacked(P.side->d.kind) || P.d.in_cat->dtype != P.side->d.in_cat->dtype) continue;
            const ps_dense *a = P.d.in_cat, *b = P.side->d.in_cat;
            auto it = joint_of.find(P.layer);
            if (it == joint_of.end()) {
                const size_t es = a->dtype == PS_BF16 ? 2 : 4, na = (size_t)a->N * a->K * es, nb = (size_t)b->N * b->K * es;
                auto j = new ps_dense();
                m->joints.push_back(j);
                j->dtype = a->dtype; j->N = a->N + b->N; j->K = a->K;
                ok = ok && alloc(&j->data, na + nb) && hipMemcpyAsync(j->data, a->data, na, hipMemcpyDeviceToDevice, c->stream) == hipSuccess &&
                     hipMemcpyAsync((char *)j->data + na, b->data, nb, hipMemcpyDeviceToDevice, c->stream) == hipSuccess;
                float *bias = nullptr;
                if (ok && (P.d.in_bias || P.side->d.in_bias)) {
                    ok = alloc((void **)&bias, (size_t)j->N * 4);
                    if (ok) {
                        psk_fill(c->stream, bias, 0.f, j->N);
                        if (P.d.in_bias) ok = ok && hipMemcpyAsync(bias, P.d.in_bias, (size_t)a->N * 4, hipMemcpyDeviceToDevice, c->stream) == hipSuccess;
                        if (P.side->d.in_bias) ok = ok && hipMemcpyAsync(bias + a->N, P.side->d.in_bias, (size_t)b->N * 4, hipMemcpyDeviceToDevice, c->stream) == hipSuccess;
                    }
                }
                ok = ok && hipStreamSynchronize(c->stream) == hipSuccess;
                it = joint_of.emplace(P.layer, std::make_pair((const ps_dense *)j, (const float *)bias)).first;
            }
            P.joint = it->second.first; P.joint_bias = it->second.second;
            P.in_ld = P.side->in_ld = a->N + b->N;
            P.in_off = 0; P.side->in_off = a->N;
            n1 = std::max(n1, P.in_ld);
        }
    }
    ok = ok && alloc((void **)&m->step, sizeof(ps_seq_step)) && alloc((void **)&m->x, B * W * 4) && alloc((void **)&m->hn, B * W * 4) && alloc((void **)&m->h, B * W * 4) &&
         alloc((void **)&m->y, B * W * 4) && alloc((void **)&m->t1, B * std::max<int64_t>(n1, 1) * 4) && alloc((void **)&m->t2, B * std::max<int64_t>(n2, 1) * 4) &&
         alloc((void **)&m->t3, B * std::max<int64_t>(n3, 1) * 4) && alloc((void **)&m->t4, B * std::max<int64_t>(n4, 1) * 4) &&
         alloc((void **)&m->kvx, std::max<int64_t>(nkv, 1) * 4) && alloc((void **)&m->xn, B * W * 4) && alloc((void **)&m->logits, B * (int64_t)desc->vocab * 4) &&
         alloc((void **)&m->tokens, B * 4) && alloc((void **)&m->want, B * 4) && alloc((void **)&m->amax, B * 4);
    if (depth) ok = ok && alloc((void **)&m->hist, (size_t)(order.size() + 1) * B * W * 4);
    if (moe_slots)
        ok = ok && alloc((void **)&m->moe_sel, moe_slots * 4) && alloc((void **)&m->moe_list, moe_slots * 4) && alloc((void **)&m->moe_seg, (moe_experts + 1) * 4) &&
             alloc((void **)&m->moe_wgt, moe_slots * 4) && alloc((void **)&m->moe_sg, B * 4) && (moe_top <= 1 || alloc((void **)&m->moe_y, moe_slots * W * 4));
    {
        size_t ab = 0;
        mixers([&](LayerPlan &P) {
            if (P.d.kind == PS_MIX_LATENT && psk_latent_absorbed_ok(P.d.dim, P.d.rot_dim, P.d.vdim, P.d.kv_rank))
                ab = std::max(ab, psk_latent_absorbed_scratch(P.d.heads, P.d.kv_rank, P.d.window));
        });
        if (ab) ok = ok && alloc((void **)&m->abs_scratch, ab);
        size_t wb = 0;
        mixers([&](LayerPlan &P) {
            if (P.d.kind == PS_MIX_WINATTN && psk_winattn_mfma_ok(P.d.dim, P.d.vdim))
                wb = std::max(wb, psk_winattn_step_scratch(P.d.heads, P.d.vdim, P.d.window, P.d.pool, m->max_context));
        });
        if (wb) ok = ok && alloc((void **)&m->win_scratch, wb);
    }
    if (desc->compute == 0) { // the wide mat-mul's operand copy: the widest input of any matrix x a portion's rows, or the window's rows x the latent
        int64_t kmax = W, kvrows = 0, kvk = 0;
        mixers([&](LayerPlan &P) {
            kmax = std::max<int64_t>({kmax, P.d.ff, P.d.shared_ff, P.d.heads * (int64_t)std::max(P.d.dim, P.d.vdim), P.d.q_rank, P.d.decay_rank});
            if (P.d.kind == PS_MIX_LATENT) { kvrows = std::max<int64_t>(kvrows, P.d.window - 1 + B); kvk = std::max<int64_t>(kvk, P.d.kv_rank); }
        });
        // (a grouped product packs its slots in list order and a tile may start anywhere in the list: one tile of rows more)
        const int64_t r128 = std::max((B + 127) / 128 * 128, moe_slots ? (moe_slots + 127) / 128 * 128 + 128 : 0), kv128 = (kvrows + 127) / 128 * 128;
        m->pack_bytes = (size_t)std::max(r128 * kmax, kv128 * kvk) * 2;
        ok = ok && alloc(&m->pack, m->pack_bytes);
    }
    m->slot_state.assign(desc->n_slots, nullptr);
    m->slot_pos.assign(desc->n_slots, -1);
    for (int s = 0; ok && s < desc->n_slots; s++) ok = alloc((void **)&m->slot_state[s], (size_t)m->state_floats * 4);
    if (!ok) return fail("out of device memory");
    *out = m;
    return 0;
}

void ps_hip_seq_destroy(ps_hip_seq *m) {
    if (!m) return;
    (void)hipSetDevice(m->ctx->device);
    (void)hipStreamSynchronize(m->ctx->stream);
    for (auto &g : m->graphs) (void)hipGraphExecDestroy(g.second);
    for (void *p : m->owned) (void)ps_dev_free(p);
    for (ps_dense *j : m->joints) delete j; // (their data is in `owned`)
    if (m->ids) (void)ps_dev_free(m->ids);
    delete m;
}

int ps_hip_seq_acquire(ps_hip_seq *m, int *slot) {
    ps_hip_ctx *c = m->ctx;
    *slot = -1;
    for (size_t s = 0; s < m->slot_pos.size(); s++)
        if (m->slot_pos[s] < 0) {
            psk_fill(c->stream, m->slot_state[s], 0.f, m->zero_floats); // (a fill kernel, not a memset: the state is read by captured launch sequences)
            PS_CHECK(c, hipGetLastError());
            m->slot_pos[s] = 0;
            *slot = (int)s;
            return 0;
        }
    return seq_fail(c, "seq_acquire: every slot is in use");
}
int ps_hip_seq_release(ps_hip_seq *m, int slot) {
    if (slot < 0 || slot >= (int)m->slot_pos.size() || m->slot_pos[slot] < 0) return seq_fail(m->ctx, "seq_release: not a live slot");
    m->slot_pos[slot] = -1;
    return 0;
}
int64_t ps_hip_seq_position(const ps_hip_seq *m, int slot) { return (slot < 0 || slot >= (int)m->slot_pos.size()) ? -1 : m->slot_pos[slot]; }
size_t ps_hip_seq_slot_bytes(const ps_hip_seq *m) { return (size_t)m->state_floats * 4; }
uint64_t ps_hip_seq_weight_bytes_per_token(const ps_hip_seq *m) { return m->weight_bytes; }
int ps_hip_seq_layer_runs(const ps_hip_seq *m) { return (int)m->L.size(); }
int ps_hip_seq_debug_layers(ps_hip_seq *m, float *buf) { m->dbg_layers = buf; return 0; }
int ps_hip_seq_set_mode(ps_hip_seq *m, int mode) { m->mode = mode; return 0; }

} // extern "C"

// The launches of one portion: T <= max_batch tokens (device ids in m->tokens, or the step's own token0 when from_step) of the slot whose state
// pointer is `state`.  any_pos: a captured sequence that must hold for any position -- whatever depends on the position (the rows of a window's
// expansion, the visible blocks) is launched for its most and cut on the device; otherwise the step's position is known on the host (pos0).
static void seq_layers(ps_hip_seq *m, float *state, int T, int64_t pos0, bool any_pos, bool from_step) {
    hipStream_t st = m->ctx->stream;
    const ps_seq_desc &D = m->d;
    const int64_t W = D.width;
    const bool tiled = (m->mode & 2) != 0;
    const int64_t BW = (int64_t)D.max_batch * W;
    psk_embed(st, D.embed, from_step ? nullptr : m->tokens, m->step, T, m->embed_scale, m->hist ? m->hist : m->x, W);
    auto mm = [&](const ps_dense *w, const float *a, int64_t lda, float *out, int64_t ldo) {
        psk_dense_args g;
        g.w = w; g.a = a; g.lda = lda; g.T = T; g.out = out; g.ldo = ldo; g.force_tiled = tiled; g.pack = m->pack; g.pack_bytes = m->pack_bytes;
        return g;
    };
    // a sublayer boundary: x += norm_b(y) (after a sublayer), then hn = norm(x), h = conv(hn) (in front of the next one); one launch for a single token
    auto boundary = [&](const float *y, const float *wb, const float *wn, const float *cw, int64_t tail_off) {
        if (T == 1 && !tiled && m->groups == 1) {
            psk_boundary1(st, m->step, m->x, y, wb, wn, cw, D.canon_taps, tail_off, D.norm_offset, D.norm_eps, W, m->h, m->hn);
            return;
        }
        if (y) psk_norm_residual(st, m->x, y, wb, D.norm_offset, D.norm_eps, W, T, m->groups);
        if (wn) {
            psk_rmsnorm(st, m->x, W, nullptr, wn, D.norm_offset, D.norm_eps, W, T, m->hn, W, m->groups);
            psk_causal_conv(st, m->step, tail_off, m->hn, W, cw, D.canon_taps, 0, W, T, m->h, W);
        }
    };
    // One mixer on the input m->h.  Its output projection writes m->y (into == NULL) or adds out_scale times its result to `into`.
    auto mixer = [&](const LayerPlan &P, float *into, float out_scale) {
        const ps_seq_layer &l = P.d;
        const int64_t H = l.heads, d = l.dim, dv = l.vdim;
        float *t1 = m->t1 + P.in_off;                       // this mixer's columns of the (possibly joint) input projection
        const int64_t ld1 = P.in_ld ? P.in_ld : P.ncat;
        auto out_proj = [&](const float *a, int64_t lda) {
            auto g = mm(l.out, a, lda, into ? into : m->y, W);
            g.alpha = out_scale; g.accum = into ? 1 : 0;
            psk_dense(st, g);
        };
        if (l.kind == PS_MIX_WKV) {
            const int64_t Hd = H * d, NW = 5 * Hd;
            const ps_dense *ws[4] = {l.in_r, l.in_k, l.in_v, l.in_g};
            for (int s = 0; s < 4; s++) {
                auto g = mm(ws[s], m->h, W, m->t1 + s * Hd, NW);
                g.mu = l.mu + s * W; g.shift0 = state + P.off_shift;
                psk_dense(st, g);
            }
            {
                auto g = mm(l.decay1, m->h, W, m->t2, l.decay_rank);
                g.mu = l.mu + 4 * W; g.shift0 = state + P.off_shift; g.act = PSD_ACT_TANH;
                psk_dense(st, g);
                auto g2 = mm(l.decay2, m->t2, l.decay_rank, m->t1 + 4 * Hd, NW);
                g2.bias = l.decay0;
                psk_dense(st, g2);
            }
            psk_state_store(st, m->step, P.off_shift, m->h + (int64_t)(T - 1) * W, W);
            psk_wkv_scan(st, m->step, P.off_S, m->t1, m->t1 + Hd, m->t1 + 2 * Hd, m->t1 + 4 * Hd, NW, l.bonus, (int)H, (int)d, T, m->t3, Hd);
            psk_headnorm_gate(st, m->t3, Hd, m->t1 + 3 * Hd, NW, l.onorm, (int)d, D.norm_eps, (int)H, (int)d, T);
            out_proj(m->t3, Hd);
        } else if (l.kind == PS_MIX_DELTA) {
            const int64_t KHd = (int64_t)l.kv_heads * d, Hv = H * dv;
            if (!P.in_ld) psk_dense(st, mm(l.in_cat, m->h, W, t1, ld1));
            psk_causal_conv(st, m->step, P.off_conv, t1, ld1, l.conv, l.conv_taps, 1, P.cqkv, T, m->t2, P.cqkv);
            psk_delta_scan(st, m->step, P.off_S, m->t2, m->t2 + KHd, m->t2 + 2 * KHd, t1 + P.cqkv + Hv, t1 + P.cqkv + Hv + H, P.cqkv, ld1, l.a_log, l.dt_bias,
                           (int)H, l.kv_heads, (int)d, (int)dv, T, m->t3, Hv);
            psk_headnorm_gate(st, m->t3, Hv, t1 + P.cqkv, ld1, l.onorm, 0, D.norm_eps, (int)H, (int)dv, T);
            out_proj(m->t3, Hv);
        } else if (l.kind == PS_MIX_GLA) {
            // t1 = [ q | k | v | g | a1 ]; the decay's second matrix (with its bias) -> t2; scan -> t3; per-head norm and gate; out
            const int64_t Hd = H * d, Hv = H * dv;
            if (!P.in_ld) psk_dense(st, mm(l.in_cat, m->h, W, t1, ld1));
            auto g2 = mm(l.decay2, t1 + 2 * Hd + 2 * Hv, ld1, m->t2, Hd);
            g2.bias = l.decay0;
            psk_dense(st, g2);
            psk_gla_scan(st, m->step, P.off_S, t1, t1 + Hd, t1 + 2 * Hd, ld1, m->t2, Hd, l.tau, (int)H, (int)d, (int)dv, T, m->t3, Hv);
            psk_headnorm_gate(st, m->t3, Hv, t1 + 2 * Hd + Hv, ld1, l.onorm, 0, D.norm_eps, (int)H, (int)dv, T);
            out_proj(m->t3, Hv);
        } else if (l.kind == PS_MIX_WINATTN) {
            // t1 = [ q | k | v | gate ] (+ bias); norms, rotation, ring append and block means; attention -> t3; out
            const int64_t G = l.kv_heads, Hd = H * d, Hv = H * dv;
            if (!P.in_ld) {
                auto g = mm(l.in_cat, m->h, W, t1, ld1);
                g.bias = l.in_bias;
                psk_dense(st, g);
            }
            psk_winattn_prep(st, m->step, P.off_ring, P.cap, P.off_pool, l.pool, t1, ld1, l.qnorm, l.knorm, D.norm_eps, (int)H, (int)G, (int)d, (int)dv, l.rot_dims,
                             l.rot_pairing, P.freq, T, m->t2, Hd, l.qtemp_coef, l.qtemp_every, l.head_norm, l.v_unit);
            const float *gate = l.gated ? t1 + Hd + G * d + G * dv : nullptr;
            const int ge = l.gated == 2; // a gate per output element
            const bool mfma = (m->mode & 2) == 0 && (G * (d + dv)) % 4 == 0 && psk_winattn_mfma_ok((int)d, (int)dv);
            if (mfma && T == 1 && m->win_scratch)
                psk_winattn_step(st, m->step, P.off_ring, P.cap, P.off_pool, l.pool, m->t2, gate, l.temp, l.sink, (int)H, (int)G, (int)d, (int)dv, l.window, l.scale,
                                 m->max_context, m->win_scratch, m->t3, l.softcap, ge);
            else if (mfma)
                psk_winattn_mfma(st, m->step, P.off_ring, P.cap, P.off_pool, l.pool, m->t2, Hd, gate, ld1, l.temp, l.sink, (int)H, (int)G, (int)d, (int)dv, l.window, l.scale,
                                 T, m->t3, Hv, l.softcap, ge);
            else
                psk_winattn(st, m->step, P.off_ring, P.cap, P.off_pool, l.pool, m->t2, Hd, gate, ld1, l.temp, l.sink, (int)H, (int)G, (int)d, (int)dv, l.window, l.scale, T,
                            m->t3, Hv, l.softcap, ge);
            out_proj(m->t3, Hv);
        } else if (l.kind == PS_MIX_MINGRU) {
            // t1 = [ z | x | g ] (+ bias); the recurrence and the gate -> t3; out
            if (!P.in_ld) {
                auto g = mm(l.in_cat, m->h, W, t1, ld1);
                g.bias = l.in_bias;
                psk_dense(st, g);
            }
            psk_mingru_scan(st, m->step, P.off_S, t1, ld1, d, T, m->t3, d);
            out_proj(m->t3, d);
        } else {
            // t1 = [ dq | dkv ], or with direct queries [ q | dkv | gate ]; the latents' norms, rotation of the shared key part and ring append; attention -> t3; out
            const int64_t dr = l.rot_dim, rs = l.kv_rank + dr, Hv = H * dv, nq = H * (d + dr);
            const bool direct = l.q_rank == 0;
            float *cq = m->t2, *q = direct ? m->t1 : m->t2 + (int64_t)D.max_batch * m->n_t2q;
            const int64_t ldq = direct ? P.ncat : nq;
            const float *gate = l.gated ? m->t1 + P.ncat - H : nullptr;
            psk_dense(st, mm(l.in_cat, m->h, W, m->t1, P.ncat));
            psk_latent_prep(st, m->step, P.off_ring, P.cap, direct ? m->t1 + nq : m->t1, P.ncat, l.qnorm, l.kvnorm, D.norm_eps, l.q_rank, l.kv_rank, (int)dr, l.rot_dims, P.freq, T,
                            cq, l.q_rank, P.rot_mag);
            if (!direct) psk_dense(st, mm(l.uq, cq, l.q_rank, q, nq));
            const bool plain = (m->mode & 2) != 0, rows4 = (l.kv_rank + dr) % 4 == 0 && l.kv_rank % 4 == 0;
            if (T == 1 && !plain && m->abs_scratch && psk_latent_absorbed_ok((int)d, (int)dr, (int)dv, l.kv_rank)) {
                psk_latent_absorbed(st, m->step, P.off_ring, P.cap, q, (int)(d + dr), l.ukv, P.freq, (int)H, (int)d, (int)dr, l.rot_dims, (int)dv, l.kv_rank, l.window,
                                    l.scale, m->abs_scratch, m->t3, P.rot_mag, gate);
            } else {
                // the window's keys and values, expanded from the ring rows  max(0, pos0 - window + 1) .. pos0 + T - 1
                auto g = mm(l.ukv, state + P.off_ring, rs, m->kvx, H * d + Hv);
                g.a_step = m->step; g.a_row0 = -(int64_t)(l.window - 1); g.a_mod = P.cap;
                g.T = any_pos ? l.window - 1 + T : (int)(std::min<int64_t>(pos0, l.window - 1) + T);
                psk_dense(st, g);
                if (!plain && rows4 && psk_latent_attn_mfma_ok((int)d, (int)dr, (int)dv))
                    psk_latent_attn_mfma(st, m->step, P.off_ring, P.cap, q, ldq, m->kvx, H * d + Hv, P.freq, (int)H, (int)d, (int)dr, l.rot_dims, (int)dv, l.kv_rank, l.window,
                                         l.scale, T, m->t3, Hv, P.rot_mag, gate, P.ncat);
                else
                    psk_latent_attn(st, m->step, P.off_ring, P.cap, q, ldq, m->kvx, H * d + Hv, P.freq, (int)H, (int)d, (int)dr, l.rot_dims, (int)dv, l.kv_rank, l.window,
                                    l.scale, T, m->t3, Hv, P.rot_mag, gate, P.ncat);
            }
            out_proj(m->t3, Hv);
        }
    };
    auto joint_in = [&](const LayerPlan &P) { // both mixers' stacked input projections in one product
        if (!P.joint) return;
        auto g = mm(P.joint, m->h, W, m->t1, P.in_ld);
        g.bias = P.joint_bias;
        psk_dense(st, g);
    };
    auto ff_up = [&](const LayerPlan &P, const float *in) {
        const ps_seq_layer &l = P.d;
        auto g = mm(l.ff_up, in, W, m->t4, l.ff);
        if (l.ff_kind == PS_FF_DENSE_SWIGLU) g.act = PSD_ACT_SILU_PAIR;
        else if (l.ff_kind == PS_FF_DENSE_RELU_GLU) g.act = PSD_ACT_RELU_PAIR;
        else { g.act = PSD_ACT_XIELU; g.act_p = P.act_p; g.act_q = P.act_q; }
        if (l.ff_kind != PS_FF_DENSE_XIELU) g.bias = l.ff_up_bias;
        psk_dense(st, g);
    };
    // The feed-forward of a parallel or pre-norm layer on `in`, added to xr times alpha.  Mixture of experts: slot s = t top + i is token t's i-th choice; the router's
    // score scales what the expert READS (the A operand of its first product) or, moe_weight_output, what it puts out (the rows of its inner activation: the second
    // product is linear); a few tokens run grouped mat-vecs, a portion tiles over the slots sorted by expert.  A choice beyond the experts that have matrices is an
    // identity expert: no product touches its slot, and its weight times the input joins the sum.
    auto feed_forward = [&](const LayerPlan &P, const float *in, float *xr, float alpha) {
        const ps_seq_layer &l = P.d;
        const bool moe = l.ff_kind == PS_FF_MOE_SWIGLU || l.ff_kind == PS_FF_MOE_RELU2;
        if (!moe) {
            ff_up(P, in);
            auto g = mm(l.ff_down, m->t4, l.ff, xr, W);
            g.accum = 1; g.alpha = alpha;
            if (l.ff_kind != PS_FF_DENSE_XIELU) g.bias = l.ff_down_bias;
            psk_dense(st, g);
            return;
        }
        const int E = l.experts, rows = E + l.moe_identity, top = l.top, S = T * top;
        const int act = l.ff_kind == PS_FF_MOE_RELU2 ? PSD_ACT_RELU2 : PSD_ACT_SILU_PAIR;
        psk_moe_route(st, in, W, l.router, l.shared_gate, rows, top, l.moe_norm_top, W, T, m->moe_sel, m->moe_wgt, m->moe_sg, l.moe_softmax, l.moe_correction, l.moe_groups,
                      l.moe_keep);
        const bool mv = !tiled && T <= 8 && (size_t)std::max<int64_t>(W, (int64_t)top * l.ff) * 4 + 64 <= 128 * 1024;
        if (!mv) psk_moe_plan(st, m->moe_sel, S, rows, m->moe_seg, m->moe_list);
        auto grouped = [&](psk_dense_args &g) {
            g.groups = E; g.g_sel = m->moe_sel;
            if (!mv) { g.g_seg = m->moe_seg; g.g_list = m->moe_list; }
        };
        {
            auto g = mm(l.ff_up, in, W, m->t4, l.ff);
            g.act = act; g.T = S; g.g_adiv = top;
            if (l.moe_weight_output) g.out_scale = m->moe_wgt; // (a row of the result is a slot)
            else g.g_scale = m->moe_wgt;
            grouped(g);
            psk_dense(st, g);
        }
        bool summed = false; // the identity slots' share has joined the stream
        {
            auto g = mm(l.ff_down, m->t4, l.ff, xr, W);
            grouped(g);
            if (mv) {
                g.T = T; g.g_inner = top; g.accum = 1; g.alpha = alpha;
                if (l.moe_identity) { g.g_ident = in; g.g_ident_ld = W; g.g_ident_w = m->moe_wgt; summed = true; } // (the identity slots' share inside the same launch)
            }
            else if (top == 1) { g.T = S; g.accum = 1; g.alpha = alpha; }
            else { g.T = S; g.out = m->moe_y; } // (two slots of a token sit in different tiles: per-slot results, summed below)
            psk_dense(st, g);
            if (!mv && top > 1) {
                psk_moe_combine(st, xr, m->moe_y, top, alpha, W, T, l.moe_identity ? m->moe_sel : nullptr, m->moe_wgt, E, in, W);
                summed = true;
            }
        }
        if (l.moe_identity && !summed) psk_moe_combine(st, xr, nullptr, top, alpha, W, T, m->moe_sel, m->moe_wgt, E, in, W);
        if (l.shared_up) {
            auto g = mm(l.shared_up, in, W, m->t4, l.shared_ff);
            g.act = act;
            psk_dense(st, g);
            auto g2 = mm(l.shared_down, m->t4, l.shared_ff, xr, W);
            g2.accum = 1; g2.alpha = alpha; g2.out_scale = l.shared_gate ? m->moe_sg : nullptr;
            psk_dense(st, g2);
        }
    };
    const int n_runs = (int)m->L.size();
    if (m->L[0].d.form == PS_LAYER_SEQUENTIAL) boundary(nullptr, nullptr, m->L[0].d.norm1, m->L[0].d.canon1, m->L[0].off_canon1);
    for (int li = 0; li < n_runs; li++) {
        const LayerPlan &P = m->L[li];
        const ps_seq_layer &l = P.d;
        const LayerPlan *next = li + 1 < n_runs ? &m->L[li + 1] : nullptr;
        const float res = l.res_scale != 0.f ? l.res_scale : 1.f;
        if (l.form == PS_LAYER_PRENORM) {
            // x += mixer(norm1(x)), then x += ff(norm2(x)): each sublayer's front is one launch, its output projection adds straight into the residual stream
            psk_front(st, m->x, 0, 1, nullptr, nullptr, nullptr, l.norm1, m->h, nullptr, nullptr, m->groups, D.norm_offset, D.norm_eps, W, T, D.norm_center);
            joint_in(P);
            mixer(P, m->x, l.mix_scale);
            if (P.side) mixer(*P.side, m->x, P.side->d.mix_scale);
            if (l.ff_kind != PS_FF_NONE) {
                psk_front(st, m->x, 0, 1, nullptr, nullptr, nullptr, l.norm2, m->h, nullptr, nullptr, m->groups, D.norm_offset, D.norm_eps, W, T, D.norm_center);
                feed_forward(P, m->h, m->x, 1.f);
            }
        } else if (l.form == PS_LAYER_PARALLEL && !l.canon1) {
            // No input filter: one launch makes the layer's input (with depth_mix: the previous layer's average over X_0 .. X_li, kept as this layer's X to add
            // into) and both sublayers' norms; mixers and feed-forward add their output projections, times res, straight into the layer's X
            float *xr = m->hist ? m->hist + (int64_t)(li + 1) * BW : m->x;
            float *h2 = l.norm2 ? m->hn : nullptr;
            if (m->hist) psk_front(st, m->hist, BW, li + 1, li ? m->L[li - 1].d.depth_mix : nullptr, nullptr, xr, l.norm1, m->h, l.norm2, h2, m->groups, D.norm_offset, D.norm_eps, W, T);
            else psk_front(st, m->x, 0, 1, nullptr, nullptr, nullptr, l.norm1, m->h, l.norm2, h2, m->groups, D.norm_offset, D.norm_eps, W, T);
            joint_in(P);
            mixer(P, xr, res * l.mix_scale);
            if (P.side) mixer(*P.side, xr, res * P.side->d.mix_scale);
            if (l.ff_kind != PS_FF_NONE) feed_forward(P, h2 ? h2 : m->h, xr, res);
            if (m->dbg_layers && !any_pos && m->hist)
                psk_front(st, m->hist, BW, li + 2, l.depth_mix, nullptr, m->dbg_layers + (int64_t)li * BW, nullptr, nullptr, nullptr, nullptr, 1, 0.f, D.norm_eps, W, T);
        } else if (l.form == PS_LAYER_PARALLEL) {
            // hn = norm(x), h = conv(hn); both mixers and the feed-forward add their output projections straight into the residual stream
            boundary(nullptr, nullptr, l.norm1, l.canon1, P.off_canon1);
            joint_in(P);
            mixer(P, m->x, res * l.mix_scale);
            if (P.side) mixer(*P.side, m->x, res * P.side->d.mix_scale);
            if (l.ff_kind != PS_FF_NONE) feed_forward(P, m->hn, m->x, res);
        } else {
            const bool summed = P.side != nullptr || l.mix_scale != 1.f;
            if (summed) psk_fill(st, m->y, 0.f, (int64_t)T * W);
            joint_in(P);
            mixer(P, summed ? m->y : nullptr, l.mix_scale);
            if (P.side) mixer(*P.side, m->y, P.side->d.mix_scale);
            const bool nseq = next && next->d.form == PS_LAYER_SEQUENTIAL;
            const float *nn = nseq ? next->d.norm1 : nullptr, *nc = nseq ? next->d.canon1 : nullptr;
            const int64_t no = nseq ? next->off_canon1 : 0;
            if (l.ff_kind != PS_FF_NONE) {
                boundary(m->y, l.norm1b, l.norm2, l.canon2, P.off_canon2);
                ff_up(P, m->h);
                psk_dense(st, mm(l.ff_down, m->t4, l.ff, m->y, W));
                boundary(m->y, l.norm2b, nn, nc, no);
            } else {
                boundary(m->y, l.norm1b, nn, nc, no);
            }
        }
        if (m->dbg_layers && !any_pos && !m->hist) psk_copy(st, m->x, m->dbg_layers + (int64_t)li * BW, (int64_t)T * W);
    }
}

// final norm on `rows` rows of x (idx: device indices, or NULL for rows 0 ..), logits, arg-max
static void seq_head(ps_hip_seq *m, const int32_t *idx, int rows) {
    hipStream_t st = m->ctx->stream;
    const ps_seq_desc &D = m->d;
    if (m->hist) { // what the last layer hands on (its depth average, or its own result) and the final norm in one launch
        const int runs = (int)m->L.size();
        psk_front(st, m->hist, (int64_t)D.max_batch * D.width, runs + 1, m->L[runs - 1].d.depth_mix, idx, nullptr, D.final_norm, m->xn, nullptr, nullptr, m->groups,
                  D.norm_offset, D.norm_eps, D.width, rows);
    } else if (D.norm_center) {
        psk_front(st, m->x, 0, 1, nullptr, idx, nullptr, D.final_norm, m->xn, nullptr, nullptr, m->groups, D.norm_offset, D.norm_eps, D.width, rows, 1);
    } else {
        psk_rmsnorm(st, m->x, D.width, idx, D.final_norm, D.norm_offset, D.norm_eps, D.width, rows, m->xn, D.width, m->groups);
    }
    psk_dense_args g;
    g.w = D.head; g.a = m->xn; g.lda = D.width; g.T = rows; g.out = m->logits; g.ldo = D.vocab; g.alpha = D.logit_scale; g.force_tiled = (m->mode & 2) != 0; g.pack = m->pack; g.pack_bytes = m->pack_bytes;
    psk_dense(st, g);
    psk_argmax_rows(st, m->logits, D.vocab, rows, m->amax);
}

extern "C" {

int ps_hip_seq_forward(ps_hip_seq *m, int slot, const int32_t *tokens, int n, const int32_t *want, int n_want, float *logits_host, int32_t *argmax_host) {
    ps_hip_ctx *c = m->ctx;
    if (slot < 0 || slot >= (int)m->slot_pos.size() || m->slot_pos[slot] < 0) return seq_fail(c, "seq_forward: not a live slot");
    if (n <= 0 || !tokens) return seq_fail(c, "seq_forward: no tokens");
    if (m->needs_context && m->slot_pos[slot] + n > m->max_context) return seq_fail(c, "seq_forward: the sequence would exceed max_context");
    for (int i = 0; i < n; i++)
        if (tokens[i] < 0 || tokens[i] >= m->d.vocab) return seq_fail(c, "seq_forward: token id outside the vocabulary");
    for (int i = 0; i < n_want; i++)
        if (want[i] < 0 || want[i] >= n || (i && want[i] < want[i - 1])) return seq_fail(c, "seq_forward: want must be ascending indices into the step's tokens");
    PS_CHECK(c, hipSetDevice(c->device));
    const int B = m->d.max_batch;
    int wi = 0;
    for (int t0 = 0; t0 < n; t0 += B) {
        const int T = std::min(B, n - t0);
        const int64_t pos0 = m->slot_pos[slot];
        PS_CHECK(c, hipMemcpyAsync(m->tokens, tokens + t0, (size_t)T * 4, hipMemcpyHostToDevice, c->stream));
        hipLaunchKernelGGL(seq_set_step_kernel, dim3(1), dim3(1), 0, c->stream, m->step, (long long)pos0, T, slot, m->slot_state[slot], (int)tokens[t0]);
        seq_layers(m, m->slot_state[slot], T, pos0, false, false);
        std::vector<int32_t> idx;
        const int w0 = wi;
        while (wi < n_want && want[wi] < t0 + T) idx.push_back(want[wi++] - t0);
        if (!idx.empty()) {
            PS_CHECK(c, hipMemcpyAsync(m->want, idx.data(), idx.size() * 4, hipMemcpyHostToDevice, c->stream));
            seq_head(m, m->want, (int)idx.size());
            if (logits_host)
                PS_CHECK(c, hipMemcpyAsync(logits_host + (size_t)w0 * m->d.vocab, m->logits, idx.size() * (size_t)m->d.vocab * 4, hipMemcpyDeviceToHost, c->stream));
            if (argmax_host) PS_CHECK(c, hipMemcpyAsync(argmax_host + w0, m->amax, idx.size() * 4, hipMemcpyDeviceToHost, c->stream));
        }
        PS_CHECK(c, hipStreamSynchronize(c->stream)); // (idx and the caller's token buffer are read by the copies above)
        PS_CHECK(c, hipGetLastError());
        m->slot_pos[slot] = pos0 + T;
    }
    return 0;
}

int ps_hip_seq_decode_greedy(ps_hip_seq *m, int slot, int32_t token, int steps, int32_t *out_ids) {
    ps_hip_ctx *c = m->ctx;
    if (slot < 0 || slot >= (int)m->slot_pos.size() || m->slot_pos[slot] < 0) return seq_fail(c, "seq_decode_greedy: not a live slot");
    if (steps <= 0) return 0;
    if (token < 0 || token >= m->d.vocab) return seq_fail(c, "seq_decode_greedy: token id outside the vocabulary");
    if (m->needs_context && m->slot_pos[slot] + steps > m->max_context) return seq_fail(c, "seq_decode_greedy: the sequence would exceed max_context");
    PS_CHECK(c, hipSetDevice(c->device));
    if (steps > m->ids_cap) {
        if (m->ids) { PS_CHECK(c, hipStreamSynchronize(c->stream)); (void)ps_dev_free(m->ids); m->ids = nullptr; }
        PS_CHECK(c, ps_dev_malloc((void **)&m->ids, (size_t)steps * 4 + 256));
        m->ids_cap = steps;
        for (auto &g : m->graphs) (void)hipGraphExecDestroy(g.second); // (the captured sequences hold the old pointer)
        m->graphs.clear();
    }
    float *state = m->slot_state[slot];
    hipLaunchKernelGGL(seq_set_step_kernel, dim3(1), dim3(1), 0, c->stream, m->step, (long long)m->slot_pos[slot], 1, slot, state, (int)token);
    auto one = [&]() {
        seq_layers(m, state, 1, 0, true, true);
        seq_head(m, nullptr, 1);
        hipLaunchKernelGGL(seq_advance_kernel, dim3(1), dim3(1), 0, c->stream, m->step, m->amax, m->ids);
    };
    if (m->mode & 1) {
        for (int i = 0; i < steps; i++) one();
    } else {
        auto it = m->graphs.find(slot);
        if (it == m->graphs.end()) {
            hipGraph_t g = nullptr;
            PS_CHECK(c, hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal));
            one();
            const hipError_t e = hipStreamEndCapture(c->stream, &g);
            if (e != hipSuccess) { if (g) (void)hipGraphDestroy(g); return seq_fail(c, std::string("seq_decode_greedy: graph capture failed: ") + hipGetErrorString(e)); }
            hipGraphExec_t ge = nullptr;
            const hipError_t e2 = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
            (void)hipGraphDestroy(g);
            if (e2 != hipSuccess) return seq_fail(c, std::string("seq_decode_greedy: graph instantiate failed: ") + hipGetErrorString(e2));
            it = m->graphs.emplace(slot, ge).first;
        }
        for (int i = 0; i < steps; i++) PS_CHECK(c, hipGraphLaunch(it->second, c->stream));
    }
    PS_CHECK(c, hipMemcpyAsync(out_ids, m->ids, (size_t)steps * 4, hipMemcpyDeviceToHost, c->stream));
    PS_CHECK(c, hipStreamSynchronize(c->stream));
    PS_CHECK(c, hipGetLastError());
    m->slot_pos[slot] += steps;
    return 0;
}

int ps_hip_seq_bench_kernel(ps_hip_seq *m, int which, int T, int reps, double *us, double *bytes, double *flops) {
    ps_hip_ctx *c = m->ctx;
    if (T <= 0 || T > m->d.max_batch || reps <= 0 || which < 0 || which > 3) return seq_fail(c, "seq_bench_kernel: bad argument");
    PS_CHECK(c, hipSetDevice(c->device));
    const bool moe = which >= 2;
    const int64_t W = m->d.width;
    auto embed_from = [&](int first) { // tokens first, first + 1, ... embedded as the input: a routing as spread as the router's rows make it
        std::vector<int32_t> ids((size_t)T);
        for (int i = 0; i < T; i++) ids[i] = (first + i) % m->d.vocab;
        if (hipMemcpyAsync(m->tokens, ids.data(), (size_t)T * 4, hipMemcpyHostToDevice, c->stream) != hipSuccess) return false;
        psk_embed(c->stream, m->d.embed, m->tokens, m->step, T, m->embed_scale, m->h, W);
        return hipStreamSynchronize(c->stream) == hipSuccess;
    };
    if (moe) {
        if (!embed_from(0)) return seq_fail(c, "seq_bench_kernel: embedding");
    } else {
        psk_fill(c->stream, m->h, 0.01f, (int64_t)m->d.max_batch * W);
    }
    std::vector<psk_dense_args> launches; // one per layer that has the matrix: every launch streams its own (cold) weights, as in a step
    double per_bytes = 0, per_flops = 0;
    for (const LayerPlan &P : m->L) {
        const bool is_moe = P.d.ff_kind == PS_FF_MOE_SWIGLU || P.d.ff_kind == PS_FF_MOE_RELU2;
        if (P.d.ff_kind == PS_FF_NONE || is_moe != moe) continue;
        psk_dense_args g;
        g.T = T; g.pack = m->pack; g.pack_bytes = m->pack_bytes;
        if (moe) {
            // the routing of this layer (all layers' launches below then reuse the LAST layer's routing: the same shapes and spread)
            const int top = P.d.top, S = T * top;
            const bool mv = T <= 8;
            const int rows = P.d.experts + P.d.moe_identity;
            std::vector<int32_t> sel((size_t)S);
            // (a few tokens: the first run of tokens none of whose choices is an identity expert, so that a mat-vec launch has its full work)
            for (int first = 0; first < (mv && P.d.moe_identity ? 64 : 1); first++) {
                if (first && !embed_from(first)) return seq_fail(c, "seq_bench_kernel: embedding");
                psk_moe_route(c->stream, m->h, W, P.d.router, P.d.shared_gate, rows, top, P.d.moe_norm_top, W, T, m->moe_sel, m->moe_wgt, m->moe_sg, P.d.moe_softmax,
                              P.d.moe_correction, P.d.moe_groups, P.d.moe_keep);
                PS_CHECK(c, hipMemcpyAsync(sel.data(), m->moe_sel, (size_t)S * 4, hipMemcpyDeviceToHost, c->stream));
                PS_CHECK(c, hipStreamSynchronize(c->stream));
                bool all_real = true;
                for (int32_t e : sel) all_real = all_real && e < P.d.experts;
                if (all_real) break;
            }
            if (!mv) psk_moe_plan(c->stream, m->moe_sel, S, rows, m->moe_seg, m->moe_list);
            g.groups = P.d.experts; g.g_sel = m->moe_sel;
            if (!mv) { g.g_seg = m->moe_seg; g.g_list = m->moe_list; }
            if (which == 2) {
                g.w = P.d.ff_up; g.a = m->h; g.lda = W; g.out = m->t4; g.ldo = P.d.ff; g.T = S; g.g_adiv = top;
                g.act = P.d.ff_kind == PS_FF_MOE_RELU2 ? PSD_ACT_RELU2 : PSD_ACT_SILU_PAIR;
                if (P.d.moe_weight_output) g.out_scale = m->moe_wgt;
                else g.g_scale = m->moe_wgt;
            } else {
                g.w = P.d.ff_down; g.a = m->t4; g.lda = P.d.ff; g.ldo = W;
                if (mv) { g.T = T; g.g_inner = top; g.out = m->y; }
                else { g.T = S; g.out = top == 1 ? m->y : m->moe_y; }
            }
            // what this routing makes a launch do: the slots that go to an expert with matrices (identity experts take none) and the matrices they touch
            std::vector<char> seen((size_t)P.d.experts, 0);
            int real = 0, used = 0;
            for (int32_t e : sel)
                if (e >= 0 && e < P.d.experts) { real++; if (!seen[e]) { seen[e] = 1; used++; } }
            per_bytes = (double)dense_bytes(g.w) / P.d.experts * used;
            per_flops = 2.0 * real * (double)(g.w->N / P.d.experts) * (double)g.w->K;
        } else if (which == 0) {
            g.w = P.d.ff_up; g.a = m->h; g.lda = m->d.width; g.out = m->t4; g.ldo = P.d.ff;
            if (P.d.ff_kind == PS_FF_DENSE_SWIGLU) g.act = PSD_ACT_SILU_PAIR;
            else if (P.d.ff_kind == PS_FF_DENSE_RELU_GLU) { g.act = PSD_ACT_RELU_PAIR; g.bias = P.d.ff_up_bias; }
            else { g.act = PSD_ACT_XIELU; g.act_p = P.act_p; g.act_q = P.act_q; }
        }
        else { g.w = P.d.ff_down; g.a = m->t4; g.lda = P.d.ff; g.out = m->y; g.ldo = m->d.width; }
        launches.push_back(g);
    }
    if (launches.empty()) return seq_fail(c, "seq_bench_kernel: no layer has a feed-forward");
    hipEvent_t e0, e1;
    PS_CHECK(c, hipEventCreate(&e0));
    PS_CHECK(c, hipEventCreate(&e1));
    for (auto &g : launches) psk_dense(c->stream, g); // warm-up (code objects, attributes)
    PS_CHECK(c, hipEventRecord(e0, c->stream));
    for (int r = 0; r < reps; r++)
        for (auto &g : launches) psk_dense(c->stream, g);
    PS_CHECK(c, hipEventRecord(e1, c->stream));
    PS_CHECK(c, hipEventSynchronize(e1));
    float ms = 0.f;
    PS_CHECK(c, hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *us = 1e3 * ms / ((double)reps * launches.size());
    *bytes = moe ? per_bytes : (double)dense_bytes(launches[0].w);
    *flops = moe ? per_flops : 2.0 * T * (double)launches[0].w->N * (double)launches[0].w->K;
    return 0;
}

} // extern "C"
