// dinilorn.cc — loading a Dinilorn folder, its retention mixer and its routed feed-forward inside Context (novorax.h describes the design, config_model.h the
// shared loader).
//
// A layer is x += norm(mixer(norm(x))), then x += norm(ff(norm(x))) - the layer loop of the sequential folder designs (novorax.cc run_layers_novorax) with all
// four norms filled.  The two attention mixers are the grouped-query attention of fidepel.cc with further switches (projection biases, the query multiplier by
// position, soft cap, distance-bucket bias, a zero sink, neighbour-pair rotation with banded frequencies, the window that keeps the first positions, two score
// maps per head); the retention mixer is new here: ONE projection [q ; k ; v ; g], the recurrence over the batch's segments from each sequence slot's state,
// the gated unit-RMS output, W_o.  The feed-forward reads its own norm, so its router rides with the shared expert's gate in a projection of its own; the
// routed and the shared expert are the ones of fidepel.cc in their gated, clamped form.  A looped span re-opens every pass but the first with the embedding
// rows added to the stream; each run owns its cache plane or its state set.
#include <cmath>

#include "config_model.h"

namespace mi355 {

void set_error(const char *fmt, ...);

#define DNL_TRY(expr)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess) {                                                                    \
            set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__);  \
            return e_;                                                                             \
        }                                                                                          \
    } while (0)

// radians per position of pair i of `dims` turning entries: base^(-2i / dims), made in double.  With a scaling object {factor, low, high, original}: a pair
// whose wavelength is below original / high keeps its frequency, above original / low it turns `factor` times slower, between the two the frequencies are
// blended linearly in original / wavelength.
static float *rot_table_banded(Bf16Loader &ld, double base, int dims, const Json &scaling, std::string &err) {
    std::vector<float> fr((size_t)std::max(dims / 2, 1), 0.0f);
    double factor = 1.0, low = 1.0, high = 1.0, orig = 1.0;
    const bool banded = scaling.is_object();
    if (banded) {
        factor = scaling["factor"].as_double(1.0); low = scaling["low"].as_double(1.0); high = scaling["high"].as_double(4.0); orig = scaling["original"].as_double(1.0);
        if (!(factor > 0.0) || !(low > 0.0) || !(high > low) || !(orig > 0.0)) { err = "configuration: rot.scaling needs factor > 0, 0 < low < high, original > 0"; return nullptr; }
    }
    for (int i = 0; i < dims / 2; i++) {
        double f = std::pow(base, -2.0 * i / dims);
        if (banded) {
            const double wl = 2.0 * M_PI / f;
            if (wl > orig / low) f = f / factor;
            else if (!(wl < orig / high)) {
                const double s = (orig / wl - low) / (high - low);
                f = (1.0 - s) * f / factor + s * f;
            }
        }
        fr[(size_t)i] = (float)f;
    }
    return (float *)ld.dev(fr.data(), fr.size() * 4);
}

// several [n_i] bf16 vectors (an empty name: n_i zeros) one behind the other, widened to f32
static float *vec_concat(Bf16Loader &ld, const std::vector<std::pair<std::string, int>> &parts) {
    std::vector<float> h;
    for (const auto &pr : parts) {
        if (pr.first.empty()) { h.insert(h.end(), (size_t)pr.second, 0.0f); continue; }
        const SafeTensor *t = ld.need(pr.first, "BF16", {pr.second});
        if (!t) return nullptr;
        const unsigned short *s = (const unsigned short *)t->data;
        for (int i = 0; i < pr.second; i++) h.push_back(Bf16Loader::widen(s[i]));
    }
    return (float *)ld.dev(h.data(), h.size() * 4);
}

// sum_i a[i] * b[i] of two [n] bf16 vectors, in f32
static bool vec_dot(Bf16Loader &ld, const std::string &a, const std::string &b, int n, float &out) {
    const SafeTensor *ta = ld.need(a, "BF16", {n}), *tb = ta ? ld.need(b, "BF16", {n}) : nullptr;
    if (!tb) return false;
    float s = 0.0f;
    for (int i = 0; i < n; i++) s += Bf16Loader::widen(((const unsigned short *)ta->data)[i]) * Bf16Loader::widen(((const unsigned short *)tb->data)[i]);
    out = s;
    return true;
}

Model *dinilorn_build(const Json &cfg, const std::string &dir, Bf16Loader &ld, std::string &err, int &status) {
    (void)dir;
    status = -102;
    Model *const m = ld.m;
    NovoraxModel &M = *m->nvx;
    M.design = "dinilorn";
    M.norm_off = 1.0f;
    M.loop_add_embed = true;
    const int W = (int)cfg["width"].as_int(), V = (int)cfg["vocab"].as_int();
    if (!cfg_positive(err, "width", W) || !cfg_positive(err, "vocab", V)) return nullptr;
    M.width = W; M.n_vocab = V;
    M.eps = (float)cfg["norm"]["eps"].as_double(1e-5);
    const Json &layers = cfg["layers"];
    if (!layers.is_array() || layers.size() == 0 || layers.size() > 1024) { err = "configuration: 'layers' must list 1 .. 1024 layers"; return nullptr; }
    const int nl = (int)layers.size();

    M.embed = ld.embedding("embed", V, W);
    M.head = ld.rows({{"head", V}}, W);
    M.final_norm = ld.vec("final.norm", W);
    std::vector<uint64_t> layer_active((size_t)nl, 0);          // weight bytes a token reads per run of the layer

    M.layers.resize((size_t)nl);
    for (int il = 0; il < nl && ld.err.empty(); il++) {
        const Json &lc = layers.at((size_t)il), &mx = lc["mixer"];
        NvxLayer &L = M.layers[(size_t)il];
        const std::string p = "l" + std::to_string(il) + ".", pm = p + "mix.";
        const std::string type = lc["type"].as_string();
        const std::string at = "configuration: layer " + std::to_string(il) + ": ";
        L.norm1 = ld.vec(p + "norm1", W);
        L.norm1b = ld.vec(p + "norm1b", W);
        L.heads = (int)mx["heads"].as_int(); L.kv_heads = (int)mx["kv_heads"].as_int(L.heads); L.dim = (int)mx["dim"].as_int(); L.vdim = (int)mx["vdim"].as_int(L.dim);
        if (!cfg_positive(err, "mixer.heads", L.heads, 4096) || !cfg_positive(err, "mixer.kv_heads", L.kv_heads, L.heads) || !cfg_positive(err, "mixer.dim", L.dim, 1 << 16) ||
            !cfg_positive(err, "mixer.vdim", L.vdim, 1 << 16)) return nullptr;
        if (L.heads % L.kv_heads != 0) { err = at + "mixer.heads must be a multiple of mixer.kv_heads"; return nullptr; }
        const int H = L.heads, G = L.kv_heads, D = L.dim, VD = L.vdim;
        const Json &rot = mx["rot"];
        L.rot_dims = rot.is_object() ? (int)rot["dims"].as_int(0) : 0;
        if (L.rot_dims > D || (L.rot_dims & 1) || L.rot_dims < 0) { err = at + "rot.dims must be even and at most mixer.dim"; return nullptr; }
        if (L.rot_dims > 0) {
            const double base = rot["base"].as_double(10000.0);
            if (!(base > 0.0)) { err = at + "rot.base must be positive"; return nullptr; }
            L.rot_freq = rot_table_banded(ld, base, L.rot_dims, type == "attention_2" ? rot["scaling"] : Json(), err);
            if (!err.empty()) return nullptr;
        }
        if (type == "retention") {
            L.type = NVX_RETENTION;
            L.kv_heads = H;
            if (!retention_shape_ok(D, VD)) { err = "retention: dim " + std::to_string(D) + " is beyond what the recurrence kernel keeps in registers (512)"; return nullptr; }
            const Json &dc = mx["decay"];
            if (!dc.is_array() || (int)dc.size() != H) { err = at + "mixer.decay must list one number per head"; return nullptr; }
            std::vector<float> dec((size_t)H);
            for (int h = 0; h < H; h++) dec[(size_t)h] = (float)dc.at((size_t)h).as_double(0.0);
            L.decay = (float *)ld.dev(dec.data(), dec.size() * 4);
            L.scale = (float)(1.0 / std::sqrt((double)D));
            L.proj = ld.rows({{pm + "q", H * D}, {pm + "k", H * D}, {pm + "v", H * VD}, {pm + "g", H * VD}}, W);
            L.off_g = 2 * H * D + H * VD;
            L.o = ld.rows({{pm + "o", W}}, H * VD);
        } else if (type == "attention" || type == "attention_2") {
            L.type = NVX_GQ;
            L.maps = type == "attention_2" ? 2 : 1;
            if (!gq_attn_shape_ok(H, G, D, VD)) { err = "attention: dim " + std::to_string(D) + " / vdim " + std::to_string(VD) + " is beyond what the attention kernel holds per lane (512)"; return nullptr; }
            L.scale = (float)mx["scale"].as_double(1.0);
            const int NQ = H * L.maps * D, NK = G * L.maps * D, NV = G * VD;
            L.off_gate = NQ + NK + NV;
            if (L.maps == 1) {
                L.rot_dims = 0; L.rot_freq = nullptr;           // (positions enter this attention through the multiplier and the bias only)
                L.softcap = (float)mx["softcap"].as_double(0.0);
                if (!(L.softcap >= 0.0f)) { err = at + "mixer.softcap must not be negative"; return nullptr; }
                const Json &qt = mx["q_temp"];
                if (qt.is_object()) {
                    L.q_temp_coef = (float)qt["coef"].as_double(0.0); L.q_temp_every = (float)qt["every"].as_double(0.0);
                    if (!(L.q_temp_every > 0.0f)) { err = at + "q_temp.every must be positive"; return nullptr; }
                }
                // distance d -> row of the bias table: one row per distance below B / 2, then rows spaced evenly in ln(d) up to bias_max (made in double; from
                // bias_max on every distance takes the last row)
                const int B = ld.rows_of(pm + "rel", H);
                if (B < 0) break;
                const int half = B / 2;
                const double far = mx["bias_max"].as_double(0.0);
                if (B > 1 && !(far > half && far <= (double)(1 << 24))) { err = at + "mixer.bias_max must lie above half the bias table's rows"; return nullptr; }
                L.rel = ld.rows_f32({{pm + "rel", B}}, H);
                L.rel_rows = B;
                L.n_dist = B > 1 ? (int)std::ceil(far) : 0;
                std::vector<int32_t> bk((size_t)std::max(L.n_dist, 1), 0);
                for (int n = 0; n < L.n_dist; n++)
                    bk[(size_t)n] = n < half ? n : (int32_t)std::min<double>(B - 1, half + std::floor(std::log((double)n / half) / std::log(far / half) * (B - half)));
                L.dist_bucket = (int32_t *)ld.dev(bk.data(), bk.size() * 4);
                std::vector<float> zero((size_t)H, 0.0f);           // one more term of score 0 in every head's softmax denominator
                L.sink = (float *)ld.dev(zero.data(), zero.size() * 4);
                L.proj = ld.rows({{pm + "q", NQ}, {pm + "k", NK}, {pm + "v", NV}, {pm + "g", H}}, W);
                L.proj_bias = vec_concat(ld, {{pm + "q.b", NQ}, {pm + "k.b", NK}, {pm + "v.b", NV}, {"", H}});
            } else {
                L.rot_neighbours = true;
                const Json &mask = mx["mask"];
                L.window = mask.is_object() ? (int)mask["size"].as_int(0) : 0;
                L.keep_first = mask.is_object() ? (int)mask["keep_first"].as_int(0) : 0;
                if (L.window < 0 || L.keep_first < 0) { err = at + "mask.size and mask.keep_first must not be negative"; return nullptr; }
                const double diff = mx["diff"].as_double(0.0);
                float d1 = 0.0f, d2 = 0.0f;
                if (!vec_dot(ld, pm + "lq1", pm + "lk1", D, d1) || !vec_dot(ld, pm + "lq2", pm + "lk2", D, d2)) break;
                L.map_lambda = expf(d1) - expf(d2) + (float)diff;
                L.map_mult = (float)(1.0 - diff);
                L.gate_per_entry = true;
                L.proj = ld.rows({{pm + "q", NQ}, {pm + "k", NK}, {pm + "v", NV}, {pm + "g", H * VD}}, W);
                L.proj_bias = vec_concat(ld, {{pm + "q.b", NQ}, {pm + "k.b", NK}, {pm + "v.b", NV}, {"", H * VD}});
                M.max_keep_first = std::max(M.max_keep_first, L.keep_first);
            }
            if (L.window > 0) M.max_window = std::max(M.max_window, L.window);
            L.o = ld.rows({{pm + "o", W}}, H * VD);
            L.o_bias = ld.vec(pm + "o.b", W);
            M.max_q = std::max(M.max_q, NQ);
        } else { err = at + "unknown type '" + type + "'"; return nullptr; }
        M.max_proj = std::max(M.max_proj, L.proj.N);
        M.max_att = std::max(M.max_att, H * L.maps * VD);
        layer_active[(size_t)il] = ((uint64_t)L.proj.N * W + (uint64_t)W * H * VD) * 2;

        const Json &mlp = lc["mlp"];
        if (mlp.is_object()) {
            const std::string pf = p + "mlp.";
            const std::string kind = mlp["kind"].as_string();
            if (kind != "moe") { err = at + "unknown mlp.kind '" + kind + "'"; return nullptr; }
            L.norm2 = ld.vec(p + "norm2", W);
            L.norm2b = ld.vec(p + "norm2b", W);
            L.ff_kind = NVX_FF_ROUTED;
            L.route_kind = NVX_ROUTE_SIGMOID_BIAS;
            const Json &rt = mlp["router"];
            L.ff = (int)mlp["expert"]["ff"].as_int();
            L.expert_limit = (float)mlp["expert"]["limit"].as_double(0.0);
            L.n_expert = (int)rt["experts"].as_int(); L.top = (int)rt["top"].as_int();
            if (!cfg_positive(err, "mlp.expert.ff", L.ff) || !cfg_positive(err, "mlp.router.experts", L.n_expert, MOE_ROUTE_MAX_EXPERTS) || !cfg_positive(err, "mlp.router.top", L.top, L.n_expert)) return nullptr;
            if (!(L.expert_limit > 0.0f)) { err = at + "mlp.expert.limit must be positive"; return nullptr; }
            const Json &gr = rt["groups"];
            L.n_group = gr.is_object() ? (int)gr["count"].as_int(1) : 1;
            L.group_keep = gr.is_object() ? (int)gr["keep"].as_int(L.n_group) : 1;
            if (!cfg_positive(err, "mlp.router.groups.count", L.n_group, L.n_expert) || !cfg_positive(err, "mlp.router.groups.keep", L.group_keep, L.n_group)) return nullptr;
            if (L.n_expert % L.n_group != 0) { err = at + "mlp.router.experts must be a multiple of groups.count"; return nullptr; }
            if ((long long)L.group_keep * (L.n_expert / L.n_group) < L.top) { err = at + "the groups kept hold fewer than router.top experts"; return nullptr; }
            std::vector<std::pair<std::string, int>> g, u, d;
            for (int e = 0; e < L.n_expert; e++) {
                const std::string pe = pf + "e" + std::to_string(e) + ".";
                g.push_back({pe + "gate", L.ff}); u.push_back({pe + "up", L.ff}); d.push_back({pe + "down", W});
            }
            L.e_gate = ld.rows(g, W); L.e_up = ld.rows(u, W); L.e_down = ld.rows(d, L.ff);
            L.route_bias = ld.vec(pf + "correction", L.n_expert);
            std::vector<std::pair<std::string, int>> route = {{pf + "router", L.n_expert}};
            layer_active[(size_t)il] += ((uint64_t)L.n_expert * W + (uint64_t)L.top * 3 * L.ff * W) * 2;
            const Json &sh = mlp["shared"];
            if (sh.is_object()) {
                L.shared_ff = (int)sh["ff"].as_int();
                L.shared_limit = (float)sh["limit"].as_double(0.0);
                if (!cfg_positive(err, "mlp.shared.ff", L.shared_ff)) return nullptr;
                if (!(L.shared_limit > 0.0f)) { err = at + "mlp.shared.limit must be positive"; return nullptr; }
                L.s_gate = ld.rows({{pf + "shared.gate", L.shared_ff}}, W);
                L.s_up = ld.rows({{pf + "shared.up", L.shared_ff}}, W);
                L.s_down = ld.rows({{pf + "shared.down", W}}, L.shared_ff);
                route.push_back({pf + "shared.sg", 1});
                L.off_sg = L.n_expert;
                M.max_shared_ff = std::max(M.max_shared_ff, L.shared_ff);
                layer_active[(size_t)il] += ((uint64_t)3 * L.shared_ff * W + W) * 2;
            }
            L.route = ld.rows(route, W);
            M.max_proj = std::max(M.max_proj, L.route.N);
            M.max_top = std::max(M.max_top, L.top);
            M.max_expert = std::max(M.max_expert, L.n_expert);
            M.max_ff = std::max(M.max_ff, L.ff);
        }
    }
    if (!ld.err.empty()) { err = ld.err; return nullptr; }

    // the order of layer runs: every run owns a cache plane (attention) or a state set (retention); `pass` marks the first layer of each pass of the span
    int times = 0;
    uint64_t active_bytes = ((uint64_t)V * W + W) * 2;
    if (!cfg_layer_runs(cfg["loop"], nl, err, times, [&](int il, int pass) {
            NvxRun r; r.layer = il; r.pass = pass;
            r.plane = M.layers[(size_t)il].type == NVX_GQ ? M.n_cache_runs++ : M.n_state_runs++;
            M.runs.push_back(r);
            active_bytes += layer_active[(size_t)il];
        })) return nullptr;

    HParams &hp = m->hp;
    hp.arch = "dinilorn";
    hp.n_embd = W; hp.n_vocab = V; hp.n_vocab_local = V; hp.n_layer = nl; hp.n_layer_runs = (int)M.runs.size();
    hp.n_head = M.layers[0].heads; hp.n_head_kv = M.layers[0].kv_heads; hp.head_dim = M.layers[0].dim; hp.eps = M.eps;
    hp.n_head_full = hp.n_head; hp.n_head_kv_full = hp.n_head_kv;
    hp.n_expert = M.max_expert; hp.n_expert_used = M.max_top;
    m->bytes_per_token = active_bytes;
    m->desc = "dinilorn " + std::to_string(nl) + " layers (" + std::to_string(M.runs.size()) + " runs) width " + std::to_string(W) + " BF16";
    status = 0;
    return m;
}

// the retention mixer of one layer run over the micro-batch: -> nvx_y_
hipError_t Context::nvx_retention_mixer(const NvxLayer &L, const NvxRun &r, int T) {
    const NovoraxModel &M = *model->nvx;
    const int W = M.width, H = L.heads, D = L.dim, VD = L.vdim, LD_P = L.proj.N;
    DNL_TRY(nvx_linear(L.proj, x_, W, T, nvx_a_, LD_P, MMB_STORE, nullptr, 1.0f, L.norm1));
    RetentionArgs ra{};
    ra.p = nvx_a_; ra.ld_p = LD_P; ra.o = nvx_o_; ra.ld_o = H * VD; ra.H = H; ra.D = D; ra.VD = VD;
    ra.decay = L.decay; ra.rot_dims = L.rot_dims; ra.rot_freq = L.rot_freq; ra.k_scale = L.scale; ra.tok_pos = d_pos_;
    ra.S = nvx_S_[(size_t)r.plane];
    const size_t TU = cp.n_ubatch;
    for (const auto &wv : nvx_waves_) {
        ra.seg_start = d_seg_ + wv.first; ra.seg_len = d_seg_ + TU + wv.first; ra.seg_slot = d_seg_ + 2 * TU + wv.first; ra.n_seg = wv.second;
        DNL_TRY(launch_retention_scan(ra, stream_));
    }
    DNL_TRY(launch_mlstm_out(nvx_o_, H * VD, nvx_a_, LD_P, L.off_g, nullptr, T, H, VD, M.eps, nvx_att_, H * VD, stream_, 0, MLSTM_GATE_SILU));
    DNL_TRY(nvx_linear(L.o, nvx_att_, H * VD, T, nvx_y_, W));
    prof_mark("retention");
    return hipSuccess;
}

// a routed feed-forward that reads its own norm: sum_j w_j expert_j(h) + sigmoid(gate) shared(h), h = norm2(x); the sum, the norm behind it and the residual
// add are one launch (x_ updated, *closed = true) where the row fits its LDS, else the sum lands in nvx_y_.  The shared expert touches no buffer of the routed
// ones until the sum: in batches it runs on a side stream (fork behind the norm, join in front of the sum)
hipError_t Context::nvx_routed_feed_forward(const NvxLayer &L, int T, bool *closed) {
    const NovoraxModel &M = *model->nvx;
    const int W = M.width;
    // up to MMB_VEC_ROWS rows every reader norms the stream itself (no launch for the norm); batches - and grouped expert batches, which gather normed rows -
    // norm once into xn_
    const bool grouped = nvx_routed_as_groups(L, T);
    const float *h = x_, *pn = L.norm2;
    if (T > MMB_VEC_ROWS || grouped) {
        DNL_TRY(launch_rmsnorm_f32(x_, W, L.norm2, M.norm_off, nullptr, xn_, W, W, T, M.eps, stream_));
        h = xn_; pn = nullptr;
    }
    // (steps of a few rows keep one stream: their launches are too short for the fork and the join to pay - measured)
    const bool shared = L.shared_ff > 0, fork = nvx_fork_ok_ && shared && !profile_ && T > MMB_VEC_ROWS;
    hipStream_t const main_stream = stream_;
    struct Back { hipStream_t &s; hipStream_t v; ~Back() { s = v; } } back{stream_, main_stream};   // (every helper launches on stream_)
    if (fork) {
        DNL_TRY(hipEventRecord(nvx_fork_ev_, main_stream));
        DNL_TRY(hipStreamWaitEvent(nvx_side_[0], nvx_fork_ev_, 0));
        stream_ = nvx_side_[0];
        DNL_TRY(nvx_shared_expert(L, h, pn, T));
        DNL_TRY(hipEventRecord(nvx_join_ev_[0], nvx_side_[0]));
        stream_ = main_stream;
    }
    DNL_TRY(nvx_linear(L.route, h, W, T, nvx_a_, L.route.N, MMB_STORE, nullptr, 1.0f, pn));
    DNL_TRY(nvx_routed_experts(L, h, pn, T, nvx_a_, L.route.N));
    if (fork) DNL_TRY(hipStreamWaitEvent(main_stream, nvx_join_ev_[0], 0));
    else if (shared) DNL_TRY(nvx_shared_expert(L, h, pn, T));
    const int32_t *slot_of = grouped ? nvx_slot_ : nullptr;
    const float *sb = shared ? nvx_ys_ : nullptr, *sg = shared && L.off_sg >= 0 ? nvx_a_ + L.off_sg : nullptr;
    if (closed && L.norm2b && W <= MOE_COMBINE_NORM_MAX_E && L.top <= MOE_COMBINE_NORM_MAX_K) {
        DNL_TRY(launch_moe_weighted_combine_norm(x_, nvx_yg_, nvx_rw_, slot_of, sb, sg, L.route.N, L.norm2b, M.norm_off, M.eps, T, W, L.top, stream_));
        *closed = true;
    } else DNL_TRY(launch_moe_weighted_combine(nvx_y_, nvx_yg_, nvx_rw_, slot_of, sb, sg, L.route.N, T, W, L.top, stream_));
    prof_mark("expert_sum_norm");
    return hipSuccess;
}

}  // namespace mi355
