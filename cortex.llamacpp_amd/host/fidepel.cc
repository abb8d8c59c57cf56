// fidepel.cc — loading a Fidepel folder and running its blocks inside Context (novorax.h describes the design, config_model.h the shared loader).
//
// A block is h = norm(x), x += m * (attention(h) + experts(h) + shared(h)).  The five things that read h as a matrix product - q, k, v, the per-head output
// gate and the router - are ONE projection [q ; k ; v ; g ; router]; the cell table, cache planes, staging block, scan bounds, graphs and output path are the
// ones the other folder design uses (novorax.cc).
#include <cmath>

#include "config_model.h"

namespace mi355 {

void set_error(const char *fmt, ...);

#define FDP_TRY(expr)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess) {                                                                    \
            set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__);  \
            return e_;                                                                             \
        }                                                                                          \
    } while (0)

Model *fidepel_build(const Json &cfg, const std::string &dir, Bf16Loader &ld, std::string &err, int &status) {
    (void)dir;
    status = -102;
    Model *const m = ld.m;
    NovoraxModel &M = *m->nvx;
    M.design = "fidepel";
    M.parallel_block = true;
    M.norm_off = 0.0f;
    const int W = (int)cfg["width"].as_int(), V = (int)cfg["vocab"].as_int();
    if (!cfg_positive(err, "width", W) || !cfg_positive(err, "vocab", V)) return nullptr;
    M.width = W; M.n_vocab = V;
    M.eps = (float)cfg["norm"]["eps"].as_double(1e-6);
    M.residual_mult = (float)cfg["residual_mult"].as_double(1.0);
    const Json &layers = cfg["layers"];
    if (!layers.is_array() || layers.size() == 0 || layers.size() > 1024) { err = "configuration: 'layers' must list 1 .. 1024 layers"; return nullptr; }
    const int nl = (int)layers.size();

    M.embed = ld.embedding("embed", V, W);
    M.head = ld.rows({{"head", V}}, W);
    M.final_norm = ld.scalar_as_vec("final.norm", W);

    bool all_windowed = true;
    uint64_t active_bytes = ((uint64_t)V * W + W) * 2;          // what one token reads of the weights: head and a table row, then per run the block's always-read part
    std::vector<uint64_t> layer_active((size_t)nl, 0);
    M.layers.resize((size_t)nl);
    for (int il = 0; il < nl && ld.err.empty(); il++) {
        const Json &lc = layers.at((size_t)il), &mx = lc["mixer"];
        NvxLayer &L = M.layers[(size_t)il];
        const std::string p = "l" + std::to_string(il) + ".", pm = p + "mix.";
        const std::string type = lc["type"].as_string();
        if (type != "attention") { err = "configuration: layer " + std::to_string(il) + " has unknown type '" + type + "'"; return nullptr; }
        L.type = NVX_GQ;
        L.norm1 = ld.scalar_as_vec(p + "norm1", W);
        L.heads = (int)mx["heads"].as_int(); L.kv_heads = (int)mx["kv_heads"].as_int(L.heads); L.dim = (int)mx["dim"].as_int(); L.vdim = (int)mx["vdim"].as_int(L.dim);
        if (!cfg_positive(err, "mixer.heads", L.heads, 4096) || !cfg_positive(err, "mixer.kv_heads", L.kv_heads, L.heads) || !cfg_positive(err, "mixer.dim", L.dim, 1 << 16) ||
            !cfg_positive(err, "mixer.vdim", L.vdim, 1 << 16)) return nullptr;
        if (L.heads % L.kv_heads != 0) { err = "configuration: mixer.heads must be a multiple of mixer.kv_heads"; return nullptr; }
        if (!gq_attn_shape_ok(L.heads, L.kv_heads, L.dim, L.vdim)) { err = "attention: dim " + std::to_string(L.dim) + " / vdim " + std::to_string(L.vdim) + " is beyond what the attention kernel holds per lane (512)"; return nullptr; }
        const int H = L.heads, G = L.kv_heads;
        L.scale = (float)mx["scale"].as_double(1.0);
        const Json &mask = mx["mask"];
        L.window = mask.is_object() ? (int)mask["size"].as_int(0) : 0;
        if (L.window < 0) L.window = 0;
        if (L.window == 0) all_windowed = false;
        M.max_window = std::max(M.max_window, L.window);
        const Json &rot = mx["rot"];
        L.rot_dims = rot.is_object() ? (int)rot["dims"].as_int(0) : 0;
        if (L.rot_dims > L.dim || (L.rot_dims & 1) || L.rot_dims < 0) { err = "configuration: rot.dims must be even and at most mixer.dim"; return nullptr; }
        if (L.rot_dims > 0) {
            // radians per position of pair i: base^(-2i / dims), every one divided by the linear scaling factor
            const int half = L.rot_dims / 2;
            const double base = rot["base"].as_double(10000.0);
            const Json &scg = rot["scaling"];
            const double factor = scg.is_object() ? scg["factor"].as_double(1.0) : 1.0;
            if (!(factor > 0.0) || !(base > 0.0)) { err = "configuration: rot.base and rot.scaling.factor must be positive"; return nullptr; }
            std::vector<float> fr((size_t)half);
            for (int i = 0; i < half; i++) fr[(size_t)i] = (float)(std::pow(base, -2.0 * i / L.rot_dims) / factor);
            L.rot_freq = (float *)ld.dev(fr.data(), fr.size() * 4);
        }
        L.q_norm = ld.vec(pm + "q.norm", H * L.dim);
        L.k_norm = ld.vec(pm + "k.norm", G * L.dim);
        L.head_scale = ld.vec(pm + "temp", H);
        L.o = ld.rows({{pm + "o", W}}, H * L.vdim);
        std::vector<std::pair<std::string, int>> proj = {{pm + "q", H * L.dim}, {pm + "k", G * L.dim}, {pm + "v", G * L.vdim}, {pm + "g", H}};
        L.off_gate = H * L.dim + G * L.dim + G * L.vdim;
        layer_active[(size_t)il] = ((uint64_t)(L.off_gate + H) * W + (uint64_t)W * H * L.vdim) * 2;

        const Json &mlp = lc["mlp"];
        if (mlp.is_object()) {
            const std::string pf = p + "mlp.";
            const std::string kind = mlp["kind"].as_string();
            if (kind != "moe") { err = "configuration: layer " + std::to_string(il) + " has unknown mlp.kind '" + kind + "'"; return nullptr; }
            L.ff_kind = NVX_FF_ROUTED;
            const Json &rt = mlp["router"];
            L.ff = (int)mlp["expert"]["ff"].as_int();
            L.n_expert = (int)rt["experts"].as_int(); L.top = (int)rt["top"].as_int();
            if (!cfg_positive(err, "mlp.expert.ff", L.ff) || !cfg_positive(err, "mlp.router.experts", L.n_expert, MOE_ROUTE_MAX_EXPERTS) || !cfg_positive(err, "mlp.router.top", L.top, L.n_expert)) return nullptr;
            L.router_scale = (float)rt["scale"].as_double(1.0);
            const Json &gr = rt["groups"];
            L.n_group = gr.is_object() ? (int)gr["count"].as_int(1) : 1;
            L.group_keep = gr.is_object() ? (int)gr["keep"].as_int(L.n_group) : 1;
            if (!cfg_positive(err, "mlp.router.groups.count", L.n_group, L.n_expert) || !cfg_positive(err, "mlp.router.groups.keep", L.group_keep, L.n_group)) return nullptr;
            if (L.n_expert % L.n_group != 0) { err = "configuration: mlp.router.experts must be a multiple of groups.count"; return nullptr; }
            if ((long long)L.group_keep * (L.n_expert / L.n_group) < L.top) { err = "configuration: the groups kept hold fewer than router.top experts"; return nullptr; }
            std::vector<std::pair<std::string, int>> u, d;
            for (int e = 0; e < L.n_expert; e++) {
                const std::string pe = pf + "e" + std::to_string(e) + ".";
                u.push_back({pe + "up", L.ff}); d.push_back({pe + "down", W});
            }
            L.e_up = ld.rows(u, W); L.e_down = ld.rows(d, L.ff);
            proj.push_back({pf + "router", L.n_expert});
            L.off_router = L.off_gate + H;
            layer_active[(size_t)il] += ((uint64_t)L.n_expert * W + (uint64_t)L.top * 2 * L.ff * W) * 2;
            const Json &sh = mlp["shared"];
            if (sh.is_object()) {
                L.shared_ff = (int)sh["ff"].as_int();
                if (!cfg_positive(err, "mlp.shared.ff", L.shared_ff)) return nullptr;
                L.s_up = ld.rows({{pf + "shared.up", L.shared_ff}}, W);
                L.s_down = ld.rows({{pf + "shared.down", W}}, L.shared_ff);
                M.max_shared_ff = std::max(M.max_shared_ff, L.shared_ff);
                layer_active[(size_t)il] += (uint64_t)2 * L.shared_ff * W * 2;
            }
            M.max_top = std::max(M.max_top, L.top);
            M.max_expert = std::max(M.max_expert, L.n_expert);
            M.max_ff = std::max(M.max_ff, L.ff);
        }
        L.proj = ld.rows(proj, W);
        M.max_proj = std::max(M.max_proj, L.proj.N);
        M.max_q = std::max(M.max_q, H * L.dim);
        M.max_att = std::max(M.max_att, H * L.vdim);
    }
    if (!ld.err.empty()) { err = ld.err; return nullptr; }
    if (!all_windowed) M.max_window = 0;

    // the order of layer runs: nothing happens between the passes of the looped span, each run owns a cache plane
    int times = 0;
    if (!cfg_layer_runs(cfg["loop"], nl, err, times, [&](int il, int) {
            NvxRun r; r.layer = il; r.pass = -1; r.plane = M.n_cache_runs++;
            M.runs.push_back(r);
            active_bytes += layer_active[(size_t)il];
        })) return nullptr;

    HParams &hp = m->hp;
    hp.arch = "fidepel";
    hp.n_embd = W; hp.n_vocab = V; hp.n_vocab_local = V; hp.n_layer = nl; hp.n_layer_runs = (int)M.runs.size();
    hp.n_head = M.layers[0].heads; hp.n_head_kv = M.layers[0].kv_heads; hp.head_dim = M.layers[0].dim; hp.eps = M.eps;
    hp.n_head_full = hp.n_head; hp.n_head_kv_full = hp.n_head_kv;
    hp.n_expert = M.max_expert; hp.n_expert_used = M.max_top;
    m->bytes_per_token = active_bytes;
    m->desc = "fidepel " + std::to_string(nl) + " layers (" + std::to_string(M.runs.size()) + " runs) width " + std::to_string(W) + " BF16";
    status = 0;
    return m;
}

// ------------------------------------------------------------------------------------------ the block
// from this many (token, rank) pairs on, the pairs are grouped by expert and every expert runs its rows as one batch (launch_moe_group holds the pair list in
// LDS and serves up to 64 experts); fewer pairs read their experts' rows directly
bool nvx_routed_as_groups(const NvxLayer &L, int T) {
    return L.ff_kind == NVX_FF_ROUTED && T * L.top > 32 && L.n_expert <= 64 && (size_t)T * L.top * 4 <= 60 * 1024;
}

// behind the block projection (nvx_a_): queries prepared, keys and values stored, attention, output projection -> nvx_y_.  With several score maps per head
// every (head, map) pair runs as a query head of its own; launch_gq_maps_out joins the maps in front of the output projection.
hipError_t Context::nvx_gq_attention(const NvxLayer &L, const NvxRun &r, int T) {
    const NovoraxModel &M = *model->nvx;
    const int W = M.width, G = L.kv_heads, LD_P = L.proj.N, maps = L.maps > 1 ? L.maps : 1;
    const int H = L.heads * maps;                               // query heads as the kernels count them
    float *cache = nvx_cache_[(size_t)r.plane];
    GqPrepArgs pa{};
    pa.p = nvx_a_; pa.ld_p = LD_P; pa.T = T; pa.H = H; pa.G = G; pa.dim = L.dim; pa.vdim = L.vdim;
    pa.wq_norm = L.q_norm; pa.wk_norm = L.k_norm; pa.eps = M.eps; pa.rot_dims = L.rot_dims; pa.rot_freq = L.rot_freq;
    pa.norm_per_head = L.qk_norm_per_head ? 1 : 0; pa.v_rot_freq = L.v_rot_freq; pa.v_cs = L.v_rot_freq ? nvx_vcs_ : nullptr;
    pa.q_scale = L.scale; pa.head_scale = L.head_scale; pa.tok_pos = d_pos_; pa.tok_cell = d_cell_;
    pa.maps = maps; pa.rot_neighbours = L.rot_neighbours ? 1 : 0; pa.q_temp_coef = L.q_temp_coef; pa.q_temp_every = L.q_temp_every;
    pa.q = nvx_q_; pa.ld_q = H * L.dim; pa.cache = cache;
    FDP_TRY(launch_gq_prep(pa, stream_));
    GqAttnArgs aa{};
    aa.q = nvx_q_; aa.ld_q = H * L.dim; aa.out = maps > 1 ? nvx_o_ : nvx_att_; aa.ld_out = H * L.vdim; aa.T = T; aa.H = H; aa.G = G; aa.dim = L.dim; aa.vdim = L.vdim;
    aa.maps = maps; aa.keep_first = L.keep_first; aa.rel = L.rel; aa.dist_bucket = L.dist_bucket; aa.n_dist = L.n_dist; aa.rel_rows = L.rel_rows;
    aa.cache = cache; aa.cell_pos = d_cell_pos_; aa.cell_seq = d_cell_seq_; aa.tok_pos = d_pos_; aa.tok_seq = d_seq_; aa.n_kv_dev = d_nkv_;
    aa.window = L.window; aa.sink = L.sink; aa.gate = L.off_gate >= 0 && !L.gate_per_entry ? nvx_a_ + L.off_gate : nullptr; aa.ld_gate = LD_P;
    aa.softcap = L.softcap; aa.v_cs = L.v_rot_freq ? nvx_vcs_ : nullptr;
    aa.tok_hi = d_seg_ + 3 * (size_t)cp.n_ubatch;
    aa.tok_lo = M.max_window > 0 && L.window > 0 ? d_seg_ + 4 * (size_t)cp.n_ubatch : nullptr;
    aa.part = nvx_part_; aa.part_floats = nvx_part_floats_; aa.n_kv_hint = n_kv_;
    aa.splits = (long long)T * H <= LATENT_ATTN_SPLIT_MAX_PAIRS ? LATENT_ATTN_SPLITS : 1;
    FDP_TRY(launch_gq_attn(aa, stream_));
    if (maps == 2)
        FDP_TRY(launch_gq_maps_out(nvx_o_, H * L.vdim, L.gate_per_entry ? nvx_a_ + L.off_gate : nullptr, LD_P, T, L.heads, L.vdim, L.map_lambda, L.map_mult, M.eps,
                                   nvx_att_, L.heads * L.vdim, stream_));
    else if (maps != 1) return hipErrorInvalidValue;
    FDP_TRY(nvx_linear(L.o, nvx_att_, L.heads * L.vdim, T, nvx_y_, W, MMB_STORE, nullptr, 1.0f, nullptr, L.o_bias));
    prof_mark("gq_attention");
    return hipSuccess;
}

// the router's logits -> experts and weights; the routed experts' rows end in nvx_yg_ (row(t, j): nvx_slot_ when grouped).  Experts are relu^2 (e_up alone)
// or the clamped gated form (e_gate set)
hipError_t Context::nvx_routed_experts(const NvxLayer &L, const float *h, const float *pn, int T, const float *z, int ld_z) {
    const NovoraxModel &M = *model->nvx;
    const int W = M.width, k = L.top, NE = L.n_expert, P = T * k;
    if (L.route_kind == NVX_ROUTE_SIGMOID_BIAS) FDP_TRY(launch_moe_route_sigmoid_bias(z, ld_z, L.route_bias, T, NE, k, L.n_group, L.group_keep, nvx_ids_, nvx_rw_, stream_));
    else FDP_TRY(launch_moe_route_groups(z, ld_z, T, NE, k, L.n_group, L.group_keep, L.router_scale, nvx_ids_, nvx_rw_, stream_));
    MMBArgs u;
    u.w = L.e_up.w; u.ldw = W; u.N = L.ff; u.K = W; u.epi = MMB_RELU2; u.f32 = cp.exact_f32 ? 1 : 0; u.w_zs = (long long)L.ff * W;
    if (L.e_gate.w) { u.w = L.e_gate.w; u.w2 = L.e_up.w; u.epi = MMB_CLAMP_SWIGLU; u.epi_limit = L.expert_limit; }
    u.y = nvx_ff_; u.ldy = L.ff;
    MMBArgs d;
    d.w = L.e_down.w; d.ldw = L.ff; d.N = W; d.K = L.ff; d.f32 = u.f32; d.w_zs = (long long)W * L.ff;
    d.x = nvx_ff_; d.ldx = L.ff; d.y = nvx_yg_; d.ldy = W;
    if (nvx_routed_as_groups(L, T)) {
        // every expert sees its (token, rank) pairs as one batch of rows: counting sort by expert, gather, two grouped products
        FDP_TRY(launch_moe_group(nvx_ids_, T, k, NE, nvx_meta_, nvx_slot_, nvx_tokof_, stream_));
        FDP_TRY(launch_gather_rows_f32(h, nvx_tokof_, P, W, nvx_xg_, stream_));
        u.x = nvx_xg_; u.ldx = W; u.T = P; u.nz = NE; u.meta = nvx_meta_;
        d.T = P; d.nz = NE; d.meta = nvx_meta_;
    } else {
        // a few tokens: one product per (token, rank) pair against the weights the pair picked
        u.x = h; u.ldx = W; u.T = 1; u.nz = P; u.sel = nvx_ids_; u.sel_div = k;
        if (pn) { u.pn_w = pn; u.pn_off = M.norm_off; u.pn_eps = M.eps; }
        d.T = 1; d.nz = P; d.sel = nvx_ids_; d.sel_div = 1;
    }
    FDP_TRY(launch_mmb(u, stream_));
    FDP_TRY(launch_mmb(d, stream_));
    prof_mark("routed_experts");
    return hipSuccess;
}

hipError_t Context::nvx_shared_expert(const NvxLayer &L, const float *h, const float *pn, int T) {
    const int W = model->nvx->width;
    if (L.s_gate.w) FDP_TRY(nvx_linear(L.s_gate, h, W, T, nvx_sh_, L.shared_ff, MMB_CLAMP_SWIGLU, &L.s_up, 1.0f, pn, nullptr, L.shared_limit));
    else FDP_TRY(nvx_linear(L.s_up, h, W, T, nvx_sh_, L.shared_ff, MMB_RELU2, nullptr, 1.0f, pn));
    FDP_TRY(nvx_linear(L.s_down, nvx_sh_, L.shared_ff, T, nvx_ys_, W));
    prof_mark("shared_expert");
    return hipSuccess;
}

hipError_t Context::nvx_parallel_block(const NvxLayer &L, const NvxRun &r, int T) {
    const NovoraxModel &M = *model->nvx;
    const int W = M.width;
    // up to MMB_VEC_ROWS rows every reader norms the stream itself (no launch for the norm); batches norm once into xn_.  A grouped expert batch gathers
    // normed rows, so it needs xn_ too - with top >= 3 that starts below MMB_VEC_ROWS rows
    const bool grouped = nvx_routed_as_groups(L, T);
    const bool fuse_norm = T <= MMB_VEC_ROWS && !grouped;
    const float *h = x_, *pn = L.norm1;
    if (!fuse_norm) {
        FDP_TRY(launch_rmsnorm_f32(x_, W, L.norm1, M.norm_off, nullptr, xn_, W, W, T, M.eps, stream_));
        h = xn_; pn = nullptr;
    }
    if (L.type != NVX_GQ) return hipErrorInvalidValue;
    const bool routed = L.ff_kind == NVX_FF_ROUTED, shared = routed && L.shared_ff > 0;
    if (!routed && L.ff_kind != NVX_FF_NONE) return hipErrorInvalidValue;
    // h: the rows every sublayer reads - the normed stream (pn == nullptr), or the stream itself with the norm weight pn for the launches that norm their
    // few rows on the way in.  One projection [q ; k ; v ; g ; router] for all of them
    FDP_TRY(nvx_linear(L.proj, h, W, T, nvx_a_, L.proj.N, MMB_STORE, nullptr, 1.0f, pn));
    // behind it the attention, the routed experts and the shared expert touch no buffer of each other until the closing sum: the two feed-forward branches
    // go to side streams (events only order them; a profile run keeps one stream so that its marks bracket whole sublayers)
    const bool fork = nvx_fork_ok_ && routed && !profile_;
    hipStream_t const main_stream = stream_;
    struct Back { hipStream_t &s; hipStream_t v; ~Back() { s = v; } } back{stream_, main_stream};   // (every helper launches on stream_)
    if (fork) {
        FDP_TRY(hipEventRecord(nvx_fork_ev_, main_stream));
        FDP_TRY(hipStreamWaitEvent(nvx_side_[0], nvx_fork_ev_, 0));
        stream_ = nvx_side_[0];
        FDP_TRY(nvx_routed_experts(L, h, pn, T, nvx_a_ + L.off_router, L.proj.N));
        FDP_TRY(hipEventRecord(nvx_join_ev_[0], nvx_side_[0]));
        if (shared) {
            FDP_TRY(hipStreamWaitEvent(nvx_side_[1], nvx_fork_ev_, 0));
            stream_ = nvx_side_[1];
            FDP_TRY(nvx_shared_expert(L, h, pn, T));
            FDP_TRY(hipEventRecord(nvx_join_ev_[1], nvx_side_[1]));
        }
        stream_ = main_stream;
    }
    FDP_TRY(nvx_gq_attention(L, r, T));
    if (fork) {
        FDP_TRY(hipStreamWaitEvent(main_stream, nvx_join_ev_[0], 0));
        if (shared) FDP_TRY(hipStreamWaitEvent(main_stream, nvx_join_ev_[1], 0));
    } else if (routed) {
        FDP_TRY(nvx_routed_experts(L, h, pn, T, nvx_a_ + L.off_router, L.proj.N));
        if (shared) FDP_TRY(nvx_shared_expert(L, h, pn, T));
    }
    FDP_TRY(launch_block_combine(x_, nvx_y_, shared ? nvx_ys_ : nullptr, nvx_yg_, nvx_rw_, routed && grouped ? nvx_slot_ : nullptr, T, W,
                                 routed ? L.top : 0, M.residual_mult, stream_));
    return hipSuccess;
}

}  // namespace mi355
