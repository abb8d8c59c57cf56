// tuterax.cc — loading a Tuterax folder and running its delta-rule mixers inside Context (novorax.h describes the design, config_model.h the shared loader).
//
// A layer is x += norm(mixer(x)), then x += norm(ff(x)): the sublayers read the stream itself, so the loader leaves the norms in front of the sublayers empty
// and fills the ones behind them - the layer loop, the cell table, cache planes, state slots, segment lists, graphs and the output path are the ones the other
// folder designs use (novorax.cc).  The attention mixer is the grouped-query attention of fidepel.cc with per-head query / key norms, a soft cap, a sink and
// turned values switched on; the delta-rule mixer is new here: ONE projection [q ; k ; v ; beta ; decay ; gate] (the per-channel form: [.. ; a1 ; g1] and a
// second, low-rank step), the convolution / gate preparation, the recurrence over the batch's segments, the gated unit-RMS output, W_o.
#include <cmath>

#include "config_model.h"

namespace mi355 {

void set_error(const char *fmt, ...);

#define TTX_TRY(expr)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess) {                                                                    \
            set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__);  \
            return e_;                                                                             \
        }                                                                                          \
    } while (0)

// radians per position of pair i of `dims` turning entries: base^(-2i / dims), made in double
static float *rot_table(Bf16Loader &ld, double base, int dims) {
    std::vector<float> fr((size_t)std::max(dims / 2, 1), 0.0f);
    for (int i = 0; i < dims / 2; i++) fr[(size_t)i] = (float)std::pow(base, -2.0 * i / dims);
    return (float *)ld.dev(fr.data(), fr.size() * 4);
}

Model *tuterax_build(const Json &cfg, const std::string &dir, Bf16Loader &ld, std::string &err, int &status) {
    (void)dir;
    status = -102;
    Model *const m = ld.m;
    NovoraxModel &M = *m->nvx;
    M.design = "tuterax";
    M.norm_off = 1.0f;
    const int W = (int)cfg["width"].as_int(), V = (int)cfg["vocab"].as_int();
    if (!cfg_positive(err, "width", W) || !cfg_positive(err, "vocab", V)) return nullptr;
    M.width = W; M.n_vocab = V;
    M.eps = (float)cfg["norm"]["eps"].as_double(1e-5);
    M.embed_scale = (float)cfg["embedding"]["scale"].as_double(1.0);
    const Json &layers = cfg["layers"];
    if (!layers.is_array() || layers.size() == 0 || layers.size() > 1024) { err = "configuration: 'layers' must list 1 .. 1024 layers"; return nullptr; }
    const int nl = (int)layers.size();

    M.embed = ld.embedding("embed", V, W);                      // the table the tokens' rows come from ...
    M.head = ld.rows({{"embed", V}}, W);                        // ... is the output head too (dense rows for the linear kernels)
    M.final_norm = ld.vec("final.norm", W);
    uint64_t active_bytes = ((uint64_t)V * W + W) * 2;          // what one token reads of the weights: the head and a table row, then every layer's matrices

    M.layers.resize((size_t)nl);
    for (int il = 0; il < nl && ld.err.empty(); il++) {
        const Json &lc = layers.at((size_t)il), &mx = lc["mixer"];
        NvxLayer &L = M.layers[(size_t)il];
        const std::string p = "l" + std::to_string(il) + ".", pm = p + "mix.";
        const std::string type = lc["type"].as_string();
        L.norm1b = ld.vec(p + "norm1", W);                       // (behind the mixer; nothing in front of it)
        L.heads = (int)mx["heads"].as_int(); L.kv_heads = (int)mx["kv_heads"].as_int(L.heads); L.dim = (int)mx["dim"].as_int(); L.vdim = (int)mx["vdim"].as_int(L.dim);
        if (!cfg_positive(err, "mixer.heads", L.heads, 4096) || !cfg_positive(err, "mixer.kv_heads", L.kv_heads, L.heads) || !cfg_positive(err, "mixer.dim", L.dim, 1 << 16) ||
            !cfg_positive(err, "mixer.vdim", L.vdim, 1 << 16)) return nullptr;
        if (L.heads % L.kv_heads != 0) { err = "configuration: mixer.heads must be a multiple of mixer.kv_heads"; return nullptr; }
        const int H = L.heads, G = L.kv_heads, D = L.dim, VD = L.vdim;
        if (type == "attention") {
            L.type = NVX_GQ;
            if (!gq_attn_shape_ok(H, G, D, VD)) { err = "attention: dim " + std::to_string(D) + " / vdim " + std::to_string(VD) + " is beyond what the attention kernel holds per lane (512)"; return nullptr; }
            L.scale = (float)mx["scale"].as_double(1.0);
            L.softcap = (float)mx["softcap"].as_double(0.0);
            if (!(L.softcap >= 0.0f)) { err = "configuration: mixer.softcap must not be negative"; return nullptr; }
            const Json &rot = mx["rot"];
            L.rot_dims = rot.is_object() ? (int)rot["dims"].as_int(0) : 0;
            if (L.rot_dims > D || (L.rot_dims & 1) || L.rot_dims < 0) { err = "configuration: rot.dims must be even and at most mixer.dim"; return nullptr; }
            if (rot.is_object()) {
                const double base = rot["base"].as_double(10000.0);
                if (!(base > 0.0)) { err = "configuration: rot.base must be positive"; return nullptr; }
                if (VD & 1) { err = "configuration: mixer.vdim must be even (the value heads turn in pairs)"; return nullptr; }
                if (L.rot_dims > 0) L.rot_freq = rot_table(ld, base, L.rot_dims);
                L.v_rot_freq = rot_table(ld, base, VD);           // the values turn over ALL their entries, with the same base
            }
            L.qk_norm_per_head = true;
            L.q_norm = ld.vec(pm + "q.norm", D);
            L.k_norm = ld.vec(pm + "k.norm", D);
            L.sink = ld.vec(pm + "sink", H);
            L.proj = ld.rows({{pm + "q", H * D}, {pm + "k", G * D}, {pm + "v", G * VD}}, W);
            L.o = ld.rows({{pm + "o", W}}, H * VD);
            M.max_q = std::max(M.max_q, H * D);
        } else if (type == "delta" || type == "channel_delta") {
            L.type = NVX_DELTA;
            L.decay_per_channel = type == "channel_delta";
            L.conv_taps = (int)mx["conv"].as_int(1);
            if (!delta_shape_ok(H, G, D, VD, L.conv_taps)) {
                err = "delta rule: dim " + std::to_string(D) + " / conv " + std::to_string(L.conv_taps) + " is beyond what the recurrence kernels hold (dim 512, " + std::to_string(DELTA_MAX_TAPS) + " taps)";
                return nullptr;
            }
            const int taps = L.conv_taps;
            std::vector<std::pair<std::string, int>> proj = {{pm + "q", G * D}, {pm + "k", G * D}, {pm + "v", H * VD}, {pm + "b", H}};
            L.off_beta = 2 * G * D + H * VD;
            L.off_a = L.off_beta + H;
            if (L.decay_per_channel) {
                L.rank_a = ld.rows_of(pm + "a1", W); L.rank_g = ld.rows_of(pm + "g1", W);
                if (L.rank_a < 0 || L.rank_g < 0) break;
                proj.push_back({pm + "a1", L.rank_a}); proj.push_back({pm + "g1", L.rank_g});
                L.off_g = L.off_a + L.rank_a;
                L.a2 = ld.rows({{pm + "a2", H * D}}, L.rank_a);
                L.g2 = ld.rows({{pm + "g2", H * VD}}, L.rank_g);
                L.dt_bias = ld.vec(pm + "dt_bias", H * D);
                M.max_qa = std::max(M.max_qa, std::max(H * D, H * VD));
                active_bytes += ((uint64_t)H * D * L.rank_a + (uint64_t)H * VD * L.rank_g) * 2;
            } else {
                proj.push_back({pm + "a", H}); proj.push_back({pm + "g", H * VD});
                L.off_g = L.off_a + H;
                L.dt_bias = ld.vec(pm + "dt_bias", H);
            }
            L.proj = ld.rows(proj, W);
            L.conv_w = ld.rows_f32({{pm + "q.conv", G * D}, {pm + "k.conv", G * D}, {pm + "v.conv", H * VD}}, taps);
            L.A_log = ld.vec(pm + "A_log", H);
            L.mix_norm = ld.vec(pm + "norm", VD);
            L.o = ld.rows({{pm + "o", W}}, H * VD);
            M.max_q = std::max(M.max_q, delta_work_row(H, G, D, VD, L.decay_per_channel ? 1 : 0));
        } else { err = "configuration: layer " + std::to_string(il) + " has unknown type '" + type + "'"; return nullptr; }
        M.max_proj = std::max(M.max_proj, L.proj.N);
        M.max_att = std::max(M.max_att, H * VD);
        active_bytes += ((uint64_t)L.proj.N * W + (uint64_t)W * H * VD) * 2;
        const Json &mlp = lc["mlp"];
        if (mlp.is_object()) {
            const std::string pf = p + "mlp.";
            const std::string kind = mlp["kind"].as_string();
            if (kind != "dense") { err = "configuration: layer " + std::to_string(il) + " has unknown mlp.kind '" + kind + "'"; return nullptr; }
            L.norm2b = ld.vec(p + "norm2", W);
            L.ff_kind = NVX_FF_DENSE;
            L.ff = (int)mlp["ff"].as_int();
            if (!cfg_positive(err, "mlp.ff", L.ff)) return nullptr;
            L.gate = ld.rows({{pf + "gate", L.ff}}, W);
            L.up = ld.rows({{pf + "up", L.ff}}, W);
            L.down_ff = ld.rows({{pf + "down", W}}, L.ff);
            M.max_ff = std::max(M.max_ff, L.ff);
            active_bytes += (uint64_t)3 * L.ff * W * 2;
        }
    }
    if (!ld.err.empty()) { err = ld.err; return nullptr; }
    for (int il = 0; il < nl; il++) {
        NvxRun r; r.layer = il; r.pass = -1;
        r.plane = M.layers[(size_t)il].type == NVX_GQ ? M.n_cache_runs++ : M.n_state_runs++;
        M.runs.push_back(r);
    }
    HParams &hp = m->hp;
    hp.arch = "tuterax";
    hp.n_embd = W; hp.n_vocab = V; hp.n_vocab_local = V; hp.n_layer = nl; hp.n_layer_runs = nl;
    hp.n_head = M.layers[0].heads; hp.n_head_kv = M.layers[0].kv_heads; hp.head_dim = M.layers[0].dim; hp.eps = M.eps;
    hp.n_head_full = hp.n_head; hp.n_head_kv_full = hp.n_head_kv;
    m->bytes_per_token = active_bytes;
    m->desc = "tuterax " + std::to_string(nl) + " layers width " + std::to_string(W) + " BF16";
    status = 0;
    return m;
}

// the delta-rule mixer of one layer run over the micro-batch: -> nvx_y_
hipError_t Context::nvx_delta_mixer(const NvxLayer &L, const NvxRun &r, int T) {
    const NovoraxModel &M = *model->nvx;
    const int W = M.width, H = L.heads, G = L.kv_heads, D = L.dim, VD = L.vdim, LD_P = L.proj.N;
    const int per_channel = L.decay_per_channel ? 1 : 0;
    TTX_TRY(nvx_linear(L.proj, x_, W, T, nvx_a_, LD_P, MMB_STORE, nullptr, 1.0f, L.norm1));
    DeltaArgs da{};
    da.p = nvx_a_; da.ld_p = LD_P; da.off_beta = L.off_beta;
    da.a = nvx_a_ + L.off_a; da.ld_a = LD_P;
    const float *gate = nvx_a_; int ld_gate = LD_P, off_gate = L.off_g;
    if (per_channel) {
        // the low-rank halves of the decay and of the output gate: their first factors rode in the projection, the second ones follow here
        TTX_TRY(nvx_linear(L.a2, nvx_a_ + L.off_a, LD_P, T, nvx_qa_, H * D));
        TTX_TRY(nvx_linear(L.g2, nvx_a_ + L.off_g, LD_P, T, nvx_lat_, H * VD));
        da.a = nvx_qa_; da.ld_a = H * D;
        gate = nvx_lat_; ld_gate = H * VD; off_gate = 0;
    }
    da.per_channel = per_channel; da.A_log = L.A_log; da.dt_bias = L.dt_bias; da.conv_w = L.conv_w; da.taps = L.conv_taps;
    da.conv_state = nvx_n_[(size_t)r.plane]; da.S = nvx_S_[(size_t)r.plane];
    da.c = nvx_q_; da.ld_c = delta_work_row(H, G, D, VD, per_channel);
    da.o = nvx_o_; da.ld_o = H * VD; da.H = H; da.G = G; da.D = D; da.VD = VD;
    const size_t TU = cp.n_ubatch;
    for (const auto &wv : nvx_waves_) {
        da.seg_start = d_seg_ + wv.first; da.seg_len = d_seg_ + TU + wv.first; da.seg_slot = d_seg_ + 2 * TU + wv.first; da.n_seg = wv.second;
        da.max_len = 0;
        for (int s = 0; s < wv.second; s++) da.max_len = std::max(da.max_len, (int)h_seg_[TU + (size_t)wv.first + (size_t)s]);
        TTX_TRY(launch_delta_prep(da, stream_));
        TTX_TRY(launch_delta_scan(da, stream_));
    }
    TTX_TRY(launch_mlstm_out(nvx_o_, H * VD, gate, ld_gate, off_gate, L.mix_norm, T, H, VD, M.eps, nvx_att_, H * VD, stream_, 0,
                             per_channel ? MLSTM_GATE_SIGMOID : MLSTM_GATE_SILU));
    TTX_TRY(nvx_linear(L.o, nvx_att_, H * VD, T, nvx_y_, W));
    prof_mark("delta_rule");
    return hipSuccess;
}

}  // namespace mi355
