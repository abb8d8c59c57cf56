// novorax.cc — the folder models (config.json + model.safetensors): the registry that picks a design's loader by "architecture", the Novorax loader, and what
// every such design shares inside Context - buffers, cache planes and state slots, segment lists and scan bounds, the layer-run loop, the output head
// (novorax.h describes the designs, runtime.h the context; the Fidepel loader and its block are in fidepel.cc, the Tuterax loader and the delta-rule mixer
// in tuterax.cc, the Dinilorn loader, its retention mixer and its feed-forward in dinilorn.cc).
//
// The context's own machinery carries them: the cell table (find / free / sequence masks) addresses the attention layers' cache planes, the micro-batch staging
// block brings tokens, positions, cells and sequence ids to the device, the sequence id is the slot of the recurrent state, logits / arg-max / top-k leave
// through the usual buffers.  What is new per micro-batch is the list of segments (runs of consecutive rows of one sequence) the recurrence walks.
#include <sys/stat.h>

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

#include "config_model.h"

namespace mi355 {

void set_error(const char *fmt, ...);

#define NVX_TRY(expr)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess) {                                                                    \
            set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__);  \
            return e_;                                                                             \
        }                                                                                          \
    } while (0)

bool config_model_path(const std::string &path, std::string &dir) {
    struct stat st;
    if (stat(path.c_str(), &st) != 0) return false;
    dir = path;
    if (!S_ISDIR(st.st_mode)) {
        const size_t sl = path.find_last_of('/');
        const std::string base = sl == std::string::npos ? path : path.substr(sl + 1);
        if (base != "config.json") return false;
        dir = sl == std::string::npos ? "." : path.substr(0, sl);
    }
    return stat((dir + "/config.json").c_str(), &st) == 0 && stat((dir + "/model.safetensors").c_str(), &st) == 0;
}

// the model registry of the folder models: configuration "architecture" -> the design's loader
Model *config_model_load(const std::string &dir, int main_gpu, std::string &err, int &status) {
    static const struct { const char *architecture; Model *(*build)(const Json &, const std::string &, Bf16Loader &, std::string &, int &); } designs[] = {
        {"Novorax", novorax_build},
        {"Fidepel", fidepel_build},
        {"Tuterax", tuterax_build},
        {"Dinilorn", dinilorn_build},
    };
    status = -102;
    std::ifstream cf(dir + "/config.json");
    if (!cf) { err = "cannot open " + dir + "/config.json"; status = -101; return nullptr; }
    std::stringstream ss;
    ss << cf.rdbuf();
    Json cfg;
    std::string jerr;
    if (!Json::parse(ss.str(), cfg, &jerr) || !cfg.is_object()) { err = "config.json: " + jerr; return nullptr; }
    const std::string arch = cfg["architecture"].as_string();
    for (const auto &d : designs) {
        if (arch != d.architecture) continue;
        std::unique_ptr<Model> m(new Model());
        m->path = dir;
        m->device = main_gpu;
        if (hipSetDevice(main_gpu) != hipSuccess) { err = "hipSetDevice failed"; status = -103; return nullptr; }
        Bf16Loader ld;
        ld.m = m.get();
        err = ld.st.open(dir + "/model.safetensors");
        if (!err.empty()) { status = err.rfind("cannot", 0) == 0 ? -101 : -102; return nullptr; }
        m->nvx.reset(new NovoraxModel());
        if (!d.build(cfg, dir, ld, err, status)) return nullptr;   // (m frees what was uploaded)
        if (hipDeviceSynchronize() != hipSuccess) { err = "device synchronise failed behind the upload"; status = -103; return nullptr; }
        m->device_bytes = ld.bytes;
        m->file_tensor_bytes = ld.st.file_bytes();
        if (!m->bytes_per_token) m->bytes_per_token = ld.bytes;
        status = 0;
        return m.release();
    }
    err = "config.json: unsupported architecture '" + arch + "'";
    return nullptr;
}

Model *novorax_build(const Json &cfg, const std::string &dir, Bf16Loader &ld, std::string &err, int &status) {
    (void)dir;
    status = -102;
    Model *const m = ld.m;
    NovoraxModel &M = *m->nvx;
    M.design = "novorax";
    const int W = (int)cfg["width"].as_int(), V = (int)cfg["vocab"].as_int();
    if (!cfg_positive(err, "width", W) || !cfg_positive(err, "vocab", V)) return nullptr;
    M.width = W; M.n_vocab = V;
    M.eps = (float)cfg["norm"]["eps"].as_double(1e-5);
    M.logit_scale = (float)cfg["logit_scale"].as_double(1.0);
    const Json &layers = cfg["layers"];
    if (!layers.is_array() || layers.size() == 0 || layers.size() > 1024) { err = "configuration: 'layers' must list 1 .. 1024 layers"; return nullptr; }
    const int nl = (int)layers.size();

    M.embed = ld.embedding("embed", V, W);
    M.head = ld.rows({{"head", V}}, W);
    M.final_norm = ld.vec("final.norm", W);

    M.layers.resize((size_t)nl);
    for (int il = 0; il < nl && ld.err.empty(); il++) {
        const Json &lc = layers.at((size_t)il), &mx = lc["mixer"];
        NvxLayer &L = M.layers[(size_t)il];
        const std::string p = "l" + std::to_string(il) + ".", pm = p + "mix.";
        const std::string type = lc["type"].as_string();
        L.norm1 = ld.vec(p + "norm1", W);
        L.norm1b = ld.vec(p + "norm1b", W);
        L.heads = (int)mx["heads"].as_int(); L.dim = (int)mx["dim"].as_int(); L.vdim = (int)mx["vdim"].as_int();
        if (!cfg_positive(err, "mixer.heads", L.heads, 4096) || !cfg_positive(err, "mixer.dim", L.dim, 1 << 16) || !cfg_positive(err, "mixer.vdim", L.vdim, 1 << 16)) return nullptr;
        const int H = L.heads;
        if (type == "latent_attention") {
            L.type = NVX_LATENT;
            L.rot = (int)mx["rot_dim"].as_int(0); L.kv_rank = (int)mx["kv_rank"].as_int(); L.q_rank = (int)mx["q_rank"].as_int();
            if (!cfg_positive(err, "mixer.kv_rank", L.kv_rank) || !cfg_positive(err, "mixer.q_rank", L.q_rank) || L.rot < 0) { if (err.empty()) err = "configuration: mixer.rot_dim is negative"; return nullptr; }
            if (!latent_attn_shape_ok(L.kv_rank, L.rot)) { err = "latent attention: kv_rank " + std::to_string(L.kv_rank) + " (+ rot_dim) is beyond what the attention kernel holds per lane (1088)"; return nullptr; }
            L.scale = (float)mx["scale"].as_double(1.0);
            const Json &mask = mx["mask"];
            L.window = mask.is_object() ? (int)mask["size"].as_int(0) : 0;
            if (L.window < 0) L.window = 0;
            const Json &rot = mx["rot"];
            L.rot_dims = rot.is_object() ? (int)rot["dims"].as_int(L.rot) : 0;
            if (L.rot_dims > L.rot || (L.rot_dims & 1) || L.rot_dims < 0) { err = "configuration: rot.dims must be even and at most rot_dim"; return nullptr; }
            {
                // radians per position of pair i: base^(-2i / dims), blended towards 1 / factor of itself where YaRN says the pair turns too slowly for the
                // original context (ramp 0 below `lo`, 1 above `hi`); cos and sin carry the attention scale 0.1 ln(factor) + 1
                const int half = L.rot_dims / 2;
                const double base = rot["base"].as_double(10000.0);
                std::vector<float> fr((size_t)std::max(half, 1), 0.0f);
                const Json &scg = rot["scaling"];
                double factor = 1.0, lo = 0.0, hi = 0.0;
                const bool yarn = scg.is_object() && half > 0;
                if (yarn) {
                    factor = scg["factor"].as_double(1.0);
                    const double orig = scg["original"].as_double(1.0), fast = scg["fast"].as_double(32.0), slow = scg["slow"].as_double(1.0);
                    if (!(factor > 0.0) || !(orig > 0.0) || !(fast > 0.0) || !(slow > 0.0) || !(base > 1.0)) { err = "configuration: rot.scaling values must be positive"; return nullptr; }
                    const auto corr = [&](double turns) { return L.rot_dims * std::log(orig / (2.0 * M_PI * turns)) / (2.0 * std::log(base)); };
                    lo = std::max(std::floor(corr(fast)), 0.0);
                    hi = std::min(std::ceil(corr(slow)), (double)(L.rot_dims - 1));
                    L.rot_mscale = (float)(0.1 * std::log(factor) + 1.0);
                }
                for (int i = 0; i < half; i++) {
                    double f = std::pow(base, -2.0 * i / L.rot_dims);
                    if (yarn) {
                        const double ramp = std::min(1.0, std::max(0.0, (i - lo) / std::max(hi - lo, 0.001)));
                        f = f / factor * ramp + f * (1.0 - ramp);
                    }
                    fr[(size_t)i] = (float)f;
                }
                L.rot_freq = (float *)ld.dev(fr.data(), fr.size() * 4);
            }
            const int QD = L.dim + L.rot;
            L.down = ld.rows({{pm + "dq", L.q_rank}, {pm + "dkv", L.kv_rank + L.rot}}, W);
            L.dq_norm = ld.vec(pm + "dq.norm", L.q_rank);
            L.dkv_norm = ld.vec(pm + "dkv.norm", L.kv_rank);
            L.uq = ld.rows({{pm + "uq", H * QD}}, L.q_rank);
            L.uv = ld.rows({{pm + "uv", H * L.vdim}}, L.kv_rank);
            L.o = ld.rows({{pm + "o", W}}, H * L.vdim);
            if (ld.st.find(pm + "sink")) L.sink = ld.vec(pm + "sink", H);
            if (const SafeTensor *t = ld.need(pm + "uk", "BF16", {(int64_t)H * L.dim, L.kv_rank})) {
                const unsigned short *s = (const unsigned short *)t->data;
                std::vector<unsigned short> tr((size_t)H * L.kv_rank * L.dim);
                for (int h = 0; h < H; h++)
                    for (int d = 0; d < L.dim; d++)
                        for (int r = 0; r < L.kv_rank; r++) tr[((size_t)h * L.kv_rank + r) * L.dim + d] = s[((size_t)h * L.dim + d) * L.kv_rank + r];
                L.uk_t.w = (unsigned short *)ld.dev(tr.data(), tr.size() * 2);
                L.uk_t.N = L.kv_rank; L.uk_t.K = L.dim;
            }
            M.max_down = std::max(M.max_down, L.q_rank + L.kv_rank + L.rot);
            M.max_q_rank = std::max(M.max_q_rank, L.q_rank);
            M.max_q = std::max(M.max_q, H * QD);
            M.max_qa = std::max(M.max_qa, H * L.kv_rank);
            M.max_att = std::max(M.max_att, H * L.vdim);
        } else if (type == "mlstm") {
            L.type = NVX_MLSTM;
            L.gate_cap = (float)mx["gate_cap"].as_double(0.0);
            if (!(L.gate_cap > 0.0f)) { err = "configuration: mixer.gate_cap must be positive"; return nullptr; }
            if (!mlstm_shape_ok(L.dim, L.vdim)) { err = "mlstm: dim " + std::to_string(L.dim) + " is beyond what the recurrence kernel keeps in registers (512)"; return nullptr; }
            L.proj = ld.rows({{pm + "q", H * L.dim}, {pm + "k", H * L.dim}, {pm + "v", H * L.vdim}, {pm + "g", H * L.vdim}, {pm + "i", H}, {pm + "f", H}}, W);
            L.i_bias = ld.vec(pm + "i.b", H);
            L.f_bias = ld.vec(pm + "f.b", H);
            L.mix_norm = ld.vec(pm + "norm", H * L.vdim);
            L.o = ld.rows({{pm + "o", W}}, H * L.vdim);
            M.max_proj = std::max(M.max_proj, L.proj.N);
            M.max_att = std::max(M.max_att, H * L.vdim);
        } else { err = "configuration: layer " + std::to_string(il) + " has unknown type '" + type + "'"; return nullptr; }
        const Json &mlp = lc["mlp"];
        if (mlp.is_object()) {
            const std::string pf = p + "mlp.";
            L.norm2 = ld.vec(p + "norm2", W);
            L.norm2b = ld.vec(p + "norm2b", W);
            const std::string kind = mlp["kind"].as_string();
            if (kind == "dense") {
                L.ff_kind = NVX_FF_DENSE;
                L.ff = (int)mlp["ff"].as_int();
                if (!cfg_positive(err, "mlp.ff", L.ff)) return nullptr;
                L.up = ld.rows({{pf + "up", L.ff}}, W);
                L.down_ff = ld.rows({{pf + "down", W}}, L.ff);
            } else if (kind == "moe") {
                L.ff_kind = NVX_FF_EXPERTS;
                L.ff = (int)mlp["expert"]["ff"].as_int();
                L.n_expert = (int)mlp["router"]["experts"].as_int(); L.top = (int)mlp["router"]["top"].as_int();
                if (!cfg_positive(err, "mlp.expert.ff", L.ff) || !cfg_positive(err, "mlp.router.experts", L.n_expert, 4096) || !cfg_positive(err, "mlp.router.top", L.top, L.n_expert)) return nullptr;
                std::vector<std::pair<std::string, int>> g, u, d;
                for (int e = 0; e < L.n_expert; e++) {
                    const std::string pe = pf + "e" + std::to_string(e) + ".";
                    g.push_back({pe + "gate", L.ff}); u.push_back({pe + "up", L.ff}); d.push_back({pe + "down", W});
                }
                L.e_gate = ld.rows(g, W); L.e_up = ld.rows(u, W); L.e_down = ld.rows(d, L.ff);
                if (const SafeTensor *t = ld.need(pf + "table", "I32", {V, L.top})) {
                    const int32_t *tb = (const int32_t *)t->data;
                    for (int64_t i = 0; i < (int64_t)V * L.top; i++)
                        if (tb[i] < 0 || tb[i] >= L.n_expert) { err = "tensor '" + pf + "table' names expert " + std::to_string(tb[i]) + " of " + std::to_string(L.n_expert); return nullptr; }
                    L.table = (int32_t *)ld.dev(t->data, t->bytes);
                }
                M.max_top = std::max(M.max_top, L.top);
                M.max_expert = std::max(M.max_expert, L.n_expert);
            } else { err = "configuration: layer " + std::to_string(il) + " has unknown mlp.kind '" + kind + "'"; return nullptr; }
            M.max_ff = std::max(M.max_ff, L.ff);
        }
    }
    if (!ld.err.empty()) { err = ld.err; return nullptr; }

    // the order of layer runs; every pass of the looped span opens with the input projection
    int times = 0;
    if (!cfg_layer_runs(cfg["loop"], nl, err, times, [&](int il, int pass) {
            NvxRun r; r.layer = il; r.pass = pass;
            r.plane = M.layers[(size_t)il].type == NVX_LATENT ? M.n_cache_runs++ : M.n_state_runs++;
            M.runs.push_back(r);
        })) return nullptr;
    if (times > 0) {
        M.loop_in = ld.rows({{"loop.in", W}}, 2 * W);
        if (const SafeTensor *t = ld.need("loop.step", "BF16", {times, W})) {
            std::vector<float> h((size_t)times * W);
            const unsigned short *s = (const unsigned short *)t->data;
            for (size_t i = 0; i < h.size(); i++) { const uint32_t u = (uint32_t)s[i] << 16; memcpy(&h[i], &u, 4); }
            M.loop_step = (float *)ld.dev(h.data(), h.size() * 4);
        }
    }
    if (!ld.err.empty()) { err = ld.err; return nullptr; }
    HParams &hp = m->hp;
    hp.arch = "novorax";
    hp.n_embd = W; hp.n_vocab = V; hp.n_vocab_local = V; hp.n_layer = nl; hp.n_layer_runs = (int)M.runs.size();
    hp.n_head = M.layers[0].heads; hp.n_head_kv = 1; hp.head_dim = M.layers[0].dim; hp.eps = M.eps;
    hp.n_head_full = hp.n_head; hp.n_head_kv_full = 1;
    m->desc = "novorax " + std::to_string(nl) + " layers (" + std::to_string(M.runs.size()) + " runs) width " + std::to_string(W) + " BF16";
    status = 0;
    return m;
}

// ------------------------------------------------------------------------------------------ context
// floats one sequence slot holds for a recurrent layer run: the state matrices; the second set (mLSTM: normalisers, delta rule: the convolutions' last
// taps - 1 inputs); the third (mLSTM: running maxima)
static void nvx_state_sizes(const NvxLayer &L, size_t &s_sz, size_t &n_sz, size_t &m_sz) {
    s_sz = (size_t)L.heads * L.dim * L.vdim;
    if (L.type == NVX_MLSTM) { n_sz = (size_t)L.heads * L.dim; m_sz = (size_t)L.heads; }
    else if (L.type == NVX_RETENTION) { n_sz = 0; m_sz = 0; }
    else { n_sz = (size_t)std::max(L.conv_taps - 1, 0) * (size_t)L.delta_channels(); m_sz = 0; }
}
static bool nvx_recurrent(const NvxLayer &L) { return L.type == NVX_MLSTM || L.type == NVX_DELTA || L.type == NVX_RETENTION; }

bool Context::init_novorax(std::string &err) {
    const NovoraxModel &M = *model->nvx;
    const size_t T = cp.n_ubatch, W = (size_t)M.width, NC = cp.n_ctx, NS = cp.n_seq_max;
    cells_.assign(NC, KVCell());
    d_cell_pos_ = (int32_t *)dalloc(NC * 4);
    d_cell_seq_ = (uint64_t *)dalloc(NC * 8);
    d_delta_ = (int32_t *)dalloc(NC * 4);
    const size_t Tp = (T + 1) & ~(size_t)1;
    stage_bytes_ = 16 + Tp * 4 * 5 + Tp * 8;
    stage_bytes_ = (stage_bytes_ + 15) & ~(size_t)15;
    d_stage_ = (uint8_t *)dalloc(stage_bytes_);
    if (!d_stage_ || hipHostMalloc((void **)&h_stage_, stage_bytes_, hipHostMallocDefault) != hipSuccess) { err = "staging allocation failed"; return false; }
    d_nkv_ = (int32_t *)d_stage_;
    d_tok_ = (int32_t *)(d_stage_ + 16);
    d_pos_ = d_tok_ + Tp; d_seq_ = d_pos_ + Tp; d_cell_ = d_seq_ + Tp; d_outrow_ = d_cell_ + Tp;
    d_seqmask_ = (uint64_t *)(d_outrow_ + Tp);
    d_seg_ = (int32_t *)dalloc(5 * T * 4);
    if (!d_seg_ || hipHostMalloc((void **)&h_seg_, 5 * T * 4, hipHostMallocDefault) != hipSuccess) { err = "segment list allocation failed"; return false; }

    // cache planes and recurrent state
    nvx_cache_.assign((size_t)M.n_cache_runs, nullptr);
    nvx_S_.assign((size_t)M.n_state_runs, nullptr); nvx_n_ = nvx_S_; nvx_m_ = nvx_S_;
    for (const NvxRun &r : M.runs) {
        const NvxLayer &L = M.layers[(size_t)r.layer];
        if (!nvx_recurrent(L)) {
            nvx_cache_[(size_t)r.plane] = (float *)dalloc(NC * (size_t)L.cache_row() * 4);
            if (!nvx_cache_[(size_t)r.plane]) { err = "attention cache allocation failed"; return false; }
        } else {
            size_t s_sz, n_sz, m_sz;
            nvx_state_sizes(L, s_sz, n_sz, m_sz);
            nvx_S_[(size_t)r.plane] = (float *)dalloc(NS * s_sz * 4);
            nvx_n_[(size_t)r.plane] = (float *)dalloc(std::max<size_t>(NS * n_sz, 1) * 4);
            nvx_m_[(size_t)r.plane] = (float *)dalloc(std::max<size_t>(NS * m_sz, 1) * 4);
            if (!nvx_S_[(size_t)r.plane] || !nvx_n_[(size_t)r.plane] || !nvx_m_[(size_t)r.plane]) { err = "recurrent state allocation failed"; return false; }
        }
    }
    nvx_seq_len_.assign(NS, 0);
    // activations
    const size_t A = (size_t)std::max(M.max_down, M.max_proj), TOP = (size_t)std::max(M.max_top, 1);
    x_ = (float *)dalloc(T * W * 4);
    xn_ = (float *)dalloc(T * W * 4);
    xo_ = (float *)dalloc(T * W * 4);
    nvx_x0_ = (float *)dalloc(T * W * 4);
    nvx_xcat_ = (float *)dalloc(T * 2 * W * 4);
    nvx_y_ = (float *)dalloc(T * W * 4);
    nvx_a_ = (float *)dalloc(T * std::max<size_t>(A, 1) * 4);
    nvx_cq_ = (float *)dalloc(T * (size_t)std::max(M.max_q_rank, 1) * 4);
    nvx_q_ = (float *)dalloc(T * (size_t)std::max(M.max_q, 1) * 4);
    nvx_qa_ = (float *)dalloc(T * (size_t)std::max(M.max_qa, 1) * 4);
    nvx_lat_ = (float *)dalloc(T * (size_t)std::max(M.max_qa, 1) * 4);
    nvx_att_ = (float *)dalloc(T * (size_t)std::max(M.max_att, 1) * 4);
    nvx_o_ = (float *)dalloc(T * (size_t)std::max(M.max_att, 1) * 4);
    nvx_ff_ = (float *)dalloc(T * TOP * (size_t)std::max(M.max_ff, 1) * 4);
    {
        int kr = 1;                                              // widest record of a split attention scan: the latent, or a value head
        for (const NvxLayer &L : M.layers) kr = std::max(kr, L.type == NVX_LATENT ? L.kv_rank : L.type == NVX_GQ ? L.vdim : 1);
        nvx_part_floats_ = (size_t)LATENT_ATTN_SPLIT_MAX_PAIRS * LATENT_ATTN_SPLITS * (size_t)(kr + 2);
        // grouped-query layers also cut the block chains of short prompt batches: records for up to 1024 rows x 4 runs of the widest layer
        for (const NvxLayer &L : M.layers)
            if (L.type == NVX_GQ) nvx_part_floats_ = std::max(nvx_part_floats_, std::min<size_t>(T, 1024) * (size_t)L.heads * (size_t)std::max(L.maps, 1) * 4 * (size_t)(L.vdim + 2));
        nvx_part_ = (float *)dalloc(nvx_part_floats_ * 4);
    }
    {
        int vd = 0;
        for (const NvxLayer &L : M.layers) if (L.v_rot_freq) vd = std::max(vd, L.vdim);
        if (vd > 0 && !(nvx_vcs_ = (float *)dalloc(T * (size_t)vd * 4))) { err = "value turn table allocation failed"; return false; }
    }
    if (!x_ || !xn_ || !xo_ || !nvx_x0_ || !nvx_xcat_ || !nvx_y_ || !nvx_a_ || !nvx_cq_ || !nvx_q_ || !nvx_qa_ || !nvx_lat_ || !nvx_att_ || !nvx_o_ || !nvx_ff_) { err = "activation buffer allocation failed"; return false; }
    if (M.max_top > 0) {
        nvx_xg_ = (float *)dalloc(T * TOP * W * 4);
        nvx_yg_ = (float *)dalloc(T * TOP * W * 4);
        nvx_ids_ = (int32_t *)dalloc(T * TOP * 4);
        nvx_meta_ = (int32_t *)dalloc((size_t)(2 * M.max_expert + 1) * 4);
        nvx_slot_ = (int32_t *)dalloc(T * TOP * 4);
        nvx_tokof_ = (int32_t *)dalloc(T * TOP * 4);
        nvx_rw_ = (float *)dalloc(T * TOP * 4);
        if (!nvx_xg_ || !nvx_yg_ || !nvx_ids_ || !nvx_meta_ || !nvx_slot_ || !nvx_tokof_ || !nvx_rw_) { err = "expert batch buffers allocation failed"; return false; }
    }
    if (M.max_shared_ff > 0) {
        nvx_sh_ = (float *)dalloc(T * (size_t)M.max_shared_ff * 4);
        nvx_ys_ = (float *)dalloc(T * W * 4);
        if (!nvx_sh_ || !nvx_ys_) { err = "shared expert buffers allocation failed"; return false; }
    }
    bool side_branches = M.parallel_block;                      // (also: a routed feed-forward whose shared expert runs beside the routed ones)
    for (const NvxLayer &L : M.layers) side_branches = side_branches || (L.ff_kind == NVX_FF_ROUTED && L.shared_ff > 0);
    if (side_branches) {
        // side streams of the block's feed-forward branches (default priority, like the main one); MI355_BLOCK_FORK=0 keeps every launch on the main stream
        const char *ev = getenv("MI355_BLOCK_FORK");
        nvx_fork_ok_ = !(ev && ev[0] == '0');
        for (int i = 0; i < 2 && nvx_fork_ok_; i++)
            nvx_fork_ok_ = hipStreamCreateWithFlags(&nvx_side_[i], hipStreamNonBlocking) == hipSuccess &&
                           hipEventCreateWithFlags(&nvx_join_ev_[i], hipEventDisableTiming) == hipSuccess;
        nvx_fork_ok_ = nvx_fork_ok_ && hipEventCreateWithFlags(&nvx_fork_ev_, hipEventDisableTiming) == hipSuccess;
    }
    d_argmax_ = (int32_t *)dalloc(T * 4);
    argmax_scratch_ = (float *)dalloc(T * 129 * 4);
    if (!d_argmax_ || !argmax_scratch_ || hipHostMalloc((void **)&h_argmax_, T * 4, hipHostMallocDefault) != hipSuccess) { err = "arg-max buffers allocation failed"; return false; }
    embeddings_enabled = false;
    kv_clear();
    nvx_state_reset(-1);
    if (hipDeviceSynchronize() != hipSuccess) { err = "device synchronise failed"; return false; }
    return true;
}

void Context::nvx_state_reset(int seq) {
    const NovoraxModel &M = *model->nvx;
    const size_t NS = cp.n_seq_max;
    for (const NvxRun &r : M.runs) {
        const NvxLayer &L = M.layers[(size_t)r.layer];
        if (!nvx_recurrent(L)) continue;
        size_t s_sz, n_sz, m_sz;
        nvx_state_sizes(L, s_sz, n_sz, m_sz);
        const size_t first = seq < 0 ? 0 : (size_t)seq, cnt = seq < 0 ? NS : 1;
        if (first >= NS) continue;
        (void)launch_mlstm_state_reset(nvx_S_[(size_t)r.plane] + first * s_sz, cnt * s_sz, nvx_n_[(size_t)r.plane] + first * n_sz, cnt * n_sz,
                                       nvx_m_[(size_t)r.plane] + first * m_sz, cnt * m_sz, stream_);
    }
    if (seq < 0) std::fill(nvx_seq_len_.begin(), nvx_seq_len_.end(), 0);
    else if ((size_t)seq < nvx_seq_len_.size()) nvx_seq_len_[(size_t)seq] = 0;
}

void Context::nvx_state_copy(int src, int dst) {
    const NovoraxModel &M = *model->nvx;
    const size_t NS = cp.n_seq_max;
    if (src < 0 || dst < 0 || (size_t)src >= NS || (size_t)dst >= NS || src == dst) return;
    for (const NvxRun &r : M.runs) {
        const NvxLayer &L = M.layers[(size_t)r.layer];
        if (!nvx_recurrent(L)) continue;
        size_t s_sz, n_sz, m_sz;
        nvx_state_sizes(L, s_sz, n_sz, m_sz);
        (void)hipMemcpyAsync(nvx_S_[(size_t)r.plane] + dst * s_sz, nvx_S_[(size_t)r.plane] + src * s_sz, s_sz * 4, hipMemcpyDeviceToDevice, stream_);
        if (n_sz) (void)hipMemcpyAsync(nvx_n_[(size_t)r.plane] + dst * n_sz, nvx_n_[(size_t)r.plane] + src * n_sz, n_sz * 4, hipMemcpyDeviceToDevice, stream_);
        if (m_sz) (void)hipMemcpyAsync(nvx_m_[(size_t)r.plane] + dst * m_sz, nvx_m_[(size_t)r.plane] + src * m_sz, m_sz * 4, hipMemcpyDeviceToDevice, stream_);
    }
    nvx_seq_len_[(size_t)dst] = nvx_seq_len_[(size_t)src];
}

bool Context::nvx_stage_segments(int n, const int32_t *seq, const int32_t *pos, const int *tcell) {
    const size_t T = cp.n_ubatch;
    {
        // per token: one past the highest cell its attention can need - the sequence's cells from earlier batches, and this batch's own cells up to the token
        // (positions grow along a sequence's rows of a batch; a row that breaks that order falls back to the high-water mark)
        // and the lowest cell that can still lie inside the widest window of any of the sequence's tokens in this batch (its earliest token decides; cells
        // of no use to a later token cost it a visibility test each)
        int32_t *hi = h_seg_ + 3 * T, *lo = h_seg_ + 4 * T;
        int base[64], last_pos[64], first_pos[64], low[64];
        for (int s = 0; s < 64; s++) { base[s] = 0; last_pos[s] = -1; first_pos[s] = 0x7fffffff; low[s] = (int)cells_.size(); }
        const int win = model->nvx->max_window, kept = model->nvx->max_keep_first;   // (cells at the first `kept` positions stay in reach of a windowed layer)
        if (win > 0) {
            for (int i = 0; i < n; i++) first_pos[seq[i] & 63] = std::min(first_pos[seq[i] & 63], (int)pos[i]);
            for (size_t c = 0; c < cells_.size(); c++) {
                if (cells_[c].pos < 0) continue;
                uint64_t mk = cells_[c].seqs;
                while (mk) { const int s = __builtin_ctzll(mk); mk &= mk - 1; if (first_pos[s] != 0x7fffffff && (cells_[c].pos > first_pos[s] - win || cells_[c].pos < kept) && (int)c < low[s]) low[s] = (int)c; }
            }
        }
        for (int i = 0; i < n; i++) lo[i] = win > 0 ? low[seq[i] & 63] : 0;
        std::vector<char> mine(cells_.size(), 0);
        for (int i = 0; i < n; i++) mine[(size_t)tcell[i]] = 1;
        for (size_t c = 0; c < cells_.size(); c++) {
            if (cells_[c].pos < 0 || mine[c]) continue;
            uint64_t mk = cells_[c].seqs;
            while (mk) { const int s = __builtin_ctzll(mk); mk &= mk - 1; base[s] = (int)c + 1; }
        }
        for (int i = 0; i < n; i++) {
            const int s = seq[i] & 63;
            if (pos[i] < last_pos[s]) base[s] = (int)cells_.size();
            last_pos[s] = pos[i];
            base[s] = std::max(base[s], tcell[i] + 1);
            hi[i] = base[s];
        }
    }
    int32_t *start = h_seg_, *len = h_seg_ + T, *slot = h_seg_ + 2 * T;
    int ns = 0;
    for (int i = 0; i < n; i++) {
        if (seq[i] < 0 || seq[i] >= (int)cp.n_seq_max) { last_error = "sequence id " + std::to_string(seq[i]) + " has no state slot (n_seq_max " + std::to_string(cp.n_seq_max) + ")"; return false; }
        if (ns > 0 && slot[ns - 1] == seq[i]) len[ns - 1]++;
        else { start[ns] = i; len[ns] = 1; slot[ns] = seq[i]; ns++; }
    }
    // segments of one launch must not share a slot: cut the list where a sequence comes back
    nvx_waves_.clear();
    int first = 0;
    uint64_t seen = 0;
    for (int s = 0; s < ns; s++) {
        const uint64_t bit = 1ull << (slot[s] & 63);
        if (seen & bit) { nvx_waves_.push_back({first, s - first}); first = s; seen = 0; }
        seen |= bit;
    }
    if (ns > first) nvx_waves_.push_back({first, ns - first});
    return hipMemcpyAsync(d_seg_, h_seg_, 5 * T * 4, hipMemcpyHostToDevice, stream_) == hipSuccess;
}

// pn != nullptr: the rows of x are RMS-normed with weight (norm_off + pn) on the way in (few rows: inside the launch; batches: a norm launch into xn_ first)
hipError_t Context::nvx_linear(const BfMat &w, const float *x, int ldx, int T, float *y, int ldy, int epi, const BfMat *w2, float out_scale, const float *pn,
                               const float *bias, float epi_limit) {
    MMBArgs a;
    if (pn && T > MMB_VEC_ROWS) {
        NVX_TRY(launch_rmsnorm_f32(x, ldx, pn, model->nvx->norm_off, nullptr, xn_, w.K, w.K, T, model->nvx->eps, stream_));
        x = xn_; ldx = w.K; pn = nullptr;
    }
    a.pn_w = pn; a.pn_off = model->nvx->norm_off; a.pn_eps = model->nvx->eps;
    a.x = x; a.ldx = ldx; a.w = w.w; a.w2 = w2 ? w2->w : nullptr; a.ldw = w.K; a.y = y; a.ldy = ldy;
    a.T = T; a.N = w.N; a.K = w.K; a.epi = epi; a.f32 = cp.exact_f32 ? 1 : 0; a.out_scale = out_scale; a.bias = bias; a.epi_limit = epi_limit;
    return launch_mmb(a, stream_);
}

hipError_t Context::nvx_feed_forward(const NvxLayer &L, int T, bool *closed) {
    const NovoraxModel &M = *model->nvx;
    const int W = M.width;
    if (L.ff_kind == NVX_FF_ROUTED) return nvx_routed_feed_forward(L, T, closed);
    if (L.ff_kind == NVX_FF_DENSE) {
        if (L.gate.w) NVX_TRY(nvx_linear(L.gate, x_, W, T, nvx_ff_, L.ff, MMB_GELU_MUL, &L.up, 1.0f, L.norm2));
        else NVX_TRY(nvx_linear(L.up, x_, W, T, nvx_ff_, L.ff, MMB_RELU2, nullptr, 1.0f, L.norm2));
        NVX_TRY(nvx_linear(L.down_ff, nvx_ff_, L.ff, T, nvx_y_, W));
        return hipSuccess;
    }
    const int k = L.top, NE = L.n_expert, P = T * k;
    NVX_TRY(launch_moe_table_ids(L.table, d_tok_, T, k, nvx_ids_, stream_));
    MMBArgs g;
    g.w = L.e_gate.w; g.w2 = L.e_up.w; g.ldw = W; g.N = L.ff; g.K = W; g.epi = MMB_SILU_MUL; g.f32 = cp.exact_f32 ? 1 : 0; g.w_zs = (long long)L.ff * W;
    g.y = nvx_ff_; g.ldy = L.ff;
    MMBArgs d;
    d.w = L.e_down.w; d.ldw = L.ff; d.N = W; d.K = L.ff; d.f32 = g.f32; d.w_zs = (long long)W * L.ff;
    d.x = nvx_ff_; d.ldx = L.ff; d.y = nvx_yg_; d.ldy = W;
    const bool grouped = P > 32 && NE <= 64 && (size_t)P * 4 <= 60 * 1024;
    const bool fuse_norm = !grouped && T <= MMB_VEC_ROWS;         // the pair products norm their row themselves
    if (!fuse_norm) NVX_TRY(launch_rmsnorm_f32(x_, W, L.norm2, 1.0f, nullptr, xn_, W, W, T, M.eps, stream_));
    if (grouped) {
        // every expert sees its (token, rank) pairs as one batch of rows: counting sort by expert, gather, two grouped products, combine per token
        NVX_TRY(launch_moe_group(nvx_ids_, T, k, NE, nvx_meta_, nvx_slot_, nvx_tokof_, stream_));
        NVX_TRY(launch_gather_rows_f32(xn_, nvx_tokof_, P, W, nvx_xg_, stream_));
        g.x = nvx_xg_; g.ldx = W; g.T = P; g.nz = NE; g.meta = nvx_meta_;
        d.T = P; d.nz = NE; d.meta = nvx_meta_;
        NVX_TRY(launch_mmb(g, stream_));
        NVX_TRY(launch_mmb(d, stream_));
        NVX_TRY(launch_moe_uniform_combine(nvx_y_, nvx_yg_, nvx_slot_, T, W, k, 1.0f / (float)k, stream_));
    } else {
        // a few tokens: one product per (token, rank) pair against the weights the pair picked
        g.x = fuse_norm ? x_ : xn_; g.ldx = W; g.T = 1; g.nz = P; g.sel = nvx_ids_; g.sel_div = k;
        if (fuse_norm) { g.pn_w = L.norm2; g.pn_off = 1.0f; g.pn_eps = M.eps; }
        d.T = 1; d.nz = P; d.sel = nvx_ids_; d.sel_div = 1;
        NVX_TRY(launch_mmb(g, stream_));
        NVX_TRY(launch_mmb(d, stream_));
        NVX_TRY(launch_moe_uniform_combine(nvx_y_, nvx_yg_, nullptr, T, W, k, 1.0f / (float)k, stream_));
    }
    return hipSuccess;
}

hipError_t Context::run_layers_novorax(int T) {
    const NovoraxModel &M = *model->nvx;
    const int W = M.width;
    const float eps = M.eps;
    cur_T_ = T;
    NVX_TRY(launch_kv_meta_set(d_cell_pos_, d_cell_seq_, d_cell_, d_pos_, d_seqmask_, T, stream_));
    NVX_TRY(launch_get_rows(T_BF16, (const uint8_t *)M.embed.w, W, d_tok_, T, x_, stream_, M.embed_scale));
    if (M.loop_add_embed) NVX_TRY(hipMemcpyAsync(nvx_x0_, x_, (size_t)T * W * 4, hipMemcpyDeviceToDevice, stream_));
    if (M.loop_in.w) NVX_TRY(hipMemcpy2DAsync(nvx_xcat_ + W, (size_t)2 * W * 4, x_, (size_t)W * 4, (size_t)W * 4, (size_t)T, hipMemcpyDeviceToDevice, stream_));
    prof_mark("embed");
    int ir = 0;
    for (const NvxRun &r : M.runs) {
        const NvxLayer &L = M.layers[(size_t)r.layer];
        if (r.pass > 0 && M.loop_add_embed) NVX_TRY(launch_add(x_, nvx_x0_, x_, (int64_t)T * W, stream_));   // a later pass opens with x += embedding rows
        if (r.pass >= 0 && M.loop_in.w) {
            // x <- W_in [x ; x0] + step[pass]: the stream and the embedding output side by side, then the pass's own vector
            NVX_TRY(hipMemcpy2DAsync(nvx_xcat_, (size_t)2 * W * 4, x_, (size_t)W * 4, (size_t)W * 4, (size_t)T, hipMemcpyDeviceToDevice, stream_));
            NVX_TRY(nvx_linear(M.loop_in, nvx_xcat_, 2 * W, T, x_, W));
            NVX_TRY(launch_add_row(x_, M.loop_step + (size_t)r.pass * W, W, T, stream_));
        }
        const int H = L.heads;
        if (M.parallel_block) {
            NVX_TRY(nvx_parallel_block(L, r, T));
            if (debug_taps_ && dbg_) NVX_TRY(hipMemcpyAsync(dbg_ + (size_t)ir * cp.n_ubatch * W, x_, (size_t)T * W * 4, hipMemcpyDeviceToDevice, stream_));
            ir++;
            continue;
        }
        if (L.type == NVX_LATENT) {
            const int QD = L.dim + L.rot, KR = L.kv_rank, LD_A = L.q_rank + KR + L.rot;
            float *cache = nvx_cache_[(size_t)r.plane];
            NVX_TRY(nvx_linear(L.down, x_, W, T, nvx_a_, LD_A, MMB_STORE, nullptr, 1.0f, L.norm1));
            LatentPrepArgs pa{};
            pa.a = nvx_a_; pa.ld_a = LD_A; pa.T = T; pa.q_rank = L.q_rank; pa.kv_rank = KR; pa.rot = L.rot; pa.rot_dims = L.rot_dims;
            pa.wq_norm = L.dq_norm; pa.wkv_norm = L.dkv_norm; pa.eps = eps; pa.rot_freq = L.rot_freq; pa.rot_mscale = L.rot_mscale;
            pa.tok_pos = d_pos_; pa.tok_cell = d_cell_; pa.cq = nvx_cq_; pa.cache = cache;
            NVX_TRY(launch_latent_prep(pa, stream_));
            NVX_TRY(nvx_linear(L.uq, nvx_cq_, L.q_rank, T, nvx_q_, H * QD));
            MMBArgs fa;                                         // qa[t][h] = W_uk_h^T q[t][h][:dim]
            fa.x = nvx_q_; fa.ldx = H * QD; fa.x_zs = QD; fa.w = L.uk_t.w; fa.ldw = L.dim; fa.w_zs = (long long)KR * L.dim;
            fa.y = nvx_qa_; fa.ldy = H * KR; fa.y_zs = KR; fa.T = T; fa.N = KR; fa.K = L.dim; fa.nz = H; fa.f32 = cp.exact_f32 ? 1 : 0;
            NVX_TRY(launch_mmb(fa, stream_));
            LatentAttnArgs aa{};
            aa.qa = nvx_qa_; aa.ld_qa = H * KR; aa.q = nvx_q_; aa.ld_q = H * QD; aa.out = nvx_lat_; aa.ld_out = H * KR;
            aa.T = T; aa.H = H; aa.dim = L.dim; aa.rot = L.rot; aa.kv_rank = KR; aa.rot_dims = L.rot_dims; aa.cache = cache;
            aa.cell_pos = d_cell_pos_; aa.cell_seq = d_cell_seq_; aa.tok_pos = d_pos_; aa.tok_seq = d_seq_; aa.n_kv_dev = d_nkv_;
            aa.window = L.window; aa.scale = L.scale; aa.sink = L.sink; aa.rot_freq = L.rot_freq; aa.rot_mscale = L.rot_mscale;
            aa.tok_hi = d_seg_ + 3 * (size_t)cp.n_ubatch;
            if (nvx_part_ && (long long)T * H <= LATENT_ATTN_SPLIT_MAX_PAIRS) { aa.part = nvx_part_; aa.splits = LATENT_ATTN_SPLITS; }
            NVX_TRY(launch_latent_attn(aa, stream_));
            MMBArgs ua;                                         // att[t][h] = W_uv_h lat[t][h]
            ua.x = nvx_lat_; ua.ldx = H * KR; ua.x_zs = KR; ua.w = L.uv.w; ua.ldw = KR; ua.w_zs = (long long)L.vdim * KR;
            ua.y = nvx_att_; ua.ldy = H * L.vdim; ua.y_zs = L.vdim; ua.T = T; ua.N = L.vdim; ua.K = KR; ua.nz = H; ua.f32 = fa.f32;
            NVX_TRY(launch_mmb(ua, stream_));
            NVX_TRY(nvx_linear(L.o, nvx_att_, H * L.vdim, T, nvx_y_, W));
            prof_mark("latent_attention");
        } else if (L.type == NVX_MLSTM) {
            const int LD_P = L.proj.N;
            NVX_TRY(nvx_linear(L.proj, x_, W, T, nvx_a_, LD_P, MMB_STORE, nullptr, 1.0f, L.norm1));
            MlstmArgs ma{};
            ma.p = nvx_a_; ma.ld_p = LD_P; ma.o = nvx_o_; ma.ld_o = H * L.vdim; ma.H = H; ma.D = L.dim; ma.VD = L.vdim; ma.gate_cap = L.gate_cap;
            ma.i_bias = L.i_bias; ma.f_bias = L.f_bias; ma.S = nvx_S_[(size_t)r.plane]; ma.n = nvx_n_[(size_t)r.plane]; ma.m = nvx_m_[(size_t)r.plane];
            NVX_TRY(launch_mlstm_gates(ma, T, stream_));
            const size_t TU = cp.n_ubatch;
            for (const auto &wv : nvx_waves_) {
                ma.seg_start = d_seg_ + wv.first; ma.seg_len = d_seg_ + TU + wv.first; ma.seg_slot = d_seg_ + 2 * TU + wv.first; ma.n_seg = wv.second;
                NVX_TRY(launch_mlstm_scan(ma, stream_));
            }
            NVX_TRY(launch_mlstm_out(nvx_o_, H * L.vdim, nvx_a_, LD_P, 2 * H * L.dim + H * L.vdim, L.mix_norm, T, H, L.vdim, eps, nvx_att_, H * L.vdim, stream_));
            NVX_TRY(nvx_linear(L.o, nvx_att_, H * L.vdim, T, nvx_y_, W));
            prof_mark("mlstm");
        } else if (L.type == NVX_GQ) {
            NVX_TRY(nvx_linear(L.proj, x_, W, T, nvx_a_, L.proj.N, MMB_STORE, nullptr, 1.0f, L.norm1, L.proj_bias));
            NVX_TRY(nvx_gq_attention(L, r, T));
        } else if (L.type == NVX_DELTA) {
            NVX_TRY(nvx_delta_mixer(L, r, T));
        } else if (L.type == NVX_RETENTION) {
            NVX_TRY(nvx_retention_mixer(L, r, T));
        } else return hipErrorInvalidValue;
        // norm on the sublayer's output, added to the stream (norm1 / norm2 in front of a sublayer are nullptr in a design whose sublayers read the stream itself)
        NVX_TRY(launch_rmsnorm_f32(nvx_y_, W, L.norm1b, 1.0f, x_, x_, W, W, T, eps, stream_));
        if (L.ff_kind != NVX_FF_NONE) {
            bool closed = false;
            NVX_TRY(nvx_feed_forward(L, T, &closed));
            if (!closed) NVX_TRY(launch_rmsnorm_f32(nvx_y_, W, L.norm2b, 1.0f, x_, x_, W, W, T, eps, stream_));
            prof_mark("feed_forward");
        }
        if (debug_taps_ && dbg_) NVX_TRY(hipMemcpyAsync(dbg_ + (size_t)ir * cp.n_ubatch * W, x_, (size_t)T * W * 4, hipMemcpyDeviceToDevice, stream_));
        ir++;
    }
    return hipSuccess;
}

hipError_t Context::run_output_novorax(int n_out, int out_base) {
    logits_on_host_ = false;
    if (n_out <= 0) return hipSuccess;
    const NovoraxModel &M = *model->nvx;
    const int W = M.width, V = M.n_vocab;
    float *const xo = cur_T_ == 1 && n_out == 1 ? x_ : xo_;
    if (xo != x_) NVX_TRY(launch_gather_rows_f32(x_, d_outrow_, n_out, W, xo_, stream_));
    float *lg = d_logits_ + (size_t)out_base * V;
    NVX_TRY(nvx_linear(M.head, xo, W, n_out, lg, V, MMB_STORE, nullptr, M.logit_scale, M.final_norm));
    prof_mark("lm_head");
    for (int r0 = 0; r0 < n_out; r0 += (int)cp.n_ubatch) {
        const int nr = std::min((int)cp.n_ubatch, n_out - r0);
        NVX_TRY(launch_argmax_rows(lg + (size_t)r0 * V, V, nr, h_argmax_ + out_base + r0, argmax_scratch_, (int)cp.n_ubatch, stream_));
    }
    prof_mark("argmax");
    return hipSuccess;
}

}  // namespace mi355
