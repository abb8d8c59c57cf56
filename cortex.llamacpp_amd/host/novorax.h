// novorax.h — the layer stack of the folder models (config.json + model.safetensors, bf16 weights) as this runtime holds it.  Four designs fill it.
//
// Novorax: a decoder whose layers each pick a token mixer (latent attention with a sliding window and a
// softmax sink, or the mLSTM matrix-memory recurrence) and a feed-forward (dense relu^2, or experts chosen by a token-id table), norms on both sides of every
// sublayer, and an optional span of layers that runs several times with shared weights, re-fed with the embedding output through an input projection.
//
// Read from a folder: config.json (every size and constant) + model.safetensors (bf16 matrices, int32 tables).  Weights stay bf16 on the device; vectors
// (norm weights, biases, sinks, rotary frequency tables) are widened to f32 at load.  A "layer run" is one execution of a layer: a looped layer has one run
// per pass, each with its own cache plane or recurrent state.
//
// Fidepel: every layer is ONE block - h = norm(x) with a one-number weight, x += m * (mixer(h) + feed_forward(h)) - whose mixer is grouped-query attention
// (RMS norm over the whole query and the whole key projection, rotate-half rotary positions on part of each head with linearly scaled frequencies, a score
// multiplier per head, a sliding window, a sigmoid output gate per head) and whose feed-forward is a routed mixture of relu^2 experts (softmax scores, expert
// groups of which only the best stay open, renormalised and scaled weights) plus an always-on shared expert; a span of layers may run several times with
// shared weights and nothing between the passes.
//
// Tuterax: every sublayer reads the stream itself and is normed on its OUTPUT (x += norm(mixer(x)), x += norm(ff(x)), zero-centred norm weights).  Mixers:
// grouped-query attention over every earlier token with RMS-normed queries and keys per head (one weight vector shared by the heads), rotate-half rotary positions
// on part of each head, values stored turned by their position and the weighted sum turned back by the query's, a soft cap on the scores, a per-head softmax
// sink; or the gated delta rule (short causal convolutions + silu on q / k / v, unit keys and queries, a write strength beta, a decay per head - "delta" - or per
// head and key channel through a low-rank projection - "channel_delta" -, per-head unit-RMS output with a silu or a low-rank sigmoid gate).  Feed-forward:
// W_down (gelu_tanh(W_gate x) * (W_up x)), or none.  The embedding rows enter times a constant and the same table is the output head.
//
// Dinilorn: norms on both sides of every sublayer (zero-centred weights).  Mixers: retention (linear attention with one fixed decay per head, rotate-half
// rotary positions on q / k, keys over sqrt(dim), per-head unit-RMS output times silu(gate)); attention over every earlier token with projection biases, a
// query multiplier that grows with the logarithm of the position, a soft cap, a learned bias per (distance bucket, head), one more term of score 0 in the softmax
// denominator and a sigmoid gate per head; two-map attention (two score maps per head over the same values, neighbour-pair rotary positions with
// three-band frequency scaling, a sliding window that keeps the first positions, a1 - lambda a2 normed per head, a sigmoid gate per entry).  Feed-forward:
// experts g sigmoid(1.702 g) (u + 1) with clamped g, u; router = sigmoid scores, a selection bias that picks but does not weigh, expert groups scored by their two
// best, un-normalised weights; a shared expert behind a one-number sigmoid gate.  A span of layers may run several times with shared weights; every pass but
// the first opens with the embedding rows added to the stream.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace mi355 {

struct BfMat {                      // bf16 rows on the device
    unsigned short *w = nullptr;
    int N = 0, K = 0;               // rows (outputs), row length (inputs)
};

enum { NVX_LATENT = 0, NVX_MLSTM = 1, NVX_GQ = 2, NVX_DELTA = 3, NVX_RETENTION = 4 };   // token mixers: latent attention, matrix-memory recurrence, grouped-query attention, gated delta rule, retention
enum { NVX_ROUTE_SOFTMAX_GROUPS = 0, NVX_ROUTE_SIGMOID_BIAS = 1 };   // routers of NVX_FF_ROUTED: softmax scores, groups by their best, normalised weights | sigmoid scores + selection bias, groups by their two best, raw weights
enum { NVX_FF_NONE = 0, NVX_FF_DENSE = 1, NVX_FF_EXPERTS = 2, NVX_FF_ROUTED = 3 };   // dense; experts by a token-id table; experts by a router

struct NvxLayer {
    int type = NVX_LATENT;
    // mixer sizes (latent attention: all; mlstm: heads, dim, vdim, gate_cap)
    int heads = 0, dim = 0, vdim = 0, rot = 0, kv_rank = 0, q_rank = 0, window = 0, rot_dims = 0;
    float scale = 1.0f, rot_mscale = 1.0f, gate_cap = 1.0f;
    float *rot_freq = nullptr;      // [rot_dims / 2] radians per position
    // norm weights in front of the mixer / the feed-forward (norm1, norm2; nullptr: the sublayer reads the stream itself) and behind them (norm1b, norm2b)
    float *norm1 = nullptr, *norm1b = nullptr, *norm2 = nullptr, *norm2b = nullptr;
    // latent attention: down = [dq ; dkv] rows, uk_t = per head [kv_rank][dim] (W_uk transposed inside each head), uv = per head [vdim][kv_rank]
    BfMat down, uq, uk_t, uv, o;
    float *dq_norm = nullptr, *dkv_norm = nullptr, *sink = nullptr;
    // mlstm: proj = [q ; k ; v ; g ; i ; f] rows
    BfMat proj;
    float *mix_norm = nullptr, *i_bias = nullptr, *f_bias = nullptr;
    // feed-forward
    int ff_kind = NVX_FF_NONE, ff = 0, n_expert = 0, top = 0;
    BfMat up, down_ff;              // dense; experts: gate / up packed [n_expert][ff][width], down packed [n_expert][width][ff]
    BfMat e_gate, e_up, e_down;
    int32_t *table = nullptr;       // [n_vocab][top]
    // grouped-query attention: proj = [q: heads*dim ; k: kv_heads*dim ; v: kv_heads*vdim ; g: heads ; router: n_expert] rows, one product per block
    // (proj above); q_norm / k_norm over the whole projection; head_scale = the per-head score multiplier; the gate and router columns start at off_gate / off_router
    int kv_heads = 0, off_gate = -1, off_router = -1;
    float *q_norm = nullptr, *k_norm = nullptr, *head_scale = nullptr;
    // ... with q_norm / k_norm per head instead ([dim] weights shared by the heads), a soft cap on the scores (0: none), values stored turned by their position
    // (v_rot_freq: [vdim / 2] radians per position, nullptr: plain values)
    bool qk_norm_per_head = false;
    float softcap = 0.0f;
    float *v_rot_freq = nullptr;
    // gated delta rule: proj = [q: kv_heads*dim ; k: kv_heads*dim ; v: heads*vdim ; beta: heads ; then a: heads ; g: heads*vdim  (one decay per head, silu gate)
    //                                                                               or   a1: rank_a ; g1: rank_g  (decay per key channel and sigmoid gate, both
    // through a second projection a2 [heads*dim][rank_a], g2 [heads*vdim][rank_g])]; conv_w [2*kv_heads*dim + heads*vdim][conv_taps] f32 in proj's channel order
    bool decay_per_channel = false;
    int conv_taps = 0, off_beta = -1, off_a = -1, off_g = -1, rank_a = 0, rank_g = 0;
    float *conv_w = nullptr, *A_log = nullptr, *dt_bias = nullptr;
    BfMat a2, g2;
    // dense feed-forward with a gate: down_ff (act(gate x) * (up x)); gate.w == nullptr: the plain form above
    BfMat gate;
    int delta_channels() const { return 2 * kv_heads * dim + heads * vdim; }
    // routed experts (e_up [n_expert][ff][width] with relu^2, e_down [n_expert][width][ff]): groups of neighbouring experts, the `group_keep` best stay open;
    // weights s / sum * router_scale; the shared expert s_up / s_down (shared_ff 0: none) runs for every token
    int n_group = 1, group_keep = 1, shared_ff = 0;
    float router_scale = 1.0f;
    BfMat s_up, s_down;
    // ... with another router (route_kind; route_bias [n_expert] joins the scores for the choice only), gated experts (e_gate set: g sigmoid(1.702 g) (u + 1),
    // g, u clamped by expert_limit; s_gate / shared_limit for the shared expert), and for a feed-forward that reads its own norm: route = [router ; shared gate]
    // rows as a projection of its own (off_sg: the column of the shared expert's one-number sigmoid gate, -1: none)
    int route_kind = NVX_ROUTE_SOFTMAX_GROUPS, off_sg = -1;
    float *route_bias = nullptr;
    float expert_limit = 0.0f, shared_limit = 0.0f;
    BfMat route, s_gate;
    // grouped-query attention, further switches: biases of the fused projection (zeros under the gate rows) and of W_o; a query multiplier
    // 1 + q_temp_coef ln(floor((p + 1) / q_temp_every) + 1) (every 0: none); rel [rel_rows][heads] added to the score by distance bucket (dist_bucket [n_dist],
    // longer distances take the last row); the first keep_first positions stay seen outside the window; rotary pairs (2i, 2i + 1); maps = 2: two score maps
    // per head ([head][map][dim] rows of q and k) joined as unit_rms(a1 - map_lambda a2) * map_mult; the gate holds one number per output entry
    float *proj_bias = nullptr, *o_bias = nullptr;
    float q_temp_coef = 0.0f, q_temp_every = 0.0f;
    float *rel = nullptr; int32_t *dist_bucket = nullptr; int n_dist = 0, rel_rows = 0;
    int keep_first = 0, maps = 1;
    bool rot_neighbours = false, gate_per_entry = false;
    float map_lambda = 0.0f, map_mult = 1.0f;
    // retention: proj = [q: heads*dim ; k: heads*dim ; v: heads*vdim ; g: heads*vdim] rows (off_g: the gate's column), decay [heads]; rot_dims / rot_freq as above
    float *decay = nullptr;
    int cache_row() const { return type == NVX_LATENT ? kv_rank + rot : type == NVX_GQ ? kv_heads * (maps * dim + vdim) : 0; }   // f32 per cell of a run's cache plane
};

struct NvxRun {
    int layer = 0;
    int pass = -1;                  // >= 0: first layer of loop pass `pass` (input projection + step vector come first)
    int plane = -1;                 // attention mixers: index of this run's cache plane; recurrent mixers: of its state set
};

struct NovoraxModel {
    std::vector<NvxLayer> layers;
    std::vector<NvxRun> runs;
    BfMat embed, head, loop_in;
    float *loop_step = nullptr;     // [times][width]
    float *final_norm = nullptr;
    float logit_scale = 1.0f, eps = 1e-5f, embed_scale = 1.0f;
    std::string design;             // "novorax" | "fidepel" | "tuterax" | "dinilorn"
    bool loop_add_embed = false;    // every pass of the looped span but the first opens with x += embedding rows
    int max_keep_first = 0;         // most first positions a windowed layer keeps seen (scan bounds)
    // norm weights: the factor is norm_off + w (1: zero-centred weights, 0: plain ones).  parallel_block: one norm per layer, mixer and feed-forward both read
    // it, x += residual_mult * (their sum); otherwise norms on both sides of each sublayer
    float norm_off = 1.0f, residual_mult = 1.0f;
    bool parallel_block = false;
    int width = 0, n_vocab = 0;
    int n_cache_runs = 0, n_state_runs = 0;   // attention runs (cache planes) and recurrent runs (state sets per sequence slot)
    int max_window = 0;             // largest window of the windowed attention layers, 0 if one of them sees every earlier cell (scan bounds)
    int max_shared_ff = 0;
    // largest sizes over the layers (activation buffers)
    int max_down = 0, max_q_rank = 0, max_q = 0, max_qa = 0, max_att = 0, max_proj = 0, max_ff = 0, max_top = 0, max_expert = 0;
};

}  // namespace mi355
