// gq_attn.hip — grouped-query attention with a sliding window on f32 cache rows, for the bf16-weight models.
//
// A token's cache row is [k_0 .. k_{G-1} | v_0 .. v_{G-1}]: G key heads of dim floats, then G value heads of vdim floats; query head h reads key / value
// head h / (H / G).  Visibility: same sequence, 0 <= pos_query - pos_cell < window (window 0: every earlier cell).  Plain softmax over the visible cells; an
// optional soft cap squashes every score to cap * tanh(score / cap) first; an optional per-head sink logit joins the denominator; an optional output gate
// multiplies head h's result by sigmoid(gate[t][h]).  Everything here is f32: positions, angles, norms, scores, weights, the running sums.
//
// gq_prep: per token, behind the fused q | k | v projection: an optional RMS norm of the queries and of the keys with plain weights - over the WHOLE projection
// (all heads at once) or over every head by itself with one weight vector shared by the heads; the rotation of the first rot_dims entries of every query and
// key head in the rotate-half layout (entry i pairs with entry i + rot_dims / 2; the per-pair angle table comes from the host); the score multipliers (one
// number for the layer, one per head) folded into the query; keys and values stored to the token's cache row.
//
// Optional per layer: a query multiplier that grows with the logarithm of the position (in steps of `every` positions); a learned bias per (distance bucket,
// head) added to the score behind the soft cap (the host hands over the distance -> bucket table); cells at the first `keep_first` positions that stay seen
// outside the window; the neighbour layout of the rotation (entry 2i with 2i + 1); several score maps per head over the same values - every (head, map) then
// runs as a query head of its own with its own key head, and gq_maps_out joins two maps: a1 - lambda a2, unit RMS, a constant, an elementwise sigmoid gate.
//
// Turned values (optional): every value head is stored turned by its own position over all its entries, in the same half-and-half pairing; the weighted sum
// of a row is turned back by the row's position - each term then carries the turn by (key position - query position), a relative position signal on the
// value side.  The turn back happens where a row's result is finished: in the per-row kernel, in the merge of split scans, or in gq_unturn behind the tiled pass.
#include "kernels.h"

namespace mi355 {

namespace {

__device__ __forceinline__ float gq_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ float gq_block_sum_256(float v, float *sh) {
    v = gq_wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    return (sh[0] + sh[1]) + (sh[2] + sh[3]);
}

constexpr int GQ_MAX_D = 512;                                   // dim and vdim the attention kernel is instantiated for (8 x 64)

__global__ __launch_bounds__(256) void gq_prep_kernel(GqPrepArgs a) {
    extern __shared__ float head_inv[];                         // norm per head: [H + G] inverse root mean squares
    __shared__ float sh[4];
    __shared__ float cs[2][GQ_MAX_D / 2];                       // cos / sin of the token's angle per pair: computed once, read by every head
    __shared__ float csv[2][GQ_MAX_D / 2];                      // the same for the value heads' pairs
    const int t = blockIdx.x, tid = threadIdx.x;
    const int GK = a.G * (a.maps > 1 ? a.maps : 1);             // key heads: one per (value head, map)
    const int NQ = a.H * a.dim, NK = GK * a.dim, NV = a.G * a.vdim, half = a.rot_dims >> 1;
    const float *qr = a.p + (size_t)t * a.ld_p, *kr = qr + NQ, *vr = kr + NK;
    float inv_q = 1.0f, inv_k = 1.0f;
    const bool per_head = a.norm_per_head && a.wq_norm && a.wk_norm;
    if (per_head) {
        // sixteen lanes per head, queries then keys (q | k lie side by side in the row): every lane group's loads are on their way at once
        for (int hh = tid >> 4; hh < a.H + GK; hh += 16) {
            const float *src = qr + (size_t)hh * a.dim;
            float ss = 0.0f;
            for (int i = tid & 15; i < a.dim; i += 16) { const float v = src[i]; ss = fmaf(v, v, ss); }
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
            if ((tid & 15) == 0) head_inv[hh] = 1.0f / sqrtf(ss / (float)a.dim + a.eps);
        }
    } else if (a.wq_norm) {
        float ss = 0.0f;
        for (int i = tid; i < NQ; i += 256) { const float v = qr[i]; ss = fmaf(v, v, ss); }
        inv_q = 1.0f / sqrtf(gq_block_sum_256(ss, sh) / (float)NQ + a.eps);
    }
    if (!per_head && a.wk_norm) {
        float ss = 0.0f;
        for (int i = tid; i < NK; i += 256) { const float v = kr[i]; ss = fmaf(v, v, ss); }
        inv_k = 1.0f / sqrtf(gq_block_sum_256(ss, sh) / (float)NK + a.eps);
    }
    const float p = (float)a.tok_pos[t];
    // (positions are exact in f32 up to 2^24, and so is the floor of the correctly rounded quotient for a whole-number step)
    const float q_temp = a.q_temp_every > 0.0f ? 1.0f + a.q_temp_coef * logf(floorf((p + 1.0f) / a.q_temp_every) + 1.0f) : 1.0f;
    if (tid < half) sincosf(p * a.rot_freq[tid], &cs[1][tid], &cs[0][tid]);
    const int vhalf = a.v_rot_freq ? a.vdim >> 1 : 0;
    if (tid >= 128 && tid - 128 < vhalf) {                       // (the upper waves: beside the key / query table of the lower ones)
        const int j = tid - 128;
        sincosf(p * a.v_rot_freq[j], &csv[1][j], &csv[0][j]);
        if (a.v_cs) { a.v_cs[(size_t)t * a.vdim + j] = csv[0][j]; a.v_cs[(size_t)t * a.vdim + vhalf + j] = csv[1][j]; }
    }
    for (int j = 128 + tid; j < vhalf; j += 256) {              // (value heads beyond 256 entries)
        sincosf(p * a.v_rot_freq[j], &csv[1][j], &csv[0][j]);
        if (a.v_cs) { a.v_cs[(size_t)t * a.vdim + j] = csv[0][j]; a.v_cs[(size_t)t * a.vdim + vhalf + j] = csv[1][j]; }
    }
    __syncthreads();
    float *qo = a.q + (size_t)t * a.ld_q;
    float *row = a.cache + (size_t)a.tok_cell[t] * (size_t)(NK + NV);
    // one loop over the query entries, then the key entries: element (head, d) of either
    for (int i = tid; i < NQ + NK; i += 256) {
        const bool isq = i < NQ;
        const int e = isq ? i : i - NQ, d = e % a.dim, b = e - d;
        const float *src = isq ? qr : kr;
        const float *wn = isq ? a.wq_norm : a.wk_norm;
        const float inv = per_head ? head_inv[i / a.dim] : isq ? inv_q : inv_k;
        const int wb = per_head ? 0 : b;                         // (a shared weight vector starts over with every head)
        float o;
        if (d < a.rot_dims && a.rot_neighbours) {
            const int j = d >> 1;
            const float c = cs[0][j], s = cs[1][j];
            float u = src[b + 2 * j] * inv, w = src[b + 2 * j + 1] * inv;
            if (wn) { u *= wn[wb + 2 * j]; w *= wn[wb + 2 * j + 1]; }
            o = (d & 1) == 0 ? u * c - w * s : w * c + u * s;
        } else if (d < a.rot_dims) {
            const int j = d < half ? d : d - half;
            const float c = cs[0][j], s = cs[1][j];
            float u = src[b + j] * inv, w = src[b + j + half] * inv;
            if (wn) { u *= wn[wb + j]; w *= wn[wb + j + half]; }
            o = d < half ? u * c - w * s : w * c + u * s;
        } else {
            o = src[e] * inv;
            if (wn) o *= wn[wb + d];
        }
        if (isq) {
            float m = a.q_scale * q_temp;
            if (a.head_scale) m *= a.head_scale[e / a.dim];
            qo[e] = o * m;
        } else row[e] = o;
    }
    if (!a.v_rot_freq) {
        for (int i = tid; i < NV; i += 256) row[NK + i] = vr[i];
        return;
    }
    for (int i = tid; i < NV; i += 256) {
        const int d = i % a.vdim, b = i - d;
        const int j = d < vhalf ? d : d - vhalf;                 // (vdim is even: every entry has a partner)
        const float c = csv[0][j], s = csv[1][j], u = vr[b + j], w = vr[b + j + vhalf];
        row[NK + i] = d < vhalf ? u * c - w * s : w * c + u * s;
    }
}

// entry i (and its partner i + vdim / 2) of a finished head output: the pair turns back by the row's position
__device__ __forceinline__ void gq_unturn_pair(float &u, float &w, float c, float s) {
    const float x = u * c + w * s, y = w * c - u * s;
    u = x; w = y;
}

// behind the tiled pass: out[t][h] turned back in place (the gate, one factor per head, commutes with the turn)
__global__ __launch_bounds__(256) void gq_unturn_kernel(GqAttnArgs a) {
    const int t = blockIdx.x, h = blockIdx.y, vhalf = a.vdim >> 1;
    float *o = a.out + (size_t)t * a.ld_out + (size_t)h * a.vdim;
    const float *cs = a.v_cs + (size_t)t * a.vdim;
    for (int i = threadIdx.x; i < vhalf; i += 256) {
        float u = o[i], w = o[i + vhalf];
        gq_unturn_pair(u, w, cs[i], cs[vhalf + i]);
        o[i] = u; o[i + vhalf] = w;
    }
}

// where query head h (a (head, map) pair when a.maps > 1) finds its key head and its value head inside a cache row, and the row's length
struct GqHeads { size_t row, koff, voff; };
__device__ __forceinline__ GqHeads gq_heads(const GqAttnArgs &a, int h) {
    const int maps = a.maps > 1 ? a.maps : 1, head = h / maps, map = h - head * maps, kvh = head / ((a.H / maps) / a.G);
    GqHeads o;
    o.row = (size_t)a.G * ((size_t)maps * a.dim + a.vdim);
    o.koff = ((size_t)kvh * maps + map) * a.dim;
    o.voff = (size_t)a.G * maps * a.dim + (size_t)kvh * a.vdim;
    return o;
}
// the learned bias of head h at distance dist >= 0
__device__ __forceinline__ float gq_rel_bias(const GqAttnArgs &a, int dist, int h) {
    const int b = dist < a.n_dist ? a.dist_bucket[dist] : a.rel_rows - 1;
    return a.rel[(size_t)b * a.H + h];
}

// y[t][h] = unit_rms(a1 - lambda a2) * out_mult * sigmoid(gate[t][h]) entry by entry; a1, a2 = the two maps' outputs of head h
__global__ __launch_bounds__(64) void gq_maps_out_kernel(const float *att, int ld_att, const float *gate, int ld_gate, int VD, float lambda, float out_mult, float eps,
                                                         float *y, int ld_y) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float *a1 = att + (size_t)t * ld_att + (size_t)(2 * h) * VD, *a2 = a1 + VD;
    float ss = 0.0f;
    for (int i = lane; i < VD; i += 64) { const float o = a1[i] - lambda * a2[i]; ss = fmaf(o, o, ss); }
    ss = gq_wave_sum(ss);
    const float inv = out_mult / sqrtf(ss / (float)VD + eps);
    for (int i = lane; i < VD; i += 64) {
        const float o = a1[i] - lambda * a2[i];
        const float g = gate ? 1.0f / (1.0f + expf(-gate[(size_t)t * ld_gate + (size_t)h * VD + i])) : 1.0f;
        y[(size_t)t * ld_y + (size_t)h * VD + i] = o * inv * g;
    }
}

// One workgroup per (token, head), NW waves.  A wave works on four cells at a time: each 16-lane group owns one cell, its lanes hold elements
// 64 j + 4 li .. + 3 of the key head and of the value head (16-byte loads) and the matching running sums; the next four cells of the wave are requested
// before the current ones are used.  Every group keeps its own running maximum / sum / weighted value; groups, then waves, are merged at the end together
// with the sink term and the output gate.  NJ = ceil(max(dim, vdim) / 64); VEC: key and value heads start on 16-byte boundaries.
template <int NJ, bool VEC>
__global__ __launch_bounds__(512) void gq_attn_kernel(GqAttnArgs a) {
    extern __shared__ float lds[];
    const int D = a.dim, VD = a.vdim, LP = NJ * 64;
    const int NW = blockDim.x >> 6;
    float *qv = lds;                                            // [LP] (zero beyond dim)
    float *wm = lds + LP, *wl = wm + NW, *wacc = wl + NW;        // [NW], [NW], [NW][LP]
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, li = lane & 15;
    const GqHeads hd = gq_heads(a, h);
    const size_t L = hd.row, koff = hd.koff, voff = hd.voff;
    const int tpos = a.tok_pos[t];
    const uint64_t sbit = 1ull << (a.tok_seq[t] & 63);
    for (int i = tid; i < LP; i += blockDim.x) qv[i] = i < D ? a.q[(size_t)t * a.ld_q + (size_t)h * D + i] : 0.0f;
    __syncthreads();
    float acc[NJ][4], ck[NJ][4], cv[NJ][4], nk[NJ][4], nv[NJ][4];
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) { acc[j][e] = 0.0f; ck[j][e] = 0.0f; cv[j][e] = 0.0f; nk[j][e] = 0.0f; nv[j][e] = 0.0f; }
    float m = -INFINITY, l = 0.0f;
    int n_kv = *a.n_kv_dev;
    if (a.tok_hi) n_kv = a.tok_hi[t] < n_kv ? a.tok_hi[t] : n_kv;
    const int stride = NW * 4;
    // the scanned cells: [first cell that can still be inside the token's window, one past the token's own cells); gridDim.z > 1 (steps of a few tokens)
    // cuts them into that many runs, one workgroup each, whose records gq_attn_merge_kernel joins
    int c_lo = a.tok_lo ? a.tok_lo[t] : 0, c_hi = n_kv;
    if (c_lo > c_hi) c_lo = c_hi;
    if (gridDim.z > 1) {
        const int per = ((c_hi - c_lo + (int)gridDim.z - 1) / (int)gridDim.z + stride - 1) / stride * stride;
        c_lo += (int)blockIdx.z * per;
        c_hi = c_lo + per < c_hi ? c_lo + per : c_hi;
    }
    const auto visible = [&](int c, int &dist) {
        if (c >= c_hi) return false;
        const int cp = a.cell_pos[c];
        dist = tpos - cp;
        return cp >= 0 && cp <= tpos && (a.cell_seq[c] & sbit) != 0 && !(a.window > 0 && tpos - cp >= a.window && cp >= a.keep_first);
    };
    const auto fetch = [&](int c, bool vis, float (&dk)[NJ][4], float (&dv)[NJ][4]) {
        const float *kr = a.cache + (size_t)c * L + koff, *vr = a.cache + (size_t)c * L + voff;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int e0 = 64 * j + 4 * li;
            if (VEC) {
                float4 k4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f), v4 = k4;
                if (vis && e0 < D) k4 = *reinterpret_cast<const float4 *>(kr + e0);
                if (vis && e0 < VD) v4 = *reinterpret_cast<const float4 *>(vr + e0);
                dk[j][0] = k4.x; dk[j][1] = k4.y; dk[j][2] = k4.z; dk[j][3] = k4.w;
                dv[j][0] = v4.x; dv[j][1] = v4.y; dv[j][2] = v4.z; dv[j][3] = v4.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    dk[j][e] = vis && e0 + e < D ? kr[e0 + e] : 0.0f;
                    dv[j][e] = vis && e0 + e < VD ? vr[e0 + e] : 0.0f;
                }
            }
        }
    };
    int c = c_lo + wave * 4 + g, dist = 0, distn = 0;
    bool vis = visible(c, dist);
    fetch(c, vis, ck, cv);
    for (int c0 = c_lo; c0 < c_hi; c0 += stride) {              // (uniform trip count: the shuffles below are executed by whole waves)
        const int cn = c + stride;
        const bool visn = visible(cn, distn);
        fetch(cn, visn, nk, nv);
        float dot = 0.0f;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const float4 q4 = *reinterpret_cast<const float4 *>(qv + 64 * j + 4 * li);
            dot = fmaf(ck[j][0], q4.x, dot); dot = fmaf(ck[j][1], q4.y, dot); dot = fmaf(ck[j][2], q4.z, dot); dot = fmaf(ck[j][3], q4.w, dot);
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64);
        if (a.softcap > 0.0f) dot = a.softcap * tanhf(dot / a.softcap);
        if (vis) {
            if (a.rel) dot += gq_rel_bias(a, dist, h);
            const float mn = fmaxf(m, dot), alpha = expf(m - mn), p = expf(dot - mn);   // (m = -inf at the group's first cell: alpha = 0)
            l = l * alpha + p;
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[j][e] = acc[j][e] * alpha + p * cv[j][e];
            m = mn;
        }
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) { ck[j][e] = nk[j][e]; cv[j][e] = nv[j][e]; }
        c = cn; vis = visn; dist = distn;
    }
    // the four groups of a wave -> one record per wave
    float M = fmaxf(m, __shfl_xor(m, 16, 64));
    M = fmaxf(M, __shfl_xor(M, 32, 64));
    const float sg = l > 0.0f ? expf(m - M) : 0.0f;
    l *= sg;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float v = acc[j][e] * sg;
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            if (g == 0) wacc[wave * LP + 64 * j + 4 * li + e] = v;
        }
    if (lane == 0) { wm[wave] = M; wl[wave] = l; }
    __syncthreads();
    if (gridDim.z > 1) {                                        // this run's record: maximum, sum, weighted value (sink and gate enter at the merge)
        float *rec = a.part + (((size_t)t * a.H + h) * gridDim.z + blockIdx.z) * (size_t)(VD + 2);
        float Ms = -INFINITY;
        for (int w = 0; w < NW; w++) if (wl[w] > 0.0f) Ms = fmaxf(Ms, wm[w]);
        float ls = 0.0f;
        for (int w = 0; w < NW; w++) ls += wl[w] > 0.0f ? wl[w] * expf(wm[w] - Ms) : 0.0f;
        if (tid == 0) { rec[0] = Ms; rec[1] = ls; }
        for (int i = tid; i < VD; i += blockDim.x) {
            float o = 0.0f;
            for (int w = 0; w < NW; w++) o += wl[w] > 0.0f ? wacc[w * LP + i] * expf(wm[w] - Ms) : 0.0f;
            rec[2 + i] = o;
        }
        return;
    }
    float MM = a.sink ? a.sink[h] : -INFINITY;
    for (int w = 0; w < NW; w++) if (wl[w] > 0.0f) MM = fmaxf(MM, wm[w]);
    float den = a.sink ? expf(a.sink[h] - MM) : 0.0f;
    for (int w = 0; w < NW; w++) den += wl[w] > 0.0f ? wl[w] * expf(wm[w] - MM) : 0.0f;
    float inv = den > 0.0f ? 1.0f / den : 0.0f;
    if (a.gate) inv *= 1.0f / (1.0f + expf(-a.gate[(size_t)t * a.ld_gate + h]));
    if (a.v_cs) {                                               // (vdim is even)
        const int vhalf = VD >> 1;
        const float *cs = a.v_cs + (size_t)t * VD;
        for (int i = tid; i < vhalf; i += blockDim.x) {
            float o = 0.0f, o2 = 0.0f;
            for (int w = 0; w < NW; w++) {
                const float f = wl[w] > 0.0f ? expf(wm[w] - MM) : 0.0f;
                o += wacc[w * LP + i] * f;
                o2 += wacc[w * LP + i + vhalf] * f;
            }
            gq_unturn_pair(o, o2, cs[i], cs[vhalf + i]);
            a.out[(size_t)t * a.ld_out + (size_t)h * VD + i] = o * inv;
            a.out[(size_t)t * a.ld_out + (size_t)h * VD + i + vhalf] = o2 * inv;
        }
        return;
    }
    for (int i = tid; i < VD; i += blockDim.x) {
        float o = 0.0f;
        for (int w = 0; w < NW; w++) o += wl[w] > 0.0f ? wacc[w * LP + i] * expf(wm[w] - MM) : 0.0f;
        a.out[(size_t)t * a.ld_out + (size_t)h * VD + i] = o * inv;
    }
}

__global__ __launch_bounds__(256) void gq_attn_merge_kernel(GqAttnArgs a, int splits) {
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, VD = a.vdim;
    const float *rec = a.part + ((size_t)t * a.H + h) * splits * (size_t)(VD + 2);
    float MM = a.sink ? a.sink[h] : -INFINITY;
    for (int s = 0; s < splits; s++) if (rec[(size_t)s * (VD + 2) + 1] > 0.0f) MM = fmaxf(MM, rec[(size_t)s * (VD + 2)]);
    float den = a.sink ? expf(a.sink[h] - MM) : 0.0f;
    for (int s = 0; s < splits; s++) { const float *r = rec + (size_t)s * (VD + 2); den += r[1] > 0.0f ? r[1] * expf(r[0] - MM) : 0.0f; }
    float inv = den > 0.0f ? 1.0f / den : 0.0f;
    if (a.gate) inv *= 1.0f / (1.0f + expf(-a.gate[(size_t)t * a.ld_gate + h]));
    if (a.v_cs) {                                               // (vdim is even)
        const int vhalf = VD >> 1;
        const float *cs = a.v_cs + (size_t)t * VD;
        for (int i = tid; i < vhalf; i += 256) {
            float o = 0.0f, o2 = 0.0f;
            for (int s = 0; s < splits; s++) {
                const float *r = rec + (size_t)s * (VD + 2);
                const float f = r[1] > 0.0f ? expf(r[0] - MM) : 0.0f;
                o += r[2 + i] * f;
                o2 += r[2 + i + vhalf] * f;
            }
            gq_unturn_pair(o, o2, cs[i], cs[vhalf + i]);
            a.out[(size_t)t * a.ld_out + (size_t)h * VD + i] = o * inv;
            a.out[(size_t)t * a.ld_out + (size_t)h * VD + i + vhalf] = o2 * inv;
        }
        return;
    }
    for (int i = tid; i < VD; i += 256) {
        float o = 0.0f;
        for (int s = 0; s < splits; s++) { const float *r = rec + (size_t)s * (VD + 2); o += r[1] > 0.0f ? r[2 + i] * expf(r[0] - MM) : 0.0f; }
        a.out[(size_t)t * a.ld_out + (size_t)h * VD + i] = o * inv;
    }
}

template <int NJ>
static hipError_t launch_gq_attn_nj(const GqAttnArgs &a, hipStream_t st) {
    // few (token, head) pairs - steps of a few tokens - get eight waves each: more cells in flight where the grid alone cannot fill the device
    const int nw = (long long)a.T * a.H <= 1024 ? 8 : 4;
    const size_t lds = (size_t)(NJ * 64 + 2 * nw + nw * NJ * 64) * sizeof(float);
    const bool vec = (a.dim & 3) == 0 && (a.vdim & 3) == 0 && (reinterpret_cast<uintptr_t>(a.cache) & 15) == 0;
    const int splits = a.part && a.splits > 1 && (size_t)a.T * a.H * a.splits * (a.vdim + 2) <= a.part_floats ? a.splits : 1;
    const dim3 grid((unsigned)a.T, (unsigned)a.H, (unsigned)splits);
    if (vec) hipLaunchKernelGGL((gq_attn_kernel<NJ, true>), grid, dim3(64 * nw), lds, st, a);
    else hipLaunchKernelGGL((gq_attn_kernel<NJ, false>), grid, dim3(64 * nw), lds, st, a);
    if (splits > 1) hipLaunchKernelGGL(gq_attn_merge_kernel, dim3((unsigned)a.T, (unsigned)a.H), dim3(256), 0, st, a, splits);
    return hipGetLastError();
}


// ---- prompt batches: the same attention as one LDS-tiled pass per (tile of 16 * RPT batch rows, head)
// The tile's rows may belong to any sequences at any positions: visibility is decided per (row, cell) pair from the cell table, exactly as above.  The
// scanned cells are walked in blocks of 64; a block none of whose cells can be seen by any row of the tile (wrong sequence, beyond the tile's last position,
// before its first window) costs one read of its cell table entries.  Per block: S = Q K^T in 32-wide slices of the head (both operands through LDS, a
// thread owns RPT rows x 4 cells), the running softmax per row (16 lanes share a row), P to LDS, O += P V in 64-column slices of the value head (a thread
// owns RPT rows x 4 columns per slice).  NVC = ceil(vdim / 64).  dim and vdim multiples of 4.  RPT = 4 (64-row tiles) where that still gives the device
// two workgroups per CU, else 2: a short prompt is bound by the chain of blocks one workgroup walks, not by arithmetic.
constexpr int GQT_B = 64, GQT_DC = 32, GQT_LDQ = GQT_DC + 4, GQT_LDP = GQT_B + 4;
constexpr size_t gqt_lds_floats(int rows) { return (size_t)(rows + GQT_B) * GQT_LDQ + (size_t)(rows + GQT_B) * GQT_LDP + 2 * rows + 3 * GQT_B; }

template <int NVC, int RPT>
__global__ __launch_bounds__(256) void gq_attn_tile_kernel(GqAttnArgs a) {
    constexpr int BQ = 16 * RPT;
    extern __shared__ float lds[];
    float *Qc = lds, *Kc = Qc + BQ * GQT_LDQ, *P = Kc + GQT_B * GQT_LDQ, *Vc = P + BQ * GQT_LDP;
    uint64_t *cseq = reinterpret_cast<uint64_t *>(Vc + GQT_B * GQT_LDP);                     // (an even number of floats in: 8-byte aligned)
    int *cpos = reinterpret_cast<int *>(cseq + GQT_B), *rpos = cpos + GQT_B, *rseq = rpos + BQ;
    __shared__ int red[4];
    const int D = a.dim, VD = a.vdim, tid = threadIdx.x, tq = tid >> 4, tc = tid & 15;
    const int row0 = blockIdx.x * BQ, h = blockIdx.y;
    const GqHeads hd = gq_heads(a, h);
    const size_t L = hd.row, koff = hd.koff, voff = hd.voff;
    const int n_kv = *a.n_kv_dev;
    // the tile's rows: position and sequence of each; over the tile: first and last position, the union of sequences, the range of cells to walk
    int my_lo = 0x7fffffff, my_hi = 0, my_pmin = 0x7fffffff, my_pmax = -1;
    if (tid < BQ) {
        const int r = row0 + tid;
        const bool live = r < a.T;
        rpos[tid] = live ? a.tok_pos[r] : -1;
        rseq[tid] = live ? (a.tok_seq[r] & 63) : -1;
        if (live) {
            my_pmin = my_pmax = rpos[tid];
            my_lo = a.tok_lo ? a.tok_lo[r] : 0;
            my_hi = a.tok_hi ? (a.tok_hi[r] < n_kv ? a.tok_hi[r] : n_kv) : n_kv;
        }
    }
    if (tid < 64) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            my_lo = min(my_lo, __shfl_xor(my_lo, o, 64)); my_hi = max(my_hi, __shfl_xor(my_hi, o, 64));
            my_pmin = min(my_pmin, __shfl_xor(my_pmin, o, 64)); my_pmax = max(my_pmax, __shfl_xor(my_pmax, o, 64));
        }
        if (tid == 0) { red[0] = my_lo; red[1] = my_hi; red[2] = my_pmin; red[3] = my_pmax; }
    }
    __syncthreads();
    int c_begin = red[0] < red[1] ? red[0] : red[1], c_end = red[1];
    const int pmin = red[2], pmax = red[3];
    if (gridDim.z > 1) {                                        // the tile's blocks cut into gridDim.z runs, one workgroup each; gq_attn_merge_kernel joins their records
        const int per = ((c_end - c_begin + GQT_B - 1) / GQT_B + (int)gridDim.z - 1) / (int)gridDim.z * GQT_B;
        c_begin += (int)blockIdx.z * per;
        c_end = c_begin + per < c_end ? c_begin + per : c_end;
    }
    uint64_t seqs = 0;
    for (int r = 0; r < BQ; r++) if (rseq[r] >= 0) seqs |= 1ull << rseq[r];
    float s[RPT][4], o[RPT][NVC * 4], m[RPT], l[RPT];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        m[i] = -INFINITY; l[i] = 0.0f;
#pragma unroll
        for (int e = 0; e < NVC * 4; e++) o[i][e] = 0.0f;
    }
    for (int c0 = c_begin; c0 < c_end; c0 += GQT_B) {
        __syncthreads();                                        // (the previous block's P / V / cell entries are no longer read)
        int any = 0;
        if (tid < GQT_B) {
            const int c = c0 + tid;
            int cp = -1; uint64_t cs = 0;
            if (c < c_end) { cp = a.cell_pos[c]; cs = a.cell_seq[c]; }
            cpos[tid] = cp; cseq[tid] = cs;
            any = cp >= 0 && cp <= pmax && (cs & seqs) != 0 && !(a.window > 0 && pmin - cp >= a.window && cp >= a.keep_first);
        }
        if (!__syncthreads_or(any)) continue;
        // ---- S = Q K^T
#pragma unroll
        for (int i = 0; i < RPT; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) s[i][j] = 0.0f;
        for (int dc = 0; dc < D; dc += GQT_DC) {
            if (dc > 0) __syncthreads();
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int idx = tid + 256 * k, r = idx >> 3, d = dc + (idx & 7) * 4;
                float4 qv = make_float4(0.0f, 0.0f, 0.0f, 0.0f), kv = qv;
                if (d < D) {
                    if (r < BQ && row0 + r < a.T) qv = *reinterpret_cast<const float4 *>(a.q + (size_t)(row0 + r) * a.ld_q + (size_t)h * D + d);
                    if (cpos[r] >= 0) kv = *reinterpret_cast<const float4 *>(a.cache + (size_t)(c0 + r) * L + koff + d);
                }
                if (r < BQ) *reinterpret_cast<float4 *>(Qc + r * GQT_LDQ + (idx & 7) * 4) = qv;
                *reinterpret_cast<float4 *>(Kc + r * GQT_LDQ + (idx & 7) * 4) = kv;
            }
            __syncthreads();
#pragma unroll
            for (int d4 = 0; d4 < GQT_DC / 4; d4++) {
                float4 qf[RPT], kf[4];
#pragma unroll
                for (int i = 0; i < RPT; i++) qf[i] = *reinterpret_cast<const float4 *>(Qc + (tq * RPT + i) * GQT_LDQ + d4 * 4);
#pragma unroll
                for (int j = 0; j < 4; j++) kf[j] = *reinterpret_cast<const float4 *>(Kc + (tc + 16 * j) * GQT_LDQ + d4 * 4);
#pragma unroll
                for (int i = 0; i < RPT; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        s[i][j] = fmaf(qf[i].x, kf[j].x, s[i][j]); s[i][j] = fmaf(qf[i].y, kf[j].y, s[i][j]);
                        s[i][j] = fmaf(qf[i].z, kf[j].z, s[i][j]); s[i][j] = fmaf(qf[i].w, kf[j].w, s[i][j]);
                    }
            }
        }
        if (a.softcap > 0.0f) {
#pragma unroll
            for (int i = 0; i < RPT; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) s[i][j] = a.softcap * tanhf(s[i][j] / a.softcap);
        }
        // ---- the running softmax of each row; P to LDS
#pragma unroll
        for (int i = 0; i < RPT; i++) {
            const int r = tq * RPT + i, rp = rpos[r];
            const uint64_t rbit = rseq[r] >= 0 ? 1ull << rseq[r] : 0ull;
            bool vis[4];
            float bm = -INFINITY;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int cp = cpos[tc + 16 * j];
                vis[j] = cp >= 0 && cp <= rp && (cseq[tc + 16 * j] & rbit) != 0 && !(a.window > 0 && rp - cp >= a.window && cp >= a.keep_first);
                if (vis[j]) {
                    if (a.rel) s[i][j] += gq_rel_bias(a, rp - cp, h);
                    bm = fmaxf(bm, s[i][j]);
                }
            }
#pragma unroll
            for (int of = 8; of > 0; of >>= 1) bm = fmaxf(bm, __shfl_xor(bm, of, 64));
            const float mn = fmaxf(m[i], bm);
            const float alpha = m[i] == -INFINITY ? 0.0f : expf(m[i] - mn);   // (mn = -inf only while m is: nothing seen yet, nothing to scale)
            float ps = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float pj = vis[j] ? expf(s[i][j] - mn) : 0.0f;
                ps += pj;
                P[r * GQT_LDP + tc + 16 * j] = pj;
            }
#pragma unroll
            for (int of = 8; of > 0; of >>= 1) ps += __shfl_xor(ps, of, 64);
            l[i] = l[i] * alpha + ps;
            m[i] = mn;
#pragma unroll
            for (int e = 0; e < NVC * 4; e++) o[i][e] *= alpha;
        }
        // ---- O += P V
#pragma unroll
        for (int vc = 0; vc < NVC; vc++) {
            __syncthreads();                                    // (P is complete; the previous slice of V has been used)
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int idx = tid + 256 * k, r = idx >> 4, col = vc * 64 + (idx & 15) * 4;
                float4 vv = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (col < VD && cpos[r] >= 0) vv = *reinterpret_cast<const float4 *>(a.cache + (size_t)(c0 + r) * L + voff + col);
                *reinterpret_cast<float4 *>(Vc + r * GQT_LDP + (idx & 15) * 4) = vv;
            }
            __syncthreads();
            for (int c = 0; c < GQT_B; c += 4) {
                float4 pf[RPT];
#pragma unroll
                for (int i = 0; i < RPT; i++) pf[i] = *reinterpret_cast<const float4 *>(P + (tq * RPT + i) * GQT_LDP + c);
#pragma unroll
                for (int cc = 0; cc < 4; cc++) {
                    const float4 vf = *reinterpret_cast<const float4 *>(Vc + (c + cc) * GQT_LDP + tc * 4);
#pragma unroll
                    for (int i = 0; i < RPT; i++) {
                        const float pw = cc == 0 ? pf[i].x : cc == 1 ? pf[i].y : cc == 2 ? pf[i].z : pf[i].w;
                        o[i][vc * 4 + 0] = fmaf(pw, vf.x, o[i][vc * 4 + 0]); o[i][vc * 4 + 1] = fmaf(pw, vf.y, o[i][vc * 4 + 1]);
                        o[i][vc * 4 + 2] = fmaf(pw, vf.z, o[i][vc * 4 + 2]); o[i][vc * 4 + 3] = fmaf(pw, vf.w, o[i][vc * 4 + 3]);
                    }
                }
            }
        }
    }
    if (gridDim.z > 1) {                                        // this run's records: maximum, sum, weighted value (sink and gate enter at the merge)
#pragma unroll
        for (int i = 0; i < RPT; i++) {
            const int r = row0 + tq * RPT + i;
            if (r >= a.T) continue;
            float *rec = a.part + (((size_t)r * a.H + h) * gridDim.z + blockIdx.z) * (size_t)(VD + 2);
            if (tc == 0) { rec[0] = m[i]; rec[1] = l[i]; }
#pragma unroll
            for (int vc = 0; vc < NVC; vc++)
#pragma unroll
                for (int e = 0; e < 4; e++) if (vc * 64 + tc * 4 + e < VD) rec[2 + vc * 64 + tc * 4 + e] = o[i][vc * 4 + e];
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        const int r = row0 + tq * RPT + i;
        if (r >= a.T) continue;
        float MM = m[i], den = l[i], sc = 1.0f;
        if (a.sink) {
            MM = fmaxf(m[i], a.sink[h]);
            sc = l[i] > 0.0f ? expf(m[i] - MM) : 0.0f;
            den = l[i] * sc + expf(a.sink[h] - MM);
        }
        float inv = den > 0.0f ? sc / den : 0.0f;
        if (a.gate) inv *= 1.0f / (1.0f + expf(-a.gate[(size_t)r * a.ld_gate + h]));   // (a factor per head: it commutes with the turn back that may follow)
#pragma unroll
        for (int vc = 0; vc < NVC; vc++) {
            const int col = vc * 64 + tc * 4;
            if (col < VD) *reinterpret_cast<float4 *>(a.out + (size_t)r * a.ld_out + (size_t)h * VD + col) =
                make_float4(o[i][vc * 4 + 0] * inv, o[i][vc * 4 + 1] * inv, o[i][vc * 4 + 2] * inv, o[i][vc * 4 + 3] * inv);
        }
    }
}

template <int NVC>
static hipError_t launch_gq_attn_tile(const GqAttnArgs &a, hipStream_t st) {
    if ((long long)((a.T + 63) / 64) * a.H >= 512) {
        const dim3 grid((unsigned)((a.T + 63) / 64), (unsigned)a.H);
        hipLaunchKernelGGL((gq_attn_tile_kernel<NVC, 4>), grid, dim3(256), gqt_lds_floats(64) * sizeof(float), st, a);
        if (a.v_cs) hipLaunchKernelGGL(gq_unturn_kernel, dim3((unsigned)a.T, (unsigned)a.H), dim3(256), 0, st, a);
        return hipGetLastError();
    }
    // too few tiles to fill the device: every tile's chain of cell blocks is cut into runs (at least two blocks each where the cells in use allow), as many
    // as bring the grid to about four workgroups per CU and as the record buffer holds
    const long long tiles = (long long)((a.T + 31) / 32) * a.H;
    long long splits = (1024 + tiles - 1) / tiles;
    const long long by_blocks = a.n_kv_hint > 0 ? ((a.n_kv_hint + GQT_B - 1) / GQT_B + 1) / 2 : 1;
    if (splits > by_blocks) splits = by_blocks;
    if (splits > GQ_TILE_MAX_SPLITS) splits = GQ_TILE_MAX_SPLITS;
    while (splits > 1 && (!a.part || (size_t)a.T * a.H * splits * (a.vdim + 2) > a.part_floats)) splits--;
    if (splits < 1) splits = 1;
    const dim3 grid((unsigned)((a.T + 31) / 32), (unsigned)a.H, (unsigned)splits);
    hipLaunchKernelGGL((gq_attn_tile_kernel<NVC, 2>), grid, dim3(256), gqt_lds_floats(32) * sizeof(float), st, a);
    if (splits > 1) hipLaunchKernelGGL(gq_attn_merge_kernel, dim3((unsigned)a.T, (unsigned)a.H), dim3(256), 0, st, a, (int)splits);
    else if (a.v_cs) hipLaunchKernelGGL(gq_unturn_kernel, dim3((unsigned)a.T, (unsigned)a.H), dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace

bool gq_attn_shape_ok(int H, int G, int dim, int vdim) { return H >= 1 && G >= 1 && H % G == 0 && dim >= 1 && vdim >= 1 && dim <= GQ_MAX_D && vdim <= GQ_MAX_D; }

hipError_t launch_gq_maps_out(const float *att, int ld_att, const float *gate, int ld_gate, int T, int H, int vdim, float lambda, float out_mult, float eps,
                              float *y, int ld_y, hipStream_t st) {
    if (T <= 0) return hipSuccess;
    if (H < 1 || vdim < 1 || !att || !y) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gq_maps_out_kernel, dim3((unsigned)T, (unsigned)H), dim3(64), 0, st, att, ld_att, gate, ld_gate, vdim, lambda, out_mult, eps, y, ld_y);
    return hipGetLastError();
}

hipError_t launch_gq_prep(const GqPrepArgs &a, hipStream_t st) {
    if (a.T <= 0) return hipSuccess;
    if (a.rot_dims < 0 || a.rot_dims > a.dim || a.rot_dims > GQ_MAX_D || (a.rot_dims & 1) || (a.rot_dims > 0 && !a.rot_freq)) return hipErrorInvalidValue;
    if (a.v_rot_freq && ((a.vdim & 1) || a.vdim > GQ_MAX_D || !a.v_cs)) return hipErrorInvalidValue;
    const int n_heads = a.H + a.G * (a.maps > 1 ? a.maps : 1);
    if (a.maps > 1 && a.H % a.maps != 0) return hipErrorInvalidValue;
    if (a.norm_per_head && (size_t)n_heads * sizeof(float) > 32 * 1024) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gq_prep_kernel, dim3((unsigned)a.T), dim3(256), a.norm_per_head ? (size_t)n_heads * sizeof(float) : 0, st, a);
    return hipGetLastError();
}

hipError_t launch_gq_attn(const GqAttnArgs &a, hipStream_t st) {
    if (a.T <= 0) return hipSuccess;
    const int maps = a.maps > 1 ? a.maps : 1;
    if (a.H % maps != 0 || !gq_attn_shape_ok(a.H / maps, a.G, a.dim, a.vdim) || (a.v_cs && (a.vdim & 1))) return hipErrorInvalidValue;
    if (a.rel && (!a.dist_bucket || a.n_dist < 0 || a.rel_rows < 1)) return hipErrorInvalidValue;
    // batches: the tiled pass (16-byte loads everywhere: head sizes, strides and bases must allow them); a few rows: one workgroup per (row, head)
    const auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (a.T >= GQ_TILE_MIN_ROWS && (a.dim & 3) == 0 && (a.vdim & 3) == 0 && (a.ld_q & 3) == 0 && (a.ld_out & 3) == 0 && al16(a.q) && al16(a.out) && al16(a.cache)) {
        if (a.vdim <= 64) return launch_gq_attn_tile<1>(a, st);
        if (a.vdim <= 128) return launch_gq_attn_tile<2>(a, st);
        if (a.vdim <= 256) return launch_gq_attn_tile<4>(a, st);
    }                                                            // (wider value heads: the per-row kernel below)
    const int Dm = a.dim > a.vdim ? a.dim : a.vdim;
    if (Dm <= 64) return launch_gq_attn_nj<1>(a, st);
    if (Dm <= 128) return launch_gq_attn_nj<2>(a, st);
    if (Dm <= 256) return launch_gq_attn_nj<4>(a, st);
    return launch_gq_attn_nj<8>(a, st);
}

}  // namespace mi355
