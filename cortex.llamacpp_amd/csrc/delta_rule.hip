// delta_rule.hip — the gated delta rule: a matrix memory that, per token, decays, corrects what it holds under the token's key towards the token's value,
// and is read with the token's query.
//
// Per value head a state S [D][VD], f32, one per sequence slot (DeltaArgs in kernels.h):
//     S <- a S            a: one decay per head, or one per key channel (row d of S times a[d])
//     u  = beta (v - S^T k)
//     S <- S + k u^T
//     o  = S^T q          (the read-out sees the token's own write)
// k is a unit vector, q a unit vector over sqrt(D); both are the silu of a short causal convolution over time of their projections, like v.
//
// delta_prep: everything per (token, channel) in front of the recurrence, one launch - the convolution with its silu (inputs before a segment's first row come
// from the slot's convolution state, which the launch also moves on), beta = sigmoid, the decays a = exp(-exp(A) softplus(pre + dt)).
// delta_scan: the columns of S evolve independently given k, q, beta and a, so a workgroup owns 16 columns of one head of one sequence segment (narrow
// blocks: a head's state spreads over many compute units, which is what a single sequence has to offer): a wave holds 16 columns x 4 row groups, the 4 or 8
// waves split the D rows further, each thread keeps its rows of its column in registers.  Per token ONE exchange across the waves: with G = a S the
// partial sums of G^T k and G^T q are formed in the same pass (row groups meet by lane shuffles, waves through LDS); u follows from the first, and
// o = G^T q + u (k . q) needs no second pass over the updated state.  The inputs of CH tokens are staged in LDS at a time and made unit vectors there.  A segment is a run of consecutive batch rows of one sequence - a
// prompt, a portion of one, a single decoded token: the same code, started from the slot's state and ending with the state written back, so the result does
// not depend on how a sequence was cut.
#include "kernels.h"

namespace mi355 {

namespace {

__device__ __forceinline__ float dl_softplus(float z) { return fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z))); }

constexpr int DELTA_PREP_TOKENS = 32;                           // rows of a segment one workgroup of the prep launch walks

// column index -> what it is: [0, C) a convolution channel; [C, C + H) a head's beta; the rest a decay
__global__ __launch_bounds__(256) void delta_prep_kernel(DeltaArgs a, int C, int NDEC, int move_state) {
    const int seg = blockIdx.x, col = blockIdx.y * 256 + threadIdx.x;
    if (col >= C + a.H + NDEC) return;
    const int start = a.seg_start[seg], len = a.seg_len[seg], slot = a.seg_slot[seg];
    const int t_lo = blockIdx.z * DELTA_PREP_TOKENS, t_hi = t_lo + DELTA_PREP_TOKENS < len ? t_lo + DELTA_PREP_TOKENS : len;
    if (col >= C) {
        const int e = col - C;
        if (e < a.H) {
            for (int t = t_lo; t < t_hi; t++) {
                const float z = a.p[(size_t)(start + t) * a.ld_p + a.off_beta + e];
                a.c[(size_t)(start + t) * a.ld_c + col] = 1.0f / (1.0f + expf(-z));
            }
        } else {
            const int i = e - a.H, head = a.per_channel ? i / a.D : i;
            const float rate = expf(a.A_log[head]), bias = a.dt_bias[i];
            for (int t = t_lo; t < t_hi; t++) a.c[(size_t)(start + t) * a.ld_c + col] = expf(-rate * dl_softplus(a.a[(size_t)(start + t) * a.ld_a + i] + bias));
        }
        return;
    }
    const int taps = a.taps, back = taps - 1;
    float w[DELTA_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < DELTA_MAX_TAPS; j++) w[j] = j < taps ? a.conv_w[(size_t)col * taps + j] : 0.0f;
    float *state = a.conv_state + (size_t)slot * back * C + col;                               // [back][C] of the slot, this channel
    // the input `ago` tokens before row t of the segment: a row of the batch, or - before the segment's first row - what the slot remembers
    const auto input = [&](int t) { return t >= 0 ? a.p[(size_t)(start + t) * a.ld_p + col] : state[(size_t)(back + t) * C]; };
    for (int t = t_lo; t < t_hi; t++) {
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < DELTA_MAX_TAPS; j++)
            if (j < taps) s = fmaf(w[j], input(t - (back - j)), s);
        a.c[(size_t)(start + t) * a.ld_c + col] = s / (1.0f + expf(-s));
    }
    if (move_state) {                                           // (this workgroup alone reads the segment's old state: every value is read before the first is written)
        float keep[DELTA_MAX_TAPS - 1];
#pragma unroll
        for (int i = 0; i < DELTA_MAX_TAPS - 1; i++) keep[i] = i < back ? input(len - back + i) : 0.0f;
#pragma unroll
        for (int i = 0; i < DELTA_MAX_TAPS - 1; i++)
            if (i < back) state[(size_t)i * C] = keep[i];
    }
}

// the convolution state of segments that several workgroups of the prep launch read: moved on by a launch of its own behind it
__global__ __launch_bounds__(256) void delta_conv_state_kernel(DeltaArgs a, int C) {
    const int seg = blockIdx.x, col = blockIdx.y * 256 + threadIdx.x;
    if (col >= C) return;
    const int start = a.seg_start[seg], len = a.seg_len[seg], slot = a.seg_slot[seg], back = a.taps - 1;
    float *state = a.conv_state + (size_t)slot * back * C + col;
    float keep[DELTA_MAX_TAPS - 1];
#pragma unroll
    for (int i = 0; i < DELTA_MAX_TAPS - 1; i++) {
        const int t = len - back + i;
        keep[i] = i < back ? (t >= 0 ? a.p[(size_t)(start + t) * a.ld_p + col] : state[(size_t)(back + t) * C]) : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < DELTA_MAX_TAPS - 1; i++)
        if (i < back) state[(size_t)i * C] = keep[i];
}

// x summed over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (the row groups of a column), the same bits in all four: the lane-swap instructions of gfx950
// exchange 16-lane (32-lane) rows between two registers - with both operands x the two results are x and its partner, in every lane
__device__ __forceinline__ float delta_rows_sum(float x) {
    static_assert(64 / 16 == 4, "four row groups of sixteen columns");
    const unsigned a = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane16_swap(a, a, false, false);
    const float y = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    const unsigned b = __float_as_uint(y);
    const auto q = __builtin_amdgcn_permlane32_swap(b, b, false, false);
    return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}

// lane = (column c of DELTA_COLS, row group rg of DELTA_RG); thread (wave, rg) keeps rows [(wave * DELTA_RG + rg) * DPER, + DPER) of its column
constexpr int DELTA_COLS = 16, DELTA_RG = 64 / DELTA_COLS;

template <int DPER, int NW, bool PERCH>
__global__ __launch_bounds__(64 * NW) void delta_scan_kernel(DeltaArgs a) {
    constexpr int DP = NW * DELTA_RG * DPER, CH = 2048 / DP < 32 ? 2048 / DP : 32, NT = 64 * NW, NLD = (CH * DP + NT - 1) / NT, NLV = (CH * DELTA_COLS + NT - 1) / NT;
    static_assert(CH <= NT, "one beta / decay load per thread and chunk");
    __shared__ __attribute__((aligned(16))) float sq[CH][DP], sk[CH][DP], sa[PERCH ? CH : 1][PERCH ? DP : 4];
    __shared__ float sv[CH][DELTA_COLS], sb[CH][4], red[2][2][NW][DELTA_COLS];
    const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane % DELTA_COLS, rg = lane / DELTA_COLS;
    const int col = blockIdx.z * DELTA_COLS + c, d0 = (wave * DELTA_RG + rg) * DPER;
    const int H = a.H, G = a.G, D = a.D, VD = a.VD, kh = h / (H / G);
    const int start = a.seg_start[seg], len = a.seg_len[seg], slot = a.seg_slot[seg];
    const int off_k = G * D, off_v = 2 * G * D, off_b = off_v + H * VD, off_a = off_b + H;
    float *Sg = a.S + ((size_t)slot * H + h) * (size_t)D * VD;
    float S[DPER];
#pragma unroll
    for (int e = 0; e < DPER; e++) S[e] = d0 + e < D && col < VD ? Sg[(size_t)(d0 + e) * VD + col] : 0.0f;
    const float qscale = 1.0f / sqrtf((float)D);
    // a chunk's inputs travel memory -> registers -> LDS; the NEXT chunk's loads are issued before this chunk's tokens are walked, so the chain of tokens
    // never waits for memory
    float rq[NLD], rk[NLD], ra[PERCH ? NLD : 1], rv[NLV], rb0 = 0.0f, rb1 = 1.0f;
    const auto request = [&](int t0) {
        const int nc = len - t0 < CH ? len - t0 : CH;
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            const int idx = tid + i * NT, tt = idx / DP, d = idx - tt * DP;
            const bool in = tt < nc && d < D;
            const float *row = a.c + (size_t)(start + t0 + (tt < nc ? tt : 0)) * a.ld_c;
            rq[i] = in ? row[kh * D + d] : 0.0f;
            rk[i] = in ? row[off_k + kh * D + d] : 0.0f;
            if (PERCH) ra[i] = in ? row[off_a + h * D + d] : 1.0f;
        }
#pragma unroll
        for (int i = 0; i < NLV; i++) {
            const int idx = tid + i * NT, tt = idx / DELTA_COLS, cc = blockIdx.z * DELTA_COLS + idx % DELTA_COLS;
            rv[i] = tt < nc && cc < VD ? a.c[(size_t)(start + t0 + tt) * a.ld_c + off_v + h * VD + cc] : 0.0f;
        }
        if (tid < nc) {
            const float *row = a.c + (size_t)(start + t0 + tid) * a.ld_c;
            rb0 = row[off_b + h];
            rb1 = PERCH ? 1.0f : row[off_a + h];
        }
    };
    request(0);
    for (int t0 = 0; t0 < len; t0 += CH) {
        const int nc = len - t0 < CH ? len - t0 : CH;
        __syncthreads();                                        // (the previous chunk has been used up)
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            const int idx = tid + i * NT, tt = idx / DP, d = idx - tt * DP;
            if (tt < CH) { sq[tt][d] = rq[i]; sk[tt][d] = rk[i]; if (PERCH) sa[tt][d] = ra[i]; }
        }
#pragma unroll
        for (int i = 0; i < NLV; i++) {
            const int idx = tid + i * NT;
            if (idx < CH * DELTA_COLS) sv[idx / DELTA_COLS][idx % DELTA_COLS] = rv[i];
        }
        if (tid < CH) { sb[tid][0] = rb0; sb[tid][1] = rb1; }
        if (t0 + CH < len) request(t0 + CH);
        __syncthreads();
        // unit vectors: sixteen lanes per token, four tokens of the chunk per wave at a time; k . q of the finished vectors goes along (the read-out needs it)
        for (int base = wave * 4; base < nc; base += NW * 4) {
            const int tt = base + (lane >> 4), li = lane & 15;
            const bool live = tt < nc;
            float qq = 0.0f, kk = 0.0f, kq = 0.0f;
            if (live)
                for (int d = li; d < D; d += 16) { const float q = sq[tt][d], k = sk[tt][d]; qq = fmaf(q, q, qq); kk = fmaf(k, k, kk); kq = fmaf(k, q, kq); }
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) { qq += __shfl_xor(qq, o, 64); kk += __shfl_xor(kk, o, 64); kq += __shfl_xor(kq, o, 64); }
            const float iq = qscale / sqrtf(qq + 1e-6f), ik = 1.0f / sqrtf(kk + 1e-6f);
            if (live) {
                for (int d = li; d < D; d += 16) { sq[tt][d] *= iq; sk[tt][d] *= ik; }
                if (li == 0) sb[tt][2] = kq * iq * ik;
            }
        }
        __syncthreads();
        // the walk: a token's k / q / a / v / beta are in registers BEFORE the barrier of the token in front of it, so that behind the barrier only the
        // exchanged sums, u and the update stand between one token and the next
        float kv[DPER], qv[DPER], av[PERCH ? DPER : 1], v, beta, ah, kq;
        const auto fetch = [&](int tt, float (&k_)[DPER], float (&q_)[DPER], float (&a_)[PERCH ? DPER : 1], float &v_, float &b_, float &ah_, float &kq_) {
            v_ = sv[tt][c]; b_ = sb[tt][0]; ah_ = sb[tt][1]; kq_ = sb[tt][2];
            if constexpr (DPER % 4 == 0) {
#pragma unroll
                for (int e = 0; e < DPER; e += 4) {
                    const float4 k4 = *reinterpret_cast<const float4 *>(&sk[tt][d0 + e]), q4 = *reinterpret_cast<const float4 *>(&sq[tt][d0 + e]);
                    k_[e] = k4.x; k_[e + 1] = k4.y; k_[e + 2] = k4.z; k_[e + 3] = k4.w;
                    q_[e] = q4.x; q_[e + 1] = q4.y; q_[e + 2] = q4.z; q_[e + 3] = q4.w;
                    if constexpr (PERCH) {
                        const float4 a4 = *reinterpret_cast<const float4 *>(&sa[tt][d0 + e]);
                        a_[e] = a4.x; a_[e + 1] = a4.y; a_[e + 2] = a4.z; a_[e + 3] = a4.w;
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < DPER; e++) {
                    k_[e] = sk[tt][d0 + e]; q_[e] = sq[tt][d0 + e];
                    if constexpr (PERCH) a_[e] = sa[tt][d0 + e];
                }
            }
        };
        fetch(0, kv, qv, av, v, beta, ah, kq);
        for (int tt = 0; tt < nc; tt++) {
            float pk = 0.0f, pq = 0.0f;
#pragma unroll
            for (int e = 0; e < DPER; e++) {
                float decay = ah;
                if constexpr (PERCH) decay = av[e];
                S[e] *= decay;
                pk = fmaf(S[e], kv[e], pk);
                pq = fmaf(S[e], qv[e], pq);
            }
            pk = delta_rows_sum(pk); pq = delta_rows_sum(pq);   // the wave's four row groups
            const int pb = tt & 1;                              // (two sets of partial sums: one barrier per token is enough)
            if (rg == 0) { red[pb][0][wave][c] = pk; red[pb][1][wave][c] = pq; }
            float kn[DPER], qn[DPER], an[PERCH ? DPER : 1], vn = 0.0f, bn = 0.0f, ahn = 1.0f, kqn = 0.0f;
            if (tt + 1 < nc) fetch(tt + 1, kn, qn, an, vn, bn, ahn, kqn);
            __syncthreads();
            float mk = 0.0f, mq = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w++) { mk += red[pb][0][w][c]; mq += red[pb][1][w][c]; }
            const float u = beta * (v - mk);
#pragma unroll
            for (int e = 0; e < DPER; e++) S[e] = fmaf(kv[e], u, S[e]);
            if (tid < DELTA_COLS && col < VD) a.o[(size_t)(start + t0 + tt) * a.ld_o + (size_t)h * VD + col] = fmaf(u, kq, mq);
            if (tt + 1 < nc) {
#pragma unroll
                for (int e = 0; e < DPER; e++) { kv[e] = kn[e]; qv[e] = qn[e]; if constexpr (PERCH) av[e] = an[e]; }
                v = vn; beta = bn; ah = ahn; kq = kqn;
            }
        }
    }
#pragma unroll
    for (int e = 0; e < DPER; e++)
        if (d0 + e < D && col < VD) Sg[(size_t)(d0 + e) * VD + col] = S[e];
}

template <bool PERCH>
hipError_t launch_delta_scan_t(const DeltaArgs &a, hipStream_t st) {
    const dim3 grid((unsigned)a.n_seg, (unsigned)a.H, (unsigned)((a.VD + DELTA_COLS - 1) / DELTA_COLS));
    // rows of the state per thread x waves per workgroup (x 4 row groups per wave): few waves keep the per-token exchange short, narrow column blocks
    // spread a head's state over many compute units
    if (a.D <= 16) hipLaunchKernelGGL((delta_scan_kernel<1, 4, PERCH>), grid, dim3(256), 0, st, a);
    else if (a.D <= 32) hipLaunchKernelGGL((delta_scan_kernel<2, 4, PERCH>), grid, dim3(256), 0, st, a);
    else if (a.D <= 64) hipLaunchKernelGGL((delta_scan_kernel<4, 4, PERCH>), grid, dim3(256), 0, st, a);
    else if (a.D <= 128) hipLaunchKernelGGL((delta_scan_kernel<8, 4, PERCH>), grid, dim3(256), 0, st, a);
    else if (a.D <= 256) hipLaunchKernelGGL((delta_scan_kernel<8, 8, PERCH>), grid, dim3(512), 0, st, a);
    else hipLaunchKernelGGL((delta_scan_kernel<16, 8, PERCH>), grid, dim3(512), 0, st, a);
    return hipGetLastError();
}

}  // namespace

bool delta_shape_ok(int H, int G, int D, int VD, int taps) {
    return H >= 1 && G >= 1 && H % G == 0 && D >= 1 && D <= 512 && VD >= 1 && taps >= 1 && taps <= DELTA_MAX_TAPS;
}

hipError_t launch_delta_prep(const DeltaArgs &a, hipStream_t st) {
    if (a.n_seg <= 0 || a.max_len <= 0) return hipSuccess;
    if (!delta_shape_ok(a.H, a.G, a.D, a.VD, a.taps)) return hipErrorInvalidValue;
    const int C = delta_channels(a), NDEC = a.per_channel ? a.H * a.D : a.H;
    const unsigned chunks = (unsigned)((a.max_len + DELTA_PREP_TOKENS - 1) / DELTA_PREP_TOKENS);
    const dim3 grid((unsigned)a.n_seg, (unsigned)((C + a.H + NDEC + 255) / 256), chunks);
    hipLaunchKernelGGL(delta_prep_kernel, grid, dim3(256), 0, st, a, C, NDEC, chunks == 1 && a.taps > 1 ? 1 : 0);
    if (chunks > 1 && a.taps > 1) hipLaunchKernelGGL(delta_conv_state_kernel, dim3((unsigned)a.n_seg, (unsigned)((C + 255) / 256)), dim3(256), 0, st, a, C);
    return hipGetLastError();
}

hipError_t launch_delta_scan(const DeltaArgs &a, hipStream_t st) {
    if (a.n_seg <= 0) return hipSuccess;
    if (!delta_shape_ok(a.H, a.G, a.D, a.VD, a.taps)) return hipErrorInvalidValue;
    return a.per_channel ? launch_delta_scan_t<true>(a, st) : launch_delta_scan_t<false>(a, st);
}

}  // namespace mi355
