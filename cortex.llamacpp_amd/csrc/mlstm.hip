// mlstm.hip — the matrix-memory recurrence (mLSTM of the xLSTM family), token by token with the state in registers.
//
// Per head: a state matrix S [dim][vdim], a normaliser n [dim] and a running maximum m of the log gates, all f32, one set per sequence slot.  For a token
// with query q (already scaled by dim^-1/2 here), key k, value v and the pre-activations of the two gates:
//     i = cap tanh(i_pre / cap)            f = logsigmoid(cap tanh(f_pre / cap))        (both made for the whole batch at once: launch_mlstm_gates)
//     m' = max(f + m, i)     S' = e^(f + m - m') S + e^(i - m') k v^T     n' likewise with k alone
//     o  = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)
// A state that has seen nothing is S = 0, n = 0, m = 0.  The columns of S evolve independently given the gates, so a workgroup owns 64 columns of one head of
// one sequence segment: lane = column, the 8 or 16 waves split the dim rows (each thread keeps its rows of its column - and of n - in registers), the per-token
// partial sums of S^T q and n . q cross the waves through LDS.  A segment is a run of consecutive rows of the batch that belong to one sequence: a prompt,
// a portion of one, or a single decoded token - the same code, started from the slot's state and ending with the state written back.
// mlstm_out: per head, the output divided by its root mean square, times the mixer's norm weight (per head and entry, one vector shared by the heads, or none), times
// sigmoid - or silu - of the output gate's pre-activation.  The delta-rule mixers close with the same launch.
#include "kernels.h"

namespace mi355 {

namespace {

template <int DPER, int NDG>
__global__ __launch_bounds__(64 * NDG) void mlstm_scan_kernel(MlstmArgs a) {
    // CH tokens' inputs are staged in LDS by the whole workgroup at once - one trip to memory per CH tokens instead of one per token in the dependency
    // chain - and the recurrence then runs out of LDS and registers
    constexpr int DP = NDG * DPER, CH = 2048 / DP, NT = 64 * NDG;
    __shared__ float sq[CH][DP], sk[CH][DP], sv[CH][64], sg[CH][2], red[2][NDG][64], redn[2][NDG];
    const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, j = tid & 63, dg = tid >> 6;
    const int col = blockIdx.z * 64 + j, d0 = dg * DPER;
    const int H = a.H, D = a.D, VD = a.VD;
    const int start = a.seg_start[seg], len = a.seg_len[seg], slot = a.seg_slot[seg];
    float *Sg = a.S + ((size_t)slot * H + h) * (size_t)D * VD;
    float *ng = a.n + ((size_t)slot * H + h) * D;
    float *mg = a.m + (size_t)slot * H + h;
    float S[DPER], n[DPER];
#pragma unroll
    for (int e = 0; e < DPER; e++) {
        const int d = d0 + e;
        S[e] = d < D && col < VD ? Sg[(size_t)d * VD + col] : 0.0f;
        n[e] = d < D ? ng[d] : 0.0f;
    }
    float m = *mg;
    const float qscale = 1.0f / sqrtf((float)D);
    const int off_k = H * D, off_v = 2 * H * D, off_i = 2 * H * D + 2 * H * VD, off_f = off_i + H;
    for (int t0 = 0; t0 < len; t0 += CH) {
        const int nc = len - t0 < CH ? len - t0 : CH;
        __syncthreads();                                        // (the previous chunk has been used up)
        for (int idx = tid; idx < nc * DP; idx += NT) {
            const int tt = idx / DP, d = idx - tt * DP;
            const float *row = a.p + (size_t)(start + t0 + tt) * a.ld_p;
            sq[tt][d] = d < D ? row[h * D + d] * qscale : 0.0f;
            sk[tt][d] = d < D ? row[off_k + h * D + d] : 0.0f;
        }
        for (int idx = tid; idx < nc * 64; idx += NT) {
            const int tt = idx >> 6, c = blockIdx.z * 64 + (idx & 63);
            sv[tt][idx & 63] = c < VD ? a.p[(size_t)(start + t0 + tt) * a.ld_p + off_v + h * VD + c] : 0.0f;
        }
        if (tid < nc * 2) sg[tid >> 1][tid & 1] = a.p[(size_t)(start + t0 + (tid >> 1)) * a.ld_p + ((tid & 1) ? off_f : off_i) + h];   // log gates (mlstm_gates_kernel)
        __syncthreads();
        for (int tt = 0; tt < nc; tt++) {
            const float v = sv[tt][j], ig = sg[tt][0], fg = sg[tt][1];
            const float mn = fmaxf(fg + m, ig), ea = expf(fg + m - mn), eb = expf(ig - mn);
            m = mn;
            float num = 0.0f, nq = 0.0f;
#pragma unroll
            for (int e = 0; e < DPER; e++) {
                const float kd = eb * sk[tt][d0 + e], q = sq[tt][d0 + e];
                S[e] = fmaf(ea, S[e], kd * v);
                n[e] = fmaf(ea, n[e], kd);
                num = fmaf(S[e], q, num);
                nq = fmaf(n[e], q, nq);
            }
            const int pb = tt & 1;                              // (two sets of partial sums: one barrier per token is enough)
            red[pb][dg][j] = num;
            if (j == 0) redn[pb][dg] = nq;
            __syncthreads();
            if (dg == 0 && col < VD) {
                float nt = 0.0f, qt = 0.0f;
#pragma unroll
                for (int w = 0; w < NDG; w++) { nt += red[pb][w][j]; qt += redn[pb][w]; }
                a.o[(size_t)(start + t0 + tt) * a.ld_o + (size_t)h * VD + col] = nt / (fmaxf(fabsf(qt), expf(-m)) + 1e-6f);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < DPER; e++) {
        const int d = d0 + e;
        if (d < D && col < VD) Sg[(size_t)d * VD + col] = S[e];
        if (d < D && blockIdx.z == 0 && j == 0) ng[d] = n[e];
    }
    if (blockIdx.z == 0 && tid == 0) *mg = m;
}

// the two log gates of every (token, head), in place over their pre-activations: i = cap tanh((x + b_i) / cap), f = logsigmoid(cap tanh((x + b_f) / cap))
__global__ void mlstm_gates_kernel(float *p, int ld_p, int off_i, int H, int T, const float *ib, const float *fb, float cap) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= T * H) return;
    const int t = i / H, h = i - t * H;
    float *row = p + (size_t)t * ld_p + off_i;
    const float ig = cap * tanhf((row[h] + (ib ? ib[h] : 0.0f)) / cap);
    const float fz = cap * tanhf((row[H + h] + (fb ? fb[h] : 0.0f)) / cap);
    row[h] = ig;
    row[H + h] = fminf(fz, 0.0f) - log1pf(expf(-fabsf(fz)));
}

__global__ __launch_bounds__(64) void mlstm_out_kernel(const float *o, int ld_o, const float *p, int ld_p, int off_g, const float *w, int H, int VD, float eps,
                                                       float *y, int ld_y, int w_stride, int gate) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float *orow = o + (size_t)t * ld_o + (size_t)h * VD;
    float ss = 0.0f;
    for (int i = lane; i < VD; i += 64) { const float v = orow[i]; ss = fmaf(v, v, ss); }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) ss += __shfl_xor(ss, s, 64);
    const float inv = 1.0f / sqrtf(ss / (float)VD + eps);
    for (int i = lane; i < VD; i += 64) {
        const float g = p[(size_t)t * ld_p + off_g + h * VD + i];
        const float sg = 1.0f / (1.0f + expf(-g));
        y[(size_t)t * ld_y + (size_t)h * VD + i] = orow[i] * inv * (w ? w[h * w_stride + i] : 1.0f) * (gate == MLSTM_GATE_SILU ? g * sg : sg);
    }
}

__global__ void mlstm_state_reset_kernel(float *S, size_t n_s, float *n, size_t n_n, float *m, size_t n_m) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_s) S[i] = 0.0f;
    if (i < n_n) n[i] = 0.0f;
    if (i < n_m) m[i] = 0.0f;
}

}  // namespace

bool mlstm_shape_ok(int D, int VD) { return D >= 1 && D <= 512 && VD >= 1; }

hipError_t launch_mlstm_gates(const MlstmArgs &a, int T, hipStream_t st) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(mlstm_gates_kernel, dim3((unsigned)((T * a.H + 255) / 256)), dim3(256), 0, st, const_cast<float *>(a.p), a.ld_p,
                       2 * a.H * a.D + 2 * a.H * a.VD, a.H, T, a.i_bias, a.f_bias, a.gate_cap);
    return hipGetLastError();
}

hipError_t launch_mlstm_scan(const MlstmArgs &a, hipStream_t st) {
    if (a.n_seg <= 0) return hipSuccess;
    if (!mlstm_shape_ok(a.D, a.VD)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)a.n_seg, (unsigned)a.H, (unsigned)((a.VD + 63) / 64));
    // dim rows per thread x waves per workgroup: the waves of a workgroup split the rows of the state, the more of them the shorter a token's chain
    if (a.D <= 16) hipLaunchKernelGGL((mlstm_scan_kernel<2, 8>), grid, dim3(512), 0, st, a);
    else if (a.D <= 32) hipLaunchKernelGGL((mlstm_scan_kernel<4, 8>), grid, dim3(512), 0, st, a);
    else if (a.D <= 64) hipLaunchKernelGGL((mlstm_scan_kernel<8, 8>), grid, dim3(512), 0, st, a);
    else if (a.D <= 128) hipLaunchKernelGGL((mlstm_scan_kernel<8, 16>), grid, dim3(1024), 0, st, a);
    else if (a.D <= 256) hipLaunchKernelGGL((mlstm_scan_kernel<16, 16>), grid, dim3(1024), 0, st, a);
    else hipLaunchKernelGGL((mlstm_scan_kernel<32, 16>), grid, dim3(1024), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_mlstm_out(const float *o, int ld_o, const float *p, int ld_p, int off_g, const float *w, int T, int H, int VD, float eps, float *y, int ld_y,
                            hipStream_t st, int w_stride, int gate) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(mlstm_out_kernel, dim3((unsigned)T, (unsigned)H), dim3(64), 0, st, o, ld_o, p, ld_p, off_g, w, H, VD, eps, y, ld_y, w_stride < 0 ? VD : w_stride, gate);
    return hipGetLastError();
}

hipError_t launch_mlstm_state_reset(float *S, size_t n_s, float *n, size_t n_n, float *m, size_t n_m, hipStream_t st) {
    const size_t mx = n_s > n_n ? (n_s > n_m ? n_s : n_m) : (n_n > n_m ? n_n : n_m);
    if (!mx) return hipSuccess;
    hipLaunchKernelGGL(mlstm_state_reset_kernel, dim3((unsigned)((mx + 255) / 256)), dim3(256), 0, st, S, n_s, n, n_n, m, n_m);
    return hipGetLastError();
}

}  // namespace mi355
