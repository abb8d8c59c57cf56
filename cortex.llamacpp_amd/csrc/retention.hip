// retention.hip — linear attention with one fixed decay per head and no softmax, token by token with the state in registers.
//
// Per head a state matrix S [dim][vdim], f32, one per sequence slot; for a token with query q, key k, value v:
//     S <- decay S + k v^T            o = S^T q
// q and k turn by the token's position on their first rot_dims entries (entry i with entry i + rot_dims / 2; the per-pair angle table comes from the host),
// k is scaled behind the turn.  A state that has seen nothing is zero.
//
// Nothing a thread needs for its part of S depends on another thread: a workgroup owns 64 columns of one head of one sequence segment, lane = column, the
// waves split the dim rows, each thread keeps its rows of its column in registers.  Only the outputs need a sum over the rows, so the waves' partial sums of
// SUB tokens at a time cross through LDS (two barriers per SUB tokens, none per token).  The inputs of CH tokens are staged in LDS by the whole workgroup
// at once, turned and scaled on the way (cos / sin once per (token, pair)).  A segment is a run of consecutive rows of the batch that belong to one sequence:
// a prompt, a portion of one, or a single decoded token - the same code, started from the slot's state and ending with the state written back, so the
// result does not depend on how a sequence was cut.
#include "kernels.h"

namespace mi355 {

namespace {

template <int DPER, int NDG>
__global__ __launch_bounds__(64 * NDG) void retention_scan_kernel(RetentionArgs a) {
    constexpr int DP = NDG * DPER, CH = 2048 / DP < 32 ? 2048 / DP : 32, NT = 64 * NDG, SUB = 8;
    __shared__ float sq[CH][DP], sk[CH][DP], sv[CH][64], red[SUB][NDG][64];
    const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, j = tid & 63, dg = tid >> 6;
    const int col = blockIdx.z * 64 + j, d0 = dg * DPER;
    const int H = a.H, D = a.D, VD = a.VD, half = a.rot_dims >> 1;
    const int start = a.seg_start[seg], len = a.seg_len[seg], slot = a.seg_slot[seg];
    float *Sg = a.S + ((size_t)slot * H + h) * (size_t)D * VD;
    float S[DPER];
#pragma unroll
    for (int e = 0; e < DPER; e++) {
        const int d = d0 + e;
        S[e] = d < D && col < VD ? Sg[(size_t)d * VD + col] : 0.0f;
    }
    const float decay = a.decay[h];
    const int off_k = H * D, off_v = 2 * H * D;
    for (int t0 = 0; t0 < len; t0 += CH) {
        const int nc = len - t0 < CH ? len - t0 : CH;
        __syncthreads();                                        // (the previous chunk has been used up)
        for (int idx = tid; idx < nc * DP; idx += NT) {
            const int tt = idx / DP, d = idx - tt * DP;
            const float *row = a.p + (size_t)(start + t0 + tt) * a.ld_p + (size_t)h * D;
            if (d < half) {                                     // the pair (d, d + half) of the query and of the key
                float sn, cs;
                sincosf((float)a.tok_pos[start + t0 + tt] * a.rot_freq[d], &sn, &cs);
                const float qu = row[d], qw = row[d + half], ku = row[off_k + d], kw = row[off_k + d + half];
                sq[tt][d] = qu * cs - qw * sn; sq[tt][d + half] = qw * cs + qu * sn;
                sk[tt][d] = (ku * cs - kw * sn) * a.k_scale; sk[tt][d + half] = (kw * cs + ku * sn) * a.k_scale;
            } else if (d >= a.rot_dims) {
                sq[tt][d] = d < D ? row[d] : 0.0f;
                sk[tt][d] = d < D ? row[off_k + d] * a.k_scale : 0.0f;
            }
        }
        for (int idx = tid; idx < nc * 64; idx += NT) {
            const int tt = idx >> 6, c = blockIdx.z * 64 + (idx & 63);
            sv[tt][idx & 63] = c < VD ? a.p[(size_t)(start + t0 + tt) * a.ld_p + off_v + (size_t)h * VD + c] : 0.0f;
        }
        __syncthreads();
        for (int s0 = 0; s0 < nc; s0 += SUB) {
            const int ns = nc - s0 < SUB ? nc - s0 : SUB;
            for (int u = 0; u < ns; u++) {
                const int tt = s0 + u;
                const float v = sv[tt][j];
                float num = 0.0f;
#pragma unroll
                for (int e = 0; e < DPER; e++) {
                    S[e] = fmaf(decay, S[e], sk[tt][d0 + e] * v);
                    num = fmaf(S[e], sq[tt][d0 + e], num);
                }
                red[u][dg][j] = num;
            }
            __syncthreads();
            for (int idx = tid; idx < ns * 64; idx += NT) {
                const int u = idx >> 6, c = blockIdx.z * 64 + (idx & 63);
                float o = 0.0f;
#pragma unroll
                for (int w = 0; w < NDG; w++) o += red[u][w][idx & 63];
                if (c < VD) a.o[(size_t)(start + t0 + s0 + u) * a.ld_o + (size_t)h * VD + c] = o;
            }
            __syncthreads();
        }
    }
#pragma unroll
    for (int e = 0; e < DPER; e++) {
        const int d = d0 + e;
        if (d < D && col < VD) Sg[(size_t)d * VD + col] = S[e];
    }
}

}  // namespace

bool retention_shape_ok(int D, int VD) { return D >= 1 && D <= 512 && VD >= 1; }

hipError_t launch_retention_scan(const RetentionArgs &a, hipStream_t st) {
    if (a.n_seg <= 0) return hipSuccess;
    if (!retention_shape_ok(a.D, a.VD) || a.rot_dims < 0 || a.rot_dims > a.D || (a.rot_dims & 1) || (a.rot_dims > 0 && !a.rot_freq) || !a.decay || !a.S) return hipErrorInvalidValue;
    const dim3 grid((unsigned)a.n_seg, (unsigned)a.H, (unsigned)((a.VD + 63) / 64));
    // dim rows per thread x waves per workgroup
    if (a.D <= 16) hipLaunchKernelGGL((retention_scan_kernel<2, 8>), grid, dim3(512), 0, st, a);
    else if (a.D <= 32) hipLaunchKernelGGL((retention_scan_kernel<4, 8>), grid, dim3(512), 0, st, a);
    else if (a.D <= 64) hipLaunchKernelGGL((retention_scan_kernel<8, 8>), grid, dim3(512), 0, st, a);
    else if (a.D <= 128) hipLaunchKernelGGL((retention_scan_kernel<8, 16>), grid, dim3(1024), 0, st, a);
    else if (a.D <= 256) hipLaunchKernelGGL((retention_scan_kernel<16, 16>), grid, dim3(1024), 0, st, a);
    else hipLaunchKernelGGL((retention_scan_kernel<32, 16>), grid, dim3(1024), 0, st, a);
    return hipGetLastError();
}

}  // namespace mi355
