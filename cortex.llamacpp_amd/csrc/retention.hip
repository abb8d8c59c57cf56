// retention.hip — linear attention with one fixed decay per head and no softmax, token by token with the state in registers.
//
// Per head a state matrix S [dim][vdim], f32, one per sequence slot; for a token with query q, key k, value v:
//     S <- decay S + k v^T            o = S^T q
// q and k turn by the token's position on their first rot_dims entries (entry i with entry i + rot_dims / 2; the per-pair angle table comes from the host),
// k is scaled behind the turn.  A state that has seen nothing is zero.
//
// Nothing a thread needs for its part of S depends on another thread: a workgroup owns 64 columns of one head of one sequence segment, lane = column, the
// waves split the dim rows, each thread keeps its rows of its column in registers.  Only the outputs need a sum over the rows, so the waves' partial sums of
// SUB tokens at a time cross through LDS (two barriers per SUB tokens, none per token).  (16-column workgroups with four row groups per wave - a head's state
// over four times as many compute units - were measured and lost, 234 against 151 us per 512 tokens: what a chunk costs is its barriers and its staging,
// not its arithmetic, and narrower workgroups stage fewer tokens per chunk.)  The inputs of CH tokens are staged in LDS by the whole workgroup at once, turned and scaled
// on the way (cos / sin once per (token, pair)); the next chunk's inputs are already on their way from memory while a chunk is walked.  A segment is a run of
// consecutive rows of the batch that belong to one sequence: a prompt, a portion of one, or a single decoded token - the same code, started from the slot's
// state and ending with the state written back, so the result does not depend on how a sequence was cut.
#include "kernels.h"

namespace mi355 {

namespace {

constexpr int RET_COLS = 64, RET_RG = 1;                        // columns per workgroup; row groups per wave

template <int DPER, int NDG>
__global__ __launch_bounds__(64 * NDG) void retention_scan_kernel(RetentionArgs a) {
    constexpr int DP = RET_RG * NDG * DPER, NT = 64 * NDG, IT = 2048 / NT, CH = 2048 / DP < 32 ? 2048 / DP : 32, SUB = 8;   // (CH * DP <= 2048, CH * 64 <= 2048)
    __shared__ float sq[CH][DP], sk[CH][DP], sv[CH][RET_COLS], red[SUB][NDG][RET_COLS];
    const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, j = lane & (RET_COLS - 1), rg = lane / RET_COLS, dg = tid >> 6;
    const int col = blockIdx.z * RET_COLS + j, d0 = (dg * RET_RG + rg) * DPER;
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
    // a chunk's inputs travel memory -> registers -> LDS: the NEXT chunk's loads are issued before this chunk's tokens are walked, so the walk does not wait
    // for memory.  Element idx of a chunk is (token idx / DP, entry idx % DP): an entry below half carries its pair (d, d + half) of q and of k, an entry
    // from rot_dims on carries itself, the entries between belong to their partners
    float rq[IT][2], rk[IT][2], rv[IT], rp[IT];
    const auto fetch = [&](int t0) {
        const int nc = len - t0 < CH ? len - t0 : CH;
#pragma unroll
        for (int it = 0; it < IT; it++) {
            const int idx = tid + it * NT, tt = idx / DP, d = idx - tt * DP;
            rq[it][0] = rq[it][1] = rk[it][0] = rk[it][1] = 0.0f; rp[it] = 0.0f;
            if (idx < nc * DP && d < D) {
                const float *row = a.p + (size_t)(start + t0 + tt) * a.ld_p + (size_t)h * D;
                if (d < half) {
                    rp[it] = (float)a.tok_pos[start + t0 + tt];
                    rq[it][0] = row[d]; rq[it][1] = row[d + half]; rk[it][0] = row[off_k + d]; rk[it][1] = row[off_k + d + half];
                } else if (d >= a.rot_dims) { rq[it][0] = row[d]; rk[it][0] = row[off_k + d]; }
            }
            const int vt = idx / RET_COLS, c = blockIdx.z * RET_COLS + (idx & (RET_COLS - 1));
            rv[it] = idx < nc * RET_COLS && c < VD ? a.p[(size_t)(start + t0 + vt) * a.ld_p + off_v + (size_t)h * VD + c] : 0.0f;
        }
    };
    const auto stage = [&](int nc) {
#pragma unroll
        for (int it = 0; it < IT; it++) {
            const int idx = tid + it * NT, tt = idx / DP, d = idx - tt * DP;
            if (idx < nc * DP) {
                if (d < half) {
                    float sn, cs;
                    sincosf(rp[it] * a.rot_freq[d], &sn, &cs);
                    sq[tt][d] = rq[it][0] * cs - rq[it][1] * sn; sq[tt][d + half] = rq[it][1] * cs + rq[it][0] * sn;
                    sk[tt][d] = (rk[it][0] * cs - rk[it][1] * sn) * a.k_scale; sk[tt][d + half] = (rk[it][1] * cs + rk[it][0] * sn) * a.k_scale;
                } else if (d >= a.rot_dims) { sq[tt][d] = rq[it][0]; sk[tt][d] = rk[it][0] * a.k_scale; }
            }
            if (idx < nc * RET_COLS) sv[idx / RET_COLS][idx & (RET_COLS - 1)] = rv[it];
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < len; t0 += CH) {
        const int nc = len - t0 < CH ? len - t0 : CH;
        __syncthreads();                                        // (the previous chunk has been used up)
        stage(nc);
        __syncthreads();
        if (t0 + CH < len) fetch(t0 + CH);
        for (int s0 = 0; s0 < nc; s0 += SUB) {
            const int ns = nc - s0 < SUB ? nc - s0 : SUB;
            const auto token = [&](int u) {
                const int tt = s0 + u;
                const float v = sv[tt][j];
                float num = 0.0f;
#pragma unroll
                for (int e = 0; e < DPER; e++) {
                    S[e] = fmaf(decay, S[e], sk[tt][d0 + e] * v);
                    num = fmaf(S[e], sq[tt][d0 + e], num);
                }
                if (RET_RG == 4) {                              // (a wave's row groups, where it has several)
                    num += __shfl_xor(num, 16, 64);
                    num += __shfl_xor(num, 32, 64);
                }
                if (rg == 0) red[u][dg][j] = num;
            };
            if (ns == SUB) {                                    // (a full round unrolled: the LDS reads of the next tokens are issued while the state's chain runs)
#pragma unroll
                for (int u = 0; u < SUB; u++) token(u);
            } else {
                for (int u = 0; u < ns; u++) token(u);
            }
            __syncthreads();
            for (int idx = tid; idx < ns * RET_COLS; idx += NT) {
                const int u = idx / RET_COLS, jj = idx & (RET_COLS - 1), c = blockIdx.z * RET_COLS + jj;
                float o = 0.0f;
#pragma unroll
                for (int w = 0; w < NDG; w++) o += red[u][w][jj];
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
    const dim3 grid((unsigned)a.n_seg, (unsigned)a.H, (unsigned)((a.VD + RET_COLS - 1) / RET_COLS));
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
