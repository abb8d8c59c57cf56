// mmb.hip — linear layers against BF16 weight rows ([out][in], K-contiguous) with f32 activations and f32 accumulation:
//
//   Y[z][t][n] = epi( sum_k X[z][t][k] * W[z][n][k] )
//
// z is an optional outer index with its own element strides on every operand: the heads of a per-head product (latent attention folds W_uk into the query
// and unfolds the attended latent through W_uv), the experts of a grouped batch (rows [offs[z], offs[z] + counts[z]) of X and Y belong to expert z), or
// the (token, rank) pairs of a few single tokens that picked their experts (sel[z] names the weight set, row z of Y, row z / sel_div of X).
//
// Three kernels behind one launch:
//   * mmb_vec   - up to a few dozen rows: one wave per output column walks K with 16-byte weight loads, the activations stay f32.  Weight-stream bound, the
//                 form of every single-token step in both precisions.
//   * mmb_mfma  - batches in bf16 mode: activations rounded to bf16 in registers, v_mfma_f32_32x32x16_bf16, one 32 x 32 (or 64 x 64) tile per wave, both operands
//                 read K-contiguous straight into the matrix-core register layout (lane = (row, k-group of 8)).
//   * mmb_f32   - batches in f32 mode (and every shape the other two refuse): LDS-tiled, v_fma_f32 only - products of an f32 activation and a bf16 weight
//                 widened exactly, no reduced-precision matrix mode anywhere.
// Epilogues: store | relu(y)^2 | silu(W x) * (W2 x) | gelu_tanh(W x) * (W2 x) | g sigmoid(1.702 g) (u + 1) with g = W x capped from above and u = W2 x clamped
// to +- the same limit (the gated ones: two weight sets, one pass over the activations).  An optional f32 bias per output column joins W x before the epilogue.
#include "kernels.h"

namespace mi355 {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf2f(unsigned short h) { return __uint_as_float((unsigned)h << 16); }
__device__ __forceinline__ unsigned short f2bf(float f) {                       // round to nearest even (NaN stays NaN)
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float epi_apply(int epi, float a, float b, float lim = 0.0f) {
    if (epi == MMB_CLAMP_SWIGLU) {
        const float g = fminf(a, lim), u = fminf(fmaxf(b, -lim), lim);
        return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
    }
    if (epi == MMB_RELU2) { const float r = a > 0.0f ? a : 0.0f; return r * r; }
    if (epi == MMB_SILU_MUL) return a / (1.0f + expf(-a)) * b;
    if (epi == MMB_GELU_MUL) return 0.5f * a * (1.0f + tanhf(0.7978845608028654f * (a + 0.044715f * a * a * a))) * b;   // the tanh form of gelu; sqrt(2 / pi)
    return a;
}

// where the rows of outer index z live: first row and row count of X / Y, the weight set
struct ZView { const float *x; const unsigned short *w, *w2; float *y; int rows; };
__device__ __forceinline__ ZView z_view(const MMBArgs &a, int z) {
    ZView v;
    int wz = z, x0 = 0, y0 = 0;
    v.rows = a.T;
    if (a.sel) { wz = a.sel[z]; x0 = z / a.sel_div; y0 = z; v.rows = 1; }
    else if (a.meta) { v.rows = a.meta[z]; x0 = y0 = a.meta[a.nz + z]; }
    v.x = a.x + (size_t)(a.sel || a.meta ? 0 : z) * a.x_zs + (size_t)x0 * a.ldx;
    v.y = a.y + (size_t)(a.sel || a.meta ? 0 : z) * a.y_zs + (size_t)y0 * a.ldy;
    v.w = a.w + (size_t)wz * a.w_zs;
    v.w2 = a.w2 ? a.w2 + (size_t)wz * a.w_zs : nullptr;
    return v;
}

// ---------------------------------------------------------------- few rows: one wave per output column
// Few rows against MANY output columns (single-token steps: the head, the feed-forward): a wave owns NR adjacent weight rows and keeps the activations of a
// 512-wide piece of k in registers for all of them - the activation and norm-weight loads, which every wave repeats out of the caches, are paid once per NR
// weight rows instead of once per row.  Up to TBR rows of X; 16-byte aligned operands; same arithmetic per output as mmb_vec_kernel.
template <int NR, int TBR>
__global__ __launch_bounds__(256) void mmb_vec_rows_kernel(MMBArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * 4 + wave) * NR;
    const ZView v = z_view(a, blockIdx.y);
    if (n0 >= a.N) return;
    const bool pn = a.pn_w != nullptr, gated = v.w2 != nullptr;
    const unsigned short *wr[NR], *wr2[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const int n = n0 + r < a.N ? n0 + r : a.N - 1;          // rows past the end read the last row; their results are never stored
        wr[r] = v.w + (size_t)n * a.ldw;
        wr2[r] = gated ? v.w2 + (size_t)n * a.ldw : wr[r];
    }
    float acc[NR][TBR], acc2[NR][TBR], ss[TBR];
#pragma unroll
    for (int i = 0; i < TBR; i++) {
        ss[i] = 0.0f;
#pragma unroll
        for (int r = 0; r < NR; r++) { acc[r][i] = 0.0f; acc2[r][i] = 0.0f; }
    }
    const int nt = v.rows < TBR ? v.rows : TBR;
    for (int k = lane * 8; k < a.K; k += 512) {
        u16x8 w8[NR], w28[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) {
            w8[r] = *reinterpret_cast<const u16x8 *>(wr[r] + k);
            if (gated) w28[r] = *reinterpret_cast<const u16x8 *>(wr2[r] + k);
        }
        float pw[8];
        if (pn) {
            const f32x4 g0 = *reinterpret_cast<const f32x4 *>(a.pn_w + k), g1 = *reinterpret_cast<const f32x4 *>(a.pn_w + k + 4);
            pw[0] = a.pn_off + g0.x; pw[1] = a.pn_off + g0.y; pw[2] = a.pn_off + g0.z; pw[3] = a.pn_off + g0.w;
            pw[4] = a.pn_off + g1.x; pw[5] = a.pn_off + g1.y; pw[6] = a.pn_off + g1.z; pw[7] = a.pn_off + g1.w;
        }
#pragma unroll
        for (int i = 0; i < TBR; i++) {
            if (i >= nt) break;
            const float *xr = v.x + (size_t)i * a.ldx + k;
            const f32x4 x0 = *reinterpret_cast<const f32x4 *>(xr), x1 = *reinterpret_cast<const f32x4 *>(xr + 4);
            float xs[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            if (pn) {
#pragma unroll
                for (int e = 0; e < 8; e++) { ss[i] = fmaf(xs[e], xs[e], ss[i]); xs[e] = xs[e] * pw[e]; }
            }
#pragma unroll
            for (int r = 0; r < NR; r++)
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    acc[r][i] = fmaf(xs[e], bf2f(w8[r][e]), acc[r][i]);
                    if (gated) acc2[r][i] = fmaf(xs[e], bf2f(w28[r][e]), acc2[r][i]);
                }
        }
    }
#pragma unroll
    for (int i = 0; i < TBR; i++) {
        if (i >= nt) break;
        float q = ss[i];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) q += __shfl_xor(q, o, 64);
        const float inv = pn ? 1.0f / sqrtf(q / (float)a.K + a.pn_eps) : 1.0f;
#pragma unroll
        for (int r = 0; r < NR; r++) {
            float s1 = acc[r][i], s2 = acc2[r][i];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) { s1 += __shfl_xor(s1, o, 64); s2 += __shfl_xor(s2, o, 64); }
            if (pn) { s1 *= inv; s2 *= inv; }
            if (lane == 0 && n0 + r < a.N) v.y[(size_t)i * a.ldy + n0 + r] = epi_apply(a.epi, a.bias ? s1 + a.bias[n0 + r] : s1, s2, a.epi_limit) * a.out_scale;
        }
    }
}

// With the norm prologue the row's sum of squares is gathered in the same pass as the products: y = inv_rms(x) * sum_k w_k (x_k (off + g_k)) - one trip
// through memory per wave, the scale applied to the finished sum.
template <bool VEC>
__global__ __launch_bounds__(256) void mmb_vec_kernel(MMBArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x * 4 + wave;
    const ZView v = z_view(a, blockIdx.y);
    if (n >= a.N) return;
    const unsigned short *wr = v.w + (size_t)n * a.ldw, *wr2 = v.w2 ? v.w2 + (size_t)n * a.ldw : nullptr;
    const bool pn = a.pn_w != nullptr;
    constexpr int TB = 8;
    for (int t0 = 0; t0 < v.rows; t0 += TB) {
        float acc[TB], acc2[TB], ss[TB];
#pragma unroll
        for (int i = 0; i < TB; i++) { acc[i] = 0.0f; acc2[i] = 0.0f; ss[i] = 0.0f; }
        const int nt = v.rows - t0 < TB ? v.rows - t0 : TB;
        if (VEC) {
            for (int k = lane * 8; k < a.K; k += 512) {
                const u16x8 w8 = *reinterpret_cast<const u16x8 *>(wr + k);
                u16x8 w28 = w8;
                if (wr2) w28 = *reinterpret_cast<const u16x8 *>(wr2 + k);
                float pw[8];
                if (pn) {
                    const f32x4 g0 = *reinterpret_cast<const f32x4 *>(a.pn_w + k), g1 = *reinterpret_cast<const f32x4 *>(a.pn_w + k + 4);
                    pw[0] = a.pn_off + g0.x; pw[1] = a.pn_off + g0.y; pw[2] = a.pn_off + g0.z; pw[3] = a.pn_off + g0.w;
                    pw[4] = a.pn_off + g1.x; pw[5] = a.pn_off + g1.y; pw[6] = a.pn_off + g1.z; pw[7] = a.pn_off + g1.w;
                }
#pragma unroll
                for (int i = 0; i < TB; i++) {
                    if (i >= nt) break;
                    const float *xr = v.x + (size_t)(t0 + i) * a.ldx + k;
                    const f32x4 x0 = *reinterpret_cast<const f32x4 *>(xr), x1 = *reinterpret_cast<const f32x4 *>(xr + 4);
                    float xs[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                    if (pn) {
#pragma unroll
                        for (int e = 0; e < 8; e++) { ss[i] = fmaf(xs[e], xs[e], ss[i]); xs[e] = xs[e] * pw[e]; }
                    }
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        acc[i] = fmaf(xs[e], bf2f(w8[e]), acc[i]);
                        if (wr2) acc2[i] = fmaf(xs[e], bf2f(w28[e]), acc2[i]);
                    }
                }
            }
        } else {
            for (int k = lane; k < a.K; k += 64) {
                const float w = bf2f(wr[k]), w2 = wr2 ? bf2f(wr2[k]) : 0.0f, pw = pn ? a.pn_off + a.pn_w[k] : 1.0f;
#pragma unroll
                for (int i = 0; i < TB; i++) {
                    if (i >= nt) break;
                    float x = v.x[(size_t)(t0 + i) * a.ldx + k];
                    if (pn) { ss[i] = fmaf(x, x, ss[i]); x = x * pw; }
                    acc[i] = fmaf(x, w, acc[i]);
                    acc2[i] = fmaf(x, w2, acc2[i]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < TB; i++) {
            if (i >= nt) break;
            float s = acc[i], s2 = acc2[i], q = ss[i];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) { s += __shfl_xor(s, o, 64); s2 += __shfl_xor(s2, o, 64); q += __shfl_xor(q, o, 64); }
            if (pn) { const float inv = 1.0f / sqrtf(q / (float)a.K + a.pn_eps); s *= inv; s2 *= inv; }
            if (lane == 0) v.y[(size_t)(t0 + i) * a.ldy + n] = epi_apply(a.epi, a.bias ? s + a.bias[n] : s, s2, a.epi_limit) * a.out_scale;
        }
    }
}

// ---------------------------------------------------------------- batches, f32: 64 x 64 outputs per workgroup, 16 of k per stage, 4 x 4 per thread
template <bool GATED>
__global__ __launch_bounds__(256) void mmb_f32_kernel(MMBArgs a) {
    constexpr int BM = 64, BN = 64, BK = 16, LD = 68;
    __shared__ float sX[BK][LD], sW[BK][LD], sW2[GATED ? BK : 1][LD];
    const ZView v = z_view(a, blockIdx.z);
    const int t0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    if (t0 >= v.rows) return;                                   // (uniform: before any barrier)
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int lr = tid >> 2, lk = (tid & 3) * 4;                 // loader: row lr of both tiles, 4 consecutive k
    float acc[4][4], acc2[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) { acc[i][j] = 0.0f; acc2[i][j] = 0.0f; }
    const bool xrow = t0 + lr < v.rows, wrow = n0 + lr < a.N;
    const float *xr = v.x + (size_t)(t0 + lr) * a.ldx;
    const unsigned short *wr = v.w + (size_t)(n0 + lr) * a.ldw;
    const unsigned short *wr2 = GATED ? v.w2 + (size_t)(n0 + lr) * a.ldw : nullptr;
    for (int k0 = 0; k0 < a.K; k0 += BK) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int k = k0 + lk + e;
            const bool in = k < a.K;
            sX[lk + e][lr] = xrow && in ? xr[k] : 0.0f;
            sW[lk + e][lr] = wrow && in ? bf2f(wr[k]) : 0.0f;
            if (GATED) sW2[lk + e][lr] = wrow && in ? bf2f(wr2[k]) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; k++) {
            const f32x4 xv = *reinterpret_cast<const f32x4 *>(&sX[k][ty * 4]);
            const f32x4 wv = *reinterpret_cast<const f32x4 *>(&sW[k][tx * 4]);
            const float xs[4] = {xv.x, xv.y, xv.z, xv.w}, ws[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = fmaf(xs[i], ws[j], acc[i][j]);
            if (GATED) {
                const f32x4 w2v = *reinterpret_cast<const f32x4 *>(&sW2[k][tx * 4]);
                const float w2s[4] = {w2v.x, w2v.y, w2v.z, w2v.w};
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) acc2[i][j] = fmaf(xs[i], w2s[j], acc2[i][j]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int t = t0 + ty * 4 + i;
        if (t >= v.rows) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int n = n0 + tx * 4 + j;
            if (n < a.N) v.y[(size_t)t * a.ldy + n] = epi_apply(a.epi, a.bias ? acc[i][j] + a.bias[n] : acc[i][j], acc2[i][j], a.epi_limit) * a.out_scale;
        }
    }
}

// ---------------------------------------------------------------- batches, bf16 on the matrix cores: a wave owns WT x WT tiles of 32 x 32 outputs
template <int WT, bool GATED>
__global__ __launch_bounds__(256) void mmb_mfma_kernel(MMBArgs a) {
    const ZView v = z_view(a, blockIdx.z);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, kg = lane >> 5;
    const int n0 = blockIdx.x * (64 * WT) + (wave & 1) * (32 * WT), t0 = blockIdx.y * (64 * WT) + (wave >> 1) * (32 * WT);
    if (n0 >= a.N || t0 >= v.rows) return;                      // (wave-uniform, no barriers in this kernel)
    const unsigned short *wr[WT], *wr2[WT];
    const float *xr[WT];
#pragma unroll
    for (int i = 0; i < WT; i++) {
        const int n = n0 + 32 * i + m, t = t0 + 32 * i + m;     // rows past the end read the last row; their results are never stored
        wr[i] = v.w + (size_t)(n < a.N ? n : a.N - 1) * a.ldw + 8 * kg;
        wr2[i] = GATED ? v.w2 + (size_t)(n < a.N ? n : a.N - 1) * a.ldw + 8 * kg : nullptr;
        xr[i] = v.x + (size_t)(t < v.rows ? t : v.rows - 1) * a.ldx + 8 * kg;
    }
    f32x16 acc[WT][WT], acc2[GATED ? WT : 1][GATED ? WT : 1];
#pragma unroll
    for (int i = 0; i < WT; i++)
#pragma unroll
        for (int j = 0; j < WT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) { acc[i][j][r] = 0.0f; if (GATED) acc2[i][j][r] = 0.0f; }
    // PD steps of k are requested together, and the next PD while these are multiplied: a request per step in the chain would wait a memory round trip
    // for every 16 of k.  Steps past K read the row's last step again and are never multiplied.
    constexpr int PD = WT == 1 ? 4 : 2;
    bf16x8 wa[2][PD][WT], wb[2][PD][GATED ? WT : 1];
    f32x4 xa[2][PD][WT][2];
    const int klast = a.K - 16;
    const auto request = [&](int buf, int k0) {
#pragma unroll
        for (int u = 0; u < PD; u++) {
            const int k = k0 + 16 * u <= klast ? k0 + 16 * u : klast;
#pragma unroll
            for (int i = 0; i < WT; i++) {
                wa[buf][u][i] = *reinterpret_cast<const bf16x8 *>(wr[i] + k);
                if (GATED) wb[buf][u][i] = *reinterpret_cast<const bf16x8 *>(wr2[i] + k);
                xa[buf][u][i][0] = *reinterpret_cast<const f32x4 *>(xr[i] + k);
                xa[buf][u][i][1] = *reinterpret_cast<const f32x4 *>(xr[i] + k + 4);
            }
        }
    };
    const auto multiply = [&](int buf, int k0) {
#pragma unroll
        for (int u = 0; u < PD; u++) {
            if (k0 + 16 * u > klast) break;
            bf16x8 xb[WT];
#pragma unroll
            for (int i = 0; i < WT; i++) {
                const f32x4 x0 = xa[buf][u][i][0], x1 = xa[buf][u][i][1];
                u16x8 xb16 = {f2bf(x0.x), f2bf(x0.y), f2bf(x0.z), f2bf(x0.w), f2bf(x1.x), f2bf(x1.y), f2bf(x1.z), f2bf(x1.w)};
                xb[i] = __builtin_bit_cast(bf16x8, xb16);
            }
#pragma unroll
            for (int i = 0; i < WT; i++)
#pragma unroll
                for (int j = 0; j < WT; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa[buf][u][i], xb[j], acc[i][j], 0, 0, 0);
                    if (GATED) acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[buf][u][i], xb[j], acc2[i][j], 0, 0, 0);
                }
        }
    };
    request(0, 0);
    for (int k0 = 0; k0 < a.K; k0 += 32 * PD) {
        request(1, k0 + 16 * PD);
        multiply(0, k0);
        request(0, k0 + 32 * PD);
        multiply(1, k0 + 16 * PD);
    }
    // register r of a lane: weight row (r & 3) + 8 (r >> 2) + 4 kg of the tile, token = lane & 31
#pragma unroll
    for (int i = 0; i < WT; i++)
#pragma unroll
        for (int j = 0; j < WT; j++) {
            const int t = t0 + 32 * j + m;
            if (t >= v.rows) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int n = n0 + 32 * i + (r & 3) + 8 * (r >> 2) + 4 * kg;
                if (n < a.N) v.y[(size_t)t * a.ldy + n] = epi_apply(a.epi, a.bias ? acc[i][j][r] + a.bias[n] : acc[i][j][r], GATED ? acc2[i][j][r] : 0.0f, a.epi_limit) * a.out_scale;
            }
        }
}

}  // namespace

hipError_t launch_mmb(const MMBArgs &a, hipStream_t st) {
    if (a.T <= 0 || a.N <= 0 || a.nz <= 0) return hipSuccess;
    const bool gated = a.epi == MMB_SILU_MUL || a.epi == MMB_GELU_MUL || a.epi == MMB_CLAMP_SWIGLU;
    if (a.K <= 0 || !a.x || !a.w || !a.y || (gated && !a.w2)) return hipErrorInvalidValue;
    const auto al = [](const void *p, size_t n) { return (reinterpret_cast<uintptr_t>(p) & (n - 1)) == 0; };
    // 16-byte loads of both operands: every row start and every stride on a 16-byte boundary
    const bool vec = (a.K % 8) == 0 && (a.ldw % 8) == 0 && (a.w_zs % 8) == 0 && (a.ldx % 4) == 0 && (a.x_zs % 4) == 0 && al(a.w, 16) && al(a.x, 16) &&
                     (!a.w2 || al(a.w2, 16)) && (!a.pn_w || al(a.pn_w, 16));
    const int rows_max = a.sel ? 1 : a.T;                        // most rows any outer index can hold
    if (a.pn_w && rows_max > MMB_VEC_ROWS) return hipErrorInvalidValue;   // (the norm prologue lives in the few-rows kernel only)
    if (rows_max <= MMB_VEC_ROWS || a.sel) {
        const dim3 grid((unsigned)((a.N + 3) / 4), (unsigned)a.nz);
        // many columns, a handful of rows: four weight rows per wave (the grid still has thousands of waves)
        if (vec && !a.sel && !a.meta && rows_max <= 4 && (long long)a.N * a.nz >= 4096) {
            const dim3 g4((unsigned)((a.N + 15) / 16), (unsigned)a.nz);
            if (rows_max == 1) hipLaunchKernelGGL((mmb_vec_rows_kernel<4, 1>), g4, dim3(256), 0, st, a);
            else hipLaunchKernelGGL((mmb_vec_rows_kernel<4, 4>), g4, dim3(256), 0, st, a);
            return hipGetLastError();
        }
        if (vec) hipLaunchKernelGGL(mmb_vec_kernel<true>, grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL(mmb_vec_kernel<false>, grid, dim3(256), 0, st, a);
        return hipGetLastError();
    }
    if (!a.f32 && vec && (a.K % 16) == 0) {
        const dim3 big((unsigned)((a.N + 127) / 128), (unsigned)((rows_max + 127) / 128), (unsigned)a.nz);
        // (a grouped batch sizes its grid for the most rows ONE expert could hold; what counts for filling the device is the rows an expert holds on average)
        const unsigned rows_avg = a.meta ? (unsigned)((a.T + a.nz - 1) / a.nz) : (unsigned)rows_max;
        if (big.x * ((rows_avg + 127) / 128) * big.z >= (a.meta ? 256u : 512u) && !gated) hipLaunchKernelGGL((mmb_mfma_kernel<2, false>), big, dim3(256), 0, st, a);
        else {
            const dim3 grid((unsigned)((a.N + 63) / 64), (unsigned)((rows_max + 63) / 64), (unsigned)a.nz);
            if (gated) hipLaunchKernelGGL((mmb_mfma_kernel<1, true>), grid, dim3(256), 0, st, a);
            else hipLaunchKernelGGL((mmb_mfma_kernel<1, false>), grid, dim3(256), 0, st, a);
        }
        return hipGetLastError();
    }
    const dim3 grid((unsigned)((a.N + 63) / 64), (unsigned)((rows_max + 63) / 64), (unsigned)a.nz);
    if (gated) hipLaunchKernelGGL(mmb_f32_kernel<true>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(mmb_f32_kernel<false>, grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace mi355
