// routed_ff.hip — the router and the closing sum of a routed feed-forward that reads its own norm (sigmoid scores, a selection bias, expert groups scored by
// their two best; weighted expert sum + gated always-on expert, alone or together with the norm behind the feed-forward and the residual add).  All f32.
#include "kernels.h"

namespace mi355 {

// Router with a selection bias: one wave per token.  s = sigmoid(z); the choice score c = s + bias decides who is taken, the weight of a taken expert is its s.
// Groups of `per` neighbouring experts score as the sum of their two largest c; the experts of all but the `keep` best groups are closed (c = -inf: choice
// scores may be negative, so nothing else can stand for "closed").  Ties go to the lower index.
__global__ __launch_bounds__(64) void moe_route_sigmoid_bias_kernel(const float *z, int ld_z, const float *bias, int E, int k, int n_group, int keep, int32_t *ids, float *w) {
    extern __shared__ float rl[];
    float *c = rl, *gs = rl + E;                                // [E] choice scores (taken or closed: -inf), [n_group] group scores (a kept group's becomes -inf)
    int *ti = reinterpret_cast<int *>(gs + n_group);            // [k] taken experts
    const int t = blockIdx.x, lane = threadIdx.x, per = E / n_group;
    const float *zr = z + (size_t)t * ld_z;
    for (int e = lane; e < E; e += 64) c[e] = 1.0f / (1.0f + expf(-zr[e])) + (bias ? bias[e] : 0.0f);
    __syncthreads();
    const auto arg_best = [&](const float *v, int n) {
        float bv = -INFINITY; int bi = n;
        for (int i = lane; i < n; i += 64) if (v[i] > bv) { bv = v[i]; bi = i; }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64); const int oi = __shfl_xor(bi, o, 64);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        return bi;
    };
    if (n_group > 1 && keep < n_group) {
        for (int gi = lane; gi < n_group; gi += 64) {
            float b1 = -INFINITY, b2 = -INFINITY;
            for (int e = gi * per; e < (gi + 1) * per; e++) {
                const float x = c[e];
                if (x > b1) { b2 = b1; b1 = x; } else if (x > b2) b2 = x;
            }
            gs[gi] = per > 1 ? b1 + b2 : b1;
        }
        __syncthreads();
        for (int r = 0; r < keep; r++) {
            const int gi = arg_best(gs, n_group);
            __syncthreads();
            if (lane == 0 && gi < n_group) gs[gi] = -INFINITY;
            __syncthreads();
        }
        for (int e = lane; e < E; e += 64) if (gs[e / per] != -INFINITY) c[e] = -INFINITY;
        __syncthreads();
    }
    for (int r = 0; r < k; r++) {
        int ei = arg_best(c, E);
        if (ei >= E) ei = 0;                                     // (fewer open experts than k: refused by the launcher)
        __syncthreads();
        if (lane == 0) { ti[r] = ei; c[ei] = -INFINITY; }
        __syncthreads();
    }
    for (int r = lane; r < k; r += 64) { ids[(size_t)t * k + r] = ti[r]; w[(size_t)t * k + r] = 1.0f / (1.0f + expf(-zr[ti[r]])); }
}
hipError_t launch_moe_route_sigmoid_bias(const float *z, int ld_z, const float *bias, int T, int E, int k, int n_group, int keep, int32_t *ids, float *w, hipStream_t st) {
    if (T <= 0) return hipSuccess;
    if (E < 1 || E > MOE_ROUTE_MAX_EXPERTS || k < 1 || k > E || n_group < 1 || E % n_group != 0 || keep < 1 || keep > n_group) return hipErrorInvalidValue;
    if ((long long)keep * (E / n_group) < k) return hipErrorInvalidValue;
    hipLaunchKernelGGL(moe_route_sigmoid_bias_kernel, dim3((unsigned)T), dim3(64), (size_t)(E + n_group + k) * sizeof(float), st, z, ld_z, bias, E, k, n_group, keep, ids, w);
    return hipGetLastError();
}

// out[t][d] = sum_j w[t][j] * y[row(t, j)][d] (rank order) + sigmoid(sg[t * ld_sg]) * b[t][d]
__global__ void moe_weighted_combine_kernel(float *out, const float *y, const float *w, const int32_t *slot_of, const float *b, const float *sg, int ld_sg, int T, int E, int k) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)T * E) return;
    const int t = (int)(i / E), d = (int)(i - (int64_t)t * E);
    float o = 0.0f;
    for (int j = 0; j < k; j++) o += y[(size_t)(slot_of ? slot_of[(size_t)t * k + j] : t * k + j) * E + d] * w[(size_t)t * k + j];
    if (b) o += (sg ? 1.0f / (1.0f + expf(-sg[(size_t)t * ld_sg])) : 1.0f) * b[i];
    out[i] = o;
}
hipError_t launch_moe_weighted_combine(float *out, const float *y, const float *w, const int32_t *slot_of, const float *b, const float *sg, int ld_sg, int T, int E, int k, hipStream_t st) {
    if ((int64_t)T * E <= 0) return hipSuccess;
    if (k > 0 && (!y || !w)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(moe_weighted_combine_kernel, dim3((unsigned)(((int64_t)T * E + 255) / 256)), dim3(256), 0, st, out, y, w, slot_of, b, sg, ld_sg, T, E, k);
    return hipGetLastError();
}

// one workgroup of 1024 threads per token: the weighted sum into LDS with its sum of squares on the way, then the normed row joins the stream.  The k rows'
// weights and places are read once into LDS; with VEC4 every thread owns four adjacent entries at a time and all its loads of a trip are independent of each
// other (a single token's launch is one workgroup: what it costs is the number of dependent trips to memory)
template <bool VEC4>
__global__ __launch_bounds__(1024) void moe_weighted_combine_norm_kernel(float *x, const float *y, const float *w, const int32_t *slot_of, const float *b, const float *sg,
                                                                         int ld_sg, const float *norm_w, float norm_off, float eps, int E, int k) {
    extern __shared__ float row[];
    __shared__ float part[16], sw[MOE_COMBINE_NORM_MAX_K];
    __shared__ int srow[MOE_COMBINE_NORM_MAX_K];
    const int t = blockIdx.x, tid = threadIdx.x;
    if (tid < k) { sw[tid] = w[(size_t)t * k + tid]; srow[tid] = slot_of ? slot_of[(size_t)t * k + tid] : t * k + tid; }
    const float g = b ? (sg ? 1.0f / (1.0f + expf(-sg[(size_t)t * ld_sg])) : 1.0f) : 0.0f;
    __syncthreads();
    float ss = 0.0f;
    if (VEC4) {
        for (int d = 4 * tid; d < E; d += 4096) {
            float4 o = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll 4
            for (int j = 0; j < k; j++) {
                const float4 v = *reinterpret_cast<const float4 *>(y + (size_t)srow[j] * E + d);
                const float wj = sw[j];
                o.x += v.x * wj; o.y += v.y * wj; o.z += v.z * wj; o.w += v.w * wj;
            }
            if (b) {
                const float4 v = *reinterpret_cast<const float4 *>(b + (size_t)t * E + d);
                o.x += g * v.x; o.y += g * v.y; o.z += g * v.z; o.w += g * v.w;
            }
            *reinterpret_cast<float4 *>(row + d) = o;
            ss = fmaf(o.x, o.x, ss); ss = fmaf(o.y, o.y, ss); ss = fmaf(o.z, o.z, ss); ss = fmaf(o.w, o.w, ss);
        }
    } else {
        for (int d = tid; d < E; d += 1024) {
            float o = 0.0f;
            for (int j = 0; j < k; j++) o += y[(size_t)srow[j] * E + d] * sw[j];
            if (b) o += g * b[(size_t)t * E + d];
            row[d] = o;
            ss = fmaf(o, o, ss);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if ((tid & 63) == 0) part[tid >> 6] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) tot += part[i];
    const float inv = 1.0f / sqrtf(tot / (float)E + eps);
    if (VEC4) {
        for (int d = 4 * tid; d < E; d += 4096) {
            const float4 o = *reinterpret_cast<const float4 *>(row + d), nw = *reinterpret_cast<const float4 *>(norm_w + d);
            float4 xv = *reinterpret_cast<float4 *>(x + (size_t)t * E + d);
            xv.x += o.x * inv * (norm_off + nw.x); xv.y += o.y * inv * (norm_off + nw.y); xv.z += o.z * inv * (norm_off + nw.z); xv.w += o.w * inv * (norm_off + nw.w);
            *reinterpret_cast<float4 *>(x + (size_t)t * E + d) = xv;
        }
    } else {
        for (int d = tid; d < E; d += 1024) x[(size_t)t * E + d] += row[d] * inv * (norm_off + norm_w[d]);
    }
}
hipError_t launch_moe_weighted_combine_norm(float *x, const float *y, const float *w, const int32_t *slot_of, const float *b, const float *sg, int ld_sg,
                                            const float *norm_w, float norm_off, float eps, int T, int E, int k, hipStream_t st) {
    if ((int64_t)T * E <= 0) return hipSuccess;
    if ((k > 0 && (!y || !w)) || !norm_w || E > MOE_COMBINE_NORM_MAX_E || k > MOE_COMBINE_NORM_MAX_K) return hipErrorInvalidValue;
    const auto al16 = [](const void *p) { return !p || (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool vec4 = (E & 3) == 0 && al16(x) && al16(y) && al16(b) && al16(norm_w);
    if (vec4) hipLaunchKernelGGL(moe_weighted_combine_norm_kernel<true>, dim3((unsigned)T), dim3(1024), (size_t)E * sizeof(float), st, x, y, w, slot_of, b, sg, ld_sg, norm_w, norm_off, eps, E, k);
    else hipLaunchKernelGGL(moe_weighted_combine_norm_kernel<false>, dim3((unsigned)T), dim3(1024), (size_t)E * sizeof(float), st, x, y, w, slot_of, b, sg, ld_sg, norm_w, norm_off, eps, E, k);
    return hipGetLastError();
}

}  // namespace mi355
