// Layer epilogue of the SC CNNs, fused into one pass over the convolution's int32 counts
// (gfx950, HBM-bound).  The reference runs it as a chain of PyTorch element-wise ops per layer
// (network.py:165-170, utils_class.py:44-65, utils_functional.py:33-39, utils_class.py:32):
//     x  = count / L                               (utils_functional.py:632)
//     v  = x * w_n[c] + b_n[c]                     fixed-point batch norm: value of BatchNorm*_fixed
//     v  = relu(v)                                 optional (network.py:167)
//     v  = AvgPool2d(2)(v)                         sum of the 2x2 window in row-major order, / 4
//     v  = Hardtanh(0, 1)(v)
//     v  = round(v * 128).clamp(-127, 127) / 128   the next layer's input quantisation
// Every step keeps PyTorch's operation order and rounding (separate multiply and add, round half
// to even), so the result is the same float the op chain produces.  Besides the fp32 activation
// the kernel can emit the 7-bit integer round(v*128) as uint8, which the activation stream
// generator reads directly in place of fp32.
#include "sc_common.h"

namespace geo_sc {

namespace {

struct EpiParams {
    const int32_t* __restrict__ counts;
    const float* __restrict__ w_n;
    const float* __restrict__ b_n;
    float* __restrict__ act;
    uint8_t* __restrict__ q7;
    int c, w, h, wo, ho;
    long long total;  // n * c * wo * ho
    float inv_len;    // 1 / L, a power of two
    int flags;
};

__device__ __forceinline__ float affine(int count, float inv_len, float wn, float bn, bool relu)
{
    // x.data * w_n + b_n as two rounded operations (no fused multiply-add)
    const float x = __fmul_rn((float)count, inv_len);
    float v = __fadd_rn(__fmul_rn(x, wn), bn);
    if (relu) v = fmaxf(v, 0.0f);
    return v;
}

__global__ __launch_bounds__(256) void k_layer_epilogue(EpiParams q)
{
    const bool relu = q.flags & GEO_SC_EPI_RELU, pool = q.flags & GEO_SC_EPI_POOL2;
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < q.total; e += (long long)gridDim.x * 256) {
        const int b = (int)(e % q.ho);
        long long t = e / q.ho;
        const int a = (int)(t % q.wo);
        t /= q.wo;  // n * c + channel
        const int ch = (int)(t % q.c);
        const float wn = q.w_n[ch], bn = q.b_n[ch];
        float v;
        if (pool) {
            const int32_t* src = q.counts + (t * q.w + 2 * a) * q.h + 2 * b;
            const float v00 = affine(src[0], q.inv_len, wn, bn, relu);
            const float v01 = affine(src[1], q.inv_len, wn, bn, relu);
            const float v10 = affine(src[q.h], q.inv_len, wn, bn, relu);
            const float v11 = affine(src[q.h + 1], q.inv_len, wn, bn, relu);
            v = __fadd_rn(__fadd_rn(__fadd_rn(v00, v01), v10), v11) / 4.0f;
        } else {
            v = affine(q.counts[e], q.inv_len, wn, bn, relu);
        }
        if (q.flags & GEO_SC_EPI_HARDTANH01) v = fminf(fmaxf(v, 0.0f), 1.0f);
        if (q.flags & GEO_SC_EPI_QUANT7) {
            const float k = fminf(fmaxf(rintf(__fmul_rn(v, 128.0f)), -127.0f), 127.0f);
            v = k / 128.0f;
            if (q.q7) q.q7[e] = (uint8_t)(int)k;
        }
        if (q.act) q.act[e] = v;
    }
}

// AvgPool2 case with h a multiple of 4: a thread produces two adjacent outputs from two 16-byte
// loads (one per input row), 32-bit index arithmetic; a wave reads two contiguous 1 KB runs.
__global__ __launch_bounds__(256) void k_layer_epilogue_pool_vec(EpiParams q, unsigned pairs_per_row, unsigned n_pairs)
{
    const bool relu = q.flags & GEO_SC_EPI_RELU;
    for (unsigned e = blockIdx.x * 256 + threadIdx.x; e < n_pairs; e += gridDim.x * 256) {
        const unsigned b2 = e % pairs_per_row;
        unsigned t = e / pairs_per_row;
        const unsigned a = t % (unsigned)q.wo;
        t /= (unsigned)q.wo;
        const unsigned ch = t % (unsigned)q.c;
        const float wn = q.w_n[ch], bn = q.b_n[ch];
        const int32_t* src = q.counts + ((size_t)t * q.w + 2 * a) * q.h + 4 * b2;
        const int4 r0 = *reinterpret_cast<const int4*>(src);
        const int4 r1 = *reinterpret_cast<const int4*>(src + q.h);
        float v[2];
        v[0] = __fadd_rn(__fadd_rn(__fadd_rn(affine(r0.x, q.inv_len, wn, bn, relu), affine(r0.y, q.inv_len, wn, bn, relu)),
                                   affine(r1.x, q.inv_len, wn, bn, relu)),
                         affine(r1.y, q.inv_len, wn, bn, relu)) / 4.0f;
        v[1] = __fadd_rn(__fadd_rn(__fadd_rn(affine(r0.z, q.inv_len, wn, bn, relu), affine(r0.w, q.inv_len, wn, bn, relu)),
                                   affine(r1.z, q.inv_len, wn, bn, relu)),
                         affine(r1.w, q.inv_len, wn, bn, relu)) / 4.0f;
        uint8_t k8[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (q.flags & GEO_SC_EPI_HARDTANH01) v[i] = fminf(fmaxf(v[i], 0.0f), 1.0f);
            if (q.flags & GEO_SC_EPI_QUANT7) {
                const float k = fminf(fmaxf(rintf(__fmul_rn(v[i], 128.0f)), -127.0f), 127.0f);
                v[i] = k / 128.0f;
                k8[i] = (uint8_t)(int)k;
            }
        }
        const size_t o = (size_t)e * 2;
        if (q.q7) *reinterpret_cast<uchar2*>(q.q7 + o) = make_uchar2(k8[0], k8[1]);
        if (q.act) *reinterpret_cast<float2*>(q.act + o) = make_float2(v[0], v[1]);
    }
}

// ---------------------------------------------------------------------------------------------
// Backward of the layer tail in training mode.  The reference's autograd sees
//     y = count / L -> F.batch_norm(y, training=True) (its value replaced by y * w_n + b_n,
//     utils_class.py:49-64) -> relu -> AvgPool2d(2) -> Hardtanh(0, 1)
// so the gradient is that of an ordinary batch norm on the batch statistics, with the relu and
// hardtanh masks taken from the fixed-point values that actually flowed forward:
//     d[n,c,i,j]  = grad_out[n,c,i/2,j/2] * [0 < pooled value < 1] / 4 * [value before relu > 0]
//     dbeta[c]    = sum d,   dgamma[c] = sum d * xhat,   xhat = (y - mean[c]) * invstd[c]
//     dy          = gamma[c] * invstd[c] * (d - dbeta[c] / M - xhat * dgamma[c] / M),  M = n*w*h
// Two kernels: per-channel partial sums (fixed-order tree per block), then the element-wise application, whose
// blocks first add the few partial sums of every channel in split order (deterministic).
struct TailParams {
    const int32_t* __restrict__ counts;
    const float* __restrict__ gout;
    const float* __restrict__ w_n;
    const float* __restrict__ b_n;
    const float* __restrict__ mean;
    const float* __restrict__ invstd;
    const float* __restrict__ gamma;  // may be null: 1
    int n, c, w, h, wo, ho;
    float inv_len;
    int flags;
    int splits;
};

// gradient reaching the batch-norm output at (item-channel plane nc, i, j)
__device__ __forceinline__ float tail_d(const TailParams& q, long long nc, int i, int j, float wn, float bn, int count_ij)
{
    const bool relu = q.flags & GEO_SC_EPI_RELU;
    float g;
    if (q.flags & GEO_SC_EPI_POOL2) {
        if (i >= 2 * q.wo || j >= 2 * q.ho) return 0.0f;
        const int a = i >> 1, b = j >> 1;
        const int32_t* src = q.counts + (nc * q.w + 2 * a) * q.h + 2 * b;
        const float v00 = affine(src[0], q.inv_len, wn, bn, relu), v01 = affine(src[1], q.inv_len, wn, bn, relu);
        const float v10 = affine(src[q.h], q.inv_len, wn, bn, relu), v11 = affine(src[q.h + 1], q.inv_len, wn, bn, relu);
        const float pooled = __fadd_rn(__fadd_rn(__fadd_rn(v00, v01), v10), v11) / 4.0f;
        g = q.gout[(nc * q.wo + a) * q.ho + b];
        if ((q.flags & GEO_SC_EPI_HARDTANH01) && !(pooled > 0.0f && pooled < 1.0f)) g = 0.0f;
        g *= 0.25f;
    } else {
        const float v = affine(count_ij, q.inv_len, wn, bn, relu);
        g = q.gout[(nc * q.w + i) * q.h + j];
        if ((q.flags & GEO_SC_EPI_HARDTANH01) && !(v > 0.0f && v < 1.0f)) g = 0.0f;
    }
    if (relu && !(affine(count_ij, q.inv_len, wn, bn, false) > 0.0f)) g = 0.0f;
    return g;
}

// partial[ch][split][2]: sums of d and d * xhat over this split's share of the channel's elements
__global__ __launch_bounds__(256) void k_tail_bwd_partial(TailParams q, float* __restrict__ partial)
{
    __shared__ float red[2][256];
    const int ch = blockIdx.y;
    const float wn = q.w_n[ch], bn = q.b_n[ch], mu = q.mean[ch], is = q.invstd[ch];
    const int plane = q.w * q.h;
    const long long per_channel = (long long)q.n * plane;
    float s1 = 0.0f, s2 = 0.0f;
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < per_channel; e += (long long)q.splits * 256) {
        const long long item = e / plane;
        const int r = (int)(e - item * plane);
        const int i = r / q.h, j = r - i * q.h;
        const long long nc = item * q.c + ch;
        const int cnt = q.counts[nc * plane + r];
        const float d = tail_d(q, nc, i, j, wn, bn, cnt);
        const float xhat = ((float)cnt * q.inv_len - mu) * is;
        s1 += d;
        s2 += d * xhat;
    }
    red[0][threadIdx.x] = s1;
    red[1][threadIdx.x] = s2;
    __syncthreads();
    for (int step = 128; step >= 1; step >>= 1) {
        if ((int)threadIdx.x < step) {
            red[0][threadIdx.x] += red[0][threadIdx.x + step];
            red[1][threadIdx.x] += red[1][threadIdx.x + step];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partial[((size_t)ch * q.splits + blockIdx.x) * 2] = red[0][0];
        partial[((size_t)ch * q.splits + blockIdx.x) * 2 + 1] = red[1][0];
    }
}

// The pooled tail with even plane sides, one 2 x 2 pool window per thread: the window's four counts as two
// 8-byte loads, the pooled value and its hardtanh mask once for the four elements (the element-wise kernels
// recompute them per element), d[0..3] and xhat[0..3] of the window in row order.
struct TailWindow {
    float d[4], xhat[4];
};
__device__ __forceinline__ TailWindow tail_window(const TailParams& q, long long nc, int a, int b, float wn, float bn,
                                                  float mu, float is)
{
    const bool relu = q.flags & GEO_SC_EPI_RELU;
    const int32_t* src = q.counts + (nc * q.w + 2 * a) * q.h + 2 * b;
    const int2 r0 = *(const int2*)src, r1 = *(const int2*)(src + q.h);
    const int cnt[4] = {r0.x, r0.y, r1.x, r1.y};
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = affine(cnt[k], q.inv_len, wn, bn, relu);
    const float pooled = __fadd_rn(__fadd_rn(__fadd_rn(v[0], v[1]), v[2]), v[3]) / 4.0f;
    float g = q.gout[(nc * q.wo + a) * q.ho + b];
    if ((q.flags & GEO_SC_EPI_HARDTANH01) && !(pooled > 0.0f && pooled < 1.0f)) g = 0.0f;
    g *= 0.25f;
    TailWindow t;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        t.d[k] = (relu && !(affine(cnt[k], q.inv_len, wn, bn, false) > 0.0f)) ? 0.0f : g;
        t.xhat[k] = ((float)cnt[k] * q.inv_len - mu) * is;
    }
    return t;
}

__global__ __launch_bounds__(256) void k_tail_bwd_partial_pool(TailParams q, float* __restrict__ partial)
{
    __shared__ float red[2][256];
    const int ch = blockIdx.y;
    const float wn = q.w_n[ch], bn = q.b_n[ch], mu = q.mean[ch], is = q.invstd[ch];
    const int windows = q.wo * q.ho;
    const long long per_channel = (long long)q.n * windows;
    float s1 = 0.0f, s2 = 0.0f;
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < per_channel; e += (long long)q.splits * 256) {
        const int item = (int)(e / windows), r = (int)(e - (long long)item * windows);
        const int a = r / q.ho, b = r - a * q.ho;
        const TailWindow t = tail_window(q, (long long)item * q.c + ch, a, b, wn, bn, mu, is);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            s1 += t.d[k];
            s2 += t.d[k] * t.xhat[k];
        }
    }
    red[0][threadIdx.x] = s1;
    red[1][threadIdx.x] = s2;
    __syncthreads();
    for (int step = 128; step >= 1; step >>= 1) {
        if ((int)threadIdx.x < step) {
            red[0][threadIdx.x] += red[0][threadIdx.x + step];
            red[1][threadIdx.x] += red[1][threadIdx.x + step];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partial[((size_t)ch * q.splits + blockIdx.x) * 2] = red[0][0];
        partial[((size_t)ch * q.splits + blockIdx.x) * 2 + 1] = red[1][0];
    }
}

// sums[c][2] (dbeta, dgamma) in LDS from partial[c][splits][2], splits <= 32: half a wave per channel, one
// partial sum per lane, then a xor tree over the 32 lanes - the same order of additions in every block, so
// all blocks hold the same bits whatever the scheduling
__device__ __forceinline__ void tail_sums_to_lds(float* __restrict__ sums, const float* __restrict__ partial, int c,
                                                 int splits)
{
    const int sub = threadIdx.x & 31;
    for (int ch0 = 0; ch0 < c; ch0 += 8) {
        const int ch = ch0 + (threadIdx.x >> 5);
        float s1 = 0.0f, s2 = 0.0f;
        if (ch < c && sub < splits) {
            const float2 p = *(const float2*)(partial + ((size_t)ch * splits + sub) * 2);
            s1 = p.x;
            s2 = p.y;
        }
        for (int step = 16; step >= 1; step >>= 1) {
            s1 += __shfl_xor(s1, step);
            s2 += __shfl_xor(s2, step);
        }
        if (ch < c && sub == 0) {
            sums[2 * ch] = s1;
            sums[2 * ch + 1] = s2;
        }
    }
    __syncthreads();
}

__global__ __launch_bounds__(256) void k_tail_bwd_apply_pool(TailParams q, const float* __restrict__ partial,
                                                             float* __restrict__ grad_y, float* __restrict__ grad_gamma,
                                                             float* __restrict__ grad_beta)
{
    extern __shared__ float sums[];
    tail_sums_to_lds(sums, partial, q.c, q.splits);
    const int windows = q.wo * q.ho;
    const long long total = (long long)q.n * q.c * windows;
    const float inv_m = 1.0f / (float)((long long)q.n * q.w * q.h);
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
        const long long nc = e / windows;
        const int r = (int)(e - nc * windows);
        const int a = r / q.ho, b = r - a * q.ho;
        const int ch = (int)(nc % q.c);
        const float is = q.invstd[ch];
        const TailWindow t = tail_window(q, nc, a, b, q.w_n[ch], q.b_n[ch], q.mean[ch], is);
        const float gm = (q.gamma ? q.gamma[ch] : 1.0f) * is, sb = sums[2 * ch] * inv_m, sg = sums[2 * ch + 1] * inv_m;
        float o[4];
#pragma unroll
        for (int k = 0; k < 4; k++) o[k] = gm * (t.d[k] - sb - t.xhat[k] * sg);
        float* dst = grad_y + (nc * q.w + 2 * a) * q.h + 2 * b;
        *(float2*)dst = make_float2(o[0], o[1]);
        *(float2*)(dst + q.h) = make_float2(o[2], o[3]);
    }
    if (blockIdx.x == 0)
        for (int ch = threadIdx.x; ch < q.c; ch += 256) {
            if (grad_beta) grad_beta[ch] = sums[2 * ch];
            if (grad_gamma) grad_gamma[ch] = sums[2 * ch + 1];
        }
}

__global__ __launch_bounds__(256) void k_tail_bwd_apply(TailParams q, const float* __restrict__ partial,
                                                        float* __restrict__ grad_y, float* __restrict__ grad_gamma,
                                                        float* __restrict__ grad_beta)
{
    extern __shared__ float sums[];
    tail_sums_to_lds(sums, partial, q.c, q.splits);
    const int plane = q.w * q.h;
    const long long total = (long long)q.n * q.c * plane;
    const float inv_m = 1.0f / (float)((long long)q.n * plane);
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
        const long long nc = e / plane;
        const int r = (int)(e - nc * plane);
        const int i = r / q.h, j = r - i * q.h;
        const int ch = (int)(nc % q.c);
        const float is = q.invstd[ch];
        const int cnt = q.counts[e];
        const float d = tail_d(q, nc, i, j, q.w_n[ch], q.b_n[ch], cnt);
        const float xhat = ((float)cnt * q.inv_len - q.mean[ch]) * is;
        const float gm = q.gamma ? q.gamma[ch] : 1.0f;
        grad_y[e] = gm * is * (d - sums[2 * ch] * inv_m - xhat * sums[2 * ch + 1] * inv_m);
    }
    if (blockIdx.x == 0)
        for (int ch = threadIdx.x; ch < q.c; ch += 256) {
            if (grad_beta) grad_beta[ch] = sums[2 * ch];
            if (grad_gamma) grad_gamma[ch] = sums[2 * ch + 1];
        }
}

// The fixed-point affine of BatchNorm*_fixed from per-channel statistics (utils_class.py:52-62 with
// quantize_shift, utils_functional.py:41-57), one workgroup:
//     inv = sqrt(var + eps);  w = gamma / inv;  b = beta - mean * gamma / inv
//     scale = 2 ** ceil(log2(mean_over_channels(w) * 3))
//     w_n = round(w / scale * 128).clamp(-127, 127) / 128 * scale,   b_n likewise with the same scale
// in PyTorch's operation order, one rounding per operation.  Also the running statistics of
// F.batch_norm(training=True) (momentum 0.1, unbiased variance) and 1 / sqrt(var + eps_grad) for the
// backward.  The channel mean is accumulated in double precision.
__global__ __launch_bounds__(256) void k_bn_fixed_affine(const float* mean, const float* var,
                                                         const float* __restrict__ gamma, const float* __restrict__ beta,
                                                         int c, float eps, float eps_grad, float unbias,
                                                         float* __restrict__ running_mean,
                                                         float* __restrict__ running_var, float* __restrict__ w_n,
                                                         float* __restrict__ b_n, float* __restrict__ invstd,
                                                         float* __restrict__ scale_out,
                                                         const unsigned long long* __restrict__ partial, int splits,
                                                         double inv_elements_len, double inv_elements_len2,
                                                         float* __restrict__ mean_out, float* __restrict__ var_out)
{
    __shared__ double red[256];
    __shared__ float scale_s;
    if (partial) {
        // the statistics themselves, from the exact integer sums of k_count_stats_partial (as
        // k_count_stats_finalize forms them); mean / var then point at mean_out / var_out
        for (int ch = threadIdx.x; ch < c; ch += 256) {
            long long s1 = 0, s2 = 0;
            for (int s = 0; s < splits; s++) {
                s1 += (long long)partial[((size_t)ch * splits + s) * 2];
                s2 += (long long)partial[((size_t)ch * splits + s) * 2 + 1];
            }
            const double m = (double)s1 * inv_elements_len;
            const double v = (double)s2 * inv_elements_len2 - m * m;
            mean_out[ch] = (float)m;
            var_out[ch] = (float)(v > 0.0 ? v : 0.0);
        }
        __threadfence_block();
        __syncthreads();
        mean = mean_out;
        var = var_out;
    }
    double part = 0.0;
    for (int ch = threadIdx.x; ch < c; ch += 256) {
        const float inv = __fsqrt_rn(__fadd_rn(var[ch], eps));
        const float gm = gamma ? gamma[ch] : 1.0f;
        part += (double)__fdiv_rn(gm, inv);
    }
    red[threadIdx.x] = part;
    __syncthreads();
    for (int step = 128; step >= 1; step >>= 1) {
        if ((int)threadIdx.x < step) red[threadIdx.x] += red[threadIdx.x + step];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float m = (float)(red[0] / (double)c);
        scale_s = exp2f(ceilf(log2f(__fmul_rn(m, 3.0f))));
        if (scale_out) *scale_out = scale_s;
    }
    __syncthreads();
    const float scale = scale_s;
    for (int ch = threadIdx.x; ch < c; ch += 256) {
        const float mu = mean[ch], vr = var[ch];
        const float inv = __fsqrt_rn(__fadd_rn(vr, eps));
        const float gm = gamma ? gamma[ch] : 1.0f, bt = beta ? beta[ch] : 0.0f;
        const float w = __fdiv_rn(gm, inv);
        const float b = __fsub_rn(bt, __fdiv_rn(__fmul_rn(mu, gm), inv));
        const float qw = fminf(fmaxf(rintf(__fmul_rn(__fdiv_rn(w, scale), 128.0f)), -127.0f), 127.0f);
        const float qb = fminf(fmaxf(rintf(__fmul_rn(__fdiv_rn(b, scale), 128.0f)), -127.0f), 127.0f);
        w_n[ch] = __fmul_rn(__fdiv_rn(qw, 128.0f), scale);
        b_n[ch] = __fmul_rn(__fdiv_rn(qb, 128.0f), scale);
        if (invstd) invstd[ch] = 1.0f / __fsqrt_rn(__fadd_rn(vr, eps_grad));
        if (running_mean) running_mean[ch] = __fadd_rn(__fmul_rn(running_mean[ch], 0.9f), __fmul_rn(mu, 0.1f));
        if (running_var)
            running_var[ch] = __fadd_rn(__fmul_rn(running_var[ch], 0.9f), __fmul_rn(__fmul_rn(vr, unbias), 0.1f));
    }
}

// Channel statistics of y = counts / bit_length (the mean and the biased variance BatchNorm*_fixed takes of
// the layer's output, utils_class.py:52-56) from the integer counts: the sums of counts and of their squares
// are exact in 64-bit integers, so the result does not depend on how the elements are dealt to threads.
// partial[ch][split][2].  VEC: four counts per load (planes of whole int4 in a 16-byte aligned tensor).
template <bool VEC>
__global__ __launch_bounds__(256) void k_count_stats_partial(const int32_t* __restrict__ counts, int n, int c, int plane,
                                                             int splits, unsigned long long* __restrict__ partial)
{
    __shared__ unsigned long long red[2][256];
    const int ch = blockIdx.y;
    const long long per_channel = (long long)n * plane;
    unsigned long long s1 = 0, s2 = 0;
    if (VEC) {
        const int quads = plane / 4;
        const long long total = (long long)n * quads;
        for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)splits * 256) {
            const long long item = e / quads;
            const int r = (int)(e - item * quads);
            const int4 v = *(const int4*)(counts + (item * c + ch) * plane + 4 * r);
            s1 += (unsigned long long)((long long)v.x + v.y + v.z + v.w);
            s2 += (unsigned long long)((long long)v.x * v.x + (long long)v.y * v.y + (long long)v.z * v.z +
                                       (long long)v.w * v.w);
        }
    } else {
        for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < per_channel; e += (long long)splits * 256) {
            const long long item = e / plane;
            const int r = (int)(e - item * plane);
            const long long v = counts[(item * c + ch) * plane + r];
            s1 += (unsigned long long)v;
            s2 += (unsigned long long)(v * v);
        }
    }
    red[0][threadIdx.x] = s1;
    red[1][threadIdx.x] = s2;
    __syncthreads();
    for (int step = 128; step >= 1; step >>= 1) {
        if ((int)threadIdx.x < step) {
            red[0][threadIdx.x] += red[0][threadIdx.x + step];
            red[1][threadIdx.x] += red[1][threadIdx.x + step];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partial[((size_t)ch * splits + blockIdx.x) * 2] = red[0][0];
        partial[((size_t)ch * splits + blockIdx.x) * 2 + 1] = red[1][0];
    }
}

// one wave per channel: mean = S1 / (elements * L), var = S2 / (elements * L^2) - mean^2, formed in double
// precision from the exact sums and rounded to fp32 once (counts may be negative: the sums are signed)
__global__ __launch_bounds__(64) void k_count_stats_finalize(const unsigned long long* __restrict__ partial, int splits,
                                                             double inv_elements_len, double inv_elements_len2,
                                                             float* __restrict__ mean, float* __restrict__ var)
{
    const int ch = blockIdx.x;
    long long s1 = 0, s2 = 0;
    for (int s = threadIdx.x; s < splits; s += 64) {
        s1 += (long long)partial[((size_t)ch * splits + s) * 2];
        s2 += (long long)partial[((size_t)ch * splits + s) * 2 + 1];
    }
    for (int step = 32; step >= 1; step >>= 1) {
        s1 += __shfl_xor(s1, step);
        s2 += __shfl_xor(s2, step);
    }
    if (threadIdx.x == 0) {
        const double m = (double)s1 * inv_elements_len;
        const double v = (double)s2 * inv_elements_len2 - m * m;
        mean[ch] = (float)m;
        var[ch] = (float)(v > 0.0 ? v : 0.0);
    }
}

// quantize of the reference (utils_functional.py:33-39), element-wise; comparisons instead of
// fminf / fmaxf so that a NaN stays a NaN as torch.clamp leaves it
__global__ __launch_bounds__(256) void k_quantize(const float* __restrict__ src, float* __restrict__ dst, size_t n,
                                                  float scale, float inv_scale)
{
    const float hi = scale - 1.0f;
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        float v = rintf(src[i] * scale);
        v = v < -hi ? -hi : (v > hi ? hi : v);
        dst[i] = v * inv_scale;
    }
}

constexpr int kTailMaxChannels = 4096;

// The end of the reference's training step (utils_own.py:108-113) for up to kMaxStepTensors parameters in one
// launch: every parameter takes its master copy's value, and where the layer keeps a full-precision buffer
// (weight_org) that buffer becomes the new value clamped to [lo, hi].  blockIdx.y = parameter.
constexpr int kMaxStepTensors = 24;
struct StepTensors {
    const float* master[kMaxStepTensors];
    float* param[kMaxStepTensors];
    float* org[kMaxStepTensors];   // null: no such buffer
    size_t n[kMaxStepTensors];
};
__global__ __launch_bounds__(256) void k_copy_back_clamp(StepTensors t, float lo, float hi)
{
    const int i = blockIdx.y;
    const float* __restrict__ src = t.master[i];
    float* __restrict__ dst = t.param[i];
    float* __restrict__ org = t.org[i];
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < t.n[i]; e += (size_t)gridDim.x * 256) {
        const float v = src[e];
        dst[e] = v;
        // torch.clamp: NaN stays NaN
        if (org) org[e] = v < lo ? lo : (v > hi ? hi : v);
    }
}

// quantize for several tensors in one launch (the weights of all layers of a network); blockIdx.y = tensor
struct QuantTensors {
    const float* src[kMaxStepTensors];
    float* dst[kMaxStepTensors];
    size_t n[kMaxStepTensors];
};
__global__ __launch_bounds__(256) void k_quantize_many(QuantTensors t, float scale, float inv_scale)
{
    const int i = blockIdx.y;
    const float* __restrict__ src = t.src[i];
    float* __restrict__ dst = t.dst[i];
    const float hi = scale - 1.0f;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < t.n[i]; e += (size_t)gridDim.x * 256) {
        float v = rintf(src[e] * scale);
        v = v < -hi ? -hi : (v > hi ? hi : v);
        dst[e] = v * inv_scale;
    }
}

int tail_splits(int n, int c, int w, int h)
{
    // enough blocks to fill the GPU, not more than the channel has 256-element chunks
    const long long per_channel = (long long)n * w * h;
    // few enough that the kernel after the partial sums adds them itself (no launch in between)
    long long s = (4096 + c - 1) / c;
    const long long chunks = (per_channel + 255) / 256;
    if (s > chunks) s = chunks;
    if (s < 1) s = 1;
    if (s > 16 && (long long)c * 16 >= 512) s = 16;
    if (s > 32) s = 32;
    return (int)s;
}

}  // namespace

}  // namespace geo_sc

using namespace geo_sc;

extern "C" int geo_sc_layer_epilogue(const int32_t* counts, int n, int c, int w, int h, int bit_length,
                                     const float* w_n, const float* b_n, int flags, float* act_out,
                                     uint8_t* q7_out, geo_sc_stream_t stream)
{
    if (!counts || !w_n || !b_n || (!act_out && !q7_out)) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (n < 1 || c < 1 || w < 1 || h < 1) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (flags & ~(GEO_SC_EPI_RELU | GEO_SC_EPI_POOL2 | GEO_SC_EPI_HARDTANH01 | GEO_SC_EPI_QUANT7))
        return GEO_SC_ERR_INVALID_ARGUMENT;
    switch (bit_length) {
    case 8: case 16: case 32: case 64: case 128: case 256: break;
    default: return GEO_SC_ERR_BIT_LENGTH;
    }
    // the 7-bit integer output is unsigned: it needs the clamp to [0, 1] and the quantisation
    if (q7_out && (flags & (GEO_SC_EPI_HARDTANH01 | GEO_SC_EPI_QUANT7)) != (GEO_SC_EPI_HARDTANH01 | GEO_SC_EPI_QUANT7))
        return GEO_SC_ERR_INVALID_ARGUMENT;
    EpiParams q;
    q.counts = counts;
    q.w_n = w_n;
    q.b_n = b_n;
    q.act = act_out;
    q.q7 = q7_out;
    q.c = c;
    q.w = w;
    q.h = h;
    q.wo = (flags & GEO_SC_EPI_POOL2) ? w / 2 : w;
    q.ho = (flags & GEO_SC_EPI_POOL2) ? h / 2 : h;
    if (q.wo < 1 || q.ho < 1) return GEO_SC_ERR_INVALID_ARGUMENT;
    q.total = (long long)n * c * q.wo * q.ho;
    q.inv_len = 1.0f / (float)bit_length;
    q.flags = flags;
    const bool aligned = (((uintptr_t)counts & 15) | ((uintptr_t)act_out & 7) | ((uintptr_t)q7_out & 1)) == 0;
    if ((flags & GEO_SC_EPI_POOL2) && h % 4 == 0 && aligned && q.total < 0xffffffffLL) {
        const unsigned n_pairs = (unsigned)(q.total / 2);
        long long vb = ((long long)n_pairs + 255) / 256;
        if (vb > 256 * 32) vb = 256 * 32;
        hipLaunchKernelGGL(k_layer_epilogue_pool_vec, dim3((unsigned)vb), dim3(256), 0, (hipStream_t)stream, q,
                           (unsigned)(q.ho / 2), n_pairs);
        return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
    }
    long long blocks = (q.total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(k_layer_epilogue, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, q);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

extern "C" int geo_sc_layer_tail_backward_workspace_size(int n, int c, int w, int h, size_t* bytes)
{
    if (!bytes || n < 1 || c < 1 || w < 1 || h < 1) return GEO_SC_ERR_INVALID_ARGUMENT;
    *bytes = sizeof(float) * 2 * (size_t)c * tail_splits(n, c, w, h);
    return GEO_SC_OK;
}

extern "C" int geo_sc_layer_tail_backward(const int32_t* counts, const float* grad_out, int n, int c, int w, int h,
                                          int bit_length, const float* w_n, const float* b_n, const float* mean,
                                          const float* invstd, const float* gamma, int flags, float* grad_y,
                                          float* grad_gamma, float* grad_beta, void* workspace,
                                          size_t workspace_bytes, geo_sc_stream_t stream)
{
    if (!counts || !grad_out || !w_n || !b_n || !mean || !invstd || !grad_y) return GEO_SC_ERR_INVALID_ARGUMENT;
    // the application kernel keeps two sums per channel in LDS
    if (n < 1 || c < 1 || w < 1 || h < 1 || c > kTailMaxChannels) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (flags & ~(GEO_SC_EPI_RELU | GEO_SC_EPI_POOL2 | GEO_SC_EPI_HARDTANH01 | GEO_SC_EPI_QUANT7))
        return GEO_SC_ERR_INVALID_ARGUMENT;
    switch (bit_length) {
    case 8: case 16: case 32: case 64: case 128: case 256: break;
    default: return GEO_SC_ERR_BIT_LENGTH;
    }
    size_t need = 0;
    geo_sc_layer_tail_backward_workspace_size(n, c, w, h, &need);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 3u)) return GEO_SC_ERR_WORKSPACE;
    TailParams q;
    q.counts = counts;
    q.gout = grad_out;
    q.w_n = w_n;
    q.b_n = b_n;
    q.mean = mean;
    q.invstd = invstd;
    q.gamma = gamma;
    q.n = n;
    q.c = c;
    q.w = w;
    q.h = h;
    q.wo = (flags & GEO_SC_EPI_POOL2) ? w / 2 : w;
    q.ho = (flags & GEO_SC_EPI_POOL2) ? h / 2 : h;
    if (q.wo < 1 || q.ho < 1) return GEO_SC_ERR_INVALID_ARGUMENT;
    q.inv_len = 1.0f / (float)bit_length;
    q.flags = flags;
    q.splits = tail_splits(n, c, w, h);
    hipStream_t s = (hipStream_t)stream;
    float* partial = (float*)workspace;
    // one pool window per thread where the plane is made of whole windows and rows of counts, of the incoming
    // gradient's source and of the result start on 8-byte boundaries
    const bool windows = (flags & GEO_SC_EPI_POOL2) && w % 2 == 0 && h % 2 == 0 && ((uintptr_t)counts & 7u) == 0 &&
                         ((uintptr_t)grad_y & 7u) == 0;
    if (windows)
        hipLaunchKernelGGL(k_tail_bwd_partial_pool, dim3(q.splits, c), dim3(256), 0, s, q, partial);
    else
        hipLaunchKernelGGL(k_tail_bwd_partial, dim3(q.splits, c), dim3(256), 0, s, q, partial);
    const long long total = (long long)n * c * w * h / (windows ? 4 : 1);
    long long blocks = (total + 255) / 256;
    if (blocks > 256 * 8) blocks = 256 * 8;   // every block first adds the partial sums of all channels
    const size_t lds = sizeof(float) * 2 * (size_t)c;
    if (windows)
        hipLaunchKernelGGL(k_tail_bwd_apply_pool, dim3((unsigned)blocks), dim3(256), lds, s, q, partial, grad_y,
                           grad_gamma, grad_beta);
    else
        hipLaunchKernelGGL(k_tail_bwd_apply, dim3((unsigned)blocks), dim3(256), lds, s, q, partial, grad_y, grad_gamma,
                           grad_beta);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

extern "C" int geo_sc_count_stats_workspace_size(int n, int c, int w, int h, size_t* bytes)
{
    if (!bytes || n < 1 || c < 1 || w < 1 || h < 1) return GEO_SC_ERR_INVALID_ARGUMENT;
    *bytes = sizeof(unsigned long long) * 2 * (size_t)c * tail_splits(n, c, w, h);
    return GEO_SC_OK;
}

extern "C" int geo_sc_count_stats(const int32_t* counts, int n, int c, int w, int h, int bit_length, float* mean,
                                  float* var, void* workspace, size_t workspace_bytes, geo_sc_stream_t stream)
{
    if (!counts || !mean || !var) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (n < 1 || c < 1 || w < 1 || h < 1 || c > 65535) return GEO_SC_ERR_INVALID_ARGUMENT;
    switch (bit_length) {
    case 8: case 16: case 32: case 64: case 128: case 256: break;
    default: return GEO_SC_ERR_BIT_LENGTH;
    }
    size_t need = 0;
    geo_sc_count_stats_workspace_size(n, c, w, h, &need);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 7u)) return GEO_SC_ERR_WORKSPACE;
    // the four-count loads need 16-byte aligned planes
    const int plane = w * h;
    const bool vec_plane = plane % 4 == 0 && ((uintptr_t)counts & 15u) == 0;
    const int splits = tail_splits(n, c, w, h);
    hipStream_t s = (hipStream_t)stream;
    unsigned long long* partial = (unsigned long long*)workspace;
    if (vec_plane)
        hipLaunchKernelGGL(k_count_stats_partial<true>, dim3(splits, c), dim3(256), 0, s, counts, n, c, plane, splits,
                           partial);
    else
        hipLaunchKernelGGL(k_count_stats_partial<false>, dim3(splits, c), dim3(256), 0, s, counts, n, c, plane, splits,
                           partial);
    const double elements = (double)n * plane;
    hipLaunchKernelGGL(k_count_stats_finalize, dim3(c), dim3(64), 0, s, partial, splits,
                       1.0 / (elements * bit_length), 1.0 / (elements * bit_length * (double)bit_length), mean, var);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

extern "C" int geo_sc_bn_fixed_affine(const float* mean, const float* var, const float* gamma, const float* beta,
                                      int c, float eps, float eps_grad, long long elements_per_channel,
                                      float* running_mean, float* running_var, float* w_n, float* b_n, float* invstd,
                                      float* scale, geo_sc_stream_t stream)
{
    if (!mean || !var || !w_n || !b_n || c < 1 || elements_per_channel < 1) return GEO_SC_ERR_INVALID_ARGUMENT;
    const float unbias = elements_per_channel > 1
                             ? (float)((double)elements_per_channel / (double)(elements_per_channel - 1))
                             : 1.0f;
    hipLaunchKernelGGL(k_bn_fixed_affine, dim3(1), dim3(256), 0, (hipStream_t)stream, mean, var, gamma, beta, c, eps,
                       eps_grad, unbias, running_mean, running_var, w_n, b_n, invstd, scale,
                       (const unsigned long long*)nullptr, 0, 0.0, 0.0, (float*)nullptr, (float*)nullptr);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

extern "C" int geo_sc_bn_fixed_from_counts(const int32_t* counts, int n, int c, int w, int h, int bit_length,
                                           const float* gamma, const float* beta, float eps, float eps_grad,
                                           float* running_mean, float* running_var, float* mean, float* var,
                                           float* w_n, float* b_n, float* invstd, float* scale, void* workspace,
                                           size_t workspace_bytes, geo_sc_stream_t stream)
{
    if (!counts || !mean || !var || !w_n || !b_n) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (n < 1 || c < 1 || w < 1 || h < 1 || c > 65535) return GEO_SC_ERR_INVALID_ARGUMENT;
    switch (bit_length) {
    case 8: case 16: case 32: case 64: case 128: case 256: break;
    default: return GEO_SC_ERR_BIT_LENGTH;
    }
    size_t need = 0;
    geo_sc_count_stats_workspace_size(n, c, w, h, &need);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 7u)) return GEO_SC_ERR_WORKSPACE;
    const int plane = w * h;
    const bool vec_plane = plane % 4 == 0 && ((uintptr_t)counts & 15u) == 0;
    const int splits = tail_splits(n, c, w, h);
    hipStream_t s = (hipStream_t)stream;
    unsigned long long* partial = (unsigned long long*)workspace;
    if (vec_plane)
        hipLaunchKernelGGL(k_count_stats_partial<true>, dim3(splits, c), dim3(256), 0, s, counts, n, c, plane, splits,
                           partial);
    else
        hipLaunchKernelGGL(k_count_stats_partial<false>, dim3(splits, c), dim3(256), 0, s, counts, n, c, plane, splits,
                           partial);
    const double elements = (double)n * plane;
    const float unbias = elements > 1 ? (float)(elements / (elements - 1)) : 1.0f;
    hipLaunchKernelGGL(k_bn_fixed_affine, dim3(1), dim3(256), 0, s, (const float*)nullptr, (const float*)nullptr, gamma,
                       beta, c, eps, eps_grad, unbias, running_mean, running_var, w_n, b_n, invstd, scale, partial, splits,
                       1.0 / (elements * bit_length), 1.0 / (elements * bit_length * (double)bit_length), mean, var);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

extern "C" int geo_sc_quantize(const float* src, float* dst, size_t n, int prec, geo_sc_stream_t stream)
{
    if (prec < 1 || prec > 23) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (n == 0) return GEO_SC_OK;
    if (!src || !dst) return GEO_SC_ERR_INVALID_ARGUMENT;
    const float scale = (float)(1u << prec);
    size_t blocks = (n + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(k_quantize, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, src, dst, n, scale,
                       1.0f / scale);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

extern "C" int geo_sc_copy_back_clamp(int count, const float* const* master, float* const* param, float* const* org,
                                      const size_t* elements, float lo, float hi, geo_sc_stream_t stream)
{
    if (count < 0 || (count > 0 && (!master || !param || !elements))) return GEO_SC_ERR_INVALID_ARGUMENT;
    for (int first = 0; first < count; first += kMaxStepTensors) {
        const int m = count - first < kMaxStepTensors ? count - first : kMaxStepTensors;
        StepTensors t = {};
        size_t most = 0;
        for (int i = 0; i < m; i++) {
            if (elements[first + i] && (!master[first + i] || !param[first + i])) return GEO_SC_ERR_INVALID_ARGUMENT;
            t.master[i] = master[first + i];
            t.param[i] = param[first + i];
            t.org[i] = org ? org[first + i] : nullptr;
            t.n[i] = elements[first + i];
            if (t.n[i] > most) most = t.n[i];
        }
        size_t blocks = (most + 255) / 256;
        if (blocks < 1) blocks = 1;
        if (blocks > 1024) blocks = 1024;
        hipLaunchKernelGGL(k_copy_back_clamp, dim3((unsigned)blocks, (unsigned)m), dim3(256), 0, (hipStream_t)stream, t, lo,
                           hi);
    }
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

extern "C" int geo_sc_quantize_many(int count, const float* const* src, float* const* dst, const size_t* elements,
                                    int prec, geo_sc_stream_t stream)
{
    if (prec < 1 || prec > 23 || count < 0 || (count > 0 && (!src || !dst || !elements)))
        return GEO_SC_ERR_INVALID_ARGUMENT;
    const float scale = (float)(1u << prec);
    for (int first = 0; first < count; first += kMaxStepTensors) {
        const int m = count - first < kMaxStepTensors ? count - first : kMaxStepTensors;
        QuantTensors t = {};
        size_t most = 0;
        for (int i = 0; i < m; i++) {
            if (elements[first + i] && (!src[first + i] || !dst[first + i])) return GEO_SC_ERR_INVALID_ARGUMENT;
            t.src[i] = src[first + i];
            t.dst[i] = dst[first + i];
            t.n[i] = elements[first + i];
            if (t.n[i] > most) most = t.n[i];
        }
        size_t blocks = (most + 255) / 256;
        if (blocks < 1) blocks = 1;
        if (blocks > 1024) blocks = 1024;
        hipLaunchKernelGGL(k_quantize_many, dim3((unsigned)blocks, (unsigned)m), dim3(256), 0, (hipStream_t)stream, t,
                           scale, 1.0f / scale);
    }
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}
