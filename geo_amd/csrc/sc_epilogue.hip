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
