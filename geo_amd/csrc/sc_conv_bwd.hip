// Surrogate-gradient backward of the SC convolution (gfx950, fp32, MFMA).
//
// The reference trains through a floating-point surrogate of the SC layer
// (utils_functional.py:611-634, :235-252): with wp = clamp(w,0,100), wn = -clamp(w,-100,0)
// and x the zero-padded activation,
//     z+-_v = corr2d(x[..., v : v+Ho], w+-[..., v:v+1])        (kernel W x 1, one per kernel row v)
//     y^    = sum_v (1 - exp(-z+_v)) - sum_v (1 - exp(-z-_v))
// and autograd differentiates y^.  Written out, with g the upstream gradient:
//     E+-_v      = g * exp(-z+-_v)
//     dL/dx      = sum_v corr2d^T(E+_v, wp_v) - corr2d^T(E-_v, wn_v)
//     dL/dw[..v] = [0 <= w <= 100] * sum x E+_v  +  [-100 <= w <= 0] * sum x E-_v
// (clamp passes its gradient on the closed interval, so both terms are live at w == 0).
//
// Per kernel row v this is three dense fp32 contractions over an im2col view of x:
//     Z  [m][j]  = sum_k col[m][k] * Wcat[k][j]        m=(n,a,b)  k=(ci,u)  j=(rail,co)
//     Gw [k][j]  = sum_m col[m][k] * E[m][j]
//     dcol[k][m] = sum_j Wd[j][k]  * E[m][j]           Wd = (wp ; -wn)
// All three run on one MFMA kernel (v_mfma_f32_32x32x2_f32, fp32 in, fp32 accumulate) that
// takes each operand either K-major or I-major; exp and the product with g are fused into
// the first GEMM's epilogue; the second is split over m and reduced deterministically.
#include "sc_common.h"

namespace geo_sc {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kTile = 128;   // block tile in I and J
constexpr int kChunk = 16;   // K per LDS stage
constexpr int kLd = 130;     // LDS row stride: 8*kLd = 16 (mod 32) keeps I-major staging conflict-free

enum Epilogue { EPI_STORE = 0, EPI_EXP_TIMES_G = 1 };

struct GemmParams {
    const float* __restrict__ a;
    const float* __restrict__ b;
    float* __restrict__ c;
    int I, J, K;              // C[I][J] = sum_k A(k,i) * B(k,j)
    long long lda, ldb, ldc;  // leading dimensions (elements)
    int k_per_split;          // K range of one blockIdx.z; c advances by c_split_stride per split
    long long c_split_stride;
    // EPI_EXP_TIMES_G: c[i][j] = g[(n*c_out + j%c_out)*npos + pos] * exp(-acc), i = n*npos + pos
    const float* __restrict__ g;
    int c_out, npos;
};

// Stage a kChunk x kTile tile of an operand into LDS as s[k][i].
//   K-major operand: element (k, i) at p[k*ld + i]  -> rows of the tile are contiguous
//   I-major operand: element (k, i) at p[i*ld + k]  -> each thread walks 8 consecutive k
template <bool KMAJOR>
__device__ __forceinline__ void stage_tile(float (*s)[kLd], const float* __restrict__ p, long long ld, int i0,
                                           int k0, int I, int k_end)
{
    const int t = threadIdx.x;
    if (KMAJOR) {
#pragma unroll
        for (int rep = 0; rep < 8; rep++) {
            const int kk = rep * 2 + (t >> 7), ii = t & 127;
            const int k = k0 + kk, i = i0 + ii;
            s[kk][ii] = (k < k_end && i < I) ? p[(long long)k * ld + i] : 0.0f;
        }
    } else {
        const int ii = t >> 1, kb = (t & 1) * 8;
        const int i = i0 + ii;
        const float* row = p + (long long)i * ld + k0 + kb;
#pragma unroll
        for (int c = 0; c < 8; c++) s[kb + c][ii] = (i < I && k0 + kb + c < k_end) ? row[c] : 0.0f;
    }
}

template <bool A_KMAJOR, bool B_KMAJOR, int EPI>
__global__ __launch_bounds__(256) void k_gemm_f32(GemmParams q)
{
    __shared__ float as[2][kChunk][kLd];
    __shared__ float bs[2][kChunk][kLd];
    const int i0 = blockIdx.x * kTile, j0 = blockIdx.y * kTile;
    const int k_begin = blockIdx.z * q.k_per_split;
    const int k_end = min(q.K, k_begin + q.k_per_split);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wi = (wave >> 1) * 64, wj = (wave & 1) * 64;  // this wave's 64x64 corner in the tile
    const int l32 = lane & 31, lk = lane >> 5;

    floatx16 acc[2][2];
#pragma unroll
    for (int x = 0; x < 2; x++)
#pragma unroll
        for (int y = 0; y < 2; y++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[x][y][r] = 0.0f;

    int buf = 0;
    if (k_begin < k_end) {
        stage_tile<A_KMAJOR>(as[0], q.a, q.lda, i0, k_begin, q.I, k_end);
        stage_tile<B_KMAJOR>(bs[0], q.b, q.ldb, j0, k_begin, q.J, k_end);
    }
    __syncthreads();
    for (int k0 = k_begin; k0 < k_end; k0 += kChunk) {
        if (k0 + kChunk < k_end) {
            stage_tile<A_KMAJOR>(as[buf ^ 1], q.a, q.lda, i0, k0 + kChunk, q.I, k_end);
            stage_tile<B_KMAJOR>(bs[buf ^ 1], q.b, q.ldb, j0, k0 + kChunk, q.J, k_end);
        }
#pragma unroll
        for (int kk = 0; kk < kChunk; kk += 2) {
            // v_mfma_f32_32x32x2_f32: lane l feeds A[i = l%32][k = l/32] and B[k = l/32][j = l%32]
            const float a0 = as[buf][kk + lk][wi + l32], a1 = as[buf][kk + lk][wi + 32 + l32];
            const float b0 = bs[buf][kk + lk][wj + l32], b1 = bs[buf][kk + lk][wj + 32 + l32];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
        __syncthreads();
        buf ^= 1;
    }

    // accumulator register r of lane l holds C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 tile
    float* c = q.c + (long long)blockIdx.z * q.c_split_stride;
#pragma unroll
    for (int x = 0; x < 2; x++)
#pragma unroll
        for (int y = 0; y < 2; y++) {
            const int j = j0 + wj + y * 32 + l32;
            if (j >= q.J) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int i = i0 + wi + x * 32 + 8 * (r >> 2) + 4 * lk + (r & 3);
                if (i >= q.I) continue;
                float v = acc[x][y][r];
                if (EPI == EPI_EXP_TIMES_G) {
                    const int n = i / q.npos, pos = i - n * q.npos;
                    const int co = j >= q.c_out ? j - q.c_out : j;
                    v = q.g[((long long)n * q.c_out + co) * q.npos + pos] * expf(-v);
                }
                c[(long long)i * q.ldc + j] = v;
            }
        }
}

// col[m][k] = x~[n, ci, a+u, b+v] for kernel row v; m = (n, a, b), k = ci*W + u; x~ is the
// zero-padded activation, read straight from the unpadded tensor.
__global__ __launch_bounds__(256) void k_im2col_row(const float* __restrict__ x, float* __restrict__ col, int v,
                                                    long long total, int c_in, int w_in, int h_in, int pad_w,
                                                    int pad_h, int w_k, int wo, int ho)
{
    const int k_or = c_in * w_k;
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
        const int k = (int)(e % k_or);
        const long long m = e / k_or;
        const int b = (int)(m % ho);
        const long long t = m / ho;
        const int a = (int)(t % wo);
        const long long n = t / wo;
        const int ci = k / w_k, u = k - ci * w_k;
        const int p = a + u - pad_w, qq = b + v - pad_h;
        float val = 0.0f;
        if (p >= 0 && p < w_in && qq >= 0 && qq < h_in) val = x[((n * c_in + ci) * w_in + p) * h_in + qq];
        col[e] = val;
    }
}

// Weight operands of kernel row v:
//   wcat[k][j]: j < c_out -> clamp(w,0,100), j >= c_out -> -clamp(w,-100,0)   (utils_functional.py:611-612)
//   wd[j][k]  : the same with the negative rail negated (it enters dL/dx with a minus sign)
__global__ __launch_bounds__(256) void k_weight_operands(const float* __restrict__ w, float* __restrict__ wcat,
                                                         float* __restrict__ wd, int v, int c_out, int c_in, int w_k,
                                                         int h_k)
{
    const int k_or = c_in * w_k;
    const int total = k_or * c_out;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        const int co = e % c_out, k = e / c_out;
        const float wv = w[((long long)co * k_or + k) * h_k + v];
        const float wp = fminf(fmaxf(wv, 0.0f), 100.0f);
        const float wn = -fminf(fmaxf(wv, -100.0f), 0.0f);
        wcat[(long long)k * 2 * c_out + co] = wp;
        wcat[(long long)k * 2 * c_out + c_out + co] = wn;
        wd[(long long)co * k_or + k] = wp;
        wd[(long long)(c_out + co) * k_or + k] = -wn;
    }
}

// dL/dw[co][ci][u][v] from the split partial sums part[s][k][j] (fixed summation order).
__global__ __launch_bounds__(256) void k_reduce_wgrad(const float* __restrict__ part, const float* __restrict__ w,
                                                      float* __restrict__ gw, int v, int splits, int c_out, int k_or,
                                                      int h_k)
{
    const int total = k_or * c_out;
    const long long stride = (long long)k_or * 2 * c_out;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        const int co = e % c_out, k = e / c_out;
        float sp = 0.0f, sn = 0.0f;
        for (int s = 0; s < splits; s++) {
            sp += part[s * stride + (long long)k * 2 * c_out + co];
            sn += part[s * stride + (long long)k * 2 * c_out + c_out + co];
        }
        const long long wi = ((long long)co * k_or + k) * h_k + v;
        const float wv = w[wi];
        float r = 0.0f;
        if (wv >= 0.0f && wv <= 100.0f) r += sp;
        if (wv >= -100.0f && wv <= 0.0f) r += sn;
        gw[wi] = r;
    }
}

// dL/dx[n][ci][p][q] (+)= sum_u dcol[ci*W+u][(n, p+pad_w-u, q+pad_h-v)] over the valid output
// positions; the first kernel row writes, the others add.
__global__ __launch_bounds__(256) void k_col2im_row(const float* __restrict__ dcol, float* __restrict__ gx, int v,
                                                    long long total, long long m_total, int c_in, int w_in,
                                                    int h_in, int pad_w, int pad_h, int w_k, int wo, int ho)
{
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
        const int qq = (int)(e % h_in);
        long long t = e / h_in;
        const int p = (int)(t % w_in);
        t /= w_in;
        const int ci = (int)(t % c_in);
        const long long n = t / c_in;
        const int b = qq + pad_h - v;
        float s = 0.0f;
        if (b >= 0 && b < ho) {
            for (int u = 0; u < w_k; u++) {
                const int a = p + pad_w - u;
                if (a >= 0 && a < wo) s += dcol[(long long)(ci * w_k + u) * m_total + (n * wo + a) * ho + b];
            }
        }
        gx[e] = v == 0 ? s : gx[e] + s;
    }
}

int grid1d(long long total)
{
    long long blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    return (int)(blocks < 1 ? 1 : blocks);
}

template <bool AK, bool BK, int EPI>
int launch_gemm(const GemmParams& q, int splits, hipStream_t s)
{
    dim3 grid((q.I + kTile - 1) / kTile, (q.J + kTile - 1) / kTile, splits);
    hipLaunchKernelGGL((k_gemm_f32<AK, BK, EPI>), grid, dim3(256), 0, s, q);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct BwdLayout {
    long long m_total;
    int splits, m_per_split;
    size_t off_col, off_e, off_dcol, off_part, off_wcat, off_wd, bytes;
};

BwdLayout bwd_layout(const Geometry& g)
{
    BwdLayout b;
    b.m_total = (long long)g.n * g.wo * g.ho;
    // split the m-reduction of the weight gradient so that the grid covers the GPU
    const long long tiles = (long long)((g.k_or + kTile - 1) / kTile) * ((2 * g.c_out + kTile - 1) / kTile);
    long long want = (1024 + tiles - 1) / tiles;
    long long per = (b.m_total + want - 1) / want;
    per = (per + kChunk - 1) / kChunk * kChunk;
    if (per < 256) per = 256;
    b.m_per_split = (int)(per > 0x7fffffffLL ? 0x7fffffffLL : per);
    b.splits = (int)((b.m_total + b.m_per_split - 1) / b.m_per_split);
    size_t o = 0;
    b.off_col = o;  o += align256(sizeof(float) * (size_t)b.m_total * g.k_or);
    b.off_e = o;    o += align256(sizeof(float) * (size_t)b.m_total * 2 * g.c_out);
    b.off_dcol = o; o += align256(sizeof(float) * (size_t)b.m_total * g.k_or);
    b.off_part = o; o += align256(sizeof(float) * (size_t)b.splits * g.k_or * 2 * g.c_out);
    b.off_wcat = o; o += align256(sizeof(float) * (size_t)g.k_or * 2 * g.c_out);
    b.off_wd = o;   o += align256(sizeof(float) * (size_t)g.k_or * 2 * g.c_out);
    b.bytes = o;
    return b;
}

}  // namespace

size_t backward_workspace_bytes(const Geometry& g) { return bwd_layout(g).bytes; }

int launch_conv_backward(const Geometry& g, const float* x, const float* w, const float* gy, float* gx, float* gw,
                         void* workspace, hipStream_t s)
{
    const BwdLayout L = bwd_layout(g);
    if (L.m_total > 0x7fffffffLL) return GEO_SC_ERR_INVALID_ARGUMENT;
    char* ws = (char*)workspace;
    float* col = (float*)(ws + L.off_col);
    float* e = (float*)(ws + L.off_e);
    float* dcol = (float*)(ws + L.off_dcol);
    float* part = (float*)(ws + L.off_part);
    float* wcat = (float*)(ws + L.off_wcat);
    float* wd = (float*)(ws + L.off_wd);
    const int M = (int)L.m_total, K = g.k_or, J = 2 * g.c_out;
    const long long col_total = L.m_total * K;
    const long long x_total = (long long)g.n * g.c_in * g.w_in * g.h_in;
    int rc;
    for (int v = 0; v < g.h_k; v++) {
        hipLaunchKernelGGL(k_im2col_row, dim3(grid1d(col_total)), dim3(256), 0, s, x, col, v, col_total, g.c_in,
                           g.w_in, g.h_in, g.pad_w, g.pad_h, g.w_k, g.wo, g.ho);
        hipLaunchKernelGGL(k_weight_operands, dim3(grid1d((long long)K * g.c_out)), dim3(256), 0, s, w, wcat, wd, v,
                           g.c_out, g.c_in, g.w_k, g.h_k);
        // E[m][j] = g * exp(-(col . wcat))
        GemmParams q1 = {};
        q1.a = col; q1.b = wcat; q1.c = e;
        q1.I = M; q1.J = J; q1.K = K;
        q1.lda = K; q1.ldb = J; q1.ldc = J;
        q1.k_per_split = K; q1.c_split_stride = 0;
        q1.g = gy; q1.c_out = g.c_out; q1.npos = g.wo * g.ho;
        if ((rc = launch_gemm<false, true, EPI_EXP_TIMES_G>(q1, 1, s)) != GEO_SC_OK) return rc;
        // partial Gw[s][k][j] = sum_{m in split s} col[m][k] * E[m][j]
        GemmParams q2 = {};
        q2.a = col; q2.b = e; q2.c = part;
        q2.I = K; q2.J = J; q2.K = M;
        q2.lda = K; q2.ldb = J; q2.ldc = J;
        q2.k_per_split = L.m_per_split; q2.c_split_stride = (long long)K * J;
        if (gw) {
            if ((rc = launch_gemm<true, true, EPI_STORE>(q2, L.splits, s)) != GEO_SC_OK) return rc;
            hipLaunchKernelGGL(k_reduce_wgrad, dim3(grid1d((long long)K * g.c_out)), dim3(256), 0, s, part, w, gw,
                               v, L.splits, g.c_out, K, g.h_k);
        }
        if (!gx) continue;
        // dcol[k][m] = sum_j wd[j][k] * E[m][j]
        GemmParams q3 = {};
        q3.a = wd; q3.b = e; q3.c = dcol;
        q3.I = K; q3.J = M; q3.K = J;
        q3.lda = K; q3.ldb = J; q3.ldc = M;
        q3.k_per_split = J; q3.c_split_stride = 0;
        if ((rc = launch_gemm<true, false, EPI_STORE>(q3, 1, s)) != GEO_SC_OK) return rc;
        hipLaunchKernelGGL(k_col2im_row, dim3(grid1d(x_total)), dim3(256), 0, s, dcol, gx, v, x_total, L.m_total,
                           g.c_in, g.w_in, g.h_in, g.pad_w, g.pad_h, g.w_k, g.wo, g.ho);
    }
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

}  // namespace geo_sc
