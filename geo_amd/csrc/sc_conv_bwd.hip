// Surrogate-gradient backward of the SC convolution (gfx950, fp32 results, MFMA).
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
// All three run on MFMA kernels (fp32 in, fp32 accumulate, fp32 out) that take each operand either
// K-major or I-major: k_gemm_split forms every fp32 product from six bf16 MFMA products of a three-way
// split of the operands (aligned operands; k_gemm_big is the same product with eight waves on tiles of
// up to 256 x 256 for the large results), k_gemm_f32 uses v_mfma_f32_32x32x2_f32 (any alignment);
// exp and the product with g are fused into the first GEMM's epilogue; the second is split over m
// and reduced deterministically.
//
// The other accumulation modes have the same surrogate with other add groups
// (utils_functional.py:254-299): one exponential per add group, whose argument sums the OR
// members of the group.  "Kernel row" above generalises to a group g with members k:
//     Y : g = v,                      k = ci*w_k + u                       (conv2d_or_bin_1d)
//     Z : g = ci,                     k = u*h_k + v                        (conv2d_or_bin_z)
//     YZ: g = (ci / z_unit)*h_k + v,  k = (ci % z_unit)*w_k + u            (conv2d_or_bin_yz)
//     FULL: g = 0,                    k = (ci*w_k + u)*h_k + v             (conv2d_or_approx, :189-210)
// Members of a ragged last channel block that do not exist carry zero weights.
#include "sc_common.h"

#include <cstdint>
#include <cstdlib>

#include <algorithm>
#include <type_traits>

namespace geo_sc {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// exp(-z) of the surrogate's OR term, z >= 0: one multiply and v_exp_f32 (about 1 ulp of the result plus
// |z| 2^-24 from the rounded argument), far inside the gradients' 1e-5; the library expf costs five
// times the instructions and the fused kernels evaluate it once per (position, group, channel, rail)
__device__ __forceinline__ float exp_neg(float z) { return __expf(-z); }

constexpr int kTile = 128;   // block tile in I and J
constexpr int kChunk = 16;   // K per LDS stage
constexpr int kLd = 132;     // LDS row stride in floats: rows stay 16-byte aligned for float4 stores

enum Epilogue { EPI_STORE = 0, EPI_EXP_TIMES_G = 1, EPI_EXP_TIMES_G_PLANES = 2, EPI_STORE_ITEMS = 3 };

struct GemmParams {
    const float* __restrict__ a;
    const float* __restrict__ b;
    float* __restrict__ c;
    int I, J, K;              // C[I][J] = sum_k A(k,i) * B(k,j)
    long long lda, ldb, ldc;  // leading dimensions (elements)
    // z = batch * splits + split.  A batch member is one kernel row: its operands
    // and result start batch_stride elements further; a split takes k_per_split of K and
    // writes its own partial result c_split_stride further.
    int splits;
    int k_per_split;
    long long c_split_stride;
    long long a_batch_stride, b_batch_stride, c_batch_stride;
    // EPI_EXP_TIMES_G: c[i][j] = g[i * c_out + (j % c_out)] * exp(-acc), g = upstream gradient stored [m][c_out]
    // EPI_EXP_TIMES_G_PLANES (g_planes set; whole tiles only): the same from the gradient as the caller
    // has it, [n][c_out][npos] with i = n * npos + position; npos a multiple of 32, g 16-byte aligned
    const float* __restrict__ g;
    int c_out, npos, g_planes;
    // A as a view of the shifted input planes instead of a materialised col (kernels with VA): row r of
    // batch member z starts a_rows[z * a_rows_batch + r] elements into `a`, and position m of that row lies
    // m + (m / a_item) * a_skip elements further (a_item positions per item, a_skip elements between the
    // items' runs); lda and a_batch_stride are not used.
    const long long* __restrict__ a_rows;
    long long a_rows_batch;
    int a_item, a_skip;
    // B as a view of E shifted by image rows and columns (kernels with VB; the input-gradient product summed
    // over all sh_wk x sh_hk kernel taps (u, v) inside the GEMM): chunk c of the k dimension holds the columns
    // j = (c / (sh_wk sh_hk)) * kChunk ... of tap t = c % (sh_wk sh_hk), u = t % sh_wk, v = t / sh_wk, and column
    // i = (n, p, c) of B (an element of the input: sh_win rows of sh_hin) is row (n, p + sh_pad - u, c + sh_padh - v)
    // of E_v (sh_j floats per row, ldb apart; E_v starts v * b_batch_stride into b) where that output position
    // exists, zero elsewhere (read from sh_zero).
    const float* __restrict__ sh_zero;
    int sh_j, sh_wo, sh_ho, sh_win, sh_hin, sh_pad, sh_padh, sh_wk, sh_hk;
    // EPI_STORE_ITEMS: column j = (n, rest) of the result goes to c[(n * I + i) * c_plane + rest] (c_plane
    // columns per item): the input gradient in the caller's layout (n, c_in, w_in, h_in)
    int c_plane;
    // tile extent per workgroup in i and j: kTile, or kTile / 2 in at most one of them (set by
    // launch_gemm): the four waves then line up along the other dimension
    int tile_i, tile_j;
    // Workgroup numbering (set by launch_gemm).  The grid is one-dimensional and the hardware deals
    // consecutive workgroup ids to the 8 XCDs in turn, each with an L2 of its own.  Workgroups that read
    // the same operand tiles form a cluster of `cluster` members (the tiles along the short dimension of
    // the result, or all tiles of one split of a small result); cluster q runs on XCD q % 8 with its members
    // next to each other, so a tile comes from memory once instead of once per member.
    int ni, nj, nz;  // tiles in i and j, batch * splits
    int cluster;     // members per cluster
    int cluster_of;  // 0: members = j tiles of one i tile, 1: i tiles of one j tile, 2: all tiles of one z
};

// The tile (it, jt, z) of workgroup w under the numbering above.
__device__ __forceinline__ void gemm_tile_of(const GemmParams& q, int w, int& it, int& jt, int& z)
{
    const int c = q.cluster;
    const int n_clusters = q.cluster_of == 2 ? q.nz : q.cluster_of == 0 ? q.nz * q.ni : q.nz * q.nj;
    const int whole = (n_clusters / 8) * 8 * c;  // workgroups of the clusters that fill all 8 XCDs evenly
    int cl, member;
    if (w < whole) {
        const int xcd = w & 7, r = w >> 3;
        member = r % c;
        cl = (r / c) * 8 + xcd;
    } else {
        const int r = w - whole;
        member = r % c;
        cl = (n_clusters / 8) * 8 + r / c;
    }
    if (q.cluster_of == 2) {
        z = cl;
        it = member % q.ni;
        jt = member / q.ni;
    } else if (q.cluster_of == 0) {
        z = cl / q.ni;
        it = cl - z * q.ni;
        jt = member;
    } else {
        z = cl / q.nj;
        jt = cl - z * q.nj;
        it = member;
    }
}

// Staging of one kChunk x kTile operand tile for the fp32 kernel, split in two so that the global
// loads of chunk c+1 are in flight while the MFMAs of chunk c run: fetch() reads 8 elements per
// thread into registers, commit() writes them to LDS as s[k][i].
//   K-major operand: element (k, i) at p[k*ld + i]
//   I-major operand: element (k, i) at p[i*ld + k]
// Guarded scalar loads for operands of any alignment and extent (lanes outside the operand read a valid
// dummy address and are zeroed by a select, no divergent branches); aligned operands take k_gemm_split.
template <bool KMAJOR>
struct Stager {
    const float* p;      // this thread's first element of the current chunk
    const float* dummy;  // any valid address of the operand
    long long ld;
    int kk0, ii;         // first k (inside the chunk) and first i (inside the tile) of this thread
    bool i_ok;
    unsigned ok;         // bit c: element c of the last fetch lies inside the operand

    // element c (0..7) of this thread sits at (k, i) = (kk0 + kdelta(c), ii)
    static __device__ __forceinline__ int kdelta(int c) { return KMAJOR ? c * 2 : c; }

    __device__ __forceinline__ void init(const float* base, long long ld_, int i0, int k_begin, int I)
    {
        const int t = threadIdx.x;
        ld = ld_;
        dummy = base;
        if (KMAJOR) {
            kk0 = t >> 7;  // rows kk0, kk0 + 2, ..., kk0 + 14, one i
            ii = t & 127;
            p = base + (long long)(k_begin + kk0) * ld + i0 + ii;
        } else {
            ii = t >> 1;
            kk0 = (t & 1) * 8;  // eight consecutive k of one i
            p = base + (long long)(i0 + ii) * ld + k_begin + kk0;
        }
        i_ok = i0 + ii < I;
    }
    // k_left = k_end - k0 of the chunk being fetched.  Only the loads are issued here; lanes outside
    // the operand are zeroed in commit(), after the MFMAs of the chunk in flight, so that nothing
    // waits for the loads before those MFMAs.
    __device__ __forceinline__ void fetch(float (&r)[8], int k_left)
    {
        ok = 0;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const bool okc = i_ok && kk0 + kdelta(c) < k_left;
            const float* qq = okc ? p + (KMAJOR ? (long long)kdelta(c) * ld : (long long)c) : dummy;
            r[c] = *qq;
            ok |= okc ? 1u << c : 0u;
        }
        p += KMAJOR ? (long long)kChunk * ld : (long long)kChunk;
    }
    __device__ __forceinline__ void commit(float (*s)[kLd], float (&r)[8]) const
    {
#pragma unroll
        for (int c = 0; c < 8; c++) s[kk0 + kdelta(c)][ii] = (ok >> c & 1u) ? r[c] : 0.0f;
    }
};

// Epilogue of one wave: accumulator register r of lane l holds C[8*(r/4) + 4*(l/32) + r%4][l%32] of a
// 32 x 32 block; (iw, jw) is the wave's corner in the result.  No branches around the loads of the
// upstream gradient: they go out 16 at a time from clamped addresses, then the exponentials, then
// stores under the range conditions (a load inside a per-element branch is waited for element by
// element: 64 memory latencies in a row).
template <int EPI, int NX, int NY, int MAXB = 2, bool WHOLE = false>
__device__ __forceinline__ void store_tile(const GemmParams& q, const floatx16 (&acc)[NX ? NX : 1][NY ? NY : 1],
                                           float* __restrict__ out, int iw, int jw, int l32, int lk)
{
    // blocks in batches of up to MAXB: the gradient loads of a whole batch are in flight together.
    // WHOLE: the wave's blocks lie inside the result, no range conditions.
    constexpr int NB = NX * NY, NYd = NY ? NY : 1;
    constexpr int BB = (MAXB >= 4 && NB % 4 == 0) ? 4 : (MAXB >= 3 && NB % 3 == 0) ? 3 : (MAXB >= 2 && NB % 2 == 0) ? 2 : 1;
#pragma unroll
    for (int b0 = 0; b0 < NB; b0 += BB) {
        float gv[BB][16];
        if (EPI == EPI_EXP_TIMES_G_PLANES) {
            // a lane's 16 rows are four runs of four consecutive positions of one item: four 16-byte loads from
            // the plane of its channel (the 32 rows of a block lie in one item)
#pragma unroll
            for (int bb = 0; bb < BB; bb++) {
                const int x = (b0 + bb) / NYd, y = (b0 + bb) % NYd;
                const int j = jw + y * 32 + l32, ib = iw + x * 32 + 4 * lk;
                const int co = j >= q.c_out ? j - q.c_out : j;
                const int item = ib / q.npos;
                const float* gp = q.g + ((long long)item * q.c_out + co) * q.npos + (ib - item * q.npos);
#pragma unroll
                for (int rg = 0; rg < 4; rg++) {
                    const float4 v = *(const float4*)(gp + 8 * rg);
                    gv[bb][4 * rg] = v.x; gv[bb][4 * rg + 1] = v.y; gv[bb][4 * rg + 2] = v.z; gv[bb][4 * rg + 3] = v.w;
                }
            }
        }
        if (EPI == EPI_EXP_TIMES_G) {
#pragma unroll
            for (int bb = 0; bb < BB; bb++) {
                const int x = (b0 + bb) / NYd, y = (b0 + bb) % NYd;
                const int j = jw + y * 32 + l32, ib = iw + x * 32 + 4 * lk;
                const int jc = (WHOLE || j < q.J) ? j : q.J - 1;
                const int co = jc >= q.c_out ? jc - q.c_out : jc;
                const float* gp = q.g + (long long)ib * q.c_out + co;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int di = 8 * (r >> 2) + (r & 3);
                    gv[bb][r] = WHOLE ? gp[di * q.c_out] : q.g[(long long)min(ib + di, q.I - 1) * q.c_out + co];
                }
            }
        }
#pragma unroll
        for (int bb = 0; bb < BB; bb++) {
            const int x = (b0 + bb) / NYd, y = (b0 + bb) % NYd;
            const int j = jw + y * 32 + l32, ib = iw + x * 32 + 4 * lk;
            const bool j_ok = WHOLE || j < q.J;
            if constexpr (EPI == EPI_STORE_ITEMS) {
                // the lane's column is one element of one item: rows are c_plane apart
                const int jc = j_ok ? j : 0;
                const int item = jc / q.c_plane;
                float* op = out + ((long long)item * q.I + ib) * q.c_plane + (jc - item * q.c_plane);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int di = 8 * (r >> 2) + (r & 3);
                    if (WHOLE || (j_ok && ib + di < q.I)) op[(long long)di * q.c_plane] = acc[x][y][r];
                }
                continue;
            }
            float* op = out + (long long)ib * q.ldc + j;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int di = 8 * (r >> 2) + (r & 3);
                const float v = (EPI == EPI_EXP_TIMES_G || EPI == EPI_EXP_TIMES_G_PLANES) ? gv[bb][r] * exp_neg(acc[x][y][r])
                                                                                        : acc[x][y][r];
                if (WHOLE)
                    op[(long long)di * q.ldc] = v;
                else if (j_ok && ib + di < q.I)
                    out[(long long)(ib + di) * q.ldc + j] = v;
            }
        }
    }
}

// The K loop and the epilogue of one wave that owns the first NX x NY of its 2 x 2 blocks of
// 32 x 32 (edge tiles and narrow operands leave blocks without results; NX = 0: none, the wave only
// stages).  A function of its own per (NX, NY), entered through a wave-uniform switch: the
// accumulators then live in one variant from zeroing to store and every MFMA is unconditional.
// Conditions on single blocks inside one loop make the compiler copy all accumulators between
// register classes on every trip.
// v_mfma_f32_32x32x2_f32: lane l feeds A[i = l%32][k = l/32] and B[k = l/32][j = l%32].
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, int NX, int NY>
__device__ __forceinline__ void gemm_wave(const GemmParams& q, float (*as)[kChunk][kLd], float (*bs)[kChunk][kLd], int i0,
                                          int j0, int batch, int split, int k_begin, int k_end, int wi, int wj, int l32,
                                          int lk)
{
    floatx16 acc[NX ? NX : 1][NY ? NY : 1];
#pragma unroll
    for (int x = 0; x < NX; x++)
#pragma unroll
        for (int y = 0; y < NY; y++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[x][y][r] = 0.0f;

    Stager<A_KMAJOR> sa;
    Stager<B_KMAJOR> sb;
    sa.init(q.a + batch * q.a_batch_stride, q.lda, i0, k_begin, min(q.I, i0 + q.tile_i));
    sb.init(q.b + batch * q.b_batch_stride, q.ldb, j0, k_begin, min(q.J, j0 + q.tile_j));
    float ra[8], rb[8];
    if (k_begin < k_end) {
        sa.fetch(ra, k_end - k_begin);
        sb.fetch(rb, k_end - k_begin);
        sa.commit(as[0], ra);
        sb.commit(bs[0], rb);
    }
    __syncthreads();
    int buf = 0;
    for (int k0 = k_begin; k0 < k_end; k0 += kChunk) {
        const bool more = k0 + kChunk < k_end;
        if (more) {
            sa.fetch(ra, k_end - k0 - kChunk);
            sb.fetch(rb, k_end - k0 - kChunk);
        }
#pragma unroll
        for (int kk = 0; kk < kChunk; kk += 2) {
            float a[NX ? NX : 1], b[NY ? NY : 1];
#pragma unroll
            for (int x = 0; x < NX; x++) a[x] = as[buf][kk + lk][wi + 32 * x + l32];
#pragma unroll
            for (int y = 0; y < NY; y++) b[y] = bs[buf][kk + lk][wj + 32 * y + l32];
#pragma unroll
            for (int x = 0; x < NX; x++)
#pragma unroll
                for (int y = 0; y < NY; y++)
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[x], b[y], acc[x][y], 0, 0, 0);
        }
        if (more) {
            // the other buffer was last read one trip ago, before that trip's barrier
            sa.commit(as[buf ^ 1], ra);
            sb.commit(bs[buf ^ 1], rb);
        }
        __syncthreads();
        buf ^= 1;
    }

    store_tile<EPI, NX, NY>(q, acc, q.c + batch * q.c_batch_stride + split * q.c_split_stride, i0 + wi, j0 + wj, l32, lk);
}

template <bool A_KMAJOR, bool B_KMAJOR, int EPI>
// four waves per SIMD (at most 128 registers: four workgroups per CU)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_gemm_f32(GemmParams q)
{
    __shared__ __attribute__((aligned(16))) float as[2][kChunk][kLd];
    __shared__ __attribute__((aligned(16))) float bs[2][kChunk][kLd];
    int it, jt, z;
    gemm_tile_of(q, blockIdx.x, it, jt, z);
    const int i0 = it * q.tile_i, j0 = jt * q.tile_j;
    const int batch = z / q.splits, split = z - batch * q.splits;
    const int k_begin = split * q.k_per_split;
    const int k_end = min(q.K, k_begin + q.k_per_split);
    // the wave index through readfirstlane: the compiler then knows that everything derived from it
    // (tile corner, block choice) is uniform and branches on it with scalar instructions
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    // this wave's corner in the tile: 2 x 2 waves of 64 x 64; with a tile of 64 in one dimension
    // (results that are narrow there) the four waves line up along the other, 32 x 64 (or 64 x 32) each
    const bool narrow_j = q.tile_j < kTile, narrow_i = q.tile_i < kTile;
    const int wi = narrow_j ? wave * 32 : narrow_i ? 0 : (wave >> 1) * 64;
    const int wj = narrow_j ? 0 : narrow_i ? wave * 32 : (wave & 1) * 64;
    const int l32 = lane & 31, lk = lane >> 5;
    // which of this wave's (up to) four 32 x 32 blocks lie inside the result
    const bool x0 = i0 + wi < q.I, x1 = !narrow_j && i0 + wi + 32 < q.I;
    const bool y0 = j0 + wj < q.J, y1 = !narrow_i && j0 + wj + 32 < q.J;
    const int blocks_xy = (x0 && y0) ? 2 * (int)x1 + (int)y1 : -1;
#define GEO_SC_GEMM_WAVE(NX, NY)                                                                                        \
    gemm_wave<A_KMAJOR, B_KMAJOR, EPI, NX, NY>(q, as, bs, i0, j0, batch, split, k_begin, k_end, wi, wj, l32, lk)
    // every variant runs the same staging and the same number of barriers
    switch (blocks_xy) {
    case 3: GEO_SC_GEMM_WAVE(2, 2); break;
    case 2: GEO_SC_GEMM_WAVE(2, 1); break;
    case 1: GEO_SC_GEMM_WAVE(1, 2); break;
    case 0: GEO_SC_GEMM_WAVE(1, 1); break;
    default: GEO_SC_GEMM_WAVE(0, 0); break;
    }
#undef GEO_SC_GEMM_WAVE
}

// ---- the same GEMM on the bf16 matrix cores, fp32 results ----
// Every fp32 operand element is split into three bf16 terms (x = hi + mid + lo to 2^-27 |x|: each
// term is the round-to-nearest bf16 of what the previous ones leave) and a product is formed from
// the six term products of relative size >= 2^-18 (hi hi, hi mid, mid hi, mid mid, hi lo, lo hi),
// each exact in fp32 and accumulated in fp32 by v_mfma_f32_32x32x16_bf16; the dropped ones
// (mid lo, lo mid, lo lo) are below 2^-26 of the product, less than the rounding of an fp32
// multiply.  Six bf16 MFMAs of 16 k take 6 x 8 passes where eight fp32 MFMAs of 2 k take
// 8 x 16.  The split happens once per element, when a staged chunk is written to LDS.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

constexpr int kLdx = 132;  // LDS stride between the two k halves of a chunk, in 16-byte slots

// bf16(a) in the low half, bf16(b) in the high half (v_cvt_pk_bf16_f32, round to nearest even)
__device__ __forceinline__ unsigned pack_bf16(float a, float b)
{
    const floatx2 v = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
}

__device__ __forceinline__ void split3(float a, float b, unsigned& hi, unsigned& mid, unsigned& lo)
{
    hi = pack_bf16(a, b);
    const float ra = a - __uint_as_float(hi << 16), rb = b - __uint_as_float(hi & 0xffff0000u);
    mid = pack_bf16(ra, rb);
    lo = pack_bf16(ra - __uint_as_float(mid << 16), rb - __uint_as_float(mid & 0xffff0000u));
}

// Staging for the split kernel: a thread owns eight consecutive k (one half of the chunk) of one i,
// which is what one lane feeds to the MFMA, and commit() writes them as s[term][k half][i], 16 bytes
// (four words of two bf16) per term.
//   K-major operand (element (k, i) at p[k*ld + i]): eight dword loads from a wave-uniform row pointer
//     each, lanes along i; the k half is the wave's (uniform)
//   I-major operand (element (k, i) at p[i*ld + k]): two float4 along k
// Rows i outside the operand are clamped to its last row: what they produce is never stored.  Only a
// partial last chunk is zeroed beyond its k range.
template <bool KMAJOR>
struct SplitStager {
    const float* p;   // K-major: row k_begin + 8 * half of the operand (uniform); I-major: this thread's first element
    long long ld;
    int off;          // K-major: this thread's i (clamped)
    int half, ii;

    // (ii_, half_): the row of the tile and the k half this thread stages (stage_slot)
    __device__ __forceinline__ void init(const float* base, long long ld_, int i0, int k_begin, int I, int ii_, int half_)
    {
        ld = ld_;
        ii = ii_;
        half = half_;
        if (KMAJOR) {
            off = min(i0 + ii, I - 1);
            p = base + (long long)(k_begin + 8 * half) * ld;
        } else {
            p = base + (long long)min(i0 + ii, I - 1) * ld + k_begin + 8 * half;
        }
    }
    // past a chunk that another thread stages
    __device__ __forceinline__ void skip_chunk() { p += KMAJOR ? (long long)kChunk * ld : (long long)kChunk; }
    // a whole chunk, no branches
    __device__ __forceinline__ void fetch_whole(float (&r)[8])
    {
        if (KMAJOR) {
#pragma unroll
            for (int c = 0; c < 8; c++) r[c] = (p + (long long)c * ld)[off];
            p += (long long)kChunk * ld;
        } else {
            const float4 v0 = *(const float4*)p, v1 = *(const float4*)(p + 4);
            r[0] = v0.x; r[1] = v0.y; r[2] = v0.z; r[3] = v0.w;
            r[4] = v1.x; r[5] = v1.y; r[6] = v1.z; r[7] = v1.w;
            p += kChunk;
        }
    }
    // k_left: what is left of the k range from this chunk's start (a partial last chunk has < kChunk)
    __device__ __forceinline__ void fetch(float (&r)[8], int k_left)
    {
        const bool tail = k_left < kChunk;
        if (KMAJOR) {
#pragma unroll
            for (int c = 0; c < 8; c++) {
                // rows past the end of a partial chunk read the chunk's first row instead
                const long long row = (tail && 8 * half + c >= k_left) ? -8 * half : c;
                r[c] = (p + row * ld)[off];
            }
            p += (long long)kChunk * ld;
        } else {
            if (!tail) {
                const float4 v0 = *(const float4*)p, v1 = *(const float4*)(p + 4);
                r[0] = v0.x; r[1] = v0.y; r[2] = v0.z; r[3] = v0.w;
                r[4] = v1.x; r[5] = v1.y; r[6] = v1.z; r[7] = v1.w;
            } else {
#pragma unroll
                for (int c = 0; c < 8; c++) r[c] = p[8 * half + c < k_left ? c : -8 * half];
            }
            p += kChunk;
        }
    }
    __device__ __forceinline__ void commit(uint4 (*s)[2][kLdx], float (&r)[8], int k_left) const
    {
        if (k_left < kChunk) {
#pragma unroll
            for (int c = 0; c < 8; c++) r[c] = 8 * half + c < k_left ? r[c] : 0.0f;
        }
        commit_whole(s, r);
    }
    __device__ __forceinline__ void commit_whole(uint4 (*s)[2][kLdx], const float (&r)[8]) const
    {
        unsigned hi[4], mid[4], lo[4];
#pragma unroll
        for (int c = 0; c < 4; c++) split3(r[2 * c], r[2 * c + 1], hi[c], mid[c], lo[c]);
        s[0][half][ii] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        s[1][half][ii] = make_uint4(mid[0], mid[1], mid[2], mid[3]);
        s[2][half][ii] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    }
};

// The same stager for an A operand that is a view of the shifted input planes (GemmParams::a_rows): the
// rows start where a table says, and the positions of one item are a_skip elements away from the next
// item's.  As the K-major operand of the first product the positions are the rows' elements (a lane keeps
// its own position, shifted once); as the I-major operand of the weight-gradient product they are the k
// dimension: a thread's eight positions and a whole chunk lie inside one item (a_item is a multiple of
// kChunk), and the pointer jumps by a_skip when it passes an item's end.
// AHEAD (K-major only): the table entries of a chunk are read when the chunk before it is fetched, so that a
// fetch issues its loads without waiting for the table first; the entries read for the chunk behind the last
// one (up to 2 * kChunk + 8 entries behind the member's part of the table) are never used.
template <bool KMAJOR, bool AHEAD = false>
struct ViewStager {
    const float* base;
    const long long* rows;  // K-major: the table of this batch member (uniform)
    const float* p;         // I-major: this thread's first element
    int off;                // K-major: this thread's element of every row
    int kr;                 // K-major: first row of this thread's half of the current chunk
    int in_item, item, skip;
    int half, ii;
    long long ahead[(KMAJOR && AHEAD) ? 8 : 1];  // the rows' starts of the chunk to fetch next

    __device__ __forceinline__ void read_ahead()
    {
        if constexpr (KMAJOR && AHEAD) {
#pragma unroll
            for (int c = 0; c < 8; c++) ahead[c] = rows[kr + c];
        }
    }

    __device__ __forceinline__ void init(const GemmParams& q, int batch, int i0, int k_begin, int I, int ii_, int half_)
    {
        base = q.a;
        rows = q.a_rows + batch * q.a_rows_batch;
        item = q.a_item;
        skip = q.a_skip;
        ii = ii_;
        half = half_;
        if (KMAJOR) {
            const int m = min(i0 + ii, I - 1);
            off = m + (m / item) * skip;
            kr = k_begin + 8 * half;
            read_ahead();
            if constexpr (AHEAD) {
                // wait for these entries here, where a tile is opened, and not where this path meets the one
                // of the later fetches: there the wait would also take in the data loads of the fetch before
#pragma unroll
                for (int c = 0; c < 8; c++) asm volatile("" ::"v"(ahead[c]));
            }
        } else {
            const int m = k_begin + 8 * half;
            in_item = m % item;
            p = base + rows[min(i0 + ii, I - 1)] + m + (long long)(m / item) * skip;
        }
    }
    __device__ __forceinline__ void advance()
    {
        if (KMAJOR) {
            kr += kChunk;
        } else {
            p += kChunk;
            in_item += kChunk;
            if (in_item >= item) {
                in_item -= item;
                p += skip;
            }
        }
    }
    __device__ __forceinline__ void skip_chunk()
    {
        advance();
        read_ahead();
    }
    __device__ __forceinline__ void fetch_whole(float (&r)[8])
    {
        if constexpr (KMAJOR && AHEAD) {
#pragma unroll
            for (int c = 0; c < 8; c++) r[c] = (base + ahead[c])[off];
            advance();
            read_ahead();
            return;
        }
        if (KMAJOR) {
#pragma unroll
            for (int c = 0; c < 8; c++) r[c] = (base + rows[kr + c])[off];
        } else {
            const float4 v0 = *(const float4*)p, v1 = *(const float4*)(p + 4);
            r[0] = v0.x; r[1] = v0.y; r[2] = v0.z; r[3] = v0.w;
            r[4] = v1.x; r[5] = v1.y; r[6] = v1.z; r[7] = v1.w;
        }
        advance();
    }
    __device__ __forceinline__ void fetch(float (&r)[8], int k_left)
    {
        const bool tail = k_left < kChunk;
        if (KMAJOR) {
#pragma unroll
            for (int c = 0; c < 8; c++) {
                // rows past the end of a partial chunk read the chunk's first row instead
                const int row = (tail && 8 * half + c >= k_left) ? kr - 8 * half : kr + c;
                r[c] = (base + rows[row])[off];
            }
        } else {
            if (!tail) {
                const float4 v0 = *(const float4*)p, v1 = *(const float4*)(p + 4);
                r[0] = v0.x; r[1] = v0.y; r[2] = v0.z; r[3] = v0.w;
                r[4] = v1.x; r[5] = v1.y; r[6] = v1.z; r[7] = v1.w;
            } else {
#pragma unroll
                for (int c = 0; c < 8; c++) r[c] = p[8 * half + c < k_left ? c : -8 * half];
            }
        }
        advance();
    }
    __device__ __forceinline__ void commit(uint4 (*s)[2][kLdx], float (&r)[8], int k_left) const
    {
        if (k_left < kChunk) {
#pragma unroll
            for (int c = 0; c < 8; c++) r[c] = 8 * half + c < k_left ? r[c] : 0.0f;
        }
        unsigned hi[4], mid[4], lo[4];
#pragma unroll
        for (int c = 0; c < 4; c++) split3(r[2 * c], r[2 * c + 1], hi[c], mid[c], lo[c]);
        s[0][half][ii] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        s[1][half][ii] = make_uint4(mid[0], mid[1], mid[2], mid[3]);
        s[2][half][ii] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    }
};

// Stager of the B operand of the input-gradient product when it sums over the kernel taps inside the GEMM
// (GemmParams::sh_*): the k dimension runs over chunks of kChunk columns j of E with the tap (u, v) as the fast
// index (u fastest), and for tap (u, v) the column (n, p, c) of B - an element of the input - is the row
// (n, p + pad_w - u, c + pad_h - v) of E_v.  I-major: a thread keeps one column and eight consecutive j; from
// chunk to chunk it moves one image row up, then one column left, and after the last tap on to the next columns
// j - so the rows of E that the taps share are read in consecutive chunks, while they are still in the CU's
// cache.  Columns whose output position does not exist for a tap read a block of zeros instead (no select on the
// loaded data, so nothing waits for the load).  sh_j is a multiple of kChunk: there are no partial chunks.
struct ShiftStager {
    const float* e0;       // E_0; E_v is group_stride floats further per v
    const float* zero;
    const float* p;
    long long ld, group_stride;
    int j, u, v, prow, pcol, wo, ho;  // j: this thread's first column of E in the current chunk; prow = p + pad_w, pcol = c + pad_h
    long long row0;                   // (n * wo + prow) * ho + pcol: the row of E for the tap (0, 0)
    int half, ii, n_u, n_v;

    __device__ __forceinline__ void point()
    {
        const int r = prow - u, c = pcol - v;
        p = (r >= 0 && r < wo && c >= 0 && c < ho)
                ? e0 + (long long)v * group_stride + (row0 - (long long)u * ho - v) * ld + j
                : zero;
    }
    __device__ __forceinline__ void init(const GemmParams& q, int batch, int j0, int k_begin, int Jn, int ii_, int half_)
    {
        ii = ii_;
        half = half_;
        n_u = q.sh_wk;
        n_v = q.sh_hk;
        // all taps in one product (E_v chosen by the tap), or one product per kernel column (batch member) over
        // its kernel rows (sh_hk = 1, sh_hin = ho, sh_padh = 0)
        e0 = q.b + (n_v == 1 ? (long long)batch * q.b_batch_stride : 0);
        group_stride = q.b_batch_stride;
        zero = q.sh_zero;
        ld = q.ldb;
        wo = q.sh_wo;
        ho = q.sh_ho;
        const int m = min(j0 + ii, Jn - 1);
        const int per_item = q.sh_win * q.sh_hin;
        const int n = m / per_item, rem = m - n * per_item;
        const int pr = rem / q.sh_hin, c = rem - pr * q.sh_hin;
        prow = pr + q.sh_pad;
        pcol = c + q.sh_padh;
        row0 = ((long long)n * wo + prow) * ho + pcol;
        // chunk c of the k dimension: tap c % (w_k h_k) of the columns (c / (w_k h_k)) * kChunk ...
        const int chunk = k_begin / kChunk, taps = n_u * n_v, t = chunk % taps;
        u = t % n_u;
        v = t / n_u;
        j = (chunk / taps) * kChunk + 8 * half;
        point();
    }
    __device__ __forceinline__ void advance()
    {
        if (++u == n_u) {
            u = 0;
            if (++v == n_v) {
                v = 0;
                j += kChunk;
            }
        }
        point();
    }
    __device__ __forceinline__ void fetch_whole(float (&r)[8])
    {
        const float4 v0 = *(const float4*)p, v1 = *(const float4*)(p + 4);
        r[0] = v0.x; r[1] = v0.y; r[2] = v0.z; r[3] = v0.w;
        r[4] = v1.x; r[5] = v1.y; r[6] = v1.z; r[7] = v1.w;
        advance();
    }
    __device__ __forceinline__ void fetch(float (&r)[8], int) { fetch_whole(r); }
    __device__ __forceinline__ void commit(uint4 (*s)[2][kLdx], float (&r)[8], int) const
    {
        unsigned hi[4], mid[4], lo[4];
#pragma unroll
        for (int c = 0; c < 4; c++) split3(r[2 * c], r[2 * c + 1], hi[c], mid[c], lo[c]);
        s[0][half][ii] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        s[1][half][ii] = make_uint4(mid[0], mid[1], mid[2], mid[3]);
        s[2][half][ii] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    }
};

// v_mfma_f32_32x32x16_bf16: lane l feeds A[i = l%32][k = 8 (l/32) .. + 7] and B[those k][j = l%32]:
// the 16 bytes at s[term][l/32][i]; results as in the fp32 instruction.
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, int NX, int NY, bool VA, bool VB>
__device__ __forceinline__ void gemm_wave_split(const GemmParams& q, uint4 (*as)[3][2][kLdx], uint4 (*bs)[3][2][kLdx],
                                                int i0, int j0, int batch, int split, int k_begin, int k_end, int wi,
                                                int wj, int l32, int lk, int wave)
{
    floatx16 acc[NX ? NX : 1][NY ? NY : 1];
#pragma unroll
    for (int x = 0; x < NX; x++)
#pragma unroll
        for (int y = 0; y < NY; y++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[x][y][r] = 0.0f;

    typename std::conditional<VA, ViewStager<A_KMAJOR>, SplitStager<A_KMAJOR>>::type sa;
    typename std::conditional<VB, ShiftStager, SplitStager<B_KMAJOR>>::type sb;
    // K-major operand: waves 0, 1 stage the first k half of the 128 rows, waves 2, 3 the second;
    // I-major operand: two threads per row, one k half each
    const int t = threadIdx.x;
    const int a_ii = A_KMAJOR ? (t & 127) : (t >> 1), a_half = A_KMAJOR ? (wave >> 1) : (t & 1);
    const int b_ii = (B_KMAJOR && !VB) ? (t & 127) : (t >> 1), b_half = (B_KMAJOR && !VB) ? (wave >> 1) : (t & 1);
    if constexpr (VA)
        sa.init(q, batch, i0, k_begin, min(q.I, i0 + q.tile_i), a_ii, a_half);
    else
        sa.init(q.a + batch * q.a_batch_stride, q.lda, i0, k_begin, min(q.I, i0 + q.tile_i), a_ii, a_half);
    if constexpr (VB)
        sb.init(q, batch, j0, k_begin, min(q.J, j0 + q.tile_j), b_ii, b_half);
    else
        sb.init(q.b + batch * q.b_batch_stride, q.ldb, j0, k_begin, min(q.J, j0 + q.tile_j), b_ii, b_half);
    // Two chunks ahead: while chunk c is multiplied out of LDS, chunk c + 1 sits in one register set
    // (its loads issued a whole trip ago) and the loads of chunk c + 2 go out into the other.
    float ra[2][8], rb[2][8];
    const int k_len = k_end - k_begin;
    const int n_chunks = k_len > 0 ? (k_len + kChunk - 1) / kChunk : 0;
    if (n_chunks > 0) {
        sa.fetch(ra[0], k_len);
        sb.fetch(rb[0], k_len);
    }
    if (n_chunks > 1) {
        sa.fetch(ra[1], k_len - kChunk);
        sb.fetch(rb[1], k_len - kChunk);
    }
    if (n_chunks > 0) {
        sa.commit(as[0], ra[0], k_len);
        sb.commit(bs[0], rb[0], k_len);
    }
    __syncthreads();
    auto multiply = [&](int buf) {
        bf16x8 a[NX ? NX : 1][3], b[NY ? NY : 1][3];
#pragma unroll
        for (int t = 0; t < 3; t++) {
#pragma unroll
            for (int x = 0; x < NX; x++) a[x][t] = __builtin_bit_cast(bf16x8, as[buf][t][lk][wi + 32 * x + l32]);
#pragma unroll
            for (int y = 0; y < NY; y++) b[y][t] = __builtin_bit_cast(bf16x8, bs[buf][t][lk][wj + 32 * y + l32]);
        }
        // smallest terms first; 0 = hi, 1 = mid, 2 = lo
        constexpr int ta[6] = {2, 0, 1, 1, 0, 0}, tb[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
        for (int t = 0; t < 6; t++)
#pragma unroll
            for (int x = 0; x < NX; x++)
#pragma unroll
                for (int y = 0; y < NY; y++)
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[x][ta[t]], b[y][tb[t]], acc[x][y], 0, 0, 0);
    };
    int c = 0;
    // Whole chunks, no branches in the trip.  The split of chunk c + 1 (vector ALU, 24 steps: three per
    // pair of elements) is written between the MFMAs of chunk c, one step per MFMA with four blocks, so
    // that it issues while the matrix pipe is busy.  (Scheduling barriers that spelled this order out held in
    // the first of the loop's two trips only: in the second the compiler chained the six MFMAs of each
    // block back to back.  Without them both trips keep the written order.)
    const int n_whole = k_len > 0 ? k_len / kChunk : 0;
    constexpr int kMfmas = NX * NY > 0 ? 6 * NX * NY : 1;  // per trip
    constexpr int kStepsPerMfma = (24 + kMfmas - 1) / kMfmas;
    auto multiply_and_split = [&](auto set) {
        constexpr int S = decltype(set)::value;
        sa.fetch_whole(ra[S]);
        sb.fetch_whole(rb[S]);
        bf16x8 a[NX ? NX : 1][3], b[NY ? NY : 1][3];
#pragma unroll
        for (int t = 0; t < 3; t++) {
#pragma unroll
            for (int x = 0; x < NX; x++) a[x][t] = __builtin_bit_cast(bf16x8, as[S][t][lk][wi + 32 * x + l32]);
#pragma unroll
            for (int y = 0; y < NY; y++) b[y][t] = __builtin_bit_cast(bf16x8, bs[S][t][lk][wj + 32 * y + l32]);
        }
        constexpr int ta[6] = {2, 0, 1, 1, 0, 0}, tb[6] = {0, 2, 1, 0, 1, 0};
        // pairs 0..3: this thread's elements of A, 4..7: of B
        unsigned hi[8], mid[8], lo[8];
        float r0[8], r1[8];
        auto step = [&](int n) {
            const int pr = n / 3, st = n % 3;
            const float* src = pr < 4 ? ra[S ^ 1] : rb[S ^ 1];
            const int e = 2 * (pr & 3);
            if (st == 0) {
                hi[pr] = pack_bf16(src[e], src[e + 1]);
                r0[pr] = src[e] - __uint_as_float(hi[pr] << 16);
                r1[pr] = src[e + 1] - __uint_as_float(hi[pr] & 0xffff0000u);
            } else if (st == 1) {
                mid[pr] = pack_bf16(r0[pr], r1[pr]);
                r0[pr] -= __uint_as_float(mid[pr] << 16);
                r1[pr] -= __uint_as_float(mid[pr] & 0xffff0000u);
            } else {
                lo[pr] = pack_bf16(r0[pr], r1[pr]);
            }
        };
#pragma unroll
        for (int m = 0; m < kMfmas; m++) {
            constexpr int kBlocks = NX * NY > 0 ? NX * NY : 1, kNy = NY > 0 ? NY : 1;
            const int t = m / kBlocks, x = (m % kBlocks) / kNy, y = m % kNy;
            acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[x][ta[t]], b[y][tb[t]], acc[x][y], 0, 0, 0);
#pragma unroll
            for (int n = m * kStepsPerMfma; n < (m + 1) * kStepsPerMfma && n < 24; n++) step(n);
        }
        as[S ^ 1][0][sa.half][sa.ii] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        as[S ^ 1][1][sa.half][sa.ii] = make_uint4(mid[0], mid[1], mid[2], mid[3]);
        as[S ^ 1][2][sa.half][sa.ii] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        bs[S ^ 1][0][sb.half][sb.ii] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
        bs[S ^ 1][1][sb.half][sb.ii] = make_uint4(mid[4], mid[5], mid[6], mid[7]);
        bs[S ^ 1][2][sb.half][sb.ii] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
        __syncthreads();
    };
    if (NX * NY > 0) {
        for (; c + 3 < n_whole; c += 2) {
            multiply_and_split(std::integral_constant<int, 0>());
            multiply_and_split(std::integral_constant<int, 1>());
        }
    }
    for (; c + 1 < n_chunks; c += 2) {
        // chunk c from LDS buffer 0; register set 1 holds chunk c + 1
        if (c + 2 < n_chunks) {
            sa.fetch(ra[0], k_len - (c + 2) * kChunk);
            sb.fetch(rb[0], k_len - (c + 2) * kChunk);
        }
        multiply(0);
        sa.commit(as[1], ra[1], k_len - (c + 1) * kChunk);
        sb.commit(bs[1], rb[1], k_len - (c + 1) * kChunk);
        __syncthreads();
        // chunk c + 1 from LDS buffer 1; register set 0 holds chunk c + 2
        if (c + 3 < n_chunks) {
            sa.fetch(ra[1], k_len - (c + 3) * kChunk);
            sb.fetch(rb[1], k_len - (c + 3) * kChunk);
        }
        multiply(1);
        if (c + 2 < n_chunks) {
            sa.commit(as[0], ra[0], k_len - (c + 2) * kChunk);
            sb.commit(bs[0], rb[0], k_len - (c + 2) * kChunk);
        }
        __syncthreads();
    }
    if (c < n_chunks) multiply(0);  // an odd last chunk, already in buffer 0

    store_tile<EPI, NX, NY>(q, acc, q.c + batch * q.c_batch_stride + split * q.c_split_stride, i0 + wi, j0 + wj, l32, lk);
}

// Operands with 16-byte aligned rows and chunks (launch_gemm checks).
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, bool VA = false, bool VB = false>
// three waves per SIMD (at most 168 registers; three workgroups' LDS fit a CU)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void k_gemm_split(GemmParams q)
{
    __shared__ uint4 as[2][3][2][kLdx];
    __shared__ uint4 bs[2][3][2][kLdx];
    int it, jt, z;
    gemm_tile_of(q, blockIdx.x, it, jt, z);
    const int i0 = it * q.tile_i, j0 = jt * q.tile_j;
    const int batch = z / q.splits, split = z - batch * q.splits;
    const int k_begin = split * q.k_per_split;
    const int k_end = min(q.K, k_begin + q.k_per_split);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const bool narrow_j = q.tile_j < kTile, narrow_i = q.tile_i < kTile;
    const int wi = narrow_j ? wave * 32 : narrow_i ? 0 : (wave >> 1) * 64;
    const int wj = narrow_j ? 0 : narrow_i ? wave * 32 : (wave & 1) * 64;
    const int l32 = lane & 31, lk = lane >> 5;
    const bool x0 = i0 + wi < q.I, x1 = !narrow_j && i0 + wi + 32 < q.I;
    const bool y0 = j0 + wj < q.J, y1 = !narrow_i && j0 + wj + 32 < q.J;
    const int blocks_xy = (x0 && y0) ? 2 * (int)x1 + (int)y1 : -1;
#define GEO_SC_GEMM_WAVE(NX, NY)                                                                                        \
    gemm_wave_split<A_KMAJOR, B_KMAJOR, EPI, NX, NY, VA, VB>(q, as, bs, i0, j0, batch, split, k_begin, k_end, wi, wj, l32, lk, wave)
    switch (blocks_xy) {
    case 3: GEO_SC_GEMM_WAVE(2, 2); break;
    case 2: GEO_SC_GEMM_WAVE(2, 1); break;
    case 1: GEO_SC_GEMM_WAVE(1, 2); break;
    case 0: GEO_SC_GEMM_WAVE(1, 1); break;
    default: GEO_SC_GEMM_WAVE(0, 0); break;
    }
#undef GEO_SC_GEMM_WAVE
}

// ---- the split kernel with eight waves per workgroup and a tile of 64 NX x 256 ----
// What the 128 x 128 kernel waits for is its operands: every tile streams 128 + 128 rows of fp32 per 128 x 128
// results through L2, and three workgroups per CU ask for more than the caches deliver.  Here one workgroup
// per CU (2 x 4 waves, 32 NX x 64 results each; 2 waves per SIMD with up to 256 registers) multiplies
// 64 NX x 256: per result a half (NX = 4) to three quarters (NX = 2) of the operand traffic.  A wave reads
// the fragments of one term product at a time (NX + 2 reads for 2 NX MFMAs), so that the second wave of the
// SIMD and the wave's own next reads fill the matrix pipe's shadow; the three-way split of the next chunk
// is written between the MFMAs as in the small kernel.
// With nobody else on the CU, a tile's first loads and its epilogue would run with the matrix pipe idle, so
// the workgroups are persistent: workgroup w takes the tiles w, w + gridDim.x, ... and treats their chunks
// as one stream - while the last chunks of a tile are multiplied, the first chunks of the next are already
// loaded, split and written to LDS, and the epilogue runs with those loads in flight.
// Whole tiles and whole, non-empty chunk ranges only (launch_gemm checks); the stagers and the epilogue
// are the small kernel's.
constexpr int kBigJ = 256;
constexpr int kBigWorkgroups = 256;  // one per CU of an MI355X
// rows of a tile for a result with I rows: 256, 192 or 128 (NX = 4, 3, 2); 0: I is no multiple of any
inline int big_rows(int I) { return I % 256 == 0 ? 256 : I % 192 == 0 ? 192 : I % 128 == 0 ? 128 : 0; }

// KC: chunks per trip.  With NX = 2 a trip of one chunk holds 24 MFMAs per wave, too few for what every trip
// costs besides (barrier, the latency of the first LDS reads, the loads' address arithmetic); two chunks per
// trip (KC = 2, 150 KB of LDS) halve that share.
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, bool VA, bool VB, int NX, int KC = 1>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_gemm_big(GemmParams q)
{
    constexpr int RA = 64 * NX, LA = RA + 4, LB = kBigJ + 4;
    constexpr int kUnit = KC * kChunk;  // k per trip
    __shared__ uint4 as[2][3][2 * KC][LA];
    __shared__ uint4 bs[2][3][2 * KC][LB];
    const int t = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(t >> 6), lane = t & 63;
    const int wi = (wave >> 2) * (32 * NX), wj = (wave & 3) * 64;
    const int l32 = lane & 31, lk = lane >> 5;
    // Staging slots.  A: 2 KC RA (row, eight k) pairs of a trip, one per thread (with fewer pairs than
    // threads the rest stage a pair a second time: same data to the same place); a K-major operand has
    // the lanes along the rows and the pair's k uniform in a wave, an I-major one neighbouring threads
    // along k.  B: 512 (row, k half) pairs per chunk, every thread one pair of each of the trip's chunks.
    static_assert(2 * KC * RA <= 512, "one pair of A per thread");
    constexpr bool BK = B_KMAJOR && !VB;
    const int wa = wave % (KC * RA / 32), ta = t % (2 * KC * RA);
    const int a_ii = A_KMAJOR ? (wa % NX) * 64 + lane : ta / (2 * KC);
    const int a_q = A_KMAJOR ? wa / NX : ta % (2 * KC);  // which eight k of the trip
    const int b_ii = BK ? (t & 255) : (t >> 1), b_half = BK ? (wave >> 2) : (t & 1);
    typename std::conditional<VA, ViewStager<A_KMAJOR, true>, SplitStager<A_KMAJOR>>::type sa;
    typename std::conditional<VB, ShiftStager, SplitStager<B_KMAJOR>>::type sb;

    const int n_tiles = q.ni * q.nj * q.nz;
    // the tile whose chunks are being loaded: the stagers point into it, left_f of its trips are still to load
    int w_f = blockIdx.x, left_f;
    auto open_tile = [&]() {
        int it, jt, z;
        gemm_tile_of(q, w_f, it, jt, z);
        const int batch = z / q.splits, split = z - batch * q.splits;
        const int k_begin = split * q.k_per_split;
        left_f = (min(q.K, k_begin + q.k_per_split) - k_begin) / kUnit;
        const int ka = k_begin + (a_q >> 1) * kChunk;  // A: this thread's chunk of every trip
        if constexpr (VA)
            sa.init(q, batch, it * RA, ka, q.I, a_ii, a_q & 1);
        else
            sa.init(q.a + batch * q.a_batch_stride, q.lda, it * RA, ka, q.I, a_ii, a_q & 1);
        if constexpr (VB)
            sb.init(q, batch, jt * kBigJ, k_begin, q.J, b_ii, b_half);
        else
            sb.init(q.b + batch * q.b_batch_stride, q.ldb, jt * kBigJ, k_begin, q.J, b_ii, b_half);
    };
    // The next trip's worth of the stream into a register set.  Once the last tile is through, the fetches go
    // round that tile again (loads of valid addresses that nobody uses): every path through here issues the
    // same loads, so the waits that the compiler places in front of the split count only the loads of the
    // set they need - with a path that issues none, they would wait for the newest loads as well.
    auto fetch_next = [&](float (&ra)[8], float (&rb)[KC][8]) {
        if (left_f == 0) {
            if (w_f + (int)gridDim.x < n_tiles) w_f += gridDim.x;
            open_tile();
        }
        sa.fetch_whole(ra);
#pragma unroll
        for (int kc = 1; kc < KC; kc++) sa.skip_chunk();
#pragma unroll
        for (int kc = 0; kc < KC; kc++) sb.fetch_whole(rb[kc]);
        --left_f;
    };
    // the tile being multiplied
    int w_m = blockIdx.x, left_m, i0_m, j0_m;
    float* out_m;
    auto describe_m = [&]() {
        int it, jt, z;
        gemm_tile_of(q, w_m, it, jt, z);
        const int batch = z / q.splits, split = z - batch * q.splits;
        const int k_begin = split * q.k_per_split;
        left_m = (min(q.K, k_begin + q.k_per_split) - k_begin) / kUnit;
        i0_m = it * RA;
        j0_m = jt * kBigJ;
        out_m = q.c + batch * q.c_batch_stride + split * q.c_split_stride;
    };

    floatx16 acc[NX][2];
    auto zero_acc = [&]() {
#pragma unroll
        for (int x = 0; x < NX; x++)
#pragma unroll
            for (int y = 0; y < 2; y++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[x][y][r] = 0.0f;
    };
    zero_acc();
    open_tile();
    describe_m();

    // Register set c % 2 holds trip c of the stream until it is split and written to LDS buffer c % 2, one
    // trip before it is multiplied; its loads go out two trips before that.
    constexpr int kPairs = 4 + 4 * KC;  // pairs of elements per thread and trip: A, then B chunk by chunk
    float ra[2][8], rb[2][KC][8];
    auto write_split = [&](int buf, const unsigned (&hi)[kPairs], const unsigned (&mid)[kPairs], const unsigned (&lo)[kPairs]) {
        as[buf][0][a_q][a_ii] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        as[buf][1][a_q][a_ii] = make_uint4(mid[0], mid[1], mid[2], mid[3]);
        as[buf][2][a_q][a_ii] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
#pragma unroll
        for (int kc = 0; kc < KC; kc++) {
            const int o = 4 + 4 * kc;
            bs[buf][0][2 * kc + b_half][b_ii] = make_uint4(hi[o], hi[o + 1], hi[o + 2], hi[o + 3]);
            bs[buf][1][2 * kc + b_half][b_ii] = make_uint4(mid[o], mid[o + 1], mid[o + 2], mid[o + 3]);
            bs[buf][2][2 * kc + b_half][b_ii] = make_uint4(lo[o], lo[o + 1], lo[o + 2], lo[o + 3]);
        }
    };
    fetch_next(ra[0], rb[0]);
    fetch_next(ra[1], rb[1]);
    {
        unsigned hi[kPairs], mid[kPairs], lo[kPairs];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            split3(ra[0][2 * c], ra[0][2 * c + 1], hi[c], mid[c], lo[c]);
#pragma unroll
            for (int kc = 0; kc < KC; kc++)
                split3(rb[0][kc][2 * c], rb[0][kc][2 * c + 1], hi[4 + 4 * kc + c], mid[4 + 4 * kc + c], lo[4 + 4 * kc + c]);
        }
        write_split(0, hi, mid, lo);
    }
    fetch_next(ra[0], rb[0]);
    __syncthreads();

    // One trip: trip c of the stream out of LDS buffer S, trip c + 1 (register set S ^ 1) split and written
    // to the other buffer, the loads of trip c + 3 into that register set.  Past the end of the stream the
    // split works on stale registers and its result is never read.
    auto trip = [&](auto set) {
        constexpr int S = decltype(set)::value, R = S ^ 1;
        constexpr int pa[6] = {2, 0, 1, 1, 0, 0}, pb[6] = {0, 2, 1, 0, 1, 0};  // smallest terms first; 0 = hi
        constexpr int kSteps = 3 * kPairs, kMfmas = 12 * NX * KC;
        unsigned hi[kPairs], mid[kPairs], lo[kPairs];
        float r0[kPairs], r1[kPairs];
        auto step = [&](int n) {
            const int pr = n / 3, st = n % 3;
            const float* src = pr < 4 ? ra[R] : rb[R][(pr - 4) >> 2];
            const int e = 2 * (pr & 3);
            if (st == 0) {
                hi[pr] = pack_bf16(src[e], src[e + 1]);
                r0[pr] = src[e] - __uint_as_float(hi[pr] << 16);
                r1[pr] = src[e + 1] - __uint_as_float(hi[pr] & 0xffff0000u);
            } else if (st == 1) {
                mid[pr] = pack_bf16(r0[pr], r1[pr]);
                r0[pr] -= __uint_as_float(mid[pr] << 16);
                r1[pr] -= __uint_as_float(mid[pr] & 0xffff0000u);
            } else {
                lo[pr] = pack_bf16(r0[pr], r1[pr]);
            }
        };
#pragma unroll
        for (int kc = 0; kc < KC; kc++)
#pragma unroll
            for (int p6 = 0; p6 < 6; p6++) {
                bf16x8 a[NX], b[2];
#pragma unroll
                for (int x = 0; x < NX; x++)
                    a[x] = __builtin_bit_cast(bf16x8, as[S][pa[p6]][2 * kc + lk][wi + 32 * x + l32]);
#pragma unroll
                for (int y = 0; y < 2; y++)
                    b[y] = __builtin_bit_cast(bf16x8, bs[S][pb[p6]][2 * kc + lk][wj + 32 * y + l32]);
#pragma unroll
                for (int m = 0; m < 2 * NX; m++) {
                    acc[m >> 1][m & 1] =
                        __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[m >> 1], b[m & 1], acc[m >> 1][m & 1], 0, 0, 0);
                    // the split's steps spread over the trip's MFMAs
                    const int gm = (kc * 6 + p6) * 2 * NX + m;
#pragma unroll
                    for (int n = kSteps * gm / kMfmas; n < kSteps * (gm + 1) / kMfmas; n++) step(n);
                }
            }
        write_split(R, hi, mid, lo);
        fetch_next(ra[R], rb[R]);
        __syncthreads();
    };
    // after a trip: was that the tile's last?  Then its results go out.  Behind the last tile nothing is stored
    // any more (a trip that still follows multiplies what the fetches past the end left in LDS).
    auto tile_done = [&]() {
        if (--left_m > 0) return;
        store_tile<EPI, NX, 2, 2, true>(q, acc, out_m, i0_m + wi, j0_m + wj, l32, lk);
        if (w_m + (int)gridDim.x >= n_tiles) {
            left_m = 0x7fffffff;
            return;
        }
        w_m += gridDim.x;
        describe_m();
        zero_acc();
    };
    // The loop leaves at its end only, after a counted number of trip pairs (one trip more than the stream has
    // when that number is odd).  With an exit between the two trips the compiler's structured form of the loop
    // has a path from the first trip straight back to itself, and on that path the register set that the
    // first trip splits is the newest one loaded: its waits would then cover the loads of the trip before
    // instead of those of two trips before.
    int trips = 0;
    for (int w = blockIdx.x; w < n_tiles; w += gridDim.x) {
        int it, jt, z;
        gemm_tile_of(q, w, it, jt, z);
        const int k_begin = (z % q.splits) * q.k_per_split;
        trips += (min(q.K, k_begin + q.k_per_split) - k_begin) / kUnit;
    }
    for (int n = (trips + 1) >> 1; n > 0; n--) {
        trip(std::integral_constant<int, 0>());
        tile_done();
        trip(std::integral_constant<int, 1>());
        tile_done();
    }
}

// gt[n*npos + pos][co] = g[n][co][pos]: the upstream gradient with the channel innermost, so that the
// first GEMM's epilogue (lanes along the channel) reads it in contiguous runs instead of one
// cache line per lane.  32 x 32 tiles through LDS; blockIdx.z = n.
__global__ __launch_bounds__(256) void k_transpose_grad(const float* __restrict__ g, float* __restrict__ gt, int c_out,
                                                        int npos)
{
    __shared__ float tile[32][33];
    const size_t item = (size_t)blockIdx.z * c_out * npos;
    const int p0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int r = ty; r < 32; r += 8) {
        const int c = c0 + r, p = p0 + tx;
        tile[r][tx] = (c < c_out && p < npos) ? g[item + (size_t)c * npos + p] : 0.0f;
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        const int p = p0 + r, c = c0 + tx;
        if (p < npos && c < c_out) gt[item + (size_t)p * c_out + c] = tile[tx][r];
    }
}

// Per output position m = (n, a, b): where its receptive field starts in the unpadded input.
//   base[m] = ((n*c_in)*w_in + (a - pad_w))*h_in + (b - pad_h),  arow[m] = a - pad_w,  bcol[m] = b - pad_h
// Built once per call; it keeps integer divisions out of the per-element kernels.
__global__ __launch_bounds__(256) void k_position_table(int* __restrict__ base, int* __restrict__ arow,
                                                        int* __restrict__ bcol, int m_total,
                                                        int c_in, int c_out, int w_in, int h_in, int pad_w, int pad_h,
                                                        int wo, int ho)
{
    for (int m = blockIdx.x * 256 + threadIdx.x; m < m_total; m += gridDim.x * 256) {
        const int b = m % ho;
        const int t = m / ho;
        const int a = t % wo;
        const int n = t / wo;
        base[m] = ((n * c_in) * w_in + (a - pad_w)) * h_in + (b - pad_h);
        arow[m] = a - pad_w;
        bcol[m] = b - pad_h;
    }
}

// Group structure of one accumulation mode: which weight element (ci, u, v) member k of add
// group g is, and the inverse.
struct Groups {
    int mode, c_in, w_k, h_k, zu;
    int n_groups, n_members;
};

struct Member {
    int ci, u, v;
    bool ok;
};

__host__ __device__ inline Member member_of(const Groups& G, int g, int k)
{
    Member e;
    if (G.mode == GEO_SC_ACC_Z) {
        e.ci = g;
        e.u = k / G.h_k;
        e.v = k - e.u * G.h_k;
        e.ok = true;
    } else if (G.mode == GEO_SC_ACC_FULL) {
        const int t = k / G.h_k;
        e.v = k - t * G.h_k;
        e.ci = t / G.w_k;
        e.u = t - e.ci * G.w_k;
        e.ok = true;
    } else if (G.mode == GEO_SC_ACC_YZ) {
        const int blk = g / G.h_k;
        const int cl = k / G.w_k;
        e.v = g - blk * G.h_k;
        e.u = k - cl * G.w_k;
        e.ci = blk * G.zu + cl;
        e.ok = e.ci < G.c_in;
    } else {
        e.ci = k / G.w_k;
        e.u = k - e.ci * G.w_k;
        e.v = g;
        e.ok = true;
    }
    return e;
}

// member k+1 of the same group from member k
__host__ __device__ inline void next_member(const Groups& G, Member& e)
{
    if (G.mode == GEO_SC_ACC_Z) {
        if (++e.v == G.h_k) {
            e.v = 0;
            ++e.u;
        }
    } else if (G.mode == GEO_SC_ACC_FULL) {
        if (++e.v == G.h_k) {
            e.v = 0;
            if (++e.u == G.w_k) {
                e.u = 0;
                ++e.ci;
            }
        }
    } else if (++e.u == G.w_k) {
        e.u = 0;
        ++e.ci;
        e.ok = e.ci < G.c_in;
    }
}

__host__ __device__ inline void group_of(const Groups& G, int ci, int u, int v, int& g, int& k)
{
    if (G.mode == GEO_SC_ACC_Z) {
        g = ci;
        k = u * G.h_k + v;
    } else if (G.mode == GEO_SC_ACC_FULL) {
        g = 0;
        k = (ci * G.w_k + u) * G.h_k + v;
    } else if (G.mode == GEO_SC_ACC_YZ) {
        const int blk = ci / G.zu;
        g = blk * G.h_k + v;
        k = (ci - blk * G.zu) * G.w_k + u;
    } else {
        g = v;
        k = ci * G.w_k + u;
    }
}

// col[g][k][m] = x~[n, ci, a+u, b+v] for groups g0 + blockIdx.z, (ci, u, v) = member k of the
// group, m = (n, a, b); x~ is the zero-padded activation, read straight from the unpadded
// tensor.  blockIdx.y selects kIm2colMembers consecutive members; a thread reads its position's
// table entry once and moves those members.  Reads and writes run along m.
constexpr int kIm2colMembers = 12;
__global__ __launch_bounds__(256) void k_im2col_rows(const float* __restrict__ x, float* __restrict__ col,
                                                     const int* __restrict__ base, const int* __restrict__ arow,
                                                     const int* __restrict__ bcol, int g0, int m_total, Groups G,
                                                     int w_in, int h_in, size_t g_stride)
{
    const int g = g0 + blockIdx.z;
    const int k0 = blockIdx.y * kIm2colMembers;
    const int k1 = min(G.n_members, k0 + kIm2colMembers);
    float* colg = col + (size_t)blockIdx.z * g_stride;
    for (int m = blockIdx.x * 256 + threadIdx.x; m < m_total; m += gridDim.x * 256) {
        const int r0 = arow[m], c0 = bcol[m], b0 = base[m];
        // all loads first, from x[0] where the member lies in the padding (a load inside a branch is
        // waited for before the next one is issued), then the stores
        float vals[kIm2colMembers];
        Member e = member_of(G, g, k0);
#pragma unroll
        for (int q = 0; q < kIm2colMembers; q++) {
            const int r = r0 + e.u, c = c0 + e.v;
            const bool ok = k0 + q < k1 && e.ok && c >= 0 && c < h_in && r >= 0 && r < w_in;
            const float val = x[ok ? b0 + (e.ci * w_in + e.u) * h_in + e.v : 0];
            vals[q] = ok ? val : 0.0f;
            next_member(G, e);
        }
#pragma unroll
        for (int q = 0; q < kIm2colMembers; q++)
            if (k0 + q < k1) colg[(size_t)(k0 + q) * m_total + m] = vals[q];
    }
}

// Four consecutive values of a row of floats starting `sh` (0..3) floats into the aligned quad a,
// continued in the next quad b.
__device__ __forceinline__ float4 shifted_quad(const float4& a, const float4& b, int sh)
{
    float4 r;
    r.x = sh == 0 ? a.x : sh == 1 ? a.y : sh == 2 ? a.z : a.w;
    r.y = sh == 0 ? a.y : sh == 1 ? a.z : sh == 2 ? a.w : b.x;
    r.z = sh == 0 ? a.z : sh == 1 ? a.w : sh == 2 ? b.x : b.y;
    r.w = sh == 0 ? a.w : sh == 1 ? b.x : sh == 2 ? b.y : b.z;
    return r;
}

// k_im2col_rows with four positions per thread, for image rows of a multiple of four elements on both
// sides (h_in, ho) and a 16-byte aligned x: the four positions are neighbours in one output row, so a
// member's four values are four consecutive elements of one input row, cut out of one or two aligned
// quads (the kernel tap shifts them by v - pad_h) and stored as one quad: a quarter of the loads,
// stores and table reads of the one-position kernel.
__global__ __launch_bounds__(256) void k_im2col_rows_v4(const float* __restrict__ x, float* __restrict__ col,
                                                        const int* __restrict__ base, const int* __restrict__ arow,
                                                        const int* __restrict__ bcol, int g0, int m_total, Groups G,
                                                        int w_in, int h_in, size_t g_stride)
{
    const int g = g0 + blockIdx.z;
    const int k0 = blockIdx.y * kIm2colMembers;
    const int k1 = min(G.n_members, k0 + kIm2colMembers);
    float* colg = col + (size_t)blockIdx.z * g_stride;
    const float4* x4 = (const float4*)x;
    const int quads = m_total >> 2;
    for (int mq = blockIdx.x * 256 + threadIdx.x; mq < quads; mq += gridDim.x * 256) {
        const int m = mq << 2;
        const int r0 = arow[m], c0 = bcol[m], b0 = base[m];
        float4 vals[kIm2colMembers];
        Member e = member_of(G, g, k0);
#pragma unroll
        for (int q = 0; q < kIm2colMembers; q++) {
            const int r = r0 + e.u, c = c0 + e.v;  // c: column of the first of the four values
            const int sh = c & 3, ca = c - sh;     // the aligned quads at columns ca and ca + 4 hold them
            const bool row_ok = k0 + q < k1 && e.ok && r >= 0 && r < w_in;
            const bool ok_a = row_ok && ca >= 0 && ca < h_in;
            const bool ok_b = row_ok && sh != 0 && ca + 4 >= 0 && ca + 4 < h_in;
            const int at = (b0 + (e.ci * w_in + e.u) * h_in + e.v - sh) >> 2;  // quad index of column ca of that row
            float4 a = x4[ok_a ? at : 0], b = x4[ok_b ? at + 1 : 0];
            if (!ok_a) a = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (!ok_b) b = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            vals[q] = shifted_quad(a, b, sh);
            next_member(G, e);
        }
#pragma unroll
        for (int q = 0; q < kIm2colMembers; q++)
            if (k0 + q < k1) *(float4*)(colg + (size_t)(k0 + q) * m_total + m) = vals[q];
    }
}

// The input as col without the copies: planes xs[v][ci][n][r][b] = x~[n, ci, r, b + v] over the padded
// rows r (w_in + 2 pad_w of them) and the output columns b, one per kernel column v and channel.  Member
// (ci, u, v) at position m = (n, a, b) is xs[v][ci][n][a + u][b]: row (ci, u) of col for kernel column v is
// the plane (v, ci) read from u * ho elements in, with the positions of item n shifted by
// n * (w_k - 1) * ho -- a third of col's bytes for a 3-wide kernel, and the rows of one channel share
// their cache lines.  Four columns per thread (ho and h_in multiples of four, 16-byte aligned x), as in
// k_im2col_rows_v4.  `total` quads; the (w_k - 1) * ho elements behind the last plane are never read.
__global__ __launch_bounds__(256) void k_shift_planes(const float* __restrict__ x, float* __restrict__ xs, long long total,
                                                      int n_items, int c_in, int w_in, int h_in, int pad_w, int pad_h,
                                                      int ho)
{
    const int wp = w_in + 2 * pad_w, hq = ho >> 2;
    const float4* x4 = (const float4*)x;
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
        // e = (((v * c_in + ci) * n_items + n) * wp + r) * hq + quad
        long long t = e;
        const int bq = (int)(t % hq);
        t /= hq;
        const int r = (int)(t % wp);
        t /= wp;
        const int n = (int)(t % n_items);
        t /= n_items;
        const int ci = (int)(t % c_in), v = (int)(t / c_in);
        const int row = r - pad_w, c = 4 * bq + v - pad_h;  // input row, and input column of the first of the four
        const int sh = c & 3, ca = c - sh;
        const bool row_ok = row >= 0 && row < w_in;
        const bool ok_a = row_ok && ca >= 0 && ca < h_in, ok_b = row_ok && sh != 0 && ca + 4 >= 0 && ca + 4 < h_in;
        const long long at = ((((long long)n * c_in + ci) * w_in + row) * h_in + ca) >> 2;
        float4 a = x4[ok_a ? at : 0], b = x4[ok_b ? at + 1 : 0];
        if (!ok_a) a = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (!ok_b) b = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        ((float4*)xs)[e] = shifted_quad(a, b, sh);
    }
}

// Weight operands of groups g0 + blockIdx.y:
//   wcat[g][k][j]: j < c_out -> clamp(w,0,100), j >= c_out -> -clamp(w,-100,0)   (utils_functional.py:611-612)
//   wd[g][j][k]  : the same with the negative rail negated (it enters dL/dx with a minus sign)
// Members that do not exist (ragged last channel block) get zeros.
__global__ __launch_bounds__(256) void k_weight_operands(const float* __restrict__ w, float* __restrict__ wcat,
                                                         float* __restrict__ wd, int g0, int c_out, Groups G,
                                                         size_t g_stride)
{
    const int K = G.n_members;
    const int total = K * c_out;
    const int g = g0 + blockIdx.y;
    float* wcatg = wcat + (size_t)blockIdx.y * g_stride;
    float* wdg = wd + (size_t)blockIdx.y * g_stride;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        const int co = e % c_out, k = e / c_out;
        const Member mb = member_of(G, g, k);
        const float wv = mb.ok ? w[(((long long)co * G.c_in + mb.ci) * G.w_k + mb.u) * G.h_k + mb.v] : 0.0f;
        const float wp = fminf(fmaxf(wv, 0.0f), 100.0f);
        const float wn = -fminf(fmaxf(wv, -100.0f), 0.0f);
        wcatg[(long long)k * 2 * c_out + co] = wp;
        wcatg[(long long)k * 2 * c_out + c_out + co] = wn;
        wdg[(long long)co * K + k] = wp;
        wdg[(long long)(c_out + co) * K + k] = -wn;
    }
}

// dL/dw of the members of group g0 + blockIdx.y from the split partial sums part[g][s][k][j].  A
// block takes 32 consecutive (k, co) entries; 8 sets of threads each sum every 8th split, the
// sets are then added in a fixed order, so the result does not depend on scheduling.
__global__ __launch_bounds__(256) void k_reduce_wgrad(const float* __restrict__ part, const float* __restrict__ w,
                                                      float* __restrict__ gw, int g0, int splits, int c_out, Groups G,
                                                      size_t g_stride)
{
    __shared__ float red[2][8][32];
    const int K = G.n_members;
    const int total = K * c_out;
    const long long stride = (long long)K * 2 * c_out;
    const int g = g0 + blockIdx.y;
    const float* partg = part + (size_t)blockIdx.y * g_stride;
    const int lane = threadIdx.x & 31, grp = threadIdx.x >> 5;
    const int e = blockIdx.x * 32 + lane;
    const bool ok = e < total;
    const int co = ok ? e % c_out : 0, k = ok ? e / c_out : 0;
    float sp = 0.0f, sn = 0.0f;
    if (ok)
        for (int s = grp; s < splits; s += 8) {
            sp += partg[s * stride + (long long)k * 2 * c_out + co];
            sn += partg[s * stride + (long long)k * 2 * c_out + c_out + co];
        }
    red[0][grp][lane] = sp;
    red[1][grp][lane] = sn;
    __syncthreads();
    const Member mb = member_of(G, g, k);
    if (grp == 0 && ok && mb.ok) {
        sp = sn = 0.0f;
#pragma unroll
        for (int gidx = 0; gidx < 8; gidx++) {
            sp += red[0][gidx][lane];
            sn += red[1][gidx][lane];
        }
        const long long wi = (((long long)co * G.c_in + mb.ci) * G.w_k + mb.u) * G.h_k + mb.v;
        const float wv = w[wi];
        float r = 0.0f;
        if (wv >= 0.0f && wv <= 100.0f) r += sp;
        if (wv >= -100.0f && wv <= 0.0f) r += sn;
        gw[wi] = r;
    }
}

// dL/dx[n][ci][p][q] (+)= sum over the kernel taps (u, v) whose group lies in [g0, g0 + ng) of
// dcol[g][k][(n, p+pad_w-u, q+pad_h-v)] over the valid output positions; the first chunk of
// groups writes, later chunks add.  Blocks stride over the planes (n, ci).
__global__ __launch_bounds__(256) void k_col2im_rows(const float* __restrict__ dcol, float* __restrict__ gx, int g0,
                                                     int ng, long long m_total, int n_planes, Groups G, int w_in,
                                                     int h_in, int pad_w, int pad_h, int wo, int ho, size_t g_stride)
{
    const int plane = w_in * h_in;
    const int k_step = (G.mode == GEO_SC_ACC_Z || G.mode == GEO_SC_ACC_FULL) ? G.h_k : 1;
    for (int nc = blockIdx.x; nc < n_planes; nc += gridDim.x) {
        const int n = nc / G.c_in, ci = nc - n * G.c_in;
        float* dst = gx + (size_t)nc * plane;
        const float* src = dcol + (size_t)n * wo * ho;
        for (int e = blockIdx.y * 256 + threadIdx.x; e < plane; e += gridDim.y * 256) {
            const int p = e / h_in, qq = e - p * h_in;
            float s = 0.0f;
            // kernel rows v whose output column b = qq + pad_h - v exists (a 1 x 256 kernel on a 256-wide
            // input has one such row per element, not 256)
            const int v_lo = max(0, qq + pad_h - (ho - 1)), v_hi = min(G.h_k - 1, qq + pad_h);
            for (int v = v_lo; v <= v_hi; v++) {
                const int b = qq + pad_h - v;
                // the group does not depend on u, and the member index advances by k_step per tap
                int g, k;
                group_of(G, ci, 0, v, g, k);
                if (g < g0 || g >= g0 + ng) continue;  // uniform
                const bool b_ok = b >= 0 && b < ho;
                const float* sg = src + (size_t)(g - g0) * g_stride + (size_t)k * m_total + (b_ok ? b : 0);
                // four taps at a time: loads from clamped addresses first, then the sum
                for (int u0 = 0; u0 < G.w_k; u0 += 4) {
                    float t[4];
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int u = u0 + q, a = p + pad_w - u;
                        const bool ok = b_ok && u < G.w_k && a >= 0 && a < wo;
                        const float val = sg[ok ? (size_t)u * k_step * m_total + a * ho : 0];
                        t[q] = ok ? val : 0.0f;
                    }
                    s += (t[0] + t[1]) + (t[2] + t[3]);
                }
            }
            dst[e] = g0 == 0 ? s : dst[e] + s;
        }
    }
}

// k_col2im_rows with four elements of an input row per thread, for image rows of a multiple of four
// elements on both sides, kernels of at most eight columns and 16-byte aligned buffers: a tap's four
// terms are four consecutive elements of one dcol row, cut out of one or two aligned quads.  One
// grid-stride loop over the quads of all planes.
__global__ __launch_bounds__(256) void k_col2im_rows_v4(const float* __restrict__ dcol, float* __restrict__ gx, int g0,
                                                        int ng, long long m_total, int n_planes, Groups G, int w_in,
                                                        int h_in, int pad_w, int pad_h, int wo, int ho, size_t g_stride)
{
    const int plane = w_in * h_in, plane_quads = plane >> 2;
    const int k_step = (G.mode == GEO_SC_ACC_Z || G.mode == GEO_SC_ACC_FULL) ? G.h_k : 1;
    const long long total = (long long)n_planes * plane_quads;
    for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long long)gridDim.x * 256) {
        const int nc = (int)(idx / plane_quads), eq = (int)(idx - (long long)nc * plane_quads);
        const int n = nc / G.c_in, ci = nc - n * G.c_in;
        float4* dst = (float4*)(gx + (size_t)nc * plane);
        const float* src = dcol + (size_t)n * wo * ho;
        const int e = eq << 2;
        const int p = e / h_in, qq = e - p * h_in;  // the thread's elements are (p, qq .. qq + 3)
        float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (int v = 0; v < G.h_k; v++) {
            int g, k;
            group_of(G, ci, 0, v, g, k);
            if (g < g0 || g >= g0 + ng) continue;
            const int b = qq + pad_h - v;  // output column of the first element's term
            const int sh = b & 3, ba = b - sh;
            const bool ok_a = ba >= 0 && ba < ho, ok_b = sh != 0 && ba + 4 >= 0 && ba + 4 < ho;
            const float* sg = src + (size_t)(g - g0) * g_stride + (size_t)k * m_total;
            for (int u = 0; u < G.w_k; u++) {
                const int a = p + pad_w - u;
                const bool row_ok = a >= 0 && a < wo;
                const float4* row = (const float4*)(sg + (size_t)u * k_step * m_total + (row_ok ? a : 0) * ho);
                float4 qa = row[(row_ok && ok_a) ? ba >> 2 : 0], qb = row[(row_ok && ok_b) ? (ba >> 2) + 1 : 0];
                if (!(row_ok && ok_a)) qa = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (!(row_ok && ok_b)) qb = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                const float4 t = shifted_quad(qa, qb, sh);
                s.x += t.x;
                s.y += t.y;
                s.z += t.z;
                s.w += t.w;
            }
        }
        if (g0 != 0) {
            const float4 o = dst[eq];
            s.x += o.x;
            s.y += o.y;
            s.z += o.z;
            s.w += o.w;
        }
        dst[eq] = s;
    }
}

// (ci, u, v) of the flat index i of one output channel's weights
__device__ __forceinline__ void weight_coords(const Groups& G, int i, int& ci, int& u, int& v)
{
    const int t = i / G.h_k;
    v = i - t * G.h_k;
    ci = t / G.w_k;
    u = t - ci * G.w_k;
}

// wcat of the groups [g0, g0 + ng) for the fused kernel (which forms wd from it): a block moves a
// tile of 32 output channels x 32 consecutive weights of each through LDS, so that w is read and wcat
// written in 128-byte runs whatever the accumulation mode (k_weight_operands reads or writes one
// element per cache line when the members of a group are not neighbours in w).  Only members that
// exist are written: not for ragged channel blocks.  blockIdx = (weight tile, channel tile).
__global__ __launch_bounds__(256) void k_weight_cat_tiled(const float* __restrict__ w, float* __restrict__ wcat, int g0,
                                                          int ng, int c_out, Groups G, size_t g_stride)
{
    __shared__ float t[32][33];  // [channel][weight]
    const int per_channel = G.c_in * G.w_k * G.h_k;
    const int i0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int q = ty; q < 32; q += 8) {
        const int co = c0 + q, i = i0 + tx;
        t[q][tx] = (co < c_out && i < per_channel) ? w[(size_t)co * per_channel + i] : 0.0f;
    }
    __syncthreads();
    for (int q = ty; q < 32; q += 8) {
        const int i = i0 + q, co = c0 + tx;
        if (i >= per_channel || co >= c_out) continue;
        int ci, u, v, g, k;
        weight_coords(G, i, ci, u, v);
        group_of(G, ci, u, v, g, k);
        if (g < g0 || g >= g0 + ng) continue;
        const float wv = t[tx][q];
        float* row = wcat + (size_t)(g - g0) * g_stride + (size_t)k * 2 * c_out;
        row[co] = fminf(fmaxf(wv, 0.0f), 100.0f);
        row[c_out + co] = -fminf(fmaxf(wv, -100.0f), 0.0f);
    }
}

// k_reduce_wgrad with the same tiles: the partial sums part[g][s][k][j] of 32 weights x 32 channels
// are read in 128-byte runs along the channel, added over the splits in their order, and dL/dw is
// written in 128-byte runs along the weights of one channel.
__global__ __launch_bounds__(256) void k_reduce_wgrad_tiled(const float* __restrict__ part, const float* __restrict__ w,
                                                            float* __restrict__ gw, int g0, int ng, int splits, int c_out,
                                                            Groups G, size_t g_stride)
{
    __shared__ float tp[32][33], tn[32][33];  // [weight][channel]
    const int per_channel = G.c_in * G.w_k * G.h_k;
    const long long stride = (long long)G.n_members * 2 * c_out;
    const int i0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int q = ty; q < 32; q += 8) {
        const int i = i0 + q, co = c0 + tx;
        float sp = 0.0f, sn = 0.0f;
        if (i < per_channel && co < c_out) {
            int ci, u, v, g, k;
            weight_coords(G, i, ci, u, v);
            group_of(G, ci, u, v, g, k);
            if (g >= g0 && g < g0 + ng) {
                const float* src = part + (size_t)(g - g0) * g_stride + (size_t)k * 2 * c_out + co;
                for (int s0 = 0; s0 < splits; s0++) {
                    sp += src[s0 * stride];
                    sn += src[s0 * stride + c_out];
                }
            }
        }
        tp[q][tx] = sp;
        tn[q][tx] = sn;
    }
    __syncthreads();
    for (int q = ty; q < 32; q += 8) {
        const int co = c0 + q, i = i0 + tx;
        if (i >= per_channel || co >= c_out) continue;
        int ci, u, v, g, k;
        weight_coords(G, i, ci, u, v);
        group_of(G, ci, u, v, g, k);
        if (g < g0 || g >= g0 + ng) continue;
        const size_t wi = (size_t)co * per_channel + i;
        const float wv = w[wi];
        float r = 0.0f;
        if (wv >= 0.0f && wv <= 100.0f) r += tp[tx][q];
        if (wv >= -100.0f && wv <= 0.0f) r += tn[tx][q];
        gw[wi] = r;
    }
}

// What a round of GEMM launches needs beforehand, in one launch (grid: blocks x groups of the round):
//  * the weight operands wcat / wd of k_weight_operands, for group g0 + blockIdx.y;
//  * with dx_rows, in wd's place, the A operand of the input-gradient product that sums kernel taps inside
//    the GEMM (y accumulation: group = kernel column v, members (ci, u)): wdx[k][ci] = wd[v][j][(ci, u)], i.e.
//    clamp(w, 0, 100) for the positive rail j < c_out and clamp(w, -100, 0) for the negative one, with the tap
//    as the fast index over chunks of kChunk columns - dx_rows = 1: one operand per group,
//    k = ((j / kChunk) * w_k + u) * kChunk + j % kChunk (the kernel rows inside the product); dx_rows = 2: one
//    operand for all groups, k = (((j / kChunk) * h_k + v) * w_k + u) * kChunk + j % kChunk (all taps inside):
//    consecutive chunks of the product then read the same columns of E one image row, then one image column
//    apart (ShiftStager);
//  * from the blocks of the round's first group: view_rows[g][k], where row k of group g's col starts in the
//    planes of k_shift_planes (elements), for every group; and 64 zeros for the shifted view of E (a store
//    rather than a memset, so that a caller may capture the launch sequence in a graph).
struct PrepParams {
    const float* __restrict__ w;
    float* __restrict__ wcat;
    float* __restrict__ wd;
    int g0, c_out;
    Groups G;
    size_t g_stride;
    int dx_rows;            // wd holds the wdx operand (y accumulation: c_in, w_k, h_k from G): 1 per group, 2 one for all
    long long* view_rows;   // null: no view
    int view_groups, view_k_pad, ho;
    long long plane;
    float* zero;            // null: no block of zeros wanted
};
__global__ __launch_bounds__(256) void k_bwd_prep(PrepParams q)
{
    const int K = q.G.n_members, c_out = q.c_out;
    const int g = q.g0 + blockIdx.y;
    float* wcatg = q.wcat + (size_t)blockIdx.y * q.g_stride;
    float* wdg = q.wd + (size_t)blockIdx.y * q.g_stride;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < K * c_out; e += gridDim.x * 256) {
        const int co = e % c_out, k = e / c_out;
        const Member mb = member_of(q.G, g, k);
        const float wv = mb.ok ? q.w[(((long long)co * q.G.c_in + mb.ci) * q.G.w_k + mb.u) * q.G.h_k + mb.v] : 0.0f;
        const float wp = fminf(fmaxf(wv, 0.0f), 100.0f);
        const float wn = -fminf(fmaxf(wv, -100.0f), 0.0f);
        wcatg[(long long)k * 2 * c_out + co] = wp;
        wcatg[(long long)k * 2 * c_out + c_out + co] = wn;
        if (!q.dx_rows) {
            wdg[(long long)co * K + k] = wp;
            wdg[(long long)(c_out + co) * K + k] = -wn;
        }
    }
    if (q.dx_rows) {
        // this block row's kernel column g: its own operand, or its part of the one operand (which starts where
        // the round's wd starts)
        const int J = 2 * c_out, c_in = q.G.c_in, w_k = q.G.w_k, h_k = q.G.h_k;
        for (int e = blockIdx.x * 256 + threadIdx.x; e < w_k * J * c_in; e += gridDim.x * 256) {
            const int ci = e % c_in, r = e / c_in;
            const int chunk = r / kChunk, u = chunk % w_k, jc = chunk / w_k, jj = r % kChunk, j = jc * kChunk + jj;
            const int co = j >= c_out ? j - c_out : j;
            const float wv = q.w[(((size_t)co * c_in + ci) * w_k + u) * h_k + g];
            const float val = j < c_out ? fminf(fmaxf(wv, 0.0f), 100.0f) : fminf(fmaxf(wv, -100.0f), 0.0f);
            if (q.dx_rows == 2)
                q.wd[((((size_t)jc * h_k + g) * w_k + u) * kChunk + jj) * c_in + ci] = val;
            else
                wdg[e] = val;
        }
    }
    if (blockIdx.y == 0) {
        if (q.view_rows)
            for (int e = blockIdx.x * 256 + threadIdx.x; e < q.view_groups * q.view_k_pad; e += gridDim.x * 256) {
                const int gi = e / q.view_k_pad, k = e - gi * q.view_k_pad;
                const Member mb = member_of(q.G, gi, k < K ? k : K - 1);
                q.view_rows[e] = ((long long)mb.v * q.G.c_in + mb.ci) * q.plane + (long long)mb.u * q.ho;
            }
        if (q.zero && blockIdx.x == 0 && threadIdx.x < 64) q.zero[threadIdx.x] = 0.0f;
    }
}

// dL/dx[n][ci][p][q] = sum over the kernel columns v of d[v][ci][(n, p, q + pad_h - v)] where that output
// column exists: what is left of col2im when the GEMM has summed the kernel rows.  Four elements of an
// input row per thread (rows of whole quads on both sides, 16-byte aligned buffers), one grid-stride loop
// over the quads of dL/dx.
__global__ __launch_bounds__(256) void k_shift_sum_v4(const float* __restrict__ d, float* __restrict__ gx, long long quads,
                                                      int n_items, int c_in, int w_in, int h_in, int h_k, int pad_h,
                                                      int ho)
{
    const int hq = h_in >> 2;
    const long long per_v = (long long)c_in * n_items * w_in * ho;
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < quads; e += (long long)gridDim.x * 256) {
        // e = ((n * c_in + ci) * w_in + p) * hq + quad
        long long t = e;
        const int qq = (int)(t % hq) << 2;
        t /= hq;
        const int p = (int)(t % w_in);
        t /= w_in;
        const int ci = (int)(t % c_in), n = (int)(t / c_in);
        const float* row = d + (((long long)ci * n_items + n) * w_in + p) * ho;
        float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (int v = 0; v < h_k; v++) {
            const int b = qq + pad_h - v;
            const int sh = b & 3, ba = b - sh;
            const bool ok_a = ba >= 0 && ba < ho, ok_b = sh != 0 && ba + 4 >= 0 && ba + 4 < ho;
            const float4* r4 = (const float4*)(row + v * per_v);
            float4 qa = r4[ok_a ? ba >> 2 : 0], qb = r4[ok_b ? (ba >> 2) + 1 : 0];
            if (!ok_a) qa = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (!ok_b) qb = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            const float4 tq = shifted_quad(qa, qb, sh);
            s.x += tq.x;
            s.y += tq.y;
            s.z += tq.z;
            s.w += tq.w;
        }
        ((float4*)gx)[e] = s;
    }
}

// a[i] += b_1[i] + ... + b_{n-1}[i] for n arrays `stride` floats apart (a is the first), four floats
// per thread, the arrays added in their order: the dcol slices of the fused kernel's column blocks.
// count and stride are multiples of 4.
__global__ __launch_bounds__(256) void k_sum_slices(float* __restrict__ a, size_t count, int n, size_t stride)
{
    const size_t n4 = count / 4;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
        float4 acc = ((const float4*)a)[i];
        for (int s0 = 1; s0 < n; s0 += 8) {
            float4 v[8];
#pragma unroll
            for (int q = 0; q < 8; q++) v[q] = ((const float4*)(a + (size_t)(s0 + q < n ? s0 + q : 0) * stride))[i];
#pragma unroll
            for (int q = 0; q < 8; q++)
                if (s0 + q < n) {
                    acc.x += v[q].x;
                    acc.y += v[q].y;
                    acc.z += v[q].z;
                    acc.w += v[q].w;
                }
        }
        ((float4*)a)[i] = acc;
    }
}

// Whole backward of layers with small OR groups (K <= 32 members: z accumulation has K = W * H,
// yz with small channel blocks K = z_unit * W, the SC linear layer K = 16) in one kernel.  With few
// members per group the general path's scratch array E[g][m][j] is c_in (z) times larger than the
// problem's tensors and its GEMMs use a fraction of each MFMA; here a workgroup loops over tiles of
// 32 output positions of one group, gathers the im2col columns into LDS, forms Z = col^T wcat with
// MFMAs, turns it into E = g exp(-Z) in LDS and feeds both Gw += col E (accumulators live over all
// tiles) and dcol = wd^T E^T from it; only dcol (the size of col) reaches memory, for the common
// col2im.  The weights of both products sit in registers for the life of the workgroup.
//   KS: k-steps of the first product (ceil(K / 2), rounded up to 5, 8, 12 or 16)
//   NB: 32-column blocks of E per wave; a workgroup covers NB * 128 columns, wider layers take
//       several column blocks, each writing a slice dcol[block][g][k][m] of its own that
//       k_sum_slices adds in a fixed order
//   DX: the input gradient is wanted
// A workgroup handles tiles s, s + S, ... of one column block of group g0 + blockIdx.y and writes
// its columns of one partial sum part[g][s][k][j] for the common split reduction.
//
// The vector ALU shares its issue slots with the MFMAs, so every instruction per element of E counts:
// the upstream gradient comes in the register order of the first product's result (k_tile_grad: four
// 16-byte loads per 32 x 32 block, no address arithmetic per element), E is stored transposed
// (E^T[j][m], rows of kFusedLd floats) with 16-byte stores, and no element is range-checked: rows
// beyond M hold zeros in col and in the gradient, columns beyond 2 * c_out meet zero weights in the
// input-gradient product and are never stored by the weight-gradient one.
constexpr int kFusedK = 32;
constexpr int kFusedTile = 32;
constexpr int kFusedLd = 36;  // floats per LDS row of a tile: 16-byte aligned rows, conflict-free MFMA operand reads

// Upstream gradient in tiles of 32 positions x 32 columns, each stored in the register order of a
// 32 x 32 MFMA result: gtt[(tile * n_blocks + block) * 1024 + lane * 16 + r] = g[m][co] with
// m = 32 tile + 8 (r / 4) + 4 (lane / 32) + r % 4 and column 32 block + lane % 32; rows beyond M and
// columns beyond the last one are zero.  With dedupe (c_out a multiple of 32) the blocks run over
// c_out and serve both rails, otherwise over the 2 * c_out rails (column j -> channel j mod c_out).
// g is [n][c_out][npos]; blockIdx = (tile, block).
__global__ __launch_bounds__(256) void k_tile_grad(const float* __restrict__ g, float* __restrict__ gtt, int M, int c_out,
                                                   int npos, int n_blocks, int dedupe)
{
    __shared__ float t[32][33];  // [position][column]
    const int m0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int n_cols = dedupe ? c_out : 2 * c_out;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    // lanes along the positions where an item has many of them, along the channels otherwise
    const bool along_m = npos >= 8;
    for (int q = ty; q < 32; q += 8) {
        const int mi = along_m ? tx : q, ci = along_m ? q : tx;
        const int m = m0 + mi, c = c0 + ci;
        const int co = c >= c_out ? c - c_out : c;
        float v = 0.0f;
        if (m < M && c < n_cols) {
            const int n = m / npos, pos = m - n * npos;
            v = g[((size_t)n * c_out + co) * npos + pos];
        }
        t[mi][ci] = v;
    }
    __syncthreads();
    const int o = threadIdx.x * 4, lane = o >> 4, r = o & 15;
    const int i = 8 * (r >> 2) + 4 * (lane >> 5), l32 = lane & 31;
    float4 v = make_float4(t[i][l32], t[i + 1][l32], t[i + 2][l32], t[i + 3][l32]);
    *(float4*)(gtt + ((size_t)blockIdx.x * n_blocks + blockIdx.y) * 1024 + o) = v;
}

template <int KS, int NB, bool DX>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void k_bwd_small_k(
    const float* __restrict__ x, const float* __restrict__ wcat, const float* __restrict__ gtt,
    const int* __restrict__ base, const int* __restrict__ arow,
    const int* __restrict__ bcol, float* __restrict__ part, float* __restrict__ dcol, Groups G, int g0, int M, int w_in,
    int h_in, int c_out, int jblocks, int splits, int store_part, int gt_blocks, int gt_dedupe, size_t w_stride,
    size_t part_stride, size_t dcol_stride, size_t dcol_slice)
{
    constexpr int KP = KS <= 8 ? 16 : 32;       // member rows held in LDS and in the weight gradient
    constexpr int TM = kFusedTile, LD = kFusedLd;
    constexpr int JW = NB * 128;                // columns of E per workgroup
    constexpr int DPARTS = KP == 16 ? 2 : 1;    // waves that share one 16 x 16 block of dcol and split j
    constexpr int DSTEPS = JW / DPARTS / 4;     // 16x16x4 MFMAs per wave and tile in the dcol product
    constexpr int GQ = KP / 8;                  // members gathered per thread
    __shared__ __attribute__((aligned(16))) float cs[KP][LD];  // col tile [k][m]
    __shared__ __attribute__((aligned(16))) float es[JW][LD];  // E^T tile [j][m]
    __shared__ float red[2][16][17];            // second j-half's partial dcol blocks (KP == 16)
    const int K = G.n_members, J = 2 * c_out;
    const int g = g0 + blockIdx.y;
    // blockIdx.x = split * jblocks + column block: the workgroups that gather the same columns of x run together
    const int split = blockIdx.x / jblocks, jblock = blockIdx.x - split * jblocks;
    const int j_begin = jblock * JW;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int l32 = lane & 31, lk = lane >> 5, l16 = lane & 15, lq = lane >> 4;

    // this group's wcat[k][j_begin .. j_begin + JW) through LDS (the space of es), read in 128-byte
    // runs; zero outside the problem
    constexpr int WLD = JW + 1;
    float* wl = &es[0][0];
    {
        const float* wg = wcat + (size_t)blockIdx.y * w_stride;
        for (int e = threadIdx.x; e < KP * JW; e += 256) {
            const int k = e / JW, jl = e - k * JW, j = j_begin + jl;
            const bool ok = k < K && j < J;
            const float v = wg[ok ? (size_t)k * J + j : 0];
            wl[k * WLD + jl] = ok ? v : 0.0f;
        }
    }
    __syncthreads();
    // weights of the first product, B operand of step t: wcat[k = 2 t + lk][j]
    float w_s[NB][KS];
#pragma unroll
    for (int y = 0; y < NB; y++)
#pragma unroll
        for (int t = 0; t < KS; t++) w_s[y][t] = wl[(2 * t + lk) * WLD + 32 * (NB * wave + y) + l32];
    // dcol: wave -> (member block kb, position block mb, j part); A operand of step t: wd[j][k = 16 kb + l16],
    // which is wcat[k][j] with the negative rail (j >= c_out) negated (it enters dL/dx with a minus sign)
    const int kb = KP == 32 ? wave >> 1 : 0, mb = wave & 1, jpart = KP == 32 ? 0 : wave >> 1;
    const int jd0 = jpart * (JW / DPARTS);
    float w_d[DX ? DSTEPS : 1];
    if (DX) {
#pragma unroll
        for (int t = 0; t < DSTEPS; t++) {
            const int jl = jd0 + 4 * t + lq;
            const float v = wl[(16 * kb + l16) * WLD + jl];
            w_d[t] = j_begin + jl >= c_out ? -v : v;
        }
    }
    // (the tile loop's first barriers come before anything is written to es)
    // im2col gather: thread -> position (t & 31) of the tile, members (t >> 5) + 8 q
    const int ml = threadIdx.x & 31, slot = threadIdx.x >> 5;
    int g_off[GQ], g_u[GQ], g_v[GQ];
    bool g_ok[GQ];
#pragma unroll
    for (int q4 = 0; q4 < GQ; q4++) {
        const int k = slot + 8 * q4;
        const Member e = member_of(G, g, k < K ? k : 0);
        g_ok[q4] = k < K && e.ok;
        g_off[q4] = (e.ci * w_in + e.u) * h_in + e.v;
        g_u[q4] = e.u;
        g_v[q4] = e.v;
    }
    // this lane's 16 values of each 32 x 32 block of the upstream gradient: block of tile 0, and the
    // distance to the next tile of this workgroup
    const float* gp[NB];
#pragma unroll
    for (int y = 0; y < NB; y++) {
        const int j0 = j_begin + 32 * (NB * wave + y);
        int blk = gt_dedupe ? (j0 >= c_out ? j0 - c_out : j0) >> 5 : j0 >> 5;
        if (j0 >= J) blk = 0;  // columns outside the problem: any finite values will do
        gp[y] = gtt + ((size_t)split * gt_blocks + blk) * 1024 + lane * 16;
    }
    const size_t g_step = (size_t)splits * gt_blocks * 1024;

    // weight-gradient accumulators: 32 x 32 blocks (lane holds rows 8 (r/4) + 4 lk + r%4 of column l32),
    // or, with at most 16 members, 16 x 16 blocks (rows 4 lq + r of column l16) at half the MFMA time
    floatx16 gw_acc[KP == 32 ? NB : 1];
    floatx4 gw_acc4[KP == 16 ? 2 * NB : 1];
    if constexpr (KP == 32) {
#pragma unroll
        for (int y = 0; y < NB; y++)
#pragma unroll
            for (int r = 0; r < 16; r++) gw_acc[y][r] = 0.0f;
    } else {
#pragma unroll
        for (int b = 0; b < 2 * NB; b++)
#pragma unroll
            for (int r = 0; r < 4; r++) gw_acc4[b][r] = 0.0f;
    }

    float* dg = dcol + (size_t)jblock * dcol_slice + (size_t)blockIdx.y * dcol_stride;
    const int n_tiles = (M + TM - 1) / TM;
    for (int tile = split; tile < n_tiles; tile += splits) {
        const int m0 = tile * TM;
        // the tile's upstream gradient, asked for before anything waits: it is needed after the first product
        float4 gv[NB][4];
#pragma unroll
        for (int y = 0; y < NB; y++) {
#pragma unroll
            for (int q = 0; q < 4; q++) gv[y][q] = ((const float4*)gp[y])[q];
            gp[y] += g_step;
        }
        __syncthreads();  // the previous tile's products have read cs, es and red
        {
            const bool m_ok = m0 + ml < M;
            const int mc = m_ok ? m0 + ml : 0;
            const int r0 = arow[mc], c0 = bcol[mc], b0 = base[mc];
            float vals[GQ];
#pragma unroll
            for (int q4 = 0; q4 < GQ; q4++) {
                const int rr = r0 + g_u[q4], cc = c0 + g_v[q4];
                const bool ok = m_ok && g_ok[q4] && cc >= 0 && cc < h_in && rr >= 0 && rr < w_in;
                const float v = x[ok ? b0 + g_off[q4] : 0];
                vals[q4] = ok ? v : 0.0f;
            }
#pragma unroll
            for (int q4 = 0; q4 < GQ; q4++) cs[slot + 8 * q4][ml] = vals[q4];
        }
        __syncthreads();
#pragma unroll
        for (int y = 0; y < NB; y++) {
            // Z[m][j] = sum_k col[k][m] * wcat[k][j] for one 32 x 32 block
            floatx16 z;
#pragma unroll
            for (int r = 0; r < 16; r++) z[r] = 0.0f;
#pragma unroll
            for (int t = 0; t < KS; t++) z = __builtin_amdgcn_mfma_f32_32x32x2f32(cs[2 * t + lk][l32], w_s[y][t], z, 0, 0, 0);
            // E^T[j][m] = g[m][co] * exp(-Z): register r of the result is position 8 (r / 4) + 4 lk + r % 4
            float* er = &es[32 * (NB * wave + y) + l32][4 * lk];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                float4 e;
                e.x = gv[y][q].x * exp_neg(z[4 * q + 0]);
                e.y = gv[y][q].y * exp_neg(z[4 * q + 1]);
                e.z = gv[y][q].z * exp_neg(z[4 * q + 2]);
                e.w = gv[y][q].w * exp_neg(z[4 * q + 3]);
                *(float4*)(er + 8 * q) = e;
            }
        }
        __syncthreads();
        // Gw[k][j] += sum_m col[k][m] * E[m][j] on this wave's column blocks; a lane's share of the sum
        // over m is a run of consecutive positions, read with 16-byte loads
        if constexpr (KP == 32) {
            float a[16];
#pragma unroll
            for (int q = 0; q < 4; q++) *(float4*)&a[4 * q] = *(const float4*)&cs[l32][16 * lk + 4 * q];
#pragma unroll
            for (int y = 0; y < NB; y++) {
                float b[16];
#pragma unroll
                for (int q = 0; q < 4; q++) *(float4*)&b[4 * q] = *(const float4*)&es[32 * (NB * wave + y) + l32][16 * lk + 4 * q];
#pragma unroll
                for (int st = 0; st < 16; st++) gw_acc[y] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[st], b[st], gw_acc[y], 0, 0, 0);
            }
        } else {
            float a[8];
#pragma unroll
            for (int q = 0; q < 2; q++) *(float4*)&a[4 * q] = *(const float4*)&cs[l16][8 * lq + 4 * q];
#pragma unroll
            for (int bq = 0; bq < 2 * NB; bq++) {
                float b[8];
#pragma unroll
                for (int q = 0; q < 2; q++) *(float4*)&b[4 * q] = *(const float4*)&es[32 * NB * wave + 16 * bq + l16][8 * lq + 4 * q];
#pragma unroll
                for (int st = 0; st < 8; st++) gw_acc4[bq] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[st], b[st], gw_acc4[bq], 0, 0, 0);
            }
        }
        if (DX) {
            // dcol[k][m] = sum_j wd[j][k] * E[m][j]: one 16 x 16 block per wave (v_mfma_f32_16x16x4_f32:
            // lane l feeds A[i = l%16][k' = l/16] and B[k' = l/16][j = l%16], holds D[4 (l/16) + r][l%16])
            floatx4 d = {0.0f, 0.0f, 0.0f, 0.0f};
            const float* eb = &es[jd0 + lq][16 * mb + l16];
#pragma unroll
            for (int t = 0; t < DSTEPS; t++) d = __builtin_amdgcn_mfma_f32_16x16x4f32(w_d[t], eb[4 * t * LD], d, 0, 0, 0);
            if (DPARTS == 2) {
                if (jpart == 1) {
#pragma unroll
                    for (int r = 0; r < 4; r++) red[mb][4 * lq + r][l16] = d[r];
                }
                __syncthreads();
                if (jpart == 0) {
#pragma unroll
                    for (int r = 0; r < 4; r++) d[r] += red[mb][4 * lq + r][l16];
                }
            }
            if (jpart == 0) {
                const int m = m0 + 16 * mb + l16;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int k = 16 * kb + 4 * lq + r;
                    if (k < K && m < M) dg[(size_t)k * M + m] = d[r];
                }
            }
        }
    }
    if (store_part) {
        float* pg = part + (size_t)blockIdx.y * part_stride + (size_t)split * K * J;
        if constexpr (KP == 32) {
#pragma unroll
            for (int y = 0; y < NB; y++) {
                const int j = j_begin + 32 * (NB * wave + y) + l32;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int k = 8 * (r >> 2) + 4 * lk + (r & 3);
                    if (k < K && j < J) pg[(size_t)k * J + j] = gw_acc[y][r];
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < 2 * NB; b++) {
                const int j = j_begin + 32 * NB * wave + 16 * b + l16;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int k = 4 * lq + r;
                    if (k < K && j < J) pg[(size_t)k * J + j] = gw_acc4[b][r];
                }
            }
        }
    }
}

// The fused kernel on the bf16 matrix cores, for K <= 16 members and more than 128 rails.  The fp32
// MFMAs of k_bwd_small_k run on the vector ALU's multipliers: while one executes, no wave of the SIMD
// issues vector instructions, and the kernel's time is the sum of its MFMA and vector work.  The bf16
// MFMAs have a pipe of their own.  Here every operand is split into three bf16 terms as in
// k_gemm_split (six term products per product, fp32 accumulation): the weights once per workgroup,
// col once per tile, E once per element (eleven vector instructions per pair), and all three
// products take 72 bf16 MFMAs per wave and tile (1152 cycles of the matrix pipe, beside the vector
// work) where the fp32 kernel takes 80 fp32 ones (3072 cycles of the vector pipe).
//   first product   32x32x16: A = col[m][k] (csz), B = wcat[k][j] (registers)
//   weight gradient 16x16x32: A = col[k][m] (csg), B = E[m][j] read from E^T[j][m]: 8 consecutive m
//   input gradient  16x16x32: A = wd[k][j] (registers), B = E[m][j] for 8 consecutive j: eight 2-byte
//                   reads down a column of E^T (rows of kBfEw words keep them free of bank conflicts)
// Same grid, arguments, tiles and outputs as k_bwd_small_k<8, 2, DX>.
constexpr int kBfEw = 18;  // words per row of E^T: 32 bf16 and padding
constexpr int kBfCw = 20;  // words per row of col[k][m]: 16-byte aligned rows

template <int NW, bool DX>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(NW == 8 ? 4 : 3))) void k_bwd_small_k_bf16(
    const float* __restrict__ x, const float* __restrict__ wcat, const float* __restrict__ gtt,
    const int* __restrict__ base, const int* __restrict__ arow, const int* __restrict__ bcol, float* __restrict__ part,
    float* __restrict__ dcol, Groups G, int g0, int M, int w_in, int h_in, int c_out, int jblocks, int splits,
    int store_part, int gt_blocks, int gt_dedupe, size_t w_stride, size_t part_stride, size_t dcol_stride,
    size_t dcol_slice)
{
    constexpr int KP = 16, TM = kFusedTile, JW = 32 * NW, EW = kBfEw, CW = kBfCw, NT = 64 * NW;
    constexpr int JPARTS = NW / 2;   // waves that share one 16 x 16 block of dcol and split j
    constexpr int GP = 256 / NT > 1 ? 256 / NT : 1;  // member pairs gathered per thread (256 (position, pair) slots)
    // col of two tiles in turn: the next tile's is written while this tile's products run
    __shared__ __attribute__((aligned(16))) uint4 csz[2][3][2][TM];      // first product: (term, k half, m) -> 8 bf16 along k
    __shared__ __attribute__((aligned(16))) unsigned csg[2][3][KP][CW];  // weight gradient: [term][k][m], two m per word
    __shared__ __attribute__((aligned(16))) unsigned est[3][JW][EW];  // E^T: [term][j][m], two m per word
    __shared__ float red[JPARTS > 1 ? JPARTS - 1 : 1][2][16][17];     // the other j parts' partial dcol blocks
    const int K = G.n_members, J = 2 * c_out;
    const int g = g0 + blockIdx.y;
    const int split = blockIdx.x / jblocks, jblock = blockIdx.x - split * jblocks;
    const int j_begin = jblock * JW;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int l32 = lane & 31, lk = lane >> 5, l16 = lane & 15, lq = lane >> 4;
    // smallest terms first; 0 = hi, 1 = mid, 2 = lo
    constexpr int ta[6] = {2, 0, 1, 1, 0, 0}, tb[6] = {0, 2, 1, 0, 1, 0};

    // this group's wcat[k][j_begin .. j_begin + JW) through LDS (the space of est); zero outside the problem
    constexpr int WLD = JW + 1;
    float* wl = (float*)&est[0][0][0];
    {
        const float* wg = wcat + (size_t)blockIdx.y * w_stride;
        for (int e = threadIdx.x; e < KP * JW; e += NT) {
            const int k = e / JW, jl = e - k * JW, j = j_begin + jl;
            const bool ok = k < K && j < J;
            const float v = wg[ok ? (size_t)k * J + j : 0];
            wl[k * WLD + jl] = ok ? v : 0.0f;
        }
    }
    __syncthreads();
    // first product, B operand: lane -> column 32 wave + l32, k = 8 lk .. + 7
    bf16x8 wz[3];
    {
        unsigned h[4], m[4], l[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const float* src = wl + (8 * lk + 2 * c) * WLD + 32 * wave + l32;
            split3(src[0], src[WLD], h[c], m[c], l[c]);
        }
        wz[0] = __builtin_bit_cast(bf16x8, make_uint4(h[0], h[1], h[2], h[3]));
        wz[1] = __builtin_bit_cast(bf16x8, make_uint4(m[0], m[1], m[2], m[3]));
        wz[2] = __builtin_bit_cast(bf16x8, make_uint4(l[0], l[1], l[2], l[3]));
    }
    // input gradient: wave -> (position block mb, j part jpart of 64 columns); A operand of step st: wd[j][k = l16] for
    // j = jd0 + 32 st + 8 lq .. + 7, which is wcat[k][j] with the negative rail (j >= c_out) negated
    const int mb = wave & 1, jpart = wave >> 1;
    const int jd0 = jpart * 64;
    bf16x8 wdr[DX ? 2 : 1][3];
    if (DX) {
#pragma unroll
        for (int st = 0; st < 2; st++) {
            unsigned h[4], m[4], l[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int jl = jd0 + 32 * st + 8 * lq + 2 * c;
                float v0 = wl[l16 * WLD + jl], v1 = wl[l16 * WLD + jl + 1];
                if (j_begin + jl >= c_out) v0 = -v0;
                if (j_begin + jl + 1 >= c_out) v1 = -v1;
                split3(v0, v1, h[c], m[c], l[c]);
            }
            wdr[st][0] = __builtin_bit_cast(bf16x8, make_uint4(h[0], h[1], h[2], h[3]));
            wdr[st][1] = __builtin_bit_cast(bf16x8, make_uint4(m[0], m[1], m[2], m[3]));
            wdr[st][2] = __builtin_bit_cast(bf16x8, make_uint4(l[0], l[1], l[2], l[3]));
        }
    }
    // (the tile loop's first barriers come before anything is written to est)

    // im2col gather: 256 slots (position t & 31 of the tile, member pair t >> 5: members 2 pair and 2 pair + 1),
    // taken by the first four waves, or GP per thread in a smaller workgroup
    const int ml = threadIdx.x & 31;
    const bool gathers = threadIdx.x < 256;
    int kg[GP];
    int g_off[GP][2], g_u[GP][2], g_v[GP][2];
    bool g_ok[GP][2];
#pragma unroll
    for (int gp = 0; gp < GP; gp++) {
        kg[gp] = ((threadIdx.x >> 5) + gp * (NT / 32)) & 7;
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int k = 2 * kg[gp] + q;
            const Member e = member_of(G, g, k < K ? k : 0);
            g_ok[gp][q] = gathers && k < K && e.ok;
            g_off[gp][q] = (e.ci * w_in + e.u) * h_in + e.v;
            g_u[gp][q] = e.u;
            g_v[gp][q] = e.v;
        }
    }
    // this lane's 16 values of the wave's 32 x 32 block of the upstream gradient: offset in tile `split`, and
    // the distance to the next tile of this workgroup
    size_t g_at;
    {
        const int j0 = j_begin + 32 * wave;
        int blk = gt_dedupe ? (j0 >= c_out ? j0 - c_out : j0) >> 5 : j0 >> 5;
        if (j0 >= J) blk = 0;  // columns outside the problem: any finite values will do
        g_at = ((size_t)split * gt_blocks + blk) * 1024 + lane * 16;
    }
    const size_t g_step = (size_t)splits * gt_blocks * 1024;

    floatx4 gw_acc4[2];
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
        for (int r = 0; r < 4; r++) gw_acc4[b][r] = 0.0f;

    float* dg = dcol + (size_t)jblock * dcol_slice + (size_t)blockIdx.y * dcol_stride;
    const int n_tiles = (M + TM - 1) / TM;
    // The gather runs a tile ahead and its table entries two: a tile's columns of x are asked for at the
    // top of the tile before and its table entries at the top of the one before that, so that no tile
    // waits for two dependent loads in a row.
    struct Where {
        int r0, c0, b0;
        bool ok;
    };
    auto where = [&](int tile) {
        Where p;
        p.ok = gathers && tile < n_tiles && tile * TM + ml < M;
        const int mc = p.ok ? tile * TM + ml : 0;
        p.r0 = arow[mc];
        p.c0 = bcol[mc];
        p.b0 = base[mc];
        return p;
    };
    auto fetch = [&](const Where& p, float (&v)[GP][2], bool (&ok)[GP][2]) {
#pragma unroll
        for (int gp = 0; gp < GP; gp++)
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const int rr = p.r0 + g_u[gp][q], cc = p.c0 + g_v[gp][q];
                ok[gp][q] = p.ok && g_ok[gp][q] && cc >= 0 && cc < h_in && rr >= 0 && rr < w_in;
                v[gp][q] = x[ok[gp][q] ? p.b0 + g_off[gp][q] : 0];
            }
    };
    float x_next[GP][2], x_after[GP][2];
    bool ok_next[GP][2], ok_after[GP][2];
    Where w_after;
    auto commit = [&](int buf, const float (&v)[GP][2], const bool (&ok)[GP][2]) {
#pragma unroll
        for (int gp = 0; gp < GP; gp++) {
            unsigned t3[3];
            split3(ok[gp][0] ? v[gp][0] : 0.0f, ok[gp][1] ? v[gp][1] : 0.0f, t3[0], t3[1], t3[2]);
#pragma unroll
            for (int t = 0; t < 3; t++) {
                ((unsigned*)&csz[buf][t][kg[gp] >> 2][ml])[kg[gp] & 3] = t3[t];
                ((unsigned short*)&csg[buf][t][2 * kg[gp]][0])[ml] = (unsigned short)t3[t];
                ((unsigned short*)&csg[buf][t][2 * kg[gp] + 1][0])[ml] = (unsigned short)(t3[t] >> 16);
            }
        }
    };
    {
        const Where w0 = where(split);
        fetch(w0, x_next, ok_next);
        if (gathers) commit(0, x_next, ok_next);
        const Where w1 = where(split + splits);
        fetch(w1, x_next, ok_next);
        w_after = where(split + 2 * splits);
    }
    __syncthreads();  // the first tile's col is in place, and every wave has taken its weights out of est's space
    int buf = 0;
    for (int tile = split; tile < n_tiles; tile += splits, buf ^= 1) {
        const int m0 = tile * TM;
        float4 gv[4];
#pragma unroll
        for (int q = 0; q < 4; q++) gv[q] = ((const float4*)(gtt + g_at))[q];
        g_at += g_step;
        fetch(w_after, x_after, ok_after);
        w_after = where(tile + 3 * splits);
        {
            // Z[m][j] = sum_k col[k][m] * wcat[k][j] for the wave's 32 x 32 block; then E^T[j][m] =
            // g[m][co] * exp(-Z), split into its terms: register r is position 8 (r / 4) + 4 lk + r % 4
            bf16x8 az[3];
#pragma unroll
            for (int t = 0; t < 3; t++) az[t] = __builtin_bit_cast(bf16x8, csz[buf][t][lk][l32]);
            floatx16 z;
#pragma unroll
            for (int r = 0; r < 16; r++) z[r] = 0.0f;
#pragma unroll
            for (int t = 0; t < 6; t++) z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(az[ta[t]], wz[tb[t]], z, 0, 0, 0);
            const int j = 32 * wave + l32;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float e0 = gv[q].x * exp_neg(z[4 * q + 0]), e1 = gv[q].y * exp_neg(z[4 * q + 1]);
                const float e2 = gv[q].z * exp_neg(z[4 * q + 2]), e3 = gv[q].w * exp_neg(z[4 * q + 3]);
                unsigned h0, m0w, l0, h1, m1w, l1;
                split3(e0, e1, h0, m0w, l0);
                split3(e2, e3, h1, m1w, l1);
                *(uint2*)&est[0][j][4 * q + 2 * lk] = make_uint2(h0, h1);
                *(uint2*)&est[1][j][4 * q + 2 * lk] = make_uint2(m0w, m1w);
                *(uint2*)&est[2][j][4 * q + 2 * lk] = make_uint2(l0, l1);
            }
        }
        __syncthreads();
        {
            // Gw[k][j] += sum_m col[k][m] * E[m][j]: two 16-column blocks of the wave, lane -> m = 8 lq .. + 7
            bf16x8 ag[3];
#pragma unroll
            for (int t = 0; t < 3; t++) ag[t] = __builtin_bit_cast(bf16x8, *(const uint4*)&csg[buf][t][l16][4 * lq]);
            bf16x8 bg[2][3];
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int t = 0; t < 3; t++) {
                    const unsigned* row = &est[t][32 * wave + 16 * b + l16][4 * lq];
                    const uint2 p0 = *(const uint2*)row, p1 = *(const uint2*)(row + 2);
                    bg[b][t] = __builtin_bit_cast(bf16x8, make_uint4(p0.x, p0.y, p1.x, p1.y));
                }
#pragma unroll
            for (int t = 0; t < 6; t++)
#pragma unroll
                for (int b = 0; b < 2; b++)
                    gw_acc4[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ag[ta[t]], bg[b][tb[t]], gw_acc4[b], 0, 0, 0);
        }
        // the next tile's col, into the buffer whose readers finished before the last barrier
        if (gathers) commit(buf ^ 1, x_next, ok_next);
        floatx4 d[2];
        if (DX) {
            // dcol[k][m] = sum_j wd[j][k] * E[m][j]: one 16 x 16 block per wave over its quarter of j, lane ->
            // position 16 mb + l16, j = jd0 + 32 st + 8 lq .. + 7; the two steps in accumulators of their own
            const unsigned short* eh = (const unsigned short*)&est[0][jd0 + 8 * lq][0] + 16 * mb + l16;
            bf16x8 bd[2][3];
#pragma unroll
            for (int st = 0; st < 2; st++)
#pragma unroll
                for (int t = 0; t < 3; t++) {
                    unsigned wv[4];
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const unsigned short* pe = eh + ((t * JW + 32 * st + 2 * c) * EW) * 2;
                        wv[c] = (unsigned)pe[0] | ((unsigned)pe[2 * EW] << 16);
                    }
                    bd[st][t] = __builtin_bit_cast(bf16x8, make_uint4(wv[0], wv[1], wv[2], wv[3]));
                }
#pragma unroll
            for (int st = 0; st < 2; st++)
#pragma unroll
                for (int r = 0; r < 4; r++) d[st][r] = 0.0f;
#pragma unroll
            for (int t = 0; t < 6; t++)
#pragma unroll
                for (int st = 0; st < 2; st++)
                    d[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wdr[st][ta[t]], bd[st][tb[t]], d[st], 0, 0, 0);
            if (JPARTS > 1 && jpart > 0) {
#pragma unroll
                for (int r = 0; r < 4; r++) red[jpart - 1][mb][4 * lq + r][l16] = d[0][r] + d[1][r];
            }
        }
        // every wave has read this tile's E and col, and written the next tile's col and its share of red
        __syncthreads();
        if (DX && jpart == 0) {
            const int m = m0 + 16 * mb + l16;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int k = 4 * lq + r;
                float sum = d[0][r] + d[1][r];
#pragma unroll
                for (int jp = 1; jp < JPARTS; jp++) sum += red[jp - 1][mb][k][l16];
                if (k < K && m < M) dg[(size_t)k * M + m] = sum;
            }
        }
#pragma unroll
        for (int gp = 0; gp < GP; gp++)
#pragma unroll
            for (int q = 0; q < 2; q++) {
                x_next[gp][q] = x_after[gp][q];
                ok_next[gp][q] = ok_after[gp][q];
            }
    }
    if (store_part) {
        float* pg = part + (size_t)blockIdx.y * part_stride + (size_t)split * K * J;
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int j = j_begin + 32 * wave + 16 * b + l16;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int k = 4 * lq + r;
                if (k < K && j < J) pg[(size_t)k * J + j] = gw_acc4[b][r];
            }
        }
    }
}

int grid1d(long long total)
{
    long long blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    return (int)(blocks < 1 ? 1 : blocks);
}

// VA: the A operand is a view of the shifted input planes (GemmParams::a_rows); the caller has checked that
// its rows and chunks are 16-byte aligned.
// Whether a product of views takes the eight-wave kernel, and with which NX (0: no): whole tiles of 64 NX x 256,
// whole chunks in every split, no empty split, an aligned B where B is read along k, and tiles for at least three
// quarters of the CUs (the callers have checked the views' alignment).
inline int big_tile_nx(const GemmParams& q, int batch, bool b_along_k)
{
    const int nx = big_rows(q.I) / 64;
    const bool b_ok = !b_along_k || (q.ldb % 4 == 0 && ((uintptr_t)q.b & 15) == 0 && q.b_batch_stride % 4 == 0);
    const bool ok = nx && q.J % kBigJ == 0 && q.K % kChunk == 0 && q.k_per_split % kChunk == 0 && b_ok &&
                    (long long)(q.splits - 1) * q.k_per_split < q.K &&
                    (long long)(q.I / (64 * nx)) * (q.J / kBigJ) * q.splits * batch >= 3 * kBigWorkgroups / 4;
    return ok ? nx : 0;
}

// Tile extents of the 128 x 128 kernel.  A dimension of at most 192 whose last (or only) 128-tile would be at
// most half full takes tiles of 64: the 2 x 2 wave arrangement would leave half of the waves of such a tile
// without work (one dimension only, j first).
inline void split_tile_extents(int I, int J, int& tile_i, int& tile_j)
{
    auto half_tiles = [](int n) { return n <= 3 * kTile / 2 && (n - 1) % kTile < kTile / 2; };
    tile_j = half_tiles(J) ? kTile / 2 : kTile;
    tile_i = tile_j == kTile && half_tiles(I) ? kTile / 2 : kTile;
}
// its tiles are all whole: what the epilogue that reads the upstream gradient in the caller's layout asks for
inline bool split_tiles_whole(int I, int J)
{
    int ti, tj;
    split_tile_extents(I, J, ti, tj);
    return I % ti == 0 && J % tj == 0;
}

template <bool AK, bool BK, int EPI, bool VA = false, bool VB = false>
int launch_gemm(const GemmParams& q0, int batch, hipStream_t s)
{
    GemmParams q = q0;
    if constexpr (VA || VB) {
        const int nx = big_tile_nx(q, batch, !VB && !BK);
        // rows of 128: two chunks per trip where the chunks pair up
        const bool kc2 = nx == 2 && q.K % (2 * kChunk) == 0 && q.k_per_split % (2 * kChunk) == 0;
        if (nx) {
            q.tile_i = 64 * nx;
            q.tile_j = kBigJ;
            q.ni = q.I / q.tile_i;
            q.nj = q.J / q.tile_j;
            q.nz = q.splits * batch;
            if ((long long)q.ni * q.nj <= 16) {
                q.cluster_of = 2;
                q.cluster = q.ni * q.nj;
            } else if (q.nj <= q.ni) {
                q.cluster_of = 0;
                q.cluster = q.nj;
            } else {
                q.cluster_of = 1;
                q.cluster = q.ni;
            }
            const long long n_wg = (long long)q.ni * q.nj * q.nz;
            if (n_wg > 0x7fffffffLL) return GEO_SC_ERR_UNSUPPORTED;
            const dim3 grid((unsigned)std::min<long long>(n_wg, kBigWorkgroups));
            auto launch = [&](auto epi) {
                constexpr int E = decltype(epi)::value;
                if (nx == 4)
                    hipLaunchKernelGGL((k_gemm_big<AK, BK, E, VA, VB, 4>), grid, dim3(512), 0, s, q);
                else if (nx == 3)
                    hipLaunchKernelGGL((k_gemm_big<AK, BK, E, VA, VB, 3>), grid, dim3(512), 0, s, q);
                else if (kc2)
                    hipLaunchKernelGGL((k_gemm_big<AK, BK, E, VA, VB, 2, 2>), grid, dim3(512), 0, s, q);
                else
                    hipLaunchKernelGGL((k_gemm_big<AK, BK, E, VA, VB, 2>), grid, dim3(512), 0, s, q);
            };
            if constexpr (EPI == EPI_EXP_TIMES_G) {
                if (q.g_planes)
                    launch(std::integral_constant<int, EPI_EXP_TIMES_G_PLANES>());
                else
                    launch(std::integral_constant<int, EPI>());
            } else {
                launch(std::integral_constant<int, EPI>());
            }
            return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
        }
    }
    // the gradient in the caller's layout: views with whole tiles only (the caller decides with big_tile_nx and
    // split_tiles_whole)
    if (EPI == EPI_EXP_TIMES_G && q.g_planes && !(VA && split_tiles_whole(q.I, q.J))) return GEO_SC_ERR_UNSUPPORTED;
    split_tile_extents(q.I, q.J, q.tile_i, q.tile_j);
    q.ni = (q.I + q.tile_i - 1) / q.tile_i;
    q.nj = (q.J + q.tile_j - 1) / q.tile_j;
    q.nz = q.splits * batch;
    if ((long long)q.ni * q.nj <= 16) {
        q.cluster_of = 2;
        q.cluster = q.ni * q.nj;
    } else if (q.nj <= q.ni) {
        q.cluster_of = 0;
        q.cluster = q.nj;
    } else {
        q.cluster_of = 1;
        q.cluster = q.ni;
    }
    const long long n_groups = (long long)q.ni * q.nj * q.nz;
    if (n_groups > 0x7fffffffLL) return GEO_SC_ERR_UNSUPPORTED;
    dim3 grid((unsigned)n_groups);
    // The split kernel reads a K-major operand with dword loads and an I-major one with float4 along k:
    // every row start and every chunk start of the latter must lie on a 16-byte boundary.
    auto rows_aligned = [&](const float* base, long long ld, long long batch_stride) {
        return ld % 4 == 0 && ((uintptr_t)base & 15) == 0 && batch_stride % 4 == 0 && q.k_per_split % 4 == 0;
    };
    const bool a_vec = VA || AK || rows_aligned(q.a, q.lda, q.a_batch_stride);
    const bool b_vec = BK || rows_aligned(q.b, q.ldb, q.b_batch_stride);
    if constexpr (VB) {
        // (the caller has checked the view's alignment: rows of E and the runs of eight columns)
        hipLaunchKernelGGL((k_gemm_split<AK, BK, EPI, false, true>), grid, dim3(256), 0, s, q);
    } else if constexpr (VA) {
        if (!b_vec) return GEO_SC_ERR_UNSUPPORTED;
        if constexpr (EPI == EPI_EXP_TIMES_G) {
            if (q.g_planes)
                hipLaunchKernelGGL((k_gemm_split<AK, BK, EPI_EXP_TIMES_G_PLANES, true>), grid, dim3(256), 0, s, q);
            else
                hipLaunchKernelGGL((k_gemm_split<AK, BK, EPI, true>), grid, dim3(256), 0, s, q);
        } else {
            hipLaunchKernelGGL((k_gemm_split<AK, BK, EPI, true>), grid, dim3(256), 0, s, q);
        }
    } else if constexpr (AK && BK) {
        hipLaunchKernelGGL((k_gemm_split<AK, BK, EPI>), grid, dim3(256), 0, s, q);
    } else {
        if (a_vec && b_vec)
            hipLaunchKernelGGL((k_gemm_split<AK, BK, EPI>), grid, dim3(256), 0, s, q);
        else
            hipLaunchKernelGGL((k_gemm_f32<AK, BK, EPI>), grid, dim3(256), 0, s, q);
    }
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct BwdLayout {
    long long m_total;
    int splits, m_per_split;
    Groups G;
    bool fused_k;        // OR groups of at most 32 members: whole backward in one kernel, no col / E scratch
    int fused_jw;        // columns of E per workgroup of that kernel
    int fused_jblocks;   // its column blocks: each writes a dcol slice of its own
    int fused_splits;    // its workgroups per add group and column block
    int gt_dedupe;       // its upstream-gradient tiles serve both rails (c_out a multiple of 32)
    int gt_blocks;       // 32-column blocks of those tiles
    int rows_per_chunk;  // add groups processed by one round of launches
    int dcol_slices;     // partial dcol arrays per round (column blocks of the fused kernel), rows_per_chunk * col_v apart
    bool dx_rows;        // the input-gradient GEMM sums the kernel rows itself (E read as a view shifted by image rows)
    bool dx_taps;        // it sums all kernel taps and writes dL/dx itself (E read as a view shifted by rows and columns)
    size_t off_zero;     // a block of zeros for that view
    bool view_col;       // the GEMMs read col as a view of the shifted input planes (k_shift_planes) kept in col's space
    int view_k_pad;      // entries per group of the view's row table
    size_t off_rows;     // the row table
    size_t col_v, e_v, part_v, w_v;  // floats per add group of each scratch array
    size_t off_col, off_e, off_dcol, off_part, off_wcat, off_wd, off_pos, off_gt, bytes;
};

// floats of the shifted input planes (one per kernel column and channel, over the padded rows and the
// output columns) including the run behind the last plane that a shifted row may touch
size_t view_floats(const Geometry& g)
{
    return (size_t)g.h_k * g.c_in * g.n * (g.w_in + 2 * g.pad_w) * g.ho + (size_t)g.w_k * g.ho;
}

BwdLayout bwd_layout(const Geometry& g, int groups_per_round)
{
    BwdLayout b;
    b.m_total = (long long)g.n * g.wo * g.ho;
    b.G.mode = g.mode;
    b.G.c_in = g.c_in;
    b.G.w_k = g.w_k;
    b.G.h_k = g.h_k;
    b.G.zu = g.z_unit;
    if (g.mode == GEO_SC_ACC_Z) {
        b.G.n_groups = g.c_in;
        b.G.n_members = g.w_k * g.h_k;
    } else if (g.mode == GEO_SC_ACC_FULL) {
        b.G.n_groups = 1;
        b.G.n_members = g.k_or * g.h_k;
    } else if (g.mode == GEO_SC_ACC_YZ) {
        b.G.n_groups = g.add_outer * g.h_k;
        b.G.n_members = g.z_unit * g.w_k;
    } else {
        b.G.n_groups = g.h_k;
        b.G.n_members = g.k_or;
    }
    const int K = b.G.n_members;
    b.fused_k = K <= kFusedK;
    // the bf16 kernel (at most 16 members) comes with 2, 4 or 8 waves of 32 columns, the fp32 one with 128 or 256 columns
    b.fused_jw = 2 * g.c_out <= 64 && K <= 16 ? 64 : 2 * g.c_out <= 128 ? 128 : 256;
    b.fused_jblocks = (2 * g.c_out + b.fused_jw - 1) / b.fused_jw;
    b.gt_dedupe = g.c_out % 32 == 0;
    b.gt_blocks = b.gt_dedupe ? g.c_out / 32 : (2 * g.c_out + 31) / 32;
    {
        // about eight workgroups per CU in all, each looping over its share of the tiles
        const long long n_tiles = (b.m_total + kFusedTile - 1) / kFusedTile;
        long long want = 2048 / ((long long)b.G.n_groups * b.fused_jblocks);
        if (want > n_tiles) want = n_tiles;
        if (want > 65535) want = 65535;
        b.fused_splits = (int)(want < 1 ? 1 : want);
    }
    // split the m-reduction of the weight gradient so that all groups' tiles together make about one
    // round of workgroups: three per CU for the 128 x 128 kernel (more splits only add partial sums to write
    // and reduce; C3: 0.85 ms with two rounds, 0.82 with one, 0.85 with a third of one), one per CU where the
    // eight-wave kernel will take the product (the shapes that read col as a view, with whole tiles)
    const bool quads = g.ho % 4 == 0 && g.h_in % 4 == 0 && (g.wo * g.ho) % kChunk == 0 && g.c_out % 2 == 0;
    const int big_i = !b.fused_k && quads && (2 * g.c_out) % kBigJ == 0 ? big_rows(K) : 0;
    const long long tiles = big_i ? (long long)(K / big_i) * (2 * g.c_out / kBigJ)
                                  : (long long)((K + kTile - 1) / kTile) * ((2 * g.c_out + kTile - 1) / kTile);
    long long want = (big_i ? kBigWorkgroups : 768) / (tiles * b.G.n_groups);
    if (want < 1) want = 1;
    long long per = (b.m_total + want - 1) / want;
    per = (per + kChunk - 1) / kChunk * kChunk;
    if (per < 256) per = 256;
    b.m_per_split = (int)(per > 0x7fffffffLL ? 0x7fffffffLL : per);
    b.splits = (int)((b.m_total + b.m_per_split - 1) / b.m_per_split);
    // per-row scratch, each row's part padded to 64 floats so that float4 staging stays aligned
    auto pad64 = [](size_t v) { return (v + 63) & ~(size_t)63; };
    b.col_v = pad64((size_t)b.m_total * K);
    b.e_v = pad64((size_t)b.m_total * 2 * g.c_out);
    b.part_v = pad64((size_t)(b.fused_k && b.fused_splits > b.splits ? b.fused_splits : b.splits) * K * 2 * g.c_out);
    b.w_v = pad64((size_t)K * 2 * g.c_out);
    // the fused kernel needs neither col nor E
    const size_t col_alloc = b.fused_k ? 0 : b.col_v, e_alloc = b.fused_k ? 0 : b.e_v;
    b.dcol_slices = b.fused_k ? b.fused_jblocks : 1;
    // all groups in one round of launches unless that needs more than ~3 GB of scratch
    const size_t per_row = sizeof(float) * (col_alloc + b.dcol_slices * b.col_v + e_alloc + b.part_v + 2 * b.w_v);
    size_t rows = ((size_t)3 << 30) / per_row;
    if (rows < 1) rows = 1;
    if (rows > (size_t)b.G.n_groups) rows = b.G.n_groups;
    // the caller's cap on the add groups per round (less scratch, more launches)
    if (groups_per_round >= 1 && (size_t)groups_per_round < rows) rows = (size_t)groups_per_round;
    if (rows * b.splits > 65535) rows = 65535 / b.splits;  // grid.z = rows * splits
    if (rows < 1) rows = 1;
    b.rows_per_chunk = (int)rows;
    // col as a view: whole quads in every row on both sides, chunks of kChunk positions inside one item, an
    // even number of rails' worth of columns (16-byte aligned rows of E), every group in one round, members
    // that all exist, and offsets that fit the stagers' 32-bit position index
    b.view_k_pad = (K + kChunk - 1) / kChunk * kChunk;
    b.view_col = !b.fused_k && g.ho % 4 == 0 && g.h_in % 4 == 0 && (g.wo * g.ho) % kChunk == 0 && g.c_out % 2 == 0 &&
                 rows == (size_t)b.G.n_groups && !(g.mode == GEO_SC_ACC_YZ && g.c_in % g.z_unit != 0) &&
                 view_floats(g) <= rows * col_alloc &&
                 (long long)g.n * (g.w_in + 2 * g.pad_w) * g.ho + (long long)g.w_k * g.ho < 0x7fffffffLL;
    // the kernel rows summed inside the input-gradient GEMM: y accumulation (group = kernel column, members =
    // (channel, kernel row)), whole quads in the rows of input and output, whole chunks of rails, every group in
    // one round, and the per-column result inside dcol's space
    b.dx_rows = !b.fused_k && g.mode == GEO_SC_ACC_Y && g.ho % 4 == 0 && g.h_in % 4 == 0 && g.h_k <= 8 &&
                (2 * g.c_out) % kChunk == 0 && rows == (size_t)b.G.n_groups &&
                (size_t)g.h_k * g.c_in * g.n * g.w_in * g.ho <= rows * b.col_v &&
                (long long)g.n * g.w_in * g.ho < 0x7fffffffLL && (long long)g.w_k * 2 * g.c_out < 0x7fffffffLL;
    // all kernel taps summed inside that GEMM, which then writes dL/dx itself (no per-column results, no pass that
    // adds them): the same without the conditions of that pass, where the result alone has tiles for the GPU
    // (a product per kernel column has h_k times as many)
    {
        int ti, tj;
        const long long m2 = (long long)g.n * g.w_in * g.h_in;
        split_tile_extents(g.c_in, m2 > 0x7fffffffLL ? 0x7fffffff : (int)m2, ti, tj);
        const long long tiles = (long long)((g.c_in + ti - 1) / ti) * ((m2 + tj - 1) / tj);
        b.dx_taps = !b.fused_k && g.mode == GEO_SC_ACC_Y && (2 * g.c_out) % kChunk == 0 &&
                    rows == (size_t)b.G.n_groups && m2 < 0x7fff0000LL &&
                    (long long)g.w_k * g.h_k * 2 * g.c_out < 0x7fffffffLL && tiles >= 2 * kBigWorkgroups;
    }
    size_t o = 0;
    b.off_col = o;  o += align256(sizeof(float) * rows * col_alloc);
    b.off_e = o;    o += align256(sizeof(float) * rows * e_alloc);
    // (no per-group input gradients where the product over all taps writes dL/dx itself)
    b.off_dcol = o; o += b.dx_taps ? 0 : align256(sizeof(float) * rows * b.col_v * b.dcol_slices);
    b.off_part = o; o += align256(sizeof(float) * rows * b.part_v);
    b.off_wcat = o; o += align256(sizeof(float) * rows * b.w_v);
    b.off_wd = o;   o += align256(sizeof(float) * rows * b.w_v);
    b.off_pos = o;  o += 3 * align256(sizeof(int) * (size_t)b.m_total);
    {
        // [m][c_out], or the fused kernel's tiles of 32 positions x 32 columns
        const size_t tiled = (size_t)((b.m_total + kFusedTile - 1) / kFusedTile) * b.gt_blocks * 1024;
        const size_t plain = (size_t)b.m_total * g.c_out;
        b.off_gt = o;
        o += align256(sizeof(float) * (b.fused_k && tiled > plain ? tiled : plain));
    }
    b.off_rows = o;
    // (and behind it the entries that the eight-wave kernel reads ahead of the last chunk)
    o += align256(sizeof(long long) * ((size_t)b.G.n_groups * b.view_k_pad + 2 * kChunk + 8));
    b.off_zero = o;
    o += 256;
    b.bytes = o;
    return b;
}

}  // namespace

size_t backward_workspace_bytes(const Geometry& g, int groups_per_round) { return bwd_layout(g, groups_per_round).bytes; }

int launch_conv_backward(const Geometry& g, int groups_per_round, const float* x, const float* w, const float* gy,
                         float* gx, float* gw, void* workspace, size_t workspace_bytes, hipStream_t s)
{
    const BwdLayout L = bwd_layout(g, groups_per_round);  // once per call: sizes the check and the launches alike
    if (workspace_bytes < L.bytes) return GEO_SC_ERR_WORKSPACE;
    if (L.m_total > 0x7fffffffLL) return GEO_SC_ERR_INVALID_ARGUMENT;
    char* ws = (char*)workspace;
    float* col = (float*)(ws + L.off_col);
    float* e = (float*)(ws + L.off_e);
    float* dcol = (float*)(ws + L.off_dcol);
    float* part = (float*)(ws + L.off_part);
    float* wcat = (float*)(ws + L.off_wcat);
    float* wd = (float*)(ws + L.off_wd);
    const Groups& G = L.G;
    const int M = (int)L.m_total, K = G.n_members, J = 2 * g.c_out;
    const long long x_total = (long long)g.n * g.c_in * g.w_in * g.h_in;
    if (x_total > 0x7fffffffLL || K > 65535 * kIm2colMembers) return GEO_SC_ERR_UNSUPPORTED;
    if ((long long)g.n * g.c_out * g.wo * g.ho > 0x7fffffffLL) return GEO_SC_ERR_UNSUPPORTED;
    const size_t pos_stride = align256(sizeof(int) * (size_t)M) / sizeof(int);
    int* pos_base = (int*)(ws + L.off_pos);
    int* pos_arow = pos_base + pos_stride;
    int* pos_bcol = pos_arow + pos_stride;
    float* gt = (float*)(ws + L.off_gt);
    const int m_blocks = grid1d(M);
    // four elements per thread in im2col / col2im where rows of the input and of the output are whole quads
    const bool quad_rows = g.h_in % 4 == 0 && g.ho % 4 == 0;
    const bool im2col_v4 = quad_rows && ((uintptr_t)x & 15) == 0;
    const bool col2im_v4 = quad_rows && g.h_k <= 8 && gx && ((uintptr_t)gx & 15) == 0;
    const bool fused = L.fused_k;
    // col as a view of the shifted input planes (one round holds every group then)
    const bool view = L.view_col && ((uintptr_t)x & 15) == 0;
    // the position tables serve the gathers of im2col and of the fused kernels
    if (fused || !view)
        hipLaunchKernelGGL(k_position_table, dim3(m_blocks), dim3(256), 0, s, pos_base, pos_arow, pos_bcol, M,
                           g.c_in, g.c_out, g.w_in, g.h_in, g.pad_w, g.pad_h, g.wo, g.ho);
    // Where the first product reads col as a view and its tiles are whole (the eight-wave kernel in every round,
    // or the 128 x 128 kernel), its epilogue reads the upstream gradient as it is (items of whole 32-position
    // blocks, 16-byte aligned): no transposed copy.
    // (the 128 x 128 kernel with full-width tiles only: with tiles of 64 columns the strided loads cost what the
    // small transposed copy does)
    bool g_planes = !fused && view && (g.wo * g.ho) % 32 == 0 && ((uintptr_t)gy & 15) == 0;
    if (g_planes && !(split_tiles_whole(M, J) && J % kTile == 0)) {
        GemmParams t = {};
        t.I = M; t.J = J; t.K = K; t.splits = 1; t.k_per_split = K;
        for (int v0 = 0; v0 < G.n_groups; v0 += L.rows_per_chunk) {
            const int nv = G.n_groups - v0 < L.rows_per_chunk ? G.n_groups - v0 : L.rows_per_chunk;
            if (!big_tile_nx(t, nv, false)) g_planes = false;
        }
    }
    {
        const int npos = g.wo * g.ho;
        if (fused) {
            hipLaunchKernelGGL(k_tile_grad, dim3((M + kFusedTile - 1) / kFusedTile, L.gt_blocks), dim3(256), 0, s, gy, gt, M,
                               g.c_out, npos, L.gt_blocks, L.gt_dedupe);
        } else if (!g_planes) {
            if (g.n > 65535) return GEO_SC_ERR_UNSUPPORTED;  // grid.z of the transpose
            hipLaunchKernelGGL(k_transpose_grad, dim3((npos + 31) / 32, (g.c_out + 31) / 32, g.n), dim3(256), 0, s, gy, gt,
                               g.c_out, npos);
        }
    }
    int rc;
    if (fused) {
        if (!gx && !gw) return GEO_SC_OK;
        const int plane_blocks = (g.w_in * g.h_in + 255) / 256;
        const int n_planes = g.n * g.c_in;
        const int pb = plane_blocks > 64 ? 64 : plane_blocks;
        const int want = 256 * 16 / pb;
        const int ks = (K + 1) / 2;
        const int jw = L.fused_jw;
        const size_t slice = (size_t)L.rows_per_chunk * L.col_v;
        if ((long long)L.fused_splits * L.fused_jblocks > 0x7fffffffLL) return GEO_SC_ERR_UNSUPPORTED;
        for (int v0 = 0; v0 < G.n_groups; v0 += L.rows_per_chunk) {
            const int nv = G.n_groups - v0 < L.rows_per_chunk ? G.n_groups - v0 : L.rows_per_chunk;
            // channel blocks with a ragged end have members that do not exist: their zeros come from the plain kernel
            const bool ragged = G.mode == GEO_SC_ACC_YZ && g.c_in % G.zu != 0;
            const dim3 w_tiles((g.c_in * g.w_k * g.h_k + 31) / 32, (g.c_out + 31) / 32);
            if (ragged) {
                int wb = grid1d((long long)K * g.c_out);
                hipLaunchKernelGGL(k_weight_operands, dim3(wb > 256 ? 256 : wb, nv), dim3(256), 0, s, w, wcat, wd, v0,
                                   g.c_out, G, L.w_v);
            } else {
                hipLaunchKernelGGL(k_weight_cat_tiled, w_tiles, dim3(256), 0, s, w, wcat, v0, nv, g.c_out, G, L.w_v);
            }
            const dim3 grid(L.fused_splits * L.fused_jblocks, nv);
            {
#define GEO_SC_FUSED_K(KS, NB, DX)                                                                                     \
    hipLaunchKernelGGL((k_bwd_small_k<KS, NB, DX>), grid, dim3(256), 0, s, x, wcat, gt, pos_base, pos_arow,             \
                       pos_bcol, part, dcol, G, v0, M, g.w_in, g.h_in, g.c_out, L.fused_jblocks, L.fused_splits,        \
                       gw ? 1 : 0, L.gt_blocks, L.gt_dedupe, L.w_v, L.part_v, L.col_v, slice)
#define GEO_SC_FUSED_NB_DX(KS)                                                                                         \
    do {                                                                                                               \
        if (jw == 128) {                                                                                               \
            if (gx) GEO_SC_FUSED_K(KS, 1, true); else GEO_SC_FUSED_K(KS, 1, false);                                    \
        } else {                                                                                                       \
            if (gx) GEO_SC_FUSED_K(KS, 2, true); else GEO_SC_FUSED_K(KS, 2, false);                                    \
        }                                                                                                              \
    } while (0)
#define GEO_SC_FUSED_BF16(NW, DX)                                                                                      \
    hipLaunchKernelGGL((k_bwd_small_k_bf16<NW, DX>), grid, dim3(64 * NW), 0, s, x, wcat, gt, pos_base, pos_arow,        \
                       pos_bcol, part, dcol, G, v0, M, g.w_in, g.h_in, g.c_out, L.fused_jblocks, L.fused_splits,        \
                       gw ? 1 : 0, L.gt_blocks, L.gt_dedupe, L.w_v, L.part_v, L.col_v, slice)
                if (ks <= 8) {
                    if (jw == 64) {
                        if (gx) GEO_SC_FUSED_BF16(2, true); else GEO_SC_FUSED_BF16(2, false);
                    } else if (jw == 128) {
                        if (gx) GEO_SC_FUSED_BF16(4, true); else GEO_SC_FUSED_BF16(4, false);
                    } else {
                        if (gx) GEO_SC_FUSED_BF16(8, true); else GEO_SC_FUSED_BF16(8, false);
                    }
                }
                else if (ks <= 12) GEO_SC_FUSED_NB_DX(12);
                else GEO_SC_FUSED_NB_DX(16);
#undef GEO_SC_FUSED_BF16
#undef GEO_SC_FUSED_NB_DX
#undef GEO_SC_FUSED_K
            }
            if (gw) {
                // few partial sums (wide layers): coalesced tiles; many: the kernel that adds eight splits side by side
                if (L.fused_splits <= 4)
                    hipLaunchKernelGGL(k_reduce_wgrad_tiled, w_tiles, dim3(256), 0, s, part, w, gw, v0, nv, L.fused_splits,
                                       g.c_out, G, L.part_v);
                else
                    hipLaunchKernelGGL(k_reduce_wgrad, dim3((K * g.c_out + 31) / 32, nv), dim3(256), 0, s, part, w, gw, v0,
                                       L.fused_splits, g.c_out, G, L.part_v);
            }
            if (gx && L.dcol_slices > 1)
                hipLaunchKernelGGL(k_sum_slices, dim3(grid1d((long long)((size_t)nv * L.col_v / 4))), dim3(256), 0, s, dcol,
                                   (size_t)nv * L.col_v, L.dcol_slices, slice);
            if (gx && col2im_v4)
                hipLaunchKernelGGL(k_col2im_rows_v4, dim3(grid1d((long long)n_planes * (g.w_in * g.h_in / 4))), dim3(256), 0, s, dcol, gx,
                                   v0, nv, L.m_total, n_planes, G, g.w_in, g.h_in, g.pad_w, g.pad_h, g.wo, g.ho, L.col_v);
            else if (gx)
                hipLaunchKernelGGL(k_col2im_rows, dim3(n_planes < want ? n_planes : want, pb), dim3(256), 0, s, dcol, gx,
                                   v0, nv, L.m_total, n_planes, G, g.w_in, g.h_in, g.pad_w, g.pad_h, g.wo, g.ho, L.col_v);
        }
        return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
    }
    long long* view_rows = (long long*)(ws + L.off_rows);
    if (view) {
        const long long plane = (long long)g.n * (g.w_in + 2 * g.pad_w) * g.ho;
        const long long quads = (long long)g.h_k * g.c_in * plane / 4;
        hipLaunchKernelGGL(k_shift_planes, dim3(grid1d(quads)), dim3(256), 0, s, x, col, quads, g.n, g.c_in, g.w_in, g.h_in,
                           g.pad_w, g.pad_h, g.ho);
    }
    for (int v0 = 0; v0 < G.n_groups; v0 += L.rows_per_chunk) {
        const int nv = G.n_groups - v0 < L.rows_per_chunk ? G.n_groups - v0 : L.rows_per_chunk;
        if (view) {
            // nothing to copy
        } else if (im2col_v4) {
            const int q_blocks = grid1d(M / 4);
            hipLaunchKernelGGL(k_im2col_rows_v4,
                               dim3(q_blocks > 1024 ? 1024 : q_blocks, (K + kIm2colMembers - 1) / kIm2colMembers, nv),
                               dim3(256), 0, s, x, col, pos_base, pos_arow, pos_bcol, v0, M, G, g.w_in, g.h_in, L.col_v);
        } else {
            hipLaunchKernelGGL(k_im2col_rows,
                               dim3(m_blocks > 1024 ? 1024 : m_blocks, (K + kIm2colMembers - 1) / kIm2colMembers, nv),
                               dim3(256), 0, s, x, col, pos_base, pos_arow, pos_bcol, v0, M, G, g.w_in, g.h_in, L.col_v);
        }
        const bool dx_taps = gx && L.dx_taps;
        const bool dx_rows = dx_taps || (gx && L.dx_rows && ((uintptr_t)gx & 15) == 0);
        {
            // weight operands of the round's groups; with the first round the view's row table and the block of zeros
            PrepParams pp = {};
            pp.w = w; pp.wcat = wcat; pp.wd = wd; pp.g0 = v0; pp.c_out = g.c_out; pp.G = G; pp.g_stride = L.w_v;
            pp.dx_rows = dx_taps ? 2 : dx_rows ? 1 : 0;
            if (v0 == 0 && view) {
                pp.view_rows = view_rows; pp.view_groups = G.n_groups; pp.view_k_pad = L.view_k_pad; pp.ho = g.ho;
                pp.plane = (long long)g.n * (g.w_in + 2 * g.pad_w) * g.ho;
            }
            if (dx_rows) pp.zero = (float*)(ws + L.off_zero);
            long long work = (long long)K * g.c_out;
            if (dx_rows && (long long)g.w_k * J * g.c_in > work) work = (long long)g.w_k * J * g.c_in;
            if (pp.view_rows && (long long)G.n_groups * L.view_k_pad > work) work = (long long)G.n_groups * L.view_k_pad;
            const int wb = grid1d(work);
            hipLaunchKernelGGL(k_bwd_prep, dim3(wb > 256 ? 256 : wb, nv), dim3(256), 0, s, pp);
        }
        // E[v][m][j] = g * exp(-(col_v^T . wcat_v)), col stored [K][M]
        GemmParams q1 = {};
        q1.a = col; q1.b = wcat; q1.c = e;
        q1.I = M; q1.J = J; q1.K = K;
        q1.lda = M; q1.ldb = J; q1.ldc = J;
        q1.splits = 1; q1.k_per_split = K; q1.c_split_stride = 0;
        q1.a_batch_stride = (long long)L.col_v; q1.b_batch_stride = (long long)L.w_v;
        q1.c_batch_stride = (long long)L.e_v;
        q1.g = g_planes ? gy : gt; q1.g_planes = g_planes; q1.c_out = g.c_out; q1.npos = g.wo * g.ho;
        q1.a_rows = view_rows; q1.a_rows_batch = L.view_k_pad; q1.a_item = g.wo * g.ho; q1.a_skip = (g.w_k - 1) * g.ho;
        rc = view ? launch_gemm<true, true, EPI_EXP_TIMES_G, true>(q1, nv, s)
                  : launch_gemm<true, true, EPI_EXP_TIMES_G>(q1, nv, s);
        if (rc != GEO_SC_OK) return rc;
        if (gw) {
            // partial Gw[v][s][k][j] = sum_{m in split s} col_v[k][m] * E_v[m][j]
            GemmParams q2 = {};
            q2.a = col; q2.b = e; q2.c = part;
            q2.I = K; q2.J = J; q2.K = M;
            q2.lda = M; q2.ldb = J; q2.ldc = J;
            q2.splits = L.splits; q2.k_per_split = L.m_per_split; q2.c_split_stride = (long long)K * J;
            q2.a_batch_stride = (long long)L.col_v; q2.b_batch_stride = (long long)L.e_v;
            q2.c_batch_stride = (long long)L.part_v;
            q2.a_rows = view_rows; q2.a_rows_batch = L.view_k_pad; q2.a_item = g.wo * g.ho; q2.a_skip = (g.w_k - 1) * g.ho;
            rc = view ? launch_gemm<false, true, EPI_STORE, true>(q2, nv, s) : launch_gemm<false, true, EPI_STORE>(q2, nv, s);
            if (rc != GEO_SC_OK) return rc;
            hipLaunchKernelGGL(k_reduce_wgrad, dim3((K * g.c_out + 31) / 32, nv), dim3(256), 0, s, part, w, gw, v0,
                               L.splits, g.c_out, G, L.part_v);
        }
        if (!gx) continue;
        if (dx_taps) {
            // gx[n][ci][(p, c)] = sum_(u, v, j) wdx[(j, v, u)][ci] * E_v[(n, p + pad_w - u, c + pad_h - v)][j]: every
            // kernel tap summed inside one GEMM (w_k h_k times the k of the product per tap, one output instead of one
            // per tap, stored in the caller's layout); the operand wdx and the block of zeros come from k_bwd_prep
            float* zero = (float*)(ws + L.off_zero);
            const int k9 = g.w_k * g.h_k * J;
            const long long m2 = (long long)g.n * g.w_in * g.h_in;
            GemmParams q3 = {};
            q3.a = wd; q3.b = e; q3.c = gx;
            q3.I = g.c_in; q3.J = (int)m2; q3.K = k9;
            q3.lda = g.c_in; q3.ldb = J; q3.ldc = m2;
            q3.splits = 1; q3.k_per_split = k9; q3.c_split_stride = 0;
            q3.a_batch_stride = 0; q3.b_batch_stride = (long long)L.e_v; q3.c_batch_stride = 0;
            q3.sh_zero = zero; q3.sh_j = J; q3.sh_wo = g.wo; q3.sh_ho = g.ho; q3.sh_win = g.w_in; q3.sh_hin = g.h_in;
            q3.sh_pad = g.pad_w; q3.sh_padh = g.pad_h; q3.sh_wk = g.w_k; q3.sh_hk = g.h_k;
            q3.c_plane = g.w_in * g.h_in;
            if ((rc = launch_gemm<true, false, EPI_STORE_ITEMS, false, true>(q3, 1, s)) != GEO_SC_OK) return rc;
            continue;
        }
        if (dx_rows) {
            // d[v][ci][(n, p, b)] = sum_(u, j) wd_v[j][(ci, u)] * E_v[(n, p + pad - u, b)][j]: the kernel rows
            // summed inside the GEMM (three times the k of the product per (ci, u), a third of its rows and of
            // its output), then the kernel columns by k_shift_sum_v4; the operand wdx and the block of zeros
            // come from k_bwd_prep
            float* zero = (float*)(ws + L.off_zero);
            const int k3 = g.w_k * J;
            const long long m2 = (long long)g.n * g.w_in * g.ho;
            GemmParams q3 = {};
            q3.a = wd; q3.b = e; q3.c = dcol;
            q3.I = g.c_in; q3.J = (int)m2; q3.K = k3;
            q3.lda = g.c_in; q3.ldb = J; q3.ldc = m2;
            q3.splits = 1; q3.k_per_split = k3; q3.c_split_stride = 0;
            q3.a_batch_stride = (long long)L.w_v; q3.b_batch_stride = (long long)L.e_v;
            q3.c_batch_stride = (long long)g.c_in * m2;
            q3.sh_zero = zero; q3.sh_j = J; q3.sh_wo = g.wo; q3.sh_ho = g.ho; q3.sh_win = g.w_in; q3.sh_hin = g.ho;
            q3.sh_pad = g.pad_w; q3.sh_padh = 0; q3.sh_wk = g.w_k; q3.sh_hk = 1;
            if ((rc = launch_gemm<true, false, EPI_STORE, false, true>(q3, nv, s)) != GEO_SC_OK) return rc;
            const long long quads = (long long)g.n * g.c_in * g.w_in * g.h_in / 4;
            hipLaunchKernelGGL(k_shift_sum_v4, dim3(grid1d(quads)), dim3(256), 0, s, dcol, gx, quads, g.n, g.c_in, g.w_in,
                               g.h_in, g.h_k, g.pad_h, g.ho);
            continue;
        }
        // dcol[v][k][m] = sum_j wd_v[j][k] * E_v[m][j]
        GemmParams q3 = {};
        q3.a = wd; q3.b = e; q3.c = dcol;
        q3.I = K; q3.J = M; q3.K = J;
        q3.lda = K; q3.ldb = J; q3.ldc = M;
        q3.splits = 1; q3.k_per_split = J; q3.c_split_stride = 0;
        q3.a_batch_stride = (long long)L.w_v; q3.b_batch_stride = (long long)L.e_v;
        q3.c_batch_stride = (long long)L.col_v;
        if ((rc = launch_gemm<true, false, EPI_STORE>(q3, nv, s)) != GEO_SC_OK) return rc;
        const int plane_blocks = (g.w_in * g.h_in + 255) / 256;
        const int n_planes = g.n * g.c_in;
        const int pb = plane_blocks > 64 ? 64 : plane_blocks;
        const int want = 256 * 16 / pb;  // a few thousand blocks in all
        if (col2im_v4)
            hipLaunchKernelGGL(k_col2im_rows_v4, dim3(grid1d((long long)n_planes * (g.w_in * g.h_in / 4))), dim3(256), 0, s, dcol, gx, v0,
                               nv, L.m_total, n_planes, G, g.w_in, g.h_in, g.pad_w, g.pad_h, g.wo, g.ho, L.col_v);
        else
            hipLaunchKernelGGL(k_col2im_rows, dim3(n_planes < want ? n_planes : want, pb), dim3(256), 0, s, dcol, gx, v0,
                               nv, L.m_total, n_planes, G, g.w_in, g.h_in, g.pad_w, g.pad_h, g.wo, g.ho, L.col_v);
    }
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

}  // namespace geo_sc
