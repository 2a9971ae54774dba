// SC convolution forward: AND / OR / popcount over bit-packed streams (gfx950).
//
//   y[n,co,a,b] = sum_{v<H} sum_{p<P} ( popc( OR_{ci,u} A[n,p,ci,a+u,b+v] & WP[p,v,ci*W+u,co] )
//                                      - popc( OR_{ci,u} A[n,p,ci,a+u,b+v] & WN[p,v,ci*W+u,co] ) )
// (sc.cpp:12-259 with the im2col of sc.cpp:440-452 folded into the addressing).
//
// Mapping.  One wave of 64 lanes per workgroup.  Lanes run over output positions: lane
// slot = (item n, row group a/R, column b) flattened, so a wave may span items.  Every
// lane keeps R consecutive rows x 16 output channels x 2 rails of OR accumulators in
// VGPRs.  The 32 weight words of one (pack, kernel row, OR-group member, c_out tile) are
// the same for all lanes: they are read with scalar loads and enter v_and_or_b32 as its
// SGPR operand, so the inner loop is one VALU instruction per (activation word, weight
// word) pair.  A kernel row's popcounts are folded into int32 sums with v_bcnt_u32_b32.
// Consecutive workgroups take the c_out tiles of the same positions.
#include "sc_common.h"
#include <stdlib.h>

namespace geo_sc {

namespace {

struct FwdParams {
    const uint32_t* __restrict__ act;  // [n][P][c_in][wi][hi]
    const uint32_t* __restrict__ wgt;  // [P][h_k][k_or][n_cotile][2][16]
    int32_t* __restrict__ y;           // [n][c_out][wo][ho]
    int c_in, wi, hi, c_out, w_k, h_k, packs;
    int wo, ho, n_cotile;
    int row_groups;        // ceil(wo / R)
    long long slots;       // n * row_groups * ho
    unsigned act_plane;    // c_in * wi * hi
    int map;
};

// acc |= a & w with w wave-uniform: a single v_and_or_b32 whose first source is the SGPR.
// Written as an instruction because the compiler otherwise re-associates chains of these
// into v_and + v_and + v_or3 (three instructions per two pairs instead of two).
__device__ __forceinline__ void and_or(uint32_t& acc, uint32_t a, uint32_t w_uniform)
{
    asm("v_and_or_b32 %0, %1, %2, %0" : "+v"(acc) : "s"(w_uniform), "v"(a));
}

// R rows per lane, WK = kernel extent in dim 2 known at compile time (0: run-time extent,
// rows handled one at a time).
template <int R, int WK>
__global__ __launch_bounds__(64) void k_conv_fwd(FwdParams q)
{
    constexpr int C = kCoTile;
    int cot, mt;
    if (q.map == 0) {
        cot = blockIdx.x % q.n_cotile;
        mt = blockIdx.x / q.n_cotile;
    } else {
        // workgroup ids are dealt round-robin to the 8 XCDs: keep all c_out tiles of one
        // position tile on one XCD so that its L2 serves their common activation words
        const unsigned per = 8u * q.n_cotile;
        const unsigned grp = blockIdx.x / per, rem = blockIdx.x % per;
        mt = grp * 8 + (rem & 7);
        cot = rem >> 3;
    }
    const long long slot0 = (long long)mt * 64 + threadIdx.x;
    const bool live = slot0 < q.slots;
    const long long slot = live ? slot0 : 0;
    const int b = (int)(slot % q.ho);
    const long long t = slot / q.ho;
    const int a0 = (int)(t % q.row_groups) * R;
    const long long n = t / q.row_groups;

    constexpr int NROWS = WK > 0 ? R + WK - 1 : 1;
    // rows a0 .. a0+NROWS-1 of the padded item; rows past the end (partial last group) are
    // clamped: they only feed outputs that are never stored
    unsigned row_off[NROWS];
#pragma unroll
    for (int j = 0; j < NROWS; j++) {
        int row = a0 + j;
        row = row < q.wi ? row : q.wi - 1;
        row_off[j] = (unsigned)row * q.hi;
    }
    const uint32_t* act_n = q.act + (size_t)n * q.packs * q.act_plane + b;
    const unsigned ch_stride = (unsigned)q.wi * q.hi;
    const int k_or = q.c_in * q.w_k;
    const unsigned k_stride = (unsigned)q.n_cotile * 2 * C;

    int sum[R][C];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int c = 0; c < C; c++) sum[r][c] = 0;

    for (int p = 0; p < q.packs; p++) {
        for (int v = 0; v < q.h_k; v++) {
            uint32_t orp[R][C], orn[R][C];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int c = 0; c < C; c++) orp[r][c] = orn[r][c] = 0u;

            const uint32_t* ap = act_n + (size_t)p * q.act_plane + v;
            const uint32_t* wp = q.wgt + ((size_t)(p * q.h_k + v) * k_or * q.n_cotile + cot) * (2 * C);

            if constexpr (WK > 0) {
                // activation words are fetched one channel ahead of their use
                uint32_t aw[NROWS], an[NROWS];
#pragma unroll
                for (int j = 0; j < NROWS; j++) an[j] = ap[row_off[j]];
#pragma unroll 2
                for (int ci = 0; ci < q.c_in; ci++) {
#pragma unroll
                    for (int j = 0; j < NROWS; j++) aw[j] = an[j];
                    ap += (ci + 1 < q.c_in) ? ch_stride : 0u;
#pragma unroll
                    for (int j = 0; j < NROWS; j++) an[j] = ap[row_off[j]];
#pragma unroll
                    for (int u = 0; u < WK; u++) {
                        uint32_t wv[2 * C];
#pragma unroll
                        for (int c = 0; c < 2 * C; c++) wv[c] = wp[c];
#pragma unroll
                        for (int r = 0; r < R; r++)
#pragma unroll
                            for (int c = 0; c < C; c++) {
                                and_or(orp[r][c], aw[r + u], wv[c]);
                                and_or(orn[r][c], aw[r + u], wv[C + c]);
                            }
                        wp += k_stride;
                    }
                }
            } else {
                for (int ci = 0; ci < q.c_in; ci++) {
                    for (int u = 0; u < q.w_k; u++) {
                        uint32_t wv[2 * C];
#pragma unroll
                        for (int c = 0; c < 2 * C; c++) wv[c] = wp[c];
#pragma unroll
                        for (int r = 0; r < R; r++) {
                            int row = a0 + r + u;
                            row = row < q.wi ? row : q.wi - 1;
                            const uint32_t aw = ap[(unsigned)row * q.hi];
#pragma unroll
                            for (int c = 0; c < C; c++) {
                                and_or(orp[r][c], aw, wv[c]);
                                and_or(orn[r][c], aw, wv[C + c]);
                            }
                        }
                        wp += k_stride;
                    }
                    ap += ch_stride;
                }
            }
            // binary add across kernel rows and packs: v_bcnt_u32_b32 folds the add
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int c = 0; c < C; c++) sum[r][c] += __popc(orp[r][c]) - __popc(orn[r][c]);
        }
    }

    if (!live) return;
    const size_t out_plane = (size_t)q.wo * q.ho;
#pragma unroll
    for (int c = 0; c < C; c++) {
        const int co = cot * C + c;
        if (co >= q.c_out) break;
        int32_t* yo = q.y + ((size_t)n * q.c_out + co) * out_plane + (size_t)a0 * q.ho + b;
#pragma unroll
        for (int r = 0; r < R; r++)
            if (a0 + r < q.wo) yo[(size_t)r * q.ho] = sum[r][c];
    }
}

template <int R, int WK>
int launch(const Geometry& g, FwdParams q, hipStream_t s)
{
    q.row_groups = (g.wo + R - 1) / R;
    q.slots = (long long)g.n * q.row_groups * g.ho;
    const long long tiles = (q.slots + 63) / 64;
    long long blocks = tiles * g.n_cotile;
    const char* e = getenv("GEO_SC_MAP");
    q.map = e ? atoi(e) : 0;
    if (q.map) blocks = (tiles + 7) / 8 * 8 * g.n_cotile;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return GEO_SC_ERR_INVALID_ARGUMENT;
    hipLaunchKernelGGL((k_conv_fwd<R, WK>), dim3((unsigned)blocks), dim3(64), 0, s, q);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

}  // namespace

int launch_conv_forward(const Geometry& g, const uint32_t* act, const uint32_t* wgt, int32_t* y, hipStream_t s)
{
    FwdParams q;
    q.act = act;
    q.wgt = wgt;
    q.y = y;
    q.c_in = g.c_in;
    q.wi = g.wi;
    q.hi = g.hi;
    q.c_out = g.c_out;
    q.w_k = g.w_k;
    q.h_k = g.h_k;
    q.packs = g.packs;
    q.wo = g.wo;
    q.ho = g.ho;
    q.n_cotile = g.n_cotile;
    q.act_plane = (unsigned)g.act_plane;
    q.row_groups = 0;
    q.slots = 0;
    // rows per lane: more rows reuse each weight word more often, but need enough lane
    // slots to fill 256 CUs
    const bool two_rows = g.wo >= 2;
    switch (g.w_k) {
    case 1: return two_rows ? launch<2, 1>(g, q, s) : launch<1, 1>(g, q, s);
    case 3: return two_rows ? launch<2, 3>(g, q, s) : launch<1, 3>(g, q, s);
    case 5: return two_rows ? launch<2, 5>(g, q, s) : launch<1, 5>(g, q, s);
    default: return launch<1, 0>(g, q, s);
    }
}

}  // namespace geo_sc
