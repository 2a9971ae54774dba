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

#include <type_traits>

namespace geo_sc {

namespace {

struct FwdParams {
    const uint32_t* __restrict__ act;  // [n][P][c_in][wi][hi], or [P][c_in][wi][hi][n] with ROWS_IN_N
    const uint32_t* __restrict__ wgt;  // [P][h_k][k_or][n_cotile][2][16]
    const uint32_t* __restrict__ wgt_rail;      // [n_cotile][line][16]: the non-zero rail's word per channel
    const uint32_t* __restrict__ wgt_rail_idx;  // [n_cotile][line][8]: a 16-bit field per channel, see k_rail_pack
    size_t rail_lines;                          // lines per c_out tile: P * lines per pack
    int32_t* __restrict__ y;           // [n][c_out][wo][ho]
    int n, c_in, wi, hi, c_out, w_k, h_k, packs;
    int wo, ho, n_cotile;
    int row_groups;        // ceil(wo / R), or ceil(n / R) when the rows of a lane are batch items
    long long slots;       // lane slots: n * row_groups * ho, or row_groups * ho
    unsigned act_plane;    // c_in * wi * hi
    int pv_per_block;      // (pack, add group) pairs per blockIdx.y
    // accumulation structure (split kernel): add groups (outer, inner), OR channels in all and
    // per outer group, and the activation strides of an inner add step / an OR channel step
    int add_outer, add_inner, or_ch_total, or_ch_per_group;
    unsigned add_stride, or_stride;
    int or_rows;  // kernel rows OR-ed together before the popcount (1, or h_k for the full OR)
    int keep_touches;  // always 0; k_conv_fwd_items_rail_wg: makes the values of its cache touches count as used
};

// acc |= a & w with w wave-uniform: a single v_and_or_b32 whose first source is the SGPR.
// Written as an instruction because the compiler otherwise re-associates chains of these
// into v_and + v_and + v_or3 (three instructions per two pairs instead of two).
__device__ __forceinline__ void and_or(uint32_t& acc, uint32_t a, uint32_t w_uniform)
{
    asm("v_and_or_b32 %0, %1, %2, %0" : "+v"(acc) : "s"(w_uniform), "v"(a));
}

// OR-accumulate CU consecutive input channels: per channel NW activation words per lane and
// WK weight lines per wave.  word(r, u) is the activation word row r meets at kernel tap u.
template <int R, int WK, int CU, int NW, bool ROWS_IN_N>
__device__ __forceinline__ void or_channels(uint32_t (&orp)[R][kCoTile], uint32_t (&orn)[R][kCoTile],
                                            const uint32_t*& ap, const uint32_t*& wp, const unsigned (&off)[NW],
                                            unsigned ch_stride, unsigned k_stride)
{
    constexpr int C = kCoTile;
    uint32_t aw[CU][NW];
#pragma unroll
    for (int cu = 0; cu < CU; cu++)
#pragma unroll
        for (int j = 0; j < NW; j++) aw[cu][j] = ap[cu * ch_stride + off[j]];
#pragma unroll
    for (int cu = 0; cu < CU; cu++)
#pragma unroll
        for (int u = 0; u < WK; u++) {
            uint32_t wv[2 * C];
#pragma unroll
            for (int c = 0; c < 2 * C; c++) wv[c] = wp[c];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint32_t a = aw[cu][ROWS_IN_N ? r * WK + u : r + u];
#pragma unroll
                for (int c = 0; c < C; c++) {
                    and_or(orp[r][c], a, wv[c]);
                    and_or(orn[r][c], a, wv[C + c]);
                }
            }
            wp += k_stride;
        }
    ap += CU * ch_stride;
}

// Template parameters:
//   R   rows of accumulators per lane.  ROWS_IN_N == false: R consecutive output rows a
//       (dim 2) of one item; the WK kernel taps slide over R+WK-1 activation words, so each
//       word is loaded once per channel.  ROWS_IN_N == true (outputs with a single row, e.g.
//       the SC-linear mapping): R consecutive batch items.
//   WK  kernel extent in dim 2 (0: run-time extent, R == 1).
//   CU  input channels per loop trip, chosen so that a trip holds ~192 and-or instructions.
template <int R, int WK, int CU, bool ROWS_IN_N>
__global__ __launch_bounds__(64) void k_conv_fwd(FwdParams q)
{
    constexpr int C = kCoTile;
    static_assert(WK > 0 || (R == 1 && !ROWS_IN_N), "run-time kernel extent handles one row per lane");
    const int cot = blockIdx.x % q.n_cotile;
    const long long slot0 = (long long)(blockIdx.x / q.n_cotile) * 64 + threadIdx.x;
    const bool live = slot0 < q.slots;
    const long long slot = live ? slot0 : 0;
    // lane slot -> (first item n, first output row a0, output column b).  With ROWS_IN_N the
    // R rows of a lane are items n and n + row_groups, consecutive lanes are consecutive
    // items, and the activation streams are stored item-innermost.
    const int b = ROWS_IN_N ? (int)(slot / q.row_groups) : (int)(slot % q.ho);
    const long long t = slot / q.ho;
    const int a0 = ROWS_IN_N ? 0 : (int)(t % q.row_groups) * R;
    const long long n = ROWS_IN_N ? slot % q.row_groups : t / q.row_groups;
    const unsigned item_stride = (unsigned)q.packs * q.act_plane;

    constexpr int NW = WK == 0 ? 1 : (ROWS_IN_N ? R * WK : R + WK - 1);
    // word offsets inside one channel plane.  Rows past the end (partial last group) are
    // clamped to valid ones: they only feed outputs that are never stored.
    unsigned off[NW];
    if constexpr (WK > 0) {
#pragma unroll
        for (int j = 0; j < NW; j++) {
            if (ROWS_IN_N) {
                const int r = j / WK, u = j % WK;
                off[j] = (n + (long long)r * q.row_groups < q.n ? (unsigned)r * q.row_groups : 0u) +
                         (unsigned)u * q.hi * q.n;
            } else {
                const int row = a0 + j < q.wi ? a0 + j : q.wi - 1;
                off[j] = (unsigned)row * q.hi;
            }
        }
    } else {
        off[0] = 0;
    }
    // strides (words) of one pack, one kernel row step, one channel
    const size_t pack_stride = ROWS_IN_N ? (size_t)q.act_plane * q.n : (size_t)q.act_plane;
    const unsigned v_stride = ROWS_IN_N ? (unsigned)q.n : 1u;
    const unsigned ch_stride = ROWS_IN_N ? (unsigned)q.wi * q.hi * q.n : (unsigned)q.wi * q.hi;
    const uint32_t* act_n = ROWS_IN_N ? q.act + (size_t)b * q.n + n : q.act + (size_t)n * item_stride + b;
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

            const uint32_t* ap = act_n + (size_t)p * pack_stride + (size_t)v * v_stride;
            const uint32_t* wp = q.wgt + ((size_t)(p * q.h_k + v) * k_or * q.n_cotile + cot) * (2 * C);

            if constexpr (WK > 0) {
                int ci = 0;
                for (; ci + CU <= q.c_in; ci += CU)
                    or_channels<R, WK, CU, NW, ROWS_IN_N>(orp, orn, ap, wp, off, ch_stride, k_stride);
                if constexpr (CU > 1)
                    for (; ci < q.c_in; ci++)
                        or_channels<R, WK, 1, NW, ROWS_IN_N>(orp, orn, ap, wp, off, ch_stride, k_stride);
            } else {
                for (int ci = 0; ci < q.c_in; ci++) {
                    for (int u = 0; u < q.w_k; u++) {
                        uint32_t wv[2 * C];
#pragma unroll
                        for (int c = 0; c < 2 * C; c++) wv[c] = wp[c];
                        int row = a0 + u;
                        row = row < q.wi ? row : q.wi - 1;
                        const uint32_t aw = ap[(unsigned)row * q.hi];
#pragma unroll
                        for (int c = 0; c < C; c++) {
                            and_or(orp[0][c], aw, wv[c]);
                            and_or(orn[0][c], aw, wv[C + c]);
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
        for (int r = 0; r < R; r++) {
            if (ROWS_IN_N) {
                if (n + (long long)r * q.row_groups < q.n)
                    yo[(size_t)r * q.row_groups * q.c_out * out_plane] = sum[r][c];
            } else {
                if (a0 + r < q.wo) yo[(size_t)r * q.ho] = sum[r][c];
            }
        }
    }
}

// The same kernel for launches that are split over blockIdx.y: each workgroup sums a
// contiguous range of (pack, add group) pairs and adds its partial result to y with integer
// atomics (y is zeroed first).  Used for small layers that would otherwise leave most of the
// GPU idle, and for the accumulation modes other than "OR over (c_in, w_k), add over h_k":
// the add groups are (outer, inner) pairs, an outer group owning a range of OR channels
//   Y : outer 1,              inner kernel rows,     OR channels = input channels
//   YZ: outer channel groups, inner kernel rows,     OR channels = the group's input channels
//   Z : outer 1,              inner input channels,  OR channels = kernel rows
//   FULL: one group per pack; the OR runs over the input channels of or_rows = h_k kernel rows
// (sc_cuda_kernel.cu:176-349, :1351-1366), expressed through the two activation strides in FwdParams; the
// weight lines arrive in exactly the order the loop consumes them.
// Template parameters:
//   R   rows of accumulators per lane.  ROWS_IN_N == false: R consecutive output rows a
//       (dim 2) of one item; the WK kernel taps slide over R+WK-1 activation words, so each
//       word is loaded once per channel.  ROWS_IN_N == true (outputs with a single row, e.g.
//       the SC-linear mapping): R consecutive batch items.
//   WK  kernel extent in dim 2 (0: run-time extent, R == 1).
//   CU  input channels per loop trip, chosen so that a trip holds ~192 and-or instructions.
template <int R, int WK, int CU, bool ROWS_IN_N>
__global__ __launch_bounds__(64) void k_conv_fwd_split(FwdParams q)
{
    constexpr int C = kCoTile;
    static_assert(WK > 0 || (R == 1 && !ROWS_IN_N), "run-time kernel extent handles one row per lane");
    const int cot = blockIdx.x % q.n_cotile;
    const long long slot0 = (long long)(blockIdx.x / q.n_cotile) * 64 + threadIdx.x;
    const bool live = slot0 < q.slots;
    const long long slot = live ? slot0 : 0;
    // lane slot -> (first item n, first output row a0, output column b).  With ROWS_IN_N the
    // R rows of a lane are items n and n + row_groups, consecutive lanes are consecutive
    // items, and the activation streams are stored item-innermost.
    const int b = ROWS_IN_N ? (int)(slot / q.row_groups) : (int)(slot % q.ho);
    const long long t = slot / q.ho;
    const int a0 = ROWS_IN_N ? 0 : (int)(t % q.row_groups) * R;
    const long long n = ROWS_IN_N ? slot % q.row_groups : t / q.row_groups;
    const unsigned item_stride = (unsigned)q.packs * q.act_plane;

    constexpr int NW = WK == 0 ? 1 : (ROWS_IN_N ? R * WK : R + WK - 1);
    // word offsets inside one channel plane.  Rows past the end (partial last group) are
    // clamped to valid ones: they only feed outputs that are never stored.
    unsigned off[NW];
    if constexpr (WK > 0) {
#pragma unroll
        for (int j = 0; j < NW; j++) {
            if (ROWS_IN_N) {
                const int r = j / WK, u = j % WK;
                off[j] = (n + (long long)r * q.row_groups < q.n ? (unsigned)r * q.row_groups : 0u) +
                         (unsigned)u * q.hi * q.n;
            } else {
                const int row = a0 + j < q.wi ? a0 + j : q.wi - 1;
                off[j] = (unsigned)row * q.hi;
            }
        }
    } else {
        off[0] = 0;
    }
    // strides (words) of one pack, one kernel row step, one channel
    const size_t pack_stride = ROWS_IN_N ? (size_t)q.act_plane * q.n : (size_t)q.act_plane;
    const unsigned v_stride = ROWS_IN_N ? (unsigned)q.n : 1u;
    const unsigned ch_stride = ROWS_IN_N ? (unsigned)q.wi * q.hi * q.n : (unsigned)q.wi * q.hi;
    const uint32_t* act_n = ROWS_IN_N ? q.act + (size_t)b * q.n + n : q.act + (size_t)n * item_stride + b;
    const unsigned k_stride = (unsigned)q.n_cotile * 2 * C;

    int sum[R][C];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int c = 0; c < C; c++) sum[r][c] = 0;

    // (pack, add group) pairs are independent partial sums: blockIdx.y takes a contiguous
    // range of them when the launch is split to fill the GPU
    const int groups = q.add_outer * q.add_inner;
    const int pv_begin = blockIdx.y * q.pv_per_block;
    const int pv_end = min(q.packs * groups, pv_begin + q.pv_per_block);
    const unsigned add_stride = ROWS_IN_N ? v_stride : q.add_stride;
    const unsigned or_stride = ROWS_IN_N ? ch_stride : q.or_stride;
    const size_t lines_per_pack = (size_t)q.or_rows * q.add_inner * q.or_ch_total * q.w_k;
    {
        for (int pv = pv_begin; pv < pv_end; pv++) {
            const int p = pv / groups, g = pv - p * groups;
            const int go = g / q.add_inner, gi = g - go * q.add_inner;
            const int ch0 = go * q.or_ch_per_group;
            const int chs = min(q.or_ch_per_group, q.or_ch_total - ch0);
            uint32_t orp[R][C], orn[R][C];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int c = 0; c < C; c++) orp[r][c] = orn[r][c] = 0u;

            const uint32_t* ap0 = act_n + (size_t)p * pack_stride + (size_t)gi * add_stride + (size_t)ch0 * or_stride;
            const size_t line = p * lines_per_pack + (size_t)ch0 * q.add_inner * q.w_k + (size_t)gi * chs * q.w_k;
            const uint32_t* wp = q.wgt + (line * q.n_cotile + cot) * (2 * C);

            for (int row = 0; row < q.or_rows; row++) {
                const uint32_t* ap = ap0 + row;  // next kernel row: one word further (never with ROWS_IN_N)
                if constexpr (WK > 0) {
                    int ci = 0;
                    for (; ci + CU <= chs; ci += CU)
                        or_channels<R, WK, CU, NW, ROWS_IN_N>(orp, orn, ap, wp, off, or_stride, k_stride);
                    if constexpr (CU > 1)
                        for (; ci < chs; ci++)
                            or_channels<R, WK, 1, NW, ROWS_IN_N>(orp, orn, ap, wp, off, or_stride, k_stride);
                } else {
                    for (int ci = 0; ci < chs; ci++) {
                        for (int u = 0; u < q.w_k; u++) {
                            uint32_t wv[2 * C];
#pragma unroll
                            for (int c = 0; c < 2 * C; c++) wv[c] = wp[c];
                            int arow = a0 + u;
                            arow = arow < q.wi ? arow : q.wi - 1;
                            const uint32_t aw = ap[(unsigned)arow * q.hi];
#pragma unroll
                            for (int c = 0; c < C; c++) {
                                and_or(orp[0][c], aw, wv[c]);
                                and_or(orn[0][c], aw, wv[C + c]);
                            }
                            wp += k_stride;
                        }
                        ap += or_stride;
                    }
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
        for (int r = 0; r < R; r++) {
            const bool row_ok = ROWS_IN_N ? n + (long long)r * q.row_groups < q.n : a0 + r < q.wo;
            int32_t* dst = yo + (ROWS_IN_N ? (size_t)r * q.row_groups * q.c_out * out_plane : (size_t)r * q.ho);
            if (!row_ok) continue;
            atomicAdd(dst, sum[r][c]);  // integer adds: order does not matter
        }
    }
}

// Layers with few output positions and large OR groups (classifier layers: 64 x 4 x 4 -> 10 at
// batch 256 has 2560 outputs of 1024 products each): one wave per (output position, c_out tile,
// pack, add group); the lanes run over the members of the OR group, each with its own weight
// line in VGPRs, and the 2 x 16 partial OR words are combined across the wave with xor shuffles.
// Results are added into the zeroed y with integer atomics.  Activation layout [n][P][c_in][wi][hi].
__global__ __launch_bounds__(64) void k_conv_fwd_thin(FwdParams q)
{
    constexpr int C = kCoTile;
    const int lane = threadIdx.x;
    const int cot = blockIdx.x % q.n_cotile;
    const long long m = blockIdx.x / q.n_cotile;
    const int b = (int)(m % q.ho);
    const long long t = m / q.ho;
    const int a = (int)(t % q.wo);
    const long long n = t / q.wo;
    const int groups = q.add_outer * q.add_inner;
    const int p = blockIdx.y / groups, g = blockIdx.y - p * groups;
    const int go = g / q.add_inner, gi = g - go * q.add_inner;
    const int ch0 = go * q.or_ch_per_group;
    const int chs = min(q.or_ch_per_group, q.or_ch_total - ch0);
    const int members = q.or_rows * chs * q.w_k;
    const size_t lines_per_pack = (size_t)q.or_rows * q.add_inner * q.or_ch_total * q.w_k;
    const size_t line0 = p * lines_per_pack + (size_t)ch0 * q.add_inner * q.w_k + (size_t)gi * chs * q.w_k;
    const uint32_t* ap0 = q.act + ((size_t)n * q.packs + p) * q.act_plane + (size_t)gi * q.add_stride +
                          (size_t)ch0 * q.or_stride + (size_t)a * q.hi + b;

    uint32_t orp[C], orn[C];
#pragma unroll
    for (int c = 0; c < C; c++) orp[c] = orn[c] = 0u;
    for (int j = lane; j < members; j += 64) {
        // member j = (kernel row of the OR, channel of the group, tap u), u fastest
        const int u = j % q.w_k, t2 = j / q.w_k;
        const int ch = t2 % chs, row = t2 / chs;
        const uint32_t aw = ap0[(size_t)ch * q.or_stride + (size_t)u * q.hi + row];
        const uint4* wl = reinterpret_cast<const uint4*>(q.wgt + ((line0 + j) * q.n_cotile + cot) * (2 * C));
        uint32_t wv[2 * C];
#pragma unroll
        for (int v4 = 0; v4 < 2 * C / 4; v4++) {
            const uint4 w4 = wl[v4];
            wv[4 * v4] = w4.x;
            wv[4 * v4 + 1] = w4.y;
            wv[4 * v4 + 2] = w4.z;
            wv[4 * v4 + 3] = w4.w;
        }
#pragma unroll
        for (int c = 0; c < C; c++) {
            orp[c] |= aw & wv[c];
            orn[c] |= aw & wv[C + c];
        }
    }
    int mine = 0;
#pragma unroll
    for (int c = 0; c < C; c++) {
        uint32_t vp = orp[c], vn = orn[c];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            vp |= (uint32_t)__shfl_xor((int)vp, off);
            vn |= (uint32_t)__shfl_xor((int)vn, off);
        }
        if (lane == c) mine = __popc(vp) - __popc(vn);
    }
    const int co = cot * C + lane;
    if (lane < C && co < q.c_out)
        atomicAdd(q.y + (((size_t)n * q.c_out + co) * q.wo + a) * q.ho + b, mine);
}

// ---------------------------------------------------------------------------------------------
// Rail-skipping kernel for the plain y-mode launches.
//
// A weight has at most one non-zero code (wp = code of clamp(w, 0, .), wn = code of -clamp(w, ., 0),
// sc.cpp:301-304), and a zero code gives an all-zero stream: of the two v_and_or_b32 that
// k_conv_fwd issues per (activation word, weight), one always ORs zeros.  Which one is uniform
// over the wave but varies per (member, channel), so it cannot select a register at compile time;
// gfx9's VGPR index mode can at run time: with s_set_gpr_idx_on(SRC2, DST) the accumulator operand of
// every following VALU instruction is offset by M0[7:0], one M0 update per (member,
// channel) points the same two v_and_or_b32 (two rows) at the channel's positive or negative
// accumulators.  The scalar instructions issue beside the vector ones (measured: one index update
// per v_and_or_b32 leaves the vector rate unchanged), so the kernel executes half of k_conv_fwd's
// vector instructions.
//
// The 64 OR accumulators sit in fixed registers v[64:127]: P[c][r] = v[64 + 2 c + r],
// N[c][r] = v[96 + 2 c + r].  The index of a channel is 2 c (positive rail or zero weight) or
// 32 + 2 c (negative rail); the asm blocks name v64 / v65 and the index does the rest.  The index
// arrives as a ready-made 16-bit M0 value per channel (index and the two operand enables), so one
// scalar instruction per channel moves it into M0 (s_and_b32 / s_lshr_b32 on a word that holds two
// of them; same effect as s_set_gpr_idx_idx, without a separate shift).  The
// compiler sees the four 16-register vectors as read and written by every block and keeps them
// in place.  Index mode is switched off at the end of every block: compiler-generated vector
// instructions in between must not be indexed.
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));

// M0 of a channel from its 16-bit field: index in bits 7:0, the SRC2 and DST enables in bits 15:12
#define GEO_SC_RAIL_LO(I) "s_and_b32 m0, %[" I "], 0xffff\n"
#define GEO_SC_RAIL_HI(I) "s_lshr_b32 m0, %[" I "], 16\n"
#define GEO_SC_RAIL_OPERANDS                                                                                           \
    [w0] "s"(w[0]), [w1] "s"(w[1]), [w2] "s"(w[2]), [w3] "s"(w[3]), [w4] "s"(w[4]), [w5] "s"(w[5]), [w6] "s"(w[6]),     \
        [w7] "s"(w[7]), [w8] "s"(w[8]), [w9] "s"(w[9]), [w10] "s"(w[10]), [w11] "s"(w[11]), [w12] "s"(w[12]),           \
        [w13] "s"(w[13]), [w14] "s"(w[14]), [w15] "s"(w[15]), [i0] "s"(ix[0]), [i1] "s"(ix[1]), [i2] "s"(ix[2]),        \
        [i3] "s"(ix[3]), [i4] "s"(ix[4]), [i5] "s"(ix[5]), [i6] "s"(ix[6]), [i7] "s"(ix[7]), [a0] "v"(a0), [a1] "v"(a1)
// 16 channels x PAIR, the M0 update of every channel but the first in front of its pair
#define GEO_SC_RAIL_16(PAIR)                                                                                           \
    PAIR("w0", "") PAIR("w1", GEO_SC_RAIL_HI("i0")) PAIR("w2", GEO_SC_RAIL_LO("i1")) PAIR("w3", GEO_SC_RAIL_HI("i1"))   \
    PAIR("w4", GEO_SC_RAIL_LO("i2")) PAIR("w5", GEO_SC_RAIL_HI("i2")) PAIR("w6", GEO_SC_RAIL_LO("i3"))                  \
    PAIR("w7", GEO_SC_RAIL_HI("i3")) PAIR("w8", GEO_SC_RAIL_LO("i4")) PAIR("w9", GEO_SC_RAIL_HI("i4"))                  \
    PAIR("w10", GEO_SC_RAIL_LO("i5")) PAIR("w11", GEO_SC_RAIL_HI("i5")) PAIR("w12", GEO_SC_RAIL_LO("i6"))               \
    PAIR("w13", GEO_SC_RAIL_HI("i6")) PAIR("w14", GEO_SC_RAIL_LO("i7")) PAIR("w15", GEO_SC_RAIL_HI("i7"))

// Defines, for accumulators pinned at v[B0 : B0 + 63] (V0 = "vB0", V1 = "v(B0 + 1)" name the first pair):
//  LINE : one weight line (16 channels) against the two activation words of the lane's two rows;
//  FIRST: the first weight line of an OR group, which assigns instead of accumulating and clears the channel's
//         other rail (index ^ 32), so that the 64 accumulators need no zeroing pass.  v_and_b32 and v_mov_b32
//         are two-operand instructions, which issue at twice the rate of v_and_or_b32: the line costs what an
//         accumulating line costs.
// Not volatile: every effect goes through the operands, and a volatile asm would count as a possible store,
// after which the compiler no longer reads the weight lines with scalar loads.
#define GEO_SC_DEFINE_RAIL_LINES(LINE, FIRST, V0, V1, RP0, RP1, RN0, RN1)                                              \
    __device__ __forceinline__ void LINE(u32x16& p0, u32x16& p1, u32x16& n0, u32x16& n1, const uint32_t (&w)[kCoTile],  \
                                         const uint32_t (&ix)[kCoTile / 2], uint32_t a0, uint32_t a1)                  \
    {                                                                                                                  \
        asm("s_set_gpr_idx_on %[i0], gpr_idx(SRC2,DST)\n" GEO_SC_RAIL_16(GEO_SC_RAIL_PAIR_##LINE) "s_set_gpr_idx_off\n" \
            : "+{" RP0 "}"(p0), "+{" RP1 "}"(p1), "+{" RN0 "}"(n0), "+{" RN1 "}"(n1)                                   \
            : GEO_SC_RAIL_OPERANDS                                                                                     \
            : "m0", "scc");                                                                                            \
    }                                                                                                                  \
    __device__ __forceinline__ void FIRST(u32x16& p0, u32x16& p1, u32x16& n0, u32x16& n1, const uint32_t (&w)[kCoTile], \
                                          const uint32_t (&ix)[kCoTile / 2], uint32_t a0, uint32_t a1)                 \
    {                                                                                                                  \
        asm("s_set_gpr_idx_on %[i0], gpr_idx(SRC2,DST)\n" GEO_SC_RAIL_16(GEO_SC_RAIL_PAIR_##FIRST) "s_set_gpr_idx_off\n" \
            : "={" RP0 "}"(p0), "={" RP1 "}"(p1), "={" RN0 "}"(n0), "={" RN1 "}"(n1)                                   \
            : GEO_SC_RAIL_OPERANDS                                                                                     \
            : "m0", "scc");                                                                                            \
    }

// accumulators at v[64:127]: the kernels with four waves per SIMD
#define GEO_SC_RAIL_PAIR_rail_line(W, SET)                                                                             \
    SET "v_and_or_b32 v64, %[" W "], %[a0], v64\n"                                                                     \
        "v_and_or_b32 v65, %[" W "], %[a1], v65\n"
#define GEO_SC_RAIL_PAIR_rail_line_first(W, SET)                                                                       \
    SET "v_and_b32 v64, %[" W "], %[a0]\n"                                                                            \
        "v_and_b32 v65, %[" W "], %[a1]\n"                                                                            \
        "s_xor_b32 m0, m0, 32\n"                                                                                      \
        "v_mov_b32 v64, 0\n"                                                                                          \
        "v_mov_b32 v65, 0\n"
GEO_SC_DEFINE_RAIL_LINES(rail_line, rail_line_first, "v64", "v65", "v[64:79]", "v[80:95]", "v[96:111]", "v[112:127]")
// accumulators at v[32:95]: the kernel with five waves per SIMD (96 registers in all)
#define GEO_SC_RAIL_PAIR_rail_line_lo(W, SET)                                                                          \
    SET "v_and_or_b32 v32, %[" W "], %[a0], v32\n"                                                                     \
        "v_and_or_b32 v33, %[" W "], %[a1], v33\n"
#define GEO_SC_RAIL_PAIR_rail_line_first_lo(W, SET)                                                                    \
    SET "v_and_b32 v32, %[" W "], %[a0]\n"                                                                            \
        "v_and_b32 v33, %[" W "], %[a1]\n"                                                                            \
        "s_xor_b32 m0, m0, 32\n"                                                                                      \
        "v_mov_b32 v32, 0\n"                                                                                          \
        "v_mov_b32 v33, 0\n"
GEO_SC_DEFINE_RAIL_LINES(rail_line_lo, rail_line_first_lo, "v32", "v33", "v[32:47]", "v[48:63]", "v[64:79]", "v[80:95]")
#undef GEO_SC_DEFINE_RAIL_LINES
#undef GEO_SC_RAIL_16
#undef GEO_SC_RAIL_OPERANDS
#undef GEO_SC_RAIL_LO
#undef GEO_SC_RAIL_HI

// sum += popcount(pos) - popcount(neg) in three instructions (the compiler's form takes four)
__device__ __forceinline__ void popc_diff(int& sum, uint32_t pos, uint32_t neg)
{
    uint32_t t;
    asm("v_bcnt_u32_b32 %0, %1, %0" : "+v"(sum) : "v"(pos));
    asm("v_bcnt_u32_b32 %0, %1, 0" : "=v"(t) : "v"(neg));
    sum -= (int)t;
}
static_assert(kCoTile == 16, "rail_line is written for tiles of 16 output channels");

// Two output rows per lane (R = 2), position-major activation streams, kernel extent WK in dim 2.
// Same lane -> position mapping, grid and result as k_conv_fwd<2, WK, 1, false>.
// CU: input channels per loop trip (their loads are issued together: 2 for 1-wide kernels, so that a
// trip holds 64 vector instructions behind one wait instead of 32).
template <int WK, int CU>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_conv_fwd_rail(FwdParams q)
{
    constexpr int C = kCoTile, R = 2, NW = R + WK - 1;
    const int cot = blockIdx.x % q.n_cotile;
    const long long slot0 = (long long)(blockIdx.x / q.n_cotile) * 64 + threadIdx.x;
    const bool live = slot0 < q.slots;
    const long long slot = live ? slot0 : 0;
    const int b = (int)(slot % q.ho);
    const long long t = slot / q.ho;
    const int a0 = (int)(t % q.row_groups) * R;
    const long long n = t / q.row_groups;
    const unsigned item_stride = (unsigned)q.packs * q.act_plane;
    // word offsets inside one channel plane; rows past the end (partial last group) are clamped to
    // valid ones: they only feed outputs that are never stored
    unsigned off[NW];
#pragma unroll
    for (int j = 0; j < NW; j++) {
        const int row = a0 + j < q.wi ? a0 + j : q.wi - 1;
        off[j] = (unsigned)row * q.hi;
    }
    const unsigned ch_stride = (unsigned)q.wi * q.hi;
    const uint32_t* act_n = q.act + (size_t)n * item_stride + b;
    const int k_or = q.c_in * q.w_k;

    int sum[2 * C];  // [2 c + r]
#pragma unroll
    for (int i = 0; i < 2 * C; i++) sum[i] = 0;

    for (int p = 0; p < q.packs; p++) {
        for (int v = 0; v < q.h_k; v++) {
            u32x16 p0 = 0u, p1 = 0u, n0 = 0u, n1 = 0u;
            const uint32_t* ap = act_n + (size_t)p * q.act_plane + v;
            // rail-packed lines are stored [c_out tile][line]: the lines of a tile follow each other in
            // the order the loops consume them
            const size_t line0 = (size_t)cot * q.rail_lines + (size_t)(p * q.h_k + v) * k_or;
            const uint32_t* wp = q.wgt_rail + line0 * C;
            const uint32_t* ip = q.wgt_rail_idx + line0 * (C / 2);
            auto channels = [&](auto cu_tag) {
                constexpr int N = decltype(cu_tag)::value;
                uint32_t aw[N][NW];
#pragma unroll
                for (int cu = 0; cu < N; cu++)
#pragma unroll
                    for (int j = 0; j < NW; j++) aw[cu][j] = ap[cu * ch_stride + off[j]];
                uint32_t wv[N * WK][C], iv[N * WK][C / 2];
#pragma unroll
                for (int l = 0; l < N * WK; l++) {
#pragma unroll
                    for (int c = 0; c < C; c++) wv[l][c] = wp[l * C + c];
#pragma unroll
                    for (int c = 0; c < C / 2; c++) iv[l][c] = ip[l * (C / 2) + c];
                }
#pragma unroll
                for (int cu = 0; cu < N; cu++)
#pragma unroll
                    for (int u = 0; u < WK; u++)
                        rail_line(p0, p1, n0, n1, wv[cu * WK + u], iv[cu * WK + u], aw[cu][u], aw[cu][u + 1]);
                wp += N * WK * C;
                ip += N * WK * (C / 2);
                ap += N * ch_stride;
            };
            int ci = 0;
            for (; ci + CU <= q.c_in; ci += CU) channels(std::integral_constant<int, CU>());
            if constexpr (CU > 1)
                for (; ci < q.c_in; ci++) channels(std::integral_constant<int, 1>());
            // binary add across kernel rows and packs: v_bcnt_u32_b32 folds the add
#pragma unroll
            for (int i = 0; i < C; i++) {
                sum[i] += __popc(p0[i]) - __popc(n0[i]);
                sum[C + i] += __popc(p1[i]) - __popc(n1[i]);
            }
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
            if (a0 + r < q.wo) yo[(size_t)r * q.ho] = sum[2 * c + r];
    }
}

// k_conv_fwd_rail for 3-wide kernels with the activation words staged through LDS.  The waves of the
// c_out tiles of one position tile read the same four activation words per lane and channel; here
// NWV of them form a workgroup, every wave fetches 8 / NWV channels of a chunk of 8 and leaves them in
// LDS as 16 bytes per lane, and all read them back with one ds_read_b128 per channel: an eighth (a
// quarter) of the global loads per wave, and the wait in front of a channel's 96 vector instructions is
// for LDS and the scalar cache instead of the vector memory path.  The chunks are double-buffered:
// the loads of chunk t + 1 are issued before chunk t is computed and written to LDS after it, one
// barrier per chunk.  NPT position tiles (NWV waves each, staged separately) share the workgroup and
// its barrier.  Needs c_in % 8 == 0 and n_cotile % NWV == 0 (the launcher checks).
constexpr int kStageChannels = 8;
template <int NWV, int NPT>
__global__ __launch_bounds__(64 * NWV * NPT) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_conv_fwd_rail_lds(FwdParams q)
{
    constexpr int C = kCoTile, R = 2, WK = 3, NW = R + WK - 1, CH = kStageChannels, CPW = CH / NWV;
    static_assert(NW == 4 && CH % NWV == 0, "a lane's words of one channel are one uint4");
    __shared__ uint4 stage_all[2][NPT][CH][64];
    const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int wave = wave_all % NWV, pt = wave_all / NWV;  // c_out tile and position tile inside the workgroup
    const int cot_groups = q.n_cotile / NWV;
    const int cot = (blockIdx.x % cot_groups) * NWV + wave;
    const long long slot0 = ((long long)(blockIdx.x / cot_groups) * NPT + pt) * 64 + lane;
    const bool live = slot0 < q.slots;
    const long long slot = live ? slot0 : 0;
    const int b = (int)(slot % q.ho);
    const long long t = slot / q.ho;
    const int a0 = (int)(t % q.row_groups) * R;
    const long long n = t / q.row_groups;
    const unsigned item_stride = (unsigned)q.packs * q.act_plane;
    // byte offsets of the lane's four rows in the stream buffer (under 4 GB: the launcher checks), read
    // with buffer loads: the chunk's and channel's offset is the scalar operand
    unsigned voff[NW];
#pragma unroll
    for (int j = 0; j < NW; j++) {
        const int row = a0 + j < q.wi ? a0 + j : q.wi - 1;
        voff[j] = 4u * ((unsigned)n * item_stride + (unsigned)b + (unsigned)row * q.hi);
    }
    const unsigned ch_b = 4u * (unsigned)q.wi * q.hi;
    const __amdgpu_buffer_rsrc_t act = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(q.act), 0, (int)(4u * (unsigned)q.n * item_stride), 0x00020000);
    const int chunks_per_pass = q.c_in / CH;
    // this launch row's share of the (pack, kernel row) passes; with more than one row the partial sums
    // are added to the zeroed y with integer atomics
    const int pass_begin = blockIdx.y * q.pv_per_block;
    const int passes = min(q.packs * q.h_k, pass_begin + q.pv_per_block);
    const int total = (passes - pass_begin) * chunks_per_pass;

    int sum[2 * C];  // [2 c + r]
#pragma unroll
    for (int i = 0; i < 2 * C; i++) sum[i] = 0;

    // this wave's channels of chunk (pass, cc): wave + NWV * i
    uint4 fetched[CPW];
    auto fetch = [&](int pass, int cc) {
        const int p = pass / q.h_k, v = pass - p * q.h_k;
        const unsigned so = 4u * ((unsigned)p * q.act_plane + (unsigned)v) + (unsigned)(cc * CH + wave) * ch_b;
#pragma unroll
        for (int i = 0; i < CPW; i++) {
            const int sc = (int)(so + (unsigned)(NWV * i) * ch_b);
            fetched[i] = make_uint4(__builtin_amdgcn_raw_buffer_load_b32(act, (int)voff[0], sc, 0),
                                    __builtin_amdgcn_raw_buffer_load_b32(act, (int)voff[1], sc, 0),
                                    __builtin_amdgcn_raw_buffer_load_b32(act, (int)voff[2], sc, 0),
                                    __builtin_amdgcn_raw_buffer_load_b32(act, (int)voff[3], sc, 0));
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < CPW; i++) stage_all[buf][pt][wave + NWV * i][lane] = fetched[i];
    };

    const size_t line0 = (size_t)cot * q.rail_lines + (size_t)pass_begin * q.c_in * WK;
    const uint32_t* wp = q.wgt_rail + line0 * C;
    const uint32_t* ip = q.wgt_rail_idx + line0 * (C / 2);
    fetch(pass_begin, 0);
    commit(0);
    __syncthreads();
    int tc = 0;
    for (int pass = pass_begin; pass < passes; pass++) {
        u32x16 p0 = 0u, p1 = 0u, n0 = 0u, n1 = 0u;
        for (int cc = 0; cc < chunks_per_pass; cc++, tc++) {
            const int buf = tc & 1;
            // the chunk after this one may belong to the next pass
            const bool last_of_pass = cc + 1 == chunks_per_pass;
            const bool more = tc + 1 < total;
            if (more) fetch(last_of_pass ? pass + 1 : pass, last_of_pass ? 0 : cc + 1);
            for (int ch = 0; ch < CH; ch++) {
                const uint4 aw = stage_all[buf][pt][ch][lane];
                uint32_t wv[WK][C], iv[WK][C / 2];
#pragma unroll
                for (int l = 0; l < WK; l++) {
#pragma unroll
                    for (int c = 0; c < C; c++) wv[l][c] = wp[l * C + c];
#pragma unroll
                    for (int c = 0; c < C / 2; c++) iv[l][c] = ip[l * (C / 2) + c];
                }
                rail_line(p0, p1, n0, n1, wv[0], iv[0], aw.x, aw.y);
                rail_line(p0, p1, n0, n1, wv[1], iv[1], aw.y, aw.z);
                rail_line(p0, p1, n0, n1, wv[2], iv[2], aw.z, aw.w);
                wp += WK * C;
                ip += WK * (C / 2);
            }
            if (more) commit(buf ^ 1);
            __syncthreads();
        }
        // end of a (pack, kernel row) pass: binary add across kernel rows and packs
#pragma unroll
        for (int i = 0; i < C; i++) {
            sum[i] += __popc(p0[i]) - __popc(n0[i]);
            sum[C + i] += __popc(p1[i]) - __popc(n1[i]);
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
        for (int r = 0; r < R; r++) {
            if (a0 + r >= q.wo) continue;
            if (gridDim.y == 1)
                yo[(size_t)r * q.ho] = sum[2 * c + r];
            else
                atomicAdd(yo + (size_t)r * q.ho, sum[2 * c + r]);  // integer adds: order does not matter
        }
    }
}

// The rail-skipping form of k_conv_fwd_split<2, WK, 1, false>: launches split over blockIdx.y and
// the accumulation modes other than y, position-major activation streams, two output rows per lane.
// Partial sums are added to the zeroed y with integer atomics.
// The add groups of the other modes are short (z mode: 9 lines of a 3 x 3 kernel), so what happens
// per group is kept scalar and small: the (pack, outer, inner) group counters advance by increments (no
// divisions), the weight lines of a c_out tile follow each other in loop order (both pointers only
// advance), and the activation words come through buffer loads (resource over the stream buffer, one
// 32-bit byte offset per lane and row, the group's and channel's offset as the scalar operand).
template <int WK, int CU>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_conv_fwd_split_rail(FwdParams q)
{
    constexpr int C = kCoTile, R = 2, NW = R + WK - 1;
    const int cot = blockIdx.x % q.n_cotile;
    const long long slot0 = (long long)(blockIdx.x / q.n_cotile) * 64 + threadIdx.x;
    const bool live = slot0 < q.slots;
    const long long slot = live ? slot0 : 0;
    const int b = (int)(slot % q.ho);
    const long long t = slot / q.ho;
    const int a0 = (int)(t % q.row_groups) * R;
    const long long n = t / q.row_groups;
    const unsigned item_stride = (unsigned)q.packs * q.act_plane;
    // byte offsets of the lane's rows in the stream buffer (the launcher keeps the buffer under 4 GB);
    // rows past the end (partial last group) are clamped to valid ones: they only feed outputs that are
    // never stored
    unsigned voff[NW];
#pragma unroll
    for (int j = 0; j < NW; j++) {
        const int row = a0 + j < q.wi ? a0 + j : q.wi - 1;
        voff[j] = 4u * ((unsigned)n * item_stride + (unsigned)b + (unsigned)row * q.hi);
    }
    const __amdgpu_buffer_rsrc_t act = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(q.act), 0, (int)(4u * (unsigned)q.n * item_stride), 0x00020000);
    const unsigned plane_b = 4u * q.act_plane, add_b = 4u * q.add_stride, or_b = 4u * q.or_stride;

    int sum[2 * C];  // [2 c + r]
#pragma unroll
    for (int i = 0; i < 2 * C; i++) sum[i] = 0;

    const int groups = q.add_outer * q.add_inner;
    const int pv_begin = blockIdx.y * q.pv_per_block;
    const int pv_end = min(q.packs * groups, pv_begin + q.pv_per_block);
    const size_t lines_per_pack = (size_t)q.or_rows * q.add_inner * q.or_ch_total * q.w_k;
    // group counters of pv_begin; the loop advances them
    int p = pv_begin / groups;
    int go = (pv_begin - p * groups) / q.add_inner;
    int gi = pv_begin - p * groups - go * q.add_inner;
    const uint32_t* wp;
    const uint32_t* ip;
    {
        const int ch0 = go * q.or_ch_per_group;
        const int chs = min(q.or_ch_per_group, q.or_ch_total - ch0);
        const size_t line = (size_t)cot * q.rail_lines + p * lines_per_pack + (size_t)ch0 * q.add_inner * q.w_k +
                            (size_t)gi * chs * q.w_k;
        wp = q.wgt_rail + line * C;
        ip = q.wgt_rail_idx + line * (C / 2);
    }
    for (int pv = pv_begin; pv < pv_end; pv++) {
        const int ch0 = go * q.or_ch_per_group;
        const int chs = min(q.or_ch_per_group, q.or_ch_total - ch0);
        u32x16 p0, p1, n0, n1;  // written by the group's first line
        bool first = true;
        const unsigned group_off = (unsigned)p * plane_b + (unsigned)gi * add_b + (unsigned)ch0 * or_b;
        for (int row = 0; row < q.or_rows; row++) {
            unsigned ch_off = group_off + 4u * (unsigned)row;  // next kernel row: one word further
            auto channels_of = [&](auto cu_tag, auto first_tag) {
                constexpr int N = decltype(cu_tag)::value;
                constexpr bool FIRST = decltype(first_tag)::value;
                uint32_t aw[N][NW];
#pragma unroll
                for (int cu = 0; cu < N; cu++)
#pragma unroll
                    for (int j = 0; j < NW; j++)
                        aw[cu][j] = __builtin_amdgcn_raw_buffer_load_b32(act, (int)voff[j],
                                                                         (int)(ch_off + (unsigned)cu * or_b), 0);
                uint32_t wv[N * WK][C], iv[N * WK][C / 2];
#pragma unroll
                for (int l = 0; l < N * WK; l++) {
#pragma unroll
                    for (int c = 0; c < C; c++) wv[l][c] = wp[l * C + c];
#pragma unroll
                    for (int c = 0; c < C / 2; c++) iv[l][c] = ip[l * (C / 2) + c];
                }
#pragma unroll
                for (int cu = 0; cu < N; cu++)
#pragma unroll
                    for (int u = 0; u < WK; u++) {
                        if (FIRST && cu == 0 && u == 0)
                            rail_line_first(p0, p1, n0, n1, wv[0], iv[0], aw[0][0], aw[0][1]);
                        else
                            rail_line(p0, p1, n0, n1, wv[cu * WK + u], iv[cu * WK + u], aw[cu][u], aw[cu][u + 1]);
                    }
                wp += N * WK * C;
                ip += N * WK * (C / 2);
                ch_off += (unsigned)N * or_b;
            };
            auto channels = [&](auto cu_tag) {
                if (first)
                    channels_of(cu_tag, std::true_type());
                else
                    channels_of(cu_tag, std::false_type());
                first = false;
            };
            int ci = 0;
            for (; ci + CU <= chs; ci += CU) channels(std::integral_constant<int, CU>());
            if constexpr (CU > 1)
                for (; ci < chs; ci++) channels(std::integral_constant<int, 1>());
        }
#pragma unroll
        for (int i = 0; i < C; i++) {
            popc_diff(sum[i], p0[i], n0[i]);
            popc_diff(sum[C + i], p1[i], n1[i]);
        }
        // next group: inner add group, then outer, then pack
        if (++gi == q.add_inner) {
            gi = 0;
            if (++go == q.add_outer) {
                go = 0;
                p++;
            }
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
            if (a0 + r < q.wo) atomicAdd(yo + (size_t)r * q.ho, sum[2 * c + r]);  // integer adds: order does not matter
    }
}

// k_conv_fwd_split_rail for launches in which every wave sums exactly one (pack, add group) pair (blockIdx.y =
// the pair): small layers split as far as they go.  Without running sums a wave needs 96 registers instead of
// 128 - the 64 accumulators sit at v[32:95], the counts go from the popcounts straight into the atomics - so
// five waves fit a SIMD instead of four: 5120 waves (the 32 -> 64 5 x 5 layer at 8 x 8, batch 256) are one
// round instead of two, of which the second would run a quarter full and bound by load latency.
// Two waves per workgroup, each with a tile of its own: a CU takes at most 16 workgroups, which single-wave
// workgroups would hit at four waves per SIMD.
// WG: the pairs of one tile as the waves of one workgroup (at most 16 pairs): their counts meet in LDS
// (ds_add_u32) and the workgroup stores the sums - no zeroing launch over y and no global atomics, whose
// drain is what such a launch otherwise ends with (the 32 -> 64 layer: waves live 59 us of the 88 us that
// the launch with atomics takes).
constexpr int kPairWaves = 2, kPairWgMax = 16;
template <int WK, int CU, bool WG = false>
__global__ __launch_bounds__(WG ? 64 * kPairWgMax : 64 * kPairWaves) __attribute__((amdgpu_waves_per_eu(5, 5)))
void k_conv_fwd_pair_rail(FwdParams q, unsigned n_tiles)
{
    constexpr int C = kCoTile, R = 2, NW = R + WK - 1;
    __shared__ int red[WG ? 2 * C * 64 : 1];  // [2 c + r][lane]
    const int wave_in_wg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned tile = WG ? blockIdx.x : blockIdx.x * kPairWaves + wave_in_wg;
    if (!WG && tile >= n_tiles) return;
    if constexpr (WG) {
        for (int i = threadIdx.x; i < 2 * C * 64; i += blockDim.x) red[i] = 0;
        __syncthreads();
    }
    const int cot = tile % q.n_cotile;
    const long long slot0 = (long long)(tile / q.n_cotile) * 64 + (threadIdx.x & 63);
    const bool live = slot0 < q.slots;
    const long long slot = live ? slot0 : 0;
    const int b = (int)(slot % q.ho);
    const long long t = slot / q.ho;
    const int a0 = (int)(t % q.row_groups) * R;
    const long long n = t / q.row_groups;
    const unsigned item_stride = (unsigned)q.packs * q.act_plane;
    unsigned voff[NW];
#pragma unroll
    for (int j = 0; j < NW; j++) {
        const int row = a0 + j < q.wi ? a0 + j : q.wi - 1;
        voff[j] = 4u * ((unsigned)n * item_stride + (unsigned)b + (unsigned)row * q.hi);
    }
    const __amdgpu_buffer_rsrc_t act = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(q.act), 0, (int)(4u * (unsigned)q.n * item_stride), 0x00020000);
    const unsigned plane_b = 4u * q.act_plane, add_b = 4u * q.add_stride, or_b = 4u * q.or_stride;

    const int groups = q.add_outer * q.add_inner;
    const int pv = WG ? wave_in_wg : blockIdx.y;
    const int p = pv / groups;
    const int go = (pv - p * groups) / q.add_inner;
    const int gi = pv - p * groups - go * q.add_inner;
    const int ch0 = go * q.or_ch_per_group;
    const int chs = min(q.or_ch_per_group, q.or_ch_total - ch0);
    const size_t lines_per_pack = (size_t)q.or_rows * q.add_inner * q.or_ch_total * q.w_k;
    const size_t line = (size_t)cot * q.rail_lines + p * lines_per_pack + (size_t)ch0 * q.add_inner * q.w_k +
                        (size_t)gi * chs * q.w_k;
    const uint32_t* wp = q.wgt_rail + line * C;
    const uint32_t* ip = q.wgt_rail_idx + line * (C / 2);
    u32x16 p0, p1, n0, n1;  // written by the group's first line
    bool first = true;
    const unsigned group_off = (unsigned)p * plane_b + (unsigned)gi * add_b + (unsigned)ch0 * or_b;
    for (int row = 0; row < q.or_rows; row++) {
        unsigned ch_off = group_off + 4u * (unsigned)row;  // next kernel row: one word further
        auto channels_of = [&](auto cu_tag, auto first_tag) {
            constexpr int N = decltype(cu_tag)::value;
            constexpr bool FIRST = decltype(first_tag)::value;
            uint32_t aw[N][NW];
#pragma unroll
            for (int cu = 0; cu < N; cu++)
#pragma unroll
                for (int j = 0; j < NW; j++)
                    aw[cu][j] = __builtin_amdgcn_raw_buffer_load_b32(act, (int)voff[j], (int)(ch_off + (unsigned)cu * or_b), 0);
            uint32_t wv[N * WK][C], iv[N * WK][C / 2];
#pragma unroll
            for (int l = 0; l < N * WK; l++) {
#pragma unroll
                for (int c = 0; c < C; c++) wv[l][c] = wp[l * C + c];
#pragma unroll
                for (int c = 0; c < C / 2; c++) iv[l][c] = ip[l * (C / 2) + c];
            }
#pragma unroll
            for (int cu = 0; cu < N; cu++)
#pragma unroll
                for (int u = 0; u < WK; u++) {
                    if (FIRST && cu == 0 && u == 0)
                        rail_line_first_lo(p0, p1, n0, n1, wv[0], iv[0], aw[0][0], aw[0][1]);
                    else
                        rail_line_lo(p0, p1, n0, n1, wv[cu * WK + u], iv[cu * WK + u], aw[cu][u], aw[cu][u + 1]);
                }
            wp += N * WK * C;
            ip += N * WK * (C / 2);
            ch_off += (unsigned)N * or_b;
        };
        auto channels = [&](auto cu_tag) {
            if (first)
                channels_of(cu_tag, std::true_type());
            else
                channels_of(cu_tag, std::false_type());
            first = false;
        };
        int ci = 0;
        for (; ci + CU <= chs; ci += CU) channels(std::integral_constant<int, CU>());
        if constexpr (CU > 1)
            for (; ci < chs; ci++) channels(std::integral_constant<int, 1>());
    }
    const size_t out_plane = (size_t)q.wo * q.ho;
    int32_t* yo = q.y + ((size_t)n * q.c_out + (size_t)cot * C) * out_plane + (size_t)a0 * q.ho + b;
    const bool row1 = a0 + 1 < q.wo;
    // accumulator (channel c, row r) is element 2 c + r of the 32: p0 / n0 hold channels 0 - 7, p1 / n1 8 - 15
    if constexpr (WG) {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int e = 0; e < 2 * C; e++) {
            const u32x16& pv16 = e < C ? p0 : p1;
            const u32x16& nv16 = e < C ? n0 : n1;
            atomicAdd(&red[e * 64 + lane], __popc(pv16[e % C]) - __popc(nv16[e % C]));  // result unused: ds_add_u32
        }
        __syncthreads();
        if (!live) return;
        const int n_waves = blockDim.x >> 6;
        for (int e = wave_in_wg; e < 2 * C; e += n_waves) {
            const int c = e >> 1, r = e & 1;
            if (cot * C + c < q.c_out && (r == 0 || row1)) yo[(size_t)c * out_plane + (size_t)r * q.ho] = red[e * 64 + lane];
        }
        return;
    }
    if (!live) return;
#pragma unroll
    for (int c = 0; c < C; c++) {
        if (cot * C + c >= q.c_out) break;
        const u32x16& pv16 = c < C / 2 ? p0 : p1;
        const u32x16& nv16 = c < C / 2 ? n0 : n1;
        const int e = 2 * (c % (C / 2));
        atomicAdd(yo + (size_t)c * out_plane, __popc(pv16[e]) - __popc(nv16[e]));  // integer adds: order does not matter
        if (row1) atomicAdd(yo + (size_t)c * out_plane + q.ho, __popc(pv16[e + 1]) - __popc(nv16[e + 1]));
    }
}

// The rail-skipping kernel for item-innermost activation streams (y mode, outputs with a single row: the
// SC-linear mapping, classifier layers) as a workgroup of S waves that share 128 items x 16 channels:
// every wave sums a contiguous range of (pack, kernel row) groups, the partial sums meet in LDS
// (ds_add_u32), and the workgroup stores the finished counts, channel fastest, so that the 16 channels of
// an item leave as one 64-byte run when the output has a single position (y is then (N, Cout)).  No
// zeroing pass over y, no global atomics.
// Everything that moves between groups is scalar: the activation words are read with buffer loads
// (resource over the whole stream buffer, per-lane byte offset of the lane's two items, the line's
// offset as the scalar operand), the rail-packed weight lines of a c_out tile follow each other in the
// order of the loop, so the two weight pointers only ever advance.
// Weight lines are a stream without reuse inside a wave (the 4096 x 4096 layer: 403 MB for 256 c_out
// tiles): every kTouchGroups groups the wave touches the lines of the groups after those with one vector
// load per 128 bytes, so that the scalar loads that follow find them in L2.
constexpr int kTouchGroups = 4;
template <int WK, int CU, int S>
__global__ __launch_bounds__(64 * S) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_conv_fwd_items_rail_wg(FwdParams q)
{
    constexpr int C = kCoTile, R = 2;
    __shared__ int red[R * 64 * C];  // [r][lane][c]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int cot = blockIdx.x % q.n_cotile;
    const long long slot_first = (long long)(blockIdx.x / q.n_cotile) * 64;  // always a live slot
    const long long slot0 = slot_first + lane;
    const bool live = slot0 < q.slots;
    const long long slot = live ? slot0 : slot_first;
    const int b = (int)(slot / q.row_groups);
    const long long n = slot % q.row_groups;
    // lane offsets (bytes) of the two items inside a line's words; an item past the end is clamped to
    // the first one: it only feeds an output that is never stored
    unsigned loff[R];
#pragma unroll
    for (int j = 0; j < R; j++)
        loff[j] = 4u * ((unsigned)b * q.n + (unsigned)n +
                        (n + (long long)j * q.row_groups < q.n ? (unsigned)j * q.row_groups : 0u));
    // byte strides inside the stream buffer [P][c_in][wi][hi][n] (the launcher keeps it under 4 GB)
    const unsigned pack_b = 4u * q.act_plane * (unsigned)q.n;
    const unsigned tap_b = 4u * (unsigned)q.hi * q.n;
    const unsigned row_b = 4u * (unsigned)q.n;
    const unsigned ch_b = 4u * (unsigned)q.wi * q.hi * q.n;
    const __amdgpu_buffer_rsrc_t act = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(q.act), 0,
                                                                          (int)(pack_b * (unsigned)q.packs), 0x00020000);

    int sum[2 * C];  // [2 c + r]
#pragma unroll
    for (int i = 0; i < 2 * C; i++) sum[i] = 0;

    const int k_or = q.c_in * WK;
    const int pv_begin = wave * q.pv_per_block;
    const int pv_end = min(q.packs * q.h_k, pv_begin + q.pv_per_block);
    int v = pv_begin % q.h_k;
    unsigned group_off = (unsigned)(pv_begin / q.h_k) * pack_b + (unsigned)v * row_b;
    const size_t line0 = (size_t)cot * q.rail_lines + (size_t)pv_begin * k_or;
    const uint32_t* wp = q.wgt_rail + line0 * C;
    const uint32_t* ip = q.wgt_rail_idx + line0 * (C / 2);
    // last words of this tile's rail-packed lines that a touch may read
    const uint32_t* wp_last = q.wgt_rail + ((size_t)(cot + 1) * q.rail_lines) * C - 1;
    const uint32_t* ip_last = q.wgt_rail_idx + ((size_t)(cot + 1) * q.rail_lines) * (C / 2) - 1;
    uint32_t touched = 0, touch_acc = 0;
    for (int pv = pv_begin; pv < pv_end; pv++) {
        u32x16 p0, p1, n0, n1;  // written by the group's first line
        bool first = true;
        if (((pv - pv_begin) & (kTouchGroups - 1)) == 0) {
            // the lines of groups pv + kTouchGroups .. pv + 2 kTouchGroups - 1: one lane per 128 bytes,
            // first of the words, then of the fields
            touch_acc ^= touched;  // the previous touch has long arrived: no wait in practice
            const size_t ahead = (size_t)kTouchGroups * k_or;
            const int w_lanes = kTouchGroups * k_or * C / 32;      // 128-byte pieces of the words
            const uint32_t* tw = wp + ahead * C + lane * 32;
            const uint32_t* ti = ip + ahead * (C / 2) + (lane - w_lanes) * 32;
            const uint32_t* t = lane < w_lanes ? (tw < wp_last ? tw : wp_last) : (ti < ip_last ? ti : ip_last);
            touched = *t;
        }
        unsigned ch_off = group_off;
        auto channels_of = [&](auto cu_tag, auto first_tag) {
            constexpr int N = decltype(cu_tag)::value;
            constexpr bool FIRST = decltype(first_tag)::value;
            uint32_t aw[N][WK][R];
#pragma unroll
            for (int cu = 0; cu < N; cu++)
#pragma unroll
                for (int u = 0; u < WK; u++)
#pragma unroll
                    for (int j = 0; j < R; j++)
                        aw[cu][u][j] = __builtin_amdgcn_raw_buffer_load_b32(
                            act, (int)loff[j], (int)(ch_off + (unsigned)cu * ch_b + (unsigned)u * tap_b), 0);
            uint32_t wv[N * WK][C], iv[N * WK][C / 2];
#pragma unroll
            for (int l = 0; l < N * WK; l++) {
#pragma unroll
                for (int c = 0; c < C; c++) wv[l][c] = wp[l * C + c];
#pragma unroll
                for (int c = 0; c < C / 2; c++) iv[l][c] = ip[l * (C / 2) + c];
            }
#pragma unroll
            for (int cu = 0; cu < N; cu++)
#pragma unroll
                for (int u = 0; u < WK; u++) {
                    if (FIRST && cu == 0 && u == 0)
                        rail_line_first(p0, p1, n0, n1, wv[0], iv[0], aw[0][0][0], aw[0][0][1]);
                    else
                        rail_line(p0, p1, n0, n1, wv[cu * WK + u], iv[cu * WK + u], aw[cu][u][0], aw[cu][u][1]);
                }
            wp += N * WK * C;
            ip += N * WK * (C / 2);
            ch_off += (unsigned)N * ch_b;
        };
        auto channels = [&](auto cu_tag) {
            if (first)
                channels_of(cu_tag, std::true_type());
            else
                channels_of(cu_tag, std::false_type());
            first = false;
        };
        // trips of CU channels, the remainder in trips of two where that avoids a trip of one (16
        // channels with CU = 3: 3 3 3 3 2 2)
        int left = q.c_in;
        if constexpr (CU > 2) {
            while (left >= CU + 2 || left == CU) {
                channels(std::integral_constant<int, CU>());
                left -= CU;
            }
        }
        if constexpr (CU > 1) {
            for (; left >= 2; left -= 2) channels(std::integral_constant<int, 2>());
        }
        for (; left > 0; left--) channels(std::integral_constant<int, 1>());
#pragma unroll
        for (int i = 0; i < C; i++) {
            popc_diff(sum[i], p0[i], n0[i]);
            popc_diff(sum[C + i], p1[i], n1[i]);
        }
        // next (pack, kernel row): one row further, or the first row of the next pack
        group_off += row_b;
        if (++v == q.h_k) {
            v = 0;
            group_off += pack_b - (unsigned)q.h_k * row_b;
        }
    }
    // keeps the touches alive: the values read are never used (q.keep_touches is 0)
    if (q.keep_touches && (touch_acc ^ touched) == 0x9e3779b9u) sum[0] += 1;

    // partial sums of the S waves meet in LDS: wave 0 writes, the others add
    if (wave == 0) {
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int r = 0; r < R; r++) red[(r * 64 + lane) * C + c] = sum[2 * c + r];
    }
    __syncthreads();
    if (wave != 0 && pv_begin < pv_end) {
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int r = 0; r < R; r++) atomicAdd(&red[(r * 64 + lane) * C + c], sum[2 * c + r]);
    }
    __syncthreads();
    const size_t out_plane = (size_t)q.wo * q.ho;
    for (int e = threadIdx.x; e < R * 64 * C; e += 64 * S) {
        const int c = e % C, sl = (e / C) % 64, r = e / (C * 64);
        const long long s_out = slot_first + sl;
        const int co = cot * C + c;
        if (s_out >= q.slots || co >= q.c_out) continue;
        const long long item = s_out % q.row_groups + (long long)r * q.row_groups;
        if (item >= q.n) continue;
        q.y[((size_t)item * q.c_out + co) * out_plane + (size_t)(s_out / q.row_groups)] = red[e];
    }
}

// The item-innermost kernel for OR groups of LPG = 16 one-wide lines (the SC-linear mapping with groups of
// 16 inputs), as one workgroup of 16 waves per (128 items, 8 c_out tiles): wave = (c_out tile, half of
// the (pack, kernel row) groups).  The eight waves of a half read the same activation words; per group
// every wave fetches two of the 16 lines (buffer loads, 4 dwords per lane) and leaves them in LDS, and
// all read a line back with one ds_read_b64: an eighth of the vector loads, and what a wave waits for in
// front of a line's 32 vector instructions is LDS and the scalar cache.  Groups are double-buffered
// (the loads of group t + 1 are issued before group t is computed and written to LDS after it), one
// barrier per group.  The two halves add their sums in LDS and the workgroup stores 128 items x 128
// channels, 512-byte runs per item.  With 8 position tiles x 32 tile groups (4096 x 4096 at batch 1024)
// that is 256 workgroups, one per CU, in a single round.
// The 256 workgroups walk their weight streams in step (768 KB of lines per group and L2): a touch two
// groups ahead is still in L2 when its lines are read (1 or 2 groups ahead 3.06 ms, 4: 3.19, 8: 4.43, none: 5.2).
constexpr int kLinLines = 16, kLinTiles = 8, kLinHalves = 2, kLinTouchGroups = 2;
__global__ __launch_bounds__(64 * kLinTiles * kLinHalves) __attribute__((amdgpu_waves_per_eu(4, 4)))
void k_conv_fwd_items_rail_lds(FwdParams q)
{
    constexpr int C = kCoTile, R = 2, LPG = kLinLines, NWV = kLinTiles, G = kLinHalves, LPW = LPG / NWV;
    __shared__ uint2 stage[G][2][LPG][64];           // 32 KB
    __shared__ int red[NWV][R * 64 * C];             // 64 KB
    const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int cw = wave_all % NWV, half = wave_all / NWV;
    const int cot_groups = q.n_cotile / NWV;
    const int cot = (blockIdx.x % cot_groups) * NWV + cw;
    const long long slot_first = (long long)(blockIdx.x / cot_groups) * 64;  // always a live slot
    const long long slot0 = slot_first + lane;
    const long long slot = slot0 < q.slots ? slot0 : slot_first;
    const int b = (int)(slot / q.row_groups);
    const long long n = slot % q.row_groups;
    unsigned loff[R];
#pragma unroll
    for (int j = 0; j < R; j++)
        loff[j] = 4u * ((unsigned)b * q.n + (unsigned)n +
                        (n + (long long)j * q.row_groups < q.n ? (unsigned)j * q.row_groups : 0u));
    const unsigned pack_b = 4u * q.act_plane * (unsigned)q.n;
    const unsigned row_b = 4u * (unsigned)q.n;
    const unsigned ch_b = 4u * (unsigned)q.wi * q.hi * q.n;
    const __amdgpu_buffer_rsrc_t act = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(q.act), 0,
                                                                          (int)(pack_b * (unsigned)q.packs), 0x00020000);
    int sum[2 * C];  // [2 c + r]
#pragma unroll
    for (int i = 0; i < 2 * C; i++) sum[i] = 0;

    // this half's groups (the launcher makes the halves equal: every wave meets every barrier)
    const int pv_begin = half * q.pv_per_block;
    const int n_groups = q.pv_per_block;
    int v = pv_begin % q.h_k;
    unsigned group_off = (unsigned)(pv_begin / q.h_k) * pack_b + (unsigned)v * row_b;
    const size_t line0 = (size_t)cot * q.rail_lines + (size_t)pv_begin * LPG;
    const uint32_t* wp = q.wgt_rail + line0 * C;
    const uint32_t* ip = q.wgt_rail_idx + line0 * (C / 2);
    const uint32_t* wp_last = q.wgt_rail + ((size_t)(cot + 1) * q.rail_lines) * C - 1;
    const uint32_t* ip_last = q.wgt_rail_idx + ((size_t)(cot + 1) * q.rail_lines) * (C / 2) - 1;
    uint32_t touched = 0, touch_acc = 0;

    // this wave's lines of a group: cw + NWV * i
    uint2 fetched[LPW];
    auto fetch = [&](unsigned goff) {
#pragma unroll
        for (int i = 0; i < LPW; i++) {
            const unsigned so = goff + (unsigned)(cw + NWV * i) * ch_b;
            fetched[i].x = __builtin_amdgcn_raw_buffer_load_b32(act, (int)loff[0], (int)so, 0);
            fetched[i].y = __builtin_amdgcn_raw_buffer_load_b32(act, (int)loff[1], (int)so, 0);
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < LPW; i++) stage[half][buf][cw + NWV * i][lane] = fetched[i];
    };
    auto next_group = [&]() {
        group_off += row_b;
        if (++v == q.h_k) {
            v = 0;
            group_off += pack_b - (unsigned)q.h_k * row_b;
        }
    };
    fetch(group_off);
    commit(0);
    __syncthreads();
    for (int t = 0; t < n_groups; t++) {
        const int buf = t & 1;
        const bool more = t + 1 < n_groups;
        next_group();
        if (more) fetch(group_off);
        if ((t & (kLinTouchGroups - 1)) == 0) {
            touch_acc ^= touched;
            const size_t ahead = (size_t)kLinTouchGroups * LPG;
            const int w_lanes = kLinTouchGroups * LPG * C / 32;
            const uint32_t* tw = wp + ahead * C + lane * 32;
            const uint32_t* ti = ip + ahead * (C / 2) + (lane - w_lanes) * 32;
            const uint32_t* tp = lane < w_lanes ? (tw < wp_last ? tw : wp_last) : (ti < ip_last ? ti : ip_last);
            touched = *tp;
        }
        u32x16 p0, p1, n0, n1;  // written by the group's first line
        auto lines = [&](auto n_tag, auto first_tag, int l0) {
            constexpr int N = decltype(n_tag)::value;
            constexpr bool FIRST = decltype(first_tag)::value;
            uint2 aw[N];
#pragma unroll
            for (int l = 0; l < N; l++) aw[l] = stage[half][buf][l0 + l][lane];
            uint32_t wv[N][C], iv[N][C / 2];
#pragma unroll
            for (int l = 0; l < N; l++) {
#pragma unroll
                for (int c = 0; c < C; c++) wv[l][c] = wp[l * C + c];
#pragma unroll
                for (int c = 0; c < C / 2; c++) iv[l][c] = ip[l * (C / 2) + c];
            }
#pragma unroll
            for (int l = 0; l < N; l++) {
                if (FIRST && l == 0)
                    rail_line_first(p0, p1, n0, n1, wv[0], iv[0], aw[0].x, aw[0].y);
                else
                    rail_line(p0, p1, n0, n1, wv[l], iv[l], aw[l].x, aw[l].y);
            }
            wp += N * C;
            ip += N * (C / 2);
        };
        using T3 = std::integral_constant<int, 3>;
        using T2 = std::integral_constant<int, 2>;
        lines(T3(), std::true_type(), 0);
        lines(T3(), std::false_type(), 3);
        lines(T3(), std::false_type(), 6);
        lines(T3(), std::false_type(), 9);
        lines(T2(), std::false_type(), 12);
        lines(T2(), std::false_type(), 14);
        static_assert(LPG == 16, "the trips above cover 16 lines");
#pragma unroll
        for (int i = 0; i < C; i++) {
            popc_diff(sum[i], p0[i], n0[i]);
            popc_diff(sum[C + i], p1[i], n1[i]);
        }
        if (more) commit(buf ^ 1);
        __syncthreads();
    }
    if (q.keep_touches && (touch_acc ^ touched) == 0x9e3779b9u) sum[0] += 1;

    // the two halves of a c_out tile add their sums in LDS: half 0 writes, half 1 adds
    if (half == 0) {
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int r = 0; r < R; r++) red[cw][(r * 64 + lane) * C + c] = sum[2 * c + r];
    }
    __syncthreads();
    if (half != 0) {
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int r = 0; r < R; r++) atomicAdd(&red[cw][(r * 64 + lane) * C + c], sum[2 * c + r]);
    }
    __syncthreads();
    // 128 items x (8 tiles x 16 channels): channel fastest across the tiles, 512-byte runs per item
    const size_t out_plane = (size_t)q.wo * q.ho;
    const int cot_first = (blockIdx.x % cot_groups) * NWV;
    for (int e = threadIdx.x; e < NWV * R * 64 * C; e += 64 * NWV * G) {
        const int c = e % C, tw = (e / C) % NWV, sl = (e / (C * NWV)) % 64, r = e / (C * NWV * 64);
        const long long s_out = slot_first + sl;
        const int co = (cot_first + tw) * C + c;
        if (s_out >= q.slots || co >= q.c_out) continue;
        const long long item = s_out % q.row_groups + (long long)r * q.row_groups;
        if (item >= q.n) continue;
        q.y[((size_t)item * q.c_out + co) * out_plane + (size_t)(s_out / q.row_groups)] = red[tw][(r * 64 + sl) * C + c];
    }
}

// Rail-packed weight lines from the two-rail lines [line][cot][2][16]: word = pos | neg (at most one
// is non-zero), stored [cot][line][16]; per channel a 16-bit field with what the rail kernels move
// into M0: bits 7:0 the register offset of the channel's accumulators, 2 c for the positive rail
// (and for zero weights), 32 + 2 c for the negative one, bits 15:12 the SRC2 and DST enables of
// the VGPR index mode; stored [cot][line][8].  One thread per (line, tile).
// `both` (one word, cleared by the launcher) is set when a channel of a line has two non-zero rails.
__global__ __launch_bounds__(256) void k_rail_pack(const uint32_t* __restrict__ lines2, uint32_t* __restrict__ words,
                                                   uint32_t* __restrict__ idx, size_t n_lines, int n_cotile,
                                                   uint32_t* __restrict__ both)
{
    constexpr int C = kCoTile;
    const size_t total = n_lines * n_cotile;
    bool two_rails = false;
    for (size_t l = (size_t)blockIdx.x * 256 + threadIdx.x; l < total; l += (size_t)gridDim.x * 256) {
        const size_t cot = l % n_cotile, line = l / n_cotile;
        const size_t dst = cot * n_lines + line;
        const uint32_t* src = lines2 + l * 2 * C;
        uint32_t packed[C / 2];
#pragma unroll
        for (int c2 = 0; c2 < C / 2; c2++) packed[c2] = 0;
#pragma unroll
        for (int c = 0; c < C; c++) {
            const uint32_t wp = src[c], wn = src[C + c];
            two_rails |= wp != 0u && wn != 0u;
            words[dst * C + c] = wp | wn;
            const uint32_t field = 0xC000u | ((wn != 0u ? 2u * C : 0u) + 2u * c);
            packed[c >> 1] |= field << (16 * (c & 1));
        }
#pragma unroll
        for (int c2 = 0; c2 < C / 2; c2++) idx[dst * (C / 2) + c2] = packed[c2];
    }
    if (two_rails) atomicOr(both, 1u);
}

__global__ __launch_bounds__(256) void k_zero_i32(int32_t* __restrict__ p, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) p[i] = 0;
}

// How a position-parallel launch (R accumulator rows per lane, kernel extent WK in dim 2, 0: run-time) is cut:
// waves of 64 lane slots per c_out tile, and the (pack, add group) pairs shared out over blockIdx.y.
struct SplitPlan {
    int row_groups;
    long long slots, tiles, waves;
    int pv, splits, pv_per_block;
    bool lds;  // the kernel that shares activation words through LDS
};
SplitPlan plan_splits(const Geometry& g, int R, int WK, bool rows_in_n)
{
    SplitPlan sp;
    sp.row_groups = rows_in_n ? (g.n + R - 1) / R : (g.wo + R - 1) / R;
    sp.slots = rows_in_n ? (long long)sp.row_groups * g.ho : (long long)g.n * sp.row_groups * g.ho;
    sp.tiles = (sp.slots + 63) / 64;
    sp.waves = sp.tiles * g.n_cotile;
    // Fewer than four waves per SIMD (small layers, the SC-linear mapping): split the (pack, add
    // group) sum over blockIdx.y until about twelve waves per SIMD exist, so that three resident
    // waves per SIMD stay available through the tail; the partial sums meet in y through integer
    // atomics.  Measured on MI355X: 4096x4096 linear at batch 1024 7.05 -> 6.24 ms.
    sp.pv = g.packs * g.add_outer * g.add_inner;
    int splits = 1;
    // the LDS-staged kernel: y mode, 3-wide kernels, whole chunks of 8 channels, 4 or 8 c_out tiles
    sp.lds = R == 2 && WK == 3 && !rows_in_n && g.rail && g.mode == GEO_SC_ACC_Y &&
             g.c_in % kStageChannels == 0 && g.n_cotile % 4 == 0;
    if (sp.waves < 4096) {
        splits = (int)((12288 + sp.waves - 1) / sp.waves);
        if (splits > sp.pv) splits = sp.pv;
    } else if (g.rail && !rows_in_n) {
        // Equal waves run in rounds of 4096 (four per SIMD): 3.06 rounds take the time of 4.  Splitting the
        // passes 2-, 3- or 4-fold makes the rounds shorter and the last one fuller (C5: 12544 waves, 0.77 ->
        // 0.94 of the rounded-up time); taken when it gains more than the atomics cost.
        auto fill = [&](int k) { const double r = (double)sp.waves * k / 4096.0; return r / (double)(long long)(r + 0.999999); };
        double best = fill(1) * 1.08;
        for (int k = 2; k <= 4; k++)
            if (sp.pv % k == 0 && fill(k) > best) {
                best = fill(k);
                splits = k;
            }
    }
    sp.pv_per_block = (sp.pv + splits - 1) / splits;
    sp.splits = (sp.pv + sp.pv_per_block - 1) / sp.pv_per_block;
    return sp;
}

template <int R, int WK, int CU, bool ROWS_IN_N>
int launch(const Geometry& g, FwdParams q, hipStream_t s)
{
    const SplitPlan sp = plan_splits(g, R, WK, ROWS_IN_N);
    q.row_groups = sp.row_groups;
    q.slots = sp.slots;
    const long long tiles = sp.tiles, blocks = sp.waves, waves = sp.waves;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return GEO_SC_ERR_INVALID_ARGUMENT;
    // per-lane word offsets are 32-bit
    if ((unsigned long long)R * g.packs * g.act_plane >= 0xffffffffull) return GEO_SC_ERR_UNSUPPORTED;
    if (ROWS_IN_N != g.act_item_inner) return GEO_SC_ERR_INVALID_ARGUMENT;
    const int pv = sp.pv;
    int splits = sp.splits;
    const bool lds = sp.lds;
    q.pv_per_block = sp.pv_per_block;
    const bool plain = splits == 1 && g.mode == GEO_SC_ACC_Y && !ROWS_IN_N;
    if constexpr (ROWS_IN_N) {
        static_assert(R == 2 && WK > 0, "item-innermost launches take two items per lane");
        // the kernel addresses the whole stream buffer with 32-bit byte offsets; y mode only
        if ((unsigned long long)g.act_words * 4 >= 0xffffffffull) return GEO_SC_ERR_UNSUPPORTED;
        if (!g.rail || g.mode != GEO_SC_ACC_Y) return GEO_SC_ERR_INVALID_ARGUMENT;  // make_geometry sets both with act_item_inner
        // OR groups of 16 one-wide lines with whole sets of 8 c_out tiles and enough of them to fill the
        // GPU: the workgroup that stages the activation words of its 8 tiles through LDS
        if (WK == 1 && g.c_in == kLinLines && g.n_cotile % kLinTiles == 0 && pv % kLinHalves == 0 &&
            tiles * (g.n_cotile / kLinTiles) >= 128) {
            q.pv_per_block = pv / kLinHalves;
            hipLaunchKernelGGL(k_conv_fwd_items_rail_lds, dim3((unsigned)(tiles * (g.n_cotile / kLinTiles))),
                               dim3(64 * kLinTiles * kLinHalves), 0, s, q);
            return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
        }
        // Eight waves per workgroup share the (pack, kernel row) groups of their 128 items x 16 channels
        // (the 4096 x 4096 layer at batch 1024: 4 or 16 waves 3 - 10 % slower than 8).
        constexpr int S = 8;
        q.pv_per_block = (pv + S - 1) / S;
        hipLaunchKernelGGL((k_conv_fwd_items_rail_wg<WK, CU, S>), dim3((unsigned)blocks), dim3(64 * S), 0, s, q);
        return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
    }
    // one (pack, add group) pair per wave and more than a round of waves: the form with five waves per SIMD,
    // with the pairs of a tile in one workgroup where they are few enough
    const bool pair = g.rail && R == 2 && WK > 0 && !lds && !plain && q.pv_per_block == 1 && waves * splits > 4096;
    // (in one round of five waves per SIMD only: with a second round, whole workgroups wait for ten free wave
    // slots of one CU, and the 32 -> 32 layer at 16 x 16 takes 161 us instead of 135 us)
    const bool pair_wg = pair && splits <= kPairWgMax && waves * splits <= 5 * 4 * 256;
    if (!plain && !pair_wg) {
        const size_t n_out = (size_t)g.n * g.c_out * g.wo * g.ho;
        size_t zb = (n_out + 255) / 256;
        hipLaunchKernelGGL(k_zero_i32, dim3((unsigned)(zb > 4096 ? 4096 : zb)), dim3(256), 0, s, q.y, n_out);
    }
    const dim3 grid((unsigned)blocks, (unsigned)(plain ? 1 : splits));
    if (g.rail) {
        if constexpr (R == 2 && WK > 0) {
            // two channels per trip for 1-wide kernels: with three, the six address pairs push the 32
            // sums out of the 128 registers
            constexpr int CR = WK == 1 ? 2 : 1;
            if (lds) {
                // c_out tiles of one position tile share their activation words through LDS
                // Four c_out tiles per workgroup.  With eight tiles or more, four position tiles share the
                // workgroup and its barrier (16 waves, the whole CU in step): the four waves of a c_out tile
                // read the same weight lines at the same time, which the scalar cache then serves once
                // (C3 1.38 -> 1.29 ms; 8 c_out tiles x 2 position tiles 1.31, 2 x 8 1.33).  With four tiles
                // in all the common barrier costs more than that saves (C5).
                const int nwv = 4;
                const int npt = g.n_cotile % 8 == 0 ? 4 : 1;
                const long long tile_sets = (tiles + npt - 1) / npt;
                const dim3 grid_lds((unsigned)(tile_sets * (g.n_cotile / nwv)), (unsigned)splits);
                if (npt == 4)
                    hipLaunchKernelGGL((k_conv_fwd_rail_lds<4, 4>), grid_lds, dim3(1024), 0, s, q);
                else
                    hipLaunchKernelGGL((k_conv_fwd_rail_lds<4, 1>), grid_lds, dim3(256), 0, s, q);
            } else if (plain)
                hipLaunchKernelGGL((k_conv_fwd_rail<WK, CR>), grid, dim3(64), 0, s, q);
            else if (pair_wg)
                hipLaunchKernelGGL((k_conv_fwd_pair_rail<WK, CR, true>), dim3((unsigned)blocks), dim3(64 * splits), 0, s, q,
                                   (unsigned)blocks);
            else if (pair)
                hipLaunchKernelGGL((k_conv_fwd_pair_rail<WK, CR>),
                                   dim3((unsigned)((blocks + kPairWaves - 1) / kPairWaves), (unsigned)splits),
                                   dim3(64 * kPairWaves), 0, s, q, (unsigned)blocks);
            else
                hipLaunchKernelGGL((k_conv_fwd_split_rail<WK, CR>), grid, dim3(64), 0, s, q);
        } else
            return GEO_SC_ERR_INVALID_ARGUMENT;  // make_geometry sets rail for two-row launches only
    } else if (plain)
        hipLaunchKernelGGL((k_conv_fwd<R, WK, CU, false>), grid, dim3(64), 0, s, q);
    else
        hipLaunchKernelGGL((k_conv_fwd_split<R, WK, CU, false>), grid, dim3(64), 0, s, q);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

}  // namespace

double conv_forward_cost(const Geometry& g)
{
    const double pv = (double)g.packs * g.add_outer * g.add_inner;
    if (g.thin || g.act_item_inner || g.wo < 2) {
        // lanes over OR members, or workgroups that share out the pairs themselves: no rounding modelled
        const double waves = ((double)g.n * g.wo * g.ho / 128.0 + 1.0) * g.n_cotile;
        return waves * pv / 4096.0;
    }
    const int wk = g.w_k == 1 || g.w_k == 3 || g.w_k == 5 ? g.w_k : 0;
    const SplitPlan sp = plan_splits(g, wk ? 2 : 1, wk, false);
    const double rounds = (double)((sp.waves * sp.splits + 4095) / 4096);
    return rounds * sp.pv_per_block;
}

int launch_rail_pack(const Geometry& g, uint32_t* wgt, hipStream_t s, bool from_generator)
{
    if (!g.wgt_rail) return GEO_SC_OK;
    if (from_generator && generator_packs_rails(g)) return GEO_SC_OK;  // written, flag area included, by the generator
    hipLaunchKernelGGL(k_zero_i32, dim3(1), dim3(256), 0, s, reinterpret_cast<int32_t*>(wgt + g.wgt_flag_off), (size_t)64);
    const size_t lines = g.wgt_rail_lines;
    size_t blocks = (lines * g.n_cotile + 255) / 256;
    hipLaunchKernelGGL(k_rail_pack, dim3((unsigned)(blocks > 4096 ? 4096 : blocks)), dim3(256), 0, s, wgt,
                       wgt + g.wgt_rail_off, wgt + g.wgt_rail_idx_off, lines, g.n_cotile, wgt + g.wgt_flag_off);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

int launch_conv_forward(const Geometry& g, const uint32_t* act, const uint32_t* wgt, int32_t* y, hipStream_t s)
{
    FwdParams q;
    q.act = act;
    q.wgt = wgt;
    q.wgt_rail = g.wgt_rail ? wgt + g.wgt_rail_off : nullptr;
    q.wgt_rail_idx = g.wgt_rail ? wgt + g.wgt_rail_idx_off : nullptr;
    q.rail_lines = g.wgt_rail_lines;
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
    q.keep_touches = 0;
    q.slots = 0;
    q.n = g.n;
    q.add_outer = g.add_outer;
    q.add_inner = g.add_inner;
    q.or_ch_total = g.or_ch_total;
    q.or_ch_per_group = g.or_ch_per_group;
    const unsigned ch_plane = (unsigned)g.wi * g.hi;
    q.add_stride = g.mode == GEO_SC_ACC_Z ? ch_plane : 1u;
    q.or_stride = g.mode == GEO_SC_ACC_Z ? 1u : ch_plane;
    q.or_rows = g.or_rows;
    if (g.thin) {
        const long long blocks = (long long)g.n * g.wo * g.ho * g.n_cotile;
        const long long pv = (long long)g.packs * g.add_outer * g.add_inner;
        if (blocks > 0x7fffffffLL || pv > 65535 || g.act_item_inner) return GEO_SC_ERR_INVALID_ARGUMENT;
        const size_t n_out = (size_t)g.n * g.c_out * g.wo * g.ho;
        size_t zb = (n_out + 255) / 256;
        hipLaunchKernelGGL(k_zero_i32, dim3((unsigned)(zb > 4096 ? 4096 : zb)), dim3(256), 0, s, q.y, n_out);
        hipLaunchKernelGGL(k_conv_fwd_thin, dim3((unsigned)blocks, (unsigned)pv), dim3(64), 0, s, q);
        return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
    }
    // Two accumulator rows per lane halve the weight traffic per instruction.  Outputs with
    // several rows take them along dim 2 (sliding-window reuse of activation words); outputs
    // with a single row (the SC-linear mapping, classifier layers) take two batch items.
    if (g.wo >= 2) {
        switch (g.w_k) {
        case 1: return launch<2, 1, 3, false>(g, q, s);
        case 3: return launch<2, 3, 1, false>(g, q, s);
        case 5: return launch<2, 5, 1, false>(g, q, s);
        default: return launch<1, 0, 1, false>(g, q, s);
        }
    }
    if (g.act_item_inner) {
        switch (g.w_k) {
        case 1: return launch<2, 1, 3, true>(g, q, s);
        case 3: return launch<2, 3, 1, true>(g, q, s);
        default: return launch<2, 5, 1, true>(g, q, s);
        }
    }
    switch (g.w_k) {
    case 1: return launch<1, 1, 3, false>(g, q, s);
    case 3: return launch<1, 3, 1, false>(g, q, s);
    case 5: return launch<1, 5, 1, false>(g, q, s);
    default: return launch<1, 0, 1, false>(g, q, s);
    }
}

}  // namespace geo_sc
