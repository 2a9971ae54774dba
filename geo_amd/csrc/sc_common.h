// Shared host/device definitions of the SC convolution kernels (gfx950).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "geo_sc.h"

namespace geo_sc {

// Output channels per weight tile: one tile = 16 positive-rail words + 16 negative-rail
// words = one 128-byte line, fetched by a wave as two scalar 16-dword loads.
constexpr int kCoTile = 16;

// Derived sizes of one problem; filled by make_geometry() after validation.
struct Geometry {
    int n, c_in, w_in, h_in, c_out, w_k, h_k, pad_w, pad_h;
    int L, n_bits, packs, bit_unit;
    int total_width, load_width, load_wait_w, load_wait_a;
    int mode;            // geo_sc_accumulate
    int z_unit;          // YZ: channels per OR group, clamped to c_in; otherwise c_in
    // Loop nest of the accumulation as the kernels walk it: for pack, for outer add group go <
    // add_outer, for inner add group gi < add_inner: OR over (or_ch channels of the group, w_k).
    //   Y : add_outer 1,              add_inner h_k,  OR channels = input channels
    //   YZ: add_outer channel groups, add_inner h_k,  OR channels = the group's input channels
    //   Z : add_outer 1,              add_inner c_in, OR channels = kernel rows (h_k)
    //   FULL: add_outer 1,            add_inner 1,    OR channels = input channels, and the OR also
    //         runs over or_rows = h_k kernel rows before the popcount (Y-mode weight line order)
    int add_outer, add_inner, or_ch_total, or_ch_per_group, or_rows;
    int generator;       // geo_sc_generator
    uint32_t seed;       // random generators
    size_t seed_wrap;    // activation seed index is (flat index % seed_wrap)
    int wi, hi;          // padded activation dims 2 / 3
    int wo, ho;          // output dims 2 / 3
    int k_or;            // OR-group size c_in * w_k
    int n_cotile;        // ceil(c_out / kCoTile)
    size_t act_plane;    // c_in * wi * hi words: one pack of one item
    // Activation stream layout.  false: [n][P][c_in][wi][hi].  true: [P][c_in][wi][hi][n] (batch item
    // innermost), used when the output has a single row so that the convolution kernel's lanes,
    // which then run over batch items, read consecutive words.
    bool act_item_inner;
    // Few output positions but large OR groups (classifier layers): the convolution runs with
    // lanes over the members of an OR group instead of over output positions.
    bool thin;
    size_t act_words;    // n * packs * act_plane
    // Weight stream buffer: lines [packs][h_k][k_or][n_cotile] of 2 x kCoTile words (both rails), then,
    // with rail, the same lines once more in the rail-packed form the plain y-mode kernel reads:
    // at wgt_rail_off kCoTile words per line (the non-zero rail's word), at wgt_rail_idx_off
    // kCoTile / 2 words per line (16 bits per channel: which rail), both ordered [n_cotile][line]
    // with wgt_rail_lines lines per tile.
    // Behind the rail-packed copy: wgt_flag_off, one word that the packing kernel sets when a caller's
    // line carries two non-zero rails for one channel (which the rail-packed form cannot hold), then
    // padding to 64 words.
    size_t wgt_words, wgt_rail_off, wgt_rail_idx_off, wgt_rail_lines, wgt_flag_off;
    // Position-major launches with two output rows per lane run the rail-skipping kernels: per weight
    // at most one rail's stream is non-zero (codes of clamp(w, 0, .) and -clamp(w, ., 0)), and only
    // that rail is processed.  wgt_rail: the weight stream buffer carries the rail-packed copy (a
    // property of the weights' shape alone); rail: this geometry's launch reads it.
    bool wgt_rail, rail;
};

// Stream tables (one per stream length, constant data of the code object):
//   posp1[r], r < L-1 : 1 + index in the LFSR cycle of state r+1  (cycle[0] = 1)
//   thr[code][j]      : bit string, MSB-first, of [code > cycle[j mod (L-1)]] for
//                       j < 32 * words_per_code, long enough to read L bits from any
//                       offset <= L-1 plus one spare word for the funnel shift.
constexpr __host__ __device__ int table_words_per_code(int L) { return (2 * L + 31) / 32 + 2; }
inline __host__ __device__ size_t table_bytes(int L)
{
    return sizeof(uint32_t) * ((size_t)L + (size_t)L * table_words_per_code(L));
}

const uint32_t* stream_tables_host(int L, size_t* words);

int make_geometry(const geo_sc_conv_desc* d, Geometry* g);

// Caller's choices that are not part of the problem (geo_sc_options with its defaults filled in).
struct Options {
    size_t forward_stream_bytes;    // budget of the forward's activation stream buffer
    int backward_groups_per_round;  // cap on the add groups per round of backward launches; 0: none
    bool forward_single_stream;     // a cut batch runs on the caller's stream alone
};
constexpr size_t kDefaultForwardStreamBytes = (size_t)256 << 20;

// launchers (each returns a geo_sc_status)
// item0: index of x's first item in the whole batch (the random generators number their sequences by it)
int launch_act_streams(const Geometry& g, const float* x, uint32_t* streams, hipStream_t s, size_t item0 = 0);
int launch_act_streams_q7(const Geometry& g, const uint8_t* x_q7, uint32_t* streams, hipStream_t s);
// rail_only: the caller's convolution kernel reads the rail-packed copy only; a generator that writes that
// copy itself may then leave the two-rail lines unwritten
int launch_weight_streams(const Geometry& g, const float* w, uint32_t* streams, hipStream_t s,
                          bool rail_only = false);
int launch_conv_forward(const Geometry& g, const uint32_t* act, const uint32_t* wgt, int32_t* y, hipStream_t s);
// Predicted duration of that launch in units of one wave walking one (pack, add group) pair on a full GPU:
// what the forward compares when it cuts a batch into chunks (waves run in rounds of four per SIMD, so a
// chunk whose waves fill whole rounds costs less per item).
double conv_forward_cost(const Geometry& g);
// fills the rail-packed part of a weight stream buffer from its two-rail lines (no-op unless g.wgt_rail;
// with from_generator also where launch_weight_streams has written that part itself)
int launch_rail_pack(const Geometry& g, uint32_t* wgt, hipStream_t s, bool from_generator);
// the LFSR weight generators of the y-mode line order write the rail-packed copy (and clear the flag area)
// themselves; kernels long in dim 3 take the row-chunked one
inline bool generator_packs_rails(const Geometry& g)
{
    return g.generator == GEO_SC_GEN_LFSR && (g.mode == GEO_SC_ACC_Y || g.mode == GEO_SC_ACC_FULL);
}
inline bool weight_rows_generator(const Geometry& g) { return generator_packs_rails(g) && g.h_k >= 16; }
size_t backward_workspace_bytes(const Geometry& g, int groups_per_round);
// GEO_SC_ERR_WORKSPACE when workspace_bytes is below backward_workspace_bytes(g, groups_per_round)
int launch_conv_backward(const Geometry& g, int groups_per_round, const float* x, const float* w, const float* gy,
                         float* gx, float* gw, void* workspace, size_t workspace_bytes, hipStream_t s);

}  // namespace geo_sc
