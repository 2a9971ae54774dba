// LFSR / comparator stream generation for gfx950.
//
// A stream bit is [code > state], the register being advanced before each comparison
// (sc.cpp:365-378, :429-432).  All six registers are maximal, so the states an element
// sees are one fixed cycle of period L-1 entered at an offset that depends on its seed
// only.  Instead of stepping a register L times per element, a table per stream length (evaluated at
// compile time, part of the code object) holds, for
// every code, the comparison results along that cycle as a bit string; an element's P
// stream words are then P funnel shifts out of the string at its seed's offset.  The few
// leading cycles that progressive loading alters are patched bit by bit from the same
// table.
#include "sc_common.h"

namespace geo_sc {

namespace {

constexpr int kGenThreads = 256;

// Fibonacci LFSR: shift left, feed back the parity of the tapped bits.
// taps (bit indices): 3:{2,1} 4:{3,2} 5:{4,2} 6:{5,4} 7:{6,5} 8:{7,5,4,3}  (sc.cpp:262-290)
constexpr uint32_t tap_mask_for(int n_bits)
{
    switch (n_bits) {
    case 3: return 0x06u;
    case 4: return 0x0Cu;
    case 5: return 0x14u;
    case 6: return 0x30u;
    case 7: return 0x60u;
    default: return 0xB8u;
    }
}

constexpr uint32_t lfsr_step(uint32_t s, uint32_t tap_mask, uint32_t state_mask)
{
    return ((s << 1) & state_mask) | ((uint32_t)__builtin_popcount(s & tap_mask) & 1u);
}

// Stream tables of one stream length L = 2^NB, evaluated by the compiler and stored in the code object:
// posp1[L] (entry L-1 unused) followed by thr[L][wpc] (see sc_common.h).  They depend on L alone, so
// no launch has to build them.
template <int NB>
struct StreamTables {
    static constexpr int L = 1 << NB, kPeriod = L - 1, kWpc = table_words_per_code(L);
    uint32_t v[L + L * kWpc];
    constexpr StreamTables() : v{}
    {
        // the register's cycle from state 1
        uint32_t cyc[L] = {};
        uint32_t s = 1;
        for (int j = 0; j < kPeriod; j++) {
            cyc[j] = s;
            s = lfsr_step(s, tap_mask_for(NB), (uint32_t)(L - 1));
        }
        for (int j = 0; j < kPeriod; j++) v[cyc[j] - 1] = (uint32_t)(j + 1);
        for (int code = 0; code < L; code++)
            for (int wi = 0; wi < kWpc; wi++) {
                int j = (wi * 32) % kPeriod;
                uint32_t word = 0;
                for (int b = 0; b < 32; b++) {
                    word = (word << 1) | (uint32_t)(code > (int)cyc[j]);
                    j = (j + 1 == kPeriod) ? 0 : j + 1;
                }
                v[L + code * kWpc + wi] = word;
            }
    }
};
__device__ const StreamTables<3> kTables8{};
__device__ const StreamTables<4> kTables16{};
__device__ const StreamTables<5> kTables32{};
__device__ const StreamTables<6> kTables64{};
__device__ const StreamTables<7> kTables128{};
__device__ const StreamTables<8> kTables256{};

__device__ __forceinline__ const uint32_t* stream_tables(int L)
{
    switch (L) {
    case 8: return kTables8.v;
    case 16: return kTables16.v;
    case 32: return kTables32.v;
    case 64: return kTables64.v;
    case 128: return kTables128.v;
    default: return kTables256.v;
    }
}

struct GenParams {
    int L, packs, bit_unit, wpc;
    int total_width, load_width, load_wait;
    int ramp;  // leading cycles whose compared code is masked by progressive loading
};

__device__ __forceinline__ int loaded_code(int code, int cycle, const GenParams& gp)
{
    // sc_cuda_kernel.cu:156-160 / :682-685
    int cw = (cycle / gp.load_wait + 1) * gp.load_width - 1;
    cw = cw > gp.total_width ? gp.total_width : cw;
    const int sh = gp.total_width - cw;
    return (code >> sh) << sh;
}

// Stream word `p` of (code, cycle offset o); thr_lds = table in LDS.
__device__ __forceinline__ uint32_t stream_word(const uint32_t* thr_lds, int code, int o, int p, const GenParams& gp)
{
    const uint32_t* row = thr_lds + code * gp.wpc;
    const int start = o + p * gp.bit_unit;
    const uint32_t hi = row[start >> 5], lo = row[(start >> 5) + 1];
    const uint64_t both = ((uint64_t)hi << 32) | lo;
    uint32_t word = (uint32_t)((both << (start & 31)) >> 32) >> (32 - gp.bit_unit);
    int nb = gp.ramp - p * gp.bit_unit;
    nb = nb > gp.bit_unit ? gp.bit_unit : nb;
    for (int b = 0; b < nb; b++) {
        const int t = p * gp.bit_unit + b;
        const int c2 = loaded_code(code, t + 1, gp);
        const int j = o + t;
        const uint32_t bit = (thr_lds[c2 * gp.wpc + (j >> 5)] >> (31 - (j & 31))) & 1u;
        const uint32_t m = 1u << (gp.bit_unit - 1 - b);
        word = (word & ~m) | (bit ? m : 0u);
    }
    return word;
}

__device__ __forceinline__ void load_tables_to_lds(uint32_t* lds, int L, int wpc)
{
    const uint32_t* __restrict__ tables = stream_tables(L);
    const int n = L + L * wpc;
    for (int i = threadIdx.x; i < n; i += kGenThreads) lds[i] = tables[i];
    __syncthreads();
}

// Activation streams from the unpadded fp32 input; padding positions produce zero words but
// keep their place in the seed numbering (sc.cpp:409-413).  Layout [n][P][c_in][Wi][Hi], or
// with ITEM_INNER [P][c_in][Wi][Hi][n]; threads run along the innermost axis of the output.
// XT: float (the activation itself) or uint8_t (the 7-bit integer k, activation k / 128).
template <bool ITEM_INNER, typename XT, int V = 1>
__global__ __launch_bounds__(kGenThreads) void k_act_streams(const XT* __restrict__ x,
                                                            uint32_t* __restrict__ streams,
                                                            GenParams gp, int n,
                                                            int c_in, int w_in, int h_in, int pad_w, int pad_h,
                                                            uint32_t seed_wrap)
{
    static_assert(V == 1 || (V == 4 && !ITEM_INNER), "four elements per thread along the item's flat index only");
    extern __shared__ uint32_t lds[];
    load_tables_to_lds(lds, gp.L, gp.wpc);
    const uint32_t* posp1 = lds;
    const uint32_t* thr = lds + gp.L;
    const int wi = w_in + 2 * pad_w, hi = h_in + 2 * pad_h;
    const uint32_t plane = (uint32_t)c_in * wi * hi;
    const size_t total = (size_t)n * plane;
    const float Lf = (float)gp.L, top = (float)(gp.L - 1);
    // V = 4: a thread takes four consecutive elements of one item (the launcher checks plane % 4 == 0 and the
    // buffer's alignment) and stores their words of a pack as one 16-byte quad
    for (size_t e = ((size_t)blockIdx.x * kGenThreads + threadIdx.x) * V; e < total;
         e += (size_t)gridDim.x * kGenThreads * V) {
        uint32_t item, i0;
        if (ITEM_INNER) {
            i0 = (uint32_t)(e / (uint32_t)n);
            item = (uint32_t)(e - (size_t)i0 * n);
        } else {
            item = (uint32_t)(e / plane);
            i0 = (uint32_t)(e - (size_t)item * plane);
        }
        int code[V], o[V];
        // coordinates and seed index of the first element by division, of the next ones by stepping
        uint32_t q = i0 % (uint32_t)hi;
        const uint32_t r0 = i0 / (uint32_t)hi;
        uint32_t p = r0 % (uint32_t)wi, c = r0 / (uint32_t)wi;
        uint32_t iw = i0 % seed_wrap, sm = iw % (uint32_t)(gp.L - 1);
#pragma unroll
        for (int j = 0; j < V; j++) {
            const int ps = (int)p - pad_w, qs = (int)q - pad_h;
            code[j] = 0;
            if (ps >= 0 && ps < w_in && qs >= 0 && qs < h_in) {
                const float v = sizeof(XT) == 1
                                    ? (float)x[(((size_t)item * c_in + c) * w_in + ps) * h_in + qs] * 0.0078125f
                                    : (float)x[(((size_t)item * c_in + c) * w_in + ps) * h_in + qs];
                // ceil(clamp(x*L, 0, L-1))  (sc.cpp:301)
                code[j] = (int)ceilf(fminf(fmaxf(v * Lf, 0.0f), top));
            }
            // seed index: flat position in the item, restarting per channel group when seed_wrap is
            // smaller than the item (sc_cuda_kernel.cu:1080)
            o[j] = (int)posp1[sm];
            if (V > 1) {
                if (++q == (uint32_t)hi) {
                    q = 0;
                    if (++p == (uint32_t)wi) {
                        p = 0;
                        ++c;
                    }
                }
                ++sm;
                if (++iw == seed_wrap) iw = sm = 0;
                if (sm == (uint32_t)(gp.L - 1)) sm = 0;
            }
        }
        if (ITEM_INNER) {
            uint32_t* dst = streams + (size_t)i0 * n + item;
            for (int pk = 0; pk < gp.packs; pk++)
                dst[(size_t)pk * plane * n] = code[0] ? stream_word(thr, code[0], o[0], pk, gp) : 0u;
        } else {
            uint32_t* dst = streams + (size_t)item * gp.packs * plane + i0;
            for (int pk = 0; pk < gp.packs; pk++) {
                uint32_t wv[V];
#pragma unroll
                for (int j = 0; j < V; j++) wv[j] = code[j] ? stream_word(thr, code[j], o[j], pk, gp) : 0u;
                if constexpr (V == 4)
                    *(uint4*)(dst + (size_t)pk * plane) = make_uint4(wv[0], wv[1], wv[2], wv[3]);
                else
                    dst[(size_t)pk * plane] = wv[0];
            }
        }
    }
}

// Weight streams, tiled layout [P][h_k][k][cotile][rail][16]; one thread per
// (h, k, padded c_out), c_out fastest so that a wave writes whole tiles.
// rail_words / rail_fields: the rail-packed copy in the same pass, [c_out tile][line][channel] with
// line = (pack, kernel row, member): the non-zero rail's word and the 16-bit M0 field of the channel's rail
// (see k_rail_pack); the first block also clears the buffer's flag area.  two_rail = 0 leaves the two-rail
// lines unwritten (a caller whose convolution kernel reads the rail-packed copy only).
__global__ __launch_bounds__(kGenThreads) void k_weight_streams(const float* __restrict__ w,
                                                               uint32_t* __restrict__ streams,
                                                               GenParams gp, int c_out, int c_in, int w_k, int h_k,
                                                               int n_cotile, uint32_t* __restrict__ rail_words,
                                                               uint16_t* __restrict__ rail_fields, size_t rail_lines,
                                                               uint32_t* __restrict__ flags, int two_rail)
{
    extern __shared__ uint32_t lds[];
    load_tables_to_lds(lds, gp.L, gp.wpc);
    const uint32_t* posp1 = lds;
    const uint32_t* thr = lds + gp.L;
    if (flags && blockIdx.x == 0 && threadIdx.x < 64) flags[threadIdx.x] = 0u;
    const int k_or = c_in * w_k;
    const int co_pad = n_cotile * kCoTile;
    const size_t total = (size_t)h_k * k_or * co_pad;
    const size_t pack_stride = (size_t)h_k * k_or * n_cotile * 2 * kCoTile;
    const float Lf = (float)gp.L, top = (float)(gp.L - 1);
    for (size_t e = (size_t)blockIdx.x * kGenThreads + threadIdx.x; e < total; e += (size_t)gridDim.x * kGenThreads) {
        const int co = (int)(e % co_pad);
        const size_t r = e / co_pad;
        const int k = (int)(r % k_or);
        const int v = (int)(r / k_or);
        const int ci = k / w_k, u = k % w_k;
        int cp = 0, cn = 0;
        if (co < c_out) {
            const float wv = w[(((size_t)co * c_in + ci) * w_k + u) * h_k + v];
            const float t = wv * Lf;
            cp = (int)ceilf(fminf(fmaxf(t, 0.0f), top));    // sc.cpp:303
            cn = (int)ceilf(-fminf(fmaxf(t, -top), 0.0f));  // sc.cpp:304
        }
        const int op = (int)posp1[(67 + k) % (gp.L - 1)];  // sc.cpp:345
        const int on = (int)posp1[(37 + k) % (gp.L - 1)];  // sc.cpp:346
        const int cot = co / kCoTile, co_l = co % kCoTile;
        const size_t base = (((size_t)v * k_or + k) * n_cotile + cot) * (2 * kCoTile) + co_l;
        for (int pk = 0; pk < gp.packs; pk++) {
            const uint32_t wp = cp ? stream_word(thr, cp, op, pk, gp) : 0u;
            const uint32_t wn = cn ? stream_word(thr, cn, on, pk, gp) : 0u;
            if (two_rail) {
                streams[pk * pack_stride + base] = wp;
                streams[pk * pack_stride + base + kCoTile] = wn;
            }
            if (rail_words) {
                const size_t dst = ((size_t)cot * rail_lines + ((size_t)pk * h_k + v) * k_or + k) * kCoTile + co_l;
                rail_words[dst] = wp | wn;
                rail_fields[dst] = (uint16_t)(0xC000u | ((cn ? 2u * kCoTile : 0u) + 2u * co_l));
            }
        }
    }
}

// Weight streams of kernels long in dim 3 (the SC linear layer's 1 x 256 rows): a block takes a
// tile of 16 output channels x 16 OR members x 16 kernel rows.  The weights come in through LDS (w is
// read in 64-byte runs along the kernel row), then a thread keeps one (channel, member) and walks the
// 16 rows: the lines of consecutive members are neighbours in the rail-packed copy, so a block writes
// it in 1 KB runs.  rail_words / rail_fields: the rail-packed copy in the same pass (these tensors are
// large: a separate pass would read all lines back): [c_out tile][line][channel], the non-zero rail's
// word and the 16-bit M0 field of the channel's rail.  two_rail = 0 leaves the two-rail lines unwritten
// (a caller whose convolution kernel reads the rail-packed copy only).
__global__ __launch_bounds__(kGenThreads) void k_weight_streams_rows(const float* __restrict__ w,
                                                                    uint32_t* __restrict__ streams,
                                                                    GenParams gp, int c_out, int c_in, int w_k,
                                                                    int h_k, int n_cotile,
                                                                    int v_chunks, uint32_t* __restrict__ rail_words,
                                                                    uint16_t* __restrict__ rail_fields,
                                                                    size_t rail_lines, uint32_t* __restrict__ flags,
                                                                    int two_rail)
{
    extern __shared__ uint32_t lds[];
    load_tables_to_lds(lds, gp.L, gp.wpc);
    if (flags && blockIdx.x == 0 && threadIdx.x < 64) flags[threadIdx.x] = 0u;
    const uint32_t* posp1 = lds;
    const uint32_t* thr = lds + gp.L;
    float* wt = reinterpret_cast<float*>(lds + gp.L + gp.L * gp.wpc);  // [row][member][channel], rows of 17
    const int k_or = c_in * w_k;
    const int k_chunks = (k_or + 15) / 16;
    const size_t pack_stride = (size_t)h_k * k_or * n_cotile * 2 * kCoTile;
    const float Lf = (float)gp.L, top = (float)(gp.L - 1);
    const size_t n_blocks = (size_t)v_chunks * k_chunks * n_cotile;
    const int co_l = threadIdx.x & 15, k_l = threadIdx.x >> 4;
    for (size_t blk = blockIdx.x; blk < n_blocks; blk += gridDim.x) {
        const int cot = (int)(blk % n_cotile);
        const size_t r = blk / n_cotile;
        const int k0 = (int)(r % k_chunks) * 16, v0 = (int)(r / k_chunks) * 16;
        __syncthreads();  // the previous tile has been read
        // element e = (channel e / 256, member (e / 16) % 16, row e % 16): 16 consecutive threads read 64 bytes
#pragma unroll 4
        for (int i = 0; i < 16; i++) {
            const int vl = threadIdx.x & 15, kl = threadIdx.x >> 4;
            const int co = cot * kCoTile + i, k = k0 + kl, v = v0 + vl;
            const bool ok = co < c_out && k < k_or && v < h_k;
            const float val = w[ok ? ((size_t)co * k_or + k) * h_k + v : 0];
            wt[(vl * 16 + kl) * 17 + i] = ok ? val : 0.0f;
        }
        __syncthreads();
        const int k = k0 + k_l;
        if (k >= k_or) continue;
        const int op = (int)posp1[(67 + k) % (gp.L - 1)];
        const int on = (int)posp1[(37 + k) % (gp.L - 1)];
        for (int vl = 0; vl < 16 && v0 + vl < h_k; vl++) {
            const int v = v0 + vl;
            const float t = wt[(vl * 16 + k_l) * 17 + co_l] * Lf;
            const int cp = (int)ceilf(fminf(fmaxf(t, 0.0f), top));
            const int cn = (int)ceilf(-fminf(fmaxf(t, -top), 0.0f));
            const size_t base = (((size_t)v * k_or + k) * n_cotile + cot) * (2 * kCoTile) + co_l;
            for (int pk = 0; pk < gp.packs; pk++) {
                const uint32_t wp = cp ? stream_word(thr, cp, op, pk, gp) : 0u;
                const uint32_t wn = cn ? stream_word(thr, cn, on, pk, gp) : 0u;
                if (two_rail) {
                    streams[pk * pack_stride + base] = wp;
                    streams[pk * pack_stride + base + kCoTile] = wn;
                }
                if (rail_words) {
                    const size_t dst = ((size_t)cot * rail_lines + ((size_t)pk * h_k + v) * k_or + k) * kCoTile + co_l;
                    rail_words[dst] = wp | wn;
                    rail_fields[dst] = (uint16_t)(0xC000u | ((cn ? 2u * kCoTile : 0u) + 2u * co_l));
                }
            }
        }
    }
}

// Weight streams of the grouped accumulation modes, same line format, lines ordered as the
// convolution kernel consumes them: [P][outer add group][inner add group][OR channel of the
// group][w_k].  z_mode: inner group = input channel, OR channel = kernel row, seed index
// u*h_k + v (sc_cuda_kernel.cu:322-324).  Otherwise: outer group = block of zu input channels,
// inner group = kernel row, seed index (channel within the block)*w_k + u (:232).
__global__ __launch_bounds__(kGenThreads) void k_weight_streams_grouped(
    const float* __restrict__ w, uint32_t* __restrict__ streams, GenParams gp, int c_out, int c_in, int w_k, int h_k, int n_cotile, int z_mode, int add_outer, int add_inner, int or_ch_total,
    int zu)
{
    extern __shared__ uint32_t lds[];
    load_tables_to_lds(lds, gp.L, gp.wpc);
    const uint32_t* posp1 = lds;
    const uint32_t* thr = lds + gp.L;
    const int co_pad = n_cotile * kCoTile;
    const size_t total = (size_t)add_outer * add_inner * zu * w_k * co_pad;
    const size_t pack_stride = (size_t)add_inner * or_ch_total * w_k * n_cotile * 2 * kCoTile;
    const float Lf = (float)gp.L, top = (float)(gp.L - 1);
    for (size_t e = (size_t)blockIdx.x * kGenThreads + threadIdx.x; e < total; e += (size_t)gridDim.x * kGenThreads) {
        const int co = (int)(e % co_pad);
        size_t r = e / co_pad;
        const int u = (int)(r % w_k);
        r /= w_k;
        const int cl = (int)(r % zu);
        r /= zu;
        const int gi = (int)(r % add_inner);
        const int go = (int)(r / add_inner);
        const int ch0 = go * zu;
        const int chs = min(zu, or_ch_total - ch0);
        if (cl >= chs) continue;  // ragged last group: no padding lines
        const int ci = z_mode ? gi : ch0 + cl;
        const int v = z_mode ? cl : gi;
        const int sidx = z_mode ? u * h_k + v : cl * w_k + u;
        int cp = 0, cn = 0;
        if (co < c_out) {
            const float wv = w[(((size_t)co * c_in + ci) * w_k + u) * h_k + v];
            const float t = wv * Lf;
            cp = (int)ceilf(fminf(fmaxf(t, 0.0f), top));
            cn = (int)ceilf(-fminf(fmaxf(t, -top), 0.0f));
        }
        const int op = (int)posp1[(67 + sidx) % (gp.L - 1)];
        const int on = (int)posp1[(37 + sidx) % (gp.L - 1)];
        const size_t line = (size_t)ch0 * add_inner * w_k + (size_t)gi * chs * w_k + (size_t)cl * w_k + u;
        const size_t base = (line * n_cotile + co / kCoTile) * (2 * kCoTile) + (co % kCoTile);
        for (int pk = 0; pk < gp.packs; pk++) {
            streams[pk * pack_stride + base] = cp ? stream_word(thr, cp, op, pk, gp) : 0u;
            streams[pk * pack_stride + base + kCoTile] = cn ? stream_word(thr, cn, on, pk, gp) : 0u;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Random stream generators (the reference's "acc" and "rand" generators, sc_cuda_kernel.cu:354-469,
// :524-545, :1319-1333, which draw from cuRAND per-thread states).  Here every element owns a
// counter-based Philox4x32-10 sequence: counter (block, index_lo, index_hi, tag), key (seed, 0);
// word j of the element is output j % 4 of block j / 4.  Results do not depend on the launch shape.
//   GEO_SC_GEN_RAND: bit t = [code > low n_bits bits of byte t % 4 of word t / 4], bytes from the
//                    least significant end: independent Bernoulli(code / L) bits.  The four comparisons
//                    of a word run as two subtractions on 16-bit lanes.
//   GEO_SC_GEN_ACC : bit t = [r16 * left_total < left_ones * 65536] with the 16-bit halves of word
//                    t / 2; left_ones -= bit, left_total -= 1: exactly `code` ones
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                              uint32_t k1, uint32_t (&out)[4])
{
#pragma unroll
    for (int r = 0; r < 10; r++) {
        // one 32 x 32 -> 64 multiply per product (v_mad_u64_u32) instead of separate high and low halves
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t h0 = (uint32_t)(p0 >> 32), l0 = (uint32_t)p0;
        const uint32_t h1 = (uint32_t)(p1 >> 32), l1 = (uint32_t)p1;
        const uint32_t n0 = h1 ^ c1 ^ k0, n2 = h0 ^ c3 ^ k1;
        c0 = n0;
        c1 = l1;
        c2 = n2;
        c3 = l0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}

struct RandParams {
    int L, n_bits, packs, bit_unit;
    int generator;  // GEO_SC_GEN_ACC or GEO_SC_GEN_RAND
    uint32_t seed;
};

// The P stream words of one element, handed to put(pack, word).  Bits are produced in stream
// order, one Philox block (four words) at a time.
template <typename Put>
__device__ __forceinline__ void random_stream(const RandParams& rp, int code, uint32_t tag, uint64_t index, Put put)
{
    if (code == 0) {
        for (int p = 0; p < rp.packs; p++) put(p, 0u);
        return;
    }
    uint32_t word = 0;
    int t = 0, in_word = 0, p = 0;
    if (rp.generator == GEO_SC_GEN_RAND) {
        // code > r on the bytes of a word, two per subtraction: with c = (code - 1) | 0x100 in both 16-bit
        // lanes and r < 0x100, bit 8 of a lane of c - r is set exactly when code - 1 >= r, and no lane borrows
        const uint32_t lane_mask = (uint32_t)(rp.L - 1) * 0x00010001u;
        const uint32_t c = (((uint32_t)code - 1u) | 0x100u) * 0x00010001u;
        for (uint32_t blk = 0; t < rp.L; blk++) {
            uint32_t r[4];
            philox4x32_10(blk, (uint32_t)index, (uint32_t)(index >> 32), tag, rp.seed, 0u, r);
#pragma unroll
            for (int w = 0; w < 4; w++) {
                if (t < rp.L) {
                    const uint32_t even = ((c - (r[w] & lane_mask)) >> 8) & 0x00010001u;         // bytes 0 and 2
                    const uint32_t odd = ((c - ((r[w] >> 8) & lane_mask)) >> 8) & 0x00010001u;   // bytes 1 and 3
                    // stream order, earlier bits more significant: byte 0, 1, 2, 3
                    const uint32_t nibble = ((even * 8u + odd * 4u) & 0xcu) | ((even >> 15) + (odd >> 16));
                    word = word * 16u + nibble;
                    t += 4;
                    in_word += 4;
                    if (in_word == rp.bit_unit) {
                        put(p++, word);
                        word = 0;
                        in_word = 0;
                    }
                }
            }
        }
        return;
    }
    uint32_t left_ones = (uint32_t)code, left_total = (uint32_t)rp.L;
    for (uint32_t blk = 0; t < rp.L; blk++) {
        uint32_t r[4];
        philox4x32_10(blk, (uint32_t)index, (uint32_t)(index >> 32), tag, rp.seed, 0u, r);
#pragma unroll
        for (int w = 0; w < 4; w++) {
            if (t < rp.L) {
#pragma unroll
                for (int f = 0; f < 2; f++) {
                    const uint32_t field = f == 0 ? (r[w] & 0xffffu) : (r[w] >> 16);
                    // both factors are below 2^24
                    const uint32_t bit = (uint32_t)__umul24(field, left_total) < (left_ones << 16);
                    left_ones -= bit;
                    left_total -= 1u;
                    word = word * 2u + bit;
                }
                t += 2;
                in_word += 2;
                if (in_word == rp.bit_unit) {
                    put(p++, word);
                    word = 0;
                    in_word = 0;
                }
            }
        }
    }
}

// Activation streams [n][P][c_in][Wi][Hi] of the random generators; element index = index0 + flat index in
// the padded tensor (n, c_in, Wi, Hi), index0 being the index of the first item when x is a slice of a
// larger batch.  Padding positions give zero words.
__global__ __launch_bounds__(kGenThreads) void k_act_streams_random(const float* __restrict__ x,
                                                                   uint32_t* __restrict__ streams, RandParams rp, int n,
                                                                   int c_in, int w_in, int h_in, int pad_w, int pad_h,
                                                                   uint64_t index0)
{
    const int wi = w_in + 2 * pad_w, hi = h_in + 2 * pad_h;
    const uint32_t plane = (uint32_t)c_in * wi * hi;
    const size_t total = (size_t)n * plane;
    const float Lf = (float)rp.L, top = (float)(rp.L - 1);
    for (size_t e = (size_t)blockIdx.x * kGenThreads + threadIdx.x; e < total; e += (size_t)gridDim.x * kGenThreads) {
        const uint32_t item = (uint32_t)(e / plane);
        const uint32_t i = (uint32_t)(e - (size_t)item * plane);
        const uint32_t q = i % (uint32_t)hi;
        const uint32_t r = i / (uint32_t)hi;
        const uint32_t p = r % (uint32_t)wi;
        const uint32_t c = r / (uint32_t)wi;
        const int ps = (int)p - pad_w, qs = (int)q - pad_h;
        int code = 0;
        if (ps >= 0 && ps < w_in && qs >= 0 && qs < h_in) {
            const float v = x[(((size_t)item * c_in + c) * w_in + ps) * h_in + qs];
            code = (int)ceilf(fminf(fmaxf(v * Lf, 0.0f), top));
        }
        uint32_t* dst = streams + (size_t)item * rp.packs * plane + i;
        random_stream(rp, code, 0u, index0 + e, [&](int pk, uint32_t word) { dst[(size_t)pk * plane] = word; });
    }
}

// Weight streams of the random generators in the tiled layout [P][h_k][k][cotile][rail][16];
// every weight element (also across c_out) has its own sequence; element index = flat index in
// (c_out, c_in, w_k, h_k), tag 1 for the positive rail and 2 for the negative rail.
__global__ __launch_bounds__(kGenThreads) void k_weight_streams_random(const float* __restrict__ w,
                                                                      uint32_t* __restrict__ streams, RandParams rp,
                                                                      int c_out, int c_in, int w_k, int h_k,
                                                                      int n_cotile)
{
    const int k_or = c_in * w_k;
    const int co_pad = n_cotile * kCoTile;
    const size_t total = (size_t)h_k * k_or * co_pad;
    const size_t pack_stride = (size_t)h_k * k_or * n_cotile * 2 * kCoTile;
    const float Lf = (float)rp.L, top = (float)(rp.L - 1);
    for (size_t e = (size_t)blockIdx.x * kGenThreads + threadIdx.x; e < total; e += (size_t)gridDim.x * kGenThreads) {
        const int co = (int)(e % co_pad);
        const size_t r = e / co_pad;
        const int k = (int)(r % k_or);
        const int v = (int)(r / k_or);
        const int ci = k / w_k, u = k % w_k;
        int cp = 0, cn = 0;
        uint64_t widx = 0;
        if (co < c_out) {
            widx = (((uint64_t)co * c_in + ci) * w_k + u) * h_k + v;
            const float t = w[widx] * Lf;
            cp = (int)ceilf(fminf(fmaxf(t, 0.0f), top));
            cn = (int)ceilf(-fminf(fmaxf(t, -top), 0.0f));
        }
        uint32_t* dst = streams + (((size_t)v * k_or + k) * n_cotile + co / kCoTile) * (2 * kCoTile) + (co % kCoTile);
        random_stream(rp, cp, 1u, widx, [&](int pk, uint32_t word) { dst[pk * pack_stride] = word; });
        random_stream(rp, cn, 2u, widx, [&](int pk, uint32_t word) { dst[pk * pack_stride + kCoTile] = word; });
    }
}

RandParams rand_params(const Geometry& g)
{
    RandParams rp;
    rp.L = g.L;
    rp.n_bits = g.n_bits;
    rp.packs = g.packs;
    rp.bit_unit = g.bit_unit;
    rp.generator = g.generator;
    rp.seed = g.seed;
    return rp;
}

GenParams gen_params(const Geometry& g, int load_wait)
{
    GenParams gp;
    gp.L = g.L;
    gp.packs = g.packs;
    gp.bit_unit = g.bit_unit;
    gp.wpc = table_words_per_code(g.L);
    gp.total_width = g.total_width;
    gp.load_width = g.load_width;
    gp.load_wait = load_wait;
    // cycles b = 1 .. m*wait-1 compare a masked code, m = ceil((tw+1)/lw) - 1
    const long long m = (g.total_width + 1 + g.load_width - 1) / g.load_width - 1;
    long long ramp = m * (long long)load_wait - 1;
    if (ramp < 0) ramp = 0;
    if (ramp > g.L) ramp = g.L;
    gp.ramp = (int)ramp;
    return gp;
}

int grid_for(size_t total)
{
    size_t blocks = (total + kGenThreads - 1) / kGenThreads;
    const size_t cap = 256 * 16;  // 256 CUs, a few blocks each; the kernels grid-stride
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (int)blocks;
}

}  // namespace

template <typename XT>
static int launch_act_streams_t(const Geometry& g, const XT* x, uint32_t* streams, hipStream_t s, size_t item0)
{
    if (g.generator != GEO_SC_GEN_LFSR) {
        if (sizeof(XT) != sizeof(float)) return GEO_SC_ERR_UNSUPPORTED;  // fp32 activations only
        const size_t n_el = (size_t)g.n * g.act_plane;
        hipLaunchKernelGGL(k_act_streams_random, dim3(grid_for(n_el)), dim3(kGenThreads), 0, s, (const float*)x,
                           streams, rand_params(g), g.n, g.c_in, g.w_in, g.h_in, g.pad_w, g.pad_h,
                           (uint64_t)item0 * g.act_plane);
        return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
    }
    const GenParams gp = gen_params(g, g.load_wait_a);
    const size_t total = (size_t)g.n * g.act_plane;
    const uint32_t wrap = (uint32_t)g.seed_wrap;
    if (g.act_item_inner)
        hipLaunchKernelGGL((k_act_streams<true, XT>), dim3(grid_for(total)), dim3(kGenThreads), table_bytes(g.L), s, x,
                           streams, gp, g.n, g.c_in, g.w_in, g.h_in, g.pad_w, g.pad_h, wrap);
    else if (g.act_plane % 4 == 0 && ((uintptr_t)streams & 15) == 0)
        hipLaunchKernelGGL((k_act_streams<false, XT, 4>), dim3(grid_for(total / 4)), dim3(kGenThreads), table_bytes(g.L),
                           s, x, streams, gp, g.n, g.c_in, g.w_in, g.h_in, g.pad_w, g.pad_h, wrap);
    else
        hipLaunchKernelGGL((k_act_streams<false, XT>), dim3(grid_for(total)), dim3(kGenThreads), table_bytes(g.L), s,
                           x, streams, gp, g.n, g.c_in, g.w_in, g.h_in, g.pad_w, g.pad_h, wrap);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

// the table the generators read for stream length L, from the host's evaluation of the same constructor
const uint32_t* stream_tables_host(int L, size_t* words)
{
    static constexpr StreamTables<3> t8{};
    static constexpr StreamTables<4> t16{};
    static constexpr StreamTables<5> t32{};
    static constexpr StreamTables<6> t64{};
    static constexpr StreamTables<7> t128{};
    static constexpr StreamTables<8> t256{};
    *words = (size_t)L + (size_t)L * table_words_per_code(L);
    switch (L) {
    case 8: return t8.v;
    case 16: return t16.v;
    case 32: return t32.v;
    case 64: return t64.v;
    case 128: return t128.v;
    case 256: return t256.v;
    default: *words = 0; return nullptr;
    }
}

int launch_act_streams(const Geometry& g, const float* x, uint32_t* streams, hipStream_t s, size_t item0)
{
    return launch_act_streams_t(g, x, streams, s, item0);
}

int launch_act_streams_q7(const Geometry& g, const uint8_t* x, uint32_t* streams, hipStream_t s)
{
    return launch_act_streams_t(g, x, streams, s, 0);
}

int launch_weight_streams(const Geometry& g, const float* w, uint32_t* streams, hipStream_t s, bool rail_only)
{
    if (g.generator != GEO_SC_GEN_LFSR) {
        const size_t n_el = (size_t)g.h_k * g.k_or * g.n_cotile * kCoTile;
        hipLaunchKernelGGL(k_weight_streams_random, dim3(grid_for(n_el)), dim3(kGenThreads), 0, s, w, streams,
                           rand_params(g), g.c_out, g.c_in, g.w_k, g.h_k, g.n_cotile);
        return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
    }
    const GenParams gp = gen_params(g, g.load_wait_w);
    if (g.mode != GEO_SC_ACC_Y && g.mode != GEO_SC_ACC_FULL) {
        const size_t padded =
            (size_t)g.add_outer * g.add_inner * g.or_ch_per_group * g.w_k * g.n_cotile * kCoTile;
        hipLaunchKernelGGL(k_weight_streams_grouped, dim3(grid_for(padded)), dim3(kGenThreads), table_bytes(g.L), s,
                           w, streams, gp, g.c_out, g.c_in, g.w_k, g.h_k, g.n_cotile,
                           g.mode == GEO_SC_ACC_Z ? 1 : 0, g.add_outer, g.add_inner, g.or_ch_total, g.or_ch_per_group);
        return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
    }
    if (weight_rows_generator(g)) {
        const int v_chunks = (g.h_k + 15) / 16, k_chunks = (g.k_or + 15) / 16;
        const size_t n_blocks = (size_t)v_chunks * k_chunks * g.n_cotile;
        const bool two_rail = !(rail_only && g.wgt_rail);
        hipLaunchKernelGGL(k_weight_streams_rows, dim3((unsigned)(n_blocks > 256 * 16 ? 256 * 16 : n_blocks)),
                           dim3(kGenThreads), table_bytes(g.L) + 16 * 16 * 17 * sizeof(float), s, w, streams, gp,
                           g.c_out, g.c_in, g.w_k, g.h_k, g.n_cotile, v_chunks,
                           g.wgt_rail ? streams + g.wgt_rail_off : nullptr,
                           g.wgt_rail ? reinterpret_cast<uint16_t*>(streams + g.wgt_rail_idx_off) : nullptr,
                           g.wgt_rail_lines, g.wgt_rail ? streams + g.wgt_flag_off : nullptr, two_rail ? 1 : 0);
        return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
    }
    const size_t total = (size_t)g.h_k * g.k_or * g.n_cotile * kCoTile;
    const bool two_rail = !(rail_only && g.wgt_rail);
    hipLaunchKernelGGL(k_weight_streams, dim3(grid_for(total)), dim3(kGenThreads), table_bytes(g.L), s, w, streams,
                       gp, g.c_out, g.c_in, g.w_k, g.h_k, g.n_cotile, g.wgt_rail ? streams + g.wgt_rail_off : nullptr,
                       g.wgt_rail ? reinterpret_cast<uint16_t*>(streams + g.wgt_rail_idx_off) : nullptr,
                       g.wgt_rail_lines, g.wgt_rail ? streams + g.wgt_flag_off : nullptr, two_rail ? 1 : 0);
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

}  // namespace geo_sc
