// C ABI of libgeo_sc.so: argument validation, workspace carve-up, kernel sequencing.
#include "sc_common.h"

#include <mutex>

namespace geo_sc {

namespace {
size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
}  // namespace

int make_geometry(const geo_sc_conv_desc* d, Geometry* g)
{
    if (!d || !g) return GEO_SC_ERR_INVALID_ARGUMENT;
    int n_bits;
    switch (d->bit_length) {
    case 8: n_bits = 3; break;
    case 16: n_bits = 4; break;
    case 32: n_bits = 5; break;
    case 64: n_bits = 6; break;
    case 128: n_bits = 7; break;
    case 256: n_bits = 8; break;
    default: return GEO_SC_ERR_BIT_LENGTH;
    }
    if (d->n < 1 || d->c_in < 1 || d->w_in < 1 || d->h_in < 1 || d->c_out < 1 || d->w_k < 1 || d->h_k < 1 ||
        d->pad_w < 0 || d->pad_h < 0)
        return GEO_SC_ERR_INVALID_ARGUMENT;
    if (d->total_width < 0 || d->total_width > 30 || d->load_width < 1 || d->load_wait_w < 1 || d->load_wait_a < 1)
        return GEO_SC_ERR_INVALID_ARGUMENT;
    g->n = d->n;
    g->c_in = d->c_in;
    g->w_in = d->w_in;
    g->h_in = d->h_in;
    g->c_out = d->c_out;
    g->w_k = d->w_k;
    g->h_k = d->h_k;
    g->pad_w = d->pad_w;
    g->pad_h = d->pad_h;
    g->L = d->bit_length;
    g->n_bits = n_bits;
    g->packs = (g->L + 31) / 32;
    g->bit_unit = g->L < 32 ? g->L : 32;
    g->total_width = d->total_width;
    // any load_width above total_width+1 behaves like total_width+1; clamp so that the
    // products in the kernels cannot overflow
    g->load_width = d->load_width > g->total_width + 1 ? g->total_width + 1 : d->load_width;
    g->load_wait_w = d->load_wait_w;
    g->load_wait_a = d->load_wait_a;
    if (d->accumulate < GEO_SC_ACC_Y || d->accumulate > GEO_SC_ACC_FULL) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (d->generator < GEO_SC_GEN_LFSR || d->generator > GEO_SC_GEN_RAND) return GEO_SC_ERR_INVALID_ARGUMENT;
    // the random generators exist for the Y and FULL accumulations only (sc_cuda.cpp:21-32, :65-76)
    if (d->generator != GEO_SC_GEN_LFSR && d->accumulate != GEO_SC_ACC_Y && d->accumulate != GEO_SC_ACC_FULL)
        return GEO_SC_ERR_INVALID_ARGUMENT;
    g->generator = d->generator;
    g->seed = (uint32_t)d->seed;
    if (d->accumulate == GEO_SC_ACC_YZ && d->z_unit < 1) return GEO_SC_ERR_INVALID_ARGUMENT;
    g->mode = d->accumulate;
    g->z_unit = (d->accumulate == GEO_SC_ACC_YZ && d->z_unit < d->c_in) ? d->z_unit : d->c_in;
    // YZ with a single channel group is exactly Y (same seeds, same groups)
    if (g->mode == GEO_SC_ACC_YZ && g->z_unit == d->c_in) g->mode = GEO_SC_ACC_Y;
    const long long wi = (long long)d->w_in + 2LL * d->pad_w, hi = (long long)d->h_in + 2LL * d->pad_h;
    const long long wo = wi - d->w_k + 1, ho = hi - d->h_k + 1;
    if (wo < 1 || ho < 1) return GEO_SC_ERR_INVALID_ARGUMENT;
    const long long plane = (long long)d->c_in * wi * hi;
    const long long k_or = (long long)d->c_in * d->w_k;
    if (plane > 0x7fffffffLL || k_or > 0x7fffffffLL || (long long)d->c_out * wo * ho > 0x7fffffffLL)
        return GEO_SC_ERR_INVALID_ARGUMENT;
    g->wi = (int)wi;
    g->hi = (int)hi;
    g->wo = (int)wo;
    g->ho = (int)ho;
    g->k_or = (int)k_or;
    g->n_cotile = (d->c_out + kCoTile - 1) / kCoTile;
    g->act_plane = (size_t)plane;
    g->act_words = (size_t)d->n * g->packs * g->act_plane;
    g->or_rows = 1;
    if (g->mode == GEO_SC_ACC_Z) {
        g->add_outer = 1;
        g->add_inner = d->c_in;
        g->or_ch_total = d->h_k;
        g->or_ch_per_group = d->h_k;
    } else if (g->mode == GEO_SC_ACC_FULL) {
        g->add_outer = 1;
        g->add_inner = 1;
        g->or_ch_total = d->c_in;
        g->or_ch_per_group = d->c_in;
        g->or_rows = d->h_k;
    } else {
        g->add_outer = (d->c_in + g->z_unit - 1) / g->z_unit;
        g->add_inner = d->h_k;
        g->or_ch_total = d->c_in;
        g->or_ch_per_group = g->z_unit;
    }
    g->seed_wrap = g->mode == GEO_SC_ACC_YZ ? (size_t)g->z_unit * wi * hi : (size_t)plane;
    {
        // waves the position-parallel kernel could start at most (one (pack, add group) pair per
        // wave) against the 1024 SIMDs; members of one OR group against the 64 lanes
        const long long pos_waves = (((long long)d->n * wo * ho + 63) / 64) * g->n_cotile * g->packs * g->add_outer *
                                    g->add_inner;
        const long long members = (long long)g->or_rows * g->or_ch_per_group * d->w_k;
        g->thin = pos_waves < 2048 && members >= 64;
    }
    g->act_item_inner = !g->thin && g->mode == GEO_SC_ACC_Y && g->generator == GEO_SC_GEN_LFSR && wo == 1 && d->n >= 2 && (d->w_k == 1 || d->w_k == 3 || d->w_k == 5) &&
                        (unsigned long long)g->act_words * 4 < 0xffffffffull;  // its kernel addresses the buffer with 32-bit byte offsets
    // Weight stream buffers of 1-, 3- and 5-wide kernels carry the rail-packed copy, whatever the
    // batch and input size (a buffer serves every geometry of the same weights); the launches with two
    // output rows (or, item-innermost, two batch items) per lane read it: the rail-skipping kernels.
    g->wgt_rail = d->w_k == 1 || d->w_k == 3 || d->w_k == 5;
    // (the rail-skipping kernels address the activation stream buffer with 32-bit byte offsets)
    g->rail = g->wgt_rail && !g->thin && (wo >= 2 || g->act_item_inner) &&
              (unsigned long long)g->act_words * 4 < 0xffffffffull;
    const size_t lines = (size_t)g->packs * d->h_k * g->k_or;
    g->wgt_words = lines * g->n_cotile * 2 * kCoTile;
    g->wgt_rail_off = g->wgt_rail_idx_off = g->wgt_flag_off = 0;
    g->wgt_rail_lines = lines;
    if (g->wgt_rail) {
        g->wgt_rail_off = (g->wgt_words + 63) & ~(size_t)63;
        g->wgt_rail_idx_off = g->wgt_rail_off + lines * g->n_cotile * kCoTile;
        g->wgt_flag_off = g->wgt_rail_idx_off + lines * g->n_cotile * (kCoTile / 2);
        g->wgt_words = g->wgt_flag_off + 64;
    }
    return GEO_SC_OK;
}

Options make_options(const geo_sc_options* o)
{
    Options r;
    r.forward_stream_bytes = kDefaultForwardStreamBytes;
    r.backward_groups_per_round = 0;
    r.forward_single_stream = false;
    if (o && o->struct_bytes >= sizeof(geo_sc_options)) {
        if (o->forward_stream_bytes) r.forward_stream_bytes = o->forward_stream_bytes;
        if (o->backward_groups_per_round > 0) r.backward_groups_per_round = o->backward_groups_per_round;
        r.forward_single_stream = o->forward_single_stream != 0;
    }
    return r;
}

// The forward walks the batch in chunks of `nc` items (the last one may be shorter): activation streams
// are generated for one chunk, consumed by its convolution launch, and the buffer is reused, so the
// scratch does not grow with the batch (the reference keeps streams for 128 blocks whatever the batch,
// sc_cuda_kernel.cu:658-662, :1787-1789).  Every item is independent (same seeds for every item,
// sc.cpp:409-413), so the counts do not depend on the cut.
// A cut batch uses the budget as two buffers, chunks alternating between them: a chunk's generator then runs
// while the chunk before it is still being convolved (on a second stream where the library may use one), and
// the draining tail of one convolution launch overlaps the head of the next.
struct ForwardPlan {
    Geometry chunk, last;  // geometry of a full chunk and of the shorter last one (n_last == 0: none)
    int nc, n_full, n_last;
    int buffers;           // 1: the whole batch at once; 2: chunks
    bool rail_only;        // every launch reads the rail-packed weight lines only
    size_t off_wgt, off_act[2], ws_bytes;
};

int plan_forward(const geo_sc_conv_desc* d, const Options& opt, ForwardPlan* p)
{
    Geometry g;
    int rc = make_geometry(d, &g);
    if (rc != GEO_SC_OK) return rc;
    const size_t item_bytes = sizeof(uint32_t) * (size_t)g.packs * g.act_plane;
    geo_sc_conv_desc dc = *d;
    auto geometry_of = [&](int n, Geometry* out) {
        dc.n = n;
        return make_geometry(&dc, out);
    };
    int nc = g.n;
    p->buffers = 1;
    if ((size_t)g.n * item_bytes > opt.forward_stream_bytes) {
        // two buffers of half the budget; largest chunk inside one (at least one item), then the size between
        // that and half of it whose launches fill the GPU's rounds of waves best
        p->buffers = 2;
        long long nc_max = (long long)(opt.forward_stream_bytes / 2 / item_bytes);
        if (nc_max < 1) nc_max = 1;
        if (nc_max > g.n) nc_max = g.n;
        double best = 0;
        for (long long c = nc_max; c >= (nc_max + 1) / 2; c--) {
            Geometry gc, gl;
            if ((rc = geometry_of((int)c, &gc)) != GEO_SC_OK) return rc;
            const int full = g.n / (int)c, rem = g.n - full * (int)c;
            double cost = full * (conv_forward_cost(gc) + 0.25);
            if (rem) {
                if ((rc = geometry_of(rem, &gl)) != GEO_SC_OK) return rc;
                cost += conv_forward_cost(gl) + 0.25;
            }
            if (c == nc_max || cost < best * 0.995) {
                best = cost;
                nc = (int)c;
            }
        }
    }
    p->nc = nc;
    p->n_full = g.n / nc;
    p->n_last = g.n - p->n_full * nc;
    if ((rc = geometry_of(nc, &p->chunk)) != GEO_SC_OK) return rc;
    p->last = p->chunk;
    if (p->n_last && (rc = geometry_of(p->n_last, &p->last)) != GEO_SC_OK) return rc;
    p->rail_only = p->chunk.rail && p->last.rail;
    p->off_wgt = 0;
    p->off_act[0] = align256(g.wgt_words * sizeof(uint32_t));
    p->off_act[1] = p->off_act[0] + (p->buffers == 2 ? align256((size_t)nc * item_bytes) : 0);
    p->ws_bytes = p->off_act[p->buffers - 1] + align256((size_t)nc * item_bytes);
    return GEO_SC_OK;
}

}  // namespace geo_sc

using namespace geo_sc;

// Workspace of geo_sc_conv2d_add_partial_forward_static.  In host code this name is only a handle
// for hipGetSymbolAddress; kernels get the address that call returns.
static __device__ __align__(256) unsigned char scratch[GEO_SC_STATIC_WORKSPACE_BYTES];

namespace {
// Device address of `scratch` on the current device (every GPU holds its own copy of the array at an
// address of its own), looked up once per device - by geo_sc_init, or by the first call that needs it;
// nullptr if the runtime refuses.  The lookup is not stream-ordered work: it must not happen first
// inside a stream capture.
void* static_workspace()
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* addr[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
        addr[dev] = p;
    }
    return addr[dev];
}

// The library's second stream on the current device, for the chunked forward: created once per device
// (geo_sc_init, or the first call that wants it), never inside a stream capture.  mu serialises the calls that
// enqueue on it (its two events are shared).
struct SideStream {
    std::mutex mu;
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    bool tried = false, ok = false;
};
SideStream* side_stream(hipStream_t caller)
{
    constexpr int kMaxDevices = 64;
    static std::mutex table_mu;
    static SideStream table[kMaxDevices];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(table_mu);
    SideStream& ss = table[dev];
    if (!ss.tried) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(caller, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return nullptr;  // not now: creating a stream is not capturable work
        }
        ss.tried = true;
        ss.ok = hipStreamCreateWithFlags(&ss.stream, hipStreamNonBlocking) == hipSuccess &&
                hipEventCreateWithFlags(&ss.fork, hipEventDisableTiming) == hipSuccess &&
                hipEventCreateWithFlags(&ss.join, hipEventDisableTiming) == hipSuccess;
        if (!ss.ok) (void)hipGetLastError();
    }
    return ss.ok ? &ss : nullptr;
}

// x is fp32, or with Q7 the uint8 integers k of activations k / 128
template <bool Q7>
int forward_impl(const geo_sc_conv_desc* desc, const Options& opt, const void* x, const float* w, int32_t* y,
                 void* workspace, size_t workspace_bytes, geo_sc_stream_t stream)
{
    ForwardPlan p;
    int rc = plan_forward(desc, opt, &p);
    if (rc != GEO_SC_OK) return rc;
    if (!x || !w || !y) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (!workspace || workspace_bytes < p.ws_bytes || ((uintptr_t)workspace & 255u)) return GEO_SC_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    uint32_t* wgt = (uint32_t*)(ws + p.off_wgt);
    // the weight stream buffer is the same for every batch size: generated once, read by every chunk
    if ((rc = launch_weight_streams(p.chunk, w, wgt, s, p.rail_only)) != GEO_SC_OK) return rc;
    if ((rc = launch_rail_pack(p.chunk, wgt, s, true)) != GEO_SC_OK) return rc;
    const size_t x_item = (size_t)desc->c_in * desc->w_in * desc->h_in * (Q7 ? 1 : sizeof(float));
    const size_t y_item = (size_t)desc->c_out * p.chunk.wo * p.chunk.ho;
    const int chunks = p.n_full + (p.n_last ? 1 : 0);
    // odd chunks on the library's second stream (forked behind the weight streams, joined at the end); a
    // chunk follows the chunk two before it on its own stream, which is the one that used its buffer
    SideStream* side = (chunks > 1 && !opt.forward_single_stream) ? side_stream(s) : nullptr;
    std::unique_lock<std::mutex> side_lock;
    if (side) {
        side_lock = std::unique_lock<std::mutex>(side->mu);
        if (hipEventRecord(side->fork, s) != hipSuccess || hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
            return GEO_SC_ERR_LAUNCH;
    }
    for (int c = 0; c < chunks; c++) {
        const Geometry& g = c < p.n_full ? p.chunk : p.last;
        const size_t n0 = (size_t)c * p.nc;
        const char* xc = (const char*)x + n0 * x_item;
        uint32_t* act = (uint32_t*)(ws + p.off_act[c & (p.buffers - 1)]);
        hipStream_t sc = (side && (c & 1)) ? side->stream : s;
        rc = Q7 ? launch_act_streams_q7(g, (const uint8_t*)xc, act, sc)
                : launch_act_streams(g, (const float*)xc, act, sc, n0);
        if (rc == GEO_SC_OK) rc = launch_conv_forward(g, act, wgt, y + n0 * y_item, sc);
        if (rc != GEO_SC_OK) break;
    }
    if (side) {
        // joined also after a failed launch: the caller's stream must not run ahead of what was enqueued
        if (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(s, side->join, 0) != hipSuccess)
            return GEO_SC_ERR_LAUNCH;
    }
    return rc;
}
}  // namespace

extern "C" {

int geo_sc_version(void) { return GEO_SC_VERSION; }

const char* geo_sc_status_string(int status)
{
    switch (status) {
    case GEO_SC_OK: return "ok";
    case GEO_SC_ERR_INVALID_ARGUMENT: return "invalid argument";
    case GEO_SC_ERR_BIT_LENGTH: return "stream length must be one of 8, 16, 32, 64, 128, 256";
    case GEO_SC_ERR_WORKSPACE: return "workspace missing, too small or not 256-byte aligned";
    case GEO_SC_ERR_LAUNCH: return "HIP launch failed";
    case GEO_SC_ERR_UNSUPPORTED: return "not implemented";
    default: return "unknown status";
    }
}

int geo_sc_init(void)
{
    side_stream(nullptr);  // optional: without it a cut batch runs on the caller's stream alone
    return static_workspace() ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

size_t geo_sc_static_workspace_bytes(void) { return GEO_SC_STATIC_WORKSPACE_BYTES; }

int geo_sc_conv2d_add_partial_workspace_size_ex(const geo_sc_conv_desc* desc, const geo_sc_options* options,
                                                size_t* bytes)
{
    ForwardPlan p;
    if (!bytes) return GEO_SC_ERR_INVALID_ARGUMENT;
    const int rc = plan_forward(desc, make_options(options), &p);
    if (rc != GEO_SC_OK) return rc;
    *bytes = p.ws_bytes;
    return GEO_SC_OK;
}

int geo_sc_conv2d_add_partial_workspace_size(const geo_sc_conv_desc* desc, size_t* bytes)
{
    return geo_sc_conv2d_add_partial_workspace_size_ex(desc, nullptr, bytes);
}

int geo_sc_conv2d_add_partial_forward_chunk(const geo_sc_conv_desc* desc, const geo_sc_options* options,
                                            int* items_per_chunk)
{
    ForwardPlan p;
    if (!items_per_chunk) return GEO_SC_ERR_INVALID_ARGUMENT;
    const int rc = plan_forward(desc, make_options(options), &p);
    if (rc != GEO_SC_OK) return rc;
    *items_per_chunk = p.nc;
    return GEO_SC_OK;
}

int geo_sc_stream_tables_size(int bit_length, size_t* bytes)
{
    if (!bytes) return GEO_SC_ERR_INVALID_ARGUMENT;
    switch (bit_length) {
    case 8: case 16: case 32: case 64: case 128: case 256: break;
    default: return GEO_SC_ERR_BIT_LENGTH;
    }
    *bytes = 0;  // the tables are constant data of the library
    return GEO_SC_OK;
}

int geo_sc_stream_table_copy(int bit_length, uint32_t* host_words, size_t capacity_words, size_t* words)
{
    size_t n = 0;
    const uint32_t* t = stream_tables_host(bit_length, &n);
    if (!t) return GEO_SC_ERR_BIT_LENGTH;
    if (words) *words = n;
    if (host_words) {
        if (capacity_words < n) return GEO_SC_ERR_INVALID_ARGUMENT;
        for (size_t i = 0; i < n; i++) host_words[i] = t[i];
    }
    return GEO_SC_OK;
}

int geo_sc_act_stream_words(const geo_sc_conv_desc* desc, size_t* words)
{
    Geometry g;
    if (!words) return GEO_SC_ERR_INVALID_ARGUMENT;
    const int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    *words = g.act_words;
    return GEO_SC_OK;
}

int geo_sc_act_stream_layout(const geo_sc_conv_desc* desc, int* item_innermost)
{
    Geometry g;
    if (!item_innermost) return GEO_SC_ERR_INVALID_ARGUMENT;
    const int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    *item_innermost = g.act_item_inner ? 1 : 0;
    return GEO_SC_OK;
}

int geo_sc_weight_stream_words(const geo_sc_conv_desc* desc, size_t* words)
{
    Geometry g;
    if (!words) return GEO_SC_ERR_INVALID_ARGUMENT;
    const int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    *words = g.wgt_words;
    return GEO_SC_OK;
}

int geo_sc_act_streams(const geo_sc_conv_desc* desc, const float* x, uint32_t* streams, void* tables,
                       geo_sc_stream_t stream)
{
    Geometry g;
    int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    (void)tables;
    if (!x || !streams) return GEO_SC_ERR_INVALID_ARGUMENT;
    return launch_act_streams(g, x, streams, (hipStream_t)stream);
}

int geo_sc_act_streams_q7(const geo_sc_conv_desc* desc, const uint8_t* x_q7, uint32_t* streams, void* tables,
                          geo_sc_stream_t stream)
{
    Geometry g;
    int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    (void)tables;
    if (!x_q7 || !streams) return GEO_SC_ERR_INVALID_ARGUMENT;
    return launch_act_streams_q7(g, x_q7, streams, (hipStream_t)stream);
}

int geo_sc_weight_streams(const geo_sc_conv_desc* desc, const float* w, uint32_t* streams, void* tables,
                          geo_sc_stream_t stream)
{
    Geometry g;
    int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    (void)tables;
    if (!w || !streams) return GEO_SC_ERR_INVALID_ARGUMENT;
    hipStream_t s = (hipStream_t)stream;
    rc = launch_weight_streams(g, w, streams, s);
    if (rc != GEO_SC_OK) return rc;
    return launch_rail_pack(g, streams, s, true);
}

int geo_sc_weight_streams_finish(const geo_sc_conv_desc* desc, uint32_t* streams, geo_sc_stream_t stream)
{
    Geometry g;
    const int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    if (!streams) return GEO_SC_ERR_INVALID_ARGUMENT;
    return launch_rail_pack(g, streams, (hipStream_t)stream, false);
}

int geo_sc_weight_streams_check(const geo_sc_conv_desc* desc, const uint32_t* streams, geo_sc_stream_t stream)
{
    Geometry g;
    const int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    if (!streams) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (!g.wgt_rail) return GEO_SC_OK;  // no rail-packed copy: the two-rail kernels take any lines
    uint32_t flag = 0;
    hipStream_t s = (hipStream_t)stream;
    if (hipMemcpyAsync(&flag, streams + g.wgt_flag_off, sizeof(flag), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
        return GEO_SC_ERR_LAUNCH;
    return flag ? GEO_SC_ERR_INVALID_ARGUMENT : GEO_SC_OK;
}

int geo_sc_conv2d_add_partial_from_streams(const geo_sc_conv_desc* desc, const uint32_t* act_streams,
                                           const uint32_t* weight_streams, int32_t* y, geo_sc_stream_t stream)
{
    Geometry g;
    const int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    if (!act_streams || !weight_streams || !y) return GEO_SC_ERR_INVALID_ARGUMENT;
    return launch_conv_forward(g, act_streams, weight_streams, y, (hipStream_t)stream);
}

int geo_sc_conv2d_add_partial_forward(const geo_sc_conv_desc* desc, const float* x, const float* w, int32_t* y,
                                      void* workspace, size_t workspace_bytes, geo_sc_stream_t stream)
{
    return forward_impl<false>(desc, make_options(nullptr), x, w, y, workspace, workspace_bytes, stream);
}

int geo_sc_conv2d_add_partial_forward_ex(const geo_sc_conv_desc* desc, const geo_sc_options* options, const float* x,
                                         const float* w, int32_t* y, void* workspace, size_t workspace_bytes,
                                         geo_sc_stream_t stream)
{
    return forward_impl<false>(desc, make_options(options), x, w, y, workspace, workspace_bytes, stream);
}

int geo_sc_conv2d_add_partial_forward_static(const geo_sc_conv_desc* desc, const float* x, const float* w,
                                             int32_t* y, geo_sc_stream_t stream)
{
    // the whole array is the budget: weight streams first, the rest holds the activation streams of as many
    // items at a time as fit (at least one, or the problem is too large for this entry point)
    Geometry g;
    int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    const size_t wgt_bytes = align256(g.wgt_words * sizeof(uint32_t));
    if (wgt_bytes >= GEO_SC_STATIC_WORKSPACE_BYTES) return GEO_SC_ERR_WORKSPACE;
    Options opt = make_options(nullptr);
    opt.forward_single_stream = true;   // nothing of the library's beyond the array
    opt.forward_stream_bytes = GEO_SC_STATIC_WORKSPACE_BYTES - wgt_bytes - 512;
    ForwardPlan p;
    if ((rc = plan_forward(desc, opt, &p)) != GEO_SC_OK) return rc;
    if (p.ws_bytes > GEO_SC_STATIC_WORKSPACE_BYTES) return GEO_SC_ERR_WORKSPACE;
    void* ws = static_workspace();
    if (!ws) return GEO_SC_ERR_LAUNCH;
    // Every word the kernels read from the workspace is written by this call's own kernels first
    // (all weight lines including the channel padding, the flag area, every activation word of a chunk
    // before its convolution launch), so nothing left by an earlier call needs clearing.
    return forward_impl<false>(desc, opt, x, w, y, ws, GEO_SC_STATIC_WORKSPACE_BYTES, stream);
}

int geo_sc_conv2d_add_partial_forward_q7(const geo_sc_conv_desc* desc, const uint8_t* x_q7, const float* w,
                                         int32_t* y, void* workspace, size_t workspace_bytes,
                                         geo_sc_stream_t stream)
{
    return forward_impl<true>(desc, make_options(nullptr), x_q7, w, y, workspace, workspace_bytes, stream);
}

int geo_sc_conv2d_add_partial_backward_workspace_size_ex(const geo_sc_conv_desc* desc, const geo_sc_options* options,
                                                         size_t* bytes)
{
    Geometry g;
    if (!bytes) return GEO_SC_ERR_INVALID_ARGUMENT;
    const int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    *bytes = backward_workspace_bytes(g, make_options(options).backward_groups_per_round);
    return GEO_SC_OK;
}

int geo_sc_conv2d_add_partial_backward_workspace_size(const geo_sc_conv_desc* desc, size_t* bytes)
{
    return geo_sc_conv2d_add_partial_backward_workspace_size_ex(desc, nullptr, bytes);
}

int geo_sc_conv2d_add_partial_backward_ex(const geo_sc_conv_desc* desc, const geo_sc_options* options, const float* x,
                                          const float* w, const float* grad_y, float* grad_x, float* grad_w,
                                          void* workspace, size_t workspace_bytes, geo_sc_stream_t stream)
{
    Geometry g;
    const int rc = make_geometry(desc, &g);
    if (rc != GEO_SC_OK) return rc;
    if (!x || !w || !grad_y || (!grad_x && !grad_w)) return GEO_SC_ERR_INVALID_ARGUMENT;
    if (!workspace || ((uintptr_t)workspace & 255u)) return GEO_SC_ERR_WORKSPACE;
    return launch_conv_backward(g, make_options(options).backward_groups_per_round, x, w, grad_y, grad_x, grad_w,
                                workspace, workspace_bytes, (hipStream_t)stream);
}

int geo_sc_conv2d_add_partial_backward(const geo_sc_conv_desc* desc, const float* x, const float* w,
                                       const float* grad_y, float* grad_x, float* grad_w, void* workspace,
                                       size_t workspace_bytes, geo_sc_stream_t stream)
{
    return geo_sc_conv2d_add_partial_backward_ex(desc, nullptr, x, w, grad_y, grad_x, grad_w, workspace, workspace_bytes,
                                                 stream);
}

}  // extern "C"
