/*
 * geo_sc.h - C ABI of the MI355X (gfx950) stochastic-computing convolution library
 * (libgeo_sc.so).
 *
 * The library implements, with hand-written HIP kernels, the one data-parallel path of
 * nanocad-lab/geo: LFSR/comparator bit-stream generation, the SC convolution / grouped
 * matmul forward with partial binary accumulation (OR inside a group, integer add across
 * groups) and the surrogate-gradient backward.  No torch types cross this boundary: plain
 * device pointers, sizes, a stream handle, int status codes.
 *
 * Tensor conventions are the reference's: weight (Cout, Cin, W, H) with W = dim 2 and
 * H = dim 3, H being the dimension that is accumulated with binary adders; activation
 * (N, Cin, Wx, Hx) dense NCHW fp32; output (N, Cout, Wo, Ho) int32 with
 * Wo = Wx + 2*pad_w - W + 1 and Ho = Hx + 2*pad_h - H + 1.  Stride is 1 (the reference's
 * native code accepts a stride and ignores it, sc.cpp:292, sc_cuda.cpp:47).
 *
 * All pointers are DEVICE pointers unless stated otherwise.  Every call enqueues work on
 * `stream` and returns without synchronising; the caller owns all buffers.
 */
#ifndef GEO_SC_H
#define GEO_SC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GEO_SC_VERSION 2
#define GEO_SC_API __attribute__((visibility("default")))

/* A hipStream_t, passed as an opaque pointer so that C consumers need no HIP headers.
 * NULL is the default stream. */
typedef void* geo_sc_stream_t;

enum geo_sc_status {
    GEO_SC_OK = 0,
    GEO_SC_ERR_INVALID_ARGUMENT = 1,   /* null pointer, non-positive size, kernel larger than input */
    GEO_SC_ERR_BIT_LENGTH = 2,         /* stream length not in {8,16,32,64,128,256} */
    GEO_SC_ERR_WORKSPACE = 3,          /* workspace pointer null / too small / misaligned */
    GEO_SC_ERR_LAUNCH = 4,             /* a HIP call or kernel launch failed */
    GEO_SC_ERR_UNSUPPORTED = 5         /* valid request the library does not implement */
};

/*
 * Accumulation modes.  Products of one OR group are OR-ed, groups (and stream packs) are added
 * with binary adders.
 *   GEO_SC_ACC_Y    OR over (c_in, w_k), add over h_k: conv2d_add_partial_new (sc.cpp:292) and
 *                   conv2d_add_partial_variable_acc with dim != 0 (sc_cuda.cpp:47-63)
 *   GEO_SC_ACC_Z    OR over (w_k, h_k), add over c_in: conv2d_add_partial_variable_acc with
 *                   dim == 0 (sc_cuda.cpp:57-59, sc_cuda_kernel.cu:2119-2285)
 *   GEO_SC_ACC_YZ   OR over (z_unit consecutive input channels, w_k), add over h_k and over the
 *                   ceil(c_in / z_unit) channel groups: conv2d_add_yz_variable_acc
 *                   (sc_cuda.cpp:34-45, sc_cuda_kernel.cu:1971-2116)
 *   GEO_SC_ACC_FULL OR over (c_in, w_k, h_k), add over packs only: conv2d_or_acc (sc_cuda.cpp:21-32,
 *                   sc_cuda_kernel.cu:1274-1366)
 * LFSR seeds.  Weights use (67+s) % (L-1) + 1 / (37+s) % (L-1) + 1 with s = c_in_index*w_k +
 * w_index (Y, FULL), w_index*h_k + h_index (Z, sc_cuda_kernel.cu:322-324) or (c_in_index %
 * z_unit)*w_k + w_index (YZ, :232).  Activations use i % (L-1) + 1 with i the flat index in the
 * padded item (Y, Z, FULL) or that index taken inside the channel group, i % (z_unit*Wi*Hi)
 * (YZ, :1080).
 */
enum geo_sc_accumulate { GEO_SC_ACC_Y = 0, GEO_SC_ACC_Z = 1, GEO_SC_ACC_YZ = 2, GEO_SC_ACC_FULL = 3 };

/*
 * Stream generators.  GEO_SC_GEN_LFSR: the deterministic LFSR / comparator streams.
 * GEO_SC_GEN_ACC ("accurate random", conv2d_add_partial_acc_acc, sc_cuda_kernel.cu:354-420,
 * :524-545): every activation and weight element gets a stream with exactly `code` ones at
 * uniformly random positions.  GEO_SC_GEN_RAND (conv2d_or_acc, :422-469, :1319-1333): independent
 * Bernoulli(code / L) bits.  The reference draws from cuRAND XORWOW states owned by threads, so
 * its bit sequences depend on its launch shape; here every element owns a counter-based
 * Philox4x32-10 sequence (counter: block, element index, tag 0 activation / 1 positive / 2
 * negative weight rail; key: geo_sc_conv_desc.seed): same distributions, reproducible, not
 * bit-identical to the reference.  No progressive loading; with GEO_SC_ACC_Y or _FULL only, fp32
 * activations only.
 */
enum geo_sc_generator { GEO_SC_GEN_LFSR = 0, GEO_SC_GEN_ACC = 1, GEO_SC_GEN_RAND = 2 };

/*
 * Problem description shared by all entry points.
 *
 * Progressive loading (sc_cuda_kernel.cu:155-165, :681-688): at stream cycle b = 1..L the
 * generators compare (code >> s) << s with s = total_width - min(total_width,
 * (b / load_wait + 1) * load_width - 1).  load_width >= total_width + 1 disables it, which
 * is what the reference CPU kernel computes; the reference's Python always passes
 * total_width = 7 (utils_functional.py:28, :497).
 */
typedef struct geo_sc_conv_desc {
    int32_t n;            /* batch */
    int32_t c_in;
    int32_t w_in;         /* activation dim 2, unpadded */
    int32_t h_in;         /* activation dim 3, unpadded */
    int32_t c_out;
    int32_t w_k;          /* kernel dim 2: OR-accumulated together with c_in */
    int32_t h_k;          /* kernel dim 3: binary-added */
    int32_t pad_w;        /* zero padding of dim 2, both sides */
    int32_t pad_h;        /* zero padding of dim 3, both sides */
    int32_t bit_length;   /* stream length L: 8,16,32,64,128,256 */
    int32_t total_width;  /* progressive loading, see above */
    int32_t load_width;
    int32_t load_wait_w;  /* load_wait of the weight generator */
    int32_t load_wait_a;  /* load_wait of the activation generator */
    int32_t accumulate;   /* enum geo_sc_accumulate: which products are OR-ed and which are added */
    int32_t z_unit;       /* GEO_SC_ACC_YZ: input channels per OR group (clamped to c_in); else unused */
    int32_t generator;    /* enum geo_sc_generator */
    int32_t seed;         /* key of the random generators (its 32 bits); unused with GEO_SC_GEN_LFSR */
} geo_sc_conv_desc;

/*
 * Choices of the caller that are not part of the problem.  No counterpart in the reference, whose GPU op
 * sizes and allocates its scratch itself on every call (sc_cuda_kernel.cu:1747-1796).  A NULL pointer, or a
 * zero field, means the default.  struct_bytes = sizeof(geo_sc_options) of the caller's build.
 *   forward_stream_bytes       budget of the forward's activation stream buffer.  A batch whose streams
 *                              exceed it is processed in chunks of items, each chunk's streams generated
 *                              into the same buffer and consumed by its own convolution launch (weight
 *                              streams once); the counts do not depend on the cut.  At least one item's
 *                              streams are always held.  Default 256 MiB.  The reference likewise keeps
 *                              activation streams for 128 thread blocks whatever the batch
 *                              (sc_cuda_kernel.cu:658-662, :1787-1789).  A cut batch uses the budget as two
 *                              buffers, chunks alternating, so that one chunk's streams are generated while
 *                              the chunk before it is convolved.
 *   forward_single_stream      0 (default): the odd chunks of a cut batch are enqueued on a second stream
 *                              that the library creates once per device, forked from `stream` behind the
 *                              weight streams and joined into it before the call returns (nothing of it is
 *                              visible to the caller; the fork and join are events, so the call stays
 *                              asynchronous and may be recorded into a HIP graph once geo_sc_init has run
 *                              on the device).  Non-zero: every launch on `stream` itself.
 *   backward_groups_per_round  the backward processes its add groups (kernel rows in mode Y) in rounds of
 *                              launches of as many groups as fit about 3 GB of scratch; this lowers that
 *                              number and the workspace size with it.  Default: no further cap.
 * The same options must be given to a size query and to the call that uses the workspace.
 */
typedef struct geo_sc_options {
    size_t struct_bytes;
    size_t forward_stream_bytes;
    int32_t backward_groups_per_round;
    int32_t forward_single_stream;
} geo_sc_options;

/* Library version (GEO_SC_VERSION of the build). */
GEO_SC_API int geo_sc_version(void);

/*
 * Optional.  Looks up or creates, for the current device, what the library keeps per device (the address of
 * the static workspace of geo_sc_conv2d_add_partial_forward_static; the second stream of the chunked forward).  Entry points do this themselves at their first
 * call on a device; a caller that records HIP graphs calls it once per device beforehand, because the
 * lookup is not stream-ordered work and must not happen inside a stream capture.  No counterpart in the
 * reference.
 */
GEO_SC_API int geo_sc_init(void);

/* Static, human-readable text of a status code. */
GEO_SC_API const char* geo_sc_status_string(int status);

/*
 * Bytes of device scratch the forward needs for `desc` (bit-packed weight streams + the bit-packed
 * activation streams of one chunk of the batch).  The reference allocates the same buffers itself with
 * cudaMallocManaged on every call (sc_cuda_kernel.cu:1747-1796); here the caller brings
 * them so that a framework allocator can be used.
 */
GEO_SC_API int geo_sc_conv2d_add_partial_workspace_size(const geo_sc_conv_desc* desc, size_t* bytes);
GEO_SC_API int geo_sc_conv2d_add_partial_workspace_size_ex(const geo_sc_conv_desc* desc, const geo_sc_options* options,
                                                           size_t* bytes);
/* Batch items per chunk of the forward under `options` (desc->n when the batch is not cut). */
GEO_SC_API int geo_sc_conv2d_add_partial_forward_chunk(const geo_sc_conv_desc* desc, const geo_sc_options* options,
                                                       int* items_per_chunk);

/*
 * SC convolution forward with y-dimension (H) partial binary accumulation and LFSR stream
 * generators:  float codes -> weight streams -> activation streams -> AND / OR / popcount.
 *
 * Replaces, behind one call:
 *   sc_extension.conv2d_add_partial_new                       (sc.cpp:292-472)
 *   sc_extension_cuda.conv2d_add_partial_variable_acc, dim!=0 (sc_cuda.cpp:47-63)
 *     -> conv2d_add_partial_direct_variable_cuda               (sc_cuda_kernel.cu:1732-1834)
 *     -> stream_generation_transpose_add_variable              (sc_cuda_kernel.cu:91-170)
 *     -> stream_compute_add_direct_variable                    (sc_cuda_kernel.cu:590-1004)
 *
 * x: (n, c_in, w_in, h_in) fp32;  w: (c_out, c_in, w_k, h_k) fp32;
 * y: (n, c_out, Wo, Ho) int32, fully overwritten.
 * workspace: at least the size reported above, 256-byte aligned.  The workspace holds the weight streams
 * and the activation streams of one chunk of the batch (geo_sc_options.forward_stream_bytes); the _ex form
 * takes the options, the plain form runs with the defaults.
 */
GEO_SC_API int geo_sc_conv2d_add_partial_forward(const geo_sc_conv_desc* desc, const float* x, const float* w, int32_t* y,
                                      void* workspace, size_t workspace_bytes, geo_sc_stream_t stream);
GEO_SC_API int geo_sc_conv2d_add_partial_forward_ex(const geo_sc_conv_desc* desc, const geo_sc_options* options,
                                                    const float* x, const float* w, int32_t* y, void* workspace,
                                                    size_t workspace_bytes, geo_sc_stream_t stream);

/*
 * The two stream generators on their own (the forward runs exactly these kernels).
 *
 * Activation streams: uint32 [n][P][c_in][Wi][Hi] over the PADDED item, P = ceil(L/32)
 * (in mode Y, when the output has a single row, Wo == 1, with n >= 2 and w_k in {1,3,5}, the same
 * words are stored batch-item-innermost, [P][c_in][Wi][Hi][n], which is what the convolution kernel
 * reads then);
 * element i (flat index in the padded item) starts its LFSR at i % (L-1) + 1; the register
 * advances before each comparison; bits enter MSB-first; for L < 32 a word holds L bits
 * (sc.cpp:405-438, sc_cuda_kernel.cu:662-692).
 *
 * Weight streams: uint32 [P][h_k][c_in*w_k][ceil(c_out/16)][2][16]: for each pack, kernel
 * row, OR-group member k = c_in_index*w_k + w_index and tile of 16 output channels, the 16
 * positive-rail words followed by the 16 negative-rail words (zero for c_out padding).
 * Seeds (67+k) % (L-1) + 1 / (37+k) % (L-1) + 1, one sequence per k shared by every h and
 * c_out (sc.cpp:336-388, sc_cuda_kernel.cu:91-170).  Modes Z and YZ keep the line format and
 * order the lines by (pack, add group, OR member): Z [P][c_in][h_k*w_k] with member
 * h_index*w_k + w_index; YZ [P][channel group][h_k][channels of the group * w_k].
 * A weight has at most one non-zero rail (its codes are those of clamp(w, 0, .) and
 * -clamp(w, ., 0), sc.cpp:301-304).  For 1-, 3- and 5-wide kernels the buffer continues behind these
 * lines with a second, rail-packed copy that the convolution kernel reads there (per line 16
 * words pos | neg, then per line 8 words holding 16 bits per channel: which rail);
 * geo_sc_weight_stream_words is the size of the whole buffer, geo_sc_weight_streams fills all of it.
 *
 * `tables` is not used and may be NULL: the comparison tables of the six stream lengths are constant
 * data of the library (until version 1 they were built per call into this scratch);
 * geo_sc_stream_tables_size reports 0 bytes.  The arguments remain so that callers need not change.
 * These stage entry points work on the whole batch at once (no chunks): above 4 GiB of activation streams
 * geo_sc_conv2d_add_partial_from_streams runs the kernels that process both rails (about half the speed),
 * and the item-innermost layout is not used.
 */
GEO_SC_API int geo_sc_stream_tables_size(int bit_length, size_t* bytes);
/*
 * The comparison table of one stream length as the generators read it, copied to HOST memory (for
 * inspection and tests; no GPU needed): posp1[L], then thr[L][wpc] with wpc = (2 L + 31) / 32 + 2.
 * posp1[s - 1] = 1 + index of LFSR state s in the register's cycle from state 1 (sc.cpp:262-290;
 * entry L - 1 unused); thr[code] = the bits [code > cycle[j mod (L - 1)]], j = 0, 1, ..., MSB-first.
 * *words receives the table's size; host_words may be NULL to query it.
 */
GEO_SC_API int geo_sc_stream_table_copy(int bit_length, uint32_t* host_words, size_t capacity_words, size_t* words);
GEO_SC_API int geo_sc_act_streams(const geo_sc_conv_desc* desc, const float* x, uint32_t* streams, void* tables,
                       geo_sc_stream_t stream);
GEO_SC_API int geo_sc_weight_streams(const geo_sc_conv_desc* desc, const float* w, uint32_t* streams, void* tables,
                          geo_sc_stream_t stream);
/*
 * The AND / OR / popcount kernel alone, on streams in the two layouts above (what the
 * forward runs after its generators; the body of stream_compute_add_direct_variable,
 * sc_cuda_kernel.cu:693-1002, and of matmul_outer, sc.cpp:12-259).  y is fully overwritten.
 * weight_streams is a buffer of geo_sc_weight_stream_words words as geo_sc_weight_streams fills it.
 */
GEO_SC_API int geo_sc_conv2d_add_partial_from_streams(const geo_sc_conv_desc* desc, const uint32_t* act_streams,
                                                      const uint32_t* weight_streams, int32_t* y,
                                                      geo_sc_stream_t stream);
/*
 * For callers that write the two-rail weight lines themselves (layout above) into a buffer of
 * geo_sc_weight_stream_words words: fills the rest of the buffer (the rail-packed copy) from those
 * lines.  geo_sc_weight_streams does this itself.  Every (line, channel) must have at most one
 * non-zero rail, as streams of the reference's codes have (sc.cpp:301-304); the rail-packed form
 * cannot hold two.  A line that breaks the rule is recorded in the buffer (its last 64 words are a
 * flag area) and reported by geo_sc_weight_streams_check, which waits for `stream` and returns
 * GEO_SC_ERR_INVALID_ARGUMENT for such a buffer, GEO_SC_OK otherwise (also for buffers filled by
 * geo_sc_weight_streams and for kernel widths that carry no rail-packed copy).  Counts computed from
 * a buffer that fails the check are undefined.
 */
GEO_SC_API int geo_sc_weight_streams_finish(const geo_sc_conv_desc* desc, uint32_t* streams, geo_sc_stream_t stream);
GEO_SC_API int geo_sc_weight_streams_check(const geo_sc_conv_desc* desc, const uint32_t* streams,
                                           geo_sc_stream_t stream);
/* Word counts of the two stream buffers above; *item_innermost = 1 when the activation streams of `desc`
 * are stored batch-item-innermost ([P][c_in][Wi][Hi][n]), 0 for [n][P][c_in][Wi][Hi]. */
GEO_SC_API int geo_sc_act_stream_words(const geo_sc_conv_desc* desc, size_t* words);
GEO_SC_API int geo_sc_act_stream_layout(const geo_sc_conv_desc* desc, int* item_innermost);
GEO_SC_API int geo_sc_weight_stream_words(const geo_sc_conv_desc* desc, size_t* words);

/*
 * Backward of the layer through the reference's floating-point surrogate
 * (utils_functional.py:611-634 with conv2d_or_bin_1d, :235-252; differentiated there by
 * torch autograd, there is no native counterpart in the reference):
 *     wp = clamp(w, 0, 100), wn = -clamp(w, -100, 0), x~ = zero-padded x
 *     z+-_v = corr2d(x~[..., v : v+Ho], w+-[..., v:v+1]),   v < h_k
 *     y^    = sum_v (1 - exp(-z+_v)) - sum_v (1 - exp(-z-_v))
 * grad_x (n, c_in, w_in, h_in) = d y^ / d x contracted with grad_y (padding sliced off);
 * grad_w (c_out, c_in, w_k, h_k) = d y^ / d w contracted with grad_y, clamp passing its
 * gradient on the closed interval.  fp32 throughout, fp32 accumulation.  Either output may
 * be NULL to skip it.  bit_length and the loading fields of `desc` are validated but do not
 * enter the result.
 * The add groups (kernel rows in mode Y) are processed in rounds of launches of as many groups as
 * fit about 3 GB of scratch; geo_sc_options.backward_groups_per_round (the _ex forms) lowers that number
 * and the workspace size with it.  The result does not depend on it beyond fp32 summation order of grad_x.
 */
GEO_SC_API int geo_sc_conv2d_add_partial_backward_workspace_size(const geo_sc_conv_desc* desc, size_t* bytes);
GEO_SC_API int geo_sc_conv2d_add_partial_backward(const geo_sc_conv_desc* desc, const float* x, const float* w,
                                                  const float* grad_y, float* grad_x, float* grad_w,
                                                  void* workspace, size_t workspace_bytes, geo_sc_stream_t stream);
GEO_SC_API int geo_sc_conv2d_add_partial_backward_workspace_size_ex(const geo_sc_conv_desc* desc,
                                                                    const geo_sc_options* options, size_t* bytes);
GEO_SC_API int geo_sc_conv2d_add_partial_backward_ex(const geo_sc_conv_desc* desc, const geo_sc_options* options,
                                                     const float* x, const float* w, const float* grad_y,
                                                     float* grad_x, float* grad_w, void* workspace,
                                                     size_t workspace_bytes, geo_sc_stream_t stream);

/*
 * Layer epilogue fused into one pass over the convolution's int32 counts.  Replaces the chain of
 * PyTorch element-wise ops between two SC layers of the reference's networks
 * (network.py:165-170): count / L (utils_functional.py:632) -> value of BatchNorm2d_fixed /
 * BatchNorm1d_fixed, x * w_n[c] + b_n[c] with the caller's quantised per-channel w_n, b_n
 * (utils_class.py:52-64) -> optional relu (network.py:167) -> optional AvgPool2d(2) (:169) ->
 * optional Hardtanh(0, 1) (:170) -> optional round(v * 128).clamp(-127, 127) / 128, the next
 * layer's input quantisation (utils_class.py:32, utils_functional.py:33-39).  Same operation order
 * and rounding as the op chain: the fp32 result is identical.
 *   counts            int32 (n, c, w, h)
 *   act_out           fp32 (n, c, wo, ho), wo = w/2, ho = h/2 with GEO_SC_EPI_POOL2 (floor), else w, h;
 *                     may be NULL when q7_out is given
 *   q7_out            uint8 (n, c, wo, ho): the integer round(v * 128) in [0, 127]; may be NULL; needs
 *                     GEO_SC_EPI_HARDTANH01 | GEO_SC_EPI_QUANT7
 */
enum geo_sc_epilogue_flags {
    GEO_SC_EPI_RELU = 1,
    GEO_SC_EPI_POOL2 = 2,
    GEO_SC_EPI_HARDTANH01 = 4,
    GEO_SC_EPI_QUANT7 = 8
};
GEO_SC_API int geo_sc_layer_epilogue(const int32_t* counts, int n, int c, int w, int h, int bit_length,
                                     const float* w_n, const float* b_n, int flags, float* act_out,
                                     uint8_t* q7_out, geo_sc_stream_t stream);

/*
 * Backward of the same tail in training mode, in which the reference's graph is
 * y = count / L -> F.batch_norm(y, training=True) with its value replaced by y * w_n + b_n
 * (utils_class.py:49-64) -> relu -> AvgPool2d(2) -> Hardtanh(0, 1) (network.py:165-170): the
 * gradient of an ordinary batch norm on the batch statistics, with the relu / hardtanh masks taken
 * from the fixed-point values that flowed forward; the quantisation passes the gradient through.
 *   counts, w_n, b_n, flags   as given to geo_sc_layer_epilogue in the forward
 *   grad_out                  fp32 (n, c, wo, ho): gradient with respect to the tail's output
 *   mean, invstd              per channel: batch mean of y and 1 / sqrt(biased variance + eps)
 *   gamma                     the batch norm's weight, or NULL for 1
 *   grad_y                    fp32 (n, c, w, h): gradient with respect to y = count / L
 *   grad_gamma, grad_beta     per channel, may be NULL
 * Deterministic (fixed summation order).  Workspace: geo_sc_layer_tail_backward_workspace_size.  At most 4096
 * channels.
 */
GEO_SC_API int geo_sc_layer_tail_backward_workspace_size(int n, int c, int w, int h, size_t* bytes);
GEO_SC_API int geo_sc_layer_tail_backward(const int32_t* counts, const float* grad_out, int n, int c, int w, int h,
                                          int bit_length, const float* w_n, const float* b_n, const float* mean,
                                          const float* invstd, const float* gamma, int flags, float* grad_y,
                                          float* grad_gamma, float* grad_beta, void* workspace,
                                          size_t workspace_bytes, geo_sc_stream_t stream);

/*
 * The channel statistics BatchNorm2d_fixed / BatchNorm1d_fixed take of an SC layer's output
 * (utils_class.py:52-56: mean and biased variance over batch and positions of y = counts / bit_length), from the
 * integer counts (n, c, w, h): the sums of the counts and of their squares are exact 64-bit integers, the two
 * results are formed from them in double precision and rounded to fp32 once, so they do not depend on a
 * reduction order.  mean, var: c floats each on the device.  Workspace: geo_sc_count_stats_workspace_size
 * bytes, 8-byte aligned.
 */
GEO_SC_API int geo_sc_count_stats_workspace_size(int n, int c, int w, int h, size_t* bytes);
GEO_SC_API int geo_sc_count_stats(const int32_t* counts, int n, int c, int w, int h, int bit_length, float* mean,
                                  float* var, void* workspace, size_t workspace_bytes, geo_sc_stream_t stream);

/*
 * The per-channel fixed-point affine of BatchNorm2d_fixed / BatchNorm1d_fixed from channel statistics
 * (utils_class.py:52-62, quantize_shift utils_functional.py:41-57) in one launch:
 * w = gamma / sqrt(var + eps), b = beta - mean * gamma / sqrt(var + eps), both rounded to 8 bits under
 * the shared power-of-two scale 2 ** ceil(log2(mean(w) * 3)).  gamma / beta may be NULL (1 / 0).
 * Optional outputs: invstd = 1 / sqrt(var + eps_grad) for geo_sc_layer_tail_backward; the running
 * statistics updated as F.batch_norm(training=True) does (momentum 0.1, variance unbiased by
 * elements_per_channel / (elements_per_channel - 1)); scale (one float).  All pointers are device
 * pointers to c floats.
 */
GEO_SC_API int geo_sc_bn_fixed_affine(const float* mean, const float* var, const float* gamma, const float* beta,
                                      int c, float eps, float eps_grad, long long elements_per_channel,
                                      float* running_mean, float* running_var, float* w_n, float* b_n, float* invstd,
                                      float* scale, geo_sc_stream_t stream);

/*
 * geo_sc_count_stats and geo_sc_bn_fixed_affine in two launches instead of three: the channel statistics of
 * y = counts / bit_length from exact integer sums (written to mean, var: c floats each), then the fixed-point
 * affine, 1 / sqrt(var + eps_grad) and the running statistics from them (utils_class.py:49-62), the number of
 * elements per channel being n * w * h.  Same values as the two calls.  Workspace:
 * geo_sc_count_stats_workspace_size bytes, 8-byte aligned.
 */
GEO_SC_API int geo_sc_bn_fixed_from_counts(const int32_t* counts, int n, int c, int w, int h, int bit_length,
                                           const float* gamma, const float* beta, float eps, float eps_grad,
                                           float* running_mean, float* running_var, float* mean, float* var,
                                           float* w_n, float* b_n, float* invstd, float* scale, void* workspace,
                                           size_t workspace_bytes, geo_sc_stream_t stream);

/*
 * quantize (utils_functional.py:33-39) in one pass: dst = clamp(round(src * 2^prec), -(2^prec - 1), 2^prec - 1)
 * / 2^prec, rounding half to even as torch.round does; prec 1..23.  The layer applies it to its input
 * and to weight_org on every call (utils_class.py:32-33).  n fp32 elements on the device; dst may be src.
 */
GEO_SC_API int geo_sc_quantize(const float* src, float* dst, size_t n, int prec, geo_sc_stream_t stream);
/* The same for `count` tensors in one launch per 24 of them (the weight_org buffers of all layers of a network
 * at the start of a forward): src, dst and elements are HOST arrays of `count` entries, the tensors are on the
 * device; a tensor of no elements may have null pointers. */
GEO_SC_API int geo_sc_quantize_many(int count, const float* const* src, float* const* dst, const size_t* elements,
                                    int prec, geo_sc_stream_t stream);

/*
 * The end of the reference's training step (utils_own.py:108-113) in one launch per 24 of `count` parameters:
 * param[i] <- master[i] (the optimiser's full-precision copy, `elements[i]` floats), and where org[i] is not
 * NULL (a layer's weight_org buffer) org[i] <- clamp(master[i], lo, hi).  master, param, org (may be NULL
 * altogether) and elements are HOST arrays of `count` entries; the tensors are on the device.
 */
GEO_SC_API int geo_sc_copy_back_clamp(int count, const float* const* master, float* const* param, float* const* org,
                                      const size_t* elements, float lo, float hi, geo_sc_stream_t stream);

/*
 * geo_sc_conv2d_add_partial_forward for activations given as the 7-bit integers k = round(x * 128)
 * that geo_sc_layer_epilogue emits (uint8 (n, c_in, w_in, h_in), k <= 127): the activation is
 * x = k / 128, exactly what the reference's layer computes from after its input quantisation
 * (utils_class.py:32), so the counts equal those of the fp32 entry point on x.  Same workspace.
 */
GEO_SC_API int geo_sc_conv2d_add_partial_forward_q7(const geo_sc_conv_desc* desc, const uint8_t* x_q7,
                                                    const float* w, int32_t* y, void* workspace,
                                                    size_t workspace_bytes, geo_sc_stream_t stream);

/* geo_sc_act_streams for the uint8 7-bit integer activations of geo_sc_conv2d_add_partial_forward_q7:
 * with weight streams generated once by geo_sc_weight_streams, an inference loop runs this, then
 * geo_sc_conv2d_add_partial_from_streams, then geo_sc_layer_epilogue per layer. */
GEO_SC_API int geo_sc_act_streams_q7(const geo_sc_conv_desc* desc, const uint8_t* x_q7, uint32_t* streams,
                                     void* tables, geo_sc_stream_t stream);

/*
 * geo_sc_conv2d_add_partial_forward for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and result, without the workspace: both stream buffers live
 * in a static device array of GEO_SC_STATIC_WORKSPACE_BYTES inside the library, which every GPU the
 * library runs on holds until the process ends.  The call allocates and frees nothing and clears
 * nothing with memset nodes.  The array is the activation stream budget: the weight streams come first,
 * the batch is cut into chunks whose streams fit behind them.  A problem whose weight streams plus one
 * item's activation streams exceed the array returns GEO_SC_ERR_WORKSPACE.  All calls on one GPU share
 * that GPU's array: calls that overlap on one GPU (different streams, different threads) race; calls on one
 * stream do not.  Under stream capture: call geo_sc_init (or this entry point once) on the device before
 * the capture begins.  geo_sc_static_workspace_bytes returns the limit of the loaded library.
 */
#define GEO_SC_STATIC_WORKSPACE_BYTES ((size_t)32 << 20)
GEO_SC_API int geo_sc_conv2d_add_partial_forward_static(const geo_sc_conv_desc* desc, const float* x, const float* w,
                                                        int32_t* y, geo_sc_stream_t stream);
GEO_SC_API size_t geo_sc_static_workspace_bytes(void);

#ifdef __cplusplus
}
#endif
#endif /* GEO_SC_H */
