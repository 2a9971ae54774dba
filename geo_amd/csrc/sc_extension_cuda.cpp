// PyTorch module `sc_extension_cuda`: the GPU entry points the reference's Python binds by
// name (utils_functional.py:12, call sites :497-513; C++ side sc_cuda.cpp:21-83), same
// positional signatures, implemented on libgeo_sc.so (gfx950).
#include "sc_torch_common.h"

using namespace geo_sc_torch;

// sc_cuda.cpp:47-63.  dim != 0: y-dimension partial binary accumulation (the default of the
// reference's training script): OR over (c_in, w_k), add over h_k.  dim == 0: z-dimension
// accumulation: OR over the kernel window, add over c_in.
at::Tensor conv2d_add_partial_variable_acc(torch::Tensor input, torch::Tensor weight, int64_t bit_length,
                                           at::IntArrayRef padding, at::IntArrayRef stride, int64_t total_width,
                                           int64_t load_width, int64_t load_wait, bool im2col, int64_t dim)
{
    (void)stride;  // accepted and ignored, as in the reference (stride 1 only)
    (void)im2col;  // selects an equivalent kernel variant in the reference; no effect on results
    // the y/z ops use one load_wait for weights and activations (sc_cuda_kernel.cu:1821-1823, :2119)
    const geo_sc_conv_desc d = make_desc(input, weight, bit_length, padding, total_width, load_width, load_wait,
                                         load_wait, dim == 0 ? GEO_SC_ACC_Z : GEO_SC_ACC_Y);
    return forward_on_device(input, weight, d);
}

// sc_cuda.cpp:34-45: OR over (z_unit consecutive input channels, w_k), add over h_k and over
// the channel groups; separate load_wait for the weight and activation generators.
at::Tensor conv2d_add_yz_variable_acc(torch::Tensor input, torch::Tensor weight, int64_t bit_length,
                                      at::IntArrayRef padding, at::IntArrayRef stride, int64_t total_width,
                                      int64_t load_width, int64_t load_wait_w, int64_t load_wait_a, bool im2col,
                                      int64_t z_unit)
{
    (void)stride;
    (void)im2col;
    const geo_sc_conv_desc d = make_desc(input, weight, bit_length, padding, total_width, load_width, load_wait_w,
                                         load_wait_a, GEO_SC_ACC_YZ, z_unit);
    return forward_on_device(input, weight, d);
}

// sc_cuda.cpp:65-76: y-dimension accumulation with the "accurate random" generator (streams with
// exactly `code` ones).  The reference seeds its generators with constants (37 for the weights, 0
// for the activations, sc_cuda_kernel.cu:1885, :1957), so it returns the same result on every call;
// so does this, with its own counter-based generator: same distribution, other bits.
at::Tensor conv2d_add_partial_acc_acc(torch::Tensor input, torch::Tensor weight, int64_t bit_length,
                                      at::IntArrayRef padding, at::IntArrayRef stride, bool share, int64_t dim)
{
    (void)stride;
    (void)share;  // forced off inside the reference's kernels (sc_cuda_kernel.cu:372, :495)
    (void)dim;    // unused by the reference (sc_cuda.cpp:75)
    const geo_sc_conv_desc d = make_desc(input, weight, bit_length, padding, 7, 8, 1, 1, GEO_SC_ACC_Y, 1,
                                         GEO_SC_GEN_ACC, 37);
    return forward_on_device(input, weight, d);
}

// sc_cuda.cpp:21-32: OR over the whole kernel window and all input channels, Bernoulli random streams.
at::Tensor conv2d_or_acc(torch::Tensor input, torch::Tensor weight, int64_t bit_length, at::IntArrayRef padding,
                         at::IntArrayRef stride, bool im2col)
{
    (void)stride;
    (void)im2col;  // selects where the reference generates its streams; same distribution either way
    const geo_sc_conv_desc d = make_desc(input, weight, bit_length, padding, 7, 8, 1, 1, GEO_SC_ACC_FULL, 1,
                                         GEO_SC_GEN_RAND, 0);
    return forward_on_device(input, weight, d);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("conv2d_add_partial_variable_acc", &conv2d_add_partial_variable_acc,
          "SC forward conv2d partial (y or z dimension) bin add, variable load, lfsr generator");
    m.def("conv2d_add_yz_variable_acc", &conv2d_add_yz_variable_acc,
          "SC forward conv2d partial (yz dimension) bin add, variable load, lfsr generator");
    m.def("conv2d_add_partial_acc_acc", &conv2d_add_partial_acc_acc,
          "SC forward conv2d partial bin add, accurate random generator");
    m.def("conv2d_or_acc", &conv2d_or_acc, "SC forward conv2d or add, random generator");
}
