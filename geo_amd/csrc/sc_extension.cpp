// PyTorch module `sc_extension`: the entry point the reference's Python calls for tensors
// that live in host memory (utils_functional.py:11, :493; C++ side sc.cpp:292-476).
//
// The reference computes this op on the CPU.  Here the same call runs the gfx950 kernels:
// the tensors are moved to the current GPU, the result is moved back.  There is no CPU
// implementation behind it; without a GPU the call raises.
#include "sc_torch_common.h"

using namespace geo_sc_torch;

at::Tensor conv2d_add_partial_new(torch::Tensor input, torch::Tensor weight, int64_t bit_length,
                                  at::IntArrayRef padding, at::IntArrayRef stride)
{
    (void)stride;  // accepted and ignored, as in the reference
    // the CPU kernel has no progressive loading: total_width 7, load_width 8 leaves codes untouched
    const geo_sc_conv_desc d = make_desc(input, weight, bit_length, padding, 7, 8, 1, 1);
    TORCH_CHECK(torch::cuda::is_available(), "sc_extension.conv2d_add_partial_new needs a GPU: this build has no "
                                             "CPU implementation");
    const at::Device origin = input.device();
    const at::Device dev(at::kCUDA, c10::hip::current_device());
    at::Tensor out = forward_on_device(input.to(dev), weight.to(dev), d);
    return out.to(origin);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("conv2d_add_partial_new", &conv2d_add_partial_new, "SC forward conv2d partial bin add");
}
