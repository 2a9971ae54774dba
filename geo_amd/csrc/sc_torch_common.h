// Shared glue of the two PyTorch extension modules: tensor checks, workspace from the
// caching allocator, launch on PyTorch's current HIP stream, status -> exception.
#pragma once

#include <torch/extension.h>

// PyTorch-ROCm presents HIP devices under the "cuda" device type; these are its own guard
// and stream accessors for that arrangement.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "geo_sc.h"

namespace geo_sc_torch {

inline void check_status(int rc, const char* what)
{
    TORCH_CHECK(rc == GEO_SC_OK, what, ": ", geo_sc_status_string(rc));
}

inline geo_sc_conv_desc make_desc(const at::Tensor& input, const at::Tensor& weight, int64_t bit_length,
                                  at::IntArrayRef padding, int64_t total_width, int64_t load_width,
                                  int64_t load_wait_w, int64_t load_wait_a, int accumulate = GEO_SC_ACC_Y,
                                  int64_t z_unit = 1, int generator = GEO_SC_GEN_LFSR, int32_t seed = 0)
{
    TORCH_CHECK(input.dim() == 4, "input must be (N, C_in, W, H), got ", input.dim(), " dims");
    TORCH_CHECK(weight.dim() == 4, "weight must be (C_out, C_in, W, H), got ", weight.dim(), " dims");
    TORCH_CHECK(input.scalar_type() == at::kFloat && weight.scalar_type() == at::kFloat,
                "input and weight must be float32");
    TORCH_CHECK(input.size(1) == weight.size(1), "channel mismatch: input has ", input.size(1), ", weight expects ",
                weight.size(1));
    TORCH_CHECK(padding.size() == 2, "padding must have two entries");
    TORCH_CHECK(bit_length == 8 || bit_length == 16 || bit_length == 32 || bit_length == 64 || bit_length == 128 ||
                    bit_length == 256,
                "bit_length must be one of 8, 16, 32, 64, 128, 256, got ", bit_length);
    TORCH_CHECK(load_width >= 1 && load_wait_w >= 1 && load_wait_a >= 1, "load_width and load_wait must be >= 1");
    geo_sc_conv_desc d;
    d.n = (int32_t)input.size(0);
    d.c_in = (int32_t)input.size(1);
    d.w_in = (int32_t)input.size(2);
    d.h_in = (int32_t)input.size(3);
    d.c_out = (int32_t)weight.size(0);
    d.w_k = (int32_t)weight.size(2);
    d.h_k = (int32_t)weight.size(3);
    // F.pad(input, {p0, p0, p1, p1}): p0 pads the last dim, p1 the one before (sc.cpp:298)
    d.pad_h = (int32_t)padding[0];
    d.pad_w = (int32_t)padding[1];
    d.bit_length = (int32_t)bit_length;
    d.total_width = (int32_t)total_width;
    d.load_width = (int32_t)load_width;
    d.load_wait_w = (int32_t)load_wait_w;
    d.load_wait_a = (int32_t)load_wait_a;
    TORCH_CHECK(z_unit >= 1, "z_units must be >= 1, got ", z_unit);
    d.accumulate = (int32_t)accumulate;
    d.z_unit = (int32_t)(z_unit > input.size(1) ? input.size(1) : z_unit);
    d.generator = (int32_t)generator;
    d.seed = seed;
    return d;
}

// input and weight on the same HIP device; returns int32 (N, C_out, Wo, Ho) on that device.
inline at::Tensor forward_on_device(const at::Tensor& input_in, const at::Tensor& weight_in,
                                    const geo_sc_conv_desc& d)
{
    TORCH_CHECK(input_in.is_cuda() && weight_in.is_cuda(), "tensors must be on the GPU");
    TORCH_CHECK(input_in.device() == weight_in.device(), "input and weight are on different devices");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input_in.device());
    at::Tensor input = input_in.contiguous(), weight = weight_in.contiguous();
    const int64_t wo = (int64_t)d.w_in + 2 * d.pad_w - d.w_k + 1, ho = (int64_t)d.h_in + 2 * d.pad_h - d.h_k + 1;
    TORCH_CHECK(wo >= 1 && ho >= 1, "kernel larger than the padded input");
    size_t ws_bytes = 0;
    check_status(geo_sc_conv2d_add_partial_workspace_size(&d, &ws_bytes), "workspace query");
    at::Tensor out = at::empty({d.n, d.c_out, wo, ho}, input.options().dtype(at::kInt));
    at::Tensor ws = at::empty({(int64_t)ws_bytes}, input.options().dtype(at::kByte));
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(input.device().index()).stream();
    check_status(geo_sc_conv2d_add_partial_forward(&d, input.data_ptr<float>(), weight.data_ptr<float>(),
                                                   out.data_ptr<int32_t>(), ws.data_ptr(), ws_bytes,
                                                   (geo_sc_stream_t)stream),
                 "conv2d_add_partial forward");
    return out;
}

}  // namespace geo_sc_torch
