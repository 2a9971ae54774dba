// Issue-rate probe: the convolution kernel's instruction (v_and_or_b32 with an SGPR weight
// operand, 64 independent accumulators, four waves per SIMD) in a loop with no memory
// traffic.  Timing it gives the rate the hardware sustains for that instruction, which is
// what the convolution kernel's achieved rate should be read against besides the nominal
// lanes x clock figure.  Built into a library of its own (libgeo_sc_probe.so) for the benchmark;
// not part of the C ABI of libgeo_sc.so.
//
// geo_sc_probe_and_or_rate enqueues `iters` x 64 v_and_or_b32 per wave on 4 waves per SIMD of 256 CUs
// and reports in *word_ops how many 32-bit lane operations that is; the caller times it.  scratch: at
// least 128 + 4096*64*4 bytes of device memory (its first 128 bytes are read as operands).
#include "sc_common.h"

namespace geo_sc {

namespace {

__global__ __launch_bounds__(64) void k_probe_and_or(const uint32_t* __restrict__ seed, uint32_t* __restrict__ sink,
                                                    int iters)
{
    uint32_t acc[64];
#pragma unroll
    for (int i = 0; i < 64; i++) acc[i] = 0;
    uint32_t w[32];
#pragma unroll
    for (int c = 0; c < 32; c++) w[c] = seed[c];  // wave-uniform: lives in SGPRs
    const uint32_t a0 = threadIdx.x * 2654435761u, a1 = a0 ^ 0x5555u;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 64; i++)
            asm volatile("v_and_or_b32 %0, %1, %2, %0" : "+v"(acc[i]) : "s"(w[i & 31]), "v"((i & 1) ? a1 : a0));
    }
    uint32_t r = 0;
#pragma unroll
    for (int i = 0; i < 64; i++) r ^= acc[i];
    sink[blockIdx.x * 64 + threadIdx.x] = r;
}

}  // namespace

}  // namespace geo_sc

extern "C" GEO_SC_API int geo_sc_probe_and_or_rate(int iters, void* scratch, size_t scratch_bytes, double* word_ops,
                                        geo_sc_stream_t stream)
{
    const int waves = 256 * 4 * 4;  // 256 CUs x 4 SIMDs x 4 waves
    const size_t need = 128 + (size_t)waves * 64 * sizeof(uint32_t);
    if (iters < 1 || !scratch || scratch_bytes < need || !word_ops) return GEO_SC_ERR_INVALID_ARGUMENT;
    uint32_t* seed = (uint32_t*)scratch;
    uint32_t* sink = seed + 32;
    hipLaunchKernelGGL(geo_sc::k_probe_and_or, dim3(waves), dim3(64), 0, (hipStream_t)stream, seed, sink, iters);
    *word_ops = (double)waves * 64.0 * 64.0 * (double)iters;
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}
