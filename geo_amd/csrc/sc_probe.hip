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

// tile of the matrix-core probe
#define GEO_SC_PROBE_MFMA_ROWS 128
#define GEO_SC_PROBE_MFMA_COLS 256
#define GEO_SC_PROBE_MFMA_K 384
#define GEO_SC_PROBE_MFMA_ROW_BYTES 208

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

// ---------------------------------------------------------------------------------------------
// Matrix-core probe: one (stream cycle, kernel row) slice of the SC forward as a GEMM tile.
// The OR over a group is not linear, but for one stream cycle t the number of members whose AND is set is a
// binary matrix product, S_t[m][j] = sum_k a_k(m)[t] * w_(j,k)[t], and the OR is S_t > 0 (sc.cpp:12-259 computes
// the same counts bit-serially).  The probe runs that product for a tile of 128 positions x 256 rail-columns
// with K = 384 members (the 128 -> 128, 3 x 3 layer: 128 channels x 3 kernel taps, both rails of 128 output
// channels), operands 0 / 1 as fp4 (E2M1: 1.0 = 0x2) in LDS, v_mfma_scale_f32_32x32x64_f8f6f4, then the
// threshold and the count.  One workgroup of 8 waves (2 x 4, 64 x 64 results each) per CU.
//   mode 0: the MFMAs alone, operands in registers
//   mode 1: + the operand fragments read from LDS for every slice
//   mode 2: + threshold (> 0) and count into int32
//   mode 3: + the next slice's operand tiles (a share of their 72 KB) loaded from memory into the other LDS
//           buffer while this slice is multiplied (through registers), one barrier per slice
//   mode 4: the same with loads that write LDS directly (global_load_lds_dwordx4)
// What it measures is an upper bound on a matrix-core forward: the operands arrive already expanded from one
// bit to one fp4 value per cycle, which a real kernel would have to do as well.
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int TM = GEO_SC_PROBE_MFMA_ROWS, TJ = GEO_SC_PROBE_MFMA_COLS, K = GEO_SC_PROBE_MFMA_K, KSTEPS = K / 64;
constexpr int ROWB = GEO_SC_PROBE_MFMA_ROW_BYTES;  // bytes per operand row (K nibbles, padded)
constexpr int A_BYTES = TM * ROWB, B_BYTES = TJ * ROWB;
static_assert(ROWB == K / 2 + 16, "row padding");

// MODE 0: MFMAs only; 1: + LDS fragment reads; 2: + threshold/count; 3: + tiles streamed from global memory
template <int MODE, int FR = 16>
__global__ __launch_bounds__(512) void k_tile(const uint8_t* __restrict__ a_glob, const uint8_t* __restrict__ b_glob,
                                              int32_t* __restrict__ out, int iters, size_t a_tiles, size_t b_tiles)
{
    extern __shared__ uint8_t lds[];
    auto a_buf = [&](int b) { return lds + b * (A_BYTES + B_BYTES); };
    auto b_buf = [&](int b) { return lds + b * (A_BYTES + B_BYTES) + A_BYTES; };
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wm = wave >> 2, wj = wave & 3;  // 2 x 4 waves, each 64 x 64
    // initial tiles
    {
        const uint4* sa = (const uint4*)(a_glob + (size_t)(blockIdx.x % a_tiles) * A_BYTES);
        const uint4* sb = (const uint4*)(b_glob);
        for (int i = threadIdx.x; i < A_BYTES / 16; i += 512) ((uint4*)a_buf(0))[i] = sa[i];
        for (int i = threadIdx.x; i < B_BYTES / 16; i += 512) ((uint4*)b_buf(0))[i] = sb[i];
    }
    __syncthreads();
    int cnt[4][16];
#pragma unroll
    for (int b = 0; b < 4; b++)
#pragma unroll
        for (int i = 0; i < 16; i++) cnt[b][i] = 0;
    const int frag_off = (lane & 31) * ROWB + (lane >> 5) * 16;
    v4i areg[2][KSTEPS], breg[2][KSTEPS];
    if (MODE == 0) {
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ks++) {
                areg[r][ks] = *(const v4i*)(a_buf(0) + (wm * 64 + r * 32) * ROWB + frag_off + ks * 32);
                breg[r][ks] = *(const v4i*)(b_buf(0) + (wj * 64 + r * 32) * ROWB + frag_off + ks * 32);
            }
    }
    constexpr int A_LOAD = A_BYTES / 16 * FR / 16, B_LOAD = B_BYTES / 16 * FR / 16;
    constexpr int A_PER = A_LOAD / 512 + 1, B_PER = B_LOAD / 512 + 1;
    for (int it = 0; it < iters; it++) {
        const int buf = MODE >= 3 ? (it & 1) : 0;
        if (MODE == 4) {
            // the next slice's tiles straight into the other LDS buffer: every wave instruction moves 64 x 16
            // bytes from per-lane addresses to one contiguous kilobyte of LDS, no registers in between
            const size_t ta = ((size_t)blockIdx.x * 131 + it + 1) % a_tiles, tb = (size_t)(it + 1) % b_tiles;
            const uint8_t* sa = a_glob + ta * A_BYTES;
            const uint8_t* sb = b_glob + tb * B_BYTES;
            constexpr int A_KB = A_BYTES / 1024 * FR / 16, B_KB = B_BYTES / 1024 * FR / 16;
            for (int kb = wave; kb < A_KB; kb += 8)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(sa + kb * 1024 + lane * 16),
                                                 (__attribute__((address_space(3))) void*)(a_buf(buf ^ 1) + kb * 1024), 16, 0, 0);
            for (int kb = wave; kb < B_KB; kb += 8)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(sb + kb * 1024 + lane * 16),
                                                 (__attribute__((address_space(3))) void*)(b_buf(buf ^ 1) + kb * 1024), 16, 0, 0);
        }
        uint4 na[A_PER], nb[B_PER];
        if (MODE == 3) {
            const size_t ta = ((size_t)blockIdx.x * 131 + it + 1) % a_tiles, tb = (size_t)(it + 1) % b_tiles;
            const uint4* sa = (const uint4*)(a_glob + ta * A_BYTES);
            const uint4* sb = (const uint4*)(b_glob + tb * B_BYTES);
#pragma unroll
            for (int i = 0; i < A_PER; i++) {
                const int e = threadIdx.x + i * 512;
                na[i] = e < A_LOAD ? sa[e] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < B_PER; i++) {
                const int e = threadIdx.x + i * 512;
                nb[i] = e < B_LOAD ? sb[e] : make_uint4(0, 0, 0, 0);
            }
        }
        v16f acc[2][2];
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            v4i af[2], bf[2];
#pragma unroll
            for (int r = 0; r < 2; r++) {
                if (MODE == 0) {
                    af[r] = areg[r][ks];
                    bf[r] = breg[r][ks];
                } else {
                    af[r] = *(const v4i*)(a_buf(buf) + (wm * 64 + r * 32) * ROWB + frag_off + ks * 32);
                    bf[r] = *(const v4i*)(b_buf(buf) + (wj * 64 + r * 32) * ROWB + frag_off + ks * 32);
                }
            }
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    v8i a8 = {af[r].x, af[r].y, af[r].z, af[r].w, 0, 0, 0, 0};
                    v8i b8 = {bf[c].x, bf[c].y, bf[c].z, bf[c].w, 0, 0, 0, 0};
                    v16f zero = {};
                    acc[r][c] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, ks == 0 ? zero : acc[r][c], 4, 4, 0,
                                                                                127, 0, 127);
                }
        }
        if (MODE >= 2) {
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int c = 0; c < 2; c++)
#pragma unroll
                    for (int i = 0; i < 16; i++) cnt[r * 2 + c][i] += acc[r][c][i] > 0.0f ? 1 : 0;
        } else {
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int c = 0; c < 2; c++) cnt[r * 2 + c][0] += (int)acc[r][c][0] + (int)acc[r][c][15];
        }
        if (MODE == 3) {
#pragma unroll
            for (int i = 0; i < A_PER; i++) {
                const int e = threadIdx.x + i * 512;
                if (e < A_LOAD) ((uint4*)a_buf(buf ^ 1))[e] = na[i];
            }
#pragma unroll
            for (int i = 0; i < B_PER; i++) {
                const int e = threadIdx.x + i * 512;
                if (e < B_LOAD) ((uint4*)b_buf(buf ^ 1))[e] = nb[i];
            }
            __syncthreads();
        }
        if (MODE == 4) {
            __builtin_amdgcn_s_waitcnt(0);   // everything this wave asked for has arrived
            __syncthreads();
        }
    }
    // result layout of the 32x32 MFMA: lane l holds column l % 32, rows 8 * (i / 4) + 4 * (l / 32)... + i % 4
#pragma unroll
    for (int r = 0; r < 2; r++)
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = wm * 64 + r * 32 + 8 * (i / 4) + 4 * (lane >> 5) + (i & 3);
                const int col = wj * 64 + c * 32 + (lane & 31);
                out[((size_t)blockIdx.x * TM + row) * TJ + col] = cnt[r * 2 + c][i];
            }
}

}  // namespace

}  // namespace geo_sc

// a_tiles: n_a tiles of GEO_SC_PROBE_MFMA_ROWS rows x ROW_BYTES (row m, member k: nibble k % 2 of byte k / 2);
// b_tiles: n_b tiles of GEO_SC_PROBE_MFMA_COLS rows likewise (row j).  out: workgroups x ROWS x COLS int32, the
// counts of workgroup w's tile over its `slices` slices (workgroup w starts on A tile w % n_a and B tile 0; mode 3
// moves on to other tiles).  reload_sixteenths: 16, 12, 8 or 4 sixteenths of both tiles reloaded per slice in mode 3.
extern "C" GEO_SC_API int geo_sc_probe_mfma_slices(int mode, int reload_sixteenths, int workgroups, int slices,
                                                   const void* a_tiles, size_t n_a, const void* b_tiles, size_t n_b,
                                                   int32_t* out, geo_sc_stream_t stream)
{
    using namespace geo_sc;
    if (workgroups < 1 || slices < 1 || !a_tiles || !b_tiles || !out || n_a < 1 || n_b < 1)
        return GEO_SC_ERR_INVALID_ARGUMENT;
    const size_t lds = 2 * (size_t)(A_BYTES + B_BYTES);
    const uint8_t* a = (const uint8_t*)a_tiles;
    const uint8_t* b = (const uint8_t*)b_tiles;
#define GEO_SC_PROBE_LAUNCH(M, F)                                                                                       \
    do {                                                                                                               \
        if (hipFuncSetAttribute((const void*)k_tile<M, F>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=     \
            hipSuccess)                                                                                                \
            return GEO_SC_ERR_LAUNCH;                                                                                  \
        hipLaunchKernelGGL((k_tile<M, F>), dim3(workgroups), dim3(512), lds, (hipStream_t)stream, a, b, out, slices,    \
                           n_a, n_b);                                                                                  \
    } while (0)
    if (mode == 0) GEO_SC_PROBE_LAUNCH(0, 16);
    else if (mode == 1) GEO_SC_PROBE_LAUNCH(1, 16);
    else if (mode == 2) GEO_SC_PROBE_LAUNCH(2, 16);
    else if (mode == 3 && reload_sixteenths == 16) GEO_SC_PROBE_LAUNCH(3, 16);
    else if (mode == 3 && reload_sixteenths == 12) GEO_SC_PROBE_LAUNCH(3, 12);
    else if (mode == 3 && reload_sixteenths == 8) GEO_SC_PROBE_LAUNCH(3, 8);
    else if (mode == 3 && reload_sixteenths == 4) GEO_SC_PROBE_LAUNCH(3, 4);
    else if (mode == 4 && reload_sixteenths == 16) GEO_SC_PROBE_LAUNCH(4, 16);
    else if (mode == 4 && reload_sixteenths == 12) GEO_SC_PROBE_LAUNCH(4, 12);
    else if (mode == 4 && reload_sixteenths == 8) GEO_SC_PROBE_LAUNCH(4, 8);
    else if (mode == 4 && reload_sixteenths == 4) GEO_SC_PROBE_LAUNCH(4, 4);
    else return GEO_SC_ERR_INVALID_ARGUMENT;
#undef GEO_SC_PROBE_LAUNCH
    return hipGetLastError() == hipSuccess ? GEO_SC_OK : GEO_SC_ERR_LAUNCH;
}

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
