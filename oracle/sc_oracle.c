/*
 * CPU oracle for the stochastic-computing (SC) convolution hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement of the
 * algorithm of the reference CPU kernel
 *     torch_c/sc-extension/sc.cpp            (conv2d_add_partial_new)
 * plus the progressive-loading mask that only the reference GPU kernels have
 *     torch_c/sc-extension/sc_cuda_kernel.cu:155-165, :681-688.
 * Only tests, the smoke check and the cpu_baseline leg of the benchmark may
 * call it; the shipped GPU path never does.
 *
 * Pinning status of each function (what, other than this file, fixes it):
 *   sco_lfsr_step        pinned  - known first states, period 2^n-1, all
 *                                  states visited (tests/test_oracle.py)
 *   sco_codes_*          pinned  - closed form, exact in fp32; end-to-end
 *                                  golden outputs of the compiled reference
 *   sco_weight_streams   pinned  - popcount invariant + end-to-end goldens
 *   sco_act_streams      pinned  - popcount invariant + end-to-end goldens
 *   sco_conv_scalar/fast pinned  - SHA-256 of compiled sc.cpp outputs, the
 *                                  committed fixtures, an independent per-bit
 *                                  numpy formulation, oracle/_ref when built
 *   sco_loaded_code (progressive loading, load_width < total_width+1)
 *                        pinned  - no CPU code in the reference executes it, so
 *                                  it is fixed by known answers worked out by
 *                                  hand, cycle by cycle, from the CUDA source
 *                                  text (tests/loading_vectors.py: 18 streams
 *                                  over three (width, unit, wait) settings,
 *                                  windows at cycles 1-8, 37-42, 77-82); the
 *                                  mistakes "first cycle counted as 0",
 *                                  "rounded-up division by the wait" and "no
 *                                  growth before the first wait has passed" each
 *                                  fail them; plus neutrality at
 *                                  load_width >= total_width+1
 *   sco_conv2d_modes, mode yz
 *                        pinned  - equals the sum over channel blocks of the
 *                                  pinned y-mode path on the blocks, for every
 *                                  z_unit (seeds restart per block); one block
 *                                  is y-mode itself (tests/test_oracle.py)
 *   sco_conv2d_modes, mode z
 *                        pinned  - one-dimensional windows (H = 1; W = 1 on
 *                        single-row signals) are y-mode itself; a general
 *                        W x H window (joint OR over (u,v), weight seed index
 *                        u*H+v) is y-mode on the restated problem "kernel
 *                        column u -> input channel u, one kernel row", whose
 *                        seeds coincide exactly for sizes with
 *                        Hi = Wo = 1 (mod L-1); the add over input channels by
 *                        the per-channel decomposition where planes hold a
 *                        multiple of L-1 words (tests/test_oracle.py).  What
 *                        stays a reading of the CUDA text
 *                        (sc_cuda_kernel.cu:270-349) is only that z-mode takes
 *                        the seed index u*H+v rather than v*W+u; an independent
 *                        per-bit formulation of the same reading agrees.
 *   sco_philox4x32_10    pinned  - the three known-answer vectors of the
 *                                  published Philox4x32-10 (Salmon et al., SC'11;
 *                                  Random123 kat_vectors)
 *   random generators (sco_random_stream_words, generator 1 "acc", 2 "rand")
 *                        STATISTICAL PARITY ONLY: the reference draws from
 *                        cuRAND's XORWOW with per-thread states
 *                        (sc_cuda_kernel.cu:354-420, :422-469, :524-545,
 *                        :1319-1333); its bit sequences are a property of that
 *                        library and its launch shape.  What is restated is the
 *                        distribution: "acc" = exactly `code` ones per stream,
 *                        drawn without replacement; "rand" = independent
 *                        Bernoulli(code / L) bits.  Pinned by the exact-count
 *                        invariant, by bit frequencies and by the closed-form
 *                        expectation of the layer output.
 *
 * Conventions (same names as the reference): weight (Cout, Cin, W, H) with
 * W = dim 2 and H = dim 3 (the binary-add dimension); padded activation
 * (N, Cin, Wi, Hi); output (N, Cout, Wo, Ho), Wo = Wi-W+1, Ho = Hi-H+1.
 * L in {8,16,32,64,128,256}; P = ceil(L/32) packs; bit_unit = min(L,32).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* One Fibonacci-LFSR step for an n-bit register, written with / and % the
 * way sc.cpp:262-290 writes it. */
int sco_lfsr_step(int n_bits, int v)
{
    switch (n_bits) {
    case 3: return ((v / 4) + (v / 2) % 2) % 2 + 2 * (v % 4);            /* sc.cpp:288-290 */
    case 4: return ((v / 8) + (v / 4) % 2) % 2 + 2 * (v % 8);            /* sc.cpp:283-285 */
    case 5: return ((v / 16) + (v / 4) % 2) % 2 + 2 * (v % 16);          /* sc.cpp:278-280 */
    case 6: return ((v / 32) + (v / 16) % 2) % 2 + 2 * (v % 32);         /* sc.cpp:273-275 */
    case 7: return ((v / 32) % 2 + v / 64) % 2 + 2 * (v % 64);           /* sc.cpp:268-270 */
    case 8: return ((v / 128) + (v / 32) % 2 + (v / 16) % 2 + (v / 8) % 2) % 2
                   + 2 * (v % 128);                                      /* sc.cpp:263-265 */
    default: return -1;
    }
}

/* Stream length -> LFSR width; -1 for an unsupported length (the reference
 * leaves its function pointer uninitialised there, sc.cpp:309-334). */
int sco_nbits_for_length(int L)
{
    switch (L) {
    case 8: return 3;
    case 16: return 4;
    case 32: return 5;
    case 64: return 6;
    case 128: return 7;
    case 256: return 8;
    default: return -1;
    }
}

/* Activation code: ceil(clamp(x*L, 0, L-1)) as int (sc.cpp:301). */
int sco_code_act(float x, int L)
{
    float t = x * (float)L;
    if (t < 0.0f) t = 0.0f;
    if (t > (float)(L - 1)) t = (float)(L - 1);
    return (int)ceilf(t);
}

/* Positive-rail weight code: ceil(clamp(w*L, 0, L-1)) (sc.cpp:303). */
int sco_code_wpos(float w, int L)
{
    return sco_code_act(w, L);
}

/* Negative-rail weight code: ceil(-clamp(w*L, 1-L, 0)) (sc.cpp:304). */
int sco_code_wneg(float w, int L)
{
    float t = w * (float)L;
    if (t < (float)(1 - L)) t = (float)(1 - L);
    if (t > 0.0f) t = 0.0f;
    return (int)ceilf(-t);
}

/* Progressive loading: the code value that is compared at stream cycle
 * b = 1..L (sc_cuda_kernel.cu:156-160, :682-685). */
static inline int sco_loaded_code(int code, int cycle, int total_width, int load_width, int load_wait)
{
    int cur_width = (cycle / load_wait + 1) * load_width - 1;
    if (cur_width > total_width) cur_width = total_width;
    int sh = total_width - cur_width;
    return (code >> sh) << sh;
}

/* Generate the P stream words of one value.  The register is advanced first
 * and compared second; bits enter MSB-first (word = word*2 + bit), and the
 * register state carries from one pack to the next (sc.cpp:365-383,
 * :426-434).  Returns the final register state. */
static inline int sco_stream_words(int code, int seed, int L, int n_bits, int total_width, int load_width,
                                   int load_wait, uint32_t* words /* [P] */)
{
    int P = (L + 31) / 32;
    int bit_unit = L < 32 ? L : 32;
    int s = seed;
    int cycle = 0;
    for (int p = 0; p < P; p++) {
        uint32_t word = 0;
        for (int b = 0; b < bit_unit; b++) {
            cycle += 1;
            int c = sco_loaded_code(code, cycle, total_width, load_width, load_wait);
            s = sco_lfsr_step(n_bits, s);
            word = word * 2u + (uint32_t)(c > s);
        }
        words[p] = word;
    }
    return s;
}

/* Exposed for tests: stream words of a single (code, seed). */
int sco_stream_of(int code, int seed, int L, int total_width, int load_width, int load_wait, uint32_t* words)
{
    int n_bits = sco_nbits_for_length(L);
    if (n_bits < 0) return -1;
    return sco_stream_words(code, seed, L, n_bits, total_width, load_width, load_wait, words);
}

/*
 * Weight streams, both rails, in the reference's transposed layout
 * [P][H][Cin][W][Cout] (sc.cpp:350-388).  One LFSR sequence per (c_in, w)
 * pair: seed (67+f)%(L-1)+1 on the positive rail and (37+f)%(L-1)+1 on the
 * negative rail with f = c_in*W + w (sc.cpp:340-347); the same sequence is
 * used for every h and every c_out.
 */
int sco_weight_streams(const float* w, int Cout, int Cin, int W, int H, int L, int total_width, int load_width,
                       int load_wait, uint32_t* wpos, uint32_t* wneg)
{
    int n_bits = sco_nbits_for_length(L);
    if (n_bits < 0) return -1;
    int P = (L + 31) / 32;
    size_t plane = (size_t)H * Cin * W * Cout;
    uint32_t words[8];
    for (int co = 0; co < Cout; co++)
        for (int ci = 0; ci < Cin; ci++)
            for (int u = 0; u < W; u++)
                for (int v = 0; v < H; v++) {
                    float wv = w[(((size_t)co * Cin + ci) * W + u) * H + v];
                    int f = ci * W + u;
                    int seed_pos = (67 + f) % (L - 1) + 1;
                    int seed_neg = (37 + f) % (L - 1) + 1;
                    size_t o = (((size_t)v * Cin + ci) * W + u) * Cout + co;
                    sco_stream_words(sco_code_wpos(wv, L), seed_pos, L, n_bits, total_width, load_width, load_wait,
                                     words);
                    for (int p = 0; p < P; p++) wpos[p * plane + o] = words[p];
                    sco_stream_words(sco_code_wneg(wv, L), seed_neg, L, n_bits, total_width, load_width, load_wait,
                                     words);
                    for (int p = 0; p < P; p++) wneg[p * plane + o] = words[p];
                }
    return 0;
}

/*
 * Activation streams of ONE batch item, layout [P][Cin][Wi][Hi]
 * (sc.cpp:405-438).  x is the already padded item (Cin, Wi, Hi).  Seed of
 * element i (flat index in the padded item) is i%(L-1)+1, identical for every
 * batch item (sc.cpp:409-413).
 */
int sco_act_streams(const float* x, int Cin, int Wi, int Hi, int L, int total_width, int load_width, int load_wait,
                    uint32_t* streams)
{
    int n_bits = sco_nbits_for_length(L);
    if (n_bits < 0) return -1;
    int P = (L + 31) / 32;
    size_t plane = (size_t)Cin * Wi * Hi;
    uint32_t words[8];
    for (size_t i = 0; i < plane; i++) {
        int seed = (int)(i % (size_t)(L - 1)) + 1;
        sco_stream_words(sco_code_act(x[i], L), seed, L, n_bits, total_width, load_width, load_wait, words);
        for (int p = 0; p < P; p++) streams[p * plane + i] = words[p];
    }
    return 0;
}

/* Zero-pad one item: F.pad(input, {p0,p0,p1,p1}) pads the LAST dim by pad_h
 * and the one before it by pad_w (sc.cpp:298). */
static void sco_pad_item(const float* x, int Cin, int Wx, int Hx, int pad_w, int pad_h, float* xp)
{
    int Wi = Wx + 2 * pad_w, Hi = Hx + 2 * pad_h;
    memset(xp, 0, sizeof(float) * (size_t)Cin * Wi * Hi);
    for (int c = 0; c < Cin; c++)
        for (int p = 0; p < Wx; p++)
            memcpy(xp + ((size_t)c * Wi + p + pad_w) * Hi + pad_h, x + ((size_t)c * Wx + p) * Hx,
                   sizeof(float) * (size_t)Hx);
}

/*
 * The accumulation itself, written straight from its definition
 * (sc.cpp:12-259 semantics with the im2col of sc.cpp:440-452 folded in):
 *   y[n,co,a,b] = sum_{v<H} sum_{p<P} ( popc(OR_{ci,u} A[p,ci,a+u,b+v] & WP[p,v,ci,u,co])
 *                                      - popc(OR_{ci,u} A[...]          & WN[p,v,ci,u,co]) )
 */
static void sco_accumulate_item(const uint32_t* A, const uint32_t* wpos, const uint32_t* wneg, int Cin, int Wi,
                                int Hi, int Cout, int W, int H, int P, int32_t* y)
{
    int Wo = Wi - W + 1, Ho = Hi - H + 1;
    size_t aplane = (size_t)Cin * Wi * Hi;
    size_t wplane = (size_t)H * Cin * W * Cout;
    for (int co = 0; co < Cout; co++)
        for (int a = 0; a < Wo; a++)
            for (int b = 0; b < Ho; b++) {
                int32_t acc = 0;
                for (int v = 0; v < H; v++)
                    for (int p = 0; p < P; p++) {
                        uint32_t orp = 0, orn = 0;
                        for (int ci = 0; ci < Cin; ci++)
                            for (int u = 0; u < W; u++) {
                                uint32_t aw = A[p * aplane + ((size_t)ci * Wi + a + u) * Hi + b + v];
                                size_t wo = p * wplane + (((size_t)v * Cin + ci) * W + u) * Cout + co;
                                orp |= aw & wpos[wo];
                                orn |= aw & wneg[wo];
                            }
                        acc += __builtin_popcount(orp) - __builtin_popcount(orn);
                    }
                y[((size_t)co * Wo + a) * Ho + b] = acc;
            }
}

/*
 * Same sums, loops arranged like the reference's matmul_outer (positions
 * innermost and contiguous so the compiler vectorises the AND/OR, sc.cpp:63-82):
 * the variant the cpu_baseline leg times when the compiled reference is absent.
 */
static void sco_accumulate_item_fast(const uint32_t* A, const uint32_t* wpos, const uint32_t* wneg, int Cin,
                                     int Wi, int Hi, int Cout, int W, int H, int P, int32_t* y, uint32_t* col,
                                     uint32_t* orp, uint32_t* orn)
{
    int Wo = Wi - W + 1, Ho = Hi - H + 1;
    int npos = Wo * Ho;
    int inner = Cin * W;
    size_t aplane = (size_t)Cin * Wi * Hi;
    size_t wplane = (size_t)H * Cin * W * Cout;
    memset(y, 0, sizeof(int32_t) * (size_t)Cout * npos);
    for (int p = 0; p < P; p++)
        for (int v = 0; v < H; v++) {
            /* im2col of this (pack, h): col[k][pos] (sc.cpp:440-452) */
            for (int k = 0; k < inner; k++) {
                int ci = k / W, u = k % W;
                for (int a = 0; a < Wo; a++)
                    memcpy(col + (size_t)k * npos + (size_t)a * Ho,
                           A + p * aplane + ((size_t)ci * Wi + a + u) * Hi + v, sizeof(uint32_t) * (size_t)Ho);
            }
            const uint32_t* wp = wpos + p * wplane + (size_t)v * inner * Cout;
            const uint32_t* wn = wneg + p * wplane + (size_t)v * inner * Cout;
            if (npos < 16) {
                /* few positions (the SC-linear mapping has one): run the contiguous c_out
                 * axis innermost instead, same sums */
                for (int i = 0; i < npos; i++) {
                    memset(orp, 0, sizeof(uint32_t) * (size_t)Cout);
                    memset(orn, 0, sizeof(uint32_t) * (size_t)Cout);
                    for (int k = 0; k < inner; k++) {
                        uint32_t aw = col[(size_t)k * npos + i];
                        const uint32_t* wpk = wp + (size_t)k * Cout;
                        const uint32_t* wnk = wn + (size_t)k * Cout;
                        for (int co = 0; co < Cout; co++) {
                            orp[co] |= aw & wpk[co];
                            orn[co] |= aw & wnk[co];
                        }
                    }
                    for (int co = 0; co < Cout; co++)
                        y[(size_t)co * npos + i] += __builtin_popcount(orp[co]) - __builtin_popcount(orn[co]);
                }
                continue;
            }
            for (int co = 0; co < Cout; co++) {
                memset(orp, 0, sizeof(uint32_t) * (size_t)npos);
                memset(orn, 0, sizeof(uint32_t) * (size_t)npos);
                for (int k = 0; k < inner; k++) {
                    uint32_t a_wp = wp[(size_t)k * Cout + co];
                    uint32_t a_wn = wn[(size_t)k * Cout + co];
                    const uint32_t* c = col + (size_t)k * npos;
                    for (int i = 0; i < npos; i++) {
                        orp[i] |= c[i] & a_wp;
                        orn[i] |= c[i] & a_wn;
                    }
                }
                int32_t* yo = y + (size_t)co * npos;
                for (int i = 0; i < npos; i++) yo[i] += __builtin_popcount(orp[i]) - __builtin_popcount(orn[i]);
            }
        }
}

/*
 * Whole op (sc.cpp:292-472): x (N,Cin,Wx,Hx) unpadded fp32, w (Cout,Cin,W,H)
 * fp32, y (N,Cout,Wo,Ho) int32.  `fast` selects the loop arrangement only;
 * both produce the same integers.  load_wait_w / load_wait_a are the
 * progressive-loading wait of the weight and activation generators.  Pass
 * load_width = total_width+1 for the CPU reference's behaviour (no
 * progressive loading).
 * Returns 0, or -1 for an unsupported L / bad arguments.
 */
int sco_conv2d_add_partial(const float* x, const float* w, int32_t* y, int N, int Cin, int Wx, int Hx, int Cout,
                           int W, int H, int pad_w, int pad_h, int L, int total_width, int load_width,
                           int load_wait_w, int load_wait_a, int fast, int n_threads)
{
    int n_bits = sco_nbits_for_length(L);
    if (n_bits < 0 || load_width < 1 || load_wait_w < 1 || load_wait_a < 1) return -1;
    int Wi = Wx + 2 * pad_w, Hi = Hx + 2 * pad_h;
    int Wo = Wi - W + 1, Ho = Hi - H + 1;
    if (Wo < 1 || Ho < 1) return -1;
    int P = (L + 31) / 32;
    size_t wwords = (size_t)P * H * Cin * W * Cout;
    uint32_t* wpos = (uint32_t*)malloc(sizeof(uint32_t) * wwords);
    uint32_t* wneg = (uint32_t*)malloc(sizeof(uint32_t) * wwords);
    sco_weight_streams(w, Cout, Cin, W, H, L, total_width, load_width, load_wait_w, wpos, wneg);
    size_t aplane = (size_t)Cin * Wi * Hi;
    size_t npos = (size_t)Wo * Ho;
#ifdef _OPENMP
    if (n_threads > 0) omp_set_num_threads(n_threads);
#else
    (void)n_threads;
#endif
#pragma omp parallel
    {
        float* xp = (float*)malloc(sizeof(float) * aplane);
        uint32_t* A = (uint32_t*)malloc(sizeof(uint32_t) * aplane * P);
        uint32_t *col = NULL, *orp = NULL, *orn = NULL;
        if (fast) {
            col = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)Cin * W * npos);
            size_t nor = npos > (size_t)Cout ? npos : (size_t)Cout;
            orp = (uint32_t*)malloc(sizeof(uint32_t) * nor);
            orn = (uint32_t*)malloc(sizeof(uint32_t) * nor);
        }
#pragma omp for schedule(dynamic, 1)
        for (int n = 0; n < N; n++) {
            sco_pad_item(x + (size_t)n * Cin * Wx * Hx, Cin, Wx, Hx, pad_w, pad_h, xp);
            sco_act_streams(xp, Cin, Wi, Hi, L, total_width, load_width, load_wait_a, A);
            int32_t* yn = y + (size_t)n * Cout * npos;
            if (fast)
                sco_accumulate_item_fast(A, wpos, wneg, Cin, Wi, Hi, Cout, W, H, P, yn, col, orp, orn);
            else
                sco_accumulate_item(A, wpos, wneg, Cin, Wi, Hi, Cout, W, H, P, yn);
        }
        free(xp);
        free(A);
        free(col);
        free(orp);
        free(orn);
    }
    free(wpos);
    free(wneg);
    return 0;
}

int sco_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------
 * The other two LFSR accumulation modes of the reference's GPU extension.  PARITY PINNED BY
 * SPEC TEXT ONLY: the reference has no CPU code for them; this follows the CUDA source text.
 *
 *   mode 0  y   OR over (c_in, w), add over h                      (above; sc.cpp)
 *   mode 1  z   OR over (w, h), add over c_in                      (sc_cuda_kernel.cu:272-349, :1141-1271)
 *   mode 2  yz  OR over (z_unit channels, w), add over h and over
 *               the ceil(c_in/z_unit) channel groups               (sc_cuda_kernel.cu:176-267, :1007-1138)
 *
 * Seeds.  Weights: index s into (67+s)%(L-1)+1 / (37+s)%(L-1)+1 is c_in*W+w (y), w*H+h (z:
 * sc_cuda_kernel.cu:322-324), (c_in % z_unit)*W+w (yz: :232).  The reference sizes the z-mode
 * seed array for c_in*W entries and reads past it when W*H is larger; here the same formula
 * is simply evaluated for every (w, h).  Activations: flat index in the padded item (y, z);
 * for yz the index wraps at z_unit*Wi*Hi (:1080), i.e. it is taken inside the channel group.
 * z_unit is clamped to c_in (:1987).
 * ------------------------------------------------------------------------------------------ */
/* Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
 * SC'11): ten rounds of two 32x32->64 multiplies, key bumped by the Weyl constants. */
void sco_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; r++) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* Random stream of one value: the P words of an L-bit stream, MSB-first like the LFSR streams.
 * The element's random words are Philox outputs with counter (block, index_lo, index_hi, tag)
 * and key (seed_lo, seed_hi); word j of the element is output j%4 of block j/4.
 *   generator 2 "rand": bit t = [code > r], r = byte t % 4 (from the least significant end) of word
 *     t / 4, reduced to its low n_bits bits: independent Bernoulli(code / L) bits,
 *     the distribution of code > curand() % L (sc_cuda_kernel.cu:459-462, :1329-1330).
 *   generator 1 "acc": bit t = [r16 * left_total < left_ones * 65536], r16 the (t % 2)-th 16-bit
 *     half of word t / 2, then left_ones -= bit, left_total -= 1: sampling without replacement,
 *     exactly `code` ones, the distribution of the reference's code_left / total_left >
 *     curand_uniform() (sc_cuda_kernel.cu:399-411, :539-545).
 * tag: 0 activations, 1 positive-rail weights, 2 negative-rail weights. */
void sco_random_stream_words(int code, int L, int generator, uint32_t tag, uint64_t index, uint64_t seed,
                             uint32_t* words /* [P] */)
{
    int n_bits = sco_nbits_for_length(L);
    int P = (L + 31) / 32, bit_unit = L < 32 ? L : 32;
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t ctr[4] = {0, (uint32_t)index, (uint32_t)(index >> 32), tag};
    uint32_t r[4] = {0, 0, 0, 0};
    int have_block = -1;
    int cpw = generator == 2 ? 4 : 2;
    int left_ones = code, left_total = L;
    (void)n_bits;
    for (int p = 0; p < P; p++) {
        uint32_t word = 0;
        for (int b = 0; b < bit_unit; b++) {
            int t = p * bit_unit + b;
            int j = t / cpw, f = t % cpw;
            if (j / 4 != have_block) {
                have_block = j / 4;
                ctr[0] = (uint32_t)have_block;
                sco_philox4x32_10(ctr, key, r);
            }
            uint32_t rw = r[j % 4];
            uint32_t bit;
            if (generator == 2) {
                bit = (uint32_t)code > ((rw >> (8 * f)) & (uint32_t)(L - 1));
            } else {
                uint32_t r16 = (rw >> (16 * f)) & 0xffffu;
                bit = r16 * (uint32_t)left_total < (uint32_t)left_ones * 65536u;
                left_ones -= (int)bit;
                left_total -= 1;
            }
            word = word * 2u + bit;
        }
        words[p] = word;
    }
}

/* generator: 0 LFSR (the seeds and loading arguments above), 1 "acc", 2 "rand" (random streams of
 * sco_random_stream_words; element index = flat index in the padded activation tensor
 * (N, Cin, Wi, Hi) resp. in the weight tensor (Cout, Cin, W, H); no progressive loading).
 * mode 3: OR over the whole kernel window and all input channels, add over packs only
 * (conv2d_or_acc: matmul_outer with inner_size = Cin*W*H and pws = packs, sc_cuda_kernel.cu:1351-1366). */
int sco_conv2d_general(const float* x, const float* w, int32_t* y, int N, int Cin, int Wx, int Hx, int Cout, int W,
                       int H, int pad_w, int pad_h, int L, int total_width, int load_width, int load_wait_w,
                       int load_wait_a, int mode, int z_unit, int generator, uint64_t seed);

int sco_conv2d_modes(const float* x, const float* w, int32_t* y, int N, int Cin, int Wx, int Hx, int Cout, int W,
                     int H, int pad_w, int pad_h, int L, int total_width, int load_width, int load_wait_w,
                     int load_wait_a, int mode, int z_unit)
{
    if (mode > 2) return -1;
    return sco_conv2d_general(x, w, y, N, Cin, Wx, Hx, Cout, W, H, pad_w, pad_h, L, total_width, load_width,
                              load_wait_w, load_wait_a, mode, z_unit, 0, 0);
}

int sco_conv2d_general(const float* x, const float* w, int32_t* y, int N, int Cin, int Wx, int Hx, int Cout, int W,
                       int H, int pad_w, int pad_h, int L, int total_width, int load_width, int load_wait_w,
                       int load_wait_a, int mode, int z_unit, int generator, uint64_t seed)
{
    int n_bits = sco_nbits_for_length(L);
    if (n_bits < 0 || load_width < 1 || load_wait_w < 1 || load_wait_a < 1 || mode < 0 || mode > 3) return -1;
    if (generator < 0 || generator > 2) return -1;
    if (mode == 2 && z_unit < 1) return -1;
    int Wi = Wx + 2 * pad_w, Hi = Hx + 2 * pad_h;
    int Wo = Wi - W + 1, Ho = Hi - H + 1;
    if (Wo < 1 || Ho < 1) return -1;
    int P = (L + 31) / 32;
    int zu = mode == 2 ? (z_unit < Cin ? z_unit : Cin) : Cin;
    int zp_n = (Cin + zu - 1) / zu;
    /* weight words [co][ci][u][v][p], both rails */
    size_t wn_el = (size_t)Cout * Cin * W * H;
    uint32_t* wp = (uint32_t*)malloc(sizeof(uint32_t) * wn_el * P);
    uint32_t* wn = (uint32_t*)malloc(sizeof(uint32_t) * wn_el * P);
    for (int co = 0; co < Cout; co++)
        for (int ci = 0; ci < Cin; ci++)
            for (int u = 0; u < W; u++)
                for (int v = 0; v < H; v++) {
                    size_t e = (((size_t)co * Cin + ci) * W + u) * H + v;
                    int s = (mode == 0 || mode == 3) ? ci * W + u : (mode == 1 ? u * H + v : (ci % zu) * W + u);
                    if (generator != 0) {
                        sco_random_stream_words(sco_code_wpos(w[e], L), L, generator, 1, e, seed, wp + e * P);
                        sco_random_stream_words(sco_code_wneg(w[e], L), L, generator, 2, e, seed, wn + e * P);
                        continue;
                    }
                    sco_stream_words(sco_code_wpos(w[e], L), (67 + s) % (L - 1) + 1, L, n_bits, total_width,
                                     load_width, load_wait_w, wp + e * P);
                    sco_stream_words(sco_code_wneg(w[e], L), (37 + s) % (L - 1) + 1, L, n_bits, total_width,
                                     load_width, load_wait_w, wn + e * P);
                }
    size_t plane = (size_t)Cin * Wi * Hi;
    size_t wrap = mode == 2 ? (size_t)zu * Wi * Hi : plane;
    float* xp = (float*)malloc(sizeof(float) * plane);
    uint32_t* A = (uint32_t*)malloc(sizeof(uint32_t) * plane * P); /* [i][p] */
    for (int n = 0; n < N; n++) {
        sco_pad_item(x + (size_t)n * Cin * Wx * Hx, Cin, Wx, Hx, pad_w, pad_h, xp);
        for (size_t i = 0; i < plane; i++) {
            if (generator != 0)
                sco_random_stream_words(sco_code_act(xp[i], L), L, generator, 0, (uint64_t)n * plane + i, seed,
                                        A + i * P);
            else
                sco_stream_words(sco_code_act(xp[i], L), (int)((i % wrap) % (size_t)(L - 1)) + 1, L, n_bits,
                                 total_width, load_width, load_wait_a, A + i * P);
        }
        for (int co = 0; co < Cout; co++)
            for (int a = 0; a < Wo; a++)
                for (int b = 0; b < Ho; b++) {
                    int32_t acc = 0;
                    /* add-groups: y: v; z: ci; yz: (channel group, v) */
                    int g_outer = mode == 1 ? Cin : (mode == 3 ? 1 : zp_n);
                    int g_inner = (mode == 1 || mode == 3) ? 1 : H;
                    for (int go = 0; go < g_outer; go++)
                        for (int gi = 0; gi < g_inner; gi++)
                            for (int p = 0; p < P; p++) {
                                uint32_t orp = 0, orn = 0;
                                int c0 = mode == 1 ? go : go * zu;
                                int c1 = mode == 1 ? go + 1 : (c0 + zu < Cin ? c0 + zu : Cin);
                                int v0 = (mode == 1 || mode == 3) ? 0 : gi, v1 = (mode == 1 || mode == 3) ? H : gi + 1;
                                for (int ci = c0; ci < c1; ci++)
                                    for (int u = 0; u < W; u++)
                                        for (int v = v0; v < v1; v++) {
                                            uint32_t aw = A[(((size_t)ci * Wi + a + u) * Hi + b + v) * P + p];
                                            size_t e = (((size_t)co * Cin + ci) * W + u) * H + v;
                                            orp |= aw & wp[e * P + p];
                                            orn |= aw & wn[e * P + p];
                                        }
                                acc += __builtin_popcount(orp) - __builtin_popcount(orn);
                            }
                    y[(((size_t)n * Cout + co) * Wo + a) * Ho + b] = acc;
                }
    }
    free(wp);
    free(wn);
    free(xp);
    free(A);
    return 0;
}
