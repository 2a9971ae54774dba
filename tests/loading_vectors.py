"""Hand-derived known answers for progressive loading (sc_cuda_kernel.cu:155-160 for weights,
:681-685 for activations).  Data only: no formula of the generators is restated here.

The reference's loop, per stream cycle, reads

    cur_bit += 1;                                         // first cycle has cur_bit == 1
    cur_width = (cur_bit / load_wait + 1) * load_width - 1;   // integer division
    if (cur_width > total_width) cur_width = total_width;
    actual = (code >> (total_width - cur_width)) << (total_width - cur_width);
    seed = lfsr(seed);                                    // advance, then compare
    bit = actual > seed;

All vectors use L = 128 (7-bit register) and LFSR seed 1, whose states after 1, 2, ... advances are
2, 4, 8, 16, 32, 65, 3, 6 (cycles 1..8), 78, 29, 58, 117, 106, 84 (cycles 37..42) and
45, 91, 55, 111, 94, 61 (cycles 77..82).  Seed 1 is the activation seed of flat index 0.

Each entry: (total_width, load_width, load_wait), first cycle of the window, {code: bits of the window}.
"""

STATES_FROM_SEED_1 = {1: 2, 2: 4, 3: 8, 4: 16, 5: 32, 6: 65, 7: 3, 8: 6,
                      37: 78, 38: 29, 39: 58, 40: 117, 41: 106, 42: 84,
                      77: 45, 78: 91, 79: 55, 80: 111, 81: 94, 82: 61}

VECTORS = [
    # (7, 2, 2): cycle      1  2  3  4  5  6  7  8
    #            cur_width  1  3  3  5  5  7  7  7      (1/2+1)*2-1 = 1, (2/2+1)*2-1 = 3, ... capped at 7
    #            low bits cleared: 6  4  4  2  2  0  0  0
    ((7, 2, 2), 1, {
        # 63 = 0111111b: masked 0, 48, 48, 60, 60, 63, 63, 63  against 2, 4, 8, 16, 32, 65, 3, 6
        63: [0, 1, 1, 1, 1, 0, 1, 1],
        # 5: masked 0, 0, 0, 4, 4, 5, 5, 5
        5: [0, 0, 0, 0, 0, 0, 1, 0],
        # 15: masked 0, 0, 0, 12, 12, 15, 15, 15
        15: [0, 0, 0, 0, 0, 0, 1, 1],
        # 19 = 0010011b: masked 0, 16, 16, 16, 16, 19, 19, 19 (16 > 16 is false at cycle 4)
        19: [0, 1, 1, 0, 0, 0, 1, 1],
        # 35 = 0100011b: masked 0, 32, 32, 32, 32, 35, 35, 35 (32 > 32 is false at cycle 5)
        35: [0, 1, 1, 1, 0, 0, 1, 1],
        # 67 = 1000011b: masked 64, 64, 64, 64, 64, 67, 67, 67
        67: [1, 1, 1, 1, 1, 1, 1, 1],
    }),
    # (7, 1, 3): cycle      1  2  3  4  5  6  7  8
    #            cur_width  0  0  1  1  1  2  2  2      (b/3+1)*1-1 = b/3
    #            low bits cleared: 7  7  6  6  6  5  5  5      width 0 clears the whole code
    ((7, 1, 3), 1, {
        # 127: masked 0, 0, 64, 64, 64, 96, 96, 96
        127: [0, 0, 1, 1, 1, 1, 1, 1],
        # 63: masked 0, 0, 0, 0, 0, 32, 32, 32
        63: [0, 0, 0, 0, 0, 0, 1, 1],
        # 95 = 1011111b: masked 0, 0, 64, 64, 64, 64, 64, 64 (64 > 65 is false at cycle 6)
        95: [0, 0, 1, 1, 1, 0, 1, 1],
        # 31: nothing above bit 4 in the first 8 cycles
        31: [0, 0, 0, 0, 0, 0, 0, 0],
    }),
    # (7, 3, 40): cur_width (b/40+1)*3-1 = 2 for cycles 1..39, 5 for 40..79, 8 -> 7 from 80 on
    #             cycle     37  38  39  40  41  42          (states 78, 29, 58, 117, 106, 84)
    #             cleared    5   5   5   2   2   2
    ((7, 3, 40), 37, {
        # 127: masked 96, 96, 96, 124, 124, 124
        127: [1, 1, 1, 1, 1, 1],
        # 97 = 1100001b: masked 96, 96, 96, 96, 96, 96
        97: [1, 1, 1, 0, 0, 1],
        # 33: masked 32, 32, 32, 32, 32, 32
        33: [0, 1, 0, 0, 0, 0],
        # 119 = 1110111b: masked 96, 96, 96, 116, 116, 116 (116 > 117 false)
        119: [1, 1, 1, 0, 1, 1],
    }),
    #             cycle     77  78  79  80  81  82          (states 45, 91, 55, 111, 94, 61)
    #             cleared    2   2   2   0   0   0
    ((7, 3, 40), 77, {
        # 97: masked 96, 96, 96, 97, 97, 97
        97: [1, 1, 1, 0, 1, 1],
        # 95 = 1011111b: masked 92, 92, 92, 95, 95, 95
        95: [1, 1, 1, 0, 1, 1],
        # 63 = 0111111b: masked 60, 60, 60, 63, 63, 63
        63: [1, 0, 1, 0, 0, 1],
        # 58 = 0111010b: masked 56, 56, 56, 58, 58, 58 (56 > 55 at cycle 79)
        58: [1, 0, 1, 0, 0, 0],
    }),
]
