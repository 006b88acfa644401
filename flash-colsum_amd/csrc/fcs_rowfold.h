// In-register reductions over the key lanes of a 32 x 32 score tile, shared by the single-pass kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fcs {

// Sum (or maximum) of v[i] over the 32 lanes of each half-wave, for all sixteen i at once, in
// registers: a reduce-scatter butterfly.  Each step combines the values of lanes 16, 8, 4, 2 apart
// while halving the number of registers: which half a lane keeps is chosen by the lane-number bit
// of that step, so after four steps a lane is left with ONE register, the total of
//     i = 8 * bit4 + 4 * bit3 + 2 * bit2 + bit1        (bits of the lane number)
// over 16 lanes; the last step (lanes 1 apart) completes it, both lanes of a pair hold the same
// total.  In the accumulator layout that is row  16*bit4 + 8*bit3 + 4*g + 2*bit2 + bit1  (g = bit5).
// 32 VALU instructions and no LDS traffic; the order of operations is fixed.
//   * 16 apart: v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even
//     rows of its second, after which first (+) second is, in even rows, the total of the first
//     register over the two rows and, in odd rows, that of the second register.
//   * 8 and 4 apart: DPP row rotations; the bank mask (banks of 4 lanes) picks the lanes that keep
//     the low or the high register of a pair, so no select is needed.
//   * 2 and 1 apart: DPP quad permutations.
// Inline assembly for the DPP forms: between a VALU write and a DPP read of the same register the
// hardware wants two wait states, which the s_nop in front of every group provides.
#define FCS_FOLD_LANES(NAME, OP, COMBINE)                                                                  \
    __device__ __forceinline__ float NAME(const float (&v)[16], int lane)                                  \
    {                                                                                                      \
        float u[8];                                                                                        \
        _Pragma("unroll") for (int i = 0; i < 8; ++i)                                                      \
        {                                                                                                  \
            float x = v[i], y = v[i + 8];                                                                  \
            asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x), "+v"(y));        \
            u[i] = COMBINE(x, y);                                                                          \
        }                                                                                                  \
        /* 8 apart: lanes with bit3 clear (banks 0, 1) keep u[j], the others u[j + 4] */                   \
        asm volatile("s_nop 1\n\t" OP " %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0x3\n\t" OP            \
                     " %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0x3\n\t" OP                             \
                     " %2, %2, %2 row_ror:8 row_mask:0xf bank_mask:0x3\n\t" OP                             \
                     " %3, %3, %3 row_ror:8 row_mask:0xf bank_mask:0x3\n\t" OP                             \
                     " %0, %4, %4 row_ror:8 row_mask:0xf bank_mask:0xc\n\t" OP                             \
                     " %1, %5, %5 row_ror:8 row_mask:0xf bank_mask:0xc\n\t" OP                             \
                     " %2, %6, %6 row_ror:8 row_mask:0xf bank_mask:0xc\n\t" OP                             \
                     " %3, %7, %7 row_ror:8 row_mask:0xf bank_mask:0xc"                                    \
                     : "+v"(u[0]), "+v"(u[1]), "+v"(u[2]), "+v"(u[3])                                      \
                     : "v"(u[4]), "v"(u[5]), "v"(u[6]), "v"(u[7]));                                        \
        /* 4 apart (a rotation to the right by n hands lane i the value of lane i - n of its row): lanes  \
           with bit2 clear (banks 0, 2) take their partner 4 lanes up, the others 4 lanes down */          \
        asm volatile("s_nop 1\n\t" OP " %0, %0, %0 row_ror:12 row_mask:0xf bank_mask:0x5\n\t" OP           \
                     " %1, %1, %1 row_ror:12 row_mask:0xf bank_mask:0x5\n\t" OP                            \
                     " %0, %2, %2 row_ror:4 row_mask:0xf bank_mask:0xa\n\t" OP                             \
                     " %1, %3, %3 row_ror:4 row_mask:0xf bank_mask:0xa"                                    \
                     : "+v"(u[0]), "+v"(u[1])                                                              \
                     : "v"(u[2]), "v"(u[3]));                                                              \
        /* 2 apart: lanes with bit1 clear keep u[0] */                                                     \
        const bool hi2 = (lane & 2) != 0;                                                                  \
        float keep = hi2 ? u[1] : u[0], send = hi2 ? u[0] : u[1];                                          \
        asm volatile("s_nop 1\n\t" OP " %0, %1, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"    \
                     "s_nop 1\n\t" OP " %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf"         \
                     : "+v"(keep)                                                                          \
                     : "v"(send));                                                                         \
        return keep;                                                                                       \
    }
__device__ __forceinline__ float fcs_add2(float x, float y) { return x + y; }
FCS_FOLD_LANES(fold_lanes_sum, "v_add_f32_dpp", fcs_add2)
FCS_FOLD_LANES(fold_lanes_max, "v_max_f32_dpp", fmaxf)
#undef FCS_FOLD_LANES

}  // namespace fcs
