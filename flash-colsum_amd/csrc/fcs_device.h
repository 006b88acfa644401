// Small device helpers shared by the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fcs {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));  // 8 fp16 or (bit pattern) 8 bf16 values
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

static constexpr half8 kZero8 = {0, 0, 0, 0, 0, 0, 0, 0};
static constexpr float kNegBig = -1.0e30f;  // "hidden" score: finite so that max/sub never make NaN

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ half8 load8(const _Float16 *p) { return *reinterpret_cast<const half8 *>(p); }

__device__ __forceinline__ half8 flip_sign(half8 v)
{
    uint4v u = __builtin_bit_cast(uint4v, v);
    u ^= 0x80008000u;
    return __builtin_bit_cast(half8, u);
}

// One 32x32x16 MFMA step, fp32 accumulate.  The operands are 8 fp16 or (BF) 8 bf16 values per
// lane; both travel through the kernels as the same 16-byte bit pattern (`half8`), and the sign
// flip above works for either because the sign bits sit in the same places.
template <bool BF>
__device__ __forceinline__ floatx16 mfma16(half8 a, half8 b, floatx16 c)
{
    if constexpr (BF)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// key head of query head h (grouped-query attention): h / group through a multiply-high
__device__ __forceinline__ int kv_head(int h, int group, uint32_t magic)
{
    return group == 1 ? h : (int)__umulhi((uint32_t)h, magic);
}

// Row of a 32x32 MFMA result tile held by accumulator register i of a lane in half-wave g
// (the column is lane % 32).
__device__ __forceinline__ int acc_row(int i, int g) { return 8 * (i >> 2) + 4 * g + (i & 3); }

// value of the lane `lane ^ mask` for mask in {1, 2} (any values), or {4, 8} when the
// value is already uniform over groups of `mask` lanes; DPP, no LDS traffic
template <int CTRL>
__device__ __forceinline__ float dpp_get(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
static constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
static constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
static constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7 - i within groups of 8
static constexpr int kDppMirror = 0x140;      // lane i <-> 15 - i within rows of 16

// Workgroups are handed to the 8 XCDs round-robin in launch order (x fastest, then y, then z), and
// each XCD has its own L2.  Neighbours along x usually read the same operand, so they should
// run on one XCD and close together in time.  This returns the grid coordinates a workgroup should
// work on instead of its own: XCD c, which receives workgroups c, c + 8, c + 16, ..., then walks a
// contiguous range of the x-fastest list of all coordinates.  A bijection for any grid size.
// `i` is the workgroup's number in launch order, nx * ny * nz the number of workgroups.
__device__ __forceinline__ void xcd_contiguous_block(int i, int nx, int ny, int nz, int &bx, int &by, int &bz)
{
    const int n_all = nx * ny * nz;
    const int c = i & 7, per = n_all >> 3, rem = n_all & 7;  // XCD c holds per + (c < rem) workgroups
    const int v = c * per + min(c, rem) + (i >> 3);
    bx = v % nx;
    const int t = v / nx;
    by = t % ny;
    bz = t / ny;
}
// the same for a kernel whose grid is (nx, ny, nz)
__device__ __forceinline__ void xcd_contiguous_block(int &bx, int &by, int &bz)
{
    const int nx = gridDim.x, ny = gridDim.y;
    xcd_contiguous_block(((int)blockIdx.z * ny + (int)blockIdx.y) * nx + (int)blockIdx.x, nx, ny, (int)gridDim.z, bx, by, bz);
}

}  // namespace fcs
