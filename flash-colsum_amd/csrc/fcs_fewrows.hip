// Few-rows path: non-causal column means when only the first R <= 4 query rows of every head are
// averaged (`cls_len` of the reference operator, reference: flash_colsum/kernel_noncausal_batched.py:63-66,
// flash_colsum/kernel_noncausal.py:66-69, where all query tiles still run and are masked afterwards).
//
// With so few rows the call is a batch of matrix-vector products over K and is bound by reading K
// once from HBM, not by the matrix pipe.  One workgroup per (batch entry, head group):
//   * K rows are read with fully coalesced 16-byte loads, D/8 lanes per row, 8 loads in flight per lane;
//   * the partial dot products of a row are added across its lanes with DPP, the scores of the
//     whole head (log2 units) go to LDS;
//   * one max-subtracted softmax per row over the block, then the R rows are added per key;
//   * the block owns one slab row of partial column sums: the first head stores, later heads of
//     its group add (same thread, same address), fcs_finalize_kernel adds the slabs in index order.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <stdio.h>

#include "fcs_device.h"
#include "fcs_kernels.h"
#include "fcs_plan.h"

namespace fcs {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// sum over the D/8 lanes that share a key row; every lane of the group gets the total
template <int LPR>
__device__ __forceinline__ float row_lanes_sum(float v)
{
    v += dpp_get<kDppXor1>(v);
    v += dpp_get<kDppXor2>(v);
    v += dpp_get<kDppHalfMirror>(v);
    if (LPR == 16) v += dpp_get<kDppMirror>(v);
    return v;
}

// dot product of 8 fp16 or (BF) 8 bf16 values per operand, fp32 accumulate
template <bool BF>
__device__ __forceinline__ float dot8(half8 x, half8 y)
{
    float s = 0.f;
    if constexpr (BF) {
        const uint4v xu = __builtin_bit_cast(uint4v, x), yu = __builtin_bit_cast(uint4v, y);
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // a bf16 value is the upper half of the fp32 with the same value
            s = fmaf(__builtin_bit_cast(float, xu[i] << 16), __builtin_bit_cast(float, yu[i] << 16), s);
            s = fmaf(__builtin_bit_cast(float, xu[i] & 0xffff0000u), __builtin_bit_cast(float, yu[i] & 0xffff0000u), s);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const half2v xa = {x[2 * i], x[2 * i + 1]}, ya = {y[2 * i], y[2 * i + 1]};
            s = __builtin_amdgcn_fdot2(xa, ya, s, false);
        }
    }
    return s;
}

// block-wide max or sum of one value per thread (256 threads); `slot` is a 4-float LDS scratch.
// Every thread gets the result.  Two barriers.
template <bool MAX>
__device__ __forceinline__ float block_reduce(float v, float *slot, int lane, int wave)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float o = __shfl_xor(v, m);
        v = MAX ? fmaxf(v, o) : v + o;
    }
    __syncthreads();  // the slot may still be read from the previous use
    if (lane == 0) slot[wave] = v;
    __syncthreads();
    const float a0 = slot[0], a1 = slot[1], a2 = slot[2], a3 = slot[3];
    return MAX ? fmaxf(fmaxf(a0, a1), fmaxf(a2, a3)) : (a0 + a1) + (a2 + a3);
}

template <int D, int R, bool BF>
__global__ __launch_bounds__(256) void fcs_fewrows_kernel(const Args a)
{
    constexpr int LPR = D / 8;     // lanes per key row (16 bytes each)
    constexpr int RPW = 64 / LPR;  // key rows per wave per load instruction
    constexpr int RPB = 4 * RPW;   // key rows per block per round
    constexpr int UN = 8;          // rounds in flight
    __shared__ float sc[kFewRowsMaxScores];  // [R][Sk] scores, then exponentials
    __shared__ float slot[4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane % LPR, rw = lane / LPR;
    const int b = blockIdx.x % a.B, hg = blockIdx.x / a.B;
    const int h_begin = hg * a.f_hpg, h_end = min(a.H, h_begin + a.f_hpg);
    const int Sk = a.Sk;
    float *dst = a.partial + ((int64_t)hg * a.B + b) * Sk;

    for (int h = h_begin; h < h_end; ++h) {
        const _Float16 *qp = a.q + (int64_t)b * a.qs_b + (int64_t)h * a.qs_h + sub * 8;
        const _Float16 *kp = a.k + (int64_t)b * a.ks_b + (int64_t)kv_head(h, a.kv_group, a.kv_magic) * a.ks_h + sub * 8;
        half8 qv[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const half8 v = load8(qp + (int64_t)r * a.qs_s);
            qv[r] = a.negate ? flip_sign(v) : v;
        }
        for (int base = 0; base < Sk; base += UN * RPB) {
            half8 kv[UN];
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const int row = min(base + u * RPB + wave * RPW + rw, Sk - 1);
                kv[u] = load8(kp + (int64_t)row * a.ks_s);
            }
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const int row = base + u * RPB + wave * RPW + rw;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float s = row_lanes_sum<LPR>(dot8<BF>(qv[r], kv[u]));
                    if (sub == 0 && row < Sk) sc[r * Sk + row] = s;  // raw score: scaled after the maximum is subtracted
                }
            }
        }
        __syncthreads();

        float w[R];  // 1 / row sum
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float m = kNegBig;
            for (int j = tid; j < Sk; j += 256) m = fmaxf(m, sc[r * Sk + j]);
            m = block_reduce<true>(m, slot, lane, wave);
            float l = 0.f;
            for (int j = tid; j < Sk; j += 256) {
                const float e = fast_exp2((sc[r * Sk + j] - m) * a.c);
                sc[r * Sk + j] = e;  // each thread re-reads only what it wrote
                l += e;
            }
            l = block_reduce<false>(l, slot, lane, wave);
            w[r] = 1.0f / l;
        }
        for (int j = tid; j < Sk; j += 256) {
            float p = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) p = fmaf(sc[r * Sk + j], w[r], p);
            dst[j] = (h == h_begin) ? p : dst[j] + p;
        }
        __syncthreads();  // the next head overwrites the scores
    }
}

template <int D, bool BF>
static hipError_t launch_fewrows_d(const Plan &p, const Args &a, hipStream_t st)
{
    const dim3 grid(p.B * p.f_hg), block(256);
    switch (p.q_rows) {
    case 1: hipLaunchKernelGGL((fcs_fewrows_kernel<D, 1, BF>), grid, block, 0, st, a); break;
    case 2: hipLaunchKernelGGL((fcs_fewrows_kernel<D, 2, BF>), grid, block, 0, st, a); break;
    case 3: hipLaunchKernelGGL((fcs_fewrows_kernel<D, 3, BF>), grid, block, 0, st, a); break;
    case 4: hipLaunchKernelGGL((fcs_fewrows_kernel<D, 4, BF>), grid, block, 0, st, a); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_fewrows(const Plan &p, const Args &a, hipStream_t st)
{
    hipError_t e;
    if (p.bf16)
        e = (p.D == 64) ? launch_fewrows_d<64, true>(p, a, st) : launch_fewrows_d<128, true>(p, a, st);
    else
        e = (p.D == 64) ? launch_fewrows_d<64, false>(p, a, st) : launch_fewrows_d<128, false>(p, a, st);
    if (e != hipSuccess) return e;
    return launch_finalize(a, st);
}

size_t describe_fewrows(const Plan &p, const Args &a, char *buf, size_t n)
{
    const int r = snprintf(buf, n, "fcs_fewrows_kernel<%d,%d,%s> grid %d, %d heads per workgroup, %d slabs", p.D, p.q_rows,
                           p.bf16 ? "true" : "false", p.B * p.f_hg, p.f_hpg, p.n_partials);
    if (r < 0) return 0;
    const size_t len = (size_t)r;
    return len + describe_finalize(a, len < n ? buf + len : nullptr, len < n ? n - len : 0);
}

}  // namespace fcs
