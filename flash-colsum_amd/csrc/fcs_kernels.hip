// Attention column means on gfx950 (MI355X): launch order of the paths and the final reduction.
//
//   pass 1 (fcs_rowstream_kernel, fcs_stream.hip)  per row (m, log2 l) with
//          l = sum_j 2^((s_ij - m) * c), c = scale*log2(e), or (m, l) per key split.
//   pass 2 (fcs_colstream_kernel, fcs_stream.hip)  column sums of 2^((s_ij - m_i) * c - log2 l_i),
//          one partial slab per group of (head, row block) units.
//   fcs_finalize_kernel (here) adds the slabs in a fixed order: no atomics anywhere, every
//          partial has exactly one writer.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <stdio.h>

#include "fcs_device.h"
#include "fcs_kernels.h"

namespace fcs {

// slab lanes for n slabs: the fewest of 8, 16, 32 that leave a lane at most four slabs (32 beyond 128 slabs)
static inline int slab_lanes(int n) { return n <= 32 ? 8 : n <= 64 ? 16 : 32; }

// The summation tree of one output over n slabs with SL slab lanes: lane sl adds the slabs sl, sl + SL,
// sl + 2 SL, ... in index order into four running sums (slab sl + j SL goes to sum j % 4, so four loads
// are in flight), and its total is (s0 + s1) + (s2 + s3).  `stride` is the distance between slabs in floats.
template <int SL>
__device__ __forceinline__ float slab_lane_total(const float *p, int64_t stride, int n, int sl)
{
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int gi = sl; gi < n; gi += 4 * SL) {
        s0 += p[(int64_t)gi * stride];
        if (gi + SL < n) s1 += p[(int64_t)(gi + SL) * stride];
        if (gi + 2 * SL < n) s2 += p[(int64_t)(gi + 2 * SL) * stride];
        if (gi + 3 * SL < n) s3 += p[(int64_t)(gi + 3 * SL) * stride];
    }
    return (s0 + s1) + (s2 + s3);
}

// out = inv_norm * (partial[0] + partial[1] + ...).  A block owns 32 consecutive outputs; its
// SL slab lanes each add every SL-th slab in index order (four running sums, so that four loads
// are in flight per thread) and the SL sub-totals are then added in lane order: the summation
// tree is fixed by (number of slabs, SL), i.e.
// bit-reproducible, while SL x 4 loads per output are in flight instead of one.  SL = 8 for the
// usual few dozen slabs, 16 or 32 for more (slab_lanes()): a small batch can leave hundreds of
// slabs per batch entry (B 1, H 16, S 1024 on the fused path: 512 slabs of 1024 outputs, where 8
// lanes took longer than the kernel that wrote the slabs).
template <int SL>
__global__ __launch_bounds__(32 * SL) void fcs_finalize_kernel(const Args a)
{
    __shared__ float sub[SL][32];
    const int64_t n = (int64_t)a.B * a.Sk;
    const int col = threadIdx.x & 31, sl = threadIdx.x >> 5;
    const int64_t idx = (int64_t)blockIdx.x * 32 + col;
    sub[sl][col] = (idx < n) ? slab_lane_total<SL>(a.partial + idx, n, a.n_partials, sl) : 0.f;
    __syncthreads();
    if (sl == 0 && idx < n) {
        float t = sub[0][col];
#pragma unroll
        for (int j = 1; j < SL; ++j) t += sub[j][col];
        a.out[idx] = t * a.inv_norm;
        if (a.out_h) a.out_h[idx] = (_Float16)(t * a.inv_norm);
    }
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------
hipError_t launch_finalize(const Args &a, hipStream_t st)
{
    const int64_t n = (int64_t)a.B * a.Sk;
    const dim3 grid((unsigned)((n + 31) / 32));
    switch (slab_lanes(a.n_partials)) {
    case 32: hipLaunchKernelGGL(fcs_finalize_kernel<32>, grid, dim3(1024), 0, st, a); break;
    case 16: hipLaunchKernelGGL(fcs_finalize_kernel<16>, grid, dim3(512), 0, st, a); break;
    default: hipLaunchKernelGGL(fcs_finalize_kernel<8>, grid, dim3(256), 0, st, a); break;
    }
    return hipGetLastError();
}

size_t describe_finalize(const Args &a, char *buf, size_t n)
{
    const int r = snprintf(buf, n, " + fcs_finalize_kernel<%d> grid %lld", slab_lanes(a.n_partials),
                           (long long)(((int64_t)a.B * a.Sk + 31) / 32));
    return r < 0 ? 0 : (size_t)r;
}

// the two-pass path: row statistics, column sums (which also merge the key splits), final reduction
static hipError_t launch_two_pass(const Plan &p, const Args &a, hipStream_t st)
{
    hipError_t e = launch_rowstream(p, a, st);
    if (e != hipSuccess) return e;
    e = launch_colstream(p, a, st);
    if (e != hipSuccess) return e;
    if (p.c_groups > 1) return launch_finalize(a, st);
    return hipSuccess;
}

int launch_colsum(const Plan &p, const Args &a, void *stream)
{
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (p.fewrows) return (int)launch_fewrows(p, a, st);
    if (p.small) return (int)launch_small(p, a, st);
    if (p.fused) return (int)launch_fused(p, a, st);
    return (int)launch_two_pass(p, a, st);
}

size_t describe_colsum(const Plan &p, const Args &a, char *buf, size_t n)
{
    if (p.fewrows) return describe_fewrows(p, a, buf, n);
    if (p.small) return describe_small(p, a, buf, n);
    if (p.fused) return describe_fused(p, a, buf, n);
    return describe_two_pass(p, a, buf, n);
}

}  // namespace fcs
