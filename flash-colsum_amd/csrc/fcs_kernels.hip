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

#include "fcs_device.h"
#include "fcs_kernels.h"

namespace fcs {

// out = inv_norm * (partial[0] + partial[1] + ...).  A block owns 32 consecutive outputs; its
// SL slab lanes each add every SL-th slab in index order (four running sums, so that four loads
// are in flight per thread) and the SL sub-totals are then added in lane order: the summation tree
// is fixed by (number of slabs, SL), i.e. bit-reproducible, while SL x 4 loads per output are in
// flight instead of one.  SL = 8 for the usual few dozen slabs; SL = 32 when a small batch leaves
// hundreds of slabs per batch entry (B 1, H 16, S 1024 on the fused path: 512 slabs of 1024
// outputs, where 8 lanes took longer than the kernel that wrote the slabs).
template <int SL>
__global__ __launch_bounds__(32 * SL) void fcs_finalize_kernel(const Args a)
{
    __shared__ float sub[SL][32];
    const int64_t n = (int64_t)a.B * a.Sk;
    const int col = threadIdx.x & 31, sl = threadIdx.x >> 5;
    const int64_t idx = (int64_t)blockIdx.x * 32 + col;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (idx < n) {
        const float *p = a.partial + idx;
        int gi = sl;
        for (; gi + 3 * SL < a.n_partials; gi += 4 * SL) {
            s0 += p[(int64_t)gi * n];
            s1 += p[(int64_t)(gi + SL) * n];
            s2 += p[(int64_t)(gi + 2 * SL) * n];
            s3 += p[(int64_t)(gi + 3 * SL) * n];
        }
        for (; gi < a.n_partials; gi += SL) s0 += p[(int64_t)gi * n];
    }
    sub[sl][col] = (s0 + s1) + (s2 + s3);
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
    if (a.n_partials >= 64) hipLaunchKernelGGL(fcs_finalize_kernel<32>, grid, dim3(1024), 0, st, a);
    else hipLaunchKernelGGL(fcs_finalize_kernel<8>, grid, dim3(256), 0, st, a);
    return hipGetLastError();
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
    if (p.fused) return (int)launch_fused(p, a, st);
    return (int)launch_two_pass(p, a, st);
}

}  // namespace fcs
