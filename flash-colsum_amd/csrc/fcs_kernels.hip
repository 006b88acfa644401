// Attention column means on gfx950 (MI355X): the general two-pass path, pass 1 and the final
// reduction.
//
//   pass 1 (fcs_rowstats_kernel, here)  32x32 score tiles  S^T = K_tile * Q_tile^T  on
//          v_mfma_f32_32x32x16_f16: a lane owns ONE query (column l%32 of the tile) and holds 16
//          keys of it in its accumulator registers (key row 8*(r/4) + 4*(l/32) + r%4).  Q tile
//          stationary in registers, K streamed through LDS.  Row max and sum-of-exp are then plain
//          in-lane running scalars; the two half-waves are combined once at the end.  Emits per row
//          (m, log2 l) with l = sum_j 2^((s_ij - m) * c), c = scale*log2(e), or (m, l) per key split.
//   pass 2 (fcs_colstream_kernel, fcs_stream.hip)  column sums of 2^((s_ij - m_i) * c - log2 l_i),
//          one partial slab per group of (head, row block) units.
//   fcs_finalize_kernel (here) adds the slabs in a fixed order: no atomics anywhere, every
//          partial has exactly one writer.
//
// The fragment <-> head-dim mapping (which 8 channels a lane feeds to which MFMA step) is
// the same for both operands, which is all the contraction needs.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fcs_device.h"
#include "fcs_kernels.h"

namespace fcs {

// ------------------------------------------------------------------------------------
// pass 1: per-row log-sum-exp (or per-split partials)
// ------------------------------------------------------------------------------------
// WAVES = 4 or 8 waves per block: a block covers WAVES * QW query rows and streams its keys
// once, so taller blocks divide the key traffic of this pass.
template <int D, int QW, int WAVES, bool BF>
__global__ __launch_bounds__(64 * WAVES, 2) void fcs_rowstats_kernel(const Args a)
{
    constexpr int THREADS = 64 * WAVES;
    constexpr int NB = QW / 32;         // query fragments per wave
    constexpr int NT = D / 16;          // MFMA steps along the head dim
    constexpr int KT = kStageKeys;      // keys per LDS stage
    constexpr int NA = KT / 32;         // key fragments per stage
    constexpr int PITCH = D + 8;        // halves per LDS row (+16 B: conflict-free b128 reads)
    constexpr int CPR = D / 8;          // 16-byte pieces per row
    constexpr int CPT = KT * CPR / THREADS;  // pieces per thread per stage
    __shared__ __attribute__((aligned(16))) _Float16 lds[2][KT * PITCH];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, g = lane >> 5;
    int bx, by, bz;  // row blocks of one (key split, head) read the same keys: same XCD
    xcd_contiguous_block(bx, by, bz);
    const int bh = bz, b = bh / a.H, h = bh - b * a.H;
    const int chunk = by;
    const int q0 = bx * (WAVES * QW);
    const int qw0 = q0 + wave * QW;
    const _Float16 *qp = a.q + (int64_t)b * a.qs_b + (int64_t)h * a.qs_h;
    const _Float16 *kp = a.k + (int64_t)b * a.ks_b + (int64_t)kv_head(h, a.kv_group, a.kv_magic) * a.ks_h;

    // key range of this block: its split, cut at the last key any of its rows may see
    const int kc0 = chunk * a.chunk_keys;
    int kc1 = min(a.Sk, kc0 + a.chunk_keys);
    if (a.causal) kc1 = min(kc1, a.k_past + min(q0 + WAVES * QW, a.q_rows));
    const int nst = (kc1 > kc0) ? (kc1 - kc0 + KT - 1) / KT : 0;

    half8 qf[NB][NT];
    int thr[NB];  // last visible key of the lane's query
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int qi = qw0 + nb * 32 + r;
        const _Float16 *row = qp + (int64_t)min(qi, a.Sq - 1) * a.qs_s + g * 8;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            half8 v = kZero8;  // channels past the tensor's head dim (D is the compiled width) are zeros
            if (t * 16 + g * 8 < a.D) v = load8(row + t * 16);
            qf[nb][t] = a.negate ? flip_sign(v) : v;
        }
        thr[nb] = a.causal ? min(a.k_past + qi, a.Sk - 1) : a.Sk - 1;
    }
    const int thr_min = a.causal ? min(a.k_past + qw0, a.Sk - 1) : a.Sk - 1;  // wave-uniform

    float m[NB], l[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) { m[nb] = kNegBig; l[nb] = 0.f; }

    half8 stg[CPT];
    auto gload = [&](int kb) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * THREADS, row = c / CPR, col = (c % CPR) * 8;
            stg[i] = kZero8;
            if (col < a.D) stg[i] = load8(kp + (int64_t)min(kb + row, a.Sk - 1) * a.ks_s + col);
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * THREADS, row = c / CPR, col = (c % CPR) * 8;
            *reinterpret_cast<half8 *>(&lds[buf][row * PITCH + col]) = stg[i];
        }
    };

    // ---------------- common path: 2^(c*s) without max subtraction, exact while the row sums stay
    // inside [2^-80, 2^120).  Software-pipelined over (key fragment x all query fragments) groups:
    // the MFMAs of a group are issued before the exponent work of the previous group, so the
    // matrix pipe and the VALU run together inside one wave.
    bool redo;
    {
        float lacc[NB][4];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int j = 0; j < 4; ++j) lacc[nb][j] = 0.f;
        floatx16 cp[NB];  // scores of the previous group, not yet exponentiated
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int i = 0; i < 16; ++i) cp[nb][i] = 0.f;
        int p_kb = 0x3fffffff;  // key base of the previous group (the initial dummy hides every key)
        auto drain = [&]() {
            const bool edge = (p_kb + 31 > thr_min);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                if (!edge) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) lacc[nb][i & 3] += fast_exp2(cp[nb][i] * a.c);
                } else {
                    // the key indices are formed inside this branch (opaque base), or the compiler
                    // computes all sixteen ahead of the branch on every group
                    int kb_e = p_kb + 4 * g;
                    asm volatile("" : "+v"(kb_e));
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const float e = fast_exp2(cp[nb][i] * a.c);
                        lacc[nb][i & 3] += (kb_e + (8 * (i >> 2) + (i & 3)) <= thr[nb]) ? e : 0.f;
                    }
                }
            }
            // keeps the exponent work of this group between the MFMAs of the next two groups
            if (NB == 2)
                asm volatile("" : "+v"(lacc[0][0]), "+v"(lacc[0][1]), "+v"(lacc[0][2]), "+v"(lacc[0][3]), "+v"(lacc[NB - 1][0]),
                             "+v"(lacc[NB - 1][1]), "+v"(lacc[NB - 1][2]), "+v"(lacc[NB - 1][3]));
            else
                asm volatile("" : "+v"(lacc[0][0]), "+v"(lacc[0][1]), "+v"(lacc[0][2]), "+v"(lacc[0][3]));
        };

        if (nst > 0) { gload(kc0); lstore(0); }
        __syncthreads();
        for (int it = 0; it < nst; ++it) {
            const int kb = kc0 + it * KT;
            if (it + 1 < nst) gload(kb + KT);
            const _Float16 *tile = lds[it & 1];
#pragma unroll
            for (int na = 0; na < NA; ++na) {
                half8 af[NT];
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    af[t] = *reinterpret_cast<const half8 *>(&tile[(na * 32 + r) * PITCH + t * 16 + g * 8]);
                floatx16 cn[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) cn[nb][i] = 0.f;
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb)
                        cn[nb] = mfma16<BF>(af[t], qf[nb][t], cn[nb]);
                // the new MFMAs are in the instruction stream before the old scores are touched
                if (NB == 2)
                    asm volatile("" : "+v"(cn[0]), "+v"(cn[NB - 1]), "+v"(cp[0]), "+v"(cp[NB - 1]));
                else
                    asm volatile("" : "+v"(cn[0]), "+v"(cp[0]));
                drain();
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) cp[nb] = cn[nb];
                p_kb = kb + na * 32;
            }
            if (it + 1 < nst) lstore((it + 1) & 1);
            __syncthreads();
        }
        drain();

        bool bad = false;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const float lh = (lacc[nb][0] + lacc[nb][1]) + (lacc[nb][2] + lacc[nb][3]);
            const float lt = lh + __shfl_xor(lh, 32);  // both half-waves: the chunk's full row sum
            const bool has_keys = (nst > 0) && (kc0 <= thr[nb]);
            bad = bad || (has_keys && !(lt >= 8.2718061e-25f && lt < 1.3292280e+36f));
            m[nb] = has_keys ? 0.f : kNegBig;  // an empty split must not set the merged maximum
            l[nb] = lh;
        }
        redo = __syncthreads_or(bad) != 0;
    }

    // ---------------- rare: online max-subtracted softmax over the same keys
    if (redo) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) { m[nb] = kNegBig; l[nb] = 0.f; }
    if (nst > 0) { gload(kc0); lstore(0); }
    __syncthreads();
    for (int it = 0; it < nst; ++it) {
        const int kb = kc0 + it * KT;
        if (it + 1 < nst) gload(kb + KT);
        const _Float16 *tile = lds[it & 1];

        floatx16 acc[NA][NB];
#pragma unroll
        for (int na = 0; na < NA; ++na) {
            half8 af[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t)
                af[t] = *reinterpret_cast<const half8 *>(&tile[(na * 32 + r) * PITCH + t * 16 + g * 8]);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                floatx16 c = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    c = mfma16<BF>(af[t], qf[nb][t], c);
                acc[na][nb] = c;
            }
        }

        const bool edge = (kb + KT - 1 > thr_min);  // stage holds keys hidden from some row of this wave
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            if (!edge) {
                float tmax = acc[0][nb][0];
#pragma unroll
                for (int na = 0; na < NA; ++na)
#pragma unroll
                    for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, acc[na][nb][i]);
                const float mn = fmaxf(m[nb], tmax);
                const float alpha = fast_exp2((m[nb] - mn) * a.c);
                float sum = 0.f;  // the maximum is subtracted BEFORE the scale: exact for scores of any size
#pragma unroll
                for (int na = 0; na < NA; ++na)
#pragma unroll
                    for (int i = 0; i < 16; ++i) sum += fast_exp2((acc[na][nb][i] - mn) * a.c);
                l[nb] = l[nb] * alpha + sum;
                m[nb] = mn;
            } else {
                float tmax = kNegBig;
#pragma unroll
                for (int na = 0; na < NA; ++na)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const bool vis = (kb + na * 32 + acc_row(i, g)) <= thr[nb];
                        tmax = fmaxf(tmax, vis ? acc[na][nb][i] : kNegBig);
                    }
                const float mn = fmaxf(m[nb], tmax);
                const float alpha = fast_exp2((m[nb] - mn) * a.c);
                float sum = 0.f;
#pragma unroll
                for (int na = 0; na < NA; ++na)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const bool vis = (kb + na * 32 + acc_row(i, g)) <= thr[nb];
                        const float e = fast_exp2((acc[na][nb][i] - mn) * a.c);
                        sum += vis ? e : 0.f;
                    }
                l[nb] = l[nb] * alpha + sum;
                m[nb] = mn;
            }
        }

        if (it + 1 < nst) lstore((it + 1) & 1);
        __syncthreads();
    }

    }  // redo

    // combine the two half-waves (same query, disjoint keys) and store
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const float m2 = __shfl_xor(m[nb], 32), l2 = __shfl_xor(l[nb], 32);
        const float mm = fmaxf(m[nb], m2);
        const float ll = l[nb] * fast_exp2((m[nb] - mm) * a.c) + l2 * fast_exp2((m2 - mm) * a.c);
        if (g == 0) {
            const int qi = qw0 + nb * 32 + r;  // < rows_pad by construction
            // the maximum stays in score units and apart from log2 l: folding m * c into one fp32
            // would round it at the magnitude of m * c, which the later 2^(...) cannot undo
            float2 v;
            v.x = mm;
            if (a.n_chunks == 1) {
                v.y = fast_log2(ll);
                a.lse[(int64_t)bh * a.rows_pad + qi] = v;
            } else {
                v.y = ll;
                a.ml[((int64_t)bh * a.n_chunks + chunk) * a.rows_pad + qi] = v;
            }
        }
    }
}

// out = inv_norm * (partial[0] + partial[1] + ...).  A block owns 32 consecutive outputs; its
// 8 slab lanes each add every 8th slab in index order and the 8 sub-totals are then added in lane
// order, so the summation tree is fixed (bit-reproducible) while 8x more loads are in flight than
// with one thread per output.
__global__ __launch_bounds__(256) void fcs_finalize_kernel(const Args a)
{
    __shared__ float sub[8][32];
    const int64_t n = (int64_t)a.B * a.Sk;
    const int col = threadIdx.x & 31, sl = threadIdx.x >> 5;
    const int64_t idx = (int64_t)blockIdx.x * 32 + col;
    float s = 0.f;
    if (idx < n)
        for (int gi = sl; gi < a.n_partials; gi += 8) s += a.partial[(int64_t)gi * n + idx];
    sub[sl][col] = s;
    __syncthreads();
    if (sl == 0 && idx < n) {
        float t = sub[0][col];
#pragma unroll
        for (int j = 1; j < 8; ++j) t += sub[j][col];
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
    hipLaunchKernelGGL(fcs_finalize_kernel, dim3((unsigned)((n + 31) / 32)), dim3(256), 0, st, a);
    return hipGetLastError();
}

template <int D, bool BF>
static hipError_t launch_d(const Plan &p, const Args &a, hipStream_t st)
{
    const dim3 blk(256);
    {
        const dim3 grid(p.n_qblk, p.n_chunks, p.B * p.H);
        if constexpr (D <= 128) {
            if (p.qw == 64 && p.k1_waves == 8)
                hipLaunchKernelGGL((fcs_rowstats_kernel<D, 64, 8, BF>), grid, dim3(512), 0, st, a);
            else if (p.qw == 64)
                hipLaunchKernelGGL((fcs_rowstats_kernel<D, 64, 4, BF>), grid, blk, 0, st, a);
            else
                hipLaunchKernelGGL((fcs_rowstats_kernel<D, 32, 4, BF>), grid, blk, 0, st, a);
        } else {  // 64 query rows per wave would not fit the registers
            if (p.qw != 32 || p.k1_waves != 4) return hipErrorInvalidValue;
            hipLaunchKernelGGL((fcs_rowstats_kernel<D, 32, 4, BF>), grid, blk, 0, st, a);
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    {
        hipError_t e = launch_colstream(p, a, st);  // merges the key splits of pass 1 itself
        if (e != hipSuccess) return e;
    }
    if (p.c_groups > 1) {
        hipError_t e = launch_finalize(a, st);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

int launch_colsum(const Plan &p, const Args &a, void *stream)
{
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (p.fewrows) return (int)launch_fewrows(p, a, st);
    if (p.fused) return (int)launch_fused(p, a, st);
    hipError_t e;
    if (p.bf16)
        e = (p.Dp == 64) ? launch_d<64, true>(p, a, st) : (p.Dp == 128) ? launch_d<128, true>(p, a, st) : launch_d<256, true>(p, a, st);
    else
        e = (p.Dp == 64) ? launch_d<64, false>(p, a, st) : (p.Dp == 128) ? launch_d<128, false>(p, a, st) : launch_d<256, false>(p, a, st);
    return (int)e;
}

}  // namespace fcs
