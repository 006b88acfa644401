// Top-k / threshold selection over the fp32 column means, on the GPU and on the caller's stream.
//
// The consumer of the column means is token-importance ranking for pruning (reference:
// README.md:10): it wants the k most-attended key positions of every batch row.  Selecting on the
// kernels' fp32 means, right behind the final reduction and without a host round trip, keeps the
// small means of long contexts that the reference's fp16 result flushes to zero
// (reference: flash_colsum/kernel_causal.py:124).
//
// One workgroup of 1024 threads per batch row:
//   1. radix select, most significant byte first: four passes over the row, each building a
//      256-bin histogram (LDS atomics on integers) of the current byte among the elements that
//      match the bytes fixed so far; the histogram's suffix sums fix the next byte of the k-th
//      largest key.  Floats are ordered through the usual monotone map to unsigned integers.
//   2. ordered compaction: tiles of 1024 elements in index order; an element is taken if it is
//      larger than the k-th largest value, or equal to it and among the first `need` such elements
//      (ties go to the LOWER index).  Ballot / popcount scans give every taken element its place,
//      so the result lists the indices in ascending order and is bit-reproducible.
//   3. optionally (k <= kTopkSortMax) a bitonic sort in LDS orders the k results by descending
//      value, ties by ascending index.
// The threshold form is step 2 alone with a given threshold.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flash_colsum.h"
#include "fcs_kernels.h"

namespace fcs {

namespace {

constexpr int kTopkSortMax = FCS_TOPK_SORT_MAX;
constexpr int kTopkThreads = 1024;
constexpr int kTopkWaves = kTopkThreads / 64;

// monotone map float -> uint32: a < b  <=>  key(a) < key(b)  (-0 < +0, NaNs at the two ends)
__device__ __forceinline__ uint32_t order_key(float v)
{
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// exclusive prefix count of `flag` over the workgroup in thread order, and the workgroup's total.
// `wsum` is LDS scratch of kTopkWaves + 1 ints.  Two barriers.
__device__ __forceinline__ int block_rank(bool flag, int *wsum, int &total)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint64_t b = __builtin_amdgcn_ballot_w64(flag);
    const int before = __builtin_popcountll(b & ((1ull << lane) - 1ull));
    __syncthreads();  // the scratch may still be read from the previous use
    if (lane == 0) wsum[wave] = __builtin_popcountll(b);
    __syncthreads();
    int base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kTopkWaves; ++w) {
        const int c = wsum[w];
        base += (w < wave) ? c : 0;
        tot += c;
    }
    total = tot;
    return base + before;
}

// taken elements of one row in ascending index order.  thr_key: elements with a larger key are taken;
// `need` more with an equal key (lowest indices first).  Returns the number written (<= cap).
// CANON: -0 counts as +0 (the value comparison `>=` of the threshold form, not the bit order of top-k).
template <bool CANON>
__device__ int compact_row(const float *row, int S, uint32_t thr_key, int need, int64_t *idx_out, float *val_out, int cap,
                           int *wsum)
{
    int written = 0, eq_seen = 0;  // block-uniform running counts
    for (int base = 0; base < S; base += kTopkThreads) {
        const int i = base + threadIdx.x;
        float v = 0.f;
        uint32_t key = 0;
        const bool in = i < S;
        if (in) {
            v = row[i];
            key = order_key(CANON ? v + 0.0f : v);
        }
        const bool eq = in && key == thr_key;
        int eq_tot;
        const int eq_rank = block_rank(eq, wsum, eq_tot);
        const bool take = in && (key > thr_key || (eq && eq_seen + eq_rank < need));
        int take_tot;
        const int pos = written + block_rank(take, wsum, take_tot);
        if (take && pos < cap) {
            idx_out[pos] = i;
            if (val_out) val_out[pos] = v;
        }
        written += take_tot;
        eq_seen += eq_tot;
    }
    return written;
}

}  // namespace

__global__ __launch_bounds__(kTopkThreads) void fcs_topk_kernel(const float *means, int S, int k, int64_t *idx_out,
                                                                float *val_out, int sorted)
{
    __shared__ int hist[256];
    __shared__ int wsum[kTopkWaves + 1];
    __shared__ uint32_t sel_s[2];  // [0] the chosen byte, [1] elements still wanted among those that match the prefix
    __shared__ float sv[kTopkSortMax];
    __shared__ int si[kTopkSortMax];

    const int tid = threadIdx.x;
    const float *row = means + (int64_t)blockIdx.x * S;
    int64_t *io = idx_out + (int64_t)blockIdx.x * k;
    float *vo = val_out ? val_out + (int64_t)blockIdx.x * k : nullptr;

    // ---- 1. the k-th largest key, byte by byte
    uint32_t prefix = 0, mask = 0;
    int want = k;  // rank (1 = largest) of the wanted key among the elements that match the prefix
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        for (int i = tid; i < S; i += kTopkThreads) {
            const uint32_t key = order_key(row[i]);
            if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1);
        }
        __syncthreads();
        if (tid < 64) {
            // lane L owns bins 4L .. 4L+3; suffix sums over lanes, then within the lane, find the bin b with
            // count(bins > b) < want <= count(bins >= b)
            const int c0 = hist[4 * tid], c1 = hist[4 * tid + 1], c2 = hist[4 * tid + 2], c3 = hist[4 * tid + 3];
            const int mine = c0 + c1 + c2 + c3;
            int above = 0;  // elements in bins of higher lanes
            for (int l = 0; l < 64; ++l) {
                const int o = __shfl(mine, l);
                above += (l > tid) ? o : 0;
            }
            const int cs[4] = {c0, c1, c2, c3};
            int acc = above;
#pragma unroll
            for (int j = 3; j >= 0; --j) {
                if (acc < want && want <= acc + cs[j]) {
                    sel_s[0] = (uint32_t)(4 * tid + j);
                    sel_s[1] = (uint32_t)(want - acc);
                }
                acc += cs[j];
            }
        }
        __syncthreads();
        prefix |= sel_s[0] << shift;
        mask |= 255u << shift;
        want = (int)sel_s[1];
        __syncthreads();
    }
    // `prefix` is the k-th largest key; `want` of the elements equal to it are taken

    // ---- 2. ordered compaction
    compact_row<false>(row, S, prefix, want, io, vo ? vo : nullptr, k, wsum);

    // ---- 3. descending values, ties by ascending index
    if (sorted && k <= kTopkSortMax) {
        __syncthreads();
        int n2 = 1;
        while (n2 < k) n2 <<= 1;
        for (int i = tid; i < n2; i += kTopkThreads) {
            if (i < k) {
                si[i] = (int)io[i];
                sv[i] = row[io[i]];
            } else {  // padding (recognised by its index) sorts behind every real entry, negative NaNs included
                si[i] = 0x7fffffff;
                sv[i] = 0.f;
            }
        }
        __syncthreads();
        // bitonic network; "a before b"  <=>  key(a) > key(b), or equal keys and index(a) < index(b)
        for (int size = 2; size <= n2; size <<= 1) {
            for (int stride = size >> 1; stride > 0; stride >>= 1) {
                for (int t = tid; t < (n2 >> 1); t += kTopkThreads) {
                    const int lo = 2 * t - (t & (stride - 1));  // index with the `stride` bit clear
                    const int hi = lo + stride;
                    const bool desc_block = ((lo & size) == 0);  // this block ends up in "before" order
                    const uint32_t ka = (si[lo] == 0x7fffffff) ? 0u : order_key(sv[lo]);
                    const uint32_t kb = (si[hi] == 0x7fffffff) ? 0u : order_key(sv[hi]);
                    const bool a_first = ka > kb || (ka == kb && si[lo] < si[hi]);
                    if (a_first != desc_block) {
                        const float tv = sv[lo];
                        sv[lo] = sv[hi];
                        sv[hi] = tv;
                        const int ti = si[lo];
                        si[lo] = si[hi];
                        si[hi] = ti;
                    }
                }
                __syncthreads();
            }
        }
        for (int i = tid; i < k; i += kTopkThreads) {
            io[i] = si[i];
            if (vo) vo[i] = sv[i];
        }
    }
}

__global__ __launch_bounds__(kTopkThreads) void fcs_threshold_kernel(const float *means, int S, float tau, int64_t *idx_out,
                                                                     int32_t *count_out)
{
    __shared__ int wsum[kTopkWaves + 1];
    const float *row = means + (int64_t)blockIdx.x * S;
    // value >= tau  <=>  key(value) >= key(tau) once -0 is read as +0 on both sides (the bit order alone puts
    // -0 below +0): "larger than thr, or equal to thr with unlimited ties" with thr = key(tau + 0)
    const int n = compact_row<true>(row, S, order_key(tau + 0.0f), 0x7fffffff, idx_out + (int64_t)blockIdx.x * S, nullptr, S, wsum);
    if (threadIdx.x == 0) count_out[blockIdx.x] = n;
}

}  // namespace fcs

extern "C" {

int fcs_topk_f32(const float *means, int B, int S, int k, int64_t *idx_out, float *val_out, int sorted, void *hip_stream)
{
    if (!means || !idx_out) return FCS_E_NULL;
    if (B < 1 || S < 1 || k < 1 || k > S) return FCS_E_DIMS;
    if (sorted && k > FCS_TOPK_SORT_MAX) return FCS_E_DIMS;
    hipLaunchKernelGGL(fcs::fcs_topk_kernel, dim3(B), dim3(fcs::kTopkThreads), 0, reinterpret_cast<hipStream_t>(hip_stream), means, S,
                       k, idx_out, val_out, sorted ? 1 : 0);
    return (int)hipGetLastError();
}

int fcs_threshold_f32(const float *means, int B, int S, float tau, int64_t *idx_out, int32_t *count_out, void *hip_stream)
{
    if (!means || !idx_out || !count_out) return FCS_E_NULL;
    if (B < 1 || S < 1) return FCS_E_DIMS;
    if (tau != tau) return FCS_E_SCALE;
    hipLaunchKernelGGL(fcs::fcs_threshold_kernel, dim3(B), dim3(fcs::kTopkThreads), 0, reinterpret_cast<hipStream_t>(hip_stream), means,
                       S, tau, idx_out, count_out);
    return (int)hipGetLastError();
}

}  // extern "C"
