// Kernel argument block and the single launch entry used by the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fcs_plan.h"

namespace fcs {

struct Args {
    const _Float16 *q;
    const _Float16 *k;
    int64_t qs_b, qs_h, qs_s;  // element strides (last dim is 1)
    int64_t ks_b, ks_h, ks_s;
    int B, H, Sq, Sk;
    int D;               // head dim of the tensors (a multiple of 8); kernels compiled for a wider head read zeros beyond it
    int kv_group;        // query heads per key head (1 unless grouped-query): key head = head / kv_group
    uint32_t kv_magic;   // ceil(2^32 / kv_group), for the division above (unused when kv_group == 1)
    int q_rows;          // query rows that are averaged
    int causal, k_past;  // key j visible to query i  <=>  j <= k_past + i
    int pre_end;         // two-pass path, pre-scaled variant: the 64-key stages that end at or below this key (a multiple
                         // of 64) run on Q * c rounded to fp16 in both passes; the keys that every averaged row sees
    int negate;          // scale < 0: scores are negated by flipping the stationary operand's sign
    float c;             // |scale| * log2(e)
    // pass 1
    int n_chunks, chunk_keys, rows_pad;
    float2 *lse;  // [B*H][rows_pad]            (m, log2 l): row maximum in score units (0 on the
                  //                            unstabilised path) and log2 of sum_j 2^((s_ij - m) * c)
    float2 *ml;   // [B*H][n_chunks][rows_pad]  (m, l) of each key split
    // pass 2
    int c_chunk, c_groups, c_upg, c_nrb;  // column pass: keys per block, unit groups, units per group, row blocks per head
    int c_nchunks;       // column pass: key chunks (its grid is c_nchunks x c_groups x B, launched as one dimension)
    int n_qblk;          // pass 1: row blocks (its grid is n_qblk x n_chunks x B*H, launched as one dimension)
    float *partial;  // [groups][B][Sk]
    float *out;      // [B][Sk]
    _Float16 *out_h; // [B][Sk] or nullptr: the same means rounded to fp16
    float inv_norm;  // 1 / (H * q_rows)
    int n_partials;  // slabs of `partial` that fcs_finalize_kernel adds up
    // fused single-kernel path (scores stay in registers)
    int f_kg;        // waves along the key axis (1, 2, 4 or 8); 8 / f_kg waves along the query axis
    int f_tpw;       // 32-key tiles per wave (<= 8)
    int f_nqblk;     // blocks along the query axis (32 * 8 / f_kg rows each; short-sequence path: 32-row tiles per head)
    int f_hpg;       // heads per block
    int f_rbpw;      // adjacent row blocks per block (a block walks over f_rbpw x f_hpg units)
    int f_nwgq;      // blocks along the query axis: ceil(f_nqblk / f_rbpw)
    int f_hg;        // head groups (fused and few-rows paths): a batch entry has f_hg * f_nwgq workgroups
};

// Enqueues every kernel of one call on `stream`; returns 0 or the hipError_t of a failed launch.
int launch_colsum(const Plan &p, const Args &a, void *stream);

// fused path, defined in fcs_fused.hip
hipError_t launch_fused(const Plan &p, const Args &a, hipStream_t st);
// few-rows path (fcs_fewrows.hip): p.fewrows == 1
hipError_t launch_fewrows(const Plan &p, const Args &a, hipStream_t st);
// short-sequence path (fcs_small.hip): p.small == 1
hipError_t launch_small(const Plan &p, const Args &a, hipStream_t st);

// row-statistics pass and column pass of the two-pass path (fcs_stream.hip)
hipError_t launch_rowstream(const Plan &p, const Args &a, hipStream_t st);
hipError_t launch_colstream(const Plan &p, const Args &a, hipStream_t st);

// shared final reduction out = inv_norm * sum of the n_partials slabs (fcs_kernels.hip)
hipError_t launch_finalize(const Args &a, hipStream_t st);

// Text description of what launch_colsum(p, a, .) launches; snprintf semantics.
size_t describe_colsum(const Plan &p, const Args &a, char *buf, size_t n);
size_t describe_fused(const Plan &p, const Args &a, char *buf, size_t n);
size_t describe_fewrows(const Plan &p, const Args &a, char *buf, size_t n);
size_t describe_small(const Plan &p, const Args &a, char *buf, size_t n);
size_t describe_two_pass(const Plan &p, const Args &a, char *buf, size_t n);
size_t describe_finalize(const Args &a, char *buf, size_t n);

}  // namespace fcs
