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
    int q_rows;          // query rows that are averaged
    int causal, k_past;  // key j visible to query i  <=>  j <= k_past + i
    int negate;          // scale < 0: scores are negated by flipping the stationary operand's sign
    float c;             // |scale| * log2(e)
    // pass 1
    int n_chunks, chunk_keys, rows_pad;
    float *lse;   // [B*H][rows_pad]
    float2 *ml;   // [B*H][n_chunks][rows_pad]
    // pass 2
    int gh, gq, heads_per_group, qtiles_per_group;
    float *partial;  // [gh*gq][B][Sk]
    float *out;      // [B][Sk]
    float inv_norm;  // 1 / (H * q_rows)
};

// Enqueues every kernel of one call on `stream`; returns 0 or the hipError_t of a failed launch.
int launch_colsum(const Plan &p, const Args &a, void *stream);

}  // namespace fcs
