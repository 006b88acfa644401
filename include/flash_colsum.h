/* flash_colsum.h -- C ABI of libflashcolsum.so (gfx950 / MI355X).
 *
 * Attention column means without materialising the attention matrix:
 *
 *     out[b][j] = 1/(H*rows) * sum_h sum_{i<rows} softmax_j( scale * <q[b,h,i,:], k[b,h,j,:]> )
 *
 * These entry points are what the host layer of the reference operator binds in place of
 * its three Triton launchers.  All pointers are DEVICE pointers unless stated otherwise.
 * The library never allocates, frees or synchronises: the caller owns the output and the
 * workspace, and every kernel is enqueued on the HIP stream passed in.  Calls are
 * re-entrant (the only state kept between calls is a per-thread memo of recent launch plans).
 *
 * Return value of the launch functions: 0 = all kernels enqueued; negative = argument
 * error detected on the host before anything touched the GPU (FCS_E_*); positive = the
 * hipError_t returned by a failed launch.
 */
#ifndef FLASH_COLSUM_H
#define FLASH_COLSUM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FCS_ABI_VERSION 5

enum {
    FCS_OK = 0,
    FCS_E_NULL = -1,      /* a required pointer is NULL                                  */
    FCS_E_DIMS = -2,      /* a dimension is < 1, or cls_n == 0, or k_past < 0, or the call
                             would need 2^31 workgroups or more                          */
    FCS_E_HEAD_DIM = -3,  /* D is not a multiple of 8 in [8, 256]                        */
    FCS_E_STRIDE = -4,    /* last-dim stride != 1, or a stride / base not 16-B aligned   */
    FCS_E_WORKSPACE = -5, /* ws_bytes smaller than fcs_workspace_bytes() for these dims,
                             or ws not 256-byte aligned                                  */
    FCS_E_SCALE = -6,     /* scale is NaN or infinite                                    */
    FCS_E_STATIC_LIMIT = -7, /* fcs_colsum_noncausal_f16_static: the call needs more workspace
                                than FCS_STATIC_SCRATCH_BYTES                              */
    FCS_E_DTYPE = -8,     /* fcs_colsum_general: dtype is not FCS_DTYPE_F16 / FCS_DTYPE_BF16 */
    FCS_E_STRUCT = -9     /* fcs_colsum_call: struct_bytes is not sizeof(fcs_call_t)      */
};

/* Size of the per-GPU static scratch array behind fcs_colsum_noncausal_f16_static(). */
#define FCS_STATIC_SCRATCH_BYTES (8u << 20)

/* ABI version of the loaded library (== FCS_ABI_VERSION of the header it was built with). */
int fcs_abi_version(void);

/* Static, human-readable text for a return code of this library (negative codes) or a
 * generic text for positive (HIP) codes.  Never NULL. */
const char *fcs_strerror(int code);

/* Bytes of device workspace the launch functions need for these dimensions (row
 * statistics and per-group partial column sums).  `causal` selects the entry point;
 * for the fcs_colsum_causal_* entry points pass B = 1 and cls_n = -1 (they average all rows);
 * H is the number of QUERY heads.  `cls_n` <= 0 means "all rows".  Returns 0 for
 * invalid dimensions.  The workspace needs no initialisation and 256-byte alignment.
 * Replaces the implicit `torch.zeros` accumulator of the reference launchers
 * (reference: flash_colsum/kernel_noncausal_batched.py:104, kernel_noncausal.py:98,
 * kernel_causal.py:105). */
size_t fcs_workspace_bytes(int causal, int B, int H, int Sq, int Sk, int D, int cls_n);

/* Non-causal column means, fp16 inputs, fp32 output.
 *   q, k       (B,H,S,D) fp16, element strides q_strides[4] / k_strides[4] (HOST arrays);
 *              the last stride must be 1 and rows must be 16-byte aligned.
 *   out        (B,S) fp32 contiguous; receives the MEANS (already divided by H*rows).
 *   out_f16    NULL, or (B,S) fp16 contiguous that additionally receives the means rounded
 *              to fp16 (the reference's result dtype) without a separate cast kernel.
 *   cls_n      <= -1 (or any negative): average over all S query rows;
 *              >= 1: average over the first min(cls_n, S) query rows only.
 * Replaces `_flash_colsum_batched(Q, K, scale, CLS_N)` and
 * `_flash_colsum_non_batched(Q, K, scale, CLS_N)` including their host epilogue
 * (reference: flash_colsum/kernel_noncausal_batched.py:102-125,
 * flash_colsum/kernel_noncausal.py:95-117; called from flash_colsum/ops.py:102-105). */
int fcs_colsum_noncausal_f16(const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes,
                             int B, int H, int S, int D,
                             const int64_t q_strides[4], const int64_t k_strides[4],
                             float scale, int cls_n, void *hip_stream);

/* fcs_colsum_noncausal_f16 for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): same arguments minus
 * the workspace, which is a static device array of FCS_STATIC_SCRATCH_BYTES that every GPU
 * the library runs on holds until the process ends.  Has no counterpart in the reference.
 * Calls no hipMalloc / hipFree or any allocating routine.  Returns FCS_E_STATIC_LIMIT when
 * fcs_workspace_bytes(0, B, H, S, S, D, cls_n) exceeds FCS_STATIC_SCRATCH_BYTES (8 MiB: enough
 * for B=8 H=16 S=2048 D=64, which needs 2 MiB).  All calls on one GPU share that GPU's array:
 * calls that overlap in time on one GPU (different streams or threads) race; calls on one
 * stream are ordered and safe.  Results are bit-identical to fcs_colsum_noncausal_f16.
 * The first call on a GPU looks up the array's device address (hipGetSymbolAddress), which may
 * load the code object: make that call, or fcs_static_scratch_init(), outside stream capture.  A
 * failed look-up is not remembered; the next call tries again. */
int fcs_colsum_noncausal_f16_static(const void *q, const void *k, float *out, void *out_f16,
                                    int B, int H, int S, int D,
                                    const int64_t q_strides[4], const int64_t k_strides[4],
                                    float scale, int cls_n, void *hip_stream);

/* Looks up the current GPU's static scratch array without launching anything (0, or a hipError_t). */
int fcs_static_scratch_init(void);

/* Causal column means for one sequence (batch 1), fp16 inputs, fp32 output.
 *   q          (1,H,Q_len,D), k (1,H,K_len,D) fp16; strides as above (index 0 ignored).
 *   out        (K_len) fp32; receives the means over the H*Q_len rows.
 *   out_f16    NULL, or (K_len) fp16 that additionally receives the rounded means.
 *   k_past     number of keys every query may see before its own position: key j is
 *              visible to query i  <=>  j <= k_past + i.  The reference infers
 *              max(0, K_len - Q_len); pass that for drop-in behaviour.  Any value >= K_len
 *              (INT_MAX included) means "no mask" and is treated as K_len.
 * Replaces `_flash_colsum_causal(Q, K, scale, K_past)` including its host epilogue
 * (reference: flash_colsum/kernel_causal.py:94-125; called from flash_colsum/ops.py:89). */
int fcs_colsum_causal_f16(const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes,
                          int H, int Q_len, int K_len, int D, int k_past,
                          const int64_t q_strides[4], const int64_t k_strides[4],
                          float scale, void *hip_stream);

/* The same two launch functions for bf16 inputs: q and k hold bfloat16 values (same shapes,
 * strides in elements, alignment rules, workspace size and outputs as above; `out_f16` is still
 * IEEE fp16, the reference's result dtype for every input dtype).  Products are exact and
 * accumulated in fp32, like the reference kernels, which upcast their operands before the
 * dot product (reference: flash_colsum/kernel_noncausal_batched.py:37,54,
 * flash_colsum/kernel_causal.py:32,52). */
int fcs_colsum_noncausal_bf16(const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes,
                              int B, int H, int S, int D,
                              const int64_t q_strides[4], const int64_t k_strides[4],
                              float scale, int cls_n, void *hip_stream);
int fcs_colsum_causal_bf16(const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes,
                           int H, int Q_len, int K_len, int D, int k_past,
                           const int64_t q_strides[4], const int64_t k_strides[4],
                           float scale, void *hip_stream);

/* General form: the shapes the reference operator still rejects, on the same kernels.
 *   dtype      FCS_DTYPE_F16 or FCS_DTYPE_BF16 (operand type of q and k).
 *   causal     0 / 1.  With causal != 0 any B >= 1 is accepted: every batch entry is masked with
 *              the same k_past (the reference raises for B != 1, flash_colsum/ops.py:79-82).
 *   Hq, Hk     query and key heads, Hq a multiple of Hk: query head h attends to key head
 *              h / (Hq / Hk), the grouping of grouped-query / multi-query attention (the
 *              reference raises for Hq != Hk, flash_colsum/ops.py:83-87).  q is (B,Hq,Sq,D),
 *              k is (B,Hk,Sk,D).
 *   Sq, Sk     may differ for causal == 0 too (cross-attention shape).
 *   cls_n      as above, and also honoured for causal != 0: the mean runs over the first
 *              min(cls_n, Sq) query rows (the reference raises, flash_colsum/ops.py:65-66).
 *   out        (B,Sk) fp32 means over the Hq * rows averaged rows; out_f16 optional as above.
 *   ws         fcs_workspace_bytes(causal, B, Hq, Sq, Sk, D, cls_n) bytes.
 * With Hq == Hk, and B == 1, cls_n < 0 when causal, the result is bit-identical to the entry
 * points above. */
enum { FCS_DTYPE_F16 = 0, FCS_DTYPE_BF16 = 1 };
int fcs_colsum_general(int dtype, int causal, const void *q, const void *k, float *out, void *out_f16,
                       void *ws, size_t ws_bytes, int B, int Hq, int Hk, int Sq, int Sk, int D,
                       int cls_n, int k_past, const int64_t q_strides[4], const int64_t k_strides[4],
                       float scale, void *hip_stream);

/* One call as a struct: the arguments of fcs_colsum_general().  For host layers whose
 * foreign-function interface pays per argument (ctypes, cgo, JNI): fill the shape, strides and dtype
 * once per tensor geometry, update the pointers and call.  The struct is only read.
 *   struct_bytes  sizeof(fcs_call_t), checked (FCS_E_STRUCT).
 *   flags         0 (reserved).
 * All other fields mean what the like-named arguments of fcs_colsum_general() mean. */
typedef struct fcs_call {
    uint32_t struct_bytes;
    uint32_t flags;
    int32_t dtype, causal;
    int32_t B, Hq, Hk, Sq, Sk, D;
    int32_t cls_n, k_past;
    float scale;
    int32_t reserved;  /* 0 */
    int64_t q_strides[4], k_strides[4];
    const void *q, *k;
    float *out;
    void *out_f16;
    void *ws;
    size_t ws_bytes;
    void *hip_stream;
} fcs_call_t;
int fcs_colsum_call(const fcs_call_t *call);

/* Text description of the launch plan fcs_colsum_call() would use for `call` (kernels with their
 * template arguments, grids, slabs), for benchmark records and logs; pointers in `call` are not
 * dereferenced and may be NULL.  Writes at most buf_bytes - 1 characters plus a terminating NUL
 * and returns the length of the full text (like snprintf); 0 for invalid dimensions. */
size_t fcs_plan_describe(const fcs_call_t *call, char *buf, size_t buf_bytes);

/* Selection over the fp32 means, for the consumer the reference names (token-importance ranking
 * for pruning, reference: README.md:10): it runs on the same stream right behind a launch function
 * above and reads its fp32 `out`, so the small means of long contexts are ranked before the fp16
 * rounding of the reference's result (reference: flash_colsum/kernel_causal.py:124) can flush them.
 *
 * fcs_topk_f32: for every row b of means (B,S) the k largest entries.
 *   idx_out   (B,k) int64: their positions.  sorted == 0: in ascending position order;
 *             sorted != 0 (k <= FCS_TOPK_SORT_MAX): by descending value, equal values by ascending
 *             position.
 *   val_out   NULL or (B,k) fp32: the values in the same order.
 *   Ties at the k-th value go to the LOWER position.  Values are compared in the total order of
 *   their bit patterns (-0 < +0).  Deterministic; needs no workspace.
 * fcs_threshold_f32: for every row the positions of the entries >= tau, ascending.
 *   idx_out   (B,S) int64: row b holds count_out[b] positions (the rest is left untouched).
 *   count_out (B) int32.
 *   `>=` is the comparison of values: -0 and +0 are equal, on either side.  (A NaN entry is listed
 *   when its sign bit is clear and skipped when it is set; the means never hold one.)
 * Return codes as above (FCS_E_DIMS: k < 1, k > S, or sorted with k > FCS_TOPK_SORT_MAX;
 * FCS_E_SCALE: tau is NaN). */
#define FCS_TOPK_SORT_MAX 4096
int fcs_topk_f32(const float *means, int B, int S, int k, int64_t *idx_out, float *val_out, int sorted,
                 void *hip_stream);
int fcs_threshold_f32(const float *means, int B, int S, float tau, int64_t *idx_out, int32_t *count_out,
                      void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_COLSUM_H */
