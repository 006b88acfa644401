// C ABI of libflashcolsum.so: argument checks, launch plan, workspace carving.
// Declarations and the reference call sites they replace: include/flash_colsum.h.
#include <math.h>
#include <string.h>

#include <mutex>

#include "flash_colsum.h"
#include "fcs_kernels.h"

// Workspace of fcs_colsum_noncausal_f16_static(): one copy per GPU, held until the process ends.
// Host code never uses this name as an address (it is only a handle for hipGetSymbolAddress).
static __device__ __align__(256) unsigned char fcs_static_scratch[FCS_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];  // device address of fcs_static_scratch on each GPU; only a successful look-up is kept
std::mutex g_scratch_mutex;

// Device address of the current GPU's copy of the static scratch array; no allocation.
hipError_t static_scratch(void **ptr)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(fcs_static_scratch));
        if (e != hipSuccess) return e;  // not remembered: the next call looks it up again
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return hipSuccess;
}

// The launch plan of a call is a pure function of its dimensions; the search behind it costs
// microseconds (more with many heads), so every thread remembers the plans of its last few
// geometries.
struct PlanKey {
    int causal, B, H, Sq, Sk, D, cls_n, k_past;
    bool operator==(const PlanKey &o) const
    {
        return causal == o.causal && B == o.B && H == o.H && Sq == o.Sq && Sk == o.Sk && D == o.D && cls_n == o.cls_n &&
               k_past == o.k_past;
    }
};
constexpr int kPlanMemo = 8;
struct PlanMemo {
    PlanKey key[kPlanMemo];
    fcs::Plan plan[kPlanMemo];
    bool used[kPlanMemo];
    int next;
};
thread_local PlanMemo t_memo;

bool cached_plan(fcs::Plan &p, int causal, int B, int H, int Sq, int Sk, int D, int cls_n, int k_past)
{
    const PlanKey key{causal, B, H, Sq, Sk, D, cls_n, k_past};
    PlanMemo &m = t_memo;
    for (int i = 0; i < kPlanMemo; ++i)
        if (m.used[i] && m.key[i] == key) {
            p = m.plan[i];
            return true;
        }
    if (!fcs::make_plan(p, causal, B, H, Sq, Sk, D, cls_n, k_past)) return false;
    const int slot = m.next;
    m.next = (slot + 1) % kPlanMemo;
    m.key[slot] = key;
    m.plan[slot] = p;
    m.used[slot] = true;
    return true;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// last-dim stride 1 and every other stride a multiple of 8 halves (16 bytes)
bool strides_ok(const int64_t s[4], bool use_batch)
{
    if (s[3] != 1) return false;
    if ((s[2] & 7) || (s[1] & 7)) return false;
    if (use_batch && (s[0] & 7)) return false;
    return true;
}

// Checks one call and fills its launch plan and kernel arguments.  H = query heads, Hk = key heads
// (H % Hk == 0; query head h reads key head h / (H / Hk)).  `need_ptrs` is false for fcs_plan_describe.
int prepare(fcs::Plan &p, fcs::Args &a, int bf16, int causal, const void *q, const void *k, float *out, void *out_f16, void *ws,
            size_t ws_bytes, int B, int H, int Hk, int Sq, int Sk, int D, const int64_t qs[4], const int64_t ks[4], float scale,
            int cls_n, int k_past, uint32_t flags, bool need_ptrs)
{
    if (need_ptrs && (!q || !k || !out)) return FCS_E_NULL;
    if (!qs || !ks) return FCS_E_NULL;
    if (B < 1 || H < 1 || Hk < 1 || Sq < 1 || Sk < 1 || D < 1 || cls_n == 0 || k_past < 0) return FCS_E_DIMS;
    if (H % Hk != 0) return FCS_E_DIMS;
    if (D < 8 || D > 256 || (D & 7)) return FCS_E_HEAD_DIM;
    if (!strides_ok(qs, B > 1) || !strides_ok(ks, B > 1) || !aligned16(q) || !aligned16(k)) return FCS_E_STRIDE;
    if (!isfinite(scale)) return FCS_E_SCALE;
    // every key is visible to every row from k_past = Sk - 1 on: larger values (INT_MAX as "no mask")
    // mean the same and must not reach the kernels' 32-bit row arithmetic
    if (k_past > Sk) k_past = Sk;

    if (!cached_plan(p, causal, B, H, Sq, Sk, D, cls_n, k_past)) return FCS_E_DIMS;
    p.bf16 = bf16;
    if (need_ptrs) {
        if (ws && (reinterpret_cast<uintptr_t>(ws) & 255u)) return FCS_E_WORKSPACE;
        if (p.total > 0 && (!ws || ws_bytes < p.total)) return ws ? FCS_E_WORKSPACE : FCS_E_NULL;
    }

    memset(&a, 0, sizeof(a));
    a.q = static_cast<const _Float16 *>(q);
    a.k = static_cast<const _Float16 *>(k);
    a.qs_b = qs[0]; a.qs_h = qs[1]; a.qs_s = qs[2];
    a.ks_b = ks[0]; a.ks_h = ks[1]; a.ks_s = ks[2];
    a.B = B; a.H = H; a.Sq = Sq; a.Sk = Sk;
    a.D = D;
    a.kv_group = H / Hk;
    a.kv_magic = (uint32_t)((0x100000000ull + (uint64_t)a.kv_group - 1) / (uint64_t)a.kv_group);  // unused when the group is 1
    a.q_rows = p.q_rows;
    a.causal = p.causal; a.k_past = p.k_past;
    // keys j <= k_past are visible to every row; whole stages of them
    a.pre_end = p.causal ? (int)((((long)p.k_past + 1) / fcs::kStageKeys) * fcs::kStageKeys) : 0x3fffffc0;
    a.negate = scale < 0.f;
    a.c = fabsf(scale) * 1.44269504088896340736f;
    a.n_chunks = p.n_chunks; a.chunk_keys = p.chunk_keys; a.rows_pad = p.rows_pad;
    char *w = static_cast<char *>(ws);
    a.lse = reinterpret_cast<float2 *>(w + p.off_lse);
    a.ml = reinterpret_cast<float2 *>(w + p.off_ml);
    a.c_chunk = p.c_chunk; a.c_groups = p.c_groups; a.c_upg = p.c_upg; a.c_nrb = p.c_nrb;
    a.c_nchunks = p.c_nchunks; a.n_qblk = p.n_qblk;
    a.partial = reinterpret_cast<float *>(w + p.off_partial);
    a.out = out;
    a.out_h = static_cast<_Float16 *>(out_f16);
    a.inv_norm = 1.0f / ((float)H * (float)p.q_rows);
    a.n_partials = p.n_partials;
    a.f_kg = p.f_kg; a.f_tpw = p.f_tpw; a.f_nqblk = p.f_nqblk; a.f_hpg = p.f_hpg;
    a.f_rbpw = p.f_rbpw; a.f_nwgq = p.f_nwgq; a.f_hg = p.f_hg;
    (void)flags;
    return FCS_OK;
}

int run(int bf16, int causal, const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes, int B, int H,
        int Hk, int Sq, int Sk, int D, const int64_t qs[4], const int64_t ks[4], float scale, int cls_n,
        int k_past, void *stream, uint32_t flags = 0)
{
    fcs::Plan p;
    fcs::Args a;
    const int rc = prepare(p, a, bf16, causal, q, k, out, out_f16, ws, ws_bytes, B, H, Hk, Sq, Sk, D, qs, ks, scale, cls_n, k_past,
                           flags, true);
    if (rc != FCS_OK) return rc;
    return fcs::launch_colsum(p, a, stream);
}

}  // namespace

extern "C" {

int fcs_abi_version(void) { return FCS_ABI_VERSION; }

const char *fcs_strerror(int code)
{
    switch (code) {
    case FCS_OK: return "ok";
    case FCS_E_NULL: return "a required pointer is NULL";
    case FCS_E_DIMS: return "invalid dimension (each of B,H,S,D must be >= 1, Hq a multiple of Hk, cls_n != 0, k_past >= 0, fewer than 2^31 workgroups)";
    case FCS_E_HEAD_DIM: return "unsupported head dim (a multiple of 8 from 8 to 256)";
    case FCS_E_STRIDE: return "unsupported layout (last stride must be 1; rows, heads and base 16-byte aligned)";
    case FCS_E_WORKSPACE: return "workspace smaller than fcs_workspace_bytes() or not 256-byte aligned";
    case FCS_E_DTYPE: return "unknown operand dtype (FCS_DTYPE_F16 or FCS_DTYPE_BF16)";
    case FCS_E_STATIC_LIMIT: return "the call needs more workspace than the static scratch holds (FCS_STATIC_SCRATCH_BYTES)";
    case FCS_E_SCALE: return "scale is not finite";
    case FCS_E_STRUCT: return "fcs_call_t.struct_bytes does not match this library's sizeof(fcs_call_t)";
    default: return code > 0 ? "HIP launch error (code is a hipError_t)" : "unknown error code";
    }
}

size_t fcs_workspace_bytes(int causal, int B, int H, int Sq, int Sk, int D, int cls_n)
{
    fcs::Plan p;
    const int k_past = (causal && Sk > Sq) ? Sk - Sq : 0;  // the layout does not depend on k_past
    if (!cached_plan(p, causal ? 1 : 0, B, H, Sq, Sk, D, cls_n < 0 ? -1 : cls_n, k_past)) return 0;
    return p.total;
}

int fcs_colsum_call(const fcs_call_t *c)
{
    if (!c) return FCS_E_NULL;
    if (c->struct_bytes != sizeof(fcs_call_t)) return FCS_E_STRUCT;
    if (c->dtype != FCS_DTYPE_F16 && c->dtype != FCS_DTYPE_BF16) return FCS_E_DTYPE;
    return run(c->dtype == FCS_DTYPE_BF16, c->causal ? 1 : 0, c->q, c->k, c->out, c->out_f16, c->ws, c->ws_bytes, c->B, c->Hq,
               c->Hk, c->Sq, c->Sk, c->D, c->q_strides, c->k_strides, c->scale, c->cls_n < 0 ? -1 : c->cls_n,
               c->causal ? c->k_past : 0, c->hip_stream, c->flags);
}

size_t fcs_plan_describe(const fcs_call_t *c, char *buf, size_t buf_bytes)
{
    if (buf && buf_bytes) buf[0] = 0;
    if (!c || c->struct_bytes != sizeof(fcs_call_t)) return 0;
    fcs::Plan p;
    fcs::Args a;
    const int rc = prepare(p, a, c->dtype == FCS_DTYPE_BF16, c->causal ? 1 : 0, c->q, c->k, c->out, c->out_f16, c->ws, c->ws_bytes,
                           c->B, c->Hq, c->Hk, c->Sq, c->Sk, c->D, c->q_strides, c->k_strides, c->scale,
                           c->cls_n < 0 ? -1 : c->cls_n, c->causal ? c->k_past : 0, c->flags, false);
    if (rc != FCS_OK) return 0;
    return fcs::describe_colsum(p, a, buf, buf_bytes);
}

int fcs_static_scratch_init(void)
{
    void *ws = nullptr;
    return (int)static_scratch(&ws);
}

int fcs_colsum_noncausal_f16(const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes, int B, int H,
                             int S, int D, const int64_t q_strides[4], const int64_t k_strides[4], float scale,
                             int cls_n, void *hip_stream)
{
    return run(0, 0, q, k, out, out_f16, ws, ws_bytes, B, H, H, S, S, D, q_strides, k_strides, scale, cls_n < 0 ? -1 : cls_n, 0,
               hip_stream);
}

int fcs_colsum_general(int dtype, int causal, const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes,
                       int B, int Hq, int Hk, int Sq, int Sk, int D, int cls_n, int k_past, const int64_t q_strides[4],
                       const int64_t k_strides[4], float scale, void *hip_stream)
{
    if (dtype != FCS_DTYPE_F16 && dtype != FCS_DTYPE_BF16) return FCS_E_DTYPE;
    return run(dtype == FCS_DTYPE_BF16, causal ? 1 : 0, q, k, out, out_f16, ws, ws_bytes, B, Hq, Hk, Sq, Sk, D, q_strides,
               k_strides, scale, cls_n < 0 ? -1 : cls_n, causal ? k_past : 0, hip_stream);
}

int fcs_colsum_noncausal_f16_static(const void *q, const void *k, float *out, void *out_f16, int B, int H, int S, int D,
                                    const int64_t q_strides[4], const int64_t k_strides[4], float scale, int cls_n,
                                    void *hip_stream)
{
    // size check first: it needs no GPU, like every other argument error
    fcs::Plan p;
    if (!cached_plan(p, 0, B, H, S, S, D, cls_n < 0 ? -1 : cls_n, 0)) return FCS_E_DIMS;
    if (p.total > (size_t)FCS_STATIC_SCRATCH_BYTES) return FCS_E_STATIC_LIMIT;
    if (!q || !k || !out || !q_strides || !k_strides) return FCS_E_NULL;
    void *ws = nullptr;
    const hipError_t e = static_scratch(&ws);
    if (e != hipSuccess) return (int)e;
    return run(0, 0, q, k, out, out_f16, ws, FCS_STATIC_SCRATCH_BYTES, B, H, H, S, S, D, q_strides, k_strides, scale,
               cls_n < 0 ? -1 : cls_n, 0, hip_stream);
}

int fcs_colsum_noncausal_bf16(const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes, int B, int H,
                              int S, int D, const int64_t q_strides[4], const int64_t k_strides[4], float scale,
                              int cls_n, void *hip_stream)
{
    return run(1, 0, q, k, out, out_f16, ws, ws_bytes, B, H, H, S, S, D, q_strides, k_strides, scale, cls_n < 0 ? -1 : cls_n, 0,
               hip_stream);
}

int fcs_colsum_causal_f16(const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes, int H, int Q_len,
                          int K_len, int D, int k_past, const int64_t q_strides[4], const int64_t k_strides[4],
                          float scale, void *hip_stream)
{
    return run(0, 1, q, k, out, out_f16, ws, ws_bytes, 1, H, H, Q_len, K_len, D, q_strides, k_strides, scale, -1, k_past,
               hip_stream);
}

int fcs_colsum_causal_bf16(const void *q, const void *k, float *out, void *out_f16, void *ws, size_t ws_bytes, int H, int Q_len,
                           int K_len, int D, int k_past, const int64_t q_strides[4], const int64_t k_strides[4],
                           float scale, void *hip_stream)
{
    return run(1, 1, q, k, out, out_f16, ws, ws_bytes, 1, H, H, Q_len, K_len, D, q_strides, k_strides, scale, -1, k_past,
               hip_stream);
}

}  // extern "C"
