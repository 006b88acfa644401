// Attention column means on gfx950 (MI355X): single-kernel path for non-causal calls with SHORT key
// sequences (S_k <= 288: nine 32-key tiles), head dims up to 64.  Token counts of vision encoders
// (197, 257) and short text live here.
//
// With so few keys ONE wave holds the whole score block of 32 query rows x S_k keys in registers
// (v_mfma_f32_32x32x16, up to nine accumulator tiles), so everything that the longer fused kernel
// (fcs_fused.hip) needs a workgroup for is wave-local here: the row sums are folded over the key lanes in
// registers, no wave waits for another inside a (head, row tile) item, and the waves of a workgroup
// only share their operands:
//   * K of a head (<= 36 KB) is fetched ONCE per workgroup with global_load_lds_dwordx4 into a ring of
//     head slots in LDS, one step ahead, by all eight waves together, and read by every wave that works
//     on that head (the longer kernel's eight waves each fetch their own copy when there is one key group);
//   * the 32 Q rows of an item travel the same way into a 4 KB slot of the wave's own, one item ahead, and are
//     pre-scaled in the operand registers (see PRE).
// A workgroup owns a group of heads of one batch entry.  Its items (head, 32-row tile) are dealt to the
// waves in turn, eight per STEP; one workgroup barrier per step lets the ring advance.  Every wave adds
// the columns of all its items into its own column sums; at the end the eight waves' sums are added in
// wave order and written as one partial slab per workgroup, which fcs_finalize_kernel adds over the
// head groups in index order: no atomics, fixed order.
//
// Per item (wave-local):
//   phase 1  for each key tile: MFMA -> e = 2^(c*s) -> in-lane partial row sums
//   reduce   row sums over the 32 key lanes in registers, w_i = 1 / L_i (0 for rows that are not averaged)
//   phase 3  col_acc[tile] += sum_r e[tile][r] * w[r]
// The exponent is taken WITHOUT max subtraction while that is exact in fp32: every row sum must land in
// [2^-80, 2^120) (below 2^28 on the pre-scaled operand); otherwise the wave redoes the item with the
// max-subtracted softmax, re-reading the head's keys from LDS.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>

#include "fcs_device.h"
#include "fcs_kernels.h"
#include "fcs_rowfold.h"

namespace fcs {

namespace {

constexpr float kSmallSumLo = 8.2718061e-25f;   // 2^-80
constexpr float kSmallSumHi = 1.3292280e+36f;   // 2^120
constexpr float kSmallSumHiPre = 268435456.f;   // 2^28: ceiling on the pre-scaled operand (bounds its score rounding error)

// source of the 16-byte pieces that lie past the tensor's head dim
__device__ unsigned int g_small_zero_piece[4];

__device__ __forceinline__ uint32_t lds_off(const void *p)
{
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}

}  // namespace

// PRE (fp16 only; chosen by the launcher when at least 2048 (head, row) pairs are averaged and
// |scale| <= 1/8): the Q rows are multiplied by c = scale * log2(e) in fp32 and rounded back to fp16 in
// the operand registers, so the scores leave the MFMAs in the exponent's unit and the per-score multiply
// disappears (-25 % VALU instructions).
template <int TPW, bool BF, bool PRE>
__global__ __launch_bounds__(512, 2) void fcs_small_kernel(const Args a)
{
    static_assert(!(PRE && BF), "the pre-scaled variant rounds Q*c to fp16; bf16 would be too coarse");
    static_assert(TPW >= 1 && TPW <= kSmallMaxTiles, "one to nine key tiles per wave");
    constexpr int NT = 4;                          // MFMA steps (and 16-byte pieces per lane) per operand tile, 64-wide heads
    constexpr int NSLOT = small_ring_heads(TPW);   // heads the ring holds
    constexpr int HEAD_BYTES = TPW * 4096;         // keys of one head: TPW tiles of 32 rows x 128 bytes
    constexpr int IPH = TPW * NT;                  // DMA instructions per head (1 KB = 8 key rows each)
    __shared__ __attribute__((aligned(16))) char ring[NSLOT * HEAD_BYTES];
    __shared__ __attribute__((aligned(16))) float wv[8 * 32];            // wave-private: the row weights of the current item
    __shared__ __attribute__((aligned(16))) float colred[8 * TPW * 32];  // the waves' column sums at the end

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b = (int)blockIdx.x % a.B, hg = (int)blockIdx.x / a.B;
    const int h_begin = hg * a.f_hpg, n_heads = min(a.H, h_begin + a.f_hpg) - h_begin;
    const int RT = a.f_nqblk;                      // 32-row tiles per head
    const int items = n_heads * RT, steps = (items + 7) >> 3;
    const int Sk = a.Sk;

    const char *q_batch = reinterpret_cast<const char *>(a.q + (int64_t)b * a.qs_b);
    const char *k_batch = reinterpret_cast<const char *>(a.k + (int64_t)b * a.ks_b);
    const int64_t q_head_b = a.qs_h * 2, k_head_b = a.ks_h * 2;
    const uint32_t q_row_b = (uint32_t)a.qs_s * 2u, k_row_b = (uint32_t)a.ks_s * 2u;
    const char *zero_piece = reinterpret_cast<const char *>(g_small_zero_piece);

    // ---- K of one head into its ring slot: DMA instruction j of IPH moves key rows [8j, 8j + 8), lane L the
    // 16-byte piece (L % 8) ^ swizzle(row) of row 8j + L / 8, which lands at position L % 8 of that row: the
    // tile sits row-major in LDS with the pieces of a row XOR-swizzled, so that the operand reads below (32
    // lanes, 128 bytes apart) stay off each other's banks.  Rows past the last key repeat it (their columns
    // count for nothing), pieces past the head dim come from a zero constant.  The eight waves share the
    // instructions: wave w moves the instructions w, w + 8, ... of EVERY head, so a lane's byte offsets from the
    // head's first key are the same for all heads and are formed once (kNoPiece marks a zero piece).
    // (The piece a lane fetches depends on its row in LDS only through (row / 2) % 8, which is the same for all of
    // a wave's instructions: rows 64 apart.)
    constexpr int JPW = (IPH + 7) / 8;  // instructions per wave and head, at most
    constexpr uint32_t kNoPiece = 0xffffffffu;
    auto fetch_heads = [&](int head_first, int head_end) {  // relative head numbers; wave-uniform
        if (head_first >= head_end) return;
        int l = lane;
        asm volatile("" : "+v"(l));  // the lane's offsets are formed here, not kept in registers through the items
        const int k_row0 = 8 * wave + (l >> 3);  // this lane's key row in the wave's first instruction
        const int k_piece = (l & 7) ^ ((k_row0 >> 1) & 7);
        const uint32_t k_piece_b = (k_piece * 8 < a.D) ? (uint32_t)(k_piece * 16) : kNoPiece;
        for (int hr = head_first; hr < head_end; ++hr) {
            const char *head = k_batch + (int64_t)kv_head(h_begin + hr, a.kv_group, a.kv_magic) * k_head_b;  // uniform
            char *slot = ring + (hr % NSLOT) * HEAD_BYTES + wave * 1024;
#pragma unroll
            for (int m = 0; m < JPW; ++m) {
                if (wave + 8 * m < IPH) {  // wave-uniform
                    const uint32_t off = (uint32_t)min(k_row0 + 64 * m, Sk - 1) * k_row_b + k_piece_b;
                    const char *src = (k_piece_b != kNoPiece) ? head + off : zero_piece;
                    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                                     (__attribute__((address_space(3))) void *)(slot + m * 8192), 16, 0, 0);
                }
            }
        }
    };

    // ---- the walk over items: this wave's item of the current step and the step's last item, as (head, row tile),
    // advanced by eight items per step without a division
    int it_h = 0, it_t = wave;        // item 8 * step + wave
    int last_h = 0, last_t = 7;       // item 8 * step + 7 (may lie past the last item)
    auto advance = [&](int &hh, int &tt, int by) {
        tt += by;
        while (tt >= RT) {
            tt -= RT;
            ++hh;
        }
    };
    advance(it_h, it_t, 0);
    advance(last_h, last_t, 0);

    // ---- Q rows of item (hr, tile) into this wave's own slot, in the layout of a key tile (four DMA instructions:
    // instruction j moves rows [8j, 8j + 8); a lane's piece is the same for j and j + 2).  Rows past the last query
    // row repeat it (they carry weight 0), pieces past the head dim are zeros.
    __shared__ __attribute__((aligned(16))) char qbuf[8 * 4096];
    auto fetch_q = [&](int hr, int tile) {  // wave-uniform
        int l = lane;
        asm volatile("" : "+v"(l));
        const int q_row0 = l >> 3;                            // this lane's row in instruction 0
        const int q_piece0 = (l & 7) ^ ((q_row0 >> 1) & 7);   // its piece in instructions 0 and 2; the others: ^ 4
        const char *head = q_batch + (int64_t)(h_begin + hr) * q_head_b;  // uniform
        char *slot = qbuf + wave * 4096;
#pragma unroll
        for (int jj = 0; jj < NT; ++jj) {
            const int piece = q_piece0 ^ ((jj & 1) * 4);
            const uint32_t off = (uint32_t)min(tile * 32 + 8 * jj + q_row0, a.Sq - 1) * q_row_b + (uint32_t)(piece * 16);
            const char *src = (piece * 8 < a.D) ? head + off : zero_piece;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                             (__attribute__((address_space(3))) void *)(slot + jj * 1024), 16, 0, 0);
        }
    };
    half8 qf[NT];
    // raw rows -> the operand the matrix pipe takes: pre-scaled (PRE, unless `exact`), the scale's sign on it
    auto shape_q = [&](const half8 (&raw)[NT], bool exact) {
#pragma unroll
        for (int tt = 0; tt < NT; ++tt) {
            half8 v = raw[tt];
            if (PRE && !exact) {
                const float cs = a.negate ? -a.c : a.c;
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = (_Float16)((float)v[e] * cs);
            } else if (a.negate) {
                v = flip_sign(v);
            }
            qf[tt] = v;
        }
    };

    // ---- operand read-back of a tile (lane (n, g): piece 2 tt + g of row n).  Inline assembly: the compiler
    // would make an ordinary LDS read wait for ALL outstanding DMA (vmcnt(0)), i.e. for the next step's keys.
    // `take_q0` is the lane's address for piece g of the wave's Q slot; pieces 2 tt + g lie at that address with
    // 32 tt XORed in (tiles start at multiples of 128 bytes, the swizzle permutes within a row's 128).  A key
    // tile's offset from the Q slot is the sum of a per-item value (the head's ring slot) and an immediate (the tile).
    auto take_q0_now = [&]() {
        int l = lane;
        asm volatile("" : "+v"(l));
        const int n_o = l & 31, g_o = l >> 5;
        return lds_off(qbuf) + (uint32_t)(wave * 4096 + n_o * 128 + ((g_o ^ ((n_o >> 1) & 7)) * 16));
    };
    const uint32_t ring_from_q = lds_off(ring) - lds_off(qbuf) - (uint32_t)(wave * 4096);  // wraps; only sums are used
    static_assert(sizeof(qbuf) % 128 == 0 && HEAD_BYTES % 128 == 0, "slots start at multiples of a row");
    uint32_t ta0 = 0, ta1 = 0, ta2 = 0, ta3 = 0;
    static_assert(NT == 4, "the operand reads below are written for four pieces");
    auto take_issue = [&](auto tile_c, half8 (&dst)[NT]) {
        constexpr int OFF = decltype(tile_c)::value * 4096;
        const uint32_t a0 = ta0, a1 = ta1, a2 = ta2, a3 = ta3;  // (locals: an asm operand does not capture)
        asm volatile("ds_read_b128 %0, %4 offset:%8\n\tds_read_b128 %1, %5 offset:%8\n\tds_read_b128 %2, %6 offset:%8\n\t"
                     "ds_read_b128 %3, %7 offset:%8"
                     : "=&v"(dst[0]), "=&v"(dst[1]), "=&v"(dst[2]), "=&v"(dst[3])
                     : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "n"(OFF)
                     : "memory");
    };
    auto take_wait = [&](half8 (&dst)[NT]) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(dst[0]), "+v"(dst[1]), "+v"(dst[2]), "+v"(dst[3])::"memory");
    };

    // a lane's key in tile t is 32 t + n; it counts while it is below Sk, i.e. for t <= tmax_lane
    const int tmax_lane = (Sk - 1 - n) >> 5;  // arithmetic shift: -1 when the lane has no key at all
    // the row whose total over the wave's keys fold_lanes_sum() leaves in this lane
    const int row_w = 16 * ((lane >> 4) & 1) + 8 * ((lane >> 3) & 1) + 4 * g + 2 * ((lane >> 2) & 1) + ((lane >> 1) & 1);
    const uint32_t wv_write = lds_off(wv) + (uint32_t)((wave * 32 + row_w) * 4);
    const uint32_t wv_read = lds_off(wv) + (uint32_t)((wave * 32 + 4 * g) * 4);
    // Hands every lane the sixteen per-row values of ITS accumulator rows (register i <-> row 8 (i / 4) + 4 g
    // + i % 4), given the value of row row_w in each lane: through the wave's 32 floats of LDS.  Inline
    // assembly for the same reason as the operand reads.
    auto spread_rows = [&](float mine, float (&out)[16]) {
        floatx4 r0, r1, r2, r3;
        asm volatile("ds_write_b32 %4, %5\n\ts_waitcnt lgkmcnt(0)\n\t"
                     "ds_read_b128 %0, %6\n\tds_read_b128 %1, %6 offset:32\n\tds_read_b128 %2, %6 offset:64\n\t"
                     "ds_read_b128 %3, %6 offset:96\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
                     : "v"(wv_write), "v"(mine), "v"(wv_read)
                     : "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            out[j] = r0[j];
            out[4 + j] = r1[j];
            out[8 + j] = r2[j];
            out[12 + j] = r3[j];
        }
    };

    float col_acc[TPW];
#pragma unroll
    for (int t = 0; t < TPW; ++t) col_acc[t] = 0.f;

    // ---- prologue: the heads of step 0 and this wave's first Q rows
    fetch_heads(0, min(n_heads - 1, last_h) + 1);
    if (wave < items) fetch_q(it_h, it_t);

    for (int step = 0; step < steps; ++step) {
        const int it = 8 * step + wave;
        const int hr = it_h, tile_r = it_t;  // this step's item
        advance(it_h, it_t, 8);
        // everything requested during the previous step has landed (this wave's share; the barrier extends
        // that to every wave's), and every wave is done with the previous step's heads
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        asm volatile("s_barrier" ::: "memory");
        // the next step's new heads take the slots of heads that no item of this step touches any more
        {
            const int from = min(n_heads - 1, last_h) + 1;
            advance(last_h, last_t, 8);
            if (step + 1 < steps) fetch_heads(from, min(n_heads - 1, last_h) + 1);
        }
        if (it >= items) continue;  // wave-uniform; an idle wave still takes its share of the fetches and the barriers

        const int row0 = tile_r * 32;  // first query row of the item
        half8 kf[2][NT];
        {
            // this item's Q rows out of the wave's slot, which then takes the next item's (waited for at the
            // top of the next step)
            const uint32_t take_q0 = take_q0_now();
            ta0 = take_q0;
            ta1 = take_q0 ^ 32u;
            ta2 = take_q0 ^ 64u;
            ta3 = take_q0 ^ 96u;
            half8 raw[NT];
            take_issue(std::integral_constant<int, 0>{}, raw);
            const uint32_t to_slot = ring_from_q + (uint32_t)((hr % NSLOT) * HEAD_BYTES);
            ta0 += to_slot;
            ta1 += to_slot;
            ta2 += to_slot;
            ta3 += to_slot;
            take_issue(std::integral_constant<int, 0>{}, kf[0]);
            take_wait(raw);
            if (it + 8 < items) fetch_q(it_h, it_t);
            shape_q(raw, false);
        }
        floatx16 acc[TPW];
        float rs[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) rs[i] = 0.f;

        // e = 2^(c*s) for tile t, in place, and its contribution to the row sums.  Only the last tile can reach past
        // the last key: a column there gets the bias -inf, so its exponential is 0; the bias rides on the scale multiply (one FMA).
        // Pre-scaled scores have no multiply to carry it: there the column's exponentials (finite: they
        // repeat the last key) enter the row sums with weight 0, and its column sum is never written.
        auto exp_tile = [&](auto t_c) {
            constexpr int t = decltype(t_c)::value;
            if constexpr (t < TPW - 1) {  // every key of these tiles exists (TPW = ceil(Sk / 32))
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float e = fast_exp2(PRE ? acc[t][i] : acc[t][i] * a.c);
                    acc[t][i] = e;
                    rs[i] += e;
                }
            } else {
                const bool counts = t <= tmax_lane;
                const float bias = counts ? 0.f : -INFINITY, one = counts ? 1.f : 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float e = fast_exp2(PRE ? acc[t][i] : fmaf(acc[t][i], a.c, bias));
                    acc[t][i] = e;
                    if (PRE) rs[i] = fmaf(e, one, rs[i]);
                    else rs[i] += e;
                }
            }
            // pinned here: otherwise the optimiser sinks every exponent below the last MFMA
            asm volatile("" : "+v"(rs[0]), "+v"(rs[1]), "+v"(rs[2]), "+v"(rs[3]), "+v"(rs[4]), "+v"(rs[5]), "+v"(rs[6]),
                         "+v"(rs[7]), "+v"(rs[8]), "+v"(rs[9]), "+v"(rs[10]), "+v"(rs[11]), "+v"(rs[12]), "+v"(rs[13]),
                         "+v"(rs[14]), "+v"(rs[15]));
        };

        // ---------------- phase 1: one step per key tile; the operands of tile t + 1 are read back under the
        // MFMAs of tile t, the exponent work of tile t - 1 runs under them too
        auto tile_step = [&](auto t_c) {
            constexpr int t = decltype(t_c)::value;
            take_wait(kf[t & 1]);
            if constexpr (t + 1 < TPW) take_issue(std::integral_constant<int, t + 1>{}, kf[(t + 1) & 1]);
            floatx16 c = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int tt = 0; tt < NT; ++tt) c = mfma16<BF>(qf[tt], kf[t & 1][tt], c);
            acc[t] = c;
            if constexpr (t > 0) exp_tile(std::integral_constant<int, t - 1>{});
        };
        tile_step(std::integral_constant<int, 0>{});
        if constexpr (TPW > 1) tile_step(std::integral_constant<int, 1>{});
        if constexpr (TPW > 2) tile_step(std::integral_constant<int, 2>{});
        if constexpr (TPW > 3) tile_step(std::integral_constant<int, 3>{});
        if constexpr (TPW > 4) tile_step(std::integral_constant<int, 4>{});
        if constexpr (TPW > 5) tile_step(std::integral_constant<int, 5>{});
        if constexpr (TPW > 6) tile_step(std::integral_constant<int, 6>{});
        if constexpr (TPW > 7) tile_step(std::integral_constant<int, 7>{});
        if constexpr (TPW > 8) tile_step(std::integral_constant<int, 8>{});
        exp_tile(std::integral_constant<int, TPW - 1>{});

        // ---------------- row sums over the key lanes (in registers); w = 1/L, 0 for rows that are not averaged
        const float L = fold_lanes_sum(rs, lane);
        const bool row_real = row0 + row_w < a.q_rows;
        // a row that is not averaged carries weight 0, but its exponentials must still be finite (inf * 0 is NaN)
        const bool bad = row_real ? !(L >= kSmallSumLo && L < (PRE ? kSmallSumHiPre : kSmallSumHi)) : !(L < kSmallSumHi);
        const bool slow = __builtin_amdgcn_ballot_w64(bad) != 0;
        if (!slow) {
            float w16[16];
            spread_rows(row_real ? __builtin_amdgcn_rcpf(L) : 0.f, w16);
            // ---------------- phase 3: column sums of e * w
#pragma unroll
            for (int i = 0; i < 16; ++i) {
#pragma unroll
                for (int t = 0; t < TPW; ++t) col_acc[t] = fmaf(acc[t][i], w16[i], col_acc[t]);
            }
        } else {
            // ------------ rare: max-subtracted softmax for this item, three passes over the head's keys in LDS with
            // one score tile in registers at a time; the raw operand (the scale's sign on it), the maximum
            // subtracted before the scale
            if (PRE) {  // the raw rows again, from memory (ordinary loads: the path is rare)
                int l = lane;
                asm volatile("" : "+v"(l));
                const char *src = q_batch + (int64_t)(h_begin + hr) * q_head_b + (size_t)min(row0 + (l & 31), a.Sq - 1) * q_row_b;
                half8 raw[NT];
#pragma unroll
                for (int tt = 0; tt < NT; ++tt) {
                    raw[tt] = kZero8;  // channels past the tensor's head dim are zeros
                    if (tt * 16 + (l >> 5) * 8 < a.D) raw[tt] = *reinterpret_cast<const half8 *>(src + tt * 32 + (l >> 5) * 16);
                }
                shape_q(raw, true);
            }
            auto score_tile = [&](int t) {  // runtime tile: the offset goes into the addresses
                half8 ks[NT];
                const uint32_t o = (uint32_t)(t * 4096);
                asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %5\n\tds_read_b128 %2, %6\n\tds_read_b128 %3, %7\n\t"
                             "s_waitcnt lgkmcnt(0)"
                             : "=&v"(ks[0]), "=&v"(ks[1]), "=&v"(ks[2]), "=&v"(ks[3])
                             : "v"(ta0 + o), "v"(ta1 + o), "v"(ta2 + o), "v"(ta3 + o)
                             : "memory");
                floatx16 c = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int tt = 0; tt < NT; ++tt) c = mfma16<BF>(qf[tt], ks[tt], c);
                return c;
            };
            float v16[16], rmax[16], w16[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) v16[i] = kNegBig;
#pragma unroll 1
            for (int t = 0; t < TPW; ++t) {
                const floatx16 c = score_tile(t);
                const bool real = t <= tmax_lane;
#pragma unroll
                for (int i = 0; i < 16; ++i) v16[i] = fmaxf(v16[i], real ? c[i] : kNegBig);
            }
            spread_rows(fold_lanes_max(v16, lane), rmax);
#pragma unroll
            for (int i = 0; i < 16; ++i) v16[i] = 0.f;
#pragma unroll 1
            for (int t = 0; t < TPW; ++t) {
                const floatx16 c = score_tile(t);
                const bool real = t <= tmax_lane;
#pragma unroll
                for (int i = 0; i < 16; ++i) v16[i] += real ? fast_exp2((c[i] - rmax[i]) * a.c) : 0.f;
            }
            const float Ls = fold_lanes_sum(v16, lane);
            spread_rows(row_real ? __builtin_amdgcn_rcpf(Ls) : 0.f, w16);
#pragma unroll 1
            for (int t = 0; t < TPW; ++t) {
                const floatx16 c = score_tile(t);
                const bool real = t <= tmax_lane;
                float sum = 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) sum = fmaf(real ? fast_exp2((c[i] - rmax[i]) * a.c) : 0.f, w16[i], sum);
#pragma unroll
                for (int u = 0; u < TPW; ++u)  // col_acc lives in registers: static index only
                    if (u == t) col_acc[u] += sum;
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---------------- the two half-waves hold different rows of the same keys; then the eight waves in wave order
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        const float both = col_acc[t] + __shfl_xor(col_acc[t], 32);
        if (g == 0) colred[(wave * TPW + t) * 32 + n] = both;
    }
    __syncthreads();
    float *dst = a.partial + ((int64_t)hg * a.B + b) * Sk;
    for (int key = tid; key < Sk; key += 512) {
        float v = colred[key];
#pragma unroll
        for (int w = 1; w < 8; ++w) v += colred[w * TPW * 32 + key];
        dst[key] = v;
    }
}

// Pre-scaled when the rounding of Q*c to fp16 cannot show in the means: the rule of the longer fused kernel,
// from 2048 averaged (head, row) pairs on (the effect on a mean falls with the square root of their number:
// measured 1.7e-4 relative at 4096 pairs, so about 2.4e-4 here; 12 heads x 197 rows are 2364).
static bool small_prescaled(const Plan &p, const Args &a)
{
    return !p.bf16 && (long)p.H * p.q_rows >= 2048 && fabsf(a.c) <= 0.1251f * 1.44269504f;
}

template <int TPW>
static void launch_small_tpw(const Plan &p, const Args &a, hipStream_t st)
{
    const dim3 grid((unsigned)((long)p.B * p.f_hg));
    if (p.bf16) hipLaunchKernelGGL((fcs_small_kernel<TPW, true, false>), grid, dim3(512), 0, st, a);
    else if (small_prescaled(p, a)) hipLaunchKernelGGL((fcs_small_kernel<TPW, false, true>), grid, dim3(512), 0, st, a);
    else hipLaunchKernelGGL((fcs_small_kernel<TPW, false, false>), grid, dim3(512), 0, st, a);
}

hipError_t launch_small(const Plan &p, const Args &a, hipStream_t st)
{
    switch (p.f_tpw) {
    case 1: launch_small_tpw<1>(p, a, st); break;
    case 2: launch_small_tpw<2>(p, a, st); break;
    case 3: launch_small_tpw<3>(p, a, st); break;
    case 4: launch_small_tpw<4>(p, a, st); break;
    case 5: launch_small_tpw<5>(p, a, st); break;
    case 6: launch_small_tpw<6>(p, a, st); break;
    case 7: launch_small_tpw<7>(p, a, st); break;
    case 8: launch_small_tpw<8>(p, a, st); break;
    case 9: launch_small_tpw<9>(p, a, st); break;
    default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_finalize(a, st);
}

size_t describe_small(const Plan &p, const Args &a, char *buf, size_t n)
{
    const int r = snprintf(buf, n, "fcs_small_kernel<%d,%s,%s> grid %ld, %d heads x %d row tiles per workgroup, %d slabs", p.f_tpw,
                           p.bf16 ? "true" : "false", (!p.bf16 && small_prescaled(p, a)) ? "true" : "false", (long)p.B * p.f_hg,
                           p.f_hpg, p.f_nqblk, p.n_partials);
    if (r < 0) return 0;
    const size_t len = (size_t)r;
    return len + describe_finalize(a, len < n ? buf + len : nullptr, len < n ? n - len : 0);
}

}  // namespace fcs
