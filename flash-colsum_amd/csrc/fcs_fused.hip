// Attention column means on gfx950 (MI355X): fused single-kernel path for non-causal
// calls whose whole key range fits in one workgroup's registers (32 <= S_k <= 2048, head dims up to 128:
// 64 channels natively, 128 as two 64-channel chunks, anything narrower on one of those two with zeros in Q).
//
// One workgroup = 8 waves.  The waves form a (query group) x (key group) grid; a wave
// computes the 32 x (32 * tiles) block of scores  S = Q_tile * K_tile^T  for its 32 query
// rows and its keys with v_mfma_f32_32x32x16_f16 and KEEPS it in registers (up to 8
// accumulator tiles = 128 VGPRs), so the scores are computed once and exponentiated
// once.  In this orientation a lane owns one key (column l % 32) and 16 query rows, so the
// column sums  sum_i e_ij / L_i  are in-lane FMAs; only the row sums L_i cross lanes and
// waves, once per (head, row block): lanes are folded in registers (DPP and lane-swap
// butterfly), the key-group waves through LDS and one workgroup barrier.
//
// Q and K never pass through staging registers: every wave streams its own operands
// with global_load_lds_dwordx4 into a private LDS ring, several tiles ahead of use, and
// reads them back as MFMA operands.  The DMA loads are waited for by hand with
// s_waitcnt vmcnt(n).
//
// Per (head, row block):
//   phase 1  for each tile: MFMA -> e = 2^(c*s) -> in-lane partial row sums
//   reduce   row sums over the 32 lanes x key-group waves, w_i = 1 / L_i
//   phase 3  col_acc[tile] += sum_r e[tile][r] * w[r]
// The exponent is taken WITHOUT max subtraction while that is exact in fp32: every row
// sum must land in [2^-80, 2^120).  If any row of the workgroup falls outside (or is not
// finite) the block redoes that (head, row block) with the usual max-subtracted softmax.
// A workgroup walks over its units (the heads of its head group times its row blocks, row blocks
// innermost) and writes one partial column-sum slab at the end;
// slabs have a single writer each and are added in index order by fcs_finalize_kernel.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include <stdio.h>

#include "fcs_device.h"
#include "fcs_kernels.h"
#include "fcs_rowfold.h"

namespace fcs {

namespace {

constexpr float kSumLo = 8.2718061e-25f;  // 2^-80
constexpr float kSumHi = 1.3292280e+36f;  // 2^120
constexpr float kSumHiPre = 268435456.f;  // 2^28: ceiling of the pre-scaled variant (bounds its score rounding error)

// source of the 16-byte pieces that lie past the tensor's head dim (kernels compiled for a wider head); 4 KB, so
// that a DMA instruction's immediate offset (up to 3 KB) stays inside
__device__ __attribute__((aligned(16))) unsigned int g_fused_zeros[1024];

#define FCS_GLDS16(gptr, lptr)                                                                \
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gptr), \
                                     (__attribute__((address_space(3))) void *)(lptr), 16, 0, 0)
// same, with an immediate byte offset that the hardware adds to BOTH the global and the LDS address
#define FCS_GLDS16_OFF(gptr, lptr, OFF)                                                       \
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gptr), \
                                     (__attribute__((address_space(3))) void *)(lptr), 16, OFF, 0)
#define FCS_WAIT_VM(N) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory")
// Hides a value's origin from the optimiser.  Used inside the walk over heads so that
// per-tile addresses are formed where they are used instead of being precomputed for the
// whole walk and held in (or spilled from) dozens of registers.
#define FCS_OPAQUE_V(x) asm volatile("" : "+v"(x))

// LDS scratch of one workgroup for the row reductions
struct RowRed {
    float *part;   // [2][256]: per-wave row partials, double-buffered by reduction parity
    float *wv_w;   // wave-private [32]: the reduced (and post-processed) value of each row
    int parity;
};

// Reduces v[16] (v[i] belongs to row acc_row(i, g) of the wave's 32 rows) over the 32 lanes of
// each half-wave (in registers: fold_lanes_sum / fold_lanes_max) and over
// the key-group waves of the same query group: sum, or max if MAX.
// `post(row_in_block, total)` maps the total to what is left in rr.wv_w[row] for the lanes to
// read back.  Returns (sum only) whether any row total of the WORKGROUP is outside
// [2^-80, 2^120) or not finite; the answer is the same in every wave.  One barrier.
template <bool MAX, typename Post>
__device__ __forceinline__ bool reduce_rows(const float (&v)[16], RowRed &rr, int kg_n, int qg, int kg, int lane, Post post,
                                            const float sum_hi = kSumHi)
{
    const int g = lane >> 5;
    const int row = lane >> 1, half = lane & 1;  // after the barrier lane L works on row L / 2
    // the row whose total over this wave's keys the lane holds before it
    const int row_w = 16 * ((lane >> 4) & 1) + 8 * ((lane >> 3) & 1) + 4 * g + 2 * ((lane >> 2) & 1) + ((lane >> 1) & 1);
    const float s = MAX ? fold_lanes_max(v, lane) : fold_lanes_sum(v, lane);
    // waves: one partial per (row, key group), dense so that 256 floats cover the workgroup
    float *part = rr.part + (rr.parity & 1) * 256;
    rr.parity ^= 1;
    const int pbase = (qg * 32 + row) * kg_n;
    if (half == 0) part[(qg * 32 + row_w) * kg_n + kg] = s;
    __syncthreads();
    float tot;
    bool out_of_range = false;
    // every wave looks at all 256 partials of the workgroup: lane L at floats [4L, 4L + 4)
    const floatx4 f = reinterpret_cast<const floatx4 *>(part)[lane];
    if (kg_n == 8) {
        // those four are key groups 4*half .. 4*half + 3 of this lane's own row: its neighbour holds the rest
        const float own = MAX ? fmaxf(fmaxf(f[0], f[1]), fmaxf(f[2], f[3])) : (f[0] + f[1]) + (f[2] + f[3]);
        const float other = dpp_get<kDppXor1>(own);
        tot = MAX ? fmaxf(own, other) : own + other;
    } else {
        tot = part[pbase];
        if (kg_n > 1) tot = MAX ? fmaxf(tot, part[pbase + 1]) : tot + part[pbase + 1];
        if (kg_n > 2) {
            const float t2 = part[pbase + 2], t3 = part[pbase + 3];
            tot = MAX ? fmaxf(tot, fmaxf(t2, t3)) : tot + (t2 + t3);
        }
    }
    if (!MAX) {
        const bool hi = !(f[0] < sum_hi) || !(f[1] < sum_hi) || !(f[2] < sum_hi) || !(f[3] < sum_hi);
        const float m01 = fmaxf(f[0], f[1]), m23 = fmaxf(f[2], f[3]);
        float lowest;  // smallest per-row maximum over key groups among the rows this lane sees
        if (kg_n >= 4) {
            lowest = fmaxf(m01, m23);
            if (kg_n == 8) lowest = fmaxf(lowest, dpp_get<kDppXor1>(lowest));
        } else if (kg_n == 2) {
            lowest = fminf(m01, m23);
        } else {
            lowest = fminf(fminf(f[0], f[1]), fminf(f[2], f[3]));
        }
        out_of_range = __builtin_amdgcn_ballot_w64(hi || !(lowest >= kSumLo)) != 0;
    }
    const float res = post(qg * 32 + row, tot);
    if (half == 0) rr.wv_w[row] = res;
    __builtin_amdgcn_wave_barrier();
    return out_of_range;
}

// the four values of rows 8*i4 + 4*g + {0..3} left by reduce_rows
__device__ __forceinline__ floatx4 row_values(const RowRed &rr, int i4, int g)
{
    return *reinterpret_cast<const floatx4 *>(rr.wv_w + 8 * i4 + 4 * g);
}

}  // namespace

// RAGGED = false: S_k is exactly (key groups) x TPW x 32, S_q a multiple of the block's rows and
//                 the rows of Q and K are dense (row stride == D): every operand tile is whole,
//                 no padding keys anywhere, and tile addresses need no per-lane arithmetic.
// RAGGED = true : anything else (any 32 <= S_k <= 2048, any S_q, any 16-byte aligned row pitch).  Key
//                 tiles still need no per-lane arithmetic and no branch: a tile that would reach
//                 past the last key is moved back to end there, and the columns that then repeat
//                 the tile before it are given no weight.  Q rows are clamped per lane, once per unit.
// QS (only with PRE): true = the shared Q tile is pre-scaled as described next; false = it is shared
//                 as it is (any operand type, any scale, any number of averaged rows; the sign of a
//                 negative scale is applied to it) and every score is still multiplied by c: the
//                 variant exists for the key-only ring, see KEEP below.
// PRE = 8 or 4 (0 = off; only with that many key groups, i.e. 1 or 2 query
//                 groups): each query group's Q tile is multiplied by
//                 c = scale * log2(e) in fp32 ONCE per head, rounded back to fp16 and shared by the
//                 eight waves through LDS, so the scores leave the MFMAs already in the exponent's
//                 unit and the per-score multiply disappears.  The extra fp16 rounding of Q perturbs
//                 each score by ~2^-12 relative; the launcher only picks this variant when at least
//                 4096 (head, row) pairs are averaged per output, where the effect on the means is
//                 below 1e-4 relative (measured 6.5e-5 at B8 H16 S2048).
// NARROW (only on the ragged private-ring variant): the tensor's head dim is smaller than the kernel's D (any
//                 multiple of 8): the operand pieces past it are fetched from a zero constant.
template <int D, int TPW, bool RAGGED, int PRE, bool BF, bool QS = true, bool NARROW = false>
__global__ __launch_bounds__(512, 2) void fcs_fused_kernel(const Args a)
{
    static_assert(!NARROW || (RAGGED && PRE == 0), "narrower heads run on the ragged private-ring variant");
    static_assert(D == 64 || (D == 128 && PRE == 0 && RAGGED), "64-wide heads, or 128-wide ones on the private-ring ragged variant");
    static_assert(!(PRE && QS && BF), "the pre-scaled variant rounds Q*c to fp16; bf16 would be too coarse");
    constexpr bool PRESCALED = PRE && QS;  // scores leave the MFMAs in the exponent's unit
    // A 128-wide head is handled as DC = 2 chunks of 64 channels: an operand tile travels as two half tiles
    // (32 rows x 64 channels, 4 KB, its own ring item each), and the MFMA chain of a score tile runs over the
    // first chunk's four steps, then the second chunk's, into the same accumulators.
    constexpr int DC = D / 64;
    constexpr int NT = 4;                  // MFMA steps (and 16-byte pieces per lane) per (half) tile
    // KEEP (shared-Q variants with five to eight key tiles per wave): the Q item of those variants is
    // a plain load that needs no ring slot, so the ring holds key tiles only, tile k of every unit in
    // slot k % NS.  The row blocks of a head, which a workgroup walks one after the other, use the
    // same key tiles: a unit leaves its last NS key tiles in the ring and the next unit of the same
    // key head starts with those, walking the tiles in another order, and fetches TPW - NS key tiles
    // instead of TPW; only the first unit of a key head fetches all of them.  Two orders alternate:
    //   * eight or six tiles (NS = TPW / 2): 0 .. TPW-1 and NS .. TPW-1, 0 .. NS-1; step t then
    //     always uses slot t % NS, a compile-time value;
    //   * otherwise (NS = 4, or 3 with two key groups): 0 .. TPW-1 and TPW-1 .. 0; the slot of a step depends on
    //     the order and is added to the read-back addresses at run time.
    // Each order has its own column sums; they are added at the end.
    // (With two key groups there are four query groups: their Q tiles take 32 KB and leave room for
    // three slots per wave, so eight tiles walk ascending / descending too.)
    constexpr bool KEEP_ROT = PRE && (TPW == 6 || (TPW == 8 && PRE != 2));
    constexpr bool KEEP_REV = PRE && !KEEP_ROT;
    constexpr bool KEEP = KEEP_ROT || KEEP_REV;
    // (two chunks: a unit starts by taking three items at once, both Q chunks and the first key half tile, so the
    // ring holds four, which leaves the fourth in flight)
    constexpr int NS = KEEP_ROT ? TPW / 2 : KEEP_REV ? (PRE == 2 ? 3 : 4) : (DC == 2 ? 4 : 3);  // ring slots per wave
    constexpr int QV = (PRE == 2) ? 2 : 1;  // load instructions of a wave's share of the raw Q rows
    static_assert(!PRE || (TPW >= 5 && TPW <= 8), "the shared-Q variants are written for five to eight key tiles per wave");
    constexpr int ITEMS = DC * (TPW + 1);  // per (head, row block): the Q tile, then TPW key tiles (chunk by chunk)
    constexpr int SLOT_BYTES = NT * 1024;  // one item: NT pieces x 64 lanes x 16 bytes
    constexpr bool STATIC_SLOTS = KEEP_ROT || (!KEEP_REV && ITEMS % NS == 0);  // then an item's slot is a compile-time value
    __shared__ __attribute__((aligned(16))) char ring[8 * NS * SLOT_BYTES];
    __shared__ __attribute__((aligned(16))) float part[2 * 256];
    __shared__ __attribute__((aligned(16))) float wv[8 * 32];
    constexpr int PQG = PRE ? 8 / PRE : 1;  // query groups of the pre-scaled variant
    __shared__ __attribute__((aligned(16))) char qshare[PRE ? 2 * PQG * 4096 : 16];  // pre-scaled Q tiles, double-buffered

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: what derives from it stays in SGPRs
    const int kg_n = PRE ? PRE : a.f_kg, qg_n = 8 / kg_n;  // a constant folds the reduction's branches away
    const int qg = wave / kg_n, kg = wave - qg * kg_n;
    // The row blocks of one (head group, batch entry) read the same K: they run on one XCD, close
    // together in time.
    int hgi, b, qwg;
    {
        int bx, by, bz;
        xcd_contiguous_block(bx, by, bz);
        qwg = bx % a.f_nwgq;
        b = bx / a.f_nwgq;
        hgi = by;
    }
    // A workgroup walks over units = (head, row block): the heads of its head group, and for each of
    // them its f_rbpw adjacent row blocks (row blocks innermost: the head's keys are fetched into the
    // L2 once and re-read from there; the workgroups of an XCD walk in step, so they read the same
    // head's keys at the same time).  Every unit adds into the same column sums.
    const int h_begin = hgi * a.f_hpg, h_end = min(a.H, h_begin + a.f_hpg);
    const int n_heads = h_end - h_begin;
    const int rb_first = qwg * a.f_rbpw, rb_n = min(a.f_rbpw, a.f_nqblk - rb_first);
    const int n_units = rb_n * n_heads;
    const int kbase = kg * TPW * 32;        // first key of this wave
    // Ragged kernel: key tile t of this wave nominally holds keys [kbase + 32 t, kbase + 32 t + 32).
    // A tile that would reach past the last key is moved back so that it ends there (every row it
    // fetches exists; S_k >= 32 on this path): MFMA column n of tile t is key tile_first(t) + n, and
    // the columns that repeat keys of the tile before it, n < kbase + 32 t + 32 - S_k, count for
    // nothing.  For a lane that is t > tmax_lane.  No branch and no per-lane address arithmetic
    // depends on where the keys end.
    auto tile_first = [&](int t) { return RAGGED ? min(kbase + t * 32, a.Sk - 32) : kbase + t * 32; };
    int tmax_lane = RAGGED ? (n + a.Sk - 32 - kbase) >> 5 : TPW;  // arithmetic shift: floor, also when negative

    RowRed rr;
    rr.part = part;
    rr.wv_w = wv + wave * 32;
    rr.parity = 0;

    // Operand tiles are 32 rows x 64 halves (128 B per row).  One DMA instruction moves 8
    // whole rows (1 KB, 8 full cache lines): lane L brings 16-byte piece L % 8 of row L / 8,
    // and the 64 pieces land in the ring in lane order, i.e. the tile sits row-major in
    // LDS.  To keep the later operand reads (32 lanes, 128 B apart) off each other's banks
    // the pieces of a row are stored XOR-swizzled: position p of row r holds piece
    // p ^ ((r >> 1) & 7).  The swizzle only depends on the parity of the instruction index.
    // Lane L's part of one DMA instruction: its row within the instruction's 8 rows, and the byte
    // offset in that row of the piece it fetches (instructions of even / odd index differ).
    auto dma_row = [](int l) { return l >> 3; };
    auto dma_piece_b = [](int l, int par) { return (uint32_t)(((l & 7) ^ ((par * 4 + (l >> 4)) & 7)) * 16); };
    // row pitch in bytes; a compile-time constant in the non-ragged kernel (rows are dense there)
    const uint32_t q_row_b = RAGGED ? (uint32_t)a.qs_s * 2u : (uint32_t)(D * 2), k_row_b = RAGGED ? (uint32_t)a.ks_s * 2u : (uint32_t)(D * 2);
    // Lane offsets from a tile's first row to this lane's piece.  Whole-tile kernel: rows are dense,
    // so instruction tt reads exactly 1 KB behind instruction tt - 2 and the offsets of instructions
    // 0 and 1 serve all four.  Ragged kernel (key tiles): rows have any pitch, so each instruction has
    // its own offset; it is stored less tt KB, because the instruction's immediate offset (which the
    // hardware adds to the LDS address AND the global address) supplies tt KB again.  (Never negative
    // where it is used: heads of 64 channels or more, whose rows are at least 128 bytes; narrower heads form
    // their offsets at the fetch.)
    auto ragged_voff = [&](int l, uint32_t row_b, int tt) {
        return (uint32_t)(dma_row(l) + 8 * tt) * row_b + dma_piece_b(l, tt & 1) - (uint32_t)(tt * 1024);
    };
    constexpr int NVOFF = RAGGED ? NT : 2;
    uint32_t q_voff[2] = {dma_row(lane) * q_row_b + dma_piece_b(lane, 0), dma_row(lane) * q_row_b + dma_piece_b(lane, 1)};
    uint32_t k_voff[NVOFF];
#pragma unroll
    for (int i = 0; i < NVOFF; ++i) k_voff[i] = RAGGED ? ragged_voff(lane, k_row_b, i) : dma_row(lane) * k_row_b + dma_piece_b(lane, i);
    // NARROW: the lane offsets of a key tile's last chunk, instruction by instruction (no immediate-offset trick:
    // rows may be shorter than 128 bytes).  A piece past the head dim is replaced by the chunk's first piece of the
    // same row: the Q operand holds zeros in those channels (fetch_ragged_q), so whatever finite values stand in
    // for the key's add nothing to a score.
    uint32_t k_voff_n[NARROW ? NT : 1];
#pragma unroll
    for (int i = 0; i < (NARROW ? NT : 1); ++i) {
        const uint32_t piece_b = dma_piece_b(lane, i & 1);
        const bool real = (int)((DC - 1) * 64 + (piece_b >> 1)) < a.D;
        k_voff_n[i] = (uint32_t)(dma_row(lane) + 8 * i) * k_row_b + (real ? piece_b : 0u);
    }
    // start of this batch entry's Q / K (head 0, row 0), and the same advanced to this wave's first
    // row.  Only the whole-tile kernel addresses through the latter: there every row it names
    // exists.  The ragged kernel works from ABSOLUTE row numbers instead (Q rows clamped to the last
    // one, key tiles moved back to end at the last key), because a wave's rows (and whole tiles of
    // them) may lie past the end of the tensor.
    const char *q_batch = reinterpret_cast<const char *>(a.q + (int64_t)b * a.qs_b);
    const char *k_batch = reinterpret_cast<const char *>(a.k + (int64_t)b * a.ks_b);
    const char *k_b = k_batch + (int64_t)min(kbase, a.Sk - 1) * k_row_b;
    const int64_t q_head_b = a.qs_h * 2, k_head_b = a.ks_h * 2;
    char *my_ring = ring + wave * (NS * SLOT_BYTES);

    // DMA instruction `tt` (of NT) of a whole tile with dense rows, first row at `tile` (wave-uniform):
    // its rows [8*tt, 8*tt + 8) go to ring slot `slot`.  Instruction tt reads 1 KB further in memory
    // and writes 1 KB further in the slot, which is exactly what the immediate offset does; base
    // pointer, lane offset and LDS base are shared by the four pieces.
    auto fetch_piece_at = [&](const char *tile, uint32_t vo, int slot, int tt) {
        char *dst = my_ring + slot * SLOT_BYTES;
        static_assert(NT == 4, "offsets below");
        const char *src = tile + vo;
        if (tt == 0) FCS_GLDS16_OFF(src, dst, 0);
        else if (tt == 1) FCS_GLDS16_OFF(src, dst, 1024);
        else if (tt == 2) FCS_GLDS16_OFF(src, dst, 2048);
        else FCS_GLDS16_OFF(src, dst, 3072);
    };
    auto fetch_piece = [&](const char *tile, auto &voff, int slot, int tt) {
        FCS_OPAQUE_V(voff[tt & 1]);
        fetch_piece_at(tile, voff[tt & 1], slot, tt);
    };
    // Ragged kernel, the Q tile at rows [first_row, first_row + 32) of a slice of `n_rows` rows of any
    // pitch (once per unit): each lane clamps its row to the last real one (repeated rows carry
    // weight 0 in the column sums).  No branch: a taken branch costs a wave far more than these few
    // address instructions.
    auto fetch_ragged_q = [&](const char *slice, uint32_t row_b, int first_row, int n_rows, int slot, int chunk) {
        char *dst = my_ring + slot * SLOT_BYTES;
        int l = lane;
        FCS_OPAQUE_V(l);
#pragma unroll
        for (int tt = 0; tt < NT; ++tt) {
            const uint32_t row = (uint32_t)min(first_row + tt * 8 + dma_row(l), n_rows - 1);
            const uint32_t col_b = dma_piece_b(l, tt & 1) + (uint32_t)(chunk * 128);
            const char *src = slice + ((size_t)row * row_b + col_b);
            if (NARROW && (int)(col_b >> 1) >= a.D) src = reinterpret_cast<const char *>(g_fused_zeros);  // channels past the head dim
            FCS_GLDS16(src, dst + tt * 1024);
        }
    };
    // Read a ring slot back as an MFMA operand: lane (n, g) takes, for step tt, piece 2*tt + g of
    // row n.  Issued from inline assembly: the compiler would otherwise make every LDS read wait
    // for ALL outstanding DMA fetches (vmcnt(0)), which would undo the look-ahead.  The reads
    // are only ISSUED here; take_wait() must sit between them and the first use of `dst`.
    uint32_t take_addr[NT];
#pragma unroll
    for (int tt = 0; tt < NT; ++tt)
        take_addr[tt] = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)my_ring +
                        (uint32_t)(n * 128 + (((2 * tt + g) ^ ((n >> 1) & 7)) * 16));
    static_assert(NT == 4 && SLOT_BYTES == 4096, "the operand reads below are written for four 1 KB pieces");
#define FCS_TAKE_ASM(OFF)                                                                                  \
    asm volatile("ds_read_b128 %0, %4 offset:" #OFF "\n\tds_read_b128 %1, %5 offset:" #OFF                 \
                 "\n\tds_read_b128 %2, %6 offset:" #OFF "\n\tds_read_b128 %3, %7 offset:" #OFF             \
                 : "=&v"(dst[0]), "=&v"(dst[1]), "=&v"(dst[2]), "=&v"(dst[3])                              \
                 : "v"(ta0), "v"(ta1), "v"(ta2), "v"(ta3)                                                   \
                 : "memory")
    auto take_issue = [&](int slot, half8 (&dst)[NT]) {
        if (STATIC_SLOTS) {  // slot is a compile-time value at every call site: it folds into the offset field
            const uint32_t ta0 = take_addr[0], ta1 = take_addr[1], ta2 = take_addr[2], ta3 = take_addr[3];
            if (slot == 0) FCS_TAKE_ASM(0);
            else if (slot == 1) FCS_TAKE_ASM(4096);
            else if (slot == 2) FCS_TAKE_ASM(8192);
            else FCS_TAKE_ASM(12288);
        } else {
            const uint32_t off = (uint32_t)(slot * SLOT_BYTES);
            const uint32_t ta0 = take_addr[0] + off, ta1 = take_addr[1] + off, ta2 = take_addr[2] + off, ta3 = take_addr[3] + off;
            FCS_TAKE_ASM(0);
        }
    };
#undef FCS_TAKE_ASM
    // all LDS reads issued so far have landed; ties the operand registers so that no use moves above
    auto take_wait = [&](half8 (&dst)[NT]) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(dst[0]), "+v"(dst[1]), "+v"(dst[2]), "+v"(dst[3])::"memory");
    };

    float col_acc[TPW];
    float col_rot[KEEP ? TPW : 1];  // KEEP: sums of the units that ran in the second order: col_rot[t] belongs to tile tile_of(t)
#pragma unroll
    for (int t = 0; t < TPW; ++t) col_acc[t] = 0.f;
#pragma unroll
    for (int t = 0; t < (KEEP ? TPW : 1); ++t) col_rot[t] = 0.f;
    int rot = 0;  // KEEP: 1 while the current unit runs in the second order
    // KEEP: the key tile of step t (compile-time) of the current unit, and its ring slot
    auto tile_of = [&](int t) { return !rot ? t : KEEP_ROT ? (t + NS) % TPW : TPW - 1 - t; };
    auto slot_of_step = [&](int t) { return KEEP_ROT ? t % NS : tile_of(t) % NS; };

    // The walk.  Every head contributes ITEMS = DC * (1 + TPW) operand (half) tiles ("items"): its Q tile, then
    // the wave's key tiles, chunk by chunk.  Item number p (counted over the whole walk) lives in ring slot p % NS.
    //   * Items are read back into registers ONE STEP BEFORE the MFMAs that use them, so the LDS
    //     latency is covered by the exponent work of the step in between.
    //   * As soon as the read-back of item p has landed its slot is free, and item p + NS is
    //     fetched into it; at most NS items (4 * NS DMA instructions) are in flight.
    //   * Past the last head the fetches repeat it, so that the number of outstanding DMA
    //     instructions at every wait is a compile-time constant.
    // PRE: the Q item of a head is not a tile in the ring but this wave's 32 / PRE rows of its query
    // group's raw tile (512 B or 1 KB), one ordinary 8- or 16-byte load per lane; the wave scales
    // them and publishes them in `qshare`.  KEEP: that item then takes no slot number either; key
    // tile k of every unit lives in slot k % NS, a unit requests the second half of its tile order
    // while it reads back the first, and the next unit's Q rows at step TPW - 2.
    // raw Q rows of the pre-scaled variant: written by an asynchronous load and read after a hand-placed
    // wait, so the variable the load names must be the one the wait names (no copies in between)
    typedef uint32_t qraw_t __attribute__((ext_vector_type(PRE == 8 ? 2 : 4)));
    qraw_t qraw = {}, qraw_hi = {};  // qraw_hi: the second 16 bytes of a lane (two key groups: 32 bytes per lane)
    auto item_vm = [&](int j_ahead) { return (PRE && (j_ahead % ITEMS) == 0) ? 1 : NT; };  // VMEM instructions of an item
    // What the fetches need to know of the current unit and of the units the look-ahead reaches,
    // refreshed once per unit instead of at every fetch: the head's Q slice, the wave's first query
    // row (unclamped; a wave whose rows all lie past the tensor re-reads the last row, its rows carry
    // weight 0), the wave's Q tile, and the byte offset of the key head (grouped key heads: head /
    // kv_group).  Past the last unit the entries repeat it.
    constexpr int HEADS_AHEAD = (ITEMS + NS - 1) / ITEMS;  // the look-ahead reaches this many units past the current one
    const char *u_qhead[HEADS_AHEAD + 1];
    const char *u_qtile[HEADS_AHEAD + 1];
    int u_qfirst[HEADS_AHEAD + 1];
    int64_t k_off[HEADS_AHEAD + 1];
    int cur_rb = 0, cur_hr = 0;  // row block (relative) and head (relative) of the current unit
    auto set_units = [&]() {
        int r = cur_rb, hr = cur_hr;
#pragma unroll
        for (int i = 0; i <= HEADS_AHEAD; ++i) {
            const int hh = h_begin + hr;
            const int first = ((rb_first + r) * qg_n + qg) * 32;
            u_qfirst[i] = first;
            u_qhead[i] = q_batch + (int64_t)hh * q_head_b;
            u_qtile[i] = u_qhead[i] + (int64_t)min(first, a.Sq - 1) * q_row_b;
            k_off[i] = (int64_t)kv_head(hh, a.kv_group, a.kv_magic) * k_head_b;
            if (r != rb_n - 1 || hr != n_heads - 1) {
                if (++r == rb_n) {
                    r = 0;
                    ++hr;
                }
            }
        }
    };
    set_units();
    auto fetch_pos_piece = [&](int j_ahead /* item index counted from the Q tile of the current unit, compile-time */,
                               int slot, int tt) {
        const int ua = j_ahead / ITEMS;
        const int j = j_ahead % ITEMS;
        if (j == 0 && PRE) {
            if (tt == 0) {
                // whole-tile kernel: the wave's rows are one contiguous run; ragged kernel: row by row,
                // clamped to the last real row (rows past the end carry weight 0)
                const char *src;
                if (RAGGED) {
                    const int row_in_tile = (PRE == 8) ? kg * 4 + (lane >> 4) : (PRE == 4) ? kg * 8 + (lane >> 3) : kg * 16 + (lane >> 2);
                    const int in_row_b = (PRE == 8) ? (lane & 15) * 8 : (PRE == 4) ? (lane & 7) * 16 : (lane & 3) * 32;
                    src = u_qhead[ua] + (size_t)min(u_qfirst[ua] + row_in_tile, a.Sq - 1) * q_row_b + in_row_b;
                } else {
                    src = u_qtile[ua] + ((PRE == 8) ? kg * 512 + lane * 8 : (PRE == 4) ? kg * 1024 + lane * 16 : kg * 2048 + lane * 32);
                }
                // Issued from inline assembly, so that the compiler does not count it among the loads
                // it waits for itself: it cannot tell how many DMA fetches were issued behind this
                // load and would drain all of them (vmcnt(0)) before the first use.  q_publish waits
                // for exactly this load.
                if (PRE == 8) asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(qraw) : "v"(src) : "memory");
                else asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(qraw) : "v"(src) : "memory");
                if (PRE == 2) asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(qraw_hi) : "v"(src) : "memory");
            }
        } else if (j == 0)
            fetch_piece(u_qtile[ua], q_voff, slot, tt);
        else
            fetch_piece(k_b + k_off[ua] + (size_t)((uint32_t)((j - 1) * 32) * k_row_b), k_voff, slot, tt);
    };
    auto fetch_pos = [&](int j_ahead, int slot) {
        if (RAGGED) {
            const int ua = j_ahead / ITEMS;
            const int j = j_ahead % ITEMS;
            if (j == 0 && PRE) fetch_pos_piece(j_ahead, slot, 0);  // the Q item of the pre-scaled variant is a plain load, not a tile
            else if (j < DC) fetch_ragged_q(u_qhead[ua], q_row_b, u_qfirst[ua], a.Sq, slot, j);
            else {
                // key tile (j - DC) / DC, chunk (j - DC) % DC
                const int chunk = (j - DC) % DC;
                const char *tile = k_batch + k_off[ua] + (size_t)tile_first((j - DC) / DC) * k_row_b + chunk * 128;
                if (NARROW && chunk == DC - 1) {
                    char *dst = my_ring + slot * SLOT_BYTES;
#pragma unroll
                    for (int tt = 0; tt < NT; ++tt) {
                        FCS_OPAQUE_V(k_voff_n[tt % (NARROW ? NT : 1)]);
                        FCS_GLDS16(tile + k_voff_n[tt % (NARROW ? NT : 1)], dst + tt * 1024);
                    }
                } else {
#pragma unroll
                    for (int tt = 0; tt < NT; ++tt) {
                        FCS_OPAQUE_V(k_voff[tt % NVOFF]);
                        fetch_piece_at(tile, k_voff[tt % NVOFF], slot, tt);
                    }
                }
            }
        } else {
#pragma unroll
            for (int tt = 0; tt < NT; ++tt) fetch_pos_piece(j_ahead, slot, tt);
        }
    };
    int sq = 0;  // ring slot of the current head's Q tile (only used when the slots are not static)
    auto slot_of = [&](int j) {  // slot of item j of the current head, j compile-time, j < ITEMS + 3
        if (STATIC_SLOTS) return j % NS;
        int s_ = sq + (j % NS);
        return s_ >= NS ? s_ - NS : s_;
    };

    // PRE: scale this wave's raw rows by c (sign included) in fp32, round to fp16 and store them at
    // their swizzled place in the query group's tile of qshare[buf]; a workgroup barrier must
    // follow before they are read
    auto q_publish = [&](int buf, auto behind_c) {
        // the raw rows have landed once at most the DMA instructions requested behind them are
        // outstanding (a compile-time count)
        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(qraw), "+v"(qraw_hi) : "n"(decltype(behind_c)::value) : "memory");
        // 16 bytes of raw rows -> 16 bytes to publish: scaled by c (sign included) in fp32 and rounded to
        // fp16, or (QS = false) as they are with only the scale's sign applied to the sign bits
        auto prepared = [&](qraw_t raw_w) {
            half8 sc = kZero8;
            if (QS) {
                const float cs = a.negate ? -a.c : a.c;
                typedef _Float16 qhalf_t __attribute__((ext_vector_type(PRE == 8 ? 4 : 8)));
                const qhalf_t raw = __builtin_bit_cast(qhalf_t, raw_w);
#pragma unroll
                for (int e = 0; e < (PRE == 8 ? 4 : 8); ++e) sc[e] = (_Float16)((float)raw[e] * cs);
            } else {
                uint4v u = {0u, 0u, 0u, 0u};
                const uint32_t flip = a.negate ? 0x80008000u : 0u;
#pragma unroll
                for (int e = 0; e < (PRE == 8 ? 2 : 4); ++e) u[e] = raw_w[e] ^ flip;
                sc = __builtin_bit_cast(half8, u);
            }
            return sc;
        };
        const half8 sc = prepared(qraw);
        char *tile = qshare + (buf * PQG + qg) * 4096;
        if (PRE == 8) {  // 4 rows per wave, 8 bytes per lane
            const int row = kg * 4 + (lane >> 4), pc = (lane & 15) >> 1, hf = lane & 1;
            const uint4v u = __builtin_bit_cast(uint4v, sc);
            *reinterpret_cast<uint2 *>(tile + row * 128 + ((pc ^ ((row >> 1) & 7)) * 16) + hf * 8) = uint2{u[0], u[1]};
        } else if (PRE == 4) {  // 8 rows per wave, one whole 16-byte piece per lane
            const int row = kg * 8 + (lane >> 3), pc = lane & 7;
            *reinterpret_cast<half8 *>(tile + row * 128 + ((pc ^ ((row >> 1) & 7)) * 16)) = sc;
        } else {  // 16 rows per wave, two adjacent pieces per lane
            const int row = kg * 16 + (lane >> 2), pc = (lane & 3) * 2;
            *reinterpret_cast<half8 *>(tile + row * 128 + ((pc ^ ((row >> 1) & 7)) * 16)) = sc;
            *reinterpret_cast<half8 *>(tile + row * 128 + (((pc + 1) ^ ((row >> 1) & 7)) * 16)) = prepared(qraw_hi);
        }
    };
    auto take_q_shared = [&](int buf, half8 (&dst)[NT]) {
        const uint32_t diff = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)qshare + (uint32_t)((buf * PQG + qg) * 4096) -
                              (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)my_ring;
        const uint32_t ta0 = take_addr[0] + diff, ta1 = take_addr[1] + diff, ta2 = take_addr[2] + diff, ta3 = take_addr[3] + diff;
        asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %5\n\tds_read_b128 %2, %6\n\tds_read_b128 %3, %7"
                     : "=&v"(dst[0]), "=&v"(dst[1]), "=&v"(dst[2]), "=&v"(dst[3])
                     : "v"(ta0), "v"(ta1), "v"(ta2), "v"(ta3)
                     : "memory");
    };

    half8 qf_c[DC][NT], kf[2][NT];
    half8 (&qf)[NT] = qf_c[0];  // the Q operand of a 64-wide head (chunk 0 of a wider one)
    constexpr int TQ = TPW - 2;  // KEEP: the step at which the next unit's Q rows are requested
    // KEEP: key tile `tile` (wave-uniform, 0 .. TPW-1) of unit `ua` (0 current, 1 next) into ring slot `slot`
    auto fetch_key_tile = [&](int ua, int tile, int slot) {
        if (RAGGED) {
            const char *src = k_batch + k_off[ua] + (size_t)tile_first(tile) * k_row_b;
#pragma unroll
            for (int tt = 0; tt < NT; ++tt) {
                FCS_OPAQUE_V(k_voff[tt % NVOFF]);
                fetch_piece_at(src, k_voff[tt % NVOFF], slot, tt);
            }
        } else {
            const char *src = k_b + k_off[ua] + (size_t)((uint32_t)(tile * 32) * k_row_b);
#pragma unroll
            for (int tt = 0; tt < NT; ++tt) fetch_piece(src, k_voff, slot, tt);
        }
    };
    if (KEEP) {
        fetch_pos(0, 0);  // the Q rows
#pragma unroll
        for (int r = 0; r < NS; ++r) fetch_key_tile(0, r, r);
    } else {
#pragma unroll
        for (int i = 0; i < NS; ++i) fetch_pos(i, i);
    }
    if (PRE) {
        // behind the Q rows: KEEP the first NS key tiles, else two key tiles
        q_publish(0, std::integral_constant<int, (KEEP ? NS : 2) * NT>{});
        __syncthreads();
    }

    for (int unit = 0; unit < n_units; ++unit) {
        const int h = h_begin + cur_hr;
        const int blk_row0 = (rb_first + cur_rb) * 32 * qg_n;  // first query row of the unit's row block
        const int q_first = blk_row0 + qg * 32;                  // this wave's first query row, unclamped
        set_units();
        // this head's Q tile and first key tile (fetched during the previous head).  (Reading them
        // back earlier, under the previous head's column-sum FMAs, makes them live across the loop
        // and the kernel spills.)
        if (PRE) {
            take_q_shared(unit & 1, qf);
        } else {
            // item i of the unit has landed once at most the NS - 1 - i items requested behind it are outstanding
            FCS_WAIT_VM((NS - 1) * NT);
            take_issue(slot_of(0), qf_c[0]);
            if constexpr (DC == 2) {
                FCS_WAIT_VM((NS - 2) * NT);
                take_issue(slot_of(1), qf_c[1]);
            }
        }
        // KEEP: does the next unit read another key head (then its first NS tiles are fetched during
        // this unit's last NS steps, in the first order; else they are the ones this unit leaves behind)
        const bool next_key_head = KEEP && k_off[1] != k_off[0];
        if (KEEP) {
            // the unit's first NS tiles are in the ring: left by the previous unit, or requested
            // during its last steps (first unit of a key head), or by the prologue.  Nothing else is
            // outstanding here, so the common case does not wait.
            FCS_WAIT_VM(0);
            take_issue(slot_of_step(0), kf[0]);
        } else {
            FCS_WAIT_VM((NS - 1 - DC) * NT);
            take_issue(slot_of(DC), kf[0]);
        }
        floatx16 acc[TPW];
        float rs[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) rs[i] = 0.f;

        // e = 2^(c*s) for tile t, in place, and its contribution to the row sums
        auto exp_tile = [&](int t) {
            // ragged: a column that counts for nothing (see tile_first) gets the bias -inf, so its
            // exponential is 0; the bias rides on the scale multiply (one FMA).  Pre-scaled scores have
            // no multiply to carry it: there the column's exponentials (finite: they repeat real keys)
            // enter the row sums with weight 0 (an FMA in place of the add).
            const bool counts = !RAGGED || (KEEP ? tile_of(t) : t) <= tmax_lane;
            const float bias = counts ? 0.f : -INFINITY, one = counts ? 1.f : 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float e = fast_exp2(PRESCALED ? acc[t][i] : (RAGGED ? fmaf(acc[t][i], a.c, bias) : acc[t][i] * a.c));
                acc[t][i] = e;
                if (PRESCALED && RAGGED) rs[i] = fmaf(e, one, rs[i]);
                else rs[i] += e;
            }
            // pinned here: otherwise the optimiser sinks every exponent below the last MFMA
            asm volatile("" : "+v"(rs[0]), "+v"(rs[1]), "+v"(rs[2]), "+v"(rs[3]), "+v"(rs[4]), "+v"(rs[5]), "+v"(rs[6]),
                         "+v"(rs[7]), "+v"(rs[8]), "+v"(rs[9]), "+v"(rs[10]), "+v"(rs[11]), "+v"(rs[12]), "+v"(rs[13]),
                         "+v"(rs[14]), "+v"(rs[15]));
        };

        // ---------------- phase 1: one step per key tile (per half tile of a 128-wide head: chunk dc of tile t)
#pragma unroll
        for (int s = 0; s < TPW * DC; ++s) {
            const int t = s / DC, dc = s % DC;
            // The two waves that share a SIMD (w and w + 4) take turns at the higher issue priority, one
            // step each.  With equal priorities the older wave wins every arbitration, finishes
            // its tiles ~20 % early and idles at the barrier while the other one runs alone, without
            // anything to overlap its MFMAs with (measured: 2-3 % of the kernel).
            if (((s & 1) != 0) == (wave >= 4)) asm volatile("s_setprio 2");
            else asm volatile("s_setprio 0");
            // the operands of this tile were read back during the previous step: they have landed,
            // their ring slots are free again and take the look-ahead fetches
            if (KEEP) {
                if (t == 0) take_wait(qf);
                take_wait(kf[t & 1]);
                if (t == TQ) fetch_pos(ITEMS, 0);  // the next unit's Q rows
                // The slot of this step's tile is free.  It takes the tile of step t + NS (which shares the
                // slot) if the unit has that step; else nothing, unless the next unit reads another key
                // head: then the tile of that head that belongs in this slot (its first NS tiles, one per
                // slot, over the unit's last NS steps).
                if (t + NS < TPW) fetch_key_tile(0, tile_of(t + NS), slot_of_step(t));
                else if (next_key_head) fetch_key_tile(1, slot_of_step(t), slot_of_step(t));
                // The tile of step t + 1 (t + 1 >= NS) was requested at step t + 1 - NS; behind it: the
                // tiles requested at the steps after that one, up to this step or step TPW - NS - 1 (the
                // last one that requests a tile), i.e. min(NS - 1, TPW - 2 - t) tiles, and the Q rows at
                // step TQ.
                // (The requests for another key head are not counted: with them outstanding the waits
                // below only wait for more than they need.)
                if (t + 1 >= NS && t + 1 < TPW) {
                    if (t >= TQ) FCS_WAIT_VM(QV);
                    else FCS_WAIT_VM((TPW - 2 - t < NS - 1 ? TPW - 2 - t : NS - 1) * NT);
                }
                if (t + 1 < TPW) take_issue(slot_of_step(t + 1), kf[(t + 1) & 1]);
            } else {
            // private rings (never pre-scaled): item DC + s is this step's key (half) tile
            if (s == 0) {
#pragma unroll
                for (int ch = 0; ch < DC; ++ch) take_wait(qf_c[ch]);
                take_wait(kf[0]);
                if (a.negate) {
#pragma unroll
                    for (int ch = 0; ch < DC; ++ch)
#pragma unroll
                        for (int tt = 0; tt < NT; ++tt) qf_c[ch][tt] = flip_sign(qf_c[ch][tt]);
                }
#pragma unroll
                for (int i = 0; i <= DC; ++i) fetch_pos(i + NS, slot_of(i));
            } else {
                take_wait(kf[s & 1]);
                fetch_pos(DC + s + NS, slot_of(DC + s));
            }
            // the next key (half) tile has landed; the NS - 1 items fetched after it may be in flight
            FCS_WAIT_VM((NS - 1) * NT);
            if (s + 1 < TPW * DC) take_issue(slot_of(DC + s + 1), kf[(s + 1) & 1]);
            }
            floatx16 c = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (dc > 0) c = acc[t];  // the second chunk's products join the first's
#pragma unroll
            for (int tt = 0; tt < NT; ++tt) c = mfma16<BF>(qf_c[dc][tt], kf[s & 1][tt], c);
            acc[t] = c;
            if (dc == DC - 1 && t > 0) exp_tile(t - 1);  // VALU work of the previous tile runs under this tile's MFMAs
        }
        exp_tile(TPW - 1);

        if (!STATIC_SLOTS) {
            sq += ITEMS % NS;
            if (sq >= NS) sq -= NS;
        }
        // next unit's Q tile; the reduction's barrier publishes it.  Behind its rows: two key tiles
        // (KEEP: nothing that may be waited past)
        if (PRE) q_publish((unit + 1) & 1, std::integral_constant<int, KEEP ? 0 : 2 * NT>{});

        // ---------------- row sums over lanes and key-group waves; w = 1/L (0 for rows not averaged)
        const bool slow = reduce_rows<false>(rs, rr, kg_n, qg, kg, lane, [&](int row, float L) {
            return (blk_row0 + row < a.q_rows) ? __builtin_amdgcn_rcpf(L) : 0.f;
        }, PRESCALED ? kSumHiPre : kSumHi);

        if (!slow && KEEP && rot) {
            // ---------------- phase 3 of a unit in the second order: step t held tile tile_of(t)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const floatx4 w4 = row_values(rr, i4, g);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int t = 0; t < (KEEP ? TPW : 1); ++t) col_rot[t] = fmaf(acc[t][4 * i4 + j], w4[j], col_rot[t]);
                }
            }
        } else if (!slow) {
            // ---------------- phase 3: column sums of e * w
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const floatx4 w4 = row_values(rr, i4, g);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int t = 0; t < TPW; ++t) col_acc[t] = fmaf(acc[t][4 * i4 + j], w4[j], col_acc[t]);
                }
            }
        } else {
            // ------------ rare: max-subtracted softmax for this (head, row block), three passes over
            // the keys with one score tile in registers at a time.  Operands come through ordinary
            // loads; the ring and the operands already read back for the next head are untouched.
            // lane-dependent values are rebuilt here from an opaque copy of the lane id, so that
            // nothing of this rare path is precomputed and kept in registers by the common path
            int lane_s = lane;
            FCS_OPAQUE_V(lane_s);
            const int n_s = lane_s & 31, g_s = lane_s >> 5;
            const int tmax_s = (n_s + a.Sk - 32 - kbase) >> 5;  // tmax_lane again
            const _Float16 *qp = reinterpret_cast<const _Float16 *>(q_batch + (int64_t)h * q_head_b) +
                                 (int64_t)min(q_first + n_s, a.Sq - 1) * a.qs_s + g_s * 8;
            const _Float16 *kp = reinterpret_cast<const _Float16 *>(k_batch + (int64_t)kv_head(h, a.kv_group, a.kv_magic) * k_head_b) + g_s * 8;
            half8 qs[DC * NT];
#pragma unroll
            for (int tt = 0; tt < DC * NT; ++tt) {
                half8 v = kZero8;  // (NARROW) channels past the tensor's head dim are zeros
                if (!NARROW || tt * 16 + g_s * 8 < a.D) v = load8(qp + tt * 16);
                qs[tt] = a.negate ? flip_sign(v) : v;
            }
            auto score_tile = [&](int t) {
                half8 ks[DC * NT];
                const int krow = RAGGED ? tile_first(t) + n_s : kbase + t * 32 + n_s;
#pragma unroll
                for (int tt = 0; tt < DC * NT; ++tt) {
                    ks[tt] = kZero8;
                    if (!NARROW || tt * 16 + g_s * 8 < a.D) ks[tt] = load8(kp + (int64_t)krow * a.ks_s + tt * 16);
                }
                floatx16 c = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int tt = 0; tt < DC * NT; ++tt) c = mfma16<BF>(qs[tt], ks[tt], c);
                return c;
            };
            float v16[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) v16[i] = kNegBig;
#pragma unroll 1
            for (int t = 0; t < TPW; ++t) {
                const floatx16 c = score_tile(t);
                const bool real = !RAGGED || t <= tmax_s;
#pragma unroll
                for (int i = 0; i < 16; ++i) v16[i] = fmaxf(v16[i], real ? c[i] : kNegBig);
            }
            reduce_rows<true>(v16, rr, kg_n, qg, kg, lane_s, [&](int, float m) { return m; });
            float rmax[16];  // subtracted from the scores BEFORE the scale: exact for scores of any size
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const floatx4 m4 = row_values(rr, i4, g_s);
#pragma unroll
                for (int j = 0; j < 4; ++j) rmax[4 * i4 + j] = m4[j];
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) v16[i] = 0.f;
#pragma unroll 1
            for (int t = 0; t < TPW; ++t) {
                const floatx16 c = score_tile(t);
                const bool real = !RAGGED || t <= tmax_s;
#pragma unroll
                for (int i = 0; i < 16; ++i) v16[i] += real ? fast_exp2((c[i] - rmax[i]) * a.c) : 0.f;
            }
            reduce_rows<false>(v16, rr, kg_n, qg, kg, lane_s, [&](int row, float L) {
                return (blk_row0 + row < a.q_rows) ? __builtin_amdgcn_rcpf(L) : 0.f;
            });
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const floatx4 w4 = row_values(rr, i4, g_s);
#pragma unroll
                for (int j = 0; j < 4; ++j) v16[4 * i4 + j] = w4[j];
            }
#pragma unroll 1
            for (int t = 0; t < TPW; ++t) {
                const floatx16 c = score_tile(t);
                const bool real = !RAGGED || t <= tmax_s;
                float sum = 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) sum = fmaf(real ? fast_exp2((c[i] - rmax[i]) * a.c) : 0.f, v16[i], sum);
#pragma unroll
                for (int u = 0; u < TPW; ++u)  // col_acc lives in registers: static index only
                    if (u == t) col_acc[u] += sum;
            }
        }
        if (KEEP) rot = next_key_head ? 0 : (rot ^ 1);
        if (++cur_rb == rb_n) {
            cur_rb = 0;
            ++cur_hr;
        }
    }
    FCS_WAIT_VM(0);  // drain the look-ahead fetches before the block's LDS is released

    // ---------------- the two half-waves hold different rows of the same keys: add, then store
    const int slab = (hgi * a.f_nwgq + qwg) * qg_n + qg;
    float *dst = a.partial + ((int64_t)slab * a.B + b) * a.Sk;
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        // KEEP: tile t was held by step (t + NS) % TPW (rotated order) or TPW - 1 - t (reversed order) of the units in the second order
        const float both = KEEP ? col_acc[t] + col_rot[KEEP_ROT ? (t + NS) % TPW : KEEP_REV ? TPW - 1 - t : 0] : col_acc[t];
        const float v = both + __shfl_xor(both, 32);
        if (g == 0 && t <= tmax_lane) dst[tile_first(t) + n] = v;
    }
}

// Which instantiation serves a call with TPW key tiles per wave (shared by the launcher and the plan description).
struct FusedVariant {
    int tpw;      // template TPW (the shared-Q variants exist for five to eight tiles)
    bool ragged;
    int pre;      // 8, 4, 2: shared Q tile with that many key groups; 0: private rings
    bool qs;      // shared Q tile pre-scaled
};
static FusedVariant pick_fused(const Plan &p, const Args &a, bool bf)
{
    const int TPW = p.f_tpw;
    // head dims other than 64: the ragged private-ring variant (two chunks per tile above 64 channels; channels past
    // the head dim read as zeros)
    if (p.D != 64) return {TPW, true, 0, true};
    const bool whole = p.Sk == p.f_kg * TPW * 32 && p.Sq % (32 * p.f_qg) == 0 && a.qs_s == 64 && a.ks_s == 64;
    // shared-Q variants: five to eight tiles per wave and 8, 4 or 2 key groups (S 257 .. 2048)
    const bool shared_q = TPW >= 5 && (p.f_kg == 8 || p.f_kg == 4 || p.f_kg == 2);
    // ... pre-scaled when the rounding of Q*c to fp16 cannot show in the means
    const bool pre = shared_q && !bf && (long)p.H * p.q_rows >= 4096 && fabsf(a.c) <= 0.1251f * 1.44269504f;
    if (pre && whole && TPW == 8 && (p.f_kg == 8 || p.f_kg == 4)) return {8, false, p.f_kg, true};
    if (pre) return {TPW, true, p.f_kg, true};
    // ... else Q shared through LDS as it is (8 or 4 key groups).  (Two key groups that cannot be
    // pre-scaled stay on the private rings: sharing the Q tile as it is was measured 4 % slower there,
    // B 64 H 16 S 512 bf16 67.2 -> 69.9 us.)
    if (shared_q && p.f_kg != 2) return {TPW, true, p.f_kg, false};
    return {TPW, !whole, 0, true};
}

template <int TPW, bool BF>
static void launch_tpw(const Plan &p, const Args &a, hipStream_t st)
{
    const dim3 grid(p.f_nwgq * p.B, p.f_hg);  // x = batch entry * f_nwgq + workgroup along the query axis
    constexpr int TPWS = (TPW >= 5) ? TPW : 8;
    const FusedVariant v = pick_fused(p, a, BF);
    if (p.Dp == 128 && p.D == 128)
        hipLaunchKernelGGL((fcs_fused_kernel<128, TPW, true, 0, BF>), grid, dim3(512), 0, st, a);
    else if (p.Dp == 128)
        hipLaunchKernelGGL((fcs_fused_kernel<128, TPW, true, 0, BF, true, true>), grid, dim3(512), 0, st, a);
    else if (p.D != 64)
        hipLaunchKernelGGL((fcs_fused_kernel<64, TPW, true, 0, BF, true, true>), grid, dim3(512), 0, st, a);
    else if (v.pre == 8 && v.qs && !v.ragged)
        hipLaunchKernelGGL((fcs_fused_kernel<64, 8, false, 8, false>), grid, dim3(512), 0, st, a);
    else if (v.pre == 4 && v.qs && !v.ragged)
        hipLaunchKernelGGL((fcs_fused_kernel<64, 8, false, 4, false>), grid, dim3(512), 0, st, a);
    else if (v.pre == 8 && v.qs)
        hipLaunchKernelGGL((fcs_fused_kernel<64, TPWS, true, 8, false>), grid, dim3(512), 0, st, a);
    else if (v.pre == 4 && v.qs)
        hipLaunchKernelGGL((fcs_fused_kernel<64, TPWS, true, 4, false>), grid, dim3(512), 0, st, a);
    else if (v.pre == 2 && v.qs)
        hipLaunchKernelGGL((fcs_fused_kernel<64, TPWS, true, 2, false>), grid, dim3(512), 0, st, a);
    else if (v.pre == 8)
        hipLaunchKernelGGL((fcs_fused_kernel<64, TPWS, true, 8, BF, false>), grid, dim3(512), 0, st, a);
    else if (v.pre == 4)
        hipLaunchKernelGGL((fcs_fused_kernel<64, TPWS, true, 4, BF, false>), grid, dim3(512), 0, st, a);
    else if (!v.ragged)
        hipLaunchKernelGGL((fcs_fused_kernel<64, TPW, false, 0, BF>), grid, dim3(512), 0, st, a);
    else
        hipLaunchKernelGGL((fcs_fused_kernel<64, TPW, true, 0, BF>), grid, dim3(512), 0, st, a);
}

size_t describe_fused(const Plan &p, const Args &a, char *buf, size_t n)
{
    const FusedVariant v = pick_fused(p, a, p.bf16 != 0);
    int r = snprintf(buf, n, "fcs_fused_kernel<%d,%d,%s,%d,%s,%s%s> grid %d x %d, %d x %d units per workgroup, %d slabs", p.Dp == 128 ? 128 : 64, v.tpw,
                     v.ragged ? "true" : "false", v.pre, (p.bf16 && !(v.pre && v.qs)) ? "true" : "false", v.qs ? "true" : "false",
                     (p.D % 64 != 0) ? ",true" : "",
                     p.f_nwgq * p.B, p.f_hg, p.f_hpg, p.f_rbpw, p.n_partials);
    if (r < 0) return 0;
    const size_t len = (size_t)r;
    return len + describe_finalize(a, len < n ? buf + len : nullptr, len < n ? n - len : 0);
}

template <bool BF>
static bool launch_fused_t(const Plan &p, const Args &a, hipStream_t st)
{
    switch (p.f_tpw) {
    case 1: launch_tpw<1, BF>(p, a, st); break;
    case 2: launch_tpw<2, BF>(p, a, st); break;
    case 3: launch_tpw<3, BF>(p, a, st); break;
    case 4: launch_tpw<4, BF>(p, a, st); break;
    case 5: launch_tpw<5, BF>(p, a, st); break;
    case 6: launch_tpw<6, BF>(p, a, st); break;
    case 7: launch_tpw<7, BF>(p, a, st); break;
    case 8: launch_tpw<8, BF>(p, a, st); break;
    default: return false;
    }
    return true;
}

hipError_t launch_fused(const Plan &p, const Args &a, hipStream_t st)
{
    if (p.Sk < 32) return hipErrorInvalidValue;  // the ragged kernel fetches whole key tiles that end at the last key
    if (!(p.bf16 ? launch_fused_t<true>(p, a, st) : launch_fused_t<false>(p, a, st))) return hipErrorInvalidValue;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_finalize(a, st);
}

}  // namespace fcs
