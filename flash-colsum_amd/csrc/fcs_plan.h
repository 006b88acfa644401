// Launch plan for the column-mean kernels: how one call is cut into workgroups and how
// the caller's workspace is laid out.  Pure host arithmetic, shared by
// fcs_workspace_bytes() and the launch functions so both always agree.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace fcs {

constexpr int kWavesPerBlock = 4;   // 256 threads
constexpr int kStageKeys = 64;      // keys staged in LDS per step of either pass
constexpr int kComputeUnits = 256;  // MI355X
constexpr int kFusedMaxKeys = 2048; // 8 waves x 8 tiles x 32 keys of fp32 scores per 32 query rows
constexpr int kFewRowsMaxRows = 4;      // few-rows path: at most this many averaged query rows per head ...
constexpr int kFewRowsMaxScores = 12288; // ... and rows * Sk scores (48 KB of LDS)
constexpr int kSmallMaxTiles = 9;        // short-sequence path: one wave holds the scores of 32 rows x (32 x 9) keys
// ... whose workgroups keep the keys of this many heads in an LDS ring (112 KB at most)
constexpr int small_ring_heads(int tiles) { return 28 / tiles < 16 ? 28 / tiles : 16; }

// column pass (fcs_stream.hip): ring slots of 64-key stages and keys per workgroup chunk, sized so
// that the LDS ring plus one accumulator slice per wave fit (twice per compute unit for 4-wave blocks)
constexpr int col_ring_slots(int D, int waves) { return (D == 256 || (D == 128 && waves == 4)) ? 3 : 4; }
constexpr int col_chunk_max(int D, int waves) { return (D == 256) ? 1024 : (D == 128 && waves == 4) ? 1536 : 2048; }

// row-statistics pass on the same stream (fcs_stream.hip): ring slots
constexpr int row_ring_slots(int D, int waves) { return (D == 256 || (D == 128 && waves == 4)) ? 3 : 4; }

struct Plan {
    int B, H, Sq, Sk, D;
    int Dp;      // head dim the kernels are compiled for: 64, 128 or 256, the smallest that holds D
    int bf16;    // operands are bf16 instead of fp16 (set by the caller after make_plan)
    int q_rows;  // query rows that are averaged: min(cls_n, Sq) or Sq
    int causal, k_past;
    // pass 1: row statistics.  grid = (n_qblk, n_chunks, B*H)
    int qw;          // query rows per wave (32 or 64)
    int k1_waves;    // waves per block (4 or 8); a block covers k1_waves*qw rows
    int n_qblk;      // blocks along the query axis
    int n_chunks;    // key-axis splits (partial (max,sum) per chunk when > 1)
    int chunk_keys;  // keys per split, multiple of kStageKeys
    int rows_pad;    // n_qblk * 4 * qw  (row pitch of the statistics arrays)
    // column pass: grid = (c_nchunks, c_groups, B); a block owns c_chunk keys and walks over c_upg
    // (head, row block) units
    int c_nb, c_waves; // 32-row fragments per wave, waves per block: a unit has 32 * c_nb * c_waves rows
    int c_nrb;         // row blocks per head
    int c_chunk, c_nchunks;
    int c_groups, c_upg;
    // fused single-kernel path: non-causal, all keys of a row block fit in one
    // workgroup's registers.  grid = (f_nwgq * B, f_hg)
    int fewrows;     // 1: few-rows path (non-causal, q_rows <= 4): grid = B * f_hg, slabs = f_hg
    int small;       // 1: short-sequence path (non-causal, Sk <= 288, D <= 64): grid = B * f_hg, slabs = f_hg,
                     //    f_tpw key tiles, f_nqblk row tiles of 32 rows per head
    int fused;       // 1: use it (then the two-pass fields above are unused)
    int f_kg, f_qg;  // waves along keys / along queries, f_kg * f_qg == 8
    int f_tpw;       // 32-key tiles per wave
    int f_nqblk;     // query blocks of 32 * f_qg rows
    int f_hg, f_hpg; // head groups, heads per group
    int f_rbpw;      // adjacent query blocks per workgroup (fused path; 1 on the few-rows path)
    int f_nwgq;      // workgroups along the query axis: ceil(f_nqblk / f_rbpw)
    int n_partials;  // slabs summed by the finalize kernel
    int gen_blocks;  // two-pass path: resident workgroups of one generation (what the GPU holds at once)
    // workspace layout (byte offsets, each 256-byte aligned)
    size_t off_lse;      // float2 [B*H][rows_pad]            row maximum and log2 of the row sum
    size_t off_ml;       // float2 [B*H][n_chunks][rows_pad]  only when n_chunks > 1
    size_t off_partial;  // float  [c_groups][B][Sk]          only when c_groups > 1
    size_t total;
};

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Returns false for invalid dimensions.  cls_n <= 0 means all rows.
inline bool make_plan(Plan &p, int causal, int B, int H, int Sq, int Sk, int D, int cls_n, int k_past)
{
    if (B < 1 || H < 1 || Sq < 1 || Sk < 1 || D < 1 || k_past < 0) return false;
    p.B = B; p.H = H; p.Sq = Sq; p.Sk = Sk; p.D = D;
    p.Dp = (D <= 64) ? 64 : (D <= 128) ? 128 : 256;
    p.bf16 = 0;
    p.causal = causal ? 1 : 0;
    p.k_past = causal ? k_past : 0;
    p.q_rows = (cls_n > 0 && cls_n < Sq) ? cls_n : Sq;

    // ---- rows per block of both passes: 512 (8 waves x 64 rows), 256 or 128 (4 waves x 64 or 32).
    // Taller blocks re-read the keys less often.  A small call takes a shorter block instead, while
    // even the finest key split (256 keys per block) of the taller one would leave most compute units
    // without a block: B 1, H 16, S 512, D 128 ran as 32 blocks of 512 rows, 13.6 + 16.0 us.
    int block_rows = (p.q_rows > 256) ? 512 : (p.q_rows > 128) ? 256 : 128;
    while (block_rows > 128 &&
           (long)ceil_div(p.q_rows, block_rows) * B * H * ceil_div(Sk, 4 * kStageKeys) < kComputeUnits)
        block_rows /= 2;

    // ---- pass 1
    p.qw = (block_rows > 128) ? 64 : 32;
    p.k1_waves = (block_rows > 256) ? 8 : 4;
    if (p.Dp == 256) { p.qw = 32; p.k1_waves = 4; }  // the stationary rows of a wider head fill the registers sooner
    const int qblk = p.k1_waves * p.qw;
    p.n_qblk = ceil_div(p.q_rows, qblk);
    p.rows_pad = p.n_qblk * qblk;
    const long base1 = (long)p.n_qblk * B * H;
    // One generation of workgroups: an 8-wave block fills a compute unit's registers, the 4-wave
    // blocks fit twice.  Every further generation pays the block start (Q fragments, first key
    // stage: ~5 us) again, which nothing overlaps.
    // (256-wide heads: the kernels' registers and LDS allow one block per compute unit whatever its waves)
    const int target1 = (p.k1_waves == 8 || p.Dp == 256) ? kComputeUnits : 2 * kComputeUnits;
    p.gen_blocks = target1;
    // as many splits as still fit one generation (rounding up could start a second one for a few blocks)
    int want = (base1 >= target1) ? 1 : (int)(target1 / base1);
    int max_chunks = ceil_div(Sk, 4 * kStageKeys);  // at least 256 keys per split
    if (want > max_chunks) want = max_chunks;
    if (want < 1) want = 1;
    p.chunk_keys = ceil_div(ceil_div(Sk, want), kStageKeys) * kStageKeys;
    p.n_chunks = ceil_div(Sk, p.chunk_keys);

    // ---- column pass (streaming kernel)
    {
        if (block_rows > 256) { p.c_nb = 2; p.c_waves = 8; }
        else if (block_rows > 128) { p.c_nb = 2; p.c_waves = 4; }
        else { p.c_nb = 1; p.c_waves = 4; }
        if (p.Dp == 256) { p.c_nb = 1; p.c_waves = (block_rows > 128) ? 8 : 4; }
        const int block_rows = 32 * p.c_nb * p.c_waves;
        p.c_nrb = ceil_div(p.q_rows, block_rows);
        const long units = (long)H * p.c_nrb;
        const int chunk_max = col_chunk_max(p.Dp, p.c_waves);
        const long target = (p.c_waves == 8 || p.Dp == 256) ? kComputeUnits : 2 * kComputeUnits;
        int chunk = ceil_div(Sk, kStageKeys) * kStageKeys;
        if (chunk > chunk_max) chunk = chunk_max;
        int nchunks = ceil_div(Sk, chunk);
        long groups = (target + (long)B * nchunks - 1) / ((long)B * nchunks);
        if (groups > units) {
            // one unit per block is still too few blocks: shorter chunks (at least four stages each)
            groups = units;
            const long want_c = target / ((long)B * units);  // rounded down: stay within one generation
            int c = ceil_div(ceil_div(Sk, (int)(want_c < 1 ? 1 : want_c)), kStageKeys) * kStageKeys;
            if (c < 4 * kStageKeys) c = 4 * kStageKeys;
            if (c < chunk) chunk = c;
            nchunks = ceil_div(Sk, chunk);
        } else {
            // Blocks run in generations of `target` (what the GPU holds at once); a launch takes
            // generations x units per block.  Among a few group counts around whole generations take
            // the cheapest: one block over a generation would double the time of the launch.
            const long per = (long)B * nchunks;
            long cand[6] = {groups, target / per, 2 * target / per, 3 * target / per, 4 * target / per, units};
            double best = 0.;
            long best_g = groups;
            for (int ci = 0; ci < 6; ++ci) {
                long gcnt = cand[ci];
                if (gcnt < 1) gcnt = 1;
                if (gcnt > units) gcnt = units;
                const long upg = (units + gcnt - 1) / gcnt;
                const long g_eff = (units + upg - 1) / upg;
                const long gens = (per * g_eff + target - 1) / target;
                const double cost = (double)gens * ((double)upg + 0.15) + 0.0005 * (double)g_eff;
                if (ci == 0 || cost < best) {
                    best = cost;
                    best_g = g_eff;
                }
            }
            groups = best_g;
        }
        if (groups < 1) groups = 1;
        p.c_chunk = chunk;
        p.c_nchunks = nchunks;
        p.c_upg = (int)((units + groups - 1) / groups);
        p.c_groups = (int)((units + p.c_upg - 1) / p.c_upg);
    }

    // ---- few-rows path: a batch of matrix-vector products, one workgroup per (batch entry, head group)
    p.fewrows = 0;
    p.small = 0;
    p.fused = 0;
    // (One workgroup streams a whole key head and computes its R x Sk scores on the VALU.  The fused
    // path, which splits a head's keys over eight waves and uses the matrix pipe, is quicker when
    // there are fewer (batch entry, head) pairs than compute units and a thousand keys or more per
    // head (B 8, H 16, S 2048, 4 rows: 24 -> 15 us), and when a head has more than 4096 scores
    // (B 16, H 16, S 2048, 4 rows: 24.4 -> 19.9 us).  The CLS-token shape B 32, H 16, S 577, 1 row
    // stays here: 13.4 us of kernels against 15.8 us on the fused path.)
    const bool fused_is_quicker = D == 64 && Sk <= kFusedMaxKeys &&
                                  ((Sk >= 1024 && (long)B * H < kComputeUnits) || (long)p.q_rows * Sk > 4096);
    if (!causal && p.q_rows <= kFewRowsMaxRows && (long)p.q_rows * Sk <= kFewRowsMaxScores && (D == 64 || D == 128) &&
        !fused_is_quicker) {
        p.fewrows = 1;
        const long bh = (long)B * H;
        int hpb = (int)((bh + 2047) / 2048);  // heads per workgroup: about 2048 workgroups at most
        if (hpb > H) hpb = H;
        p.f_hpg = hpb;
        p.f_hg = ceil_div(H, hpb);
        p.f_rbpw = 1;
        p.f_nwgq = 1;
        p.n_partials = p.f_hg;
        p.off_lse = p.off_ml = p.off_partial = 0;
        p.total = align256(sizeof(float) * (size_t)p.n_partials * B * Sk);
        return (long)B * p.f_hg < (1L << 31);
    }

    // ---- short-sequence path: a wave holds all the keys of its 32 rows, a workgroup owns f_hpg heads of a
    // batch entry and deals their (head, 32-row tile) items to its eight waves, eight per step
    if (!causal && Sk <= 32 * kSmallMaxTiles && D <= 64) {
        const int tiles = ceil_div(Sk, 32), rt = ceil_div(p.q_rows, 32);
        // the keys of the heads that two consecutive steps touch must fit the ring: items 8t .. 8t + 15
        int span = 0;
        for (int t = 0; t < rt; ++t) {
            const int c = (8 * t + 15) / rt - (8 * t) / rt + 1;
            if (c > span) span = c;
        }
        if (span <= small_ring_heads(tiles)) {
            p.small = 1;
            p.f_tpw = tiles;
            p.f_nqblk = rt;
            // Heads per workgroup: one workgroup is resident per compute unit, so the launch runs in generations
            // of kComputeUnits workgroups, each as long as its steps plus about one step for starting and finishing.
            p.f_hpg = H;
            double best = 0.;
            for (int hg = 1, hpg = H; hpg >= 1; hg = (hpg > 1) ? ceil_div(H, hpg - 1) : H + 1, hpg = (hg <= H) ? ceil_div(H, hg) : 0) {
                const long gens = ((long)B * hg + kComputeUnits - 1) / kComputeUnits;
                const double cost = (double)gens * (ceil_div(hpg * rt, 8) + 1.0) + 0.01 * hg;
                if (hg == 1 || cost < best) {
                    best = cost;
                    p.f_hpg = hpg;
                }
            }
            p.f_hg = ceil_div(H, p.f_hpg);
            p.f_rbpw = 1;
            p.f_nwgq = 1;
            p.f_kg = 1;
            p.f_qg = 8;
            p.n_partials = p.f_hg;
            p.off_lse = p.off_ml = p.off_partial = 0;
            p.total = align256(sizeof(float) * (size_t)p.n_partials * B * Sk);
            return (long)B * p.f_hg < (1L << 31);
        }
    }

    // ---- fused path
    p.n_partials = p.c_groups;
    // (at least one whole key tile: the kernel moves a tile that reaches past the last key back to end there)
    // (64-wide kernels for head dims up to 64, 128-wide ones up to 128; wider heads take the two-pass path)
    // (Heads of 72 .. 120 channels: the 128-wide kernel's variant for narrower heads runs out of registers at seven
    // and eight key tiles per wave, so it takes at most six, i.e. 1536 keys; longer calls take the two-pass path.)
    const bool narrow128 = D > 64 && D < 128;
    if (!causal && Sk >= 32 && Sk <= (narrow128 ? 8 * 6 * 32 : kFusedMaxKeys) && D <= 128) {
        p.fused = 1;
        const int tiles = ceil_div(Sk, 32);
        p.f_kg = 1;
        while (p.f_kg * 8 < tiles) p.f_kg *= 2;  // <= 8 tiles per wave
        if (narrow128) while (p.f_kg * 6 < tiles) p.f_kg *= 2;  // <= 6 there
        p.f_qg = 8 / p.f_kg;
        p.f_tpw = ceil_div(tiles, p.f_kg);
        p.f_nqblk = ceil_div(p.q_rows, 32 * p.f_qg);
        // Units per workgroup: a unit is one (query block, head); a workgroup takes f_rbpw adjacent
        // query blocks times f_hpg heads.  One workgroup is resident per compute unit, so the launch
        // runs in generations of kComputeUnits workgroups, each as long as its units plus about 0.7 of
        // a unit for starting and finishing.  Fewer units per workgroup fill the last generation
        // better (528 workgroups of 16 units take three generations, 2112 of 4 take nine quarter-
        // length ones) at the price of more starts and more partial slabs; more units per workgroup
        // save starts (512 workgroups of 16 units take two generations, 256 of 32 one).
        p.f_hpg = H;
        p.f_rbpw = 1;
        double best = 0.;
        bool first = true;
        for (int rbpw = 1; rbpw <= 16 && (rbpw == 1 || rbpw <= p.f_nqblk); ++rbpw) {
            const int nwgq = ceil_div(p.f_nqblk, rbpw);
            if (ceil_div(p.f_nqblk, nwgq) != rbpw) continue;  // same grouping as a smaller rbpw
            // heads per workgroup, descending, one value per distinct grouping: hpg = ceil(H / hg) for
            // hg = 1, then the next hg that lowers it (about 2 sqrt(H) values)
            for (int hg = 1, hpg = H; hpg >= 1; hg = (hpg > 1) ? ceil_div(H, hpg - 1) : H + 1, hpg = (hg <= H) ? ceil_div(H, hg) : 0) {
                const long gens = ((long)nwgq * B * hg + kComputeUnits - 1) / kComputeUnits;
                // a unit that follows another row block of the same head finds half of its key tiles in
                // the LDS ring (the shared-Q kernels; measured 4 % of a unit): row blocks per head count
                // a little less than heads
                double cost = (double)gens * ((double)hpg * (rbpw - 0.04 * (rbpw - 1)) + 0.7) + 0.01 * hg + 0.002 * rbpw;
                // The 32 workgroups that an XCD runs at a time are neighbours in launch order: nwgq of
                // them share a batch entry, i.e. one head's keys.  When the key heads they stream at
                // the same time outgrow the XCD's 4 MiB L2, the re-reads of a head's keys by its row
                // blocks miss (measured +6 % at B 256, S 1024 with 32 batch entries per XCD).
                const long streams = (nwgq >= 32) ? 1 : (32 + nwgq - 1) / nwgq;
                if (streams * (long)Sk * (2 * p.Dp) > (5L << 19)) cost *= 1.08;
                if (first || cost < best) {
                    first = false;
                    best = cost;
                    p.f_hpg = hpg;
                    p.f_rbpw = rbpw;
                }
            }
        }
        p.f_hg = ceil_div(H, p.f_hpg);
        p.f_nwgq = ceil_div(p.f_nqblk, p.f_rbpw);
        p.n_partials = p.f_hg * p.f_nwgq * p.f_qg;
        p.off_lse = p.off_ml = p.off_partial = 0;
        p.total = align256(sizeof(float) * (size_t)p.n_partials * B * Sk);
        return (long)p.f_nwgq * B * p.f_hg < (1L << 31);
    }

    // ---- workspace
    size_t off = 0;
    p.off_lse = off;
    off = align256(off + 2 * sizeof(float) * (size_t)B * H * p.rows_pad);
    p.off_ml = off;
    if (p.n_chunks > 1) off = align256(off + 2 * sizeof(float) * (size_t)B * H * p.n_chunks * p.rows_pad);
    p.off_partial = off;
    if (p.c_groups > 1) off = align256(off + sizeof(float) * (size_t)p.c_groups * B * Sk);
    p.total = off;
    // both passes launch one-dimensional grids
    return (long)p.n_qblk * p.n_chunks * B * H < (1L << 31) && (long)p.c_nchunks * p.c_groups * B < (1L << 31);
}

}  // namespace fcs
