// MFMA search + sparse attention kernel: bf16 keys/centers in the tiled layout
// (HIRA_TILE16), fan-out a multiple of 16, D = Dv in {64, 128, 256}, at least two levels.
//
// One workgroup (8 waves; 256 registers a wave, so the only one on its CU) owns a few
// tiles of 16 level-1 nodes of one tree, a stride apart; workgroup ids run fastest over the trees
// so that, with 8 L2 slices (XCDs) served round-robin, the workgroups of one tree share a
// slice.  After a common gate every wave scans and gathers on its own; the waves meet again
// for the merge:
//   gate   wave w gates the workgroup's tile w: it issues, before it waits for anything, every
//          load it needs (queries, the 16 x D tile of level-1 centres, the tiles holding the
//          tile's ancestors, radii, child counts) and gates with v_mfma_f32_16x16x32_bf16:
//          a wave-wide 128-bit load fetches a 16 x 32 operand tile from 1 KiB of contiguous
//          memory (that is what the tiled layout is for), the B operand holds the (up to 16)
//          query heads of the GQA group, so the D registers hold score(row, head) with
//          head = lane % 16 and row = 4*(lane/16) + j; a node survives for a head when
//          score + ||q|| r >= tau.  Head masks and child counts of the nodes go to LDS.
//   scan   the surviving nodes of these tiles are dealt round-robin to the waves; from here to
//          the merge a wave works on its own (no barrier).  In each round it takes NB of its
//          nodes: their key tiles were requested a round earlier (buffer loads: scalar base and
//          tile offset, no address registers), the B operand now comes from LDS; all products
//          first, then the next round's tiles are requested, then the leaf filter (q.k >= tau
//          against the lane's own threshold).  A tile with a selected row writes the scaled
//          scores of its rows to the wave's stretch of a table in LDS (-inf: not selected) and
//          appends the selected rows to the wave's row list.
//   gather the wave raises its running maximum per head, turns the listed scores into weights
//          2^(z - m) with lane = (row, head), and fetches the value rows of its list, kVBatch
//          in flight, each row once however many heads selected it:
//          acc[head][:] += weight(row, head) * v[:] with the accumulators in registers
//          (lane owns Dv/64 columns of every head).
//   merge  the waves agree on one maximum per head, rescale their sums to it and add them up
//          through LDS.
// Keys queued since the tree was last updated (row-major, attended by every head) get one
// more workgroup per tree.  One partial (m, l, acc) per head and workgroup goes to global
// memory; the last workgroup of a tree to arrive folds the tree's partials.
//
// Register arrays are only ever indexed by compile-time constants: a run-time index would
// push them to scratch memory.
#pragma once

#include "search.h"
#include "search_mfma_timeline.h"

namespace hira {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;

constexpr int kHeadsPerPass = 16;   // MFMA N
constexpr int kMaxTiles = 4;        // key tiles per block: bf <= 64
constexpr int kMfmaWaves = kMfmaThreads / 64;  // waves per workgroup, at most: one workgroup of 8
                                                // waves on a CU leaves every wave 256 registers
#ifndef HIRA_VBATCH
#define HIRA_VBATCH 32
#endif
constexpr int kVBatch = HIRA_VBATCH;         // value rows in flight per wave

__device__ __forceinline__ bf16x8_t as_bf16x8(const uint4& v) {
    return __builtin_bit_cast(bf16x8_t, v);
}

// Tile `tile` of one tree's tiled matrix (D = 32*KS columns): a uniform base address, to
// which every lane adds its own 16 bytes' offset, so that the loads can take the base from
// scalar registers.
struct TilePtr {
    const char* base;  // uniform
    unsigned lane_off; // lane * 16
};
template <int KS>
__device__ __forceinline__ TilePtr tile_ptr(const void* base, size_t tree_row0, size_t tile, int lane) {
    return TilePtr{reinterpret_cast<const char*>(base) +
                       (tree_row0 * (size_t)(32 * KS) * 2 + tile * (size_t)(KS * 1024)),
                   (unsigned)lane * 16u};
}

template <int KS>
__device__ __forceinline__ void load_tile(const TilePtr tp, uint4 (&a)[KS]) {
#pragma unroll
    for (int s = 0; s < KS; ++s)
        a[s] = *reinterpret_cast<const uint4*>(tp.base + (size_t)tp.lane_off + s * 1024);
}

template <int KS>
__device__ __forceinline__ f32x4_t tile_scores(const uint4 (&a)[KS], const bf16x8_t (&bq)[KS]) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[s]), bq[s], acc, 0, 0, 0);
    return acc;
}

// Buffer addressing for the two streams of the scan and the gather (key tiles, value rows): the
// base sits in a scalar resource descriptor, the part that differs per load in a scalar offset,
// and every lane adds the same small offset of its own, so that no load needs vector registers
// for its address.  (One tree's keys or values must stay under 4 GiB.)
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(uint32_t)bytes, 0x00020000);
}

// Cache policy of the scan's two streams.  A step reads a key tile once, so where the keys of a
// launch are more than the L2s hold they are better loaded non-temporal: they then do not push the
// centres, the queries and the value rows out on their way through.  POL 0: default policy for
// both; 1: key tiles non-temporal; 2: key tiles and value rows non-temporal.  Measured per step
// (keys of the launch: 67 MB / 268 MB / 1.07 GB): POL 0 20.11 / 65.05 / 197.3 us, POL 1 21.34 /
// 65.6 / 181.3 us, POL 2 19.86 / 66.1 / 185.1 us; with eight 67 MB indexes taking turns 22.9 /
// 22.2 / 22.2 us; and 15 % MORE than POL 0 where a caller searches the same 23 MB of keys again
// and again, which the L2s would have kept.  The host picks by the size of the launch's keys; a
// branch around the loads instead of instantiations costs the small launches a microsecond.  The
// coherence bits of the policy (sc0, sc1) change nothing.  The tiles of the 8-bit shadow keep the
// default policy: non-temporal they lose more than they gain.
constexpr int kReadOnce = 2;   // the `nt` bit of a buffer load's cache policy

template <int KS, bool ONCE>
__device__ __forceinline__ void load_tile_buf(__amdgpu_buffer_rsrc_t rsrc, unsigned lane_off,
                                              unsigned tile_off, uint4 (&a)[KS]) {
#pragma unroll
    for (int s = 0; s < KS; ++s)
        a[s] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                                             rsrc, lane_off + (unsigned)(s * 1024), tile_off,
                                             ONCE ? kReadOnce : 0));
}

// the same with the B operand parked in LDS (chunk s of lane l at [s*64 + l]): the scan keeps
// its registers for keys in flight
template <int KS>
__device__ __forceinline__ f32x4_t tile_scores_lds(const uint4 (&a)[KS], const uint4* bq_lds, int lane) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[s]), as_bf16x8(bq_lds[s * 64 + lane]),
                                                      acc, 0, 0, 0);
    return acc;
}

// A 16 x 64 tile of the keys' 8-bit shadow against the 16-bit query steps of up to 16 heads,
// split into a high and a low byte (two v_mfma_i32_16x16x64_i8 per 64 columns): exact integers
//   sum_j (256 hi_j + lo_j) k8_j
// for (row 4*(lane/16) + j, head lane % 16).  Lane (kb, i) of the A operand and lane (kb, head)
// of the B operands both hold columns [64 s + 16 kb, +16): the order of the columns inside the
// instruction does not matter as long as both sides agree.
template <int KS8>
__device__ __forceinline__ i32x4_t tile_scores_i8(const uint4 (&a)[KS8], const uint4 (&bhi)[KS8],
                                                  const uint4 (&blo)[KS8]) {
    i32x4_t hi = {0, 0, 0, 0}, lo = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < KS8; ++s) {
        hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4_t, a[s]),
                                                   __builtin_bit_cast(i32x4_t, bhi[s]), hi, 0, 0, 0);
        lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4_t, a[s]),
                                                   __builtin_bit_cast(i32x4_t, blo[s]), lo, 0, 0, 0);
    }
    return hi * 256 + lo;
}

constexpr float kQ8Steps = 32000.0f;   // the largest |q_j kscale_j| of a head, in its 16-bit steps
constexpr float kQ8KeySlack = 4e-3f;   // added to a node's error bound (in steps of the shadow):
                                       // rounding in the bound itself, in sum |q_j kscale_j| and
                                       // in the fp32 scores of the exact test (D <= 256)
constexpr float kQ8QuerySlack = 0.51f; // a query component is at most this many steps off

__device__ __forceinline__ float pick4(const f32x4_t& v, int j) {
    return j == 0 ? v[0] : (j == 1 ? v[1] : (j == 2 ? v[2] : v[3]));
}

// score of row `i` (0..15) of a scored tile for this lane's head
__device__ __forceinline__ float row_score(const f32x4_t& acc, int i, int col) {
    return __shfl(pick4(acc, i & 3), col + 16 * (i >> 2), 64);
}

__device__ __forceinline__ void stat_add(unsigned long long* st, int slot, unsigned v) {
    if (v) atomicAdd(&st[slot], (unsigned long long)v);
}

// Compile-time shape of one instantiation.
template <int KS, int MT, int GS, bool Q8 = false>
struct MfmaShape {
    static constexpr int D = 32 * KS;
    static constexpr int ROWS = MT * 16;  // key slots of one node
    static constexpr int KA = Q8 ? KS / 2 : KS;  // 16-byte chunks a lane holds of a scanned tile
    // nodes whose key tiles one wave keeps in flight: what the budget of 256 registers leaves
    // after twice the accumulators (GS x D/64) and some seventy registers of everything else
    // (with the 8-bit shadow: also its B operands, one batch of key rows of the exact test and
    // the value rows asked for ahead of it), and what keeps the round's list under 48 KiB of LDS
    static constexpr int KEY_REGS =
        256 - 72 - 2 * GS * (KS / 2) - (Q8 ? 4 * KS + (KS <= 4 ? 8 : 4) * KS + 32 : 0);
    static constexpr int NB_REGS = KEY_REGS / (MT * KA * 4);
    static constexpr int NB_LDS = (12000 / (GS + 1)) / (kMfmaWaves * ROWS);
    static constexpr int NB_MIN = NB_REGS < NB_LDS ? NB_REGS : NB_LDS;
    static constexpr int NB_MAX = Q8 ? 8 : 4;
    static constexpr int NB = NB_MIN < 1 ? 1 : (NB_MIN > NB_MAX ? NB_MAX : NB_MIN);
    static constexpr int LIST = kMfmaWaves * NB * ROWS;  // rows of the list of one round
    static constexpr int SCAN_WORDS = LIST * (GS + 1) + LIST / 16;  // row list, tile slots, GS scores per row
    static constexpr int MERGE_WORDS = kMfmaWaves * 4 * D;  // four heads of every wave
    static constexpr int WORDS = SCAN_WORDS > MERGE_WORDS ? SCAN_WORDS : MERGE_WORDS;
};

// What a wave needs to gate one tile of 16 level-1 nodes, as it comes from memory.
template <int KS>
struct GateLoads {
    uint4 a1[KS];      // the tile of level-1 centres
    float4 r4;         // radii of rows 4*kb .. 4*kb+3
    int4 c4;           // child counts of the same rows
    float4 e4;         // (8-bit shadow) error bounds of the same rows
    uint4 anc[2][KS];  // tiles holding the ancestors at levels min(L-1,3) and the one below
    float arad[2];
    size_t aid[2];
};

template <int KS, bool Q8>
__device__ __forceinline__ void gate_issue(const SearchParams& p, int tree, int t1, int lane,
                                           int kb, GateLoads<KS>& g) {
    const int L = p.num_levels;
    const size_t row1 = (size_t)tree * p.cap[1];
    load_tile<KS>(tile_ptr<KS>(p.centers[1], row1, (size_t)t1, lane), g.a1);
    g.r4 = *reinterpret_cast<const float4*>(p.radii[1] + row1 + (size_t)t1 * 16 + 4 * kb);
    g.c4 = *reinterpret_cast<const int4*>(p.counts[1] + row1 + (size_t)t1 * 16 + 4 * kb);
    if (Q8) g.e4 = *reinterpret_cast<const float4*>(p.keps + row1 + (size_t)t1 * 16 + 4 * kb);
    size_t sp = 1;  // level-1 nodes under one node of level min(L-1, 3)
    for (int l = 2; l <= min(L - 1, 3); ++l) sp *= (size_t)p.bf;
    const int n_par = min(max(L - 2, 0), 2);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        g.arad[i] = 0.f;
        g.aid[i] = 0;
        if (i < n_par) {
            const int l = min(L - 1, 3) - i;
            g.aid[i] = ((size_t)t1 * 16) / sp;
            load_tile<KS>(tile_ptr<KS>(p.centers[l], (size_t)tree * p.cap[l], g.aid[i] / 16, lane),
                          g.anc[i]);
            g.arad[i] = p.radii[l][(size_t)tree * p.cap[l] + g.aid[i]];
            sp /= (size_t)p.bf;
        }
    }
}

// OUT: the launch also wants dense scores or selection lists (kept out of the attention-only
// instantiation, whose registers are all spoken for).
// Q8: the index keeps an 8-bit shadow of its keys (HIRA_TILE16_Q8).  The scan then reads the
// shadow's tiles (half the bytes) and lists the rows that the shadow cannot rule out for some
// head; their bf16 rows (row-major) are fetched, 16 at a time as one MFMA operand, and take the
// exact test -- with the very products of the other layout, so the selected set and the scores
// are the same bit for bit.
// ONE: every workgroup of the launch scans in a single round (the host knows: its tiles hold no
// more nodes than its waves take at once).  The round is then straight-line code without a loop
// around it, in which the compiler's waits count the loads still in flight and a node's products
// start when ITS tiles have arrived; at the head of a loop they fall back to waiting for
// everything asked for so far.
template <int KS, int MT, int GS, bool OUT, bool Q8, int POL, int HV, bool ONE>
__global__ __launch_bounds__(64 * kMfmaWaves, 2) void search_mfma_kernel(const SearchParams p) {
    using S = MfmaShape<KS, MT, GS, Q8>;
    constexpr int D = S::D;
    constexpr int NB = S::NB;
    constexpr int KA = S::KA;          // 16-byte chunks per lane of a scanned tile
    constexpr int KS8 = Q8 ? KS / 2 : 1;
    constexpr int VPL = KS / 2;        // value elements per lane: Dv = D = 64 * VPL
    constexpr int VW = (VPL + 1) / 2;  // dwords of a value row per lane
    __shared__ __align__(16) uint32_t s_words[S::WORDS];  // the round's list; the merge; the fold
    // a node of my tiles: heads for which it survives (16 bits) | child count << 16
    __shared__ uint32_t s_ninfo[kMfmaMaxTilesPerWg * 16];
    // the surviving ones in order, a copy per wave (each wave makes its own: no barrier):
    // node | child count << 8 | heads << 16
    __shared__ uint32_t s_order[kMfmaWaves][kMfmaMaxTilesPerWg * 16 * HV];
    __shared__ float s_mxw[kMfmaWaves * 16];           // a wave's running maximum per head
    __shared__ float s_lw[kMfmaWaves * 16];
    __shared__ float s_mh[kHeadsPerPass];
    __shared__ float s_red[2 * kHeadsPerPass];
    __shared__ int s_nc[kHeadsPerPass];
    __shared__ int s_last;
    __shared__ uint4 s_bq[KS * 64];  // the B operand (queries) of the scan
    // 8-bit shadow: the queries in steps of the shadow, high and low bytes, as B operands; the
    // step and sum_j |q_j kscale_j| of every head; the error bounds of my nodes
    __shared__ uint4 s_bq8[Q8 ? 2 * KS8 * 64 : 1];
    __shared__ float s_qc[Q8 ? 2 * kHeadsPerPass : 1];
    __shared__ float s_keps[Q8 ? kMfmaMaxTilesPerWg * 16 : 1];

    touch_kernel_arguments();
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nw = blockDim.x >> 6;
    const int col = lane & 15;  // head within the pass
    const int kb = lane >> 4;   // column block of 8 inside each 32-column step
    const int tree = blockIdx.x;
    const int L = p.num_levels, bf = p.bf;
    const bool want_attn = p.part_acc != nullptr;
    // Workgroup y of a tree owns the tree's tiles y, y + (workgroups of the tree), ...: a stride
    // apart, since neighbouring tiles hold sibling nodes, which tend to survive (and be selected
    // from) together.
    const int wg_tiles = (p.size[1] + 15) >> 4;
    const int n_groups = p.tree_blocks;
    const int grp = (int)blockIdx.y;
    const int ntile = (int)blockIdx.y < p.tree_blocks
                          ? min(p.nodes_per_wave, (wg_tiles - grp + n_groups - 1) / n_groups)
                          : 0;
    auto tile_of = [&](int tl) { return grp + tl * n_groups; };
    // level-1 node behind entry n (tile n / 16 of mine, node n % 16 of the tile)
    auto node_of = [&](int n) { return tile_of(n >> 4) * 16 + (n & 15); };
    const bool is_queue = (int)blockIdx.y >= p.tree_blocks;  // the workgroup after the tree's
    Timeline tline(p);  // (empty unless the library is built with time stamps)
    unsigned long long* stats =
        (p.stats && !Timeline::kOn) ? p.stats + (size_t)tree * HIRA_STATS_COLS : nullptr;
    tline.stamp(kTlStart);

    // ---- heads of this pass ----------------------------------------------------------
    int hoff, G;
    if (p.group_size > 0) {  // head h of the launch belongs to tree h / group_size
        hoff = tree * p.group_size + blockIdx.z * kHeadsPerPass;
        G = min(kHeadsPerPass, p.group_size - (int)blockIdx.z * kHeadsPerPass);
    } else {
        hoff = p.tree_q_off[tree] + blockIdx.z * kHeadsPerPass;
        G = min(kHeadsPerPass, p.tree_q_off[tree + 1] - hoff);
    }
    if (G <= 0 || (ntile <= 0 && !is_queue)) return;  // uniform
    G = min(G, GS);
    tline.stamp(kTlArgs);
    const bool head_ok = col < G;
    int qh = 0;
    if (head_ok) qh = p.group_size > 0 ? hoff + col : p.tree_q_heads[hoff + col];

    // ---- softmax state: running maximum m of the lane's head (the same in every wave);
    // per wave: l over the rows it gathered, acc[g][e] = column lane*VPL + e of head g -------
    float m_run = -INFINITY;
    float l_mine = 0.0f;  // this lane's share of l of head lane % GS, over the rows this wave gathered
    float acc[GS][VPL];
#pragma unroll
    for (int g = 0; g < GS; ++g)
#pragma unroll
        for (int e = 0; e < VPL; ++e) acc[g][e] = 0.0f;
    // The gather of the single-round instantiations (up to 8 heads a pass, rows of 256 bytes)
    // fetches value rows 16 bytes a lane: LR lanes share a row, one load instruction brings RPI
    // rows, and lane (row group rg, chunk cc) sums columns 8 cc .. 8 cc + 7 of the rows of its
    // group in acc8; the row groups' sums meet before the merge.  (A quarter of the load
    // instructions and half the instructions per row of the gather below, which holds a row in
    // 4 bytes a lane.  A launch of several rounds keeps the next round's tiles in flight during
    // the gather: its registers take the eight columns of up to four heads, 233 in all.)
    constexpr bool WIDE = (ONE ? GS <= 8 : GS <= 4) && !Q8 && KS == 4;
    constexpr int LR = D / 8;     // lanes per value row
    constexpr int RPI = 64 / LR;  // rows per load instruction
    const int rg = lane / LR, cc = lane % LR;
    float acc8[WIDE ? GS : 1][8];
#pragma unroll
    for (int g = 0; g < (WIDE ? GS : 1); ++g)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc8[g][j] = 0.0f;

    if (is_queue) {
        // ---- the queue of keys appended since the last update of the tree: row-major, every
        // row counts for every head (no threshold).  Lane owns VPL columns; a wave takes rows
        // wave, wave + nw, ..., eight at a time, and keeps its own (m, l, acc) per head. -------
        float qf[GS][VPL], sc2g[GS], mq[GS], lq[GS];
#pragma unroll
        for (int g = 0; g < GS; ++g) {
            mq[g] = -INFINITY;
            lq[g] = 0.0f;
            sc2g[g] = 0.0f;
#pragma unroll
            for (int e = 0; e < VPL; ++e) qf[g][e] = 0.0f;
            if (g < G) {  // uniform
                const int head = p.group_size > 0 ? hoff + g : p.tree_q_heads[hoff + g];
                sc2g[g] = p.scaling[head] * kLog2e;
                const uint16_t* qp = reinterpret_cast<const uint16_t*>(p.q) + (size_t)head * D + lane * VPL;
#pragma unroll
                for (int e = 0; e < VPL; ++e) qf[g][e] = bf16_lo((uint32_t)qp[e]);
            }
        }
        const uint16_t* qk = reinterpret_cast<const uint16_t*>(p.queue_keys) + (size_t)tree * p.queue_cap * D + lane * VPL;
        const uint16_t* qv = reinterpret_cast<const uint16_t*>(p.queue_values) + (size_t)tree * p.queue_cap * D + lane * VPL;
        for (int r0 = wave; r0 < p.queue_len; r0 += 8 * nw) {  // uniform in the wave
            uint16_t kraw[8][VPL], vraw[8][VPL];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int row = min(r0 + i * nw, p.queue_len - 1);
#pragma unroll
                for (int e = 0; e < VPL; ++e) {
                    kraw[i][e] = qk[(size_t)row * D + e];
                    vraw[i][e] = qv[(size_t)row * D + e];
                }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (r0 + i * nw >= p.queue_len) break;  // uniform
#pragma unroll
                for (int g = 0; g < GS; ++g) {
                    if (g >= G) continue;  // uniform (no break: the loop has to unroll)
                    float sdot = 0.0f;
#pragma unroll
                    for (int e = 0; e < VPL; ++e) sdot += bf16_lo((uint32_t)kraw[i][e]) * qf[g][e];
#pragma unroll
                    for (int off = 1; off < 64; off <<= 1) sdot += __shfl_xor(sdot, off, 64);
                    const float z = sdot * sc2g[g];
                    const float mnew = fmaxf(mq[g], z);
                    const float f = exp2f(mq[g] - mnew);  // 0 the first time
                    const float w = exp2f(z - mnew);
                    lq[g] = lq[g] * f + w;
#pragma unroll
                    for (int e = 0; e < VPL; ++e)
                        acc[g][e] = acc[g][e] * f + w * bf16_lo((uint32_t)vraw[i][e]);
                    mq[g] = mnew;
                }
            }
        }
        // hand the wave's state over in the form the merge below expects
#pragma unroll
        for (int g = 0; g < GS; ++g) {
            if (lane == g) l_mine = lq[g];
            if (col == g) m_run = mq[g];
        }
    } else {
        // ---- queries and the first tile's gate operands, issued before the first wait --------
        // (only the waves that gate need the queries in registers: the scan reads them from LDS)
        // (No load here depends on whether the LANE has a head: a lane without one asks for head
        // 0 of the launch and drops what comes back.  Loads under a per-lane condition end up in
        // blocks of their own, and a use that the compiler moves into such a block is waited for
        // there, with everything else still in flight -- the scaling times log2 e was: a whole
        // trip to memory before the gates' operands were even asked for.  Measured on the 32k
        // benchmark step, with the arguments touched as above: 19.74 -> 19.40 us.)
        int tl_mine = wave;  // of my tiles, the one this wave gates next
        uint4 qraw[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) qraw[s] = make_uint4(0, 0, 0, 0);
        float tau = p.tau[qh];
        float sc = p.scaling[qh];
        GateLoads<KS> gl;
        if (tl_mine < ntile) {
#pragma unroll
            for (int s = 0; s < KS; ++s)
                qraw[s] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.q) +
                                                          (size_t)qh * D + s * 32 + kb * 8);
            gate_issue<KS, Q8>(p, tree, tile_of(tl_mine), lane, kb, gl);
        }
        __builtin_amdgcn_sched_barrier(0);  // (nothing that uses a load moves above this line)
        tline.stamp(kTlGateIssued);
        if (!head_ok) {
            tau = INFINITY;
            sc = 0.0f;
#pragma unroll
            for (int s = 0; s < KS; ++s) qraw[s] = make_uint4(0, 0, 0, 0);
        }
        if constexpr (Q8) {
            // ---- the queries in steps of the shadow (the last wave, which has the fewest tiles to
            // gate, for all): lane (kb, head) takes
            // columns [64 s + 16 kb, +16) as the shadow's tiles hold them: u_j = q_j kscale_j,
            // the head's step su = max_j |u_j| / kQ8Steps, U_j = round(u_j / su) in two bytes -------
            if (wave == nw - 1) {
                float uf[KS8][16];
                float umax = 0.0f, asum = 0.0f;
#pragma unroll
                for (int s = 0; s < KS8; ++s) {
                    const int c0 = 64 * s + 16 * kb;
                    uint4 qa = make_uint4(0, 0, 0, 0), qb = make_uint4(0, 0, 0, 0);
                    if (head_ok) {
                        const uint16_t* qp = reinterpret_cast<const uint16_t*>(p.q) + (size_t)qh * D + c0;
                        qa = *reinterpret_cast<const uint4*>(qp);
                        qb = *reinterpret_cast<const uint4*>(qp + 8);
                    }
                    float qf[16];
                    {
                        float f[8];
                        unpack<bf16_t>(qa, f);
#pragma unroll
                        for (int e = 0; e < 8; ++e) qf[e] = f[e];
                        unpack<bf16_t>(qb, f);
#pragma unroll
                        for (int e = 0; e < 8; ++e) qf[8 + e] = f[e];
                    }
                    const float4* kp = reinterpret_cast<const float4*>(p.kscale + (size_t)tree * D + c0);
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float4 k4 = kp[c];
                        uf[s][4 * c + 0] = qf[4 * c + 0] * k4.x;
                        uf[s][4 * c + 1] = qf[4 * c + 1] * k4.y;
                        uf[s][4 * c + 2] = qf[4 * c + 2] * k4.z;
                        uf[s][4 * c + 3] = qf[4 * c + 3] * k4.w;
                    }
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        umax = fmaxf(umax, fabsf(uf[s][e]));
                        asum += fabsf(uf[s][e]);
                    }
                }
                umax = fmaxf(umax, __shfl_xor(umax, 16, 64));
                umax = fmaxf(umax, __shfl_xor(umax, 32, 64));
                asum += __shfl_xor(asum, 16, 64);
                asum += __shfl_xor(asum, 32, 64);
                const float su = fmaxf(umax, 1e-30f) / kQ8Steps;
                const float inv = kQ8Steps / fmaxf(umax, 1e-30f);  // (u * inv: within 0.004 of u / su)
#pragma unroll
                for (int s = 0; s < KS8; ++s) {
                    uint32_t hi[4], lo[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        hi[c] = 0u;
                        lo[c] = 0u;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int U = (int)rintf(uf[s][4 * c + e] * inv);
                            const int h = (U + 128) >> 8;  // U = 256 h + l, l in [-128, 127]
                            const int l = U - (h << 8);
                            hi[c] |= ((uint32_t)h & 0xFFu) << (8 * e);
                            lo[c] |= ((uint32_t)l & 0xFFu) << (8 * e);
                        }
                    }
                    s_bq8[s * 64 + lane] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                    s_bq8[(KS8 + s) * 64 + lane] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                }
                if (kb == 0) {
                    s_qc[col] = su;
                    s_qc[kHeadsPerPass + col] = asum;
                }
            }
        }

        // ---- B operand and ||q|| -----------------------------------------------------------
        bf16x8_t bq[KS];
        float ss = 0.0f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            bq[s] = as_bf16x8(qraw[s]);
            float f[8];
            unpack<bf16_t>(qraw[s], f);
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
        }
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        const float qn = sqrtf(ss);
        if (wave == 0) {
#pragma unroll
            for (int s = 0; s < KS; ++s) s_bq[s * 64 + lane] = qraw[s];
        }

        // ---- gate: one tile per wave at a time ------------------------------------------------
        while (tl_mine < ntile) {  // uniform in the wave
            const int t1 = tile_of(tl_mine);
            if constexpr (OUT) {
                // the dense output's stretch under this tile starts out as the fill value (the
                // barrier behind the gates has every wave wait for these stores, so the scores
                // that any wave writes later come after them)
                if (p.dense_fill) {
                    const int r0 = t1 * 16 * bf, r1 = min(r0 + 16 * bf, p.size[0]);
                    for (int g = 0; g < G; ++g) {
                        const int head = p.group_size > 0 ? hoff + g : p.tree_q_heads[hoff + g];
                        for (int i = r0 + lane; i < r1; i += 64)
                            p.dense[(int64_t)head * p.dense_stride + i] = p.dense_fill_value;
                    }
                }
            }
            const bool count_nodes = stats != nullptr && lane == 0;
            size_t span = 1;  // level-1 nodes under one node of the current level
            for (int l = 2; l < L; ++l) span *= (size_t)bf;
            int lcur = L - 1;
            bool chain = head_ok;  // this head is still alive above the current level
            for (; lcur > 3; --lcur) {  // trees deeper than four levels: one level at a time
                const size_t a = ((size_t)t1 * 16) / span;
                uint4 t[KS];
                load_tile<KS>(tile_ptr<KS>(p.centers[lcur], (size_t)tree * p.cap[lcur], a / 16, lane), t);
                const float rad = p.radii[lcur][(size_t)tree * p.cap[lcur] + a];
                const bool any_alive = __ballot(chain) != 0ull;
                if (count_nodes && ((size_t)t1 * 16) % span == 0 && any_alive && rad > -INFINITY)
                    stat_add(stats, lcur, 1u);
                const float d = row_score(tile_scores<KS>(t, bq), (int)(a % 16), col);
                chain = chain && (d + qn * rad >= tau);
                span /= (size_t)bf;
            }
            const int n_par = min(max(L - 2, 0), 2);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                if (i < n_par) {
                    const bool any_alive = __ballot(chain) != 0ull;
                    if (count_nodes && ((size_t)t1 * 16) % span == 0 && any_alive &&
                        gl.arad[i] > -INFINITY)
                        stat_add(stats, lcur, 1u);
                    const float d = row_score(tile_scores<KS>(gl.anc[i], bq), (int)(gl.aid[i] % 16), col);
                    chain = chain && (d + qn * gl.arad[i] >= tau);
                    span /= (size_t)bf;
                    --lcur;
                }
            }
            const bool tile_live = __ballot(chain) != 0ull;  // uniform

            // level-1 gates: 16 nodes at once
            unsigned alive4 = 0u;
            const int cc[4] = {gl.c4.x, gl.c4.y, gl.c4.z, gl.c4.w};
            if (tile_live) {
                const f32x4_t g1 = tile_scores<KS>(gl.a1, bq);
                const float rr[4] = {gl.r4.x, gl.r4.y, gl.r4.z, gl.r4.w};
                unsigned real = 0u;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (chain && (g1[j] + qn * rr[j] >= tau)) alive4 |= 1u << j;
                    if (stats) real += (unsigned)__popcll(__ballot(col == 0 && rr[j] > -INFINITY));
                }
                if (count_nodes) stat_add(stats, 1, real);
            }
            unsigned long long nb[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) nb[j] = __ballot((alive4 >> j) & 1u);
            // node n = 4*kb' + j of the tile: its heads are field kb' of nb[j]
            // (its child count sits in lane 16*kb', element j, of cc)
            int cnt_n = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = __shfl(cc[j], 16 * ((lane >> 2) & 3), 64);
                if ((lane & 3) == j) cnt_n = c;
            }
            if (lane < 16) {
                const int jn = lane & 3;
                const unsigned long long bits = jn == 0 ? nb[0] : (jn == 1 ? nb[1] : (jn == 2 ? nb[2] : nb[3]));
                s_ninfo[tl_mine * 16 + lane] =
                    (uint32_t)((bits >> (16 * (lane >> 2))) & 0xFFFFull) | ((uint32_t)cnt_n << 16);
            }
            if constexpr (Q8) {  // the error bounds of the tile's nodes travel like the counts
                const float ee[4] = {gl.e4.x, gl.e4.y, gl.e4.z, gl.e4.w};
                float eps_n = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float e = __shfl(ee[j], 16 * ((lane >> 2) & 3), 64);
                    if ((lane & 3) == j) eps_n = e;
                }
                if (lane < 16) s_keps[tl_mine * 16 + lane] = eps_n;
            }
            tl_mine += nw;
            if (tl_mine < ntile) gate_issue<KS, Q8>(p, tree, tile_of(tl_mine), lane, kb, gl);
        }
        tline.stamp(kTlGated);
        __syncthreads();
        tline.stamp(kTlBarrier);

        // ---- the surviving nodes of my tiles in order, dealt round-robin to the waves ----------
        int rounds, alive = 0;
        {
            const int n_info = ntile * 16;
            const unsigned long long lt = (1ull << lane) - 1ull;
#pragma unroll
            for (int i = 0; i < kMfmaMaxTilesPerWg * 16 / 64; ++i) {
                if (64 * i >= n_info) break;  // uniform
                const uint32_t info = 64 * i + lane < n_info ? s_ninfo[64 * i + lane] : 0u;
                const bool live = (info & 0xFFFFu) != 0u;
                const unsigned long long all = __ballot(live);
                if (live) {
                    // (HV = 2: a node goes in as two entries of MT tiles each, the second marked
                    // by bit 15; a half without keys costs its wave nothing but the entry)
                    const int at = (alive + __popcll(all & lt)) * HV;
                    const int cnt_n = (int)(info >> 16);
#pragma unroll
                    for (int h = 0; h < HV; ++h)
                        s_order[wave][at + h] =
                            (uint32_t)(64 * i + lane) | ((uint32_t)min(max(cnt_n - h * MT * 16, 0), MT * 16) << 8) |
                            ((uint32_t)h << 15) | (info << 16);
                }
                alive += __popcll(all);
            }
            alive *= HV;
            rounds = ((alive + nw - 1) / nw + NB - 1) / NB;
            tline.set(kTlAlive, (unsigned long long)alive);
        }

        float sc2 = sc * kLog2e;
        asm volatile("" : "+v"(sc2));  // (computed here, where its load has long arrived, and not
                                       // behind the key tiles' requests, where it would be waited
                                       // for with all of them)
        const size_t row0 = (size_t)tree * p.cap[0];

        // (8-bit shadow: krsrc = the bf16 rows of the exact test, row-major; k8rsrc = the tiles
        // of the shadow, which the scan reads)
        const __amdgpu_buffer_rsrc_t krsrc = make_rsrc(
            reinterpret_cast<const uint16_t*>(p.keys) + row0 * (size_t)D, (size_t)p.cap[0] * D * 2);
        const __amdgpu_buffer_rsrc_t k8rsrc =
            Q8 ? make_rsrc(p.keys8 + row0 * (size_t)D, (size_t)p.cap[0] * D) : krsrc;
        uint4 bq8h[KS8], bq8l[KS8];
        float su = 0.0f, asum = 0.0f;
        if constexpr (Q8) {
#pragma unroll
            for (int s = 0; s < KS8; ++s) {
                bq8h[s] = s_bq8[s * 64 + lane];
                bq8l[s] = s_bq8[(KS8 + s) * 64 + lane];
            }
            su = s_qc[col];
            asum = s_qc[kHeadsPerPass + col];
        }
        const __amdgpu_buffer_rsrc_t vrsrc = make_rsrc(
            reinterpret_cast<const uint16_t*>(p.values) + row0 * (size_t)D, (size_t)p.cap[0] * D * 2);
        // The nodes a wave takes in a round (up to NB of its share), what LDS says about them,
        // and the loads of their key tiles.
        int nx_node[NB], nx_cnt[NB], nx_half[NB];
        uint32_t nx_mask[NB];
        float nx_eps[Q8 ? NB : 1];
        uint4 a[NB][MT][KA];
        auto fetch = [&](int round, int u_only) {  // u_only < 0: all NB nodes of the round
            // my nodes of the round: entries (round*NB + u) * nw + wave of the survivors
            uint32_t ent[NB];
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                if (u_only >= 0 && u != u_only) continue;
                const int k = (round * NB + u) * nw + wave;
                ent[u] = k < alive ? s_order[wave][k] : 0xFFu;
            }
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                if (u_only >= 0 && u != u_only) continue;
                const uint32_t e = (uint32_t)__builtin_amdgcn_readfirstlane((int)ent[u]);
                const int n = (e >> 16) != 0u ? (int)(e & 0xFFu) : -1;
                nx_node[u] = n;
                nx_cnt[u] = (int)((e >> 8) & 0x7Fu);
                nx_half[u] = (int)((e >> 15) & 1u);
                nx_mask[u] = e >> 16;
                if constexpr (Q8) nx_eps[u] = s_keps[max(n, 0)];
                const unsigned tile_first = (unsigned)(node_of(max(n, 0)) * bf) / 16u + (unsigned)(nx_half[u] * MT);
#pragma unroll
                for (int tt = 0; tt < MT; ++tt) {
                    if constexpr (Q8) {
                        // every load is issued, whatever the node (straight-line code, so that the
                        // waits further down can count the loads behind them); a tile that is not
                        // there is asked for beyond the end of the buffer: zeros, no memory access
                        load_tile_buf<KA, false>(k8rsrc, (unsigned)lane * 16u + (tt * 16 < nx_cnt[u] ? 0u : 0x80000000u),
                                          (tile_first + tt) * (unsigned)(KA * 1024), a[u][tt]);
                    } else {
                        // (every load is issued, a tile that is not there beyond the end of the
                        // buffer -- zeros, no memory access: straight-line code, in which the waits
                        // further down can count the loads behind them)
                        load_tile_buf<KA, POL != 0>(krsrc, (unsigned)lane * 16u + (tt * 16 < nx_cnt[u] ? 0u : 0x80000000u),
                                          (tile_first + tt) * (unsigned)(KA * 1024), a[u][tt]);
                    }
                }
            }
        };
        if (rounds > 0) fetch(0, -1);
        tline.stamp(kTlFetched);

        constexpr int KB0 = KS <= 4 ? 2 : 1;      // batches of 16 key rows asked for ahead
        constexpr int RP = 64 / GS;               // rows whose weights one pass over the lanes computes
        constexpr int NPASS = kVBatch / RP;       // GS = 4: 2, GS = 8: 4, GS = 16: 8
        // one round of a wave
        auto do_round = [&](const int r) {
            constexpr bool SINGLE = ONE;
            // the round's score table and row list; every wave has a stretch of ROWS * NB rows of
            // its own and nobody else looks at it: no barrier inside the rounds
            uint32_t* lst_row = s_words;                                        // (LIST) listed row -> table row
            uint32_t* lst_tslot = lst_row + S::LIST;                            // (LIST/16) table tile -> key slot
            float* lst_z = reinterpret_cast<float*>(lst_tslot + S::LIST / 16);  // (LIST, GS) the table

            // ---- scan: the key tiles of this round's nodes were asked for a round ago; node by
            // node: the products, at once the request for the node that takes its place in the
            // next round, then the node's bookkeeping while the other tiles arrive -------------------
            // The bookkeeping below derives everything per-lane from this copy, which the compiler
            // cannot see through: otherwise it computes those values once, ahead of the loop, and
            // they crowd out the registers that the loads above need.
            int lane_o = lane;
            asm volatile("" : "+v"(lane_o));
            const int col = lane_o & 15, kb = lane_o >> 4;

            int nsel = 0;  // rows of my stretch of the list
            float zmax = -INFINITY;
            const int zrow0 = wave * (NB * S::ROWS);  // my stretch of the round's rows
            int node[NB], cnt[NB];
            uint32_t nmask[NB];
            // dense scores / compact lists of the selected rows among 16 scored ones: lane
            // (kb, head) holds rows 4*kb + j, whose key slots are slot4[j]
            auto emit = [&](unsigned sel4, const f32x4_t& sco, const unsigned (&slot4)[4]) {
                unsigned long long sb[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) sb[j] = __ballot((sel4 >> j) & 1u);
                int base = 0;
                if (p.sel_count != nullptr) {  // one atomic per head of the tile (kb = 0)
                    int mine = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        mine += __popcll(sb[j] & (0x0001000100010001ull << col));
                    int b0 = 0;
                    if (kb == 0 && mine > 0) b0 = atomicAdd(&p.sel_count[qh], mine);
                    base = __shfl(b0, col, 64);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if ((sel4 >> j) & 1u) {
                        const unsigned slot = slot4[j];
                        int idx = (int)slot;
                        if (p.dense_by_position) idx = p.perm[row0 + slot];
                        if (p.dense != nullptr)
                            p.dense[(int64_t)qh * p.dense_stride + idx] = sco[j] * sc;
                        if (p.sel_count != nullptr) {
                            // hits of my head ordered before (kb, j): rows j' < j of any
                            // kb, then row j of lower kb
                            int before = 0;
#pragma unroll
                            for (int j2 = 0; j2 < 4; ++j2) {
                                unsigned long long bits = sb[j2] & (0x0001000100010001ull << col);
                                if (j2 == j) bits &= (1ull << (16 * kb)) - 1ull;
                                if (j2 <= j) before += __popcll(bits);
                            }
                            const int pos = base + before;
                            if (pos < p.sel_cap) {
                                p.sel_index[(int64_t)qh * p.sel_cap + pos] = idx;
                                p.sel_score[(int64_t)qh * p.sel_cap + pos] = sco[j];
                            }
                        }
                    }
                }
            };
            // rows (of 16) for which some head's bit is set: OR over the 16 lanes (heads) of my
            // row group by rotating inside the group, then the four groups side by side
            auto rows_of = [&](unsigned sel4) {
                unsigned any4 = sel4;
                any4 |= (unsigned)__builtin_amdgcn_update_dpp(0, (int)any4, 0x121, 0xF, 0xF, false);
                any4 |= (unsigned)__builtin_amdgcn_update_dpp(0, (int)any4, 0x122, 0xF, 0xF, false);
                any4 |= (unsigned)__builtin_amdgcn_update_dpp(0, (int)any4, 0x124, 0xF, 0xF, false);
                any4 |= (unsigned)__builtin_amdgcn_update_dpp(0, (int)any4, 0x128, 0xF, 0xF, false);
                return (unsigned)__builtin_amdgcn_readlane((int)any4, 0) |
                       ((unsigned)__builtin_amdgcn_readlane((int)any4, 16) << 4) |
                       ((unsigned)__builtin_amdgcn_readlane((int)any4, 32) << 8) |
                       ((unsigned)__builtin_amdgcn_readlane((int)any4, 48) << 12);
            };
            auto count_selected = [&](unsigned sel4, unsigned rowmask) {
                const unsigned pairs = (unsigned)__popcll(__ballot(sel4 & 1u)) +
                                       (unsigned)__popcll(__ballot(sel4 & 2u)) +
                                       (unsigned)__popcll(__ballot(sel4 & 4u)) +
                                       (unsigned)__popcll(__ballot(sel4 & 8u));
                if (lane == 0) {
                    stat_add(stats, HIRA_MAX_LEVELS, (unsigned)__popc(rowmask));
                    stat_add(stats, HIRA_MAX_LEVELS + 1, pairs);
                }
            };
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                node[u] = nx_node[u];
                cnt[u] = nx_cnt[u];
                nmask[u] = nx_mask[u];
                const unsigned slot0 = (unsigned)(node_of(max(node[u], 0)) * bf) + (unsigned)(nx_half[u] * MT * 16);
                if constexpr (Q8) {
                    // ---- the shadow's tiles: which rows can it not rule out, for which heads? ----
                    const float eps_u = nx_eps[u];
                    i32x4_t est_u[MT];
#pragma unroll
                    for (int tt = 0; tt < MT; ++tt)  // (every tile: one that is not there came as zeros)
                        est_u[tt] = tile_scores_i8<KS8>(a[u][tt], bq8h, bq8l);
                    // the score q.k lies within `marg` of su * (the integer): the keys' rounding
                    // (eps_u steps a component at most) and the query's (kQ8QuerySlack steps of su)
                    const float marg = (eps_u + kQ8KeySlack) * asum + su * (kQ8QuerySlack * 127.0f * (float)D);
                    const bool head_on = head_ok && ((nmask[u] >> col) & 1u);
                    const float thr_u = head_on ? tau - marg - 1e-6f * (fabsf(tau) + marg) : INFINITY;
                    if (stats && lane == 0) stat_add(stats, 0, (unsigned)cnt[u]);
#pragma unroll
                    for (int tt = 0; tt < MT; ++tt) {
                        if (tt * 16 >= cnt[u]) continue;  // uniform
                        const int lim = cnt[u] - tt * 16 - 4 * kb;  // my rows j < lim hold keys
                        unsigned pass4 = 0u;
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (su * (float)est_u[tt][j] >= thr_u && j < lim) pass4 |= 1u << j;
                        if (__ballot(pass4 != 0u) == 0ull) continue;  // uniform
                        const unsigned rowmask = rows_of(pass4);
                        if (stats && lane == 0) stat_add(stats, HIRA_MAX_LEVELS + 2, (unsigned)__popc(rowmask));
                        const unsigned tslot = slot0 + tt * 16;
                        // the tile's rows in the table say, for now, which heads a row passed for
                        // (0 / -inf); the rows that passed for some head join my list
                        const int trow = zrow0 + (u * MT + tt) * 16;
                        if (col < GS) {
                            float* zp = lst_z + (trow + 4 * kb) * GS + col;
#pragma unroll
                            for (int j = 0; j < 4; ++j) zp[j * GS] = ((pass4 >> j) & 1u) ? 0.0f : -INFINITY;
                        }
                        if (lane_o < 16 && ((rowmask >> lane_o) & 1u))
                            lst_row[zrow0 + nsel + __popc(rowmask & ((1u << lane_o) - 1u))] = (uint32_t)(trow + lane_o);
                        if (lane_o == 0) lst_tslot[trow >> 4] = tslot;
                        nsel += __popc(rowmask);
                    }
                } else {
                f32x4_t sco_u[MT];
#pragma unroll
                for (int tt = 0; tt < MT; ++tt)  // (a tile that is not there came as zeros)
                    sco_u[tt] = tile_scores_lds<KS>(a[u][tt], s_bq, lane);
                if (r == 0 && u == 0) tline.stamp(kTlTiles);
                if constexpr (!SINGLE) fetch(r + 1, u);  // (past the last round: no node, nothing read)
                // a head for which the node did not survive selects nothing
                const float tau_u = ((nmask[u] >> col) & 1u) ? tau : INFINITY;
                if (stats && lane == 0) stat_add(stats, 0, (unsigned)cnt[u]);
#pragma unroll
                for (int tt = 0; tt < MT; ++tt) {
                    if (tt * 16 >= cnt[u]) continue;  // uniform
                    const f32x4_t sco = sco_u[tt];
                    const int lim = cnt[u] - tt * 16 - 4 * kb;  // my rows j < lim hold keys
                    unsigned sel4 = 0u;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (sco[j] >= tau_u && j < lim) sel4 |= 1u << j;
                    if (__ballot(sel4 != 0u) == 0ull) continue;  // uniform
                    const unsigned rowmask = rows_of(sel4);  // rows selected by some head
                    if (stats) count_selected(sel4, rowmask);
                    const unsigned tslot = slot0 + tt * 16;

                    // ---- dense scores / compact lists ------------------------------------------
                    if (OUT && (p.dense != nullptr || p.sel_count != nullptr)) {
                        const unsigned slot4[4] = {tslot + 4 * kb, tslot + 4 * kb + 1, tslot + 4 * kb + 2,
                                                   tslot + 4 * kb + 3};
                        emit(sel4, sco, slot4);
                    }

                    // ---- the tile's scores go to the table, its selected rows join my list -----------
                    if (want_attn) {
                        const int trow = zrow0 + (u * MT + tt) * 16;  // the tile's rows in the table
                        float zs[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            zs[j] = ((sel4 >> j) & 1u) ? sco[j] * sc2 : -INFINITY;
                            zmax = fmaxf(zmax, zs[j]);
                        }
                        if (col < GS) {
                            float* zp = lst_z + (trow + 4 * kb) * GS + col;
#pragma unroll
                            for (int j = 0; j < 4; ++j) zp[j * GS] = zs[j];
                        }
                        if (lane_o < 16 && ((rowmask >> lane_o) & 1u))
                            lst_row[zrow0 + nsel + __popc(rowmask & ((1u << lane_o) - 1u))] = (uint32_t)(trow + lane_o);
                        if (lane_o == 0) lst_tslot[trow >> 4] = tslot;
                    }
                    nsel += __popc(rowmask);
                }
                }  // shadow or bf16 tiles
            }
            const int tot = nsel;  // rows on my list
            if (r == 0) {
                tline.stamp_wave(kTlWaveScanned);
                tline.stamp(kTlListed);
                tline.set(kTlRows, (unsigned long long)tot);
                tline.set(kTlRounds, (unsigned long long)rounds);
            }
            tline.add_rows(tot);

            // ---- value rows: kVBatch in flight; the rows of a batch in the score table (lane =
            // (row of the pass, head)), their key slots, and the loads ---------------------------------
            auto issue = [&](int e0, int (&at_v)[NPASS], uint32_t (&vraw)[kVBatch][VW]) {
#pragma unroll
                for (int ps = 0; ps < NPASS; ++ps) {
                    const int le = e0 + ps * RP + lane_o / GS;
                    at_v[ps] = le < tot ? (int)lst_row[zrow0 + le] : -1;  // (-1: past the end)
                }
                int slot_v[NPASS];  // the key slots of all the rows of a pass
#pragma unroll
                for (int ps = 0; ps < NPASS; ++ps)
                    slot_v[ps] = at_v[ps] >= 0 ? (int)(lst_tslot[at_v[ps] >> 4] + (unsigned)(at_v[ps] & 15)) : 0;
                // (a batch is always loaded whole, rows past the end as slot 0: straight-line code;
                // loads under conditions of their own cost more than they save)
#pragma unroll
                for (int i = 0; i < kVBatch; ++i) {
                    {
                        const unsigned slot = (unsigned)__builtin_amdgcn_readlane(slot_v[i / RP], (i % RP) * GS);
                        const unsigned voff = (unsigned)lane_o * (unsigned)(VPL * 2);
                        const unsigned soff = slot * (unsigned)(D * 2);
                        if (VPL == 1) {
                            vraw[i][0] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(vrsrc, voff, soff, POL == 2 ? kReadOnce : 0);
                        } else if (VPL == 2) {
                            vraw[i][0] = __builtin_amdgcn_raw_buffer_load_b32(vrsrc, voff, soff, POL == 2 ? kReadOnce : 0);
                        } else {
                            const u32x2_t v2 = __builtin_amdgcn_raw_buffer_load_b64(vrsrc, voff, soff, POL == 2 ? kReadOnce : 0);
                            vraw[i][0] = v2.x;
                            vraw[i][VW - 1] = v2.y;
                        }
                    }
                }
            };
            // ---- the exact test (8-bit shadow): the listed rows' bf16 keys, 16 at a time as one A
            // operand (lane (kb, i): columns [32 s + 8 kb, +8) of the i-th of them) ---------------------
            auto rows16 = [&](int e0, int& at, unsigned& slot, uint4 (&kr)[KS]) {
                const int le = e0 + (lane_o & 15);
                at = le < tot ? (int)lst_row[zrow0 + le] : -1;  // (-1: past the end)
                slot = at >= 0 ? lst_tslot[at >> 4] + (unsigned)(at & 15) : 0u;
#pragma unroll
                for (int s = 0; s < KS; ++s)
                    kr[s] = __builtin_bit_cast(
                        uint4, __builtin_amdgcn_raw_buffer_load_b128(
                                   krsrc, slot * (unsigned)(D * 2) + (unsigned)(kb * 16 + s * 64), 0, 0));
            };
            auto exact16 = [&](int at, unsigned slot, const uint4 (&kr)[KS]) {
                const f32x4_t sco = tile_scores_lds<KS>(kr, s_bq, lane_o);
                unsigned sel4 = 0u;
                int at4[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    at4[j] = __shfl(at, 4 * kb + j, 64);
                    const bool mine = col < GS && at4[j] >= 0;
                    // (the table holds 0 where the shadow let the row pass for my head)
                    const float pz = mine ? lst_z[at4[j] * GS + col] : -INFINITY;
                    const bool sel = pz == 0.0f && sco[j] >= tau;
                    if (sel) sel4 |= 1u << j;
                    const float z = sel ? sco[j] * sc2 : -INFINITY;
                    zmax = fmaxf(zmax, z);
                    if (mine) lst_z[at4[j] * GS + col] = z;
                }
                if (stats) count_selected(sel4, rows_of(sel4));
                if (OUT && (p.dense != nullptr || p.sel_count != nullptr)) {
                    unsigned slot4[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) slot4[j] = (unsigned)__shfl((int)slot, 4 * kb + j, 64);
                    emit(sel4, sco, slot4);
                }
            };
            // ---- what is left to do with the rows of a round (`pr`; the lists and `tot` are its):
            // the best selected score of every head, the sums rescaled to it, the value rows ----------
            // ---- the best selected score of every head among rows just scored (zmax), the new
            // running maximum, and what it does to the sums so far; head g lives in lane g; the
            // weights are computed with lane = (row, head), head = lane % GS -----------------------
            float m_lane = 0.0f;  // the running maximum of head lane % GS (a finite stand-in for -inf)
            auto raise_max = [&]() {
                zmax = fmaxf(zmax, __shfl_xor(zmax, 16, 64));
                zmax = fmaxf(zmax, __shfl_xor(zmax, 32, 64));
                const float mnew = fmaxf(m_run, zmax);
                const float f = (m_run == mnew) ? 1.0f : exp2f(m_run - mnew);
                m_run = mnew;
                // a head without a selected key has m = -inf and only z = -inf: any finite stand-in
                m_lane = __shfl(mnew == -INFINITY ? 0.0f : mnew, lane_o & (GS - 1), 64);
                if (__ballot(f != 1.0f) != 0ull) {  // uniform
                    l_mine *= __shfl(f, lane_o & (GS - 1), 64);
#pragma unroll
                    for (int g = 0; g < GS; ++g) {
                        const float fg = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), g));
                        if constexpr (WIDE) {
#pragma unroll
                            for (int j = 0; j < 8; ++j) acc8[g][j] *= fg;
                        } else {
#pragma unroll
                            for (int e = 0; e < VPL; ++e) acc[g][e] *= fg;
                        }
                    }
                }
            };
            // ---- a batch of value rows into the sums -----------------------------------------------
            auto consume = [&](int e0, const int (&at_v)[NPASS], const uint32_t (&vraw)[kVBatch][VW]) {
                // (nothing of what follows may be scheduled ahead of loads issued before this point)
                __builtin_amdgcn_sched_barrier(0);
                // scores -> weights, in place, 64 (row, head) pairs at a time
#pragma unroll
                for (int ps = 0; ps < NPASS; ++ps) {
                    if (at_v[ps] >= 0) {
                        float* zp = lst_z + at_v[ps] * GS + (lane_o & (GS - 1));
                        const float w = __builtin_amdgcn_exp2f(*zp - m_lane);
                        l_mine += w;
                        *zp = w;
                    }
                }
                // eight rows at a time: one test whether the list goes that far, no branch between
                // the rows of an eight (their weights and products can then be in flight together);
                // a row past the end reads the weights of the batch's first row and counts for nothing
                const int at_first = __builtin_amdgcn_readlane(at_v[0], 0);
#pragma unroll
                for (int i = 0; i < kVBatch; ++i) {
                    if ((i & 7) == 0 && e0 + i >= tot) break;  // uniform
                    const bool there = e0 + i < tot;           // uniform
                    const int at_i = __builtin_amdgcn_readlane(at_v[i / RP], (i % RP) * GS);
                    const int at = there ? at_i : at_first;
                    float vf[VPL];
                    if (VPL == 1) {
                        vf[0] = there ? bf16_lo(vraw[i][0]) : 0.0f;
                    } else {
#pragma unroll
                        for (int e = 0; e < VPL / 2; ++e) {
                            vf[2 * e] = there ? bf16_lo(vraw[i][e]) : 0.0f;
                            vf[2 * e + 1] = there ? bf16_hi(vraw[i][e]) : 0.0f;
                        }
                    }
                    const float* wr = lst_z + at * GS;  // weights of this row, one per head
#pragma unroll
                    for (int g = 0; g < GS; ++g) {
                        const float w = wr[g];  // same address in every lane: a broadcast read
#pragma unroll
                        for (int e = 0; e < VPL; ++e) acc[g][e] += w * vf[e];
                    }
                }
            };
            if constexpr (Q8) {
                // The listed rows go kVBatch at a time: the value rows of the batch (most rows that
                // the shadow lets through are selected) and their key rows are asked for together,
                // so a batch costs one trip to memory: exact test, the running maximum raised to the
                // batch's best scores, the batch's values into the sums.  The first batch is asked
                // for ahead of the next round's tiles -- loads come back in the order they were asked
                // for, so its rows are waited for alone, and its work runs while the tiles are on
                // their way.
                constexpr int KBV = kVBatch / 16;  // batches of 16 key rows per batch of value rows
                {
                    int at_v0[NPASS], at_k[KB0];
                    uint32_t vraw0[kVBatch][VW];
                    unsigned slot_k[KB0];
                    uint4 kr0[KB0][KS];
                    // (these loads go out whatever the list holds, rows past its end as slot 0: under
                    // a condition -- even one for all of them -- the waits below can no longer count
                    // the loads behind them and wait for the next round's tiles as well)
                    __builtin_amdgcn_sched_barrier(0);
                    if (want_attn) issue(0, at_v0, vraw0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int b = 0; b < KB0; ++b) rows16(16 * b, at_k[b], slot_k[b], kr0[b]);
                    __builtin_amdgcn_sched_barrier(0);
                    fetch(r + 1, -1);  // (past the last round: no node, nothing read)
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int b = 0; b < KB0; ++b)
                        if (16 * b < tot) exact16(at_k[b], slot_k[b], kr0[b]);  // uniform
                    for (int e0 = 16 * KB0; e0 < min(tot, kVBatch); e0 += 16) {  // (wide rows only)
                        int at;
                        unsigned slot;
                        uint4 kr[KS];
                        rows16(e0, at, slot, kr);
                        exact16(at, slot, kr);
                    }
                    if (r == 0) tline.stamp_wave(kTlWaveIssued);
                    if (want_attn && tot > 0) {  // uniform
                        raise_max();
                        consume(0, at_v0, vraw0);
                    }
                    if (r == 0) tline.stamp_wave(kTlWaveConsumed);
                }
                for (int e0 = kVBatch; e0 < tot; e0 += kVBatch) {  // uniform in the wave; a hot wave
                    int at_v[NPASS], at_k[KB0];
                    uint32_t vraw[kVBatch][VW];
                    unsigned slot_k[KB0];
                    uint4 kr[KB0][KS];
                    zmax = -INFINITY;
                    if (want_attn) issue(e0, at_v, vraw);
#pragma unroll
                    for (int b0 = 0; b0 < KBV; b0 += KB0) {
#pragma unroll
                        for (int b = 0; b < KB0; ++b) rows16(e0 + 16 * (b0 + b), at_k[b], slot_k[b], kr[b]);
#pragma unroll
                        for (int b = 0; b < KB0; ++b)
                            if (e0 + 16 * (b0 + b) < tot) exact16(at_k[b], slot_k[b], kr[b]);  // uniform
                    }
                    if (want_attn) {
                        raise_max();
                        consume(e0, at_v, vraw);
                    }
                }
            } else {
                if constexpr (WIDE) {
                    if (want_attn && tot > 0) {  // uniform in the launch / in the wave
                        raise_max();
                        constexpr int NLD = kVBatch / RPI;  // load instructions of a batch
                        for (int e0 = 0; e0 < tot; e0 += kVBatch) {  // uniform in the wave
                            // the batch's rows in the score table: for the weights (lane = (row of
                            // the pass, head)) and for the loads (lane = (row group, chunk))
                            int at_w[NPASS], at_r[NLD];
#pragma unroll
                            for (int ps = 0; ps < NPASS; ++ps) {
                                const int le = e0 + ps * RP + lane_o / GS;
                                at_w[ps] = le < tot ? (int)lst_row[zrow0 + le] : -1;  // (-1: past the end)
                            }
#pragma unroll
                            for (int i = 0; i < NLD; ++i) {
                                const int le = e0 + i * RPI + rg;
                                at_r[i] = le < tot ? (int)lst_row[zrow0 + le] : -1;
                            }
                            uint4 vr[NLD];
#pragma unroll
                            for (int i = 0; i < NLD; ++i) {  // (rows past the end: slot 0, weight 0)
                                const unsigned slot =
                                    at_r[i] >= 0 ? lst_tslot[at_r[i] >> 4] + (unsigned)(at_r[i] & 15) : 0u;
                                vr[i] = __builtin_bit_cast(
                                    uint4, __builtin_amdgcn_raw_buffer_load_b128(
                                               vrsrc, slot * (unsigned)(D * 2) + (unsigned)cc * 16u, 0,
                                               POL == 2 ? kReadOnce : 0));
                            }
                            if (r == 0 && e0 == 0) tline.stamp_wave(kTlWaveIssued);
                            __builtin_amdgcn_sched_barrier(0);
                            // scores -> weights, in place, 64 (row, head) pairs at a time
#pragma unroll
                            for (int ps = 0; ps < NPASS; ++ps) {
                                if (at_w[ps] >= 0) {
                                    float* zp = lst_z + at_w[ps] * GS + (lane_o & (GS - 1));
                                    const float w = __builtin_amdgcn_exp2f(*zp - m_lane);
                                    l_mine += w;
                                    *zp = w;
                                }
                            }
#pragma unroll
                            for (int i = 0; i < NLD; ++i) {
                                if (e0 + i * RPI >= tot) break;  // uniform
                                float wv[GS];
#pragma unroll
                                for (int g4 = 0; g4 < GS / 4; ++g4) {
                                    float4 w4 = make_float4(0.f, 0.f, 0.f, 0.f);
                                    if (at_r[i] >= 0)
                                        w4 = *reinterpret_cast<const float4*>(lst_z + at_r[i] * GS + 4 * g4);
                                    wv[4 * g4 + 0] = w4.x;
                                    wv[4 * g4 + 1] = w4.y;
                                    wv[4 * g4 + 2] = w4.z;
                                    wv[4 * g4 + 3] = w4.w;
                                }
                                const uint4 raw = at_r[i] >= 0 ? vr[i] : make_uint4(0, 0, 0, 0);
                                float vf[8];
                                unpack<bf16_t>(raw, vf);
#pragma unroll
                                for (int g = 0; g < GS; ++g)
#pragma unroll
                                    for (int j = 0; j < 8; ++j) acc8[g][j] += wv[g] * vf[j];
                            }
                            if (r == 0 && e0 == 0) tline.stamp_wave(kTlWaveConsumed);
                        }
                    }
                } else
                if (want_attn && tot > 0) {  // uniform in the launch / in the wave
                    raise_max();
                    for (int e0 = 0; e0 < tot; e0 += kVBatch) {  // uniform in the wave
                        int at_v[NPASS];
                        uint32_t vraw[kVBatch][VW];
                        issue(e0, at_v, vraw);
                        if (r == 0 && e0 == 0) tline.stamp_wave(kTlWaveIssued);
                        consume(e0, at_v, vraw);
                        if (r == 0 && e0 == 0) tline.stamp_wave(kTlWaveConsumed);
                    }
                }
            }
            if (r == 0) tline.stamp(kTlGathered);
        };
        if constexpr (ONE) {
            if (rounds > 0) do_round(0);
        } else {
            for (int r = 0; r < rounds; ++r) do_round(r);  // uniform in the workgroup
        }
    }  // tree or queue
    if (!want_attn) return;  // uniform
    tline.stamp_wave(kTlWaveEnd);
    tline.set_wave(kTlWaveRows, tline.rows);
    tline.stamp(kTlWave0Done);

    // ---- merge the waves: first one maximum per head for the workgroup, to which every wave
    // brings its sums (m_run: lane = head col; l_mine: head lane % GS); then l and acc add up ---
    if (kb == 0) s_mxw[wave * 16 + col] = m_run;
    const bool wide = WIDE && !is_queue;  // uniform: my sums are in acc8
    __syncthreads();
    {
        float m_all = -INFINITY;
        for (int w = 0; w < nw; ++w) m_all = fmaxf(m_all, s_mxw[w * 16 + col]);
        const float fw = m_run == -INFINITY ? 0.0f : exp2f(m_run - m_all);
        l_mine *= __shfl(fw, lane & (GS - 1), 64);
#pragma unroll
        for (int g = 0; g < GS; ++g) {
            const float fg = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fw), g));
#pragma unroll
            for (int e = 0; e < VPL; ++e) acc[g][e] *= fg;
            if constexpr (WIDE) {
#pragma unroll
                for (int j = 0; j < 8; ++j) acc8[g][j] *= fg;
            }
        }
        m_run = m_all;
    }
#pragma unroll
    for (int off = GS; off < 64; off <<= 1) l_mine += __shfl_xor(l_mine, off, 64);
    if (lane < GS) s_lw[wave * 16 + lane] = l_mine;
    if (wave == 0 && kb == 0) s_mh[col] = m_run;
    int tid = threadIdx.x;  // (opaque, like lane_o above: nothing of the merge is computed early)
    asm volatile("" : "+v"(tid));
    float* macc = reinterpret_cast<float*>(s_words);  // (nw, 4, D): four heads at a time
    const int P = p.num_parts;
#pragma unroll
    for (int c = 0; c < GS / 4; ++c) {
        if (c * 4 >= G) continue;  // uniform (no break: the loop has to unroll)
        __syncthreads();           // the list (or the previous four heads) is not needed any more
        if (wide) {
            if constexpr (WIDE) {
                // The four row groups' sums of the four heads meet so that group rg ends up with
                // head rg: the halves of the wave trade heads (0,1) against (2,3) -- one swap
                // leaves, in the lower half, both halves' sums of head 0 or 1, in the upper half
                // those of head 2 or 3 --, then the rows of 16 lanes trade (0,2) against (1,3).
                float mine[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const auto s02 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc8[c * 4 + 0][j]),
                                                                      __float_as_uint(acc8[c * 4 + 2][j]), false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc8[c * 4 + 1][j]),
                                                                      __float_as_uint(acc8[c * 4 + 3][j]), false, false);
                    const float r02 = __uint_as_float(s02[0]) + __uint_as_float(s02[1]);
                    const float r13 = __uint_as_float(s13[0]) + __uint_as_float(s13[1]);
                    const auto t = __builtin_amdgcn_permlane16_swap(__float_as_uint(r02), __float_as_uint(r13), false, false);
                    mine[j] = __uint_as_float(t[0]) + __uint_as_float(t[1]);
                }
                float4* dst = reinterpret_cast<float4*>(macc + (wave * 4 + ((tid & 63) / LR)) * D + ((tid & 63) % LR) * 8);
                dst[0] = make_float4(mine[0], mine[1], mine[2], mine[3]);
                dst[1] = make_float4(mine[4], mine[5], mine[6], mine[7]);
            }
        } else {
#pragma unroll
            for (int gi = 0; gi < 4; ++gi)
#pragma unroll
                for (int e = 0; e < VPL; ++e) macc[(wave * 4 + gi) * D + (tid & 63) * VPL + e] = acc[c * 4 + gi][e];
        }
        __syncthreads();
        if (c == 0) tline.stamp(kTlMerged);
        for (int t = tid; t < 4 * D; t += blockDim.x) {
            const int gi = t / D, e = t % D, g = c * 4 + gi;
            if (g >= G) break;
            float a_sum = 0.0f, lsum = 0.0f;
            for (int w = 0; w < nw; ++w) {
                a_sum += macc[(w * 4 + gi) * D + e];
                lsum += s_lw[w * 16 + g];
            }
            const int head = p.group_size > 0 ? hoff + g : p.tree_q_heads[hoff + g];
            const size_t slot = (size_t)head * P + blockIdx.y;
            // device-scope stores: written through, so that the workgroup that folds the
            // partials (maybe on another L2 slice) reads them without cache-wide flushes;
            // a head without a selected key only says so (m = -inf)
            if (lsum > 0.0f)
                __hip_atomic_store(&p.part_acc[slot * D + e], a_sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (e == 0) {
                __hip_atomic_store(&p.part_m[slot], lsum > 0.0f ? s_mh[g] : -INFINITY, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&p.part_l[slot], lsum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    tline.stamp(kTlStoresIssued);
    if (p.done == nullptr) return;  // the caller folds the partials in a second launch

    // ---- the last workgroup of this tree (and pass) to arrive folds the tree's partials ----
    hand_off_release();
    tline.stamp(kTlStored);
    __syncthreads();
    if (threadIdx.x == 0) {
        int* ctr = p.done + (size_t)tree * gridDim.z + blockIdx.z;
        const int ticket = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = ticket == (int)gridDim.y - 1;
        if (s_last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    tline.stamp(kTlTicket);
    if (!s_last) return;

    auto ld = [](const float* q) {
        return __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    // phase 1: wave w handles heads w, w + nw, ...: M = max m_p, L = sum 2^(m_p - M) l_p, and
    // the list of the partials that hold anything, with their weights 2^(m_p - M)
    const bool listed = 2 * (size_t)G * P <= (size_t)S::WORDS;
    int* clist = reinterpret_cast<int*>(s_words);                // (G, P)
    float* cwt = reinterpret_cast<float*>(s_words) + (size_t)G * P;  // (G, P)
    for (int g = wave; g < G; g += nw) {
        const int head = p.group_size > 0 ? hoff + g : p.tree_q_heads[hoff + g];
        const float* pm = p.part_m + (size_t)head * P;
        const float* pl = p.part_l + (size_t)head * P;
        const float mp0 = lane < P ? ld(pm + lane) : -INFINITY;
        const float lp0 = lane < P ? ld(pl + lane) : 0.0f;
        float mx = mp0;
        for (int i = lane + 64; i < P; i += 64) mx = fmaxf(mx, ld(pm + i));
        mx = wave_max(mx);
        float ls = 0.0f;
        int nc = 0;
        for (int i0 = 0; i0 < P; i0 += 64) {  // uniform
            const int i = i0 + lane;
            const float mp = i0 == 0 ? mp0 : (i < P ? ld(pm + i) : -INFINITY);
            const float lp = i0 == 0 ? lp0 : (i < P ? ld(pl + i) : 0.0f);
            const float w = (mp > -INFINITY) ? exp2f(mp - mx) : 0.0f;
            ls += w * lp;
            const bool nz = w > 0.0f && lp > 0.0f;
            const unsigned long long bal = __ballot(nz);
            if (listed && nz) {
                const int k = nc + __popcll(bal & ((1ull << lane) - 1ull));
                clist[g * P + k] = i;
                cwt[g * P + k] = w;
            }
            nc += __popcll(bal);
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) ls += __shfl_xor(ls, off, 64);
        if (lane == 0) {
            s_red[2 * g] = mx;
            s_red[2 * g + 1] = ls;
            s_nc[g] = nc;
        }
    }
    __syncthreads();
    tline.stamp(kTlFoldListed);
    // phase 2, only partials that hold something.  Where the heads of the tree are consecutive and
    // the workgroup has threads to spare: a thread owns four output columns of a head and every
    // n_grp-th listed partial, eight 16-byte loads in flight (one or two trips to memory for the
    // whole fold instead of one per eight partials and column); the groups' sums meet in LDS.
    // Worth its set-up where the other way takes more than four trips (measured: 8 heads x 32
    // partials 5.9 -> 3.5 us; 4 heads x 32 partials 0.3 us slower).
    const int items = G * (D / 4);
    const int n_grp = items <= (int)blockDim.x ? (int)blockDim.x / items : 0;
    const int narrow_trips = ((G * D + (int)blockDim.x - 1) / (int)blockDim.x) * ((P + 7) / 8);
    if (narrow_trips > 4 && listed && p.group_size > 0 && n_grp >= 1 &&
        2 * (size_t)G * P + (size_t)n_grp * G * D <= (size_t)S::WORDS) {
        float* red = reinterpret_cast<float*>(s_words) + 2 * (size_t)G * P;  // (n_grp, G, D)
        const __amdgpu_buffer_rsrc_t arsrc =
            make_rsrc(p.part_acc + (size_t)hoff * P * D, (size_t)G * P * D * sizeof(float));
        const int item = tid % items, grp = tid / items;
        if (grp < n_grp) {
            const int g = item / (D / 4), qd = item % (D / 4);
            const int nc = s_red[2 * g + 1] > 0.0f ? s_nc[g] : 0;
            const int* cl = clist + g * P;
            const float* cw = cwt + g * P;
            const unsigned col0 = ((unsigned)g * (unsigned)P * (unsigned)D + 4u * (unsigned)qd) * 4u;
            float sx = 0.0f, sy = 0.0f, sz = 0.0f, sw = 0.0f;
            for (int k0 = grp; k0 < nc; k0 += 8 * n_grp) {
                u32x4_t v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)  // (16: the device-scope bit, as in `ld` above)
                    v[u] = __builtin_amdgcn_raw_buffer_load_b128(
                        arsrc, col0 + (unsigned)cl[min(k0 + u * n_grp, nc - 1)] * (unsigned)(D * 4), 0, 16);
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const float w = k0 + u * n_grp < nc ? cw[k0 + u * n_grp] : 0.0f;
                    sx += w * __uint_as_float(v[u].x);
                    sy += w * __uint_as_float(v[u].y);
                    sz += w * __uint_as_float(v[u].z);
                    sw += w * __uint_as_float(v[u].w);
                }
            }
            *reinterpret_cast<float4*>(red + ((size_t)grp * G + g) * D + 4 * qd) = make_float4(sx, sy, sz, sw);
        }
        __syncthreads();
        for (int t = tid; t < G * D; t += blockDim.x) {
            const int g = t / D;
            const float Lg = s_red[2 * g + 1];
            float sum = 0.0f;
            for (int r = 0; r < n_grp; ++r) sum += red[(size_t)r * G * D + t];
            p.attn_out[(size_t)(hoff + g) * D + (t % D)] = Lg > 0.0f ? sum / Lg : 0.0f;
        }
        tline.stamp(kTlFoldDone);
        return;
    }
    // otherwise: thread t owns output column e of head g
    for (int t = tid; t < G * D; t += blockDim.x) {
        const int g = t / D, e = t % D;
        const int head = p.group_size > 0 ? hoff + g : p.tree_q_heads[hoff + g];
        const float M = s_red[2 * g], Lg = s_red[2 * g + 1];
        const float* pm = p.part_m + (size_t)head * P;
        const float* pa = p.part_acc + (size_t)head * P * D + e;
        float s0 = 0.0f, s1 = 0.0f;
        if (Lg > 0.0f) {
            if (listed) {
                const int nc = s_nc[g];
                const int* cl = clist + g * P;
                const float* cw = cwt + g * P;
                int k = 0;
                for (; k + 8 < nc; k += 16) {  // uniform over the columns of a head (32 in flight: slower)
                    float v[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u) v[u] = ld(pa + (size_t)cl[min(k + u, nc - 1)] * D);
#pragma unroll
                    for (int u = 0; u < 16; u += 2) {
                        s0 += (k + u < nc ? cw[k + u] : 0.0f) * v[u];
                        s1 += (k + u + 1 < nc ? cw[k + u + 1] : 0.0f) * v[u + 1];
                    }
                }
                for (; k < nc; k += 8) {  // (at most eight are left)
                    float v[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) v[u] = ld(pa + (size_t)cl[min(k + u, nc - 1)] * D);
#pragma unroll
                    for (int u = 0; u < 8; u += 2) {
                        s0 += (k + u < nc ? cw[k + u] : 0.0f) * v[u];
                        s1 += (k + u + 1 < nc ? cw[k + u + 1] : 0.0f) * v[u + 1];
                    }
                }
            } else {
                for (int i = 0; i < P; ++i) {
                    const float mi = ld(pm + i);
                    const float w = mi > -INFINITY ? exp2f(mi - M) : 0.0f;
                    if (w > 0.0f) s0 += w * ld(pa + (size_t)i * D);
                }
            }
        }
        const float inv = Lg > 0.0f ? 1.0f / Lg : 0.0f;
        p.attn_out[(size_t)head * D + e] = (s0 + s1) * inv;
    }
    tline.stamp(kTlFoldDone);
}

// the attention-only scan of bf16 tiles has an instantiation for launches of a single round
template <int KS, int MT, int GS, bool Q8, int POL, int HV>
void launch_mfma_one(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    const dim3 block(plan.threads);
    const bool out = p.dense != nullptr || p.sel_count != nullptr;
    // nodes (entries of the survivors' list) a workgroup's tiles hold at most, against those its
    // waves take in one round
    const bool one = plan.nodes_per_wave * 16 * HV <= (plan.threads / 64) * MfmaShape<KS, MT, GS, Q8>::NB;
    if (out) {
        hipLaunchKernelGGL((search_mfma_kernel<KS, MT, GS, true, Q8, POL, HV, false>), grid, block, 0, s, p);
    } else if constexpr (!Q8) {
        if (one) hipLaunchKernelGGL((search_mfma_kernel<KS, MT, GS, false, Q8, POL, HV, true>), grid, block, 0, s, p);
        else hipLaunchKernelGGL((search_mfma_kernel<KS, MT, GS, false, Q8, POL, HV, false>), grid, block, 0, s, p);
    } else {
        hipLaunchKernelGGL((search_mfma_kernel<KS, MT, GS, false, Q8, POL, HV, false>), grid, block, 0, s, p);
    }
}

template <int KS, int MT, bool Q8, int POL, int HV = 1>
void launch_mfma_gs(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    if (plan.gmax <= 4) launch_mfma_one<KS, MT, 4, Q8, POL, HV>(plan, p, grid, s);
    else if (plan.gmax <= 8) launch_mfma_one<KS, MT, 8, Q8, POL, HV>(plan, p, grid, s);
    else launch_mfma_one<KS, MT, 16, Q8, POL, HV>(plan, p, grid, s);
}

template <int KS, bool Q8, int POL>
void launch_mfma_mt(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s) {
    const int mt = p.bf / 16;
    if (mt <= 1)
        launch_mfma_gs<KS, 1, Q8, POL>(plan, p, grid, s);
    else if (mt == 2)
        launch_mfma_gs<KS, 2, Q8, POL>(plan, p, grid, s);
    else if (KS == 8 && plan.gmax > 4)
        // 256 columns x 64 keys a node x 8 or 16 heads: a node's four tiles do not fit the
        // registers next to the accumulators; it is scanned as two halves of two tiles
        launch_mfma_gs<KS, (KS == 8 ? 2 : 4), Q8, POL, (KS == 8 ? 2 : 1)>(plan, p, grid, s);
    else
        launch_mfma_gs<KS, 4, Q8, POL>(plan, p, grid, s);
}

// one translation unit per key width and per kind of scan (bf16 tiles under each cache policy,
// 8-bit shadow) keeps the build parallel
void launch_mfma_d64(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_d128(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_d256(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_nt1_d64(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_nt2_d64(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_nt1_d128(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_nt2_d128(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_nt1_d256(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_nt2_d256(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_q8_d64(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
void launch_mfma_q8_d128(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);

}  // namespace hira
