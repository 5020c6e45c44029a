// Span attention forward, MFMA tile kernel (16-bit element types, canonical tree tables).
//
// Work decomposition
//   A wavefront owns one (batch, head) and a strip of consecutive blocks of 16 queries.
//   For a 16-query block starting at q0 (a multiple of 16) the keys every query of the
//   block can attend to are
//     - the leaf blocks q0-16*NBW .. q0 (.. q0+16*NBW when not causal), NBW = ceil(R/16);
//       the level-0 neighbour n^1 lies inside the block's own leaf block;
//     - the 14 tree nodes of levels 1..3 under the block's level-4 ancestor
//       (8 + 4 + 2 consecutive rows) and one sibling node per level 4..L-1, which is the
//       same for all 16 queries.  Levels 1..5 form a "near" key block that changes with
//       every query block; levels 6..L-1 form a "far" key block that is the same for a
//       whole aligned strip of up to 64 queries and is loaded once per strip.
//   So the block's scores are a handful of dense 16x16 tiles with a per-element
//   multiplicity mask (0: not attended, 1, or 2 for the leaf n^1 that is both a window
//   key and the level-0 neighbour).
//
// Data flow: operands are fetched row-contiguously, 16 bytes per lane, and re-laid out per
// wavefront through LDS into MFMA operand order (lane = row, four lane groups = four
// 8-element pieces of 32 channels).
//     S^T[key, query] = K_blk . Q_blk^T            v_mfma_f32_16x16x32 (A = K rows, B = Q rows)
//     V^T-operand     = V_blk . Pi                 the same MFMA with a 0/1 selection matrix
//                                                  moves V into "lane = channel, regs = keys"
//     O^T[ch, query]  = V^T . P^T                  v_mfma_f32_16x16x16 (A, B both come from
//                                                  MFMA results, whose layouts agree)
// The selection matrix orders channels so that a lane ends up holding 8 consecutive
// output channels of one query: the result is stored with one 16-byte store per 32
// channels, in the same addressing pattern as the Q loads.
// Leaf K / transposed-V operands slide along the strip in registers, so inside a strip
// every K/V row is fetched once; later blocks' operands are requested before the current
// block is computed (the strip loop is fully unrolled, every load has its own registers).
// Lanes whose tree slot does not exist (level >= L) issue no load.
#pragma once

#include "hsa_common.h"
#include "hsa_mma.h"

#include <type_traits>

namespace hsa {

constexpr int TILE_Q = 16;           // queries per block
constexpr int TILE_MAX_SB = 4;        // a strip is at most 64 aligned queries
constexpr int TILE_MAX_LEVELS = 22;  // near block: levels 1..5, far block: levels 6..21
constexpr float NEG_INF = -__builtin_inff();

// Which global accesses carry the streaming (non-temporal) hint, as a bit set: 1 = query rows,
// 2 / 16 = the key / value leaf block that enters per query block, 8 = the leaf blocks carried
// into a strip, 4 = tree nodes, 32 = plain instead of streaming output stores.  Rows that one
// wavefront touches once per launch (queries, entering leaf blocks, output) are marked; rows
// that neighbouring strips share (carried-in blocks, tree nodes) stay cacheable.  Measured on
// the headline shape with inputs rotated through 1.2 GB (nothing cache-resident): 20.6 us with
// 1|2|16, 20.8 us with 1 alone or none of the load hints, 21.1 us with every load marked; plain
// output stores cost 2.5 us.  (With only 400 MB rotated the hint on the query rows alone looks
// like 12 %: it keeps them out of the 256 MB memory-side cache, which then holds more of the
// other tensors -- an artefact of too small a rotation, not a property of the kernel.)
#ifndef HSA_TILE_NT
#define HSA_TILE_NT 19
#endif
// 16-byte global load, optionally with the streaming (non-temporal) hint
template <bool NT> __device__ __forceinline__ u32x4_t ld16(const uint16_t *p) {
    if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
    else return *reinterpret_cast<const u32x4_t *>(p);
}

struct TileParams {
    const uint16_t *q, *k, *v;
    uint16_t *out;
    float *weights;  // [B, N, H, 2R+1+L] or null (kernels built with WT only)
    float *lse;      // [B, N, H]: log-sum-exp of a query's biased logits, log2 domain (kernels built with LSE only)
    int B, N, M, H, L, R;
    int NS;       // strips per sequence
    int n_units;  // B * NS * H
    int runs;     // runs of SB blocks one wavefront walks (a strip is SB * runs blocks): the kernel's RUNS
    int xcd_swizzle;
    int alternate;    // neighbouring strips walk in opposite directions
    float scale_log2e;
};

// wavefronts per workgroup: 8 (two per SIMD, <= 256 VGPRs each) up to 64 channels and five
// leaf blocks per query block, 4 (one per SIMD, <= 512 VGPRs) for 128 channels or more leaf blocks
template <int D, int NKL = 1> constexpr int tile_max_wpb() { return (D > 64 || NKL > 5) ? 4 : 8; }

// SB = query blocks per strip.  The strip loop is fully unrolled so that every load lands
// in its own (virtual) registers: no loop-carried copies, the compiler's waits then cover
// exactly the block being computed while later blocks' loads stay in flight.
//
// Global accesses are row-contiguous: the D/8 lanes that share a row fetch its D*2 bytes as
// one contiguous piece (a load instruction covers 64*8/D whole head-rows), which the memory
// pipeline serves markedly faster than a "lane = row" gather (measured on the same byte mix:
// 19.5 us against 23.4 us).  Each wavefront re-lays the 16-byte pieces out into MFMA operand
// order through a private, padded LDS region (no workgroup barrier: a wavefront's LDS
// operations execute in order), and the output takes the reverse route.
// WT: also write the fp32 softmax weights [B, N, H, 2R+1+L] (window slots first, then levels;
// dead slots zero).  A block's 16 rows of weights are assembled in the wavefront's LDS region
// (the operand slots are free once the MFMA operands have been read) and written out as
// whole rows.  Needs 2R+1+L <= D*2+16 floats per row to fit.
// RUNS > 1: a wavefront walks RUNS consecutive runs of SB = 4 blocks (long sequences).  The leaf
// blocks slide on across the runs, so the neighbouring blocks of the window are fetched once per
// strip of 4 * RUNS blocks instead of once per four; only the far tree block (the same for the 64
// queries of a run) is exchanged between runs, requested two blocks ahead.  Straight-line code
// like a single run; two runs are built.
template <typename T, int D, int NBW, bool CAUSAL, int SB, bool WT = false, bool LSE = false, int RUNS = 1>
__global__ void __launch_bounds__((tile_max_wpb<D, (CAUSAL ? NBW + 1 : 2 * NBW + 1)>() * 64))
attn_tile_kernel(TileParams p) {
    using M_ = Mma<T>;
    constexpr bool MULTI = RUNS > 1;
    static_assert(!MULTI || (SB == 4 && !WT), "runs are the 64 queries that share a far tree block");
    constexpr int KS = D / 32;                         // 32-channel steps of the QK contraction
    constexpr int NJ = D / 16;                         // 16-channel output tiles
    constexpr int NKL = CAUSAL ? NBW + 1 : 2 * NBW + 1;  // leaf key blocks per query block
    constexpr int CPR = D / 8;                         // 16-byte pieces per head-row
    constexpr int RPI = 64 / CPR;                      // rows covered by one load instruction
    constexpr int NLD = TILE_Q / RPI;                  // load instructions per 16-row block
    // One 16-row block in LDS: rows back to back (RB bytes each), the 16-byte pieces of row r
    // stored at piece index p ^ swz(r).  The LDS serves a 16-byte access of 16 lanes per cycle
    // from 64 four-byte banks: the row-major side (D/8 lanes per row, consecutive rows) then
    // covers every bank once, and so does the operand side (lane = row, same piece), because
    // rows that share banks get different swz values.  (A padded pitch of RB + 16 made only the
    // operand side conflict-free: two rows of 144 bytes wrap around the 256 bytes of the banks.)
    constexpr int RB = D * 2;
    constexpr int RPB = RB >= 256 ? 1 : 256 / RB;      // rows per pass over the banks
    constexpr int BLK_BYTES = TILE_Q * (RB + 16);      // a block's slot (the weights staging below uses the slack)
    constexpr int WAVE_LDS = 5 * BLK_BYTES;            // q, k, v, near-tree k, near-tree v

    __shared__ __align__(16) unsigned char smem[tile_max_wpb<D, NKL>() * WAVE_LDS];

    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15;   // MFMA operand row / result column
    const int g = lane >> 4;     // MFMA 8-element piece / result row group
    const int lrow = lane / CPR; // row inside a load instruction
    const int lchk = lane % CPR; // 16-byte piece of that row
    const int wpb = blockDim.x >> 6;

    // workgroups that are consecutive in `logical` run on the same XCD (hardware hands
    // consecutive workgroup ids to the 8 XCDs in turn), so strips that share halo rows
    // and upper tree nodes share an L2.
    int wg = blockIdx.x;
    const int nwg = gridDim.x;
    if (p.xcd_swizzle && (nwg & 7) == 0) wg = (wg & 7) * (nwg >> 3) + (wg >> 3);
    // the wavefront index is the same in every lane: keep everything derived from it scalar
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = wg * wpb + wave;
    if (unit >= p.n_units) return;
    const int h = unit % p.H;
    const int s = (unit / p.H) % p.NS;
    const int b = unit / (p.H * p.NS);
    unsigned char *lds = smem + wave * WAVE_LDS;

    const int N = p.N, L = p.L, R = p.R;
    const int NB = N / TILE_Q;
    constexpr int TOT = SB * RUNS;  // blocks per strip
    const int blk0 = s * TOT;       // NB is a multiple of the strip length (powers of two, strip <= NB)
    const size_t rs = (size_t)p.H * D;  // elements between consecutive rows
    const uint16_t *Qb = p.q + ((size_t)b * N * p.H + h) * D + 8 * lchk;
    const uint16_t *Kb = p.k + ((size_t)b * p.M * p.H + h) * D + 8 * lchk;
    const uint16_t *Vb = p.v + ((size_t)b * p.M * p.H + h) * D + 8 * lchk;
    uint16_t *Ob = p.out + ((size_t)b * N * p.H + h) * D + 8 * lchk;

    // ---- lane constants -------------------------------------------------------------
    // selection matrices: output column n of tile jj picks channel 8*(n/4) + 4*jj + n%4
    // of the 32-channel step; as a B operand this lane (column r16, rows 8g..8g+7) holds
    // a single one when g == r16/4.
    u32x4_t Pi[2];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
        const int e = 4 * jj + (r16 & 3);  // element 0..7 inside this lane's 8 rows
        const uint32_t one = (g == (r16 >> 2)) ? (uint32_t)M_::kOne << (16 * (e & 1)) : 0u;
        const int wi = e >> 1;
        Pi[jj] = u32x4_t{wi == 0 ? one : 0u, wi == 1 ? one : 0u, wi == 2 ? one : 0u, wi == 3 ? one : 0u};
    }

    // additive score bias of the leaf blocks (log2 of the multiplicity, -inf = not attended)
    float biasL[NKL][4];
#pragma unroll
    for (int c = 0; c < NKL; ++c) {
        const int dlt = TILE_Q * (c - NBW);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kl = 4 * g + i;
            const int diff = dlt + kl - r16;
            const bool win = diff >= -R && diff <= (CAUSAL ? 0 : R);
            const bool sib = dlt == 0 && kl == (r16 ^ 1) && (!CAUSAL || (r16 & 1));
            const int cnt = (int)win + (int)sib;
            biasL[c][i] = cnt == 0 ? NEG_INF : (cnt == 2 ? 1.0f : 0.0f);
        }
    }

    // tree slots.  Block T ("near", reloaded for every query block): slots 0..7 level 1,
    // 8..11 level 2, 12..13 level 3 (the nodes under the block's level-4 ancestor), slot 14
    // level 4, slot 15 level 5 (siblings of the ancestors).  Block U ("far", loaded once per
    // strip): slot u is the sibling of the level-(6+u) ancestor, the same node for every
    // query of an aligned 64-query strip.  Slots of levels >= L do not exist: not loaded.
    // (a) the near/far slots whose rows this lane fetches, one per load instruction
    int t_lvl[NLD], t_add[NLD], t_xor[NLD], t_off[NLD];
    bool t_valid[NLD], u_valid[NLD];
    int u_lvl[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int sl = i * RPI + lrow;
        if (sl < 8) { t_lvl[i] = 1; t_add[i] = sl; t_xor[i] = 0; }
        else if (sl < 12) { t_lvl[i] = 2; t_add[i] = sl - 8; t_xor[i] = 0; }
        else if (sl < 14) { t_lvl[i] = 3; t_add[i] = sl - 12; t_xor[i] = 0; }
        else { t_lvl[i] = 4 + (sl - 14); t_add[i] = 0; t_xor[i] = 1; }
        t_valid[i] = t_lvl[i] < L;
        t_off[i] = level_offset(N, t_lvl[i]);
        u_lvl[i] = 6 + sl;
        u_valid[i] = u_lvl[i] < L;
    }
    // (b) liveness of the slots whose scores this lane holds (slot 4g+i of each block)
    float biasT[4];  // near block, constant part
    int upT[4];      // level (4 or 5) of a near slot whose liveness depends on the block, or -1
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int sl = 4 * g + i;
        int lvl, pl;
        if (sl < 8) { lvl = 1; pl = sl; }
        else if (sl < 12) { lvl = 2; pl = sl - 8; }
        else if (sl < 14) { lvl = 3; pl = sl - 12; }
        else { lvl = 4 + (sl - 14); pl = -1; }
        bool live;
        upT[i] = -1;
        if (pl >= 0) {
            live = pl == ((r16 >> lvl) ^ 1) && (!CAUSAL || ((r16 >> lvl) & 1));
        } else {
            live = lvl < L;
            if (CAUSAL && live) upT[i] = lvl;
        }
        biasT[i] = live ? 0.0f : NEG_INF;
    }
    float biasU[4];
    auto far_biases = [&](int qs) {  // qs: first query of the run (64 aligned queries)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int lvl = 6 + 4 * g + i;
            const bool live = lvl < L && (!CAUSAL || ((qs >> lvl) & 1));
            biasU[i] = live ? 0.0f : NEG_INF;
        }
    };

    // ---- loaders: raw[i] = piece lchk of row (i*RPI + lrow) of a 16-row block ---------------
    auto load_block = [&](const uint16_t *base, int row0, u32x4_t (&dst)[NLD], auto nt) {  // consecutive rows
        const uint16_t *ptr = base + (size_t)(row0 + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) dst[i] = ld16<decltype(nt)::value>(ptr + (size_t)(i * RPI) * rs);
    };
    constexpr std::integral_constant<bool, (HSA_TILE_NT & 1) != 0> nt_q{};
    constexpr std::integral_constant<bool, (HSA_TILE_NT & 2) != 0> nt_leaf{};
    constexpr std::integral_constant<bool, (HSA_TILE_NT & 16) != 0> nt_leafv{};
    constexpr std::integral_constant<bool, (HSA_TILE_NT & 8) != 0> nt_halo{};
    constexpr bool nt_tree = (HSA_TILE_NT & 4) != 0;
    auto leaf_row0 = [&](int kb) {  // first row of leaf block kb, clamped into the sequence
        kb = kb < 0 ? 0 : (kb >= NB ? NB - 1 : kb);
        return kb * TILE_Q;
    };
    auto load_near = [&](const uint16_t *base, int q0, u32x4_t (&dst)[NLD]) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int tr = t_off[i] + (((q0 >> t_lvl[i]) + t_add[i]) ^ t_xor[i]);
            dst[i] = u32x4_t{0u, 0u, 0u, 0u};
            if (t_valid[i]) dst[i] = ld16<nt_tree>(base + (size_t)tr * rs);
        }
    };
    auto load_far = [&](const uint16_t *base, int qs, u32x4_t (&dst)[NLD]) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            dst[i] = u32x4_t{0u, 0u, 0u, 0u};
            if (u_valid[i]) {
                const int ur = level_offset(N, u_lvl[i]) + ((qs >> u_lvl[i]) ^ 1);
                dst[i] = ld16<nt_tree>(base + (size_t)ur * rs);
            }
        }
    };
    // LDS re-layout of one block: rows in, MFMA operand pieces out
    auto swz = [](int row) { return (row / RPB) % CPR; };
    const int op_swz = swz(r16);
    auto lds_put = [&](int slot, const u32x4_t (&raw)[NLD]) {
        unsigned char *reg = lds + slot * BLK_BYTES;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int row = i * RPI + lrow;
            *reinterpret_cast<u32x4_t *>(reg + row * RB + 16 * (lchk ^ swz(row))) = raw[i];
        }
    };
    auto lds_get = [&](int slot, u32x4_t (&dst)[KS]) {
        const unsigned char *reg = lds + slot * BLK_BYTES + r16 * RB;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            dst[ks] = *reinterpret_cast<const u32x4_t *>(reg + 16 * ((4 * ks + g) ^ op_swz));
    };
    auto transpose_v = [&](const u32x4_t (&op)[KS], u32x2_t (&dst)[NJ]) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            f32x4 z = {0.f, 0.f, 0.f, 0.f};
            f32x4 r = M_::k32(op[j >> 1], Pi[j & 1], z);
            dst[j] = u32x2_t{M_::pack_exact(r[0], r[1]), M_::pack_exact(r[2], r[3])};
        }
    };

    // ---- per-block operand stage (raw, row-contiguous) ----------------------------------------
    struct Stage {
        u32x4_t q[NLD], k[NLD], v[NLD], kt[NLD], vt[NLD];
    };
    // One strip, walked upwards (REV = false) or downwards (REV = true).  Neighbouring strips
    // walk in opposite directions, so the leaf block that two strips share (the last block of
    // one, the left neighbour of the other's first) is fetched by both at the same moment and
    // the second fetch hits in L2 instead of going back to memory.
    // Kl[c] / Vl[c] hold leaf block (blk - NBW + c) of the query block being processed; the
    // block that enters per step is the top one walking upwards, the bottom one downwards.
    auto run = [&](auto rev_tag) {
    constexpr bool REV = decltype(rev_tag)::value;
    constexpr int NEWI = REV ? 0 : NKL - 1;
    auto seq = [&](int it) { return REV ? blk0 + TOT - 1 - it : blk0 + it; };
    // first query of the run that block `blk` belongs to
    auto run_q = [&](int blk) { return MULTI ? (blk & ~(SB - 1)) * TILE_Q : blk0 * TILE_Q; };
    auto request = [&](Stage &sg, int blk) {
        const int q0 = blk * TILE_Q;
        load_block(Qb, q0, sg.q, nt_q);
        const int row0 = leaf_row0(blk - NBW + NEWI);
        load_block(Kb, row0, sg.k, nt_leaf);
        load_block(Vb, row0, sg.v, nt_leafv);
        load_near(Kb, q0, sg.kt);
        load_near(Vb, q0, sg.vt);
    };

    // requests run AHEAD blocks in front of the computation
    constexpr int AHEAD = (D <= 64) ? 2 : 1;
    Stage st[SB];

    // ---- per-strip operands: far tree block, leaf blocks carried into the first query block ----
    // Everything the strip's first block needs is requested before anything is consumed, in
    // the order of use (loads return in order): one memory round trip for the prologue.
    u32x4_t far_k[NLD], far_v[NLD];
    load_far(Kb, run_q(seq(0)), far_k);
    load_far(Vb, run_q(seq(0)), far_v);
    far_biases(run_q(seq(0)));
    u32x4_t halo_k[NKL][NLD], halo_v[NKL][NLD];
#pragma unroll
    for (int c = 0; c < NKL; ++c) {
        if (c == NEWI) continue;
        const int row0 = leaf_row0(seq(0) - NBW + c);
        load_block(Kb, row0, halo_k[c], nt_halo);
        load_block(Vb, row0, halo_v[c], nt_halo);
    }
#pragma unroll
    for (int i = 0; i < AHEAD && i < SB; ++i) request(st[i], seq(i));

    u32x4_t Ku[KS];
    u32x2_t Vu[NJ];
    auto far_operands = [&]() {
        u32x4_t vop[KS];
        lds_put(0, far_k);
        lds_put(1, far_v);
        lds_get(0, Ku);
        lds_get(1, vop);
        transpose_v(vop, Vu);
    };
    far_operands();
    u32x4_t Kl[NKL][KS];
    u32x2_t Vl[NKL][NJ];
#pragma unroll
    for (int c = 0; c < NKL; ++c) {
        if (c == NEWI) continue;
        u32x4_t vop[KS];
        lds_put(2, halo_k[c]);
        lds_put(3, halo_v[c]);
        lds_get(2, Kl[c]);
        lds_get(3, vop);
        transpose_v(vop, Vl[c]);
    }

    // always_tag: `next_blk` exists, its request is unconditional.  (In a ring of stages a request
    // under a run-time condition keeps the stage's previous contents alive as the other arm.)
    auto process = [&](Stage &sg, int blk, Stage &nsg, int next_blk, auto always_tag) {
        const int q0 = blk * TILE_Q;
        // rows -> MFMA operand pieces
        u32x4_t Qf[KS], Vn[KS], Kt[KS], Vtn[KS];
        lds_put(0, sg.q);
        lds_put(1, sg.k);
        lds_put(2, sg.v);
        lds_put(3, sg.kt);
        lds_put(4, sg.vt);
        // this block's raw registers are consumed: request a later block's
        if (decltype(always_tag)::value || next_blk >= 0) request(nsg, next_blk);
        lds_get(0, Qf);
        lds_get(1, Kl[NEWI]);
        lds_get(2, Vn);
        lds_get(3, Kt);
        lds_get(4, Vtn);

        // scores, transposed: acc[i] = <key 4g+i of the block, query r16>
        f32x4 accL[NKL], accT, accU;
#pragma unroll
        for (int c = 0; c < NKL; ++c) {
            accL[c] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) accL[c] = M_::k32(Kl[c][ks], Qf[ks], accL[c]);
        }
        accT = f32x4{0.f, 0.f, 0.f, 0.f};
        accU = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            accT = M_::k32(Kt[ks], Qf[ks], accT);
            accU = M_::k32(Ku[ks], Qf[ks], accU);
        }
        // new value blocks into "lane = channel, regs = keys" form
        u32x2_t Vt[NJ];
        transpose_v(Vn, Vl[NEWI]);
        transpose_v(Vtn, Vt);

        float sc[NKL + 2][4];
        float mx = NEG_INF;
#pragma unroll
        for (int c = 0; c < NKL; ++c) {
            const int kb = blk - NBW + c;
            const bool inside = kb >= 0 && kb < NB;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = inside ? fmaf(accL[c][i], p.scale_log2e, biasL[c][i]) : NEG_INF;
                sc[c][i] = v;
                mx = fmaxf(mx, v);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float bias = biasT[i];
            if (CAUSAL) {
                const int lv = upT[i];
                if (lv >= 0 && ((q0 >> lv) & 1) == 0) bias = NEG_INF;
            }
            float v = fmaf(accT[i], p.scale_log2e, bias);
            sc[NKL][i] = v;
            mx = fmaxf(mx, v);
            float u = fmaf(accU[i], p.scale_log2e, biasU[i]);
            sc[NKL + 1][i] = u;
            mx = fmaxf(mx, u);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));

        float den = 0.f;
        u32x2_t P[NKL + 2];
        float ew[WT ? NKL + 2 : 1][4];
#pragma unroll
        for (int c = 0; c < NKL + 2; ++c) {
            float e[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                e[i] = __builtin_amdgcn_exp2f(sc[c][i] - mx);
                den += e[i];
                if constexpr (WT) ew[c][i] = e[i];
            }
            P[c] = u32x2_t{M_::pack(e[0], e[1]), M_::pack(e[2], e[3])};
        }
        den += __shfl_xor(den, 16, 64);
        den += __shfl_xor(den, 32, 64);
        const float inv = 1.0f / den;
        // what a backward pass needs to rebuild this query's weights without its whole row:
        // P = exp2(logit * log2(e) / sqrt(D) + bias - lse)
        // (a variant of its own: as a run-time branch it cost the widest variants their last
        // registers, B8 H8 N2048 D64 without the causal mask 20.4 -> 23.7 us)
        if constexpr (LSE) {
            if (g == 0) p.lse[((size_t)b * p.N + q0 + r16) * p.H + h] = mx + __builtin_amdgcn_logf(den);
        }

        if constexpr (WT) {
            // rows of weights in LDS: query r of the block at float offset r * S, in operand slots 1..4
            const int S = 2 * R + 1 + L;
            float *wrow = reinterpret_cast<float *>(lds + BLK_BYTES);
            for (int t = lane; t < TILE_Q * S; t += 64) wrow[t] = 0.f;
            __builtin_amdgcn_wave_barrier();
            float *mine = wrow + r16 * S;
#pragma unroll
            for (int c = 0; c < NKL; ++c) {
                const int kb = blk - NBW + c;
                if (kb < 0 || kb >= NB) continue;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int kl = 4 * g + i;
                    const int diff = TILE_Q * (c - NBW) + kl - r16;  // key row - query row
                    const bool win = diff >= -R && diff <= (CAUSAL ? 0 : R);
                    const bool sib = c == NBW && kl == (r16 ^ 1) && (!CAUSAL || (r16 & 1));
                    // a key that is both a window slot and the level-0 neighbour carries twice the weight
                    const float w = ew[c][i] * inv * ((win && sib) ? 0.5f : 1.0f);
                    if (win) mine[diff + R] = w;
                    if (sib) mine[2 * R + 1] = w;
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int sl = 4 * g + i;
                const int lvl = sl < 8 ? 1 : (sl < 12 ? 2 : (sl < 14 ? 3 : 4 + (sl - 14)));
                if (sc[NKL][i] > NEG_INF) mine[2 * R + 1 + lvl] = ew[NKL][i] * inv;
                const int ul = 6 + sl;
                if (sc[NKL + 1][i] > NEG_INF) mine[2 * R + 1 + ul] = ew[NKL + 1][i] * inv;
            }
            __builtin_amdgcn_wave_barrier();
            float *wg_out = p.weights + (((size_t)b * N + q0) * p.H + h) * S;
            for (int r = 0; r < TILE_Q; ++r)
                for (int t = lane; t < S; t += 64) wg_out[(size_t)r * p.H * S + t] = wrow[r * S + t];
            __builtin_amdgcn_wave_barrier();
        }

        // O^T tiles: this lane ends with channels [32ks + 8g, +8) of query r16; through LDS
        // back to whole rows, then streaming stores (the output is not read again here)
        unsigned char *oreg = lds + r16 * RB;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint32_t w[4];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const int j = 2 * ks + jj;
                f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < NKL; ++c) o = M_::k16(Vl[c][j], P[c], o);
                o = M_::k16(Vt[j], P[NKL], o);
                o = M_::k16(Vu[j], P[NKL + 1], o);
                w[2 * jj] = M_::pack(o[0] * inv, o[1] * inv);
                w[2 * jj + 1] = M_::pack(o[2] * inv, o[3] * inv);
            }
            *reinterpret_cast<u32x4_t *>(oreg + 16 * ((4 * ks + g) ^ op_swz)) = u32x4_t{w[0], w[1], w[2], w[3]};
        }
        {
            uint16_t *optr = Ob + (size_t)(q0 + lrow) * rs;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int row = i * RPI + lrow;
                const u32x4_t val = *reinterpret_cast<const u32x4_t *>(lds + row * RB + 16 * (lchk ^ swz(row)));
                if constexpr ((HSA_TILE_NT & 32) != 0) *reinterpret_cast<u32x4_t *>(optr + (size_t)(i * RPI) * rs) = val;
                else __builtin_nontemporal_store(val, reinterpret_cast<u32x4_t *>(optr + (size_t)(i * RPI) * rs));
            }
        }

        // slide the leaf window by one block
        if (REV) {
#pragma unroll
            for (int c = NKL - 1; c > 0; --c) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) Kl[c][ks] = Kl[c - 1][ks];
#pragma unroll
                for (int j = 0; j < NJ; ++j) Vl[c][j] = Vl[c - 1][j];
            }
        } else {
#pragma unroll
            for (int c = 0; c + 1 < NKL; ++c) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) Kl[c][ks] = Kl[c + 1][ks];
#pragma unroll
                for (int j = 0; j < NJ; ++j) Vl[c][j] = Vl[c + 1][j];
            }
        }
    };

    if constexpr (!MULTI) {
#pragma unroll
        for (int it = 0; it < SB; ++it) {
            if (it + AHEAD < SB) process(st[it], seq(it), st[it + AHEAD], seq(it + AHEAD), std::false_type{});
            else process(st[it], seq(it), st[it], -1, std::false_type{});
        }
    } else {
        // the stages are a ring that runs on across the runs; straight-line code like the single run
#pragma unroll
        for (int i = 0; i < TOT; ++i) {
            const int it = i % SB, r = i / SB;
            if (it == 0 && r > 0) {
                far_operands();
                far_biases(run_q(seq(i)));
            }
            if (it == SB - 2 && r + 1 < RUNS) {  // the next run's far block, two blocks ahead
                load_far(Kb, run_q(seq(SB * (r + 1))), far_k);
                load_far(Vb, run_q(seq(SB * (r + 1))), far_v);
            }
            if (i + AHEAD < TOT) process(st[it], seq(i), st[(it + AHEAD) % SB], seq(i + AHEAD), std::true_type{});
            else process(st[it], seq(i), st[it], -1, std::false_type{});
        }
    }
    };  // run

    if (p.alternate && (s & 1)) run(std::true_type{});
    else run(std::false_type{});
}

template <typename T, int D>
int attn_tile_launch_td(const TileParams &p, int nbw, bool causal, int sb, int wpb, hipStream_t st);
// the variant that also writes the softmax weights (one query block per wavefront)
template <typename T, int D>
int attn_tile_weights_launch_td(const TileParams &p, int nbw, bool causal, int wpb, hipStream_t st);
template <typename T, int D>
int attn_tile_lse_launch_td(const TileParams &p, int nbw, bool causal, int sb, int wpb, hipStream_t st);

}  // namespace hsa
