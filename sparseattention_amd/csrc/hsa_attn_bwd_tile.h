// Span attention backward, MFMA tile kernels (16-bit element types, canonical tree tables).
//
// Two launches, the flash-attention split adapted to the window + tree structure:
//
//  (A) query-stationary, one wavefront per (batch, head, 16-query block): recomputes the score
//      tiles S^T[key, query] exactly like the forward, then
//          dP^T = V_blk . dO_blk^T          delta[q] = sum_key P dP
//          dS^T = P (dP - delta) / sqrt(D)   dQ^T[ch, q] = K_blk^T . dS^T
//      and stores dQ plus two numbers per (query, head): the log2-domain log-sum-exp and delta.
//      The tree key blocks are also evaluated in the other orientation (S[query, slot]), which
//      puts the queries into the MFMA contraction: dK^T[ch, slot] = Q^T . dS, dV^T = dO^T . P.
//      Nodes of levels 1..4 are attended only from inside the block: their rows are final and
//      written directly.  A node of level l >= 5 collects from the 2^(l-4) blocks under its
//      sibling: a wavefront that walks a strip of four blocks finishes level 5 itself and sums
//      the levels above over its strip; what is left is stored as fp32 partial rows (per strip
//      and level >= 6, or per block and level >= 5 for strips of one block), and pass (B)'s
//      trailing workgroups sum each node's contiguous run (deterministic, no atomics).
//  (B) key-stationary, one wavefront per (batch, head, 16-leaf key block): loops over the query
//      blocks whose window reaches the key block, rebuilds P and dS from the saved statistics
//      and accumulates dK^T = Q^T . dS, dV^T = dO^T . P in registers.  Every leaf row of dK / dV
//      is written once; no atomics.
//
// Operand plumbing is the forward kernel's: row-contiguous 16-byte global accesses, per-wavefront
// LDS re-layout into MFMA operand order, transposed operands through an MFMA with a 0/1
// selection matrix.
#pragma once

#include "hsa_attn_tile.h"

namespace hsa {

struct BwdTileParams {
    const uint16_t *q, *k, *v, *dout;
    uint16_t *dq, *dk, *dv;
    float *stats;   // [B, N, H, 2]: log2-domain lse, delta
    float *partial; // [2, B, N/16, H, L-4, D] fp32 per-block partial rows of dK, dV for levels >= 4
    int B, N, M, H, L, R;
    int n_units;
    float scale_log2e, scale;
    // rows the key pass's trailing workgroups finish from the partial rows (none: red_wgs == 0)
    int causal, red_first_row, red_wgs, red_lg_sb;  // red_lg_sb: log2 of the query pass's blocks per strip
};

// the one-pass variant (hsa_attn_bwd_fused.h) also takes what the forward left behind
struct BwdFusedParams {
    BwdTileParams t;
    const uint16_t *out;  // forward output [B, N, H, D]
    const float *lse;     // forward log-sum-exp [B, N, H], log2 domain
};

constexpr int BWD_WPB = 4;  // wavefronts per workgroup
// threads that share one output row piece in the one-pass variant's second launch
constexpr int BWD_FUSED_RED_SPLIT = 8;

// Hardware hands consecutive workgroup ids to the 8 XCDs in turn; with this remap workgroups that
// are consecutive in the returned index run on the same XCD, so neighbouring strips (which share
// halo rows and upper tree nodes) share an L2.
__device__ __forceinline__ int bwd_xcd_remap(int wg, int nwg) {
    return (nwg & 7) == 0 ? (wg & 7) * (nwg >> 3) + (wg >> 3) : wg;
}

// Blocks one wavefront of either pass walks (1 only for sequences whose block count is no multiple
// of it): leaf blocks (query pass) or query blocks (key pass) slide along the strip in operand
// form, NBW+1 of them when causal, 2 NBW+1 otherwise.
constexpr int BWD_STRIP = 4;  // the reduction and the level-5 pairing assume four: a strip is the 64 leaves under a level-6 node
// Wavefronts per SIMD the query pass is compiled for: two (256 registers) where that holds its
// operands without spilling, which a strip with five sliding leaf blocks at D = 64 and every
// variant at D = 128 do not.
constexpr int bwd_query_waves(int D, int nkl, int sb) {
    return (nkl <= 5 && (D <= 32 || (D <= 64 && (nkl <= 3 || sb == 1)))) ? 2 : 1;
}

template <typename T, int D>
struct BwdTile {
    using M_ = Mma<T>;
    static constexpr int KS = D / 32, NJ = D / 16, CPR = D / 8, RPI = 64 / CPR, NLD = TILE_Q / RPI;
    // a block in LDS: rows back to back, the 16-byte pieces of row r at piece index p ^ swz(r)
    // (conflict-free from both sides, see hsa_attn_tile.h); slots keep the size of a padded block
    static constexpr int RB = D * 2, RPB = RB >= 256 ? 1 : 256 / RB, BLK_BYTES = TILE_Q * (RB + 16);
    __device__ static __forceinline__ int swz(int row) { return (row / RPB) % CPR; }

    int lane, r16, g, lrow, lchk, op_swz;
    unsigned char *lds;
    u32x4_t Pi[2];

    __device__ __forceinline__ void init(unsigned char *wave_lds) {
        lane = threadIdx.x & 63;
        r16 = lane & 15;
        g = lane >> 4;
        lrow = lane / CPR;
        lchk = lane % CPR;
        op_swz = swz(r16);
        lds = wave_lds;
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int e = 4 * jj + (r16 & 3);
            const uint32_t one = (g == (r16 >> 2)) ? (uint32_t)M_::kOne << (16 * (e & 1)) : 0u;
            const int wi = e >> 1;
            Pi[jj] = u32x4_t{wi == 0 ? one : 0u, wi == 1 ? one : 0u, wi == 2 ? one : 0u, wi == 3 ? one : 0u};
        }
    }
    // rows -> LDS -> operand pieces
    __device__ __forceinline__ void put(int slot, const u32x4_t (&raw)[NLD]) const {
        unsigned char *reg = lds + slot * BLK_BYTES;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int row = i * RPI + lrow;
            *reinterpret_cast<u32x4_t *>(reg + row * RB + 16 * (lchk ^ swz(row))) = raw[i];
        }
    }
    __device__ __forceinline__ void get(int slot, u32x4_t (&dst)[KS]) const {
        const unsigned char *reg = lds + slot * BLK_BYTES + r16 * RB;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dst[ks] = *reinterpret_cast<const u32x4_t *>(reg + 16 * ((4 * ks + g) ^ op_swz));
    }
    // operand rows -> "lane = channel, regs = rows" form
    __device__ __forceinline__ void transpose(const u32x4_t (&op)[KS], u32x2_t (&dst)[NJ]) const {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            f32x4 z = {0.f, 0.f, 0.f, 0.f};
            f32x4 r = M_::k32(op[j >> 1], Pi[j & 1], z);
            dst[j] = u32x2_t{M_::pack_exact(r[0], r[1]), M_::pack_exact(r[2], r[3])};
        }
    }
    // result tiles [channel, column] (this lane: column r16, channels 32ks+8g+4jj+i) -> packed
    // 16-bit pieces in LDS slot `slot`, one row per column
    __device__ __forceinline__ void put_result(int slot, const f32x4 (&t)[NJ], float mul) const {
        unsigned char *reg = lds + slot * BLK_BYTES + r16 * RB;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const f32x4 a = t[2 * ks], b = t[2 * ks + 1];
            *reinterpret_cast<u32x4_t *>(reg + 16 * ((4 * ks + g) ^ op_swz)) =
                u32x4_t{M_::pack(a[0] * mul, a[1] * mul), M_::pack(a[2] * mul, a[3] * mul),
                        M_::pack(b[0] * mul, b[1] * mul), M_::pack(b[2] * mul, b[3] * mul)};
        }
    }
    __device__ __forceinline__ u32x4_t get_row_piece(int slot, int i) const {
        const int row = i * RPI + lrow;
        return *reinterpret_cast<const u32x4_t *>(lds + slot * BLK_BYTES + row * RB + 16 * (lchk ^ swz(row)));
    }
};

// ---------------------------------------------------------------------------------------------
// (A) query-stationary pass
// ---------------------------------------------------------------------------------------------
// A wavefront walks a strip of SB consecutive query blocks (SB * 16 <= 64 queries, aligned): the
// leaf key / value operands slide along the strip in registers (each leaf row is fetched once per
// strip), the far tree block (levels >= 6, the same nodes for the whole strip) is fetched once,
// and the partial rows it collects are summed over the strip's blocks before they are written.
// A block's rows are requested when its turn comes: holding the next block's rows in registers
// as well would cost the second wavefront per SIMD (more than 256 registers at D = 64), and two
// wavefronts that cover each other's waits are worth more than the prefetch.
//
// Partial rows (fp32): level 5 per query block when SB == 1, entry 1 of [2][B][N/16][H][2][D]
// (dK then dV; entry 0 and, for longer strips, the whole area stay unused); levels >= 6 per
// strip, [2][B][N/16/SB][H][L-6][D], right behind.
template <typename T, int D, int NBW, bool CAUSAL, int SB>
__global__ void __launch_bounds__(BWD_WPB * 64)
__attribute__((amdgpu_waves_per_eu(bwd_query_waves(D, CAUSAL ? NBW + 1 : 2 * NBW + 1, SB))))
attn_bwd_tile_query_kernel(BwdTileParams p) {
    using BT = BwdTile<T, D>;
    using M_ = Mma<T>;
    constexpr int KS = BT::KS, NJ = BT::NJ, RPI = BT::RPI, NLD = BT::NLD;
    constexpr int NKL = CAUSAL ? NBW + 1 : 2 * NBW + 1;
    constexpr int NKB = NKL + 2;  // leaf blocks, near tree block, far tree block
    constexpr int LDS_SLOTS = 4;
    __shared__ __align__(16) unsigned char smem[BWD_WPB * LDS_SLOTS * BT::BLK_BYTES];
    // level-5 rows (dK, dV) of an even block, kept until the odd block of the pair adds its own
    __shared__ __align__(16) float carry_mem[SB > 1 ? BWD_WPB * 2 * D : 4];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = bwd_xcd_remap((int)blockIdx.x, (int)gridDim.x) * BWD_WPB + wave;
    if (unit >= p.n_units) return;
    BT bt;
    bt.init(smem + wave * LDS_SLOTS * BT::BLK_BYTES);
    const int r16 = bt.r16, g = bt.g, lrow = bt.lrow, lchk = bt.lchk;
    float *carry = carry_mem + (SB > 1 ? wave * 2 * D : 0);

    const int N = p.N, L = p.L, R = p.R, H = p.H;
    const int NB = N / TILE_Q, NS = NB / SB;
    const int h = unit % H;
    const int strip = (unit / H) % NS;
    const int b = unit / (H * NS);
    const int blk0 = strip * SB;
    const int qs = blk0 * TILE_Q;  // first query of the strip
    const size_t rs = (size_t)H * D;
    const uint16_t *Qb = p.q + ((size_t)b * N * H + h) * D + 8 * lchk;
    const uint16_t *Gb = p.dout + ((size_t)b * N * H + h) * D + 8 * lchk;
    const uint16_t *Kb = p.k + ((size_t)b * p.M * H + h) * D + 8 * lchk;
    const uint16_t *Vb = p.v + ((size_t)b * p.M * H + h) * D + 8 * lchk;
    uint16_t *dKb = p.dk + ((size_t)b * p.M * H + h) * D + 8 * lchk;
    uint16_t *dVb = p.dv + ((size_t)b * p.M * H + h) * D + 8 * lchk;

    // ---- tree slot constants (same slot layout as the forward kernel) -------------------------
    int t_lvl[NLD], t_add[NLD], t_xor[NLD], u_row[NLD];  // rows this lane fetches; u_row -1 = no such slot
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int sl = i * RPI + lrow;
        if (sl < 8) { t_lvl[i] = 1; t_add[i] = sl; t_xor[i] = 0; }
        else if (sl < 12) { t_lvl[i] = 2; t_add[i] = sl - 8; t_xor[i] = 0; }
        else if (sl < 14) { t_lvl[i] = 3; t_add[i] = sl - 12; t_xor[i] = 0; }
        else { t_lvl[i] = 4 + (sl - 14); t_add[i] = 0; t_xor[i] = 1; }
        const int ul = 6 + sl;
        u_row[i] = ul < L ? level_offset(N, ul) + ((qs >> ul) ^ 1) : -1;
    }
    auto near_row = [&](int i, int q0) {  // -1 = the slot's level does not exist
        return t_lvl[i] < L ? level_offset(N, t_lvl[i]) + (((q0 >> t_lvl[i]) + t_add[i]) ^ t_xor[i]) : -1;
    };
    auto slot_level = [](int sl, int &pl) {  // near slot -> level, position under the ancestor (-1: sibling slot)
        if (sl < 8) { pl = sl; return 1; }
        if (sl < 12) { pl = sl - 8; return 2; }
        if (sl < 14) { pl = sl - 12; return 3; }
        pl = -1;
        return 4 + (sl - 14);
    };
    // far block liveness in orientation 1 (lane = query r16, regs = slots 4g+i) and orientation 2
    // (lane = slot r16, regs = queries 4g+i): the same for every block of the strip
    float b1U[4], b2U[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ul1 = 6 + 4 * g + i;
        b1U[i] = (ul1 < L && (!CAUSAL || ((qs >> ul1) & 1))) ? 0.f : NEG_INF;
        const int ul2 = 6 + r16;
        b2U[i] = (ul2 < L && (!CAUSAL || ((qs >> ul2) & 1))) ? 0.f : NEG_INF;
    }

    // ---- loads ------------------------------------------------------------------------------
    auto load_block = [&](const uint16_t *base, int row0, u32x4_t (&dst)[NLD]) {
        const uint16_t *ptr = base + (size_t)(row0 + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) dst[i] = *reinterpret_cast<const u32x4_t *>(ptr + (size_t)(i * RPI) * rs);
    };
    auto leaf_row0 = [&](int kb) {
        kb = kb < 0 ? 0 : (kb >= NB ? NB - 1 : kb);
        return kb * TILE_Q;
    };
    struct Stage {
        u32x4_t q[NLD], g[NLD], k[NLD], v[NLD], kt[NLD], vt[NLD];
    };
    auto request = [&](Stage &sg, int blk) {
        const int q0 = blk * TILE_Q;
        load_block(Qb, q0, sg.q);
        load_block(Gb, q0, sg.g);
        const int row0 = leaf_row0(blk - NBW + NKL - 1);  // the leaf block that enters with this query block
        load_block(Kb, row0, sg.k);
        load_block(Vb, row0, sg.v);
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int tr = near_row(i, q0);
            sg.kt[i] = *reinterpret_cast<const u32x4_t *>(Kb + (size_t)(tr < 0 ? q0 : tr) * rs);
            sg.vt[i] = *reinterpret_cast<const u32x4_t *>(Vb + (size_t)(tr < 0 ? q0 : tr) * rs);
        }
    };

    // everything the first block needs is requested before anything is consumed
    u32x4_t Kc[NKB][KS], Vc[NKB][KS];
    Stage sg;
    {
        u32x4_t rKu[NLD], rVu[NLD], rKh[NKL][NLD], rVh[NKL][NLD];
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            rKu[i] = *reinterpret_cast<const u32x4_t *>(Kb + (size_t)(u_row[i] < 0 ? qs : u_row[i]) * rs);
            rVu[i] = *reinterpret_cast<const u32x4_t *>(Vb + (size_t)(u_row[i] < 0 ? qs : u_row[i]) * rs);
        }
#pragma unroll
        for (int c = 0; c + 1 < NKL; ++c) {
            load_block(Kb, leaf_row0(blk0 - NBW + c), rKh[c]);
            load_block(Vb, leaf_row0(blk0 - NBW + c), rVh[c]);
        }
        request(sg, blk0);
        bt.put(2, rKu);
        bt.put(3, rVu);
        bt.get(2, Kc[NKL + 1]);
        bt.get(3, Vc[NKL + 1]);
#pragma unroll
        for (int c = 0; c + 1 < NKL; ++c) {
            bt.put(2, rKh[c]);
            bt.put(3, rVh[c]);
            bt.get(2, Kc[c]);
            bt.get(3, Vc[c]);
        }
    }
    // partial rows of the far block, summed over the strip
    f32x4 fk[NJ], fv[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { fk[j] = f32x4{0.f, 0.f, 0.f, 0.f}; fv[j] = f32x4{0.f, 0.f, 0.f, 0.f}; }

#pragma unroll
    for (int it = 0; it < SB; ++it) {
        const int blk = blk0 + it;
        const int q0 = blk * TILE_Q;
        if (it > 0) request(sg, blk);
        // rows -> operand pieces
        u32x4_t Qf[KS], Gf[KS];
        bt.put(0, sg.q);
        bt.put(1, sg.g);
        bt.put(2, sg.k);
        bt.put(3, sg.v);
        bt.get(0, Qf);
        bt.get(1, Gf);
        bt.get(2, Kc[NKL - 1]);
        bt.get(3, Vc[NKL - 1]);
        bt.put(2, sg.kt);
        bt.put(3, sg.vt);
        bt.get(2, Kc[NKL]);
        bt.get(3, Vc[NKL]);

        // liveness of the near block and of the leaf blocks for this query block
        int t_row[NLD];
#pragma unroll
        for (int i = 0; i < NLD; ++i) t_row[i] = near_row(i, q0);
        float b1T[4], b2T[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            {
                int pl;
                const int lvl = slot_level(4 * g + i, pl);
                const bool live = pl >= 0 ? (pl == ((r16 >> lvl) ^ 1) && (!CAUSAL || ((r16 >> lvl) & 1)))
                                          : (lvl < L && (!CAUSAL || ((q0 >> lvl) & 1)));
                b1T[i] = live ? 0.f : NEG_INF;
            }
            {
                int pl;
                const int lvl = slot_level(r16, pl);
                const int ql = 4 * g + i;
                const bool live = pl >= 0 ? (pl == ((ql >> lvl) ^ 1) && (!CAUSAL || ((ql >> lvl) & 1)))
                                          : (lvl < L && (!CAUSAL || ((q0 >> lvl) & 1)));
                b2T[i] = live ? 0.f : NEG_INF;
            }
        }
        float biasL[NKL][4];
#pragma unroll
        for (int c = 0; c < NKL; ++c) {
            const int dlt = TILE_Q * (c - NBW);
            const int kb = blk - NBW + c;
            const bool inside = kb >= 0 && kb < NB;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int kl = 4 * g + i;
                const int diff = dlt + kl - r16;
                const bool win = diff >= -R && diff <= (CAUSAL ? 0 : R);
                const bool sib = dlt == 0 && kl == (r16 ^ 1) && (!CAUSAL || (r16 & 1));
                const int cnt = (int)win + (int)sib;
                biasL[c][i] = (!inside || cnt == 0) ? NEG_INF : (cnt == 2 ? 1.0f : 0.0f);
            }
        }

        // ---- orientation 1: S^T, dP^T [key, query] ---------------------------------------------------
        float sc[NKB][4], dp[NKB][4];
        float mx = NEG_INF;
#pragma unroll
        for (int c = 0; c < NKB; ++c) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                a = M_::k32(Kc[c][ks], Qf[ks], a);
                d = M_::k32(Vc[c][ks], Gf[ks], d);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float bias = c < NKL ? biasL[c < NKL ? c : 0][i] : (c == NKL ? b1T[i] : b1U[i]);
                sc[c][i] = fmaf(a[i], p.scale_log2e, bias);
                dp[c][i] = d[i];
                mx = fmaxf(mx, sc[c][i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        float den = 0.f;
#pragma unroll
        for (int c = 0; c < NKB; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sc[c][i] = __builtin_amdgcn_exp2f(sc[c][i] - mx);
                den += sc[c][i];
            }
        den += __shfl_xor(den, 16, 64);
        den += __shfl_xor(den, 32, 64);
        const float inv = 1.0f / den;
        float delta = 0.f;
#pragma unroll
        for (int c = 0; c < NKB; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sc[c][i] *= inv;  // P
                delta = fmaf(sc[c][i], dp[c][i], delta);
            }
        delta += __shfl_xor(delta, 16, 64);
        delta += __shfl_xor(delta, 32, 64);
        const float lse = mx + __builtin_amdgcn_logf(den);  // log2 domain: P = exp2(s' - lse)
        if (g == 0) {
            float *stp = p.stats + (((size_t)b * N + q0 + r16) * H + h) * 2;
            stp[0] = lse;
            stp[1] = delta;
        }

        // ---- dQ^T = sum_c K_c^T . dS_c^T ---------------------------------------------------------------
        {
            f32x4 acc[NJ];
#pragma unroll
            for (int j = 0; j < NJ; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NKB; ++c) {
                u32x2_t KT[NJ];
                bt.transpose(Kc[c], KT);
                float ds[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) ds[i] = sc[c][i] * (dp[c][i] - delta) * p.scale;
                const u32x2_t dsp = u32x2_t{M_::pack(ds[0], ds[1]), M_::pack(ds[2], ds[3])};
#pragma unroll
                for (int j = 0; j < NJ; ++j) acc[j] = M_::k16(KT[j], dsp, acc[j]);
            }
            bt.put_result(0, acc, 1.0f);
            uint16_t *optr = p.dq + ((size_t)b * N * H + h) * D + 8 * lchk + (size_t)(q0 + lrow) * rs;
#pragma unroll
            for (int i = 0; i < NLD; ++i)
                *reinterpret_cast<u32x4_t *>(optr + (size_t)(i * RPI) * rs) = bt.get_row_piece(0, i);
        }

        // ---- orientation 2 for the tree blocks: dK^T, dV^T [channel, slot] ------------------------------
        u32x2_t QT[NJ], GT[NJ];
        bt.transpose(Qf, QT);
        bt.transpose(Gf, GT);
        float lse4[4], del4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lse4[i] = __shfl(lse, 4 * g + i, 64);
            del4[i] = __shfl(delta, 4 * g + i, 64);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int c = NKL + t;
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                a = M_::k32(Qf[ks], Kc[c][ks], a);   // S[query 4g+i, slot r16]
                d = M_::k32(Gf[ks], Vc[c][ks], d);   // dP[query, slot]
            }
            float pp[4], ds[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float bias = t == 0 ? b2T[i] : b2U[i];
                pp[i] = __builtin_amdgcn_exp2f(fmaf(a[i], p.scale_log2e, bias) - lse4[i]);
                ds[i] = pp[i] * (d[i] - del4[i]) * p.scale;
            }
            const u32x2_t pk = u32x2_t{M_::pack(pp[0], pp[1]), M_::pack(pp[2], pp[3])};
            const u32x2_t dk = u32x2_t{M_::pack(ds[0], ds[1]), M_::pack(ds[2], ds[3])};
            if (t == 0) {
                f32x4 tk[NJ], tv[NJ];
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    f32x4 z = {0.f, 0.f, 0.f, 0.f};
                    tk[j] = M_::k16(QT[j], dk, z);
                    tv[j] = M_::k16(GT[j], pk, z);
                }
                // A level-5 node collects from the two blocks under its sibling.  In a strip both
                // are this wavefront's: the even block parks its row, the odd block adds it and
                // the sum is final.  A strip of one block stores a partial row instead.
                bool five_final = false;
                if constexpr (SB > 1) {
                    if (r16 == 15) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j) {
                            const int ch = 32 * (j >> 1) + 8 * g + 4 * (j & 1);
                            if (it & 1) {
                                const f32x4 ck = *reinterpret_cast<const f32x4 *>(carry + ch);
                                const f32x4 cv = *reinterpret_cast<const f32x4 *>(carry + D + ch);
                                tk[j] += ck;
                                tv[j] += cv;
                            } else {
                                *reinterpret_cast<f32x4 *>(carry + ch) = tk[j];
                                *reinterpret_cast<f32x4 *>(carry + D + ch) = tv[j];
                            }
                        }
                    }
                    five_final = (it & 1) != 0;
                } else if (r16 == 15 && 5 < L) {
                    const size_t po = ((((size_t)b * NB + blk) * H + h) * 2 + 1) * D;
                    float *pkp = p.partial + po;
                    float *pvp = p.partial + (size_t)p.B * NB * H * 2 * D + po;
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        const int ch = 32 * (j >> 1) + 8 * g + 4 * (j & 1);
                        *reinterpret_cast<f32x4 *>(pkp + ch) = tk[j];
                        *reinterpret_cast<f32x4 *>(pvp + ch) = tv[j];
                    }
                }
                // slots 0..14 (levels 1..4) are attended from inside the block only: rows written
                // directly, and so is the finished level-5 row
                bt.put_result(0, tk, 1.0f);
                bt.put_result(1, tv, 1.0f);
#pragma unroll
                for (int i = 0; i < NLD; ++i) {
                    const int sl = i * RPI + lrow;
                    if ((sl < 15 || five_final) && t_row[i] >= 0) {
                        *reinterpret_cast<u32x4_t *>(dKb + (size_t)t_row[i] * rs) = bt.get_row_piece(0, i);
                        *reinterpret_cast<u32x4_t *>(dVb + (size_t)t_row[i] * rs) = bt.get_row_piece(1, i);
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    fk[j] = M_::k16(QT[j], dk, fk[j]);
                    fv[j] = M_::k16(GT[j], pk, fv[j]);
                }
            }
        }

        // slide the leaf window by one block
#pragma unroll
        for (int c = 0; c + 1 < NKL; ++c) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) { Kc[c][ks] = Kc[c + 1][ks]; Vc[c][ks] = Vc[c + 1][ks]; }
        }
    }

    // levels >= 6: the strip's partial rows
    {
        const int lvl = 6 + r16;
        const int LF = L - 6;
        if (lvl < L) {
            float *far = p.partial + 2 * (size_t)p.B * NB * H * 2 * D;
            const size_t po = ((((size_t)b * NS + strip) * H + h) * LF + (lvl - 6)) * D;
            float *pkp = far + po;
            float *pvp = far + (size_t)p.B * NS * H * LF * D + po;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int ch = 32 * (j >> 1) + 8 * g + 4 * (j & 1);
                *reinterpret_cast<f32x4 *>(pkp + ch) = fk[j];
                *reinterpret_cast<f32x4 *>(pvp + ch) = fv[j];
            }
        }
    }
}

template <typename T, int SPLIT = 1>
__device__ __forceinline__ void bwd_reduce_rows(const float *__restrict__ partial, typename T::storage *__restrict__ dk,
                                                typename T::storage *__restrict__ dv, int B, int N, int M, int H, int D,
                                                int L, int causal, int first_row, int lg_sb, size_t t);

// ---------------------------------------------------------------------------------------------
// (B) key-stationary pass over the leaf key blocks
// ---------------------------------------------------------------------------------------------
// A wavefront walks SB consecutive key blocks; the query blocks whose window reaches a key block
// (NQB of them) slide along in registers in operand form, so each query / dO row is fetched once
// per strip instead of once per key block it touches.
// The last red_wgs workgroups of the grid do not take key blocks: they sum the query pass's
// partial rows into the upper tree levels' dK / dV rows (independent of the leaf rows this pass
// writes), which fills the chip while the key blocks' last loads and stores drain.
template <typename T, int D, int NBW, bool CAUSAL, int SB>
__global__ void __launch_bounds__(BWD_WPB * 64)
attn_bwd_tile_key_kernel(BwdTileParams p) {
    using BT = BwdTile<T, D>;
    using M_ = Mma<T>;
    constexpr int KS = BT::KS, NJ = BT::NJ, RPI = BT::RPI, NLD = BT::NLD;
    constexpr int NQB = CAUSAL ? NBW + 1 : 2 * NBW + 1;  // query blocks that reach a key block
    constexpr int QOFF = CAUSAL ? 0 : -NBW;              // first of them, relative to the key block
    constexpr int LDS_SLOTS = 4;
    __shared__ __align__(16) unsigned char smem[BWD_WPB * LDS_SLOTS * BT::BLK_BYTES];

    const int key_wgs = (int)gridDim.x - p.red_wgs;
    if ((int)blockIdx.x >= key_wgs) {
        using S = typename T::storage;
        bwd_reduce_rows<T>(p.partial, reinterpret_cast<S *>(p.dk), reinterpret_cast<S *>(p.dv), p.B, p.N, p.M, p.H, D,
                           p.L, p.causal, p.red_first_row, p.red_lg_sb,
                           (size_t)((int)blockIdx.x - key_wgs) * (BWD_WPB * 64) + threadIdx.x);
        return;
    }
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = bwd_xcd_remap((int)blockIdx.x, key_wgs) * BWD_WPB + wave;
    if (unit >= p.n_units) return;
    BT bt;
    bt.init(smem + wave * LDS_SLOTS * BT::BLK_BYTES);
    const int r16 = bt.r16, g = bt.g, lrow = bt.lrow, lchk = bt.lchk;

    const int N = p.N, R = p.R, H = p.H;
    const int NB = N / TILE_Q, NS = NB / SB;
    const int h = unit % H;
    const int strip = (unit / H) % NS;
    const int b = unit / (H * NS);
    const int kb0 = strip * SB;
    const size_t rs = (size_t)H * D;
    const uint16_t *Qb = p.q + ((size_t)b * N * H + h) * D + 8 * lchk;
    const uint16_t *Gb = p.dout + ((size_t)b * N * H + h) * D + 8 * lchk;
    const uint16_t *Kb = p.k + ((size_t)b * p.M * H + h) * D + 8 * lchk;
    const uint16_t *Vb = p.v + ((size_t)b * p.M * H + h) * D + 8 * lchk;

    auto load_block = [&](const uint16_t *base, int row0, u32x4_t (&dst)[NLD]) {
        const uint16_t *ptr = base + (size_t)(row0 + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) dst[i] = *reinterpret_cast<const u32x4_t *>(ptr + (size_t)(i * RPI) * rs);
    };
    auto clampb = [&](int qb) { return qb < 0 ? 0 : (qb >= NB ? NB - 1 : qb); };
    // a query block in the forms the key pass needs
    struct QBlock {
        u32x4_t Qf[KS], Gf[KS];
        u32x2_t QT[NJ], GT[NJ];
        float lse4[4], del4[4];
    };
    struct Stage {
        u32x4_t k[NLD], v[NLD], q[NLD], g[NLD];
        float lse4[4], del4[4];
    };
    auto request = [&](Stage &sg, int kb) {  // key block kb and the query block that enters with it
        load_block(Kb, kb * TILE_Q, sg.k);
        load_block(Vb, kb * TILE_Q, sg.v);
        const int qb = clampb(kb + QOFF + NQB - 1);
        load_block(Qb, qb * TILE_Q, sg.q);
        load_block(Gb, qb * TILE_Q, sg.g);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float *stp = p.stats + (((size_t)b * N + qb * TILE_Q + 4 * g + i) * H + h) * 2;
            sg.lse4[i] = stp[0];
            sg.del4[i] = stp[1];
        }
    };
    auto absorb = [&](QBlock &qq, const u32x4_t (&rq)[NLD], const u32x4_t (&rg)[NLD], const float (&l4)[4],
                      const float (&d4)[4]) {
        bt.put(2, rq);
        bt.put(3, rg);
        bt.get(2, qq.Qf);
        bt.get(3, qq.Gf);
        bt.transpose(qq.Qf, qq.QT);
        bt.transpose(qq.Gf, qq.GT);
#pragma unroll
        for (int i = 0; i < 4; ++i) { qq.lse4[i] = l4[i]; qq.del4[i] = d4[i]; }
    };

    QBlock qblk[NQB];
    Stage st[SB];
    {
        // the query blocks carried into the first key block, then the first stage
        u32x4_t rq[NQB][NLD], rg[NQB][NLD];
        float l4[NQB][4], d4[NQB][4];
#pragma unroll
        for (int c = 0; c + 1 < NQB; ++c) {
            const int qb = clampb(kb0 + QOFF + c);
            load_block(Qb, qb * TILE_Q, rq[c]);
            load_block(Gb, qb * TILE_Q, rg[c]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float *stp = p.stats + (((size_t)b * N + qb * TILE_Q + 4 * g + i) * H + h) * 2;
                l4[c][i] = stp[0];
                d4[c][i] = stp[1];
            }
        }
        request(st[0], kb0);
#pragma unroll
        for (int c = 0; c + 1 < NQB; ++c) absorb(qblk[c], rq[c], rg[c], l4[c], d4[c]);
    }

#pragma unroll
    for (int it = 0; it < SB; ++it) {
        const int kb = kb0 + it;
        const int k0 = kb * TILE_Q;
        Stage &sg = st[it];
        u32x4_t Kf[KS], Vf[KS];
        bt.put(0, sg.k);
        bt.put(1, sg.v);
        bt.get(0, Kf);
        bt.get(1, Vf);
        absorb(qblk[NQB - 1], sg.q, sg.g, sg.lse4, sg.del4);
        if (it + 1 < SB) request(st[it + 1 < SB ? it + 1 : it], kb + 1);

        f32x4 tk[NJ], tv[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) { tk[j] = f32x4{0.f, 0.f, 0.f, 0.f}; tv[j] = f32x4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
        for (int c = 0; c < NQB; ++c) {
            const int qb = kb + QOFF + c;
            const bool inside = qb >= 0 && qb < NB;  // uniform
            const QBlock &qq = qblk[c];
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                a = M_::k32(qq.Qf[ks], Kf[ks], a);  // S[query 4g+i of block qb, key r16]
                d = M_::k32(qq.Gf[ks], Vf[ks], d);
            }
            float pp[4], ds[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int ql = 4 * g + i;
                const int diff = (kb - qb) * TILE_Q + r16 - ql;  // key - query
                const bool win = diff >= -R && diff <= (CAUSAL ? 0 : R);
                const bool sib = qb == kb && r16 == (ql ^ 1) && (!CAUSAL || (ql & 1));
                const int cnt = (int)win + (int)sib;
                const float bias = (!inside || cnt == 0) ? NEG_INF : (cnt == 2 ? 1.0f : 0.0f);
                pp[i] = __builtin_amdgcn_exp2f(fmaf(a[i], p.scale_log2e, bias) - qq.lse4[i]);
                ds[i] = pp[i] * (d[i] - qq.del4[i]) * p.scale;
            }
            const u32x2_t pk = u32x2_t{M_::pack(pp[0], pp[1]), M_::pack(pp[2], pp[3])};
            const u32x2_t dk = u32x2_t{M_::pack(ds[0], ds[1]), M_::pack(ds[2], ds[3])};
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                tk[j] = M_::k16(qq.QT[j], dk, tk[j]);
                tv[j] = M_::k16(qq.GT[j], pk, tv[j]);
            }
        }
        bt.put_result(0, tk, 1.0f);
        bt.put_result(1, tv, 1.0f);
        uint16_t *dKp = p.dk + ((size_t)b * p.M * H + h) * D + 8 * lchk + (size_t)(k0 + lrow) * rs;
        uint16_t *dVp = p.dv + ((size_t)b * p.M * H + h) * D + 8 * lchk + (size_t)(k0 + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            *reinterpret_cast<u32x4_t *>(dKp + (size_t)(i * RPI) * rs) = bt.get_row_piece(0, i);
            *reinterpret_cast<u32x4_t *>(dVp + (size_t)(i * RPI) * rs) = bt.get_row_piece(1, i);
        }
        // slide the query blocks by one
#pragma unroll
        for (int c = 0; c + 1 < NQB; ++c) qblk[c] = qblk[c + 1];
    }
}

// Rows from first_row on (a level the query pass left unfinished, up to anything above row 2N-2):
// node (l, p) sums the partial rows of the query blocks (levels 4, 5) or strips (levels >= 6)
// under its sibling; nodes nobody attends (the root, right-hand nodes when causal, rows past
// 2N-1) get zeros.  SPLIT consecutive threads per (batch, row, head, four channels) share the
// partial rows of one output (the top levels have the most: one per strip of the sequence),
// index t.  lg_sb = log2 of the blocks per strip of the query pass.
template <typename T, int SPLIT>
__device__ __forceinline__ void bwd_reduce_rows(const float *__restrict__ partial, typename T::storage *__restrict__ dk,
                                                typename T::storage *__restrict__ dv, int B, int N, int M, int H, int D,
                                                int L, int causal, int first_row, int lg_sb, size_t t) {
    using S = typename T::storage;
    struct alignas(4 * sizeof(S)) Pack { S e[4]; };
    static_assert(SPLIT == 1 || SPLIT == 2 || SPLIT == 4 || SPLIT == 8, "lanes that share an output");
    const int sub = (int)(t % SPLIT);
    t /= SPLIT;
    const int D4 = D / 4;
    const size_t per_b = (size_t)(M - first_row) * H * D4;
    if (t >= (size_t)B * per_b) return;
    const int b = (int)(t / per_b);
    const size_t r = t % per_b;
    const int row = first_row + (int)(r / ((size_t)H * D4));
    const int h = (int)((r / D4) % H);
    const int d = 4 * (int)(r % D4);
    f32x4 vk = {0.f, 0.f, 0.f, 0.f}, vv = {0.f, 0.f, 0.f, 0.f};
    if (row < 2 * N - 2) {
        int lvl = 4;
        while (row >= level_offset(N, lvl + 1)) ++lvl;
        const int pidx = row - level_offset(N, lvl);
        if (!causal || (pidx & 1) == 0) {
            const int NB = N / TILE_Q;
            const int blk0 = (pidx ^ 1) << (lvl - 4);  // first query block under the sibling
            const float *pk, *pv;
            size_t stride;
            int n;
            if (lvl < 6) {
                n = 1 << (lvl - 4);
                stride = (size_t)H * 2 * D;
                pk = partial + (((size_t)b * NB + blk0) * H + h) * 2 * D + (size_t)(lvl - 4) * D + d;
                pv = pk + (size_t)B * NB * H * 2 * D;
            } else {
                // lg_sb >= 3 (the one-pass variant's strips of eight or more blocks): the area is laid out per
                // run of four blocks; level 6 has a row per run, the levels above one per strip, in
                // the strip's first run
                const int LF = L - 6;
                const int lgl = lg_sb >= 3 ? 2 : lg_sb;             // layout granularity
                const int lg = (lg_sb >= 3 && lvl == 6) ? 2 : lg_sb;  // blocks summed into one row
                const int NR = NB >> lgl;
                n = (1 << (lvl - 4)) >> lg;
                stride = ((size_t)H * LF * D) << (lg - lgl);
                const float *far = partial + 2 * (size_t)B * NB * H * 2 * D;
                pk = far + (((size_t)b * NR + (blk0 >> lgl)) * H + h) * LF * D + (size_t)(lvl - 6) * D + d;
                pv = pk + (size_t)B * NR * H * LF * D;
            }
            // eight independent 16-byte loads per tensor in flight per round trip
            int i = 0;
            if constexpr (SPLIT > 1) {
                for (i = sub; i + 3 * SPLIT < n; i += 4 * SPLIT) {
                    f32x4 a[4], c[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        a[u] = *reinterpret_cast<const f32x4 *>(pk + (size_t)(i + u * SPLIT) * stride);
                        c[u] = *reinterpret_cast<const f32x4 *>(pv + (size_t)(i + u * SPLIT) * stride);
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) { vk += a[u]; vv += c[u]; }
                }
                for (; i < n; i += SPLIT) {
                    vk += *reinterpret_cast<const f32x4 *>(pk + (size_t)i * stride);
                    vv += *reinterpret_cast<const f32x4 *>(pv + (size_t)i * stride);
                }
                i = n;
            }
            for (; i + 8 <= n; i += 8) {
                f32x4 a[8], c[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    a[u] = *reinterpret_cast<const f32x4 *>(pk + (size_t)(i + u) * stride);
                    c[u] = *reinterpret_cast<const f32x4 *>(pv + (size_t)(i + u) * stride);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) { vk += a[u]; vv += c[u]; }
            }
            for (; i < n; ++i) {
                vk += *reinterpret_cast<const f32x4 *>(pk + (size_t)i * stride);
                vv += *reinterpret_cast<const f32x4 *>(pv + (size_t)i * stride);
            }
        }
    }
    if constexpr (SPLIT > 1) {
        // the lanes of a group are neighbours in the wavefront and all of them get here
#pragma unroll
        for (int m = 1; m < SPLIT; m <<= 1)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                vk[u] += __shfl_xor(vk[u], m, 64);
                vv[u] += __shfl_xor(vv[u], m, 64);
            }
        if (sub != 0) return;
    }
    const size_t o = ((size_t)b * M + row) * H * D + (size_t)h * D + d;
    Pack ok, ov;
#pragma unroll
    for (int u = 0; u < 4; ++u) { ok.e[u] = from_float<T>(vk[u]); ov.e[u] = from_float<T>(vv[u]); }
    *reinterpret_cast<Pack *>(dk + o) = ok;
    *reinterpret_cast<Pack *>(dv + o) = ov;
}

}  // namespace hsa
