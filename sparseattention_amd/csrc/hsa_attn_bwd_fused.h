// Span attention backward in ONE pass over the strips (16-bit element types, canonical tables,
// window radius up to 16, or 32 with the causal mask), for callers that kept the forward's output
// and log-sum-exp.
//
// The two-pass split (hsa_attn_bwd_tile.h) reads Q, dO and the leaf K / V twice: once per query
// block for dQ, once per key block for dK / dV.  Here the wavefront that walks a strip of 4 to
// 32 query blocks also finishes dK / dV of the strip's own leaf key blocks: while a query block's
// operands are in registers, its contribution to each leaf key block it attends is evaluated in
// the second orientation (S[query, key], the queries in the MFMA contraction) and added to that
// key block's accumulators; a key block is complete once the query block after it has been done.
// What a strip's key blocks collect from the neighbouring strips' queries (the query block after
// the strip, and without the causal mask the one before it) is rebuilt from three pieces of saved
// state instead of being exchanged: the neighbour's Q and dO rows, the forward's log-sum-exp of
// those queries (P = exp2(logit - lse)) and delta = <dO, O> from the forward's output rows.
// So every row of Q, dO, K, V is fetched once per strip plus one halo block per strip (or two),
// nothing leaves as a partial result except the rows of the levels whose nodes collect from more
// than one strip (from level 7 with strips of four blocks, level 8 with eight, ... level 10 with 32: one
// fp32 row per strip and level, summed by a small second launch), and there are no atomics.
//
// What it costs: a wavefront carries the waiting key blocks' accumulators on top of everything the
// query pass holds: 300-360 registers at 64 channels per head, i.e. one wavefront per SIMD (two at
// 32 channels).  A block's rows therefore do not wait in registers: they are transferred from
// global memory straight into the wavefront's LDS staging area one block ahead (hsa_lds_dma.h) and
// read from there in operand form.  Measured at B8 H8 N2048 D64 with the causal mask, inputs
// rotated through 1 GiB, both launches: 50.8 us against 56.4 us for the two passes (strips of
// four blocks with the rows staged in registers: 56.0); with every load or every store removed
// the same instruction stream takes 44 / 47 us, with both removed 36: the wavefront's own
// instruction time is what is left to hide behind the memory system.
// Requesting two blocks ahead (into the area whose operands have just left for the registers) is
// slower: 52.4 us.
// Strips of 8, 16 or 32 blocks where that still fills every wavefront slot: one neighbour's block
// per 128 .. 512 queries instead of per 64, and the tree levels whose nodes collect from up to that
// many queries are final inside the strip (the far tree block changes every four blocks, the leaf
// key blocks' accumulators just carry on).
#pragma once

#include "hsa_attn_bwd_tile.h"
#include "hsa_lds_dma.h"

namespace hsa {

// blocks per strip forced through hsa_attn_bwd_saved_tune (0: automatic); defined in hsa_backward.hip
int &bwd_fused_strip_knob();

// Wavefronts per SIMD the fused pass is compiled for.
constexpr int bwd_fused_waves(int D, bool causal) { return D <= 32 ? 2 : 1; }

// NBW: 16-row blocks the window reaches to either side (window radius up to 16 NBW); two only with
// the causal mask (without it four key blocks would wait for their last query block at a time).
//
// SPLIT = 2 (heads of 128 channels): a wavefront cannot hold the accumulators of 128 channels, so
// two wavefronts share a (batch, strip, head): each owns 64 of the channels (its half of every
// row, its half of dQ, dK, dV) and computes its half of every dot product over the channels; the
// halves of the score and dP tiles are exchanged through LDS and added (both wavefronts then hold
// bit-identical sums, so their softmax statistics agree).  The two are a workgroup of their own,
// so that its barrier couples nobody else.
template <typename T, int D, bool CAUSAL, int SB, int NBW, int SPLIT>
__global__ void __launch_bounds__((SPLIT == 2 ? 2 : BWD_WPB) * 64)
__attribute__((amdgpu_waves_per_eu(bwd_fused_waves(D / SPLIT, CAUSAL))))
attn_bwd_tile_fused_kernel(BwdFusedParams fp) {
    static_assert(SPLIT == 1 || SPLIT == 2, "one wavefront per head, or two");
    constexpr int HD = D / SPLIT;                       // channels a wavefront owns
    constexpr int WPB = SPLIT == 2 ? 2 : BWD_WPB;       // wavefronts per workgroup
    using BT = BwdTile<T, HD>;
    using M_ = Mma<T>;
    static_assert(SB == 4 || SB == 8 || SB == 16 || SB == 32, "a strip is 1, 2, 4 or 8 runs of four blocks (the 64 leaves under a level-6 node)");
    static_assert(NBW == 1 || (NBW == 2 && CAUSAL), "window radius up to 16, or up to 32 with the causal mask");
    constexpr int FAR = BWD_STRIP;  // blocks that share the far tree block
    constexpr int KS = BT::KS, NJ = BT::NJ, RPI = BT::RPI, NLD = BT::NLD, CPR = BT::CPR;
    constexpr int NKL = CAUSAL ? NBW + 1 : 2 * NBW + 1;
    constexpr int NKB = NKL + 2;  // leaf blocks, near tree block, far tree block
    constexpr int LDS_SLOTS = 2;
    const BwdTileParams &p = fp.t;
    __shared__ __align__(16) unsigned char smem[WPB * LDS_SLOTS * BT::BLK_BYTES];
    __shared__ __align__(16) float carry_mem[WPB * 2 * HD];
    __shared__ __align__(16) float delta_mem[WPB * TILE_Q];
    // A block's rows (Q, dO, entering leaf K / V, near tree K / V: six 16-row blocks) go from
    // global memory straight into the wavefront's staging area, unpadded, with the pieces of each
    // row permuted (hsa_lds_dma.h).  One area is enough: a block's operands leave it for the
    // registers at the top of its iteration, and the next block's rows are requested right after.
    // The neighbour's query blocks after the strip (three staged blocks each) use the area once
    // the last block has left it; the one before the strip (no causal mask) has three blocks of
    // its own behind the area.
    constexpr int RB = 2 * HD, ARR = TILE_Q * RB, STG = 6 * ARR, RPB = 256 / RB;
    constexpr int WAVE_STG = STG + (CAUSAL ? 0 : 3 * ARR);
    __shared__ __align__(16) unsigned char stage_mem[WPB * WAVE_STG];
    // exchange of partial tiles between the two wavefronts of a head: two slots per wavefront,
    // used in turn, of XF4 16-byte values per lane
    constexpr int XF4 = 2 * NKB;
    __shared__ __align__(16) f32x4 xch_mem[SPLIT == 2 ? 2 * 2 * XF4 * 64 : 1];
    // dK^T / dV^T of the key blocks that wait for their remaining query blocks: NBW when causal,
    // 2 NBW otherwise; the slot of key block j is j mod NPARK
    constexpr int NPARK = CAUSAL ? NBW : 2 * NBW;
    static_assert(NPARK <= 2, "the slot is taken from the block's parity");

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // SPLIT == 2: the workgroup is one unit, its wavefronts the two channel halves
    const int unit = SPLIT == 2 ? bwd_xcd_remap((int)blockIdx.x, (int)gridDim.x)
                                : bwd_xcd_remap((int)blockIdx.x, (int)gridDim.x) * WPB + wave;
    const int half = SPLIT == 2 ? wave : 0;
    if (unit >= p.n_units) return;
    BT bt;
    bt.init(smem + wave * LDS_SLOTS * BT::BLK_BYTES);
    const int r16 = bt.r16, g = bt.g, lrow = bt.lrow, lchk = bt.lchk;
    float *carry = carry_mem + wave * 2 * HD;
    float *delta_lds = delta_mem + wave * TILE_Q;
    // slots are compile-time constants: plain registers
    f32x4 PK[NPARK][NJ], PV[NPARK][NJ];
    auto park_put = [&](int slot, const f32x4 (&tk)[NJ], const f32x4 (&tv)[NJ]) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) { PK[slot][j] = tk[j]; PV[slot][j] = tv[j]; }
    };
    auto park_get = [&](int slot, f32x4 (&tk)[NJ], f32x4 (&tv)[NJ]) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) { tk[j] = PK[slot][j]; tv[j] = PV[slot][j]; }
    };

    const int N = p.N, L = p.L, R = p.R, H = p.H;
    const int NB = N / TILE_Q, NS = NB / SB;
    const int h = unit % H;
    const int strip = (unit / H) % NS;
    const int b = unit / (H * NS);
    const int blk0 = strip * SB;
    const size_t rs = (size_t)H * D;
    const size_t qo = ((size_t)b * N * H + h) * D + half * HD, ko = ((size_t)b * p.M * H + h) * D + half * HD;
    const uint16_t *Q0 = p.q + qo, *G0 = p.dout + qo, *O0 = fp.out + qo;
    const uint16_t *K0 = p.k + ko, *V0 = p.v + ko;
    const uint16_t *Kb = K0 + 8 * lchk, *Vb = V0 + 8 * lchk;
    uint16_t *dKb = p.dk + ko + 8 * lchk;
    uint16_t *dVb = p.dv + ko + 8 * lchk;
    // key / value blocks in operand form: the leaf blocks a query block reaches (they slide along
    // the strip), the near tree block, the far tree block
    u32x4_t Kc[NKB][KS], Vc[NKB][KS];
    // adds the other wavefront's partial tiles to n of this wavefront's (SPLIT == 2 only; both
    // wavefronts of the workgroup get here the same number of times)
    int xslot = 0;
    auto exchange = [&](auto n_tag, f32x4 *vals) {
        constexpr int NX = decltype(n_tag)::value;
        static_assert(NX <= XF4, "more values than a slot holds");
        if constexpr (SPLIT == 2) {
            f32x4 *mine = xch_mem + ((wave * 2 + xslot) * XF4) * 64 + bt.lane;
            const f32x4 *other = xch_mem + (((wave ^ 1) * 2 + xslot) * XF4) * 64 + bt.lane;
#pragma unroll
            for (int k = 0; k < NX; ++k) mine[k * 64] = vals[k];
            lds_only_barrier();
#pragma unroll
            for (int k = 0; k < NX; ++k) vals[k] += other[k * 64];
            // the slot is written again two exchanges on, after the barrier of the next one,
            // which the other wavefront passes only with these reads behind it
            xslot ^= 1;
        }
    };
    // staging: the piece of its row a lane fetches (in elements), the lane's operand addresses for
    // the two contraction steps, and its own 16 bytes of a transfer
    const uint32_t stg_base = lds_address(stage_mem) + wave * WAVE_STG;
    int pc8[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) pc8[i] = 8 * (lchk ^ (((i * RPI + lrow) / RPB) % CPR));
    const uint32_t opa0 = stg_base + r16 * RB + ((g ^ ((r16 / RPB) % CPR)) << 4);
    const uint32_t opa1 = stg_base + r16 * RB + ((((4 + g) % CPR) ^ ((r16 / RPB) % CPR)) << 4);
    const uint32_t lin = stg_base + 16 * bt.lane;

    // ---- tree slot constants (same slot layout as the forward kernel) -------------------------
    int t_lvl[NLD], t_add[NLD], t_xor[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int sl = i * RPI + lrow;
        if (sl < 8) { t_lvl[i] = 1; t_add[i] = sl; t_xor[i] = 0; }
        else if (sl < 12) { t_lvl[i] = 2; t_add[i] = sl - 8; t_xor[i] = 0; }
        else if (sl < 14) { t_lvl[i] = 3; t_add[i] = sl - 12; t_xor[i] = 0; }
        else { t_lvl[i] = 4 + (sl - 14); t_add[i] = 0; t_xor[i] = 1; }
    }
    auto near_row = [&](int i, int q0) {
        return t_lvl[i] < L ? level_offset(N, t_lvl[i]) + (((q0 >> t_lvl[i]) + t_add[i]) ^ t_xor[i]) : -1;
    };
    auto slot_level = [](int sl, int &pl) {
        if (sl < 8) { pl = sl; return 1; }
        if (sl < 12) { pl = sl - 8; return 2; }
        if (sl < 14) { pl = sl - 12; return 3; }
        pl = -1;
        return 4 + (sl - 14);
    };
    // the far tree block (levels >= 6) of the run of four blocks that starts at query qr: one row
    // per level, the same for the 64 queries of the run
    float b1U[4], b2U[4];
    auto far_biases = [&](int qr) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ul1 = 6 + 4 * g + i;
            b1U[i] = (ul1 < L && (!CAUSAL || ((qr >> ul1) & 1))) ? 0.f : NEG_INF;
            const int ul2 = 6 + r16;
            b2U[i] = (ul2 < L && (!CAUSAL || ((qr >> ul2) & 1))) ? 0.f : NEG_INF;
        }
    };
    auto load_far = [&](int qr, u32x4_t (&rKu)[NLD], u32x4_t (&rVu)[NLD]) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int ul = 6 + i * RPI + lrow;
            const int ur = ul < L ? level_offset(N, ul) + ((qr >> ul) ^ 1) : qr;
            rKu[i] = *reinterpret_cast<const u32x4_t *>(Kb + (size_t)ur * rs);
            rVu[i] = *reinterpret_cast<const u32x4_t *>(Vb + (size_t)ur * rs);
        }
    };

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
    // transfers into the staging area at byte offset `area`
    auto dma_block = [&](const uint16_t *base0, int row0, uint32_t dst) {
        const uint16_t *ptr = base0 + (size_t)(row0 + lrow) * rs;
        if constexpr (NLD == 2) lds_dma16_pair(ptr + pc8[0], ptr + (size_t)RPI * rs + pc8[1], dst, dst + 1024);
        else lds_dma16(ptr + pc8[0], dst);
    };
    auto request_dma = [&](int area, int blk) {  // 6 * NLD transfers
        const uint32_t dst = stg_base + area;
        const int q0 = blk * TILE_Q;
        dma_block(Q0, q0, dst);
        dma_block(G0, q0, dst + ARR);
        const int row0 = leaf_row0(blk - NBW + NKL - 1);
        dma_block(K0, row0, dst + 2 * ARR);
        dma_block(V0, row0, dst + 3 * ARR);
        const uint16_t *kp[NLD], *vp[NLD];
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int tr = near_row(i, q0);
            kp[i] = K0 + (size_t)(tr < 0 ? q0 : tr) * rs + pc8[i];
            vp[i] = V0 + (size_t)(tr < 0 ? q0 : tr) * rs + pc8[i];
        }
        if constexpr (NLD == 2) {
            lds_dma16_pair(kp[0], kp[1], dst + 4 * ARR, dst + 4 * ARR + 1024);
            lds_dma16_pair(vp[0], vp[1], dst + 5 * ARR, dst + 5 * ARR + 1024);
        } else {
            lds_dma16(kp[0], dst + 4 * ARR);
            lds_dma16(vp[0], dst + 5 * ARR);
        }
    };
    // a neighbouring strip's query block: 3 * NLD transfers (Q, dO, forward output); the
    // log-sum-exp values of its queries (4g + i) go to registers and are requested first, so that
    // the wait that follows the transfers covers them
    auto request_halo_dma = [&](int area, int qb, float (&lse4)[4]) {
        qb = qb < 0 ? 0 : (qb >= NB ? NB - 1 : qb);
#pragma unroll
        for (int i = 0; i < 4; ++i) lse4[i] = fp.lse[((size_t)b * N + qb * TILE_Q + 4 * g + i) * H + h];
        asm volatile("" ::: "memory");
        const uint32_t dst = stg_base + area;
        dma_block(Q0, qb * TILE_Q, dst);
        dma_block(G0, qb * TILE_Q, dst + ARR);
        dma_block(O0, qb * TILE_Q, dst + 2 * ARR);
    };

    // One query block (operands Qf / Gf) against one leaf key block (operands Kf / Vf), second
    // orientation: this wavefront's part of S[query 4g+i, key r16] and dP[query, key] ...
    auto leaf_scores = [&](const u32x4_t (&Qf)[KS], const u32x4_t (&Gf)[KS], const u32x4_t (&Kf)[KS],
                           const u32x4_t (&Vf)[KS], f32x4 &a, f32x4 &d) {
        a = f32x4{0.f, 0.f, 0.f, 0.f};
        d = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            a = M_::k32(Qf[ks], Kf[ks], a);
            d = M_::k32(Gf[ks], Vf[ks], d);
        }
    };
    // ... and, from the complete tiles, the block's contribution to dK^T / dV^T of key block kb (the
    // queries' transposed operands, their lse and delta in the "regs = queries 4g+i" form)
    auto leaf_apply = [&](const f32x4 &a, const f32x4 &d, const u32x2_t (&QT)[NJ], const u32x2_t (&GT)[NJ],
                          const float (&lse4)[4], const float (&del4)[4], int qb, int kb, f32x4 (&tk)[NJ],
                          f32x4 (&tv)[NJ]) {
        float pp[4], ds[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ql = 4 * g + i;
            const int diff = (kb - qb) * TILE_Q + r16 - ql;  // key - query
            const bool win = diff >= -R && diff <= (CAUSAL ? 0 : R);
            const bool sib = qb == kb && r16 == (ql ^ 1) && (!CAUSAL || (ql & 1));
            const int cnt = (int)win + (int)sib;
            const float bias = cnt == 0 ? NEG_INF : (cnt == 2 ? 1.0f : 0.0f);
            pp[i] = __builtin_amdgcn_exp2f(fmaf(a[i], p.scale_log2e, bias) - lse4[i]);
            ds[i] = pp[i] * (d[i] - del4[i]) * p.scale;
        }
        const u32x2_t pk = u32x2_t{M_::pack(pp[0], pp[1]), M_::pack(pp[2], pp[3])};
        const u32x2_t dk = u32x2_t{M_::pack(ds[0], ds[1]), M_::pack(ds[2], ds[3])};
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            tk[j] = M_::k16(QT[j], dk, tk[j]);
            tv[j] = M_::k16(GT[j], pk, tv[j]);
        }
    };
    // A neighbouring strip's staged query block qb (area offset as a compile-time tag) against NK
    // of this strip's key blocks (operand slots e0 .. e0 + NK - 1, key blocks kb0 ...): rebuilt
    // from the block's Q and dO rows, its log-sum-exp and delta[q] = <dO[q], O[q]>.
    auto halo_block = [&](auto area_tag, auto nk_tag, const float (&lse4)[4], int qb, int e0, int kb0,
                          f32x4 (*tk)[NJ], f32x4 (*tv)[NJ]) {
        constexpr int OFF = decltype(area_tag)::value;
        constexpr int NK = decltype(nk_tag)::value;
        u32x4_t Qf[KS], Gf[KS], gw[NLD], ow[NLD];
        if constexpr (KS == 2) {
            lds_read16_x4<OFF, OFF, OFF + ARR, OFF + ARR>(opa0, opa1, opa0, opa1, Qf[0], Qf[1], Gf[0], Gf[1]);
            lds_read16_x4<OFF + ARR, OFF + ARR + 1024, OFF + 2 * ARR, OFF + 2 * ARR + 1024>(lin, lin, lin, lin, gw[0],
                                                                                          gw[1], ow[0], ow[1]);
        } else {
            lds_read16_x4<OFF, OFF + ARR, OFF + ARR, OFF + 2 * ARR>(opa0, opa0, lin, lin, Qf[0], Gf[0], gw[0], ow[0]);
        }
        // the exchanged values: the tiles of the NK key blocks and the rows' sums for delta
        f32x4 xv[2 * NK + 1];
        // the lanes that share a row sum their pieces (both rows carry the same permutation of
        // pieces); afterwards every lane of the row holds the sum over this wavefront's channels
        xv[2 * NK] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            float sd = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t a = gw[i][w], o = ow[i][w];
                sd = fmaf(to_float<T>((uint16_t)(a & 0xffffu)), to_float<T>((uint16_t)(o & 0xffffu)), sd);
                sd = fmaf(to_float<T>((uint16_t)(a >> 16)), to_float<T>((uint16_t)(o >> 16)), sd);
            }
#pragma unroll
            for (int m = 1; m < CPR; m <<= 1) sd += __shfl_xor(sd, m, 64);
            xv[2 * NK][i] = sd;
        }
#pragma unroll
        for (int e = 0; e < NK; ++e) leaf_scores(Qf, Gf, Kc[e0 + e], Vc[e0 + e], xv[2 * e], xv[2 * e + 1]);
        exchange(std::integral_constant<int, 2 * NK + 1>{}, xv);
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            if (lchk == 0) delta_lds[i * RPI + lrow] = xv[2 * NK][i];
        u32x2_t QT[NJ], GT[NJ];
        bt.transpose(Qf, QT);
        bt.transpose(Gf, GT);
        float del4[4];
        const f32x4 dl = *reinterpret_cast<const f32x4 *>(delta_lds + 4 * g);
#pragma unroll
        for (int i = 0; i < 4; ++i) del4[i] = dl[i];
#pragma unroll
        for (int e = 0; e < NK; ++e) leaf_apply(xv[2 * e], xv[2 * e + 1], QT, GT, lse4, del4, qb, kb0 + e, tk[e], tv[e]);
    };
    auto store_key_block = [&](int kb, const f32x4 (&tk)[NJ], const f32x4 (&tv)[NJ]) {
        bt.put_result(0, tk, 1.0f);
        bt.put_result(1, tv, 1.0f);
        uint16_t *dKp = dKb + (size_t)(kb * TILE_Q + lrow) * rs;
        uint16_t *dVp = dVb + (size_t)(kb * TILE_Q + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            *reinterpret_cast<u32x4_t *>(dKp + (size_t)(i * RPI) * rs) = bt.get_row_piece(0, i);
            *reinterpret_cast<u32x4_t *>(dVp + (size_t)(i * RPI) * rs) = bt.get_row_piece(1, i);
        }
    };

    // everything the first block needs is requested before anything is consumed
    u32x4_t rKu[NLD], rVu[NLD];  // the far block's rows on their way
    float halo_lse4[NBW][4];
    using Area0 = std::integral_constant<int, 0>;
    using AreaBefore = std::integral_constant<int, STG>;  // the block before the strip
    const bool left_halo = !CAUSAL && blk0 > 0;  // uniform
    {
        u32x4_t rKh[NKL][NLD], rVh[NKL][NLD];
        load_far(blk0 * TILE_Q, rKu, rVu);
#pragma unroll
        for (int c = 0; c + 1 < NKL; ++c) {
            load_block(Kb, leaf_row0(blk0 - NBW + c), rKh[c]);
            load_block(Vb, leaf_row0(blk0 - NBW + c), rVh[c]);
        }
        if constexpr (!CAUSAL) request_halo_dma(STG, blk0 - 1, halo_lse4[0]);
        request_dma(0, blk0);
#pragma unroll
        for (int c = 0; c + 1 < NKL; ++c) {
            bt.put(0, rKh[c]);
            bt.put(1, rVh[c]);
            bt.get(0, Kc[c]);
            bt.get(1, Vc[c]);
        }
    }
    if constexpr (!CAUSAL) {
        // the query block before the strip reaches the strip's first key block (leaf block blk0,
        // already here as the second carried-in block)
        f32x4 tk[NJ], tv[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) { tk[j] = f32x4{0.f, 0.f, 0.f, 0.f}; tv[j] = f32x4{0.f, 0.f, 0.f, 0.f}; }
        wait_vmem_all_but<6 * NLD>();  // everything older than the first block's transfers
        if (left_halo) halo_block(AreaBefore{}, std::integral_constant<int, 1>{}, halo_lse4[0], blk0 - 1, 1, blk0, &tk, &tv);
        park_put(0, tk, tv);
    }
    // partial rows of the far block, summed over a run of four blocks
    f32x4 fk[NJ], fv[NJ];

    // one query block; PAR = parity of `it`, the block's index within the strip
    auto body = [&](auto par_tag, const int it) {
        constexpr int PAR = decltype(par_tag)::value;
        const int blk = blk0 + it;
        const int q0 = blk * TILE_Q;
        if ((it & (FAR - 1)) == 0) {
            // a new run: its far block (requested a block ahead), nothing summed yet
            bt.put(0, rKu);
            bt.put(1, rVu);
            bt.get(0, Kc[NKL + 1]);
            bt.get(1, Vc[NKL + 1]);
            far_biases(q0);
            // a later run of the strip goes on summing the levels whose nodes it shares with the
            // runs before: slot r16 (level 6 + r16) starts over every 4 << r16 blocks
            if ((it & ((4 << r16) - 1)) == 0) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) { fk[j] = f32x4{0.f, 0.f, 0.f, 0.f}; fv[j] = f32x4{0.f, 0.f, 0.f, 0.f}; }
            }
        }
        u32x4_t Qf[KS], Gf[KS];
        // the next block's rows (after the last block: the neighbour's query block) into the other
        // area, whose reads finished an iteration ago; then everything older is here
        // This block's rows were requested an iteration ago, right after the block before had
        // left the area.  The counter the wait looks at retires loads, transfers and stores in the
        // order of issue, so the wait names how many younger operations may still be in flight:
        // the previous block's stores, which follow the request in program order.  Only stores
        // that are certainly issued are counted (dQ: NLD; the finished leaf key block: 2 NLD from
        // block NBW of the strip on; near tree rows: 2 NLD, some lane always has a row); counting
        // too few only waits longer.
        if (it == 0) wait_vmem_all_but<0>();
        else if (it <= NBW) wait_vmem_all_but<3 * NLD>();
        else wait_vmem_all_but<5 * NLD>();
        if constexpr (KS == 2) lds_read16_6x2<0, ARR>(opa0, opa1, Qf, Gf, Kc[NKL - 1], Vc[NKL - 1], Kc[NKL], Vc[NKL]);
        else lds_read16_6x1<0, ARR>(opa0, Qf, Gf, Kc[NKL - 1], Vc[NKL - 1], Kc[NKL], Vc[NKL]);
        // the operands are in registers: the area takes the next block's rows, after the last
        // block the neighbour's query blocks (three staged blocks each, in the halves of the area)
        if (it + 1 < SB) {
            request_dma(0, blk + 1);
        } else {
#pragma unroll
            for (int hq = 0; hq < NBW; ++hq) request_halo_dma(hq * 3 * ARR, blk0 + SB + hq, halo_lse4[hq]);
        }
        if constexpr (SB > FAR)
            if ((it & (FAR - 1)) == FAR - 1 && it + 1 < SB) load_far(q0 + TILE_Q, rKu, rVu);  // the next run's far block

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
        {
            f32x4 ad[2 * NKB];  // this wavefront's channels' part of the tiles, completed by the exchange
#pragma unroll
            for (int c = 0; c < NKB; ++c) {
                f32x4 a = {0.f, 0.f, 0.f, 0.f}, d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    a = M_::k32(Kc[c][ks], Qf[ks], a);
                    d = M_::k32(Vc[c][ks], Gf[ks], d);
                }
                ad[2 * c] = a;
                ad[2 * c + 1] = d;
            }
            exchange(std::integral_constant<int, 2 * NKB>{}, ad);
#pragma unroll
            for (int c = 0; c < NKB; ++c) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float bias = c < NKL ? biasL[c < NKL ? c : 0][i] : (c == NKL ? b1T[i] : b1U[i]);
                    sc[c][i] = fmaf(ad[2 * c][i], p.scale_log2e, bias);
                    dp[c][i] = ad[2 * c + 1][i];
                    mx = fmaxf(mx, sc[c][i]);
                }
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
            uint16_t *optr = p.dq + qo + 8 * lchk + (size_t)(q0 + lrow) * rs;
#pragma unroll
            for (int i = 0; i < NLD; ++i)
                *reinterpret_cast<u32x4_t *>(optr + (size_t)(i * RPI) * rs) = bt.get_row_piece(0, i);
        }

        // ---- orientation 2: dK^T, dV^T [channel, key] ---------------------------------------------------
        u32x2_t QT[NJ], GT[NJ];
        bt.transpose(Qf, QT);
        bt.transpose(Gf, GT);
        float lse4[4], del4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lse4[i] = __shfl(lse, 4 * g + i, 64);
            del4[i] = __shfl(delta, 4 * g + i, 64);
        }
        // second orientation, S[query 4g+i, key or slot r16] and dP[query, key]: every key block's
        // tiles first (this wavefront's channels' part, completed by the exchange)
        f32x4 ad2[2 * NKB];
#pragma unroll
        for (int c = 0; c < NKB; ++c) leaf_scores(Qf, Gf, Kc[c], Vc[c], ad2[2 * c], ad2[2 * c + 1]);
        exchange(std::integral_constant<int, 2 * NKB>{}, ad2);
        // the strip's own leaf key blocks this query block reaches, oldest first: the block before
        // the query block is complete afterwards and leaves; the others wait in registers
#pragma unroll
        for (int c = 0; c < NKL; ++c) {
            const int j = it - NBW + c;                                // key block within the strip
            const int SLOT = ((PAR + NBW + c) & 1) & (NPARK - 1);      // j % NPARK (NBW + it + c has j's parity)
            if (j >= 0 && j < SB) {
                f32x4 tk[NJ], tv[NJ];
                const bool fresh = c == NKL - 1 && (CAUSAL || j >= NBW);  // nobody has contributed yet
                if (fresh) {
#pragma unroll
                    for (int jj = 0; jj < NJ; ++jj) { tk[jj] = f32x4{0.f, 0.f, 0.f, 0.f}; tv[jj] = f32x4{0.f, 0.f, 0.f, 0.f}; }
                } else {
                    park_get(SLOT, tk, tv);
                }
                leaf_apply(ad2[2 * c], ad2[2 * c + 1], QT, GT, lse4, del4, blk, blk0 + j, tk, tv);
                if (c == 0) store_key_block(blk0 + j, tk, tv);
                else park_put(SLOT, tk, tv);
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int c = NKL + t;
            const f32x4 a = ad2[2 * c], d = ad2[2 * c + 1];  // S[query 4g+i, slot r16], dP[query, slot]
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
                // a level-5 node collects from the two blocks under its sibling, both this
                // wavefront's: the even block parks its row, the odd block adds it: final
                if (r16 == 15) {
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        const int ch = 32 * (j >> 1) + 8 * g + 4 * (j & 1);
                        if constexpr (PAR == 1) {
                            const f32x4 ck = *reinterpret_cast<const f32x4 *>(carry + ch);
                            const f32x4 cv = *reinterpret_cast<const f32x4 *>(carry + HD + ch);
                            tk[j] += ck;
                            tv[j] += cv;
                        } else {
                            *reinterpret_cast<f32x4 *>(carry + ch) = tk[j];
                            *reinterpret_cast<f32x4 *>(carry + HD + ch) = tv[j];
                        }
                    }
                }
                constexpr bool five_final = PAR == 1;
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

        // levels >= 6.  The node of level 6 + r collects from the 4 << r blocks under its sibling:
        // where the strip holds all of them (level 6: a run of four blocks, level 7: eight, ...) the
        // row is final when the last of them ends here and goes straight to dK / dV (zeros where
        // the causal mask leaves the node to nobody: the probabilities were zero).  The levels above
        // have several strips under the sibling: partial rows, laid out per run of four blocks and
        // stored with the strip's last block in the strip's first run, summed by the second launch.
        if ((it & (FAR - 1)) == FAR - 1) {
            const int lvl = 6 + r16;
            const int LF = L - 6;
            const bool final_row = ((it + 1) & ((4 << r16) - 1)) == 0;  // never for 4 << r16 > SB
            if (lvl < L && (final_row || it == SB - 1)) {
                if (final_row) {
                    const int node = (blk >> (lvl - 4)) ^ 1;
                    const size_t ro = ko + (size_t)(level_offset(N, lvl) + node) * rs;
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        const int ch = 32 * (j >> 1) + 8 * g + 4 * (j & 1);
                        *reinterpret_cast<u32x2_t *>(p.dk + ro + ch) =
                            u32x2_t{M_::pack(fk[j][0], fk[j][1]), M_::pack(fk[j][2], fk[j][3])};
                        *reinterpret_cast<u32x2_t *>(p.dv + ro + ch) =
                            u32x2_t{M_::pack(fv[j][0], fv[j][1]), M_::pack(fv[j][2], fv[j][3])};
                    }
                } else {
                    const int NR = NB / FAR;
                    float *far = p.partial + 2 * (size_t)p.B * NB * H * 2 * D;
                    const size_t po = ((((size_t)b * NR + blk0 / FAR) * H + h) * LF + (lvl - 6)) * D;
                    float *pkp = far + po + half * HD;
                    float *pvp = far + (size_t)p.B * NR * H * LF * D + po + half * HD;
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        const int ch = 32 * (j >> 1) + 8 * g + 4 * (j & 1);
                        *reinterpret_cast<f32x4 *>(pkp + ch) = fk[j];
                        *reinterpret_cast<f32x4 *>(pvp + ch) = fv[j];
                    }
                }
            }
        }

        // slide the leaf window by one block
#pragma unroll
        for (int c = 0; c + 1 < NKL; ++c) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) { Kc[c][ks] = Kc[c + 1][ks]; Vc[c][ks] = Vc[c + 1][ks]; }
        }
    };

    if constexpr (SB == FAR) {
#pragma unroll
        for (int ip = 0; ip < SB / 2; ++ip) {
            body(std::integral_constant<int, 0>{}, 2 * ip);
            body(std::integral_constant<int, 1>{}, 2 * ip + 1);
        }
    } else {
#pragma unroll 1  // unrolled it is slower (53.6 against 52.2 us at B8 H8 N2048 D64)
        for (int ip = 0; ip < SB / 2; ++ip) {
            body(std::integral_constant<int, 0>{}, 2 * ip);
            body(std::integral_constant<int, 1>{}, 2 * ip + 1);
        }
    }

    // the strip's last NBW key blocks: the query blocks after the strip reach them (their operands
    // sit in the first slots after the last slide; the neighbour's block hq reaches the last
    // NBW - hq of them)
    {
        static_assert(SB % 2 == 0, "the neighbour's blocks are staged in the first area");
        f32x4 tk[NBW][NJ], tv[NBW][NJ];
#pragma unroll
        for (int e = 0; e < NBW; ++e) park_get(((SB - NBW + e) & 1) & (NPARK - 1), tk[e], tv[e]);
        wait_vmem_all_but<0>();
        if (blk0 + SB < NB)  // uniform; the sequence's block count is a multiple of the strip's, so all NBW exist
            halo_block(Area0{}, std::integral_constant<int, NBW>{}, halo_lse4[0], blk0 + SB, 0, blk0 + SB - NBW, tk, tv);
        if constexpr (NBW == 2) {
            if (blk0 + SB < NB)
                halo_block(std::integral_constant<int, 3 * ARR>{}, std::integral_constant<int, 1>{}, halo_lse4[NBW - 1],
                           blk0 + SB + 1, 1, blk0 + SB - 1, tk + 1, tv + 1);
        }
#pragma unroll
        for (int e = 0; e < NBW; ++e) store_key_block(blk0 + SB - NBW + e, tk[e], tv[e]);
    }
}

// the rows of the levels no strip finishes alone (from level 7 with strips of four blocks up to
// from level 10 with strips of 32; and the root row, the rows nobody attends, the rows past 2N-1)
// from the strips' partial rows
template <typename T>
__global__ void __launch_bounds__(BWD_WPB * 64) attn_bwd_reduce_kernel(BwdTileParams p, int D) {
    using S = typename T::storage;
    bwd_reduce_rows<T, BWD_FUSED_RED_SPLIT>(p.partial, reinterpret_cast<S *>(p.dk), reinterpret_cast<S *>(p.dv), p.B, p.N,
                                            p.M, p.H, D, p.L, p.causal, p.red_first_row, p.red_lg_sb,
                                            (size_t)blockIdx.x * (BWD_WPB * 64) + threadIdx.x);
}

template <typename T, int D>
int attn_bwd_fused_launch_td(const BwdFusedParams &fp, bool causal, hipStream_t st);

// launches one variant: a workgroup is four wavefronts (heads), or the two halves of one head
template <typename T, int D, bool CAUSAL, int SB, int NBW>
static int bwd_fused_launch_one(const BwdFusedParams &q, hipStream_t st) {
    constexpr int SPLIT = D > 64 ? 2 : 1;
    constexpr int WPB = SPLIT == 2 ? 2 : BWD_WPB;
    const int nwg = SPLIT == 2 ? q.t.n_units : (q.t.n_units + WPB - 1) / WPB;
    attn_bwd_tile_fused_kernel<T, D, CAUSAL, SB, NBW, SPLIT><<<dim3(nwg), dim3(WPB * 64), 0, st>>>(q);
    return check_launch("attn_bwd_tile_fused_kernel");
}

template <typename T, int D, bool CAUSAL, int NBW>
static int bwd_fused_launch_sb(const BwdFusedParams &q, int sb, hipStream_t st) {
    switch (sb) {
        case 32: return bwd_fused_launch_one<T, D, CAUSAL, 32, NBW>(q, st);
        case 16: return bwd_fused_launch_one<T, D, CAUSAL, 16, NBW>(q, st);
        case 8: return bwd_fused_launch_one<T, D, CAUSAL, 8, NBW>(q, st);
        default: return bwd_fused_launch_one<T, D, CAUSAL, 4, NBW>(q, st);
    }
}

#define HSA_BWD_FUSED_INSTANTIATE(T, D)                                                                     \
    template <>                                                                                             \
    int attn_bwd_fused_launch_td<T, D>(const BwdFusedParams &fp, bool causal, hipStream_t st) {             \
        BwdFusedParams q = fp;                                                                              \
        const int NB = fp.t.N / TILE_Q;                                                                     \
        /* the longest strips (8, 16, 32 blocks) whose wavefronts still fill the chip once (one per SIMD */ \
        /* on 256 CUs): fewer halo blocks, more tree levels final inside the strip.  Measured (us, strips */ \
        /* of 8 / 16 / 32): B8 H8 N4096 D64 93 / 88 / 119, B8 H8 N8192 D64 180 / 173 / 166, B1 H16 N65536 */ \
        /* D64 348 / 327 / 317, B1 H16 N65536 D128 R32 734 / 679 / 657, B1 H16 N16384 D64 92.6 / 94.2 / 120 */ \
        const long waves8 = (long)(fp.t.n_units / 8) * (D > 64 ? 2 : 1);                                    \
        const int knob = bwd_fused_strip_knob();                                                            \
        int sb = (NB % 8 == 0 && knob != 4 && (knob >= 8 || (D >= 64 && waves8 >= 1024))) ? 8 : 4;          \
        if (sb == 8 && NB % 16 == 0 && (knob >= 16 || (knob == 0 && waves8 >= 2 * 1024))) sb = 16;          \
        if (sb == 16 && NB % 32 == 0 && (knob >= 32 || (knob == 0 && waves8 >= 4 * 1024))) sb = 32;         \
        const int nbw = fp.t.R > TILE_Q ? 2 : 1;                                                            \
        if (nbw == 2 && !causal) return fail(HSA_ERR_UNSUPPORTED, "one-pass backward: window radius above 16 needs the causal mask"); \
        q.t.n_units = fp.t.n_units / sb;                                                                    \
        q.t.red_lg_sb = sb == 32 ? 5 : sb == 16 ? 4 : sb == 8 ? 3 : 2;                                      \
        {   /* the second launch starts above the levels the strips finish themselves */                    \
            int first = level_offset(fp.t.N, q.t.red_lg_sb + 5);                                            \
            if (first > 2 * fp.t.N - 2) first = 2 * fp.t.N - 2;                                             \
            const size_t threads = (size_t)fp.t.B * (fp.t.M - first) * fp.t.H * (D / 4) * BWD_FUSED_RED_SPLIT; \
            q.t.red_first_row = first;                                                                      \
            q.t.red_wgs = (int)((threads + BWD_WPB * 64 - 1) / (BWD_WPB * 64));                             \
        }                                                                                                   \
        int rc;                                                                                             \
        if (nbw == 2) rc = bwd_fused_launch_sb<T, D, true, 2>(q, sb, st);                                   \
        else if (causal) rc = bwd_fused_launch_sb<T, D, true, 1>(q, sb, st);                                \
        else rc = bwd_fused_launch_sb<T, D, false, 1>(q, sb, st);                                           \
        if (rc != HSA_OK || q.t.red_wgs == 0) return rc;                                                    \
        attn_bwd_reduce_kernel<T><<<q.t.red_wgs, BWD_WPB * 64, 0, st>>>(q.t, D);                            \
        return check_launch("attn_bwd_reduce_kernel");                                                      \
    }

}  // namespace hsa
