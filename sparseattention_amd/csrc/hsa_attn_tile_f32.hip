// Span attention forward, fp32 tensors, on the fp32 matrix cores (v_mfma_f32_16x16x4_f32).
//
// Same decomposition as the 16-bit tile kernel (hsa_attn_tile.h): a wavefront owns one
// (batch, head) and a strip of 1/2/4 consecutive 16-query blocks; per block the attended keys are
// NBW+1 (causal) or 2*NBW+1 leaf blocks, the "near" tree block (levels 1..5) and the "far" tree
// block (levels 6..L-1, one per strip); leaf operands slide along the strip in registers, global
// accesses are row-contiguous 16-byte pieces re-laid out through a private LDS region.
//
// What differs is the operand plumbing of the 4-deep fp32 MFMA (A: lane = (row r16, k = g), one
// float per step; result: lane = column r16, rows 4g..4g+3):
//  * S^T[key, query] = K Q^T.  The order of the contraction is free as long as both operands
//    agree, so lane (r16, g) holds the D/4 consecutive channels [g*D/4, (g+1)*D/4) of its row
//    (a few 16-byte LDS reads) and step s contracts channel g*D/4 + s of every lane group.
//  * O^T[channel, query] = V^T P^T.  The scores' result layout (lane = query, registers = keys
//    4g+i) is exactly the B operand of step i if that step contracts key 4g+i, so P never moves;
//    the A operand V^T[channel, key 4g+i] is read from the row-major LDS block transposed; column
//    r16 of output tile j stands for channel r16*D/16 + j, so a lane's values of one key row are
//    consecutive floats (one 16-byte read per row).
// Scores, softmax and accumulation are fp32 throughout; exp2 is the hardware instruction (1 ulp;
// its arguments are <= 0, so only results below 2^-126 differ from the library routine: they flush
// to zero) and the outputs are scaled by one correctly rounded reciprocal per query: errors of a
// few 1e-7 against the 1e-5 bar of the fp64 oracle.
#include "hsa_common.h"

#include <stdlib.h>
#include <type_traits>

namespace hsa {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int TQ = 16;            // queries per block
// wavefronts per workgroup: two per SIMD (256 registers each) where the variant fits, so that one
// wavefront's matrix work overlaps the other's loads; else one per SIMD (up to 512 registers)
template <int D, int NBW, bool CAUSAL> constexpr bool f32_fits_two_per_simd() { return D <= 32 || (D <= 64 && CAUSAL && NBW <= 1); }
// longest strip whose operands stay in registers
template <int D, int NBW, bool CAUSAL> constexpr int f32_max_strip() { return D <= 64 ? 4 : ((CAUSAL && NBW <= 1) ? 2 : 1); }
constexpr int F32_MAX_LEVELS = 22;
constexpr int F32_MAX_NBW = 2;
constexpr float NEG_INF_F = -__builtin_inff();

struct TileF32Params {
    const float *q, *k, *v;
    float *out;
    int B, N, M, H, L, R;
    int NS, n_units, xcd_swizzle;
    float scale_log2e;
};

template <int D, int NBW, bool CAUSAL, int SB, int F32_WPB>
__global__ void __launch_bounds__(F32_WPB * 64) attn_tile_f32_kernel(TileF32Params p) {
    constexpr int DS = D / 4;                           // contraction steps of QK^T
    constexpr int NJ = D / 16;                          // 16-channel output tiles
    constexpr int NKL = CAUSAL ? NBW + 1 : 2 * NBW + 1;  // leaf key blocks per query block
    constexpr int NEWC = NKL - 1;                       // the leaf block that enters each step
    constexpr int CPR = D / 4;                          // 16-byte pieces per head-row
    constexpr int RPI = 64 / CPR;                       // rows covered by one load instruction
    constexpr int NLD = TQ / RPI;                       // load instructions per 16-row block
    constexpr int PITCH = D * 4 + 16;                   // LDS row pitch in bytes
    constexpr int BLK_BYTES = TQ * PITCH;
    constexpr int WAVE_LDS = 3 * BLK_BYTES;             // three operand blocks at a time
    __shared__ __align__(16) unsigned char smem[F32_WPB * WAVE_LDS];

    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15, g = lane >> 4;
    const int lrow = lane / CPR, lchk = lane % CPR;
    int wg = blockIdx.x;
    const int nwg = gridDim.x;
    if (p.xcd_swizzle && (nwg & 7) == 0) wg = (wg & 7) * (nwg >> 3) + (wg >> 3);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = wg * F32_WPB + wave;
    if (unit >= p.n_units) return;
    const int h = unit % p.H;
    const int s = (unit / p.H) % p.NS;
    const int b = unit / (p.H * p.NS);
    unsigned char *lds = smem + wave * WAVE_LDS;

    const int N = p.N, L = p.L, R = p.R;
    const int NB = N / TQ;
    const int blk0 = s * SB;
    const size_t rs = (size_t)p.H * D;
    const float *Qb = p.q + ((size_t)b * N * p.H + h) * D + 4 * lchk;
    const float *Kb = p.k + ((size_t)b * p.M * p.H + h) * D + 4 * lchk;
    const float *Vb = p.v + ((size_t)b * p.M * p.H + h) * D + 4 * lchk;
    float *Ob = p.out + ((size_t)b * N * p.H + h) * D + 4 * lchk;

    // additive score bias of the leaf blocks (log2 of the multiplicity, -inf = not attended)
    float biasL[NKL][4];
#pragma unroll
    for (int c = 0; c < NKL; ++c) {
        const int dlt = TQ * (c - NBW);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kl = 4 * g + i;
            const int diff = dlt + kl - r16;
            const bool win = diff >= -R && diff <= (CAUSAL ? 0 : R);
            const bool sib = dlt == 0 && kl == (r16 ^ 1) && (!CAUSAL || (r16 & 1));
            const int cnt = (int)win + (int)sib;
            biasL[c][i] = cnt == 0 ? NEG_INF_F : (cnt == 2 ? 1.0f : 0.0f);
        }
    }
    // tree slots, as in the 16-bit kernel: near block = slots 0..7 level 1, 8..11 level 2,
    // 12..13 level 3 (nodes under the block's level-4 ancestor), 14 / 15 = siblings of the level-4 /
    // level-5 ancestors; far block slot u = sibling of the level-(6+u) ancestor
    int t_lvl[NLD], t_add[NLD], t_xor[NLD], t_off[NLD], u_lvl[NLD];
    bool t_valid[NLD], u_valid[NLD];
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
    float biasT[4];
    int upT[4];
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
        biasT[i] = live ? 0.0f : NEG_INF_F;
    }
    const int qs = blk0 * TQ;
    float biasU[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int lvl = 6 + 4 * g + i;
        biasU[i] = (lvl < L && (!CAUSAL || ((qs >> lvl) & 1))) ? 0.0f : NEG_INF_F;
    }

    // ---- loaders: raw[i] = piece lchk of row (i*RPI + lrow) of a 16-row block ---------------
    auto load_block = [&](const float *base, int row0, u32x4_t (&dst)[NLD]) {
        const float *ptr = base + (size_t)(row0 + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) dst[i] = *reinterpret_cast<const u32x4_t *>(ptr + (size_t)(i * RPI) * rs);
    };
    auto leaf_row0 = [&](int kb) {
        kb = kb < 0 ? 0 : (kb >= NB ? NB - 1 : kb);
        return kb * TQ;
    };
    auto load_near = [&](const float *base, int q0, u32x4_t (&dst)[NLD]) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int tr = t_off[i] + (((q0 >> t_lvl[i]) + t_add[i]) ^ t_xor[i]);
            dst[i] = u32x4_t{0u, 0u, 0u, 0u};
            if (t_valid[i]) dst[i] = *reinterpret_cast<const u32x4_t *>(base + (size_t)tr * rs);
        }
    };
    auto load_far = [&](const float *base, u32x4_t (&dst)[NLD]) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            dst[i] = u32x4_t{0u, 0u, 0u, 0u};
            if (u_valid[i]) {
                const int ur = level_offset(N, u_lvl[i]) + ((qs >> u_lvl[i]) ^ 1);
                dst[i] = *reinterpret_cast<const u32x4_t *>(base + (size_t)ur * rs);
            }
        }
    };
    auto lds_put = [&](int slot, const u32x4_t (&raw)[NLD]) {
        unsigned char *reg = lds + slot * BLK_BYTES + lrow * PITCH + 16 * lchk;
#pragma unroll
        for (int i = 0; i < NLD; ++i) *reinterpret_cast<u32x4_t *>(reg + i * RPI * PITCH) = raw[i];
    };
    // row operand (keys or queries): channels [g*DS, (g+1)*DS) of row r16
    auto get_rows = [&](int slot, float (&dst)[DS]) {
        const unsigned char *reg = lds + slot * BLK_BYTES + r16 * PITCH + g * (DS * 4);
#pragma unroll
        for (int t = 0; t < DS / 4; ++t) {
            const f32x4 x = *reinterpret_cast<const f32x4 *>(reg + 16 * t);
            dst[4 * t] = x[0]; dst[4 * t + 1] = x[1]; dst[4 * t + 2] = x[2]; dst[4 * t + 3] = x[3];
        }
    };
    // transposed value operand: dst[j][i] = V[row 4g+i][channel r16*NJ + j].  Column r16 of output
    // tile j stands for channel r16*NJ + j, so that a lane's NJ values of one row are consecutive
    // floats: one 16-byte LDS read per row (two at D = 128) instead of NJ 4-byte ones.
    auto get_cols = [&](int slot, float (&dst)[NJ][4]) {
        const unsigned char *reg = lds + slot * BLK_BYTES + (4 * g) * PITCH + r16 * (NJ * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (NJ == 2) {
                const f32x2 x = *reinterpret_cast<const f32x2 *>(reg + i * PITCH);
                dst[0][i] = x[0]; dst[1][i] = x[1];
            } else {
#pragma unroll
                for (int t = 0; t < NJ / 4; ++t) {
                    const f32x4 x = *reinterpret_cast<const f32x4 *>(reg + i * PITCH + 16 * t);
                    dst[4 * t][i] = x[0]; dst[4 * t + 1][i] = x[1]; dst[4 * t + 2][i] = x[2]; dst[4 * t + 3][i] = x[3];
                }
            }
        }
    };

    struct Stage {
        u32x4_t q[NLD], k[NLD], v[NLD], kt[NLD], vt[NLD];
    };
    auto request = [&](Stage &sg, int blk) {
        const int q0 = blk * TQ;
        load_block(Qb, q0, sg.q);
        const int row0 = leaf_row0(blk + (CAUSAL ? 0 : NBW));
        load_block(Kb, row0, sg.k);
        load_block(Vb, row0, sg.v);
        load_near(Kb, q0, sg.kt);
        load_near(Vb, q0, sg.vt);
    };
    Stage st[SB];
    request(st[0], blk0);

    // ---- per-strip operands: far tree block, leaf blocks left of the first query block ----
    float Ku[DS], Vu[NJ][4];
    {
        u32x4_t rk[NLD], rv[NLD];
        load_far(Kb, rk);
        load_far(Vb, rv);
        lds_put(0, rk);
        lds_put(1, rv);
        get_rows(0, Ku);
        get_cols(1, Vu);
    }
    float Kl[NKL][DS], Vl[NKL][NJ][4];
#pragma unroll
    for (int c = 0; c < NKL - 1; ++c) {
        u32x4_t rk[NLD], rv[NLD];
        const int row0 = leaf_row0(blk0 - NBW + c);
        load_block(Kb, row0, rk);
        load_block(Vb, row0, rv);
        lds_put(0, rk);
        lds_put(1, rv);
        get_rows(0, Kl[c]);
        get_cols(1, Vl[c]);
    }

    auto process = [&](Stage &sg, int blk, Stage &nsg, int next_blk) {
        const int q0 = blk * TQ;
        float Qf[DS], Kt[DS], Vt[NJ][4];
        // three LDS blocks, reused: a wavefront's LDS operations execute in order, so a block may
        // be overwritten as soon as the reads of its previous content have been issued
        lds_put(0, sg.q);
        lds_put(1, sg.k);
        lds_put(2, sg.v);
        get_rows(0, Qf);
        get_rows(1, Kl[NEWC]);
        get_cols(2, Vl[NEWC]);
        lds_put(0, sg.kt);
        lds_put(1, sg.vt);
        if (next_blk >= 0) request(nsg, next_blk);  // this block's raw registers are consumed
        get_rows(0, Kt);
        get_cols(1, Vt);

        // scores, transposed: acc[i] = <key 4g+i of the block, query r16>
        f32x4 accL[NKL], accT = {0.f, 0.f, 0.f, 0.f}, accU = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NKL; ++c) {
            accL[c] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < DS; ++t) accL[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(Kl[c][t], Qf[t], accL[c], 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < DS; ++t) {
            accT = __builtin_amdgcn_mfma_f32_16x16x4f32(Kt[t], Qf[t], accT, 0, 0, 0);
            accU = __builtin_amdgcn_mfma_f32_16x16x4f32(Ku[t], Qf[t], accU, 0, 0, 0);
        }

        float sc[NKL + 2][4];
        float mx = NEG_INF_F;
#pragma unroll
        for (int c = 0; c < NKL; ++c) {
            const int kb = blk - NBW + c;
            const bool inside = kb >= 0 && kb < NB;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sc[c][i] = inside ? fmaf(accL[c][i], p.scale_log2e, biasL[c][i]) : NEG_INF_F;
                mx = fmaxf(mx, sc[c][i]);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float bias = biasT[i];
            if (CAUSAL) {
                const int lv = upT[i];
                if (lv >= 0 && ((q0 >> lv) & 1) == 0) bias = NEG_INF_F;
            }
            sc[NKL][i] = fmaf(accT[i], p.scale_log2e, bias);
            sc[NKL + 1][i] = fmaf(accU[i], p.scale_log2e, biasU[i]);
            mx = fmaxf(mx, fmaxf(sc[NKL][i], sc[NKL + 1][i]));
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        float den = 0.f;
#pragma unroll
        for (int c = 0; c < NKL + 2; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sc[c][i] = __builtin_amdgcn_exp2f(sc[c][i] - mx);
                den += sc[c][i];
            }
        den += __shfl_xor(den, 16, 64);
        den += __shfl_xor(den, 32, 64);
        const float inv = 1.0f / den;  // one correctly rounded reciprocal per query instead of a division per output

        // O^T tiles: lane = query r16, row 4g+i of tile j = channel (4g+i)*NJ + j; back to whole rows
        // through LDS
        unsigned char *oreg = lds + r16 * PITCH + (4 * g) * (NJ * 4);
        if constexpr (NJ <= 4) {
            f32x4 o[NJ];
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                o[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
#pragma unroll
                    for (int c = 0; c < NKL; ++c) o[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(Vl[c][j][i], sc[c][i], o[j], 0, 0, 0);
                    o[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(Vt[j][i], sc[NKL][i], o[j], 0, 0, 0);
                    o[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(Vu[j][i], sc[NKL + 1][i], o[j], 0, 0, 0);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if constexpr (NJ == 2)
                    *reinterpret_cast<f32x2 *>(oreg + i * 8) = f32x2{o[0][i] * inv, o[1][i] * inv};
                else
                    *reinterpret_cast<f32x4 *>(oreg + i * 16) =
                        f32x4{o[0][i] * inv, o[1][i] * inv, o[2][i] * inv, o[3][i] * inv};
            }
        } else {
            // eight tiles: written as they are finished, one float each (holding them all would spill)
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
#pragma unroll
                    for (int c = 0; c < NKL; ++c) o = __builtin_amdgcn_mfma_f32_16x16x4f32(Vl[c][j][i], sc[c][i], o, 0, 0, 0);
                    o = __builtin_amdgcn_mfma_f32_16x16x4f32(Vt[j][i], sc[NKL][i], o, 0, 0, 0);
                    o = __builtin_amdgcn_mfma_f32_16x16x4f32(Vu[j][i], sc[NKL + 1][i], o, 0, 0, 0);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) *reinterpret_cast<float *>(oreg + (i * NJ + j) * 4) = o[i] * inv;
            }
        }
        {
            const unsigned char *src = lds + lrow * PITCH + 16 * lchk;
            float *optr = Ob + (size_t)(q0 + lrow) * rs;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const u32x4_t val = *reinterpret_cast<const u32x4_t *>(src + i * RPI * PITCH);
                __builtin_nontemporal_store(val, reinterpret_cast<u32x4_t *>(optr + (size_t)(i * RPI) * rs));
            }
        }
        // slide the leaf window by one block
#pragma unroll
        for (int c = 0; c + 1 < NKL; ++c) {
#pragma unroll
            for (int t = 0; t < DS; ++t) Kl[c][t] = Kl[c + 1][t];
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) Vl[c][j][i] = Vl[c + 1][j][i];
        }
    };

#pragma unroll
    for (int it = 0; it < SB; ++it) {
        if (it + 1 < SB) process(st[it], blk0 + it, st[it + 1], blk0 + it + 1);
        else process(st[it], blk0 + it, st[it], -1);
    }
}

template <int D, int NBW, bool CAUSAL, int WPB>
int launch_wpb(const TileF32Params &p, int sb, hipStream_t st) {
    const int nwg = (p.n_units + WPB - 1) / WPB;
    constexpr int MAXSB = f32_max_strip<D, NBW, CAUSAL>();
    if (sb == 1) {
        attn_tile_f32_kernel<D, NBW, CAUSAL, 1, WPB><<<nwg, WPB * 64, 0, st>>>(p);
        return check_launch("attn_tile_f32_kernel");
    }
    if constexpr (MAXSB >= 2) {
        if (sb == 2) {
            attn_tile_f32_kernel<D, NBW, CAUSAL, 2, WPB><<<nwg, WPB * 64, 0, st>>>(p);
            return check_launch("attn_tile_f32_kernel");
        }
    }
    if constexpr (MAXSB >= 4) {
        if (sb == 4) {
            attn_tile_f32_kernel<D, NBW, CAUSAL, 4, WPB><<<nwg, WPB * 64, 0, st>>>(p);
            return check_launch("attn_tile_f32_kernel");
        }
    }
    return fail(HSA_ERR_UNSUPPORTED, "strip length %d not built for this variant", sb);
}

template <int D, int NBW, bool CAUSAL>
int launch_sb(const TileF32Params &p, int sb, hipStream_t st) {
    // eight wavefronts per workgroup only if that still gives every CU a workgroup
    if constexpr (f32_fits_two_per_simd<D, NBW, CAUSAL>()) {
        if (p.n_units >= 8 * 256) return launch_wpb<D, NBW, CAUSAL, 8>(p, sb, st);
    }
    return launch_wpb<D, NBW, CAUSAL, 4>(p, sb, st);
}

template <int D>
int launch_d(const TileF32Params &p, int nbw, bool causal, int sb, hipStream_t st) {
    switch (nbw * 2 + (causal ? 1 : 0)) {
        case 0: return launch_sb<D, 0, false>(p, sb, st);
        case 1: return launch_sb<D, 0, true>(p, sb, st);
        case 2: return launch_sb<D, 1, false>(p, sb, st);
        case 3: return launch_sb<D, 1, true>(p, sb, st);
        case 4: return launch_sb<D, 2, false>(p, sb, st);
        case 5: return launch_sb<D, 2, true>(p, sb, st);
    }
    return fail(HSA_ERR_UNSUPPORTED, "window radius too large for the tile kernel");
}

}  // namespace

void attn_tile_knobs_sb_swizzle(int *sb, int *swizzle);  // hsa_attn_tile.hip

bool attn_tile_f32_eligible(int N, int M, int D, int L, int R, bool canonical, bool want_weights) {
    if (!canonical || want_weights) return false;
    if (D != 32 && D != 64 && D != 128) return false;
    if (N < TQ || ilog2_exact(N) != L || L > F32_MAX_LEVELS) return false;
    if (M < 2 * N - 1) return false;
    return (R + TQ - 1) / TQ <= F32_MAX_NBW;
}

int attn_tile_f32_dispatch(const void *q, const void *k, const void *v, void *out, int B, int N, int M, int H,
                           int D, int L, int R, int causal, hipStream_t st) {
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0)
        return fail(HSA_ERR_INVALID, "tile kernel needs 16-byte aligned tensors");
    TileF32Params p;
    p.q = (const float *)q; p.k = (const float *)k; p.v = (const float *)v;
    p.out = (float *)out;
    p.B = B; p.N = N; p.M = M; p.H = H; p.L = L; p.R = R;
    const int NB = N / TQ;
    const int nbw = (R + TQ - 1) / TQ;
    const long block_units = (long)B * H * NB;
    int sb = block_units >= 4 * 2048 ? 4 : (block_units >= 2 * 2048 ? 2 : 1);
    int forced_sb = 0, swizzle = 1;
    attn_tile_knobs_sb_swizzle(&forced_sb, &swizzle);
    if (forced_sb) sb = forced_sb;
    if (!causal && nbw >= 2 && sb > 2) sb = 2;  // five leaf blocks: registers
    if (D == 128) sb = sb > 1 && causal && nbw <= 1 ? 2 : 1;
    while (sb > NB) sb >>= 1;
    p.NS = NB / sb;
    const long units = (long)B * p.NS * H;
    if (units > 0x3fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.n_units = (int)units;
    p.xcd_swizzle = swizzle;
    p.scale_log2e = 1.4426950408889634f / sqrtf((float)D);
    if (D == 32) return launch_d<32>(p, nbw, causal != 0, sb, st);
    if (D == 128) return launch_d<128>(p, nbw, causal != 0, sb, st);
    return launch_d<64>(p, nbw, causal != 0, sb, st);
}

}  // namespace hsa
