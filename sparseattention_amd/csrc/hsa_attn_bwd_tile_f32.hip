// Span attention backward, fp32 tensors, on the fp32 matrix cores (v_mfma_f32_16x16x4_f32).
//
// The same two passes as the 16-bit tile backward (hsa_attn_bwd_tile.h) with the operand
// plumbing of the fp32 forward kernel (hsa_attn_tile_f32.hip).  A 16-row block X of D floats is
// held in up to two register forms:
//   rows form  X.r[t]    = X[row r16][channel g*D/4 + t]        (contracts channels)
//   cols form  X.c[j][i] = X[row 4g+i][channel 16j + r16]       (contracts rows)
// and an MFMA(A, B) with A lane = (row r16, k = g), B lane = (k = g, column r16) leaves the
// result in lane = column r16, registers = rows 4g+i.  With that
//   S^T[key, query]  = mfma(K.r, Q.r)      dP^T[key, query] = mfma(V.r, dO.r)
//   dQ^T[ch, query]  = mfma(K.c, dS^T)     (dS^T is already the B operand: lane = query, regs = keys)
//   S[query, key]    = mfma(Q.r, K.r)      dP[query, key]   = mfma(dO.r, V.r)
//   dK^T[ch, key]    = mfma(Q.c, dS)       dV^T[ch, key]    = mfma(dO.c, P)
//
//  (A) query pass, one wavefront per (batch, head, 16-query block): log-sum-exp and delta of its
//      queries (saved), dQ, and the rows of dK / dV of the tree nodes: levels 1..3 are attended
//      only from inside the block and written directly, levels >= 4 leave an fp32 partial row per
//      block and level; the key pass's trailing workgroups sum them.
//  (B) key pass, one wavefront per (batch, head, 16-leaf key block): dK / dV of the leaves from
//      the query blocks whose window reaches the block.
// Scores, softmax and accumulation are fp32; exp2 is the hardware instruction (1 ulp, arguments
// <= 0), the log-sum-exp uses the library log2, and P is scaled by one correctly rounded reciprocal
// per query.
#include "hsa_attn_bwd_tile.h"

namespace hsa {

namespace {

constexpr int F32B_WPB = 4;  // wavefronts per workgroup, one per SIMD (the query pass takes > 256 registers)

struct BwdF32Params {
    const float *q, *k, *v, *dout;
    float *dq, *dk, *dv;
    float *stats;    // [B, N, H, 2]: log2-domain lse, delta
    float *partial;  // layout of the 16-bit backward with strips of one block
    int B, N, M, H, L, R;
    int n_units;
    float scale_log2e, scale;
    // rows the key pass's trailing workgroups finish from the partial rows
    int causal, red_first_row, red_wgs;
};

template <int D>
struct F32Blk {
    static constexpr int DS = D / 4, NJ = D / 16, CPR = D / 4, RPI = 64 / CPR, NLD = TILE_Q / RPI;
    static constexpr int PITCH = D * 4 + 16, BLK_BYTES = TILE_Q * PITCH;

    int r16, g, lrow, lchk;
    unsigned char *lds;

    __device__ __forceinline__ void init(unsigned char *wave_lds) {
        const int lane = threadIdx.x & 63;
        r16 = lane & 15;
        g = lane >> 4;
        lrow = lane / CPR;
        lchk = lane % CPR;
        lds = wave_lds;
    }
    __device__ __forceinline__ void put(int slot, const u32x4_t (&raw)[NLD]) const {
        unsigned char *reg = lds + slot * BLK_BYTES + lrow * PITCH + 16 * lchk;
#pragma unroll
        for (int i = 0; i < NLD; ++i) *reinterpret_cast<u32x4_t *>(reg + i * RPI * PITCH) = raw[i];
    }
    __device__ __forceinline__ void rows(int slot, float (&dst)[DS]) const {
        const unsigned char *reg = lds + slot * BLK_BYTES + r16 * PITCH + g * (DS * 4);
#pragma unroll
        for (int t = 0; t < DS / 4; ++t) {
            const f32x4 x = *reinterpret_cast<const f32x4 *>(reg + 16 * t);
            dst[4 * t] = x[0]; dst[4 * t + 1] = x[1]; dst[4 * t + 2] = x[2]; dst[4 * t + 3] = x[3];
        }
    }
    __device__ __forceinline__ void cols(int slot, float (&dst)[NJ][4]) const {
        const unsigned char *reg = lds + slot * BLK_BYTES + (4 * g) * PITCH + r16 * 4;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[j][i] = *reinterpret_cast<const float *>(reg + i * PITCH + 64 * j);
    }
    // result tiles (this lane: column r16, channels 16j + 4g + i) -> row r16 of LDS slot `slot`
    __device__ __forceinline__ void put_result(int slot, const f32x4 (&t)[NJ]) const {
        unsigned char *reg = lds + slot * BLK_BYTES + r16 * PITCH + 16 * g;
#pragma unroll
        for (int j = 0; j < NJ; ++j) *reinterpret_cast<f32x4 *>(reg + 64 * j) = t[j];
    }
    __device__ __forceinline__ u32x4_t row_piece(int slot, int i) const {
        return *reinterpret_cast<const u32x4_t *>(lds + slot * BLK_BYTES + (i * RPI + lrow) * PITCH + 16 * lchk);
    }
};

__device__ __forceinline__ f32x4 mma4(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// near tree slot -> level and position under the block's ancestor (-1: the sibling slots of levels 4, 5)
__device__ __forceinline__ int near_slot_level(int sl, int &pl) {
    if (sl < 8) { pl = sl; return 1; }
    if (sl < 12) { pl = sl - 8; return 2; }
    if (sl < 14) { pl = sl - 12; return 3; }
    pl = -1;
    return 4 + (sl - 14);
}

// ---------------------------------------------------------------------------------------------
// (A) query pass
// ---------------------------------------------------------------------------------------------
// Wavefronts per SIMD the query pass is compiled for: two (256 registers) up to three leaf blocks
// per query block, where at most a few words spill; one with five leaf blocks at D = 64 and
// always at D = 128 (there part of the operands lives in per-lane scratch memory).
constexpr int f32b_query_waves(int D, int nkl) { return D >= 128 ? 1 : ((D <= 32 || nkl <= 3) ? 2 : 1); }

template <int D, int NBW, bool CAUSAL>
__global__ void __launch_bounds__(F32B_WPB * 64)
__attribute__((amdgpu_waves_per_eu(f32b_query_waves(D, CAUSAL ? NBW + 1 : 2 * NBW + 1))))
attn_bwd_f32_query_kernel(BwdF32Params p) {
    using BT = F32Blk<D>;
    constexpr int DS = BT::DS, NJ = BT::NJ, RPI = BT::RPI, NLD = BT::NLD;
    constexpr int NKL = CAUSAL ? NBW + 1 : 2 * NBW + 1;
    constexpr int NKB = NKL + 2;  // leaf blocks, near tree block, far tree block
    constexpr int LDS_SLOTS = 2;
    __shared__ __align__(16) unsigned char smem[F32B_WPB * LDS_SLOTS * BT::BLK_BYTES];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = bwd_xcd_remap((int)blockIdx.x, (int)gridDim.x) * F32B_WPB + wave;
    if (unit >= p.n_units) return;
    BT bt;
    bt.init(smem + wave * LDS_SLOTS * BT::BLK_BYTES);
    const int r16 = bt.r16, g = bt.g, lrow = bt.lrow, lchk = bt.lchk;

    const int N = p.N, L = p.L, R = p.R, H = p.H;
    const int NB = N / TILE_Q;
    const int h = unit % H;
    const int blk = (unit / H) % NB;
    const int b = unit / (H * NB);
    const int q0 = blk * TILE_Q;
    const size_t rs = (size_t)H * D;
    const float *Qb = p.q + ((size_t)b * N * H + h) * D + 4 * lchk;
    const float *Gb = p.dout + ((size_t)b * N * H + h) * D + 4 * lchk;
    const float *Kb = p.k + ((size_t)b * p.M * H + h) * D + 4 * lchk;
    const float *Vb = p.v + ((size_t)b * p.M * H + h) * D + 4 * lchk;
    float *dKb = p.dk + ((size_t)b * p.M * H + h) * D + 4 * lchk;
    float *dVb = p.dv + ((size_t)b * p.M * H + h) * D + 4 * lchk;

    // rows of the tree nodes this lane fetches (and, for levels 1..3, writes); -1 = no such node
    int t_row[NLD], u_row[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int sl = i * RPI + lrow;
        int pl;
        const int lvl = near_slot_level(sl, pl);
        t_row[i] = lvl < L ? level_offset(N, lvl) + (pl >= 0 ? (q0 >> lvl) + pl : ((q0 >> lvl) ^ 1)) : -1;
        const int ul = 6 + sl;
        u_row[i] = ul < L ? level_offset(N, ul) + ((q0 >> ul) ^ 1) : -1;
    }

    // ---- every row the block needs is requested before anything is consumed ------------------
    auto load_block = [&](const float *base, int row0, u32x4_t (&dst)[NLD]) {
        const float *ptr = base + (size_t)(row0 + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) dst[i] = *reinterpret_cast<const u32x4_t *>(ptr + (size_t)(i * RPI) * rs);
    };
    auto leaf_row0 = [&](int kb) {
        kb = kb < 0 ? 0 : (kb >= NB ? NB - 1 : kb);
        return kb * TILE_Q;
    };
    u32x4_t rQ[NLD], rG[NLD], rK[NKB][NLD], rV[NKB][NLD];
    load_block(Qb, q0, rQ);
    load_block(Gb, q0, rG);
#pragma unroll
    for (int c = 0; c < NKL; ++c) {
        load_block(Kb, leaf_row0(blk - NBW + c), rK[c]);
        load_block(Vb, leaf_row0(blk - NBW + c), rV[c]);
    }
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const size_t tr = (size_t)(t_row[i] < 0 ? q0 : t_row[i]) * rs;
        const size_t ur = (size_t)(u_row[i] < 0 ? q0 : u_row[i]) * rs;
        rK[NKL][i] = *reinterpret_cast<const u32x4_t *>(Kb + tr);
        rV[NKL][i] = *reinterpret_cast<const u32x4_t *>(Vb + tr);
        rK[NKL + 1][i] = *reinterpret_cast<const u32x4_t *>(Kb + ur);
        rV[NKL + 1][i] = *reinterpret_cast<const u32x4_t *>(Vb + ur);
    }

    // ---- score biases (log2 of the multiplicity, -inf = not attended) ------------------------
    // orientation 1: lane = query r16, registers = keys / slots 4g+i; orientation 2 (tree blocks):
    // lane = slot r16, registers = queries 4g+i
    float b1T[4], b2T[4], b1U[4], b2U[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        {
            int pl;
            const int lvl = near_slot_level(4 * g + i, pl);
            const bool live = pl >= 0 ? (pl == ((r16 >> lvl) ^ 1) && (!CAUSAL || ((r16 >> lvl) & 1)))
                                      : (lvl < L && (!CAUSAL || ((q0 >> lvl) & 1)));
            b1T[i] = live ? 0.f : NEG_INF;
        }
        {
            int pl;
            const int lvl = near_slot_level(r16, pl);
            const int ql = 4 * g + i;
            const bool live = pl >= 0 ? (pl == ((ql >> lvl) ^ 1) && (!CAUSAL || ((ql >> lvl) & 1)))
                                      : (lvl < L && (!CAUSAL || ((q0 >> lvl) & 1)));
            b2T[i] = live ? 0.f : NEG_INF;
        }
        const int ul1 = 6 + 4 * g + i, ul2 = 6 + r16;
        b1U[i] = (ul1 < L && (!CAUSAL || ((q0 >> ul1) & 1))) ? 0.f : NEG_INF;
        b2U[i] = (ul2 < L && (!CAUSAL || ((q0 >> ul2) & 1))) ? 0.f : NEG_INF;
    }

    // ---- rows -> operand forms ---------------------------------------------------------------
    float Qr[DS], Gr[DS], Qc[NJ][4], Gc[NJ][4];
    bt.put(0, rQ);
    bt.put(1, rG);
    bt.rows(0, Qr);
    bt.cols(0, Qc);
    bt.rows(1, Gr);
    bt.cols(1, Gc);

    // ---- orientation 1 over all key blocks: S^T, dP^T ----------------------------------------
    float Kc[NKB][NJ][4], KrT[2][DS], VrT[2][DS];  // K in cols form; the tree blocks also keep their rows forms
    float sc[NKB][4], dp[NKB][4];
    float mx = NEG_INF;
#pragma unroll
    for (int c = 0; c < NKB; ++c) {
        float Kr[DS], Vr[DS];
        bt.put(0, rK[c]);
        bt.put(1, rV[c]);
        bt.rows(0, Kr);
        bt.cols(0, Kc[c]);
        bt.rows(1, Vr);
        f32x4 a = {0.f, 0.f, 0.f, 0.f}, d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < DS; ++t) {
            a = mma4(Kr[t], Qr[t], a);
            d = mma4(Vr[t], Gr[t], d);
        }
        if (c >= NKL) {
#pragma unroll
            for (int t = 0; t < DS; ++t) { KrT[c >= NKL ? c - NKL : 0][t] = Kr[t]; VrT[c >= NKL ? c - NKL : 0][t] = Vr[t]; }
        }
        const int kb = blk - NBW + c;
        const bool inside = c >= NKL || (kb >= 0 && kb < NB);
        const int dlt = TILE_Q * (c - NBW);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float bias;
            if (c < NKL) {
                const int kl = 4 * g + i;
                const int diff = dlt + kl - r16;
                const bool win = diff >= -R && diff <= (CAUSAL ? 0 : R);
                const bool sib = dlt == 0 && kl == (r16 ^ 1) && (!CAUSAL || (r16 & 1));
                const int cnt = (int)win + (int)sib;
                bias = (!inside || cnt == 0) ? NEG_INF : (cnt == 2 ? 1.0f : 0.0f);
            } else {
                bias = c == NKL ? b1T[i] : b1U[i];
            }
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
    const float inv = 1.0f / den;  // one correctly rounded reciprocal per query
    float delta = 0.f;
#pragma unroll
    for (int c = 0; c < NKB; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sc[c][i] = sc[c][i] * inv;  // P
            delta = fmaf(sc[c][i], dp[c][i], delta);
        }
    delta += __shfl_xor(delta, 16, 64);
    delta += __shfl_xor(delta, 32, 64);
    const float lse = mx + log2f(den);  // log2 domain: P = exp2(s' - lse)
    if (g == 0) {
        float *stp = p.stats + (((size_t)b * N + q0 + r16) * H + h) * 2;
        stp[0] = lse;
        stp[1] = delta;
    }

    // ---- dQ^T = sum_c K_c^T . dS_c^T ----------------------------------------------------------
    {
        f32x4 acc[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NKB; ++c) {
            float ds[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) ds[i] = sc[c][i] * (dp[c][i] - delta) * p.scale;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[j] = mma4(Kc[c][j][i], ds[i], acc[j]);
        }
        bt.put_result(0, acc);
        float *optr = p.dq + ((size_t)b * N * H + h) * D + 4 * lchk + (size_t)(q0 + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            *reinterpret_cast<u32x4_t *>(optr + (size_t)(i * RPI) * rs) = bt.row_piece(0, i);
    }

    // ---- orientation 2 for the tree blocks: dK^T, dV^T [channel, slot] ------------------------
    float lse4[4], del4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        lse4[i] = __shfl(lse, 4 * g + i, 64);
        del4[i] = __shfl(delta, 4 * g + i, 64);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        f32x4 a = {0.f, 0.f, 0.f, 0.f}, d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            a = mma4(Qr[s], KrT[t][s], a);  // S[query 4g+i, slot r16]
            d = mma4(Gr[s], VrT[t][s], d);  // dP[query, slot]
        }
        float pp[4], ds[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float bias = t == 0 ? b2T[i] : b2U[i];
            pp[i] = __builtin_amdgcn_exp2f(fmaf(a[i], p.scale_log2e, bias) - lse4[i]);
            ds[i] = pp[i] * (d[i] - del4[i]) * p.scale;
        }
        f32x4 tk[NJ], tv[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            tk[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            tv[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                tk[j] = mma4(Qc[j][i], ds[i], tk[j]);
                tv[j] = mma4(Gc[j][i], pp[i], tv[j]);
            }
        }
        if (t == 0) {
            // slots 0..13 (levels 1..3) are complete: rows written directly
            bt.put_result(0, tk);
            bt.put_result(1, tv);
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int sl = i * RPI + lrow;
                if (sl < 14 && t_row[i] >= 0) {
                    *reinterpret_cast<u32x4_t *>(dKb + (size_t)t_row[i] * rs) = bt.row_piece(0, i);
                    *reinterpret_cast<u32x4_t *>(dVb + (size_t)t_row[i] * rs) = bt.row_piece(1, i);
                }
            }
            // levels 4 and 5 collect from one or two blocks: this block's partial rows
            const int lvl = r16 >= 14 ? 4 + (r16 - 14) : -1;
            if (lvl >= 4 && lvl < L) {
                const size_t po = ((((size_t)b * NB + blk) * H + h) * 2 + (lvl - 4)) * D;
                float *pkp = p.partial + po;
                float *pvp = p.partial + (size_t)p.B * NB * H * 2 * D + po;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    *reinterpret_cast<f32x4 *>(pkp + 16 * j + 4 * g) = tk[j];
                    *reinterpret_cast<f32x4 *>(pvp + 16 * j + 4 * g) = tv[j];
                }
            }
        } else {
            // levels >= 6: this block's partial rows
            const int lvl = 6 + r16;
            const int LF = L - 6;
            if (lvl < L) {
                float *far = p.partial + 2 * (size_t)p.B * NB * H * 2 * D;
                const size_t po = ((((size_t)b * NB + blk) * H + h) * LF + (lvl - 6)) * D;
                float *pkp = far + po;
                float *pvp = far + (size_t)p.B * NB * H * LF * D + po;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    *reinterpret_cast<f32x4 *>(pkp + 16 * j + 4 * g) = tk[j];
                    *reinterpret_cast<f32x4 *>(pvp + 16 * j + 4 * g) = tv[j];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// (B) key pass over the leaf key blocks
// ---------------------------------------------------------------------------------------------
template <int D, int NBW, bool CAUSAL>
__global__ void __launch_bounds__(F32B_WPB * 64) attn_bwd_f32_key_kernel(BwdF32Params p) {
    using BT = F32Blk<D>;
    constexpr int DS = BT::DS, NJ = BT::NJ, RPI = BT::RPI, NLD = BT::NLD;
    constexpr int NQB = CAUSAL ? NBW + 1 : 2 * NBW + 1;  // query blocks that reach a key block
    constexpr int QOFF = CAUSAL ? 0 : -NBW;              // first of them, relative to the key block
    constexpr int LDS_SLOTS = 2;
    __shared__ __align__(16) unsigned char smem[F32B_WPB * LDS_SLOTS * BT::BLK_BYTES];

    // the last red_wgs workgroups take no key block: they sum the query pass's partial rows into
    // the dK / dV rows of tree levels >= 4 (rows this pass does not write)
    const int key_wgs = (int)gridDim.x - p.red_wgs;
    if ((int)blockIdx.x >= key_wgs) {
        bwd_reduce_rows<F32>(p.partial, p.dk, p.dv, p.B, p.N, p.M, p.H, D, p.L, p.causal, p.red_first_row, 0,
                             (size_t)((int)blockIdx.x - key_wgs) * (F32B_WPB * 64) + threadIdx.x);
        return;
    }
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = bwd_xcd_remap((int)blockIdx.x, key_wgs) * F32B_WPB + wave;
    if (unit >= p.n_units) return;
    BT bt;
    bt.init(smem + wave * LDS_SLOTS * BT::BLK_BYTES);
    const int r16 = bt.r16, g = bt.g, lrow = bt.lrow, lchk = bt.lchk;

    const int N = p.N, R = p.R, H = p.H;
    const int NB = N / TILE_Q;
    const int h = unit % H;
    const int kb = (unit / H) % NB;
    const int b = unit / (H * NB);
    const int k0 = kb * TILE_Q;
    const size_t rs = (size_t)H * D;
    const float *Qb = p.q + ((size_t)b * N * H + h) * D + 4 * lchk;
    const float *Gb = p.dout + ((size_t)b * N * H + h) * D + 4 * lchk;
    const float *Kb = p.k + ((size_t)b * p.M * H + h) * D + 4 * lchk;
    const float *Vb = p.v + ((size_t)b * p.M * H + h) * D + 4 * lchk;

    auto load_block = [&](const float *base, int row0, u32x4_t (&dst)[NLD]) {
        const float *ptr = base + (size_t)(row0 + lrow) * rs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) dst[i] = *reinterpret_cast<const u32x4_t *>(ptr + (size_t)(i * RPI) * rs);
    };
    auto clampb = [&](int qb) { return qb < 0 ? 0 : (qb >= NB ? NB - 1 : qb); };

    u32x4_t rK[NLD], rV[NLD], rQ[NQB][NLD], rG[NQB][NLD];
    float lse4[NQB][4], del4[NQB][4];
    load_block(Kb, k0, rK);
    load_block(Vb, k0, rV);
#pragma unroll
    for (int c = 0; c < NQB; ++c) {
        const int qb = clampb(kb + QOFF + c);
        load_block(Qb, qb * TILE_Q, rQ[c]);
        load_block(Gb, qb * TILE_Q, rG[c]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float *stp = p.stats + (((size_t)b * N + qb * TILE_Q + 4 * g + i) * H + h) * 2;
            lse4[c][i] = stp[0];
            del4[c][i] = stp[1];
        }
    }
    float Kr[DS], Vr[DS];
    bt.put(0, rK);
    bt.put(1, rV);
    bt.rows(0, Kr);
    bt.rows(1, Vr);

    f32x4 tk[NJ], tv[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { tk[j] = f32x4{0.f, 0.f, 0.f, 0.f}; tv[j] = f32x4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
    for (int c = 0; c < NQB; ++c) {
        const int qb = kb + QOFF + c;
        const bool inside = qb >= 0 && qb < NB;  // uniform
        float Qr[DS], Gr[DS], Qc[NJ][4], Gc[NJ][4];
        bt.put(0, rQ[c]);
        bt.put(1, rG[c]);
        bt.rows(0, Qr);
        bt.cols(0, Qc);
        bt.rows(1, Gr);
        bt.cols(1, Gc);
        f32x4 a = {0.f, 0.f, 0.f, 0.f}, d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < DS; ++t) {
            a = mma4(Qr[t], Kr[t], a);  // S[query 4g+i of block qb, key r16]
            d = mma4(Gr[t], Vr[t], d);
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
            pp[i] = __builtin_amdgcn_exp2f(fmaf(a[i], p.scale_log2e, bias) - lse4[c][i]);
            ds[i] = pp[i] * (d[i] - del4[c][i]) * p.scale;
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                tk[j] = mma4(Qc[j][i], ds[i], tk[j]);
                tv[j] = mma4(Gc[j][i], pp[i], tv[j]);
            }
    }
    bt.put_result(0, tk);
    bt.put_result(1, tv);
    float *dKp = p.dk + ((size_t)b * p.M * H + h) * D + 4 * lchk + (size_t)(k0 + lrow) * rs;
    float *dVp = p.dv + ((size_t)b * p.M * H + h) * D + 4 * lchk + (size_t)(k0 + lrow) * rs;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        *reinterpret_cast<u32x4_t *>(dKp + (size_t)(i * RPI) * rs) = bt.row_piece(0, i);
        *reinterpret_cast<u32x4_t *>(dVp + (size_t)(i * RPI) * rs) = bt.row_piece(1, i);
    }
}

template <int D, int NBW, bool CAUSAL>
int launch_both(const BwdF32Params &p, hipStream_t st) {
    const int nwg = (p.n_units + F32B_WPB - 1) / F32B_WPB;
    attn_bwd_f32_query_kernel<D, NBW, CAUSAL><<<nwg, F32B_WPB * 64, 0, st>>>(p);
    int rc = check_launch("attn_bwd_f32_query_kernel");
    if (rc != HSA_OK) return rc;
    attn_bwd_f32_key_kernel<D, NBW, CAUSAL><<<nwg + p.red_wgs, F32B_WPB * 64, 0, st>>>(p);
    return check_launch("attn_bwd_f32_key_kernel");
}

template <int D>
int launch_d(const BwdF32Params &p, int nbw, bool causal, hipStream_t st) {
    switch (nbw * 2 + (causal ? 1 : 0)) {
        case 0: return launch_both<D, 0, false>(p, st);
        case 1: return launch_both<D, 0, true>(p, st);
        case 2: return launch_both<D, 1, false>(p, st);
        case 3: return launch_both<D, 1, true>(p, st);
        case 4: return launch_both<D, 2, false>(p, st);
        case 5: return launch_both<D, 2, true>(p, st);
    }
    return fail(HSA_ERR_UNSUPPORTED, "window radius too large for the fp32 tile backward");
}

}  // namespace

// fp32 tensors, head size 32, 64 or 128, canonical tables, R <= 32 (at most five leaf blocks per
// query block: all of a block's rows are in flight at once)
bool attn_bwd_tile_f32_eligible(int N, int M, int D, int L, int R) {
    if (D != 32 && D != 64 && D != 128) return false;
    if (N < TILE_Q || ilog2_exact(N) != L || L > TILE_MAX_LEVELS || M < 2 * N - 1) return false;
    return R <= 2 * TILE_Q;
}

int attn_bwd_tile_f32_dispatch(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                               void *dv, float *ws, int B, int N, int M, int H, int D, int L, int R, int causal,
                               hipStream_t st) {
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)dout | (uintptr_t)dq | (uintptr_t)dk |
          (uintptr_t)dv) & 15) != 0)
        return fail(HSA_ERR_INVALID, "tile backward needs 16-byte aligned tensors");
    BwdF32Params p;
    p.q = (const float *)q; p.k = (const float *)k; p.v = (const float *)v; p.dout = (const float *)dout;
    p.dq = (float *)dq; p.dk = (float *)dk; p.dv = (float *)dv;
    p.stats = ws;
    p.partial = ws + (size_t)B * N * H * 2;
    p.B = B; p.N = N; p.M = M; p.H = H; p.L = L; p.R = R;
    const long units = (long)B * (N / TILE_Q) * H;
    if (units > 0x3fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.n_units = (int)units;
    p.scale = 1.0f / sqrtf((float)D);
    p.scale_log2e = 1.4426950408889634f * p.scale;
    const int nbw = (R + TILE_Q - 1) / TILE_Q;
    // levels 1..3 are finished by the query pass; everything above, the root row and the rows past
    // 2N-1 by the key pass's trailing workgroups, one thread per four channels
    const int first = level_offset(N, 4);
    const size_t red_threads = (size_t)B * (M - first) * H * (D / 4);
    const size_t red_wgs = (red_threads + F32B_WPB * 64 - 1) / (F32B_WPB * 64);
    if (red_wgs > 0x3fffffffUL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.causal = causal != 0;
    p.red_first_row = first;
    p.red_wgs = (int)red_wgs;
    return D == 32 ? launch_d<32>(p, nbw, causal != 0, st)
         : D == 64 ? launch_d<64>(p, nbw, causal != 0, st)
                   : launch_d<128>(p, nbw, causal != 0, st);
}

}  // namespace hsa
