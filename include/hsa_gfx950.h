/*
 * hsa_gfx950.h - C ABI of libhsa_gfx950.so: the forward path of hierarchical sparse
 * attention (sliding window + O(log N) tree neighbours) for AMD MI355X (gfx950).
 *
 * Conventions shared by every entry point
 *   - Plain pointers and sizes only.  Device pointers are borrowed for the call;
 *     the library allocates nothing and never synchronises: kernels are enqueued
 *     on `stream` (a hipStream_t passed as void*, NULL = the default stream).
 *   - Tensors are dense, token-major:  [B, rows, H, D], D fastest.  This is the
 *     layout of an nn.Linear output viewed as heads, which is what the reference
 *     kernels consume (hierarchical_attention/modules/attention.py:100-103,182-187).
 *   - Node index space per batch: rows 0..N-1 are the leaves, row N + ... are the
 *     tree nodes level by level (level 1 first, root = row 2N-2), the order of
 *     hierarchical_attention/ops/topology.py:153-169.
 *   - Return value: 0 on success, a negative errno-style code otherwise; the text
 *     of the last failure on the calling thread is available from hsa_last_error().
 *     Nothing throws.  The reference signals misuse with Python `assert`; the
 *     Python layer above this ABI raises AssertionError for the same conditions.
 */
#ifndef HSA_GFX950_H
#define HSA_GFX950_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HSA_OK 0
#define HSA_ERR_INVALID (-22)     /* bad shape / pointer / combination of arguments   */
#define HSA_ERR_UNSUPPORTED (-95) /* valid request this build has no kernel for        */
#define HSA_ERR_LAUNCH (-5)       /* the HIP runtime rejected the launch               */

/* element types of Q/K/V/Out */
#define HSA_F32 0
#define HSA_F16 1
#define HSA_BF16 2

/* kernel selection for hsa_attn_fwd */
#define HSA_ATTN_AUTO 0    /* tile kernel when eligible, else the gather kernel */
#define HSA_ATTN_GATHER 1  /* per-query gather kernel (any dtype, any table)    */
#define HSA_ATTN_TILE 2    /* MFMA tile kernel or HSA_ERR_UNSUPPORTED           */

int hsa_abi_version(void);
const char *hsa_last_error(void);

/*
 * Span attention forward.
 * Replaces HierarchicalAttentionFunc.forward + hierarchical_attention_forward_kernel
 * (hierarchical_attention/ops/functional.py:116-168,
 *  hierarchical_attention/ops/triton/sparse_attn.py:8-179).
 *
 *   q, out      [B, N, H, D]
 *   k, v        [B, M, H, D]   M = 2N-1 in normal use
 *   idx         device int32 [N, L] neighbour rows (-1 = dead slot), or NULL: use
 *               the canonical complete-binary-tree table
 *               idx[n,l] = off_l + ((n >> l) ^ 1), off_0 = 0, off_l = 2N - (N >> (l-1));
 *               L must then be log2 N and M >= 2N-1
 *   mask        device bytes [N, L], non-zero = slot masked out.  With idx != NULL:
 *               NULL means non-causal (the reference's `mask_table is None`), non-NULL
 *               also masks window keys j > n.  With idx == NULL it must be NULL and
 *               `causal` selects the canonical mask (bit l of n clear => masked)
 *   weights     device float [B, N, H, 2R+1+L] softmax weights (window slots first,
 *               then levels; dead slots 0) or NULL to skip them
 *   R           window radius: keys n-R..n+R (the reference's `window_size`)
 *   causal      used only when idx == NULL
 *   dtype       HSA_F32 / HSA_F16 / HSA_BF16
 *   algo        HSA_ATTN_*.  The MFMA tile kernels take canonical tables (idx == NULL),
 *               16 <= N <= 2^22, R <= 32 (16-bit types: R <= 64), head sizes 32 / 64 / 128, and
 *               write weights only for the 16-bit types; everything else runs on the gather
 *               kernel
 */
int hsa_attn_fwd(const void *q, const void *k, const void *v, const int32_t *idx,
                 const uint8_t *mask, void *out, float *weights, int B, int N, int M, int H,
                 int D, int L, int R, int causal, int dtype, int algo, void *stream);

/*
 * hsa_attn_fwd that also reports the kernel's own execution interval: `start_event` and
 * `stop_event` (hipEvent_t, created by the caller with timing enabled) are attached to the
 * span-attention dispatch and carry the kernel's begin and end timestamps, so
 * hipEventElapsedTime(start, stop) is the kernel duration without the idle gap between
 * consecutive launches that events recorded around a call include.  (The gather kernels and the
 * fp32 tile kernel record the events around the launch instead.)  The reference times its kernels with torch events
 * around the Python call (hierarchical_attention_project/Hierarchical_Attention_Triton_Test.py
 * :523-568); this is the same measurement taken at the dispatch.
 */
int hsa_attn_fwd_timed(const void *q, const void *k, const void *v, const int32_t *idx,
                       const uint8_t *mask, void *out, float *weights, int B, int N, int M, int H,
                       int D, int L, int R, int causal, int dtype, int algo, void *stream,
                       void *start_event, void *stop_event);

/*
 * Launch parameters of the 16-bit MFMA tile kernel, for experiments (no counterpart in the
 * reference, whose Triton launch fixes one program per query, ops/functional.py:143-161).
 *   strip_blocks     16-query blocks one wavefront walks: 1, 2, 4, or 8 (two runs of four; four
 *                    where the window radius does not allow runs); 0 = chosen by problem size
 *   waves_per_group  wavefronts per workgroup, 1..8; 0 = chosen by head count (default)
 *   xcd_remap        0 = workgroup ids map to strips in order, 1 = neighbouring strips share an XCD
 *   alternate        0 = every strip walks upwards, 1 = neighbouring strips walk towards each other
 * An argument of -1 keeps the current value.  Process-wide; the initial values come from the
 * environment variables HSA_ATTN_TILE_SB / _WPB / _SWZ / _ALT, read once.  Results do not depend
 * on any of them.
 */
int hsa_attn_tile_tune(int strip_blocks, int waves_per_group, int xcd_remap, int alternate);

/* 1 if HSA_ATTN_AUTO would pick the MFMA tile kernel for this problem, else 0.
 * canonical_tables: 0 = tables given explicitly, 1 = canonical tables, not causal,
 * 2 = canonical tables, causal (the causal kernels take a larger window radius). */
int hsa_attn_fwd_uses_tile(int N, int M, int H, int D, int L, int R, int dtype,
                           int canonical_tables, int want_weights);

/*
 * One level of the bottom-up parent build.
 * Replaces BuildParentNodesFunc.forward + build_parent_nodes_forward_kernel
 * (hierarchical_attention/ops/functional.py:30-63,
 *  hierarchical_attention/ops/triton/build_parents.py:8-99).
 *
 *   qp, kp, vp, out  [B, P, H, D]
 *   kc, vc           [B, 2P, H, D]    children of parent i are rows 2i, 2i+1
 *   weights          [B, P, H, 3] in the element type of qp, or NULL
 *   *_bs             batch strides in elements (0 = dense), so a level can be read
 *                    from / written into a slice of a larger [B, rows, H, D] buffer
 */
int hsa_build_parents_fwd(const void *qp, const void *kp, const void *vp, const void *kc,
                          const void *vc, void *out, void *weights, int B, int P, int H, int D,
                          int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kc_bs,
                          int64_t vc_bs, int64_t out_bs, int dtype, void *stream);

/*
 * One level of the parent build whose operands are column slices of wider matrices: the level
 * step of HierarchicalAttention.cross_update_Y
 * (hierarchical_attention/modules/attention.py:119-157) once the projections that feed it are
 * fused, so that q/k/v of the parents are thirds of one [B, N-1, 3*H*D] projection and the
 * children's k/v are halves of one [B, 2P, 2*H*D] projection.  Same arithmetic as
 * hsa_build_parents_fwd.
 *
 *   batch_strides, row_strides   host arrays of 7 element counts in the order
 *                                qp, kp, vp, kc, vc, out, out2; an entry of 0, or a NULL
 *                                array, means dense (rows H*D apart, batches rows*row apart)
 *   out2                         optional second copy of the result (NULL to skip), e.g. the
 *                                level's slice of the concatenated [B, N-1, H*D] result
 */
int hsa_build_parents_strided_fwd(const void *qp, const void *kp, const void *vp, const void *kc,
                                  const void *vc, void *out, void *out2, int B, int P, int H,
                                  int D, const int64_t *batch_strides, const int64_t *row_strides,
                                  int dtype, void *stream);

/*
 * The last levels of HierarchicalAttention.cross_update_Y in one call
 * (hierarchical_attention/modules/attention.py:119-157: per level the children's
 * Wk_y / Wv_y projections :141-142, build_parent_nodes :145-153, the output feeding the next
 * level :157).  16-bit element types.  Starting from C rows `src` (the output of the level
 * below, or the leaves of a short sequence), every remaining level up to the root is computed
 * by fused kernels: projection by MFMA, rounded to the element type like a separate GEMM's
 * output, then the 3-way softmax per parent and head, without the projected keys and values ever
 * reaching memory.  Two forms with identical results: one launch per level with a wavefront per
 * (batch element, head), all heads streaming their weights on different CUs at once (the default
 * where `out` allows 16-byte reads: 16-byte aligned, strides multiples of 8 elements), or a single
 * launch with one workgroup per batch element that keeps the levels in LDS.
 * hsa_cross_update_top_tune(1) selects the single launch always, (0) the default, (-1) keeps the
 * setting; process-wide, initial value from HSA_CROSS_TOP_SINGLE.
 *
 *   src    [B, C, H*Dh]      dense rows; C a power of two >= 2 (see hsa_cross_update_top_rows)
 *   qkv    parents' q | k | v rows ([.., 3*H*Dh] per row), pointing at the first parent of the
 *          first level computed here; the C-1 parents follow level after level, root last
 *   w_kv   the Wk_y / Wv_y weights in the kernel's operand order, 2*(H*Dh)^2 elements,
 *          written by hsa_cross_update_pack_weights from the two [H*Dh, H*Dh] row-major
 *          weight matrices (row = output feature); repack after the weights change
 *   out    result rows, numbered like qkv's, H*Dh elements each
 *   *_bs, *_rs  batch / row strides in elements (0 = dense)
 *
 * hsa_cross_update_top_rows returns the largest C the single launch holds for this head layout
 * (0 = not handled: fp32, or a head size other than 32 / 64 / 128, or H*Dh not a multiple of
 * 128); hsa_cross_update_top_fwd returns HSA_ERR_UNSUPPORTED for such shapes, and for a larger C
 * unless `out` allows the launch per level, which takes any power of two.
 * hsa_cross_update_level_rows returns the C from which on a caller with such an `out` should hand
 * the remaining levels to hsa_cross_update_top_fwd instead of running a GEMM and a parent build
 * per level: every level where a head's key and value weights fit 128 KiB of LDS (heads of up to
 * 64 channels), else at least hsa_cross_update_top_rows and more for small batches (B*C <= 8192).
 * hsa_cross_update_level_tune (experiments and tests; -1 keeps a value): levels with at least
 * wg_min_tiles 16-row tiles run on the kernels that keep a head's weights in LDS (0: never), and
 * rows_limit, when positive, is the bound on B*C for every shape (0: the rule above).  Process-wide.
 */
int hsa_cross_update_top_tune(int single_launch);
int hsa_cross_update_level_tune(int wg_min_tiles, long rows_limit);
int hsa_cross_update_top_rows(int H, int Dh, int dtype);
int hsa_cross_update_level_rows(int B, int H, int Dh, int dtype);
int hsa_cross_update_pack_weights(const void *wk, const void *wv, void *packed, int H, int Dh,
                                  int dtype, void *stream);
int hsa_cross_update_top_fwd(const void *src, const void *qkv, const void *w_kv, void *out, int B,
                             int C, int H, int Dh, int64_t src_bs, int64_t qkv_bs, int64_t qkv_rs,
                             int64_t out_bs, int64_t out_rs, int dtype, void *stream);

/*
 * Whole tree in one call: level 1 from the leaves, every further level from the
 * previous level's output used as both child K and child V (the composition
 * Out_l = build_parent_nodes(Qp_l, Kp_l, Vp_l, Out_{l-1}, Out_{l-1}) of the op at
 * hierarchical_attention/ops/functional.py:271-272, i.e. the level loop of
 * hierarchical_attention/modules/attention.py:119-157 with an identity map
 * between levels).  Intermediate levels stay on chip; one kernel launch for the whole tree
 * (see hsa_build_tree_tune for the conditions).
 *
 *   qp, kp, vp  [B, N-1, H, D] level-concatenated (level 1 first, root last)
 *   k_leaf, v_leaf [B, N, H, D]
 *   out         [B, N-1, H, D] level-concatenated
 *   out2        optional second copy of the result (NULL to skip), e.g. the node rows of
 *               V_full when `out` is the node rows of K_full
 *   *_bs        batch strides in elements (0 = dense)
 */
int hsa_build_tree_fwd(const void *qp, const void *kp, const void *vp, const void *k_leaf,
                       const void *v_leaf, void *out, void *out2, int B, int N, int H, int D,
                       int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kleaf_bs,
                       int64_t vleaf_bs, int64_t out_bs, int64_t out2_bs, int dtype, void *stream);

/*
 * How hsa_build_tree_fwd runs, for experiments and tests (no counterpart in the reference).
 *   mode               0 = always a few levels per launch;
 *                      1 = (default) the whole tree in one kernel where that is faster: shapes
 *                          whose workgroups all fit on the chip at once;
 *                      2 = one kernel wherever the shape allows it (16-byte rows, power-of-two
 *                          head count, N >= 8).
 *                      In the single launch, workgroups finish their own subtrees and the last
 *                      one of each group to arrive continues upwards, counted by arrival
 *                      counters inside the library image (one slice per stream, and counters
 *                      of its own, never handed back, for every launch recorded into a graph;
 *                      a launch on the 32nd distinct stream, or recorded when those are used up
 *                      or before any eager call on the device, takes the multi-launch path).
 *   workgroup_threads  64 / 128 / 256 / 512: workgroup size of the single launch, 0 = by
 *                      problem size (default)
 * -1 keeps a value.  Process-wide.  Results do not depend on either.
 */
int hsa_build_tree_tune(int mode, int workgroup_threads);

/*
 * Topology tables.  Replaces build_tree_topology
 * (hierarchical_attention/ops/topology.py:6-150).
 *   idx [N, L] int32, mask [N, L] bytes (1 = masked), gather [2N-1, 3] int32;
 *   any of the three may be NULL to skip it.  N must be a power of two.
 * _host fills host memory on the calling thread; _device enqueues a fill kernel.
 */
int hsa_topology_host(int N, int causal, int32_t *idx, uint8_t *mask, int32_t *gather);
int hsa_topology_device(int N, int causal, int32_t *idx, uint8_t *mask, int32_t *gather,
                        void *stream);

/*
 * Initial span nodes: level-by-level pairwise means of x, each level rounded to
 * the element type.  Replaces generate_span_input_Y
 * (hierarchical_attention/ops/topology.py:153-169) for any N >= 2: level l holds N >> l
 * rows (an unpaired last row of a level has no parent), N - popcount(N) rows in all.
 *   x [B, N, C], y [B, N - popcount(N), C]  (N-1 rows for a power of two)
 */
int hsa_span_input_y(const void *x, void *y, int B, int N, int C, int dtype, void *stream);

/*
 * Backward of one parent-build level.
 * Replaces BuildParentNodesFunc.backward + build_parent_nodes_backward_kernel
 * (hierarchical_attention/ops/functional.py:66-111,
 *  hierarchical_attention/ops/triton/build_parents.py:106-204).  The three weights are
 * recomputed from the inputs, so the forward does not have to save them.
 *   dout, qp, kp, vp, dqp, dkp, dvp  [B, P, H, D];  kc, vc, dkc, dvc  [B, 2P, H, D]; all dense.
 */
int hsa_build_parents_bwd(const void *dout, const void *qp, const void *kp, const void *vp,
                          const void *kc, const void *vc, void *dqp, void *dkp, void *dvp, void *dkc,
                          void *dvc, int B, int P, int H, int D, int dtype, void *stream);

/*
 * hsa_build_parents_bwd on operands that are column slices of wider matrices: the backward of the
 * level step of HierarchicalAttention.cross_update_Y
 * (hierarchical_attention/modules/attention.py:119-157; the reference differentiates it through
 * BuildParentNodesFunc.backward, ops/functional.py:66-111, and the autograd of its Linear layers)
 * when the projections that feed the level are fused: q/k/v of the parents are thirds of one
 * [B, N-1, 3*H*D] projection, the children's k/v halves of one [B, 2P, 2*H*D] projection, and
 * their gradients are written into buffers of the same shapes (which the fused weight-gradient
 * and input-gradient GEMMs then read whole).
 *   batch_strides, row_strides   host arrays of 11 element counts in the order dout, qp, kp, vp,
 *                                kc, vc, dqp, dkp, dvp, dkc, dvc; an entry of 0, or a NULL array,
 *                                means dense
 */
int hsa_build_parents_strided_bwd(const void *dout, const void *qp, const void *kp, const void *vp,
                                  const void *kc, const void *vc, void *dqp, void *dkp, void *dvp,
                                  void *dkc, void *dvc, int B, int P, int H, int D,
                                  const int64_t *batch_strides, const int64_t *row_strides, int dtype,
                                  void *stream);

/*
 * Backward of the span attention for the canonical tables.
 * Replaces HierarchicalAttentionFunc.backward and its five kernels
 * (hierarchical_attention/ops/functional.py:171-264,
 *  hierarchical_attention/ops/triton/sparse_attn.py:185-623): the per-query pass recomputes the
 * weights and writes dQ plus the weights / dS workspaces, the per-key pass gathers dK and dV
 * (fp32 accumulation, written once in the element type; rows that nobody attends get zeros).
 *   q, dout, dq  [B, N, H, D];  k, v, dk, dv  [B, M, H, D], M >= 2N-1
 *   workspace    device memory of at least hsa_attn_bwd_workspace_bytes(...) bytes, provided by
 *                the caller (scratch only: nothing in it has to survive the call)
 *   algo         HSA_ATTN_AUTO: MFMA tile kernels when eligible (head size 32, 64 or 128; 16-bit:
 *                R <= 64; fp32: R <= 32: a query-stationary pass and a key-stationary pass that
 *                also sums the first pass's fp32 partial rows for the upper tree levels), else the
 *                gather kernels; both are deterministic (no atomics).
 *                Tensors that are not 16-byte aligned run on the gather kernels and need the
 *                workspace size reported for HSA_ATTN_GATHER.
 */
#include <stddef.h>
size_t hsa_attn_bwd_workspace_bytes(int B, int N, int M, int H, int D, int L, int R, int dtype, int algo);
int hsa_attn_bwd(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                 void *dv, void *workspace, size_t workspace_bytes, int B, int N, int M, int H, int D,
                 int L, int R, int causal, int dtype, int algo, void *stream);

/*
 * Span attention backward in one pass, for callers that kept two pieces of forward state, as the
 * reference's autograd Function keeps its Weights tensor for the same purpose
 * (hierarchical_attention/ops/functional.py:163-167, 171-264; kernels ops/triton/sparse_attn.py:185-623):
 *   out  [B, N, H, D]  the forward's output
 *   lse  [B, N, H] fp32 the log-sum-exp of every (query, head)'s biased logits in the log2 domain,
 *                      written by hsa_attn_fwd_lse
 * With them a strip of queries also finishes the gradients of its own leaf keys (what the
 * neighbouring strips' queries add is rebuilt from their Q, dO rows, lse and delta = <dO, out>),
 * so Q, dO, K, V are read once instead of twice.  Same results as hsa_attn_bwd to the rounding of
 * the element type; deterministic.  Canonical tables only; fp16 / bf16, 32 or 64 channels per
 * head (128 with the causal mask), window radius up to 16 (up to 32 with the causal mask), N >= 64,
 * 16-byte aligned tensors: anything else returns
 * HSA_ERR_UNSUPPORTED (hsa_attn_bwd_saved_workspace_bytes returns 0) and the caller uses
 * hsa_attn_bwd.  workspace: hsa_attn_bwd_saved_workspace_bytes(...) bytes, written before read.
 *
 * hsa_attn_fwd_lse: hsa_attn_fwd on the canonical tables that also writes lse (a variant of the
 * 16-bit tile kernel, built for window radius up to 16, or up to 32 with the causal mask; HSA_ERR_UNSUPPORTED otherwise, nothing
 * launched).
 */
int hsa_attn_fwd_lse(const void *q, const void *k, const void *v, void *out, float *lse, int B, int N, int M,
                     int H, int D, int L, int R, int causal, int dtype, void *stream);
size_t hsa_attn_bwd_saved_workspace_bytes(int B, int N, int M, int H, int D, int L, int R, int causal, int dtype);
int hsa_attn_bwd_saved(const void *q, const void *k, const void *v, const void *out, const float *lse,
                       const void *dout, void *dq, void *dk, void *dv, void *workspace, size_t workspace_bytes,
                       int B, int N, int M, int H, int D, int L, int R, int causal, int dtype, void *stream);
/*
 * Query blocks one wavefront of hsa_attn_bwd_saved walks (no counterpart in the reference; for
 * experiments and tests, results do not depend on it beyond rounding): 0 = automatic (eight where
 * that many wavefronts still fill the chip, 64 channels per head and the sequence has a multiple
 * of eight blocks; 16 or 32 where that still leaves four rounds of wavefronts; else four), or 4,
 * 8, 16, 32 (the largest of these up to the argument that divides the sequence's block count).
 * Process-wide.
 */
int hsa_attn_bwd_saved_tune(int strip_blocks);

/*
 * Backward of the span attention from caller-supplied tables, replacing
 * HierarchicalAttentionFunc.backward for tables that are not the canonical ones
 * (hierarchical_attention/ops/functional.py:171-264): like the reference's kernels
 * (ops/triton/sparse_attn.py:185-623) it takes each query's key rows and dead slots from
 * idx [N, L] / mask [N, L] (mask NULL: nothing masked; an entry outside [0, M) is a dead slot),
 * keeps the tree's row layout (level l starts at row 2N - (N >> (l-1)), a node of level l collects
 * from 2^l consecutive queries) and reads from gather [rows, 3] only each node row's first
 * attending query (column 0; -1: none).  `causal` restricts the window to keys <= the query, as the
 * reference does when a mask table is given.  Per-query / per-key-row gather kernels, any head
 * size, fp32 workspaces of hsa_attn_bwd_workspace_bytes(..., HSA_ATTN_GATHER) bytes; deterministic.
 */
int hsa_attn_bwd_tables(const void *q, const void *k, const void *v, const void *dout, const int32_t *idx,
                        const uint8_t *mask, const int32_t *gather, void *dq, void *dk, void *dv, void *workspace,
                        size_t workspace_bytes, int B, int N, int M, int H, int D, int L, int R, int causal, int dtype,
                        void *stream);

/*
 * hsa_attn_bwd for callers that cannot allocate device memory or hand over a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference: its backward allocates its workspaces through torch
 * (hierarchical_attention/ops/functional.py:171-264).  Same arguments, kernels and results as
 * hsa_attn_bwd, but the scratch is a buffer of HSA_ATTN_BWD_STATIC_BYTES that is part of the
 * library's device image (each GPU the library runs on holds one until the process ends); the
 * call allocates nothing.  Problems with hsa_attn_bwd_workspace_bytes(...) above that size are
 * refused with HSA_ERR_UNSUPPORTED.  Every call on a GPU shares that GPU's buffer: calls that
 * overlap on one GPU (two streams, two host threads) race; calls on one stream do not.
 * Nothing in the buffer has to be cleared between calls.
 * The buffer's address on a GPU is looked up once per GPU: by hsa_attn_bwd_static_capacity() (the
 * set-up call: make it once on every GPU before recording a graph there) or by the first
 * hsa_attn_bwd_static on an ordinary stream.  A first use on a stream that is being captured is
 * refused with HSA_ERR_UNSUPPORTED instead of doing the look-up inside the capture.
 */
#define HSA_ATTN_BWD_STATIC_BYTES (32u << 20)
size_t hsa_attn_bwd_static_capacity(void);
int hsa_attn_bwd_static(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                        void *dv, int B, int N, int M, int H, int D, int L, int R, int causal, int dtype,
                        int algo, void *stream);

/*
 * Backward of the initial span nodes (the reference differentiates generate_span_input_Y,
 * hierarchical_attention/ops/topology.py:153-169, through torch autograd):
 *   dx[b, n, :] = sum over levels l >= 1 with n >> l < N >> l of 2^-l * dy[b, level l node n >> l, :]
 *   dy [B, N - popcount(N), C], dx [B, N, C]
 */
int hsa_span_input_y_bwd(const void *dy, void *dx, int B, int N, int C, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HSA_GFX950_H */
