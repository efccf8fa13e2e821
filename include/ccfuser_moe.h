/*
 * ccfuser_moe.h -- C ABI of the MI355X (gfx950) MoE layer forward.
 *
 * One shared library, libccfuser_moe.so, exports the functions below.  They
 * take raw device pointers, sizes and a HIP stream, enqueue kernels on that
 * stream and return without synchronising the host.  No torch types cross
 * this boundary.  Every function returns 0 on success or a CCF_ERR_* code; the
 * text of the last error on the calling thread is available from
 * ccf_last_error().  Nothing here calls exit().
 *
 * Each declaration names the reference interface it replaces; paths are
 * relative to the reference repository root.
 *
 * Conventions
 *   - fp16 tensors are IEEE binary16, row-major, rows 16-byte aligned
 *     (d_model and d_ffn multiples of 8; the grouped GEMMs need multiples of 64).
 *   - expert weights keep the layout of the reference's parameter containers
 *     (mix_moe/mix_moe/linear.py:198-202): w1 [E, d_ffn, d_model],
 *     b1 [E, d_ffn], w2 [E, d_model, d_ffn], b2 [E, d_model].  The reference
 *     transposes them to [E, K, N] on every call (linear.py:74, 129); this
 *     library consumes the stored layout directly.
 *   - "flat index" i = token * top_k + slot, as in the reference's pos vector.
 *   - workspaces are caller-owned device memory, 256-byte aligned; the
 *     *_workspace_bytes functions give the size to allocate.
 */
#ifndef CCFUSER_MOE_H
#define CCFUSER_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *ccf_stream_t; /* a hipStream_t; NULL is the null stream */

enum {
  CCF_OK = 0,
  CCF_ERR_ARG = 1,         /* null pointer, negative size, bad enum            */
  CCF_ERR_SHAPE = 2,       /* a size the kernels do not support                */
  CCF_ERR_WORKSPACE = 3,   /* workspace missing or too small                   */
  CCF_ERR_HIP = 4,         /* a HIP runtime call or a launch failed            */
  CCF_ERR_UNSUPPORTED = 5  /* dtype or option not implemented                  */
};

enum { CCF_F16 = 0, CCF_F32 = 1 };

/* Library version (major*10000 + minor*100 + patch). */
int ccf_version(void);

/* Text of the last error raised on this thread ("" if none). */
const char *ccf_last_error(void);

/*
 * Tuning knobs (no counterpart in the reference).  Process-wide; not meant to
 * be changed while work is in flight.
 *   "gemm_variant"    0 (default, also -1) = the grouped GEMMs run as persistent workgroups of four wavefronts,
 *                     one per CU; 1 = one workgroup per tile for every K (otherwise only K < 256 runs that
 *                     way); 2 = as 0; 3 = the forward GEMMs as persistent workgroups of eight wavefronts
 *                     (same bits, measured no faster)
 *   "split_tail"      0 = off, 1 = default, n > 1 = for K of n*64 and more: the tiles of a launch's
 *                     last, partly filled round are cut along K and reduced by a second kernel
 *   "split_parts"     2..8 (default 8): most parts such a tile is cut into
 *   "skinny"          0 = off, 1 = default: rows an expert has beyond its full 256-row tiles (at most 128:
 *                     one or two tiles of 64 rows) may run as 64-row tiles in a few workgroups set aside
 *                     for them or cut along K over all workgroups, when the tile plan's cost model says
 *                     that beats a padded 256-row tile; n > 1 sets the model's cost of
 *                     such a tile's K step in percent of a 256-row tile's (default 70); -n (1..4) forces
 *                     them with n workgroups per XCD; -5 forces them as a launch of their own behind the
 *                     persistent kernel, cut along K over all workgroups (the model's third choice); -6 forces
 *                     them cut along K inside the persistent launch, each workgroup running its range at
 *                     some point between its 256-row tiles (the fourth)
 *   "skinny_tail"     0/1 (default 0): the plan may choose that third way (it costs a launch that the
 *                     fourth way does without, and measured slower wherever both apply)
 *   "split_inside"    0/1 (default 1): the parts of a split last round are run by the persistent workgroups
 *                     themselves, each one part behind its tiles, instead of by a launch of their own
 *   "skinny_positions" 0 (default) or n >= 2: over how many points in time the fourth way spreads the
 *                     workgroups' ranges (0: one in front of every round of tiles and one behind the last;
 *                     2: half of the workgroups in front of all their tiles, half behind)
 *   "fused_combine"   0/1 (default 0): ccf_moe_forward with top_k = 2 adds the gate-weighted expert outputs
 *                     into the output in the second GEMM's epilogue (packed fp16 atomic adds onto zeros)
 *                     instead of running the combine pass; measured slower, kept for comparison
 *   "route_rows_max"  0..32768 (default 16384): the largest table of per-run expert counts (entries) that the
 *                     routing stage's last launch sums itself instead of running a scan launch; in
 *                     ccf_moe_forward the gate kernel leaves such a table when it fits (and top_k is a power
 *                     of two), and the routing stage is then one launch.  0 = always histogram, scan, pos
 *   "gate_slots"      0, 1, 2 or 4: parts of K a gate wavefront works on at a time, which divides the tokens
 *                     of a workgroup by the same number (0 = chosen by the token count)
 *   "dgrad_transpose" 0/1: the backward's input-gradient GEMM runs on a transposed copy of the
 *                     weight instead of reading the stored one
 *   "wgrad_transpose" 0/1: the backward's weight-gradient GEMM runs on transposed copies of the two
 *                     activation matrices instead of reading them row-major
 *   "gate_waves"      1..8 (default 8): most wavefronts of a gate workgroup; each takes other parts of K
 *   "gate_stream"     -1 (default), 0 or 1: form of the fp16 gate kernel.  1: every wavefront takes its tokens
 *                     through all of K alone, in one stream of loads and MFMAs; 0: the wavefronts of a
 *                     workgroup share the parts of K; -1: the first with 1024 wavefronts of tokens or more
 */
int ccf_set_option(const char *name, int value);

/* ------------------------------------------------------------------ gate */

/*
 * Top-k gate: logits = x * wg^T + bg (fp32 accumulation in a fixed order:
 * parts of 128 consecutive K elements, each a chain of multiply-adds in
 * ascending K from zero, the part sums added in ascending order, the bias
 * last; rounded once to the input dtype), top-k per token (slot 0 = largest,
 * ties to the lower expert id), softmax over the k selected logits.
 * Replaces NaiveGate.forward, mix_moe/mix_moe/gates/naive_gate.py:26-45.
 *   x [tokens, d_model], wg [tot_expert, d_model], bg [tot_expert] or NULL,
 *   idx_out int64 [tokens, top_k], score_out [tokens, top_k] in the input
 *   dtype, logits_out [tokens, tot_expert] in the input dtype or NULL.
 *   dtype is CCF_F16 or CCF_F32.  d_model % 8 == 0, 1 <= top_k <= 8,
 *   top_k <= tot_expert <= 1024.
 */
int ccf_gate_topk_softmax(const void *x, const void *wg, const void *bg,
                          int tokens, int d_model, int tot_expert, int top_k,
                          int dtype, int64_t *idx_out, void *score_out,
                          void *logits_out, ccf_stream_t stream);

/* Bytes of workspace ccf_gate_backward needs when it returns the bias gradient (no counterpart in the reference). */
size_t ccf_gate_backward_workspace_bytes(int tokens, int tot_expert);

/*
 * Backward of the gate's softmax over the k selected logits and of the selection:
 *   grad_logits[t, idx[t, j]] = s_j * (g_j - sum_i s_i g_i),  s = score[t, :], g = grad_score[t, :],
 * zero in every other column (fp32 arithmetic, rounded once to fp16), and grad_bias[e] = the sum of column e
 * over the tokens (of the unrounded values, in a fixed order).  The two products of grad_logits with the input
 * and with the gate weight, which complete the linear layer's backward, are plain GEMMs and stay with the caller.
 * What autograd derives for NaiveGate.forward's topk -> softmax, mix_moe/mix_moe/gates/naive_gate.py:31-38.
 *   score, grad_score fp16 [tokens, top_k]; idx int64 [tokens, top_k] (entries outside 0 .. tot_expert-1 are
 *   skipped); grad_logits fp16 [tokens, tot_expert]; grad_bias fp16 [tot_expert] or NULL (then no workspace).
 */
int ccf_gate_backward(const void *score, const void *grad_score, const int64_t *idx,
                      int tokens, int top_k, int tot_expert, void *grad_logits,
                      void *grad_bias, void *workspace, size_t workspace_bytes,
                      ccf_stream_t stream);

/* --------------------------------------------------------------- routing */

/* Bytes of workspace ccf_route / ccf_assign_pos need for n_flat indices. */
size_t ccf_route_workspace_bytes(int n_flat, int num_expert);

/*
 * Histogram of gate indices, accumulated into expert_count (the caller zero
 * fills, as mix_moe/mix_moe/functions.py:85-88 does).  Entries < 0 or
 * >= num_expert are skipped.
 * Replaces _expert_count / expert_count_kernel,
 * mix_moe/csrc/cuda/local_exchange.cu:37-79, 98-108.
 */
int ccf_expert_count(const int64_t *gate_idx, int n_flat, int32_t *expert_count,
                     int num_expert, ccf_stream_t stream);

/*
 * pos from an inclusive cumulative count: the flat indices routed to expert e
 * fill pos[cum[e]-count[e] .. cum[e]) in ascending order; on return
 * cum_count[e] holds the start of that segment (the reference decrements it
 * once per routed index, so it ends at the same value).
 * Replaces _assign_pos / assign_pos_kernel,
 * mix_moe/csrc/cuda/local_exchange.cu:6-27, 81-96, whose order inside a
 * segment is left to an atomic race.
 */
int ccf_assign_pos(int32_t *cum_count, const int64_t *gate_idx, int n_flat,
                   int num_expert, int64_t *pos, void *workspace,
                   size_t workspace_bytes, ccf_stream_t stream);

/*
 * Count + exclusive scan + deterministic pos in one call, with optional
 * capacity limiting, all on the device and without a host synchronisation.
 * Replaces perpare_expert_assignment at world_size 1,
 * mix_moe/mix_moe/functions.py:83-105.
 *   gate_idx int64 [n_flat] (-1 = already dropped)
 *   capacity  rows an expert keeps (first come in flat order), < 0 = no limit
 *   counts  int32 [num_expert]      kept rows per expert
 *   offsets int32 [num_expert + 1]  exclusive scan; offsets[num_expert] = R
 *   pos     int64 [n_flat]          first R entries valid
 *   src_row int32 [n_flat] or NULL  pos[j] / top_k  (row of x to read)
 *   dst_row int32 [n_flat] or NULL  pos[j]          (row of y_flat to write)
 *   inv_pos int32 [n_flat] or NULL  j for kept flat index i, else -1
 *   idx_kept int64 [n_flat] or NULL gate_idx with dropped entries set to -1
 */
int ccf_route(const int64_t *gate_idx, int n_flat, int num_expert, int top_k,
              int capacity, int32_t *counts, int32_t *offsets, int64_t *pos,
              int32_t *src_row, int32_t *dst_row, int32_t *inv_pos,
              int64_t *idx_kept, void *workspace, size_t workspace_bytes,
              ccf_stream_t stream);

/*
 * ccf_route without a workspace and without any allocation: the per-chunk count
 * table that ccf_route keeps in its workspace lives in a 1 MiB device array
 * inside the library image instead.  It has no counterpart in the reference and is for
 * callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  Same arguments and
 * results as ccf_route.  Limit: ceil(n_flat / 1024) * num_expert must not exceed
 * ccf_route_static_max_entries() (262144), e.g. 1M indices for 256 experts;
 * larger inputs return CCF_ERR_SHAPE.  All calls on one GPU share that GPU's
 * array: calls that overlap in time on one GPU (different streams or threads)
 * race and must be serialised by the caller.
 */
int ccf_route_static(const int64_t *gate_idx, int n_flat, int num_expert, int top_k,
                     int capacity, int32_t *counts, int32_t *offsets, int64_t *pos,
                     int32_t *src_row, int32_t *dst_row, int32_t *inv_pos,
                     int64_t *idx_kept, ccf_stream_t stream);

/* Entries of the built-in scratch of ccf_route_static (no counterpart in the reference). */
int ccf_route_static_max_entries(void);

/*
 * Block plan in the reference's wire format, built on the device from the
 * per-expert counts: what AsyncExpertAssignment.divide_into_block computes in
 * Python loops and ships with seven blocking copies
 * (mix_moe/mix_moe/transformer.py:150-250) at world_size 1 with the identity
 * expert plan.  Per expert the full block_size-row blocks and a shorter tail;
 * full blocks and tails interleaved l0, r0, l1, r1, ... (transformer.py:199).
 * Unlike the reference an expert with fewer than block_size rows keeps its
 * tail block (transformer.py:184-193 plans a tail only next to a full block).
 *   counts int32 [num_expert]
 *   expert_ids, ranks, lens, start_addrs, expert_block_ids int32 [max_blocks];
 *     max_blocks >= sum(counts) / block_size + num_expert holds every plan,
 *     blocks beyond max_blocks are not written; ranks[] = rank
 *   expert_block_id_idxs int32 [num_expert + 1]  CSR expert -> expert_block_ids
 *   block_nums int32 [2]  {total_block_num, remote_block_num (= tails)}
 * local_expert_id_indexs of the reference equals expert_ids on one GPU.
 */
int ccf_plan_blocks(const int32_t *counts, int num_expert, int block_size, int rank,
                    int max_blocks, int32_t *expert_ids, int32_t *ranks, int32_t *lens,
                    int32_t *start_addrs, int32_t *expert_block_ids,
                    int32_t *expert_block_id_idxs, int32_t *block_nums,
                    ccf_stream_t stream);

/*
 * Rows addressed by (start, len, expert) triples -> per-expert counts,
 * offsets and a row list grouped by expert (segment order, then row order).
 * The triple is what the reference plans per block
 * (mix_moe/mix_moe/transformer.py:242-250: start_addrs, lens, expert_ids) and
 * its kernels address blocks with (mix_moe/csrc/cuda/mix_gemm.cu:296-301).
 *   rows int32 [total_rows] out; counts int32 [E]; offsets int32 [E+1].
 */
int ccf_segments_to_rows(const int32_t *seg_start, const int32_t *seg_len,
                         const int32_t *seg_expert, int n_seg, int num_expert,
                         int total_rows, int32_t *counts, int32_t *offsets,
                         int32_t *rows, ccf_stream_t stream);

/* ------------------------------------------------- row moves and combine */

/*
 * out[j, :] = in[pos[j], :] for j < pos_len (fp16 rows of `hidden`).
 * Replaces _local_scatter_launch, mix_moe/csrc/cuda/mix_moe_kernel.cu:18-42
 * (which needs pos_len % 32 == 0; this one does not).
 */
int ccf_local_scatter(const void *in, void *out, const int32_t *pos,
                      int pos_len, int hidden, ccf_stream_t stream);

/*
 * out[pos[j], :] = in[j, :].
 * Replaces _local_gather_launch, mix_moe/csrc/cuda/mix_moe_kernel.cu:56-79.
 */
int ccf_local_gather(const void *in, void *out, const int32_t *pos,
                     int pos_len, int hidden, ccf_stream_t stream);

/*
 * out[t, :] = sum_s score[t, s] * y_flat[t*top_k + s, :], fp32 accumulation,
 * one rounding to fp16.  If inv_pos is not NULL, slots with inv_pos < 0
 * (dropped) contribute zero and their y_flat rows are never read.
 * Replaces the bmm combine of MixMOE.forward, mix_moe/mix_moe/layers.py:550-559.
 */
int ccf_combine(const void *y_flat, const void *score, const int32_t *inv_pos,
                void *out, int tokens, int top_k, int hidden,
                ccf_stream_t stream);

/* ------------------------------------------------------------ expert FFN */

/* Bytes of workspace the FFN entry points need (the device-built tile plan). */
size_t ccf_ffn_workspace_bytes(int max_rows, int num_expert, int d_model, int d_ffn);

/*
 * Diagnostic (no counterpart in the reference): what the tile plan that the last call left in
 * `workspace` decided, for which = 1 (the first GEMM: ccf_ffn1_forward, ccf_ffn1_forward_keep) or 2
 * (ccf_ffn2_forward); for ccf_moe_forward's plans pass the FFN part of its workspace.  Copies a few
 * integers to the host and synchronises the stream.  info (host, 8 ints):
 *   [0] tiles of the split last round, [1] parts each is cut into (0 = not split)
 *   [2] skinny tiles, [3] workgroups per XCD that run them beside the 256-row tiles,
 *   [4] skinny tiles per XCD, [5] K steps per workgroup when they are cut along K: > 0 as a launch of their
 *       own, < 0 inside the persistent launch, 0 = not cut
 *   [6] workgroups of the persistent launch (0 = one workgroup per tile), [7] worst-case tile count
 */
int ccf_ffn_plan_info(const void *workspace, int max_rows, int num_expert, int d_model, int d_ffn,
                      int which, int32_t *info, ccf_stream_t stream);

/*
 * FFN1 as a grouped GEMM with the scatter fused into the A-tile loads:
 *   h[dst_row[j], :] = gelu(x[src_row[j], :] * w1[e]^T + b1[e])   for offsets[e] <= j < offsets[e+1]
 * erf-form GELU, fp16 operands, fp32 MFMA accumulation, fp16 h.
 * src_row / dst_row NULL mean row j.  offsets lives on the device; max_rows
 * bounds offsets[num_expert].  apply_gelu = 0 stores the pre-activation instead.
 * Replaces _MixMOE::first_gemm_forward -> first_mix_gemm -> moe_first_mm,
 * mix_moe/csrc/mix_moe.h:236-298, mix_moe/csrc/cuda/mix_gemm.cu:282-436, 557-610,
 * together with the activation the reference runs as a separate kernel
 * (mix_moe/mix_moe/transformer.py:88).
 */
int ccf_ffn1_forward(const void *x, const int32_t *src_row, const int32_t *dst_row,
                     const int32_t *offsets, int max_rows, int num_expert,
                     int d_model, int d_ffn, const void *w1, const void *b1,
                     int apply_gelu, void *h, void *workspace,
                     size_t workspace_bytes, ccf_stream_t stream);

/*
 * FFN2 as a grouped GEMM with the un-permute fused into the epilogue:
 *   y[dst_row[j], :] = (h[src_row[j], :] * w2[e]^T + b2[e]) * (row_scale ? row_scale[j] : 1)
 * src_row / dst_row NULL mean row j.  Rows of y that no j maps to are left
 * untouched.
 * Replaces _MixMOE::second_gemm_forward -> second_mix_gemm -> moe_second_mm and
 * the index_copy_ that follows it, mix_moe/csrc/mix_moe.h:390-437,
 * mix_moe/csrc/cuda/mix_gemm.cu:439-555, 668-720.
 */
int ccf_ffn2_forward(const void *h, const int32_t *src_row, const int32_t *dst_row,
                     const int32_t *offsets, int max_rows, int num_expert,
                     int d_model, int d_ffn, const void *w2, const void *b2,
                     const void *row_scale, void *y, void *workspace,
                     size_t workspace_bytes, ccf_stream_t stream);

/* ------------------------------------------------------- the whole layer */

/* Bytes of workspace ccf_moe_forward needs. */
size_t ccf_moe_workspace_bytes(int tokens, int d_model, int d_ffn, int num_expert, int top_k);

/*
 * The MoE layer forward on one GPU: gate -> count/scan/pos (with optional
 * capacity) -> FFN1 (gather fused) -> GELU -> FFN2 (un-permute fused) ->
 * gate-weighted combine.  out [tokens, d_model] fp16.
 * Replaces MixMOETransformerMLP.forward, mix_moe/mix_moe/transformer.py:475-497,
 * i.e. AsyncExpertAssignment.process_data (376-402) followed by MixMOE.forward
 * (mix_moe/mix_moe/layers.py:501-559); its single-call C++ form is
 * _MixMOE::forward, mix_moe/csrc/mix_moe.h:507-598.
 * Optional outputs (NULL to skip): idx_out int64 [tokens*top_k] (after
 * capacity), score_out fp16 [tokens*top_k], pos_out int64 [tokens*top_k],
 * counts_out int32 [num_expert], offsets_out int32 [num_expert+1].
 */
int ccf_moe_forward(const void *x, const void *wg, const void *bg,
                    const void *w1, const void *b1, const void *w2, const void *b2,
                    int tokens, int d_model, int d_ffn, int num_expert, int top_k,
                    int capacity, void *out, int64_t *idx_out, void *score_out,
                    int64_t *pos_out, int32_t *counts_out, int32_t *offsets_out,
                    void *workspace, size_t workspace_bytes, ccf_stream_t stream);

/*
 * Profiling hook (no counterpart in the reference).  Gives up to six hipEvent_t
 * handles; every later ccf_moe_forward on this thread records them on its
 * stream: [0] before the gate, then after the gate, the count/scan/pos, FFN1,
 * FFN2 and the combine.  ccf_moe_ffn_segments records the same six, with the
 * regrouping of the segments as its count/scan/pos stage and nothing between
 * [0] and [1] or [4] and [5].  count = 0 switches the recording off.
 */
int ccf_moe_forward_set_events(void *const *events, int count);

/* Bytes of workspace ccf_moe_ffn_segments needs. */
size_t ccf_segments_workspace_bytes(int total_rows, int n_seg, int num_expert,
                                    int d_model, int d_ffn);

/*
 * One GPU's expert-parallel share: the expert FFN over an inbound buffer whose
 * rows are addressed by (start, len, expert) triples; y[r, :] is the FFN
 * output of inbound row r (same layout as x, ready to be returned to the
 * senders).  Rows no triple covers are left untouched.
 * Replaces the block-addressed form of the two fused kernels, where each
 * block carries (expert_ids, start_addrs, lens),
 * mix_moe/csrc/cuda/mix_gemm.cu:282-345, 439-490, as called from
 * _MixMOE::forward, mix_moe/csrc/mix_moe.h:539-575.
 */
int ccf_moe_ffn_segments(const void *x, const int32_t *seg_start,
                         const int32_t *seg_len, const int32_t *seg_expert,
                         int n_seg, int total_rows, int d_model, int d_ffn,
                         int num_expert, const void *w1, const void *b1,
                         const void *w2, const void *b2, void *y,
                         void *workspace, size_t workspace_bytes,
                         ccf_stream_t stream);

/* ------------------------------------------------------------ backward */

/*
 * Backward of ccf_combine (the bmm at mix_moe/mix_moe/layers.py:556, which the
 * reference leaves to autograd):
 *   grad_y_flat[t*k+s, :] = score[t*k+s] * grad_out[t, :]
 *   grad_score[t*k+s]     = <grad_out[t, :], y_flat[t*k+s, :]>
 * both zero for dropped slots (inv_pos[i] < 0; inv_pos NULL = none dropped).
 * All fp16; grad_y_flat [tokens*top_k, hidden], grad_score [tokens*top_k].
 */
int ccf_combine_backward(const void *grad_out, const void *y_flat, const void *score,
                         const int32_t *inv_pos, int tokens, int top_k, int hidden,
                         void *grad_y_flat, void *grad_score, ccf_stream_t stream);

/*
 * ccf_ffn1_forward with the erf GELU, for a forward whose backward will follow:
 * act = gelu(x[src_row] * w1[e]^T + b1[e]) as ccf_ffn1_forward(apply_gelu = 1)
 * writes it, and the pre-activation besides, both [max_rows, d_ffn] in expert
 * order.  The reference's first_gemm_forward (mix_moe/csrc/mix_moe.h:236-298)
 * returns the pre-activation and applies the activation as a separate torch op
 * (mix_moe/mix_moe/transformer.py:88), which keeps both for autograd the same way.
 * Workspace: ccf_ffn_workspace_bytes.
 */
int ccf_ffn1_forward_keep(const void *x, const int32_t *src_row, const int32_t *offsets,
                          int max_rows, int num_expert, int d_model, int d_ffn,
                          const void *w1, const void *b1, void *h_pre, void *act,
                          void *workspace, size_t workspace_bytes, ccf_stream_t stream);

/* Workspace of ccf_ffn1_backward / ccf_ffn2_backward (transposed weight, transposed
 * and padded activations, tile plans, bias partial sums).  No counterpart in the
 * reference, whose backward allocates its temporaries per call
 * (mix_moe/csrc/mix_moe.h:316, 340-343, 458-460). */
size_t ccf_ffn_backward_workspace_bytes(int max_rows, int num_expert, int d_model, int d_ffn);

/*
 * Backward of ccf_ffn2_forward.  Replaces _MixMOE::second_gemm_backward,
 * mix_moe/csrc/mix_moe.h:439-505 (MixMOELinear2.backward,
 * mix_moe/mix_moe/linear.py:148-173): the row scatter of grad_out into expert
 * order (453-454) is the row index of the A loads, the input gradient is the
 * grouped GEMM on the transposed weight, the weight gradient
 * (launch_compute_weight_grad, 497-503) is the same grouped GEMM contracting
 * over each expert's rows; grad_b2 is the column sum of the gradient rows (the
 * reference returns it uninitialised, 489).
 *   grad_y_flat fp16 [n_flat, d_model]  gradient of ccf_ffn2_forward's y
 *   act         fp16 [max_rows, d_ffn]  the forward's input, expert order
 *   h_pre       fp16 [max_rows, d_ffn] or NULL.  Given (from ccf_ffn1_forward_keep,
 *               act = gelu(h_pre)), grad_act is taken through the GELU in the GEMM's
 *               epilogue and is the gradient of h_pre, ready for ccf_ffn1_backward
 *               (the reference leaves the activation's backward to autograd,
 *               mix_moe/mix_moe/transformer.py:88)
 *   dst_row, offsets                    as in the forward
 *   w2          fp16 [E, d_model, d_ffn]
 *   grad_act    fp16 [max_rows, d_ffn]  out; rows >= offsets[E] untouched
 *   grad_w2     fp16 [E, d_model, d_ffn], grad_b2 fp16 [E, d_model]  out
 * d_model and d_ffn must be multiples of 64.
 */
int ccf_ffn2_backward(const void *grad_y_flat, const void *act, const void *h_pre,
                      const int32_t *dst_row,
                      const int32_t *offsets, int max_rows, int num_expert, int d_model,
                      int d_ffn, const void *w2, void *grad_act, void *grad_w2,
                      void *grad_b2, void *workspace, size_t workspace_bytes,
                      ccf_stream_t stream);

/*
 * Backward of ccf_ffn1_forward without the fused GELU (grad_h is the gradient
 * of the pre-activation).  Replaces _MixMOE::first_gemm_backward,
 * mix_moe/csrc/mix_moe.h:300-388 (MixMOELinear1.backward,
 * mix_moe/mix_moe/linear.py:91-113).
 *   grad_h      fp16 [max_rows, d_ffn]  expert order
 *   x           fp16 [tokens, d_model]  the forward's input, read through src_row
 *   w1          fp16 [E, d_ffn, d_model]
 *   grad_x_flat fp16 [n_flat, d_model]  out: row dst_row[j] = gradient of sorted
 *               row j; rows of dropped slots untouched.  The reference's
 *               index_add_ onto tokens (359-365) is ccf_combine over these rows
 *               with unit scores.
 *   grad_w1     fp16 [E, d_ffn, d_model], grad_b1 fp16 [E, d_ffn]  out
 */
int ccf_ffn1_backward(const void *grad_h, const void *x, const int32_t *src_row,
                      const int32_t *dst_row, const int32_t *offsets, int max_rows,
                      int num_expert, int d_model, int d_ffn, const void *w1,
                      void *grad_x_flat, void *grad_w1, void *grad_b1, void *workspace,
                      size_t workspace_bytes, ccf_stream_t stream);

/*
 * Backward of ccf_ffn1_forward_keep: through the erf GELU and the first linear layer in one
 * call.  grad_act holds the gradient of act = gelu(h_pre) on entry; the call multiplies it by
 * gelu'(h_pre) in place (in the pass that also transposes it for the weight gradient), so on
 * return it holds the gradient of the pre-activation, and everything else is ccf_ffn1_backward
 * on that.  The reference leaves this product to autograd's GeluBackward between
 * MixMOELinear2.backward and MixMOELinear1.backward (mix_moe/mix_moe/transformer.py:88,
 * mix_moe/mix_moe/linear.py:91-113); mix_moe/csrc/mix_moe.h:300-388 is the rest.
 *   grad_act    fp16 [max_rows, d_ffn]  in/out, expert order
 *   h_pre       fp16 [max_rows, d_ffn]  from ccf_ffn1_forward_keep
 *   the other arguments as in ccf_ffn1_backward
 */
int ccf_ffn1_backward_gelu(void *grad_act, const void *h_pre, const void *x, const int32_t *src_row,
                           const int32_t *dst_row, const int32_t *offsets, int max_rows,
                           int num_expert, int d_model, int d_ffn, const void *w1,
                           void *grad_x_flat, void *grad_w1, void *grad_b1, void *workspace,
                           size_t workspace_bytes, ccf_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* CCFUSER_MOE_H */
