/* C ABI of the MI355X tree-mask attention / Gated DeltaNet library (libspinf_tree.so).
 *
 * Plain pointers and sizes only; every function returns SPINF_OK (0) or a negative SPINF_E_* code and never throws.
 * spinf_last_error() returns a thread-local message for the last failing call.  Device pointers are HIP device
 * pointers of the current device; `stream` is a hipStream_t passed as void* (NULL = the default stream).  All
 * launches are asynchronous on that stream.
 *
 * Each entry point names the reference interface (file:line under the reference tree) that it stands in for.
 */
#ifndef SPINF_TREE_H
#define SPINF_TREE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPINF_OK 0
#define SPINF_E_ARG (-1)      /* bad argument (null pointer, unsupported shape, misaligned stride) */
#define SPINF_E_HIP (-2)      /* a HIP runtime call failed */
#define SPINF_E_NOMEM (-3)    /* host allocation failed */

#define SPINF_QTILE 128       /* query tokens per tile (the reference's BLOCK, spinf_serve/packer.py:22) */
#define SPINF_KTILE 64        /* key tokens per tile entry */
#define SPINF_SUB 32          /* rows / keys of one sub-tile bit */

const char* spinf_last_error(void);
int spinf_version(void);

/* ------------------------------------------------------------------------------------------------ tile plan
 * Replaces block_tables() (spinf_serve/packer.py:426-491) and the BlockMask built from it
 * (spinf_serve/scorer.py:207-238): the stream metadata is compiled into, per 128-token query tile, the ascending list
 * of 64-key tiles it may see.  No dense mask and no nb x nb table is built.  Host only, deterministic, thread-safe.
 *
 *   art, end, pos   [n] int32 host arrays: job slot (-1 pad), exclusive subtree end, depth on the path
 *   window          sliding window of the layer (pos[q] - pos[k] < window); <= 0 for the global layers
 *
 * Entry e of query tile t (qt_ptr[t] <= e < qt_ptr[t+1]) names key tile kv_idx[e]; kv_bits[e] bit (2*w + s) says that
 * rows 32w..32w+31 of the query tile see at least one key of keys 32s..32s+31 of the key tile, bit 8 + (2*w + s) that
 * some pair of that 32 x 32 block is masked (the kernel then evaluates spinf_serve/scorer.py:173-177 per element).
 * order[] lists the query tiles job by job, heaviest first inside a job.
 *
 * spinf_tileplan_schedule turns the plan into the kernel's work lists for a given number of head groups (query heads /
 * heads per work item, see spinf_attn_heads_per_item): items[4*i..4*i+3] = {query tile, first entry, entries | head
 * group << 20, first key tile}; list_ptr[0..8] delimits eight lists of roughly equal weight (one per XCD), inside a list
 * the items of a job stay together, head group by head group, heaviest query tile first; the lightest items of a list
 * (8 % of its weight) sit at its end.  The order of the items never changes a result.
 */
typedef struct spinf_tileplan spinf_tileplan;

int spinf_tileplan_build(const int32_t* art, const int32_t* end, const int32_t* pos, int64_t n, int32_t window,
                         spinf_tileplan** out);
/* The same with image groups (spinf_serve/scorer.py:184-198, spinf_serve/packer.py:456-468,485): grp [n], -1 = no group; tokens
 * of one group also see each other both ways.  grp_mode 1: also past the window (the "unified" checkpoint: every layer);
 * 2: only within the window (sliding layers of the other checkpoint; its global layers take no groups). */
int spinf_tileplan_build_groups(const int32_t* art, const int32_t* end, const int32_t* pos, const int32_t* grp, int32_t grp_mode,
                                int64_t n, int32_t window, spinf_tileplan** out);
/* The same with the keys per entry chosen: 64 (SPINF_KTILE, what the two calls above build) or 32, where an entry is a single
 * 32-key sub-tile (bits 2w and 8+2w only).  The attention kernel takes 32-key plans for head dim 512, 64-key plans otherwise. */
int spinf_tileplan_build_ktile(const int32_t* art, const int32_t* end, const int32_t* pos, const int32_t* grp, int32_t grp_mode,
                               int64_t n, int32_t window, int32_t ktile, spinf_tileplan** out);
/* counts[0] query tiles, [1] entries, [2] active 32x32 blocks, [3] masked 32x32 blocks, [4] n */
int spinf_tileplan_counts(const spinf_tileplan* plan, int64_t counts[5]);
/* qt_ptr [n_qtiles+1], kv_idx [entries], kv_bits [entries], order [n_qtiles]: caller-allocated host arrays */
int spinf_tileplan_export(const spinf_tileplan* plan, int32_t* qt_ptr, int32_t* kv_idx, uint32_t* kv_bits, int32_t* order);
/* items [4 * n_qtiles * head_groups], list_ptr [9]: caller-allocated host arrays */
int spinf_tileplan_schedule(const spinf_tileplan* plan, int32_t head_groups, int32_t* items, int32_t* list_ptr);
/* The same items dealt out to n_lists workgroups ahead of the launch (a simulation of "the workgroup that is free first takes the
 * next item of its XCD's list" under a cost model): items [4 * n_qtiles * head_groups] regrouped list by list, list_ptr [n_lists + 1].
 * For spinf_attn_args.n_lists > 0; n_lists = the number of workgroups to launch, normally the GPU's compute units.  Host arrays. */
int spinf_tileplan_schedule_static(const spinf_tileplan* plan, int32_t head_groups, int32_t n_lists, int32_t* items, int32_t* list_ptr);
/* Compact rows (tree_attention with sidx, spinf_serve/models/qwen35/qwen.py:613-622): row_of [n] = row of each stream
 * position in tensors that hold the real tokens only, -1 for a pad position.  kv_row0 [entries] (caller-allocated) receives,
 * per plan entry, the row of the entry's first key if its 64 keys are 64 consecutive rows, else -1.  Host arrays. */
int spinf_tileplan_row0(const spinf_tileplan* plan, const int32_t* row_of, int32_t* kv_row0);
void spinf_tileplan_free(spinf_tileplan* plan);

/* ------------------------------------------------------------------------------------------------ attention
 * Replaces the compiled flex_attention call of tree_flex_forward (spinf_serve/models/gemma4.py:107-118) and of
 * tree_attention (spinf_serve/models/qwen35/qwen.py:614,620): out = softmax(scale * Q K^T under the tree mask) V with
 * GQA (query head h reads key/value head h / (hq / hkv)).  bf16 in, fp32 softmax and accumulation, bf16 out.
 *
 *   q [n, hq, d], k / v [n, hkv, d], out [n, hq, d]: bf16 device tensors, d contiguous; *_tok / *_head are the token
 *   and head strides in elements (multiples of 8).  d is 64, 128, 256 or 512 (512: one head per item, and a plan of 32-key entries).
 *   art, end, pos, kv_idx, kv_bits: device copies of the metadata and of the exported plan; items, list_ptr: device copy of
 *   the schedule for hq / spinf_attn_heads_per_item(hq, hkv, d, variant) head groups, n_items = query tiles x head groups
 *   window: the window the plan was built with (<= 0 global)
 *   row_of, kv_row0 (both NULL, or both device arrays as spinf_tileplan_row0 describes them): compact rows.  q, k, v, out
 *   then hold the real tokens only; the kernel reads and writes them through row_of instead of the three zero-filled
 *   scatters and the gather of qwen.py:617-622.  Pad positions write nothing.  Results equal the scattered call's bit for bit.
 *   grp, grp_mode: the image groups the plan was built with (spinf_tileplan_build_groups); stream layout, variant 0 / 1.
 *
 * The kernel is persistent (one workgroup per CU pulling items from the lists).  Its list cursors live in a block that the
 * library keeps per stream (allocated with hipMalloc at a stream's first call, or when a bigger schedule comes; never freed):
 * calls on one stream follow each other, calls on different streams may overlap, from any host thread.  Under stream capture
 * the stream's block is recorded into the graph and stays with it (nothing can be allocated then: the stream must have made
 * one call of that size before); callers that record graphs or must not allocate take spinf_tree_attn_fwd_noalloc.
 * Image groups: grp_mode 1 goes with every layer, grp_mode 2 with sliding layers only (window > 0; a global layer of that
 * checkpoint passes grp = NULL, anything else is rejected).
 */
typedef struct spinf_attn_args {
    const void* q; const void* k; const void* v; void* out;
    int64_t q_tok, q_head, k_tok, k_head, v_tok, v_head, o_tok, o_head;
    int64_t n; int32_t hq, hkv, d; float scale; int32_t window;
    const int32_t* art; const int32_t* end; const int32_t* pos;
    const int32_t* kv_idx; const uint32_t* kv_bits; const int32_t* items; const int32_t* list_ptr;
    int64_t n_items;
    int32_t variant;   /* 0 = default kernel choice (eight waves, two heads of a GQA group per work item, where the group is even);
                          1 = one head per work item, four waves; 2 = four waves with two heads each (head dim <= 128,
                          no compact rows); 3 = the kernel with decoupled waves at head dim 128 (items as for 0; needs an even
                          group, a static schedule (n_lists > 0) over 64-key entries, the stream layout, no image groups) */
    const int32_t* row_of; const int32_t* kv_row0;
    const int32_t* grp; int32_t grp_mode;   /* image groups, as given to spinf_tileplan_build_groups (device copy of grp), or NULL */
    int32_t ktile;                          /* keys per plan entry: 0 or 64; 32 with d = 512, and with a static schedule */
    int32_t n_lists;                        /* 0: items / list_ptr are the eight work lists of spinf_tileplan_schedule, shared by all
                                               workgroups.  > 0: a static schedule (spinf_tileplan_schedule_static) of n_lists item lists,
                                               list_ptr [n_lists + 1]; the pass runs as n_lists workgroups, each through its own list.  With
                                               ktile 32 (and d = 512, or d = 256 with an even number of query heads per key / value head and
                                               variant 0; stream layout, no groups) that is the kernel with decoupled waves, which at
                                               d = 512 computes the pass in one launch instead of two */
    int32_t debug_expire;                   /* 0 in production.  Test hook of the kernel with decoupled waves (no counterpart in the reference):
                                               k > 0 = polls of one wait before a wave gives up (2^18 otherwise; a healthy wait takes a handful).
                                               With k = 1 every wave that has to wait at all gives up, which takes its workgroup through the
                                               landing a real time-out would take (every wave leaves the ring and the workgroup computes its list
                                               again, one tile at a time between barriers).  Same results bit for bit; spinf_attn_ring_aborts counts it */
} spinf_attn_args;

/* query heads one work item covers for this geometry (1 or 2); 0 for an invalid geometry */
int spinf_attn_heads_per_item(int32_t hq, int32_t hkv, int32_t d, int32_t variant);
int spinf_tree_attn_fwd(const spinf_attn_args* args, void* stream);
/* The same pass with nothing allocated.  No counterpart in the reference: it is for callers that cannot call hipMalloc (code
 * under HIP graph capture, tight serving loops, harnesses that forbid allocation).  spinf_tree_attn_fwd keeps its list cursors,
 * counts and redo list in a buffer that the library allocates (and regrows) on the device; this entry point keeps them in a
 * file-scope device array of 64 + 65,536 ints (256.25 KiB per GPU, held until the process ends) and calls no hipMalloc /
 * hipFree nor any allocating routine.  Same arguments, same kernels, same results bit for bit.  Limit: n_items (query tiles x
 * head groups) <= 65,536, more is SPINF_E_ARG.  The cursors and counts are cleared by a small kernel in front of every pass that
 * uses them (the kernel with decoupled waves uses none: such a call is one launch), so a call does not depend on what the
 * previous one left.  Every call on a GPU shares that GPU's array: calls that overlap on
 * one GPU (different streams or threads) race; order them on one stream. */
int spinf_tree_attn_fwd_noalloc(const spinf_attn_args* args, void* stream);
/* Diagnostics (no counterpart in the reference): *total = work items that the exact (rescaling) pass has recomputed on the
 * current device since the library was loaded, i.e. query tiles whose scores ranged too widely for the fast pass.
 * Synchronises the device. */
int spinf_attn_exact_items(int64_t* total);
/* Diagnostics (no counterpart in the reference): *total = waves of the static-schedule kernel that gave up a bounded wait on
 * the current device since the library was loaded.  Always 0 unless the kernel has a bug (or debug_expire asked for it).  The
 * results of such a pass are still complete and the same bit for bit: such a workgroup computes its list again before it ends,
 * one tile at a time between barriers; the count says that time was lost.
 * Synchronises the device. */
int spinf_attn_ring_aborts(int64_t* total);

/* ------------------------------------------------------------------------------------------------ Gated DeltaNet
 * Replaces gdn.recurrent / gdn.chunked (spinf_serve/models/qwen35/gdn.py:197-235 and :109-133): the gated delta rule
 * over a set of segments; segment s covers call rows cu[s] .. cu[s+1]-1, call row r is stream row idx[r] (idx NULL:
 * row r itself); it starts from h0[h0_idx[s]] (h0 or h0_idx NULL, or index < 0: zero state) and, where ht_idx[s] >= 0,
 * leaves its final state in ht[ht_idx[s]].  States are fp32 [*, hv, dk, dv].
 *
 *   q, k [rows, h, dk] (l2-normalised), v, o [rows, hv, dv] bf16; g [rows, hv] fp32 log decay; beta [rows, hv] bf16;
 *   strides in elements (q and k share q_tok, g and beta share g_tok; heads are dense inside a row); dk = dv = 128.
 *   cu, idx, h0_idx, ht_idx: int64 device arrays.  mode 0 = the recurrent entry point (short
 *   segments; consecutive segments of at most 16 tokens that start from the same state and leave none behind are taken
 *   two to a chunk), 1 = the chunked entry point (one workgroup per segment and head, 32-token chunks); both are the WY
 *   form of the same recurrence and either mode accepts any segment length.
 *   v and o must be 16-byte aligned with row strides that are multiples of 8 elements.
 */
typedef struct spinf_gdn_args {
    const void* q; const void* k; const void* v; const float* g; const void* beta; void* o;
    int64_t q_tok, v_tok, g_tok, o_tok;
    int32_t h, hv, dk, dv; float scale;
    const int64_t* cu; const int64_t* idx; int64_t n_seg; int64_t max_len;
    const float* h0; const int64_t* h0_idx; float* ht; const int64_t* ht_idx;
    int32_t mode;
} spinf_gdn_args;

int spinf_gdn_fwd(const spinf_gdn_args* args, void* stream);

/* ------------------------------------------------------------------------------------------------ Gated DeltaNet plan
 * Replaces tree_plan (spinf_serve/models/qwen35/qwen.py:158-276): from the path predecessors of a packed stream, the segments
 * (maximal stream-consecutive runs one scan takes in one go: a segment begins where the predecessor is missing, is not the stream
 * token right before, or has several children, qwen.py:185-187), their levels, and per level the calls spinf_gdn_fwd runs.
 *
 *   prev [n] int64: the token before each token on its path, -1 none; real [n] uint8: not a pad.  Host arrays.
 *   path 0 ("indexed", qwen.py:220-241): a level's segments longer than short_len go to the chunked entry point, in calls of at most
 *   call_tokens tokens (a call holds at least one segment), the others to the recurrent entry point in one call; segments that are
 *   continued from (or that hold a token of `keep`) leave their state in a slot of their level.  path 1 ("levels"): per level the
 *   keeping segments first, then the others, below the roots in calls of at most max_init segments.
 *   rows >= 0: the tensors hold the real tokens first (compact rows, qwen.py:179-184,266-275): row indices are compact rows and
 *   `rows` stands for "no row"; rows < 0: rows are stream positions and n stands for "no row".
 * Export (host arrays, caller-allocated from spinf_gdn_plan_counts: [0] segments, [1] levels, [2] calls, [3] call segments in all,
 * [4] rows in all calls, [5] conv rows):
 *   level_ptr [levels + 1] -> calls; call_kind [calls] (1 chunked, 0 recurrent); call_keep [calls] (some segment leaves its state);
 *   call_seg_ptr / call_row_ptr [calls + 1] -> seg_len, h0_idx, ht_idx [call segments] (length; slot of the start state in the level
 *   above, -1 zero state; slot of the final state in this level, -1 not kept) and idx [rows] (the segments' rows back to back);
 *   n_keep [levels] slots per level; conv [conv rows, 4]: rows of the three path predecessors (oldest first) and of the token itself
 *   (qwen.py:260-265); seg_of_row [conv rows] (-1 pad); seg_level, seg_slot [segments]. */
typedef struct spinf_gdn_plan spinf_gdn_plan;
int spinf_gdn_plan_build(const int64_t* prev, const uint8_t* real, int64_t n, int32_t path, int32_t short_len, int64_t call_tokens,
                         int32_t max_init, int64_t rows, const int64_t* keep, int64_t n_keep, spinf_gdn_plan** out);
int spinf_gdn_plan_counts(const spinf_gdn_plan* plan, int64_t counts[6]);
int spinf_gdn_plan_export(const spinf_gdn_plan* plan, int64_t* level_ptr, int32_t* call_kind, int32_t* call_keep, int64_t* call_seg_ptr,
                          int64_t* call_row_ptr, int64_t* seg_len, int64_t* h0_idx, int64_t* ht_idx, int64_t* idx, int64_t* n_keep,
                          int64_t* conv, int64_t* seg_of_row, int64_t* seg_level, int64_t* seg_slot);
void spinf_gdn_plan_free(spinf_gdn_plan* plan);

/* ------------------------------------------------------------------------------------------------ Gated DeltaNet layer, around the scan
 * spinf_gdn_prologue replaces the element-wise work of GatedDeltaNet.forward before the scan
 * (spinf_serve/models/qwen35/qwen.py:657-668): the 4-tap convolution along each token's path (conv [T, 4]: rows of the
 * 3 path predecessors and of the token itself, a row index outside 0 .. T-1 = a zero row; weights conv_w [conv_dim, 4] fp32),
 * silu, the split into q / k / v, with `normalize` the l2 norm x / sqrt(sum x^2 + 1e-6) of q and k per head, beta = sigmoid(b)
 * and g = -exp(a_log) softplus(a + dt_bias).
 *   y [T, y_tok] bf16: the input projection's rows, columns q (h dk) | k (h dk) | v (hv dv) | z (hv dv) | b (hv) | a (hv)
 *   q, k [T, h, dk], v [T, hv, dv], beta [T, hv] bf16 and g [T, hv] fp32: dense outputs.  Values are rounded to bf16 where
 *   the reference rounds them (after the silu, after the norm).
 * spinf_gdn_gate replaces qwen.py:670-672 after the scan: out = bf16(norm_w * bf16(rms_norm(o))) * silu(z), rms_norm per
 * head over dv with eps; o [T, hv, dv] (row stride o_tok), z = the z columns of y (row stride z_tok), out [T, hv dv] dense.
 */
typedef struct spinf_gdn_pre_args {
    const void* y; int64_t y_tok;
    const int64_t* conv; const float* conv_w; const float* a_log; const float* dt_bias;
    void* q; void* k; void* v; float* g; void* beta;
    int64_t T; int32_t h, hv, dk, dv; int32_t normalize;
} spinf_gdn_pre_args;
int spinf_gdn_prologue(const spinf_gdn_pre_args* args, void* stream);

typedef struct spinf_gdn_gate_args {
    const void* o; int64_t o_tok; const void* z; int64_t z_tok; const void* norm_w; float eps;
    void* out; int64_t T; int32_t hv, dv;
} spinf_gdn_gate_args;
int spinf_gdn_gate(const spinf_gdn_gate_args* args, void* stream);

/* ------------------------------------------------------------------------------------------------ lm head read-out
 * Replaces the lines after the logits GEMM in Scorer._logprobs and the column selection of Scorer._forward
 * (spinf_serve/scorer.py:351-353 and :254): out[r, c] = log_softmax(softcap * tanh(logits[r] / softcap))[cols[c]], or the whole
 * row with cols == NULL (the extraction rows, scorer.py:260).  softcap 0 = none.
 *   logits [rows, ld >= vocab]: fp32 (dtype 0) or bf16 (dtype 1) device matrix, rows 16-byte aligned; cols [n_cols] int64
 *   device array of column indices in 0 .. vocab-1 (any other is not read and gives NaN); out [rows, out_ld] fp32.
 */
typedef struct spinf_lm_args {
    const void* logits; int64_t ld; int32_t dtype;
    int64_t rows, vocab; float softcap;
    const int64_t* cols; int64_t n_cols;
    float* out; int64_t out_ld;
} spinf_lm_args;
int spinf_lm_logprobs(const spinf_lm_args* args, void* stream);

/* The whole read-out in one pass: replaces the row gather Hf[sel], the chunked logits GEMM, the soft-capping, the log-softmax and
 * the column selection of Scorer._forward / Scorer._logprobs (spinf_serve/scorer.py:247-261 and :340-355).  The logits matrix is
 * never stored: out[r, c] = log_softmax(cap(h[sel[r]] . W^T))[cols[c]], or the whole row with cols == NULL (scorer.py:260).
 *   h [h_rows, h_ld >= hidden] bf16: the final hidden states (after the final norm); sel [rows] int64 device: their rows to read,
 *   each in -h_rows .. h_rows-1 (a negative entry counts from the end, as the reference's tensor indexing Hf[sel] does; any other
 *   entry reads nothing outside h and gives a row of NaN), NULL = rows 0 .. rows-1 (rows <= h_rows); w [vocab, w_ld >= hidden] bf16: the lm head's weight (nn.Linear layout); hidden a multiple of 64;
 *   rows of h and w 16-byte aligned.
 *   logits_dtype 0: the logits stay fp32 (the reference's "f32out" and "fp32" modes, scorer.py:345-348); 1: they are rounded to
 *   bf16 and soft-capped in bf16 steps, as `h @ W.t()` on bf16 tensors gives them (scorer.py:349-352).
 *   cols [n_cols] int64 device: columns in 0 .. vocab-1 (any other gives NaN); out [rows, out_ld] fp32.
 *   workspace: device memory of the size spinf_lm_head_workspace reports (the per-tile log-sum-exp partials), owned by the caller.
 * A row's results do not depend on which rows it is computed with (the reference pads chunks to lm_rows for that,
 * spinf_serve/config.py:56-57).  Stream-ordered; nothing is allocated.
 */
typedef struct spinf_lm_head_args {
    const void* h; int64_t h_ld;
    const int64_t* sel; int64_t rows;
    const void* w; int64_t w_ld;
    int64_t vocab, hidden;
    float softcap; int32_t logits_dtype;
    const int64_t* cols; int64_t n_cols;
    float* out; int64_t out_ld;
    void* workspace; int64_t workspace_bytes;
    int64_t h_rows;                          /* rows of h (> 0): what sel is checked against */
} spinf_lm_head_args;
int spinf_lm_head_workspace(const spinf_lm_head_args* args, int64_t* bytes);
int spinf_lm_head_fwd(const spinf_lm_head_args* args, void* stream);

/* ------------------------------------------------------------------------------------------------ extraction-decode attention
 * Replaces _x_attention of spinf_serve/decode.py:71-104 (the attention interface "x_decode"): one decoding step for the
 * Q = slots x beams queries of each of G groups.  A query attends to its group's prefix, to its own slot's template and to the
 * tokens its own beam generated; the three key ranges stay in the decoder's three caches (decode.py:129-155):
 *   q [G, H, Q, d] bf16 with element strides q_g, q_h, q_q (head dim contiguous); out [G, Q, H, d] bf16 contiguous;
 *   kp, vp [G, h, Lp, d], pos_p [G, Lp] (position, -1 = padding: decode.py:136,146,152);
 *   kt, vt [G, h, Tt, d], pos_t [G, Tt], own_t [G, Tt] (slot that owns the template token, -1 = padding; the reference's mask_t
 *   is own_t == q / beam, decode.py:161-162);
 *   gk, gv [G, h, Q, S, d]: entry s of query q is visible to q alone, for s <= *step (device scalar, decode.py:92; step >= 0);
 *   qpos [G, Q] int64 device (decode.py:170), read on sliding layers only: window > 0 hides prefix / template keys with
 *   qpos - pos >= window (decode.py:88-89); window 0 = global layer.  softcap 0 = none (decode.py:86-87).
 *   len_p, len_t [G] int32 device, each may be NULL: a group's prefix holds keys (pos_p >= 0) only in its first len_p[g] entries,
 *   its template range (own_t >= 0) only in its first len_t[g]; the entries behind are padding and are not read.  NULL = Lp / Tt.
 * All caches contiguous, 16-byte aligned, d in {64, 128, 256, 512}, H a multiple of h.  The key stream of a (group, kv head) can be
 * split over nsplit workgroups; nsplit > 1 needs a workspace of the size spinf_xdecode_plan reports (partial results, fp32),
 * which the caller owns.  A split is tiles_per_split 32-key tiles of a (group, kv head, 128 rows) list, 0 = the longest list's
 * tiles (spinf_xdecode_tiles) / nsplit, rounded up; nsplit x tiles_per_split must cover the longest list.  Lists that fit one
 * split (short groups, once len_p / len_t are given) are computed by one workgroup and leave no partial results.
 * Calls are stream-ordered; nothing is allocated.
 */
typedef struct spinf_xdec_args {
    const void* q; int64_t q_g, q_h, q_q;
    const void* kp; const void* vp; const int32_t* pos_p;
    const void* kt; const void* vt; const int32_t* pos_t; const int32_t* own_t;
    const int32_t* len_p; const int32_t* len_t;
    const void* gk; const void* gv;
    const int64_t* qpos; const int64_t* step;
    void* out;
    void* workspace; int64_t workspace_bytes; int32_t nsplit;
    int32_t tiles_per_split;
    int32_t G, H, h, Q, S, Lp, Tt, d, beam, window;
    float scale, softcap;
} spinf_xdec_args;
/* suggested nsplit for these sizes (enough workgroups to fill the GPU) and the workspace it needs (0 for nsplit 1) */
int spinf_xdecode_plan(const spinf_xdec_args* args, int32_t* nsplit, int64_t* workspace_bytes);
/* tiles of the longest list of these sizes (a group whose prefix and template ranges are full) */
int spinf_xdecode_tiles(const spinf_xdec_args* args, int32_t* tiles);
int spinf_xdecode_attn_fwd(const spinf_xdec_args* args, void* stream);

/* ------------------------------------------------------------------------------------------------ yardstick
 * No counterpart in the reference: one launch of a pure v_mfma_f32_32x32x16_bf16 loop on every compute unit (one workgroup of eight
 * waves per CU, iters x 8 MFMAs per wave, operands in registers), for the benchmark's "what do the matrix cores sustain on this
 * part" figure, as a plain device copy is the yardstick for HBM.  out: device scratch of at least 512 floats per compute unit;
 * *flops receives the floating-point operations of the launch.  Timing is the caller's (events on the stream).
 */
int spinf_diag_mfma_rate(int64_t iters, float* out, int64_t out_floats, double* flops, void* stream);
/* Diagnostics (no counterpart in the reference): do a wave's LDS reads of different kinds (ds_read_b64_tr_b16, ds_read_b128) return
 * in issue order, as every s_waitcnt lgkmcnt(n) of the kernels above assumes?  `workgroups` workgroups of four waves each run
 * `iters` rounds of six interleavings of eight reads, waiting with the partial counts an in-order LDS allows, and compare with the
 * same reads done one at a time.  out: 7 device ints, zeroed by the caller: [0..5] += mismatches per interleaving, [6] += workgroups
 * that ran.  Any nonzero count in [0..5] means out-of-order returns. */
int spinf_diag_lds_order(int32_t iters, int32_t workgroups, int32_t* out, void* stream);
/* Diagnostics (no counterpart in the reference): the wait states around an MFMA issued from inline assembly, which the compiler's
 * hazard recogniser does not see.  out: 21 device ints, zeroed by the caller: [5 kind + g] += lanes with a wrong result for gap g
 * of (0, 1, 2, 4, 8) instructions; kind 0: v_mov writes the B registers, gap, MFMA; kind 1: MFMA, gap, v_mov overwrites B; kind 2:
 * v_exp_f32 -> v_cvt_pk_bf16_f32 writes B, gap, MFMA; kind 3: as 2 with, in place of the five gaps: one satisfied s_waitcnt
 * lgkmcnt(0), two of them, a satisfied s_waitcnt vmcnt(0), v_nop, s_waitcnt + s_nop 0; [20] += workgroups (of eight waves) that
 * ran.  out: 21 device ints. */
int spinf_diag_mfma_hazard(int32_t iters, int32_t workgroups, int32_t* out, void* stream);
/* Diagnostics (no counterpart in the reference): do a wave's vector instructions run in the shadow of its own MFMAs?  One workgroup
 * per compute unit, waves_per_simd (1, 2 or 4) waves on every SIMD, each wave iters rounds of { one v_mfma_f32_32x32x16_bf16 on one
 * accumulator, nv (0, 2, 4, 6, 8, 12 or 16) independent vector instructions: v_fma_f32 (kind 0) or v_exp_f32 (kind 1) } (kind 2:
 * rounds shaped like a 32 x 32 attention block at head dim 128: 8 chained MFMAs, 3 nv v_fma_f32 + nv v_exp_f32, 8 MFMAs on four
 * accumulators).  out:
 * 2 x 4 x waves_per_simd device int64: the clock before and after the loop of every wave of workgroup 0 (wave w = SIMD w % 4).
 * Clocks per round of a wave alone on its SIMD: 36 + 4 nv measured (36 + 8 nv for v_exp_f32), i.e. nothing runs in the shadow. */
int spinf_diag_mfma_valu(int32_t nv, int32_t kind, int32_t waves_per_simd, int32_t iters, int64_t* out, void* stream);
/* Diagnostics (no counterpart in the reference): the byte pattern of spinf_tree_attn_fwd's kernel with decoupled waves, with
 * nothing computed.  args as for a head-dim-256 call with a static schedule over 32-key entries (n_lists > 0, ktile 32, stream
 * layout, no image groups): per work item the query loads, every K / V tile through a four-slot LDS ring by the same DMA requests
 * (four in flight), and the output stores in the kernel's pattern; out comes back as 1.0 on the stream's rows.  status: 2 device
 * ints, zeroed by the caller: [0] += waves that gave up a bounded wait (never), [1] += tiles seen landed (the schedule's plan
 * entries x head groups).  parts: 3 = all of it, 1 = the K / V tiles only, 2 = the queries and outputs only (out is written
 * with 2 and 3), 5 / 7 = as 1 / 3 with each tile's requests dealt out over the eight waves instead of made by one; nslot (1 .. 4):
 * ring slots in use, i.e. tile requests in flight (the kernel has 4).  Its time is the floor that data movement alone sets for that
 * kernel on that schedule. */
int spinf_diag_attn_stream(const spinf_attn_args* args, int32_t parts, int32_t nslot, int32_t* status, void* stream);

/* For bindings in other languages (no counterpart in the reference): sizes[0..6] = sizeof of spinf_attn_args, spinf_gdn_args,
 * spinf_gdn_pre_args, spinf_gdn_gate_args, spinf_lm_args, spinf_lm_head_args, spinf_xdec_args as this library was built (n must be
 * 7): a binding compares them with its own mirrors of the structures before its first call. */
int spinf_struct_sizes(int64_t* sizes, int32_t n);

#ifdef __cplusplus
}
#endif
#endif
