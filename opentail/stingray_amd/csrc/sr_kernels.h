// Kernel argument blocks and host-callable launchers (one per .hip file).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "sr_types.h"

// out_flags bits written by the kernels; identical to SR_OUT_* of the public header
#define SR_KFLAG_GREEDY (1u << 0)
#define SR_KFLAG_TOPK (1u << 1)
#define SR_KFLAG_FULL (1u << 2)
#define SR_KFLAG_DEGENERATE (1u << 3)
#define SR_KFLAG_AMBIGUOUS (1u << 4)
#define SR_KFLAG_UNSUPPORTED (1u << 31)
// the public bits of SrRow.flags as device code sees them (the public header is not included on the device side)
#define SR_ROWBIT_HAS_LOGIT_BIAS (1u << 0)
#define SR_ROWBIT_DRAFT_FROM_LOOKUP (1u << 1)
// internal bit of SrRow.flags: the row has a history and at least one active penalty
#define SR_ROWFLAG_HAS_PENALTY (1u << 8)
// internal bit: the penalties can only lower a logit, so the scan skips the history ids (scan mask) and
// the row tail fetches their logits by id instead of over-selecting by the history length
#define SR_ROWFLAG_HIST_EXCL (1u << 9)
// the row's edits are sorted by id (else they stand in order of first appearance in the history)
#define SR_ROWFLAG_EDITS_SORTED (1u << 10)

// A sampled full-vocabulary row that keeps no adjusted copy of its logits although bias or penalties touch some ids
// (host and device agree on this: the host provides the rows' tables when a batch holds such a row).
#define SR_FULL_EDIT_VALUES 2048
static inline __host__ __device__ bool sr_row_edits_on_the_fly(const SrRow& rd, int)
{
    return rd.temperature > 0.0f && rd.edit_cnt > 0 && rd.edit_cnt <= SR_FULL_EDIT_VALUES;
}

#define SR_TK_MAX_XCD 16
struct SrTopkArgs {
    const void* logits;
    int64_t row_stride;      // elements
    int32_t vocab;
    int32_t dtype;           // 0 = f32, 1 = bf16
    int32_t chunks;          // chunk items per row
    int32_t n_rows;          // rows in this launch
    int32_t chunk_vecs;      // 16-byte vectors per chunk, a multiple of 64
    // Workgroup b runs the program progs[b] = (first item, number of items, launch slot of the row it finishes at
    // the end or -1, 1 when its items are exactly that row's chunks): it streams items[first .. first + n) in order.  An item is x = bits 24..30 chunk |
    // bits 0..23 launch slot of the row, y = batch row, z = scan-mask row, w = sel.
    const int4* items;
    const int4* progs;
    int32_t n_workers, n_items;
    int32_t cu_count;        // compute units of the device
    int32_t own_rows;        // every worker's program is one whole row (all its chunks, then its tail)
    int32_t kept;            // ... and there is at most one worker per compute unit
    int32_t short_lists;     // no row of the launch asks for more than SR_TK_SHORT_SEL entries
    const int32_t* sel_list; // [n_rows] batch row of every launch slot
    const SrRow* rows;
    const SrEdit* edits;
    const uint32_t* mask;
    int64_t mask_stride;     // words
    const uint32_t* scan_mask; // keep-bits of every row in the kernel's access order (SrRow.scan_row)
    int64_t scan_stride;     // 32-bit words per scan row: chunks x threads x SR_TK_MASK_WORDS
    float4* gmax;            // [n_rows][chunks][SR_TK_THREADS]: the four group maxima of every thread of every chunk
    float4* gmax2;           // ... the second largest element of each of those groups
    uint32_t* gpos;          // ... the position of the largest inside its group, 8 bits per group
    uint32_t* gbound;        // [n_rows][chunks][waves][2]: every chunk wave's share of the row's bound and its largest kept
                             // element (ordered keys)
    unsigned long long* cand; // [n_rows][SR_TK_ROW_CAP] (value bits << 32 | index), built by the row's tail
    // Counters, two sets of done_cap entries: a launch counts the chunks of slot s in row_done[parity * done_cap + s]
    // and clears the other set for the launch after it, so that whatever a launch leaves behind never reaches a
    // later one.
    uint32_t* row_done;
    uint32_t done_cap;
    uint32_t parity;
    uint32_t spin_limit;     // polls of a row's counter before its tail stops waiting and selects from the logits alone
    const double* uniforms;
    int32_t uniforms_per_row;
    int32_t* out_tokens;
    uint32_t* out_flags;     // may be null
    unsigned long long* prof; // phase timestamps [chunk items + rows][16] in profiling builds, else unused
};
hipError_t sr_launch_topk(const SrTopkArgs& a, int n_rows, hipStream_t stream);
// Builds scan row i for descs[i]; base_addr / stride_bytes are those of the logits the mask is used with
// (they decide where a row starts inside its first 16-byte vector), epv = 4 (fp32) or 8 (bf16).
// all pieces of an upload in one launch: segs (itself in pinned host memory) lists n pieces
hipError_t sr_launch_scatter(const SrCopySeg* segs, int n, hipStream_t stream);
// scan_ids: the n_scan scan rows to build (NULL: rows 0 .. n_scan - 1)
hipError_t sr_launch_pack_allow_mask(const void* logits, int dtype, int rows, int vocab, int64_t row_stride, uint32_t* out,
                                     int64_t out_stride, hipStream_t stream);
// AND of the n (<= SR_MASK_AND_MAX) registered masks ids_host[] into slot dst of the pool; *any (zero before) becomes 1
// when a bit inside the vocabulary is left
#define SR_MASK_AND_MAX 8
hipError_t sr_launch_mask_and(uint32_t* pool, int64_t pool_words, const int32_t* ids_host, int n, int dst, int vocab, uint32_t* any,
                              hipStream_t stream);
hipError_t sr_launch_build_scan_mask(const SrScanDesc* descs, const int32_t* scan_ids, int n_scan, const SrRow* rows, const SrEdit* edits,
                                     const uint32_t* mask, int64_t mask_stride, uint32_t* scan_mask, int64_t scan_stride,
                                     int vocab, int epv, int chunks, int chunk_vecs, unsigned long long base_addr,
                                     long long stride_bytes, hipStream_t stream);

// What one appended token per row changes (sr_batch_append_tokens): history length and edit count of n_rowp rows,
// n_edits whole edits, n_clears keep-bits of scan masks built with the given geometry, n_uni uniforms.  The lists
// may lie in pinned host memory.
hipError_t sr_launch_apply_patches(SrRow* rows, const SrRowPatch* rp, int n_rowp, SrEdit* edits, const SrEditPatch* ep,
                                   int n_edits, const SrMaskClear* mc, int n_clears, uint32_t* scan_mask,
                                   int64_t scan_stride, int epv, int chunk_vecs, unsigned long long base_addr,
                                   long long stride_bytes, double* uni_dst, const double* uni_src, int n_uni,
                                   hipStream_t stream);

struct SrArgmaxArgs {
    const void* logits;
    int64_t row_stride;
    int32_t vocab;
    int32_t dtype;
    int32_t rows;
    int32_t chunks;           // workgroups per row
    int32_t chunk_len;        // elements per chunk, a multiple of the elements of a 16-byte vector
    int32_t vec;              // rows start on 16-byte boundaries: 16-byte loads
    // rows of more than one chunk: [rows] packed (key << 32 | ~idx) and [rows] chunks counted in; both zero before
    // the launch and zero again after it
    unsigned long long* best;
    uint32_t* done;
    int32_t* out_idx;
    float* out_val;           // may be null
};
// fills chunks, chunk_len and vec from the other fields
void sr_argmax_plan(SrArgmaxArgs& a, int cu_count);
// clear_first: best and done may hold anything (a fill precedes the kernel)
hipError_t sr_launch_argmax_rows(const SrArgmaxArgs& a, bool clear_first, hipStream_t stream);
// the current device's copy of the scratch that belongs to the library's code object: SR_ARGMAX_STATIC_ROWS rows
hipError_t sr_argmax_static_scratch(int device, unsigned long long** best, uint32_t** done);

hipError_t sr_launch_selftest_expf(const float* x, float* y, int64_t n, hipStream_t stream);

// ---- full-vocabulary path (sr_full.hip) ---------------------------------------------------------------
struct SrFullState {
    // launch number << 32 | ordered key of the row's largest adjusted logit (0xffffffff = the row holds a NaN; 0 = none
    // yet), raised with 64-bit atomic maxima: what an earlier launch left is below anything of the present one, so the
    // word needs no clearing between launches
    unsigned long long maxkey;
    uint32_t flags;
    int32_t n_survivors;  // entries with probability > 0 when top-p starts
    float mul1, mul2;     // the row's entries are to be multiplied by these two, in this order (1 unless lazy_scale)
    uint32_t late;        // the number of the last launch in which a workgroup of the row stopped waiting at the meeting point
    int32_t pad;
};
static_assert(sizeof(SrFullState) == 32, "the 8-byte word, aligned, in front");
// SrFullArgs::row_sync, a word per row (rows 256 bytes apart: every workgroup of a row adds to its word and polls it):
// launch number << 32 | workgroups of k_full_softmax_seg behind the row's meeting point << 16 | workgroups counted in.
// The number is put in by an atomic maximum before the first count of a launch, so nothing clears the words.
#define SR_ROW_SYNC_STRIDE 32

struct SeqSegFunc;
struct SrFullArgs {
    const void* logits;
    int64_t row_stride;
    int32_t vocab;
    int32_t dtype;
    const int32_t* row_list;   // rows handled (device)
    const SrRow* rows;
    const SrEdit* edits;
    const uint32_t* mask;
    int64_t mask_stride;
    float* work;               // fp32 rows: [slot] or, with work_by_row, [row]
    int64_t work_stride;
    int32_t work_by_row;
    int32_t mode;              // 0 = sample, 1 = distribution only, 2 = distribution and sample
    int32_t lazy_scale;        // mode 1 only: rows that no filter touches keep expf(x - max); their two normalising
                               // factors go to state[slot].mul1 / mul2 for the reader to apply
    uint32_t* edit_tab;        // [slot][edit_tab_stride]: per row a bitmap of the ids its edits touch and one float per
    int64_t edit_tab_stride;   // edit (the adjusted value), for sampled rows that keep no adjusted copy; or null
    int32_t any_copy;          // some row keeps an adjusted copy of its logits (greedy rows, rows the table does not take)
    SrFullState* state;        // [slot]
    uint32_t* sort_keys_in;    // [slot][sort_stride]
    int32_t* sort_vals_in;
    int64_t sort_stride;       // entries per row segment in the sort buffers
    int32_t* wide_ids;         // [slot][sort_stride]: wide top-k rows, the token id of every place of the first order
    const double* uniforms;
    int32_t uniforms_per_row;
    int32_t* out_tokens;       // [row], may be null in mode 1
    uint32_t* out_flags;       // [row], may be null
    unsigned long long* prof;  // optional phase timestamps of slot 0 [32] (test hook), normally null
    // The softmax denominators prepared by the whole device (k_full_softmax_seg, seg_walk); seg_func is
    // null when the launch is not laid out for it (short or unaligned rows) and the rows are added by their workgroups.
    SeqSegFunc* seg_func;          // [slot][seg_stride]
    float2* seg_ms;                // [slot][seg_stride], 8 bytes each: a segment's maximum m (as an ordered key) and the
                                   // sum of exp(x - m) over it, approximately
    int32_t seg_stride;
    unsigned long long* watch;     // [slot][SR_FULL_SMALL_CAP]: the entries that can survive a row's min-p cut (value << 32 | ~index)
    uint32_t* watch_cnt;           // [slot]
    uint16_t* seg_keys;            // [slot][seg_key_stride]: the upper 16 bits of every e of a row that only top-p cuts (0: e = 0)
    int64_t seg_key_stride;
    uint32_t seq;                  // the launch's number (never 0): see SrFullState::maxkey
    int32_t n_sampled;             // rows of the launch with a temperature above 0 (greedy rows leave the passes at once)
    int32_t any_edits;             // some row of the launch has edits for k_full_edits (else it is not launched)
    int32_t edits_in_pass;         // seg_func is set: sampled rows with up to SR_FULL_EDIT_VALUES edits keep no adjusted copy and
                                   // need no table either (k_full_softmax_seg applies their edits where it loads the row)
    unsigned long long* row_sync;  // [slot * SR_ROW_SYNC_STRIDE]
    uint32_t row_wait_limit;       // polls of a row's count before a workgroup of k_full_softmax_seg stops waiting for it
    int32_t big_slabs;             // k_full_row gets 64 KB of shared memory more: slabs of 8,192 entries for rows that only top-p cuts
};
hipError_t sr_launch_full_prep(const SrFullArgs& a, int n_rows, hipStream_t st);
hipError_t sr_launch_full_row(const SrFullArgs& a, int n_rows, hipStream_t st);
// SampleTopK by sorts of the whole row (rows beyond the selection kernel's limits): keys of the whole row, the row's
// sort by its own workgroup (first != 0) or that of its adjusted first `sel` entries, the adjustment, the walk over
// the sorted result
hipError_t sr_launch_wide_keys(const SrFullArgs& a, int n_rows, hipStream_t st);
hipError_t sr_launch_wide_adjust(const SrFullArgs& a, int n_rows, hipStream_t st);
hipError_t sr_launch_wide_sort(const SrFullArgs& a, int n_rows, int first, hipStream_t st);
hipError_t sr_launch_wide_tail(const SrFullArgs& a, int n_rows, hipStream_t st);
hipError_t sr_launch_draw_rows(const float* probs, int64_t stride, int n, int rows, const double* u, int* out,
                               hipStream_t st);
hipError_t sr_launch_residual_rows(const float* p, int64_t ps, const float* q, int64_t qs, int n, int rows,
                                   const double* u, int* out, hipStream_t st);

// One segment of SR_SEG_TERMS terms of a row whose exact sum the whole device prepares (k_seq_funcs, seg_walk in
// sr_full.hip): the increment function n -> n + a[n & 1] of its terms in the binade `eb` (sr_seqsum.h), and for a
// segment in which the running sum is expected to change binade once, inside the 16 terms of lane `cross`: the function
// of the terms in front of those 16 (a0, a1, eb), the 16 terms themselves, and the function of the terms behind them
// (b0, b1) in the binade eb2.  The row's first segment, whose start is known exactly, carries its exact end instead.
#define SR_SEG_PLAIN 0u
#define SR_SEG_EXACT 1u
#define SR_SEG_SPLIT 2u
#define SR_SEG_LATE 3u   // no record yet: left by a workgroup that stopped waiting, with the launch's number in a0
struct SeqSegFunc {  // 96 bytes
    uint32_t a0, a1;
    int32_t eb;
    uint32_t kind;   // SR_SEG_* | cross << 8
    uint32_t b0, b1;
    int32_t eb2;
    uint32_t end_bits;  // SR_SEG_EXACT: the running sum behind the segment when the sum in front of it is +0
    float x[16];
};
struct SrSpecArgs {
    const SrRow* rows;
    int32_t vocab;
    int32_t n_draft;
    const float* p_all;          // [rows][n_draft + 1][vocab] filtered target distributions, to be multiplied by ...
    const SrFullState* state;    // ... mul1 and mul2 of [rows][n_draft + 1]
    const float* target_logits;  // [rows][n_draft + 1][vocab]
    const float* draft_probs;    // [rows][n_draft][vocab]
    const int32_t* draft_tokens; // [rows][n_draft]
    const double* uniforms;
    int32_t uniforms_per_row;
    int32_t* out_accepted;       // [rows]
    int32_t* out_tokens;         // [rows][n_draft + 1]
    float* resid;                // [rows][resid_stride]: max(0, p - q) of the row's first rejected position
    int64_t resid_stride;
    int32_t* reject;             // [rows]: that position, or -1 (none, or a row that does not take the ratio test), or
                                 // n_draft (every draft accepted and a bonus token to draw: resid holds the scaled row)
    double* seg_part;            // [rows][seg_stride]: approximate sum of every SR_SEG_TERMS terms of the row of resid
    SeqSegFunc* seg_func;        // [rows][seg_stride]: the increment functions of those segments; null: not prepared
    int32_t seg_stride;
};
hipError_t sr_launch_spec_verify(const SrSpecArgs& a, int rows, hipStream_t st);
hipError_t sr_launch_expand_rows(const SrRow* src, SrRow* dst, int rows, int positions, hipStream_t st);
hipError_t sr_launch_mtp_verify(const float* logits, int64_t stride, int n, int rows, const int* draft, float p_min,
                                int* out_argmax, int* out_accept, float* out_prob, hipStream_t st);
hipError_t sr_launch_selftest_seqsum(const float* x, int n, float s0, float target, float* out_sum, int* out_idx,
                                     hipStream_t st);
hipError_t sr_launch_selftest_segsum(const float* x, int n, double skew, float target, double* part, SeqSegFunc* funcs,
                                     float* out_sum, int* out_idx, hipStream_t st);
