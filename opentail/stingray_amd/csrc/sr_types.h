// Structures shared by the host packer and the kernels.
#pragma once
#include <stdint.h>

// How a row is dispatched; mirrors Sampler.Sample (Sampler.cs:17-39 of the reference engine).
enum SrPath : int32_t {
    SR_PATH_GREEDY = 0,      // Temperature <= 0, no history penalty      -> Greedy(masked logits)
    SR_PATH_GREEDY_PEN = 1,  // Temperature <= 0 with history penalties   -> GreedyWithHistoryPenalties
    SR_PATH_TOPK = 2,        // 0 < TopK < vocab and no logit bias        -> SampleTopK
    SR_PATH_FULL = 3,        // everything else                           -> full-vocabulary pipeline
    SR_PATH_TOPK_WIDE = 4    // SampleTopK beyond the selection kernel's limits -> device-wide sort of the row
};

struct SrRow {
    float temperature;
    float top_p;
    float min_p;
    float rep;
    float presence;
    float frequency;
    float p_min;
    int32_t top_k;
    int32_t sel;        // how many of the largest scanned logits the row needs (see the packer)
    int32_t path;       // SrPath
    int32_t edit_off;   // first SrEdit of this row
    int32_t edit_cnt;
    int32_t mask_row;   // row index into the allow-mask array, or -1
    int32_t n_prev;
    uint32_t flags;     // SR_ROW_* from the public header
    int32_t scan_row;   // row index into the scan-mask array (row edges, allow-mask, history ids)
};

// One distinct in-range token id that the row's history or logit bias touches; sorted by id per row where a kernel
// searches them (SR_ROWFLAG_EDITS_SORTED), else in order of first appearance in the history.
struct SrEdit {
    int32_t id;
    float bias;         // LogitBias value (applied first); valid when has_bias
    int32_t occ_win;    // occurrences inside the trailing repetition window
    int32_t occ_all;    // occurrences in the whole history
    float pen;          // powf(repetition_penalty, occ_win), computed with the host libm (1 when unused)
    uint32_t has_bias;
};

// One row of the scan-mask array of the selection kernel: which batch row it is built for, and from what.
struct SrScanDesc {
    int32_t row;
    uint32_t flags;
};
// What sr_batch_append_tokens sends to the device: an edit to be written at a position of the edit array, and a
// keep-bit of a scan-mask row to be cleared (the id entered the row's history).
struct SrEditPatch {
    int32_t index;
    SrEdit edit;
};
// one piece of an upload: bytes that lie in pinned host memory and belong at a device address
struct SrCopySeg {
    const void* src;
    void* dst;
    unsigned long long bytes;
};
struct SrRowPatch {
    int32_t row;
    int32_t n_prev;
    int32_t edit_cnt;
    int32_t mask_row;  // the row's allow-mask from now on (-1 none); rows of batches without registered masks keep theirs
    int32_t sel;
    int32_t edit_off;  // where the row's edits lie from now on (a row that ran out of room moves to the array's end)
};
struct SrMaskClear {
    int32_t scan_row;
    int32_t row;
    int32_t id;
};
#define SR_SCAN_ALLOW 1u  // start from the row's allow-mask
#define SR_SCAN_HIST 2u   // clear the row's history ids

// Limits of the top-k selection kernel.
#define SR_TK_THREADS 512
#define SR_TK_VEC 19                       // 16-byte vectors of fp32 logits held per thread
#define SR_TK_VEC_BF16 10                  // ... of bf16 logits: the same 40 thousand elements per workgroup
#define SR_ARGMAX_STATIC_ROWS 16384        // rows the argmax entry point that allocates nothing takes per call
#define SR_TK_WINDOW 5                     // ... of which a thread has in flight or in registers at a time
#define SR_TK_WINDOW_OWN 10                // ... when every worker streams one row of its own
#define SR_TK_WINDOW_KEPT 5                // ... and has a compute unit to itself (the whole chunk in flight, 19, was the setting while
                                           // every chunk ended with a bound loop for the loads to hide; without those loops it costs
                                           // 1.3 us a launch at 256 rows: what is in flight beyond the window only queues)
#define SR_TK_MASK_WORDS 3                 // 32-bit keep-words per chunk thread: 19 x 4 and 10 x 8 bits both fit 96
#define SR_TK_GROUPS 4                     // group maxima per thread
#define SR_TK_SHORT_SEL 64                 // a launch whose rows all ask for at most this many entries: see k_topk_rows
#define SR_TK_SEL_MAX 2048                 // most entries (candidates + history ids) the row tail sorts
#define SR_TK_ROW_CAP 8192                 // candidates all chunks of a row may hand to its tail (16 per thread)
#define SR_TK_MAX_CHUNKS 128               // most workgroups one row is split over

// Full-vocabulary path: nucleus candidates up to this count are sorted inside the row kernel.
#define SR_FULL_SMALL_CAP 4096
#define SR_SEG_TERMS 1024                  // terms per segment of a sum that the whole device prepares (64 lanes x 16)
#define SR_SEG_MIN_VOCAB 4096              // shorter rows are not worth the preparation
#define SR_SEG_MAX 1024                    // most segments of such a row: longer rows are added the plain way
