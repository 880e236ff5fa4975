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
#define SR_KFLAG_UNSUPPORTED (1u << 31)
// internal bit of SrRow.flags: the row has a history and at least one active penalty
#define SR_ROWFLAG_HAS_PENALTY (1u << 8)

struct SrTopkArgs {
    const void* logits;
    int64_t row_stride;      // elements
    int32_t vocab;
    int32_t dtype;           // 0 = f32, 1 = bf16
    int32_t chunks;          // workgroups per row
    int32_t chunk_len;       // elements per chunk
    const int32_t* row_list; // rows handled by this launch (device)
    const SrRow* rows;
    const SrEdit* edits;
    const uint32_t* mask;
    int64_t mask_stride;     // words
    float* cand_val;         // [n_rows][chunks][SR_TK_CAP]
    int32_t* cand_idx;
    int32_t* cand_cnt;       // [n_rows][chunks]
    uint32_t* row_done;      // [n_rows], zero on entry, left zero on exit
    const double* uniforms;
    int32_t uniforms_per_row;
    int32_t* out_tokens;
    uint32_t* out_flags;     // may be null
    unsigned long long* prof; // optional phase timestamps [grid][16] (test hook), normally null
};
hipError_t sr_launch_topk(const SrTopkArgs& a, int n_rows, hipStream_t stream);

struct SrArgmaxArgs {
    const void* logits;
    int64_t row_stride;
    int32_t vocab;
    int32_t dtype;
    int32_t rows;
    int32_t chunks;
    int32_t chunk_len;
    unsigned long long* best; // [rows] packed (key << 32 | ~idx), zeroed by the launcher
    int32_t* out_idx;
    float* out_val;           // may be null
};
hipError_t sr_launch_argmax_rows(const SrArgmaxArgs& a, hipStream_t stream);

hipError_t sr_launch_selftest_expf(const float* x, float* y, int64_t n, hipStream_t stream);
