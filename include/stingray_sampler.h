/*
 * stingray_sampler.h -- C ABI of the MI355X (gfx950) token-sampling library.
 *
 * Plain C, blittable arguments only (pointers, int32/int64, float/double), int status returns
 * (0 = success), opaque handles.  These are the entry points a managed [LibraryImport] binding
 * attaches to; each one names the managed interface of the reference it stands behind
 * (paths relative to the reference tree).
 *
 * Conventions
 *   - A context (sr_ctx) belongs to one engine.  Calls on one context must not overlap; they may
 *     come from different OS threads over time (call sr_bind_thread after moving threads), which
 *     is the contract of IThreadAffineBackend.BindToCurrentThread
 *     (src/OpenTail.Stingray.Engine/IThreadAffineBackend.cs:9-21).
 *   - "_launch" entry points take DEVICE pointers for tensors and results, enqueue on the context's
 *     stream and return without synchronising.  The other entry points take HOST result buffers,
 *     and return after the (small) result download, the only synchronisation, as the device-argmax
 *     wrappers do at src/OpenTail.Stingray.Cuda/CudaBackend.cs:4110-4123.
 *   - Row parameters, token histories, logit bias, allow-masks and uniforms are HOST arrays; the
 *     library packs and uploads them (sr_batch_upload).  Token ids are int32, uniforms are the
 *     doubles Random.NextDouble() returned, in the order the managed sampler would have drawn them.
 *   - Results equal the managed CPU sampler's on the same logits, parameters and uniforms: token
 *     ids bit for bit (ties to the lower index), probabilities within 1e-5 relative.
 */
#ifndef STINGRAY_SAMPLER_H
#define STINGRAY_SAMPLER_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(_WIN32)
#define SR_API __declspec(dllexport)
#else
#define SR_API __attribute__((visibility("default")))
#endif

typedef struct sr_ctx sr_ctx;
typedef struct sr_batch sr_batch;

/* status codes */
enum {
    SR_OK = 0,
    SR_ERR_INVALID_ARGUMENT = 1, /* ArgumentException (e.g. length mismatch, Sampler.cs:121-123, 590-592) */
    SR_ERR_NULL_ARGUMENT = 2,    /* ArgumentNullException (Sampler.cs:197, 589)                            */
    SR_ERR_HIP = 3,              /* a HIP runtime call failed; text in sr_last_error                       */
    SR_ERR_UNSUPPORTED = 4,      /* shape outside what the kernels handle; text in sr_last_error           */
    SR_ERR_OUT_OF_MEMORY = 5,
    SR_ERR_NO_DEVICE = 6
};

/* logits element type */
enum { SR_DTYPE_F32 = 0, SR_DTYPE_BF16 = 1 };

/* per-row flags in sr_row_params.flags */
enum {
    SR_ROW_HAS_LOGIT_BIAS = 1u << 0, /* LogitBias.Count > 0: selects the full-vocabulary path even when
                                        every id is out of range (Sampler.cs:27,38)                      */
    SR_ROW_DRAFT_FROM_LOOKUP = 1u << 1 /* sr_spec_verify_launch: the row's draft tokens came from prompt lookup
                                          (usedPld, SpeculativeDecoder.cs:488-501): there are no draft
                                          distributions, the accept rule is px >= spec_draft_p_min or the
                                          draft is the argmax, a rejection draws from p (:538-552), whatever
                                          spec_draft_p_min is; draft_probs_dev is not read for the row     */
};

/* bits reported per row in out_flags */
enum {
    SR_OUT_PATH_GREEDY = 1u << 0,      /* Temperature <= 0 (Sampler.cs:19-22)                   */
    SR_OUT_PATH_TOPK_FAST = 1u << 1,   /* SampleTopK (Sampler.cs:216-357)                       */
    SR_OUT_PATH_FULL_VOCAB = 1u << 2,  /* slow path (Sampler.cs:41-95)                          */
    SR_OUT_DEGENERATE = 1u << 3,       /* all -inf row: greedy / uniform fallback was taken     */
    SR_OUT_AMBIGUOUS = 1u << 4,        /* the token depends on a convention the managed runtime leaves open: a cut or the
                                          draw fell within a few ulp of a boundary of the running sum, or a top-p cut
                                          split a run of equal probabilities (Sampler.cs:533 unstable sort, :555 lane
                                          order of TensorPrimitives.Sum).  The token is still the one the documented
                                          conventions give; a caller that wants certainty re-runs the row on the CPU  */
    SR_OUT_ROW_UNSUPPORTED = 1u << 31  /* an internal limit of the selection kernel was met although sr_batch_upload
                                          routes every row by those limits: token is -1.  No input is known to set it;
                                          sr_sample_batch finishes such a row with sr_resample_rows_launch            */
};

/*
 * The scalar fields of SamplingParams the sampler reads
 * (src/OpenTail.Stingray.Engine/Sampler.cs:648-813).  Defaults: temperature 1, top_k 0 (off),
 * top_p 1 (active iff 0 < p < 1), min_p 0, repetition_penalty 1, repeat_last_n 64
 * (<= 0 = whole history), presence/frequency 0, spec_draft_p_min 1.
 */
typedef struct sr_row_params {
    float temperature;
    int32_t top_k;
    float top_p;
    float min_p;
    float repetition_penalty;
    int32_t repeat_last_n;
    float presence_penalty;
    float frequency_penalty;
    float spec_draft_p_min;
    uint32_t flags;
} sr_row_params;

/* ---- context ------------------------------------------------------------------------------- */

/* Creates a context on HIP device `device_ordinal` with its own stream and scratch.  Mirrors the
 * cached availability probe + backend construction of the reference's native backends
 * (src/OpenTail.Stingray.Cpu/BlasInterop.cs:39-71, src/OpenTail.Stingray.Cuda/CudaBackend.cs:493-494):
 * SR_ERR_NO_DEVICE means "fall back to the managed sampler". */
SR_API int sr_create(int device_ordinal, sr_ctx** out);
SR_API void sr_destroy(sr_ctx* ctx);
/* IThreadAffineBackend.BindToCurrentThread (IThreadAffineBackend.cs:9-21): makes the context's device
 * current on the calling thread. */
SR_API int sr_bind_thread(sr_ctx* ctx);
/* Kernels are enqueued on this stream (a hipStream_t).  Lets the forward pass that produced the logits and the
 * sampler share one stream, so no event is needed between them (the pattern of CudaBackend.cs:4119-4123).
 * NULL means what it means everywhere in HIP: the device's default stream -- a managed caller that passes a zero
 * handle is ordered behind work on the default stream, not silently beside it.  A new context runs on a stream of
 * its own, which is non-blocking (not ordered with the default stream); sr_use_own_stream goes back to it.
 * Either call first waits for what the context has in flight on the stream it leaves. */
SR_API int sr_set_stream(sr_ctx* ctx, void* hip_stream);
SR_API int sr_use_own_stream(sr_ctx* ctx);
SR_API int sr_synchronize(sr_ctx* ctx);
/* Text of the last failure on this context (never NULL). */
SR_API const char* sr_last_error(sr_ctx* ctx);
/* Library version, "major.minor.patch". */
SR_API const char* sr_version(void);

/* ---- per-step row inputs ------------------------------------------------------------------- */

/* A batch holds the packed, device-resident side inputs of one decode step: the rows' parameters,
 * token histories (as per-token occurrence counts), logit-bias entries, allow-masks and uniforms.
 * It is what ContinuousBatchingEngine's hot loop gathers per row before calling
 * Sampler.Greedy|Sample (src/OpenTail.Stingray.Engine/ContinuousBatchingEngine.cs:609-650). */
SR_API int sr_batch_create(sr_ctx* ctx, sr_batch** out);
SR_API void sr_batch_destroy(sr_batch* batch);

/*
 * Packs and uploads the side inputs of `rows` rows over a vocabulary of `vocab` tokens.
 *   params        [rows]
 *   hist_ids      PreviousTokens of all rows, concatenated in order, duplicates kept (the
 *                 repetition window is positional, Sampler.cs:272-279); may be NULL when
 *   hist_offsets  [rows+1] is NULL (no history anywhere).
 *   bias_ids / bias_vals / bias_offsets [rows+1]: LogitBias entries per row, or all NULL.
 *                 A row with a non-empty range gets SR_ROW_HAS_LOGIT_BIAS set.
 *   allow_mask    [rows x mask_stride_words] packed allow-bits, bit (i & 31) of word (i >> 5) set =
 *                 token i allowed; NULL = no row is constrained.  This is the packed form of
 *                 ITokenConstraint.Filter's masked row
 *                 (src/OpenTail.Stingray.Core/Grammar/ITokenConstraint.cs:31-42).
 *   mask_active   [rows] non-zero = row is constrained (ITokenConstraint.IsConstraining and Filter did
 *                 not return the input span); NULL = every row when allow_mask is given.
 *   uniforms      [rows x uniforms_per_row] NextDouble() values, consumed in order per row.
 * Every host array may be reused when the call returns.  The copies to the device run on the context's stream
 * and are not waited for (except for an allow-mask): launches that follow on the same stream see the batch
 * complete; sr_set_stream synchronises the stream it leaves.
 */
SR_API int sr_batch_upload(sr_batch* batch, int32_t rows, int32_t vocab,
                           const sr_row_params* params,
                           const int32_t* hist_ids, const int32_t* hist_offsets,
                           const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                           const uint32_t* allow_mask, int64_t mask_stride_words,
                           const uint8_t* mask_active,
                           const double* uniforms, int32_t uniforms_per_row);
/* One more token at the end of every row's history, as the engine appends the sampled token to the sequence's
 * RecentTokens after each step (src/OpenTail.Stingray.Engine/ContinuousBatchingEngine.cs:650, 1280): afterwards the
 * batch is what sr_batch_upload would build from the longer histories and the same other inputs, for the cost of
 * the few entries that change instead of a pass over every history.
 *   tokens    [rows] host array; a negative entry leaves its row's history as it is.
 *   uniforms  [rows x uniforms_per_row] for the next step, or NULL to keep those on the device.
 * A row that runs out of the room it was given for new ids (32 and more per row) moves to the end of the batch's edit
 * array, with twice the room.  Rows the in-place update does not cover (the first history token of a row with penalties,
 * a top-k beyond 2,048 entries, an edit array that is full) make the call rebuild the whole batch from the inputs it
 * kept: same result, the cost of an upload.  A call that fails after it has changed the host's copies leaves the batch
 * marked, and the next call rebuilds it.  Like sr_sample_launch, the call keeps host-side state and must not be
 * recorded into a HIP graph.  A batch uploaded with allow-masks of its own returns
 * SR_ERR_UNSUPPORTED (its masks change with every step: register them and use sr_batch_upload_mask_ids /
 * sr_batch_append_tokens_masks).  Copies run on the context's stream and are not waited for, as in sr_batch_upload. */
SR_API int sr_batch_append_tokens(sr_batch* batch, const int32_t* tokens, const double* uniforms);
/* Replaces only the uniforms of an uploaded batch (same rows and uniforms_per_row). */
SR_API int sr_batch_set_uniforms(sr_batch* batch, const double* uniforms);

/* ---- sampling ------------------------------------------------------------------------------- */

/*
 * int Sampler.Sample(ReadOnlySpan<float> logits, SamplingParams p, Random? rng) for every row of a
 * batch (Sampler.cs:17-102), preceded by the row's constraint mask
 * (ContinuousBatchingEngine.cs:635-643).  logits is a DEVICE tensor [rows x row_stride_elems] of
 * `dtype`; bf16 is upcast to fp32 exactly.  out_tokens / out_flags: DEVICE int32[rows] /
 * uint32[rows] (out_flags may be NULL).  One uniform per row is consumed by non-greedy rows.
 * This is the batched sibling of IBatchedForwardPass.BatchForwardMultiArgmax
 * (src/OpenTail.Stingray.Engine/IBatchedForwardPass.cs:105-117) for rows that are not greedy.
 * The call keeps host-side state per launch (which of two sets of hand-over counters the launch uses): it must not be
 * recorded into a HIP graph and replayed; sr_argmax_rows_launch_noalloc is the entry point made for that.
 */
SR_API int sr_sample_launch(sr_ctx* ctx, const sr_batch* batch, const void* logits_dev, int dtype,
                            int64_t row_stride_elems, int32_t* out_tokens_dev, uint32_t* out_flags_dev);

/*
 * SampleTopK (Sampler.cs:216-357) once more, by device-wide sorts of the whole row, for the SampleTopK rows of a batch
 * named in rows_host (HOST int32 row indices into the batch); the same logits, outputs and uniforms as the launch
 * before.  The finisher for rows flagged SR_OUT_ROW_UNSUPPORTED, and an independent second way to the same answer
 * for any SampleTopK row.  No counterpart in the reference, which has no row limit.
 */
SR_API int sr_resample_rows_launch(sr_ctx* ctx, const sr_batch* batch, const void* logits_dev, int dtype,
                                   int64_t row_stride_elems, const int32_t* rows_host, int32_t n_rows,
                                   int32_t* out_tokens_dev, uint32_t* out_flags_dev);

/* sr_sample_launch with the side inputs given directly and results in HOST buffers.  logits may be a device
 * (logits_on_device != 0) or a host tensor.  out_flags may be NULL. */
SR_API int sr_sample_batch(sr_ctx* ctx, const void* logits, int dtype, int logits_on_device,
                           int32_t rows, int32_t vocab, int64_t row_stride_elems,
                           const sr_row_params* params,
                           const int32_t* hist_ids, const int32_t* hist_offsets,
                           const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                           const uint32_t* allow_mask, int64_t mask_stride_words, const uint8_t* mask_active,
                           const double* uniforms,
                           int32_t* out_tokens, uint32_t* out_flags);

/*
 * int Sampler.Greedy(ReadOnlySpan<float>) per row (Sampler.cs:442-446): index of the maximum, lowest
 * index on ties, and its value; the device counterpart already in the reference is
 * llm_argmax_rows (src/OpenTail.Stingray.Cuda/CudaTextKernels.cs:465-479) behind
 * CudaBackend.ArgmaxRows.  Device inputs and outputs; out_val_dev may be NULL.
 */
SR_API int sr_argmax_rows_launch(sr_ctx* ctx, const void* logits_dev, int dtype, int32_t rows,
                                 int32_t vocab, int64_t row_stride_elems,
                                 int32_t* out_idx_dev, float* out_val_dev);
/*
 * sr_argmax_rows_launch for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, results
 * and errors; it calls no hipMalloc/hipFree: the per-row slots and counters that rows split over several
 * workgroups need lie in a fixed array inside the library's code object (192 KiB per GPU, held until the
 * process ends), whose part for this call a small fill kernel clears first.  At most SR_ARGMAX_NOALLOC_MAX_ROWS
 * rows per call (SR_ERR_INVALID_ARGUMENT beyond).  All contexts of one GPU share the array: two calls that
 * overlap on one GPU (different streams, different contexts) race; order them on one stream.
 */
#define SR_ARGMAX_NOALLOC_MAX_ROWS 16384
SR_API int sr_argmax_rows_launch_noalloc(sr_ctx* ctx, const void* logits_dev, int dtype, int32_t rows,
                                         int32_t vocab, int64_t row_stride_elems,
                                         int32_t* out_idx_dev, float* out_val_dev);
/* Host-result form: (int Token, float Logit)[] as BatchForwardMultiArgmax returns it. */
SR_API int sr_argmax_rows(sr_ctx* ctx, const void* logits, int dtype, int logits_on_device,
                          int32_t rows, int32_t vocab, int64_t row_stride_elems,
                          int32_t* out_idx, float* out_val);

/*
 * void Sampler.BuildFilteredDistribution(logits, p, Span<float> probs) per row (Sampler.cs:118-163).
 * out_probs_dev: DEVICE float [rows x probs_stride_elems].  probs_len is the caller's probs length:
 * SR_ERR_INVALID_ARGUMENT when it differs from the batch's vocab (the ArgumentException of
 * Sampler.cs:121-123).
 */
SR_API int sr_build_distribution_launch(sr_ctx* ctx, const sr_batch* batch, const void* logits_dev,
                                        int dtype, int64_t row_stride_elems,
                                        float* out_probs_dev, int64_t probs_stride_elems,
                                        int32_t probs_len);

/*
 * int Sampler.SampleWithDistribution(logits, p, Span<float> probs, Random? rng) per row
 * (Sampler.cs:172-187): the distribution as above plus the token drawn from it (greedy rows: one-hot
 * and no draw).
 */
SR_API int sr_sample_with_distribution_launch(sr_ctx* ctx, const sr_batch* batch, const void* logits_dev,
                                              int dtype, int64_t row_stride_elems,
                                              float* out_probs_dev, int64_t probs_stride_elems,
                                              int32_t probs_len, int32_t* out_tokens_dev);

/* Span-shaped forms of the two calls above: HOST fp32 logits in, HOST probabilities (and tokens) out, side inputs
 * as for sr_sample_batch (no allow-mask: the managed methods take none).  uniforms: HOST double[rows], one per row
 * (may be NULL for sr_build_distribution and when every row is greedy). */
SR_API int sr_build_distribution(sr_ctx* ctx, const float* logits, int32_t rows, int32_t vocab, int64_t row_stride_elems,
                                 const sr_row_params* params,
                                 const int32_t* hist_ids, const int32_t* hist_offsets,
                                 const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                                 float* out_probs, int64_t probs_stride_elems, int32_t probs_len);
SR_API int sr_sample_with_distribution(sr_ctx* ctx, const float* logits, int32_t rows, int32_t vocab,
                                       int64_t row_stride_elems, const sr_row_params* params,
                                       const int32_t* hist_ids, const int32_t* hist_offsets,
                                       const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                                       const double* uniforms,
                                       float* out_probs, int64_t probs_stride_elems, int32_t probs_len,
                                       int32_t* out_tokens);

/*
 * int Sampler.SampleFromProbs(ReadOnlySpan<float> probs, Random rng) per row (Sampler.cs:195-199):
 * first index whose running fp32 sum reaches (float)u, last index as the rounding fallback.
 * uniforms: HOST double[rows] (NULL -> SR_ERR_NULL_ARGUMENT, the ArgumentNullException of :197); they are copied
 * into pinned memory of the context, so the array may be reused at once and the call does not wait for the device.
 */
SR_API int sr_sample_from_probs_launch(sr_ctx* ctx, const float* probs_dev, int32_t rows, int32_t vocab,
                                       int64_t probs_stride_elems, const double* uniforms,
                                       int32_t* out_tokens_dev);

/* Span-shaped form: HOST probabilities in, HOST tokens out. */
SR_API int sr_sample_from_probs(sr_ctx* ctx, const float* probs, int32_t rows, int32_t vocab,
                                int64_t probs_stride_elems, const double* uniforms, int32_t* out_tokens);

/*
 * int Sampler.ResampleResidual(p, q, rng) per row (Sampler.cs:587-618).  p_len != q_len ->
 * SR_ERR_INVALID_ARGUMENT; uniforms NULL -> SR_ERR_NULL_ARGUMENT.
 */
SR_API int sr_resample_residual_launch(sr_ctx* ctx, const float* p_dev, int32_t p_len, int64_t p_stride_elems,
                                       const float* q_dev, int32_t q_len, int64_t q_stride_elems,
                                       int32_t rows, const double* uniforms, int32_t* out_tokens_dev);

/* Span-shaped form: HOST distributions in, HOST tokens out. */
SR_API int sr_resample_residual(sr_ctx* ctx, const float* p, int32_t p_len, int64_t p_stride_elems,
                                const float* q, int32_t q_len, int64_t q_stride_elems,
                                int32_t rows, const double* uniforms, int32_t* out_tokens);

/*
 * The accept / reject loop of SpeculativeDecoder.StepSampled
 * (src/OpenTail.Stingray.Engine/SpeculativeDecoder.cs:530-559) for every row of a batch.
 *   target_logits_dev [rows x (n_draft+1) x vocab]  position i verifies draft i; the last is the bonus
 *   draft_probs_dev   [rows x n_draft x vocab]       q_i, as SampleWithDistribution left them (:509-513)
 *   draft_tokens_dev  [rows x n_draft]
 * The batch supplies the rows' parameters and n_draft+1 uniforms per row (accept draws in position
 * order, then the residual / bonus draw).  spec_draft_p_min in (0,1), or SR_ROW_DRAFT_FROM_LOOKUP in the
 * row's flags, selects the looser accept of :546,552; draft_probs_dev may be NULL when every row does.
 * Outputs (DEVICE): out_accepted[rows]; out_tokens[rows x (n_draft+1)] = accepted drafts followed by the
 * correction or bonus token, the rest -1.  A draft id outside [0, vocab) ends its row at that
 * position with -1 in place of the correction token (the managed loop throws IndexOutOfRangeException at
 * pDist[x_i], :536); out_accepted counts the drafts accepted before it.
 * The call enqueues its kernels on the context's stream and returns without waiting for them.
 */
SR_API int sr_spec_verify_launch(sr_ctx* ctx, const sr_batch* batch, const float* target_logits_dev,
                                 const float* draft_probs_dev, const int32_t* draft_tokens_dev,
                                 int32_t n_draft, int32_t* out_accepted_dev, int32_t* out_tokens_dev);

/*
 * MtpDecoder.AcceptDraft + SoftmaxProbAt per row (src/OpenTail.Stingray.Engine/MtpDecoder.cs:562-596):
 * out_argmax = Greedy(row); accept iff draft == argmax, or, when p_min < 1, iff the draft's softmax
 * probability (double-precision sum, cast to float) >= p_min.  out_prob is 0 where no softmax was
 * needed.  All outputs DEVICE arrays [rows]; out_prob_dev may be NULL.
 */
SR_API int sr_mtp_verify_launch(sr_ctx* ctx, const float* logits_dev, int32_t rows, int32_t vocab,
                                int64_t row_stride_elems, const int32_t* draft_tokens_dev, float p_min,
                                int32_t* out_argmax_dev, int32_t* out_accept_dev, float* out_prob_dev);

/*
 * Host helper: packs the masked row an ITokenConstraint.Filter call returned into allow-bits
 * (bit set iff the entry is not negative infinity).  ceil(vocab / 32) words are written.
 */
SR_API int sr_pack_allow_mask(const float* masked_logits, int32_t vocab, uint32_t* out_words);
/* The same for `rows` masked rows that are already on the device (fp32 or bf16): out_words_dev is a DEVICE array
 * [rows x out_stride_words], out_stride_words >= ceil(vocab / 32).  Asynchronous on the context's stream. */
SR_API int sr_pack_allow_mask_launch(sr_ctx* ctx, const void* masked_logits_dev, int dtype, int32_t rows, int32_t vocab,
                                     int64_t row_stride_elems, uint32_t* out_words_dev, int64_t out_stride_words);

/*
 * Registered allow-masks.  A grammar constraint has few distinct masks -- one per automaton state
 * (JsonToolArgumentConstraint.ComputeMask, src/OpenTail.Stingray.Core/Grammar/JsonToolArgumentConstraint.cs:434-478,
 * computes the mask of a state by walking the vocabulary; JsonSchemaGrammarMasker.Filter :55-103) -- and meets them
 * again and again.  sr_mask_register copies the packed bits of one mask (ceil(vocab / 32) words, the format of
 * sr_batch_upload's allow_mask; host memory, or device memory when words_on_device is non-zero, e.g. what
 * sr_pack_allow_mask_launch wrote) into device memory once and returns its id; batches then name masks by id
 * (sr_batch_upload_mask_ids, sr_batch_append_tokens_masks) and a constrained decode step uploads 4 bytes per row
 * instead of 19 KB.  A context holds masks of one vocabulary size at a time.  sr_mask_release frees an id for
 * reuse.  A batch that still names a released id (or an id of a pool that was started again for another vocabulary) is
 * stale: every launch with it returns SR_ERR_INVALID_ARGUMENT until it is uploaded again or the row is given a
 * registered id by sr_batch_append_tokens_masks.
 */
SR_API int sr_mask_register(sr_ctx* ctx, const uint32_t* words, int words_on_device, int32_t vocab, int32_t* out_id);
SR_API int sr_mask_release(sr_ctx* ctx, int32_t mask_id);
/*
 * AndTokenConstraint.Filter (src/OpenTail.Stingray.Core/Grammar/AndTokenConstraint.cs:44-86) over registered masks: the
 * intersection of mask_ids[0..n) is written into a NEW registered mask whose id is returned in *out_id (released like any
 * other).  An entry of -1 (an inner constraint in its dead state, :74) is skipped.  *out_id is -1 -- "no mask", the row
 * goes unmasked -- when nothing is left to intersect, and when the intersection allows no token of the vocabulary (the
 * dead-intersection rule, :80-85).  At most 8 ids per call.  The call waits for the 4-byte answer "any token left";
 * a constraint pair meets the same pair of states again and again, so callers keep the result per tuple of ids.
 */
SR_API int sr_mask_and(sr_ctx* ctx, const int32_t* mask_ids, int32_t n, int32_t* out_id);
/* sr_batch_upload with the allow-mask of every row named by id: mask_ids [rows], -1 = the row is not constrained
 * (ITokenConstraint.Filter returned its input, ITokenConstraint.cs:36-41).  No copy is waited for. */
SR_API int sr_batch_upload_mask_ids(sr_batch* batch, int32_t rows, int32_t vocab,
                                    const sr_row_params* params,
                                    const int32_t* hist_ids, const int32_t* hist_offsets,
                                    const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                                    const int32_t* mask_ids,
                                    const double* uniforms, int32_t uniforms_per_row);
/* sr_batch_append_tokens for a batch uploaded with mask ids: every row also gets the mask of its constraint's next
 * state (mask_ids [rows], -1 = none), as the engine filters with the advanced constraint before the next Sample
 * (ContinuousBatchingEngine.cs:635-650: Filter -> Sample -> Accept -> RecentTokens.Add).  In place: a changed id is
 * 4 bytes in the row's descriptor, plus one rebuilt row of keep-bits for rows of the selection kernel. */
SR_API int sr_batch_append_tokens_masks(sr_batch* batch, const int32_t* tokens, const double* uniforms,
                                        const int32_t* mask_ids);

#ifdef __cplusplus
}
#endif
#endif /* STINGRAY_SAMPLER_H */
