// Host side of the full-vocabulary entry points: the slow path of Sampler.Sample, BuildFilteredDistribution,
// SampleWithDistribution, SampleFromProbs, ResampleResidual, the speculative accept loop and the MTP
// accept test.  Launch sequences only; all arithmetic is in sr_full.hip.
#include <cstring>

#include "sr_host.h"
#include "../../../include/stingray_sampler_test.h"

namespace {

// Runs the full-vocabulary pipeline for the rows in `list` (device array of n_rows row indices).
//   mode 0: work rows live in ctx scratch, tokens out.   mode 1/2: work rows ARE the caller's probs rows.
int run_full(sr_ctx* ctx, const sr_batch* b, const int32_t* list_dev, int n_rows, bool any_top_p, const void* logits_dev,
             int dtype, int64_t row_stride, int mode, float* probs_dev, int64_t probs_stride, int32_t* out_tokens_dev,
             uint32_t* out_flags_dev, bool lazy_scale = false, const std::vector<SrRow>* host_rows = nullptr)
{
    if (n_rows <= 0) return SR_OK;
    hipStream_t st = ctx->stream;
    const int vocab = b->vocab;
    SrFullArgs a{};
    a.logits = logits_dev;
    a.row_stride = row_stride;
    a.vocab = vocab;
    a.dtype = dtype;
    a.row_list = list_dev;
    a.rows = b->d_rows.as<SrRow>();
    a.edits = b->d_edits.as<SrEdit>();
    a.mask = sr_batch_mask_ptr(b);
    a.mask_stride = sr_batch_mask_stride(b);
    a.mode = mode;
    a.prof = ctx->prof;
    if (mode == 0) {
        const int64_t ws = (vocab + 3) & ~3;
        SR_HIP(ctx, ctx->work.reserve((size_t)n_rows * ws * sizeof(float), st));
        a.work = ctx->work.as<float>();
        a.work_stride = ws;
        a.work_by_row = 0;
    } else {
        a.work = probs_dev;
        a.work_stride = probs_stride;
        a.work_by_row = 1;
    }
    a.lazy_scale = lazy_scale ? 1 : 0;
    // Which of the rows that come here keep an adjusted copy, and which have their edits applied where they are read
    // (the rows of the batch that take this path: every row in modes 1 / 2).
    // Long rows that start on 16-byte boundaries, logits and work rows alike: the softmax denominators are prepared by
    // the pass over the whole device (k_full_softmax_seg) and the rows' workgroups only walk the records.  That pass also
    // applies the edits of the rows without an adjusted copy itself: they need no table and no kernel in front.
    const int nseg = (vocab + SR_SEG_TERMS - 1) / SR_SEG_TERMS;
    const bool seg_mode = [&] {
        const int es = dtype == SR_DTYPE_BF16 ? 2 : 4;
        const bool aligned = (((uintptr_t)logits_dev) & 15u) == 0u && ((row_stride * es) & 15) == 0 &&
                             (((uintptr_t)a.work) & 15u) == 0u && ((a.work_stride * 4) & 15) == 0;
        return vocab >= SR_SEG_MIN_VOCAB && nseg <= SR_SEG_MAX && aligned;
    }();
    a.edits_in_pass = seg_mode ? 1 : 0;
    bool any_table = false, any_copy = false, any_edits = false;
    int n_sampled = 0, n_seen = 0;
    for (const SrRow& r : (host_rows ? *host_rows : b->h_rows)) {
        if (mode == 0 && r.path != SR_PATH_FULL) continue;
        const bool on_the_fly = sr_row_edits_on_the_fly(r, vocab);
        any_table = any_table || (on_the_fly && !seg_mode);
        n_sampled += r.temperature > 0.0f ? 1 : 0;
        n_seen++;
        any_edits = any_edits || (r.edit_cnt > 0 && !(on_the_fly && seg_mode));
        any_copy = any_copy || !(r.temperature > 0.0f && (r.edit_cnt <= 0 || on_the_fly));
    }
    a.any_copy = any_copy ? 1 : 0;
    a.any_edits = any_edits ? 1 : 0;
    a.n_sampled = (int)((long long)n_sampled * n_rows / std::max(1, n_seen));  // (a verifier's launch has every row several times)
    a.edit_tab = nullptr;
    a.edit_tab_stride = (((int64_t)vocab + 31) / 32 + SR_FULL_EDIT_VALUES + 3) & ~(int64_t)3;
    if (any_table) {
        SR_HIP(ctx, ctx->edit_tab.reserve((size_t)n_rows * (size_t)a.edit_tab_stride * sizeof(uint32_t), st));
        a.edit_tab = ctx->edit_tab.as<uint32_t>();
    }
    // (cleared when new: the rows' maxima carry the number of the launch that wrote them, and the rows' scalars are
    // otherwise left by each launch the way the next one expects them)
    SR_HIP(ctx, ctx->full_state.reserve((size_t)n_rows * sizeof(SrFullState), st, true));
    a.state = ctx->full_state.as<SrFullState>();
    if (++ctx->full_seq == 0u) {  // the numbers have gone round: nothing of an earlier launch may look like this one's
        SR_HIP(ctx, hipMemsetAsync(ctx->full_state.p, 0, ctx->full_state.cap, st));
        if (ctx->full_seg_func.p) SR_HIP(ctx, hipMemsetAsync(ctx->full_seg_func.p, 0, ctx->full_seg_func.cap, st));
        if (ctx->full_row_sync.p) SR_HIP(ctx, hipMemsetAsync(ctx->full_row_sync.p, 0, ctx->full_row_sync.cap, st));
        ctx->full_seq = 1u;
    }
    a.seq = ctx->full_seq;
    a.row_wait_limit = ctx->row_wait_limit;
    // sort segments are laid out with the work stride of mode 0; in modes 1/2 use a private stride
    const int64_t seg_stride = (vocab + 3) & ~3;
    if ((int64_t)n_rows * seg_stride >= (int64_t)1 << 31)
        return sr_fail(ctx, SR_ERR_UNSUPPORTED, "full-vocabulary path: rows x vocab exceeds 2^31 entries");
    if (any_top_p) {
        // a row's segment: scratch of its top-p stage (histogram sums, the members of a long nucleus, and the survivors
        // of a row that the walk by slabs cannot close, sorted there by the row's workgroup)
        const size_t items = (size_t)n_rows * seg_stride;
        SR_HIP(ctx, ctx->sort_k0.reserve(items * 4, st));
        SR_HIP(ctx, ctx->sort_v0.reserve(items * 4, st));
        a.sort_keys_in = ctx->sort_k0.as<uint32_t>();
        a.sort_vals_in = ctx->sort_v0.as<int32_t>();
    }
    // the kernels index sort segments with work_stride; keep both strides equal in mode 0 and pass the
    // segment stride separately otherwise
    a.sort_stride = seg_stride;
    {
        if (seg_mode) {
            SR_HIP(ctx, ctx->full_seg_func.reserve((size_t)n_rows * (size_t)nseg * sizeof(SeqSegFunc), st, true));
            SR_HIP(ctx, ctx->full_seg_ms.reserve((size_t)n_rows * (size_t)nseg * sizeof(float2), st));
            SR_HIP(ctx, ctx->full_watch.reserve((size_t)n_rows * SR_FULL_SMALL_CAP * sizeof(unsigned long long), st));
            SR_HIP(ctx, ctx->full_watch_cnt.reserve((size_t)n_rows * sizeof(uint32_t), st, true));
            SR_HIP(ctx, ctx->full_row_sync.reserve((size_t)n_rows * SR_ROW_SYNC_STRIDE * sizeof(unsigned long long), st, true));
            a.row_sync = ctx->full_row_sync.as<unsigned long long>();
            a.seg_func = (SeqSegFunc*)ctx->full_seg_func.p;
            a.seg_ms = (float2*)ctx->full_seg_ms.p;
            a.seg_stride = nseg;
            a.watch = ctx->full_watch.as<unsigned long long>();
            a.watch_cnt = ctx->full_watch_cnt.as<uint32_t>();
            if (any_top_p && mode == 0) {
                a.seg_key_stride = ((int64_t)vocab + 7) & ~(int64_t)7;
                SR_HIP(ctx, ctx->full_seg_keys.reserve((size_t)n_rows * (size_t)a.seg_key_stride * sizeof(uint16_t), st));
                a.seg_keys = ctx->full_seg_keys.as<uint16_t>();
            }
        }
    }
    a.uniforms = b->d_uniforms.as<double>();
    a.uniforms_per_row = b->upr;
    a.out_tokens = out_tokens_dev;
    a.out_flags = out_flags_dev;
    // With a compute unit per row the row kernel's workgroups can have more shared memory each: rows that only top-p
    // cuts then walk their nucleus in slabs of twice the size.  (With more rows, two workgroups share a compute unit.)
    a.big_slabs = (mode == 0 && any_top_p && n_rows <= ctx->cu_count) ? 1 : 0;

    SR_HIP(ctx, sr_launch_full_prep(a, n_rows, st));
    SR_HIP(ctx, sr_launch_full_row(a, n_rows, st));  // (every row is finished by this one launch)
    return SR_OK;
}

bool row_uses_top_p(const SrRow& r) { return r.temperature > 0.0f && r.top_p < 1.0f && r.top_p > 0.0f; }

int check_batch_call(sr_ctx* ctx, const sr_batch* b, const void* logits_dev, int dtype, int64_t row_stride, const char* who)
{
    if (!logits_dev) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, std::string(who) + ": logits is null");
    if (dtype != SR_DTYPE_F32 && dtype != SR_DTYPE_BF16) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, std::string(who) + ": unknown dtype");
    if (b->vocab <= 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, std::string(who) + ": empty vocabulary");
    if (row_stride < b->vocab) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, std::string(who) + ": row stride < vocab");
    return sr_batch_masks_valid(ctx, b, who);
}

// identity row list [0, rows) on the device
int identity_list(sr_ctx* ctx, int rows, const int32_t** out)
{
    if (ctx->ident_rows < rows) {
        std::vector<int32_t> h((size_t)rows);
        for (int i = 0; i < rows; i++) h[(size_t)i] = i;
        SR_HIP(ctx, ctx->ident.reserve((size_t)rows * sizeof(int32_t), ctx->stream));
        SR_HIP(ctx, hipMemcpyAsync(ctx->ident.p, h.data(), (size_t)rows * sizeof(int32_t), hipMemcpyHostToDevice, ctx->stream));
        SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
        ctx->ident_rows = rows;
    }
    *out = ctx->ident.as<int32_t>();
    return SR_OK;
}

// The caller's uniforms for a kernel enqueued on the context's stream: copied into pinned memory of the context, which
// the kernel reads in place, so the call neither waits nor depends on the caller's array afterwards.
int upload_uniforms(sr_ctx* ctx, const double* uniforms, int rows, const double** dev)
{
    const size_t bytes = (size_t)rows * sizeof(double);
    SR_HIP(ctx, ctx->uni_ring.begin(bytes + 256, ctx->stream, 0, ctx->stream_epoch));
    const void* at = ctx->uni_ring.put(uniforms, bytes);
    if (!at) return sr_fail(ctx, SR_ERR_OUT_OF_MEMORY, "no pinned memory for the uniforms");
    *dev = (const double*)at;
    return SR_OK;
}

}  // namespace

int sr_full_rows_launch(sr_ctx* ctx, const sr_batch* b, const void* logits_dev, int dtype, int64_t row_stride,
                        int32_t* out_tokens_dev, uint32_t* out_flags_dev)
{
    bool any_top_p = false;
    for (int32_t r : b->h_full_list) any_top_p = any_top_p || row_uses_top_p(b->h_rows[(size_t)r]);
    return run_full(ctx, b, b->d_full_list.as<int32_t>(), (int)b->h_full_list.size(), any_top_p, logits_dev, dtype,
                    row_stride, 0, nullptr, 0, out_tokens_dev, out_flags_dev);
}

// SampleTopK (Sampler.cs:216-357) for rows whose k + history length exceeds what the selection kernel's row tail
// sorts: the row sorted where it lies by one workgroup, its first k + history-length entries adjusted and sorted
// again, and a walk over the result by the same workgroup.
int sr_wide_rows_launch(sr_ctx* ctx, const sr_batch* b, const int32_t* list_dev, int n_rows, const void* logits_dev,
                        int dtype, int64_t row_stride, int32_t* out_tokens_dev, uint32_t* out_flags_dev)
{
    if (n_rows <= 0) return SR_OK;
    hipStream_t st = ctx->stream;
    const int vocab = b->vocab;
    const int64_t stride = (vocab + 3) & ~3;
    if ((int64_t)n_rows * stride >= (int64_t)1 << 31)
        return sr_fail(ctx, SR_ERR_UNSUPPORTED, "wide top-k rows: rows x vocab exceeds 2^31 entries");
    const size_t items = (size_t)n_rows * (size_t)stride;
    SrFullArgs a{};
    a.logits = logits_dev;
    a.row_stride = row_stride;
    a.vocab = vocab;
    a.dtype = dtype;
    a.row_list = list_dev;
    a.rows = b->d_rows.as<SrRow>();
    a.edits = b->d_edits.as<SrEdit>();
    a.mask = sr_batch_mask_ptr(b);
    a.mask_stride = sr_batch_mask_stride(b);
    SR_HIP(ctx, ctx->work.reserve(items * sizeof(float), st));
    a.work = ctx->work.as<float>();
    a.work_stride = stride;
    SR_HIP(ctx, ctx->sort_k0.reserve(items * 4, st));
    SR_HIP(ctx, ctx->sort_v0.reserve(items * 4, st));
    SR_HIP(ctx, ctx->sort_v1.reserve(items * 4, st));
    a.sort_keys_in = ctx->sort_k0.as<uint32_t>();
    a.sort_vals_in = ctx->sort_v0.as<int32_t>();
    a.wide_ids = ctx->sort_v1.as<int32_t>();
    a.sort_stride = stride;
    a.uniforms = b->d_uniforms.as<double>();
    a.uniforms_per_row = b->upr;
    a.out_tokens = out_tokens_dev;
    a.out_flags = out_flags_dev;

    SR_HIP(ctx, sr_launch_wide_keys(a, n_rows, st));
    SR_HIP(ctx, sr_launch_wide_sort(a, n_rows, 1, st));
    SR_HIP(ctx, sr_launch_wide_adjust(a, n_rows, st));
    SR_HIP(ctx, sr_launch_wide_sort(a, n_rows, 0, st));
    SR_HIP(ctx, sr_launch_wide_tail(a, n_rows, st));
    return SR_OK;
}

extern "C" {

int sr_build_distribution_launch(sr_ctx* ctx, const sr_batch* b, const void* logits_dev, int dtype, int64_t row_stride,
                                 float* out_probs_dev, int64_t probs_stride, int32_t probs_len)
{
    if (!ctx || !b) return SR_ERR_NULL_ARGUMENT;
    if (b->rows == 0) return SR_OK;
    if (probs_len != b->vocab)  // Sampler.cs:121-123
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "probs length (" + std::to_string(probs_len) + ") must equal logits length (" +
                                                         std::to_string(b->vocab) + ").");
    int rc = check_batch_call(ctx, b, logits_dev, dtype, row_stride, "sr_build_distribution_launch");
    if (rc != SR_OK) return rc;
    if (!out_probs_dev) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_build_distribution_launch: probs is null");
    if (probs_stride < b->vocab) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_build_distribution_launch: probs stride < vocab");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    const int32_t* list = nullptr;
    rc = identity_list(ctx, b->rows, &list);
    if (rc != SR_OK) return rc;
    bool any_top_p = false;
    for (const SrRow& r : b->h_rows) any_top_p = any_top_p || row_uses_top_p(r);
    return run_full(ctx, b, list, b->rows, any_top_p, logits_dev, dtype, row_stride, 1, out_probs_dev, probs_stride, nullptr, nullptr);
}

int sr_sample_with_distribution_launch(sr_ctx* ctx, const sr_batch* b, const void* logits_dev, int dtype, int64_t row_stride,
                                       float* out_probs_dev, int64_t probs_stride, int32_t probs_len, int32_t* out_tokens_dev)
{
    if (!ctx || !b) return SR_ERR_NULL_ARGUMENT;
    if (b->rows == 0) return SR_OK;
    if (probs_len != b->vocab)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "probs length (" + std::to_string(probs_len) + ") must equal logits length (" +
                                                         std::to_string(b->vocab) + ").");
    int rc = check_batch_call(ctx, b, logits_dev, dtype, row_stride, "sr_sample_with_distribution_launch");
    if (rc != SR_OK) return rc;
    if (!out_probs_dev || !out_tokens_dev) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_sample_with_distribution_launch: null output");
    if (probs_stride < b->vocab) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_sample_with_distribution_launch: probs stride < vocab");
    for (const SrRow& r : b->h_rows)
        if (r.temperature > 0.0f && b->upr < 1)
            return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_sample_with_distribution_launch: a sampled row needs a uniform");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    const int32_t* list = nullptr;
    rc = identity_list(ctx, b->rows, &list);
    if (rc != SR_OK) return rc;
    bool any_top_p = false;
    for (const SrRow& r : b->h_rows) any_top_p = any_top_p || row_uses_top_p(r);
    return run_full(ctx, b, list, b->rows, any_top_p, logits_dev, dtype, row_stride, 2, out_probs_dev, probs_stride, out_tokens_dev, nullptr);
}

int sr_sample_from_probs_launch(sr_ctx* ctx, const float* probs_dev, int32_t rows, int32_t vocab, int64_t probs_stride,
                                const double* uniforms, int32_t* out_tokens_dev)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (!uniforms) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "rng");  // ArgumentNullException(rng), Sampler.cs:197
    if (rows == 0) return SR_OK;
    if (!probs_dev || !out_tokens_dev) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_sample_from_probs_launch: null tensor");
    if (rows < 0 || vocab <= 0 || probs_stride < vocab) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_sample_from_probs_launch: bad shape");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    const double* u = nullptr;
    int rc = upload_uniforms(ctx, uniforms, rows, &u);
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, sr_launch_draw_rows(probs_dev, probs_stride, vocab, rows, u, out_tokens_dev, ctx->stream));
    return SR_OK;
}

int sr_resample_residual_launch(sr_ctx* ctx, const float* p_dev, int32_t p_len, int64_t p_stride, const float* q_dev,
                                int32_t q_len, int64_t q_stride, int32_t rows, const double* uniforms, int32_t* out_tokens_dev)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (!uniforms) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "rng");  // Sampler.cs:589
    if (p_len != q_len)                                                // Sampler.cs:590-592
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT,
                       "p and q must have equal length (" + std::to_string(p_len) + " vs " + std::to_string(q_len) + ").");
    if (rows == 0) return SR_OK;
    if (!p_dev || !q_dev || !out_tokens_dev) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_resample_residual_launch: null tensor");
    if (rows < 0 || p_len <= 0 || p_stride < p_len || q_stride < q_len)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_resample_residual_launch: bad shape");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    const double* u = nullptr;
    int rc = upload_uniforms(ctx, uniforms, rows, &u);
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, sr_launch_residual_rows(p_dev, p_stride, q_dev, q_stride, p_len, rows, u, out_tokens_dev, ctx->stream));
    return SR_OK;
}


// ---- span-shaped forms: host buffers in, host results out ------------------------------------------------

static int stage_up(sr_ctx* ctx, DeviceBuf& buf, const void* src, size_t bytes)
{
    SR_HIP(ctx, buf.reserve(bytes, ctx->stream));
    SR_HIP(ctx, hipMemcpyAsync(buf.p, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    return SR_OK;
}

static int distribution_host(sr_ctx* ctx, const char* what, bool sample, const float* logits, int32_t rows, int32_t vocab,
                             int64_t row_stride, const sr_row_params* params, const int32_t* hist_ids,
                             const int32_t* hist_offsets, const int32_t* bias_ids, const float* bias_vals,
                             const int32_t* bias_offsets, const double* uniforms, float* out_probs, int64_t probs_stride,
                             int32_t probs_len, int32_t* out_tokens)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (rows == 0) return SR_OK;
    if (probs_len != vocab)  // Sampler.cs:121-123
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "probs length (" + std::to_string(probs_len) + ") must equal logits length (" +
                                                         std::to_string(vocab) + ").");
    if (!logits || !params || !out_probs || (sample && !out_tokens))
        return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, std::string(what) + ": null argument");
    if (rows < 0 || vocab <= 0 || row_stride < vocab || probs_stride < vocab)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, std::string(what) + ": bad shape");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    if (!ctx->tmp_batch) {
        int rc = sr_batch_create(ctx, &ctx->tmp_batch);
        if (rc != SR_OK) return rc;
    }
    int rc = sr_batch_upload(ctx->tmp_batch, rows, vocab, params, hist_ids, hist_offsets, bias_ids, bias_vals, bias_offsets,
                             nullptr, 0, nullptr, uniforms, uniforms ? 1 : 0);
    if (rc != SR_OK) return rc;
    const size_t in_bytes = ((size_t)(rows - 1) * (size_t)row_stride + (size_t)vocab) * sizeof(float);
    rc = stage_up(ctx, ctx->host_logits, logits, in_bytes);
    if (rc != SR_OK) return rc;
    const int64_t ps = (vocab + 3) & ~3;
    SR_HIP(ctx, ctx->stage_probs.reserve((size_t)rows * (size_t)ps * sizeof(float), ctx->stream));
    SR_HIP(ctx, ctx->out_tokens.reserve((size_t)rows * sizeof(int32_t), ctx->stream));
    if (sample)
        rc = sr_sample_with_distribution_launch(ctx, ctx->tmp_batch, ctx->host_logits.p, SR_DTYPE_F32, row_stride,
                                                ctx->stage_probs.as<float>(), ps, probs_len, ctx->out_tokens.as<int32_t>());
    else
        rc = sr_build_distribution_launch(ctx, ctx->tmp_batch, ctx->host_logits.p, SR_DTYPE_F32, row_stride,
                                          ctx->stage_probs.as<float>(), ps, probs_len);
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, hipMemcpy2DAsync(out_probs, (size_t)probs_stride * sizeof(float), ctx->stage_probs.p, (size_t)ps * sizeof(float),
                                 (size_t)vocab * sizeof(float), (size_t)rows, hipMemcpyDeviceToHost, ctx->stream));
    if (sample)
        SR_HIP(ctx, hipMemcpyAsync(out_tokens, ctx->out_tokens.p, (size_t)rows * sizeof(int32_t), hipMemcpyDeviceToHost, ctx->stream));
    SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SR_OK;
}

int sr_build_distribution(sr_ctx* ctx, const float* logits, int32_t rows, int32_t vocab, int64_t row_stride,
                          const sr_row_params* params, const int32_t* hist_ids, const int32_t* hist_offsets,
                          const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets, float* out_probs,
                          int64_t probs_stride, int32_t probs_len)
{
    return distribution_host(ctx, "sr_build_distribution", false, logits, rows, vocab, row_stride, params, hist_ids, hist_offsets,
                             bias_ids, bias_vals, bias_offsets, nullptr, out_probs, probs_stride, probs_len, nullptr);
}

int sr_sample_with_distribution(sr_ctx* ctx, const float* logits, int32_t rows, int32_t vocab, int64_t row_stride,
                                const sr_row_params* params, const int32_t* hist_ids, const int32_t* hist_offsets,
                                const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                                const double* uniforms, float* out_probs, int64_t probs_stride, int32_t probs_len,
                                int32_t* out_tokens)
{
    return distribution_host(ctx, "sr_sample_with_distribution", true, logits, rows, vocab, row_stride, params, hist_ids,
                             hist_offsets, bias_ids, bias_vals, bias_offsets, uniforms, out_probs, probs_stride, probs_len,
                             out_tokens);
}

int sr_sample_from_probs(sr_ctx* ctx, const float* probs, int32_t rows, int32_t vocab, int64_t probs_stride,
                         const double* uniforms, int32_t* out_tokens)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (!uniforms) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "rng");  // ArgumentNullException(rng), Sampler.cs:197
    if (rows == 0) return SR_OK;
    if (!probs || !out_tokens) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_sample_from_probs: null argument");
    if (rows < 0 || vocab <= 0 || probs_stride < vocab) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_sample_from_probs: bad shape");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    int rc = stage_up(ctx, ctx->host_logits, probs, ((size_t)(rows - 1) * (size_t)probs_stride + (size_t)vocab) * sizeof(float));
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, ctx->out_tokens.reserve((size_t)rows * sizeof(int32_t), ctx->stream));
    rc = sr_sample_from_probs_launch(ctx, ctx->host_logits.as<float>(), rows, vocab, probs_stride, uniforms, ctx->out_tokens.as<int32_t>());
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, hipMemcpyAsync(out_tokens, ctx->out_tokens.p, (size_t)rows * sizeof(int32_t), hipMemcpyDeviceToHost, ctx->stream));
    SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SR_OK;
}

int sr_resample_residual(sr_ctx* ctx, const float* p, int32_t p_len, int64_t p_stride, const float* q, int32_t q_len,
                         int64_t q_stride, int32_t rows, const double* uniforms, int32_t* out_tokens)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (!uniforms) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "rng");  // Sampler.cs:589
    if (p_len != q_len)                                                // Sampler.cs:590-592
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT,
                       "p and q must have equal length (" + std::to_string(p_len) + " vs " + std::to_string(q_len) + ").");
    if (rows == 0) return SR_OK;
    if (!p || !q || !out_tokens) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_resample_residual: null argument");
    if (rows < 0 || p_len <= 0 || p_stride < p_len || q_stride < q_len)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_resample_residual: bad shape");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    int rc = stage_up(ctx, ctx->host_logits, p, ((size_t)(rows - 1) * (size_t)p_stride + (size_t)p_len) * sizeof(float));
    if (rc != SR_OK) return rc;
    rc = stage_up(ctx, ctx->stage_probs, q, ((size_t)(rows - 1) * (size_t)q_stride + (size_t)q_len) * sizeof(float));
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, ctx->out_tokens.reserve((size_t)rows * sizeof(int32_t), ctx->stream));
    rc = sr_resample_residual_launch(ctx, ctx->host_logits.as<float>(), p_len, p_stride, ctx->stage_probs.as<float>(), q_len, q_stride,
                                     rows, uniforms, ctx->out_tokens.as<int32_t>());
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, hipMemcpyAsync(out_tokens, ctx->out_tokens.p, (size_t)rows * sizeof(int32_t), hipMemcpyDeviceToHost, ctx->stream));
    SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SR_OK;
}

int sr_spec_verify_launch(sr_ctx* ctx, const sr_batch* b, const float* target_logits_dev, const float* draft_probs_dev,
                          const int32_t* draft_tokens_dev, int32_t n_draft, int32_t* out_accepted_dev, int32_t* out_tokens_dev)
{
    if (!ctx || !b) return SR_ERR_NULL_ARGUMENT;
    if (b->rows == 0) return SR_OK;
    if (n_draft < 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_spec_verify_launch: negative draft length");
    if (!target_logits_dev || !out_accepted_dev || !out_tokens_dev || (n_draft > 0 && !draft_tokens_dev))
        return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_spec_verify_launch: null tensor");
    if (n_draft > 0 && !draft_probs_dev) {
        // only rows under the ratio test read q (SpeculativeDecoder.cs:538-543)
        for (int r = 0; r < b->rows; r++) {
            const SrRow& d = b->h_rows[(size_t)r];
            if (!(d.p_min > 0.0f && d.p_min < 1.0f) && !(d.flags & SR_ROW_DRAFT_FROM_LOOKUP))
                return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_spec_verify_launch: a row under the ratio test needs the draft distributions");
        }
    }
    if (b->vocab <= 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_spec_verify_launch: empty vocabulary");
    if (b->upr < n_draft + 1) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_spec_verify_launch: needs n_draft + 1 uniforms per row");
    if (b->has_mask) return sr_fail(ctx, SR_ERR_UNSUPPORTED, "sr_spec_verify_launch: allow-masks are not part of speculative verification");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    const int rows = b->rows, V = b->vocab, P = n_draft + 1;
    // Every position of a row is filtered with the row's parameters (SpeculativeDecoder.cs:535): expand the
    // batch's row descriptors to rows x positions and build all distributions in one pass.
    if ((int64_t)rows * P * V >= (int64_t)1 << 31)
        return sr_fail(ctx, SR_ERR_UNSUPPORTED, "sr_spec_verify_launch: rows x positions x vocab exceeds 2^31 entries");
    bool any_top_p = false;
    for (int r = 0; r < rows; r++) any_top_p = any_top_p || row_uses_top_p(b->h_rows[(size_t)r]);
    // (made by a kernel, so that the call does not wait for the host; kept with the batch until its descriptors change)
    if (b->spec_positions != P) {
        SR_HIP(ctx, b->spec_rows.reserve((size_t)rows * P * sizeof(SrRow), st));
        SR_HIP(ctx, sr_launch_expand_rows(b->d_rows.as<SrRow>(), b->spec_rows.as<SrRow>(), rows, P, st));
        b->spec_positions = P;
    }
    SR_HIP(ctx, ctx->spec_probs.reserve((size_t)rows * P * V * sizeof(float), st));
    sr_batch tmp;  // a view: expanded rows, the original edits
    tmp.ctx = ctx;
    tmp.rows = rows * P;
    tmp.vocab = V;
    tmp.upr = 0;
    tmp.d_rows.p = b->spec_rows.p;
    tmp.d_edits.p = b->d_edits.p;
    tmp.mask_stride = 0;
    const int32_t* list = nullptr;
    int rc = identity_list(ctx, rows * P, &list);
    if (rc == SR_OK)
        rc = run_full(ctx, &tmp, list, rows * P, any_top_p, target_logits_dev, SR_DTYPE_F32, V, 1, ctx->spec_probs.as<float>(), V,
                      nullptr, nullptr, true, &b->h_rows);  // (the verifier applies the normalising factors of unfiltered rows itself)
    tmp.d_rows.p = nullptr;  // borrowed
    tmp.d_edits.p = nullptr;
    if (rc != SR_OK) return rc;
    SrSpecArgs a{};
    a.rows = b->d_rows.as<SrRow>();
    a.vocab = V;
    a.n_draft = n_draft;
    a.p_all = ctx->spec_probs.as<float>();
    a.state = ctx->full_state.as<SrFullState>();
    a.target_logits = target_logits_dev;
    a.draft_probs = draft_probs_dev;
    a.draft_tokens = draft_tokens_dev;
    a.uniforms = b->d_uniforms.as<double>();
    a.uniforms_per_row = b->upr;
    a.out_accepted = out_accepted_dev;
    a.out_tokens = out_tokens_dev;
    a.resid_stride = ((int64_t)V + 3) & ~(int64_t)3;
    SR_HIP(ctx, ctx->spec_resid.reserve((size_t)rows * (size_t)a.resid_stride * sizeof(float), st));
    SR_HIP(ctx, ctx->spec_reject.reserve((size_t)rows * sizeof(int32_t), st));
    a.resid = ctx->spec_resid.as<float>();
    a.reject = ctx->spec_reject.as<int32_t>();
    a.seg_stride = (V + SR_SEG_TERMS - 1) / SR_SEG_TERMS;
    if (a.seg_stride <= SR_SEG_MAX) {  // (longer rows are added by their workgroups alone)
        SR_HIP(ctx, ctx->seg_part.reserve((size_t)rows * (size_t)a.seg_stride * sizeof(double), st));
        SR_HIP(ctx, ctx->seg_func.reserve((size_t)rows * (size_t)a.seg_stride * sizeof(SeqSegFunc), st));
        a.seg_part = ctx->seg_part.as<double>();
        a.seg_func = (SeqSegFunc*)ctx->seg_func.p;
    }
    SR_HIP(ctx, sr_launch_spec_verify(a, rows, st));
    return SR_OK;
}

int sr_mtp_verify_launch(sr_ctx* ctx, const float* logits_dev, int32_t rows, int32_t vocab, int64_t row_stride,
                         const int32_t* draft_tokens_dev, float p_min, int32_t* out_argmax_dev, int32_t* out_accept_dev,
                         float* out_prob_dev)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (rows == 0) return SR_OK;
    if (!logits_dev || !draft_tokens_dev || !out_argmax_dev || !out_accept_dev)
        return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_mtp_verify_launch: null tensor");
    if (rows < 0 || vocab <= 0 || row_stride < vocab) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_mtp_verify_launch: bad shape");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    // p_min <= 0 means "argmax match only" (SamplingParams.SpecDraftPMin, Sampler.cs:791)
    const float pm = p_min > 0.0f ? p_min : 1.0f;
    SR_HIP(ctx, sr_launch_mtp_verify(logits_dev, row_stride, vocab, rows, draft_tokens_dev, pm, out_argmax_dev, out_accept_dev,
                                     out_prob_dev, ctx->stream));
    return SR_OK;
}

#ifdef SR_TEST_HOOKS
// Test hook (include/stingray_sampler_test.h): exact left-to-right sum of x_dev[0..n) from s0
int sr_selftest_seqsum(sr_ctx* ctx, const float* x_dev, int32_t n, float s0, float target, float* out_sum_dev,
                              int32_t* out_idx_dev)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    SR_HIP(ctx, hipSetDevice(ctx->device));
    SR_HIP(ctx, sr_launch_selftest_seqsum(x_dev, n, s0, target, out_sum_dev, out_idx_dev, ctx->stream));
    return SR_OK;
}
// Test hook: the same sum as the whole device prepares it (segments' records made for predictions that are `skew`
// times the segments' true sums, the walk of one wave): out_sum_dev[0], out_idx_dev[0] from the sum and the search
// over its states, [1] from the walk that searches by itself
int sr_selftest_segsum(sr_ctx* ctx, const float* x_dev, int32_t n, double skew, float target, float* out_sum_dev,
                       int32_t* out_idx_dev)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (n <= 0 || (n + SR_SEG_TERMS - 1) / SR_SEG_TERMS > SR_SEG_MAX) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_selftest_segsum: length");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    const size_t nseg = (size_t)(n + SR_SEG_TERMS - 1) / SR_SEG_TERMS;
    SR_HIP(ctx, ctx->seg_part.reserve(nseg * sizeof(double), ctx->stream));
    SR_HIP(ctx, ctx->seg_func.reserve(nseg * sizeof(SeqSegFunc), ctx->stream));
    SR_HIP(ctx, sr_launch_selftest_segsum(x_dev, n, skew, target, ctx->seg_part.as<double>(), (SeqSegFunc*)ctx->seg_func.p,
                                          out_sum_dev, out_idx_dev, ctx->stream));
    return SR_OK;
}
#endif  // SR_TEST_HOOKS

}  // extern "C"
