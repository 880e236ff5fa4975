// Host side of the C ABI declared in include/stingray_sampler.h: context and scratch ownership, the
// packer that turns SamplingParams / PreviousTokens / LogitBias into device row descriptors, and the
// per-entry-point launch sequences.  No vocabulary-sized work happens on the host.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>

#include "sr_host.h"
#include "../../../include/stingray_sampler_test.h"

// where a batch's allow-masks lie: its own upload, or the context's registered masks
const uint32_t* sr_batch_mask_ptr(const sr_batch* b) { return b->mask_ids ? b->ctx->mask_pool.as<uint32_t>() : b->d_mask.as<uint32_t>(); }
int64_t sr_batch_mask_stride(const sr_batch* b) { return b->mask_ids ? (int64_t)b->ctx->pool_words : b->mask_stride; }

int sr_batch_masks_valid(sr_ctx* ctx, const sr_batch* b, const char* who)
{
    if (!b->mask_ids) return SR_OK;
    bool stale = b->keep_mask_ids.size() != (size_t)b->rows;
    for (int32_t r = 0; r < b->rows && !stale; r++) {
        const int32_t id = b->keep_mask_ids[(size_t)r];
        if (id < 0) continue;  // (a batch whose rows name no mask reads none)
        stale = b->mask_pool_gen != ctx->pool_gen || ctx->pool_vocab != b->vocab || id >= ctx->pool_cap ||
                !ctx->pool_used[(size_t)id] || ctx->pool_slot_gen[(size_t)id] != b->keep_mask_gen[(size_t)r];
    }
    if (stale)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, std::string(who) + ": the batch names a registered mask that was released, or whose "
                                                         "pool was started again for another vocabulary, after the batch took its id; "
                                                         "upload the batch again");
    return SR_OK;
}

namespace {

inline bool has_history_penalty(const sr_row_params& p)
{
    return p.repetition_penalty != 1.0f || p.presence_penalty != 0.0f || p.frequency_penalty != 0.0f;
}

// Chunking of a row for the selection kernel: a chunk is a whole number of 64-vector blocks of the row's
// window of 16-byte vectors and must fit the per-workgroup register window.
void topk_geometry(int vocab, int dtype, int n_rows, int cu_count, int* chunks, int* chunk_vecs)
{
    const int epv = dtype == SR_DTYPE_BF16 ? 8 : 4;
    const int window = (dtype == SR_DTYPE_BF16 ? SR_TK_VEC_BF16 : SR_TK_VEC) * SR_TK_THREADS;  // vectors a workgroup holds
    const int nvt = (vocab + 2 * epv - 2) / epv;                   // vectors of a row that starts mid-vector
    int s_min = (nvt + window - 1) / window;
    int s_par = (2 * cu_count + n_rows - 1) / std::max(n_rows, 1);  // aim for two workgroups per CU
    // the row tail keeps the per-group results of up to 4 chunks in registers; more chunks only when the row needs them
    int s_cap = std::min(4, std::max(1, vocab / 8192));
    int s = std::max(s_min, std::min(s_par, s_cap));
    int cv = (nvt + s - 1) / s;
    cv = (cv + 63) & ~63;
    if (cv > window) cv = window;  // window is a multiple of 64
    s = (nvt + cv - 1) / cv;
    *chunks = std::max(s, 1);
    *chunk_vecs = cv;
}

// Sends the packed pieces: one kernel reads them from the pinned memory and writes them where they belong.  To be
// called before anything that reads the destinations is enqueued.
hipError_t batch_flush(sr_batch* b, hipStream_t st)
{
    if (b->segs.empty()) return hipSuccess;
    const SrCopySeg* table = (const SrCopySeg*)b->stage.put(b->segs.data(), b->segs.size() * sizeof(SrCopySeg));
    hipError_t e = hipSuccess;
    if (table) {
        e = sr_launch_scatter(table, (int)b->segs.size(), st);
    } else {  // no room for the list (the pinned memory grows for the next upload): one copy per piece
        for (const SrCopySeg& s : b->segs) {
            e = hipMemcpyAsync(s.dst, s.src, (size_t)s.bytes, hipMemcpyHostToDevice, st);
            if (e != hipSuccess) break;
        }
    }
    b->segs.clear();
    return e;
}

// Copies host data of a batch to the device on `st`: through the batch's pinned memory when `staged` (no wait
// needed), else straight from `src`, which the caller then has to keep alive until the stream is synchronised.
hipError_t batch_copy(sr_batch* b, bool staged, void* dst, const void* src, size_t bytes, hipStream_t st)
{
    if (bytes == 0) return hipSuccess;
    const void* from = staged ? b->stage.put(src, bytes) : nullptr;
    if (from) {  // packed: sent with the other pieces by batch_flush; a later version of the same array replaces the earlier
        for (SrCopySeg& s : b->segs)
            if (s.dst == dst) { s.src = from; s.bytes = (unsigned long long)bytes; return hipSuccess; }
        b->segs.push_back(SrCopySeg{from, dst, (unsigned long long)bytes});
        return hipSuccess;
    }
    // Straight from the caller's memory.  The packed pieces go first: one of them may be an earlier version of this
    // very array (the row descriptors are sent again once their scan-mask rows are known), and the order of the
    // two must stay the order of the calls.
    hipError_t e = batch_flush(b, st);
    if (e != hipSuccess) return e;
    b->upload_must_wait = true;
    return hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, st);
}

// (Re)builds the scan masks of a batch for logits of the given vector width and alignment.  Rows without an
// allow-mask and without excluded history ids share one mask row when every row starts at the same offset
// inside its first vector.
int prepare_scan(sr_batch* b, int epv, unsigned long long base_addr, long long stride_bytes, bool staged = false)
{
    sr_ctx* ctx = b->ctx;
    hipStream_t st = ctx->stream;
    const int base_mod = (int)(base_addr & 15ull), stride_mod = (int)(stride_bytes & 15ll);
    if (b->scan_epv == epv && b->scan_base_mod == base_mod && b->scan_stride_mod == stride_mod) return SR_OK;
    const bool can_share = stride_mod == 0 || b->rows <= 1;
    b->h_scan.clear();
    int shared = -1;
    bool rows_changed = false;
    for (int32_t r : b->h_sel_list) {
        SrRow& d = b->h_rows[(size_t)r];
        const uint32_t need = b->h_scan_need[(size_t)r];
        int32_t idx;
        if (need == 0u && can_share) {
            if (shared < 0) { shared = (int)b->h_scan.size(); b->h_scan.push_back(SrScanDesc{r, 0u}); }
            idx = shared;
        } else {
            idx = (int32_t)b->h_scan.size();
            b->h_scan.push_back(SrScanDesc{r, need});
        }
        if (d.scan_row != idx) { d.scan_row = idx; rows_changed = true; }
    }
    b->scan_epv = epv;
    b->scan_base_mod = base_mod;
    b->scan_stride_mod = stride_mod;
    if (b->h_scan.empty()) return SR_OK;
    const int n_sel = (int)b->h_sel_list.size();
    int chunks = 1, chunk_vecs = 0;
    topk_geometry(b->vocab, epv == 8 ? SR_DTYPE_BF16 : SR_DTYPE_F32, n_sel, ctx->cu_count, &chunks, &chunk_vecs);
    {
        // The selection kernel's grid: workers with a program each -- chunk items to stream, then at most one row to
        // finish.  One worker per CU is resident from the start and a later one starts when one of them ends.  (A CU
        // holds two workgroups of the kernel that launches of more workers than CUs take; with one per CU the launch
        // takes the kernel that is compiled for half as many waves and keeps its row tails' registers: 80 rows
        // 29.8 -> 27.3 us, 112 rows 32.5 -> 31.1 us against two workers per CU, measured.)
        //
        // The programs are written by a simulation of the launch: the chunk items, rows in order of decreasing tail
        // length, are dealt out one by one to the worker that will be free first; the worker that gets a row's last
        // chunk also gets the row's tail, which ends its program, and frees a slot for the next worker of the grid
        // when the tail is done.  The estimates (a chunk, a tail of a given size) only have to be roughly right: a
        // tail that starts before its row's other chunks are in waits for them, a worker that is late delays nobody
        // but its own items.
        //
        // The device's compute dies (XCDs, 32 CUs and one L2 each) take the workgroups of a grid in turn: workgroup i
        // runs on die i mod n_xcd.  Row slot s is given to die s mod n_xcd, and only workers of that die get its items,
        // so that what a row's chunks write is in the L2 that its tail reads from.  Nothing depends on that placement
        // for correctness.  A batch of few rows deals its items out to all dies instead.
        const int n_xcd = std::min(SR_TK_MAX_XCD, std::max(1, ctx->cu_count / 32));
        const int resident = std::max(ctx->cu_count, n_xcd);
        const int total_items = n_sel * chunks;
        const bool spread = n_sel < 2 * n_xcd;
        const int n_pool = spread ? 1 : n_xcd;        // pools of workers that share a list of items
        const int per_pool = resident / n_pool;         // resident workers of a pool
        const double t_item = epv == 8 ? 6.0 : 9.0;     // microseconds: one chunk, streamed under the loads of the next
        auto t_tail = [](const SrRow& d) { return d.sel <= 1 ? 8.0 : 11.0 + 0.0105 * (double)(d.sel + d.edit_cnt); };
        struct Worker { double free_at; int id; };
        auto later = [](const Worker& p, const Worker& q) { return p.free_at > q.free_at || (p.free_at == q.free_at && p.id > q.id); };
        std::vector<std::vector<int32_t>> prog_items;   // per worker: indices into `entries`
        std::vector<int32_t> prog_tail;
        std::vector<int32_t> entries;                    // 4 ints per item, in list order
        std::vector<std::vector<Worker>> heap((size_t)n_pool);
        std::vector<std::vector<double>> slot_free((size_t)n_pool);  // when the slots of ended workers fall free
        // worker ids: pool p owns the grid positions p, p + n_pool, ... (= die p when every die is a pool)
        std::vector<int> next_id((size_t)n_pool);
        auto new_worker = [&](int p, double at) {
            const int id = next_id[(size_t)p];
            next_id[(size_t)p] += n_pool;
            if ((size_t)id >= prog_items.size()) { prog_items.resize((size_t)id + 1); prog_tail.resize((size_t)id + 1, -1); }
            heap[(size_t)p].push_back(Worker{at, id});
            std::push_heap(heap[(size_t)p].begin(), heap[(size_t)p].end(), later);
        };
        for (int p = 0; p < n_pool; p++) {
            next_id[(size_t)p] = p;
            const int n_first = std::min(per_pool, (total_items + n_pool - 1) / n_pool);
            for (int w = 0; w < n_first; w++) new_worker(p, 0.0);
        }
        // With rows for more than about half the compute units nothing is gained by spreading a row over workers
        // (a compute unit streams at little more than its share of the memory bandwidth anyway, and tails that run
        // beside the streaming slow it down by more than they gain): every worker streams all chunks of one row and
        // finishes it, waits for nobody and hands nothing over.  (Measured on 256 compute units, 151,936 fp32 logits
        // a row: the two ways cost the same at 136 rows; at 192 rows 37.8 against 45.9 us, at 128 rows 36.0 against
        // 33.2 us.)
        const bool affine = n_sel * 32 >= ctx->cu_count * 17;
        if (affine) {
            prog_items.assign((size_t)n_sel, {});
            prog_tail.assign((size_t)n_sel, -1);
        }
        for (int slot = 0; slot < n_sel; slot++) {
            const int32_t r = b->h_sel_list[(size_t)slot];
            const SrRow& d = b->h_rows[(size_t)r];
            const int p = spread ? 0 : slot % n_xcd;
            if (affine) {
                for (int c = 0; c < chunks; c++) {
                    prog_items[(size_t)slot].push_back((int32_t)(entries.size() / 4));
                    entries.push_back((int32_t)(((uint32_t)c << 24) | (uint32_t)slot));
                    entries.push_back(r);
                    entries.push_back(d.scan_row);
                    entries.push_back(b->sel_cap[(size_t)r]);
                }
                prog_tail[(size_t)slot] = slot;
                continue;
            }
            for (int c = 0; c < chunks; c++) {
                std::vector<Worker>& h = heap[(size_t)p];
                if (h.empty()) {  // every worker of the pool has ended with a tail: the next one takes over its slot
                    std::vector<double>& sf = slot_free[(size_t)p];
                    std::sort(sf.begin(), sf.end());
                    new_worker(p, sf.empty() ? 0.0 : sf.front());
                    if (!sf.empty()) sf.erase(sf.begin());
                }
                std::pop_heap(h.begin(), h.end(), later);
                Worker w = h.back();
                h.pop_back();
                prog_items[(size_t)w.id].push_back((int32_t)(entries.size() / 4));
                entries.push_back((int32_t)(((uint32_t)c << 24) | (uint32_t)slot));
                entries.push_back(r);
                entries.push_back(d.scan_row);
                entries.push_back(b->sel_cap[(size_t)r]);
                w.free_at += t_item;
                if (c == chunks - 1) {
                    prog_tail[(size_t)w.id] = slot;
                    slot_free[(size_t)p].push_back(w.free_at + t_tail(d));
                } else {
                    h.push_back(w);
                    std::push_heap(h.begin(), h.end(), later);
                }
            }
        }
        // the programs, each worker's items contiguous
        const int n_workers = (int)prog_items.size();
        std::vector<int32_t>& sched = b->h_sched;
        sched.assign((size_t)n_workers * 4 + (size_t)total_items * 4, 0);
        int32_t* progs = sched.data();
        int32_t* items = sched.data() + (size_t)n_workers * 4;
        int32_t at = 0;
        for (int w = 0; w < n_workers; w++) {
            progs[w * 4 + 0] = at;
            progs[w * 4 + 1] = (int32_t)prog_items[(size_t)w].size();
            progs[w * 4 + 2] = prog_tail[(size_t)w];
            progs[w * 4 + 3] = affine ? 1 : 0;
            for (int32_t e : prog_items[(size_t)w]) {
                std::copy(entries.begin() + (size_t)e * 4, entries.begin() + (size_t)e * 4 + 4, items + (size_t)at * 4);
                at++;
            }
        }
        b->n_workers = n_workers;
        b->n_items = total_items;
        b->own_rows = affine;
        SR_HIP(ctx, b->d_sched.reserve(sched.size() * sizeof(int32_t), st));
        SR_HIP(ctx, batch_copy(b, staged, b->d_sched.p, sched.data(), sched.size() * sizeof(int32_t), st));
    }
    b->scan_stride = (int64_t)chunks * SR_TK_THREADS * SR_TK_MASK_WORDS;
    b->scan_chunks = chunks;
    b->scan_chunk_vecs = chunk_vecs;
    b->scan_base_addr = base_addr;
    b->scan_stride_bytes = stride_bytes;
    if (rows_changed) {
        b->spec_positions = 0;
        SR_HIP(ctx, batch_copy(b, staged, b->d_rows.p, b->h_rows.data(), b->h_rows.size() * sizeof(SrRow), st));
    }
    SR_HIP(ctx, b->d_scan_desc.reserve(b->h_scan.size() * sizeof(SrScanDesc), st));
    SR_HIP(ctx, batch_copy(b, staged, b->d_scan_desc.p, b->h_scan.data(), b->h_scan.size() * sizeof(SrScanDesc), st));
    SR_HIP(ctx, b->d_scan_mask.reserve(b->h_scan.size() * (size_t)b->scan_stride * sizeof(uint32_t), st));
    SR_HIP(ctx, batch_flush(b, st));
    SR_HIP(ctx, sr_launch_build_scan_mask(b->d_scan_desc.as<SrScanDesc>(), nullptr, (int)b->h_scan.size(), b->d_rows.as<SrRow>(),
                                          b->d_edits.as<SrEdit>(), sr_batch_mask_ptr(b), sr_batch_mask_stride(b),
                                          b->d_scan_mask.as<uint32_t>(), b->scan_stride, b->vocab, epv, chunks, chunk_vecs,
                                          base_addr, stride_bytes, st));
    // the host vectors are read by the async copies above
    if (!staged) SR_HIP(ctx, hipStreamSynchronize(st));
    return SR_OK;
}

}  // namespace

extern "C" {

const char* sr_version(void) { return "0.1.0"; }

int sr_create(int device_ordinal, sr_ctx** out)
{
    if (!out) return SR_ERR_NULL_ARGUMENT;
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0 || device_ordinal < 0 || device_ordinal >= n)
        return SR_ERR_NO_DEVICE;
    sr_ctx* ctx = new (std::nothrow) sr_ctx();
    if (!ctx) return SR_ERR_OUT_OF_MEMORY;
    ctx->device = device_ordinal;
    if (hipSetDevice(device_ordinal) != hipSuccess) { delete ctx; return SR_ERR_NO_DEVICE; }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_ordinal) == hipSuccess) ctx->cu_count = prop.multiProcessorCount;
    if (hipStreamCreateWithFlags(&ctx->own_stream, hipStreamNonBlocking) != hipSuccess) {
        delete ctx;
        return SR_ERR_HIP;
    }
    ctx->stream = ctx->own_stream;
    // where this device keeps its copy of the scratch that belongs to the library's code object
    if (sr_argmax_static_scratch(device_ordinal, &ctx->static_best, &ctx->static_done) != hipSuccess) {
        (void)hipStreamDestroy(ctx->own_stream);
        delete ctx;
        return SR_ERR_HIP;
    }
    *out = ctx;
    return SR_OK;
}

void sr_destroy(sr_ctx* ctx)
{
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->tmp_batch) sr_batch_destroy(ctx->tmp_batch);
    DeviceBuf* bufs[] = {&ctx->cand, &ctx->gmax, &ctx->gmax2, &ctx->gpos, &ctx->gbound, &ctx->row_done, &ctx->argmax_best, &ctx->argmax_done, &ctx->mask_pool, &ctx->mask_any,
                         &ctx->work, &ctx->edit_tab, &ctx->host_logits, &ctx->stage_probs, &ctx->out_tokens, &ctx->out_flags, &ctx->out_val,
                         &ctx->full_state, &ctx->sort_k0, &ctx->sort_v0,
                         &ctx->sort_v1, &ctx->ident, &ctx->redo_list, &ctx->spec_probs, &ctx->spec_resid, &ctx->spec_reject,
                         &ctx->seg_part, &ctx->seg_func, &ctx->full_row_sync, &ctx->full_seg_func, &ctx->full_seg_ms, &ctx->full_watch, &ctx->full_watch_cnt, &ctx->full_seg_keys};
    for (DeviceBuf* b : bufs) b->release();
    ctx->uni_ring.release();
    if (ctx->own_stream) (void)hipStreamDestroy(ctx->own_stream);
    delete ctx;
}

int sr_bind_thread(sr_ctx* ctx)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    SR_HIP(ctx, hipSetDevice(ctx->device));
    return SR_OK;
}

static int switch_stream(sr_ctx* ctx, hipStream_t next)
{
    // uploads of batches may still be running on the stream that is left: later launches are ordered behind them
    // only on the same stream
    if (next != ctx->stream) {
        SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
        ctx->stream_epoch++;  // (pinned rings of the context and its batches: nothing of the old stream reads them any more)
    }
    ctx->stream = next;
    return SR_OK;
}

int sr_set_stream(sr_ctx* ctx, void* hip_stream)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    return switch_stream(ctx, (hipStream_t)hip_stream);  // NULL is HIP's default stream, as everywhere in HIP
}

int sr_use_own_stream(sr_ctx* ctx)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    return switch_stream(ctx, ctx->own_stream);
}

int sr_synchronize(sr_ctx* ctx)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SR_OK;
}

const char* sr_last_error(sr_ctx* ctx) { return ctx ? ctx->err.c_str() : "null context"; }

int sr_batch_create(sr_ctx* ctx, sr_batch** out)
{
    if (!ctx || !out) return SR_ERR_NULL_ARGUMENT;
    sr_batch* b = new (std::nothrow) sr_batch();
    if (!b) return sr_fail(ctx, SR_ERR_OUT_OF_MEMORY, "sr_batch_create: out of host memory");
    b->ctx = ctx;
    *out = b;
    return SR_OK;
}

void sr_batch_destroy(sr_batch* b)
{
    if (!b) return;
    if (b->ctx) (void)hipStreamSynchronize(b->ctx->stream);
    DeviceBuf* bufs[] = {&b->d_rows, &b->d_edits, &b->d_sel_list, &b->d_full_list, &b->d_wide_list, &b->d_scan_desc,
                         &b->d_mask, &b->d_scan_mask, &b->d_uniforms, &b->d_sched, &b->spec_rows};
    for (DeviceBuf* d : bufs) d->release();
    b->stage.release();
    b->patch_ring.release();
    delete b;
}

// sr_batch_upload.  retain: keep what sr_batch_append_tokens needs of the inputs; keep_uniforms: the uniforms on the
// device stay as they are (uniforms is not read).
static int batch_upload_impl(sr_batch* b, int32_t rows, int32_t vocab, const sr_row_params* params,
                             const int32_t* hist_ids, const int32_t* hist_offsets,
                             const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                             const uint32_t* allow_mask, int64_t mask_stride_words, const uint8_t* mask_active,
                             const double* uniforms, int32_t uniforms_per_row, bool retain, bool keep_uniforms,
                             const int32_t* mask_ids = nullptr)
{
    if (!b || !b->ctx) return SR_ERR_NULL_ARGUMENT;
    sr_ctx* ctx = b->ctx;
    if (!params) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_batch_upload: params is null");
    if (rows < 0 || vocab < 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_batch_upload: negative shape");
    if (hist_offsets && !hist_ids && hist_offsets[rows] > hist_offsets[0])
        return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_batch_upload: hist_ids is null");
    if (bias_offsets && (!bias_ids || !bias_vals) && bias_offsets[rows] > bias_offsets[0])
        return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_batch_upload: bias arrays are null");
    if (allow_mask && mask_stride_words < (vocab + 31) / 32)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_batch_upload: mask stride shorter than ceil(vocab/32)");
    if (uniforms_per_row < 0 || (uniforms_per_row > 0 && !uniforms && !keep_uniforms))
        return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_batch_upload: uniforms is null");
    if (mask_ids) {
        if (allow_mask) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_batch_upload: allow-masks and mask ids are exclusive");
        for (int32_t r = 0; r < rows; r++) {
            const int32_t id = mask_ids[r];
            if (id < -1 || (id >= 0 && (id >= ctx->pool_cap || !ctx->pool_used[(size_t)id])))
                return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_batch_upload_mask_ids: row " + std::to_string(r) + " names mask " +
                                                                 std::to_string(id) + ", which is not registered");
            if (id >= 0 && ctx->pool_vocab != vocab)
                return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_batch_upload_mask_ids: the masks were registered for another vocabulary size");
        }
    }
    SR_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    SR_HIP(ctx, b->stage.begin());  // (waits for the copies of this batch's previous upload)
    b->segs.clear();
    b->upload_must_wait = false;

    b->rows = rows;
    b->vocab = vocab;
    b->upr = uniforms_per_row;
    b->h_rows.assign((size_t)rows, SrRow{});
    b->h_edits.clear();
    b->h_sel_list.clear();
    b->h_full_list.clear();
    b->h_wide_list.clear();
    b->h_scan.clear();
    b->h_scan_need.assign((size_t)rows, 0u);
    b->scan_epv = 0;
    b->has_mask = allow_mask != nullptr || mask_ids != nullptr;
    b->mask_stride = allow_mask ? mask_stride_words : 0;
    b->mask_ids = mask_ids != nullptr;
    if (mask_ids) b->keep_mask_ids.assign(mask_ids, mask_ids + rows); else b->keep_mask_ids.clear();
    b->keep_mask_gen.assign(mask_ids ? (size_t)rows : 0, 0u);
    b->mask_pool_gen = ctx->pool_gen;
    if (mask_ids)
        for (int32_t r = 0; r < rows; r++)
            if (mask_ids[r] >= 0) b->keep_mask_gen[(size_t)r] = ctx->pool_slot_gen[(size_t)mask_ids[r]];
    b->max_sel = 0;
    b->edit_cap.assign((size_t)rows, 0);
    b->sel_cap.assign((size_t)rows, 0);
    b->edit_ids.clear();
    if (retain) {
        b->can_append = allow_mask == nullptr;
        b->hist_split = false;
        b->keep_hist.clear();
        if (b->can_append) {
            b->keep_params.assign(params, params + rows);
            const int32_t n_hist = hist_offsets ? hist_offsets[rows] : 0, n_bias = bias_offsets ? bias_offsets[rows] : 0;
            b->keep_hist_off.assign((size_t)rows + 1, 0);
            if (hist_offsets) b->keep_hist_off.assign(hist_offsets, hist_offsets + rows + 1);
            b->keep_hist_ids.clear();
            if (n_hist > 0) b->keep_hist_ids.assign(hist_ids, hist_ids + n_hist);
            b->keep_bias_off.clear();
            b->keep_bias_ids.clear();
            b->keep_bias_vals.clear();
            if (bias_offsets) {
                b->keep_bias_off.assign(bias_offsets, bias_offsets + rows + 1);
                if (n_bias > 0) {
                    b->keep_bias_ids.assign(bias_ids, bias_ids + n_bias);
                    b->keep_bias_vals.assign(bias_vals, bias_vals + n_bias);
                }
            }
        }
    }

    std::vector<int32_t> slots;  // scratch of the history de-duplication
    for (int32_t r = 0; r < rows; r++) {
        const sr_row_params& p = params[r];
        SrRow& d = b->h_rows[(size_t)r];
        const int32_t h0 = hist_offsets ? hist_offsets[r] : 0, h1 = hist_offsets ? hist_offsets[r + 1] : 0;
        const int32_t n_prev = std::max(0, h1 - h0);
        const int32_t* prev = hist_ids ? hist_ids + h0 : nullptr;
        const int32_t b0 = bias_offsets ? bias_offsets[r] : 0, b1 = bias_offsets ? bias_offsets[r + 1] : 0;
        const int32_t n_bias = std::max(0, b1 - b0);
        const bool has_bias = n_bias > 0 || (p.flags & SR_ROW_HAS_LOGIT_BIAS);
        const bool hist_pen = has_history_penalty(p);
        const bool has_penalty = n_prev > 0 && hist_pen;

        d.temperature = p.temperature;
        d.top_p = p.top_p;
        d.min_p = p.min_p;
        d.rep = p.repetition_penalty;
        d.presence = p.presence_penalty;
        d.frequency = p.frequency_penalty;
        d.p_min = p.spec_draft_p_min;
        d.top_k = p.top_k;
        d.n_prev = n_prev;
        d.flags = (p.flags & 0xffu) | (has_bias ? (uint32_t)SR_ROW_HAS_LOGIT_BIAS : 0u) |
                  (has_penalty ? SR_ROWFLAG_HAS_PENALTY : 0u);
        d.mask_row = mask_ids ? mask_ids[r] : (allow_mask && (!mask_active || mask_active[r])) ? r : -1;
        d.edit_off = (int32_t)b->h_edits.size();
        d.edit_cnt = 0;
        d.scan_row = -1;
        d.sel = 1;

        // Sampler.Sample dispatch (Sampler.cs:19-39)
        if (p.temperature <= 0.0f) {
            d.path = has_penalty ? SR_PATH_GREEDY_PEN : SR_PATH_GREEDY;
        } else if (p.top_k > 0 && p.top_k < vocab && !has_bias) {
            d.path = SR_PATH_TOPK;
            int64_t sel = (int64_t)p.top_k + (has_penalty ? n_prev : 0);
            d.sel = (int32_t)std::min<int64_t>(sel, vocab);
        } else {
            d.path = SR_PATH_FULL;
        }
        const bool greedy = p.temperature <= 0.0f;
        const bool want_hist = has_penalty;
        const bool want_bias = n_bias > 0 && !greedy;  // LogitBias is ignored by the greedy paths
        if (want_hist || want_bias) {
            // occurrence counts of every in-range id (whole history and trailing repetition window), one edit per
            // distinct id in order of first appearance: an open-addressing table over the row's edits
            std::vector<SrEdit>& ed = b->h_edits;
            if (want_hist) {
                const int32_t ws = (p.repeat_last_n <= 0 || p.repeat_last_n >= n_prev) ? 0 : n_prev - p.repeat_last_n;
                size_t cap = 16;
                while (cap < 2 * (size_t)n_prev) cap <<= 1;
                slots.assign(cap, 0);  // 1 + index of the id's edit, 0 = free
                for (int32_t i = 0; i < n_prev; i++) {
                    const int32_t id = prev[i];
                    if ((uint32_t)id >= (uint32_t)vocab) continue;
                    size_t h = ((uint32_t)id * 2654435761u) & (cap - 1);
                    while (slots[h] != 0 && ed[(size_t)slots[h] - 1].id != id) h = (h + 1) & (cap - 1);
                    if (slots[h] == 0) {
                        SrEdit e{};
                        e.id = id;
                        e.pen = 1.0f;
                        ed.push_back(e);
                        slots[h] = (int32_t)ed.size();
                    }
                    SrEdit& e = ed[(size_t)slots[h] - 1];
                    e.occ_all++;
                    if (i >= ws) e.occ_win++;
                }
                if (p.repetition_penalty != 1.0f) {
                    // powf(repetition_penalty, occurrences in the window): the same few exponents over and over
                    float pow_of[9];
                    bool pow_known[9] = {false, false, false, false, false, false, false, false, false};
                    for (size_t i = (size_t)d.edit_off; i < ed.size(); i++) {
                        const int32_t win = ed[i].occ_win;
                        if (win <= 0) continue;
                        if (win < 9) {
                            if (!pow_known[win]) { pow_of[win] = powf(p.repetition_penalty, (float)win); pow_known[win] = true; }
                            ed[i].pen = pow_of[win];
                        } else {
                            ed[i].pen = powf(p.repetition_penalty, (float)win);
                        }
                    }
                }
            }
            // sorted by id where something searches them: the bias merge below, the rows whose penalties may raise a
            // logit (the row tail looks candidates up) and the rows of the sort-based path
            const bool lowering_only = p.repetition_penalty >= 1.0f && p.presence_penalty >= 0.0f && p.frequency_penalty >= 0.0f;
            const bool searched = want_bias || (d.path == SR_PATH_TOPK && !lowering_only) ||
                                  (d.path == SR_PATH_TOPK && (int64_t)p.top_k + (int64_t)(ed.size() - (size_t)d.edit_off) > SR_TK_SEL_MAX) ||
                                  ed.size() - (size_t)d.edit_off > (size_t)SR_TK_SEL_MAX;
            if (searched) {
                std::sort(ed.begin() + d.edit_off, ed.end(), [](const SrEdit& x, const SrEdit& y) { return x.id < y.id; });
                d.flags |= SR_ROWFLAG_EDITS_SORTED;
            }
            if (want_bias) {
                for (int32_t i = b0; i < b1; i++) {
                    int32_t id = bias_ids[i];
                    if ((uint32_t)id >= (uint32_t)vocab) continue;
                    auto first = ed.begin() + d.edit_off;
                    auto it = std::lower_bound(first, ed.end(), id, [](const SrEdit& e, int32_t v) { return e.id < v; });
                    if (it == ed.end() || it->id != id) {
                        SrEdit e{};
                        e.id = id;
                        e.pen = 1.0f;
                        it = ed.insert(it, e);
                    }
                    it->bias = it->has_bias ? it->bias + bias_vals[i] : bias_vals[i];
                    it->has_bias = 1u;
                }
            }
            d.edit_cnt = (int32_t)ed.size() - d.edit_off;
            b->edit_cap[(size_t)r] = d.edit_cnt;
            if (want_hist && d.edit_cnt > 0) {
                // room for the ids that appended tokens bring: a fixed minimum, and half as much again as the row has
                // (a batch that was rebuilt because a row ran out of room is not rebuilt again soon)
                const int32_t slack = std::max(SR_EDIT_SLACK, d.edit_cnt / 2);
                ed.resize(ed.size() + (size_t)slack);
                b->edit_cap[(size_t)r] += slack;
            }
        }
        // Penalties that can only lower a logit (Sampler.cs:281-286 with repetition >= 1, presence >= 0 and
        // frequency >= 0) cannot lift a history token past a token outside the history: the scan then skips
        // the history ids and asks for the k best of the rest, and the row tail fetches the history logits by
        // id.  GreedyWithHistoryPenalties changes history ids only, whatever the sign.  Penalties that may
        // raise a logit keep the reference's over-selection by the history length (Sampler.cs:224-225).
        const bool lowering = p.repetition_penalty >= 1.0f && p.presence_penalty >= 0.0f && p.frequency_penalty >= 0.0f;
        if (d.path == SR_PATH_TOPK) {
            // The selection kernel's row tail sorts up to SR_TK_SEL_MAX entries: the k best outside the history plus
            // the history ids (lowering penalties), or the k + history-length best (penalties that may raise).
            const bool excl = has_penalty && d.edit_cnt > 0 && lowering;
            const int64_t need = excl ? (int64_t)p.top_k + d.edit_cnt : (d.edit_cnt == 0 ? (int64_t)p.top_k : (int64_t)d.sel);
            if (need > SR_TK_SEL_MAX || d.edit_cnt > SR_TK_SEL_MAX) d.path = SR_PATH_TOPK_WIDE;  // d.sel stays k + history length
        }
        if (has_penalty && d.edit_cnt > 0 &&
            (d.path == SR_PATH_GREEDY_PEN || (d.path == SR_PATH_TOPK && lowering))) {
            d.flags |= SR_ROWFLAG_HIST_EXCL;
            b->h_scan_need[(size_t)r] |= SR_SCAN_HIST;
            d.sel = d.path == SR_PATH_TOPK ? p.top_k : 1;
        } else if (d.path == SR_PATH_TOPK && d.edit_cnt == 0) {
            d.sel = p.top_k;  // no history id inside the vocabulary: nothing is ever penalised
        }
        // A row that over-selects by its history length asks for one more with every appended token: the chunk items
        // of the launch (which carry sel for the waves' shares of the bound) are written for a little more, so that
        // appended tokens need no new items; any value with that many group maxima above it is a bound for less too.
        b->sel_cap[(size_t)r] = d.sel;
        if (d.path == SR_PATH_TOPK && has_penalty && d.edit_cnt > 0 && !lowering)
            b->sel_cap[(size_t)r] = (int32_t)std::min<int64_t>((int64_t)d.sel + (b->edit_cap[(size_t)r] - d.edit_cnt), vocab);
        if (d.path == SR_PATH_TOPK_WIDE) {
            b->h_wide_list.push_back(r);
        } else if (d.path != SR_PATH_FULL) {
            // (with registered masks every row gets a scan-mask row of its own: its mask may come, go and change in place)
            if (d.mask_row >= 0 || mask_ids) b->h_scan_need[(size_t)r] |= SR_SCAN_ALLOW;
            b->h_sel_list.push_back(r);
            b->max_sel = std::max(b->max_sel, d.sel);
        } else {
            b->h_full_list.push_back(r);
        }
    }

    // Rows with the longest tails (largest top_k + history) go first, so that their sequential tails
    // overlap the streaming of the rows behind them and only short tails are left at the end.
    std::stable_sort(b->h_sel_list.begin(), b->h_sel_list.end(), [&](int32_t x, int32_t y) {
        return b->h_rows[(size_t)x].sel > b->h_rows[(size_t)y].sel;
    });

    auto up = [&](DeviceBuf& dst, const void* src, size_t bytes) -> hipError_t {
        if (bytes == 0) return hipSuccess;
        hipError_t e = dst.reserve(bytes, st);
        if (e != hipSuccess) return e;
        return batch_copy(b, true, dst.p, src, bytes, st);
    };
    b->spec_positions = 0;
    SR_HIP(ctx, up(b->d_rows, b->h_rows.data(), b->h_rows.size() * sizeof(SrRow)));
    // (the edit lists of a batch that tokens are appended to grow with every rebuild: room for four times their size, so
    // that a rebuild finds its device memory in place)
    if (b->can_append && b->d_edits.cap < b->h_edits.size() * sizeof(SrEdit))
        SR_HIP(ctx, b->d_edits.reserve(4 * b->h_edits.size() * sizeof(SrEdit), st));
    SR_HIP(ctx, up(b->d_edits, b->h_edits.data(), b->h_edits.size() * sizeof(SrEdit)));
    SR_HIP(ctx, up(b->d_sel_list, b->h_sel_list.data(), b->h_sel_list.size() * sizeof(int32_t)));
    SR_HIP(ctx, up(b->d_full_list, b->h_full_list.data(), b->h_full_list.size() * sizeof(int32_t)));
    SR_HIP(ctx, up(b->d_wide_list, b->h_wide_list.data(), b->h_wide_list.size() * sizeof(int32_t)));
    if (allow_mask) {  // large: straight from the caller's memory, which the wait at the end covers
        const size_t bytes = (size_t)rows * (size_t)mask_stride_words * sizeof(uint32_t);
        SR_HIP(ctx, b->d_mask.reserve(bytes, st));
        SR_HIP(ctx, batch_copy(b, false, b->d_mask.p, allow_mask, bytes, st));
    }
    if (uniforms_per_row > 0 && !keep_uniforms)
        SR_HIP(ctx, up(b->d_uniforms, uniforms, (size_t)rows * (size_t)uniforms_per_row * sizeof(double)));
    // scan masks for the layout of the last launch (16-byte aligned rows); a launch with another layout rebuilds
    if (!b->h_sel_list.empty()) {
        const int epv = ctx->last_epv;
        int rc = prepare_scan(b, epv, 0ull, 0ll, true);
        if (rc != SR_OK) return rc;
    }
    // Everything small went through the batch's pinned memory: the copies and the scan-mask kernel run on while
    // the caller goes on (launches on this stream are ordered behind them).  Pageable memory that a copy reads
    // directly (the caller's allow-mask; anything the pinned memory had no room for yet) must be waited for.
    SR_HIP(ctx, batch_flush(b, st));
    if (b->upload_must_wait) SR_HIP(ctx, hipStreamSynchronize(st));
    SR_HIP(ctx, b->stage.end(st));
    return SR_OK;
}

int sr_batch_upload(sr_batch* b, int32_t rows, int32_t vocab, const sr_row_params* params,
                    const int32_t* hist_ids, const int32_t* hist_offsets,
                    const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                    const uint32_t* allow_mask, int64_t mask_stride_words, const uint8_t* mask_active,
                    const double* uniforms, int32_t uniforms_per_row)
{
    return batch_upload_impl(b, rows, vocab, params, hist_ids, hist_offsets, bias_ids, bias_vals, bias_offsets, allow_mask,
                             mask_stride_words, mask_active, uniforms, uniforms_per_row, true, false);
}

// The batch as sr_batch_upload would build it for the histories as they are now (rows the in-place update does not
// cover: a first history token, sorted edit lists, an edit range without room, a change of path).
static int append_rebuild(sr_batch* b, const double* uniforms)
{
    const int32_t rows = b->rows;
    std::vector<sr_row_params> params = b->keep_params;
    std::vector<int32_t> ids, off((size_t)rows + 1, 0);
    for (int32_t r = 0; r < rows; r++) {
        ids.insert(ids.end(), b->keep_hist[(size_t)r].begin(), b->keep_hist[(size_t)r].end());
        off[(size_t)r + 1] = (int32_t)ids.size();
    }
    const std::vector<int32_t> bias_ids = b->keep_bias_ids, bias_off = b->keep_bias_off;
    const std::vector<float> bias_vals = b->keep_bias_vals;
    const std::vector<int32_t> mids = b->keep_mask_ids;
    return batch_upload_impl(b, rows, b->vocab, params.data(), ids.data(), off.data(),
                             bias_off.empty() ? nullptr : bias_ids.data(), bias_off.empty() ? nullptr : bias_vals.data(),
                             bias_off.empty() ? nullptr : bias_off.data(), nullptr, 0, nullptr, uniforms, b->upr, false,
                             uniforms == nullptr, b->mask_ids ? mids.data() : nullptr);
}

static int append_impl(sr_batch* b, const int32_t* tokens, const double* uniforms, const int32_t* new_mask_ids)
{
    if (!b || !b->ctx) return SR_ERR_NULL_ARGUMENT;
    sr_ctx* ctx = b->ctx;
    if (!tokens) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_batch_append_tokens: tokens is null");
    if (!b->can_append)
        return sr_fail(ctx, SR_ERR_UNSUPPORTED, "sr_batch_append_tokens: the batch was not uploaded, or was uploaded with "
                                                "allow-masks of its own (register the masks and upload their ids, or "
                                                "upload it again with the new masks)");
    if (new_mask_ids && !b->mask_ids)
        return sr_fail(ctx, SR_ERR_UNSUPPORTED, "sr_batch_append_tokens_masks: the batch was not uploaded with mask ids");
    const int32_t rows = b->rows, vocab = b->vocab;
    if (rows == 0) return SR_OK;
    std::vector<int32_t> scan_again;  // scan-mask rows whose allow-mask changes
    bool names_mask = false;
    for (int32_t r = 0; new_mask_ids && r < b->rows && !names_mask; r++) names_mask = b->keep_mask_ids[(size_t)r] >= 0;
    if (new_mask_ids && !names_mask) b->mask_pool_gen = ctx->pool_gen;  // no row held an id of an older pool
    if (new_mask_ids && b->mask_pool_gen != ctx->pool_gen)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_batch_append_tokens_masks: the registered masks were started again for another "
                                                         "vocabulary since the batch was uploaded; upload the batch again");
    if (new_mask_ids) {
        for (int32_t r = 0; r < rows; r++) {
            const int32_t id = new_mask_ids[r];
            if (id < -1 || (id >= 0 && (id >= ctx->pool_cap || !ctx->pool_used[(size_t)id] || ctx->pool_vocab != vocab)))
                return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_batch_append_tokens_masks: row " + std::to_string(r) +
                                                                 " names mask " + std::to_string(id) + ", which is not registered");
        }
    }
    if (!b->hist_split) {
        b->keep_hist.assign((size_t)rows, std::vector<int32_t>());
        for (int32_t r = 0; r < rows; r++) {
            const int32_t h0 = b->keep_hist_off[(size_t)r], h1 = b->keep_hist_off[(size_t)r + 1];
            if (h1 > h0) b->keep_hist[(size_t)r].assign(b->keep_hist_ids.begin() + h0, b->keep_hist_ids.begin() + h1);
        }
        b->hist_split = true;
    }
    for (int32_t r = 0; r < rows; r++)
        if (tokens[r] >= 0) b->keep_hist[(size_t)r].push_back(tokens[r]);

    // In place: one token more in the history of a row changes the occurrence counts of at most two ids (the one that
    // enters, the one that leaves the repetition window, Sampler.cs:272-279) and may add one id.
    if (b->edit_ids.size() != b->h_edits.size()) {
        b->edit_ids.resize(b->h_edits.size());
        for (size_t i = 0; i < b->h_edits.size(); i++) b->edit_ids[i] = b->h_edits[i].id;
    }
    // powf(repetition_penalty, occurrences): rows mostly share the penalty, and the counts are small
    float pow_rep = 1.0f, pow_of[16];
    bool pow_known[16] = {};
    auto pow_cached = [&](float rep, int32_t occ) -> float {
        if (occ >= 16) return powf(rep, (float)occ);
        if (rep != pow_rep) {
            pow_rep = rep;
            for (bool& k : pow_known) k = false;
        }
        if (!pow_known[occ]) {
            pow_of[occ] = powf(rep, (float)occ);
            pow_known[occ] = true;
        }
        return pow_of[occ];
    };
    std::vector<SrRowPatch> rp;
    std::vector<SrEditPatch> ep;
    std::vector<SrMaskClear> mc;
    std::vector<int32_t> touched;
    // (a call that failed after it had changed the host's copies left them ahead of the device: rebuild from the inputs)
    bool rebuild = b->host_ahead;
    for (int32_t r = 0; r < rows && !rebuild; r++) {
        SrRow& d = b->h_rows[(size_t)r];
        bool mask_changed = false;
        // (an id that was released and registered again since the row took it names another mask now)
        const uint32_t slot_gen = (new_mask_ids && new_mask_ids[r] >= 0) ? ctx->pool_slot_gen[(size_t)new_mask_ids[r]] : 0u;
        if (new_mask_ids && (new_mask_ids[r] != d.mask_row || slot_gen != b->keep_mask_gen[(size_t)r])) {
            d.mask_row = new_mask_ids[r];
            b->keep_mask_ids[(size_t)r] = new_mask_ids[r];
            b->keep_mask_gen[(size_t)r] = slot_gen;
            mask_changed = true;
            if (d.scan_row >= 0 && (b->h_scan_need[(size_t)r] & SR_SCAN_ALLOW)) scan_again.push_back(d.scan_row);
        }
        if (tokens[r] < 0) {
            if (mask_changed) rp.push_back(SrRowPatch{r, d.n_prev, d.edit_cnt, d.mask_row, d.sel, d.edit_off});
            continue;
        }
        const sr_row_params& p = b->keep_params[(size_t)r];
        const std::vector<int32_t>& hist = b->keep_hist[(size_t)r];
        const int32_t n_new = (int32_t)hist.size(), n_old = n_new - 1;
        if (!has_history_penalty(p)) {  // the history is never looked at
            d.n_prev = n_new;
            rp.push_back(SrRowPatch{r, d.n_prev, d.edit_cnt, d.mask_row, d.sel, d.edit_off});
            continue;
        }
        if (n_old == 0 || d.edit_cnt == 0 || d.path == SR_PATH_TOPK_WIDE) {
            rebuild = true;
            break;
        }
        const bool sorted = (d.flags & SR_ROWFLAG_EDITS_SORTED) != 0u;
        // a row that over-selects by its history length (penalties that may raise a logit, Sampler.cs:224-225)
        const bool literal = d.path == SR_PATH_TOPK && (d.flags & SR_ROWFLAG_HIST_EXCL) == 0u;
        SrEdit* ed = b->h_edits.data() + d.edit_off;
        int32_t* eids = b->edit_ids.data() + d.edit_off;
        auto find = [&](int32_t id) -> int32_t {
            const int32_t* f = std::find(eids, eids + d.edit_cnt, id);
            return f == eids + d.edit_cnt ? -1 : (int32_t)(f - eids);
        };
        auto repow = [&](SrEdit& e) {
            e.pen = (p.repetition_penalty != 1.0f && e.occ_win > 0) ? pow_cached(p.repetition_penalty, e.occ_win) : 1.0f;
        };
        touched.clear();
        const int32_t rl = p.repeat_last_n;
        const int32_t ws_old = (rl <= 0 || rl >= n_old) ? 0 : n_old - rl, ws_new = (rl <= 0 || rl >= n_new) ? 0 : n_new - rl;
        for (int32_t i = ws_old; i < ws_new; i++) {  // leaves the window
            const int32_t id = hist[(size_t)i];
            if ((uint32_t)id >= (uint32_t)vocab) continue;
            const int32_t k = find(id);
            if (k < 0) { rebuild = true; break; }
            ed[k].occ_win--;
            repow(ed[k]);
            touched.push_back(k);
        }
        if (rebuild) break;
        const int32_t t = tokens[r];
        if ((uint32_t)t < (uint32_t)vocab) {
            int32_t k = find(t);
            if (k < 0) {
                const bool topk = d.path == SR_PATH_TOPK;
                if (d.edit_cnt + 1 > SR_TK_SEL_MAX || (topk && (int64_t)p.top_k + d.edit_cnt + 1 > SR_TK_SEL_MAX)) {
                    rebuild = true;  // (the row leaves the selection kernel's limits: another path)
                    break;
                }
                if (d.edit_cnt >= b->edit_cap[(size_t)r]) {
                    // No room behind the row's edits: the row moves to the end of the array, with room for as many again,
                    // and all its edits are sent -- a patch like any other.  Only when the device array itself has no room
                    // left (it was made for four times what the upload needed) is the batch rebuilt, which packs it again.
                    const int32_t new_cap = std::max(2 * b->edit_cap[(size_t)r], d.edit_cnt + SR_EDIT_SLACK);
                    const size_t new_off = b->h_edits.size();
                    if ((new_off + (size_t)new_cap) * sizeof(SrEdit) > b->d_edits.cap || new_off + (size_t)new_cap > 0x7fffffffull) {
                        rebuild = true;
                        break;
                    }
                    b->h_edits.resize(new_off + (size_t)new_cap);
                    b->edit_ids.resize(new_off + (size_t)new_cap, 0);
                    std::copy(b->h_edits.begin() + d.edit_off, b->h_edits.begin() + d.edit_off + d.edit_cnt, b->h_edits.begin() + (ptrdiff_t)new_off);
                    std::copy(b->edit_ids.begin() + d.edit_off, b->edit_ids.begin() + d.edit_off + d.edit_cnt, b->edit_ids.begin() + (ptrdiff_t)new_off);
                    d.edit_off = (int32_t)new_off;
                    b->edit_cap[(size_t)r] = new_cap;
                    ed = b->h_edits.data() + d.edit_off;
                    eids = b->edit_ids.data() + d.edit_off;
                    touched.clear();
                    for (int32_t j = 0; j < d.edit_cnt; j++) touched.push_back(j);
                    b->append_moves++;
                }
                if (sorted) {
                    // the edits stay in order of their ids (a kernel searches them): the new one goes where it
                    // belongs, the ones behind it move up by one and are sent again
                    k = (int32_t)(std::lower_bound(eids, eids + d.edit_cnt, t) - eids);
                    for (int32_t j = d.edit_cnt; j > k; j--) { ed[j] = ed[j - 1]; eids[j] = eids[j - 1]; }
                    for (int32_t& j : touched) j += j >= k ? 1 : 0;
                    d.edit_cnt++;
                    for (int32_t j = k + 1; j < d.edit_cnt; j++) touched.push_back(j);
                } else {
                    k = d.edit_cnt++;
                }
                ed[k] = SrEdit{};
                ed[k].id = t;
                ed[k].pen = 1.0f;
                eids[k] = t;
                if (b->h_scan_need[(size_t)r] & SR_SCAN_HIST) mc.push_back(SrMaskClear{d.scan_row, r, t});
            }
            ed[k].occ_all++;
            ed[k].occ_win++;
            repow(ed[k]);
            touched.push_back(k);
        }
        d.n_prev = n_new;
        if (literal) {
            const int64_t sel = std::min<int64_t>((int64_t)p.top_k + n_new, vocab);
            if (sel > b->sel_cap[(size_t)r] || sel > SR_TK_SEL_MAX) {  // new chunk items, or the sort-based path
                rebuild = true;
                break;
            }
            d.sel = (int32_t)sel;
            b->max_sel = std::max(b->max_sel, d.sel);
        }
        rp.push_back(SrRowPatch{r, d.n_prev, d.edit_cnt, d.mask_row, d.sel, d.edit_off});
        std::sort(touched.begin(), touched.end());
        touched.erase(std::unique(touched.begin(), touched.end()), touched.end());
        for (int32_t k : touched) ep.push_back(SrEditPatch{d.edit_off + k, ed[k]});
    }
    if (rebuild) {
        b->append_rebuilds++;
        if (new_mask_ids) b->keep_mask_ids.assign(new_mask_ids, new_mask_ids + rows);  // (the loop above stopped early)
        b->host_ahead = true;
        const int rc = append_rebuild(b, uniforms);
        if (rc == SR_OK) b->host_ahead = false;
        return rc;
    }

    // One kernel applies everything, reading the lists straight from the batch's pinned memory: no copy calls.
    SR_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    const size_t n_uni = (uniforms && b->upr > 0) ? (size_t)rows * (size_t)b->upr : 0;
    const size_t need = rp.size() * sizeof(SrRowPatch) + ep.size() * sizeof(SrEditPatch) + mc.size() * sizeof(SrMaskClear) +
                        n_uni * sizeof(double) + scan_again.size() * sizeof(int32_t) + 5 * 256;
    // (a ring that is made now is made for the largest call to come as well: every row of the batch out of room at once,
    // all edits sent again -- rows that were uploaded together run out of room together)
    b->host_ahead = true;  // (until everything below has been enqueued)
    SR_HIP(ctx, b->patch_ring.begin(need, st, b->h_edits.size() * sizeof(SrEditPatch) + (size_t)rows * 64 + n_uni * sizeof(double) + 65536,
                                    ctx->stream_epoch));
    const SrRowPatch* rp_d = (const SrRowPatch*)b->patch_ring.put(rp.data(), rp.size() * sizeof(SrRowPatch));
    const SrEditPatch* ep_d = (const SrEditPatch*)b->patch_ring.put(ep.data(), ep.size() * sizeof(SrEditPatch));
    const SrMaskClear* mc_d = (const SrMaskClear*)b->patch_ring.put(mc.data(), mc.size() * sizeof(SrMaskClear));
    const double* un_d = (const double*)b->patch_ring.put(uniforms, n_uni * sizeof(double));
    const int32_t* sa_d = (const int32_t*)b->patch_ring.put(scan_again.data(), scan_again.size() * sizeof(int32_t));
    if (!rp_d || !ep_d || !mc_d || !un_d || !sa_d) return sr_fail(ctx, SR_ERR_OUT_OF_MEMORY, "sr_batch_append_tokens: no pinned memory");
    // scan masks that are not built yet are built from the patched edits when they are needed
    const bool masks = b->scan_epv != 0 && b->d_scan_mask.p != nullptr;
    b->spec_positions = 0;
    SR_HIP(ctx, sr_launch_apply_patches(b->d_rows.as<SrRow>(), rp_d, (int)rp.size(), b->d_edits.as<SrEdit>(), ep_d,
                                        (int)ep.size(), mc_d, masks ? (int)mc.size() : 0, b->d_scan_mask.as<uint32_t>(),
                                        b->scan_stride, masks ? b->scan_epv : 4, masks ? b->scan_chunk_vecs : 64,
                                        b->scan_base_addr, b->scan_stride_bytes, b->d_uniforms.as<double>(), un_d,
                                        (int)n_uni, st));
    // rows whose allow-mask changed: their scan-mask rows are built again, from the new mask and the patched history
    if (masks && !scan_again.empty())
        SR_HIP(ctx, sr_launch_build_scan_mask(b->d_scan_desc.as<SrScanDesc>(), sa_d, (int)scan_again.size(), b->d_rows.as<SrRow>(),
                                              b->d_edits.as<SrEdit>(), sr_batch_mask_ptr(b), sr_batch_mask_stride(b),
                                              b->d_scan_mask.as<uint32_t>(), b->scan_stride, b->vocab, b->scan_epv,
                                              b->scan_chunks, b->scan_chunk_vecs, b->scan_base_addr, b->scan_stride_bytes, st));
    b->host_ahead = false;
    return SR_OK;
}

int sr_batch_append_tokens(sr_batch* b, const int32_t* tokens, const double* uniforms)
{
    return append_impl(b, tokens, uniforms, nullptr);
}

int sr_batch_append_tokens_masks(sr_batch* b, const int32_t* tokens, const double* uniforms, const int32_t* mask_ids)
{
    if (b && b->ctx && !mask_ids) return sr_fail(b->ctx, SR_ERR_NULL_ARGUMENT, "sr_batch_append_tokens_masks: mask_ids is null");
    return append_impl(b, tokens, uniforms, mask_ids);
}

int sr_batch_upload_mask_ids(sr_batch* b, int32_t rows, int32_t vocab, const sr_row_params* params,
                             const int32_t* hist_ids, const int32_t* hist_offsets,
                             const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                             const int32_t* mask_ids, const double* uniforms, int32_t uniforms_per_row)
{
    if (b && b->ctx && !mask_ids) return sr_fail(b->ctx, SR_ERR_NULL_ARGUMENT, "sr_batch_upload_mask_ids: mask_ids is null");
    return batch_upload_impl(b, rows, vocab, params, hist_ids, hist_offsets, bias_ids, bias_vals, bias_offsets, nullptr, 0,
                             nullptr, uniforms, uniforms_per_row, true, false, mask_ids);
}

// ---- registered allow-masks ---------------------------------------------------------------------------
// A free slot of the pool of registered masks for vocabulary `vocab` (the pool starts again for a new vocabulary
// when no mask is held, and grows when it is full).  The slot is not marked used yet.
static int pool_take_slot(sr_ctx* ctx, int32_t vocab, const char* who, int32_t* out_slot)
{
    hipStream_t st = ctx->stream;
    const bool any_used = std::find(ctx->pool_used.begin(), ctx->pool_used.end(), (uint8_t)1) != ctx->pool_used.end();
    if (any_used && vocab != ctx->pool_vocab)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, std::string(who) + ": a context holds masks of one vocabulary size at a time (" +
                                                         std::to_string(ctx->pool_vocab) + " now); release them first");
    const int32_t nw = (vocab + 31) / 32;
    if (!any_used && vocab != ctx->pool_vocab) {  // a new vocabulary: the pool starts again
        SR_HIP(ctx, hipStreamSynchronize(st));
        ctx->mask_pool.release();
        ctx->pool_cap = 0;
        ctx->pool_used.clear();
        ctx->pool_slot_gen.clear();
        ctx->pool_vocab = vocab;
        ctx->pool_words = (nw + 3) & ~3;  // rows of the pool start on 16 bytes
        ctx->pool_gen++;                  // batches that name masks of the old pool are stale from here on
    }
    int32_t id = -1;
    for (int32_t i = 0; i < ctx->pool_cap; i++)
        if (!ctx->pool_used[(size_t)i]) { id = i; break; }
    if (id < 0) {  // grow: a larger array, the masks moved over on the stream, the old one freed when that is done
        const int32_t cap = std::max(16, ctx->pool_cap * 2);
        void* bigger = nullptr;
        SR_HIP(ctx, hipMalloc(&bigger, (size_t)cap * (size_t)ctx->pool_words * sizeof(uint32_t)));
        if (ctx->pool_cap > 0) {
            hipError_t e = hipMemcpyAsync(bigger, ctx->mask_pool.p, (size_t)ctx->pool_cap * (size_t)ctx->pool_words * sizeof(uint32_t),
                                          hipMemcpyDeviceToDevice, st);
            if (e == hipSuccess) e = hipStreamSynchronize(st);
            if (e != hipSuccess) { (void)hipFree(bigger); return sr_fail_hip(ctx, e, "moving the registered masks"); }
        }
        ctx->mask_pool.release();
        ctx->mask_pool.p = bigger;
        ctx->mask_pool.cap = (size_t)cap * (size_t)ctx->pool_words * sizeof(uint32_t);
        id = ctx->pool_cap;
        ctx->pool_cap = cap;
        ctx->pool_used.resize((size_t)cap, 0);
        ctx->pool_slot_gen.resize((size_t)cap, 0u);
    }
    *out_slot = id;
    return SR_OK;
}

int sr_mask_register(sr_ctx* ctx, const uint32_t* words, int words_on_device, int32_t vocab, int32_t* out_id)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (!words || !out_id) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_mask_register: null argument");
    if (vocab <= 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_mask_register: empty vocabulary");
    *out_id = -1;
    SR_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    int32_t id = -1;
    int rc = pool_take_slot(ctx, vocab, "sr_mask_register", &id);
    if (rc != SR_OK) return rc;
    const int32_t nw = (vocab + 31) / 32;
    uint32_t* dst = ctx->mask_pool.as<uint32_t>() + (size_t)id * (size_t)ctx->pool_words;
    SR_HIP(ctx, hipMemcpyAsync(dst, words, (size_t)nw * sizeof(uint32_t),
                               words_on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, st));
    // the caller's array may be reused when the call returns (a mask is registered once per grammar state, not per step)
    if (!words_on_device) SR_HIP(ctx, hipStreamSynchronize(st));
    ctx->pool_used[(size_t)id] = 1;
    *out_id = id;
    return SR_OK;
}

int sr_mask_and(sr_ctx* ctx, const int32_t* mask_ids, int32_t n, int32_t* out_id)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (!out_id || (!mask_ids && n > 0)) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_mask_and: null argument");
    *out_id = -1;
    if (n < 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_mask_and: negative count");
    int32_t ids[SR_MASK_AND_MAX];
    int32_t m = 0;
    for (int32_t i = 0; i < n; i++) {
        const int32_t id = mask_ids[i];
        if (id == -1) continue;  // an inner constraint in its dead state contributes nothing (AndTokenConstraint.cs:74)
        if (id < -1 || id >= ctx->pool_cap || !ctx->pool_used[(size_t)id])
            return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_mask_and: mask " + std::to_string(id) + " is not registered");
        if (m == SR_MASK_AND_MAX)
            return sr_fail(ctx, SR_ERR_UNSUPPORTED, "sr_mask_and: at most " + std::to_string(SR_MASK_AND_MAX) + " masks per call (combine in steps)");
        ids[m++] = id;
    }
    if (m == 0) return SR_OK;  // nothing constrains: no mask
    SR_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    int32_t slot = -1;
    int rc = pool_take_slot(ctx, ctx->pool_vocab, "sr_mask_and", &slot);
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, ctx->mask_any.reserve(sizeof(uint32_t), st));
    SR_HIP(ctx, hipMemsetAsync(ctx->mask_any.p, 0, sizeof(uint32_t), st));
    SR_HIP(ctx, sr_launch_mask_and(ctx->mask_pool.as<uint32_t>(), ctx->pool_words, ids, m, slot, ctx->pool_vocab,
                                   ctx->mask_any.as<uint32_t>(), st));
    uint32_t any = 0u;
    SR_HIP(ctx, hipMemcpyAsync(&any, ctx->mask_any.p, sizeof(uint32_t), hipMemcpyDeviceToHost, st));
    SR_HIP(ctx, hipStreamSynchronize(st));
    if (!any) return SR_OK;  // dead intersection: never wedge, the row goes unmasked (AndTokenConstraint.cs:80-85); the slot stays free
    ctx->pool_used[(size_t)slot] = 1;
    *out_id = slot;
    return SR_OK;
}

int sr_mask_release(sr_ctx* ctx, int32_t id)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (id < 0 || id >= ctx->pool_cap || !ctx->pool_used[(size_t)id])
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_mask_release: mask " + std::to_string(id) + " is not registered");
    ctx->pool_used[(size_t)id] = 0;
    ctx->pool_slot_gen[(size_t)id]++;  // a batch that still names the id is stale from here on
    return SR_OK;
}

int sr_pack_allow_mask_launch(sr_ctx* ctx, const void* masked_logits_dev, int dtype, int32_t rows, int32_t vocab,
                              int64_t row_stride_elems, uint32_t* out_words_dev, int64_t out_stride_words)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (rows == 0 || vocab == 0) return SR_OK;
    if (!masked_logits_dev || !out_words_dev) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_pack_allow_mask_launch: null tensor");
    if (rows < 0 || vocab < 0 || row_stride_elems < vocab || out_stride_words < (vocab + 31) / 32)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_pack_allow_mask_launch: bad shape");
    if (dtype != SR_DTYPE_F32 && dtype != SR_DTYPE_BF16)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_pack_allow_mask_launch: unknown dtype");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    SR_HIP(ctx, sr_launch_pack_allow_mask(masked_logits_dev, dtype, rows, vocab, row_stride_elems, out_words_dev,
                                          out_stride_words, ctx->stream));
    return SR_OK;
}

int sr_batch_set_uniforms(sr_batch* b, const double* uniforms)
{
    if (!b || !b->ctx) return SR_ERR_NULL_ARGUMENT;
    sr_ctx* ctx = b->ctx;
    if (!uniforms) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_batch_set_uniforms: uniforms is null");
    if (b->upr <= 0 || b->rows <= 0) return SR_OK;
    SR_HIP(ctx, hipSetDevice(ctx->device));
    SR_HIP(ctx, hipMemcpyAsync(b->d_uniforms.p, uniforms, (size_t)b->rows * b->upr * sizeof(double),
                               hipMemcpyHostToDevice, ctx->stream));
    SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SR_OK;
}

int sr_sample_launch(sr_ctx* ctx, const sr_batch* b, const void* logits_dev, int dtype, int64_t row_stride_elems,
                     int32_t* out_tokens_dev, uint32_t* out_flags_dev)
{
    if (!ctx || !b) return SR_ERR_NULL_ARGUMENT;
    if (b->rows == 0) return SR_OK;
    if (!logits_dev || !out_tokens_dev) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_sample_launch: null tensor");
    if (dtype != SR_DTYPE_F32 && dtype != SR_DTYPE_BF16)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_sample_launch: unknown dtype");
    if (row_stride_elems < b->vocab) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_sample_launch: row stride < vocab");
    if (b->vocab <= 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_sample_launch: empty vocabulary");
    if (int rc = sr_batch_masks_valid(ctx, b, "sr_sample_launch")) return rc;
    for (const SrRow& r : b->h_rows)
        if (r.path != SR_PATH_GREEDY && r.path != SR_PATH_GREEDY_PEN && b->upr < 1)
            return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_sample_launch: a sampled row needs a uniform");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;

    const int n_sel = (int)b->h_sel_list.size();
    if (n_sel > 0) {
        SrTopkArgs a{};
        a.logits = logits_dev;
        a.row_stride = row_stride_elems;
        a.vocab = b->vocab;
        a.dtype = dtype;
        a.n_rows = n_sel;
        const int epv = dtype == SR_DTYPE_BF16 ? 8 : 4;
        ctx->last_epv = epv;
        int rc = prepare_scan(const_cast<sr_batch*>(b), epv, (unsigned long long)(uintptr_t)logits_dev,
                              (long long)row_stride_elems * (dtype == SR_DTYPE_BF16 ? 2 : 4));
        if (rc != SR_OK) return rc;
        topk_geometry(b->vocab, dtype, n_sel, ctx->cu_count, &a.chunks, &a.chunk_vecs);
        if (a.chunks > SR_TK_MAX_CHUNKS)
            return sr_fail(ctx, SR_ERR_UNSUPPORTED, "sr_sample_launch: vocabulary too large for the selection kernel");
        a.progs = b->d_sched.as<int4>();
        a.items = b->d_sched.as<int4>() + b->n_workers;
        a.n_workers = b->n_workers;
        a.cu_count = ctx->cu_count;
        a.own_rows = b->own_rows ? 1 : 0;
        a.kept = (b->own_rows && b->n_workers <= ctx->cu_count) ? 1 : 0;
        a.short_lists = b->max_sel <= SR_TK_SHORT_SEL ? 1 : 0;
        a.n_items = b->n_items;
        a.sel_list = b->d_sel_list.as<int32_t>();
        SR_HIP(ctx, ctx->cand.reserve((size_t)n_sel * SR_TK_ROW_CAP * sizeof(unsigned long long), st));
        SR_HIP(ctx, ctx->gmax.reserve((size_t)n_sel * a.chunks * SR_TK_THREADS * 4 * sizeof(float), st));
        SR_HIP(ctx, ctx->gmax2.reserve((size_t)n_sel * a.chunks * SR_TK_THREADS * 4 * sizeof(float), st));
        SR_HIP(ctx, ctx->gpos.reserve((size_t)n_sel * a.chunks * SR_TK_THREADS * sizeof(uint32_t), st));
        SR_HIP(ctx, ctx->gbound.reserve((size_t)n_sel * a.chunks * (SR_TK_THREADS / 64) * 2 * sizeof(uint32_t), st));
        // two sets of counters (see SrTopkArgs); a new allocation starts zeroed
        if ((size_t)n_sel > ctx->done_cap || !ctx->row_done.p) {
            const size_t cap = std::max((size_t)n_sel, (size_t)1024);
            SR_HIP(ctx, ctx->row_done.reserve(2 * cap * sizeof(uint32_t), st, true));
            ctx->done_cap = cap;
            ctx->launch_no = 0;
        }
        a.rows = b->d_rows.as<SrRow>();
        a.edits = b->d_edits.as<SrEdit>();
        a.mask = sr_batch_mask_ptr(b);
        a.mask_stride = sr_batch_mask_stride(b);
        a.scan_mask = b->d_scan_mask.as<uint32_t>();
        a.scan_stride = b->scan_stride;
        a.cand = ctx->cand.as<unsigned long long>();
        a.gmax = ctx->gmax.as<float4>();
        a.gmax2 = ctx->gmax2.as<float4>();
        a.gpos = ctx->gpos.as<uint32_t>();
        a.gbound = ctx->gbound.as<uint32_t>();
        a.row_done = ctx->row_done.as<uint32_t>();
        a.done_cap = (uint32_t)ctx->done_cap;
        a.parity = (uint32_t)(ctx->launch_no++ & 1u);
        a.spin_limit = ctx->spin_limit;
        a.uniforms = b->d_uniforms.as<double>();
        a.uniforms_per_row = b->upr;
        a.out_tokens = out_tokens_dev;
        a.out_flags = out_flags_dev;
        a.prof = ctx->prof;
        SR_HIP(ctx, sr_launch_topk(a, n_sel, st));
    }
    if (!b->h_full_list.empty()) {
        int rc = sr_full_rows_launch(ctx, b, logits_dev, dtype, row_stride_elems, out_tokens_dev, out_flags_dev);
        if (rc != SR_OK) return rc;
    }
    if (!b->h_wide_list.empty()) {
        int rc = sr_wide_rows_launch(ctx, b, b->d_wide_list.as<int32_t>(), (int)b->h_wide_list.size(), logits_dev, dtype,
                                     row_stride_elems, out_tokens_dev, out_flags_dev);
        if (rc != SR_OK) return rc;
    }
    return SR_OK;
}

int sr_resample_rows_launch(sr_ctx* ctx, const sr_batch* b, const void* logits_dev, int dtype, int64_t row_stride_elems,
                            const int32_t* rows_host, int32_t n_rows, int32_t* out_tokens_dev, uint32_t* out_flags_dev)
{
    if (!ctx || !b) return SR_ERR_NULL_ARGUMENT;
    if (n_rows == 0) return SR_OK;
    if (!logits_dev || !out_tokens_dev || !rows_host)
        return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_resample_rows_launch: null argument");
    if (n_rows < 0 || (dtype != SR_DTYPE_F32 && dtype != SR_DTYPE_BF16) || row_stride_elems < b->vocab)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_resample_rows_launch: bad shape or dtype");
    for (int32_t i = 0; i < n_rows; i++) {
        const int32_t r = rows_host[i];
        if (r < 0 || r >= b->rows) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_resample_rows_launch: row out of range");
        const int32_t path = b->h_rows[(size_t)r].path;
        if (path != SR_PATH_TOPK && path != SR_PATH_TOPK_WIDE)
            return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_resample_rows_launch: not a SampleTopK row");
    }
    if (b->upr < 1) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_resample_rows_launch: a sampled row needs a uniform");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    SR_HIP(ctx, ctx->redo_list.reserve((size_t)n_rows * sizeof(int32_t), ctx->stream));
    SR_HIP(ctx, hipMemcpyAsync(ctx->redo_list.p, rows_host, (size_t)n_rows * sizeof(int32_t), hipMemcpyHostToDevice, ctx->stream));
    SR_HIP(ctx, hipStreamSynchronize(ctx->stream));  // the host array may go away
    return sr_wide_rows_launch(ctx, b, ctx->redo_list.as<int32_t>(), n_rows, logits_dev, dtype, row_stride_elems,
                               out_tokens_dev, out_flags_dev);
}

static int stage_logits(sr_ctx* ctx, const void* logits, int dtype, int on_device, int32_t rows, int32_t vocab,
                        int64_t stride, const void** dev)
{
    if (on_device) { *dev = logits; return SR_OK; }
    const size_t es = dtype == SR_DTYPE_BF16 ? 2 : 4;
    const size_t bytes = ((size_t)(rows - 1) * (size_t)stride + (size_t)vocab) * es;
    SR_HIP(ctx, ctx->host_logits.reserve(bytes, ctx->stream));
    SR_HIP(ctx, hipMemcpyAsync(ctx->host_logits.p, logits, bytes, hipMemcpyHostToDevice, ctx->stream));
    *dev = ctx->host_logits.p;
    return SR_OK;
}

int sr_sample_batch(sr_ctx* ctx, const void* logits, int dtype, int logits_on_device, int32_t rows, int32_t vocab,
                    int64_t row_stride_elems, const sr_row_params* params,
                    const int32_t* hist_ids, const int32_t* hist_offsets,
                    const int32_t* bias_ids, const float* bias_vals, const int32_t* bias_offsets,
                    const uint32_t* allow_mask, int64_t mask_stride_words, const uint8_t* mask_active,
                    const double* uniforms, int32_t* out_tokens, uint32_t* out_flags)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (rows == 0) return SR_OK;
    if (!logits || !out_tokens || !params) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_sample_batch: null argument");
    if (rows < 0 || vocab <= 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_sample_batch: bad shape");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    if (!ctx->tmp_batch) {
        int rc = sr_batch_create(ctx, &ctx->tmp_batch);
        if (rc != SR_OK) return rc;
    }
    int rc = sr_batch_upload(ctx->tmp_batch, rows, vocab, params, hist_ids, hist_offsets, bias_ids, bias_vals,
                             bias_offsets, allow_mask, mask_stride_words, mask_active, uniforms, uniforms ? 1 : 0);
    if (rc != SR_OK) return rc;
    const void* dev = nullptr;
    rc = stage_logits(ctx, logits, dtype, logits_on_device, rows, vocab, row_stride_elems, &dev);
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, ctx->out_tokens.reserve((size_t)rows * sizeof(int32_t), ctx->stream));
    SR_HIP(ctx, ctx->out_flags.reserve((size_t)rows * sizeof(uint32_t), ctx->stream));
    rc = sr_sample_launch(ctx, ctx->tmp_batch, dev, dtype, row_stride_elems, ctx->out_tokens.as<int32_t>(),
                          ctx->out_flags.as<uint32_t>());
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, hipMemcpyAsync(out_tokens, ctx->out_tokens.p, (size_t)rows * sizeof(int32_t), hipMemcpyDeviceToHost,
                               ctx->stream));
    std::vector<uint32_t> flags((size_t)rows);
    SR_HIP(ctx, hipMemcpyAsync(flags.data(), ctx->out_flags.p, (size_t)rows * sizeof(uint32_t), hipMemcpyDeviceToHost,
                               ctx->stream));
    SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    // rows that overflowed the selection kernel's row tail (thousands of equal logits at the cut) take the sort path
    std::vector<int32_t> redo;
    for (int32_t r = 0; r < rows; r++)
        if (flags[(size_t)r] & SR_KFLAG_UNSUPPORTED) redo.push_back(r);
    if (!redo.empty()) {
        rc = sr_resample_rows_launch(ctx, ctx->tmp_batch, dev, dtype, row_stride_elems, redo.data(), (int32_t)redo.size(),
                                     ctx->out_tokens.as<int32_t>(), ctx->out_flags.as<uint32_t>());
        if (rc != SR_OK) return rc;
        SR_HIP(ctx, hipMemcpyAsync(out_tokens, ctx->out_tokens.p, (size_t)rows * sizeof(int32_t), hipMemcpyDeviceToHost,
                                   ctx->stream));
        SR_HIP(ctx, hipMemcpyAsync(flags.data(), ctx->out_flags.p, (size_t)rows * sizeof(uint32_t), hipMemcpyDeviceToHost,
                                   ctx->stream));
        SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    }
    if (out_flags) memcpy(out_flags, flags.data(), (size_t)rows * sizeof(uint32_t));
    return SR_OK;
}

static int argmax_check(sr_ctx* ctx, const void* logits_dev, int dtype, int32_t rows, int32_t vocab, int64_t row_stride_elems,
                        const int32_t* out_idx_dev)
{
    if (!out_idx_dev || (!logits_dev && vocab > 0)) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_argmax_rows: null tensor");
    if (rows < 0 || vocab < 0 || (vocab > 0 && row_stride_elems < vocab))
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_argmax_rows: bad shape");
    if (dtype != SR_DTYPE_F32 && dtype != SR_DTYPE_BF16)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_argmax_rows: unknown dtype");
    return SR_OK;
}

static SrArgmaxArgs argmax_args(sr_ctx* ctx, const void* logits_dev, int dtype, int32_t rows, int32_t vocab,
                                int64_t row_stride_elems, int32_t* out_idx_dev, float* out_val_dev)
{
    SrArgmaxArgs a{};
    a.logits = logits_dev;
    a.row_stride = row_stride_elems;
    a.vocab = vocab;
    a.dtype = dtype;
    a.rows = rows;
    a.out_idx = out_idx_dev;
    a.out_val = out_val_dev;
    sr_argmax_plan(a, ctx->cu_count);
    return a;
}

int sr_argmax_rows_launch(sr_ctx* ctx, const void* logits_dev, int dtype, int32_t rows, int32_t vocab,
                          int64_t row_stride_elems, int32_t* out_idx_dev, float* out_val_dev)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (rows == 0) return SR_OK;
    int rc = argmax_check(ctx, logits_dev, dtype, rows, vocab, row_stride_elems, out_idx_dev);
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, hipSetDevice(ctx->device));
    // slots and counters: zero when allocated, and every launch leaves them zero again
    SR_HIP(ctx, ctx->argmax_best.reserve((size_t)rows * sizeof(unsigned long long), ctx->stream, true));
    SR_HIP(ctx, ctx->argmax_done.reserve((size_t)rows * sizeof(uint32_t), ctx->stream, true));
    SrArgmaxArgs a = argmax_args(ctx, logits_dev, dtype, rows, vocab, row_stride_elems, out_idx_dev, out_val_dev);
    a.best = ctx->argmax_best.as<unsigned long long>();
    a.done = ctx->argmax_done.as<uint32_t>();
    // (a launch that failed may have left slots and counters that are not zero: every later call would be wrong, silently)
    if (ctx->argmax_scratch_dirty) {
        SR_HIP(ctx, hipMemsetAsync(ctx->argmax_best.p, 0, ctx->argmax_best.cap, ctx->stream));
        SR_HIP(ctx, hipMemsetAsync(ctx->argmax_done.p, 0, ctx->argmax_done.cap, ctx->stream));
        ctx->argmax_scratch_dirty = false;
    }
    const hipError_t e = sr_launch_argmax_rows(a, false, ctx->stream);
    if (e != hipSuccess) ctx->argmax_scratch_dirty = true;
    SR_HIP(ctx, e);
    return SR_OK;
}

static_assert(SR_ARGMAX_STATIC_ROWS == SR_ARGMAX_NOALLOC_MAX_ROWS, "the header states the size of the static scratch");
static_assert(SR_ROWBIT_HAS_LOGIT_BIAS == SR_ROW_HAS_LOGIT_BIAS && SR_ROWBIT_DRAFT_FROM_LOOKUP == SR_ROW_DRAFT_FROM_LOOKUP,
              "the kernels' names for the public flag bits");

int sr_argmax_rows_launch_noalloc(sr_ctx* ctx, const void* logits_dev, int dtype, int32_t rows, int32_t vocab,
                                  int64_t row_stride_elems, int32_t* out_idx_dev, float* out_val_dev)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (rows == 0) return SR_OK;
    int rc = argmax_check(ctx, logits_dev, dtype, rows, vocab, row_stride_elems, out_idx_dev);
    if (rc != SR_OK) return rc;
    if (rows > SR_ARGMAX_STATIC_ROWS)
        return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT,
                       "sr_argmax_rows_launch_noalloc: " + std::to_string(rows) + " rows, the static scratch holds " +
                           std::to_string(SR_ARGMAX_STATIC_ROWS) + " (use sr_argmax_rows_launch, or split the call)");
    if (!ctx->static_best) return sr_fail(ctx, SR_ERR_HIP, "sr_argmax_rows_launch_noalloc: the static scratch was not found at sr_create");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    SrArgmaxArgs a = argmax_args(ctx, logits_dev, dtype, rows, vocab, row_stride_elems, out_idx_dev, out_val_dev);
    a.best = ctx->static_best;
    a.done = ctx->static_done;
    // every caller on this device shares the array and it keeps what the last call left: clear the part this call uses
    SR_HIP(ctx, sr_launch_argmax_rows(a, true, ctx->stream));
    return SR_OK;
}

int sr_argmax_rows(sr_ctx* ctx, const void* logits, int dtype, int logits_on_device, int32_t rows, int32_t vocab,
                   int64_t row_stride_elems, int32_t* out_idx, float* out_val)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    if (rows == 0) return SR_OK;
    if (!out_idx) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_argmax_rows: out_idx is null");
    if (rows < 0 || vocab < 0) return sr_fail(ctx, SR_ERR_INVALID_ARGUMENT, "sr_argmax_rows: bad shape");
    SR_HIP(ctx, hipSetDevice(ctx->device));
    const void* dev = logits;
    if (vocab > 0) {
        if (!logits) return sr_fail(ctx, SR_ERR_NULL_ARGUMENT, "sr_argmax_rows: logits is null");
        int rc = stage_logits(ctx, logits, dtype, logits_on_device, rows, vocab, row_stride_elems, &dev);
        if (rc != SR_OK) return rc;
    }
    SR_HIP(ctx, ctx->out_tokens.reserve((size_t)rows * sizeof(int32_t), ctx->stream));
    SR_HIP(ctx, ctx->out_val.reserve((size_t)rows * sizeof(float), ctx->stream));
    int rc = sr_argmax_rows_launch(ctx, dev, dtype, rows, vocab, row_stride_elems, ctx->out_tokens.as<int32_t>(),
                                   ctx->out_val.as<float>());
    if (rc != SR_OK) return rc;
    SR_HIP(ctx, hipMemcpyAsync(out_idx, ctx->out_tokens.p, (size_t)rows * sizeof(int32_t), hipMemcpyDeviceToHost, ctx->stream));
    if (out_val)
        SR_HIP(ctx, hipMemcpyAsync(out_val, ctx->out_val.p, (size_t)rows * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    SR_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return SR_OK;
}

int sr_pack_allow_mask(const float* masked_logits, int32_t vocab, uint32_t* out_words)
{
    if (!masked_logits || !out_words) return SR_ERR_NULL_ARGUMENT;
    if (vocab < 0) return SR_ERR_INVALID_ARGUMENT;
    const int32_t nw = (vocab + 31) / 32;
    for (int32_t w = 0; w < nw; w++) {
        uint32_t bits = 0;
        const int32_t base = w * 32, n = std::min(32, vocab - base);
        for (int32_t i = 0; i < n; i++) {
            uint32_t u;
            memcpy(&u, &masked_logits[base + i], 4);
            if (u != 0xff800000u) bits |= 1u << i;
        }
        out_words[w] = bits;
    }
    return SR_OK;
}

#ifdef SR_TEST_HOOKS
// ---- test and measurement hooks (include/stingray_sampler_test.h) ------------------------------------------

int sr_debug_append_rebuilds(const sr_batch* b) { return b ? b->append_rebuilds : -1; }
int sr_debug_append_moves(const sr_batch* b) { return b ? b->append_moves : -1; }

int sr_debug_set_spin_limit(sr_ctx* ctx, uint32_t polls)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    ctx->spin_limit = polls;
    return SR_OK;
}

int sr_debug_set_row_wait_limit(sr_ctx* ctx, uint32_t polls)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    ctx->row_wait_limit = polls;
    return SR_OK;
}

int sr_debug_set_profile(sr_ctx* ctx, unsigned long long* prof_dev)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
#ifdef SR_PROFILE
    ctx->prof = prof_dev;
    return SR_OK;
#else
    (void)prof_dev;
    return sr_fail(ctx, SR_ERR_UNSUPPORTED, "sr_debug_set_profile: this library was built without -DSR_PROFILE");
#endif
}

int sr_selftest_expf(sr_ctx* ctx, const float* x_dev, float* y_dev, int64_t n)
{
    if (!ctx) return SR_ERR_NULL_ARGUMENT;
    SR_HIP(ctx, hipSetDevice(ctx->device));
    SR_HIP(ctx, sr_launch_selftest_expf(x_dev, y_dev, n, ctx->stream));
    return SR_OK;
}

#endif  // SR_TEST_HOOKS

}  // extern "C"
