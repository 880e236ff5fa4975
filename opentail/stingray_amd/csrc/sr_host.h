// Host-side state shared by the translation units behind the C ABI.
#pragma once
#include "../../../include/stingray_sampler.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <string>
#include <vector>

#include "sr_kernels.h"
#include "sr_types.h"

struct DeviceBuf {
    void* p = nullptr;
    size_t cap = 0;
    // Grows (never shrinks), by half at least: a buffer that grows a little with every call (the edit lists of a
    // decode loop) is not allocated anew every time.  zero_new clears a newly allocated buffer on `stream`.
    hipError_t reserve(size_t bytes, hipStream_t stream, bool zero_new = false)
    {
        if (bytes <= cap) return hipSuccess;
        if (p) bytes = std::max(bytes, cap + cap / 2);
        if (p) {
            hipError_t e = hipStreamSynchronize(stream);
            if (e != hipSuccess) return e;
            (void)hipFree(p);
            p = nullptr;
            cap = 0;
        }
        size_t want = std::max(bytes, (size_t)256);
        hipError_t e = hipMalloc(&p, want);
        if (e != hipSuccess) { p = nullptr; return e; }
        cap = want;
        if (zero_new) return hipMemsetAsync(p, 0, want, stream);
        return hipSuccess;
    }
    void release()
    {
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
    }
    template <typename T> T* as() const { return (T*)p; }
};

// Pinned host memory that a batch packs its small uploads into, so that the copies to the device are truly
// asynchronous and the upload need not wait for them.  An event marks the end of the copies of one upload; the next
// upload waits for it before it overwrites the memory.
struct HostStage {
    char* p = nullptr;
    size_t cap = 0, used = 0, wanted = 0;
    hipEvent_t ev = nullptr;
    bool busy = false;
    hipError_t begin()
    {
        if (busy) {
            hipError_t e = hipEventSynchronize(ev);
            if (e != hipSuccess) return e;
            busy = false;
        }
        if (wanted > cap) {
            if (p) (void)hipHostFree(p);
            p = nullptr;
            cap = 0;
            // roomy (a decode loop's edit lists grow; an upload that does not fit sends pieces unpacked and waits)
            const size_t want = 4 * wanted + 65536;
            hipError_t e = hipHostMalloc((void**)&p, want, hipHostMallocDefault);
            if (e != hipSuccess) { p = nullptr; return e; }
            cap = want;
        }
        used = wanted = 0;
        return hipSuccess;
    }
    // a copy of src inside the pinned memory, or nullptr when it does not fit (it will the next time)
    const void* put(const void* src, size_t bytes)
    {
        const size_t need = (bytes + 255) & ~(size_t)255;
        wanted += need;
        if (used + need > cap) return nullptr;
        void* dst = p + used;
        memcpy(dst, src, bytes);
        used += need;
        return dst;
    }
    hipError_t end(hipStream_t st)
    {
        if (!ev) {
            hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
            if (e != hipSuccess) return e;
        }
        hipError_t e = hipEventRecord(ev, st);
        if (e == hipSuccess) busy = true;
        return e;
    }
    void release()
    {
        if (p) (void)hipHostFree(p);
        if (ev) (void)hipEventDestroy(ev);
        p = nullptr;
        ev = nullptr;
        cap = used = wanted = 0;
        busy = false;
    }
};

// Pinned host memory for the short lists of a decode step (the changes of one appended token per row), which a
// kernel reads in place.  An event after every step's kernel would tell when its piece may be overwritten, but an
// event between two kernels of a stream costs about 4 us of device time here; so the memory is two halves, each filled
// piece by piece over many steps, and only the change of halves records an event (for everything enqueued so far) and
// waits for the one recorded when the other half was left, many steps ago.
struct HostRing {
    char* p = nullptr;
    size_t half = 0, used = 0;
    int cur = 0;
    hipEvent_t ev[2] = {nullptr, nullptr};
    bool pending[2] = {false, false};
    bool dirty = false;             // pieces handed out since the last wait for a whole stream
    hipStream_t last = nullptr;     // the stream of those pieces' kernels
    uint32_t epoch = 0;             // the owner's count of stream changes when the ring was last used
    // room for `need` bytes in the present half (its pieces are handed out by put)
    // (want_half: what a half should hold when the ring has to be made or made again anyway)
    // (owner_epoch: the context counts its changes of stream, and waits for the stream it leaves at every one of them)
    hipError_t begin(size_t need, hipStream_t st, size_t want_half = 0, uint32_t owner_epoch = 0)
    {
        hipError_t e = hipSuccess;
        if (dirty && st != last) {  // the caller changed streams: nothing orders the old stream's readers before new events
            // When the context itself made the change it has waited for the old stream already -- which the caller may
            // have destroyed since: it is not touched again.
            if (owner_epoch == epoch && (e = hipStreamSynchronize(last)) != hipSuccess) return e;
            pending[0] = pending[1] = dirty = false;
            used = 0;
        }
        epoch = owner_epoch;
        last = st;
        if (need > half) {  // grow: nothing may still be reading the old memory
            if (dirty && (e = hipStreamSynchronize(st)) != hipSuccess) return e;
            if (p) (void)hipHostFree(p);
            p = nullptr;
            half = used = 0;
            pending[0] = pending[1] = dirty = false;
            // (room for many calls of the usual size; a call that needs much -- every row of a batch moving its edits at
            // once -- gets room for two of its kind: pinned memory is slow to allocate)
            const size_t want = std::max(want_half, (need <= 65536 ? 16 * need : 2 * need) + 65536);
            if ((e = hipHostMalloc((void**)&p, 2 * want, hipHostMallocDefault)) != hipSuccess) { p = nullptr; return e; }
            half = want;
            cur = 0;
        }
        if (used + need > half) {
            for (int h = 0; h < 2; h++)
                if (!ev[h] && (e = hipEventCreateWithFlags(&ev[h], hipEventDisableTiming)) != hipSuccess) return e;
            if ((e = hipEventRecord(ev[cur], st)) != hipSuccess) return e;
            pending[cur] = true;
            cur ^= 1;
            if (pending[cur]) {
                if ((e = hipEventSynchronize(ev[cur])) != hipSuccess) return e;
                pending[cur] = false;
            }
            used = 0;
        }
        return hipSuccess;
    }
    // a copy of src inside the present half (begin made the room); nullptr when it does not fit after all
    const void* put(const void* src, size_t bytes)
    {
        const size_t need = std::max((bytes + 255) & ~(size_t)255, (size_t)256);  // (an empty list has an address too)
        if (!p || used + need > half) return nullptr;
        void* dst = p + (size_t)cur * half + used;
        if (bytes) memcpy(dst, src, bytes);
        used += need;
        dirty = true;
        return dst;
    }
    void release()  // (the owner has waited for the stream)
    {
        if (p) (void)hipHostFree(p);
        for (int h = 0; h < 2; h++)
            if (ev[h]) (void)hipEventDestroy(ev[h]);
        p = nullptr;
        ev[0] = ev[1] = nullptr;
        half = used = 0;
        pending[0] = pending[1] = dirty = false;
    }
};

struct sr_ctx {
    int device = 0;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    std::string err;
    int cu_count = 256;
    // scratch, lazily grown and reused across calls
    DeviceBuf cand, gmax, gmax2, gpos, gbound, row_done, argmax_best, argmax_done;
    // this device's copy of the scratch inside the library's code object (looked up once, at sr_create)
    unsigned long long* static_best = nullptr;
    uint32_t* static_done = nullptr;
    DeviceBuf work;          // fp32 rows of the full-vocabulary path
    DeviceBuf edit_tab;      // per row: the table of its edits (bitmap of the vocabulary + slots)
    DeviceBuf full_state;    // per-row scalars of the full-vocabulary path
    uint32_t full_seq = 0;   // number of the last launch of that path (SrFullState::maxkey)
    DeviceBuf host_logits;   // staging for host-resident logits
    DeviceBuf stage_probs;   // staging for host-resident distributions
    DeviceBuf out_tokens, out_flags, out_val;
    HostRing uni_ring;       // uniforms of the calls that take them as host arrays and enqueue a kernel (read in place)
    DeviceBuf sort_k0, sort_v0, sort_v1;  // sort segments of rows: top-p survivors, wide top-k rows (and their token ids)
    DeviceBuf ident;         // identity row list
    DeviceBuf redo_list;     // rows given to sr_resample_rows_launch
    int ident_rows = 0;
    DeviceBuf spec_probs;    // speculative verification: the target distributions of every position
    uint32_t stream_epoch = 0;  // changes of stream so far (each waits for the stream that is left)
    bool argmax_scratch_dirty = false;  // a launch of sr_argmax_rows_launch failed: its slots and counters are cleared before the next
    DeviceBuf spec_resid, spec_reject;  // ... the residual row of every row's first rejected position, that position
    DeviceBuf seg_part, seg_func;       // approximate sums and increment functions of the segments of prepared rows
    DeviceBuf full_row_sync;
    DeviceBuf full_seg_func, full_seg_ms, full_watch, full_watch_cnt, full_seg_keys;  // ... of the full-vocabulary path's denominators
    sr_batch* tmp_batch = nullptr;
    unsigned long long* prof = nullptr;  // test hook: phase timestamps of the selection kernel
    int last_epv = 4;                    // vector width of the last launch: what an upload builds scan masks for
    // Registered allow-masks (sr_mask_register): one device array of `pool_cap` slots of `pool_words` words each, the
    // id of a mask is its slot.  One vocabulary size per context at a time.
    DeviceBuf mask_pool;
    int32_t pool_vocab = 0, pool_words = 0, pool_cap = 0;
    std::vector<uint8_t> pool_used;
    // pool_gen counts the times the pool started again (another vocabulary), pool_slot_gen[id] the releases of a slot:
    // a batch remembers both for the ids it names, and a launch refuses a batch whose ids have changed hands since
    unsigned pool_gen = 0;
    std::vector<uint32_t> pool_slot_gen;
    DeviceBuf mask_any;      // sr_mask_and: "a bit is left" word
    // selection kernel: entries per set of counters, launches so far (its parity picks the set), and how often a row
    // tail polls its row's counter before it stops waiting and selects from the logits alone
    size_t done_cap = 0;
    unsigned launch_no = 0;
    uint32_t spin_limit = 1u << 22;
    uint32_t row_wait_limit = 1u << 15;  // SrFullArgs::row_wait_limit (a poll is a round trip to device memory: tens of ms)
};

struct sr_batch {
    sr_ctx* ctx = nullptr;
    int32_t rows = 0, vocab = 0, upr = 0;
    std::vector<SrRow> h_rows;
    std::vector<SrEdit> h_edits;
    std::vector<int32_t> h_sel_list;   // rows on the selection kernel: TOPK and plain GREEDY
    std::vector<int32_t> h_full_list;  // rows on the full-vocabulary path
    std::vector<int32_t> h_sched;     // the selection kernel's programs and chunk items (host copy, read by an async upload)
    // the selection kernel's grid (see SrTopkArgs): workers (= programs at the head of d_sched) and chunk items
    int32_t n_workers = 0, n_items = 0;
    bool own_rows = false;  // one worker per row
    std::vector<int32_t> h_wide_list;  // SampleTopK rows too wide for the selection kernel
    std::vector<SrScanDesc> h_scan;    // scan-mask rows of the selection kernel
    std::vector<uint32_t> h_scan_need; // per batch row: SR_SCAN_* bits the row's scan mask must carry
    DeviceBuf d_rows, d_edits, d_sel_list, d_full_list, d_wide_list, d_scan_desc, d_mask, d_scan_mask, d_uniforms, d_sched;
    // speculative verification: the rows' descriptors, one copy per position, for `spec_positions` positions (0: to be
    // made again, because the descriptors have changed since)
    mutable DeviceBuf spec_rows;
    mutable int spec_positions = 0;
    int64_t mask_stride = 0, scan_stride = 0;
    // what the scan masks were built for: elements per 16-byte vector, the logits base address modulo 16 and
    // the row stride in bytes modulo 16 (rows share a mask row only when all start at the same offset)
    int32_t scan_epv = 0, scan_base_mod = -1, scan_stride_mod = -1;
    bool has_mask = false;
    bool mask_ids = false;               // the rows' allow-masks are registered masks of the context (mask_row = id)
    std::vector<int32_t> keep_mask_ids;  // ... per row, -1 none
    std::vector<uint32_t> keep_mask_gen; // ... the release count of the row's slot when the row took the id
    unsigned mask_pool_gen = 0;          // ... the pool's generation at that time
    int32_t max_sel = 0;
    HostStage stage;
    HostRing patch_ring;  // the lists of sr_batch_append_tokens          // pinned copies of what an upload sends to the device
    std::vector<SrCopySeg> segs;  // ... the pieces that are packed and not yet sent
    bool upload_must_wait = false;  // some copy of the running upload reads pageable memory directly
    // geometry the scan masks were built with (sr_batch_append_tokens clears single bits in place)
    int32_t scan_chunks = 0, scan_chunk_vecs = 0;
    unsigned long long scan_base_addr = 0;
    long long scan_stride_bytes = 0;
    // What sr_batch_append_tokens needs of the last upload: the inputs of a batch without allow-masks (kept flat as
    // they came; the histories are split per row by the first append) and the room each row's edit range has.
    bool can_append = false, hist_split = false;
    bool host_ahead = false;  // an append call failed after it had changed the host's copies: the next one rebuilds the batch
    int32_t append_rebuilds = 0;  // calls of sr_batch_append_tokens that rebuilt the batch (test hook)
    int32_t append_moves = 0;     // ... rows that were moved to the end of the edit array instead
    std::vector<sr_row_params> keep_params;
    std::vector<int32_t> keep_hist_ids, keep_hist_off, keep_bias_ids, keep_bias_off;
    std::vector<float> keep_bias_vals;
    std::vector<std::vector<int32_t>> keep_hist;
    std::vector<int32_t> edit_cap;
    std::vector<int32_t> sel_cap;   // per row: the sel that the launch's chunk items were written for (>= the row's sel)
    std::vector<int32_t> edit_ids;  // the ids of h_edits, contiguous (searched by the append; made when first needed)
};

// room left behind the edits of a row whose edits are kept in order of first appearance, for ids that
// sr_batch_append_tokens adds
#define SR_EDIT_SLACK 32

inline int sr_fail(sr_ctx* ctx, int code, const std::string& msg)
{
    if (ctx) ctx->err = msg;
    return code;
}
inline int sr_fail_hip(sr_ctx* ctx, hipError_t e, const char* what)
{
    return sr_fail(ctx, SR_ERR_HIP, std::string(what) + " failed: " + hipGetErrorString(e));
}
#define SR_HIP(ctx, call)                                             \
    do {                                                              \
        hipError_t _e = (call);                                       \
        if (_e != hipSuccess) return sr_fail_hip((ctx), _e, #call);   \
    } while (0)

// SR_OK, or SR_ERR_INVALID_ARGUMENT when the batch names a registered mask that was released (or whose pool was
// started again for another vocabulary) after the batch took the id: to be called before every launch that reads masks
int sr_batch_masks_valid(sr_ctx* ctx, const sr_batch* b, const char* who);
// where a batch's allow-masks lie: its own upload, or the context's registered masks (sr_api.cpp)
const uint32_t* sr_batch_mask_ptr(const sr_batch* b);
int64_t sr_batch_mask_stride(const sr_batch* b);

// Full-vocabulary rows of a batch (sr_full_host.cpp).  mode: 0 = sample, 1 = build distribution,
// 2 = build distribution and sample from it.
int sr_full_rows_launch(sr_ctx* ctx, const sr_batch* b, const void* logits_dev, int dtype, int64_t row_stride,
                        int32_t* out_tokens_dev, uint32_t* out_flags_dev);
// SampleTopK by device-wide sorts for the SampleTopK rows in list_dev (sr_full_host.cpp)
int sr_wide_rows_launch(sr_ctx* ctx, const sr_batch* b, const int32_t* list_dev, int n_rows, const void* logits_dev,
                        int dtype, int64_t row_stride, int32_t* out_tokens_dev, uint32_t* out_flags_dev);
