// Top-k-first sampling (the reference's SampleTopK, Sampler.cs:216-357) and plain greedy rows.
//
// One launch, grid = rows x chunks.  A workgroup loads one contiguous chunk of a row ONCE into
// registers (19 x 16 B per thread), derives a safe chunk-local threshold from per-thread group maxima
// (the sel-th largest of 2048 disjoint-group maxima can never exceed the chunk's sel-th largest
// element), emits the few elements at or above it, and signals the row.  The workgroup that arrives
// last for a row runs the row tail: exact top-(k + history) selection of the merged candidates by
// (value desc, index asc) with LDS radix histograms, a bitonic sort, penalties + stable re-sort, then
// the softmax / min-p / top-p / draw arithmetic in the reference's sequential fp32 order.
#include "sr_device.cuh"
#include "sr_types.h"
#include "sr_kernels.h"

namespace {

constexpr int kThreads = SR_TK_THREADS;
constexpr int kWaves = kThreads / SR_WAVE;
constexpr int kVec = SR_TK_VEC;
constexpr int kCap = SR_TK_CAP;
constexpr int kSortCap = SR_TK_SORT_CAP;
constexpr int kSelMax = SR_TK_SEL_MAX;
constexpr uint32_t kKeyNegInf = 0x007fffffu;  // sr_okey(-inf)
constexpr uint32_t kRowHasPenalty = SR_ROWFLAG_HAS_PENALTY;

struct TopkSmem {
    unsigned long long sortbuf[kSortCap];
    float vals[kSelMax];
    int idxs[kSelMax];
    float probs[kSelMax];
    uint32_t hist[256];
    uint32_t red[2 * kWaves];
    uint32_t bcast[8];
};

// ---- block-wide radix select over keys produced by a per-thread enumerator -----------------------
// Returns the need-th largest key (1-based) among all keys every thread enumerates.  Keys equal to 0
// act as "absent".  Must be called by all threads of the block.
template <typename ForEach>
__device__ uint32_t block_radix_select(ForEach for_each_key, int need, TopkSmem& sm)
{
    const int tid = threadIdx.x, lane = sr_lane(), wave = sr_wave_id();
    uint32_t lmax = 0u, lmin = 0xffffffffu;
    for_each_key([&](uint32_t k) { lmax = k > lmax ? k : lmax; lmin = k < lmin ? k : lmin; });
    lmax = sr_wave_max_u32(lmax);
    lmin = sr_wave_min_u32(lmin);
    __syncthreads();  // protects red/bcast/hist against a previous call's readers
    if (lane == 0) { sm.red[wave] = lmax; sm.red[kWaves + wave] = lmin; }
    __syncthreads();
    uint32_t bmax = 0u, bmin = 0xffffffffu;
#pragma unroll
    for (int w = 0; w < kWaves; w++) {
        uint32_t a = sm.red[w], b = sm.red[kWaves + w];
        bmax = a > bmax ? a : bmax;
        bmin = b < bmin ? b : bmin;
    }
    uint32_t diff = bmax ^ bmin;
    if (diff == 0u) return bmax;
    int shift = 32 - __clz(diff);  // bits [0, shift) are undecided
    uint32_t pmask = (shift >= 32) ? 0u : ~((1u << shift) - 1u);
    uint32_t prefix = bmax & pmask;
    while (shift > 0) {
        int nb = shift < 8 ? shift : 8;
        shift -= nb;
        const uint32_t dmask = (1u << nb) - 1u;
        if (tid < 256) sm.hist[tid] = 0u;
        __syncthreads();
        for_each_key([&](uint32_t k) {
            if ((k & pmask) == prefix) atomicAdd(&sm.hist[(k >> shift) & dmask], 1u);
        });
        __syncthreads();
        if (wave == 0) {
            uint32_t h0 = sm.hist[4 * lane], h1 = sm.hist[4 * lane + 1], h2 = sm.hist[4 * lane + 2],
                     h3 = sm.hist[4 * lane + 3];
            int tot = (int)(h0 + h1 + h2 + h3);
            int incl = sr_wave_incl_scan_i32(tot);
            int total = __shfl(incl, SR_WAVE - 1);
            int suffix = total - incl + tot;  // keys in bins of this lane and higher lanes
            unsigned long long b = __ballot(suffix >= need);
            int L = b ? (63 - __clzll(b)) : 0;
            if (lane == L) {
                int c = suffix - tot;  // keys in strictly higher lanes
                uint32_t hs[4] = {h0, h1, h2, h3};
                int digit = 4 * L, nn = need - c;
                bool found = false;
#pragma unroll
                for (int q = 3; q >= 0; q--) {
                    if (!found && c + (int)hs[q] >= need) { digit = 4 * L + q; nn = need - c; found = true; }
                    if (!found) c += (int)hs[q];
                }
                if (!found) { digit = 0; nn = 1; }  // need exceeds the population: take the lowest bin
                sm.bcast[0] = (uint32_t)digit;
                sm.bcast[1] = (uint32_t)nn;
            }
        }
        __syncthreads();
        uint32_t digit = sm.bcast[0];
        need = (int)sm.bcast[1];
        prefix |= digit << shift;
        pmask |= dmask << shift;
    }
    return prefix;
}

// ---- bitonic sort, descending, of sm.sortbuf[0 .. n_pow2) ----------------------------------------
__device__ void block_bitonic_sort_desc(unsigned long long* s, int n_pow2)
{
    const int tid = threadIdx.x;
    for (int k2 = 2; k2 <= n_pow2; k2 <<= 1) {
        for (int j2 = k2 >> 1; j2 > 0; j2 >>= 1) {
            for (int i = tid; i < n_pow2; i += kThreads) {
                int ixj = i ^ j2;
                if (ixj > i) {
                    unsigned long long a = s[i], b = s[ixj];
                    bool desc_block = ((i & k2) == 0);
                    if ((a < b) == desc_block) { s[i] = b; s[ixj] = a; }
                }
            }
            __syncthreads();
        }
    }
}

__device__ __forceinline__ int next_pow2(int n)
{
    int p = 1;
    while (p < n) p <<= 1;
    return p;
}

// ---- block-wide exclusive scan of one int per thread; returns the exclusive prefix, total in *tot ---
__device__ __forceinline__ int block_excl_scan(int v, int* tot, TopkSmem& sm)
{
    const int lane = sr_lane(), wave = sr_wave_id();
    int incl = sr_wave_incl_scan_i32(v);
    __syncthreads();
    if (lane == SR_WAVE - 1) sm.red[wave] = (uint32_t)incl;
    __syncthreads();
    int base = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; w++) {
        int t = (int)sm.red[w];
        if (w < wave) base += t;
        total += t;
    }
    *tot = total;
    return base + incl - v;
}

// ---- element access into the register-resident chunk ---------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <int EPV> struct VecOps;
template <> struct VecOps<4> {  // four fp32 per 16-byte vector
    static __device__ __forceinline__ float get(const u32x4& v, int c) { return sr_u2f(v[c]); }
    static __device__ __forceinline__ void kill(u32x4& v, int c) { v[c] = 0xff800000u; }
    static __device__ __forceinline__ u32x4 neg_inf() { return (u32x4)(0xff800000u); }
};
template <> struct VecOps<8> {  // eight bf16 per 16-byte vector; the upcast to fp32 is exact
    static __device__ __forceinline__ float get(const u32x4& v, int c)
    {
        uint32_t w = v[c >> 1];
        return sr_u2f((c & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    static __device__ __forceinline__ void kill(u32x4& v, int c)
    {
        uint32_t w = v[c >> 1];
        v[c >> 1] = (c & 1) ? ((w & 0x0000ffffu) | 0xff800000u) : ((w & 0xffff0000u) | 0x0000ff80u);
    }
    static __device__ __forceinline__ u32x4 neg_inf() { return (u32x4)(0xff80ff80u); }
};

__device__ __forceinline__ bool mask_bit(const uint32_t* m, int e) { return ((m[e >> 5] >> (e & 31)) & 1u) != 0u; }

// ---- the row tail ----------------------------------------------------------------------------------
// Called by every thread of the last workgroup of a row.  slot = position of the row in this launch.
__device__ void topk_row_tail(const SrTopkArgs& a, int slot, int row, const SrRow& rd, TopkSmem& sm)
{
    const int tid = threadIdx.x;
    const int S = a.chunks;
    const float* cval = a.cand_val + (size_t)slot * S * kCap;
    const int* cidx = a.cand_idx + (size_t)slot * S * kCap;
    const int* ccnt = a.cand_cnt + (size_t)slot * S;

    uint32_t out_flag = (rd.path == SR_PATH_TOPK) ? SR_KFLAG_TOPK : SR_KFLAG_GREEDY;
    bool overflow = false;
    int n_total = 0;
    for (int c = 0; c < S; c++) {
        int n = ccnt[c];
        if (n > kCap) overflow = true;
        n_total += n;
    }
    const int sel = rd.sel;
    if (overflow || sel > kSelMax) {
        if (tid == 0) {
            a.out_tokens[row] = -1;
            if (a.out_flags) a.out_flags[row] = out_flag | SR_KFLAG_UNSUPPORTED;
        }
        return;
    }
    if (n_total == 0) {
        // no finite logit anywhere: Greedy over the raw row = index 0 (Sampler.cs:254-255, :442-446)
        if (tid == 0) {
            a.out_tokens[row] = 0;
            if (a.out_flags) a.out_flags[row] = out_flag | SR_KFLAG_DEGENERATE;
        }
        return;
    }

    // exact key of the sel-th largest candidate
    auto each_key = [&](auto&& body) {
        for (int c = 0; c < S; c++) {
            int n = ccnt[c];
            const float* v = cval + (size_t)c * kCap;
            for (int i = tid; i < n; i += kThreads) body(sr_okey(v[i]));
        }
    };
    uint32_t tkey = (n_total <= sel) ? 0u : block_radix_select(each_key, sel, sm);

    // How many candidates sit at or above that key?  With few ties they are all sorted; with many
    // (quantised or constant rows) only the lowest-index ties that still fit into sel are kept.
    int c_ge = 0, c_gt = 0;
    each_key([&](uint32_t k) { c_ge += (k >= tkey) ? 1 : 0; c_gt += (k > tkey) ? 1 : 0; });
    int m_ge, m_gt;
    block_excl_scan(c_ge, &m_ge, sm);
    block_excl_scan(c_gt, &m_gt, sm);
    uint32_t tidx_key = 0u;  // ties need (0xffffffff - idx) >= tidx_key
    if (m_ge > kSortCap) {
        auto each_tie = [&](auto&& body) {
            for (int c = 0; c < S; c++) {
                int n = ccnt[c];
                const float* v = cval + (size_t)c * kCap;
                const int* ix = cidx + (size_t)c * kCap;
                for (int i = tid; i < n; i += kThreads)
                    if (sr_okey(v[i]) == tkey) body(0xffffffffu - (uint32_t)ix[i]);
            }
        };
        tidx_key = block_radix_select(each_tie, sel - m_gt, sm);
    }
    __syncthreads();
    if (tid == 0) sm.bcast[4] = 0u;
    __syncthreads();
    for (int c = 0; c < S; c++) {
        int n = ccnt[c];
        const float* v = cval + (size_t)c * kCap;
        const int* ix = cidx + (size_t)c * kCap;
        for (int i = tid; i < n; i += kThreads) {
            uint32_t k = sr_okey(v[i]);
            uint32_t ik = 0xffffffffu - (uint32_t)ix[i];
            if (k > tkey || (k == tkey && ik >= tidx_key)) {
                uint32_t pos = atomicAdd(&sm.bcast[4], 1u);
                if (pos < (uint32_t)kSortCap) sm.sortbuf[pos] = ((unsigned long long)k << 32) | (unsigned long long)ik;
            }
        }
    }
    __syncthreads();
    const int m = (int)sm.bcast[4];
    if (m > kSortCap) {  // cannot happen: m <= max(sel, kSortCap); kept as a guard
        if (tid == 0) {
            a.out_tokens[row] = -1;
            if (a.out_flags) a.out_flags[row] = out_flag | SR_KFLAG_UNSUPPORTED;
        }
        return;
    }
    int P = next_pow2(m < 2 ? 2 : m);
    for (int i = m + tid; i < P; i += kThreads) sm.sortbuf[i] = 0ull;
    __syncthreads();
    block_bitonic_sort_desc(sm.sortbuf, P);

    if (rd.path == SR_PATH_GREEDY_PEN) {
        // GreedyWithHistoryPenalties (Sampler.cs:421-437): only the history ids change value, so the
        // argmax is the better of (a) the best adjusted history id and (b) the best raw candidate that is
        // not a history id -- one exists among the top (distinct ids + 1) candidates.
        const SrEdit* ed = a.edits + rd.edit_off;
        const int ne = rd.edit_cnt;
        unsigned long long best = 0ull;
        int first_free = 0x7fffffff;
        for (int t = tid; t < m; t += kThreads) {
            int id = (int)(0xffffffffu - (uint32_t)(sm.sortbuf[t] & 0xffffffffull));
            int lo = 0, hi = ne;
            while (lo < hi) {
                int mid = (lo + hi) >> 1;
                if (ed[mid].id < id) lo = mid + 1; else hi = mid;
            }
            if (!(lo < ne && ed[lo].id == id)) { first_free = t; break; }
        }
        const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * (a.dtype == 1 ? 2 : 4);
        const uint32_t* mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
        for (int e = tid; e < ne; e += kThreads) {
            const int id = ed[e].id;
            float x = (a.dtype == 1) ? sr_bf16_to_f32(((const uint16_t*)rowp)[id]) : ((const float*)rowp)[id];
            if (mrow && !mask_bit(mrow, id)) x = SR_NEG_INF;
            if (rd.rep != 1.0f)
                for (int o = 0; o < ed[e].occ_win; o++) x = x > 0.0f ? __fdiv_rn(x, rd.rep) : __fmul_rn(x, rd.rep);
            if (rd.presence != 0.0f || rd.frequency != 0.0f)
                x = __fsub_rn(x, __fadd_rn(rd.presence, __fmul_rn(rd.frequency, (float)ed[e].occ_all)));
            if (sr_f2u(x) != 0xff800000u && x == x) {
                unsigned long long c = ((unsigned long long)sr_okey(x) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)id);
                best = c > best ? c : best;
            }
        }
        first_free = sr_wave_min_i32(first_free);
        best = sr_wave_max_u64(best);
        __syncthreads();
        if (sr_lane() == 0) {
            sm.red[sr_wave_id()] = (uint32_t)first_free;
            ((unsigned long long*)sm.vals)[sr_wave_id()] = best;  // vals is unused on this path
        }
        __syncthreads();
        if (tid == 0) {
            int ff = 0x7fffffff;
            for (int w = 0; w < kWaves; w++) {
                ff = min(ff, (int)sm.red[w]);
                unsigned long long c = ((unsigned long long*)sm.vals)[w];
                best = c > best ? c : best;
            }
            if (ff != 0x7fffffff && sm.sortbuf[ff] > best) best = sm.sortbuf[ff];
            // nothing finite at all: every adjusted logit is -inf and the first index wins
            a.out_tokens[row] = best ? (int)(0xffffffffu - (uint32_t)(best & 0xffffffffull)) : 0;
            if (a.out_flags) a.out_flags[row] = out_flag | (best ? 0u : SR_KFLAG_DEGENERATE);
        }
        return;
    }
    if (rd.path == SR_PATH_GREEDY) {
        if (tid == 0) {
            a.out_tokens[row] = (int)(0xffffffffu - (uint32_t)(sm.sortbuf[0] & 0xffffffffull));
            if (a.out_flags) a.out_flags[row] = out_flag;
        }
        return;
    }

    // vals/idx: the sel best in (value desc, index asc) order; unfilled slots are (-inf, -1)
    for (int t = tid; t < sel; t += kThreads) {
        if (t < m) {
            unsigned long long e = sm.sortbuf[t];
            sm.vals[t] = sr_okey_inv((uint32_t)(e >> 32));
            sm.idxs[t] = (int)(0xffffffffu - (uint32_t)(e & 0xffffffffull));
        } else {
            sm.vals[t] = SR_NEG_INF;
            sm.idxs[t] = -1;
        }
    }
    __syncthreads();

    if (rd.flags & kRowHasPenalty) {
        // Sampler.cs:261-294: pen = pow(rep, occWindow) once, presence/frequency over the whole
        // history, then a stable re-sort by value.
        const SrEdit* ed = a.edits + rd.edit_off;
        const int ne = rd.edit_cnt;
        for (int t = tid; t < sel; t += kThreads) {
            int id = sm.idxs[t];
            if (id < 0) continue;
            int lo = 0, hi = ne;
            while (lo < hi) {
                int mid = (lo + hi) >> 1;
                if (ed[mid].id < id) lo = mid + 1; else hi = mid;
            }
            if (lo < ne && ed[lo].id == id && ed[lo].occ_all > 0) {
                float v = sm.vals[t];
                if (rd.rep != 1.0f && ed[lo].occ_win > 0) {
                    float pen = ed[lo].pen;
                    v = v > 0.0f ? __fdiv_rn(v, pen) : __fmul_rn(v, pen);
                }
                float sub = __fadd_rn(rd.presence, __fmul_rn(rd.frequency, (float)ed[lo].occ_all));
                sm.vals[t] = __fsub_rn(v, sub);
            }
        }
        __syncthreads();
        int P2 = next_pow2(sel < 2 ? 2 : sel);
        for (int t = tid; t < P2; t += kThreads)
            sm.sortbuf[t] = (t < sel) ? (((unsigned long long)sr_okey(sm.vals[t]) << 32) |
                                         (unsigned long long)(0xffffffffu - (uint32_t)t))
                                      : 0ull;
        __syncthreads();
        block_bitonic_sort_desc(sm.sortbuf, P2);
        // permute (value, idx) by the sorted ranks; read everything before anything is overwritten
        float nv[kSelMax / kThreads];
        int ni[kSelMax / kThreads];
#pragma unroll
        for (int q = 0; q < kSelMax / kThreads; q++) {
            int t = tid + q * kThreads;
            if (t < sel) {
                unsigned long long e = sm.sortbuf[t];
                int old = (int)(0xffffffffu - (uint32_t)(e & 0xffffffffull));
                nv[q] = sm.vals[old];
                ni[q] = sm.idxs[old];
            }
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kSelMax / kThreads; q++) {
            int t = tid + q * kThreads;
            if (t < sel) { sm.vals[t] = nv[q]; sm.idxs[t] = ni[q]; }
        }
        __syncthreads();
    }

    // Sampler.cs:297-349
    const int k = rd.top_k;  // k <= sel
    const float inv_temp = rd.temperature == 1.0f ? 1.0f : __fdiv_rn(1.0f, rd.temperature);
    const float mx = __fmul_rn(sm.vals[0], inv_temp);
    for (int t = tid; t < k; t += kThreads) {
        float v = sm.vals[t];
        sm.probs[t] = (sr_f2u(v) == 0xff800000u) ? 0.0f : sr_expf(__fsub_rn(__fmul_rn(v, inv_temp), mx));
    }
    __syncthreads();
    if (tid == 0) {
        float sum = 0.0f;
        for (int t = 0; t < k; t++) sum = __fadd_rn(sum, sm.probs[t]);
        sm.bcast[5] = sr_f2u(sum);
    }
    __syncthreads();
    const float sum = sr_u2f(sm.bcast[5]);
    const float inv_sum = sum > 0.0f ? __fdiv_rn(1.0f, sum) : 0.0f;
    for (int t = tid; t < k; t += kThreads) sm.probs[t] = __fmul_rn(sm.probs[t], inv_sum);
    __syncthreads();

    // min-p: first t with probs[t] < thr bounds the survivors
    int count = k;
    if (rd.min_p > 0.0f) {
        const float thr = __fmul_rn(rd.min_p, sm.probs[0]);
        int first = k;
        for (int t = tid; t < k; t += kThreads)
            if (sm.probs[t] < thr) { first = t; break; }
        first = sr_wave_min_i32(first);
        __syncthreads();
        if (sr_lane() == 0) sm.red[sr_wave_id()] = (uint32_t)first;
        __syncthreads();
        for (int w = 0; w < kWaves; w++) count = min(count, (int)sm.red[w]);
    }
    // running sum; probs[t] becomes cum[t].  top-p cuts after the first cum >= TopP.
    if (tid == 0) {
        const bool use_top_p = rd.top_p < 1.0f && rd.top_p > 0.0f;
        float cum = 0.0f;
        int cnt = count;
        for (int t = 0; t < count; t++) {
            cum = __fadd_rn(cum, sm.probs[t]);
            sm.probs[t] = cum;
            if (use_top_p && cum >= rd.top_p) { cnt = t + 1; break; }
        }
        sm.bcast[6] = (uint32_t)cnt;
    }
    __syncthreads();
    count = (int)sm.bcast[6];
    const float kept_sum = count > 0 ? sm.probs[count - 1] : 0.0f;
    const float r = __fmul_rn(__double2float_rn(a.uniforms[(size_t)row * a.uniforms_per_row]), kept_sum);
    int first = 0x7fffffff;
    for (int t = tid; t < count; t += kThreads)
        if (r <= sm.probs[t] && sm.idxs[t] >= 0) { first = t; break; }
    first = sr_wave_min_i32(first);
    __syncthreads();
    if (sr_lane() == 0) sm.red[sr_wave_id()] = (uint32_t)first;
    __syncthreads();
    if (tid == 0) {
        int best = 0x7fffffff;
        for (int w = 0; w < kWaves; w++) best = min(best, (int)sm.red[w]);
        a.out_tokens[row] = (best != 0x7fffffff) ? sm.idxs[best] : sm.idxs[0];
        if (a.out_flags) a.out_flags[row] = out_flag;
    }
}

// ---- the kernel --------------------------------------------------------------------------------------
template <int EPV>
__global__ __launch_bounds__(kThreads, 4) void k_topk_rows(SrTopkArgs a)
{
    __shared__ TopkSmem sm;
    using VO = VecOps<EPV>;
    const int tid = threadIdx.x, lane = sr_lane(), wave = sr_wave_id();
    const int S = a.chunks;
    const int slot = blockIdx.x / S, c = blockIdx.x - slot * S;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    const int V = a.vocab;
    const int lo = c * a.chunk_len;
    const int hi = min(V, lo + a.chunk_len);
    const int sel = rd.sel;
    int total = 0;

    if (lo < hi && sel <= kSelMax) {
        constexpr int ES = (EPV == 4) ? 4 : 2;  // element size in bytes
        const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
        const uintptr_t addr = (uintptr_t)(rowp + (size_t)lo * ES);
        const int mis = (int)((addr & 15u) / ES);
        const u32x4* wp = (const u32x4*)(addr - (uintptr_t)mis * ES);
        const int wbase = lo - mis;  // row element index of window element 0
        const int nvec = (hi - wbase + EPV - 1) / EPV;
        const uint32_t* mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;

        u32x4 v[kVec];
#pragma unroll
        for (int j = 0; j < kVec; j++) {
            int f = j * kThreads + tid;
            v[j] = (f < nvec) ? __builtin_nontemporal_load(&wp[f]) : VO::neg_inf();
        }
        // edges of the window and the allow-mask: one keep-bit per element of the vector
        const int mask_words = (int)a.mask_stride;
#pragma unroll
        for (int j = 0; j < kVec; j++) {
            const int f = j * kThreads + tid;
            if (f < nvec) {
                const int e0 = wbase + f * EPV;
                uint32_t keep = (1u << EPV) - 1u;
                if (e0 < lo || e0 + EPV > hi) {
#pragma unroll
                    for (int q = 0; q < EPV; q++)
                        if (e0 + q < lo || e0 + q >= hi) keep &= ~(1u << q);
                }
                if (mrow) {
                    const int es = e0 < 0 ? 0 : e0;       // first bit that exists
                    const int wi = es >> 5, sh = es & 31;
                    unsigned long long bits = mrow[wi];
                    if (wi + 1 < mask_words) bits |= (unsigned long long)mrow[wi + 1] << 32;
                    keep &= (uint32_t)(bits >> sh) << (es - e0);
                }
                if (keep != (1u << EPV) - 1u) {
#pragma unroll
                    for (int q = 0; q < EPV; q++)
                        if (!((keep >> q) & 1u)) VO::kill(v[j], q);
                }
            }
        }

        // A safe lower bound on the chunk's sel-th largest element.
        uint32_t tkey;
        if (nvec <= 4 * kThreads) {
            // short chunk (at most four vectors per thread): select exactly over its elements
            auto each_elem = [&](auto&& body) {
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int q = 0; q < EPV; q++) body(sr_okey(VO::get(v[j], q)));
            };
            tkey = block_radix_select(each_elem, sel, sm);
        } else {
            // every thread owns four interleaved groups of vectors (j mod 4), all populated here; the
            // sel-th largest of the 2048 disjoint-group maxima cannot exceed the sel-th largest element
            uint32_t gk[SR_TK_GROUPS];
#pragma unroll
            for (int g = 0; g < SR_TK_GROUPS; g++) {
                float mxv = SR_NEG_INF;
#pragma unroll
                for (int j = g; j < kVec; j += SR_TK_GROUPS)
#pragma unroll
                    for (int q = 0; q < EPV; q++) mxv = fmaxf(mxv, VO::get(v[j], q));
                gk[g] = sr_okey(mxv);
            }
            auto each_gk = [&](auto&& body) {
#pragma unroll
                for (int g = 0; g < SR_TK_GROUPS; g++) body(gk[g]);
            };
            tkey = (sel > SR_TK_M) ? 0u : block_radix_select(each_gk, sel, sm);
        }
        // -inf never enters the candidate set (Sampler.cs:240-249: strict v <= -inf rejects it)
        const float tval = (tkey <= kKeyNegInf) ? -3.402823466e38f : sr_okey_inv(tkey);

        float* cv = a.cand_val + ((size_t)slot * S + c) * kCap;
        int* ci = a.cand_idx + ((size_t)slot * S + c) * kCap;
        int cnt = 0;
#pragma unroll
        for (int j = 0; j < kVec; j++)
#pragma unroll
            for (int q = 0; q < EPV; q++) cnt += (VO::get(v[j], q) >= tval) ? 1 : 0;
        int pos = block_excl_scan(cnt, &total, sm);
        if (total <= kCap) {
            if (cnt > 0) {
#pragma unroll
                for (int j = 0; j < kVec; j++) {
                    int e0 = wbase + (j * kThreads + tid) * EPV;
#pragma unroll
                    for (int q = 0; q < EPV; q++) {
                        float x = VO::get(v[j], q);
                        if (x >= tval) { cv[pos] = x; ci[pos] = e0 + q; pos++; }
                    }
                }
            }
        } else {
            // Many elements tie with the threshold value.  Equal values rank by ascending index, so
            // besides everything above the threshold only the first (sel - #above) ties can matter.
            int cgt = 0;
#pragma unroll
            for (int j = 0; j < kVec; j++)
#pragma unroll
                for (int q = 0; q < EPV; q++) cgt += (VO::get(v[j], q) > tval) ? 1 : 0;
            int total_gt;
            int pgt = block_excl_scan(cgt, &total_gt, sm);
            if (total_gt > kCap) {
                total = total_gt;  // genuine overflow: the row is reported as unsupported
            } else {
                if (cgt > 0) {
#pragma unroll
                    for (int j = 0; j < kVec; j++) {
                        int e0 = wbase + (j * kThreads + tid) * EPV;
#pragma unroll
                        for (int q = 0; q < EPV; q++) {
                            float x = VO::get(v[j], q);
                            if (x > tval) { cv[pgt] = x; ci[pgt] = e0 + q; pgt++; }
                        }
                    }
                }
                const int need_eq = min(sel - total_gt, kCap - total_gt);
                int emitted = 0;
                if (need_eq > 0) {
#pragma unroll
                    for (int j = 0; j < kVec; j++) {  // ascending j, then tid, then q = ascending index
                        if (emitted >= need_eq) continue;  // block-uniform
                        int ceq = 0;
#pragma unroll
                        for (int q = 0; q < EPV; q++) ceq += (VO::get(v[j], q) == tval) ? 1 : 0;
                        int tj;
                        int rank = emitted + block_excl_scan(ceq, &tj, sm);
                        if (ceq > 0) {
                            int e0 = wbase + (j * kThreads + tid) * EPV;
#pragma unroll
                            for (int q = 0; q < EPV; q++) {
                                if (VO::get(v[j], q) == tval) {
                                    if (rank < need_eq) { cv[total_gt + rank] = tval; ci[total_gt + rank] = e0 + q; }
                                    rank++;
                                }
                            }
                        }
                        emitted += tj;
                    }
                }
                total = total_gt + max(0, min(need_eq, emitted));
            }
        }
    }
    if (tid == 0) a.cand_cnt[(size_t)slot * S + c] = total;

    // publish, then let the last workgroup of the row run the tail
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        uint32_t prev = atomicAdd(&a.row_done[slot], 1u);
        sm.bcast[7] = (prev == (uint32_t)(S - 1)) ? 1u : 0u;
    }
    __syncthreads();
    if (!sm.bcast[7]) return;
    __threadfence();
    if (tid == 0) a.row_done[slot] = 0u;  // ready for the next launch
    topk_row_tail(a, slot, row, rd, sm);
}

}  // namespace

hipError_t sr_launch_topk(const SrTopkArgs& a, int n_rows, hipStream_t stream)
{
    if (n_rows <= 0) return hipSuccess;
    dim3 grid((unsigned)(n_rows * a.chunks)), block(kThreads);
    if (a.dtype == 1)
        hipLaunchKernelGGL(k_topk_rows<8>, grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL(k_topk_rows<4>, grid, block, 0, stream, a);
    return hipGetLastError();
}
