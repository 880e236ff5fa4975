// Top-k-first sampling (the reference's SampleTopK, Sampler.cs:216-357) and the greedy rows.
//
// One launch of persistent workgroups, each with a short list of chunks to stream and at most one row to finish.  A
// chunk is a contiguous piece of a row that a workgroup holds in registers ONCE (19 x 16 B per thread); it applies
// the row's scan mask and leaves, per lane and group of ~19 elements, the largest element, its position and the
// second largest, plus per wave a share of the row's bound.  Nothing is selected there: the workgroup streams.
// The worker that streams a row's last chunk then finishes the row (the row tail) and ends.
//
// The row tail derives a lower bound on the row's sel-th largest element from the waves' shares, takes the
// largest element of every group whose second largest is below the bound directly, fetches the few groups
// with more than one element above it again, and merges: penalties, pruning of candidates too small to
// change any fp32 sum, an order by (value after penalties, value before, index), then the softmax / min-p /
// top-p / draw arithmetic in the reference's sequential fp32 order.  A row whose candidates overflow the
// tail's lists (thousands of equal logits at the cut), or whose chunks were not handed over in time, is selected
// exactly from the logits themselves instead: every row gets its token in this launch.
//
// When the history penalties can only lower a logit (repetition >= 1, presence and frequency >= 0) the
// scan skips the history ids (a per-row scan mask built when the batch is uploaded) and asks for the
// top k only; the row tail fetches the history logits by id.  That set holds every token the
// reference's top (k + history length) selection can rank among its final k: a token outside the
// history is in the final k only if it is among the k best outside the history, and a history token
// that the reference's over-selection misses has more than k unpenalised tokens above it.  Penalties
// that can raise a logit keep the reference's literal over-selection.
#include "sr_device.h"
#include "sr_types.h"
#include "sr_kernels.h"
#include "sr_seqsum.h"

namespace {

// Phase timestamps exist in profiling builds only (-DSR_PROFILE); (a).prof then points at the 16 slots of the
// unit (chunk item or row) at work.
#ifdef SR_PROFILE
#define SR_PROF(a, slot_) do { if ((a).prof && threadIdx.x == 0) (a).prof[(slot_)] = (unsigned long long)wall_clock64(); } while (0)
#define SR_PROF_VAL(a, slot_, v_) do { if ((a).prof && threadIdx.x == 0) (a).prof[(slot_)] = (unsigned long long)(v_); } while (0)
#else
#define SR_PROF(a, slot_) do { } while (0)
#define SR_PROF_VAL(a, slot_, v_) do { } while (0)
#endif

constexpr int kThreads = SR_TK_THREADS;
constexpr int kWaves = kThreads / SR_WAVE;
constexpr int kSelMax = SR_TK_SEL_MAX;
constexpr int kRowCap = SR_TK_ROW_CAP;
constexpr uint32_t kKeyNegInf = 0x007fffffu;  // sr_okey(-inf)
constexpr uint32_t kRowHasPenalty = SR_ROWFLAG_HAS_PENALTY;
constexpr uint32_t kRowHistExcl = SR_ROWFLAG_HIST_EXCL;
constexpr int kQCap = 2 * kSelMax;            // groups of a row whose elements the row tail fetches

constexpr int kCandRegs = kRowCap / kThreads;   // candidates a thread holds in the row tail (16)
constexpr int kSortRegs = kSelMax / kThreads;   // sort elements per thread (4)
constexpr int kHistRegs = kSelMax / kThreads;   // history ids per thread (4)
constexpr int kShortList = 128;                 // most entries (candidates + history ids) ranked by counting
constexpr int kShortSel = SR_TK_SHORT_SEL;      // launches whose rows all ask for at most this many take the steps for short lists
constexpr int kBins = 1024;                     // histogram bins of the row tail
constexpr int kBinsPerLane = kBins / SR_WAVE;
// Bin b lives at word b + b / kBinsPerLane: the strip of kBinsPerLane bins that a lane scans starts one word
// further than a multiple of the strip length, so that the 64 lanes of a wave fall on different LDS banks.
constexpr int kBinsPad = kBins + SR_WAVE + 1;
__device__ __forceinline__ int bin_word(int b) { return b + b / kBinsPerLane; }
// The bin of an entry of the row tail, from xs = (its value) x (1 / temperature): 0 .. kBins - 1, never decreasing as
// the value falls (all that the ranking needs of it).  Two maps.  The plain one: equal steps of xs down from the
// origin.  The other one, when the candidates' lower bound is known: steps that grow with the distance u above that
// bound like the bit pattern of the float u + c does (128 bins per doubling, c = span / 256: eight doublings, all
// the bins), so that the crowd just above the bound is spread over many bins and the few entries far above it share
// few.
constexpr int kBinShift = 16;               // 2^(23 - 16) bins per doubling
constexpr float kBinOffset = 0.00390625f;   // c / span
struct BinMap {
    float mx = 0.0f;        // the origin: the largest kept element, scaled
    float bscale = -56.0f;  // plain map: bins per unit, negated
    float span = 0.0f;      // the other map: origin minus bound (scaled), the offset c and its bits, the bin of u = 0
    float c = 0.0f;
    uint32_t cbits = 0u;
    int ftop = 0;
    bool by_bits = false;
    // A third map, for rows of bf16 logits that no penalty touches: one bin per distinct value (the upper 16 bits of the
    // ordered key are the whole value), counted down from the row's largest.  Entries of one bin are then equal, no
    // order among them is needed for any sum, and the one entry whose index matters -- the draw's -- is picked from its
    // bin at the end: see topk_row_tail.
    bool exact = false;
    uint32_t ktop = 0u;     // ordered key of the row's largest kept element >> 16
    __device__ __forceinline__ int of_raw(float x) const { return min(max((int)(ktop - (sr_okey(x) >> 16)), 0), kBins - 1); }
    __device__ __forceinline__ int of(float xs) const
    {
        const float d = __fsub_rn(xs, mx);
        if (!by_bits) return min(max((int)__fmul_rn(d, bscale), 0), kBins - 1);
        const float u = fmaxf(__fadd_rn(d, span), 0.0f);
        const int f = (int)((sr_f2u(__fadd_rn(u, c)) - cbits) >> kBinShift);
        return min(max(ftop - f, 0), kBins - 1);
    }
};

struct TopkSmem {
    uint32_t xa[kSelMax];  // list of groups to fetch (xa and xb), then the kept entries by bin / the sort exchange
                           // (three 32-bit words per entry)
    uint32_t xb[kSelMax];
    uint32_t xc[kSelMax];
    float vals[kSelMax];   // candidate values, later the k best in order
    int idxs[kSelMax];     // ... and their indices
    __attribute__((aligned(16))) float probs[kSelMax + 8];  // per candidate (bin, arrival), later e, then the running sums
    uint32_t hist[256];
    uint32_t red[2 * kWaves];
    uint32_t bcast[16];
    uint32_t bhist[kBinsPad];  // live entries per bin of distance below the maximum
    uint32_t boff[kBinsPad];   // first list position of every bin
    uint32_t bfill[kBinsPad];  // entries scattered into the bin so far
};

// ---- block-wide radix select over keys produced by a per-thread enumerator -----------------------
// Returns the need-th largest key (1-based) among all keys every thread enumerates.  Keys equal to 0
// act as "absent".  Must be called by all threads of the block.
template <typename ForEach>
__device__ __forceinline__ uint32_t block_radix_select(ForEach for_each_key, int need, TopkSmem& sm)
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
    static __device__ __forceinline__ u32x4 neg_inf() { return (u32x4)(0xff800000u); }
};
template <> struct VecOps<8> {  // eight bf16 per 16-byte vector; the upcast to fp32 is exact
    static __device__ __forceinline__ float get(const u32x4& v, int c)
    {
        uint32_t w = v[c >> 1];
        return sr_u2f((c & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    static __device__ __forceinline__ u32x4 neg_inf() { return (u32x4)(0xff80ff80u); }
};

__device__ __forceinline__ bool mask_bit(const uint32_t* m, int e) { return ((m[e >> 5] >> (e & 31)) & 1u) != 0u; }

// ---- bitonic sort, descending, of 3-word keys held in registers -----------------------------------
// Element i lives in thread (i mod 512), register (i div 512).  Strides of 512 and more pair registers
// of one thread, strides below 64 pair lanes of one wave (shuffles), only the strides in between go
// through LDS.  n_pow2 <= 2048.  Keys are compared as (hi, mid, lo).
__device__ __forceinline__ bool key3_less(uint32_t ah, uint32_t am, uint32_t al, uint32_t bh, uint32_t bm, uint32_t bl)
{
    return ah < bh || (ah == bh && (am < bm || (am == bm && al < bl)));
}

template <bool kThree>
__device__ __forceinline__ void block_bitonic_sort_desc(uint32_t (&hi)[kSortRegs], uint32_t (&mid)[kSortRegs],
                                                        uint32_t (&lo)[kSortRegs], int n_pow2, TopkSmem& sm)
{
    const int tid = threadIdx.x;
    auto less = [&](uint32_t ah, uint32_t am, uint32_t al, uint32_t bh, uint32_t bm, uint32_t bl) -> bool {
        if (kThree) return key3_less(ah, am, al, bh, bm, bl);
        return ah < bh || (ah == bh && al < bl);
    };
    auto cx = [&](int r0, int r1, int k2) {  // compare-exchange two registers of this thread (r0 < r1)
        const bool desc = (((r0 * kThreads + tid) & k2) == 0);
        const bool l = less(hi[r0], mid[r0], lo[r0], hi[r1], mid[r1], lo[r1]);
        if (l == desc) {
            uint32_t t;
            t = hi[r0]; hi[r0] = hi[r1]; hi[r1] = t;
            if (kThree) { t = mid[r0]; mid[r0] = mid[r1]; mid[r1] = t; }
            t = lo[r0]; lo[r0] = lo[r1]; lo[r1] = t;
        }
    };
    const int regs = (n_pow2 + kThreads - 1) / kThreads;  // registers that hold real elements
    for (int k2 = 2; k2 <= n_pow2; k2 <<= 1) {
        for (int j2 = k2 >> 1; j2 > 0; j2 >>= 1) {
            if (j2 == 2 * kThreads) {
                cx(0, 2, k2); cx(1, 3, k2);
            } else if (j2 == kThreads) {
                cx(0, 1, k2);
                if (regs > 2) cx(2, 3, k2);
            } else if (j2 >= SR_WAVE) {
                __syncthreads();
#pragma unroll
                for (int r = 0; r < kSortRegs; r++) {
                    if (r < regs) {
                        const int i = r * kThreads + tid;
                        sm.xa[i] = hi[r];
                        if (kThree) sm.xb[i] = mid[r];
                        sm.xc[i] = lo[r];
                    }
                }
                __syncthreads();
#pragma unroll
                for (int r = 0; r < kSortRegs; r++) {
                    const int i = r * kThreads + tid;
                    if (r < regs && i < n_pow2) {
                        const int pi = i ^ j2;
                        const uint32_t ph = sm.xa[pi], pm = kThree ? sm.xb[pi] : 0u, pl = sm.xc[pi];
                        const bool want_max = (((i & k2) == 0) == ((i & j2) == 0));
                        const bool l = less(hi[r], mid[r], lo[r], ph, pm, pl);
                        if (want_max == l) { hi[r] = ph; if (kThree) mid[r] = pm; lo[r] = pl; }
                    }
                }
            } else {
#pragma unroll
                for (int r = 0; r < kSortRegs; r++) {
                    if (r < regs) {
                        const int i = r * kThreads + tid;
                        const uint32_t ph = __shfl_xor(hi[r], j2), pm = kThree ? __shfl_xor(mid[r], j2) : 0u,
                                       pl = __shfl_xor(lo[r], j2);
                        const bool want_max = (((i & k2) == 0) == ((i & j2) == 0));
                        const bool l = less(hi[r], mid[r], lo[r], ph, pm, pl);
                        if (want_max == l) { hi[r] = ph; if (kThree) mid[r] = pm; lo[r] = pl; }
                    }
                }
            }
        }
    }
    __syncthreads();
}

// ---- sample sort, descending, of m (> 128) 3-word keys held in registers ---------------------------
// 63 splitters (a 64-element sample sorted by one wave) cut the keys into 64..65 buckets; every key finds
// its bucket by binary search, is scattered bucket-contiguously, and ranks itself against the few members
// of its own bucket.  Far fewer instructions than a full bitonic network.  The sorted (hi, lo) words end
// up in sm.xa / sm.xc at positions [0, m); sm.vals / idxs / probs are used as the scatter area.
template <bool kThree>
__device__ __forceinline__ void block_sample_sort_desc(const uint32_t (&hi)[kSortRegs], const uint32_t (&mid)[kSortRegs],
                                                       const uint32_t (&lo)[kSortRegs], int m, TopkSmem& sm)
{
    const int tid = threadIdx.x, lane = sr_lane();
    uint32_t* bh = (uint32_t*)sm.vals;
    uint32_t* bm = (uint32_t*)sm.idxs;
    uint32_t* bl = (uint32_t*)sm.probs;
    uint32_t* bcnt = sm.hist;        // [0, 65)
    uint32_t* boff = sm.hist + 128;  // [0, 66)
    uint32_t* sph = sm.hist + 64;    // splitters do not fit hist: kept in xb tail-free slots below
    auto less = [&](uint32_t ah, uint32_t am, uint32_t al, uint32_t b_h, uint32_t b_m, uint32_t b_l) -> bool {
        if (kThree) return key3_less(ah, am, al, b_h, b_m, b_l);
        return ah < b_h || (ah == b_h && al < b_l);
    };
    (void)sph;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortRegs; r++) {
        const int i = r * kThreads + tid;
        if (i < m) { sm.xa[i] = hi[r]; sm.xb[i] = mid[r]; sm.xc[i] = lo[r]; }
    }
    if (tid < 65) bcnt[tid] = 0u;
    __syncthreads();
    // every wave sorts the same 64-element sample (no barrier needed to share the splitters)
    uint32_t sh, smid, sl;
    {
        const int src = (int)(((long long)lane * m) >> 6);
        sh = sm.xa[src]; smid = sm.xb[src]; sl = sm.xc[src];
#pragma unroll
        for (int k2 = 2; k2 <= SR_WAVE; k2 <<= 1) {
#pragma unroll
            for (int j2 = k2 >> 1; j2 > 0; j2 >>= 1) {
                const uint32_t ph = __shfl_xor(sh, j2), pm = kThree ? __shfl_xor(smid, j2) : 0u, pl = __shfl_xor(sl, j2);
                const bool want_max = (((lane & k2) == 0) == ((lane & j2) == 0));
                const bool l = less(sh, smid, sl, ph, pm, pl);
                if (want_max == l) { sh = ph; smid = pm; sl = pl; }
            }
        }
    }
    // lane j now holds the j-th largest sample element; lanes 0..62 are the splitters
    int bucket[kSortRegs], slot[kSortRegs];
#pragma unroll
    for (int r = 0; r < kSortRegs; r++) {
        const int i = r * kThreads + tid;
        bucket[r] = 0; slot[r] = 0;
        // number of splitters strictly greater than the key (binary search over lanes 0..62)
        int lo_b = 0, hi_b = 63;
#pragma unroll
        for (int it = 0; it < 6; it++) {
            const int midb = (lo_b + hi_b) >> 1;
            const uint32_t ph = __shfl(sh, midb), pm = kThree ? __shfl(smid, midb) : 0u, pl = __shfl(sl, midb);
            const bool splitter_greater = less(hi[r], mid[r], lo[r], ph, pm, pl);
            if (lo_b < hi_b) { if (splitter_greater) lo_b = midb + 1; else hi_b = midb; }
        }
        if (i < m) {
            bucket[r] = lo_b;
            slot[r] = (int)atomicAdd(&bcnt[lo_b], 1u);
        }
    }
    __syncthreads();
    if (tid < SR_WAVE) {
        // exclusive scan of the 65 bucket counts (lane l owns bucket l; bucket 64 follows the total)
        const int c = (int)bcnt[lane];
        const int incl = sr_wave_incl_scan_i32(c);
        boff[lane] = (uint32_t)(incl - c);
        if (lane == SR_WAVE - 1) { boff[64] = (uint32_t)incl; boff[65] = (uint32_t)incl + bcnt[64]; }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortRegs; r++) {
        const int i = r * kThreads + tid;
        if (i < m) {
            const int p = (int)boff[bucket[r]] + slot[r];
            bh[p] = hi[r]; if (kThree) bm[p] = mid[r]; bl[p] = lo[r];
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortRegs; r++) {
        const int i = r * kThreads + tid;
        if (i < m) {
            const int b0 = (int)boff[bucket[r]], b1 = (int)boff[bucket[r] + 1];
            int rank = b0;
            for (int p = b0; p < b1; p++)
                rank += less(hi[r], mid[r], lo[r], bh[p], kThree ? bm[p] : 0u, bl[p]) ? 1 : 0;
            sm.xa[rank] = hi[r];
            sm.xc[rank] = lo[r];
        }
    }
    __syncthreads();
}

__device__ __forceinline__ int next_pow2(int n)
{
    int p = 1;
    while (p < n) p <<= 1;
    return p;
}

// block-wide reductions through sm.red (all threads must call)
__device__ __forceinline__ int block_sum_i32(int v, TopkSmem& sm)
{
    v = sr_wave_sum_i32(v);
    __syncthreads();
    if (sr_lane() == 0) sm.red[sr_wave_id()] = (uint32_t)v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int w = 0; w < kWaves; w++) t += (int)sm.red[w];
    return t;
}
__device__ __forceinline__ uint32_t block_max_u32(uint32_t v, TopkSmem& sm)
{
    v = sr_wave_max_u32(v);
    __syncthreads();
    if (sr_lane() == 0) sm.red[sr_wave_id()] = v;
    __syncthreads();
    uint32_t t = 0u;
#pragma unroll
    for (int w = 0; w < kWaves; w++) t = sm.red[w] > t ? sm.red[w] : t;
    return t;
}
__device__ __forceinline__ int block_min_i32(int v, TopkSmem& sm)
{
    v = sr_wave_min_i32(v);
    __syncthreads();
    if (sr_lane() == 0) sm.red[sr_wave_id()] = (uint32_t)v;
    __syncthreads();
    int t = 0x7fffffff;
#pragma unroll
    for (int w = 0; w < kWaves; w++) t = min(t, (int)sm.red[w]);
    return t;
}

#define SR_INL __attribute__((always_inline))

// The largest key, to its upper 16 bits, for which `enough` holds (0: none); `enough` must hold for every key below one
// for which it holds, must not hold above `kmax`, and must be the same in every lane.  The answer nearly always has the
// sign and exponent of kmax or one of the exponents just below (a peaked row's k-th largest lies two below its
// largest): those nine bits are tried as a whole, from kmax's downwards, four times at most, and then the seven bits
// below them one by one -- eight to eleven tries instead of sixteen; all sixteen bits one by one when none of the four
// holds.
template <typename Enough>
__device__ __forceinline__ uint32_t largest_key16(uint32_t kmax, Enough enough)
{
    uint32_t K = kmax & 0xff800000u;  // nothing lies at or above the next exponent's first key
    bool head = false;
#pragma unroll 1
    for (int t = 0; t < 4 && !head; t++) {
        if (enough(K)) head = true;
        else if (K >= 0x00800000u) K -= 0x00800000u;
        else break;
    }
    if (head) {
#pragma unroll 1
        for (int bit = 22; bit >= 16; bit--) {
            const uint32_t cnd = K | (1u << bit);
            if (enough(cnd)) K = cnd;
        }
    } else {
        K = 0u;
#pragma unroll 1
        for (int bit = 31; bit >= 16; bit--) {
            const uint32_t cnd = K | (1u << bit);
            if (enough(cnd)) K = cnd;
        }
    }
    return K;
}

// ---- the row tail ----------------------------------------------------------------------------------
// Called by every thread of the tail workgroup of a row once all chunks of the row have been counted in.
// slot = position of the row in this launch.
// What a worker that streams all chunks of its own row keeps of them in registers instead of writing it out: per
// chunk (at most kKeptChunks) the thread's four group maxima, second maxima and packed positions.  The waves' shares
// of the row's bound and their largest kept elements lie in sm.hist, two words per (chunk, wave).
constexpr int kKeptChunks = 4;
struct KeptGroups {
    float4 g1[kKeptChunks], g2[kKeptChunks];
    uint32_t gp[kKeptChunks];
};
// ... and what it fetches of its row's history before it starts to stream: the thread's history ids with their
// counts, and their (masked) logits
struct KeptHistory {
    SrEdit hee[kHistRegs];
    float hx[kHistRegs];
};
// The masked logit of one token id of a row.
__device__ __forceinline__ float row_logit(const SrTopkArgs& a, int row, const SrRow& rd, int id)
{
    const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * (a.dtype == 1 ? 2 : 4);
    float x = (a.dtype == 1) ? sr_bf16_to_f32(((const uint16_t*)rowp)[id]) : ((const float*)rowp)[id];
    if (rd.mask_row >= 0 && !mask_bit(a.mask + (size_t)rd.mask_row * a.mask_stride, id)) x = SR_NEG_INF;
    return x;
}
// A row descriptor read through the constant address space: one scalar load for the whole workgroup, in nobody's way
// (the descriptors were written before the launch).
__device__ __forceinline__ SrRow load_row_uniform(const SrRow* p)
{
    static_assert(sizeof(SrRow) == 64, "four 16-byte loads");
    typedef int __attribute__((ext_vector_type(4))) i32x4;
    typedef const i32x4 __attribute__((address_space(4))) const_i32x4;
    const const_i32x4* q = (const const_i32x4*)(uintptr_t)p;
    union { SrRow r; i32x4 v[4]; } u;
    u.v[0] = q[0]; u.v[1] = q[1]; u.v[2] = q[2]; u.v[3] = q[3];
    return u.r;
}
// Whether the row tail holds the row's history ids in registers (penalties that only lower, few enough ids).
__device__ __forceinline__ bool row_history_in_registers(const SrRow& rd)
{
    const bool use_edits = (rd.flags & kRowHasPenalty) != 0u && rd.edit_cnt > 0;
    return use_edits && (rd.flags & kRowHistExcl) != 0u && rd.path == SR_PATH_TOPK && rd.edit_cnt <= kHistRegs * kThreads;
}

template <int EPV, int kVec, bool kKept, bool kShort, typename Early, typename Late>
__device__ __forceinline__ int build_candidates(const SrTopkArgs& a, int slot, int row, const SrRow& rd, bool want_bins,
                                                bool force_exact, float inv_temp, BinMap* map_out,
                                                float* bound_out, bool* binned, const KeptGroups& kept, Early&& early,
                                                Late&& late, TopkSmem& sm);

// force_exact: the chunk results of the row are not used, the candidates come from the logits themselves (what a row
// whose candidates overflow the lists falls back to, and a row whose chunks were not handed over in time).
// kShort: the launch holds no row that asks for more than kShortSel entries; the tail then carries the two steps that
// pay for such rows only (a closer bound from the waves' pairs, ranking a short list by counting).  They are compiled
// into launches of their own because their mere presence costs the long tails of other launches 0.6 us.
template <int EPV, int kVec, bool kKept, bool kShort>
__device__ __forceinline__ void topk_row_tail(const SrTopkArgs& a, int slot, int row, const SrRow& rd, bool force_exact,
                                              const KeptGroups& kept, const KeptHistory& kept_hist, TopkSmem& sm)
{
    const int tid = threadIdx.x;
    const unsigned long long* cand = a.cand + (size_t)slot * kRowCap;
    const uint32_t out_flag = (rd.path == SR_PATH_TOPK) ? SR_KFLAG_TOPK : SR_KFLAG_GREEDY;
    const int sel = rd.sel;
    auto give_up = [&](uint32_t extra, int token) SR_INL {
        if (tid == 0) {
            a.out_tokens[row] = token;
            if (a.out_flags) a.out_flags[row] = out_flag | extra;
        }
    };
    const SrEdit* ed = a.edits + rd.edit_off;
    const bool use_edits = (rd.flags & kRowHasPenalty) != 0u && rd.edit_cnt > 0;
    const bool excl = use_edits && (rd.flags & kRowHistExcl) != 0u;  // the scan skipped the history ids
    const int ne = use_edits ? rd.edit_cnt : 0;
    const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * (a.dtype == 1 ? 2 : 4);
    const uint32_t* mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
    auto hist_logit = [&](int id) SR_INL -> float {  // the masked logit of one token id
        float x = (a.dtype == 1) ? sr_bf16_to_f32(((const uint16_t*)rowp)[id]) : ((const float*)rowp)[id];
        if (mrow && !mask_bit(mrow, id)) x = SR_NEG_INF;
        return x;
    };

    // The history ids and their logits are fetched behind the candidate builder's own loads, so that neither
    // waits for the other.
    const bool hist_regs = row_history_in_registers(rd);
    SrEdit hee[kHistRegs];
    float hx[kHistRegs];
#pragma unroll
    for (int r = 0; r < kHistRegs; r++) {
        if constexpr (kKept) { hee[r] = kept_hist.hee[r]; hx[r] = kept_hist.hx[r]; }
        else { hee[r] = SrEdit{}; hx[r] = SR_NEG_INF; }
    }
    const float inv_temp = rd.temperature == 1.0f ? 1.0f : __fdiv_rn(1.0f, rd.temperature);
    // the row's uniform is asked for now: at the draw, the last step of the chain, it would be waited for
    const float u_row = rd.path == SR_PATH_TOPK ? __double2float_rn(a.uniforms[(size_t)row * a.uniforms_per_row]) : 0.0f;
    // rows without penalties that may raise a logit have their candidates binned while they are collected
    const bool want_bins = rd.path == SR_PATH_TOPK && (!use_edits || hist_regs);
    bool binned = false;
    if (tid == 0) sm.bcast[4] = 0u;  // the short list's count of history entries (the barriers of the next call publish it)
    BinMap map0;
    float bound0 = 0.0f;
    const int n_c = build_candidates<EPV, kVec, kKept, kShort>(
        a, slot, row, rd, want_bins, force_exact, inv_temp, &map0, &bound0, &binned, kept,
        [&]() SR_INL {
            if constexpr (!(kKept)) {
#pragma unroll
                for (int r = 0; r < kHistRegs; r++) {
                    const int e = r * kThreads + tid;
                    if (hist_regs && e < ne) hee[r] = ed[e];
                }
            }
        },
        [&]() SR_INL {
            if constexpr (!(kKept)) {
#pragma unroll
                for (int r = 0; r < kHistRegs; r++) {
                    const int e = r * kThreads + tid;
                    if (hist_regs && e < ne) hx[r] = hist_logit(hee[r].id);
                }
            }
        },
        sm);
    if (sel > kSelMax || n_c < 0 || n_c > kRowCap) { give_up(SR_KFLAG_UNSUPPORTED, -1); return; }

    SR_PROF(a, 11);
    const int nr = (n_c + kThreads - 1) / kThreads;  // register slots that can hold a candidate
    uint32_t kreg[kCandRegs];                         // 0 = no candidate in this slot
    int kid[kCandRegs];
    auto load_cands = [&]() SR_INL {
#pragma unroll
        for (int r = 0; r < kCandRegs; r++) {
            kreg[r] = 0u;
            kid[r] = 0;
            if (r >= nr) continue;
            const int g = r * kThreads + tid;
            if (g < n_c) {
                if (g < kSelMax) {  // the first candidates lie in LDS, only an unusually long list continues in memory
                    kreg[r] = sr_okey(sm.vals[g]);
                    kid[r] = sm.idxs[g];
                } else {
                    const unsigned long long cv = sr_load_agent(&cand[g]);
                    kreg[r] = sr_okey(sr_u2f((uint32_t)(cv >> 32)));
                    kid[r] = (int)(uint32_t)cv;
                }
            }
        }
        __syncthreads();  // sm.vals / sm.idxs may be reused from here on
    };
    if (!binned) load_cands();  // binned candidates stay in their list until they are laid out by bins
    auto cand_id = [&](int r) SR_INL -> int { return kid[r]; };
    SR_PROF(a, 12);
    auto each_key = [&](auto&& body) SR_INL {
#pragma unroll
        for (int r = 0; r < kCandRegs; r++)
            if (r < nr) body(kreg[r]);
    };

    if (rd.path == SR_PATH_GREEDY || rd.path == SR_PATH_GREEDY_PEN) {
        // best candidate: highest key, lowest index among its ties.  With penalties the candidates are
        // the tokens outside the history (GreedyWithHistoryPenalties, Sampler.cs:421-437: only history ids
        // change value), and the adjusted history ids compete with the best of them.
        uint32_t kmax = 0u;
        each_key([&](uint32_t k) { kmax = k > kmax ? k : kmax; });
        kmax = block_max_u32(kmax, sm);
        unsigned long long best = 0ull;
#pragma unroll
        for (int r = 0; r < kCandRegs; r++)
            if (r < nr && kreg[r] == kmax && kreg[r] != 0u) {
                unsigned long long cmp = ((unsigned long long)kreg[r] << 32) | (unsigned long long)(0xffffffffu - (uint32_t)cand_id(r));
                best = cmp > best ? cmp : best;
            }
        if (rd.path == SR_PATH_GREEDY_PEN) {
            for (int e = tid; e < ne; e += kThreads) {
                const int id = ed[e].id;
                float x = hist_logit(id);
                if (rd.rep != 1.0f)
                    for (int o = 0; o < ed[e].occ_win; o++) x = x > 0.0f ? __fdiv_rn(x, rd.rep) : __fmul_rn(x, rd.rep);
                if (rd.presence != 0.0f || rd.frequency != 0.0f)
                    x = __fsub_rn(x, __fadd_rn(rd.presence, __fmul_rn(rd.frequency, (float)ed[e].occ_all)));
                if (sr_f2u(x) != 0xff800000u && x == x) {
                    unsigned long long cmp = ((unsigned long long)sr_okey(x) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)id);
                    best = cmp > best ? cmp : best;
                }
            }
        }
        best = sr_wave_max_u64(best);
        __syncthreads();
        if (sr_lane() == 0) ((unsigned long long*)sm.vals)[sr_wave_id()] = best;
        __syncthreads();
        if (tid == 0) {
            for (int w = 0; w < kWaves; w++) {
                unsigned long long cmp = ((unsigned long long*)sm.vals)[w];
                best = cmp > best ? cmp : best;
            }
            // nothing finite at all: every (adjusted) logit is -inf and the first index wins
            a.out_tokens[row] = best ? (int)(0xffffffffu - (uint32_t)(best & 0xffffffffull)) : 0;
            if (a.out_flags) a.out_flags[row] = out_flag | (best ? 0u : SR_KFLAG_DEGENERATE);
        }
        return;
    }

    // ---- SampleTopK (Sampler.cs:216-357) ---------------------------------------------------------
    // exact top-`need` of the candidates by (value desc, index asc): key of the need-th largest, and for
    // its ties the (0xffffffff - index) bound that admits only the lowest indices
    uint32_t tkey = 0u, tidx_key = 0u;
    auto select_top = [&](int need) SR_INL {
        tkey = block_radix_select(each_key, need, sm);
        int c_ge = 0, c_gt = 0;
        each_key([&](uint32_t k) { c_ge += (k != 0u && k >= tkey) ? 1 : 0; c_gt += (k != 0u && k > tkey) ? 1 : 0; });
        const int m_ge = block_sum_i32(c_ge, sm);
        if (m_ge > need) {
            const int m_gt = block_sum_i32(c_gt, sm);
            uint32_t tie_key[kCandRegs];
#pragma unroll
            for (int r = 0; r < kCandRegs; r++)
                tie_key[r] = (r < nr && kreg[r] != 0u && kreg[r] == tkey) ? 0xffffffffu - (uint32_t)cand_id(r) : 0u;
            auto each_tie = [&](auto&& body) SR_INL {
#pragma unroll
                for (int r = 0; r < kCandRegs; r++)
                    if (r < nr) body(tie_key[r]);
            };
            tidx_key = block_radix_select(each_tie, need - m_gt, sm);
        }
    };
    auto in_set = [&](int r) SR_INL -> bool {
        if (kreg[r] == 0u || kreg[r] < tkey) return false;
        if (kreg[r] > tkey || tidx_key == 0u) return true;
        return (0xffffffffu - (uint32_t)cand_id(r)) >= tidx_key;
    };

    float mx;
    BinMap bmap;  // its origin: mx, or the largest kept element outside the history
    // Candidates whose e = expf(v / T - max) is below 2^-26 are dropped before the sort: with e_0 = 1
    // they change neither running sum (they are under half an ulp of a sum >= 1, and of a cumulative
    // probability >= probs[0]) and the draw can never stop on them, so the result is bit-identical.
    // x < -18.1 implies e < 1.4e-8 < 2^-26.
    auto alive_key = [&](uint32_t key) SR_INL -> bool {
        const float x = __fsub_rn(__fmul_rn(sr_okey_inv(key), inv_temp), mx);
        return key != 0u && !(x < -18.1f);
    };
    // sort keys: (value after penalties, value before, ~index) descending -- the reference's selection
    // order (value desc, index asc) followed by its stable re-sort after penalties, in one sort
    uint32_t hi[kSortRegs], mid[kSortRegs], lo[kSortRegs];
    int m2;          // live entries (at most top_k of them are used)
    int sort_n = 0;  // entries handed to the sort
    bool ranked = false;  // sm.vals / sm.idxs already hold the k first entries
    bool placed = false;  // ... laid out from the binned candidate list: the maximum is the first ranked entry
    bool exact_bins = false;  // ... one bin per distinct value: entries of a bin stand in no order (see BinMap::exact)

    if (use_edits && !excl) {
        // ---- penalties that may raise a logit: the reference's literal top-(k + history length) set ------
        if (n_c == 0) { give_up(SR_KFLAG_DEGENERATE, 0); return; }  // Sampler.cs:254-255: Greedy(raw) = index 0
        if (ne > kSelMax) { give_up(SR_KFLAG_UNSUPPORTED, -1); return; }
        int* edit_ids = sm.idxs;  // history ids of the row, staged for binary search
        for (int e = tid; e < ne; e += kThreads) edit_ids[e] = ed[e].id;
        auto find_edit = [&](int id) SR_INL -> int {
            int lo_e = 0, hi_e = ne;
            while (lo_e < hi_e) {
                int mid_e = (lo_e + hi_e) >> 1;
                if (edit_ids[mid_e] < id) lo_e = mid_e + 1; else hi_e = mid_e;
            }
            return (lo_e < ne && edit_ids[lo_e] == id) ? lo_e : -1;
        };
        if (n_c > sel) select_top(sel);
        SR_PROF(a, 5);
        int mine = 0;
#pragma unroll
        for (int r = 0; r < kCandRegs; r++)
            if (r < nr) mine += in_set(r) ? 1 : 0;
        int m;
        int pos = block_excl_scan(mine, &m, sm);
        if (mine > 0) {
#pragma unroll
            for (int r = 0; r < kCandRegs; r++)
                if (r < nr && in_set(r) && pos < kSelMax) {
                    sm.xa[pos] = kreg[r];
                    sm.xb[pos] = (uint32_t)cand_id(r);
                    pos++;
                }
        }
        __syncthreads();  // also orders the staging of edit_ids
        if (m > kSelMax) { give_up(SR_KFLAG_UNSUPPORTED, -1); return; }  // guard; m <= sel
        SR_PROF(a, 6);
#pragma unroll
        for (int r = 0; r < kSortRegs; r++) {
            const int i = r * kThreads + tid;
            hi[r] = mid[r] = lo[r] = 0u;
            if (i < m) {
                const uint32_t key = sm.xa[i];
                const int id = (int)sm.xb[i];
                uint32_t nkey = key;
                // Sampler.cs:261-287: pen = pow(rep, occWindow) once; presence/frequency over the whole history
                const int e = find_edit(id);
                if (e >= 0) {
                    const SrEdit ee = ed[e];
                    if (ee.occ_all > 0) {
                        float v = sr_okey_inv(key);
                        if (rd.rep != 1.0f && ee.occ_win > 0) v = v > 0.0f ? __fdiv_rn(v, ee.pen) : __fmul_rn(v, ee.pen);
                        v = __fsub_rn(v, __fadd_rn(rd.presence, __fmul_rn(rd.frequency, (float)ee.occ_all)));
                        nkey = sr_okey(v);
                    }
                }
                hi[r] = nkey; mid[r] = key; lo[r] = 0xffffffffu - (uint32_t)id;
            }
        }
        SR_PROF(a, 7);
        uint32_t lmaxk = 0u;
#pragma unroll
        for (int r = 0; r < kSortRegs; r++) lmaxk = hi[r] > lmaxk ? hi[r] : lmaxk;
        const uint32_t kmaxn = block_max_u32(lmaxk, sm);
        mx = __fmul_rn(sr_okey_inv(kmaxn), inv_temp);
        int nlive = 0;
        bool alive[kSortRegs];
#pragma unroll
        for (int r = 0; r < kSortRegs; r++) {
            const int i = r * kThreads + tid;
            alive[r] = (i < m) && alive_key(hi[r]);
            nlive += alive[r] ? 1 : 0;
        }
        int lpos = block_excl_scan(nlive, &m2, sm);
        if (m2 < m) {
            // compact the live candidates (all threads have their elements in registers by now)
#pragma unroll
            for (int r = 0; r < kSortRegs; r++)
                if (alive[r]) { sm.xa[lpos] = hi[r]; sm.xb[lpos] = mid[r]; sm.xc[lpos] = lo[r]; lpos++; }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < kSortRegs; r++) {
                const int i = r * kThreads + tid;
                hi[r] = (i < m2) ? sm.xa[i] : 0u;
                mid[r] = (i < m2) ? sm.xb[i] : 0u;
                lo[r] = (i < m2) ? sm.xc[i] : 0u;
            }
        }
        sort_n = m2;
    } else {
        // ---- no penalties, or penalties that only lower: candidates outside the history + the history ids --
        if (ne > kHistRegs * kThreads) { give_up(SR_KFLAG_UNSUPPORTED, -1); return; }
        uint32_t hadj[kHistRegs], hraw[kHistRegs];
#pragma unroll
        for (int r = 0; r < kHistRegs; r++) {
            hadj[r] = hraw[r] = 0u;
            const int e = r * kThreads + tid;
            if (e < ne) {
                const SrEdit ee = hee[r];
                const float x = hx[r];
                // -inf never enters the reference's selection (Sampler.cs:240-249)
                if (x == x && sr_f2u(x) != 0xff800000u) {
                    float v = x;
                    // Sampler.cs:261-287: pen = pow(rep, occWindow) once; presence/frequency over the whole history
                    if (ee.occ_all > 0) {
                        if (rd.rep != 1.0f && ee.occ_win > 0) v = v > 0.0f ? __fdiv_rn(v, ee.pen) : __fmul_rn(v, ee.pen);
                        v = __fsub_rn(v, __fadd_rn(rd.presence, __fmul_rn(rd.frequency, (float)ee.occ_all)));
                    }
                    hraw[r] = sr_okey(x);
                    hadj[r] = sr_okey(v);
                }
            }
        }
        SR_PROF(a, 5);
        // How far an entry lies below the bins' origin, in 1/56 of a log-unit: -1 = absent or dropped, else
        // 0..1023.  Never increasing with the key, so "bin <= b" is a prefix of the descending order.
        auto bin_of = [&](uint32_t key) SR_INL -> int {
            if (key == 0u) return -1;
            const float xs = __fmul_rn(sr_okey_inv(key), inv_temp);
            if (__fsub_rn(xs, bmap.mx) < -18.1f) return -1;
            return bmap.of(xs);
        };
        // the bin of an entry that was kept (binned candidates are never dropped once they are on the list)
        auto bin_kept = [&](uint32_t key) SR_INL -> int {
            return bmap.of(__fmul_rn(sr_okey_inv(key), inv_temp));
        };
        // A short list (top-k of a few dozen) is ranked by counting: every entry against every other, four threads to
        // an entry.  No histogram, no layout by bins.  A history id whose adjusted logit is below the candidates' bound
        // stays out (it has at least top_k candidates above it, or lies too far below the maximum to matter); entries
        // too small to matter are not dropped here: they rank last and change no sum (see above), as in the
        // reference, which keeps them too.
        bool short_list = false;
        if (kShort && n_c <= kShortList && ne <= kThreads) {
            const uint32_t bound_key = sr_okey(bound0);
            // (xa .. xc are free and the counter is zero: see where the candidates are built)
            if (tid < n_c) {  // (candidates of a list this short: the first register slot, or the head of the list in LDS)
                const uint32_t key = binned ? sr_okey(sm.vals[tid]) : kreg[0];
                const int id = binned ? sm.idxs[tid] : kid[0];
                sm.xa[tid] = key;
                sm.xb[tid] = key;
                sm.xc[tid] = 0xffffffffu - (uint32_t)id;
            }
            if (hraw[0] != 0u && hadj[0] >= bound_key) {  // (this thread's history id, if its logit is finite)
                const int pos = n_c + (int)atomicAdd(&sm.bcast[4], 1u);
                sm.xa[pos] = hadj[0];
                sm.xb[pos] = hraw[0];
                sm.xc[pos] = 0xffffffffu - (uint32_t)hee[0].id;
            }
            __syncthreads();
            const int n_all = n_c + (int)sm.bcast[4];
            short_list = n_all <= kShortList;
            if (!short_list) __syncthreads();  // (every thread has read the count: the other way uses the word again)
            // no finite logit in the row: Greedy over the raw row = index 0 (Sampler.cs:254-255, :442-446)
            if (n_all == 0) { give_up(SR_KFLAG_DEGENERATE, 0); return; }
            if (short_list) {
                const int kk = min(rd.top_k, n_all);
                // four threads to an entry, eight when the list is at most half as long
                static_assert(kShortList * 4 <= kThreads, "four threads to an entry");
                const bool eight = n_all * 8 <= kThreads;
                const int e = eight ? tid >> 3 : tid >> 2, part = eight ? tid & 7 : tid & 3, parts = eight ? 8 : 4;
                uint32_t mh = 0u, mm = 0u, ml = 0u;
                int ahead = 0;
                if (e < n_all) {
                    mh = sm.xa[e]; mm = sm.xb[e]; ml = sm.xc[e];
                    for (int j = part; j < n_all; j += parts) ahead += key3_less(mh, mm, ml, sm.xa[j], sm.xb[j], sm.xc[j]) ? 1 : 0;
                }
                ahead += __shfl_xor(ahead, 1);
                ahead += __shfl_xor(ahead, 2);
                if (eight) ahead += __shfl_xor(ahead, 4);
                if (e < n_all && part == 0 && ahead < kk) {
                    sm.vals[ahead] = sr_okey_inv(mh);
                    sm.idxs[ahead] = (int)(0xffffffffu - ml);
                }
                ranked = true;
                placed = true;  // the maximum is the first ranked entry
                m2 = n_all;
                sort_n = n_all;
                SR_PROF(a, 6);
                SR_PROF(a, 7);
            }
        }
        if (!short_list) {
        int bstar = kBins - 1, n_live = 0, n_keep = 0, max_bin = 0;
        // one wave reads the histogram: live entries, the first bin at which the k best are complete, and every bin's
        // first list position (sm.boff); its results go out through sm.bcast[8..11], see scan_results
        auto scan_bins = [&]() SR_INL {
            // (two waves share a SIMD: what every wave does for itself takes twice as long as what one wave does for all)
            if (sr_wave_id() != 0) return;
            // lane l owns bins [l * kBinsPerLane, (l + 1) * kBinsPerLane)
            const int lane = sr_lane();
            const uint32_t* hb = sm.bhist + lane * (kBinsPerLane + 1);
            int tot = 0;
#pragma unroll
            for (int q = 0; q < kBinsPerLane; q++) tot += (int)hb[q];
            const int incl = sr_wave_incl_scan_i32(tot);
            n_live = __shfl(incl, SR_WAVE - 1);
            const int need = min(rd.top_k, n_live);
            const unsigned long long bal = __ballot(incl >= need);
            const int L = bal ? (int)__ffsll((long long)bal) - 1 : SR_WAVE - 1;
            int c = incl - tot, bq = lane * kBinsPerLane + kBinsPerLane - 1, cq = incl;
            bool found = false;
            uint32_t hm = 0u;
#pragma unroll
            for (int q = 0; q < kBinsPerLane; q++) {
                const uint32_t h = hb[q];
                sm.boff[lane * (kBinsPerLane + 1) + q] = (uint32_t)c;
                c += (int)h;
                if (!found) hm = max(hm, h);  // bins up to and including the one that completes the k best
                if (!found && c >= need) { bq = lane * kBinsPerLane + q; cq = c; found = true; }
            }
            bstar = __shfl(bq, L);
            n_keep = __shfl(cq, L);
            // the fullest kept bin bounds the ranking loop below
            if (lane > L) hm = 0u;
            max_bin = (int)sr_wave_max_u32(hm);
            if (lane == 0) { sm.bcast[8] = (uint32_t)bstar; sm.bcast[9] = (uint32_t)n_live; sm.bcast[10] = (uint32_t)n_keep; sm.bcast[11] = (uint32_t)max_bin; }
        };
        // (one wave scans; the others take its results behind the barrier that follows)
        auto scan_results = [&]() SR_INL {
            bstar = (int)sm.bcast[8]; n_live = (int)sm.bcast[9]; n_keep = (int)sm.bcast[10]; max_bin = (int)sm.bcast[11];
        };
        bool by_bins = true;  // kept entries are laid out bin by bin and ranked inside their bin
        if (binned) {
            // The candidates were counted into the histogram as they were collected; the history ids join them.
            bmap = map0;
            // a history id whose adjusted logit is below the candidates' bound has at least top_k candidates above
            // it, or lies too far below the maximum to matter
            const uint32_t bound_key = sr_okey(bound0);
            // (here and not where the candidates are collected: a thread's few atomics are in flight together, where
            // each candidate handed over waited for the one before it)
            {
                uint32_t* meta_w = (uint32_t*)sm.probs;
                for (int i = tid; i < n_c; i += kThreads) {
                    const int b = (EPV == 8 && bmap.exact) ? bmap.of_raw(sm.vals[i]) : bmap.of(__fmul_rn(sm.vals[i], inv_temp));
                    meta_w[i] = ((uint32_t)b << 16) | atomicAdd(&sm.bhist[bin_word(b)], 1u);
                }
            }
            uint32_t hmeta[kHistRegs];
#pragma unroll
            for (int r = 0; r < kHistRegs; r++) {
                const int b = (hraw[r] != 0u && hadj[r] >= bound_key) ? bin_of(hadj[r]) : -1;
                hmeta[r] = b >= 0 ? (((uint32_t)b << 16) | atomicAdd(&sm.bhist[bin_word(b)], 1u)) : 0xffffffffu;
            }
            __syncthreads();
            scan_bins();
            __syncthreads();  // sm.boff written, the scan's results out
            scan_results();
            // no finite logit in the row: Greedy over the raw row = index 0 (Sampler.cs:254-255, :442-446)
            if (n_live == 0) { give_up(SR_KFLAG_DEGENERATE, 0); return; }
            SR_PROF(a, 6);
            if (n_keep <= kSelMax && max_bin <= ((EPV == 8 && bmap.exact) ? 256 : 96)) {
                const uint32_t* meta = (const uint32_t*)sm.probs;
                for (int i = tid; i < n_c; i += kThreads) {
                    const uint32_t mt = meta[i];
                    const int b = (int)(mt >> 16);
                    if (b <= bstar) {
                        const int pos = (int)(sm.boff[bin_word(b)] + (mt & 0xffffu));
                        const uint32_t key = sr_okey(sm.vals[i]);
                        sm.xa[pos] = key;
                        sm.xb[pos] = key;
                        sm.xc[pos] = 0xffffffffu - (uint32_t)sm.idxs[i];
                    }
                }
#pragma unroll
                for (int r = 0; r < kHistRegs; r++) {
                    const int b = (int)(hmeta[r] >> 16);
                    if (hmeta[r] != 0xffffffffu && b <= bstar) {
                        const int pos = (int)(sm.boff[bin_word(b)] + (hmeta[r] & 0xffffu));
                        sm.xa[pos] = hadj[r];
                        sm.xb[pos] = hraw[r];
                        sm.xc[pos] = 0xffffffffu - (uint32_t)hee[r].id;
                    }
                }
                __syncthreads();
                placed = true;
            } else {
                load_cands();  // a flat or heavily tied row: the general way below
                bmap = BinMap{};
            }
            if constexpr (EPV == 8) exact_bins = placed && bmap.exact;
        }
        if (!placed) {
        uint32_t lmaxk = 0u;
        each_key([&](uint32_t k) { lmaxk = k > lmaxk ? k : lmaxk; });
#pragma unroll
        for (int r = 0; r < kHistRegs; r++) lmaxk = (hraw[r] != 0u && hadj[r] > lmaxk) ? hadj[r] : lmaxk;
        for (int i = tid; i < kBinsPad; i += kThreads) { sm.bhist[i] = 0u; sm.bfill[i] = 0u; }
        if (tid == 0) sm.bcast[4] = 0u;
        const uint32_t kmaxn = block_max_u32(lmaxk, sm);  // its barriers also publish the cleared histogram
        // no finite logit in the row: Greedy over the raw row = index 0 (Sampler.cs:254-255, :442-446)
        if (kmaxn == 0u) { give_up(SR_KFLAG_DEGENERATE, 0); return; }
        mx = __fmul_rn(sr_okey_inv(kmaxn), inv_temp);
        bmap.mx = mx;
#pragma unroll
        for (int r = 0; r < kCandRegs; r++)
            if (r < nr) { const int b = bin_of(kreg[r]); if (b >= 0) atomicAdd(&sm.bhist[bin_word(b)], 1u); }
#pragma unroll
        for (int r = 0; r < kHistRegs; r++) {
            const int b = hraw[r] != 0u ? bin_of(hadj[r]) : -1;
            if (b >= 0) atomicAdd(&sm.bhist[bin_word(b)], 1u);
        }
        __syncthreads();
        scan_bins();
        __syncthreads();
        scan_results();
        if (n_keep > kSelMax) {
            // a flat row: only the k best candidates outside the history can matter
            by_bins = false;
            if (n_c > rd.top_k) select_top(rd.top_k);
            bstar = kBins - 1;
            int mine = 0;
#pragma unroll
            for (int r = 0; r < kCandRegs; r++)
                if (r < nr) mine += (bin_of(kreg[r]) >= 0 && in_set(r)) ? 1 : 0;
#pragma unroll
            for (int r = 0; r < kHistRegs; r++) mine += (hraw[r] != 0u && bin_of(hadj[r]) >= 0) ? 1 : 0;
            n_keep = block_sum_i32(mine, sm);
            if (n_keep > kSelMax) { give_up(SR_KFLAG_UNSUPPORTED, -1); return; }
        } else if (max_bin > 96) {
            by_bins = false;
        }
        __syncthreads();  // boff / bfill written
        SR_PROF(a, 6);
        // gather the kept entries: bin by bin, or in any order when a sort follows
        {
            int mine = 0;
            if (!by_bins) {
#pragma unroll
                for (int r = 0; r < kCandRegs; r++)
                    if (r < nr) { const int b = bin_of(kreg[r]); mine += (b >= 0 && b <= bstar && in_set(r)) ? 1 : 0; }
#pragma unroll
                for (int r = 0; r < kHistRegs; r++) {
                    const int b = hraw[r] != 0u ? bin_of(hadj[r]) : -1;
                    mine += (b >= 0 && b <= bstar) ? 1 : 0;
                }
            }
            int pos_any = (mine > 0) ? (int)atomicAdd(&sm.bcast[4], (uint32_t)mine) : 0;
#pragma unroll
            for (int r = 0; r < kCandRegs; r++)
                if (r < nr) {
                    const int b = bin_of(kreg[r]);
                    if (b >= 0 && b <= bstar && in_set(r)) {
                        const int pos = by_bins ? (int)(sm.boff[bin_word(b)] + atomicAdd(&sm.bfill[bin_word(b)], 1u)) : pos_any++;
                        if (pos < kSelMax) {
                            sm.xa[pos] = kreg[r];
                            sm.xb[pos] = kreg[r];
                            sm.xc[pos] = 0xffffffffu - (uint32_t)cand_id(r);
                        }
                    }
                }
#pragma unroll
            for (int r = 0; r < kHistRegs; r++) {
                const int b = hraw[r] != 0u ? bin_of(hadj[r]) : -1;
                if (b >= 0 && b <= bstar) {
                    const int pos = by_bins ? (int)(sm.boff[bin_word(b)] + atomicAdd(&sm.bfill[bin_word(b)], 1u)) : pos_any++;
                    if (pos < kSelMax) {
                        sm.xa[pos] = hadj[r];
                        sm.xb[pos] = hraw[r];
                        sm.xc[pos] = 0xffffffffu - (uint32_t)hee[r].id;
                    }
                }
            }
        }
        __syncthreads();
        }  // !placed
        m2 = n_live;
        const int ms = by_bins ? min(n_keep, kSelMax) : min((int)sm.bcast[4], kSelMax);
        // the first min(top_k, live) of the kept entries are the first of all live entries
        m2 = min(min(m2, max(rd.top_k, 0)), ms);
        sort_n = ms;
        SR_PROF_VAL(a, 13, n_c);
        SR_PROF_VAL(a, 14, ((unsigned long long)n_live << 32) | (unsigned long long)ms);
        if (by_bins) {
            // bins descend with the key, so an entry's rank is its bin's first position plus the entries of
            // the bin that precede it
            ranked = true;
            const int kk = min(rd.top_k, m2);
            if (EPV == 8 && exact_bins) {
                // every bin holds one value: the layout is the order by value already, and which of a bin's equal
                // entries stands where makes no difference to any sum
                for (int i = tid; i < kk; i += kThreads) {
                    sm.vals[i] = sr_okey_inv(sm.xa[i]);
                    sm.idxs[i] = (int)(0xffffffffu - sm.xc[i]);
                }
            }
            for (int i = tid; i < ((EPV == 8 && exact_bins) ? 0 : ms); i += kThreads) {
                const uint32_t mh = sm.xa[i], mm = sm.xb[i], ml = sm.xc[i];
                const int b = bin_kept(mh);
                const int p0 = (int)sm.boff[bin_word(b)], p1 = p0 + (int)sm.bhist[bin_word(b)];
                int rank = p0;
                // four entries of the bin per step, their twelve words fetched together (an index past the bin's end
                // reads the bin's last entry and does not count)
                for (int j = p0; j < p1; j += 4) {
                    uint32_t eh[4], em[4], el[4];
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int jj = min(j + q, p1 - 1);
                        eh[q] = sm.xa[jj]; em[q] = sm.xb[jj]; el[q] = sm.xc[jj];
                    }
#pragma unroll
                    for (int q = 0; q < 4; q++) rank += (j + q < p1 && key3_less(mh, mm, ml, eh[q], em[q], el[q])) ? 1 : 0;
                }
                if (rank < kk) {
                    sm.vals[rank] = sr_okey_inv(mh);
                    sm.idxs[rank] = (int)(0xffffffffu - ml);
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < kSortRegs; r++) {
                const int i = r * kThreads + tid;
                hi[r] = (i < ms) ? sm.xa[i] : 0u;
                mid[r] = (i < ms) ? sm.xb[i] : 0u;
                lo[r] = (i < ms) ? sm.xc[i] : 0u;
            }
        }
        SR_PROF(a, 7);
        }  // !short_list
    }

    // the k best that are still alive
    const int k = min(rd.top_k, m2);  // everything past m2 is a no-op or does not exist
    if (ranked) {
    } else if (sort_n > 128) {
        if (use_edits) block_sample_sort_desc<true>(hi, mid, lo, sort_n, sm);
        else block_sample_sort_desc<false>(hi, mid, lo, sort_n, sm);
        // sorted (value key, ~index) are in xa / xc; the scatter area (vals / idxs / probs) is free again
        for (int i = tid; i < k; i += kThreads) {
            sm.vals[i] = sr_okey_inv(sm.xa[i]);
            sm.idxs[i] = (int)(0xffffffffu - sm.xc[i]);
        }
    } else {
        if (use_edits) block_bitonic_sort_desc<true>(hi, mid, lo, next_pow2(sort_n < 2 ? 2 : sort_n), sm);
        else block_bitonic_sort_desc<false>(hi, mid, lo, next_pow2(sort_n < 2 ? 2 : sort_n), sm);
#pragma unroll
        for (int r = 0; r < kSortRegs; r++) {
            const int i = r * kThreads + tid;
            if (i < k) {
                sm.vals[i] = sr_okey_inv(hi[r]);
                sm.idxs[i] = (int)(0xffffffffu - lo[r]);
            }
        }
    }
    __syncthreads();
    if (placed) mx = __fmul_rn(sm.vals[0], inv_temp);
    SR_PROF(a, 8);

    // Sampler.cs:297-313: e_t = expf(v_t / T - max), sequential fp32 sum, probs = e * (1 / sum)
    int live = 0;  // one past the last e_t that can still change a sum that is already >= 1
    for (int t = tid; t < k; t += kThreads) {
        const float v = sm.vals[t];
        const float e = sr_expf(__fsub_rn(__fmul_rn(v, inv_temp), mx));
        sm.probs[t] = e;
        if (!(e < 5.9604644775390625e-08f)) live = t + 1;  // 2^-24: below half an ulp of any sum >= 1
    }
    if (tid < 8) sm.probs[k + tid] = 0.0f;
    live = (int)block_max_u32((uint32_t)live, sm);
    // The left-to-right sum of a long list, bit for bit, by one wave: every lane takes kRun consecutive entries, the
    // wave composes their increment functions and replays only the runs in which the sum changes binade -- a few
    // rounds (0.4 us each) instead of a chain of a thousand dependent additions (4 us); a short list is quicker
    // summed by one lane.
    constexpr int kRun = 16;
    constexpr int kSumByOneLane = 384;
    auto load_run = [&](int base, int limit, float (&x)[kRun]) SR_INL {
        const float4* p4 = (const float4*)(sm.probs + base) + sr_lane() * (kRun / 4);
#pragma unroll
        for (int j4 = 0; j4 < kRun / 4; j4++) {
            const int i = base + sr_lane() * kRun + j4 * 4;
            float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (i < limit) v = p4[j4];  // (the array is longer than any list by two such vectors)
            x[j4 * 4 + 0] = v.x;
            x[j4 * 4 + 1] = i + 1 < limit ? v.y : 0.0f;
            x[j4 * 4 + 2] = i + 2 < limit ? v.z : 0.0f;
            x[j4 * 4 + 3] = i + 3 < limit ? v.w : 0.0f;
        }
    };
    // e_0 = expf(0) = 1, so from t = 1 on the running sum is >= 1 and terms below 2^-24 leave it
    // unchanged: stopping at `live` gives the same bits as running to k
    const int n_sum = max(live, 1);
    if (n_sum > kSumByOneLane) {
        if (sr_wave_id() == 0) {
            float sum = 0.0f;
            constexpr int kHead = 32;
            static_assert(kHead % 4 == 0 && kHead <= kSumByOneLane, "whole vectors of a list that is longer");
            {
                // (the sum doubles quickly at first: its first entries are added as a chain, every lane the same one, so
                // that the scan behind them starts in the binade in which most of the list is added)
                const float4* p4 = (const float4*)sm.probs;
                float4 v[kHead / 4];
#pragma unroll
                for (int i = 0; i < kHead / 4; i++) v[i] = p4[i];
#pragma unroll
                for (int i = 0; i < kHead / 4; i++) {
                    sum = __fadd_rn(sum, v[i].x); sum = __fadd_rn(sum, v[i].y);
                    sum = __fadd_rn(sum, v[i].z); sum = __fadd_rn(sum, v[i].w);
                }
            }
            for (int base = kHead; base < n_sum; base += SR_WAVE * kRun) {
                float x[kRun];
                load_run(base, n_sum, x);
                int unused;
                sum = sr_seq_wave<kRun, false>(x, sum, 0.0f, &unused);
            }
            if (sr_lane() == 0) sm.bcast[5] = sr_f2u(sum);
        }
    } else if (tid == 0) {
        float sum = 0.0f;
        const float4* p4 = (const float4*)sm.probs;
        float4 cur = p4[0];
        for (int t = 0; t < n_sum; t += 4) {
            const float4 nxt = p4[(t >> 2) + 1];
            sum = __fadd_rn(sum, cur.x); sum = __fadd_rn(sum, cur.y);
            sum = __fadd_rn(sum, cur.z); sum = __fadd_rn(sum, cur.w);
            cur = nxt;
        }
        sm.bcast[5] = sr_f2u(sum);
    }
    __syncthreads();
    SR_PROF(a, 9);
    const float sum = sr_u2f(sm.bcast[5]);
    const float inv_sum = sum > 0.0f ? __fdiv_rn(1.0f, sum) : 0.0f;
    for (int t = tid; t < k; t += kThreads) sm.probs[t] = __fmul_rn(sm.probs[t], inv_sum);
    __syncthreads();

    // Sampler.cs:315-324 min-p: the first probs[t] < thr bounds the survivors
    int count = k;
    if (rd.min_p > 0.0f) {
        const float thr = __fmul_rn(rd.min_p, sm.probs[0]);
        int first = k;
        for (int t = tid; t < k; t += kThreads)
            if (sm.probs[t] < thr) { first = t; break; }
        count = min(count, block_min_i32(first, sm));
    }
    // Sampler.cs:326-349: running sum; top-p cuts after the first cum >= TopP.  Then the draw (:351-357): the first
    // entry whose running sum reaches r = u * (sum of the kept entries).  One wave runs both searches and nothing is
    // stored in between: the second repeats the additions of the first (same operands, same order, same bits) up to
    // where the draw stops.  A search mostly ends early in the list, so its first kChainFirst entries are walked as
    // one chain of additions (every lane the same one): whole blocks of 32 entries without a look (eight loads in
    // flight, the sums never decrease) until a block's last sum has reached the target, then that block entry by
    // entry.  A search that goes on from there takes the wave's exact scan.
    constexpr int kChainFirst = 32;
    if (sr_wave_id() == 0) {
        const bool use_top_p = rd.top_p < 1.0f && rd.top_p > 0.0f;
        const float top_p = use_top_p ? rd.top_p : __uint_as_float(0x7f800000u);  // +inf: never reached
        const float4* p4 = (const float4*)sm.probs;
        // first t < limit whose running sum is >= target (else -1); *val = that sum, or the sum of all `limit` entries
        auto first_reach = [&](float target, int limit_all, float* val) SR_INL -> int {
            const int limit = min(limit_all, kChainFirst);
            float cum = 0.0f;
            int t = 0;
            while (t + 32 <= limit) {
                float4 v[8];
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = p4[(t >> 2) + i];
                float c = cum;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    c = __fadd_rn(c, v[i].x); c = __fadd_rn(c, v[i].y);
                    c = __fadd_rn(c, v[i].z); c = __fadd_rn(c, v[i].w);
                }
                if (c >= target) break;
                cum = c;
                t += 32;
            }
            for (; t < limit; t += 4) {
                const float4 v = p4[t >> 2];
                const float cx = __fadd_rn(cum, v.x), cy = __fadd_rn(cx, v.y), cz = __fadd_rn(cy, v.z), cw = __fadd_rn(cz, v.w);
                const int left = limit - t;  // entries of this step that exist
                if (cx >= target) { *val = cx; return t; }
                if (left == 1) { *val = cx; return -1; }
                if (cy >= target) { *val = cy; return t + 1; }
                if (left == 2) { *val = cy; return -1; }
                if (cz >= target) { *val = cz; return t + 2; }
                if (left == 3) { *val = cz; return -1; }
                if (cw >= target) { *val = cw; return t + 3; }
                cum = cw;
            }
            for (int base = kChainFirst; base < limit_all; base += SR_WAVE * kRun) {
                float x[kRun];
                load_run(base, limit_all, x);
                int f;
                cum = sr_seq_wave<kRun, true>(x, cum, target, &f);
                if (f >= 0) { *val = cum; return base + f; }
            }
            *val = cum;
            return -1;
        };
        float kept_sum = 0.0f;
        const int hit = first_reach(top_p, count, &kept_sum);
        const int cnt = hit >= 0 ? hit + 1 : count;
        SR_PROF(a, 10);
        const float r = __fmul_rn(u_row, kept_sum);
        float at = 0.0f;
        const int first = first_reach(r, cnt, &at);
        int token = sm.idxs[first >= 0 ? first : 0];
        if (EPV == 8 && exact_bins) {
            // The draw stopped at place t of the order by value; the entries of that value -- all of them, also those
            // that the top-k cut left out -- lie side by side in the laid-out list, in no order.  The reference orders
            // equal values by index (Sampler.cs:245-248): the token is the one with as many smaller indices in its bin
            // as t has places before it in the bin.
            const int t = first >= 0 ? first : 0;
            const int b = bmap.of_raw(sm.vals[t]);
            const int p0 = (int)sm.boff[bin_word(b)], m = (int)sm.bhist[bin_word(b)], j = t - p0;
            for (int e0 = 0; e0 < m; e0 += SR_WAVE) {
                const int e = e0 + sr_lane();
                const uint32_t mine = e < m ? sm.xc[p0 + e] : 0u;  // ~index: a smaller index is a larger word
                int before = 0;
                for (int q = 0; q < m; q++) before += sm.xc[p0 + q] > mine ? 1 : 0;
                const unsigned long long is = __ballot(e < m && before == j);
                if (is != 0ull) token = (int)(0xffffffffu - (uint32_t)__shfl((int)mine, (int)__ffsll((long long)is) - 1));
            }
        }
        if (sr_lane() == 0) {
            a.out_tokens[row] = token;
            if (a.out_flags) {
                // SR_OUT_AMBIGUOUS (behind the token, for callers that ask for flags): the draw, the top-p cut or the
                // min-p cut lies on its boundary -- the entries on either side of the min-p cut (the list descends) on
                // the threshold, the running sum at the top-p cut or at the draw barely past its target, or the sum
                // before it barely short of it
                const float thr = __fmul_rn(rd.min_p, sm.probs[0]);
                bool amb = rd.min_p > 0.0f && ((count > 0 && sr_near(sm.probs[count - 1], thr)) || (count < k && sr_near(sm.probs[count], thr)));
                if (use_top_p) amb = amb || (hit >= 0 ? sr_stop_near(kept_sum, sm.probs[hit], top_p) : sr_near(kept_sum, top_p));
                amb = amb || (first >= 0 ? sr_stop_near(at, sm.probs[first], r) : sr_near(at, r));
                a.out_flags[row] = out_flag | (amb ? SR_KFLAG_AMBIGUOUS : 0u);
            }
        }
    }
}


// ---- candidates of a row from its group maxima ---------------------------------------------------------
// The chunk workgroups left, per thread and chunk, the maxima of four disjoint groups of the row's elements.
// Any value with at least sel group maxima at or above it is a lower bound on the row's sel-th largest element,
// so only the groups at or above it can hold one of the sel largest: their elements are fetched again (a few
// KB, from L2 / memory-side cache) and those at or above the bound become the row's candidates -- the first
// SR_TK_SEL_MAX in sm.vals / sm.idxs, the rest of an unusually long list in a.cand.  Returns the number of
// candidates, or -1 when the row cannot be handled.  Called by every thread of the tail workgroup; the two
// hooks let the caller issue loads of its own behind the group maxima's (early) and after the first wait (late).
// With want_bins the tail's histogram (sm.bhist) is cleared and the map of its bins is made (the bins run from the
// row's largest kept element down to the bound, see BinMap); the caller then counts the candidates into it, each
// remembering its bin and its arrival number inside the bin (sm.probs, as integers), and lays them out bin by bin.
// *binned tells whether the list is fit for that (few chunks, a short enough list, a finite maximum); *map_out is
// the map.
// force_exact, and any row whose candidates overflow the lists: the row's sel-th largest kept element is found by a
// radix select over the logits themselves, and the candidates are exactly the sel largest in (value desc, index asc)
// order.  Slow (several passes over the row), exact for any data, and independent of the chunk results.
template <int EPV, int kVec, bool kKept, bool kShort, typename Early, typename Late>
__device__ __forceinline__ int build_candidates(const SrTopkArgs& a, int slot, int row, const SrRow& rd, bool want_bins,
                                                bool force_exact, float inv_temp, BinMap* map_out,
                                                float* bound_out, bool* binned, const KeptGroups& kept, Early&& early,
                                                Late&& late, TopkSmem& sm)
{
    *binned = false;
    *map_out = BinMap{};
    *bound_out = -3.402823466e38f;
    using VO = VecOps<EPV>;
    constexpr int ES = (EPV == 4) ? 4 : 2;
    constexpr int kGV = (kVec + SR_TK_GROUPS - 1) / SR_TK_GROUPS;  // vectors per group
    constexpr int kGmRegs = 4;                                     // chunks whose maxima a thread keeps in registers
    // (group, vector) items a thread fetches at once.  One: batches of four and eight, whose loads are in flight together,
    // measured slower by 0.1 - 0.4 us per launch at 256 rows (the machinery around a batch costs more than the second
    // and third trip to memory that it saves a tail whose list has more than 512 items)
    constexpr int kBatch = 1;
    const int tid = threadIdx.x, lane = sr_lane(), S = a.chunks, sel = rd.sel;
    const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
    const int mis = (int)(((uintptr_t)rowp & 15u) / ES);
    const int nvt = (a.vocab + mis + EPV - 1) / EPV;
    const u32x4* wp = (const u32x4*)(rowp - (size_t)mis * ES);
    const uint32_t* keep32 = a.scan_mask + (size_t)rd.scan_row * (size_t)a.scan_stride;
    // the EPV keep-bits of vector j of thread t of chunk c (they never straddle a word: EPV divides 32)
    auto keep_bits = [&](int c, int j, int t) SR_INL -> uint32_t {
        return (keep32[((size_t)c * kThreads + t) * SR_TK_MASK_WORDS + ((j * EPV) >> 5)] >> ((j * EPV) & 31)) & ((1u << EPV) - 1u);
    };
    const float4* gm = a.gmax + (size_t)slot * S * kThreads + tid;
    unsigned long long* crow = a.cand + (size_t)slot * kRowCap;
    uint32_t* qlist = sm.xa;  // kQCap entries: xa and xb lie back to back
    auto gm_load = [&](int c) SR_INL -> float4 { return gm[(size_t)c * kThreads]; };
    // the element index of the largest element of group g of chunk c: p = (vector inside the group) * EPV + q
    auto idx_of = [&](int c, int g, uint32_t p) SR_INL -> int {
        const int fv = c * a.chunk_vecs + (g + (int)(p / EPV) * SR_TK_GROUPS) * kThreads + tid;
        return fv * EPV + (int)(p % EPV) - mis;
    };
    // wave-aggregated append to a list in LDS: one atomic per wave and call
    auto wave_slot = [&](bool want, uint32_t* counter) SR_INL -> int {
        const unsigned long long bal = __ballot(want);
        if (bal == 0ull) return -1;
        uint32_t base = 0u;
        if (lane == (int)__ffsll((long long)bal) - 1) base = atomicAdd(counter, (uint32_t)__popcll(bal));
        base = __shfl(base, (int)__ffsll((long long)bal) - 1);
        return want ? (int)(base + __builtin_amdgcn_mbcnt_hi((uint32_t)(bal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bal, 0u))) : -1;
    };
    auto append = [&](bool want, float x, int idx) SR_INL {
        const int pos = wave_slot(want, &sm.bcast[12]);
        if (pos >= 0) {
            if (pos < kSelMax) {
                sm.vals[pos] = x;
                sm.idxs[pos] = idx;
            } else if (pos < kRowCap) {
                sr_store_agent(&crow[pos], ((unsigned long long)sr_f2u(x) << 32) | (unsigned long long)(uint32_t)idx);
            }
        }
    };
    // Of the kept elements equal to tx, the first need_eq by index join the candidates: a scan of the row in index
    // order that stops as soon as it has them (equal values rank by ascending index, Sampler.cs:245-248).
    auto take_ties = [&](float tx, int need_eq) SR_INL {
        int emitted = 0;
        for (int f_base = 0; f_base < nvt && emitted < need_eq; f_base += kThreads) {
            const int fv = f_base + tid;
            int ceq = 0;
            bool is_eq[EPV];
#pragma unroll
            for (int q = 0; q < EPV; q++) is_eq[q] = false;
            if (fv < nvt) {
                const u32x4 v = wp[fv];
                const int c = fv / a.chunk_vecs, fl = fv - c * a.chunk_vecs;
                const uint32_t kb = keep_bits(c, fl / kThreads, fl % kThreads);
#pragma unroll
                for (int q = 0; q < EPV; q++) {
                    is_eq[q] = VO::get(v, q) == tx && ((kb >> q) & 1u) != 0u;
                    ceq += is_eq[q] ? 1 : 0;
                }
            }
            int tile_total;
            int rank = emitted + block_excl_scan(ceq, &tile_total, sm);
#pragma unroll
            for (int q = 0; q < EPV; q++) {
                append(is_eq[q] && rank < need_eq, tx, fv * EPV + q - mis);
                rank += is_eq[q] ? 1 : 0;
            }
            emitted += tile_total;
        }
    };
    // The exact candidates of the row, from the logits alone.  Returns their number (at most sel).
    auto exact_row = [&]() SR_INL -> int {
        __syncthreads();
        if (tid == 0) { sm.bcast[12] = 0u; sm.bcast[13] = 0u; }
        // ordered key of every kept finite element, 0 for everything else
        auto each_key = [&](auto&& body) SR_INL {
            for (int f_base = 0; f_base < nvt; f_base += kThreads) {
                const int fv = f_base + tid;
                if (fv < nvt) {
                    const u32x4 v = wp[fv];
                    const int c = fv / a.chunk_vecs, fl = fv - c * a.chunk_vecs;
                    const uint32_t kb = keep_bits(c, fl / kThreads, fl % kThreads);
#pragma unroll
                    for (int q = 0; q < EPV; q++) {
                        const float x = VO::get(v, q);
                        const bool ok = ((kb >> q) & 1u) != 0u && x == x && sr_f2u(x) != 0xff800000u;
                        body(ok ? sr_okey(x) : 0u);
                    }
                }
            }
        };
        // the sel-th largest key; 0 when the row has fewer than sel kept finite elements (all of them are taken)
        const uint32_t tkey = block_radix_select(each_key, sel, sm);
        __syncthreads();
        for (int f_base = 0; f_base < nvt; f_base += kThreads) {
            const int fv = f_base + tid;
            u32x4 v = VO::neg_inf();
            uint32_t kb = 0u;
            if (fv < nvt) {
                v = wp[fv];
                const int c = fv / a.chunk_vecs, fl = fv - c * a.chunk_vecs;
                kb = keep_bits(c, fl / kThreads, fl % kThreads);
            }
#pragma unroll
            for (int q = 0; q < EPV; q++) {
                const float x = VO::get(v, q);
                const bool ok = ((kb >> q) & 1u) != 0u && x == x && sr_f2u(x) != 0xff800000u;
                append(ok && sr_okey(x) > tkey, x, fv * EPV + q - mis);
            }
        }
        __syncthreads();
        const int n_gt = (int)sm.bcast[12];  // fewer than sel
        if (tkey != 0u) take_ties(sr_okey_inv(tkey), sel - n_gt);
        sr_drain_stores();
        __syncthreads();
        const int n = (int)sm.bcast[12];
        __syncthreads();
        return n;
    };
    if (force_exact) {
        early();
        late();
        if (sel > kSelMax || sel < 1) return -1;
        return exact_row();
    }
    if (sel == 1) {
        // one candidate: the row's largest kept element, the first by index among equals -- the largest group
        // maximum, and of the groups that reach it the lowest position of their (first) largest element
        early();
        uint32_t km = 0u;
        auto fold_max = [&](const float4& m) SR_INL {
            km = max(max(max(km, sr_okey(m.x)), max(sr_okey(m.y), sr_okey(m.z))), sr_okey(m.w));
        };
        if constexpr (kKept) {
#pragma unroll
            for (int c = 0; c < kKeptChunks; c++)
                if (c < S) fold_max(kept.g1[c]);
        } else {
            for (int c = 0; c < S; c++) fold_max(gm_load(c));
        }
        late();
        km = block_max_u32(km, sm);
        const bool any = km > kKeyNegInf;
        int best = 0x7fffffff;
        auto fold_best = [&](int c, const float4& m, auto&& gpos_of) SR_INL {
            if (max(max(sr_okey(m.x), sr_okey(m.y)), max(sr_okey(m.z), sr_okey(m.w))) != km) return;
            const uint32_t gp = gpos_of();
            const float m1[4] = {m.x, m.y, m.z, m.w};
#pragma unroll
            for (int g = 0; g < 4; g++)
                if (sr_okey(m1[g]) == km) best = min(best, idx_of(c, g, (gp >> (8 * g)) & 0xffu));
        };
        if constexpr (kKept) {
#pragma unroll
            for (int c = 0; c < kKeptChunks; c++)
                if (c < S && any) fold_best(c, kept.g1[c], [&]() SR_INL { return kept.gp[c]; });
        } else {
            for (int c = 0; c < S && any; c++)
                fold_best(c, gm_load(c), [&]() SR_INL { return a.gpos[((size_t)slot * S + c) * kThreads + tid]; });
        }
        best = block_min_i32(best, sm);
        if (tid == 0 && any) {
            sm.vals[0] = sr_okey_inv(km);
            sm.idxs[0] = best;
        }
        __syncthreads();
        return any ? 1 : 0;
    }
    float4 gmr[kGmRegs];
#pragma unroll
    for (int c = 0; c < kGmRegs; c++) {
        if constexpr (kKept) gmr[c] = c < S ? kept.g1[c] : make_float4(SR_NEG_INF, SR_NEG_INF, SR_NEG_INF, SR_NEG_INF);
        else gmr[c] = c < S ? gm_load(c) : make_float4(SR_NEG_INF, SR_NEG_INF, SR_NEG_INF, SR_NEG_INF);
    }
    static_assert(kGmRegs == kKeptChunks, "kept chunks fill the direct path's registers");
    // with few chunks the second maxima and the positions of the maxima come along in the same batch of loads
    constexpr int kG2Regs = 4;
    const bool direct = S <= kG2Regs;  // a group whose second largest is below the bound hands over its largest directly
    float4 g2r[kG2Regs];
    uint32_t gpr[kG2Regs];
#pragma unroll
    for (int c = 0; c < kG2Regs; c++) {
        const bool in = direct && c < S;
        if constexpr (kKept) {
            g2r[c] = in ? kept.g2[c] : make_float4(SR_NEG_INF, SR_NEG_INF, SR_NEG_INF, SR_NEG_INF);
            gpr[c] = in ? kept.gp[c] : 0u;
        } else {
            g2r[c] = in ? a.gmax2[((size_t)slot * S + c) * kThreads + tid] : make_float4(SR_NEG_INF, SR_NEG_INF, SR_NEG_INF, SR_NEG_INF);
            gpr[c] = in ? a.gpos[((size_t)slot * S + c) * kThreads + tid] : 0u;
        }
    }
    // (not kKept) the waves' shares of the bound, asked for with the group results: behind the barrier below they
    // would be a round trip to memory of their own
    const int nb = kKept ? kWaves : S * kWaves;  // (a worker that keeps its row's results: one share per wave and row)
    uint2 gb0 = make_uint2(0xffffffffu, 0u);
    if constexpr (!kKept) {
        if (lane < nb) gb0 = ((const uint2*)a.gbound + (size_t)slot * nb)[lane];
    }
    early();
    auto each_gm = [&](auto&& f) SR_INL {
#pragma unroll
        for (int c = 0; c < kGmRegs; c++)
            if (c < S) f(c, gmr[c]);
        for (int c = kGmRegs; c < S; c++) f(c, gm_load(c));
    };
    bool bins = false;
    BinMap map;
    // one candidate at list position pos
    auto place = [&](uint32_t pos, float x, int idx) SR_INL {
        if (pos < (uint32_t)kSelMax) {
            sm.vals[pos] = x;
            sm.idxs[pos] = idx;

        } else if (pos < (uint32_t)kRowCap) {
            sr_store_agent(&crow[pos], ((unsigned long long)sr_f2u(x) << 32) | (unsigned long long)(uint32_t)idx);
        }
    };
    // Every lane brings n_own entries for a list: one atomic per wave reserves the wave's slice, the lane's own
    // slice starts at the returned position.  All lanes of the wave call this.
    auto wave_reserve = [&](int n_own, uint32_t* counter) SR_INL -> uint32_t {
        const int incl = sr_wave_incl_scan_i32(n_own);
        const int total = __builtin_amdgcn_readlane(incl, SR_WAVE - 1);
        uint32_t base = 0u;
        if (total > 0 && lane == 0) base = atomicAdd(counter, (uint32_t)total);
        return (uint32_t)__builtin_amdgcn_readfirstlane((int)base) + (uint32_t)(incl - n_own);
    };
    auto list_group = [&](bool want, int c, int g) SR_INL {
        const int pos = wave_slot(want, &sm.bcast[13]);
        if (pos >= 0 && pos < kQCap) qlist[pos] = ((uint32_t)(c * kThreads + tid) << 2) | (uint32_t)g;
    };
    // fetches the listed groups, kBatch (group, vector) items per thread at a time -- values and keep-bits
    // of all of them in one batch of loads -- and appends every kept element that pred admits to the candidates
    auto gather = [&](int nq, auto&& pred) SR_INL {
        const int n_items = nq * kGV;
        for (int i0 = 0; i0 < n_items; i0 += kBatch * kThreads) {
            u32x4 v[kBatch];
            uint32_t kw[kBatch];
            int fvs[kBatch];
#pragma unroll
            for (int r = 0; r < kBatch; r++) {
                const int i = i0 + r * kThreads + tid;
                fvs[r] = -1;
                v[r] = VO::neg_inf();
                kw[r] = 0u;
                if (i0 + r * kThreads < n_items && i < n_items) {  // the first test is uniform: unused slots cost nothing
                    const uint32_t gid = qlist[i / kGV];
                    const int m = i - (i / kGV) * kGV;
                    const int g = (int)(gid & 3u), t = (int)((gid >> 2) & (kThreads - 1)), c = (int)(gid >> 11);
                    const int f0 = c * a.chunk_vecs;
                    const int nv = min(a.chunk_vecs, nvt - f0);
                    const int j = g + m * SR_TK_GROUPS;
                    const int fl = j * kThreads + t;
                    if (j < kVec && fl < nv) {
                        const int fv = f0 + fl;
                        fvs[r] = fv;
                        v[r] = wp[fv];
                        kw[r] = keep_bits(c, j, t);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < kBatch; r++) {
                if (i0 + r * kThreads >= n_items) continue;  // uniform
                uint32_t own = 0u;
#pragma unroll
                for (int q = 0; q < EPV; q++) {
                    const bool kept = ((kw[r] >> q) & 1u) != 0u;
                    own |= (kept && pred(VO::get(v[r], q))) ? (1u << q) : 0u;
                }
                uint32_t pos = wave_reserve(__popc(own), &sm.bcast[12]);
#pragma unroll
                for (int q = 0; q < EPV; q++)
                    if ((own >> q) & 1u) place(pos++, VO::get(v[r], q), fvs[r] * EPV + q - mis);
            }
        }
    };

    if (tid == 0) { sm.bcast[12] = 0u; sm.bcast[13] = 0u; }
    if (want_bins)
        for (int i = tid; i < kBinsPad; i += kThreads) sm.bhist[i] = 0u;
    __syncthreads();
    if (sel > kSelMax || sel < 1) return -1;
    // The chunk workgroups' waves each left a value with their share of sel group maxima at or above it: the
    // smallest of them has at least sel group maxima of the row at or above it.
    float tval = -3.402823466e38f;
    {
        uint32_t k = 0xffffffffu, km = 0u;
        if constexpr (kKept) {
            if (lane < nb) {
                k = sm.hist[2 * lane];
                km = sm.hist[2 * lane + 1];
            }
        } else {
            k = gb0.x;
            km = gb0.y;
            const uint2* gb = (const uint2*)a.gbound + (size_t)slot * nb;
            for (int i = lane + SR_WAVE; i < nb; i += SR_WAVE) {
                const uint2 b = gb[i];
                k = min(k, b.x);
                km = max(km, b.y);
            }
        }
        // Every wave's pair stands for distinct group maxima of the row: one that equals its second word and (its
        // share - 1) that are at least its first.  The largest value with sel of all those at or above it is a bound
        // too, and a much closer one than the smallest first word when sel is small (a top-k of 40 asks every wave
        // for its second largest: the smallest of 32 of those has some 250 elements above it, the 40th largest of the
        // 64 words about 50).  With one pair per lane it is found with ballots, to 16 bits, rounded down (worth its
        // eight or nine pairs of ballots only where the shares are that small).
        uint32_t k_close = 0u;
        const int share = (sel + nb - 1) / nb;  // (the waves' share was this or more)
        const uint32_t km_lane = km;
        km = sr_wave_max_u32(km);
        if (kShort && nb <= SR_WAVE && share <= 2) {
            const bool in = lane < nb;
            k_close = largest_key16(km, [&](uint32_t cnd) SR_INL -> bool {
                return __popcll(__ballot(in && k >= cnd)) * (share - 1) + __popcll(__ballot(in && km_lane >= cnd)) >= sel;
            });
        }
        k = sr_wave_min_u32(k);
        k = max(k, k_close);
        if (k > kKeyNegInf) tval = sr_okey_inv(k);
        // An element 19 T below the row's largest kept element has expf((v - max) / T) < 2^-26 whatever else
        // joins the row (penalties that only lower cannot raise the maximum's rivals above it, and the maximum of
        // the final set is at least this one): such entries change neither running sum nor can the draw stop on
        // them, so they need not become candidates.  Rows whose penalties may raise a logit keep the plain bound.
        const bool lowering_only = (rd.flags & kRowHasPenalty) == 0u || rd.edit_cnt <= 0 || (rd.flags & kRowHistExcl) != 0u;
        if (rd.path == SR_PATH_TOPK && lowering_only && km > kKeyNegInf && rd.temperature > 0.0f) {
            const float tdead = __fsub_rn(sr_okey_inv(km), __fmul_rn(19.0f, rd.temperature));
            tval = fmaxf(tval, tdead);
        }
        bins = want_bins && direct && km > kKeyNegInf;
        map.mx = __fmul_rn(sr_okey_inv(km), inv_temp);
        // the bins span what can become a candidate: from the maximum down to the bound
        const float span = __fsub_rn(map.mx, __fmul_rn(tval, inv_temp));
        if (EPV == 8 && bins && ((rd.flags & kRowHasPenalty) == 0u || rd.edit_cnt <= 0) && tval > -3.0e38f &&
            (km >> 16) - (sr_okey(tval) >> 16) < (uint32_t)kBins) {
            map.exact = true;
            map.ktop = km >> 16;
        } else if (bins && span > 1e-3f && span < 1e30f) {
            map.by_bits = true;
            map.span = span;
            map.c = __fmul_rn(span, kBinOffset);
            map.cbits = sr_f2u(map.c);
            map.ftop = (int)((sr_f2u(__fadd_rn(span, map.c)) - map.cbits) >> kBinShift);
        }
    }
    late();
    SR_PROF(a, 1);
    uint32_t mq1 = 0u, base_a = 0u;
    if (direct) {
        // The thread's 16 groups as two bit masks -- largest element at or above the bound with the second largest
        // below it (handed over directly), second largest at or above it (listed, fetched below) --, one
        // reservation per wave and list, then every lane places its own.
        uint32_t mq2 = 0u;
#pragma unroll
        for (int c = 0; c < kG2Regs; c++) {
            if (c < S) {
                const float m1[4] = {gmr[c].x, gmr[c].y, gmr[c].z, gmr[c].w};
                const float m2[4] = {g2r[c].x, g2r[c].y, g2r[c].z, g2r[c].w};
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const bool q2 = m2[g] >= tval, q1 = m1[g] >= tval && !q2;
                    mq2 |= q2 ? (1u << (c * 4 + g)) : 0u;
                    mq1 |= q1 ? (1u << (c * 4 + g)) : 0u;
                }
            }
        }
        // both counts in one scan: at most 16 per lane, 1,024 per wave
        const int n_own = __popc(mq1) | (__popc(mq2) << 16);
        const int incl = sr_wave_incl_scan_i32(n_own);
        const int total = __builtin_amdgcn_readlane(incl, SR_WAVE - 1);
        uint32_t base_l = 0u;
        if (lane == 0) {
            if ((total & 0xffff) > 0) base_a = atomicAdd(&sm.bcast[12], (uint32_t)(total & 0xffff));
            if ((total >> 16) > 0) base_l = atomicAdd(&sm.bcast[13], (uint32_t)(total >> 16));
        }
        base_a = (uint32_t)__builtin_amdgcn_readfirstlane((int)base_a) + (uint32_t)((incl - n_own) & 0xffff);
        base_l = (uint32_t)__builtin_amdgcn_readfirstlane((int)base_l) + (uint32_t)((incl - n_own) >> 16);
        // Every lane walks its own set bits, lowest first: the wave makes as many rounds as its busiest lane has
        // groups (a handful) instead of one per group of the thread (16).
        {
            uint32_t m = mq2, pos = base_l;
            while (__ballot(m != 0u) != 0ull) {
                const bool on = m != 0u;
                const int bit = on ? __ffs((int)m) - 1 : 0;
                m &= m - 1u;
                if (on && pos < (uint32_t)kQCap) qlist[pos] = ((uint32_t)((bit >> 2) * kThreads + tid) << 2) | (uint32_t)(bit & 3);
                pos++;
            }
        }
    } else {
        each_gm([&](int c, const float4& v) {
            list_group(v.x >= tval, c, 0);
            list_group(v.y >= tval, c, 1);
            list_group(v.z >= tval, c, 2);
            list_group(v.w >= tval, c, 3);
        });
    }
    __syncthreads();
    const int n_q = (int)sm.bcast[13];
    SR_PROF(a, 2);
    // The largest element of every group with one element at or above the bound, picked out of the thread's registers
    // by the bit number and handed over as it is.  Selects written as mask arithmetic: as conditionals the compiler
    // may turn them into branches.
    auto hand_over_direct = [&]() SR_INL {
        auto sel = [](uint32_t x0, uint32_t x1, int bit) SR_INL -> uint32_t {
            const uint32_t m = 0u - (uint32_t)(bit & 1);
            return (x0 & ~m) | (x1 & m);
        };
        auto pick4 = [&](const float4& v, int g) SR_INL -> uint32_t {
            return sel(sel(sr_f2u(v.x), sr_f2u(v.y), g), sel(sr_f2u(v.z), sr_f2u(v.w), g), g >> 1);
        };
        uint32_t m = mq1, pos = base_a;
        while (__ballot(m != 0u) != 0ull) {
            const bool on = m != 0u;
            const int bit = on ? __ffs((int)m) - 1 : 0;
            m &= m - 1u;
            const int c = bit >> 2, g = bit & 3;
            const float x = sr_u2f(sel(sel(pick4(gmr[0], g), pick4(gmr[1], g), c), sel(pick4(gmr[2], g), pick4(gmr[3], g), c), c >> 1));
            const uint32_t gp = sel(sel(gpr[0], gpr[1], c), sel(gpr[2], gpr[3], c), c >> 1);
            if (on) place(pos++, x, idx_of(c, g, (gp >> (8 * g)) & 0xffu));
        }
    };
    bool listed = false;
    if (n_q <= kQCap) {
        SR_PROF(a, 3);
        hand_over_direct();  // (no bits set unless direct)
        gather(n_q, [&](float x) { return x >= tval; });
        listed = true;
    } else {
        bins = false;  // the exact bound below starts the list again
        // Too many groups at or above the bound: the row is flat or heavily tied (or has too many chunks for the
        // per-wave bound).  Exact bound instead: the sel-th largest group maximum; every element above it lies in a
        // group whose maximum is above it (fewer than sel groups); of the elements equal to it only the first few by
        // index can matter, and those come from a scan of the row in index order that stops as soon as it has them.
        auto each_gk = [&](auto&& body) SR_INL {
            each_gm([&](int, const float4& v) {
                body(sr_okey(v.x)); body(sr_okey(v.y)); body(sr_okey(v.z)); body(sr_okey(v.w));
            });
        };
        const uint32_t tkey = block_radix_select(each_gk, sel, sm);
        const float tx = (tkey <= kKeyNegInf) ? -3.402823466e38f : sr_okey_inv(tkey);
        __syncthreads();
        if (tid == 0) { sm.bcast[13] = 0u; sm.bcast[12] = 0u; }  // candidates handed over so far are found again below
        __syncthreads();
        each_gm([&](int c, const float4& v) {
            list_group(v.x > tx, c, 0);
            list_group(v.y > tx, c, 1);
            list_group(v.z > tx, c, 2);
            list_group(v.w > tx, c, 3);
        });
        __syncthreads();
        const int nq = min((int)sm.bcast[13], kQCap);  // < sel
        gather(nq, [&](float x) { return x > tx; });
        __syncthreads();
        const int n_gt = (int)sm.bcast[12];
        take_ties(tx, sel - n_gt);
    }
    sr_drain_stores();
    __syncthreads();
    const uint32_t n_c = sm.bcast[12];
    __syncthreads();
    if (n_c > (uint32_t)kRowCap) return exact_row();  // more candidates than the lists hold: the exact way
    *binned = bins && listed && n_c <= (uint32_t)kSelMax;
    *map_out = map;
    *bound_out = tval;
    return (int)n_c;
}

// ---- the kernel --------------------------------------------------------------------------------------
// Every workgroup is a worker with a short program that the host wrote when the batch was uploaded: a list of chunk
// items, and possibly one row to finish at the end (the row tail) -- the row whose last chunk closes the list.  The
// host deals the items out in order of decreasing tail length to whichever worker will be free first by its
// estimate, so the rows with the longest tails are streamed first and finished while the others are still
// streaming; a worker ends with its tail, and a worker of a grid larger than the device holds starts when one ends.
// The row's other chunks were dealt out just before the last one, to workers that are running: the wait for them is
// short and bounded, and a worker that waits is never waited for.
//
// A chunk is kVec 16-byte vectors per thread, each read once into registers and folded into the thread's four
// groups.  When a vector has been folded, the load of the same vector of the worker's NEXT chunk is issued into its
// registers, so every thread has up to kVec loads in flight from its first chunk to its last, and the stores, the
// per-wave bound and the hand-off of a chunk run under the loads of the next one.
//
// kKept: every worker streams all chunks (at most kKeptChunks) of the one row it finishes and there is at most one
// worker per compute unit.  Nothing is handed over then, so nothing is written out: the group results of all chunks
// stay in the thread's registers (the workgroup has the register file of its compute unit to itself) and the waves'
// shares of the bound go through LDS.
// kRoomy: a launch of at most one worker per compute unit whose rows' chunks several workers stream (a batch of few
// rows): compiled for two waves a SIMD like the register-keeping shape, so that the row tail keeps its registers
// (with four waves a SIMD it spills a hundred bytes a lane, which the tails of a launch that has the compute units to
// itself need not pay for).
template <int EPV, int kVec, int kWindow, bool kKept, bool kShort, bool kRoomy = false>
__global__ __launch_bounds__(kThreads, (kKept || kRoomy) ? 2 : 4) void k_topk_rows(SrTopkArgs a)
{
    __shared__ TopkSmem sm;
    using VO = VecOps<EPV>;
    constexpr int ES = (EPV == 4) ? 4 : 2;  // element size in bytes
    const int tid = threadIdx.x, lane = sr_lane();
    const int S = a.chunks, V = a.vocab;
    // programs and items are read through the constant address space (the host wrote them before the launch): one
    // scalar 16-byte load each
    typedef int __attribute__((ext_vector_type(4))) i32x4;
    typedef const i32x4 __attribute__((address_space(4))) const_i32x4;
    // (first item, items, row slot to finish or -1, 1 = the items are all the chunks of that row and of no other)
    const i32x4 prog = ((const const_i32x4*)(uintptr_t)a.progs)[blockIdx.x];
    const const_i32x4* q = (const const_i32x4*)(uintptr_t)a.items + prog.x;
    const int n_items = prog.y;
    // A worker that streams all chunks of the one row it finishes hands nothing over: no other workgroup reads what
    // its chunks leave, so the chunks are neither waited for one by one nor counted in.
    const bool own_row = prog.w != 0;
    // this launch's counters: chunks counted in per row slot; the other set is cleared for the launch after this one,
    // so that nothing a launch leaves behind reaches a later one
    uint32_t* done = a.row_done + (size_t)a.parity * a.done_cap;
    {
        uint32_t* other = a.row_done + (size_t)(a.parity ^ 1u) * a.done_cap;
        for (uint32_t e = blockIdx.x * kThreads + (uint32_t)tid; e < a.done_cap; e += gridDim.x * kThreads)
            sr_store_agent(&other[e], 0u);
    }
    // Where an item's data lies.  The row is read as 16-byte vectors from the aligned address at or below its
    // start: window element p is row element p - mis; chunks are whole multiples of 64 vectors of that window.
    // Every load of a chunk is unconditional: a vector past the chunk's end (the last chunk of a row is ragged, and
    // a row that starts late in its first vector may leave a chunk empty) is read from the last vector that exists
    // instead -- the first vector of the row for an empty chunk -- and its keep-bits, all zero, turn it into -inf.
    struct Geom {
        const u32x4* cp;  // first vector of the chunk (of the row, for an empty chunk)
        int last;         // index of the last vector that exists, relative to cp
        int slot, c, sel, scan_row;
    };
    auto geom = [&](const i32x4& inf) SR_INL -> Geom {
        Geom g;
        g.slot = inf.x & 0xffffff;
        g.c = (inf.x >> 24) & 0x7f;
        g.sel = inf.w;
        g.scan_row = inf.z;
        const char* rowp = (const char*)a.logits + (size_t)inf.y * (size_t)a.row_stride * ES;
        const int mis = (int)(((uintptr_t)rowp & 15u) / ES);
        const int nvt = (V + mis + EPV - 1) / EPV;  // vectors of the row window
        const int f0 = g.c * a.chunk_vecs;          // first vector of this chunk
        const int nv = min(a.chunk_vecs, nvt - f0);  // vectors of this chunk that exist
        g.cp = (const u32x4*)(rowp - (size_t)mis * ES) + (nv > 0 ? f0 : 0);
        g.last = max(nv - 1, 0);
        return g;
    };
    auto keep_words = [&](const Geom& g) SR_INL -> const uint32_t* {
        return a.scan_mask + (size_t)g.scan_row * (size_t)a.scan_stride + ((size_t)g.c * kThreads + tid) * SR_TK_MASK_WORDS;
    };
    auto load_vec = [&](const Geom& g, int j) SR_INL -> u32x4 {
        const uint32_t off = (uint32_t)min(j * kThreads + tid, g.last) * 16u;
        return __builtin_nontemporal_load((const u32x4*)((const char*)g.cp + off));
    };

    KeptGroups kept;
    KeptHistory kept_hist;
    int trow = 0;
    SrRow trd;
    if constexpr (kKept) {
#pragma unroll
        for (int c = 0; c < kKeptChunks; c++) {
            kept.g1[c] = make_float4(SR_NEG_INF, SR_NEG_INF, SR_NEG_INF, SR_NEG_INF);
            kept.g2[c] = kept.g1[c];
            kept.gp[c] = 0u;
        }
        // the row to finish is known from the start: its descriptor, and the history ids with their logits, are
        // fetched now and wait in registers while the row streams
        if (prog.z >= 0) {
            typedef const int __attribute__((address_space(4))) const_i32;
            trow = ((const_i32*)(uintptr_t)a.sel_list)[prog.z];
            trd = load_row_uniform(a.rows + trow);
            const bool hist_regs = row_history_in_registers(trd);
#pragma unroll
            for (int r = 0; r < kHistRegs; r++) {
                const int e = r * kThreads + tid;
                const bool in = hist_regs && e < trd.edit_cnt;
                kept_hist.hee[r] = in ? a.edits[trd.edit_off + e] : SrEdit{};
                kept_hist.hx[r] = in ? row_logit(a, trow, trd, kept_hist.hee[r].id) : SR_NEG_INF;
            }
        }
    }
    if (n_items > 0) {
        const i32x4 info = q[0];  // (chunk | launch slot of the row, batch row, scan-mask row, sel)
        Geom cur = geom(info);
        // The scan mask holds one keep-bit per window element in this kernel's access order: the thread's own three
        // words, bit j * EPV + q = element q of its j-th vector.  They carry the row's edges, its allow-mask and, when
        // the row tail fetches them, its history ids: two operations per element replace all of that logic.
        uint32_t kw0, kw1, kw2;
        {
            const uint32_t* mw = keep_words(cur);
            kw0 = mw[0]; kw1 = mw[1]; kw2 = mw[2];
        }
        // A thread has kWin of its vectors in flight or in registers at a time: enough, over all workers, to keep the
        // memory busy, and no more -- what is in flight beyond that only queues, and the row tails' few loads queue
        // behind it.  Vector j passes through register slot j mod kWin; a chunk counts as kVecP vectors, a multiple
        // of kWin, the ones past kVec being neither loaded nor folded.
        constexpr int kWin = kWindow < kVec ? kWindow : kVec;
        constexpr int kVecP = (kVec + kWin - 1) / kWin * kWin;
        u32x4 t[kWin];
#pragma unroll
        for (int j = 0; j < kWin; j++) t[j] = load_vec(cur, j);

        // One chunk per turn.  Behind the worker's last chunk the registers are refilled from that chunk's first
        // vector, to no effect (one line, already in cache), so that the loop body is the same for every chunk: with
        // two bodies, or a condition around the loads, the compiler keeps the incoming vectors in registers of their
        // own and spills.
        int last_sel = 0;
        // (kKept) The wave's share of the row's bound, taken from the largest group maximum of every lane and chunk folded
        // so far (one value per lane and chunk instead of four: a lane with two groups of a chunk at or above the value
        // counts once, which can only lower the value and keeps it a bound -- a twelfth of the count at the largest
        // shares -- and a count costs four ballots instead of sixteen): the largest key, to 16 bits, with at least
        // `need` of those values at or above it; 0 when there is none.  *wmax = the wave's largest kept element.
        auto kept_share = [&](int need, uint32_t* wmax_out) SR_INL -> uint32_t {
            float pool[kKeptChunks];
#pragma unroll
            for (int c = 0; c < kKeptChunks; c++)
                pool[c] = fmaxf(fmaxf(kept.g1[c].x, kept.g1[c].y), fmaxf(kept.g1[c].z, kept.g1[c].w));
            auto enough = [&](uint32_t cnd) SR_INL -> bool {
                const float fc = sr_okey_inv(cnd);  // a key in the NaN range compares false: the right answer for it
                int cge = 0;
#pragma unroll
                for (int c = 0; c < kKeptChunks; c++) cge += __popcll(__ballot(pool[c] >= fc));
                return cge >= need;
            };
            const uint32_t wmax = sr_wave_max_u32(sr_okey(fmaxf(fmaxf(pool[0], pool[1]), fmaxf(pool[2], pool[3]))));
            static_assert(kKeptChunks == 4, "four pool values");
            *wmax_out = wmax;
            const uint32_t K = largest_key16(wmax, enough);
            return K;
        };
        for (int k = 0; k < n_items; k++) {
            const bool has_next = k + 1 < n_items;
            Geom nxt = cur;
            if (has_next) {
                const i32x4 ninfo = q[k + 1];
                nxt = geom(ninfo);
            } else {
                nxt.last = 0;
            }
#ifdef SR_PROFILE
            SrTopkArgs ap = a;
            if (a.prof) ap.prof = a.prof + ((size_t)prog.x + (size_t)k) * 16;
            SR_PROF(ap, 0);
#endif
            // Every lane owns four interleaved groups of vectors (j mod 4).  Of each group the row tail gets the
            // largest element with its position inside the group, and the second largest: a group whose second
            // largest is below the row's bound contributes its largest element directly and is never read again.
            float gm1[SR_TK_GROUPS], gm2[SR_TK_GROUPS];
            int gp1[SR_TK_GROUPS];
#pragma unroll
            for (int g = 0; g < SR_TK_GROUPS; g++) { gm1[g] = SR_NEG_INF; gm2[g] = SR_NEG_INF; gp1[g] = 0; }
#pragma unroll
            for (int j = 0; j < kVecP; j++) {
                const int g = j % SR_TK_GROUPS;
                const int slot = j % kWin;
                if (j < kVec) {
#pragma unroll
                    for (int e = 0; e < EPV; e++) {
                        const int bit = j * EPV + e;
                        const uint32_t wd = bit < 32 ? kw0 : bit < 64 ? kw1 : kw2;
                        const uint32_t keep = (uint32_t)((int)(wd << (31 - (bit & 31))) >> 31);  // all ones = keep
                        const float xe = sr_u2f((sr_f2u(VO::get(t[slot], e)) & keep) | (0xff800000u & ~keep));
                        gp1[g] = xe > gm1[g] ? (j / SR_TK_GROUPS) * EPV + e : gp1[g];  // strict: the first of equal values stays
                        gm2[g] = __builtin_amdgcn_fmed3f(gm1[g], gm2[g], xe);  // gm2 <= gm1: the median is the new second largest
                        gm1[g] = sr_max_f32(gm1[g], xe);
                    }
                }
                // The slot is free: the vector kWin places down the stream goes there -- of this chunk, or of the next.
                // The empty statement pins the order (the group's results exist before it, the load is issued after
                // it) and the scheduling barrier keeps the next vector's arithmetic behind this one's: left to itself
                // the compiler issues the loads first, into registers of their own.
                if (j + kWin < kVec) {
                    asm volatile("" : "+v"(gm1[g]), "+v"(gm2[g]), "+v"(gp1[g]) : : "memory");
                    t[slot] = load_vec(cur, j + kWin);
                } else if (j + kWin >= kVecP) {
                    asm volatile("" : "+v"(gm1[g]), "+v"(gm2[g]), "+v"(gp1[g]) : : "memory");
                    t[slot] = load_vec(nxt, j + kWin - kVecP);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#ifdef SR_PROFILE
            SR_PROF(ap, 1);
#endif
            // the next chunk's keep-words arrive under the stores and the bound loop
            {
                const uint32_t* mw = keep_words(nxt);
                kw0 = mw[0]; kw1 = mw[1]; kw2 = mw[2];
            }
            const uint32_t gpk = (uint32_t)gp1[0] | ((uint32_t)gp1[1] << 8) | ((uint32_t)gp1[2] << 16) | ((uint32_t)gp1[3] << 24);
            if constexpr (kKept) {
#pragma unroll
                for (int c = 0; c < kKeptChunks; c++) {
                    const bool on = cur.c == c;
                    kept.g1[c].x = on ? gm1[0] : kept.g1[c].x; kept.g1[c].y = on ? gm1[1] : kept.g1[c].y;
                    kept.g1[c].z = on ? gm1[2] : kept.g1[c].z; kept.g1[c].w = on ? gm1[3] : kept.g1[c].w;
                    kept.g2[c].x = on ? gm2[0] : kept.g2[c].x; kept.g2[c].y = on ? gm2[1] : kept.g2[c].y;
                    kept.g2[c].z = on ? gm2[2] : kept.g2[c].z; kept.g2[c].w = on ? gm2[3] : kept.g2[c].w;
                    kept.gp[c] = on ? gpk : kept.gp[c];
                }
            } else {
                const size_t go = ((size_t)cur.slot * S + cur.c) * kThreads + tid;
                sr_store_agent_f4(a.gmax + go, gm1[0], gm1[1], gm1[2], gm1[3]);
                sr_store_agent_f4(a.gmax2 + go, gm2[0], gm2[1], gm2[2], gm2[3]);
                __hip_atomic_store(a.gpos + go, gpk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            // The wave's share of the row's bound: a value, to 16 bits and rounded down, with at least
            // ceil(sel / (chunks x 8)) of the wave's 256 group maxima at or above it (found bit by bit with ballots).
            // The smallest of all the row's waves' values then has at least sel group maxima at or above it.
            // (A worker that keeps its row's results takes its share once, behind the row's last chunk, from the
            // group maxima of all its chunks.)
            last_sel = cur.sel;
            if constexpr (!kKept) {
                const int need = max((cur.sel + S * kWaves - 1) / (S * kWaves), 1);
                // the wave's largest kept element: the row tail drops what lies hopelessly far below the row's
                const float pa = fmaxf(gm1[0], gm1[1]), pb = fminf(gm1[0], gm1[1]), pc = fmaxf(gm1[2], gm1[3]), pd = fminf(gm1[2], gm1[3]);
                const uint32_t k1 = sr_okey(fmaxf(pa, pc));  // the lane's largest group maximum
                const uint32_t wmax = sr_wave_max_u32(k1);
                uint32_t K;
                if (kShort && need <= 2) {
                    // (a share of one or two, as every launch of short lists asks for: the wave's largest or second
                    // largest group maximum itself, from two reductions instead of a search with ballots)
                    const uint32_t k2 = sr_okey(fmaxf(fminf(pa, pc), fmaxf(pb, pd)));  // the lane's second largest
                    const unsigned long long top = __ballot(k1 == wmax);
                    const bool owner = lane == (int)__ffsll((long long)top) - 1;
                    const uint32_t w2 = sr_wave_max_u32(owner ? k2 : k1);
                    K = (need == 1 ? wmax : w2) & 0xffff0000u;
                } else {
                    K = largest_key16(wmax, [&](uint32_t cnd) SR_INL -> bool {
                        const float fc = sr_okey_inv(cnd);  // a key in the NaN range compares false: the right answer for it
                        return __popcll(__ballot(gm1[0] >= fc)) + __popcll(__ballot(gm1[1] >= fc)) +
                               __popcll(__ballot(gm1[2] >= fc)) + __popcll(__ballot(gm1[3] >= fc)) >= need;
                    });
                }
                if (lane == 0) {
                    uint32_t* gb = a.gbound + (((size_t)cur.slot * S + cur.c) * kWaves + (tid >> 6)) * 2;
                    __hip_atomic_store(gb, K, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(gb + 1, wmax, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
#ifdef SR_PROFILE
            SR_PROF(ap, 2);
            SR_PROF_VAL(ap, 13, cur.sel);
            SR_PROF_VAL(ap, 14, cur.slot);
#endif
            // hand the chunk over: this wave's write-through stores (and, older than them, the loads of the next
            // chunk) have completed, the workgroup meets, then the chunk is counted in
            if (!kKept && !own_row) {
                sr_drain_stores();
                __syncthreads();
                if (tid == 0) __hip_atomic_fetch_add(&done[cur.slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#ifdef SR_PROFILE
            SR_PROF(ap, 5);
#endif
            cur = nxt;
        }
        // One share per wave for the whole row, behind its last chunk: with at least ceil(sel / 8) of the wave's group
        // maxima at or above every wave's value, the smallest of the eight has sel of the row's at or above it.  The
        // larger pools over-select less than a share per chunk did (a share of 125 of 1,024 scatters by a tenth, a
        // share of 32 of 256 by a fifth, and the bound is the smallest of the shares), and one loop replaces four.
        if constexpr (kKept) {
            uint32_t wmax;
            const uint32_t K = kept_share(max((last_sel + kWaves - 1) / kWaves, 1), &wmax);
            if (lane == 0) {
                sm.hist[(tid >> 6) * 2] = K;
                sm.hist[(tid >> 6) * 2 + 1] = wmax;
            }
        }
    }
    if (prog.z < 0) return;

    // ---- the row tail
    const int tslot = prog.z;
    if constexpr (!kKept) {
        trow = a.sel_list[tslot];
        trd = a.rows[trow];
    }
#ifdef SR_PROFILE
    SrTopkArgs ap = a;
    if (a.prof) ap.prof = a.prof + ((size_t)a.n_items + (size_t)tslot) * 16;
    SR_PROF(ap, 0);
#else
    const SrTopkArgs& ap = a;
#endif
    // The row's other chunks are in the hands of workers that are running; they are nearly always in already.
    // Should they not come (the wait is bounded), the row is selected from its logits alone.
    bool handed_over;
    if constexpr (kKept) {
        // the row's results are in this workgroup's registers and LDS; a worker whose program is not of that kind (the
        // host writes none for this kernel) selects its row from the logits alone
        // (the waves' shares of the bound are read behind the barrier that follows the clearing of the tail's lists)
        handed_over = own_row && S <= kKeptChunks && a.spin_limit != 0u;
    } else {
        if (own_row) sr_drain_stores();  // every wave's own stores; the barrier below joins them
        if (tid == 0) {
            uint32_t ok = own_row && a.spin_limit != 0u ? 1u : 0u;
            for (uint32_t it = 0; !own_row && it < a.spin_limit; it++) {
                if (sr_load_agent(&done[tslot]) == (uint32_t)S) { ok = 1u; break; }
                __builtin_amdgcn_s_sleep(2);
            }
            // the chunks' results were written through to L2: drop what this CU's L1 may hold of an earlier launch
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            sm.bcast[7] = ok;
        }
        __syncthreads();
        handed_over = sm.bcast[7] != 0u;
    }
    SR_PROF(ap, 4);
    __builtin_amdgcn_s_setprio(3);  // the tail is the longer dependent chain: its waves go first
    topk_row_tail<EPV, kVec, kKept, kShort>(ap, tslot, trow, trd, !handed_over, kept, kept_hist, sm);
    SR_PROF(ap, 15);
}

// ---- scan mask ---------------------------------------------------------------------------------------
// One keep-bit per window element of a row, in the selection kernel's access order: SR_TK_MASK_WORDS 32-bit words
// per chunk and thread, bit j * epv + q = element q of the thread's j-th vector.  A bit is set when the element
// lies inside the row, its allow-mask (if any) admits it and, for rows whose tail fetches the history logits by
// id, it is not a history id.  One workgroup per (scan row, chunk): the words are built in LDS, the history ids
// that fall into the chunk are cleared there, then the words are written out.
__global__ __launch_bounds__(kThreads) void k_build_scan_mask(const SrScanDesc* descs, const int32_t* scan_ids,
                                                              const SrRow* rows, const SrEdit* edits,
                                                              const uint32_t* mask, int64_t mask_stride, uint32_t* scan_mask,
                                                              int64_t scan_stride, int vocab, int epv, int es, int chunks,
                                                              int chunk_vecs, int vecs_per_thread,
                                                              unsigned long long base_addr, long long stride_bytes)
{
    __shared__ uint32_t words[kThreads * SR_TK_MASK_WORDS];
    const int nth = blockIdx.x / chunks, c = blockIdx.x - nth * chunks;
    const int srow = scan_ids ? scan_ids[nth] : nth;  // a list of scan rows to build again, or all of them
    const int t = threadIdx.x;
    const SrScanDesc d = descs[srow];
    const SrRow rd = rows[d.row];
    const int mis = (int)(((base_addr + (unsigned long long)d.row * (unsigned long long)stride_bytes) & 15ull) / (unsigned)es);
    const int nvt = (vocab + mis + epv - 1) / epv;
    const int f0 = c * chunk_vecs;
    const int nv = min(chunk_vecs, nvt - f0);
    const uint32_t* src = ((d.flags & SR_SCAN_ALLOW) && rd.mask_row >= 0) ? mask + (size_t)rd.mask_row * mask_stride : nullptr;
    uint32_t w[SR_TK_MASK_WORDS];
#pragma unroll
    for (int k = 0; k < SR_TK_MASK_WORDS; k++) w[k] = 0u;
    for (int j = 0; j < vecs_per_thread; j++) {
        const int fl = j * kThreads + t;
        if (fl >= nv) break;
        const long long e0 = (long long)(f0 + fl) * epv - mis;  // row element under q = 0
        uint32_t bits = 0u;
        if (!src && e0 >= 0 && e0 + epv <= vocab) {
            bits = (1u << epv) - 1u;
        } else {
            for (int q = 0; q < epv; q++) {
                const long long e = e0 + q;
                if (e >= 0 && e < vocab && (!src || mask_bit(src, (int)e))) bits |= 1u << q;
            }
        }
        const int b = j * epv;
        w[b >> 5] |= bits << (b & 31);
    }
#pragma unroll
    for (int k = 0; k < SR_TK_MASK_WORDS; k++) words[t * SR_TK_MASK_WORDS + k] = w[k];
    __syncthreads();
    if (d.flags & SR_SCAN_HIST) {
        const SrEdit* ed = edits + rd.edit_off;
        for (int e = t; e < rd.edit_cnt; e += kThreads) {
            const int p = ed[e].id + mis;
            const int fv = p / epv, q = p - fv * epv;
            const int fl = fv - f0;
            if (fl < 0 || fl >= nv) continue;
            const int j = fl / kThreads, tt = fl - j * kThreads;
            const int b = j * epv + q;
            atomicAnd(&words[tt * SR_TK_MASK_WORDS + (b >> 5)], ~(1u << (b & 31)));
        }
        __syncthreads();
    }
    uint32_t* dst = scan_mask + (size_t)srow * scan_stride + (size_t)c * kThreads * SR_TK_MASK_WORDS;
    for (int i = t; i < kThreads * SR_TK_MASK_WORDS; i += kThreads) dst[i] = words[i];
}

// Applies what one appended token per row changes: history length and edit count of rows, whole edits at given
// positions of the edit array, single keep-bits of scan-mask rows cleared for ids that entered a history (same
// element -> bit mapping as above), and the uniforms of the next step.  The lists are read where the host wrote
// them (pinned host memory).
__global__ __launch_bounds__(256) void k_apply_patches(SrRow* rows, const SrRowPatch* rp, int n_rowp, SrEdit* edits,
                                                       const SrEditPatch* ep, int n_edits, const SrMaskClear* mc,
                                                       int n_clears, uint32_t* scan_mask, int64_t scan_stride, int epv,
                                                       int es, int chunk_vecs, unsigned long long base_addr,
                                                       long long stride_bytes, double* uni_dst, const double* uni_src,
                                                       int n_uni)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    // The lists lie in pinned host memory: every read is a trip over the bus.  All four are read first, without
    // conditions (a thread past a list's end reads the list's last entry, or whatever stands at the head of an empty
    // list's 256 bytes), so that the trips run side by side; then the changes are applied.
    const SrRowPatch r = rp[min(i, max(n_rowp, 1) - 1)];
    const SrEditPatch e = ep[min(i, max(n_edits, 1) - 1)];
    const SrMaskClear m = mc[min(i, max(n_clears, 1) - 1)];
    const double u = uni_src[min(i, max(n_uni, 1) - 1)];
    if (i < n_rowp) {
        rows[r.row].n_prev = r.n_prev;
        rows[r.row].edit_cnt = r.edit_cnt;
        rows[r.row].mask_row = r.mask_row;
        rows[r.row].sel = r.sel;
        rows[r.row].edit_off = r.edit_off;
    }
    if (i < n_edits) edits[e.index] = e.edit;
    if (i < n_clears) {
        const int mis = (int)(((base_addr + (unsigned long long)m.row * (unsigned long long)stride_bytes) & 15ull) / (unsigned)es);
        const int p = m.id + mis;
        const int fv = p / epv, q = p - fv * epv;
        const int c = fv / chunk_vecs, fl = fv - c * chunk_vecs;
        const int j = fl / kThreads, tt = fl - j * kThreads;
        const int b = j * epv + q;
        atomicAnd(&scan_mask[(size_t)m.scan_row * scan_stride + ((size_t)c * kThreads + tt) * SR_TK_MASK_WORDS + (b >> 5)],
                  ~(1u << (b & 31)));
    }
    if (i < n_uni) uni_dst[i] = u;
}

// The pieces of a batch upload, read where the host packed them (pinned host memory, over the bus) and written
// where they belong: one launch instead of one copy command per piece (each of which costs the stream about 20 us
// whatever its size).  Sources and destinations are 16-byte aligned.
__global__ __launch_bounds__(256) void k_scatter(const SrCopySeg* segs)
{
    const SrCopySeg s = segs[blockIdx.y];
    const unsigned long long n16 = s.bytes / 16;
    const uint4* src = (const uint4*)s.src;
    uint4* dst = (uint4*)s.dst;
    for (unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x; i < n16; i += (unsigned long long)gridDim.x * 256)
        dst[i] = src[i];
    if (blockIdx.x == 0) {
        const unsigned long long done = n16 * 16;
        if (done + threadIdx.x < s.bytes) ((char*)s.dst)[done + threadIdx.x] = ((const char*)s.src)[done + threadIdx.x];
    }
}

// Packed allow-bits of rows that hold -inf where a token is not allowed (ITokenConstraint.Filter's output,
// ITokenConstraint.cs:31-42): bit (i & 31) of word (i >> 5) = the row's element i is not -inf.  One wave per 64
// elements: a coalesced load, one ballot, two words.
template <int ES>
__global__ __launch_bounds__(256) void k_pack_allow_mask(const void* logits, int64_t row_stride, int vocab, uint32_t* out,
                                                         int64_t out_stride)
{
    const int row = blockIdx.y;
    const char* rowp = (const char*)logits + (size_t)row * (size_t)row_stride * ES;
    const int n64 = (vocab + 63) / 64;
    const int wave = (int)((blockIdx.x * blockDim.x + threadIdx.x) >> 6), lane = sr_lane();
    const int n_waves = (int)((gridDim.x * blockDim.x) >> 6);
    for (int g = wave; g < n64; g += n_waves) {
        const int i = g * 64 + lane;
        bool allowed = false;
        if (i < vocab) {
            const uint32_t bits = ES == 4 ? ((const uint32_t*)rowp)[i] : ((uint32_t)((const uint16_t*)rowp)[i] << 16);
            allowed = bits != 0xff800000u;
        }
        const unsigned long long bal = __ballot(allowed);
        if (lane < 2 && g * 2 + lane < (vocab + 31) / 32)
            out[(size_t)row * out_stride + g * 2 + lane] = (uint32_t)(bal >> (32 * lane));
    }
}

// AND of n registered masks (slots ids[0..n) of the pool) into slot `dst`; *any is set when a bit of the vocabulary
// is left.  ids lie in the kernel's arguments (few constraints are ever combined).
struct SrMaskAndIds { int32_t id[SR_MASK_AND_MAX]; };
__global__ __launch_bounds__(256) void k_mask_and(uint32_t* pool, int64_t pool_words, SrMaskAndIds ids, int n, int dst, int vocab,
                                                  uint32_t* any)
{
    const int nw = (vocab + 31) / 32;
    uint32_t seen = 0u;
    for (int w = blockIdx.x * blockDim.x + threadIdx.x; w < (int)pool_words; w += gridDim.x * blockDim.x) {
        uint32_t v = 0u;
        if (w < nw) {
            v = 0xffffffffu;
            for (int k = 0; k < n; k++) v &= pool[(size_t)ids.id[k] * (size_t)pool_words + w];
            if (w == nw - 1 && (vocab & 31)) v &= (1u << (vocab & 31)) - 1u;  // bits beyond the vocabulary never count
        }
        pool[(size_t)dst * (size_t)pool_words + w] = v;
        seen |= v;
    }
    if (__ballot(seen != 0u) != 0ull && sr_lane() == 0) atomicOr(any, 1u);
}
}  // namespace

hipError_t sr_launch_scatter(const SrCopySeg* segs, int n, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_scatter, dim3(24, (unsigned)n), dim3(256), 0, stream, segs);
    return hipGetLastError();
}

hipError_t sr_launch_pack_allow_mask(const void* logits, int dtype, int rows, int vocab, int64_t row_stride, uint32_t* out,
                                     int64_t out_stride, hipStream_t stream)
{
    if (rows <= 0 || vocab <= 0) return hipSuccess;
    const int n64 = (vocab + 63) / 64;
    const dim3 grid((unsigned)std::min((n64 + 3) / 4, 1024), (unsigned)rows), block(256);
    if (dtype == 1) hipLaunchKernelGGL(k_pack_allow_mask<2>, grid, block, 0, stream, logits, row_stride, vocab, out, out_stride);
    else hipLaunchKernelGGL(k_pack_allow_mask<4>, grid, block, 0, stream, logits, row_stride, vocab, out, out_stride);
    return hipGetLastError();
}

hipError_t sr_launch_mask_and(uint32_t* pool, int64_t pool_words, const int32_t* ids_host, int n, int dst, int vocab, uint32_t* any,
                              hipStream_t stream)
{
    SrMaskAndIds ids{};
    for (int k = 0; k < n && k < SR_MASK_AND_MAX; k++) ids.id[k] = ids_host[k];
    const int blocks = (int)std::min<int64_t>((pool_words + 255) / 256, 64);
    hipLaunchKernelGGL(k_mask_and, dim3((unsigned)std::max(blocks, 1)), dim3(256), 0, stream, pool, pool_words, ids, n, dst, vocab, any);
    return hipGetLastError();
}

hipError_t sr_launch_apply_patches(SrRow* rows, const SrRowPatch* rp, int n_rowp, SrEdit* edits, const SrEditPatch* ep,
                                   int n_edits, const SrMaskClear* mc, int n_clears, uint32_t* scan_mask,
                                   int64_t scan_stride, int epv, int chunk_vecs, unsigned long long base_addr,
                                   long long stride_bytes, double* uni_dst, const double* uni_src, int n_uni,
                                   hipStream_t stream)
{
    const int n = std::max(std::max(n_rowp, n_edits), std::max(n_clears, n_uni));
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_apply_patches, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, rows, rp, n_rowp, edits, ep,
                       n_edits, mc, n_clears, scan_mask, scan_stride, epv, epv == 8 ? 2 : 4, chunk_vecs, base_addr,
                       stride_bytes, uni_dst, uni_src, n_uni);
    return hipGetLastError();
}

hipError_t sr_launch_topk(const SrTopkArgs& a, int n_rows, hipStream_t stream)
{
    if (n_rows <= 0) return hipSuccess;
    dim3 grid((unsigned)a.n_workers), block(kThreads);
    // workers with a row of their own are few per compute unit: each keeps more of its vectors in flight
    // ... and where there is at most one of them per compute unit, the results of its chunks stay in its registers
    const bool kept = a.own_rows && a.kept && a.chunks <= kKeptChunks;
    // ... and a launch whose rows all ask for few entries carries the steps that pay for such rows only
    auto launch = [&](auto epv, auto vec, auto shrt) {
        constexpr int kE = decltype(epv)::value, kV = decltype(vec)::value;
        constexpr bool kS = decltype(shrt)::value;
        if (kept) hipLaunchKernelGGL((k_topk_rows<kE, kV, SR_TK_WINDOW_KEPT, true, kS>), grid, block, 0, stream, a);
        else if (a.own_rows) hipLaunchKernelGGL((k_topk_rows<kE, kV, SR_TK_WINDOW_OWN, false, kS>), grid, block, 0, stream, a);
        else if (a.n_workers <= a.cu_count) hipLaunchKernelGGL((k_topk_rows<kE, kV, SR_TK_WINDOW, false, kS, true>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((k_topk_rows<kE, kV, SR_TK_WINDOW, false, kS>), grid, block, 0, stream, a);
    };
    using std::integral_constant;
    if (a.dtype == 1) {
        if (a.short_lists) launch(integral_constant<int, 8>{}, integral_constant<int, SR_TK_VEC_BF16>{}, std::true_type{});
        else launch(integral_constant<int, 8>{}, integral_constant<int, SR_TK_VEC_BF16>{}, std::false_type{});
    } else {
        if (a.short_lists) launch(integral_constant<int, 4>{}, integral_constant<int, SR_TK_VEC>{}, std::true_type{});
        else launch(integral_constant<int, 4>{}, integral_constant<int, SR_TK_VEC>{}, std::false_type{});
    }
    return hipGetLastError();
}

hipError_t sr_launch_build_scan_mask(const SrScanDesc* descs, const int32_t* scan_ids, int n_scan, const SrRow* rows, const SrEdit* edits,
                                     const uint32_t* mask, int64_t mask_stride, uint32_t* scan_mask, int64_t scan_stride,
                                     int vocab, int epv, int chunks, int chunk_vecs, unsigned long long base_addr,
                                     long long stride_bytes, hipStream_t stream)
{
    if (n_scan <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_build_scan_mask, dim3((unsigned)(n_scan * chunks)), dim3(kThreads), 0, stream, descs, scan_ids, rows, edits,
                       mask, mask_stride, scan_mask, scan_stride, vocab, epv, epv == 8 ? 2 : 4, chunks, chunk_vecs,
                       epv == 8 ? SR_TK_VEC_BF16 : SR_TK_VEC, base_addr, stride_bytes);
    return hipGetLastError();
}
