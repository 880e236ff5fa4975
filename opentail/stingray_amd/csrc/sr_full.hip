// Full-vocabulary sampling: the reference's slow path (Sampler.cs:41-95), BuildFilteredDistribution
// (:118-163), GreedyWithHistoryPenalties (:421-437), SampleFromDistribution (:564-576) and
// ResampleResidual (:587-618).
//
// The row is materialised in an fp32 work row exactly as the reference copies it, and every stage is
// one pass of a 1024-thread workgroup over that row.  All running sums that the reference evaluates
// left to right go through the exact evaluator in sr_seqsum.h, so probabilities, cut-offs and draws
// carry the reference's bits.
#include "sr_device.h"
#include "sr_kernels.h"
#include "sr_seqsum.h"
#include "sr_types.h"

namespace {

#ifdef SR_PROFILE
#define FPROF(a, slot_, i_) do { if ((a).prof && (slot_) == 0 && threadIdx.x == 0) (a).prof[(i_)] = (unsigned long long)wall_clock64(); } while (0)
// (adds the time since *t_ to stamp i_ and moves *t_ on: for the steps of a loop)
#define FPROF_ADD(a, slot_, i_, t_) do { if ((a).prof && (slot_) == 0 && threadIdx.x == 0) { const unsigned long long now_ = (unsigned long long)wall_clock64(); (a).prof[(i_)] += now_ - (t_); (t_) = now_; } } while (0)
#else
#define FPROF(a, slot_, i_) do { } while (0)
#define FPROF_ADD(a, slot_, i_, t_) do { } while (0)
#endif

constexpr int kT = SR_SEQ_THREADS;
constexpr int kW = SR_SEQ_WAVES;
constexpr int kSmall = SR_FULL_SMALL_CAP;  // survivors sorted inside the kernel
constexpr int kTagIndexBits = 19;          // a find's tag in the walk by slabs: rank << 19 | index
constexpr int kCkpt = 128;                 // tiles of a row whose running sums are kept for the search that follows

struct FullSmem {
    SrSeqSmem seq;
    SrSeq8Smem seq8;
    float lane_sum[SR_SEQ_CHAINS];
    float redf[kW];
    uint32_t redu[kW];
    int redi[kW];
    uint32_t hist[256];
    uint32_t bc[16];
    float ckpt[kCkpt];  // running sum behind every tile of a row's exact sum (SeqMarks)
    float segst[SR_SEG_MAX];  // running sum behind every segment of a prepared row (seg_walk)
    uint32_t segbc[4];
    unsigned long long sortbuf[kSmall];
    float sprob[kSmall];
    uint32_t tags[kSmall];
};

// SR_OUT_AMBIGUOUS of the row at work: any thread that sees a cut or the draw land on its boundary (sr_near /
// sr_stop_near) stores here; the row's flags are written behind a barrier that follows.
#define SR_AMB_WORD 15
#define SR_AMB_IF(cond_) do { if (cond_) sm.bc[SR_AMB_WORD] = 1u; } while (0)

// ---- block reductions ------------------------------------------------------------------------------
__device__ __forceinline__ float blk_max_f(float v, bool* any_nan, FullSmem& sm)
{
    // NaN propagates (TensorPrimitives.Max)
    uint32_t nanf = (v != v) ? 1u : 0u;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float w = __shfl_xor(v, o);
        uint32_t wn = __shfl_xor(nanf, o);
        v = fmaxf(v, w);
        nanf |= wn;
    }
    __syncthreads();
    if (sr_lane() == 0) { sm.redf[sr_wave_id()] = v; sm.redu[sr_wave_id()] = nanf; }
    __syncthreads();
    float m = sm.redf[0];
    uint32_t n = sm.redu[0];
#pragma unroll
    for (int w = 1; w < kW; w++) { m = fmaxf(m, sm.redf[w]); n |= sm.redu[w]; }
    *any_nan = n != 0u;
    return m;
}
__device__ __forceinline__ int blk_sum_i(int v, FullSmem& sm)
{
    v = sr_wave_sum_i32(v);
    __syncthreads();
    if (sr_lane() == 0) sm.redi[sr_wave_id()] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int w = 0; w < kW; w++) t += sm.redi[w];
    return t;
}
__device__ __forceinline__ unsigned long long blk_max_u64(unsigned long long v, FullSmem& sm)
{
    v = sr_wave_max_u64(v);
    __syncthreads();
    if (sr_lane() == 0) sm.sortbuf[sr_wave_id()] = v;
    __syncthreads();
    unsigned long long t = 0ull;
#pragma unroll
    for (int w = 0; w < kW; w++) t = sm.sortbuf[w] > t ? sm.sortbuf[w] : t;
    __syncthreads();
    return t;
}
// exclusive scan of one int per thread
__device__ __forceinline__ int blk_excl_scan(int v, int* total, FullSmem& sm)
{
    int incl = sr_wave_incl_scan_i32(v);
    __syncthreads();
    if (sr_lane() == SR_WAVE - 1) sm.redi[sr_wave_id()] = incl;
    __syncthreads();
    int base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kW; w++) {
        int t = sm.redi[w];
        if (w < sr_wave_id()) base += t;
        tot += t;
    }
    *total = tot;
    return base + incl - v;
}


// ---- one pass of the workgroup over a row ---------------------------------------------------------------
// Calls f(value, index) for every element, any order, with 16-byte loads (four in flight per thread) where the
// row allows it; with kWrite the value returned by f is stored back.  The caller synchronises.
template <bool kWrite, typename F>
__device__ __forceinline__ void row_pass(float* p, int n, F f)
{
    const int tid = threadIdx.x;
    const int head = min(n, (int)((4u - (unsigned)(((uintptr_t)p >> 2) & 3u)) & 3u));  // elements before 16-byte alignment
    if (tid < head) {
        const float y = f(p[tid], tid);
        if (kWrite) p[tid] = y;
    }
    float4* p4 = (float4*)(p + head);
    const int nv = (n - head) >> 2;
    auto one = [&](float4& a, int v) __attribute__((always_inline)) {
        const int i = head + 4 * v;
        a.x = f(a.x, i); a.y = f(a.y, i + 1); a.z = f(a.z, i + 2); a.w = f(a.w, i + 3);
    };
    int v = tid;
    for (; v + 3 * kT < nv; v += 4 * kT) {
        float4 a = p4[v], b = p4[v + kT], c = p4[v + 2 * kT], d = p4[v + 3 * kT];
        one(a, v); one(b, v + kT); one(c, v + 2 * kT); one(d, v + 3 * kT);
        if (kWrite) { p4[v] = a; p4[v + kT] = b; p4[v + 2 * kT] = c; p4[v + 3 * kT] = d; }
    }
    for (; v < nv; v += kT) {
        float4 a = p4[v];
        one(a, v);
        if (kWrite) p4[v] = a;
    }
    const int done = head + 4 * nv;
    if (tid < n - done) {
        const float y = f(p[done + tid], done + tid);
        if (kWrite) p[done + tid] = y;
    }
}

// ---- exact left-to-right sum over term(i), i in [0, n) ------------------------------------------------
// term(i) must be >= 0 (or +0 for "skipped").  With kSearch, stops at the first i whose running sum is
// >= target and returns it in *found (else -1).
template <bool kSearch, typename Term>
__device__ __forceinline__ float seq_sum(Term term, int n, float s0, float target, int* found, FullSmem& sm)
{
    float s = s0;
    *found = -1;
    for (int base = 0; base < n; base += SR_SEQ_TILE) {
        float x[SR_SEQ_RUN];
        const int i0 = base + (int)threadIdx.x * SR_SEQ_RUN;
#pragma unroll
        for (int j = 0; j < SR_SEQ_RUN; j++) x[j] = (threadIdx.x < SR_SEQ_ACTIVE && i0 + j < n) ? term(i0 + j) : 0.0f;
        int f;
        sr_seq_tile<kSearch>(x, &s, target, &f, sm.seq);
        if (kSearch && f >= 0) {
            *found = base + f;
            return s;
        }
    }
    return s;
}

// The same over rows in memory.  A thread's SR_SEQ_RUN consecutive terms come in with 16-byte loads when the row
// is 16-byte aligned (one 4-byte load per term makes every load instruction of a wave touch 64 cache lines).
// The whole tiles of an aligned row are loaded kDepth - 1 tiles ahead of the tile that is scanned, into register
// sets that take turns: one workgroup has to keep that much in flight to cover the latency of memory.  Two things
// keep the loads in flight: what is loaded is turned into terms only when its tile is up, and the loop issues the
// same number of loads on every path -- behind the last tile it loads that tile again, to no effect -- because the
// compiler can wait for "all but the newest n loads" only where it can count them, and otherwise waits for all.
//   issue_fast(base, raw)  starts the loads of the whole tile whose first term is `base`, no conditions
//   issue_any(base, raw)   the same for any tile of any row (ragged end, unaligned row)
//   finish(raw, x)         the tile's terms from what was loaded
//
// A sum that is followed by a search over the same terms (residual resampling: Sampler.cs:594-614) leaves marks: the
// running sum behind every tile (SeqMarks::keep, rows of at most kCkpt tiles).  The running sum never decreases, so
// the search's answer lies in the first tile whose mark has reached the target, and the state in front of that tile is
// the mark before it: the search starts there (SeqMarks::from) instead of at the row's first term, and reads one
// tile instead of, on average, half the row.
struct SeqMarks {
    float* keep = nullptr;  // a sum writes the running sum behind tile t to keep[t]
    int from = 0;           // first tile that is looked at; s0 is the running sum in front of it
};
__device__ __forceinline__ bool seq_marks_fit(int n) { return (n + SR_SEQ_TILE - 1) / SR_SEQ_TILE <= kCkpt; }
// the tile at which a search for `target` over the marked row starts, and the running sum in front of it (*s0); behind a
// barrier that follows the sum
__device__ __forceinline__ int seq_marks_find(const float* marks, int n, float target, float* s0)
{
    const int tiles = (n + SR_SEQ_TILE - 1) / SR_SEQ_TILE;
    int t = 0;
    while (t < tiles - 1 && !(marks[t] >= target)) t++;
    *s0 = t > 0 ? marks[t - 1] : 0.0f;
    return t;
}
template <bool kSearch, int kDepth, typename Raw, typename IssueFast, typename IssueAny, typename Finish>
__device__ __forceinline__ float seq_sum_tiles(IssueFast issue_fast, IssueAny issue_any, Finish finish, bool fast_ok, int n,
                                               float s0, float target, int* found, FullSmem& sm, SeqMarks marks = SeqMarks())
{
    float s = s0;
    *found = -1;
    const int n_full = fast_ok ? n / SR_SEQ_TILE : 0;  // whole tiles, taken by the pipelined loop
    const int tb = marks.from;
    if (n_full > tb) {
        Raw r[kDepth];
#pragma unroll
        for (int k = 0; k < kDepth - 1; k++) issue_fast(min(tb + k, n_full - 1) * SR_SEQ_TILE, r[k]);
        for (int t0 = tb; t0 < n_full; t0 += kDepth) {
#pragma unroll
            for (int k = 0; k < kDepth; k++) {
                const int t = t0 + k;
                if (t >= n_full) break;
                issue_fast(min(t + kDepth - 1, n_full - 1) * SR_SEQ_TILE, r[(k + kDepth - 1) % kDepth]);
                float x[SR_SEQ_RUN];
                finish(r[k], x, t * SR_SEQ_TILE);
                int f;
                sr_seq_tile<kSearch>(x, &s, target, &f, sm.seq);
                if (kSearch && f >= 0) {
                    *found = t * SR_SEQ_TILE + f;
                    return s;
                }
                if (!kSearch && marks.keep && threadIdx.x == 0) marks.keep[t] = s;
            }
        }
    }
    for (int base = max(n_full, tb) * SR_SEQ_TILE; base < n; base += SR_SEQ_TILE) {
        Raw r;
        issue_any(base, r);
        float x[SR_SEQ_RUN];
        finish(r, x, base);
        int f;
        sr_seq_tile<kSearch>(x, &s, target, &f, sm.seq);
        if (kSearch && f >= 0) {
            *found = base + f;
            return s;
        }
        if (!kSearch && marks.keep && threadIdx.x == 0) marks.keep[base / SR_SEQ_TILE] = s;
    }
    return s;
}

struct SeqRaw1 { float v[SR_SEQ_RUN]; };
struct SeqRaw2 { float p[SR_SEQ_RUN], q[SR_SEQ_RUN]; };

// SR_SEQ_RUN consecutive elements of an aligned row from index i0 on, all inside the row
__device__ __forceinline__ void seq_load_run_fast(const float* p, int i0, float (&v)[SR_SEQ_RUN])
{
    static_assert(SR_SEQ_RUN % 4 == 0, "whole float4 per thread");
    const float4* vp = (const float4*)(p + i0);
#pragma unroll
    for (int k = 0; k < SR_SEQ_RUN / 4; k++) {
        const float4 a = vp[k];
        v[4 * k] = a.x; v[4 * k + 1] = a.y; v[4 * k + 2] = a.z; v[4 * k + 3] = a.w;
    }
}
// ... of any row, zeros past the row's end
__device__ __forceinline__ void seq_load_run(const float* p, bool aligned, int i0, int n, float (&v)[SR_SEQ_RUN])
{
    if (threadIdx.x >= SR_SEQ_ACTIVE) {  // (these threads carry no terms)
#pragma unroll
        for (int j = 0; j < SR_SEQ_RUN; j++) v[j] = 0.0f;
    } else if (aligned && i0 + SR_SEQ_RUN <= n) {
        seq_load_run_fast(p, i0, v);
    } else {
#pragma unroll
        for (int j = 0; j < SR_SEQ_RUN; j++) v[j] = (i0 + j < n) ? p[i0 + j] : 0.0f;
    }
}

// (every term is multiplied by m1 and then by m2 first: the two normalising factors of a row that was left unscaled)
struct SeqNoWatch {
    __device__ __forceinline__ void operator()(float, int) const {}
};
// watch(x, i) sees every term with its index as it passes (the terms of a tile are looked at before the tile is added)
struct SeqNoMap {
    __device__ __forceinline__ float operator()(float x, int) const { return x; }
};
// map(x, i) stands between a scaled term and the sum: the term that is added (and watched) is what it returns
template <bool kSearch, typename Watch = SeqNoWatch, typename Map = SeqNoMap>
__device__ __forceinline__ float seq_sum_row(const float* p, int n, float s0, float target, int* found, FullSmem& sm,
                                             float m1 = 1.0f, float m2 = 1.0f, Watch watch = Watch(), Map map = Map(),
                                             SeqMarks marks = SeqMarks())
{
    static_assert(SR_SEQ_ACTIVE == SR_SEQ_THREADS, "every thread of the block loads a run");
    const bool aligned = ((uintptr_t)p & 15u) == 0u;
    auto issue_fast = [&](int base, SeqRaw1& r) __attribute__((always_inline)) {
        seq_load_run_fast(p, base + (int)threadIdx.x * SR_SEQ_RUN, r.v);
    };
    auto issue_any = [&](int base, SeqRaw1& r) __attribute__((always_inline)) {
        seq_load_run(p, aligned, base + (int)threadIdx.x * SR_SEQ_RUN, n, r.v);
    };
    auto finish = [&](const SeqRaw1& r, float (&x)[SR_SEQ_RUN], int base) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < SR_SEQ_RUN; j++) {
            x[j] = map(__fmul_rn(__fmul_rn(r.v[j], m1), m2), base + (int)threadIdx.x * SR_SEQ_RUN + j);
            watch(x[j], base + (int)threadIdx.x * SR_SEQ_RUN + j);
        }
    };
    return seq_sum_tiles<kSearch, 3, SeqRaw1>(issue_fast, issue_any, finish, aligned, n, s0, target, found, sm, marks);
}

// ... and over the positive part of the difference of two rows (residual resampling)
template <bool kSearch>
__device__ __forceinline__ float seq_sum_residual(const float* p, const float* q, int n, float s0, float target, int* found,
                                                  FullSmem& sm, float m1 = 1.0f, float m2 = 1.0f, SeqMarks marks = SeqMarks())
{
    const bool aligned = (((uintptr_t)p | (uintptr_t)q) & 15u) == 0u;
    auto issue_fast = [&](int base, SeqRaw2& r) __attribute__((always_inline)) {
        const int i0 = base + (int)threadIdx.x * SR_SEQ_RUN;
        seq_load_run_fast(p, i0, r.p);
        seq_load_run_fast(q, i0, r.q);
    };
    auto issue_any = [&](int base, SeqRaw2& r) __attribute__((always_inline)) {
        const int i0 = base + (int)threadIdx.x * SR_SEQ_RUN;
        seq_load_run(p, aligned, i0, n, r.p);
        seq_load_run(q, aligned, i0, n, r.q);
    };
    auto finish = [&](const SeqRaw2& r, float (&x)[SR_SEQ_RUN], int) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < SR_SEQ_RUN; j++) {
            const float d = __fsub_rn(__fmul_rn(__fmul_rn(r.p[j], m1), m2), r.q[j]);
            x[j] = d > 0.0f ? d : 0.0f;
        }
    };
    return seq_sum_tiles<kSearch, 2, SeqRaw2>(issue_fast, issue_any, finish, aligned, n, s0, target, found, sm, marks);
}

// ---- exact sums prepared by the whole device ---------------------------------------------------------------
// One workgroup adds a row at the rate at which one compute unit reads and scans it (1 MB in ~45 us).  Where the terms
// lie in memory before that workgroup starts, the whole device prepares the sum: the row is cut into segments of
// SR_SEG_TERMS terms, a first kernel leaves an approximate sum of every segment (double precision, any order), and
// k_seq_funcs turns every segment into its increment function n -> n + a[n & 1] (sr_seqsum.h) for the binade that the
// approximate prefix predicts for the segment's start.  The workgroup that needs the sum then only walks the
// functions (seg_walk, one wave): a function is applied when the exact running sum in front of its segment lies in the
// binade it was made for and stays there; any other segment -- one in which the sum changes binade (a sum that starts
// at zero does that ~17 times, mostly within the first segments), a prediction that missed -- is added from its terms
// by the wave's own exact scan (sr_seq_wave).  The result never depends on the prediction: only the time does.
__device__ __forceinline__ int seg_count(int n) { return (n + SR_SEG_TERMS - 1) / SR_SEG_TERMS; }
static_assert(SR_SEG_TERMS == SR_WAVE * SR_SEQ_RUN && sizeof(SeqSegFunc) == 96, "one run of 16 terms per lane; six 16-byte loads per record");

struct SegRec {
    uint4 f, g, x0, x1, x2, x3;
};
__device__ __forceinline__ void seg_load_rec(const SeqSegFunc* funcs, int seg, int nseg, SegRec& r)
{
    const uint4 z = make_uint4(0u, 0u, 0u, 0u);
    r.f = r.g = r.x0 = r.x1 = r.x2 = r.x3 = z;
    if (seg < nseg) {
        const uint4* q = (const uint4*)(funcs + seg);
        r.f = q[0]; r.g = q[1]; r.x0 = q[2]; r.x1 = q[3]; r.x2 = q[4]; r.x3 = q[5];
    }
}

// The exact running sum over terms[0, n) from s0, by the 64 lanes of ONE wave.  With kSearch it stops at the first term at
// which the running sum reaches `target`: *found = its index and the returned value is the running sum at that term.
// With `states` (not with kSearch) the running sum behind segment g is left at states[g].
template <bool kSearch>
__device__ __forceinline__ float seg_walk(const float* terms, int n, const SeqSegFunc* funcs, float s0, float target, int* found,
                                          float* states)
{
    const int lane = sr_lane();
    const int nseg = seg_count(n);
    const bool aligned = ((uintptr_t)terms & 15u) == 0u;
    float s = s0;
    *found = -1;
    SegRec next;
    seg_load_rec(funcs, lane, nseg, next);
    for (int base = 0; base < nseg; base += SR_WAVE) {
        const int seg = base + lane;
        const bool have = seg < nseg;
        const SegRec r = next;
        seg_load_rec(funcs, seg + SR_WAVE, nseg, next);  // (the records of the next 64 segments come in meanwhile)
        const uint32_t kind = r.f.w & 0xffu;
        int lstart = 0;  // the segments of the lanes below are settled
        for (;;) {
            uint32_t n_in;
            int eb;
            sr_split(s, &n_in, &eb);
            SrInc m;
            m.a0 = 0u; m.a1 = 0u;
            if (have && lane >= lstart) {
                if (kind == SR_SEG_PLAIN && (int)r.f.z == eb) { m.a0 = r.f.x; m.a1 = r.f.y; }
                else { m.a0 = SR_SEQ_SAT; m.a1 = SR_SEQ_SAT; }  // made for another binade, or not one function
            }
            const SrInc sc = sr_scan_inc<false>(m);
            SrInc ex;
            ex.a0 = __shfl_up(sc.a0, 1);
            ex.a1 = __shfl_up(sc.a1, 1);
            if (lane == 0) { ex.a0 = 0u; ex.a1 = 0u; }
            const bool odd = (n_in & 1u) != 0u;
            const uint32_t before = sr_sat_add(n_in, odd ? ex.a1 : ex.a0);
            const uint32_t after = sr_sat_add(n_in, odd ? sc.a1 : sc.a0);
            bool ev = after >= (1u << 24);
            if (kSearch) ev = ev || sr_join(after, eb) >= target;
            const unsigned long long evl = __ballot(ev && have && lane >= lstart);
            const int fl = evl ? (int)__ffsll((long long)evl) - 1 : SR_WAVE;
            if (!kSearch && states && have && lane >= lstart && lane < fl) states[seg] = sr_join(after, eb);
            if (!evl) {
                const uint32_t tot = (uint32_t)__builtin_amdgcn_readlane((int)(odd ? sc.a1 : sc.a0), SR_WAVE - 1);
                s = sr_join(n_in + tot, eb);
                break;
            }
            // The first segment that the plain functions do not settle.  Its lane tries what its record offers, from
            // the exact sum in front of the segment; every step is checked, and a record that does not fit that sum
            // (or a search that would end inside the segment) leaves the segment to be added from its terms.
            const float s_before = sr_u2f((uint32_t)__builtin_amdgcn_readlane((int)sr_f2u(sr_join(before, eb)), fl));
            float s_try = 0.0f;
            bool ok = false;
            if (lane == fl) {
                if (kind == SR_SEG_EXACT && sr_f2u(s_before) == 0u) {
                    s_try = sr_u2f(r.g.w);
                    ok = true;
                } else if (kind == SR_SEG_SPLIT && (int)r.f.z == eb) {
                    const uint32_t n1 = sr_sat_add(before, (before & 1u) ? r.f.y : r.f.x);
                    if (n1 < (1u << 24)) {
                        float acc = sr_join(n1, eb);
                        const uint32_t xs[16] = {r.x0.x, r.x0.y, r.x0.z, r.x0.w, r.x1.x, r.x1.y, r.x1.z, r.x1.w,
                                                 r.x2.x, r.x2.y, r.x2.z, r.x2.w, r.x3.x, r.x3.y, r.x3.z, r.x3.w};
#pragma unroll
                        for (int j = 0; j < 16; j++) acc = __fadd_rn(acc, sr_u2f(xs[j]));
                        uint32_t n2;
                        int eb2;
                        sr_split(acc, &n2, &eb2);
                        if (eb2 == (int)r.g.z) {
                            const uint32_t n3 = sr_sat_add(n2, (n2 & 1u) ? r.g.y : r.g.x);
                            if (n3 < (1u << 24)) {
                                s_try = sr_join(n3, eb2);
                                ok = true;
                            }
                        }
                    }
                }
                if (kSearch && ok && s_try >= target) ok = false;  // the answer lies inside: from the terms
            }
            ok = __builtin_amdgcn_readlane((int)ok, fl) != 0;
            if (ok) {
                s = sr_u2f((uint32_t)__builtin_amdgcn_readlane((int)sr_f2u(s_try), fl));
            } else {
                float x[SR_SEQ_RUN];
                seq_load_run(terms, aligned, (base + fl) * SR_SEG_TERMS + lane * SR_SEQ_RUN, n, x);
                int at;
                s = sr_seq_wave<SR_SEQ_RUN, kSearch>(x, s_before, target, &at);
                if (kSearch && at >= 0) {
                    *found = (base + fl) * SR_SEG_TERMS + at;
                    return s;
                }
            }
            if (!kSearch && states && lane == 0) states[base + fl] = s;
            lstart = fl + 1;
            if (lstart >= SR_WAVE) break;
        }
    }
    return s;
}

// The record of one segment (SeqSegFunc) from its terms x (lane l holds the terms 16 l ... 16 l + 15 of the segment) and
// the approximate sum `before` of everything in front of the segment.  One wave.
// With `seg_sum` (>= 0: the approximate sum of the segment's own terms, known beforehand) a segment whose start and
// end lie well inside one binade gets its one function without a look at where inside it the sum would change binade.
__device__ __forceinline__ void seg_make_record(const float (&x)[SR_SEQ_RUN], int seg, double before, SeqSegFunc* out,
                                                float seg_sum = -1.0f)
{
    const int lane = sr_lane();
    if (seg > 0 && seg_sum >= 0.0f) {
        const float lo = __double2float_rn(before), hi = lo + seg_sum;
        uint32_t nn;
        int eb_lo, eb_hi;
        sr_split(lo * 0.9999f, &nn, &eb_lo);
        sr_split(hi * 1.0001f, &nn, &eb_hi);
        if (eb_lo == eb_hi) {  // (wave-uniform: both are the same in every lane)
            const SrInc sc = sr_scan_inc<false>(sr_run_inc(x, eb_lo));
            if (lane == SR_WAVE - 1) {
                uint4* q = (uint4*)out;
                q[0] = make_uint4(sc.a0, sc.a1, (uint32_t)eb_lo, SR_SEG_PLAIN);
                q[1] = make_uint4(SR_SEQ_SAT, SR_SEQ_SAT, (uint32_t)eb_lo, 0u);
            }
            return;
        }
    }
    // approximate running sum behind every lane's run (single precision does: a prediction that misses costs time only)
    float own = 0.0f;
#pragma unroll
    for (int j = 0; j < SR_SEQ_RUN; j++) own += x[j];
    const float incl = sr_wave_incl_sum_f32(own);
    const float before_f = __double2float_rn(before);
    const float p_end = before_f + incl;
    uint32_t nn;
    int eb_first, eb_last, eb_mine_end;
    sr_split(before_f, &nn, &eb_first);
    sr_split(__shfl(p_end, SR_WAVE - 1), &nn, &eb_last);
    sr_split(p_end, &nn, &eb_mine_end);
    SeqSegFunc f;
    f.a0 = f.a1 = f.b0 = f.b1 = SR_SEQ_SAT;
    f.eb = eb_first; f.eb2 = eb_last; f.kind = SR_SEG_PLAIN; f.end_bits = 0u;
    int cross = -1;
    if (seg == 0) {
        // the row's first segment starts from +0 exactly: its end, once and for all
        int dummy;
        const float end = sr_seq_wave<SR_SEQ_RUN, false>(x, 0.0f, 0.0f, &dummy);
        f.kind = SR_SEG_EXACT;
        f.end_bits = sr_f2u(end);
    } else if (eb_first == eb_last) {
        const SrInc sc = sr_scan_inc<false>(sr_run_inc(x, eb_first));
        f.a0 = (uint32_t)__builtin_amdgcn_readlane((int)sc.a0, SR_WAVE - 1);
        f.a1 = (uint32_t)__builtin_amdgcn_readlane((int)sc.a1, SR_WAVE - 1);
    } else {
        // the first lane behind whose run the sum is expected in another binade; everything behind that lane must then
        // lie in the segment's last binade, or the segment is no two functions
        const unsigned long long left = __ballot(eb_mine_end != eb_first);
        cross = left ? (int)__ffsll((long long)left) - 1 : SR_WAVE - 1;
        const int eb_behind = __builtin_amdgcn_readlane(eb_mine_end, cross);
        if (eb_behind == eb_last) {
            SrInc m1, m2;
            m1.a0 = m1.a1 = m2.a0 = m2.a1 = 0u;
            if (lane < cross) m1 = sr_run_inc(x, eb_first);
            if (lane > cross) m2 = sr_run_inc(x, eb_last);
            const SrInc s1 = sr_scan_inc<false>(m1), s2 = sr_scan_inc<false>(m2);
            f.a0 = (uint32_t)__builtin_amdgcn_readlane((int)s1.a0, SR_WAVE - 1);
            f.a1 = (uint32_t)__builtin_amdgcn_readlane((int)s1.a1, SR_WAVE - 1);
            f.b0 = (uint32_t)__builtin_amdgcn_readlane((int)s2.a0, SR_WAVE - 1);
            f.b1 = (uint32_t)__builtin_amdgcn_readlane((int)s2.a1, SR_WAVE - 1);
            f.kind = SR_SEG_SPLIT | ((uint32_t)cross << 8);
        } else {
            cross = -1;
        }
    }
    if (lane == 0) {
        uint4* q = (uint4*)out;
        q[0] = make_uint4(f.a0, f.a1, (uint32_t)f.eb, f.kind);
        q[1] = make_uint4(f.b0, f.b1, (uint32_t)f.eb2, f.end_bits);
    }
    if (lane == cross) {
#pragma unroll
        for (int j = 0; j < 16; j++) out->x[j] = x[j];
    }
}

// The search that follows a sum over the same terms: the first term at which the running sum reaches `target`, from
// the states the sum left (one wave; -1 when the sum stays below the target).
__device__ __forceinline__ int seg_search_states(const float* terms, int n, const float* states, float target, float* at_sum)
{
    const int lane = sr_lane();
    const int nseg = seg_count(n);
    const bool aligned = ((uintptr_t)terms & 15u) == 0u;
    int first = nseg;
    for (int g = lane; g < nseg; g += SR_WAVE)
        if (states[g] >= target) { first = g; break; }
    first = sr_wave_min_i32(first);
    if (first >= nseg) return -1;
    const float s_before = first > 0 ? states[first - 1] : 0.0f;
    float x[SR_SEQ_RUN];
    seq_load_run(terms, aligned, first * SR_SEG_TERMS + lane * SR_SEQ_RUN, n, x);
    int at;
    *at_sum = sr_seq_wave<SR_SEQ_RUN, true>(x, s_before, target, &at);
    return at >= 0 ? first * SR_SEG_TERMS + at : -1;
}

// TensorPrimitives.Sum in its 256-bit shape: strided lane accumulators seeded with the first vector, the
// ragged tail folded in through an overlapped last vector, pairwise horizontal add.
template <typename Term>
__device__ __forceinline__ float tp_sum(Term term, int n, FullSmem& sm)
{
    int dummy;
    if (n < 4) {
        return seq_sum<false>(term, n, 0.0f, 0.0f, &dummy, sm);
    }
    if (n >= 8) {
        // the eight lane accumulators as eight chains advanced together: one pass over the row
        const int nv = n / 8, rem = n - nv * 8;
        const int g = (int)threadIdx.x & (SR_SEQ_CHAINS - 1), lt = (int)threadIdx.x >> 3;
        const bool extra = rem > 0 && g >= 8 - rem;
        const int cnt = nv + (extra ? 1 : 0);
        float s = 0.0f;
        auto load = [&](int base, float (&x)[SR_SEQ_RUN8]) __attribute__((always_inline)) {
            const int i0 = base + lt * SR_SEQ_RUN8;
            if (i0 + SR_SEQ_RUN8 <= nv) {
#pragma unroll
                for (int j = 0; j < SR_SEQ_RUN8; j++) x[j] = term((i0 + j) * 8 + g);
            } else {
#pragma unroll
                for (int j = 0; j < SR_SEQ_RUN8; j++) {
                    const int i = i0 + j;
                    x[j] = (i < cnt) ? (i < nv ? term(i * 8 + g) : term(n - 8 + g)) : 0.0f;
                }
            }
        };
        // two register sets take turns: no copy, which would wait for the loads, sits between the tiles
        float xa[SR_SEQ_RUN8], xb[SR_SEQ_RUN8];
#pragma unroll
        for (int j = 0; j < SR_SEQ_RUN8; j++) xa[j] = xb[j] = 0.0f;
        load(0, xa);
        for (int base = 0; base < nv + 1; base += 2 * SR_SEQ_CHAIN_TILE) {
            if (base + SR_SEQ_CHAIN_TILE < nv + 1) load(base + SR_SEQ_CHAIN_TILE, xb);
            sr_seq_tile8(xa, &s, sm.seq8);
            if (base + SR_SEQ_CHAIN_TILE >= nv + 1) break;
            if (base + 2 * SR_SEQ_CHAIN_TILE < nv + 1) load(base + 2 * SR_SEQ_CHAIN_TILE, xa);
            sr_seq_tile8(xb, &s, sm.seq8);
        }
        __syncthreads();
        if (lt == 0) sm.lane_sum[g] = s;
        __syncthreads();
        const float l0 = sm.lane_sum[0], l1 = sm.lane_sum[1], l2 = sm.lane_sum[2], l3 = sm.lane_sum[3],
                    l4 = sm.lane_sum[4], l5 = sm.lane_sum[5], l6 = sm.lane_sum[6], l7 = sm.lane_sum[7];
        __syncthreads();
        return __fadd_rn(__fadd_rn(__fadd_rn(l0, l1), __fadd_rn(l2, l3)), __fadd_rn(__fadd_rn(l4, l5), __fadd_rn(l6, l7)));
    }
    const int w = 4;
    const int nv = n / w, rem = n - nv * w;
    float lane_sum[4];
#pragma unroll
    for (int l = 0; l < 4; l++) {
        const bool extra = rem > 0 && l >= w - rem;
        const int cnt = nv + (extra ? 1 : 0);
        auto lt = [&](int i) -> float { return i < nv ? term(i * w + l) : term(n - w + l); };
        lane_sum[l] = seq_sum<false>(lt, cnt, 0.0f, 0.0f, &dummy, sm);
    }
    return __fadd_rn(__fadd_rn(lane_sum[0], lane_sum[1]), __fadd_rn(lane_sum[2], lane_sum[3]));
}

// The same sum over a long row in memory (times mul when do_mul), one wave per lane accumulator.  The row comes in
// through LDS 8,192 entries at a time -- every thread brings two 16-byte pieces, two rounds ahead of the round that is
// added --, laid out chain by chain, and the wave of a chain adds its 1,024 terms of the round with the wave's own
// exact scan (sr_seq_wave): no block-wide step but one barrier per round, so a round costs what its 32 KB take to
// arrive.  The place of term v = 16 l + j of chain g is g * 1024 + 64 j + (l + 2 j) mod 64: the 64 lanes of a wave
// read a term from 64 consecutive places, and the stores of a piece's four entries fall two to a bank.
__device__ __forceinline__ float tp_sum_row(const float* p, int n, float mul, bool do_mul, FullSmem& sm)
{
    constexpr int kRound = 8192;
    static_assert(offsetof(FullSmem, sprob) == offsetof(FullSmem, sortbuf) + sizeof(FullSmem::sortbuf) &&
                  offsetof(FullSmem, tags) == offsetof(FullSmem, sprob) + sizeof(FullSmem::sprob) &&
                  sizeof(FullSmem::sortbuf) + sizeof(FullSmem::sprob) + sizeof(FullSmem::tags) >= 2 * kRound * sizeof(float),
                  "two rounds fit the three arrays, which lie one behind the other");
    static_assert(kRound == 8 * kT, "two 16-byte pieces per thread and round");
    if (n < 2 * kRound || ((uintptr_t)p & 15u) != 0u) {
        if (do_mul) return tp_sum([&](int i) -> float { return __fmul_rn(p[i], mul); }, n, sm);
        return tp_sum([&](int i) -> float { return p[i]; }, n, sm);
    }
    float* buf = (float*)sm.sortbuf;
    const int tid = threadIdx.x, lane = sr_lane(), wave = sr_wave_id();
    const int nv = n / 8, rem = n - nv * 8, body = nv * 8;
    const int rounds = (body + kRound - 1) / kRound;
    auto fetch = [&](int r, float4 (&v)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int x0 = r * kRound + 4 * (tid + h * kT);
            if (x0 + 4 <= body) {
                v[h] = *(const float4*)(p + x0);
            } else {
                v[h].x = x0 < body ? p[x0] : 0.0f;
                v[h].y = x0 + 1 < body ? p[x0 + 1] : 0.0f;
                v[h].z = x0 + 2 < body ? p[x0 + 2] : 0.0f;
                v[h].w = 0.0f;  // (x0 + 3 < body would have taken the other way)
            }
        }
    };
    auto stash = [&](int r, const float4 (&v)[2]) __attribute__((always_inline)) {
        float* b = buf + (r & 1) * kRound;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int t2 = tid + h * kT;  // the piece's number within the round
            const int vec = t2 >> 1, j = vec & 15, l = vec >> 4;
            float* at = b + (4 * (t2 & 1)) * 1024 + 64 * j + ((l + 2 * j) & 63);
            at[0] = do_mul ? __fmul_rn(v[h].x, mul) : v[h].x;
            at[1024] = do_mul ? __fmul_rn(v[h].y, mul) : v[h].y;
            at[2048] = do_mul ? __fmul_rn(v[h].z, mul) : v[h].z;
            at[3072] = do_mul ? __fmul_rn(v[h].w, mul) : v[h].w;
        }
    };
    float sc = 0.0f;
    auto add_round = [&](int r) __attribute__((always_inline)) {
        if (wave < SR_SEQ_CHAINS) {
            const float* b = buf + (r & 1) * kRound + wave * 1024;
            float x[16];
#pragma unroll
            for (int j = 0; j < 16; j++) x[j] = b[64 * j + ((lane + 2 * j) & 63)];
            int dummy;
            sc = sr_seq_wave<16, false>(x, sc, 0.0f, &dummy);
        }
    };
    // (behind the last round the loop fetches that round again, to no effect: the compiler can wait for "all but the
    // newest loads" only where it can count them)
    float4 va[2], vb[2];
    __syncthreads();  // (whoever used the arrays before is done)
    fetch(0, va);
    fetch(min(1, rounds - 1), vb);
    stash(0, va);
    for (int r = 0; r < rounds; r += 2) {
        fetch(min(r + 2, rounds - 1), va);
        __syncthreads();
        add_round(r);
        if (r + 1 >= rounds) break;
        stash(r + 1, vb);
        fetch(min(r + 3, rounds - 1), vb);
        __syncthreads();
        add_round(r + 1);
        if (r + 2 < rounds) stash(r + 2, va);
    }
    if (wave < SR_SEQ_CHAINS) {
        if (rem > 0 && wave >= 8 - rem) {  // the overlapped last vector's entry of this chain
            float x[1];
            const float t = p[n - 8 + wave];
            x[0] = lane == 0 ? (do_mul ? __fmul_rn(t, mul) : t) : 0.0f;
            int dummy;
            sc = sr_seq_wave<1, false>(x, sc, 0.0f, &dummy);
        }
        if (lane == 0) sm.lane_sum[wave] = sc;
    }
    __syncthreads();
    const float l0 = sm.lane_sum[0], l1 = sm.lane_sum[1], l2 = sm.lane_sum[2], l3 = sm.lane_sum[3],
                l4 = sm.lane_sum[4], l5 = sm.lane_sum[5], l6 = sm.lane_sum[6], l7 = sm.lane_sum[7];
    __syncthreads();
    return __fadd_rn(__fadd_rn(__fadd_rn(l0, l1), __fadd_rn(l2, l3)), __fadd_rn(__fadd_rn(l4, l5), __fadd_rn(l6, l7)));
}

// Normalize (Sampler.cs:553-562)
__device__ __forceinline__ void normalize_row(float* p, int n, FullSmem& sm)
{
    const float sum = tp_sum_row(p, n, 1.0f, false, sm);
    if (sum > 0.0f && sum != 1.0f) {
        const float inv = __fdiv_rn(1.0f, sum);
        row_pass<true>(p, n, [&](float x, int) -> float { return __fmul_rn(x, inv); });
    }
    __syncthreads();
}

// k-th largest value of p[0..n) (1-based), p >= 0: FindKthLargest (Sampler.cs:624-645).
// With last_shift = 16 only the upper 16 bits are resolved: the result is then the smallest value of the
// 65536-value bucket that holds the k-th largest.
// Keys above hi_key are left out (they count as absent).
__device__ __forceinline__ float kth_largest(const float* p, int n, int k, FullSmem& sm, int last_shift = 0,
                                             uint32_t hi_key = 0xffffffffu)
{
    uint32_t prefix = 0u, pmask = 0u;
    int need = k;
    for (int shift = 24; shift >= last_shift; shift -= 8) {
        if (threadIdx.x < 256) sm.hist[threadIdx.x] = 0u;
        __syncthreads();
        // Zeros (masked or filtered entries, often most of the row) are left out: they are the smallest keys and
        // only matter when fewer than k entries are positive, and then the answer is zero either way.
        row_pass<false>(const_cast<float*>(p), n, [&](float x, int) -> float {
            const uint32_t key = sr_f2u(x);
            if (key != 0u && (key & pmask) == prefix && key <= hi_key) atomicAdd(&sm.hist[(key >> shift) & 0xffu], 1u);
            return x;
        });
        __syncthreads();
        if (threadIdx.x == 0) {
            int c = 0, d = 255;
            for (; d > 0; d--) {
                if (c + (int)sm.hist[d] >= need) break;
                c += (int)sm.hist[d];
            }
            sm.bc[0] = (uint32_t)d;
            sm.bc[1] = (uint32_t)(need - c);
        }
        __syncthreads();
        prefix |= sm.bc[0] << shift;
        pmask |= 0xffu << shift;
        need = (int)sm.bc[1];
        __syncthreads();
    }
    return sr_u2f(prefix);
}

// The value of lane (lane ^ kMask), moved by the vector unit alone (no LDS): DPP inside rows of 16 lanes, the swaps of
// rows and of wave halves beyond.  Every lane of the wave must be active.
template <int kMask> __device__ __forceinline__ uint32_t lane_xor_u32(uint32_t v)
{
    static_assert(kMask == 1 || kMask == 2 || kMask == 4 || kMask == 8 || kMask == 16 || kMask == 32, "one bit of the lane number");
    if (kMask == 1) return sr_dpp_u32<0xB1>(v);                        // quad_perm [1, 0, 3, 2]
    if (kMask == 2) return sr_dpp_u32<0x4E>(v);                        // quad_perm [2, 3, 0, 1]
    if (kMask == 4) return sr_dpp_u32<0x1B>(sr_dpp_u32<0x141>(v));     // 7 - l inside eight lanes, then 3 - l inside four
    if (kMask == 8) return sr_dpp_u32<0x128>(v);                       // a row rotated by half its length
    if (kMask == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
        return (sr_lane() & 16) ? r[0] : r[1];
    }
    const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return (sr_lane() & 32) ? r[0] : r[1];
}
template <int kMask> __device__ __forceinline__ unsigned long long lane_xor_key(unsigned long long v)
{
    return ((unsigned long long)lane_xor_u32<kMask>((uint32_t)(v >> 32)) << 32) | (unsigned long long)lane_xor_u32<kMask>((uint32_t)v);
}
template <int kMask> __device__ __forceinline__ uint32_t lane_xor_key(uint32_t v) { return lane_xor_u32<kMask>(v); }

// Bitonic sort (descending) of buf[0 .. n_pow2) in LDS, n_pow2 a power of two <= kSmall, keys of 32 or 64 bits; entries
// that must come last are zero.  All threads call, behind a barrier that follows the last write of the entries.
//
// The entries live in registers, four consecutive ones per thread (a wave holds 256 consecutive entries): strides 1 and
// 2 pair registers of one thread, strides 4..128 pair lanes of one wave, and LDS is needed only for the strides of 256
// and more.  Those come at the start of the last merges (sizes 512 and up); all of them of one merge are done in one
// visit to LDS, by 256 threads that each hold one column (entries c, c + 256, c + 512, ...).
template <typename K>
__device__ __forceinline__ void sort_lds_desc(K* buf, int n_pow2)
{
    constexpr int kRow = 256;                 // entries of one wave
    constexpr int kCols = kSmall / kRow;      // most entries of one column
    static_assert(kRow == 4 * SR_WAVE && kRow * kW >= kSmall && kCols == 16, "the layout described above");
    const int tid = threadIdx.x, wave = sr_wave_id();
    if (n_pow2 <= kRow) {
        // A short list: every entry counts the entries that come before it (equal ones by their place).
        K key = 0;
        int rank = 0;
        if (tid < n_pow2) {
            key = buf[tid];
            for (int j = 0; j < n_pow2; j++) {
                const K o = buf[j];
                rank += (o > key || (o == key && j < tid)) ? 1 : 0;
            }
        }
        __syncthreads();
        if (tid < n_pow2) buf[rank] = key;
        __syncthreads();
        return;
    }
    const int base = 4 * tid;
    const int pe = max(n_pow2, 4);
    const bool wave_has = wave * kRow < pe;   // (the other waves only meet at the barriers)
    K v[4];
    auto load_rows = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] = (base + r < n_pow2) ? buf[base + r] : (K)0;
    };
    auto store_rows = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (base + r < n_pow2) buf[base + r] = v[r];
    };
    auto cx = [&](K& lo_i, K& hi_i, bool desc) __attribute__((always_inline)) {  // lo_i is the entry with the smaller index
        const K mx = lo_i > hi_i ? lo_i : hi_i, mn = lo_i > hi_i ? hi_i : lo_i;
        lo_i = desc ? mx : mn;
        hi_i = desc ? mn : mx;
    };
    auto lane_step = [&](auto mask, bool want_max) __attribute__((always_inline)) {
        constexpr int kM = decltype(mask)::value;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const K o = lane_xor_key<kM>(v[r]);
            const K mx = v[r] > o ? v[r] : o, mn = v[r] > o ? o : v[r];
            v[r] = want_max ? mx : mn;
        }
    };
    // the steps of merge size k2 with strides j_first, j_first / 2, ..., 1 (j_first <= 128)
    auto row_steps = [&](int k2, int j_first) __attribute__((always_inline)) {
        const bool desc = (base & k2) == 0;  // (k2 >= 4: the four entries share it; k2 == 2 is handled below)
        if (j_first >= 128) lane_step(std::integral_constant<int, 32>{}, desc == ((base & 128) == 0));
        if (j_first >= 64) lane_step(std::integral_constant<int, 16>{}, desc == ((base & 64) == 0));
        if (j_first >= 32) lane_step(std::integral_constant<int, 8>{}, desc == ((base & 32) == 0));
        if (j_first >= 16) lane_step(std::integral_constant<int, 4>{}, desc == ((base & 16) == 0));
        if (j_first >= 8) lane_step(std::integral_constant<int, 2>{}, desc == ((base & 8) == 0));
        if (j_first >= 4) lane_step(std::integral_constant<int, 1>{}, desc == ((base & 4) == 0));
        if (k2 == 2) {
            cx(v[0], v[1], true);
            cx(v[2], v[3], false);
        } else {
            cx(v[0], v[2], desc);
            cx(v[1], v[3], desc);
            cx(v[0], v[1], desc);
            cx(v[2], v[3], desc);
        }
    };
    if (wave_has) {
        load_rows();
        for (int k2 = 2; k2 <= min(pe, kRow); k2 <<= 1) row_steps(k2, k2 >> 1);
    }
    for (int k2 = 2 * kRow; k2 <= pe; k2 <<= 1) {
        if (wave_has) store_rows();
        __syncthreads();
        if (tid < kRow) {
            const int cols = pe / kRow;  // 2, 4, 8 or 16 entries in this thread's column
            K c[kCols];
#pragma unroll
            for (int a2 = 0; a2 < kCols; a2++) c[a2] = a2 < cols ? buf[tid + a2 * kRow] : (K)0;
#pragma unroll
            for (int ja = kCols / 2; ja >= 1; ja >>= 1) {
                if (ja * kRow * 2 <= k2) {
#pragma unroll
                    for (int a2 = 0; a2 < kCols; a2++)
                        if ((a2 & ja) == 0 && (a2 | ja) < cols) cx(c[a2], c[a2 | ja], ((a2 * kRow) & k2) == 0);
                }
            }
#pragma unroll
            for (int a2 = 0; a2 < kCols; a2++)
                if (a2 < cols) buf[tid + a2 * kRow] = c[a2];
        }
        __syncthreads();
        if (wave_has) {
            load_rows();
            row_steps(k2, kRow / 2);
        }
    }
    if (wave_has) store_rows();
    __syncthreads();
}
__device__ __forceinline__ void sort_small_desc(FullSmem& sm, int n_pow2) { sort_lds_desc(sm.sortbuf, n_pow2); }

template <int ES>
__device__ __forceinline__ float load_logit(const char* rowp, int i)
{
    if (ES == 4) return ((const float*)rowp)[i];
    return sr_bf16_to_f32(((const uint16_t*)rowp)[i]);
}

// A sampled row needs no adjusted copy: the masked, scaled logit is recomputed from the input where it is read (the
// row maximum and the expf pass), which saves one pass over the row and one write of it.  The few ids that a logit
// bias or a history penalty touches are left out of those two passes -- a bitmap of the vocabulary, read beside the
// logits like an allow-mask, names them -- and handled by the kernels that run one workgroup per row: k_full_edits
// computes their adjusted values, keeps them (a.edit_tab: the bitmap, then one float per edit) and folds them into the
// row's maximum; k_full_row writes their expf before it reads the row.  Without the table (the host gives it when the
// batch holds such a row), and for a row with more edits than it takes, the row keeps its adjusted copy.
__device__ __forceinline__ bool row_edits_on_the_fly(const SrRow& rd, const SrFullArgs& a)
{
    return (a.edit_tab != nullptr || a.edits_in_pass) && sr_row_edits_on_the_fly(rd, a.vocab);
}
__device__ __forceinline__ bool row_is_direct(const SrRow& rd, const SrFullArgs& a)
{
    return rd.temperature > 0.0f && (rd.edit_cnt <= 0 || row_edits_on_the_fly(rd, a));
}

// The value of an edited id before the temperature: LogitBias (Sampler.cs:51-58), then the history penalties
// (:367-419), on the masked logit.
__device__ __forceinline__ float edited_logit(float x, const SrEdit& e, const SrRow& rd, bool sampled, bool pen)
{
    if (sampled && e.has_bias) x = __fadd_rn(x, e.bias);
    if (pen && e.occ_all > 0) {
        if (rd.rep != 1.0f)
            for (int o = 0; o < e.occ_win; o++) x = x > 0.0f ? __fdiv_rn(x, rd.rep) : __fmul_rn(x, rd.rep);
        if (rd.presence != 0.0f || rd.frequency != 0.0f)
            x = __fsub_rn(x, __fadd_rn(rd.presence, __fmul_rn(rd.frequency, (float)e.occ_all)));
    }
    return x;
}

// ---- one pass of the grid's x dimension over a row of logits ---------------------------------------------
// The masked (and temperature-scaled) logits of a row, sixteen input bytes per thread and load, four loads in flight;
// body(i, x, c) gets c consecutive values starting at element i (c = 4 or 8 on the vector path, 1 on the scalar
// path that rows with an unaligned start and the last elements of a row take).
template <int ES>
struct RowSource {
    const char* rowp;
    const uint32_t* mrow;
    bool scale;
    float inv_temp;
    const uint32_t* erow = nullptr;  // bitmap of the ids the row's edits touch (body gets the bits of its run), or null
    __device__ __forceinline__ float fix(float x, uint32_t keep) const
    {
        if (!keep) x = SR_NEG_INF;
        return scale ? __fmul_rn(x, inv_temp) : x;
    }
};
template <int ES, typename Body>
__device__ __forceinline__ void stream_row(const RowSource<ES>& src, int n, Body body)
{
    constexpr int E = 16 / ES, kU = 4;
    const int nv = (((uintptr_t)src.rowp & 15u) == 0u) ? n / E : 0;
    const int step = (int)gridDim.x * 256;
    for (int v0 = (int)blockIdx.x * 256 + (int)threadIdx.x; v0 < nv; v0 += step * kU) {
        uint4 raw[kU];
        uint32_t keep[kU], hit[kU];
#pragma unroll
        for (int u = 0; u < kU; u++) {
            const int v = v0 + u * step;
            raw[u] = make_uint4(0u, 0u, 0u, 0u);
            keep[u] = 0xffu;
            hit[u] = 0u;
            if (v < nv) {
                raw[u] = ((const uint4*)src.rowp)[v];
                if (src.mrow) keep[u] = src.mrow[(v * E) >> 5] >> ((v * E) & 31);
                if (src.erow) hit[u] = (src.erow[(v * E) >> 5] >> ((v * E) & 31)) & ((1u << E) - 1u);
            }
        }
#pragma unroll
        for (int u = 0; u < kU; u++) {
            const int v = v0 + u * step;
            if (v >= nv) break;
            float x[E];
            if (ES == 4) {
                x[0] = sr_u2f(raw[u].x); x[1] = sr_u2f(raw[u].y); x[2] = sr_u2f(raw[u].z); x[3] = sr_u2f(raw[u].w);
            } else {
                const uint32_t r[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    x[(2 * q) % E] = sr_u2f(r[q] << 16);
                    x[(2 * q + 1) % E] = sr_u2f(r[q] & 0xffff0000u);
                }
            }
#pragma unroll
            for (int q = 0; q < E; q++) x[q] = src.fix(x[q], (keep[u] >> q) & 1u);
            body(v * E, x, E, hit[u]);
        }
    }
    for (int i = nv * E + (int)blockIdx.x * 256 + (int)threadIdx.x; i < n; i += step) {
        float x[E];
        x[0] = src.fix(load_logit<ES>(src.rowp, i), src.mrow ? (src.mrow[i >> 5] >> (i & 31)) & 1u : 1u);
        body(i, x, 1, src.erow ? (src.erow[i >> 5] >> (i & 31)) & 1u : 0u);
    }
}
// stores c values (c = 1, 4 or 8) at w + i, with 16-byte stores where the address allows
template <int E>
__device__ __forceinline__ void store_run(float* w, int i, const float (&x)[E], int c)
{
    if (c == E && (((uintptr_t)(w + i)) & 15u) == 0u) {
#pragma unroll
        for (int q = 0; q < E; q += 4) *(float4*)(w + i + q) = make_float4(x[q], x[q + 1], x[q + 2], x[q + 3]);
    } else {
#pragma unroll
        for (int q = 0; q < E; q++)
            if (q < c) w[i + q] = x[q];
    }
}

// The histogram of a row's e = expf(x - max) by their upper 16 bits (kHistPos positions: position d holds the keys
// 0x3f80 - d, position 0 is e = 1, the last position everything below): see nucleus_from_histogram
constexpr int kHistPos = 8192;
constexpr uint32_t kHistTopKey = 0x3f80u;
__device__ __forceinline__ void hist_count(uint32_t* hcnt, uint32_t* bad, float e)
{
    if (e > 0.0f) {
        const uint32_t key = sr_f2u(e) >> 16;
        if (key <= kHistTopKey) atomicAdd(&hcnt[min(kHistTopKey - key, (uint32_t)(kHistPos - 1))], 1u);
        else *bad = 1u;  // (no e exceeds 1; if one does, the general way takes the row)
    }
}

// which rows take which way: asked by the passes over the whole device and by the row's workgroup alike
__device__ __forceinline__ bool row_watch_min_p(const SrRow& rd, const SrFullArgs& a)
{
    return rd.min_p > 0.0f && !(rd.top_k > 0 && rd.top_k < a.vocab) && a.mode == 0 && a.vocab >= 8;
}
__device__ __forceinline__ bool row_fast_nucleus(const SrRow& rd, const SrFullArgs& a)
{
    const bool use_top_p = rd.top_p < 1.0f && rd.top_p > 0.0f;
    return use_top_p && !(rd.top_k > 0 && rd.top_k < a.vocab) && !(rd.min_p > 0.0f) && a.mode == 0 && a.vocab >= 8 &&
           a.vocab <= (1 << kTagIndexBits) && a.sort_stride >= a.vocab;
}
// the row's maximum in SrFullState: this launch's number in front of the key, and what the word holds of this launch
__device__ __forceinline__ unsigned long long full_maxkey(const SrFullArgs& a, uint32_t key)
{
    return ((unsigned long long)a.seq << 32) | (unsigned long long)key;
}
__device__ __forceinline__ uint32_t full_maxkey_of(const SrFullArgs& a, unsigned long long word)
{
    return (uint32_t)(word >> 32) == a.seq ? (uint32_t)word : 0u;
}

// ---- stage 1: the masked (and temperature-scaled) copy of the row ------------------------------------
template <int ES>
__global__ __launch_bounds__(256) void k_full_prep(SrFullArgs a)
{
    const int slot = blockIdx.y;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    float* w = a.work + (size_t)(a.work_by_row ? row : slot) * a.work_stride;
    RowSource<ES> src;
    src.rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
    src.mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
    src.scale = rd.temperature > 0.0f && rd.temperature != 1.0f;
    src.inv_temp = src.scale ? __fdiv_rn(1.0f, rd.temperature) : 1.0f;
    if (row_is_direct(rd, a)) return;  // the kernels behind read the logits themselves
    stream_row<ES>(src, a.vocab, [&](int i, const float (&x)[16 / ES], int c, uint32_t) { store_run(w, i, x, c); });
}

// ---- stage 2: logit bias and history penalties on the few ids they touch (Sampler.cs:51-58, :367-419)
template <int ES>
__global__ __launch_bounds__(256) void k_full_edits(SrFullArgs a)
{
    const int slot = blockIdx.x;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    if (rd.edit_cnt <= 0) return;
    const SrEdit* ed = a.edits + rd.edit_off;
    if (a.edits_in_pass && row_edits_on_the_fly(rd, a)) return;  // (k_full_softmax_seg applies them where it loads the row)
    if (row_edits_on_the_fly(rd, a)) {
        // the row's bitmap (cleared first: the barrier's wait for the stores stands between them and the atomics on
        // the same words), the adjusted and scaled values of its edits, and their share of the row's maximum
        const int words = (a.vocab + 31) / 32;
        uint32_t* tab = a.edit_tab + (size_t)slot * (size_t)a.edit_tab_stride;
        float* vals = (float*)(tab + words);
        for (int i = threadIdx.x; i < words; i += 256) tab[i] = 0u;
        sr_drain_stores();  // (not a fence: a release at device scope writes the whole L2 back)
        __syncthreads();
        const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
        const uint32_t* mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
        const bool scale = rd.temperature != 1.0f;
        const float inv_temp = scale ? __fdiv_rn(1.0f, rd.temperature) : 1.0f;
        const bool pen = (rd.flags & SR_ROWFLAG_HAS_PENALTY) != 0u;
        uint32_t k = 0u;
        for (int e = threadIdx.x; e < rd.edit_cnt; e += 256) {
            const int id = ed[e].id;
            atomicOr(&tab[id >> 5], 1u << (id & 31));
            float x = load_logit<ES>(rowp, id);
            if (mrow && !((mrow[id >> 5] >> (id & 31)) & 1u)) x = SR_NEG_INF;
            x = edited_logit(x, ed[e], rd, true, pen);
            if (scale) x = __fmul_rn(x, inv_temp);
            vals[e] = x;
            const uint32_t kv = (x != x) ? 0xffffffffu : sr_okey(x);  // NaN propagates (TensorPrimitives.Max)
            k = kv > k ? kv : k;
        }
        k = sr_wave_max_u32(k);
        if (sr_lane() == 0 && k != 0u) atomicMax(&a.state[slot].maxkey, full_maxkey(a, k));
        return;
    }
    const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
    float* w = a.work + (size_t)(a.work_by_row ? row : slot) * a.work_stride;
    const uint32_t* mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
    const bool sampled = rd.temperature > 0.0f;
    const bool scale = sampled && rd.temperature != 1.0f;
    const float inv_temp = scale ? __fdiv_rn(1.0f, rd.temperature) : 1.0f;
    const bool pen = (rd.flags & SR_ROWFLAG_HAS_PENALTY) != 0u;
    for (int e = threadIdx.x; e < rd.edit_cnt; e += 256) {
        const int id = ed[e].id;
        float x = load_logit<ES>(rowp, id);
        if (mrow && !((mrow[id >> 5] >> (id & 31)) & 1u)) x = SR_NEG_INF;
        x = edited_logit(x, ed[e], rd, sampled, pen);
        if (scale) x = __fmul_rn(x, inv_temp);
        w[id] = x;
    }
}

// ---- stage 2b: the row maximum and expf(x - max) of the sampled rows, spread over the whole device ------
// (Softmax, Sampler.cs:448-459.)  One workgroup per row would spend most of its time in the double-precision
// expf of 150 thousand entries; here every row is cut into up to 64 pieces.
template <int ES>
__global__ __launch_bounds__(256) void k_full_max(SrFullArgs a)
{
    __shared__ uint32_t wmax[4];
    const int slot = blockIdx.y;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    if (rd.temperature <= 0.0f) return;  // greedy rows keep their logits
    uint32_t k = 0u;
    auto fold = [&](float v) {
        const uint32_t kv = (v != v) ? 0xffffffffu : sr_okey(v);  // NaN propagates (TensorPrimitives.Max)
        k = kv > k ? kv : k;
    };
    if (row_is_direct(rd, a)) {
        RowSource<ES> src;
        src.rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
        src.mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
        src.scale = rd.temperature != 1.0f;
        src.inv_temp = src.scale ? __fdiv_rn(1.0f, rd.temperature) : 1.0f;
        // (ids that the row's edits touch are not looked at: k_full_edits has folded their adjusted values in)
        src.erow = rd.edit_cnt > 0 ? a.edit_tab + (size_t)slot * (size_t)a.edit_tab_stride : nullptr;
        stream_row<ES>(src, a.vocab, [&](int, const float (&x)[16 / ES], int c, uint32_t hit) {
#pragma unroll
            for (int q = 0; q < 16 / ES; q++)
                if (q < c && ((hit >> q) & 1u) == 0u) fold(x[q]);
        });
    } else {
        RowSource<4> src;  // the adjusted copy
        src.rowp = (const char*)(a.work + (size_t)(a.work_by_row ? row : slot) * a.work_stride);
        src.mrow = nullptr;
        src.scale = false;
        src.inv_temp = 1.0f;
        stream_row<4>(src, a.vocab, [&](int, const float (&x)[4], int c, uint32_t) {
#pragma unroll
            for (int q = 0; q < 4; q++)
                if (q < c) fold(x[q]);
        });
    }
    k = sr_wave_max_u32(k);
    if (sr_lane() == 0) wmax[sr_wave_id()] = k;
    __syncthreads();
    if (threadIdx.x == 0) {
        k = max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3]));
        if (k != 0u) atomicMax(&a.state[slot].maxkey, full_maxkey(a, k));
    }
}
template <int ES>
__global__ __launch_bounds__(256) void k_full_exp(SrFullArgs a)
{
    const int slot = blockIdx.y;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    if (rd.temperature <= 0.0f) return;
    const uint32_t mk = full_maxkey_of(a, a.state[slot].maxkey);
    if (mk == 0xffffffffu || mk <= 0x007fffffu) return;  // NaN, or nothing above -inf: the row kernel makes it uniform
    const float m = sr_okey_inv(mk);
    __shared__ uint64_t tab[32];  // the expf table: a lookup per element from global memory is a long dependent load
    if (threadIdx.x < 32) tab[threadIdx.x] = sr_exp2f_tab[threadIdx.x];
    __syncthreads();
    float* w = a.work + (size_t)(a.work_by_row ? row : slot) * a.work_stride;
    if (row_is_direct(rd, a)) {
        RowSource<ES> src;
        src.rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
        src.mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
        src.scale = rd.temperature != 1.0f;
        src.inv_temp = src.scale ? __fdiv_rn(1.0f, rd.temperature) : 1.0f;
        // (what is written for an id that the row's edits touch does not matter: k_full_row writes it again)
        stream_row<ES>(src, a.vocab, [&](int i, const float (&x)[16 / ES], int c, uint32_t) {
            float e[16 / ES];
#pragma unroll
            for (int q = 0; q < 16 / ES; q++) e[q] = q < c ? sr_expf_tab(__fsub_rn(x[q], m), tab) : 0.0f;
            store_run(w, i, e, c);
        });
    } else {
        RowSource<4> src;  // the adjusted copy, replaced in place
        src.rowp = (const char*)w;
        src.mrow = nullptr;
        src.scale = false;
        src.inv_temp = 1.0f;
        stream_row<4>(src, a.vocab, [&](int i, const float (&x)[4], int c, uint32_t) {
            float e[4];
#pragma unroll
            for (int q = 0; q < 4; q++) e[q] = q < c ? sr_expf_tab(__fsub_rn(x[q], m), tab) : 0.0f;
            store_run(w, i, e, c);
        });
    }
}

// ---- the same two passes, laid out for a denominator that the whole device prepares -------------------------
// (launches whose rows are long and start on 16-byte boundaries: a.seg_func is set.)  A wave takes whole segments of
// SR_SEG_TERMS elements, every lane 16 consecutive ones, so that the second pass can leave, beside e = expf(x - max), the
// record of the segment's exact sum (SeqSegFunc) for the row's workgroup to walk (seg_walk).  The binade that a
// record is made for comes from approximate sums: the first pass leaves every segment's own maximum m and the sum
// of exp(x - m) over it, and the second, which knows the row's maximum M, adds up S exp(m - M) over the segments in
// front.  The ids that the row's edits touch take their adjusted values from the work row, where k_full_edits left
// them: e is final when the second pass has written it.
template <int ES>
struct SegSource {
    const char* rowp;      // the row's logits, or null: the adjusted copy in w
    const uint32_t* mrow;
    const float* w;
    bool scale;
    float inv_temp;
};
template <int ES>
__device__ __forceinline__ SegSource<ES> seg_source(const SrRow& rd, const SrFullArgs& a, int slot, int row)
{
    SegSource<ES> src;
    src.w = a.work + (size_t)(a.work_by_row ? row : slot) * a.work_stride;
    src.rowp = nullptr;
    src.mrow = nullptr;
    src.scale = false;
    src.inv_temp = 1.0f;
    if (row_is_direct(rd, a)) {
        src.rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
        src.mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
        src.scale = rd.temperature != 1.0f;
        src.inv_temp = src.scale ? __fdiv_rn(1.0f, rd.temperature) : 1.0f;
    }
    return src;
}
// The wave's segment as it is loaded: 16-byte vectors, lane l the vectors l, 64 + l, ... of the segment, so that every
// load instruction of the wave covers consecutive memory.  x[k E + q] is element (k 64 + l) E + q of the segment
// (E elements per vector: 4 for fp32 logits, 8 for bf16); -inf past the row's end.
template <int ES>
__device__ __forceinline__ int seg_elem(int seg, int lane, int slot_kq)
{
    constexpr int E = 16 / ES;
    return seg * SR_SEG_TERMS + ((slot_kq / E) * SR_WAVE + lane) * E + (slot_kq % E);
}
template <int ES>
__device__ __forceinline__ void seg_load_logits(const SegSource<ES>& src, int seg, int lane, int n, float (&x)[SR_SEQ_RUN])
{
    constexpr int E = 16 / ES, K = SR_SEG_TERMS / (SR_WAVE * E);
    static_assert(K * E == SR_SEQ_RUN, "sixteen elements per lane");
    if ((seg + 1) * SR_SEG_TERMS <= n) {
        // a whole segment (all but a row's last): every load is issued before anything is done with one of them
        if (src.rowp) {
            uint4 raw[K];
            uint32_t keep[K];
#pragma unroll
            for (int k = 0; k < K; k++) {
                const int i0 = seg * SR_SEG_TERMS + (k * SR_WAVE + lane) * E;
                raw[k] = *(const uint4*)(src.rowp + (size_t)i0 * ES);
                keep[k] = 0xffffffffu;
                if (src.mrow) keep[k] = src.mrow[i0 >> 5] >> (i0 & 31);
            }
#pragma unroll
            for (int k = 0; k < K; k++) {
                float* xv = &x[k * E];
                if (ES == 4) {
                    xv[0] = sr_u2f(raw[k].x); xv[1] = sr_u2f(raw[k].y); xv[2] = sr_u2f(raw[k].z); xv[3] = sr_u2f(raw[k].w);
                } else {
                    const uint32_t r[4] = {raw[k].x, raw[k].y, raw[k].z, raw[k].w};
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        xv[(2 * q) % E] = sr_u2f(r[q] << 16);
                        xv[(2 * q + 1) % E] = sr_u2f(r[q] & 0xffff0000u);
                    }
                }
#pragma unroll
                for (int q = 0; q < E; q++) {
                    const float v = ((keep[k] >> q) & 1u) ? xv[q] : SR_NEG_INF;
                    xv[q] = src.scale ? __fmul_rn(v, src.inv_temp) : v;
                }
            }
        } else {
            float4 rw[K * E / 4];
#pragma unroll
            for (int k = 0; k < K; k++)
#pragma unroll
                for (int q4 = 0; q4 < E / 4; q4++)
                    rw[k * (E / 4) + q4] = *(const float4*)(src.w + seg * SR_SEG_TERMS + (k * SR_WAVE + lane) * E + 4 * q4);
#pragma unroll
            for (int v = 0; v < K * E / 4; v++) {
                x[4 * v] = rw[v].x; x[4 * v + 1] = rw[v].y; x[4 * v + 2] = rw[v].z; x[4 * v + 3] = rw[v].w;
            }
        }
        return;
    }
#pragma unroll
    for (int k = 0; k < K; k++) {
        const int i0 = seg * SR_SEG_TERMS + (k * SR_WAVE + lane) * E;
        float* xv = &x[k * E];
        if (i0 >= n) {
#pragma unroll
            for (int q = 0; q < E; q++) xv[q] = SR_NEG_INF;
            continue;
        }
        const bool whole = i0 + E <= n;
        if (!src.rowp) {  // the adjusted copy
#pragma unroll
            for (int q4 = 0; q4 < E; q4 += 4) {
                if (whole) {
                    const float4 v = *(const float4*)(src.w + i0 + q4);
                    xv[q4] = v.x; xv[q4 + 1] = v.y; xv[q4 + 2] = v.z; xv[q4 + 3] = v.w;
                } else {
#pragma unroll
                    for (int q = q4; q < q4 + 4; q++) xv[q] = (i0 + q < n) ? src.w[i0 + q] : SR_NEG_INF;
                }
            }
            continue;
        }
        uint32_t keep = (1u << E) - 1u;
        if (src.mrow) keep = src.mrow[i0 >> 5] >> (i0 & 31);
        if (whole) {
            const uint4 v = *(const uint4*)(src.rowp + (size_t)i0 * ES);
            if (ES == 4) {
                xv[0] = sr_u2f(v.x); xv[1] = sr_u2f(v.y); xv[2] = sr_u2f(v.z); xv[3] = sr_u2f(v.w);
            } else {
                const uint32_t r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    xv[(2 * q) % E] = sr_u2f(r[q] << 16);
                    xv[(2 * q + 1) % E] = sr_u2f(r[q] & 0xffff0000u);
                }
            }
        } else {
#pragma unroll
            for (int q = 0; q < E; q++) xv[q] = (i0 + q < n) ? load_logit<ES>(src.rowp, i0 + q) : 0.0f;
        }
#pragma unroll
        for (int q = 0; q < E; q++) {
            float v = ((keep >> q) & 1u) ? xv[q] : SR_NEG_INF;
            if (src.scale) v = __fmul_rn(v, src.inv_temp);
            xv[q] = (i0 + q < n) ? v : SR_NEG_INF;
        }
    }
}
// The ids of segment `seg` that the row's edits touch (a row that keeps no adjusted copy): their values in x, as
// seg_load_logits left them, are replaced by the adjusted ones -- LogitBias and the history penalties on the masked
// logit, then the temperature (Sampler.cs:51-58, :367-419).  entry(i, id, e) names the i-th candidate of `count`: an id and
// its place in the row's edit list; 64 candidates at a time, a lane each, then the owners of the hits take them one
// by one.
template <int ES, typename Entry>
__device__ __forceinline__ void seg_apply_edits(const SrFullArgs& a, const SrRow& rd, const SegSource<ES>& src, int seg, int lane,
                                                int count, Entry entry, float (&x)[SR_SEQ_RUN])
{
    constexpr int E = 16 / ES;
    const SrEdit* ed = a.edits + rd.edit_off;
    const bool pen = (rd.flags & SR_ROWFLAG_HAS_PENALTY) != 0u;
    const int lo = seg * SR_SEG_TERMS;
    for (int base = 0; base < count; base += SR_WAVE) {
        int id = -1;
        float val = 0.0f;
        if (base + lane < count) {
            int e = 0;
            entry(base + lane, id, e);
            if (id >= lo && id < lo + SR_SEG_TERMS && id < a.vocab) {
                float v = load_logit<ES>(src.rowp, id);
                if (src.mrow && !((src.mrow[id >> 5] >> (id & 31)) & 1u)) v = SR_NEG_INF;
                v = edited_logit(v, ed[e], rd, true, pen);
                val = src.scale ? __fmul_rn(v, src.inv_temp) : v;
            } else {
                id = -1;
            }
        }
        unsigned long long todo = __ballot(id >= 0);
        while (todo != 0ull) {
            const int h = __ffsll((long long)todo) - 1;
            todo &= todo - 1ull;
            const int local = __shfl(id, h) - lo;
            const float vh = __shfl(val, h);
            const int v = local / E, j = (v / SR_WAVE) * E + local % E;
            const bool mine = lane == v % SR_WAVE;
#pragma unroll
            for (int jj = 0; jj < SR_SEQ_RUN; jj++) x[jj] = (mine && jj == j) ? vh : x[jj];
        }
    }
}

// Both passes are one launch (k_full_softmax_seg): a wave keeps its segments in registers in between, so the logits
// are read once.  The workgroups of a row meet between the passes: each leaves its segments' maxima and approximate
// sums, counts itself in (SR_ROW_SYNC_STRIDE), and waits until the row's count is full.  Workgroups start in the order
// of their numbers, a row's side by side, so those that a waiting workgroup waits for are running or next to start;
// the wait is bounded all the same.  A workgroup whose wait runs out marks its segments (SR_SEG_LATE) and leaves;
// whichever workgroup of the row is the last to get behind the meeting point -- the row's maxima are all in then --
// finds the marks and finishes those segments, whose inputs nobody has touched.  What a segment gets is the same
// whichever way it is finished.
struct SegPass2 {
    const uint64_t* tab;   // the expf table in shared memory
    float4* turn;          // the wave's SR_WAVE * 5 vectors of shared memory
    float* w;
    uint16_t* keys;
    bool watch;
    float e_low, m;
    int slot, n;
};
// e = expf(x - m) of one segment (x as seg_load_logits left it): written to the work row, its 16-bit keys and the
// entries a min-p cut watches where the row asks for them, and the segment's record
template <int ES>
__device__ __forceinline__ void seg_pass2(const SrFullArgs& a, const SegPass2& c, int seg, int lane, const float (&x)[SR_SEQ_RUN],
                                          float before, float own_sum)
{
    constexpr int E = 16 / ES, K = SR_SEG_TERMS / (SR_WAVE * E);
    const int n = c.n;
    float e[SR_SEQ_RUN];
    // (a whole segment without a test per element: the 16 chains of a lane then run interleaved)
    if ((seg + 1) * SR_SEG_TERMS <= n) {
#pragma unroll
        for (int j = 0; j < SR_SEQ_RUN; j++) e[j] = sr_expf_tab(__fsub_rn(x[j], c.m), c.tab);
    } else {
#pragma unroll
        for (int k = 0; k < K; k++)
#pragma unroll
            for (int q = 0; q < E; q++) {
                const int i = seg * SR_SEG_TERMS + (k * SR_WAVE + lane) * E + q;
                e[k * E + q] = i < n ? sr_expf_tab(__fsub_rn(x[k * E + q], c.m), c.tab) : 0.0f;
            }
    }
#pragma unroll
    for (int k = 0; k < K; k++) {
        const int i0 = seg * SR_SEG_TERMS + (k * SR_WAVE + lane) * E;
        if (i0 + E <= n) {
#pragma unroll
            for (int q = 0; q < E; q += 4)
                *(float4*)(c.w + i0 + q) = make_float4(e[k * E + q], e[k * E + q + 1], e[k * E + q + 2], e[k * E + q + 3]);
        } else {
#pragma unroll
            for (int q = 0; q < E; q++)
                if (i0 + q < n) c.w[i0 + q] = e[k * E + q];
        }
        if (c.keys) {
            uint32_t kk[E];
#pragma unroll
            for (int q = 0; q < E; q++) kk[q] = e[k * E + q] > 0.0f ? max(sr_f2u(e[k * E + q]) >> 16, 1u) : 0u;
            if (i0 + E <= n) {
#pragma unroll
                for (int q = 0; q < E; q += 4)
                    *(uint2*)(c.keys + i0 + q) = make_uint2(kk[q] | (kk[q + 1] << 16), kk[q + 2] | (kk[q + 3] << 16));
            } else {
#pragma unroll
                for (int q = 0; q < E; q++)
                    if (i0 + q < n) c.keys[i0 + q] = (uint16_t)kk[q];
            }
        }
        if (c.watch) {
#pragma unroll
            for (int q = 0; q < E; q++)
                if (e[k * E + q] >= c.e_low && i0 + q < n) {
                    const uint32_t pos = atomicAdd(&a.watch_cnt[c.slot], 1u);
                    if (pos < (uint32_t)kSmall)
                        a.watch[(size_t)c.slot * kSmall + pos] = ((unsigned long long)sr_f2u(e[k * E + q]) << 32) |
                                                                 (unsigned long long)(0xffffffffu - (uint32_t)(i0 + q));
                }
        }
    }
    // through shared memory into the order of the sum: lane l gets the terms 16 l ... 16 l + 15 of the segment (only
    // this wave touches its part: the wave's own order of shared-memory operations is all it needs)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
    for (int k = 0; k < K; k++)
#pragma unroll
        for (int q = 0; q < E; q += 4) {
            const int i = (k * SR_WAVE + lane) * E + q;  // the element's place in the segment
            c.turn[(i >> 4) * 5 + ((i & 15) >> 2)] = make_float4(e[k * E + q], e[k * E + q + 1], e[k * E + q + 2], e[k * E + q + 3]);
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float t[SR_SEQ_RUN];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const float4 v = c.turn[lane * 5 + k];
        t[4 * k] = v.x; t[4 * k + 1] = v.y; t[4 * k + 2] = v.z; t[4 * k + 3] = v.w;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    seg_make_record(t, seg, (double)before, a.seg_func + (size_t)c.slot * a.seg_stride + seg, own_sum);
}
// a segment's own maximum (as an ordered key; 0xffffffff = it holds a NaN) and the sum of exp(x - that maximum)
__device__ __forceinline__ unsigned long long seg_pass1(const float (&x)[SR_SEQ_RUN])
{
    uint32_t k = 0u;
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const uint32_t kv = (x[j] != x[j]) ? 0xffffffffu : sr_okey(x[j]);  // NaN propagates (TensorPrimitives.Max)
        k = kv > k ? kv : k;
    }
    k = sr_wave_max_u32(k);
    float sum = 0.0f;
    if (k != 0xffffffffu && k > 0x007fffffu) {
        const float m = sr_okey_inv(k);
#pragma unroll
        for (int j = 0; j < 16; j++) sum += __expf(x[j] - m);
    }
    sum = sr_wave_sum_f32(sum);
    return ((unsigned long long)sr_f2u(sum) << 32) | (unsigned long long)k;
}
// what a segment's (maximum, sum) adds to the row's approximate sum when the row's maximum is m
__device__ __forceinline__ float seg_share(unsigned long long ms, float m)
{
    const uint32_t k = (uint32_t)ms;
    const float sum = sr_u2f((uint32_t)(ms >> 32));
    return (sum > 0.0f && k != 0xffffffffu) ? sum * __expf(sr_okey_inv(k) - m) : 0.0f;
}
template <int ES, int kW, int kS>
__global__ __launch_bounds__(kW * SR_WAVE, kS == 2 ? 5 : 3) void k_full_softmax_seg(SrFullArgs a)
{
    constexpr int kThreads = kW * SR_WAVE;
    const int slot = blockIdx.y, lane = sr_lane(), wave = sr_wave_id();
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    if (rd.temperature <= 0.0f) return;  // greedy rows keep their logits
    __shared__ uint64_t tab[32];  // the expf table: a lookup per element from global memory is a long dependent load
    // a wave's segment on its way from the order of the loads to 16 terms a lane: a lane's 16 terms lie together, 16
    // bytes apart from the next lane's, so that neither the stores nor the loads of 16 bytes a lane collide on a bank
    __shared__ float4 turn[kW][SR_WAVE * 5];
    __shared__ float share[SR_SEG_MAX];  // every segment's part of the row's approximate sum
    __shared__ uint32_t wkey[kW];
    __shared__ uint32_t bc[2];           // 0: the row's count came in   1: what k_full_edits made the row's maximum
    // the row's edits that fall into this workgroup's segments (id << 32 | place in the row's edit list), and how many
    // there are (more than the list holds: the waves go through the row's whole edit list instead)
    constexpr int kHitCap = 256;
    __shared__ unsigned long long hits[kHitCap];
    __shared__ uint32_t n_hits;
    const int n = a.vocab, nseg = seg_count(n);
    SrFullState* st = a.state + slot;
    unsigned long long* sync = a.row_sync + (size_t)slot * SR_ROW_SYNC_STRIDE;
    unsigned long long* ms = (unsigned long long*)(a.seg_ms + (size_t)slot * a.seg_stride);
    const unsigned long long stamp = (unsigned long long)a.seq << 32;
    SeqSegFunc* recs = a.seg_func + (size_t)slot * a.seg_stride;
    if (threadIdx.x < 32) tab[threadIdx.x] = sr_exp2f_tab[threadIdx.x];
    const SegSource<ES> src = seg_source<ES>(rd, a, slot, row);
    SegPass2 c;
    c.tab = tab;
    c.turn = turn[wave];
    c.w = a.work + (size_t)(a.work_by_row ? row : slot) * a.work_stride;
    // (a row that only top-p cuts needs the histogram of its e by their upper 16 bits: counting it here, one atomic per
    // element, took longer than it saved, so the pass leaves those 16 bits of every e beside the row, and the row's
    // workgroup counts them -- half the bytes of the row -- while one of its waves walks the sum)
    c.keys = (row_fast_nucleus(rd, a) && a.seg_keys) ? a.seg_keys + (size_t)slot * (size_t)a.seg_key_stride : nullptr;
    c.watch = row_watch_min_p(rd, a);
    c.e_low = __fmul_rn(rd.min_p, 0.999999f);
    c.slot = slot;
    c.n = n;
    c.m = 0.0f;

    // the first pass: the segment's maximum and approximate sum, written through for the row's other workgroups
    // A row that keeps no adjusted copy although bias or penalties touch some of its ids: the workgroup looks through
    // the row's edit list for the ids of its own segments, and its waves put the adjusted values in place of what they load
    // (the ids are asked for in front of the logits and looked at behind them: the loads overlap)
    const bool edits = src.rowp != nullptr && rd.edit_cnt > 0;
    const SrEdit* ed = a.edits + rd.edit_off;
    constexpr int kIds = SR_FULL_EDIT_VALUES / kThreads;
    static_assert(kIds * kThreads == SR_FULL_EDIT_VALUES, "every edit of a row without an adjusted copy is looked at");
    int ids[kIds];
    if (edits) {
        if (threadIdx.x == 0) n_hits = 0u;
        sr_barrier_lds();
#pragma unroll
        for (int j = 0; j < kIds; j++) {
            const int e = (int)threadIdx.x + j * kThreads;
            ids[j] = e < rd.edit_cnt ? ed[e].id : -1;
        }
    }
    auto apply_edits = [&](int seg, float (&x)[SR_SEQ_RUN], bool from_hits) {
        if (from_hits && n_hits <= (uint32_t)kHitCap)
            seg_apply_edits<ES>(a, rd, src, seg, lane, (int)n_hits, [&](int i, int& id, int& e) {
                const unsigned long long h = hits[i];
                id = (int)(h >> 32);
                e = (int)(uint32_t)h;
            }, x);
        else
            seg_apply_edits<ES>(a, rd, src, seg, lane, rd.edit_cnt, [&](int i, int& id, int& e) {
                id = ed[i].id;
                e = i;
            }, x);
    };
    // (a wave takes kS segments, the workgroup's waves side by side: every one of its loads is out before the first is used)
    const int seg0 = (int)blockIdx.x * (kW * kS) + wave;
    float xs[kS][SR_SEQ_RUN];
#pragma unroll
    for (int s = 0; s < kS; s++)
        if (seg0 + s * kW < nseg) seg_load_logits<ES>(src, seg0 + s * kW, lane, n, xs[s]);
    if (edits) {
        const int lo = (int)blockIdx.x * (kW * kS) * SR_SEG_TERMS, hi = lo + kW * kS * SR_SEG_TERMS;
#pragma unroll
        for (int j = 0; j < kIds; j++) {
            if (ids[j] >= lo && ids[j] < hi) {
                const uint32_t pos = atomicAdd(&n_hits, 1u);
                if (pos < (uint32_t)kHitCap)
                    hits[pos] = ((unsigned long long)(uint32_t)ids[j] << 32) | (unsigned long long)(uint32_t)((int)threadIdx.x + j * kThreads);
            }
        }
        sr_barrier_lds();
#pragma unroll
        for (int s = 0; s < kS; s++)
            if (seg0 + s * kW < nseg) apply_edits(seg0 + s * kW, xs[s], true);
    }
#pragma unroll
    for (int s = 0; s < kS; s++)
        if (seg0 + s * kW < nseg) {
            const unsigned long long v = seg_pass1(xs[s]);
            if (lane == 0) sr_store_agent(&ms[seg0 + s * kW], v);
        }
    sr_drain_stores();
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_max(sync, stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_fetch_add(sync, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long edited = sr_load_agent(&st->maxkey);  // (final: k_full_edits ran before)
        uint32_t ok = 0u;
        for (uint32_t it = 0; it < a.row_wait_limit; it++) {
            const unsigned long long v = sr_load_agent(sync);
            if ((uint32_t)(v >> 32) == a.seq && (uint32_t)(v & 0xffffu) == gridDim.x) { ok = 1u; break; }
            __builtin_amdgcn_s_sleep(8);
        }
        bc[0] = ok;
        bc[1] = full_maxkey_of(a, edited);
    }
    __syncthreads();
    const bool met = bc[0] != 0u;
    if (!met) {
        // the wait ran out: the segments are left, marked, to the last of the row's workgroups
#pragma unroll
        for (int s = 0; s < kS; s++)
            if (seg0 + s * kW < nseg && lane == 0) {
                sr_store_agent(&recs[seg0 + s * kW].kind, SR_SEG_LATE);
                sr_store_agent(&recs[seg0 + s * kW].a0, a.seq);
            }
        sr_drain_stores();
        __syncthreads();
        if (threadIdx.x == 0) {
            sr_store_agent(&st->late, a.seq);
            sr_drain_stores();
        }
    }
    // (the count as this workgroup found it is looked at behind the second pass: nothing waits for it here)
    unsigned long long behind = 0ull;
    if (threadIdx.x == 0) behind = __hip_atomic_fetch_add(sync, 1ull << 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    uint32_t mk = 0u;
    if (met) {
        // the row's maximum and the segments' shares of the approximate sum (single precision does: a prediction that
        // misses costs time only)
        constexpr int kPer = (SR_SEG_MAX + kThreads - 1) / kThreads;
        unsigned long long mv[kPer];
        uint32_t kk = 0u;
#pragma unroll
        for (int j = 0; j < kPer; j++) {
            const int g = (int)threadIdx.x + kThreads * j;
            mv[j] = g < nseg ? sr_load_agent(&ms[g]) : 0ull;
            kk = max(kk, (uint32_t)mv[j]);
        }
        kk = sr_wave_max_u32(kk);
        if (lane == 0) wkey[wave] = kk;
        __syncthreads();
        mk = bc[1];
#pragma unroll
        for (int j = 0; j < kW; j++) mk = max(mk, wkey[j]);
        if (blockIdx.x == 0 && threadIdx.x == 0 && mk != 0u) atomicMax(&st->maxkey, full_maxkey(a, mk));  // for the row's kernel
        if (mk != 0xffffffffu && mk > 0x007fffffu) {  // (else a NaN, or nothing above -inf: the row kernel makes it uniform)
            c.m = sr_okey_inv(mk);
#pragma unroll
            for (int j = 0; j < kPer; j++) {
                const int g = (int)threadIdx.x + kThreads * j;
                if (g < nseg) share[g] = seg_share(mv[j], c.m);
            }
            __syncthreads();
#pragma unroll
            for (int s = 0; s < kS; s++) {
                const int seg = seg0 + s * kW;
                if (seg < nseg) {
                    float before = 0.0f;
                    for (int g = lane; g < seg; g += SR_WAVE) before += share[g];
                    before = sr_wave_sum_f32(before);
                    seg_pass2<ES>(a, c, seg, lane, xs[s], before, share[seg]);
                }
            }
        }
    }
    if (wave != 0) return;

    // The last of the row's workgroups to get behind the meeting point finishes what others left: one wave, segment by
    // segment.  (Every workgroup's first pass is complete by then, and the marks were written before their workgroup
    // counted itself.)
    const uint32_t was = __shfl((uint32_t)(behind >> 16) & 0xffffu, 0);
    if (was != gridDim.x - 1u) return;
    if (sr_load_agent(&st->late) != a.seq) return;
    if (!met) {
        uint32_t kk = bc[1];
        for (int g = lane; g < nseg; g += SR_WAVE) kk = max(kk, (uint32_t)sr_load_agent(&ms[g]));
        mk = sr_wave_max_u32(kk);
    }
    // (the row's first workgroup, which leaves the maximum for the row's kernel, may be one of those that left)
    if (lane == 0 && mk != 0u) atomicMax(&st->maxkey, full_maxkey(a, mk));
    if (mk == 0xffffffffu || mk <= 0x007fffffu) return;
    if (!met) {
        c.m = sr_okey_inv(mk);
        for (int g = lane; g < nseg; g += SR_WAVE) share[g] = seg_share(sr_load_agent(&ms[g]), c.m);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    for (int g = 0; g < nseg; g++) {
        uint32_t kind = 0u, whose = 0u;
        if (lane == 0) {
            kind = sr_load_agent(&recs[g].kind);
            whose = sr_load_agent(&recs[g].a0);
        }
        kind = __shfl(kind, 0);
        whose = __shfl(whose, 0);
        if (kind != SR_SEG_LATE || whose != a.seq) continue;
        seg_load_logits<ES>(src, g, lane, n, xs[0]);
        if (edits) apply_edits(g, xs[0], false);  // (the list in shared memory is of this workgroup's own segments)
        float before = 0.0f;
        for (int h = lane; h < g; h += SR_WAVE) before += share[h];
        before = sr_wave_sum_f32(before);
        seg_pass2<ES>(a, c, g, lane, xs[0], before, share[g]);
    }
}

// ---- argmax of an fp32 row: first index of the maximum, first NaN wins -------------------------------
__device__ __forceinline__ int row_argmax(const float* w, int n, FullSmem& sm)
{
    unsigned long long best = 0ull;
    row_pass<false>(const_cast<float*>(w), n, [&](float v, int i) -> float {
        const uint32_t k = (v != v) ? 0xffffffffu : sr_okey(v);
        const unsigned long long e = ((unsigned long long)k << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
        best = e > best ? e : best;
        return v;
    });
    best = blk_max_u64(best, sm);
    return best ? (int)(0xffffffffu - (uint32_t)(best & 0xffffffffull)) : 0;
}

// first index whose running fp32 sum reaches r = (float)u; last index as the rounding fallback
// (SampleFromDistribution, Sampler.cs:564-576)
__device__ __forceinline__ int draw_from_row(const float* p, int n, double u, FullSmem& sm, float m1 = 1.0f, float m2 = 1.0f)
{
    const float r = __double2float_rn(u);
    int found;
    const float at = seq_sum_row<true>(p, n, 0.0f, r, &found, sm, m1, m2);
    if (threadIdx.x == 0)
        SR_AMB_IF(found >= 0 ? sr_stop_near(at, __fmul_rn(__fmul_rn(p[found], m1), m2), r) : sr_near(at, r));
    return found >= 0 ? found : n - 1;
}

// Final Normalize (Sampler.cs:91-92, :553-562) and draw (:564-576) of a row whose survivors are listed in index order
// in sm.sortbuf[0, m) (~index << 32 | probability bits; an entry with probability bits of zero is no survivor) and
// whose other entries are all zero.  Adding zero changes no running sum, so the eight strided chains of
// TensorPrimitives.Sum (plus its overlapped tail) and the running sum of the draw are taken over the survivors alone,
// in index order: a chain's terms are the survivors whose index falls on it, and the tail's indices lie behind every
// body index, so one order serves all eight chains.  Behind a barrier that follows the last write of the list.
// A list of more than kSmall entries comes through sm.sortbuf a block of kSmall at a time: fill(first, count), called
// by all threads between two barriers, puts the entries [first, first + count) at sm.sortbuf[0, count).  A list that is
// in sm.sortbuf already has m <= kSmall and a fill that does nothing.
struct NoFill {
    __device__ __forceinline__ void operator()(int, int) const {}
};
template <typename Fill = NoFill>
__device__ __forceinline__ void finish_from_ordered_list(const SrFullArgs& a, float* p, int n, int m, int row, FullSmem& sm,
                                                         Fill fill = Fill(), int cap = kSmall)
{
    // (cap: what a list that is in shared memory already may hold -- kSmall, or 2 kSmall where the launch gave the
    // workgroup the room: the list then runs on from sm.sortbuf through the two arrays behind it)
    constexpr bool kResident = std::is_same<Fill, NoFill>::value;
    constexpr int kPerT = 2 * kSmall / kT;
    unsigned long long* const buf = &sm.sortbuf[0];
    const int cpt = (kResident ? cap : kSmall) / kT;  // entries per thread of the list's new layout
    const int nv8 = (n / 8) * 8;
    const int lane = sr_lane(), wave = sr_wave_id();
    // One wave per chain: it passes over the whole list in index order, sixteen entries per lane at a time, with the
    // entries of the other chains as zeros.
    // A lane's sixteen consecutive entries would all lie in the same LDS banks as every other lane's: inside each
    // thousand entries the list is laid out anew, entry 16 l + j at place 64 j + l.
    auto place_of = [](int i) -> int { return (i & ~1023) | ((i & 15) << 6) | ((i >> 4) & 63); };
    auto lay_out = [&]() __attribute__((always_inline)) {
        static_assert(kSmall == 4 * kT, "four entries per thread, or eight");
        unsigned long long t[kPerT];
#pragma unroll
        for (int r = 0; r < kPerT; r++) t[r] = r < cpt ? buf[cpt * (int)threadIdx.x + r] : 0ull;
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kPerT; r++)
            if (r < cpt) buf[place_of(cpt * (int)threadIdx.x + r)] = t[r];
        __syncthreads();
    };
    auto load_terms = [&](int i0, int cnt, int chain, float mul, bool scale, float (&x)[16]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int i = i0 + j;
            const unsigned long long v = i < cnt ? buf[place_of(i)] : 0ull;
            const int e = (int)(0xffffffffu - (uint32_t)(v >> 32));
            const bool mine = chain < 0 || (e < nv8 ? (e & 7) : e - (n - 8)) == chain;
            const float t = sr_u2f((uint32_t)v);
            x[j] = (i < cnt && mine) ? (scale ? __fmul_rn(t, mul) : t) : 0.0f;
        }
    };
    if (kResident && m <= SR_WAVE) {
        // A short list: one thread per chain adds its members as they come, and one thread draws.
        const int tid = threadIdx.x;
        if (tid < SR_SEQ_CHAINS) {
            float s = 0.0f;
            for (int i = 0; i < m; i++) {
                const unsigned long long v = sm.sortbuf[i];
                const int e = (int)(0xffffffffu - (uint32_t)(v >> 32));
                const int chain = e < nv8 ? (e & 7) : e - (n - 8);
                if (chain == tid) s = __fadd_rn(s, sr_u2f((uint32_t)v));
            }
            sm.lane_sum[tid] = s;
        }
        __syncthreads();
        const float l0 = sm.lane_sum[0], l1 = sm.lane_sum[1], l2 = sm.lane_sum[2], l3 = sm.lane_sum[3],
                    l4 = sm.lane_sum[4], l5 = sm.lane_sum[5], l6 = sm.lane_sum[6], l7 = sm.lane_sum[7];
        const float sum = __fadd_rn(__fadd_rn(__fadd_rn(l0, l1), __fadd_rn(l2, l3)), __fadd_rn(__fadd_rn(l4, l5), __fadd_rn(l6, l7)));
        const bool scale = sum > 0.0f && sum != 1.0f;
        const float inv = scale ? __fdiv_rn(1.0f, sum) : 1.0f;
        if (a.mode != 0 && scale) row_pass<true>(p, n, [&](float x, int) -> float { return __fmul_rn(x, inv); });
        if (a.mode != 1 && tid == 0) {
            const float r = __double2float_rn(a.uniforms[(size_t)row * a.uniforms_per_row]);
            int token = n - 1;
            if (!(r > 0.0f)) {
                token = 0;  // the running sum starts at p[0] >= 0: index 0 reaches a target of zero whatever it holds
            } else {
                float acc = 0.0f;
                bool hit = false;
                for (int i = 0; i < m && !hit; i++) {
                    const unsigned long long v = sm.sortbuf[i];
                    const float x = sr_u2f((uint32_t)v), xs = scale ? __fmul_rn(x, inv) : x;
                    acc = __fadd_rn(acc, xs);
                    if (acc >= r) {
                        token = (int)(0xffffffffu - (uint32_t)(v >> 32));
                        hit = true;
                        SR_AMB_IF(sr_stop_near(acc, xs, r));
                    }
                }
                if (!hit) SR_AMB_IF(sr_near(acc, r));
            }
            if (a.out_tokens) a.out_tokens[row] = token;
        }
        return;
    }
    float sc = 0.0f;
    if (kResident) lay_out();
    const int step = kResident ? cap : kSmall;  // (a resident list is one block)
    for (int first = 0; first < m; first += step) {
        const int cnt = min(step, m - first);
        if (!kResident) {
            __syncthreads();
            fill(first, cnt);
            __syncthreads();
            lay_out();
        }
        if (wave < SR_SEQ_CHAINS) {
            for (int b0 = 0; b0 < cnt; b0 += 16 * SR_WAVE) {
                float x[16];
                load_terms(b0 + 16 * lane, cnt, wave, 1.0f, false, x);
                int dummy;
                sc = sr_seq_wave<16, false>(x, sc, 0.0f, &dummy);
            }
        }
    }
    if (wave < SR_SEQ_CHAINS && lane == 0) sm.lane_sum[wave] = sc;
    __syncthreads();
    FPROF(a, blockIdx.x, 18);
    const float l0 = sm.lane_sum[0], l1 = sm.lane_sum[1], l2 = sm.lane_sum[2], l3 = sm.lane_sum[3],
                l4 = sm.lane_sum[4], l5 = sm.lane_sum[5], l6 = sm.lane_sum[6], l7 = sm.lane_sum[7];
    const float sum = __fadd_rn(__fadd_rn(__fadd_rn(l0, l1), __fadd_rn(l2, l3)), __fadd_rn(__fadd_rn(l4, l5), __fadd_rn(l6, l7)));
    const bool scale = sum > 0.0f && sum != 1.0f;
    const float inv = scale ? __fdiv_rn(1.0f, sum) : 1.0f;
    if (a.mode != 0 && scale) row_pass<true>(p, n, [&](float x, int) -> float { return __fmul_rn(x, inv); });
    if (a.mode == 1) return;
    const float r = __double2float_rn(a.uniforms[(size_t)row * a.uniforms_per_row]);
    int token = n - 1;
    bool done = false;  // (what wave 0 knows)
    if (!(r > 0.0f)) {
        token = 0;  // the running sum starts at p[0] >= 0: index 0 reaches a target of zero whatever it holds
        done = true;
    }
    float acc = 0.0f;
    for (int first = 0; first < m; first += step) {
        const int cnt = min(step, m - first);
        if (!kResident) {
            if (wave == 0 && lane == 0) sm.bc[10] = done ? 1u : 0u;
            __syncthreads();
            if (sm.bc[10] != 0u) break;
            fill(first, cnt);
            __syncthreads();
            lay_out();
        }
        if (wave == 0 && !done) {
            for (int b0 = 0; b0 < cnt; b0 += 16 * SR_WAVE) {
                float x[16];
                load_terms(b0 + 16 * lane, cnt, -1, inv, scale, x);
                int f;
                acc = sr_seq_wave<16, true>(x, acc, r, &f);
                if (f >= 0) {
                    const unsigned long long v = buf[place_of(b0 + f)];
                    token = (int)(0xffffffffu - (uint32_t)(v >> 32));
                    done = true;
                    const float t = sr_u2f((uint32_t)v);
                    SR_AMB_IF(lane == 0 && sr_stop_near(acc, scale ? __fmul_rn(t, inv) : t, r));
                    break;
                }
            }
        }
    }
    if (wave == 0 && lane == 0) {
        SR_AMB_IF(!done && sr_near(acc, r));  // (the draw ran off the end of the list: the last index, by the rounding fallback)
        if (a.out_tokens) a.out_tokens[row] = token;
    }
}
// ... of a list in any order, its entries as probability bits << 32 | ~index
__device__ __forceinline__ void finish_from_list(const SrFullArgs& a, float* p, int n, int m, int row, FullSmem& sm)
{
    const int tid = threadIdx.x;
    int P = 2;
    while (P < m) P <<= 1;
    __syncthreads();
    for (int i = tid; i < P; i += kT) {
        const unsigned long long v = sm.sortbuf[i];
        sm.sortbuf[i] = (i < m) ? ((v & 0xffffffffull) << 32) | (v >> 32) : 0ull;  // ~index on top: descending = index ascending
    }
    __syncthreads();
    sort_small_desc(sm, P);
    finish_from_ordered_list(a, p, n, m, row, sm);
}

// Every wave passes over its stretch [w0, w1) of a row (w0 a multiple of 4) and hands the entries for which pred(y, i)
// holds to a sink, in index order -- y being the entry times inv (the entry itself without do_scale).  Returns the
// wave's count.  The loads of the next thousand entries are on their way while a thousand are looked at.
//   sink.reserve(before, count)   room for `count` more finds of this wave, `before` found so far: the first one's place
//   sink.put(place, rank, y bits, index)   rank = the find's number within the wave
// The pass is bound by its instructions, not by memory: about 8 us for a row of 151,936 entries with few finds, 30 us
// when every 256 entries hold some.
struct StretchToSegment {  // at the stretch's own positions of the row's sort segment
    uint32_t* gk;
    int32_t* gi;
    int w0;
    __device__ __forceinline__ int reserve(int before, int) const { return w0 + before; }
    __device__ __forceinline__ void put(int place, int, uint32_t ybits, int i) const { gk[place] = ybits; gi[place] = i; }
};
struct StretchToPool {  // appended to a pool in LDS that all waves share: values to vals, tags to tags
    uint32_t* counter;
    uint32_t* vals;
    uint32_t* tags;
    int cap;  // entries the pool holds
    __device__ __forceinline__ int reserve(int, int count) const
    {
        int b = 0;
        if (sr_lane() == 0) b = (int)atomicAdd(counter, (uint32_t)count);
        return __builtin_amdgcn_readfirstlane(b);
    }
    __device__ __forceinline__ void put(int place, int rank, uint32_t ybits, int i) const
    {
        if (place < cap) { vals[place] = ybits; tags[place] = ((uint32_t)rank << kTagIndexBits) | (uint32_t)i; }
    }
};
struct StretchCount {  // nothing is kept: the wave's count is what list_stretch returns
    __device__ __forceinline__ int reserve(int, int) const { return 0; }
    __device__ __forceinline__ void put(int, int, uint32_t, int) const {}
};
struct StretchFind {  // the index of the wave's find number `target` (none for a negative target)
    int target;
    uint32_t* out;
    __device__ __forceinline__ int reserve(int, int) const { return 0; }
    __device__ __forceinline__ void put(int, int rank, uint32_t, int i) const
    {
        if (rank == target) *out = (uint32_t)i;
    }
};
template <typename Sink, typename Pred>
__device__ __forceinline__ int list_stretch(const float* p, int w0, int w1, bool do_scale, float inv, Sink sink, Pred pred)
{
    const int lane = sr_lane();
    const bool aligned = ((uintptr_t)p & 15u) == 0u;
    int cw = 0;
    auto load = [&](int i0, float (&v)[4][4]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = i0 + u * 256 + 4 * lane;
            if (aligned && i + 4 <= w1) {
                const float4 t = *(const float4*)(p + i);
                v[u][0] = t.x; v[u][1] = t.y; v[u][2] = t.z; v[u][3] = t.w;
            } else {
#pragma unroll
                for (int k = 0; k < 4; k++) v[u][k] = (i + k < w1) ? p[i + k] : 0.0f;
            }
        }
    };
    auto look = [&](int i0, const float (&v)[4][4]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = i0 + u * 256 + 4 * lane;
            float y[4];
            bool pr[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                y[k] = do_scale ? __fmul_rn(v[u][k], inv) : v[u][k];
                pr[k] = i + k < w1 && pred(y[k], i + k);
            }
            if (__ballot(pr[0] || pr[1] || pr[2] || pr[3]) == 0ull) continue;
            int before = 0, total = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const unsigned long long b = __ballot(pr[k]);
                before += (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(b >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)b, 0u));
                total += __popcll(b);
            }
            int place = sink.reserve(cw, total) + before, rank = cw + before;
#pragma unroll
            for (int k = 0; k < 4; k++)
                if (pr[k]) { sink.put(place, rank, sr_f2u(y[k]), i + k); place++; rank++; }
            cw += total;
        }
    };
    if (w0 >= w1) return 0;
    float va[4][4], vb[4][4];
    load(w0, va);
    for (int i0 = w0; i0 < w1; i0 += 2048) {
        // (the scheduling barriers keep the loads where they are written: left alone, the compiler moves them down
        // to where their values are used, and every thousand entries wait for memory once more)
        if (i0 + 1024 < w1) load(i0 + 1024, vb);
        __builtin_amdgcn_sched_barrier(0);
        look(i0, va);
        if (i0 + 1024 >= w1) break;
        if (i0 + 2048 < w1) load(i0 + 2048, va);
        __builtin_amdgcn_sched_barrier(0);
        look(i0 + 1024, vb);
    }
    return cw;
}

// ---- the nucleus of a row that only top-p cuts, without a pass that writes the row ---------------------------------
// The row holds e = expf(x - max); its probabilities are y = fl(e * inv) (y = e when the sum is 1), which rise with e.
// While the exact sum passed over the row, the caller counted the e by their upper 16 bits in hcnt (LDS, kHistPos
// positions: position d holds the keys 0x3f80 - d, position 0 is e = 1, the last position everything below).  From the
// counts: the longest run of positions from the top that holds at most kSmall entries (a slab), the first one shortened
// to where a lower bound of its probability mass (count x the position's smallest value) passes top_p with a margin.
// One read of the row lists a slab's entries (every wave takes a stretch of the row; the finds go to a pool in LDS
// with their number within the wave, from which their places in index order follow); their values alone are sorted,
// the exact running sum goes on through them, and slab follows slab until it reaches top_p.  The members -- the values
// above the value at the cut and the first few equal to it by index -- are marked in the last slab's index-ordered
// list, from which a nucleus of one slab is finished; one of several slabs has its members listed by one more read
// of the row into the row's sort segment and is finished from there a block at a time.  Returns kNucleusDone, or
// which general way the row has to go (nothing is written then but LDS and the row's sort segment).
enum NucleusWay : int { kNucleusDone = 0, kNucleusGeneral = 1, kNucleusGeneralNoSlabs = 2 };
constexpr int kNucleusMaxSlabs = 40;
constexpr int kNucleusRowFinish = 4;  // a nucleus that took more slabs than this is finished by passes over the row
// `extra`: 16 kSmall bytes of shared memory beyond sm, or null.  With them a slab holds 2 kSmall entries -- most nuclei of
// a few thousand entries then close in one slab, which is listed by one read of the row and finished from the list,
// where two slabs cost three reads --: the pool of values and tags lies there, and the lists that are sm.sortbuf
// otherwise run on through the two arrays behind it.
__device__ __forceinline__ int nucleus_from_histogram(const SrFullArgs& a, float top_p, const float* p, int n, int slot,
                                                      int row, bool do_scale, float inv, FullSmem& sm, uint32_t* extra)
{
    constexpr int kPer = kHistPos / kT;
    static_assert(kHistPos * 4 <= kSmall * 8 && kHistPos % kT == 0, "the histogram fits the sort buffer");
    static_assert(offsetof(FullSmem, sprob) == offsetof(FullSmem, sortbuf) + sizeof(FullSmem::sortbuf) &&
                  offsetof(FullSmem, tags) == offsetof(FullSmem, sprob) + sizeof(FullSmem::sprob) &&
                  sizeof(FullSmem::sortbuf) + sizeof(FullSmem::sprob) + sizeof(FullSmem::tags) >= 2 * kSmall * sizeof(unsigned long long),
                  "a list of 2 kSmall entries fits the three arrays, which lie one behind the other");
    constexpr int kPerT = 2 * kSmall / kT;  // most entries of a slab per thread
    const int tid = threadIdx.x, lane = sr_lane(), wave = sr_wave_id();
    const int S = extra ? 2 * kSmall : kSmall;  // entries a slab may hold
    const int cpt = S / kT;
    const uint32_t* hcnt = (const uint32_t*)sm.sortbuf;
    uint32_t* sval = extra ? extra : (uint32_t*)sm.sprob;
    uint32_t* const tags = extra ? extra + 2 * kSmall : sm.tags;
    unsigned long long* const list = &sm.sortbuf[0];  // [S]
    [[maybe_unused]] unsigned long long t_step = 0ull;
    FPROF_ADD(a, slot, 16, t_step);
    if (sm.bc[5] != 0u) return kNucleusGeneral;
    // counts and mass bounds (in units of 2^-28) of this thread's positions
    uint32_t mine[kPer], mq[kPer];
    int own = 0;
    uint32_t ownq = 0u;
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        const int d = tid * kPer + j;
        mine[j] = hcnt[d];
        const float e_low = d < kHistPos - 1 ? sr_u2f((kHistTopKey - (uint32_t)d) << 16) : 0.0f;
        const float y_low = do_scale ? __fmul_rn(e_low, inv) : e_low;
        mq[j] = (uint32_t)fminf((float)mine[j] * y_low * 268435456.0f, 268435456.0f);
        own += (int)mine[j];
        ownq += mq[j];
    }
    int tot, totq;
    const int c0 = blk_excl_scan(own, &tot, sm);
    const uint32_t q0 = (uint32_t)blk_excl_scan((int)ownq, &totq, sm);
    int crowd = 0;  // entries at positions that hold more than a slab (runs of one value, if the row can be walked at all)
#pragma unroll
    for (int j = 0; j < kPer; j++) crowd += mine[j] > (uint32_t)S ? (int)mine[j] : 0;
    const int crowded_total = blk_sum_i(crowd, sm);
    if (tid == 0) { sm.bc[7] = (uint32_t)kHistPos; sm.bc[11] = (uint32_t)tot; }
    __syncthreads();
    {
        const uint32_t target_q = (uint32_t)(top_p * 1.001f * 268435456.0f) + 64u;
        uint32_t q = q0;
        int c = c0, d_first = kHistPos, c_first = 0;
#pragma unroll
        for (int j = 0; j < kPer; j++) {
            q += mq[j];
            c += (int)mine[j];
            if (q >= target_q && d_first == kHistPos) { d_first = tid * kPer + j; c_first = c; }
        }
        if (d_first < kHistPos) {
            atomicMin(&sm.bc[7], (uint32_t)d_first);
            atomicMin(&sm.bc[11], (uint32_t)c_first);  // (counts rise with the positions: the least belongs to the first)
        }
    }
    const int chunk = ((n + kW * 256 - 1) / (kW * 256)) * 256;
    const int w0 = min(n, wave * chunk), w1 = min(n, w0 + chunk);
    uint32_t* gk = a.sort_keys_in + (size_t)slot * a.sort_stride;
    int32_t* gi = a.sort_vals_in + (size_t)slot * a.sort_stride;
    FPROF_ADD(a, slot, 11, t_step);

    // The nucleus is walked from the top, a slab of at most kSmall entries at a time: the positions [d_prev, d_end).
    constexpr int kMaxSlabs = kNucleusMaxSlabs;
    float run = 0.0f;      // exact running sum behind the slabs before
    float hi_y = 0.0f;     // what is left has y <= hi_y (from the second slab on)
    int d_prev = 0;
    int taken = 0;         // entries that the histogram holds at the positions before d_prev
    int found = -1, nc = 0, slab = 0;
    bool all_in = false;
    int runs = 0;              // positions passed as runs of one value
    bool was_capped = false;   // ... after which what is left is bounded from above too
    bool cut_in_run = false;   // the cut fell inside such a run: ycut / idx_last are set by the walk
    uint32_t ycut = 0u;
    int idx_last = -1;         // the last member among the entries equal to the cut value
    uint32_t pv[kPerT];  // the last slab's entries that this thread read from the pool: their values (index and place in
                         // index order stay in the pool's tags)
#pragma unroll
    for (int r = 0; r < kPerT; r++) pv[r] = 0u;
    for (;; slab++) {
        if (slab >= kMaxSlabs) return kNucleusGeneralNoSlabs;  // (the general way would walk the same slabs)
        if (tid == 0) sm.bc[6] = (uint32_t)kHistPos;
        __syncthreads();
        {
            int c = c0, d_first = kHistPos;
#pragma unroll
            for (int j = 0; j < kPer; j++) {
                c += (int)mine[j];
                if (tid * kPer + j >= d_prev && c - taken > S && d_first == kHistPos) d_first = tid * kPer + j;
            }
            if (d_first < kHistPos) atomicMin(&sm.bc[6], (uint32_t)d_first);
        }
        __syncthreads();
        // about how many entries the nucleus holds: a row that would need more slabs than are walked goes the general
        // way at once (its survivors are sorted where they lie)
        if (slab == 0 && runs == 0 && (int)sm.bc[11] - min((int)sm.bc[11], crowded_total) > (kMaxSlabs - 2) * S)
            return kNucleusGeneralNoSlabs;
        const int d_cnt = (int)sm.bc[6], d_mass = (int)sm.bc[7];
        const int d_end = d_mass + 1 > d_prev ? min(d_cnt, d_mass + 1) : d_cnt;
        if (d_end <= d_prev) {
            // One position alone holds more than a slab.  Where all its entries share one probability -- the equal
            // logits of a coarse grid, of bf16 -- no order among them is needed: the running sum goes through them
            // as through so many equal terms, and if the cut falls among them, the members are the first ones by
            // index.  Anything else is left to the general way's sort.
            if (++runs > 256) return kNucleusGeneralNoSlabs;
            const uint32_t key_d = kHistTopKey - (uint32_t)d_prev;
            const bool last_pos = d_prev == kHistPos - 1;
            // the position's distinct probabilities (a few at most, or the row is left to the sort) and their counts
            constexpr int kDistinct = 16;
            uint32_t* dval = sm.hist + 32;
            uint32_t* dcnt = sm.hist + 32 + kDistinct;
            __syncthreads();
            if (tid < 2 * kDistinct) sm.hist[32 + tid] = 0u;
            if (tid == 0) sm.bc[12] = 0u;
            __syncthreads();
            row_pass<false>(const_cast<float*>(p), n, [&](float e, int) -> float {
                const uint32_t k16 = sr_f2u(e) >> 16;
                if (e > 0.0f && (last_pos ? k16 <= key_d : k16 == key_d)) {
                    const uint32_t yb = sr_f2u(do_scale ? __fmul_rn(e, inv) : e);
                    bool placed = false;
                    for (int sl = 0; sl < kDistinct && !placed; sl++) {
                        const uint32_t old = atomicCAS(&dval[sl], 0u, yb);
                        if (old == 0u || old == yb) {
                            atomicAdd(&dcnt[sl], 1u);
                            placed = true;
                        }
                    }
                    if (!placed || yb < 0x00800000u) sm.bc[12] = 1u;  // (too many values, or one below the normal range)
                }
                return e;
            });
            __syncthreads();
            if (sm.bc[12] != 0u) return kNucleusGeneralNoSlabs;
            // from the largest value down (every thread finds the same order)
            uint32_t below = 0xffffffffu;  // values at or above this one are done
            bool cut_here = false;
            for (int round = 0; round < kDistinct; round++) {
                uint32_t mn = 0u;
                int c_run = 0;
                for (int sl = 0; sl < kDistinct; sl++) {
                    const uint32_t v = dval[sl];
                    if (v != 0u && v < below && v > mn) { mn = v; c_run = (int)dcnt[sl]; }
                }
                if (mn == 0u) break;  // all of the position's values are done
                below = mn;
                const float yv = sr_u2f(mn);
                int f;
                run = seq_sum<true>([&](int) -> float { return yv; }, c_run, run, top_p, &f, sm);
                if (f < 0) continue;
                // (a cut inside a run of equal probabilities keeps the first ones by index: the managed sort leaves
                // their order open)
                SR_AMB_IF(f + 1 < c_run || sr_stop_near(run, yv, top_p));
                // the cut falls inside this run: its first f + 1 entries by index are members
                const int cw = list_stretch(p, w0, w1, do_scale, inv, StretchCount{}, [&](float y, int) -> bool { return sr_f2u(y) == mn; });
                __syncthreads();
                if (lane == 0) sm.redi[wave] = cw;
                if (tid == 0) sm.bc[9] = 0xffffffffu;
                __syncthreads();
                int before_w = 0;
#pragma unroll
                for (int w = 0; w < kW; w++) before_w += w < wave ? sm.redi[w] : 0;
                const int target = (f >= before_w && f < before_w + cw) ? f - before_w : -1;
                __syncthreads();
                (void)list_stretch(p, w0, w1, do_scale, inv, StretchFind{target, &sm.bc[9]}, [&](float y, int) -> bool { return sr_f2u(y) == mn; });
                __syncthreads();
                if (sm.bc[9] == 0xffffffffu) return kNucleusGeneralNoSlabs;  // (the counts of the two reads differ: not possible)
                ycut = mn;
                idx_last = (int)sm.bc[9];
                cut_in_run = true;
                cut_here = true;
                break;
            }
            if (cut_here) { nc = 0; break; }
            const uint32_t mn = below;  // the position's smallest value: what is left of the row lies below it
            // the whole run lies inside the nucleus: on to the position behind it
            {
                int c = c0;
#pragma unroll
                for (int j = 0; j < kPer; j++) {
                    c += (int)mine[j];
                    if (tid * kPer + j == d_prev) sm.bc[8] = (uint32_t)c;
                }
            }
            __syncthreads();
            taken = (int)sm.bc[8];
            hi_y = sr_u2f(mn - 1u);  // what is left lies below the run's value
            d_prev = d_prev + 1;
            __syncthreads();
            if (d_prev >= kHistPos) { all_in = true; nc = 0; break; }
            slab--;  // (a run is not one of the slabs that the limit counts; the for's increment puts it back)
            was_capped = true;
            continue;
        }
        {
            int c = c0;
#pragma unroll
            for (int j = 0; j < kPer; j++) {
                c += (int)mine[j];
                if (tid * kPer + j == d_end - 1) sm.bc[8] = (uint32_t)c;
            }
        }
        all_in = d_end >= kHistPos;
        const float c_e = all_in ? 0.0f : sr_u2f(((kHistTopKey - (uint32_t)d_end) << 16) | 0xffffu);
        const float c_y = do_scale ? __fmul_rn(c_e, inv) : c_e;  // taken: y > c_y, which e > c_e follows from
        const bool capped = slab > 0 || was_capped;

        // the slab's entries: every wave lists those of its stretch of the row in a pool in LDS, each with its number
        // within the wave, from which its place in index order follows once all waves' counts are known
        if (tid == 0) sm.bc[4] = 0u;
        __syncthreads();
        const int cw = list_stretch(p, w0, w1, do_scale, inv, StretchToPool{&sm.bc[4], sval, tags, S},
                                    [&](float y, int) -> bool { return y > c_y && !(capped && y > hi_y); });
        if (lane == 0) sm.redi[wave] = cw;
        __syncthreads();
        taken = (int)sm.bc[8];
        nc = (int)sm.bc[4];
        if (nc > S) return kNucleusGeneral;
        FPROF_ADD(a, slot, 12, t_step);
        if (nc > 0) {
            // this thread's entries of the pool; their places in index order take the place of their numbers within
            // the wave in the tags
#pragma unroll
            for (int r = 0; r < kPerT; r++) {
                const int e = r * kT + tid;
                pv[r] = e < nc ? sval[e] : 0u;
                if (e < nc) {
                    const uint32_t tag = tags[e];
                    const int i = (int)(tag & ((1u << kTagIndexBits) - 1u)), w = i / chunk;
                    int off = (int)(tag >> kTagIndexBits);
#pragma unroll
                    for (int k = 0; k < kW - 1; k++) off += k < w ? sm.redi[k] : 0;
                    tags[e] = ((uint32_t)off << kTagIndexBits) | (uint32_t)i;
                }
            }
            // The values are sorted.  A long list is first cut into 4,096 groups of equal width in the values' bit
            // patterns between the slab's bounds -- counted, the counts summed, the values put group by group -- and
            // then every value finds its rank among the values of its group (equal values are interchangeable in the
            // sum that follows): far fewer steps than the sorting network, unless a group holds more than a few dozen.
            const uint32_t bhi = sr_f2u(capped ? hi_y : (do_scale ? __fmul_rn(1.0f, inv) : 1.0f)), blo = sr_f2u(c_y);
            const uint32_t span = bhi >= blo ? bhi - blo : 0xffffffffu;
            const int gshift = span < (uint32_t)kSmall ? 0 : 20 - __clz((int)span);  // (span >> gshift) < kSmall
            auto group_of = [&](uint32_t v) -> uint32_t { return min((bhi - v) >> gshift, (uint32_t)(kSmall - 1)); };
            bool counted = false;
            if (nc > 1024 && bhi >= blo) {
                uint32_t* cur = (uint32_t*)sm.sortbuf;
                uint32_t* grp = cur + kSmall;
                __syncthreads();  // (sval has been read)
#pragma unroll
                for (int r = 0; r < 4; r++) cur[r * kT + tid] = 0u;
                if (tid == 0) sm.bc[12] = 0u;
                __syncthreads();
#pragma unroll
                for (int r = 0; r < kPerT; r++)
                    if (r * kT + tid < nc) atomicAdd(&cur[group_of(pv[r])], 1u);
                __syncthreads();
                uint32_t c4[4];
                int own = 0;
                uint32_t big = 0u;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    c4[r] = cur[4 * tid + r];
                    own += (int)c4[r];
                    big = max(big, c4[r]);
                }
                if (big > 128u) sm.bc[12] = 1u;
                int tot_c;
                int at = blk_excl_scan(own, &tot_c, sm);
                counted = sm.bc[12] == 0u;  // (the scan's barriers lie between the store and this load)
                if (counted) {
#pragma unroll
                    for (int r = 0; r < 4; r++) { cur[4 * tid + r] = (uint32_t)at; at += (int)c4[r]; }
                    __syncthreads();
#pragma unroll
                    for (int r = 0; r < kPerT; r++)
                        if (r * kT + tid < nc) grp[atomicAdd(&cur[group_of(pv[r])], 1u)] = pv[r];
                    __syncthreads();  // cur[g] is now where group g ends
#pragma unroll
                    for (int r = 0; r < kPerT; r++) {
                        const int i = r * kT + tid;
                        if (i < nc) {
                            const uint32_t v = grp[i];
                            const uint32_t g = group_of(v);
                            const int from = g > 0u ? (int)cur[g - 1u] : 0, to = (int)cur[g];
                            int rank = from;
                            for (int j = from; j < to; j++) {
                                const uint32_t o = grp[j];
                                rank += (o > v || (o == v && j < i)) ? 1 : 0;
                            }
                            sval[rank] = v;
                        }
                    }
                    __syncthreads();
                }
            }
            if (!counted) {
                if (nc > kSmall) return kNucleusGeneral;  // (the network sorts kSmall entries at most)
                int P = 2;
                while (P < nc) P <<= 1;
                __syncthreads();
                for (int e = nc + tid; e < P; e += kT) sval[e] = 0u;
                __syncthreads();
                sort_lds_desc(sval, P);
            }
            FPROF_ADD(a, slot, 13, t_step);
            run = seq_sum<true>([&](int i) -> float { return sr_u2f(sval[i]); }, nc, run, top_p, &found, sm);
            if (found >= 0)
                SR_AMB_IF(sr_stop_near(run, sr_u2f(sval[found]), top_p) || (found + 1 < nc && sval[found + 1] == sval[found]));
            FPROF_ADD(a, slot, 14, t_step);
        }
        if (a.prof && slot == 0 && tid == 0) a.prof[15] += 1ull;
        if (found >= 0 || all_in) break;
        hi_y = c_y;
        d_prev = d_end;
    }
    if (found < 0 && !cut_in_run) SR_AMB_IF(sr_near(run, top_p));  // the whole row is the nucleus: barely?

    // the last slab's entries in index order (the sort's scratch memory is free again)
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kPerT; r++)
        if (r * kT + tid < nc) {
            const uint32_t tag = tags[r * kT + tid];
            list[tag >> kTagIndexBits] = ((unsigned long long)(0xffffffffu - (tag & ((1u << kTagIndexBits) - 1u))) << 32) | (unsigned long long)pv[r];
        }
    __syncthreads();
    // Members: everything above the value at the cut, and of the entries equal to it the first ones by index.
    if (found >= 0 && !cut_in_run) {
        ycut = sval[found];
        int gt = 0;
        for (int e = tid; e < nc; e += kT) gt += sval[e] > ycut ? 1 : 0;
        const int keep_eq = found + 1 - blk_sum_i(gt, sm);
        unsigned long long ent[kPerT];
        int eqc = 0;
#pragma unroll
        for (int r = 0; r < kPerT; r++) {
            const int e = cpt * tid + r;
            ent[r] = (r < cpt && e < nc) ? list[e] : 0ull;
            eqc += (r < cpt && e < nc && (uint32_t)ent[r] == ycut) ? 1 : 0;
        }
        int tot_eq;
        int rank = blk_excl_scan(eqc, &tot_eq, sm);
#pragma unroll
        for (int r = 0; r < kPerT; r++) {
            const int e = cpt * tid + r;
            if (r < cpt && e < nc) {
                const uint32_t yb = (uint32_t)ent[r];
                const bool keep = yb > ycut || (yb == ycut && rank < keep_eq);
                if (yb == ycut && rank == keep_eq - 1) sm.bc[9] = 0xffffffffu - (uint32_t)(ent[r] >> 32);
                if (yb == ycut) rank++;
                if (!keep) list[e] = ent[r] & 0xffffffff00000000ull;
            }
        }
        __syncthreads();
        idx_last = (int)sm.bc[9];
    }
    if (slab == 0 && runs == 0) {
        finish_from_ordered_list(a, const_cast<float*>(p), n, nc, row, sm, NoFill(), S);
        return kNucleusDone;
    }
    // Several slabs: the members -- known by value and, at the cut value, by index -- are listed by one more read of
    // the row, again in index order in the waves' stretches of the sort segment, and the final Normalize and the draw
    // take them from there a block at a time.
    const float ycut_f = sr_u2f(ycut);
    if (slab >= kNucleusRowFinish || runs > 0) {
        // A nucleus of many thousands of members: listing them and passing over the list, 5 us per thousand, costs more
        // than writing the row -- scaled, everything outside the nucleus zero -- and the two passes over it of the
        // final Normalize and the pass of the draw (about 70 us for 151,936 entries).
        float* w = const_cast<float*>(p);
        row_pass<true>(w, n, [&](float e, int i) -> float {
            const float y = do_scale ? __fmul_rn(e, inv) : e;
            return (y > ycut_f || (y == ycut_f && i <= idx_last)) ? y : 0.0f;
        });
        __syncthreads();
        normalize_row(w, n, sm);
        if (a.mode != 1) {
            const int token = draw_from_row(w, n, a.uniforms[(size_t)row * a.uniforms_per_row], sm);
            if (tid == 0 && a.out_tokens) a.out_tokens[row] = token;
        }
        return kNucleusDone;
    }
    const int cm = list_stretch(p, w0, w1, do_scale, inv, StretchToSegment{gk, gi, w0},
                                [&](float y, int i) -> bool { return y > ycut_f || (y == ycut_f && i <= idx_last); });
    sr_drain_stores();
    __syncthreads();  // (the last readers of sm.hist are long past; this one orders the stretches' stores before the fills)
    if (lane == 0) sm.hist[wave] = (uint32_t)cm;
    __syncthreads();
    int members = 0;
#pragma unroll
    for (int w = 0; w < kW; w++) members += (int)sm.hist[w];
    FPROF_ADD(a, slot, 17, t_step);
    finish_from_ordered_list(a, const_cast<float*>(p), n, members, row, sm, [&](int first, int cnt) {
        // (all of a thread's loads are on their way before the first of them is waited for)
        int src[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int g = first + min(r * kT + tid, cnt - 1);
            int w = 0, off = 0;
#pragma unroll
            for (int k = 0; k < kW - 1; k++) {
                const int ck = (int)sm.hist[k];
                if (w == k && g >= off + ck) { off += ck; w = k + 1; }
            }
            src[r] = min(n, w * chunk) + (g - off);
        }
        uint32_t yb[4];
        int32_t ix[4];
#pragma unroll
        for (int r = 0; r < 4; r++) { yb[r] = gk[src[r]]; ix[r] = gi[src[r]]; }
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (r * kT + tid < cnt) sm.sortbuf[r * kT + tid] = ((unsigned long long)(0xffffffffu - (uint32_t)ix[r]) << 32) | (unsigned long long)yb[r];
    });
    return kNucleusDone;
}

// ---- the survivors of a row sorted where they lie -------------------------------------------------------------------
// keys[i] (probability bits) and ids[i] (indices) of ns entries in device memory, sorted by descending key, equal keys
// by ascending index, by this workgroup alone: a bitonic network whose comparators all point the same way (a merge
// starts by comparing every entry with its mirror image in the block, then halves), so that a length that is no power of
// two needs no padding in memory -- the entries past the end count as the smallest and never move.  Tiles of kSmall
// entries are sorted and merged in LDS; only the steps that reach across tiles go through memory.  For the rare row
// whose nucleus the walk by slabs cannot close: about 2 ms for 130 thousand survivors.
__device__ __forceinline__ void sort_survivors_in_place(uint32_t* keys, int32_t* ids, int ns, FullSmem& sm)
{
    typedef unsigned long long u64;
    const int tid = threadIdx.x;
    auto ld = [&](int i) -> u64 { return ((u64)keys[i] << 32) | (u64)(0xffffffffu - (uint32_t)ids[i]); };
    auto st = [&](int i, u64 v) { keys[i] = (uint32_t)(v >> 32); ids[i] = (int32_t)(0xffffffffu - (uint32_t)v); };
    auto tile_in = [&](int t0) {
        for (int e = tid; e < kSmall; e += kT) sm.sortbuf[e] = t0 + e < ns ? ld(t0 + e) : 0ull;
        __syncthreads();
    };
    auto tile_out = [&](int t0) {
        for (int e = tid; e < kSmall; e += kT)
            if (t0 + e < ns) st(t0 + e, sm.sortbuf[e]);
        sr_drain_stores();
        __syncthreads();
    };
    __syncthreads();
    for (int t0 = 0; t0 < ns; t0 += kSmall) {
        tile_in(t0);
        sort_lds_desc(sm.sortbuf, kSmall);
        tile_out(t0);
    }
    int total = kSmall;  // the power of two that the network is laid out for
    while (total < ns) total <<= 1;
    for (int k2 = 2 * kSmall; k2 <= total; k2 <<= 1) {
        // every entry of a block's first half against its mirror image in the second
        for (int pr = tid; pr < total / 2; pr += kT) {
            const int blk = pr / (k2 / 2), off = pr - blk * (k2 / 2);
            const int i = blk * k2 + off, j = blk * k2 + k2 - 1 - off;
            if (j < ns) {
                const u64 x = ld(i), y = ld(j);
                if (x < y) { st(i, y); st(j, x); }
            }
        }
        sr_drain_stores();
        __syncthreads();
        // halves, quarters, ... of the block down to the size of a tile
        for (int j2 = k2 / 4; j2 >= kSmall; j2 >>= 1) {
            for (int pr = tid; pr < total / 2; pr += kT) {
                const int i = ((pr & ~(j2 - 1)) << 1) | (pr & (j2 - 1)), j = i | j2;
                if (j < ns) {
                    const u64 x = ld(i), y = ld(j);
                    if (x < y) { st(i, y); st(j, x); }
                }
            }
            sr_drain_stores();
            __syncthreads();
        }
        // the rest of the merge inside every tile
        for (int t0 = 0; t0 < ns; t0 += kSmall) {
            tile_in(t0);
            for (int j2 = kSmall / 2; j2 >= 1; j2 >>= 1) {
                for (int pr = tid; pr < kSmall / 2; pr += kT) {
                    const int i = ((pr & ~(j2 - 1)) << 1) | (pr & (j2 - 1)), j = i | j2;
                    const u64 x = sm.sortbuf[i], y = sm.sortbuf[j];
                    if (x < y) { sm.sortbuf[i] = y; sm.sortbuf[j] = x; }
                }
                __syncthreads();
            }
            tile_out(t0);
        }
    }
}

// ---- stage 3: softmax, top-k, min-p, top-p on the work row --------------------------------------------
// One workgroup per row, one launch: the row is cut, normalised and drawn from here.  A nucleus that the walk by
// slabs cannot close has its survivors compacted into the row's sort segment and sorted there by this workgroup.
__global__ __launch_bounds__(kT) void k_full_row(SrFullArgs a)
{
    __shared__ FullSmem sm;
    const int tid = threadIdx.x;
    const int slot = blockIdx.x;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    const int n = a.vocab;
    float* p = a.work + (size_t)(a.work_by_row ? row : slot) * a.work_stride;
    SrFullState* st = a.state + slot;
    const bool greedy = rd.temperature <= 0.0f;
    const bool use_top_p = rd.top_p < 1.0f && rd.top_p > 0.0f;
    if (tid == 0) {
        sm.bc[SR_AMB_WORD] = 0u;  // (every path that can set it passes a barrier first)
        // What the launch after this one expects of the row's scalars: the factors of a row that is not left to its
        // reader are 1, and the list of entries to watch is empty (the expf pass only appends to it).  No kernel of the
        // pipeline before this one runs for every row of every launch.
        st->mul1 = st->mul2 = 1.0f;
        if (a.watch_cnt) {
            sm.segbc[3] = a.watch_cnt[slot];
            a.watch_cnt[slot] = 0u;
        }
    }

    if (greedy) {
        // Greedy / GreedyWithHistoryPenalties on the adjusted row; distributions become one-hot
        const int am = row_argmax(p, n, sm);
        if (a.mode != 0) {
            __syncthreads();
            row_pass<true>(p, n, [&](float, int i) -> float { return (i == am) ? 1.0f : 0.0f; });
        }
        if (tid == 0) {
            if (a.out_tokens) a.out_tokens[row] = am;
            if (a.out_flags) a.out_flags[row] = SR_KFLAG_GREEDY | SR_KFLAG_FULL;
        }
        return;
    }

    {
        FPROF(a, slot, 0);
        // Softmax (Sampler.cs:448-472): the maximum and e = expf(x - max) were computed by the kernels before
        const uint32_t mk = full_maxkey_of(a, st->maxkey);
        const bool any_nan = mk == 0xffffffffu;
        const float m = mk == 0u ? SR_NEG_INF : sr_okey_inv(mk);
        FPROF(a, slot, 1);
        uint32_t flags = SR_KFLAG_FULL;
        bool fused = false;  // scaling, min-p and the count of survivors were done in one pass
        int survivors = 0;   // ... this thread's share of the count
        int ns_listed = -1;  // >= 0: the block-wide count, and sm.sortbuf[0, ns_listed) holds the survivors
        bool row_unwritten = false;  // the row still holds expf(x - max): it will be finished from the list
        bool no_slabs = false;       // the nucleus is known to be too large for the walk by slabs
        if (any_nan || sr_f2u(m) == 0xff800000u) {
            const float uni = n > 0 ? __fdiv_rn(1.0f, (float)n) : 0.0f;
            row_pass<true>(p, n, [&](float, int) -> float { return uni; });
            flags |= SR_KFLAG_DEGENERATE;
            __syncthreads();
        } else {
            if (row_edits_on_the_fly(rd, a) && !a.seg_func) {
                // the ids that the row's edits touch were left out of the expf pass: their e, from the adjusted values
                // that k_full_edits kept
                const float* vals = (const float*)(a.edit_tab + (size_t)slot * (size_t)a.edit_tab_stride + (n + 31) / 32);
                const SrEdit* ed = a.edits + rd.edit_off;
                for (int e = tid; e < rd.edit_cnt; e += kT) p[ed[e].id] = sr_expf(__fsub_rn(vals[e], m));
                sr_drain_stores();  // (this compute unit has not read these lines before: the loads below find them in L2)
                __syncthreads();
            }
            int dummy;
            // A row that min-p cuts, with no top-k stage before the cut and no distribution to hand out, is not read a
            // second time for the cut: a survivor has fl(e * inv) >= fl(min_p * inv), so e >= min_p * (1 - 2^-22), and
            // the few entries that large are listed while the sum passes over them; the exact test follows below.
            const bool watch_min_p = row_watch_min_p(rd, a);
            const float e_low = __fmul_rn(rd.min_p, 0.999999f);
            if (watch_min_p) {
                if (tid == 0) sm.bc[4] = 0u;
                __syncthreads();
            }
            // A row that only top-p cuts and that is only sampled from: see nucleus_from_histogram
            const bool fast_nucleus = row_fast_nucleus(rd, a);
            const bool walked = a.seg_func != nullptr && (!fast_nucleus || a.seg_keys != nullptr);
            if (fast_nucleus) {
                uint32_t* hcnt = (uint32_t*)sm.sortbuf;
                for (int i = tid; i < kHistPos; i += kT) hcnt[i] = 0u;
                if (tid == 0) sm.bc[5] = 0u;
                __syncthreads();
            }
            float sum;
            if (walked) {
                // the whole device has prepared the sum (k_full_softmax_seg): one wave walks the segments' records, and the
                // entries that can survive the min-p cut were listed by the same pass
                __syncthreads();
                if (sr_wave_id() == 0) {
                    const float s = seg_walk<false>(p, n, a.seg_func + (size_t)slot * a.seg_stride, 0.0f, 0.0f, &dummy, nullptr);
                    if (sr_lane() == 0) sm.segbc[0] = sr_f2u(s);
                } else if (fast_nucleus) {
                    // the histogram of e from the 16 bits per entry that the expf pass left
                    uint32_t* hcnt = (uint32_t*)sm.sortbuf;
                    const uint16_t* keys = a.seg_keys + (size_t)slot * (size_t)a.seg_key_stride;
                    auto count = [&](uint32_t key) {
                        if (key != 0u) {
                            if (key <= kHistTopKey) atomicAdd(&hcnt[min(kHistTopKey - key, (uint32_t)(kHistPos - 1))], 1u);
                            else sm.bc[5] = 1u;  // (no e exceeds 1; if one does, the general way takes the row)
                        }
                    };
                    const int n8 = n / 8;  // (the rows of keys start on 16-byte boundaries)
                    for (int v0 = tid - SR_WAVE; v0 < n8; v0 += 2 * (kT - SR_WAVE)) {
                        const int v1 = v0 + (kT - SR_WAVE);
                        const uint4 ka = ((const uint4*)keys)[v0];
                        const uint4 kb = v1 < n8 ? ((const uint4*)keys)[v1] : make_uint4(0u, 0u, 0u, 0u);
                        const uint32_t ww[8] = {ka.x, ka.y, ka.z, ka.w, kb.x, kb.y, kb.z, kb.w};
#pragma unroll
                        for (int q = 0; q < 8; q++) { count(ww[q] & 0xffffu); count(ww[q] >> 16); }
                    }
                    for (int i = n8 * 8 + tid - SR_WAVE; i < n; i += kT - SR_WAVE) count(keys[i]);
                } else if (watch_min_p) {
                    const uint32_t cw = sm.segbc[3];
                    const unsigned long long* wl = a.watch + (size_t)slot * kSmall;
                    for (int i = tid - SR_WAVE; i < (int)min(cw, (uint32_t)kSmall); i += kT - SR_WAVE) sm.sortbuf[i] = wl[i];
                    if (tid == SR_WAVE) sm.bc[4] = cw;
                }
                __syncthreads();
                sum = sr_u2f(sm.segbc[0]);
            } else if (fast_nucleus) {
                uint32_t* hcnt = (uint32_t*)sm.sortbuf;
                sum = seq_sum_row<false>(p, n, 0.0f, 0.0f, &dummy, sm, 1.0f, 1.0f, [&](float x, int) { hist_count(hcnt, &sm.bc[5], x); });
            } else if (watch_min_p) {
                sum = seq_sum_row<false>(p, n, 0.0f, 0.0f, &dummy, sm, 1.0f, 1.0f, [&](float x, int i) {
                    if (x >= e_low) {
                        const uint32_t pos = atomicAdd(&sm.bc[4], 1u);
                        if (pos < (uint32_t)kSmall)
                            sm.sortbuf[pos] = ((unsigned long long)sr_f2u(x) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
                    }
                });
            } else {
                sum = seq_sum_row<false>(p, n, 0.0f, 0.0f, &dummy, sm);
            }
            __syncthreads();
            const int n_watched = watch_min_p ? (int)sm.bc[4] : -1;
            const bool from_watch = n_watched >= 0 && n_watched <= kSmall;  // (else the row is read again, as before)
            FPROF(a, slot, 2);
            const bool do_scale = sum > 0.0f && sum != 1.0f;
            const float inv = do_scale ? __fdiv_rn(1.0f, sum) : 1.0f;
            if (a.lazy_scale && a.mode == 1 && !(rd.top_k > 0 && rd.top_k < n) && !(rd.min_p > 0.0f) && !use_top_p) {
                // No filter touches the row: its final entries are fmul(fmul(e, inv), inv2) with inv2 from the final
                // Normalize (Sampler.cs:91-92) over the scaled values.  The reader applies the two factors; the row
                // keeps e and is not written again.
                const float sum2 = tp_sum_row(p, n, inv, true, sm);
                const float inv2 = (sum2 > 0.0f && sum2 != 1.0f) ? __fdiv_rn(1.0f, sum2) : 1.0f;
                if (tid == 0) {
                    st->mul1 = inv;
                    st->mul2 = inv2;
                    st->n_survivors = 0;
                    st->flags = flags;
                    if (a.out_flags) a.out_flags[row] = flags;
                }
                return;
            }
            extern __shared__ uint32_t more_lds[];  // 16 kSmall bytes when a.big_slabs, else nothing
            const int way = fast_nucleus ? nucleus_from_histogram(a, rd.top_p, p, n, slot, row, do_scale, inv, sm,
                                                                  a.big_slabs ? more_lds : nullptr)
                                         : kNucleusGeneral;
            no_slabs = way == kNucleusGeneralNoSlabs;
            if (way == kNucleusDone) {
                FPROF(a, slot, 9);
                __syncthreads();
                if (tid == 0) {
                    st->n_survivors = 0;
                    st->flags = flags;
                    if (a.out_flags) a.out_flags[row] = flags | (sm.bc[SR_AMB_WORD] ? SR_KFLAG_AMBIGUOUS : 0u);
                }
                return;
            }
            if (!(rd.top_k > 0 && rd.top_k < n) && (rd.min_p > 0.0f || use_top_p)) {
                // No top-k stage in between: the scaling, the min-p cut (Sampler.cs:493-503) and the count of
                // survivors that top-p starts from share one pass.  The largest probability needs no search: the
                // largest e is expf(0) = 1, so it is 1 * (1 / sum).
                const float mp = do_scale ? __fmul_rn(1.0f, inv) : 1.0f;
                const bool use_min_p = rd.min_p > 0.0f;
                const float thr = use_min_p ? __fmul_rn(rd.min_p, mp) : 0.0f;
                int c = 0;
                // A min-p cut leaves few survivors: they are listed while the row is read, which saves the pass that
                // would collect them; a row that is only sampled from (no distribution out) and ends with at most
                // 4,096 survivors is finished from that list and need not be written at all.
                const bool list_now = use_min_p;
                if (list_now) {
                    if (tid == 0) sm.bc[4] = 0u;
                    __syncthreads();
                }
                auto body = [&](float x, int i) -> float {
                    float y = do_scale ? __fmul_rn(x, inv) : x;
                    if (use_min_p) SR_AMB_IF(sr_near(y, thr));  // an entry on the threshold
                    if (use_min_p && y < thr) y = 0.0f;
                    if (y > 0.0f) {
                        c++;
                        if (list_now) {
                            const uint32_t pos = atomicAdd(&sm.bc[4], 1u);
                            if (pos < (uint32_t)kSmall)
                                sm.sortbuf[pos] = ((unsigned long long)sr_f2u(y) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
                        }
                    }
                    return y;
                };
                const bool read_only = list_now && a.mode == 0 && n >= 8;
                if (from_watch) {
                    // the entries listed during the sum, put to the exact test; the survivors are listed again
                    static_assert(kSmall % kT == 0, "whole candidates per thread");
                    unsigned long long cand[kSmall / kT];
#pragma unroll
                    for (int r = 0; r < kSmall / kT; r++) cand[r] = (r * kT + tid < n_watched) ? sm.sortbuf[r * kT + tid] : 0ull;
                    __syncthreads();
                    if (tid == 0) sm.bc[4] = 0u;
                    __syncthreads();
#pragma unroll
                    for (int r = 0; r < kSmall / kT; r++)
                        if (r * kT + tid < n_watched)
                            (void)body(sr_u2f((uint32_t)(cand[r] >> 32)), (int)(0xffffffffu - (uint32_t)cand[r]));
                } else if (read_only) {
                    row_pass<false>(p, n, body);
                } else {
                    row_pass<true>(p, n, body);
                }
                survivors = c;
                fused = true;
                if (list_now) {
                    const int ns_now = blk_sum_i(c, sm);
                    if (ns_now <= kSmall) ns_listed = ns_now;
                    row_unwritten = read_only && ns_now > 0 && ns_now <= kSmall;
                    if (read_only && !row_unwritten) {
                        // too many survivors to finish from the list: the scaled row is needed after all
                        row_pass<true>(p, n, [&](float x, int) -> float {
                            float y = do_scale ? __fmul_rn(x, inv) : x;
                            if (use_min_p && y < thr) y = 0.0f;
                            return y;
                        });
                    }
                }
            } else if (do_scale) {
                row_pass<true>(p, n, [&](float x, int) -> float { return __fmul_rn(x, inv); });
            }
            __syncthreads();
        }
        FPROF(a, slot, 3);
        // ApplyTopK + Normalize (Sampler.cs:71-81, :477-488): everything equal to the k-th value survives
        if (rd.top_k > 0 && rd.top_k < n) {
            const float kth = kth_largest(p, n, rd.top_k, sm);
            row_pass<true>(p, n, [&](float x, int) -> float { return x < kth ? 0.0f : x; });
            __syncthreads();
            normalize_row(p, n, sm);
        }
        FPROF(a, slot, 4);
        // ApplyMinP (Sampler.cs:493-503)
        if (rd.min_p > 0.0f && !fused) {
            float mp = 0.0f;
            row_pass<false>(p, n, [&](float x, int) -> float { mp = fmaxf(mp, x); return x; });
            bool nn;
            mp = blk_max_f(mp, &nn, sm);
            const float thr = __fmul_rn(rd.min_p, mp);
            row_pass<true>(p, n, [&](float x, int) -> float {
                SR_AMB_IF(x > 0.0f && sr_near(x, thr));
                return x < thr ? 0.0f : x;
            });
            __syncthreads();
        }
        FPROF(a, slot, 5);
        // ApplyTopP (Sampler.cs:516-551)
        int listed = -1;  // the row's survivors are sm.sortbuf[0, listed)
        if (use_top_p) {
            int cnt = survivors;
            if (!fused) row_pass<false>(p, n, [&](float x, int) -> float { cnt += x > 0.0f ? 1 : 0; return x; });
            int ns;
            ns = blk_sum_i(cnt, sm);
            const bool have_list = ns_listed >= 0;  // (then ns == ns_listed <= kSmall)
            // The nucleus is walked in descending order, a slab of at most kSmall probabilities at a time: the slab
            // is everything above the 65536-value bucket that holds the kSmall-th largest of what is left, it is
            // sorted here and the exact running sum goes on through it from where the slab before ended.  Most
            // nuclei close in the first slab; a masked row without min-p (tens of thousands of survivors) takes a
            // few.  Only a row that makes no progress (more than kSmall probabilities inside one bucket) or needs
            // more than kMaxSlabs slabs has all its survivors sorted (sort_survivors_in_place).
            constexpr int kMaxSlabs = 24;
            // A row that needs several slabs has all their bounds from one histogram of its probabilities' 16-bit keys
            // instead of two select passes per slab.  The histogram is counted in LDS (the slabs' sort buffer, free
            // until the first slab): position d = 0x3fff - key, so that positions ascend as the values fall; 8,192
            // positions reach down to 2^-63, what lies below shares the last one.  Its running sums go to the row's
            // segment of the sort buffers: sums[d] = survivors at positions <= d, and the position that holds the
            // kSmall-th largest of what is left is the first d with sums[d] >= taken + kSmall.
            constexpr int kPos = 8192;
            static_assert(kPos * 4 <= kSmall * 8 && kPos % kT == 0, "the histogram fits the sort buffer");
            constexpr int kPer = kPos / kT;
            uint32_t* sums = a.sort_keys_in + (size_t)slot * a.sort_stride;
            bool use_hist = !have_list && ns > kSmall && a.sort_stride >= kPos && !no_slabs;
            if (use_hist) {
                uint32_t* cnt = (uint32_t*)sm.sortbuf;
                for (int i = tid; i < kPos; i += kT) cnt[i] = 0u;
                if (tid == 0) sm.bc[5] = 0u;
                __syncthreads();
                row_pass<false>(p, n, [&](float v, int) -> float {
                    if (v > 0.0f) {
                        const uint32_t key = sr_f2u(v) >> 16;
                        if (key <= 0x3fffu) atomicAdd(&cnt[min(0x3fffu - key, (uint32_t)(kPos - 1))], 1u);
                        else sm.bc[5] = 1u;  // (no probability is 2 or more; if one is, the slabs take the other way)
                    }
                    return v;
                });
                __syncthreads();
                use_hist = sm.bc[5] == 0u;
                uint32_t mine[kPer];
                int own = 0;
#pragma unroll
                for (int q = 0; q < kPer; q++) { mine[q] = cnt[tid * kPer + q]; own += (int)mine[q]; }
                int tot;
                int upto = blk_excl_scan(own, &tot, sm);
#pragma unroll
                for (int q = 0; q < kPer; q++) { upto += (int)mine[q]; sums[tid * kPer + q] = (uint32_t)upto; }
                // The first slab need not be full: count x the position's smallest value bounds the mass of the
                // positions from below (in units of 2^-28), and the slab ends where that bound passes top-p (+ 0.1 %) --
                // a few hundred entries for a sharp row instead of 4,096 to gather and sort.
                uint32_t ownq = 0u, mq[kPer];
#pragma unroll
                for (int q = 0; q < kPer; q++) {
                    const int d = tid * kPer + q;
                    const float y_low = d < kPos - 1 ? sr_u2f((0x3fffu - (uint32_t)d) << 16) : 0.0f;
                    mq[q] = (uint32_t)fminf((float)mine[q] * y_low * 268435456.0f, 268435456.0f);
                    ownq += mq[q];
                }
                int totq;
                uint32_t uptoq = (uint32_t)blk_excl_scan((int)ownq, &totq, sm);
                if (tid == 0) sm.bc[7] = (uint32_t)kPos;
                __syncthreads();
                const uint32_t target_q = (uint32_t)(rd.top_p * 1.001f * 268435456.0f) + 64u;
                int d_first = kPos;
#pragma unroll
                for (int q = 0; q < kPer; q++) {
                    uptoq += mq[q];
                    if (uptoq >= target_q && d_first == kPos) d_first = tid * kPer + q;
                }
                if (d_first < kPos) atomicMin(&sm.bc[7], (uint32_t)d_first);
                sr_drain_stores();
                __syncthreads();
            }
            const uint32_t d_mass = use_hist ? sm.bc[7] : (uint32_t)kPos;
            FPROF(a, slot, 10);
            [[maybe_unused]] unsigned long long t_step = 0ull;
            FPROF_ADD(a, slot, 16, t_step);
            bool closed = false;
            float run = 0.0f;                  // exact running sum behind the slabs taken so far
            int taken = 0;                     // survivors in those slabs
            uint32_t hi_key = 0xffffffffu;     // what is left are the probabilities with keys <= hi_key
            float c_above = -1.0f;             // the current slab: probabilities strictly above this value ...
            for (int slab = 0; slab < kMaxSlabs && ns > 0 && !closed && !no_slabs; slab++) {
                const bool last_slab = ns - taken <= kSmall;  // everything that is left fits
                if (last_slab) {
                    c_above = 0.0f;
                } else if (use_hist) {
                    const uint32_t target = (uint32_t)(taken + kSmall);
                    // the one thread whose positions hold the first d with sums[d] >= target names it
                    const uint32_t last = sums[tid * kPer + kPer - 1], before = tid > 0 ? sums[tid * kPer - 1] : 0u;
                    if (last >= target && before < target) {
                        int d = tid * kPer + kPer - 1;
#pragma unroll
                        for (int q = kPer - 2; q >= 0; q--)
                            if (sums[tid * kPer + q] >= target) d = tid * kPer + q;
                        sm.bc[5] = (uint32_t)d;
                    }
                    __syncthreads();
                    uint32_t d = sm.bc[5];
                    __syncthreads();
                    if (slab == 0) d = min(d, d_mass + 1u);
                    if (d < (uint32_t)(kPos - 1)) {
                        c_above = sr_u2f(((0x3fffu - d) << 16) | 0xffffu);
                    } else {  // (the shared last position: its keys are not one bucket)
                        use_hist = false;
                        c_above = sr_u2f(sr_f2u(kth_largest(p, n, kSmall, sm, 16, hi_key)) | 0xffffu);
                    }
                } else {
                    c_above = sr_u2f(sr_f2u(kth_largest(p, n, kSmall, sm, 16, hi_key)) | 0xffffu);
                }
                FPROF_ADD(a, slot, 11, t_step);
                int nc;
                if (have_list) {
                    nc = ns;  // (ns <= kSmall: the survivors were listed while the row was scaled)
                } else {
                    if (tid == 0) sm.bc[4] = 0u;
                    __syncthreads();
                    row_pass<false>(p, n, [&](float v, int i) -> float {
                        if (v > c_above && sr_f2u(v) <= hi_key) {
                            const uint32_t pos = atomicAdd(&sm.bc[4], 1u);
                            if (pos < (uint32_t)kSmall)
                                sm.sortbuf[pos] = ((unsigned long long)sr_f2u(v) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
                        }
                        return v;
                    });
                    __syncthreads();
                    nc = (int)sm.bc[4];
                    __syncthreads();
                }
                FPROF_ADD(a, slot, 12, t_step);
                if (nc <= 0 || nc > kSmall) break;  // no progress: the row's survivors are sorted as a whole
                int P = 2;
                while (P < nc) P <<= 1;
                for (int i = nc + tid; i < P; i += kT) sm.sortbuf[i] = 0ull;
                __syncthreads();
                sort_small_desc(sm, P);
                FPROF_ADD(a, slot, 13, t_step);
                for (int i = tid; i < nc; i += kT) sm.sprob[i] = sr_u2f((uint32_t)(sm.sortbuf[i] >> 32));
                __syncthreads();
                int found;
                if (nc <= SR_WAVE) {
                    // a handful of survivors (a row that min-p has cut): one thread adds them the way the scalar loop does
                    if (tid == 0) {
                        float s = run;
                        int f = -1;
                        for (int i = 0; i < nc && f < 0; i++) {
                            s = __fadd_rn(s, sm.sprob[i]);
                            if (s >= rd.top_p) f = i;
                        }
                        sm.segbc[1] = (uint32_t)f;
                        sm.segbc[2] = sr_f2u(s);
                    }
                    __syncthreads();
                    found = (int)sm.segbc[1];
                    run = sr_u2f(sm.segbc[2]);
                    __syncthreads();  // (the words may be written again for the next slab)
                } else {
                    run = seq_sum<true>([&](int i) -> float { return sm.sprob[i]; }, nc, run, rd.top_p, &found, sm);
                }
                if (found >= 0)
                    SR_AMB_IF(sr_stop_near(run, sm.sprob[found], rd.top_p) || (found + 1 < nc && sm.sprob[found + 1] == sm.sprob[found]));
                else if (taken + nc == ns)
                    SR_AMB_IF(sr_near(run, rd.top_p));
                FPROF_ADD(a, slot, 14, t_step);
                if (a.prof && slot == 0 && tid == 0) a.prof[15] += 1ull;
                taken += nc;
                closed = found >= 0 || taken == ns;
                if (closed) {
                    const int cutoff = found >= 0 ? found + 1 : nc;
                    if (!row_unwritten)
                        for (int i = cutoff + tid; i < nc; i += kT)
                            p[0xffffffffu - (uint32_t)(sm.sortbuf[i] & 0xffffffffull)] = 0.0f;
                    __syncthreads();
                    if (taken < ns) {  // everything that was in no slab comes later in the order
                        row_pass<true>(p, n, [&](float x, int) -> float { return x > c_above ? x : 0.0f; });
                        __syncthreads();
                    }
                    if (slab == 0) listed = cutoff;  // the members are all at hand
                } else {
                    hi_key = sr_f2u(c_above);
                }
            }
            if (ns > 0 && !closed) {
                // the nucleus reaches past what the walk by slabs takes: the survivors go to the row's sort segment and
                // are sorted there
                uint32_t* keys = a.sort_keys_in + (size_t)slot * a.sort_stride;
                int32_t* ids = a.sort_vals_in + (size_t)slot * a.sort_stride;
                const bool aligned = ((uintptr_t)p & 15u) == 0u;
                int base = 0;
                for (int i0 = 0; i0 < n; i0 += 4 * kT) {
                    const int i = i0 + 4 * tid;
                    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                    if (aligned && i + 4 <= n) {
                        const float4 t = *(const float4*)(p + i);
                        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
                    } else {
#pragma unroll
                        for (int q = 0; q < 4; q++)
                            if (i + q < n) v[q] = p[i + q];
                    }
                    const int mine = (v[0] > 0.0f ? 1 : 0) + (v[1] > 0.0f ? 1 : 0) + (v[2] > 0.0f ? 1 : 0) + (v[3] > 0.0f ? 1 : 0);
                    int tot;
                    int pos = base + blk_excl_scan(mine, &tot, sm);
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        if (v[q] > 0.0f) { keys[pos] = sr_f2u(v[q]); ids[pos] = i + q; pos++; }
                    base += tot;
                }
                sr_drain_stores();
                sort_survivors_in_place(keys, ids, ns, sm);
                // the nucleus over the sorted survivors (descending probability, ascending index among equal ones)
                int found;
                const float at = seq_sum<true>([&](int i) -> float { return sr_u2f(keys[i]); }, ns, 0.0f, rd.top_p, &found, sm);
                if (tid == 0)
                    SR_AMB_IF(found >= 0 ? (sr_stop_near(at, sr_u2f(keys[found]), rd.top_p) || (found + 1 < ns && keys[found + 1] == keys[found]))
                                         : sr_near(at, rd.top_p));
                const int cutoff = found >= 0 ? found + 1 : ns;
                for (int i = cutoff + tid; i < ns; i += kT) p[ids[i]] = 0.0f;
                __syncthreads();
            }
            if (tid == 0) st->n_survivors = ns;
        } else if (ns_listed > 0 && ns_listed <= kSmall && n >= 8) {
            listed = ns_listed;  // min-p alone: its survivors are the members
        }
        FPROF(a, slot, 6);
        const bool finish_here = listed > 0 && listed <= kSmall && n >= 8;
        if (tid == 0) {
            st->flags = flags;
        }
        if (finish_here) {
            // the nucleus closed inside the kernel and its members are at hand: no pass over the row is needed
            finish_from_list(a, p, n, listed, row, sm);
            FPROF(a, slot, 9);
            __syncthreads();
            if (tid == 0 && a.out_flags) a.out_flags[row] = flags | (sm.bc[SR_AMB_WORD] ? SR_KFLAG_AMBIGUOUS : 0u);
            return;
        }
        __syncthreads();
    }
    FPROF(a, slot, 7);
    // final Normalize (Sampler.cs:91-92)
    normalize_row(p, n, sm);
    FPROF(a, slot, 8);
    int token = -1;
    if (a.mode != 1) {
        token = draw_from_row(p, n, a.uniforms[(size_t)row * a.uniforms_per_row], sm);
        if (tid == 0 && a.out_tokens) a.out_tokens[row] = token;
    }
    FPROF(a, slot, 9);
    __syncthreads();
    if (tid == 0 && a.out_flags) a.out_flags[row] = st->flags | (sm.bc[SR_AMB_WORD] ? SR_KFLAG_AMBIGUOUS : 0u);
}

// ---- SampleTopK (Sampler.cs:216-357) for rows wider than the selection kernel takes -----------------------
// The reference keeps the k + history-length largest raw logits (earlier index first among equals), applies the
// history penalties to those, orders them again (stable), and samples among the first k.  Here the whole row is
// sorted device-wide by (raw logit descending, index ascending), the first `sel` entries are adjusted and sorted
// again, and one workgroup per row walks the result.
// the reference's selection size: k + history length when the row has history penalties (Sampler.cs:224-225)
__device__ __forceinline__ int wide_sel(const SrRow& rd, int vocab)
{
    const long long s = (long long)rd.top_k + ((rd.flags & SR_ROWFLAG_HAS_PENALTY) ? (long long)rd.n_prev : 0ll);
    return (int)(s < (long long)vocab ? s : (long long)vocab);
}
template <int ES>
__global__ __launch_bounds__(256) void k_wide_keys(SrFullArgs a)
{
    const int slot = blockIdx.y;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
    const uint32_t* mrow = (rd.mask_row >= 0) ? a.mask + (size_t)rd.mask_row * a.mask_stride : nullptr;
    uint32_t* keys = a.sort_keys_in + (size_t)slot * a.sort_stride;
    int32_t* ids = a.sort_vals_in + (size_t)slot * a.sort_stride;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < a.vocab; i += gridDim.x * 256) {
        float x = load_logit<ES>(rowp, i);
        if (mrow && !((mrow[i >> 5] >> (i & 31)) & 1u)) x = SR_NEG_INF;
        keys[i] = sr_okey(x);
        ids[i] = i;
    }
}

// the first `sel` sorted entries with the history penalties of SampleTopK applied (Sampler.cs:262-297); entries
// that hold -inf are the reference's unfilled slots (index -1)
__global__ __launch_bounds__(256) void k_wide_adjust(SrFullArgs a)
{
    const int slot = blockIdx.y;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    // In place: entry t of the sorted row becomes (adjusted key, t) -- the place in the first order is what the second
    // sort breaks ties by, which makes it the stable sort that the reference's insertion is (Sampler.cs:289-294) --
    // and its token id goes to wide_ids[t].
    uint32_t* keys = a.sort_keys_in + (size_t)slot * a.sort_stride;
    int32_t* ids = a.sort_vals_in + (size_t)slot * a.sort_stride;
    const uint32_t* skeys = keys;
    const int32_t* sids = ids;
    int32_t* tok = a.wide_ids + (size_t)slot * a.sort_stride;
    const int sel = wide_sel(rd, a.vocab);
    const bool pen = (rd.flags & SR_ROWFLAG_HAS_PENALTY) != 0u && rd.edit_cnt > 0;
    const SrEdit* ed = a.edits + rd.edit_off;
    for (int t = blockIdx.x * 256 + threadIdx.x; t < sel; t += gridDim.x * 256) {
        float v = sr_okey_inv(skeys[t]);
        int id = sids[t];
        if (sr_f2u(v) == 0xff800000u) {
            id = -1;
        } else if (pen) {
            int lo = 0;
            if (rd.flags & SR_ROWFLAG_EDITS_SORTED) {
                int hi = rd.edit_cnt;
                while (lo < hi) {
                    const int mid = (lo + hi) >> 1;
                    if (ed[mid].id < id) lo = mid + 1; else hi = mid;
                }
            } else {
                // (a row that was meant for the selection kernel and is redone here: its few edits are unsorted)
                while (lo < rd.edit_cnt && ed[lo].id != id) lo++;
            }
            if (lo < rd.edit_cnt && ed[lo].id == id && ed[lo].occ_all > 0) {
                const SrEdit ee = ed[lo];
                if (rd.rep != 1.0f && ee.occ_win > 0) v = v > 0.0f ? __fdiv_rn(v, ee.pen) : __fmul_rn(v, ee.pen);
                v = __fsub_rn(v, __fadd_rn(rd.presence, __fmul_rn(rd.frequency, (float)ee.occ_all)));
            }
        }
        keys[t] = sr_okey(v);
        ids[t] = t;
        tok[t] = id;
    }
}

// One row's (key, id) pairs sorted where they lie by the row's workgroup: descending key, ascending id among equal
// keys.  first != 0: the whole row (ids = token indices: the order the reference's selection keeps, Sampler.cs:232-247);
// else its first `sel` entries after the penalties (ids = places in the first order).
__global__ __launch_bounds__(kT) void k_wide_sort(SrFullArgs a, int first)
{
    __shared__ FullSmem sm;
    const int slot = blockIdx.x;
    const SrRow rd = a.rows[a.row_list[slot]];
    sort_survivors_in_place(a.sort_keys_in + (size_t)slot * a.sort_stride, a.sort_vals_in + (size_t)slot * a.sort_stride,
                            first ? a.vocab : wide_sel(rd, a.vocab), sm);
}

// temperature softmax over the first k entries, min-p, top-p and the draw, all left to right (Sampler.cs:299-356)
__global__ __launch_bounds__(kT) void k_wide_tail(SrFullArgs a)
{
    __shared__ FullSmem sm;
    const int tid = threadIdx.x;
    const int slot = blockIdx.x;
    const int row = a.row_list[slot];
    const SrRow rd = a.rows[row];
    const uint32_t* keys = a.sort_keys_in + (size_t)slot * a.sort_stride;
    const int32_t* pos = a.sort_vals_in + (size_t)slot * a.sort_stride;   // an entry's place in the first order ...
    const int32_t* tok = a.wide_ids + (size_t)slot * a.sort_stride;       // ... names its token id
    float* probs = a.work + (size_t)slot * a.work_stride;
    const int k = min(rd.top_k, wide_sel(rd, a.vocab));
    const float v0 = sr_okey_inv(keys[0]);
    const int id0 = tok[pos[0]];
    if (id0 < 0 || sr_f2u(v0) == 0xff800000u) {
        // nothing above -inf (Sampler.cs:254-255): Greedy over a row of -inf returns index 0
        if (tid == 0) {
            a.out_tokens[row] = 0;
            if (a.out_flags) a.out_flags[row] = SR_KFLAG_TOPK | SR_KFLAG_DEGENERATE;
        }
        return;
    }
    const float inv_temp = rd.temperature == 1.0f ? 1.0f : __fdiv_rn(1.0f, rd.temperature);
    const float mx = __fmul_rn(v0, inv_temp);
    for (int t = tid; t < k; t += kT) {
        const float v = sr_okey_inv(keys[t]);
        probs[t] = sr_f2u(v) == 0xff800000u ? 0.0f : sr_expf(__fsub_rn(__fmul_rn(v, inv_temp), mx));
    }
    __syncthreads();
    int found;
    const float sum = seq_sum_row<false>(probs, k, 0.0f, 0.0f, &found, sm);
    const float inv_sum = sum > 0.0f ? __fdiv_rn(1.0f, sum) : 0.0f;
    __syncthreads();
    row_pass<true>(probs, k, [&](float x, int) -> float { return __fmul_rn(x, inv_sum); });
    __syncthreads();
    int count = k;
    bool amb = false;  // SR_OUT_AMBIGUOUS: a cut or the draw lies on its boundary
    if (rd.min_p > 0.0f) {
        const float thr = __fmul_rn(rd.min_p, probs[0]);
        unsigned long long first = 0ull;  // ~index of the first entry below the threshold
        row_pass<false>(probs, k, [&](float x, int i) -> float {
            if (x < thr) {
                const unsigned long long e = 0xffffffffull - (unsigned long long)(uint32_t)i;
                first = e > first ? e : first;
            }
            return x;
        });
        first = blk_max_u64(first, sm);
        if (first) count = (int)(0xffffffffull - first);
        amb = (count > 0 && sr_near(probs[count - 1], thr)) || (count < k && sr_near(probs[count], thr));
    }
    if (rd.top_p < 1.0f && rd.top_p > 0.0f) {
        const float at = seq_sum_row<true>(probs, count, 0.0f, rd.top_p, &found, sm);
        amb = amb || (found >= 0 ? sr_stop_near(at, probs[found], rd.top_p) : sr_near(at, rd.top_p));
        if (found >= 0) count = found + 1;
    }
    const float kept = seq_sum_row<false>(probs, count, 0.0f, 0.0f, &found, sm);
    const float r = __fmul_rn(__double2float_rn(a.uniforms[(size_t)row * a.uniforms_per_row]), kept);
    const float at = seq_sum_row<true>(probs, count, 0.0f, r, &found, sm);
    amb = amb || (found >= 0 ? sr_stop_near(at, probs[found], r) : sr_near(at, r));
    if (tid == 0) {
        int token = id0;
        if (found >= 0 && tok[pos[found]] >= 0) token = tok[pos[found]];
        a.out_tokens[row] = token;
        if (a.out_flags) a.out_flags[row] = SR_KFLAG_TOPK | (amb ? SR_KFLAG_AMBIGUOUS : 0u);
    }
}

// ---- SampleFromProbs / ResampleResidual on caller-provided distributions ------------------------------
__global__ __launch_bounds__(kT) void k_draw_rows(const float* probs, int64_t stride, int n, const double* uniforms,
                                                   int* out_tokens)
{
    __shared__ FullSmem sm;
    const int row = blockIdx.x;
    const int t = draw_from_row(probs + (size_t)row * stride, n, uniforms[row], sm);
    if (threadIdx.x == 0) out_tokens[row] = t;
}

// residual = max(0, p - q): first the left-to-right sum of the positive residuals, then the first index
// whose running residual reaches (float)u * sum; degenerate residual -> draw from p (Sampler.cs:587-618)
__device__ __forceinline__ int resample_residual_row(const float* p, const float* q, int n, double u, FullSmem& sm,
                                                     float m1 = 1.0f, float m2 = 1.0f)
{
    int dummy;
    auto res = [&](int i) -> float {
        const float r = __fsub_rn(__fmul_rn(__fmul_rn(p[i], m1), m2), q[i]);
        return r > 0.0f ? r : 0.0f;
    };
    SeqMarks marks;
    if (seq_marks_fit(n)) marks.keep = sm.ckpt;
    const float sum = seq_sum_residual<false>(p, q, n, 0.0f, 0.0f, &dummy, sm, m1, m2, marks);
    if (!(sum > 0.0f)) return draw_from_row(p, n, u, sm, m1, m2);  // sum <= 0 or NaN
    const float target = __fmul_rn(__double2float_rn(u), sum);
    // `target <= cum` is only tested on positive residuals: a zero target must not stop on a zero term
    int found;
    if (target <= 0.0f) {
        int first = 0x7fffffff;
        for (int i = threadIdx.x; i < n; i += kT)
            if (res(i) > 0.0f) { first = i; break; }
        first = sr_wave_min_i32(first);
        __syncthreads();
        if (sr_lane() == 0) sm.redi[sr_wave_id()] = first;
        __syncthreads();
        int f = 0x7fffffff;
        for (int w = 0; w < kW; w++) f = min(f, sm.redi[w]);
        __syncthreads();
        return f;  // sum > 0 guarantees a positive residual exists
    }
    float s0 = 0.0f;
    SeqMarks from;
    if (marks.keep) {
        __syncthreads();  // (the marks were written by thread 0)
        from.from = seq_marks_find(sm.ckpt, n, target, &s0);
    }
    seq_sum_residual<true>(p, q, n, s0, target, &found, sm, m1, m2, from);
    if (found >= 0) return found;
    // rounding fallback: the last index with a positive residual
    int last = -1;
    for (int i = threadIdx.x; i < n; i += kT)
        if (res(i) > 0.0f) last = i;
    last = -sr_wave_min_i32(-last);
    __syncthreads();
    if (sr_lane() == 0) sm.redi[sr_wave_id()] = last;
    __syncthreads();
    int l = -1;
    for (int w = 0; w < kW; w++) l = max(l, sm.redi[w]);
    __syncthreads();
    return l;
}

__global__ __launch_bounds__(kT) void k_residual_rows(const float* p, int64_t ps, const float* q, int64_t qs, int n,
                                                       const double* uniforms, int* out_tokens)
{
    __shared__ FullSmem sm;
    const int row = blockIdx.x;
    const int t = resample_residual_row(p + (size_t)row * ps, q + (size_t)row * qs, n, uniforms[row], sm);
    if (threadIdx.x == 0) out_tokens[row] = t;
}

// ... from the residual row itself (res[i] = max(0, fl(fl(p[i] m1) m2) - q[i]), written by k_spec_residual): the same
// terms in the same order, read from one row instead of computed from two
__device__ __forceinline__ int resample_residual_stored(const float* res, const float* p, int n, double u, FullSmem& sm,
                                                        float m1, float m2)
{
    int dummy;
    SeqMarks marks;
    if (seq_marks_fit(n)) marks.keep = sm.ckpt;
    const float sum = seq_sum_row<false>(res, n, 0.0f, 0.0f, &dummy, sm, 1.0f, 1.0f, SeqNoWatch(), SeqNoMap(), marks);
    if (!(sum > 0.0f)) return draw_from_row(p, n, u, sm, m1, m2);  // sum <= 0 or NaN
    const float target = __fmul_rn(__double2float_rn(u), sum);
    auto edge = [&](bool first_one) -> int {  // the first / the last index with a positive residual
        int at = first_one ? 0x7fffffff : -1;
        for (int i = threadIdx.x; i < n; i += kT)
            if (res[i] > 0.0f) {
                at = i;
                if (first_one) break;
            }
        at = first_one ? sr_wave_min_i32(at) : -sr_wave_min_i32(-at);
        __syncthreads();
        if (sr_lane() == 0) sm.redi[sr_wave_id()] = at;
        __syncthreads();
        int f = first_one ? 0x7fffffff : -1;
        for (int w = 0; w < kW; w++) f = first_one ? min(f, sm.redi[w]) : max(f, sm.redi[w]);
        __syncthreads();
        return f;
    };
    if (target <= 0.0f) return edge(true);  // a zero target must not stop on a zero term
    int found;
    float s0 = 0.0f;
    SeqMarks from;
    if (marks.keep) {
        __syncthreads();  // (the marks were written by thread 0)
        from.from = seq_marks_find(sm.ckpt, n, target, &s0);
    }
    seq_sum_row<true>(res, n, s0, target, &found, sm, 1.0f, 1.0f, SeqNoWatch(), SeqNoMap(), from);
    return found >= 0 ? found : edge(false);  // (rounding: the sum of the search fell short of the target)
}

// ... with the increment functions of the stored row's segments at hand (k_seq_funcs): one wave walks them
__device__ __forceinline__ int residual_edge(const float* res, int n, bool first_one, FullSmem& sm)
{
    // the first / the last index with a positive residual
    int at = first_one ? 0x7fffffff : -1;
    for (int i = threadIdx.x; i < n; i += kT)
        if (res[i] > 0.0f) {
            at = i;
            if (first_one) break;
        }
    at = first_one ? sr_wave_min_i32(at) : -sr_wave_min_i32(-at);
    __syncthreads();
    if (sr_lane() == 0) sm.redi[sr_wave_id()] = at;
    __syncthreads();
    int f = first_one ? 0x7fffffff : -1;
    for (int w = 0; w < kW; w++) f = first_one ? min(f, sm.redi[w]) : max(f, sm.redi[w]);
    __syncthreads();
    return f;
}
__device__ __forceinline__ int resample_residual_prepared(const float* res, const SeqSegFunc* funcs, const float* p, int n, double u,
                                                          FullSmem& sm, float m1, float m2)
{
    const bool walker = sr_wave_id() == 0;
    int dummy;
    __syncthreads();  // (sm.segst and sm.segbc are free)
    if (walker) {
        const float sum = seg_walk<false>(res, n, funcs, 0.0f, 0.0f, &dummy, sm.segst);
        if (sr_lane() == 0) sm.segbc[0] = sr_f2u(sum);
    }
    __syncthreads();
    const float sum = sr_u2f(sm.segbc[0]);
    if (!(sum > 0.0f)) return draw_from_row(p, n, u, sm, m1, m2);  // sum <= 0 or NaN
    const float target = __fmul_rn(__double2float_rn(u), sum);
    if (target <= 0.0f) return residual_edge(res, n, true, sm);  // a zero target must not stop on a zero term
    if (walker) {
        float at;
        const int found = seg_search_states(res, n, sm.segst, target, &at);
        if (sr_lane() == 0) sm.segbc[1] = (uint32_t)found;
    }
    __syncthreads();
    const int found = (int)sm.segbc[1];
    return found >= 0 ? found : residual_edge(res, n, false, sm);  // (rounding: the sum of the search fell short of the target)
}
// SampleFromDistribution (Sampler.cs:564-576) over a stored row with its segments' functions: draw_from_row by one wave
__device__ __forceinline__ int draw_from_prepared(const float* terms, const SeqSegFunc* funcs, int n, double u, FullSmem& sm)
{
    const float r = __double2float_rn(u);
    __syncthreads();
    if (sr_wave_id() == 0) {
        int found;
        const float at = seg_walk<true>(terms, n, funcs, 0.0f, r, &found, nullptr);
        if (sr_lane() == 0) {
            sm.segbc[1] = (uint32_t)found;
            SR_AMB_IF(found >= 0 ? sr_stop_near(at, terms[found], r) : sr_near(at, r));
        }
    }
    __syncthreads();
    const int found = (int)sm.segbc[1];
    return found >= 0 ? found : n - 1;
}

// Every position of a row is filtered with the row's own parameters (SpeculativeDecoder.cs:535): the batch's row
// descriptors, one copy per position, without their allow-masks
__global__ __launch_bounds__(256) void k_expand_rows(const SrRow* src, SrRow* dst, int rows, int positions)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * positions) return;
    SrRow d = src[i / positions];
    d.mask_row = -1;
    dst[i] = d;
}

// The accept loop of a row under the ratio test needs one element of p and of q per position, no pass over a row:
// one wave walks it ahead of everything else and names the first rejected position, so that the residual row of
// that position -- which the row's workgroup would otherwise compute twice, from two rows, at the rate of one compute
// unit -- can be written by the whole device (k_spec_residual) before k_spec_verify reads it.
__global__ __launch_bounds__(SR_WAVE) void k_spec_walk(SrSpecArgs a)
{
    const int row = blockIdx.x, lane = sr_lane();
    const SrRow rd = a.rows[row];
    const int n = a.vocab, L = a.n_draft;
    const bool true_spec = !(rd.p_min > 0.0f && rd.p_min < 1.0f) && (rd.flags & SR_ROWBIT_DRAFT_FROM_LOOKUP) == 0u;
    int reject = -1;
    if (true_spec) {
        // (every draft accepted, and a bonus token to draw: position L, whose scaled row k_spec_residual writes out)
        if (a.seg_func && rd.temperature > 0.0f) reject = L;
        const float* pr = a.p_all + (size_t)row * (L + 1) * n;
        const double* u = a.uniforms + (size_t)row * a.uniforms_per_row;
        for (int i0 = 0; i0 < L; i0 += SR_WAVE) {
            const int i = i0 + lane;
            bool stop = false, bad = false;
            if (i < L) {
                const int tok = a.draft_tokens[(size_t)row * L + i];
                bad = (uint32_t)tok >= (uint32_t)n;
                if (!bad) {
                    const SrFullState* sl = a.state + (size_t)row * (L + 1) + i;
                    const float px = __fmul_rn(__fmul_rn(pr[(size_t)i * n + tok], sl->mul1), sl->mul2);
                    const float qx = a.draft_probs[((size_t)row * L + i) * n + tok];
                    const float acc = qx > 0.0f ? fminf(1.0f, __fdiv_rn(px, qx)) : (px > 0.0f ? 1.0f : 0.0f);
                    stop = !(u[i] < (double)acc);  // (every position before it was accepted and drew one uniform)
                }
            }
            const unsigned long long ends = __ballot(stop || bad);
            if (ends != 0ull) {
                const int l = (int)__ffsll((long long)ends) - 1;
                const bool is_bad = ((__ballot(bad) >> l) & 1ull) != 0ull;
                reject = is_bad ? -1 : i0 + l;  // (an id outside the vocabulary ends the row without a correction)
                break;
            }
        }
    }
    if (lane == 0) a.reject[row] = reject;
}

// The terms the row's workgroup will add, written by the whole device: max(0, fl(fl(p m1) m2) - q) of the first rejected
// position, or the scaled target row fl(fl(p m1) m2) of the bonus position when every draft was accepted (reject == L).
// A wave takes whole segments of SR_SEG_TERMS terms and leaves each segment's approximate sum for k_seq_funcs.
__global__ __launch_bounds__(256) void k_spec_residual(SrSpecArgs a)
{
    const int row = blockIdx.y;
    const int i = a.reject[row];
    if (i < 0) return;
    const int n = a.vocab, L = a.n_draft, lane = sr_lane();
    const bool bonus = i == L;
    const float* pd = a.p_all + ((size_t)row * (L + 1) + i) * n;
    const float* qd = bonus ? pd : a.draft_probs + ((size_t)row * L + i) * n;
    const SrFullState* sl = a.state + (size_t)row * (L + 1) + i;
    const float m1 = sl->mul1, m2 = sl->mul2;
    float* out = a.resid + (size_t)row * (size_t)a.resid_stride;
    auto res = [&](float pv, float qv) -> float {
        const float sp = __fmul_rn(__fmul_rn(pv, m1), m2);
        if (bonus) return sp;
        const float r = __fsub_rn(sp, qv);
        return r > 0.0f ? r : 0.0f;
    };
    const bool aligned = ((((uintptr_t)pd) | ((uintptr_t)qd)) & 15u) == 0u;
    const int nseg = seg_count(n);
    for (int seg = (int)blockIdx.x * 4 + sr_wave_id(); seg < nseg; seg += (int)gridDim.x * 4) {
        double acc = 0.0;
#pragma unroll
        for (int k = 0; k < SR_SEG_TERMS / (4 * SR_WAVE); k++) {
            const int x0 = seg * SR_SEG_TERMS + (k * SR_WAVE + lane) * 4;
            if (aligned && x0 + 4 <= n) {
                const float4 pv = *(const float4*)(pd + x0), qv = *(const float4*)(qd + x0);
                float4 o;
                o.x = res(pv.x, qv.x); o.y = res(pv.y, qv.y); o.z = res(pv.z, qv.z); o.w = res(pv.w, qv.w);
                *(float4*)(out + x0) = o;  // (the rows of a.resid start on 16-byte boundaries)
                acc += ((double)o.x + (double)o.y) + ((double)o.z + (double)o.w);
            } else {
                for (int x = x0; x < min(x0 + 4, n); x++) {
                    const float o = res(pd[x], qd[x]);
                    out[x] = o;
                    acc += (double)o;
                }
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
        if (a.seg_part && lane == 0) a.seg_part[(size_t)row * a.seg_stride + seg] = acc;
    }
}

// The record of every segment of every row of terms (SeqSegFunc), for the binades that the approximate sums predict:
// the sums of the segments in front (part, left by the kernel that wrote the terms) and, inside the segment, of the
// lanes in front.  One wave per segment.
__global__ __launch_bounds__(256) void k_seq_funcs(const float* terms, int64_t stride, int n, const double* part, SeqSegFunc* func,
                                                   int seg_stride, const int32_t* active)
{
    const int row = blockIdx.y, lane = sr_lane();
    if (active && active[row] < 0) return;
    const int seg = (int)blockIdx.x * 4 + sr_wave_id();
    if (seg >= seg_count(n)) return;
    const double* pr = part + (size_t)row * seg_stride;
    double before = 0.0;
    for (int g = lane; g < seg; g += SR_WAVE) before += pr[g];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) before += __shfl_xor(before, o);
    const float* t = terms + (size_t)row * (size_t)stride;
    float x[SR_SEQ_RUN];
    seq_load_run(t, ((uintptr_t)t & 15u) == 0u, seg * SR_SEG_TERMS + lane * SR_SEQ_RUN, n, x);
    seg_make_record(x, seg, before, func + (size_t)row * seg_stride + seg);
}

// ---- speculative verification: the accept loop of StepSampled (SpeculativeDecoder.cs:530-559) ---------
// p_all holds the filtered target distributions of every position, [rows][n_draft + 1][n].
__global__ __launch_bounds__(kT) void k_spec_verify(SrSpecArgs a)
{
    __shared__ FullSmem sm;
    const int row = blockIdx.x;
    const SrRow rd = a.rows[row];
    const int n = a.vocab, L = a.n_draft;
    const float* pr = a.p_all + (size_t)row * (L + 1) * n;
    const float* lg = a.target_logits + (size_t)row * (L + 1) * n;
    const double* u = a.uniforms + (size_t)row * a.uniforms_per_row;
    int* out = a.out_tokens + (size_t)row * (L + 1);
    // SpeculativeDecoder.cs:192 and :538, :549 (`_trueSpecSampling && !usedPld`)
    const bool true_spec = !(rd.p_min > 0.0f && rd.p_min < 1.0f) && (rd.flags & SR_ROWBIT_DRAFT_FROM_LOOKUP) == 0u;
    for (int i = threadIdx.x; i <= L; i += kT) out[i] = -1;
    __syncthreads();
    int accepted = 0, udraws = 0, correction = -1;
    bool bad_id = false;
    // What the accept tests need of every position -- the draft token, its target and draft probabilities -- is
    // fetched for all positions at once: three dependent loads per position would otherwise line up one behind
    // the other along the walk.
    constexpr int kStage = 1024;
    const bool staged = L <= kStage;
    if (staged) {
        for (int i = (int)threadIdx.x; i < L; i += kT) {
            const int tok = a.draft_tokens[(size_t)row * L + i];
            const SrFullState* sl = a.state + (size_t)row * (L + 1) + i;
            const bool in_range = (uint32_t)tok < (uint32_t)n;  // an id outside the vocabulary is never dereferenced
            sm.sprob[i] = in_range ? __fmul_rn(__fmul_rn(pr[(size_t)i * n + tok], sl->mul1), sl->mul2) : 0.0f;
            sm.sprob[kStage + i] = (true_spec && in_range) ? a.draft_probs[((size_t)row * L + i) * n + tok] : 0.0f;
            sm.sprob[2 * kStage + i] = __int_as_float(tok);
        }
        for (int i = (int)threadIdx.x; i <= L && i < a.uniforms_per_row; i += kT)
            sm.sortbuf[i] = (unsigned long long)__double_as_longlong(u[i]);
        __syncthreads();
    }
    for (int i = 0; i < L; i++) {
        const float* pd = pr + (size_t)i * n;
        const float* qd = a.draft_probs + ((size_t)row * L + i) * n;
        const int tok = staged ? __float_as_int(sm.sprob[2 * kStage + i]) : a.draft_tokens[(size_t)row * L + i];
        const SrFullState* sl = a.state + (size_t)row * (L + 1) + i;
        // The managed loop indexes pDist[x_i] (SpeculativeDecoder.cs:536) and throws on an id outside the
        // vocabulary: the row ends here, with -1 where its correction token would stand.
        if ((uint32_t)tok >= (uint32_t)n) { bad_id = true; break; }
        const float px = staged ? sm.sprob[i] : __fmul_rn(__fmul_rn(pd[tok], sl->mul1), sl->mul2);
        bool accept;
        if (true_spec) {
            const float qx = staged ? sm.sprob[kStage + i] : qd[tok];
            const float acc = qx > 0.0f ? fminf(1.0f, __fdiv_rn(px, qx)) : (px > 0.0f ? 1.0f : 0.0f);
            const double ui = staged ? __longlong_as_double((long long)sm.sortbuf[udraws]) : u[udraws];
            udraws++;
            accept = ui < (double)acc;
        } else {
            accept = px >= rd.p_min;
            if (!accept) accept = tok == row_argmax(lg + (size_t)i * n, n, sm);  // block-uniform branch
        }
        if (accept) {
            if (threadIdx.x == 0) out[accepted] = tok;
            accepted++;
            continue;
        }
        const float m1 = sl->mul1, m2 = sl->mul2;
        const double uc = u[udraws++];
        if (true_spec && a.reject && a.reject[row] == i && a.seg_func)  // the residual row and its segments' functions are there
            correction = resample_residual_prepared(a.resid + (size_t)row * (size_t)a.resid_stride,
                                                    a.seg_func + (size_t)row * a.seg_stride, pd, n, uc, sm, m1, m2);
        else if (true_spec && a.reject && a.reject[row] == i)  // the residual row is there already
            correction = resample_residual_stored(a.resid + (size_t)row * (size_t)a.resid_stride, pd, n, uc, sm, m1, m2);
        else
            correction = true_spec ? resample_residual_row(pd, qd, n, uc, sm, m1, m2) : draw_from_row(pd, n, uc, sm, m1, m2);
        break;
    }
    if (correction < 0 && !bad_id) {
        // every draft accepted: bonus token from the last position (greedy rows: its argmax, no draw)
        const float* pd = pr + (size_t)L * n;
        const SrFullState* sl = a.state + (size_t)row * (L + 1) + L;
        if (rd.temperature <= 0.0f) correction = row_argmax(pd, n, sm);
        else if (a.seg_func && a.reject[row] == L)  // the scaled row and its segments' functions are there
            correction = draw_from_prepared(a.resid + (size_t)row * (size_t)a.resid_stride, a.seg_func + (size_t)row * a.seg_stride, n,
                                            u[udraws++], sm);
        else correction = draw_from_row(pd, n, u[udraws++], sm, sl->mul1, sl->mul2);
    }
    if (threadIdx.x == 0) {
        out[accepted] = correction;
        a.out_accepted[row] = accepted;
    }
}

// ---- MtpDecoder.AcceptDraft / SoftmaxProbAt (MtpDecoder.cs:562-596) ------------------------------------
__global__ __launch_bounds__(kT) void k_mtp_verify(const float* logits, int64_t stride, int n, const int* draft,
                                                    float p_min, int* out_argmax, int* out_accept, float* out_prob)
{
    __shared__ FullSmem sm;
    __shared__ double dred[kW];
    const int row = blockIdx.x;
    const float* l = logits + (size_t)row * stride;
    const int am = row_argmax(l, n, sm);
    const int d = draft[row];
    float prob = 0.0f;
    int ok = d == am ? 1 : 0;
    if (!ok && p_min < 1.0f) {
        // max, sum of exp(l - max) in double, ratio cast to float.  The double sum is a tree reduction:
        // it can differ from the reference's left-to-right double sum in the last bits, far below the
        // float result's 1e-5 tolerance.
        float m = l[0];
        for (int i = threadIdx.x; i < n; i += kT) m = fmaxf(m, l[i]);
        bool nn;
        m = blk_max_f(m, &nn, sm);
        double s = 0.0;
        for (int i = threadIdx.x; i < n; i += kT) s += exp((double)__fsub_rn(l[i], m));
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
        __syncthreads();
        if (sr_lane() == 0) dred[sr_wave_id()] = s;
        __syncthreads();
        double tot = 0.0;
        for (int w = 0; w < kW; w++) tot += dred[w];
        if (tot > 0.0 && d >= 0 && d < n) prob = (float)(exp((double)__fsub_rn(l[d], m)) / tot);
        ok = prob >= p_min ? 1 : 0;
    }
    if (threadIdx.x == 0) {
        out_argmax[row] = am;
        out_accept[row] = ok;
        if (out_prob) out_prob[row] = prob;
    }
}

#ifdef SR_TEST_HOOKS
__global__ __launch_bounds__(kT) void k_selftest_seqsum(const float* x, int n, float s0, float target, float* out_sum,
                                                         int* out_idx)
{
    __shared__ FullSmem sm;
    int found;
    float s;
    if (target == target)
        s = seq_sum_row<true>(x, n, s0, target, &found, sm);
    else
        s = seq_sum_row<false>(x, n, s0, 0.0f, &found, sm);
    if (threadIdx.x == 0) { *out_sum = s; *out_idx = found; }
}
// The same sum the prepared way: approximate sums of the segments (times `skew`, to make the predictions miss), the
// segments' records, and the walk of one wave -- the sum with the states it leaves and the search from those states
// (out[0], idx[0]), and the walk that searches by itself (out[1], idx[1]).
__global__ __launch_bounds__(256) void k_selftest_segpart(const float* x, int n, double skew, double* part)
{
    const int seg = (int)blockIdx.x * 4 + sr_wave_id(), lane = sr_lane();
    if (seg >= seg_count(n)) return;
    double acc = 0.0;
    for (int j = 0; j < SR_SEQ_RUN; j++) {
        const int i = seg * SR_SEG_TERMS + lane * SR_SEQ_RUN + j;
        if (i < n) acc += (double)x[i];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
    if (lane == 0) part[seg] = acc * skew;
}
__global__ __launch_bounds__(kT) void k_selftest_segwalk(const float* x, int n, const SeqSegFunc* funcs, float target, float* out_sum,
                                                          int* out_idx)
{
    __shared__ FullSmem sm;
    if (sr_wave_id() != 0) return;
    int found = -1, found2 = -1;
    const float s = seg_walk<false>(x, n, funcs, 0.0f, 0.0f, &found, sm.segst);
    float s2 = s;
    if (target == target) {
        float at = 0.0f;
        found = seg_search_states(x, n, sm.segst, target, &at);
        s2 = seg_walk<true>(x, n, funcs, 0.0f, target, &found2, nullptr);
    }
    if (sr_lane() == 0) { out_sum[0] = s; out_sum[1] = s2; out_idx[0] = found; out_idx[1] = found2; }
}
#endif

}  // namespace

hipError_t sr_launch_full_prep(const SrFullArgs& a, int n_rows, hipStream_t st)
{
    if (n_rows <= 0) return hipSuccess;
    const int bx = max(1, min(64, (a.vocab + 256 * 16 - 1) / (256 * 16)));
    dim3 grid(bx, n_rows);
    // (the adjusted copy only where some row keeps one: the host knows)
    if (a.dtype == 1) {
        if (a.any_copy) hipLaunchKernelGGL(k_full_prep<2>, grid, dim3(256), 0, st, a);
        if (a.any_edits) hipLaunchKernelGGL(k_full_edits<2>, dim3(n_rows), dim3(256), 0, st, a);
    } else {
        if (a.any_copy) hipLaunchKernelGGL(k_full_prep<4>, grid, dim3(256), 0, st, a);
        if (a.any_edits) hipLaunchKernelGGL(k_full_edits<4>, dim3(n_rows), dim3(256), 0, st, a);
    }
    if (a.seg_func) {
        const int nseg = (a.vocab + SR_SEG_TERMS - 1) / SR_SEG_TERMS;
        // a wave takes one segment, or two where the launch's sampled rows have more segments than the device holds waves
        // of the one-segment kind at a time: the waves of a row's workgroups wait for each other between the passes
        const bool two = (long long)a.n_sampled * nseg > 3072;
        const int per_group = 4 * (two ? 2 : 1);
        dim3 fgrid((unsigned)((nseg + per_group - 1) / per_group), n_rows);
        if (a.dtype == 1) {
            if (two) hipLaunchKernelGGL((k_full_softmax_seg<2, 4, 2>), fgrid, dim3(256), 0, st, a);
            else hipLaunchKernelGGL((k_full_softmax_seg<2, 4, 1>), fgrid, dim3(256), 0, st, a);
        } else {
            if (two) hipLaunchKernelGGL((k_full_softmax_seg<4, 4, 2>), fgrid, dim3(256), 0, st, a);
            else hipLaunchKernelGGL((k_full_softmax_seg<4, 4, 1>), fgrid, dim3(256), 0, st, a);
        }
    } else if (a.dtype == 1) {
        hipLaunchKernelGGL(k_full_max<2>, grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL(k_full_exp<2>, grid, dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL(k_full_max<4>, grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL(k_full_exp<4>, grid, dim3(256), 0, st, a);
    }
    return hipGetLastError();
}
hipError_t sr_launch_wide_keys(const SrFullArgs& a, int n_rows, hipStream_t st)
{
    if (n_rows <= 0) return hipSuccess;
    dim3 grid(max(1, min(64, (a.vocab + 256 * 16 - 1) / (256 * 16))), n_rows);
    if (a.dtype == 1) hipLaunchKernelGGL(k_wide_keys<2>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(k_wide_keys<4>, grid, dim3(256), 0, st, a);
    return hipGetLastError();
}
hipError_t sr_launch_wide_adjust(const SrFullArgs& a, int n_rows, hipStream_t st)
{
    if (n_rows <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_wide_adjust, dim3(32, n_rows), dim3(256), 0, st, a);
    return hipGetLastError();
}
hipError_t sr_launch_wide_sort(const SrFullArgs& a, int n_rows, int first, hipStream_t st)
{
    hipLaunchKernelGGL(k_wide_sort, dim3((unsigned)n_rows), dim3(kT), 0, st, a, first);
    return hipGetLastError();
}
hipError_t sr_launch_wide_tail(const SrFullArgs& a, int n_rows, hipStream_t st)
{
    if (n_rows <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_wide_tail, dim3(n_rows), dim3(kT), 0, st, a);
    return hipGetLastError();
}
hipError_t sr_launch_full_row(const SrFullArgs& a, int n_rows, hipStream_t st)
{
    if (n_rows <= 0) return hipSuccess;
    // (rows that only top-p cuts walk their nucleus in slabs of twice the size when the launch gives the room: see
    // nucleus_from_histogram)
    const unsigned more = a.big_slabs ? 16u * (unsigned)kSmall : 0u;
    if (more) {
        static bool allowed[64] = {};  // (once per device)
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        if (dev < 0 || dev >= 64 || !allowed[dev]) {
            e = hipFuncSetAttribute((const void*)k_full_row, hipFuncAttributeMaxDynamicSharedMemorySize, (int)more);
            if (e != hipSuccess) return e;
            if (dev >= 0 && dev < 64) allowed[dev] = true;
        }
    }
    hipLaunchKernelGGL(k_full_row, dim3(n_rows), dim3(kT), more, st, a);
    return hipGetLastError();
}
hipError_t sr_launch_draw_rows(const float* probs, int64_t stride, int n, int rows, const double* u, int* out,
                               hipStream_t st)
{
    if (rows <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_draw_rows, dim3(rows), dim3(kT), 0, st, probs, stride, n, u, out);
    return hipGetLastError();
}
hipError_t sr_launch_residual_rows(const float* p, int64_t ps, const float* q, int64_t qs, int n, int rows,
                                   const double* u, int* out, hipStream_t st)
{
    if (rows <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_residual_rows, dim3(rows), dim3(kT), 0, st, p, ps, q, qs, n, u, out);
    return hipGetLastError();
}
hipError_t sr_launch_expand_rows(const SrRow* src, SrRow* dst, int rows, int positions, hipStream_t st)
{
    if (rows <= 0 || positions <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_expand_rows, dim3((unsigned)((rows * positions + 255) / 256)), dim3(256), 0, st, src, dst, rows, positions);
    return hipGetLastError();
}
hipError_t sr_launch_spec_verify(const SrSpecArgs& a, int rows, hipStream_t st)
{
    if (rows <= 0) return hipSuccess;
    SrSpecArgs b = a;
    if (!(b.resid && b.reject && b.n_draft > 0 && b.draft_probs && rows <= 65535)) {  // (rows are the grid's second dimension)
        b.resid = nullptr;
        b.reject = nullptr;
        b.seg_func = nullptr;
    } else {
        const int nseg = (b.vocab + SR_SEG_TERMS - 1) / SR_SEG_TERMS;
        if (!(b.seg_func && b.seg_part && nseg <= SR_SEG_MAX && nseg <= b.seg_stride)) b.seg_func = nullptr;
        hipLaunchKernelGGL(k_spec_walk, dim3(rows), dim3(SR_WAVE), 0, st, b);
        hipLaunchKernelGGL(k_spec_residual, dim3((unsigned)std::min(64, (nseg + 3) / 4), rows), dim3(256), 0, st, b);
        if (b.seg_func)
            hipLaunchKernelGGL(k_seq_funcs, dim3((unsigned)((nseg + 3) / 4), rows), dim3(256), 0, st, b.resid, b.resid_stride, b.vocab,
                               b.seg_part, (SeqSegFunc*)b.seg_func, b.seg_stride, b.reject);
    }
    hipLaunchKernelGGL(k_spec_verify, dim3(rows), dim3(kT), 0, st, b);
    return hipGetLastError();
}
hipError_t sr_launch_mtp_verify(const float* logits, int64_t stride, int n, int rows, const int* draft, float p_min,
                                int* out_argmax, int* out_accept, float* out_prob, hipStream_t st)
{
    if (rows <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_mtp_verify, dim3(rows), dim3(kT), 0, st, logits, stride, n, draft, p_min, out_argmax,
                       out_accept, out_prob);
    return hipGetLastError();
}
#ifdef SR_TEST_HOOKS
hipError_t sr_launch_selftest_seqsum(const float* x, int n, float s0, float target, float* out_sum, int* out_idx,
                                     hipStream_t st)
{
    hipLaunchKernelGGL(k_selftest_seqsum, dim3(1), dim3(kT), 0, st, x, n, s0, target, out_sum, out_idx);
    return hipGetLastError();
}
hipError_t sr_launch_selftest_segsum(const float* x, int n, double skew, float target, double* part, SeqSegFunc* funcs,
                                     float* out_sum, int* out_idx, hipStream_t st)
{
    const int nseg = (n + SR_SEG_TERMS - 1) / SR_SEG_TERMS;
    hipLaunchKernelGGL(k_selftest_segpart, dim3((unsigned)((nseg + 3) / 4)), dim3(256), 0, st, x, n, skew, part);
    hipLaunchKernelGGL(k_seq_funcs, dim3((unsigned)((nseg + 3) / 4), 1), dim3(256), 0, st, x, (int64_t)0, n, part, funcs, nseg,
                       (const int32_t*)nullptr);
    hipLaunchKernelGGL(k_selftest_segwalk, dim3(1), dim3(kT), 0, st, x, n, funcs, target, out_sum, out_idx);
    return hipGetLastError();
}
#endif
