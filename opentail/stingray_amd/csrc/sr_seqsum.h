// Exact parallel evaluation of a SEQUENTIAL fp32 running sum  s <- fl(s + x_i),  x_i >= 0,  i ascending.
//
// The reference sampler accumulates its softmax denominator, its nucleus cut-off and its multinomial
// draw with plain left-to-right float adds (Sampler.cs:460-465, :536-546, :564-576, :594-614).  The
// rounding of every add depends on the running value, so a tree reduction gives different bits.  This
// primitive reproduces the left-to-right result bit for bit, in parallel:
//
//   * While s stays inside one binade [2^E, 2^(E+1)) its ulp u is fixed and s = n*u with an integer n.
//     A round-to-nearest-even add of x is then  n <- n + floor(x/u) + [frac > 1/2] + [frac == 1/2 and
//     (n + floor(x/u)) odd]:  an integer add that depends on n only through its parity.
//   * A run of terms is therefore a function n -> n + a[n & 1]; such functions compose associatively
//     (c[p] = a[p] + b[(p + a[p]) & 1]), so a block-wide scan gives the exact state at every run boundary.
//   * When the scan shows that some run would carry n to 2^24 (the sum leaves the binade), everything
//     before that run is already exact; the one run is replayed with real float adds from its exact
//     input, and the rest of the tile is rescanned in the new binade.  A sum crosses at most ~150
//     binades, in practice a handful.
//
// Block size: SR_SEQ_THREADS threads, of which the first SR_SEQ_ACTIVE carry SR_SEQ_RUN consecutive terms each, so
// one tile covers SR_SEQ_ACTIVE * SR_SEQ_RUN terms (a round of the tile costs what its waves' scans cost: with the
// terms in half as many waves, twice as many each, a round takes about half the time).  All threads of the block
// must call.
#pragma once
#include "sr_device.h"

#define SR_SEQ_THREADS 1024
#define SR_SEQ_ACTIVE 1024  // threads that carry terms in sr_seq_tile: the first eight waves (the others only meet at the barriers)
#define SR_SEQ_RUN 16
#define SR_SEQ_RUN8 16  // terms per thread of the eight-chain tile
#define SR_SEQ_TILE (SR_SEQ_ACTIVE * SR_SEQ_RUN)
#define SR_SEQ_WAVES (SR_SEQ_THREADS / SR_WAVE)
#define SR_SEQ_SAT (1u << 26)  // saturated increment: "this run leaves the binade"

// The guard band behind SR_OUT_AMBIGUOUS: two values count as "on the same boundary" when they are within about four
// ulps of each other.  The managed runtime leaves three things open that can move a running sum by an ulp or two --
// the lane order of TensorPrimitives.Sum, the last bit of expf, the order of equal keys in its sort --; a draw or a
// cut that clears its boundary by more than this band comes out the same whichever way those fall.
#define SR_AMBIG_REL 4.8e-7f
__device__ __forceinline__ bool sr_near(float a, float b) { return fabsf(a - b) <= fmaxf(fabsf(a), fabsf(b)) * SR_AMBIG_REL; }
// A search stopped at a term of size `term` where the running sum `at` reached `target`: the stop is on a boundary
// when the sum barely reached the target, or the sum before the term (at - term) barely missed it.
__device__ __forceinline__ bool sr_stop_near(float at, float term, float target)
{
    return sr_near(at, target) || (term - (at - target)) <= at * SR_AMBIG_REL;
}

struct SrSeqSmem {
    uint32_t wa0[2][SR_SEQ_WAVES];  // every wave's increment function, rounds alternate between the two copies
    uint32_t wa1[2][SR_SEQ_WAVES];
    uint32_t misc[8];
};
static_assert(SR_SEQ_WAVES == 16, "the wave totals are scanned inside one DPP row of 16 lanes");

// n -> n + a[n & 1]
struct SrInc {
    uint32_t a0, a1;
};
__device__ __forceinline__ uint32_t sr_sat_add(uint32_t x, uint32_t y)
{
    uint32_t r = x + y;
    return r > SR_SEQ_SAT ? SR_SEQ_SAT : r;
}
// apply f first, then g
__device__ __forceinline__ SrInc sr_compose(SrInc f, SrInc g)
{
    SrInc c;
    c.a0 = sr_sat_add(f.a0, (f.a0 & 1u) ? g.a1 : g.a0);
    c.a1 = sr_sat_add(f.a1, ((1u + f.a1) & 1u) ? g.a1 : g.a0);
    return c;
}

// integer view of a non-negative float: s = n * 2^(eb - 150) with eb = max(biased exponent, 1)
__device__ __forceinline__ void sr_split(float s, uint32_t* n, int* eb)
{
    const uint32_t b = sr_f2u(s);
    const uint32_t e = b >> 23;
    *n = (b & 0x7fffffu) | (e ? 0x800000u : 0u);
    *eb = e ? (int)e : 1;
}
__device__ __forceinline__ float sr_join(uint32_t n, int eb) { return sr_u2f(n + ((uint32_t)(eb - 1) << 23)); }

// The increment function of the terms x[0..N) in the binade with exponent field eb: the hardware's
// own round-to-nearest-even adds, run once from the binade's first even value and once from its first odd
// value.  While such a chain stays inside the binade its bit pattern minus the start's is the number of ulps
// gained, and that number is the same for every start of the same parity.  A chain that leaves the binade
// (the run gains 2^23 ulps or more, or a term is too large for it) saturates: the caller replays that run.
template <int N> __device__ __forceinline__ SrInc sr_run_inc(const float (&x)[N], int eb)
{
    const uint32_t base = eb > 1 ? ((uint32_t)eb << 23) : 0u;    // n = 2^23 (or 0 below the normal range): even
    const uint32_t limit = eb > 1 ? base + (1u << 23) : (1u << 24);  // first bit pattern outside the binade
    float sa = sr_u2f(base), sb = sr_u2f(base + 1u);
#pragma unroll
    for (int j = 0; j < N; j++) {
        sa = __fadd_rn(sa, x[j]);
        sb = __fadd_rn(sb, x[j]);
    }
    const uint32_t ba = sr_f2u(sa), bb = sr_f2u(sb);
    SrInc r;
    r.a0 = (ba < limit) ? ba - base : SR_SEQ_SAT;
    r.a1 = (bb < limit) ? bb - (base + 1u) : SR_SEQ_SAT;
    return r;
}

// Inclusive scan of increment functions: DPP shifts with zero fill inside rows of 16 lanes ((0, 0) is the identity
// of sr_compose), v_readlane for the rows before.  With kRowOnly the rows stay separate.
template <bool kRowOnly>
__device__ __forceinline__ SrInc sr_scan_inc(SrInc v)
{
    // Nearly always every lane's increment is the same for both parities (they differ only behind an add that fell
    // exactly half way between two values): the functions are then plain numbers and their composition is a sum.
    if (__ballot(v.a0 != v.a1) == 0ull) {
        uint32_t t = v.a0;
        t = sr_sat_add(t, sr_dpp_u32<0x111>(t));
        t = sr_sat_add(t, sr_dpp_u32<0x112>(t));
        t = sr_sat_add(t, sr_dpp_u32<0x114>(t));
        t = sr_sat_add(t, sr_dpp_u32<0x118>(t));
        if (!kRowOnly) {
            const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)t, 15);
            const uint32_t r1 = sr_sat_add(r0, (uint32_t)__builtin_amdgcn_readlane((int)t, 31));
            const uint32_t r2 = sr_sat_add(r1, (uint32_t)__builtin_amdgcn_readlane((int)t, 47));
            const int row = sr_lane() >> 4;
            t = sr_sat_add(row == 1 ? r0 : row == 2 ? r1 : row == 3 ? r2 : 0u, t);
        }
        v.a0 = v.a1 = t;
        return v;
    }
    auto step = [&](auto ctrl) {
        constexpr int kC = decltype(ctrl)::value;
        SrInc lo;
        lo.a0 = sr_dpp_u32<kC>(v.a0);
        lo.a1 = sr_dpp_u32<kC>(v.a1);
        v = sr_compose(lo, v);
    };
    step(std::integral_constant<int, 0x111>{});
    step(std::integral_constant<int, 0x112>{});
    step(std::integral_constant<int, 0x114>{});
    step(std::integral_constant<int, 0x118>{});
    if (kRowOnly) return v;
    auto total = [&](int l) {
        SrInc t;
        t.a0 = (uint32_t)__builtin_amdgcn_readlane((int)v.a0, l);
        t.a1 = (uint32_t)__builtin_amdgcn_readlane((int)v.a1, l);
        return t;
    };
    const SrInc p1 = total(15), p2 = sr_compose(p1, total(31)), p3 = sr_compose(p2, total(47));
    const int row = sr_lane() >> 4;
    SrInc pre;
    pre.a0 = row == 1 ? p1.a0 : row == 2 ? p2.a0 : row == 3 ? p3.a0 : 0u;
    pre.a1 = row == 1 ? p1.a1 : row == 2 ? p2.a1 : row == 3 ? p3.a1 : 0u;
    return sr_compose(pre, v);
}

// One tile: adds this thread's SR_SEQ_RUN terms (thread order = term order) to the running sum *s
// (uniform across the block on entry and exit).  When kSearch, also looks for the first term index at
// which the running sum reaches `target` (fl(s) >= target); on success returns its tile-local index
// (thread * SR_SEQ_RUN + j) in *found (uniform) and *s is the running sum at that term; else leaves -1.  Terms
// past the end must be 0.
//
// Per round: every wave scans its threads' increment functions and publishes its total; every wave then scans the
// sixteen totals itself, which also shows the first wave in which the sum leaves the binade (or reaches the
// target); that wave alone finds the thread and replays its run with real float adds; everything after it is
// rescanned in the new binade.  A tile that stays in its binade costs two barriers.
//
// A sum that starts small doubles within a few terms, again within twice as many, and so on: after a crossing at
// thread f the next one is expected near thread 2f.  The round after a crossing therefore looks at the threads up to
// 2f + 64 only (waves outside that window skip the arithmetic and the scan); a window that passes without a
// crossing is settled like a whole tile and the rest of the tile follows in one more round.  The wave that holds a
// crossing finishes all of its 64 threads by itself before the block goes on.
template <bool kSearch>
__device__ __forceinline__ void sr_seq_tile(const float (&x)[SR_SEQ_RUN], float* s, float target, int* found,
                                            SrSeqSmem& sm)
{
    const int tid = threadIdx.x, lane = sr_lane();
    const int wave = __builtin_amdgcn_readfirstlane(sr_wave_id());
    int start = 0;             // threads below `start` are settled
    int wend = SR_SEQ_ACTIVE;  // this round looks at the threads [start, wend); a multiple of the wave size
    float s_in = *s;
    *found = -1;
    sr_barrier_lds();  // the previous call's readers are done with the arrays below
    for (int round = 0;; round++) {
        const int buf = round & 1;
        uint32_t n_in;
        int eb;
        sr_split(s_in, &n_in, &eb);
        SrInc mine;
        mine.a0 = 0u; mine.a1 = 0u;
        SrInc incl = mine;
        if ((wave + 1) * SR_WAVE > start && wave * SR_WAVE < wend) {  // (uniform per wave)
            if (tid >= start) mine = sr_run_inc(x, eb);
            incl = sr_scan_inc<false>(mine);
        }
        // (this copy is written again two rounds on, behind a barrier that every reader of it has passed)
        if (lane == SR_WAVE - 1) { sm.wa0[buf][wave] = incl.a0; sm.wa1[buf][wave] = incl.a1; }
        sr_barrier_lds();
        SrInc ti; ti.a0 = 0u; ti.a1 = 0u;
        if (lane < SR_SEQ_WAVES) { ti.a0 = sm.wa0[buf][lane]; ti.a1 = sm.wa1[buf][lane]; }
        ti = sr_scan_inc<true>(ti);  // lanes 0..15: the state function at the end of every wave
        // the running value never decreases, so the first wave whose end state has left the binade (or reached
        // the target) holds the first such thread
        const uint32_t end_n = sr_sat_add(n_in, (n_in & 1u) ? ti.a1 : ti.a0);
        bool event = end_n >= (1u << 24);
        if (kSearch) event = event || sr_join(end_n, eb) >= target;
        const unsigned long long ev = __ballot(event && lane < SR_SEQ_WAVES);
        if (!ev) {
            // everything up to the window's end stays in the binade: settle with the total
            const uint32_t tot = (uint32_t)__builtin_amdgcn_readlane((int)((n_in & 1u) ? ti.a1 : ti.a0), SR_SEQ_WAVES - 1);
            s_in = sr_join(n_in + tot, eb);
            if (wend >= SR_SEQ_ACTIVE) { *s = s_in; return; }
            start = wend;
            wend = SR_SEQ_ACTIVE;
            continue;
        }
        const int ev_wave = (int)__ffsll((long long)ev) - 1;
        if (wave == ev_wave) {
            SrInc pre; pre.a0 = 0u; pre.a1 = 0u;
            if (wave > 0) {
                pre.a0 = (uint32_t)__builtin_amdgcn_readlane((int)ti.a0, wave - 1);
                pre.a1 = (uint32_t)__builtin_amdgcn_readlane((int)ti.a1, wave - 1);
            }
            // The exact state at this wave's first lane; from here the wave goes on alone, crossing after crossing
            // (a sum that starts small crosses several binades inside one wave), and hands the block the state
            // behind its last lane: no barrier and no shared memory per crossing.
            uint32_t n_w = n_in + ((n_in & 1u) ? pre.a1 : pre.a0);
            int eb_w = eb;
            SrInc sc = incl;  // inclusive scan of the wave's increments in the binade eb_w, from n_w
            int lstart = max(start - wave * SR_WAVE, 0);  // lanes below are settled
            float s_w = 0.0f;
            int where = -1, last = SR_WAVE - 1;
            for (;;) {
                SrInc ex;
                ex.a0 = __shfl_up(sc.a0, 1);
                ex.a1 = __shfl_up(sc.a1, 1);
                if (lane == 0) { ex.a0 = 0u; ex.a1 = 0u; }
                const bool odd = (n_w & 1u) != 0u;
                // exact integer state before / after this thread's run, valid while below 2^24
                const uint32_t before = sr_sat_add(n_w, odd ? ex.a1 : ex.a0);
                const uint32_t after = sr_sat_add(n_w, odd ? sc.a1 : sc.a0);
                bool mine_ev = after >= (1u << 24);
                if (kSearch) mine_ev = mine_ev || sr_join(after, eb_w) >= target;
                const unsigned long long evl = __ballot(mine_ev && lane >= lstart);
                if (!evl) {
                    // the rest of the wave stays in the binade
                    const uint32_t tot = (uint32_t)__builtin_amdgcn_readlane((int)(odd ? sc.a1 : sc.a0), SR_WAVE - 1);
                    s_w = sr_join(n_w + tot, eb_w);
                    last = SR_WAVE - 1;
                    break;
                }
                const int fl = (int)__ffsll((long long)evl) - 1;
                // every lane replays its run with real float adds from its own input; the first event lane's counts
                float acc = sr_join(before, eb_w), hit = 0.0f;
                int wj = -1;
#pragma unroll
                for (int j = 0; j < SR_SEQ_RUN; j++) {
                    acc = __fadd_rn(acc, x[j]);
                    if (kSearch && wj < 0 && acc >= target) { wj = j; hit = acc; }
                }
                s_w = sr_u2f((uint32_t)__builtin_amdgcn_readlane((int)sr_f2u(acc), fl));
                wj = __builtin_amdgcn_readlane(wj, fl);
                last = fl;
                if (kSearch && wj >= 0) {  // (the sum handed back is the running sum AT the term that reached the target)
                    s_w = sr_u2f((uint32_t)__builtin_amdgcn_readlane((int)sr_f2u(hit), fl));
                    where = (wave * SR_WAVE + fl) * SR_SEQ_RUN + wj;
                    break;
                }
                lstart = fl + 1;
                if (lstart >= SR_WAVE) break;
                // the lanes behind it, scanned again in the binade the sum has reached
                sr_split(s_w, &n_w, &eb_w);
                SrInc m;
                m.a0 = 0u; m.a1 = 0u;
                if (lane >= lstart) m = sr_run_inc(x, eb_w);
                sc = sr_scan_inc<false>(m);
            }
            if (lane == 0) {
                sm.misc[0] = sr_f2u(s_w);
                sm.misc[1] = (uint32_t)where;
                sm.misc[2] = (uint32_t)(wave * SR_WAVE + last);
            }
        }
        sr_barrier_lds();
        s_in = sr_u2f(sm.misc[0]);
        const int where = (int)sm.misc[1];
        const int fst = (int)sm.misc[2];
        if (kSearch && where >= 0) { *found = where; *s = s_in; return; }
        start = fst + 1;
        if (start >= SR_SEQ_ACTIVE) { *s = s_in; return; }
        // (a tile's first crossing is mostly its only one -- a sum that has grown doubles once in many tiles --, so the
        // round after it takes the whole rest; from the second crossing on the sum is doubling fast)
        wend = round == 0 ? SR_SEQ_ACTIVE : min(SR_SEQ_ACTIVE, (2 * start + 2 * SR_WAVE - 1) & ~(SR_WAVE - 1));
    }
}

// ---- one wave by itself --------------------------------------------------------------------------------
// The running sum s of the wave's 64 x N terms (lane order = term order, N consecutive terms per lane), crossing after
// crossing, with no barrier and no shared memory: what a short list needs (a row tail's few hundred probabilities).
// When kSearch, stops at the first term at which the running sum reaches `target`: *found = its index (lane * N + j,
// else -1) and the returned value is the running sum AT that term.  Terms past the end must be 0.  All 64 lanes call.
template <int N, bool kSearch>
__device__ __forceinline__ float sr_seq_wave(const float (&x)[N], float s, float target, int* found)
{
    const int lane = sr_lane();
    int lstart = 0;  // lanes below are settled
    *found = -1;
    for (;;) {
        uint32_t n_w;
        int eb_w;
        sr_split(s, &n_w, &eb_w);
        SrInc m;
        m.a0 = 0u; m.a1 = 0u;
        if (lane >= lstart) m = sr_run_inc(x, eb_w);
        const SrInc sc = sr_scan_inc<false>(m);
        SrInc ex;
        ex.a0 = __shfl_up(sc.a0, 1);
        ex.a1 = __shfl_up(sc.a1, 1);
        if (lane == 0) { ex.a0 = 0u; ex.a1 = 0u; }
        const bool odd = (n_w & 1u) != 0u;
        // exact integer state before / after this lane's run, valid while below 2^24
        const uint32_t before = sr_sat_add(n_w, odd ? ex.a1 : ex.a0);
        const uint32_t after = sr_sat_add(n_w, odd ? sc.a1 : sc.a0);
        bool ev = after >= (1u << 24);
        if (kSearch) ev = ev || sr_join(after, eb_w) >= target;
        const unsigned long long evl = __ballot(ev && lane >= lstart);
        if (!evl) {  // the rest of the wave stays in the binade and below the target
            const uint32_t tot = (uint32_t)__builtin_amdgcn_readlane((int)(odd ? sc.a1 : sc.a0), SR_WAVE - 1);
            return sr_join(n_w + tot, eb_w);
        }
        const int fl = (int)__ffsll((long long)evl) - 1;
        // the first such lane's run, replayed with real float adds from its exact input (every lane replays its own)
        float acc = sr_join(before, eb_w), hit = 0.0f;
        int wj = -1;
#pragma unroll
        for (int j = 0; j < N; j++) {
            acc = __fadd_rn(acc, x[j]);
            if (kSearch && wj < 0 && acc >= target) { wj = j; hit = acc; }
        }
        wj = __builtin_amdgcn_readlane(wj, fl);
        if (kSearch && wj >= 0) {
            *found = fl * N + wj;
            return sr_u2f((uint32_t)__builtin_amdgcn_readlane((int)sr_f2u(hit), fl));
        }
        s = sr_u2f((uint32_t)__builtin_amdgcn_readlane((int)sr_f2u(acc), fl));
        lstart = fl + 1;
        if (lstart >= SR_WAVE) return s;
    }
}

// ---- eight independent chains at once -----------------------------------------------------------------
// Thread t serves chain (t & 7) with the SR_SEQ_RUN8 terms number (t >> 3) * SR_SEQ_RUN8 ... of that chain's
// tile, so one tile covers SR_SEQ_THREADS / 8 * SR_SEQ_RUN8 terms of every chain.  *s is the running sum
// of the caller's chain (uniform across the threads of a chain).  Terms past the end must be 0.  All
// threads of the block must call.
#define SR_SEQ_CHAINS 8
#define SR_SEQ_CHAIN_THREADS (SR_SEQ_THREADS / SR_SEQ_CHAINS)
#define SR_SEQ_CHAIN_TILE (SR_SEQ_CHAIN_THREADS * SR_SEQ_RUN8)

struct SrSeq8Smem {
    uint32_t wa0[2][SR_SEQ_WAVES][SR_SEQ_CHAINS];  // every wave's increment function per chain; rounds alternate
    uint32_t wa1[2][SR_SEQ_WAVES][SR_SEQ_CHAINS];
    uint32_t acc[SR_SEQ_CHAINS];                   // a chain's exact sum behind the run that left the binade ...
    int first[SR_SEQ_CHAINS];                      // ... and the chain thread that run belongs to
};

// inclusive scan of increment functions over the lanes of a wave that are 8, 16, ... apart (one chain's lanes)
__device__ __forceinline__ SrInc sr_scan_inc_chain(SrInc v)
{
    const int lane = sr_lane();
    SrInc lo;
#pragma unroll
    for (int o = SR_SEQ_CHAINS; o < SR_WAVE; o <<= 1) {
        lo.a0 = __shfl_up(v.a0, o);
        lo.a1 = __shfl_up(v.a1, o);
        if (lane >= o) v = sr_compose(lo, v);
    }
    return v;
}

// One tile of all eight chains.  Per round: every wave scans its threads' increment functions chain by chain and
// publishes the eight wave totals; every wave then scans the 16 x 8 totals itself (two per lane), which gives each
// thread its chain's state at its wave's start and at the tile's end, and shows, per chain, the first wave in which
// the chain's sum leaves the binade.  That wave finds the thread and replays its run with real float adds; the
// chain's later threads are rescanned in the new binade.  A tile in which no chain leaves its binade costs two
// barriers.
__device__ __forceinline__ void sr_seq_tile8(const float (&x)[SR_SEQ_RUN8], float* s, SrSeq8Smem& sm)
{
    static_assert(SR_SEQ_WAVES == 16 && SR_SEQ_CHAINS == 8 && SR_WAVE == 64, "two wave totals per lane and chain");
    const int tid = threadIdx.x, lane = sr_lane();
    const int wave = __builtin_amdgcn_readfirstlane(sr_wave_id());
    const int g = tid & (SR_SEQ_CHAINS - 1), lt = tid >> 3;  // chain, position inside the chain
    const unsigned long long chain_lanes = 0x0101010101010101ull << g;
    int start = 0;     // chain threads below `start` are settled
    bool done = false; // this chain has finished the tile
    float s_in = *s;
    sr_barrier_lds();  // the previous call's readers are done with the arrays below
    for (int round = 0;; round++) {
        const int buf = round & 1;
        uint32_t n_in;
        int eb;
        sr_split(s_in, &n_in, &eb);
        const bool odd = (n_in & 1u) != 0u;
        SrInc mine;
        mine.a0 = 0u; mine.a1 = 0u;
        if (!done && lt >= start) mine = sr_run_inc(x, eb);
        const SrInc incl = sr_scan_inc_chain(mine);
        // (this copy is written again two rounds on, behind a barrier that every reader of it has passed)
        if (lane >= SR_WAVE - SR_SEQ_CHAINS) { sm.wa0[buf][wave][g] = incl.a0; sm.wa1[buf][wave][g] = incl.a1; }
        sr_barrier_lds();
        // lane l holds, for chain l & 7, the totals of wave l >> 3 and of wave 8 + (l >> 3)
        SrInc ta, tb;
        ta.a0 = sm.wa0[buf][lane >> 3][g]; ta.a1 = sm.wa1[buf][lane >> 3][g];
        tb.a0 = sm.wa0[buf][8 + (lane >> 3)][g]; tb.a1 = sm.wa1[buf][8 + (lane >> 3)][g];
        ta = sr_scan_inc_chain(ta);
        tb = sr_scan_inc_chain(tb);
        SrInc half;
        half.a0 = __shfl(ta.a0, SR_WAVE - SR_SEQ_CHAINS + g);
        half.a1 = __shfl(ta.a1, SR_WAVE - SR_SEQ_CHAINS + g);
        tb = sr_compose(half, tb);  // the chain's state function at the end of waves 8..15
        const uint32_t t0 = __shfl(tb.a0, SR_WAVE - SR_SEQ_CHAINS + g), t1 = __shfl(tb.a1, SR_WAVE - SR_SEQ_CHAINS + g);
        // the first wave at whose end the chain has left the binade (the running value never decreases)
        const bool gone_a = !done && sr_sat_add(n_in, odd ? ta.a1 : ta.a0) >= (1u << 24);
        const bool gone_b = !done && sr_sat_add(n_in, odd ? tb.a1 : tb.a0) >= (1u << 24);
        const unsigned long long ba = __ballot(gone_a), bb = __ballot(gone_b);
        if ((ba | bb) == 0ull) {
            // no chain leaves its binade: settle every chain that is still open with its total
            if (!done) s_in = sr_join(n_in + (odd ? t1 : t0), eb);
            break;
        }
        // (every lane takes part in the shuffles below: what differs per chain comes after them)
        const unsigned long long ma = ba & chain_lanes, mb = bb & chain_lanes;
        const int ev_wave = ma ? ((int)__ffsll((long long)ma) - 1) >> 3 : (mb ? 8 + (((int)__ffsll((long long)mb) - 1) >> 3) : -1);
        // the chain's state function at the start of this wave
        const int src_lane = ((wave - 1) & 7) * SR_SEQ_CHAINS + g;
        SrInc pa, pb;
        pa.a0 = __shfl(ta.a0, src_lane); pa.a1 = __shfl(ta.a1, src_lane);
        pb.a0 = __shfl(tb.a0, src_lane); pb.a1 = __shfl(tb.a1, src_lane);
        SrInc pre;
        pre.a0 = wave == 0 ? 0u : (wave <= 8 ? pa.a0 : pb.a0);
        pre.a1 = wave == 0 ? 0u : (wave <= 8 ? pa.a1 : pb.a1);
        SrInc ex;
        ex.a0 = __shfl_up(incl.a0, SR_SEQ_CHAINS);
        ex.a1 = __shfl_up(incl.a1, SR_SEQ_CHAINS);
        if (lane < SR_SEQ_CHAINS) { ex.a0 = 0u; ex.a1 = 0u; }
        ex = sr_compose(pre, ex);
        const uint32_t before = sr_sat_add(n_in, odd ? ex.a1 : ex.a0);
        const SrInc thr = sr_compose(ex, mine);
        const uint32_t after = sr_sat_add(n_in, odd ? thr.a1 : thr.a0);
        const bool leaves = !done && lt >= start && wave == ev_wave && after >= (1u << 24);
        const unsigned long long bl = __ballot(leaves) & chain_lanes;
        if (leaves && lane == (int)__ffsll((long long)bl) - 1) {
            // the chain's first thread that leaves: replay its run with real float adds from its exact input
            float acc = sr_join(before, eb);
#pragma unroll
            for (int j = 0; j < SR_SEQ_RUN8; j++) acc = __fadd_rn(acc, x[j]);
            sm.acc[g] = sr_f2u(acc);
            sm.first[g] = lt;
        }
        sr_barrier_lds();
        if (!done) {
            if (ev_wave < 0) {
                s_in = sr_join(n_in + (odd ? t1 : t0), eb);  // this chain stays in its binade to the tile's end
                done = true;
            } else {
                s_in = sr_u2f(sm.acc[g]);
                start = sm.first[g] + 1;
                if (start >= SR_SEQ_CHAIN_THREADS) done = true;
            }
        }
    }
    *s = s_in;
}
