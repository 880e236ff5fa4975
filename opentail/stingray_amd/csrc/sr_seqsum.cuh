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
// Block size: SR_SEQ_THREADS threads, SR_SEQ_RUN consecutive terms per thread, so one tile covers
// SR_SEQ_THREADS * SR_SEQ_RUN terms.  All threads of the block must call.
#pragma once
#include "sr_device.cuh"

#define SR_SEQ_THREADS 1024
#define SR_SEQ_RUN 16
#define SR_SEQ_TILE (SR_SEQ_THREADS * SR_SEQ_RUN)
#define SR_SEQ_WAVES (SR_SEQ_THREADS / SR_WAVE)
#define SR_SEQ_SAT (1u << 26)  // saturated increment: "this run leaves the binade"

struct SrSeqSmem {
    uint32_t wa0[SR_SEQ_WAVES];
    uint32_t wa1[SR_SEQ_WAVES];
    uint32_t misc[8];
    int first[SR_SEQ_WAVES];
};

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

// The increment function of `cnt` terms x[0..cnt) in the binade with exponent field eb.
__device__ __forceinline__ SrInc sr_run_inc(const float (&x)[SR_SEQ_RUN], int eb)
{
    uint32_t A = 0u, B = 1u;  // running n for an even / odd start
    bool hard = false;
#pragma unroll
    for (int j = 0; j < SR_SEQ_RUN; j++) {
        const uint32_t b = sr_f2u(x[j]);
        const uint32_t e = b >> 23;
        const uint32_t M = (b & 0x7fffffu) | (e ? 0x800000u : 0u);
        const int d = eb - (e ? (int)e : 1);
        uint32_t fl = 0u, up = 0u, tie = 0u;
        if (M != 0u) {
            if (d < 0) {
                hard = true;
            } else if (d == 0) {
                fl = M;  // same ulp: exact integer add (a normal s then leaves the binade, caught below)
            } else if (d <= 24) {
                fl = M >> d;
                const uint32_t rem = M & ((1u << d) - 1u), half = 1u << (d - 1);
                up = rem > half ? 1u : 0u;
                tie = rem == half ? 1u : 0u;
            }
        }
        A = A + fl + up + (tie & (A + fl) & 1u);
        B = B + fl + up + (tie & (B + fl) & 1u);
    }
    SrInc r;
    r.a0 = hard ? SR_SEQ_SAT : (A > SR_SEQ_SAT ? SR_SEQ_SAT : A);
    r.a1 = hard ? SR_SEQ_SAT : (B - 1u > SR_SEQ_SAT ? SR_SEQ_SAT : B - 1u);
    return r;
}

// Inclusive scan of the per-thread increment functions over the block.  Returns the EXCLUSIVE prefix
// (the function of all lower threads); *total receives the function of the whole block.
__device__ __forceinline__ SrInc sr_block_scan_inc(SrInc v, SrInc* total, SrSeqSmem& sm)
{
    const int lane = sr_lane(), wave = sr_wave_id();
    SrInc incl = v;
#pragma unroll
    for (int o = 1; o < SR_WAVE; o <<= 1) {
        SrInc lo;
        lo.a0 = __shfl_up(incl.a0, o);
        lo.a1 = __shfl_up(incl.a1, o);
        if (lane >= o) incl = sr_compose(lo, incl);
    }
    __syncthreads();
    if (lane == SR_WAVE - 1) { sm.wa0[wave] = incl.a0; sm.wa1[wave] = incl.a1; }
    __syncthreads();
    SrInc pre; pre.a0 = 0u; pre.a1 = 0u;
    SrInc all; all.a0 = 0u; all.a1 = 0u;
#pragma unroll
    for (int w = 0; w < SR_SEQ_WAVES; w++) {
        SrInc t; t.a0 = sm.wa0[w]; t.a1 = sm.wa1[w];
        if (w < wave) pre = sr_compose(pre, t);
        all = sr_compose(all, t);
    }
    *total = all;
    // exclusive within the wave
    SrInc ex;
    ex.a0 = __shfl_up(incl.a0, 1);
    ex.a1 = __shfl_up(incl.a1, 1);
    if (lane == 0) { ex.a0 = 0u; ex.a1 = 0u; }
    return sr_compose(pre, ex);
}

// One tile: adds this thread's SR_SEQ_RUN terms (thread order = term order) to the running sum *s
// (uniform across the block on entry and exit).  When kSearch, also looks for the first term index at
// which the running sum reaches `target` (fl(s) >= target); on success returns its tile-local index
// (thread * SR_SEQ_RUN + j) in *found (uniform), else leaves -1.  Terms past the end must be 0.
template <bool kSearch>
__device__ __forceinline__ void sr_seq_tile(const float (&x)[SR_SEQ_RUN], float* s, float target, int* found,
                                            SrSeqSmem& sm)
{
    const int tid = threadIdx.x;
    int start = 0;  // threads below `start` are settled
    float s_in = *s;
    *found = -1;
    for (;;) {
        uint32_t n_in;
        int eb;
        sr_split(s_in, &n_in, &eb);
        SrInc mine;
        mine.a0 = 0u; mine.a1 = 0u;
        if (tid >= start) mine = sr_run_inc(x, eb);
        SrInc total;
        const SrInc ex = sr_block_scan_inc(mine, &total, sm);
        // exact integer state before / after this thread's run, valid while below 2^24
        const uint32_t before = sr_sat_add(n_in, (n_in & 1u) ? ex.a1 : ex.a0);
        const SrInc thr = sr_compose(ex, mine);
        const uint32_t after = sr_sat_add(n_in, (n_in & 1u) ? thr.a1 : thr.a0);
        const bool leaves = tid >= start && after >= (1u << 24);
        bool hit = false;
        if (kSearch) hit = tid >= start && !leaves && sr_join(after, eb) >= target;
        // first thread that leaves the binade, first thread that reaches the target
        int cand = (leaves || hit) ? tid : 0x7fffffff;
        cand = sr_wave_min_i32(cand);
        __syncthreads();
        if (sr_lane() == 0) sm.first[sr_wave_id()] = cand;
        __syncthreads();
        int fst = 0x7fffffff;
#pragma unroll
        for (int w = 0; w < SR_SEQ_WAVES; w++) fst = min(fst, sm.first[w]);
        if (fst == 0x7fffffff) {
            // the whole remainder stays in the binade: settle with the block total
            const uint32_t n_out = n_in + ((n_in & 1u) ? total.a1 : total.a0);
            *s = sr_join(n_out, eb);
            return;
        }
        // thread fst replays its run with real float adds from its exact input
        if (tid == fst) {
            float acc = sr_join(before, eb);
            int where = -1;
#pragma unroll
            for (int j = 0; j < SR_SEQ_RUN; j++) {
                acc = __fadd_rn(acc, x[j]);
                if (kSearch && where < 0 && acc >= target) where = fst * SR_SEQ_RUN + j;
            }
            sm.misc[0] = sr_f2u(acc);
            sm.misc[1] = (uint32_t)where;
        }
        __syncthreads();
        s_in = sr_u2f(sm.misc[0]);
        const int where = (int)sm.misc[1];
        __syncthreads();
        if (kSearch && where >= 0) { *found = where; *s = s_in; return; }
        start = fst + 1;
        if (start >= SR_SEQ_THREADS) { *s = s_in; return; }
    }
}
