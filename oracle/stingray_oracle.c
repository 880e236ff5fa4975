/*
 * CPU oracle: plain-C restatement of the reference sampler.  TEST INFRASTRUCTURE ONLY -- see
 * stingray_oracle.h for what it is, what it pins and what stays unpinned.
 *
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fno-fast-math -mfma (see oracle/Makefile).
 * -ffp-contract=off matters: the managed JIT never fuses a*b+c, so neither may this file; the only
 * fused operations are the explicit fma() calls inside oracle_expf.
 */
#include "stingray_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------ */
/* bit helpers                                                                                 */
/* ------------------------------------------------------------------------------------------ */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline uint64_t d2u(double d) { uint64_t u; memcpy(&u, &d, 8); return u; }
static inline double u2d(uint64_t u) { double d; memcpy(&d, &u, 8); return d; }
static inline int is_neg_inf(float v) { return f2u(v) == 0xff800000u; }

/* ------------------------------------------------------------------------------------------ */
/* MathF.Exp -> glibc expf (published algorithm: sysdeps/ieee754/flt-32/e_expf.c, data in       */
/* e_exp2f_data.c), with the contractions of the -mfma build.  Called at Sampler.cs:308,463.    */
/* ------------------------------------------------------------------------------------------ */
static const uint64_t k_exp2f_tab[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

float oracle_expf(float x)
{
    const double N = 32.0;
    const double inv_ln2_n = 0x1.71547652b82fep+0 * N;
    const double shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / N / N / N;
    const double c1 = 0x1.ebfce50fac4f3p-3 / N / N;
    const double c2 = 0x1.62e42ff0c52d6p-1 / N;

    uint32_t abstop = (f2u(x) >> 20) & 0x7ff;
    if (abstop >= (0x42b00000u >> 20)) { /* |x| >= 88 or NaN */
        if (f2u(x) == 0xff800000u) return 0.0f;
        if (abstop >= (0x7f800000u >> 20)) return x + x;
        if (x > 0x1.62e42ep6f) return INFINITY;
        if (x < -0x1.9fe368p6f) return 0.0f;
    }
    double xd = (double)x;
    double z = inv_ln2_n * xd;
    double kd = z + shift;
    uint64_t ki = d2u(kd);
    kd -= shift;
    double r = fma(inv_ln2_n, xd, -kd);
    uint64_t t = k_exp2f_tab[ki % 32];
    t += ki << (52 - 5);
    double s = u2d(t);
    double zz = fma(c0, r, c1);
    double r2 = r * r;
    double y = fma(c2, r, 1.0);
    y = fma(zz, r2, y);
    y = y * s;
    return (float)y;
}

/* ------------------------------------------------------------------------------------------ */
/* System.Random(seed) (runtime: Random.Net5CompatImpl / CompatPrng, Knuth subtractive)        */
/* ------------------------------------------------------------------------------------------ */
void oracle_rng_replay(oracle_rng* r, const double* values, int64_t n)
{
    memset(r, 0, sizeof(*r));
    r->replay = values;
    r->replay_len = n;
}

void oracle_dotnet_random_init(oracle_rng* r, int32_t seed)
{
    memset(r, 0, sizeof(*r));
    int32_t* sa = r->seed_array;
    int32_t subtraction = (seed == INT32_MIN) ? INT32_MAX : (seed < 0 ? -seed : seed);
    int32_t mj = 161803398 - subtraction;
    sa[55] = mj;
    int32_t mk = 1;
    int ii = 0;
    for (int i = 1; i < 55; i++) {
        if ((ii += 21) >= 55) ii -= 55;
        sa[ii] = mk;
        mk = mj - mk;
        if (mk < 0) mk += INT32_MAX;
        mj = sa[ii];
    }
    for (int k = 1; k < 5; k++) {
        for (int i = 1; i < 56; i++) {
            int n = i + 30;
            if (n >= 55) n -= 55;
            /* wraps like the runtime's unchecked int arithmetic */
            sa[i] = (int32_t)((uint32_t)sa[i] - (uint32_t)sa[1 + n]);
            if (sa[i] < 0) sa[i] += INT32_MAX;
        }
    }
    r->inext = 0;
    r->inextp = 21;
}

int32_t oracle_dotnet_random_next(oracle_rng* r)
{
    int32_t* sa = r->seed_array;
    int li = r->inext, lp = r->inextp;
    if (++li >= 56) li = 1;
    if (++lp >= 56) lp = 1;
    int32_t ret = (int32_t)((uint32_t)sa[li] - (uint32_t)sa[lp]);
    if (ret == INT32_MAX) ret--;
    if (ret < 0) ret += INT32_MAX;
    sa[li] = ret;
    r->inext = li;
    r->inextp = lp;
    r->pos++;
    return ret;
}

double oracle_rng_next_double(oracle_rng* r)
{
    if (r->replay) {
        double v = (r->pos < r->replay_len) ? r->replay[r->pos] : 0.0;
        r->pos++;
        return v;
    }
    return oracle_dotnet_random_next(r) * (1.0 / INT32_MAX);
}

/* ------------------------------------------------------------------------------------------ */
/* TensorPrimitives                                                                            */
/* ------------------------------------------------------------------------------------------ */
float oracle_tp_max(const float* x, int32_t n)
{
    float m = x[0];
    for (int32_t i = 0; i < n; i++) {
        float v = x[i];
        if (v != v) return v;                 /* NaN propagates */
        if (v > m) m = v;
    }
    return m;
}

int32_t oracle_tp_index_of_max(const float* x, int32_t n)
{
    if (n <= 0) return -1;
    int32_t best = 0;
    float m = x[0];
    if (m != m) return 0;
    for (int32_t i = 1; i < n; i++) {
        float v = x[i];
        if (v != v) return i;                 /* first NaN wins */
        if (v > m) { m = v; best = i; }       /* strict: first maximum survives */
    }
    return best;
}

float oracle_tp_sum(const float* x, int32_t n)
{
    if (n < 4) {
        float s = 0.0f;
        for (int32_t i = 0; i < n; i++) s += x[i];
        return s;
    }
    const int w = (n >= 8) ? 8 : 4;
    float acc[8];
    for (int j = 0; j < w; j++) acc[j] = x[j];
    int32_t i = w;
    const int32_t one_from_end = n - w;
    while (i <= one_from_end) {
        for (int j = 0; j < w; j++) acc[j] += x[i + j];
        i += w;
    }
    if (i != n) {
        const int rem = n - i;
        for (int j = 0; j < w; j++)
            acc[j] += (j >= w - rem) ? x[n - w + j] : 0.0f;
    }
    if (w == 8)
        return ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    return (acc[0] + acc[1]) + (acc[2] + acc[3]);
}

/* ------------------------------------------------------------------------------------------ */
/* scratch                                                                                     */
/* ------------------------------------------------------------------------------------------ */
static _Thread_local float* tl_probs = NULL;
static _Thread_local int32_t tl_probs_cap = 0;
static _Thread_local float* tl_aux = NULL;
static _Thread_local int32_t tl_aux_cap = 0;

static float* scratch_probs(int32_t n)
{
    if (n > tl_probs_cap) {
        free(tl_probs);
        tl_probs = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
        tl_probs_cap = n;
    }
    return tl_probs;
}
static float* scratch_aux(int32_t n)
{
    if (n > tl_aux_cap) {
        free(tl_aux);
        tl_aux = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
        tl_aux_cap = n;
    }
    return tl_aux;
}

void oracle_params_default(oracle_params* p)
{
    memset(p, 0, sizeof(*p));
    p->temperature = 1.0f;
    p->top_p = 1.0f;
    p->repetition_penalty = 1.0f;
    p->repeat_last_n = 64;
    p->spec_draft_p_min = 1.0f;
    p->draft_from_lookup = 0;
}

static inline int has_history_penalty(const oracle_params* p) /* Sampler.cs:686 */
{
    return p->repetition_penalty != 1.0f || p->presence_penalty != 0.0f || p->frequency_penalty != 0.0f;
}

/* Sampler.cs:442-446 */
int32_t oracle_greedy(const float* logits, int32_t n)
{
    if (n <= 0) return 0;
    return oracle_tp_index_of_max(logits, n);
}

/* Sampler.cs:364-365 */
static inline int32_t repeat_window_start(int32_t count, int32_t last_n)
{
    return (last_n <= 0 || last_n >= count) ? 0 : count - last_n;
}

static int cmp_int(const void* a, const void* b)
{
    int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
    return (x > y) - (x < y);
}

/* Sampler.cs:367-419 */
static void apply_history_penalties(float* logits, int32_t n, const oracle_params* p)
{
    if (!p->prev || p->n_prev <= 0) return;
    const int32_t count = p->n_prev;

    if (p->repetition_penalty != 1.0f) {
        int32_t start = repeat_window_start(count, p->repeat_last_n);
        for (int32_t i = start; i < count; i++) {
            int32_t id = p->prev[i];
            if ((uint32_t)id < (uint32_t)n)
                logits[id] = logits[id] > 0.0f ? logits[id] / p->repetition_penalty
                                               : logits[id] * p->repetition_penalty;
        }
    }
    if (p->presence_penalty == 0.0f && p->frequency_penalty == 0.0f) return;

    int32_t* ids = (int32_t*)malloc(sizeof(int32_t) * (size_t)count);
    int32_t kept = 0;
    for (int32_t i = 0; i < count; i++) {
        int32_t id = p->prev[i];
        if ((uint32_t)id < (uint32_t)n) ids[kept++] = id;
    }
    qsort(ids, (size_t)kept, sizeof(int32_t), cmp_int);
    for (int32_t i = 0; i < kept;) {
        int32_t id = ids[i];
        int32_t end = i + 1;
        while (end < kept && ids[end] == id) end++;
        float sub = p->presence_penalty + p->frequency_penalty * (float)(end - i);
        logits[id] -= sub;
        i = end;
    }
    free(ids);
}

/* Sampler.cs:421-437 */
static int32_t greedy_with_history_penalties(const float* logits, int32_t n, const oracle_params* p)
{
    float* adj = scratch_probs(n);
    memcpy(adj, logits, sizeof(float) * (size_t)n);
    apply_history_penalties(adj, n, p);
    return oracle_greedy(adj, n);
}

static inline int32_t greedy_dispatch(const float* logits, int32_t n, const oracle_params* p)
{
    return (has_history_penalty(p) && p->prev && p->n_prev > 0)
               ? greedy_with_history_penalties(logits, n, p)
               : oracle_greedy(logits, n);
}

/* Sampler.cs:448-472 */
static void softmax(float* x, int32_t n)
{
    float max = oracle_tp_max(x, n);
    if (is_neg_inf(max) || max != max) {
        float uniform = n > 0 ? 1.0f / (float)n : 0.0f;
        for (int32_t i = 0; i < n; i++) x[i] = uniform;
        return;
    }
    float sum = 0.0f;
    for (int32_t i = 0; i < n; i++) {
        x[i] = oracle_expf(x[i] - max);
        sum += x[i];
    }
    if (sum > 0.0f && sum != 1.0f) {
        float inv = 1.0f / sum;
        for (int32_t i = 0; i < n; i++) x[i] = x[i] * inv;
    }
}

/* Sampler.cs:624-645 */
static float find_kth_largest(const float* data, int32_t n, int32_t k)
{
    float* top = (float*)malloc(sizeof(float) * (size_t)k);
    for (int32_t i = 0; i < k; i++) top[i] = -INFINITY;
    for (int32_t i = 0; i < n; i++) {
        float val = data[i];
        if (val > top[k - 1]) {
            top[k - 1] = val;
            for (int32_t j = k - 1; j > 0 && top[j] > top[j - 1]; j--) {
                float t = top[j]; top[j] = top[j - 1]; top[j - 1] = t;
            }
        }
    }
    float kth = top[k - 1];
    free(top);
    return kth;
}

/* Sampler.cs:477-488 */
static void apply_top_k(float* probs, int32_t n, int32_t k)
{
    float kth = find_kth_largest(probs, n, k);
    for (int32_t i = 0; i < n; i++)
        if (probs[i] < kth) probs[i] = 0.0f;
}

/* Sampler.cs:493-503 */
static void apply_min_p(float* probs, int32_t n, float min_p)
{
    float max_prob = oracle_tp_max(probs, n);
    float thr = min_p * max_prob;
    for (int32_t i = 0; i < n; i++)
        if (probs[i] < thr) probs[i] = 0.0f;
}

typedef struct { int32_t idx; float prob; } idx_prob;
static int cmp_prob_desc_idx_asc(const void* a, const void* b)
{
    const idx_prob* x = (const idx_prob*)a;
    const idx_prob* y = (const idx_prob*)b;
    if (x->prob > y->prob) return -1;
    if (x->prob < y->prob) return 1;
    return (x->idx > y->idx) - (x->idx < y->idx);
}

/* Sampler.cs:516-551 */
static void apply_top_p(float* probs, int32_t n, float top_p)
{
    int32_t cnt = 0;
    for (int32_t i = 0; i < n; i++)
        if (probs[i] > 0.0f) cnt++;
    if (cnt == 0) return;
    idx_prob* ix = (idx_prob*)malloc(sizeof(idx_prob) * (size_t)cnt);
    int32_t j = 0;
    for (int32_t i = 0; i < n; i++)
        if (probs[i] > 0.0f) { ix[j].idx = i; ix[j].prob = probs[i]; j++; }
    qsort(ix, (size_t)cnt, sizeof(idx_prob), cmp_prob_desc_idx_asc);
    float cum = 0.0f;
    int32_t cutoff = cnt;
    for (int32_t i = 0; i < cnt; i++) {
        cum += ix[i].prob;
        if (cum >= top_p) { cutoff = i + 1; break; }
    }
    for (int32_t i = cutoff; i < cnt; i++) probs[ix[i].idx] = 0.0f;
    free(ix);
}

/* Sampler.cs:553-562 */
static void normalize(float* probs, int32_t n)
{
    float sum = oracle_tp_sum(probs, n);
    if (sum > 0.0f && sum != 1.0f) {
        float inv = 1.0f / sum;
        for (int32_t i = 0; i < n; i++) probs[i] = probs[i] * inv;
    }
}

/* Sampler.cs:564-576 */
static int32_t sample_from_distribution(const float* probs, int32_t n, oracle_rng* rng)
{
    float r = (float)oracle_rng_next_double(rng);
    float cum = 0.0f;
    for (int32_t i = 0; i < n; i++) {
        cum += probs[i];
        if (r <= cum) return i;
    }
    return n - 1;
}

int32_t oracle_sample_from_probs(const float* probs, int32_t n, oracle_rng* rng)
{
    return sample_from_distribution(probs, n, rng);
}

/* Sampler.cs:216-357 */
static int32_t sample_top_k(const float* logits, int32_t vocab, const oracle_params* p,
                            oracle_rng* rng, int has_penalty)
{
    const int32_t k = p->top_k;
    const int32_t prev_count = has_penalty ? p->n_prev : 0;
    int64_t sel64 = (int64_t)k + prev_count;
    const int32_t sel = (int32_t)(sel64 < vocab ? sel64 : vocab);

    int32_t* idx = (int32_t*)malloc(sizeof(int32_t) * (size_t)sel);
    float* vals = (float*)malloc(sizeof(float) * (size_t)sel);
    float* probs = (float*)malloc(sizeof(float) * (size_t)k);
    int32_t result;

    for (int32_t i = 0; i < sel; i++) { vals[i] = -INFINITY; idx[i] = -1; }
    for (int32_t i = 0; i < vocab; i++) {
        float v = logits[i];
        if (v <= vals[sel - 1]) continue;
        int32_t j = sel - 1;
        while (j > 0 && vals[j - 1] < v) { vals[j] = vals[j - 1]; idx[j] = idx[j - 1]; j--; }
        vals[j] = v; idx[j] = i;
    }

    if (idx[0] < 0 || is_neg_inf(vals[0])) {
        result = oracle_greedy(logits, vocab);
        goto done;
    }

    if (has_penalty) {
        for (int32_t t = 0; t < sel; t++) {
            if (idx[t] < 0) continue;
            int32_t window_start = repeat_window_start(p->n_prev, p->repeat_last_n);
            int32_t occ_window = 0, occ_all = 0;
            for (int32_t h = 0; h < p->n_prev; h++) {
                if (p->prev[h] != idx[t]) continue;
                occ_all++;
                if (h >= window_start) occ_window++;
            }
            if (occ_all == 0) continue;
            if (p->repetition_penalty != 1.0f && occ_window > 0) {
                float pen = powf(p->repetition_penalty, (float)occ_window);
                vals[t] = vals[t] > 0.0f ? vals[t] / pen : vals[t] * pen;
            }
            float sub = p->presence_penalty + p->frequency_penalty * (float)occ_all;
            vals[t] -= sub;
        }
        for (int32_t a = 1; a < sel; a++) {
            float v = vals[a]; int32_t id = idx[a]; int32_t b = a - 1;
            while (b >= 0 && vals[b] < v) { vals[b + 1] = vals[b]; idx[b + 1] = idx[b]; b--; }
            vals[b + 1] = v; idx[b + 1] = id;
        }
    }

    {
        /* With k + prev_count > vocab, sel is clamped to vocab and may be < k only when k >= vocab,
         * which the dispatch excludes; so k <= sel always holds here. */
        float inv_temp = p->temperature == 1.0f ? 1.0f : 1.0f / p->temperature;
        float max = vals[0] * inv_temp;
        float sum = 0.0f;
        for (int32_t t = 0; t < k; t++) {
            float e = is_neg_inf(vals[t]) ? 0.0f : oracle_expf(vals[t] * inv_temp - max);
            probs[t] = e;
            sum += e;
        }
        float inv_sum = sum > 0.0f ? 1.0f / sum : 0.0f;
        for (int32_t t = 0; t < k; t++) probs[t] *= inv_sum;

        int32_t count = k;
        if (p->min_p > 0.0f) {
            float thr = p->min_p * probs[0];
            for (int32_t t = 0; t < count; t++)
                if (probs[t] < thr) { count = t; break; }
        }
        if (p->top_p < 1.0f && p->top_p > 0.0f) {
            float cum = 0.0f;
            for (int32_t t = 0; t < count; t++) {
                cum += probs[t];
                if (cum >= p->top_p) { count = t + 1; break; }
            }
        }
        float kept_sum = 0.0f;
        for (int32_t t = 0; t < count; t++) kept_sum += probs[t];
        float r = (float)oracle_rng_next_double(rng) * kept_sum;
        float c = 0.0f;
        result = idx[0];
        for (int32_t t = 0; t < count; t++) {
            c += probs[t];
            if (r <= c && idx[t] >= 0) { result = idx[t]; break; }
        }
    }
done:
    free(idx); free(vals); free(probs);
    return result;
}

/* The slow-path pipeline shared by Sample (:48-92) and BuildFilteredDistribution (:134-162).
 * The two differ only in how the temperature multiply is spelled (TensorPrimitives.Multiply vs a
 * scalar loop), which is the same element-wise fp32 product. */
static void slow_pipeline(const float* logits, int32_t n, const oracle_params* p, float* probs)
{
    memcpy(probs, logits, sizeof(float) * (size_t)n);
    if (p->n_bias > 0)
        for (int32_t b = 0; b < p->n_bias; b++) {
            int32_t id = p->bias_ids[b];
            if ((uint32_t)id < (uint32_t)n) probs[id] += p->bias_vals[b];
        }
    apply_history_penalties(probs, n, p);
    if (p->temperature != 1.0f) {
        float inv_temp = 1.0f / p->temperature;
        for (int32_t i = 0; i < n; i++) probs[i] = probs[i] * inv_temp;
    }
    softmax(probs, n);
    if (p->top_k > 0 && p->top_k < n) {
        apply_top_k(probs, n, p->top_k);
        normalize(probs, n);
    }
    if (p->min_p > 0.0f) apply_min_p(probs, n, p->min_p);
    if (p->top_p < 1.0f && p->top_p > 0.0f) apply_top_p(probs, n, p->top_p);
    normalize(probs, n);
}

/* Sampler.cs:17-102 */
int32_t oracle_sample(const float* logits, int32_t n, const oracle_params* p, oracle_rng* rng)
{
    if (p->temperature <= 0.0f) return greedy_dispatch(logits, n, p);

    int has_bias = p->n_bias > 0;
    int has_penalty = (p->prev && p->n_prev > 0) &&
                      (p->repetition_penalty != 1.0f || p->presence_penalty != 0.0f ||
                       p->frequency_penalty != 0.0f);
    if (p->top_k > 0 && p->top_k < n && !has_bias)
        return sample_top_k(logits, n, p, rng, has_penalty);

    float* probs = scratch_aux(n);
    slow_pipeline(logits, n, p, probs);
    return sample_from_distribution(probs, n, rng);
}

/* Sampler.cs:118-163 */
int32_t oracle_build_filtered_distribution(const float* logits, int32_t n, const oracle_params* p,
                                           float* probs, int32_t n_probs)
{
    if (n_probs != n) return -1; /* ArgumentException */
    if (p->temperature <= 0.0f) {
        memset(probs, 0, sizeof(float) * (size_t)n);
        probs[greedy_dispatch(logits, n, p)] = 1.0f;
        return 0;
    }
    slow_pipeline(logits, n, p, probs);
    return 0;
}

/* Sampler.cs:172-187 */
int32_t oracle_sample_with_distribution(const float* logits, int32_t n, const oracle_params* p,
                                        float* probs, oracle_rng* rng)
{
    if (p->temperature <= 0.0f) {
        int32_t am = greedy_dispatch(logits, n, p);
        memset(probs, 0, sizeof(float) * (size_t)n);
        probs[am] = 1.0f;
        return am;
    }
    oracle_build_filtered_distribution(logits, n, p, probs, n);
    return sample_from_distribution(probs, n, rng);
}

/* Sampler.cs:587-618 */
int32_t oracle_resample_residual(const float* p, int32_t np, const float* q, int32_t nq, oracle_rng* rng)
{
    if (np != nq) return -1; /* ArgumentException */
    float sum = 0.0f;
    for (int32_t i = 0; i < np; i++) {
        float r = p[i] - q[i];
        if (r > 0.0f) sum += r;
    }
    if (sum <= 0.0f || sum != sum) return sample_from_distribution(p, np, rng);

    float target = (float)oracle_rng_next_double(rng) * sum;
    float cum = 0.0f;
    int32_t last_positive = -1;
    for (int32_t i = 0; i < np; i++) {
        float r = p[i] - q[i];
        if (r > 0.0f) {
            last_positive = i;
            cum += r;
            if (target <= cum) return i;
        }
    }
    return last_positive >= 0 ? last_positive : sample_from_distribution(p, np, rng);
}

/* Core/Grammar/ITokenConstraint.cs:31-42; producers e.g. ChoiceConstraint.cs:84-105 */
void oracle_apply_allow_mask(const float* logits, const uint32_t* mask_words, int32_t n, float* out)
{
    for (int32_t i = 0; i < n; i++)
        out[i] = ((mask_words[i >> 5] >> (i & 31)) & 1u) ? logits[i] : -INFINITY;
}

/* SpeculativeDecoder.cs:530-559 (tokens[0], the certain token, is not part of this loop) */
int32_t oracle_spec_verify_row(const float* target_logits, const float* draft_probs,
                               const int32_t* draft_tokens, int32_t n_draft, int32_t n,
                               const oracle_params* p, oracle_rng* rng, float* p_dist,
                               int32_t* out_tokens)
{
    /* SpeculativeDecoder.cs:192 */
    int true_spec = !(p->spec_draft_p_min > 0.0f && p->spec_draft_p_min < 1.0f);
    /* :538, :549: `_trueSpecSampling && !usedPld` -- lookup drafts have no q, so they take the other rule */
    if (p->draft_from_lookup) true_spec = 0;
    int32_t accepted = 0;
    int32_t correction = -1;
    for (int32_t i = 0; i < n_draft; i++) {
        const float* tl = target_logits + (int64_t)i * n;
        const float* qd = draft_probs + (int64_t)i * n;
        int32_t tok = draft_tokens[i];
        oracle_build_filtered_distribution(tl, n, p, p_dist, n);
        /* pDist[x_i] with x_i outside the vocabulary throws IndexOutOfRangeException (SpeculativeDecoder.cs:536):
         * the row ends at this position, reported as -1 in place of its correction token */
        if (tok < 0 || tok >= n) { out_tokens[accepted] = -1; return accepted; }
        float px = p_dist[tok];
        int accept;
        if (true_spec) {
            float qx = qd[tok];
            float a = qx > 0.0f ? fminf(1.0f, px / qx) : (px > 0.0f ? 1.0f : 0.0f);
            accept = oracle_rng_next_double(rng) < (double)a;
        } else {
            accept = px >= p->spec_draft_p_min || tok == oracle_greedy(tl, n);
        }
        if (accept) { out_tokens[accepted++] = tok; continue; }
        correction = true_spec ? oracle_resample_residual(p_dist, n, qd, n, rng)
                               : oracle_sample_from_probs(p_dist, n, rng);
        break;
    }
    if (correction < 0)
        correction = oracle_sample_with_distribution(target_logits + (int64_t)n_draft * n, n, p, p_dist, rng);
    out_tokens[accepted] = correction;
    return accepted;
}

/* MtpDecoder.cs:584-596 */
float oracle_softmax_prob_at(const float* logits, int32_t n, int32_t idx)
{
    float max = logits[0];
    for (int32_t i = 1; i < n; i++)
        if (logits[i] > max) max = logits[i];
    double sum_exp = 0.0;
    for (int32_t i = 0; i < n; i++) sum_exp += exp((double)(logits[i] - max));
    if (sum_exp <= 0.0 || sum_exp != sum_exp) return 0.0f;
    return (float)(exp((double)(logits[idx] - max)) / sum_exp);
}

/* MtpDecoder.cs:562-577 */
int32_t oracle_mtp_accept_draft(int32_t draft, int32_t target, const float* logits, int32_t n,
                                float p_min, float* draft_prob)
{
    if (draft == target) { *draft_prob = 0.0f; return 1; }
    if (p_min >= 1.0f) { *draft_prob = 0.0f; return 0; }
    *draft_prob = oracle_softmax_prob_at(logits, n, draft);
    return *draft_prob >= p_min;
}

float oracle_seq_sum(const float* x, int64_t n, float s0, float target, int64_t* first_reach)
{
    float s = s0;
    int64_t at = -1;
    for (int64_t i = 0; i < n; i++) {
        s += x[i];
        if (at < 0 && s >= target) at = i;
    }
    if (first_reach) *first_reach = at;
    return s;
}

/* ContinuousBatchingEngine.cs:609-650: rows in order, Filter(row) then Greedy|Sample. */
void oracle_sample_batch(const float* logits, int64_t row_stride, int32_t rows, int32_t n,
                         const oracle_params* params, const uint32_t* allow_mask,
                         int64_t mask_stride_words, const uint8_t* mask_active,
                         const double* uniforms, float* scratch, int32_t* out_tokens)
{
    for (int32_t r = 0; r < rows; r++) {
        const float* row = logits + (int64_t)r * row_stride;
        if (allow_mask && (!mask_active || mask_active[r])) {
            oracle_apply_allow_mask(row, allow_mask + (int64_t)r * mask_stride_words, n, scratch);
            row = scratch;
        }
        oracle_rng rng;
        oracle_rng_replay(&rng, uniforms + r, 1);
        out_tokens[r] = oracle_sample(row, n, &params[r], &rng);
    }
}
