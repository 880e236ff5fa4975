/*
 * CPU oracle for the token-sampling / constrained-decoding / speculative-verification path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a plain-C restatement of the reference's
 * managed sampler, function by function, and exists only so that tests, the smoke check and the
 * bench's CPU-baseline leg have something to compare the HIP path against.  Nothing in the shipped
 * library links, loads or calls it.
 *
 * Every function cites the reference lines it follows (paths relative to the reference tree,
 * src/OpenTail.Stingray.Engine/ unless stated).
 *
 * Arithmetic the reference delegates to code that is not in its tree, and how it is fixed here:
 *   - MathF.Exp  -> oracle_expf(): the published glibc >= 2.27 / ARM optimized-routines expf
 *                   (32-entry 2^(i/32) table, cubic in double, one rounding to float) with the
 *                   FMA contractions the x86-64 "-mfma" build of glibc performs.  Pinned: equal,
 *                   bit for bit, to this image's libm expf on every float in [-inf, 89).
 *   - MathF.Pow  -> host libm powf (called directly).
 *   - TensorPrimitives.Max / Multiply / IndexOfMax: value-exact specifications (IEEE max with NaN
 *                   propagation; element-wise product; first index of the maximum).
 *   - TensorPrimitives.Sum: PARITY UNPINNED at the bit level (lane order depends on the host's
 *                   vector width and, in newer runtimes, on buffer alignment).  Fixed here BY
 *                   DEFINITION as the 256-bit shape: 8 strided lane accumulators seeded with the
 *                   first vector, the ragged tail added through an overlapped last vector whose
 *                   already-consumed lanes are zeroed, then ((l0+l1)+(l2+l3))+((l4+l5)+(l6+l7));
 *                   4 <= n < 8 uses the same scheme with 4 lanes; n < 4 is a scalar loop.
 *   - MemoryExtensions.Sort with a comparison (top-p): PARITY UNPINNED for the order of equal
 *                   probabilities (introsort is unstable).  Fixed here by definition: equal
 *                   probabilities keep ascending index order.
 *   - System.Random(seed): the Knuth subtractive generator of the runtime's seeded compat
 *                   implementation, restated from its public source (oracle_dotnet_random_*).
 */
#ifndef STINGRAY_ORACLE_H
#define STINGRAY_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* SamplingParams (Sampler.cs:648-813), the fields the sampler reads. */
typedef struct oracle_params {
    float temperature;          /* 1.0  */
    int32_t top_k;              /* 0 = off */
    float top_p;                /* 1.0 = off; active iff 0 < p < 1 */
    float min_p;                /* 0 = off */
    float repetition_penalty;   /* 1.0 = off */
    int32_t repeat_last_n;      /* 64; <= 0 or >= count means whole history (Sampler.cs:364-365) */
    float presence_penalty;
    float frequency_penalty;
    const int32_t* prev;        /* PreviousTokens, ordered, duplicates meaningful; may be NULL */
    int32_t n_prev;
    const int32_t* bias_ids;    /* LogitBias entries; n_bias > 0 selects the slow path even when */
    const float* bias_vals;     /*   every id is out of range (SamplerTests.cs:215-216)           */
    int32_t n_bias;
    float spec_draft_p_min;     /* 1.0 */
    int32_t draft_from_lookup;  /* the step's draft tokens came from prompt lookup: no draft distributions exist
                                   (usedPld, SpeculativeDecoder.cs:488-501, 538, 549) */
} oracle_params;

void oracle_params_default(oracle_params* p);

/* Source of NextDouble() values: either a replayed array or a seeded .NET-compatible generator. */
typedef struct oracle_rng {
    const double* replay;       /* when non-NULL, values are taken from here in order */
    int64_t replay_len;
    int64_t pos;                /* number of draws taken so far (both modes) */
    int32_t seed_array[56];     /* Knuth subtractive state */
    int32_t inext, inextp;
} oracle_rng;

void oracle_rng_replay(oracle_rng* r, const double* values, int64_t n);
void oracle_dotnet_random_init(oracle_rng* r, int32_t seed);
int32_t oracle_dotnet_random_next(oracle_rng* r);        /* Random.Next()       */
double oracle_rng_next_double(oracle_rng* r);            /* Random.NextDouble() */

float oracle_expf(float x);

/* TensorPrimitives restatements. */
float oracle_tp_max(const float* x, int32_t n);
float oracle_tp_sum(const float* x, int32_t n);
int32_t oracle_tp_index_of_max(const float* x, int32_t n);

/* Sampler.cs */
int32_t oracle_greedy(const float* logits, int32_t n);                                   /* :442-446 */
int32_t oracle_sample(const float* logits, int32_t n, const oracle_params* p, oracle_rng* rng); /* :17-102 */
int32_t oracle_build_filtered_distribution(const float* logits, int32_t n, const oracle_params* p,
                                           float* probs, int32_t n_probs);               /* :118-163; -1 on length mismatch */
int32_t oracle_sample_with_distribution(const float* logits, int32_t n, const oracle_params* p,
                                        float* probs, oracle_rng* rng);                  /* :172-187 */
int32_t oracle_sample_from_probs(const float* probs, int32_t n, oracle_rng* rng);         /* :195-199 */
int32_t oracle_resample_residual(const float* p, int32_t np, const float* q, int32_t nq,
                                 oracle_rng* rng);                                        /* :587-618; -1 on mismatch */

/* Grammar mask application (Core/Grammar/ITokenConstraint.cs:31-42): out[i] = bit i ? in[i] : -inf. */
void oracle_apply_allow_mask(const float* logits, const uint32_t* mask_words, int32_t n, float* out);

/*
 * SpeculativeDecoder.StepSampled accept loop (SpeculativeDecoder.cs:530-559) for one row.
 *   target_logits : [(n_draft + 1) x n]  row i verifies draft i, the last row is the bonus position
 *   draft_probs   : [n_draft x n]        q_i, the draft proposal distributions
 *   draft_tokens  : [n_draft]
 * Writes accepted drafts followed by the correction / bonus token into out_tokens[n_draft + 1];
 * returns the number of accepted drafts.  scratch must hold n floats.
 */
int32_t oracle_spec_verify_row(const float* target_logits, const float* draft_probs,
                               const int32_t* draft_tokens, int32_t n_draft, int32_t n,
                               const oracle_params* p, oracle_rng* rng, float* scratch,
                               int32_t* out_tokens);

/* MtpDecoder.cs:562-596 */
float oracle_softmax_prob_at(const float* logits, int32_t n, int32_t idx);
int32_t oracle_mtp_accept_draft(int32_t draft, int32_t target, const float* logits, int32_t n,
                                float p_min, float* draft_prob);

/* Plain left-to-right fp32 running sum of x[0..n) starting from s0, as the reference's scalar loops do
 * (e.g. Sampler.cs:460-465).  When first_reach is non-NULL it receives the first index at which the running
 * sum is >= target (-1 if never).  Used to pin the GPU's parallel evaluation of such sums. */
float oracle_seq_sum(const float* x, int64_t n, float s0, float target, int64_t* first_reach);

/* Row loops used by tests and by the bench's CPU-baseline leg (one thread, rows in order, as the
 * reference's batcher does at ContinuousBatchingEngine.cs:609-650). */
void oracle_sample_batch(const float* logits, int64_t row_stride, int32_t rows, int32_t n,
                         const oracle_params* params, const uint32_t* allow_mask,
                         int64_t mask_stride_words, const uint8_t* mask_active,
                         const double* uniforms, float* scratch, int32_t* out_tokens);

#ifdef __cplusplus
}
#endif
#endif
