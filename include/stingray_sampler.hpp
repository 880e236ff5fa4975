// stingray_sampler.hpp -- the reference's sampler interface over the C ABI of stingray_sampler.h.
//
// Header-only C++17; needs nothing but the C ABI library.  Names, argument meaning and error behaviour
// follow the managed static class (src/OpenTail.Stingray.Engine/Sampler.cs of the reference):
//   Sampler.Greedy                       :442-446      Sampler::Greedy
//   Sampler.Sample                       :17-102       Sampler::Sample
//   Sampler.BuildFilteredDistribution    :118-163      Sampler::BuildFilteredDistribution
//   Sampler.SampleWithDistribution       :172-187      Sampler::SampleWithDistribution
//   Sampler.SampleFromProbs              :195-199      Sampler::SampleFromProbs
//   Sampler.ResampleResidual             :587-618      Sampler::ResampleResidual
//   SamplingParams                       :648-813      SamplingParams (the fields the sampler reads)
// A Random is anything with NextDouble(); draws are taken from it exactly when the managed sampler would
// (none for Temperature <= 0).  ArgumentException / ArgumentNullException map the managed exceptions of the
// same names; every other failure is a SamplerError carrying the library's message.
#ifndef STINGRAY_SAMPLER_HPP
#define STINGRAY_SAMPLER_HPP

#include <cstddef>
#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "stingray_sampler.h"

namespace OpenTail {
namespace Stingray {
namespace Rocm {

struct ArgumentException : std::invalid_argument {
    using std::invalid_argument::invalid_argument;
};
struct ArgumentNullException : ArgumentException {
    using ArgumentException::ArgumentException;
};
struct SamplerError : std::runtime_error {
    int code;
    SamplerError(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};

// System.Random's one method the sampler uses
struct Random {
    virtual double NextDouble() = 0;
    virtual ~Random() = default;
};

struct SamplingParams {
    float Temperature = 1.0f;
    int TopK = 0;
    float TopP = 1.0f;
    float MinP = 0.0f;
    float RepetitionPenalty = 1.0f;
    int RepeatLastN = 64;
    float PresencePenalty = 0.0f;
    float FrequencyPenalty = 0.0f;
    std::map<int, float> LogitBias;
    std::vector<int> PreviousTokens;
    float SpecDraftPMin = 1.0f;
    // not a field of the managed class: the step's `usedPld` (SpeculativeDecoder.cs:488-501), read beside the
    // parameters by the accept loop (:538, :549)
    bool SpecDraftFromLookup = false;

    bool HasHistoryPenalty() const
    {
        return RepetitionPenalty != 1.0f || PresencePenalty != 0.0f || FrequencyPenalty != 0.0f;
    }
};

class Sampler {
public:
    explicit Sampler(int device = 0)
    {
        const int rc = sr_create(device, &ctx_);
        if (rc != SR_OK) throw SamplerError(rc, rc == SR_ERR_NO_DEVICE ? "no HIP device: use the managed sampler" : "sr_create failed");
    }
    ~Sampler() { sr_destroy(ctx_); }
    Sampler(const Sampler&) = delete;
    Sampler& operator=(const Sampler&) = delete;

    int Greedy(const float* logits, std::size_t n)
    {
        if (n == 0) return 0;
        int32_t idx = 0;
        Check(sr_argmax_rows(ctx_, logits, SR_DTYPE_F32, 0, 1, (int32_t)n, (int64_t)n, &idx, nullptr));
        return idx;
    }

    int Sample(const float* logits, std::size_t n, const SamplingParams& p, Random* rng = nullptr)
    {
        Packed k(p);
        double u = 0.0;
        const bool greedy = p.Temperature <= 0.0f;
        if (!greedy) {
            if (!rng) throw ArgumentNullException("rng");
            u = rng->NextDouble();
        }
        int32_t tok = -1;
        Check(sr_sample_batch(ctx_, logits, SR_DTYPE_F32, 0, 1, (int32_t)n, (int64_t)n, &k.row, k.hist(), k.hist_off,
                              k.bias_ids(), k.bias_vals(), k.bias_off, nullptr, 0, nullptr, greedy ? nullptr : &u, &tok, nullptr));
        return tok;
    }

    // rows x vocab logits, one SamplingParams and one uniform per row (uniforms of greedy rows are ignored)
    std::vector<int> SampleBatch(const float* logits, std::size_t rows, std::size_t vocab, const std::vector<SamplingParams>& params,
                                 const std::vector<double>& uniforms)
    {
        if (params.size() != rows || uniforms.size() != rows) throw ArgumentException("one SamplingParams and one uniform per row");
        std::vector<sr_row_params> rp(rows);
        std::vector<int32_t> hist, hoff(rows + 1, 0), bids, boff(rows + 1, 0);
        std::vector<float> bvals;
        for (std::size_t r = 0; r < rows; r++) {
            Packed k(params[r]);
            rp[r] = k.row;
            hist.insert(hist.end(), k.h.begin(), k.h.end());
            bids.insert(bids.end(), k.bi.begin(), k.bi.end());
            bvals.insert(bvals.end(), k.bv.begin(), k.bv.end());
            hoff[r + 1] = (int32_t)hist.size();
            boff[r + 1] = (int32_t)bids.size();
        }
        std::vector<int32_t> out(rows, -1);
        Check(sr_sample_batch(ctx_, logits, SR_DTYPE_F32, 0, (int32_t)rows, (int32_t)vocab, (int64_t)vocab, rp.data(),
                              hist.empty() ? nullptr : hist.data(), hoff.data(), bids.empty() ? nullptr : bids.data(),
                              bvals.empty() ? nullptr : bvals.data(), boff.data(), nullptr, 0, nullptr, uniforms.data(),
                              out.data(), nullptr));
        return std::vector<int>(out.begin(), out.end());
    }

    void BuildFilteredDistribution(const float* logits, std::size_t n, const SamplingParams& p, float* probs, std::size_t probs_len)
    {
        Packed k(p);
        Check(sr_build_distribution(ctx_, logits, 1, (int32_t)n, (int64_t)n, &k.row, k.hist(), k.hist_off, k.bias_ids(),
                                    k.bias_vals(), k.bias_off, probs, (int64_t)(probs_len > n ? probs_len : n), (int32_t)probs_len));
    }

    int SampleWithDistribution(const float* logits, std::size_t n, const SamplingParams& p, float* probs, std::size_t probs_len,
                               Random* rng = nullptr)
    {
        Packed k(p);
        double u = 0.0;
        if (p.Temperature > 0.0f) {
            if (probs_len != n)  // the managed method validates before it draws (Sampler.cs:121-123)
                throw ArgumentException("probs length (" + std::to_string(probs_len) + ") must equal logits length (" +
                                        std::to_string(n) + ").");
            if (!rng) throw ArgumentNullException("rng");
            u = rng->NextDouble();
        }
        int32_t tok = -1;
        Check(sr_sample_with_distribution(ctx_, logits, 1, (int32_t)n, (int64_t)n, &k.row, k.hist(), k.hist_off, k.bias_ids(),
                                          k.bias_vals(), k.bias_off, &u, probs, (int64_t)(probs_len > n ? probs_len : n),
                                          (int32_t)probs_len, &tok));
        return tok;
    }

    int SampleFromProbs(const float* probs, std::size_t n, Random* rng)
    {
        if (!rng) throw ArgumentNullException("rng");
        const double u = rng->NextDouble();
        int32_t tok = -1;
        Check(sr_sample_from_probs(ctx_, probs, 1, (int32_t)n, (int64_t)n, &u, &tok));
        return tok;
    }

    int ResampleResidual(const float* p, std::size_t np, const float* q, std::size_t nq, Random* rng)
    {
        if (!rng) throw ArgumentNullException("rng");
        if (np != nq)
            throw ArgumentException("p and q must have equal length (" + std::to_string(np) + " vs " + std::to_string(nq) + ").");
        const double u = rng->NextDouble();
        int32_t tok = -1;
        Check(sr_resample_residual(ctx_, p, (int32_t)np, (int64_t)np, q, (int32_t)nq, (int64_t)nq, 1, &u, &tok));
        return tok;
    }

    sr_ctx* Handle() const { return ctx_; }

private:
    // one row's side inputs in the C ABI's shape
    struct Packed {
        sr_row_params row{};
        std::vector<int32_t> h, bi;
        std::vector<float> bv;
        int32_t hist_off[2] = {0, 0}, bias_off[2] = {0, 0};
        explicit Packed(const SamplingParams& p)
        {
            row.temperature = p.Temperature;
            row.top_k = p.TopK;
            row.top_p = p.TopP;
            row.min_p = p.MinP;
            row.repetition_penalty = p.RepetitionPenalty;
            row.repeat_last_n = p.RepeatLastN;
            row.presence_penalty = p.PresencePenalty;
            row.frequency_penalty = p.FrequencyPenalty;
            row.spec_draft_p_min = p.SpecDraftPMin;
            row.flags = (p.LogitBias.empty() ? 0u : (uint32_t)SR_ROW_HAS_LOGIT_BIAS) |
                        (p.SpecDraftFromLookup ? (uint32_t)SR_ROW_DRAFT_FROM_LOOKUP : 0u);
            h.assign(p.PreviousTokens.begin(), p.PreviousTokens.end());
            for (const auto& kv : p.LogitBias) { bi.push_back(kv.first); bv.push_back(kv.second); }
            hist_off[1] = (int32_t)h.size();
            bias_off[1] = (int32_t)bi.size();
        }
        const int32_t* hist() const { return h.empty() ? nullptr : h.data(); }
        const int32_t* bias_ids() const { return bi.empty() ? nullptr : bi.data(); }
        const float* bias_vals() const { return bv.empty() ? nullptr : bv.data(); }
    };

    void Check(int rc)
    {
        if (rc == SR_OK) return;
        const std::string msg = sr_last_error(ctx_);
        if (rc == SR_ERR_NULL_ARGUMENT) throw ArgumentNullException(msg);
        if (rc == SR_ERR_INVALID_ARGUMENT) throw ArgumentException(msg);
        throw SamplerError(rc, msg);
    }

    sr_ctx* ctx_ = nullptr;
};

}  // namespace Rocm
}  // namespace Stingray
}  // namespace OpenTail

#endif  // STINGRAY_SAMPLER_HPP
