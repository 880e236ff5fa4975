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

// ---- the seam in the engine -----------------------------------------------------------------------------------------
// The batched sampling sibling of IBatchedForwardPass.BatchForwardMultiArgmax
// (src/OpenTail.Stingray.Engine/IBatchedForwardPass.cs:105-117) and the gate that uses it where the batcher loop
// gathers its rows (src/OpenTail.Stingray.Engine/ContinuousBatchingEngine.cs:580-650); the C++ twins of
// managed/RocmBatchSampler.cs and managed/EngineSeam.cs.

// A sequence's Random as the gate needs it: the next values can be looked at before it is known how many the sampler
// consumes (SampleTopK on a row without a finite logit falls back to Greedy and draws nothing, Sampler.cs:251-255).
// Values looked at and not consumed are handed out again, in order.
class PeekableRandom : public Random {
public:
    explicit PeekableRandom(Random* inner) : inner_(inner) {}
    double Peek(std::size_t i = 0)
    {
        while (pending_.size() <= i) pending_.push_back(inner_->NextDouble());
        return pending_[i];
    }
    void Commit(std::size_t n = 1)
    {
        pending_.erase(pending_.begin(), pending_.begin() + (std::ptrdiff_t)n);
        draws += n;
    }
    double NextDouble() override
    {
        const double v = Peek();
        Commit();
        return v;
    }
    std::size_t draws = 0;  // values consumed

private:
    Random* inner_;
    std::vector<double> pending_;
};

// What one decode step hands over per row (ContinuousBatchingEngine.cs:609-650)
struct BatchedSamplingInputs {
    std::vector<const SamplingParams*> Params;          // seq.Sp (PreviousTokens ignored: Histories is used)
    std::vector<const std::vector<int>*> Histories;     // seq.RecentTokens, nullptr without a history penalty (:1280)
    std::vector<int32_t> MaskIds;                       // registered mask of the constraint's state, -1 none / dead state
    std::vector<double> Uniforms;                       // one NextDouble() per row with Temperature > 0, else 0
    std::vector<int32_t> PreviousTokens;                // the token sampled in the previous step, -1 for rows without history; empty = none
};

class BatchSampler {
public:
    explicit BatchSampler(int device = 0, void* hip_stream = nullptr, bool use_stream = false)
    {
        int rc = sr_create(device, &ctx_);
        if (rc != SR_OK) throw SamplerError(rc, rc == SR_ERR_NO_DEVICE ? "no HIP device: use the managed sampler" : "sr_create failed");
        if (use_stream) Check(sr_set_stream(ctx_, hip_stream), "sr_set_stream");
        Check(sr_batch_create(ctx_, &batch_), "sr_batch_create");
    }
    ~BatchSampler()
    {
        if (batch_) sr_batch_destroy(batch_);
        sr_destroy(ctx_);
    }
    BatchSampler(const BatchSampler&) = delete;
    BatchSampler& operator=(const BatchSampler&) = delete;

    void BindToCurrentThread() { Check(sr_bind_thread(ctx_), "sr_bind_thread"); }
    int RegisterMask(const uint32_t* words, int vocab)
    {
        int32_t id = -1;
        Check(sr_mask_register(ctx_, words, 0, vocab, &id), "sr_mask_register");
        return id;
    }
    void ReleaseMask(int id) { Check(sr_mask_release(ctx_, id), "sr_mask_release"); }
    int MaskAnd(const std::vector<int32_t>& ids)
    {
        int32_t id = -1;
        Check(sr_mask_and(ctx_, ids.data(), (int32_t)ids.size(), &id), "sr_mask_and");
        return id;
    }
    // a decode step did not go through Sample: the next one uploads, whatever the caller says about its rows
    void InvalidateHistory() { history_valid_ = false; }
    void Synchronize() { Check(sr_synchronize(ctx_), "sr_synchronize"); }

    // One step: enqueues the sampling of `rows` rows of device logits into tokens_dev (and flags_dev, may be null).
    // First step, changed rows, an invalidated history: pack and upload; else append the previous tokens, the mask ids
    // and the uniforms.  Nothing here waits for the device.
    void Sample(const void* logits_dev, int dtype, int rows, int vocab, int64_t row_stride, int32_t* tokens_dev, uint32_t* flags_dev,
                const BatchedSamplingInputs& in, bool same_rows_as_last_step)
    {
        if ((int)in.Params.size() != rows || (int)in.Histories.size() != rows || (int)in.MaskIds.size() != rows ||
            (int)in.Uniforms.size() != rows)
            throw ArgumentException("one entry per row");
        if (same_rows_as_last_step && history_valid_ && rows == rows_ && vocab == vocab_ && (int)in.PreviousTokens.size() == rows) {
            Check(sr_batch_append_tokens_masks(batch_, in.PreviousTokens.data(), in.Uniforms.data(), in.MaskIds.data()),
                  "sr_batch_append_tokens_masks");
            appends++;
        } else {
            std::vector<sr_row_params> rp((std::size_t)rows);
            std::vector<int32_t> hist, hoff((std::size_t)rows + 1, 0), bids, boff((std::size_t)rows + 1, 0);
            std::vector<float> bvals;
            for (int r = 0; r < rows; r++) {
                const SamplingParams& p = *in.Params[(std::size_t)r];
                sr_row_params& d = rp[(std::size_t)r];
                d.temperature = p.Temperature; d.top_k = p.TopK; d.top_p = p.TopP; d.min_p = p.MinP;
                d.repetition_penalty = p.RepetitionPenalty; d.repeat_last_n = p.RepeatLastN;
                d.presence_penalty = p.PresencePenalty; d.frequency_penalty = p.FrequencyPenalty;
                d.spec_draft_p_min = p.SpecDraftPMin;
                d.flags = p.LogitBias.empty() ? 0u : (uint32_t)SR_ROW_HAS_LOGIT_BIAS;
                if (in.Histories[(std::size_t)r]) hist.insert(hist.end(), in.Histories[(std::size_t)r]->begin(), in.Histories[(std::size_t)r]->end());
                hoff[(std::size_t)r + 1] = (int32_t)hist.size();
                for (const auto& kv : p.LogitBias) { bids.push_back(kv.first); bvals.push_back(kv.second); }
                boff[(std::size_t)r + 1] = (int32_t)bids.size();
            }
            Check(sr_batch_upload_mask_ids(batch_, rows, vocab, rp.data(), hist.empty() ? nullptr : hist.data(), hoff.data(),
                                           bids.empty() ? nullptr : bids.data(), bvals.empty() ? nullptr : bvals.data(),
                                           bids.empty() ? nullptr : boff.data(), in.MaskIds.data(), in.Uniforms.data(), 1),
                  "sr_batch_upload_mask_ids");
            rows_ = rows;
            vocab_ = vocab;
            uploads++;
        }
        Check(sr_sample_launch(ctx_, batch_, logits_dev, dtype, row_stride, tokens_dev, flags_dev), "sr_sample_launch");
        history_valid_ = true;
    }

    int uploads = 0, appends = 0;

private:
    void Check(int rc, const char* what)
    {
        if (rc == SR_OK) return;
        const std::string msg = std::string(what) + ": " + sr_last_error(ctx_);
        if (rc == SR_ERR_NULL_ARGUMENT) throw ArgumentNullException(msg);
        if (rc == SR_ERR_INVALID_ARGUMENT) throw ArgumentException(msg);
        throw SamplerError(rc, msg);
    }
    sr_ctx* ctx_ = nullptr;
    sr_batch* batch_ = nullptr;
    int rows_ = -1, vocab_ = -1;
    bool history_valid_ = false;
};

// The gate (ContinuousBatchingEngine.cs:580-606).  Seq needs: Sp (SamplingParams), RecentTokens (std::vector<int>* or
// nullptr), Rng (PeekableRandom*), ForcedClose (bool), MaskId (int: the registered mask of its constraint's state, -1
// none), Id (int).  Fwd needs: bool SupportsBatchedGpuSampling(); void InvalidateSamplingState();
// void BatchForwardMultiSample(tokens, inputs, same_rows, out_tokens, out_flags) -- the forward step, the launch and
// the rows x 8-byte download.
struct DeviceSamplingGate {
    std::vector<int> last_ids;
    long last_step = -2;

    // false: the step must take the full-logits path; nothing was consumed (no uniform drawn)
    template <class Fwd, class Seq>
    bool TrySample(Fwd& fwd, std::vector<Seq>& active, const std::vector<int>& tokens, long step_no, std::vector<int>& out_tokens)
    {
        if (!fwd.SupportsBatchedGpuSampling()) return false;
        for (const Seq& s : active)            // first pass: decisions only
            if (s.ForcedClose) { fwd.InvalidateSamplingState(); return false; }
        BatchedSamplingInputs in;
        std::vector<int> ids;
        for (Seq& s : active) {                // the step is committed to the device: look at one uniform per sampled row
            in.Params.push_back(&s.Sp);
            in.Histories.push_back(s.RecentTokens);
            in.MaskIds.push_back(s.MaskId);
            in.Uniforms.push_back(s.Sp.Temperature > 0.0f ? s.Rng->Peek() : 0.0);
            ids.push_back(s.Id);
        }
        const bool same_rows = ids == last_ids && step_no == last_step + 1;
        if (same_rows)
            for (std::size_t i = 0; i < active.size(); i++) in.PreviousTokens.push_back(active[i].RecentTokens ? tokens[i] : -1);
        std::vector<uint32_t> flags;
        fwd.BatchForwardMultiSample(tokens, in, same_rows, out_tokens, flags);
        for (std::size_t i = 0; i < active.size(); i++)
            if (active[i].Sp.Temperature > 0.0f && !((flags[i] & SR_OUT_DEGENERATE) && (flags[i] & SR_OUT_PATH_TOPK_FAST)))
                active[i].Rng->Commit();
        last_ids = ids;
        last_step = step_no;
        return true;
    }
};

}  // namespace Rocm
}  // namespace Stingray
}  // namespace OpenTail

#endif  // STINGRAY_SAMPLER_HPP
