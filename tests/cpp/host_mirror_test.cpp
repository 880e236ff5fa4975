// The C++ host mirror (include/stingray_sampler.hpp) against the CPU oracle, through the C ABI.
// Written after the reference's SamplerTests.cs: the same calls, on the GPU, must give the oracle's answers.
// Prints one line per group and "OK <checks>" at the end; exit status 0 only if every check passed.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <limits>
#include <random>

#include "stingray_oracle.h"
#include "stingray_sampler.hpp"

using namespace OpenTail::Stingray::Rocm;

namespace {

int g_checks = 0, g_failed = 0;
#define CHECK(cond, ...)                                  \
    do {                                                  \
        g_checks++;                                       \
        if (!(cond)) {                                    \
            g_failed++;                                   \
            std::printf("FAILED %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                     \
            std::printf("\n");                            \
        }                                                 \
    } while (0)

struct Replay : Random {
    std::vector<double> v;
    size_t pos = 0;
    explicit Replay(std::vector<double> x) : v(std::move(x)) {}
    double NextDouble() override { return v.at(pos++); }
};

struct OracleParams {
    oracle_params p;
    std::vector<int32_t> bi;
    std::vector<float> bv;
    explicit OracleParams(const SamplingParams& s)
    {
        oracle_params_default(&p);
        p.temperature = s.Temperature; p.top_k = s.TopK; p.top_p = s.TopP; p.min_p = s.MinP;
        p.repetition_penalty = s.RepetitionPenalty; p.repeat_last_n = s.RepeatLastN;
        p.presence_penalty = s.PresencePenalty; p.frequency_penalty = s.FrequencyPenalty;
        p.spec_draft_p_min = s.SpecDraftPMin;
        p.prev = s.PreviousTokens.empty() ? nullptr : s.PreviousTokens.data();
        p.n_prev = (int32_t)s.PreviousTokens.size();
        for (const auto& kv : s.LogitBias) { bi.push_back(kv.first); bv.push_back(kv.second); }
        p.bias_ids = bi.empty() ? nullptr : bi.data();
        p.bias_vals = bv.empty() ? nullptr : bv.data();
        p.n_bias = (int32_t)bi.size();
    }
};

std::vector<float> make_logits(std::mt19937& g, size_t n, float sigma)
{
    std::normal_distribution<float> d(0.0f, sigma);
    std::vector<float> x(n);
    for (auto& v : x) v = d(g);
    for (int i = 0; i < 20 && (size_t)i < n; i++) x[(size_t)(g() % n)] += 12.0f / std::pow((float)(i + 1), 1.1f);
    return x;
}

}  // namespace

int main()
{
    Sampler gpu(0);
    std::mt19937 g(1234);
    std::uniform_real_distribution<double> U(0.0, 1.0);

    // SamplerTests.cs known answers
    {
        const float a[] = {1, 5, 3, 2}, b[] = {10, 1, 2, 3}, c[] = {1, 2, 3, 100};
        CHECK(gpu.Greedy(a, 4) == 1 && gpu.Greedy(b, 4) == 0 && gpu.Greedy(c, 4) == 3, "Greedy known answers");
        CHECK(gpu.Greedy(nullptr, 0) == 0, "Greedy of an empty span");
        SamplingParams greedy;
        greedy.Temperature = 0.0f;
        Replay r({0.3});
        CHECK(gpu.Sample(a, 4, greedy, &r) == 1 && r.pos == 0, "temperature 0 is greedy and draws nothing");
        const float l3[] = {10, 9.8f, 0};
        SamplingParams pres;
        pres.TopK = 1; pres.PresencePenalty = 1.0f; pres.PreviousTokens = {0};
        for (double u : {0.0, 0.4, 0.999999}) {
            Replay rr({u});
            CHECK(gpu.Sample(l3, 3, pres, &rr) == 1, "presence penalty moves the argmax");
        }
    }
    std::printf("known answers done\n");

    // Sample / BuildFilteredDistribution / SampleWithDistribution against the oracle
    for (size_t n : {(size_t)257, (size_t)5000, (size_t)49152}) {
        for (int trial = 0; trial < 12; trial++) {
            std::vector<float> x = make_logits(g, n, 1.5f);
            SamplingParams p;
            p.Temperature = (trial % 6 == 5) ? 0.0f : 0.5f + 0.1f * (float)(trial % 7);
            p.TopK = (trial % 3 == 0) ? 0 : (int)(1 + g() % 300);
            p.TopP = (trial % 2) ? 0.9f : 1.0f;
            p.MinP = (trial % 4 == 3) ? 0.05f : 0.0f;
            if (trial % 3 == 1) { p.RepetitionPenalty = 1.2f; p.PresencePenalty = 0.3f; }
            if (trial % 5 == 2) p.FrequencyPenalty = -0.2f;
            for (int i = 0; i < 40; i++) p.PreviousTokens.push_back((int)(g() % n));
            if (trial % 4 == 2) { p.LogitBias[(int)(g() % n)] = 3.5f; p.LogitBias[(int)(g() % n)] = -100.0f; }
            OracleParams op(p);
            const double u = U(g);
            Replay r({u});
            oracle_rng orng;
            oracle_rng_replay(&orng, &u, 1);
            const int want = oracle_sample(x.data(), (int32_t)n, &op.p, &orng);
            const int got = gpu.Sample(x.data(), n, p, &r);
            CHECK(got == want, "Sample n=%zu trial %d: gpu %d oracle %d", n, trial, got, want);

            std::vector<float> pg(n), po(n);
            gpu.BuildFilteredDistribution(x.data(), n, p, pg.data(), n);
            oracle_build_filtered_distribution(x.data(), (int32_t)n, &op.p, po.data(), (int32_t)n);
            CHECK(std::memcmp(pg.data(), po.data(), n * sizeof(float)) == 0, "BuildFilteredDistribution n=%zu trial %d differs", n, trial);

            Replay r2({u});
            oracle_rng_replay(&orng, &u, 1);
            std::vector<float> pg2(n), po2(n);
            const int t_want = oracle_sample_with_distribution(x.data(), (int32_t)n, &op.p, po2.data(), &orng);
            const int t_got = gpu.SampleWithDistribution(x.data(), n, p, pg2.data(), n, &r2);
            CHECK(t_got == t_want && std::memcmp(pg2.data(), po2.data(), n * sizeof(float)) == 0,
                  "SampleWithDistribution n=%zu trial %d: gpu %d oracle %d", n, trial, t_got, t_want);

            // SampleFromProbs / ResampleResidual on those distributions
            const double u2 = U(g);
            Replay r3({u2});
            oracle_rng_replay(&orng, &u2, 1);
            CHECK(gpu.SampleFromProbs(po.data(), n, &r3) == oracle_sample_from_probs(po.data(), (int32_t)n, &orng),
                  "SampleFromProbs n=%zu trial %d", n, trial);
            std::vector<float> q(n);
            {
                SamplingParams qp;  // a flatter proposal
                qp.Temperature = 1.3f;
                OracleParams oq(qp);
                std::vector<float> y = x;
                for (auto& v : y) v += 0.5f * (float)std::sin((double)(&v - y.data()));
                oracle_build_filtered_distribution(y.data(), (int32_t)n, &oq.p, q.data(), (int32_t)n);
            }
            Replay r4({u2});
            oracle_rng_replay(&orng, &u2, 1);
            CHECK(gpu.ResampleResidual(po.data(), n, q.data(), n, &r4) ==
                      oracle_resample_residual(po.data(), (int32_t)n, q.data(), (int32_t)n, &orng),
                  "ResampleResidual n=%zu trial %d", n, trial);
        }
    }
    std::printf("oracle comparisons done\n");

    // batched rows
    {
        const size_t rows = 9, n = 30011;
        std::vector<float> x;
        std::vector<SamplingParams> ps(rows);
        std::vector<double> us(rows);
        for (size_t r = 0; r < rows; r++) {
            auto row = make_logits(g, n, 2.0f);
            x.insert(x.end(), row.begin(), row.end());
            ps[r].Temperature = r == 4 ? 0.0f : 0.8f;
            ps[r].TopK = (int)(1 + 37 * r);
            ps[r].TopP = 0.95f;
            if (r % 2) { ps[r].RepetitionPenalty = 1.1f; for (int i = 0; i < 64; i++) ps[r].PreviousTokens.push_back((int)(g() % n)); }
            us[r] = U(g);
        }
        const std::vector<int> got = gpu.SampleBatch(x.data(), rows, n, ps, us);
        for (size_t r = 0; r < rows; r++) {
            OracleParams op(ps[r]);
            oracle_rng orng;
            oracle_rng_replay(&orng, &us[r], 1);
            const int want = oracle_sample(x.data() + r * n, (int32_t)n, &op.p, &orng);
            CHECK(got[r] == want, "SampleBatch row %zu: gpu %d oracle %d", r, got[r], want);
        }
    }
    std::printf("batched rows done\n");

    // error behaviour (Sampler.cs:121-123, :197, :589-592)
    {
        std::vector<float> x(100, 0.0f), p(100, 0.01f), q(99, 0.01f), probs(99);
        SamplingParams sp;
        bool threw = false;
        try { gpu.BuildFilteredDistribution(x.data(), 100, sp, probs.data(), 99); } catch (const ArgumentException&) { threw = true; }
        CHECK(threw, "probs length mismatch must throw ArgumentException");
        threw = false;
        try { gpu.SampleFromProbs(p.data(), 100, nullptr); } catch (const ArgumentNullException&) { threw = true; }
        CHECK(threw, "null rng must throw ArgumentNullException");
        threw = false;
        Replay r({0.5});
        try { gpu.ResampleResidual(p.data(), 100, q.data(), 99, &r); } catch (const ArgumentException&) { threw = true; }
        CHECK(threw && r.pos == 0, "p/q length mismatch must throw before drawing");
        threw = false;
        try { gpu.Sample(x.data(), 100, sp, nullptr); } catch (const ArgumentNullException&) { threw = true; }
        CHECK(threw, "a sampled row without rng must throw ArgumentNullException");
    }
    std::printf("error behaviour done\n");

    if (g_failed) {
        std::printf("FAILED %d of %d checks\n", g_failed, g_checks);
        return 1;
    }
    std::printf("OK %d\n", g_checks);
    return 0;
}
