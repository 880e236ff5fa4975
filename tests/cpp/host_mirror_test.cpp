// The C++ host mirror (include/stingray_sampler.hpp) against the CPU oracle, through the C ABI.
// Written after the reference's SamplerTests.cs: the same calls, on the GPU, must give the oracle's answers.
// Prints one line per group and "OK <checks>" at the end; exit status 0 only if every check passed.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <limits>
#include <random>

#include <hip/hip_runtime_api.h>

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

    // The gate of the batcher loop (ContinuousBatchingEngine.cs:580-650) against the loop's own way (full logits on
    // the host, the oracle sampling): a step that is skipped, a forced token in the middle, the draws per sequence.
    {
        const int rows = 3, n = 6007, steps = 16;
        struct Seq {
            SamplingParams Sp;
            std::vector<int> hist;
            std::vector<int>* RecentTokens = nullptr;
            PeekableRandom* Rng = nullptr;
            bool ForcedClose = false;
            int MaskId = -1;
            int Id = 0;
        };
        struct SeededRandom : Random {  // any generator will do: both engines replay the same values
            std::mt19937_64 g;
            std::uniform_real_distribution<double> d{0.0, 1.0};
            explicit SeededRandom(unsigned s) : g(s) {}
            double NextDouble() override { return d(g); }
        };
        struct Fwd {
            BatchSampler* sampler;
            const std::vector<float>* host_rows;
            float* dev = nullptr;
            int32_t* tok = nullptr;
            uint32_t* flg = nullptr;
            int rows, n, sample_calls = 0;
            bool SupportsBatchedGpuSampling() { return true; }
            void InvalidateSamplingState() { sampler->InvalidateHistory(); }
            void BatchForwardMultiSample(const std::vector<int>&, const BatchedSamplingInputs& in, bool same, std::vector<int>& out,
                                         std::vector<uint32_t>& flags)
            {
                sample_calls++;
                (void)hipMemcpy(dev, host_rows->data(), (size_t)rows * n * sizeof(float), hipMemcpyHostToDevice);
                sampler->Sample(dev, SR_DTYPE_F32, rows, n, n, tok, flg, in, same);
                sampler->Synchronize();
                std::vector<int32_t> t((size_t)rows);
                flags.assign((size_t)rows, 0u);
                (void)hipMemcpy(t.data(), tok, (size_t)rows * 4, hipMemcpyDeviceToHost);
                (void)hipMemcpy(flags.data(), flg, (size_t)rows * 4, hipMemcpyDeviceToHost);
                out.assign(t.begin(), t.end());
            }
        };
        BatchSampler bs(0);
        std::vector<float> host_rows((size_t)rows * n);
        Fwd fwd{&bs, &host_rows};
        fwd.rows = rows;
        fwd.n = n;
        (void)hipMalloc((void**)&fwd.dev, (size_t)rows * n * sizeof(float));
        (void)hipMalloc((void**)&fwd.tok, (size_t)rows * 4);
        (void)hipMalloc((void**)&fwd.flg, (size_t)rows * 4);
        std::vector<Seq> dev_seqs((size_t)rows), ref_seqs((size_t)rows);
        std::vector<SeededRandom> dev_src, ref_src;
        std::vector<PeekableRandom> dev_rng, ref_rng;
        for (int r = 0; r < rows; r++) { dev_src.emplace_back(77u + (unsigned)r); ref_src.emplace_back(77u + (unsigned)r); }
        for (int r = 0; r < rows; r++) { dev_rng.emplace_back(&dev_src[(size_t)r]); ref_rng.emplace_back(&ref_src[(size_t)r]); }
        for (int r = 0; r < rows; r++) {
            SamplingParams p;
            if (r == 0) { p.Temperature = 0.8f; p.TopK = 40; p.TopP = 0.95f; p.RepetitionPenalty = 1.15f; p.FrequencyPenalty = 0.3f; }
            if (r == 1) { p.Temperature = 0.7f; p.TopP = 0.9f; p.PresencePenalty = 0.6f; }
            if (r == 2) { p.Temperature = 1.0f; p.TopK = 12; }
            for (auto* v : {&dev_seqs, &ref_seqs}) {
                Seq& q = (*v)[(size_t)r];
                q.Sp = p;
                q.Id = r;
                q.RecentTokens = p.HasHistoryPenalty() ? &q.hist : nullptr;
            }
            dev_seqs[(size_t)r].Rng = &dev_rng[(size_t)r];
            ref_seqs[(size_t)r].Rng = &ref_rng[(size_t)r];
        }
        DeviceSamplingGate gate;
        std::vector<int> cur((size_t)rows, 1);
        int host_steps = 0;
        for (int step = 0; step < steps; step++) {
            for (int r = 0; r < rows; r++) {
                auto row = make_logits(g, (size_t)n, 1.5f);
                if (step == 9 && r == 2) std::fill(row.begin(), row.end(), -std::numeric_limits<float>::infinity());  // draws nothing
                std::copy(row.begin(), row.end(), host_rows.begin() + (size_t)r * n);
            }
            // the reference's way for every row
            std::vector<int> want((size_t)rows);
            for (int r = 0; r < rows; r++) {
                Seq& q = ref_seqs[(size_t)r];
                SamplingParams sp = q.Sp;
                if (q.RecentTokens) sp.PreviousTokens = *q.RecentTokens;
                OracleParams op(sp);
                const double u = q.Rng->Peek();
                oracle_rng orng;
                oracle_rng_replay(&orng, &u, 1);
                want[(size_t)r] = (step == 5 && r == 1) ? 90 : oracle_sample(host_rows.data() + (size_t)r * n, n, &op.p, &orng);
                if (!(step == 5 && r == 1) && orng.pos > 0) q.Rng->Commit();
            }
            // the device engine: step 5 has a forced token in the middle row, step 11 is skipped by the engine (sampled on the host)
            dev_seqs[1].ForcedClose = step == 5;
            std::vector<int> got;
            const size_t draws_before = dev_rng[0].draws + dev_rng[1].draws + dev_rng[2].draws;
            const bool on_device = step != 11 && gate.TrySample(fwd, dev_seqs, cur, step, got);
            if (!on_device) {
                host_steps++;
                if (step == 5) CHECK(dev_rng[0].draws + dev_rng[1].draws + dev_rng[2].draws == draws_before, "the refused step consumed a uniform");
                if (step == 11) bs.InvalidateHistory();
                got.assign((size_t)rows, 0);
                for (int r = 0; r < rows; r++) {
                    Seq& q = dev_seqs[(size_t)r];
                    if (q.ForcedClose) { got[(size_t)r] = 90; continue; }
                    SamplingParams sp = q.Sp;
                    if (q.RecentTokens) sp.PreviousTokens = *q.RecentTokens;
                    OracleParams op(sp);
                    const double u = q.Rng->Peek();
                    oracle_rng orng;
                    oracle_rng_replay(&orng, &u, 1);
                    got[(size_t)r] = oracle_sample(host_rows.data() + (size_t)r * n, n, &op.p, &orng);
                    if (orng.pos > 0) q.Rng->Commit();
                }
            }
            for (int r = 0; r < rows; r++) {
                CHECK(got[(size_t)r] == want[(size_t)r], "gate step %d row %d: device engine %d, reference %d", step, r, got[(size_t)r], want[(size_t)r]);
                if (dev_seqs[(size_t)r].RecentTokens) dev_seqs[(size_t)r].hist.push_back(want[(size_t)r]);
                if (ref_seqs[(size_t)r].RecentTokens) ref_seqs[(size_t)r].hist.push_back(want[(size_t)r]);
                cur[(size_t)r] = want[(size_t)r];
            }
        }
        for (int r = 0; r < rows; r++)
            CHECK(dev_rng[(size_t)r].draws == ref_rng[(size_t)r].draws, "row %d drew %zu values, the reference %zu", r, dev_rng[(size_t)r].draws,
                  ref_rng[(size_t)r].draws);
        CHECK(ref_rng[2].draws == (size_t)steps - 1, "the row without a finite logit must not draw");
        CHECK(host_steps == 2 && fwd.sample_calls == steps - 2, "two steps on the host, the others on the device");
        CHECK(bs.uploads == 3 && bs.appends == steps - 2 - 3, "uploads %d appends %d: the first step and the step after each host step upload", bs.uploads, bs.appends);
        (void)hipFree(fwd.dev);
        (void)hipFree(fwd.tok);
        (void)hipFree(fwd.flg);
    }
    std::printf("engine gate done\n");

    if (g_failed) {
        std::printf("FAILED %d of %d checks\n", g_failed, g_checks);
        return 1;
    }
    std::printf("OK %d\n", g_checks);
    return 0;
}
