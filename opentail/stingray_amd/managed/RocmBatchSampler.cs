// The batched device sampler the engine talks to: one instance per engine, kept across decode steps.
// Goes to src/OpenTail.Stingray.Rocm/RocmBatchSampler.cs.  It stands where the per-row
// `Sampler.Greedy | Sampler.Sample` calls of the batcher loop stand today
// (src/OpenTail.Stingray.Engine/ContinuousBatchingEngine.cs:609-650) and gives the same tokens for the same logits,
// parameters, histories, masks and uniforms; the logits never leave the device.
// Not compiled in this repository (no .NET SDK in its build image).
using System.Runtime.InteropServices;

namespace OpenTail.Stingray.Rocm;

/// <summary>What one decode step hands over per row (the inputs the hot loop gathers today, :609-650).</summary>
public readonly ref struct BatchedSamplingInputs
{
    /// <summary>Per row: the request's parameters (`seq.Sp`); PreviousTokens is ignored, Histories is used.</summary>
    public required ReadOnlySpan<SamplingParams> Params { get; init; }
    /// <summary>Per row: `seq.RecentTokens` (null where the request has no history penalty, :1280).</summary>
    public required ReadOnlySpan<List<int>?> Histories { get; init; }
    /// <summary>Per row: the registered mask of the constraint's current state, -1 when it is not constraining or
    /// Filter would return its input (dead state, ITokenConstraint.cs:36-41).</summary>
    public required ReadOnlySpan<int> MaskIds { get; init; }
    /// <summary>Per row: one `seq.Rng.NextDouble()`, drawn in row order for rows with Temperature > 0 only
    /// (Sampler.Sample draws exactly once per sampled call and never for greedy ones, Sampler.cs:19-22).</summary>
    public required ReadOnlySpan<double> Uniforms { get; init; }
    /// <summary>Per row: the token sampled in the previous step (joins the history), or null on the first step
    /// and whenever the set of rows changed.</summary>
    public ReadOnlySpan<int> PreviousTokens { get; init; }
}

public sealed unsafe class RocmBatchSampler : IDisposable
{
    private readonly nint _ctx;
    private nint _batch;
    private int _rows = -1, _vocab;
    // the library's copy of the histories is what the engine's RecentTokens are: true after a step that went through
    // Sample, false after any step that did not
    private bool _historyValid;

    public static bool IsAvailable => StingraySamplerInterop.IsAvailable;

    public RocmBatchSampler(int deviceOrdinal, nint hipStream)
    {
        int rc = StingraySamplerInterop.Create(deviceOrdinal, out _ctx);
        if (rc != 0) throw new InvalidOperationException($"sr_create failed: {rc}");
        // the stream that produces the logits: launches are ordered behind the LM head without an event
        StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.SetStream(_ctx, hipStream), "sr_set_stream");
        StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.BatchCreate(_ctx, out _batch), "sr_batch_create");
    }

    /// <summary>IThreadAffineBackend.BindToCurrentThread (IThreadAffineBackend.cs:9-21): the batcher task re-binds
    /// each iteration (ContinuousBatchingEngine.cs:495-500).</summary>
    public void BindToCurrentThread() =>
        StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.BindThread(_ctx), "sr_bind_thread");

    /// <summary>Registers the packed allow-bits of one constraint state (ceil(vocab / 32) words); the constraint keeps
    /// the id with the state (JsonToolArgumentConstraint caches its masks per automaton state, :434-478).</summary>
    public int RegisterMask(ReadOnlySpan<uint> words, int vocab)
    {
        fixed (uint* w = words)
        {
            StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.MaskRegister(_ctx, w, 0, vocab, out int id), "sr_mask_register");
            return id;
        }
    }

    /// <summary>The masked row a Filter call returned -> allow-bits (allowed iff not negative infinity).</summary>
    public static void PackMask(ReadOnlySpan<float> masked, Span<uint> words)
    {
        fixed (float* m = masked)
        fixed (uint* w = words)
        {
            int rc = StingraySamplerInterop.PackAllowMask(m, masked.Length, w);
            if (rc != 0) throw new InvalidOperationException($"sr_pack_allow_mask failed: {rc}");
        }
    }

    /// <summary>AndTokenConstraint.Filter over registered masks (AndTokenConstraint.cs:44-86): the id of the intersection,
    /// or -1 (no mask) when no id is left to intersect or no token survives.</summary>
    public int MaskAnd(ReadOnlySpan<int> ids)
    {
        fixed (int* p = ids)
        {
            StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.MaskAnd(_ctx, p, ids.Length, out int id), "sr_mask_and");
            return id;
        }
    }

    /// <summary>A decode step did not go through Sample: the next one uploads, whatever the caller says about its rows.</summary>
    public void InvalidateHistory() => _historyValid = false;

    public void ReleaseMask(int id) =>
        StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.MaskRelease(_ctx, id), "sr_mask_release");

    /// <summary>
    /// One step: enqueues the sampling of `rows` rows of logits that lie on the device ([rows x vocab], dtype 0 = fp32,
    /// 1 = bf16) into tokensDev (rows x int32, device).  On the first step, and whenever the rows changed, the inputs
    /// are packed and uploaded; on the following steps only the previous tokens, the mask ids and the uniforms go over
    /// (sr_batch_append_tokens_masks).  Nothing here waits for the device: the caller's rows x 4-byte download of
    /// tokensDev on the same stream is the only synchronisation, the shape of traffic BatchForwardMultiArgmax has
    /// (CudaForwardPass.cs:5229-5232).
    /// </summary>
    public void Sample(nint logitsDev, int dtype, int rows, int vocab, long rowStrideElems,
                       nint tokensDev, nint flagsDev, in BatchedSamplingInputs inputs, bool sameRowsAsLastStep)
    {
        if (sameRowsAsLastStep && _historyValid && rows == _rows && vocab == _vocab && inputs.PreviousTokens.Length == rows)
        {
            fixed (int* t = inputs.PreviousTokens)
            fixed (double* u = inputs.Uniforms)
            fixed (int* m = inputs.MaskIds)
                StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.BatchAppendTokensMasks(_batch, t, u, m),
                                             "sr_batch_append_tokens_masks");
        }
        else
        {
            Upload(rows, vocab, inputs);
        }
        StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.SampleLaunch(_ctx, _batch, logitsDev, dtype, rowStrideElems,
                                                                             tokensDev, flagsDev), "sr_sample_launch");
        _historyValid = true;
    }

    private void Upload(int rows, int vocab, in BatchedSamplingInputs inputs)
    {
        var rp = new SrRowParams[rows];
        var histOffsets = new int[rows + 1];
        var biasOffsets = new int[rows + 1];
        int nHist = 0, nBias = 0;
        for (int r = 0; r < rows; r++)
        {
            nHist += inputs.Histories[r]?.Count ?? 0;
            nBias += inputs.Params[r].LogitBias?.Count ?? 0;
        }
        var histIds = new int[Math.Max(nHist, 1)];
        var biasIds = new int[Math.Max(nBias, 1)];
        var biasVals = new float[Math.Max(nBias, 1)];
        int h = 0, b = 0;
        for (int r = 0; r < rows; r++)
        {
            SamplingParams p = inputs.Params[r];
            rp[r] = new SrRowParams
            {
                Temperature = p.Temperature, TopK = p.TopK, TopP = p.TopP, MinP = p.MinP,
                RepetitionPenalty = p.RepetitionPenalty, RepeatLastN = p.RepeatLastN,
                PresencePenalty = p.PresencePenalty, FrequencyPenalty = p.FrequencyPenalty,
                SpecDraftPMin = 0f, Flags = p.LogitBias is { Count: > 0 } ? 1u : 0u,
            };
            if (inputs.Histories[r] is { } hist)
                foreach (int id in hist) histIds[h++] = id;   // in order, duplicates kept: the window is positional
            histOffsets[r + 1] = h;
            if (p.LogitBias is { Count: > 0 } bias)
                foreach (var (id, v) in bias) { biasIds[b] = id; biasVals[b++] = v; }
            biasOffsets[r + 1] = b;
        }
        fixed (SrRowParams* prp = rp)
        fixed (int* ph = histIds, pho = histOffsets, pb = biasIds, pbo = biasOffsets, pm = inputs.MaskIds)
        fixed (float* pbv = biasVals)
        fixed (double* pu = inputs.Uniforms)
            StingraySamplerInterop.Check(_ctx, StingraySamplerInterop.BatchUploadMaskIds(
                _batch, rows, vocab, prp, ph, pho, nBias > 0 ? pb : null, nBias > 0 ? pbv : null, nBias > 0 ? pbo : null,
                pm, pu, 1), "sr_batch_upload_mask_ids");
        _rows = rows;
        _vocab = vocab;
    }

    public void Dispose()
    {
        if (_batch != 0) { StingraySamplerInterop.BatchDestroy(_batch); _batch = 0; }
        StingraySamplerInterop.Destroy(_ctx);
    }
}
