// The seam in the engine: a sampling sibling of the batched argmax capability and the gate that uses it.
// Two additions to existing files, shown here as the code that goes in; not compiled in this repository.
using OpenTail.Stingray.Rocm;

namespace OpenTail.Stingray.Engine;

// ---- 1. src/OpenTail.Stingray.Engine/IBatchedForwardPass.cs, beside SupportsBatchedGpuArgmax (:105-117) ---------
public partial interface IBatchedForwardPass
{
    /// <summary>
    /// Whether <see cref="BatchForwardMultiSample"/> samples every row on the device, so that a step with sampled,
    /// penalised or constrained rows downloads rows x 4 bytes instead of the N x vocab logits. Default false.
    /// </summary>
    bool SupportsBatchedGpuSampling => false;

    /// <summary>
    /// Sampling counterpart of <see cref="BatchForwardMultiArgmax"/>: runs the forward pass, leaves the logits on
    /// the device and returns the token of every row: what Sampler.Greedy / Sampler.Sample give for the same
    /// logits, parameters, histories, masks and uniforms, and the SR_OUT_* flags of every row (rows x 8 bytes come back).
    /// </summary>
    (int[] Tokens, uint[] Flags) BatchForwardMultiSample(int[] tokens, int[] positions, ISequenceKvCache[] caches,
                                  in BatchedSamplingInputs inputs, bool sameRowsAsLastStep) =>
        throw new NotSupportedException(
            $"{GetType().Name} does not implement BatchForwardMultiSample. Check SupportsBatchedGpuSampling first.");

    /// <summary>A decode step did not go through BatchForwardMultiSample (all-greedy argmax step, host fallback): the
    /// device sampler's copy of the histories is stale and the next sampled step uploads them again.</summary>
    void InvalidateSamplingState() { }
}

// ---- 2. src/OpenTail.Stingray.Engine/ContinuousBatchingEngine.cs, in BatcherLoop after the allGreedy gate (:580-606) --

/// <summary>
/// A sequence's Random as the gate needs it: the next NextDouble() can be looked at before it is known whether the
/// sampler consumes it.  Sampler.Sample draws exactly once per sampled call, except that SampleTopK on a row without a
/// finite logit falls back to Greedy and draws nothing (Sampler.cs:251-255).  The device needs the uniform before it
/// knows; a row that reports that fall-back leaves the value pending and the sequence's next draw returns it, so the
/// values a sequence consumes are the reference's.  ActiveSeq.Rng becomes one of these (seeded or not, as today).
/// </summary>
internal sealed class PeekableRandom : Random
{
    private readonly Random _inner;
    private readonly Queue<double> _pending = new();
    public PeekableRandom(Random inner) => _inner = inner;
    public double Peek(int i = 0)
    {
        while (_pending.Count <= i) _pending.Enqueue(_inner.NextDouble());
        return i == 0 ? _pending.Peek() : _pending.ElementAt(i);
    }
    public void Commit(int n = 1) { for (int i = 0; i < n; i++) _pending.Dequeue(); }
    public override double NextDouble() { double v = Peek(); Commit(); return v; }
}

internal sealed class DeviceSamplingGate
{
    private int[] _lastIds = [];
    private long _lastStep = -2;

    /// <summary>
    /// Called where the loop today falls back to BatchForwardMulti (full logits) because some row is sampled, has
    /// history penalties or is constraining.  Returns the tokens, or null when the step must take today's path (the
    /// forward pass cannot sample; a row's token is forced, :618-622).  Nothing is consumed when it returns null: no
    /// Filter call, no uniform.  stepNo counts the engine's decode steps: rows are appended to only when the previous
    /// step sampled the same sequences here; any other step uploads their histories again.
    /// </summary>
    internal int[]? TrySample(IBatchedForwardPass fwd, ReadOnlySpan<ActiveSequenceView> active, int[] tokens,
                              int[] positions, ISequenceKvCache[] caches, StepScratch scratch, long stepNo)
    {
        if (!fwd.SupportsBatchedGpuSampling) return null;
        int n = active.Length;
        // first pass: decisions only
        for (int i = 0; i < n; i++)
            if (active[i].ForcedClose) { fwd.InvalidateSamplingState(); return null; }   // the loop injects the token itself
        // second pass: the mask of every constraint's current state, registered the first time the state is met; a dead
        // state (Filter returns its input) and a constraint that is not constraining are both "no mask"
        for (int i = 0; i < n; i++)
            scratch.MaskIds[i] = active[i].Constraint is { IsConstraining: true } c ? scratch.MaskIdOf(c) : -1;
        // third pass: the step is committed to the device.  One uniform per sampled row is looked at, none for greedy
        // rows: what Sampler.Sample consumes (Sampler.cs:19-22)
        bool sameRows = stepNo == _lastStep + 1 && _lastIds.Length == n;
        for (int i = 0; i < n; i++)
        {
            ActiveSequenceView s = active[i];
            scratch.Params[i] = s.Sp;
            scratch.Histories[i] = s.RecentTokens;                 // null unless Sp.HasHistoryPenalty (:1280)
            scratch.Uniforms[i] = s.Sp.Temperature > 0f ? s.Rng.Peek() : 0.0;
            // the token fed to this forward step is the one the previous step sampled: it joined RecentTokens (:650)
            scratch.PreviousTokens[i] = s.RecentTokens is null ? -1 : tokens[i];
            sameRows &= i < _lastIds.Length && _lastIds[i] == s.Id;
        }
        var inputs = new BatchedSamplingInputs
        {
            Params = scratch.Params.AsSpan(0, n), Histories = scratch.Histories.AsSpan(0, n),
            MaskIds = scratch.MaskIds.AsSpan(0, n), Uniforms = scratch.Uniforms.AsSpan(0, n),
            PreviousTokens = sameRows ? scratch.PreviousTokens.AsSpan(0, n) : default,
        };
        (int[] next, uint[] flags) = fwd.BatchForwardMultiSample(tokens, positions, caches, inputs, sameRows);
        for (int i = 0; i < n; i++)
        {
            const uint degenerateTopK = StingraySamplerInterop.OutDegenerate | StingraySamplerInterop.OutPathTopKFast;
            if (active[i].Sp.Temperature > 0f && (flags[i] & degenerateTopK) != degenerateTopK) active[i].Rng.Commit();
        }
        if (_lastIds.Length != n) _lastIds = new int[n];
        for (int i = 0; i < n; i++) _lastIds[i] = active[i].Id;
        _lastStep = stepNo;
        return next;
        // afterwards the loop does what it does today with every token: Constraint.Accept(next), RecentTokens.Add(next)
        // (:648-650).  In the all-greedy branch (BatchForwardMultiArgmax) the loop calls fwd.InvalidateSamplingState().
    }
}
