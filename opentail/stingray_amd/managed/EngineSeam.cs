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
    /// logits, parameters, histories, masks and uniforms.
    /// </summary>
    int[] BatchForwardMultiSample(int[] tokens, int[] positions, ISequenceKvCache[] caches,
                                  in BatchedSamplingInputs inputs, bool sameRowsAsLastStep) =>
        throw new NotSupportedException(
            $"{GetType().Name} does not implement BatchForwardMultiSample. Check SupportsBatchedGpuSampling first.");
}

// ---- 2. src/OpenTail.Stingray.Engine/ContinuousBatchingEngine.cs, in BatcherLoop after the allGreedy gate (:580-606) --
internal static class DeviceSamplingGate
{
    /// <summary>
    /// Called where the loop today falls back to BatchForwardMulti (full logits) because some row is sampled, has
    /// history penalties or is constraining.  Returns the tokens, or null when the step must take today's path
    /// (a forced close token, a constraint whose state has no registered mask yet and cannot make one).
    /// </summary>
    internal static int[]? TrySample(IBatchedForwardPass fwd, ReadOnlySpan<ActiveSequenceView> active, int[] tokens,
                                     int[] positions, ISequenceKvCache[] caches, StepScratch scratch, bool sameRows)
    {
        if (!fwd.SupportsBatchedGpuSampling) return null;
        int n = active.Length;
        for (int i = 0; i < n; i++)
        {
            ActiveSequenceView s = active[i];
            if (s.ForcedClose) return null;                        // the loop injects the token itself (:618-622)
            scratch.Params[i] = s.Sp;
            scratch.Histories[i] = s.RecentTokens;                 // null unless Sp.HasHistoryPenalty (:1280)
            // the mask of the constraint's current state, registered the first time the state is met; a dead state
            // (Filter returns its input) and a constraint that is not constraining are both "no mask"
            scratch.MaskIds[i] = s.Constraint is { IsConstraining: true } c ? scratch.MaskIdOf(c) : -1;
            // one draw per sampled row, in row order, none for greedy rows: what Sampler.Sample consumes (Sampler.cs:19-22)
            scratch.Uniforms[i] = s.Sp.Temperature > 0f ? s.Rng.NextDouble() : 0.0;
            scratch.PreviousTokens[i] = s.LastToken;
        }
        var inputs = new BatchedSamplingInputs
        {
            Params = scratch.Params.AsSpan(0, n), Histories = scratch.Histories.AsSpan(0, n),
            MaskIds = scratch.MaskIds.AsSpan(0, n), Uniforms = scratch.Uniforms.AsSpan(0, n),
            PreviousTokens = sameRows ? scratch.PreviousTokens.AsSpan(0, n) : default,
        };
        return fwd.BatchForwardMultiSample(tokens, positions, caches, inputs, sameRows);
        // afterwards the loop does what it does today with every token: Constraint.Accept(next), RecentTokens.Add(next)
        // (:648-650); the library appended the same token to its copy of the history when the next step passes it in
        // PreviousTokens.
    }
}
