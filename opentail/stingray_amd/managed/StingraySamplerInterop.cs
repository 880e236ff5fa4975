// P/Invoke layer over libstingray_sampler.so (include/stingray_sampler.h), in the house style of
// src/OpenTail.Stingray.Cuda/NvrtcInterop.cs:13-131 and src/OpenTail.Stingray.Cpu/BlasInterop.cs:10-71:
// source-generated LibraryImport, blittable arguments, int status returns (0 = success), opaque handles as nint.
// Goes to src/OpenTail.Stingray.Rocm/StingraySamplerInterop.cs.  Not compiled in this repository (no .NET SDK in
// its build image); tests/test_abi_surface.py checks that every entry point of the header is bound here.
using System.Runtime.InteropServices;

namespace OpenTail.Stingray.Rocm;

[StructLayout(LayoutKind.Sequential)]
internal struct SrRowParams            // sr_row_params
{
    public float Temperature; public int TopK; public float TopP; public float MinP;
    public float RepetitionPenalty; public int RepeatLastN; public float PresencePenalty; public float FrequencyPenalty;
    public float SpecDraftPMin; public uint Flags;      // bit 0: LogitBias.Count > 0; bit 1: drafts from prompt lookup
}

internal static unsafe partial class StingraySamplerInterop
{
    private const string Lib = "stingray_sampler";

    // SR_OUT_* bits of the per-row flags
    internal const uint OutPathGreedy = 1u << 0, OutPathTopKFast = 1u << 1, OutPathFullVocab = 1u << 2,
                        OutDegenerate = 1u << 3, OutAmbiguous = 1u << 4;

    [LibraryImport(Lib, EntryPoint = "sr_create")]        internal static partial int Create(int deviceOrdinal, out nint ctx);
    [LibraryImport(Lib, EntryPoint = "sr_destroy")]       internal static partial void Destroy(nint ctx);
    [LibraryImport(Lib, EntryPoint = "sr_bind_thread")]   internal static partial int BindThread(nint ctx);
    [LibraryImport(Lib, EntryPoint = "sr_set_stream")]    internal static partial int SetStream(nint ctx, nint hipStream);
    [LibraryImport(Lib, EntryPoint = "sr_use_own_stream")] internal static partial int UseOwnStream(nint ctx);
    [LibraryImport(Lib, EntryPoint = "sr_synchronize")]   internal static partial int Synchronize(nint ctx);
    [LibraryImport(Lib, EntryPoint = "sr_last_error")]    internal static partial nint LastError(nint ctx);

    [LibraryImport(Lib, EntryPoint = "sr_batch_create")]  internal static partial int BatchCreate(nint ctx, out nint batch);
    [LibraryImport(Lib, EntryPoint = "sr_batch_destroy")] internal static partial void BatchDestroy(nint batch);
    [LibraryImport(Lib, EntryPoint = "sr_batch_upload")]
    internal static partial int BatchUpload(nint batch, int rows, int vocab, SrRowParams* rowParams,
        int* histIds, int* histOffsets, int* biasIds, float* biasVals, int* biasOffsets,
        uint* allowMask, long maskStrideWords, byte* maskActive, double* uniforms, int uniformsPerRow);
    [LibraryImport(Lib, EntryPoint = "sr_batch_set_uniforms")] internal static partial int BatchSetUniforms(nint batch, double* uniforms);
    [LibraryImport(Lib, EntryPoint = "sr_batch_append_tokens")] internal static partial int BatchAppendTokens(nint batch, int* tokens, double* uniforms);

    [LibraryImport(Lib, EntryPoint = "sr_sample_launch")]
    internal static partial int SampleLaunch(nint ctx, nint batch, nint logitsDev, int dtype, long rowStrideElems,
        nint outTokensDev, nint outFlagsDev);
    [LibraryImport(Lib, EntryPoint = "sr_resample_rows_launch")]
    internal static partial int ResampleRowsLaunch(nint ctx, nint batch, nint logitsDev, int dtype, long rowStrideElems,
        int* rowsHost, int nRows, nint outTokensDev, nint outFlagsDev);
    [LibraryImport(Lib, EntryPoint = "sr_sample_batch")]
    internal static partial int SampleBatch(nint ctx, nint logits, int dtype, int logitsOnDevice, int rows, int vocab,
        long rowStrideElems, SrRowParams* rowParams, int* histIds, int* histOffsets, int* biasIds, float* biasVals,
        int* biasOffsets, uint* allowMask, long maskStrideWords, byte* maskActive, double* uniforms,
        int* outTokens, uint* outFlags);
    [LibraryImport(Lib, EntryPoint = "sr_argmax_rows")]
    internal static partial int ArgmaxRows(nint ctx, nint logits, int dtype, int logitsOnDevice, int rows, int vocab,
        long rowStrideElems, int* outIdx, float* outVal);
    [LibraryImport(Lib, EntryPoint = "sr_build_distribution_launch")]
    internal static partial int BuildDistributionLaunch(nint ctx, nint batch, nint logitsDev, int dtype, long rowStrideElems,
        nint outProbsDev, long probsStrideElems, int probsLen);
    [LibraryImport(Lib, EntryPoint = "sr_sample_with_distribution_launch")]
    internal static partial int SampleWithDistributionLaunch(nint ctx, nint batch, nint logitsDev, int dtype,
        long rowStrideElems, nint outProbsDev, long probsStrideElems, int probsLen, nint outTokensDev);
    [LibraryImport(Lib, EntryPoint = "sr_sample_from_probs_launch")]
    internal static partial int SampleFromProbsLaunch(nint ctx, nint probsDev, int rows, int vocab, long probsStrideElems,
        double* uniforms, nint outTokensDev);
    [LibraryImport(Lib, EntryPoint = "sr_resample_residual_launch")]
    internal static partial int ResampleResidualLaunch(nint ctx, nint pDev, int pLen, long pStride, nint qDev, int qLen,
        long qStride, int rows, double* uniforms, nint outTokensDev);
    [LibraryImport(Lib, EntryPoint = "sr_spec_verify_launch")]
    internal static partial int SpecVerifyLaunch(nint ctx, nint batch, nint targetLogitsDev, nint draftProbsDev,
        nint draftTokensDev, int nDraft, nint outAcceptedDev, nint outTokensDev);
    [LibraryImport(Lib, EntryPoint = "sr_mtp_verify_launch")]
    internal static partial int MtpVerifyLaunch(nint ctx, nint logitsDev, int rows, int vocab, long rowStrideElems,
        nint draftTokensDev, float pMin, nint outArgmaxDev, nint outAcceptDev, nint outProbDev);
    [LibraryImport(Lib, EntryPoint = "sr_argmax_rows_launch")]
    internal static partial int ArgmaxRowsLaunch(nint ctx, nint logitsDev, int dtype, int rows, int vocab,
        long rowStrideElems, nint outIdxDev, nint outValDev);
    [LibraryImport(Lib, EntryPoint = "sr_mask_register")]
    internal static partial int MaskRegister(nint ctx, uint* words, int wordsOnDevice, int vocab, out int maskId);
    [LibraryImport(Lib, EntryPoint = "sr_mask_release")]
    internal static partial int MaskRelease(nint ctx, int maskId);
    [LibraryImport(Lib, EntryPoint = "sr_mask_and")]
    internal static partial int MaskAnd(nint ctx, int* maskIds, int n, out int maskId);
    [LibraryImport(Lib, EntryPoint = "sr_pack_allow_mask_launch")]
    internal static partial int PackAllowMaskLaunch(nint ctx, nint maskedLogitsDev, int dtype, int rows, int vocab,
        long rowStrideElems, nint outWordsDev, long outStrideWords);
    [LibraryImport(Lib, EntryPoint = "sr_batch_upload_mask_ids")]
    internal static partial int BatchUploadMaskIds(nint batch, int rows, int vocab, SrRowParams* rowParams,
        int* histIds, int* histOffsets, int* biasIds, float* biasVals, int* biasOffsets, int* maskIds,
        double* uniforms, int uniformsPerRow);
    [LibraryImport(Lib, EntryPoint = "sr_batch_append_tokens_masks")]
    internal static partial int BatchAppendTokensMasks(nint batch, int* tokens, double* uniforms, int* maskIds);
    [LibraryImport(Lib, EntryPoint = "sr_argmax_rows_launch_noalloc")]
    internal static partial int ArgmaxRowsLaunchNoAlloc(nint ctx, nint logitsDev, int dtype, int rows, int vocab,
        long rowStrideElems, nint outIdxDev, nint outValDev);
    // span-shaped forms (host buffers in and out) of the four calls above
    [LibraryImport(Lib, EntryPoint = "sr_build_distribution")]
    internal static partial int BuildDistribution(nint ctx, float* logits, int rows, int vocab, long rowStrideElems,
        SrRowParams* rowParams, int* histIds, int* histOffsets, int* biasIds, float* biasVals, int* biasOffsets,
        float* outProbs, long probsStrideElems, int probsLen);
    [LibraryImport(Lib, EntryPoint = "sr_sample_with_distribution")]
    internal static partial int SampleWithDistribution(nint ctx, float* logits, int rows, int vocab, long rowStrideElems,
        SrRowParams* rowParams, int* histIds, int* histOffsets, int* biasIds, float* biasVals, int* biasOffsets,
        double* uniforms, float* outProbs, long probsStrideElems, int probsLen, int* outTokens);
    [LibraryImport(Lib, EntryPoint = "sr_sample_from_probs")]
    internal static partial int SampleFromProbs(nint ctx, float* probs, int rows, int vocab, long probsStrideElems,
        double* uniforms, int* outTokens);
    [LibraryImport(Lib, EntryPoint = "sr_resample_residual")]
    internal static partial int ResampleResidual(nint ctx, float* p, int pLen, long pStrideElems, float* q, int qLen,
        long qStrideElems, int rows, double* uniforms, int* outTokens);
    [LibraryImport(Lib, EntryPoint = "sr_version")] internal static partial nint Version();
    [LibraryImport(Lib, EntryPoint = "sr_pack_allow_mask")]
    internal static partial int PackAllowMask(float* maskedLogits, int vocab, uint* outWords);

    // cached availability probe with a kill switch, as BlasInterop.IsAvailable / STINGRAY_GPU_ARGMAX
    private static readonly Lazy<bool> s_available = new(() =>
        Environment.GetEnvironmentVariable("STINGRAY_GPU_SAMPLER") != "0" && NativeLibrary.TryLoad(Lib, out _));
    internal static bool IsAvailable => s_available.Value;

    internal static void Check(nint ctx, int rc, string what)
    {
        if (rc == 0) return;
        string msg = Marshal.PtrToStringUTF8(LastError(ctx)) ?? "";
        throw rc switch
        {
            1 => new ArgumentException(msg),                 // SR_ERR_INVALID_ARGUMENT
            2 => new ArgumentNullException(msg),             // SR_ERR_NULL_ARGUMENT
            _ => new InvalidOperationException($"{what} failed: {rc} {msg}"),   // CudaBackend.cs:4110-4117 style
        };
    }
}
