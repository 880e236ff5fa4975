// Full-vocabulary rows (Sampler.cs:41-95, :118-163, :421-437): placeholder until the kernels land.
#include "sr_host.h"

int sr_full_rows_launch(sr_ctx* ctx, const sr_batch*, const void*, int, int64_t, int32_t*, uint32_t*)
{
    return sr_fail(ctx, SR_ERR_UNSUPPORTED, "full-vocabulary sampling path is not built yet");
}

extern "C" {
int sr_build_distribution_launch(sr_ctx* ctx, const sr_batch*, const void*, int, int64_t, float*, int64_t, int32_t)
{
    return sr_fail(ctx, SR_ERR_UNSUPPORTED, "not built yet");
}
int sr_sample_with_distribution_launch(sr_ctx* ctx, const sr_batch*, const void*, int, int64_t, float*, int64_t,
                                       int32_t, int32_t*)
{
    return sr_fail(ctx, SR_ERR_UNSUPPORTED, "not built yet");
}
int sr_sample_from_probs_launch(sr_ctx* ctx, const float*, int32_t, int32_t, int64_t, const double*, int32_t*)
{
    return sr_fail(ctx, SR_ERR_UNSUPPORTED, "not built yet");
}
int sr_resample_residual_launch(sr_ctx* ctx, const float*, int32_t, int64_t, const float*, int32_t, int64_t, int32_t,
                                const double*, int32_t*)
{
    return sr_fail(ctx, SR_ERR_UNSUPPORTED, "not built yet");
}
int sr_spec_verify_launch(sr_ctx* ctx, const sr_batch*, const float*, const float*, const int32_t*, int32_t, int32_t*,
                          int32_t*)
{
    return sr_fail(ctx, SR_ERR_UNSUPPORTED, "not built yet");
}
int sr_mtp_verify_launch(sr_ctx* ctx, const float*, int32_t, int32_t, int64_t, const int32_t*, float, int32_t*,
                         int32_t*, float*)
{
    return sr_fail(ctx, SR_ERR_UNSUPPORTED, "not built yet");
}
}
