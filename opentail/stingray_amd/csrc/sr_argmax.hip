// Row-wise argmax: Sampler.Greedy (Sampler.cs:442-446) for a [rows x vocab] tensor, the counterpart of
// the reference's llm_argmax_rows (CudaTextKernels.cs:465-479).  Lowest index wins on equal values; a NaN
// element wins outright (first NaN), as TensorPrimitives.IndexOfMax documents.
//
// grid = rows x chunks; each workgroup reduces one chunk to a packed (key << 32 | ~index) and folds it
// into the row's slot with a 64-bit atomic max, so no second pass is needed.
#include "sr_device.cuh"
#include "sr_kernels.h"

namespace {
constexpr int kThreads = 256;

__global__ void k_fill_u64(unsigned long long* p, int n, unsigned long long v)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

template <int ES>
__device__ __forceinline__ float load_elem(const char* p, int64_t i)
{
    if (ES == 4) return ((const float*)p)[i];
    return sr_bf16_to_f32(((const uint16_t*)p)[i]);
}

template <int ES>
__global__ __launch_bounds__(kThreads) void k_argmax_chunks(SrArgmaxArgs a)
{
    __shared__ unsigned long long s_best[kThreads / SR_WAVE];
    const int row = blockIdx.x / a.chunks, c = blockIdx.x - row * a.chunks;
    const int lo = c * a.chunk_len, hi = min(a.vocab, lo + a.chunk_len);
    const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
    unsigned long long best = 0ull;
    for (int i = lo + (int)threadIdx.x; i < hi; i += kThreads) {
        float v = load_elem<ES>(rowp, i);
        uint32_t k = (v != v) ? 0xffffffffu : sr_okey(v);
        unsigned long long e = ((unsigned long long)k << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
        best = e > best ? e : best;
    }
    best = sr_wave_max_u64(best);
    if (sr_lane() == 0) s_best[sr_wave_id()] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kThreads / SR_WAVE; w++) best = s_best[w] > best ? s_best[w] : best;
        if (best) atomicMax(&a.best[row], best);
    }
}

template <int ES>
__global__ void k_argmax_finish(SrArgmaxArgs a)
{
    int row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= a.rows) return;
    unsigned long long e = a.best[row];
    int idx = e ? (int)(0xffffffffu - (uint32_t)(e & 0xffffffffull)) : 0;  // empty row -> 0
    a.out_idx[row] = idx;
    if (a.out_val) {
        const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
        a.out_val[row] = a.vocab > 0 ? load_elem<ES>(rowp, idx) : 0.0f;  // the original bits, not a decode
    }
}

__global__ void k_selftest_expf(const float* x, float* y, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = sr_expf(x[i]);
}
}  // namespace

hipError_t sr_launch_argmax_rows(const SrArgmaxArgs& a, hipStream_t stream)
{
    if (a.rows <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill_u64, dim3((a.rows + 255) / 256), dim3(256), 0, stream, a.best, a.rows, 0ull);
    if (a.vocab > 0) {
        dim3 grid((unsigned)(a.rows * a.chunks));
        if (a.dtype == 1) hipLaunchKernelGGL(k_argmax_chunks<2>, grid, dim3(kThreads), 0, stream, a);
        else hipLaunchKernelGGL(k_argmax_chunks<4>, grid, dim3(kThreads), 0, stream, a);
    }
    if (a.dtype == 1) hipLaunchKernelGGL(k_argmax_finish<2>, dim3((a.rows + 255) / 256), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(k_argmax_finish<4>, dim3((a.rows + 255) / 256), dim3(256), 0, stream, a);
    return hipGetLastError();
}

hipError_t sr_launch_selftest_expf(const float* x, float* y, int64_t n, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_selftest_expf, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, y, n);
    return hipGetLastError();
}
