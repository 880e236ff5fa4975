// Row-wise argmax: Sampler.Greedy (Sampler.cs:442-446) for a [rows x vocab] tensor, the counterpart of
// the reference's llm_argmax_rows (CudaTextKernels.cs:465-479).  Lowest index wins on equal values; a NaN
// element wins outright (first NaN), as TensorPrimitives.IndexOfMax documents.
//
// One launch, grid = rows x chunks.  A workgroup streams its chunk with 16-byte non-temporal loads (eight in
// flight per thread), reduces it to a packed (key << 32 | ~index) and, when the row has more than one chunk,
// folds that into the row's slot with a 64-bit atomic max and counts itself in; the workgroup that counts in
// last writes the row's result and puts slot and counter back to zero, so the scratch of one launch is ready
// for the next without a fill.  Rows of one chunk write their result directly.
//
// This file also holds the scratch of the entry point that allocates nothing: a zero-initialised array in
// device memory that belongs to the library's code object, one copy per GPU.
#include <algorithm>

#include "sr_device.h"
#include "sr_kernels.h"
#include "sr_types.h"

// best[SR_ARGMAX_STATIC_ROWS] (8 bytes each) followed by done[SR_ARGMAX_STATIC_ROWS] (4 bytes each): 192 KiB.
// In host code this name is only a handle for hipGetSymbolAddress, never an address to give a kernel.
static __device__ __align__(256) unsigned long long scratch[SR_ARGMAX_STATIC_ROWS + SR_ARGMAX_STATIC_ROWS / 2];

namespace {
constexpr int kThreads = 256;
constexpr int kUnroll = 8;

typedef uint32_t __attribute__((ext_vector_type(4))) u32x4;

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];  // per device: where that device's copy of `scratch` lies

__global__ void k_fill_u32(uint32_t* p, int n, uint32_t v)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

template <int ES> __device__ __forceinline__ float load_elem(const char* p, int64_t i)
{
    if (ES == 4) return ((const float*)p)[i];
    return sr_bf16_to_f32(((const uint16_t*)p)[i]);
}

// A thread's best element so far: key (NaN above everything) and index.  A thread meets its elements in ascending
// index order, so "strictly larger" keeps the first of equal keys.
struct Best {
    uint32_t key, idx;
};
__device__ __forceinline__ void fold(Best& b, float v, uint32_t i)
{
    const uint32_t k = (v != v) ? 0xffffffffu : sr_okey(v);
    const bool up = k > b.key;
    b.idx = up ? i : b.idx;
    b.key = up ? k : b.key;
}

template <int ES> __device__ __forceinline__ void fold_vec(Best& best, const u32x4 t, uint32_t first)
{
#pragma unroll
    for (int w = 0; w < 4; w++) {
        if (ES == 4) {
            fold(best, sr_u2f(t[w]), first + w);
        } else {
            fold(best, sr_u2f(t[w] << 16), first + 2 * w);
            fold(best, sr_u2f(t[w] & 0xffff0000u), first + 2 * w + 1);
        }
    }
}

// kVec: the rows start on 16-byte boundaries and chunk_len is a multiple of the elements of a vector
template <int ES, bool kVec> __global__ __launch_bounds__(kThreads) void k_argmax_rows(SrArgmaxArgs a)
{
    __shared__ unsigned long long s_best[kThreads / SR_WAVE];
    constexpr int EPV = 16 / ES;
    const int row = __builtin_amdgcn_readfirstlane((int)(blockIdx.x / (unsigned)a.chunks));
    const int c = (int)blockIdx.x - row * a.chunks;
    const int lo = c * a.chunk_len, hi = min(a.vocab, lo + a.chunk_len);
    const char* rowp = (const char*)a.logits + (size_t)row * (size_t)a.row_stride * ES;
    const int tid = (int)threadIdx.x;
    Best tb;
    tb.key = 0u;  // (no element has the key 0: an empty chunk leaves it)
    tb.idx = 0u;
    int scalar_from = lo;
    if (kVec) {
        const u32x4* vp = (const u32x4*)rowp;
        const int v_lo = lo / EPV, v_hi = hi / EPV;  // whole vectors; only the row's last chunk can leave elements over
        // Sets of kUnroll vectors per thread, all of a set's loads issued before the first is folded.  The chunk's last
        // set is loaded whole too -- a vector past the chunk's end is the chunk's last one again and is not folded --
        // rather than vector by vector, each of which would be a trip to memory of its own.
        const int last = v_hi - 1;
        for (int base = v_lo; base < v_hi; base += kUnroll * kThreads) {
            const int i = base + tid;
            u32x4 t[kUnroll];
            if (base + kUnroll * kThreads <= v_hi) {
#pragma unroll
                for (int j = 0; j < kUnroll; j++) t[j] = __builtin_nontemporal_load(vp + i + j * kThreads);
#pragma unroll
                for (int j = 0; j < kUnroll; j++) fold_vec<ES>(tb, t[j], (uint32_t)(i + j * kThreads) * EPV);
            } else {
#pragma unroll
                for (int j = 0; j < kUnroll; j++) t[j] = __builtin_nontemporal_load(vp + min(i + j * kThreads, last));
#pragma unroll
                for (int j = 0; j < kUnroll; j++)
                    if (i + j * kThreads < v_hi) fold_vec<ES>(tb, t[j], (uint32_t)(i + j * kThreads) * EPV);
            }
        }
        scalar_from = max(lo, v_hi * EPV);
    }
    for (int i = scalar_from + tid; i < hi; i += kThreads) fold(tb, load_elem<ES>(rowp, i), (uint32_t)i);

    // (key << 32 | ~index): the largest key wins, among equal keys the lowest index
    unsigned long long best = tb.key ? ((unsigned long long)tb.key << 32) | (unsigned long long)(0xffffffffu - tb.idx) : 0ull;
    best = sr_wave_max_u64(best);
    if (sr_lane() == 0) s_best[sr_wave_id()] = best;
    __syncthreads();
    if (tid != 0) return;
    for (int w = 1; w < kThreads / SR_WAVE; w++) best = s_best[w] > best ? s_best[w] : best;
    if (a.chunks > 1) {
        // Both are device-scope atomics without a fence (a release fence would write back the whole L2): the maximum
        // is waited for -- its old value comes back -- before the chunk is counted in, so whoever counts in last
        // finds every chunk's maximum in the slot.
        const unsigned long long seen = __hip_atomic_fetch_max(&a.best[row], best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("" : : "v"(seen) : "memory");
        const uint32_t before = __hip_atomic_fetch_add(&a.done[row], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (before != (uint32_t)a.chunks - 1u) return;
        best = __hip_atomic_load(&a.best[row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&a.best[row], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&a.done[row], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const int idx = best ? (int)(0xffffffffu - (uint32_t)(best & 0xffffffffull)) : 0;  // empty row -> 0
    a.out_idx[row] = idx;
    if (a.out_val) a.out_val[row] = a.vocab > 0 ? load_elem<ES>(rowp, idx) : 0.0f;  // the original bits, not a decode
}

#ifdef SR_TEST_HOOKS
__global__ void k_selftest_expf(const float* x, float* y, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = sr_expf(x[i]);
}
#endif
}  // namespace

void sr_argmax_plan(SrArgmaxArgs& a, int cu_count)
{
    const int es = a.dtype == 1 ? 2 : 4, epv = 16 / es;
    a.vec = ((uintptr_t)a.logits % 16 == 0 && ((size_t)a.row_stride * es) % 16 == 0) ? 1 : 0;
    // enough workgroups for two per compute unit (64 KB of loads in flight on each: what the memory's latency takes at
    // the machine's rate; eight per compute unit, with their dispatch and their atomics, were 5 us slower on 256 rows of
    // 151,936), none with less than one unrolled pass of work
    const int per_pass = kThreads * kUnroll * epv;
    int s = std::max(1, std::min((2 * cu_count + a.rows - 1) / std::max(a.rows, 1), a.vocab / per_pass));
    int len = (a.vocab + s - 1) / s;
    len = (len + epv - 1) / epv * epv;
    a.chunk_len = std::max(len, epv);
    a.chunks = a.vocab > 0 ? (a.vocab + a.chunk_len - 1) / a.chunk_len : 1;
}

hipError_t sr_launch_argmax_rows(const SrArgmaxArgs& a, bool clear_first, hipStream_t stream)
{
    if (a.rows <= 0) return hipSuccess;
    if (clear_first && a.chunks > 1) {
        // best and done are separate arrays: clear each where it is
        hipLaunchKernelGGL(k_fill_u32, dim3((2 * a.rows + 255) / 256), dim3(256), 0, stream, (uint32_t*)a.best, 2 * a.rows, 0u);
        hipLaunchKernelGGL(k_fill_u32, dim3((a.rows + 255) / 256), dim3(256), 0, stream, a.done, a.rows, 0u);
    }
    const dim3 grid((unsigned)a.rows * (unsigned)a.chunks), block(kThreads);
    if (a.dtype == 1) {
        if (a.vec) hipLaunchKernelGGL((k_argmax_rows<2, true>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((k_argmax_rows<2, false>), grid, block, 0, stream, a);
    } else {
        if (a.vec) hipLaunchKernelGGL((k_argmax_rows<4, true>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((k_argmax_rows<4, false>), grid, block, 0, stream, a);
    }
    return hipGetLastError();
}

// The address of the current device's copy of the static scratch, looked up once per device.
hipError_t sr_argmax_static_scratch(int device, unsigned long long** best, uint32_t** done)
{
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    void* p = __atomic_load_n(&g_scratch_ptr[device], __ATOMIC_ACQUIRE);
    if (!p) {
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        __atomic_store_n(&g_scratch_ptr[device], p, __ATOMIC_RELEASE);
    }
    *best = (unsigned long long*)p;
    *done = (uint32_t*)((unsigned long long*)p + SR_ARGMAX_STATIC_ROWS);
    return hipSuccess;
}

#ifdef SR_TEST_HOOKS
hipError_t sr_launch_selftest_expf(const float* x, float* y, int64_t n, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_selftest_expf, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, y, n);
    return hipGetLastError();
}
#endif
