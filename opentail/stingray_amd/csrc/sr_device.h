// Device helpers shared by the kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#define SR_WAVE 64
#define SR_NEG_INF (__uint_as_float(0xff800000u))

__device__ __forceinline__ uint32_t sr_f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float sr_u2f(uint32_t u) { return __uint_as_float(u); }

// Order-preserving map float -> uint32 (larger float = larger key).  -0 is folded onto +0 so that
// key equality is float equality; NaN handling is the caller's business.
__device__ __forceinline__ uint32_t sr_okey(float v)
{
    uint32_t b = sr_f2u(v);
    if (b == 0x80000000u) b = 0u;
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float sr_okey_inv(uint32_t k)
{
    uint32_t b = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return sr_u2f(b);
}

// The larger of two values that are not NaN, in one instruction (fmaxf first quiets a possible signalling NaN with
// an instruction of its own).
__device__ __forceinline__ float sr_max_f32(float a, float b)
{
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

__device__ __forceinline__ float sr_bf16_to_f32(uint16_t h) { return sr_u2f(((uint32_t)h) << 16); }

// glibc expf (2^(i/32) table, cubic in double, one rounding to float) with the FMA contractions of the
// x86-64 -mfma build: the managed sampler's MathF.Exp on Linux.  Every operation is spelled with an
// explicitly rounded intrinsic so the compiler can neither fuse nor reorder.
__device__ static const uint64_t sr_exp2f_tab[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

// tab: the 32-entry table above, or a copy of it in LDS (a lookup per element from global memory is a long
// dependent load)
__device__ __forceinline__ float sr_expf_tab(float x, const uint64_t* tab)
{
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;
    const double shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double c1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double c2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    const uint32_t xb = sr_f2u(x);
    const uint32_t abstop = (xb >> 20) & 0x7ffu;
    // The main path runs for every input and the special ones are put in place of its result afterwards, by selects:
    // without a branch per element the compiler interleaves the chains of several elements (each is a dozen dependent
    // double-precision operations with a table lookup in the middle) instead of running them one behind the other.
    double xd = (double)x;
    double z = __dmul_rn(inv_ln2_n, xd);
    double kd = __dadd_rn(z, shift);
    uint64_t ki = (uint64_t)__double_as_longlong(kd);
    kd = __dsub_rn(kd, shift);
    double r = __fma_rn(inv_ln2_n, xd, -kd);
    uint64_t t = tab[ki & 31u];
    t += ki << (52 - 5);
    double s = __longlong_as_double((long long)t);
    double zz = __fma_rn(c0, r, c1);
    double r2 = __dmul_rn(r, r);
    double y = __fma_rn(c2, r, 1.0);
    y = __fma_rn(zz, r2, y);
    y = __dmul_rn(y, s);
    float e = __double2float_rn(y);
    // underflow to 0, overflow to +inf, NaN and +inf propagate, -inf gives 0 (the later line wins)
    e = (x < -0x1.9fe368p6f) ? 0.0f : e;
    e = (x > 0x1.62e42ep6f) ? sr_u2f(0x7f800000u) : e;
    e = (abstop >= (0x7f800000u >> 20)) ? __fadd_rn(x, x) : e;
    e = (xb == 0xff800000u) ? 0.0f : e;
    return e;
}
__device__ __forceinline__ float sr_expf(float x) { return sr_expf_tab(x, sr_exp2f_tab); }

// ---- cross-workgroup hand-off without a full L2 write-back ----------------------------------------
// Data one workgroup leaves for another (possibly on another XCD) is written with agent-scope stores
// (write-through past the XCD-private L2) and read back with agent-scope loads; the writer drains its
// own stores (s_waitcnt) before the workgroup barrier that precedes the hand-off counter.  A release
// fence would instead write back every dirty line of the L2.
template <typename T> __device__ __forceinline__ void sr_store_agent(T* p, T v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T> __device__ __forceinline__ T sr_load_agent(const T* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16 bytes in one write-through store (four separate 4-byte stores of a thread reach memory as four partial
// writes of the same line).  The compiler neither counts this store (sr_drain_stores() waits for it) nor
// knows its hazards: a store of more than 8 bytes reads its data registers a few cycles after issue, so the
// wait states that must separate it from the next write of those registers are part of the statement.
__device__ __forceinline__ void sr_store_agent_f4(float4* p, float x, float y, float z, float w)
{
    typedef float __attribute__((ext_vector_type(4))) f32x4;
    const f32x4 v = {x, y, z, w};
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 3" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void sr_drain_stores() { __builtin_amdgcn_s_waitcnt(0); }

// A workgroup barrier for data exchanged through LDS only: waits for this wave's LDS operations, not for its loads
// from memory.  __syncthreads() carries a fence that also waits for every load in flight, which throws away
// whatever a loop has prefetched for its next turn.
__device__ __forceinline__ void sr_barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- wave / block primitives --------------------------------------------------------------------
__device__ __forceinline__ int sr_lane() { return (int)(threadIdx.x & (SR_WAVE - 1)); }
__device__ __forceinline__ int sr_wave_id() { return (int)(threadIdx.x >> 6); }

// Wave-wide reductions and the scan move data with DPP inside rows of 16 lanes and with v_readlane across
// rows: no LDS traffic and no address registers.  Every lane of the wave must be active.
template <int kCtrl> __device__ __forceinline__ uint32_t sr_dpp_u32(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kCtrl, 0xf, 0xf, true);
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;
template <typename Op> __device__ __forceinline__ uint32_t sr_wave_reduce_u32(uint32_t v, Op op)
{
    v = op(v, sr_dpp_u32<kDppXor1>(v));
    v = op(v, sr_dpp_u32<kDppXor2>(v));
    v = op(v, sr_dpp_u32<kDppHalfMirror>(v));
    v = op(v, sr_dpp_u32<kDppMirror>(v));
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return op(op(a, b), op(c, d));
}
__device__ __forceinline__ uint32_t sr_wave_max_u32(uint32_t v)
{
    return sr_wave_reduce_u32(v, [](uint32_t x, uint32_t y) { return x > y ? x : y; });
}
__device__ __forceinline__ uint32_t sr_wave_min_u32(uint32_t v)
{
    return sr_wave_reduce_u32(v, [](uint32_t x, uint32_t y) { return x < y ? x : y; });
}
__device__ __forceinline__ int sr_wave_sum_i32(int v)
{
    return (int)sr_wave_reduce_u32((uint32_t)v, [](uint32_t x, uint32_t y) { return x + y; });
}
__device__ __forceinline__ int sr_wave_min_i32(int v)
{
    return (int)sr_wave_reduce_u32((uint32_t)v, [](uint32_t x, uint32_t y) { return (int)x < (int)y ? x : y; });
}
__device__ __forceinline__ unsigned long long sr_wave_max_u64(unsigned long long v)
{
    auto step = [&](auto ctrl) {
        constexpr int kC = decltype(ctrl)::value;
        const unsigned long long w = ((unsigned long long)sr_dpp_u32<kC>((uint32_t)(v >> 32)) << 32) | sr_dpp_u32<kC>((uint32_t)v);
        v = w > v ? w : v;
    };
    step(std::integral_constant<int, kDppXor1>{});
    step(std::integral_constant<int, kDppXor2>{});
    step(std::integral_constant<int, kDppHalfMirror>{});
    step(std::integral_constant<int, kDppMirror>{});
    unsigned long long r = 0ull;
#pragma unroll
    for (int l = 0; l < SR_WAVE; l += 16) {
        const unsigned long long w = ((unsigned long long)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), l) << 32) |
                                     (unsigned long long)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, l);
        r = w > r ? w : r;
    }
    return r;
}
// the sum of v over the wave, single precision, the same in every lane (the order of the additions is the reduction's own)
__device__ __forceinline__ float sr_wave_sum_f32(float v)
{
    v += __uint_as_float(sr_dpp_u32<kDppXor1>(__float_as_uint(v)));
    v += __uint_as_float(sr_dpp_u32<kDppXor2>(__float_as_uint(v)));
    v += __uint_as_float(sr_dpp_u32<kDppHalfMirror>(__float_as_uint(v)));
    v += __uint_as_float(sr_dpp_u32<kDppMirror>(__float_as_uint(v)));
    const float a = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 0));
    const float b = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 16));
    const float c = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 32));
    const float d = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 48));
    return (a + b) + (c + d);
}
// inclusive prefix sum across the wave, single precision (the order of the additions is the scan's own)
__device__ __forceinline__ float sr_wave_incl_sum_f32(float v)
{
    v += __uint_as_float(sr_dpp_u32<0x111>(__float_as_uint(v)));
    v += __uint_as_float(sr_dpp_u32<0x112>(__float_as_uint(v)));
    v += __uint_as_float(sr_dpp_u32<0x114>(__float_as_uint(v)));
    v += __uint_as_float(sr_dpp_u32<0x118>(__float_as_uint(v)));
    const float r0 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 15));
    const float r1 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 31));
    const float r2 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 47));
    const int row = (int)(threadIdx.x & 63u) >> 4;
    return v + ((row >= 1 ? r0 : 0.0f) + (row >= 2 ? r1 : 0.0f) + (row >= 3 ? r2 : 0.0f));
}
// inclusive prefix sum across the wave
__device__ __forceinline__ int sr_wave_incl_scan_i32(int v)
{
    // inside every row of 16 lanes: shifts by 1, 2, 4, 8 with zero fill
    v += (int)sr_dpp_u32<0x111>((uint32_t)v);
    v += (int)sr_dpp_u32<0x112>((uint32_t)v);
    v += (int)sr_dpp_u32<0x114>((uint32_t)v);
    v += (int)sr_dpp_u32<0x118>((uint32_t)v);
    // the rows before this lane's
    const int r0 = __builtin_amdgcn_readlane(v, 15), r1 = __builtin_amdgcn_readlane(v, 31), r2 = __builtin_amdgcn_readlane(v, 47);
    const int row = sr_lane() >> 4;
    return v + (row >= 1 ? r0 : 0) + (row >= 2 ? r1 : 0) + (row >= 3 ? r2 : 0);
}
