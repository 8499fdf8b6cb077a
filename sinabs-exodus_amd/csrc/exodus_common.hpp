// Device-side helpers shared by the row-major (rows, time) kernels and the layer-layout
// (batch, time, neurons) kernels of libexodus_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "exodus_hip.h"

namespace {

constexpr int WAVE = 64;

typedef float f32x4 __attribute__((ext_vector_type(4)));    // one 16-byte chunk = 4 time steps

// Tile lengths (time steps per tile) by number of (n,t) tensors an op keeps in LDS.  Longer tiles
// mean longer contiguous segments per row; more slots mean more LDS per wave.
#ifndef EXODUS_TT_1
#define EXODUS_TT_1 32    // one or two LDS slots
#endif
#ifndef EXODUS_TT_3
#define EXODUS_TT_3 32    // three or more LDS slots
#endif

// The same for the driver that addresses a wave's rows as one span of memory, by LDS tiles per wave.
#ifndef EXODUS_TT_S1
#define EXODUS_TT_S1 32
#endif
#ifndef EXODUS_TT_S2
#define EXODUS_TT_S2 32
#endif
#ifndef EXODUS_TT_S3
#define EXODUS_TT_S3 32
#endif
// most waves per SIMD the span driver's register budget is set for, and how many 4-step chunks of a
// tile its recurrence loop is unrolled by
#ifndef EXODUS_WPE_MAX
#define EXODUS_WPE_MAX 4
#endif
#ifndef EXODUS_SPAN_UNROLL_Q
#define EXODUS_SPAN_UNROLL_Q 2
#endif
// bytes of LDS asked for beyond what the span driver uses (an experiment's knob: fewer waves fit a CU)
#ifndef EXODUS_SPAN_EXTRA_LDS
#define EXODUS_SPAN_EXTRA_LDS 0
#endif
// 64-byte sectors shared by two rows of a wave are written in one piece (0: each row writes its part)
#ifndef EXODUS_WHOLE_SECTORS
#define EXODUS_WHOLE_SECTORS 1
#endif

// Unroll factor of the per-tile chunk loop (each chunk = 4 time steps).  Full unrolling lets the
// compiler hoist every LDS read of the tile, which costs registers and therefore resident waves.
#ifndef EXODUS_UNROLL_Q
#define EXODUS_UNROLL_Q 8
#endif
#define EXODUS_PRAGMA(x) _Pragma(#x)
#define EXODUS_UNROLL(n) EXODUS_PRAGMA(unroll n)

// streaming (non-temporal) hints on the (n,t) tensors, which are read once and written once
#ifndef EXODUS_NT_LOAD
#define EXODUS_NT_LOAD 1
#endif
#ifndef EXODUS_NT_STORE
#define EXODUS_NT_STORE 1
#endif
template <class T> __device__ __forceinline__ T ld_stream(const T *p)
{
#if EXODUS_NT_LOAD
    return __builtin_nontemporal_load(p);
#else
    return *p;
#endif
}
template <class T> __device__ __forceinline__ void st_stream(T v, T *p)
{
#if EXODUS_NT_STORE
    __builtin_nontemporal_store(v, p);
#else
    *p = v;
#endif
}

__device__ __forceinline__ void wave_sync()
{
    // All lanes of a wave execute an instruction together and the LDS serves one wave's requests
    // in issue order; what remains is to stop the compiler from moving LDS accesses across here.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------------------------
// per-row helpers
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float spike_count(float v, float theta, unsigned cap)
{
    // count = v >= theta ? min(unsigned(v / theta), cap) : 0      (IEEE division, truncation)
    //
    // The quotient is only formed where it can exceed 2.  For theta > 0 and fp32 v, theta:
    //   v >= theta            <=>  RN(v/theta) >= 1
    //   v >= 2*theta (exact)  <=>  RN(v/theta) >= 2   (no fp32 number lies strictly between the
    //                              predecessor of 2*theta and 2*theta, and the rounding boundary
    //                              2*theta*(1 - 2^-25) falls inside that gap)
    // so counts up to 2 come from two comparisons and selects, without branches; the one (rare)
    // branch is taken from 2*theta on when the cap allows more than two spikes, and for thresholds
    // that are not positive.
    const float one = cap >= 1u ? 1.f : 0.f;
    const float two = cap >= 2u ? 2.f : one;
    const bool fire = v >= theta;
    const bool plain = theta > 0.f;
    const bool second = plain & (v >= __fadd_rn(theta, theta));
    float count = fire ? one : 0.f;
    count = second ? two : count;
    if (fire & (!plain | (second & (cap > 2u)))) {
        const unsigned k = static_cast<unsigned>(__fdiv_rn(v, theta));
        count = static_cast<float>(k < cap ? k : cap);
    }
    return count;
}

// Per-row constants of the in-kernel surrogate gradients.  Surrogate values enter gradients only
// (tolerance rtol 1e-4), never spike decisions, so divisions by per-row constants become
// multiplications by their reciprocals and exp() is the hardware exponential (relative error
// about |argument| * 6e-8).
struct SurrConst { float a, b, c; };

constexpr float NEG_LOG2_E = -1.44269504088896340736f;         // exp(-x) = exp2(x * NEG_LOG2_E)

template <int KIND>
__device__ __forceinline__ SurrConst surrogate_consts(float theta, float p0, float p1)
{
    SurrConst k;
    k.c = 0.f;
    if (KIND == EXODUS_SURR_SINGLE_EXP) {
        const float w = __fmul_rn(theta, p0);                 // p1/(theta p0) * exp(-|v - theta| / (theta p0))
        k.a = __fdiv_rn(NEG_LOG2_E, w);
        k.b = __fdiv_rn(p1, w);
    } else if (KIND == EXODUS_SURR_PERIODIC_EXP) {
        k.a = __fmul_rn(theta, 0.5f);                          // p1 * exp(-|u - theta/2| / p0) / theta
        k.b = __fdiv_rn(p1, theta);
        k.c = __fdiv_rn(1.f, theta);
    } else {
        k.a = __fsub_rn(theta, p0);                            // (v >= theta - p0) / theta
        k.b = __fdiv_rn(1.f, theta);
    }
    return k;
}

// u modulo theta for theta > 0 (result in [0, theta), as the floor-modulo of the Python definition gives it), without
// the library's fmodf, whose loop costs the backward kernels a third of their registers and half their speed.  The
// quotient comes from the reciprocal; floor(u * inv) is the true quotient or one off next to a multiple of theta, and
// the fused multiply-add takes q * theta away without rounding when q is right.  A second pass deals with quotients
// beyond 2^24 (q itself rounded), the two corrections with a quotient that was one off.  Exact whenever the first
// quotient is (then the second pass and the corrections change nothing); otherwise within an ulp of theta.
__device__ __forceinline__ float wrap_into_period(float u, float theta, float inv_theta)
{
    float r = u;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) r = __fmaf_rn(-floorf(__fmul_rn(r, inv_theta)), theta, r);
    if (r < 0.f) r = __fadd_rn(r, theta);
    if (r >= theta) r = __fsub_rn(r, theta);
    return r;
}

// exp() is the hardware's base-2 exponential with the change of base folded into the constants
// (results below the smallest normal number come out as 0, which no gradient notices).
template <int KIND>
__device__ __forceinline__ float surrogate(float v, float theta, float inv_p0, SurrConst k)
{
    if (KIND == EXODUS_SURR_SINGLE_EXP) {
        return k.b * __builtin_amdgcn_exp2f(fabsf(v - theta) * k.a);
    } else if (KIND == EXODUS_SURR_PERIODIC_EXP) {
        float u = v - k.a;
        if (v >= theta) u = wrap_into_period(u, theta, k.c);
        return k.b * __builtin_amdgcn_exp2f(fabsf(u - k.a) * (NEG_LOG2_E * inv_p0));
    } else {
        return v >= k.a ? k.b : 0.f;
    }
}

// Sum of many products for the per-row parameter gradients: fp32 fused multiply-adds within a
// tile (at most TT terms), folded into an fp64 total at every tile end.
struct TileSum {
    float part;
    double total;
    __device__ __forceinline__ void clear() { part = 0.f; total = 0.0; }
    __device__ __forceinline__ void add(float a, float b) { part = __fmaf_rn(a, b, part); }
    __device__ __forceinline__ void sub(float a, float b) { part = __fmaf_rn(-a, b, part); }
    __device__ __forceinline__ void fold() { total += static_cast<double>(part); part = 0.f; }
};

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace
