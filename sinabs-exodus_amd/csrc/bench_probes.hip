// Streaming probes for bench.py -- a library of its own (libexodus_bench_probes.so), not part of
// libexodus_hip.so and not declared in its header.  They show what the memory system gives a kernel
// that does nothing but move floats, flat (consecutive addresses per block): bench.py --ceilings
// puts these rates next to those of the recurrence kernels, and counter runs use the copy as a
// kernel of exactly known traffic to scale readings by.
//
//   exodus_probe_stream(dst, a, b, n, stream)   dst[i] = a[i] (b == NULL) or a[i] + b[i]
//   exodus_probe_read(a, n, stream)             read n floats, write nothing
//   exodus_probe_write(dst, n, stream)          write n zeros
// n floats, a multiple of 4; pointers 16-byte aligned; the same non-temporal 16-byte accesses the
// recurrence kernels use.  Return value: 0 or a hipError_t.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "exodus_common.hpp"

namespace {

constexpr int PROBE_PER_THREAD = 4;                            // 16-byte chunks per thread

template <bool TWO_INPUTS>
__global__ void __launch_bounds__(256) probe_stream(f32x4 *__restrict__ dst, const f32x4 *__restrict__ a,
                                                    const f32x4 *__restrict__ b, const int64_t n_chunks)
{
    const int64_t base = (static_cast<int64_t>(blockIdx.x) * PROBE_PER_THREAD) * 256 + threadIdx.x;
    f32x4 va[PROBE_PER_THREAD], vb[PROBE_PER_THREAD];
#pragma unroll
    for (int k = 0; k < PROBE_PER_THREAD; ++k) {
        const int64_t i = base + k * 256;
        if (i < n_chunks) {
            va[k] = ld_stream(a + i);
            if (TWO_INPUTS) vb[k] = ld_stream(b + i);
        }
    }
#pragma unroll
    for (int k = 0; k < PROBE_PER_THREAD; ++k) {
        const int64_t i = base + k * 256;
        if (i < n_chunks) st_stream(TWO_INPUTS ? va[k] + vb[k] : va[k], dst + i);
    }
}

// one direction only: READ loads and hands every value to an empty asm statement (so the loads stay
// although nothing is done with them), !READ writes zeros
template <bool READ>
__global__ void __launch_bounds__(256) probe_one_way(f32x4 *__restrict__ dst, const f32x4 *__restrict__ a,
                                                     const int64_t n_chunks)
{
    const int64_t base = (static_cast<int64_t>(blockIdx.x) * PROBE_PER_THREAD) * 256 + threadIdx.x;
#pragma unroll
    for (int k = 0; k < PROBE_PER_THREAD; ++k) {
        const int64_t i = base + k * 256;
        if (i < n_chunks) {
            if (READ) {
                const f32x4 v = ld_stream(a + i);
                asm volatile("" : : "v"(v));
            } else {
                st_stream(f32x4{0.f, 0.f, 0.f, 0.f}, dst + i);
            }
        }
    }
}

}  // namespace

extern "C" {

#define EXODUS_API __attribute__((visibility("default")))

EXODUS_API int exodus_probe_stream(float *dst, const float *a, const float *b, int64_t n, void *stream)
{
    if (n < 0 || (n % 4) != 0 || !dst || !a) return hipErrorInvalidValue;
    for (const void *q : {static_cast<const void *>(dst), static_cast<const void *>(a), static_cast<const void *>(b)})
        if (reinterpret_cast<uintptr_t>(q) & 15u) return hipErrorInvalidValue;
    if (n == 0) return hipSuccess;
    const int64_t n_chunks = n / 4;
    const int64_t blocks = (n_chunks + 256 * PROBE_PER_THREAD - 1) / (256 * PROBE_PER_THREAD);
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (b)
        hipLaunchKernelGGL((probe_stream<true>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s,
                           reinterpret_cast<f32x4 *>(dst), reinterpret_cast<const f32x4 *>(a),
                           reinterpret_cast<const f32x4 *>(b), n_chunks);
    else
        hipLaunchKernelGGL((probe_stream<false>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s,
                           reinterpret_cast<f32x4 *>(dst), reinterpret_cast<const f32x4 *>(a),
                           static_cast<const f32x4 *>(nullptr), n_chunks);
    return static_cast<int>(hipGetLastError());
}

EXODUS_API int exodus_probe_read(const float *a, int64_t n, void *stream)
{
    if (n < 0 || (n % 4) != 0 || !a || (reinterpret_cast<uintptr_t>(a) & 15u)) return hipErrorInvalidValue;
    if (n == 0) return hipSuccess;
    const int64_t n_chunks = n / 4;
    const int64_t blocks = (n_chunks + 256 * PROBE_PER_THREAD - 1) / (256 * PROBE_PER_THREAD);
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((probe_one_way<true>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<f32x4 *>(nullptr),
                       reinterpret_cast<const f32x4 *>(a), n_chunks);
    return static_cast<int>(hipGetLastError());
}

EXODUS_API int exodus_probe_write(float *dst, int64_t n, void *stream)
{
    if (n < 0 || (n % 4) != 0 || !dst || (reinterpret_cast<uintptr_t>(dst) & 15u)) return hipErrorInvalidValue;
    if (n == 0) return hipSuccess;
    const int64_t n_chunks = n / 4;
    const int64_t blocks = (n_chunks + 256 * PROBE_PER_THREAD - 1) / (256 * PROBE_PER_THREAD);
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((probe_one_way<false>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), reinterpret_cast<f32x4 *>(dst),
                       static_cast<const f32x4 *>(nullptr), n_chunks);
    return static_cast<int>(hipGetLastError());
}

}  // extern "C"
