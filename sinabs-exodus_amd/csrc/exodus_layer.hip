// Layer-layout kernels of libexodus_hip.so: the spiking layer computed directly on the layer's own
// (batch, time, neurons) tensors, neurons contiguous.
//
// In this layout the time recurrence of a neuron walks memory with stride `neurons`, and
// adjacent lanes hold adjacent neurons: every wave-wide load or store is one contiguous segment,
// so nothing has to be transposed (neither by torch before the kernel, as the (rows, time)
// Functions need, nor through LDS).  One lane owns NPL adjacent neurons of one batch element.
//
// The forward pass writes only what the layer hands out -- the spike raster and the final
// states -- plus one checkpoint of (post-reset potential, synaptic current) every CKPT steps.
// The backward pass reads the input again, rebuilds each CKPT-step chunk of membrane potential
// and synaptic current in registers from its checkpoint (same operations, same order, hence the
// same bits as the forward pass produced) and then walks the chunk in reverse.  Per
// neuron-timestep this moves 8 B forward (x in, spikes out) and 12 B backward (grad_spikes and x
// in, grad_x out) plus 16 B per 32 steps of checkpoints, instead of the 32 B of a forward that
// stores v_mem and i_syn for the backward to read.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <initializer_list>
#include <mutex>
#include <type_traits>

#include "exodus_common.hpp"

namespace {

#ifndef EXODUS_LAYER_FWD_UNROLL
#define EXODUS_LAYER_FWD_UNROLL 16
#endif
#ifndef EXODUS_LAYER_BLOCK
#define EXODUS_LAYER_BLOCK 256        // lanes per block of the kernels that hold several neurons per lane
#endif
#ifndef EXODUS_LIF_FWD_WIDEST
#define EXODUS_LIF_FWD_WIDEST 2       // most neurons per lane of the spiking forward kernel
#endif
#ifndef EXODUS_LAYER_BWD_BLOCK
#define EXODUS_LAYER_BWD_BLOCK 256    // lanes per block of the spiking backward kernel (one neuron per lane)
#endif
#ifndef EXODUS_LEAKY_WAVES
#define EXODUS_LEAKY_WAVES 8          // waves per CU the leaky kernels want before a lane takes more than one neuron
#endif
#ifndef EXODUS_LAYER_CKPT
#define EXODUS_LAYER_CKPT 32          // steps between checkpoints (a multiple of 2 * EXODUS_LAYER_FWD_UNROLL)
#endif
#ifndef EXODUS_WHOLE_NEURONS
#define EXODUS_WHOLE_NEURONS 16       // neurons per step must be a multiple of this for the non-temporal kernel instances
#endif
#ifndef EXODUS_LAYER_BWD_WAVES
#define EXODUS_LAYER_BWD_WAVES 3      // resident waves per SIMD the backward kernel is compiled for
#endif
#ifndef EXODUS_LAYER_BWD_WAVES_G1
#define EXODUS_LAYER_BWD_WAVES_G1 3   // ... and its instances that stream one tensor less (one gradient value for all): a
                                      // fourth wave fits them only with spills and measures no faster
#endif
constexpr int CKPT = EXODUS_LAYER_CKPT;               // steps between checkpoints = length of a backward chunk
constexpr int FWD_UNROLL = EXODUS_LAYER_FWD_UNROLL;  // forward steps per software-pipeline stage (divides CKPT)
constexpr int BLOCK = EXODUS_LAYER_BLOCK;
constexpr int BWD_BLOCK = EXODUS_LAYER_BWD_BLOCK;

struct LayerConsts {
    const float *v_init, *i_init, *alpha_mem, *alpha_syn, *c, *theta, *theta_low;
    int apply_low, decay_early, norm_input;
    unsigned cap;
    int rec_pre;        // the potential record holds the value before the reset instead of after it
};

template <int NPL> struct Vec;
typedef float f32x2 __attribute__((ext_vector_type(2)));
template <> struct Vec<1> { typedef float type; };
template <> struct Vec<2> { typedef f32x2 type; };
template <> struct Vec<4> { typedef f32x4 type; };

template <int NPL> __device__ __forceinline__ float lane_get(const typename Vec<NPL>::type &v, int e);
template <> __device__ __forceinline__ float lane_get<1>(const float &v, int) { return v; }
template <> __device__ __forceinline__ float lane_get<2>(const f32x2 &v, int e) { return v[e]; }
template <> __device__ __forceinline__ float lane_get<4>(const f32x4 &v, int e) { return v[e]; }
template <int NPL> __device__ __forceinline__ void lane_put(typename Vec<NPL>::type &v, int e, float x);
template <> __device__ __forceinline__ void lane_put<1>(float &v, int, float x) { v = x; }
template <> __device__ __forceinline__ void lane_put<2>(f32x2 &v, int e, float x) { v[e] = x; }
template <> __device__ __forceinline__ void lane_put<4>(f32x4 &v, int e, float x) { v[e] = x; }

// ---------------------------------------------------------------------------------------------
// memory access: raw buffer instructions
// ---------------------------------------------------------------------------------------------
// Every (batch, time, neurons) access of a block has the form
//     block-uniform base (SGPR pair inside a buffer resource)  +  step * neurons * 4 (SGPR)
//                                                              +  lane offset (one VGPR, loop-invariant)
// which is exactly what a buffer instruction adds up by itself, so no access needs vector
// arithmetic or 64-bit address registers.  num_records is set to the maximum: every access is
// guarded by the code, not by the hardware range check.
typedef __amdgpu_buffer_rsrc_t Rsrc;
// Cache hint of the streamed accesses (bit 1 = non-temporal).  Streaming data that nobody reads twice
// is marked non-temporal, which measures a few percent faster; but when a step's neurons do not start
// and end on 64-byte sectors (neuron count not a multiple of 16, or a view at an odd offset) neighbouring
// waves and blocks share sectors, and a non-temporal line is dropped before the neighbour gets to it:
// reads from memory grow by a third and partial writes appear.  Such layers use NT = false.
// All kernels put a workgroup barrier in front of every group of loads (the waves of a block share no
// data; the barrier only keeps them at the same step): waves that ask for the two halves of a line at
// the same moment are served by one fetch, waves that have drifted apart are not (+10-15 % where lines
// are shared), and neighbouring pieces requested together also suit the memory better when nothing is
// shared (+1-2 %).
template <bool NT> struct Aux {
    static constexpr int load = (NT && EXODUS_NT_LOAD) ? 2 : 0;
    static constexpr int store = (NT && EXODUS_NT_STORE) ? 2 : 0;
};

__device__ __forceinline__ Rsrc make_rsrc(const float *base)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(base), 0, -1, 0x00020000);
}

typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <int NPL, bool NT> struct BufIO;
template <bool NT> struct BufIO<1, NT> {
    static __device__ __forceinline__ float load(Rsrc r, unsigned voff, unsigned soff)
    {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, Aux<NT>::load));
    }
    static __device__ __forceinline__ void store(float v, Rsrc r, unsigned voff, unsigned soff)
    {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, voff, soff, Aux<NT>::store);
    }
};
template <bool NT> struct BufIO<2, NT> {
    static __device__ __forceinline__ f32x2 load(Rsrc r, unsigned voff, unsigned soff)
    {
        return __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, Aux<NT>::load));
    }
    static __device__ __forceinline__ void store(f32x2 v, Rsrc r, unsigned voff, unsigned soff)
    {
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), r, voff, soff, Aux<NT>::store);
    }
};
template <bool NT> struct BufIO<4, NT> {
    static __device__ __forceinline__ f32x4 load(Rsrc r, unsigned voff, unsigned soff)
    {
        return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, Aux<NT>::load));
    }
    // A 16-byte store takes more than one pass to read its data registers.  The compiler keeps the
    // next instruction from overwriting them only when the store has no SGPR offset; with one, a
    // vector instruction that rewrites the data right behind the store corrupted the last lanes of
    // each group of 16 on gfx950 (seen as sporadic wrong outputs when two blocks shared a compute
    // unit).  So the step offset travels in the vector offset here and the scalar offset stays 0, and a
    // short wait that reads the data keeps every writer away until the store has taken it.
    static __device__ __forceinline__ void store(f32x4 v, Rsrc r, unsigned voff, unsigned soff)
    {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, voff + soff, 0, Aux<NT>::store);
        asm volatile("s_nop 1" : : "v"(v));                    // the data registers stay untouched two more cycles
    }
};

// ---------------------------------------------------------------------------------------------
// one neuron
// ---------------------------------------------------------------------------------------------
// Per-neuron constants and running state.  The layer's options are folded into the constants so
// that the step itself has no option-dependent code: a factor that an option switches off is 1
// (multiplying by 1 is exact), a bound that is switched off is an infinity.
struct Neuron {
    float am, as;       // decay factors of membrane and synapse
    float k;            // factor on the current entering the membrane: 1 - alpha_mem (norm_input) or 1
    float xs;           // factor on the input entering the synapse: alpha_syn (decay_early) or 1
    float c, th;        // subtract value, threshold
    float c2;           // 2 * subtract value (exact), what two spikes take away
    float th2;          // 2 * threshold: from here on a second spike (+inf where th <= 0)
    float thd;          // from here on the spike count needs the quotient v / th (+inf if never)
    float lo;           // lower bound of the potential, -inf without one
    float vpost, i;     // potential after the reset of the previous step, synaptic current
};

// spike-count cap as the kernels use it (block-uniform)
struct Cap {
    float one, two;     // min(cap, 1), min(cap, 2)
    unsigned cap;
};

// CAPK: 1 = at most one spike per step, 2 = at most two, 0 = any other cap (none, 0, >= 3)
template <bool SYN, int CAPK>
__device__ __forceinline__ void neuron_load(Neuron &n, const LayerConsts &p, int64_t row)
{
    n.am = p.alpha_mem[row];
    n.as = SYN ? p.alpha_syn[row] : 0.f;
    n.k = p.norm_input ? __fsub_rn(1.0f, n.am) : 1.0f;
    n.xs = (SYN && p.decay_early) ? n.as : 1.0f;
    n.c = p.c[row];
    n.c2 = __fadd_rn(n.c, n.c);
    n.th = p.theta[row];
    // For th > 0:  v >= th <=> RN(v/th) >= 1  and  v >= 2 th <=> RN(v/th) >= 2  (2 th is exact and no
    // float lies between its predecessor and the rounding boundary of the quotient), so counts up to
    // 2 need no division.  Everything else -- more than two spikes, or a threshold that is not
    // positive -- takes the quotient.
    const bool plain = n.th > 0.f;
    n.th2 = plain ? __fadd_rn(n.th, n.th) : __builtin_inff();
    n.thd = plain ? (CAPK == 0 ? n.th2 : __builtin_inff()) : n.th;
    n.lo = p.apply_low ? p.theta_low[row] : -__builtin_inff();
}

// Advance synapse and membrane by one step, in the order the composed layer does it
// (input scaling, synapse, input normalisation, membrane, clamp):
//   xin = x * xs;  i = i * a_syn + xin   (SYN; otherwise i = x)
//   u = k * i;   v = vpost * a_mem + u;   v = max(v, lo)
// Returns the pre-reset potential v; n.i is advanced, n.vpost is left to the caller (it needs the
// spike count).
template <bool SYN>
__device__ __forceinline__ float neuron_advance(Neuron &n, float x)
{
    if (SYN) {
        const float xin = __fmul_rn(x, n.xs);
        n.i = __fadd_rn(__fmul_rn(n.i, n.as), xin);
    } else {
        n.i = x;
    }
    const float u = __fmul_rn(n.k, n.i);
    const float v = __fadd_rn(__fmul_rn(n.vpost, n.am), u);
    return v < n.lo ? n.lo : v;
}

// count = v >= th ? min(unsigned(v / th), cap) : 0   (IEEE division, truncation), in two parts:
// the count by comparisons, and the quotient for the rare potentials at or above n.thd.
template <int CAPK>
__device__ __forceinline__ float count_by_compare(float v, const Neuron &n, const Cap &cc)
{
    const float count = v >= n.th ? (CAPK == 0 ? cc.one : 1.f) : 0.f;
    if (CAPK == 1) return count;
    return v >= n.th2 ? (CAPK == 0 ? cc.two : 2.f) : count;
}

__device__ __forceinline__ float count_by_quotient(float v, const Neuron &n, const Cap &cc)
{
    const unsigned q = static_cast<unsigned>(__fdiv_rn(v, n.th));
    return static_cast<float>(q < cc.cap ? q : cc.cap);
}

template <int CAPK>
__device__ __forceinline__ float spike_count_fast(float v, const Neuron &n, const Cap &cc)
{
    float count = count_by_compare<CAPK>(v, n, cc);
    if (v >= n.thd) count = count_by_quotient(v, n, cc);
    return count;
}

// count * c, what the reset subtracts from the potential, for callers that do not need the count itself: with a cap
// of one or two spikes the product is 0, c or 2c (all exact), picked by the comparisons that would have picked the
// count -- the same bits as the multiplication, one instruction less.
template <int CAPK>
__device__ __forceinline__ float reset_amount(float v, const Neuron &n, const Cap &cc)
{
    if (CAPK == 0) return __fmul_rn(spike_count_fast<0>(v, n, cc), n.c);
    float taken = v >= n.th ? n.c : 0.f;
    if (CAPK == 2) taken = v >= n.th2 ? n.c2 : taken;
    if (v >= n.thd) taken = __fmul_rn(count_by_quotient(v, n, cc), n.c);   // thresholds that are not positive
    return taken;
}

// ---------------------------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------------------------
// Time is walked in blocks of CKPT steps = an even number of stages of FWD_UNROLL steps.  Two
// register buffers of one stage each alternate: while one is consumed the loads of the other are in flight.  Every fetch issues
// the same number of loads (past the end it re-reads the last step), so the number of outstanding
// loads at each wait is a compile-time constant.  A last, partial block runs through a guarded copy
// of the same code.
// OUT = false keeps only the checkpoints: no spike raster, no final states, no spike total (what a
// backward pass that was handed no checkpoints runs first).
template <bool SYN, int NPL, int CAPK, bool REC, bool NT, bool OUT = true>
__global__ void __launch_bounds__(BLOCK) layer_lif_forward(
    float *__restrict__ spikes, float *__restrict__ v_rec, float *__restrict__ i_rec, float *__restrict__ ckpt_v,
    float *__restrict__ ckpt_i, float *__restrict__ v_last, float *__restrict__ i_last, double *spike_sum,
    const float *__restrict__ x, const LayerConsts p, const int64_t blocks_per_batch, const int64_t T,
    const int64_t M)
{
    constexpr int STAGES = CKPT / FWD_UNROLL;                 // pipeline stages per checkpoint interval
    static_assert(STAGES * FWD_UNROLL == CKPT && STAGES % 2 == 0, "an even number of stages per checkpoint interval");
    typedef typename Vec<NPL>::type V;
    typedef BufIO<NPL, NT> IO;
    // A block works inside one batch element, so all bases are block-uniform.
    const int64_t b = blockIdx.x / blocks_per_batch;
    const int64_t m0 = static_cast<int64_t>(blockIdx.x - b * blocks_per_batch) * (BLOCK * NPL);
    const unsigned lane_off = threadIdx.x * NPL;
    const int64_t first = b * M + m0 + lane_off;              // first neuron (row) of this lane
    // Lanes past the end of the layer (only the last block of a batch element has any) walk the same
    // loops and meet every barrier, but touch no memory and compute nothing: all work sits behind
    // `active`, all barriers in front of it.
    const bool active = m0 + lane_off < M;
    double my_spikes = 0.0;
    {
        const int64_t n_ck = (T + CKPT - 1) / CKPT;
        const float *xp = x + (b * T) * M + m0;
        float *sp = spikes + (b * T) * M + m0;
        float *vrp = REC && v_rec ? v_rec + (b * T) * M + m0 : nullptr;
        float *irp = REC && i_rec ? i_rec + (b * T) * M + m0 : nullptr;
        float *cvp = ckpt_v ? ckpt_v + (b * n_ck) * M + m0 : nullptr;
        float *cip = (SYN && ckpt_i) ? ckpt_i + (b * n_ck) * M + m0 : nullptr;
        const unsigned voff = lane_off * 4u;                  // byte offset of this lane within a step
        const unsigned step_bytes = static_cast<unsigned>(M) * 4u;   // the host keeps CKPT * M * 4 below 2^32

        Cap cc;
        cc.cap = p.cap;
        cc.one = p.cap >= 1u ? 1.f : 0.f;
        cc.two = p.cap >= 2u ? 2.f : cc.one;
        Neuron nr[NPL] = {};
        if (active) {
#pragma unroll
            for (int e = 0; e < NPL; ++e) {
                neuron_load<SYN, CAPK>(nr[e], p, first + e);
                nr[e].vpost = p.v_init[first + e];
                nr[e].i = SYN ? p.i_init[first + e] : 0.f;
            }
        }

        V bufa[FWD_UNROLL], bufb[FWD_UNROLL];
        // FWD_UNROLL steps from t0; steps past the end re-read the last step (also when t0 itself lies
        // past the end), so every call issues exactly FWD_UNROLL loads
        auto fetch = [&](V(&dst)[FWD_UNROLL], int64_t t0) {
            __syncthreads();                                   // keeps the block's waves at the same step
            if (!active) return;
            if (t0 + FWD_UNROLL <= T) {
                const Rsrc r = make_rsrc(xp + t0 * M);
#pragma unroll
                for (int u = 0; u < FWD_UNROLL; ++u) dst[u] = IO::load(r, voff, u * step_bytes);
            } else {
                const int64_t tc = t0 < T ? t0 : T - 1;
                const Rsrc r = make_rsrc(xp + tc * M);
                const unsigned last = static_cast<unsigned>(T - 1 - tc);
#pragma unroll
                for (int u = 0; u < FWD_UNROLL; ++u) dst[u] = IO::load(r, voff, (u < last ? u : last) * step_bytes);
            }
        };
        float part = 0.f;                                     // spike count since the last checkpoint (exact in fp32)
        auto checkpoint = [&](int64_t j) {
            if (!active) return;
            if (cvp) {
                V cv, ci;
#pragma unroll
                for (int e = 0; e < NPL; ++e) {
                    lane_put<NPL>(cv, e, nr[e].vpost);
                    lane_put<NPL>(ci, e, nr[e].i);
                }
                // checkpoints follow the hint of the other streamed tensors (their rows share lines alike)
                V *cvq = reinterpret_cast<V *>(cvp + j * M + lane_off);
                if (NT) st_stream(cv, cvq); else *cvq = cv;
                if (cip) {
                    V *ciq = reinterpret_cast<V *>(cip + j * M + lane_off);
                    if (NT) st_stream(ci, ciq); else *ciq = ci;
                }
            }
            my_spikes += static_cast<double>(part);
            part = 0.f;
        };
        auto compute = [&](const V(&buf)[FWD_UNROLL], int64_t t0, auto guard) {
            constexpr bool GUARD = decltype(guard)::value;
            if (!active) return;
            const Rsrc rs = make_rsrc(sp + t0 * M);
            const Rsrc rv = make_rsrc(REC ? vrp + t0 * M : nullptr);
            const Rsrc ri = make_rsrc(REC ? irp + t0 * M : nullptr);
#pragma unroll
            for (int u = 0; u < FWD_UNROLL; ++u) {
                if (!GUARD || t0 + u < T) {
                    V s, vr, ir;
                    float v[NPL], count[NPL];
                    bool rare = false;                        // one branch per step for all neurons of the lane
#pragma unroll
                    for (int e = 0; e < NPL; ++e) {
                        v[e] = neuron_advance<SYN>(nr[e], lane_get<NPL>(buf[u], e));
                        count[e] = count_by_compare<CAPK>(v[e], nr[e], cc);
                        rare = rare | (v[e] >= nr[e].thd);
                    }
                    if (rare) {
#pragma unroll
                        for (int e = 0; e < NPL; ++e)
                            if (v[e] >= nr[e].thd) count[e] = count_by_quotient(v[e], nr[e], cc);
                    }
#pragma unroll
                    for (int e = 0; e < NPL; ++e) {
                        nr[e].vpost = __fsub_rn(v[e], __fmul_rn(count[e], nr[e].c));
                        part += count[e];
                        lane_put<NPL>(s, e, count[e]);
                        lane_put<NPL>(vr, e, (REC && p.rec_pre) ? v[e] : nr[e].vpost);
                        lane_put<NPL>(ir, e, nr[e].i);
                    }
                    if (OUT) IO::store(s, rs, voff, u * step_bytes);
                    if (REC && vrp) IO::store(vr, rv, voff, u * step_bytes);
                    if (REC && irp) IO::store(ir, ri, voff, u * step_bytes);
                }
            }
        };

        const int64_t n_full = T / CKPT;                      // blocks that lie inside the sequence
        fetch(bufa, 0);
        for (int64_t j = 0; j < n_full; ++j) {
            const int64_t t0 = j * CKPT;
            checkpoint(j);
#pragma unroll
            for (int s = 0; s < STAGES; s += 2) {
                fetch(bufb, t0 + (s + 1) * FWD_UNROLL);
                compute(bufa, t0 + s * FWD_UNROLL, std::false_type{});
                fetch(bufa, t0 + (s + 2) * FWD_UNROLL);       // next pair, next block, or the start of the partial block
                compute(bufb, t0 + (s + 1) * FWD_UNROLL, std::false_type{});
            }
        }
        if (n_full * CKPT < T) {                              // partial block: bufa holds its first stage
            checkpoint(n_full);
            for (int64_t t0 = n_full * CKPT; t0 < T; t0 += FWD_UNROLL) {
                if (t0 > n_full * CKPT) fetch(bufa, t0);
                compute(bufa, t0, std::true_type{});
            }
        }
        my_spikes += static_cast<double>(part);
        if (active && OUT) {
#pragma unroll
            for (int e = 0; e < NPL; ++e) {
                v_last[first + e] = nr[e].vpost;
                if (SYN && i_last) i_last[first + e] = nr[e].i;
            }
        }
    }
    if (OUT && spike_sum) {
        // wave reduction, then one atomic per wave
#pragma unroll
        for (int off = WAVE / 2; off > 0; off >>= 1) my_spikes += __shfl_xor(my_spikes, off, WAVE);
        if ((threadIdx.x & (WAVE - 1)) == 0 && my_spikes != 0.0) atomicAdd(spike_sum, my_spikes);
    }
}

// ---------------------------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------------------------
// With lambda_t = dL/du_t (membrane adjoint) and mu_t = dL/di_t (synapse adjoint):
//   g_t      = s_t * grad_spikes_t              (at the last step the gradients of the final states
//                                                join in: see below)
//   lambda_t = nc_t (g_t + (a_mem - a_mem c s_t) lambda_{t+1})
//   mu_t     = a_syn mu_{t+1} + k lambda_t,     k = norm_input ? 1 - a_mem : 1
//   grad_x_t = decay_early ? a_syn mu_t : mu_t  (no synapse: grad_x_t = k lambda_t)
//   grad_alpha_mem = sum_t lambda_t vpost_{t-1} - (norm_input ? sum_t lambda_t i_t : 0)
//   grad_alpha_syn = decay_early ? (sum_t mu_t i_t) / a_syn : sum_t mu_t i_{t-1}
//   grad_v_init = a_mem lambda_0,  grad_i_init = a_syn mu_0
// The final potential handed out by the forward is vpost_{T-1} = v_{T-1} - c count_{T-1}; a gradient
// gv on it reaches v_{T-1} directly and the spike count with weight -c, a gradient on the final
// synaptic current adds to mu_{T-1}.
// KIND == EXODUS_SURR_TENSOR reads the surrogate derivative of every step from `surr` (a third
// streamed tensor, whose register buffer costs the kernel one wave per SIMD); the other kinds
// evaluate it from the rebuilt potential and ignore `surr`.
// EXTRA: gradients also arrive at the per-step state records of the forward (grad_v_rec on the potential
// after each reset, with synapse grad_i_rec on each synaptic current): two more streamed inputs.
// GO1: the gradient of the spikes is one value for every neuron and step (the gradient of a sum of the
// output, which autograd hands over as a broadcast scalar): `grad_spikes` then points at that one float and the
// kernel streams one tensor less (8 instead of 12 bytes per neuron-timestep).
template <bool SYN, int KIND, int CAPK, bool NT, bool EXTRA, bool GO1 = false>
__global__ void __launch_bounds__(BWD_BLOCK)
    __attribute__((amdgpu_waves_per_eu(
        (KIND == EXODUS_SURR_TENSOR || EXTRA) ? 2 : (GO1 ? EXODUS_LAYER_BWD_WAVES_G1 : EXODUS_LAYER_BWD_WAVES),
        (KIND == EXODUS_SURR_TENSOR || EXTRA) ? 2 : (GO1 ? EXODUS_LAYER_BWD_WAVES_G1 : EXODUS_LAYER_BWD_WAVES))))
layer_lif_backward(
    float *__restrict__ grad_x, float *__restrict__ alpha_mem_grad, float *__restrict__ alpha_syn_grad,
    float *__restrict__ v_init_grad, float *__restrict__ i_init_grad, const float *__restrict__ grad_spikes,
    const float *__restrict__ grad_v_last, const float *__restrict__ grad_i_last, const float *__restrict__ x,
    const float *__restrict__ surr, const float *__restrict__ grad_v_rec, const float *__restrict__ grad_i_rec,
    const float *__restrict__ ckpt_v, const float *__restrict__ ckpt_i, const LayerConsts p, const float p0,
    const float p1, const float inv_p0, const int64_t blocks_per_batch, const int64_t T, const int64_t M)
{
    typedef BufIO<1, NT> IO;
    const int64_t b = blockIdx.x / blocks_per_batch;
    const int64_t m0 = static_cast<int64_t>(blockIdx.x - b * blocks_per_batch) * BWD_BLOCK;
    const unsigned lane_off = threadIdx.x;
    // lanes past the end of the layer walk the same loops and meet every barrier, but all memory
    // accesses and all arithmetic sit behind `active`
    const bool active = m0 + lane_off < M;
    const int64_t row = b * M + m0 + lane_off;
    const int64_t n_ck = (T + CKPT - 1) / CKPT;
    // block-uniform bases; lane and step offsets are added by the buffer instructions
    const float *xp = x + (b * T) * M + m0;
    const float *gp = GO1 ? nullptr : grad_spikes + (b * T) * M + m0;
    const float g1 = GO1 ? grad_spikes[0] : 0.f;
    float *op = grad_x + (b * T) * M + m0;
    constexpr bool FROM_TENSOR = KIND == EXODUS_SURR_TENSOR;
    const float *srp = FROM_TENSOR ? surr + (b * T) * M + m0 : nullptr;
    const float *qvp = EXTRA ? grad_v_rec + (b * T) * M + m0 : nullptr;
    const float *qip = (EXTRA && SYN) ? grad_i_rec + (b * T) * M + m0 : nullptr;
    const float *cvp = ckpt_v + (b * n_ck) * M + m0;
    const float *cip = SYN ? ckpt_i + (b * n_ck) * M + m0 : nullptr;
    const unsigned voff = lane_off * 4u;
    const unsigned step_bytes = static_cast<unsigned>(M) * 4u;

    Cap cc;
    cc.cap = p.cap;
    cc.one = p.cap >= 1u ? 1.f : 0.f;
    cc.two = p.cap >= 2u ? 2.f : cc.one;
    Neuron nr = {};
    if (active) neuron_load<SYN, CAPK>(nr, p, row);
    const float xg = (SYN && p.decay_early) ? nr.as : 1.0f;   // factor between mu and grad_x
    const bool pair_new = p.decay_early != 0;                  // the synapse sum pairs i_t with mu_t (else mu_{t+1})
    const SurrConst sk = surrogate_consts<KIND>(nr.th, p0, p1);

    // Running adjoints.  Besides lambda_{t+1} and mu_{t+1} themselves the walk carries what reaches the
    // step below them, h = a_mem lambda_{t+1} and hm = a_syn mu_{t+1}: a gradient arriving at the final
    // states is then nothing but their initial value (the final potential is vpost_{T-1}, whose
    // gradient enters v_{T-1} with the same factor 1 - c s_{T-1} as a_mem lambda_T would), and no step
    // needs a special case.
    float lam = 0.f, mu = 0.f;
    float h = (active && grad_v_last) ? grad_v_last[row] : 0.f;
    float hm = (active && SYN && grad_i_last) ? grad_i_last[row] : 0.f;
    TileSum acc_m, acc_n, acc_s;                               // sums of lambda_{t+1} vpost_t, lambda_t i_t, mu i
    acc_m.clear();
    acc_n.clear();
    acc_s.clear();

    // One block of CKPT steps: load, rebuild forward from the checkpoint, walk in reverse, store.
    // GUARD = the block may end before CKPT steps (only the newest block of a sequence can).
    auto block = [&](const int64_t j, auto guard) {
        constexpr bool GUARD = decltype(guard)::value;
        const int64_t t0 = j * CKPT;
        const int len = GUARD ? static_cast<int>(T - t0) : CKPT;
        float xr[CKPT], gr[GO1 ? 1 : CKPT], vr[CKPT], sr[FROM_TENSOR ? CKPT : 1];   // (GO1: results go where the inputs were)
        float qv[EXTRA ? CKPT : 1], qi[(EXTRA && SYN) ? CKPT : 1];
        __syncthreads();                                   // keeps the block's waves at the same step
        if (!active) return;
        {
            // always CKPT loads per tensor (steps past the end re-read the last step): a constant number
            // of loads in flight lets each use wait for its own load only
            const Rsrc rx = make_rsrc(xp + t0 * M), rg = make_rsrc(GO1 ? nullptr : gp + t0 * M);
            const Rsrc rs = make_rsrc(FROM_TENSOR ? srp + t0 * M : nullptr);
            const Rsrc rqv = make_rsrc(EXTRA ? qvp + t0 * M : nullptr);
            const Rsrc rqi = make_rsrc((EXTRA && SYN) ? qip + t0 * M : nullptr);
            const unsigned last = static_cast<unsigned>(len - 1);
#pragma unroll
            for (int k = 0; k < CKPT; ++k) {
                const unsigned so = (GUARD ? (k < last ? k : last) : k) * step_bytes;
                xr[k] = IO::load(rx, voff, so);
                if (!GO1) gr[GO1 ? 0 : k] = IO::load(rg, voff, so);
                if (FROM_TENSOR) sr[k] = IO::load(rs, voff, so);
                if (EXTRA) qv[k] = IO::load(rqv, voff, so);
                if (EXTRA && SYN) qi[k] = IO::load(rqi, voff, so);
            }
        }
        nr.vpost = NT ? ld_stream(cvp + j * M + lane_off) : cvp[j * M + lane_off];
        nr.i = SYN ? (NT ? ld_stream(cip + j * M + lane_off) : cip[j * M + lane_off]) : 0.f;

        // rebuild the block: vr[k] = pre-reset potential, xr[k] = synaptic current (the value that
        // was normalised and fed to the membrane; without synapse that is the input itself)
#pragma unroll
        for (int k = 0; k < CKPT; ++k)
            if (!GUARD || k < len) {
                const float v = neuron_advance<SYN>(nr, xr[k]);
                nr.vpost = __fsub_rn(v, reset_amount<CAPK>(v, nr, cc));
                vr[k] = v;
                xr[k] = nr.i;
            }

        // reverse walk
#pragma unroll
        for (int kq = 0; kq < CKPT; ++kq) {
            const int k = CKPT - 1 - kq;
            if (!GUARD || k < len) {
                float v = vr[k];
                const float cur_i = xr[k];
                // The longer surrogate is evaluated when its step is reached, not for all 32 steps ahead of the walk
                // (which the compiler otherwise does: 32 more live values, spilled to memory): the empty statement makes
                // this step's potential depend on the adjoint that the previous one has produced.
                if (KIND == EXODUS_SURR_PERIODIC_EXP) asm volatile("" : "+v"(v) : "v"(h));
                const float sg = FROM_TENSOR ? sr[FROM_TENSOR ? k : 0] : surrogate<KIND>(v, nr.th, inv_p0, sk);
                const float vpost = __fsub_rn(v, reset_amount<CAPK>(v, nr, cc));
                acc_m.add(lam, vpost);                          // lambda_{t+1} * vpost_t
                const float through = __fsub_rn(1.0f, __fmul_rn(nr.c, sg));   // d vpost_t / d v_t
                // a gradient on the recorded vpost_t joins what the next step sends down to vpost_t
                const float below = EXTRA ? __fadd_rn(h, qv[EXTRA ? k : 0]) : h;
                const float l = __fadd_rn(__fmul_rn(sg, GO1 ? g1 : gr[GO1 ? 0 : k]), __fmul_rn(through, below));
                lam = v > nr.lo ? l : 0.f;                      // clamped (or NaN) steps pass nothing on
                h = __fmul_rn(nr.am, lam);
                acc_n.add(lam, cur_i);                          // lambda_t * i_t
                const float du = __fmul_rn(lam, nr.k);
                if (SYN) {
                    const float mu_next = mu;
                    mu = __fadd_rn(hm, du);
                    if (EXTRA) mu = __fadd_rn(mu, qi[(EXTRA && SYN) ? k : 0]);
                    hm = __fmul_rn(nr.as, mu);
                    acc_s.add(pair_new ? mu : mu_next, cur_i);
                    (GO1 ? xr[k] : gr[GO1 ? 0 : k]) = __fmul_rn(mu, xg);
                } else {
                    (GO1 ? xr[k] : gr[GO1 ? 0 : k]) = du;
                }
            }
        }
        {
            const Rsrc ro = make_rsrc(op + t0 * M);
#pragma unroll
            for (int k = 0; k < CKPT; ++k)
                if (!GUARD || k < len) IO::store(GO1 ? xr[k] : gr[GO1 ? 0 : k], ro, voff, k * step_bytes);
        }
        acc_m.fold();
        acc_n.fold();
        acc_s.fold();
    };

    int64_t j = n_ck - 1;
    if (T - j * CKPT < CKPT) {
        block(j, std::true_type{});
        --j;
    }
    for (; j >= 0; --j) block(j, std::false_type{});

    if (!active) return;                                       // no barrier follows
    if (v_init_grad) v_init_grad[row] = h;
    if (SYN && i_init_grad) i_init_grad[row] = hm;
    if (alpha_mem_grad) {
        acc_m.add(lam, p.v_init[row]);
        acc_m.fold();
        alpha_mem_grad[row] = static_cast<float>(p.norm_input ? acc_m.total - acc_n.total : acc_m.total);
    }
    if (SYN && alpha_syn_grad) {
        if (p.decay_early) {
            acc_s.total = acc_s.total / static_cast<double>(nr.as);
        } else {
            acc_s.add(mu, p.i_init[row]);
            acc_s.fold();
        }
        alpha_syn_grad[row] = static_cast<float>(acc_s.total);
    }
}

// ---------------------------------------------------------------------------------------------
// non-spiking leaky integrator layer (ExpLeak) on the layer layout
// ---------------------------------------------------------------------------------------------
struct LeakyConsts {
    const float *v_init, *alpha;
    int decay_early, norm_input;
};

#ifndef EXODUS_LEAKY_UNROLL
#define EXODUS_LEAKY_UNROLL 8
#endif
constexpr int LEAKY_UNROLL = EXODUS_LEAKY_UNROLL;

// Both leaky kernels walk time in pairs of stages of LEAKY_UNROLL steps with two register buffers:
// while one stage is consumed, the loads of the other are in flight, and because every fetch
// issues the same number of loads, each wait covers only the loads it needs.  The steps that do
// not fill a pair (fewer than 2 * LEAKY_UNROLL) are done one at a time.

// xin = norm_input ? (1 - alpha) * x : x;  xin = decay_early ? xin * alpha : xin;  v = v * alpha + xin
// (the two input factors are applied as kn = 1 - alpha or 1 and kd = alpha or 1: a factor of 1 is exact)
template <int NPL, bool NT>
__global__ void __launch_bounds__(BLOCK) layer_leaky_forward(float *__restrict__ out, float *__restrict__ v_last,
                                                             double *out_sum, const float *__restrict__ x,
                                                             const LeakyConsts p,
                                                             const int64_t blocks_per_batch, const int64_t T,
                                                             const int64_t M)
{
    typedef typename Vec<NPL>::type V;
    typedef BufIO<NPL, NT> IO;
    constexpr int U = LEAKY_UNROLL;
    const int64_t b = blockIdx.x / blocks_per_batch;
    const int64_t m0 = static_cast<int64_t>(blockIdx.x - b * blocks_per_batch) * (BLOCK * NPL);
    const unsigned lane_off = threadIdx.x * NPL;
    double my_sum = 0.0;                                       // sum of this lane's outputs (for the layer's mean)
    // lanes past the end of the layer walk the same loops and meet every barrier, but all memory
    // accesses and all arithmetic sit behind `active`
    const bool active = m0 + lane_off < M;
    {
    const int64_t first = b * M + m0 + lane_off;
    const float *xp = x + (b * T) * M + m0;
    float *op = out + (b * T) * M + m0;
    const unsigned voff = lane_off * 4u;
    const unsigned step_bytes = static_cast<unsigned>(M) * 4u;
    float a[NPL] = {}, kn[NPL] = {}, kd[NPL] = {}, v[NPL] = {};
    float part = 0.f;                                          // outputs of one stage, then folded into my_sum
    if (active) {
#pragma unroll
        for (int e = 0; e < NPL; ++e) {
            a[e] = p.alpha[first + e];
            kn[e] = p.norm_input ? __fsub_rn(1.0f, a[e]) : 1.0f;
            kd[e] = p.decay_early ? a[e] : 1.0f;
            v[e] = p.v_init[first + e];
        }
    }
    auto advance = [&](const V &xv) {
        V o;
#pragma unroll
        for (int e = 0; e < NPL; ++e) {
            const float xin = __fmul_rn(__fmul_rn(kn[e], lane_get<NPL>(xv, e)), kd[e]);
            v[e] = __fadd_rn(__fmul_rn(v[e], a[e]), xin);
            part += v[e];
            lane_put<NPL>(o, e, v[e]);
        }
        return o;
    };
    // `spread` = step_bytes, or 0 for a fetch whose data will not be used (same count of loads, one step)
    auto fetch = [&](V(&dst)[U], int64_t t0, unsigned spread) {
        __syncthreads();                                   // keeps the block's waves at the same step
        if (!active) return;
        const Rsrc r = make_rsrc(xp + t0 * M);
#pragma unroll
        for (int u = 0; u < U; ++u) dst[u] = IO::load(r, voff, u * spread);
    };
    auto compute = [&](const V(&buf)[U], int64_t t0) {
        if (!active) return;
        const Rsrc r = make_rsrc(op + t0 * M);
#pragma unroll
        for (int u = 0; u < U; ++u) IO::store(advance(buf[u]), r, voff, u * step_bytes);
        my_sum += static_cast<double>(part);
        part = 0.f;
    };
    const int64_t pairs = T / (2 * U);
    V bufa[U], bufb[U];
    if (pairs > 0) fetch(bufa, 0, step_bytes);
    for (int64_t q = 0; q < pairs; ++q) {
        const int64_t t0 = q * 2 * U;
        fetch(bufb, t0 + U, step_bytes);
        compute(bufa, t0);
        const bool more = q + 1 < pairs;
        fetch(bufa, more ? t0 + 2 * U : t0, more ? step_bytes : 0u);
        compute(bufb, t0 + U);
    }
    if (active) {
        for (int64_t t = pairs * 2 * U; t < T; ++t) {
            const V xv = IO::load(make_rsrc(xp + t * M), voff, 0u);
            IO::store(advance(xv), make_rsrc(op + t * M), voff, 0u);
        }
        my_sum += static_cast<double>(part);
#pragma unroll
        for (int e = 0; e < NPL; ++e) v_last[first + e] = v[e];
    }
    }
    if (out_sum) {
        // wave reduction, then one atomic per wave
#pragma unroll
        for (int off = WAVE / 2; off > 0; off >>= 1) my_sum += __shfl_xor(my_sum, off, WAVE);
        if ((threadIdx.x & (WAVE - 1)) == 0 && my_sum != 0.0) atomicAdd(out_sum, my_sum);
    }
}

// g_t = alpha g_{t+1} + grad_out_t (+ grad_v_last at the last step)
// grad_x_t = ((decay_early ? g_t alpha : g_t) * (norm_input ? 1 - alpha : 1))
// grad_alpha = sum_t g_t out_{t-1}  +  (decay_early ? sum_t g_t (k x_t) : 0)  -  (norm_input ? sum_t (g_t [alpha]) x_t : 0)
// `x` is only read when WITH_X (alpha gradient wanted and one of the input scalings is on).
// GO1: grad_out points at one float that stands for every element (the gradient of a sum of the output).
template <int NPL, bool ALPHA, bool WITH_X, bool NT, bool GO1 = false>
__global__ void __launch_bounds__(BLOCK) layer_leaky_backward(
    float *__restrict__ grad_x, float *__restrict__ alpha_grad, float *__restrict__ v_init_grad,
    const float *__restrict__ grad_out, const float *__restrict__ grad_v_last, const float *__restrict__ out,
    const float *__restrict__ x, const LeakyConsts p, const int64_t blocks_per_batch, const int64_t T, const int64_t M)
{
    typedef typename Vec<NPL>::type V;
    typedef BufIO<NPL, NT> IO;
    constexpr int U = LEAKY_UNROLL;
    const int64_t b = blockIdx.x / blocks_per_batch;
    const int64_t m0 = static_cast<int64_t>(blockIdx.x - b * blocks_per_batch) * (BLOCK * NPL);
    const unsigned lane_off = threadIdx.x * NPL;
    // lanes past the end of the layer walk the same loops and meet every barrier, but all memory
    // accesses and all arithmetic sit behind `active`
    const bool active = m0 + lane_off < M;
    const int64_t first = b * M + m0 + lane_off;
    const float *gp = GO1 ? nullptr : grad_out + (b * T) * M + m0;
    V g_all;                                                   // GO1: the one gradient value in every lane element
#pragma unroll
    for (int e = 0; e < NPL; ++e) lane_put<NPL>(g_all, e, GO1 ? grad_out[0] : 0.f);
    const float *outp = ALPHA ? out + (b * T) * M + m0 : nullptr;
    const float *xp = WITH_X ? x + (b * T) * M + m0 : nullptr;
    float *op = grad_x + (b * T) * M + m0;
    const unsigned voff = lane_off * 4u;
    const unsigned step_bytes = static_cast<unsigned>(M) * 4u;
    float a[NPL] = {}, k[NPL] = {}, h[NPL] = {}, g[NPL] = {};
    TileSum acc[NPL];
#pragma unroll
    for (int e = 0; e < NPL; ++e) acc[e].clear();
    if (active) {
#pragma unroll
        for (int e = 0; e < NPL; ++e) {
            a[e] = p.alpha[first + e];
            k[e] = __fsub_rn(1.0f, a[e]);
            h[e] = grad_v_last ? grad_v_last[first + e] : 0.f; // what reaches step t from later steps: alpha g_{t+1}
        }
    }
    // one step; `ov` = out_{t-1} (ignored at t = 0, where the initial state takes its place)
    auto advance = [&](int64_t t, const V &gv, const V &ov, const V &xv) {
        V o;
#pragma unroll
        for (int e = 0; e < NPL; ++e) {
            g[e] = __fadd_rn(h[e], lane_get<NPL>(gv, e));
            h[e] = __fmul_rn(g[e], a[e]);
            float gx = p.decay_early ? h[e] : g[e];
            if (ALPHA) {
                const float prev = t >= 1 ? lane_get<NPL>(ov, e) : p.v_init[first + e];
                acc[e].add(g[e], prev);
                if (WITH_X) {
                    const float xe = lane_get<NPL>(xv, e);
                    if (p.decay_early) acc[e].add(g[e], p.norm_input ? __fmul_rn(k[e], xe) : xe);
                    if (p.norm_input) acc[e].sub(gx, xe);
                }
            }
            if (p.norm_input) gx = __fmul_rn(gx, k[e]);
            lane_put<NPL>(o, e, gx);
        }
        return o;
    };
    struct Stage {
        V g[GO1 ? 1 : U], o[ALPHA ? U : 1], x[WITH_X ? U : 1];
    };
    // steps t0 .. t0 + U - 1; `spread` = step_bytes, or 0 for a fetch whose data will not be used
    auto fetch = [&](Stage &s, int64_t t0, unsigned spread) {
        __syncthreads();                                   // keeps the block's waves at the same step
        if (!active) return;
        if (!GO1) {
            const Rsrc rg = make_rsrc(gp + t0 * M);
#pragma unroll
            for (int u = 0; u < U; ++u) s.g[GO1 ? 0 : u] = IO::load(rg, voff, u * spread);
        }
        if (WITH_X) {
            const Rsrc rx = make_rsrc(xp + t0 * M);
#pragma unroll
            for (int u = 0; u < U; ++u) s.x[u] = IO::load(rx, voff, u * spread);
        }
        if (ALPHA) {
            // out_{t-1}: one step back, except that step 0 has no predecessor (it re-reads out_0, unused)
            const Rsrc ro = make_rsrc(outp + (t0 >= 1 ? t0 - 1 : 0) * M);
            const unsigned shift = t0 >= 1 ? 0u : 1u;
#pragma unroll
            for (int u = 0; u < U; ++u) s.o[u] = IO::load(ro, voff, (u >= shift ? u - shift : 0u) * spread);
        }
    };
    auto compute = [&](const Stage &s, int64_t t0) {          // newest step first
        if (!active) return;
        const Rsrc r = make_rsrc(op + t0 * M);
#pragma unroll
        for (int uu = 0; uu < U; ++uu) {
            const int u = U - 1 - uu;
            IO::store(advance(t0 + u, GO1 ? g_all : s.g[GO1 ? 0 : u], s.o[ALPHA ? u : 0], s.x[WITH_X ? u : 0]), r, voff,
                      u * step_bytes);
        }
    };
    const int64_t pairs = T / (2 * U);
    // the steps that do not fill a pair are the newest ones: one at a time
    for (int64_t t = T - 1; active && t >= pairs * 2 * U; --t) {
        const V gv = GO1 ? g_all : IO::load(make_rsrc(gp + t * M), voff, 0u);
        V ov = gv, xv = gv;
        if (ALPHA && t >= 1) ov = IO::load(make_rsrc(outp + (t - 1) * M), voff, 0u);
        if (WITH_X) xv = IO::load(make_rsrc(xp + t * M), voff, 0u);
        IO::store(advance(t, gv, ov, xv), make_rsrc(op + t * M), voff, 0u);
    }
    if (ALPHA) {
#pragma unroll
        for (int e = 0; e < NPL; ++e) acc[e].fold();
    }
    Stage sa, sb;
    if (pairs > 0) fetch(sa, (pairs - 1) * 2 * U + U, step_bytes);
    for (int64_t q = pairs - 1; q >= 0; --q) {
        const int64_t t0 = q * 2 * U;
        fetch(sb, t0, step_bytes);
        compute(sa, t0 + U);
        fetch(sa, q > 0 ? t0 - U : t0, q > 0 ? step_bytes : 0u);
        compute(sb, t0);
        if (ALPHA) {
#pragma unroll
            for (int e = 0; e < NPL; ++e) acc[e].fold();
        }
    }
    if (!active) return;                                       // no barrier follows
#pragma unroll
    for (int e = 0; e < NPL; ++e) {
        if (v_init_grad) v_init_grad[first + e] = h[e];
        if (ALPHA) alpha_grad[first + e] = static_cast<float>(acc[e].total);
    }
}

// Neurons per lane of the kernels that support several.  Wider lanes mean wider memory accesses
// but fewer lanes: stay at the widest width that still gives every compute unit `waves_per_cu`
// waves, so that small layers are not starved of parallelism (the spiking forward kernel has a long
// dependent chain per step and wants 16; the leaky kernels measure best from 8 on).  `align` is the
// common alignment (bytes) of all (batch, time, neurons) pointers involved.
// compute units of the current device, asked for once per device
inline int compute_units()
{
    static std::atomic<int> known[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int cus = known[dev].load(std::memory_order_relaxed);
    if (cus > 0) return cus;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    known[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

inline int pick_neurons_per_lane(int64_t batch, int64_t neurons, unsigned align, int widest, int waves_per_cu)
{
    const int cus = compute_units();
    const int64_t wanted_lanes = static_cast<int64_t>(cus) * waves_per_cu * WAVE;
    const int64_t n = batch * neurons;
#ifdef EXODUS_FORCE_NPL
    if (EXODUS_FORCE_NPL <= widest) widest = EXODUS_FORCE_NPL;
#endif
    if (widest >= 4 && (neurons % 4) == 0 && (align % 16) == 0 && n / 4 >= wanted_lanes) return 4;
    if (widest >= 2 && (neurons % 2) == 0 && (align % 8) == 0 && n / 2 >= wanted_lanes) return 2;
    return 1;
}

inline unsigned common_alignment(std::initializer_list<const void *> ptrs)
{
    uintptr_t bits = 0;
    for (const void *q : ptrs) bits |= reinterpret_cast<uintptr_t>(q);   // null pointers do not constrain
    return static_cast<unsigned>(bits & 15u) == 0 ? 16u : ((bits & 7u) == 0 ? 8u : 4u);
}

// true when every step's neurons start and end on 64-byte sectors of memory for all the given tensors: then no
// sector is shared between waves and the streamed accesses can be marked non-temporal (with whole 128-byte lines
// and with whole sectors that measures 1-5 % faster than without the mark; with steps that start on 32-byte
// boundaries 10 % slower)
inline bool whole_lines(int64_t neurons, std::initializer_list<const void *> ptrs)
{
    uintptr_t bits = 0;
    for (const void *q : ptrs) bits |= reinterpret_cast<uintptr_t>(q);
    return (neurons % EXODUS_WHOLE_NEURONS) == 0 && (bits & (4u * EXODUS_WHOLE_NEURONS - 1u)) == 0;
}

inline bool bad3(int64_t b, int64_t t, int64_t m)
{
    if (b < 0 || t < 0 || m < 0) return true;
    if (b == 0 || t == 0 || m == 0) return false;
    if (b > INT64_MAX / t) return true;
    return (b * t) > INT64_MAX / m;
}

// ---------------------------------------------------------------------------------------------
// backward, split over time (layers with few neurons and many steps)
// ---------------------------------------------------------------------------------------------
// The kernel above gives every neuron one lane, which walks the whole sequence: a layer of a few thousand neurons
// fills a fraction of the machine, and its run time is the length of one lane's chain, 2 T steps.  Two facts allow
// cutting the chain into pieces: the chunks of CKPT steps can be rebuilt independently from their checkpoints, and
// the adjoint recurrence is affine once the forward values are known,
//     lambda_t = nc_t (s_t g_t + (1 - c s_t) h_{t+1}),   h_t = a_mem lambda_t,   h_T = gradient on the final potential,
// so a chunk maps the h that enters it (from later steps) to the h that leaves it as h_out = A + B h_in, and every
// lambda_t inside the chunk is P_t + Q_t h_in.  Here a lane owns one chunk of one neuron (threadIdx.x = neuron,
// threadIdx.y = chunk): it rebuilds the chunk, walks it in reverse ONCE carrying (P, Q), the chunks of a neuron
// exchange (A, B) through LDS, every lane folds the maps of the chunks after its own into its h_in, and turns its
// (P_t, Q_t) into gradients.  The chain is then 2 CKPT steps plus the fold over at most SPLIT_MAX_CHUNKS entries,
// whatever T is.  Layers without synapse, with an in-kernel surrogate and without gradients on state records (the
// spiking layers of the small configurations); everything else, and every layer large enough to fill the machine,
// takes the kernel above.  Sums associate differently than in the sequential walk: results agree with it to fp32
// rounding, not bit for bit.
constexpr int SPLIT_MAX_CHUNKS = 16;       // chunks per neuron (= threadIdx.y range): sequences of up to 512 steps
constexpr int SPLIT_NEURONS = 64;          // neurons per block: one wave per chunk

template <int KIND, int CAPK, bool GO1>
__global__ void __launch_bounds__(SPLIT_NEURONS *SPLIT_MAX_CHUNKS) layer_lif_backward_split(
    float *__restrict__ grad_x, float *__restrict__ alpha_mem_grad, float *__restrict__ v_init_grad,
    const float *__restrict__ grad_spikes, const float *__restrict__ grad_v_last, const float *__restrict__ x,
    const float *__restrict__ ckpt_v, const LayerConsts p, const float p0, const float p1, const float inv_p0,
    const int64_t blocks_per_batch, const int64_t T, const int64_t M)
{
    __shared__ float map_a[SPLIT_MAX_CHUNKS][SPLIT_NEURONS], map_b[SPLIT_MAX_CHUNKS][SPLIT_NEURONS];
    __shared__ float first_lambda[SPLIT_MAX_CHUNKS + 1][SPLIT_NEURONS];
    __shared__ double partial[SPLIT_MAX_CHUNKS][SPLIT_NEURONS];
    const int64_t b = blockIdx.x / blocks_per_batch;
    const int64_t m0 = static_cast<int64_t>(blockIdx.x - b * blocks_per_batch) * SPLIT_NEURONS;
    const int lane = threadIdx.x, j = threadIdx.y;
    const int n_ck = blockDim.y;                                 // = ceil(T / CKPT), the host sees to that
    const bool active = m0 + lane < M;
    const int64_t row = b * M + m0 + lane;
    const int64_t t0 = static_cast<int64_t>(j) * CKPT;
    const int len = static_cast<int>(T - t0 < CKPT ? T - t0 : CKPT);   // uniform over a wave (one chunk per wave)

    Cap cc;
    cc.cap = p.cap;
    cc.one = p.cap >= 1u ? 1.f : 0.f;
    cc.two = p.cap >= 2u ? 2.f : cc.one;
    Neuron nr = {};
    float lam_p[CKPT], lam_q[CKPT];                              // first x and v of the chunk, then P_t and Q_t
    float hp = 0.f, hq = 1.f;                                    // h_{t+1} = hp + hq h_in
    TileSum m1, m2, n1, n2;                                      // sums of lambda_{t+1} vpost_t and lambda_t i_t, split by h_in
    m1.clear(); m2.clear(); n1.clear(); n2.clear();
    float vpost_last = 0.f;                                      // potential after the reset of the chunk's last step
    const float g1 = GO1 ? grad_spikes[0] : 0.f;
    if (active) {
        neuron_load<false, CAPK>(nr, p, row);
        const SurrConst sk = surrogate_consts<KIND>(nr.th, p0, p1);
        const float *xp = x + (b * T + t0) * M + m0 + lane;
        const float *gp = GO1 ? nullptr : grad_spikes + (b * T + t0) * M + m0 + lane;
        float gr[GO1 ? 1 : CKPT];
#pragma unroll
        for (int k = 0; k < CKPT; ++k)
            if (k < len) {
                lam_q[k] = xp[k * M];
                if (!GO1) gr[GO1 ? 0 : k] = gp[k * M];
            }
        nr.vpost = ckpt_v[(b * n_ck + j) * M + m0 + lane];
        // rebuild: the same operations in the same order as the forward pass; lam_p[k] = pre-reset potential
#pragma unroll
        for (int k = 0; k < CKPT; ++k)
            if (k < len) {
                const float v = neuron_advance<false>(nr, lam_q[k]);
                nr.vpost = __fsub_rn(v, reset_amount<CAPK>(v, nr, cc));
                lam_p[k] = v;
            }
        // reverse walk with the affine pair instead of the value
        float next_p = 0.f, next_q = 0.f;                        // lambda_{t+1} of the step above, inside this chunk
#pragma unroll
        for (int kq = 0; kq < CKPT; ++kq) {
            const int k = CKPT - 1 - kq;
            if (k < len) {
                const float v = lam_p[k], cur_i = lam_q[k];
                const float sg = surrogate<KIND>(v, nr.th, inv_p0, sk);
                const float vpost = __fsub_rn(v, reset_amount<CAPK>(v, nr, cc));
                if (k == len - 1) vpost_last = vpost;            // its partner lambda belongs to the next chunk
                else { m1.add(next_p, vpost); m2.add(next_q, vpost); }
                const float through = __fsub_rn(1.0f, __fmul_rn(nr.c, sg));
                const bool open = v > nr.lo;                     // clamped (or NaN) steps pass nothing on
                const float lp = open ? __fadd_rn(__fmul_rn(sg, GO1 ? g1 : gr[GO1 ? 0 : k]), __fmul_rn(through, hp)) : 0.f;
                const float lq = open ? __fmul_rn(through, hq) : 0.f;
                hp = __fmul_rn(nr.am, lp);
                hq = __fmul_rn(nr.am, lq);
                n1.add(lp, cur_i);
                n2.add(lq, cur_i);
                lam_p[k] = lp;
                lam_q[k] = lq;
                next_p = lp;
                next_q = lq;
            }
        }
    }
    map_a[j][lane] = hp;
    map_b[j][lane] = hq;
    __syncthreads();
    // what enters this chunk from later steps: the gradient on the final potential, through the chunks after this one
    float h_in = (active && grad_v_last) ? grad_v_last[row] : 0.f;
    for (int c = n_ck - 1; c > j; --c) h_in = __fadd_rn(map_a[c][lane], __fmul_rn(map_b[c][lane], h_in));
    if (active) {
        float *op = grad_x + (b * T + t0) * M + m0 + lane;
#pragma unroll
        for (int k = 0; k < CKPT; ++k)
            if (k < len) {
                lam_p[k] = __fadd_rn(lam_p[k], __fmul_rn(lam_q[k], h_in));     // lambda_t
                op[k * M] = __fmul_rn(lam_p[k], nr.k);
            }
    }
    first_lambda[j][lane] = active ? lam_p[0] : 0.f;
    if (j == 0) first_lambda[n_ck][lane] = 0.f;                  // beyond the sequence: lambda_T = 0
    m1.fold(); m2.fold(); n1.fold(); n2.fold();
    __syncthreads();
    double mine = 0.0;
    if (active && alpha_mem_grad) {
        // sum_t lambda_{t+1} vpost_t over this chunk (the last step pairs with the next chunk's first lambda) ...
        mine = m1.total + m2.total * static_cast<double>(h_in) +
               static_cast<double>(first_lambda[j + 1][lane]) * static_cast<double>(vpost_last);
        // ... the initial state's term, and what the input normalisation contributes: - sum_t lambda_t i_t
        if (j == 0) mine += static_cast<double>(lam_p[0]) * static_cast<double>(p.v_init[row]);
        if (p.norm_input) mine -= n1.total + n2.total * static_cast<double>(h_in);
    }
    partial[j][lane] = mine;
    __syncthreads();
    if (j == 0 && active) {
        if (alpha_mem_grad) {
            double total = 0.0;
            for (int c = 0; c < n_ck; ++c) total += partial[c][lane];
            alpha_mem_grad[row] = static_cast<float>(total);
        }
        if (v_init_grad) v_init_grad[row] = __fadd_rn(hp, __fmul_rn(hq, h_in));    // h_0 = a_mem lambda_0
    }
}

// 0: never, 1: for layers that leave most of the machine idle (default), 2: whenever the kernel applies
std::atomic<int> split_mode{1};
constexpr int64_t SPLIT_MOST_NEURONS = 16384;                    // batch * neurons up to which mode 1 splits

template <int KIND, int CAPK>
int launch_bwd_split(float *grad_x, float *am_g, float *v0_g, const float *grad_spikes, const float *gvl, const float *x,
                     const float *ckpt_v, const LayerConsts &p, float p0, float p1, bool uniform, int64_t B, int64_t T,
                     int64_t M, hipStream_t s)
{
    const int64_t blocks_per_batch = (M + SPLIT_NEURONS - 1) / SPLIT_NEURONS;
    if (blocks_per_batch > 0x7fffffffLL / B) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks_per_batch * B));
    const dim3 block(SPLIT_NEURONS, static_cast<unsigned>((T + CKPT - 1) / CKPT));
    const float inv_p0 = p0 != 0.f ? 1.f / p0 : 0.f;
    if (uniform)
        hipLaunchKernelGGL((layer_lif_backward_split<KIND, CAPK, true>), grid, block, 0, s, grad_x, am_g, v0_g, grad_spikes,
                           gvl, x, ckpt_v, p, p0, p1, inv_p0, blocks_per_batch, T, M);
    else
        hipLaunchKernelGGL((layer_lif_backward_split<KIND, CAPK, false>), grid, block, 0, s, grad_x, am_g, v0_g, grad_spikes,
                           gvl, x, ckpt_v, p, p0, p1, inv_p0, blocks_per_batch, T, M);
    return static_cast<int>(hipGetLastError());
}

template <int KIND, class... A>
int dispatch_bwd_split_cap(unsigned cap, A... a)
{
    if (cap == 1u) return launch_bwd_split<KIND, 1>(a...);
    if (cap == 2u) return launch_bwd_split<KIND, 2>(a...);
    return launch_bwd_split<KIND, 0>(a...);
}

template <bool SYN, int KIND, int CAPK>
int launch_bwd(float *grad_x, float *am_g, float *as_g, float *v0_g, float *i0_g, const float *grad_spikes,
               const float *gvl, const float *gil, const float *x, const float *surr, const float *gvr,
               const float *gir, const float *ckpt_v, const float *ckpt_i, const LayerConsts &p, float p0, float p1,
               bool uniform, int64_t B, int64_t T, int64_t M, hipStream_t s)
{
    const int64_t blocks_per_batch = (M + BWD_BLOCK - 1) / BWD_BLOCK;
    if (blocks_per_batch > 0x7fffffffLL / B) return hipErrorInvalidValue;
    const int64_t blocks = blocks_per_batch * B;
#define EXODUS_LAUNCH(CK, NT, EX, G1)                                                                              \
    hipLaunchKernelGGL((layer_lif_backward<SYN, KIND, CK, NT, EX, G1>), dim3(static_cast<unsigned>(blocks)),      \
                       dim3(BWD_BLOCK), 0, s, grad_x, am_g, as_g, v0_g, i0_g, grad_spikes, gvl, gil, x, surr, gvr, \
                       gir, ckpt_v, ckpt_i, p, p0, p1, p0 != 0.f ? 1.f / p0 : 0.f, blocks_per_batch, T, M)
    if (uniform) {
        // one value as the gradient of every spike: instances exist for the in-kernel surrogates, without
        // gradients on the state records
        if constexpr (KIND == EXODUS_SURR_TENSOR) {
            return hipErrorInvalidValue;
        } else {
            if (gvr) return hipErrorInvalidValue;
            if (whole_lines(M, {grad_x, x})) EXODUS_LAUNCH(CAPK, true, false, true);
            else EXODUS_LAUNCH(CAPK, false, false, true);
        }
    } else if (gvr) {
        // gradients on the state records: one general instance per surrogate kind
        EXODUS_LAUNCH(0, false, true, false);
    } else if (whole_lines(M, {grad_x, grad_spikes, x, surr})) {
        EXODUS_LAUNCH(CAPK, true, false, false);
    } else {
        EXODUS_LAUNCH(CAPK, false, false, false);
    }
#undef EXODUS_LAUNCH
    return static_cast<int>(hipGetLastError());
}

template <bool SYN, int KIND, class... A>
int dispatch_bwd_cap(unsigned cap, A... a)
{
    if (cap == 1u) return launch_bwd<SYN, KIND, 1>(a...);
    if (cap == 2u) return launch_bwd<SYN, KIND, 2>(a...);
    return launch_bwd<SYN, KIND, 0>(a...);
}

struct FwdArgs {
    float *spikes, *v_rec, *i_rec, *ckpt_v, *ckpt_i, *v_last, *i_last;
    double *spike_sum;
    const float *x;
    LayerConsts p;
    int64_t B, T, M;
    hipStream_t s;
};

template <bool SYN, int NPL, int CAPK, bool REC>
int launch_fwd(const FwdArgs &a)
{
    const int64_t blocks_per_batch = (a.M + BLOCK * NPL - 1) / (BLOCK * NPL);
    if (blocks_per_batch > 0x7fffffffLL / a.B) return hipErrorInvalidValue;
    if (whole_lines(a.M, {a.x, a.spikes, a.v_rec, a.i_rec}))
        hipLaunchKernelGGL((layer_lif_forward<SYN, NPL, CAPK, REC, true>), dim3(static_cast<unsigned>(blocks_per_batch * a.B)),
                           dim3(BLOCK), 0, a.s, a.spikes, a.v_rec, a.i_rec, a.ckpt_v, a.ckpt_i, a.v_last, a.i_last,
                           a.spike_sum, a.x, a.p, blocks_per_batch, a.T, a.M);
    else
        hipLaunchKernelGGL((layer_lif_forward<SYN, NPL, CAPK, REC, false>), dim3(static_cast<unsigned>(blocks_per_batch * a.B)),
                           dim3(BLOCK), 0, a.s, a.spikes, a.v_rec, a.i_rec, a.ckpt_v, a.ckpt_i, a.v_last, a.i_last,
                           a.spike_sum, a.x, a.p, blocks_per_batch, a.T, a.M);
    return static_cast<int>(hipGetLastError());
}

// the specialisations for caps of one and two spikes exist for the layer's usual outputs only;
// the general kernel serves every cap and also writes the per-step state records
template <bool SYN, int NPL>
int dispatch_fwd_cap(const FwdArgs &a)
{
    if (a.p.cap == 1u) return launch_fwd<SYN, NPL, 1, false>(a);
    if (a.p.cap == 2u) return launch_fwd<SYN, NPL, 2, false>(a);
    return launch_fwd<SYN, NPL, 0, false>(a);
}

template <bool SYN>
int dispatch_fwd(const FwdArgs &a, int npl)
{
    if (a.v_rec || a.i_rec) return launch_fwd<SYN, 1, 0, true>(a);
#if EXODUS_LIF_FWD_WIDEST >= 4
    if (npl == 4) return dispatch_fwd_cap<SYN, 4>(a);
#endif
    if (npl == 2) return dispatch_fwd_cap<SYN, 2>(a);
    return dispatch_fwd_cap<SYN, 1>(a);
}

// the forward pass again, keeping nothing but the checkpoints (one neuron per lane, general spike count:
// the values do not depend on either choice)
template <bool SYN>
int launch_checkpoints_only(float *ckpt_v, float *ckpt_i, const float *x, const LayerConsts &p, int64_t B, int64_t T,
                            int64_t M, hipStream_t s)
{
    const int64_t blocks_per_batch = (M + BLOCK - 1) / BLOCK;
    if (blocks_per_batch > 0x7fffffffLL / B) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks_per_batch * B)), block(BLOCK);
    float *const none = nullptr;
    double *const no_sum = nullptr;
    if (whole_lines(M, {x, ckpt_v, ckpt_i}))
        hipLaunchKernelGGL((layer_lif_forward<SYN, 1, 0, false, true, false>), grid, block, 0, s, none, none, none, ckpt_v,
                           ckpt_i, none, none, no_sum, x, p, blocks_per_batch, T, M);
    else
        hipLaunchKernelGGL((layer_lif_forward<SYN, 1, 0, false, false, false>), grid, block, 0, s, none, none, none,
                           ckpt_v, ckpt_i, none, none, no_sum, x, p, blocks_per_batch, T, M);
    return static_cast<int>(hipGetLastError());
}

// step offsets inside a block of CKPT steps are 32-bit byte offsets
inline bool too_wide(int64_t neurons) { return neurons >= (int64_t{1} << 25); }

}  // namespace

// ---------------------------------------------------------------------------------------------
// Checkpoint memory of exodus_layer_lif_backward_from_input, the one entry point that must not
// allocate.  Every GPU the library runs on holds its own copy of this array, at its own address,
// until the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress:
// kernels get the device address looked up below, never the name.
// ---------------------------------------------------------------------------------------------
constexpr int64_t SCRATCH_FLOATS = int64_t{1} << 24;           // 64 MiB
static __device__ __align__(256) float scratch[SCRATCH_FLOATS];

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex scratch_lock;
float *scratch_of_device[MAX_DEVICES] = {};

// device address of `scratch` on the current device (looked up once per device)
int scratch_address(float **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_of_device[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!ptr) return hipErrorInvalidSymbol;
        scratch_of_device[dev] = static_cast<float *>(ptr);
    }
    *out = scratch_of_device[dev];
    return hipSuccess;
}

}  // namespace

extern "C" {

#define EXODUS_API __attribute__((visibility("default")))

EXODUS_API int exodus_layer_checkpoint_interval(void) { return CKPT; }

EXODUS_API int exodus_layer_lif_forward(float *out_spikes, float *out_vmem_rec, float *out_isyn_rec, float *ckpt_v,
                                        float *ckpt_i, float *v_last, float *i_last, double *spike_sum,
                                        const float *input, const float *vmem_post_initial,
                                        const float *isyn_initial, const float *alpha_mem, const float *alpha_syn,
                                        const float *membr_subtract, const float *theta, const float *theta_low,
                                        int apply_theta_low, int max_num_spikes, int decay_early, int norm_input,
                                        int record_pre_reset, int64_t batch, int64_t t, int64_t neurons,
                                        void *stream)
{
    if (bad3(batch, t, neurons)) return hipErrorInvalidValue;
    if (batch == 0 || t == 0 || neurons == 0) return hipSuccess;
    if (too_wide(neurons)) return hipErrorInvalidValue;
    const bool syn = alpha_syn != nullptr;
    if (!out_spikes || !v_last || !input || !vmem_post_initial || !alpha_mem || !membr_subtract || !theta ||
        (apply_theta_low && !theta_low) || (syn && !isyn_initial) || (syn && ckpt_v && !ckpt_i))
        return hipErrorInvalidValue;
    LayerConsts p;
    p.v_init = vmem_post_initial;
    p.i_init = isyn_initial;
    p.alpha_mem = alpha_mem;
    p.alpha_syn = alpha_syn;
    p.c = membr_subtract;
    p.theta = theta;
    p.theta_low = theta_low;
    p.apply_low = apply_theta_low ? 1 : 0;
    p.decay_early = decay_early ? 1 : 0;
    p.norm_input = norm_input ? 1 : 0;
    p.cap = static_cast<unsigned>(max_num_spikes);
    p.rec_pre = record_pre_reset ? 1 : 0;
    // two neurons per lane at most: with four the spiking kernel needs so many registers for its two
    // load buffers that only two waves fit a SIMD, and it measures slower than two neurons, three waves
    const int npl = pick_neurons_per_lane(
        batch, neurons, common_alignment({input, out_spikes, out_vmem_rec, out_isyn_rec, ckpt_v, ckpt_i}), EXODUS_LIF_FWD_WIDEST, 16);
    FwdArgs a{out_spikes, out_vmem_rec, out_isyn_rec, ckpt_v, ckpt_i, v_last, i_last, spike_sum, input, p,
              batch, t, neurons, static_cast<hipStream_t>(stream)};
    return syn ? dispatch_fwd<true>(a, npl) : dispatch_fwd<false>(a, npl);
}

EXODUS_API int exodus_layer_lif_backward(float *grad_input, float *alpha_mem_grad, float *alpha_syn_grad,
                                         float *vmem_init_grad, float *isyn_init_grad, const float *grad_spikes,
                                         const float *grad_v_last, const float *grad_i_last, const float *input,
                                         const float *ckpt_v, const float *ckpt_i, const float *vmem_post_initial,
                                         const float *isyn_initial, const float *alpha_mem, const float *alpha_syn,
                                         const float *membr_subtract, const float *theta, const float *theta_low,
                                         int apply_theta_low, int max_num_spikes, int decay_early, int norm_input,
                                         int surrogate_kind, float surr_p0, float surr_p1, const float *surr,
                                         const float *grad_v_rec, const float *grad_i_rec, int grad_spikes_uniform,
                                         int64_t batch, int64_t t, int64_t neurons, void *stream)
{
    if (bad3(batch, t, neurons)) return hipErrorInvalidValue;
    if (batch == 0 || t == 0 || neurons == 0) return hipSuccess;
    if (too_wide(neurons)) return hipErrorInvalidValue;
    const bool syn = alpha_syn != nullptr;
    if (grad_spikes_uniform && (surrogate_kind == EXODUS_SURR_TENSOR || grad_v_rec || grad_i_rec))
        return hipErrorInvalidValue;
    if (!grad_input || !grad_spikes || !input || !ckpt_v || !alpha_mem || !membr_subtract || !theta ||
        (apply_theta_low && !theta_low) || (syn && !ckpt_i) || (surrogate_kind == EXODUS_SURR_TENSOR && !surr))
        return hipErrorInvalidValue;
    if (surrogate_kind != EXODUS_SURR_TENSOR) surr = nullptr;
    if (syn ? ((grad_v_rec != nullptr) != (grad_i_rec != nullptr)) : grad_i_rec != nullptr) return hipErrorInvalidValue;
    if (alpha_mem_grad && !vmem_post_initial) return hipErrorInvalidValue;
    if (syn && alpha_syn_grad && !decay_early && !isyn_initial) return hipErrorInvalidValue;
    LayerConsts p;
    p.v_init = vmem_post_initial;
    p.i_init = isyn_initial;
    p.alpha_mem = alpha_mem;
    p.alpha_syn = alpha_syn;
    p.c = membr_subtract;
    p.theta = theta;
    p.theta_low = theta_low;
    p.apply_low = apply_theta_low ? 1 : 0;
    p.decay_early = decay_early ? 1 : 0;
    p.norm_input = norm_input ? 1 : 0;
    p.cap = static_cast<unsigned>(max_num_spikes);
    p.rec_pre = 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // few neurons, many steps: one lane per chunk of 32 steps instead of one lane per neuron
    const int mode = split_mode.load(std::memory_order_relaxed);
    const int64_t n_ck = (t + CKPT - 1) / CKPT;
    if (mode != 0 && !syn && surrogate_kind != EXODUS_SURR_TENSOR && !grad_v_rec && n_ck >= 2 && n_ck <= SPLIT_MAX_CHUNKS &&
        (mode == 2 || batch * neurons <= SPLIT_MOST_NEURONS)) {
#define EXODUS_SPLIT(K)                                                                                           \
    return dispatch_bwd_split_cap<K>(p.cap, grad_input, alpha_mem_grad, vmem_init_grad, grad_spikes, grad_v_last, \
                                     input, ckpt_v, p, surr_p0, surr_p1, grad_spikes_uniform != 0, batch, t,      \
                                     neurons, s)
        switch (surrogate_kind) {
            case EXODUS_SURR_SINGLE_EXP: EXODUS_SPLIT(EXODUS_SURR_SINGLE_EXP);
            case EXODUS_SURR_PERIODIC_EXP: EXODUS_SPLIT(EXODUS_SURR_PERIODIC_EXP);
            case EXODUS_SURR_HEAVISIDE: EXODUS_SPLIT(EXODUS_SURR_HEAVISIDE);
            default: return hipErrorInvalidValue;
        }
#undef EXODUS_SPLIT
    }
#define EXODUS_BWD(SYN, K)                                                                                        \
    return dispatch_bwd_cap<SYN, K>(p.cap, grad_input, alpha_mem_grad, alpha_syn_grad, vmem_init_grad,            \
                                    isyn_init_grad, grad_spikes, grad_v_last, grad_i_last, input, surr,           \
                                    grad_v_rec, grad_i_rec, ckpt_v, ckpt_i, p, surr_p0, surr_p1,                  \
                                    grad_spikes_uniform != 0, batch, t, neurons, s)
    switch (surrogate_kind) {
        case EXODUS_SURR_TENSOR: if (syn) EXODUS_BWD(true, EXODUS_SURR_TENSOR); EXODUS_BWD(false, EXODUS_SURR_TENSOR);
        case EXODUS_SURR_SINGLE_EXP: if (syn) EXODUS_BWD(true, EXODUS_SURR_SINGLE_EXP); EXODUS_BWD(false, EXODUS_SURR_SINGLE_EXP);
        case EXODUS_SURR_PERIODIC_EXP: if (syn) EXODUS_BWD(true, EXODUS_SURR_PERIODIC_EXP); EXODUS_BWD(false, EXODUS_SURR_PERIODIC_EXP);
        case EXODUS_SURR_HEAVISIDE: if (syn) EXODUS_BWD(true, EXODUS_SURR_HEAVISIDE); EXODUS_BWD(false, EXODUS_SURR_HEAVISIDE);
        default: return hipErrorInvalidValue;
    }
#undef EXODUS_BWD
}

EXODUS_API int exodus_layer_backward_time_split(int mode)
{
    const int before = split_mode.load(std::memory_order_relaxed);
    if (mode >= 0 && mode <= 2) split_mode.store(mode, std::memory_order_relaxed);
    return before;
}

EXODUS_API int64_t exodus_layer_scratch_floats(void) { return SCRATCH_FLOATS; }

EXODUS_API int exodus_layer_lif_backward_from_input(
    float *grad_input, float *alpha_mem_grad, float *alpha_syn_grad, float *vmem_init_grad, float *isyn_init_grad,
    const float *grad_spikes, const float *grad_v_last, const float *grad_i_last, const float *input,
    const float *vmem_post_initial, const float *isyn_initial, const float *alpha_mem, const float *alpha_syn,
    const float *membr_subtract, const float *theta, const float *theta_low, int apply_theta_low, int max_num_spikes,
    int decay_early, int norm_input, int surrogate_kind, float surr_p0, float surr_p1, const float *surr,
    const float *grad_v_rec, const float *grad_i_rec, int grad_spikes_uniform, int64_t batch, int64_t t,
    int64_t neurons, void *stream)
{
    if (bad3(batch, t, neurons)) return hipErrorInvalidValue;
    if (batch == 0 || t == 0 || neurons == 0) return hipSuccess;
    if (too_wide(neurons)) return hipErrorInvalidValue;
    const bool syn = alpha_syn != nullptr;
    if (!grad_input || !grad_spikes || !input || !vmem_post_initial || !alpha_mem || !membr_subtract || !theta ||
        (apply_theta_low && !theta_low) || (syn && !isyn_initial) ||
        (surrogate_kind == EXODUS_SURR_TENSOR && !surr) || surrogate_kind < EXODUS_SURR_TENSOR ||
        surrogate_kind > EXODUS_SURR_HEAVISIDE ||
        (grad_spikes_uniform && (surrogate_kind == EXODUS_SURR_TENSOR || grad_v_rec || grad_i_rec)))
        return hipErrorInvalidValue;
    if (syn ? ((grad_v_rec != nullptr) != (grad_i_rec != nullptr)) : grad_i_rec != nullptr) return hipErrorInvalidValue;
    // checkpoints of one batch element; the batch is walked in slices of as many elements as fit
    const int64_t n_ck = (t + CKPT - 1) / CKPT;
    if (n_ck > SCRATCH_FLOATS / neurons) return EXODUS_ERROR_SCRATCH_TOO_SMALL;
    const int64_t per_element = ((n_ck * neurons + 63) / 64) * 64;          // each tensor starts on a 256-byte boundary
    const int64_t fit = SCRATCH_FLOATS / (per_element * (syn ? 2 : 1));
    if (fit < 1) return EXODUS_ERROR_SCRATCH_TOO_SMALL;
    float *base = nullptr;
    if (const int rc = scratch_address(&base)) return rc;
    LayerConsts p;
    p.v_init = vmem_post_initial;
    p.i_init = isyn_initial;
    p.alpha_mem = alpha_mem;
    p.alpha_syn = alpha_syn;
    p.c = membr_subtract;
    p.theta = theta;
    p.theta_low = theta_low;
    p.apply_low = apply_theta_low ? 1 : 0;
    p.decay_early = decay_early ? 1 : 0;
    p.norm_input = norm_input ? 1 : 0;
    p.cap = static_cast<unsigned>(max_num_spikes);
    p.rec_pre = 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto at = [](auto *q, int64_t offset) { return q ? q + offset : q; };   // absent tensors stay absent
    for (int64_t b0 = 0; b0 < batch; b0 += fit) {
        const int64_t nb = batch - b0 < fit ? batch - b0 : fit;
        const int64_t el = b0 * t * neurons, row = b0 * neurons;             // offsets of this slice
        float *ckpt_v = base, *ckpt_i = syn ? base + fit * per_element : nullptr;
        // the checkpoints of a slice are laid out (nb, n_ck, neurons) without padding between elements
        LayerConsts q = p;
        q.v_init = at(p.v_init, row);
        q.i_init = at(p.i_init, row);
        q.alpha_mem = at(p.alpha_mem, row);
        q.alpha_syn = at(p.alpha_syn, row);
        q.c = at(p.c, row);
        q.theta = at(p.theta, row);
        q.theta_low = at(p.theta_low, row);
        const int rc = syn ? launch_checkpoints_only<true>(ckpt_v, ckpt_i, input + el, q, nb, t, neurons, s)
                           : launch_checkpoints_only<false>(ckpt_v, ckpt_i, input + el, q, nb, t, neurons, s);
        if (rc) return rc;
        const int rb = exodus_layer_lif_backward(
            at(grad_input, el), at(alpha_mem_grad, row), at(alpha_syn_grad, row), at(vmem_init_grad, row),
            at(isyn_init_grad, row), grad_spikes_uniform ? grad_spikes : at(grad_spikes, el), at(grad_v_last, row),
            at(grad_i_last, row), input + el,
            ckpt_v, ckpt_i, q.v_init, q.i_init, q.alpha_mem, q.alpha_syn, q.c, q.theta, q.theta_low, apply_theta_low,
            max_num_spikes, decay_early, norm_input, surrogate_kind, surr_p0, surr_p1, at(surr, el), at(grad_v_rec, el),
            at(grad_i_rec, el), grad_spikes_uniform, nb, t, neurons, stream);
        if (rb) return rb;
    }
    return hipSuccess;
}

EXODUS_API int exodus_layer_leaky_forward(float *out, float *v_last, double *out_sum, const float *input,
                                          const float *vmem_initial, const float *alpha, int decay_early,
                                          int norm_input, int64_t batch, int64_t t, int64_t neurons, void *stream)
{
    if (bad3(batch, t, neurons)) return hipErrorInvalidValue;
    if (batch == 0 || t == 0 || neurons == 0) return hipSuccess;
    if (too_wide(neurons)) return hipErrorInvalidValue;
    if (!out || !v_last || !input || !vmem_initial || !alpha) return hipErrorInvalidValue;
    LeakyConsts p;
    p.v_init = vmem_initial;
    p.alpha = alpha;
    p.decay_early = decay_early ? 1 : 0;
    p.norm_input = norm_input ? 1 : 0;
    const int npl = pick_neurons_per_lane(batch, neurons, common_alignment({input, out}), 4, EXODUS_LEAKY_WAVES);
    const int64_t blocks_per_batch = (neurons + BLOCK * npl - 1) / (BLOCK * npl);
    if (blocks_per_batch > 0x7fffffffLL / batch) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks_per_batch * batch)), block(BLOCK);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool nt = whole_lines(neurons, {input, out});
#define EXODUS_LF(NPL, NT)                                                                                     \
    hipLaunchKernelGGL((layer_leaky_forward<NPL, NT>), grid, block, 0, s, out, v_last, out_sum, input, p,     \
                       blocks_per_batch, t, neurons)
    if (npl == 4) {
        if (nt) EXODUS_LF(4, true); else EXODUS_LF(4, false);
    } else if (npl == 2) {
        if (nt) EXODUS_LF(2, true); else EXODUS_LF(2, false);
    } else {
        if (nt) EXODUS_LF(1, true); else EXODUS_LF(1, false);
    }
#undef EXODUS_LF
    return static_cast<int>(hipGetLastError());
}

EXODUS_API int exodus_layer_leaky_backward(float *grad_input, float *alpha_grad, float *vmem_init_grad,
                                           const float *grad_out, const float *grad_v_last, const float *out,
                                           const float *input, const float *vmem_initial, const float *alpha,
                                           int decay_early, int norm_input, int grad_out_uniform, int64_t batch,
                                           int64_t t, int64_t neurons, void *stream)
{
    if (bad3(batch, t, neurons)) return hipErrorInvalidValue;
    if (batch == 0 || t == 0 || neurons == 0) return hipSuccess;
    if (too_wide(neurons)) return hipErrorInvalidValue;
    if (!grad_input || !grad_out || !alpha) return hipErrorInvalidValue;
    const bool want_alpha = alpha_grad != nullptr;
    const bool with_x = want_alpha && (decay_early || norm_input);
    if (want_alpha && (!out || !vmem_initial)) return hipErrorInvalidValue;
    if (with_x && !input) return hipErrorInvalidValue;
    LeakyConsts p;
    p.v_init = vmem_initial;
    p.alpha = alpha;
    p.decay_early = decay_early ? 1 : 0;
    p.norm_input = norm_input ? 1 : 0;
    // with the alpha gradient two or three tensors are double-buffered: two neurons per lane at most
    const bool g1 = grad_out_uniform != 0;
    const int npl = pick_neurons_per_lane(batch, neurons, common_alignment({grad_input, g1 ? nullptr : grad_out, out, input}),
                                          want_alpha ? 2 : 4, EXODUS_LEAKY_WAVES);
    const int64_t blocks_per_batch = (neurons + BLOCK * npl - 1) / (BLOCK * npl);
    if (blocks_per_batch > 0x7fffffffLL / batch) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks_per_batch * batch)), block(BLOCK);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool nt = whole_lines(neurons, {grad_input, g1 ? nullptr : grad_out, out, input});
#define EXODUS_LK1(NPL, AL, WX, NT, G1)                                                                        \
    hipLaunchKernelGGL((layer_leaky_backward<NPL, AL, WX, NT, G1>), grid, block, 0, s, grad_input, alpha_grad, \
                       vmem_init_grad, grad_out, grad_v_last, out, input, p, blocks_per_batch, t, neurons)
#define EXODUS_LK(NPL, AL, WX)                                                                                 \
    do {                                                                                                       \
        if (g1) {                                                                                              \
            if (nt) EXODUS_LK1(NPL, AL, WX, true, true); else EXODUS_LK1(NPL, AL, WX, false, true);            \
        } else {                                                                                               \
            if (nt) EXODUS_LK1(NPL, AL, WX, true, false); else EXODUS_LK1(NPL, AL, WX, false, false);          \
        }                                                                                                      \
    } while (0)
    if (npl == 4) {
        EXODUS_LK(4, false, false);
    } else if (npl == 2) {
        if (with_x) EXODUS_LK(2, true, true); else if (want_alpha) EXODUS_LK(2, true, false); else EXODUS_LK(2, false, false);
    } else {
        if (with_x) EXODUS_LK(1, true, true); else if (want_alpha) EXODUS_LK(1, true, false); else EXODUS_LK(1, false, false);
    }
#undef EXODUS_LK
#undef EXODUS_LK1
    return static_cast<int>(hipGetLastError());
}

}  // extern "C"
