/*
 * exodus_hip.h -- C ABI of libexodus_hip.so, the gfx950 (MI355X) implementation of the
 * EXODUS neuron-dynamics path.
 *
 * Conventions shared by every entry point
 *   - All tensors are device pointers to contiguous fp32.  "(n,t)" means a row-major matrix
 *     of n rows (one row = one neuron of one batch element) by t time steps, time contiguous;
 *     "(n)" is one value per row.  Offsets are 64-bit: n*t may exceed 2^31.
 *   - The library never allocates, frees or synchronises.  Kernels are enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL = the null stream) of the CURRENT device; the caller
 *     selects the device that owns the pointers.
 *   - Return value: 0 on success, otherwise a hipError_t value (1 = invalid value for a bad
 *     argument detected on the host before any launch).  exodus_hip_error_string() names it.
 *   - n == 0 or t == 0 is a successful no-op (per-row outputs are then left untouched).
 *   - Thread safe: no global state (one exception, stated there: exodus_layer_lif_backward_from_input).
 *
 * The first six entry points map one-to-one onto the six production functions the reference
 * exports from its CUDA extension (reference cuda/bindings.cu:362-373), so that the same unit
 * tests can be written against either.  The "fused" entry points below them are what the
 * autograd Functions call: one pass per direction.
 */
#ifndef EXODUS_HIP_H
#define EXODUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ABI version of this header; bumped on any signature change. */
#define EXODUS_HIP_ABI_VERSION 8

int exodus_hip_abi_version(void);
const char *exodus_hip_error_string(int status);

/* Status values of this library's own (negative, so that they cannot collide with a hipError_t). */
#define EXODUS_ERROR_SCRATCH_TOO_SMALL (-2)
#define EXODUS_ERROR_REGIONS_NOT_FOUND (-3)
#define EXODUS_ERROR_RANGE_IN_USE (-4)

/* ---------------------------------------------------------------------------------------------
 * One-to-one counterparts of the reference bindings
 * ------------------------------------------------------------------------------------------- */

/* Replaces lifForward (reference cuda/bindings.cu:14-70, kernel cuda/lif_kernels.h:40-93).
 * Per row, for each step:  v = (v - count*membr_subtract) * alpha + input;  if apply_theta_low
 * and v < theta_low: v = theta_low;  count = v >= theta ? min((unsigned)(v/theta), cap) : 0.
 * Writes count as float to out_spikes and v (before its own reset) to out_vmem.
 * max_num_spikes < 0 means no cap.  theta_low may be NULL when apply_theta_low == 0. */
int exodus_lif_forward(float *out_spikes, float *out_vmem, const float *input,
                       const float *vmem_post_initial, const float *alpha,
                       const float *membr_subtract, const float *theta, const float *theta_low,
                       int apply_theta_low, int max_num_spikes, int64_t n, int64_t t,
                       void *stream);

/* Replaces lifBackward (reference cuda/bindings.cu:72-110, kernel cuda/lif_kernels.h:122-168).
 * input_grad_i = nc_i g_i + sum_{j>i} g_j nc_i prod_{k=i+1..j} (alpha - membr_subtract*surr_{k-1}) nc_k,
 * evaluated as the linear-time reverse recurrence lambda_t = nc_t (g_t + (alpha - membr_subtract*surr_t) lambda_{t+1}).
 * As in the reference, `membr_subtract` here is alpha times the subtract value. */
int exodus_lif_backward(float *input_grad, const float *surr, const float *output_grad,
                        const float *not_clipped, const float *alpha, const float *membr_subtract,
                        int64_t n, int64_t t, void *stream);

/* Replaces lifBackwardAlpha (reference cuda/bindings.cu:112-158, kernel cuda/lif_kernels.h:199-246).
 * alpha_grad = sum_j D_j g_j with D_0 = vmem_post_initial, D_j = nc_j (alpha (1 - c surr_{j-1}) D_{j-1} + vmem_post_{j-1}).
 * gate_initial == 0 reproduces the reference exactly (D_0 enters step 1 even when step 0 was clipped);
 * gate_initial != 0 multiplies D_0 by nc_0 first, which is the exact derivative. */
int exodus_lif_backward_alpha(float *alpha_grad, const float *surr, const float *output_grad,
                              const float *vmem_post, const float *vmem_post_initial,
                              const float *not_clipped, const float *alpha,
                              const float *membr_subtract, int gate_initial, int64_t n, int64_t t,
                              void *stream);

/* Replaces leakyForward (reference cuda/bindings.cu:163-193, kernel cuda/leaky_kernels.h:29-58).
 * out_t = alpha * out_{t-1} + input_t, out_{-1} = vmem_initial. */
int exodus_leaky_forward(float *out, const float *input, const float *vmem_initial,
                         const float *alpha, int64_t n, int64_t t, void *stream);

/* Replaces leakyBackward (reference cuda/bindings.cu:195-221, kernel cuda/leaky_kernels.h:82-110).
 * input_grad_t = alpha * input_grad_{t+1} + output_grad_t. */
int exodus_leaky_backward(float *input_grad, const float *output_grad, const float *alpha,
                          int64_t n, int64_t t, void *stream);

/* Replaces leakyBackwardAlpha (reference cuda/bindings.cu:223-257, kernel cuda/leaky_kernels.h:133-165).
 * alpha_grad = sum_t input_grad_t * output_{t-1}, output_{-1} = vmem_initial (the same sum the
 * reference accumulates forward in time as sum_t D_t output_grad_t). */
int exodus_leaky_backward_alpha(float *alpha_grad, const float *output_grad, const float *output,
                                const float *vmem_initial, const float *alpha, int64_t n,
                                int64_t t, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Fused entry points (one pass per direction)
 * ------------------------------------------------------------------------------------------- */

/* Everything LeakyIntegrator.backward needs (reference sinabs/exodus/leaky.py:53-76) in one
 * reverse pass: input_grad (n,t); init_grad (n) = alpha * input_grad[:,0]; and, when
 * alpha_grad != NULL, alpha_grad (n) as above (then `output` and `vmem_initial` are required).
 * alpha_grad, init_grad may each be NULL. */
int exodus_leaky_backward_fused(float *input_grad, float *alpha_grad, float *init_grad,
                                const float *output_grad, const float *output,
                                const float *vmem_initial, const float *alpha, int64_t n,
                                int64_t t, void *stream);

/* Surrogate-gradient functions evaluated inside exodus_lif_backward_fused. */
enum exodus_surrogate_kind {
    EXODUS_SURR_TENSOR = 0,          /* read ds/dv from the `surr` argument                          */
    EXODUS_SURR_SINGLE_EXP = 1,      /* p1/(theta*p0) * exp(-|v-theta|/(theta*p0))    p0=width p1=scale */
    EXODUS_SURR_PERIODIC_EXP = 2,    /* p1*exp(-|u-theta/2|/p0)/theta, u=v-theta/2 wrapped mod theta for v>=theta */
    EXODUS_SURR_HEAVISIDE = 3        /* (v >= theta-p0) / theta                       p0=window       */
};

/* Everything IntegrateAndFire.backward computes (reference sinabs/exodus/spike.py:229-291) in one
 * reverse pass over the saved pre-reset membrane potential `vmem`:
 *   s_t  = surrogate(vmem_t, theta)            (or surr_t when kind == EXODUS_SURR_TENSOR)
 *   nc_t = apply_theta_low ? vmem_t > theta_low : 1
 *   g_t  = s_t * grad_spikes_t + grad_vmem_t   (grad_vmem may be NULL = zeros)
 *   lambda_t = nc_t (g_t + (alpha - alpha*c*s_t) lambda_{t+1})           -> input_grad (n,t)
 *   init_grad  = alpha * lambda_0                                         (n), may be NULL
 *   alpha_grad = sum_t lambda_t * vpost_{t-1}, vpost_t = vmem_t - c*count_t, vpost_{-1} = vmem_post_initial
 *                (n), may be NULL; count_t is recomputed from vmem_t, theta and max_num_spikes.
 * The alpha gradient is the exact one (initial step gated), see exodus_lif_backward_alpha. */
int exodus_lif_backward_fused(float *input_grad, float *alpha_grad, float *init_grad,
                              const float *grad_spikes, const float *grad_vmem, const float *vmem,
                              const float *surr, const float *vmem_post_initial,
                              const float *alpha, const float *membr_subtract, const float *theta,
                              const float *theta_low, int apply_theta_low, int max_num_spikes,
                              int surrogate_kind, float surr_p0, float surr_p1, int64_t n,
                              int64_t t, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Synapse + membrane in one kernel per direction.  The reference composes this stage from four
 * passes: input * alpha_syn (reference sinabs/exodus/layers/lif.py:190-191), LeakyIntegrator
 * (lif.py:194-198), (1 - alpha_mem) * i_syn (lif.py:206-209) and IntegrateAndFire (lif.py:245-254),
 * and lets torch autograd chain their gradients.  These two entry points compute the same
 * values with the operations in the same order.
 * ------------------------------------------------------------------------------------------- */

/* Per row and step:
 *   xin = decay_early ? input*alpha_syn : input;  i = i*alpha_syn + xin;
 *   u = norm_input ? (1 - alpha_mem)*i : i;       v = (v - count*membr_subtract)*alpha_mem + u;
 *   clamp at theta_low if apply_theta_low;        count = v >= theta ? min((unsigned)(v/theta), cap) : 0
 * Writes count to out_spikes, v (before reset) to out_vmem and i to out_isyn, all (n,t). */
int exodus_synlif_forward(float *out_spikes, float *out_vmem, float *out_isyn, const float *input,
                          const float *vmem_post_initial, const float *isyn_initial,
                          const float *alpha_mem, const float *alpha_syn, const float *membr_subtract,
                          const float *theta, const float *theta_low, int apply_theta_low,
                          int max_num_spikes, int decay_early, int norm_input, int64_t n, int64_t t,
                          void *stream);

/* Reverse pass of the above from the saved vmem and isyn.  grad_vmem and grad_isyn (gradients
 * arriving at the vmem / isyn outputs) must be both given or both NULL.  Outputs: grad_input (n,t)
 * and, each optional (NULL = not wanted), the per-row alpha_mem_grad, alpha_syn_grad,
 * vmem_init_grad, isyn_init_grad.  surrogate_kind must be one of the in-kernel kinds (1..3).
 * alpha_syn_grad with decay_early divides by alpha_syn and is therefore undefined for rows
 * whose alpha_syn is exactly 0. */
int exodus_synlif_backward(float *grad_input, float *alpha_mem_grad, float *alpha_syn_grad,
                           float *vmem_init_grad, float *isyn_init_grad, const float *grad_spikes,
                           const float *grad_vmem, const float *grad_isyn, const float *vmem,
                           const float *isyn, const float *vmem_post_initial, const float *isyn_initial,
                           const float *alpha_mem, const float *alpha_syn, const float *membr_subtract,
                           const float *theta, const float *theta_low, int apply_theta_low,
                           int max_num_spikes, int decay_early, int norm_input, int surrogate_kind,
                           float surr_p0, float surr_p1, int64_t n, int64_t t, void *stream);

/* ---------------------------------------------------------------------------------------------
 * The spiking layer on its own memory layout.  The reference layer transposes its
 * (batch, time, *neurons) input into (rows, time), runs the Functions and views the results back
 * (reference sinabs/exodus/layers/lif.py:152-183, 260-307).  These entry points work on the
 * (batch, t, neurons) tensors directly (neurons = product of the trailing dimensions, contiguous)
 * and write only what the layer hands out (neurons < 2^25 per batch element: step offsets are
 * 32-bit byte offsets; wider layers get hipErrorInvalidValue and belong on the (rows, time)
 * entry points).  Per-neuron vectors have batch*neurons entries, in
 * the order of the layer's state tensors.
 * ------------------------------------------------------------------------------------------- */

/* Steps between two checkpoints; ckpt tensors hold ceil(t / interval) entries per neuron. */
int exodus_layer_checkpoint_interval(void);

/* Forward of a LIF/IAF layer with (alpha_syn != NULL) or without synaptic current; arithmetic and
 * order as exodus_synlif_forward / exodus_lif_forward after the layer's input scalings.
 *   out_spikes (batch,t,neurons); v_last, i_last (batch*neurons): potential after the last reset
 *   and last synaptic current (i_last may be NULL without synapse).
 * Optional (NULL = skip): out_vmem_rec / out_isyn_rec (batch,t,neurons) potential and synaptic
 * current of every step, the potential after the reset (what the layer records, reference
 * sinabs/exodus/layers/lif.py:256) or, with record_pre_reset != 0, before it (what
 * IntegrateAndFire hands to the surrogate function, reference sinabs/exodus/spike.py:251); ckpt_v / ckpt_i (batch, ceil(t/interval), neurons) state at the
 * start of every checkpoint interval, needed by exodus_layer_lif_backward; spike_sum, one double
 * to which the total spike count is added atomically. */
int exodus_layer_lif_forward(float *out_spikes, float *out_vmem_rec, float *out_isyn_rec, float *ckpt_v,
                             float *ckpt_i, float *v_last, float *i_last, double *spike_sum,
                             const float *input, const float *vmem_post_initial,
                             const float *isyn_initial, const float *alpha_mem, const float *alpha_syn,
                             const float *membr_subtract, const float *theta, const float *theta_low,
                             int apply_theta_low, int max_num_spikes, int decay_early, int norm_input,
                             int record_pre_reset, int64_t batch, int64_t t, int64_t neurons, void *stream);

/* Backward of the above.  Re-reads `input`, rebuilds membrane potential and synaptic current of
 * each checkpoint interval from ckpt_v / ckpt_i and walks it in reverse.  grad_v_last /
 * grad_i_last (batch*neurons, optional) are gradients arriving at the final states.  Outputs:
 * grad_input (batch,t,neurons) and the optional per-neuron alpha_mem_grad, alpha_syn_grad,
 * vmem_init_grad, isyn_init_grad.  With surrogate_kind == EXODUS_SURR_TENSOR the derivative of
 * the spike function at every step comes from `surr` (batch,t,neurons) — what a caller computes
 * from the pre-reset potential record with any function of its own (the reference evaluates an
 * arbitrary Python callable there, sinabs/exodus/spike.py:251); otherwise `surr` is ignored.
 * grad_v_rec / grad_i_rec (batch,t,neurons, optional; with synapse both or none) are gradients
 * arriving at the forward's per-step records of the post-reset potential and the synaptic current
 * (the layer's `recordings` are differentiable, reference sinabs/exodus/layers/lif.py:256,290-293).
 * grad_spikes_uniform != 0: `grad_spikes` points at ONE float that is the gradient of every spike -- what the loss
 * `out.sum()` of the reference's own tests (reference tests/test_spike_functions.py:50, tests/test_leak_functions.py:22) hands back, which
 * autograd represents as a broadcast scalar.  The kernel then streams one tensor less (8 instead of 12 bytes per
 * neuron-timestep).  Only with an in-kernel surrogate (kind 1..3) and without grad_v_rec / grad_i_rec
 * (hipErrorInvalidValue otherwise). */
int exodus_layer_lif_backward(float *grad_input, float *alpha_mem_grad, float *alpha_syn_grad,
                              float *vmem_init_grad, float *isyn_init_grad, const float *grad_spikes,
                              const float *grad_v_last, const float *grad_i_last, const float *input,
                              const float *ckpt_v, const float *ckpt_i, const float *vmem_post_initial,
                              const float *isyn_initial, const float *alpha_mem, const float *alpha_syn,
                              const float *membr_subtract, const float *theta, const float *theta_low,
                              int apply_theta_low, int max_num_spikes, int decay_early, int norm_input,
                              int surrogate_kind, float surr_p0, float surr_p1, const float *surr,
                              const float *grad_v_rec, const float *grad_i_rec, int grad_spikes_uniform,
                              int64_t batch, int64_t t, int64_t neurons, void *stream);

/* How exodus_layer_lif_backward spreads a layer over the machine.  Its ordinary kernel gives every neuron one lane that
 * walks the whole sequence, which leaves most of the GPU idle when a layer has few neurons (the reference's kernels
 * have the same shape: one thread per row, reference cuda/lif_kernels.h:296-311).  For layers without synapse, with an
 * in-kernel surrogate (kind 1..3), without grad_v_rec and with 33 to 512 steps a second kernel gives every chunk of 32
 * steps of every neuron a lane of its own (the adjoint recurrence is affine, so the chunks can be composed afterwards):
 * the same gradients to fp32 rounding, not bit for bit.  mode 0: never use it; 1 (default): for layers of up to 16 384
 * neurons (batch * neurons); 2: whenever it applies; any other value changes nothing.  Returns the mode that was set
 * before.  Process-wide. */
int exodus_layer_backward_time_split(int mode);

/* exodus_layer_lif_backward for callers that cannot allocate device memory -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, outputs and arithmetic as exodus_layer_lif_backward, except that no
 * checkpoints are passed: the checkpoints live in a fixed array of exodus_layer_scratch_floats()
 * floats (2^24 = 64 MiB) inside the library's device image, and this call first runs the forward
 * recurrence once more over `input` to fill them (so vmem_post_initial, and isyn_initial with synapse,
 * are always required), then the backward pass.  A forward that was run without checkpoints
 * (ckpt_v == NULL) therefore suffices.  The batch is walked in slices of as many batch elements as
 * fit the array; if a single batch element does not fit -- ceil(t / interval) * neurons floats, twice
 * that with synapse, more than the array holds -- nothing is launched and
 * EXODUS_ERROR_SCRATCH_TOO_SMALL is returned.  The call allocates and frees nothing and does not
 * synchronise.  Every GPU holds one such array for the life of the process and all calls on a GPU
 * share it: calls on different streams of one GPU that may overlap race on it and must be ordered by
 * the caller. */
int64_t exodus_layer_scratch_floats(void);
int exodus_layer_lif_backward_from_input(float *grad_input, float *alpha_mem_grad, float *alpha_syn_grad,
                                         float *vmem_init_grad, float *isyn_init_grad, const float *grad_spikes,
                                         const float *grad_v_last, const float *grad_i_last, const float *input,
                                         const float *vmem_post_initial, const float *isyn_initial,
                                         const float *alpha_mem, const float *alpha_syn, const float *membr_subtract,
                                         const float *theta, const float *theta_low, int apply_theta_low,
                                         int max_num_spikes, int decay_early, int norm_input, int surrogate_kind,
                                         float surr_p0, float surr_p1, const float *surr, const float *grad_v_rec,
                                         const float *grad_i_rec, int grad_spikes_uniform, int64_t batch, int64_t t,
                                         int64_t neurons, void *stream);

/* Forward of the non-spiking leaky-integrator layer (ExpLeak) on (batch,t,neurons): per neuron
 *   xin = norm_input ? (1 - alpha) * input : input;  xin = decay_early ? xin * alpha : xin;
 *   out_t = alpha * out_{t-1} + xin_t,  out_{-1} = vmem_initial
 * (reference sinabs/exodus/layers/lif.py:206-223).  v_last (batch*neurons) receives out[:, -1];
 * out_sum (optional, one double that the caller has zeroed) receives the sum of all outputs, which
 * the layer divides by their number (lif.py:305) without reading the output again. */
int exodus_layer_leaky_forward(float *out, float *v_last, double *out_sum, const float *input,
                               const float *vmem_initial, const float *alpha, int decay_early, int norm_input,
                               int64_t batch, int64_t t, int64_t neurons, void *stream);

/* Backward of the above: grad_input (batch,t,neurons); optional per-neuron alpha_grad (needs `out`
 * and `vmem_initial`, and `input` when one of the input scalings is on) and vmem_init_grad;
 * grad_v_last (batch*neurons, optional) is a gradient arriving at the final state.
 * grad_out_uniform != 0: `grad_out` points at ONE float that stands for every element (as grad_spikes_uniform of
 * exodus_layer_lif_backward). */
int exodus_layer_leaky_backward(float *grad_input, float *alpha_grad, float *vmem_init_grad,
                                const float *grad_out, const float *grad_v_last, const float *out,
                                const float *input, const float *vmem_initial, const float *alpha,
                                int decay_early, int norm_input, int grad_out_uniform, int64_t batch, int64_t t,
                                int64_t neurons, void *stream);

/* ---- experimental spike generation on a precomputed membrane potential -------------------------
 * Replaces spikeForward (reference cuda/bindings.cu:262-290, kernel
 * cuda/experimental_kernels.h:16-65).  vmem (n, t) holds the response to the input and is updated
 * in place with the effect of resets (each spike lowers every later step by alpha^j *
 * membr_subtract * count) and of the lower bound (a step below theta_low keeps its value and raises
 * every later step by alpha^j * (theta_low - u)); out_spikes (n, t) receives
 * min(trunc(u / theta), max_num_spikes) where u >= theta, else 0 (max_num_spikes < 0: no cap).
 * Parameters are scalars, as in the reference.  The corrections are accumulated in one running
 * value per row (O(t) instead of the reference's O(t^2)), so potentials agree with the reference to
 * float rounding, not bit for bit.  spikeBackwardRefr (cuda/bindings.cu:292-325), which no Python
 * code of the reference calls, has no counterpart. */
int exodus_spike_forward(float *out_spikes, float *vmem, float alpha, float membr_subtract, float theta,
                         float theta_low, int apply_theta_low, int max_num_spikes, int64_t n, int64_t t,
                         void *stream);

/* Replaces spikeBackward (reference cuda/bindings.cu:327-359, kernel
 * cuda/experimental_kernels.h:95-141): gradient with respect to the potential handed to
 * exodus_spike_forward, from surr, output_grad and not_clipped (all (n, t)), as one reverse pass. */
int exodus_spike_backward(float *input_grad, const float *surr, const float *output_grad,
                          const float *not_clipped, float alpha, float membr_subtract, int64_t n,
                          int64_t t, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Device memory sorted by HBM region (no counterpart in the reference, whose extension leaves the
 * placement of its tensors to torch's allocator, reference cuda/bindings.cu:98,144,183)
 * ------------------------------------------------------------------------------------------- */

/* The HBM of an MI355X behaves as three regions.  A kernel's writes are held back by the region they go to: the
 * layer kernels write at 5.6 TB/s into one region and at 6.0-6.3 TB/s into memory whose 64 MiB pages alternate
 * between the regions; a kernel that reads one region and writes another moves 8-12 % more than one that does both
 * inside one region.
 * exodus_hbm_regions_create takes nearly all free device memory in chunks of chunk_bytes (a multiple of
 * EXODUS_HBM_PAGE_BYTES; 4 GiB is a good value: copies of less tell the regions apart less clearly), finds by timed
 * copies which chunks lie in one region, and builds four address ranges: ranges 0-2 hold
 * ceil(bytes_per_region / chunk_bytes) chunks of one region each; range 3 (the striped one) holds bytes_striped,
 * rounded up to a multiple of three chunks, in pages of EXODUS_HBM_PAGE_BYTES that come from chunks of regions 0, 1,
 * 2, 0, 1, 2, ... in turn.  Either size may be 0 (that range is then absent, base NULL).  The rest goes back to the
 * driver.  report->base[k] / bytes[k] are the ranges; the caller hands out memory from them as it likes (the Python
 * host side is sinabs/exodus/hbm.py) and must stop using them before exodus_hbm_regions_destroy.
 * When the copies do not show three kinds of chunks with a clear gap (memory that earlier processes allocated and
 * freed in small pieces comes back as a mixture of the regions below the size of a chunk): with bytes_per_region > 0
 * the call returns EXODUS_ERROR_REGIONS_NOT_FOUND (the report's fields up to kinds_found are then filled); with only
 * a striped range asked for it succeeds with kinds_found < 3, the pages taking turns between chunks spread evenly
 * over the memory instead.  sort = 0 skips the timed copies and builds the striped range that way at once
 * (kinds_found = 0; bytes_per_region must be 0): cheaper, and enough on a machine whose memory is known to come back
 * mixed.  hipErrorOutOfMemory when too little memory is free to find or fill the ranges,
 * hipErrorInvalidValue for bad arguments or a device that already has its ranges.  Takes a second or two;
 * synchronises the device.
 * While it works the call holds nearly all free memory of the device (all but 6 GiB, then all but 512 MiB): another
 * process that allocates on the same GPU in that second can run out of memory.  take_limit_bytes > 0 bounds what is
 * held (rounded down to whole chunks; hipErrorOutOfMemory when that is less than the ranges plus the 15 probe chunks
 * need): memory beyond the bound is neither sorted nor kept from supplying pages, so on a machine that hands memory
 * out in address order a bound below two thirds of the device leaves the ranges in one or two regions. */
#define EXODUS_HBM_REGIONS 3
#define EXODUS_HBM_ARENAS 4                          /* one range per region, and the striped one */
#define EXODUS_HBM_PAGE_BYTES (64ull << 20)          /* stripe width; 32-128 MiB measured alike, 8 and 512 MiB worse */
#define EXODUS_HBM_PROBES 15
typedef struct exodus_hbm_report {
    void *base[EXODUS_HBM_ARENAS];
    uint64_t bytes[EXODUS_HBM_ARENAS];
    uint64_t chunk_bytes, page_bytes;
    int32_t chunks_examined;                         /* physical chunks taken for sorting */
    int32_t kinds_found;                             /* groups among the probe chunks; 3 on success */
    int32_t chunks_ambiguous;                        /* chunks that matched no region clearly (not used) */
    int32_t chunks_of_region[EXODUS_HBM_REGIONS];    /* chunks sorted into each region before enough were found */
    float threshold_GBs;                             /* copy rate that separated "same region" from "other" */
    float probe_same_kind_GBs, probe_other_kind_GBs; /* mean copy rate between probe chunks of one / of two regions */
    float copy_inside_GBs[EXODUS_HBM_REGIONS];       /* finished ranges: first half of range k into its second half */
    float copy_across_GBs[6];                        /* range j into range k: (0,1) (0,2) (1,0) (1,2) (2,0) (2,1) */
    float copy_striped_GBs;                          /* first half of the striped range into its second half */
    int32_t probe_chunk[EXODUS_HBM_PROBES];          /* the probe chunks (position in the order of creation), */
    int32_t probe_kind[EXODUS_HBM_PROBES];           /* the group each was put in, and the copy rate between every */
    float probe_pair_GBs[EXODUS_HBM_PROBES][EXODUS_HBM_PROBES];   /* two of them (mean of both directions) */
    float phase_s[4];                                /* seconds spent taking the memory, sorting it, building the ranges, checking them */
} exodus_hbm_report;
int exodus_hbm_regions_create(int device, uint64_t bytes_per_region, uint64_t bytes_striped, uint64_t chunk_bytes,
                              int sort, uint64_t take_limit_bytes, exodus_hbm_report *report);
/* Gives the ranges' memory back to the driver.  EXODUS_ERROR_RANGE_IN_USE, and nothing happens, while any piece
 * handed out by exodus_hbm_alloc_* has not come back through exodus_hbm_free. */
int exodus_hbm_regions_destroy(int device);

/* Pieces of the ranges, in the signature PyTorch's pluggable allocator binds
 * (torch.cuda.memory.CUDAPluggableAllocator(path, "exodus_hbm_alloc_striped", "exodus_hbm_free")), so that a
 * torch.cuda.MemPool can sit on top of a range: PyTorch's caching allocator then asks these functions for whole
 * segments, splits and reuses them itself and keeps track of which stream still uses what, as it does for ordinary
 * memory -- the tensors of such a pool are as safe across streams as any other tensor.  exodus_hbm_alloc_striped
 * takes from the striped range, _region0/1/2 from the range of one region: first fit from the lowest address, sizes
 * rounded up to 2 MiB, neighbours joined on release.  When the device has no such range (never created, destroyed,
 * size 0) or the range has no room, the memory comes from hipMalloc instead and exodus_hbm_free returns it with
 * hipFree: the caller always gets memory, only the placement is lost.  NULL only when hipMalloc fails too.  `stream`
 * is ignored (nothing here is ordered by streams: a caller without an allocator like PyTorch's on top must free a
 * piece only after all work that uses it has finished).  exodus_hbm_free ignores pointers it did not hand out.
 * Thread safe.  exodus_hbm_usage reports the bytes handed out from each range (bytes_in_use[4]) and, optionally,
 * what was taken from hipMalloc instead. */
void *exodus_hbm_alloc_striped(size_t size, int device, void *stream);
void *exodus_hbm_alloc_region0(size_t size, int device, void *stream);
void *exodus_hbm_alloc_region1(size_t size, int device, void *stream);
void *exodus_hbm_alloc_region2(size_t size, int device, void *stream);
void exodus_hbm_free(void *ptr, size_t size, int device, void *stream);
int exodus_hbm_usage(int device, uint64_t *bytes_in_use, uint64_t *bytes_elsewhere);

#ifdef __cplusplus
}
#endif
#endif /* EXODUS_HIP_H */
