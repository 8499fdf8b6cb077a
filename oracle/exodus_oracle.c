/*
 * TEST INFRASTRUCTURE ONLY -- not part of the shipped library.
 *
 * Scalar CPU restatement of the arithmetic of the six production device
 * routines of the EXODUS reference and of its experimental spike-generation
 * pair (one row = one neuron, sequential in time).  Each function names the reference lines it follows.  The loops are
 * written row-major over an (n_rows, n_steps) fp32 matrix with 64-bit
 * offsets.  Build with -ffp-contract=off so that every multiply and add is
 * rounded on its own, which is what the HIP kernels are checked against
 * bit for bit in the forward direction.
 *
 * Only tests, the smoke check and the benchmark's CPU-baseline leg may load
 * this file's shared object.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   oracle_leaky_forward        closed form a^(t+1) v0 + sum a^(t-k) x_k, cumsum at a=1,
 *                               single-pulse decay of reference tests/test_exp_leak.py:53-75
 *   oracle_leaky_backward       transpose identity <go, F(x)> == <B(go), x>, flip identity
 *   oracle_leaky_backward_alpha central finite differences of the forward in fp64
 *   oracle_lif_forward          Gradient_analysis.ipynb cells 2/4/6 known answers,
 *                               floor(cumsum(x)/theta) identity for IAF
 *   oracle_lif_backward         notebook cell 4/6 gradients, product closed form of cell 0/7,
 *                               the O(T) reverse recurrence, torch autograd BPTT
 *   oracle_lif_backward_alpha   torch autograd BPTT (only where step 0 is not clipped or
 *                               v_init == 0, see the note at the function)
 *   oracle_spike_forward        notebook cells 2/4/6 on cumsum(input); bit-equality with
 *                               oracle_lif_forward on a dyadic grid where all arithmetic is exact
 *   oracle_spike_backward       equality with oracle_lif_backward at alpha == 1; for every alpha and
 *                               with clipped steps: torch autograd through an independent step loop of
 *                               the model whose exact gradient the reference's sum is (a spike reaches the
 *                               next step undecayed, a clipped step's lift counts as a constant); its
 *                               distance to the exact gradient of oracle_spike_forward is measured there
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define EXPORT __attribute__((visibility("default")))

/* float -> unsigned the way the device does it (saturating: negative and NaN give 0, values
 * beyond 32 bits give UINT_MAX).  A plain C cast is undefined for those inputs; they occur when a
 * threshold is not positive. */
static unsigned to_unsigned_sat(float q)
{
    if (!(q > 0.0f))
        return 0u;
    if (q >= 4294967296.0f)
        return 0xffffffffu;
    return (unsigned)q;
}

/* number of worker threads used by the row loops (1 = scalar) */
static int g_threads = 1;

EXPORT void oracle_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
EXPORT int oracle_get_threads(void) { return g_threads; }

/* v_t = alpha * v_{t-1} + x_t            reference cuda/leaky_kernels.h:41-56 */
EXPORT void oracle_leaky_forward(float *out, const float *in, const float *v_init,
                                 const float *alpha, int64_t n_rows, int64_t n_steps)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        const float a = alpha[r];
        const float *x = in + r * n_steps;
        float *o = out + r * n_steps;
        float v = v_init[r];
        for (int64_t t = 0; t < n_steps; ++t) {
            v = v * a;
            v = v + x[t];
            o[t] = v;
        }
    }
}

/* g_t = alpha * g_{t+1} + go_t, walking time backwards
 *                                        reference cuda/leaky_kernels.h:94-108 */
EXPORT void oracle_leaky_backward(float *grad_in, const float *grad_out, const float *alpha,
                                  int64_t n_rows, int64_t n_steps)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        const float a = alpha[r];
        const float *go = grad_out + r * n_steps;
        float *gi = grad_in + r * n_steps;
        float g = 0.0f;
        for (int64_t t = n_steps - 1; t >= 0; --t) {
            g = g * a + go[t];
            gi[t] = g;
        }
    }
}

/* d/d alpha of sum_t go_t * out_t: D_0 = v_init, D_t = alpha D_{t-1} + out_{t-1},
 * result = sum_t D_t go_t                reference cuda/leaky_kernels.h:146-163 */
EXPORT void oracle_leaky_backward_alpha(float *grad_alpha, const float *grad_out, const float *out,
                                        const float *v_init, const float *alpha, int64_t n_rows,
                                        int64_t n_steps)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        const float a = alpha[r];
        const float *go = grad_out + r * n_steps;
        const float *o = out + r * n_steps;
        float d = v_init[r];
        float acc = d * go[0];
        for (int64_t t = 1; t < n_steps; ++t) {
            d = a * d + o[t - 1];
            acc += d * go[t];
        }
        grad_alpha[r] = acc;
    }
}

/* Spiking membrane update; v is stored BEFORE the reset of its own step.
 *   v -= count_prev * c;  v *= alpha;  v += x_t;  clamp at lo;  count = v >= theta ?
 *   min((unsigned)(v / theta), max_spikes) : 0
 * max_spikes < 0 means "no cap" (the reference passes -1 converted to unsigned)
 *                                        reference cuda/lif_kernels.h:55-91, cuda/bindings.cu:50-51 */
EXPORT void oracle_lif_forward(float *spikes, float *v_mem, const float *in, const float *v_init,
                               const float *alpha, const float *membr_subtract, const float *theta,
                               const float *theta_low, int apply_theta_low, int max_spikes,
                               int64_t n_rows, int64_t n_steps)
{
    const unsigned cap = (unsigned)max_spikes; /* -1 -> UINT_MAX */
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        const float a = alpha[r], c = membr_subtract[r], th = theta[r];
        const float lo = apply_theta_low ? theta_low[r] : 0.0f;
        const float *x = in + r * n_steps;
        float *s = spikes + r * n_steps;
        float *vm = v_mem + r * n_steps;
        float v = v_init[r];
        unsigned count = 0;
        for (int64_t t = 0; t < n_steps; ++t) {
            v = v - (float)count * c;
            v = v * a;
            v = v + x[t];
            if (apply_theta_low && v < lo)
                v = lo;
            if (v >= th) {
                unsigned k = to_unsigned_sat(v / th);
                count = k < cap ? k : cap;
            } else {
                count = 0;
            }
            s[t] = (float)count;
            vm[t] = v;
        }
    }
}

/* Input gradient as the reference defines it, one output element at a time
 * (quadratic in n_steps):
 *   gi_i = nc_i g_i + sum_{j>i} g_j nc_i prod_{k=i+1..j} (alpha - csub * s_{k-1}) nc_k
 * csub is alpha * membrane_subtract (the caller pre-multiplies, spike.py:269).
 * The early exit on an exactly-zero running product is kept.
 *                                        reference cuda/lif_kernels.h:136-166 */
EXPORT void oracle_lif_backward(float *grad_in, const float *grad_out, const float *surr,
                                const float *not_clipped, const float *alpha, const float *csub,
                                int64_t n_rows, int64_t n_steps)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        const float a = alpha[r], cs = csub[r];
        const float *g = grad_out + r * n_steps;
        const float *s = surr + r * n_steps;
        const float *nc = not_clipped + r * n_steps;
        float *gi = grad_in + r * n_steps;
        for (int64_t i = 0; i < n_steps; ++i) {
            float prod = nc[i];
            float acc = g[i] * prod;
            for (int64_t j = i + 1; j < n_steps && prod != 0.0f; ++j) {
                float f = a - cs * s[j - 1];
                prod *= f * nc[j];
                acc += prod * g[j];
            }
            gi[i] = acc;
        }
    }
}

/* Gradient with respect to alpha, forward in time:
 *   D_0 = v_init;  contribution_0 = nc_0 D_0 g_0
 *   D_j = (D_{j-1} * alpha (1 - c s_{j-1}) + vpost_{j-1}) * nc_j;  result += D_j g_j
 * The factor alpha*(1 - c*s) is evaluated in double and then rounded into the
 * float product, as the reference's "1.0 -" literal makes it.
 * NOTE: D_0 enters step 1 without the nc_0 gate.  When step 0 is clipped and
 * v_init != 0 this differs from the exact derivative (which gates it).
 * gate_initial != 0 selects the exact form instead.
 *                                        reference cuda/lif_kernels.h:212-244 */
EXPORT void oracle_lif_backward_alpha(float *grad_alpha, const float *grad_out,
                                      const float *v_post, const float *v_post_init,
                                      const float *surr, const float *not_clipped,
                                      const float *alpha, const float *membr_subtract,
                                      int gate_initial, int64_t n_rows, int64_t n_steps)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        const float a = alpha[r], c = membr_subtract[r];
        const float *g = grad_out + r * n_steps;
        const float *s = surr + r * n_steps;
        const float *nc = not_clipped + r * n_steps;
        const float *vp = v_post + r * n_steps;
        float d = v_post_init[r];
        float first = nc[0] * d;
        float acc = g[0] * first;
        if (gate_initial)
            d = first;
        for (int64_t j = 1; j < n_steps; ++j) {
            d = (float)((double)d * ((double)a * (1.0 - (double)(c * s[j - 1]))));
            d += vp[j - 1];
            d *= nc[j];
            acc += d * g[j];
        }
        grad_alpha[r] = acc;
    }
}

/* ---------------------------------------------------------------------------
 * Experimental spike-generation pair of the reference (spikes from a membrane
 * potential that already contains the response to the input; only the reset
 * and the lower bound act here).  Scalar parameters, as in the reference.
 *
 * What pins these two (tests/test_oracle_pins.py):
 *   oracle_spike_forward   notebook cells 2/4 known answer on cumsum(input); on a dyadic grid
 *                          (all arithmetic exact) it equals oracle_lif_forward applied to the
 *                          input whose leaky integral is the given potential
 *   oracle_spike_backward  alpha = 1, nothing clipped: its leaky adjoint equals the notebook's
 *                          cell 4/6 gradients and oracle_lif_backward.  Any alpha, clipped steps: the
 *                          sum has factors (alpha - c y_k) where the forward pass above would give
 *                          alpha (1 - c y_k); it is the exact gradient of a forward pass in which a
 *                          spike reaches the next step undecayed and the lift of a clipped step is a
 *                          constant, and equals torch autograd through a step loop of that model.  It
 *                          is restated as the reference has it, not corrected.
 * ------------------------------------------------------------------------- */

/* For each step in turn: a potential at or above theta emits min(trunc(u/theta), cap) spikes and
 * every later step of the row loses alpha^j * c * count; otherwise, with the lower bound on, a
 * potential below theta_low leaves its own step untouched and raises every later step by
 * alpha^j * (theta_low - u).  u is updated in place.
 *                                        reference cuda/experimental_kernels.h:33-63 */
EXPORT void oracle_spike_forward(float *spikes, float *u, float alpha, float membr_subtract,
                                 float theta, float theta_low, int apply_theta_low,
                                 int max_num_spikes, int64_t n_rows, int64_t n_steps)
{
    const unsigned cap = (unsigned)max_num_spikes;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        float *v = u + r * n_steps;
        float *s = spikes + r * n_steps;
        for (int64_t i = 0; i < n_steps; ++i) {
            s[i] = 0.0f;
            if (v[i] >= theta) {
                unsigned k = to_unsigned_sat(v[i] / theta);
                if (k > cap)
                    k = cap;
                s[i] = (float)k;
                float w = alpha;
                for (int64_t j = i + 1; j < n_steps; ++j) {
                    float drop = w * membr_subtract;
                    drop = drop * (float)k;
                    v[j] -= drop;
                    w *= alpha;
                }
            } else if (apply_theta_low && v[i] < theta_low) {
                float lift = theta_low - v[i];
                for (int64_t j = i + 1; j < n_steps; ++j) {
                    lift *= alpha;
                    v[j] += lift;
                }
            }
        }
    }
}

/* gi_i = y_i go_i - sum_{j>i} go_j y_j * (y_i c) * prod_{i<k<j} (alpha - c y_k),  y = surr * nc,
 * summed term by term in float with the running product, stopping once the product is zero.
 *                                        reference cuda/experimental_kernels.h:118-140 */
EXPORT void oracle_spike_backward(float *grad_in, const float *grad_out, const float *surr,
                                  const float *not_clipped, float alpha, float membr_subtract,
                                  int64_t n_rows, int64_t n_steps)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        const float *go = grad_out + r * n_steps;
        const float *s = surr + r * n_steps;
        const float *nc = not_clipped + r * n_steps;
        float *gi = grad_in + r * n_steps;
        for (int64_t i = 0; i < n_steps; ++i) {
            float acc = s[i] * nc[i];
            float prod = acc * membr_subtract;
            acc = acc * go[i];
            for (int64_t j = i + 1; j < n_steps && prod != 0.0f; ++j) {
                float term = go[j] * s[j];
                term = term * nc[j];
                term = term * prod;
                acc -= term;
                float f = membr_subtract * nc[j];
                f = f * s[j];
                prod *= alpha - f;
            }
            gi[i] = acc;
        }
    }
}
