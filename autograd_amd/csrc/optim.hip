// Fused parameter updates for the training loop around the gradient evaluation: one pass over
// the flat parameter vector instead of the 6-12 whole-array NumPy passes of the reference's
// optimizers (autograd/misc/optimizers.py:33-75).  Element arithmetic follows the reference
// expression by expression, so results are bit-identical to the NumPy passes:
//   sgd      (40-47): velocity = mass * velocity - (1.0 - mass) * g;  x = x + step_size * velocity
//   rmsprop  (54-59): avg = avg * gamma + g**2 * (1 - gamma);  x = x - step_size * g / (sqrt(avg) + eps)
//   adam     (66-75): m = (1 - b1) * g + b1 * m;  v = (1 - b2) * (g**2) + b2 * v;
//                     mhat = m / (1 - b1**(i + 1));  vhat = v / (1 - b2**(i + 1));
//                     x = x - step_size * mhat / (sqrt(vhat) + eps)
// The reference creates its state with np.zeros/np.ones (float64), so under NumPy promotion state
// and updated parameters are float64 whatever the parameter dtype; sub-expressions that involve
// only g (float32 gradients on the first step) are rounded in g's dtype first, as NumPy does.
// HBM-bound: adam reads x, g, m, v and writes m, v, x once each.
#include "common.h"

namespace agmi {

struct OptParams {
    const void *x_in;
    const void *g;
    double *s0;
    double *s1;
    double *x_out;
    int64_t n;
    double h[8];
};

template <int KIND, typename TX, typename TG>
__global__ __launch_bounds__(kBlock) void optimizer_step_kernel(const OptParams p) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= p.n) return;
    const double x = static_cast<double>(static_cast<const TX *>(p.x_in)[e]);
    const TG g = static_cast<const TG *>(p.g)[e];
    if (KIND == AGMI_OPT_SGD) {  // h = {mass, 1 - mass, step}
        const double t1 = p.h[0] * p.s0[e];
        const double t2 = static_cast<double>(static_cast<TG>(p.h[1]) * g);
        const double vel = t1 - t2;
        p.s0[e] = vel;
        p.x_out[e] = x + p.h[2] * vel;
    } else if (KIND == AGMI_OPT_RMSPROP) {  // h = {gamma, 1 - gamma, step, eps}
        const double t1 = p.s0[e] * p.h[0];
        const double t2 = static_cast<double>((g * g) * static_cast<TG>(p.h[1]));
        const double avg = t1 + t2;
        p.s0[e] = avg;
        const double num = static_cast<double>(static_cast<TG>(p.h[2]) * g);
        p.x_out[e] = x - num / (sqrt(avg) + p.h[3]);
    } else {  // adam: h = {1 - b1, b1, 1 - b2, b2, 1 - b1**t, 1 - b2**t, step, eps}
        const double m = static_cast<double>(static_cast<TG>(p.h[0]) * g) + p.h[1] * p.s0[e];
        const double v = static_cast<double>(static_cast<TG>(p.h[2]) * (g * g)) + p.h[3] * p.s1[e];
        p.s0[e] = m;
        p.s1[e] = v;
        const double mhat = m / p.h[4];
        const double vhat = v / p.h[5];
        p.x_out[e] = x - (p.h[6] * mhat) / (sqrt(vhat) + p.h[7]);
    }
}

template <int KIND>
static void launch_kind(int x_dtype, int g_dtype, const OptParams &p, dim3 grid, hipStream_t s) {
    if (x_dtype == AGMI_F32 && g_dtype == AGMI_F32)
        hipLaunchKernelGGL((optimizer_step_kernel<KIND, float, float>), grid, dim3(kBlock), 0, s, p);
    else if (x_dtype == AGMI_F32)
        hipLaunchKernelGGL((optimizer_step_kernel<KIND, float, double>), grid, dim3(kBlock), 0, s, p);
    else if (g_dtype == AGMI_F32)
        hipLaunchKernelGGL((optimizer_step_kernel<KIND, double, float>), grid, dim3(kBlock), 0, s, p);
    else
        hipLaunchKernelGGL((optimizer_step_kernel<KIND, double, double>), grid, dim3(kBlock), 0, s, p);
}

}  // namespace agmi

using namespace agmi;

extern "C" int agmi_optimizer_step(int kind, int x_dtype, int g_dtype, int64_t n, const void *x_in, const void *g,
                                   void *s0, void *s1, void *x_out, const double *hyper, void *stream) {
    if (kind != AGMI_OPT_SGD && kind != AGMI_OPT_RMSPROP && kind != AGMI_OPT_ADAM) {
        set_error("optimizer_step: unknown kind %d", kind);
        return AGMI_ERR_ARG;
    }
    if ((x_dtype != AGMI_F32 && x_dtype != AGMI_F64) || (g_dtype != AGMI_F32 && g_dtype != AGMI_F64)) {
        set_error("optimizer_step: parameters and gradients must be float32 or float64");
        return AGMI_ERR_ARG;
    }
    if (n < 0) {
        set_error("optimizer_step: negative length");
        return AGMI_ERR_ARG;
    }
    if (n == 0) return 0;
    if (!x_in || !g || !s0 || !x_out || !hyper || (kind == AGMI_OPT_ADAM && !s1)) {
        set_error("optimizer_step: null operand");
        return AGMI_ERR_ARG;
    }
    const int64_t blocks = ceil_div(n, kBlock);
    if (blocks > 0x7fffffffLL) {
        set_error("optimizer_step: too many elements");
        return AGMI_ERR_UNSUPPORTED;
    }
    OptParams p;
    p.x_in = x_in;
    p.g = g;
    p.s0 = static_cast<double *>(s0);
    p.s1 = static_cast<double *>(s1);
    p.x_out = static_cast<double *>(x_out);
    p.n = n;
    const int n_hyper = kind == AGMI_OPT_SGD ? 3 : kind == AGMI_OPT_RMSPROP ? 4 : 8;
    for (int k = 0; k < 8; ++k) p.h[k] = k < n_hyper ? hyper[k] : 0.0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<unsigned>(blocks));
    if (kind == AGMI_OPT_SGD) {
        set_kernel_name("optimizer_step<sgd>");
        launch_kind<AGMI_OPT_SGD>(x_dtype, g_dtype, p, grid, s);
    } else if (kind == AGMI_OPT_RMSPROP) {
        set_kernel_name("optimizer_step<rmsprop>");
        launch_kind<AGMI_OPT_RMSPROP>(x_dtype, g_dtype, p, grid, s);
    } else {
        set_kernel_name("optimizer_step<adam>");
        launch_kind<AGMI_OPT_ADAM>(x_dtype, g_dtype, p, grid, s);
    }
    return hip_check(hipGetLastError(), "optimizer_step launch");
}
