// Sliding-window contraction behind N-d convolution and its cotangents:
//
//   out[i, j, p] = sum_{d, k} filter[i, d, k] * signal[j, d, p + k - pad]     (zero outside the signal)
//
// The reference forms an as_strided window view of the (explicitly zero-padded) signal and hands
// it to einsum (scipy/signal.py:45-65).  Here neither the padding nor the view exists: a thread
// owns one output position, walks the window, and skips the taps that fall off the signal.  Flips
// arrive as negative strides.  The filter address is the same for every lane of a block (i comes
// from the block index), so those loads are wave-uniform; neighbouring lanes read neighbouring
// signal elements.
//
// Two shapes of problem occur.  The forward pass and the signal's cotangent have many outputs and
// a short reduction (channels x window): one lane per output (LANES == 1).  The filter's
// cotangent has few outputs (channels x channels x window) and a reduction over batch x image:
// LANES lanes share one output, stride through the flattened reduction index and combine in LDS
// in a fixed tree order.
#include "common.h"

namespace agmi {

struct CorrParams {
    int64_t I, J, D;
    int64_t K[3], N[3], pad[3], P[3];
    int64_t f_bs, f_ds, f_s[3];
    int64_t s_bs, s_ds, s_s[3];
    int64_t o_fs, o_ss, o_s[3];
    uint32_t p_total;  // P[0] * P[1] * P[2]
    uint32_t k_total;  // K[0] * K[1] * K[2]
    uint32_t tiles;    // blocks per (i, j) pair
};

template <typename T>
__device__ __forceinline__ T fused_mul_add(T a, T b, T c);
template <>
__device__ __forceinline__ float fused_mul_add<float>(float a, float b, float c) {
    return __builtin_fmaf(a, b, c);
}
template <>
__device__ __forceinline__ double fused_mul_add<double>(double a, double b, double c) {
    return __builtin_fma(a, b, c);
}

template <typename T, int LANES>
__global__ __launch_bounds__(kBlock) void correlate_kernel(const T *__restrict__ filter, const T *__restrict__ signal,
                                                           T *__restrict__ out, const CorrParams c) {
    constexpr int kPositions = kBlock / LANES;
    const uint32_t tile = blockIdx.x % c.tiles;
    const uint32_t pair = blockIdx.x / c.tiles;
    const int64_t j = pair / static_cast<uint32_t>(c.I), i = pair % static_cast<uint32_t>(c.I);
    const int lane = threadIdx.x % LANES;
    const uint32_t flat = tile * kPositions + threadIdx.x / LANES;
    const bool live = flat < c.p_total;
    uint32_t q = live ? flat : 0u;
    const int64_t p2 = q % static_cast<uint32_t>(c.P[2]);
    q /= static_cast<uint32_t>(c.P[2]);
    const int64_t p1 = q % static_cast<uint32_t>(c.P[1]);
    const int64_t p0 = q / static_cast<uint32_t>(c.P[1]);
    const T *f = filter + i * c.f_bs;
    const T *s = signal + j * c.s_bs;
    // signal position of window tap 0 on each axis
    const int64_t b0 = p0 - c.pad[0], b1 = p1 - c.pad[1], b2 = p2 - c.pad[2];
    T acc = T(0);
    if constexpr (LANES == 1) {
        for (int64_t d = 0; d < c.D; ++d) {
            const T *fd = f + d * c.f_ds;
            const T *sd = s + d * c.s_ds;
            for (int64_t k0 = 0; k0 < c.K[0]; ++k0) {
                const int64_t s0 = b0 + k0;
                if (static_cast<uint64_t>(s0) >= static_cast<uint64_t>(c.N[0])) continue;
                for (int64_t k1 = 0; k1 < c.K[1]; ++k1) {
                    const int64_t s1 = b1 + k1;
                    if (static_cast<uint64_t>(s1) >= static_cast<uint64_t>(c.N[1])) continue;
                    const T *fr = fd + k0 * c.f_s[0] + k1 * c.f_s[1];
                    const T *sr = sd + s0 * c.s_s[0] + s1 * c.s_s[1];
                    for (int64_t k2 = 0; k2 < c.K[2]; ++k2) {
                        const int64_t s2 = b2 + k2;
                        if (static_cast<uint64_t>(s2) < static_cast<uint64_t>(c.N[2]))
                            acc = fused_mul_add(fr[k2 * c.f_s[2]], sr[s2 * c.s_s[2]], acc);
                    }
                }
            }
        }
        if (live) out[i * c.o_fs + j * c.o_ss + p0 * c.o_s[0] + p1 * c.o_s[1] + p2 * c.o_s[2]] = acc;
    } else {
        const uint32_t r_total = static_cast<uint32_t>(c.D) * c.k_total;
        const uint32_t K2 = static_cast<uint32_t>(c.K[2]), K1 = static_cast<uint32_t>(c.K[1]),
                       K0 = static_cast<uint32_t>(c.K[0]);
        for (uint32_t r = lane; r < r_total; r += LANES) {
            uint32_t t = r;
            const int64_t k2 = t % K2;
            t /= K2;
            const int64_t k1 = t % K1;
            t /= K1;
            const int64_t k0 = t % K0;
            const int64_t d = t / K0;
            const int64_t s0 = b0 + k0, s1 = b1 + k1, s2 = b2 + k2;
            if (static_cast<uint64_t>(s0) < static_cast<uint64_t>(c.N[0]) &&
                static_cast<uint64_t>(s1) < static_cast<uint64_t>(c.N[1]) &&
                static_cast<uint64_t>(s2) < static_cast<uint64_t>(c.N[2]))
                acc = fused_mul_add(f[d * c.f_ds + k0 * c.f_s[0] + k1 * c.f_s[1] + k2 * c.f_s[2]],
                                    s[d * c.s_ds + s0 * c.s_s[0] + s1 * c.s_s[1] + s2 * c.s_s[2]], acc);
        }
        __shared__ T partial[kBlock];
        partial[threadIdx.x] = acc;
        __syncthreads();
        for (int half = LANES / 2; half > 0; half >>= 1) {
            if (lane < half) partial[threadIdx.x] = partial[threadIdx.x] + partial[threadIdx.x + half];
            __syncthreads();
        }
        if (lane == 0 && live)
            out[i * c.o_fs + j * c.o_ss + p0 * c.o_s[0] + p1 * c.o_s[1] + p2 * c.o_s[2]] = partial[threadIdx.x];
    }
}

template <typename T, int LANES>
void launch_correlate(const agmi_correlation *a, CorrParams &c, hipStream_t s) {
    constexpr int kPositions = kBlock / LANES;
    c.tiles = static_cast<uint32_t>(ceil_div(c.p_total, kPositions));
    const int64_t blocks = static_cast<int64_t>(c.tiles) * c.I * c.J;
    hipLaunchKernelGGL((correlate_kernel<T, LANES>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, s,
                       static_cast<const T *>(a->filter.data), static_cast<const T *>(a->signal.data),
                       static_cast<T *>(a->out), c);
}

}  // namespace agmi

using namespace agmi;

extern "C" int agmi_correlate(int dtype, const agmi_correlation *a, void *stream) {
    if (!a) {
        set_error("correlate: null argument block");
        return AGMI_ERR_ARG;
    }
    if (dtype != AGMI_F32 && dtype != AGMI_F64) {
        set_error("correlate: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    if (a->n_conv < 1 || a->n_conv > AGMI_MAX_CONV_DIMS) {
        set_error("correlate: %d convolved axes (1..%d supported)", a->n_conv, AGMI_MAX_CONV_DIMS);
        return AGMI_ERR_UNSUPPORTED;
    }
    if (a->filter_batch < 0 || a->signal_batch < 0 || a->dot < 0) {
        set_error("correlate: negative extent");
        return AGMI_ERR_ARG;
    }
    CorrParams c{};
    c.I = a->filter_batch;
    c.J = a->signal_batch;
    c.D = a->dot;
    // unused leading slots are axes of extent 1, so the innermost convolved axis is always slot 2
    for (int d = 0; d < 3; ++d) {
        c.K[d] = c.N[d] = c.P[d] = 1;
        c.pad[d] = c.f_s[d] = c.s_s[d] = c.o_s[d] = 0;
    }
    int64_t p_total = 1, k_total = 1;
    for (int d = 0; d < a->n_conv; ++d) {
        const int slot = 3 - a->n_conv + d;
        if (a->window[d] < 0 || a->extent[d] < 0 || a->out_extent[d] < 0) {
            set_error("correlate: negative extent on convolved axis %d", d);
            return AGMI_ERR_ARG;
        }
        c.K[slot] = a->window[d];
        c.N[slot] = a->extent[d];
        c.pad[slot] = a->pad_before[d];
        c.P[slot] = a->out_extent[d];
        c.f_s[slot] = a->filter.strides[d];
        c.s_s[slot] = a->signal.strides[d];
        c.o_s[slot] = a->out_strides[d];
        p_total *= c.P[slot];
        k_total *= c.K[slot];
        if (p_total > 0x7fffffffLL || k_total > 0x7fffffffLL) {
            set_error("correlate: more than 2^31 output positions or window taps");
            return AGMI_ERR_UNSUPPORTED;
        }
    }
    const int64_t outputs = c.I * c.J * p_total;
    if (outputs == 0) return 0;
    const int64_t r_total = c.D * k_total;
    if (r_total > 0x7fffffffLL || c.I > 0x7fffffffLL || c.J > 0x7fffffffLL) {
        set_error("correlate: reduction of %lld terms is too long", static_cast<long long>(r_total));
        return AGMI_ERR_UNSUPPORTED;
    }
    if (!a->out || (r_total > 0 && (!a->filter.data || !a->signal.data))) {
        set_error("correlate: null operand");
        return AGMI_ERR_ARG;
    }
    c.f_bs = a->filter.batch_stride;
    c.f_ds = a->filter.dot_stride;
    c.s_bs = a->signal.batch_stride;
    c.s_ds = a->signal.dot_stride;
    c.o_fs = a->out_filter_stride;
    c.o_ss = a->out_signal_stride;
    c.p_total = static_cast<uint32_t>(p_total);
    c.k_total = static_cast<uint32_t>(k_total);

    // lanes per output: enough threads to occupy 256 CUs, never more lanes than half the reduction
    int lanes = 1;
    constexpr int64_t kThreadsWanted = 1 << 18;
    for (int cand : {8, 64, 256})
        if (outputs * lanes < kThreadsWanted && r_total >= 2 * cand) lanes = cand;
    const int64_t blocks = ceil_div(p_total, kBlock / lanes) * c.I * c.J;
    if (blocks > 0x7fffffffLL) {
        set_error("correlate: too many outputs for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    set_kernel_name("correlate_kernel<%s, %d>", dtype == AGMI_F32 ? "float" : "double", lanes);
#define AGMI_CORR(T)                                               \
    switch (lanes) {                                               \
        case 1: launch_correlate<T, 1>(a, c, s); break;            \
        case 8: launch_correlate<T, 8>(a, c, s); break;            \
        case 64: launch_correlate<T, 64>(a, c, s); break;          \
        default: launch_correlate<T, 256>(a, c, s); break;         \
    }
    if (dtype == AGMI_F32) {
        AGMI_CORR(float)
    } else {
        AGMI_CORR(double)
    }
#undef AGMI_CORR
    return hip_check(hipGetLastError(), "correlate launch");
}
