// Sliding-window contraction behind N-d convolution and its cotangents:
//
//   out[i, j, p] = sum_{d, k} filter[i, d, k] * signal[j, d, p + k - pad]     (zero outside the signal)
//
// The reference forms an as_strided window view of the (explicitly zero-padded) signal and hands
// it to einsum (scipy/signal.py:45-65).  Here neither the padding nor the view exists: the window
// is walked in place and the taps that fall off the signal are skipped.  Flips arrive as negative
// strides.
//
// Two shapes of problem occur, and each has its kernel.
//
// correlate_positions: the forward pass and the signal's cotangent have many output positions and
// a short reduction (channels x window).  A thread owns one (signal batch, position) pair and a
// tile of TI filter-batch entries (output channels): each signal element it loads feeds TI
// multiply-adds whose filter operands are wave-uniform.
//
// correlate_reduce: the filter's cotangent has few outputs (channels x channels x window) and a
// reduction over batch x image.  A block owns one output; its 256 lanes split the contracted
// axis and the innermost window axis between them (so neighbouring lanes read neighbouring
// elements of both operands), walk the other window axes in nested loops, and combine in LDS in
// a fixed tree order.
#include "common.h"

namespace agmi {

struct CorrParams {
    int64_t I, J, D;
    int64_t K[3], N[3], pad[3], P[3];
    int64_t f_bs, f_ds, f_s[3];
    int64_t s_bs, s_ds, s_s[3];
    int64_t o_fs, o_ss, o_s[3];
    uint32_t p_total;    // P[0] * P[1] * P[2]
    uint32_t tiles;      // correlate_positions: blocks per filter-batch tile
    uint32_t lane_bits;  // correlate_reduce: log2 of the lanes that share the innermost window axis
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

template <typename T, int TI>
__global__ __launch_bounds__(kBlock) void correlate_positions(const T *__restrict__ filter,
                                                              const T *__restrict__ signal, T *__restrict__ out,
                                                              const CorrParams c) {
    const uint32_t tile = blockIdx.x % c.tiles;
    const int64_t i0 = static_cast<int64_t>(blockIdx.x / c.tiles) * TI;
    const uint32_t flat = tile * kBlock + threadIdx.x;
    const bool live = flat < static_cast<uint32_t>(c.J) * c.p_total;
    uint32_t q = live ? flat : 0u;
    const int64_t p2 = q % static_cast<uint32_t>(c.P[2]);
    q /= static_cast<uint32_t>(c.P[2]);
    const int64_t p1 = q % static_cast<uint32_t>(c.P[1]);
    q /= static_cast<uint32_t>(c.P[1]);
    const int64_t p0 = q % static_cast<uint32_t>(c.P[0]);
    const int64_t j = q / static_cast<uint32_t>(c.P[0]);
    // rows of the filter for this block's tile; entries past the last one repeat it (computed, never stored)
    const T *f[TI];
#pragma unroll
    for (int t = 0; t < TI; ++t) {
        const int64_t i = i0 + t < c.I ? i0 + t : c.I - 1;
        f[t] = filter + i * c.f_bs;
    }
    const T *s = signal + j * c.s_bs;
    const int64_t b0 = p0 - c.pad[0], b1 = p1 - c.pad[1], b2 = p2 - c.pad[2];  // signal position of tap 0
    T acc[TI];
#pragma unroll
    for (int t = 0; t < TI; ++t) acc[t] = T(0);
    for (int64_t d = 0; d < c.D; ++d) {
        const T *sd = s + d * c.s_ds;
        const int64_t fd = d * c.f_ds;
        for (int64_t k0 = 0; k0 < c.K[0]; ++k0) {
            const int64_t s0 = b0 + k0;
            const bool in0 = static_cast<uint64_t>(s0) < static_cast<uint64_t>(c.N[0]);
            for (int64_t k1 = 0; k1 < c.K[1]; ++k1) {
                const int64_t s1 = b1 + k1;
                const bool in1 = in0 && static_cast<uint64_t>(s1) < static_cast<uint64_t>(c.N[1]);
                const int64_t fr = fd + k0 * c.f_s[0] + k1 * c.f_s[1];
                const T *sr = sd + s0 * c.s_s[0] + s1 * c.s_s[1];
                for (int64_t k2 = 0; k2 < c.K[2]; ++k2) {
                    const int64_t s2 = b2 + k2;
                    const bool in = in1 && static_cast<uint64_t>(s2) < static_cast<uint64_t>(c.N[2]);
                    const T sv = in ? sr[s2 * c.s_s[2]] : T(0);  // a tap that falls off the signal is padding
                    const int64_t fo = fr + k2 * c.f_s[2];
#pragma unroll
                    for (int t = 0; t < TI; ++t) acc[t] = fused_mul_add(f[t][fo], sv, acc[t]);
                }
            }
        }
    }
    if (!live) return;
    T *o = out + j * c.o_ss + p0 * c.o_s[0] + p1 * c.o_s[1] + p2 * c.o_s[2];
#pragma unroll
    for (int t = 0; t < TI; ++t)
        if (i0 + t < c.I) o[(i0 + t) * c.o_fs] = acc[t];
}

template <typename T>
__global__ __launch_bounds__(kBlock) void correlate_reduce(const T *__restrict__ filter, const T *__restrict__ signal,
                                                           T *__restrict__ out, const CorrParams c) {
    uint32_t q = blockIdx.x;
    const int64_t p2 = q % static_cast<uint32_t>(c.P[2]);
    q /= static_cast<uint32_t>(c.P[2]);
    const int64_t p1 = q % static_cast<uint32_t>(c.P[1]);
    q /= static_cast<uint32_t>(c.P[1]);
    const int64_t p0 = q % static_cast<uint32_t>(c.P[0]);
    q /= static_cast<uint32_t>(c.P[0]);
    const int64_t i = q % static_cast<uint32_t>(c.I), j = q / static_cast<uint32_t>(c.I);
    const int64_t lanes_k = int64_t(1) << c.lane_bits, lanes_d = kBlock >> c.lane_bits;
    const int64_t lk = threadIdx.x & (lanes_k - 1), ld = threadIdx.x >> c.lane_bits;
    const T *f = filter + i * c.f_bs;
    const T *s = signal + j * c.s_bs;
    const int64_t b0 = p0 - c.pad[0], b1 = p1 - c.pad[1], b2 = p2 - c.pad[2];
    // The window rows that meet the signal are found up front (the position is the same for the whole block),
    // so the inner loop is free of bounds tests and the loads of four rows are issued together.
    T acc0 = T(0), acc1 = T(0);
    const int64_t lo = b1 < 0 ? -b1 : 0;                                     // k1 in [lo, hi)
    const int64_t hi = c.N[1] - b1 < c.K[1] ? c.N[1] - b1 : c.K[1];
    for (int64_t k2 = lk; k2 < c.K[2]; k2 += lanes_k) {
        const int64_t s2 = b2 + k2;
        if (static_cast<uint64_t>(s2) >= static_cast<uint64_t>(c.N[2])) continue;
        const T *f2 = f + k2 * c.f_s[2];
        const T *sg2 = s + s2 * c.s_s[2] + b1 * c.s_s[1];
        for (int64_t d = ld; d < c.D; d += lanes_d) {
            for (int64_t k0 = 0; k0 < c.K[0]; ++k0) {
                const int64_t s0 = b0 + k0;
                if (static_cast<uint64_t>(s0) >= static_cast<uint64_t>(c.N[0])) continue;
                const T *fr = f2 + d * c.f_ds + k0 * c.f_s[0];
                const T *sr = sg2 + d * c.s_ds + s0 * c.s_s[0];
                int64_t k1 = lo;
                for (; k1 + 4 <= hi; k1 += 4) {
                    const T fa = fr[k1 * c.f_s[1]], fb = fr[(k1 + 1) * c.f_s[1]];
                    const T fc = fr[(k1 + 2) * c.f_s[1]], fe = fr[(k1 + 3) * c.f_s[1]];
                    const T sa = sr[k1 * c.s_s[1]], sb = sr[(k1 + 1) * c.s_s[1]];
                    const T sc = sr[(k1 + 2) * c.s_s[1]], se = sr[(k1 + 3) * c.s_s[1]];
                    acc0 = fused_mul_add(fa, sa, acc0);
                    acc1 = fused_mul_add(fb, sb, acc1);
                    acc0 = fused_mul_add(fc, sc, acc0);
                    acc1 = fused_mul_add(fe, se, acc1);
                }
                for (; k1 < hi; ++k1) acc0 = fused_mul_add(fr[k1 * c.f_s[1]], sr[k1 * c.s_s[1]], acc0);
            }
        }
    }
    const T acc = acc0 + acc1;
    __shared__ T partial[kBlock];
    partial[threadIdx.x] = acc;
    __syncthreads();
    for (int half = kBlock / 2; half > 0; half >>= 1) {
        if (static_cast<int>(threadIdx.x) < half)
            partial[threadIdx.x] = partial[threadIdx.x] + partial[threadIdx.x + half];
        __syncthreads();
    }
    if (threadIdx.x == 0)
        out[i * c.o_fs + j * c.o_ss + p0 * c.o_s[0] + p1 * c.o_s[1] + p2 * c.o_s[2]] = partial[0];
}

template <typename T, int TI>
void launch_positions(const agmi_correlation *a, CorrParams &c, hipStream_t s) {
    c.tiles = static_cast<uint32_t>(ceil_div(c.J * c.p_total, kBlock));
    const int64_t blocks = static_cast<int64_t>(c.tiles) * ceil_div(c.I, TI);
    hipLaunchKernelGGL((correlate_positions<T, TI>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, s,
                       static_cast<const T *>(a->filter.data), static_cast<const T *>(a->signal.data),
                       static_cast<T *>(a->out), c);
}

template <typename T>
void launch(const agmi_correlation *a, CorrParams &c, int tile, hipStream_t s) {
    switch (tile) {
        case 0:
            hipLaunchKernelGGL((correlate_reduce<T>), dim3(static_cast<unsigned>(c.I * c.J * c.p_total)), dim3(kBlock),
                               0, s, static_cast<const T *>(a->filter.data), static_cast<const T *>(a->signal.data),
                               static_cast<T *>(a->out), c);
            break;
        case 1: launch_positions<T, 1>(a, c, s); break;
        case 2: launch_positions<T, 2>(a, c, s); break;
        case 4: launch_positions<T, 4>(a, c, s); break;
        default: launch_positions<T, 8>(a, c, s); break;
    }
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
    for (int d = 0; d < 3; ++d)
        if (c.N[d] == 0) c.D = 0;  // an empty signal: every tap is padding, the result is all zeros
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

    // Widest filter-batch tile that still leaves four waves per SIMD of position threads; when even
    // single entries do not give 64 blocks and the reduction is long enough to share, one block per output.
    const int64_t pairs = c.J * p_total;
    if (pairs > 0x7fffffffLL) {
        set_error("correlate: too many output positions for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    int tile = 1;
    for (int cand : {2, 4, 8})
        if (c.I > cand / 2 && ceil_div(c.I, cand) * pairs >= 65536) tile = cand;
    if (tile == 1 && c.I * pairs < 16384 && r_total >= 64) tile = 0;
    if (tile == 0) {
        // lanes along the innermost window axis: the power of two that covers it, at most the block
        c.lane_bits = 0;
        while (c.lane_bits < 8 && (int64_t(1) << c.lane_bits) < c.K[2]) ++c.lane_bits;
    }
    const int64_t blocks = tile == 0 ? outputs : ceil_div(pairs, kBlock) * ceil_div(c.I, tile);
    if (blocks > 0x7fffffffLL) {
        set_error("correlate: too many outputs for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    if (tile == 0)
        set_kernel_name("correlate_reduce<%s>", dtype == AGMI_F32 ? "float" : "double");
    else
        set_kernel_name("correlate_positions<%s, %d>", dtype == AGMI_F32 ? "float" : "double", tile);
    if (dtype == AGMI_F32)
        launch<float>(a, c, tile, s);
    else
        launch<double>(a, c, tile, s);
    return hip_check(hipGetLastError(), "correlate launch");
}
