// Sliding-window contraction behind N-d convolution and its cotangents:
//
//   out[i, j, p] = sum_{d, k} filter[i, d, k] * signal[j, d, p + k - pad]     (zero outside the signal)
//
// The reference forms an as_strided window view of the (explicitly zero-padded) signal and hands
// it to einsum (scipy/signal.py:45-65).  Here neither the padding nor the view exists: the window
// is walked in place and the taps that fall off the signal are skipped.  Flips arrive as negative
// strides.
//
// Two shapes of problem occur, and each has its kernels.
//
// correlate_tiled / correlate_positions: the forward pass and the signal's cotangent have many output positions and
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
    // correlate_tiled: a block covers 2^jt_bits images x 2^p1_bits rows x 2^p2_bits columns of output
    // (256 positions) and stages the H x W window of signal they read, per image, in LDS
    int jt_bits, p1_bits, p2_bits, H, W;
    int DT;                     // contracted indices staged per step
    uint32_t n_tj, n_t1, n_t2;  // tiles along each
    uint32_t s_elems_padded;    // LDS elements reserved for the signal tile (a multiple of 8)
};

constexpr int kTileLoads = 8;    // signal elements a thread stages per step: tiles of up to 2048 elements
constexpr int kFilterLoads = 4;  // filter elements a thread stages per step: DT * K1 * K2 * TI up to 1024

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

// The same contraction with the operands staged in LDS.  A block owns 256 output positions (a tile of
// images x rows x columns) and TI filter-batch entries.  For every contracted index d (and tap k0 of
// a third convolved axis) it copies the window of signal its positions read (zero where the window
// leaves the signal: the padding is made here, once per element, not tested per tap) and the
// K1 x K2 x TI filter taps into LDS (several d per step while they fit), then every thread walks the
// window row by row: the LDS reads of a row (signal and broadcast taps) are issued together, then its
// K2 x TI multiply-adds (rows of width 2, 3, 5, 7 are unrolled; LDS latency, not bandwidth, is what a
// tap-by-tap loop pays for).  Which
// global element each thread stages is fixed for the whole kernel and computed once; the loads
// of step n+1 are issued before the multiply-adds of step n.
template <typename T, int TI, int K2T>
__global__ __launch_bounds__(kBlock) void correlate_tiled(const T *__restrict__ filter, const T *__restrict__ signal,
                                                          T *__restrict__ out, const CorrParams c) {
    extern __shared__ __align__(64) unsigned char lds_raw[];
    T *S = reinterpret_cast<T *>(lds_raw);  // [DT][2^jt_bits][H][W]
    T *F = S + c.s_elems_padded;            // [DT][K1 * K2][TI]
    uint32_t q = blockIdx.x;
    const uint32_t t2 = q % c.n_t2;
    q /= c.n_t2;
    const uint32_t t1 = q % c.n_t1;
    q /= c.n_t1;
    const uint32_t tj = q % c.n_tj;
    q /= c.n_tj;
    const int64_t p0 = q % static_cast<uint32_t>(c.P[0]);
    const int64_t i0 = static_cast<int64_t>(q / static_cast<uint32_t>(c.P[0])) * TI;
    const int tid = threadIdx.x;
    const int x = tid & ((1 << c.p2_bits) - 1);
    const int y = (tid >> c.p2_bits) & ((1 << c.p1_bits) - 1);
    const int jj = tid >> (c.p2_bits + c.p1_bits);
    const int64_t j0 = static_cast<int64_t>(tj) << c.jt_bits;
    const int64_t r0 = static_cast<int64_t>(t1) << c.p1_bits, c0 = static_cast<int64_t>(t2) << c.p2_bits;
    const int HW = c.H * c.W, s_slice = HW << c.jt_bits, s_elems = s_slice * c.DT;
    const int K1 = static_cast<int>(c.K[1]), K2 = K2T > 0 ? K2T : static_cast<int>(c.K[2]);
    const int f_slice = K1 * K2 * TI, f_elems = f_slice * c.DT;

    // what this thread stages: LDS slot tid + n * 256 of either tile.  Slots that fall on padding
    // (or past the last contracted index) read a valid address and store zero.
    int64_t s_off[kTileLoads], f_off[kFilterLoads];
    int s_dd[kTileLoads], f_dd[kFilterLoads];
    unsigned s_ok = 0;
#pragma unroll
    for (int n = 0; n < kTileLoads; ++n) {
        const int e = tid + n * kBlock;
        s_off[n] = 0;
        s_dd[n] = 0;
        if (e < s_elems) {
            const int dd = e / s_slice, e1 = e - dd * s_slice;
            const int ej = e1 / HW, rem = e1 - ej * HW, h = rem / c.W, w = rem - h * c.W;
            const int64_t j = j0 + ej, s1 = r0 + h - c.pad[1], s2 = c0 + w - c.pad[2];
            s_dd[n] = dd;
            if (j < c.J && static_cast<uint64_t>(s1) < static_cast<uint64_t>(c.N[1]) &&
                static_cast<uint64_t>(s2) < static_cast<uint64_t>(c.N[2])) {
                s_ok |= 1u << n;
                s_off[n] = j * c.s_bs + s1 * c.s_s[1] + s2 * c.s_s[2];
            }
        }
    }
#pragma unroll
    for (int m = 0; m < kFilterLoads; ++m) {
        const int e = tid + m * kBlock;
        f_off[m] = 0;
        f_dd[m] = 0;
        if (e < f_elems) {
            const int dd = e / f_slice, e1 = e - dd * f_slice;
            const int kk = e1 / TI, t = e1 - kk * TI, k1 = kk / K2, k2 = kk - k1 * K2;
            const int64_t i = i0 + t < c.I ? i0 + t : c.I - 1;  // rows past the last repeat it (computed, never stored)
            f_dd[m] = dd;
            f_off[m] = i * c.f_bs + k1 * c.f_s[1] + k2 * c.f_s[2];
        }
    }
    // taps of the third convolved axis that meet the signal (the same for the whole block)
    const int64_t b0 = p0 - c.pad[0];
    const int k0_lo = static_cast<int>(b0 < 0 ? -b0 : 0);
    const int k0_hi = static_cast<int>(c.N[0] - b0 < c.K[0] ? c.N[0] - b0 : c.K[0]);
    const int d_groups = k0_hi > k0_lo ? static_cast<int>((c.D + c.DT - 1) / c.DT) : 0;

    // a step = DT contracted indices (group g) at one tap k0 of the third axis.  Every thread issues all
    // its loads unconditionally (slots it does not own read element 0 again), so none waits on another.
    T s_reg[kTileLoads], f_reg[kFilterLoads];
    auto fetch = [&](int g, int k0) {
        const int64_t d0 = static_cast<int64_t>(g) * c.DT;
        const int last = static_cast<int>(c.D - 1 - d0 < c.DT ? c.D - 1 - d0 : c.DT);  // indices past the end repeat the last
        const T *sg = signal + d0 * c.s_ds + (b0 + k0) * c.s_s[0];
        const T *fg = filter + d0 * c.f_ds + k0 * c.f_s[0];
#pragma unroll
        for (int n = 0; n < kTileLoads; ++n) s_reg[n] = sg[(s_dd[n] < last ? s_dd[n] : last) * c.s_ds + s_off[n]];
#pragma unroll
        for (int m = 0; m < kFilterLoads; ++m) f_reg[m] = fg[(f_dd[m] < last ? f_dd[m] : last) * c.f_ds + f_off[m]];
    };
    T acc[TI];
#pragma unroll
    for (int t = 0; t < TI; ++t) acc[t] = T(0);
    const T *Sp = S + jj * HW + y * c.W + x;
    int g = 0, k0 = k0_lo;
    if (d_groups > 0) fetch(g, k0);
    while (g < d_groups) {
        const int64_t left = c.D - static_cast<int64_t>(g) * c.DT;
        const int live = static_cast<int>(left < c.DT ? left : c.DT);  // contracted indices in this step
        __syncthreads();  // everyone has finished reading the previous step's tiles
#pragma unroll
        for (int n = 0; n < kTileLoads; ++n)
            if (tid + n * kBlock < s_elems)
                S[tid + n * kBlock] = ((s_ok >> n & 1u) && s_dd[n] < live) ? s_reg[n] : T(0);
#pragma unroll
        for (int m = 0; m < kFilterLoads; ++m)
            if (tid + m * kBlock < f_elems) F[tid + m * kBlock] = f_reg[m];
        __syncthreads();
        int g_next = g, k0_next = k0 + 1;
        if (k0_next >= k0_hi) {
            k0_next = k0_lo;
            ++g_next;
        }
        if (g_next < d_groups) fetch(g_next, k0_next);  // in flight during the multiply-adds below
        for (int dd = 0; dd < live; ++dd) {
            for (int k1 = 0; k1 < K1; ++k1) {
                const T *row = Sp + dd * s_slice + k1 * c.W;
                const T *taps = F + dd * f_slice + k1 * K2 * TI;
                if constexpr (K2T > 0) {
                    // a window row of known width: its LDS reads are issued together, then the multiply-adds
                    T sv[K2T], fv[K2T][TI];
#pragma unroll
                    for (int k2 = 0; k2 < K2T; ++k2) {
                        sv[k2] = row[k2];
#pragma unroll
                        for (int t = 0; t < TI; ++t) fv[k2][t] = taps[k2 * TI + t];
                    }
#pragma unroll
                    for (int k2 = 0; k2 < K2T; ++k2)
#pragma unroll
                        for (int t = 0; t < TI; ++t) acc[t] = fused_mul_add(fv[k2][t], sv[k2], acc[t]);
                } else {
                    for (int k2 = 0; k2 < K2; ++k2) {
                        const T sv = row[k2];
#pragma unroll
                        for (int t = 0; t < TI; ++t) acc[t] = fused_mul_add(taps[k2 * TI + t], sv, acc[t]);
                    }
                }
            }
        }
        g = g_next;
        k0 = k0_next;
    }
    const int64_t j = j0 + jj, p1 = r0 + y, p2 = c0 + x;
    if (j >= c.J || p1 >= c.P[1] || p2 >= c.P[2]) return;
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

template <typename T, int TI, int K2T>
void launch_tiled_width(const agmi_correlation *a, CorrParams &c, hipStream_t s) {
    const int64_t blocks = ceil_div(c.I, TI) * c.P[0] * c.n_tj * c.n_t1 * c.n_t2;
    const size_t lds = (static_cast<size_t>(c.s_elems_padded) + static_cast<size_t>(c.K[1] * c.K[2]) * TI * c.DT) * sizeof(T);
    hipLaunchKernelGGL((correlate_tiled<T, TI, K2T>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), lds, s,
                       static_cast<const T *>(a->filter.data), static_cast<const T *>(a->signal.data),
                       static_cast<T *>(a->out), c);
}

// the common window widths get a fully unrolled row; any other width runs the generic loop
template <typename T, int TI>
void launch_tiled(const agmi_correlation *a, CorrParams &c, hipStream_t s) {
    switch (c.K[2]) {
        case 2: launch_tiled_width<T, TI, 2>(a, c, s); break;
        case 3: launch_tiled_width<T, TI, 3>(a, c, s); break;
        case 5: launch_tiled_width<T, TI, 5>(a, c, s); break;
        case 7: launch_tiled_width<T, TI, 7>(a, c, s); break;
        default: launch_tiled_width<T, TI, 0>(a, c, s); break;
    }
}

template <typename T>
void launch(const agmi_correlation *a, CorrParams &c, int tile, bool tiled, hipStream_t s) {
    if (tiled) {
        switch (tile) {
            case 1: launch_tiled<T, 1>(a, c, s); break;
            case 2: launch_tiled<T, 2>(a, c, s); break;
            case 4: launch_tiled<T, 4>(a, c, s); break;
            default: launch_tiled<T, 8>(a, c, s); break;
        }
        return;
    }
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
    // The LDS-staged kernel when its tiles fit: 256 positions per block shaped to the output (columns
    // first), the window of signal they read within kTileLoads x 256 elements, the taps within
    // kFilterLoads x 256.
    bool tiled = false;
    if (tile != 0 && c.D > 0) {
        // tile shape: columns first (up to 32: whole LDS rows per wave), then rows, then images.  A shape fitted
        // to the output (12 x 12 as 4 x 4 x 16 images instead of 16 x 16 x 1) wastes fewer threads but was slower
        // when measured: narrow rows mean more steps and LDS bank conflicts.
        auto bits_for = [](int64_t n, int cap) {
            int b = 0;
            while (b < cap && (int64_t(1) << b) < n) ++b;
            return b;
        };
        c.p2_bits = bits_for(c.P[2], 5);
        c.p1_bits = bits_for(c.P[1], 8 - c.p2_bits);
        c.jt_bits = 8 - c.p2_bits - c.p1_bits;
        const int64_t H = (int64_t(1) << c.p1_bits) + c.K[1] - 1, W = (int64_t(1) << c.p2_bits) + c.K[2] - 1;
        const int64_t s_elems = (H * W) << c.jt_bits;
        if (s_elems <= kTileLoads * kBlock && c.K[1] * c.K[2] * tile <= kFilterLoads * kBlock) {
            tiled = true;
            c.H = static_cast<int>(H);
            c.W = static_cast<int>(W);
            // several contracted indices per step while both tiles still fit: fewer barriers and more loads in flight
            c.DT = 1;
            while (c.DT < 8 && c.DT * 2 <= c.D && s_elems * c.DT * 2 <= kTileLoads * kBlock &&
                   c.K[1] * c.K[2] * tile * c.DT * 2 <= kFilterLoads * kBlock)
                c.DT *= 2;
            c.s_elems_padded = static_cast<uint32_t>((s_elems * c.DT + 7) / 8 * 8);
            c.n_tj = static_cast<uint32_t>(ceil_div(c.J, int64_t(1) << c.jt_bits));
            c.n_t1 = static_cast<uint32_t>(ceil_div(c.P[1], int64_t(1) << c.p1_bits));
            c.n_t2 = static_cast<uint32_t>(ceil_div(c.P[2], int64_t(1) << c.p2_bits));
        }
    }
    const int64_t blocks = tile == 0 ? outputs
                           : tiled   ? ceil_div(c.I, tile) * c.P[0] * c.n_tj * c.n_t1 * c.n_t2
                                     : ceil_div(pairs, kBlock) * ceil_div(c.I, tile);
    if (blocks > 0x7fffffffLL) {
        set_error("correlate: too many outputs for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    const char *tname = dtype == AGMI_F32 ? "float" : "double";
    if (tile == 0)
        set_kernel_name("correlate_reduce<%s>", tname);
    else
        set_kernel_name("correlate_%s<%s, %d>", tiled ? "tiled" : "positions", tname, tile);
    if (dtype == AGMI_F32)
        launch<float>(a, c, tile, tiled, s);
    else
        launch<double>(a, c, tile, tiled, s);
    return hip_check(hipGetLastError(), "correlate launch");
}
