// Map-reduce kernels: out[kept] = REDUCE_{reduced axes} op(in[0][idx], in[1][idx], ...).
//
// One kernel family serves unbroadcast (sum of a rule's cotangent over broadcast axes, fused
// with the rule itself), numpy.sum/max/min/prod, scipy's logsumexp (as a reduction over
// (max, scaled-sum) pairs, single pass over memory), inner products and matrix-vector dot.
//
// After axis merging the index space is (O, R, I): outer kept, reduced, inner kept.
//   I == 1  "row" form : red_row_block (one 256-thread block per row chunk, 16-byte loads
//                        along R) or red_row_group (G <= 64 lanes per row for short rows);
//   I  > 1  "col" form : red_cols, threads along I (coalesced, 16-byte loads when possible),
//                        a TX x TY block walks R, LDS tree over TY.
// When one pass cannot fill 256 CUs, R is cut into chunks whose partial accumulators go to a
// caller-provided workspace and red_finish combines them.  Combination order is a fixed
// function of the shapes: wave-level butterflies (__shfl_xor over 64 lanes), then an LDS
// tree over the block's 4 waves, then chunks in index order - never atomics - so results
// are reproducible run to run.
#include <algorithm>
#include <mutex>
#include <type_traits>

#include "common.h"
#include "functors.h"

namespace agmi {

// (the accumulators AccSum ... AccLse live in functors.h: the program kernels reduce rows with them too)

struct RedParams {
    void *out;  // T* when final, Acc* (chunk-major) when partial
    const void *in[kMaxPhysIn];     // the op's inputs, then n_aux auxiliary operands of pending maps
    double scalar[AGMI_MAX_INPUTS];
    double scale[AGMI_MAX_INPUTS];  // pending affine map of an input: value = mem * scale + shift
    double shift[AGMI_MAX_INPUTS];
    unsigned scalar_mask;
    unsigned scale_mask, shift_mask;
    signed char scale_aux[AGMI_MAX_INPUTS], shift_aux[AGMI_MAX_INPUTS];  // index of the auxiliary input, or -1
    int n_aux;
    int n_chunks;
    int64_t O, R, I;
    int64_t r_chunk;
    int64_t ostr_o, ostr_i;
    int64_t istr[kMaxPhysIn][3];  // (o, r, i)
};

template <typename T>
struct RVec {
    static constexpr int N = 16 / sizeof(T);
    typedef T type __attribute__((ext_vector_type(N), aligned(sizeof(T))));
};

// load V consecutive points along axis `ax` (1 = r, 2 = i) starting at element offsets given
template <template <typename> class F, typename T, int V, int AX>
__device__ __forceinline__ void load_points(const RedParams &p, int64_t o, int64_t r, int64_t i,
                                            T (&x)[F<T>::NIN + AGMI_MAX_AUX][V]) {
    using vec_t = typename RVec<T>::type;
#pragma unroll
    for (int k = 0; k < F<T>::NIN + AGMI_MAX_AUX; ++k) {
        if (k >= F<T>::NIN + p.n_aux) {  // wave-uniform: no auxiliary operand in this slot
        } else if (k < F<T>::NIN && (p.scalar_mask & (1u << k))) {
            const T s = static_cast<T>(p.scalar[k]);
#pragma unroll
            for (int j = 0; j < V; ++j) x[k][j] = s;
        } else {
            const T *base = static_cast<const T *>(p.in[k]) + o * p.istr[k][0] + r * p.istr[k][1] + i * p.istr[k][2];
            if (V == 1) {
                x[k][0] = *base;
            } else if (p.istr[k][AX] == 0) {
                const T s = *base;
#pragma unroll
                for (int j = 0; j < V; ++j) x[k][j] = s;
            } else {  // stride 1 along AX, guaranteed by the planner when V > 1
                const vec_t *src = reinterpret_cast<const vec_t *>(base);
                const vec_t v = *src;
#pragma unroll
                for (int j = 0; j < V; ++j) x[k][j] = v[j];
            }
        }
    }
    // pending affine maps: multiply, then add, each rounded on its own (wave-uniform tests, once per input)
    if ((p.scale_mask | p.shift_mask) == 0 && p.n_aux == 0) return;
    constexpr int NIN = F<T>::NIN;
#pragma unroll
    for (int k = 0; k < NIN; ++k) {
        if (p.scale_mask & (1u << k)) {
            const T s = static_cast<T>(p.scale[k]);
#pragma unroll
            for (int j = 0; j < V; ++j) x[k][j] = x[k][j] * s;
        }
        if (p.scale_aux[k] >= 0) {
#pragma unroll
            for (int a = 0; a < AGMI_MAX_AUX; ++a)
                if (p.scale_aux[k] == NIN + a) {
#pragma unroll
                    for (int j = 0; j < V; ++j) x[k][j] = x[k][j] * x[NIN + a][j];
                }
        }
        if (p.shift_mask & (1u << k)) {
            const T s = static_cast<T>(p.shift[k]);
#pragma unroll
            for (int j = 0; j < V; ++j) x[k][j] = x[k][j] + s;
        }
        if (p.shift_aux[k] >= 0) {
#pragma unroll
            for (int a = 0; a < AGMI_MAX_AUX; ++a)
                if (p.shift_aux[k] == NIN + a) {
#pragma unroll
                    for (int j = 0; j < V; ++j) x[k][j] = x[k][j] + x[NIN + a][j];
                }
        }
    }
}

// one point of the mapped operand (pending maps have been applied by load_points)
template <template <typename> class F, typename T, int V>
__device__ __forceinline__ T map_point(const RedParams &p, const T (&x)[F<T>::NIN + AGMI_MAX_AUX][V], int j) {
    constexpr int NIN = F<T>::NIN;
    T xi[NIN], oi[F<T>::NOUT];
#pragma unroll
    for (int k = 0; k < NIN; ++k) xi[k] = x[k][j];
    F<T>::apply(xi, oi);
    return oi[0];
}

template <class Acc>
__device__ __forceinline__ typename Acc::type wave_reduce(typename Acc::type a, int lanes) {
    for (int m = lanes >> 1; m > 0; m >>= 1) a = Acc::combine(a, Acc::shfl_xor(a, m));
    return a;
}

// all 256 threads call; result valid in thread 0
template <class Acc>
__device__ __forceinline__ typename Acc::type block_reduce(typename Acc::type a) {
    __shared__ typename Acc::type wave_part[kBlock / 64];
    a = wave_reduce<Acc>(a, 64);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) wave_part[wave] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kBlock / 64; ++w) a = Acc::combine(a, wave_part[w]);
    }
    return a;
}

template <class Acc, typename T, bool FINAL>
__device__ __forceinline__ void store_result(const RedParams &p, typename Acc::type a, int64_t o, int64_t i, int chunk) {
    if (FINAL)
        static_cast<T *>(p.out)[o * p.ostr_o + i * p.ostr_i] = Acc::finish(a);
    else
        static_cast<typename Acc::type *>(p.out)[(static_cast<int64_t>(chunk) * p.O + o) * p.I + i] = a;
}

// ---- row form, one block per (row, chunk) ----------------------------------------------------
template <template <typename> class F, template <typename> class AccT, typename T, int V, bool FINAL>
__global__ __launch_bounds__(kBlock) void red_row_block(const RedParams p) {
    using Acc = AccT<T>;
    const int64_t o = blockIdx.x;
    const int chunk = blockIdx.y;
    const int64_t r_begin = static_cast<int64_t>(chunk) * p.r_chunk;
    const int64_t r_end = min(r_begin + p.r_chunk, p.R);
    typename Acc::type acc = Acc::identity();
    const int64_t n_vec = (r_end - r_begin) / V;
    for (int64_t v = threadIdx.x; v < n_vec; v += kBlock) {
        T x[F<T>::NIN + AGMI_MAX_AUX][V];
        load_points<F, T, V, 1>(p, o, r_begin + v * V, 0, x);
#pragma unroll
        for (int j = 0; j < V; ++j) acc = Acc::combine(acc, Acc::lift(map_point<F, T, V>(p, x, j)));
    }
    if (V > 1) {  // ragged tail, fewer than V points
        const int64_t r = r_begin + n_vec * V + threadIdx.x;
        if (r < r_end) {
            T x[F<T>::NIN + AGMI_MAX_AUX][1];
            load_points<F, T, 1, 1>(p, o, r, 0, x);
            acc = Acc::combine(acc, Acc::lift(map_point<F, T, 1>(p, x, 0)));
        }
    }
    acc = block_reduce<Acc>(acc);
    if (threadIdx.x == 0) store_result<Acc, T, FINAL>(p, acc, o, 0, chunk);
}

// exp(d) for d <= 0 (or NaN) as a term of a sum that contains exp(0) = 1.  float: one v_exp_f32 on
// d * log2(e); the rounding of that product perturbs the term by at most |d| e^d 2^-24 <= 0.37 * 2^-24
// of the sum, below the rounding of the sum itself, and results under the normal range flush to
// zero (they are below 1e-38 of the sum).  double: the library routine.
__device__ __forceinline__ float max_skipping_nan(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double max_skipping_nan(double a, double b) { return __builtin_fmax(a, b); }
__device__ __forceinline__ float exp_nonpositive(float d) { return __builtin_amdgcn_exp2f(d * 1.44269504088896340736f); }
__device__ __forceinline__ double exp_nonpositive(double d) { return exp(d); }

// ---- logsumexp of a row chunk held in registers ------------------------------------------------
// The generic pair accumulator costs one exp per element on a serial dependency chain.  When a
// row chunk fits in registers (<= 256 * V * ITERS elements) each thread instead takes the plain
// maximum of its elements and then sums exp(x - max) with independent exps, and only the
// per-thread (max, sum) pairs go through the pair reduction: one pass over memory.
// V elements of physical input k of row o, starting at reduced index r0 (n_left of them in range);
// out-of-range lanes get `fill`
template <typename T, int V>
__device__ __forceinline__ void lse_load(const RedParams &p, int k, int64_t o, int64_t r0, int64_t n_left, T fill,
                                         T (&dst)[V]) {
    using vec_t = typename RVec<T>::type;
    const int64_t sr = p.istr[k][1];
    const T *base = static_cast<const T *>(p.in[k]) + o * p.istr[k][0] + r0 * sr;
    if (sr == 0) {
        const T v = n_left > 0 ? *base : fill;
#pragma unroll
        for (int j = 0; j < V; ++j) dst[j] = j < n_left ? v : fill;
    } else if (V > 1 && sr == 1 && n_left >= V) {
        const vec_t *src = reinterpret_cast<const vec_t *>(base);
        const vec_t v = *src;
#pragma unroll
        for (int j = 0; j < V; ++j) dst[j] = v[j];
    } else {
#pragma unroll
        for (int j = 0; j < V; ++j) dst[j] = j < n_left ? base[j * sr] : fill;
    }
}

// MODE: 0 = plain input; otherwise the input carries a pending map applied on load:
//   kLseAffine        scalar steps and auxiliary operands that are constant along the row (one value per block)
//   | kLseVecScale    the auxiliary factor varies along the row (registers for it)
//   | kLseVecShift    the auxiliary offset varies along the row
// Separate instantiations keep the register count (and so the blocks per CU) of the plain form.
constexpr int kLseAffine = 1, kLseVecScale = 2, kLseVecShift = 4;

template <typename T, int V, int ITERS, bool FINAL, int MODE>
__global__ __launch_bounds__(kBlock) void lse_row_block(const RedParams p) {
    using Acc = AccLse<T>;
    const int64_t o = blockIdx.x;
    const int chunk = blockIdx.y;
    const int64_t r_begin = static_cast<int64_t>(chunk) * p.r_chunk;
    const int64_t r_end = min(r_begin + p.r_chunk, p.R);
    const int64_t n = r_end - r_begin;
    constexpr bool VEC_A = (MODE & kLseVecScale) != 0, VEC_B = (MODE & kLseVecShift) != 0;
    T x[ITERS][V];
    T a[VEC_A ? ITERS : 1][V], b[VEC_B ? ITERS : 1][V];
    // The chunk fills every lane and every operand that varies along the row has unit stride: the same
    // for the whole block, so the loads below carry no per-lane conditions and all of them are in flight
    // together (with per-lane conditions the compiler waits for each load where its branches join).
    const bool dense = V > 1 && n == static_cast<int64_t>(ITERS) * kBlock * V && p.istr[0][1] == 1 &&
                       (!VEC_A || p.istr[p.scale_aux[0]][1] == 1) && (!VEC_B || p.istr[p.shift_aux[0]][1] == 1);
    if (V > 1 && dense) {
        typedef T vec_t __attribute__((ext_vector_type(V > 1 ? V : 2), aligned(sizeof(T))));
        const auto address = [&](int k, int it) __attribute__((always_inline)) {
            return reinterpret_cast<const vec_t *>(static_cast<const T *>(p.in[k]) + o * p.istr[k][0] + r_begin +
                                                   (it * kBlock + static_cast<int>(threadIdx.x)) * V);
        };
        vec_t xv[ITERS], av[VEC_A ? ITERS : 1], bv[VEC_B ? ITERS : 1];
        // Plain loads, not streaming ones: the rule that differentiates this reduction reads the same operand
        // again a few launches later and finds what these loads left in the last-level cache (with streaming
        // loads here that kernel took 65 us instead of 48 on a 134 MB operand).
#pragma unroll
        for (int it = 0; it < ITERS; ++it) xv[it] = *address(0, it);
        if (VEC_A) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) av[it] = *address(p.scale_aux[0], it);
        }
        if (VEC_B) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) bv[it] = *address(p.shift_aux[0], it);
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < V; ++j) {
                x[it][j] = xv[it][j];
                if (VEC_A) a[it][j] = av[it][j];
                if (VEC_B) b[it][j] = bv[it][j];
            }
    } else {
        // every load is issued before the first use (memory-level parallelism)
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int64_t e0 = (static_cast<int64_t>(it) * kBlock + threadIdx.x) * V;
            lse_load<T, V>(p, 0, o, r_begin + e0, n - e0, T(-INFINITY), x[it]);
        }
        if (VEC_A) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int64_t e0 = (static_cast<int64_t>(it) * kBlock + threadIdx.x) * V;
                lse_load<T, V>(p, p.scale_aux[0], o, r_begin + e0, n - e0, T(1), a[it]);
            }
        }
        if (VEC_B) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int64_t e0 = (static_cast<int64_t>(it) * kBlock + threadIdx.x) * V;
                lse_load<T, V>(p, p.shift_aux[0], o, r_begin + e0, n - e0, T(0), b[it]);
            }
        }
    }
    if (MODE != 0) {
        // steps that are absent are the neutral element (x * 1 is exact; x + 0 only loses the sign
        // of a zero, which neither max nor exp can see), so the arithmetic below is branch-free
        T ua = T(1), ub = T(0);  // auxiliary operands that do not vary along the row
        if (!VEC_A && p.scale_aux[0] >= 0) ua = static_cast<const T *>(p.in[p.scale_aux[0]])[o * p.istr[p.scale_aux[0]][0]];
        if (!VEC_B && p.shift_aux[0] >= 0) ub = static_cast<const T *>(p.in[p.shift_aux[0]])[o * p.istr[p.shift_aux[0]][0]];
        const T sc = (p.scale_mask & 1u) ? static_cast<T>(p.scale[0]) : T(1);
        const T sh = (p.shift_mask & 1u) ? static_cast<T>(p.shift[0]) : T(0);
        if (n == static_cast<int64_t>(ITERS) * kBlock * V && !((p.scale_mask | p.shift_mask) & 1u)) {
            // the same without the absent scalar steps (a block-wide choice; the VALU work of this kernel is
            // not hidden behind its loads, every instruction per element shows in its duration)
#pragma unroll
            for (int it = 0; it < ITERS; ++it)
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const T v = x[it][j] * (VEC_A ? a[it][j] : ua);
                    x[it][j] = v + (VEC_B ? b[it][j] : ub);
                }
        } else if (n == static_cast<int64_t>(ITERS) * kBlock * V) {  // the chunk fills every lane: no padding to protect
#pragma unroll
            for (int it = 0; it < ITERS; ++it)
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    T v = x[it][j] * sc;
                    v = v * (VEC_A ? a[it][j] : ua);
                    v = v + sh;
                    x[it][j] = v + (VEC_B ? b[it][j] : ub);
                }
        } else {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int64_t n_left = n - (static_cast<int64_t>(it) * kBlock + threadIdx.x) * V;
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    T v = x[it][j] * sc;
                    v = v * (VEC_A ? a[it][j] : ua);
                    v = v + sh;
                    v = v + (VEC_B ? b[it][j] : ub);
                    x[it][j] = j < n_left ? v : T(-INFINITY);  // padding stays neutral
                }
            }
        }
    }
    // The maximum that skips NaNs is one instruction per element, the one that keeps them four.  A NaN among
    // finite terms reaches the sum through exp(NaN - m); only where no exp is taken (m infinite) is it looked for.
    T m = T(-INFINITY);
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int j = 0; j < V; ++j) m = max_skipping_nan(x[it][j], m);
    if (m == T(INFINITY) || m == T(-INFINITY)) {
        bool any_nan = false;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < V; ++j) any_nan |= x[it][j] != x[it][j];
        if (any_nan) m = T(NAN);
    }
    T sum = T(0);
    if (m == T(INFINITY)) {
        sum = T(1);
    } else if (m != T(-INFINITY)) {  // also taken for NaN, which then propagates through exp
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < V; ++j) sum += exp_nonpositive(x[it][j] - m);
    }
    const typename Acc::type acc = wave_reduce<Acc>({m, sum}, 64);
    __shared__ typename Acc::type part[kBlock / 64];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        typename Acc::type t = acc;
#pragma unroll
        for (int w = 1; w < kBlock / 64; ++w) t = Acc::combine(t, part[w]);
        store_result<Acc, T, FINAL>(p, t, o, 0, chunk);
    }
}

constexpr int kLseIters = 8;

// ---- row form, G lanes per row (short rows) --------------------------------------------------
template <template <typename> class F, template <typename> class AccT, typename T>
__global__ __launch_bounds__(kBlock) void red_row_group(const RedParams p, const int G) {
    using Acc = AccT<T>;
    const int rows_per_block = kBlock / G;
    const int64_t o = static_cast<int64_t>(blockIdx.x) * rows_per_block + threadIdx.x / G;
    const int lane = threadIdx.x % G;
    typename Acc::type acc = Acc::identity();
    if (o < p.O) {
        for (int64_t r = lane; r < p.R; r += G) {
            T x[F<T>::NIN + AGMI_MAX_AUX][1];
            load_points<F, T, 1, 1>(p, o, r, 0, x);
            acc = Acc::combine(acc, Acc::lift(map_point<F, T, 1>(p, x, 0)));
        }
    }
    acc = wave_reduce<Acc>(acc, G);  // every lane of the wave takes part (rows past O hold identities)
    if (o < p.O && lane == 0) store_result<Acc, T, true>(p, acc, o, 0, 0);
}

// ---- col form ----------------------------------------------------------------------------------
// block = TX x TY threads (TX * TY == 256); a thread owns V consecutive i and walks r with step TY.
template <template <typename> class F, template <typename> class AccT, typename T, int V, bool FINAL>
__global__ __launch_bounds__(kBlock) void red_cols(const RedParams p, const int TX) {
    using Acc = AccT<T>;
    using acc_t = typename Acc::type;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    acc_t *smem = reinterpret_cast<acc_t *>(smem_raw);
    const int TY = kBlock / TX;
    const int tx = threadIdx.x % TX;
    const int ty = threadIdx.x / TX;
    const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * TX + tx) * V;
    const int64_t o = blockIdx.y / p.n_chunks;
    const int chunk = blockIdx.y % p.n_chunks;
    const int64_t r_begin = static_cast<int64_t>(chunk) * p.r_chunk;
    const int64_t r_end = min(r_begin + p.r_chunk, p.R);
    const bool active = i0 < p.I;  // planner guarantees I % V == 0 when V > 1
    acc_t acc[V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = Acc::identity();
    if (active) {
#pragma unroll 16
        for (int64_t r = r_begin + ty; r < r_end; r += TY) {
            T x[F<T>::NIN + AGMI_MAX_AUX][V];
            load_points<F, T, V, 2>(p, o, r, i0, x);
#pragma unroll
            for (int j = 0; j < V; ++j) acc[j] = Acc::combine(acc[j], Acc::lift(map_point<F, T, V>(p, x, j)));
        }
    }
    if (TY > 1) {
#pragma unroll
        for (int j = 0; j < V; ++j) smem[(ty * TX + tx) * V + j] = acc[j];
        __syncthreads();
        for (int half = TY >> 1; half > 0; half >>= 1) {
            if (ty < half) {
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    acc[j] = Acc::combine(acc[j], smem[((ty + half) * TX + tx) * V + j]);
                    smem[(ty * TX + tx) * V + j] = acc[j];
                }
            }
            __syncthreads();
        }
    }
    if (active && ty == 0) {
#pragma unroll
        for (int j = 0; j < V; ++j) store_result<Acc, T, FINAL>(p, acc[j], o, i0 + j, chunk);
    }
}

// Column sums of one plain operand with unit stride along i, whole extent of r in one block (the single-launch plan of
// small operands).  The general kernel above decides per operand how to load (scalar, broadcast, pending map) inside
// its row loop, and a load behind a condition is waited for where the branches join: a thread's rows went out one
// round trip at a time (10 us for 1024 rows).  Here the loads carry no conditions and eight rows are in flight.
// Same order of additions as the general kernel's single-chunk form.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void col_sums_plain(const T *__restrict__ x, int64_t R, int64_t I, int64_t x_o, int64_t x_r,
                                                         T *__restrict__ out, int64_t out_o, int64_t out_i, const int TX) {
    typedef T vec_t __attribute__((ext_vector_type(V > 1 ? V : 2), aligned(sizeof(T))));
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *smem = reinterpret_cast<T *>(smem_raw);
    const int TY = kBlock / TX;
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * TX + tx) * V;
    const int64_t o = blockIdx.y;
    const bool active = i0 < I;  // (I % V == 0 when V > 1)
    const T *col = x + o * x_o + (active ? i0 : 0);
    T acc[V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = T(0);
    int64_t r = ty;
    for (; r + 7 * static_cast<int64_t>(TY) < R; r += 8 * static_cast<int64_t>(TY)) {
        T v[8][V];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const T *src = col + (r + u * static_cast<int64_t>(TY)) * x_r;
            if (V > 1) {
                const vec_t t = *reinterpret_cast<const vec_t *>(src);
#pragma unroll
                for (int j = 0; j < V; ++j) v[u][j] = t[j];
            } else {
                v[u][0] = *src;
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int j = 0; j < V; ++j) acc[j] = acc[j] + v[u][j];
    }
    for (; r < R; r += TY) {
#pragma unroll
        for (int j = 0; j < V; ++j) acc[j] = acc[j] + col[r * x_r + j];
    }
    if (TY > 1) {
#pragma unroll
        for (int j = 0; j < V; ++j) smem[(ty * TX + tx) * V + j] = acc[j];
        __syncthreads();
        for (int half = TY >> 1; half > 0; half >>= 1) {
            if (ty < half) {
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    acc[j] = acc[j] + smem[((ty + half) * TX + tx) * V + j];
                    smem[(ty * TX + tx) * V + j] = acc[j];
                }
            }
            __syncthreads();
        }
    }
    if (active && ty == 0) {
#pragma unroll
        for (int j = 0; j < V; ++j) out[o * out_o + (i0 + j) * out_i] = acc[j];
    }
}

// ---- short form ------------------------------------------------------------------------------
// Few reduced elements per output and many outputs (a 2x2 pooling window, a short middle axis): a
// thread owns V consecutive i of one o and walks the R reduced elements itself, so no lane idles.
template <template <typename> class F, template <typename> class AccT, typename T, int V>
__global__ __launch_bounds__(kBlock) void red_short(const RedParams p, const int64_t i_vecs) {
    using Acc = AccT<T>;
    using acc_t = typename Acc::type;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= p.O * i_vecs) return;
    const int64_t o = e / i_vecs, i0 = (e - o * i_vecs) * V;
    acc_t acc[V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = Acc::identity();
#pragma unroll 2
    for (int64_t r = 0; r < p.R; ++r) {
        T x[F<T>::NIN + AGMI_MAX_AUX][V];
        load_points<F, T, V, 2>(p, o, r, i0, x);
#pragma unroll
        for (int j = 0; j < V; ++j) acc[j] = Acc::combine(acc[j], Acc::lift(map_point<F, T, V>(p, x, j)));
    }
#pragma unroll
    for (int j = 0; j < V; ++j) store_result<Acc, T, true>(p, acc[j], o, i0 + j, 0);
}

// ---- second stage: combine chunk partials ---------------------------------------------------------
// block = FX x FY threads (FX * FY = 256): FX consecutive outputs (coalesced reads of one chunk's
// partials), FY strided walkers over the chunks, LDS tree over FY.  FX shrinks with the number of
// outputs so that a full reduction (one output) still uses all 256 threads.  The order of
// combination is fixed by (n_chunks, FY).
template <template <typename> class AccT, typename T>
__global__ __launch_bounds__(kBlock) void red_finish(const void *partial, T *out, const int n_chunks, const int64_t O,
                                                     const int64_t I, const int64_t ostr_o, const int64_t ostr_i,
                                                     const int FX) {
    using Acc = AccT<T>;
    using acc_t = typename Acc::type;
    __shared__ acc_t smem[kBlock];
    const acc_t *part = static_cast<const acc_t *>(partial);
    const int FY = kBlock / FX;
    const int tx = threadIdx.x % FX, ty = threadIdx.x / FX;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * FX + tx;
    const int64_t n_out = O * I;
    acc_t acc = Acc::identity();
    if (e < n_out) {
#pragma unroll 4
        for (int c = ty; c < n_chunks; c += FY) acc = Acc::combine(acc, part[static_cast<int64_t>(c) * n_out + e]);
    }
    smem[ty * FX + tx] = acc;
    __syncthreads();
    for (int half = FY >> 1; half > 0; half >>= 1) {
        if (ty < half) {
            acc = Acc::combine(acc, smem[(ty + half) * FX + tx]);
            smem[ty * FX + tx] = acc;
        }
        __syncthreads();
    }
    if (ty == 0 && e < n_out) out[(e / I) * ostr_o + (e % I) * ostr_i] = Acc::finish(acc);
}

// ---- planning ------------------------------------------------------------------------------------
constexpr int64_t kShortReduce = 16;  // reduced extents up to this are walked by one thread (column form)

struct RedPlan {
    bool row_form;
    bool block_per_row;
    bool short_form;
    int G;         // row_group lanes per row, or finish lanes per output
    int V;         // vector width in elements (1 or 16 / sizeof(T))
    int TX;        // col form
    int n_chunks;
    int64_t r_chunk;
};

static int pow2_ceil(int64_t v) {
    int p = 1;
    while (p < v && p < (1 << 30)) p <<= 1;
    return p;
}

// enough blocks to give each of the 256 CUs several
constexpr int64_t kTargetBlocks = 2048;

static RedPlan plan_reduce(int64_t O, int64_t R, int64_t I, int vec, bool vec_ok, size_t acc_size, size_t elem_size,
                           size_t workspace_bytes) {
    RedPlan pl = {};
    pl.n_chunks = 1;
    pl.r_chunk = R;
    pl.V = 1;
    const int64_t max_chunks_ws = static_cast<int64_t>(workspace_bytes / (acc_size * (size_t)(O * I)));
    if (I == 1) {
        pl.row_form = true;
        if (R > 1024 || (R > 64 && O < 64)) {
            pl.block_per_row = true;
            pl.V = vec_ok ? vec : 1;
            const int64_t per_block_min = static_cast<int64_t>(kBlock) * pl.V * 16;  // >= 16 vectors per thread
            int64_t chunks = std::min<int64_t>(ceil_div(kTargetBlocks, O), ceil_div(R, per_block_min));
            chunks = std::min<int64_t>(chunks, std::min<int64_t>(max_chunks_ws, 65535));
            if (chunks > 1) {
                int64_t rc = ceil_div(R, chunks);
                rc = ceil_div(rc, pl.V) * pl.V;  // chunk starts stay vector-aligned within the row
                pl.r_chunk = rc;
                pl.n_chunks = static_cast<int>(ceil_div(R, rc));
            }
        } else {
            pl.G = std::min(64, pow2_ceil(ceil_div(R, 4)));
        }
    } else {
        pl.row_form = false;
        pl.V = (vec_ok && I % vec == 0) ? vec : 1;
        if (R <= kShortReduce) {
            pl.short_form = true;
            return pl;
        }
        // a thread-row covers ~256 contiguous bytes of one row of the operands; the rest of the
        // block's threads walk different rows, so many blocks fit across I and few chunks are needed
        const int tx_full = std::max<int>(1, 256 / (pl.V * static_cast<int>(elem_size)));
        pl.TX = std::min<int>(tx_full, pow2_ceil(ceil_div(I, pl.V)));
        // A small operand (the column sums of a 1024 x 1024 cotangent: a bias gradient) is one launch: cutting R into
        // chunks would fill the machine, but the second kernel that adds the chunks costs more than the first one saves.
        // Narrower thread rows (down to 64 bytes) put more blocks across I instead.
        if (R <= 4096 && static_cast<size_t>(O * R * I) * elem_size <= (size_t(8) << 20)) {
            while (pl.TX > 4 && ceil_div(ceil_div(I, pl.V), pl.TX) * O < 64) pl.TX >>= 1;
            return pl;
        }
        const int TY = kBlock / pl.TX;
        const int64_t blocks_x = ceil_div(ceil_div(I, pl.V), pl.TX);
        int64_t chunks = std::min<int64_t>(ceil_div(kTargetBlocks, blocks_x * O), ceil_div(R, static_cast<int64_t>(TY) * 8));
        chunks = std::min<int64_t>(chunks, max_chunks_ws);
        if (O * chunks > 65535) chunks = std::max<int64_t>(1, 65535 / O);
        if (chunks > 1) {
            pl.r_chunk = ceil_div(R, chunks);
            pl.n_chunks = static_cast<int>(ceil_div(R, pl.r_chunk));
        }
    }
    return pl;
}

// `strict`: the workspace has a fixed size that must not change the plan (the summation tree would
// differ from the one a roomy workspace gives); a problem whose partials do not fit is rejected.
template <template <typename> class F, template <typename> class AccT, typename T>
static int launch_reduce(const char *fname, const RedParams &base, bool vec_ok, void *workspace,
                         size_t workspace_bytes, bool strict, hipStream_t s) {
    using Acc = AccT<T>;
    using acc_t = typename Acc::type;
    constexpr int VEC = RVec<T>::N;
    const RedPlan pl = plan_reduce(base.O, base.R, base.I, VEC, vec_ok, sizeof(acc_t), sizeof(T),
                                   strict ? SIZE_MAX : (workspace ? workspace_bytes : 0));
    if (strict && pl.n_chunks > 1) {
        const size_t need = sizeof(acc_t) * static_cast<size_t>(pl.n_chunks) * static_cast<size_t>(base.O * base.I);
        if (need > workspace_bytes) {
            set_error("map_reduce: this reduction stages %zu bytes of partial results; the built-in scratch holds %zu",
                      need, workspace_bytes);
            return AGMI_ERR_WORKSPACE;
        }
    }
    RedParams p = base;
    p.n_chunks = pl.n_chunks;
    p.r_chunk = pl.r_chunk;
    const bool two_stage = pl.n_chunks > 1;
    void *final_out = p.out;
    if (two_stage) p.out = workspace;

    if (pl.row_form && !pl.block_per_row) {
        const int rows_per_block = kBlock / pl.G;
        const int64_t blocks = ceil_div(p.O, rows_per_block);
        if (blocks > 0x7fffffffLL) {
            set_error("map_reduce: too many rows");
            return AGMI_ERR_UNSUPPORTED;
        }
        set_kernel_name("red_row_group<%s>[%lldx%lld]", fname, (long long)p.O, (long long)p.R);
        hipLaunchKernelGGL((red_row_group<F, AccT, T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p, pl.G);
    } else if (pl.row_form) {
        if (p.O > 0x7fffffffLL) {
            set_error("map_reduce: too many rows");
            return AGMI_ERR_UNSUPPORTED;
        }
        const dim3 grid((unsigned)p.O, (unsigned)pl.n_chunks);
        if constexpr (std::is_same<AccT<T>, AccLse<T>>::value && std::is_same<F<T>, FCopy<T>>::value) {
            const bool unit = p.istr[0][1] == 1 || p.r_chunk == 1;
            const int v = (pl.V > 1 && unit) ? VEC : 1;
            if (!(p.scalar_mask & 1u) && p.r_chunk <= static_cast<int64_t>(kBlock) * v * kLseIters) {
                set_kernel_name("lse_row_block%s[%lldx%lld]", two_stage ? "+red_finish" : "", (long long)p.O, (long long)p.R);
                const int64_t need = ceil_div(p.r_chunk, static_cast<int64_t>(kBlock) * v);
                // form of the pending map: auxiliary operands that vary along the reduced axis need registers
                int mode = 0;
                if (((p.scale_mask | p.shift_mask) & 1u) || p.n_aux > 0) mode = kLseAffine;
                if (p.scale_aux[0] >= 0 && p.istr[p.scale_aux[0]][1] != 0) mode |= kLseVecScale;
                if (p.shift_aux[0] >= 0 && p.istr[p.shift_aux[0]][1] != 0) mode |= kLseVecShift;
#define AGMI_LSE_ONE(VV, IT, FIN, MD) \
    hipLaunchKernelGGL((lse_row_block<T, VV, IT, FIN, MD>), grid, dim3(kBlock), 0, s, p)
#define AGMI_LSE_MODE(VV, IT, FIN)                                                                        \
    do {                                                                                                  \
        switch (mode) {                                                                                   \
            case 0: AGMI_LSE_ONE(VV, IT, FIN, 0); break;                                                  \
            case kLseAffine: AGMI_LSE_ONE(VV, IT, FIN, kLseAffine); break;                                \
            case kLseAffine | kLseVecScale: AGMI_LSE_ONE(VV, IT, FIN, kLseAffine | kLseVecScale); break;  \
            case kLseAffine | kLseVecShift: AGMI_LSE_ONE(VV, IT, FIN, kLseAffine | kLseVecShift); break;  \
            default: AGMI_LSE_ONE(VV, IT, FIN, kLseAffine | kLseVecScale | kLseVecShift);                 \
        }                                                                                                 \
    } while (0)
#define AGMI_LSE(VV, IT)                     \
    do {                                     \
        if (two_stage)                       \
            AGMI_LSE_MODE(VV, IT, false);    \
        else                                 \
            AGMI_LSE_MODE(VV, IT, true);     \
    } while (0)
#define AGMI_LSE_IT(VV)                      \
    do {                                     \
        if (need <= 1) AGMI_LSE(VV, 1);      \
        else if (need <= 2) AGMI_LSE(VV, 2); \
        else if (need <= 4) AGMI_LSE(VV, 4); \
        else AGMI_LSE(VV, kLseIters);        \
    } while (0)
                if (v > 1)
                    AGMI_LSE_IT(VEC);
                else
                    AGMI_LSE_IT(1);
#undef AGMI_LSE_IT
#undef AGMI_LSE
#undef AGMI_LSE_MODE
#undef AGMI_LSE_ONE
                goto launched;
            }
        }
        set_kernel_name("red_row_block<%s>%s[%lldx%lld]", fname, two_stage ? "+red_finish" : "", (long long)p.O, (long long)p.R);
#define AGMI_ROW(VV)                                                                                          \
    do {                                                                                                      \
        if (two_stage)                                                                                        \
            hipLaunchKernelGGL((red_row_block<F, AccT, T, VV, false>), grid, dim3(kBlock), 0, s, p);          \
        else                                                                                                  \
            hipLaunchKernelGGL((red_row_block<F, AccT, T, VV, true>), grid, dim3(kBlock), 0, s, p);           \
    } while (0)
        if (pl.V > 1)
            AGMI_ROW(VEC);
        else
            AGMI_ROW(1);
#undef AGMI_ROW
    } else if (pl.short_form) {
        const int64_t i_vecs = p.I / pl.V;
        const int64_t blocks = ceil_div(p.O * i_vecs, kBlock);
        if (blocks > 0x7fffffffLL) {
            set_error("map_reduce: too many outputs");
            return AGMI_ERR_UNSUPPORTED;
        }
        set_kernel_name("red_short<%s>[%lldx%lldx%lld]", fname, (long long)p.O, (long long)p.R, (long long)p.I);
        if (pl.V > 1)
            hipLaunchKernelGGL((red_short<F, AccT, T, VEC>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p, i_vecs);
        else
            hipLaunchKernelGGL((red_short<F, AccT, T, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p, i_vecs);
    } else {
        const int64_t blocks_x = ceil_div(ceil_div(p.I, pl.V), pl.TX);
        if (blocks_x > 0x7fffffffLL || p.O * pl.n_chunks > 65535) {
            set_error("map_reduce: grid too large (outer extent %lld)", (long long)p.O);
            return AGMI_ERR_UNSUPPORTED;
        }
        const dim3 grid((unsigned)blocks_x, (unsigned)(p.O * pl.n_chunks));
        const size_t smem = (kBlock / pl.TX > 1) ? sizeof(acc_t) * kBlock * pl.V : 0;
        if constexpr (std::is_same<AccT<T>, AccSum<T>>::value && std::is_same<F<T>, FCopy<T>>::value) {
            // one plain operand, unit stride along i, one chunk: the kernel whose loads carry no conditions
            if (!two_stage && !(p.scalar_mask & 1u) && !((p.scale_mask | p.shift_mask) & 1u) && p.n_aux == 0 && p.istr[0][2] == 1 &&
                p.scale_aux[0] < 0 && p.shift_aux[0] < 0) {
                set_kernel_name("col_sums_plain[%lldx%lldx%lld]", (long long)p.O, (long long)p.R, (long long)p.I);
                const T *x = static_cast<const T *>(p.in[0]);
                T *out = static_cast<T *>(p.out);
                if (pl.V > 1)
                    hipLaunchKernelGGL((col_sums_plain<T, VEC>), grid, dim3(kBlock), smem, s, x, p.R, p.I, p.istr[0][0], p.istr[0][1], out,
                                       p.ostr_o, p.ostr_i, pl.TX);
                else
                    hipLaunchKernelGGL((col_sums_plain<T, 1>), grid, dim3(kBlock), smem, s, x, p.R, p.I, p.istr[0][0], p.istr[0][1], out,
                                       p.ostr_o, p.ostr_i, pl.TX);
                goto launched;
            }
        }
        set_kernel_name("red_cols<%s>%s[%lldx%lldx%lld]", fname, two_stage ? "+red_finish" : "", (long long)p.O, (long long)p.R, (long long)p.I);
#define AGMI_COL(VV)                                                                                          \
    do {                                                                                                      \
        if (two_stage)                                                                                        \
            hipLaunchKernelGGL((red_cols<F, AccT, T, VV, false>), grid, dim3(kBlock), smem, s, p, pl.TX);     \
        else                                                                                                  \
            hipLaunchKernelGGL((red_cols<F, AccT, T, VV, true>), grid, dim3(kBlock), smem, s, p, pl.TX);      \
    } while (0)
        if (pl.V > 1)
            AGMI_COL(VEC);
        else
            AGMI_COL(1);
#undef AGMI_COL
    }
launched:
    if (int rc = hip_check(hipGetLastError(), "map_reduce launch")) return rc;
    if (two_stage) {
        const int fx = static_cast<int>(std::min<int64_t>(32, pow2_ceil(p.O * p.I)));
        const int64_t blocks = ceil_div(p.O * p.I, fx);
        hipLaunchKernelGGL((red_finish<AccT, T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, workspace,
                           static_cast<T *>(final_out), pl.n_chunks, p.O, p.I, p.ostr_o, p.ostr_i, fx);
        if (int rc = hip_check(hipGetLastError(), "map_reduce finish launch")) return rc;
    }
    return 0;
}

// Canonical (O, R, I) view of a merged index space, or failure for patterns such as
// reduced-kept-reduced that need two passes.
static bool canonical_ori(const Merged &m, int n_operands, RedParams *p, int64_t (*ostr)[3]) {
    // pattern of groups after merging: sequences K, R, KR, RK, KRK
    int idx_o = -1, idx_r = -1, idx_i = -1;
    if (m.ndim == 1) {
        (m.group[0] ? idx_r : idx_i) = 0;
    } else if (m.ndim == 2) {
        if (!m.group[0] && m.group[1]) {
            idx_o = 0;
            idx_r = 1;
        } else if (m.group[0] && !m.group[1]) {
            idx_r = 0;
            idx_i = 1;
        } else {
            return false;
        }
    } else if (m.ndim == 3 && !m.group[0] && m.group[1] && !m.group[2]) {
        idx_o = 0;
        idx_r = 1;
        idx_i = 2;
    } else {
        return false;
    }
    p->O = idx_o >= 0 ? m.shape[idx_o] : 1;
    p->R = idx_r >= 0 ? m.shape[idx_r] : 1;
    p->I = idx_i >= 0 ? m.shape[idx_i] : 1;
    for (int k = 0; k < n_operands; ++k) {
        ostr[k][0] = idx_o >= 0 ? m.stride[k][idx_o] : 0;
        ostr[k][1] = idx_r >= 0 ? m.stride[k][idx_r] : 0;
        ostr[k][2] = idx_i >= 0 ? m.stride[k][idx_i] : 0;
    }
    return true;
}

struct RedSetup {
    RedParams p;
    bool vec_ok;
    bool ws_strict = false;  // see launch_reduce
};

// `arity` = number of inputs of the op itself; ins[arity .. n_in) are auxiliary operands of pending maps
static int setup_reduce(int ndim, const int64_t *shape, const uint8_t *reduce_axes, const agmi_array *out, int arity,
                        int n_in, const agmi_array *ins, const double *scalars, RedSetup *st, bool *empty) {
    if (!out || !ins || !reduce_axes || n_in < 1 || n_in > kMaxPhysIn || arity < 1 || arity > n_in || n_in - arity > AGMI_MAX_AUX) {
        set_error("map_reduce: bad arguments");
        return AGMI_ERR_ARG;
    }
    int64_t out_strides[AGMI_MAX_DIMS];
    uint8_t group[AGMI_MAX_DIMS];
    if (ndim > AGMI_MAX_DIMS || ndim < 0) {
        set_error("map_reduce: rank %d", ndim);
        return AGMI_ERR_ARG;
    }
    for (int d = 0; d < ndim; ++d) {
        group[d] = reduce_axes[d] ? 1 : 0;
        out_strides[d] = group[d] ? 0 : out->strides[d];
    }
    const int64_t *strides[kMaxOperands];
    strides[0] = out_strides;
    for (int k = 0; k < n_in; ++k) strides[1 + k] = ins[k].data ? ins[k].strides : nullptr;
    Merged m;
    if (!merge_axes(ndim, shape, group, 1 + n_in, strides, &m)) return AGMI_ERR_ARG;
    *empty = false;
    if (m.n == 0) {
        // an empty reduced axis still produces identities; callers handle that case with fill
        *empty = true;
        return 0;
    }
    RedParams &p = st->p;
    p = RedParams{};
    int64_t ori[kMaxOperands][3];
    if (!canonical_ori(m, 1 + n_in, &p, ori)) {
        set_error("map_reduce: reduced axes are not one contiguous group after merging; reduce in two calls");
        return AGMI_ERR_UNSUPPORTED;
    }
    p.out = out->data;
    p.ostr_o = ori[0][0];
    p.ostr_i = ori[0][2];
    st->vec_ok = true;
    const int ax = (p.I == 1) ? 1 : 2;
    p.n_aux = n_in - arity;
    for (int k = 0; k < AGMI_MAX_INPUTS; ++k) p.scale_aux[k] = p.shift_aux[k] = -1;
    for (int k = 0; k < n_in; ++k) {
        p.in[k] = ins[k].data;
        if (!ins[k].data) {
            if (!scalars || k >= arity) {
                set_error("map_reduce: scalar slot %d without scalars array (auxiliary inputs must be arrays)", k);
                return AGMI_ERR_ARG;
            }
            p.scalar_mask |= 1u << k;
            p.scalar[k] = scalars[k];
        } else {
            if (k < arity && !read_affine(ins[k], arity, n_in, k, &p)) return AGMI_ERR_ARG;
            for (int a = 0; a < 3; ++a) p.istr[k][a] = ori[1 + k][a];
            if (p.istr[k][ax] != 0 && p.istr[k][ax] != 1) st->vec_ok = false;
        }
    }
    if (p.out == nullptr) {
        set_error("map_reduce: output is null");
        return AGMI_ERR_ARG;
    }
    return 0;
}

template <typename T>
static size_t acc_size_of(int red) {
    return red == AGMI_RED_LOGSUMEXP ? sizeof(LsePair<T>) : sizeof(T);
}

template <template <typename> class F, typename T>
static int dispatch_red(const char *fname, int red, const RedSetup &st, void *ws, size_t ws_bytes, hipStream_t s) {
    if (F<T>::NOUT != 1) {
        set_error("map_reduce: op has %d outputs", F<T>::NOUT);
        return AGMI_ERR_ARG;
    }
    switch (red) {
        case AGMI_RED_SUM: return launch_reduce<F, AccSum, T>(fname, st.p, st.vec_ok, ws, ws_bytes, st.ws_strict, s);
        default: break;
    }
    set_error("map_reduce: reduction %d is only available with AGMI_OP_COPY", red);
    return AGMI_ERR_UNSUPPORTED;
}

template <typename T>
static int dispatch_red_copy(int red, const RedSetup &st, void *ws, size_t ws_bytes, hipStream_t s) {
    switch (red) {
        case AGMI_RED_SUM: return launch_reduce<FCopy, AccSum, T>("sum", st.p, st.vec_ok, ws, ws_bytes, st.ws_strict, s);
        case AGMI_RED_MAX: return launch_reduce<FCopy, AccMax, T>("max", st.p, st.vec_ok, ws, ws_bytes, st.ws_strict, s);
        case AGMI_RED_MIN: return launch_reduce<FCopy, AccMin, T>("min", st.p, st.vec_ok, ws, ws_bytes, st.ws_strict, s);
        case AGMI_RED_PROD: return launch_reduce<FCopy, AccProd, T>("prod", st.p, st.vec_ok, ws, ws_bytes, st.ws_strict, s);
        case AGMI_RED_LOGSUMEXP: return launch_reduce<FCopy, AccLse, T>("logsumexp", st.p, st.vec_ok, ws, ws_bytes, st.ws_strict, s);
        default: set_error("map_reduce: unknown reduction %d", red); return AGMI_ERR_ARG;
    }
}

}  // namespace agmi

using namespace agmi;

// ops that may feed a sum: the rules whose cotangent is unbroadcast, the logsumexp JVP, products
#define AGMI_FOR_EACH_REDUCE_OP(X) \
    X(AGMI_OP_NEG, FNeg)           \
    X(AGMI_OP_MUL, FMul)           \
    X(AGMI_OP_DIV, FDiv)           \
    X(AGMI_OP_SQUARE, FSquare)     \
    X(AGMI_OP_ABS, FAbs)           \
    X(AGMI_OP_DIV_VJP1, FDivVjp1)  \
    X(AGMI_OP_TANH_VJP, FTanhVjp)  \
    X(AGMI_OP_POW_VJP0, FPowVjp0)  \
    X(AGMI_OP_POW_VJP1, FPowVjp1)  \
    X(AGMI_OP_LSE_VJP, FLseVjp)    \
    X(AGMI_OP_CHOOSE_VJP, FChooseVjp) \
    X(AGMI_OP_EQUAL_AS_FLOAT, FEqualAsFloat)

// This file is compiled twice, once per precision (-DAGMI_PART=32 / 64), so that the two halves of
// the kernel instantiations build in parallel; the entry points live in the float32 half.
#ifndef AGMI_PART
#error "compile with -DAGMI_PART=32 or -DAGMI_PART=64"
#endif
namespace agmi {
int reduce_part_f32(int op, int red, const RedSetup &st, void *ws, size_t ws_bytes, hipStream_t s);
int reduce_part_f64(int op, int red, const RedSetup &st, void *ws, size_t ws_bytes, hipStream_t s);
#if AGMI_PART == 32
#define AGMI_PART_FN reduce_part_f32
using PartT = float;
#else
#define AGMI_PART_FN reduce_part_f64
using PartT = double;
#endif
int AGMI_PART_FN(int op, int red, const RedSetup &st, void *ws, size_t ws_bytes, hipStream_t s) {
    if (op == AGMI_OP_COPY) return dispatch_red_copy<PartT>(red, st, ws, ws_bytes, s);
#define AGMI_CASE(OP, FN) \
    case OP: return dispatch_red<FN, PartT>(#FN, red, st, ws, ws_bytes, s);
    switch (op) {
        AGMI_FOR_EACH_REDUCE_OP(AGMI_CASE)
        default: break;
    }
#undef AGMI_CASE
    set_error("map_reduce: op %d cannot be fused into a reduction", op);
    return AGMI_ERR_UNSUPPORTED;
}
#undef AGMI_PART_FN
}  // namespace agmi

#if AGMI_PART == 32
static int map_reduce_entry(int op, int red, int dtype, int ndim, const int64_t *shape, const uint8_t *reduce_axes,
                            const agmi_array *out, int n_in, const agmi_array *ins, const double *scalars,
                            void *(*workspace_of)(void *), void *workspace, size_t workspace_bytes, bool strict,
                            void *stream) {
    int arity = op == AGMI_OP_COPY ? 1 : -1;
#define AGMI_CASE(OP, FN) \
    if (op == OP) arity = FN<float>::NIN;
    AGMI_FOR_EACH_REDUCE_OP(AGMI_CASE)
#undef AGMI_CASE
    if (arity < 0) {
        set_error("map_reduce: op %d cannot be fused into a reduction", op);
        return AGMI_ERR_UNSUPPORTED;
    }
    RedSetup st;
    bool empty = false;
    if (int rc = setup_reduce(ndim, shape, reduce_axes, out, arity, n_in, ins, scalars, &st, &empty)) return rc;
    if (empty) return 0;
    st.ws_strict = strict;
    hipStream_t s = as_stream(stream);
    if (dtype != AGMI_F32 && dtype != AGMI_F64) {
        set_error("map_reduce: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    if (workspace_of) {  // resolved only once the arguments have been accepted
        workspace = workspace_of(nullptr);
        if (!workspace) return AGMI_ERR_WORKSPACE;
    }
    return dtype == AGMI_F32 ? reduce_part_f32(op, red, st, workspace, workspace_bytes, s)
                             : reduce_part_f64(op, red, st, workspace, workspace_bytes, s);
}

extern "C" int agmi_map_reduce(int op, int red, int dtype, int ndim, const int64_t *shape,
                               const uint8_t *reduce_axes, const agmi_array *out, int n_in,
                               const agmi_array *ins, const double *scalars, void *workspace,
                               size_t workspace_bytes, void *stream) {
    return map_reduce_entry(op, red, dtype, ndim, shape, reduce_axes, out, n_in, ins, scalars, nullptr, workspace,
                            workspace_bytes, false, stream);
}

// Staging memory of agmi_map_reduce_static: part of the library's device image, one copy on every
// GPU the process uses, held until the process ends.  Two-stage reductions write every partial
// result they later read, so nothing in it has to start at zero.
static __device__ __align__(256) unsigned char scratch[AGMI_STATIC_SCRATCH_BYTES];

// Device address of `scratch` on the current GPU.  In host code the array's name is only a handle
// for this lookup, never an address a kernel may be given.
static void *static_scratch(void *) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void *ptr[kMaxDevices] = {};
    int dev = -1;
    if (hip_check(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        set_error("map_reduce_static: device ordinal %d out of range", dev);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr[dev]) {
        void *p = nullptr;
        if (hip_check(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
        if (!p) {
            set_error("map_reduce_static: the scratch symbol has no address on device %d", dev);
            return nullptr;
        }
        ptr[dev] = p;
    }
    return ptr[dev];
}

extern "C" int agmi_map_reduce_static(int op, int red, int dtype, int ndim, const int64_t *shape,
                                      const uint8_t *reduce_axes, const agmi_array *out, int n_in,
                                      const agmi_array *ins, const double *scalars, void *stream) {
    return map_reduce_entry(op, red, dtype, ndim, shape, reduce_axes, out, n_in, ins, scalars, static_scratch, nullptr,
                            AGMI_STATIC_SCRATCH_BYTES, true, stream);
}

extern "C" size_t agmi_map_reduce_workspace_bytes(int red, int dtype, int ndim, const int64_t *shape,
                                                  const uint8_t *reduce_axes) {
    // Upper bound over every layout: partials for kTargetBlocks chunks can never be needed for
    // more than kTargetBlocks * (number of outputs) accumulators, and never more chunks than
    // there are reduced points.
    if (ndim < 0 || ndim > AGMI_MAX_DIMS || !shape || !reduce_axes) return 0;
    int64_t kept = 1, reduced = 1;
    for (int d = 0; d < ndim; ++d) (reduce_axes[d] ? reduced : kept) *= shape[d];
    if (kept <= 0 || reduced <= 1) return 0;
    const size_t acc = dtype == AGMI_F64 ? acc_size_of<double>(red) : acc_size_of<float>(red);
    const int64_t chunks = std::min<int64_t>(kTargetBlocks, reduced);
    return static_cast<size_t>(chunks) * static_cast<size_t>(kept) * acc;
}
#endif  // AGMI_PART == 32
