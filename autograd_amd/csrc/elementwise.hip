// Elementwise ("map") kernels: out[k][idx] = op(in[0][idx], ...) over a strided index space.
//
// All of these are HBM-bound on MI355X, so the design goal is one pass with full-width,
// coalesced accesses: every thread moves one 16-byte vector per array operand and there is
// no loop (measured on the target: one vector per thread, 256-thread blocks, grid = exactly
// the element count saturates HBM; unrolled variants were slower).  Three layouts:
//   flat  - after axis merging every array operand is contiguous or a single element;
//   rows  - two merged axes whose inner stride is 1 or 0 for every operand
//           (A * b[None, :], x + c[:, None], row slices): vectors along the inner axis,
//           broadcast operands cost one scalar load;
//   nd    - anything else up to 6 merged axes, one element per thread with div/mod indexing.
// A by-value scalar operand lives in kernel arguments (SGPRs); which slots are scalars is a
// run-time, wave-uniform mask, so one kernel serves array/scalar combinations.
#include <type_traits>

#include "common.h"
#include "functors.h"

namespace agmi {

struct EwParams {
    void *out[AGMI_MAX_OUTPUTS];
    const void *in[kMaxPhysIn];
    double scalar[AGMI_MAX_INPUTS];
    double scale[AGMI_MAX_INPUTS];  // pending affine map of an input: value = mem * scale + shift
    double shift[AGMI_MAX_INPUTS];
    unsigned scalar_mask;
    unsigned scale_mask, shift_mask;
    // pending maps whose factor / offset is an array: index (>= the op's arity) of the auxiliary
    // input that holds it, or -1
    signed char scale_aux[AGMI_MAX_INPUTS], shift_aux[AGMI_MAX_INPUTS];
    int ndim;
    int64_t n;
    int64_t shape[kMaxMerged];
    int64_t ostr[AGMI_MAX_OUTPUTS][kMaxMerged];
    int64_t istr[kMaxPhysIn][kMaxMerged];
};

// The pending affine maps of an op's inputs, read out of the launch parameters in one go.  Every
// field is read unconditionally, so the reads become a few wide scalar loads at the top of the
// kernel whose latency overlaps with the operand loads, instead of one dependent scalar load
// behind each branch.
template <typename T, int NIN>
struct AffineRegs {
    unsigned scale_mask, shift_mask;
    T scale[NIN], shift[NIN];
    int scale_aux[NIN], shift_aux[NIN];
    template <class P>
    __device__ __forceinline__ explicit AffineRegs(const P &p) : scale_mask(p.scale_mask), shift_mask(p.shift_mask) {
#pragma unroll
        for (int k = 0; k < NIN; ++k) {
            scale[k] = static_cast<T>(p.scale[k]);
            shift[k] = static_cast<T>(p.shift[k]);
            scale_aux[k] = p.scale_aux[k];
            shift_aux[k] = p.shift_aux[k];
        }
    }
};

// Apply the inputs' pending affine maps to the V points a thread has gathered: multiply, then
// add, each rounded on its own.  `x` holds the op's NIN inputs followed by NAUX auxiliary
// operands (array-valued factors / offsets).  All tests are wave-uniform and made once per
// input, not once per point, so plain operands pay a few scalar branches per thread.
template <typename T, int NIN, int NAUX, int V>
__device__ __forceinline__ void apply_affine(const AffineRegs<T, NIN> &r, T (&x)[NIN + NAUX][V]) {
    if (NAUX == 0 && (r.scale_mask | r.shift_mask) == 0) return;
#pragma unroll
    for (int k = 0; k < NIN; ++k) {
        if (r.scale_mask & (1u << k)) {
#pragma unroll
            for (int j = 0; j < V; ++j) x[k][j] = x[k][j] * r.scale[k];
        }
        if (NAUX > 0 && r.scale_aux[k] >= 0) {
#pragma unroll
            for (int a = 0; a < NAUX; ++a)
                if (r.scale_aux[k] == NIN + a) {
#pragma unroll
                    for (int j = 0; j < V; ++j) x[k][j] = x[k][j] * x[NIN + a][j];
                }
        }
        if (r.shift_mask & (1u << k)) {
#pragma unroll
            for (int j = 0; j < V; ++j) x[k][j] = x[k][j] + r.shift[k];
        }
        if (NAUX > 0 && r.shift_aux[k] >= 0) {
#pragma unroll
            for (int a = 0; a < NAUX; ++a)
                if (r.shift_aux[k] == NIN + a) {
#pragma unroll
                    for (int j = 0; j < V; ++j) x[k][j] = x[k][j] + x[NIN + a][j];
                }
        }
    }
}

template <typename T>
struct Vec {
    static constexpr int N = 16 / sizeof(T);
    // element-aligned vector: 16-byte global accesses that only need sizeof(T) alignment, so
    // views that start at an odd element (x[1:]) still move 16 bytes per lane
    typedef T type __attribute__((ext_vector_type(N), aligned(sizeof(T))));
};

// ---- flat ------------------------------------------------------------------------------
template <template <typename> class F, typename T, int NAUX>
__global__ __launch_bounds__(kBlock) void ew_flat(const EwParams p) {
    using Fn = F<T>;
    constexpr int NP = Fn::NIN + NAUX;
    constexpr int V = Vec<T>::N;
    using vec_t = typename Vec<T>::type;
    const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) * V;
    if (i0 >= p.n) return;
    const AffineRegs<T, Fn::NIN> affine(p);
    T x[NP][V];
    T o[Fn::NOUT][V];
    if (i0 + V <= p.n) {
#pragma unroll
        for (int k = 0; k < NP; ++k) {
            if (k < Fn::NIN && (p.scalar_mask & (1u << k))) {
                const T s = static_cast<T>(p.scalar[k]);
#pragma unroll
                for (int j = 0; j < V; ++j) x[k][j] = s;
            } else if (p.istr[k][0] == 0) {
                const T s = *static_cast<const T *>(p.in[k]);
#pragma unroll
                for (int j = 0; j < V; ++j) x[k][j] = s;
            } else {
                // each element is read once: a streaming (nontemporal) load keeps it from displacing
                // cache lines that will be read again (measured: +5..10 % on arrays beyond the caches)
                const vec_t v = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(static_cast<const T *>(p.in[k]) + i0));
#pragma unroll
                for (int j = 0; j < V; ++j) x[k][j] = v[j];
            }
        }
        apply_affine<T, Fn::NIN, NAUX, V>(affine, x);
#pragma unroll
        for (int j = 0; j < V; ++j) {
            T xi[Fn::NIN], oi[Fn::NOUT];
#pragma unroll
            for (int k = 0; k < Fn::NIN; ++k) xi[k] = x[k][j];
            Fn::apply(xi, oi);
#pragma unroll
            for (int k = 0; k < Fn::NOUT; ++k) o[k][j] = oi[k];
        }
#pragma unroll
        for (int k = 0; k < Fn::NOUT; ++k) {
            vec_t v;
#pragma unroll
            for (int j = 0; j < V; ++j) v[j] = o[k][j];
            *reinterpret_cast<vec_t *>(static_cast<T *>(p.out[k]) + i0) = v;
        }
    } else {
        for (int64_t i = i0; i < p.n; ++i) {
            T x1[NP][1], xi[Fn::NIN], oi[Fn::NOUT];
#pragma unroll
            for (int k = 0; k < NP; ++k) {
                if (k < Fn::NIN && (p.scalar_mask & (1u << k)))
                    x1[k][0] = static_cast<T>(p.scalar[k]);
                else
                    x1[k][0] = static_cast<const T *>(p.in[k])[p.istr[k][0] == 0 ? 0 : i];
            }
            apply_affine<T, Fn::NIN, NAUX, 1>(affine, x1);
#pragma unroll
            for (int k = 0; k < Fn::NIN; ++k) xi[k] = x1[k][0];
            Fn::apply(xi, oi);
#pragma unroll
            for (int k = 0; k < Fn::NOUT; ++k) static_cast<T *>(p.out[k])[i] = oi[k];
        }
    }
}

// ---- rows ------------------------------------------------------------------------------
// shape = (R, C); every operand has inner stride 1 or 0.  `tpr` = threads per row.
template <template <typename> class F, typename T, typename Index, int NAUX>
__global__ __launch_bounds__(kBlock) void ew_rows(const EwParams p, const Index tpr, const Index total,
                                                  const int tile_shift) {
    using Fn = F<T>;
    constexpr int NP = Fn::NIN + NAUX;
    constexpr int V = Vec<T>::N;
    using vec_t = typename Vec<T>::type;
    Index row, in_row;
    if (tile_shift >= 0) {
        // a row spans 2^tile_shift whole blocks: the row comes from the block index with scalar shifts,
        // where the general mapping below spends some 25 vector instructions on an integer division
        row = static_cast<Index>(blockIdx.x >> tile_shift);
        in_row = static_cast<Index>(((blockIdx.x & ((1u << tile_shift) - 1u)) * kBlock) + threadIdx.x);
        if (in_row >= tpr) return;
    } else {
        const Index t = static_cast<Index>(blockIdx.x) * kBlock + threadIdx.x;
        if (t >= total) return;
        row = t / tpr;
        in_row = t - row * tpr;
    }
    const int64_t c0 = static_cast<int64_t>(in_row) * V;
    const int64_t C = p.shape[1];
    const bool full = c0 + V <= C;
    const int nvalid = full ? V : static_cast<int>(C - c0);
    // every operand's descriptor is read before the first load is issued (see AffineRegs)
    const unsigned scalar_mask = p.scalar_mask;
    const AffineRegs<T, Fn::NIN> affine(p);
    const T *bases[NP];
    bool broadcast[NP];
#pragma unroll
    for (int k = 0; k < NP; ++k) {
        const int64_t outer = p.istr[k][0];
        bases[k] = static_cast<const T *>(p.in[k]) + static_cast<int64_t>(row) * outer;
        const int64_t inner = p.istr[k][1];
        // keep the compiler from sinking these reads back behind the branches that use them
        asm volatile("" : : "v"(bases[k]), "s"(inner));
        broadcast[k] = inner == 0;
    }
    T x[NP][V];
#pragma unroll
    for (int k = 0; k < NP; ++k) {
        if (k < Fn::NIN && (scalar_mask & (1u << k))) {
            const T s = static_cast<T>(p.scalar[k]);
#pragma unroll
            for (int j = 0; j < V; ++j) x[k][j] = s;
        } else {
            const T *base = bases[k];
            if (broadcast[k]) {
                const T s = *base;
#pragma unroll
                for (int j = 0; j < V; ++j) x[k][j] = s;
            } else if (full) {
                const vec_t *src = reinterpret_cast<const vec_t *>(base + c0);
                // (an ordinary load: written as `once ? nontemporal : ordinary` the two loads are merged by the
                // optimiser and the hint is lost, and rows of a matrix are often read again by the next rule)
                const vec_t v = *src;
#pragma unroll
                for (int j = 0; j < V; ++j) x[k][j] = v[j];
            } else {
#pragma unroll
                for (int j = 0; j < V; ++j) x[k][j] = j < nvalid ? base[c0 + j] : T(1);
            }
        }
    }
    apply_affine<T, Fn::NIN, NAUX, V>(affine, x);
    T o[Fn::NOUT][V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        T xi[Fn::NIN], oi[Fn::NOUT];
#pragma unroll
        for (int k = 0; k < Fn::NIN; ++k) xi[k] = x[k][j];
        Fn::apply(xi, oi);
#pragma unroll
        for (int k = 0; k < Fn::NOUT; ++k) o[k][j] = oi[k];
    }
#pragma unroll
    for (int k = 0; k < Fn::NOUT; ++k) {
        T *base = static_cast<T *>(p.out[k]) + static_cast<int64_t>(row) * p.ostr[k][0];
        if (full) {
            vec_t v;
#pragma unroll
            for (int j = 0; j < V; ++j) v[j] = o[k][j];
            *reinterpret_cast<vec_t *>(base + c0) = v;
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j)
                if (j < nvalid) base[c0 + j] = o[k][j];
        }
    }
}

// ---- nd --------------------------------------------------------------------------------
template <template <typename> class F, typename T, typename Index, int NAUX>
__global__ __launch_bounds__(kBlock) void ew_nd(const EwParams p) {
    using Fn = F<T>;
    constexpr int NP = Fn::NIN + NAUX;
    Index rem = static_cast<Index>(blockIdx.x) * kBlock + threadIdx.x;
    if (static_cast<int64_t>(rem) >= p.n) return;
    int64_t ioff[NP];
    int64_t ooff[Fn::NOUT];
#pragma unroll
    for (int k = 0; k < NP; ++k) ioff[k] = 0;
#pragma unroll
    for (int k = 0; k < Fn::NOUT; ++k) ooff[k] = 0;
    for (int d = p.ndim - 1; d >= 0; --d) {
        const Index extent = static_cast<Index>(p.shape[d]);
        const Index q = rem / extent;
        const int64_t c = static_cast<int64_t>(rem - q * extent);
        rem = q;
#pragma unroll
        for (int k = 0; k < NP; ++k) ioff[k] += c * p.istr[k][d];
#pragma unroll
        for (int k = 0; k < Fn::NOUT; ++k) ooff[k] += c * p.ostr[k][d];
    }
    const AffineRegs<T, Fn::NIN> affine(p);
    T x1[NP][1], xi[Fn::NIN], oi[Fn::NOUT];
#pragma unroll
    for (int k = 0; k < NP; ++k)
        x1[k][0] = (k < Fn::NIN && (p.scalar_mask & (1u << k))) ? static_cast<T>(p.scalar[k]) : static_cast<const T *>(p.in[k])[ioff[k]];
    apply_affine<T, Fn::NIN, NAUX, 1>(affine, x1);
#pragma unroll
    for (int k = 0; k < Fn::NIN; ++k) xi[k] = x1[k][0];
    Fn::apply(xi, oi);
#pragma unroll
    for (int k = 0; k < Fn::NOUT; ++k) static_cast<T *>(p.out[k])[ooff[k]] = oi[k];
}

// ---- host side -------------------------------------------------------------------------
static int check_blocks(int64_t blocks) {
    if (blocks > 0x7fffffffLL) {
        set_error("elementwise: index space too large for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    return 0;
}

template <template <typename> class F, typename T>
static int launch_ew(const char *fname, const Merged &m, int n_out, const agmi_array *outs, int n_in,
                     const agmi_array *ins, const double *scalars, hipStream_t s) {
    using Fn = F<T>;
    const int n_aux = n_in - Fn::NIN;
    if (n_aux < 0 || n_aux > AGMI_MAX_AUX || n_out != Fn::NOUT) {
        set_error("elementwise: op takes %d inputs (+ at most %d auxiliary) and %d outputs, got %d and %d", Fn::NIN,
                  AGMI_MAX_AUX, Fn::NOUT, n_in, n_out);
        return AGMI_ERR_ARG;
    }
    if (m.ndim > kMaxMerged) {
        set_error("elementwise: %d axes remain after merging, at most %d are supported", m.ndim, kMaxMerged);
        return AGMI_ERR_UNSUPPORTED;
    }
    EwParams p = {};
    p.ndim = m.ndim;
    p.n = m.n;
    for (int d = 0; d < m.ndim; ++d) p.shape[d] = m.shape[d];
    for (int k = 0; k < n_out; ++k) {
        p.out[k] = outs[k].data;
        for (int d = 0; d < m.ndim; ++d) {
            p.ostr[k][d] = m.stride[k][d];
            if (m.stride[k][d] == 0 && m.shape[d] > 1) {
                set_error("elementwise: output %d has stride 0 on an axis of extent %lld", k, (long long)m.shape[d]);
                return AGMI_ERR_ARG;
            }
        }
    }
    for (int k = 0; k < AGMI_MAX_INPUTS; ++k) p.scale_aux[k] = p.shift_aux[k] = -1;
    for (int k = 0; k < n_in; ++k) {
        p.in[k] = ins[k].data;
        if (ins[k].data == nullptr) {
            if (scalars == nullptr || k >= Fn::NIN) {
                set_error("elementwise: scalar slot %d without scalars array (auxiliary inputs must be arrays)", k);
                return AGMI_ERR_ARG;
            }
            p.scalar_mask |= 1u << k;
            p.scalar[k] = scalars[k];
        } else if (k < Fn::NIN) {
            if (!read_affine(ins[k], Fn::NIN, n_in, k, &p)) return AGMI_ERR_ARG;
        }
        for (int d = 0; d < m.ndim; ++d) p.istr[k][d] = m.stride[n_out + k][d];
    }

    constexpr int V = Vec<T>::N;
    bool inner_unit = true;  // every operand's innermost stride is 1 (outputs) or 0/1 (inputs)
    const int last = m.ndim - 1;
    for (int k = 0; k < n_out; ++k) inner_unit &= (p.ostr[k][last] == 1 || m.shape[last] == 1);
    for (int k = 0; k < n_in; ++k)
        inner_unit &= (p.scalar_mask & (1u << k)) || p.istr[k][last] == 1 || p.istr[k][last] == 0;
    // the kernels are instantiated for 0, 1 and 2 auxiliary operands
    auto with_naux = [&](auto launch) {
        if (n_aux == 0) launch(std::integral_constant<int, 0>{});
        else if (n_aux == 1) launch(std::integral_constant<int, 1>{});
        else launch(std::integral_constant<int, 2>{});
    };
    if (m.ndim == 1 && inner_unit) {
        const int64_t blocks = ceil_div(ceil_div(m.n, V), kBlock);
        if (int rc = check_blocks(blocks)) return rc;
        set_kernel_name("ew_flat<%s>[%lld]", fname, (long long)m.n);
        with_naux([&](auto na) {
            hipLaunchKernelGGL((ew_flat<F, T, decltype(na)::value>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p);
        });
    } else if (m.ndim == 2 && inner_unit) {
        const int64_t tpr = ceil_div(m.shape[1], V);
        const int64_t total = tpr * m.shape[0];
        int64_t blocks = ceil_div(total, kBlock);
        // whole blocks per row, a power of two of them, and little idle tail: block index -> row by shifts
        const int64_t tiles = ceil_div(tpr, kBlock);
        int tile_shift = -1;
        if ((tiles & (tiles - 1)) == 0 && (tpr % kBlock == 0 || tiles >= 4) && tiles * m.shape[0] < 0x7fffffffLL) {
            tile_shift = 0;
            while ((int64_t(1) << tile_shift) < tiles) ++tile_shift;
            blocks = tiles * m.shape[0];
        }
        if (int rc = check_blocks(blocks)) return rc;
        set_kernel_name("ew_rows<%s>[%lldx%lld]", fname, (long long)m.shape[0], (long long)m.shape[1]);
        if (total < 0x7fffffffLL)
            with_naux([&](auto na) {
                hipLaunchKernelGGL((ew_rows<F, T, unsigned, decltype(na)::value>), dim3((unsigned)blocks), dim3(kBlock), 0,
                                   s, p, (unsigned)tpr, (unsigned)total, tile_shift);
            });
        else
            with_naux([&](auto na) {
                hipLaunchKernelGGL((ew_rows<F, T, int64_t, decltype(na)::value>), dim3((unsigned)blocks), dim3(kBlock), 0,
                                   s, p, tpr, total, tile_shift);
            });
    } else {
        const int64_t blocks = ceil_div(m.n, kBlock);
        if (int rc = check_blocks(blocks)) return rc;
        set_kernel_name("ew_nd<%s>[%lld]", fname, (long long)m.n);
        if (m.n < 0x7fffffffLL)
            with_naux([&](auto na) {
                hipLaunchKernelGGL((ew_nd<F, T, unsigned, decltype(na)::value>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p);
            });
        else
            with_naux([&](auto na) {
                hipLaunchKernelGGL((ew_nd<F, T, int64_t, decltype(na)::value>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p);
            });
    }
    return hip_check(hipGetLastError(), "elementwise launch");
}

// ---- compare and cast (not on the bandwidth-critical path: nd indexing only) -----------------
struct MixParams {
    void *out;
    const void *in[2];
    double scalar[2];
    unsigned scalar_mask;
    int ndim;
    int64_t n;
    int64_t shape[kMaxMerged];
    int64_t ostr[kMaxMerged];
    int64_t istr[2][kMaxMerged];
};

template <typename Index>
__device__ __forceinline__ void nd_offsets(const MixParams &p, Index rem, int n_in, int64_t *ioff, int64_t *ooff) {
    for (int d = p.ndim - 1; d >= 0; --d) {
        const Index extent = static_cast<Index>(p.shape[d]);
        const Index q = rem / extent;
        const int64_t c = static_cast<int64_t>(rem - q * extent);
        rem = q;
        for (int k = 0; k < n_in; ++k) ioff[k] += c * p.istr[k][d];
        *ooff += c * p.ostr[d];
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void compare_nd(const MixParams p, const int cmp) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= p.n) return;
    int64_t ioff[2] = {0, 0}, ooff = 0;
    nd_offsets<int64_t>(p, i, 2, ioff, &ooff);
    const T a = (p.scalar_mask & 1u) ? static_cast<T>(p.scalar[0]) : static_cast<const T *>(p.in[0])[ioff[0]];
    const T b = (p.scalar_mask & 2u) ? static_cast<T>(p.scalar[1]) : static_cast<const T *>(p.in[1])[ioff[1]];
    bool r;
    switch (cmp) {
        case AGMI_EQ: r = a == b; break;
        case AGMI_NE: r = a != b; break;
        case AGMI_LT: r = a < b; break;
        case AGMI_LE: r = a <= b; break;
        case AGMI_GT: r = a > b; break;
        default: r = a >= b; break;
    }
    static_cast<uint8_t *>(p.out)[ooff] = r ? 1 : 0;
}

template <typename S, typename D>
__global__ __launch_bounds__(kBlock) void cast_nd(const MixParams p) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= p.n) return;
    int64_t ioff[2] = {0, 0}, ooff = 0;
    nd_offsets<int64_t>(p, i, 1, ioff, &ooff);
    const S v = static_cast<const S *>(p.in[0])[ioff[0]];
    D r;
    if constexpr (sizeof(D) == 1)
        r = static_cast<D>(v != S(0) ? 1 : 0);  // to bool
    else
        r = static_cast<D>(v);
    static_cast<D *>(p.out)[ooff] = r;
}

static bool fill_mix(const Merged &m, const agmi_array *out, int n_in, const agmi_array *ins, const double *scalars,
                     MixParams *p) {
    if (m.ndim > kMaxMerged) {
        set_error("%d axes remain after merging, at most %d are supported", m.ndim, kMaxMerged);
        return false;
    }
    *p = MixParams{};
    p->ndim = m.ndim;
    p->n = m.n;
    p->out = out->data;
    for (int d = 0; d < m.ndim; ++d) {
        p->shape[d] = m.shape[d];
        p->ostr[d] = m.stride[0][d];
    }
    for (int k = 0; k < n_in; ++k) {
        p->in[k] = ins[k].data;
        if (ins[k].data == nullptr) {
            if (!scalars) {
                set_error("scalar slot %d without scalars array", k);
                return false;
            }
            p->scalar_mask |= 1u << k;
            p->scalar[k] = scalars[k];
        }
        for (int d = 0; d < m.ndim; ++d) p->istr[k][d] = m.stride[1 + k][d];
    }
    return true;
}

template <typename S>
static int launch_cast_from(int dst_dtype, const MixParams &p, unsigned blocks, hipStream_t s) {
    switch (dst_dtype) {
        case AGMI_F32: hipLaunchKernelGGL((cast_nd<S, float>), dim3(blocks), dim3(kBlock), 0, s, p); break;
        case AGMI_F64: hipLaunchKernelGGL((cast_nd<S, double>), dim3(blocks), dim3(kBlock), 0, s, p); break;
        case AGMI_BOOL: hipLaunchKernelGGL((cast_nd<S, uint8_t>), dim3(blocks), dim3(kBlock), 0, s, p); break;
        case AGMI_I64: hipLaunchKernelGGL((cast_nd<S, int64_t>), dim3(blocks), dim3(kBlock), 0, s, p); break;
        case AGMI_I32: hipLaunchKernelGGL((cast_nd<S, int32_t>), dim3(blocks), dim3(kBlock), 0, s, p); break;
        default: set_error("cast: unknown destination dtype %d", dst_dtype); return AGMI_ERR_ARG;
    }
    return hip_check(hipGetLastError(), "cast launch");
}

}  // namespace agmi

using namespace agmi;

// This file is compiled twice, once per precision (-DAGMI_PART=32 / 64), so that the two halves of
// the functor x layout instantiations build in parallel; the entry points live in the float32 half.
#ifndef AGMI_PART
#error "compile with -DAGMI_PART=32 or -DAGMI_PART=64"
#endif
namespace agmi {
int elementwise_part_f32(int op, const Merged &m, int n_out, const agmi_array *outs, int n_in, const agmi_array *ins,
                         const double *scalars, hipStream_t s);
int elementwise_part_f64(int op, const Merged &m, int n_out, const agmi_array *outs, int n_in, const agmi_array *ins,
                         const double *scalars, hipStream_t s);
#if AGMI_PART == 32
#define AGMI_PART_FN elementwise_part_f32
using PartT = float;
#else
#define AGMI_PART_FN elementwise_part_f64
using PartT = double;
#endif
int AGMI_PART_FN(int op, const Merged &m, int n_out, const agmi_array *outs, int n_in, const agmi_array *ins,
                 const double *scalars, hipStream_t s) {
#define AGMI_CASE(OP, FN) \
    case OP: return launch_ew<FN, PartT>(#FN, m, n_out, outs, n_in, ins, scalars, s);
    switch (op) {
        AGMI_FOR_EACH_OP(AGMI_CASE)
        default: set_error("elementwise: unknown op %d", op); return AGMI_ERR_ARG;
    }
#undef AGMI_CASE
}
#undef AGMI_PART_FN
}  // namespace agmi

#if AGMI_PART == 32
extern "C" int agmi_elementwise(int op, int dtype, int ndim, const int64_t *shape, int n_out,
                                const agmi_array *outs, int n_in, const agmi_array *ins,
                                const double *scalars, void *stream) {
    if (n_out < 1 || n_out > AGMI_MAX_OUTPUTS || n_in < 1 || n_in > kMaxPhysIn || !outs || !ins) {
        set_error("elementwise: bad operand counts or null operand arrays");
        return AGMI_ERR_ARG;
    }
    if (index_space_is_empty(ndim, shape)) return 0;  // nothing to compute; empty arrays have null data
    const int64_t *strides[kMaxOperands];
    for (int k = 0; k < n_out; ++k) {
        if (outs[k].data == nullptr) {
            set_error("elementwise: output %d is null", k);
            return AGMI_ERR_ARG;
        }
        strides[k] = outs[k].strides;
    }
    for (int k = 0; k < n_in; ++k) strides[n_out + k] = ins[k].data ? ins[k].strides : nullptr;
    Merged m;
    if (!merge_axes(ndim, shape, nullptr, n_out + n_in, strides, &m)) return AGMI_ERR_ARG;
    if (m.n == 0) return 0;
    hipStream_t s = as_stream(stream);
    if (dtype == AGMI_F32) return elementwise_part_f32(op, m, n_out, outs, n_in, ins, scalars, s);
    if (dtype == AGMI_F64) return elementwise_part_f64(op, m, n_out, outs, n_in, ins, scalars, s);
    set_error("elementwise: dtype %d is not a floating type", dtype);
    return AGMI_ERR_ARG;
}

extern "C" int agmi_compare(int cmp, int dtype, int ndim, const int64_t *shape, const agmi_array *out,
                            const agmi_array *ins, const double *scalars, void *stream) {
    if (index_space_is_empty(ndim, shape)) return 0;
    if (!out || !ins || !out->data || cmp < AGMI_EQ || cmp > AGMI_GE) {
        set_error("compare: bad arguments");
        return AGMI_ERR_ARG;
    }
    const int64_t *strides[3] = {out->strides, ins[0].data ? ins[0].strides : nullptr,
                                 ins[1].data ? ins[1].strides : nullptr};
    Merged m;
    if (!merge_axes(ndim, shape, nullptr, 3, strides, &m)) return AGMI_ERR_ARG;
    if (m.n == 0) return 0;
    MixParams p;
    if (!fill_mix(m, out, 2, ins, scalars, &p)) return AGMI_ERR_UNSUPPORTED;
    const int64_t blocks = ceil_div(m.n, kBlock);
    if (int rc = check_blocks(blocks)) return rc;
    hipStream_t s = as_stream(stream);
    set_kernel_name("compare_nd");
    if (dtype == AGMI_F32)
        hipLaunchKernelGGL(compare_nd<float>, dim3((unsigned)blocks), dim3(kBlock), 0, s, p, cmp);
    else if (dtype == AGMI_F64)
        hipLaunchKernelGGL(compare_nd<double>, dim3((unsigned)blocks), dim3(kBlock), 0, s, p, cmp);
    else {
        set_error("compare: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    return hip_check(hipGetLastError(), "compare launch");
}

extern "C" int agmi_cast(int src_dtype, int dst_dtype, int ndim, const int64_t *shape, const agmi_array *out,
                         const agmi_array *in, void *stream) {
    if (index_space_is_empty(ndim, shape)) return 0;
    if (!out || !in || !out->data || !in->data) {
        set_error("cast: null operand");
        return AGMI_ERR_ARG;
    }
    const int64_t *strides[2] = {out->strides, in->strides};
    Merged m;
    if (!merge_axes(ndim, shape, nullptr, 2, strides, &m)) return AGMI_ERR_ARG;
    if (m.n == 0) return 0;
    MixParams p;
    if (!fill_mix(m, out, 1, in, nullptr, &p)) return AGMI_ERR_UNSUPPORTED;
    const int64_t blocks = ceil_div(m.n, kBlock);
    if (int rc = check_blocks(blocks)) return rc;
    hipStream_t s = as_stream(stream);
    set_kernel_name("cast_nd");
    switch (src_dtype) {
        case AGMI_F32: return launch_cast_from<float>(dst_dtype, p, (unsigned)blocks, s);
        case AGMI_F64: return launch_cast_from<double>(dst_dtype, p, (unsigned)blocks, s);
        case AGMI_BOOL: return launch_cast_from<uint8_t>(dst_dtype, p, (unsigned)blocks, s);
        case AGMI_I64: return launch_cast_from<int64_t>(dst_dtype, p, (unsigned)blocks, s);
        case AGMI_I32: return launch_cast_from<int32_t>(dst_dtype, p, (unsigned)blocks, s);
        default: set_error("cast: unknown source dtype %d", src_dtype); return AGMI_ERR_ARG;
    }
}
#endif  // AGMI_PART == 32
