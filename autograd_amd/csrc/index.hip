// Integer-array indexing along the leading axis: gather (forward of A[idx]) and the ordered
// scatter-add that is its cotangent (numpy.add.at semantics, bit for bit).
//
// Basic slices never come here: they are strided views and their cotangent is a strided
// in-place add through agmi_elementwise.  For an index ARRAY, several positions may name the
// same destination row and NumPy adds them one after another in index order; floating-point
// addition is not associative, so the kernel reproduces exactly that order: the caller
// supplies the stable argsort of the destinations and the run boundaries, one thread owns
// one (destination row, column) pair and walks its run sequentially.  No atomics.
#include <algorithm>
#include <cstdint>

#include <type_traits>

#include "common.h"

namespace agmi {

template <typename T>
__device__ __forceinline__ T out_of_range_fill() {
    if constexpr (std::is_floating_point<T>::value)
        return static_cast<T>(__builtin_nanf(""));
    else
        return T(0);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void take_rows_kernel(const T *__restrict__ src, int64_t n_rows, int64_t inner,
                                                           const int64_t *__restrict__ index, int64_t n_index,
                                                           T *__restrict__ out) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= n_index * inner) return;
    const int64_t i = e / inner, c = e - i * inner;
    int64_t r = index[i];
    if (r < 0) r += n_rows;
    // An index outside [-n_rows, n_rows) never reaches memory (NumPy raises IndexError; the values of a
    // device-resident index are not known on the host): the row reads as NaN (zero for integer arrays).
    if (static_cast<uint64_t>(r) >= static_cast<uint64_t>(n_rows)) {
        out[e] = out_of_range_fill<T>();
        return;
    }
    out[e] = src[r * inner + c];
}

// The same accumulation when the runs of equal destination are not listed: one thread per position of the
// sorted order (and column); a thread whose position starts a run (its destination differs from the
// previous position's) adds the whole run in order, the others leave.  Nothing about the index has to be
// known on the host, so the call can be recorded into a graph with a device-resident index.
template <typename T>
__global__ __launch_bounds__(kBlock) void scatter_add_runs_kernel(T *__restrict__ dst, int64_t n_rows, int64_t inner,
                                                                  const T *__restrict__ src,
                                                                  const int64_t *__restrict__ index,
                                                                  const int64_t *__restrict__ order, int64_t n_index) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= n_index * inner) return;
    const int64_t pos = e / inner, c = e - pos * inner;
    int64_t r = index[order[pos]];
    if (r < 0) r += n_rows;
    if (static_cast<uint64_t>(r) >= static_cast<uint64_t>(n_rows)) return;  // no such row: the addends are dropped, nothing is touched
    if (pos > 0) {
        int64_t before = index[order[pos - 1]];
        if (before < 0) before += n_rows;
        if (before == r) return;  // inside a run: its first position does the work
    }
    T acc = dst[r * inner + c];
    for (int64_t k = pos; k < n_index; ++k) {
        int64_t rk = index[order[k]];
        if (rk < 0) rk += n_rows;
        if (rk != r) break;
        acc = acc + src[order[k] * inner + c];
    }
    dst[r * inner + c] = acc;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void scatter_add_rows_kernel(T *__restrict__ dst, int64_t n_rows, int64_t inner,
                                                                  const T *__restrict__ src,
                                                                  const int64_t *__restrict__ index,
                                                                  const int64_t *__restrict__ order,
                                                                  const int64_t *__restrict__ seg_start, int64_t n_seg) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= n_seg * inner) return;
    const int64_t seg = e / inner, c = e - seg * inner;
    const int64_t begin = seg_start[seg], end = seg_start[seg + 1];
    int64_t r = index[order[begin]];
    if (r < 0) r += n_rows;
    if (static_cast<uint64_t>(r) >= static_cast<uint64_t>(n_rows)) return;  // no such row: the addends are dropped
    T acc = dst[r * inner + c];
    for (int64_t k = begin; k < end; ++k) acc = acc + src[order[k] * inner + c];
    dst[r * inner + c] = acc;
}

// Running sums along the middle axis of a contiguous (outer, n, inner) array, added in index order like
// numpy.add.accumulate, so the result is bit-identical to NumPy's.  One thread owns one (outer, inner) line;
// neighbouring threads read neighbouring `inner` positions.
template <typename T>
__global__ __launch_bounds__(kBlock) void cumsum_lines(const T *__restrict__ src, int64_t outer, int64_t n,
                                                       int64_t inner, T *__restrict__ out) {
    const int64_t line = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (line >= outer * inner) return;
    const int64_t o = line / inner, c = line - o * inner;
    const T *p = src + o * n * inner + c;
    T *q = out + o * n * inner + c;
    // the additions form one chain, but the loads do not depend on it: fetch kLineChunk elements at once (the bytes in flight per thread set the rate)
    constexpr int kLineChunk = 64;
    T acc = p[0];
    q[0] = acc;
    int64_t k = 1;
    for (; k + kLineChunk <= n; k += kLineChunk) {
        T v[kLineChunk];
#pragma unroll
        for (int u = 0; u < kLineChunk; ++u) v[u] = p[(k + u) * inner];
#pragma unroll
        for (int u = 0; u < kLineChunk; ++u) {
            acc = acc + v[u];
            q[(k + u) * inner] = acc;
        }
    }
    for (; k < n; ++k) {
        acc = acc + p[k * inner];
        q[k * inner] = acc;
    }
}

// The same along the last axis (inner == 1): one wavefront takes kScanRows rows and walks them in chunks of
// kScanCols columns staged through LDS, so that global loads and stores run along the rows (coalesced, all of a
// chunk's loads in flight together) while one lane per row still adds that row's elements one after the other.
// Few rows per wavefront and wide chunks: the chain of additions is short next to the memory latency of a
// chunk, so throughput comes from the number of wavefronts in flight.
constexpr int kScanRows = 16, kScanCols = 256, kScanGroups = kScanCols / 64;

template <typename T>
__global__ __launch_bounds__(64) void cumsum_rows(const T *__restrict__ src, int64_t rows, int64_t n,
                                                  T *__restrict__ out) {
    __shared__ T tile[kScanRows][kScanCols + 1];
    const int lane = threadIdx.x;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kScanRows;
    const int live = static_cast<int>(rows - row0 < kScanRows ? rows - row0 : kScanRows);
    T acc = T(0);
    for (int64_t c0 = 0; c0 < n; c0 += kScanCols) {
        {
            T v[kScanRows * kScanGroups];
#pragma unroll
            for (int r = 0; r < kScanRows; ++r)
#pragma unroll
                for (int g = 0; g < kScanGroups; ++g) {
                    const int64_t col = c0 + g * 64 + lane;
                    v[r * kScanGroups + g] = (r < live && col < n) ? src[(row0 + r) * n + col] : T(0);
                }
#pragma unroll
            for (int r = 0; r < kScanRows; ++r)
#pragma unroll
                for (int g = 0; g < kScanGroups; ++g) tile[r][g * 64 + lane] = v[r * kScanGroups + g];
        }
        __syncthreads();
        if (lane < live) {
            const int width = static_cast<int>(n - c0 < kScanCols ? n - c0 : kScanCols);
            int j = 0;
            if (c0 == 0) {  // the row's first element starts the chain as it is (0 + x would turn -0.0 into +0.0)
                acc = tile[lane][0];
                j = 1;
            }
#pragma unroll 8
            for (; j < width; ++j) {
                acc = acc + tile[lane][j];
                tile[lane][j] = acc;
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kScanRows; ++r)
#pragma unroll
            for (int g = 0; g < kScanGroups; ++g) {
                const int64_t col = c0 + g * 64 + lane;
                if (r < live && col < n) out[(row0 + r) * n + col] = tile[r][g * 64 + lane];
            }
        __syncthreads();
    }
}

// out[o, k, c] = src[o, n - 1 - k, c] on contiguous (outer, n, inner) arrays: the copy behind a slice
// that steps backwards (device views cannot carry negative strides).
template <typename T>
__global__ __launch_bounds__(kBlock) void reverse_axis_kernel(const T *__restrict__ src, int64_t total, int64_t n,
                                                              int64_t inner, T *__restrict__ out) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    const int64_t line = e / inner, c = e - line * inner;
    const int64_t o = line / n, k = line - o * n;
    out[e] = src[(o * n + (n - 1 - k)) * inner + c];
}

// 16-byte variants of the reversal: V = 16 / sizeof(T) consecutive elements per thread.  `reverse_axis_vec_inner`
// copies V neighbours of one line position (inner % V == 0); `reverse_axis_vec_last` is the reversal of the
// contiguous axis itself (inner == 1, n % V == 0): V results come from one aligned vector read backwards.
template <typename T>
struct IndexVec {
    static constexpr int N = 16 / sizeof(T);
    typedef T type __attribute__((ext_vector_type(N)));
};

template <typename T>
__global__ __launch_bounds__(kBlock) void reverse_axis_vec_inner(const T *__restrict__ src, int64_t total_vecs, int64_t n,
                                                                 int64_t inner_vecs, T *__restrict__ out) {
    using vec_t = typename IndexVec<T>::type;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total_vecs) return;
    const int64_t line = e / inner_vecs, c = e - line * inner_vecs;
    const int64_t o = line / n, k = line - o * n;
    reinterpret_cast<vec_t *>(out)[e] = reinterpret_cast<const vec_t *>(src)[(o * n + (n - 1 - k)) * inner_vecs + c];
}

template <typename T>
__global__ __launch_bounds__(kBlock) void reverse_axis_vec_last(const T *__restrict__ src, int64_t total_vecs,
                                                                int64_t n_vecs, T *__restrict__ out) {
    using vec_t = typename IndexVec<T>::type;
    constexpr int V = IndexVec<T>::N;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total_vecs) return;
    const int64_t o = e / n_vecs, kv = e - o * n_vecs;
    const vec_t v = reinterpret_cast<const vec_t *>(src)[o * n_vecs + (n_vecs - 1 - kv)];
    vec_t r;
#pragma unroll
    for (int j = 0; j < V; ++j) r[j] = v[V - 1 - j];
    reinterpret_cast<vec_t *>(out)[e] = r;
}

// tril / triu with V columns per thread (cols % V == 0)
template <typename T>
__global__ __launch_bounds__(kBlock) void triangle_vec_kernel(const T *__restrict__ src, int64_t total_vecs, int64_t rows,
                                                              int64_t col_vecs, int64_t k, int lower, T *__restrict__ out) {
    using vec_t = typename IndexVec<T>::type;
    constexpr int V = IndexVec<T>::N;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total_vecs) return;
    const int64_t line = e / col_vecs, j0 = (e - line * col_vecs) * V;
    const int64_t i = line % rows;
    vec_t v = reinterpret_cast<const vec_t *>(src)[e];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int64_t d = j0 + j - i;
        if (!(lower ? (d <= k) : (d >= k))) v[j] = T(0);
    }
    reinterpret_cast<vec_t *>(out)[e] = v;
}

// out[b, i, j] = src[b, i, j] where j - i <= k (lower) or j - i >= k (upper), else 0: numpy.tril / triu on
// contiguous (batch, rows, cols) arrays.  Masked entries are zeros whatever the source holds (NaN included).
template <typename T>
__global__ __launch_bounds__(kBlock) void triangle_kernel(const T *__restrict__ src, int64_t total, int64_t rows,
                                                          int64_t cols, int64_t k, int lower, T *__restrict__ out) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    const int64_t line = e / cols, j = e - line * cols;
    const int64_t i = line % rows;
    const bool keep = lower ? (j - i <= k) : (j - i >= k);
    out[e] = keep ? src[e] : T(0);
}

// Stable sort of each row of a contiguous (rows, n) array by counting: the rank of an element is the number
// of elements ordered before it (smaller; equal and earlier; any number before a NaN), so no element moves
// until its final place is known and equal elements keep their order.  O(n^2) comparisons per row, tiles of
// the row staged through LDS; meant for the vector lengths sort rules are used on (see kMaxSortLength).
constexpr int64_t kMaxSortLength = 65536;

template <typename T>
__device__ __forceinline__ bool ordered_before(T a, int64_t ja, T b, int64_t jb) {
    const bool a_nan = a != a, b_nan = b != b;
    if (a_nan || b_nan) return (!a_nan && b_nan) || (a_nan && b_nan && ja < jb);
    return a < b || (a == b && ja < jb);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void rank_sort_rows(const T *__restrict__ src, int64_t n, T *__restrict__ sorted,
                                                         int64_t *__restrict__ order, int64_t *__restrict__ rank) {
    __shared__ T tile[kBlock];
    const int64_t row = blockIdx.y;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const T *line = src + row * n;
    const bool live = i < n;
    const T mine = live ? line[i] : T(0);
    int64_t before = 0;
    for (int64_t j0 = 0; j0 < n; j0 += kBlock) {
        const int64_t j = j0 + threadIdx.x;
        tile[threadIdx.x] = j < n ? line[j] : T(0);
        __syncthreads();
        const int width = static_cast<int>(n - j0 < kBlock ? n - j0 : kBlock);
        if (live)
            for (int t = 0; t < width; ++t) before += ordered_before(tile[t], j0 + t, mine, i) ? 1 : 0;
        __syncthreads();
    }
    if (!live) return;
    if (sorted) sorted[row * n + before] = mine;
    if (order) order[row * n + before] = i;
    if (rank) rank[row * n + i] = before;
}

// The same count split over `slices` parts of the row (blockIdx.z), so that a long row fills the chip: every
// block adds its partial count to rank[] with an integer atomic (exact in any order); rank[] starts at zero and
// `place_by_rank` moves the elements once all counts are in.
template <typename T>
__global__ __launch_bounds__(kBlock) void rank_count_slices(const T *__restrict__ src, int64_t n, int64_t tiles_per_slice,
                                                            int64_t *__restrict__ rank) {
    __shared__ T tile[kBlock];
    const int64_t row = blockIdx.y;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const T *line = src + row * n;
    const bool live = i < n;
    const T mine = live ? line[i] : T(0);
    const int64_t j_begin = static_cast<int64_t>(blockIdx.z) * tiles_per_slice * kBlock;
    const int64_t j_end = j_begin + tiles_per_slice * kBlock < n ? j_begin + tiles_per_slice * kBlock : n;
    int64_t before = 0;
    for (int64_t j0 = j_begin; j0 < j_end; j0 += kBlock) {
        const int64_t j = j0 + threadIdx.x;
        tile[threadIdx.x] = j < j_end ? line[j] : T(0);
        __syncthreads();
        const int width = static_cast<int>(j_end - j0 < kBlock ? j_end - j0 : kBlock);
        if (live)
            for (int t = 0; t < width; ++t) before += ordered_before(tile[t], j0 + t, mine, i) ? 1 : 0;
        __syncthreads();
    }
    if (live && before)
        atomicAdd(reinterpret_cast<unsigned long long *>(rank + row * n + i), static_cast<unsigned long long>(before));
}

__global__ __launch_bounds__(kBlock) void zero_ranks(int64_t *__restrict__ rank, int64_t total) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e < total) rank[e] = 0;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void place_by_rank(const T *__restrict__ src, int64_t n, int64_t total,
                                                        const int64_t *__restrict__ rank, T *__restrict__ sorted,
                                                        int64_t *__restrict__ order) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    const int64_t row = e / n, i = e - row * n;
    const int64_t k = rank[e];
    if (sorted) sorted[row * n + k] = src[e];
    if (order) order[row * n + k] = i;
}

// ---- concatenation ------------------------------------------------------------------------------
struct ConcatParams {
    const void *data[AGMI_MAX_CONCAT];
    int64_t end[AGMI_MAX_CONCAT];  // one past the piece's last position along the joined axis
    int64_t so[AGMI_MAX_CONCAT], sa[AGMI_MAX_CONCAT], si[AGMI_MAX_CONCAT];
    int n_pieces;
    int64_t total, inner, n;
};

// one thread per element of the contiguous (outer, total, inner) result; I is the type the element's position is split
// in (32-bit division is a handful of instructions, 64-bit a long routine that tiny joins spend most of their time in)
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void concat_kernel(const ConcatParams p, T *__restrict__ out) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= p.n) return;
    const I inner = static_cast<I>(p.inner), total = static_cast<I>(p.total);
    const I rest = inner == 1 ? static_cast<I>(e) : static_cast<I>(e) / inner;
    const I i = static_cast<I>(e) - rest * inner;
    const I o = rest / total, a = rest - o * total;
    // the piece's pointer and strides are picked by selects between values every lane loads at the same (scalar)
    // addresses: no load waits on the piece number (indexing the table by it would be a second round trip to memory
    // before the element's own)
    const T *src = static_cast<const T *>(p.data[0]);
    int64_t so = p.so[0], sa = p.sa[0], si = p.si[0], begin = 0;
    for (int j = 1; j < p.n_pieces; ++j) {  // (the same trip count for every thread; `end` is non-decreasing)
        if (static_cast<int64_t>(a) >= p.end[j - 1]) {
            src = static_cast<const T *>(p.data[j]);
            so = p.so[j];
            sa = p.sa[j];
            si = p.si[j];
            begin = p.end[j - 1];
        }
    }
    out[e] = src[static_cast<int64_t>(o) * so + (static_cast<int64_t>(a) - begin) * sa + static_cast<int64_t>(i) * si];
}

}  // namespace agmi

using namespace agmi;

extern "C" int agmi_concat(int dtype, int64_t outer, int64_t inner, int n_pieces, const agmi_concat_piece *pieces, void *out,
                           void *stream) {
    if (outer < 0 || inner < 0 || n_pieces < 0 || n_pieces > AGMI_MAX_CONCAT) {
        set_error("concat: bad extents or more than %d pieces", AGMI_MAX_CONCAT);
        return AGMI_ERR_ARG;
    }
    if (n_pieces > 0 && !pieces) {
        set_error("concat: null piece table");
        return AGMI_ERR_ARG;
    }
    ConcatParams p = {};
    int64_t total = 0;
    for (int k = 0; k < n_pieces; ++k) {
        if (pieces[k].extent < 0 || (pieces[k].extent > 0 && outer > 0 && inner > 0 && !pieces[k].data)) {
            set_error("concat: piece %d has a negative extent or no data", k);
            return AGMI_ERR_ARG;
        }
        total += pieces[k].extent;
        p.data[k] = pieces[k].data;
        p.end[k] = total;
        p.so[k] = pieces[k].stride_outer;
        p.sa[k] = pieces[k].stride_axis;
        p.si[k] = pieces[k].stride_inner;
    }
    for (int k = n_pieces; k < AGMI_MAX_CONCAT; ++k) p.end[k] = total;
    p.n_pieces = n_pieces;
    p.total = total;
    p.inner = inner;
    p.n = outer * total * inner;
    if (p.n == 0) return 0;
    if (!out) {
        set_error("concat: null output");
        return AGMI_ERR_ARG;
    }
    const int64_t blocks = ceil_div(p.n, kBlock);
    if (blocks > 0x7fffffffLL) {
        set_error("concat: too many elements");
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    set_kernel_name("concat_kernel");
    const bool narrow = p.n <= 0x7fffffffLL;
    if (dtype == AGMI_F32 && narrow)
        hipLaunchKernelGGL((concat_kernel<float, uint32_t>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p, static_cast<float *>(out));
    else if (dtype == AGMI_F32)
        hipLaunchKernelGGL((concat_kernel<float, int64_t>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p, static_cast<float *>(out));
    else if (dtype == AGMI_F64 && narrow)
        hipLaunchKernelGGL((concat_kernel<double, uint32_t>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p, static_cast<double *>(out));
    else if (dtype == AGMI_F64)
        hipLaunchKernelGGL((concat_kernel<double, int64_t>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p, static_cast<double *>(out));
    else {
        set_error("concat: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    return hip_check(hipGetLastError(), "concat launch");
}

extern "C" int agmi_take_rows(int dtype, const void *src, int64_t n_rows, int64_t inner, const int64_t *index,
                              int64_t n_index, void *out, void *stream) {
    if (n_rows < 0 || inner < 0 || n_index < 0) {
        set_error("take_rows: negative extent");
        return AGMI_ERR_ARG;
    }
    const int64_t n = n_index * inner;
    if (n == 0) return 0;
    if (!src || !index || !out || n_rows == 0) {
        set_error("take_rows: null operand or empty source");
        return AGMI_ERR_ARG;
    }
    const int64_t blocks = ceil_div(n, kBlock);
    if (blocks > 0x7fffffffLL) {
        set_error("take_rows: too many elements");
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    set_kernel_name("take_rows_kernel");
    if (dtype == AGMI_F32)
        hipLaunchKernelGGL(take_rows_kernel<float>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<const float *>(src), n_rows, inner, index, n_index, static_cast<float *>(out));
    else if (dtype == AGMI_F64)
        hipLaunchKernelGGL(take_rows_kernel<double>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<const double *>(src), n_rows, inner, index, n_index, static_cast<double *>(out));
    else {
        set_error("take_rows: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    return hip_check(hipGetLastError(), "take_rows launch");
}

extern "C" int agmi_scatter_add_rows(int dtype, void *dst, int64_t n_rows, int64_t inner, const void *src,
                                     const int64_t *index, const int64_t *order, const int64_t *seg_start,
                                     int64_t n_seg, void *stream) {
    if (n_rows < 0 || inner < 0 || n_seg < 0) {
        set_error("scatter_add_rows: negative extent");
        return AGMI_ERR_ARG;
    }
    const int64_t n = n_seg * inner;
    if (n == 0) return 0;
    if (!dst || !src || !index || !order) {
        set_error("scatter_add_rows: null operand");
        return AGMI_ERR_ARG;
    }
    if (dtype != AGMI_F32 && dtype != AGMI_F64) {
        set_error("scatter_add_rows: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    const int64_t blocks = ceil_div(n, kBlock);
    if (blocks > 0x7fffffffLL) {
        set_error("scatter_add_rows: too many elements");
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    if (!seg_start) {  // runs found on the device: n_seg counts index entries
        set_kernel_name("scatter_add_runs_kernel");
        if (dtype == AGMI_F32)
            hipLaunchKernelGGL(scatter_add_runs_kernel<float>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                               static_cast<float *>(dst), n_rows, inner, static_cast<const float *>(src), index, order, n_seg);
        else
            hipLaunchKernelGGL(scatter_add_runs_kernel<double>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                               static_cast<double *>(dst), n_rows, inner, static_cast<const double *>(src), index, order, n_seg);
        return hip_check(hipGetLastError(), "scatter_add_rows launch");
    }
    set_kernel_name("scatter_add_rows_kernel");
    if (dtype == AGMI_F32)
        hipLaunchKernelGGL(scatter_add_rows_kernel<float>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<float *>(dst), n_rows, inner, static_cast<const float *>(src), index, order,
                           seg_start, n_seg);
    else
        hipLaunchKernelGGL(scatter_add_rows_kernel<double>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<double *>(dst), n_rows, inner, static_cast<const double *>(src), index, order,
                           seg_start, n_seg);
    return hip_check(hipGetLastError(), "scatter_add_rows launch");
}

extern "C" int agmi_cumsum(int dtype, const void *src, int64_t outer, int64_t n, int64_t inner, void *out,
                           void *stream) {
    if (outer < 0 || n < 0 || inner < 0) {
        set_error("cumsum: negative extent");
        return AGMI_ERR_ARG;
    }
    if (outer == 0 || n == 0 || inner == 0) return 0;
    if (!src || !out) {
        set_error("cumsum: null operand");
        return AGMI_ERR_ARG;
    }
    if (dtype != AGMI_F32 && dtype != AGMI_F64) {
        set_error("cumsum: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    const bool rows = inner == 1;
    const int64_t blocks = rows ? ceil_div(outer, kScanRows) : ceil_div(outer * inner, kBlock);
    if (blocks > 0x7fffffffLL) {
        set_error("cumsum: too many lines");
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    set_kernel_name(rows ? "cumsum_rows" : "cumsum_lines");
    if (dtype == AGMI_F32) {
        if (rows)
            hipLaunchKernelGGL(cumsum_rows<float>, dim3((unsigned)blocks), dim3(64), 0, s,
                               static_cast<const float *>(src), outer, n, static_cast<float *>(out));
        else
            hipLaunchKernelGGL(cumsum_lines<float>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                               static_cast<const float *>(src), outer, n, inner, static_cast<float *>(out));
    } else {
        if (rows)
            hipLaunchKernelGGL(cumsum_rows<double>, dim3((unsigned)blocks), dim3(64), 0, s,
                               static_cast<const double *>(src), outer, n, static_cast<double *>(out));
        else
            hipLaunchKernelGGL(cumsum_lines<double>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                               static_cast<const double *>(src), outer, n, inner, static_cast<double *>(out));
    }
    return hip_check(hipGetLastError(), "cumsum launch");
}

namespace {

// shared argument checks of the two copy-shaped entry points below; returns the block count or a negative error
int64_t plan_copy(const char *what, int dtype, const void *src, const void *out, int64_t total) {
    if (!src || !out) {
        set_error("%s: null operand", what);
        return AGMI_ERR_ARG;
    }
    if (dtype != AGMI_F32 && dtype != AGMI_F64) {
        set_error("%s: dtype %d is not a floating type", what, dtype);
        return AGMI_ERR_ARG;
    }
    const int64_t blocks = ceil_div(total, kBlock);
    if (blocks > 0x7fffffffLL) {
        set_error("%s: too many elements", what);
        return AGMI_ERR_UNSUPPORTED;
    }
    return blocks;
}

}  // namespace

extern "C" int agmi_reverse(int dtype, const void *src, int64_t outer, int64_t n, int64_t inner, void *out,
                            void *stream) {
    if (outer < 0 || n < 0 || inner < 0) {
        set_error("reverse: negative extent");
        return AGMI_ERR_ARG;
    }
    const int64_t total = outer * n * inner;
    if (total == 0) return 0;
    int64_t blocks = plan_copy("reverse", dtype, src, out, total);
    if (blocks < 0) return static_cast<int>(blocks);
    hipStream_t s = as_stream(stream);
    {
        const int64_t V = dtype == AGMI_F32 ? 4 : 2;
        const bool aligned = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
        const bool vec_inner = aligned && inner % V == 0, vec_last = aligned && inner == 1 && n % V == 0;
        if (vec_inner || vec_last) {
            const int64_t vecs = total / V;
            const dim3 grid((unsigned)ceil_div(vecs, kBlock));
            set_kernel_name(vec_inner ? "reverse_axis_vec_inner" : "reverse_axis_vec_last");
            if (dtype == AGMI_F32) {
                if (vec_inner)
                    hipLaunchKernelGGL(reverse_axis_vec_inner<float>, grid, dim3(kBlock), 0, s, static_cast<const float *>(src),
                                       vecs, n, inner / V, static_cast<float *>(out));
                else
                    hipLaunchKernelGGL(reverse_axis_vec_last<float>, grid, dim3(kBlock), 0, s, static_cast<const float *>(src),
                                       vecs, n / V, static_cast<float *>(out));
            } else {
                if (vec_inner)
                    hipLaunchKernelGGL(reverse_axis_vec_inner<double>, grid, dim3(kBlock), 0, s,
                                       static_cast<const double *>(src), vecs, n, inner / V, static_cast<double *>(out));
                else
                    hipLaunchKernelGGL(reverse_axis_vec_last<double>, grid, dim3(kBlock), 0, s,
                                       static_cast<const double *>(src), vecs, n / V, static_cast<double *>(out));
            }
            return hip_check(hipGetLastError(), "reverse launch");
        }
    }
    set_kernel_name("reverse_axis_kernel");
    if (dtype == AGMI_F32)
        hipLaunchKernelGGL(reverse_axis_kernel<float>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<const float *>(src), total, n, inner, static_cast<float *>(out));
    else
        hipLaunchKernelGGL(reverse_axis_kernel<double>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<const double *>(src), total, n, inner, static_cast<double *>(out));
    return hip_check(hipGetLastError(), "reverse launch");
}

extern "C" int agmi_triangle(int dtype, const void *src, int64_t batch, int64_t rows, int64_t cols, int64_t k,
                             int lower, void *out, void *stream) {
    if (batch < 0 || rows < 0 || cols < 0) {
        set_error("triangle: negative extent");
        return AGMI_ERR_ARG;
    }
    const int64_t total = batch * rows * cols;
    if (total == 0) return 0;
    const int64_t blocks = plan_copy("triangle", dtype, src, out, total);
    if (blocks < 0) return static_cast<int>(blocks);
    hipStream_t s = as_stream(stream);
    {
        const int64_t V = dtype == AGMI_F32 ? 4 : 2;
        const bool aligned = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
        if (aligned && cols % V == 0) {
            const int64_t vecs = total / V;
            const dim3 grid((unsigned)ceil_div(vecs, kBlock));
            set_kernel_name("triangle_vec_kernel");
            if (dtype == AGMI_F32)
                hipLaunchKernelGGL(triangle_vec_kernel<float>, grid, dim3(kBlock), 0, s, static_cast<const float *>(src), vecs,
                                   rows, cols / V, k, lower, static_cast<float *>(out));
            else
                hipLaunchKernelGGL(triangle_vec_kernel<double>, grid, dim3(kBlock), 0, s, static_cast<const double *>(src), vecs,
                                   rows, cols / V, k, lower, static_cast<double *>(out));
            return hip_check(hipGetLastError(), "triangle launch");
        }
    }
    set_kernel_name("triangle_kernel");
    if (dtype == AGMI_F32)
        hipLaunchKernelGGL(triangle_kernel<float>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<const float *>(src), total, rows, cols, k, lower, static_cast<float *>(out));
    else
        hipLaunchKernelGGL(triangle_kernel<double>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<const double *>(src), total, rows, cols, k, lower, static_cast<double *>(out));
    return hip_check(hipGetLastError(), "triangle launch");
}

extern "C" int agmi_sort_rows(int dtype, const void *src, int64_t rows, int64_t n, void *sorted, int64_t *order,
                              int64_t *rank, void *stream) {
    if (rows < 0 || n < 0) {
        set_error("sort_rows: negative extent");
        return AGMI_ERR_ARG;
    }
    if (rows == 0 || n == 0) return 0;
    if (!src || (!sorted && !order && !rank)) {
        set_error("sort_rows: null source, or no result asked for");
        return AGMI_ERR_ARG;
    }
    if (dtype != AGMI_F32 && dtype != AGMI_F64) {
        set_error("sort_rows: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    if (n > kMaxSortLength || rows > 65535) {
        set_error("sort_rows: %lld rows of %lld elements; at most 65535 rows of %lld are supported", (long long)rows,
                  (long long)n, (long long)kMaxSortLength);
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    const int64_t tiles = ceil_div(n, kBlock);
    if (rank && tiles >= 8) {
        // long rows: the count is split over slices of the row; rank[] is both a result and the accumulator
        const int64_t slices = std::min<int64_t>(32, tiles);
        const int64_t tiles_per_slice = ceil_div(tiles, slices);
        const int64_t total = rows * n;
        const dim3 grid3((unsigned)tiles, (unsigned)rows, (unsigned)ceil_div(tiles, tiles_per_slice));
        set_kernel_name("rank_count_slices+place_by_rank");
        hipLaunchKernelGGL(zero_ranks, dim3((unsigned)ceil_div(total, kBlock)), dim3(kBlock), 0, s, rank, total);
        if (dtype == AGMI_F32) {
            hipLaunchKernelGGL(rank_count_slices<float>, grid3, dim3(kBlock), 0, s, static_cast<const float *>(src), n,
                               tiles_per_slice, rank);
            if (sorted || order)
                hipLaunchKernelGGL(place_by_rank<float>, dim3((unsigned)ceil_div(total, kBlock)), dim3(kBlock), 0, s,
                                   static_cast<const float *>(src), n, total, rank, static_cast<float *>(sorted), order);
        } else {
            hipLaunchKernelGGL(rank_count_slices<double>, grid3, dim3(kBlock), 0, s, static_cast<const double *>(src), n,
                               tiles_per_slice, rank);
            if (sorted || order)
                hipLaunchKernelGGL(place_by_rank<double>, dim3((unsigned)ceil_div(total, kBlock)), dim3(kBlock), 0, s,
                                   static_cast<const double *>(src), n, total, rank, static_cast<double *>(sorted), order);
        }
        return hip_check(hipGetLastError(), "sort_rows launch");
    }
    const dim3 grid((unsigned)tiles, (unsigned)rows);
    set_kernel_name("rank_sort_rows");
    if (dtype == AGMI_F32)
        hipLaunchKernelGGL(rank_sort_rows<float>, grid, dim3(kBlock), 0, s, static_cast<const float *>(src), n,
                           static_cast<float *>(sorted), order, rank);
    else
        hipLaunchKernelGGL(rank_sort_rows<double>, grid, dim3(kBlock), 0, s, static_cast<const double *>(src), n,
                           static_cast<double *>(sorted), order, rank);
    return hip_check(hipGetLastError(), "sort_rows launch");
}
