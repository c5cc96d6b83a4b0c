// The cotangent of a row-wise logsumexp and what consumes it, in one pass over the operand.
//
// For x = mem * scale * scale_vec + shift + shift_vec (a matrix with a pending affine map, e.g.
// A * b[None, :] + c[:, None]) and ans = logsumexp(x, axis=1), the cotangent of x is
//     S[r, k] = g[r] * exp(x[r, k] - ans[r])
// (autograd/scipy/special.py:123-134).  The rules that run next on the tape consume S three ways
// (autograd/numpy/numpy_vjps.py:79-83 with unbroadcast, 883-892):
//     row sums      sum_k S[r, k]                   (cotangent of an offset broadcast along the row)
//     scaled copy   col_factor[k] * S[r, k]         (cotangent of mem when x = mem * col_factor)
//     column sums   sum_r mem[r, k] * S[r, k]       (cotangent of the factor broadcast along the column)
// Launched one by one these are four passes over matrix-sized data (write S, read it three times,
// read mem again for the product).  Here a block walks a band of rows; each thread keeps its
// columns' factors and column accumulators in registers, forms S from mem on the fly, writes the
// scaled copy, and S itself never reaches memory: read mem once, write the scaled copy once.
//
// Row sums: per-thread sum in column order, wave butterfly, the four wave partials added in wave
// order.  Column sums: a thread adds its rows in row order; each block writes one partial row to the
// workspace and a second kernel adds the blocks' partials in a fixed order.  Nothing is atomic, so
// results depend only on the shape.
#include <algorithm>

#include "common.h"
#include "functors.h"

namespace agmi {

constexpr int kLseCotMaxRowsPerBlock = 64;
constexpr int kLseCotMaxIters = 8;

struct LseCotParams {
    int64_t rows, cols;
    const void *x;
    int64_t x_rs;
    double scale, shift;
    const void *scale_vec;  // one factor per column (scale_by_col) or per row, or null
    int64_t scale_rs;
    int scale_by_col;
    const void *shift_vec;
    int64_t shift_rs;
    int shift_by_col;
    const void *ans;
    int64_t ans_rs;
    const void *g;
    int64_t g_rs;
    void *row_sums;
    const void *col_factor;
    void *scaled;
    int64_t scaled_rs;
    void *partials;  // [blocks][cols]
    int rows_per_block;
};

enum { kWantScaled = 1, kWantRowSums = 2, kWantColSums = 4 };

template <typename T, int ITERS, int WANT>
__global__ __launch_bounds__(kBlock) void lse_cotangent_rows(const LseCotParams p) {
    constexpr int V = 16 / sizeof(T);
    typedef T vec_t __attribute__((ext_vector_type(V), aligned(sizeof(T))));
    __shared__ T wave_sums[kLseCotMaxRowsPerBlock][kBlock / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row_begin = static_cast<int64_t>(blockIdx.x) * p.rows_per_block;
    const int64_t row_end = min(p.rows, row_begin + p.rows_per_block);

    int64_t col[ITERS];
    bool ok[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        col[it] = (static_cast<int64_t>(it) * kBlock + tid) * V;  // cols % V == 0: a vector is all in or all out
        ok[it] = col[it] < p.cols;
    }
    // absent steps are neutral elements (x * 1 is exact; x + 0 can only change the sign of a zero,
    // which exp(x - ans) cannot see), so the arithmetic below has no branches
    const T sc = static_cast<T>(p.scale), sh = static_cast<T>(p.shift);
    const bool scale_col = p.scale_vec != nullptr && p.scale_by_col, scale_row = p.scale_vec != nullptr && !p.scale_by_col;
    const bool shift_col = p.shift_vec != nullptr && p.shift_by_col, shift_row = p.shift_vec != nullptr && !p.shift_by_col;
    T sv[ITERS][V], hv[ITERS][V], fv[(WANT & kWantScaled) ? ITERS : 1][V];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
            sv[it][j] = T(1);
            hv[it][j] = T(0);
        }
        if (ok[it]) {
            if (scale_col) {
                const vec_t v = *reinterpret_cast<const vec_t *>(static_cast<const T *>(p.scale_vec) + col[it]);
#pragma unroll
                for (int j = 0; j < V; ++j) sv[it][j] = v[j];
            }
            if (shift_col) {
                const vec_t v = *reinterpret_cast<const vec_t *>(static_cast<const T *>(p.shift_vec) + col[it]);
#pragma unroll
                for (int j = 0; j < V; ++j) hv[it][j] = v[j];
            }
            if (WANT & kWantScaled) {
                const vec_t v = *reinterpret_cast<const vec_t *>(static_cast<const T *>(p.col_factor) + col[it]);
#pragma unroll
                for (int j = 0; j < V; ++j) fv[it][j] = v[j];
            }
        }
    }
    T colacc[(WANT & kWantColSums) ? ITERS : 1][V];
    if (WANT & kWantColSums) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < V; ++j) colacc[it][j] = T(0);
    }

    auto load_row = [&](int64_t r, vec_t (&a)[ITERS]) __attribute__((always_inline)) {
        const T *base = static_cast<const T *>(p.x) + r * p.x_rs;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
            if (ok[it]) a[it] = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(base + col[it]));  // last reader
    };
    auto process_row = [&](int64_t r, const vec_t (&a)[ITERS]) __attribute__((always_inline)) {
        const T sr = scale_row ? static_cast<const T *>(p.scale_vec)[r * p.scale_rs] : T(1);
        const T hr = shift_row ? static_cast<const T *>(p.shift_vec)[r * p.shift_rs] : T(0);
        const T ans_r = static_cast<const T *>(p.ans)[r * p.ans_rs];
        const T g_r = static_cast<const T *>(p.g)[r * p.g_rs];
        T rsum = T(0);
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            if (!ok[it]) continue;
            vec_t o;
#pragma unroll
            for (int j = 0; j < V; ++j) {
                T xv = a[it][j] * sc;
                xv = xv * (scale_col ? sv[it][j] : sr);
                xv = xv + sh;
                xv = xv + (shift_col ? hv[it][j] : hr);
                const T s = g_r * exp_of_nonpositive(xv - ans_r);
                if (WANT & kWantRowSums) rsum += s;
                if (WANT & kWantColSums) colacc[it][j] += a[it][j] * s;
                if (WANT & kWantScaled) o[j] = fv[it][j] * s;
            }
            if (WANT & kWantScaled)
                // a matrix-sized result that no kernel of this pass reads back: a streaming store (measured +4 %)
                __builtin_nontemporal_store(o, reinterpret_cast<vec_t *>(static_cast<T *>(p.scaled) + r * p.scaled_rs + col[it]));
        }
        if (WANT & kWantRowSums) {
#pragma unroll
            for (int m = 32; m > 0; m >>= 1) rsum += __shfl_xor(rsum, m, 64);
            if (lane == 0) wave_sums[r - row_begin][wave] = rsum;
        }
    };

    // the loads of the next two rows are in flight while a row is worked on
    vec_t a0[ITERS], a1[ITERS], a2[ITERS];
    if (row_begin < row_end) load_row(row_begin, a0);
    if (row_begin + 1 < row_end) load_row(row_begin + 1, a1);
    for (int64_t r = row_begin; r < row_end; r += 3) {
        if (r + 2 < row_end) load_row(r + 2, a2);
        process_row(r, a0);
        if (r + 1 < row_end) {
            if (r + 3 < row_end) load_row(r + 3, a0);
            process_row(r + 1, a1);
        }
        if (r + 2 < row_end) {
            if (r + 4 < row_end) load_row(r + 4, a1);
            process_row(r + 2, a2);
        }
    }

    if (WANT & kWantRowSums) {
        __syncthreads();
        const int64_t r = row_begin + tid;
        if (r < row_end) {
            T t = wave_sums[tid][0];
#pragma unroll
            for (int w = 1; w < kBlock / 64; ++w) t += wave_sums[tid][w];
            static_cast<T *>(p.row_sums)[r] = t;
        }
    }
    if (WANT & kWantColSums) {
        T *dst = static_cast<T *>(p.partials) + static_cast<int64_t>(blockIdx.x) * p.cols;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            if (!ok[it]) continue;
            vec_t v;
#pragma unroll
            for (int j = 0; j < V; ++j) v[j] = colacc[it][j];
            *reinterpret_cast<vec_t *>(dst + col[it]) = v;
        }
    }
}

// out[k] = sum over blocks (in block order within each of the 16 walkers, walkers added in order) of partials[b][k]
constexpr int kFinishThreads = 1024;

template <typename T>
__global__ __launch_bounds__(kFinishThreads) void lse_cotangent_col_finish(const T *__restrict__ partials, int n_blocks, int64_t cols,
                                                                   T *__restrict__ out) {
    constexpr int kCols = 64, kWalkers = kFinishThreads / kCols;
    __shared__ T part[kWalkers][kCols];
    const int c = threadIdx.x % kCols, w = threadIdx.x / kCols;
    const int64_t k = static_cast<int64_t>(blockIdx.x) * kCols + c;
    T acc = T(0);
    if (k < cols) {
#pragma unroll 8
        for (int b = w; b < n_blocks; b += kWalkers) acc += partials[static_cast<int64_t>(b) * cols + k];
    }
    part[w][c] = acc;
    __syncthreads();
    if (w == 0 && k < cols) {
        T t = part[0][c];
#pragma unroll
        for (int i = 1; i < kWalkers; ++i) t += part[i][c];
        out[k] = t;
    }
}

template <typename T, int ITERS>
static void launch_rows(int want, const LseCotParams &p, unsigned blocks, hipStream_t s) {
#define AGMI_LSECOT(W) \
    case W: hipLaunchKernelGGL((lse_cotangent_rows<T, ITERS, W>), dim3(blocks), dim3(kBlock), 0, s, p); break;
    switch (want) {
        AGMI_LSECOT(1) AGMI_LSECOT(2) AGMI_LSECOT(3) AGMI_LSECOT(4) AGMI_LSECOT(5) AGMI_LSECOT(6) AGMI_LSECOT(7)
        default: break;
    }
#undef AGMI_LSECOT
}

template <typename T>
static int launch_lse_cotangent(const agmi_lse_cotangent &c, void *workspace, size_t workspace_bytes, hipStream_t s) {
    constexpr int V = 16 / sizeof(T);
    const int64_t max_cols = static_cast<int64_t>(kBlock) * V * kLseCotMaxIters;
    if (c.cols % V != 0 || c.cols > max_cols) {
        set_error("lse_cotangent: %lld columns (must be a multiple of %d and at most %lld)", (long long)c.cols, V, (long long)max_cols);
        return AGMI_ERR_UNSUPPORTED;
    }
    int want = 0;
    if (c.scaled) want |= kWantScaled;
    if (c.row_sums) want |= kWantRowSums;
    if (c.col_sums) want |= kWantColSums;
    if (want == 0) return 0;
    LseCotParams p = {};
    p.rows = c.rows; p.cols = c.cols;
    p.x = c.x; p.x_rs = c.x_row_stride;
    p.scale = (c.affine & AGMI_AFFINE_SCALE) ? c.scale : 1.0;
    p.shift = (c.affine & AGMI_AFFINE_SHIFT) ? c.shift : 0.0;
    if (c.affine & AGMI_AFFINE_SCALE_AUX) {
        if (!c.scale_vec || (c.scale_col_stride != 0 && (c.scale_col_stride != 1 || c.scale_row_stride != 0))) {
            set_error("lse_cotangent: the array factor must vary along rows only or along columns only (unit stride)");
            return AGMI_ERR_UNSUPPORTED;
        }
        p.scale_vec = c.scale_vec; p.scale_rs = c.scale_row_stride; p.scale_by_col = c.scale_col_stride == 1;
    }
    if (c.affine & AGMI_AFFINE_SHIFT_AUX) {
        if (!c.shift_vec || (c.shift_col_stride != 0 && (c.shift_col_stride != 1 || c.shift_row_stride != 0))) {
            set_error("lse_cotangent: the array offset must vary along rows only or along columns only (unit stride)");
            return AGMI_ERR_UNSUPPORTED;
        }
        p.shift_vec = c.shift_vec; p.shift_rs = c.shift_row_stride; p.shift_by_col = c.shift_col_stride == 1;
    }
    p.ans = c.ans; p.ans_rs = c.ans_stride;
    p.g = c.g; p.g_rs = c.g_stride;
    p.row_sums = c.row_sums;
    p.col_factor = c.col_factor; p.scaled = c.scaled; p.scaled_rs = c.scaled_row_stride;
    if ((want & kWantScaled) && (!c.col_factor || c.scaled_row_stride < c.cols)) {
        set_error("lse_cotangent: the scaled copy needs a column factor and a row stride >= cols");
        return AGMI_ERR_ARG;
    }
    // 512 bands (two blocks of four waves per CU, each with two rows of loads in flight) measured best on
    // 8192 x 4096: more bands make the column partials (one row per band) and their summation cost more
    // than the extra waves gain, fewer leave CUs short of loads in flight
    int64_t rpb = std::max<int64_t>(8, ceil_div(c.rows, 512));
    if (want & kWantColSums) {
        if (!workspace) {
            set_error("lse_cotangent: column sums need a workspace");
            return AGMI_ERR_WORKSPACE;
        }
        const int64_t fit = static_cast<int64_t>(workspace_bytes / (sizeof(T) * static_cast<size_t>(c.cols)));
        if (fit < 1) {
            set_error("lse_cotangent: workspace smaller than one row of partial sums");
            return AGMI_ERR_WORKSPACE;
        }
        rpb = std::max(rpb, ceil_div(c.rows, fit));
    }
    if (rpb > kLseCotMaxRowsPerBlock) {
        // more rows than 512 (or the workspace allows) bands of 64: take more blocks, the band length is what LDS holds
        rpb = kLseCotMaxRowsPerBlock;
        if ((want & kWantColSums) &&
            static_cast<size_t>(ceil_div(c.rows, rpb)) * static_cast<size_t>(c.cols) * sizeof(T) > workspace_bytes) {
            set_error("lse_cotangent: workspace too small for %lld bands of partial sums", (long long)ceil_div(c.rows, rpb));
            return AGMI_ERR_WORKSPACE;
        }
    }
    const int64_t blocks = ceil_div(c.rows, rpb);
    if (blocks > 0x7fffffffLL) {
        set_error("lse_cotangent: too many rows");
        return AGMI_ERR_UNSUPPORTED;
    }
    p.rows_per_block = static_cast<int>(rpb);
    p.partials = workspace;
    const int64_t need = ceil_div(c.cols, static_cast<int64_t>(kBlock) * V);
    set_kernel_name("lse_cotangent_rows<%s%s%s>", (want & kWantScaled) ? "scaled," : "", (want & kWantRowSums) ? "rowsum," : "",
                    (want & kWantColSums) ? "colsum" : "");
    if (need <= 1) launch_rows<T, 1>(want, p, static_cast<unsigned>(blocks), s);
    else if (need <= 2) launch_rows<T, 2>(want, p, static_cast<unsigned>(blocks), s);
    else if (need <= 4) launch_rows<T, 4>(want, p, static_cast<unsigned>(blocks), s);
    else launch_rows<T, 8>(want, p, static_cast<unsigned>(blocks), s);
    if (int rc = hip_check(hipGetLastError(), "lse_cotangent launch")) return rc;
    if (want & kWantColSums) {
        hipLaunchKernelGGL(lse_cotangent_col_finish<T>, dim3(static_cast<unsigned>(ceil_div(c.cols, 64))), dim3(kFinishThreads), 0, s,
                           static_cast<const T *>(workspace), static_cast<int>(blocks), c.cols, static_cast<T *>(c.col_sums));
        return hip_check(hipGetLastError(), "lse_cotangent finish launch");
    }
    return 0;
}

}  // namespace agmi

using namespace agmi;

extern "C" int agmi_lse_cotangent_fused(int dtype, const agmi_lse_cotangent *c, void *workspace, size_t workspace_bytes,
                                  void *stream) {
    if (!c) {
        set_error("lse_cotangent: null descriptor");
        return AGMI_ERR_ARG;
    }
    if (c->rows < 0 || c->cols < 0) {
        set_error("lse_cotangent: negative extent");
        return AGMI_ERR_ARG;
    }
    if (c->rows == 0 || c->cols == 0) return 0;  // empty results; a caller that wants zeros for empty rows fills them
    if (!c->x || !c->ans || !c->g) {
        set_error("lse_cotangent: null operand");
        return AGMI_ERR_ARG;
    }
    hipStream_t s = as_stream(stream);
    if (dtype == AGMI_F32) return launch_lse_cotangent<float>(*c, workspace, workspace_bytes, s);
    if (dtype == AGMI_F64) return launch_lse_cotangent<double>(*c, workspace, workspace_bytes, s);
    set_error("lse_cotangent: dtype %d is not a floating type", dtype);
    return AGMI_ERR_ARG;
}
