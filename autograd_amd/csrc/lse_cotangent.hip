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
// read mem again for the product).  Here a block owns a tile of 16 (or a multiple of 16) rows by
// 256 vectors of columns; each thread keeps its columns' factors and column accumulators in
// registers, walks the tile's rows with four rows of loads in flight, forms S from mem on the fly and
// writes the scaled copy; S itself never reaches memory: read mem once, write the scaled copy once.
// Tiles this small give thousands of blocks (2048 for 8192 x 4096 float32), which streams measurably
// better than a few hundred long-lived ones, at the price of partial results in both directions:
//
// Row sums: per-thread sum over its vector, wave butterfly, the block's wave partials added in wave
// order; with more than one tile across, the tiles' partials go to the workspace and are added in tile
// order by the finishing kernel.  Column sums: a thread adds its rows in row order; each band of rows
// writes one partial row to the workspace and the finishing kernel adds the bands' partials in a
// fixed order.  Nothing is atomic, so results depend only on the shape.
#include <algorithm>

#include "common.h"
#include "functors.h"

namespace agmi {

constexpr int kLseCotRowGroup = 16;         // rows of a tile are taken in groups of this many
constexpr int kLseCotMaxRowsPerBlock = 64;  // wave partials of a tile's rows are held in LDS
constexpr int kLseCotDepth = 4;             // rows of loads in flight per thread

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
    void *row_sums;      // final row sums (one tile across) ...
    void *row_partials;  // ... or [tiles across][rows] partial sums
    const void *col_factor;
    void *scaled;
    int64_t scaled_rs;
    void *partials;  // [bands][cols]
    int rows_per_block;
};

enum { kWantScaled = 1, kWantRowSums = 2, kWantColSums = 4 };

// the value lane `q` holds, as a wave-uniform scalar (q is the same for the whole wave)
__device__ __forceinline__ float from_lane(float v, int q) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), q));
}
__device__ __forceinline__ double from_lane(double v, int q) {
    const unsigned long long bits = __builtin_bit_cast(unsigned long long, v);
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(bits), q));
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(bits >> 32), q));
    return __builtin_bit_cast(double, (static_cast<unsigned long long>(hi) << 32) | lo);
}

// Register use is left to the compiler on purpose: with the group's code in a straight line it hoists all 16 rows'
// loads (192 VGPRs, two waves per SIMD) and that is the fastest form measured: bounding it to 3 / 4 / 6 / 8 waves per
// SIMD took 43.6 -> 58 / 91 / 178 / 221 us on 8192 x 4096.
template <typename T, int WANT>
__global__ __launch_bounds__(kBlock) void lse_cotangent_tile(const LseCotParams p) {
    constexpr int V = 16 / sizeof(T);
    constexpr int D = kLseCotDepth;
    typedef T vec_t __attribute__((ext_vector_type(V), aligned(sizeof(T))));
    __shared__ T wave_sums[kLseCotMaxRowsPerBlock][kBlock / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t own_col = (static_cast<int64_t>(blockIdx.x) * kBlock + tid) * V;  // cols % V == 0: a vector is all in or all out
    const bool ok = own_col < p.cols;
    // lanes past the last column work on column 0 and throw the result away: a load under a per-lane condition
    // makes the compiler wait for it where the branches join, which would serialise the rows in flight
    const int64_t col = ok ? own_col : 0;
    const int64_t row_begin = static_cast<int64_t>(blockIdx.y) * p.rows_per_block;
    const int64_t row_end = min(p.rows, row_begin + p.rows_per_block);

    // absent steps are neutral elements (x * 1 is exact; x + 0 can only change the sign of a zero,
    // which exp(x - ans) cannot see), so the arithmetic below has no branches
    const T sc = static_cast<T>(p.scale), sh = static_cast<T>(p.shift);
    const bool scale_col = p.scale_vec != nullptr && p.scale_by_col, scale_row = p.scale_vec != nullptr && !p.scale_by_col;
    const bool shift_col = p.shift_vec != nullptr && p.shift_by_col, shift_row = p.shift_vec != nullptr && !p.shift_by_col;
    vec_t sv, hv, fv, colacc;
#pragma unroll
    for (int j = 0; j < V; ++j) {
        sv[j] = T(1);
        hv[j] = T(0);
        fv[j] = T(0);
        colacc[j] = T(0);
    }
    if (scale_col) sv = *reinterpret_cast<const vec_t *>(static_cast<const T *>(p.scale_vec) + col);
    if (shift_col) hv = *reinterpret_cast<const vec_t *>(static_cast<const T *>(p.shift_vec) + col);
    if (WANT & kWantScaled) fv = *reinterpret_cast<const vec_t *>(static_cast<const T *>(p.col_factor) + col);

    const auto load_row = [&](int64_t r, vec_t &a) __attribute__((always_inline)) {
        // last reader of this operand: a streaming load (the row test is the same for the whole block)
        if (r < row_end) a = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(static_cast<const T *>(p.x) + r * p.x_rs + col));
    };
    // The per-row operands (ans, g, a factor / offset that varies along rows) of a group of 16 rows: lane l of every
    // wave fetches those of row l with ONE load each, ahead of the group's matrix loads, and the rows read them
    // back as wave-uniform scalars.  Fetched row by row instead they are vector loads issued after the prefetched
    // matrix rows, and waiting for one of them waits for every load before it: no rows in flight any more.
    T ans_v, g_v, sr_v = T(1), hr_v = T(0);
    const auto load_row_operands = [&](int64_t r) __attribute__((always_inline)) {
        const int64_t rr = min(r + (lane & (kLseCotRowGroup - 1)), row_end - 1);
        ans_v = static_cast<const T *>(p.ans)[rr * p.ans_rs];
        g_v = static_cast<const T *>(p.g)[rr * p.g_rs];
        if (scale_row) sr_v = static_cast<const T *>(p.scale_vec)[rr * p.scale_rs];
        if (shift_row) hr_v = static_cast<const T *>(p.shift_vec)[rr * p.shift_rs];
    };
    // process_row returns this lane's share of the row sum (zero for lanes past the last column)
    const auto process_row = [&](int64_t r, int q, const vec_t &a) __attribute__((always_inline)) -> T {
        const T sr = from_lane(sr_v, q), hr = from_lane(hr_v, q), ans_r = from_lane(ans_v, q), g_r = from_lane(g_v, q);
        T rsum = T(0);
        vec_t o;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            T xv = a[j] * sc;
            xv = xv * (scale_col ? sv[j] : sr);
            xv = xv + sh;
            xv = xv + (shift_col ? hv[j] : hr);
            const T s = g_r * exp_of_nonpositive(xv - ans_r);
            if (WANT & kWantRowSums) rsum += s;
            if (WANT & kWantColSums) colacc[j] += a[j] * s;
            if (WANT & kWantScaled) o[j] = fv[j] * s;
        }
        if ((WANT & kWantScaled) && ok)
            // a matrix-sized result that no kernel of this pass reads back: a streaming store
            __builtin_nontemporal_store(o, reinterpret_cast<vec_t *>(static_cast<T *>(p.scaled) + r * p.scaled_rs + col));
        return ok ? rsum : T(0);
    };
    // one row's sum over the wave, lane by lane (the short last group of the matrix)
    const auto reduce_row = [&](int64_t r, T rsum) __attribute__((always_inline)) {
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) rsum += __shfl_xor(rsum, m, 64);
        if (lane == 0) wave_sums[r - row_begin][wave] = rsum;
    };
    // The sums of a whole group of 16 rows over the wave, together: at each of the first four exchanges a lane
    // hands over the half of its rows that its partner keeps, so 8 + 4 + 2 + 1 values cross instead of 16 each
    // time, and two plain exchanges finish the one row a lane is left with: 17 cross-lane moves for 16 rows, not
    // 96.  Lane bits 5..2 say which row a lane ends up with; the order of the additions is fixed.
    const auto reduce_group = [&](int64_t r0, T (&part)[kLseCotRowGroup]) __attribute__((always_inline)) {
        T v8[8], v4[4], v2[2];
        const bool b5 = (lane & 32) != 0, b4 = (lane & 16) != 0, b3 = (lane & 8) != 0, b2 = (lane & 4) != 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) v8[i] = (b5 ? part[i + 8] : part[i]) + __shfl_xor(b5 ? part[i] : part[i + 8], 32, 64);
#pragma unroll
        for (int i = 0; i < 4; ++i) v4[i] = (b4 ? v8[i + 4] : v8[i]) + __shfl_xor(b4 ? v8[i] : v8[i + 4], 16, 64);
#pragma unroll
        for (int i = 0; i < 2; ++i) v2[i] = (b3 ? v4[i + 2] : v4[i]) + __shfl_xor(b3 ? v4[i] : v4[i + 2], 8, 64);
        T v = (b2 ? v2[1] : v2[0]) + __shfl_xor(b2 ? v2[0] : v2[1], 4, 64);
        v += __shfl_xor(v, 2, 64);
        v += __shfl_xor(v, 1, 64);
        if ((lane & 3) == 0) wave_sums[(r0 - row_begin) + (lane >> 2)][wave] = v;
    };

    // D rows of loads are in flight while a row is worked on.  Whole groups of 16 rows run as straight-line code (no
    // row tests between the loads and the arithmetic, so the compiler is free to order them); the pipeline is refilled
    // at each group's start, which only tiles taller than one group notice.
    vec_t a[D];
    int64_t r = row_begin;
    for (; r + kLseCotRowGroup <= row_end; r += kLseCotRowGroup) {
        load_row_operands(r);
#pragma unroll
        for (int d = 0; d < D; ++d)
            a[d] = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(static_cast<const T *>(p.x) + (r + d) * p.x_rs + col));
        T part[kLseCotRowGroup];
#pragma unroll
        for (int q = 0; q < kLseCotRowGroup; ++q) {
            const vec_t cur = a[q % D];
            if (q + D < kLseCotRowGroup)
                a[q % D] = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(static_cast<const T *>(p.x) + (r + q + D) * p.x_rs + col));
            part[q] = process_row(r + q, q, cur);
        }
        if (WANT & kWantRowSums) reduce_group(r, part);
    }
    if (r < row_end) {  // the last rows of the matrix (fewer than 16)
        load_row_operands(r);
        const int64_t group = r;
#pragma unroll
        for (int d = 0; d < D; ++d) load_row(r + d, a[d]);
        for (; r < row_end; r += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                if (r + d < row_end) {  // the same for the whole block
                    const vec_t cur = a[d];
                    load_row(r + d + D, a[d]);
                    const T part = process_row(r + d, static_cast<int>(r + d - group), cur);
                    if (WANT & kWantRowSums) reduce_row(r + d, part);
                }
            }
        }
    }

    if (WANT & kWantRowSums) {
        __syncthreads();
        const int64_t r = row_begin + tid;
        if (r < row_end) {
            T t = wave_sums[tid][0];
#pragma unroll
            for (int w = 1; w < kBlock / 64; ++w) t += wave_sums[tid][w];
            if (gridDim.x == 1) static_cast<T *>(p.row_sums)[r] = t;
            else static_cast<T *>(p.row_partials)[static_cast<int64_t>(blockIdx.x) * p.rows + r] = t;
        }
    }
    if ((WANT & kWantColSums) && ok)
        *reinterpret_cast<vec_t *>(static_cast<T *>(p.partials) + static_cast<int64_t>(blockIdx.y) * p.cols + col) = colacc;
}

// Column blocks (the first `col_blocks`): out[k] = sum over bands of partials[band][k], in band order within each of 16
// walkers, the walkers added in order.  Row blocks (the rest): out[r] = sum over tiles of row_partials[tile][r], in
// tile order.
constexpr int kFinishThreads = 1024;

template <typename T>
__global__ __launch_bounds__(kFinishThreads) void lse_cotangent_finish(const T *__restrict__ partials, int n_bands, int64_t cols,
                                                               T *__restrict__ col_out, int col_blocks,
                                                               const T *__restrict__ row_partials, int n_tiles, int64_t rows,
                                                               T *__restrict__ row_out) {
    constexpr int kCols = 64, kWalkers = kFinishThreads / kCols;
    __shared__ T part[kWalkers][kCols];
    if (static_cast<int>(blockIdx.x) >= col_blocks) {  // the same for the whole block
        const int64_t r = static_cast<int64_t>(blockIdx.x - col_blocks) * kFinishThreads + threadIdx.x;
        if (r < rows) {
            T t = row_partials[r];
            for (int k = 1; k < n_tiles; ++k) t += row_partials[static_cast<int64_t>(k) * rows + r];
            row_out[r] = t;
        }
        return;
    }
    const int c = threadIdx.x % kCols, w = threadIdx.x / kCols;
    const int64_t k = static_cast<int64_t>(blockIdx.x) * kCols + c;
    T acc = T(0);
    if (k < cols) {
#pragma unroll 8
        for (int b = w; b < n_bands; b += kWalkers) acc += partials[static_cast<int64_t>(b) * cols + k];
    }
    part[w][c] = acc;
    __syncthreads();
    if (w == 0 && k < cols) {
        T t = part[0][c];
#pragma unroll
        for (int i = 1; i < kWalkers; ++i) t += part[i][c];
        col_out[k] = t;
    }
}

template <typename T>
static void launch_tiles(int want, const LseCotParams &p, dim3 grid, hipStream_t s) {
#define AGMI_LSECOT(W) \
    case W: hipLaunchKernelGGL((lse_cotangent_tile<T, W>), grid, dim3(kBlock), 0, s, p); break;
    switch (want) {
        AGMI_LSECOT(1) AGMI_LSECOT(2) AGMI_LSECOT(3) AGMI_LSECOT(4) AGMI_LSECOT(5) AGMI_LSECOT(6) AGMI_LSECOT(7)
        default: break;
    }
#undef AGMI_LSECOT
}

template <typename T>
static int launch_lse_cotangent(const agmi_lse_cotangent &c, void *workspace, size_t workspace_bytes, hipStream_t s) {
    constexpr int V = 16 / sizeof(T);
    if (c.cols % V != 0) {
        set_error("lse_cotangent: %lld columns (must be a multiple of %d)", (long long)c.cols, V);
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
    // (the stride of an axis of extent 1 is never used: any value is as good as 0)
    const int64_t scale_row_stride = c.rows == 1 ? 0 : c.scale_row_stride, shift_row_stride = c.rows == 1 ? 0 : c.shift_row_stride;
    if (c.affine & AGMI_AFFINE_SCALE_AUX) {
        if (!c.scale_vec || (c.scale_col_stride != 0 && (c.scale_col_stride != 1 || scale_row_stride != 0))) {
            set_error("lse_cotangent: the array factor must vary along rows only or along columns only (unit stride)");
            return AGMI_ERR_UNSUPPORTED;
        }
        p.scale_vec = c.scale_vec; p.scale_rs = scale_row_stride; p.scale_by_col = c.scale_col_stride == 1;
    }
    if (c.affine & AGMI_AFFINE_SHIFT_AUX) {
        if (!c.shift_vec || (c.shift_col_stride != 0 && (c.shift_col_stride != 1 || shift_row_stride != 0))) {
            set_error("lse_cotangent: the array offset must vary along rows only or along columns only (unit stride)");
            return AGMI_ERR_UNSUPPORTED;
        }
        p.shift_vec = c.shift_vec; p.shift_rs = shift_row_stride; p.shift_by_col = c.shift_col_stride == 1;
    }
    p.ans = c.ans; p.ans_rs = c.ans_stride;
    p.g = c.g; p.g_rs = c.g_stride;
    p.row_sums = c.row_sums;
    p.col_factor = c.col_factor; p.scaled = c.scaled; p.scaled_rs = c.scaled_row_stride;
    if ((want & kWantScaled) && (!c.col_factor || c.scaled_row_stride < c.cols)) {
        set_error("lse_cotangent: the scaled copy needs a column factor and a row stride >= cols");
        return AGMI_ERR_ARG;
    }
    const int64_t tiles_across = ceil_div(c.cols, static_cast<int64_t>(kBlock) * V);
    const bool row_partials = (want & kWantRowSums) && tiles_across > 1;
    // Tiles of 16 rows measured best on 8192 x 4096 (2048 blocks: 74 us for the forward reduction, this pass and its
    // finish against 79 us with 512 long bands, 86 us with tiles of 32 rows); taller tiles only when the
    // partial column sums (one row per band of rows) would not fit the workspace.
    int64_t rpb = kLseCotRowGroup;
    const auto staged = [&](int64_t rows_per_band, size_t *col_bytes) {
        *col_bytes = (want & kWantColSums) ? static_cast<size_t>(ceil_div(c.rows, rows_per_band)) * static_cast<size_t>(c.cols) * sizeof(T) : 0;
        *col_bytes = (*col_bytes + 255) / 256 * 256;
        return *col_bytes + (row_partials ? static_cast<size_t>(tiles_across) * static_cast<size_t>(c.rows) * sizeof(T) : 0);
    };
    size_t col_bytes = 0;
    size_t need = staged(rpb, &col_bytes);
    while ((need > workspace_bytes || ceil_div(c.rows, rpb) > 65535) && rpb < kLseCotMaxRowsPerBlock) {  // (65535: the grid's y extent)
        rpb += kLseCotRowGroup;
        need = staged(rpb, &col_bytes);
    }
    if (need > 0 && !workspace) {
        set_error("lse_cotangent: partial sums need a workspace (%zu bytes)", need);
        return AGMI_ERR_WORKSPACE;
    }
    if (need > workspace_bytes) {
        set_error("lse_cotangent: workspace of %zu bytes is too small for the partial sums (%zu bytes)", workspace_bytes, need);
        return AGMI_ERR_UNSUPPORTED;
    }
    const int64_t bands = ceil_div(c.rows, rpb);
    if (bands > 65535 || tiles_across > 0x7fffffffLL) {
        set_error("lse_cotangent: too many rows or columns for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    p.rows_per_block = static_cast<int>(rpb);
    p.partials = workspace;
    p.row_partials = row_partials ? static_cast<unsigned char *>(workspace) + col_bytes : nullptr;
    set_kernel_name("lse_cotangent_tile<%s%s%s>", (want & kWantScaled) ? "scaled," : "", (want & kWantRowSums) ? "rowsum," : "",
                    (want & kWantColSums) ? "colsum" : "");
    probe_begin(s);
    launch_tiles<T>(want, p, dim3(static_cast<unsigned>(tiles_across), static_cast<unsigned>(bands)), s);
    probe_end(s);
    if (int rc = hip_check(hipGetLastError(), "lse_cotangent launch")) return rc;
    const int col_blocks = (want & kWantColSums) ? static_cast<int>(ceil_div(c.cols, 64)) : 0;
    const int row_blocks = row_partials ? static_cast<int>(ceil_div(c.rows, kFinishThreads)) : 0;
    if (col_blocks + row_blocks > 0) {
        hipLaunchKernelGGL(lse_cotangent_finish<T>, dim3(static_cast<unsigned>(col_blocks + row_blocks)), dim3(kFinishThreads), 0, s,
                           static_cast<const T *>(workspace), static_cast<int>(bands), c.cols, static_cast<T *>(c.col_sums), col_blocks,
                           static_cast<const T *>(p.row_partials), static_cast<int>(tiles_across), c.rows, static_cast<T *>(c.row_sums));
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
