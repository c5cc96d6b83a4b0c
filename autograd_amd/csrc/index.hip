// Integer-array indexing along the leading axis: gather (forward of A[idx]) and the ordered
// scatter-add that is its cotangent (numpy.add.at semantics, bit for bit).
//
// Basic slices never come here: they are strided views and their cotangent is a strided
// in-place add through agmi_elementwise.  For an index ARRAY, several positions may name the
// same destination row and NumPy adds them one after another in index order; floating-point
// addition is not associative, so the kernel reproduces exactly that order: the caller
// supplies the stable argsort of the destinations and the run boundaries, one thread owns
// one (destination row, column) pair and walks its run sequentially.  No atomics.
#include "common.h"

namespace agmi {

template <typename T>
__global__ __launch_bounds__(kBlock) void take_rows_kernel(const T *__restrict__ src, int64_t n_rows, int64_t inner,
                                                           const int64_t *__restrict__ index, int64_t n_index,
                                                           T *__restrict__ out) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= n_index * inner) return;
    const int64_t i = e / inner, c = e - i * inner;
    int64_t r = index[i];
    if (r < 0) r += n_rows;
    out[e] = src[r * inner + c];
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
    T acc = dst[r * inner + c];
    for (int64_t k = begin; k < end; ++k) acc = acc + src[order[k] * inner + c];
    dst[r * inner + c] = acc;
}

}  // namespace agmi

using namespace agmi;

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
    if (!dst || !src || !index || !order || !seg_start) {
        set_error("scatter_add_rows: null operand");
        return AGMI_ERR_ARG;
    }
    const int64_t blocks = ceil_div(n, kBlock);
    if (blocks > 0x7fffffffLL) {
        set_error("scatter_add_rows: too many elements");
        return AGMI_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    set_kernel_name("scatter_add_rows_kernel");
    if (dtype == AGMI_F32)
        hipLaunchKernelGGL(scatter_add_rows_kernel<float>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<float *>(dst), n_rows, inner, static_cast<const float *>(src), index, order,
                           seg_start, n_seg);
    else if (dtype == AGMI_F64)
        hipLaunchKernelGGL(scatter_add_rows_kernel<double>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                           static_cast<double *>(dst), n_rows, inner, static_cast<const double *>(src), index, order,
                           seg_start, n_seg);
    else {
        set_error("scatter_add_rows: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    return hip_check(hipGetLastError(), "scatter_add_rows launch");
}
