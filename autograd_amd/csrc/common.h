// Host-side helpers shared by the kernel files of libagmi.so: error reporting, dtype
// dispatch and the axis-merging planner that turns an N-d strided index space into the
// smallest equivalent one.  gfx950 only; no other target is considered anywhere.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "agmi.h"

namespace agmi {

void set_error(const char *fmt, ...);
// name of the kernel family the last successful entry point launched (for profilers' labels)
void set_kernel_name(const char *fmt, ...);
// around the first kernel of an entry point that launches several (see agmi_probe_arm): no-ops unless armed
void probe_begin(hipStream_t s);
void probe_end(hipStream_t s);
int hip_check(hipError_t e, const char *what);

constexpr int kBlock = 256;        // 4 wavefronts of 64 lanes
constexpr int kMaxMerged = 6;      // rank the strided kernels index with div/mod
constexpr int kMaxPhysIn = AGMI_MAX_INPUTS + AGMI_MAX_AUX;  // an op's own inputs + auxiliary operands of pending maps
constexpr int kMaxOperands = kMaxPhysIn + AGMI_MAX_OUTPUTS;

inline size_t dtype_size(int dtype) {
    switch (dtype) {
        case AGMI_F32: return 4;
        case AGMI_F64: return 8;
        case AGMI_BOOL: return 1;
        case AGMI_I64: return 8;
        case AGMI_I32: return 4;
        default: return 0;
    }
}

// An index space after dropping size-1 axes and fusing neighbours that every operand walks
// contiguously (stride[d] == stride[d+1] * shape[d+1], which also holds for two broadcast
// axes).  `group[d]`, when given, forbids fusing axes of different groups (kept vs reduced).
struct Merged {
    int ndim;
    int64_t n;  // number of points
    int64_t shape[AGMI_MAX_DIMS];
    uint8_t group[AGMI_MAX_DIMS];
    int64_t stride[kMaxOperands][AGMI_MAX_DIMS];
};

// Returns false (and sets the error) on rank/shape errors.  `strides[k]` may be nullptr for a
// by-value scalar slot (all zeros are stored).
bool merge_axes(int ndim, const int64_t *shape, const uint8_t *group, int n_operands,
                const int64_t *const *strides, Merged *out);

// true when some extent is 0 (valid rank and shape pointer assumed checked elsewhere)
inline bool index_space_is_empty(int ndim, const int64_t *shape) {
    if (ndim <= 0 || ndim > AGMI_MAX_DIMS || shape == nullptr) return false;
    for (int d = 0; d < ndim; ++d)
        if (shape[d] == 0) return true;
    return false;
}

// Copy input k's pending map into the kernel parameters; auxiliary slots must lie in [arity, n_in).
template <class P>
inline bool read_affine(const agmi_array &a, int arity, int n_in, int k, P *p) {
    if (a.affine & AGMI_AFFINE_SCALE) {
        p->scale_mask |= 1u << k;
        p->scale[k] = a.scale;
    }
    if (a.affine & AGMI_AFFINE_SHIFT) {
        p->shift_mask |= 1u << k;
        p->shift[k] = a.shift;
    }
    if (a.affine & AGMI_AFFINE_SCALE_AUX) {
        if (a.scale_slot < arity || a.scale_slot >= n_in) {
            set_error("input %d: scale_slot %d is not an auxiliary input", k, a.scale_slot);
            return false;
        }
        p->scale_aux[k] = static_cast<signed char>(a.scale_slot);
    }
    if (a.affine & AGMI_AFFINE_SHIFT_AUX) {
        if (a.shift_slot < arity || a.shift_slot >= n_in) {
            set_error("input %d: shift_slot %d is not an auxiliary input", k, a.shift_slot);
            return false;
        }
        p->shift_aux[k] = static_cast<signed char>(a.shift_slot);
    }
    return true;
}

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace agmi
