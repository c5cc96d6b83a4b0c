// Error reporting, the axis-merging planner, fill, and the library version.
#include "common.h"

#include <cstring>

namespace agmi {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

static thread_local char g_kernel[128] = "";

void set_kernel_name(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_kernel, sizeof(g_kernel), fmt, ap);
    va_end(ap);
}

int hip_check(hipError_t e, const char *what) {
    if (e == hipSuccess) return 0;
    set_error("%s: %s", what, hipGetErrorString(e));
    return static_cast<int>(e);
}

bool merge_axes(int ndim, const int64_t *shape, const uint8_t *group, int n_operands,
                const int64_t *const *strides, Merged *out) {
    if (ndim < 0 || ndim > AGMI_MAX_DIMS) {
        set_error("rank %d outside [0, %d]", ndim, AGMI_MAX_DIMS);
        return false;
    }
    if (ndim > 0 && shape == nullptr) {
        set_error("shape is null");
        return false;
    }
    if (n_operands > kMaxOperands) {
        set_error("too many operands");
        return false;
    }
    Merged &m = *out;
    m.ndim = 0;
    m.n = 1;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] < 0) {
            set_error("negative extent %lld on axis %d", (long long)shape[d], d);
            return false;
        }
        m.n *= shape[d];
    }
    if (m.n == 0) return true;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] == 1) continue;  // contributes nothing to any offset
        const uint8_t g = group ? group[d] : 0;
        bool fused = false;
        if (m.ndim > 0 && m.group[m.ndim - 1] == g) {
            const int p = m.ndim - 1;
            fused = true;
            for (int k = 0; k < n_operands && fused; ++k) {
                const int64_t inner = strides[k] ? strides[k][d] : 0;
                if (m.stride[k][p] != inner * shape[d]) fused = false;
            }
            if (fused) {
                m.shape[p] *= shape[d];
                for (int k = 0; k < n_operands; ++k) m.stride[k][p] = strides[k] ? strides[k][d] : 0;
            }
        }
        if (!fused) {
            const int p = m.ndim++;
            m.shape[p] = shape[d];
            m.group[p] = g;
            for (int k = 0; k < n_operands; ++k) m.stride[k][p] = strides[k] ? strides[k][d] : 0;
        }
    }
    if (m.ndim == 0) {  // a single point
        m.ndim = 1;
        m.shape[0] = 1;
        m.group[0] = group && ndim > 0 ? group[0] : 0;
        if (group) {  // a one-point reduction is still a reduction if any axis was reduced
            m.group[0] = 0;
            for (int d = 0; d < ndim; ++d) m.group[0] |= group[d];
        }
        for (int k = 0; k < n_operands; ++k) m.stride[k][0] = 0;
    }
    return true;
}

// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void fill_kernel(T *__restrict__ p, int64_t n, T value) {
    constexpr int V = 16 / sizeof(T);
    typedef T vec_t __attribute__((ext_vector_type(V), aligned(sizeof(T))));
    const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) * V;
    if (i0 + V <= n) {
        vec_t v;
#pragma unroll
        for (int j = 0; j < V; ++j) v[j] = value;
        *reinterpret_cast<vec_t *>(p + i0) = v;
    } else {
        for (int64_t i = i0; i < n; ++i) p[i] = value;
    }
}

template <typename T>
static int launch_fill(void *ptr, int64_t n, double value, hipStream_t s) {
    constexpr int V = 16 / sizeof(T);
    const int64_t threads = ceil_div(n, V);
    const int64_t blocks = ceil_div(threads, kBlock);
    if (blocks > 0x7fffffffLL) {
        set_error("fill: too many elements");
        return AGMI_ERR_UNSUPPORTED;
    }
    set_kernel_name("fill_kernel");
    hipLaunchKernelGGL(fill_kernel<T>, dim3((unsigned)blocks), dim3(kBlock), 0, s, static_cast<T *>(ptr), n,
                       static_cast<T>(value));
    return hip_check(hipGetLastError(), "fill launch");
}

// ---- event pairs around the first kernel of a multi-kernel entry point (agmi_probe_arm) -------------------------
constexpr int kProbePairs = 4096;
static hipEvent_t g_probe_ev[kProbePairs][2];
static unsigned char g_probe_state[kProbePairs];  // 0: no events yet, 1: created, 2: filled
static long long g_probe_serial[kProbePairs];
static long long g_probe_next = 0;
static int g_probe_armed = -1;

void probe_begin(hipStream_t s) {
    if (g_probe_armed >= 0) (void)hipEventRecord(g_probe_ev[g_probe_armed][0], s);
}

void probe_end(hipStream_t s) {
    if (g_probe_armed >= 0) {
        if (hipEventRecord(g_probe_ev[g_probe_armed][1], s) == hipSuccess) g_probe_state[g_probe_armed] = 2;
        g_probe_armed = -1;
    }
}

}  // namespace agmi

using namespace agmi;

extern "C" int agmi_probe_arm(void) {
    const int slot = static_cast<int>(g_probe_next % kProbePairs);
    if (g_probe_state[slot] == 0) {
        if (int rc = hip_check(hipEventCreate(&g_probe_ev[slot][0]), "hipEventCreate")) return rc > 0 ? -rc : rc;
        if (int rc = hip_check(hipEventCreate(&g_probe_ev[slot][1]), "hipEventCreate")) return rc > 0 ? -rc : rc;
    }
    g_probe_state[slot] = 1;
    g_probe_serial[slot] = g_probe_next;
    g_probe_armed = slot;
    const long long index = g_probe_next++;
    return static_cast<int>(index & 0x7fffffff);
}

extern "C" int agmi_probe_elapsed(int index, float *ms) {
    const int slot = index % kProbePairs;
    if (index < 0 || !ms || g_probe_state[slot] != 2 || (g_probe_serial[slot] & 0x7fffffff) != index) {
        set_error("probe: pair %d was never filled (or has been overwritten)", index);
        return AGMI_ERR_ARG;
    }
    if (int rc = hip_check(hipEventSynchronize(g_probe_ev[slot][1]), "hipEventSynchronize")) return rc;
    return hip_check(hipEventElapsedTime(ms, g_probe_ev[slot][0], g_probe_ev[slot][1]), "hipEventElapsedTime");
}

extern "C" const char *agmi_last_error(void) { return g_error; }

extern "C" const char *agmi_last_kernel(void) { return g_kernel; }

extern "C" int agmi_version(void) { return 100; }

extern "C" int agmi_fill(int dtype, void *ptr, int64_t n, double value, void *stream) {
    if (n < 0 || (n > 0 && ptr == nullptr)) {
        set_error("fill: bad pointer or size");
        return AGMI_ERR_ARG;
    }
    if (n == 0) return 0;
    hipStream_t s = as_stream(stream);
    switch (dtype) {
        case AGMI_F32: return launch_fill<float>(ptr, n, value, s);
        case AGMI_F64: return launch_fill<double>(ptr, n, value, s);
        case AGMI_I64: return launch_fill<int64_t>(ptr, n, value, s);
        case AGMI_I32: return launch_fill<int32_t>(ptr, n, value, s);
        case AGMI_BOOL: return launch_fill<uint8_t>(ptr, n, value != 0.0 ? 1.0 : 0.0, s);
        default: set_error("fill: unknown dtype %d", dtype); return AGMI_ERR_ARG;
    }
}
