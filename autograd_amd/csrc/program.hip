// Elementwise programs: a chain of derivative rules evaluated in ONE pass over memory.
//
// The rules of a backward pass are mostly elementwise (numpy_vjps.py:76-191: y*g, g/y, -g*x/y**2,
// ans*g, the adds of core.py:185-205).  Launched one by one, every rule reads its operands from
// HBM and writes its result back; evaluated together, only the leaves of the expression are read
// and only its roots are written.  The host hands over the expression as a short straight-line
// program over a small register file; this kernel interprets it:
//
//   * every lane owns U 16-byte vectors of the index space per tile and keeps the program's
//     registers for them in VGPRs (NREG registers x U vectors), so an instruction costs no memory
//     traffic at all;
//   * the program sits in kernel arguments; instruction words are fetched with scalar loads one
//     instruction ahead, decoded on the scalar unit, and dispatched by a wave-uniform switch over
//     the same functors the one-rule kernels use (functors.h), each operation rounded on its own
//     (-ffp-contract=off): results are bit for bit those of the separate passes;
//   * a wave walks over tiles with a fixed stride and issues the loads of its next tile before it
//     interprets the current one, so HBM latency hides behind the interpretation.
//
// Index space: (rows, cols) after axis merging, every leaf with column stride 1 or 0 (flat arrays
// are one row).  Registers 0 .. n_leaf-1 hold the leaves when the program starts, registers
// NREG-1, NREG-2, ... the immediates.  Beside the one-rule functors an instruction may hold two
// rules (a * b + c and its kin: what an interpreted instruction costs is operand moves and dispatch,
// not arithmetic), select by index range (the scattered cotangent of a slice), or sum its operand
// over the row (the ROWS variant: programs whose rows fit one wave's tile).
//
// The interpreter runs whatever it is handed, at once.  A program that keeps coming back is
// compiled into a kernel of its own (specialize.hip), which takes the same argument block.
#include <algorithm>
#include <type_traits>

#include "common.h"

#include "functors.h"
#include "program_params.h"

namespace agmi {

template <typename T, int NREG>
struct RegVec {
    typedef T type __attribute__((ext_vector_type(NREG)));
};

// Operations of a few instructions are expanded in place; every other functor is ONE function that the
// interpreter calls element by element, so that the temporaries and constants of the long routines (exp, pow,
// the trigonometric family) live in the callee's registers for the length of a call instead of adding to what
// the kernel holds for its whole run: the register file of the program and the waves a SIMD keeps resident
// depend on that.
constexpr bool is_short_op(int op) {
    switch (op) {
        case AGMI_OP_COPY: case AGMI_OP_NEG: case AGMI_OP_SQUARE: case AGMI_OP_ABS:
        case AGMI_OP_RECIPROCAL: case AGMI_OP_ADD: case AGMI_OP_SUB: case AGMI_OP_MUL: case AGMI_OP_DIV:
        case AGMI_OP_MAXIMUM: case AGMI_OP_MINIMUM: case AGMI_OP_FMAX: case AGMI_OP_FMIN: case AGMI_OP_WHERE:
        case AGMI_OP_DIV_VJP1: case AGMI_OP_RECIPROCAL_VJP: case AGMI_OP_SQUARE_VJP: case AGMI_OP_ABS_VJP:
        case AGMI_OP_LOG1P_VJP: case AGMI_OP_EXPM1_VJP: case AGMI_OP_MUL_ADD: case AGMI_OP_EQUAL_AS_FLOAT:
        case AGMI_OP_CHOOSE_VJP: case AGMI_OP_EXTREMUM_VJP: case AGMI_OP_FLOOR: case AGMI_OP_CEIL:
        case AGMI_OP_RINT: case AGMI_OP_TRUNC:
        case AGMI_OP_MUL_MUL: case AGMI_OP_MUL_SUB: case AGMI_OP_MUL_RSUB: case AGMI_OP_ADD_MUL: case AGMI_OP_SUB_MUL:
            return true;
        default:
            return false;
    }
}

// The operations most chains are made of.  A program that uses nothing else runs on a kernel whose dispatch
// holds only these (a shallower compare tree per instruction, fewer registers, exp / log / sqrt expanded in place).
#define AGMI_FOR_EACH_LIGHT_OP(X)            \
    X(AGMI_OP_COPY, FCopy)                   \
    X(AGMI_OP_NEG, FNeg)                     \
    X(AGMI_OP_EXP, FExp)                     \
    X(AGMI_OP_LOG, FLog)                     \
    X(AGMI_OP_SQRT, FSqrt)                   \
    X(AGMI_OP_SQUARE, FSquare)               \
    X(AGMI_OP_RECIPROCAL, FReciprocal)       \
    X(AGMI_OP_TANH, FTanh)                   \
    X(AGMI_OP_ADD, FAdd)                     \
    X(AGMI_OP_SUB, FSub)                     \
    X(AGMI_OP_MUL, FMul)                     \
    X(AGMI_OP_DIV, FDiv)                     \
    X(AGMI_OP_DIV_VJP1, FDivVjp1)            \
    X(AGMI_OP_TANH_VJP, FTanhVjp)            \
    X(AGMI_OP_MUL_ADD, FMulAdd)              \
    AGMI_FOR_EACH_CHAINED_OP(X)

constexpr bool is_light_op(int op) {
#define AGMI_LIGHT_CASE(OP, FN) case OP:
    switch (op) {
        AGMI_FOR_EACH_LIGHT_OP(AGMI_LIGHT_CASE)
        case AGMI_PROGRAM_STORE:
        case AGMI_PROGRAM_MASK:
            return true;
        default:
            return false;
    }
#undef AGMI_LIGHT_CASE
}

// expanded in place by the light kernel (the full kernel calls them)
constexpr bool is_light_inline_op(int op) {
    return op == AGMI_OP_EXP || op == AGMI_OP_LOG || op == AGMI_OP_SQRT;
}

template <class Fn, typename T>
static __device__ __noinline__ T apply_called(T a, T b, T c, T d) {
    const T xi[4] = {a, b, c, d};
    T oi[1];
    Fn::apply(xi, oi);
    return oi[0];
}

template <class Fn, typename T, bool SHORT>
__device__ __forceinline__ T apply_one(const T (&xi)[4]) {
    if constexpr (SHORT) {
        T oi[1];
        Fn::apply(xi, oi);
        return oi[0];
    } else {
        return apply_called<Fn, T>(xi[0], Fn::NIN > 1 ? xi[1] : T(0), Fn::NIN > 2 ? xi[2] : T(0), Fn::NIN > 3 ? xi[3] : T(0));
    }
}

// op | dst << 8 | a << 12 | b << 16 | c << 20 | d << 24
__device__ __forceinline__ int field(uint32_t w, int shift, int mask) { return static_cast<int>(w >> shift) & mask; }

// ROWS: the variant that knows AGMI_PROGRAM_ROWSUM (a row per tile; the row's values cross the wave through LDS)
template <typename T, int NREG, int U, bool LIGHT, bool ROWS>
__global__ __launch_bounds__(kBlock) void ew_program(const ProgParams p) {
    constexpr int VL = 16 / sizeof(T);
    constexpr int V = VL * U;
    constexpr int TW = 64 * V;  // columns per tile (one wave)
    __shared__ __align__(16) T row_values[ROWS ? kBlock / 64 : 1][ROWS ? TW : 1];
    typedef T vec_t __attribute__((ext_vector_type(VL), aligned(sizeof(T))));
    using reg_t = typename RegVec<T, NREG>::type;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6));
    uint32_t t = wave;
    if (t >= p.n_tiles) return;
    const uint32_t tpr = p.tiles_per_row;
    uint32_t row = t / tpr;
    uint32_t chunk = t - row * tpr;
    const int64_t cols = p.cols;
    const int nl = p.n_leaf;

    reg_t r[V];
#pragma unroll
    for (int j = 0; j < V; ++j) r[j] = T(0);
    {
        const int ni = p.n_imm;
#pragma unroll
        for (int k = 0; k < kProgMaxImm; ++k) {
            if (k < ni) {
                const T s = static_cast<T>(p.imm[k]);
#pragma unroll
                for (int j = 0; j < V; ++j) r[j][NREG - 1 - k] = s;
            }
        }
    }

    const int n_instr = p.n_instr;
    for (;;) {
        // the tile's leaves go straight into the register file
        const uint32_t cur_row = row, cur_chunk = chunk;
        const int64_t c0 = static_cast<int64_t>(cur_chunk) * TW + lane * VL;
        const int64_t tile_begin = static_cast<int64_t>(cur_chunk) * TW;
        const bool interior = tile_begin + TW <= cols;
        const bool readable = interior && tile_begin >= p.safe_lo && tile_begin + TW <= p.safe_hi;
        {
            vec_t L[kProgMaxLeaf][U];
#pragma unroll
            for (int k = 0; k < kProgMaxLeaf; ++k) {
                if (k < nl) {
                    const T *base = static_cast<const T *>(p.leaf[k]) + static_cast<int64_t>(cur_row) * p.leaf_rs[k];
                    if (p.leaf_cs[k] == 0) {
                        const T s = *base;
#pragma unroll
                        for (int u = 0; u < U; ++u)
#pragma unroll
                            for (int j = 0; j < VL; ++j) L[k][u][j] = s;
                    } else if (readable) {
#pragma unroll
                        for (int u = 0; u < U; ++u)
                            L[k][u] = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(base + c0 + u * (64 * VL)));
                    } else {
#pragma unroll
                        for (int u = 0; u < U; ++u)
#pragma unroll
                            for (int j = 0; j < VL; ++j) {
                                const int64_t c = c0 + u * (64 * VL) + j;
                                L[k][u][j] = (c < cols && c >= p.leaf_lo[k] && c < p.leaf_hi[k]) ? base[c] : T(1);
                            }
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < kProgMaxLeaf; ++k) {
                if (k < nl) {
#pragma unroll
                    for (int u = 0; u < U; ++u)
#pragma unroll
                        for (int j = 0; j < VL; ++j) r[u * VL + j][k] = L[k][u][j];
                }
            }
        }
        // The wave's next tile: one element per lane and vector is read now and thrown away, which brings the
        // tile's cache lines into the L2 while the program runs on the current tile; the loads above then find
        // them there.  (Holding the next tile in registers instead would cost U vectors per leaf for the whole
        // length of the program, and with them a third of the waves a SIMD can keep resident.)
        t += p.step_rows * tpr + p.step_chunks;
        row += p.step_rows;
        chunk += p.step_chunks;
        if (chunk >= tpr) {
            chunk -= tpr;
            ++row;
        }
        const bool more = t < p.n_tiles;
        T touched[kProgMaxLeaf];
#pragma unroll
        for (int k = 0; k < kProgMaxLeaf; ++k) touched[k] = T(0);
        if (more) {
            const int64_t n0 = static_cast<int64_t>(chunk) * TW + lane * VL;
#pragma unroll
            for (int k = 0; k < kProgMaxLeaf; ++k) {
                if (k < nl && p.leaf_cs[k] != 0) {
                    const T *base = static_cast<const T *>(p.leaf[k]) + static_cast<int64_t>(row) * p.leaf_rs[k];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int64_t c = n0 + u * (64 * VL);
                        if (c < cols && c >= p.leaf_lo[k] && c < p.leaf_hi[k]) touched[k] = base[c];
                    }
                }
            }
        }

        uint32_t next = p.code[0];
        for (int pc = 0; pc < n_instr; ++pc) {
            const uint32_t w = next;
            next = p.code[pc + 1];
            const int op = field(w, 0, 0xff), dst = field(w, 8, NREG - 1);
            const int a = field(w, 12, NREG - 1), b = field(w, 16, NREG - 1);
            const int c = field(w, 20, NREG - 1), d = field(w, 24, NREG - 1);
            T x[4][V], o[V];
#pragma unroll
            for (int j = 0; j < V; ++j) x[0][j] = r[j][a];
#pragma unroll
            for (int j = 0; j < V; ++j) x[1][j] = r[j][b];
#define AGMI_PROG_APPLY(OP, FN)                                               \
    {                                                                         \
        _Pragma("unroll") for (int j = 0; j < V; ++j) {                       \
            T xi[4] = {x[0][j], x[1][j], x[2][j], x[3][j]};                   \
            o[j] = apply_one<FN<T>, T, is_short_op(OP) || (LIGHT && is_light_inline_op(OP))>(xi); \
        }                                                                     \
    }
#define AGMI_PROG_CASE(OP, FN)                                                        \
    case OP: {                                                                        \
        if (FN<T>::NIN >= 3) {                                                        \
            _Pragma("unroll") for (int j = 0; j < V; ++j) x[2][j] = r[j][c];          \
        }                                                                             \
        if (FN<T>::NIN >= 4) {                                                        \
            _Pragma("unroll") for (int j = 0; j < V; ++j) x[3][j] = r[j][d];          \
        }                                                                             \
        AGMI_PROG_APPLY(OP, FN)                                                       \
        break;                                                                        \
    }
#define AGMI_PROG_STORE_AND_DEFAULT                                                                        \
    case AGMI_PROGRAM_MASK: {                                                                             \
        const int64_t lo = p.mask_lo[b & (kProgMaxMask - 1)], hi = p.mask_hi[b & (kProgMaxMask - 1)];     \
        _Pragma("unroll") for (int j = 0; j < V; ++j) x[2][j] = r[j][c];                                  \
        _Pragma("unroll") for (int u = 0; u < U; ++u)                                                     \
            _Pragma("unroll") for (int j = 0; j < VL; ++j) {                                              \
                const int64_t cc = c0 + u * (64 * VL) + j;                                                \
                o[u * VL + j] = (cc >= lo && cc < hi) ? x[0][u * VL + j] : x[2][u * VL + j];              \
            }                                                                                             \
        break;                                                                                            \
    }                                                                                                     \
    case AGMI_PROGRAM_ROWSUM:                                                                             \
    case AGMI_PROGRAM_ROWLSE: {                                                                           \
        if constexpr (ROWS) {                                                                             \
            const T total = op == AGMI_PROGRAM_ROWSUM                                                     \
                ? program_row_reduce<AccSum<T>, T, VL, U>(row_values[threadIdx.x >> 6], lane, cols, p.row_group, x[0]) \
                : program_row_reduce<AccLse<T>, T, VL, U>(row_values[threadIdx.x >> 6], lane, cols, p.row_group, x[0]); \
            _Pragma("unroll") for (int j = 0; j < V; ++j) o[j] = total;                                   \
        } else {                                                                                          \
            _Pragma("unroll") for (int j = 0; j < V; ++j) o[j] = x[0][j];                                 \
        }                                                                                                 \
        break;                                                                                            \
    }                                                                                                     \
    case AGMI_PROGRAM_STORE: {                                                                            \
        T *base = static_cast<T *>(p.out[b]) + static_cast<int64_t>(cur_row) * p.out_rs[b];               \
        _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                   \
            vec_t v;                                                                                      \
            _Pragma("unroll") for (int j = 0; j < VL; ++j) v[j] = x[0][u * VL + j];                       \
            if (interior)                                                                                 \
                *reinterpret_cast<vec_t *>(base + c0 + u * (64 * VL)) = v;                                \
            else                                                                                          \
                store_partial<T, VL>(base, c0 + u * (64 * VL), cols, v);                                  \
        }                                                                                                 \
    }                                                                                                     \
        [[fallthrough]];                                                                                  \
    default:                                                                                              \
        _Pragma("unroll") for (int j = 0; j < V; ++j) o[j] = x[0][j];                                     \
        break;
            if constexpr (LIGHT) {
                switch (op) {
                    AGMI_FOR_EACH_LIGHT_OP(AGMI_PROG_CASE)
                    AGMI_PROG_STORE_AND_DEFAULT
                }
            } else {
                switch (op) {
                    AGMI_FOR_EACH_PROGRAM_OP(AGMI_PROG_CASE)
                    AGMI_FOR_EACH_CHAINED_OP(AGMI_PROG_CASE)
                    AGMI_PROG_STORE_AND_DEFAULT
                }
            }
#undef AGMI_PROG_STORE_AND_DEFAULT
#undef AGMI_PROG_CASE
#undef AGMI_PROG_APPLY
#pragma unroll
            for (int j = 0; j < V; ++j) r[j][dst] = o[j];
        }
#pragma unroll
        for (int k = 0; k < kProgMaxLeaf; ++k) asm volatile("" : : "v"(touched[k]));  // (the touch loads are not dead code)
        if (!more) break;
    }
}

// ---- host side -------------------------------------------------------------------------
static int op_arity(int op) {
#define AGMI_ARITY_CASE(OP, FN) \
    case OP: return FN<float>::NIN;
    switch (op) {
        AGMI_FOR_EACH_PROGRAM_OP(AGMI_ARITY_CASE)
        AGMI_FOR_EACH_CHAINED_OP(AGMI_ARITY_CASE)
        default: return -1;
    }
#undef AGMI_ARITY_CASE
}

template <typename T, int NREG, int U, bool LIGHT, bool ROWS = false>
static int launch_program(const ProgParams &p0, int64_t rows, hipStream_t s) {
    ProgParams p = p0;
    constexpr int V = (16 / sizeof(T)) * U;
    constexpr int64_t TW = 64 * V;
    const int64_t tpr = ceil_div(p.cols, TW);
    const int64_t n_tiles = tpr * rows;
    if (tpr >= 0x7fffffffLL || n_tiles >= 0x7fffffffLL) {
        set_error("program: index space too large for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    // enough waves to fill the part several times over, few enough that each walks more than one tile on
    // large arrays (its next tile's loads are in flight while it interprets the current one)
    constexpr int64_t kMaxBlocks = 256 * 8;
    const int64_t blocks = std::min<int64_t>(ceil_div(n_tiles, kBlock / 64), kMaxBlocks);
    const int64_t n_waves = blocks * (kBlock / 64);
    p.tiles_per_row = static_cast<uint32_t>(tpr);
    p.n_tiles = static_cast<uint32_t>(n_tiles);
    p.step_rows = static_cast<uint32_t>(n_waves / tpr);
    p.step_chunks = static_cast<uint32_t>(n_waves % tpr);
    if (ROWS && tpr != 1) {
        set_error("program: a row sum needs rows of at most %lld columns", (long long)TW);
        return AGMI_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL((ew_program<T, NREG, U, LIGHT, ROWS>), dim3((unsigned)blocks), dim3(kBlock), 0, s, p);
    return hip_check(hipGetLastError(), "program launch");
}

// This file is compiled once per precision (-DAGMI_PART=32 / 64); the entry point lives in the float32 half.
#ifndef AGMI_PART
#error "compile with -DAGMI_PART=32 or -DAGMI_PART=64"
#endif
int launch_specialized(bool f32, int nreg, const ProgParams &p, int64_t rows, hipStream_t s);  // specialize.hip
int program_part_f32(int nreg, bool light, const ProgParams &p, int64_t rows, hipStream_t s);
int program_part_f64(int nreg, bool light, const ProgParams &p, int64_t rows, hipStream_t s);
// Two vectors per lane in every variant (measured on the 4M-element float64 tanh-gradient chain: 40 us against 42 with one;
// the scalar unit's decode work per instruction is shared by twice the elements, which outweighs the lost occupancy).
template <typename T>
static int launch_variant(int nreg, bool light, const ProgParams &p, int64_t rows, hipStream_t s) {
    if (p.row_group > 0) return launch_program<T, 16, 2, false, true>(p, rows, s);
    if (light) return nreg == 8 ? launch_program<T, 8, 2, true>(p, rows, s) : launch_program<T, 16, 2, true>(p, rows, s);
    return nreg == 8 ? launch_program<T, 8, 2, false>(p, rows, s) : launch_program<T, 16, 2, false>(p, rows, s);
}
#if AGMI_PART == 32
int program_part_f32(int nreg, bool light, const ProgParams &p, int64_t rows, hipStream_t s) {
    return launch_variant<float>(16, light, p, rows, s);
}
#else
int program_part_f64(int nreg, bool light, const ProgParams &p, int64_t rows, hipStream_t s) {
    return launch_variant<double>(nreg, light, p, rows, s);
}
#endif

}  // namespace agmi

using namespace agmi;

#if AGMI_PART == 32
extern "C" int agmi_program(int dtype, int ndim, const int64_t *shape, int n_out, const agmi_array *outs, int n_leaf,
                            const agmi_array *leaves, const int64_t *leaf_ranges, int n_imm, const double *imms,
                            int n_mask, const int64_t *mask_ranges, int n_instr, const uint32_t *code, int n_regs,
                            void *stream) {
    if (n_out < 1 || n_out > kProgMaxOut || n_leaf < 0 || n_leaf > kProgMaxLeaf || n_imm < 0 || n_imm > kProgMaxImm ||
        n_instr < 1 || n_instr > kProgMaxInstr || n_mask < 0 || n_mask > kProgMaxMask || !outs || (n_leaf && !leaves) ||
        (n_imm && !imms) || (n_mask && !mask_ranges) || !code) {
        set_error("program: bad counts (outputs %d, leaves %d, immediates %d, instructions %d) or null arrays", n_out,
                  n_leaf, n_imm, n_instr);
        return AGMI_ERR_ARG;
    }
    if (dtype != AGMI_F32 && dtype != AGMI_F64) {
        set_error("program: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    const int nreg = (n_regs <= 8 && dtype == AGMI_F64) ? 8 : 16;
    if (n_regs < 1 || n_regs > 16 || n_leaf + n_imm > nreg) {
        set_error("program: %d registers asked for (at most 16), %d leaves and %d immediates", n_regs, n_leaf, n_imm);
        return AGMI_ERR_ARG;
    }
    // every register an instruction names must exist, every value it reads must have been written
    uint32_t defined = 0;
    for (int k = 0; k < n_leaf; ++k) defined |= 1u << k;
    for (int k = 0; k < n_imm; ++k) defined |= 1u << (nreg - 1 - k);
    uint32_t stored = 0;
    bool light = true;
    bool row_sums = false;
    for (int i = 0; i < n_instr; ++i) {
        const uint32_t w = code[i];
        const int op = w & 0xff, dst = (w >> 8) & 15;
        light = light && is_light_op(op);
        const int src[4] = {int(w >> 12) & 15, int(w >> 16) & 15, int(w >> 20) & 15, int(w >> 24) & 15};
        if (w >> 28) {
            set_error("program: instruction %d has bits set above its fields", i);
            return AGMI_ERR_ARG;
        }
        if (op == AGMI_PROGRAM_MASK) {
            if (src[0] >= nreg || !(defined >> src[0] & 1u) || src[2] >= nreg || !(defined >> src[2] & 1u) ||
                src[1] >= n_mask || dst >= nreg) {
                set_error("program: instruction %d selects between registers %d and %d by range %d of %d", i, src[0],
                          src[2], src[1], n_mask);
                return AGMI_ERR_ARG;
            }
            defined |= 1u << dst;
            continue;
        }
        if (op == AGMI_PROGRAM_ROWSUM || op == AGMI_PROGRAM_ROWLSE) {
            if (src[0] >= nreg || !(defined >> src[0] & 1u) || dst >= nreg) {
                set_error("program: instruction %d sums register %d, which holds nothing, or writes register %d of %d", i,
                          src[0], dst, nreg);
                return AGMI_ERR_ARG;
            }
            row_sums = true;
            defined |= 1u << dst;
            continue;
        }
        if (op == AGMI_PROGRAM_STORE) {
            if (src[0] >= nreg || !(defined >> src[0] & 1u) || src[1] >= n_out || dst != src[0]) {
                set_error("program: instruction %d stores register %d to output %d", i, src[0], src[1]);
                return AGMI_ERR_ARG;
            }
            stored |= 1u << src[1];
            continue;
        }
        const int arity = op_arity(op);
        if (arity < 0) {
            set_error("program: instruction %d has unknown op %d", i, op);
            return AGMI_ERR_ARG;
        }
        for (int k = 0; k < arity; ++k)
            if (src[k] >= nreg || !(defined >> src[k] & 1u)) {
                set_error("program: instruction %d (op %d) reads register %d, which holds nothing", i, op, src[k]);
                return AGMI_ERR_ARG;
            }
        if (dst >= nreg) {
            set_error("program: instruction %d writes register %d of %d", i, dst, nreg);
            return AGMI_ERR_ARG;
        }
        defined |= 1u << dst;
    }
    if (stored != (1u << n_out) - 1u) {
        set_error("program: not every output is stored");
        return AGMI_ERR_ARG;
    }
    if (index_space_is_empty(ndim, shape)) return 0;
    const int64_t *strides[kProgMaxOut + kProgMaxLeaf];
    for (int k = 0; k < n_out; ++k) {
        if (outs[k].data == nullptr) {
            set_error("program: output %d is null", k);
            return AGMI_ERR_ARG;
        }
        strides[k] = outs[k].strides;
    }
    for (int k = 0; k < n_leaf; ++k) {
        if (leaves[k].data == nullptr) {
            set_error("program: leaf %d is null (scalars travel as immediates)", k);
            return AGMI_ERR_ARG;
        }
        strides[n_out + k] = leaves[k].strides;
    }
    Merged m;
    int row_group = 0;
    if (row_sums) {
        // rows stay rows: no merging, and only the shapes whose standalone row sums a group of lanes adds up
        constexpr int64_t kRowMax[2] = {64 * 2 * 4, 64 * 2 * 2};  // a wave's tile in float32 / float64
        const int64_t widest = kRowMax[dtype == AGMI_F32 ? 0 : 1];
        if (ndim != 2 || shape[1] > widest || (shape[1] > 64 && shape[0] < 64) || n_regs != 16 || leaf_ranges || n_mask) {
            set_error("program: row sums need a (rows, columns <= %lld) index space with at least 64 rows when the rows "
                      "are longer than 64, 16 registers, no leaf ranges and no masks", (long long)widest);
            return AGMI_ERR_UNSUPPORTED;
        }
        m.ndim = 2;
        m.n = shape[0] * shape[1];
        m.shape[0] = shape[0];
        m.shape[1] = shape[1];
        for (int k = 0; k < n_out + n_leaf; ++k) {
            m.stride[k][0] = shape[0] == 1 ? 0 : strides[k][0];
            m.stride[k][1] = shape[1] == 1 ? 0 : strides[k][1];
        }
        const int64_t quarter = (shape[1] + 3) / 4;
        row_group = 1;
        while (row_group < quarter && row_group < 64) row_group <<= 1;
    } else if (!merge_axes(ndim, shape, nullptr, n_out + n_leaf, strides, &m)) {
        return AGMI_ERR_ARG;
    }
    if (m.n == 0) return 0;
    if (m.ndim > 2) {
        set_error("program: %d axes remain after merging, at most 2 are supported", m.ndim);
        return AGMI_ERR_UNSUPPORTED;
    }
    const int last = m.ndim - 1;
    ProgParams p = {};
    p.cols = m.shape[last];
    const int64_t rows = m.ndim == 2 ? m.shape[0] : 1;
    for (int k = 0; k < n_out; ++k) {
        if (m.stride[k][last] != 1 && m.shape[last] != 1) {
            set_error("program: output %d is not contiguous along the innermost axis", k);
            return AGMI_ERR_UNSUPPORTED;
        }
        p.out[k] = outs[k].data;
        p.out_rs[k] = m.ndim == 2 ? m.stride[k][0] : 0;
        if (m.ndim == 2 && m.shape[0] > 1 && p.out_rs[k] == 0) {
            set_error("program: output %d has stride 0 on an axis of extent %lld", k, (long long)m.shape[0]);
            return AGMI_ERR_ARG;
        }
    }
    for (int k = 0; k < n_leaf; ++k) {
        const int64_t cs = m.stride[n_out + k][last];
        if (cs != 0 && cs != 1) {
            set_error("program: leaf %d has stride %lld along the innermost axis", k, (long long)cs);
            return AGMI_ERR_UNSUPPORTED;
        }
        p.leaf[k] = leaves[k].data;
        p.leaf_cs[k] = static_cast<int32_t>(cs);
        p.leaf_rs[k] = m.ndim == 2 ? m.stride[n_out + k][0] : 0;
    }
    // Shifted reads: a leaf of a one-row program may come with the columns [lo, hi) at which its address is
    // readable (its pointer is already moved by the shift, so columns outside would fall before or behind its
    // storage); such columns read as 1 and the program masks them.  No range: every column.
    p.safe_lo = 0;
    p.safe_hi = p.cols;
    for (int k = 0; k < n_leaf; ++k) {
        p.leaf_lo[k] = 0;
        p.leaf_hi[k] = p.cols;
        if (leaf_ranges && p.leaf_cs[k] != 0) {
            if (rows != 1) {
                set_error("program: leaf ranges need a one-row index space");
                return AGMI_ERR_UNSUPPORTED;
            }
            p.leaf_lo[k] = std::max<int64_t>(leaf_ranges[2 * k], 0);
            p.leaf_hi[k] = std::min<int64_t>(leaf_ranges[2 * k + 1], p.cols);
        }
        p.safe_lo = std::max(p.safe_lo, p.leaf_lo[k]);
        p.safe_hi = std::min(p.safe_hi, p.leaf_hi[k]);
    }
    for (int k = 0; k < n_mask; ++k) {
        p.mask_lo[k] = mask_ranges[2 * k];
        p.mask_hi[k] = mask_ranges[2 * k + 1];
    }
    if (n_mask && rows != 1) {
        set_error("program: masks need a one-row index space");
        return AGMI_ERR_UNSUPPORTED;
    }
    p.row_group = row_group;
    p.n_leaf = n_leaf;
    p.n_imm = n_imm;
    p.n_instr = n_instr;
    for (int k = 0; k < n_imm; ++k) p.imm[k] = imms[k];
    for (int i = 0; i < n_instr; ++i) p.code[i] = code[i];
    p.code[n_instr] = 0;
    hipStream_t s = as_stream(stream);
    // a program that keeps coming back runs on a kernel compiled for it (1: not this one, or not yet)
    const int specialised = launch_specialized(dtype == AGMI_F32, nreg, p, rows, s);
    if (specialised <= 0) return specialised;
    set_kernel_name("ew_program<%s,%d,%s>[%d instr, %lldx%lld]", dtype == AGMI_F32 ? "float" : "double", nreg,
                    row_group ? "rows" : (light ? "light" : "full"), n_instr, (long long)rows, (long long)p.cols);
    return dtype == AGMI_F32 ? program_part_f32(nreg, light, p, rows, s) : program_part_f64(nreg, light, p, rows, s);
}
#endif  // AGMI_PART == 32
