// What the program kernels take as their argument, and the one helper they share.  This file is also handed, as
// text, to the run-time compiler that specialises recurring programs (specialize.hip): the interpreter and a
// specialised kernel are launched with the same argument block over the same tiling.
#pragma once

namespace agmi {

constexpr int kProgMaxLeaf = AGMI_PROGRAM_MAX_LEAVES;
constexpr int kProgMaxImm = AGMI_PROGRAM_MAX_IMMEDIATES;
constexpr int kProgMaxOut = AGMI_PROGRAM_MAX_OUTPUTS;
constexpr int kProgMaxInstr = AGMI_PROGRAM_MAX_INSTRUCTIONS;
constexpr int kProgMaxMask = AGMI_PROGRAM_MAX_MASKS;

struct ProgParams {
    int64_t cols;
    uint32_t tiles_per_row, n_tiles;
    uint32_t step_rows, step_chunks;  // the wave stride (number of waves in the grid) split by tiles_per_row
    int32_t n_leaf, n_imm, n_instr;
    int32_t row_group;  // programs with row sums: the lanes that share a row in the reduction kernel's order
    const void *leaf[kProgMaxLeaf];
    int64_t leaf_rs[kProgMaxLeaf];
    int32_t leaf_cs[kProgMaxLeaf];  // 0 or 1
    // columns a leaf may be read at (one-row programs whose leaves are read at shifted positions); all columns otherwise
    int64_t leaf_lo[kProgMaxLeaf], leaf_hi[kProgMaxLeaf];
    int64_t safe_lo, safe_hi;  // the columns every leaf may be read at
    int64_t mask_lo[kProgMaxMask], mask_hi[kProgMaxMask];
    void *out[kProgMaxOut];
    int64_t out_rs[kProgMaxOut];
    double imm[kProgMaxImm];
    uint32_t code[kProgMaxInstr + 1];  // one word of padding: the fetch runs one instruction ahead
};

// The last, partly filled vector of a row.  A function of its own: its per-lane branches would otherwise make
// the compiler restructure the whole interpreter loop around them (every wave-uniform branch of the dispatch
// would then cost several scalar instructions more).
template <typename T, int VL>
struct ProgVec {
    typedef T type __attribute__((ext_vector_type(VL)));
};
template <typename T, int VL>
static __device__ __noinline__ void store_partial(T *base, int64_t c, int64_t cols, typename ProgVec<T, VL>::type v) {
#pragma unroll
    for (int j = 0; j < VL; ++j)
        if (c + j < cols) base[c + j] = v[j];
}

// The reduction of a program register over a row that one wave holds (AGMI_PROGRAM_ROWSUM, AGMI_PROGRAM_ROWLSE), in
// the order of the reduction kernel red_row_group for a row of that length: the wave writes the row to its stretch of
// LDS, lane g of the first G adds up (combines) columns g, g + G, ... starting from the identity, the G partial results
// meet in a butterfly, and lane 0 holds what that kernel would store; every lane gets it.  Bit for bit the reduction
// kernel's result, so a value does not depend on whether a chain formed it inside or read it from memory.
template <class Acc, typename T, int VL, int U>
__device__ __forceinline__ T program_row_reduce(T *mine, uint32_t lane, int64_t cols, int G, const T (&v)[VL * U]) {
    typedef T vec_t __attribute__((ext_vector_type(VL), aligned(sizeof(T))));
#pragma unroll
    for (int u = 0; u < U; ++u) {
        vec_t w;
#pragma unroll
        for (int j = 0; j < VL; ++j) w[j] = v[u * VL + j];
        *reinterpret_cast<vec_t *>(mine + u * (64 * VL) + lane * VL) = w;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    typename Acc::type acc = Acc::identity();
    if (static_cast<int>(lane) < G)
        for (int64_t rr = lane; rr < cols; rr += G) acc = Acc::combine(acc, Acc::lift(mine[rr]));
    for (int m = G >> 1; m > 0; m >>= 1) acc = Acc::combine(acc, Acc::shfl_xor(acc, m));
    const T total = __shfl(Acc::finish(acc), 0, 64);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    return total;
}

}  // namespace agmi
