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

}  // namespace agmi
