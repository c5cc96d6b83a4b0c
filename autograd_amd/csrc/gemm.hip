// Dense contraction on the CDNA4 matrix cores:  C = alpha * A.B + beta * C.
//
// fp32 uses v_mfma_f32_32x32x2_f32 (true fp32 multiply-accumulate, 256 FLOP/clk/CU), fp64
// v_mfma_f64_16x16x4_f64.  Operands are addressed through (row, column) element strides, so
// the transposed factors of the dot adjoints (G.B^T, A^T.G) are read in place; only the
// global->LDS copy depends on the layout, the LDS image and the MFMA loop do not.
//
// Block: 256 threads = 4 waves in a 2 x 2 arrangement over a BM x BN tile of C, each wave
// owning a (BM/2) x (BN/2) sub-tile as a grid of MFMA blocks.  LDS holds the current K-slab
// of A as As[k][m] and of B as Bs[k][n] (m / n contiguous, padded), double-buffered: while
// the matrix cores work on slab t, the global loads of slab t+1 are in flight in registers
// and are written to the other buffer afterwards - one barrier per slab.
// Operand lane mapping (verified on gfx950): fp32 32x32x2 - lane l supplies A[row=l%32][k=l/32],
// B[k=l/32][col=l%32]; accumulator register v of lane l is C[8*(v/4)+4*(l/32)+v%4][l%32].
// fp64 16x16x4 - lane l supplies A[l%16][l/16], B[l/16][l%16]; register v is C[4*v+l/16][l%16].
//
// Two kernels share that scheme.  gemm_mfma stages operands through registers (any strides, both
// precisions).  gemm_direct (fp32, operands with a unit stride and 16-byte aligned rows) lets the
// memory pipeline write each K-slab straight into LDS (buffer_load ... lds): no staging registers,
// no LDS store instructions, no wait for global data in the middle of the MFMA stream; a ring of
// four slab buffers keeps three slabs in flight ahead of the matrix cores.
//
// Workgroup ids are dealt round-robin to the 8 XCDs (each with its own L2), so the tile
// order is remapped: XCD x works on a contiguous range of tiles, walked in column-major
// groups of kGroupM tile-rows, which keeps one XCD's A rows and B columns resident in its L2.
#include <algorithm>

#include <cstdio>

#include "common.h"

namespace agmi {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef double v4d __attribute__((ext_vector_type(4)));

struct MfmaF32x32 {
    typedef float elem_t;
    static constexpr int TM = 32;   // rows = cols of one MFMA block
    static constexpr int TK = 2;    // K depth of one instruction
    static constexpr int NACC = 16; // accumulator registers per lane
    typedef v16f acc_t;
    __device__ __forceinline__ static acc_t mma(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    __device__ __forceinline__ static int d_row(int v, int lane) { return 8 * (v / 4) + 4 * (lane / 32) + (v % 4); }
};

typedef float v4f __attribute__((ext_vector_type(4)));

struct MfmaF32x16 {  // 16x16x4: four independent accumulators per 32x32 wave tile instead of one chain
    typedef float elem_t;
    static constexpr int TM = 16;
    static constexpr int TK = 4;
    static constexpr int NACC = 4;
    typedef v4f acc_t;
    __device__ __forceinline__ static acc_t mma(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    __device__ __forceinline__ static int d_row(int v, int lane) { return 4 * (lane / 16) + v; }
};

struct MfmaF64x16 {
    typedef double elem_t;
    static constexpr int TM = 16;
    static constexpr int TK = 4;
    static constexpr int NACC = 4;
    typedef v4d acc_t;
    __device__ __forceinline__ static acc_t mma(double a, double b, acc_t c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    __device__ __forceinline__ static int d_row(int v, int lane) { return 4 * v + lane / 16; }
};

struct GemmParams {
    const void *A;
    const void *B;
    void *C;
    int64_t M, N, K;
    int64_t a_rs, a_cs, a_bs;
    int64_t b_rs, b_cs, b_bs;
    int64_t ldc, c_bs;
    double alpha, beta;
    int tiles_m, tiles_n;
    // cross-block K split (blockIdx.z): split z covers k in [z * k_per_split, min(K, (z+1) * k_per_split))
    // and writes its raw partial tile to ws[(z * batch + b) * M * N + row * N + col]
    int splits;
    int64_t k_per_split;
    void *ws;
    // gemm_direct only: bytes from element (0, 0) of one matrix of the batch to one past its last
    // element (the extent of the buffer descriptor the loads are range-checked against)
    uint32_t a_span_bytes, b_span_bytes;
    // gemm_block_split only: a second product A2 . B2 (M x K2, K2 x N; no batch) added to the first before the epilogue
    const void *A2, *B2;
    int64_t K2, a2_rs, a2_cs, b2_rs, b2_cs, k_per_split2;
    int splits2;
    uint32_t a2_span_bytes, b2_span_bytes;
    // epilogue of the float32 direct kernel and of the split finish (agmi_gemm_fused):
    //   1: beside C, epi_out[m, n] = tanh(C[m, n] + epi_bias[n])
    //   2: C[m, n] = acc / cosh(epi_x[m, n] + epi_bias[n])**2 (the product itself is not stored)
    // epi_bias may be null (nothing added)
    int epi;
    const float *epi_bias;
    float *epi_out;
    int64_t epi_ld;
    const float *epi_x;
    int64_t epi_x_ld;
};

// What follows the contraction in an evaluation of a dense layer and of its adjoint, applied to the accumulators
// before they are stored.  The arithmetic is the one-rule kernels' (functors.h: FTanh, FTanhVjp; a pending
// `+ bias` is one rounded add), so the results are the separate launches' bit for bit.
__device__ __forceinline__ float epi_tanh(float acc, float bias, bool has_bias) {
    const float z = has_bias ? acc + bias : acc;
    return tanhf(z);
}
__device__ __forceinline__ float epi_tanh_vjp(float acc, float x, float bias, bool has_bias) {
    const float z = has_bias ? x + bias : x;
    const float c = coshf(z);
    return acc / (c * c);
}

constexpr int kGroupM = 8;
constexpr int kXcds = 8;

// Copy one K-slab of an operand into LDS as S[k][x] (x = m for A, n for B).
//   xs: element stride along x, ks: element stride along k in global memory.
// MODE fixes, at compile time, how a thread's groups of 4 elements lie in global memory:
//   kXC - 4 consecutive x at one k (xs == 1, X % 4 == 0): one 16-byte load, one 16-byte LDS store
//   kKC - 4 consecutive k at one x (ks == 1, K % 4 == 0): one 16-byte load, stored transposed
//   kGen - any strides / ragged extents: four 4-byte loads
// Loads are branch-free (out-of-range groups read a clamped address), so the number of loads in
// flight is the same on every path and the compiler can wait for exactly the slab it needs
// (s_waitcnt vmcnt(n)) while younger prefetches stay in flight.  Out-of-range groups are zeroed
// when the slab is copied to LDS, not when it is loaded: a select right after the load would
// make every iteration wait for the load it has just issued.
enum LoadMode { kXC = 0, kKC = 1, kGen = 2 };

template <typename T, int BX, int BK, int LOADS, int MODE, int NT>
struct SlabLoader {
    T reg[LOADS][4];

    __device__ __forceinline__ void load(const T *__restrict__ g, int64_t xs, int64_t ks, int64_t x0, int64_t X,
                                         int64_t k0, int64_t K, int tid) {
        typedef T vec_t __attribute__((ext_vector_type(4), aligned(sizeof(T))));
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int e = tid + i * NT;
            if (MODE == kKC) {
                const int xx = e / (BK / 4), kk = (e % (BK / 4)) * 4;
                const int64_t k = k0 + kk, x = x0 + xx;
                const bool ok = x < X && k < K;  // K % 4 == 0: the group is all in or all out
                const vec_t v = *reinterpret_cast<const vec_t *>(ok ? g + x * xs + k : g);
#pragma unroll
                for (int j = 0; j < 4; ++j) reg[i][j] = v[j];
            } else {
                const int kk = e / (BX / 4), xx = (e % (BX / 4)) * 4;
                const int64_t k = k0 + kk, x = x0 + xx;
                if (MODE == kXC) {
                    const bool ok = k < K && x < X;  // X % 4 == 0
                    const vec_t v = *reinterpret_cast<const vec_t *>(ok ? g + k * ks + x : g);
#pragma unroll
                    for (int j = 0; j < 4; ++j) reg[i][j] = v[j];
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const bool ok = k < K && x + j < X;
                        reg[i][j] = *(ok ? g + k * ks + (x + j) * xs : g);
                    }
                }
            }
        }
    }

    // (x0, X, k0, K): the bounds the slab in `reg` was loaded with
    template <int LDX>
    __device__ __forceinline__ void store(T (*S)[LDX], int64_t x0, int64_t X, int64_t k0, int64_t K, int tid) const {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int e = tid + i * NT;
            if (MODE == kKC) {
                const int xx = e / (BK / 4), kk = (e % (BK / 4)) * 4;
                const bool ok = x0 + xx < X && k0 + kk < K;
#pragma unroll
                for (int j = 0; j < 4; ++j) S[kk + j][xx] = ok ? reg[i][j] : T(0);
            } else {
                const int kk = e / (BX / 4), xx = (e % (BX / 4)) * 4;
                const bool k_ok = k0 + kk < K;
#pragma unroll
                for (int j = 0; j < 4; ++j) S[kk][xx + j] = (k_ok && x0 + xx + (MODE == kXC ? 0 : j) < X) ? reg[i][j] : T(0);
            }
        }
    }
};

template <class MF, int BM, int BN, int BK, int DEPTH, int MODE_A, int MODE_B, int KS>
__global__ __launch_bounds__(kBlock *KS) void gemm_mfma(const GemmParams p) {
    using T = typename MF::elem_t;
    constexpr int TM = MF::TM, TK = MF::TK;
    constexpr int WM = BM / 2, WN = BN / 2;      // wave tile
    constexpr int FM = WM / TM, FN = WN / TM;    // MFMA blocks per wave
    // row padding of the LDS images: 16-byte rows for vector stores, or (transposed 4-byte stores)
    // a pitch that spreads a wave's stores over all 32 banks
    constexpr int PAD_A = MODE_A == kKC ? 2 : 4, PAD_B = MODE_B == kKC ? 2 : 4;
    // KS groups of 4 waves share one C tile and split every K-slab between them (two waves per
    // SIMD keep the matrix core fed while the other waits on LDS or the barrier); their partial
    // accumulators are summed through LDS once, in group order, before the epilogue.
    constexpr int NT = kBlock * KS;
    constexpr int LA = (BM * BK) / (NT * 4), LB = (BN * BK) / (NT * 4);
    static_assert(LA >= 1 && LB >= 1, "slab too small for the thread count");
    constexpr int STEPS = BK / TK / KS;  // MFMA k-steps per wave per slab
    static_assert(STEPS >= 1 && (BK / TK) % KS == 0, "K split");
    static_assert(WM % TM == 0 && WN % TM == 0 && BK % TK == 0 && BK % 4 == 0, "tile shape");
    static_assert(DEPTH >= 2 && DEPTH % 2 == 0, "prefetch depth must be even (buffer parity is fixed at compile time)");

    // one LDS allocation: the two double-buffered slab images, reused as scratch by the K-group sum
    constexpr int kAsElems = 2 * BK * (BM + PAD_A), kBsElems = 2 * BK * (BN + PAD_B);
    constexpr int kScratchElems = (KS - 1) * 4 * FM * FN * MF::NACC * 64;
    constexpr int kLdsElems = (kAsElems + kBsElems) > kScratchElems ? (kAsElems + kBsElems) : kScratchElems;
    __shared__ T lds[kLdsElems];
    T(*As)[BK][BM + PAD_A] = reinterpret_cast<T(*)[BK][BM + PAD_A]>(lds);
    T(*Bs)[BK][BN + PAD_B] = reinterpret_cast<T(*)[BK][BN + PAD_B]>(lds + kAsElems);

    // XCD-aware tile order
    const int n_tiles = p.tiles_m * p.tiles_n;
    int bid = blockIdx.x;
    {
        const int per_xcd = n_tiles / kXcds;  // the ragged remainder keeps its natural ids
        if (bid < per_xcd * kXcds) bid = (bid % kXcds) * per_xcd + bid / kXcds;
    }
    const int group_size = kGroupM * p.tiles_n;
    const int group = bid / group_size;
    const int first_m = group * kGroupM;
    const int rows_in_group = min(p.tiles_m - first_m, kGroupM);
    const int tile_m = first_m + (bid % group_size) % rows_in_group;
    const int tile_n = (bid % group_size) / rows_in_group;

    const int64_t batch = blockIdx.y;
    const T *__restrict__ A = static_cast<const T *>(p.A) + batch * p.a_bs;
    const T *__restrict__ B = static_cast<const T *>(p.B) + batch * p.b_bs;
    T *__restrict__ C = static_cast<T *>(p.C) + batch * p.c_bs;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int kgroup = wave >> 2, quad = wave & 3;
    const int wm0 = (quad >> 1) * WM, wn0 = (quad & 1) * WN;
    const int ks0 = kgroup * STEPS * TK;  // this wave's first k inside a slab
    const int64_t m0 = static_cast<int64_t>(tile_m) * BM, n0 = static_cast<int64_t>(tile_n) * BN;
    const int op_x = lane % TM, op_k = lane / TM;

    typename MF::acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < MF::NACC; ++v) acc[i][j][v] = T(0);

    // Global loads run DEPTH slabs ahead of the matrix cores: with one 4-wave block per CU there
    // is nothing else to hide HBM/L2 latency behind, and a slab is only ~1 us of MFMA work.
    SlabLoader<T, BM, BK, LA, MODE_A, NT> la[DEPTH];
    SlabLoader<T, BN, BK, LB, MODE_B, NT> lb[DEPTH];
    const int64_t k_first = static_cast<int64_t>(blockIdx.z) * p.k_per_split;   // multiple of BK
    const int64_t k_limit = min(p.K, k_first + p.k_per_split);
    const int64_t n_slabs = (k_limit - k_first + BK - 1) / BK;
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        // slabs past the end load zeros (their k range fails the bounds test), harmless and branch-free
        la[d].load(A, p.a_rs, p.a_cs, m0, p.M, k_first + static_cast<int64_t>(d) * BK, k_limit, tid);
        lb[d].load(B, p.b_cs, p.b_rs, n0, p.N, k_first + static_cast<int64_t>(d) * BK, k_limit, tid);
    }
    // Register slot s % DEPTH holds slab s until it has been copied to LDS (two iterations before
    // the matrix cores reach it), then is refilled with slab s + DEPTH.  Operand fragments are double-buffered in registers as well: the fragments
    // of slab t + 1 are read from LDS while the matrix cores work on slab t, so that LDS latency
    // is not paid in front of every group of MFMAs.
    T fa[2][STEPS][FM], fb[2][STEPS][FN];
    auto read_fragment = [&](int f, int buf, int s) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[f][s][i] = As[buf][ks0 + s * TK + op_k][wm0 + i * TM + op_x];
#pragma unroll
        for (int j = 0; j < FN; ++j) fb[f][s][j] = Bs[buf][ks0 + s * TK + op_k][wn0 + j * TM + op_x];
    };
    auto read_fragments = [&](int f, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < STEPS; ++s) read_fragment(f, buf, s);
    };
    auto slab_k = [&](int64_t slab) { return k_first + slab * BK; };
    la[0].template store<BM + PAD_A>(As[0], m0, p.M, slab_k(0), k_limit, tid);
    lb[0].template store<BN + PAD_B>(Bs[0], n0, p.N, slab_k(0), k_limit, tid);
    __syncthreads();
    read_fragments(0, 0);
    if (n_slabs > 1) {
        la[1 % DEPTH].template store<BM + PAD_A>(As[1], m0, p.M, slab_k(1), k_limit, tid);
        lb[1 % DEPTH].template store<BN + PAD_B>(Bs[1], n0, p.N, slab_k(1), k_limit, tid);
    }

    // One slab step.  `d` = t % DEPTH and `guarded` are compile-time constants after unrolling.
    // A wave's MFMAs form one dependent chain per accumulator, so each one issues only when the
    // previous has finished; everything else the step has to do (the global loads of slab
    // t + DEPTH, the LDS reads of slab t + 1's fragments, the LDS writes of slab t + 2) is placed
    // between the MFMAs and runs in their shadow.  The scheduling barriers pin that order (the
    // scheduler would otherwise sink each LDS read next to its use, one step later).  Reads and
    // writes of one step go to different LDS buffers, so their order within the step is free.
    auto step = [&](const int d, const int64_t t, const bool guarded) __attribute__((always_inline)) {
        const int cur = d & 1;  // DEPTH is even: slab t lives in LDS buffer t % 2
        constexpr int kStoreAt = STEPS / 2;
        // slab t + 1 is complete in LDS, and every wave is done reading buffer `cur`
        __syncthreads();
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = MF::mma(fa[cur][s][i], fb[cur][s][j], acc[i][j]);
            // two fragment reads per MFMA in the first half of the step: every read has returned
            // long before the wave reaches the barrier
            if ((!guarded || t + 1 < n_slabs) && 2 * s < STEPS) {
                read_fragment(cur ^ 1, cur ^ 1, 2 * s);
                if (2 * s + 1 < STEPS) read_fragment(cur ^ 1, cur ^ 1, 2 * s + 1);
            }
            if (s == 0) {
                // slot d held slab t, which went to LDS two steps ago: refill it
                la[d].load(A, p.a_rs, p.a_cs, m0, p.M, slab_k(t + DEPTH), k_limit, tid);
                lb[d].load(B, p.b_cs, p.b_rs, n0, p.N, slab_k(t + DEPTH), k_limit, tid);
            }
            if (s == kStoreAt && (!guarded || t + 2 < n_slabs)) {
                const int slot = (d + 2) % DEPTH;
                la[slot].template store<BM + PAD_A>(As[cur], m0, p.M, slab_k(t + 2), k_limit, tid);
                lb[slot].template store<BN + PAD_B>(Bs[cur], n0, p.N, slab_k(t + 2), k_limit, tid);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // main loop: groups of DEPTH steps that need no bounds tests form one straight-line block, so
    // the count of loads in flight is known exactly at every wait; the last steps are guarded
    int64_t t0 = 0;
    for (; t0 + DEPTH + 2 <= n_slabs; t0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) step(d, t0 + d, false);
    }
    for (; t0 < n_slabs; t0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d)
            if (t0 + d < n_slabs) step(d, t0 + d, true);  // uniform across the block
    }

    if (KS > 1) {
        // sum the K-split partial accumulators: groups 1.. park theirs in LDS (the slab buffers are
        // free after the last barrier), group 0 adds them in group order
        T *scratch = lds;
        if (kgroup > 0) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int v = 0; v < MF::NACC; ++v)
                        scratch[((((kgroup - 1) * 4 + quad) * FM * FN + i * FN + j) * MF::NACC + v) * 64 + lane] = acc[i][j][v];
        }
        __syncthreads();
        if (kgroup > 0) return;
#pragma unroll
        for (int g = 1; g < KS; ++g)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int v = 0; v < MF::NACC; ++v)
                        acc[i][j][v] += scratch[((((g - 1) * 4 + quad) * FM * FN + i * FN + j) * MF::NACC + v) * 64 + lane];
    }

    if (p.splits > 1) {  // raw partial tile; gemm_split_finish applies alpha / beta
        T *W = static_cast<T *>(p.ws) + (static_cast<int64_t>(blockIdx.z) * gridDim.y + batch) * p.M * p.N;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int64_t col = n0 + wn0 + j * TM + op_x;
#pragma unroll
                for (int v = 0; v < MF::NACC; ++v) {
                    const int64_t row = m0 + wm0 + i * TM + MF::d_row(v, lane);
                    if (row < p.M && col < p.N) W[row * p.N + col] = acc[i][j][v];
                }
            }
        return;
    }

    const T alpha = static_cast<T>(p.alpha), beta = static_cast<T>(p.beta);
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int64_t col = n0 + wn0 + j * TM + op_x;
#pragma unroll
            for (int v = 0; v < MF::NACC; ++v) {
                const int64_t row = m0 + wm0 + i * TM + MF::d_row(v, lane);
                if (row < p.M && col < p.N) {
                    T *dst = C + row * p.ldc + col;
                    T r = acc[i][j][v];
                    if (p.alpha != 1.0) r = alpha * r;
                    if (p.beta != 0.0) r = r + beta * *dst;
                    *dst = r;
                }
            }
        }
}


// ---- direct-to-LDS kernel ------------------------------------------------------------------------
//
// Tile 64 x 64 x 32, 512 threads = 8 waves: two K-groups of 2 x 2 waves, each wave one 32 x 32
// accumulator over its half of every slab (two waves per SIMD keep the matrix core fed).
//
// Loads.  One wave-wide `buffer_load_dwordx4 ... lds` moves 1 KB; lane e's 16 bytes land at LDS
// offset 16 e of the chunk, so the LDS image is fixed by which global address each lane reads:
//   x-contiguous operand (kXC): slab image [k][x], 64 x per row; chunk c = k rows 4c .. 4c+3;
//                               lane e reads k = 4c + e/16, x = 4 (e%16)
//   k-contiguous operand (kKC): slab image [x][k], 32 k per row in eight 16-byte groups; chunk c =
//                               x rows 8c .. 8c+7; the group that holds k-group g of row x sits at
//                               position g ^ (x % 8), so that the 16-byte fragment reads of 8
//                               consecutive rows fall on 8 different bank groups
// Wave w loads chunk w of both operands, behind two different MFMAs of the step (sixteen loads
// issued together right after the barrier queue up in the CU's one address unit and hold back the
// MFMAs behind them).  Out-of-range lanes (x beyond the matrix edge, k beyond this block's K range)
// get an offset beyond the descriptor's extent: the hardware then writes zeros, which is exactly
// the padding the product needs, so ragged edges cost one select per load and no extra code.
// Offsets are 32-bit: operands must span less than 2 GiB (the caller checks).
//
// MFMA k order.  Within a group q of 8 k, instruction j (0..3) multiplies k = 8q + 4h + j in lane
// half h: a k-contiguous operand delivers a lane's four j values with one 16-byte LDS read, an
// x-contiguous one with four 4-byte reads at a fixed row pitch.
//
// Pipeline per step t (slab t):  wait until this wave's loads of slab t+1 have landed; barrier
// (now slab t+1 is complete for everyone, and everyone is done reading slab t-1's buffer); 8 MFMAs
// on slab t's fragments (in registers since step t-1) with, in their shadow, the loads of slab t+3
// into slab t-1's buffer and the LDS reads of slab t+1's fragments.
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kDirectThreads = 512;
constexpr uint32_t kDirectOob = 0x80000000u;  // beyond any extent the caller admits

// The destination of an LDS-direct load is M0 (wave-uniform LDS byte address) + 16 * lane.  Written
// as inline assembly so that the compiler's wait-count bookkeeping does not make every later LDS
// read wait for all loads in flight; the kernel waits with explicit s_waitcnt vmcnt(n) instead.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // M0 is written on purpose: it is the load's destination register
__device__ __forceinline__ void load_to_lds_16(v4i rsrc, uint32_t byte_offset, uint32_t lds_byte_addr) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, 0 offen lds"
        :
        : "s"(lds_byte_addr), "v"(byte_offset), "s"(rsrc)
        : "memory", "m0");
}
#pragma clang diagnostic pop

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt range");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ v4i raw_buffer(const void *base, uint32_t bytes) {
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    v4i r;
    r[0] = static_cast<int>(b & 0xffffffffu);
    r[1] = static_cast<int>((b >> 32) & 0xffffu);  // stride 0: raw buffer, offsets checked against `bytes`
    r[2] = static_cast<int>(bytes);
    r[3] = 0x00020000;                             // 32-bit raw data format
    return r;
}

// TAIL: K is not a multiple of 4 and an operand is contiguous along k, so the 16 bytes a lane fetches at the end of
// a row run past k = K into whatever follows in memory (the next row); those elements are zeroed in LDS before
// any wave reads the slab.
template <int MODE_A, int MODE_B, bool TAIL, int EPI>
__global__ __launch_bounds__(kDirectThreads) void gemm_direct(const GemmParams p) {
    constexpr int BM = 64, BN = 64, BK = 32, NBUF = 4;
    constexpr int kOpFloats = 64 * BK;         // one operand slab
    constexpr int kBufFloats = 2 * kOpFloats;  // A then B
    constexpr int NQ = BK / 16;                // groups of 8 k per K-group per slab
    constexpr int G = BK / 4;                  // 16-byte groups per row of a k-contiguous operand
    constexpr int kDist = NBUF - 1;            // slabs in flight ahead of the matrix cores
    constexpr int kSlotA = 1, kSlotB = 5;      // MFMAs of the step the two loads are issued behind
    __shared__ __attribute__((aligned(1024))) float lds[NBUF * kBufFloats];

    const int n_tiles = p.tiles_m * p.tiles_n;
    int bid = blockIdx.x;
    {
        const int per_xcd = n_tiles / kXcds;
        if (bid < per_xcd * kXcds) bid = (bid % kXcds) * per_xcd + bid / kXcds;
    }
    const int group_size = kGroupM * p.tiles_n;
    const int group = bid / group_size;
    const int first_m = group * kGroupM;
    const int rows_in_group = min(p.tiles_m - first_m, kGroupM);
    const int tile_m = first_m + (bid % group_size) % rows_in_group;
    const int tile_n = (bid % group_size) / rows_in_group;

    const int64_t batch = blockIdx.y;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kgroup = wave >> 2, quad = wave & 3;
    const int wm0 = (quad >> 1) * 32, wn0 = (quad & 1) * 32;
    const int64_t m0 = static_cast<int64_t>(tile_m) * BM, n0 = static_cast<int64_t>(tile_n) * BN;
    const int r = lane & 31, h = lane >> 5;

    const int64_t k_first = static_cast<int64_t>(blockIdx.z) * p.k_per_split;  // multiple of BK
    const int64_t k_limit = min(p.K, k_first + p.k_per_split);
    const int n_slabs = static_cast<int>((k_limit - k_first + BK - 1) / BK);

    const v4i rsrc_a = raw_buffer(static_cast<const float *>(p.A) + batch * p.a_bs, p.a_span_bytes);
    const v4i rsrc_b = raw_buffer(static_cast<const float *>(p.B) + batch * p.b_bs, p.b_span_bytes);

    // this lane's 16 bytes of chunk `wave`: byte offset of slab 0, advance per slab, and how many k
    // remain from its k position to the end of the block's range (<= 0: load zeros)
    uint32_t off_a, off_b, step_a, step_b;
    int krem_a, krem_b;
    if (MODE_A == kXC) {
        const int kl = 4 * wave + lane / 16, xl = 4 * (lane % 16);
        off_a = static_cast<uint32_t>(((k_first + kl) * p.a_cs + (m0 + xl)) * 4);
        step_a = static_cast<uint32_t>(BK * p.a_cs * 4);
        krem_a = (m0 + xl < p.M) ? static_cast<int>(k_limit - k_first) - kl : 0;
    } else {
        const int xl = (64 / G) * wave + lane / G, k4 = (lane % G) ^ (xl & 7);
        off_a = static_cast<uint32_t>(((m0 + xl) * p.a_rs + k_first + 4 * k4) * 4);
        step_a = BK * 4;
        krem_a = (m0 + xl < p.M) ? static_cast<int>(k_limit - k_first) - 4 * k4 : 0;
    }
    if (MODE_B == kXC) {
        const int kl = 4 * wave + lane / 16, xl = 4 * (lane % 16);
        off_b = static_cast<uint32_t>(((k_first + kl) * p.b_rs + (n0 + xl)) * 4);
        step_b = static_cast<uint32_t>(BK * p.b_rs * 4);
        krem_b = (n0 + xl < p.N) ? static_cast<int>(k_limit - k_first) - kl : 0;
    } else {
        const int xl = (64 / G) * wave + lane / G, k4 = (lane % G) ^ (xl & 7);
        off_b = static_cast<uint32_t>(((n0 + xl) * p.b_cs + k_first + 4 * k4) * 4);
        step_b = BK * 4;
        krem_b = (n0 + xl < p.N) ? static_cast<int>(k_limit - k_first) - 4 * k4 : 0;
    }
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));  // LDS byte address
    // TAIL: where (float index in `lds`), in which slab and from which element on this lane's group runs past K
    int fix_a_at = 0, fix_a_from = 4, fix_a_slab = -1, fix_b_at = 0, fix_b_from = 4, fix_b_slab = -1, issued = 0;
    auto issue_a = [&](int buf) __attribute__((always_inline)) {
        if (TAIL && MODE_A == kKC && krem_a > 0 && krem_a < 4) {
            fix_a_at = buf * kBufFloats + wave * 256 + lane * 4;
            fix_a_from = krem_a;
            fix_a_slab = issued;
        }
        load_to_lds_16(rsrc_a, krem_a > 0 ? off_a : kDirectOob,
                       lds_base + static_cast<uint32_t>(buf * kBufFloats + wave * 256) * 4u);
        off_a += step_a;
        krem_a -= BK;
    };
    auto issue_b = [&](int buf) __attribute__((always_inline)) {
        if (TAIL && MODE_B == kKC && krem_b > 0 && krem_b < 4) {
            fix_b_at = buf * kBufFloats + kOpFloats + wave * 256 + lane * 4;
            fix_b_from = krem_b;
            fix_b_slab = issued;
        }
        load_to_lds_16(rsrc_b, krem_b > 0 ? off_b : kDirectOob,
                       lds_base + static_cast<uint32_t>(buf * kBufFloats + kOpFloats + wave * 256) * 4u);
        off_b += step_b;
        krem_b -= BK;
        ++issued;  // (a slab's A is always issued before its B)
    };
    // called once this lane's loads of `slab` have landed and before the barrier that publishes the slab
    auto zero_tail = [&](int slab) __attribute__((always_inline)) {
        if (!TAIL) return;
        if (MODE_A == kKC && fix_a_slab == slab) {
#pragma unroll
            for (int j = 1; j < 4; ++j)
                if (j >= fix_a_from) lds[fix_a_at + j] = 0.f;
        }
        if (MODE_B == kKC && fix_b_slab == slab) {
#pragma unroll
            for (int j = 1; j < 4; ++j)
                if (j >= fix_b_from) lds[fix_b_at + j] = 0.f;
        }
    };

    // fragment addresses (floats within one operand slab) of this wave's groups q = NQ * kgroup + qq
    int fa_addr[NQ], fb_addr[NQ];
#pragma unroll
    for (int qq = 0; qq < NQ; ++qq) {
        const int q = NQ * kgroup + qq;
        fa_addr[qq] = MODE_A == kXC ? (8 * q + 4 * h) * 64 + wm0 + r : (wm0 + r) * BK + (((2 * q + h) ^ (r & 7)) * 4);
        fb_addr[qq] = MODE_B == kXC ? (8 * q + 4 * h) * 64 + wn0 + r : (wn0 + r) * BK + (((2 * q + h) ^ (r & 7)) * 4);
    }
    float fa[2][NQ][4], fb[2][NQ][4];
    auto read_frag = [&](int f, int buf, int qq) __attribute__((always_inline)) {
        const float *sa = lds + buf * kBufFloats;
        const float *sb = sa + kOpFloats;
        if (MODE_A == kXC) {
#pragma unroll
            for (int j = 0; j < 4; ++j) fa[f][qq][j] = sa[fa_addr[qq] + j * 64];
        } else {
            const v4f v = *reinterpret_cast<const v4f *>(sa + fa_addr[qq]);
#pragma unroll
            for (int j = 0; j < 4; ++j) fa[f][qq][j] = v[j];
        }
        if (MODE_B == kXC) {
#pragma unroll
            for (int j = 0; j < 4; ++j) fb[f][qq][j] = sb[fb_addr[qq] + j * 64];
        } else {
            const v4f v = *reinterpret_cast<const v4f *>(sb + fb_addr[qq]);
#pragma unroll
            for (int j = 0; j < 4; ++j) fb[f][qq][j] = v[j];
        }
    };

    v16f acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;

    // prologue: kDist slabs in flight (slabs past the end load zeros); slab 0's fragments to registers
#pragma unroll
    for (int d = 0; d < kDist; ++d) {
        issue_a(d);
        issue_b(d);
    }
    wait_vmcnt<(kDist - 1) * 2>();
    zero_tail(0);
    __syncthreads();
#pragma unroll
    for (int qq = 0; qq < NQ; ++qq) read_frag(0, 0, qq);

    auto step = [&](const int tb /* t % NBUF */, const int f /* t % 2 */, const int t) __attribute__((always_inline)) {
        wait_vmcnt<(kDist - 2) * 2>();  // all but the youngest slab's two loads: slab t+1 is in LDS
        zero_tail(t + 1);
        __syncthreads();
#pragma unroll
        for (int qq = 0; qq < NQ; ++qq) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[f][qq][j], fb[f][qq][j], acc, 0, 0, 0);
                const int slot = qq * 4 + j;
                if (slot == kSlotA) issue_a((tb + kDist) % NBUF);
                if (slot == kSlotB) issue_b((tb + kDist) % NBUF);
                if (slot % 2 == 0 && slot / 2 < NQ) read_frag(f ^ 1, (tb + 1) % NBUF, slot / 2);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    static_assert(NBUF % 2 == 0, "the fragment register set alternates with the buffer index");
    int t = 0;
    for (; t + NBUF <= n_slabs; t += NBUF) {
#pragma unroll
        for (int d = 0; d < NBUF; ++d) step(d, d & 1, t + d);
    }
#pragma unroll
    for (int d = 0; d < NBUF - 1; ++d)
        if (t + d < n_slabs) step(d, d & 1, t + d);  // uniform across the block

    // the loads still in flight (zeros for slabs past the end) must land before LDS is reused
    wait_vmcnt<0>();
    __syncthreads();
    float *scratch = lds;
    if (kgroup > 0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) scratch[(quad * 16 + v) * 64 + lane] = acc[v];
    }
    __syncthreads();
    if (kgroup > 0) return;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] += scratch[(quad * 16 + v) * 64 + lane];

    // accumulator register v of lane (r, h) is C[8 (v/4) + 4 h + v%4][r] of the wave's 32 x 32 block
    const int64_t col = n0 + wn0 + r;
    const int64_t row0 = m0 + wm0 + 4 * h;
    const bool interior = m0 + BM <= p.M && n0 + BN <= p.N;  // uniform: no per-element bounds tests
    if (p.splits > 1) {  // raw partial tile; gemm_split_finish applies alpha / beta
        // (Adding the partial tiles up in the block that arrives last at a tile, behind an arrival counter, was
        // measured: the device-wide fences it needs write back and invalidate a whole XCD's L2 per block, and the
        // recurrent-net tape ran at half the rate.  The second kernel stays.)
        float *W = static_cast<float *>(p.ws) + (static_cast<int64_t>(blockIdx.z) * gridDim.y + batch) * p.M * p.N +
                   row0 * p.N + col;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int dr = 8 * (v / 4) + (v % 4);
            if (interior || (row0 + dr < p.M && col < p.N)) W[dr * p.N] = acc[v];
        }
        return;
    }
    float *C = static_cast<float *>(p.C) + batch * p.c_bs + row0 * p.ldc + col;
    const float alpha = static_cast<float>(p.alpha), beta = static_cast<float>(p.beta);
    if (p.alpha != 1.0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = alpha * acc[v];
    }
    if (p.beta != 0.0) {
        float old[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int dr = 8 * (v / 4) + (v % 4);
            old[v] = (interior || (row0 + dr < p.M && col < p.N)) ? C[dr * p.ldc] : 0.f;
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = acc[v] + beta * old[v];
    }
    if constexpr (EPI == 2) {
        const bool has_bias = p.epi_bias != nullptr;
        const float bias = (has_bias && col < p.N) ? p.epi_bias[col] : 0.f;
        const float *X = p.epi_x + row0 * p.epi_x_ld + col;
        float xs[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int dr = 8 * (v / 4) + (v % 4);
            xs[v] = (interior || (row0 + dr < p.M && col < p.N)) ? X[dr * p.epi_x_ld] : 0.f;
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = epi_tanh_vjp(acc[v], xs[v], bias, has_bias);
    }
    if (interior) {
#pragma unroll
        for (int v = 0; v < 16; ++v) C[(8 * (v / 4) + (v % 4)) * p.ldc] = acc[v];
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int dr = 8 * (v / 4) + (v % 4);
            if (row0 + dr < p.M && col < p.N) C[dr * p.ldc] = acc[v];
        }
    }
    if constexpr (EPI == 1) {
        const bool has_bias = p.epi_bias != nullptr;
        const float bias = (has_bias && col < p.N) ? p.epi_bias[col] : 0.f;
        float *Y = p.epi_out + row0 * p.epi_ld + col;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int dr = 8 * (v / 4) + (v % 4);
            const float y = epi_tanh(acc[v], bias, has_bias);
            if (interior || (row0 + dr < p.M && col < p.N)) Y[dr * p.epi_ld] = y;
        }
    }
}

// ---- small outputs, long K: the K split inside one block ---------------------------------------------------
//
// A product with few output tiles and a long K (the steps of a recurrent net: 256 x 512 from K = 641) cannot fill the
// machine with one block per 64 x 64 tile; cutting K across blocks does, but leaves partial tiles in memory for a
// second launch to add up, and at this size a launch costs as much as the arithmetic.  Here a block of up to 16 waves
// owns one 32 x 32 tile of C and every wave a slice of K: a wave streams its slice of both operands from global memory
// (they are a few hundred KB and sit in the L2) straight into the matrix core's operand registers, two chunks of
// 32 k in flight, no LDS staging; the waves' accumulators meet in LDS and are added in wave order by the thread that
// then applies alpha / beta or a dense-layer epilogue and stores the element.  One launch, nothing atomic, results
// fixed by the shape.
//
// k order inside a chunk: instruction i of 16 multiplies k = 8 (i / 4) + 4 h + i % 4 for lane half h, so an operand
// that is contiguous along k delivers a lane's four values of a group with one 16-byte load; an operand contiguous
// along its other axis loads 4 bytes per instruction, 128 contiguous bytes per half wave.
constexpr int kSmallTile = 32;
constexpr int kSmallChunk = 32;
constexpr int kSmallMaxWaves = 16;

// An operand contiguous along k: plain 16-byte loads (four 64-bit addresses per chunk).  `row` points at the lane's
// row (or column), `kc + 4 h` is the lane's first k of the chunk; only used where the whole chunk lies inside the slice.
__device__ __forceinline__ void small_load_k(const float *__restrict__ row, int64_t kc, int h, float (&v)[16]) {
    typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const f4 t = *reinterpret_cast<const f4 *>(row + kc + 8 * g + 4 * h);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[4 * g + j] = t[j];
    }
}

// Any other layout, and every operand in the last (partial) chunk of a slice: sixteen 4-byte loads through a buffer
// descriptor.  The address is the descriptor's base + a wave-uniform offset (which k of which chunk: a scalar
// register) + the lane's offset (its row or column and its half's 4 k: ONE vector register per operand) instead of a
// 64-bit vector address per load; that is what lets two chunks of both operands stay in flight inside the 128
// registers a wave of a 1024-thread block may hold.  Offsets past the operand's extent read as zero; k past the
// wave's slice but inside the operand is zeroed by MASK.
template <bool MASK>
__device__ __forceinline__ void small_load_x(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, int64_t ks, int64_t kc, int64_t kend,
                                             int h, float (&v)[16]) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
        v[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                             rsrc, lane_off, static_cast<uint32_t>((kc + 8 * (i / 4) + (i % 4)) * ks * 4), 0));
    if (MASK) {
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = (kc + 8 * (i / 4) + 4 * h + (i % 4) < kend) ? v[i] : 0.f;
    }
}

// (the kernel's body: `bid` is the block's number among the blocks of the problem `p`, `batch` its matrix of the batch)
template <bool KCA, bool KCB>
__device__ __forceinline__ void block_split_tile(const GemmParams &p, const int64_t bid, const int64_t batch, float *part_lds) {
    float (*part)[kSmallTile * kSmallTile] = reinterpret_cast<float (*)[kSmallTile * kSmallTile]>(part_lds);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same for the whole wave: offsets made of it are scalar
    const int r = lane & 31, h = lane >> 5;
    // Workgroups go to the 8 XCDs in turn and each XCD has an L2 of its own: XCD x takes a contiguous range of the
    // tiles in column-major order (a few columns of tiles, every row), so its L2 fetches all of A but only its
    // columns of B, not both operands whole.
    const int64_t n_tiles = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    const int64_t xcd = bid % kXcds, turn = bid / kXcds;
    const int64_t tile = xcd * (n_tiles / kXcds) + min(xcd, n_tiles % kXcds) + turn;
    const int64_t tile_m = tile % p.tiles_m, tile_n = tile / p.tiles_m;
    const int64_t m0 = tile_m * kSmallTile, n0 = tile_n * kSmallTile;
    // One product's share of this wave: the K slice [wave * k_per_split, ...) of A . B into `slot` of the LDS array.
    const auto contract = [&](const float *A, const float *B, int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t K,
                              int64_t k_per_split, uint32_t a_span_bytes, uint32_t b_span_bytes,
                              float *slot) __attribute__((always_inline)) {
        // (the host admits only operands that span less than 2 GiB with non-negative strides: offsets fit 32 bits)
        const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(A), 0, a_span_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(B), 0, b_span_bytes, 0x00020000);
        // rows / columns past the edge read the last one: their products land in elements that are never stored
        const uint32_t a_lane = static_cast<uint32_t>((min(m0 + r, p.M - 1) * a_rs + 4 * h * a_cs) * 4);
        const uint32_t b_lane = static_cast<uint32_t>((min(n0 + r, p.N - 1) * b_cs + 4 * h * b_rs) * 4);
        const float *a_row = A + min(m0 + r, p.M - 1) * a_rs;
        const float *b_col = B + min(n0 + r, p.N - 1) * b_cs;
        const int64_t kbeg = wave * k_per_split, kend = min(K, kbeg + k_per_split);

        v16f acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        float a0[16], b0[16], a1[16], b1[16];
        const auto load = [&](int64_t kc, float (&a)[16], float (&b)[16]) __attribute__((always_inline)) {
            if (kc + kSmallChunk <= kend) {  // the same for the whole wave
                if (KCA) small_load_k(a_row, kc, h, a);
                else small_load_x<false>(rsrc_a, a_lane, a_cs, kc, kend, h, a);
                if (KCB) small_load_k(b_col, kc, h, b);
                else small_load_x<false>(rsrc_b, b_lane, b_rs, kc, kend, h, b);
            } else {
                small_load_x<true>(rsrc_a, a_lane, a_cs, kc, kend, h, a);
                small_load_x<true>(rsrc_b, b_lane, b_rs, kc, kend, h, b);
            }
        };
        const auto multiply = [&](const float (&a)[16], const float (&b)[16]) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < 16; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[i], acc, 0, 0, 0);
        };
        if (kbeg < kend) {
            int64_t k = kbeg;
            load(k, a0, b0);
            while (true) {
                if (k + kSmallChunk < kend) load(k + kSmallChunk, a1, b1);
                multiply(a0, b0);
                k += kSmallChunk;
                if (k >= kend) break;
                if (k + kSmallChunk < kend) load(k + kSmallChunk, a0, b0);
                multiply(a1, b1);
                k += kSmallChunk;
                if (k >= kend) break;
            }
        }
        // accumulator register v of lane (r, h) is C[8 (v/4) + 4 h + v%4][r] of the tile
#pragma unroll
        for (int v = 0; v < 16; ++v) slot[(8 * (v / 4) + 4 * h + (v % 4)) * kSmallTile + r] = acc[v];
    };
    if (wave < p.splits)
        contract(static_cast<const float *>(p.A) + batch * p.a_bs, static_cast<const float *>(p.B) + batch * p.b_bs, p.a_rs, p.a_cs,
                 p.b_rs, p.b_cs, p.K, p.k_per_split, p.a_span_bytes, p.b_span_bytes, part[wave]);
    // A second product of the same shape (the other cotangent of a state that two consumers read) is contracted by the
    // same block into slots of its own: the sum below is then what two launches, the second with beta = 1, would give.
    if (p.A2 != nullptr && wave < p.splits2)
        contract(static_cast<const float *>(p.A2), static_cast<const float *>(p.B2), p.a2_rs, p.a2_cs, p.b2_rs, p.b2_cs, p.K2,
                 p.k_per_split2, p.a2_span_bytes, p.b2_span_bytes, part[p.splits + wave]);
    __syncthreads();

    const float alpha = static_cast<float>(p.alpha), beta = static_cast<float>(p.beta);
    const bool has_bias = p.epi_bias != nullptr;
    for (int e = tid; e < kSmallTile * kSmallTile; e += blockDim.x) {
        const int64_t row = m0 + e / kSmallTile, col = n0 + e % kSmallTile;
        if (row >= p.M || col >= p.N) continue;
        float t = part[0][e];
        for (int w = 1; w < p.splits; ++w) t += part[w][e];
        float *C = static_cast<float *>(p.C) + batch * p.c_bs + row * p.ldc + col;
        if (p.alpha != 1.0) t = alpha * t;
        if (p.beta != 0.0) t = t + beta * *C;
        if (p.A2 != nullptr) {  // (what the first launch would have stored, then the second's sum plus 1 * that)
            const float first = t;
            t = part[p.splits][e];
            for (int w = 1; w < p.splits2; ++w) t += part[p.splits + w][e];
            t = t + 1.0f * first;
        }
        const float bias = has_bias ? p.epi_bias[col] : 0.f;
        if (p.epi == 2) t = epi_tanh_vjp(t, p.epi_x[row * p.epi_x_ld + col], bias, has_bias);
        *C = t;
        if (p.epi == 1) p.epi_out[row * p.epi_ld + col] = epi_tanh(t, bias, has_bias);
    }
}

template <bool KCA, bool KCB>
__global__ __launch_bounds__(kSmallMaxWaves * 64) void gemm_block_split(const GemmParams p) {
    extern __shared__ float part_lds[];  // [waves][32 * 32]
    block_split_tile<KCA, KCB>(p, blockIdx.x, blockIdx.y, part_lds);
}

// Two independent problems in one launch: the first `blocks_p` blocks are the tiles of `p`, the others the tiles of `q`
// (one matrix each).  Every block does exactly what it would do in a launch of its own problem.  For the contraction of
// one time step of a recurrent net and the output head's contraction of the step before, which both wait for the same
// state and not for each other (examples/rnn.py:37-50): one chain link instead of two.
template <bool KCA, bool KCB>
__global__ __launch_bounds__(kSmallMaxWaves * 64) void gemm_block_split_pair(const GemmParams p, const GemmParams q, const int blocks_p) {
    extern __shared__ float part_lds[];
    if (static_cast<int>(blockIdx.x) < blocks_p) block_split_tile<KCA, KCB>(p, blockIdx.x, 0, part_lds);
    else block_split_tile<KCA, KCB>(q, static_cast<int64_t>(blockIdx.x) - blocks_p, 0, part_lds);
}

// Whether a float32 product goes to gemm_block_split: too few 64 x 64 tiles to fill the machine and a K long enough
// to cut, but not so long that one block per 32 x 32 tile would be the slower way to cut it.
static bool wants_block_split(const GemmParams &p, int64_t batch) {
    const int64_t tiles64 = ceil_div(p.M, 64) * ceil_div(p.N, 64) * batch;
    const int64_t tiles32 = ceil_div(p.M, kSmallTile) * ceil_div(p.N, kSmallTile) * batch;
    const int64_t a_span = ((p.M - 1) * p.a_rs + (p.K - 1) * p.a_cs + 1) * 4, b_span = ((p.K - 1) * p.b_rs + (p.N - 1) * p.b_cs + 1) * 4;
    const bool addressable = p.a_rs >= 0 && p.a_cs >= 0 && p.b_rs >= 0 && p.b_cs >= 0 && a_span < 0x7fff0000LL && b_span < 0x7fff0000LL;
    return addressable && tiles64 < 128 && p.K >= 128 && p.K <= 4096 && tiles32 <= 0x7fffffffLL && batch <= 65535;
}

// Tiles, slices and extents of a problem for gemm_block_split; returns the waves a block needs and, in *lds, its LDS bytes.
static int plan_block_split(GemmParams &p, size_t *lds) {
    p.tiles_m = static_cast<int>(ceil_div(p.M, kSmallTile));
    p.tiles_n = static_cast<int>(ceil_div(p.N, kSmallTile));
    // whole chunks per wave (only the slice that holds the end of K has a partial one), as many waves as there are chunks
    const int waves = static_cast<int>(std::min<int64_t>(kSmallMaxWaves, ceil_div(p.K, kSmallChunk)));
    p.splits = waves;
    p.k_per_split = ceil_div(ceil_div(p.K, waves), kSmallChunk) * kSmallChunk;
    p.a_span_bytes = static_cast<uint32_t>(((p.M - 1) * p.a_rs + (p.K - 1) * p.a_cs + 1) * 4);
    p.b_span_bytes = static_cast<uint32_t>(((p.K - 1) * p.b_rs + (p.N - 1) * p.b_cs + 1) * 4);
    int block_waves = waves;
    if (p.A2 != nullptr) {  // the second product of a pair: slices and extents of its own, the same block
        const int waves2 = static_cast<int>(std::min<int64_t>(kSmallMaxWaves, ceil_div(p.K2, kSmallChunk)));
        p.splits2 = waves2;
        p.k_per_split2 = ceil_div(ceil_div(p.K2, waves2), kSmallChunk) * kSmallChunk;
        p.a2_span_bytes = static_cast<uint32_t>(((p.M - 1) * p.a2_rs + (p.K2 - 1) * p.a2_cs + 1) * 4);
        p.b2_span_bytes = static_cast<uint32_t>(((p.K2 - 1) * p.b2_rs + (p.N - 1) * p.b2_cs + 1) * 4);
        block_waves = std::max(waves, waves2);
    }
    *lds = static_cast<size_t>(waves + (p.A2 != nullptr ? p.splits2 : 0)) * kSmallTile * kSmallTile * sizeof(float);
    return block_waves;
}

static void name_block_split(const GemmParams &p, char *text, size_t n) {
    std::snprintf(text, n, "<f32,32,32,%s%s%s>[%lldx%lldx%lld]", p.a_cs == 1 ? "k" : "x", p.b_rs == 1 ? "k" : "x",
                  p.epi == 1 ? ",+bias,tanh" : (p.epi == 2 ? (p.A2 != nullptr ? ",two products,tanh_vjp" : ",tanh_vjp") : ""),
                  (long long)p.M, (long long)p.N, (long long)(p.K + (p.A2 != nullptr ? p.K2 : 0)));
}

static int launch_block_split(GemmParams p, int64_t batch, hipStream_t s) {
    size_t lds = 0;
    const int block_waves = plan_block_split(p, &lds);
    const bool kca = p.a_cs == 1, kcb = p.b_rs == 1;
    char name[160];
    name_block_split(p, name, sizeof(name));
    set_kernel_name("gemm_block_split%s", name);
    const dim3 grid((unsigned)(static_cast<int64_t>(p.tiles_m) * p.tiles_n), (unsigned)batch), block(block_waves * 64);
    if (kca && kcb) hipLaunchKernelGGL((gemm_block_split<true, true>), grid, block, lds, s, p);
    else if (kca) hipLaunchKernelGGL((gemm_block_split<true, false>), grid, block, lds, s, p);
    else if (kcb) hipLaunchKernelGGL((gemm_block_split<false, true>), grid, block, lds, s, p);
    else hipLaunchKernelGGL((gemm_block_split<false, false>), grid, block, lds, s, p);
    return hip_check(hipGetLastError(), "gemm launch");
}

// Two problems that are each gemm_block_split's, with the same operands contiguous along k, in one launch.
static int launch_block_split_pair(GemmParams p, GemmParams q, hipStream_t s) {
    size_t lds_p = 0, lds_q = 0;
    const int waves_p = plan_block_split(p, &lds_p), waves_q = plan_block_split(q, &lds_q);
    const bool kca = p.a_cs == 1, kcb = p.b_rs == 1;
    char name_p[160], name_q[160];
    name_block_split(p, name_p, sizeof(name_p));
    name_block_split(q, name_q, sizeof(name_q));
    set_kernel_name("gemm_block_split_pair%s+%s", name_p, name_q);
    const int64_t blocks_p = static_cast<int64_t>(p.tiles_m) * p.tiles_n, blocks_q = static_cast<int64_t>(q.tiles_m) * q.tiles_n;
    const dim3 grid((unsigned)(blocks_p + blocks_q)), block(std::max(waves_p, waves_q) * 64);
    const size_t lds = std::max(lds_p, lds_q);
    const int bp = static_cast<int>(blocks_p);
    if (kca && kcb) hipLaunchKernelGGL((gemm_block_split_pair<true, true>), grid, block, lds, s, p, q, bp);
    else if (kca) hipLaunchKernelGGL((gemm_block_split_pair<true, false>), grid, block, lds, s, p, q, bp);
    else if (kcb) hipLaunchKernelGGL((gemm_block_split_pair<false, true>), grid, block, lds, s, p, q, bp);
    else hipLaunchKernelGGL((gemm_block_split_pair<false, false>), grid, block, lds, s, p, q, bp);
    return hip_check(hipGetLastError(), "gemm launch");
}

// C = alpha * (sum over splits, in split order) + beta * C
template <typename T>
__global__ __launch_bounds__(kBlock) void gemm_split_finish(const T *__restrict__ ws, T *__restrict__ C, int splits,
                                                            int64_t batch, int64_t M, int64_t N, int64_t ldc, int64_t c_bs,
                                                            T alpha, T beta) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const int64_t per = M * N;
    if (e >= batch * per) return;
    const int64_t b = e / per, r = (e - b * per) / N, c = e - b * per - r * N;
    T acc = ws[e];
    for (int s = 1; s < splits; ++s) acc += ws[static_cast<int64_t>(s) * batch * per + e];
    T *dst = C + b * c_bs + r * ldc + c;
    T v = alpha * acc;
    if (beta != T(0)) v = v + beta * *dst;
    *dst = v;
}

// the same with the dense-layer epilogues (one matrix, alpha = 1, beta = 0)
template <int EPI>
__global__ __launch_bounds__(kBlock) void gemm_split_finish_fused(const float *__restrict__ ws, float *__restrict__ C, int splits,
                                                                  int64_t M, int64_t N, int64_t ldc, const float *bias,
                                                                  float *out, int64_t out_ld, const float *x, int64_t x_ld) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const int64_t per = M * N;
    if (e >= per) return;
    const int64_t r = e / N, c = e - r * N;
    float acc = ws[e];
    for (int s = 1; s < splits; ++s) acc += ws[static_cast<int64_t>(s) * per + e];
    const bool has_bias = bias != nullptr;
    const float b = has_bias ? bias[c] : 0.f;
    if (EPI == 2) acc = epi_tanh_vjp(acc, x[r * x_ld + c], b, has_bias);
    C[r * ldc + c] = acc;
    if (EPI == 1) out[r * out_ld + c] = epi_tanh(acc, b, has_bias);
}

// K == 0: the product is empty, C = beta * C.  Handled apart because the tile kernel's branch-free
// loads read the operand base address for out-of-range elements, and empty operands have none.
template <typename T>
__global__ __launch_bounds__(kBlock) void gemm_empty_k(T *__restrict__ C, int64_t batch, int64_t M, int64_t N, int64_t ldc,
                                                       int64_t c_bs, T beta) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const int64_t per = M * N;
    if (e >= batch * per) return;
    const int64_t b = e / per, r = (e - b * per) / N, c = e - b * per - r * N;
    T *dst = C + b * c_bs + r * ldc + c;
    *dst = beta != T(0) ? beta * *dst : T(0);
}

template <typename T>
static int launch_empty_k(const GemmParams &p, int64_t batch, hipStream_t s) {
    const int64_t n = batch * p.M * p.N;
    set_kernel_name("gemm_empty_k");
    hipLaunchKernelGGL(gemm_empty_k<T>, dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, s, static_cast<T *>(p.C), batch,
                       p.M, p.N, p.ldc, p.c_bs, static_cast<T>(p.beta));
    return hip_check(hipGetLastError(), "gemm launch");
}

template <class MF, int BM, int BN, int BK, int DEPTH, int KS, int MODE_A, int MODE_B>
static void launch_modes(const GemmParams &p, dim3 grid, hipStream_t s) {
    hipLaunchKernelGGL((gemm_mfma<MF, BM, BN, BK, DEPTH, MODE_A, MODE_B, KS>), grid, dim3(kBlock * KS), 0, s, p);
}

template <class MF, int BM, int BN, int BK, int DEPTH, int KS, int MODE_A>
static void launch_mode_b(int mode_b, const GemmParams &p, dim3 grid, hipStream_t s) {
    if (mode_b == kXC)
        launch_modes<MF, BM, BN, BK, DEPTH, KS, MODE_A, kXC>(p, grid, s);
    else if (mode_b == kKC)
        launch_modes<MF, BM, BN, BK, DEPTH, KS, MODE_A, kKC>(p, grid, s);
    else
        launch_modes<MF, BM, BN, BK, DEPTH, KS, MODE_A, kGen>(p, grid, s);
}

static const char *mode_name(int m) { return m == kXC ? "x" : (m == kKC ? "k" : "g"); }

template <class MF, int BM, int BN, int BK, int DEPTH, int KS = 1>
static int launch_gemm(GemmParams p, int64_t batch, hipStream_t s, void *ws = nullptr, size_t ws_bytes = 0) {
    using T = typename MF::elem_t;
    const int64_t tm = ceil_div(p.M, BM), tn = ceil_div(p.N, BN);
    if (tm * tn > 0x7fffffffLL || batch > 65535) {
        set_error("gemm: problem too large for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    p.tiles_m = static_cast<int>(tm);
    p.tiles_n = static_cast<int>(tn);
    // how each operand's 4-element groups lie in memory (see SlabLoader)
    const int mode_a = (p.a_rs == 1 && p.M % 4 == 0) ? kXC : ((p.a_cs == 1 && p.K % 4 == 0) ? kKC : kGen);
    const int mode_b = (p.b_cs == 1 && p.N % 4 == 0) ? kXC : ((p.b_rs == 1 && p.K % 4 == 0) ? kKC : kGen);
    set_kernel_name("gemm_mfma<%s,%d,%d,%d,%s%s>[%lldx%lldx%lld]", sizeof(typename MF::elem_t) == 4 ? "f32" : "f64", BM, BN, BK,
                    mode_name(mode_a), mode_name(mode_b), (long long)p.M, (long long)p.N, (long long)p.K);
    // Few tiles but a long K (skinny outputs, small batches of a recurrent net): cut K across blocks so
    // the machine fills up; partial tiles go to the workspace and are summed in split order.
    p.splits = 1;
    p.k_per_split = ceil_div(p.K, BK) * BK;
    const int64_t tiles = tm * tn * batch;
    if (ws != nullptr && tiles < 128 && p.K >= 8 * BK) {
        int64_t splits = std::min<int64_t>(ceil_div(256, tiles), p.K / (4 * BK));
        splits = std::min<int64_t>(splits, static_cast<int64_t>(ws_bytes / (sizeof(T) * (size_t)(batch * p.M * p.N))));
        splits = std::min<int64_t>(splits, 64);
        if (splits > 1) {
            p.k_per_split = ceil_div(ceil_div(p.K, splits), BK) * BK;
            p.splits = static_cast<int>(ceil_div(p.K, p.k_per_split));
            p.ws = ws;
        }
    }
    const dim3 grid((unsigned)(tm * tn), (unsigned)batch, (unsigned)p.splits);
    if (p.splits > 1)
        set_kernel_name("gemm_mfma<%s,%d,%d,%d,%s%s>+split%d[%lldx%lldx%lld]", sizeof(T) == 4 ? "f32" : "f64", BM, BN, BK,
                        mode_name(mode_a), mode_name(mode_b), p.splits, (long long)p.M, (long long)p.N, (long long)p.K);
    if (mode_a == kXC)
        launch_mode_b<MF, BM, BN, BK, DEPTH, KS, kXC>(mode_b, p, grid, s);
    else if (mode_a == kKC)
        launch_mode_b<MF, BM, BN, BK, DEPTH, KS, kKC>(mode_b, p, grid, s);
    else
        launch_mode_b<MF, BM, BN, BK, DEPTH, KS, kGen>(mode_b, p, grid, s);
    if (int rc = hip_check(hipGetLastError(), "gemm launch")) return rc;
    if (p.splits > 1) {
        const int64_t n = batch * p.M * p.N;
        hipLaunchKernelGGL(gemm_split_finish<T>, dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, s,
                           static_cast<const T *>(p.ws), static_cast<T *>(p.C), p.splits, batch, p.M, p.N, p.ldc,
                           p.c_bs, static_cast<T>(p.alpha), static_cast<T>(p.beta));
    }
    return hip_check(hipGetLastError(), "gemm launch");
}

// Operand layouts gemm_direct accepts: a unit stride along x or k and a positive other stride.  Returns kXC, kKC
// or -1.  Nothing needs 16-byte alignment: the loads take any 4-byte aligned address, the buffer range check is made
// dword by dword (what lies past the operand's last element reads as zero), a group that runs past the last x only
// feeds rows / columns of the tile that are never stored, and a group that runs past the last k is zeroed in LDS
// (the TAIL instantiations).
static int direct_mode(int64_t x_stride, int64_t k_stride, int64_t X, int64_t K) {
    if (x_stride == 1 && (K == 1 || k_stride > 0)) return kXC;
    if (k_stride == 1 && (X == 1 || x_stride > 0)) return kKC;
    return -1;
}

// fp32 product through gemm_direct; returns 1 when the operands do not qualify (nothing launched).
static int launch_direct(GemmParams p, int64_t batch, hipStream_t s, void *ws, size_t ws_bytes) {
    constexpr int BM = 64, BN = 64, BK = 32;
    constexpr int64_t kMaxSpan = 0x7fff0000LL;  // 32-bit byte offsets, with room for the slabs issued past the end
    const int mode_a = direct_mode(p.a_rs, p.a_cs, p.M, p.K);
    const int mode_b = direct_mode(p.b_cs, p.b_rs, p.N, p.K);
    if (mode_a < 0 || mode_b < 0) return 1;
    if (batch > 1 && (p.a_bs < 0 || p.b_bs < 0)) return 1;
    const int64_t a_span = ((p.M - 1) * p.a_rs + (p.K - 1) * p.a_cs + 1) * 4;
    const int64_t b_span = ((p.K - 1) * p.b_rs + (p.N - 1) * p.b_cs + 1) * 4;
    if (a_span > kMaxSpan || b_span > kMaxSpan || BK * p.a_cs * 4 > kMaxSpan || BK * p.b_rs * 4 > kMaxSpan) return 1;
    const int64_t tm = ceil_div(p.M, BM), tn = ceil_div(p.N, BN);
    if (tm * tn > 0x7fffffffLL || batch > 65535) return 1;
    p.a_span_bytes = static_cast<uint32_t>(a_span);
    p.b_span_bytes = static_cast<uint32_t>(b_span);
    p.tiles_m = static_cast<int>(tm);
    p.tiles_n = static_cast<int>(tn);
    p.splits = 1;
    p.k_per_split = ceil_div(p.K, BK) * BK;
    const int64_t tiles = tm * tn * batch;
    if (ws != nullptr && tiles < 128 && p.K >= 8 * BK) {  // few tiles, long K: cut K across blocks
        int64_t splits = std::min<int64_t>(ceil_div(256, tiles), p.K / (4 * BK));
        splits = std::min<int64_t>(splits, static_cast<int64_t>(ws_bytes / (sizeof(float) * (size_t)(batch * p.M * p.N))));
        splits = std::min<int64_t>(splits, 64);
        if (splits > 1) {
            p.k_per_split = ceil_div(ceil_div(p.K, splits), BK) * BK;
            p.splits = static_cast<int>(ceil_div(p.K, p.k_per_split));
            p.ws = ws;
        }
    }
    if (p.splits > 1 && p.epi != 0 && p.beta != 0.0) {
        set_error("gemm_fused: a product cut along K across blocks takes no beta together with an epilogue");
        return AGMI_ERR_UNSUPPORTED;
    }
    if (p.splits > 1)
        set_kernel_name("gemm_direct<f32,64,64,32,%s%s>+split%d[%lldx%lldx%lld]", mode_name(mode_a), mode_name(mode_b), p.splits,
                        (long long)p.M, (long long)p.N, (long long)p.K);
    else
        set_kernel_name("gemm_direct<f32,64,64,32,%s%s%s>[%lldx%lldx%lld]", mode_name(mode_a), mode_name(mode_b),
                        p.epi == 1 ? ",+bias,tanh" : (p.epi == 2 ? ",tanh_vjp" : ""), (long long)p.M, (long long)p.N,
                        (long long)p.K);
    const dim3 grid((unsigned)(tm * tn), (unsigned)batch, (unsigned)p.splits);
    const dim3 block(kDirectThreads);
    const bool tail = p.K % 4 != 0 && (mode_a == kKC || mode_b == kKC);
    // (a product cut along K leaves raw partial tiles; its epilogue runs in the finishing kernel)
    const int epi = p.splits > 1 ? 0 : p.epi;
    const auto launch = [&](auto ma, auto mb, auto tl) {
        constexpr int MA = decltype(ma)::value, MB = decltype(mb)::value;
        constexpr bool TL = decltype(tl)::value;
        if (epi == 1) hipLaunchKernelGGL((gemm_direct<MA, MB, TL, 1>), grid, block, 0, s, p);
        else if (epi == 2) hipLaunchKernelGGL((gemm_direct<MA, MB, TL, 2>), grid, block, 0, s, p);
        else hipLaunchKernelGGL((gemm_direct<MA, MB, TL, 0>), grid, block, 0, s, p);
    };
    using XC = std::integral_constant<int, kXC>;
    using KC = std::integral_constant<int, kKC>;
    using Yes = std::integral_constant<bool, true>;
    using No = std::integral_constant<bool, false>;
    if (mode_a == kXC && mode_b == kXC) launch(XC{}, XC{}, No{});
    else if (mode_a == kXC && tail) launch(XC{}, KC{}, Yes{});
    else if (mode_a == kXC) launch(XC{}, KC{}, No{});
    else if (mode_b == kXC && tail) launch(KC{}, XC{}, Yes{});
    else if (mode_b == kXC) launch(KC{}, XC{}, No{});
    else if (tail) launch(KC{}, KC{}, Yes{});
    else launch(KC{}, KC{}, No{});
    if (int rc = hip_check(hipGetLastError(), "gemm launch")) return rc;
    if (p.splits > 1 && p.epi != 0) {
        const int64_t n = p.M * p.N;
        const dim3 fgrid((unsigned)ceil_div(n, kBlock));
        if (p.epi == 1)
            hipLaunchKernelGGL(gemm_split_finish_fused<1>, fgrid, dim3(kBlock), 0, s, static_cast<const float *>(p.ws),
                               static_cast<float *>(p.C), p.splits, p.M, p.N, p.ldc, p.epi_bias, p.epi_out, p.epi_ld, p.epi_x,
                               p.epi_x_ld);
        else
            hipLaunchKernelGGL(gemm_split_finish_fused<2>, fgrid, dim3(kBlock), 0, s, static_cast<const float *>(p.ws),
                               static_cast<float *>(p.C), p.splits, p.M, p.N, p.ldc, p.epi_bias, p.epi_out, p.epi_ld, p.epi_x,
                               p.epi_x_ld);
        return hip_check(hipGetLastError(), "gemm launch");
    }
    if (p.splits > 1) {
        const int64_t n = batch * p.M * p.N;
        hipLaunchKernelGGL(gemm_split_finish<float>, dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, s,
                           static_cast<const float *>(p.ws), static_cast<float *>(p.C), p.splits, batch, p.M, p.N, p.ldc,
                           p.c_bs, static_cast<float>(p.alpha), static_cast<float>(p.beta));
        return hip_check(hipGetLastError(), "gemm launch");
    }
    return 0;
}

}  // namespace agmi

using namespace agmi;

extern "C" int agmi_gemm(int dtype, int64_t batch, int64_t M, int64_t N, int64_t K, double alpha,
                         const void *A, int64_t a_rs, int64_t a_cs, int64_t a_bs,
                         const void *B, int64_t b_rs, int64_t b_cs, int64_t b_bs,
                         double beta, void *C, int64_t ldc, int64_t c_bs, void *workspace,
                         size_t workspace_bytes, void *stream) {
    if (M < 0 || N < 0 || K < 0 || batch < 0) {
        set_error("gemm: negative extent");
        return AGMI_ERR_ARG;
    }
    if (M == 0 || N == 0 || batch == 0) return 0;
    if (!C || (K > 0 && (!A || !B))) {
        set_error("gemm: null operand");
        return AGMI_ERR_ARG;
    }
    if (ldc < N) {
        set_error("gemm: ldc %lld < N %lld", (long long)ldc, (long long)N);
        return AGMI_ERR_ARG;
    }
    GemmParams p = {};
    p.A = A; p.B = B; p.C = C;
    p.M = M; p.N = N; p.K = K;
    p.a_rs = a_rs; p.a_cs = a_cs; p.a_bs = a_bs;
    p.b_rs = b_rs; p.b_cs = b_cs; p.b_bs = b_bs;
    p.ldc = ldc; p.c_bs = c_bs;
    p.alpha = alpha; p.beta = beta;
    hipStream_t s = as_stream(stream);
    if (batch * M * N > 0x7fffffffLL * kBlock) {
        set_error("gemm: output too large for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    if (K == 0) {
        if (dtype == AGMI_F32) return launch_empty_k<float>(p, batch, s);
        if (dtype == AGMI_F64) return launch_empty_k<double>(p, batch, s);
        set_error("gemm: dtype %d is not a floating type", dtype);
        return AGMI_ERR_ARG;
    }
    if (dtype == AGMI_F32) {
        // 64x64 tiles (the direct-to-LDS kernel): best measured on the 1024-cubed contractions of the MLP
        // workload (one tile per CU).  128x128 tiles only once they alone give every CU two tiles (less L2
        // traffic per flop for large problems) and fill their last round of CUs well enough.
        const int64_t big_tiles = ceil_div(M, 128) * ceil_div(N, 128) * batch;
        // Which tile: measured on full grids, the 128x128 kernel sustains about 117 TFLOP/s and the direct-to-LDS 64x64
        // kernel about 107; each is then scaled by how well its tile count fills whole rounds of the 256 CUs
        // (2944 x 2944: 529 big tiles are 2.07 rounds, i.e. three, 76 TFLOP/s; 2116 small ones are 8.3 rounds).
        const int64_t small_tiles = ceil_div(M, 64) * ceil_div(N, 64) * batch;
        const auto fill = [](int64_t tiles) { return static_cast<double>(tiles) / static_cast<double>(ceil_div(tiles, 256) * 256); };
        const bool prefer_big = big_tiles >= 512 && 117.0 * fill(big_tiles) > 107.0 * fill(small_tiles);
        if (wants_block_split(p, batch)) return launch_block_split(p, batch, s);
        if (!prefer_big) {
            const int rc = launch_direct(p, batch, s, workspace, workspace_bytes);
            if (rc != 1) return rc;  // launched (0) or failed; 1 = operands do not qualify
        }
        if (big_tiles >= 512) return launch_gemm<MfmaF32x32, 128, 128, 16, 2, 1>(p, batch, s);
        return launch_gemm<MfmaF32x32, 64, 64, 32, 2, 2>(p, batch, s, workspace, workspace_bytes);
    }
    if (dtype == AGMI_F64) return launch_gemm<MfmaF64x16, 64, 64, 16, 2, 1>(p, batch, s, workspace, workspace_bytes);
    set_error("gemm: dtype %d is not a floating type", dtype);
    return AGMI_ERR_ARG;
}

extern "C" int agmi_gemm_fused(int dtype, int64_t M, int64_t N, int64_t K, const void *A, int64_t a_rs, int64_t a_cs,
                               const void *B, int64_t b_rs, int64_t b_cs, void *C, int64_t ldc,
                               const agmi_gemm_epilogue *e, void *workspace, size_t workspace_bytes, void *stream) {
    if (!e || (e->kind != AGMI_EPILOGUE_BIAS_TANH && e->kind != AGMI_EPILOGUE_TANH_VJP)) {
        set_error("gemm_fused: unknown epilogue");
        return AGMI_ERR_ARG;
    }
    if (M <= 0 || N <= 0 || K <= 0 || !A || !B || !C || ldc < N) {
        set_error("gemm_fused: empty or null operands");
        return AGMI_ERR_ARG;
    }
    if (e->kind == AGMI_EPILOGUE_BIAS_TANH && (!e->out || e->out_ld < N)) {
        set_error("gemm_fused: the activation needs an output matrix");
        return AGMI_ERR_ARG;
    }
    if (e->kind == AGMI_EPILOGUE_TANH_VJP && (!e->x || e->x_ld < N)) {
        set_error("gemm_fused: the tanh cotangent needs the saved pre-activation");
        return AGMI_ERR_ARG;
    }
    if (dtype != AGMI_F32) {
        set_error("gemm_fused: float32 only");
        return AGMI_ERR_UNSUPPORTED;
    }
    GemmParams p = {};
    p.A = A; p.B = B; p.C = C;
    p.M = M; p.N = N; p.K = K;
    p.a_rs = a_rs; p.a_cs = a_cs;
    p.b_rs = b_rs; p.b_cs = b_cs;
    p.ldc = ldc;
    p.alpha = 1.0; p.beta = e->beta;
    p.epi = e->kind;
    p.epi_bias = static_cast<const float *>(e->bias);
    p.epi_out = static_cast<float *>(e->out);
    p.epi_ld = e->out_ld;
    p.epi_x = static_cast<const float *>(e->x);
    p.epi_x_ld = e->x_ld;
    if (e->with_c != nullptr) {
        // An independent plain product computed by further blocks of the same launch (no second product then).
        GemmParams q = {};
        q.A = e->with_a; q.B = e->with_b; q.C = e->with_c;
        q.M = e->with_m; q.N = e->with_n; q.K = e->with_k;
        q.a_rs = e->with_a_rs; q.a_cs = e->with_a_cs; q.b_rs = e->with_b_rs; q.b_cs = e->with_b_cs;
        q.ldc = e->with_ldc;
        q.alpha = 1.0; q.beta = 0.0;
        if (!e->with_a || !e->with_b || q.M <= 0 || q.N <= 0 || q.K <= 0 || q.ldc < q.N || e->a2 != nullptr || e->b2 != nullptr) {
            set_error("gemm_fused: the accompanying product needs its operands and extents, and excludes a second product");
            return AGMI_ERR_ARG;
        }
        if (!wants_block_split(p, 1) || !wants_block_split(q, 1) || (p.a_cs == 1) != (q.a_cs == 1) || (p.b_rs == 1) != (q.b_rs == 1)) {
            set_error("gemm_fused: the two problems are not both cut inside a block, or differ in which operand is contiguous along k");
            return AGMI_ERR_UNSUPPORTED;
        }
        return launch_block_split_pair(p, q, as_stream(stream));
    }
    if (e->a2 != nullptr || e->b2 != nullptr) {
        // Two products of one shape under one rule, in one launch, exactly when each alone would be cut over the waves
        // of a block in the same way: the launch then gives what the two launches (the second adding to the first)
        // give, bit for bit.  Anything else is the caller's to run one after the other.
        GemmParams q = p;
        q.A = e->a2; q.B = e->b2; q.K = e->k2;
        q.a_rs = e->a2_rs; q.a_cs = e->a2_cs; q.b_rs = e->b2_rs; q.b_cs = e->b2_cs;
        if (!e->a2 || !e->b2 || e->k2 <= 0 || e->kind != AGMI_EPILOGUE_TANH_VJP || e->beta != 0.0) {
            set_error("gemm_fused: a second product needs both operands, the tanh rule and beta = 0");
            return AGMI_ERR_ARG;
        }
        if (!wants_block_split(p, 1) || !wants_block_split(q, 1) || (p.a_cs == 1) != (q.a_cs == 1) || (p.b_rs == 1) != (q.b_rs == 1)) {
            set_error("gemm_fused: the two products are not both cut inside a block, or differ in which operand is contiguous along k");
            return AGMI_ERR_UNSUPPORTED;
        }
        p.A2 = e->a2; p.B2 = e->b2; p.K2 = e->k2;
        p.a2_rs = e->a2_rs; p.a2_cs = e->a2_cs; p.b2_rs = e->b2_rs; p.b2_cs = e->b2_cs;
        return launch_block_split(p, 1, as_stream(stream));
    }
    if (wants_block_split(p, 1)) return launch_block_split(p, 1, as_stream(stream));
    const int rc = launch_direct(p, 1, as_stream(stream), workspace, workspace_bytes);
    if (rc == 1) {
        set_error("gemm_fused: operands outside the direct kernel's layouts (one unit stride each)");
        return AGMI_ERR_UNSUPPORTED;
    }
    return rc;
}
