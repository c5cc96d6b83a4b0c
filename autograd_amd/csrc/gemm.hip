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
// Workgroup ids are dealt round-robin to the 8 XCDs (each with its own L2), so the tile
// order is remapped: XCD x works on a contiguous range of tiles, walked in column-major
// groups of kGroupM tile-rows, which keeps one XCD's A rows and B columns resident in its L2.
#include "common.h"

namespace agmi {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef double v4d __attribute__((ext_vector_type(4)));

template <typename T>
struct Mfma;

template <>
struct Mfma<float> {
    static constexpr int TM = 32;   // rows = cols of one MFMA block
    static constexpr int TK = 2;    // K depth of one instruction
    static constexpr int NACC = 16; // accumulator registers per lane
    typedef v16f acc_t;
    __device__ __forceinline__ static acc_t mma(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    __device__ __forceinline__ static int d_row(int v, int lane) { return 8 * (v / 4) + 4 * (lane / 32) + (v % 4); }
};

template <>
struct Mfma<double> {
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
};

constexpr int kGroupM = 8;
constexpr int kXcds = 8;

// Copy one K-slab of an operand into LDS as S[k][x] (x = m for A, n for B).
//   xs: element stride along x, ks: element stride along k in global memory.
// Each thread owns LOADS groups of 4 elements: contiguous along x when xs == 1, along k when
// ks == 1 (then written transposed), and falls back to scalar loads otherwise.
template <typename T, int BX, int BK, int LOADS>
struct SlabLoader {
    T reg[LOADS][4];

    __device__ __forceinline__ void load(const T *__restrict__ g, int64_t xs, int64_t ks, int64_t x0, int64_t X,
                                         int64_t k0, int64_t K, int tid) {
        typedef T vec_t __attribute__((ext_vector_type(4), aligned(sizeof(T))));
        if (xs == 1) {  // 4 consecutive x at one k
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const int e = tid + i * kBlock;
                const int kk = e / (BX / 4), xx = (e % (BX / 4)) * 4;
                const int64_t k = k0 + kk, x = x0 + xx;
                if (k < K && x + 3 < X) {
                    const vec_t v = *reinterpret_cast<const vec_t *>(g + k * ks + x);
#pragma unroll
                    for (int j = 0; j < 4; ++j) reg[i][j] = v[j];
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) reg[i][j] = (k < K && x + j < X) ? g[k * ks + x + j] : T(0);
                }
            }
        } else if (ks == 1) {  // 4 consecutive k at one x
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const int e = tid + i * kBlock;
                const int xx = e / (BK / 4), kk = (e % (BK / 4)) * 4;
                const int64_t k = k0 + kk, x = x0 + xx;
                if (x < X && k + 3 < K) {
                    const vec_t v = *reinterpret_cast<const vec_t *>(g + x * xs + k);
#pragma unroll
                    for (int j = 0; j < 4; ++j) reg[i][j] = v[j];
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) reg[i][j] = (x < X && k + j < K) ? g[x * xs + k + j] : T(0);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const int e = tid + i * kBlock;
                const int kk = e / (BX / 4), xx = (e % (BX / 4)) * 4;
                const int64_t k = k0 + kk, x = x0 + xx;
#pragma unroll
                for (int j = 0; j < 4; ++j) reg[i][j] = (k < K && x + j < X) ? g[k * ks + (x + j) * xs] : T(0);
            }
        }
    }

    template <int LDX>
    __device__ __forceinline__ void store(T (*S)[LDX], int64_t xs, int64_t ks, int tid) const {
        if (xs != 1 && ks == 1) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const int e = tid + i * kBlock;
                const int xx = e / (BK / 4), kk = (e % (BK / 4)) * 4;
#pragma unroll
                for (int j = 0; j < 4; ++j) S[kk + j][xx] = reg[i][j];
            }
        } else {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const int e = tid + i * kBlock;
                const int kk = e / (BX / 4), xx = (e % (BX / 4)) * 4;
#pragma unroll
                for (int j = 0; j < 4; ++j) S[kk][xx + j] = reg[i][j];
            }
        }
    }
};

template <typename T, int BM, int BN, int BK>
__global__ __launch_bounds__(kBlock) void gemm_mfma(const GemmParams p) {
    using MF = Mfma<T>;
    constexpr int TM = MF::TM, TK = MF::TK;
    constexpr int WM = BM / 2, WN = BN / 2;      // wave tile
    constexpr int FM = WM / TM, FN = WN / TM;    // MFMA blocks per wave
    constexpr int PAD = 4;
    constexpr int LA = (BM * BK) / (kBlock * 4), LB = (BN * BK) / (kBlock * 4);
    static_assert(LA >= 1 && LB >= 1, "slab too small for 256 threads");
    static_assert(WM % TM == 0 && WN % TM == 0 && BK % TK == 0 && BK % 4 == 0, "tile shape");

    __shared__ T As[2][BK][BM + PAD];
    __shared__ T Bs[2][BK][BN + PAD];

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
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const int64_t m0 = static_cast<int64_t>(tile_m) * BM, n0 = static_cast<int64_t>(tile_n) * BN;
    const int op_x = lane % TM, op_k = lane / TM;

    typename MF::acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < MF::NACC; ++v) acc[i][j][v] = T(0);

    SlabLoader<T, BM, BK, LA> la;
    SlabLoader<T, BN, BK, LB> lb;
    la.load(A, p.a_rs, p.a_cs, m0, p.M, 0, p.K, tid);
    lb.load(B, p.b_cs, p.b_rs, n0, p.N, 0, p.K, tid);
    la.template store<BM + PAD>(As[0], p.a_rs, p.a_cs, tid);
    lb.template store<BN + PAD>(Bs[0], p.b_cs, p.b_rs, tid);
    __syncthreads();

    const int64_t n_slabs = (p.K + BK - 1) / BK;
    for (int64_t t = 0; t < n_slabs; ++t) {
        const int cur = t & 1;
        if (t + 1 < n_slabs) {
            la.load(A, p.a_rs, p.a_cs, m0, p.M, (t + 1) * BK, p.K, tid);
            lb.load(B, p.b_cs, p.b_rs, n0, p.N, (t + 1) * BK, p.K, tid);
        }
#pragma unroll
        for (int kk = 0; kk < BK; kk += TK) {
            T a[FM], b[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) a[i] = As[cur][kk + op_k][wm0 + i * TM + op_x];
#pragma unroll
            for (int j = 0; j < FN; ++j) b[j] = Bs[cur][kk + op_k][wn0 + j * TM + op_x];
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] = MF::mma(a[i], b[j], acc[i][j]);
        }
        if (t + 1 < n_slabs) {
            la.template store<BM + PAD>(As[cur ^ 1], p.a_rs, p.a_cs, tid);
            lb.template store<BN + PAD>(Bs[cur ^ 1], p.b_cs, p.b_rs, tid);
        }
        __syncthreads();
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

template <typename T, int BM, int BN, int BK>
static int launch_gemm(GemmParams p, int64_t batch, hipStream_t s) {
    const int64_t tm = ceil_div(p.M, BM), tn = ceil_div(p.N, BN);
    if (tm * tn > 0x7fffffffLL || batch > 65535) {
        set_error("gemm: problem too large for one launch");
        return AGMI_ERR_UNSUPPORTED;
    }
    p.tiles_m = static_cast<int>(tm);
    p.tiles_n = static_cast<int>(tn);
    set_kernel_name("gemm_mfma<%s,%d,%d,%d>", sizeof(T) == 4 ? "f32" : "f64", BM, BN, BK);
    hipLaunchKernelGGL((gemm_mfma<T, BM, BN, BK>), dim3((unsigned)(tm * tn), (unsigned)batch), dim3(kBlock), 0, s, p);
    return hip_check(hipGetLastError(), "gemm launch");
}

}  // namespace agmi

using namespace agmi;

extern "C" int agmi_gemm(int dtype, int64_t batch, int64_t M, int64_t N, int64_t K, double alpha,
                         const void *A, int64_t a_rs, int64_t a_cs, int64_t a_bs,
                         const void *B, int64_t b_rs, int64_t b_cs, int64_t b_bs,
                         double beta, void *C, int64_t ldc, int64_t c_bs, void *stream) {
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
    if (dtype == AGMI_F32) {
        // 128x128 tiles once they alone give every CU work, 64x64 otherwise
        const int64_t big_tiles = ceil_div(M, 128) * ceil_div(N, 128) * batch;
        if (big_tiles >= 256) return launch_gemm<float, 128, 128, 16>(p, batch, s);
        return launch_gemm<float, 64, 64, 16>(p, batch, s);
    }
    if (dtype == AGMI_F64) return launch_gemm<double, 64, 64, 16>(p, batch, s);
    set_error("gemm: dtype %d is not a floating type", dtype);
    return AGMI_ERR_ARG;
}
