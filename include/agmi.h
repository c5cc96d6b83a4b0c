/*
 * agmi.h - C ABI of libagmi.so: the MI355X (gfx950) kernels under the VJP/JVP hot path.
 *
 * The reference (HIPS/autograd) is pure Python; the arithmetic of its hot path is the
 * NumPy / SciPy / BLAS call inside each derivative rule.  Each entry point below replaces
 * one family of those calls; the comment on each names the reference call sites it stands
 * in for (paths relative to the reference tree).
 *
 * Conventions
 *  - Every pointer named "device" is GPU memory owned by the caller.  The library never
 *    allocates, frees or synchronises; work is enqueued on `stream` (a hipStream_t passed
 *    as void*, NULL = the default stream) and the call returns immediately.  (One exception,
 *    which agmi_program_specialize(0) switches off: agmi_program compiles a program that it
 *    is handed for the third time and loads the code object; see there.)
 *  - Strides are in ELEMENTS, may be 0 (broadcast axis) and may be negative.
 *  - Return value: 0 on success; AGMI_ERR_* (negative) for a rejected argument, in which
 *    case nothing was launched; a positive value is a hipError_t from the launch.
 *    agmi_last_error() returns a static, thread-local description of the last failure.
 *  - Operands may alias only where a function says so.
 */
#ifndef AGMI_H
#define AGMI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AGMI_MAX_DIMS 8      /* rank accepted at the ABI (before axis merging) */
#define AGMI_MAX_INPUTS 4
#define AGMI_MAX_OUTPUTS 2

#define AGMI_ERR_ARG (-1)          /* null pointer, bad enum, rank > AGMI_MAX_DIMS, negative size */
#define AGMI_ERR_UNSUPPORTED (-2)  /* layout the kernels do not cover (e.g. > 6 unmergeable axes) */
#define AGMI_ERR_WORKSPACE (-3)    /* workspace smaller than agmi_*_workspace_bytes() asked for */

typedef enum agmi_dtype {
    AGMI_F32 = 0,
    AGMI_F64 = 1,
    AGMI_BOOL = 2, /* one byte per element, 0 or 1: comparison results, masks */
    AGMI_I64 = 3,  /* index arrays */
    AGMI_I32 = 4
} agmi_dtype;

/* One strided operand.  data == NULL in an INPUT slot means "scalar passed by value": the
 * value is taken from scalars[slot] and converted to the array dtype (a weak Python scalar
 * in NumPy's promotion rules).
 * An INPUT may carry a pending affine map: its element value is then mem * scale + shift,
 * computed on load as two separately rounded operations (exactly what the NumPy passes
 * `x * scale` and `+ shift` would have produced), so that negation, scalar multiples and
 * scalar offsets of an array (numpy_vjps.py:87, 157; `2 * g`, `1.0 - e` in user code) and
 * products / sums with a BROADCAST operand (`A * b[None, :] + c[:, None]`, a bias added to a
 * matrix product: examples/neural_net.py:34) cost no pass of their own.  `affine` is a bit set;
 * 0 = plain (zero-initialised structs are plain).  A scale or shift that is itself an array is
 * passed as an AUXILIARY input: an extra entry of the `ins` array after the op's own inputs
 * (at most AGMI_MAX_AUX of them per call), named by `scale_slot` / `shift_slot` = its index in
 * `ins`; it is read with its own strides (stride 0 on the axes it is broadcast along).  When several
 * bits are set the steps run in the order of the bit values: * scale, * ins[scale_slot],
 * + shift, + ins[shift_slot].
 * Ignored for outputs and by agmi_gemm / agmi_cast / agmi_compare. */
#define AGMI_AFFINE_SCALE 1u      /* multiply by `scale` */
#define AGMI_AFFINE_SHIFT 2u      /* then add `shift` */
#define AGMI_AFFINE_SCALE_AUX 4u  /* multiply by ins[scale_slot] */
#define AGMI_AFFINE_SHIFT_AUX 8u  /* then add ins[shift_slot] */
#define AGMI_MAX_AUX 2
typedef struct agmi_array {
    void *data;                     /* device pointer to the element at index (0, ..., 0) */
    int64_t strides[AGMI_MAX_DIMS]; /* elements */
    double scale;
    double shift;
    uint32_t affine;
    int32_t scale_slot;
    int32_t shift_slot;
} agmi_array;

/* Elementwise operations.  Unary/binary/ternary ufuncs are the forward primitives
 * (autograd/numpy/numpy_wrapper.py:25-52 wraps numpy.add, numpy.exp, ...); the *_VJP entries
 * are whole derivative rules of autograd/numpy/numpy_vjps.py fused into one pass, with the
 * reference's operation order kept inside. */
typedef enum agmi_op {
    /* one input */
    AGMI_OP_COPY = 0, /* out = x                    (materialise a view / broadcast)          */
    AGMI_OP_NEG,      /* -x                         numpy_vjps.py:157, 87                     */
    AGMI_OP_EXP,
    AGMI_OP_LOG,
    AGMI_OP_TANH,
    AGMI_OP_SINH,
    AGMI_OP_COSH,
    AGMI_OP_SIN,
    AGMI_OP_COS,
    AGMI_OP_SQRT,
    AGMI_OP_SQUARE,
    AGMI_OP_ABS,
    AGMI_OP_SIGN,
    AGMI_OP_RECIPROCAL,
    AGMI_OP_LOG1P,
    AGMI_OP_EXPM1,
    AGMI_OP_EXP2,     /* the rest of the unary ufunc table, numpy_vjps.py:164-182 (forward passes) */
    AGMI_OP_LOG2,
    AGMI_OP_LOG10,
    AGMI_OP_TAN,
    AGMI_OP_ARCSIN,
    AGMI_OP_ARCCOS,
    AGMI_OP_ARCTAN,
    AGMI_OP_ARCSINH,
    AGMI_OP_ARCCOSH,
    AGMI_OP_ARCTANH,
    AGMI_OP_FLOOR,    /* rounding functions: no derivative (numpy_vjps.py:13-20)                   */
    AGMI_OP_CEIL,
    AGMI_OP_RINT,     /* round half to even: numpy.rint, numpy.round(x) with decimals=0            */
    AGMI_OP_TRUNC,
    AGMI_OP_NAN_TO_NUM, /* NaN -> 0, +-inf -> +-largest finite (numpy.nan_to_num defaults), numpy_vjps.py:216 */
    /* two inputs */
    AGMI_OP_ADD = 32, /* also VSpace._add / _mut_add, autograd/core.py:259-264 (out may alias in0) */
    AGMI_OP_SUB,
    AGMI_OP_MUL,      /* y*g, x*g                   numpy_vjps.py:79-83, 163                  */
    AGMI_OP_DIV,      /* g/y                        numpy_vjps.py:91, 126, 166                */
    AGMI_OP_POW,
    AGMI_OP_MAXIMUM,
    AGMI_OP_MINIMUM,
    AGMI_OP_FMAX,     /* NaN-ignoring choosers        numpy_vjps.py:104-113                     */
    AGMI_OP_FMIN,
    AGMI_OP_ARCTAN2,  /* (y, x)                       numpy_vjps.py:131-135                     */
    AGMI_OP_HYPOT,
    AGMI_OP_LOGADDEXP,/* numpy_vjps.py:114-118 */
    AGMI_OP_REMAINDER,/* numpy.mod / numpy.remainder: result takes the sign of the divisor, numpy_vjps.py:128-137 */
    AGMI_OP_LOGADDEXP2,/* log2(2**x + 2**y) the way NumPy evaluates it, numpy_vjps.py:119-123 */
    /* three inputs */
    AGMI_OP_WHERE = 64, /* c != 0 ? x : y  (c in the array dtype)                             */
    /* fused derivative rules; inputs in the order listed */
    AGMI_OP_DIV_VJP1 = 96, /* (g, x, y)      -g * x / y**2            numpy_vjps.py:92, 127       */
    AGMI_OP_TANH_VJP,      /* (g, x)         g / cosh(x)**2           numpy_vjps.py:178           */
    AGMI_OP_POW_VJP0,      /* (g, x, y)      g * y * x**where(y, y-1, 1)   numpy_vjps.py:141      */
    AGMI_OP_POW_VJP1,      /* (g, x, ans)    g * log(where(x, x, 1)) * ans numpy_vjps.py:142      */
    AGMI_OP_LSE_VJP,       /* (g, b, x, ans) g * b * exp(x - ans)     scipy/special.py:123-134    */
    AGMI_OP_RECIPROCAL_VJP,/* (g, x)         -g / x**2                numpy_vjps.py:162           */
    AGMI_OP_SQRT_VJP,      /* (g, x)         g * 0.5 * x**-0.5        numpy_vjps.py:187           */
    AGMI_OP_SIN_VJP,       /* (g, x)         g * cos(x)               numpy_vjps.py:170           */
    AGMI_OP_COS_VJP,       /* (g, x)         -g * sin(x)              numpy_vjps.py:171           */
    AGMI_OP_SINH_VJP,      /* (g, x)         g * cosh(x)              numpy_vjps.py:176           */
    AGMI_OP_COSH_VJP,      /* (g, x)         g * sinh(x)              numpy_vjps.py:177           */
    AGMI_OP_SQUARE_VJP,    /* (g, x)         g * 2 * x                numpy_vjps.py:186           */
    AGMI_OP_ABS_VJP,       /* (g, x, ans)    g * where(x,x,0) / where(ans,ans,1)  numpy_vjps.py:158 */
    AGMI_OP_CHOOSE_VJP,    /* (g, x, ans, y) g * (x==ans) / (1 + (x==y))   numpy_vjps.py:94-113, 911 */
    AGMI_OP_LOG1P_VJP,     /* (g, x)         g / (x + 1)              numpy_vjps.py:169           */
    AGMI_OP_EXPM1_VJP,     /* (g, ans)       (ans + 1) * g            numpy_vjps.py:165           */
    AGMI_OP_DIV_VJP_BOTH,  /* (g, x, y) -> two outputs: g / y and -g * x / y**2  (91-92)          */
    AGMI_OP_MUL_ADD,       /* (a, x, y)      a * x + y  (two roundings; scalar_mul + add)         */
    AGMI_OP_EQUAL_AS_FLOAT,/* (x, y)         1.0 where x == y else 0.0: astype(x == ans, dtype)   numpy_vjps.py:524 */
    AGMI_OP_EXTREMUM_VJP,  /* (g, x, ans, n) g * (x == ans) / n, n = number of positions that attain the
                              extremum of their group (max / min over axes)  numpy_vjps.py:515-530 */
    /* Two arithmetic rules in one instruction of agmi_program (each rounded on its own, as the two separate
     * instructions would be).  An interpreted instruction costs far more in operand moves and dispatch than in
     * arithmetic, so a product that only one sum, difference or product reads travels with its reader.  Programs
     * only: agmi_elementwise and agmi_map_reduce do not know these. */
    AGMI_OP_MUL_MUL,       /* (a, b, c)      (a * b) * c                                           */
    AGMI_OP_MUL_SUB,       /* (a, b, c)      a * b - c                                             */
    AGMI_OP_MUL_RSUB,      /* (a, b, c)      c - a * b                                             */
    AGMI_OP_ADD_MUL,       /* (a, b, c)      (a + b) * c                                           */
    AGMI_OP_SUB_MUL        /* (a, b, c)      (a - b) * c                                           */
} agmi_op;

/* comparison producing AGMI_BOOL: numpy.equal ... (non-differentiable, numpy_vjps.py:13-68) */
typedef enum agmi_cmp { AGMI_EQ = 0, AGMI_NE, AGMI_LT, AGMI_LE, AGMI_GT, AGMI_GE } agmi_cmp;

/* reduction kinds of agmi_map_reduce */
typedef enum agmi_reduce_kind {
    AGMI_RED_SUM = 0, /* numpy.sum: unbroadcast (numpy_vjps.py:883-892), repeat VJP (345-362)   */
    AGMI_RED_MAX,
    AGMI_RED_MIN,
    AGMI_RED_PROD,
    AGMI_RED_LOGSUMEXP /* scipy.special.logsumexp wrapped at autograd/scipy/special.py:120      */
} agmi_reduce_kind;

const char *agmi_last_error(void);
int agmi_version(void);
/* Name of the kernel the calling thread's last entry point launched, e.g. "ew_rows<FMul>"
 * (static storage; for labelling profiles). */
const char *agmi_last_kernel(void);

/* Profiling aid with no counterpart in the reference.  An entry point that launches more than one kernel (the kernel
 * that does the work, then one that adds up partial results) cannot be timed kernel by kernel from outside: events
 * around the call bracket all of them.  agmi_probe_arm makes the NEXT such entry point (agmi_lse_cotangent_fused)
 * record a pair of HIP events on its stream around the FIRST of its kernels and returns the index of that pair;
 * agmi_probe_elapsed waits for the pair and gives the milliseconds between its events (AGMI_ERR_ARG for an index that
 * was armed but never filled, or too old: the library keeps the last 4096 pairs).  Nothing is recorded unless armed. */
int agmi_probe_arm(void);
int agmi_probe_elapsed(int index, float *ms);

/* out[k][idx] = op(in[0][idx], in[1][idx], ...) over the index space `shape` (rank `ndim`).
 * dtype is AGMI_F32 or AGMI_F64 for all operands.  An output may alias an input only when
 * both have identical strides (in-place update: VSpace._mut_add, core.py:262-264).
 * Replaces: one NumPy ufunc pass per arithmetic step of a rule in numpy_vjps.py:76-230. */
int agmi_elementwise(int op, int dtype, int ndim, const int64_t *shape,
                     int n_out, const agmi_array *outs,
                     int n_in, const agmi_array *ins, const double *scalars,
                     void *stream);

/* A chain of elementwise rules evaluated in one pass: out[k][idx] = the value the straight-line
 * program `code` leaves in the register it stores to output k, for every idx of `shape`.
 * The program runs on a file of n_regs registers (at most AGMI_PROGRAM_MAX_REGISTERS) per point.
 * When it starts, register i holds leaves[i][idx] (i < n_leaf: strided arrays, stride 0 on
 * broadcast axes; pending maps are not applied) and register n - 1 - k holds imms[k] converted to
 * `dtype` (k < n_imm; n = 8 when n_regs <= 8, else 16).  Instruction word:
 *     op | dst << 8 | a << 12 | b << 16 | c << 20 | d << 24
 * `op` is any single-result agmi_op: reg[dst] = op(reg[a], reg[b], reg[c], reg[d]) (as many operands
 * as the op takes, in the order agmi_op lists them), rounded exactly as agmi_elementwise rounds
 * it, so a program gives bit for bit what the same ops give as separate agmi_elementwise calls;
 * op AGMI_PROGRAM_STORE writes reg[a] to output b (dst must equal a).  Every register read must
 * have been written, every output stored, else AGMI_ERR_ARG and nothing is launched.
 * Shifted reads (slices of a vector and the zero-padded vectors their cotangents are:
 * x[1:], x[:-1] and `untake`, autograd/numpy/numpy_vjps.py:919-950).  On a one-axis index space a
 * leaf may be a vector read at a shifted position: its `data` then points at the element that
 * index 0 reads (possibly before the vector's first element) and leaf_ranges[2i], leaf_ranges[2i+1]
 * give the indices [lo, hi) at which that address may be dereferenced; outside them the register
 * gets an unspecified finite value, which the program is expected to discard with op
 * AGMI_PROGRAM_MASK: reg[dst] = (mask_ranges[2b] <= idx < mask_ranges[2b+1]) ? reg[a] : reg[c].
 * leaf_ranges may be NULL (every index readable); n_mask <= AGMI_PROGRAM_MAX_MASKS.
 * Row sums (the unbroadcast of a cotangent that a later rule of the same chain reads again, as in the
 * log-softmax of examples/rnn.py:50-52: g - exp(x - lse) * sum(g, axis=1)): AGMI_PROGRAM_ROWSUM sets
 * reg[dst], at every index of a row, to the sum of reg[a] over that row, added up in the order in which
 * agmi_map_reduce adds a row of that length (bit for bit its result).  A program that holds one runs on
 * `shape` as given: exactly two axes, the second at most 512 (float32) / 256 (float64) long and,
 * beyond 64, at least 64 rows (the shapes for which agmi_map_reduce gives a row to a group of lanes);
 * n_regs must be 16, no leaf ranges and no masks; else AGMI_ERR_UNSUPPORTED.  AGMI_PROGRAM_ROWLSE is the
 * same for the logsumexp of a row (autograd/scipy/special.py:119-147: the log-softmax x - logsumexp(x) and its
 * rule g * exp(x - logsumexp(x)) then need no reduction launch of their own), again in agmi_map_reduce's order.
 * Layout: after axis merging at most two axes may remain and every operand must have stride 1 or
 * 0 (leaves only) along the innermost one; anything else returns AGMI_ERR_UNSUPPORTED.  Outputs
 * may not overlap leaves unless they are the same view (in-place update).
 * Replaces: the NumPy passes of consecutive elementwise rules of a backward or forward pass
 * (autograd/numpy/numpy_vjps.py:76-93, 139-143, 157-191; numpy_jvps.py:60-120) together with the
 * cotangent sums between them (autograd/core.py:185-205). */
#define AGMI_PROGRAM_MAX_LEAVES 6
#define AGMI_PROGRAM_MAX_IMMEDIATES 6
#define AGMI_PROGRAM_MAX_OUTPUTS 4
#define AGMI_PROGRAM_MAX_INSTRUCTIONS 96
#define AGMI_PROGRAM_MAX_REGISTERS 16
#define AGMI_PROGRAM_MAX_MASKS 4
#define AGMI_PROGRAM_STORE 255
#define AGMI_PROGRAM_MASK 254
#define AGMI_PROGRAM_ROWSUM 253
#define AGMI_PROGRAM_ROWLSE 252
int agmi_program(int dtype, int ndim, const int64_t *shape, int n_out, const agmi_array *outs,
                 int n_leaf, const agmi_array *leaves, const int64_t *leaf_ranges,
                 int n_imm, const double *imms, int n_mask, const int64_t *mask_ranges,
                 int n_instr, const uint32_t *code, int n_regs, void *stream);

/* Programs that recur are specialised: once agmi_program has been handed the same program (dtype, register
 * count, leaf and immediate counts, instruction words) `after` times on a device, the library writes it out
 * as straight-line HIP over the same functors, compiles it for gfx950 with the run-time compiler (the
 * library's own flags: -ffp-contract=off, no packed float32 forms) and from then on launches that kernel
 * in the interpreter's place: same argument block, same tiling, same bits, no decode and no register moves
 * (config 1's first derivative: 41 us interpreted, 15 us specialised).  Nothing is compiled while the stream
 * records a graph; a program whose compilation fails stays with the interpreter (agmi_last_error says why).
 * agmi_program_specialize sets `after` (0: never; default 3, or AUTOGRAD_AMD_SPECIALIZE from the
 * environment; negative: leave as is) and returns the previous value; agmi_program_specialized reports how
 * many programs have been compiled and how many launches they have served.  No counterpart in the reference
 * (its rules are NumPy calls). */
int agmi_program_specialize(int after);
void agmi_program_specialized(long long *compiled, long long *launches);
/* The HIP source of the kernel a program is specialised to (for inspection and for checking, without a GPU, that
 * it compiles): written to `text` (at most capacity - 1 characters and a terminating zero; may be NULL); returns
 * its full length, or a negative error.  `row_sums`: the program holds AGMI_PROGRAM_ROWSUM. */
long long agmi_program_source(int dtype, int n_leaf, int n_imm, int n_instr, const uint32_t *code, int n_regs,
                              int row_sums, char *text, size_t capacity);

/* out[idx] = (in0[idx] <cmp> in1[idx]) as AGMI_BOOL; inputs as in agmi_elementwise. */
int agmi_compare(int cmp, int dtype, int ndim, const int64_t *shape,
                 const agmi_array *out, const agmi_array *ins, const double *scalars,
                 void *stream);

/* out[idx] = (dst_dtype) in[idx] for any pair of dtypes (numpy astype, numpy_vjps.py:246-251;
 * the dtype=A_dtype casts of dot_adjoint_*, 624, 638). */
int agmi_cast(int src_dtype, int dst_dtype, int ndim, const int64_t *shape,
              const agmi_array *out, const agmi_array *in, void *stream);

/* out[kept idx] = REDUCE over the axes with reduce_axes[d] != 0 of op(in[0][idx], ...).
 * `out->strides` are given for all `ndim` axes and are ignored on reduced axes.  `op` is any
 * single-output agmi_op (AGMI_OP_COPY for a plain reduction).  Deterministic: the summation
 * tree depends only on shapes, never on timing.  Large reductions run in two stages through
 * `workspace` (device memory, at least agmi_map_reduce_workspace_bytes() bytes; may be NULL
 * when that returns 0).
 * Replaces: anp.sum inside unbroadcast (numpy_vjps.py:883-892) fused with the rule that feeds
 * it (x*g then sum: 79-83), numpy.sum/max/min forward, scipy.special.logsumexp forward,
 * the logsumexp JVP (scipy/special.py:137-147), ArrayVSpace._inner_prod (numpy_vspaces.py:36-37),
 * and matrix-vector numpy.dot. */
int agmi_map_reduce(int op, int red, int dtype, int ndim, const int64_t *shape,
                    const uint8_t *reduce_axes, const agmi_array *out,
                    int n_in, const agmi_array *ins, const double *scalars,
                    void *workspace, size_t workspace_bytes, void *stream);
size_t agmi_map_reduce_workspace_bytes(int red, int dtype, int ndim, const int64_t *shape,
                                       const uint8_t *reduce_axes);

/* agmi_map_reduce for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and results as agmi_map_reduce given a roomy workspace (bit for bit: the
 * summation tree is the same), but the partial results of a two-stage reduction are staged in a
 * fixed array of AGMI_STATIC_SCRATCH_BYTES bytes that is part of the library's device image (each
 * GPU the process uses holds its own copy until the process ends).  The call allocates and frees
 * nothing.  A reduction whose partial results need more than that is rejected with
 * AGMI_ERR_WORKSPACE and nothing is launched.  All calls on one GPU share the array: calls that
 * overlap in time (different streams, or graphs replayed concurrently) race; calls on one
 * stream are ordered and safe.  The first call on each GPU looks the array's device address up
 * (hipGetSymbolAddress); make that call outside stream capture. */
#define AGMI_STATIC_SCRATCH_BYTES (1u << 20)
int agmi_map_reduce_static(int op, int red, int dtype, int ndim, const int64_t *shape,
                           const uint8_t *reduce_axes, const agmi_array *out,
                           int n_in, const agmi_array *ins, const double *scalars,
                           void *stream);

/* The cotangent of a row-wise logsumexp together with the rules that consume it, in one pass.
 * With x[r,k] = mem[r,k] * scale * scale_vec + shift + shift_vec (the steps selected by `affine`,
 * AGMI_AFFINE_* bits, in that order, each rounded on its own: a matrix that carries a pending map,
 * e.g. A * b[None, :] + c[:, None]), ans[r] = logsumexp(x[r, :]) and the incoming cotangent g[r],
 *     S[r,k] = g[r] * exp(x[r,k] - ans[r])                      autograd/scipy/special.py:123-134
 * is never written; any of its consumers (null pointer = not wanted) is produced instead:
 *     row_sums[r]  = sum_k S[r,k]              unbroadcast of S to an operand broadcast along the row
 *                                              (add rule, autograd/numpy/numpy_vjps.py:77, 883-892)
 *     scaled[r,k]  = col_factor[k] * S[r,k]    multiply rule for mem * col_factor[None, :] (79)
 *     col_sums[k]  = sum_r mem[r,k] * S[r,k]   multiply rule for the broadcast factor (80-83, 883-892)
 * mem is row-major with unit column stride; scale_vec / shift_vec vary along rows only (column
 * stride 0) or along columns only (row stride 0, column stride 1); cols must be a multiple of the
 * 16-byte vector (4 float32 / 2 float64).  The matrix is cut into tiles of 16 rows by 256 vectors;
 * column sums are staged per band of rows and, when the matrix is more than one tile wide, row
 * sums per tile, in `workspace` (cols * ceil(rows / 16) + rows * ceil(cols / 1024) float32 elements,
 * / 512 for float64; a smaller workspace is met with bands of up to 64 rows) and added in a fixed
 * order by a second kernel; nothing is atomic.  Returns AGMI_ERR_UNSUPPORTED for layouts outside
 * this or a workspace that cannot hold the partial sums (the caller then forms S with
 * AGMI_OP_LSE_VJP and reduces it with agmi_map_reduce). */
typedef struct agmi_lse_cotangent {
    int64_t rows, cols;
    const void *x;              /* mem */
    int64_t x_row_stride;
    uint32_t affine;
    double scale, shift;
    const void *scale_vec;
    int64_t scale_row_stride, scale_col_stride;
    const void *shift_vec;
    int64_t shift_row_stride, shift_col_stride;
    const void *ans;
    int64_t ans_stride;
    const void *g;
    int64_t g_stride;           /* 0: one value for every row */
    void *row_sums;             /* [rows], contiguous */
    const void *col_factor;     /* [cols], contiguous */
    void *scaled;               /* [rows][cols] */
    int64_t scaled_row_stride;
    void *col_sums;             /* [cols], contiguous */
} agmi_lse_cotangent;
int agmi_lse_cotangent_fused(int dtype, const agmi_lse_cotangent *c, void *workspace, size_t workspace_bytes,
                             void *stream);

/* C[m,n] = alpha * sum_k A[m,k] B[k,n] + beta * C[m,n] on the matrix cores (MFMA), dtype
 * AGMI_F32 or AGMI_F64.  A and B are addressed as A[m*a_rs + k*a_cs], B[k*b_rs + n*b_cs], so
 * the transposed operands of the adjoints need no copy; C is row-major with leading
 * dimension ldc.  `batch` independent products with element strides *_bs (batch >= 1).
 * `workspace` (device memory, may be NULL) lets problems with few output tiles and a long K be
 * cut across workgroups along K; partial tiles are then summed in a fixed order (deterministic).
 * Replaces: numpy.dot forward (numpy_wrapper.py:39-40), onp.tensordot in dot_adjoint_0/1
 * (numpy_vjps.py:615-638: G.B^T and A^T.G), matmul adjoints (567-612), tensordot_adjoint_0/1
 * (666-719) after axis permutation. */
int agmi_gemm(int dtype, int64_t batch, int64_t M, int64_t N, int64_t K, double alpha,
              const void *A, int64_t a_rs, int64_t a_cs, int64_t a_bs,
              const void *B, int64_t b_rs, int64_t b_cs, int64_t b_bs,
              double beta, void *C, int64_t ldc, int64_t c_bs,
              void *workspace, size_t workspace_bytes, void *stream);

/* agmi_gemm (float32, one matrix, alpha = 1) with what follows the contraction in a dense layer
 * applied to the accumulators before they are stored, so that the layer costs one launch:
 *   AGMI_EPILOGUE_BIAS_TANH  C = A.B as agmi_gemm stores it, and beside it
 *                            out[m,n] = tanh(C[m,n] + bias[n])          examples/neural_net.py:33-35
 *   AGMI_EPILOGUE_TANH_VJP   C[m,n] = (A.B)[m,n] / cosh(x[m,n] + bias[n])**2: the tanh rule applied to the
 *                            cotangent G.W^T while it is formed          autograd/numpy/numpy_vjps.py:178, 615-624
 * bias may be NULL (nothing is added).  With beta != 0 the product is A.B + beta * C (what C held) before the
 * epilogue: the cotangent that reaches a tanh is often the sum of two such products (the state of a recurrent net is
 * read by the next step and by the output head, examples/rnn.py:37-50; core.py:185-205), the first of which has been
 * stored in C.  Each step is rounded as the separate kernels round it (the bias as a pending `+ bias`, the sum as
 * agmi_gemm's beta, tanh / cosh as AGMI_OP_TANH / AGMI_OP_TANH_VJP), so the results are theirs bit for bit.
 * A and B as in agmi_gemm; each needs one unit stride and byte spans below 2 GiB, else AGMI_ERR_UNSUPPORTED (the
 * caller then runs agmi_gemm and the elementwise kernel). */
#define AGMI_EPILOGUE_BIAS_TANH 1
#define AGMI_EPILOGUE_TANH_VJP 2
typedef struct agmi_gemm_epilogue {
    int32_t kind;
    const void *bias;  /* [N], contiguous, or NULL */
    void *out;         /* BIAS_TANH: [M][N] with leading dimension out_ld */
    int64_t out_ld;
    const void *x;     /* TANH_VJP: [M][N] with leading dimension x_ld */
    int64_t x_ld;
    double beta;       /* 0: C is only written */
    /* TANH_VJP with beta = 0: a second product a2 (M x k2) . b2 (k2 x N) added before the rule (the state of a
     * recurrent net has two readers, examples/rnn.py:37-50: its cotangent is the sum of two G . W^T products,
     * core.py:185-205).  Taken only when each product alone would run on the kernel that cuts K over the waves of one
     * block (AGMI_ERR_UNSUPPORTED otherwise: run them one after the other, the second with beta = 1); the result is
     * bit for bit that of those two launches.  NULL: one product. */
    const void *a2;
    int64_t a2_rs, a2_cs;
    const void *b2;
    int64_t b2_rs, b2_cs;
    int64_t k2;
    /* An independent product with_c (with_m x with_n, leading dimension with_ldc) = with_a . with_b computed by further
     * blocks of the same launch: a second problem that waits for the same inputs and not for this one (the output
     * head of a recurrent net's previous step beside the recurrence of this step, examples/rnn.py:37-50) rides
     * along instead of being a link of the chain of launches.  Taken only when both problems would run on the kernel
     * that cuts K over the waves of one block (AGMI_ERR_UNSUPPORTED otherwise, nothing launched); each result is bit
     * for bit that of its own launch.  with_c NULL: none.  Excludes a2 / b2. */
    const void *with_a;
    int64_t with_a_rs, with_a_cs;
    const void *with_b;
    int64_t with_b_rs, with_b_cs;
    void *with_c;
    int64_t with_ldc, with_m, with_n, with_k;
} agmi_gemm_epilogue;
int agmi_gemm_fused(int dtype, int64_t M, int64_t N, int64_t K,
                    const void *A, int64_t a_rs, int64_t a_cs, const void *B, int64_t b_rs, int64_t b_cs,
                    void *C, int64_t ldc, const agmi_gemm_epilogue *e,
                    void *workspace, size_t workspace_bytes, void *stream);

/* ptr[0..n) = value (vspace zeros/ones, numpy_vspaces.py:21-25; sparse_add's zero fill,
 * core.py:212-215). */
int agmi_fill(int dtype, void *ptr, int64_t n, double value, void *stream);

/* Gather rows: out[i, :] = src[index[i], :] for i in [0, n_index); rows have `inner` elements,
 * src has `n_rows` rows.  Negative indices count from the end; an index outside [-n_rows, n_rows)
 * reads nothing: its output row is NaN (0 for integer dtypes).  Forward of A[idx] with an
 * integer-array idx on the leading axis (numpy_boxes.py:16-18). */
int agmi_take_rows(int dtype, const void *src, int64_t n_rows, int64_t inner,
                   const int64_t *index, int64_t n_index, void *out, void *stream);

/* numpy.concatenate (autograd/numpy/numpy_wrapper.py:58-62, concatenate_args) in one launch: the pieces are
 * strided (outer, extent, inner) views that are laid one after another along the middle axis of the contiguous
 * result (outer, sum of extents, inner).  A piece with all strides 0 is a constant column (the ones that
 * examples/rnn.py:21 appends to its state).  At most AGMI_MAX_CONCAT pieces; none may overlap `out`. */
#define AGMI_MAX_CONCAT 32
typedef struct agmi_concat_piece {
    const void *data;
    int64_t extent;                                   /* along the joined axis */
    int64_t stride_outer, stride_axis, stride_inner;  /* element strides */
} agmi_concat_piece;
int agmi_concat(int dtype, int64_t outer, int64_t inner, int n_pieces, const agmi_concat_piece *pieces,
                void *out, void *stream);

/* out[o, k, c] = src[o, n-1-k, c] on contiguous (outer, n, inner) arrays: numpy.flipud / fliplr / rot90
 * (numpy_vjps.py:202-204) and slices that step backwards, A[::-1] (numpy_boxes.py:16-18), whose
 * NumPy form is a view with a negative stride.  src and out must not overlap. */
int agmi_reverse(int dtype, const void *src, int64_t outer, int64_t n, int64_t inner, void *out,
                 void *stream);

/* numpy.tril (lower != 0) / numpy.triu (lower == 0) with diagonal offset k on contiguous
 * (batch, rows, cols) arrays (numpy_vjps.py:212-213): entries on the other side are written as
 * zeros.  src and out may be the same buffer. */
int agmi_triangle(int dtype, const void *src, int64_t batch, int64_t rows, int64_t cols, int64_t k,
                  int lower, void *out, void *stream);

/* Stable ascending sort of every row of a contiguous (rows, n) array, NaNs last: any of
 *   sorted[r, k]  the k-th smallest element of row r,
 *   order[r, k]   its position in the row (numpy.argsort, kind="stable"),
 *   rank[r, i]    the place element i of the row takes (the inverse permutation)
 * (null pointers are skipped).  Forward of numpy.sort / partition and the permutations their
 * rules route cotangents and tangents through (numpy_vjps.py:773-802, numpy_jvps.py:256-271).
 * n is limited to 65536 (the ranks are found by counting), rows to 65535. */
int agmi_sort_rows(int dtype, const void *src, int64_t rows, int64_t n, void *sorted, int64_t *order,
                   int64_t *rank, void *stream);

/* Running sums along the middle axis of a contiguous (outer, n, inner) array:
 * out[o, k, c] = src[o, 0, c] + ... + src[o, k, c], added in that order (bit-identical to
 * numpy.cumsum).  Forward of numpy.cumsum and, on reversed operands, its cotangent
 * (numpy_vjps.py:533-549).  src and out must not overlap. */
int agmi_cumsum(int dtype, const void *src, int64_t outer, int64_t n, int64_t inner, void *out,
                void *stream);

/* Ordered scatter-add: for i = 0 .. n_index-1 IN THIS ORDER: dst[index[i], :] += src[i, :].
 * Bit-identical to numpy.add.at (numpy_vjps.py:941-950): a destination row that occurs several
 * times receives its addends sequentially in index order.  `order` is the stable argsort of
 * the (wrapped) index values and `seg_start[s] .. seg_start[s+1]` delimit runs of equal
 * destination in that order (n_seg runs); both are device arrays prepared by the caller.
 * seg_start may be NULL: n_seg then counts the index entries and the runs are found on the device
 * (nothing about the index needs to be known on the host: agmi_sort_rows on the index values gives
 * `order`, so a device-resident index can be scattered from inside a recorded graph).
 * An index outside [-n_rows, n_rows) names no row: its addends are dropped. */
int agmi_scatter_add_rows(int dtype, void *dst, int64_t n_rows, int64_t inner,
                          const void *src, const int64_t *index, const int64_t *order,
                          const int64_t *seg_start, int64_t n_seg, void *stream);

/* One fused update of a flat, contiguous parameter vector of n elements: the whole-array NumPy
 * passes of the reference's optimizers (misc/optimizers.py: sgd 40-47, rmsprop 54-59, adam 66-75)
 * in one pass, element arithmetic in the reference's order.
 *   AGMI_OPT_SGD:     s0 = velocity;             hyper = {mass, 1-mass, step_size}
 *   AGMI_OPT_RMSPROP: s0 = avg_sq_grad;          hyper = {gamma, 1-gamma, step_size, eps}
 *   AGMI_OPT_ADAM:    s0 = m, s1 = v;            hyper = {1-b1, b1, 1-b2, b2, 1-b1**t, 1-b2**t, step_size, eps}
 * x_in has dtype x_dtype, g has g_dtype (float32 or float64); the state arrays and x_out are
 * float64, as in the reference (its state starts as np.zeros/np.ones, float64, and NumPy promotion
 * carries that into the parameters).  State is updated in place; x_out may be x_in when x_dtype is
 * float64. */
enum agmi_optimizer { AGMI_OPT_SGD = 0, AGMI_OPT_RMSPROP = 1, AGMI_OPT_ADAM = 2 };
int agmi_optimizer_step(int kind, int x_dtype, int g_dtype, int64_t n, const void *x_in, const void *g,
                        void *s0, void *s1, void *x_out, const double *hyper, void *stream);

/* Sliding-window contraction: the strided window view + einsum of the reference's N-d convolution
 * (scipy/signal.py:45-65; its cotangents, 153-214, are the same contraction on other operands):
 *
 *   out[i, j, p] = sum over d and k of  filter[i, d, k] * signal[j, d, p + k - pad_before]
 *
 * where p, k and pad_before are multi-indices over n_conv <= AGMI_MAX_CONV_DIMS convolved axes,
 * 0 <= k < window, 0 <= p < out_extent, and terms whose signal position falls outside
 * [0, extent) are zero (the reference's explicit zero padding, never written out).  i runs over
 * the filter's free axes (merged to one, filter_batch values), j over the signal's
 * (signal_batch), d over the contracted non-convolved axes (dot).  Strides are in elements and
 * may be negative: an operand read back to front along an axis (the flip of the convolution
 * proper) passes the address of its LAST element on that axis and a negated stride.  Entries of
 * window / extent / pad_before / out_extent / strides beyond n_conv are ignored.  Products are
 * accumulated with fused multiply-adds in the operand type; the summation order is fixed for a
 * given problem shape (no atomics).  float32 and float64 only. */
#define AGMI_MAX_CONV_DIMS 3
typedef struct agmi_window_operand {
    const void *data;
    int64_t batch_stride;
    int64_t dot_stride;
    int64_t strides[AGMI_MAX_CONV_DIMS];
} agmi_window_operand;
typedef struct agmi_correlation {
    int32_t n_conv;
    int64_t filter_batch, signal_batch, dot;
    int64_t window[AGMI_MAX_CONV_DIMS];
    int64_t extent[AGMI_MAX_CONV_DIMS];
    int64_t pad_before[AGMI_MAX_CONV_DIMS];
    int64_t out_extent[AGMI_MAX_CONV_DIMS];
    agmi_window_operand filter, signal;
    void *out;
    int64_t out_filter_stride, out_signal_stride;
    int64_t out_strides[AGMI_MAX_CONV_DIMS];
} agmi_correlation;
int agmi_correlate(int dtype, const agmi_correlation *c, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* AGMI_H */
