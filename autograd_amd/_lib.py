"""ctypes binding of ``libagmi.so`` (the C ABI declared in ``include/agmi.h``).

This module is the only place that touches the native library.  Everything above
it works with ``torch.Tensor`` objects, which are used purely as device-memory
handles (allocation through torch's caching allocator, views as metadata,
``data_ptr()`` + element strides handed to the kernels, launches on torch's
current HIP stream).  No arithmetic is ever done by torch.

There is NO fallback: if the library is missing or a launch is rejected, the
call raises.
"""

import ctypes
import os
import sys

import numpy as onp
import torch

_HERE = os.path.dirname(os.path.abspath(sys.modules[__name__.rsplit(".", 1)[0]].__file__))  # the package's folder, wherever this module was loaded from
LIB_PATH = os.environ.get("AGMI_LIBRARY", os.path.join(_HERE, "libagmi.so"))

MAX_DIMS = 8
MAX_IN = 4
MAX_AUX = 2  # auxiliary operands (array-valued factors / offsets of pending maps) per launch
MAX_OUT = 2

# agmi_dtype
F32, F64, BOOL, I64, I32 = 0, 1, 2, 3, 4
DTYPE_CODE = {
    onp.dtype("float32"): F32,
    onp.dtype("float64"): F64,
    onp.dtype("bool"): BOOL,
    onp.dtype("int64"): I64,
    onp.dtype("int32"): I32,
}
TORCH_DTYPE = {
    onp.dtype("float32"): torch.float32,
    onp.dtype("float64"): torch.float64,
    onp.dtype("bool"): torch.bool,
    onp.dtype("int64"): torch.int64,
    onp.dtype("int32"): torch.int32,
}
NUMPY_DTYPE = {v: k for k, v in TORCH_DTYPE.items()}


# agmi_op (values fixed by include/agmi.h)
class Op:
    COPY, NEG, EXP, LOG, TANH, SINH, COSH, SIN, COS, SQRT, SQUARE, ABS, SIGN, RECIPROCAL, LOG1P, EXPM1 = range(16)
    EXP2, LOG2, LOG10, TAN, ARCSIN, ARCCOS, ARCTAN, ARCSINH, ARCCOSH, ARCTANH = range(16, 26)
    FLOOR, CEIL, RINT, TRUNC, NAN_TO_NUM = range(26, 31)
    ADD, SUB, MUL, DIV, POW, MAXIMUM, MINIMUM, FMAX, FMIN, ARCTAN2, HYPOT, LOGADDEXP, REMAINDER, LOGADDEXP2 = range(32, 46)
    WHERE = 64
    (
        DIV_VJP1,
        TANH_VJP,
        POW_VJP0,
        POW_VJP1,
        LSE_VJP,
        RECIPROCAL_VJP,
        SQRT_VJP,
        SIN_VJP,
        COS_VJP,
        SINH_VJP,
        COSH_VJP,
        SQUARE_VJP,
        ABS_VJP,
        CHOOSE_VJP,
        LOG1P_VJP,
        EXPM1_VJP,
        DIV_VJP_BOTH,
        MUL_ADD,
        EQUAL_AS_FLOAT,
        EXTREMUM_VJP,
        MUL_MUL,   # the last five: two rules in one program instruction (programs only)
        MUL_SUB,
        MUL_RSUB,
        ADD_MUL,
        SUB_MUL,
    ) = range(96, 121)


class Cmp:
    EQ, NE, LT, LE, GT, GE = range(6)


class Red:
    SUM, MAX, MIN, PROD, LOGSUMEXP = range(5)


# ops agmi_map_reduce can fuse in front of a sum (reduce.hip: AGMI_FOR_EACH_REDUCE_OP)
REDUCE_FUSABLE = frozenset(
    {Op.COPY, Op.NEG, Op.MUL, Op.DIV, Op.SQUARE, Op.ABS, Op.DIV_VJP1, Op.TANH_VJP, Op.POW_VJP0, Op.POW_VJP1,
     Op.LSE_VJP, Op.CHOOSE_VJP, Op.EQUAL_AS_FLOAT}
)


class AgmiArray(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("strides", ctypes.c_int64 * MAX_DIMS), ("scale", ctypes.c_double),
                ("shift", ctypes.c_double), ("affine", ctypes.c_uint32), ("scale_slot", ctypes.c_int32),
                ("shift_slot", ctypes.c_int32)]


class AgmiWindowOperand(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("batch_stride", ctypes.c_int64), ("dot_stride", ctypes.c_int64),
                ("strides", ctypes.c_int64 * 3)]


class AgmiCorrelation(ctypes.Structure):
    _fields_ = [("n_conv", ctypes.c_int32), ("filter_batch", ctypes.c_int64), ("signal_batch", ctypes.c_int64),
                ("dot", ctypes.c_int64), ("window", ctypes.c_int64 * 3), ("extent", ctypes.c_int64 * 3),
                ("pad_before", ctypes.c_int64 * 3), ("out_extent", ctypes.c_int64 * 3),
                ("filter", AgmiWindowOperand), ("signal", AgmiWindowOperand), ("out", ctypes.c_void_p),
                ("out_filter_stride", ctypes.c_int64), ("out_signal_stride", ctypes.c_int64),
                ("out_strides", ctypes.c_int64 * 3)]


class AgmiGemmEpilogue(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("bias", ctypes.c_void_p), ("out", ctypes.c_void_p), ("out_ld", ctypes.c_int64),
                ("x", ctypes.c_void_p), ("x_ld", ctypes.c_int64), ("beta", ctypes.c_double),
                ("a2", ctypes.c_void_p), ("a2_rs", ctypes.c_int64), ("a2_cs", ctypes.c_int64),
                ("b2", ctypes.c_void_p), ("b2_rs", ctypes.c_int64), ("b2_cs", ctypes.c_int64), ("k2", ctypes.c_int64),
                ("with_a", ctypes.c_void_p), ("with_a_rs", ctypes.c_int64), ("with_a_cs", ctypes.c_int64),
                ("with_b", ctypes.c_void_p), ("with_b_rs", ctypes.c_int64), ("with_b_cs", ctypes.c_int64),
                ("with_c", ctypes.c_void_p), ("with_ldc", ctypes.c_int64), ("with_m", ctypes.c_int64),
                ("with_n", ctypes.c_int64), ("with_k", ctypes.c_int64)]


class AgmiLseCotangent(ctypes.Structure):
    _fields_ = [("rows", ctypes.c_int64), ("cols", ctypes.c_int64), ("x", ctypes.c_void_p), ("x_row_stride", ctypes.c_int64),
                ("affine", ctypes.c_uint32), ("scale", ctypes.c_double), ("shift", ctypes.c_double),
                ("scale_vec", ctypes.c_void_p), ("scale_row_stride", ctypes.c_int64), ("scale_col_stride", ctypes.c_int64),
                ("shift_vec", ctypes.c_void_p), ("shift_row_stride", ctypes.c_int64), ("shift_col_stride", ctypes.c_int64),
                ("ans", ctypes.c_void_p), ("ans_stride", ctypes.c_int64), ("g", ctypes.c_void_p), ("g_stride", ctypes.c_int64),
                ("row_sums", ctypes.c_void_p), ("col_factor", ctypes.c_void_p), ("scaled", ctypes.c_void_p),
                ("scaled_row_stride", ctypes.c_int64), ("col_sums", ctypes.c_void_p)]


class Affine:
    """Kernel input slot ``t * scale * ascale + shift``, applied on load in that order, each step
    rounded on its own.  ``scale`` is a Python float (1.0: no multiply); ``ascale`` is None or a tensor
    of ``t``'s shape (a broadcast view); ``shift`` is None (no add), a Python float or such a tensor."""

    __slots__ = ("t", "scale", "shift", "ascale")

    def __init__(self, t, scale, shift, ascale=None):
        self.t, self.scale, self.shift, self.ascale = t, scale, shift, ascale


class AgmiError(RuntimeError):
    pass


_LIB = None


def lib():
    """Load ``libagmi.so`` once.  Raises ImportError when it has not been built."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: the HIP library is not built. Run `make -C autograd_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`). There is no CPU fallback."
        )
    L = ctypes.CDLL(LIB_PATH)
    c_i, c_i64, c_d, c_p, c_sz = ctypes.c_int, ctypes.c_int64, ctypes.c_double, ctypes.c_void_p, ctypes.c_size_t
    p_i64 = ctypes.POINTER(ctypes.c_int64)
    p_arr = ctypes.POINTER(AgmiArray)
    p_d = ctypes.POINTER(ctypes.c_double)
    p_u8 = ctypes.POINTER(ctypes.c_uint8)
    L.agmi_last_error.restype = ctypes.c_char_p
    L.agmi_last_error.argtypes = []
    L.agmi_version.restype = c_i
    L.agmi_version.argtypes = []
    L.agmi_last_kernel.restype = ctypes.c_char_p
    L.agmi_last_kernel.argtypes = []
    L.agmi_probe_arm.restype = ctypes.c_int
    L.agmi_probe_arm.argtypes = []
    L.agmi_probe_elapsed.restype = ctypes.c_int
    L.agmi_probe_elapsed.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
    L.agmi_elementwise.restype = c_i
    L.agmi_elementwise.argtypes = [c_i, c_i, c_i, p_i64, c_i, p_arr, c_i, p_arr, p_d, c_p]
    L.agmi_program.restype = c_i
    L.agmi_program.argtypes = [c_i, c_i, p_i64, c_i, p_arr, c_i, p_arr, p_i64, c_i, p_d, c_i, p_i64, c_i,
                               ctypes.POINTER(ctypes.c_uint32), c_i, c_p]
    L.agmi_program_specialize.restype = c_i
    L.agmi_program_specialize.argtypes = [c_i]
    L.agmi_program_specialized.restype = None
    L.agmi_program_specialized.argtypes = [ctypes.POINTER(ctypes.c_longlong), ctypes.POINTER(ctypes.c_longlong)]
    L.agmi_program_source.restype = ctypes.c_longlong
    L.agmi_program_source.argtypes = [c_i, c_i, c_i, c_i, ctypes.POINTER(ctypes.c_uint32), c_i, c_i, ctypes.c_char_p, ctypes.c_size_t]
    L.agmi_compare.restype = c_i
    L.agmi_compare.argtypes = [c_i, c_i, c_i, p_i64, p_arr, p_arr, p_d, c_p]
    L.agmi_cast.restype = c_i
    L.agmi_cast.argtypes = [c_i, c_i, c_i, p_i64, p_arr, p_arr, c_p]
    L.agmi_map_reduce.restype = c_i
    L.agmi_map_reduce.argtypes = [c_i, c_i, c_i, c_i, p_i64, p_u8, p_arr, c_i, p_arr, p_d, c_p, c_sz, c_p]
    L.agmi_map_reduce_static.restype = c_i
    L.agmi_map_reduce_static.argtypes = [c_i, c_i, c_i, c_i, p_i64, p_u8, p_arr, c_i, p_arr, p_d, c_p]
    L.agmi_map_reduce_workspace_bytes.restype = c_sz
    L.agmi_map_reduce_workspace_bytes.argtypes = [c_i, c_i, c_i, p_i64, p_u8]
    L.agmi_gemm.restype = c_i
    L.agmi_gemm.argtypes = [c_i, c_i64, c_i64, c_i64, c_i64, c_d, c_p, c_i64, c_i64, c_i64, c_p, c_i64, c_i64,
                            c_i64, c_d, c_p, c_i64, c_i64, c_p, c_sz, c_p]
    L.agmi_gemm_fused.restype = c_i
    L.agmi_gemm_fused.argtypes = [c_i, c_i64, c_i64, c_i64, c_p, c_i64, c_i64, c_p, c_i64, c_i64, c_p, c_i64,
                                  ctypes.POINTER(AgmiGemmEpilogue), c_p, c_sz, c_p]
    L.agmi_fill.restype = c_i
    L.agmi_fill.argtypes = [c_i, c_p, c_i64, c_d, c_p]
    L.agmi_reverse.restype = c_i
    L.agmi_reverse.argtypes = [c_i, c_p, c_i64, c_i64, c_i64, c_p, c_p]
    L.agmi_triangle.restype = c_i
    L.agmi_triangle.argtypes = [c_i, c_p, c_i64, c_i64, c_i64, c_i64, c_i, c_p, c_p]
    L.agmi_sort_rows.restype = c_i
    L.agmi_sort_rows.argtypes = [c_i, c_p, c_i64, c_i64, c_p, c_p, c_p, c_p]
    L.agmi_cumsum.restype = c_i
    L.agmi_cumsum.argtypes = [c_i, c_p, c_i64, c_i64, c_i64, c_p, c_p]
    L.agmi_concat.restype = c_i
    L.agmi_concat.argtypes = [c_i, c_i64, c_i64, c_i, c_p, c_p, c_p]
    L.agmi_take_rows.restype = c_i
    L.agmi_take_rows.argtypes = [c_i, c_p, c_i64, c_i64, c_p, c_i64, c_p, c_p]
    L.agmi_scatter_add_rows.restype = c_i
    L.agmi_scatter_add_rows.argtypes = [c_i, c_p, c_i64, c_i64, c_p, c_p, c_p, c_p, c_i64, c_p]
    L.agmi_optimizer_step.restype = c_i
    L.agmi_optimizer_step.argtypes = [c_i, c_i, c_i, c_i64, c_p, c_p, c_p, c_p, c_p, p_d, c_p]
    L.agmi_lse_cotangent_fused.restype = c_i
    L.agmi_lse_cotangent_fused.argtypes = [c_i, ctypes.POINTER(AgmiLseCotangent), c_p, c_sz, c_p]
    L.agmi_correlate.restype = c_i
    L.agmi_correlate.argtypes = [c_i, ctypes.POINTER(AgmiCorrelation), c_p]
    _LIB = L
    return L


EXPORTS = (
    "agmi_last_error agmi_version agmi_last_kernel agmi_elementwise agmi_program agmi_compare agmi_cast agmi_map_reduce "
    "agmi_map_reduce_workspace_bytes agmi_map_reduce_static agmi_gemm agmi_gemm_fused agmi_fill agmi_take_rows agmi_sort_rows agmi_cumsum agmi_reverse agmi_triangle agmi_scatter_add_rows agmi_optimizer_step "
    "agmi_correlate agmi_lse_cotangent_fused agmi_concat agmi_probe_arm agmi_probe_elapsed "
    "agmi_program_specialize agmi_program_specialized agmi_program_source"
).split()


def _check(rc, what):
    if rc != 0:
        msg = lib().agmi_last_error().decode("utf-8", "replace")
        raise AgmiError(f"{what} failed (code {rc}): {msg}")


# ---- device / stream ---------------------------------------------------------------------
_DEVICE = None


def device():
    """The GPU all device arrays live on.  Raises when no GPU is visible."""
    global _DEVICE
    if _DEVICE is None:
        if not torch.cuda.is_available():
            raise RuntimeError(
                "autograd_amd needs an AMD GPU (MI355X / gfx950) visible to PyTorch-ROCm; none found. "
                "There is no CPU fallback."
            )
        _DEVICE = torch.device("cuda", torch.cuda.current_device())
        lib()
    return _DEVICE


def _stream():
    return torch._C._cuda_getCurrentRawStream(_DEVICE.index)


def empty(shape, np_dtype):
    return torch.empty(tuple(shape), dtype=TORCH_DTYPE[np_dtype], device=device())


def synchronize():
    torch.cuda.synchronize(device())


# True while a HIP graph is being recorded: only kernel launches are legal then
CAPTURING = False


def check_not_capturing(what):
    if CAPTURING:
        raise RuntimeError(
            f"{what} moves data between host and device, which cannot be recorded into a HIP graph; "
            "do it outside the captured function"
        )


# ---- optional per-launch timing (HIP events on the launch stream) ------------------------------
class KernelTimer:
    """Times launches with HIP events recorded on the stream the kernels run on.

    ``with KernelTimer() as kt: ...`` brackets every launch whose ``(entry point, op)`` key is in
    ``only`` (all launches when ``only`` is None; every ``every``-th of them when that is given: an event pair costs
    the host a few microseconds and delays the launch behind it).  ``summary()`` (after a device synchronise)
    gives, per kernel name, the launch count, the average duration and the average algorithmic
    traffic: every distinct input element read once plus every output element written once
    (2*M*N*K flops for a contraction).
    """

    def __init__(self, only=None, events=0, every=1):
        self.only = only
        self.every, self._seen = every, 0  # `every` = n: only every n-th matching launch carries events
        self.records = []
        self._traffic = {}  # (key, shape of the first result) -> algorithmic bytes, computed once
        # events made ahead of time keep the cost inside a timed region to the two records per launch
        self._spare = [torch.cuda.Event(enable_timing=True) for _ in range(events)]
        self._stream = None

    def __enter__(self):
        global _TIMER
        self._prev, _TIMER = _TIMER, self
        self._stream = torch.cuda.current_stream(device())
        for ev in self._spare:  # the underlying HIP event is only created by the first record: do that now
            ev.record(self._stream)
        return self

    def __exit__(self, *exc):
        global _TIMER
        _TIMER = self._prev

    def _event(self):
        ev = self._spare.pop() if self._spare else torch.cuda.Event(enable_timing=True)
        ev.record(self._stream)
        return ev

    def begin(self, key):
        if self.only is not None and key not in self.only:
            return None
        if self.every > 1:
            self._seen += 1
            if self._seen % self.every:
                return None
        return self._event()

    def end(self, ev0, key, nbytes, flops=0.0, probe=None):
        """``nbytes``: the algorithmic bytes, or ``(outs, ins)`` to have them counted (once per key and shape).
        ``probe``: index of the event pair the library itself recorded around the first kernel of an entry point that
        launches several (``agmi_probe_arm``): that pair gives the kernel's duration, this one the whole call's."""
        ev1 = self._event()
        if type(nbytes) is tuple:
            outs, ins = nbytes
            if self.only is None:
                nbytes = _traffic(outs, ins)
            else:  # a few selected kernels of a step that repeats: count once per key and shape
                sig = (key, tuple(outs[0].shape))
                nbytes = self._traffic.get(sig)
                if nbytes is None:
                    nbytes = self._traffic[sig] = _traffic(outs, ins)
        name = _LIB.agmi_last_kernel().decode()
        self.records.append((name, key, ev0, ev1, nbytes, flops, probe))

    def summary(self):
        synchronize()
        out = {}
        took = ctypes.c_float()
        for name, key, ev0, ev1, nbytes, flops, probe in self.records:
            r = out.setdefault(name, {"key": key, "launches": 0, "ms": 0.0, "bytes": 0.0, "flops": 0.0, "call_ms": 0.0})
            r["launches"] += 1
            whole = ev0.elapsed_time(ev1)
            if probe is not None and _LIB.agmi_probe_elapsed(probe, ctypes.byref(took)) == 0:
                r["ms"] += took.value   # the named kernel alone
                r["call_ms"] += whole   # the entry point's call: that kernel and the one that adds up its partial results
            else:
                r["ms"] += whole
                r["call_ms"] += whole
            r["bytes"] += nbytes
            r["flops"] += flops
        for r in out.values():
            n = r["launches"]
            r["avg_ms"], r["avg_bytes"], r["avg_flops"] = r["ms"] / n, r["bytes"] / n, r["flops"] / n
            r["avg_call_ms"] = r["call_ms"] / n
        return out


_TIMER = None


class untimed:
    """``with untimed(): ...``: launches inside are not seen by the active ``KernelTimer`` (filler work of a
    measurement, for instance)."""

    def __enter__(self):
        global _TIMER
        self._prev, _TIMER = _TIMER, None

    def __exit__(self, *exc):
        global _TIMER
        _TIMER = self._prev


def _distinct_bytes(t):
    n = 1
    for extent, stride in zip(t.shape, t.stride()):
        if stride != 0:
            n *= extent
    return n * t.element_size()


def _traffic(outs, ins):
    """Algorithmic bytes of a launch: every result element written once, every distinct operand element read once
    (views of one storage, such as a vector read at several shifts, count as the stretch of memory they cover
    together, not once each)."""
    total = 0
    for t in outs:
        total += t.numel() * t.element_size()
    by_storage = {}

    def read(t):
        es = t.element_size()
        begin = t.data_ptr()
        span = 1
        for extent, stride in zip(t.shape, t.stride()):
            if extent == 0:
                return
            span += (extent - 1) * abs(stride)
        entry = by_storage.setdefault(begin - t.storage_offset() * es, [0, begin, begin])
        entry[0] += _distinct_bytes(t)
        entry[1] = min(entry[1], begin)
        entry[2] = max(entry[2], begin + span * es)

    for t in ins:
        if type(t) is Affine:
            for aux in (t.ascale, t.shift):
                if isinstance(aux, torch.Tensor):
                    read(aux)
            t = t.t
        if isinstance(t, torch.Tensor):
            read(t)
    for distinct, begin, end in by_storage.values():
        total += min(distinct, end - begin)
    return total


# ---- argument marshalling (buffers reused: single-threaded by contract) ----------------------
_outs = (AgmiArray * MAX_OUT)()
_ins = (AgmiArray * (MAX_IN + MAX_AUX))()
_shape = (ctypes.c_int64 * MAX_DIMS)()
_scalars = (ctypes.c_double * MAX_IN)()
_mask = (ctypes.c_uint8 * MAX_DIMS)()


def _set_array(slot, t):
    slot.data = t.data_ptr()
    st = t.stride()
    if st:
        slot.strides[: len(st)] = st


def _set_shape(shape):
    n = len(shape)
    if n > MAX_DIMS:
        raise AgmiError(f"rank {n} arrays are not supported (max {MAX_DIMS})")
    if n:
        _shape[:n] = shape
    return n


def _set_inputs(ins):
    """Fill the input slots; array-valued factors / offsets of pending maps go to auxiliary slots
    after the op's own inputs.  Returns the total number of slots used."""
    n = len(ins)
    for k, x in enumerate(ins):
        slot = _ins[k]
        if isinstance(x, torch.Tensor):
            _set_array(slot, x)
            slot.affine = 0
        elif type(x) is Affine:
            _set_array(slot, x.t)
            flags = 0
            if x.scale != 1.0:
                slot.scale = x.scale
                flags = 1
            if x.ascale is not None:
                if n >= MAX_IN + MAX_AUX:
                    raise AgmiError("too many array-valued pending maps in one launch")
                _set_array(_ins[n], x.ascale)
                _ins[n].affine = 0
                slot.scale_slot = n
                flags |= 4
                n += 1
            sh = x.shift
            if sh is not None:
                if type(sh) is float:
                    slot.shift = sh
                    flags |= 2
                else:
                    if n >= MAX_IN + MAX_AUX:
                        raise AgmiError("too many array-valued pending maps in one launch")
                    _set_array(_ins[n], sh)
                    _ins[n].affine = 0
                    slot.shift_slot = n
                    flags |= 8
                    n += 1
            slot.affine = flags
        else:
            slot.data = None
            _scalars[k] = x
    return n


def elementwise(op, code, shape, outs, ins):
    """``outs[k][idx] = op(ins...)`` over ``shape``.

    ``outs`` are tensors of exactly ``shape``; ``ins`` are tensors already expanded to
    ``shape`` (stride 0 on broadcast axes) or Python floats (by-value scalars).
    """
    nd = _set_shape(shape)
    for k, t in enumerate(outs):
        _set_array(_outs[k], t)
    n_in = _set_inputs(ins)
    ev = _TIMER.begin(("elementwise", op)) if _TIMER is not None else None
    rc = _LIB.agmi_elementwise(op, code, nd, _shape, len(outs), _outs, n_in, _ins, _scalars, _stream())
    if rc:
        _check(rc, "agmi_elementwise")
    if ev is not None:
        _TIMER.end(ev, ("elementwise", op), (outs, ins))


PROGRAM_MAX_LEAVES, PROGRAM_MAX_IMMEDIATES, PROGRAM_MAX_OUTPUTS, PROGRAM_MAX_INSTRUCTIONS = 6, 6, 4, 96
PROGRAM_MAX_REGISTERS = 16
PROGRAM_MAX_MASKS = 4
PROGRAM_STORE, PROGRAM_MASK, PROGRAM_ROWSUM, PROGRAM_ROWLSE = 255, 254, 253, 252
_prog_leaf_ranges = (ctypes.c_int64 * (2 * PROGRAM_MAX_LEAVES))()
_prog_mask_ranges = (ctypes.c_int64 * (2 * PROGRAM_MAX_MASKS))()
_prog_outs = (AgmiArray * PROGRAM_MAX_OUTPUTS)()
_prog_leaves = (AgmiArray * PROGRAM_MAX_LEAVES)()
_prog_imms = (ctypes.c_double * PROGRAM_MAX_IMMEDIATES)()
_prog_code = (ctypes.c_uint32 * PROGRAM_MAX_INSTRUCTIONS)()


def program(code, shape, outs, leaves, imms, words, n_regs, shifted=None, masks=()):
    """Run the elementwise program ``words`` (instruction words of ``agmi_program``) over ``shape``.

    ``outs`` are tensors of exactly ``shape``; ``leaves`` tensors expanded to ``shape`` (stride 0 on
    broadcast axes); ``imms`` Python floats.  ``shifted`` (one-axis programs): per leaf ``(shift, lo, hi)``, the
    leaf is read ``shift`` elements further on and only at indices in [lo, hi); ``masks``: the (lo, hi) ranges of
    the program's mask instructions.  Returns False when the layout is outside what the kernel covers (the
    caller then evaluates the steps one by one)."""
    nd = _set_shape(shape)
    for k, t in enumerate(outs):
        _set_array(_prog_outs[k], t)
    ranges = None
    if shifted is None:
        for k, t in enumerate(leaves):
            _set_array(_prog_leaves[k], t)
    else:
        ranges = _prog_leaf_ranges
        for k, t in enumerate(leaves):
            slot = _prog_leaves[k]
            shift, lo, hi = shifted[k]
            _set_array(slot, t)
            if shift:
                slot.data = t.data_ptr() + shift * t.stride(0) * t.element_size()
            ranges[2 * k], ranges[2 * k + 1] = lo, hi
    n_mask = len(masks)
    for k in range(n_mask):
        _prog_mask_ranges[2 * k], _prog_mask_ranges[2 * k + 1] = masks[k]
    n_imm = len(imms)
    if n_imm:
        _prog_imms[:n_imm] = imms
    n = len(words)
    _prog_code[:n] = words
    ev = _TIMER.begin(("program",)) if _TIMER is not None else None
    rc = _LIB.agmi_program(code, nd, _shape, len(outs), _prog_outs, len(leaves), _prog_leaves, ranges, n_imm, _prog_imms,
                           n_mask, _prog_mask_ranges, n, _prog_code, n_regs, _stream())
    if rc == -2:  # AGMI_ERR_UNSUPPORTED
        return False
    if rc:
        _check(rc, "agmi_program")
    if ev is not None:
        _TIMER.end(ev, ("program",), (outs, leaves))
    return True


def specialize_after(sightings):
    """Programs handed to :func:`program` this many times get a kernel compiled for them (0: never; negative: only
    ask).  Returns the previous setting."""
    return lib().agmi_program_specialize(int(sightings))


def specialized_programs():
    """(programs compiled so far, launches they have served)."""
    compiled, launches = ctypes.c_longlong(), ctypes.c_longlong()
    lib().agmi_program_specialized(ctypes.byref(compiled), ctypes.byref(launches))
    return compiled.value, launches.value


def program_source(code, n_leaf, n_imm, words, n_regs, row_sums=False):
    """The HIP source of the kernel a recurring program is specialised to."""
    L = lib()
    n = len(words)
    arr = (ctypes.c_uint32 * n)(*words)
    size = L.agmi_program_source(code, n_leaf, n_imm, n, arr, n_regs, 1 if row_sums else 0, None, 0)
    if size < 0:
        _check(int(size), "agmi_program_source")
    text = ctypes.create_string_buffer(size + 1)
    L.agmi_program_source(code, n_leaf, n_imm, n, arr, n_regs, 1 if row_sums else 0, text, size + 1)
    return text.value.decode()


def compare(cmp, code, shape, out, ins):
    nd = _set_shape(shape)
    _set_array(_outs[0], out)
    _set_inputs(ins)
    _check(_LIB.agmi_compare(cmp, code, nd, _shape, _outs, _ins, _scalars, _stream()), "agmi_compare")


def cast(src_code, dst_code, shape, out, src):
    nd = _set_shape(shape)
    _set_array(_outs[0], out)
    _set_array(_ins[0], src)
    _ins[0].affine = 0
    _check(_LIB.agmi_cast(src_code, dst_code, nd, _shape, _outs, _ins, _stream()), "agmi_cast")


_WORKSPACE = None
_WORKSPACE_BYTES = 32 << 20


def _workspace():
    global _WORKSPACE
    if _WORKSPACE is None:
        _WORKSPACE = torch.empty(_WORKSPACE_BYTES, dtype=torch.uint8, device=device())
    return _WORKSPACE


def map_reduce(op, red, code, shape, reduce_mask, out, ins):
    """``out[kept] = RED over masked axes of op(ins...)``.

    ``out`` is a tensor whose strides are given for ALL axes of ``shape`` (any value on the
    reduced ones); ``ins`` as in :func:`elementwise`.  Returns False when the reduced axes do
    not form one group after merging (caller then reduces in two steps).
    """
    nd = _set_shape(shape)
    for d, m in enumerate(reduce_mask):
        _mask[d] = 1 if m else 0
    _set_array(_outs[0], out)
    n_in = _set_inputs(ins)
    ws = _workspace()
    ev = _TIMER.begin(("map_reduce", op, red)) if _TIMER is not None else None
    rc = _LIB.agmi_map_reduce(op, red, code, nd, _shape, _mask, _outs, n_in, _ins, _scalars, ws.data_ptr(),
                              _WORKSPACE_BYTES, _stream())
    if rc == -2:  # AGMI_ERR_UNSUPPORTED
        return False
    if rc:
        _check(rc, "agmi_map_reduce")
    if ev is not None:
        _TIMER.end(ev, ("map_reduce", op, red), ((out,), ins))
    return True


STATIC_SCRATCH_BYTES = 1 << 20


def map_reduce_static(op, red, code, shape, reduce_mask, out, ins):
    """:func:`map_reduce` through ``agmi_map_reduce_static``: partial results are staged in the
    library's built-in scratch array, nothing is allocated.  Raises :class:`AgmiError` when the
    reduction's partial results exceed ``STATIC_SCRATCH_BYTES``."""
    nd = _set_shape(shape)
    for d, m in enumerate(reduce_mask):
        _mask[d] = 1 if m else 0
    _set_array(_outs[0], out)
    n_in = _set_inputs(ins)
    rc = _LIB.agmi_map_reduce_static(op, red, code, nd, _shape, _mask, _outs, n_in, _ins, _scalars, _stream())
    if rc == -2:  # AGMI_ERR_UNSUPPORTED
        return False
    if rc:
        _check(rc, "agmi_map_reduce_static")
    return True


_lse_cot = AgmiLseCotangent()


def lse_cotangent(code, x, ans, g, row_sums=None, col_factor=None, scaled=None, col_sums=None):
    """One pass of ``agmi_lse_cotangent_fused`` over the 2-d operand ``x`` (a tensor, or an :class:`Affine` whose array
    steps are 2-d broadcast views); ``ans`` and ``g`` are (rows, 1) tensors (``g`` may be broadcast).  Outputs are
    contiguous tensors or None.  Returns False when the layout is outside what the kernel covers."""
    c = _lse_cot
    raw = x.t if type(x) is Affine else x
    c.rows, c.cols = raw.shape
    if raw.stride(1) != 1 and raw.shape[1] > 1:
        return False
    c.x, c.x_row_stride = raw.data_ptr(), raw.stride(0)
    flags, c.scale, c.shift, c.scale_vec, c.shift_vec = 0, 1.0, 0.0, None, None
    if type(x) is Affine:
        if x.scale != 1.0:
            c.scale = x.scale
            flags |= 1
        if x.ascale is not None:
            c.scale_vec, c.scale_row_stride, c.scale_col_stride = x.ascale.data_ptr(), x.ascale.stride(0), x.ascale.stride(1)
            flags |= 4
        if x.shift is not None:
            if type(x.shift) is float:
                c.shift = x.shift
                flags |= 2
            else:
                c.shift_vec, c.shift_row_stride, c.shift_col_stride = x.shift.data_ptr(), x.shift.stride(0), x.shift.stride(1)
                flags |= 8
    c.affine = flags
    c.ans, c.ans_stride = ans.data_ptr(), ans.stride(0)
    c.g, c.g_stride = g.data_ptr(), g.stride(0)
    c.row_sums = row_sums.data_ptr() if row_sums is not None else None
    c.col_factor = col_factor.data_ptr() if col_factor is not None else None
    c.scaled = scaled.data_ptr() if scaled is not None else None
    c.scaled_row_stride = scaled.stride(0) if scaled is not None else 0
    c.col_sums = col_sums.data_ptr() if col_sums is not None else None
    ev = _TIMER.begin(("lse_cotangent",)) if _TIMER is not None else None
    probe = _LIB.agmi_probe_arm() if ev is not None else None  # (the tile kernel alone; `ev` brackets it and the finishing kernel)
    rc = _LIB.agmi_lse_cotangent_fused(code, ctypes.byref(c), _workspace().data_ptr(), _WORKSPACE_BYTES, _stream())
    if rc == -2:  # AGMI_ERR_UNSUPPORTED
        return False
    if rc:
        _check(rc, "agmi_lse_cotangent_fused")
    if ev is not None:
        outs = tuple(t for t in (row_sums, scaled, col_sums) if t is not None)
        _TIMER.end(ev, ("lse_cotangent",), (outs, (x, ans, g) + ((col_factor,) if col_factor is not None else ())),
                   probe=probe if probe is not None and probe >= 0 else None)
    return True


def gemm(code, batch, M, N, K, alpha, A, a_rs, a_cs, a_bs, B, b_rs, b_cs, b_bs, beta, C, ldc, c_bs):
    ev = _TIMER.begin(("gemm",)) if _TIMER is not None else None
    rc = _LIB.agmi_gemm(code, batch, M, N, K, alpha, A.data_ptr(), a_rs, a_cs, a_bs, B.data_ptr(), b_rs, b_cs, b_bs,
                        beta, C.data_ptr(), ldc, c_bs, _workspace().data_ptr(), _WORKSPACE_BYTES, _stream())
    if rc:
        _check(rc, "agmi_gemm")
    if ev is not None:
        es = A.element_size()
        _TIMER.end(ev, ("gemm",), batch * (M * K + K * N + M * N) * es, 2.0 * batch * M * N * K)


EPILOGUE_BIAS_TANH, EPILOGUE_TANH_VJP = 1, 2
_epilogue = AgmiGemmEpilogue()


def gemm_fused(code, A, B, C, kind, bias=None, out=None, x=None, beta=0.0, second=None, beside=None):
    """``agmi_gemm_fused``: ``A @ B`` (2-d tensors, any strides; plus ``beta`` times what ``C`` holds) into the
    contiguous ``C`` with a dense layer's epilogue: ``out = tanh(C + bias)`` beside it, or
    ``C = (A @ B + beta * C) / cosh(x + bias)**2`` (``bias``: contiguous vector or None).  ``second``: a pair
    ``(A2, B2)`` whose product is added before the tanh rule, in the same launch (bit for bit what running ``A @ B``
    into ``C`` and then ``A2 @ B2`` with ``beta = 1`` gives).  ``beside``: ``(A3, B3, C3)``, an independent plain product
    ``C3 = A3 @ B3`` computed by further blocks of the same launch.  Returns False when the operands are outside what
    the fused kernel covers (nothing has run then)."""
    M, K = A.shape
    N = B.shape[1]
    e = _epilogue
    e.kind = kind
    e.bias = bias.data_ptr() if bias is not None else None
    e.out, e.out_ld = (out.data_ptr(), out.stride(0)) if out is not None else (None, 0)
    e.x, e.x_ld = (x.data_ptr(), x.stride(0)) if x is not None else (None, 0)
    e.beta = beta
    flops = 2.0 * M * N * K
    if second is None:
        e.a2 = e.b2 = None
        e.k2 = 0
    else:
        A2, B2 = second
        e.a2, e.a2_rs, e.a2_cs = A2.data_ptr(), A2.stride(0), A2.stride(1)
        e.b2, e.b2_rs, e.b2_cs = B2.data_ptr(), B2.stride(0), B2.stride(1)
        e.k2 = A2.shape[1]
        flops += 2.0 * M * N * A2.shape[1]
    nbytes = 0
    if beside is None:
        e.with_c = None
    else:
        A3, B3, C3 = beside
        e.with_a, e.with_a_rs, e.with_a_cs = A3.data_ptr(), A3.stride(0), A3.stride(1)
        e.with_b, e.with_b_rs, e.with_b_cs = B3.data_ptr(), B3.stride(0), B3.stride(1)
        e.with_c, e.with_ldc = C3.data_ptr(), C3.stride(0)
        e.with_m, e.with_n, e.with_k = A3.shape[0], B3.shape[1], A3.shape[1]
        flops += 2.0 * A3.shape[0] * B3.shape[1] * A3.shape[1]
        nbytes = (A3.numel() + B3.numel() + C3.numel()) * A3.element_size()
    ev = _TIMER.begin(("gemm",)) if _TIMER is not None else None
    rc = _LIB.agmi_gemm_fused(code, M, N, K, A.data_ptr(), A.stride(0), A.stride(1), B.data_ptr(), B.stride(0), B.stride(1),
                              C.data_ptr(), C.stride(0), ctypes.byref(e), _workspace().data_ptr(), _WORKSPACE_BYTES, _stream())
    if rc == -2:  # AGMI_ERR_UNSUPPORTED
        return False
    if rc:
        _check(rc, "agmi_gemm_fused")
    if ev is not None:
        es = A.element_size()
        k_all = K + (second[0].shape[1] if second is not None else 0)
        _TIMER.end(ev, ("gemm",), (M * k_all + k_all * N + 2 * M * N) * es + nbytes, flops)
    return True


def fill(code, t, value):
    """Fill a CONTIGUOUS tensor."""
    rc = _LIB.agmi_fill(code, t.data_ptr(), t.numel(), float(value), _stream())
    if rc:
        _check(rc, "agmi_fill")


MAX_CONCAT = 32


class AgmiConcatPiece(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("extent", ctypes.c_int64), ("stride_outer", ctypes.c_int64),
                ("stride_axis", ctypes.c_int64), ("stride_inner", ctypes.c_int64)]


_concat_pieces = (AgmiConcatPiece * MAX_CONCAT)()


def concat(code, outer, inner, pieces, out):
    """``pieces``: (tensor, extent, stride_outer, stride_axis, stride_inner) per piece, joined along the middle axis
    of the contiguous (outer, total, inner) tensor ``out`` in one launch."""
    for k, (t, extent, so, sa, si) in enumerate(pieces):
        slot = _concat_pieces[k]
        slot.data, slot.extent, slot.stride_outer, slot.stride_axis, slot.stride_inner = t.data_ptr(), extent, so, sa, si
    ev = _TIMER.begin(("concat",)) if _TIMER is not None else None
    _check(_LIB.agmi_concat(code, outer, inner, len(pieces), _concat_pieces, out.data_ptr(), _stream()), "agmi_concat")
    if ev is not None:
        _TIMER.end(ev, ("concat",), 2 * out.numel() * out.element_size())


def take_rows(code, src, n_rows, inner, index, n_index, out):
    _check(_LIB.agmi_take_rows(code, src.data_ptr(), n_rows, inner, index.data_ptr(), n_index, out.data_ptr(),
                               _stream()), "agmi_take_rows")


def reverse(code, src, outer, n, inner, out):
    _check(_LIB.agmi_reverse(code, src.data_ptr(), outer, n, inner, out.data_ptr(), _stream()), "agmi_reverse")


def triangle(code, src, batch, rows, cols, k, lower, out):
    _check(_LIB.agmi_triangle(code, src.data_ptr(), batch, rows, cols, k, 1 if lower else 0, out.data_ptr(), _stream()),
           "agmi_triangle")


def sort_rows(code, src, rows, n, sorted_out=None, order=None, rank=None):
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    rc = _LIB.agmi_sort_rows(code, src.data_ptr(), rows, n, ptr(sorted_out), ptr(order), ptr(rank), _stream())
    if rc == -2:  # AGMI_ERR_UNSUPPORTED
        raise NotImplementedError(_LIB.agmi_last_error().decode())
    _check(rc, "agmi_sort_rows")


def cumsum(code, src, outer, n, inner, out):
    _check(_LIB.agmi_cumsum(code, src.data_ptr(), outer, n, inner, out.data_ptr(), _stream()), "agmi_cumsum")


def scatter_add_rows(code, dst, n_rows, inner, src, index, order, seg_start, n_seg):
    """``seg_start`` None: the runs of equal destination are found on the device and ``n_seg`` counts index entries."""
    _check(_LIB.agmi_scatter_add_rows(code, dst.data_ptr(), n_rows, inner, src.data_ptr(), index.data_ptr(),
                                      order.data_ptr(), None if seg_start is None else seg_start.data_ptr(), n_seg,
                                      _stream()),
           "agmi_scatter_add_rows")


def correlate(code, args, n_bytes, n_flops):
    """Launch the sliding-window contraction described by the ``AgmiCorrelation`` block ``args``."""
    ev = _TIMER.begin(("correlate",)) if _TIMER is not None else None
    rc = _LIB.agmi_correlate(code, ctypes.byref(args), _stream())
    if rc:
        _check(rc, "agmi_correlate")
    if ev is not None:
        _TIMER.end(ev, ("correlate",), n_bytes, n_flops)


OPT_SGD, OPT_RMSPROP, OPT_ADAM = 0, 1, 2
_hyper = (ctypes.c_double * 8)()


def optimizer_step(kind, x_in, g, s0, s1, x_out, hyper):
    """One fused optimizer update on flat contiguous tensors (state and ``x_out`` float64)."""
    n = x_in.numel()
    for t in (x_in, g, s0, s1, x_out):
        if t is not None and (t.numel() != n or not t.is_contiguous()):
            raise AgmiError("optimizer_step: operands must be contiguous and of equal length")
    _hyper[: len(hyper)] = hyper
    ev = _TIMER.begin(("optimizer_step", kind)) if _TIMER is not None else None
    rc = _LIB.agmi_optimizer_step(kind, DTYPE_CODE[NUMPY_DTYPE[x_in.dtype]], DTYPE_CODE[NUMPY_DTYPE[g.dtype]], n,
                                  x_in.data_ptr(), g.data_ptr(), s0.data_ptr(), s1.data_ptr() if s1 is not None else None,
                                  x_out.data_ptr(), _hyper, _stream())
    if rc:
        _check(rc, "agmi_optimizer_step")
    if ev is not None:
        _TIMER.end(ev, ("optimizer_step", kind), _traffic((x_out, s0) + ((s1,) if s1 is not None else ()),
                                                           (x_in, g, s0) + ((s1,) if s1 is not None else ())))
