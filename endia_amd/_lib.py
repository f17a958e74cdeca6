"""ctypes binding of libendia_hip.so (the C ABI declared in include/endia_hip.h).

There is no CPU fallback: if the library is missing, or no gfx950 device can be initialised, every
entry point raises. `lib()` loads the shared object (possible without a GPU, e.g. to check the
exported symbols); `ensure_init()` additionally creates the device context.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int32, c_int64, c_uint32, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libendia_hip.so")

# enums of include/endia_hip.h
(OP_RELU, OP_TANH, OP_SIN, OP_COS, OP_NEG, OP_SQUARE, OP_SQRT, OP_ABS, OP_IDENTITY, OP_GREATER0, OP_EXP, OP_LOG,
 OP_SIGMOID, OP_SINH, OP_COSH, OP_TAN, OP_ASIN, OP_ACOS, OP_ATAN, OP_RECIPROCAL, OP_SIGN) = range(21)
(BIN_ADD, BIN_SUB, BIN_MUL, BIN_DIV, BIN_GREATER, BIN_POW, BIN_GREATER_EQUAL, BIN_LESS, BIN_LESS_EQUAL, BIN_EQUAL,
 BIN_NOT_EQUAL) = range(11)
EW_LOAD, EW_UNARY, EW_BINARY, EW_RBINARY, EW_SAVE, EW_STORE = range(6)
EW_SRC_INPUT, EW_SRC_SLOT, EW_SRC_IMM = range(3)
EW_FULL, EW_ROW_VECTOR, EW_SCALAR = range(3)
EW_MAX_INPUTS, EW_MAX_OUTPUTS, EW_MAX_SLOTS, EW_MAX_STEPS = 8, 4, 4, 48
EPI_NONE, EPI_BIAS, EPI_BIAS_ACT, EPI_ACT_GRAD = range(4)
ACT_FROM_OUTPUT = 0x100
GEMM_ACCUMULATE = 0x200
GEMM_COLSUM_B = 0x400
CGEMM_4M, CGEMM_3M = 0, 1
REDUCE_MAX, REDUCE_MIN, REDUCE_MUL, REDUCE_ARGMAX, REDUCE_ARGMIN = range(5)

ERR_INVALID, ERR_NOT_INIT, ERR_RUNTIME, ERR_NOMEM, ERR_UNSUPPORTED = -1, -2, -3, -4, -5


class EndiaHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("libendia_hip: error %d: %s" % (code, message))
        self.code = code


class Conv2dDesc(ctypes.Structure):
    _fields_ = [(n, c_int64) for n in (
        "N", "C", "H", "W", "K", "R", "S",
        "stride_h", "stride_w", "pad_h", "pad_w", "dil_h", "dil_w", "groups")]


class EwStep(ctypes.Structure):
    _fields_ = [("kind", c_int32), ("op", c_int32), ("src_kind", c_int32), ("src_index", c_int32), ("imm", c_float)]


class Conv3dDesc(ctypes.Structure):
    _fields_ = [(n, c_int64) for n in ("N", "C", "D", "H", "W", "K", "T", "R", "S")] + [
        (n, c_int64 * 3) for n in ("stride", "padding", "dilation")] + [("groups", c_int64)]


class PoolDesc(ctypes.Structure):
    _fields_ = [(n, c_int64) for n in ("N", "C", "D", "H", "W")] + [
        (n, c_int64 * 3) for n in ("kernel", "stride", "padding", "dilation")]


POOL_MAX, POOL_AVG = 0, 1
MLP_MAX_LAYERS, MLP_MAX_WIDTH = 16, 128


class MlpDesc(ctypes.Structure):
    _fields_ = [("layers", c_int32), ("act", c_int32), ("batch", c_int64), ("widths", c_int64 * (MLP_MAX_LAYERS + 1))]

class SgemmDesc(ctypes.Structure):
    _fields_ = [("transA", c_int32), ("transB", c_int32), ("M", c_int64), ("N", c_int64), ("K", c_int64), ("A", c_void_p),
                ("lda", c_int64), ("B", c_void_p), ("ldb", c_int64), ("C", c_void_p), ("ldc", c_int64), ("epilogue", c_int32),
                ("bias", c_void_p)]


class ColSumDesc(ctypes.Structure):
    _fields_ = [("R", c_int64), ("C", c_int64), ("x", c_void_p), ("out", c_void_p), ("scale", c_float)]


_fp = c_void_p  # device pointers travel as plain addresses
_i64p = POINTER(c_int64)

SIGNATURES = {
    "endia_hip_init": [c_int32],
    "endia_hip_shutdown": [],
    "endia_hip_sync": [],
    "endia_hip_device_info": [c_char_p, c_int64, POINTER(c_int32), POINTER(c_int32)],
    "endia_hip_malloc": [c_int64, POINTER(c_void_p)],
    "endia_hip_free": [c_void_p],
    "endia_hip_memcpy_h2d": [c_void_p, c_void_p, c_int64],
    "endia_hip_memcpy_d2h": [c_void_p, c_void_p, c_int64],
    "endia_hip_memcpy_d2d": [c_void_p, c_void_p, c_int64],
    "endia_hip_memset0": [c_void_p, c_int64],
    "endia_hip_fill": [_fp, c_int64, c_float],
    "endia_hip_pool_stats": [_i64p, _i64p, _i64p],
    "endia_hip_pool_trim": [],
    "endia_hip_timer_start": [c_int32],
    "endia_hip_timer_stop": [c_int32],
    "endia_hip_timer_elapsed_ms": [c_int32, POINTER(c_float)],
    "endia_hip_graph_begin": [],
    "endia_hip_graph_end": [_i64p],
    "endia_hip_graph_launch": [c_int64],
    "endia_hip_graph_destroy": [c_int64],
    "endia_hip_gemm_force_tile": [c_int32],
    "endia_hip_gemm_timing_begin": [],
    "endia_hip_gemm_timing_end": [_i64p, POINTER(c_double), POINTER(c_double)],
    "endia_hip_strided_copy": [c_int32, _i64p, _i64p, c_int64, _fp, _fp, c_int32],
    "endia_hip_strided_scatter": [c_int32, _i64p, _i64p, c_int64, _fp, _fp, c_int32, c_int32],
    "endia_hip_sgemm": [c_int32, c_int32, c_int64, c_int64, c_int64, _fp, c_int64, _fp, c_int64, _fp, c_int64,
                        c_int64, c_int64, c_int64, c_int64, c_int32, c_int32, _fp, _fp, _fp],
    "endia_hip_sgemm_grouped": [c_int32, POINTER(SgemmDesc), c_int32, POINTER(c_int32)],
    "endia_hip_linear_bwd": [c_int64, c_int64, c_int64, _fp, _fp, _fp, c_int32, _fp, _fp, _fp, _fp],
    "endia_hip_mlp_fwd": [POINTER(MlpDesc), _fp, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p)],
    "endia_hip_mlp_fwd_mse": [POINTER(MlpDesc), _fp, POINTER(c_void_p), POINTER(c_void_p), _fp, POINTER(c_void_p), _fp, _fp],
    "endia_hip_mlp_bwd": [POINTER(MlpDesc), _fp, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                          POINTER(c_void_p), _fp],
    "endia_hip_mlp_fwd_mse_delta": [POINTER(MlpDesc), _fp, POINTER(c_void_p), POINTER(c_void_p), _fp, POINTER(c_void_p),
                                    POINTER(c_void_p), _fp, _fp],
    "endia_hip_mlp_wgrad": [POINTER(MlpDesc), _fp, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p)],
    "endia_hip_cgemm": [c_int32, c_int32, c_int32, c_int32, c_int64, c_int64, c_int64, _fp, c_int64, _fp, c_int64,
                        _fp, c_int64, c_int64, c_int64, c_int64, c_int64, c_int32, c_int32],
    "endia_hip_unary_fwd": [c_int32, c_int64, _fp, _fp, c_int32],
    "endia_hip_unary_vjp": [c_int32, c_int64, _fp, _fp, _fp, c_int32],
    "endia_hip_unary_vjp_from_output": [c_int32, c_int64, _fp, _fp, _fp],
    "endia_hip_binary": [c_int32, c_int32, _i64p, _i64p, _i64p, _fp, _fp, _fp, c_int32],
    "endia_hip_ew_program": [c_int64, c_int64, c_int32, POINTER(c_void_p), POINTER(c_int32), c_int32, POINTER(c_void_p),
                             c_int32, POINTER(EwStep)],
    "endia_hip_axpby": [c_int64, c_float, _fp, c_float, _fp, _fp],
    "endia_hip_complex_pack": [c_int64, _fp, _fp, _fp],
    "endia_hip_reduce_add": [c_int32, _i64p, c_uint32, _fp, _fp, c_float, c_int32],
    "endia_hip_col_sum_static": [c_int64, c_int64, _fp, _fp, c_float],
    "endia_hip_col_sum_plan": [c_int64, c_int64, c_int64, c_int64, c_int32, _i64p, _i64p],
    "endia_hip_col_sum_multi": [c_int32, POINTER(ColSumDesc)],
    "endia_hip_reduce": [c_int32, c_int32, _i64p, c_uint32, _fp, _fp],
    "endia_hip_mse_fwd_bwd": [c_int64, _fp, _fp, _fp, _fp],
    "endia_hip_conv2d_out_shape": [POINTER(Conv2dDesc), _i64p, _i64p],
    "endia_hip_conv2d_fwd": [POINTER(Conv2dDesc), _fp, _fp, _fp, _fp, c_int32],
    "endia_hip_conv2d_bwd_data": [POINTER(Conv2dDesc), _fp, _fp, _fp],
    "endia_hip_conv2d_bwd_weight": [POINTER(Conv2dDesc), _fp, _fp, _fp],
    "endia_hip_conv2d_bwd_bias": [POINTER(Conv2dDesc), _fp, _fp],
    "endia_hip_conv2d_bwd_relu": [POINTER(Conv2dDesc), _fp, _fp, _fp, _fp, c_int32, _fp, _fp, _fp],
    "endia_hip_conv_force_path": [c_int32],
    "endia_hip_conv3d_out_shape": [POINTER(Conv3dDesc), _i64p],
    "endia_hip_conv3d_fwd": [POINTER(Conv3dDesc), _fp, _fp, _fp, _fp, c_int32],
    "endia_hip_conv3d_bwd_data": [POINTER(Conv3dDesc), _fp, _fp, _fp],
    "endia_hip_conv3d_bwd_weight": [POINTER(Conv3dDesc), _fp, _fp, _fp],
    "endia_hip_conv3d_bwd_bias": [POINTER(Conv3dDesc), _fp, _fp],
    "endia_hip_pool_out_shape": [POINTER(PoolDesc), _i64p],
    "endia_hip_pool_fwd": [POINTER(PoolDesc), c_int32, _fp, _fp, _fp],
    "endia_hip_pool_bwd": [POINTER(PoolDesc), c_int32, _fp, _fp, _fp],
    "endia_hip_sgd_step": [c_int64, _fp, _fp, c_float],
    "endia_hip_sgd_step_multi": [c_int32, _i64p, POINTER(c_void_p), POINTER(c_void_p), c_float],
    "endia_hip_adam_step_multi": [c_int32, _i64p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                  c_float, c_float, c_float, c_float, _fp],
    "endia_hip_sgd_momentum_step": [c_int64, _fp, _fp, _fp, c_float, c_float, c_float],
    "endia_hip_adagrad_step": [c_int64, _fp, _fp, _fp, c_float, c_float],
    "endia_hip_rmsprop_step": [c_int64, _fp, _fp, _fp, c_float, c_float, c_float],
    "endia_hip_adam_step": [c_int64, _fp, _fp, _fp, _fp, c_float, c_float, c_float, c_float, c_float],
}

_lib = None
_ready = False
capturing = False  # set by endia_amd.graph while a step is being recorded


def lib():
    """Load libendia_hip.so and attach argument types. Raises if the library has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python endia_amd/csrc/build.py` (there is no CPU fallback)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = c_int32
        handle.endia_hip_last_error.argtypes = []
        handle.endia_hip_last_error.restype = c_char_p
        _lib = handle
    return _lib


def check(code):
    if code != 0:
        raise EndiaHipError(code, lib().endia_hip_last_error().decode("utf-8", "replace"))


def ensure_init(device=0):
    """Create the device context once. Raises EndiaHipError when no gfx950 device is usable."""
    global _ready
    if not _ready:
        check(lib().endia_hip_init(device))
        _ready = True
    return lib()


_entry = {}


def _raw_call(name, *args):
    fn = _entry.get(name)
    if fn is None:
        fn = _entry[name] = getattr(ensure_init(), name)
    code = fn(*args)
    if code:
        check(code)


# ---- products waiting for a shared launch -----------------------------------------------------------------
# A backward pass (above all a second-order one) issues many fp32 products that do not depend on each other, each too
# small to fill the chip. functional._sgemm parks such a product here instead of launching it; flush() hands everything
# parked to endia_hip_sgemm_grouped, which lets the members that fit together share a launch. What keeps this invisible:
#   * a parked product's output buffer is marked `pending`, and reading the address of a pending buffer (Buffer.ptr,
#     the only way to it) flushes first, so nothing ever consumes a result that has not been launched;
#   * every library call flushes first unless it is one of _WRITES_FRESH below, the entry points this package only ever
#     calls with outputs it has just allocated: nothing parked can depend on, or be overtaken by, such a call (a parked
#     product holds its operands' buffers, so a fresh buffer is never one of them). Everything that writes into existing
#     memory, synchronises, copies to the host, records or replays a graph flushes;
#   * a product that accumulates into a buffer which a parked product reads or writes flushes before it is parked.
_WRITES_FRESH = frozenset({
    "endia_hip_malloc", "endia_hip_free", "endia_hip_binary", "endia_hip_unary_fwd", "endia_hip_unary_vjp",
    "endia_hip_unary_vjp_from_output", "endia_hip_ew_program", "endia_hip_reduce_add", "endia_hip_reduce",
    "endia_hip_strided_copy", "endia_hip_mse_fwd_bwd", "endia_hip_complex_pack", "endia_hip_linear_bwd",
    "endia_hip_conv2d_out_shape", "endia_hip_conv3d_out_shape", "endia_hip_pool_out_shape",
})
_parked = []          # (fields of an endia_hip_sgemm_desc, buffers kept alive, output buffer)
MAX_PARKED = 16
defer_products = [True]  # tests switch the parking off to compare
flush_observer = [None]  # tests and probes: called with (descriptor fields of what was parked, index needed or -1, launched flags)


def park_product(fields, buffers, out_buffer):
    if len(_parked) >= MAX_PARKED:
        flush()
    out_buffer.pending = True
    _parked.append((fields, buffers, out_buffer))


_parked_sums = []     # column sums nobody has asked for yet: (R, C, x address, out address, scale, input buffer, output buffer)
MAX_PARKED_SUMS = 16


def park_col_sum(R, C, x_ptr, out_ptr, scale, in_buffer, out_buffer):
    """out = scale * (sum of the rows of x), put off: a bias gradient is a leaf of the backward pass, so as a rule nothing reads
    it before the pass is over, and the sums of a pass then go out as ONE endia_hip_col_sum_multi call (a launch of its own
    costs each of them more than its memory traffic). The input buffer is held until then; reading the output's address
    (Buffer.ptr) launches them."""
    if len(_parked_sums) >= MAX_PARKED_SUMS:
        flush_col_sums()
    out_buffer.pending = True
    _parked_sums.append((R, C, x_ptr, out_ptr, scale, in_buffer, out_buffer))


def flush_col_sums():
    """Launch the column sums that were put off (the end of a reverse pass does; so does anything that reads one of them)."""
    if not _parked_sums:
        return
    items = _parked_sums[:]
    del _parked_sums[:]
    descs = (ColSumDesc * len(items))()
    for d, it in zip(descs, items):
        d.R, d.C, d.x, d.out, d.scale = it[0], it[1], it[2], it[3], it[4]
    for it in items:
        it[6].pending = False  # (also when the call fails: the error is the caller's to see, once)
    _raw_call("endia_hip_col_sum_multi", len(items), descs)


def park_launch(launch, out_buffers):
    """Park any other launch whose outputs are all fresh buffers: `launch()` issues it. Besides being run by flush() it
    can be withdrawn (withdraw_launch) by an op that computes the same outputs as part of a larger launch."""
    if len(_parked) >= MAX_PARKED:
        flush()
    for b in out_buffers:
        b.pending = True
    item = (None, launch, list(out_buffers))
    _parked.append(item)
    return item


def withdraw_launch(item):
    """Take a parked launch back; True when it was still parked (its buffers are then no longer pending, and whoever
    withdrew it writes them)."""
    for i, it in enumerate(_parked):
        if it is item:
            del _parked[i]
            for b in item[2]:
                b.pending = False
            return True
    return False


def parked_uses(buffer):
    """True when a parked product reads or writes `buffer`."""
    for it in _parked_sums:
        if it[5] is buffer or it[6] is buffer:
            return True
    for fields, buffers, out in _parked:
        if fields is None:
            if any(b is buffer for b in out):
                return True
            continue
        if out is buffer:
            return True
        for b in buffers:
            if b is buffer:
                return True
    return False


def flush(need=None):
    """Launch what is parked: everything, or, when `need` names the output buffer somebody is about to read, the launch
    that writes it; for a product that means one endia_hip_sgemm_grouped call with that product and whichever parked
    products make its launch a better one (the rest stay parked and may find better company later)."""
    if _parked_sums and (need is None or any(it[6] is need for it in _parked_sums)):
        # (a sum's input is never pending: its address was read when the sum was put off)
        flush_col_sums()
        if need is not None:
            return
    if not _parked:
        return
    items = _parked[:]
    if need is not None:
        for it in items:
            if it[0] is None and any(b is need for b in it[2]):
                _parked.remove(it)
                for b in it[2]:
                    b.pending = False
                it[1]()
                return
    else:
        for it in items:
            if it[0] is None:
                _parked.remove(it)
                for b in it[2]:
                    b.pending = False
                it[1]()
        items = _parked[:]
        if not items:
            return
    products = [it for it in items if it[0] is not None]
    index = -1
    if need is not None:
        for i, (_, _, out) in enumerate(products):
            if out is need:
                index = i
        if index < 0:
            return
    descs = (SgemmDesc * len(products))()
    for d, (f, _, _) in zip(descs, products):
        (d.transA, d.transB, d.M, d.N, d.K, d.A, d.lda, d.B, d.ldb, d.C, d.ldc, d.epilogue, d.bias) = f
    done = (c_int32 * len(products))()
    for it in products:
        _parked.remove(it)  # (nothing below comes back here: the raw call flushes nothing)
    try:
        _raw_call("endia_hip_sgemm_grouped", len(products), descs, index, done)
    except BaseException:
        for item in products:  # a launch that failed is not tried again: the error is the caller's to see, once
            item[2].pending = False
        raise
    if flush_observer[0] is not None:
        flush_observer[0]([item[0] for item in products], index, list(done))
    for item, flag in zip(products, done):
        if flag or index < 0:
            item[2].pending = False
        else:
            _parked.append(item)


def call(name, *args):
    """Call an entry point on the initialised library and raise on a non-zero status."""
    if (_parked or _parked_sums) and name not in _WRITES_FRESH and not (name == "endia_hip_sgemm" and not (args[15] & GEMM_ACCUMULATE)):
        flush()
    _raw_call(name, *args)


def i64_array(values):
    values = list(values)
    return (c_int64 * max(len(values), 1))(*values)


def device_info():
    buf = ctypes.create_string_buffer(256)
    cu, mhz = c_int32(), c_int32()
    call("endia_hip_device_info", buf, 256, ctypes.byref(cu), ctypes.byref(mhz))
    return buf.value.decode(), cu.value, mhz.value
