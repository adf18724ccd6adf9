"""TEST INFRASTRUCTURE ONLY -- numpy front end of the CPU oracle (oracle/libqoracle.so).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the
product library never does.  Functions mirror the reference's operator entry points for the
quaternion Conv2D / Dense path (src/upstride.hpp:18-86) on plain numpy arrays:

    x    [4n, ci, h, w]     component p in batch rows [p*n, (p+1)*n)
    w    [4, co, ci, kh, kw]
    bias [4, co] or None
    y    [4n, co, ho, wo]
    dense: x [4n, ni], w [4, ni, no] (layout IO), bias [4, no], y [4n, no]
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libqoracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_shim.so")

REAL, COMPLEX, QUATERNION, GA_300 = 0, 1, 2, 3
PAD_SAME, PAD_VALID, PAD_EXPLICIT = 0, 1, 2


class Geom(ctypes.Structure):
    """Per-blade convolution geometry (qo_geom)."""
    _fields_ = [(k, ctypes.c_int) for k in
                ("n", "ci", "co", "h", "w", "kh", "kw", "sh", "sw", "dh", "dw", "pt", "pl", "pb", "pr")]

    @property
    def ho(self):
        return lib().qo_out_h(ctypes.byref(self))

    @property
    def wo(self):
        return lib().qo_out_w(ctypes.byref(self))


class _Term(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int) for k in ("left", "right", "dim", "positive", "fill")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.isfile(_LIB_PATH):
            from . import build
            build.build_oracle()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.qo_padding_preset.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_int)] * 2
        _lib.qo_env_memory_optimized.argtypes = [ctypes.c_char_p]
        _lib.qo_env_fp16_policy.argtypes = [ctypes.c_char_p]
    return _lib


def ref_lib():
    """The reference-derived checker (sign tables, term order, Context switches), or None."""
    if not os.path.isfile(_REF_PATH):
        return None
    return ctypes.CDLL(_REF_PATH)


def make_geom(n, ci, co, h, w, kh, kw, stride=(1, 1), dilation=(1, 1), padding="VALID"):
    """Geometry with the reference's padding presets (src/utils.cc:10-39) or explicit
    (top, left, bottom, right) padding."""
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    dh, dw = (dilation, dilation) if isinstance(dilation, int) else dilation
    if isinstance(padding, str):
        preset = {"SAME": PAD_SAME, "VALID": PAD_VALID}[padding]
        pt, pb = padding_preset(h, kh, dh, sh, preset)[1:]
        pl, pr = padding_preset(w, kw, dw, sw, preset)[1:]
    else:
        pt, pl, pb, pr = padding
    return Geom(n, ci, co, h, w, kh, kw, sh, sw, dh, dw, pt, pl, pb, pr)


def padding_preset(size, filt, dilation, stride, preset):
    before, after = ctypes.c_int(0), ctypes.c_int(0)
    out = lib().qo_padding_preset(size, filt, dilation, stride, preset, ctypes.byref(before), ctypes.byref(after))
    if out < 0:
        raise ValueError("Invalid padding")
    return out, before.value, after.value


def output_size(size, filt, dilation, stride, before, after):
    return lib().qo_output_size(size, filt, dilation, stride, before, after)


def env_memory_optimized(value):
    return bool(lib().qo_env_memory_optimized(None if value is None else value.encode()))


def env_fp16_policy(value):
    return ("full16", "backward32", "fp32")[lib().qo_env_fp16_policy(None if value is None else value.encode())]


def sign_table(algebra):
    """(dims, [(left, right, positive)], layout, backprop_order) as restated in qoracle.c."""
    class _Sign(ctypes.Structure):
        _fields_ = [("left", ctypes.c_int), ("right", ctypes.c_int), ("positive", ctypes.c_int)]

    class _Spec(ctypes.Structure):
        _fields_ = [("dims", ctypes.c_int), ("table", ctypes.POINTER(_Sign)),
                    ("layout", ctypes.POINTER(ctypes.c_int)), ("order", ctypes.POINTER(ctypes.c_int))]

    fn = lib().qo_get_algebra
    fn.restype = ctypes.POINTER(_Spec)
    spec = fn(algebra).contents
    d = spec.dims
    table = [(spec.table[i].left, spec.table[i].right, bool(spec.table[i].positive)) for i in range(d * d)]
    return d, table, [spec.layout[i] for i in range(d + 1)], [spec.order[i] for i in range(d * d)]


def product_terms(algebra, backprop=False):
    """[(left, right, dim, positive, fill)] in execution order."""
    buf = (_Term * 64)()
    fn = lib().qo_backprop_terms if backprop else lib().qo_product_terms
    k = fn(algebra, buf)
    if k < 0:
        raise ValueError("bad algebra")
    return [(t.left, t.right, t.dim, bool(t.positive), bool(t.fill)) for t in buf[:k]]


def _suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "_f32", ctypes.c_float
    if dtype == np.float64:
        return "_f64", ctypes.c_double
    raise TypeError("oracle computes in float32 or float64")


def _ptr(a, ctype):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ctype))


def _prep(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def _check(status):
    if status != 0:
        raise RuntimeError("oracle call failed with status %d" % status)


def scalar_conv2d_fwd(geom, x, w, bias=None, dtype=np.float64):
    sfx, ct = _suffix(dtype)
    x, w, bias = _prep(x, dtype), _prep(w, dtype), _prep(bias, dtype)
    y = np.empty((geom.n, geom.co, geom.ho, geom.wo), dtype)
    getattr(lib(), "qo_scalar_conv2d_fwd" + sfx)(ctypes.byref(geom), _ptr(x, ct), _ptr(w, ct), _ptr(bias, ct), _ptr(y, ct))
    return y


def scalar_conv2d_bwd(geom, x, w, grad, dtype=np.float64):
    sfx, ct = _suffix(dtype)
    x, w, grad = _prep(x, dtype), _prep(w, dtype), _prep(grad, dtype)
    dw = np.empty((geom.co, geom.ci, geom.kh, geom.kw), dtype)
    dx = np.empty((geom.n, geom.ci, geom.h, geom.w), dtype)
    getattr(lib(), "qo_scalar_conv2d_bwd_weights" + sfx)(ctypes.byref(geom), _ptr(x, ct), _ptr(grad, ct), _ptr(dw, ct))
    getattr(lib(), "qo_scalar_conv2d_bwd_data" + sfx)(ctypes.byref(geom), _ptr(w, ct), _ptr(grad, ct), _ptr(dx, ct))
    return dw, dx


def conv2d_fwd(geom, x, w, bias=None, mode="generic", algebra=QUATERNION, real_valued_input=False,
               dtype=np.float64):
    """Algebra-dispatched Conv2D forward.  mode: 'generic' (N^2 scalar convolutions in the
    reference's term order), 'factorized' (8-lane quaternion path) or 'hamilton' (closed form,
    float64 quaternion only)."""
    sfx, ct = _suffix(dtype)
    dims = lib().qo_multivector_dim(algebra)
    x, w, bias = _prep(x, dtype), _prep(w, dtype), _prep(bias, dtype)
    rows = geom.n * dims
    y = np.empty((rows, geom.co, geom.ho, geom.wo), dtype)
    g = ctypes.byref(geom)
    if mode == "generic":
        _check(getattr(lib(), "qo_conv2d_fwd_generic" + sfx)(algebra, int(real_valued_input), g, _ptr(x, ct),
                                                             _ptr(w, ct), _ptr(bias, ct), _ptr(y, ct)))
    elif mode == "factorized":
        assert algebra == QUATERNION and not real_valued_input
        _check(getattr(lib(), "qo_conv2d_fwd_factorized" + sfx)(g, _ptr(x, ct), _ptr(w, ct), _ptr(bias, ct), _ptr(y, ct)))
    elif mode == "hamilton":
        assert algebra == QUATERNION and np.dtype(dtype) == np.float64
        lib().qo_qconv2d_fwd_hamilton(g, _ptr(x, ct), _ptr(w, ct), _ptr(bias, ct), _ptr(y, ct))
    else:
        raise ValueError(mode)
    return y


def conv2d_bwd(geom, x, w, grad, mode="generic", algebra=QUATERNION, need_dx=True, real_valued_input=False,
               dtype=np.float64):
    """Algebra-dispatched Conv2D backward: returns (dw, dx); dx is None when not required."""
    sfx, ct = _suffix(dtype)
    dims = lib().qo_multivector_dim(algebra)
    x, w, grad = _prep(x, dtype), _prep(w, dtype), _prep(grad, dtype)
    dw = np.empty((dims, geom.co, geom.ci, geom.kh, geom.kw), dtype)
    g = ctypes.byref(geom)
    if real_valued_input:
        _check(getattr(lib(), "qo_conv2d_bwd_real_input" + sfx)(algebra, g, _ptr(x, ct), _ptr(w, ct), _ptr(grad, ct),
                                                                _ptr(dw, ct)))
        return dw, None
    dx = np.empty((geom.n * dims, geom.ci, geom.h, geom.w), dtype) if need_dx else None
    if mode == "generic":
        _check(getattr(lib(), "qo_conv2d_bwd_generic" + sfx)(algebra, g, _ptr(x, ct), _ptr(w, ct), _ptr(grad, ct),
                                                             _ptr(dw, ct), _ptr(dx, ct), int(need_dx)))
    elif mode == "factorized":
        assert algebra == QUATERNION
        _check(getattr(lib(), "qo_conv2d_bwd_factorized" + sfx)(g, _ptr(x, ct), _ptr(w, ct), _ptr(grad, ct),
                                                                _ptr(dw, ct), _ptr(dx, ct), int(need_dx)))
    elif mode == "hamilton":
        assert algebra == QUATERNION and np.dtype(dtype) == np.float64
        lib().qo_qconv2d_bwd_weights_hamilton(g, _ptr(x, ct), _ptr(grad, ct), _ptr(dw, ct))
        if need_dx:
            lib().qo_qconv2d_bwd_data_hamilton(g, _ptr(w, ct), _ptr(grad, ct), _ptr(dx, ct))
    else:
        raise ValueError(mode)
    return dw, dx


def dense_fwd(x, w, bias=None, mode="generic", algebra=QUATERNION, dtype=np.float64):
    sfx, ct = _suffix(dtype)
    dims = lib().qo_multivector_dim(algebra)
    x, w, bias = _prep(x, dtype), _prep(w, dtype), _prep(bias, dtype)
    n, ni, no = x.shape[0] // dims, x.shape[1], w.shape[-1]
    assert w.shape[-2] == ni
    y = np.empty((n * dims, no), dtype)
    if mode == "generic":
        _check(getattr(lib(), "qo_dense_fwd_generic" + sfx)(algebra, n, ni, no, _ptr(x, ct), _ptr(w, ct), _ptr(bias, ct),
                                                            _ptr(y, ct)))
    elif mode == "factorized":
        assert algebra == QUATERNION
        _check(getattr(lib(), "qo_dense_fwd_factorized" + sfx)(n, ni, no, _ptr(x, ct), _ptr(w, ct), _ptr(bias, ct),
                                                               _ptr(y, ct)))
    else:
        raise ValueError(mode)
    return y


def dense_bwd(x, w, grad, mode="generic", algebra=QUATERNION, need_dx=True, dtype=np.float64):
    sfx, ct = _suffix(dtype)
    dims = lib().qo_multivector_dim(algebra)
    x, w, grad = _prep(x, dtype), _prep(w, dtype), _prep(grad, dtype)
    n, ni, no = x.shape[0] // dims, x.shape[1], w.shape[-1]
    dw = np.empty((dims, ni, no), dtype)
    dx = np.empty((n * dims, ni), dtype)
    if mode == "generic":
        _check(getattr(lib(), "qo_dense_bwd_generic" + sfx)(algebra, n, ni, no, _ptr(x, ct), _ptr(w, ct), _ptr(grad, ct),
                                                            _ptr(dw, ct), _ptr(dx, ct), int(need_dx)))
    elif mode == "factorized":
        assert algebra == QUATERNION
        _check(getattr(lib(), "qo_dense_bwd_factorized" + sfx)(n, ni, no, _ptr(x, ct), _ptr(w, ct), _ptr(grad, ct),
                                                               _ptr(dw, ct), _ptr(dx, ct), int(need_dx)))
    else:
        raise ValueError(mode)
    return dw, (dx if need_dx else None)


def lane_maps(dtype=np.float32):
    """The six elementwise lane maps of the factorized path as numpy-callable functions."""
    sfx, ct = _suffix(dtype)

    def make(name, nin, nout):
        fn = getattr(lib(), name + sfx)

        def call(arrs):
            arrs = [np.ascontiguousarray(a, dtype=dtype) for a in arrs]
            assert len(arrs) == nin
            outs = [np.empty_like(arrs[0]) for _ in range(nout)]
            pin = (ctypes.POINTER(ct) * nin)(*[_ptr(a, ct) for a in arrs])
            pout = (ctypes.POINTER(ct) * nout)(*[_ptr(a, ct) for a in outs])
            fn(pin, pout, ctypes.c_size_t(arrs[0].size))
            return outs
        return call

    return {
        "decompose_left": make("qo_decompose_left", 4, 8),
        "decompose_right": make("qo_decompose_right", 4, 8),
        "decompose_grad": make("qo_decompose_grad", 4, 8),
        "recompose_output": make("qo_recompose_output", 8, 4),
        "recompose_left_grad": make("qo_recompose_left_grad", 8, 4),
        "recompose_right_grad": make("qo_recompose_right_grad", 8, 4),
    }
