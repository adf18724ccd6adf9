"""Descriptors of Conv2D and Dense in the reference's other algebras -- REAL, COMPLEX, GA_300 (src/algebras.hpp:17-22;
sign tables src/algebras.cc:5-145).

The library runs them as one quaternion call on rearranged tensors (csrc/phx_algebra.hip): a GA_300 multivector
(blades 1, e1, e2, e3, e12, e13, e23, e123) is A + e123 B with quaternion-like A = (m0, m4, m5, -m6) and
B = (m7, -m3, m2, m1), and (A1 + I B1)(A2 + I B2) = (A1 A2 - B1 B2) + I (A1 B2 + B1 A2), i.e. one quaternion
convolution of twice the channel counts; COMPLEX and REAL run in place as a quaternion problem on paired /
quadrupled images (half / a quarter of the batch; batches that do not divide are embedded with zero components).
This module only
resolves shapes and fills the C descriptors with the algebra; the entry points of `ops` then take the tensors in
the algebra's own layout: activations [D n, C, H, W] (or [D n, H, W, C]), filters [D] x the layout's axes (OIHW,
OHWI, HWIO; Dense IO, OI; REAL: no blade axis; with groups the input-channel axis holds one group's channels),
bias [D, Co] -- as the reference's generic path takes them for every algebra (src/conv2d.hpp:237-275).  A
real-valued input is taken by the quaternion algebra only."""
import ctypes

from . import capi, ops

DIMS = {ops.REAL: 1, ops.COMPLEX: 2, ops.QUATERNION: 4, ops.GA_300: 8}  # MULTIVECTOR_DIM, src/algebras.hpp:26
_C_ALGEBRA = {ops.REAL: capi.PHX_REAL, ops.COMPLEX: capi.PHX_COMPLEX, ops.QUATERNION: capi.PHX_QUATERNION,
              ops.GA_300: capi.PHX_GA_300}


def blade_map(algebra):
    """(dims, halves, blade[8], sign[8]) of the library's rearrangement: quaternion component p of half h is
    sign[4 h + p] * blade[4 h + p] (blade -1: zero).  Host-only call."""
    dims, halves = ctypes.c_int32(), ctypes.c_int32()
    blade, sign = (ctypes.c_int32 * 8)(), (ctypes.c_int32 * 8)()
    capi.check(capi.lib().phx_algebra_map(_C_ALGEBRA[algebra], ctypes.byref(dims), ctypes.byref(halves), blade, sign),
               "phx_algebra_map")
    return dims.value, halves.value, list(blade), list(sign)


def init_conv_descriptor(desc, input_shape, filter_shape, algebra, groups, filter_layout, data_format, real_valued_input,
                         **kwargs):
    """Fills an ops.Conv2DDescriptor of a non-quaternion algebra: the geometry is that of a quaternion convolution of
    the same channel counts (resolved by a descriptor of that kind), the shapes carry the algebra's blade count."""
    if algebra not in DIMS:
        raise ValueError("unknown algebra")
    if real_valued_input:
        raise NotImplementedError("a real-valued input is taken by the quaternion algebra only")
    d = DIMS[algebra]
    # a real-valued filter has no blade axis (src/backend/conv2d_descriptor.hpp:14-37)
    if len(filter_shape) != (4 if algebra == ops.REAL else 5):
        raise ValueError("filter rank does not match the algebra")
    fs = tuple(filter_shape) if algebra != ops.REAL else (1,) + tuple(filter_shape)
    if fs[0] != d:
        raise ValueError("First filter dimension mismatch, got %d" % fs[0])
    if input_shape[0] % d:
        raise ValueError("Cannot split %d onto %d parts" % (input_shape[0], d))
    n = input_shape[0] // d
    geom = ops.Conv2DDescriptor((4 * n,) + tuple(input_shape[1:]), (4,) + fs[1:], groups=groups, filter_layout=filter_layout,
                                data_format=data_format, **kwargs)
    desc.c = capi.QConvDesc.from_buffer_copy(geom.c)
    desc.c.algebra = _C_ALGEBRA[algebra]
    desc.algebra = algebra
    desc.input_shape, desc.filter_shape = tuple(input_shape), tuple(filter_shape)
    desc.output_shape = (d * n,) + geom.output_shape[1:]
    desc.use_bias, desc.require_input_grad, desc.dtype = geom.use_bias, geom.require_input_grad, geom.dtype
    co = geom.c.co
    desc.bias_shape = ((d, co) if algebra != ops.REAL else (co,)) if desc.use_bias else ()
    desc.stride, desc.dilation, desc.pad_before, desc.pad_after = geom.stride, geom.dilation, geom.pad_before, geom.pad_after
    desc.context, desc.groups, desc.filter_layout, desc.data_format = geom.context, groups, filter_layout, data_format
    desc.real_valued_input = False


def init_dense_descriptor(desc, input_shape, filter_shape, algebra, filter_layout, **kwargs):
    if algebra not in DIMS:
        raise ValueError("unknown algebra")
    if filter_layout not in ("IO", "OI"):
        raise ValueError("Unsupported Dense filter layout")
    d = DIMS[algebra]
    if len(input_shape) != 2 or len(filter_shape) != (2 if algebra == ops.REAL else 3):
        raise ValueError("expected input [D n, in] and filter [D, in, out] (IO) or [D, out, in] (OI)")
    fs = tuple(filter_shape) if algebra != ops.REAL else (1,) + tuple(filter_shape)
    n_in, n_out = fs[1:] if filter_layout == "IO" else fs[:0:-1]
    if fs[0] != d or input_shape[0] % d or input_shape[1] != n_in:
        raise ValueError("Dense shapes do not match the algebra")
    n = input_shape[0] // d
    geom = ops.DenseDescriptor((4 * n, n_in), (4,) + fs[1:], filter_layout=filter_layout, **kwargs)
    desc.c = capi.QDenseDesc.from_buffer_copy(geom.c)
    desc.c.algebra = _C_ALGEBRA[algebra]
    desc.algebra, desc.filter_layout = algebra, filter_layout
    desc.input_shape, desc.filter_shape, desc.output_shape = tuple(input_shape), tuple(filter_shape), (d * n, n_out)
    desc.use_bias, desc.require_input_grad, desc.dtype, desc.context = geom.use_bias, geom.require_input_grad, geom.dtype, geom.context
    desc.bias_shape = ((d, n_out) if algebra != ops.REAL else (n_out,)) if desc.use_bias else ()
