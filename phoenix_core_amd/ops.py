"""Python host side of the quaternion Conv2D / Dense operators.

Mirrors the reference's operator interface for this path -- descriptors that resolve padding and
output shapes (src/backend/conv2d_descriptor.hpp, src/backend/dense_descriptor.hpp, src/utils.cc),
a Context that reads the UPSTRIDE_* switches once (src/backend/backend.cc:45-48) and the four
entry points conv2DFwd / conv2DBwd / denseFwd / denseBwd (src/upstride.hpp:18-86) -- on torch
tensors, which serve only as device memory.  All arithmetic happens in the HIP library behind the
C ABI; nothing here computes on the CPU.  The algebras other than the quaternions are carried onto
the same kernels by rearrangement kernels inside the library (csrc/phx_algebra.hip).
"""
import ctypes
import os

import torch

from . import capi

REAL, COMPLEX, QUATERNION, GA_300 = 0, 1, 2, 3  # src/algebras.hpp:17-22


class Context:
    """Process-wide switches, read from the environment at construction like the reference's
    Context: UPSTRIDE_MEMORY_OPTIMIZED > 0 selects the 16-product path instead of the factorized
    8-product one; UPSTRIDE_CONV_FP16_POLICY in {full16, backward32} allows fp16 matrix-core
    arithmetic forward+backward / forward only (anything else: fp32)."""

    def __init__(self, environ=None):
        env = os.environ if environ is None else environ
        self.memory_optimized = _strtol(env.get("UPSTRIDE_MEMORY_OPTIMIZED")) > 0
        policy = env.get("UPSTRIDE_CONV_FP16_POLICY", "")
        self.fp16_policy = {"full16": capi.PHX_FP16_FULL16, "backward32": capi.PHX_FP16_BACKWARD32}.get(
            policy, capi.PHX_FP16_FULL32)

    def prefer_speed_to_memory(self):
        return not self.memory_optimized

    def is_fp16_conv_forward_allowed(self):
        return self.fp16_policy in (capi.PHX_FP16_FULL16, capi.PHX_FP16_BACKWARD32)

    def is_fp16_conv_backward_allowed(self):
        return self.fp16_policy == capi.PHX_FP16_FULL16

    @property
    def product_mode(self):
        return capi.PHX_PRODUCT_8 if self.prefer_speed_to_memory() else capi.PHX_PRODUCT_16


def _strtol(value):
    """C strtol(value, NULL, 10) semantics: leading blanks, optional sign, longest digit prefix."""
    if not value:
        return 0
    s = value.lstrip(" \t\n\v\f\r")
    sign = 1
    if s[:1] in "+-" and s[:1]:
        sign = -1 if s[0] == "-" else 1
        s = s[1:]
    digits = ""
    for ch in s:
        if not ch.isdigit() or not ch.isascii():
            break
        digits += ch
    return sign * int(digits) if digits else 0


def windowed_output_size_and_padding(size, filt, dilation, stride, padding):
    """SAME / VALID presets (src/utils.cc:10-39). Returns (out, before, after)."""
    effective = (filt - 1) * dilation + 1
    if padding == "VALID":
        return (size - effective + stride) // stride, 0, 0
    if padding == "SAME":
        out = (size + stride - 1) // stride
        needed = max(0, (out - 1) * stride + effective - size)
        return out, needed // 2, needed - needed // 2
    raise ValueError("Invalid padding")


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


_DTYPES = {torch.float32: capi.PHX_F32, torch.float16: capi.PHX_F16}


class Conv2DDescriptor:
    """Geometry of one convolution (Conv2DFwdDescriptor / Conv2DBwdDescriptor of the reference).  The quaternion
    algebra runs on the HIP kernels directly; REAL, COMPLEX and GA_300 run inside the library as one
    quaternion call on rearranged tensors (algebras.py resolves their shapes).  data_format "NCHW" takes activations [4n, c, h, w],
    "NHWC" [4n, h, w, c] (transposed inside the call: the kernels compute on channels-first planes)."""

    def __init__(self, input_shape, filter_shape, stride=1, dilation=1, padding="VALID", groups=1,
                 algebra=QUATERNION, filter_layout="OIHW", use_bias=False, dtype=torch.float32, context=None,
                 require_input_grad=True, real_valued_input=False, data_format="NCHW"):
        if len(input_shape) != 4:
            raise ValueError("Four-dimensional input tensor expected")
        self.algebra = algebra
        if algebra != QUATERNION:
            # the other algebras: same entry points, the descriptor carries the algebra (algebras.py)
            from . import algebras
            algebras.init_conv_descriptor(self, input_shape, filter_shape, algebra, groups, filter_layout, data_format,
                                          real_valued_input, stride=stride, dilation=dilation, padding=padding,
                                          use_bias=use_bias, dtype=dtype, context=context,
                                          require_input_grad=require_input_grad)
            return
        if len(filter_shape) != 5:
            raise ValueError("Five-dimensional filter tensor expected")
        if filter_shape[0] != 4:
            raise ValueError("First filter dimension mismatch, got %d" % filter_shape[0])
        if groups < 1:
            raise ValueError("groups must be positive")
        if not real_valued_input and input_shape[0] % 4:
            raise ValueError("Cannot split %d onto 4 parts" % input_shape[0])
        if filter_layout == "OIHW":
            _, co, ci, kh, kw = filter_shape
        elif filter_layout == "OHWI":
            _, co, kh, kw, ci = filter_shape
        elif filter_layout == "HWIO":
            _, kh, kw, ci, co = filter_shape
        else:
            raise ValueError("Unsupported Conv2D filter layout")
        # grouped convolution: the filter holds the input channels of one group (src/backend/conv2d_descriptor.hpp)
        ci *= groups
        if data_format not in ("NCHW", "NHWC"):
            raise ValueError("Unsupported data format")
        self.data_format = data_format
        n4, c_in, h, w = input_shape if data_format == "NCHW" else (input_shape[i] for i in (0, 3, 1, 2))
        if c_in != ci:
            raise ValueError("input channels %d do not match the filter's %d" % (c_in, ci))
        if co % groups:
            raise ValueError("output channels %d are not a multiple of %d groups" % (co, groups))
        self.groups = groups
        self.context = context or default_context()
        self.input_shape = tuple(input_shape)
        self.filter_shape = tuple(filter_shape)
        self.filter_layout = filter_layout
        self.stride, self.dilation = _pair(stride), _pair(dilation)
        self.use_bias = bool(use_bias)
        self.require_input_grad = bool(require_input_grad)
        self.dtype = dtype
        # real-valued input (realValuedInput of the reference's descriptors): [n, ci, h, w] without imaginary
        # parts; the output still has the four components stacked on the batch axis
        self.real_valued_input = bool(real_valued_input)
        if self.real_valued_input:
            n4 *= 4
        if isinstance(padding, str):
            ho, pt, pb = windowed_output_size_and_padding(h, kh, self.dilation[0], self.stride[0], padding)
            wo, pl, pr = windowed_output_size_and_padding(w, kw, self.dilation[1], self.stride[1], padding)
        else:  # explicit (top, left, bottom, right)
            pt, pl, pb, pr = padding
            ho = (h + pt + pb - ((kh - 1) * self.dilation[0] + 1) + self.stride[0]) // self.stride[0]
            wo = (w + pl + pr - ((kw - 1) * self.dilation[1] + 1) + self.stride[1]) // self.stride[1]
        self.pad_before, self.pad_after = (pt, pl), (pb, pr)
        self.output_shape = (n4, co, ho, wo) if data_format == "NCHW" else (n4, ho, wo, co)
        self.bias_shape = (4, co) if use_bias else ()
        self.c = capi.QConvDesc(
            _DTYPES[dtype], n4 // 4, ci, co, h, w, kh, kw, self.stride[0], self.stride[1], self.dilation[0],
            self.dilation[1], pt, pl, pb, pr, {"OIHW": capi.PHX_OIHW, "OHWI": capi.PHX_OHWI, "HWIO": capi.PHX_HWIO}[filter_layout],
            self.context.product_mode, self.context.fp16_policy, int(self.use_bias and not self.real_valued_input),
            int(self.real_valued_input), groups, capi.PHX_NCHW if data_format == "NCHW" else capi.PHX_NHWC)

    def workspace_bytes(self, which):
        return capi.lib().phx_qconv2d_workspace_bytes(ctypes.byref(self.c), which)


class DenseDescriptor:
    """DenseFwdDescriptor / DenseBwdDescriptor for the quaternion algebra; filter [4, in, out] ("IO") or
    [4, out, in] ("OI")."""

    def __init__(self, input_shape, filter_shape, algebra=QUATERNION, filter_layout="IO", use_bias=False,
                 dtype=torch.float32, context=None, require_input_grad=True):
        self.algebra = algebra
        if algebra != QUATERNION:
            from . import algebras
            algebras.init_dense_descriptor(self, input_shape, filter_shape, algebra, filter_layout, use_bias=use_bias,
                                           dtype=dtype, context=context, require_input_grad=require_input_grad)
            return
        if filter_layout not in ("IO", "OI"):
            raise ValueError("Unsupported Dense filter layout")
        if len(input_shape) != 2 or len(filter_shape) != 3 or filter_shape[0] != 4:
            raise ValueError("expected input [4n, in] and filter [4, in, out] (IO) or [4, out, in] (OI)")
        n_in, n_out = filter_shape[1:] if filter_layout == "IO" else filter_shape[:0:-1]
        self.filter_layout = filter_layout
        if input_shape[0] % 4:
            raise ValueError("Cannot split %d onto 4 parts" % input_shape[0])
        if input_shape[1] != n_in:
            raise ValueError("input features do not match the filter")
        self.context = context or default_context()
        self.input_shape, self.filter_shape = tuple(input_shape), tuple(filter_shape)
        self.use_bias, self.require_input_grad, self.dtype = bool(use_bias), bool(require_input_grad), dtype
        self.output_shape = (input_shape[0], n_out)
        self.bias_shape = (4, n_out) if use_bias else ()
        self.c = capi.QDenseDesc(_DTYPES[dtype], input_shape[0] // 4, n_in, n_out,
                                 self.context.product_mode, self.context.fp16_policy, int(self.use_bias),
                                 capi.PHX_IO if filter_layout == "IO" else capi.PHX_OI)

    def workspace_bytes(self, which):
        return capi.lib().phx_qdense_workspace_bytes(ctypes.byref(self.c), which)


_default_context = None


def default_context():
    global _default_context
    if _default_context is None:
        _default_context = Context()
    return _default_context


class _Workspace:
    """Grow-only scratch buffer per device and stream, shared by the operations enqueued there (the reference's
    Device keeps one workspace for all its operations, src/backend/device.hpp:75-84, and serializes them with a
    mutex; here the stream's own order serializes them, and calls on different streams get different buffers)."""

    def __init__(self):
        self.buffers = {}

    def get(self, device, nbytes, stream=None):
        key = (device, current_stream_handle(device) if stream is None else stream)
        buf = self.buffers.get(key)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
            self.buffers[key] = buf
        return buf


    def holds(self, device, stream, nbytes):
        """Whether the buffer of that stream is already large enough (no allocation would happen)."""
        buf = self.buffers.get((device, stream))
        return buf is not None and buf.numel() >= nbytes


_workspace = _Workspace()

# torch.cuda.current_stream() builds a Stream object through several Python layers (6-7 us per call, twice per
# operator call); the raw handle is all the library needs
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_handle(device):
    """The handle of the device's current stream, as an integer."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _dev_check(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("phoenix_core_amd operators run on the GPU only; got a %s tensor" % t.device)
        if not t.is_contiguous():
            raise ValueError("tensors must be contiguous")
        dev = t.device
    return dev


def _expect(t, shape, dtype, what):
    """The library reads raw device memory in the descriptor's type and shape: anything else is refused here."""
    if t is None:
        raise ValueError("%s tensor missing" % what)
    if tuple(t.shape) != tuple(shape):
        raise ValueError("%s has shape %s, the descriptor says %s" % (what, tuple(t.shape), tuple(shape)))
    if t.dtype != dtype:
        raise ValueError("%s has dtype %s, the descriptor says %s" % (what, t.dtype, dtype))


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def workspace_holds(device, stream, nbytes):
    """Whether the scratch buffer of that stream (a handle) already has nbytes: a call on it then allocates nothing."""
    return _workspace.holds(device, stream, int(nbytes))


def reserve_workspace(nbytes, device=None):
    """Grows the scratch buffer of the current stream to at least nbytes ahead of time -- in front of a stream
    capture, inside which the buffer must not be reallocated."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    return _workspace.get(device, int(nbytes))


def _stream(device, stream=None):
    return ctypes.c_void_p(current_stream_handle(device) if stream is None else stream)


class PackedFilters:
    """A convolution's filter in the operand order of its forward and input-gradient kernels
    (phx_qconv2d_pack_filters): made once per filter update, read by conv2d_fwd / conv2d_bwd_data through their
    `packed` argument instead of packing in every call.  Either image may be None (no prepacked form for that
    pass, or not asked for)."""

    def __init__(self, fwd, bwd_data, filter_shape, dtype, layout_key=None):
        self.fwd, self.bwd_data, self.filter_shape, self.dtype = fwd, bwd_data, tuple(filter_shape), dtype
        self.layout_key = layout_key

    def check(self, desc):
        """The images' layout follows the plan of the descriptor they were packed for (sizes, strides, padding,
        product mode, policy, groups, data format) under the tuning in force then: any other descriptor is refused."""
        if self.filter_shape != tuple(desc.filter_shape) or self.dtype != desc.dtype or \
                (self.layout_key is not None and self.layout_key != _layout_key(desc)):
            raise ValueError("these packed filters belong to another descriptor")


def _layout_key(desc):
    """Everything of a descriptor that a packed image depends on: its C struct without the bias flag (the forward
    and backward descriptors of one layer differ in it and share their images) + the tuning generation."""
    c = capi.QConvDesc.from_buffer_copy(bytes(desc.c))
    c.has_bias = 0
    return bytes(c), capi.tuning_generation


def conv2d_packed_filter_bytes(desc, which):
    """Bytes of the packed filter image of a pass (0: that pass of this descriptor has no prepacked form)."""
    if desc.algebra != QUATERNION:
        return 0
    return capi.lib().phx_qconv2d_packed_filter_bytes(ctypes.byref(desc.c), which)


def conv2d_pack_filters(w, desc, bwd_data=True, into=None):
    """Packs w for the forward pass and (bwd_data) the input gradient of desc with one kernel launch; `into`: a
    PackedFilters of the same descriptor to overwrite (no allocation).  Returns None when neither pass has a
    prepacked form."""
    dev = _dev_check(w)
    _expect(w, desc.filter_shape, desc.dtype, "filter")
    if into is None:
        nf = conv2d_packed_filter_bytes(desc, capi.PHX_PASS_FWD)
        nb = conv2d_packed_filter_bytes(desc, capi.PHX_PASS_BWD_DATA) if bwd_data and not desc.real_valued_input else 0
        if nf == 0 and nb == 0:
            return None
        into = PackedFilters(torch.empty(nf, dtype=torch.uint8, device=dev) if nf else None,
                             torch.empty(nb, dtype=torch.uint8, device=dev) if nb else None, desc.filter_shape, desc.dtype,
                             _layout_key(desc))
    else:
        into.check(desc)
    f, b = into.fwd, into.bwd_data
    capi.check(capi.lib().phx_qconv2d_pack_filters(ctypes.byref(desc.c), _stream(dev), _ptr(w), _ptr(f), f.numel() if f is not None else 0,
                                                   _ptr(b), b.numel() if b is not None else 0), "phx_qconv2d_pack_filters")
    return into


def conv2d_fwd(x, w, bias, desc, out=None, packed=None):
    """conv2DFwd (src/upstride.hpp:18-33): y = x (x) w (+ bias).  packed: PackedFilters of (w, desc) -- the call
    then reads the packed image and not w."""
    dev = _dev_check(x, w, bias, out)
    _expect(x, desc.input_shape, desc.dtype, "input")
    _expect(w, desc.filter_shape, desc.dtype, "filter")
    if desc.use_bias:
        _expect(bias, desc.bias_shape, desc.dtype, "bias")
    if desc.real_valued_input and desc.use_bias:  # src/conv2d.hpp:125-127
        raise RuntimeError("Bias addition is not supported for type0 inputs")
    if out is not None:
        _expect(out, desc.output_shape, desc.dtype, "output")
    y = out if out is not None else torch.empty(desc.output_shape, dtype=desc.dtype, device=dev)
    nbytes = desc.workspace_bytes(capi.PHX_PASS_FWD)
    ws = _workspace.get(dev, nbytes)
    if packed is not None and packed.fwd is not None:
        packed.check(desc)
        capi.check(capi.lib().phx_qconv2d_fwd_prepacked(ctypes.byref(desc.c), _stream(dev), _ptr(x), _ptr(packed.fwd),
                                                        packed.fwd.numel(), _ptr(bias if desc.use_bias else None), _ptr(y),
                                                        _ptr(ws), nbytes), "phx_qconv2d_fwd_prepacked")
        return y
    capi.check(capi.lib().phx_qconv2d_fwd(ctypes.byref(desc.c), _stream(dev), _ptr(x), _ptr(w),
                                          _ptr(bias if desc.use_bias else None), _ptr(y), _ptr(ws), nbytes),
               "phx_qconv2d_fwd")
    return y


def conv2d_bwd_weights(x, grad, desc, stream=None):
    """The filter-gradient half of conv2DBwd (src/conv2d.hpp:330-440): dw.  stream: the handle of a stream to enqueue
    on instead of the device's current one; the caller then orders that stream behind the producers of x and grad
    and the consumers of dw behind it (dw itself is allocated on the current stream)."""
    dev = _dev_check(x, grad)
    _expect(x, desc.input_shape, desc.dtype, "input")
    _expect(grad, desc.output_shape, desc.dtype, "output gradient")
    dw = torch.empty(desc.filter_shape, dtype=desc.dtype, device=dev)
    nbytes = desc.workspace_bytes(capi.PHX_PASS_BWD_WEIGHTS)
    ws = _workspace.get(dev, nbytes, stream)
    capi.check(capi.lib().phx_qconv2d_bwd_weights(ctypes.byref(desc.c), _stream(dev, stream), _ptr(x), _ptr(grad), _ptr(dw),
                                                  _ptr(ws), nbytes), "phx_qconv2d_bwd_weights")
    return dw


def conv2d_bwd_data(w, grad, desc, packed=None, addend=None):
    """The input-gradient half of conv2DBwd: dx (the descriptor must ask for it).  packed: as in conv2d_fwd.
    addend: a tensor like dx that is added to it (phx_qconv2d_bwd_data_add: in the kernel's epilogue where it can,
    the same values as dx + addend either way); quaternion descriptors only."""
    dev = _dev_check(w, grad, addend)
    _expect(w, desc.filter_shape, desc.dtype, "filter")
    _expect(grad, desc.output_shape, desc.dtype, "output gradient")
    if desc.real_valued_input:  # src/conv2d.hpp:394-398
        raise RuntimeError("Input gradient required for type0 input tensor")
    dx = torch.empty(desc.input_shape, dtype=desc.dtype, device=dev)
    nbytes = desc.workspace_bytes(capi.PHX_PASS_BWD_DATA)
    ws = _workspace.get(dev, nbytes)
    if addend is not None:
        _expect(addend, desc.input_shape, desc.dtype, "addend")
        image = packed.bwd_data if packed is not None else None
        if image is not None:
            packed.check(desc)
        capi.check(capi.lib().phx_qconv2d_bwd_data_add(ctypes.byref(desc.c), _stream(dev), _ptr(grad), _ptr(w), _ptr(image),
                                                       image.numel() if image is not None else 0, _ptr(addend), _ptr(dx),
                                                       _ptr(ws), nbytes), "phx_qconv2d_bwd_data_add")
        return dx
    if packed is not None and packed.bwd_data is not None:
        packed.check(desc)
        capi.check(capi.lib().phx_qconv2d_bwd_data_prepacked(ctypes.byref(desc.c), _stream(dev), _ptr(grad), _ptr(packed.bwd_data),
                                                             packed.bwd_data.numel(), _ptr(dx), _ptr(ws), nbytes),
                   "phx_qconv2d_bwd_data_prepacked")
        return dx
    capi.check(capi.lib().phx_qconv2d_bwd_data(ctypes.byref(desc.c), _stream(dev), _ptr(grad), _ptr(w), _ptr(dx),
                                               _ptr(ws), nbytes), "phx_qconv2d_bwd_data")
    return dx


def conv2d_bwd(x, w, grad, desc):
    """conv2DBwd (src/upstride.hpp:35-51): returns (dw, dx); dx is None when the descriptor does
    not require the input gradient."""
    _dev_check(x, w, grad)
    _expect(w, desc.filter_shape, desc.dtype, "filter")
    dw = conv2d_bwd_weights(x, grad, desc)
    dx = conv2d_bwd_data(w, grad, desc) if desc.require_input_grad else None
    return dw, dx


def dense_fwd(x, w, bias, desc, out=None):
    """denseFwd (src/upstride.hpp:53-68)."""
    dev = _dev_check(x, w, bias, out)
    _expect(x, desc.input_shape, desc.dtype, "input")
    _expect(w, desc.filter_shape, desc.dtype, "filter")
    if desc.use_bias:
        _expect(bias, desc.bias_shape, desc.dtype, "bias")
    if out is not None:
        _expect(out, desc.output_shape, desc.dtype, "output")
    y = out if out is not None else torch.empty(desc.output_shape, dtype=desc.dtype, device=dev)
    nbytes = desc.workspace_bytes(capi.PHX_PASS_FWD)
    ws = _workspace.get(dev, nbytes)
    capi.check(capi.lib().phx_qdense_fwd(ctypes.byref(desc.c), _stream(dev), _ptr(x), _ptr(w),
                                         _ptr(bias if desc.use_bias else None), _ptr(y), _ptr(ws), nbytes),
               "phx_qdense_fwd")
    return y


def dense_bwd(x, w, grad, desc):
    """denseBwd (src/upstride.hpp:70-86): returns (dw, dx)."""
    dev = _dev_check(x, w, grad)
    _expect(x, desc.input_shape, desc.dtype, "input")
    _expect(w, desc.filter_shape, desc.dtype, "filter")
    _expect(grad, desc.output_shape, desc.dtype, "output gradient")
    dw = torch.empty(desc.filter_shape, dtype=desc.dtype, device=dev)
    nbytes = desc.workspace_bytes(capi.PHX_PASS_BWD_WEIGHTS)
    ws = _workspace.get(dev, nbytes)
    capi.check(capi.lib().phx_qdense_bwd_weights(ctypes.byref(desc.c), _stream(dev), _ptr(x), _ptr(grad), _ptr(dw),
                                                 _ptr(ws), nbytes), "phx_qdense_bwd_weights")
    dx = None
    if desc.require_input_grad:
        dx = torch.empty(desc.input_shape, dtype=desc.dtype, device=dev)
        nbytes = desc.workspace_bytes(capi.PHX_PASS_BWD_DATA)
        ws = _workspace.get(dev, nbytes)
        capi.check(capi.lib().phx_qdense_bwd_data(ctypes.byref(desc.c), _stream(dev), _ptr(grad), _ptr(w), _ptr(dx),
                                                  _ptr(ws), nbytes), "phx_qdense_bwd_data")
    return dw, dx


def batch_norm_fwd(x, gamma, beta, running_mean, running_var, eps, momentum, relu, residual=None):
    """Training-mode batch normalisation (+ residual, + ReLU) of [rows, C, H, W] (include/phx_bn.h; no counterpart in
    the reference, which holds no model code).  Returns (y, save_mean, save_invstd); the running statistics are
    updated in place when given."""
    dev = _dev_check(x, gamma, beta, running_mean, running_var, residual)
    if residual is not None and (residual.shape != x.shape or residual.dtype != x.dtype):
        raise ValueError("the residual must have the shape and type of the input")
    rows, c = x.shape[0], x.shape[1]
    if x.dtype not in _DTYPES:
        raise ValueError("batch normalisation takes float32 or float16 activations")
    for t, what in ((gamma, "gamma"), (beta, "beta"), (running_mean, "running_mean"), (running_var, "running_var")):
        if t is not None:
            _expect(t, (c,), torch.float32, what)
    hw = x.numel() // max(rows * c, 1)
    desc = capi.BnDesc(_DTYPES[x.dtype], rows, c, hw, eps, momentum, int(relu))
    y = torch.empty_like(x)
    mean = torch.empty(c, dtype=torch.float32, device=dev)
    invstd = torch.empty(c, dtype=torch.float32, device=dev)
    nbytes = capi.lib().phx_bn_workspace_bytes(ctypes.byref(desc))
    ws = _workspace.get(dev, nbytes)
    capi.check(capi.lib().phx_bn_fwd_train(ctypes.byref(desc), _stream(dev), _ptr(x), _ptr(residual), _ptr(gamma), _ptr(beta),
                                           _ptr(y), _ptr(mean), _ptr(invstd), _ptr(running_mean), _ptr(running_var),
                                           _ptr(ws), nbytes), "phx_bn_fwd_train")
    return y, mean, invstd


def batch_norm_bwd(x, dy, gamma, beta, mean, invstd, eps, relu, residual=None):
    """Returns (dx, dgamma, dbeta, dresidual) of batch_norm_fwd; dresidual is None without a residual."""
    dev = _dev_check(x, dy, gamma, beta, mean, invstd, residual)
    rows, c = x.shape[0], x.shape[1]
    if x.dtype not in _DTYPES:
        raise ValueError("batch normalisation takes float32 or float16 activations")
    _expect(dy, x.shape, x.dtype, "output gradient")
    if residual is not None:
        _expect(residual, x.shape, x.dtype, "residual")
    for t, what in ((gamma, "gamma"), (beta, "beta"), (mean, "mean"), (invstd, "invstd")):
        _expect(t, (c,), torch.float32, what)
    hw = x.numel() // max(rows * c, 1)
    desc = capi.BnDesc(_DTYPES[x.dtype], rows, c, hw, eps, 0.0, int(relu))
    dx = torch.empty_like(x)
    dres = torch.empty_like(x) if residual is not None else None
    empty = rows * hw == 0  # nothing is enqueued then: the parameter gradients are zero
    dgamma = (torch.zeros if empty else torch.empty)(c, dtype=torch.float32, device=dev)
    dbeta = (torch.zeros if empty else torch.empty)(c, dtype=torch.float32, device=dev)
    nbytes = capi.lib().phx_bn_workspace_bytes(ctypes.byref(desc))
    ws = _workspace.get(dev, nbytes)
    capi.check(capi.lib().phx_bn_bwd(ctypes.byref(desc), _stream(dev), _ptr(x), _ptr(residual), _ptr(dy), _ptr(gamma),
                                     _ptr(beta), _ptr(mean), _ptr(invstd), _ptr(dx), _ptr(dres), _ptr(dgamma), _ptr(dbeta),
                                     _ptr(ws), nbytes), "phx_bn_bwd")
    return dx, dgamma, dbeta, dres


def max_pool_3x3s2_fwd(x):
    """3x3 max pooling, stride 2, padding 1, of x [rows, C, H, W] (include/phx_pool.h): returns (y, index) with
    index [rows, C, Ho, Wo] uint8 = the window position 0..8 that held the maximum (max_pool_3x3s2_bwd reads it)."""
    dev = _dev_check(x)
    if x.dtype not in _DTYPES or x.dim() != 4:
        raise ValueError("max pooling takes a float32 or float16 tensor [rows, C, H, W]")
    rows, c, h, w = x.shape
    ho, wo = ((h - 1) // 2 + 1, (w - 1) // 2 + 1) if h and w else (0, 0)
    y = torch.empty((rows, c, ho, wo), dtype=x.dtype, device=dev)
    index = torch.empty((rows, c, ho, wo), dtype=torch.uint8, device=dev)
    capi.check(capi.lib().phx_maxpool3x3s2_fwd(_DTYPES[x.dtype], rows * c, h, w, _stream(dev), _ptr(x), _ptr(y), _ptr(index)),
               "phx_maxpool3x3s2_fwd")
    return y, index


def max_pool_3x3s2_bwd(dy, index, input_shape):
    """Gradient of max_pool_3x3s2_fwd with respect to its input of shape input_shape."""
    dev = _dev_check(dy, index)
    rows, c, h, w = input_shape
    ho, wo = ((h - 1) // 2 + 1, (w - 1) // 2 + 1) if h and w else (0, 0)
    if dy.dtype not in _DTYPES:
        raise ValueError("max pooling takes float32 or float16 gradients")
    _expect(dy, (rows, c, ho, wo), dy.dtype, "output gradient")
    _expect(index, (rows, c, ho, wo), torch.uint8, "index")
    dx = torch.empty(tuple(input_shape), dtype=dy.dtype, device=dev)
    capi.check(capi.lib().phx_maxpool3x3s2_bwd(_DTYPES[dy.dtype], rows * c, h, w, _stream(dev), _ptr(dy), _ptr(index), _ptr(dx)),
               "phx_maxpool3x3s2_bwd")
    return dx
