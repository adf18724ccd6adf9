"""torch.autograd wrappers over the quaternion operators and a quaternion ResNet-50.

The reference engine was consumed by an external framework plugin that registered its operators
with gradients; this module plays that role for PyTorch.  QConv2d / QLinear hold the reference's
tensor layouts (components stacked on the batch axis, filters [4, Co, Ci, Kh, Kw], dense filters
[4, I, O]); every forward / backward call goes through the HIP library.  The ResNet-50 below is
the standard bottleneck stack with every channel count divided by four (quaternion channels);
batch-norm with its ReLU and the stem's max-pool run on the library's streaming kernels (include/phx_bn.h,
include/phx_pool.h) or on torch's modules; the loss is plain PyTorch (the reference has no model code).
"""
import math
import os

import torch
from torch import nn

from . import capi, ops


# The two gradients of a convolution are independent of each other.  With OVERLAP_BACKWARD the filter gradient is
# enqueued on a second stream (default priority) between two joins with the caller's stream, so that on layers too
# small to fill the GPU the two kernels run side by side.
OVERLAP_BACKWARD = True
# The bottleneck blocks' first convolution takes the identity branch's gradient into its own input gradient.
FUSE_BRANCH_GRADIENT = True
_side_streams = {}


def _side_stream(device):
    s = _side_streams.get(device)
    if s is None:
        s = _side_streams[device] = torch.cuda.Stream(device=device)
    return s


_stream_objects = {}


def _current_stream(device):
    """torch.cuda.current_stream(device) without building a new Stream object per call (6-7 us): one object per
    stream handle is kept."""
    key = (device, ops.current_stream_handle(device))
    s = _stream_objects.get(key)
    if s is None:
        s = _stream_objects[key] = torch.cuda.current_stream(device)
    return s


def _capturing():
    return torch.cuda.is_current_stream_capturing()


_events = {}


def _fork_join_events(device):
    e = _events.get(device)
    if e is None:
        e = _events[device] = (torch.cuda.Event(), torch.cuda.Event())
    return e


# QConv2d keeps its filter packed for the forward and input-gradient kernels (ops.PackedFilters) and packs again
# only after the filter has changed -- once per optimizer step while training, never while serving -- instead of
# in every forward and every backward call.
PREPACK_FILTERS = os.environ.get("PHX_NO_PREPACK", "") in ("", "0")


def _conv_backward(x, w, grad, bdesc, packed=None, addend=None):
    """(dw, dx); addend: a second gradient of x (from another consumer of x) that the input gradient takes in."""
    if not (OVERLAP_BACKWARD and bdesc.require_input_grad):
        dw = ops.conv2d_bwd_weights(x, grad, bdesc)
        return dw, (ops.conv2d_bwd_data(w, grad, bdesc, packed=packed, addend=addend) if bdesc.require_input_grad else None)
    dev = x.device
    main, side = _current_stream(dev), _side_stream(dev)
    side_handle = side.cuda_stream
    if (not torch.cuda.is_current_stream_capturing()
            and ops.workspace_holds(dev, side_handle, bdesc.workspace_bytes(capi.PHX_PASS_BWD_WEIGHTS))):
        # The short way (an eager training step is bound by the host): the filter gradient goes to the side stream
        # by its handle, torch's current stream stays what it is, and the fork and the join are two events kept
        # per device.  dw is allocated on the caller's stream, which waits for the side stream before anything
        # else touches dw, x or grad, so the allocator's per-stream bookkeeping needs no help.
        fork, join = _fork_join_events(dev)
        fork.record(main)
        side.wait_event(fork)
        dw = ops.conv2d_bwd_weights(x, grad, bdesc, stream=side_handle)
        dx = ops.conv2d_bwd_data(w, grad, bdesc, packed=packed, addend=addend)
        join.record(side)
        main.wait_event(join)
        return dw, dx
    # under stream capture, or while the side stream's scratch buffer still has to grow (an allocation, which
    # must happen with the side stream current): torch's own stream switch and fresh events
    side.wait_stream(main)  # x and grad are complete where the side stream starts
    with torch.cuda.stream(side):
        dw = ops.conv2d_bwd_weights(x, grad, bdesc)
    dx = ops.conv2d_bwd_data(w, grad, bdesc, packed=packed, addend=addend)
    main.wait_stream(side)  # whatever follows on the caller's stream may read dw (and free x, grad)
    dw.record_stream(main)
    return dw, dx


class _QConv2dFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, bias, fdesc, bdesc, packed=None, passthrough=False):
        ctx.save_for_backward(x, w)
        ctx.bdesc = bdesc
        ctx.has_bias = bias is not None
        ctx.packed = packed
        ctx.passthrough = passthrough
        y = ops.conv2d_fwd(x, w, bias, fdesc, packed=packed)
        if passthrough:
            # x is handed on as a second output: whatever else consumes x consumes THAT, so its gradient arrives
            # here with y's, and the input gradient adds it in its own kernel instead of autograd in a pass of its own
            ctx.set_materialize_grads(False)
            return y, x.view_as(x)
        return y

    @staticmethod
    def backward(ctx, grad, grad_through=None):
        x, w = ctx.saved_tensors  # (autograd refuses a filter modified since the forward pass: the packed images match it)
        if grad is None:  # (only with passthrough: y had no consumer)
            return grad_through, None, None, None, None, None, None
        grad = grad.contiguous()
        addend = grad_through.contiguous() if grad_through is not None and ctx.bdesc.require_input_grad else None
        dw, dx = _conv_backward(x, w, grad, ctx.bdesc, ctx.packed, addend)
        db = None
        if ctx.has_bias:  # bias enters every output component once: plain reduction
            n = grad.shape[0] // 4
            if ctx.bdesc.data_format == "NHWC":
                db = grad.view(4, n, -1, grad.shape[3]).float().sum(dim=(1, 2)).to(grad.dtype)
            else:
                db = grad.view(4, n, grad.shape[1], -1).float().sum(dim=(1, 3)).to(grad.dtype)
        return dx, dw, db, None, None, None, None


class _QLinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, bias, fdesc, bdesc):
        ctx.save_for_backward(x, w)
        ctx.bdesc = bdesc
        ctx.has_bias = bias is not None
        return ops.dense_fwd(x, w, bias, fdesc)

    @staticmethod
    def backward(ctx, grad):
        x, w = ctx.saved_tensors
        grad = grad.contiguous()
        dw, dx = ops.dense_bwd(x, w, grad, ctx.bdesc)
        db = None
        if ctx.has_bias:
            n = grad.shape[0] // 4
            db = grad.view(4, n, -1).float().sum(dim=1).to(grad.dtype)
        return dx, dw, db, None, None


class QConv2d(nn.Module):
    """Quaternion Conv2D: x [4N, Ci, H, W] -> y [4N, Co, Ho, Wo]; padding 'SAME' / 'VALID' as in
    the reference's descriptors (src/backend/conv2d_descriptor.hpp:132-174).  With real_input the
    layer takes a real tensor [N, Ci, H, W] (realValuedInput of the reference) and, as there, gives
    no gradient for it.  groups > 1: grouped convolution, filter [4, Co, Ci / groups, Kh, Kw].  data_format
    "NHWC": activations [4N, H, W, C] (the filter stays OIHW)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding="SAME", dilation=1, bias=False,
                 dtype=torch.float32, context=None, input_requires_grad=True, real_input=False, groups=1,
                 data_format="NCHW"):
        super().__init__()
        if in_channels % groups or out_channels % groups:
            raise ValueError("channel counts must be multiples of groups")
        self.real_input, self.groups, self.data_format = real_input, groups, data_format
        in_channels //= groups  # per group from here on: fan-in and the filter's input-channel axis
        input_requires_grad = input_requires_grad and not real_input
        k = (kernel_size, kernel_size) if isinstance(kernel_size, int) else tuple(kernel_size)
        self.stride, self.padding, self.dilation = stride, padding, dilation
        self.context = context
        self.input_requires_grad = input_requires_grad
        fan_in = in_channels * k[0] * k[1]
        w = torch.randn(4, out_channels, in_channels, k[0], k[1]) * math.sqrt(2.0 / fan_in)  # He-normal per component
        self.weight = nn.Parameter(w.to(dtype))
        self.bias = nn.Parameter(torch.zeros(4, out_channels, dtype=dtype)) if bias else None
        self._descs = {}
        self._packed = {}  # per descriptor pair: [filter state the images were packed from, ops.PackedFilters or None]
        self._pack_event = None    # kept per layer: marks the end of a pack enqueued on another stream (repack_filters)
        self._pack_pending = False  # ... which the next forward call has to wait for

    def _packed_filters(self, key, fwd):
        """The filter packed for this input shape, repacked (one launch, no allocation) if the filter has changed
        since: in-place updates are seen by the tensor's version counter, replaced storage by its address."""
        if not PREPACK_FILTERS:
            return None
        packed_ahead = self._pack_pending  # repack_filters() has packed this step's images on the second stream
        if self._pack_pending:
            _current_stream(self.weight.device).wait_event(self._pack_event)
            self._pack_pending = False
        w = self.weight
        state = (w._version, w.data_ptr())
        ent = self._packed.get(key)
        if ent is None:
            ent = self._packed[key] = [state, ops.conv2d_pack_filters(w.detach(), fwd, bwd_data=self.input_requires_grad)]
        elif ent[1] is not None and (ent[0] != state or (_capturing() and not packed_ahead)):
            # Under stream capture the check above runs once, at capture time, while the graph is replayed after
            # every later update of the filter: the packing launch has to be part of the graph whether or not the
            # filter has changed since the last call.
            ops.conv2d_pack_filters(w.detach(), fwd, into=ent[1])
            ent[0] = state
        return ent[1]

    def _repack_stale(self):
        """Packs again, on the current stream, every image whose filter has changed; True if there was one."""
        w = self.weight
        state = (w._version, w.data_ptr())
        packed = False
        capturing = _capturing()  # (a captured step packs unconditionally: see _packed_filters)
        for key, ent in self._packed.items():
            if ent[1] is not None and (ent[0] != state or capturing):
                ops.conv2d_pack_filters(w.detach(), self._descs[key][0], into=ent[1])
                ent[0] = state
                packed = True
        return packed

    def invalidate_packed_filters(self):
        """Forces the next forward call to pack again (for a filter changed behind the version counter's back,
        e.g. through .data)."""
        for ent in self._packed.values():
            ent[0] = None

    def _descriptors(self, x):
        key = (tuple(x.shape), x.dtype)
        if key not in self._descs:
            common = dict(stride=self.stride, dilation=self.dilation, padding=self.padding, dtype=x.dtype,
                          context=self.context, real_valued_input=self.real_input, groups=self.groups,
                          data_format=self.data_format)
            fwd = ops.Conv2DDescriptor(x.shape, self.weight.shape, use_bias=self.bias is not None, **common)
            bwd = ops.Conv2DDescriptor(x.shape, self.weight.shape, require_input_grad=self.input_requires_grad, **common)
            self._descs[key] = (fwd, bwd)
        return self._descs[key]

    def forward(self, x, passthrough=False):
        """passthrough: returns (y, x') with x' an alias of x for the OTHER consumers of x (the identity branch of a
        residual block): the gradient that comes back through x' is added to the input gradient inside the
        convolution's backward call (ops.conv2d_bwd_data(addend=...)) instead of by autograd's accumulation."""
        fwd, bwd = self._descriptors(x)
        packed = self._packed_filters((tuple(x.shape), x.dtype), fwd)
        if passthrough and self.input_requires_grad:
            return _QConv2dFn.apply(x.contiguous(), self.weight, self.bias, fwd, bwd, packed, True)
        y = _QConv2dFn.apply(x.contiguous(), self.weight, self.bias, fwd, bwd, packed)
        return (y, x) if passthrough else y


def repack_filters(module):
    """For the top of a training step, after the optimizer has changed the filters: packs the filters of every
    QConv2d below `module` again NOW, on the second stream, instead of each layer doing so in its forward call in
    front of its convolution -- fifty small launches leave the caller's stream and run beside the first layers.
    Each layer's next forward call waits for its own pack.  Returns an event behind the last pack (None if nothing
    had to be packed); a caller that captures the step into a graph makes its stream wait for it before the capture
    ends, in case a layer that was packed did not run.  Layers that have not run yet have nothing to repack and pack
    in their first forward call as always."""
    convs = [m for m in module.modules() if isinstance(m, QConv2d)]
    if not convs or not PREPACK_FILTERS:
        return None
    dev = convs[0].weight.device
    main, side = torch.cuda.current_stream(dev), _side_stream(dev)
    side.wait_stream(main)  # the images are overwritten: every kernel enqueued so far that reads them comes first
    last = None
    with torch.cuda.stream(side):
        for m in convs:
            if m._repack_stale():
                if m._pack_event is None:
                    m._pack_event = torch.cuda.Event()
                m._pack_event.record(side)
                m._pack_pending = True
                last = m._pack_event
    return last


class QLinear(nn.Module):
    """Quaternion Dense: x [4N, I] -> y [4N, O], filter layout IO."""

    def __init__(self, in_features, out_features, bias=True, dtype=torch.float32, context=None):
        super().__init__()
        lim = math.sqrt(6.0 / (in_features + out_features))  # Glorot-uniform per component
        self.weight = nn.Parameter(torch.empty(4, in_features, out_features).uniform_(-lim, lim).to(dtype))
        self.bias = nn.Parameter(torch.zeros(4, out_features, dtype=dtype)) if bias else None
        self.context = context
        self._descs = {}

    def forward(self, x):
        key = (tuple(x.shape), x.dtype)
        if key not in self._descs:
            fwd = ops.DenseDescriptor(x.shape, self.weight.shape, use_bias=self.bias is not None, dtype=x.dtype,
                                      context=self.context)
            bwd = ops.DenseDescriptor(x.shape, self.weight.shape, dtype=x.dtype, context=self.context)
            self._descs[key] = (fwd, bwd)
        fwd, bwd = self._descs[key]
        return _QLinearFn.apply(x.contiguous(), self.weight, self.bias, fwd, bwd)


class _QBatchNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, residual, gamma, beta, running_mean, running_var, eps, momentum, relu):
        y, mean, invstd = ops.batch_norm_fwd(x, gamma, beta, running_mean, running_var, eps, momentum, relu, residual)
        ctx.save_for_backward(x, residual, gamma, beta, mean, invstd)
        ctx.eps, ctx.relu = eps, relu
        return y

    @staticmethod
    def backward(ctx, dy):
        x, residual, gamma, beta, mean, invstd = ctx.saved_tensors
        dx, dgamma, dbeta, dres = ops.batch_norm_bwd(x, dy.contiguous(), gamma, beta, mean, invstd, ctx.eps, ctx.relu,
                                                     residual)
        return dx, dres, dgamma, dbeta, None, None, None, None, None


class QBatchNorm2d(nn.Module):
    """torch.nn.BatchNorm2d semantics on [4N, C, H, W] (the four components of a quaternion channel share the
    statistics of their channel), optionally followed by ReLU, on the library's streaming kernels in
    training mode: a channel is spread over many workgroups, where one-workgroup-per-channel library kernels
    leave a 16-channel layer on 16 of 256 CUs.  Parameters and statistics are fp32 whatever the tensor type.
    Evaluation mode uses torch.nn.functional.batch_norm with the running statistics."""

    def __init__(self, num_features, eps=1e-5, momentum=0.1, relu=False):
        super().__init__()
        self.eps, self.momentum, self.relu = eps, momentum, relu
        self.weight = nn.Parameter(torch.ones(num_features))
        self.bias = nn.Parameter(torch.zeros(num_features))
        self.register_buffer("running_mean", torch.zeros(num_features))
        self.register_buffer("running_var", torch.ones(num_features))

    def forward(self, x, residual=None):
        """residual (relu=True only): added to the normalised tensor in front of the ReLU, as the identity branch
        of a bottleneck block is."""
        if residual is not None and not self.relu:
            raise ValueError("a residual goes in front of the ReLU: construct the module with relu=True")
        if self.training:
            return _QBatchNormFn.apply(x.contiguous(), None if residual is None else residual.contiguous(), self.weight,
                                       self.bias, self.running_mean, self.running_var, self.eps, self.momentum, self.relu)
        y = nn.functional.batch_norm(x, self.running_mean, self.running_var, self.weight, self.bias, False, 0.0, self.eps)
        if residual is not None:
            y = y + residual
        return torch.relu(y) if self.relu else y


class _QMaxPoolFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        y, index = ops.max_pool_3x3s2_fwd(x)
        ctx.save_for_backward(index)
        ctx.input_shape = tuple(x.shape)
        return y

    @staticmethod
    def backward(ctx, dy):
        (index,) = ctx.saved_tensors
        return ops.max_pool_3x3s2_bwd(dy.contiguous(), index, ctx.input_shape)


class QMaxPool3x3s2(nn.Module):
    """torch.nn.MaxPool2d(3, 2, 1) on the library's streaming kernels (include/phx_pool.h): same outputs and
    gradients, one byte of index per output element instead of eight."""

    def forward(self, x):
        return _QMaxPoolFn.apply(x.contiguous())


class _Bottleneck(nn.Module):
    def __init__(self, cin, width, cout, stride, dtype, context, fused_bn):
        super().__init__()
        mk = lambda ci, co, k, s: QConv2d(ci, co, k, stride=s, padding="SAME", dtype=dtype, context=context)
        # fused_bn: batch-norm (+ the ReLU behind it) on the library's kernels; otherwise torch's modules
        bn = (lambda c, relu: QBatchNorm2d(c, relu=relu)) if fused_bn else (lambda c, relu: nn.BatchNorm2d(c))
        self.fused_bn = fused_bn
        self.conv1, self.bn1 = mk(cin, width, 1, 1), bn(width, True)
        self.conv2, self.bn2 = mk(width, width, 3, stride), bn(width, True)
        self.conv3, self.bn3 = mk(width, cout, 1, 1), bn(cout, True)  # (fused: ReLU behind the residual add)
        self.down = None
        if stride != 1 or cin != cout:
            self.down = nn.Sequential(mk(cin, cout, 1, stride), bn(cout, False))
        self.relu = nn.ReLU(inplace=True)

    def forward(self, x):
        if self.fused_bn:
            # (conv1 hands x on to the identity branch, see QConv2d.forward: one elementwise pass less per block)
            y, x = self.conv1(x, passthrough=True) if FUSE_BRANCH_GRADIENT else (self.conv1(x), x)
            idt = x if self.down is None else self.down(x)
            y = self.bn1(y)
            y = self.bn2(self.conv2(y))
            return self.bn3(self.conv3(y), idt)
        idt = x if self.down is None else self.down(x)
        y = self.relu(self.bn1(self.conv1(x)))
        y = self.relu(self.bn2(self.conv2(y)))
        y = self.bn3(self.conv3(y))
        return self.relu(y + idt)


class QResNet50(nn.Module):
    """ResNet-50 with quaternion channels = real channels / 4: stem 3->16 (7x7 s2), stages of
    (3, 4, 6, 3) bottlenecks with widths 16/32/64/128 and outputs 64/128/256/512, head = quaternion
    Dense 512 -> 250 units (= 1000 logits).  53 convolutions.  Batch-norm (with the ReLU behind it) runs on the
    library's kernels (fused_bn=True) or on torch's modules.  The stem takes the real images
    [N, 3, H, W] directly (real_input=True) or, with real_input=False, their lift() to quaternions."""

    def __init__(self, num_classes=1000, dtype=torch.float32, context=None, real_input=True, fused_bn=True):
        super().__init__()
        assert num_classes % 4 == 0
        self.stem = QConv2d(3, 16, 7, stride=2, padding="SAME", dtype=dtype, context=context, input_requires_grad=False,
                            real_input=real_input)
        self.fused_bn = fused_bn
        self.bn = QBatchNorm2d(16, relu=True) if fused_bn else nn.BatchNorm2d(16)
        self.relu = nn.ReLU(inplace=True)
        self.pool = QMaxPool3x3s2() if fused_bn else nn.MaxPool2d(3, 2, 1)
        blocks, cin = [], 16
        for width, cout, count, stride in ((16, 64, 3, 1), (32, 128, 4, 2), (64, 256, 6, 2), (128, 512, 3, 2)):
            for i in range(count):
                blocks.append(_Bottleneck(cin, width, cout, stride if i == 0 else 1, dtype, context, fused_bn))
                cin = cout
        self.blocks = nn.Sequential(*blocks)
        self.head = QLinear(512, num_classes // 4, bias=True, dtype=dtype, context=context)

    @staticmethod
    def lift(images):
        """Real images [N, 3, H, W] -> quaternion input [4N, 3, H, W]: real part = image, imaginary parts zero."""
        z = torch.zeros_like(images)
        return torch.cat([images, z, z, z], dim=0)

    def forward(self, x):
        y = self.bn(self.stem(x))
        y = self.pool(y if self.fused_bn else self.relu(y))
        y = self.blocks(y)
        y = y.float().mean(dim=(2, 3)).to(x.dtype)            # [4N, 512]
        y = self.head(y)                                      # [4N, 250]
        n = y.shape[0] // 4
        return y.view(4, n, -1).permute(1, 0, 2).reshape(n, -1)  # [N, 1000]: the four components side by side

    def conv_layers(self):
        return [m for m in self.modules() if isinstance(m, QConv2d)]
