"""Conv2D and Dense for the reference's other algebras -- REAL, COMPLEX, GA_300 (src/algebras.hpp:17-22; sign
tables src/algebras.cc:5-145) -- as compositions on the quaternion kernels.

GA_300 is the Clifford algebra of three-dimensional space with the blades in the order 1, e1, e2, e3, e12, e13,
e23, e123 (src/algebras.cc:58-131).  Its even part {1, e12, e13, -e23} multiplies like the quaternion units
{1, i, j, k}, and the pseudoscalar I = e123 commutes with everything and squares to -1, so every multivector is
M = A + I B with quaternion-like A = (m0, m4, m5, -m6) and B = (m7, -m3, m2, m1), and

    (A1 + I B1)(A2 + I B2) = (A1 A2 - B1 B2) + I (A1 B2 + B1 A2).

A GA_300 convolution of Ci -> Co channels is therefore ONE quaternion convolution of 2 Ci -> 2 Co channels on
the activations [A | B] with the filter blocks [[A2, B2], [-B2, A2]] (input half x output half): 64 real
products per multivector product, exactly what the algebra's own table holds.  COMPLEX and REAL are the
sub-algebras {1, i} and {1} of the quaternions: their tensors are embedded with zero components, which is
correct but runs the full quaternion arithmetic (4x and 16x the products these algebras need).

Everything here is rearrangement of device tensors (signed blade permutations, channel concatenation) around
phoenix_core_amd.ops; the gradients are the transposes of the same linear maps.  Filter layouts: OIHW / IO,
activations NCHW, no groups."""
import torch

from . import ops

DIMS = {ops.REAL: 1, ops.COMPLEX: 2, ops.QUATERNION: 4, ops.GA_300: 8}  # MULTIVECTOR_DIM, src/algebras.hpp:26

# per algebra: its quaternion-like halves; a half lists (blade, sign) for the quaternion components 0..3
# (None: the component is zero)
_HALVES = {
    ops.REAL: [[(0, 1), None, None, None]],
    ops.COMPLEX: [[(0, 1), (1, 1), None, None]],
    ops.GA_300: [[(0, 1), (4, 1), (5, 1), (6, -1)], [(7, 1), (3, -1), (2, 1), (1, 1)]],
}


def _parts(v, algebra):
    """[D, ...] -> one [4, ...] tensor per half."""
    out = []
    for half in _HALVES[algebra]:
        comps = [torch.zeros_like(v[0]) if e is None else (v[e[0]] if e[1] > 0 else -v[e[0]]) for e in half]
        out.append(torch.stack(comps))
    return out


def _scatter(parts, algebra, like):
    """Inverse (= transpose) of _parts: one [4, ...] tensor per half -> [D, ...]."""
    out = like.new_empty((DIMS[algebra],) + tuple(parts[0].shape[1:]))
    for half, part in zip(_HALVES[algebra], parts):
        for p, e in enumerate(half):
            if e is not None:
                out[e[0]] = part[p] if e[1] > 0 else -part[p]
    return out


def to_quaternion(t, algebra):
    """Activations / bias [D*n, C, ...] -> [4*n, H*C, ...] (H halves side by side on the channel axis)."""
    d = DIMS[algebra]
    n = t.shape[0] // d
    parts = _parts(t.reshape(d, n, *t.shape[1:]), algebra)
    q = torch.cat(parts, dim=2) if len(parts) > 1 else parts[0]
    return q.reshape(4 * n, *q.shape[2:]).contiguous()


def from_quaternion(q, algebra):
    """[4*n, H*C, ...] -> [D*n, C, ...]."""
    halves = len(_HALVES[algebra])
    n, c = q.shape[0] // 4, q.shape[1] // halves
    v = q.reshape(4, n, halves, c, *q.shape[2:])
    out = _scatter([v[:, :, h] for h in range(halves)], algebra, q)
    return out.reshape(DIMS[algebra] * n, c, *q.shape[2:]).contiguous()


def filter_to_quaternion(w, algebra, out_dim, in_dim):
    """Filter [D, ...] -> quaternion filter [4, ...], both channel axes multiplied by the number of halves."""
    parts = _parts(w, algebra)
    if len(parts) == 1:
        return parts[0].contiguous()
    a, b = parts
    return torch.cat([torch.cat([a, -b], dim=in_dim), torch.cat([b, a], dim=in_dim)], dim=out_dim).contiguous()


def filter_grad_from_quaternion(dq, algebra, out_dim, in_dim):
    """Transpose of filter_to_quaternion."""
    if len(_HALVES[algebra]) == 1:
        return _scatter([dq], algebra, dq).contiguous()
    co, ci = dq.shape[out_dim] // 2, dq.shape[in_dim] // 2
    blk = lambda o, i: dq.narrow(out_dim, o * co, co).narrow(in_dim, i * ci, ci)  # noqa: E731
    return _scatter([blk(0, 0) + blk(1, 1), blk(1, 0) - blk(0, 1)], algebra, dq).contiguous()


def init_conv_descriptor(desc, input_shape, filter_shape, algebra, groups, filter_layout, data_format, real_valued_input,
                         **kwargs):
    """Fills an ops.Conv2DDescriptor of a non-quaternion algebra: shapes in that algebra, `inner` = the descriptor of
    the quaternion convolution that computes it."""
    if algebra not in _HALVES:
        raise ValueError("unknown algebra")
    if groups != 1 or filter_layout != "OIHW" or data_format != "NCHW" or real_valued_input:
        raise NotImplementedError("non-quaternion algebras take NCHW activations and OIHW filters, without groups")
    d, halves = DIMS[algebra], len(_HALVES[algebra])
    # a real-valued filter has no blade axis (src/backend/conv2d_descriptor.hpp:14-37)
    if len(filter_shape) != (4 if algebra == ops.REAL else 5):
        raise ValueError("filter rank does not match the algebra")
    fs = tuple(filter_shape) if algebra != ops.REAL else (1,) + tuple(filter_shape)
    if fs[0] != d:
        raise ValueError("First filter dimension mismatch, got %d" % fs[0])
    if input_shape[0] % d:
        raise ValueError("Cannot split %d onto %d parts" % (input_shape[0], d))
    n, (_, co, ci, kh, kw) = input_shape[0] // d, fs
    inner = ops.Conv2DDescriptor((4 * n, halves * input_shape[1], input_shape[2], input_shape[3]),
                                 (4, halves * co, halves * ci, kh, kw), **kwargs)
    desc.inner, desc.algebra = inner, algebra
    desc.input_shape, desc.filter_shape = tuple(input_shape), tuple(filter_shape)
    desc.output_shape = (d * n, co) + inner.output_shape[2:]
    desc.use_bias, desc.require_input_grad, desc.dtype = inner.use_bias, inner.require_input_grad, inner.dtype
    desc.bias_shape = ((d, co) if algebra != ops.REAL else (co,)) if desc.use_bias else ()
    desc.stride, desc.dilation, desc.pad_before, desc.pad_after = inner.stride, inner.dilation, inner.pad_before, inner.pad_after
    desc.context, desc.groups, desc.filter_layout, desc.data_format = inner.context, 1, filter_layout, data_format
    desc.real_valued_input = False


def _blades(t, algebra):
    """A real-valued filter / bias has no blade axis: give it one."""
    return t.unsqueeze(0) if algebra == ops.REAL else t


def conv2d_fwd(x, w, bias, desc):
    a = desc.algebra
    if tuple(x.shape) != desc.input_shape or tuple(w.shape) != desc.filter_shape or x.dtype != desc.dtype:
        raise ValueError("tensor shapes / dtype do not match the descriptor")
    if desc.use_bias and (bias is None or tuple(bias.shape) != desc.bias_shape):
        raise ValueError("bias tensor missing or of wrong shape")
    qb = to_quaternion(_blades(bias, a), a) if desc.use_bias else None
    y = ops.conv2d_fwd(to_quaternion(x, a), filter_to_quaternion(_blades(w, a), a, 1, 2), qb, desc.inner)
    return from_quaternion(y, a)


def conv2d_bwd(x, w, grad, desc):
    a = desc.algebra
    if tuple(x.shape) != desc.input_shape or tuple(w.shape) != desc.filter_shape or tuple(grad.shape) != desc.output_shape:
        raise ValueError("tensor shapes do not match the descriptor")
    dwq, dxq = ops.conv2d_bwd(to_quaternion(x, a), filter_to_quaternion(_blades(w, a), a, 1, 2), to_quaternion(grad, a),
                              desc.inner)
    dw = filter_grad_from_quaternion(dwq, a, 1, 2)
    return (dw[0] if a == ops.REAL else dw), (from_quaternion(dxq, a) if dxq is not None else None)


def init_dense_descriptor(desc, input_shape, filter_shape, algebra, filter_layout, **kwargs):
    if algebra not in _HALVES:
        raise ValueError("unknown algebra")
    if filter_layout != "IO":
        raise NotImplementedError("non-quaternion algebras take Dense filters in IO layout")
    d, halves = DIMS[algebra], len(_HALVES[algebra])
    if len(input_shape) != 2 or len(filter_shape) != (2 if algebra == ops.REAL else 3):
        raise ValueError("expected input [D n, in] and filter [D, in, out]")
    fs = tuple(filter_shape) if algebra != ops.REAL else (1,) + tuple(filter_shape)
    if fs[0] != d or input_shape[0] % d or input_shape[1] != fs[1]:
        raise ValueError("Dense shapes do not match the algebra")
    n = input_shape[0] // d
    inner = ops.DenseDescriptor((4 * n, halves * fs[1]), (4, halves * fs[1], halves * fs[2]), **kwargs)
    desc.inner, desc.algebra, desc.filter_layout = inner, algebra, filter_layout
    desc.input_shape, desc.filter_shape, desc.output_shape = tuple(input_shape), tuple(filter_shape), (d * n, fs[2])
    desc.use_bias, desc.require_input_grad, desc.dtype, desc.context = inner.use_bias, inner.require_input_grad, inner.dtype, inner.context
    desc.bias_shape = ((d, fs[2]) if algebra != ops.REAL else (fs[2],)) if desc.use_bias else ()


def dense_fwd(x, w, bias, desc):
    a = desc.algebra
    if tuple(x.shape) != desc.input_shape or tuple(w.shape) != desc.filter_shape or x.dtype != desc.dtype:
        raise ValueError("tensor shapes / dtype do not match the descriptor")
    if desc.use_bias and (bias is None or tuple(bias.shape) != desc.bias_shape):
        raise ValueError("bias tensor missing or of wrong shape")
    qb = to_quaternion(_blades(bias, a), a) if desc.use_bias else None
    y = ops.dense_fwd(to_quaternion(x, a), filter_to_quaternion(_blades(w, a), a, 2, 1), qb, desc.inner)
    return from_quaternion(y, a)


def dense_bwd(x, w, grad, desc):
    a = desc.algebra
    if tuple(x.shape) != desc.input_shape or tuple(w.shape) != desc.filter_shape or tuple(grad.shape) != desc.output_shape:
        raise ValueError("tensor shapes do not match the descriptor")
    dwq, dxq = ops.dense_bwd(to_quaternion(x, a), filter_to_quaternion(_blades(w, a), a, 2, 1), to_quaternion(grad, a),
                             desc.inner)
    dw = filter_grad_from_quaternion(dwq, a, 2, 1)
    return (dw[0] if a == ops.REAL else dw), (from_quaternion(dxq, a) if dxq is not None else None)
