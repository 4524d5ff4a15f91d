"""A small, TVM-free tensor-expression description.

The reference builds its operators with TVM's ``te.placeholder`` / ``te.compute``
and only ever inspects a handful of attributes of the resulting objects:
``op.axis`` / ``op.reduce_axis`` (names and extents, flextensor/space.py:399-402),
``op.input_tensors``, ``op.num_outputs`` / ``op.output(i)`` and ``tensor.shape`` /
``tensor.dtype`` (flextensor/scheduler.py:36-55, flextensor/measure.py:94-98).
This module provides exactly those attributes. An operator is not an
expression tree: it names one of the operator kinds the gfx950 kernel
templates implement and carries its parameters in ``attrs``.
"""
import itertools

_counter = itertools.count()


class IterVar(object):
    """A loop axis: a name and an integer extent."""

    def __init__(self, name, extent, kind="spatial"):
        self.name = name
        self.extent = int(extent)
        self.kind = kind

    def __repr__(self):
        return "IterVar(%s, %d, %s)" % (self.name, self.extent, self.kind)


class Tensor(object):
    def __init__(self, shape, dtype, op, value_index=0, name=None):
        self.shape = tuple(int(x) for x in shape)
        self.dtype = dtype
        self.op = op
        self.value_index = value_index
        self.name = name or op.name

    @property
    def ndim(self):
        return len(self.shape)

    def __repr__(self):
        return "Tensor(%s, shape=%s, dtype=%s)" % (self.name, self.shape, self.dtype)


class Operation(object):
    num_outputs = 1

    def __init__(self, name):
        self.name = name
        self.uid = next(_counter)
        self.input_tensors = []
        self._outputs = []

    def output(self, i):
        return self._outputs[i]

    def __hash__(self):
        return hash(self.uid)

    def __eq__(self, other):
        return isinstance(other, Operation) and self.uid == other.uid


class PlaceholderOp(Operation):
    def __init__(self, shape, dtype, name):
        super(PlaceholderOp, self).__init__(name)
        self._outputs = [Tensor(shape, dtype, self, 0, name)]


class ComputeOp(Operation):
    """One operator instance.

    kind          operator family ("gemm", "gemm_int8", "conv2d_nchw",
                  "depthwise_conv2d_nchw", "zero_pad2d")
    axis          spatial IterVars in declaration order
    reduce_axis   reduce IterVars in the order the reference declares them
    attrs         operator parameters (stride, padding, ...)
    """

    def __init__(self, name, kind, out_shape, out_dtype, axis, reduce_axis, inputs, attrs=None):
        super(ComputeOp, self).__init__(name)
        self.kind = kind
        self.axis = list(axis)
        self.reduce_axis = list(reduce_axis)
        self.input_tensors = list(inputs)
        self.attrs = dict(attrs or {})
        self._outputs = [Tensor(out_shape, out_dtype, self, 0, name)]

    def __repr__(self):
        return "ComputeOp(%s:%s)" % (self.kind, self.name)


def placeholder(shape, dtype="float32", name=None):
    """Counterpart of tvm.te.placeholder: returns the tensor of a new input."""
    name = name or "placeholder%d" % next(_counter)
    return PlaceholderOp(shape, dtype, name).output(0)
