"""A define-by-run tape over a device object, for tests that replay the reference's graph tests.

It calls the device the way primitiv's Graph does (primitiv/core/graph.cc:116-223 with the
operators of primitiv/core/operator_impl.cc): forward at once, one device call per operator;
backward in reverse order of creation, an operator is skipped when nothing reached its output,
arguments without a gradient get a zero tensor of their own shape first, then the operator's
backward adds into them.  It holds no arithmetic: every number comes out of the device.
"""
import primitiv_amd as pa


class Tape:
    def __init__(self, dev):
        self.dev = dev
        self.values = []      # Tensor per node
        self.ops = []         # (argument node ids, backward(gy, argument gradients) or None) per node
        self.grads = {}

    # ---- leaves ----
    def _push(self, value, args=(), backward=None):
        self.values.append(value)
        self.ops.append((tuple(args), backward))
        return len(self.values) - 1

    def input(self, shape, values):
        return self._push(self.dev.new_tensor_by_vector(shape, values))

    def constant(self, shape, k):
        return self._push(self.dev.new_tensor_by_constant(shape, k))

    def value(self, n):
        return self.values[n]

    def gradient(self, n):
        return self.grads[n]

    # ---- operators (forward now, backward as the reference's operator does it) ----
    def matmul(self, a, b):
        d, v = self.dev, self.values
        y = d.matmul_fw(v[a], v[b])                             # operator_impl.cc:421
        return self._push(y, (a, b), lambda gy, g: d.matmul_bw(v[a], v[b], y, gy, g[0], g[1]))   # :734-736

    def _binary(self, op, a, b):
        d, v = self.dev, self.values
        y = d.binary_fw(op, v[a], v[b])
        return self._push(y, (a, b), lambda gy, g: d.binary_bw(op, v[a], v[b], y, gy, g[0], g[1]))

    def add(self, a, b):
        return self._binary("add", a, b)

    def subtract(self, a, b):
        return self._binary("subtract", a, b)

    def multiply(self, a, b):
        return self._binary("multiply", a, b)

    def _unary(self, op, x):
        d, v = self.dev, self.values
        y = d.unary_fw(op, v[x])
        return self._push(y, (x,), lambda gy, g: d.unary_bw(op, v[x], y, gy, g[0]))

    def sigmoid(self, x):
        return self._unary("sigmoid", x)

    def tanh(self, x):
        return self._unary("tanh", x)

    def slice(self, x, dim, lower, upper):
        d, v = self.dev, self.values
        y = d.slice_fw(v[x], dim, lower, upper)
        return self._push(y, (x,), lambda gy, g: d.slice_bw(gy, dim, lower, g[0]))       # operator_impl.cc Slice::backward

    def concat(self, xs, dim):
        d, v = self.dev, self.values
        y = d.concat_fw([v[x] for x in xs], dim)

        def backward(gy, g):                                    # operator_impl.cc Concat::backward: slices of gy
            offset = 0
            for x, gx in zip(xs, g):
                span = v[x].shape()[dim]
                d.inplace_add(d.slice_fw(gy, dim, offset, offset + span), gx)
                offset += span
        return self._push(y, tuple(xs), backward)

    def sum(self, x, dim):
        d, v = self.dev, self.values
        y = d.reduce_fw("sum", v[x], dim)
        n = v[x].shape()[dim]
        return self._push(y, (x,), lambda gy, g: d.inplace_add(d.broadcast_fw(gy, dim, n), g[0]))

    def batch_sum(self, x):
        d, v = self.dev, self.values
        y = d.batch_sum_fw(v[x])
        return self._push(y, (x,), lambda gy, g: d.inplace_add(gy, g[0]))                # gx += gy, broadcast over the minibatch

    def num_operators(self):
        return len(self.values)

    # ---- backward (graph.cc:153-223) ----
    def backward(self, node):
        d = self.dev
        self.grads = {node: d.new_tensor_by_constant(self.values[node].shape(), 1)}
        for n in range(node, -1, -1):
            args, bw = self.ops[n]
            if n not in self.grads or bw is None:
                continue
            for a in args:
                if a not in self.grads:
                    self.grads[a] = d.new_tensor_by_constant(self.values[a].shape(), 0)
            bw(self.grads[n], [self.grads[a] for a in args])


S = pa.Shape
