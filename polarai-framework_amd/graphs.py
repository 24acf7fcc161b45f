"""Kernel DAGs of the two model configurations, built the way the framework
builds them, for the mini-executor.

`Graph` mirrors what the framework's graph front-end hands to its compiler:
input nodes (with a data, constant or "holder" loader) and compute nodes (one
builtin each), grouped into clusters by dependency level -- every input node
in cluster 0, every other node one level after its latest operand
(tests/unit/core/Traverse.cpp:45-46,74-75).  `emit` turns a graph into a
mini-executor program; running it reaches every kernel through
Device::launch.

The backward graphs follow the framework's own derivative rules, which are not
textbook back-propagation for batches (the matmul rule multiplies by element 0
of the incoming gradient only):
  logloss   (p - y) / (p - p*p) * g      LogLossOperationInternal.cpp:127-170
  sigmoid   g * ((1 - s) * s)            SigmoidOperationInternal.cpp:107-135
  matmul    wrt left:  g[0] * (ones[MxN] x B^T)   MatMulOperationInternal.cpp:120-133
            wrt right: g[0] * (A^T x ones[MxN])   MatMulOperationInternal.cpp:147-160
  every node's gradient is summed into a zero tensor with fadd
                                         GraphInternal.cpp:260-327
  update    W <- (grad * lr) + W in place, lr = -0.01
                                         GraphInternal.cpp:381-470
"""
import numpy as np


class Value:
    def __init__(self, graph, kind, shape, level, **kw):
        self.graph, self.kind, self.shape, self.level = graph, kind, tuple(shape), level
        self.kernel = kw.get("kernel")
        self.args = kw.get("args", [])
        self.result_index = kw.get("result_index")
        self.data = kw.get("data")          # input nodes with data
        self.tensor_key = kw.get("tensor_key", id(self))  # aliasing (holders, in place)
        self.name = kw.get("name", "")


class Graph:
    def __init__(self, name):
        self.name = name
        self.nodes = []

    # -- input nodes (always cluster 0) -------------------------------------
    def input(self, data, name=""):
        data = np.ascontiguousarray(data, dtype=np.float32)
        v = Value(self, "input", data.shape, 0, data=data, name=name)
        self.nodes.append(v)
        return v

    def constant(self, value, shape, name=""):
        return self.input(np.full(shape, value, dtype=np.float32), name=name)

    def holder(self, other, name=""):
        """Input node that holds the tensor of `other` (a value of this or of
        an earlier graph) and loads nothing."""
        v = Value(self, "holder", other.shape, 0, tensor_key=other.tensor_key, name=name)
        self.nodes.append(v)
        return v

    # -- compute nodes ------------------------------------------------------
    def _op(self, kernel, args, shape, name="", into=None):
        level = 1 + max(a.level for a in args if isinstance(a, Value))
        key = into.tensor_key if into is not None else None
        out = Value(self, "op", shape, level, kernel=kernel, name=name,
                    **({"tensor_key": key} if key is not None else {}))
        out.args = list(args) + [out]
        out.result_index = len(args)
        self.nodes.append(out)
        return out

    def add(self, a, b, sa=1.0, sb=1.0, name="", into=None):
        return self._op("fadd", [a, sa, b, sb], a.shape, name, into)  # shape of operand 0

    def mul(self, a, b, name=""):
        return self._op("fmul", [a, b], a.shape, name)

    def divide(self, num, den, name=""):
        return self._op("fdivide", [num, den], num.shape, name)

    def sigmoid(self, x, name=""):
        return self._op("fsigmoid", [x], x.shape, name)

    def logloss(self, pred, truth, name=""):
        return self._op("flogloss", [pred, truth], pred.shape, name)

    def mulconcat(self, grad, local, name=""):
        return self._op("fmulconcat", [grad, local], local.shape, name)

    def matmul(self, a, b, ta=False, tb=False, name=""):
        m = a.shape[1] if ta else a.shape[0]
        n = b.shape[0] if tb else b.shape[1]
        return self._op(f"fmatmul_{'t' if ta else 'f'}_{'t' if tb else 'f'}", [a, b], (m, n), name)

    def clusters(self):
        top = max(n.level for n in self.nodes)
        return [[n for n in self.nodes if n.level == lv] for lv in range(top + 1)]


def emit(graph, harness, tensors):
    """Append `graph` to the harness program.  `tensors` maps tensor keys to
    harness tensors and is shared between the graphs of one model so that
    holders and in-place nodes address the same memory."""
    def tensor_of(v):
        if v.tensor_key not in tensors:
            tensors[v.tensor_key] = harness.tensor(*v.shape)
        return tensors[v.tensor_key]

    for cluster in graph.clusters():
        for n in cluster:
            t = tensor_of(n)
            if n.kind == "input":
                harness.input_into(t, n.data)
            elif n.kind == "holder":
                harness.holder(t)
            else:
                args = [tensor_of(a) if isinstance(a, Value) else a for a in n.args]
                harness.node(n.kernel, args, n.result_index)
        harness.end_cluster()


def logreg_forward(x, w, bias_full, y):
    """Z = matmul(X, W) + B, P = sigmoid(Z), L = logloss(P, Y).  The framework's
    add has no broadcasting (AddOperationInternal.cpp:32-33), so the bias comes
    in already expanded to Z's shape."""
    g = Graph("logreg")
    X, W, B, Y = g.input(x, "X"), g.input(w, "W"), g.input(bias_full, "B"), g.input(y, "Y")
    z0 = g.matmul(X, W, name="Z0")
    z = g.add(z0, B, name="Z")
    p = g.sigmoid(z, name="P")
    loss = g.logloss(p, Y, name="L")
    return g, dict(X=X, W=W, B=B, Y=Y, Z0=z0, Z=z, P=p, L=loss)


def mlp_graphs(x, w1, w2, y, learning_rate=-0.01):
    """Two-layer MLP: H = sigmoid(X W1), P = sigmoid(H W2), L = logloss(P, Y);
    then the framework's gradient graph and weight-changing graph.  Returns
    (forward, gradient, update, named values)."""
    f = Graph("mlp_forward")
    X, W1, W2, Y = f.input(x, "X"), f.input(w1, "W1"), f.input(w2, "W2"), f.input(y, "Y")
    a1 = f.matmul(X, W1, name="A1")
    h = f.sigmoid(a1, name="H")
    a2 = f.matmul(h, W2, name="A2")
    p = f.sigmoid(a2, name="P")
    loss = f.logloss(p, Y, name="L")

    g = Graph("mlp_gradient")
    seed = g.constant(1.0, loss.shape, "seed")  # GraphInternal.cpp:237-252

    def accumulate(shape, contributions, name):
        total = g.constant(0.0, shape, "zero_" + name)
        for c in contributions:
            total = g.add(c, total, name="sum_" + name)
        return total

    def d_logloss(grad):
        yh, ph, ph2 = g.holder(Y), g.holder(p), g.holder(p)
        num = g.add(ph, yh, 1.0, -1.0, name="p-y")
        pp = g.mul(ph, ph2, name="p*p")
        den = g.add(ph, pp, 1.0, -1.0, name="p-p*p")
        return g.mul(g.divide(num, den, name="dL/dp"), grad, name="g_P_local")

    def d_sigmoid(s, grad, tag):
        sh = g.holder(s)
        ones = g.constant(1.0, s.shape, "ones_" + tag)
        one_minus = g.add(ones, sh, 1.0, -1.0, name="1-s_" + tag)
        return g.mul(grad, g.mul(one_minus, sh, name="s(1-s)_" + tag), name="g_" + tag + "_local")

    def d_matmul_left(a_val, b_val, grad, tag):   # A [MxK], B [KxN] -> [MxK]
        bh = g.holder(b_val)
        ones = g.constant(1.0, (a_val.shape[0], b_val.shape[1]), "ones_" + tag)
        return g.mulconcat(grad, g.matmul(ones, bh, tb=True, name="onesxBt_" + tag), name="g_" + tag)

    def d_matmul_right(a_val, b_val, grad, tag):  # -> [KxN]
        ah = g.holder(a_val)
        ones = g.constant(1.0, (a_val.shape[0], b_val.shape[1]), "ones_" + tag)
        return g.mulconcat(grad, g.matmul(ah, ones, ta=True, name="Atxones_" + tag), name="g_" + tag)

    g_p = accumulate(p.shape, [d_logloss(seed)], "P")
    g_a2 = accumulate(a2.shape, [d_sigmoid(p, g_p, "A2")], "A2")
    g_h = accumulate(h.shape, [d_matmul_left(h, W2, g_a2, "H")], "H")
    g_w2 = accumulate(W2.shape, [d_matmul_right(h, W2, g_a2, "W2")], "W2")
    g_a1 = accumulate(a1.shape, [d_sigmoid(h, g_h, "A1")], "A1")
    g_w1 = accumulate(W1.shape, [d_matmul_right(X, W1, g_a1, "W1")], "W1")

    u = Graph("mlp_update")
    for w, gw, tag in ((W1, g_w1, "W1"), (W2, g_w2, "W2")):
        gh = u.holder(gw)
        lr = u.constant(learning_rate, gw.shape, "lr_" + tag)
        step = u.mul(gh, lr, name="step_" + tag)
        wh = u.holder(w)
        u.add(step, wh, name="new_" + tag, into=w)  # result written over the weight

    named = dict(X=X, W1=W1, W2=W2, Y=Y, A1=a1, H=h, A2=a2, P=p, L=loss,
                 gP=g_p, gA2=g_a2, gH=g_h, gW2=g_w2, gA1=g_a1, gW1=g_w1)
    return f, g, u, named
