"""A few lines of reverse-mode bookkeeping over the element-wise operators, so that the functions of
the reference's tests/autodiff/coopvec.slang can be written down once and evaluated either with the CPU
oracle or with the GPU library: `ops` supplies forward(op, a, b, c, param) and
backward(op, dOut, a, b, c, param) on arrays of one element type."""
from __future__ import annotations

ADD, SUB, MUL, DIV, NEG, MIN, MAX, CLAMP, STEP, SIN, COS, EXP, LOG, LOG2, EXP2, TANH, ATAN, FMA = range(18)
RELU, LEAKY_RELU, SIGMOID, SILU, QUICK_GELU, SCALE = range(18, 24)
N_OPERANDS = {ADD: 2, SUB: 2, MUL: 2, DIV: 2, MIN: 2, MAX: 2, STEP: 2, CLAMP: 3, FMA: 3}


class Var:
    def __init__(self, tape, value, parents=(), op=None, param=0.0):
        self.tape, self.value, self.parents, self.op, self.param = tape, value, parents, op, param
        self.grad = None
        tape.nodes.append(self)

    def _bin(self, op, other):
        return self.tape.apply(op, self, other)

    def __add__(self, o): return self._bin(ADD, o)
    def __sub__(self, o): return self._bin(SUB, o)
    def __mul__(self, o): return self._bin(MUL, o)
    def __truediv__(self, o): return self._bin(DIV, o)
    def __neg__(self): return self.tape.apply(NEG, self)


class Tape:
    def __init__(self, ops):
        self.ops, self.nodes = ops, []

    def leaf(self, value):
        return Var(self, value)

    def apply(self, op, *args, param=0.0):
        vals = [a.value for a in args] + [None] * (3 - len(args))
        return Var(self, self.ops.forward(op, vals[0], vals[1], vals[2], param), tuple(args), op, param)

    def backward(self, out, d_out):
        out.grad = d_out
        for node in reversed(self.nodes):
            if node.grad is None or node.op is None:
                continue
            vals = [a.value for a in node.parents] + [None] * (3 - len(node.parents))
            grads = self.ops.backward(node.op, node.grad, vals[0], vals[1], vals[2], node.param)
            for parent, g in zip(node.parents, grads):
                parent.grad = g if parent.grad is None else self.ops.forward(ADD, parent.grad, g, None, 0.0)


# the functions of tests/autodiff/coopvec.slang:166-219
def compound(t, x, y):
    return (x + y) * (x - y)


def common_math(t, x):
    return t.apply(EXP, x) + t.apply(SIN, x) + t.apply(COS, x)


def division_negation(t, x, y):
    return -(x / y)


def additional_math(t, x, one):
    return (t.apply(EXP2, x) + t.apply(TANH, x) + t.apply(LOG, one + x) + t.apply(LOG2, one + x) + t.apply(ATAN, x))


def forward_arithmetic(t, x, y):
    return (x + y) * (x - y) - (x / y)


def same_operand(t, x):
    return (x + x) + (x - x) + (x * x) + (x / x)


def min_max_clamp_fma(t, x, y, lo, hi, one):
    return t.apply(MIN, x, y) + t.apply(MAX, x, y) + t.apply(CLAMP, x, lo, hi) + t.apply(FMA, x, y, one)


def run_case(ops, name, case, make):
    """Evaluates one block of the reference test: returns (primal, dx, dy, tangent) as lists; entries
    the block does not have are None.  `make(list_or_scalar)` builds a 4-vector of the element type."""
    t = Tape(ops)
    x = t.leaf(make(case["x"]))
    y = t.leaf(make(case["y"])) if "y" in case else None
    if name in ("compound", "forward_arithmetic", "division_negation"):
        f = {"compound": compound, "forward_arithmetic": forward_arithmetic, "division_negation": division_negation}[name]
        out = f(t, x, y)
    elif name == "common_math":
        out = common_math(t, x)
    elif name == "additional_math":
        out = additional_math(t, x, t.leaf(make(1.0)))
    elif name == "same_operand":
        out = same_operand(t, x)
    elif name == "min_max_clamp_fma":
        out = min_max_clamp_fma(t, x, y, t.leaf(make(case["lo"])), t.leaf(make(case["hi"])), t.leaf(make(1.0)))
    else:
        raise KeyError(name)
    primal = out.value
    dx = dy = tangent = None
    if "dOut" in case:
        t.backward(out, make(case["dOut"]))
        dx = x.grad
        dy = y.grad if y is not None else None
    if "xT" in case:
        # forward mode of an element-wise function: J v = df/dx * xT + df/dy * yT, the partials being the
        # reverse-mode gradients for dOut = 1
        t2 = Tape(ops)
        x2 = t2.leaf(make(case["x"]))
        y2 = t2.leaf(make(case["y"])) if "y" in case else None
        if name in ("compound", "forward_arithmetic", "division_negation"):
            o2 = {"compound": compound, "forward_arithmetic": forward_arithmetic, "division_negation": division_negation}[name](t2, x2, y2)
        elif name == "common_math":
            o2 = common_math(t2, x2)
        elif name == "additional_math":
            o2 = additional_math(t2, x2, t2.leaf(make(1.0)))
        elif name == "same_operand":
            o2 = same_operand(t2, x2)
        else:
            o2 = min_max_clamp_fma(t2, x2, y2, t2.leaf(make(case["lo"])), t2.leaf(make(case["hi"])), t2.leaf(make(1.0)))
        t2.backward(o2, make(1.0))
        tangent = ops.forward(MUL, x2.grad, make(case["xT"]), None, 0.0)
        if y2 is not None and "yT" in case:
            tangent = ops.forward(ADD, tangent, ops.forward(MUL, y2.grad, make(case["yT"]), None, 0.0), None, 0.0)
    return primal, dx, dy, tangent
