"""A small assembler for the index-expression programs of include/pet_hip.h: MemBound
operators written down as expressions (the C++ host layer flattens the reference's nnet
trees into the same format):

    I("h") + 1, I("w") % 2, C(3)            index expressions (iterators, constants)
    T(0, [idx, ...])                         tensor 0 read at the indices, 0 outside
    R(loops, sums, body, pads)               a range: loops / sums are [(name, lo, hi)]
    RS(range, [idx, ...])                    a range read at a position (0 in its padding)
    relu(v), tanh(v), v + w, v * w, v - w    value expressions

assemble(tensor_shapes, top_range) gives the list of ints. The output shape is the top
range's loop extents (its iterators start at 0, as MemBoundOp::compute assumes,
src/Graph/operator.cc:3625-3640)."""

OPS = dict(END=0, ICONST=1, IVAR=2, IADD=3, ISUB=4, IMUL=5, IDIV=6, IMOD=7, LOAD=8, I2F=9,
           FADD=10, FSUB=11, FMUL=12, FDIV=13, FMOD=14, FRELU=15, FTANH=16, RANGE=17, SUM=18,
           SUMEND=19)
MAGIC = 0x50455401


class Node:
    def _bin(self, other, iop, fop):
        other = other if isinstance(other, Node) else C(other)
        return Bin(iop, fop, self, other)

    def __add__(self, o):
        return self._bin(o, "IADD", "FADD")

    def __sub__(self, o):
        return self._bin(o, "ISUB", "FSUB")

    def __mul__(self, o):
        return self._bin(o, "IMUL", "FMUL")

    def __floordiv__(self, o):
        return self._bin(o, "IDIV", "FDIV")

    def __mod__(self, o):
        return self._bin(o, "IMOD", "FMOD")


class C(Node):
    is_index = True

    def __init__(self, v):
        self.v = int(v)


class I(Node):
    is_index = True

    def __init__(self, name):
        self.name = name


class Bin(Node):
    def __init__(self, iop, fop, a, b):
        self.iop, self.fop, self.a, self.b = iop, fop, a, b
        self.is_index = a.is_index and b.is_index


class T(Node):
    is_index = False

    def __init__(self, tensor, idx):
        self.tensor, self.idx = tensor, [i if isinstance(i, Node) else C(i) for i in idx]


class R(Node):
    is_index = False

    def __init__(self, loops, sums, body, pads=None):
        self.loops, self.sums, self.body = loops, sums, body
        self.pads = pads or [0] * len(loops)


class RS(Node):
    is_index = False

    def __init__(self, rng, idx):
        self.rng, self.idx = rng, [i if isinstance(i, Node) else C(i) for i in idx]


class Fn(Node):
    is_index = False

    def __init__(self, op, a):
        self.op, self.a = op, a


def relu(a):
    return Fn("FRELU", a)


def tanh(a):
    return Fn("FTANH", a)


def assemble(tensor_shapes, top):
    code = [MAGIC, len(tensor_shapes)]
    for s in tensor_shapes:
        code += [len(s)] + [int(d) for d in s]
    code += [len(top.loops)] + [hi - lo for _, lo, hi in top.loops]
    slots = [0]

    def emit_index(n, scope):
        if isinstance(n, C):
            code.extend([OPS["ICONST"], n.v])
        elif isinstance(n, I):
            code.extend([OPS["IVAR"], scope[n.name]])
        else:
            assert n.is_index, "a tensor value cannot be an index"
            emit_index(n.a, scope)
            emit_index(n.b, scope)
            code.append(OPS[n.iop])

    def emit_value(n, scope):
        if n.is_index:
            emit_index(n, scope)
            code.append(OPS["I2F"])
        elif isinstance(n, T):
            for i in n.idx:
                emit_index(i, scope)
            code.extend([OPS["LOAD"], n.tensor])
        elif isinstance(n, Fn):
            emit_value(n.a, scope)
            code.append(OPS[n.op])
        elif isinstance(n, Bin):
            emit_value(n.a, scope)
            emit_value(n.b, scope)
            code.append(OPS[n.fop])
        elif isinstance(n, RS):
            for i in n.idx:
                emit_index(i, scope)
            emit_range(n.rng)
        else:
            raise TypeError(n)

    def emit_range(r):
        scope = {}
        for name, _, _ in list(r.loops) + list(r.sums):
            scope[name] = slots[0]
            slots[0] += 1
        at = len(code)
        code.extend([OPS["RANGE"], len(r.loops), -1])
        for name, lo, hi in r.loops:
            code.extend([scope[name], lo, hi, 0])
        for j, p in enumerate(r.pads):
            code[at + 3 + 4 * j + 3] = p
        if r.sums:
            code.extend([OPS["SUM"], len(r.sums)])
            for name, lo, hi in r.sums:
                code.extend([scope[name], lo, hi])
            body = len(code)
            emit_value(r.body, scope)
            code.extend([OPS["SUMEND"], len(r.sums), body])
            for name, lo, hi in r.sums:
                code.extend([scope[name], lo, hi])
        else:
            emit_value(r.body, scope)
        code[at + 2] = len(code)  # where a read in the padding continues

    emit_range(top)
    code.append(OPS["END"])
    return code
