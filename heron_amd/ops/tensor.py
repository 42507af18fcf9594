"""A minimal tensor-expression layer: just enough structure for operator definitions.

The reference declares operators with TVM's ``te.placeholder`` / ``te.compute``; the template
backend only needs the *declaration* (names, shapes, dtypes, which tensors feed which), not a
loop nest, so this is a few plain classes with the same attribute names (``.name``, ``.shape``,
``.dtype``, ``.op.name``, ``.op.input_tensors``, ``.op.tag``).
"""


class Operation:
    def __init__(self, name, tag, input_tensors, attrs=None):
        self.name = name
        self.tag = tag
        self.input_tensors = list(input_tensors)
        self.attrs = dict(attrs or {})


class Tensor:
    def __init__(self, shape, dtype, op):
        self.shape = tuple(int(x) for x in shape)
        self.dtype = dtype
        self.op = op

    @property
    def name(self):
        return self.op.name

    def __repr__(self):
        return "Tensor(%s, %s, %s)" % (self.name, self.shape, self.dtype)


def placeholder(shape, name, dtype):
    return Tensor(shape, dtype, Operation(name, "placeholder", []))


def compute(shape, name, dtype, inputs, tag="", attrs=None):
    return Tensor(shape, dtype, Operation(name, tag, inputs, attrs))
