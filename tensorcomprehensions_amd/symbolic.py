"""Size-parametric range inference (tc/core/tc2halide.cc:270-498 in the reference, whose inference
works on expressions of the size parameters): tensor bounds and index ranges of a TC definition as
formulas, before any tensor exists.  The formulas come from the C++ front end
(`tc_lang_dump(..., "ranges")`); this module parses that text and evaluates it for given sizes."""
import re

from . import lang_dump

_TOKEN = re.compile(r"\s*(?:\d+|[A-Za-z_]\w*|//|[-+*(),])")


def evaluate(expression, sizes):
    """Value of a bound for the sizes {parameter: value}.  Only integers, size parameters,
    + - * // and min/max are accepted."""
    pos = 0
    while pos < len(expression):
        m = _TOKEN.match(expression, pos)
        if not m:
            if expression[pos:].strip() == "":
                break
            raise ValueError(f"not a bound expression: {expression!r}")
        pos = m.end()
    names = dict(sizes)
    names.update({"min": min, "max": max})
    return eval(expression, {"__builtins__": {}}, names)  # noqa: S307 (tokens checked above)


class SymbolicRanges:
    """inputs / outputs: {tensor: (mins, extents)} as lists of expression texts;
    statements: [(tensor, [(variable, lo, hi), ...]), ...] (inclusive bounds);
    parameters: the size parameters in order of first appearance."""

    def __init__(self, text):
        self.text = text
        self.inputs, self.outputs, self.statements = {}, {}, []
        order, mins, extents, section = [], {}, {}, None
        for line in text.splitlines():
            if line in ("mins:", "extents:", "statements:"):
                section = line[:-1]
                continue
            if not line.strip():
                continue
            if section in ("mins", "extents"):
                name, rest = line.split("@[", 1)
                dims = [d.strip() for d in rest.rstrip("]").split(";") if d.strip()]
                (mins if section == "mins" else extents)[name] = dims
                if section == "mins":
                    order.append(name)
            else:
                name, rest = line.split(":", 1)
                vs = []
                for item in rest.split(";"):
                    m = re.match(r"\s*(\w+) in \[(.*), (.*)\]\s*$", item)
                    if m:
                        vs.append((m.group(1), m.group(2), m.group(3)))
                self.statements.append((name, vs))
        written = {name for name, _ in self.statements}
        for name in order:
            (self.outputs if name in written else self.inputs)[name] = (mins[name], extents[name])
        self.parameters = []
        for _, (_, ext) in self.inputs.items():
            for e in ext:
                if re.fullmatch(r"[A-Za-z_]\w*", e) and e not in self.parameters:
                    self.parameters.append(e)

    def sizes_from(self, input_shapes):
        """{parameter: value} from the shapes of the inputs, in declaration order."""
        sizes = {}
        for (name, (_, ext)), shape in zip(self.inputs.items(), input_shapes):
            if len(ext) != len(shape):
                raise ValueError(f"{name}: expected {len(ext)} dimensions, got {len(shape)}")
            for e, s in zip(ext, shape):
                if re.fullmatch(r"\d+", e):
                    if int(e) != s:
                        raise ValueError(f"{name}: constant dimension {e} but found {s}")
                elif sizes.setdefault(e, s) != s:
                    raise ValueError(f"mismatched sizes for dimension {e}: {sizes[e]} and {s}")
        return sizes

    def output_bounds(self, input_shapes):
        """[(mins, extents)] of the outputs for these input shapes: the late specialisation."""
        sizes = self.sizes_from(input_shapes)
        return [([evaluate(e, sizes) for e in mins], [evaluate(e, sizes) for e in ext])
                for mins, ext in self.outputs.values()]


def infer_ranges(tc):
    """Symbolic bounds and ranges of the single definition in `tc`."""
    return SymbolicRanges(lang_dump(tc, "ranges"))
