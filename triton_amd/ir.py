"""Front end for Trinity's tile-level IR: parse a candidate and decide which hand-written module computes it.

The reference turns every IR candidate into a Triton module (IrParser.py:20-134 -> TritonGen.py:348-424).  With the
code generator bypassed, a candidate is instead *recognised*: all candidates of a workload are equivalent by
construction (they come out of equality saturation over one seed program) and differ in loop structure, tiling and
fusion, which the hand-written kernels fix themselves.  What identifies the workload is its dataflow -- which inputs
reach which outputs through which operators -- so that is what is matched; anything else (other inputs, sigmoid, a
combination no module implements) is reported as unsupported and the drivers record it as a failed candidate, as the
reference records a candidate that fails to compile (vanilla_llama_benchmark.py:206-210).

Grammar (IrParser.py:13-19, :44-134): s-expressions `(op child ...)`; `;` starts a comment; integers are numbers, any
other bare token a variable, except `fulltile` and `dummy`, which are nodes of their own; `input`, `output` and
`tensor` take one name or a comma-separated list of names.  Child layouts (TritonGen.py:2273-2281, :2474-2480,
:2573-2578): `(ploop|sloop start end tile var body)`, `(load tensor index)`, `(store tensor value index)`.
"""
from __future__ import annotations

import re
from dataclasses import dataclass, field
from typing import Dict, FrozenSet, List, Optional, Tuple, Union

# operator token -> number of children (None: any)
OPS: Dict[str, Optional[int]] = {
    "ploop": 5, "sloop": 5, "seq": None, "input": None, "output": None, "tensor": None, "tile": None, "fulltile": None,
    "index": None, "load": 2, "store": 3, "+": 2, "-": 2, "x": 2, "/": 2, "*": 2, "exp": 1, "sqr": 1, "sqrt": 1,
    "sigmoid": 1, "rsum": 2, "concat": None, "bcast": 2, "dummy": None, "elem": None, "permute3": None,
    "squeeze": 2, "unsqueeze": 2, "const_tile": 2,
}
NAMED = ("input", "output", "tensor")
Atom = Union[int, str]


@dataclass(frozen=True)
class Node:
    op: str
    args: Tuple[Union["Node", Atom], ...] = ()

    def __str__(self) -> str:
        return f"({' '.join([self.op, *map(str, self.args)])})" if self.args else (self.op if self.op in ("fulltile", "dummy") else f"({self.op})")


_TOKEN = re.compile(r"\(|\)|,|[^\s(),]+")


def tokenize(code: str) -> List[str]:
    return _TOKEN.findall(re.sub(r";.*", "", code))


def parse(code: str) -> Union[Node, Atom]:
    """One expression.  Errors are ValueError with the reference parser's wording (IrParser.py:32, :61, :98, :134)."""
    toks = tokenize(code)
    pos = 0

    def expr():
        nonlocal pos
        if pos >= len(toks):
            raise ValueError("Unexpected end of input")
        t = toks[pos]
        pos += 1
        if t == "(":
            return lst()
        if t in (")", ","):
            raise ValueError(f"Unexpected token: {t}")
        if t.isdigit() or (t.startswith("-") and t[1:].isdigit()):
            return int(t)
        return Node(t) if t in ("fulltile", "dummy") else t

    def lst():
        nonlocal pos
        if pos >= len(toks):
            raise ValueError("Unexpected end of input")
        op = toks[pos]
        pos += 1
        args = []
        while pos < len(toks) and toks[pos] != ")":
            if toks[pos] == ",":
                if op not in NAMED:
                    raise ValueError("Unexpected token: ,")
                pos += 1
                continue
            args.append(expr())
        if pos >= len(toks):
            raise ValueError("Missing closing parenthesis")
        pos += 1
        if op not in OPS:
            raise ValueError(f"Unknown operation: {op}")
        if OPS[op] is not None and len(args) != OPS[op]:
            raise ValueError(f"{op} expects {OPS[op]} children, got {len(args)}")
        return Node(op, tuple(args))

    tree = expr()
    if pos != len(toks):
        raise ValueError(f"Unexpected token: {toks[pos]}")
    return tree


def read_ir_file(path: str) -> List[Tuple[int, str]]:
    """`id: expression` lines; lines without an integer id, and expressions that mention `dummydata`, are skipped
    (vanilla_llama_benchmark.py:141-161)."""
    out = []
    with open(path) as f:
        for line in f:
            line = line.strip()
            if not line or ":" not in line:
                continue
            head, body = line.split(":", 1)
            try:
                ir_id = int(head)
            except ValueError:
                continue
            if "dummydata" not in body:
                out.append((ir_id, body.strip()))
    return out


# ---------------------------------------------------------------------------------------------------------------------
# Dataflow: every value is summarised by the inputs it derives from and the operators on the way.

@dataclass(frozen=True)
class Val:
    srcs: FrozenSet[str] = frozenset()
    ops: FrozenSet[str] = frozenset()
    raw: FrozenSet[str] = frozenset()     # the sources that reach the value as a linear factor or term: through
                                          # sums, products, matrix products and numerators only

    def __or__(self, o: "Val") -> "Val":
        return Val(self.srcs | o.srcs, self.ops | o.ops, self.raw | o.raw)

    def via(self, op: str) -> "Val":
        return Val(self.srcs, self.ops | {op}, self.raw if op in _LINEAR_OPS else frozenset())


_LINEAR_OPS = ("add", "sub", "mul", "div", "matmul", "rsum")


_OPNAME = {"+": "add", "-": "sub", "x": "mul", "/": "div", "*": "matmul", "exp": "exp", "sqr": "sqr", "sqrt": "sqrt",
           "sigmoid": "sigmoid", "rsum": "rsum"}
_SHAPE_ONLY = ("bcast", "permute3", "squeeze", "unsqueeze")        # value of the first child, rearranged


@dataclass
class Dataflow:
    inputs: set = field(default_factory=set)          # names under (input ...) that are loaded
    stored: Dict[str, Val] = field(default_factory=dict)     # every name that is stored to -> what reaches it
    squares: List[Val] = field(default_factory=list)         # operand of every squaring
    ops: set = field(default_factory=set)
    noise_divisors: set = field(default_factory=set)         # right operand of every division of a noise-carrying sum

    def value_of(self, name: str, kind: str) -> Val:
        v = self.stored.get(name, Val())
        return v | Val(frozenset({name}), frozenset(), frozenset({name})) if kind == "input" else v


def _names(n: Node) -> List[str]:
    if not isinstance(n, Node) or n.op not in NAMED or not n.args or not all(isinstance(a, str) for a in n.args):
        raise ValueError(f"expected (input|output|tensor name...), got {n}")
    return list(n.args)


def analyse(tree: Union[Node, Atom]) -> Dataflow:
    """Fixpoint of the dataflow summary over the whole program (loops only repeat their body, and accumulations
    `T = T + e` read what they wrote, so the stores are iterated until nothing grows)."""
    df = Dataflow()

    def value(n, sq_out) -> Val:
        if not isinstance(n, Node):
            return Val()                                     # a number or a loop variable
        if n.op == "load":
            kind = n.args[0].op if isinstance(n.args[0], Node) else ""
            v = Val()
            for name in _names(n.args[0]):
                if kind == "input":
                    df.inputs.add(name)
                v = v | df.value_of(name, kind)
            return v
        if n.op in _SHAPE_ONLY:
            return value(n.args[0], sq_out)
        if n.op == "concat":
            v = Val()
            for a in n.args[:-1]:
                v = v | value(a, sq_out)
            return v
        if n.op in _OPNAME:
            df.ops.add(_OPNAME[n.op])
            kids = n.args[:1] if n.op == "rsum" else n.args
            vals = [value(a, sq_out) for a in kids]
            if n.op == "sqr" or (n.op == "x" and n.args[0] == n.args[1]):
                sq_out.append(vals[0])
                return vals[0].via("sqr")
            if n.op == "/":
                if "noise" in vals[0].srcs and "exp" not in vals[0].ops:
                    df.noise_divisors.add(n.args[1] if not isinstance(n.args[1], Node) else str(n.args[1]))
                vals[1] = Val(vals[1].srcs, vals[1].ops)          # a denominator is not a linear factor
            v = Val()
            for x in vals:
                v = v | x
            return v.via(_OPNAME[n.op])
        raise ValueError(f"{n.op} cannot appear in a value")

    def run(n, sq_out) -> bool:
        if not isinstance(n, Node) or n.op == "dummy":
            return False
        if n.op == "seq":
            return any([run(a, sq_out) for a in n.args])
        if n.op in ("ploop", "sloop"):
            return run(n.args[4], sq_out)
        if n.op == "store":
            v = value(n.args[1], sq_out)
            grew = False
            for name in _names(n.args[0]):
                old = df.stored.get(name, Val())
                new = old | v
                if new != old:
                    df.stored[name] = new
                    grew = True
            return grew
        raise ValueError(f"{n.op} cannot appear as a statement")

    for _ in range(64):
        squares: List[Val] = []
        if not run(tree, squares):
            df.squares = squares
            return df
    raise ValueError("dataflow did not converge")


# ---------------------------------------------------------------------------------------------------------------------

@dataclass(frozen=True)
class Match:
    variant: Optional[str]          # one of modules' variants, or None
    reason: str                     # why, or why not
    params: Tuple[Tuple[str, object], ...] = ()     # constructor arguments read off the candidate (KeyFormer's tau,
                                                    # the gated MLP's gate), as sorted (name, value) pairs

    def __bool__(self) -> bool:
        return self.variant is not None

    @property
    def kwargs(self) -> Dict[str, object]:
        return dict(self.params)


ATTENTION_INPUTS = frozenset({"X", "WQ", "WK", "WV", "K_cache", "V_cache"})
FINAL_OUTPUTS = ("O2", "C_out", "C_out1", "C_out2")


def _recognise_linear(df: Dataflow) -> Optional[Match]:
    """The reference's two other workloads, told apart from attention by their input names: LoRA reads X, W, A, B
    (lora_benchmark.py:41-53) and writes O = X W + (X A) B; the gated MLP reads X, W1, W2 (gmlp_benchmark.py:53-64)
    and writes O = gate(X W1) * (X W2)."""
    o = df.stored.get("O")
    if df.inputs == {"X", "W", "A", "B"}:
        if o is None or o.srcs != df.inputs:
            return Match(None, "LoRA inputs, but O does not depend on all of X, W, A, B")
        if o.ops != {"matmul", "add"}:
            return Match(None, f"LoRA inputs, but O is not a sum of matrix products (operators {sorted(o.ops)})")
        return Match("lora", "O sums the base product and the two-step adapter product")
    if df.inputs == {"X", "W1", "W2"}:
        if o is None or o.srcs != df.inputs:
            return Match(None, "gated-MLP inputs, but O does not depend on all of X, W1, W2")
        if not {"matmul", "mul"} <= o.ops or not ({"sigmoid"} <= o.ops or {"exp", "div"} <= o.ops):
            return Match(None, f"gated-MLP inputs, but O is not a gated product (operators {sorted(o.ops)})")
        if "W2" not in o.raw:
            return Match(None, "gated-MLP inputs, but the product with W2 does not reach O as a factor")
        # sigmoid(X W1) * (X W2), or SiLU: (X W1) * sigmoid(X W1) * (X W2) -- there the W1 product is also a factor
        gate = "silu" if "W1" in o.raw else "sigmoid"
        return Match("gmlp", f"the product with W1, through a {gate} gate, multiplies the product with W2", (("gate", gate),))
    return None


def recognise(ir: Union[str, Node]) -> Match:
    """Which workload an IR candidate computes: LoRA or the gated MLP (by their input names, see above), or one of
    the five decode-append attention workloads (ref_rms.py:45-83 Vanila, :101-127 PreNorm, :147-179 KeyFormer,
    :197-231 QKNorm, :249-280 RoCo) an IR candidate computes, by dataflow:

    * O2 derives from X, WQ, WK, WV and both caches through matmul, exp and a division (softmax attention);
    * a squaring of something that comes from X alone, before any matmul: PreNorm (`X * rsqrt(mean(X^2))`);
    * squarings after the Q / K projections but before the exponential: QKNorm;
    * `noise` read and `C_out` written from it through an exponential: KeyFormer;
    * `C_out1` and `C_out2` written, the latter through a squaring of the exponentials: RoCo.
    """
    try:
        tree = parse(ir) if isinstance(ir, str) else ir
        df = analyse(tree)
    except (ValueError, IndexError, RecursionError) as e:
        return Match(None, f"cannot parse: {e}")
    linear = _recognise_linear(df)
    if linear is not None:
        return linear
    extra = df.inputs - ATTENTION_INPUTS - {"noise"}
    if extra:
        return Match(None, f"reads inputs no attention variant has: {sorted(extra)}")
    if "sigmoid" in df.ops:
        return Match(None, "uses sigmoid: not an attention variant")
    o2 = df.stored.get("O2")
    if o2 is None:
        return Match(None, "does not write O2")
    if not ATTENTION_INPUTS <= o2.srcs:
        return Match(None, f"O2 does not depend on {sorted(ATTENTION_INPUTS - o2.srcs)}")
    if not {"matmul", "exp", "div"} <= o2.ops:
        return Match(None, f"O2 is not a softmax attention (missing {sorted({'matmul', 'exp', 'div'} - o2.ops)})")
    for cache, w in (("K_cache", "WK"), ("V_cache", "WV")):
        if w not in df.stored.get(cache, Val()).srcs:
            return Match(None, f"the new rows of {cache} are not appended")
    kinds = set()
    for v in df.squares:
        if "exp" in v.ops:
            kinds.add("prob")
        elif "matmul" in v.ops:
            kinds.add("qk:" + ",".join(sorted(v.srcs & {"WQ", "WK"})))
        elif v.srcs == {"X"}:
            kinds.add("x")
        else:
            return Match(None, f"a squaring of {sorted(v.srcs)} fits no variant")
    finals = {n for n in FINAL_OUTPUTS if n in df.stored}
    uses_noise = "noise" in df.inputs
    if finals == {"O2", "C_out"} and uses_noise and not kinds:
        c = df.stored["C_out"]
        if "noise" in c.srcs and "exp" in c.ops and "noise" not in o2.srcs:
            # the temperature: what the noise-carrying scores are divided by before the exponential (none: 1)
            if len(df.noise_divisors) > 1:
                return Match(None, f"the perturbed scores are divided by more than one thing: {sorted(map(str, df.noise_divisors))}")
            tau = 1.0
            for dv in df.noise_divisors:
                try:
                    tau = float(dv)
                except (TypeError, ValueError):
                    return Match(None, f"the temperature {dv} of the perturbed scores is not a number")
            if not tau > 0:
                return Match(None, f"the temperature {tau} of the perturbed scores is not positive")
            return Match("keyformer", f"noise reaches C_out through an exponential (temperature {tau:g}), O2 is plain attention",
                         (("tau", tau),))
        return Match(None, "C_out is not a perturbed-softmax column sum")
    if uses_noise:
        return Match(None, "reads noise without the KeyFormer outputs")
    if finals == {"O2", "C_out1", "C_out2"} and kinds == {"prob"}:
        c1, c2 = df.stored["C_out1"], df.stored["C_out2"]
        if "exp" in c1.ops and "sqr" not in c1.ops and {"exp", "sqr"} <= c2.ops:
            return Match("roco", "C_out1 sums the probabilities, C_out2 their squares")
        return Match(None, "C_out1 / C_out2 are not the sum and the sum of squares of the probabilities")
    if finals != {"O2"}:
        return Match(None, f"outputs {sorted(finals)} with squarings {sorted(kinds)} fit no variant")
    if not kinds:
        return Match("vanilla", "softmax attention over the appended cache")
    if kinds == {"x"} and "sqrt" in o2.ops:
        return Match("prenorm", "X is RMS-normalised before the projections")
    if kinds == {"qk:WK", "qk:WQ"} and "sqrt" in o2.ops:
        return Match("qknorm", "the projected queries and keys are RMS-normalised")
    return Match(None, f"squarings {sorted(kinds)} fit no variant")
