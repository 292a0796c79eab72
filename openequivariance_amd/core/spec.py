"""Problem specification for Clebsch-Gordan tensor products (numpy only).

API-compatible with the reference front-end
(openequivariance/openequivariance/core/e3nn_lite.py:57-654): ``Irrep``,
``Irreps``, ``Instruction`` and ``TPProblem`` accept the same arguments, expose
the same attributes and apply the same path normalisation, so that user code
and e3nn-style instruction lists carry over unchanged.
"""

from __future__ import annotations

import collections
import copy
import itertools
import math
from typing import List, NamedTuple, Optional, Tuple

import numpy as np

_PARITY_CHAR = {"e": 1, "o": -1}
_CHAR_OF_PARITY = {1: "e", -1: "o"}


class Irrep(tuple):
    """An irreducible representation of O(3): degree ``l`` and parity ``p``.

    Mirrors e3nn_lite.py:57-160 (string forms ``"2e"``, ``"1o"``, ``"3y"``).
    """

    def __new__(cls, l, p=None):
        if p is None:
            if isinstance(l, Irrep):
                return l
            if isinstance(l, str):
                text = l.strip()
                try:
                    deg = int(text[:-1])
                    if deg < 0:
                        raise ValueError
                    tag = text[-1]
                    par = (-1) ** deg if tag == "y" else _PARITY_CHAR[tag]
                except Exception:
                    raise ValueError(f'unable to convert string "{text}" into an Irrep')
                l, p = deg, par
            elif isinstance(l, tuple):
                l, p = l
        if not isinstance(l, (int, np.integer)) or l < 0:
            raise ValueError(f"l must be positive integer, got {l}")
        if p not in (-1, 1):
            raise ValueError(f"parity must be on of (-1, 1), got {p}")
        return super().__new__(cls, (int(l), int(p)))

    @property
    def l(self) -> int:
        return self[0]

    @property
    def p(self) -> int:
        return self[1]

    @property
    def dim(self) -> int:
        return 2 * self[0] + 1

    def is_scalar(self) -> bool:
        return self[0] == 0 and self[1] == 1

    def __repr__(self) -> str:
        return f"{self[0]}{_CHAR_OF_PARITY[self[1]]}"

    @classmethod
    def iterator(cls, lmax=None):
        for l in itertools.count():
            yield Irrep(l, (-1) ** l)
            yield Irrep(l, -((-1) ** l))
            if l == lmax:
                break

    def __mul__(self, other):
        """Selection rule: all irreps in the product ``self (x) other``."""
        other = Irrep(other)
        par = self.p * other.p
        return (Irrep(l, par) for l in range(abs(self.l - other.l), self.l + other.l + 1))

    def __rmul__(self, count):
        assert isinstance(count, int)
        return Irreps([(count, self)])

    def __add__(self, other):
        return Irreps(self) + Irreps(other)

    def count(self, _value):
        raise NotImplementedError

    def index(self, _value):
        raise NotImplementedError

    def __contains__(self, _object):
        raise NotImplementedError

    def __len__(self):
        raise NotImplementedError


class _MulIr(tuple):
    """``mul`` copies of one irrep (e3nn_lite.py:162-193)."""

    def __new__(cls, mul, ir=None):
        if ir is None:
            mul, ir = mul
        assert isinstance(mul, int)
        assert isinstance(ir, Irrep)
        return super().__new__(cls, (mul, ir))

    @property
    def mul(self) -> int:
        return self[0]

    @property
    def ir(self) -> Irrep:
        return self[1]

    @property
    def dim(self) -> int:
        return self[0] * self[1].dim

    def __repr__(self) -> str:
        return f"{self[0]}x{self[1]}"

    def count(self, _value):
        raise NotImplementedError

    def index(self, _value):
        raise NotImplementedError


def _parse_irreps_string(text: str):
    blocks = []
    if text.strip() == "":
        return blocks
    for token in text.split("+"):
        if "x" in token:
            mul_s, ir_s = token.split("x")
            mul, ir = int(mul_s), Irrep(ir_s)
        else:
            mul, ir = 1, Irrep(token)
        assert mul >= 0
        blocks.append(_MulIr(mul, ir))
    return blocks


class Irreps(tuple):
    """Direct sum of irreps with multiplicities (e3nn_lite.py:196-350).

    Accepts a string such as ``"128x0e+128x1o"``, another ``Irreps``, a single
    ``Irrep`` or any iterable of ``(mul, ir)`` pairs (this is also how e3nn's
    own ``o3.Irreps`` objects are accepted).
    """

    def __new__(cls, irreps=None):
        if isinstance(irreps, Irreps):
            return super().__new__(cls, irreps)
        blocks = []
        if isinstance(irreps, Irrep):
            blocks.append(_MulIr(1, irreps))
        elif isinstance(irreps, str):
            try:
                blocks = _parse_irreps_string(irreps)
            except Exception:
                raise ValueError(f'Unable to convert string "{irreps}" into an Irreps')
        elif irreps is not None:
            for item in irreps:
                mul, ir = None, None
                if isinstance(item, str):
                    mul, ir = 1, Irrep(item)
                elif isinstance(item, Irrep):
                    mul, ir = 1, item
                elif isinstance(item, _MulIr):
                    mul, ir = item
                elif len(item) == 2:
                    mul, ir = item
                    ir = Irrep(ir if not (hasattr(ir, "l") and hasattr(ir, "p")) else (int(ir.l), int(ir.p)))
                if not (isinstance(mul, int) and mul >= 0 and ir is not None):
                    raise ValueError(f'Unable to interpret "{item}" as an irrep.')
                blocks.append(_MulIr(mul, ir))
        return super().__new__(cls, blocks)

    @staticmethod
    def spherical_harmonics(lmax: int, p: int = -1) -> "Irreps":
        return Irreps([(1, (l, p**l)) for l in range(lmax + 1)])

    def slices(self):
        out, start = [], 0
        for block in self:
            out.append(slice(start, start + block.dim))
            start += block.dim
        return out

    def __getitem__(self, i):
        got = super().__getitem__(i)
        return Irreps(got) if isinstance(i, slice) else got

    def __contains__(self, ir) -> bool:
        ir = Irrep(ir)
        return any(ir == block_ir for _, block_ir in self)

    def count(self, ir) -> int:
        ir = Irrep(ir)
        return sum(mul for mul, block_ir in self if block_ir == ir)

    def index(self, _object):
        raise NotImplementedError

    def __add__(self, other) -> "Irreps":
        return Irreps(super().__add__(Irreps(other)))

    def __mul__(self, other) -> "Irreps":
        if isinstance(other, Irreps):
            raise NotImplementedError("Use a TPProblem for products of Irreps")
        return Irreps(super().__mul__(other))

    def __rmul__(self, other) -> "Irreps":
        return Irreps(super().__rmul__(other))

    def simplify(self) -> "Irreps":
        merged = []
        for mul, ir in self:
            if merged and merged[-1][1] == ir:
                merged[-1] = (merged[-1][0] + mul, ir)
            elif mul > 0:
                merged.append((mul, ir))
        return Irreps(merged)

    def remove_zero_multiplicities(self) -> "Irreps":
        return Irreps([(mul, ir) for mul, ir in self if mul > 0])

    def sort(self):
        """Stable sort of the blocks by ``(l, p)``; returns ``(irreps, p, inv)``
        with ``p[old_index] = new_index`` (e3nn_lite.py:319-326)."""
        Ret = collections.namedtuple("sort", ["irreps", "p", "inv"])
        order = sorted(range(len(self)), key=lambda i: (self[i].ir.l, self[i].ir.p, i))
        inv = tuple(order)
        perm = tuple(inv.index(i) for i in range(len(inv)))
        return Ret(Irreps([self[i] for i in order]), perm, inv)

    def regroup(self) -> "Irreps":
        return self.sort().irreps.simplify()

    @property
    def dim(self) -> int:
        return sum(block.dim for block in self)

    @property
    def num_irreps(self) -> int:
        return sum(mul for mul, _ in self)

    @property
    def ls(self) -> List[int]:
        return [ir.l for mul, ir in self for _ in range(mul)]

    @property
    def lmax(self) -> int:
        if len(self) == 0:
            raise ValueError("Cannot get lmax of empty Irreps")
        return max(self.ls)

    def __repr__(self) -> str:
        return "+".join(repr(block) for block in self)


class Instruction(NamedTuple):
    i_in1: int
    i_in2: int
    i_out: int
    connection_mode: str
    has_weight: bool
    path_weight: float
    path_shape: tuple


_CONNECTION_MODES = ("uvw", "uvu", "uvv", "uuw", "uuu", "uvuv", "uvu<v", "u<vw")


def _path_shape(mode: str, m1: int, m2: int, mo: int) -> tuple:
    if mode == "uvw":
        return (m1, m2, mo)
    if mode in ("uvu", "uvv", "uvuv"):
        return (m1, m2)
    if mode == "uuw":
        return (m1, mo)
    if mode == "uuu":
        return (m1,)
    if mode == "uvu<v":
        return (m1 * (m2 - 1) // 2,)
    if mode == "u<vw":
        return (m1 * (m2 - 1) // 2, mo)
    raise AssertionError(f"unknown connection mode {mode}")


def _fan_in(mode: str, m1: int, m2: int) -> int:
    """Number of products summed into one output element by one instruction
    (e3nn_lite.py:502-516)."""
    if mode == "uvw":
        return m1 * m2
    if mode == "uvu":
        return m2
    if mode in ("uvv", "uuw"):
        return m1
    if mode in ("uuu", "uvuv", "uvu<v"):
        return 1
    if mode == "u<vw":
        return m1 * (m2 - 1) // 2
    raise AssertionError(mode)


class TPProblem:
    """Specification of a weighted CG tensor product.

    Same constructor, attributes and normalisation as the reference
    (e3nn_lite.py:363-654): ``instructions`` are 5- or 6-tuples
    ``(i_in1, i_in2, i_out, mode, has_weight[, path_weight])``; after
    construction ``self.instructions`` holds ``Instruction`` tuples whose
    ``path_weight`` is the square root of the normalisation factor alpha.
    """

    def __init__(
        self,
        irreps_in1,
        irreps_in2,
        irreps_out,
        instructions: List[tuple],
        in1_var: Optional[List[float]] = None,
        in2_var: Optional[List[float]] = None,
        out_var: Optional[List[float]] = None,
        irrep_normalization: str = "component",
        path_normalization: str = "element",
        internal_weights: Optional[bool] = False,
        shared_weights: Optional[bool] = None,
        label: Optional[str] = None,
        irrep_dtype=np.float32,
        weight_dtype=np.float32,
        layout: str = "mul_ir",
    ) -> None:
        assert irrep_normalization in ["component", "norm", "none"]
        assert path_normalization in ["element", "path", "none"]
        assert layout in ["mul_ir", "ir_mul"]
        assert issubclass(irrep_dtype, np.generic)
        assert issubclass(weight_dtype, np.generic)

        self.irreps_in1 = Irreps(irreps_in1)
        self.irreps_in2 = Irreps(irreps_in2)
        self.irreps_out = Irreps(irreps_out)
        self.instructions_raw = instructions
        self.in1_var = in1_var
        self.in2_var = in2_var
        self.out_var = out_var
        self.irrep_normalization = irrep_normalization
        self.path_normalization = path_normalization
        self.label = label if label is not None else ""
        self.layout = layout

        a, b, o = self.irreps_in1, self.irreps_in2, self.irreps_out
        parsed = []
        for raw in instructions:
            raw = tuple(raw)
            if len(raw) == 5:
                raw = raw + (1.0,)
            i1, i2, io, mode, has_w, pw = raw
            assert mode in _CONNECTION_MODES
            parsed.append(
                Instruction(i1, i2, io, mode, has_w, pw, _path_shape(mode, a[i1].mul, b[i2].mul, o[io].mul))
            )

        def variances(given, irreps, name):
            if given is None:
                return [1.0] * len(irreps)
            vals = [float(v) for v in given]
            assert len(vals) == len(irreps), f"Len of {name} must be equal to the number of irreps"
            return vals

        var1 = variances(in1_var, a, "in1_var")
        var2 = variances(in2_var, b, "in2_var")
        varo = variances(out_var, o, "out_var")

        def weight_of(ins):
            return var1[ins.i_in1] * var2[ins.i_in2] * _fan_in(ins.connection_mode, a[ins.i_in1].mul, b[ins.i_in2].mul)

        normalised = []
        for ins in parsed:
            ir1, ir2, iro = a[ins.i_in1].ir, b[ins.i_in2].ir, o[ins.i_out].ir
            assert ir1.p * ir2.p == iro.p
            assert abs(ir1.l - ir2.l) <= iro.l <= ir1.l + ir2.l

            alpha = {"component": iro.dim, "norm": ir1.dim * ir2.dim, "none": 1}[irrep_normalization]
            siblings = [other for other in parsed if other.i_out == ins.i_out]
            if path_normalization == "element":
                denom = sum(weight_of(other) for other in siblings)
            elif path_normalization == "path":
                denom = weight_of(ins) * len(siblings)
            else:
                denom = 1
            if denom > 0.0:
                alpha /= denom
            alpha *= varo[ins.i_out]
            alpha *= ins.path_weight
            normalised.append(ins._replace(path_weight=math.sqrt(alpha)))
        self.instructions = normalised

        self._in1_dim = a.dim
        self._in2_dim = b.dim

        if shared_weights is False and internal_weights is None:
            internal_weights = False
        if shared_weights is None:
            shared_weights = True
        assert shared_weights or not internal_weights
        self.internal_weights = internal_weights
        self.shared_weights = shared_weights

        self.weight_numel = sum(math.prod(ins.path_shape) for ins in self.instructions if ins.has_weight)
        self.output_mask = None
        self.irrep_dtype = irrep_dtype
        self.weight_dtype = weight_dtype

    def weight_range_and_shape_for_instruction(self, instruction: int) -> Tuple[int, int, tuple]:
        ins = self.instructions[instruction]
        if not ins.has_weight:
            raise ValueError(f"Instruction {instruction} has no weights.")
        start = sum(math.prod(prev.path_shape) for prev in self.instructions[:instruction])
        return start, start + math.prod(ins.path_shape), ins.path_shape

    def clone(self) -> "TPProblem":
        return copy.deepcopy(self)

    def __str__(self) -> str:
        return (
            f"{self.__class__.__name__}({self.irreps_in1.simplify()} x "
            f"{self.irreps_in2.simplify()}) -> {self.irreps_out.simplify()}"
        )

    def __repr__(self) -> str:
        lines = [
            str(self),
            f"irrep_normalization = {self.irrep_normalization!r}",
            f"path_normalization = {self.path_normalization!r}",
            f"internal_weights = {self.internal_weights!r}",
            f"shared_weights = {self.shared_weights!r}",
            f"num weights {self.weight_numel}",
            "| in1 | in2 | out | l1 | l2 | l3 | mul1 | mul2 | mul3 | mode | weight | coeff |",
        ]
        for ins in self.instructions:
            m1, m2, mo = self.irreps_in1[ins.i_in1], self.irreps_in2[ins.i_in2], self.irreps_out[ins.i_out]
            lines.append(
                f"| {ins.i_in1:3} | {ins.i_in2:3} | {ins.i_out:3} | {m1.ir.l:2} | {m2.ir.l:2} | {mo.ir.l:2} |"
                f" {m1.mul:4} | {m2.mul:4} | {mo.mul:4} | {ins.connection_mode:<5}| {str(ins.has_weight):<5} |"
                f" {ins.path_weight:<6.4f} |"
            )
        return "\n".join(lines) + "\n"


def problem_to_dict(problem: TPProblem) -> dict:
    """The state of a problem as plain JSON-able data, for ``problem_from_dict`` in another process: the
    constructor's arguments plus what callers may have changed afterwards (dtypes, weight sharing, layout,
    the normalised instructions). Floats are written as hexadecimal strings, so nothing is rounded.
    (The reference ships its kernels' description to its ops as JSON bytes the same way,
    openequivariance/openequivariance/extension/torch_core.hpp:144-178, 637-643.)"""
    def fl(v):
        return None if v is None else [float(x).hex() for x in v]

    def raw(ins):
        ins = tuple(ins)
        return [int(ins[0]), int(ins[1]), int(ins[2]), str(ins[3]), bool(ins[4])] + \
            ([float(ins[5]).hex()] if len(ins) > 5 else [])

    return {
        "irreps_in1": str(problem.irreps_in1), "irreps_in2": str(problem.irreps_in2),
        "irreps_out": str(problem.irreps_out),
        "instructions_raw": [raw(i) for i in problem.instructions_raw],
        "instructions": [[int(i.i_in1), int(i.i_in2), int(i.i_out), str(i.connection_mode), bool(i.has_weight),
                          float(i.path_weight).hex(), [int(d) for d in i.path_shape]] for i in problem.instructions],
        "in1_var": fl(problem.in1_var), "in2_var": fl(problem.in2_var), "out_var": fl(problem.out_var),
        "irrep_normalization": problem.irrep_normalization, "path_normalization": problem.path_normalization,
        "internal_weights": bool(problem.internal_weights), "shared_weights": bool(problem.shared_weights),
        "label": problem.label, "layout": problem.layout,
        "irrep_dtype": np.dtype(problem.irrep_dtype).name, "weight_dtype": np.dtype(problem.weight_dtype).name,
    }


def problem_from_dict(d: dict) -> TPProblem:
    def fl(v):
        return None if v is None else [float.fromhex(x) for x in v]

    raw = [tuple(i[:5]) + ((float.fromhex(i[5]),) if len(i) > 5 else ()) for i in d["instructions_raw"]]
    problem = TPProblem(
        d["irreps_in1"], d["irreps_in2"], d["irreps_out"], raw, in1_var=fl(d["in1_var"]), in2_var=fl(d["in2_var"]),
        out_var=fl(d["out_var"]), irrep_normalization=d["irrep_normalization"],
        path_normalization=d["path_normalization"], internal_weights=d["internal_weights"],
        shared_weights=d["shared_weights"], label=d["label"],
        irrep_dtype=np.dtype(d["irrep_dtype"]).type, weight_dtype=np.dtype(d["weight_dtype"]).type, layout=d["layout"])
    problem.instructions = [Instruction(i[0], i[1], i[2], i[3], i[4], float.fromhex(i[5]), tuple(i[6]))
                            for i in d["instructions"]]
    problem.weight_numel = sum(math.prod(ins.path_shape) for ins in problem.instructions if ins.has_weight)
    return problem
