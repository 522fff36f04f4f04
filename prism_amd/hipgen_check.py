"""Perspective checking for Prism kernels, run before any HIP text is printed.

Every value in a Prism program lives at a perspective, `level[n]`: the value is the same for each aligned
group of n members of that level (grid, block or thread). The reference refuses programs that move data
from a narrower perspective into a broader one (prism/type_checker.py, prism/perspective.py); printing such
a program would give a kernel in which, say, a "per block" variable holds a different value in every thread.
This module states the same rules for the surface syntax hipgen accepts:

  order          grid is broader than block, block broader than thread; within a level a[m] is broader than
                 or equal to a[n] when m is a multiple of n (prism/perspective.py:52-68). narrowest(a, b) is
                 the narrower of two comparable perspectives (:78-91).
  bound          `@requires(...)` gives one perspective per level, narrower levels default to [1]
                 (:112-121); `with group(p)` needs the bound's entry at p's level to be broader than p and
                 then drops every broader level (:150-173); `match split(level): case n:` gives each case
                 the bound level[n], n at most what is left of the level (prism/type_checker.py:1244-1330).
  expressions    a name has its declared perspective, a constant is grid[1], `id()` takes the perspective of
                 what it is assigned to (the broadest entry of the bound elsewhere), a call of a Prism
                 function has that function's return perspective, anything else the narrowest of its parts;
                 `p[i]` needs p to be a pointer or array (:515-617).
  assignment     `x = e` and `x: T @ p = e` need e broader than or equal to x; a pointer is never assigned
                 (:270-379). `p[i] = e` needs p at thread[1] unless p is a private array, and e broader than
                 or equal to narrowest(p, i) (:381-415). `return e` likewise against the declared return
                 perspective (:319-329).
  LDS            `shared(...)` is declared `@ block[1]` and the declarations fit the `smem=` budget of
                 `@requires` (:282-293).
  control flow   conditions of `if` / `while` and the arguments of `range` are broader than or equal to the
                 broadest entry of the bound, where the loop variable lives too (:858-920).
  views          `partition(a, p=q, offset=e | f=lambda)` needs a to be a global or LDS pointer that is not
                 already partitioned in an enclosing scope, q narrower than or equal to a's perspective, the
                 broadest entry of the bound equal to a's perspective, and e (the lambda's body) broader
                 than or equal to q; the view lives at q (:975-1074). `claim` is the same with q strictly
                 narrower, and a claimed view is only touched inside one case of a split
                 (:1076-1178,1196-1204,1330-1345).
  calls          the caller's bound is broader than the callee's at every level the callee requires; an
                 argument for a non-const pointer parameter has exactly the parameter's perspective, any
                 other argument is broader than or equal to it; template arguments are grid[1] (:785-853).

`float4_cast[...] = v`, `v.x = e`, `unsafe("...")` and `intrinsic.*` statements are not checked, as in the
reference (:344-355).
"""
from __future__ import annotations

import ast
from dataclasses import dataclass
from typing import Dict, List, Optional, Set, Tuple

from .hipgen import HipgenError, _REGISTRY, address_space_of

_ORDER = {"grid": 0, "block": 1, "thread": 2}
_SKIPPED_CALLS = {"id", "range", "group", "split", "requires", "prism", "shared", "ptr", "const", "restrict",
                  "unsafe", "float4_cast", "min", "max", "float", "int"}


class PerspectiveError(HipgenError):
    """The program moves data against the perspective order, or breaks a rule built on it."""


@dataclass(frozen=True)
class P:
    level: str
    size: int

    def __str__(self) -> str:
        return f"{self.level}[{self.size}]"

    def covers(self, other: "P") -> bool:
        """Broader than or equal to `other`."""
        if _ORDER[self.level] != _ORDER[other.level]:
            return _ORDER[self.level] < _ORDER[other.level]
        return self.size % other.size == 0

    def narrowest(self, other: "P") -> "P":
        if self.covers(other):
            return other
        return self  # also when the two are incomparable: the assignment rules then refuse the statement


GRID1 = P("grid", 1)


@dataclass
class Bound:
    grid: Optional[P]
    block: Optional[P]
    thread: Optional[P]

    def broadest(self) -> P:
        for p in (self.grid, self.block, self.thread):
            if p is not None:
                return p
        raise PerspectiveError("@requires names no perspective")

    def at(self, level: str) -> Optional[P]:
        return getattr(self, level)

    def entered(self, p: P, where: str) -> "Bound":
        """The bound inside `with group(p)`."""
        have = self.at(p.level)
        if have is None or not have.covers(p):
            raise PerspectiveError(f"{where}: cannot enter group({p}): the bound at {p.level} level is "
                                   f"{have if have is not None else 'gone'}")
        if p.level == "grid":
            return Bound(p, self.block, self.thread)
        if p.level == "block":
            return Bound(None, p, self.thread)
        return Bound(None, None, p)


@dataclass
class Symbol:
    kind: str   # "scalar", "pointer" (global or LDS), "const pointer", "array" (private)
    where: P


@dataclass
class Signature:
    bound: Bound
    params: List[Tuple[str, Symbol]]
    returns: Optional[P]
    smem: int


def _where(node: ast.AST) -> str:
    return f"line {getattr(node, 'lineno', '?')}"


def _perspective(node: ast.AST) -> P:
    if (isinstance(node, ast.Subscript) and isinstance(node.value, ast.Name) and node.value.id in _ORDER
            and isinstance(node.slice, ast.Constant) and isinstance(node.slice.value, int) and node.slice.value > 0):
        return P(node.value.id, node.slice.value)
    raise PerspectiveError(f"{_where(node)}: expected a perspective such as block[1]")


def _kind_of_type(t: ast.AST) -> str:
    """Which of the four symbol kinds a type expression declares."""
    if isinstance(t, ast.Subscript):
        return "array"
    if isinstance(t, ast.Call) and isinstance(t.func, ast.Name):
        name = t.func.id
        if name == "shared":
            return "pointer"
        if name == "ptr":
            try:
                space = address_space_of(t)
            except HipgenError as e:
                raise PerspectiveError(str(e)) from None
            if space == "LOCAL":    # a thread's private array: indexed and stored through like one
                return "array"      # (prism/type_checker.py:399-403, 436-441)
            inner = t.args[0] if t.args else None
            if isinstance(inner, ast.Call) and isinstance(inner.func, ast.Name) and inner.func.id == "const":
                return "const pointer"
            return "pointer"
        if name in ("const", "restrict", "constexpr") and t.args:
            inner = _kind_of_type(t.args[0])
            return "const pointer" if (name == "const" and inner == "pointer") else inner
    return "scalar"


def _shared_bytes(t: ast.Call, constants: Dict[str, int]) -> int:
    sizes = {"int": 4, "float": 4, "double": 8, "bool": 1, "uint": 4, "unsigned": 4, "uint32_t": 4, "uint64_t": 8,
             "float4": 16, "bf16": 2}
    # static=True arrays are sized by the compiler and do not draw on the budget (prism/type_checker.py:466-473)
    if any(kw.arg == "static" and isinstance(kw.value, ast.Constant) and kw.value.value is True for kw in t.keywords):
        return 0
    arg = t.args[0] if t.args else None
    if not isinstance(arg, ast.Subscript) or not isinstance(arg.value, ast.Name):
        return 0
    try:
        count = _fold(arg.slice, constants)
    except PerspectiveError:
        return 0   # an extent written with template parameters is only known to the compiler
    return count * sizes.get(arg.value.id, 4)


def _fold(n: ast.AST, constants: Dict[str, int]) -> int:
    if isinstance(n, ast.Constant) and isinstance(n.value, int):
        return n.value
    if isinstance(n, ast.Name) and n.id in constants:
        return constants[n.id]
    if isinstance(n, ast.BinOp):
        a, b = _fold(n.left, constants), _fold(n.right, constants)
        ops = {ast.Add: a + b, ast.Sub: a - b, ast.Mult: a * b}
        if type(n.op) in ops:
            return ops[type(n.op)]
        if isinstance(n.op, (ast.Div, ast.FloorDiv)) and b:
            return a // b
    raise PerspectiveError("not a constant")


_SIGNATURES: Dict[str, Tuple[str, Signature]] = {}   # name -> (source it was made from, signature)


class _Checker:
    def __init__(self, name: str):
        k = _REGISTRY[name]
        self.name = name
        self.kernel = k
        self.fn = ast.parse(k.source).body[0]
        if not k.requires:
            raise PerspectiveError(f"{name}: missing @requires(...)")
        got: Dict[str, P] = {}
        for r in k.requires:
            if r.level not in _ORDER:
                raise PerspectiveError(f"{name}: @requires({r.level}[...]) is not grid, block or thread")
            if r.level in got:
                raise PerspectiveError(f"{name}: @requires names {r.level} twice")
            got[r.level] = P(r.level, r.size)
        grid, block, thread = got.get("grid"), got.get("block"), got.get("thread")
        if grid is not None:
            block = block or P("block", 1)
        if grid is not None or block is not None:
            thread = thread or P("thread", 1)
        self.bound = Bound(grid, block, thread)
        self.smem_left = k.smem if k.smem is not None else 0   # no smem=: no budget (prism/type_checker.py:288-292)
        self.scopes: List[Dict[str, Symbol]] = [{}]
        self.partitioned: List[Set[str]] = [set()]
        self.claimed: List[Set[str]] = []
        self.in_split = 0
        self.claimed_touched: Set[str] = set()
        self.returns: Optional[P] = None
        self.constants: Dict[str, int] = {}

    # symbols
    def define(self, name: str, sym: Symbol) -> None:
        self.scopes[-1][name] = sym

    def lookup(self, node: ast.Name) -> Symbol:
        for scope in reversed(self.scopes):
            if node.id in scope:
                return scope[node.id]
        raise PerspectiveError(f"{_where(node)}: '{node.id}' is not declared")

    def touch(self, node: ast.Name) -> None:
        if any(node.id in c for c in self.claimed):
            if not self.in_split:
                raise PerspectiveError(f"{_where(node)}: claimed view '{node.id}' is only accessed inside a case of a split")
            self.claimed_touched.add(node.id)

    # expressions
    def of(self, n: ast.AST, target: Optional[P] = None) -> P:
        if isinstance(n, ast.Name):
            sym = self.lookup(n)
            self.touch(n)
            return sym.where
        if isinstance(n, ast.Constant):
            return GRID1
        if isinstance(n, ast.Call):
            if isinstance(n.func, ast.Name) and n.func.id == "id" and not n.args:
                return target if target is not None else self.bound.broadest()
            if isinstance(n.func, ast.Name) and n.func.id in _REGISTRY:
                sig = signature(n.func.id)
                if sig.returns is not None:
                    return sig.returns
            out = GRID1
            for a in n.args:
                out = out.narrowest(self.of(a, target))
            return out
        if isinstance(n, ast.Subscript):
            if isinstance(n.value, ast.Name):
                if n.value.id == "float4_cast":
                    return self.of(n.slice, target)
                if self.lookup(n.value).kind == "scalar":
                    raise PerspectiveError(f"{_where(n)}: '{n.value.id}' is not a pointer or an array and cannot be indexed")
            return self.of(n.value, target).narrowest(self.of(n.slice, target))
        if isinstance(n, ast.Attribute):  # v.x of a float4
            return self.of(n.value, target)
        out = GRID1
        for child in ast.iter_child_nodes(n):
            if isinstance(child, (ast.operator, ast.unaryop, ast.cmpop, ast.boolop, ast.expr_context)):
                continue
            out = out.narrowest(self.of(child, target))
        return out

    def in_a_vacuum(self, n: ast.AST, what: str) -> None:
        got, need = self.of(n), self.bound.broadest()
        if not got.covers(need):
            raise PerspectiveError(f"{_where(n)}: the {what} is at {got}; it must be broader than or equal to {need}, "
                                   "the broadest perspective here")

    # statements
    def body(self, stmts: List[ast.stmt]) -> None:
        for s in stmts:
            self.stmt(s)

    def stmt(self, s: ast.stmt) -> None:
        if isinstance(s, ast.AnnAssign):
            self.declare(s)
        elif isinstance(s, ast.Assign):
            if len(s.targets) != 1:
                raise PerspectiveError(f"{_where(s)}: one target per assignment")
            self.assign(s.targets[0], s.value)
            self.calls_in(s.value)
        elif isinstance(s, ast.AugAssign):
            self.assign(s.target, s.value)
            self.calls_in(s.value)
        elif isinstance(s, ast.Return):
            if s.value is not None and self.returns is not None:
                got = self.of(s.value, self.returns)
                if not got.covers(self.returns):
                    raise PerspectiveError(f"{_where(s)}: returns a value at {got} from a function declared to return at {self.returns}")
                self.calls_in(s.value)
        elif isinstance(s, ast.Expr):
            self.calls_in(s.value)
        elif isinstance(s, ast.If):
            self.in_a_vacuum(s.test, "condition of this `if`")
            self.scoped(s.body)
            self.scoped(s.orelse)
        elif isinstance(s, ast.While):
            self.in_a_vacuum(s.test, "condition of this `while`")
            self.scoped(s.body)
        elif isinstance(s, ast.For):
            if not (isinstance(s.iter, ast.Call) and isinstance(s.iter.func, ast.Name) and s.iter.func.id == "range"
                    and isinstance(s.target, ast.Name)):
                raise PerspectiveError(f"{_where(s)}: loops are `for name in range(...)`")
            for a in s.iter.args:
                self.in_a_vacuum(a, "range of this loop")
            self.scopes.append({s.target.id: Symbol("scalar", self.bound.broadest())})
            self.body(s.body)
            self.scopes.pop()
        elif isinstance(s, ast.With):
            self.with_(s)
        elif isinstance(s, ast.Match):
            self.split(s)
        elif isinstance(s, ast.Pass):
            pass
        else:
            raise PerspectiveError(f"{_where(s)}: unsupported statement {type(s).__name__}")

    def scoped(self, stmts: List[ast.stmt]) -> None:
        self.scopes.append({})
        self.body(stmts)
        self.scopes.pop()

    def declare(self, s: ast.AnnAssign) -> None:
        if not isinstance(s.target, ast.Name):
            raise PerspectiveError(f"{_where(s)}: a declaration names one variable")
        if not (isinstance(s.annotation, ast.BinOp) and isinstance(s.annotation.op, ast.MatMult)):
            raise PerspectiveError(f"{_where(s)}: '{s.target.id}' needs a `type @ perspective` annotation")
        t, p = s.annotation.left, _perspective(s.annotation.right)
        kind = _kind_of_type(t)
        if isinstance(t, ast.Call) and isinstance(t.func, ast.Name) and t.func.id == "shared":
            if p != P("block", 1):
                raise PerspectiveError(f"{_where(s)}: LDS array '{s.target.id}' is declared at {p}; shared memory lives at block[1]")
            need = _shared_bytes(t, self.constants)
            if self.smem_left is not None:
                if need > self.smem_left:
                    raise PerspectiveError(f"{_where(s)}: LDS array '{s.target.id}' needs {need} bytes, {self.smem_left} "
                                           "are left of the smem= budget")
                self.smem_left -= need
        self.define(s.target.id, Symbol(kind, p))
        if s.value is None or isinstance(s.value, ast.Set):   # `= {0}` zero-fills an array
            return
        if kind in ("pointer", "const pointer"):
            got = self.of(s.value, p)
            if not got.covers(p):
                raise PerspectiveError(f"{_where(s)}: '{s.target.id}' at {p} is initialised from a value at {got}")
        else:
            self.assign(s.target, s.value)
        if kind == "scalar" and p == GRID1:
            try:
                self.constants[s.target.id] = _fold(s.value, self.constants)
            except PerspectiveError:
                pass
        self.calls_in(s.value)

    def assign(self, target: ast.AST, value: ast.AST) -> None:
        if isinstance(target, ast.Subscript):
            if isinstance(target.value, ast.Name) and target.value.id == "float4_cast":
                return
            if not isinstance(target.value, ast.Name):
                raise PerspectiveError(f"{_where(target)}: a store goes through a named pointer or array")
            sym = self.lookup(target.value)
            self.touch(target.value)
            if sym.kind == "scalar":
                raise PerspectiveError(f"{_where(target)}: '{target.value.id}' is not a pointer or an array and cannot be indexed")
            if sym.kind != "array" and sym.where != P("thread", 1):
                raise PerspectiveError(f"{_where(target)}: a store through '{target.value.id}' at {sym.where}: partition it down to "
                                       "thread[1] first, so that one thread owns each element it writes")
            to = sym.where.narrowest(self.of(target.slice))
            got = self.of(value)
            if not got.covers(to):
                raise PerspectiveError(f"{_where(target)}: '{target.value.id}[...]' at {to} cannot take a value at {got}")
            return
        if isinstance(target, ast.Attribute):
            return
        if not isinstance(target, ast.Name):
            raise PerspectiveError(f"{_where(target)}: cannot assign to this")
        sym = self.lookup(target)
        if sym.kind in ("pointer", "const pointer"):
            raise PerspectiveError(f"{_where(target)}: pointer '{target.id}' is not assignable")
        got = self.of(value, sym.where)
        if not got.covers(sym.where):
            raise PerspectiveError(f"{_where(target)}: '{target.id}' at {sym.where} cannot take a value at {got}: the right-hand "
                                   "side must be broader than or equal to the left")

    # calls of other Prism functions, anywhere inside an expression
    def calls_in(self, n: ast.AST) -> None:
        for c in ast.walk(n):
            if isinstance(c, ast.Call) and isinstance(c.func, ast.Name) and c.func.id in _REGISTRY \
                    and c.func.id not in _SKIPPED_CALLS and c.func.id != self.name:
                self.call(c)

    def call(self, c: ast.Call) -> None:
        name = c.func.id
        sig = signature(name)
        if self.smem_left is not None and sig.smem > self.smem_left:
            raise PerspectiveError(f"{_where(c)}: {name} needs {sig.smem} bytes of LDS, {self.smem_left} are left")
        for level in ("grid", "block", "thread"):
            need, have = sig.bound.at(level), self.bound.at(level)
            if need is not None and (have is None or not have.covers(need)):
                raise PerspectiveError(f"{_where(c)}: {name} requires {need}; the caller is at "
                                       f"{have if have is not None else 'no ' + level + ' level'}")
        for a, (pname, psym) in zip(c.args, sig.params):
            got = self.of(a)
            if psym.kind == "pointer":
                if got != psym.where:
                    raise PerspectiveError(f"{_where(c)}: {name}({pname}=...) takes a pointer at exactly {psym.where}, got {got}")
            elif not got.covers(psym.where):
                raise PerspectiveError(f"{_where(c)}: {name}({pname}=...) is at {psym.where}; the argument at {got} is narrower")
        for kw in c.keywords:
            if kw.arg == "template" and isinstance(kw.value, (ast.List, ast.Tuple)):
                for e in kw.value.elts:
                    if self.of(e) != GRID1:
                        raise PerspectiveError(f"{_where(c)}: template arguments of {name} are grid[1] values")

    # with group / partition / claim
    def with_(self, s: ast.With) -> None:
        call = s.items[0].context_expr if len(s.items) == 1 else None
        if not (isinstance(call, ast.Call) and isinstance(call.func, ast.Name)
                and call.func.id in ("group", "partition", "claim")):
            raise PerspectiveError(f"{_where(s)}: `with` takes group(), partition() or claim()")
        if call.func.id == "group":
            if len(call.args) != 1:
                raise PerspectiveError(f"{_where(s)}: group() takes one perspective")
            old = self.bound
            self.bound = old.entered(_perspective(call.args[0]), _where(s))
            self.scoped(s.body)
            self.bound = old
            return
        what = call.func.id
        target = s.items[0].optional_vars
        if not isinstance(target, ast.Name):
            raise PerspectiveError(f"{_where(s)}: {what}() needs `as name`")
        if len(call.args) != 1 or not isinstance(call.args[0], ast.Name):
            raise PerspectiveError(f"{_where(s)}: {what}() takes the pointer's name and keywords")
        base = call.args[0]
        sym = self.lookup(base)
        if sym.kind == "scalar":
            raise PerspectiveError(f"{_where(s)}: '{base.id}' is not a pointer")
        if sym.kind == "array":
            raise PerspectiveError(f"{_where(s)}: '{base.id}' is a private array; only global and LDS pointers are partitioned")
        to, f, offset = None, None, None
        for kw in call.keywords:
            if kw.arg == "p":
                to = _perspective(kw.value)
            elif kw.arg == "f":
                if not isinstance(kw.value, ast.Lambda):
                    raise PerspectiveError(f"{_where(s)}: f= takes a lambda")
                f = kw.value
            elif kw.arg == "offset":
                offset = kw.value
            else:
                raise PerspectiveError(f"{_where(s)}: {what}() has no keyword '{kw.arg}'")
        if to is None:
            raise PerspectiveError(f"{_where(s)}: {what}() needs p=<perspective>")
        if f is not None and offset is not None:
            raise PerspectiveError(f"{_where(s)}: {what}() takes f= or offset=, not both")
        if what == "partition" and f is None and offset is None:
            raise PerspectiveError(f"{_where(s)}: partition() needs f= or offset=")
        if not sym.where.covers(to) or (what == "claim" and sym.where == to):
            raise PerspectiveError(f"{_where(s)}: '{base.id}' at {sym.where} cannot be narrowed to {to}")
        if self.bound.broadest() != sym.where:
            raise PerspectiveError(f"{_where(s)}: '{base.id}' lives at {sym.where} but the broadest perspective here is "
                                   f"{self.bound.broadest()}: {what} it where all of {sym.where} is present")
        if any(base.id in held for held in self.partitioned):
            raise PerspectiveError(f"{_where(s)}: '{base.id}' is already partitioned")
        if f is not None:
            self.scopes.append({a.arg: Symbol("scalar", to) for a in f.args.args})
            got = self.of(f.body, to)
            self.scopes.pop()
        elif offset is not None:
            got = self.of(offset, to)
        else:
            got = GRID1
        if not got.covers(to):
            raise PerspectiveError(f"{_where(s)}: the offset of view '{target.id}' is at {got}, narrower than the view's {to}")
        self.partitioned[-1].add(base.id)
        self.partitioned.append(set())
        self.scopes.append({target.id: Symbol(sym.kind, to)})
        if what == "claim":
            self.claimed.append({target.id})
        self.body(s.body)
        if what == "claim":
            self.claimed.pop()
        self.scopes.pop()
        self.partitioned.pop()
        self.partitioned[-1].discard(base.id)

    def split(self, s: ast.Match) -> None:
        subject = s.subject
        if not (isinstance(subject, ast.Call) and isinstance(subject.func, ast.Name) and subject.func.id == "split"
                and len(subject.args) == 1 and isinstance(subject.args[0], ast.Name) and subject.args[0].id in _ORDER):
            raise PerspectiveError(f"{_where(s)}: `match` takes split(grid | block | thread)")
        level = subject.args[0].id
        have = self.bound.at(level)
        if have is None:
            raise PerspectiveError(f"{_where(s)}: cannot split {level}: that level is not part of the bound here")
        old, left = self.bound, have.size
        seen_claimed: Set[str] = set()
        for case in s.cases:
            v = case.pattern.value if isinstance(case.pattern, ast.MatchValue) else None
            if not (isinstance(v, ast.Constant) and isinstance(v.value, int)):
                raise PerspectiveError(f"{_where(case.pattern)}: a case of a split is a member count")
            n = v.value
            if n > left or n <= 0:
                raise PerspectiveError(f"{_where(case.pattern)}: case {n} of split({level}): only {left} of {have} are left")
            mine = P(level, n)
            self.bound = (Bound(mine, old.block, old.thread) if level == "grid" else
                          Bound(None, mine, old.thread) if level == "block" else Bound(None, None, mine))
            self.partitioned.append(set())
            outer_touched, self.claimed_touched = self.claimed_touched, set()
            self.in_split += 1
            self.scoped(case.body)
            self.in_split -= 1
            both = self.claimed_touched & seen_claimed
            if both:
                raise PerspectiveError(f"{_where(s)}: claimed view '{sorted(both)[0]}' is accessed in more than one case of the split")
            self.partitioned.pop()   # a view ends with its `with`: siblings may partition the same pointer again
            seen_claimed |= self.claimed_touched
            self.claimed_touched = outer_touched | self.claimed_touched
            left -= n
        self.bound = old

    # the function
    def run(self) -> Signature:
        fn = self.fn
        if not isinstance(fn, ast.FunctionDef):
            raise PerspectiveError(f"{self.name}: expected a function definition")
        params: List[Tuple[str, Symbol]] = []
        args = fn.args.args
        defaults = dict(zip([a.arg for a in args[len(args) - len(fn.args.defaults):]], fn.args.defaults))
        for a in args:
            if a.arg == "template":
                d = defaults.get("template")
                for item in getattr(d, "elts", []):
                    if isinstance(item, ast.Tuple) and item.elts and isinstance(item.elts[0], ast.Constant):
                        self.define(str(item.elts[0].value), Symbol("scalar", GRID1))
                continue
            if not (isinstance(a.annotation, ast.BinOp) and isinstance(a.annotation.op, ast.MatMult)):
                raise PerspectiveError(f"{self.name}: parameter {a.arg} needs a `type @ perspective` annotation")
            sym = Symbol(_kind_of_type(a.annotation.left), _perspective(a.annotation.right))
            params.append((a.arg, sym))
            self.define(a.arg, sym)
        if fn.returns is not None and isinstance(fn.returns, ast.BinOp) and isinstance(fn.returns.op, ast.MatMult):
            self.returns = _perspective(fn.returns.right)
        sig = Signature(self.bound, params, self.returns, self.kernel.smem or 0)
        _SIGNATURES[self.name] = (self.kernel.source, sig)   # in place before the body: a recursive call finds it
        try:
            self.scoped(fn.body)
        except Exception:
            _SIGNATURES.pop(self.name, None)
            raise
        return sig


def signature(name: str) -> Signature:
    """Checks function `name` (once per source text) and returns what its callers are checked against."""
    if name not in _REGISTRY:
        raise HipgenError(f"no kernel named {name!r} has been defined with @prism")
    cached = _SIGNATURES.get(name)
    if cached is not None and cached[0] == _REGISTRY[name].source:
        return cached[1]
    return _Checker(name).run()


def check(name: str) -> None:
    """Raises PerspectiveError if kernel or device function `name`, or anything it calls, breaks a rule."""
    signature(name)
