"""A HIP emitter for the thread-level subset of the Prism DSL (gfx950).

The reference's product is a source-to-source compiler: kernels are Python
functions decorated with ``@prism("global")`` whose parameters and locals carry a
perspective (``@ grid[1]``, ``@ thread[1]``), and ``generate(name)`` prints CUDA
(prism/codegen.py:321-384,758-849; surface syntax in examples/add_m_thread.py:10-19,
expected text in README.md:133-140). This module is the first slice of a HIP
back-end for that front end: it accepts the same surface syntax for kernels whose
work is expressed per thread --

    @requires(grid[1], thread[1])
    @prism("global")
    def add_m_thread(x: ptr(const(int)) @ grid[1], y: ptr(int) @ grid[1], m: int @ grid[1]):
        tid: int @ thread[1] = id()
        with partition(x, p=thread[1], offset=tid) as x_thread:
            with partition(y, p=thread[1], offset=tid) as y_thread:
                with group(thread[1]):
                    y_thread[0] = x_thread[0] + m

-- and prints a HIP kernel, optionally with an element count and a bounds guard
(the reference kernel has neither and must be launched with exactly n threads),
plus an ``extern "C"`` launcher that picks the grid. ``build()`` compiles the text
with hipcc for gfx950 and returns a ctypes handle; nothing is interpreted on the
CPU and there is no fallback.

Supported here: scalar and pointer parameters of int / float / unsigned, ``id()`` at
thread perspective, nested ``partition(..., p=thread[1], offset=e)`` views,
``group(thread[1])`` bodies with assignments, augmented assignments, arithmetic,
comparisons and ``if``. Kernels that declare a block perspective (block-level ids
and views, LDS arrays with automatic barriers, loops, templates, device functions)
are handed to hipgen_blocks.py, which keeps the reference's nested structure.
Anything else raises ``HipgenError`` naming the construct.

The decorators only register the function's source; annotations are evaluated by
Python at definition time, so the perspective objects below implement ``[]`` and
``@`` and nothing else.
"""
from __future__ import annotations

import ast
import ctypes
import inspect
import subprocess
import tempfile
import textwrap
from dataclasses import dataclass, field
from pathlib import Path
from typing import Callable, Dict, List, Optional

__all__ = ["prism", "requires", "attr", "grid", "block", "thread", "ptr", "const", "restrict", "constexpr",
           "GLOBAL", "SHARED", "LOCAL",
           "shared", "uint", "double", "uint32_t", "uint64_t", "group", "partition", "claim", "split", "unsafe",
           "generate", "generate_launcher", "build", "HipgenError"]


class HipgenError(Exception):
    """The kernel uses something outside the supported subset."""


# ------------------------------------------------------------ surface syntax --

@dataclass(frozen=True)
class Perspective:
    level: str
    size: int = 1

    def __getitem__(self, size: int) -> "Perspective":
        return Perspective(self.level, int(size))

    def __rmatmul__(self, other):  # `int @ thread[1]`
        return Located(other, self)


@dataclass(frozen=True)
class Located:
    ctype: object
    where: Perspective


@dataclass(frozen=True)
class CType:
    text: str

    def __matmul__(self, where: Perspective):  # `ptr(int) @ grid[1]`
        return Located(self, where)


# The levels of the reference (prism/perspective.py:10-14); its "warps" are thread[32] groups, here thread[64].
grid, block, thread = (Perspective(n) for n in ("grid", "block", "thread"))

_SCALARS = {"int": "int", "float": "float", "unsigned": "unsigned int", "uint": "unsigned int", "bool": "bool",
            "double": "double", "uint32_t": "uint32_t", "uint64_t": "uint64_t", "bf16": "__bf16", "float4": "float4",
            "void": "void"}


def _ctype_text(t) -> str:
    if isinstance(t, CType):
        return t.text
    name = getattr(t, "__name__", str(t))
    if name in _SCALARS:
        return _SCALARS[name]
    if isinstance(t, _TypeName):  # shared(T) inside ptr(...): kernels are compiled from their source text,
        return name               # these objects only have to let the annotations evaluate
    raise HipgenError(f"unsupported element type {t!r}")


def const(t) -> CType:
    return CType("const " + _ctype_text(t))


def restrict(t) -> CType:
    return CType(_ctype_text(t) + " __restrict__")


def constexpr(t) -> CType:
    return CType("constexpr " + _ctype_text(t))


class _TypeName:
    """A type that Python has no builtin name for (`uint`, `double`, ...): annotations are parsed from
    the source, so these only have to exist, be callable and be indexable."""

    def __init__(self, name: str):
        self.__name__ = name

    def __getitem__(self, _size):
        return self

    def __call__(self, *args, **kwargs):
        return self

    def __matmul__(self, where):
        return Located(self, where)


uint, double, uint32_t, uint64_t = (_TypeName(n) for n in ("uint", "double", "uint32_t", "uint64_t"))
shared = _TypeName("shared")
bf16, void = _TypeName("bf16"), _TypeName("void")
float4 = _TypeName("float4")
float4_cast = _TypeName("float4_cast")  # float4_cast(x[i]) reads, float4_cast[x[i]] = v writes 16 bytes at &x[i]


def ptr(t, space=None) -> CType:
    """`ptr(T)` or `ptr(T, GLOBAL | SHARED | LOCAL)` (prism/type_checker.py:656-667); the address space does not
    show in the C text: HIP's generic pointers cover global memory, LDS and private arrays alike."""
    return CType(_ctype_text(t) + "*")


# The address spaces a pointer type may name. `ptr(T, SHARED)` is what `shared(T)` is as a parameter type: a
# pointer into LDS, which the barrier analysis follows; `ptr(T, LOCAL)` points at a thread's private array
# and may be stored through at any perspective.
GLOBAL, SHARED, LOCAL = (_TypeName(n) for n in ("GLOBAL", "SHARED", "LOCAL"))
ADDRESS_SPACES = ("GLOBAL", "SHARED", "LOCAL")


def address_space_of(node: ast.AST) -> str:
    """The address space a `ptr(T[, SPACE])` call node names (GLOBAL when it names none)."""
    if len(node.args) < 2:
        return "GLOBAL"
    space = node.args[1]
    if not isinstance(space, ast.Name) or space.id not in ADDRESS_SPACES:
        raise HipgenError(f"line {getattr(node, 'lineno', '?')}: the address space of a pointer is GLOBAL, SHARED or LOCAL")
    return space.id


def group(_where):  # only ever appears inside kernel bodies, which are parsed, not run
    raise HipgenError("group() is part of a kernel body; kernels are compiled with generate(), not called")


partition = group
claim = group
split = group
unsafe = group


class _Intrinsics:
    """`intrinsic.<name>(...)` statements in kernel bodies (parsed, never run)."""

    def __getattr__(self, name):
        return group


intrinsic = _Intrinsics()

_REGISTRY: Dict[str, "Kernel"] = {}


@dataclass
class Kernel:
    name: str
    kind: str
    source: str
    requires: tuple = ()
    smem: Optional[int] = None   # @requires(..., smem=bytes): LDS budget the author states
    attr: str = ""               # @attr("..."): text between the qualifier and the return type
    fn: Optional[Callable] = field(default=None, repr=False)


def prism(kind: str):
    if kind not in ("global", "device"):
        raise HipgenError(f'@prism("{kind}"): expected "global" or "device"')

    def deco(fn):
        _REGISTRY[fn.__name__] = Kernel(fn.__name__, kind, textwrap.dedent(inspect.getsource(fn)), fn=fn)
        return fn
    return deco


def requires(*perspectives: Perspective, smem: Optional[int] = None):
    def deco(fn):
        k = _REGISTRY.get(fn.__name__)
        if k is None:
            raise HipgenError("@requires must be applied above @prism")
        k.requires = tuple(perspectives)
        k.smem = smem
        return fn
    return deco


def attr(text: str):
    """`@attr("__launch_bounds__(256)")`, above @prism: printed between the qualifier and the return type."""
    def deco(fn):
        k = _REGISTRY.get(fn.__name__)
        if k is None:
            raise HipgenError("@attr must be applied above @prism")
        k.attr = str(text)
        return fn
    return deco


# ------------------------------------------------------------------ emitter --

_BINOPS = {ast.Add: "+", ast.Sub: "-", ast.Mult: "*", ast.Div: "/", ast.Mod: "%", ast.LShift: "<<",
           ast.RShift: ">>", ast.BitAnd: "&", ast.BitOr: "|", ast.BitXor: "^", ast.FloorDiv: "/"}
_CMPOPS = {ast.Lt: "<", ast.LtE: "<=", ast.Gt: ">", ast.GtE: ">=", ast.Eq: "==", ast.NotEq: "!="}
_UNOPS = {ast.USub: "-", ast.Invert: "~", ast.Not: "!"}


def _perspective_of(node: ast.AST) -> Perspective:
    """`thread[1]` / `grid[1]` as written in the source."""
    if isinstance(node, ast.Subscript) and isinstance(node.value, ast.Name) and node.value.id in (
            "grid", "block", "thread"):
        size = node.slice
        if isinstance(size, ast.Constant) and isinstance(size.value, int):
            return Perspective(node.value.id, size.value)
    raise HipgenError(f"line {getattr(node, 'lineno', '?')}: expected a perspective such as thread[1]")


def _type_of(node: ast.AST) -> str:
    """`ptr(const(int))`, `int` ... as written in the source."""
    if isinstance(node, ast.Name):
        if node.id in _SCALARS:
            return _SCALARS[node.id]
        raise HipgenError(f"line {node.lineno}: unsupported type {node.id}")
    if isinstance(node, ast.Call) and isinstance(node.func, ast.Name) and node.func.id == "ptr" and len(node.args) == 2:
        address_space_of(node)
        return _type_of(node.args[0]) + "*"
    if isinstance(node, ast.Call) and isinstance(node.func, ast.Name) and len(node.args) == 1:
        inner = _type_of(node.args[0])
        if node.func.id == "ptr":
            return inner + "*"
        if node.func.id == "const":
            return "const " + inner
    raise HipgenError(f"line {getattr(node, 'lineno', '?')}: unsupported type expression")


def _split_annotation(node: ast.AST):
    """`T @ where` -> (C type text, Perspective)."""
    if isinstance(node, ast.BinOp) and isinstance(node.op, ast.MatMult):
        return _type_of(node.left), _perspective_of(node.right)
    raise HipgenError(f"line {getattr(node, 'lineno', '?')}: annotation must be `type @ perspective`")


class _Emitter:
    def __init__(self, kernel: Kernel, bounded: bool):
        self.k = kernel
        self.bounded = bounded
        self.lines: List[str] = []
        self.views: Dict[str, tuple] = {}   # view name -> (base expression text, offset expression text)
        self.params: List[tuple] = []       # (ctype, name)
        self.thread_ids: List[str] = []

    # expressions
    def expr(self, n: ast.AST) -> str:
        if isinstance(n, ast.Constant):
            if isinstance(n.value, bool):
                return "true" if n.value else "false"
            if isinstance(n.value, int):
                return str(n.value)
            if isinstance(n.value, float):
                return repr(n.value) + "f"
            raise HipgenError(f"line {n.lineno}: unsupported constant {n.value!r}")
        if isinstance(n, ast.Name):
            if n.id in self.views:
                raise HipgenError(f"line {n.lineno}: view {n.id} must be indexed")
            return n.id
        if isinstance(n, ast.BinOp) and type(n.op) in _BINOPS:
            return f"{self.operand(n.left)} {_BINOPS[type(n.op)]} {self.operand(n.right)}"
        if isinstance(n, ast.UnaryOp) and type(n.op) in _UNOPS:
            return f"{_UNOPS[type(n.op)]}{self.operand(n.operand)}"
        if isinstance(n, ast.Compare) and len(n.ops) == 1 and type(n.ops[0]) in _CMPOPS:
            return f"{self.operand(n.left)} {_CMPOPS[type(n.ops[0])]} {self.operand(n.comparators[0])}"
        if isinstance(n, ast.Subscript):
            return self.element(n)
        raise HipgenError(f"line {getattr(n, 'lineno', '?')}: unsupported expression {ast.dump(n)[:60]}")

    def operand(self, n: ast.AST) -> str:
        text = self.expr(n)
        return f"({text})" if isinstance(n, (ast.BinOp, ast.Compare)) else text

    def element(self, n: ast.Subscript) -> str:
        if not isinstance(n.value, ast.Name):
            raise HipgenError(f"line {n.lineno}: only named arrays and views can be indexed")
        idx = self.expr(n.slice)
        name = n.value.id
        if name in self.views:
            base, off = self.views[name]
            return f"{base}[{off}]" if idx == "0" else f"{base}[{off} + {idx}]"
        return f"{name}[{idx}]"

    # statements
    def stmt(self, n: ast.stmt, depth: int) -> None:
        pad = "    " * depth
        if isinstance(n, ast.AnnAssign) and isinstance(n.target, ast.Name):
            ctype, where = _split_annotation(n.annotation)
            if isinstance(n.value, ast.Call) and isinstance(n.value.func, ast.Name) and n.value.func.id == "id":
                if where != Perspective("thread", 1):
                    raise HipgenError(f"line {n.lineno}: id() is supported at thread[1] only (got {where.level}[{where.size}])")
                self.lines.append(f"{pad}{ctype} {n.target.id} = blockIdx.x * blockDim.x + threadIdx.x;")
                self.thread_ids.append(n.target.id)
                if self.bounded and len(self.thread_ids) == 1:
                    self.lines.append(f"{pad}if ({n.target.id} >= prism_n) return;")
                return
            if n.value is None:
                self.lines.append(f"{pad}{ctype} {n.target.id};")
            else:
                self.lines.append(f"{pad}{ctype} {n.target.id} = {self.expr(n.value)};")
            return
        if isinstance(n, ast.With) and len(n.items) == 1:
            call = n.items[0].context_expr
            if isinstance(call, ast.Call) and isinstance(call.func, ast.Name):
                if call.func.id == "partition":
                    self.partition(call, n.items[0].optional_vars, n)
                    for s in n.body:
                        self.stmt(s, depth)
                    return
                if call.func.id == "group":
                    where = _perspective_of(call.args[0]) if call.args else None
                    if where != Perspective("thread", 1):
                        raise HipgenError(f"line {n.lineno}: group() is supported at thread[1] only")
                    for s in n.body:
                        self.stmt(s, depth)
                    return
            raise HipgenError(f"line {n.lineno}: unsupported with-statement")
        if isinstance(n, ast.Assign) and len(n.targets) == 1:
            self.lines.append(f"{pad}{self.expr(n.targets[0])} = {self.expr(n.value)};")
            return
        if isinstance(n, ast.AugAssign) and type(n.op) in _BINOPS:
            self.lines.append(f"{pad}{self.expr(n.target)} {_BINOPS[type(n.op)]}= {self.expr(n.value)};")
            return
        if isinstance(n, ast.If):
            self.lines.append(f"{pad}if ({self.expr(n.test)}) {{")
            for s in n.body:
                self.stmt(s, depth + 1)
            if n.orelse:
                self.lines.append(f"{pad}}} else {{")
                for s in n.orelse:
                    self.stmt(s, depth + 1)
            self.lines.append(f"{pad}}}")
            return
        if isinstance(n, ast.Expr) and isinstance(n.value, ast.Constant) and isinstance(n.value.value, str):
            return  # docstring
        if isinstance(n, ast.Pass):
            return
        raise HipgenError(f"line {n.lineno}: unsupported statement {type(n).__name__}")

    def partition(self, call: ast.Call, target, node) -> None:
        if not isinstance(target, ast.Name) or not call.args or not isinstance(call.args[0], ast.Name):
            raise HipgenError(f"line {node.lineno}: expected `with partition(array, p=..., offset=...) as view`")
        kw = {k.arg: k.value for k in call.keywords}
        if set(kw) != {"p", "offset"}:
            raise HipgenError(f"line {node.lineno}: partition() takes p= and offset=")
        where = _perspective_of(kw["p"])
        if where != Perspective("thread", 1):
            raise HipgenError(f"line {node.lineno}: partition() is supported at p=thread[1] only (got {where.level}[{where.size}])")
        off = self.operand(kw["offset"])
        parent = call.args[0].id
        if parent in self.views:  # a view of a view: offsets add up
            base, parent_off = self.views[parent]
            self.views[target.id] = (base, f"{parent_off} + {off}")
        else:
            self.views[target.id] = (parent, off)

    def emit(self) -> str:
        tree = ast.parse(self.k.source)
        fn = tree.body[0]
        if not isinstance(fn, ast.FunctionDef):
            raise HipgenError("expected a function definition")
        for a in fn.args.args:
            if a.annotation is None:
                raise HipgenError(f"parameter {a.arg} needs a `type @ perspective` annotation")
            ctype, where = _split_annotation(a.annotation)
            if where.level != "grid":
                raise HipgenError(f"parameter {a.arg}: kernel parameters live at grid perspective")
            self.params.append((ctype, a.arg))
        for s in fn.body:
            self.stmt(s, 1)
        if self.bounded and not self.thread_ids:
            raise HipgenError("a bounded kernel needs a thread id (`tid: int @ thread[1] = id()`)")
        params = ", ".join(f"{t} {n}" for t, n in self.params)
        if self.bounded:
            params += (", " if params else "") + "size_t prism_n"
        qualifier = "__global__" if self.k.kind == "global" else "__device__"
        head = f"{qualifier} void {self.k.name}({params}) {{"
        return "\n".join([head, *self.lines, "}"]) + "\n"


def _kernel(name: str) -> Kernel:
    try:
        return _REGISTRY[name]
    except KeyError:
        raise HipgenError(f"no kernel named {name!r} has been defined with @prism") from None


def _structured(k: Kernel) -> bool:
    """Kernels with a block perspective (or device functions) keep the nested form of hipgen_blocks.py."""
    return k.kind == "device" or any(p.level == "block" for p in k.requires)


def _check_perspectives(name: str) -> None:
    """Nothing is printed for a program that moves data against the perspective order
    (the reference type-checks before it generates, prism/codegen.py:1000-1014)."""
    from .hipgen_check import check
    check(name)


def generate(name: str, bounded: bool = False, auto_sync: bool = True, annotate: bool = False) -> str:
    """HIP text of kernel `name`.

    Thread-level kernels (@requires without a block perspective) are printed flat. bounded=False prints
    what the reference prints for the same source (one thread per element, no guard); bounded=True
    appends a `size_t prism_n` parameter and returns early for thread ids beyond it, so that any grid
    covering n is legal. Kernels with a block perspective are printed by hipgen_blocks.generate_blocks
    (auto_sync places the barriers, annotate=True says in a comment what each is for); they carry their own
    guards, so bounded does not apply."""
    k = _kernel(name)
    _check_perspectives(name)
    if _structured(k):
        if bounded:
            raise HipgenError("bounded=True applies to thread-level kernels only")
        from .hipgen_blocks import generate_blocks
        return generate_blocks(name, auto_sync, annotate)
    return _Emitter(k, bounded).emit()


def generate_launcher(name: str, block_size: int = 256, template: Optional[List[int]] = None,
                      handover_spins: Optional[int] = None) -> str:
    """The kernel plus an `extern "C"` launcher.

    Thread-level kernel: bounded kernel and `int <name>_launch(<params>, size_t n, void* stream)`, which
    starts ceil(n / block_size) workgroups. Kernel with a block perspective:
    `int <name>_launch(<params>, unsigned grid_blocks, void* stream)`, which starts grid_blocks workgroups
    of block_size threads with the dynamic LDS the kernel's shared() arrays need; `template` gives the
    values of its template parameters. block_size is a multiple of the 64-lane wavefront.

    A kernel that hands LDS arrays between the cases of a split also gets `int <name>_status(void* stream)`:
    it waits for the stream and returns 0, or, when a hand-over wait of any launch since the last call ran
    out of polls (handover_spins of them; the default is the emitter's), 0x40000000 | code, where the code's
    low byte is 1 + 2 * (number of the array in declaration order) + (1 for a wait for a filled array) and
    the bits above it the round; the results of that launch are invalid. The call clears the report."""
    if block_size % 64 or not 64 <= block_size <= 1024:
        raise HipgenError("block_size must be a multiple of 64 between 64 and 1024")
    k = _kernel(name)
    _check_perspectives(name)
    head = "#include <hip/hip_runtime.h>\n#include <cstddef>\n#include <cstdint>\n\n"
    if _structured(k):
        from .hipgen_blocks import BlockEmitter, device_functions_used, generate_blocks
        if k.kind != "global":
            raise HipgenError("only global kernels have launchers")
        em = BlockEmitter(k, True, handover_spins=handover_spins)
        text = em.emit_function()
        if len(template or []) != len(em.template):
            raise HipgenError(f"{name} has {len(em.template)} template parameters, {len(template or [])} values given")
        if k.smem is not None and em.smem_offset > k.smem:
            raise HipgenError(f"{name} declares smem={k.smem} but its shared() arrays take {em.smem_offset} bytes")
        from .hipgen_blocks import HANDOVER_REPORT
        helpers = "".join(generate_blocks(d, handover_spins=handover_spins) + "\n" for d in device_functions_used(name))
        status = ""
        if HANDOVER_REPORT in helpers + text:
            status = (
                f'\nextern "C" int {name}_status(void* stream) {{\n'
                "    hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(stream));\n"
                "    if (e != hipSuccess) return static_cast<int>(e);\n"
                "    unsigned int word = 0;\n"
                f"    e = hipMemcpyFromSymbol(&word, HIP_SYMBOL({HANDOVER_REPORT}), sizeof(word));\n"
                "    if (e != hipSuccess) return static_cast<int>(e);\n"
                "    if (word == 0) return 0;\n"
                "    const unsigned int zero = 0;\n"
                f"    e = hipMemcpyToSymbol(HIP_SYMBOL({HANDOVER_REPORT}), &zero, sizeof(zero));\n"
                "    if (e != hipSuccess) return static_cast<int>(e);\n"
                "    return static_cast<int>(0x40000000u | (word & 0x3fffffffu));\n"
                "}\n")
        targs = "<" + ", ".join(str(int(v)) for v in template) + ">" if template else ""
        params = ", ".join(f"{t} {n}" for t, n in em.params)
        args = ", ".join(n for _, n in em.params)
        sep = ", " if params else ""
        return (
            head + helpers + text + "\n"
            f'extern "C" int {name}_launch({params}{sep}unsigned grid_blocks, void* stream) {{\n'
            "    if (grid_blocks == 0) return 0;\n"
            f"    {name}{targs}<<<dim3(grid_blocks), dim3({block_size}), {em.smem_offset}, static_cast<hipStream_t>(stream)>>>"
            f"({args});\n"
            "    return static_cast<int>(hipGetLastError());\n"
            "}\n" + status)
    if template:
        raise HipgenError("thread-level kernels take no template values")
    em = _Emitter(k, True)
    text = em.emit()
    params = ", ".join(f"{t} {n}" for t, n in em.params)
    args = ", ".join(n for _, n in em.params)
    sep = ", " if params else ""
    return (
        head + text + "\n"
        f'extern "C" int {name}_launch({params}{sep}size_t n, void* stream) {{\n'
        "    if (n == 0) return 0;\n"
        f"    const size_t blocks = (n + {block_size - 1}) / {block_size};\n"
        "    if (blocks > 0x7fffffffull) return 1;\n"
        f"    {name}<<<dim3(static_cast<unsigned>(blocks)), dim3({block_size}), 0, static_cast<hipStream_t>(stream)>>>"
        f"({args}{sep}n);\n"
        "    return static_cast<int>(hipGetLastError());\n"
        "}\n")


def build(name: str, out_dir: Optional[str] = None, block_size: int = 256,
          template: Optional[List[int]] = None, handover_spins: Optional[int] = None) -> ctypes.CDLL:
    """Compile `generate_launcher(name, block_size, template)` for gfx950 and load it. The handle's
    `<name>_launch` takes the kernel's parameters (device pointers as integers), then the element count
    (thread-level kernels) or the number of workgroups (kernels with a block perspective), then a stream."""
    from .build import HIPCC_FLAGS, hipcc_path
    d = Path(out_dir) if out_dir else Path(tempfile.mkdtemp(prefix="prism_hipgen_"))
    d.mkdir(parents=True, exist_ok=True)
    src, lib = d / f"{name}.hip", d / f"lib{name}.so"
    src.write_text(generate_launcher(name, block_size, template, handover_spins))
    proc = subprocess.run([hipcc_path(), *HIPCC_FLAGS, "-shared", "-o", str(lib), str(src)],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        hint = ""
        if "Operand has incorrect register class" in proc.stderr and "global_load_lds" in src.read_text():
            hint = ("\n(a device function that calls intrinsic.load_to_lds was probably not inlined: the compiler cannot "
                    "turn its pointer into an LDS address then; make the function smaller or call it from fewer places)")
        raise HipgenError(f"hipcc failed for {name}:\n{proc.stderr}{hint}")
    return ctypes.CDLL(str(lib))
