"""HIP emitter for Prism kernels with block- and thread-level structure (gfx950).

The second slice of the HIP back-end for the reference's front end (prism/codegen.py:321-384 prologue,
:422-530 declarations, :700-738 loops, :744-849 group/partition; surface syntax in
examples/sgemm_kernel_1.py, examples/sgemm_shared_mem_block.py, examples/sgemm_kernel_3.py,
examples/add_m_block_thread.py, examples/function_call.py). hipgen.py's first slice folds a purely
per-thread kernel into a flat body; this one keeps the reference's structure:

  * every kernel starts from `__block_id_0 = blockIdx.x` and
    `__thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x`; `with group(level[n])` opens a scope with
    the ids of the next depth (block: `__block_id_d = outer % n`, thread id rebuilt from it; thread:
    `__thread_id_d = outer % n`), and `id()` in a declaration `@ level[n]` reads the id of that level
    at the current depth (divided by n when n > 1);
  * `with partition(a, p=..., offset=e) as v` opens a scope with `T* v = a + (e);`;
  * `shared(T[n], static=True)` is a `__shared__` array, `shared(T[n])` a window of the dynamic LDS
    block `__smem` at the running offset; `T[n] @ thread[1]` is a private array;
  * `template=[("BM", int), ...]` becomes `template<int BM, ...>`, `@attr("...")` goes between
    `__global__` and the return type; `@prism("device")` functions take the caller's ids and `__smem`
    as three leading arguments, which calls to them pass along.

Barriers. The reference places `__syncthreads()` from a phase analysis per LDS array (prism/sync_analysis.py:
each array is in a READ or WRITE phase since the last barrier; a read after a write or a write after a read
conflicts, two writes do not). The plan here is that analysis at the same granularity: walking a block's
statements in program order, a barrier goes in front of the first statement that reads an LDS array written
since the last barrier (by any thread), or writes one read since then (in front of the whole loop when that
statement sits in one); a loop whose body would meet such a hazard with its own previous iteration gets a
barrier at the end of the body. What a call does to an array it is handed is read off the callee's signature
(a pointer to const is only read, :871-940), and a `ptr(shared(T))` parameter is an LDS array of its own
(:151-158); a pointer that a call returns is not followed. A barrier is never placed inside an `if` (threads
may disagree on the branch): the hazard is resolved in front of the `if`. One that lies wholly inside an `if`
gets its barrier inside when the condition is the same for every thread of the workgroup (it names nothing but
numbers, grid- or block-level parameters and variables, and the variables of loops over such ranges), as the
reference does for any branch (it walks into branches, :424-447); inside any other `if` it is an error. For programs in the shapes of the reference's
LDS-tiled SGEMMs, its kernel 5 and its scan this gives the barriers the reference prints
(generated/sgemm_shared_mem_block.cu:38,42, my_sgemm_kernel_4.cu:48,65, my_sgemm_kernel_5.cu:41,46,
scan_kernel.cu:17,19).

Thread groups (`group(thread[n])`, the reference's warps for n = 32) are index arithmetic only
(`__thread_id_d = outer % n`), so they carry over to 64-lane wavefronts unchanged as long as a group
does not share a wavefront with another: n is a power of two up to 64 (a 32-wide group is one half of a
wavefront) or a multiple of 64 (the reference's 128-thread warp groups are two wavefronts). Cross-lane traffic inside a group comes from `unsafe("...")` statements, whose text is
printed as it stands and must therefore be HIP: the counterpart of the reference's
`__shfl_up_sync(static_cast<uint32_t>(-1), val, delta)` (examples/scan.py:23-29) is
`__shfl_up(val, delta, 32)`, which shifts within each aligned group of 32 lanes. The barrier plan
does not look into unsafe() text.

`match split(level): case n: ...` hands the first n members of a level one body and the next ones
another (ids restart in every case; the reference's producer / consumer split,
examples/h100_matmul.py:203-206); `claim(...)` prints like `partition(...)`. No workgroup barrier is placed
inside a case. An LDS array that one case of `match split(thread)` writes and other cases read is handed
from case to case through two round counters in LDS (_SyncPlan._plan_handovers), the counterpart of the
mbarrier waits and arrives the reference inserts (prism/sync_analysis.py:500-570, prism/codegen.py:886-934).

Vector accesses (prism/codegen.py:239-242,544-549; examples/sgemm_kernel_4.py:53-60,78-84):
`float4_cast(a[i])` reads and `float4_cast[a[i]] = v` writes the 16 bytes at `&a[i]`
(`reinterpret_cast<float4 *>(&a[i])[0]`, one `global_load_dwordx4` / `ds_read_b128` when the address is
16-byte aligned, which is the kernel author's responsibility as in the reference); a `float4` variable's
`.x .y .z .w` read and assign like scalars. The barrier plan counts the cast as an access of the array
inside it.

`with partition(a, p=..., f=lambda i: e) as v` declares no pointer: every `v[i]` is printed as `a[e(i)]`
(prism/codegen.py:816-826,552-562), also through a chain of such views.

Matrix instructions. The reference's `intrinsic.mma(a0..a3, b0, b1, c0..c3, out=[d0..d3])` prints one
`mma.sync.aligned.m16n8k8` of inline PTX for a warp (prism/codegen.py:627-661, used by
examples/simple_mma.py and examples/mmaTF32NaiveKernel.py). The counterparts here are wavefront-wide
fp32 MFMAs, printed as compiler builtins:
`intrinsic.mfma_f32_16x16x4_f32(a, b, c0, c1, c2, c3, out=[d0, d1, d2, d3])` (lane l supplies
a = A[l % 16][l / 16] and b = B[l / 16][l % 16] of a 16 x 4 by 4 x 16 product and holds
C[4 (l / 16) + v][l % 16] in c<v>) and `intrinsic.mfma_f32_32x32x2_f32(a, b, c0..c15, out=[d0..d15])`
(a = A[l % 32][l / 32], b = B[l / 32][l % 32], c<v> = C[8 (v / 4) + 4 (l / 32) + v % 4][l % 32]). The bf16
forms, `intrinsic.mfma_f32_16x16x32_bf16(a, b, c0..c3, out=[...])` and `intrinsic.mfma_f32_32x32x16_bf16(a, b,
c0..c15, out=[...])`, take `float4` operands that carry eight consecutive bf16 of a row, the way
`float4_cast(P[i])` reads them from a `ptr(bf16)`: a = P[l % 16][8 (l / 16) .. + 7], b = Q[l % 16][same k] for
C = P Q^T (32-row form: l % 32 and 8 (l / 32)); accumulators as in the fp32 forms. All 64
lanes of the wavefront must reach the statement together. `intrinsic.load_to_lds(dst[i], src[j])` is the
asynchronous copy of this target (BlockEmitter.load_to_lds). Inline PTX itself (`intrinsic.mma`,
`intrinsic.wgmma256`) has no meaning here and is refused by name.
"""
from __future__ import annotations

import ast
from dataclasses import dataclass
from typing import Dict, List, Optional, Set, Tuple

from .hipgen import HipgenError, Kernel, _BINOPS, _CMPOPS, _REGISTRY, _UNOPS, address_space_of

_TYPES = {"int": ("int", 4), "float": ("float", 4), "double": ("double", 8), "bool": ("bool", 1),
          "uint": ("unsigned int", 4), "unsigned": ("unsigned int", 4), "uint32_t": ("uint32_t", 4),
          "uint64_t": ("uint64_t", 8), "float4": ("float4", 16), "bf16": ("__bf16", 2), "void": ("void", 0)}
_LEVELS = ("grid", "block", "thread")
# intrinsic.<name> -> (compiler builtin, accumulator registers per lane, operands are 16-byte packets of 8 bf16)
_MFMA = {"mfma_f32_16x16x4_f32": ("__builtin_amdgcn_mfma_f32_16x16x4f32", 4, False),
         "mfma_f32_32x32x2_f32": ("__builtin_amdgcn_mfma_f32_32x32x2f32", 16, False),
         "mfma_f32_16x16x32_bf16": ("__builtin_amdgcn_mfma_f32_16x16x32_bf16", 4, True),
         "mfma_f32_32x32x16_bf16": ("__builtin_amdgcn_mfma_f32_32x32x16_bf16", 16, True)}


@dataclass(frozen=True)
class _Ids:
    block_id: str
    thread_id: str
    depth: int


def _line(node: ast.AST) -> str:
    return f"line {getattr(node, 'lineno', '?')}"


def _level(node: ast.AST) -> Tuple[str, int]:
    """`block[16]` as written -> ("block", 16)."""
    if (isinstance(node, ast.Subscript) and isinstance(node.value, ast.Name) and node.value.id in _LEVELS
            and isinstance(node.slice, ast.Constant) and isinstance(node.slice.value, int)):
        return node.value.id, node.slice.value
    raise HipgenError(f"{_line(node)}: expected a perspective such as block[1]")


def _is_call(node: ast.AST, name: str) -> bool:
    return isinstance(node, ast.Call) and isinstance(node.func, ast.Name) and node.func.id == name


class _Scalar:
    """C text of a type expression as written in an annotation."""

    @staticmethod
    def text(node: ast.AST) -> str:
        if isinstance(node, ast.Name):
            if node.id in _TYPES:
                return _TYPES[node.id][0]
            raise HipgenError(f"{_line(node)}: unsupported type {node.id}")
        if isinstance(node, ast.Call) and isinstance(node.func, ast.Name) and node.args:
            inner = _Scalar.text(node.args[0])
            if node.func.id == "ptr":
                address_space_of(node)   # ptr(T, GLOBAL | SHARED | LOCAL): checked here, the same `T*` in the text
                # ptr(shared(T)) and ptr(const(shared(T))): shared() already made the pointer
                a = node.args[0]
                into_lds = _is_call(a, "shared") or (_is_call(a, "const") and a.args and _is_call(a.args[0], "shared"))
                return inner if into_lds else inner + "*"
            if node.func.id == "shared":  # ptr(shared(T)): a pointer into LDS is a plain pointer in the text
                return inner + "*"
            if node.func.id == "const":
                return "const " + inner
            if node.func.id == "restrict":
                return inner + " __restrict__"
            if node.func.id == "constexpr":
                return "constexpr " + inner
        raise HipgenError(f"{_line(node)}: unsupported type expression")


def _annotation(node: ast.AST) -> Tuple[ast.AST, Optional[Tuple[str, int]]]:
    """`T @ level[n]` -> (T, (level, n)); a bare `T` -> (T, None)."""
    if isinstance(node, ast.BinOp) and isinstance(node.op, ast.MatMult):
        return node.left, _level(node.right)
    return node, None


def _is_intrinsic(node: ast.AST, name: str) -> bool:
    return (isinstance(node, ast.Call) and isinstance(node.func, ast.Attribute) and node.func.attr == name
            and isinstance(node.func.value, ast.Name) and node.func.value.id == "intrinsic")


def _const_pointer_params(name: str) -> Set[int]:
    """Positions of the parameters of Prism function `name` that are declared `ptr(const(T))`."""
    fn = ast.parse(_REGISTRY[name].source).body[0]
    out: Set[int] = set()
    for i, a in enumerate(x for x in fn.args.args if x.arg != "template"):
        t = _annotation(a.annotation)[0] if a.annotation is not None else None
        if _is_call(t, "ptr") and t.args and _is_call(t.args[0], "const"):
            out.add(i)
    return out


# --------------------------------------------------------------- barrier plan --

def _static_load_count(stmts: List[ast.stmt], depth: int = 0) -> Optional[int]:
    """How many vector memory operations a thread issues in `stmts`, when the text alone says so: direct-to-LDS
    loads under loops over constant ranges, `with` scopes and calls of device functions of the same kind, and
    besides them only declarations and assignments of index arithmetic (no element access, no other call than
    id()). None for anything else."""
    total = 0
    for s in stmts:
        if isinstance(s, ast.Expr) and isinstance(s.value, ast.Constant):
            continue
        if isinstance(s, ast.Return) and s.value is None:
            continue
        if isinstance(s, ast.Pass):
            continue
        if isinstance(s, ast.Expr) and isinstance(s.value, ast.Call):
            call = s.value
            if _is_intrinsic(call, "load_to_lds"):
                if any(isinstance(n, ast.Call) for a in call.args for n in ast.walk(a)):
                    return None
                total += 1
                continue
            if isinstance(call.func, ast.Name) and call.func.id in _REGISTRY and depth < 8:
                inner = _static_load_count(ast.parse(_REGISTRY[call.func.id].source).body[0].body, depth + 1)
                if inner is None or any(isinstance(n, (ast.Subscript, ast.Call)) for a in call.args for n in ast.walk(a)):
                    return None
                total += inner
                continue
            return None
        if isinstance(s, (ast.AnnAssign, ast.Assign)):
            value = s.value
            if value is not None and any(isinstance(n, ast.Subscript) or (isinstance(n, ast.Call) and not _is_call(n, "id"))
                                         for n in ast.walk(value)):
                return None
            if isinstance(s, ast.Assign) and any(isinstance(n, ast.Subscript) for t in s.targets for n in ast.walk(t)):
                return None
            continue
        if isinstance(s, ast.With):
            inner = _static_load_count(s.body, depth)
            if inner is None:
                return None
            total += inner
            continue
        if isinstance(s, ast.For) and _is_call(s.iter, "range") and 1 <= len(s.iter.args) <= 3 \
                and all(isinstance(a, ast.Constant) and isinstance(a.value, int) for a in s.iter.args) and not s.orelse:
            inner = _static_load_count(s.body, depth)
            if inner is None:
                return None
            total += len(range(*[a.value for a in s.iter.args])) * inner
            continue
        return None
    return total


class _SyncPlan:
    """Which statements get a barrier in front of them / at the end of their body."""

    def __init__(self, fn: ast.FunctionDef):
        self.before: Set[int] = set()     # id(stmt)
        self.at_end: Set[int] = set()     # id(loop stmt)
        self.why: Dict[int, str] = {}     # id(stmt) -> what the barrier there is for (see explain_barriers)
        self.root: Dict[str, str] = {}    # LDS array or view of one -> the array
        # hand-over of LDS arrays between the cases of a split (see _plan_handovers)
        self.declared_here: Set[str] = set()                       # LDS arrays declared in this function's body, outside loops
        self.handed: Dict[str, Tuple[int, int]] = {}               # array -> (writing wavefronts, reading wavefronts)
        self.covered: Dict[int, Set[str]] = {}                     # id(match) -> arrays handed over inside it
        self.wait_before: Dict[int, List[Tuple[str, str]]] = {}    # id(stmt) -> [(array, "full" | "empty")]
        self.signal_after: Dict[int, List[Tuple[str, str]]] = {}
        self.filled_together: Dict[str, List[str]] = {}            # array -> the arrays its writing case fills (itself included)
        self.flush_after: Dict[int, List[str]] = {}                # id(loop or match) -> arrays whose last filling is announced behind it
        self.flush_in_case: Dict[int, Tuple[List[str], Optional[ast.stmt]]] = {}  # id(last stmt of the writing case) -> (arrays, loop)
        self.announce_before_wait: Dict[int, List[str]] = {}       # id(stmt with a wait in front) -> arrays its case announces late
        for a in fn.args.args:            # a parameter declared ptr(shared(T)) or ptr(T, SHARED) points into LDS
            if a.arg != "template" and a.annotation is not None and any(   # (prism/sync_analysis.py:151-158)
                    _is_call(n, "shared") or (_is_call(n, "ptr") and address_space_of(n) == "SHARED")
                    for n in ast.walk(_annotation(a.annotation)[0])):
                self.root[a.arg] = a.arg
        # names whose value is the same for every thread of a workgroup: parameters and variables declared at
        # grid or block perspective (the perspective rules keep thread-level values out of them), and, while the
        # walk is inside them, the variables of loops over ranges of such values
        self.uniform: Set[str] = set()
        for a in fn.args.args:
            if a.arg != "template" and a.annotation is not None:
                level = _annotation(a.annotation)[1]
                if level is not None and level[0] in ("grid", "block"):
                    self.uniform.add(a.arg)
        for n in ast.walk(fn):
            if isinstance(n, ast.AnnAssign) and isinstance(n.target, ast.Name):
                level = _annotation(n.annotation)[1]
                if level is not None and level[0] in ("grid", "block"):
                    self.uniform.add(n.target.id)
        self._collect(fn.body)
        self._plan_handovers(fn.body)
        self._walk(fn.body, (set(), set()), True)

    def _collect(self, stmts: List[ast.stmt], in_loop: bool = False) -> None:
        for s in stmts:
            if isinstance(s, ast.AnnAssign) and isinstance(s.target, ast.Name):
                t, _ = _annotation(s.annotation)
                if _is_call(t, "shared"):
                    self.root[s.target.id] = s.target.id
                    if not in_loop:   # a declaration inside a loop would start its round counters afresh in every trip
                        self.declared_here.add(s.target.id)
            elif isinstance(s, ast.With):
                call = s.items[0].context_expr
                target = s.items[0].optional_vars
                if ((_is_call(call, "partition") or _is_call(call, "claim")) and call.args
                        and isinstance(call.args[0], ast.Name) and isinstance(target, ast.Name)
                        and call.args[0].id in self.root):
                    self.root[target.id] = self.root[call.args[0].id]
            for field in ("body", "orelse"):
                self._collect(getattr(s, field, []) or [], in_loop or isinstance(s, (ast.For, ast.While)))
            if isinstance(s, ast.Match):
                for case in s.cases:
                    self._collect(case.body, in_loop)

    # read / write sets of LDS arrays
    def _reads(self, node: Optional[ast.AST]) -> Set[str]:
        out: Set[str] = set()
        if node is None:
            return out
        for n in ast.walk(node):
            if isinstance(n, ast.Name) and n.id in self.root:
                out.add(self.root[n.id])  # an element read, or the array handed to a function
        return out

    def _handed_over(self, node: Optional[ast.AST]) -> Set[str]:
        """LDS arrays named as a whole among the arguments of a call of a Prism function: the callee may write
        them, unless it declares the parameter a pointer to const (the way the reference's consumer takes its
        tiles, examples/sgemm_kernel_5.py:16-17). An element read (`f(a[i])`) passes a value and is not meant."""
        out: Set[str] = set()
        if node is None:
            return out
        for n in ast.walk(node):
            if isinstance(n, ast.Call) and isinstance(n.func, ast.Name) and n.func.id in _REGISTRY:
                read_only = _const_pointer_params(n.func.id)
                for i, a in enumerate(n.args):
                    if isinstance(a, ast.Name) and a.id in self.root and i not in read_only:
                        out.add(self.root[a.id])
        return out

    def _with_reads(self, s: ast.With) -> Set[str]:
        """A view is pointer arithmetic; only its offset expression can read memory."""
        out: Set[str] = set()
        for item in s.items:
            call = item.context_expr
            if isinstance(call, ast.Call):
                for kw in call.keywords:
                    if kw.arg == "offset":
                        out |= self._reads(kw.value)
        return out

    def _access(self, s: ast.stmt) -> Tuple[Set[str], Set[str]]:
        """(reads, writes) of a statement that holds no other statements."""
        if isinstance(s, ast.Assign):
            r, w = self._reads(s.value), self._handed_over(s.value)
            for t in s.targets:
                if (isinstance(t, ast.Subscript) and isinstance(t.value, ast.Name) and t.value.id == "float4_cast"
                        and isinstance(t.slice, ast.Subscript)):
                    t = t.slice  # float4_cast[a[i]] = v stores through a[i]
                if isinstance(t, ast.Subscript) and isinstance(t.value, ast.Name) and t.value.id in self.root:
                    w.add(self.root[t.value.id])
                    r |= self._reads(t.slice)
                else:
                    r |= self._reads(t)
            return r, w
        if isinstance(s, ast.AugAssign):
            r = self._reads(s.value) | self._reads(s.target)
            w = self._handed_over(s.value)
            if isinstance(s.target, ast.Subscript) and isinstance(s.target.value, ast.Name) and s.target.value.id in self.root:
                w.add(self.root[s.target.value.id])
            return r, w
        if isinstance(s, ast.AnnAssign):
            r = self._reads(s.value)
            return r, self._handed_over(s.value)
        if isinstance(s, ast.Expr):
            if _is_intrinsic(s.value, "load_to_lds") and len(s.value.args) == 2:
                dst, src = s.value.args   # the destination element is written, its index and the source are read
                w = {self.root[dst.value.id]} if (isinstance(dst, ast.Subscript) and isinstance(dst.value, ast.Name)
                                                  and dst.value.id in self.root) else set()
                return self._reads(src) | self._reads(getattr(dst, "slice", None)), w
            return self._reads(s.value), self._handed_over(s.value)
        if isinstance(s, ast.Return):
            return self._reads(s.value), set()
        return set(), set()

    def _whole(self, stmts: List[ast.stmt]) -> Tuple[Set[str], Set[str]]:
        r: Set[str] = set()
        w: Set[str] = set()
        for s in stmts:
            if isinstance(s, ast.With):
                r |= self._with_reads(s)
                a, b = self._whole(s.body)
            elif isinstance(s, (ast.For, ast.While)):
                r |= self._reads(s.iter if isinstance(s, ast.For) else s.test)
                a, b = self._whole(s.body)
            elif isinstance(s, ast.If):
                r |= self._reads(s.test)
                a, b = self._whole(s.body + s.orelse)
            elif isinstance(s, ast.Match):
                a, b = self._whole([x for c in s.cases for x in c.body])
            else:
                a, b = self._access(s)
            r |= a
            w |= b
        return r, w

    def _plan_handovers(self, stmts: List[ast.stmt], enclosing: Optional[ast.stmt] = None, alone: bool = False) -> None:
        """An LDS array that one case of `match split(thread)` writes and other cases read is handed from case
        to case: the writing wavefronts wait until the array is empty, fill it and signal that it is full; the
        reading wavefronts wait until it is full, read it and signal that it is empty (the reference's split
        barriers, prism/sync_analysis.py:500-570, which it lowers to mbarrier arrive / wait; here the two
        sides count rounds in two LDS words per array). In each case the wait goes in front of the first
        statement that touches the array and the signal behind the last one, in the innermost statement list
        that `with` scopes alone lead to. No workgroup
        barrier is involved, so a writer may run as many arrays ahead of the readers as there are arrays.

        A case that fills several arrays announces a filling late (BlockEmitter.announce_later): `filled_together`
        names the arrays of such a case, and `flush_after` the statement (the innermost loop around the split, or
        the split itself) behind which the last filling is announced at the latest. A filling stays unannounced
        from one trip of that loop to the next only when the split is all the loop does (`alone`: declarations
        and `with` scopes aside) and the loop ends without a workgroup barrier; otherwise the writing case
        announces it before it leaves the split (`flush_in_case`), because a barrier further down would wait for
        readers that wait for the announcement."""
        doing = [t for t in stmts if not isinstance(t, (ast.AnnAssign, ast.Pass))
                 and not (isinstance(t, ast.Expr) and isinstance(t.value, ast.Constant))]
        sole = len(doing) == 1
        for s in stmts:
            if isinstance(s, ast.Match) and _is_call(s.subject, "split") and s.subject.args \
                    and isinstance(s.subject.args[0], ast.Name) and s.subject.args[0].id == "thread":
                access = [self._whole(c.body) for c in s.cases]
                counts = [c.pattern.value.value if isinstance(c.pattern, ast.MatchValue)
                          and isinstance(c.pattern.value, ast.Constant) else 0 for c in s.cases]
                wait_sites: Dict[int, List[int]] = {}   # case -> id(stmt) of every statement of it with a wait in front
                for array in sorted(set().union(*(r | w for r, w in access))):
                    writers = [i for i, (_, w) in enumerate(access) if array in w]
                    readers = [i for i, (r, w) in enumerate(access) if array in r and array not in w]
                    if len(writers) > 1 and any(array in r for r, _ in access):
                        raise HipgenError(f"{_line(s)}: {array} is written by more than one case of the split and read "
                                          "in it: a hand-over has one writing case")
                    if not writers or not readers:
                        continue
                    if array in self.handed:
                        raise HipgenError(f"{_line(s)}: {array} is already handed over in another split")
                    if array not in self.declared_here:
                        raise HipgenError(f"{_line(s)}: {array} is handed from case to case; it must be declared in this function, "
                                          "outside any loop: its round counters live beside its declaration")
                    involved = writers + readers
                    if any(counts[i] <= 0 or counts[i] % 64 for i in involved):
                        raise HipgenError(f"{_line(s)}: {array} is handed from case to case; those cases must be whole "
                                          "wavefronts (multiples of 64 threads)")
                    self.handed[array] = (counts[writers[0]] // 64, sum(counts[i] for i in readers) // 64)
                    self.covered.setdefault(id(s), set()).add(array)
                    for i in involved:
                        body = s.cases[i].body
                        while True:   # through `with` scopes (every thread of the case runs them), not into loops or branches
                            touching = [t for t in body if array in set().union(*self._whole([t]))]
                            if len(touching) == 1 and isinstance(touching[0], ast.With):
                                body = touching[0].body
                            else:
                                break
                        wait, signal = ("empty", "full") if i in writers else ("full", "empty")
                        self.wait_before.setdefault(id(touching[0]), []).append((array, wait))
                        self.signal_after.setdefault(id(touching[-1]), []).append((array, signal))
                        wait_sites.setdefault(i, []).append(id(touching[0]))
                by_case: Dict[int, List[str]] = {}
                for array in self.covered.get(id(s), ()):
                    by_case.setdefault(next(i for i, (_, w) in enumerate(access) if array in w), []).append(array)
                for i, arrays in by_case.items():
                    if len(arrays) > 1:
                        for array in arrays:
                            self.filled_together[array] = sorted(arrays)
                        self.flush_after.setdefault(id(enclosing if enclosing is not None else s), []).extend(sorted(arrays))
                        carried = enclosing if alone and sole else None
                        self.flush_in_case[id(s.cases[i].body[-1])] = (sorted(arrays), carried)
                        for site in wait_sites.get(i, []):   # whatever this case waits for, filled arrays or others
                            self.announce_before_wait[site] = sorted(arrays)
            if isinstance(s, (ast.For, ast.While)):
                self._plan_handovers(s.body, s, True)
                self._plan_handovers(getattr(s, "orelse", []) or [], enclosing, False)
            elif isinstance(s, ast.With):
                self._plan_handovers(s.body, enclosing, alone and sole)
            elif isinstance(s, ast.Match):
                for case in s.cases:
                    self._plan_handovers(case.body, enclosing, False)
            else:
                for field in ("body", "orelse"):
                    self._plan_handovers(getattr(s, field, []) or [], enclosing, False)

    def _block_uniform(self, node: Optional[ast.AST]) -> bool:
        """True when the expression is built from numbers, names in self.uniform, arithmetic and comparisons
        only: no call (id() differs from thread to thread), no memory access."""
        if node is None:
            return True
        for n in ast.walk(node):
            if isinstance(n, ast.Name):
                if n.id not in self.uniform:
                    return False
            elif isinstance(n, ast.Constant):
                if not isinstance(n.value, (int, float, bool)):
                    return False
            elif not isinstance(n, (ast.BinOp, ast.UnaryOp, ast.BoolOp, ast.Compare, ast.operator, ast.unaryop,
                                    ast.boolop, ast.cmpop, ast.expr_context)):
                return False
        return True

    @staticmethod
    def _hazard(r: Set[str], w: Set[str], pending: Tuple[Set[str], Set[str]]) -> bool:
        pr, pw = pending
        return bool((r & pw) or (w & pr))

    def _walk(self, stmts: List[ast.stmt], pending: Tuple[Set[str], Set[str]], may_sync: bool) -> Tuple[Set[str], Set[str]]:
        """Plans barriers for `stmts` entered with `pending` = (reads, writes) since the last barrier;
        returns the same pair at the end."""
        pr, pw = set(pending[0]), set(pending[1])
        for s in stmts:
            if isinstance(s, ast.With):
                r = self._with_reads(s)
                if self._hazard(r, set(), (pr, pw)):
                    self._mark(s, may_sync, self._reason(r, set(), (pr, pw)))
                    pr, pw = set(), set()
                pr |= r
                pr, pw = self._walk(s.body, (pr, pw), may_sync)
            elif isinstance(s, (ast.For, ast.While)):
                # A hazard between what is pending and anything in the loop is resolved once, in front
                # of the loop, not in every iteration.
                r, w = self._whole([s])
                if self._hazard(r, w, (pr, pw)):
                    self._mark(s, may_sync, self._reason(r, w, (pr, pw)))
                    pr, pw = set(), set()
                pr |= self._reads(s.iter if isinstance(s, ast.For) else s.test)
                before_loop = (set(pr), set(pw))
                # the variable of a loop over a range of workgroup-uniform values is uniform inside the loop
                loop_var = (s.target.id if isinstance(s, ast.For) and isinstance(s.target, ast.Name) and may_sync
                            and s.target.id not in self.uniform and _is_call(s.iter, "range")
                            and all(self._block_uniform(a) for a in s.iter.args) else None)
                if loop_var is not None:
                    self.uniform.add(loop_var)
                pr, pw = self._walk(s.body, (pr, pw), may_sync)
                if loop_var is not None:
                    self.uniform.discard(loop_var)
                if self._probe(s.body, (pr, pw)) == "hazard":
                    if not may_sync:
                        raise HipgenError(f"{_line(s)}: a loop inside an `if` needs a barrier between its iterations")
                    self.at_end.add(id(s))
                    self.why[id(s)] = "the next trip of the loop " + self._reason(*self._whole(s.body), (pr, pw))
                    pr, pw = set(), set()
                if not self._runs_at_least_once(s):
                    # With zero trips none of the body's barriers is executed: what was pending in front
                    # of the loop is still pending behind it.
                    pr |= before_loop[0]
                    pw |= before_loop[1]
            elif isinstance(s, (ast.If, ast.Match)):
                r, w = self._whole([s])
                if self._hazard(r, w, (pr, pw)):
                    self._mark(s, may_sync, self._reason(r, w, (pr, pw)))
                    pr, pw = set(), set()
                # Inside the cases of a split, and inside an `if` on which the threads of a workgroup may
                # disagree, no barrier may be placed: not every thread gets there, and a hazard inside is an
                # error. An `if` whose condition is the same for the whole workgroup is entered by all of its
                # threads or by none, so a hazard that lies wholly inside gets its barrier inside.
                bodies = [s.body, s.orelse] if isinstance(s, ast.If) else [c.body for c in s.cases]
                inside = may_sync and isinstance(s, ast.If) and self._block_uniform(s.test)
                for body in bodies:
                    a = self._walk(body, (set(), set()), inside)
                    pr |= a[0]
                    pw |= a[1]
                pr |= r
                pw |= w
            else:
                r, w = self._access(s)
                if self._hazard(r, w, (pr, pw)):
                    self._mark(s, may_sync, self._reason(r, w, (pr, pw)))
                    pr, pw = set(), set()
                pr |= r
                pw |= w
        return pr, pw

    @staticmethod
    def _runs_at_least_once(s: ast.stmt) -> bool:
        """True only for `for ... in range(...)` whose bounds are integer literals with at least one trip."""
        if not (isinstance(s, ast.For) and _is_call(s.iter, "range") and not s.iter.keywords):
            return False
        args = s.iter.args
        if not (1 <= len(args) <= 3) or not all(isinstance(a, ast.Constant) and isinstance(a.value, int)
                                                and not isinstance(a.value, bool) for a in args):
            return False
        try:
            return len(range(*(a.value for a in args))) >= 1
        except ValueError:
            return False

    @staticmethod
    def _reason(r: Set[str], w: Set[str], pending: Tuple[Set[str], Set[str]]) -> str:
        pr, pw = pending
        parts = []
        if r & pw:
            parts.append("reads " + ", ".join(sorted(r & pw)) + " (written since the last barrier)")
        if w & pr:
            parts.append("writes " + ", ".join(sorted(w & pr)) + " (read since the last barrier)")
        return " and ".join(parts)

    def _mark(self, s: ast.stmt, may_sync: bool, why: str = "") -> None:
        if not may_sync:
            raise HipgenError(f"{_line(s)}: LDS is written and read inside one `if`; the barrier between "
                              "them cannot be placed in divergent code")
        self.before.add(id(s))
        self.why[id(s)] = why

    def _probe(self, stmts: List[ast.stmt], pending: Tuple[Set[str], Set[str]]) -> str:
        """Runs the next iteration's statements against what the previous one left pending:
        "hazard" if one is met before the first planned barrier, "barrier" if a barrier comes first,
        "none" if the body ends without either."""
        for s in stmts:
            if id(s) in self.before:
                return "barrier"
            if isinstance(s, ast.With):
                if self._hazard(self._with_reads(s), set(), pending):
                    return "hazard"
                got = self._probe(s.body, pending)
            elif isinstance(s, (ast.For, ast.While)):
                r, w = self._whole([s])
                # the barrier at the end of an inner loop's body only counts if that loop is sure to run
                got = "hazard" if self._hazard(r, w, pending) else (
                    "barrier" if id(s) in self.at_end and self._runs_at_least_once(s) else "none")
            elif isinstance(s, (ast.If, ast.Match)):
                r, w = self._whole([s])
                flagged = self.covered.get(id(s), set())  # ordered from round to round by their full / empty words
                got = "hazard" if self._hazard(r - flagged, w - flagged, pending) else "none"
            else:
                r, w = self._access(s)
                got = "hazard" if self._hazard(r, w, pending) else "none"
            if got != "none":
                return got
        return "none"


# -------------------------------------------------------------------- emitter --

HANDOVER_REPORT = "__prism_handover_report"   # file-scope device word a hand-over wait that gives up writes
HANDOVER_REPORT_DEFINITION = (
    "#ifndef PRISM_HANDOVER_REPORT\n#define PRISM_HANDOVER_REPORT\n"
    "// written by a hand-over wait that ran out of polls: 1 + 2 * (array number) + (1 when waiting for a filled\n"
    "// array) in the low byte, the round above it; the launcher's <name>_status call reads and clears it\n"
    f"__device__ unsigned int {HANDOVER_REPORT} = 0;\n#endif\n")
# A wavefront with direct-to-LDS loads in flight touches its hand-over words through these: in front of every LDS
# access it can see, the compiler waits for all such loads (it does not know which part of LDS they write), and
# a wavefront that announces fillings late (BlockEmitter.announce_later) lives on having loads in flight.
LATE_ANNOUNCEMENT_HELPERS = (
    "#ifndef PRISM_LDS_WORD_HELPERS\n#define PRISM_LDS_WORD_HELPERS\n"
    "// one LDS word read / counted up without the compiler seeing an LDS access (the address is the low half of the\n"
    "// generic one); the memory clobber keeps every memory operation on its side of the call\n"
    "__device__ __forceinline__ unsigned int __prism_lds_peek(const unsigned int* word) {\n"
    "    unsigned int value;\n"
    "    asm volatile(\"ds_read_b32 %0, %1\\n\\ts_waitcnt lgkmcnt(0)\" : \"=v\"(value) : \"v\"((unsigned int)(unsigned long long)word) : \"memory\");\n"
    "    return value;\n"
    "}\n"
    "__device__ __forceinline__ void __prism_lds_count(unsigned int* word) {\n"
    "    asm volatile(\"ds_add_u32 %0, %1\" :: \"v\"((unsigned int)(unsigned long long)word), \"v\"(1u) : \"memory\");\n"
    "}\n#endif\n")


class BlockEmitter:
    def __init__(self, kernel: Kernel, auto_sync: bool = True, annotate: bool = False,
                 handover_spins: Optional[int] = None):
        self.k = kernel
        if handover_spins is not None:
            if not 0 <= handover_spins <= 1 << 30:
                raise HipgenError("handover_spins must lie between 0 and 2^30")
            self.HANDOVER_SPINS = handover_spins  # 0: every wait gives up at once (a way to exercise the give-up path)
        self.annotate = annotate          # a comment in front of every barrier says what it is for
        self.auto_sync = auto_sync
        self.out: List[str] = []
        self.indent = 0
        self.ids = _Ids("__block_id_0", "__thread_id_0", 0)
        self.pointer_type: Dict[str, str] = {}   # name -> C pointer type text (parameters, views, arrays)
        self.smem_offset = 0                     # bytes of __smem handed out so far
        self.template: List[Tuple[str, str]] = []
        self.params: List[Tuple[str, str]] = []
        self.id_level: Optional[Tuple[str, int]] = None  # perspective `id()` resolves against
        self.returns_value = False
        self.plan: Optional[_SyncPlan] = None
        # f=lambda view -> (array it indexes, the lambda, the level p= names: what id() means inside the lambda)
        self.views: Dict[str, Tuple[str, ast.Lambda, Optional[Tuple[str, int]]]] = {}
        self.bound: Dict[str, str] = {}                     # lambda parameter -> text of the index in hand

    # -- text helpers
    def emit(self, text: str) -> None:
        self.out.append("    " * self.indent + text)

    def open(self) -> None:
        self.emit("{")
        self.indent += 1

    def close(self) -> None:
        self.indent -= 1
        self.emit("}")

    # -- expressions (every binary operation parenthesised, like the reference prints them)
    def expr(self, n: ast.AST) -> str:
        if isinstance(n, ast.Constant):
            if isinstance(n.value, bool):
                return "true" if n.value else "false"
            if isinstance(n.value, (int, float)):
                return str(n.value)
            raise HipgenError(f"{_line(n)}: unsupported constant {n.value!r}")
        if isinstance(n, ast.Name):
            if n.id in self.views:
                raise HipgenError(f"{_line(n)}: {n.id} is an index-mapped view; only its elements can be named")
            return self.bound.get(n.id, n.id)
        if isinstance(n, ast.BinOp) and type(n.op) in _BINOPS:
            return f"({self.expr(n.left)} {_BINOPS[type(n.op)]} {self.expr(n.right)})"
        if isinstance(n, ast.UnaryOp) and type(n.op) in _UNOPS:
            return f"({_UNOPS[type(n.op)]}{self.expr(n.operand)})"
        if isinstance(n, ast.Compare) and all(type(o) in _CMPOPS for o in n.ops):
            text = self.expr(n.left)
            for op, right in zip(n.ops, n.comparators):
                text = f"({text} {_CMPOPS[type(op)]} {self.expr(right)})"
            return text
        if isinstance(n, ast.BoolOp):
            joiner = " && " if isinstance(n.op, ast.And) else " || "
            return "(" + joiner.join(self.expr(v) for v in n.values) + ")"
        if isinstance(n, ast.IfExp):
            return f"({self.expr(n.test)} ? {self.expr(n.body)} : {self.expr(n.orelse)})"
        if isinstance(n, ast.Subscript):
            if isinstance(n.value, ast.Name) and n.value.id in self.views:
                return self.view_element(n.value.id, self.expr(n.slice))
            return f"{self.expr(n.value)}[{self.expr(n.slice)}]"
        if isinstance(n, ast.Attribute):
            return f"{self.expr(n.value)}.{n.attr}"
        if isinstance(n, ast.Call):
            return self.call(n)
        raise HipgenError(f"{_line(n)}: unsupported expression {type(n).__name__}")

    def view_element(self, view: str, index: str) -> str:
        """`view[index]` for a view declared with f=lambda: the element of the underlying array."""
        parent, fn, level = self.views[view]
        param = fn.args.args[0].arg
        saved = self.bound.get(param)
        self.bound[param] = index
        saved_level, self.id_level = self.id_level, (level or self.id_level)
        mapped = self.expr(fn.body)
        self.id_level = saved_level
        if saved is None:
            del self.bound[param]
        else:
            self.bound[param] = saved
        return self.view_element(parent, mapped) if parent in self.views else f"{parent}[{mapped}]"

    def level_id(self, level: str, size: int) -> str:
        if level == "grid":
            return "0"
        base = self.ids.block_id if level == "block" else self.ids.thread_id
        return base if size == 1 else f"({base} / {size})"

    def call(self, n: ast.Call) -> str:
        if not isinstance(n.func, ast.Name):
            raise HipgenError(f"{_line(n)}: unsupported call (intrinsic.<name>(...) is a statement; method calls are "
                              "not part of this slice)")
        name = n.func.id
        if name == "id":
            if n.args:
                return self.level_id(*_level(n.args[0]))
            if self.id_level is None:
                raise HipgenError(f"{_line(n)}: id() needs a perspective: use it in a declaration `x: T @ level[n] = ...`")
            return self.level_id(*self.id_level)
        if name == "unsafe":
            raise HipgenError(f"{_line(n)}: unsafe() is a statement")
        if name == "float4_cast":
            if len(n.args) != 1 or n.keywords or not isinstance(n.args[0], ast.Subscript):
                raise HipgenError(f"{_line(n)}: float4_cast() takes one array element")
            # Reading through a pointer to const needs the const in the cast (the reference prints the
            # plain form, which only compiles for non-const arrays; its examples declare theirs that way).
            base = n.args[0].value
            while isinstance(base, ast.Name) and base.id in self.views:
                base = ast.Name(id=self.views[base.id][0])
            const = isinstance(base, ast.Name) and self.pointer_type.get(base.id, "").startswith("const ")
            return f"reinterpret_cast<{'const ' if const else ''}float4 *>(&{self.expr(n.args[0])})[0]"

        targs = ""
        for kw in n.keywords:
            if kw.arg == "template" and isinstance(kw.value, ast.List):
                targs = "<" + ", ".join(self.expr(e) for e in kw.value.elts) + ">"
            else:
                raise HipgenError(f"{_line(n)}: unsupported keyword argument {kw.arg}")
        args = [self.expr(a) for a in n.args]
        if name in _REGISTRY and _REGISTRY[name].kind == "device":
            args = [self.ids.block_id, self.ids.thread_id, "__smem"] + args
        return f"{name}{targs}({', '.join(args)})"

    # -- statements
    def block(self, stmts: List[ast.stmt]) -> None:
        for s in stmts:
            if self.plan is not None and id(s) in self.plan.before:
                if self.annotate:
                    self.emit(f"// {_line(s)} {self.plan.why.get(id(s), '')}")
                self.emit("__syncthreads();")
            for array, what in (self.plan.wait_before.get(id(s), []) if self.plan is not None else []):
                self.wait_for(array, what, self.plan.announce_before_wait.get(id(s)))
            self.stmt(s)
            signals = self.plan.signal_after.get(id(s), []) if self.plan is not None else []
            late = [array for array, what in signals if what == "full" and array in self.plan.filled_together]
            if late:
                self.announce_later(late, s)
            for array, what in signals:
                if array not in late:
                    self.signal(array, what)
            if self.plan is not None and id(s) in self.plan.flush_in_case:
                arrays, loop = self.plan.flush_in_case[id(s)]
                if loop is None or id(loop) in self.plan.at_end:   # nothing stays unannounced beyond this case
                    for array in arrays:
                        self.announce_pending(array, None)
            for array in (self.plan.flush_after.get(id(s), []) if self.plan is not None else []):
                self.announce_pending(array, None)

    def stmt(self, s: ast.stmt) -> None:
        if isinstance(s, ast.AnnAssign) and isinstance(s.target, ast.Name):
            return self.declare(s)
        if isinstance(s, ast.With) and len(s.items) == 1 and isinstance(s.items[0].context_expr, ast.Call):
            call = s.items[0].context_expr
            if _is_call(call, "group"):
                return self.group(s, call)
            if _is_call(call, "partition") or _is_call(call, "claim"):  # both are pointer arithmetic in the text
                return self.partition(s, call, s.items[0].optional_vars)
            raise HipgenError(f"{_line(s)}: `with {getattr(call.func, 'id', '?')}(...)` is not part of this slice")
        if isinstance(s, ast.Assign) and len(s.targets) == 1:
            t = s.targets[0]
            if isinstance(t, ast.Subscript) and isinstance(t.value, ast.Name) and t.value.id == "float4_cast":
                if not isinstance(t.slice, ast.Subscript):
                    raise HipgenError(f"{_line(s)}: float4_cast[...] takes one array element")
                return self.emit(f"reinterpret_cast<float4 *>(&{self.expr(t.slice)})[0] = {self.expr(s.value)};")
            return self.emit(f"{self.expr(t)} = {self.expr(s.value)};")
        if isinstance(s, ast.AugAssign) and type(s.op) in _BINOPS:
            return self.emit(f"{self.expr(s.target)} {_BINOPS[type(s.op)]}= {self.expr(s.value)};")
        if isinstance(s, ast.For):
            return self.loop(s)
        if isinstance(s, ast.While):
            self.emit(f"while ({self.expr(s.test)}) {{")
            return self.body_and_close(s)
        if isinstance(s, ast.If):
            return self.branch(s)
        if isinstance(s, ast.Match):
            return self.split(s)
        if isinstance(s, ast.Return):
            if s.value is None:
                # A value-returning function whose value comes from unsafe() text ends in a bare `return`
                # in the source; printing it would not compile.
                return None if self.returns_value else self.emit("return;")
            return self.emit(f"return {self.expr(s.value)};")
        if isinstance(s, ast.Break):
            return self.emit("break;")
        if isinstance(s, ast.Continue):
            return self.emit("continue;")
        if isinstance(s, ast.Pass):
            return None
        if isinstance(s, ast.Expr):
            if isinstance(s.value, ast.Constant) and isinstance(s.value.value, str):
                return None  # docstring
            if (isinstance(s.value, ast.Call) and isinstance(s.value.func, ast.Attribute)
                    and isinstance(s.value.func.value, ast.Name) and s.value.func.value.id == "intrinsic"):
                return self.matrix_instruction(s.value)
            if _is_call(s.value, "unsafe"):
                # Target text, printed as it stands (HIP here, where the reference's examples hold CUDA).
                a = s.value.args
                if len(a) != 1 or not (isinstance(a[0], ast.Constant) and isinstance(a[0].value, str)):
                    raise HipgenError(f"{_line(s)}: unsafe() takes one string")
                for text in a[0].value.strip().splitlines():
                    self.emit(text.rstrip())
                return None
            return self.emit(f"{self.expr(s.value)};")
        raise HipgenError(f"{_line(s)}: unsupported statement {type(s).__name__}")

    # -- hand-over of an LDS array between the cases of a split: two words per array count the rounds
    HANDOVER_SPINS = 1 << 16   # a wait gives up after this many polls (milliseconds; a real wait takes microseconds), so that a broken protocol cannot hang the GPU

    def wait_for(self, array: str, what: str, unannounced: Optional[List[str]] = None) -> None:
        """A bounded wait. A wavefront that runs out of polls goes on (the kernel always exits) but says so: it
        stores a non-zero code into the file-scope word HANDOVER_REPORT, which the launcher's `<name>_status`
        call turns into an error, because what such a wavefront goes on to read or overwrite is not what the
        program meant. unannounced: the arrays this wavefront's case fills and announces late; whatever of them
        is still unannounced is announced before the wavefront blocks, in any wait, because the other side may
        need it before it lets this wait go."""
        writers, readers = self.plan.handed[array]
        need = f"(__round_{array} + 1) * {writers}" if what == "full" else f"__round_{array} * {readers}"
        code = 1 + 2 * list(self.plan.handed).index(array) + (1 if what == "full" else 0)
        self.uses_handover_report = True
        # The loop is written as a scalar loop that stays a loop: every lane reads the same LDS word and compares
        # it with the same count, and said so (readfirstlane) the compiler branches on scalar registers. Left to
        # itself it treats the exit as per-lane, unrolls eight polls and threads the live poll counter through
        # every exit with execution-mask bookkeeping: measured 12 % of a producer / consumer GEMM's time.
        late = unannounced is not None   # a wavefront that may have direct-to-LDS loads in flight
        word = f"&__{what}_{array}"
        peek = (f"__prism_lds_peek({word})" if late else
                f"static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load({word}, "
                "__ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP))))")
        if late:
            peek = f"static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>({peek})))"
        self.open()
        self.emit("int __spin = 0;")
        self.emit(f"const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>({need})));")
        if late:
            # About to block: whatever this wavefront has filled and not announced yet is announced first, see
            # announce_later.
            self.emit(f"if ({peek} < __need) {{")
            self.indent += 1
            for other in unannounced:
                self.announce_pending(other, None)
            self.indent -= 1
            self.emit("}")
        self.emit("#pragma nounroll")
        self.emit(f"for (; __spin < {self.HANDOVER_SPINS} && {peek} < __need; ++__spin) __builtin_amdgcn_s_sleep(1);")
        self.emit(f"if (__spin == {self.HANDOVER_SPINS} && (threadIdx.x & 63) == 0) __hip_atomic_store(&{HANDOVER_REPORT}, "
                  f"{code}u | (static_cast<unsigned int>(__round_{array}) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        self.close()
        if not late:   # (the peek's memory clobber orders the late form: what follows is issued behind it)
            self.emit('__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");')

    def signal(self, array: str, what: str) -> None:
        # every memory operation of the wavefront is complete (direct-to-LDS loads count as vector memory
        # operations), then one lane counts the wavefront in
        self.emit("__builtin_amdgcn_s_waitcnt(0);")
        self.emit('__builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");')
        self.emit(f"if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__{what}_{array}, 1u, __ATOMIC_RELAXED, "
                  "__HIP_MEMORY_SCOPE_WORKGROUP);")
        self.emit(f"__round_{array} += 1;")

    def announce_later(self, arrays: List[str], filling: ast.stmt) -> None:
        """Behind a statement that fills `arrays`, in a case that fills several arrays: the filling is counted
        (its round) but announced ("full") only when the wavefront has issued the loads of the NEXT filling,
        or is about to block in a wait, or leaves the loop, whichever comes first. The announcement needs the
        filling's loads to have landed; made right away, as signal() does, it keeps a wavefront from having
        more than one filling's loads in flight, and a filling then costs the whole memory latency. Behind the
        next filling it waits only until at most that filling's loads are outstanding (a wavefront's loads
        complete in order, so everything older has landed then), when their number is known from the program
        text."""
        for array in arrays:
            self.emit(f"__round_{array} += 1;")
        n = _static_load_count([filling])
        for other in self.plan.filled_together[arrays[0]]:
            if other not in arrays:   # filled by an earlier statement
                self.announce_pending(other, n)
        for array in arrays:
            self.emit(f"__pending_{array} = true;")

    def announce_pending(self, array: str, may_fly: Optional[int]) -> None:
        """Announces the last filling of `array` if that is still to do. may_fly: how many of the wavefront's
        latest vector memory operations may still be in flight (None: none)."""
        if may_fly is None or not 0 < may_fly < 64:
            wait = "__builtin_amdgcn_s_waitcnt(0);"
        else:  # s_waitcnt immediate of gfx9: vmcnt in bits 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at "no wait"
            wait = f"__builtin_amdgcn_s_waitcnt({(may_fly & 15) | ((may_fly >> 4) << 14) | (7 << 4) | (15 << 8)});  // vmcnt({may_fly})"
        self.uses_late_announcements = True
        self.emit(f"if (__pending_{array}) {{")
        self.indent += 1
        self.emit(wait)   # the filling has landed in LDS; the count below is issued behind it
        self.emit(f"if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_{array});")
        self.emit(f"__pending_{array} = false;")
        self.indent -= 1
        self.emit("}")

    def load_to_lds(self, n: ast.Call) -> None:
        """`intrinsic.load_to_lds(dst[i], src[j])`: the wavefront copies 64 x 16 bytes from global memory into LDS
        without staging registers: lane l's 16 bytes at &src[j] (j is the lane's own) land at &dst[i] + 16 l
        (i is the same for the whole wavefront). The counterpart of the reference's asynchronous tile load
        (load_tma, examples/h100_helpers.py); completion is what the hand-over's signal waits for."""
        if len(n.args) != 2 or n.keywords or not all(isinstance(a, ast.Subscript) for a in n.args):
            raise HipgenError(f"{_line(n)}: intrinsic.load_to_lds(dst[i], src[j])")
        dst, src = self.expr(n.args[0]), self.expr(n.args[1])
        # The LDS address comes from a pointer conversion, which the compiler folds into the array's LDS offset once
        # the device function is inlined (taking the low half of the generic address instead keeps the 64-bit
        # address arithmetic alive: measured 8 % of a GEMM whose wavefronts all load). A device function that is
        # NOT inlined keeps the conversion's null check, and this compiler then fails in its back end ("Operand
        # has incorrect register class"); build() says so when it sees that message.
        self.emit(f"__builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&{src}), "
                  f"(__attribute__((address_space(3))) void*)(&{dst}), 16, 0, 0);")

    # kinds of instructions a scheduling group may name -> mask bits of __builtin_amdgcn_sched_group_barrier
    _SCHED_KINDS = {"mfma": 0x008, "valu": 0x002, "salu": 0x004, "vmem": 0x010, "vmem_read": 0x020, "vmem_write": 0x040,
                    "lds": 0x080, "lds_read": 0x100, "lds_write": 0x200, "any": 0x000}

    def sched_group(self, n: ast.Call) -> None:
        """`intrinsic.sched_group("lds_read", 4)`: the next scheduling group holds 4 LDS reads. A run of such
        statements behind a stretch of straight-line code states the order in which the compiler's scheduler is
        to interleave that stretch's instructions (LDS reads, matrix instructions, loads), which is what the
        hand-written kernels' pipelines rest on; `intrinsic.sched_group("barrier")` keeps the scheduler from
        moving anything across the statement. Prints __builtin_amdgcn_sched_group_barrier / sched_barrier; the
        reference has no counterpart (its tensor-core path issues whole tiles per instruction)."""
        a = n.args
        if len(a) == 1 and isinstance(a[0], ast.Constant) and a[0].value == "barrier" and not n.keywords:
            return self.emit("__builtin_amdgcn_sched_barrier(0);")
        if (len(a) not in (2, 3) or n.keywords or not all(isinstance(x, ast.Constant) for x in a)
                or a[0].value not in self._SCHED_KINDS or not isinstance(a[1].value, int) or a[1].value < 1
                or (len(a) == 3 and not isinstance(a[2].value, int))):
            raise HipgenError(f"{_line(n)}: intrinsic.sched_group(kind, count[, id]) with kind one of "
                              f"{', '.join(sorted(self._SCHED_KINDS))}, or intrinsic.sched_group(\"barrier\")")
        self.emit(f"__builtin_amdgcn_sched_group_barrier({self._SCHED_KINDS[a[0].value]:#05x}, {a[1].value}, "
                  f"{a[2].value if len(a) == 3 else 0});")

    def matrix_instruction(self, n: ast.Call) -> None:
        name = n.func.attr
        if name == "load_to_lds":
            return self.load_to_lds(n)
        if name == "sched_group":
            return self.sched_group(n)
        if name not in _MFMA:
            raise HipgenError(f"{_line(n)}: intrinsic.{name} is not an instruction of this target "
                              f"(available: {', '.join(sorted(_MFMA))})")
        builtin, regs, packets = _MFMA[name]
        out = [kw.value for kw in n.keywords if kw.arg == "out"]
        if (len(n.args) != 2 + regs or len(n.keywords) != 1 or len(out) != 1 or not isinstance(out[0], ast.List)
                or len(out[0].elts) != regs):
            raise HipgenError(f"{_line(n)}: intrinsic.{name}(a, b, c0..c{regs - 1}, out=[d0..d{regs - 1}])")
        a, b = self.expr(n.args[0]), self.expr(n.args[1])
        acc = ", ".join(self.expr(c) for c in n.args[2:])
        self.open()
        self.emit(f"typedef float __acc_t __attribute__((ext_vector_type({regs})));")
        self.emit(f"__acc_t __acc = {{{acc}}};")
        if packets:  # a float4 carries eight consecutive bf16 of a row, as float4_cast reads them
            self.emit("typedef __bf16 __packet_t __attribute__((ext_vector_type(8)));")
            a, b = f"__builtin_bit_cast(__packet_t, {a})", f"__builtin_bit_cast(__packet_t, {b})"
        self.emit(f"__acc = {builtin}({a}, {b}, __acc, 0, 0, 0);")
        for v, d in enumerate(out[0].elts):
            self.emit(f"{self.expr(d)} = __acc[{v}];")
        self.close()

    def body_and_close(self, s) -> None:
        self.indent += 1
        self.block(s.body)
        if self.plan is not None and id(s) in self.plan.at_end:
            if self.annotate:
                self.emit(f"// {self.plan.why.get(id(s), '')}")
            self.emit("__syncthreads();")
        self.indent -= 1
        self.emit("}")

    def loop(self, s: ast.For) -> None:
        if not (isinstance(s.target, ast.Name) and _is_call(s.iter, "range") and 1 <= len(s.iter.args) <= 3):
            raise HipgenError(f"{_line(s)}: loops are `for i in range(...)`")
        a = [self.expr(x) for x in s.iter.args]
        start, stop, step = ("0", a[0], "1") if len(a) == 1 else (a[0], a[1], "1") if len(a) == 2 else a
        i = s.target.id
        bump = f"{i}++" if step == "1" else f"{i} += {step}"
        self.emit(f"for (int {i} = {start}; {i} < {stop}; {bump}) {{")
        self.body_and_close(s)

    def branch(self, s: ast.If) -> None:
        self.emit(f"if ({self.expr(s.test)}) {{")
        self.indent += 1
        self.block(s.body)
        self.indent -= 1
        rest = s.orelse
        while rest:
            if len(rest) == 1 and isinstance(rest[0], ast.If):
                self.emit(f"}} else if ({self.expr(rest[0].test)}) {{")
                self.indent += 1
                self.block(rest[0].body)
                self.indent -= 1
                rest = rest[0].orelse
            else:
                self.emit("} else {")
                self.indent += 1
                self.block(rest)
                self.indent -= 1
                rest = []
        self.emit("}")

    def split(self, s: ast.Match) -> None:
        """`match split(level): case n: ... case m: ...` gives the first n members of the level one body, the
        next m another, ...; inside a case ids restart at 0 (prism/codegen.py:936-993)."""
        if not (_is_call(s.subject, "split") and len(s.subject.args) == 1 and isinstance(s.subject.args[0], ast.Name)
                and s.subject.args[0].id in _LEVELS):
            raise HipgenError(f"{_line(s)}: expected `match split(block)` or `match split(thread)`")
        level = s.subject.args[0].id
        outer, before = self.ids, 0
        for case in s.cases:
            pat = case.pattern
            if not (isinstance(pat, ast.MatchValue) and isinstance(pat.value, ast.Constant)
                    and isinstance(pat.value.value, int) and pat.value.value > 0) or case.guard is not None:
                raise HipgenError(f"{_line(case.pattern)}: a case of split() is a positive member count")
            count = pat.value.value
            inner = _Ids(f"__block_id_{outer.depth + 1}", f"__thread_id_{outer.depth + 1}", outer.depth + 1)
            shift = f" - {before}" if before else ""
            self.open()
            if level == "block":
                self.emit(f"int {inner.block_id} = {outer.block_id}{shift};")
                self.emit(f"int {inner.thread_id} = {inner.block_id} * blockDim.x + threadIdx.x;")
                self.emit(f"if ({inner.block_id} >= 0 && {inner.block_id} < {count}) {{")
            elif level == "thread":
                self.emit(f"int {inner.block_id} = {outer.block_id};")
                self.emit(f"int {inner.thread_id} = {outer.thread_id}{shift};")
                self.emit(f"if ({inner.thread_id} >= 0 && {inner.thread_id} < {count}) {{")
            else:
                self.emit(f"int {inner.block_id} = {outer.block_id};")
                self.emit(f"int {inner.thread_id} = {outer.thread_id};")
                self.emit("if (true) {")
            self.indent += 1
            saved_level, self.id_level = self.id_level, (level, 1)
            self.ids = inner
            self.block(case.body)
            self.ids = outer
            self.id_level = saved_level
            self.indent -= 1
            self.emit("}")
            self.close()
            before += count

    def declare(self, s: ast.AnnAssign) -> None:
        name = s.target.id
        t, where = _annotation(s.annotation)
        if _is_call(t, "shared"):
            return self.shared(name, t)
        if isinstance(t, ast.Subscript):  # T[n] or T[a][b]: a private array
            dims = []
            base = t
            while isinstance(base, ast.Subscript):
                dims.append(base.slice)
                base = base.value
            if not (isinstance(base, ast.Name) and base.id in _TYPES):
                raise HipgenError(f"{_line(s)}: unsupported array type")
            ctype = _TYPES[base.id][0]
            extent = "".join(f"[{self.expr(d)}]" for d in reversed(dims))
            zero = (isinstance(s.value, ast.Set) and len(s.value.elts) == 1
                    and isinstance(s.value.elts[0], ast.Constant) and s.value.elts[0].value == 0)
            if s.value is not None and not zero:
                raise HipgenError(f"{_line(s)}: a private array is declared bare or with `= {{0}}`")
            self.emit(f"{ctype} {name}{extent}{' = {0}' if zero else ''};")
            self.pointer_type[name] = ctype + "*"
            return
        ctype = _Scalar.text(t)
        if ctype.endswith("*"):
            self.pointer_type[name] = ctype
        if s.value is None:
            return self.emit(f"{ctype} {name};")
        saved, self.id_level = self.id_level, where or self.id_level
        self.emit(f"{ctype} {name} = {self.expr(s.value)};")
        self.id_level = saved

    def shared(self, name: str, t: ast.Call) -> None:
        arg = t.args[0] if t.args else None
        if not (isinstance(arg, ast.Subscript) and isinstance(arg.value, ast.Name) and arg.value.id in _TYPES):
            raise HipgenError(f"{_line(t)}: expected shared(type[size])")
        ctype, nbytes = _TYPES[arg.value.id]
        size = self.expr(arg.slice)
        align, static = None, False
        for kw in t.keywords:
            if kw.arg == "align" and isinstance(kw.value, ast.Constant):
                align = int(kw.value.value)
            elif kw.arg == "static" and isinstance(kw.value, ast.Constant):
                static = bool(kw.value.value)
            else:
                raise HipgenError(f"{_line(t)}: shared() takes align= and static=")
        self.pointer_type[name] = ctype + "*"
        if static:
            self.emit(f"__shared__ {f'__align__({align}) ' if align else ''}{ctype} {name}[{size}];")
        else:
            count = self.constant(arg.slice)
            if align:
                self.smem_offset = (self.smem_offset + align - 1) // align * align
            self.emit(f"{f'__align__({align}) ' if align else ''}{ctype} (&{name})[{size}] = "
                      f"*(({ctype} (*)[{size}])(__smem + {self.smem_offset}));")
            self.smem_offset += count * nbytes
        if self.plan is not None and name in self.plan.handed:
            # the array is handed between the cases of a split: its two round counters, cleared before anyone waits
            self.emit(f"__shared__ unsigned int __full_{name}, __empty_{name};")
            self.emit(f"int __round_{name} = 0;")
            if name in self.plan.filled_together:
                self.emit(f"bool __pending_{name} = false;  // filled by this wavefront and not announced yet")
            self.emit(f"if (threadIdx.x == 0) {{ __full_{name} = 0; __empty_{name} = 0; }}")
            self.emit("__syncthreads();")

    def constant(self, n: ast.AST) -> int:
        """Element count of a dynamic LDS window: it fixes the next window's offset, so it must be a number."""
        if isinstance(n, ast.Constant) and isinstance(n.value, int) and not isinstance(n.value, bool):
            return n.value
        if isinstance(n, ast.BinOp) and type(n.op) in (ast.Add, ast.Sub, ast.Mult, ast.FloorDiv, ast.Div):
            a, b = self.constant(n.left), self.constant(n.right)
            if isinstance(n.op, ast.Add):
                return a + b
            if isinstance(n.op, ast.Sub):
                return a - b
            if isinstance(n.op, ast.Mult):
                return a * b
            return a // b
        raise HipgenError(f"{_line(n)}: the size of a dynamic shared() array must be a constant "
                          "(use static=True for sizes that depend on template parameters)")

    def group(self, s: ast.With, call: ast.Call) -> None:
        if not call.args:
            raise HipgenError(f"{_line(s)}: group() takes a perspective")
        level, size = _level(call.args[0])
        if size < 1:
            raise HipgenError(f"{_line(s)}: a group has at least one member")
        if level == "thread" and size > 1 and size % 64 and (size & (size - 1) or size > 64):
            raise HipgenError(f"{_line(s)}: group(thread[{size}]): a thread group is a power of two up to the 64-lane "
                              "wavefront or a whole number of wavefronts, so that no wavefront is shared between groups")
        outer = self.ids
        inner = _Ids(f"__block_id_{outer.depth + 1}", f"__thread_id_{outer.depth + 1}", outer.depth + 1)
        self.open()
        if level == "block":
            self.emit(f"int {inner.block_id} = {outer.block_id} % {size};")
            self.emit(f"int {inner.thread_id} = {inner.block_id} * blockDim.x + threadIdx.x;")
        elif level == "thread":
            self.emit(f"int {inner.block_id} = {outer.block_id};")
            self.emit(f"int {inner.thread_id} = {outer.thread_id} % {size};")
        else:
            self.emit(f"int {inner.block_id} = {outer.block_id};")
            self.emit(f"int {inner.thread_id} = {outer.thread_id};")
        saved_level, self.id_level = self.id_level, (level, size)
        self.ids = inner
        self.block(s.body)
        self.ids = outer
        self.id_level = saved_level
        self.close()

    def partition(self, s: ast.With, call: ast.Call, target) -> None:
        if not (isinstance(target, ast.Name) and call.args and isinstance(call.args[0], ast.Name)):
            raise HipgenError(f"{_line(s)}: expected `with partition(array, p=..., offset=...) as view`")
        kw = {k.arg: k.value for k in call.keywords}
        if not set(kw) <= {"p", "offset", "f"} or ("f" in kw and "offset" in kw):
            raise HipgenError(f"{_line(s)}: partition() takes p= and one of offset= and f=")
        if "p" in kw:
            _level(kw["p"])  # checked for shape only: the view is plain pointer arithmetic
        parent = call.args[0].id
        ctype = self.pointer_type.get(parent)
        if ctype is None:
            raise HipgenError(f"{_line(s)}: {parent} is not a pointer or array")
        if "f" in kw:
            fn = kw["f"]
            if not (isinstance(fn, ast.Lambda) and len(fn.args.args) == 1 and not fn.args.defaults):
                raise HipgenError(f"{_line(s)}: f= takes a lambda of one index")
            if target.id in self.views or target.id in self.pointer_type:
                raise HipgenError(f"{_line(s)}: {target.id} is already the name of an array or view")
            # No pointer is declared: every element access goes through the index map.
            self.views[target.id] = (parent, fn, _level(kw["p"]) if "p" in kw else None)
            self.pointer_type[target.id] = ctype
            self.block(s.body)
            del self.views[target.id]
            del self.pointer_type[target.id]
            return
        if parent in self.views:
            raise HipgenError(f"{_line(s)}: {parent} is an index-mapped view; it has no address to offset "
                              "(use f=lambda i: i + offset)")
        saved, self.id_level = self.id_level, (_level(kw["p"]) if "p" in kw else self.id_level)
        offset = self.expr(kw["offset"]) if "offset" in kw else "0"
        self.id_level = saved
        self.open()
        self.emit(f"{ctype} {target.id} = {parent} + ({offset});")
        self.pointer_type[target.id] = ctype
        self.block(s.body)
        self.close()

    # -- the function
    def emit_function(self) -> str:
        tree = ast.parse(self.k.source)
        fn = tree.body[0]
        if not isinstance(fn, ast.FunctionDef):
            raise HipgenError("expected a function definition")
        args = fn.args.args
        defaults = dict(zip([a.arg for a in args[len(args) - len(fn.args.defaults):]], fn.args.defaults))
        for a in args:
            if a.arg == "template":
                d = defaults.get("template")
                if not isinstance(d, ast.List):
                    raise HipgenError("template= takes a list of (name, type) pairs")
                for item in d.elts:
                    if not (isinstance(item, ast.Tuple) and len(item.elts) == 2 and isinstance(item.elts[0], ast.Constant)):
                        raise HipgenError("template= takes a list of (name, type) pairs")
                    ttype = item.elts[1]
                    if _is_call(ttype, "constexpr") and ttype.args:   # every template parameter is a constant already
                        ttype = ttype.args[0]
                    self.template.append((_Scalar.text(ttype), str(item.elts[0].value)))
                continue
            if a.annotation is None:
                raise HipgenError(f"parameter {a.arg} needs a `type @ perspective` annotation")
            t, _ = _annotation(a.annotation)
            ctype = _Scalar.text(t)
            self.params.append((ctype, a.arg))
            if ctype.endswith("*") or ctype.endswith("__restrict__"):
                self.pointer_type[a.arg] = ctype
        device = self.k.kind == "device"
        ret = "void"
        if fn.returns is not None:
            ret = _Scalar.text(_annotation(fn.returns)[0])
            self.returns_value = ret != "void"
        elif not device and any(isinstance(n, ast.Return) and n.value is not None for n in ast.walk(fn)):
            raise HipgenError("a global kernel returns nothing")
        if self.auto_sync:
            self.plan = _SyncPlan(fn)
        plist = (["int __block_id", "int __thread_id", "char* __smem"] if device else []) + [f"{t} {n}" for t, n in self.params]
        if self.template:
            self.emit("template<" + ", ".join(f"{t} {n}" for t, n in self.template) + ">")
        attr = f" {self.k.attr}" if getattr(self.k, "attr", "") else ""
        self.emit(f"{'__device__' if device else '__global__'}{attr} {ret} {self.k.name}({', '.join(plist)}) {{")
        self.indent += 1
        if device:
            self.emit(f"int {self.ids.block_id} = __block_id;")
            self.emit(f"int {self.ids.thread_id} = __thread_id;")
        else:
            self.emit("extern __shared__ __align__(128) char __smem[];")
            self.emit(f"int {self.ids.block_id} = blockIdx.x;")
            self.emit(f"int {self.ids.thread_id} = {self.ids.block_id} * blockDim.x + threadIdx.x;")
        self.block(fn.body)
        self.indent -= 1
        self.emit("}")
        text = "\n".join(self.out) + "\n"
        # the word the hand-over waits report into is defined once per file, whichever function comes first
        if getattr(self, "uses_late_announcements", False):
            text = LATE_ANNOUNCEMENT_HELPERS + text
        return (HANDOVER_REPORT_DEFINITION + text) if getattr(self, "uses_handover_report", False) else text


def generate_blocks(name: str, auto_sync: bool = True, annotate: bool = False, handover_spins: Optional[int] = None) -> str:
    """HIP text of kernel or device function `name` in the structured form described above. annotate=True puts a
    comment in front of every barrier that names the statement's source line and the arrays the barrier is for
    (the reference keeps such a record per barrier as well, SyncReason, prism/sync_analysis.py:40-73)."""
    if name not in _REGISTRY:
        raise HipgenError(f"no kernel named {name!r} has been defined with @prism")
    return BlockEmitter(_REGISTRY[name], auto_sync, annotate, handover_spins).emit_function()


def explain_barriers(name: str) -> List[str]:
    """One line per barrier of `name`, in program order: where it stands and which arrays it orders."""
    text = generate_blocks(name, True, annotate=True).splitlines()
    return [text[n - 1].strip()[3:] for n, ln in enumerate(text) if ln.strip() == "__syncthreads();" and text[n - 1].strip().startswith("// ")]


def dynamic_lds_bytes(name: str) -> int:
    """Bytes of the dynamic LDS block (`__smem`) the kernel's non-static shared() arrays take."""
    em = BlockEmitter(_REGISTRY[name], False)
    em.emit_function()
    return em.smem_offset


def device_functions_used(name: str) -> List[str]:
    """Names of the @prism("device") functions kernel `name` calls, callees first."""
    order: List[str] = []

    def visit(n: str) -> None:
        tree = ast.parse(_REGISTRY[n].source)
        for node in ast.walk(tree):
            if (isinstance(node, ast.Call) and isinstance(node.func, ast.Name) and node.func.id in _REGISTRY
                    and _REGISTRY[node.func.id].kind == "device" and node.func.id not in order and node.func.id != n):
                visit(node.func.id)
                order.append(node.func.id)
    visit(name)
    return order
