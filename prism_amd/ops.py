"""Host-side mirror of the reference's launchers, over libprism_amd.so.

Names, argument order and meaning follow the C++ entry points of the
reference's evaluation harnesses so that a test written against those reads the
same here:

  get_workspace_size / launch_scan   evals/4090_scan/main.cu:63-86
  run_my_kernel                      evals/4090_sgemm/runner.cu:245-267
  runmyh100                          evals/h100_bench/utils.cuh:504-533
  add_m                              kernel signature in README.md:133-140

plus tensor-shaped conveniences (scan, sgemm, gemm_bf16). Device memory is a
PyTorch-ROCm tensor (or a raw integer device pointer where noted); torch is
only the allocator and the stream provider, every computation is a HIP kernel
in the shared library. All calls are asynchronous on torch's current stream
unless the reference's shape fixes the default stream.
"""
from __future__ import annotations

from typing import Optional, Union

import torch

from . import _lib

SGEMM_KERNELS = {
    1: "naive",
    2: "coalesced",
    3: "lds_block",
    4: "thread_tile_vec",
    5: "wave_tile_mfma",
    6: "thread_tile_scalar",
}

Ptr = Union[int, "torch.Tensor"]


class PrismError(RuntimeError):
    """A launcher in libprism_amd.so reported a failure."""


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = _lib.last_error()
        if rc == 1:
            raise ValueError(f"{what}: {msg}")
        raise PrismError(f"{what}: HIP error {rc}: {msg}")


def _ptr(t: Ptr) -> int:
    if isinstance(t, int):
        return t
    if t is None:
        return 0
    if not t.is_cuda:
        raise ValueError("expected a tensor in device memory (cuda), got a host tensor")
    if not t.is_contiguous():
        raise ValueError("expected a contiguous tensor")
    return t.data_ptr()


def _need(t: "torch.Tensor", dtypes, numel: int, name: str) -> None:
    if t.dtype not in dtypes:
        raise TypeError(f"{name}: dtype {t.dtype} not in {tuple(dtypes)}")
    if t.numel() < numel:
        raise ValueError(f"{name}: holds {t.numel()} elements, {numel} needed")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


# ------------------------------------------------------------------- add_m --

def add_m(x: "torch.Tensor", y: "torch.Tensor", m: int) -> "torch.Tensor":
    """y[i] = x[i] + m (int32 wrap-around) for every element of x; returns y."""
    _need(x, (torch.int32,), 0, "x")
    _need(y, (torch.int32,), x.numel(), "y")
    m = ((int(m) + 2**31) % 2**32) - 2**31  # wrap m itself like an int32 argument
    _check(_lib.load().prism_add_m(_ptr(x), _ptr(y), m, x.numel(), _stream()), "add_m")
    return y


def wave_regroup(inp: "torch.Tensor", items_per_lane: int, to_striped: bool = True,
                 out: Optional["torch.Tensor"] = None) -> "torch.Tensor":
    """Moves every chunk of 64 * items_per_lane int32 between the blocked arrangement of the reference's warp_load
    (lane l holds items_per_lane consecutive items) and the striped one (item j of lane l is element 64 j + l)."""
    _need(inp, (torch.int32,), 0, "inp")
    if out is None:
        out = torch.empty_like(inp)
    _need(out, (torch.int32,), inp.numel(), "out")
    _check(_lib.load().prism_wave_regroup_i32(_ptr(inp), _ptr(out), inp.numel(), int(items_per_lane),
                                              0 if to_striped else 1, _stream()), "wave_regroup")
    return out


# -------------------------------------------------------------------- scan --

SCAN_EXCLUSIVE = 1       # flag values of include/prism_amd.h
SCAN_TICKET_ORDER = 2
SCAN_NO_HELP = 4
SCAN_OP = {"sum": 0x00, "max": 0x10, "min": 0x20}
ERROR_SCAN_ORDER = 10001
ERROR_SCAN_WORKSPACE = 10002


class ScanOrderError(PrismError):
    """A tile of a scan gave up waiting for its predecessors; that call's output is invalid."""


class ScanWorkspaceError(PrismError):
    """A scan ran on a workspace that was never initialised (or was overwritten); its output is invalid."""


def get_workspace_size(n: int) -> int:
    """Workspace bytes for an n-element scan (scan_gpu::get_workspace_size)."""
    if n < 0:
        raise ValueError("n must be >= 0")
    return int(_lib.load().prism_scan_workspace_bytes(n))


def _ws_bytes(workspace: "torch.Tensor") -> int:
    return workspace.numel() * workspace.element_size()


def new_scan_workspace(n: int, device="cuda") -> "torch.Tensor":
    """An initialised workspace for scans of up to n elements (the fill is enqueued on the current stream)."""
    return scan_workspace_init(torch.empty(get_workspace_size(n), dtype=torch.uint8, device=device))


def scan_workspace_init(workspace: "torch.Tensor") -> "torch.Tensor":
    """Bring a workspace into its initial state (needed once; every scan leaves it ready for the next)."""
    _check(_lib.load().prism_scan_workspace_init(_ptr(workspace), _ws_bytes(workspace), _stream()),
           "scan_workspace_init")
    return workspace


def scan_status(workspace: "torch.Tensor", stream: Optional[int] = None) -> None:
    """Wait for the stream; raise ScanWorkspaceError if a scan found the workspace uninitialised, ScanOrderError
    if one that does not help its predecessors gave up in its look-back."""
    rc = _lib.load().prism_scan_status(_ptr(workspace), _ws_bytes(workspace), _stream() if stream is None else stream)
    if rc == ERROR_SCAN_ORDER:
        raise ScanOrderError(_lib.last_error())
    if rc == ERROR_SCAN_WORKSPACE:
        raise ScanWorkspaceError(_lib.last_error())
    _check(rc, "scan_status")


def launch_scan(n: int, x: "torch.Tensor", workspace: "torch.Tensor", check: bool = True) -> "torch.Tensor":
    """In-place inclusive scan of the first n elements of x (scan_gpu::launch_scan).

    Returns the tensor that holds the result (x itself), as the reference
    returns its device pointer. Runs on the default stream like the reference,
    and like the reference accepts a workspace with any contents. With
    check=True (default) it then waits for the result and raises ScanOrderError
    if the look-back gave up; check=False leaves the call asynchronous and the
    check (scan_status) to the caller.
    """
    _need(x, (torch.int32, torch.uint32), n, "x")
    if _ws_bytes(workspace) < get_workspace_size(n):
        raise ValueError("workspace smaller than get_workspace_size(n)")
    out = _lib.load().prism_launch_scan(n, _ptr(x), _ptr(workspace))
    if n > 0 and not out:
        raise PrismError(f"launch_scan: {_lib.last_error()}")
    if check and n > 0:
        scan_status(workspace, stream=0)
    return x


def scan(inp: "torch.Tensor", out: Optional["torch.Tensor"] = None,
         workspace: Optional["torch.Tensor"] = None, exclusive: bool = False, op: str = "sum",
         ticket_order: bool = False, spin_limit: int = -1, check: bool = True, help: bool = True) -> "torch.Tensor":
    """Prefix sum modulo 2^32 of a 1-D int32/uint32 tensor (modulo 2^64 of an int64/uint64 one); out may be inp. Inclusive (out[i] includes
    inp[i]) unless exclusive=True (out[0] = 0, out[i] = inp[0] + ... + inp[i-1]). op="max" / op="min": the
    running maximum / minimum of an int32 tensor instead (inclusive only).

    workspace: an initialised workspace (new_scan_workspace / scan_workspace_init) that calls on one stream
    may share; None allocates one. ticket_order numbers tiles by the reference's ticket counter instead of
    by workgroup id; spin_limit bounds the polls of a look-back window before the tile helps a silent
    predecessor (-1: library default, 0: no waiting); help=False makes a look-back that runs out of polls
    report instead (ScanOrderError), the plain bounded wait. check=True (default) waits for the result and
    raises if the workspace was uninitialised or such a look-back gave up; check=False leaves the call
    asynchronous and the check (scan_status) to the caller.
    """
    if op not in SCAN_OP:
        raise ValueError("scan: op must be 'sum', 'max' or 'min'")
    if inp.dtype in (torch.int64, torch.uint64):  # 64-bit elements: inclusive sums modulo 2^64 only
        if op != "sum" or exclusive or ticket_order:
            raise ValueError("scan: 64-bit elements support the inclusive sum in workgroup-id order only")
        n = inp.numel()
        if out is None:
            out = torch.empty_like(inp)
        _need(out, (inp.dtype,), n, "out")
        if workspace is None:
            workspace = new_scan_workspace(n, inp.device)
        _check(_lib.load().prism_scan_i64_ex(_ptr(inp), _ptr(out), n, _ptr(workspace), _ws_bytes(workspace),
                                             0 if help else SCAN_NO_HELP, int(spin_limit), _stream()), "scan")
        if check and n > 0:
            scan_status(workspace)
        return out
    if op != "sum" and (exclusive or ticket_order):
        raise ValueError("scan: the running maximum and minimum are inclusive and use workgroup-id order")
    _need(inp, (torch.int32,) if op != "sum" else (torch.int32, torch.uint32), 0, "inp")
    n = inp.numel()
    if out is None:
        out = torch.empty_like(inp)
    _need(out, (inp.dtype,), n, "out")
    if workspace is None:
        workspace = new_scan_workspace(n, inp.device)
    flags = (SCAN_OP[op] | (SCAN_EXCLUSIVE if exclusive else 0) | (SCAN_TICKET_ORDER if ticket_order else 0)
             | (0 if help else SCAN_NO_HELP))
    _check(_lib.load().prism_scan_i32_ex(_ptr(inp), _ptr(out), n, _ptr(workspace), _ws_bytes(workspace), flags,
                                         int(spin_limit), _stream()), "scan")
    if check and n > 0:
        scan_status(workspace)
    return out


def segmented_scan(inp: "torch.Tensor", heads: "torch.Tensor", out: Optional["torch.Tensor"] = None,
                   workspace: Optional["torch.Tensor"] = None, check: bool = True, spin_limit: int = -1,
                   help: bool = True) -> "torch.Tensor":
    """Inclusive sums modulo 2^32 that start again at every element whose byte in `heads` (uint8 / bool, one per
    element) is non-zero; element 0 always starts a segment. out may be inp. workspace, check, spin_limit and help
    as for scan()."""
    _need(inp, (torch.int32, torch.uint32), 0, "inp")
    n = inp.numel()
    _need(heads, (torch.uint8, torch.bool), n, "heads")
    if out is None:
        out = torch.empty_like(inp)
    _need(out, (inp.dtype,), n, "out")
    if workspace is None:
        workspace = new_scan_workspace(n, inp.device)
    _check(_lib.load().prism_segmented_scan_i32_ex(_ptr(inp), _ptr(heads), _ptr(out), n, _ptr(workspace), _ws_bytes(workspace),
                                                   0 if help else SCAN_NO_HELP, int(spin_limit), _stream()), "segmented_scan")
    if check and n > 0:
        scan_status(workspace)
    return out


# ------------------------------------------------------------------- sgemm --

def run_my_kernel(my_kernel_num: int, M: int, N: int, K: int, alpha: float, A: Ptr, B: Ptr,
                  beta: float, C: Ptr) -> None:
    """C = alpha*A@B + beta*C with kernel 1..5 on the default stream (run_my_kernel).

    Raises ValueError for an unknown kernel number, where the reference throws
    std::invalid_argument.
    """
    if my_kernel_num not in (1, 2, 3, 4, 5):
        raise ValueError("Unknown my_kernel number")
    _check(_lib.load().prism_run_my_kernel(my_kernel_num, M, N, K, alpha, _ptr(A), _ptr(B), beta, _ptr(C)),
           "run_my_kernel")


def sgemm_workspace_size(M: int, N: int, K: int) -> int:
    """Workspace bytes with which kernel 5 shares K ranges between workgroups for this shape on the current
    device (0: it would not)."""
    return int(_lib.load().prism_sgemm_workspace_bytes(M, N, K))


def sgemm_workspace_plan(M: int, N: int, K: int, workspace_bytes: int):
    """(workgroups that share K ranges, tiles they share) for a call with aligned operands and that much
    workspace; (0, 0) when the call would be the plain one."""
    import ctypes
    groups, tiles = ctypes.c_int(0), ctypes.c_int(0)
    _check(_lib.load().prism_sgemm_ws_plan(M, N, K, workspace_bytes, ctypes.byref(groups), ctypes.byref(tiles)), "sgemm_ws_plan")
    return groups.value, tiles.value


def sgemm(M: int, N: int, K: int, alpha: float, A: "torch.Tensor", B: "torch.Tensor", beta: float,
          C: "torch.Tensor", variant: int = 5, workspace: Optional["torch.Tensor"] = None) -> "torch.Tensor":
    """sgemm(M,N,K,alpha,A,B,beta,C): the kernel signature of generated/my_sgemm_kernel_*.cu.

    workspace: a device buffer of at least sgemm_workspace_size(M, N, K) bytes lets kernel 5 share the K ranges
    of the tiles of a partial last round (or of all tiles of a skinny shape) between all compute units
    (deterministic: a tile's partial products are added in the order of k); calls that share one must be
    ordered on one stream. Without it the call is the reference-shaped one.
    """
    if variant not in (0, 1, 2, 3, 4, 5, 6):
        raise ValueError("Unknown my_kernel number")
    _need(A, (torch.float32,), M * K, "A")
    _need(B, (torch.float32,), K * N, "B")
    _need(C, (torch.float32,), M * N, "C")
    if workspace is None:
        _check(_lib.load().prism_sgemm(variant, M, N, K, alpha, _ptr(A), _ptr(B), beta, _ptr(C), _stream()), "sgemm")
    else:
        _check(_lib.load().prism_sgemm_ws(variant, M, N, K, alpha, _ptr(A), _ptr(B), beta, _ptr(C), _ptr(workspace),
                                          _ws_bytes(workspace), _stream()), "sgemm")
    return C


# --------------------------------------------------------------- bf16 gemm --

def gemm_bf16(A: "torch.Tensor", B: "torch.Tensor", D: Optional["torch.Tensor"] = None) -> "torch.Tensor":
    """D[M,N] (fp32) = A[M,K] @ B[N,K]^T for bf16 A and B."""
    _need(A, (torch.bfloat16,), 0, "A")
    _need(B, (torch.bfloat16,), 0, "B")
    if A.dim() != 2 or B.dim() != 2 or A.shape[1] != B.shape[1]:
        raise ValueError("A must be MxK and B NxK")
    M, K = A.shape
    N = B.shape[0]
    if D is None:
        D = torch.empty((M, N), dtype=torch.float32, device=A.device)
    _need(D, (torch.float32,), M * N, "D")
    _check(_lib.load().prism_gemm_bf16(M, N, K, _ptr(A), _ptr(B), _ptr(D), _stream()), "gemm_bf16")
    return D


def runmyh100(M: int, N: int, K: int, A: Ptr, B: Ptr, C: Ptr, DB: Optional[Ptr] = None) -> None:
    """bf16 C, column-major MxN, = A[M,K] @ B[N,K]^T on the default stream (runmyh100)."""
    _check(_lib.load().prism_runmyh100(M, N, K, _ptr(A), _ptr(B), _ptr(C), _ptr(DB) if DB is not None else 0),
           "runmyh100")


# -------------------------------------------------------------------- misc --

def device_info() -> dict:
    import ctypes as C
    cu, khz, wave = C.c_int(), C.c_int(), C.c_int()
    lds, hbm = C.c_size_t(), C.c_size_t()
    name = C.create_string_buffer(128)
    _check(_lib.load().prism_device_info(C.byref(cu), C.byref(khz), C.byref(wave), C.byref(lds), C.byref(hbm),
                                         name, 128), "device_info")
    return {"cu_count": cu.value, "clock_khz": khz.value, "wavefront_size": wave.value,
            "lds_bytes": lds.value, "hbm_bytes": hbm.value, "name": name.value.decode()}


def tile_coords(workgroup_id: int, tiles_m: int, tiles_n: int) -> tuple:
    import ctypes as C
    tm, tn = C.c_int(), C.c_int()
    _check(_lib.load().prism_tile_coords(workgroup_id, tiles_m, tiles_n, C.byref(tm), C.byref(tn)), "tile_coords")
    return tm.value, tn.value
