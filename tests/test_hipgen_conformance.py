"""The checker's verdict on every behaviour the reference's front-end tests pin, one small program each.

The reference fixes its perspective rules in test/test_pointers.py, test/test_perspective_bounds.py,
test/test_group.py, test/test_split.py, test/test_partition.py, test/test_claim.py, test/test_local_arrays.py,
test/test_shared_memory.py and test/test_function_calls.py (the assignment rules of test/test_type_checker.py
are covered in test_hipgen_check.py). Each section below names the file whose cases it follows, in that file's
order; the programs are this repository's own and only the verdicts (accepted / refused) are the reference's.
Where the reference raises one of its error classes, hipgen_check raises PerspectiveError with a message that
names the rule; a program that the reference accepts must pass check() untouched. CPU only.
"""
import pytest

from prism_amd.hipgen import (GLOBAL, LOCAL, SHARED, bf16, block, claim, const, double, grid, group, partition,
                              prism, ptr, requires, restrict, shared, split, thread)
from prism_amd.hipgen_blocks import generate_blocks
from prism_amd.hipgen_check import PerspectiveError, check

CASES = []
REFUSED = "refused"


def case(expect):
    def note(name):
        CASES.append((name, expect))
        return name
    return note

def case(expect):
    def deco(fn_name):
        CASES.append((fn_name, expect)); return fn_name
    return deco

# ------------------------------------------------------------ test/test_pointers.py --
@requires(grid[1])
@prism("device")
def ptr_decl_in_body():
    p: ptr(int) @ grid[1]
case(None)("ptr_decl_in_body")

@requires(grid[1])
@prism("device")
def const_ptr_decl_in_body():
    p: const(ptr(float)) @ block[1]
case(None)("const_ptr_decl_in_body")

@requires(grid[1])
@prism("device")
def restrict_ptr_decl_in_body():
    p: restrict(ptr(int)) @ grid[1]
case(None)("restrict_ptr_decl_in_body")

@requires(grid[1])
@prism("device")
def ptr_param_read(p: ptr(int) @ block[1]):
    x: int @ thread[1]
    x = p[0]
case(None)("ptr_param_read")

@requires(grid[1])
@prism("device")
def ptr_assigned(p: ptr(int) @ block[1], q: ptr(int) @ grid[1]):
    p = q
case(REFUSED)("ptr_assigned")

@requires(grid[1])
@prism("device")
def deref_thread_index(p: ptr(int) @ block[1]):
    i: int @ thread[1]
    x: int @ thread[1]
    x = p[i]
case(None)("deref_thread_index")

@requires(grid[1])
@prism("device")
def deref_block_index(p: ptr(int) @ block[1]):
    j: int @ block[1]
    x: int @ thread[1]
    x = p[j]
case(None)("deref_block_index")

@requires(grid[1])
@prism("device")
def deref_narrowed_into_block(p: ptr(int) @ block[1]):
    i: int @ thread[1]
    y: int @ block[1]
    y = p[i]
case(REFUSED)("deref_narrowed_into_block")

@requires(grid[1])
@prism("device")
def subscript_scalar():
    x: int @ thread[1]
    y: int @ thread[1]
    y = x[0]
case(REFUSED)("subscript_scalar")

@requires(grid[1])
@prism("device")
def subscript_scalar_param(n: int @ grid[1]):
    x: int @ thread[1]
    x = n[0]
case(REFUSED)("subscript_scalar_param")

@requires(grid[1])
@prism("device")
def constant_everywhere():
    a: int @ thread[1]
    b: int @ block[1]
    c: int @ grid[1]
    a = 5
    b = 42
    c = 100
    a = b + 5
case(None)("constant_everywhere")

@requires(grid[1])
@prism("device")
def store_thread_ptr(p: ptr(int) @ thread[1]):
    x: int @ thread[1]
    p[0] = x
case(None)("store_thread_ptr")

@requires(grid[1])
@prism("device")
def store_block_ptr(p: ptr(int) @ block[1]):
    x: int @ thread[1]
    p[0] = x
case(REFUSED)("store_block_ptr")

@requires(grid[1])
@prism("device")
def store_scalar(n: int @ thread[1]):
    n[0] = 5
case(REFUSED)("store_scalar")

# The same file writes its pointer types with an address space, ptr(T, GLOBAL | SHARED | LOCAL)
# (prism/type_checker.py:656-667, 728-737).
@requires(grid[1])
@prism("device")
def lds_pointer_read(p: ptr(int, SHARED) @ block[1]):
    i: int @ thread[1]
    x: int @ thread[1]
    x = p[i]
case(None)("lds_pointer_read")

@requires(grid[1])
@prism("device")
def global_pointer_read(p: ptr(float, GLOBAL) @ grid[1]):
    i: int @ thread[1]
    x: float @ thread[1]
    x = p[i]
case(None)("global_pointer_read")

@requires(grid[1])
@prism("device")
def lds_pointer_store_from_block(p: ptr(int, SHARED) @ block[1]):
    x: int @ thread[1]
    p[0] = x
case(REFUSED)("lds_pointer_store_from_block")

@requires(block[1], thread[1])
@prism("device")
def private_pointer_store_from_block(acc: ptr(float, LOCAL) @ block[1], v: float @ block[1]):
    acc[0] = v                      # a thread's own array: any perspective (prism/type_checker.py:399-403)
case(None)("private_pointer_store_from_block")

@requires(grid[1])
@prism("device")
def unknown_address_space(p: ptr(int, thread) @ block[1]):
    x: int @ thread[1]
    x = p[0]
case(REFUSED)("unknown_address_space")


# -------------------------------------------------- test/test_perspective_bounds.py --
@prism("device")
def no_requires():
    x: int @ thread[1]
case(REFUSED)("no_requires")

@requires(grid[1], grid[2])
@prism("device")
def duplicate_level():
    x: int @ thread[1]
case(REFUSED)("duplicate_level")

@requires(thread[1])
@prism("device")
def if_on_grid_value(x: int @ grid[1]):
    if x > 0:
        pass
case(None)("if_on_grid_value")

@requires(grid[1])
@prism("device")
def if_on_thread_value(x: int @ thread[1]):
    if x > 0:
        pass
case(REFUSED)("if_on_thread_value")

@requires(thread[1])
@prism("device")
def for_on_grid_value(n: int @ grid[1]):
    for i in range(n):
        pass
case(None)("for_on_grid_value")

@requires(grid[1])
@prism("device")
def for_on_thread_value(n: int @ thread[1]):
    for i in range(n):
        pass
case(REFUSED)("for_on_thread_value")

@requires(thread[1])
@prism("device")
def for_over_a_name(items: int @ grid[1]):
    for i in items:
        pass
case(REFUSED)("for_over_a_name")

@requires(thread[1])
@prism("device")
def while_on_block_value(x: int @ block[1]):
    while x > 0:
        pass
case(None)("while_on_block_value")

@requires(block[1])
@prism("device")
def while_on_thread_value(x: int @ thread[1]):
    while x > 0:
        pass
case(REFUSED)("while_on_thread_value")

# --------------------------------------------------------------- test/test_group.py --
@requires(grid[1], block[4])
@prism("device")
def group_narrower_blocks():
    with group(block[2]):
        pass
case(None)("group_narrower_blocks")

@requires(grid[1], block[2])
@prism("device")
def group_wider_blocks():
    with group(block[4]):
        pass
case(REFUSED)("group_wider_blocks")

@requires(grid[2], block[4], thread[8])
@prism("device")
def grid_value_in_block_group(x: int @ grid[2]):
    with group(block[4]):
        if x > 0:
            pass
case(None)("grid_value_in_block_group")

@requires(grid[2], block[4], thread[8])
@prism("device")
def thread_value_in_block_group(x: int @ thread[8]):
    with group(block[4]):
        if x > 0:
            pass
case(REFUSED)("thread_value_in_block_group")

@requires(grid[1], block[2], thread[4])
@prism("device")
def groups_nest(x: int @ block[2], y: int @ thread[4]):
    with group(block[2]):
        if x > 0:
            pass
        with group(thread[4]):
            if y > 0:
                pass
        if x > 0:
            pass
case(None)("groups_nest")

@requires(grid[1], block[2], thread[4])
@prism("device")
def same_group_again():
    with group(block[2]):
        with group(block[2]):
            pass
case(None)("same_group_again")

@requires(grid[1], block[2], thread[4])
@prism("device")
def group_back_to_grid():
    with group(block[2]):
        with group(grid[1]):
            pass
case(REFUSED)("group_back_to_grid")

# --------------------------------------------------------------- test/test_split.py --
@requires(grid[1], block[8], thread[8])
@prism("device")
def split_blocks_224():
    match split(block):
        case 2:
            with group(thread[8]):
                pass
        case 2:
            with group(thread[8]):
                pass
        case 4:
            with group(thread[8]):
                pass
case(None)("split_blocks_224")

@requires(grid[1], block[4], thread[8])
@prism("device")
def split_3_1():
    match split(block):
        case 3:
            pass
        case 1:
            pass
case(None)("split_3_1")

@requires(grid[1], block[4], thread[8])
@prism("device")
def split_5_of_4():
    match split(block):
        case 5:
            pass
case(REFUSED)("split_5_of_4")

@requires(grid[1], block[4], thread[8])
@prism("device")
def split_2_then_3_of_4():
    match split(block):
        case 2:
            pass
        case 3:
            pass
case(REFUSED)("split_2_then_3_of_4")

@requires(grid[1], block[4], thread[8])
@prism("device")
def split_thread_value_in_case(x: int @ thread[8]):
    match split(block):
        case 2:
            if x > 0:
                pass
case(REFUSED)("split_thread_value_in_case")

@requires(grid[1], block[4], thread[8])
@prism("device")
def split_1_2():
    match split(block):
        case 1:
            pass
        case 2:
            pass
case(None)("split_1_2")

@requires(grid[1], block[4], thread[8])
@prism("device")
def split_3_2_of_4():
    match split(block):
        case 3:
            pass
        case 2:
            pass
case(REFUSED)("split_3_2_of_4")

# ----------------------------------------------------------- test/test_partition.py --
@requires(grid[1], block[1], thread[1])
@prism("device")
def partition_lambda_ok(data: ptr(int) @ grid[1], n: int @ grid[1]):
    with partition(data, p=thread[1], f=lambda i: i + id() * n) as mine:
        mine[0] = 42
case(None)("partition_lambda_ok")

@requires(grid[1], block[1], thread[1])
@prism("device")
def partition_wrong_bound(data: ptr(int) @ block[1]):
    with partition(data, p=thread[1], f=lambda i: i) as mine:
        mine[0] = 42
case(REFUSED)("partition_wrong_bound")

@requires(grid[1], block[1], thread[1])
@prism("device")
def partition_reads_original(data: ptr(int) @ grid[1]):
    with partition(data, p=thread[1], f=lambda i: i) as mine:
        mine[0] = data[0]
case(None)("partition_reads_original")

@requires(grid[1], block[1], thread[1])
@prism("device")
def partition_lambda_narrow_var(data: ptr(int) @ grid[1], off: int @ thread[1]):
    with partition(data, p=block[1], f=lambda i: i + off) as mine:
        pass
case(REFUSED)("partition_lambda_narrow_var")

@requires(block[4], thread[1])
@prism("device")
def partition_in_sibling_cases(data: ptr(int) @ block[2]):
    match split(block):
        case 2:
            with partition(data, p=thread[1], f=lambda i: i) as mine:
                mine[0] = 1
        case 2:
            with partition(data, p=thread[1], f=lambda i: i) as mine:
                mine[0] = 2
case(None)("partition_in_sibling_cases")

@requires(grid[1], block[1], thread[1])
@prism("device")
def partition_offset_ok(data: ptr(int) @ grid[1], n: int @ grid[1]):
    with partition(data, p=thread[1], offset=id() * n) as mine:
        mine[0] = 42
case(None)("partition_offset_ok")

@requires(grid[1], block[1], thread[1])
@prism("device")
def partition_offset_narrow_var(data: ptr(int) @ grid[1], narrow: int @ thread[1]):
    with partition(data, p=block[1], offset=narrow) as mine:
        pass
case(REFUSED)("partition_offset_narrow_var")

# --------------------------------------------------------------- test/test_claim.py --
@requires(block[4], thread[1])
@prism("device")
def claim_one_case(data: ptr(int) @ block[4]):
    with claim(data, p=thread[1]) as mine:
        match split(block):
            case 2:
                x: int @ thread[1] = mine[0]
            case 2:
                pass
case(None)("claim_one_case")

@requires(block[4], thread[1])
@prism("device")
def claim_two_cases(data: ptr(int) @ block[4]):
    with claim(data, p=thread[1]) as mine:
        match split(block):
            case 2:
                x: int @ thread[1] = mine[0]
            case 2:
                y: int @ thread[1] = mine[0]
case(REFUSED)("claim_two_cases")

@requires(grid[1], block[1], thread[1])
@prism("device")
def claim_outside_split(data: ptr(int) @ grid[1]):
    with claim(data, p=thread[1]) as mine:
        x: int @ thread[1] = mine[0]
case(REFUSED)("claim_outside_split")

@requires(block[4], thread[1])
@prism("device")
def claim_offset(data: ptr(int) @ block[4], n: int @ block[4]):
    with claim(data, p=thread[1], offset=id() * n) as mine:
        match split(block):
            case 2:
                x: int @ thread[1] = mine[0]
            case 2:
                pass
case(None)("claim_offset")

@requires(block[4], thread[1])
@prism("device")
def claim_reads_original(data: ptr(int) @ block[4]):
    with claim(data, p=thread[1]) as mine:
        match split(block):
            case 2:
                mine[0] = data[0]
            case 2:
                pass
case(None)("claim_reads_original")

# -------------------------------------------------------- test/test_local_arrays.py --
@requires(grid[1], block[2], thread[4])
@prism("device")
def local_array_block_store():
    buf: int[16] @ block[1]
    x: int @ block[1]
    buf[0] = x
case(None)("local_array_block_store")

@requires(grid[1], block[2], thread[4])
@prism("device")
def local_array_narrow_index(idx: int @ thread[4]):
    buf: int[16] @ block[2]
    r: int @ block[1]
    r = buf[idx]
case(REFUSED)("local_array_narrow_index")

# ------------------------------------------------------- test/test_shared_memory.py --
@requires(grid[1], block[1], thread[1], smem=1024)
@prism("device")
def shared_fits():
    buf: shared(int[64]) @ block[1]
case(None)("shared_fits")

@requires(grid[1], block[1], thread[1], smem=100)
@prism("device")
def shared_too_big():
    buf: shared(int[64]) @ block[1]
case(REFUSED)("shared_too_big")

@requires(grid[1], block[2], thread[1], smem=1024)
@prism("device")
def shared_at_two_blocks():
    buf: shared(int[64]) @ block[2]
case(REFUSED)("shared_at_two_blocks")

@requires(grid[1], block[1], thread[4], smem=1024)
@prism("device")
def shared_at_threads():
    buf: shared(int[64]) @ thread[4]
case(REFUSED)("shared_at_threads")

@requires(grid[1], block[1], thread[1], smem=512)
@prism("device")
def shared_two_fit():
    a: shared(int[64]) @ block[1]
    b: shared(int[64]) @ block[1]
case(None)("shared_two_fit")

@requires(grid[1], block[1], thread[1], smem=400)
@prism("device")
def shared_two_exceed():
    a: shared(int[64]) @ block[1]
    b: shared(int[64]) @ block[1]
case(REFUSED)("shared_two_exceed")

@requires(grid[1], block[1], thread[1], smem=1024)
@prism("device")
def shared_types():
    a: shared(int[64]) @ block[1]
    b: shared(float[64]) @ block[1]
    c: shared(double[32]) @ block[1]
    d: shared(bf16[128]) @ block[1]
case(None)("shared_types")

@requires(grid[1], block[1], thread[1], smem=1023)
@prism("device")
def shared_types_one_byte_short():
    a: shared(int[64]) @ block[1]
    b: shared(float[64]) @ block[1]
    c: shared(double[32]) @ block[1]
    d: shared(bf16[128]) @ block[1]
case(REFUSED)("shared_types_one_byte_short")

@requires(grid[1], block[1], thread[1])
@prism("device")
def shared_without_budget():
    a: shared(int[1]) @ block[1]
case(REFUSED)("shared_without_budget")

# ------------------------------------------------------ test/test_function_calls.py --
@requires(block[1], thread[4], smem=512)
@prism("device")
def callee_smem512():
    pass

@requires(grid[1], block[2], thread[8], smem=1024)
@prism("device")
def caller_smem1024():
    callee_smem512()
case(None)("caller_smem1024")

@requires(grid[1], block[2], thread[8], smem=256)
@prism("device")
def caller_smem256():
    callee_smem512()
case(REFUSED)("caller_smem256")

@requires(block[2], thread[4])
@prism("device")
def callee_b2t4():
    pass

@requires(grid[1], block[4], thread[8])
@prism("device")
def caller_b4t8():
    callee_b2t4()
case(None)("caller_b4t8")

@requires(grid[1], block[2], thread[4])
@prism("device")
def caller_b2t4():
    callee_b2t4()
case(None)("caller_b2t4")

@requires(block[4], thread[8])
@prism("device")
def callee_b4t8():
    pass

@requires(grid[1], block[2], thread[8])
@prism("device")
def caller_b2t8():
    callee_b4t8()
case(REFUSED)("caller_b2t8")

@requires(thread[8])
@prism("device")
def caller_t8_only():
    callee_b2t4()
case(REFUSED)("caller_t8_only")

@requires(block[1], thread[4])
@prism("device")
def callee_int_t4(x: int @ thread[4]):
    pass

@requires(grid[1], block[2], thread[8])
@prism("device")
def pass_t8_to_t4(a: int @ thread[8]):
    callee_int_t4(a)
case(None)("pass_t8_to_t4")

@requires(grid[1], block[2], thread[8])
@prism("device")
def pass_t2_to_t4(a: int @ thread[2]):
    callee_int_t4(a)
case(REFUSED)("pass_t2_to_t4")

@requires(block[1], thread[4])
@prism("device")
def callee_constptr_t4(p: const(ptr(float)) @ thread[4]):
    pass

@requires(grid[1], block[2], thread[8])
@prism("device")
def pass_ptr_t8_to_const_t4(p: ptr(float) @ thread[8]):
    callee_constptr_t4(p)
case(None)("pass_ptr_t8_to_const_t4")

@requires(block[1], thread[4])
@prism("device")
def callee_ptr_t4(p: ptr(float) @ thread[4]):
    pass

@requires(grid[1], block[2], thread[8])
@prism("device")
def pass_ptr_t4_to_t4(p: ptr(float) @ thread[4]):
    callee_ptr_t4(p)
case(None)("pass_ptr_t4_to_t4")

@requires(grid[1], block[2], thread[8])
@prism("device")
def pass_ptr_t8_to_t4(p: ptr(float) @ thread[8]):
    callee_ptr_t4(p)
case(REFUSED)("pass_ptr_t8_to_t4")

@requires(block[1], thread[4])
@prism("device")
def value_at_t4() -> int @ thread[4]:
    return id()

@requires(grid[1], block[2], thread[8])
@prism("device")
def result_into_t4():
    x: int @ thread[4]
    x = value_at_t4()
case(None)("result_into_t4")

@requires(grid[1], block[2], thread[8])
@prism("device")
def result_into_t2():
    x: int @ thread[2]
    x = value_at_t4()
case(None)("result_into_t2")

@requires(grid[1], block[2], thread[8])
@prism("device")
def result_into_t8():
    x: int @ thread[8]
    x = value_at_t4()
case(REFUSED)("result_into_t8")


@pytest.mark.parametrize("name,expect", CASES, ids=[c[0] for c in CASES])
def test_verdict_matches_the_reference(name, expect):
    if expect is None:
        check(name)
    else:
        with pytest.raises(PerspectiveError):
            check(name)


def test_every_refusal_names_its_line_or_function():
    for name, expect in CASES:
        if expect is REFUSED:
            with pytest.raises(PerspectiveError, match=r"line \d+|" + name):
                check(name)


@requires(block[1], thread[64])
@prism("device")
def reversed_through_lds(buf: ptr(int, SHARED) @ block[1], out: ptr(int) @ block[1]):
    t: int @ thread[1] = id()
    with partition(buf, p=thread[1], offset=t) as mine:
        mine[0] = t
    with partition(out, p=thread[1], offset=t) as o:
        o[0] = buf[63 - t]


def test_pointer_into_lds_by_address_space_gets_its_barrier():
    """`ptr(T, SHARED)` is the type `shared(T)` has as a parameter (prism/type_checker.py:694-707), so the
    barrier analysis follows it like one (prism/sync_analysis.py:151-158): a barrier between the store and
    the read of another thread's element. The address space leaves no trace in the C text."""
    check("reversed_through_lds")
    text = generate_blocks("reversed_through_lds")
    assert "int* buf, int* out" in text
    store, barrier, read = text.index("mine[0] = t;"), text.index("__syncthreads();"), text.index("buf[(63 - t)]")
    assert store < barrier < read and text.count("__syncthreads();") == 1
