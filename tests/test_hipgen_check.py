"""Perspective rules (prism_amd/hipgen_check.py): which programs are printed and which are refused.

The cases follow the rule groups the reference tests (test/test_type_checker.py: reads from broader / same /
multiple-index perspectives pass, writes towards broader or incomparable ones fail; test/test_pointers.py:
stores need a thread[1] pointer, only pointers are indexed, pointers are not assigned;
test/test_perspective_bounds.py: @requires, conditions and loop ranges against the bound; test/test_group.py,
test/test_partition.py, test/test_claim.py, test/test_split.py, test/test_shared_memory.py,
test/test_function_calls.py), each with a program of this repository's own. Everything here runs on the CPU:
a refused program never reaches hipcc.
"""
import re

import pytest

from prism_amd.hipgen import (HipgenError, block, claim, const, generate, grid, group, partition, prism, ptr,
                              requires, shared, split, thread)
from prism_amd.hipgen_check import P, PerspectiveError, check, signature


# ------------------------------------------------------------------ the order --

def test_order_of_perspectives():
    g, b, t4, t2, t3, t1 = P("grid", 1), P("block", 1), P("thread", 4), P("thread", 2), P("thread", 3), P("thread", 1)
    assert g.covers(b) and b.covers(t4) and g.covers(t1) and not t1.covers(b) and not b.covers(g)
    assert t4.covers(t2) and t4.covers(t1) and t2.covers(t2) and not t2.covers(t4)
    assert not t3.covers(t2) and not t2.covers(t3)            # neither index divides the other
    assert g.narrowest(t2) == t2 and t2.narrowest(g) == t2 and t4.narrowest(t2) == t2


# ---------------------------------------------------------------- assignments --

@requires(grid[1], block[1], thread[4])
@prism("global")
def reads_go_down(n: int @ grid[1]):
    per_block: int @ block[1] = n + 1              # grid -> block
    four: int @ thread[4] = per_block * 2          # block -> thread[4]
    two: int @ thread[2] = four + per_block        # thread[4] -> thread[2]: 4 is a multiple of 2
    one: int @ thread[1] = two + four + n + 3      # everything is broader than thread[1]
    same: int @ thread[1] = one
    two = four                                     # plain assignment, same rule


@requires(grid[1], block[1], thread[4])
@prism("global")
def thread_into_block(n: int @ grid[1]):
    t: int @ thread[1] = id()
    b: int @ block[1] = t


@requires(grid[1], block[1], thread[4])
@prism("global")
def narrower_index_into_broader(n: int @ grid[1]):
    two: int @ thread[2] = id()
    four: int @ thread[4] = two


@requires(grid[1], block[1], thread[6])
@prism("global")
def incomparable_indices(n: int @ grid[1]):
    three: int @ thread[3] = id()
    two: int @ thread[2] = three


@requires(grid[1], block[1], thread[1])
@prism("global")
def one_narrow_term_spoils_the_sum(n: int @ grid[1]):
    t: int @ thread[1] = id()
    b: int @ block[1] = 0
    b = n + 2 * (t + 1)


@requires(grid[1], block[1], thread[1])
@prism("global")
def uses_an_unknown_name(n: int @ grid[1]):
    t: int @ thread[1] = m + 1


def test_values_only_flow_from_broader_to_narrower():
    check("reads_go_down")
    for name, lhs in (("thread_into_block", "'b' at block[1]"), ("narrower_index_into_broader", "'four' at thread[4]"),
                      ("incomparable_indices", "'two' at thread[2]"), ("one_narrow_term_spoils_the_sum", "'b' at block[1]")):
        with pytest.raises(PerspectiveError, match=re.escape(lhs)):
            check(name)
        with pytest.raises(HipgenError):       # and nothing is printed for it
            generate(name)
    with pytest.raises(PerspectiveError, match="'m' is not declared"):
        check("uses_an_unknown_name")


# ------------------------------------------------------------------- pointers --

@requires(grid[1], block[1], thread[1])
@prism("global")
def element_reads(p: ptr(const(int)) @ grid[1], n: int @ grid[1]):
    b: int @ block[1] = p[3]                       # grid pointer, constant index: grid[1]
    t: int @ thread[1] = id()
    mine: int @ thread[1] = p[t] + p[b]            # narrowed by the index
    held: int[4] @ thread[1] = {0}
    held[1] = mine                                 # a private array takes stores as it is


@requires(grid[1], block[1], thread[1])
@prism("global")
def element_narrowed_by_its_index(p: ptr(const(int)) @ grid[1]):
    t: int @ thread[1] = id()
    b: int @ block[1] = p[t]


@requires(grid[1], block[1], thread[1])
@prism("global")
def store_through_a_broad_pointer(p: ptr(int) @ grid[1]):
    t: int @ thread[1] = id()
    p[t] = 1


@requires(grid[1], block[1], thread[1])
@prism("global")
def store_through_a_thread_view(p: ptr(int) @ grid[1]):
    t: int @ thread[1] = id()
    with partition(p, p=thread[1], offset=t) as mine:
        mine[0] = t


@requires(grid[1], block[1], thread[1])
@prism("global")
def indexes_a_scalar(n: int @ grid[1]):
    t: int @ thread[1] = n[0]


@requires(grid[1], block[1], thread[1])
@prism("global")
def stores_into_a_scalar(n: int @ grid[1]):
    t: int @ thread[1] = 0
    t[0] = n


@requires(grid[1], block[1], thread[1])
@prism("global")
def assigns_a_pointer(p: ptr(int) @ grid[1], q: ptr(int) @ grid[1]):
    p = q


def test_pointer_rules():
    check("element_reads")
    check("store_through_a_thread_view")
    with pytest.raises(PerspectiveError, match="'b' at block\\[1\\] cannot take a value at thread\\[1\\]"):
        check("element_narrowed_by_its_index")
    with pytest.raises(PerspectiveError, match="store through 'p' at grid\\[1\\]"):
        check("store_through_a_broad_pointer")
    with pytest.raises(PerspectiveError, match="'n' is not a pointer or an array"):
        check("indexes_a_scalar")
    with pytest.raises(PerspectiveError, match="'t' is not a pointer or an array"):
        check("stores_into_a_scalar")
    with pytest.raises(PerspectiveError, match="pointer 'p' is not assignable"):
        check("assigns_a_pointer")


# ---------------------------------------------------------- bound and control --

@prism("global")
def no_requires(n: int @ grid[1]):
    t: int @ thread[1] = id()


@requires(grid[1], thread[2], thread[4])
@prism("global")
def thread_named_twice(n: int @ grid[1]):
    t: int @ thread[1] = id()


@requires(block[1], thread[1])
@prism("device")
def control_at_the_bound(n: int @ block[1]):
    t: int @ thread[1] = id()
    if n > 3:                                       # block value, block bound
        for i in range(n):
            t = t + i
    with group(thread[1]):
        if t > n:                                   # thread value under a thread bound
            while t > 0:
                t = t - 1
    return


@requires(block[1], thread[1])
@prism("device")
def thread_condition_at_block_level(n: int @ block[1]):
    t: int @ thread[1] = id()
    if t > n:
        t = 0
    return


@requires(block[1], thread[1])
@prism("device")
def thread_range_at_block_level(n: int @ block[1]):
    t: int @ thread[1] = id()
    for i in range(t):
        n = n
    return


@requires(block[1], thread[1])
@prism("device")
def thread_while_at_block_level(n: int @ block[1]):
    t: int @ thread[1] = id()
    while t > 0:
        n = n
    return


@requires(block[1], thread[1])
@prism("device")
def loop_over_a_list(n: int @ block[1]):
    for i in [1, 2, 3]:
        n = n
    return


def test_requires_and_control_flow():
    with pytest.raises(PerspectiveError, match="missing @requires"):
        check("no_requires")
    with pytest.raises(PerspectiveError, match="names thread twice"):
        check("thread_named_twice")
    sig = signature("control_at_the_bound")
    assert (sig.bound.grid, str(sig.bound.block), str(sig.bound.thread)) == (None, "block[1]", "thread[1]")
    for name, what in (("thread_condition_at_block_level", "condition of this `if` is at thread\\[1\\]"),
                       ("thread_range_at_block_level", "range of this loop is at thread\\[1\\]"),
                       ("thread_while_at_block_level", "condition of this `while` is at thread\\[1\\]"),
                       ("loop_over_a_list", "range")):
        with pytest.raises(PerspectiveError, match=what):
            check(name)


# --------------------------------------------------------------------- groups --

@requires(grid[1], block[1], thread[8])
@prism("global")
def groups_go_down(n: int @ grid[1]):
    with group(block[1]):
        with group(thread[4]):
            with group(thread[2]):
                with group(thread[1]):
                    t: int @ thread[1] = id()


@requires(grid[1], block[1], thread[4])
@prism("global")
def group_wider_than_the_bound(n: int @ grid[1]):
    with group(thread[8]):
        t: int @ thread[1] = id()


@requires(grid[1], block[1], thread[4])
@prism("global")
def group_back_up(n: int @ grid[1]):
    with group(thread[1]):
        with group(block[1]):
            t: int @ thread[1] = id()


@requires(grid[1], block[1], thread[6])
@prism("global")
def group_that_does_not_divide(n: int @ grid[1]):
    with group(thread[4]):
        t: int @ thread[1] = id()


def test_groups_only_narrow_the_bound():
    check("groups_go_down")
    with pytest.raises(PerspectiveError, match="cannot enter group\\(thread\\[8\\]\\)"):
        check("group_wider_than_the_bound")
    with pytest.raises(PerspectiveError, match="cannot enter group\\(block\\[1\\]\\).*gone"):
        check("group_back_up")
    with pytest.raises(PerspectiveError, match="cannot enter group\\(thread\\[4\\]\\)"):
        check("group_that_does_not_divide")


# ---------------------------------------------------------------------- views --

@requires(grid[1], block[1], thread[1])
@prism("global")
def views_step_by_step(x: ptr(int) @ grid[1], n: int @ grid[1]):
    b: int @ block[1] = id()
    with partition(x, p=block[1], offset=b * n) as x_blk:
        with group(block[1]):
            t: int @ thread[1] = id()
            with partition(x_blk, p=thread[1], f=lambda i: 2 * i + t) as x_mine:
                with group(thread[1]):
                    x_mine[0] = b


@requires(grid[1], block[1], thread[1])
@prism("global")
def view_with_a_narrow_offset(x: ptr(int) @ grid[1]):
    t: int @ thread[1] = id()
    with partition(x, p=block[1], offset=t) as x_blk:
        with group(block[1]):
            n: int @ block[1] = x_blk[0]


@requires(grid[1], block[1], thread[1])
@prism("global")
def view_taken_too_deep(x: ptr(int) @ grid[1]):
    with group(block[1]):
        t: int @ thread[1] = id()
        with partition(x, p=thread[1], offset=t) as x_mine:
            x_mine[0] = 0


@requires(grid[1], block[1], thread[1])
@prism("global")
def view_taken_twice(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1], offset=0) as a:
        with partition(x, p=block[1], offset=1) as b:
            with group(block[1]):
                n: int @ block[1] = a[0] + b[0]


@requires(grid[1], block[1], thread[1])
@prism("global")
def view_taken_again_afterwards(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1], offset=0) as a:
        with group(block[1]):
            n: int @ block[1] = a[0]
    with partition(x, p=block[1], offset=1) as b:
        with group(block[1]):
            m: int @ block[1] = b[0]


@requires(grid[1], block[1], thread[1])
@prism("global")
def view_broader_than_its_pointer(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            with partition(x_blk, p=grid[1], offset=0) as up:
                n: int @ block[1] = up[0]


@requires(grid[1], block[1], thread[1])
@prism("global")
def view_of_a_private_array(x: ptr(int) @ grid[1]):
    with group(block[1]):
        with group(thread[1]):
            held: int[4] @ thread[1] = {0}
            with partition(held, p=thread[1], offset=1) as later:
                later[0] = 1


@requires(grid[1], block[1], thread[1])
@prism("global")
def view_without_an_offset(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1]) as x_blk:
        with group(block[1]):
            n: int @ block[1] = x_blk[0]


def test_partition_rules():
    check("views_step_by_step")
    check("view_taken_again_afterwards")
    for name, what in (("view_with_a_narrow_offset", "offset of view 'x_blk' is at thread\\[1\\]"),
                       ("view_taken_too_deep", "'x' lives at grid\\[1\\] but the broadest perspective here is block\\[1\\]"),
                       ("view_taken_twice", "'x' is already partitioned"),
                       ("view_broader_than_its_pointer", "cannot be narrowed to grid\\[1\\]"),
                       ("view_of_a_private_array", "private array"),
                       ("view_without_an_offset", "needs f= or offset=")):
        with pytest.raises(PerspectiveError, match=what):
            check(name)


# ------------------------------------------------------------ split and claim --

@requires(grid[1], block[1], thread[256])
@prism("global")
def producer_and_consumers(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            with claim(x_blk, p=thread[128]) as first_half:
                match split(thread):
                    case 128:
                        with group(thread[128]):
                            t: int @ thread[1] = id()
                            with partition(first_half, p=thread[1], offset=t) as mine:
                                with group(thread[1]):
                                    mine[0] = t
                    case 64:
                        with group(thread[64]):
                            w: int @ thread[64] = id()
                    case 64:
                        u: int @ thread[1] = id()


@requires(grid[1], block[1], thread[128])
@prism("global")
def split_asks_for_too_many(x: ptr(int) @ grid[1]):
    with group(block[1]):
        match split(thread):
            case 96:
                t: int @ thread[1] = id()
            case 64:
                u: int @ thread[1] = id()


@requires(grid[1], block[1], thread[128])
@prism("global")
def claim_used_outside_a_split(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            with claim(x_blk, p=thread[64]) as part:
                n: int @ thread[64] = part[0]


@requires(grid[1], block[1], thread[128])
@prism("global")
def claim_used_in_two_cases(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            with claim(x_blk, p=thread[64]) as part:
                match split(thread):
                    case 64:
                        a: int @ thread[64] = part[0]
                    case 64:
                        b: int @ thread[64] = part[1]


@requires(grid[1], block[1], thread[128])
@prism("global")
def claim_at_the_same_perspective(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            with claim(x_blk, p=block[1]) as part:
                match split(thread):
                    case 64:
                        a: int @ thread[64] = part[0]


@requires(grid[1], block[1], thread[128])
@prism("global")
def same_view_taken_in_two_cases(x: ptr(int) @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            with partition(x_blk, p=thread[64], offset=0) as x_part:
                match split(thread):
                    case 64:
                        with partition(x_part, p=thread[1], offset=0) as a:
                            n: int @ thread[1] = a[0]
                    case 64:
                        with partition(x_part, p=thread[1], offset=64) as b:
                            m: int @ thread[1] = b[0]


def test_split_and_claim_rules():
    check("producer_and_consumers")
    with pytest.raises(PerspectiveError, match="case 64 of split\\(thread\\): only 32 of thread\\[128\\] are left"):
        check("split_asks_for_too_many")
    with pytest.raises(PerspectiveError, match="claimed view 'part' is only accessed inside a case of a split"):
        check("claim_used_outside_a_split")
    with pytest.raises(PerspectiveError, match="claimed view 'part' is accessed in more than one case"):
        check("claim_used_in_two_cases")
    with pytest.raises(PerspectiveError, match="cannot be narrowed to block\\[1\\]"):
        check("claim_at_the_same_perspective")
    check("same_view_taken_in_two_cases")   # a view ends with its `with`; the next case may take its own


# ------------------------------------------------------------------------ LDS --

@requires(grid[1], block[1], thread[1], smem=1024)
@prism("global")
def lds_within_budget(x: ptr(int) @ grid[1]):
    with group(block[1]):
        a: shared(int[128]) @ block[1]
        b: shared(float[64], static=True) @ block[1]
        c: shared(int[64]) @ block[1]


@requires(grid[1], block[1], thread[1], smem=1024)
@prism("global")
def lds_over_budget(x: ptr(int) @ grid[1]):
    with group(block[1]):
        a: shared(int[128]) @ block[1]
        b: shared(int[2 * 64 + 1]) @ block[1]


@requires(grid[1], block[1], thread[1])
@prism("global")
def lds_per_thread(x: ptr(int) @ grid[1]):
    with group(block[1]):
        a: shared(int[128]) @ thread[1]


def test_lds_declarations():
    check("lds_within_budget")
    with pytest.raises(PerspectiveError, match="'b' needs 516 bytes, 512 are left"):
        check("lds_over_budget")
    with pytest.raises(PerspectiveError, match="'a' is declared at thread\\[1\\]; shared memory lives at block\\[1\\]"):
        check("lds_per_thread")


# ---------------------------------------------------------------------- calls --

@requires(block[1], thread[1])
@prism("device")
def block_helper(dst: ptr(int) @ block[1], src: ptr(const(int)) @ block[1], n: int @ block[1]) -> int @ block[1]:
    with group(block[1]):
        t: int @ thread[1] = id()
        with partition(dst, p=thread[1], offset=t) as mine:
            with group(thread[1]):
                if t < n:
                    mine[0] = src[t]
    return n


@requires(thread[1])
@prism("device")
def returns_too_narrow(n: int @ thread[1]) -> int @ thread[4]:
    return n


@requires(grid[1], block[1], thread[1])
@prism("global")
def calls_with_matching_arguments(x: ptr(int) @ grid[1], y: ptr(const(int)) @ grid[1], n: int @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            got: int @ block[1] = block_helper(x_blk, y, n)      # const pointer and scalar may come from above
            t: int @ thread[1] = got                                 # the result is a block value


@requires(grid[1], block[1], thread[1])
@prism("global")
def passes_a_grid_pointer_for_a_block_one(x: ptr(int) @ grid[1], y: ptr(const(int)) @ grid[1], n: int @ grid[1]):
    with group(block[1]):
        block_helper(x, y, n)


@requires(grid[1], block[1], thread[1])
@prism("global")
def passes_a_thread_value_for_a_block_one(x: ptr(int) @ grid[1], y: ptr(const(int)) @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            t: int @ thread[1] = id()
            block_helper(x_blk, y, t)


@requires(grid[1], block[1], thread[1])
@prism("global")
def calls_from_too_deep(x: ptr(int) @ grid[1], y: ptr(const(int)) @ grid[1], n: int @ grid[1]):
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            with group(thread[1]):
                block_helper(x_blk, y, n)


@requires(grid[1], block[1], thread[1])
@prism("global")
def result_into_a_broader_variable(x: ptr(int) @ grid[1], y: ptr(const(int)) @ grid[1], n: int @ grid[1]):
    m: int @ grid[1] = 0
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            m = block_helper(x_blk, y, n)


def test_call_rules():
    check("calls_with_matching_arguments")
    with pytest.raises(PerspectiveError, match="block_helper\\(dst=...\\) takes a pointer at exactly block\\[1\\], got grid\\[1\\]"):
        check("passes_a_grid_pointer_for_a_block_one")
    with pytest.raises(PerspectiveError, match="block_helper\\(n=...\\) is at block\\[1\\]; the argument at thread\\[1\\] is narrower"):
        check("passes_a_thread_value_for_a_block_one")
    with pytest.raises(PerspectiveError, match="block_helper requires block\\[1\\]; the caller is at no block level"):
        check("calls_from_too_deep")
    with pytest.raises(PerspectiveError, match="'m' at grid\\[1\\] cannot take a value at block\\[1\\]"):
        check("result_into_a_broader_variable")
    with pytest.raises(PerspectiveError, match="returns a value at thread\\[1\\]"):
        check("returns_too_narrow")
