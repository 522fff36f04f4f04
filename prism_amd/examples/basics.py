"""Small programs, one per construct: a device function called from a kernel (examples/function_call.py), two
roles in one workgroup through `match split` (the producer / consumer split of examples/h100_matmul.py:203-206),
and index-mapped views stacked on one another (partition with f=lambda, prism/codegen.py:816-826).
"""
from prism_amd.hipgen import block, const, grid, group, partition, prism, ptr, requires, split, thread


@requires(thread[1])
@prism("device")
def scaled_sum(a: float @ thread[1], b: float @ thread[1], s: float @ thread[1]) -> float @ thread[1]:
    return s * (a + b)


@requires(grid[1], block[1], thread[1])
@prism("global")
def scaled_sum_all(x: ptr(const(float)) @ grid[1], y: ptr(float) @ grid[1], s: float @ grid[1], n: int @ grid[1]):
    i: int @ thread[1] = id()  # outside every group: the thread's number in the whole grid
    with partition(y, p=thread[1], offset=i) as y_one:
        with group(block[1]):
            with group(thread[1]):
                if i < n:
                    y_one[0] = scaled_sum(x[i], y_one[0], s)


@requires(grid[1], block[1], thread[256])
@prism("global")
def two_roles(x: ptr(const(int)) @ grid[1], y: ptr(int) @ grid[1], n: int @ grid[1]):
    """The first 128 threads of a block double their element, the next 128 add one to theirs (the shape of
    the reference's producer / consumer split, examples/h100_matmul.py:203-206)."""
    base: int @ block[1] = id() * 256
    with partition(y, p=thread[1], offset=base) as y_mine:
        with group(block[1]):
            match split(thread):
                case 128:
                    t: int @ thread[1] = id()
                    with group(thread[1]):
                        if base + t < n:
                            y_mine[t] = x[base + t] * 2
                case 128:
                    t: int @ thread[1] = id()
                    with group(thread[1]):
                        if base + 128 + t < n:
                            y_mine[128 + t] = x[base + 128 + t] + 1


@requires(grid[1], block[1], thread[1])
@prism("global")
def gather_columns(x: ptr(const(int)) @ grid[1], y: ptr(int) @ grid[1], rows: int @ grid[1], cols: int @ grid[1]):
    """y = x transposed, written through two stacked index-mapped views: `column` picks every cols-th element
    starting at the thread's column, `shifted` skips its first element; thread c writes column c."""
    c: int @ thread[1] = id()
    with partition(x, p=thread[1], f=lambda r: r * cols + c) as column:
        with partition(y, p=thread[1], offset=c * rows) as mine:
            with group(block[1]):
                with group(thread[1]):
                    with partition(column, p=thread[1], f=lambda r: r + 1) as shifted:
                        if c < cols:
                            mine[0] = column[0]
                            for r in range(rows - 1):
                                mine[r + 1] = shifted[r]
