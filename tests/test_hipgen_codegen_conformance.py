"""The printed text for the constructs the reference's code-generator tests cover (test/test_codegen.py), one
small program of this repository's own per construct.

The HIP back-end keeps the reference's calling convention and naming for what is not target-specific: a device
function takes `__block_id, __thread_id, __smem` in front of its own parameters (prism/codegen.py:328-337),
every group / split level declares `__block_id_k` / `__thread_id_k` (the k-th nesting level), `id()` is the id
of the enclosing level divided by the perspective's index (prism/codegen.py:149-160), and an f=lambda view
rewrites each access instead of declaring a pointer (prism/codegen.py:862-880). The fragments asserted here are
the ones the reference's tests assert on its CUDA text; they hold verbatim for the HIP text. CPU only.
"""
from prism_amd.hipgen import (block, claim, const, constexpr, double, grid, group, partition, prism, ptr, requires,
                              restrict, shared, split, thread)
from prism_amd.hipgen_blocks import generate_blocks


@requires(grid[1], block[4], thread[4])
@prism("global")
def k_global(x: ptr(int) @ thread[1], n: int @ grid[1]):
    pass

@requires(block[1], thread[4])
@prism("device")
def k_device(x: ptr(int) @ thread[1]):
    pass

@requires(block[1], thread[1])
@prism("device")
def k_ptrs(a: ptr(float) @ thread[1], b: const(ptr(int)) @ thread[1], c: restrict(ptr(double)) @ thread[1]):
    pass

@requires(block[1], thread[1])
@prism("device")
def k_tmpl(x: int @ thread[1], template=[("N", int), ("M", constexpr(int))]):
    pass

@requires(block[1], thread[1])
@prism("device")
def k_ret(x: int @ thread[1]) -> int @ thread[1]:
    return x

@requires(block[1], thread[1])
@prism("device")
def k_decls(x: int @ thread[1], y: int @ thread[1]):
    a: int @ thread[1] = 42
    b: int @ thread[1]
    buf: int[16] @ thread[1]
    z: int @ thread[1] = x + y * 2
    f: bool @ thread[1] = True

@requires(grid[1], block[1], thread[1], smem=2048)
@prism("device")
def k_smem():
    a: shared(int[64]) @ block[1]
    b: shared(float[32]) @ block[1]

@requires(grid[1], block[4], thread[4])
@prism("device")
def k_ids():
    x: int @ thread[1] = id()
    y: int @ block[4] = id()

@requires(block[1], thread[1])
@prism("device")
def k_flow(n: int @ block[1]):
    for i in range(n):
        if n > 5:
            break
        if n > 3:
            continue
    for j in range(1, 10):
        pass
    for k in range(0, 100, 4):
        pass
    if n > 10:
        n = 1
    elif n > 5:
        n = 2
    else:
        n = 3

@requires(thread[1])
@prism("device")
def k_while(x: int @ thread[1]):
    while x > 0:
        x = x - 1

@requires(grid[1], block[4], thread[8])
@prism("device")
def k_groups():
    with group(block[2]):
        a: int @ block[2] = id()
        with group(thread[4]):
            b: int @ thread[4] = id()

@requires(grid[1], block[8], thread[8])
@prism("device")
def k_split_blocks():
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

@requires(grid[1], block[1], thread[4])
@prism("device")
def k_split_threads():
    match split(thread):
        case 2:
            pass
        case 2:
            pass

@requires(grid[1], block[1], thread[1])
@prism("device")
def k_part(data: ptr(int) @ grid[1], n: int @ grid[1]):
    with partition(data, p=thread[1], offset=id() * n) as mine:
        mine[0] = 42
    with partition(data, p=thread[1], f=lambda i: i + id() * n) as view:
        view[0] = 42
        x: int @ thread[1] = view[3]
        view[0] += 1

@requires(block[1], thread[1])
@prism("device")
def callee_off(x: ptr(int) @ thread[1]):
    pass

@requires(block[1], thread[1])
@prism("device")
def callee_tmpl(x: int @ thread[1], template=[("N", int)]):
    pass

@requires(grid[1], block[1], thread[1])
@prism("device")
def k_calls(data: ptr(int) @ grid[1], n: int @ grid[1]):
    with partition(data, p=thread[1], offset=id() * n) as mine:
        callee_off(mine)
    callee_tmpl(n, template=[16])

@requires(block[4], thread[1])
@prism("device")
def k_claim(data: ptr(int) @ block[4]):
    with claim(data, p=thread[1]) as mine:
        match split(block):
            case 2:
                x: int @ thread[1] = mine[0]
            case 2:
                pass

@requires(thread[1])
@prism("global")
def vec_sum(a: ptr(float) @ thread[1], b: ptr(float) @ thread[1], c: ptr(float) @ thread[1], n: int @ thread[1]):
    i: int @ thread[1] = id()
    if i < n:
        c[i] = a[i] + b[i]


def test_function_signatures():
    text = generate_blocks("k_global")
    assert "__global__ void k_global(int* x, int n)" in text
    assert "extern __shared__ __align__(128) char __smem[];" in text and "blockIdx.x" in text and "blockDim.x" in text
    text = generate_blocks("k_device")
    assert "__device__" in text and "int __block_id, int __thread_id, char* __smem, int* x" in text
    assert "__block_id_0 = __block_id;" in text and "__thread_id_0 = __thread_id;" in text
    text = generate_blocks("k_ptrs")
    assert "float* a" in text and "const int* b" in text and "double* __restrict__ c" in text
    text = generate_blocks("k_tmpl")  # a template parameter is no function parameter; constexpr(int) prints as int
    assert "template<int N, int M>" in text and "int __block_id, int __thread_id, char* __smem, int x)" in text
    text = generate_blocks("k_ret")
    assert "__device__ int k_ret(" in text and "return x;" in text


def test_declarations_and_expressions():
    text = generate_blocks("k_decls")
    for line in ("int a = 42;", "int b;", "int buf[16];", "int z = (x + (y * 2));", "bool f = true;"):
        assert line in text
    text = generate_blocks("k_smem")  # LDS arrays are carved out of __smem one after the other
    assert "int (&a)[64]" in text and "__smem + 0" in text and "__smem + 256" in text
    text = generate_blocks("k_ids")
    assert "int x = __thread_id_0;" in text and "int y = (__block_id_0 / 4);" in text


def test_control_flow():
    text = generate_blocks("k_flow")
    for line in ("for (int i = 0; i < n; i++)", "for (int j = 1; j < 10; j++)", "for (int k = 0; k < 100; k += 4)",
                 "break;", "continue;", "if ((n > 10))", "} else if ((n > 5))", "} else {"):
        assert line in text
    text = generate_blocks("k_while")
    assert "while ((x > 0))" in text and "x = (x - 1);" in text


def test_groups_and_splits_renumber_the_ids():
    text = generate_blocks("k_groups")
    assert "__block_id_1 = __block_id_0 % 2;" in text
    assert "__thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;" in text
    assert "__block_id_2 = __block_id_1;" in text and "__thread_id_2 = __thread_id_1 % 4;" in text
    text = generate_blocks("k_split_blocks")  # cases of 2, 2 and 4 blocks: offsets 0, 2 and 4
    assert "__block_id_1 = __block_id_0;" in text and "__block_id_1 >= 0 && __block_id_1 < 2" in text
    assert "__block_id_1 = __block_id_0 - 2;" in text and "__block_id_1 = __block_id_0 - 4;" in text
    assert "__block_id_1 < 4" in text
    text = generate_blocks("k_split_threads")
    assert "__thread_id_1 = __thread_id_0;" in text and "__thread_id_1 >= 0 && __thread_id_1 < 2" in text
    assert "__thread_id_1 = __thread_id_0 - 2;" in text


def test_partitions_and_claims():
    text = generate_blocks("k_part")
    assert "int* mine = data + (" in text and "mine[0] = 42;" in text      # offset=: a pointer
    assert "int* view" not in text                                          # f=lambda: every access is rewritten,
    assert "data[(0 + (__thread_id_0 * n))] = 42;" in text                  # and id() inside the lambda is the id
    assert "int x = data[(3 + (__thread_id_0 * n))];" in text               # at the view's own perspective
    assert "data[(0 + (__thread_id_0 * n))] += 1;" in text
    text = generate_blocks("k_claim")
    assert "int* mine = data + (0);" in text


def test_calls_pass_the_ids_on():
    text = generate_blocks("k_calls")
    assert "callee_off(__block_id_0, __thread_id_0, __smem, mine);" in text
    assert "callee_tmpl<16>(__block_id_0, __thread_id_0, __smem, n);" in text


def test_a_whole_kernel():
    text = generate_blocks("vec_sum")
    assert "__global__" in text and "float* a, float* b, float* c, int n" in text
    assert "int i = __thread_id_0;" in text and "if ((i < n))" in text and "c[i] = (a[i] + b[i]);" in text
