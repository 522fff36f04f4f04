"""The HIP emitter for Prism kernels with block-level structure (prism_amd/hipgen_blocks.py).

The programs are the example set under prism_amd/examples (add_m, the SGEMM steps, matrix-instruction kernels,
the row scan, small one-construct programs), written in the reference's surface syntax; the few kernels defined
here exist to be refused or to probe one rule of the barrier plan.
CPU: structure of the printed text (id chain, scopes, LDS declarations, where the barriers land), refusals
by name, and that every launcher cross-compiles for gfx950.
GPU: the compiled kernels run through their C launchers; add_m bit for bit against numpy, the SGEMMs
within 1e-5 * sqrt(K) * max|A| * max|B| of the fp64 oracle (the compiler is free to contract a * b + c).
"""
import ctypes

import numpy as np
import pytest

from prism_amd import hipgen
from prism_amd.examples import add_m, basics, mfma, scan, sgemm  # noqa: F401  (define the kernels)
from prism_amd.hipgen import (HipgenError, block, const, generate, generate_launcher, grid, group, intrinsic, partition, prism,
                              ptr, requires, shared, split, thread)
from prism_amd.hipgen_blocks import dynamic_lds_bytes, explain_barriers


@requires(grid[1], block[1], thread[1])
@prism("global")
def hazard_in_branch(x: ptr(float) @ grid[1]):
    with partition(x, p=thread[1], offset=0) as x_mine:
        with group(block[1]):
            buf: shared(float[64], static=True) @ block[1]
            t: int @ thread[1] = id()
            with partition(buf, p=thread[1], offset=t) as slot:
                with group(thread[1]):
                    if t < 32:
                        slot[0] = x_mine[t]
                        x_mine[t] = buf[31 - t]


@requires(grid[1], block[1], thread[128])
@prism("global")
def split_with_hazard(x: ptr(float) @ grid[1]):
    with partition(x, p=thread[1], offset=0) as x_mine:
        with group(block[1]):
            buf: shared(float[256], static=True) @ block[1]
            with partition(buf, p=thread[1], offset=0) as buf_mine:
                match split(thread):
                    case 128:
                        t: int @ thread[1] = id()
                        with group(thread[1]):
                            buf_mine[t] = x_mine[t]
                            x_mine[t] = buf[127 - t]


@requires(grid[1], block[1], thread[1])
@prism("global")
def hazard_in_uniform_branch(x: ptr(float) @ grid[1], rounds: int @ grid[1]):
    """The same write-then-read of LDS, inside an `if` on which all threads of a workgroup agree (a loop variable
    over a grid-level range against a grid-level parameter), reversed once per round."""
    with partition(x, p=thread[1], offset=0) as x_mine:
        with group(block[1]):
            buf: shared(float[64], static=True) @ block[1]
            t: int @ thread[1] = id()
            with partition(buf, p=thread[1], offset=t) as slot:
                with group(thread[1]):
                    for r in range(rounds):
                        if r % 2 == 0:
                            slot[0] = x_mine[t]
                            x_mine[t] = buf[63 - t]
                        intrinsic.sched_group("barrier")


@requires(grid[1], block[1], thread[48])
@prism("global")
def straddling_groups(x: ptr(float) @ grid[1]):
    with group(block[1]):
        with group(thread[48]):
            w: int @ thread[48] = id()


@requires(grid[1], block[1], thread[1])
@prism("global")
def view_without_address(x: ptr(int) @ grid[1]):
    with partition(x, p=thread[1], f=lambda i: 2 * i) as evens:
        with group(block[1]):
            with group(thread[1]):
                with partition(evens, p=thread[1], offset=4) as later:
                    later[0] = 1


@requires(grid[1], block[1], thread[64])
@prism("global")
def foreign_instruction(x: ptr(float) @ grid[1]):
    a: float @ thread[1] = 0
    intrinsic.mma(a, a, a, a, a, a, a, a, a, a, out=[a, a, a, a])


@requires(grid[1], block[1], thread[1])
@prism("global")
def two_readers(x: ptr(const(float)) @ grid[1], y: ptr(float) @ grid[1], template=[("BM", int), ("BN", int), ("BK", int)]):
    """One fill, then two calls that take the tiles as pointers to const: a barrier in front of the first only."""
    with partition(x, p=block[1], offset=0) as x_blk:
        with group(block[1]):
            a_lds: shared(float[1024], static=True) @ block[1]
            b_lds: shared(float[1024], static=True) @ block[1]
            acc: float[16] @ thread[1] = {0}
            stage_tiles(BN, BK, x_blk, x_blk, a_lds, b_lds, template=[BM, BN, BK, 256])
            multiply_tiles(acc, a_lds, b_lds, 0, 0, template=[BM, BN, BK, 4, 4])
            multiply_tiles(acc, b_lds, a_lds, 0, 0, template=[BM, BN, BK, 4, 4])
            stage_tiles(BN, BK, x_blk, x_blk, a_lds, b_lds, template=[BM, BN, BK, 256])


def lines(text):
    return [ln.strip() for ln in text.splitlines()]


def test_id_chain_and_scopes_of_a_block_thread_kernel():
    text = generate("add_m_blocks")
    got = lines(text)
    assert got[0] == "__global__ void add_m_blocks(const int* x, int* y, int m, int per_block, int n) {"
    assert got[1:4] == ["extern __shared__ __align__(128) char __smem[];", "int __block_id_0 = blockIdx.x;",
                        "int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;"]
    assert "int first = (__block_id_0 * per_block);" in got
    assert "const int* x_blk = x + (first);" in got and "int* y_blk = y + (first);" in got
    # group(block[1]) opens depth 1: the thread id inside it is the id within the block
    i = got.index("int __block_id_1 = __block_id_0 % 1;")
    assert got[i + 1] == "int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;"
    assert got[i + 2] == "int lane = __thread_id_1;"
    j = got.index("int __block_id_2 = __block_id_1;")
    assert got[j + 1] == "int __thread_id_2 = __thread_id_1 % 1;"
    assert "if (((first + lane) < n)) {" in got and "y_one[0] = (x_one[0] + m);" in got
    assert text.count("{") == text.count("}") and "__syncthreads();" not in got


def test_loops_guards_and_expressions():
    got = lines(generate("naive_sgemm"))
    assert "int e = ((blk * per_block) + __thread_id_1);" in got
    assert "const int row = (e / N);" in got and "const int col = (e % N);" in got
    assert "for (int k = 0; k < K; k++) {" in got
    assert "acc += (A[((row * K) + k)] * B[((k * N) + col)]);" in got
    assert "C_mine[((row * N) + col)] = ((alpha * acc) + (beta * C_mine[((row * N) + col)]));" in got


def test_barriers_of_the_lds_tiled_kernel():
    """Stores into both LDS tiles, barrier, the dot-product loop that reads them, barrier at the end of the
    K loop's body (the next iteration overwrites what this one read): the two barriers the reference
    prints for its LDS-tiled example (generated/sgemm_shared_mem_block.cu:38,42)."""
    got = lines(generate("tiled_sgemm"))
    assert got[0] == "template<int TILE>"
    assert "__shared__ float a_lds[(TILE * TILE)];" in got and "__shared__ float b_lds[(TILE * TILE)];" in got
    assert got.count("__syncthreads();") == 2
    first = got.index("__syncthreads();")
    assert got[first - 1].startswith("b_mine[") and got[first + 1] == "for (int d = 0; d < TILE; d++) {"
    second = got.index("__syncthreads();", first + 1)
    # the d loop, the thread group and the two views close; the barrier is the last statement of the k0 loop
    assert got[second - 4:second] == ["}"] * 4 and got[second + 1] == "}"
    assert got[second + 3].startswith("float* C_mine = C_tile + ")
    assert "for (int k0 = 0; k0 < K; k0 += TILE) {" in got
    assert "__syncthreads();" not in lines(generate("tiled_sgemm", auto_sync=False))


@requires(grid[1], block[1], thread[1])
@prism("global")
def maybe_no_trips(x: ptr(const(int)) @ grid[1], y: ptr(int) @ grid[1], trips: int @ grid[1]):
    a: shared(int[64], static=True) @ block[1]
    b: shared(int[64], static=True) @ block[1]
    with partition(y, p=thread[1], offset=0) as y_mine:
        with group(block[1]):
            t: int @ thread[1] = id()
            with partition(a, p=thread[1], offset=t) as a_one:
                with partition(b, p=thread[1], offset=t) as b_one:
                    with group(thread[1]):
                        a_one[0] = x[t]
                        for i in range(trips):
                            b_one[0] = i
                            y_mine[t] = b[63 - t]
                        y_mine[t] = a[63 - t]


@requires(grid[1], block[1], thread[1])
@prism("global")
def surely_some_trips(x: ptr(const(int)) @ grid[1], y: ptr(int) @ grid[1]):
    a: shared(int[64], static=True) @ block[1]
    b: shared(int[64], static=True) @ block[1]
    with partition(y, p=thread[1], offset=0) as y_mine:
        with group(block[1]):
            t: int @ thread[1] = id()
            with partition(a, p=thread[1], offset=t) as a_one:
                with partition(b, p=thread[1], offset=t) as b_one:
                    with group(thread[1]):
                        a_one[0] = x[t]
                        for i in range(3):
                            b_one[0] = i
                            y_mine[t] = b[63 - t]
                        y_mine[t] = a[63 - t]


def test_a_loop_that_may_not_run_keeps_what_was_pending_in_front_of_it():
    """A write of `a`, a loop with a run-time trip count whose body only touches `b` (and gets its own two
    barriers), then a cross-thread read of `a`. With zero trips none of the loop's barriers runs, so the
    read needs a barrier of its own behind the loop. With a literal trip count of at least one the
    barriers inside the loop are sure to run and order the write of `a` as well: no third barrier."""
    got = lines(generate("maybe_no_trips"))
    read = got.index("y_mine[t] = a[(63 - t)];")
    assert got[read - 1] == "__syncthreads();" and got[read - 2] == "}"
    assert got.count("__syncthreads();") == 3
    got = lines(generate("surely_some_trips"))
    read = got.index("y_mine[t] = a[(63 - t)];")
    assert got[read - 1] == "}" and got.count("__syncthreads();") == 2


def test_barriers_between_device_functions_that_are_handed_the_tiles():
    """Filling call, barrier, reading call, and a barrier as the last statement of the K loop's body: where the
    reference prints them for its kernel 5 (generated/my_sgemm_kernel_5.cu:40-46). What a call does to an LDS
    array it is handed is read off the callee's signature: a pointer to const is only read, any other pointer
    may be written (prism/sync_analysis.py:871-877)."""
    got = lines(generate("staged_sgemm"))
    assert got[0] == "template<int BM, int BN, int BK, int TM, int TN, int THREADS>"
    fill = got.index("stage_tiles<BM, BN, BK, THREADS>(__block_id_1, __thread_id_1, __smem, N, K, A_now, B_now, a_lds, b_lds);")
    assert got[fill + 1] == "__syncthreads();"
    assert got[fill + 2] == ("multiply_tiles<BM, BN, BK, TM, TN>(__block_id_1, __thread_id_1, __smem, acc, a_lds, b_lds, "
                             "out_r, out_c);")
    assert got[fill + 3:fill + 7] == ["}", "}", "__syncthreads();", "}"]   # the two views close, barrier, the loop closes
    assert got.count("__syncthreads();") == 2
    # the callees' own text: stores through thread[1] views of the pointer parameters, no barrier of their own
    filler = lines(generate("stage_tiles"))
    assert filler[0] == "template<int BM, int BN, int BK, int THREADS>"
    assert filler[1] == ("__device__ void stage_tiles(int __block_id, int __thread_id, char* __smem, int N, int K, "
                         "const float* A_from, const float* B_from, float* a_tile, float* b_tile) {")
    assert "float* a_mine = a_tile + (0);" in filler and "__syncthreads();" not in filler
    # two readers in a row need nothing between them; the fill behind them does
    got = lines(generate("two_readers"))
    calls = [n for n, ln in enumerate(got) if ln.startswith(("stage_tiles<", "multiply_tiles<"))]
    sync = [n for n, ln in enumerate(got) if ln == "__syncthreads();"]
    assert len(calls) == 4 and sync == [calls[0] + 1, calls[3] - 1] and calls[2] == calls[1] + 1


def test_every_barrier_can_say_what_it_is_for():
    from prism_amd.hipgen_blocks import explain_barriers
    assert explain_barriers("staged_sgemm") == [
        "line 27 reads a_lds, b_lds (written since the last barrier)",
        "the next trip of the loop writes a_lds, b_lds (read since the last barrier)"]
    got = lines(generate("tiled_sgemm", annotate=True))
    first = got.index("__syncthreads();")
    assert got[first - 1] == "// line 23 reads a_lds, b_lds (written since the last barrier)"
    assert not any(ln.startswith("//") for ln in lines(generate("tiled_sgemm")))   # only on request


def test_dynamic_lds_windows_private_arrays_and_attr():
    text = generate("thread_tile_sgemm")
    got = lines(text)
    assert got[0] == "template<int BM, int BN, int BK, int TM, int TN>"
    assert got[1].startswith("__global__ __launch_bounds__((BM * BN) / (TM * TN)) void thread_tile_sgemm(")
    assert "float (&a_lds)[1024] = *((float (*)[1024])(__smem + 0));" in got
    assert "float (&b_lds)[1024] = *((float (*)[1024])(__smem + 4096));" in got
    assert dynamic_lds_bytes("thread_tile_sgemm") == 8192
    assert "float acc[16] = {0};" in got and "float a_reg[4] = {0};" in got
    assert "for (int e = t; e < (BM * BK); e += threads) {" in got
    # one barrier between the two staging loops and the compute loop, one before the next K step
    assert got.count("__syncthreads();") == 2
    first = got.index("__syncthreads();")
    assert got[first + 1] == "for (int kk = 0; kk < BK; kk++) {"
    launcher = generate_launcher("thread_tile_sgemm", block_size=256, template=[64, 64, 8, 4, 4])
    assert "thread_tile_sgemm<64, 64, 8, 4, 4><<<dim3(grid_blocks), dim3(256), 8192," in launcher
    with pytest.raises(HipgenError, match="template parameters"):
        generate_launcher("thread_tile_sgemm", block_size=256)


def test_vector_casts_and_index_mapped_views():
    got = lines(generate("vector_tile_sgemm"))
    assert "float4 quad = reinterpret_cast<float4 *>(&A_rows[(((a_row * K) + k0) + (a_quad * 4))])[0];" in got
    # the view declares no pointer; its elements are elements of a_lds at the mapped index
    assert not any("a_by_row" in ln for ln in got)
    e = "(((a_row * BK) + (a_quad * 4)) + 1)"
    assert f"a_lds[((({e} % BK) * BM) + ({e} / BK))] = quad.y;" in got
    assert ("reinterpret_cast<float4 *>(&b_lds[((b_row * BN) + (b_quad * 4))])[0] = "
            "reinterpret_cast<float4 *>(&B_cols[(((k0 + b_row) * N) + (b_quad * 4))])[0];") in got
    assert "float4 was = reinterpret_cast<float4 *>(&c4[0])[0];" in got
    assert "was.w = ((alpha * acc[(((i * TN) + j) + 3)]) + (beta * was.w));" in got
    assert "reinterpret_cast<float4 *>(&c4[0])[0] = was;" in got
    # stores through the cast and through the view count as writes of the LDS arrays: a barrier between them
    # and the loop that reads the tiles, and one before the next K step overwrites them
    assert got.count("__syncthreads();") == 2
    first = got.index("__syncthreads();")
    assert got[first + 1] == "for (int kk = 0; kk < BK; kk++) {"
    assert got[first - 1].startswith("reinterpret_cast<float4 *>(&b_lds[")
    chain = lines(generate("gather_columns"))
    assert "mine[0] = x[((0 * cols) + c)];" in chain
    assert "mine[(r + 1)] = x[(((r + 1) * cols) + c)];" in chain
    with pytest.raises(HipgenError, match="no address to offset"):
        generate("view_without_address")


def test_wavefront_load_and_store_primitives():
    got = lines(generate("wave_load"))
    assert got[0] == "__device__ void wave_load(int __block_id, int __thread_id, char* __smem, const int* src, int* dst, int items) {"
    i = got.index("int __thread_id_1 = __thread_id_0 % 64;")
    assert got[i + 1] == "int lane = __thread_id_1;"
    assert "const int* mine = src + ((lane * items));" in got
    assert "lane_load(__block_id_2, __thread_id_2, __smem, mine, dst, items);" in got
    caller = lines(generate("add_m_by_wavefronts"))
    assert "int w = (__thread_id_0 / 64);" in caller and "int held[4];" in caller
    launcher = generate_launcher("add_m_by_wavefronts")
    order = [launcher.index(f"void {name}(") for name in ("lane_load", "wave_load", "add_m_by_wavefronts")]
    assert order == sorted(order)  # callees are defined before their callers


def test_matrix_instruction_statement():
    got = lines(generate("one_mfma_per_wavefront"))
    i = got.index("typedef float __acc_t __attribute__((ext_vector_type(4)));")
    assert got[i + 1] == "__acc_t __acc = {c0, c1, c2, c3};"
    assert got[i + 2] == ("__acc = __builtin_amdgcn_mfma_f32_16x16x4f32(A_rows[(((r * K) + k0) + q)], "
                          "B_cols[(((k0 + q) * N) + r)], __acc, 0, 0, 0);")
    assert got[i + 3:i + 7] == [f"c{v} = __acc[{v}];" for v in range(4)]
    assert "const int w = (__thread_id_0 / 64);" in got
    with pytest.raises(HipgenError, match="intrinsic.mma is not an instruction of this target"):
        generate("foreign_instruction")
    tiled = lines(generate("mfma_tile_sgemm"))
    i = tiled.index("typedef float __acc_t __attribute__((ext_vector_type(16)));")
    assert tiled[i + 2].startswith("__acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_lds[((((kk + q) * 64) + corner_r) + r)], b_lds[")
    assert tiled[i + 3] == "acc[0] = __acc[0];" and tiled[i + 18] == "acc[15] = __acc[15];"
    # a barrier between the staging loop and the matrix instructions, one before the next K step
    assert tiled.count("__syncthreads();") == 2
    assert tiled[tiled.index("__syncthreads();") + 1] == "for (int kk = 0; kk < 8; kk += 2) {"
    half = lines(generate("one_bf16_mfma_per_wavefront"))
    assert half[0].startswith("__global__ void one_bf16_mfma_per_wavefront(const __bf16* P, const __bf16* Q, float* D,")
    assert "float4 a = reinterpret_cast<const float4 *>(&P_rows[(((r * K) + k0) + (8 * q))])[0];" in half
    i = half.index("typedef __bf16 __packet_t __attribute__((ext_vector_type(8)));")
    assert half[i + 1] == ("__acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(__packet_t, a), "
                           "__builtin_bit_cast(__packet_t, b), __acc, 0, 0, 0);")


def test_device_function_gets_the_callers_ids():
    helper = lines(generate("scaled_sum"))
    assert helper[0] == "__device__ float scaled_sum(int __block_id, int __thread_id, char* __smem, float a, float b, float s) {"
    assert helper[1:3] == ["int __block_id_0 = __block_id;", "int __thread_id_0 = __thread_id;"]
    assert "return (s * (a + b));" in helper
    caller = generate("scaled_sum_all")
    assert "y_one[0] = scaled_sum(__block_id_2, __thread_id_2, __smem, x[i], y_one[0], s);" in caller
    launcher = generate_launcher("scaled_sum_all")
    assert launcher.index("__device__ float scaled_sum(") < launcher.index("__global__ void scaled_sum_all(")


def test_split_restarts_ids_in_every_case():
    got = lines(generate("two_roles"))
    i = got.index("int __thread_id_2 = __thread_id_1;")
    assert got[i - 1] == "int __block_id_2 = __block_id_1;"
    assert got[i + 1] == "if (__thread_id_2 >= 0 && __thread_id_2 < 128) {" and got[i + 2] == "int t = __thread_id_2;"
    k = got.index("int __thread_id_2 = __thread_id_1 - 128;")
    assert got[k + 1] == "if (__thread_id_2 >= 0 && __thread_id_2 < 128) {" and k > i
    assert "y_mine[(128 + t)] = (x[((base + 128) + t)] + 1);" in got
    with pytest.raises(HipgenError, match="inside one `if`"):
        generate("split_with_hazard")  # a barrier inside a case would not be reached by the other threads


def test_a_hazard_inside_a_workgroup_uniform_if_gets_its_barrier_inside():
    """The reference's pass walks into branches and places barriers there (prism/sync_analysis.py:424-447). Here that
    is done when every thread of the workgroup takes the same side: the condition names only numbers, grid- or
    block-level values and variables of loops over such ranges. The barrier stands between the store and the
    read, inside the `if`; the loop then needs one more at the end of its body (the next round's store against
    this round's read)."""
    got = lines(generate("hazard_in_uniform_branch"))
    at = got.index("if (((r % 2) == 0)) {")
    assert got[at + 1] == "slot[0] = x_mine[t];" and got[at + 2] == "__syncthreads();" and got[at + 3] == "x_mine[t] = buf[(63 - t)];"
    assert got[at + 4] == "}" and got[at + 5] == "__builtin_amdgcn_sched_barrier(0);" and got[at + 6] == "__syncthreads();"
    assert got.count("__syncthreads();") == 2
    why = explain_barriers("hazard_in_uniform_branch")
    assert len(why) == 2 and "reads buf (written since the last barrier)" in why[0]


def test_scheduling_group_statements():
    @requires(grid[1], block[1], thread[1])
    @prism("global")
    def scheduled(x: ptr(float) @ grid[1]):
        with group(block[1]):
            intrinsic.sched_group("lds_read", 4)
            intrinsic.sched_group("mfma", 8, 1)
            intrinsic.sched_group("vmem_read", 1)
            intrinsic.sched_group("barrier")

    got = lines(generate("scheduled"))
    assert got[got.index("__builtin_amdgcn_sched_group_barrier(0x100, 4, 0);") + 1] == "__builtin_amdgcn_sched_group_barrier(0x008, 8, 1);"
    assert "__builtin_amdgcn_sched_group_barrier(0x020, 1, 0);" in got and "__builtin_amdgcn_sched_barrier(0);" in got

    @requires(grid[1], block[1], thread[1])
    @prism("global")
    def badly_scheduled(x: ptr(float) @ grid[1]):
        with group(block[1]):
            intrinsic.sched_group("tensor", 4)

    with pytest.raises(HipgenError, match="kind one of"):
        generate("badly_scheduled")


def test_refusals_name_the_construct():
    with pytest.raises(HipgenError, match="inside one `if`"):
        generate("hazard_in_branch")
    with pytest.raises(HipgenError, match="a power of two up to the 64-lane wavefront or a whole number of wavefronts"):
        generate("straddling_groups")
    with pytest.raises(HipgenError, match="thread-level kernels only"):
        generate("naive_sgemm", bounded=True)


def test_thread_groups_of_32_and_target_text():
    """A group of 32 threads is index arithmetic (`% 32`, `/ 32`); unsafe() text is printed as it stands, and
    the bare `return` that follows it in a value-returning function is dropped."""
    helper = lines(generate("lane_shift_up"))
    assert helper[0] == "__device__ uint32_t lane_shift_up(int __block_id, int __thread_id, char* __smem, uint32_t val, uint32_t delta) {"
    assert "return __shfl_up(val, delta, 32);" in helper and "return;" not in helper
    got = lines(generate("row_scan32"))
    assert "int g = (__thread_id_1 / 32);" in got
    i = got.index("int __thread_id_2 = __thread_id_1 % 32;")
    assert got[i - 1] == "int __block_id_2 = __block_id_1;" and got[i + 1] == "uint32_t lane = __thread_id_2;"
    assert "while ((step < 32)) {" in got
    assert "uint32_t got = lane_shift_up(__block_id_3, __thread_id_3, __smem, v, step);" in got


BUILDS = {"two_roles": (256, None), "row_scan32": (256, None), "add_m_blocks": (256, None), "naive_sgemm": (256, None), "tiled_sgemm": (1024, [32]),
          "thread_tile_sgemm": (256, [64, 64, 8, 4, 4]), "scaled_sum_all": (256, None),
          "vector_tile_sgemm": (256, [128, 128, 8, 8, 8]), "gather_columns": (256, None),
          "add_m_by_wavefronts": (256, None), "one_mfma_per_wavefront": (256, None),
          "one_bf16_mfma_per_wavefront": (256, None), "mfma_tile_sgemm": (256, None),
          "staged_sgemm": (256, [64, 64, 8, 4, 4, 256])}


@pytest.fixture(scope="module")
def built(tmp_path_factory):
    """Every kernel above, generated and cross-compiled for gfx950 once for this module."""
    d = tmp_path_factory.mktemp("hipgen_blocks")
    return {name: hipgen.build(name, out_dir=str(d), block_size=bs, template=targs) for name, (bs, targs) in BUILDS.items()}


def test_launchers_compile_for_gfx950(built):
    for name in BUILDS:
        assert hasattr(built[name], f"{name}_launch")


SGEMM_ARGS = [ctypes.c_int] * 3 + [ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p,
                                   ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]


def run_sgemm(lib, name, oracle, M, N, K, last_arg, grid_blocks):
    import torch
    fn = getattr(lib, f"{name}_launch")
    fn.argtypes = SGEMM_ARGS
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + N + K)
    a, b = torch.from_numpy(A).to("cuda:0"), torch.from_numpy(B).to("cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    c = buf[64:64 + M * N].view(M, N)
    c.copy_(torch.from_numpy(Cm))
    assert fn(M, N, K, 0.5, a.data_ptr(), b.data_ptr(), 3.0, c.data_ptr(), last_arg, grid_blocks, None) == 0
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)
    want = oracle.np_sgemm_f64(0.5, A, B, 3.0, Cm)
    tol = oracle.sgemm_tolerance(K, A, B) + 3.0 * float(np.abs(Cm).max()) * 2**-22
    assert np.max(np.abs(out[64:64 + M * N].reshape(M, N) - want)) <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 255, 256, 1000, (1 << 20) + 5])
def test_generated_block_thread_add_m_is_bit_exact(built, n):
    import torch
    fn = built["add_m_blocks"].add_m_blocks_launch
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    x = np.random.default_rng(n).integers(-2**20, 2**20, n, dtype=np.int32)
    x[0] = 2**31 - 2
    xd = torch.from_numpy(x).to("cuda:0")
    yd = torch.full((n + 4,), -1, dtype=torch.int32, device="cuda:0")
    assert fn(xd.data_ptr(), yd.data_ptr(), 7, 256, n, (n + 255) // 256, None) == 0
    torch.cuda.synchronize()
    y = yd.cpu().numpy()
    assert np.array_equal(y[:n], x + np.int32(7)) and np.all(y[n:] == -1)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 1, 1), (33, 47, 29), (128, 96, 200)])
def test_generated_naive_sgemm(built, oracle, shape):
    M, N, K = shape
    run_sgemm(built["naive_sgemm"], "naive_sgemm", oracle, M, N, K, 256, (M * N + 255) // 256)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(32, 32, 32), (64, 96, 160), (256, 128, 64)])
def test_generated_lds_tiled_sgemm(built, oracle, shape):
    """Needs the barriers to be where they belong: without them the tiles are read half-written."""
    M, N, K = shape
    run_sgemm(built["tiled_sgemm"], "tiled_sgemm", oracle, M, N, K, N // 32, (M // 32) * (N // 32))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(64, 64, 8), (128, 192, 72), (256, 64, 256)])
def test_generated_thread_tile_sgemm(built, oracle, shape):
    M, N, K = shape
    run_sgemm(built["thread_tile_sgemm"], "thread_tile_sgemm", oracle, M, N, K, N // 64, (M // 64) * (N // 64))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(64, 64, 8), (128, 192, 72), (256, 64, 256)])
def test_generated_sgemm_staged_by_device_functions(built, oracle, shape):
    """The tiles are filled and read by device functions; the barriers around the calls make it right."""
    M, N, K = shape
    run_sgemm(built["staged_sgemm"], "staged_sgemm", oracle, M, N, K, N // 64, (M // 64) * (N // 64))


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [1, 8, 9, 1000])
def test_generated_row_scan_on_half_wavefronts(built, rows):
    """Groups of 32 threads on 64-lane wavefronts: two rows per wavefront, the shuffle stays inside each."""
    import torch
    fn = built["row_scan32"].row_scan32_launch
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    x = np.random.default_rng(rows).integers(0, 2**32, (rows, 32), dtype=np.uint32)
    xd = torch.from_numpy(x.view(np.int32)).to("cuda:0")
    yd = torch.full((rows * 32 + 64,), -1, dtype=torch.int32, device="cuda:0")
    assert fn(xd.data_ptr(), yd.data_ptr(), rows, (rows + 7) // 8, None) == 0
    torch.cuda.synchronize()
    y = yd.cpu().numpy().view(np.uint32)
    assert np.array_equal(y[:rows * 32].reshape(rows, 32), np.cumsum(x, axis=1, dtype=np.uint32))
    assert np.all(y[rows * 32:] == 0xFFFFFFFF)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 128, 129, 256, 1000])
def test_generated_split_runs_both_roles(built, n):
    import torch
    fn = built["two_roles"].two_roles_launch
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    x = np.random.default_rng(n).integers(-1000, 1000, n, dtype=np.int32)
    xd = torch.from_numpy(x).to("cuda:0")
    yd = torch.full((n + 4,), -1, dtype=torch.int32, device="cuda:0")
    assert fn(xd.data_ptr(), yd.data_ptr(), n, (n + 255) // 256, None) == 0
    torch.cuda.synchronize()
    first_role = (np.arange(n) % 256) < 128
    y = yd.cpu().numpy()
    assert np.array_equal(y[:n], np.where(first_role, x * 2, x + 1)) and np.all(y[n:] == -1)


@pytest.mark.gpu
def test_generated_kernel_calls_its_device_function(built):
    import torch
    fn = built["scaled_sum_all"].scaled_sum_all_launch
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    n = 10_001
    rng = np.random.default_rng(5)
    x, y = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    xd, yd = torch.from_numpy(x).to("cuda:0"), torch.from_numpy(y).to("cuda:0")
    assert fn(xd.data_ptr(), yd.data_ptr(), 0.25, n, (n + 255) // 256, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(yd.cpu().numpy(), np.float32(0.25) * (x + y))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(128, 128, 8), (256, 384, 72), (384, 128, 256)])
def test_generated_vector_tile_sgemm(built, oracle, shape):
    """16-byte loads of A and B, a transposed A tile behind an index-mapped view, 16-byte read-modify-write of C."""
    M, N, K = shape
    run_sgemm(built["vector_tile_sgemm"], "vector_tile_sgemm", oracle, M, N, K, N // 128, (M // 128) * (N // 128))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 1), (7, 300), (33, 256), (50, 1000)])
def test_generated_stacked_views_transpose(built, shape):
    import torch
    rows, cols = shape
    fn = built["gather_columns"].gather_columns_launch
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    x = np.random.default_rng(rows * cols).integers(-2**31, 2**31 - 1, (rows, cols), dtype=np.int32)
    xd = torch.from_numpy(x).to("cuda:0")
    yd = torch.full((rows * cols + 8,), -5, dtype=torch.int32, device="cuda:0")
    assert fn(xd.data_ptr(), yd.data_ptr(), rows, cols, (cols + 255) // 256, None) == 0
    torch.cuda.synchronize()
    y = yd.cpu().numpy()
    assert np.array_equal(y[:rows * cols].reshape(cols, rows), x.T) and np.all(y[rows * cols:] == -5)


@pytest.mark.gpu
@pytest.mark.parametrize("wavefronts", [1, 4, 5, 1000])
def test_generated_wavefront_load_store(built, wavefronts):
    import torch
    fn = built["add_m_by_wavefronts"].add_m_by_wavefronts_launch
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    n = wavefronts * 256
    x = np.random.default_rng(wavefronts).integers(-2**30, 2**30, n, dtype=np.int32)
    xd = torch.from_numpy(x).to("cuda:0")
    yd = torch.full((n + 8,), -5, dtype=torch.int32, device="cuda:0")
    assert fn(xd.data_ptr(), yd.data_ptr(), 7, wavefronts, (wavefronts + 3) // 4, None) == 0
    torch.cuda.synchronize()
    y = yd.cpu().numpy()
    assert np.array_equal(y[:n], x + np.int32(7)) and np.all(y[n:] == -5)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(16, 16, 4), (48, 80, 36), (256, 128, 512)])
def test_generated_one_mfma_per_wavefront(built, oracle, shape):
    import torch
    M, N, K = shape
    fn = built["one_mfma_per_wavefront"].one_mfma_per_wavefront_launch
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_uint, ctypes.c_void_p]
    A, B, _ = oracle.gen_sgemm(M, N, K, seed=M + K)
    a, b = torch.from_numpy(A).to("cuda:0"), torch.from_numpy(B).to("cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    c = buf[64:64 + M * N]
    tiles = (M // 16) * (N // 16)
    assert fn(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, (tiles + 3) // 4, None) == 0
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)
    want = oracle.np_sgemm_f64(1.0, A, B, 0.0, np.zeros((M, N), np.float32))
    assert np.max(np.abs(out[64:64 + M * N].reshape(M, N) - want)) <= oracle.sgemm_tolerance(K, A, B)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(16, 16, 32), (48, 80, 96), (256, 128, 512)])
def test_generated_one_bf16_mfma_per_wavefront(built, oracle, shape):
    import torch
    M, N, K = shape
    fn = built["one_bf16_mfma_per_wavefront"].one_bf16_mfma_per_wavefront_launch
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_uint, ctypes.c_void_p]
    P16, Q16 = oracle.gen_gemm_bf16(M, N, K, seed=M + K)
    p = torch.from_numpy(P16.view(np.int16)).to("cuda:0")
    q = torch.from_numpy(Q16.view(np.int16)).to("cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    d = buf[64:64 + M * N]
    tiles = (M // 16) * (N // 16)
    assert fn(p.data_ptr(), q.data_ptr(), d.data_ptr(), M, N, K, (tiles + 3) // 4, None) == 0
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)
    ref = oracle.gemm_bf16_f64(P16, Q16)
    assert np.max(np.abs(out[64:64 + M * N].reshape(M, N) - ref)) <= 1e-3 * np.abs(ref).max()


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(64, 64, 8), (128, 192, 72), (256, 128, 256)])
def test_generated_lds_tiled_mfma_sgemm(built, oracle, shape):
    """LDS staging with the emitter's barriers around wavefront-wide matrix instructions."""
    M, N, K = shape
    run_sgemm(built["mfma_tile_sgemm"], "mfma_tile_sgemm", oracle, M, N, K, N // 64, (M // 64) * (N // 64))


@pytest.mark.gpu
@pytest.mark.parametrize("rounds", [0, 1, 2, 3, 6])
def test_generated_barrier_inside_a_uniform_if_runs(tmp_path_factory, rounds):
    """hazard_in_uniform_branch reverses its 64 values through LDS once per even round, behind a barrier that
    stands inside the `if`: wrong or missing barriers show as values from the wrong round."""
    import torch
    from prism_amd import hipgen
    lib = hipgen.build("hazard_in_uniform_branch", out_dir=str(tmp_path_factory.mktemp("uniform_if")), block_size=64)
    fn = lib.hazard_in_uniform_branch_launch
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    x = np.arange(64, dtype=np.float32) * 1.5
    xd = torch.from_numpy(x).to("cuda:0")
    assert fn(xd.data_ptr(), rounds, 1, None) == 0
    torch.cuda.synchronize()
    want = x[::-1] if ((rounds + 1) // 2) % 2 else x
    assert np.array_equal(xd.cpu().numpy(), want)
