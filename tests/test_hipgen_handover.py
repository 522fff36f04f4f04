"""LDS arrays handed between the cases of `match split(thread)` (prism_amd/hipgen_blocks.py, _plan_handovers) and the
producer / consumer GEMM built on it (prism_amd/examples/handover.py).

CPU: where the waits and signals land in each case, the round arithmetic, that the K loop carries no workgroup
barrier, and what is refused. GPU: the kernel against the fp64 oracle of the bf16 GEMM (1e-3 of the largest
|element|, the tolerance of the library's own bf16 kernel; sums are fp32).
"""
import ctypes

import numpy as np
import pytest

from prism_amd import hipgen
from prism_amd.examples import handover  # noqa: F401  (defines the kernel)
from prism_amd.hipgen import HipgenError, block, claim, generate, grid, group, intrinsic, partition, prism, ptr, requires, shared, split, thread


def lines(text):
    return [ln.strip() for ln in text.splitlines()]


def test_waits_and_signals_of_the_producer_consumer_gemm():
    got = lines(generate("handed_over_gemm"))
    # two round counters per slot beside its declaration, cleared before anyone can wait
    at = got.index("__shared__ __bf16 p_first[2048];")
    assert got[at + 1:at + 6] == ["__shared__ unsigned int __full_p_first, __empty_p_first;", "int __round_p_first = 0;",
                                  "bool __pending_p_first = false;  // filled by this wavefront and not announced yet",
                                  "if (threadIdx.x == 0) { __full_p_first = 0; __empty_p_first = 0; }", "__syncthreads();"]
    # the only workgroup barriers are those four: none in the K loop, whose iterations are ordered by the counters
    loop = got.index("for (int k0 = 0; k0 < K; k0 += 64) {")
    assert got.count("__syncthreads();") == 4 and all(n < loop for n, ln in enumerate(got) if ln == "__syncthreads();")

    def events(start, stop):
        """Waits, work and announcements in order. An announcement is ("signal", word) when it is made at once
        (behind a wait for everything in flight) and ("announce", word, what may still fly) when it is one a
        writer has put off; the blocks in which a writer announces everything before it blocks are left out."""
        out, depth_of_flush = [], None
        for n, ln in enumerate(got[start:stop], start):
            if ln.startswith("const unsigned int __need = "):
                need = ln.split("static_cast<int>(")[1].split(")));")[0]
            elif ln.startswith("if (static_cast<unsigned int>(") and "__prism_lds_peek(" in ln and ln.endswith("< __need) {"):
                depth_of_flush = 0   # the writer's "about to block" block: skipped up to its closing brace
            elif depth_of_flush is not None:
                depth_of_flush += ln.endswith("{") - (ln == "}")
                if depth_of_flush < 0:
                    depth_of_flush = None
            elif ln.startswith("for (; __spin"):
                word = ln.split("(&__")[1].split(",")[0].split(")")[0]
                out.append(("wait", word, need))
            elif "__hip_atomic_fetch_add(&__" in ln:
                out.append(("signal", ln.split("__hip_atomic_fetch_add(&__")[1].split(",")[0]))
            elif "__prism_lds_count(&__" in ln:
                wait = got[n - 1]
                out.append(("announce", ln.split("__prism_lds_count(&__")[1].split(")")[0],
                            wait.split("// ")[1] if "//" in wait else "nothing in flight"))
            elif ln.startswith(("for (int part", "for (int n", "float4 a")):
                out.append(("work", ln.split(" = ")[0] if ln.startswith("float4") else ln.split(";")[0]))
        return out

    producer = got.index("if (__thread_id_2 >= 0 && __thread_id_2 < 64) {")
    consumer = got.index("if (__thread_id_2 >= 0 && __thread_id_2 < 256) {")
    end = got.index("float* D_mine = D_tile + (0);")
    # The producer (one wavefront) fills two pairs of slots per trip. It waits for the four reading wavefronts of
    # the round before and fills; the filling is announced only behind the NEXT filling's eight loads, once at
    # most those are in flight, so that two fillings' loads overlap (and across trips: the second pair is
    # announced behind the first pair's loads of the next trip, or behind the loop).
    assert events(producer, consumer) == [
        ("wait", "empty_p_first", "__round_p_first * 4"), ("wait", "empty_q_first", "__round_q_first * 4"),
        ("work", "for (int part = 0"), ("announce", "full_p_second", "vmcnt(8)"), ("announce", "full_q_second", "vmcnt(8)"),
        ("wait", "empty_p_second", "__round_p_second * 4"), ("wait", "empty_q_second", "__round_q_second * 4"),
        ("work", "for (int part = 0"), ("announce", "full_p_first", "vmcnt(8)"), ("announce", "full_q_first", "vmcnt(8)")]
    # a consumer gives a slot back as soon as its last read of it is behind it
    assert events(consumer, end) == [
        ("wait", "full_p_first", "(__round_p_first + 1) * 1"), ("work", "float4 a"), ("signal", "empty_p_first"),
        ("wait", "full_q_first", "(__round_q_first + 1) * 1"), ("work", "for (int n = 0"), ("signal", "empty_q_first"),
        ("wait", "full_p_second", "(__round_p_second + 1) * 1"), ("work", "float4 a2"), ("signal", "empty_p_second"),
        ("wait", "full_q_second", "(__round_q_second + 1) * 1"), ("work", "for (int n = 0"), ("signal", "empty_q_second"),
        # behind the loop: whatever the producer has not announced yet
        ("announce", "full_p_first", "nothing in flight"), ("announce", "full_p_second", "nothing in flight"),
        ("announce", "full_q_first", "nothing in flight"), ("announce", "full_q_second", "nothing in flight")]
    # a filling counts its round at once (the next wait for "empty" must include it) and is marked unannounced
    at = got.index("__round_p_first += 1;")
    assert got[at + 1] == "__round_q_first += 1;" and got[at + 2] == "if (__pending_p_second) {"
    assert got[at + 3] == "__builtin_amdgcn_s_waitcnt(3960);  // vmcnt(8)"   # vmcnt 8, expcnt and lgkmcnt not waited for
    assert got[at + 12:at + 14] == ["__pending_p_first = true;", "__pending_q_first = true;"]
    # before it blocks in a wait, a writer announces everything it has filled, behind a wait for all its loads
    block = got.index("if (static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_p_second)))) < __need) {")
    assert got[block + 1:block + 5] == ["if (__pending_p_first) {", "__builtin_amdgcn_s_waitcnt(0);",
                                        "if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_first);", "__pending_p_first = false;"]
    # a reader's signal follows the completion of everything the wavefront has in flight
    first_signal = next(n for n, ln in enumerate(got) if "__hip_atomic_fetch_add(&__empty_p_first" in ln)
    assert got[first_signal - 2:first_signal] == ["__builtin_amdgcn_s_waitcnt(0);", '__builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");']
    assert got[first_signal + 1] == "__round_p_first += 1;"
    assert ("__builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&P_rows[(((((16 * part) + row) * K) "
            "+ k0) + k8)]), (__attribute__((address_space(3))) void*)(&p_first_fill[(512 * part)]), 16, 0, 0);") in got
    # the writer reads and counts its hand-over words through helpers the compiler does not see into: it would
    # otherwise wait for all direct loads in front of every LDS access
    assert "__device__ __forceinline__ unsigned int __prism_lds_peek(const unsigned int* word) {" in got
    assert "__device__ __forceinline__ void __prism_lds_count(unsigned int* word) {" in got
    # every wait is bounded, and one that runs out of polls reports it (array and round) into the file-scope word
    waits = [n for n, ln in enumerate(got) if ln.startswith("for (; __spin")]
    assert len(waits) == 8 and all("__spin < 65536 &&" in got[n] for n in waits)
    assert all(got[n - 1] == "#pragma nounroll" and "__builtin_amdgcn_readfirstlane(" in got[n]
               and got[n + 1].startswith("if (__spin == 65536 && (threadIdx.x & 63) == 0) "
                                         "__hip_atomic_store(&__prism_handover_report, ") for n in waits)
    n = waits[0]   # first wait of the producer: array 0 (p_first), waiting for "empty" -> code 1
    assert "1u | (static_cast<unsigned int>(__round_p_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);" in got[n + 1]
    assert got[0] == "#ifndef PRISM_HANDOVER_REPORT" and "__device__ unsigned int __prism_handover_report = 0;" in got[:6]


@requires(grid[1], block[1], thread[128])
@prism("global")
def two_slots_and_a_barrier(x: ptr(int) @ grid[1], trips: int @ grid[1]):
    with group(block[1]):
        one: shared(int[256], static=True) @ block[1]
        two: shared(int[256], static=True) @ block[1]
        other: shared(int[128], static=True) @ block[1]
        for i in range(trips):
            with claim(one, p=thread[64], offset=0) as one_fill:
                with claim(two, p=thread[64], offset=0) as two_fill:
                    match split(thread):
                        case 64:
                            with group(thread[64]):
                                lane: int @ thread[1] = id()
                                intrinsic.load_to_lds(one_fill[0], x[4 * lane])
                                intrinsic.load_to_lds(two_fill[0], x[4 * lane + 256])
                        case 64:
                            t: int @ thread[1] = one[0] + two[1]
            with partition(other, p=thread[1], offset=0) as slot:
                me: int @ thread[1] = id()
                slot[me] = i
            u: int @ thread[1] = other[5]


def test_nothing_stays_unannounced_where_the_loop_does_more_than_the_split():
    """A filling may stay unannounced from one trip to the next only when the split is all the loop does. Here a
    barrier follows the split inside the loop (another array is written and read across threads); the readers
    would wait for the announcement and the writer for the readers at the barrier, so the writing case
    announces everything before it leaves the split."""
    got = lines(generate("two_slots_and_a_barrier"))
    loop = got.index("for (int i = 0; i < trips; i++) {")
    assert any(ln == "__syncthreads();" for ln in got[loop:])
    writer = got.index("if (__thread_id_2 >= 0 && __thread_id_2 < 64) {")
    reader = got.index("if (__thread_id_2 >= 0 && __thread_id_2 < 64) {", writer + 1)
    tail = got[writer:reader]
    last = max(n for n, ln in enumerate(tail) if ln == "__pending_two = true;")
    assert "if (__pending_one) {" in tail[last:] and "if (__pending_two) {" in tail[last:]
    assert tail[tail.index("if (__pending_two) {", last) + 1] == "__builtin_amdgcn_s_waitcnt(0);"
    # the full-size kernel's loop holds the split alone: nothing is announced between the last filling and the loop's end
    big = lines(generate("handed_over_gemm_big"))
    w = big.index("if (__thread_id_2 >= 0 && __thread_id_2 < 256) {")
    r = big.index("if (__thread_id_2 >= 0 && __thread_id_2 < 256) {", w + 1)
    assert big[r - 7:r - 3] == ["}", "__pending_third = true;", "}", "}"]   # ... and the writing case ends there


@requires(grid[1], block[1], thread[128])
@prism("global")
def two_writers(x: ptr(int) @ grid[1]):
    with group(block[1]):
        buf: shared(int[128], static=True) @ block[1]
        with partition(buf, p=thread[64], offset=0) as mine:
            match split(thread):
                case 64:
                    with partition(mine, p=thread[1], offset=0) as one:
                        one[0] = 1
                    t: int @ thread[1] = buf[1]
                case 64:
                    with partition(mine, p=thread[1], offset=1) as other:
                        other[0] = buf[0]


@requires(grid[1], block[1], thread[96])
@prism("global")
def half_a_wavefront_reads(x: ptr(int) @ grid[1]):
    with group(block[1]):
        buf: shared(int[128], static=True) @ block[1]
        with partition(buf, p=thread[64], offset=0) as mine:
            match split(thread):
                case 64:
                    with partition(mine, p=thread[1], offset=0) as one:
                        one[0] = 1
                case 32:
                    t: int @ thread[1] = buf[0]


@requires(grid[1], block[1], thread[128])
@prism("global")
def one_side_only(x: ptr(int) @ grid[1]):
    with group(block[1]):
        buf: shared(int[128], static=True) @ block[1]
        match split(thread):
            case 64:
                t: int @ thread[1] = buf[0]
            case 64:
                u: int @ thread[1] = buf[1]


def test_what_is_refused_and_what_needs_no_handover():
    with pytest.raises(HipgenError, match="buf is written by more than one case"):
        generate("two_writers")
    with pytest.raises(HipgenError, match="whole wavefronts"):
        generate("half_a_wavefront_reads")
    assert "__full_buf" not in generate("one_side_only")      # read by both cases, written by none


@requires(grid[1], block[1], thread[128])
@prism("global")
def there_and_back(x: ptr(int) @ grid[1], trips: int @ grid[1]):
    with group(block[1]):
        one: shared(int[256], static=True) @ block[1]
        two: shared(int[256], static=True) @ block[1]
        back: shared(int[64], static=True) @ block[1]
        for i in range(trips):
            with claim(one, p=thread[64], offset=0) as one_fill:
                with claim(two, p=thread[64], offset=0) as two_fill:
                    with claim(back, p=thread[64], offset=0) as back_fill:
                        match split(thread):
                            case 64:
                                with group(thread[64]):
                                    lane: int @ thread[1] = id()
                                    intrinsic.load_to_lds(one_fill[0], x[4 * lane])
                                    intrinsic.load_to_lds(two_fill[0], x[4 * lane + 256])
                                t: int @ thread[1] = back[3]
                            case 64:
                                u: int @ thread[1] = one[0] + two[1]
                                with partition(back_fill, p=thread[1], offset=0) as mine:
                                    mine[0] = u


def test_a_late_announcing_case_announces_before_it_blocks_in_any_wait():
    """The first case fills two arrays (announced late) and then waits for an array the second case fills from
    them: blocked in that wait with the second filling unannounced, both cases would wait for each other. Every
    wait of a late-announcing case, for whichever array, announces first when it has to block; and its polls go
    through the helper (the wavefront may have direct loads in flight)."""
    got = lines(generate("there_and_back"))
    wait = next(n for n, ln in enumerate(got) if ln.startswith("for (; __spin") and "__full_back" in ln)
    assert "__prism_lds_peek(&__full_back)" in got[wait]
    block = [n for n, ln in enumerate(got[:wait]) if ln.startswith("if (static_cast<unsigned int>(") and "__prism_lds_peek(&__full_back)" in ln][-1]
    between = got[block:wait]
    assert "if (__pending_one) {" in between and "if (__pending_two) {" in between
    assert between.count("__builtin_amdgcn_s_waitcnt(0);") == 2
    # the other case fills one array only: it announces at once, the ordinary way
    assert any("__hip_atomic_fetch_add(&__full_back, 1u" in ln for ln in got) and "__pending_back" not in "\n".join(got)


def test_loads_of_a_filling_are_counted_from_the_program_text():
    import ast
    from prism_amd.hipgen_blocks import _static_load_count
    from prism_amd import examples
    examples.load()

    def count(text):
        return _static_load_count(ast.parse(text).body)

    assert count("fill_slot(a, P, Q, K, k0)") == 12           # four and eight direct loads per thread
    assert count("fill_slot(a, P, Q, K, k0)\nfill_slot(b, P, Q, K, k1)") == 24
    assert count("for part in range(3):\n    intrinsic.load_to_lds(a[512 * part], P[part * K + lane])") == 3
    assert count("row: int @ thread[1] = lane / 4\nintrinsic.load_to_lds(a[0], P[row])") == 1
    # anything the text does not settle: a condition, a loop whose trips are not constants, an element read or written
    assert count("if k0 + 64 < K:\n    fill_slot(a, P, Q, K, k0)") is None
    assert count("for part in range(n):\n    intrinsic.load_to_lds(a[0], P[part])") is None
    assert count("v: int @ thread[1] = P[0]\nintrinsic.load_to_lds(a[0], P[v])") is None
    assert count("fill_slot(a, P, Q, K, table[0])") is None


@pytest.fixture(scope="module")
def built(tmp_path_factory):
    return hipgen.build("handed_over_gemm", out_dir=str(tmp_path_factory.mktemp("hipgen_handover")), block_size=320)


@pytest.fixture(scope="module")
def built_big(tmp_path_factory):
    return hipgen.build("handed_over_gemm_big", out_dir=str(tmp_path_factory.mktemp("hipgen_handover_big")), block_size=512)


def test_launcher_compiles_for_gfx950(built, built_big):
    assert hasattr(built, "handed_over_gemm_launch") and hasattr(built_big, "handed_over_gemm_big_launch")


def test_hand_over_through_device_functions():
    """The full-size kernel fills and multiplies its slots in device functions: what a call does to a slot is read
    off the callee's signature (a pointer to const is read, another pointer written), as for the barriers."""
    got = lines(generate("handed_over_gemm_big"))
    fills = [n for n, ln in enumerate(got) if ln.startswith("fill_slot(")]
    mults = [n for n, ln in enumerate(got) if ln.startswith("multiply_slot(")]
    assert len(fills) == 3 and len(mults) == 3
    before = {"first": "third", "second": "first", "third": "second"}
    for name, n in zip(("first", "second", "third"), fills):
        # wait until the four readers are done (announcing what is unannounced before blocking), fill, count the
        # round, and announce the slot filled BEFORE this one once at most this filling's twelve loads are in flight
        assert got[n - 3].startswith("for (; __spin < 65536 && ") and f"__prism_lds_peek(&__empty_{name})" in got[n - 3]
        assert got[n + 1] == f"__round_{name} += 1;"
        after = got[n + 2:n + 13]
        at = after.index(f"if (__pending_{before[name]}) {{")
        assert after[at + 1] == "__builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)"
        assert after[at + 2] == f"if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_{before[name]});"
        assert after[-1] == f"__pending_{name} = true;"
    for name, n in zip(("first", "second", "third"), mults):   # wait until the four writers are done, multiply, give back
        m = n if name == "first" else n - 1                    # (the second and third slot are multiplied under `if`: K may end inside a trip)
        assert f"__hip_atomic_load(&__full_{name}," in got[m - 4] and f"(__round_{name} + 1) * 4" in got[m - 6]
        give_back = n + 3 if name == "first" else n + 4
        assert f"__hip_atomic_fetch_add(&__empty_{name}, 1u" in got[give_back]
    assert got[mults[1] - 1] == "if (((k0 + 64) < K)) {" and got[mults[2] - 1] == "if (((k0 + 128) < K)) {"
    loop = got.index("for (int k0 = 0; k0 < K; k0 += 192) {")
    assert got.count("__syncthreads();") == 3 and all(n < loop for n, ln in enumerate(got) if ln == "__syncthreads();")
    assert any("__launch_bounds__(512)" in ln for ln in got[:30])
    # a thread group may be a whole number of wavefronts (the callee's group of 256 producer threads)
    assert "int __thread_id_1 = __thread_id_0 % 256;" in lines(generate("fill_slot"))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(64, 64, 64), (128, 192, 256), (256, 128, 1024), (512, 512, 4096)])
def test_producer_consumer_gemm_against_the_oracle(built, oracle, shape):
    """Up to 64 rounds of hand-over per workgroup; a lost or early signal shows as a wrong tile."""
    import torch
    M, N, K = shape
    fn = built.handed_over_gemm_launch
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_uint, ctypes.c_void_p]
    p16, q16 = oracle.gen_gemm_bf16(M, N, K, seed=M + N + K)
    P = torch.from_numpy(p16.view(np.int16)).to("cuda:0")
    Q = torch.from_numpy(q16.view(np.int16)).to("cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    D = buf[64:64 + M * N]
    torch.cuda.synchronize()
    print(f"handed_over_gemm M={M} N={N} K={K}", flush=True)
    assert fn(P.data_ptr(), Q.data_ptr(), D.data_ptr(), N, K, N // 64, (M // 64) * (N // 64), None) == 0
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)
    ref = oracle.gemm_bf16_f64(p16, q16)
    assert np.max(np.abs(out[64:64 + M * N].reshape(M, N) - ref)) <= 1e-3 * np.abs(ref).max()


def test_the_launcher_text_has_a_status_call_and_the_poll_bound_is_an_argument():
    text = hipgen.generate_launcher("handed_over_gemm", block_size=320)
    assert 'extern "C" int handed_over_gemm_status(void* stream)' in text
    assert text.count("__device__ unsigned int __prism_handover_report = 0;") == 1
    assert "hipMemcpyFromSymbol(&word, HIP_SYMBOL(__prism_handover_report)" in text
    # the full-size kernel's waits sit in the kernel, its device functions come first in the file: one definition
    big = hipgen.generate_launcher("handed_over_gemm_big", block_size=512)
    assert big.count("__device__ unsigned int __prism_handover_report = 0;") == 1 and "handed_over_gemm_big_status" in big
    # a kernel without hand-over has neither the word nor the call
    from prism_amd import examples
    examples.load()
    plain = hipgen.generate_launcher("tiled_sgemm", block_size=1024, template=[32])
    assert "__prism_handover_report" not in plain and "_status" not in plain
    none = hipgen.generate_launcher("handed_over_gemm", block_size=320, handover_spins=0)
    assert "for (; __spin < 0 &&" in none and "if (__spin == 0 && (threadIdx.x & 63) == 0)" in none
    with pytest.raises(HipgenError):
        hipgen.generate_launcher("handed_over_gemm", block_size=320, handover_spins=-1)


@pytest.mark.gpu
def test_a_wait_that_gives_up_is_reported_and_the_kernel_still_exits(built, tmp_path_factory):
    """Driven from the host: a build whose waits give up before their first poll (handover_spins = 0). Every
    wavefront runs through all its rounds without waiting, the kernel exits normally, its result is not
    trusted, and the status call reports the give-up once and clears it. The ordinary build reports nothing."""
    import torch
    impatient = hipgen.build("handed_over_gemm", out_dir=str(tmp_path_factory.mktemp("hipgen_handover_spins0")),
                             block_size=320, handover_spins=0)
    M, N, K = 128, 128, 256
    P = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda:0")
    Q = torch.zeros((N, K), dtype=torch.bfloat16, device="cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    D = buf[64:64 + M * N]
    torch.cuda.synchronize()
    for lib in (impatient, built):
        lib.handed_over_gemm_launch.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_uint, ctypes.c_void_p]
        lib.handed_over_gemm_status.argtypes = [ctypes.c_void_p]
    print("handed_over_gemm with handover_spins=0", flush=True)
    assert impatient.handed_over_gemm_launch(P.data_ptr(), Q.data_ptr(), D.data_ptr(), N, K, N // 64, (M // 64) * (N // 64), None) == 0
    rc = impatient.handed_over_gemm_status(None)
    assert rc & 0x40000000 and 1 <= (rc & 0xff) <= 8, hex(rc)   # four arrays, "empty" and "full" waits
    assert impatient.handed_over_gemm_status(None) == 0             # reported once, then cleared
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)   # stores stayed inside the tile grid
    assert built.handed_over_gemm_launch(P.data_ptr(), Q.data_ptr(), D.data_ptr(), N, K, N // 64, (M // 64) * (N // 64), None) == 0
    assert built.handed_over_gemm_status(None) == 0
    assert bool((D == 0).all())


@requires(grid[1], block[1], thread[128])
@prism("global")
def slot_declared_in_the_loop(x: ptr(int) @ grid[1], trips: int @ grid[1]):
    with group(block[1]):
        for i in range(trips):
            buf: shared(int[128], static=True) @ block[1]
            with partition(buf, p=thread[64], offset=0) as mine:
                match split(thread):
                    case 64:
                        with partition(mine, p=thread[1], offset=0) as one:
                            one[0] = i
                    case 64:
                        t: int @ thread[1] = buf[0]


def test_a_handed_over_array_is_declared_outside_loops():
    with pytest.raises(HipgenError, match="outside any loop"):
        generate("slot_declared_in_the_loop")


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1024, 256, 64), (1024, 256, 128), (1024, 256, 192), (1024, 256, 320), (1024, 512, 1024),
                                   (2048, 1024, 4096), (2048, 2048, 512)])
def test_full_size_producer_consumer_gemm_against_the_oracle(built_big, oracle, shape):
    """128 x 256 tiles, four producer and four consumer wavefronts, three slots of 64 k with late announcements,
    tiles dealt to the XCDs in patches; K that ends in the first, second and third slot of a trip. The status call
    says that no wait gave up."""
    import torch
    M, N, K = shape
    fn = built_big.handed_over_gemm_big_launch
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4 + [ctypes.c_uint, ctypes.c_void_p]
    p16, q16 = oracle.gen_gemm_bf16(M, N, K, seed=M + N + K + 1)
    P = torch.from_numpy(p16.view(np.int16)).to("cuda:0")
    Q = torch.from_numpy(q16.view(np.int16)).to("cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    D = buf[64:64 + M * N]
    torch.cuda.synchronize()
    print(f"handed_over_gemm_big M={M} N={N} K={K}", flush=True)
    assert fn(P.data_ptr(), Q.data_ptr(), D.data_ptr(), N, K, M // 128, N // 256, (M // 128) * (N // 256), None) == 0
    built_big.handed_over_gemm_big_status.argtypes = [ctypes.c_void_p]
    assert built_big.handed_over_gemm_big_status(None) == 0
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)
    ref = oracle.gemm_bf16_f64(p16, q16)
    assert np.max(np.abs(out[64:64 + M * N].reshape(M, N) - ref)) <= 1e-3 * np.abs(ref).max()


@pytest.fixture(scope="module")
def built_sgemm(tmp_path_factory):
    return hipgen.build("handed_over_sgemm", out_dir=str(tmp_path_factory.mktemp("hipgen_handover_sgemm")), block_size=768)


def test_sgemm_launcher_compiles_for_gfx950(built_sgemm):
    assert hasattr(built_sgemm, "handed_over_sgemm_launch")
    got = lines(generate("handed_over_sgemm"))
    loop = got.index("for (int k0 = 0; k0 < K; k0 += 64) {")
    assert got.count("__syncthreads();") == 2 and all(n < loop for n, ln in enumerate(got) if ln == "__syncthreads();")


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1024, 256, 64), (1024, 768, 1000 // 64 * 64), (2048, 1024, 2048)])
def test_producer_consumer_sgemm_against_the_oracle(built_sgemm, oracle, shape):
    """fp32 matrix instructions fed through handed-over slots; the kernel-5 tolerance against fp64."""
    import torch
    M, N, K = shape
    fn = built_sgemm.handed_over_sgemm_launch
    fn.argtypes = [ctypes.c_int] * 3 + [ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p,
                                       ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + N + K)
    a, b = torch.from_numpy(A).to("cuda:0"), torch.from_numpy(B).to("cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    c = buf[64:64 + M * N].view(M, N)
    c.copy_(torch.from_numpy(Cm))
    torch.cuda.synchronize()
    print(f"handed_over_sgemm M={M} N={N} K={K}", flush=True)
    assert fn(M, N, K, 0.5, a.data_ptr(), b.data_ptr(), 3.0, c.data_ptr(), N // 256, (M // 128) * (N // 256), None) == 0
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)
    want = oracle.np_sgemm_f64(0.5, A, B, 3.0, Cm)
    tol = oracle.sgemm_tolerance(K, A, B) + 3.0 * float(np.abs(Cm).max()) * 2**-22
    assert np.max(np.abs(out[64:64 + M * N].reshape(M, N) - want)) <= tol
