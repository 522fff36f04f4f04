// Single-pass inclusive prefix sum with decoupled look-back, uint32 modulo 2^32.
//
// What the reference does (examples/scan.py:200-227, generated/scan_kernel.cu):
// every block takes a ticket, scans 16384 elements as 512 rows of 32 staged in
// shared memory, scans the 512 row totals, publishes its aggregate, walks back
// over its predecessors' {ready,data} records with one thread, publishes its
// inclusive prefix and writes the tile back.
//
// What this file does on 64-lane wavefronts:
//   * a tile lives in registers: every lane owns VPT packets of 4 consecutive
//     elements (16 B loads/stores, 1 KiB contiguous per wave instruction);
//   * lane-local serial sums, then one 6-step DPP scan per packet row across
//     the wave (row_shr 1/2/4/8, row_bcast 15, row_bcast 31) - the wave64
//     counterpart of scan_warps + shfl_up_sync_wrapper
//     (examples/scan.py:23-29,106-128);
//   * wave totals meet in LDS (<= 16 words) instead of the 512-entry
//     Hillis-Steele pass (examples/scan.py:131-171);
//   * one 64-bit status word per tile, {state, value}, written and polled with
//     agent-scope atomics so that the word is coherent across the eight XCD
//     L2s (the reference's volatile accesses assume one device-wide L2:
//     evals/4090_scan/main.cu:21-37, generated/lookback_to_prev_blocks.cu:12-21);
//   * the look-back is wave-parallel: 64 predecessors per poll, a ballot finds
//     the nearest published prefix (examples/scan.py:60-85 walks them one by
//     one with a single thread).
//
// Two measured facts about MI355X shape the tile size. Tickets are atomic adds
// on one address and retire at about one per 12 ns, so a 2^30-element scan can
// afford at most ~10^5 tiles. A status word takes a few microseconds to travel
// between XCDs, during which hundreds of small tiles would start, and the
// nearest published prefix would sit hundreds of tiles back. Large inputs
// therefore use 256 KiB tiles (few tiles in flight, one or two polls per
// look-back); small inputs use 64 KiB tiles so that more CUs get work. Polling
// with more than one wave per tile was measured slower: the extra status
// traffic costs more than the round trips it saves.
//
// Tile order. The reference numbers tiles with a ticket counter (examples/scan.py:88-99), in the order blocks
// start, so that a tile only ever waits for tiles that are already running. The ticket is an agent-scope
// atomic on one address, and its round trip (about 2 us) sits in front of every block's first load: measured
// 12 % of the run time at 2^30. The default here is tile = a fixed function of the workgroup id (chunks of 4
// consecutive tiles go to workgroups of one XCD, see the kernel), which waits least when the dispatcher starts
// the workgroups of a 1-D grid in id order on every XCD. Correctness does not rest on that order: a look-back
// that has polled a window kHelpAfter times without an answer (milliseconds; a running predecessor answers in
// microseconds) stops waiting and HELPS: wave 0 reads the silent predecessor's input itself, reduces it and
// uses that aggregate. Every tile therefore finishes on its own whatever the others do, the GPU never hangs
// and the result is the same bits. (In place, a predecessor might finish and overwrite its input while it is
// being helped: the helper polls the tile's status once more after its reads have returned and, if anything
// has been published by then, takes the published value instead; a tile's first publication is complete
// before any of its output stores are issued.) The flag kFlagTicket selects the reference's ticket order
// instead, kFlagNoHelp the behaviour of a plain bounded wait: a wave that runs out stores the tile number plus
// one into the workspace header (kHdrReport) and carries on with a wrong prefix; scan_status() reads that word
// after the stream has drained and turns it into an error. The segmented and the 64-bit scans help in the same
// way. scan_status() also reports a workspace that was never initialised (the header holds a magic word).
//
// Workspace protocol (no reset launch per call). Every tile owns TWO status words,
// one per parity of the workspace's call counter. A call with parity p publishes
// and polls the p words and stores zeros into the other ones, which the previous
// call on this workspace used (calls that share a workspace are ordered on one
// stream, so that call has finished). The header records up to which tile each
// parity may hold non-zero words, so a short call after a long one clears the
// long one's words as well. The last tile, once its look-back is complete,
// advances the call counter: by then every tile has published and therefore has
// read the header (a tile's status address depends on the parity it read). The
// reference clears its workspace with two memsets in front of every launch
// (evals/4090_scan/main.cu:81-82); here a workspace is cleared once, by
// scan_workspace_init(), and each call leaves it ready for the next.
//
// Status words use RELAXED agent-scope atomics: the value travels inside the
// atomic word, no other memory is communicated between tiles, so no fence is
// needed (acquire/release here would write back and invalidate a whole L2 per
// poll, measured 10x slower).
//
// HBM-bound: 8 algorithmic bytes per element (4 B read + 4 B write); status
// traffic is 8 B per tile plus the polls.
#include <mutex>
#include <type_traits>

#include "common.h"
#include "direct_load.h"
#include "wave_io.h"

namespace prism {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;

// Workspace: a 256-byte header, then two 64-bit status words per tile (word 2 t + p for parity p).
constexpr size_t kHeaderBytes = 256;
enum : int {                // header fields, as indices of 32-bit words
    kHdrTicket = 0,         // ticket counter (ticket order only); 0 between calls
    kHdrBadWorkspace = 1,   // a tile found no magic word or an impossible state: tile number + 1, sticky like kHdrReport
    kHdrReport = 2,         // look-back time-out report: tile number + 1, sticky until scan_status() reads it
    kHdrDone = 3,           // tiles that have read the header (plain scan) / finished (segmented scan); 0 between calls
    kHdrCalls = 4,          // calls completed on this workspace; its low bit is the parity of the next call
    kHdrDirty0 = 5,         // tiles whose parity-0 words may be non-zero
    kHdrDirty1 = 6,         // same for parity 1
    kHdrMagic = 7,          // kMagic once scan_workspace_init() has run (read together with words 4-6)
};
constexpr uint32_t kMagic = 0x5ca9b10cu;
constexpr uint32_t kSpinLimit = 1u << 22;  // polls of one look-back window / of the closing tile's wait before giving up
constexpr uint32_t kHelpAfter = 1u << 12;  // polls of one look-back window before a silent predecessor is helped

// Tile shapes: {threads, 16 B packets per lane}.
struct SmallCfg { static constexpr int BLOCK = 1024, VPT = 4; };
struct BigCfg { static constexpr int BLOCK = 1024, VPT = 16; };
template <typename Cfg> constexpr int tile_elems() { return Cfg::BLOCK * Cfg::VPT * 4; }
constexpr int kChunk = 4;  // consecutive tiles per XCD in workgroup-id order; 4-5 measured best, 1 and 32 worst
// Inputs up to this many elements use the small tile; so do inputs that are not 16-byte aligned (their
// element-wise loads would need more registers than the big tile leaves). Measured: level at 2^23 elements,
// the small tile ahead below (6 M: 5.4 against 5.2 TB/s), the big one above (12 M: 5.85 against 4.8).
constexpr size_t kSmallMax = size_t{1} << 23;
// Status words are sized for the small tile whatever tile a call ends up using.
constexpr size_t kWorkspaceTileElems = 16384;
static_assert(tile_elems<SmallCfg>() == kWorkspaceTileElems && tile_elems<BigCfg>() >= kWorkspaceTileElems, "");

// Tile states, the three-valued form of the reference's two ready flags
// (BlockInfo::prefix.ready / aggregate.ready, evals/4090_scan/main.cu:21-37).
constexpr uint32_t kInvalid = 0;    // nothing published yet
constexpr uint32_t kAggregate = 1;  // value = sum of this tile only
constexpr uint32_t kPrefix = 2;     // value = sum of everything up to and including this tile

__device__ __forceinline__ u64 pack_status(uint32_t state, uint32_t value) {
    return static_cast<u64>(state) | (static_cast<u64>(value) << 32);
}

__device__ __forceinline__ void publish(u64* word, uint32_t state, uint32_t value) {
    __hip_atomic_store(word, pack_status(state, value), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ u64 poll(const u64* word) {
    return __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// DPP controls (gfx9): row_shr:n = 0x110 + n, row_bcast:15 = 0x142, row_bcast:31 = 0x143.
template <int CTRL, int ROW_MASK, bool ZERO_FILL>
__device__ __forceinline__ uint32_t dpp(uint32_t x) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), CTRL, ROW_MASK,
                                                             0xf, ZERO_FILL));
}

// Inclusive scan across the 64 lanes of a wavefront, no LDS.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t x) {
    x += dpp<0x111, 0xf, true>(x);   // within each row of 16 lanes
    x += dpp<0x112, 0xf, true>(x);
    x += dpp<0x114, 0xf, true>(x);
    x += dpp<0x118, 0xf, true>(x);
    x += dpp<0x142, 0xa, false>(x);  // lane 15 of rows 0,2 into rows 1,3
    x += dpp<0x143, 0xc, false>(x);  // lane 31 into rows 2,3
    return x;
}

__device__ __forceinline__ uint32_t wave_last_lane(uint32_t x) {
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(x), 63));
}


// The operator of the scan: elements travel as 32-bit patterns; `identity` is what padding and "nothing
// before this" contribute.
struct SumOp {
    static constexpr bool kIsSum = true;
    static constexpr uint32_t identity = 0u;
    static __device__ __forceinline__ uint32_t apply(uint32_t a, uint32_t b) { return a + b; }
};
struct MaxI32Op {  // running maximum of signed 32-bit integers
    static constexpr bool kIsSum = false;
    static constexpr uint32_t identity = 0x80000000u;  // INT32_MIN
    static __device__ __forceinline__ uint32_t apply(uint32_t a, uint32_t b) {
        const int x = static_cast<int>(a), y = static_cast<int>(b);
        return static_cast<uint32_t>(x > y ? x : y);
    }
};

struct MinI32Op {  // running minimum of signed 32-bit integers
    static constexpr bool kIsSum = false;
    static constexpr uint32_t identity = 0x7fffffffu;  // INT32_MAX
    static __device__ __forceinline__ uint32_t apply(uint32_t a, uint32_t b) {
        const int x = static_cast<int>(a), y = static_cast<int>(b);
        return static_cast<uint32_t>(x < y ? x : y);
    }
};

// Inclusive scan across the wavefront for any operator: lanes without a source (the first lanes of a row
// for the shifts, the rows a broadcast is masked off for) receive the identity, through the DPP `old`
// operand instead of the zero fill.
template <typename Op, int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_or_identity(uint32_t x) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(Op::identity), static_cast<int>(x), CTRL,
                                                             ROW_MASK, 0xf, false));
}
template <typename Op>
__device__ __forceinline__ uint32_t wave_inclusive_scan_op(uint32_t x) {
    if constexpr (Op::kIsSum) {
        return wave_inclusive_scan(x);
    } else {
        x = Op::apply(x, dpp_or_identity<Op, 0x111, 0xf>(x));
        x = Op::apply(x, dpp_or_identity<Op, 0x112, 0xf>(x));
        x = Op::apply(x, dpp_or_identity<Op, 0x114, 0xf>(x));
        x = Op::apply(x, dpp_or_identity<Op, 0x118, 0xf>(x));
        x = Op::apply(x, dpp_or_identity<Op, 0x142, 0xa>(x));
        x = Op::apply(x, dpp_or_identity<Op, 0x143, 0xc>(x));
        return x;
    }
}
// What the lanes before this one combine to (the identity in lane 0), from the inclusive result.
template <typename Op>
__device__ __forceinline__ uint32_t wave_exclusive_from_inclusive(uint32_t inclusive, uint32_t own, int lane) {
    if constexpr (Op::kIsSum) {
        return inclusive - own;
    } else {
        const uint32_t up = static_cast<uint32_t>(__shfl_up(static_cast<int>(inclusive), 1, kWave));
        return lane == 0 ? Op::identity : up;
    }
}

// Tile number of a workgroup in workgroup-id order. Consecutive workgroup ids go to the 8 XCDs in turn, and
// the XCDs drift apart, so in plain id order half of all tiles start before their predecessor and wait
// longer for it. Chunks of kChunk consecutive tiles are given to workgroups of one XCD instead (every 8th
// id), which start in order; only chunk boundaries cross XCDs. A tile's predecessors then have ids at most
// 8 * kChunk above its own, far fewer than the workgroups resident at once, so the lowest unfinished tile
// is still always running.
__device__ __forceinline__ uint32_t tile_of_workgroup(uint32_t workgroup, uint32_t tiles) {
    constexpr uint32_t G = kChunk, SPAN = 8 * G;
    const uint32_t whole = (tiles / SPAN) * SPAN;
    if (workgroup >= whole) return workgroup;
    const uint32_t xcd = workgroup % 8, j = workgroup / 8;
    return (j / G) * SPAN + xcd * G + (j % G);
}

// What wave 0 of every tile does for the workspace once its own status word is final. hdr = the header
// words {calls, dirty0, dirty1, -} as read at the start of the kernel.
__device__ __forceinline__ void clear_other_parity(u64* status, u32x4 hdr, uint32_t tile, uint32_t tiles, int lane) {
    // Tile t clears words t, t + tiles, ... below the other parity's mark.
    const uint32_t parity = hdr.x & 1u, dirty_other = parity ? hdr.y : hdr.z;
    for (size_t w = tile + static_cast<size_t>(lane) * tiles; w < dirty_other; w += static_cast<size_t>(kWave) * tiles)
        __hip_atomic_store(&status[2 * w + (parity ^ 1u)], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Closes a call (one lane of one tile): counters back to zero, marks set, call counter advanced. Only when
// every tile of the call has read the header.
__device__ __forceinline__ void close_call(uint32_t* header, u32x4 hdr, uint32_t tiles) {
    const uint32_t calls = hdr.x, parity = calls & 1u;
    __hip_atomic_store(&header[kHdrTicket], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&header[kHdrDone], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&header[kHdrDirty0 + parity], tiles, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&header[kHdrDirty0 + (parity ^ 1u)], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&header[kHdrCalls], calls + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The aggregate of one whole tile, formed by one wavefront from the tile's input: what a look-back does for a
// predecessor that does not answer. Slow (one wavefront reads the whole tile) and rare.
template <typename Op, bool VEC, int TILE>
__device__ __forceinline__ uint32_t tile_aggregate(const uint32_t* in, size_t tile_base, int lane) {
    // Two loads in flight and a loop that stays a loop: this code sits inside the look-back of every tile and
    // must not cost the common path registers.
    uint32_t acc = Op::identity;
    if constexpr (VEC) {
        const u32x4* src = reinterpret_cast<const u32x4*>(in + tile_base) + lane;
#pragma unroll 1
        for (int i = 0; i < TILE / 4 / kWave; i += 2) {
            const u32x4 x = src[static_cast<size_t>(i) * kWave], y = src[static_cast<size_t>(i + 1) * kWave];
            acc = Op::apply(acc, Op::apply(Op::apply(x.x, x.y), Op::apply(x.z, x.w)));
            acc = Op::apply(acc, Op::apply(Op::apply(y.x, y.y), Op::apply(y.z, y.w)));
        }
    } else {
        const uint32_t* src = in + tile_base + lane;
#pragma unroll 1
        for (int i = 0; i < TILE / kWave; i += 4) {
            const uint32_t x0 = src[static_cast<size_t>(i) * kWave], x1 = src[static_cast<size_t>(i + 1) * kWave];
            const uint32_t x2 = src[static_cast<size_t>(i + 2) * kWave], x3 = src[static_cast<size_t>(i + 3) * kWave];
            acc = Op::apply(acc, Op::apply(Op::apply(x0, x1), Op::apply(x2, x3)));
        }
    }
    return wave_last_lane(wave_inclusive_scan_op<Op>(acc));
}

// Exclusive prefix of tile `tile` (> 0): the sum of all earlier tiles. Run by
// one whole wavefront; lane l inspects tile (window_end - l), whose status word
// of this call's parity is status[2 * tile + parity]. A predecessor that is
// running publishes within microseconds without waiting for anything later. One
// that has not answered after spin_limit polls of its window is not waited for
// any longer: with `help` the wavefront forms that tile's aggregate from the
// input itself (tile_aggregate; see "Tile order" at the top for why that is also
// right in place), so the loop always ends with the right sum; without `help`
// it reports tile + 1 into *report and returns what it has. spin_limit == 0
// skips the waiting altogether, which exercises either way out from the host.
// A state that no tile ever writes means the workspace holds something else
// (never initialised, or overwritten): reported into *bad_workspace.
template <typename Op, bool VEC, int TILE>
__device__ __forceinline__ uint32_t look_back(const u64* status, uint32_t parity, uint32_t tile, int lane,
                                              uint32_t spin_limit, bool help, const uint32_t* in, uint32_t* report,
                                              uint32_t* bad_workspace) {
    uint32_t sum = Op::identity;
    uint32_t spins = 0;
    long long window_end = static_cast<long long>(tile) - 1;
    while (true) {
        const long long t = window_end - lane;
        // Tiles "before the first" count as a published prefix of nothing.
        u64 w = (t >= 0) ? poll(&status[2 * t + parity]) : pack_status(kPrefix, Op::identity);
        uint32_t state = static_cast<uint32_t>(w);
        if (__ballot(state > kPrefix)) {
            if (lane == 0) __hip_atomic_store(bad_workspace, tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
        u64 has_prefix = __ballot(state == kPrefix);
        u64 is_invalid = __ballot(state == kInvalid);
        // Lanes 0..first-prefix-lane are needed; all 64 when no prefix is in the window.
        u64 needed = has_prefix ? ((2ull << __builtin_ctzll(has_prefix)) - 1ull) : ~0ull;
        if (is_invalid & needed) {
            if (spins < spin_limit) {
                ++spins;  // no s_sleep: the wait for the poll's answer paces the loop (sleeping measured 1 % slower)
                continue;
            }
            if (!help) {
                if (lane == 0) __hip_atomic_store(report, tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            for (u64 todo = is_invalid & needed; todo != 0; todo &= todo - 1) {
                const int l = __builtin_ctzll(todo);
                const uint32_t formed = tile_aggregate<Op, VEC, TILE>(in, static_cast<size_t>(window_end - l) * TILE, lane);
                // Every read of that tile's input has returned (the reduction used them). If the tile has
                // published anything by now, its word is the truth (in place, the input may be turning into
                // output); if not, it has not stored any output yet and `formed` is the sum of its input.
                const u64 again = poll(&status[2 * (window_end - l) + parity]);
                if (lane == l) w = static_cast<uint32_t>(again) != kInvalid ? again : pack_status(kAggregate, formed);
            }
            state = static_cast<uint32_t>(w);
            has_prefix = __ballot(state == kPrefix);
            needed = has_prefix ? ((2ull << __builtin_ctzll(has_prefix)) - 1ull) : ~0ull;
        }
        spins = 0;
        const uint32_t value = static_cast<uint32_t>(w >> 32);
        const uint32_t contrib = ((needed >> lane) & 1ull) ? value : Op::identity;
        sum = Op::apply(sum, wave_last_lane(wave_inclusive_scan_op<Op>(contrib)));
        if (has_prefix) break;
        window_end -= kWave;
    }
    return sum;
}

// 16-byte streaming store. `sc1 nt` writes through towards memory and marks the line for early
// eviction: measured on 4 GiB streams, stores with sc1 run 2-5 % faster than plain or nt-only ones
// (every line of the output is written exactly once and never read again by this kernel). The
// two wait states keep the next instruction from overwriting the data registers while the store
// still reads them (the compiler does not see a store inside the assembly).
__device__ __forceinline__ void stream_store(u32x4* p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

// VEC: in and out are 16 B aligned, full tiles use 16 B accesses.
// TICKET: tiles are numbered by the ticket counter, else by workgroup id.
// EXCLUSIVE: out[i] is the sum of the elements before i (out[0] = 0) instead of up to and including i;
// only the write-back differs.
// Op: the operator (sums by default; the other operators are inclusive only).
template <typename Cfg, bool VEC, bool TICKET, bool EXCLUSIVE, typename Op = SumOp>
__global__ __launch_bounds__(Cfg::BLOCK) void scan_lookback_kernel(const uint32_t* in, uint32_t* out,
                                                                   size_t n, uint32_t* header,
                                                                   u64* status, uint32_t spin_limit, bool help) {
    constexpr int BLOCK = Cfg::BLOCK, VPT = Cfg::VPT;
    constexpr int WAVES = BLOCK / kWave;
    constexpr int TILE = BLOCK * VPT * 4;
    constexpr int WAVE_ELEMS = kWave * VPT * 4;
    constexpr int ROW_ELEMS = kWave * 4;  // elements one wave instruction covers
    static_assert(BLOCK % kWave == 0 && BLOCK <= 1024, "block must be whole waves");
    static_assert(Op::kIsSum || !EXCLUSIVE, "the exclusive write-back is written for sums");

    __shared__ uint32_t s_tile;
    __shared__ uint32_t s_wave_total[WAVES];
    __shared__ uint32_t s_tile_prefix;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // uniform: what only wave 0 does stays in scalar registers
    const uint32_t tiles = gridDim.x;

    uint32_t tile = tile_of_workgroup(blockIdx.x, tiles);
    if constexpr (TICKET) {
        // Dynamic tile id: tiles are numbered in the order blocks start running (examples/scan.py:88-99).
        if (tid == 0)
            s_tile = __hip_atomic_fetch_add(&header[kHdrTicket], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        tile = s_tile;
    }

    const size_t tile_base = static_cast<size_t>(tile) * TILE;
    const size_t lane_base = tile_base + static_cast<size_t>(wave) * WAVE_ELEMS + lane * 4;
    const bool full = VEC && (tile_base + TILE <= n);

    u32x4 v[VPT];
    if (full) {
        wave_load_striped_streaming(reinterpret_cast<const u32x4*>(in + tile_base + static_cast<size_t>(wave) * WAVE_ELEMS), lane, v);
    } else {
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const size_t i = lane_base + j * ROW_ELEMS + c;
                v[j][c] = (i < n) ? in[i] : Op::identity;
            }
        }
    }
    // {calls, dirty0, dirty1, -} in one load: the status addresses below depend on it, so it has
    // completed before this tile publishes anything. Only the last tile of a call writes these words,
    // and only after every tile has published.
    u32x4 hdr = {0u, 0u, 0u, 0u};
    if (wave == 0) hdr = *reinterpret_cast<const u32x4*>(header + kHdrCalls);

    // Lane-local inclusive sums of each packet, then the packet totals are scanned across the wave; rows
    // are chained by the wave-uniform carry. Afterwards v[j] holds the running sums within this wave's
    // 4 * VPT * 64 elements (what comes before the wave is added at the write-back).
    uint32_t carry = Op::identity;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        v[j].y = Op::apply(v[j].y, v[j].x);
        v[j].z = Op::apply(v[j].z, v[j].y);
        v[j].w = Op::apply(v[j].w, v[j].z);
        const uint32_t inclusive = wave_inclusive_scan_op<Op>(v[j].w);
        const uint32_t before = Op::apply(carry, wave_exclusive_from_inclusive<Op>(inclusive, v[j].w, lane));
#pragma unroll
        for (int c = 0; c < 4; ++c) v[j][c] = Op::apply(v[j][c], before);
        carry = Op::apply(carry, wave_last_lane(inclusive));
    }
    if (lane == 0) s_wave_total[wave] = carry;
    __syncthreads();

    uint32_t wave_prefix = Op::identity;
    uint32_t aggregate = Op::identity;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        const uint32_t t = s_wave_total[w];
        if (w < wave) wave_prefix = Op::apply(wave_prefix, t);
        aggregate = Op::apply(aggregate, t);
    }

    if (wave == 0) {
        const uint32_t calls = hdr.x;
        const uint32_t parity = calls & 1u;
        u64* const mine = &status[2 * static_cast<size_t>(tile) + parity];
        uint32_t prefix = Op::identity;
        if (hdr.w != kMagic) {
            // Not a workspace scan_workspace_init() has seen: nothing in it can be trusted, so nothing is read
            // or written beyond this report, and the output of the call is invalid.
            if (lane == 0) __hip_atomic_store(&header[kHdrBadWorkspace], tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            // Counted in before anything is published: the tile that closes the call waits for this count,
            // because with helping its look-back can be complete before every tile has read the header.
            if (lane == 0) __hip_atomic_fetch_add(&header[kHdrDone], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (tile == 0) {
                if (lane == 0) publish(mine, kPrefix, aggregate);
            } else {
                if (lane == 0) publish(mine, kAggregate, aggregate);
                prefix = look_back<Op, VEC, TILE>(status, parity, tile, lane, spin_limit, help, in, &header[kHdrReport],
                                                  &header[kHdrBadWorkspace]);
            }
            // The first publication is complete (and with it every poll) before the second one and, behind the
            // barrier below, the output stores are issued: a helper that finds this tile unpublished after its
            // reads have returned has read input, not output.
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kLgkmMax));
            if (tile != 0 && lane == 0) publish(mine, kPrefix, Op::apply(aggregate, prefix));
            clear_other_parity(status, hdr, tile, tiles, lane);
            if (tile == tiles - 1 && lane == 0) {
                // The last tile closes the call once every tile has read the header (normally all have: its
                // look-back saw them published; only tiles it helped may be missing, and they need no one).
                uint32_t spins = 0;
                while (__hip_atomic_load(&header[kHdrDone], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != tiles) {
                    if (++spins > kSpinLimit) {
                        __hip_atomic_store(&header[kHdrReport], tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(8);
                }
                close_call(header, hdr, tiles);
            }
        }
        if (lane == 0) s_tile_prefix = prefix;
    }
    __syncthreads();
    const uint32_t base_sum = Op::apply(s_tile_prefix, wave_prefix);

    // Exclusive sums: element c of a packet gets the running sum of element c - 1; element 0 that of the
    // previous lane's last element (wave_shr:1), lane 0 that of the row before (0 for the first row).
    uint32_t row_before = 0u;
    auto shifted = [&](int j) {
        const uint32_t from_lane_below = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(
            static_cast<int>(row_before), static_cast<int>(v[j].w), 0x138 /* wave_shr:1 */, 0xf, 0xf, false));
        row_before = wave_last_lane(v[j].w);
        return u32x4{from_lane_below, v[j].x, v[j].y, v[j].z};
    };
    if (full) {
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            u32x4 r;
            if constexpr (EXCLUSIVE) {
                r = shifted(j) + base_sum;
            } else if constexpr (Op::kIsSum) {
                r = v[j] + base_sum;
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) r[c] = Op::apply(v[j][c], base_sum);
            }
            stream_store(reinterpret_cast<u32x4*>(out + lane_base + j * ROW_ELEMS), r);
        }
    } else {
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            u32x4 r;
            if constexpr (EXCLUSIVE) r = shifted(j);
            else r = v[j];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const size_t i = lane_base + j * ROW_ELEMS + c;
                if (i < n) out[i] = Op::apply(r[c], base_sum);
            }
        }
    }
}

// ------------------------------------------------------------------ segmented scan --
//
// Inclusive sums that start again at every element whose head flag is set: the same single pass over
// (flag, value) pairs, flag = "a head lies in the range the value covers", combined as
// (fa, va) (+) (fb, vb) = (fa | fb, fb ? vb : va + vb), a earlier than b. The operator is associative but not
// commutative, so every combination below keeps the order of the elements. The reference scans one segment
// (examples/scan.py:200-227); this is the decomposition of that kernel with the pair in place of the sum.
// A status word carries the pair: state in bits 0-7, flag in bit 8, value in the upper half.
struct Seg {
    uint32_t f, v;
};
__device__ __forceinline__ Seg seg_combine(Seg a, Seg b) { return Seg{a.f | b.f, b.f ? b.v : a.v + b.v}; }

template <int CTRL, int ROW_MASK, bool ZERO_FILL>
__device__ __forceinline__ Seg seg_dpp(Seg x) {  // lanes without a source receive (0, 0), the identity
    return Seg{dpp<CTRL, ROW_MASK, ZERO_FILL>(x.f), dpp<CTRL, ROW_MASK, ZERO_FILL>(x.v)};
}
__device__ __forceinline__ Seg wave_inclusive_scan_seg(Seg x) {
    x = seg_combine(seg_dpp<0x111, 0xf, true>(x), x);
    x = seg_combine(seg_dpp<0x112, 0xf, true>(x), x);
    x = seg_combine(seg_dpp<0x114, 0xf, true>(x), x);
    x = seg_combine(seg_dpp<0x118, 0xf, true>(x), x);
    x = seg_combine(seg_dpp<0x142, 0xa, false>(x), x);
    x = seg_combine(seg_dpp<0x143, 0xc, false>(x), x);
    return x;
}
__device__ __forceinline__ u64 pack_seg_status(uint32_t state, Seg p) {
    return static_cast<u64>(state | (p.f << 8)) | (static_cast<u64>(p.v) << 32);
}

// The pair of one whole tile, formed by one wavefront from the tile's input and head bytes: what a look-back
// does for a predecessor that does not answer (see tile_aggregate). Two commutative reductions stand in for the
// ordered one: the position of the tile's last head, then the sum of everything from there on.
template <bool VEC, int TILE>
__device__ __forceinline__ Seg tile_aggregate_seg(const uint32_t* in, const uint8_t* heads, size_t tile_base, int lane) {
    int last = -1;  // index within the tile of the last head this lane has seen
    uint32_t acc = 0u;
    if constexpr (VEC) {
        const uint32_t* hsrc = reinterpret_cast<const uint32_t*>(heads + tile_base) + lane;
#pragma unroll 1
        for (int i = 0; i < TILE / 4 / kWave; ++i) {
            const uint32_t hb = hsrc[static_cast<size_t>(i) * kWave];
            if (hb != 0u) last = 4 * (i * kWave + lane) + (31 - __builtin_clz(hb)) / 8;  // increasing with i
        }
        last = static_cast<int>(wave_last_lane(wave_inclusive_scan_op<MaxI32Op>(static_cast<uint32_t>(last))));
        const u32x4* src = reinterpret_cast<const u32x4*>(in + tile_base) + lane;
#pragma unroll 1
        for (int i = 0; i < TILE / 4 / kWave; ++i) {
            const u32x4 x = src[static_cast<size_t>(i) * kWave];
            const int at = 4 * (i * kWave + lane);
            acc += (at >= last ? x.x : 0u) + (at + 1 >= last ? x.y : 0u) + (at + 2 >= last ? x.z : 0u) + (at + 3 >= last ? x.w : 0u);
        }
    } else {
        const uint8_t* hsrc = heads + tile_base + lane;
#pragma unroll 1
        for (int i = 0; i < TILE / kWave; ++i)
            if (hsrc[static_cast<size_t>(i) * kWave] != 0) last = i * kWave + lane;
        last = static_cast<int>(wave_last_lane(wave_inclusive_scan_op<MaxI32Op>(static_cast<uint32_t>(last))));
        const uint32_t* src = in + tile_base + lane;
#pragma unroll 1
        for (int i = 0; i < TILE / kWave; ++i) {
            const uint32_t x = src[static_cast<size_t>(i) * kWave];
            acc += (i * kWave + lane >= last) ? x : 0u;
        }
    }
    return Seg{last >= 0 ? 1u : 0u, wave_last_lane(wave_inclusive_scan(acc))};
}

// The pair that everything before tile `tile` (> 0) contributes to it. The walk back ends at the nearest
// tile that has published a prefix or whose own range holds a head: what lies before a head does not matter.
// A predecessor that has not answered after spin_limit polls is helped (tile_aggregate_seg) or, without
// `help`, reported, as in look_back.
template <bool VEC, int TILE>
__device__ __forceinline__ Seg look_back_seg(const u64* status, uint32_t parity, uint32_t tile, int lane,
                                             uint32_t spin_limit, bool help, const uint32_t* in, const uint8_t* heads,
                                             uint32_t* report, uint32_t* bad_workspace) {
    Seg sum{0u, 0u};
    uint32_t spins = 0;
    long long window_end = static_cast<long long>(tile) - 1;
    while (true) {
        const long long t = window_end - lane;
        const u64 w = (t >= 0) ? poll(&status[2 * t + parity]) : pack_status(kPrefix, 0u);
        uint32_t state = static_cast<uint32_t>(w) & 0xffu;
        uint32_t flag = (static_cast<uint32_t>(w) >> 8) & 1u;
        uint32_t value = static_cast<uint32_t>(w >> 32);
        if (__ballot(state > kPrefix || (static_cast<uint32_t>(w) >> 9) != 0u)) {  // no tile writes such a word
            if (lane == 0) __hip_atomic_store(bad_workspace, tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
        const u64 is_invalid = __ballot(state == kInvalid);
        const u64 ends_walk = __ballot(state == kPrefix || flag != 0u);
        const int first_invalid = is_invalid ? __builtin_ctzll(is_invalid) : kWave;
        int first_end = ends_walk ? __builtin_ctzll(ends_walk) : kWave;
        if (first_end >= first_invalid && first_invalid < kWave) {  // a tile that has not answered is needed
            if (spins < spin_limit) {
                ++spins;
                continue;
            }
            if (!help) {
                if (lane == 0) __hip_atomic_store(report, tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            // Nearest first, until the end of the walk is known: a helped tile that holds a head ends it.
            for (u64 todo = is_invalid; todo != 0; todo &= todo - 1) {
                const int l = __builtin_ctzll(todo);
                if (l > first_end) break;
                const Seg formed = tile_aggregate_seg<VEC, TILE>(in, heads, static_cast<size_t>(window_end - l) * TILE, lane);
                // As in look_back: all reads of that tile's input have returned; a word it has published by now
                // is the truth, otherwise it has stored no output yet and `formed` is the pair of its input.
                const u64 again = poll(&status[2 * (window_end - l) + parity]);
                const uint32_t st = static_cast<uint32_t>(again) & 0xffu;
                const uint32_t s_l = st != kInvalid ? st : kAggregate;
                const uint32_t f_l = st != kInvalid ? (static_cast<uint32_t>(again) >> 8) & 1u : formed.f;
                const uint32_t v_l = st != kInvalid ? static_cast<uint32_t>(again >> 32) : formed.v;
                if (lane == l) {
                    state = s_l;
                    flag = f_l;
                    value = v_l;
                }
                if ((s_l == kPrefix || f_l != 0u) && l < first_end) first_end = l;
            }
        }
        spins = 0;
        // Lanes 0 .. last are valid; none before `last` holds a head, so their values simply add up
        // (lane 0 is the nearest tile; the order does not matter for flagless pairs).
        const int last = first_end < kWave ? first_end : kWave - 1;
        const uint32_t contrib = lane <= last ? value : 0u;
        sum.v += wave_last_lane(wave_inclusive_scan(contrib));
        if (first_end < kWave) {
            sum.f = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(flag), first_end));
            break;
        }
        window_end -= kWave;
    }
    return sum;
}

// heads: one byte per element, non-zero = the element starts a segment. VEC: in and out 16 B aligned and
// heads 4 B aligned.
template <typename Cfg, bool VEC>
__global__ __launch_bounds__(Cfg::BLOCK) void segmented_scan_lookback_kernel(const uint32_t* in, const uint8_t* heads,
                                                                             uint32_t* out, size_t n, uint32_t* header,
                                                                             u64* status, uint32_t spin_limit, bool help) {
    constexpr int BLOCK = Cfg::BLOCK, VPT = Cfg::VPT;
    constexpr int WAVES = BLOCK / kWave;
    constexpr int TILE = BLOCK * VPT * 4;
    constexpr int WAVE_ELEMS = kWave * VPT * 4;
    constexpr int ROW_ELEMS = kWave * 4;
    static_assert(VPT <= 16, "four `head seen` bits per packet are kept in two 32-bit masks");

    __shared__ uint32_t s_wave_f[WAVES], s_wave_v[WAVES];
    __shared__ uint32_t s_tile_prefix_v;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t tiles = gridDim.x;
    const uint32_t tile = tile_of_workgroup(blockIdx.x, tiles);

    const size_t tile_base = static_cast<size_t>(tile) * TILE;
    const size_t lane_base = tile_base + static_cast<size_t>(wave) * WAVE_ELEMS + lane * 4;
    const bool full = VEC && (tile_base + TILE <= n);

    // The head bytes of the tile wait in LDS (a dword per packet, row j of a wave at my_heads + 64 j) until
    // the packet is scanned: sixteen more registers per lane would not fit beside the tile itself. Whole
    // tiles fetch them with direct-to-LDS loads, issued in front of the value loads.
    __shared__ uint32_t s_heads[BLOCK * VPT];
    uint32_t* const my_heads = &s_heads[wave * VPT * kWave];
    u32x4 v[VPT];
    if (full) {
        const char* wave_heads = reinterpret_cast<const char*>(heads + tile_base + static_cast<size_t>(wave) * WAVE_ELEMS);
#pragma unroll
        for (int j = 0; j < VPT; ++j) direct_load4(wave_heads + j * ROW_ELEMS, lane * 4u, my_heads + j * kWave);
#pragma unroll
        for (int j = 0; j < VPT; ++j)
            v[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(in + lane_base + j * ROW_ELEMS));
    } else {
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            uint32_t hb = 0u;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const size_t i = lane_base + j * ROW_ELEMS + c;
                v[j][c] = (i < n) ? in[i] : 0u;
                if (i < n && heads[i] != 0) hb |= 1u << (8 * c);
            }
            my_heads[j * kWave + lane] = hb;
        }
    }
    u32x4 hdr = {0u, 0u, 0u, 0u};
    if (wave == 0) hdr = *reinterpret_cast<const u32x4*>(header + kHdrCalls);
    // The direct loads are invisible to the compiler's wait counts; a wave reads only what it loaded itself.
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("" ::: "memory");

    // seen[j / 8], bit 4 (j % 8) + c: a head lies between the start of this wave's part and element c of packet j.
    uint32_t seen[2] = {0u, 0u};
    Seg carry{0u, 0u};
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const uint32_t hb = my_heads[j * kWave + lane];
        const bool h0 = (hb & 0x000000ffu) != 0, h1 = (hb & 0x0000ff00u) != 0, h2 = (hb & 0x00ff0000u) != 0,
                   h3 = (hb & 0xff000000u) != 0;
        v[j].y = h1 ? v[j].y : v[j].x + v[j].y;
        v[j].z = h2 ? v[j].z : v[j].y + v[j].z;
        v[j].w = h3 ? v[j].w : v[j].z + v[j].w;
        const uint32_t s0 = h0, s1 = s0 | h1, s2 = s1 | h2, s3 = s2 | h3;  // head seen up to element c of the packet
        const Seg inclusive = wave_inclusive_scan_seg(Seg{s3, v[j].w});
        // what the lanes below contribute (identity in lane 0), then what the rows before do
        Seg below{static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(inclusive.f), 0x138, 0xf, 0xf, false)),
                  static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(inclusive.v), 0x138, 0xf, 0xf, false))};
        const Seg before = seg_combine(carry, below);
        v[j].x += s0 ? 0u : before.v;
        v[j].y += s1 ? 0u : before.v;
        v[j].z += s2 ? 0u : before.v;
        v[j].w += s3 ? 0u : before.v;
        const uint32_t bf = before.f;
        seen[j / 8] |= ((s0 | bf) | ((s1 | bf) << 1) | ((s2 | bf) << 2) | ((s3 | bf) << 3)) << (4 * (j % 8));
        carry = seg_combine(carry, Seg{wave_last_lane(inclusive.f), wave_last_lane(inclusive.v)});
        // The packet's sums are final here: said explicitly, because the compiler otherwise postpones the
        // additions above to the write-back and keeps their operands and conditions alive until then.
        asm volatile("" : "+v"(v[j]));
    }
    // From here on the masks are all the compiler knows about the heads (it would otherwise keep three
    // conditions per packet alive until the write-back: 48 spilled registers in the big tile).
    asm volatile("" : "+v"(seen[0]), "+v"(seen[1]));
    if (lane == 0) {
        s_wave_f[wave] = carry.f;
        s_wave_v[wave] = carry.v;
    }
    __syncthreads();

    Seg wave_prefix{0u, 0u}, aggregate{0u, 0u};
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        const Seg t{s_wave_f[w], s_wave_v[w]};
        if (w < wave) wave_prefix = seg_combine(wave_prefix, t);
        aggregate = seg_combine(aggregate, t);
    }

    if (wave == 0) {
        const uint32_t parity = hdr.x & 1u;
        u64* const mine = &status[2 * static_cast<size_t>(tile) + parity];
        Seg prefix{0u, 0u};
        if (hdr.w != kMagic) {  // not an initialised workspace: report, touch nothing else
            if (lane == 0) __hip_atomic_store(&header[kHdrBadWorkspace], tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (tile == 0) {
            if (lane == 0) __hip_atomic_store(mine, pack_seg_status(kPrefix, aggregate), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            if (lane == 0) __hip_atomic_store(mine, pack_seg_status(kAggregate, aggregate), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            prefix = look_back_seg<VEC, TILE>(status, parity, tile, lane, spin_limit, help, in, heads, &header[kHdrReport],
                                              &header[kHdrBadWorkspace]);
        }
        // The first publication is complete before the second one and, behind the barrier below, the output
        // stores are issued: a helper that finds this tile unpublished after its reads have returned has read
        // input, not output.
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kLgkmMax));
        if (hdr.w == kMagic && tile != 0 && lane == 0)
            __hip_atomic_store(mine, pack_seg_status(kPrefix, seg_combine(prefix, aggregate)), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        if (lane == 0) s_tile_prefix_v = prefix.v;
        if (hdr.w == kMagic) clear_other_parity(status, hdr, tile, tiles, lane);
    }
    __syncthreads();
    // What comes before this wave: the tile's prefix, unless a head in an earlier wave of the tile cuts it off.
    const uint32_t base = seg_combine(Seg{0u, s_tile_prefix_v}, wave_prefix).v;

    if (full) {
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            const uint32_t bits = seen[j / 8] >> (4 * (j % 8));
            u32x4 r = v[j];
            r.x += (bits & 1u) ? 0u : base;
            r.y += (bits & 2u) ? 0u : base;
            r.z += (bits & 4u) ? 0u : base;
            r.w += (bits & 8u) ? 0u : base;
            stream_store(reinterpret_cast<u32x4*>(out + lane_base + j * ROW_ELEMS), r);
        }
    } else {
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            const uint32_t bits = seen[j / 8] >> (4 * (j % 8));
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const size_t i = lane_base + j * ROW_ELEMS + c;
                if (i < n) out[i] = v[j][c] + (((bits >> c) & 1u) ? 0u : base);
            }
        }
    }
    // A look-back that ended at a head says nothing about the tiles before that head, so the last tile's
    // look-back cannot tell that every tile has read the header. Tiles count themselves off instead, and
    // the one that counts last closes the call.
    if (tid == 0 && hdr.w == kMagic) {
        const uint32_t done = __hip_atomic_fetch_add(&header[kHdrDone], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (done == tiles - 1) close_call(header, hdr, tiles);
    }
}

// ------------------------------------------------------------------ 64-bit elements --
//
// Inclusive sums of 64-bit elements modulo 2^64 (int64 and uint64 share the bits): the same single pass with
// two elements per 16 B packet. A 64-bit value does not fit a 64-bit status word beside its state, so a tile
// owns two status slots, {state, low half} and {state, high half}; a reader accepts the pair only when both
// carry the same state (a tile rewrites both on its way from aggregate to prefix, low half first) and polls
// again otherwise. The reference scans uint32 (evals/4090_scan/scan_harness.cuh:30-36); this is its
// decomposition (examples/scan.py:106-227) on wider elements.
typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));

template <int CTRL, int ROW_MASK, bool ZERO_FILL>
__device__ __forceinline__ u64 dpp64(u64 x) {
    return static_cast<u64>(dpp<CTRL, ROW_MASK, ZERO_FILL>(static_cast<uint32_t>(x))) |
           (static_cast<u64>(dpp<CTRL, ROW_MASK, ZERO_FILL>(static_cast<uint32_t>(x >> 32))) << 32);
}
__device__ __forceinline__ u64 wave_inclusive_scan64(u64 x) {
    x += dpp64<0x111, 0xf, true>(x);
    x += dpp64<0x112, 0xf, true>(x);
    x += dpp64<0x114, 0xf, true>(x);
    x += dpp64<0x118, 0xf, true>(x);
    x += dpp64<0x142, 0xa, false>(x);
    x += dpp64<0x143, 0xc, false>(x);
    return x;
}
__device__ __forceinline__ u64 wave_last_lane64(u64 x) {
    return static_cast<u64>(wave_last_lane(static_cast<uint32_t>(x))) | (static_cast<u64>(wave_last_lane(static_cast<uint32_t>(x >> 32))) << 32);
}
__device__ __forceinline__ void publish64(u64* lo_word, uint32_t state, u64 value) {  // the high half sits one slot on
    publish(lo_word, state, static_cast<uint32_t>(value));
    publish(lo_word + 2, state, static_cast<uint32_t>(value >> 32));
}

// The sum of one whole tile of 64-bit elements, formed by one wavefront from the tile's input (see tile_aggregate).
template <bool VEC, int TILE>
__device__ __forceinline__ u64 tile_aggregate64(const u64* in, size_t tile_base, int lane) {
    u64 acc = 0;
    if constexpr (VEC) {
        const u64x2* src = reinterpret_cast<const u64x2*>(in + tile_base) + lane;
#pragma unroll 1
        for (int i = 0; i < TILE / 2 / kWave; i += 2) {
            const u64x2 x = src[static_cast<size_t>(i) * kWave], y = src[static_cast<size_t>(i + 1) * kWave];
            acc += (x.x + x.y) + (y.x + y.y);
        }
    } else {
        const u64* src = in + tile_base + lane;
#pragma unroll 1
        for (int i = 0; i < TILE / kWave; i += 2) acc += src[static_cast<size_t>(i) * kWave] + src[static_cast<size_t>(i + 1) * kWave];
    }
    return wave_last_lane64(wave_inclusive_scan64(acc));
}

// Sum of all tiles before `tile` (> 0). Lane l inspects tile window_end - l: slots 2 t and 2 t + 1. A
// predecessor that has not answered after spin_limit polls is helped (tile_aggregate64) or, without `help`,
// reported, as in look_back.
template <bool VEC, int TILE>
__device__ __forceinline__ u64 look_back64(const u64* status, uint32_t parity, uint32_t tile, int lane, uint32_t spin_limit,
                                           bool help, const u64* in, uint32_t* report, uint32_t* bad_workspace) {
    u64 sum = 0;
    uint32_t spins = 0;
    long long window_end = static_cast<long long>(tile) - 1;
    while (true) {
        const long long t = window_end - lane;
        const u64 lo = (t >= 0) ? poll(&status[4 * t + parity]) : pack_status(kPrefix, 0u);
        const u64 hi = (t >= 0) ? poll(&status[4 * t + 2 + parity]) : pack_status(kPrefix, 0u);
        const uint32_t state_lo = static_cast<uint32_t>(lo), state_hi = static_cast<uint32_t>(hi);
        if (__ballot(state_lo > kPrefix || state_hi > kPrefix)) {  // no tile writes such a word
            if (lane == 0) __hip_atomic_store(bad_workspace, tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
        // halves of two different publications (or one still missing) count as "nothing yet"
        uint32_t state = state_lo == state_hi ? state_lo : kInvalid;
        u64 value = (lo >> 32) | (hi & 0xffffffff00000000ull);
        u64 has_prefix = __ballot(state == kPrefix);
        const u64 is_invalid = __ballot(state == kInvalid);
        u64 needed = has_prefix ? ((2ull << __builtin_ctzll(has_prefix)) - 1ull) : ~0ull;
        if (is_invalid & needed) {
            if (spins < spin_limit) {
                ++spins;
                continue;
            }
            if (!help) {
                if (lane == 0) __hip_atomic_store(report, tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            for (u64 todo = is_invalid & needed; todo != 0; todo &= todo - 1) {
                const int l = __builtin_ctzll(todo);
                const u64 formed = tile_aggregate64<VEC, TILE>(in, static_cast<size_t>(window_end - l) * TILE, lane);
                // As in look_back. A tile stores output only after both halves of its prefix are published, so a
                // pair that is still missing or mixed here means that `formed` is the sum of its input.
                const u64 lo2 = poll(&status[4 * (window_end - l) + parity]), hi2 = poll(&status[4 * (window_end - l) + 2 + parity]);
                const uint32_t s2 = static_cast<uint32_t>(lo2);
                const bool published = s2 == static_cast<uint32_t>(hi2) && s2 != kInvalid;
                if (lane == l) {
                    state = published ? s2 : kAggregate;
                    value = published ? ((lo2 >> 32) | (hi2 & 0xffffffff00000000ull)) : formed;
                }
            }
            has_prefix = __ballot(state == kPrefix);
            needed = has_prefix ? ((2ull << __builtin_ctzll(has_prefix)) - 1ull) : ~0ull;
        }
        spins = 0;
        const u64 contrib = ((needed >> lane) & 1ull) ? value : 0ull;
        sum += wave_last_lane64(wave_inclusive_scan64(contrib));
        if (has_prefix) break;
        window_end -= kWave;
    }
    return sum;
}

// VEC: in and out are 16 B aligned. One tile shape: a tile of 2 * BLOCK * VPT elements owns two status slots,
// which is what the workspace holds per 32768 elements.
template <typename Cfg, bool VEC>
__global__ __launch_bounds__(Cfg::BLOCK) void scan64_lookback_kernel(const u64* in, u64* out, size_t n, uint32_t* header,
                                                                     u64* status, uint32_t spin_limit, bool help) {
    constexpr int BLOCK = Cfg::BLOCK, VPT = Cfg::VPT;
    constexpr int WAVES = BLOCK / kWave;
    constexpr int TILE = BLOCK * VPT * 2;
    constexpr int WAVE_ELEMS = kWave * VPT * 2;
    constexpr int ROW_ELEMS = kWave * 2;
    static_assert(TILE >= 2 * static_cast<int>(kWorkspaceTileElems), "two status slots per tile");

    __shared__ u64 s_wave_total[WAVES];
    __shared__ u64 s_tile_prefix;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t tiles = gridDim.x;
    const uint32_t tile = tile_of_workgroup(blockIdx.x, tiles);

    const size_t tile_base = static_cast<size_t>(tile) * TILE;
    const size_t lane_base = tile_base + static_cast<size_t>(wave) * WAVE_ELEMS + lane * 2;
    const bool full = VEC && (tile_base + TILE <= n);

    u64x2 v[VPT];
    if (full) {
#pragma unroll
        for (int j = 0; j < VPT; ++j)
            v[j] = __builtin_nontemporal_load(reinterpret_cast<const u64x2*>(in + lane_base + j * ROW_ELEMS));
    } else {
#pragma unroll
        for (int j = 0; j < VPT; ++j)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const size_t i = lane_base + j * ROW_ELEMS + c;
                v[j][c] = (i < n) ? in[i] : 0ull;
            }
    }
    u32x4 hdr = {0u, 0u, 0u, 0u};
    if (wave == 0) hdr = *reinterpret_cast<const u32x4*>(header + kHdrCalls);

    u64 carry = 0;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        v[j].y += v[j].x;
        const u64 inclusive = wave_inclusive_scan64(v[j].y);
        const u64 before = carry + (inclusive - v[j].y);
        v[j].x += before;
        v[j].y += before;
        carry += wave_last_lane64(inclusive);
    }
    if (lane == 0) s_wave_total[wave] = carry;
    __syncthreads();

    u64 wave_prefix = 0, aggregate = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        const u64 t = s_wave_total[w];
        if (w < wave) wave_prefix += t;
        aggregate += t;
    }

    if (wave == 0) {
        const uint32_t parity = hdr.x & 1u;
        u64* const mine = &status[4 * static_cast<size_t>(tile) + parity];
        u64 prefix = 0;
        if (hdr.w != kMagic) {  // not an initialised workspace: report, touch nothing else
            if (lane == 0) __hip_atomic_store(&header[kHdrBadWorkspace], tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            // Counted in before anything is published, as in scan_lookback_kernel: with helping the last tile's
            // look-back can be complete before every tile has read the header.
            if (lane == 0) __hip_atomic_fetch_add(&header[kHdrDone], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (tile == 0) {
                if (lane == 0) publish64(mine, kPrefix, aggregate);
            } else {
                if (lane == 0) publish64(mine, kAggregate, aggregate);
                prefix = look_back64<VEC, TILE>(status, parity, tile, lane, spin_limit, help, in, &header[kHdrReport],
                                                &header[kHdrBadWorkspace]);
            }
            // The first publication is complete before the second one and the output stores are issued (see
            // scan_lookback_kernel).
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kLgkmMax));
            if (tile != 0 && lane == 0) publish64(mine, kPrefix, aggregate + prefix);
            // The workspace protocol counts status slots: this tile's are 2 t and 2 t + 1 of 2 * tiles.
            clear_other_parity(status, hdr, 2 * tile, 2 * tiles, lane);
            clear_other_parity(status, hdr, 2 * tile + 1, 2 * tiles, lane);
            if (tile == tiles - 1 && lane == 0) {  // closes the call once every tile has read the header
                uint32_t waited = 0;
                while (__hip_atomic_load(&header[kHdrDone], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != tiles) {
                    if (++waited > kSpinLimit) {
                        __hip_atomic_store(&header[kHdrReport], tile + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(8);
                }
                close_call(header, hdr, 2 * tiles);
            }
        }
        if (lane == 0) s_tile_prefix = prefix;
    }
    __syncthreads();
    const u64 base = s_tile_prefix + wave_prefix;

    if (full) {
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            const u64x2 r = v[j] + base;
            u32x4 bits;
            __builtin_memcpy(&bits, &r, 16);
            stream_store(reinterpret_cast<u32x4*>(out + lane_base + j * ROW_ELEMS), bits);
        }
    } else {
#pragma unroll
        for (int j = 0; j < VPT; ++j)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const size_t i = lane_base + j * ROW_ELEMS + c;
                if (i < n) out[i] = v[j][c] + base;
            }
    }
}

// Initial state of a workspace: all zeros but for the magic word of the header (a kernel, not hipMemsetAsync, so
// that it can be captured into a graph). Words 6 and 7 of the header share 64-bit word 3.
__global__ __launch_bounds__(256) void scan_fill_zero_kernel(u64* words, size_t n_words) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n_words) words[i] = (i == kHdrMagic / 2) ? (static_cast<u64>(kMagic) << 32) : 0ull;
}

inline bool use_small(size_t n, bool vec) { return n <= kSmallMax || !vec; }

// Calls f with std::true_type or std::false_type for a run-time flag.
template <typename F>
void with_flag(bool flag, F&& f) {
    if (flag) f(std::true_type{});
    else f(std::false_type{});
}

template <typename Cfg, bool VEC>
int launch_cfg(const uint32_t* in, uint32_t* out, size_t n, uint32_t* header, u64* status, unsigned flags,
               uint32_t limit, hipStream_t s) {
    const size_t tiles = ceil_div(n, static_cast<size_t>(tile_elems<Cfg>()));
    const dim3 grid(static_cast<unsigned>(tiles)), block(Cfg::BLOCK);
    const int op = static_cast<int>(flags & kFlagOpMask);
    const bool help = (flags & kFlagNoHelp) == 0;
    if (op == kFlagOpMax)
        scan_lookback_kernel<Cfg, VEC, false, false, MaxI32Op><<<grid, block, 0, s>>>(in, out, n, header, status, limit, help);
    else if (op == kFlagOpMin)
        scan_lookback_kernel<Cfg, VEC, false, false, MinI32Op><<<grid, block, 0, s>>>(in, out, n, header, status, limit, help);
    else
        with_flag((flags & kFlagTicket) != 0, [&](auto ticket) {
            with_flag((flags & kFlagExclusive) != 0, [&](auto excl) {
                scan_lookback_kernel<Cfg, VEC, decltype(ticket)::value, decltype(excl)::value>
                    <<<grid, block, 0, s>>>(in, out, n, header, status, limit, help);
            });
        });
    return check_launch("scan_lookback_kernel");
}

// ------------------------------------------------------------- library-owned scratch --
//
// Workspace for callers that cannot allocate (prism_scan_i32_static): a device array that lives as
// long as the module. Every GPU holds its own copy at its own address; host code must use the
// address hipGetSymbolAddress returns, never the array's name.
constexpr size_t kStaticMaxElems = size_t{1} << 31;
constexpr size_t kStaticBytes = kHeaderBytes + 16 * (kStaticMaxElems / kWorkspaceTileElems + 1);
static __device__ __align__(256) unsigned char scratch[kStaticBytes];  // initialised by the first call on a device

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int scan_workspace_init_impl(void* ws, size_t ws_bytes, hipStream_t s);

// Device address of `scratch` on the current device. Looked up once per device; that first call also
// enqueues a zero fill on `s`, so that nothing rests on what the array held before.
int static_scratch(void** ptr, hipStream_t s) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(1, "prism_scan: device %d outside the supported range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        // The one-time set-up must not end up in a graph (its fill would run again on every replay).
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
            return fail(1, "prism_scan_i32_static: the first call on a device sets the library's scratch array up and must be "
                           "made outside stream capture (prism_scan_status(NULL, 0, stream) does it as well)");
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        if (p == nullptr) return fail(1, "hipGetSymbolAddress(scratch) returned no address");
        if (int rc = scan_workspace_init_impl(p, kStaticBytes, s)) return rc;
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

}  // namespace

size_t scan_workspace_bytes(size_t n) {
    // One 16-byte slot per 16384 elements and one to spare: a tile of 64-bit elements (32768 of them) owns two.
    return kHeaderBytes + 16 * (ceil_div(n, kWorkspaceTileElems) + 1);
}

int scan_workspace_init(void* ws, size_t ws_bytes, hipStream_t s) { return scan_workspace_init_impl(ws, ws_bytes, s); }

namespace {
int scan_workspace_init_impl(void* ws, size_t ws_bytes, hipStream_t s) {
    if (ws == nullptr || ws_bytes < kHeaderBytes + 16)
        return fail(1, "prism_scan_workspace_init: workspace of %zu bytes is too small", ws_bytes);
    if ((reinterpret_cast<uintptr_t>(ws) & 15u) != 0)
        return fail(1, "prism_scan_workspace_init: workspace must be 16-byte aligned");
    const size_t n_words = ws_bytes / sizeof(u64);
    scan_fill_zero_kernel<<<dim3(static_cast<unsigned>(ceil_div(n_words, size_t{256}))), dim3(256), 0, s>>>(
        reinterpret_cast<u64*>(ws), n_words);
    return check_launch("scan_fill_zero_kernel");
}
}  // namespace

int launch_scan(const uint32_t* in, uint32_t* out, size_t n, void* ws, size_t ws_bytes, unsigned flags,
                long long spin_limit, hipStream_t s) {
    if (n == 0) return 0;
    if (in == nullptr || out == nullptr || ws == nullptr)
        return fail(1, "prism_scan: null pointer with n=%zu", n);
    if (!aligned4(in) || !aligned4(out)) return fail(1, "prism_scan: data pointers must be 4-byte aligned");
    if ((reinterpret_cast<uintptr_t>(ws) & 15u) != 0)
        return fail(1, "prism_scan: workspace must be 16-byte aligned");
    const int op = static_cast<int>(flags & kFlagOpMask);
    if ((flags & ~(kFlagExclusive | kFlagTicket | kFlagNoHelp | kFlagOpMask)) != 0 || op > kFlagOpMin)
        return fail(1, "prism_scan: unknown flag bits 0x%x", flags);
    if (op != kFlagOpSum && (flags & (kFlagExclusive | kFlagTicket)) != 0)
        return fail(1, "prism_scan: the running maximum / minimum is inclusive and numbers tiles by workgroup id");
    const size_t need = scan_workspace_bytes(n);
    if (ws_bytes < need)
        return fail(1, "prism_scan: workspace of %zu bytes is smaller than the %zu needed for n=%zu",
                    ws_bytes, need, n);
    if (in != out) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(in), b = reinterpret_cast<uintptr_t>(out);
        const uintptr_t bytes = n * sizeof(uint32_t);
        if (a < b + bytes && b < a + bytes)
            return fail(1, "prism_scan: in and out overlap without being equal");
    }
    if (ceil_div(n, kWorkspaceTileElems) > 0x7fffffffull) return fail(1, "prism_scan: n=%zu too large", n);
    const uint32_t limit = spin_limit < 0 ? ((flags & kFlagNoHelp) ? kSpinLimit : kHelpAfter)
                                          : static_cast<uint32_t>(spin_limit > 0xffffffffll ? 0xffffffffll : spin_limit);

    uint32_t* header = reinterpret_cast<uint32_t*>(ws);
    u64* status = reinterpret_cast<u64*>(static_cast<char*>(ws) + kHeaderBytes);
    const bool vec = aligned16(in) && aligned16(out);
    if (!vec) return launch_cfg<SmallCfg, false>(in, out, n, header, status, flags, limit, s);
    if (use_small(n, vec)) return launch_cfg<SmallCfg, true>(in, out, n, header, status, flags, limit, s);
    return launch_cfg<BigCfg, true>(in, out, n, header, status, flags, limit, s);
}

// The limit on the polls of one look-back window for the kinds of scan that take only the no-help flag.
static int help_and_limit(const char* who, unsigned flags, long long spin_limit, bool* help, uint32_t* limit) {
    if ((flags & ~kFlagNoHelp) != 0) return fail(1, "%s: unknown flag bits 0x%x (only PRISM_SCAN_NO_HELP applies)", who, flags);
    *help = (flags & kFlagNoHelp) == 0;
    *limit = spin_limit < 0 ? (*help ? kHelpAfter : kSpinLimit)
                            : static_cast<uint32_t>(spin_limit > 0xffffffffll ? 0xffffffffll : spin_limit);
    return 0;
}

int launch_segmented_scan(const uint32_t* in, const uint8_t* heads, uint32_t* out, size_t n, void* ws, size_t ws_bytes,
                          unsigned flags, long long spin_limit, hipStream_t s) {
    bool help = true;
    uint32_t limit = 0;
    if (int rc = help_and_limit("prism_segmented_scan", flags, spin_limit, &help, &limit)) return rc;
    if (n == 0) return 0;
    if (in == nullptr || out == nullptr || heads == nullptr || ws == nullptr)
        return fail(1, "prism_segmented_scan: null pointer with n=%zu", n);
    if (!aligned4(in) || !aligned4(out)) return fail(1, "prism_segmented_scan: data pointers must be 4-byte aligned");
    if ((reinterpret_cast<uintptr_t>(ws) & 15u) != 0)
        return fail(1, "prism_segmented_scan: workspace must be 16-byte aligned");
    const size_t need = scan_workspace_bytes(n);
    if (ws_bytes < need)
        return fail(1, "prism_segmented_scan: workspace of %zu bytes is smaller than the %zu needed for n=%zu",
                    ws_bytes, need, n);
    const uintptr_t a = reinterpret_cast<uintptr_t>(in), b = reinterpret_cast<uintptr_t>(out),
                    h = reinterpret_cast<uintptr_t>(heads), bytes = n * sizeof(uint32_t);
    if (in != out && a < b + bytes && b < a + bytes)
        return fail(1, "prism_segmented_scan: in and out overlap without being equal");
    if (h < b + bytes && b < h + n) return fail(1, "prism_segmented_scan: heads and out overlap");
    if (ceil_div(n, kWorkspaceTileElems) > 0x7fffffffull) return fail(1, "prism_segmented_scan: n=%zu too large", n);
    uint32_t* header = reinterpret_cast<uint32_t*>(ws);
    u64* status = reinterpret_cast<u64*>(static_cast<char*>(ws) + kHeaderBytes);
    const bool vec = aligned16(in) && aligned16(out) && aligned4(heads);
    const bool small = use_small(n, vec);
    const size_t tiles = ceil_div(n, static_cast<size_t>(small ? tile_elems<SmallCfg>() : tile_elems<BigCfg>()));
    const dim3 grid(static_cast<unsigned>(tiles));
    if (!vec)
        segmented_scan_lookback_kernel<SmallCfg, false><<<grid, dim3(SmallCfg::BLOCK), 0, s>>>(in, heads, out, n, header, status, limit, help);
    else if (small)
        segmented_scan_lookback_kernel<SmallCfg, true><<<grid, dim3(SmallCfg::BLOCK), 0, s>>>(in, heads, out, n, header, status, limit, help);
    else
        segmented_scan_lookback_kernel<BigCfg, true><<<grid, dim3(BigCfg::BLOCK), 0, s>>>(in, heads, out, n, header, status, limit, help);
    return check_launch("segmented_scan_lookback_kernel");
}

int launch_scan64(const unsigned long long* in, unsigned long long* out, size_t n, void* ws, size_t ws_bytes, unsigned flags,
                  long long spin_limit, hipStream_t s) {
    bool help = true;
    uint32_t limit = 0;
    if (int rc = help_and_limit("prism_scan_i64", flags, spin_limit, &help, &limit)) return rc;
    if (n == 0) return 0;
    if (in == nullptr || out == nullptr || ws == nullptr) return fail(1, "prism_scan_i64: null pointer with n=%zu", n);
    if ((reinterpret_cast<uintptr_t>(in) & 7u) != 0 || (reinterpret_cast<uintptr_t>(out) & 7u) != 0)
        return fail(1, "prism_scan_i64: data pointers must be 8-byte aligned");
    if ((reinterpret_cast<uintptr_t>(ws) & 15u) != 0) return fail(1, "prism_scan_i64: workspace must be 16-byte aligned");
    const size_t need = scan_workspace_bytes(n);
    if (ws_bytes < need)
        return fail(1, "prism_scan_i64: workspace of %zu bytes is smaller than the %zu needed for n=%zu", ws_bytes, need, n);
    if (in != out) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(in), b = reinterpret_cast<uintptr_t>(out), bytes = n * sizeof(u64);
        if (a < b + bytes && b < a + bytes) return fail(1, "prism_scan_i64: in and out overlap without being equal");
    }
    constexpr size_t tile = 2 * static_cast<size_t>(BigCfg::BLOCK) * BigCfg::VPT;
    const size_t tiles = ceil_div(n, tile);
    if (tiles > 0x3fffffffull) return fail(1, "prism_scan_i64: n=%zu too large", n);
    uint32_t* header = reinterpret_cast<uint32_t*>(ws);
    u64* status = reinterpret_cast<u64*>(static_cast<char*>(ws) + kHeaderBytes);
    const dim3 grid(static_cast<unsigned>(tiles)), block(BigCfg::BLOCK);
    if (aligned16(in) && aligned16(out))
        scan64_lookback_kernel<BigCfg, true><<<grid, block, 0, s>>>(in, out, n, header, status, limit, help);
    else
        scan64_lookback_kernel<BigCfg, false><<<grid, block, 0, s>>>(in, out, n, header, status, limit, help);
    return check_launch("scan64_lookback_kernel");
}

int launch_scan_static(const uint32_t* in, uint32_t* out, size_t n, hipStream_t s) {
    if (n > kStaticMaxElems)
        return fail(1, "prism_scan_i32_static: n=%zu exceeds the %zu elements the library's scratch array covers",
                    n, kStaticMaxElems);
    if (n == 0) return 0;
    void* ws = nullptr;
    if (int rc = static_scratch(&ws, s)) return rc;
    return launch_scan(in, out, n, ws, kStaticBytes, 0u, -1, s);
}

int scan_status(void* ws, size_t ws_bytes, hipStream_t s) {
    if (ws == nullptr) {  // the library's own scratch array on the current device
        if (int rc = static_scratch(&ws, s)) return rc;
        ws_bytes = kStaticBytes;
    }
    if (ws_bytes < kHeaderBytes + 16) return fail(1, "prism_scan_status: workspace of %zu bytes is too small", ws_bytes);
    hipError_t e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_fail(e, "prism_scan_status: hipStreamSynchronize");
    uint32_t hdr[8] = {};
    e = hipMemcpy(hdr, ws, sizeof(hdr), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "prism_scan_status: hipMemcpy");
    const bool bad_workspace = hdr[kHdrMagic] != kMagic || hdr[kHdrBadWorkspace] != 0;
    const uint32_t report = hdr[kHdrReport];
    if (!bad_workspace && report == 0) return 0;
    // The output of the call that reported is invalid, and the workspace may be in any state (the tile that
    // closes a call may have done so before every tile had started). Bring it back to its initial state.
    if (int rc = scan_workspace_init(ws, ws_bytes, s)) return rc;
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_fail(e, "prism_scan_status: hipStreamSynchronize");
    if (bad_workspace)
        return fail(kScanWorkspaceError,
                    "prism_scan: the workspace was not initialised with prism_scan_workspace_init (or something else "
                    "wrote into it); the output of the scans that used it is invalid. It is initialised now");
    return fail(kScanOrderError,
                "prism_scan: tile %u gave up waiting for its predecessors (a scan without helping whose workgroups did "
                "not start in the assumed order, or a spin limit set too low); the output of that call is invalid",
                report - 1u);
}

}  // namespace prism
