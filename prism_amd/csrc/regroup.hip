// prism_wave_regroup_i32: moves every chunk of 64 N ints between the two arrangements a wavefront can hold it
// in, built from the load / store primitives of wave_io.h (the reference's warp_load / warp_store /
// thread_load / thread_store, examples/warp_load.py:13-22, warp_store.py:13-22, for 64 lanes).
//   direction 0: out[c][64 j + l] = in[c][N l + j]   (loaded blocked as warp_load does, stored striped)
//   direction 1: out[c][N l + j] = in[c][64 j + l]   (the inverse)
// for chunk c, lane l < 64, item j < N. A last, partial chunk counts as one padded with zeros: positions at or
// beyond n are neither read nor written, every position below n is written.
#include "common.h"
#include "wave_io.h"

namespace prism {
namespace {

template <int N, int DIRECTION>
__global__ __launch_bounds__(256) void wave_regroup_kernel(const int32_t* in, int32_t* out, size_t n) {
    const int lane = threadIdx.x % kWave;
    const size_t chunk = static_cast<size_t>(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
    const size_t first = chunk * kWave * N;
    if (first >= n) return;
    const size_t valid = n - first < static_cast<size_t>(kWave) * N ? n - first : static_cast<size_t>(kWave) * N;
    int32_t items[N];
    if (DIRECTION == 0) {
        wave_load_blocked<int32_t, N>(in + first, lane, items, valid);
        wave_store_striped<int32_t, N>(out + first, lane, items, valid);
    } else {
        wave_load_striped<int32_t, N>(in + first, lane, items, valid);
        wave_store_blocked<int32_t, N>(out + first, lane, items, valid);
    }
}

template <int N>
void launch(int direction, const int32_t* in, int32_t* out, size_t n, hipStream_t s) {
    const size_t chunks = ceil_div(n, static_cast<size_t>(kWave) * N);
    const dim3 grid(static_cast<unsigned>(ceil_div(chunks, size_t{256 / kWave})));
    if (direction == 0) wave_regroup_kernel<N, 0><<<grid, dim3(256), 0, s>>>(in, out, n);
    else wave_regroup_kernel<N, 1><<<grid, dim3(256), 0, s>>>(in, out, n);
}

}  // namespace

int launch_wave_regroup(const int32_t* in, int32_t* out, size_t n, int items_per_lane, int direction, hipStream_t s) {
    if (direction != 0 && direction != 1) return fail(1, "prism_wave_regroup_i32: direction must be 0 or 1");
    if (n == 0) return 0;
    if (in == nullptr || out == nullptr) return fail(1, "prism_wave_regroup_i32: null pointer with n=%zu", n);
    if (!aligned4(in) || !aligned4(out)) return fail(1, "prism_wave_regroup_i32: pointers must be 4-byte aligned");
    const uintptr_t a = reinterpret_cast<uintptr_t>(in), b = reinterpret_cast<uintptr_t>(out), bytes = n * 4;
    if (a < b + bytes && b < a + bytes) return fail(1, "prism_wave_regroup_i32: in and out overlap");
    if (ceil_div(n, size_t{kWave}) > 0x7fffffffull) return fail(1, "prism_wave_regroup_i32: n=%zu too large", n);
    switch (items_per_lane) {
        case 1: launch<1>(direction, in, out, n, s); break;
        case 2: launch<2>(direction, in, out, n, s); break;
        case 4: launch<4>(direction, in, out, n, s); break;
        case 8: launch<8>(direction, in, out, n, s); break;
        case 16: launch<16>(direction, in, out, n, s); break;
        default: return fail(1, "prism_wave_regroup_i32: items_per_lane must be 1, 2, 4, 8 or 16, not %d", items_per_lane);
    }
    return check_launch("wave_regroup_kernel");
}

}  // namespace prism
