// Register <-> memory primitives for 64-lane wavefronts: the counterparts of the reference's thread_load /
// thread_store / warp_load / warp_store device functions (examples/thread_load.py:10-18, thread_store.py,
// warp_load.py:13-22, warp_store.py:13-22), which move `items_per_thread` consecutive ints per thread of a
// 32-thread warp.
//
//   thread_load / thread_store   N consecutive items of one lane
//   wave_load_blocked / _store   lane l owns items [l N, l N + N) of the wave's 64 N items: the reference's
//                                arrangement (partition(input, offset = tid * items_per_thread)); one lane reads
//                                consecutive addresses, the 64 lanes of an instruction addresses N items apart
//   wave_load_striped / _store   item j of lane l is element 64 j + l: every instruction of the wave touches 64
//                                consecutive items (with 16-byte items: 1 KiB of contiguous memory), which is what
//                                the memory system wants; the scans load and store their tiles this way with
//                                T = a 16-byte packet
// All are bounded: items at or beyond `valid` are not touched (loads give `fill`).
#pragma once

#include <cstddef>

#include "common.h"

namespace prism {

template <typename T, int N>
__device__ __forceinline__ void thread_load(const T* in, T (&items)[N], size_t valid = N, T fill = T{}) {
#pragma unroll
    for (int i = 0; i < N; ++i) items[i] = static_cast<size_t>(i) < valid ? in[i] : fill;
}

template <typename T, int N>
__device__ __forceinline__ void thread_store(T* out, const T (&items)[N], size_t valid = N) {
#pragma unroll
    for (int i = 0; i < N; ++i)
        if (static_cast<size_t>(i) < valid) out[i] = items[i];
}

// `base` points at the wave's first item; `valid` counts the items of the wave's 64 N that exist.
template <typename T, int N>
__device__ __forceinline__ void wave_load_blocked(const T* base, int lane, T (&items)[N], size_t valid = size_t{kWave} * N,
                                                  T fill = T{}) {
    const size_t first = static_cast<size_t>(lane) * N;
    thread_load<T, N>(base + first, items, valid > first ? valid - first : 0, fill);
}

template <typename T, int N>
__device__ __forceinline__ void wave_store_blocked(T* base, int lane, const T (&items)[N], size_t valid = size_t{kWave} * N) {
    const size_t first = static_cast<size_t>(lane) * N;
    thread_store<T, N>(base + first, items, valid > first ? valid - first : 0);
}

template <typename T, int N>
__device__ __forceinline__ void wave_load_striped(const T* base, int lane, T (&items)[N], size_t valid = size_t{kWave} * N,
                                                  T fill = T{}) {
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const size_t i = static_cast<size_t>(j) * kWave + lane;
        items[j] = i < valid ? base[i] : fill;
    }
}

template <typename T, int N>
__device__ __forceinline__ void wave_store_striped(T* base, int lane, const T (&items)[N], size_t valid = size_t{kWave} * N) {
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const size_t i = static_cast<size_t>(j) * kWave + lane;
        if (i < valid) base[i] = items[j];
    }
}

// The striped load of whole 16-byte packets with the streaming hint, unbounded: the form the scans' whole
// tiles use (a wave's packets j = 0 .. N - 1 cover N KiB of contiguous memory).
template <typename P, int N>
__device__ __forceinline__ void wave_load_striped_streaming(const P* base, int lane, P (&items)[N]) {
#pragma unroll
    for (int j = 0; j < N; ++j) items[j] = __builtin_nontemporal_load(base + j * kWave + lane);
}

}  // namespace prism
