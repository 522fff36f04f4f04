// add_m: y[i] = x[i] + m over int32 (wrap-around), the streaming plumbing kernel.
// Semantics follow the kernel Prism prints for add_m_thread
// (examples/add_m_thread.py:10-19; text in README.md:133-140): one element per
// thread id, y[tid] = x[tid] + m. Here every lane moves 16 B per access and the
// element count is an argument, so any n is legal.
//
// HBM-bound: 8 algorithmic bytes per element (one 4 B read, one 4 B write).
#include "common.h"

namespace prism {
namespace {

constexpr int kAddBlock = 256;
// One 16 B packet per lane, so a workgroup is 4 KiB and a wavefront lives for one load and one store.
// Measured at 2^30 elements, 1 / 2 / 4 / 8 packets per lane give 6.50 / 5.96 / 5.84 / 4.05 TB/s: with
// one packet the workgroups sweep memory in dispatch order as one compact front (about 8 MiB in
// flight on the whole chip), which is what the write side of HBM wants: a write-only kernel of this
// shape reaches 7.0 TB/s, the same kernel writing its 4 KiB chunks in a scattered order 5.4.
// Streams larger than this use non-temporal loads and `sc1 nt` stores (write through towards memory,
// evict early: 6.68 against 6.51 TB/s for nt-only stores and 6.44 for plain ones at 2^30); smaller ones
// use ordinary accesses so that repeated passes over the same buffers are served by the 256 MiB
// memory-side cache (6.8 against 6.4 TB/s at 2^24, the size the reference quotes).
constexpr size_t kAddStreamingBytes = size_t{192} << 20;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// The two wait states keep the next instruction from overwriting the data registers while the store
// still reads them (the compiler does not see a store inside the assembly).
__device__ __forceinline__ void stream_store(u32x4* p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

// Lane t of block b handles packet (b * kAddBlock + t): a wavefront touches 1 KiB of contiguous
// memory per instruction.
template <bool STREAMING>
__global__ __launch_bounds__(kAddBlock) void add_m_vec4_kernel(const u32x4* __restrict__ x,
                                                               u32x4* __restrict__ y, uint32_t m,
                                                               size_t n_vec) {
    const size_t i = static_cast<size_t>(blockIdx.x) * kAddBlock + threadIdx.x;
    if (i >= n_vec) return;
    if (STREAMING) stream_store(&y[i], __builtin_nontemporal_load(&x[i]) + m);
    else y[i] = x[i] + m;
}

// Same as above when x and y are the same buffer (no __restrict__ promise).
template <bool STREAMING>
__global__ __launch_bounds__(kAddBlock) void add_m_vec4_inplace_kernel(u32x4* xy, uint32_t m, size_t n_vec) {
    const size_t i = static_cast<size_t>(blockIdx.x) * kAddBlock + threadIdx.x;
    if (i >= n_vec) return;
    if (STREAMING) stream_store(&xy[i], __builtin_nontemporal_load(&xy[i]) + m);
    else xy[i] = xy[i] + m;
}

// One element per thread: the tail of a vector launch, or the whole array when
// a pointer is not 16 B aligned. x may alias y.
__global__ __launch_bounds__(kAddBlock) void add_m_scalar_kernel(const uint32_t* x, uint32_t* y,
                                                                 uint32_t m, size_t first,
                                                                 size_t n) {
    const size_t i = first + static_cast<size_t>(blockIdx.x) * kAddBlock + threadIdx.x;
    if (i < n) y[i] = x[i] + m;
}

}  // namespace

int launch_add_m(const int32_t* x_, int32_t* y_, int32_t m_, size_t n, hipStream_t s) {
    if (n == 0) return 0;
    if (x_ == nullptr || y_ == nullptr) return fail(1, "prism_add_m: null pointer with n=%zu", n);
    if (!aligned4(x_) || !aligned4(y_)) return fail(1, "prism_add_m: pointers must be 4-byte aligned");
    const uint32_t* x = reinterpret_cast<const uint32_t*>(x_);
    uint32_t* y = reinterpret_cast<uint32_t*>(y_);
    const uint32_t m = static_cast<uint32_t>(m_);
    // Overlap other than exact aliasing would make the result depend on the
    // order blocks run in.
    if (x != y) {
        const uintptr_t xa = reinterpret_cast<uintptr_t>(x), ya = reinterpret_cast<uintptr_t>(y);
        const uintptr_t bytes = n * sizeof(uint32_t);
        if (xa < ya + bytes && ya < xa + bytes)
            return fail(1, "prism_add_m: x and y overlap without being equal");
    }

    size_t n_vec = 0;
    if (aligned16(x) && aligned16(y)) n_vec = n / 4;
    if (n_vec > 0) {
        const size_t blocks = ceil_div(n_vec, static_cast<size_t>(kAddBlock));
        if (blocks > 0x7fffffffull) return fail(1, "prism_add_m: n=%zu too large", n);
        const bool streaming = (x == y ? 1 : 2) * n * sizeof(uint32_t) > kAddStreamingBytes;
        if (x == y && streaming)
            add_m_vec4_inplace_kernel<true><<<dim3(static_cast<unsigned>(blocks)), dim3(kAddBlock), 0, s>>>(
                reinterpret_cast<u32x4*>(y), m, n_vec);
        else if (x == y)
            add_m_vec4_inplace_kernel<false><<<dim3(static_cast<unsigned>(blocks)), dim3(kAddBlock), 0, s>>>(
                reinterpret_cast<u32x4*>(y), m, n_vec);
        else if (streaming)
            add_m_vec4_kernel<true><<<dim3(static_cast<unsigned>(blocks)), dim3(kAddBlock), 0, s>>>(
                reinterpret_cast<const u32x4*>(x), reinterpret_cast<u32x4*>(y), m, n_vec);
        else
            add_m_vec4_kernel<false><<<dim3(static_cast<unsigned>(blocks)), dim3(kAddBlock), 0, s>>>(
                reinterpret_cast<const u32x4*>(x), reinterpret_cast<u32x4*>(y), m, n_vec);
        if (int rc = check_launch("add_m_vec4_kernel")) return rc;
    }
    const size_t first = n_vec * 4;
    if (first < n) {
        const size_t blocks = ceil_div(n - first, static_cast<size_t>(kAddBlock));
        if (blocks > 0x7fffffffull) return fail(1, "prism_add_m: n=%zu too large", n);
        add_m_scalar_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(kAddBlock), 0, s>>>(x, y, m,
                                                                                            first, n);
        if (int rc = check_launch("add_m_scalar_kernel")) return rc;
    }
    return 0;
}

}  // namespace prism
