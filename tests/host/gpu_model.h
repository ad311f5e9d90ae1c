// A CPU build of the library's kernel sources, for checking ADDRESSES, not values.
//
// The .hip files are compiled as plain C++ with this header in front of them (HIPC_HOST_MODEL is
// defined). A launch (hipLaunchKernelGGL) runs the kernel function once per thread of every workgroup,
// one thread after the other, as ordinary host code. Device allocations are host allocations of
// exactly the requested size (hipMalloc -> malloc, remembered in a registry), so
//   * a buffer load (__builtin_amdgcn_raw_buffer_load_*) is replaced by a checker that applies the
//     hardware's rule -- the per-lane offset is compared with the descriptor's size and a load past it
//     returns zeros; the SCALAR offset is not part of that check -- and then requires the bytes at
//     base + scalar offset + lane offset to lie inside one registered allocation;
//   * every ordinary load and store of a kernel is checked by AddressSanitizer (the model is built
//     with -fsanitize=address).
// Cross-lane operations, matrix-core products and barriers are stubs: values come out wrong, which
// does not matter as long as no address depends on them (in these kernels addresses follow from
// launch parameters, thread and workgroup indices and the decode state's position only).
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <string>

// ---- the registry of "device" allocations ---------------------------------------------------
namespace gpu_model {

struct Registry {
    std::map<uintptr_t, size_t> blocks;   // start -> bytes
    size_t loads = 0, loads_clipped = 0, launches = 0, threads = 0;
    bool failed = false;
    std::string where;   // what is being launched (printed with a failure)
};
// one registry per host thread: a thread of the driver builds its own model (its own allocations)
inline Registry &reg() {
    static thread_local Registry r;
    return r;
}
inline void *alloc(size_t bytes) {
    void *p = std::malloc(bytes ? bytes : 1);
    std::memset(p, 0, bytes);
    reg().blocks[reinterpret_cast<uintptr_t>(p)] = bytes;
    return p;
}
inline void release(void *p) {
    if (!p) return;
    reg().blocks.erase(reinterpret_cast<uintptr_t>(p));
    std::free(p);
}
// [addr, addr + n) inside one allocation?
inline bool inside(uintptr_t addr, size_t n) {
    auto it = reg().blocks.upper_bound(addr);
    if (it == reg().blocks.begin()) return false;
    --it;
    return addr >= it->first && addr + n <= it->first + it->second;
}
[[noreturn]] inline void fail(const char *what, uintptr_t base, uint32_t records, uint32_t voff, uint32_t soff, int n);

}  // namespace gpu_model

// ---- thread coordinates -----------------------------------------------------------------------
inline thread_local dim3 threadIdx, blockIdx, blockDim, gridDim;
// LDS arrays, static or dynamic (`extern __shared__`, defined by the driver), are per host thread
#undef __shared__
#define __shared__ thread_local

// ---- buffer descriptors and loads ---------------------------------------------------------------
struct gpu_model_rsrc {
    uintptr_t base;
    uint32_t records;
};
#define __amdgpu_buffer_rsrc_t gpu_model_rsrc
inline gpu_model_rsrc gpu_model_make_rsrc(void *p, int /*stride*/, int records, int /*flags*/) {
    return gpu_model_rsrc{reinterpret_cast<uintptr_t>(p), (uint32_t)records};
}
#define __builtin_amdgcn_make_buffer_rsrc gpu_model_make_rsrc

inline void gpu_model::fail(const char *what, uintptr_t base, uint32_t records, uint32_t voff, uint32_t soff, int n) {
    std::printf("FAILED (%s): %s of %d bytes at base %#zx + scalar %u + lane %u (descriptor of %u bytes) leaves every allocation; "
                "workgroup (%u, %u, %u) thread %u\n",
                reg().where.c_str(), what, n, (size_t)base, soff, voff, records, blockIdx.x, blockIdx.y, blockIdx.z, threadIdx.x);
    std::fflush(stdout);
    std::exit(1);
}

template <int BYTES>
inline void gpu_model_load(const gpu_model_rsrc &r, int voff_, int soff_, int ioff_, void *out) {
    const uint32_t voff = (uint32_t)voff_ + (uint32_t)ioff_, soff = (uint32_t)soff_;
    gpu_model::Registry &g = gpu_model::reg();
    g.loads++;
    std::memset(out, 0, BYTES);
    // raw buffer, stride 0: out of range when offset + bytes > num_records; the offset is the lane's (plus the
    // instruction's immediate) -- the scalar offset is added to the address afterwards, unchecked
    if ((uint64_t)voff + BYTES > r.records) {
        g.loads_clipped++;
        return;
    }
    const uintptr_t addr = r.base + soff + voff;
    if (!gpu_model::inside(addr, BYTES)) gpu_model::fail("buffer load", r.base, r.records, voff, soff, BYTES);
    std::memcpy(out, reinterpret_cast<const void *>(addr), BYTES);
}
typedef unsigned int gpu_model_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int gpu_model_u32x2 __attribute__((ext_vector_type(2)));
inline gpu_model_u32x4 gpu_model_load_b128(gpu_model_rsrc r, int v, int s, int aux) { gpu_model_u32x4 o; (void)aux; gpu_model_load<16>(r, v, s, 0, &o); return o; }
inline gpu_model_u32x2 gpu_model_load_b64(gpu_model_rsrc r, int v, int s, int aux) { gpu_model_u32x2 o; (void)aux; gpu_model_load<8>(r, v, s, 0, &o); return o; }
inline uint32_t gpu_model_load_b32(gpu_model_rsrc r, int v, int s, int aux) { uint32_t o; (void)aux; gpu_model_load<4>(r, v, s, 0, &o); return o; }
inline uint16_t gpu_model_load_b16(gpu_model_rsrc r, int v, int s, int aux) { uint16_t o; (void)aux; gpu_model_load<2>(r, v, s, 0, &o); return o; }
inline uint8_t gpu_model_load_b8(gpu_model_rsrc r, int v, int s, int aux) { uint8_t o; (void)aux; gpu_model_load<1>(r, v, s, 0, &o); return o; }
#define __builtin_amdgcn_raw_buffer_load_b128 gpu_model_load_b128
#define __builtin_amdgcn_raw_buffer_load_b64 gpu_model_load_b64
#define __builtin_amdgcn_raw_buffer_load_b32 gpu_model_load_b32
#define __builtin_amdgcn_raw_buffer_load_b16 gpu_model_load_b16
#define __builtin_amdgcn_raw_buffer_load_b8 gpu_model_load_b8

// ---- stubs: cross-lane operations, matrix cores, barriers, device math -------------------------
template <typename T>
inline T gpu_model_same(T v) { return v; }
template <typename T>
inline T gpu_model_readlane(T v, int) { return v; }
template <typename T>
inline T gpu_model_dpp(T, T src, int, int, int, bool) { return src; }
template <typename A, typename B, typename C>
inline C gpu_model_mfma(A, B, C c, int, int, int) { return c; }
inline void gpu_model_nothing(...) {}
template <typename T>
__attribute__((noinline)) T gpu_model_nt_load(const T *p) { return *p; }   // (never inlined: performed even where its value ends up unused)
// a load that happens even if its value is dropped afterwards (never inlined: the optimizer cannot move it under a condition)
template <typename T>
__attribute__((noinline)) T gpu_model_load_always(const T *p) { return *p; }
template <typename T, typename U>
inline void gpu_model_nt_store(U v, T *p) { *p = v; }
#define __builtin_amdgcn_readfirstlane gpu_model_same
#define __builtin_amdgcn_readlane gpu_model_readlane
#define __builtin_amdgcn_update_dpp gpu_model_dpp
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16 gpu_model_mfma
#define __builtin_amdgcn_mfma_f32_16x16x32_f16 gpu_model_mfma
#define __builtin_amdgcn_mfma_i32_32x32x32_i8 gpu_model_mfma
#define __builtin_amdgcn_mfma_f32_32x32x16_f16 gpu_model_mfma
inline float gpu_model_rcp(float v) { return 1.f / v; }
#define __builtin_amdgcn_rcpf gpu_model_rcp
inline int gpu_model_sdot4(int, int, int c, bool) { return c; }
#define __builtin_amdgcn_sdot4 gpu_model_sdot4
template <typename P>
inline float gpu_model_fdot2(P, P, float c, bool) { return c; }
#define __builtin_amdgcn_fdot2_f32_bf16 gpu_model_fdot2
inline uint32_t gpu_model_perm(uint32_t a, uint32_t, uint32_t) { return a; }
#define __builtin_amdgcn_perm gpu_model_perm
template <typename T>
inline T atomicMax(T *p, T v) { const T old = *p; if (v > old) *p = v; return old; }
#define __builtin_amdgcn_sched_barrier gpu_model_nothing
#define __builtin_amdgcn_sched_group_barrier gpu_model_nothing
#define __builtin_amdgcn_fence gpu_model_nothing
#define __builtin_amdgcn_wave_barrier gpu_model_nothing
#define __builtin_nontemporal_load gpu_model_nt_load
#define __builtin_nontemporal_store gpu_model_nt_store
#define __launch_bounds__(...)
inline void __syncthreads() {}
template <typename T>
inline T __shfl_xor(T v, int, int = 64) { return v; }
inline float __uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
inline uint32_t __float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float __expf(float v) { return std::exp(v); }
inline float rsqrtf(float v) { return 1.f / std::sqrt(v); }
inline float __fmul_rn(float a, float b) { return a * b; }
inline float __fdiv_rn(float a, float b) { return a / b; }
inline float __fadd_rn(float a, float b) { return a + b; }
using std::max;
using std::min;

// ---- the host API the sources call: allocations are registered host blocks, the stream is immediate ----
#define hipMalloc gpu_model_hipMalloc
#define hipFree gpu_model_hipFree
#define hipMemsetAsync gpu_model_hipMemsetAsync
#define hipMemcpyAsync gpu_model_hipMemcpyAsync
#define hipGetLastError gpu_model_hipGetLastError
#ifndef __align__
#define __align__(n) __attribute__((aligned(n)))
#endif
#undef HIP_SYMBOL
#define HIP_SYMBOL(x) (x)   // a "device" array of the sources is a host array here
#define hipGetSymbolAddress(pp, sym) (*(pp) = const_cast<void *>(static_cast<const void *>(sym)), hipSuccess)
#define hipFuncSetAttribute(...) hipSuccess
template <typename T>
inline hipError_t gpu_model_hipMalloc(T **p, size_t bytes) { *p = static_cast<T *>(gpu_model::alloc(bytes)); return hipSuccess; }
inline hipError_t gpu_model_hipFree(void *p) { gpu_model::release(p); return hipSuccess; }
inline hipError_t gpu_model_hipMemsetAsync(void *p, int v, size_t n, hipStream_t) { std::memset(p, v, n); return hipSuccess; }
inline hipError_t gpu_model_hipMemcpyAsync(void *d, const void *s, size_t n, hipMemcpyKind, hipStream_t) { std::memcpy(d, s, n); return hipSuccess; }
inline hipError_t gpu_model_hipGetLastError() { return hipSuccess; }

// A launch: every thread of every workgroup, one after the other. gpu_model_select (set by the driver)
// may skip a launch or restrict it to the rows [y0, y1) of its grid.
inline std::function<bool(const char *name, dim3 grid, unsigned *y0, unsigned *y1)> gpu_model_select;
template <typename F>
inline void gpu_model_launch(const char *name, dim3 grid, dim3 block, size_t lds, F &&body) {
    gpu_model::Registry &g = gpu_model::reg();
    unsigned y0 = 0, y1 = grid.y;
    if (gpu_model_select && !gpu_model_select(name, grid, &y0, &y1)) return;
    y1 = std::min(y1, grid.y);
    if (lds > 160 * 1024) {
        std::printf("FAILED (%s): %zu bytes of dynamic LDS\n", name, lds);
        std::exit(1);
    }
    g.launches++;
    const std::string outer = g.where;
    g.where = outer + " / " + name;
    gridDim = grid, blockDim = block;
    for (unsigned bz = 0; bz < grid.z; bz++)
        for (unsigned by = y0; by < y1; by++)
            for (unsigned bx = 0; bx < grid.x; bx++) {
                blockIdx = dim3(bx, by, bz);
                for (unsigned tz = 0; tz < block.z; tz++)
                    for (unsigned ty = 0; ty < block.y; ty++)
                        for (unsigned tx = 0; tx < block.x; tx++) {
                            threadIdx = dim3(tx, ty, tz);
                            g.threads++;
                            body();
                        }
            }
    g.where = outer;
}
#undef hipLaunchKernelGGL
#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
    gpu_model_launch(#kernel, dim3(grid), dim3(block), (size_t)(lds), [&] { kernel(__VA_ARGS__); })
