// Shared helpers of libcgnet_hip: error reporting, argument checks, small device utilities.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/cgnet_hip.h"

namespace cgnet {

// Records a printf-style message for cgnet_last_error() of the calling thread.
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();

#define CGNET_HIP(expr)                                                                       \
    do {                                                                                      \
        hipError_t e__ = (expr);                                                              \
        if (e__ != hipSuccess) {                                                              \
            ::cgnet::set_error("%s: %s (%s:%d)", #expr, hipGetErrorString(e__), __FILE__,     \
                               __LINE__);                                                     \
            return CGNET_ERR_HIP;                                                             \
        }                                                                                     \
    } while (0)

#define CGNET_REQUIRE(cond, code, ...)                                                        \
    do {                                                                                      \
        if (!(cond)) {                                                                        \
            ::cgnet::set_error(__VA_ARGS__);                                                  \
            return (code);                                                                    \
        }                                                                                     \
    } while (0)

constexpr int kMaxL = 47;          // 2L+1 <= 96 complex columns per sample in the mixing kernel; CG table (2L+1)^2 floats in LDS
constexpr int kMaxTau = 1024;      // channels of one degree

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Makes sure `func` may be launched with `bytes` of dynamic LDS on the current device.  The
// attribute is per kernel and device, not per plan: the largest size any plan of this process has
// asked for is kept and only ever raised, so plans with different needs can be launched in any order.
// Returns CGNET_OK or CGNET_ERR_HIP (message recorded).
int raise_dynamic_lds(const void* func, size_t bytes);

// ---- what the fused layer backward (CG product side) needs to know of a mixing plan -----------
struct WmmDegInfo { int K, tO, cumO, cumW, cumT; };                 // per degree: mid / output channels, offsets of gO, W, stds
bool wmm_gradff_operand_ok(const cgnet_wmm_plan* plan);             // every degree has t_O <= 16
int wmm_plan_degrees(const cgnet_wmm_plan* plan);                   // L + 1
int wmm_plan_degree(const cgnet_wmm_plan* plan, int l, WmmDegInfo* info);

// Optional per-kernel timing (cgnet_profile_*): when enabled, every launch is bracketed by a
// pair of HIP events recorded on the launch stream.
class KernelTimer {
public:
    KernelTimer(const char* name, hipStream_t stream);
    ~KernelTimer();
private:
    const char* name_;
    hipStream_t stream_;
    hipEvent_t start_ = nullptr, stop_ = nullptr;
};

#define CGNET_LAUNCH(kernel, grid, block, lds, stream, ...)                                   \
    do {                                                                                      \
        ::cgnet::KernelTimer timer__(#kernel, stream);                                        \
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                    \
    } while (0)

// ---- per-thread lookup in a short ascending table -------------------------------------------
// Index k with base(k) <= x < base(k+1) (k = n-1 if x is past the last base) for a table of n
// bases that lives in global memory.  The group first copies the table to `s_tab` (n ints of
// shared memory), so the search itself costs LDS reads instead of a chain of global loads.
// Every thread of the group must call it (one barrier inside).
constexpr int kMaxLookup = 64;
template <typename BaseOf>
__device__ __forceinline__ int lookup_in_group(int n, int x, BaseOf base_of, int* s_tab) {
    for (int k = threadIdx.x; k < n; k += blockDim.x) s_tab[k] = base_of(k);
    __syncthreads();
    int k = 0;
    while (k + 1 < n && s_tab[k + 1] <= x) ++k;
    return k;
}

// ---- matrix cores -----------------------------------------------------------------------------
// v_mfma_f32_16x16x4_f32: A[i][k] sits in lane 16*k + i, B[k][j] in lane 16*k + j, and lane n holds
// D[4*(n/16) + v][n%16] in component v of the accumulator.
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mfma4(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// ---- global memory -> LDS copies that bypass the registers (gfx950 LDS-direct loads) ----------
// The hardware places lane i of a wave 16*i (4*i for dword copies) bytes behind the LDS address
// the wave passes; the copy is tracked by vmcnt.  Nothing may read the destination before the
// issuing wave has executed dma_wait() and a barrier has been passed.
typedef __attribute__((address_space(3))) void* lds_void_ptr;

// Starts the copy of `nchunks` 16-byte pieces from `src` (8-byte aligned is enough) to the LDS
// address `dst` (16-byte aligned) by NT cooperating threads, `tid` = 0 .. NT-1 (NT a multiple of 64).
template <int NT>
__device__ __forceinline__ void dma16(const void* __restrict__ src, void* dst, int nchunks, int tid) {
    const char* s = reinterpret_cast<const char*>(src);
    char* d = reinterpret_cast<char*>(dst);
    // a 32-bit byte offset from the (wave-uniform) source: one vector add per piece instead of 64-bit address arithmetic
    const unsigned end = 16u * (unsigned)nchunks;
    for (unsigned off = 16u * (unsigned)tid; off < end; off += 16u * NT)
        __builtin_amdgcn_global_load_lds(s + off, (lds_void_ptr)(d + (off & ~1023u)), 16, 0, 0);
}

// One complex entry (8 bytes, any 8-byte alignment on both sides) copied by lanes 0 and 1 of the
// wave whose threads have tid 0 and 1.
__device__ __forceinline__ void dma8(const void* __restrict__ src, void* dst, int tid) {
    if (tid < 2)
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const char*>(src) + 4 * tid, (lds_void_ptr)dst, 4, 0, 0);
}

// Grids over (unit, part) pairs -- a unit is a task or a run of channels, a part a sample or a group
// of samples -- are launched one-dimensional and unit-major: all parts of the first unit, then all
// parts of the second ...  With the units sorted longest first every long unit is under way before
// any short one starts, and the grid drains through short work-groups.
struct UnitPart { int unit, part; };
__device__ __forceinline__ UnitPart unit_major(int nparts) {
    UnitPart r;
    r.unit = (int)(blockIdx.x / (unsigned)nparts);
    r.part = (int)(blockIdx.x - (unsigned)r.unit * (unsigned)nparts);
    return r;
}

// The other order: all units of the first part, then all units of the second ...  Work-groups that
// run at the same time then stream neighbouring channel runs of the same samples, which spreads
// their traffic evenly over the memory channels (the same run of many samples lies a whole sample
// apart).  The kernels bound by memory use this one, the one bound by arithmetic the one above.
__device__ __forceinline__ UnitPart part_major(int nparts) {
    const unsigned nunits = gridDim.x / (unsigned)nparts;
    UnitPart r;
    r.part = (int)(blockIdx.x / nunits);
    r.unit = (int)(blockIdx.x - (unsigned)r.part * nunits);
    return r;
}

// 16-byte store of data that is not read again soon: marked non-temporal, so a long output stream
// does not push the (small, re-read) operands of the kernel out of the L2 cache.
__device__ __forceinline__ void stream_store16(void* dst, float a, float b, float c, float d) {
#ifdef CGNET_NO_STREAM_HINT
    *reinterpret_cast<f32x4*>(dst) = (f32x4){a, b, c, d};
#else
    __builtin_nontemporal_store((f32x4){a, b, c, d}, reinterpret_cast<f32x4*>(dst));
#endif
}

// All copies (and loads) this wave has started have landed (vmcnt == 0).
__device__ __forceinline__ void dma_wait() { __builtin_amdgcn_s_waitcnt(0x0f70); }

// s_waitcnt vmcnt(n) for a run-time n (the instruction takes an immediate); n above the table waits for all.
__device__ __forceinline__ void wait_vmcnt(int n) {
#define CGNET_VMCNT(N) case N: __builtin_amdgcn_s_waitcnt(0x0f70 | ((N) & 15) | (((N) >> 4) << 14)); break;
    switch (n) {
        CGNET_VMCNT(1) CGNET_VMCNT(2) CGNET_VMCNT(3) CGNET_VMCNT(4) CGNET_VMCNT(5) CGNET_VMCNT(6) CGNET_VMCNT(7)
        CGNET_VMCNT(8) CGNET_VMCNT(9) CGNET_VMCNT(10) CGNET_VMCNT(11) CGNET_VMCNT(12) CGNET_VMCNT(13)
        CGNET_VMCNT(14) CGNET_VMCNT(15) CGNET_VMCNT(16) CGNET_VMCNT(17) CGNET_VMCNT(18) CGNET_VMCNT(19)
        CGNET_VMCNT(20) CGNET_VMCNT(21) CGNET_VMCNT(22) CGNET_VMCNT(23) CGNET_VMCNT(24) CGNET_VMCNT(25)
        CGNET_VMCNT(26) CGNET_VMCNT(27) CGNET_VMCNT(28)
        default: __builtin_amdgcn_s_waitcnt(0x0f70); break;
    }
#undef CGNET_VMCNT
    asm volatile("" ::: "memory");
}


}  // namespace cgnet
