// Shared host-side helpers of libplexus_hip: error reporting and argument checks.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "plexus_hip.h"

namespace plx {

void set_last_error(const char *fmt, ...);

inline int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
inline int fail(int status, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    set_last_error("%s", buf);
    return status;
}

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

constexpr int kWave = 64;

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// fp32 MFMA products that run only if one of n_run_if device words is non-zero (gemm.hip); same arguments as
// plx_gemm_nn_f32 / plx_gemm_nt_f32 otherwise
int gemm_nn_f32_if(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                   int64_t ldc, unsigned flags, const unsigned *run_if, int n_run_if, void *stream);
int gemm_nt_f32_if(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                   int64_t ldc, const float *mask, int64_t ldmask, const unsigned *run_if, int n_run_if, void *stream, float alpha = 1.f);

// GRAD_W on the fp32 MFMA (gemm.hip) for the split product of gemm_split_tn.hip: its workspace and split count, the
// guarded form (runs, and writes C, only if *run_if is non-zero; the result times alpha), and the fixed-order sum of
// partial tiles that both products end with
size_t gemm_tn_f32_workspace_bytes(int64_t M, int64_t N, int64_t K);
int64_t gemm_tn_f32_splits(int64_t M, int64_t N, int64_t K);
int gemm_tn_f32_if(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int64_t ldc,
                   const float *mask, int64_t ldmask, void *workspace, size_t workspace_bytes, const unsigned *run_if, float alpha, void *stream);
int gemm_tn_reduce_tiles(const float *ws, int64_t ws_ld, int64_t ws_slab, int splits, int64_t K, int64_t N, float *C, int64_t ldc, float alpha,
                         void *stream);
// dinv[r] = 1 / sqrt(sum of val[rowptr[r] .. rowptr[r + 1])), 0 where the sum is not positive (elementwise.hip)
int row_sums_rsqrt(int64_t M, const int32_t *rowptr, const float *val, float *dinv, void *stream);

#if defined(__HIPCC__)
// Orders the LDS accesses of one wavefront for the compiler: lanes that exchange data through a tile private to their
// wavefront (no workgroup barrier) put this between the stores of one phase and the loads of the next.  The hardware
// executes a wavefront's LDS instructions in order; this keeps the compiler from reordering them.  No instruction
// besides what the fence needs at wavefront scope.
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
#endif

}  // namespace plx

#define PLX_HIP_CHECK(expr)                                                                            \
    do {                                                                                               \
        hipError_t e__ = (expr);                                                                       \
        if (e__ != hipSuccess)                                                                         \
            return plx::fail(PLX_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e__), __FILE__, \
                             __LINE__);                                                                \
    } while (0)

#define PLX_LAUNCH_CHECK(name)                                                                        \
    do {                                                                                               \
        hipError_t e__ = hipGetLastError();                                                            \
        if (e__ != hipSuccess)                                                                         \
            return plx::fail(PLX_ERR_HIP, "launch of %s failed: %s", name, hipGetErrorString(e__));   \
    } while (0)

#define PLX_REQUIRE(cond, ...)                                  \
    do {                                                        \
        if (!(cond)) return plx::fail(PLX_ERR_INVALID, __VA_ARGS__); \
    } while (0)

namespace plx {

// A kernel that takes more than 64 KB of dynamic LDS has to be allowed to, per kernel and device.  The setting is a
// runtime call, so a launcher makes it once per (kernel instantiation, device) and remembers it in `done`, one bit per
// device ordinal (ordinals past 63 make the call every time); later launches only ask which device is current.
inline int allow_dynamic_lds(const void *kernel, size_t bytes, std::atomic<uint64_t> &done)
{
    int dev = 0;
    PLX_HIP_CHECK(hipGetDevice(&dev));
    const uint64_t bit = (dev >= 0 && dev < 64) ? (1ull << dev) : 0ull;
    if (bit != 0 && (done.load(std::memory_order_acquire) & bit) != 0) return PLX_OK;
    PLX_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    if (bit != 0) done.fetch_or(bit, std::memory_order_release);
    return PLX_OK;
}

}  // namespace plx
