// Stand-in for <hip/hip_runtime.h> used ONLY by the CPU emulation build under tests/emu: test infrastructure,
// never part of the product (the package hccl_amd loads libhccl_amd.so and nothing else).
//
// With this header first on the include path, the library's own sources (host layer and gfx950 kernels, the
// latter with their inline assembly replaced by tests/emu/build_emu.py) compile for the host:
//   * "device memory" is host memory, streams and events are empty handles, every launch runs to completion
//     inside hipLaunchKernelGGL;
//   * a launch runs its workgroups one after the other; the lanes of a workgroup run one after the other on the
//     calling thread while they need nothing from each other, and as one OS thread per lane from the first
//     barrier or cross-lane operation on (emu_runtime.cc);
//   * the few amdgcn builtins the kernels use are functions of namespace emu, mapped by -D on the compiler's
//     command line.
// What this gives: the kernels' index arithmetic, fold interpreter, heads / tails and table lookups run under
// AddressSanitizer and are compared with the oracle on a machine without a GPU.  What it cannot show: anything
// about timing, memory ordering between wavefronts, or the code the GPU compiler generates.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>

#define __host__
#define __device__
#define __global__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
// One workgroup runs at a time, so a function-scope static is the workgroup's LDS.
#define __shared__ static

struct dim3 {
    unsigned x, y, z;
    constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

namespace emu {
struct Idx {
    unsigned x, y, z;
};
extern thread_local Idx tIdx;   // threadIdx of the lane this OS thread is running
extern thread_local Idx bIdx;   // blockIdx
extern Idx gDim, bDim;          // gridDim, blockDim of the launch in progress

// Runs body() once per lane of every workgroup of the grid.
void Launch(dim3 grid, dim3 block, const std::function<void()>& body);
void SyncThreads();
// v_mov_b32 with DPP wave_shl:1: lane i receives src of lane i + 1 of its wavefront, the last lane keeps old.
uint32_t WaveShl1(uint32_t old, uint32_t src);
inline uint32_t UpdateDpp(uint32_t old, uint32_t src, int ctrl, int rowMask, int bankMask, bool boundCtrl)
{
    if (ctrl != 0x130 || rowMask != 0xF || bankMask != 0xF || boundCtrl) {
        abort();   // only the form the copy kernel uses is emulated
    }
    return WaveShl1(old, src);
}
// Values the kernels declare uniform are uniform in every test of the emulation; the first lane's value is the lane's own.
inline uint32_t ReadFirstLane(uint32_t v) { return v; }
inline uint32_t AlignByte(uint32_t hi, uint32_t lo, uint32_t shift)
{
    const uint64_t both = (static_cast<uint64_t>(hi) << 32) | lo;
    return static_cast<uint32_t>(both >> (8u * (shift & 3u)));
}
inline void WaitCnt(int) {}
}  // namespace emu

#define threadIdx (emu::tIdx)
#define blockIdx (emu::bIdx)
#define gridDim (emu::gDim)
#define blockDim (emu::bDim)
#define __syncthreads() emu::SyncThreads()

// ---- runtime API (the subset the library calls) ---------------------------------------------------
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
constexpr hipError_t hipErrorInvalidValue = 1;
constexpr hipError_t hipErrorOutOfMemory = 2;
constexpr hipError_t hipErrorInvalidDevice = 101;
typedef struct emuStream_st* hipStream_t;
typedef struct emuEvent_st* hipEvent_t;
constexpr unsigned hipEventDisableTiming = 2;
constexpr unsigned hipHostMallocDefault = 0;
enum hipMemcpyKind { hipMemcpyHostToHost = 0, hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };

inline const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "emulated HIP error"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidDevice; }
inline hipError_t hipDeviceSynchronize() { return hipSuccess; }
// Whole 16-byte granules, as little as the GPU's allocator guarantees: the irregular copy path loads the aligned
// vectors that cover its source bytes and may read, never use, the rest of the last granule.
inline hipError_t hipMalloc(void** p, size_t n) { *p = malloc(n ? (n + 15) & ~size_t(15) : 16); return *p ? hipSuccess : hipErrorOutOfMemory; }
inline hipError_t hipFree(void* p) { free(p); return hipSuccess; }
inline hipError_t hipHostMalloc(void** p, size_t n, unsigned) { return hipMalloc(p, n); }
inline hipError_t hipHostFree(void* p) { free(p); return hipSuccess; }
inline hipError_t hipMemcpy(void* d, const void* s, size_t n, hipMemcpyKind) { memcpy(d, s, n); return hipSuccess; }
inline hipError_t hipMemcpyAsync(void* d, const void* s, size_t n, hipMemcpyKind, hipStream_t) { memcpy(d, s, n); return hipSuccess; }
inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { *e = reinterpret_cast<hipEvent_t>(malloc(1)); return hipSuccess; }
inline hipError_t hipEventDestroy(hipEvent_t e) { free(e); return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t = nullptr) { return hipSuccess; }
inline hipError_t hipEventQuery(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
enum hipStreamCaptureStatus { hipStreamCaptureStatusNone = 0, hipStreamCaptureStatusActive = 1 };
inline hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* status) { *status = hipStreamCaptureStatusNone; return hipSuccess; }
inline hipError_t hipStreamCreate(hipStream_t* s) { *s = reinterpret_cast<hipStream_t>(malloc(1)); return hipSuccess; }
inline hipError_t hipStreamDestroy(hipStream_t s) { free(s); return hipSuccess; }
inline hipError_t hipMemset(void* p, int value, size_t n) { memset(p, value, n); return hipSuccess; }
constexpr unsigned hipStreamNonBlocking = 1;
inline hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) { return hipStreamCreate(s); }
inline hipError_t hipEventCreate(hipEvent_t* e) { return hipEventCreateWithFlags(e, 0); }
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 1.0f; return hipSuccess; }   // no clock here
inline hipError_t hipGetSymbolAddress(void** p, const void* symbol) { *p = const_cast<void*>(symbol); return hipSuccess; }
#define HIP_SYMBOL(x) (&(x))

#define hipLaunchKernelGGL(kernel, grid, block, ldsBytes, stream, ...) \
    emu::Launch((grid), (block), [&] { kernel(__VA_ARGS__); })
