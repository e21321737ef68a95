// Step time of AllReduce SUM fp32 on an 8-rank loopback world from native code: one host thread drives all ranks
// inside HcclGroupStart / HcclGroupEnd on one stream.  Prints, per element count, the device time per step (HIP
// events around the timed steps), the host time spent submitting a step and the wall time per step.
//
// Build: make -C examples      Run: examples/bin/allreduce_latency [ranks]
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "hccl.h"

#define HIPCHECK(x)                                                                            \
    do {                                                                                       \
        hipError_t e_ = (x);                                                                   \
        if (e_ != hipSuccess) {                                                                \
            fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_));  \
            exit(2);                                                                           \
        }                                                                                      \
    } while (0)
#define HCCLCHECK(x)                                                                           \
    do {                                                                                       \
        HcclResult r_ = (x);                                                                   \
        if (r_ != HCCL_SUCCESS) {                                                              \
            fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, HcclGetErrorString(r_)); \
            exit(3);                                                                           \
        }                                                                                      \
    } while (0)

int main(int argc, char** argv)
{
    const uint32_t n = argc > 1 ? static_cast<uint32_t>(atoi(argv[1])) : 8u;
    if (n < 1 || n > HCCL_AMD_MAX_RANKS) {
        fprintf(stderr, "ranks must be in [1, %d]\n", HCCL_AMD_MAX_RANKS);
        return 1;
    }
    std::vector<HcclComm> comms(n);
    std::vector<int32_t> devices(n, 0);
    HCCLCHECK(HcclCommInitAll(n, devices.data(), comms.data()));
    hipStream_t stream;
    HIPCHECK(hipStreamCreate(&stream));
    const uint64_t maxCount = 1ull << 22;
    std::vector<void*> in(n), out(n);
    for (uint32_t r = 0; r < n; ++r) {
        HIPCHECK(hipMalloc(&in[r], maxCount * sizeof(float)));
        HIPCHECK(hipMalloc(&out[r], maxCount * sizeof(float)));
        HIPCHECK(hipMemset(in[r], 0, maxCount * sizeof(float)));
    }
    hipEvent_t begin, end;
    HIPCHECK(hipEventCreate(&begin));
    HIPCHECK(hipEventCreate(&end));
    printf("AllReduce SUM fp32, %u ranks\n%10s %14s %14s %14s %12s\n", n, "count", "device us", "submit us", "wall us",
           "HBM GB/s");
    for (uint64_t count : {1ull, 1024ull, 65536ull, 1ull << 18, 1ull << 20, 1ull << 22}) {
        auto step = [&] {
            HCCLCHECK(HcclGroupStart());
            for (uint32_t r = 0; r < n; ++r) {
                HCCLCHECK(HcclAllReduce(in[r], out[r], count, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comms[r], stream));
            }
            HCCLCHECK(HcclGroupEnd());
        };
        for (int i = 0; i < 50; ++i) {
            step();
        }
        HIPCHECK(hipStreamSynchronize(stream));
        const int steps = 500;
        const auto t0 = std::chrono::steady_clock::now();
        HIPCHECK(hipEventRecord(begin, stream));
        for (int i = 0; i < steps; ++i) {
            step();
        }
        HIPCHECK(hipEventRecord(end, stream));
        const auto t1 = std::chrono::steady_clock::now();
        HIPCHECK(hipStreamSynchronize(stream));
        const auto t2 = std::chrono::steady_clock::now();
        float ms = 0;
        HIPCHECK(hipEventElapsedTime(&ms, begin, end));
        const double deviceUs = ms * 1e3 / steps;
        printf("%10llu %14.2f %14.2f %14.2f %12.0f\n", static_cast<unsigned long long>(count), deviceUs,
               std::chrono::duration<double, std::micro>(t1 - t0).count() / steps,
               std::chrono::duration<double, std::micro>(t2 - t0).count() / steps,
               2.0 * n * count * sizeof(float) / deviceUs / 1e3);
    }
    for (uint32_t r = 0; r < n; ++r) {
        HIPCHECK(hipFree(in[r]));
        HIPCHECK(hipFree(out[r]));
        HCCLCHECK(HcclCommDestroy(comms[r]));
    }
    return 0;
}
