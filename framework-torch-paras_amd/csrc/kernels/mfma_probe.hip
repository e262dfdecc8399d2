// Measurement aids.  First: the rate this GPU sustains on nothing but v_mfma_f32_32x32x16_bf16.
// (Second, further down: what a CU pulls from L2 and beyond when it does nothing but ask.)
//
// The published dense bf16 figure (2.5 PFLOP/s) is 1024 flop per cycle and SIMD at 2.4 GHz.  Under
// MFMA load on random operands the part is power limited and clocks lower; how much lower depends
// on the box and on what else the loop issues.  bench.py reports this loop's rate next to the
// attention and GEMM figures of the same process, so that their distance from the published peak
// can be split into "the kernel" and "the clock".
//
// The loop: every wavefront issues 32 MFMAs per trip on operands that stay in registers (eight A
// fragments and four B fragments of pseudo-random bf16 values in [1, 2) with random signs, two
// accumulators used alternately), with `valu` independent v_fma_f32 after each MFMA; one or two
// wavefronts per SIMD on every CU.  No memory traffic inside the loop.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "core/status.h"
#include "paras_hip.h"

namespace paras {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short i16x8 __attribute__((ext_vector_type(8)));

template <int WPS, int VALU>
__global__ __launch_bounds__(256, WPS) void mfma_probe_kernel(float* out, int trips, float c0) {
    f32x16 acc[2];
    for (int c = 0; c < 2; ++c)
        for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
    i16x8 a[8], b[4];
    unsigned h = threadIdx.x * 2654435761u + blockIdx.x;
    auto next = [&]() {
        h = h * 1664525u + 1013904223u;
        return static_cast<short>(0x3f80 + ((h >> 20) & 0x7f) + ((h >> 9) & 0x8000));
    };
    for (int j = 0; j < 8; ++j)
        for (int i = 0; i < 8; ++i) a[j][i] = next();
    for (int j = 0; j < 4; ++j)
        for (int i = 0; i < 8; ++i) b[j][i] = next();
    float f[8];
    for (int i = 0; i < 8; ++i) f[i] = 0.001f * static_cast<float>(threadIdx.x + i);
    for (int t = 0; t < trips; ++t) {
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            acc[u & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[u & 7]), __builtin_bit_cast(bf16x8, b[(u >> 3) & 3]),
                                                                 acc[u & 1], 0, 0, 0);
#pragma unroll
            for (int i = 0; i < VALU; ++i) {
                const int x = (u + i) & 7;
                f[x] = fmaf(f[x], c0, 0.25f);
                asm volatile("" : "+v"(f[x]));      // keeps the fma where it is
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float sum = acc[0][0] + acc[1][0];
    for (int i = 0; i < 8; ++i) sum += f[i];
    out[blockIdx.x * 256 + threadIdx.x] = sum;
}

// What one CU pulls through its vector cache when it does nothing else: every workgroup (one per
// CU, four wavefronts) streams a region of its own over and over -- larger than the 32 KB vector
// cache, so every request goes out to L2; whether L2 holds the regions of its XCD's 32 workgroups
// (4 MB per XCD) is the caller's choice of size.  16 bytes per lane and request, eight requests in
// flight per wavefront; kToLds: buffer loads that write LDS directly, else loads into registers.
template <bool kToLds>
__global__ __launch_bounds__(256, 1) void l2_stream_kernel(const char* base, int region_bytes, int passes, unsigned* sink) {
    __shared__ __attribute__((aligned(16))) char lds[65536];
    typedef std::uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) void* lptr_t;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const char* mine = base + static_cast<long>(blockIdx.x) * region_bytes;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(mine), 0, region_bytes, 0x00020000);
    const int requests = region_bytes / 1024;       // 1 KB per wave-wide request
    u32x4 acc = {0, 0, 0, 0};
    for (int it = 0; it < passes; ++it) {
        for (int r = wave; r < requests; r += 32) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int rr = r + 4 * u;
                if (rr < requests) {
                    if constexpr (kToLds) {
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lptr_t)(lds + ((rr * 1024) & 65535)), 16, rr * 1024 + lane * 16, 0, 0, 0);
                    } else {
                        acc += *reinterpret_cast<const u32x4*>(mine + rr * 1024 + lane * 16);
                    }
                }
            }
        }
        if constexpr (kToLds) __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
    }
    if constexpr (kToLds) {
        __syncthreads();
        acc[0] = reinterpret_cast<const unsigned*>(lds)[threadIdx.x];
    }
    if (acc[0] + acc[1] + acc[2] + acc[3] == 0x12345678u) sink[0] = 1;     // keeps the loads alive
}

}  // namespace
}  // namespace paras

extern "C" int paras_l2_stream_probe(int to_lds, int region_kib, double* bytes_per_ns_per_cu) {
    using namespace paras;
    PARAS_REQUIRE(bytes_per_ns_per_cu != nullptr, "paras_l2_stream_probe: null result pointer");
    PARAS_REQUIRE(region_kib >= 8 && region_kib <= 1024 && (region_kib & (region_kib - 1)) == 0,
                  "paras_l2_stream_probe: the region is a power of two from 8 to 1024 KiB");
    int dev = 0, cus = 0;
    PARAS_HIP_TRY(hipGetDevice(&dev));
    PARAS_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int region = region_kib * 1024;
    const int passes = static_cast<int>((64L << 20) / region);        // 64 MiB per workgroup and launch
    char* buf = nullptr;
    unsigned* sink = nullptr;
    PARAS_HIP_TRY(hipMalloc(&buf, static_cast<size_t>(cus) * region + 4));
    sink = reinterpret_cast<unsigned*>(buf + static_cast<size_t>(cus) * region);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto launch = [&]() {
        if (to_lds) hipLaunchKernelGGL((l2_stream_kernel<true>), dim3(cus), dim3(256), 0, nullptr, buf, region, passes, sink);
        else        hipLaunchKernelGGL((l2_stream_kernel<false>), dim3(cus), dim3(256), 0, nullptr, buf, region, passes, sink);
    };
    hipError_t err = hipMemset(buf, 1, static_cast<size_t>(cus) * region + 4);
    if (err == hipSuccess) err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    float ms = 0.f;
    if (err == hipSuccess) {
        launch();                                                     // untimed: brings the regions into L2
        err = hipEventRecord(e0, nullptr);
        launch();
        launch();
        if (err == hipSuccess) err = hipEventRecord(e1, nullptr);
        if (err == hipSuccess) err = hipEventSynchronize(e1);
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
        if (err == hipSuccess) err = hipGetLastError();
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(buf);
    PARAS_HIP_TRY(err);
    *bytes_per_ns_per_cu = 2.0 * static_cast<double>(passes) * region / (static_cast<double>(ms) * 1e6);
    return PARAS_OK;
}

extern "C" int paras_mfma_rate_probe(int waves_per_simd, int valu_per_mfma, double* tflops) {
    using namespace paras;
    PARAS_REQUIRE(tflops != nullptr, "paras_mfma_rate_probe: null result pointer");
    PARAS_REQUIRE(waves_per_simd == 1 || waves_per_simd == 2, "paras_mfma_rate_probe: one or two wavefronts per SIMD");
    PARAS_REQUIRE(valu_per_mfma == 0 || valu_per_mfma == 2, "paras_mfma_rate_probe: zero or two fp32 instructions per MFMA");
    int dev = 0, cus = 0;
    PARAS_HIP_TRY(hipGetDevice(&dev));
    PARAS_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int blocks = cus * waves_per_simd;
    float* out = nullptr;
    PARAS_HIP_TRY(hipMalloc(&out, static_cast<size_t>(blocks) * 256 * sizeof(float)));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto launch = [&](int trips) {
        const dim3 g(blocks), wg(256);
        if (waves_per_simd == 1 && valu_per_mfma == 0) hipLaunchKernelGGL((mfma_probe_kernel<1, 0>), g, wg, 0, nullptr, out, trips, 0.1f);
        if (waves_per_simd == 1 && valu_per_mfma == 2) hipLaunchKernelGGL((mfma_probe_kernel<1, 2>), g, wg, 0, nullptr, out, trips, 0.1f);
        if (waves_per_simd == 2 && valu_per_mfma == 0) hipLaunchKernelGGL((mfma_probe_kernel<2, 0>), g, wg, 0, nullptr, out, trips, 0.1f);
        if (waves_per_simd == 2 && valu_per_mfma == 2) hipLaunchKernelGGL((mfma_probe_kernel<2, 2>), g, wg, 0, nullptr, out, trips, 0.1f);
    };
    constexpr int kWarmTrips = 250000, kTrips = 100000;     // about 150 ms untimed, then 60 ms timed: the clock under sustained load
                                                            // (the first milliseconds of a burst run at a clock the part does not hold)
    hipError_t err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    float ms = 0.f;
    if (err == hipSuccess) {
        launch(kWarmTrips);
        err = hipEventRecord(e0, nullptr);
        launch(kTrips);
        if (err == hipSuccess) err = hipEventRecord(e1, nullptr);
        if (err == hipSuccess) err = hipEventSynchronize(e1);
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
        if (err == hipSuccess) err = hipGetLastError();
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(out);
    PARAS_HIP_TRY(err);
    const double flop = static_cast<double>(blocks) * 4.0 * kTrips * 32.0 * (2.0 * 32 * 32 * 16);
    *tflops = flop / (static_cast<double>(ms) * 1e-3) / 1e12;
    return PARAS_OK;
}
