// Measurement helpers for benchmarks of the attention library (gfx950), built into a library of their own
// (libltr_probe.so, include/ltr_probe.h): what this device sustains on the matrix pipe, and at which shader clock, so
// that a benchmark can print the kernels' rates beside the device's own ceiling.  Nothing here is on the attention path.
//   mfma_probe_kernel   every wave runs four independent accumulation chains of v_mfma_f32_32x32x16_bf16 on operands that
//                       stay in registers (no memory traffic inside the loop): the matrix pipe is the only limit.  With
//                       operands taken from the caller's workspace (random data) the chip runs at the clock its power
//                       limit allows; with constant operands it toggles few bits and keeps a higher clock.
//   The first wave of block 0 reports the ticks of the constant 100 MHz wall clock and of the shader clock counter over its own
//   loop (their ratio is the shader clock under this load); the rate is taken by the caller over the whole launch.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ltr_probe.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(512) void mfma_probe_kernel(const uint4 *operands, int n_operands, int iters, int random,
                                                         float *sink, long long *ticks) {
    const int tid = threadIdx.x + blockIdx.x * 512;
    union { uint4 u; bf16x8 v; } a, b;
    if (random) {
        a.u = operands[(2 * tid) % n_operands];
        b.u = operands[(2 * tid + 1) % n_operands];
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            a.v[e] = (__bf16)1.0f;
            b.v[e] = (__bf16)2.0f;
        }
    }
    // four DIFFERENT chains (distinct start values), or the compiler folds them into one
    f32x16 c0, c1, c2, c3;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        c0[r] = 0.f;
        c1[r] = 1.f;
        c2[r] = 2.f;
        c3[r] = 3.f;
    }
    const long long w0 = wall_clock64(), m0 = __builtin_amdgcn_s_memtime();
    for (int it = 0; it < iters; it++) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c3, 0, 0, 0);
    }
    const long long w1 = wall_clock64(), m1 = __builtin_amdgcn_s_memtime();
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) s += c0[r] + c1[r] + c2[r] + c3[r];
    if (s == 12345.678f) sink[tid & 1023] = s;   // keeps the chains alive; practically never taken
    if (tid == 0) {
        ticks[0] = w1 - w0;
        ticks[1] = m1 - m0;
    }
}

}  // namespace

extern "C" int ltr_device_info(ltr_device_info_t *out) {
    if (!out) return LTR_PROBE_EINVAL;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return LTR_PROBE_EDEVICE;
    out->compute_units = prop.multiProcessorCount;
    out->clock_khz = prop.clockRate;
    out->memory_clock_khz = prop.memoryClockRate;
    out->memory_bus_bits = prop.memoryBusWidth;
    out->lds_bytes_per_block = (int64_t)prop.maxSharedMemoryPerMultiProcessor;
    out->hbm_bytes = (int64_t)prop.totalGlobalMem;
    int i = 0;
    for (; i < 63 && prop.gcnArchName[i]; i++) out->arch[i] = prop.gcnArchName[i];
    out->arch[i] = 0;
    return LTR_PROBE_OK;
}

extern "C" int ltr_probe_mfma(void *workspace, int64_t workspace_bytes, int32_t iters, int32_t random_operands, void *stream) {
    if (!workspace || iters <= 0) return LTR_PROBE_EINVAL;
    if (workspace_bytes < LTR_PROBE_MIN_WORKSPACE) return LTR_PROBE_EINVAL;
    if ((uintptr_t)workspace & 15) return LTR_PROBE_EALIGN;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return LTR_PROBE_EDEVICE;
    const char *a = prop.gcnArchName;
    if (!(a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0')) return LTR_PROBE_EDEVICE;
    // layout of the workspace: [0, 16) two tick counts (results), [4096, 8192) sink, [8192, ...) operands (read only)
    long long *ticks = (long long *)workspace;
    float *sink = (float *)((char *)workspace + 4096);
    const uint4 *operands = (const uint4 *)((char *)workspace + 8192);
    int n_operands = (int)((workspace_bytes - 8192) / 16);
    int iters_ = iters, random_ = random_operands;
    void *args[] = {(void *)&operands, (void *)&n_operands, (void *)&iters_, (void *)&random_, (void *)&sink, (void *)&ticks};
    return hipLaunchKernel((const void *)mfma_probe_kernel, dim3(prop.multiProcessorCount), dim3(512), args, 0, (hipStream_t)stream) ==
                   hipSuccess
               ? LTR_PROBE_OK
               : LTR_PROBE_ELAUNCH;
}

