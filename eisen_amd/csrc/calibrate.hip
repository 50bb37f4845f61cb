// Measured ceilings for the MFMA roofline figures: what this GPU sustains on nothing but v_mfma_f32_32x32x16_bf16, and on
// the same loop with its operands re-read from LDS at the rate of a GEMM's wave tile.  The published peak (2.5 PFLOP/s
// dense bf16) assumes the boost clock; under sustained matrix load the part holds a lower clock, so a kernel's distance
// from what is reachable is better read against these numbers, measured in the same process as the kernel.
// No counterpart in the reference (its kernels use no matrix instructions); a measurement aid, not an operator.
#include "device_utils.cuh"
#include "runtime.h"

namespace {

// Each wave: four independent 32x32 accumulators (a 64x64 wave tile), 16 MFMAs per iteration = four contraction steps.
// READS: 16-byte LDS operand reads (1 KB per wave instruction) per 16 MFMAs: 0 = operands stay in registers; 16 = the
// 64x64 wave tile of the 8-wave GEMM kernels (two A and two B reads per step); 8 = the ratio of a 128x128 wave tile.
template <int READS>
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(int iters, float* sink) {
    __shared__ __attribute__((aligned(16))) bf16_t tile[16 * 512];  // 16 operand reads' worth of chunks
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 16 * 512; i += 512) tile[i] = (bf16_t)(0.002f * (float)((i * 37) % 113) - 0.11f);
    __syncthreads();
    bf16x8 a[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            a[j][e] = (bf16_t)(0.003f * (float)((lane * 7 + j * 13 + e * 5) % 61) - 0.09f);
            b[j][e] = (bf16_t)(0.004f * (float)((lane * 11 + j * 3 + e * 17) % 53) - 0.10f);
        }
    f32x16 acc[4];
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.f;
    const bf16x8* src = reinterpret_cast<const bf16x8*>(tile) + lane;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if (READS > 0) {
                constexpr int PER_STEP = READS / 4;  // 4 or 2
                const int base = ((it * 4 + s) * PER_STEP) & 15;
#pragma unroll
                for (int r = 0; r < PER_STEP; r++) {
                    const bf16x8 x = src[((base + r) & 15) * 64];
                    if (r & 1) b[(s + (r >> 1)) & 3] = x;
                    else a[(s + (r >> 1)) & 3] = x;
                }
            }
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s], b[s], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s], b[(s + 1) & 3], acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(s + 1) & 3], b[s], acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(s + 1) & 3], b[(s + 1) & 3], acc[3], 0, 0, 0);
        }
    }
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 4; k++)
#pragma unroll
        for (int v = 0; v < 16; v++) t += acc[k][v];
    if (t == 12345.678f) sink[blockIdx.x * 512 + threadIdx.x] = t;  // keeps the loop alive; never true for these operands
}

}  // namespace

extern "C" int eisen_hip_mfma_ceiling(eisen_ctx* ctx, int lds_reads_per_16_mfma, int iters, double* tflops_out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, tflops_out != nullptr, EISEN_E_ARG, "mfma_ceiling: tflops_out is null");
    EISEN_REQUIRE(ctx, lds_reads_per_16_mfma == 0 || lds_reads_per_16_mfma == 8 || lds_reads_per_16_mfma == 16, EISEN_E_ARG,
                  "mfma_ceiling: lds_reads_per_16_mfma must be 0, 8 or 16, got %d", lds_reads_per_16_mfma);
    EISEN_REQUIRE(ctx, iters > 0 && iters <= (1 << 20), EISEN_E_ARG, "mfma_ceiling: iters %d outside (0, 2^20]", iters);
    hipDeviceProp_t prop;
    EISEN_HIP_TRY(ctx, hipGetDeviceProperties(&prop, ctx->device));
    const int blocks = prop.multiProcessorCount;  // one 8-wave workgroup per CU: two waves per SIMD
    void* sink = nullptr;
    int rc = eisen_workspace(ctx, (size_t)blocks * 512 * sizeof(float), &sink);
    if (rc) return rc;
    hipEvent_t e0, e1;
    EISEN_HIP_TRY(ctx, hipEventCreate(&e0));
    EISEN_HIP_TRY(ctx, hipEventCreate(&e1));
    auto launch = [&](int n) {
        if (lds_reads_per_16_mfma == 0) mfma_ceiling_kernel<0><<<blocks, 512, 0, ctx->stream>>>(n, (float*)sink);
        else if (lds_reads_per_16_mfma == 8) mfma_ceiling_kernel<8><<<blocks, 512, 0, ctx->stream>>>(n, (float*)sink);
        else mfma_ceiling_kernel<16><<<blocks, 512, 0, ctx->stream>>>(n, (float*)sink);
    };
    launch(iters);  // warm-up: clocks and code object
    hipError_t err = hipEventRecord(e0, ctx->stream);
    launch(iters);
    if (err == hipSuccess) err = hipGetLastError();
    if (err == hipSuccess) err = hipEventRecord(e1, ctx->stream);
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    float ms = 0.f;
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess) return eisen_set_error(ctx, (int)err, "mfma_ceiling: %s", hipGetErrorString(err));
    const double flops = (double)blocks * 8.0 * (double)iters * 16.0 * 32768.0;  // waves x iterations x MFMAs x flop per MFMA
    *tflops_out = ms > 0.f ? flops / (ms * 1e-3) / 1e12 : 0.0;
    return 0;
}
