// Two probes of the machine itself, for the roofline figures: how fast memory can be read by a
// kernel that does nothing else, and how fast the matrix cores run with operands in registers.
// The reference measured its kernels against a pure read of the same bytes in the same way
// (engine/bench/bench_matvec_batch.cu, docs/kernels/010_matvec_batch.md:20).
#include "common.h"

namespace {

__global__ void probe_read_kernel(const f32x4* __restrict__ in, float* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    float s = 0.0f;
    for (; i < n; i += stride) {
        f32x4 v = in[i];
        s += v[0] + v[1] + v[2] + v[3];
    }
    if (s == 123.456f) out[0] = s;  // keeps the loads alive
}

template <bool HALF>
__global__ __launch_bounds__(256) void probe_mfma_kernel(float* __restrict__ out, int iterations) {
    f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    if constexpr (HALF) {
        bf16x8 a, b;
        for (int i = 0; i < 8; i++) {
            a[i] = static_cast<bf16_t>(threadIdx.x * 0.001f + i);
            b[i] = static_cast<bf16_t>(i * 0.5f);
        }
        for (int it = 0; it < iterations; it++) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
        }
    } else {
        float a = threadIdx.x * 0.001f, b = 0.5f;
        for (int it = 0; it < iterations; it++) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c3, 0, 0, 0);
        }
    }
    float s = 0.0f;
    for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace

// Reads n_bytes (a multiple of 16) once with `blocks` blocks of 256 threads; out needs one float.
MLLM_API int mllm_probe_read(const void* buffer, long long n_bytes, float* out, int blocks, hipStream_t stream) {
    MLLM_REQUIRE(n_bytes >= 0 && n_bytes % 16 == 0 && blocks > 0, "probe_read: bad size");
    mllm_count_kernel(MLLM_K_PROBE);
    probe_read_kernel<<<blocks, 256, 0, stream>>>((const f32x4*)buffer, out, (size_t)n_bytes / 16);
    return mllm_check_launch("probe_read");
}

// 4 * iterations 32x32 MFMAs per wave, 4 waves per block; out needs blocks * 256 floats. The work
// is blocks * 4 * iterations * 4 * (32768 flops for bfloat16, 4096 for float32).
MLLM_API int mllm_probe_mfma(float* out, int blocks, int iterations, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(blocks > 0 && iterations > 0, "probe_mfma: bad size");
    mllm_count_kernel(MLLM_K_PROBE);
    if (dtype == MLLM_BF16) probe_mfma_kernel<true><<<blocks, 256, 0, stream>>>(out, iterations);
    else if (dtype == MLLM_F32) probe_mfma_kernel<false><<<blocks, 256, 0, stream>>>(out, iterations);
    else MLLM_REQUIRE(false, "probe_mfma: unknown dtype %d", dtype);
    return mllm_check_launch("probe_mfma");
}
