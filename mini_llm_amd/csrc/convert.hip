// Load-time work on weights: element type conversion with an optional transpose (GPT-2 stores its
// matrices [in, out]; the matrix kernels read [out, in]). The reference converts its fp16 weight
// copy with a kernel of this kind (engine/src/matvec.cu:190-195) and transposes the head on the
// host (engine/src/gpt2_gpu.cu:30-48).
#include "common.h"

namespace {

template <typename S, typename D>
__global__ void convert_kernel(const S* __restrict__ src, D* __restrict__ dst, int rows, int cols, int transpose) {
    // 32x32 tiles through LDS so that both the read and the write run along rows
    __shared__ float tile[32][33];
    int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    for (int i = threadIdx.y; i < 32; i += blockDim.y) {
        int r = r0 + i, c = c0 + threadIdx.x;
        if (r < rows && c < cols) tile[i][threadIdx.x] = to_float(src[(size_t)r * cols + c]);
    }
    __syncthreads();
    if (!transpose) {
        for (int i = threadIdx.y; i < 32; i += blockDim.y) {
            int r = r0 + i, c = c0 + threadIdx.x;
            if (r < rows && c < cols) dst[(size_t)r * cols + c] = from_float<D>(tile[i][threadIdx.x]);
        }
    } else {
        for (int i = threadIdx.y; i < 32; i += blockDim.y) {
            int c = c0 + i, r = r0 + threadIdx.x;  // dst is [cols, rows]
            if (r < rows && c < cols) dst[(size_t)c * rows + r] = from_float<D>(tile[threadIdx.x][i]);
        }
    }
}

template <typename S, typename D>
void launch_convert(const void* src, void* dst, int rows, int cols, int transpose, hipStream_t stream) {
    dim3 grid(ceil_div(cols, 32), ceil_div(rows, 32)), block(32, 8);
    convert_kernel<S, D><<<grid, block, 0, stream>>>((const S*)src, (D*)dst, rows, cols, transpose);
}

}  // namespace

// dst = src (rows x cols, row-major) in another element type; with transpose, dst is cols x rows.
MLLM_API int mllm_convert(const void* src, void* dst, int rows, int cols, int src_dtype, int dst_dtype,
                          int transpose, hipStream_t stream) {
    MLLM_REQUIRE(rows >= 0 && cols >= 0, "convert: negative size");
    MLLM_REQUIRE(ceil_div(rows, 32) <= 65535, "convert: too many rows for one launch");
    if (rows == 0 || cols == 0) return 0;
    if (src_dtype == MLLM_F32 && dst_dtype == MLLM_F32) launch_convert<float, float>(src, dst, rows, cols, transpose, stream);
    else if (src_dtype == MLLM_F32 && dst_dtype == MLLM_BF16) launch_convert<float, bf16_t>(src, dst, rows, cols, transpose, stream);
    else if (src_dtype == MLLM_BF16 && dst_dtype == MLLM_F32) launch_convert<bf16_t, float>(src, dst, rows, cols, transpose, stream);
    else if (src_dtype == MLLM_BF16 && dst_dtype == MLLM_BF16) launch_convert<bf16_t, bf16_t>(src, dst, rows, cols, transpose, stream);
    else MLLM_REQUIRE(false, "convert: unknown element types %d -> %d", src_dtype, dst_dtype);
    return mllm_check_launch("convert");
}
