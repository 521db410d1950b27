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

// dst: the matrix W [rows, cols] (src row-major, or stored [cols, rows] with `transpose`) in the
// packed layout of the matrix kernels (common.h, packed_offset): chunks of 16 rows x 64 bytes, a
// chunk's 64 pieces of 16 bytes in the order the lanes of a wave take them as MFMA operands. One
// wave a chunk; zeros beyond the matrix.
template <typename S, typename D>
__global__ __launch_bounds__(256) void pack_kernel(const S* __restrict__ src, D* __restrict__ dst, int rows, int cols, int transpose) {
    constexpr int VEC = 16 / sizeof(D);
    const int k_steps = ceil_div(cols, 4 * VEC);
    const size_t chunk = (size_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (chunk >= (size_t)ceil_div(rows, 16) * k_steps) return;
    const int lane = threadIdx.x % WAVE;
    const int row = (int)(chunk / k_steps) * 16 + lane % 16;
    const int col = (int)(chunk % k_steps) * 4 * VEC + (lane / 16) * VEC;
    D* at = dst + (chunk * WAVE + lane) * VEC;
#pragma unroll
    for (int i = 0; i < VEC; i++) {
        float value = 0.0f;
        if (row < rows && col + i < cols)
            value = to_float(transpose ? src[(size_t)(col + i) * rows + row] : src[(size_t)row * cols + col + i]);
        at[i] = from_float<D>(value);
    }
}

template <typename S, typename D>
void launch_pack(const void* src, void* dst, int rows, int cols, int transpose, hipStream_t stream) {
    const size_t chunks = (size_t)ceil_div(rows, 16) * ceil_div(cols, 4 * (16 / (int)sizeof(D)));
    mllm_count_kernel(MLLM_K_PACK);
    pack_kernel<S, D><<<(unsigned)((chunks + 3) / 4), 256, 0, stream>>>((const S*)src, (D*)dst, rows, cols, transpose);
}

template <typename S, typename D>
void launch_convert(const void* src, void* dst, int rows, int cols, int transpose, hipStream_t stream) {
    dim3 grid(ceil_div(cols, 32), ceil_div(rows, 32)), block(32, 8);
    mllm_count_kernel(MLLM_K_CONVERT);
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

// Elements the packed form of a rows x cols matrix takes (rows padded to 16, cols to 64 bytes).
MLLM_API long long mllm_packed_elements(int rows, int cols, int dtype) {
    const int vec = dtype == MLLM_F32 ? 4 : 8;
    return (long long)ceil_div(rows, 16) * ceil_div(cols, 4 * vec) * 64 * vec;
}

// dst = the matrix [rows, cols] in the packed layout; src is row-major [rows, cols], or with
// `transpose` the stored [cols, rows].
MLLM_API int mllm_pack_matrix(const void* src, void* dst, int rows, int cols, int src_dtype, int dst_dtype,
                              int transpose, hipStream_t stream) {
    MLLM_REQUIRE(rows > 0 && cols > 0, "pack_matrix: bad size %d x %d", rows, cols);
    if (src_dtype == MLLM_F32 && dst_dtype == MLLM_F32) launch_pack<float, float>(src, dst, rows, cols, transpose, stream);
    else if (src_dtype == MLLM_F32 && dst_dtype == MLLM_BF16) launch_pack<float, bf16_t>(src, dst, rows, cols, transpose, stream);
    else if (src_dtype == MLLM_BF16 && dst_dtype == MLLM_F32) launch_pack<bf16_t, float>(src, dst, rows, cols, transpose, stream);
    else if (src_dtype == MLLM_BF16 && dst_dtype == MLLM_BF16) launch_pack<bf16_t, bf16_t>(src, dst, rows, cols, transpose, stream);
    else MLLM_REQUIRE(false, "pack_matrix: unknown element types %d -> %d", src_dtype, dst_dtype);
    return mllm_check_launch("pack_matrix");
}
