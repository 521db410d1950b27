// Attention over the paged cache, and the kernel that puts new keys and values into the pages.
//
// Pages of one cache layer: [num_pages, n_kv_heads, page_size, head_size], so the rows of one
// head inside a page lie together. A request's block table names its pages in order. A token at
// position p attends to the cached keys max(0, p - window + 1) .. p of its request (window 0 =
// all), which after cache_write include the tokens of its own step: decoding and prompt
// portions are the same kernel.
#include "common.h"

namespace {

// k_pages/v_pages[slot] <- the key/value columns of the step's rows. slot = page * page_size +
// offset; a negative slot is a padding row.
template <typename T>
__global__ void cache_write_kernel(const T* __restrict__ k_src, const T* __restrict__ v_src,
                                   int src_stride, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                   const int* __restrict__ slots, int n_kv_heads, int head_size,
                                   int page_size) {
    int row = blockIdx.x;
    int slot = slots[row];
    if (slot < 0) return;
    int page = slot / page_size, offset = slot % page_size;
    int width = n_kv_heads * head_size;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        int head = i / head_size, d = i % head_size;
        size_t at = (((size_t)page * n_kv_heads + head) * page_size + offset) * head_size + d;
        k_pages[at] = k_src[(size_t)row * src_stride + i];
        v_pages[at] = v_src[(size_t)row * src_stride + i];
    }
}

constexpr int MAX_HEAD = 256;

// The general kernel: one wave per (token, head), any head size up to MAX_HEAD. Keys in tiles of
// 64, a lane per key for the scores; softmax statistics in 32-bit, carried from tile to tile
// (online softmax, as the reference's prefill kernel does: engine/src/attention.cu:71-124).
template <typename T>
__global__ __launch_bounds__(256) void attention_general_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, T* __restrict__ out, int out_stride,
    const int* __restrict__ token_request, const int* __restrict__ positions,
    const int* __restrict__ block_tables, int max_blocks, int n_heads, int n_kv_heads,
    int head_size, int page_size, int window, float scale) {
    __shared__ float q_shared[4][MAX_HEAD];
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int token = blockIdx.x;
    const int head = blockIdx.y * 4 + wave;
    if (head >= n_heads) return;  // no block-wide barrier below
    const int request = token_request[token];
    T* out_row = out + (size_t)token * out_stride + head * head_size;
    if (request < 0) {
        for (int d = lane; d < head_size; d += WAVE) out_row[d] = from_float<T>(0.0f);
        return;
    }
    const int kv_head = head / (n_heads / n_kv_heads);
    const int position = positions[token];
    const int first_key = window > 0 ? max(0, position - window + 1) : 0;
    const int* table = block_tables + (size_t)request * max_blocks;

    float* my_q = q_shared[wave];
    for (int d = lane; d < head_size; d += WAVE)
        my_q[d] = to_float(q[(size_t)token * q_stride + head * head_size + d]) * scale;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();

    constexpr int REGS = MAX_HEAD / WAVE;
    float o[REGS];
#pragma unroll
    for (int r = 0; r < REGS; r++) o[r] = 0.0f;
    float running_max = -INFINITY, running_sum = 0.0f;

    for (int tile = (first_key / WAVE) * WAVE; tile <= position; tile += WAVE) {
        int key = tile + lane;
        bool valid = key >= first_key && key <= position;
        int row = 0;
        float score = -INFINITY;
        if (valid) {
            int page = table[key / page_size];
            row = (page * n_kv_heads + kv_head) * page_size + key % page_size;
            const T* k_row = k_pages + (size_t)row * head_size;
            float dot = 0.0f;
            for (int d = 0; d < head_size; d++) dot += my_q[d] * to_float(k_row[d]);
            score = dot;
        }
        float new_max = fmaxf(running_max, wave_max(score));
        float p = valid ? expf(score - new_max) : 0.0f;
        float rescale = expf(running_max - new_max);
        running_sum = running_sum * rescale + wave_sum(p);
        running_max = new_max;
#pragma unroll
        for (int r = 0; r < REGS; r++) o[r] *= rescale;
        int first = max(first_key - tile, 0), last = min(WAVE - 1, position - tile);
        for (int j = first; j <= last; j++) {
            float pj = __shfl(p, j, WAVE);
            int row_j = __shfl(row, j, WAVE);
            const T* v_row = v_pages + (size_t)row_j * head_size;
#pragma unroll
            for (int r = 0; r < REGS; r++) {
                int d = lane + r * WAVE;
                if (d < head_size) o[r] += pj * to_float(v_row[d]);
            }
        }
    }
    float inverse = 1.0f / running_sum;
#pragma unroll
    for (int r = 0; r < REGS; r++) {
        int d = lane + r * WAVE;
        if (d < head_size) out_row[d] = from_float<T>(o[r] * inverse);
    }
}

}  // namespace

MLLM_API int mllm_cache_write(const void* k_src, const void* v_src, int src_stride, void* k_pages,
                              void* v_pages, const int* slots, int n_rows, int n_kv_heads,
                              int head_size, int page_size, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_kv_heads > 0 && head_size > 0 && page_size > 0,
                 "cache_write: bad sizes");
    MLLM_REQUIRE(src_stride >= n_kv_heads * head_size, "cache_write: source rows are too short");
    if (n_rows == 0) return 0;
    int width = n_kv_heads * head_size;
    int threads = width >= 256 ? 256 : (width >= 128 ? 128 : 64);
    if (dtype == MLLM_F32)
        cache_write_kernel<float><<<n_rows, threads, 0, stream>>>(
            (const float*)k_src, (const float*)v_src, src_stride, (float*)k_pages, (float*)v_pages,
            slots, n_kv_heads, head_size, page_size);
    else if (dtype == MLLM_BF16)
        cache_write_kernel<bf16_t><<<n_rows, threads, 0, stream>>>(
            (const bf16_t*)k_src, (const bf16_t*)v_src, src_stride, (bf16_t*)k_pages,
            (bf16_t*)v_pages, slots, n_kv_heads, head_size, page_size);
    else
        MLLM_REQUIRE(false, "cache_write: unknown dtype %d", dtype);
    return mllm_check_launch("cache_write");
}

MLLM_API int mllm_attention(const void* q, int q_stride, const void* k_pages, const void* v_pages,
                            void* out, int out_stride, const int* token_request,
                            const int* positions, const int* block_tables, int max_blocks,
                            int n_tokens, int n_heads, int n_kv_heads, int head_size, int page_size,
                            int window, float scale, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && max_blocks > 0, "attention: bad sizes");
    MLLM_REQUIRE(n_heads % n_kv_heads == 0, "attention: %d heads do not divide into %d key/value heads",
                 n_heads, n_kv_heads);
    MLLM_REQUIRE(head_size > 0 && head_size <= MAX_HEAD,
                 "attention: head size %d is not in 1..%d", head_size, MAX_HEAD);
    MLLM_REQUIRE(page_size > 0 && window >= 0, "attention: bad page size or window");
    MLLM_REQUIRE(q_stride >= n_heads * head_size && out_stride >= n_heads * head_size,
                 "attention: rows are too short for the heads");
    if (n_tokens == 0) return 0;
    dim3 grid(n_tokens, ceil_div(n_heads, 4));
    if (dtype == MLLM_F32)
        attention_general_kernel<float><<<grid, 256, 0, stream>>>(
            (const float*)q, q_stride, (const float*)k_pages, (const float*)v_pages, (float*)out,
            out_stride, token_request, positions, block_tables, max_blocks, n_heads, n_kv_heads,
            head_size, page_size, window, scale);
    else if (dtype == MLLM_BF16)
        attention_general_kernel<bf16_t><<<grid, 256, 0, stream>>>(
            (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,
            (bf16_t*)out, out_stride, token_request, positions, block_tables, max_blocks, n_heads,
            n_kv_heads, head_size, page_size, window, scale);
    else
        MLLM_REQUIRE(false, "attention: unknown dtype %d", dtype);
    return mllm_check_launch("attention");
}
