// Embedding gather with the learned position rows added, row LayerNorm, and the plain residual
// add for parts that do not fuse it into a matrix product.
#include "common.h"

// out[t, :] = wte[token[t], :] + wpe[position[t], :]   (reference: engine/src/embedding.cu:7-27,
// per-row positions as in embed_batch_kernel :89-104). One block per row; a negative token marks
// a padding row, which is filled with zeros. With `sources`, the token of a row whose source is
// not negative is taken from token_slots[source] (a token the sampler left on the device, as the
// reference's queued decode reads its token: engine/src/gpt2_gpu_greedy.cu:94-107) and written into tokens.
template <typename T>
__global__ void embed_kernel(int* __restrict__ tokens, const int* __restrict__ positions,
                             const int* __restrict__ sources, const int* __restrict__ token_slots,
                             const T* __restrict__ wte, const T* __restrict__ wpe,
                             float* __restrict__ out, int width) {
    int row = blockIdx.x;
    int token = tokens[row];
    if (sources) {
        int source = sources[row];
        if (source >= 0) {
            token = token_slots[source];
            if (threadIdx.x == 0) tokens[row] = token;
        }
    }
    float* out_row = out + (size_t)row * width;
    if (token < 0) {
        for (int i = threadIdx.x; i < width; i += blockDim.x) out_row[i] = 0.0f;
        return;
    }
    const T* token_row = wte + (size_t)token * width;
    if (wpe == nullptr) {  // positions enter the model elsewhere (or nowhere)
        for (int i = threadIdx.x; i < width; i += blockDim.x) out_row[i] = to_float(token_row[i]);
        return;
    }
    const T* position_row = wpe + (size_t)positions[row] * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x)
        out_row[i] = to_float(token_row[i]) + to_float(position_row[i]);
}

MLLM_API int mllm_embed(int* tokens, const int* positions, const int* sources, const int* token_slots,
                        const void* wte, const void* wpe, float* out, int n_rows, int width, int table_dtype,
                        hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && width > 0, "embed: bad sizes rows=%d width=%d", n_rows, width);
    MLLM_REQUIRE(sources == nullptr || token_slots != nullptr, "embed: sources without token slots");
    if (n_rows == 0) return 0;
    int threads = width >= 256 ? 256 : 64;
    mllm_count_kernel(MLLM_K_EMBED);
    if (table_dtype == MLLM_F32)
        embed_kernel<float><<<n_rows, threads, 0, stream>>>(tokens, positions, sources, token_slots, (const float*)wte,
                                                            (const float*)wpe, out, width);
    else if (table_dtype == MLLM_BF16)
        embed_kernel<bf16_t><<<n_rows, threads, 0, stream>>>(tokens, positions, sources, token_slots, (const bf16_t*)wte,
                                                             (const bf16_t*)wpe, out, width);
    else
        MLLM_REQUIRE(false, "embed: unknown table dtype %d", table_dtype);
    return mllm_check_launch("embed");
}

// Row LayerNorm in 32-bit with a centred second pass (reference: engine/src/layernorm.cu:44-72):
// mean = sum/n, var = sum((x-mean)^2)/n, y = (x-mean) * 1/sqrt(var+eps) * gamma + beta.
// One wave per row, the row kept in registers when it fits (ROW_REGS*64 >= width), re-read
// otherwise. row_index, if given, names the input row of each output row.
template <typename OutT, int ROW_REGS>
__global__ void layernorm_kernel(const float* __restrict__ x, const int* __restrict__ row_index,
                                 const float* __restrict__ gamma, const float* __restrict__ beta,
                                 OutT* __restrict__ out, int n_rows, int width, float eps, int packed_out) {
    int lane = threadIdx.x % WAVE;
    int row = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (row >= n_rows) return;
    int source = row_index ? row_index[row] : row;
    const float* in_row = x + (size_t)source * width;
    const float n = (float)width;  // divided by, not multiplied with its inverse: a constant row has mean exactly itself

    if constexpr (ROW_REGS > 0) {
        // the row, the gains and the offsets are all asked for before anything is reduced, so the
        // kernel waits for memory once; a long row leaves the gains and offsets (which every wave
        // reads, so they come from the cache) for when they are used: three times its length in
        // registers would leave too few waves to keep the memory busy
        constexpr bool EARLY = ROW_REGS <= 16;
        constexpr int KEPT = EARLY ? ROW_REGS : 1;
        float values[ROW_REGS], gains[KEPT], offsets[KEPT];
#pragma unroll
        for (int r = 0; r < ROW_REGS; r++) {
            int i = min(lane + r * WAVE, width - 1);
            values[r] = in_row[i];
            if constexpr (EARLY) {
                gains[r] = gamma[i];
                offsets[r] = beta[i];
            }
        }
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < ROW_REGS; r++) {
            if (lane + r * WAVE >= width) values[r] = 0.0f;
            sum += values[r];
        }
        float mean = wave_sum(sum) / n;
        float squares = 0.0f;
#pragma unroll
        for (int r = 0; r < ROW_REGS; r++) {
            int i = lane + r * WAVE;
            float diff = i < width ? values[r] - mean : 0.0f;
            squares += diff * diff;
        }
        float inverse_stddev = 1.0f / sqrtf(wave_sum(squares) / n + eps);
#pragma unroll
        for (int r = 0; r < ROW_REGS; r++) {
            int i = lane + r * WAVE;
            if (i < width) {
                float gain = EARLY ? gains[EARLY ? r : 0] : gamma[i], offset = EARLY ? offsets[EARLY ? r : 0] : beta[i];
                out[packed_out ? packed_element<OutT>(row, i, width) : (size_t)row * width + i] = from_float<OutT>((values[r] - mean) * inverse_stddev * gain + offset);
            }
        }
    } else {
        float sum = 0.0f;
        for (int i = lane; i < width; i += WAVE) sum += in_row[i];
        float mean = wave_sum(sum) / n;
        float squares = 0.0f;
        for (int i = lane; i < width; i += WAVE) {
            float diff = in_row[i] - mean;
            squares += diff * diff;
        }
        float inverse_stddev = 1.0f / sqrtf(wave_sum(squares) / n + eps);
        for (int i = lane; i < width; i += WAVE)
            out[packed_out ? packed_element<OutT>(row, i, width) : (size_t)row * width + i] = from_float<OutT>((in_row[i] - mean) * inverse_stddev * gamma[i] + beta[i]);
    }
}

// The same for rows whose length is a multiple of four: 16-byte pieces, PIECES of them per lane in
// registers (PIECES * 256 >= width), so a row of 1,600 is seven loads a lane instead of twenty-five.
// The gains and offsets are asked for with the row while they fit beside it (PIECES <= 4).
template <typename OutT, int PIECES>
__global__ void layernorm_pieces_kernel(const float* __restrict__ x, const int* __restrict__ row_index,
                                        const float* __restrict__ gamma, const float* __restrict__ beta,
                                        OutT* __restrict__ out, int n_rows, int width, float eps, int packed_out) {
    int lane = threadIdx.x % WAVE;
    int row = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (row >= n_rows) return;
    int source = row_index ? row_index[row] : row;
    const f32x4* in_row = reinterpret_cast<const f32x4*>(x + (size_t)source * width);
    const f32x4* gain_pieces = reinterpret_cast<const f32x4*>(gamma);
    const f32x4* offset_pieces = reinterpret_cast<const f32x4*>(beta);
    const int n_pieces = width / 4;
    const float n = (float)width;
    constexpr bool EARLY = PIECES <= 4;
    constexpr int KEPT = EARLY ? PIECES : 1;
    f32x4 values[PIECES], gains[KEPT], offsets[KEPT];
#pragma unroll
    for (int r = 0; r < PIECES; r++) {
        int piece = min(lane + r * WAVE, n_pieces - 1);
        values[r] = in_row[piece];
        if constexpr (EARLY) {
            gains[r] = gain_pieces[piece];
            offsets[r] = offset_pieces[piece];
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (int r = 0; r < PIECES; r++) {
        if (lane + r * WAVE >= n_pieces) values[r] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        sum += (values[r][0] + values[r][1]) + (values[r][2] + values[r][3]);
    }
    float mean = wave_sum(sum) / n;
    float squares = 0.0f;
#pragma unroll
    for (int r = 0; r < PIECES; r++) {
        if (lane + r * WAVE < n_pieces) {
            f32x4 d = values[r] - mean;
            squares += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
        }
    }
    float inverse_stddev = 1.0f / sqrtf(wave_sum(squares) / n + eps);
#pragma unroll
    for (int r = 0; r < PIECES; r++) {
        int piece = lane + r * WAVE;
        if (piece < n_pieces) {
            f32x4 gain = EARLY ? gains[EARLY ? r : 0] : gain_pieces[piece], offset = EARLY ? offsets[EARLY ? r : 0] : offset_pieces[piece];
            f32x4 y = (values[r] - mean) * inverse_stddev * gain + offset;
            // four consecutive columns lie together in the packed layout too (inside one 16-byte piece)
            OutT* at = out + (packed_out ? packed_element<OutT>(row, 4 * piece, width) : (size_t)row * width + 4 * piece);
            if constexpr (sizeof(OutT) == 2) {
                bf16x4 rounded;
#pragma unroll
                for (int e = 0; e < 4; e++) rounded[e] = from_float<OutT>(y[e]);
                *reinterpret_cast<bf16x4*>(at) = rounded;
            } else {
                *reinterpret_cast<f32x4*>(at) = y;
            }
        }
    }
}

template <typename OutT>
static void launch_layernorm(const float* x, const int* row_index, const float* gamma,
                             const float* beta, void* out, int n_rows, int width, float eps,
                             int packed_out, hipStream_t stream) {
    const int waves = 4;
    dim3 grid(ceil_div(n_rows, waves)), block(waves * WAVE);
    OutT* o = (OutT*)out;
    mllm_count_kernel(MLLM_K_LAYERNORM);
    const bool aligned = (((size_t)x | (size_t)gamma | (size_t)beta | (size_t)out) & 15) == 0;  // 16-byte pieces need it
    if (aligned && width % 4 == 0 && width <= 16 * 4 * WAVE) {
        if (width <= 1 * 4 * WAVE)
            layernorm_pieces_kernel<OutT, 1><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
        else if (width <= 2 * 4 * WAVE)
            layernorm_pieces_kernel<OutT, 2><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
        else if (width <= 4 * 4 * WAVE)
            layernorm_pieces_kernel<OutT, 4><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
        else if (width <= 8 * 4 * WAVE)
            layernorm_pieces_kernel<OutT, 8><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
        else
            layernorm_pieces_kernel<OutT, 16><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
        return;
    }
    if (width <= 4 * WAVE)
        layernorm_kernel<OutT, 4><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
    else if (width <= 12 * WAVE)
        layernorm_kernel<OutT, 12><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
    else if (width <= 16 * WAVE)
        layernorm_kernel<OutT, 16><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
    else if (width <= 32 * WAVE)
        layernorm_kernel<OutT, 32><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
    else
        layernorm_kernel<OutT, 0><<<grid, block, 0, stream>>>(x, row_index, gamma, beta, o, n_rows, width, eps, packed_out);
}

// packed_out: out is in the packed layout of a [n_rows, width] matrix (room for whole chunks: rows up
// to a multiple of 16, columns up to a multiple of 64 bytes; what lies beyond the rows is not written).
MLLM_API int mllm_layernorm(const float* x, const int* row_index, const float* gamma,
                            const float* beta, void* out, int n_rows, int width, float eps,
                            int out_dtype, int packed_out, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && width > 0, "layernorm: bad sizes rows=%d width=%d", n_rows, width);
    MLLM_REQUIRE(eps > 0.0f, "layernorm: eps must be positive");
    if (n_rows == 0) return 0;
    if (out_dtype == MLLM_F32)
        launch_layernorm<float>(x, row_index, gamma, beta, out, n_rows, width, eps, packed_out, stream);
    else if (out_dtype == MLLM_BF16)
        launch_layernorm<bf16_t>(x, row_index, gamma, beta, out, n_rows, width, eps, packed_out, stream);
    else
        MLLM_REQUIRE(false, "layernorm: unknown output dtype %d", out_dtype);
    return mllm_check_launch("layernorm");
}

// out = a + b in 32-bit, b of either element type (the residual sum of a part that does not
// fuse it; reference: engine/src/vector_addition.cu:5-11).
template <typename T>
__global__ void add_kernel(const float* __restrict__ a, const T* __restrict__ b,
                           float* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] + to_float(b[i]);
}

MLLM_API int mllm_add(const float* a, const void* b, float* out, long long n, int b_dtype,
                      hipStream_t stream) {
    MLLM_REQUIRE(n >= 0, "add: negative size");
    if (n == 0) return 0;
    unsigned blocks = (unsigned)((n + 255) / 256);
    mllm_count_kernel(MLLM_K_ADD);
    if (b_dtype == MLLM_F32)
        add_kernel<float><<<blocks, 256, 0, stream>>>(a, (const float*)b, out, (size_t)n);
    else if (b_dtype == MLLM_BF16)
        add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(a, (const bf16_t*)b, out, (size_t)n);
    else
        MLLM_REQUIRE(false, "add: unknown dtype %d", b_dtype);
    return mllm_check_launch("add");
}
