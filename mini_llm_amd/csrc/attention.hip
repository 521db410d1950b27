// Attention over the paged cache, and the kernel that puts new keys and values into the pages.
//
// Pages of one cache layer: [num_pages, n_kv_heads, page_size, head_size], so the rows of one
// head inside a page lie together. A request's block table names its pages in order. A token at
// position p attends to the cached keys max(0, p - window + 1) .. p of its request (window 0 =
// all), which after cache_write include the tokens of its own step: decoding and prompt
// portions are the same kernel.
#include "common.h"
#include "key_sweep.h"

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
    mllm_count_kernel(MLLM_K_CACHE_WRITE);
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
    mllm_count_kernel(MLLM_K_ATTENTION_GENERAL);
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

// ------------------------------------------------------------------------------------------------
// Decoding and short portions: a block per (token, head), a wave per share of the keys.
//
// The rows of one head inside a page lie together, so a wave reads them as one contiguous
// stream: each lane loads 16 bytes, LPR = head bytes / 16 lanes share a row, and one load
// instruction covers 64 / LPR consecutive keys. A lane therefore holds a slice of the head
// dimensions of several keys; the dot products are finished with shuffles inside the LPR lanes,
// and the value sums stay per lane until the end. The waves of a block take equal shares of
// one token's keys; their (max, sum, unnormalised output) triples are merged in LDS.
// ------------------------------------------------------------------------------------------------
namespace {

constexpr int DECODE_MAX_SPLITS = 16;

// A block per (token, head); its waves (blockDim.x / 64 of them, a power of two up to 16) split
// the token's keys evenly among themselves, and their partial results meet in LDS.
// TOGETHER: how a wave starts (see there); the host chooses.
// parts (gridDim.z) > 1: few tokens with many keys, where a block per (token, head) would leave most of the chip idle.
// The token's keys are cut into so many runs, a block each. A block leaves its unnormalised sums with their maximum and
// weight in `parts_out` ([token, head, part, HD + 2] floats) and counts itself in arrivals[token, head] (zero before the
// launch); the block that is through last puts the runs together, out = sum_p o_p e^(m_p - M) / sum_p l_p e^(m_p - M),
// and the count is zero again behind it (it wraps), so the same counters serve the next launch.
template <typename T, int HD, bool TOGETHER>
__global__ __launch_bounds__(1024) void attention_decode_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, T* __restrict__ out, int out_stride,
    const int* __restrict__ token_request, const int* __restrict__ positions,
    const int* __restrict__ block_tables, int max_blocks, int n_heads, int n_kv_heads,
    int page_shift, int window, float scale, int out_packed, float* parts_out, int* __restrict__ arrivals) {
    constexpr int VEC = KeySweep<T, HD>::VEC, LPR = KeySweep<T, HD>::LPR, RPI = KeySweep<T, HD>::RPI;
    __shared__ float partial[DECODE_MAX_SPLITS][HD + 2];
    __shared__ int through_last;

    const int lane = threadIdx.x % WAVE, split = threadIdx.x / WAVE, n_splits = blockDim.x / WAVE;
    const int head = blockIdx.x, token = blockIdx.y;
    const int request = token_request[token];
    // out_packed: the rows go out in the packed layout of a [tokens, n_heads * HD] matrix, for the
    // output product of few rows that reads them next
    auto out_at = [&](int d) -> T* {
        return out + (out_packed ? packed_element<T>(token, head * HD + d, n_heads * HD) : (size_t)token * out_stride + head * HD + d);
    };
    const int n_parts = gridDim.z, part = blockIdx.z;
    if (request < 0) {  // a padding row; the whole block leaves together (its zeros come from the block of the first run)
        if (part == 0)
            for (int d = threadIdx.x; d < HD; d += blockDim.x) *out_at(d) = from_float<T>(0.0f);
        return;
    }
    const int position = positions[token];
    constexpr int KPI = KeySweep<T, HD>::KPI;
    int first_key = window > 0 ? max(0, position - window + 1) : 0;
    int last_key = position + 1;  // exclusive
    if (n_parts > 1) {  // this block's run of the keys, in whole rounds of the sweep
        const int run = (((last_key - first_key + n_parts - 1) / n_parts + KPI - 1) / KPI) * KPI;
        first_key = min(first_key + part * run, last_key);
        last_key = min(last_key, first_key + run);
    }
    const int n_keys = last_key - first_key;
    // keys per wave: whole rounds of the sweep (a round asks for KPI keys whether it needs them or
    // not), so that a wave either has a full round to do or none
    const int chunk = (((n_keys + n_splits - 1) / n_splits + KPI - 1) / KPI) * KPI;
    const int begin = first_key + split * chunk;
    const int end = min(last_key, begin + chunk);  // exclusive
    const int sub = lane % LPR;
    const int kv_head = head / (n_heads / n_kv_heads);
    const int* table = block_tables + (size_t)request * max_blocks;

    KeySweep<T, HD> sweep;
    sweep.init();
    if (begin < end && !TOGETHER) {
        // the plain order: the query, then round by round the pages, their rows, the softmax
        float qf[VEC];
        {
            typename Chunk<T>::Raw raw = *reinterpret_cast<const typename Chunk<T>::Raw*>(q + (size_t)token * q_stride + head * HD + sub * VEC);
#pragma unroll
            for (int i = 0; i < VEC; i++) qf[i] = Chunk<T>::get(raw, i) * scale;
        }
        sweep.keys(qf, k_pages, v_pages, table, kv_head, n_kv_heads, page_shift, begin, end, lane);
    }
    if (begin < end && TOGETHER) {
        // The query and the pages of the first round are asked for together, the rows of that round
        // as soon as the pages are known, and only then is the query looked at; the pages of a
        // round are asked for before the round before it is taken into the softmax. So a wave's
        // first keys are three trips to memory away (request and position; pages; rows), not five.
        constexpr int UNROLL = KeySweep<T, HD>::UNROLL;
        const int spare_key = end - 1;
        const typename Chunk<T>::Raw raw = *reinterpret_cast<const typename Chunk<T>::Raw*>(q + (size_t)token * q_stride + head * HD + sub * VEC);
        int page[UNROLL];
        sweep.look_up(page, table, page_shift, begin, end, spare_key, lane);
        typename KeySweep<T, HD>::Fetched f;
        sweep.fetch_rows(f, page, k_pages, v_pages, kv_head, n_kv_heads, page_shift, begin, end, spare_key, lane);
        float qf[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) qf[i] = Chunk<T>::get(raw, i) * scale;
        // (in 32-bit the pages are asked for after the round: held across it they cost registers,
        // and over the many rounds of a long context that lost 5 %)
        constexpr bool PAGES_AHEAD = sizeof(T) == 2;
        for (int base = begin; base < end; base += KPI) {
            const int next = base + KPI;
            if (PAGES_AHEAD && next < end) sweep.look_up(page, table, page_shift, next, end, spare_key, lane);
            if constexpr (sizeof(T) == 2) sweep.consume(f, raw, scale, base, end, lane);  // bfloat16: the query as it is stored
            else sweep.consume(f, qf, base, end, lane);
            if (!PAGES_AHEAD && next < end) sweep.look_up(page, table, page_shift, next, end, spare_key, lane);
            if (next < end) sweep.fetch_rows(f, page, k_pages, v_pages, kv_head, n_kv_heads, page_shift, next, end, spare_key, lane);
        }
    }
    sweep.merge_groups();
    const float* o = sweep.o;
    const float running_max = sweep.running_max, running_sum = sweep.running_sum;
    if (lane < LPR) {
#pragma unroll
        for (int i = 0; i < VEC; i++) partial[split][sub * VEC + i] = o[i];
    }
    if (lane == 0) {
        partial[split][HD] = running_max;
        partial[split][HD + 1] = running_sum;
    }
    __syncthreads();
    // out = sum_s o_s e^(m_s - M) / sum_s l_s e^(m_s - M); a wave without keys has m = -inf, l = 0
    float total_max = -INFINITY;
    for (int s = 0; s < n_splits; s++) total_max = fmaxf(total_max, partial[s][HD]);
    float total = 0.0f;
    for (int s = 0; s < n_splits; s++) total += total_max == -INFINITY ? 0.0f : partial[s][HD + 1] * expf(partial[s][HD] - total_max);
    if (n_parts > 1) {  // a run without keys (a short sequence in a launch cut for long ones) leaves max -inf and weight 0
        float* runs = parts_out + ((size_t)token * n_heads + head) * n_parts * (HD + 2);
        float* mine = runs + part * (HD + 2);
        // Stored through to where every compute unit sees it; one thread then counts the block in with release and
        // acquire (a fence in every wave writes the whole L2 back sixteen times a block: 16 -> 60 us at 96 pairs).
        auto put = [&](float* at, float value) { __hip_atomic_store(at, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
        for (int d = threadIdx.x; d < HD; d += blockDim.x) {
            float value = 0.0f;
            for (int s = 0; s < n_splits; s++) value += total_max == -INFINITY ? 0.0f : partial[s][d] * expf(partial[s][HD] - total_max);
            put(mine + d, value);
        }
        if (threadIdx.x == 0) {
            put(mine + HD, total_max);
            put(mine + HD + 1, total);
        }
        __syncthreads();
        if (threadIdx.x == 0)
            through_last = __builtin_amdgcn_atomic_inc32(reinterpret_cast<unsigned*>(arrivals + token * n_heads + head), (unsigned)(n_parts - 1),
                                                          __ATOMIC_ACQ_REL, "agent") == (unsigned)(n_parts - 1);
        __syncthreads();
        if (!through_last || split != 0) return;
        // The last block's first wave: lane p takes run p's maximum and weight (up to 64 runs), the wave settles M and
        // the sum with shuffles, and each lane adds up its head dimensions over the runs, four runs' loads under way at
        // a time. The other blocks' stores are read past this compute unit's caches.
        auto far = [&](int index) { return __hip_atomic_load(runs + index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
        const float run_max = lane < n_parts ? far(lane * (HD + 2) + HD) : -INFINITY;
        const float run_sum = lane < n_parts ? far(lane * (HD + 2) + HD + 1) : 0.0f;
        const float all_max = wave_max_total(run_max);               // finite: the first run always has a key
        const float factor = run_max == -INFINITY ? 0.0f : expf(run_max - all_max);
        const float one_over = 1.0f / wave_total(run_sum * factor);
        for (int d0 = 0; d0 < HD; d0 += WAVE) {
            const int d = min(d0 + lane, HD - 1);
            float value = 0.0f;
            for (int p0 = 0; p0 < n_parts; p0 += 4) {
                float o[4];
#pragma unroll
                for (int u = 0; u < 4; u++) o[u] = far(min(p0 + u, n_parts - 1) * (HD + 2) + d);
#pragma unroll
                for (int u = 0; u < 4; u++) value += p0 + u < n_parts ? o[u] * __shfl(factor, p0 + u, WAVE) : 0.0f;
            }
            if (d0 + lane < HD) *out_at(d) = from_float<T>(value * one_over);
        }
        return;
    }
    float inverse = 1.0f / total;
    for (int d = threadIdx.x; d < HD; d += blockDim.x) {
        float value = 0.0f;
        for (int s = 0; s < n_splits; s++) value += partial[s][d] * expf(partial[s][HD] - total_max);
        *out_at(d) = from_float<T>(value * inverse);
    }
}

template <typename T>
int dispatch_decode(int head_size, const void* q, int q_stride, const void* k_pages, const void* v_pages,
                    void* out, int out_stride, const int* token_request, const int* positions,
                    const int* block_tables, int max_blocks, int n_tokens, int n_heads, int n_kv_heads,
                    int page_shift, int window, float scale, int n_splits, int out_packed, int n_parts, float* parts,
                    int* arrivals, hipStream_t stream) {
    dim3 grid(n_heads, n_tokens, n_parts), block(WAVE * n_splits);
    // Measured on MI355X: starting with query and pages together (and, in bfloat16, the pages a
    // round ahead) is 3 to 15 % faster wherever a wave has few rounds, which is where a kernel's
    // start counts; in 32-bit it takes twice the registers, and over the many rounds of long
    // contexts with few waves a token (64 x 25 heads at 900 keys, two waves each) the plain
    // order is 5 % faster.
    const int reach = max_blocks << page_shift;
    const int keys_per_round = (sizeof(T) == 2 ? 4096 : 2048) / head_size;  // KeySweep's KPI
    const int rounds = ceil_div(ceil_div(window > 0 && window < reach ? window : reach, n_splits * n_parts), keys_per_round);
    const bool together = sizeof(T) == 2 || rounds <= 12;
#define MLLM_DECODE_CASE(HD)                                                                                   \
    case HD:                                                                                                   \
        mllm_count_kernel(MLLM_K_ATTENTION_DECODE);                                                            \
        if (together)                                                                                          \
            attention_decode_kernel<T, HD, true><<<grid, block, 0, stream>>>(                                  \
                (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, (T*)out, out_stride, token_request,   \
                positions, block_tables, max_blocks, n_heads, n_kv_heads, page_shift, window, scale, out_packed, parts, arrivals);  \
        else                                                                                                   \
            attention_decode_kernel<T, HD, false><<<grid, block, 0, stream>>>(                                 \
                (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, (T*)out, out_stride, token_request,   \
                positions, block_tables, max_blocks, n_heads, n_kv_heads, page_shift, window, scale, out_packed, parts, arrivals);  \
        return 0;
    switch (head_size) {
        MLLM_DECODE_CASE(16)
        MLLM_DECODE_CASE(32)
        MLLM_DECODE_CASE(64)
        MLLM_DECODE_CASE(128)
        MLLM_DECODE_CASE(256)
    }
#undef MLLM_DECODE_CASE
    return 1;
}

}  // namespace

// 1 if the split-key decode kernel takes this head size and page size for this element type.
MLLM_API int mllm_attention_decode_supported(int head_size, int page_size, int dtype) {
    if (head_size != 16 && head_size != 32 && head_size != 64 && head_size != 128 && head_size != 256) return 0;
    if (dtype != MLLM_F32 && dtype != MLLM_BF16) return 0;
    return page_size > 0 && (page_size & (page_size - 1)) == 0 ? 1 : 0;
}

MLLM_API int mllm_attention_decode(const void* q, int q_stride, const void* k_pages, const void* v_pages,
                                   void* out, int out_stride, const int* token_request, const int* positions,
                                   const int* block_tables, int max_blocks, int n_tokens, int n_heads,
                                   int n_kv_heads, int head_size, int page_size, int window, float scale,
                                   int n_splits, int dtype, int out_packed, int n_parts, float* parts, int* arrivals,
                                   hipStream_t stream) {
    MLLM_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && max_blocks > 0, "attention_decode: bad sizes");
    MLLM_REQUIRE(n_heads % n_kv_heads == 0, "attention_decode: %d heads do not divide into %d key/value heads", n_heads, n_kv_heads);
    MLLM_REQUIRE(mllm_attention_decode_supported(head_size, page_size, dtype),
                 "attention_decode: head size %d is not one of 16, 32, 64, 128, 256, or page size %d is no power of two", head_size, page_size);
    MLLM_REQUIRE(window >= 0, "attention_decode: bad window");
    MLLM_REQUIRE(n_splits >= 1 && n_splits <= DECODE_MAX_SPLITS && (n_splits & (n_splits - 1)) == 0,
                 "attention_decode: %d splits is not a power of two in 1..%d", n_splits, DECODE_MAX_SPLITS);
    MLLM_REQUIRE(q_stride >= n_heads * head_size && out_stride >= n_heads * head_size, "attention_decode: rows are too short for the heads");
    MLLM_REQUIRE(n_tokens <= 65535, "attention_decode: too many tokens for one launch");
    // parts: the keys of a token in so many runs, a block each; `parts` then holds n_tokens * n_heads * n_parts * (head_size + 2)
    // floats and `arrivals` n_tokens * n_heads counters that are zero (and are zero again when the kernel is through)
    MLLM_REQUIRE(n_parts >= 1 && n_parts <= 64 && (n_parts == 1 || (parts != nullptr && arrivals != nullptr)), "attention_decode: %d parts (1..64, with memory and counters for them)", n_parts);
    if (n_tokens == 0) return 0;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) page_shift++;
    int refused = 1;
    if (dtype == MLLM_F32)
        refused = dispatch_decode<float>(head_size, q, q_stride, k_pages, v_pages, out, out_stride, token_request, positions,
                                         block_tables, max_blocks, n_tokens, n_heads, n_kv_heads, page_shift, window, scale, n_splits, out_packed, n_parts, parts, arrivals, stream);
    else
        refused = dispatch_decode<bf16_t>(head_size, q, q_stride, k_pages, v_pages, out, out_stride, token_request, positions,
                                          block_tables, max_blocks, n_tokens, n_heads, n_kv_heads, page_shift, window, scale, n_splits, out_packed, n_parts, parts, arrivals, stream);
    MLLM_REQUIRE(!refused, "attention_decode: no kernel for dtype %d and head size %d", dtype, head_size);
    return mllm_check_launch("attention_decode");
}

// ------------------------------------------------------------------------------------------------
// Prompt portions: a block per (request, head, tile of 32*QG queries). A wave owns 32 queries and
// every KS-th tile of 64 keys: the block stages KS key tiles at a time in LDS, the KS waves of a
// query group work on them side by side (the chain of dependent softmax updates is KS times
// shorter than the sequence), and their (max, sum, output) triples are merged at the end. Both
// products run on the matrix cores, the softmax statistics in 32-bit.
//
// The scores are computed transposed, S^T = K . Q^T (keys are the rows): a lane then holds one
// query's scores for 32 of the 64 keys, so the row maximum and sum need one exchange with the
// lane 32 further on and nothing else, and the same registers are the B operand of
// O^T = V^T . P^T with no shuffle. The order of the keys inside an MFMA's k index is free as long
// as both operands agree; V^T is read from LDS in the order the score registers have.
// bfloat16: V is transposed on its way into LDS (two keys packed per 32-bit word).
// float32: the 32-bit MFMA takes single elements, V is read as stored.
// ------------------------------------------------------------------------------------------------
namespace {

constexpr int PF_KEYS = 64;     // keys per tile
constexpr int PF_TABLE = 1024;  // block table entries a block keeps in LDS (longer tables are read from memory)

template <typename T, int HD_PAD, int QG, int KS>
struct PrefillLds {
    static constexpr bool HALF = sizeof(T) == 2;
    static constexpr int K_STRIDE = HD_PAD + (HALF ? 8 : 4);            // elements per key row
    static constexpr int V_STRIDE = HALF ? PF_KEYS + 4 : HD_PAD + 4;    // bf16: [d][key]; f32: [key][d]
    static constexpr int V_ROWS = HALF ? HD_PAD : PF_KEYS;
    static constexpr int K_ELEMS = PF_KEYS * K_STRIDE, V_ELEMS = V_ROWS * V_STRIDE;
    static constexpr int TILE_BYTES = KS * (K_ELEMS + V_ELEMS) * (int)sizeof(T);
    // merge: every wave but the first of its query group leaves 16*DT + 2 floats per lane
    static constexpr int MERGE_BYTES = QG * (KS - 1) * WAVE * (16 * (HD_PAD / 32) + 2) * 4;
    static constexpr int BYTES = TILE_BYTES > MERGE_BYTES ? TILE_BYTES : MERGE_BYTES;
    // bfloat16 V^T: the group of four keys g of row d lies at group g ^ swizzle(d). The rows a wave
    // writes at once are 8 apart, which without this would all fall on the same banks.
    static __device__ __forceinline__ int swizzle(int d) { return ((d >> 4) & 3) << 2; }
};

template <bool HALF>
__device__ __forceinline__ float softmax_exp(float x) {
    if constexpr (HALF) return __builtin_amdgcn_exp2f(x);  // scores are prescaled by log2(e)
    else return expf(x);
}

template <typename T, int HD_PAD, int QG, int KS>
__global__ __launch_bounds__(64 * QG * KS) void attention_prefill_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, T* __restrict__ out, int out_stride,
    const int* __restrict__ q_starts, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, int max_blocks, int n_heads, int n_kv_heads,
    int head_size, int page_shift, int window, float scale) {
    typedef PrefillLds<T, HD_PAD, QG, KS> L;
    constexpr bool HALF = L::HALF;
    constexpr int VEC = HALF ? 8 : 4;
    constexpr int THREADS = 64 * QG * KS;
    constexpr int QSTEPS = HALF ? HD_PAD / 16 : HD_PAD / 8;   // k-steps of the score product
    constexpr int DT = HD_PAD / 32;                           // 32-row tiles of the output's head dimension
    constexpr int SPAN = KS * PF_KEYS;                        // keys the block covers per iteration
    __shared__ __attribute__((aligned(16))) unsigned char lds_raw[L::BYTES];
    __shared__ int table_lds[PF_TABLE];
    T* const k_tiles = reinterpret_cast<T*>(lds_raw);
    T* const v_tiles = k_tiles + KS * L::K_ELEMS;

    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int lane32 = lane % 32, half = lane / 32;
    const int query_group = wave % QG, key_split = wave / QG;
    const int request = blockIdx.z, head = blockIdx.y;
    const int q_first = q_starts[request];
    const int q_len = q_starts[request + 1] - q_first;
    const int tile_q0 = (gridDim.x - 1 - blockIdx.x) * (32 * QG);  // long tiles first
    if (tile_q0 >= q_len) return;
    const int context = context_lens[request];
    if (context < 0) return;  // a padding request of a padded batch: its rows (if it has any) are nobody's, and it has no pages
    const int kv_head = head / (n_heads / n_kv_heads);
    const int* table = block_tables + (size_t)request * max_blocks;
    const int page_mask = (1 << page_shift) - 1;

    // this lane's query
    const int q_local = tile_q0 + query_group * 32 + lane32;
    const bool q_valid = q_local < q_len;
    const int q_position = context + q_local;
    const int wave_first_position = context + tile_q0 + query_group * 32;
    const int wave_last_position = context + min(tile_q0 + query_group * 32 + 31, q_len - 1);
    const bool wave_active = tile_q0 + query_group * 32 < q_len;
    const bool wave_full = tile_q0 + query_group * 32 + 31 < q_len;

    // Q^T operand, kept in registers: dims (step, half, element)
    Vec16 q_reg[QSTEPS];
    {
        const T* q_row = q + (size_t)(q_first + (q_valid ? q_local : 0)) * q_stride + head * head_size;
#pragma unroll
        for (int s = 0; s < QSTEPS; s++) {
            int d = s * (2 * VEC) + half * VEC;
            q_reg[s] = *reinterpret_cast<const Vec16*>(q_row + min(d, head_size - VEC));
            if (!(q_valid && d < head_size)) q_reg[s] = Vec16{{0u, 0u, 0u, 0u}};
        }
    }

    f32x16 acc_o[DT];
#pragma unroll
    for (int i = 0; i < DT; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc_o[i][v] = 0.0f;
    float running_max = -INFINITY, running_sum = 0.0f;

    const int block_last_position = context + min(tile_q0 + 32 * QG, q_len) - 1;
    const int block_first_key = window > 0 ? max(0, context + tile_q0 - window + 1) : 0;
    // the pages this block walks, copied to LDS once: a tile's loads then do not wait for a lookup in memory
    const int first_page = block_first_key >> page_shift, last_page = block_last_position >> page_shift;
    const bool table_in_lds = last_page - first_page < PF_TABLE;
    if (table_in_lds)
        for (int i = tid; i <= last_page - first_page; i += THREADS) table_lds[i] = table[first_page + i];
    __syncthreads();
    constexpr float LOG2E = 1.4426950408889634f;
    const float score_scale = HALF ? scale * LOG2E : scale;  // bfloat16 runs take 2^x of a prescaled score

    // K and V tiles go memory -> registers -> LDS; the loads of the next tiles are issued before the
    // products of the current ones, so their latency hides behind the matrix cores.
    constexpr int PIECES_PER_ROW = HD_PAD / VEC;
    constexpr int ROWS_PER_UNIT = HALF ? 2 : 1;  // bfloat16 takes two keys per step, to pack V^T words
    constexpr int UNITS = (SPAN / ROWS_PER_UNIT) * PIECES_PER_ROW;
    constexpr int UNITS_PER_THREAD = (UNITS + THREADS - 1) / THREADS;
    Vec16 k_regs[UNITS_PER_THREAD][ROWS_PER_UNIT], v_regs[UNITS_PER_THREAD][ROWS_PER_UNIT];
    bool kv_valid[UNITS_PER_THREAD][ROWS_PER_UNIT];
    auto fetch = [&](int k_base) {
#pragma unroll
        for (int i = 0; i < UNITS_PER_THREAD; i++) {
            int unit = min(tid + i * THREADS, UNITS - 1);
            int c = unit % PIECES_PER_ROW, row = (unit / PIECES_PER_ROW) * ROWS_PER_UNIT;
#pragma unroll
            for (int e = 0; e < ROWS_PER_UNIT; e++) {
                int key = k_base + row + e;
                // pages before a window may be gone, keys beyond the last query are not stored yet:
                // the load goes to a clamped key and column, the result is zeroed afterwards
                bool valid = key >= block_first_key && key <= block_last_position && c * VEC < head_size;
                int safe_key = min(max(key, block_first_key), block_last_position);
                int page = table_in_lds ? table_lds[(safe_key >> page_shift) - first_page] : table[safe_key >> page_shift];
                size_t at = ((((size_t)page * n_kv_heads + kv_head) << page_shift) + (safe_key & page_mask)) * head_size + min(c * VEC, head_size - VEC);
                k_regs[i][e] = *reinterpret_cast<const Vec16*>(k_pages + at);
                v_regs[i][e] = *reinterpret_cast<const Vec16*>(v_pages + at);
                kv_valid[i][e] = valid;  // applied when the tile is staged: nothing here waits for a load
            }
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < UNITS_PER_THREAD; i++) {
            int unit = tid + i * THREADS;
            if (unit >= UNITS) continue;
            int c = unit % PIECES_PER_ROW, row = (unit / PIECES_PER_ROW) * ROWS_PER_UNIT;
            int tile = row / PF_KEYS, in_tile = row % PF_KEYS;
            T* k_tile = k_tiles + tile * L::K_ELEMS;
            T* v_tile = v_tiles + tile * L::V_ELEMS;
#pragma unroll
            for (int e = 0; e < ROWS_PER_UNIT; e++) {
                uint32_t mask = kv_valid[i][e] ? 0xffffffffu : 0u;
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    k_regs[i][e].w[w] &= mask;
                    v_regs[i][e].w[w] &= mask;
                }
                *reinterpret_cast<Vec16*>(&k_tile[(in_tile + e) * L::K_STRIDE + c * VEC]) = k_regs[i][e];
            }
            if constexpr (HALF) {
                const uint16_t* v0 = reinterpret_cast<const uint16_t*>(&v_regs[i][0]);
                const uint16_t* v1 = reinterpret_cast<const uint16_t*>(&v_regs[i][ROWS_PER_UNIT - 1]);
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    uint32_t packed = (uint32_t)v0[j] | ((uint32_t)v1[j] << 16);
                    int d = c * VEC + j;
                    *reinterpret_cast<uint32_t*>(&v_tile[d * L::V_STRIDE + (((in_tile >> 2) ^ L::swizzle(d)) << 2) + (in_tile & 3)]) = packed;
                }
            } else {
                *reinterpret_cast<Vec16*>(&v_tile[in_tile * L::V_STRIDE + c * VEC]) = v_regs[i][0];
            }
        }
    };

    const T* const k_tile = k_tiles + key_split * L::K_ELEMS;
    const T* const v_tile = v_tiles + key_split * L::V_ELEMS;
    const int first_base = (block_first_key / PF_KEYS) * PF_KEYS;
    fetch(first_base);
    for (int k_base = first_base; k_base <= block_last_position; k_base += SPAN) {
        __syncthreads();  // the previous tiles have been consumed
        stage();
        __syncthreads();
        fetch(k_base + SPAN);  // unconditional: beyond the last key it reads a clamped address and is masked away
        const int k0 = k_base + key_split * PF_KEYS;
        // a wave whose queries all lie before its tile, or whose windows have all passed it, has nothing to add
        if (!wave_active || k0 > wave_last_position) continue;
        if (window > 0 && k0 + PF_KEYS - 1 < wave_first_position - window + 1) continue;

        // ---- S^T = K . Q^T : two 32-key tiles ----
        f32x16 s_acc[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
            for (int v = 0; v < 16; v++) s_acc[j][v] = 0.0f;
#pragma unroll
            for (int s = 0; s < QSTEPS; s++) {
                const T* k_at = &k_tile[(j * 32 + lane32) * L::K_STRIDE + s * (2 * VEC) + half * VEC];
                if constexpr (HALF) {
                    s_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(k_at),
                                                                       *reinterpret_cast<const bf16x8*>(&q_reg[s]), s_acc[j], 0, 0, 0);
                } else {
                    f32x4 a = *reinterpret_cast<const f32x4*>(k_at);
                    f32x4 b = *reinterpret_cast<const f32x4*>(&q_reg[s]);
#pragma unroll
                    for (int c = 0; c < 4; c++) s_acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c], b[c], s_acc[j], 0, 0, 0);
                }
            }
        }
        // ---- scale, mask (only where the tile touches the diagonal, a window or the tile's end), maximum ----
        float tile_max = -INFINITY;
        const bool interior = wave_full && window == 0 && k0 + PF_KEYS - 1 <= wave_first_position;
        if (interior) {
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    s_acc[j][v] *= score_scale;
                    tile_max = fmaxf(tile_max, s_acc[j][v]);
                }
        } else {
            const int first_allowed = window > 0 ? q_position - window + 1 : 0;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    int key = k0 + j * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                    bool allowed = q_valid && key <= q_position && key >= first_allowed;
                    float s = allowed ? s_acc[j][v] * score_scale : -INFINITY;
                    s_acc[j][v] = s;
                    tile_max = fmaxf(tile_max, s);
                }
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE));
        float new_max = fmaxf(running_max, tile_max);
        float safe_max = new_max == -INFINITY ? 0.0f : new_max;  // a query with no key yet
        float rescale = softmax_exp<HALF>(running_max - safe_max);
        running_max = new_max;
        running_sum *= rescale;
#pragma unroll
        for (int i = 0; i < DT; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc_o[i][v] *= rescale;
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float p = softmax_exp<HALF>(s_acc[j][v] - safe_max);
                s_acc[j][v] = p;
                running_sum += p;
            }
        // ---- O^T += V^T . P^T ----
        if constexpr (HALF) {
#pragma unroll
            for (int slab = 0; slab < 4; slab++) {  // 16 keys each: score registers 8*(slab%2) .. +7 of tile slab/2
                bf16x8 p;
#pragma unroll
                for (int e = 0; e < 8; e++) p[e] = static_cast<bf16_t>(s_acc[slab / 2][8 * (slab % 2) + e]);
#pragma unroll
                for (int i = 0; i < DT; i++) {
                    const int d = i * 32 + lane32, group = 4 * slab + half;
                    const T* v_row = &v_tile[d * L::V_STRIDE];
                    bf16x4 lo = *reinterpret_cast<const bf16x4*>(v_row + ((group ^ L::swizzle(d)) << 2));
                    bf16x4 hi = *reinterpret_cast<const bf16x4*>(v_row + (((group + 2) ^ L::swizzle(d)) << 2));
                    bf16x8 a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, p, acc_o[i], 0, 0, 0);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    int key = j * 32 + 8 * (v / 4) + 4 * half + (v % 4);
#pragma unroll
                    for (int i = 0; i < DT; i++)
                        acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(v_tile[key * L::V_STRIDE + i * 32 + lane32], s_acc[j][v], acc_o[i], 0, 0, 0);
                }
        }
    }

    running_sum += __shfl_xor(running_sum, 32, WAVE);

    // ---- merge the key splits of each query group: the first wave of the group gathers ----
    if constexpr (KS > 1) {
        constexpr int PER_LANE = 16 * DT + 2;
        float* merge = reinterpret_cast<float*>(lds_raw);
        __syncthreads();  // the tiles are no longer read
        if (key_split > 0) {
            float* mine = merge + (((key_split - 1) * QG + query_group) * WAVE + lane) * PER_LANE;
#pragma unroll
            for (int i = 0; i < DT; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) mine[i * 16 + v] = acc_o[i][v];
            mine[16 * DT] = running_max;
            mine[16 * DT + 1] = running_sum;
        }
        __syncthreads();
        if (key_split > 0) return;
        float total_max = running_max;
#pragma unroll
        for (int s = 1; s < KS; s++)
            total_max = fmaxf(total_max, merge[(((s - 1) * QG + query_group) * WAVE + lane) * PER_LANE + 16 * DT]);
        float safe_max = total_max == -INFINITY ? 0.0f : total_max;
        float weight = softmax_exp<HALF>(running_max - safe_max);
        running_sum *= weight;
#pragma unroll
        for (int i = 0; i < DT; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc_o[i][v] *= weight;
#pragma unroll
        for (int s = 1; s < KS; s++) {
            const float* other = merge + (((s - 1) * QG + query_group) * WAVE + lane) * PER_LANE;
            float w = softmax_exp<HALF>(other[16 * DT] - safe_max);
            running_sum += other[16 * DT + 1] * w;
#pragma unroll
            for (int i = 0; i < DT; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc_o[i][v] += other[i * 16 + v] * w;
        }
    }

    if (!q_valid) return;
    float inverse = 1.0f / running_sum;  // every query sees at least its own key
    T* out_row = out + (size_t)(q_first + q_local) * out_stride + head * head_size;
#pragma unroll
    for (int i = 0; i < DT; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            int d = i * 32 + 8 * (v / 4) + 4 * half + (v % 4);
            if (d < head_size) out_row[d] = from_float<T>(acc_o[i][v] * inverse);
        }
}

template <typename T, int HD_PAD>
void launch_prefill(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out, int out_stride,
                    const int* q_starts, const int* context_lens, const int* block_tables, int max_blocks,
                    int n_requests, int max_q_len, int n_heads, int n_kv_heads, int head_size, int page_shift,
                    int window, float scale, hipStream_t stream) {
    // Queries per block (32*QG) set how often keys and values are read again from the cache;
    // waves along the keys (KS) set the length of the chain of dependent softmax updates.
    constexpr bool ROOMY = PrefillLds<T, HD_PAD, 1, 4>::TILE_BYTES <= 80 * 1024;
    // Measured on MI355X (two 1,024-token prompts, 12 heads of 64): 128 queries per block run 2.5
    // times faster than 32, because every block reads its keys and values again from the cache.
    const int shape = max_q_len > 64 ? 3 : (max_q_len > 32 ? 5 : (ROOMY ? 1 : 4));
#define MLLM_PREFILL_LAUNCH(QG, KS)                                                                                   \
    {                                                                                                                  \
        dim3 grid(ceil_div(max_q_len, 32 * QG), n_heads, n_requests);                                                  \
        mllm_count_kernel(MLLM_K_ATTENTION_PREFILL);                                                                   \
        attention_prefill_kernel<T, HD_PAD, QG, KS><<<grid, 64 * QG * KS, 0, stream>>>(                                \
            (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, (T*)out, out_stride, q_starts, context_lens, \
            block_tables, max_blocks, n_heads, n_kv_heads, head_size, page_shift, window, scale);                      \
    }
    if constexpr (ROOMY) {
        if (shape == 1) MLLM_PREFILL_LAUNCH(1, 4)
        else if (shape == 2) MLLM_PREFILL_LAUNCH(2, 4)
        else if (shape == 3) MLLM_PREFILL_LAUNCH(4, 2)
        else if (shape == 4) MLLM_PREFILL_LAUNCH(1, 2)
        else MLLM_PREFILL_LAUNCH(2, 2)
    } else {
        if (shape == 3) MLLM_PREFILL_LAUNCH(4, 2)
        else if (shape == 5) MLLM_PREFILL_LAUNCH(2, 2)
        else MLLM_PREFILL_LAUNCH(1, 2)
    }
#undef MLLM_PREFILL_LAUNCH
}

}  // namespace

#include "attention_stream.h"

// 1 if the matrix-core prefill kernel takes this head size and page size.
MLLM_API int mllm_attention_prefill_supported(int head_size, int page_size) {
    bool page_ok = page_size > 0 && (page_size & (page_size - 1)) == 0;
    return head_size >= 16 && head_size <= 128 && head_size % 16 == 0 && page_ok ? 1 : 0;
}

MLLM_API int mllm_attention_prefill(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out,
                                    int out_stride, const int* q_starts, const int* context_lens,
                                    const int* block_tables, int max_blocks, int n_requests, int max_q_len,
                                    int max_len, int n_heads, int n_kv_heads, int head_size, int page_size, int window,
                                    float scale, int dtype, hipStream_t stream) {
    // max_len: the longest sequence after this step, or a bound on it (0 or less: what the block tables can hold); it only
    // decides how many waves share a block's keys
    MLLM_REQUIRE(n_requests >= 0 && max_q_len >= 0 && n_heads > 0 && n_kv_heads > 0 && max_blocks > 0, "attention_prefill: bad sizes");
    MLLM_REQUIRE(n_heads % n_kv_heads == 0, "attention_prefill: %d heads do not divide into %d key/value heads", n_heads, n_kv_heads);
    MLLM_REQUIRE(mllm_attention_prefill_supported(head_size, page_size),
                 "attention_prefill: head size %d is not a multiple of 16 in 16..128, or page size %d is no power of two", head_size, page_size);
    MLLM_REQUIRE(window >= 0, "attention_prefill: bad window");
    MLLM_REQUIRE(q_stride >= n_heads * head_size && out_stride >= n_heads * head_size, "attention_prefill: rows are too short for the heads");
    MLLM_REQUIRE(n_requests <= 65535 && n_heads <= 65535, "attention_prefill: too many requests or heads for one launch");
    if (n_requests == 0 || max_q_len == 0) return 0;
    int padded = ceil_div(head_size, 32) * 32;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) page_shift++;
#define MLLM_PREFILL_CASE(T, PAD)                                                                                      \
    launch_prefill<T, PAD>(q, q_stride, k_pages, v_pages, out, out_stride, q_starts, context_lens, block_tables,      \
                           max_blocks, n_requests, max_q_len, n_heads, n_kv_heads, head_size, page_shift, window, scale, stream)
    const long table_reach = (long)max_blocks * page_size;
    const int reach = (int)(max_len > 0 && max_len < table_reach ? max_len : (table_reach < (1 << 30) ? table_reach : (1 << 30)));
#define MLLM_STREAM_CASE(T, HD)                                                                                            \
    prefill_stream::launch<T, HD>(q, q_stride, k_pages, v_pages, out, out_stride, q_starts, context_lens, block_tables,    \
                                  max_blocks, n_requests, max_q_len, reach, n_heads, n_kv_heads, page_shift, window, scale, stream)
    if (dtype == MLLM_BF16 && prefill_stream::takes<bf16_t>(head_size, page_size, max_q_len, scale, q_stride, out_stride, q, out)) {
        // long portions, rows of 64 / 128 / 256 bytes, pages of 32 keys or more: keys and values stream from the pages straight into LDS
        if (head_size == 32) MLLM_STREAM_CASE(bf16_t, 32);
        else if (head_size == 64) MLLM_STREAM_CASE(bf16_t, 64);
        else MLLM_STREAM_CASE(bf16_t, 128);
        return mllm_check_launch("attention_prefill");
    }
    if (dtype == MLLM_F32 && prefill_stream::takes<float>(head_size, page_size, max_q_len, scale, q_stride, out_stride, q, out)) {
        if (head_size == 32) MLLM_STREAM_CASE(float, 32);
        else MLLM_STREAM_CASE(float, 64);
        return mllm_check_launch("attention_prefill");
    }
#undef MLLM_STREAM_CASE
    if (dtype == MLLM_F32) {
        if (padded == 32) MLLM_PREFILL_CASE(float, 32);
        else if (padded == 64) MLLM_PREFILL_CASE(float, 64);
        else if (padded == 96) MLLM_PREFILL_CASE(float, 96);
        else MLLM_PREFILL_CASE(float, 128);
    } else if (dtype == MLLM_BF16) {
        if (padded == 32) MLLM_PREFILL_CASE(bf16_t, 32);
        else if (padded == 64) MLLM_PREFILL_CASE(bf16_t, 64);
        else if (padded == 96) MLLM_PREFILL_CASE(bf16_t, 96);
        else MLLM_PREFILL_CASE(bf16_t, 128);
    } else {
        MLLM_REQUIRE(false, "attention_prefill: unknown dtype %d", dtype);
    }
#undef MLLM_PREFILL_CASE
    return mllm_check_launch("attention_prefill");
}
