// Token choice on the device: argmax with numpy's rules, and temperature / top-p sampling.
#include "common.h"

namespace {

constexpr int SAMPLE_THREADS = 1024;

__device__ __forceinline__ void block_best(float& value, int& index, float* shared_values,
                                           int* shared_indices) {
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
        float other = __shfl_xor(value, offset, WAVE);
        int other_index = __shfl_xor(index, offset, WAVE);
        if (beats(other, other_index, value, index)) {
            value = other;
            index = other_index;
        }
    }
    int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    __syncthreads();
    if (lane == 0) {
        shared_values[wave] = value;
        shared_indices[wave] = index;
    }
    __syncthreads();
    value = shared_values[0];
    index = shared_indices[0];
    for (int w = 1; w < n_waves; w++)
        if (beats(shared_values[w], shared_indices[w], value, index)) {
            value = shared_values[w];
            index = shared_indices[w];
        }
}

__device__ __forceinline__ float block_sum(float value, float* shared_values) {
    value = wave_sum(value);
    int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    __syncthreads();
    if (lane == 0) shared_values[wave] = value;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < n_waves; w++) total += shared_values[w];  // same order in every thread
    return total;
}

// Counter-based generator: the uniform number of (seed, step, index) is a pure function of the
// three, so a draw does not depend on the batch, the launch shape or the order of evaluation.
__device__ __forceinline__ float uniform_open(uint64_t seed, uint32_t step, uint32_t index) {
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * ((uint64_t)step + 1) + 0xD1B54A32D192ED03ull * ((uint64_t)index + 1);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    // 23 bits: (v + 0.5) / 2^23 with v < 2^23 is exact in 32-bit (24 significant bits hold 2v + 1) and
    // lies in [2^-24, 1 - 2^-24]: never 0 or 1, so -log(-log(u)) is finite
    return ((float)(z >> 41) + 0.5f) * (1.0f / 8388608.0f);
}

// One block per row. With token_slots the chosen token is also left in token_slots[slot_of_row[row]]
// (the request's last-token slot), from where the next step can take it without the host having
// seen it. temperature 0: argmax. Otherwise a draw from softmax(logits / temperature)
// cut to the nucleus top_p (token i stays if the mass of all strictly more likely tokens is
// below top_p), taken as argmax(logit/temperature + Gumbel noise): it reuses the argmax
// reduction and does not depend on a summation order.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int vocab, const float* __restrict__ temperatures,
    const float* __restrict__ top_ps, const uint64_t* __restrict__ seeds,
    const int* __restrict__ steps, int* __restrict__ out_tokens, int* __restrict__ token_slots,
    const int* __restrict__ slot_of_row) {
    __shared__ float shared_values[SAMPLE_THREADS / WAVE];
    __shared__ int shared_indices[SAMPLE_THREADS / WAVE];
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* x = logits + (size_t)row * vocab;
    const float temperature = temperatures ? temperatures[row] : 0.0f;
    const int token_slot = token_slots ? slot_of_row[row] : -1;  // asked for now: at the end it would cost a trip to memory of its own

    float best = -INFINITY;
    int best_index = 0x7fffffff;
    // The row is read in 16-byte pieces, eight of them in flight per thread before any is compared:
    // a few trips to memory for the whole row. A row starts wherever rows * vocab puts it, so the
    // elements before the first 16-byte boundary and after the last one are read one by one.
    const int head = min(vocab, (int)((16 - ((size_t)x & 15)) & 15) / 4);  // elements before the boundary
    const int n_pieces = (vocab - head) / 4;
    const f32x4* pieces = reinterpret_cast<const f32x4*>(x + head);
    if (tid < head && beats(x[tid], tid, best, best_index)) {
        best = x[tid];
        best_index = tid;
    }
    for (int i = head + 4 * n_pieces + tid; i < vocab; i += SAMPLE_THREADS)
        if (beats(x[i], i, best, best_index)) {
            best = x[i];
            best_index = i;
        }
    constexpr int BATCH = 8;
    for (int p0 = tid; p0 < n_pieces; p0 += SAMPLE_THREADS * BATCH) {
        f32x4 values[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; u++) values[u] = pieces[min(p0 + u * SAMPLE_THREADS, n_pieces - 1)];
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            int p = p0 + u * SAMPLE_THREADS;
            if (p < n_pieces) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int i = head + 4 * p + e;
                    if (beats(values[u][e], i, best, best_index)) {
                        best = values[u][e];
                        best_index = i;
                    }
                }
            }
        }
    }
    block_best(best, best_index, shared_values, shared_indices);
    if (!(temperature > 0.0f) || best != best) {  // greedy, or a NaN in the row
        if (tid == 0) {
            out_tokens[row] = best_index;
            if (token_slot >= 0) token_slots[token_slot] = best_index;
        }
        return;
    }

    const float inverse_t = 1.0f / temperature;
    const float top_p = top_ps ? top_ps[row] : 1.0f;
    float cut = 0.0f;  // keep tokens whose weight exp((x - max)/T) is >= cut
    if (top_p < 1.0f) {
        float local = 0.0f;
        for (int i = tid; i < vocab; i += SAMPLE_THREADS) local += expf((x[i] - best) * inverse_t);
        float mass = block_sum(local, shared_values) * top_p;
        // Smallest weight w (as an ordered bit pattern) with sum(weights > w) < mass. The sum is
        // monotone in w, the weights lie in [0, 1], and the largest one is exactly 1.
        uint32_t low = 0u, high = 0x3f800000u;  // high always satisfies it: nothing is above 1
        while (low < high) {
            uint32_t middle = low + (high - low) / 2;
            float w = __uint_as_float(middle);
            float above = 0.0f;
            for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
                float e = expf((x[i] - best) * inverse_t);
                above += e > w ? e : 0.0f;
            }
            if (block_sum(above, shared_values) < mass) high = middle;
            else low = middle + 1;
        }
        cut = __uint_as_float(low);
    }

    const uint64_t seed = seeds ? seeds[row] : 0ull;
    const uint32_t step = steps ? (uint32_t)steps[row] : 0u;
    float chosen = -INFINITY;
    int chosen_index = 0x7fffffff;
    for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
        float scaled = (x[i] - best) * inverse_t;
        if (expf(scaled) >= cut) {
            float u = uniform_open(seed, step, (uint32_t)i);
            float noisy = scaled - logf(-logf(u));
            if (beats(noisy, i, chosen, chosen_index)) {
                chosen = noisy;
                chosen_index = i;
            }
        }
    }
    block_best(chosen, chosen_index, shared_values, shared_indices);
    if (tid == 0) {
        out_tokens[row] = chosen_index;
        if (token_slot >= 0) token_slots[token_slot] = chosen_index;
    }
}

// The end of a decode step that chooses its tokens on the device: per row the best of its candidates
// (what mllm_gemm_best left of a greedy step's logits; or one candidate a row, the token another
// kernel drew), and everything the next step of the same requests needs, so that the host neither
// reads nor writes device memory between two steps (the reference feeds the token back on the
// device and reads it from the host later: engine/src/gpt2_gpu_greedy.cu:80-123,
// docs/kernels/007_fewer_launches.md:54).
//
// Per live row r (state_slots[r] >= 0; other rows are padding and give -1): the token goes to out_tokens[r], to the
// request's last-token slot token_slots[state_slots[r]], and to row *cursor of the ring of token rows in page-locked host
// memory (one store of the whole row by the first lanes: the host reads it after the event that
// follows the step). With `advance` the row's position and stored length grow by one, its cache row
// of every group is looked up in the block table for the new position (-1 where the table has no page
// there yet: the host brings the table before that step runs), its token source becomes its own
// slot, and its entry of draw_counts (if given: how many tokens the row's request has drawn, which the
// sampler's random numbers are a function of) grows by one. A block takes 16 rows, a wave a row.
struct StepGroups {
    const int* tables[4];
    int* slots[4];
    int count, table_width, page_shift;
};

constexpr int CHOOSE_THREADS = 1024;
constexpr int CHOOSE_ROWS = CHOOSE_THREADS / WAVE;  // rows a block takes: a wave a row

__global__ __launch_bounds__(CHOOSE_THREADS) void choose_kernel(
    const float* __restrict__ values, const int* __restrict__ indices, int per_row, int n_rows,
    const int* __restrict__ state_slots, int* __restrict__ token_slots,
    int* __restrict__ out_tokens, int* __restrict__ host_ring, int ring_rows, int ring_stride, int* __restrict__ cursor,
    int advance, int* __restrict__ positions, int* __restrict__ context_lens, int* __restrict__ token_sources,
    int* __restrict__ draw_counts, StepGroups groups) {
    __shared__ int chosen[CHOOSE_ROWS];
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int ring_row = cursor ? cursor[0] : 0;
    const int sequence = cursor ? cursor[1] : 0;
    // A wave takes a row; its candidates are asked for eight a lane at a time before any is compared: a candidate was
    // written by some other compute unit and comes from memory.
    const int row = blockIdx.x * CHOOSE_ROWS + wave;
    constexpr int BATCH = 8;
    if (row < n_rows) {
        float best = -INFINITY;
        int best_index = 0x7fffffff;
        const size_t base = (size_t)row * per_row;
        for (int c0 = lane; c0 < per_row; c0 += WAVE * BATCH) {
            float value[BATCH];
            int index[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; u++) {
                int c = min(c0 + u * WAVE, per_row - 1);
                value[u] = values ? values[base + c] : 0.0f;
                index[u] = indices[base + c];
            }
#pragma unroll
            for (int u = 0; u < BATCH; u++)
                if (c0 + u * WAVE < per_row && beats(value[u], index[u], best, best_index)) {
                    best = value[u];
                    best_index = index[u];
                }
        }
#pragma unroll
        for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
            float other = __shfl_xor(best, offset, WAVE);
            int other_index = __shfl_xor(best_index, offset, WAVE);
            if (beats(other, other_index, best, best_index)) {
                best = other;
                best_index = other_index;
            }
        }
        if (lane == 0) chosen[wave] = best_index;
    }
    __syncthreads();
    if (tid < CHOOSE_ROWS && blockIdx.x * CHOOSE_ROWS + tid < n_rows) {   // the block's rows, a lane each: one store of their tokens
        const int row = blockIdx.x * CHOOSE_ROWS + tid;
        const int slot = state_slots[row];
        const bool live = slot >= 0;
        const int token = live ? chosen[tid] : -1;
        out_tokens[row] = token;
        if (host_ring) {
            host_ring[(size_t)ring_row * ring_stride + row] = token;
            __threadfence_system();   // the token is in host memory before the block's number (below) can be
        }
        if (live) {
            token_slots[slot] = token;
            if (advance) {
                const int position = positions[row] + 1;
                positions[row] = position;
                context_lens[row] = position;
                token_sources[row] = slot;
                if (draw_counts) draw_counts[row] += 1;   // a sampled row's next draw is its request's next one
                const int block = position >> groups.page_shift, offset = position & ((1 << groups.page_shift) - 1);
                for (int g = 0; g < groups.count; g++) {
                    int page = block < groups.table_width ? groups.tables[g][(size_t)row * groups.table_width + block] : -1;
                    groups.slots[g][row] = page >= 0 ? (page << groups.page_shift) + offset : -1;
                }
            }
        }
    }
    if (cursor) {
        // The row's last entries, one a block, say which step's tokens the row holds: whoever reads the ring on the
        // host waits for that number in all of them instead of an event behind the step (which costs the device about
        // 6 us between two steps). The block that finishes last moves the cursor on: every block has read it by then.
        __syncthreads();
        if (tid == 0) {
            host_ring[(size_t)ring_row * ring_stride + ring_stride - 1 - blockIdx.x] = sequence;
            const int arrived = atomicAdd(&cursor[2], 1);
            if (arrived == (int)gridDim.x - 1) {
                cursor[2] = 0;
                cursor[0] = (ring_row + 1) % ring_rows;
                cursor[1] = (sequence + 1) & 0x3fffffff;
            }
        }
    }
}

}  // namespace

MLLM_API int mllm_sample(const float* logits, int n_rows, int vocab, const float* temperatures,
                         const float* top_ps, const unsigned long long* seeds, const int* steps,
                         int* out_tokens, int* token_slots, const int* slot_of_row, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", n_rows, vocab);
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_SAMPLE);
    sample_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, vocab, temperatures, top_ps,
                                                         (const uint64_t*)seeds, steps, out_tokens, token_slots, slot_of_row);
    return mllm_check_launch("sample");
}

// See choose_kernel. values may be null (every row has candidates of equal rank: the first index
// wins, with per_row = 1 the one given); host_ring and cursor may be null; without `advance` the
// arrays behind it are not touched. group_tables / group_slots: n_groups pointers each.
MLLM_API int mllm_choose(const float* values, const int* indices, int per_row, int n_rows,
                         const int* state_slots, int* token_slots, int* out_tokens, int* host_ring, int ring_rows,
                         int ring_stride, int* cursor, int advance, int* positions, int* context_lens, int* token_sources,
                         int* draw_counts, const int* const* group_tables, int* const* group_slots, int n_groups, int table_width,
                         int page_size, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_rows <= 8192 && per_row >= 1, "choose: bad sizes rows=%d candidates=%d", n_rows, per_row);
    MLLM_REQUIRE(indices && state_slots && token_slots && out_tokens, "choose: an operand is missing");
    const int n_blocks = ceil_div(n_rows, CHOOSE_ROWS);
    MLLM_REQUIRE(!host_ring || (ring_rows >= 1 && ring_stride >= n_rows + (cursor ? n_blocks : 0)), "choose: the ring's rows are shorter than the batch (and, with a cursor, an entry for each 16 rows' step number)");
    MLLM_REQUIRE(!cursor || host_ring, "choose: a cursor without a ring");
    StepGroups groups{};
    if (advance) {
        MLLM_REQUIRE(positions && context_lens && token_sources, "choose: nothing to advance");
        MLLM_REQUIRE(n_groups >= 0 && n_groups <= 4, "choose: %d cache groups, at most 4 are advanced on the device", n_groups);
        MLLM_REQUIRE(page_size > 0 && (page_size & (page_size - 1)) == 0 && (n_groups == 0 || table_width > 0), "choose: bad page size or table width");
        for (int g = 0; g < n_groups; g++) {
            MLLM_REQUIRE(group_tables[g] && group_slots[g], "choose: group %d has no table or slots", g);
            groups.tables[g] = group_tables[g];
            groups.slots[g] = group_slots[g];
        }
        groups.count = n_groups;
        groups.table_width = table_width;
        while ((1 << groups.page_shift) < page_size) groups.page_shift++;
    }
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_CHOOSE);
    choose_kernel<<<n_blocks, CHOOSE_THREADS, 0, stream>>>(
        values, indices, per_row, n_rows, state_slots, token_slots, out_tokens, host_ring, ring_rows, ring_stride,
        cursor, advance, positions, context_lens, token_sources, advance ? draw_counts : nullptr, groups);
    return mllm_check_launch("choose");
}
