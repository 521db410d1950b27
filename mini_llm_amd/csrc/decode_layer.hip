// A pre-norm layer for rows that bring one token each (decoding), in two kernels instead of
// seven. bfloat16 matrices and cache, everything between them in 32-bit.
//
// A kernel boundary costs a few microseconds whatever the kernel does, and a decode step of a
// small model is little else. Two observations remove most boundaries:
//   * norm -> q/k/v product -> attention -> output product depends, for one head of one token,
//     on that head's rows of the q/k/v matrix and that head's columns of the output matrix only.
//     A block per (token, head) runs the whole chain and leaves its head's share of the output
//     product, a partial row [width], unsummed.
//   * norm -> up product -> activation -> down product depends, for one slice of the hidden
//     units, on that slice's rows of the up matrix and columns of the down matrix only. A block
//     per (slice, 16 tokens) runs the chain and leaves a partial row per token, unsummed.
// The residual stream between the kernels is therefore "pending": a base row, a bias, and a
// stack of partial rows that the next kernel adds up, always in the same order, while it
// computes the norm it needs anyway. Nothing is accumulated with atomics: the result does not
// depend on the order in which blocks finish.
//
// Matrix products run on the matrix cores with W as the 16-row operand, streamed from memory
// straight into registers (a lane loads 16 bytes of one of 16 rows), and the activations, which
// are tiny, as the other operand from LDS.
#include "common.h"
#include "key_sweep.h"

namespace {

constexpr int DL_WAVES = 16;
constexpr int DL_THREADS = DL_WAVES * WAVE;
constexpr int DL_MAX_WIDTH = 2048;  // a row's 4-column pieces: at most 2 per thread of a block, 8 per lane of a wave
constexpr int DL_KSPLIT = 4;        // waves that share the k range of one 16-row tile
constexpr int DL_TOKENS = 16;       // tokens a feed-forward block takes: the matrix core's other 16

// Tuning aid, compiled in with -DMLLM_PHASE_STAMPS only: block (1, 1) notes the 100 MHz clock at
// the numbered places of a kernel (places 20.. by the first lane of wave 8, the others by thread
// 0); mllm_phase_stamps() copies the notes out.
#ifdef MLLM_PHASE_STAMPS
__device__ long long dl_stamps[32];
#define DL_STAMP(i)                                                                         \
    do {                                                                                    \
        if (blockIdx.x == 1 && blockIdx.y == (gridDim.y > 1) && threadIdx.x == ((i) >= 20 ? 512 : 0)) dl_stamps[i] = wall_clock64(); \
    } while (0)
#else
#define DL_STAMP(i)
#endif

struct PendingSum {
    const float* base;      // [rows, width]
    const float* partials;  // [n_partials, rows, width]
    const float* bias;      // [width] or null, added once
    int n_partials;
    int rows;
};

__device__ __forceinline__ f32x4 load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }

__device__ __forceinline__ Vec16 mask16(Vec16 v, bool keep) {
    Vec16 out;
#pragma unroll
    for (int i = 0; i < 4; i++) out.w[i] = keep ? v.w[i] : 0u;
    return out;
}

__device__ __forceinline__ void store_bf16x4(bf16_t* at, f32x4 v) {
    bf16x4 packed;
#pragma unroll
    for (int e = 0; e < 4; e++) packed[e] = static_cast<bf16_t>(v[e]);
    *reinterpret_cast<bf16x4*>(at) = packed;
}

// The block's waves meet once this wave's LDS traffic is done. Unlike __syncthreads() it does not
// wait for this wave's loads from memory: what was asked for early stays in flight across it. Only
// LDS carries data between the waves of a block here, so nothing more is needed.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ------------------------------------------------------------------------------------------------
// norm -> q/k/v -> cache write -> attention over the cache -> this head's share of the output
// product. grid (n_heads, tokens), 1024 threads in two roles:
//   waves 0..7  "project": norm, q/k/v product, output product;
//   waves 8..15 "attend":  ask for their shares of the cached keys and values at once, wait for
//                          the query, then run the softmax over them.
// A wave's loads from memory complete in the order they were issued, so a wave that asks for the
// keys early cannot use anything it asks for later before the keys have come: hence the roles.
// All 16 waves share the pending sums first (short loads from the cache of the chip).
// ------------------------------------------------------------------------------------------------
constexpr int DL_PROJECT_WAVES = 8, DL_ATTEND_WAVES = DL_WAVES - DL_PROJECT_WAVES;
constexpr int DL_PROJECT_THREADS = DL_PROJECT_WAVES * WAVE;

template <int HD>
__global__ __launch_bounds__(DL_THREADS) void decode_attention_half_kernel(
    PendingSum in, float* __restrict__ summed,  // [tokens, width]: the stream with its sums taken, written by head 0
    const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
    const bf16_t* __restrict__ w_qkv, const float* __restrict__ b_qkv,  // [q_width + 2 kv_width, width]
    const bf16_t* __restrict__ w_out,                                    // [width, q_width]
    bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, const int* __restrict__ slots,
    const int* __restrict__ token_request, const int* __restrict__ positions,
    const int* __restrict__ block_tables, int max_blocks,
    float* __restrict__ partial_out,  // [n_heads, tokens, width]
    int n_tokens, int width, int n_heads, int n_kv_heads, int page_shift, int window, float scale, int write_cache) {
    typedef KeySweep<bf16_t, HD> Sweep;
    constexpr int VEC = Sweep::VEC, LPR = Sweep::LPR, RPI = Sweep::RPI, KPI = Sweep::KPI;
    constexpr int ROW_TILES = 3 * HD / 16;
    constexpr int UNITS = (ROW_TILES * DL_KSPLIT + DL_PROJECT_WAVES - 1) / DL_PROJECT_WAVES;  // (tile, k share) pairs a wave owns
    constexpr int AT_ONCE = UNITS < 3 ? UNITS : 3;  // of which it works on so many at a time,
    constexpr int ROUND = 18 / AT_ONCE;             // with so many k steps of each in flight
    constexpr int HD_PAD = (HD + 31) / 32 * 32;
    constexpr int OUT_STEPS = HD_PAD / 32, OUT_GROUP = OUT_STEPS <= 2 ? 12 / OUT_STEPS : (OUT_STEPS <= 4 ? 2 : 1);
    constexpr int ROWS_PER_THREAD = (3 * HD + DL_PROJECT_THREADS - 1) / DL_PROJECT_THREADS;
    constexpr int MAX_PIECES = DL_MAX_WIDTH / 4;

    __shared__ f32x4 stage[4][MAX_PIECES];
    __shared__ f32x4 row_lds[MAX_PIECES];
    __shared__ __attribute__((aligned(16))) bf16_t x_hat[DL_MAX_WIDTH];
    __shared__ float qkv_part[DL_KSPLIT][3 * HD];
    __shared__ float qkv_row[3][HD];  // q, k, v of this token and head, rounded as the cache holds them
    __shared__ float merged[DL_ATTEND_WAVES][HD + 2];
    __shared__ __attribute__((aligned(16))) bf16_t mixed[HD_PAD];

    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);  // the same in every lane: kept in a scalar register
    const bool attends = wave >= DL_PROJECT_WAVES;
    const int head = blockIdx.x, token = blockIdx.y;
    const int n_pieces = width / 4;
    DL_STAMP(0);
    float* out_row = partial_out + ((size_t)head * n_tokens + token) * width;
    const int request = token_request[token];
    if (request < 0) {  // a padding row: zeros, so that what follows stays finite
        for (int c = tid; c < width; c += DL_THREADS) {
            out_row[c] = 0.0f;
            if (head == 0) summed[(size_t)token * width + c] = 0.0f;
        }
        return;
    }
    const int position = positions[token];
    const int slot = slots[token];
    const int kv_head = head / (n_heads / n_kv_heads);
    const int q_width = n_heads * HD, kv_width = n_kv_heads * HD;
    const int row16 = lane % 16, quad = lane / 16;

    // ---- the pending sums of this token's row, by all waves: four groups of 256 threads take
    // every fourth partial row each; the four sums meet in LDS and are added in a fixed order
    {
        const int group = tid / 256, piece0 = tid % 256;
#pragma unroll
        for (int j = 0; j < MAX_PIECES / 256; j++) {
            if (256 * j >= n_pieces) break;  // the same for every thread
            int piece = piece0 + 256 * j;
            int safe_piece = min(piece, n_pieces - 1);
            f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int s0 = group; s0 < in.n_partials; s0 += 4 * 12) {
                f32x4 part[12];
#pragma unroll
                for (int u = 0; u < 12; u++) {
                    int s = min(s0 + 4 * u, in.n_partials - 1);
                    part[u] = load4(in.partials + ((size_t)s * in.rows + token) * width + 4 * safe_piece);
                }
#pragma unroll
                for (int u = 0; u < 12; u++)
                    if (s0 + 4 * u < in.n_partials) sum += part[u];
            }
            stage[group][piece] = sum;
        }
    }

    // From here on the two roles run apart: each passes the same seven meetings of the waves, so
    // that a role's registers hold that role's data only.
    if (attends) {
        // ---- the waves that attend ask for their shares of the cached keys and values now, and
        // for nothing else until they have used them
        const int first_key = window > 0 ? max(0, position - window + 1) : 0;
        const int n_cached = position - first_key;
        const int chunk = (((n_cached + DL_ATTEND_WAVES - 1) / DL_ATTEND_WAVES + RPI - 1) / RPI) * RPI;
        const int begin = first_key + (wave - DL_PROJECT_WAVES) * chunk;
        const int end = min(position, begin + chunk);
        const int* table = block_tables + (size_t)request * max_blocks;
        Sweep sweep;
        typename Sweep::Fetched fetched;
        // a wave without keys asks for the token's own slot instead: a page the table holds, never used
        sweep.fetch(fetched, k_pages, v_pages, table, kv_head, n_kv_heads, page_shift, begin, end, begin < end ? end - 1 : position, lane);
        DL_STAMP(20);
        lds_barrier();  // 1
        lds_barrier();  // 2
        lds_barrier();  // 3
        lds_barrier();  // 4
        lds_barrier();  // 5: q, k, v of this token are in LDS
        // the waves that attend share the cached keys before this token; the token's own key and
        // value come from LDS (the first of them)
        DL_STAMP(21);
        const int sub = lane % LPR;
        float qf[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) qf[i] = qkv_row[0][sub * VEC + i] * scale;
        sweep.init();
        if (begin < end) {
            sweep.consume(fetched, qf, begin, end, lane);
            if (begin + KPI < end)  // a context longer than the first round of every wave covers
                sweep.keys(qf, k_pages, v_pages, table, kv_head, n_kv_heads, page_shift, begin + KPI, end, lane);
        }
        if (wave == DL_PROJECT_WAVES) sweep.one_key(qf, qkv_row[1], qkv_row[2], lane);
        sweep.merge_groups();
        if (lane < LPR) {
#pragma unroll
            for (int i = 0; i < VEC; i++) merged[wave - DL_PROJECT_WAVES][sub * VEC + i] = sweep.o[i];
        }
        if (lane == 0) {
            merged[wave - DL_PROJECT_WAVES][HD] = sweep.running_max;
            merged[wave - DL_PROJECT_WAVES][HD + 1] = sweep.running_sum;
        }
        DL_STAMP(22);
        lds_barrier();  // 6: every wave's (max, sum, output) is in LDS
        lds_barrier();  // 7
        return;
    }

    // ---- the waves that project: first what they need of the vectors
    const bool owns = tid < n_pieces;  // threads 0 .. width/4-1 own four columns of the row each
    const int own_piece = min(tid, n_pieces - 1);
    f32x4 row = load4(in.base + (size_t)token * width + 4 * own_piece);
    if (in.bias) row += load4(in.bias + 4 * own_piece);
    const f32x4 gain = load4(gamma + 4 * own_piece), offset = load4(beta + 4 * own_piece);
    float qkv_bias[ROWS_PER_THREAD];
#pragma unroll
    for (int i = 0; i < ROWS_PER_THREAD; i++) {
        int r = min(tid + DL_PROJECT_THREADS * i, 3 * HD - 1), which = r / HD, within = r % HD;
        int w_row = which == 0 ? head * HD + within : q_width + (which - 1) * kv_width + kv_head * HD + within;
        qkv_bias[i] = b_qkv ? b_qkv[w_row] : 0.0f;
    }
    DL_STAMP(1);
    lds_barrier();  // 1: the four groups' sums are in LDS
    // width / 4 <= 512: the threads of these waves cover the row
    if (owns) {
        row += ((stage[0][tid] + stage[1][tid]) + stage[2][tid]) + stage[3][tid];
        if (head == 0) *reinterpret_cast<f32x4*>(summed + (size_t)token * width + 4 * tid) = row;
    } else {
        row = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    row_lds[tid] = row;
    lds_barrier();  // 2: the row with its sums taken is in LDS

    // the norm, centred, in 32-bit: every wave takes the statistics of the whole row for itself (no
    // further meeting of the waves), then norms the four columns it owns
    {
        const float n = (float)width;
        f32x4 others[MAX_PIECES / WAVE];
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < MAX_PIECES / WAVE; j++) {
            others[j] = row_lds[lane + WAVE * j];  // zeros beyond the width
            sum += (others[j][0] + others[j][1]) + (others[j][2] + others[j][3]);
        }
        const float mean = wave_sum(sum) / n;
        float squares = 0.0f;
#pragma unroll
        for (int j = 0; j < MAX_PIECES / WAVE; j++) {
            f32x4 d = lane + WAVE * j < n_pieces ? others[j] - mean : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            squares += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
        }
        const float inverse_stddev = 1.0f / sqrtf(wave_sum(squares) / n + eps);
        f32x4 y = (row - mean) * inverse_stddev * gain + offset;
        if (!owns) y = f32x4{0.0f, 0.0f, 0.0f, 0.0f};  // beyond the width: zeros, the products read whole 32-column steps
        store_bf16x4(x_hat + 4 * tid, y);
    }
    lds_barrier();  // 3: the normed row is in LDS
    DL_STAMP(2);

    // q, k, v of this head: 3*HD rows of the matrix in tiles of 16, each tile's k range shared by
    // DL_KSPLIT waves; a wave owns UNITS (tile, share) pairs
    {
        const int n_steps = (width + 31) / 32;
        const int steps_per_unit = (n_steps + DL_KSPLIT - 1) / DL_KSPLIT;
#pragma unroll 1
        for (int u0 = 0; u0 < UNITS; u0 += AT_ONCE) {
            int w_at[AT_ONCE];  // offsets into w_qkv: the matrix has fewer than 2^31 elements
            int part[AT_ONCE], tile[AT_ONCE];
            f32x4 acc[AT_ONCE];
#pragma unroll
            for (int u = 0; u < AT_ONCE; u++) {
                int unit = min(wave + DL_PROJECT_WAVES * (u0 + u), ROW_TILES * DL_KSPLIT - 1);  // beyond the last: computed again, not kept
                tile[u] = unit % ROW_TILES, part[u] = unit / ROW_TILES;
                int local = tile[u] * 16 + row16, which = local / HD, within = local % HD;
                int w_row = which == 0 ? head * HD + within : q_width + (which - 1) * kv_width + kv_head * HD + within;
                w_at[u] = w_row * width;
                acc[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
#pragma unroll 1
            for (int i0 = 0; i0 < steps_per_unit; i0 += ROUND) {
                Vec16 w_piece[AT_ONCE][ROUND];
#pragma unroll
                for (int u = 0; u < AT_ONCE; u++)
#pragma unroll
                    for (int j = 0; j < ROUND; j++) {
                        int k = (part[u] + DL_KSPLIT * (i0 + j)) * 32 + quad * 8;
                        w_piece[u][j] = *reinterpret_cast<const Vec16*>(w_qkv + (w_at[u] + min(k, width - 8)));
                    }
#pragma unroll
                for (int u = 0; u < AT_ONCE; u++)
#pragma unroll
                    for (int j = 0; j < ROUND; j++) {
                        int step = part[u] + DL_KSPLIT * (i0 + j);
                        Vec16 w = mask16(w_piece[u][j], step * 32 + quad * 8 < width);
                        bf16x8 x = *reinterpret_cast<const bf16x8*>(x_hat + min(step, n_steps - 1) * 32 + quad * 8);
                        acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&w), x, acc[u], 0, 0, 0);
                    }
            }
            // every column of the product is this one token; column 0 is kept
#pragma unroll
            for (int u = 0; u < AT_ONCE; u++)
                if (row16 == 0 && wave + DL_PROJECT_WAVES * (u0 + u) < ROW_TILES * DL_KSPLIT) {
#pragma unroll
                    for (int r = 0; r < 4; r++) qkv_part[part[u]][tile[u] * 16 + 4 * quad + r] = acc[u][r];
                }
        }
    }
    // the output product's rows are asked for now, not earlier (the compiler would move these loads
    // up among the ones above and run out of registers): they are needed last
    asm volatile("" ::: "memory");
    Vec16 out_piece[OUT_GROUP][OUT_STEPS];
#pragma unroll
    for (int g = 0; g < OUT_GROUP; g++) {
        int out_col = min((wave + DL_PROJECT_WAVES * g) * 16 + row16, width - 1);
#pragma unroll
        for (int s = 0; s < OUT_STEPS; s++)
            out_piece[g][s] = *reinterpret_cast<const Vec16*>(w_out + (size_t)out_col * q_width + head * HD + min(s * 32 + quad * 8, HD - 8));
    }
    DL_STAMP(3);
    lds_barrier();  // 4: the shares of the q/k/v product are in LDS
#pragma unroll
    for (int i = 0; i < ROWS_PER_THREAD; i++) {
        const int r = tid + DL_PROJECT_THREADS * i;
        if (r < 3 * HD) {
            const int which = r / HD, within = r % HD;
            float value = ((qkv_part[0][r] + qkv_part[1][r]) + qkv_part[2][r]) + qkv_part[3][r] + qkv_bias[i];
            bf16_t kept = static_cast<bf16_t>(value);
            qkv_row[which][within] = static_cast<float>(kept);
            if (which > 0 && write_cache && slot >= 0 && head % (n_heads / n_kv_heads) == 0) {
                int page = slot >> page_shift, at = slot & ((1 << page_shift) - 1);
                bf16_t* pages = which == 1 ? k_pages : v_pages;
                pages[((((size_t)page * n_kv_heads + kv_head) << page_shift) + at) * HD + within] = kept;
            }
        }
    }
    lds_barrier();  // 5: q, k, v of this token are in LDS
    DL_STAMP(4);
    lds_barrier();  // 6: the waves that attend are done
    DL_STAMP(5);
    if (tid < HD_PAD) {  // HD_PAD <= 256 threads
        float value = 0.0f;
        if (tid < HD) {
            float total_max = -INFINITY;
            for (int s = 0; s < DL_ATTEND_WAVES; s++) total_max = fmaxf(total_max, merged[s][HD]);
            float total = 0.0f;
            for (int s = 0; s < DL_ATTEND_WAVES; s++) {
                float weight = expf(merged[s][HD] - total_max);
                total += merged[s][HD + 1] * weight;
                value += merged[s][tid] * weight;
            }
            value /= total;
        }
        mixed[tid] = static_cast<bf16_t>(value);
    }
    lds_barrier();  // 7: the mixed row of this head is in LDS
    DL_STAMP(6);

    // this head's share of the output product: rows of w_out in tiles of 16, columns head*HD ..
    {
        const int n_tiles = (width + 15) / 16;
        for (int tile0 = wave; tile0 < n_tiles; tile0 += DL_PROJECT_WAVES * OUT_GROUP) {
            if (tile0 != wave) {  // wider than the rows asked for above cover
#pragma unroll
                for (int g = 0; g < OUT_GROUP; g++) {
                    int out_col = min((tile0 + DL_PROJECT_WAVES * g) * 16 + row16, width - 1);
#pragma unroll
                    for (int s = 0; s < OUT_STEPS; s++)
                        out_piece[g][s] = *reinterpret_cast<const Vec16*>(w_out + (size_t)out_col * q_width + head * HD + min(s * 32 + quad * 8, HD - 8));
                }
            }
#pragma unroll
            for (int g = 0; g < OUT_GROUP; g++) {
                int tile = tile0 + DL_PROJECT_WAVES * g;
                f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int s = 0; s < OUT_STEPS; s++) {
                    Vec16 w = mask16(out_piece[g][s], s * 32 + quad * 8 < HD && tile * 16 + row16 < width);
                    bf16x8 x = *reinterpret_cast<const bf16x8*>(mixed + s * 32 + quad * 8);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&w), x, acc, 0, 0, 0);
                }
                int out_col = tile * 16 + 4 * quad;  // 4 columns; the width is a multiple of 4
                if (row16 == 0 && out_col < width) *reinterpret_cast<f32x4*>(out_row + out_col) = acc;
            }
        }
    }
    DL_STAMP(7);
}

// ------------------------------------------------------------------------------------------------
// norm -> up product -> activation -> this slice's share of the down product.
// grid (slices of U hidden units, groups of 16 tokens), 1024 threads. The first pieces of both
// matrices are asked for at once; while they come, the waves take the pending sums (16 / tokens
// waves a token, every so-manieth partial row each) and the norm; then all waves run the two
// products.
// ------------------------------------------------------------------------------------------------
template <int NV, int U>
__global__ __launch_bounds__(DL_THREADS) void decode_mlp_half_kernel(
    PendingSum in, float* __restrict__ summed, const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
    const bf16_t* __restrict__ w_up, const float* __restrict__ b_up,  // [inner, width]
    const bf16_t* __restrict__ w_down,                                 // [width, inner]
    float* __restrict__ partial_out,                                   // [slices, tokens, width]
    int n_tokens, int width, int inner, int epilogue, int stage_pieces) {
    constexpr int TILES = U / 16, K_STEPS_DOWN = U / 32, H_STRIDE = U + 8;
    constexpr int UP_UNITS = (TILES * DL_KSPLIT + DL_WAVES - 1) / DL_WAVES;  // (tile, k share) pairs a wave owns
    constexpr int UP_ROUND = 6 / UP_UNITS;                                   // k steps of each in flight together
    constexpr int DOWN_GROUP = 6 / K_STEPS_DOWN;                             // output tiles a wave works on at a time
    constexpr int ROWS_AT_ONCE = NV <= 3 ? 4 : (NV <= 4 ? 2 : 1);            // partial rows asked for before any is added
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int x_stride = (width + 31) / 32 * 32 + 8;  // 16 bytes of padding: the 16 rows fall on different banks
    bf16_t* x_hat = reinterpret_cast<bf16_t*>(lds);                                          // [16][x_stride]
    float* up_part = reinterpret_cast<float*>(lds + (size_t)DL_TOKENS * x_stride * 2);        // [KSPLIT][TILES][4][64]
    bf16_t* hidden = reinterpret_cast<bf16_t*>(up_part + DL_KSPLIT * TILES * 256);            // [16][H_STRIDE]
    f32x4* stage = reinterpret_cast<f32x4*>(hidden + DL_TOKENS * H_STRIDE);                   // [16 waves][stage_pieces]

    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int slice = blockIdx.x, token0 = blockIdx.y * DL_TOKENS;
    const int n_pieces = width / 4;
    const int row16 = lane % 16, quad = lane / 16;
    const int n_steps = (width + 31) / 32;
    const int steps_per_unit = (n_steps + DL_KSPLIT - 1) / DL_KSPLIT;
    DL_STAMP(10);

    // ---- the pending sums and the norm. With T tokens in this block (rounded up to a power of
    // two), wave w works for token w % T and takes the partial rows w / T, w / T + 16 / T, ...
    // A wave's loads complete in the order they were issued: the first partial rows are asked for
    // first, then the first pieces of both matrices, which stay in flight through all that follows
    // until the products need them.
    const int tokens_here = min(DL_TOKENS, n_tokens - token0);
    int t2 = 1;
    while (t2 < tokens_here) t2 *= 2;
    if (stage_pieces < n_pieces) t2 = DL_TOKENS;  // no room to share a token's sums among waves
    const int waves_per_token = DL_WAVES / t2;
    const int local = wave % t2, sub = wave / t2;
    const int token = token0 + local;
    const bool live = token < n_tokens;
    const int safe_token = live ? token : n_tokens - 1;
    f32x4 row[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        int piece = min(lane + WAVE * j, n_pieces - 1);
        row[j] = load4(in.base + (size_t)safe_token * width + 4 * piece);
        if (in.bias) row[j] += load4(in.bias + 4 * piece);
        if (sub != 0) row[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    f32x4 part[ROWS_AT_ONCE][NV];
    auto ask_for_partial_rows = [&](int s0) {
#pragma unroll
        for (int u = 0; u < ROWS_AT_ONCE; u++) {
            int s = max(0, min(s0 + waves_per_token * u, in.n_partials - 1));
#pragma unroll
            for (int j = 0; j < NV; j++)
                part[u][j] = load4((in.n_partials ? in.partials : in.base) + ((size_t)s * in.rows + safe_token) * width + 4 * min(lane + WAVE * j, n_pieces - 1));
        }
    };
    ask_for_partial_rows(sub);

    int up_at[UP_UNITS], up_part_of[UP_UNITS], up_tile[UP_UNITS];
    bool up_valid[UP_UNITS];
    Vec16 up_piece[UP_UNITS][UP_ROUND];
#pragma unroll
    for (int u = 0; u < UP_UNITS; u++) {
        int unit = min(wave + DL_WAVES * u, TILES * DL_KSPLIT - 1);
        up_tile[u] = unit % TILES, up_part_of[u] = unit / TILES;
        int h = slice * U + up_tile[u] * 16 + row16;
        up_valid[u] = h < inner;
        up_at[u] = min(h, inner - 1) * width;
#pragma unroll
        for (int j = 0; j < UP_ROUND; j++) {
            int k = (up_part_of[u] + DL_KSPLIT * j) * 32 + quad * 8;
            up_piece[u][j] = *reinterpret_cast<const Vec16*>(w_up + (up_at[u] + min(k, width - 8)));
        }
    }
    Vec16 down_piece[DOWN_GROUP][K_STEPS_DOWN];
#pragma unroll
    for (int g = 0; g < DOWN_GROUP; g++) {
        int out_col = min((wave + DL_WAVES * g) * 16 + row16, width - 1);
#pragma unroll
        for (int s = 0; s < K_STEPS_DOWN; s++)
            down_piece[g][s] = *reinterpret_cast<const Vec16*>(w_down + (size_t)out_col * inner + min(slice * U + s * 32 + quad * 8, inner - 8));
    }

    {
        for (int s0 = sub; s0 < in.n_partials; s0 += waves_per_token * ROWS_AT_ONCE) {
            if (s0 != sub) ask_for_partial_rows(s0);
#pragma unroll
            for (int u = 0; u < ROWS_AT_ONCE; u++)
                if (s0 + waves_per_token * u < in.n_partials) {
#pragma unroll
                    for (int j = 0; j < NV; j++) row[j] += part[u][j];
                }
        }
        if (waves_per_token > 1) {  // the same for the whole block
#pragma unroll
            for (int j = 0; j < NV; j++)
                if (lane + WAVE * j < n_pieces) stage[wave * stage_pieces + lane + WAVE * j] = row[j];
            lds_barrier();
            if (sub == 0) {
                for (int other = 1; other < waves_per_token; other++) {
#pragma unroll
                    for (int j = 0; j < NV; j++)
                        if (lane + WAVE * j < n_pieces) row[j] += stage[(other * t2 + local) * stage_pieces + lane + WAVE * j];
                }
            }
        }
        DL_STAMP(11);
        bf16_t* x_row = x_hat + wave * x_stride;  // wave w < t2 is token w's first wave; the others clear the rows from t2 on
        if (sub == 0 && live) {
            float sum = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++) {
                if (lane + WAVE * j >= n_pieces) row[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                else if (slice == 0) *reinterpret_cast<f32x4*>(summed + (size_t)token * width + 4 * (lane + WAVE * j)) = row[j];
                sum += (row[j][0] + row[j][1]) + (row[j][2] + row[j][3]);
            }
            const float n = (float)width;
            const float mean = wave_sum(sum) / n;
            float squares = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++) {
                row[j] = lane + WAVE * j < n_pieces ? row[j] - mean : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                squares += (row[j][0] * row[j][0] + row[j][1] * row[j][1]) + (row[j][2] * row[j][2] + row[j][3] * row[j][3]);
            }
            const float inverse_stddev = 1.0f / sqrtf(wave_sum(squares) / n + eps);
#pragma unroll
            for (int j = 0; j < NV; j++)
                if (lane + WAVE * j < n_pieces) {
                    int piece = lane + WAVE * j;
                    store_bf16x4(x_row + 4 * piece, row[j] * inverse_stddev * load4(gamma + 4 * piece) + load4(beta + 4 * piece));
                }
            for (int c = width + lane; c < x_stride - 8; c += WAVE) x_row[c] = static_cast<bf16_t>(0.0f);
        } else {
            for (int c = lane; c < x_stride - 8; c += WAVE) x_row[c] = static_cast<bf16_t>(0.0f);
        }
    }
    lds_barrier();
    DL_STAMP(12);

    // ---- up product for this slice's U hidden units: TILES tiles of 16 rows, DL_KSPLIT waves a tile
    {
        f32x4 acc[UP_UNITS];
#pragma unroll
        for (int u = 0; u < UP_UNITS; u++) acc[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        for (int i0 = 0; i0 < steps_per_unit; i0 += UP_ROUND) {
            if (i0 > 0) {  // wider than the first round covers
#pragma unroll
                for (int u = 0; u < UP_UNITS; u++)
#pragma unroll
                    for (int j = 0; j < UP_ROUND; j++) {
                        int k = (up_part_of[u] + DL_KSPLIT * (i0 + j)) * 32 + quad * 8;
                        up_piece[u][j] = *reinterpret_cast<const Vec16*>(w_up + (up_at[u] + min(k, width - 8)));
                    }
            }
#pragma unroll
            for (int u = 0; u < UP_UNITS; u++)
#pragma unroll
                for (int j = 0; j < UP_ROUND; j++) {
                    int step = up_part_of[u] + DL_KSPLIT * (i0 + j);
                    Vec16 w = mask16(up_piece[u][j], step * 32 + quad * 8 < width && up_valid[u]);
                    bf16x8 x = *reinterpret_cast<const bf16x8*>(x_hat + row16 * x_stride + min(step, n_steps - 1) * 32 + quad * 8);
                    acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&w), x, acc[u], 0, 0, 0);
                }
        }
#pragma unroll
        for (int u = 0; u < UP_UNITS; u++)
            if (wave + DL_WAVES * u < TILES * DL_KSPLIT) {
#pragma unroll
                for (int r = 0; r < 4; r++) up_part[((up_part_of[u] * TILES + up_tile[u]) * 4 + r) * WAVE + lane] = acc[u][r];
            }
    }
    DL_STAMP(13);
    lds_barrier();
    // acc[r] of lane l in tile t is (token l % 16, hidden unit 16 t + 4 (l / 16) + r)
    for (int index = tid; index < TILES * 256; index += DL_THREADS) {
        const int tile = index / 256, r = (index / WAVE) % 4, l = index % WAVE;
        float value = 0.0f;
#pragma unroll
        for (int p = 0; p < DL_KSPLIT; p++) value += up_part[((p * TILES + tile) * 4 + r) * WAVE + l];
        const int unit = tile * 16 + 4 * (l / 16) + r, h = slice * U + unit;
        if (h < inner) {
            if (b_up) value += b_up[h];
            if (epilogue == MLLM_EPI_GELU_TANH) value = gelu_tanh(value);
            else if (epilogue == MLLM_EPI_GELU_ERF) value = gelu_erf(value);
        } else {
            value = 0.0f;
        }
        hidden[(l % 16) * H_STRIDE + unit] = static_cast<bf16_t>(value);
    }
    lds_barrier();
    DL_STAMP(14);

    // ---- this slice's share of the down product: rows of w_down in tiles of 16, columns slice*U ..
    {
        const int n_tiles = (width + 15) / 16;
        const int token = token0 + row16;
        for (int tile0 = wave; tile0 < n_tiles; tile0 += DL_WAVES * DOWN_GROUP) {
            if (tile0 != wave) {  // wider than the rows asked for at the start cover
#pragma unroll
                for (int g = 0; g < DOWN_GROUP; g++) {
                    int out_col = min((tile0 + DL_WAVES * g) * 16 + row16, width - 1);
#pragma unroll
                    for (int s = 0; s < K_STEPS_DOWN; s++)
                        down_piece[g][s] = *reinterpret_cast<const Vec16*>(w_down + (size_t)out_col * inner + min(slice * U + s * 32 + quad * 8, inner - 8));
                }
            }
#pragma unroll
            for (int g = 0; g < DOWN_GROUP; g++) {
                int tile = tile0 + DL_WAVES * g;
                f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int s = 0; s < K_STEPS_DOWN; s++) {
                    Vec16 w = mask16(down_piece[g][s], slice * U + s * 32 + quad * 8 < inner && tile * 16 + row16 < width);
                    bf16x8 x = *reinterpret_cast<const bf16x8*>(hidden + row16 * H_STRIDE + s * 32 + quad * 8);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&w), x, acc, 0, 0, 0);
                }
                int out_col = tile * 16 + 4 * quad;
                if (token < n_tokens && out_col < width)
                    *reinterpret_cast<f32x4*>(partial_out + ((size_t)slice * n_tokens + token) * width + out_col) = acc;
            }
        }
    }
    DL_STAMP(15);
}

// out = base + bias + the partial rows: the pending stream as plain rows, for whatever does not
// take it pending. grid (pieces of 256 x 4 columns, rows).
__global__ __launch_bounds__(256) void pending_sum_kernel(PendingSum in, float* __restrict__ out, int width) {
    const int piece = blockIdx.x * 256 + threadIdx.x, row_index = blockIdx.y;
    if (piece * 4 >= width) return;
    f32x4 row = load4(in.base + (size_t)row_index * width + 4 * piece);
    if (in.bias) row += load4(in.bias + 4 * piece);
    for (int s = 0; s < in.n_partials; s++) row += load4(in.partials + ((size_t)s * in.rows + row_index) * width + 4 * piece);
    *reinterpret_cast<f32x4*>(out + (size_t)row_index * width + 4 * piece) = row;
}

int check_pending(const char* what, const float* base, const float* partials, int n_partials, int width) {
    MLLM_REQUIRE(base != nullptr, "%s: no base rows", what);
    MLLM_REQUIRE(n_partials >= 0 && (n_partials == 0 || partials != nullptr), "%s: %d partial rows without memory", what, n_partials);
    MLLM_REQUIRE(width > 0 && width % 8 == 0 && width <= DL_MAX_WIDTH, "%s: width %d is not a multiple of 8 up to %d", what, width, DL_MAX_WIDTH);
    return 0;
}

template <int NV, int U>
int launch_mlp_half(PendingSum in, float* summed, const float* gamma, const float* beta, float eps, const bf16_t* w_up,
                    const float* b_up, const bf16_t* w_down, float* partial_out, int n_tokens, int width, int inner,
                    int epilogue, hipStream_t stream) {
    const int x_stride = (width + 31) / 32 * 32 + 8;
    size_t lds = (size_t)DL_TOKENS * x_stride * 2 + (size_t)DL_KSPLIT * (U / 16) * 256 * 4 + (size_t)DL_TOKENS * (U + 8) * 2;
    // room for the waves of a token to share its pending sums, if the row is short enough
    int stage_pieces = 0;
    if (lds + (size_t)DL_WAVES * (width / 4) * 16 <= 128 * 1024) {
        stage_pieces = width / 4;
        lds += (size_t)DL_WAVES * stage_pieces * 16;
    }
    static bool raised = false;  // per instantiation: the limit on dynamic LDS is a property of the kernel
    if (!raised && lds > 64 * 1024) {
        hipError_t status = hipFuncSetAttribute((const void*)decode_mlp_half_kernel<NV, U>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 1024);
        MLLM_REQUIRE(status == hipSuccess, "decode_mlp_half: cannot raise the LDS limit: %s", hipGetErrorString(status));
        raised = true;
    }
    dim3 grid((inner + U - 1) / U, (n_tokens + DL_TOKENS - 1) / DL_TOKENS);
    decode_mlp_half_kernel<NV, U><<<grid, DL_THREADS, lds, stream>>>(in, summed, gamma, beta, eps, w_up, b_up, w_down, partial_out,
                                                                      n_tokens, width, inner, epilogue, stage_pieces);
    return 0;
}

}  // namespace

// 1 if the two layer kernels take these sizes (bfloat16 only).
MLLM_API int mllm_decode_layer_supported(int width, int head_size, int page_size, int inner) {
    if (width <= 0 || width % 8 || width > DL_MAX_WIDTH) return 0;
    if (head_size != 0 && head_size != 16 && head_size != 32 && head_size != 64 && head_size != 128 && head_size != 256) return 0;
    if (head_size != 0 && (page_size <= 0 || (page_size & (page_size - 1)))) return 0;
    if (inner != 0 && (inner < 8 || inner % 8)) return 0;
    return 1;
}

MLLM_API int mllm_decode_attention_half(
    const float* base, const float* partials, const float* pending_bias, int n_partials, float* summed,
    const float* gamma, const float* beta, float eps, const void* w_qkv, const float* b_qkv, const void* w_out,
    void* k_pages, void* v_pages, const int* slots, const int* token_request, const int* positions,
    const int* block_tables, int max_blocks, float* partial_out, int n_tokens, int width, int n_heads, int n_kv_heads,
    int head_size, int page_size, int window, float scale, int write_cache, hipStream_t stream) {
    if (check_pending("decode_attention_half", base, partials, n_partials, width)) return 1;
    MLLM_REQUIRE(n_tokens >= 0 && n_tokens <= 65535, "decode_attention_half: %d tokens", n_tokens);
    MLLM_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "decode_attention_half: %d heads do not divide into %d key/value heads", n_heads, n_kv_heads);
    MLLM_REQUIRE(mllm_decode_layer_supported(width, head_size, page_size, 0) && head_size != 0,
                 "decode_attention_half: head size %d is not one of 16, 32, 64, 128, 256, or page size %d is no power of two", head_size, page_size);
    MLLM_REQUIRE(window >= 0 && max_blocks > 0, "decode_attention_half: bad window or table");
    if (n_tokens == 0) return 0;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) page_shift++;
    PendingSum in{base, partials, pending_bias, n_partials, n_tokens};
    dim3 grid(n_heads, n_tokens);
#define MLLM_HALF_CASE(HD)                                                                                              \
    case HD:                                                                                                            \
        decode_attention_half_kernel<HD><<<grid, DL_THREADS, 0, stream>>>(                                              \
            in, summed, gamma, beta, eps, (const bf16_t*)w_qkv, b_qkv, (const bf16_t*)w_out, (bf16_t*)k_pages,          \
            (bf16_t*)v_pages, slots, token_request, positions, block_tables, max_blocks, partial_out, n_tokens, width,  \
            n_heads, n_kv_heads, page_shift, window, scale, write_cache);                                               \
        break;
    switch (head_size) {
        MLLM_HALF_CASE(16)
        MLLM_HALF_CASE(32)
        MLLM_HALF_CASE(64)
        MLLM_HALF_CASE(128)
        MLLM_HALF_CASE(256)
    }
#undef MLLM_HALF_CASE
    return mllm_check_launch("decode_attention_half");
}

MLLM_API int mllm_decode_mlp_half(const float* base, const float* partials, const float* pending_bias, int n_partials,
                                  float* summed, const float* gamma, const float* beta, float eps, const void* w_up,
                                  const float* b_up, const void* w_down, float* partial_out, int n_tokens, int width,
                                  int inner, int slice_units, int epilogue, hipStream_t stream) {
    if (check_pending("decode_mlp_half", base, partials, n_partials, width)) return 1;
    MLLM_REQUIRE(n_tokens >= 0 && n_tokens <= 65535 * DL_TOKENS, "decode_mlp_half: %d tokens", n_tokens);
    MLLM_REQUIRE(inner >= 8 && inner % 8 == 0, "decode_mlp_half: %d hidden units is not a multiple of 8", inner);
    MLLM_REQUIRE(slice_units == 64 || slice_units == 128, "decode_mlp_half: slices of %d hidden units; 64 or 128", slice_units);
    MLLM_REQUIRE(epilogue >= 0 && epilogue <= 2, "decode_mlp_half: unknown epilogue %d", epilogue);
    if (n_tokens == 0) return 0;
    PendingSum in{base, partials, pending_bias, n_partials, n_tokens};
    const int pieces_per_lane = (width / 4 + WAVE - 1) / WAVE;
    const bf16_t* up = (const bf16_t*)w_up;
    const bf16_t* down = (const bf16_t*)w_down;
    int refused = 0;
#define MLLM_MLP_CASE(NV)                                                                                                     \
    (slice_units == 64 ? launch_mlp_half<NV, 64>(in, summed, gamma, beta, eps, up, b_up, down, partial_out, n_tokens, width, \
                                                 inner, epilogue, stream)                                                    \
                       : launch_mlp_half<NV, 128>(in, summed, gamma, beta, eps, up, b_up, down, partial_out, n_tokens, width, \
                                                  inner, epilogue, stream))
    if (pieces_per_lane <= 2) refused = MLLM_MLP_CASE(2);
    else if (pieces_per_lane <= 3) refused = MLLM_MLP_CASE(3);
    else if (pieces_per_lane <= 4) refused = MLLM_MLP_CASE(4);
    else if (pieces_per_lane <= 6) refused = MLLM_MLP_CASE(6);
    else refused = MLLM_MLP_CASE(8);
#undef MLLM_MLP_CASE
    if (refused) return 1;
    return mllm_check_launch("decode_mlp_half");
}

MLLM_API int mllm_pending_sum(const float* base, const float* partials, const float* pending_bias, int n_partials,
                              float* out, int n_rows, int width, hipStream_t stream) {
    MLLM_REQUIRE(base != nullptr && out != nullptr, "pending_sum: no rows");
    MLLM_REQUIRE(n_partials >= 0 && (n_partials == 0 || partials != nullptr), "pending_sum: %d partial rows without memory", n_partials);
    MLLM_REQUIRE(width > 0 && width % 4 == 0, "pending_sum: width %d is not a multiple of 4", width);
    MLLM_REQUIRE(n_rows >= 0 && n_rows <= 65535, "pending_sum: %d rows", n_rows);
    if (n_rows == 0) return 0;
    PendingSum in{base, partials, pending_bias, n_partials, n_rows};
    dim3 grid((width / 4 + 255) / 256, n_rows);
    pending_sum_kernel<<<grid, 256, 0, stream>>>(in, out, width);
    return mllm_check_launch("pending_sum");
}

#ifdef MLLM_PHASE_STAMPS
MLLM_API int mllm_phase_stamps(long long* out) { return hipMemcpyFromSymbol(out, HIP_SYMBOL(dl_stamps), sizeof(long long) * 32) == hipSuccess ? 0 : 1; }
#endif
