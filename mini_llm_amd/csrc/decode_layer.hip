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
// straight into registers (the matrices are in the packed layout: a wave's operand is 1 KiB of
// contiguous memory), and the activations, which are tiny, as the other operand from LDS.
#include "common.h"
#include "key_sweep.h"

namespace {

constexpr int DL_WAVES = 16;
constexpr int DL_THREADS = DL_WAVES * WAVE;
constexpr int DL_MAX_WIDTH = 2048;  // a row's 4-column pieces: at most 2 per thread of a block, 8 per lane of a wave
constexpr int DL_KSPLIT = 4;        // waves that share the k range of one 16-row tile
constexpr int DL_TOKENS = 16;       // tokens a feed-forward block takes: the matrix core's other 16

struct PendingSum {
    const float* base;      // [rows, width]
    const float* partials;  // [n_partials, rows, width]
    const float* bias;      // [width] or null, added once
    int n_partials;
    int rows;
};

__device__ __forceinline__ f32x4 load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }

// 16 bytes at base + byte_offset, where base is the same in every lane (it then lives in scalar
// registers) and only the 32-bit offset differs: the address costs a lane one register, not two.
template <typename V>
__device__ __forceinline__ V load16(const void* uniform_base, unsigned byte_offset) {
    return *reinterpret_cast<const V*>(reinterpret_cast<const char*>(uniform_base) + byte_offset);
}

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

// The compiler moves loads up as far as it can, across loads the code asks for earlier on purpose,
// and then runs out of registers: this keeps what is above it above and what is below it below.
__device__ __forceinline__ void keep_order() { __builtin_amdgcn_sched_barrier(0); }

// The block's waves meet once this wave's LDS traffic is done: what __syncthreads() comes to on
// this target, spelled out because the kernels below count on it. It does not wait for this wave's
// loads from memory, so what was asked for early stays in flight across it; and only LDS carries
// data between the waves of a block here, so nothing more is needed.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// A wave's share of the q/k/v product of one (token, head): 3*HD rows of the matrix in tiles of 16,
// each tile's k range cut into DL_KSPLIT shares; a (tile, share) pair is a unit. The wave owns the
// units first_unit, first_unit + 8, ... (n_units of them), works on AT_ONCE at a time and keeps
// ROUND k steps of each in flight. The shares' sums meet in LDS (qkv_part).
template <int HD, int AT_ONCE>
struct QkvShare {
    static constexpr int ROW_TILES = 3 * HD / 16, ALL_UNITS = ROW_TILES * DL_KSPLIT, ROUND = 6;
    const bf16_t* w_qkv;
    int head, kv_head, q_width, kv_width, n_steps, lane, first_unit;
    int w_at[AT_ONCE], part_of[AT_ONCE], tile_of[AT_ONCE];
    Vec16 w_piece[AT_ONCE][ROUND];

    __device__ __forceinline__ void choose(int u0) {
#pragma unroll
        for (int u = 0; u < AT_ONCE; u++) {
            int unit = min(first_unit + 8 * (u0 + u), ALL_UNITS - 1);  // beyond the last: computed again, not kept
            tile_of[u] = unit % ROW_TILES, part_of[u] = unit / ROW_TILES;
            int local = tile_of[u] * 16, which = local / HD, within = local % HD;  // HD is a multiple of 16: a tile lies in one of q, k, v
            int w_row = which == 0 ? head * HD + within : q_width + (which - 1) * kv_width + kv_head * HD + within;
            w_at[u] = w_row / 16;
        }
    }
    __device__ __forceinline__ void ask(int i0) {
#pragma unroll
        for (int u = 0; u < AT_ONCE; u++)
#pragma unroll
            for (int j = 0; j < ROUND; j++) {
                int step = min(part_of[u] + DL_KSPLIT * (i0 + j), n_steps - 1);
                w_piece[u][j] = load16<Vec16>(w_qkv + packed_offset<bf16_t>(w_at[u], step, n_steps, 0), lane * 16);
            }
    }
    // All N_UNITS units; `asked`: choose(0) and ask(0) have been called already (the first round has
    // been under way for a while). x_hat: the normed row in LDS, zeros beyond the width.
    template <int N_UNITS>
    __device__ __forceinline__ void run(bool asked, const bf16_t* x_hat, float (*qkv_part)[3 * HD]) {
        const int row16 = lane % 16, quad = lane / 16;
        const int steps_per_unit = (n_steps + DL_KSPLIT - 1) / DL_KSPLIT;
#pragma unroll 1
        for (int u0 = 0; u0 < N_UNITS; u0 += AT_ONCE) {
            f32x4 acc[AT_ONCE];
#pragma unroll
            for (int u = 0; u < AT_ONCE; u++) acc[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (u0 > 0 || !asked) choose(u0);
#pragma unroll 1
            for (int i0 = 0; i0 < steps_per_unit; i0 += ROUND) {
                if (u0 > 0 || i0 > 0 || !asked) ask(i0);
#pragma unroll
                for (int u = 0; u < AT_ONCE; u++)
#pragma unroll
                    for (int j = 0; j < ROUND; j++) {
                        int step = part_of[u] + DL_KSPLIT * (i0 + j);
                        Vec16 w = mask16(w_piece[u][j], step < n_steps);
                        bf16x8 x = *reinterpret_cast<const bf16x8*>(x_hat + min(step, n_steps - 1) * 32 + quad * 8);
                        acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&w), x, acc[u], 0, 0, 0);
                    }
            }
            // every column of the product is this one token; column 0 is kept
#pragma unroll
            for (int u = 0; u < AT_ONCE; u++)
                if (row16 == 0 && first_unit + 8 * (u0 + u) < ALL_UNITS) {
#pragma unroll
                    for (int r = 0; r < 4; r++) qkv_part[part_of[u]][tile_of[u] * 16 + 4 * quad + r] = acc[u][r];
                }
        }
    }
};

// ------------------------------------------------------------------------------------------------
// norm -> q/k/v -> cache write -> attention over the cache -> this head's share of the output
// product. grid (n_heads, tokens), 1024 threads in two roles:
//   waves 0..7  "project": norm, q/k/v product, output product;
//   waves 8..15 "attend":  the pending sums, then their shares of the cached keys and values, asked
//                          for long before the query exists, then the softmax over them.
// A wave's loads from memory complete in the order they were issued, and every trip to memory
// costs microseconds: so each role asks early, in the order of use, for all it will need, and the
// roles are split so that no wave has to wait for the keys before it can use something else.
// What the waves exchange goes through LDS, between meetings that both roles pass in step.
// ------------------------------------------------------------------------------------------------
constexpr int DL_PROJECT_WAVES = 8, DL_ATTEND_WAVES = DL_WAVES - DL_PROJECT_WAVES;
constexpr int DL_PROJECT_THREADS = DL_PROJECT_WAVES * WAVE;

template <int HD>
__global__ __launch_bounds__(DL_THREADS) void decode_attention_half_kernel(
    PendingSum in, float* __restrict__ summed,  // [tokens, width]: the stream with its sums taken, written by head 0
    const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
    const bf16_t* __restrict__ w_qkv, const float* __restrict__ b_qkv,  // [q_width + 2 kv_width, width], packed
    const bf16_t* __restrict__ w_out,                                    // [width, q_width], packed
    bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, const int* __restrict__ slots,
    const int* __restrict__ token_request, const int* __restrict__ positions,
    const int* __restrict__ block_tables, int max_blocks,
    float* __restrict__ partial_out,  // [n_heads, tokens, width]
    int n_tokens, int width, int n_heads, int n_kv_heads, int page_shift, int window, float scale, int write_cache) {
    typedef KeySweep<bf16_t, HD> Sweep;
    constexpr int VEC = Sweep::VEC, LPR = Sweep::LPR, RPI = Sweep::RPI, KPI = Sweep::KPI;
    constexpr int ROW_TILES = 3 * HD / 16;
    // the q/k/v product: two thirds of its units go to the waves that project, one third to the
    // waves that attend (which have nothing else to do while they wait for the query)
    constexpr int ALL_UNITS = ROW_TILES * DL_KSPLIT;
    constexpr int UNITS_PROJECT = (2 * ALL_UNITS / 3 + 7) / 8, UNITS_ATTEND = (ALL_UNITS - 8 * UNITS_PROJECT + 7) / 8;
    constexpr int AT_ONCE_PROJECT = UNITS_PROJECT < 2 ? UNITS_PROJECT : 2, AT_ONCE_ATTEND = UNITS_ATTEND < 2 ? UNITS_ATTEND : 2;
    static_assert(UNITS_ATTEND >= 1 && 8 * (UNITS_PROJECT + UNITS_ATTEND) >= ALL_UNITS, "every unit of the q/k/v product has a wave");
    constexpr int HD_PAD = (HD + 31) / 32 * 32;
    constexpr int OUT_STEPS = HD_PAD / 32, OUT_GROUP = OUT_STEPS <= 2 ? 12 / OUT_STEPS : (OUT_STEPS <= 4 ? 2 : 1);
    constexpr int ROWS_PER_THREAD = (3 * HD + DL_PROJECT_THREADS - 1) / DL_PROJECT_THREADS;
    constexpr int MAX_PIECES = DL_MAX_WIDTH / 4, PIECES_PER_LANE = MAX_PIECES / WAVE;
    constexpr int NEAR_KEYS = DL_ATTEND_WAVES * KPI;  // keys the waves that attend can ask for in one go
    // a wave leaves one (max, sum, output) triple for each of its rows of 16 lanes (for each group
    // of lanes, if a group is wider): adding them up in LDS is cheaper than across the rows of a wave
    constexpr int MERGE_SPAN = LPR < 16 ? 16 : LPR, MERGE_ENTRIES = WAVE / MERGE_SPAN;

    __shared__ f32x4 stage[DL_ATTEND_WAVES][MAX_PIECES];
    __shared__ f32x4 row_lds[MAX_PIECES];
    __shared__ __attribute__((aligned(16))) bf16_t x_hat[DL_MAX_WIDTH];
    __shared__ float qkv_part[DL_KSPLIT][3 * HD];
    __shared__ float qkv_row[3][HD];  // q, k, v of this token and head, rounded as the cache holds them
    __shared__ float merged[DL_WAVES * MERGE_ENTRIES][HD + 2];
    __shared__ float merge_weight[HD_PAD / WAVE > 0 ? HD_PAD / WAVE : 1][WAVE];
    __shared__ __attribute__((aligned(16))) bf16_t mixed[HD_PAD];

    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);  // the same in every lane: kept in a scalar register
    const bool attends = wave >= DL_PROJECT_WAVES;
    const int role_wave = attends ? wave - DL_PROJECT_WAVES : wave;
    const int head = blockIdx.x, token = blockIdx.y;
    const int n_pieces = width / 4;
    float* out_row = partial_out + ((size_t)head * n_tokens + token) * width;
    const int request = token_request[token];
    const int position = positions[token];
    const int slot = slots[token];
    // A padding row (request < 0) leaves zeros, so that what follows stays finite. Each role finds
    // that out only after it has asked for what does not depend on the request: the wait for the
    // request then costs nothing. No wave has met another by then, and all of them leave.
    auto leave_zeros = [&]() {
        for (int c = tid; c < width; c += DL_THREADS) {
            out_row[c] = 0.0f;
            if (head == 0) summed[(size_t)token * width + c] = 0.0f;
        }
    };
    const int kv_head = head / (n_heads / n_kv_heads);
    const int q_width = n_heads * HD, kv_width = n_kv_heads * HD;
    const int row16 = lane % 16, quad = lane / 16;
    const int sub = lane % LPR;

    // The cached keys first_key .. position-1: the first NEAR_KEYS of them are shared by the waves
    // that attend, KPI or fewer each, asked for in one go; what a long context has beyond them is
    // shared by the waves that project, which ask when the q/k/v product has given their registers
    // back. A wave without keys asks for the token's own slot instead: a page the table holds,
    // memory that may not be written yet, never counted. (Worked out by each role after its first
    // loads are under way: it is the first use of the position and would wait for it.)
    int n_far, begin, end, spare_key;
    const int* table;
    auto share_of_keys = [&]() {
        const int first_key = window > 0 ? max(0, position - window + 1) : 0;
        const int n_cached = position - first_key;
        const int n_near = min(n_cached, NEAR_KEYS);
        n_far = n_cached - n_near;
        const int chunk = attends ? (((n_near + DL_ATTEND_WAVES - 1) / DL_ATTEND_WAVES + RPI - 1) / RPI) * RPI
                                  : (((n_far + DL_PROJECT_WAVES - 1) / DL_PROJECT_WAVES + RPI - 1) / RPI) * RPI;
        const int share_first = attends ? first_key : first_key + n_near, share_end = attends ? first_key + n_near : position;
        begin = share_first + role_wave * chunk;
        end = min(share_end, begin + chunk);
        spare_key = begin < end ? end - 1 : position;
        table = block_tables + (size_t)request * max_blocks;
    };
    Sweep sweep;

    if (attends) {
        // ---- the pending sums of this token's row: wave a takes the partial rows a, a + 8, ..., a
        // lane the pieces lane, lane + 64, ...; the eight sums meet in LDS
        {
            const int pieces_here = (n_pieces + WAVE - 1) / WAVE;  // pieces a lane has: 3 for a width of 768
            for (int j0 = 0; j0 < pieces_here; j0 += 3) {          // three at a time, six partial rows of each in flight
                f32x4 sum[3];
#pragma unroll
                for (int j = 0; j < 3; j++) sum[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                for (int s0 = role_wave; s0 < in.n_partials; s0 += DL_ATTEND_WAVES * 6) {
                    f32x4 part[6][3];
#pragma unroll
                    for (int u = 0; u < 6; u++) {
                        const int s = __builtin_amdgcn_readfirstlane(min(s0 + DL_ATTEND_WAVES * u, in.n_partials - 1));
                        const float* partial_row = in.partials + ((size_t)s * in.rows + token) * width;
#pragma unroll
                        for (int j = 0; j < 3; j++) part[u][j] = load16<f32x4>(partial_row, 16 * min(lane + WAVE * (j0 + j), n_pieces - 1));
                    }
#pragma unroll
                    for (int u = 0; u < 6; u++) {
                        const float counts = s0 + DL_ATTEND_WAVES * u < in.n_partials ? 1.0f : 0.0f;  // times zero, not a branch
#pragma unroll
                        for (int j = 0; j < 3; j++) sum[j] += part[u][j] * counts;
                    }
                }
#pragma unroll
                for (int j = 0; j < 3; j++)
                    if (lane + WAVE * (j0 + j) < n_pieces) stage[role_wave][lane + WAVE * (j0 + j)] = sum[j];
            }
        }
        if (request < 0) {
            leave_zeros();
            return;
        }
        share_of_keys();
        int key_page[Sweep::UNROLL];
        sweep.look_up(key_page, table, page_shift, begin, end, spare_key, lane);  // the table's answer is under way early
        lds_barrier();  // 1: the eight sums are in LDS
        lds_barrier();  // 2
        lds_barrier();  // 3: the normed row is in LDS
        // ---- their share of the q/k/v product (measured: asking for the matrix before the meetings
        // above, or for the keys before the matrix, only delays the other waves or costs registers)
        QkvShare<HD, AT_ONCE_ATTEND> qkv{w_qkv, head, kv_head, q_width, kv_width, (width + 31) / 32, lane, 8 * UNITS_PROJECT + role_wave};
        qkv.template run<UNITS_ATTEND>(false, x_hat, qkv_part);
        // ---- their shares of the cached keys and values, asked for now (the pages are known by
        // now); they ask for nothing else until they have used them
        keep_order();
        typename Sweep::Fetched fetched;
        sweep.fetch_rows(fetched, key_page, k_pages, v_pages, kv_head, n_kv_heads, page_shift, begin, end, spare_key, lane);
        lds_barrier();  // 4
        lds_barrier();  // 5: q, k, v of this token are in LDS
        float qf[VEC];
        bf16x8 q_stored;  // the query as a kernel of its own would have stored it: the cached keys meet it in pairs
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            qf[i] = qkv_row[0][sub * VEC + i] * scale;
            q_stored[i] = static_cast<bf16_t>(qkv_row[0][sub * VEC + i]);
        }
        sweep.init();
        // not under a condition (a wave without keys counts none): the compiler would move the loads
        // above down into a conditional block, behind the meetings of the waves
        sweep.template consume<true>(fetched, q_stored, scale, begin, end, lane);
        if (wave == DL_PROJECT_WAVES) sweep.one_key(qf, qkv_row[1], qkv_row[2], lane);  // the token's own key and value, from LDS
        sweep.merge_inside_rows();
        {
            const int entry = wave * MERGE_ENTRIES + lane / MERGE_SPAN;
            if (lane % MERGE_SPAN < LPR) {
#pragma unroll
                for (int i = 0; i < VEC; i++) merged[entry][sub * VEC + i] = sweep.o[i];
            }
            if (lane % MERGE_SPAN == 0) {
                merged[entry][HD] = sweep.running_max;
                merged[entry][HD + 1] = sweep.running_sum;
            }
        }
        lds_barrier();  // 6: every wave's (max, sum, output) is in LDS
        lds_barrier();  // 7
        return;
    }

    // ---- the waves that project: what they need of the vectors, and the first round of the
    // q/k/v matrix, in one trip to memory
    const bool owns = tid < n_pieces;  // threads 0 .. width/4-1 own four columns of the row each
    const int own_piece = min(tid, n_pieces - 1);
    f32x4 row = load4(in.base + (size_t)token * width + 4 * own_piece);
    const f32x4 pending_bias = load4((in.bias ? in.bias : gamma) + 4 * own_piece);  // a vector that is there stands in for one that is not
    const f32x4 gain = load4(gamma + 4 * own_piece), offset = load4(beta + 4 * own_piece);
    float qkv_bias[ROWS_PER_THREAD];
#pragma unroll
    for (int i = 0; i < ROWS_PER_THREAD; i++) {
        int r = min(tid + DL_PROJECT_THREADS * i, 3 * HD - 1), which = r / HD, within = r % HD;
        int w_row = which == 0 ? head * HD + within : q_width + (which - 1) * kv_width + kv_head * HD + within;
        qkv_bias[i] = (b_qkv ? b_qkv : gamma)[b_qkv ? w_row : 0];
    }
    QkvShare<HD, AT_ONCE_PROJECT> qkv{w_qkv, head, kv_head, q_width, kv_width, (width + 31) / 32, lane, wave};
    qkv.choose(0);
    qkv.ask(0);
    if (request < 0) {
        leave_zeros();
        return;
    }
    share_of_keys();
    lds_barrier();  // 1: the eight sums of the partial rows are in LDS
    // width / 4 <= 512: the threads of these waves cover the row
    row += pending_bias * (in.bias ? 1.0f : 0.0f);
    if (owns) {
        row += ((stage[0][tid] + stage[1][tid]) + (stage[2][tid] + stage[3][tid])) + ((stage[4][tid] + stage[5][tid]) + (stage[6][tid] + stage[7][tid]));
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
        // the row is read from LDS twice rather than kept: the registers are full of the matrix
        const int pieces_here = (n_pieces + WAVE - 1) / WAVE;
        float sum = 0.0f;
#pragma unroll 2
        for (int j = 0; j < pieces_here; j++) {
            f32x4 piece = row_lds[lane + WAVE * j];  // zeros beyond the width
            sum += (piece[0] + piece[1]) + (piece[2] + piece[3]);
        }
        const float mean = wave_total(sum) / n;
        float squares = 0.0f;
#pragma unroll 2
        for (int j = 0; j < pieces_here; j++) {
            f32x4 d = lane + WAVE * j < n_pieces ? row_lds[lane + WAVE * j] - mean : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            squares += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
        }
        const float inverse_stddev = 1.0f / sqrtf(wave_total(squares) / n + eps);
        f32x4 y = (row - mean) * inverse_stddev * gain + offset;
        if (!owns) y = f32x4{0.0f, 0.0f, 0.0f, 0.0f};  // beyond the width: zeros, the products read whole 32-column steps
        store_bf16x4(x_hat + 4 * tid, y);
    }
    lds_barrier();  // 3: the normed row is in LDS
    int far_page[Sweep::UNROLL];  // the pages of this wave's share of the far keys (of the spare key, if there are none)
    sweep.look_up(far_page, table, page_shift, begin, end, spare_key, lane);

    qkv.template run<UNITS_PROJECT>(true, x_hat, qkv_part);
    auto finish_qkv_rows = [&]() {  // sums of the k shares, bias, rounding; k and v go into their cache slot
#pragma unroll
        for (int i = 0; i < ROWS_PER_THREAD; i++) {
            const int r = tid + DL_PROJECT_THREADS * i;
            if (r < 3 * HD) {
                const int which = r / HD, within = r % HD;
                float value = ((qkv_part[0][r] + qkv_part[1][r]) + qkv_part[2][r]) + qkv_part[3][r] + (b_qkv ? qkv_bias[i] : 0.0f);
                bf16_t kept = static_cast<bf16_t>(value);
                qkv_row[which][within] = static_cast<float>(kept);
                if (which > 0 && write_cache && slot >= 0 && head % (n_heads / n_kv_heads) == 0) {
                    int page = slot >> page_shift, at = slot & ((1 << page_shift) - 1);
                    bf16_t* pages = which == 1 ? k_pages : v_pages;
                    pages[((((size_t)page * n_kv_heads + kv_head) << page_shift) + at) * HD + within] = kept;
                }
            }
        }
    };
    if (n_far > 0) {  // a long context (the same for the whole block): these waves attend to their shares of the far keys
        typename Sweep::Fetched fetched;
        sweep.fetch_rows(fetched, far_page, k_pages, v_pages, kv_head, n_kv_heads, page_shift, begin, end, spare_key, lane);
        lds_barrier();  // 4: the shares of the q/k/v product are in LDS
        finish_qkv_rows();
        lds_barrier();  // 5: q, k, v of this token are in LDS
        bf16x8 q_stored;
#pragma unroll
        for (int i = 0; i < VEC; i++) q_stored[i] = static_cast<bf16_t>(qkv_row[0][sub * VEC + i]);
        sweep.init();
        sweep.template consume<true>(fetched, q_stored, scale, begin, end, lane);  // not under a further condition, as above
        if (begin + KPI < end)  // a context longer than one round of every wave of the block covers
            sweep.keys(q_stored, scale, k_pages, v_pages, table, kv_head, n_kv_heads, page_shift, begin + KPI, end, lane);
        sweep.merge_inside_rows();
    } else {
        lds_barrier();  // 4
        finish_qkv_rows();
        lds_barrier();  // 5
        sweep.init();
    }
    {
        const int entry = wave * MERGE_ENTRIES + lane / MERGE_SPAN;
        if (lane % MERGE_SPAN < LPR) {
#pragma unroll
            for (int i = 0; i < VEC; i++) merged[entry][sub * VEC + i] = sweep.o[i];
        }
        if (lane % MERGE_SPAN == 0) {
            merged[entry][HD] = sweep.running_max;
            merged[entry][HD + 1] = sweep.running_sum;
        }
    }
    // the output product's rows are asked for now: they are needed last
    keep_order();
    // w_out [width, q_width]: this head's columns start in chunk out_step0, at column out_shift of
    // it (not 0 only for heads of 16, two of which share a chunk of 32 columns)
    const int out_tiles = (width + 15) / 16, out_k_steps = packed_k_steps<bf16_t>(q_width);
    const int out_step0 = head * HD / 32, out_shift = head * HD % 32;
    Vec16 out_piece[OUT_GROUP][OUT_STEPS];
#pragma unroll
    for (int g = 0; g < OUT_GROUP; g++) {
        int out_tile = min(wave + DL_PROJECT_WAVES * g, out_tiles - 1);
#pragma unroll
        for (int s = 0; s < OUT_STEPS; s++)
            out_piece[g][s] = load16<Vec16>(w_out + packed_offset<bf16_t>(out_tile, out_step0 + s, out_k_steps, 0), lane * 16);
    }
    lds_barrier();  // 6: every wave's (max, sum, output) is in LDS
    if (wave < (HD_PAD + WAVE - 1) / WAVE) {  // whole waves (the wave sums below need every lane); the mixed row lies where its columns lie in the chunks of w_out, zeros around it
        // out = sum_s o_s e^(m_s - M) / sum_s l_s e^(m_s - M) over the triples s (one without keys has
        // m = -inf, l = 0). Each wave works the weights out once, a lane a triple, and keeps them in
        // LDS for itself.
        constexpr int N_TRIPLES = DL_WAVES * MERGE_ENTRIES;
        static_assert(N_TRIPLES <= WAVE, "a lane a triple");
        const float triple_max = lane < N_TRIPLES ? merged[min(lane, N_TRIPLES - 1)][HD] : -INFINITY;
        const float triple_sum = lane < N_TRIPLES ? merged[min(lane, N_TRIPLES - 1)][HD + 1] : 0.0f;
        const float weight = expf(triple_max - wave_max_total(triple_max));
        const float total = wave_total(triple_sum * weight);
        merge_weight[wave][lane] = weight / total;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's own writes, read back below
        float value = 0.0f;
        const int d = tid - out_shift;
        if (d >= 0 && d < HD) {
#pragma unroll 8
            for (int s = 0; s < N_TRIPLES; s++) value += merged[s][d] * merge_weight[wave][s];
        }
        if (tid < HD_PAD) mixed[tid] = static_cast<bf16_t>(value);
    }
    lds_barrier();  // 7: the mixed row of this head is in LDS

    // this head's share of the output product: rows of w_out in tiles of 16, columns head*HD ..
    for (int tile0 = wave; tile0 < out_tiles; tile0 += DL_PROJECT_WAVES * OUT_GROUP) {
        if (tile0 != wave) {  // wider than the rows asked for above cover
#pragma unroll
            for (int g = 0; g < OUT_GROUP; g++) {
                int out_tile = min(tile0 + DL_PROJECT_WAVES * g, out_tiles - 1);
#pragma unroll
                for (int s = 0; s < OUT_STEPS; s++)
                    out_piece[g][s] = load16<Vec16>(w_out + packed_offset<bf16_t>(out_tile, out_step0 + s, out_k_steps, 0), lane * 16);
            }
        }
#pragma unroll
        for (int g = 0; g < OUT_GROUP; g++) {
            int tile = tile0 + DL_PROJECT_WAVES * g;
            f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < OUT_STEPS; s++) {
                bf16x8 x = *reinterpret_cast<const bf16x8*>(mixed + s * 32 + quad * 8);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&out_piece[g][s]), x, acc, 0, 0, 0);
            }
            int out_col = tile * 16 + 4 * quad;  // 4 columns; the width is a multiple of 4
            if (row16 == 0 && out_col < width) *reinterpret_cast<f32x4*>(out_row + out_col) = acc;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// norm -> up product -> activation -> this slice's share of the down product.
// grid (slices of U hidden units, groups of 1 to 16 tokens), 1024 threads. The partial rows are asked
// for first and the first pieces of both matrices right behind them; while the matrices come, the
// waves take the pending sums (16 / tokens waves a token, every so-manieth partial row each) and the
// norm; then all waves run the two products.
// ------------------------------------------------------------------------------------------------
template <int NV, int U>
__global__ __launch_bounds__(DL_THREADS) void decode_mlp_half_kernel(
    PendingSum in, float* __restrict__ summed, const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
    const bf16_t* __restrict__ w_up, const float* __restrict__ b_up,  // [inner, width], packed
    const bf16_t* __restrict__ w_down,                                 // [width, inner], packed
    float* __restrict__ partial_out,                                   // [slices, tokens, width]
    int n_tokens, int width, int inner, int epilogue, int stage_pieces, int tokens_per_block) {
    constexpr int TILES = U / 16, K_STEPS_DOWN = U / 32, H_STRIDE = U + 8;
    constexpr int UP_UNITS = (TILES * DL_KSPLIT + DL_WAVES - 1) / DL_WAVES;  // (tile, k share) pairs a wave owns
    constexpr int UP_ROUND = 6 / UP_UNITS;                                   // k steps of each in flight together
    constexpr int DOWN_GROUP = 6 / K_STEPS_DOWN;                             // output tiles a wave works on at a time
    constexpr int ROWS_AT_ONCE = NV <= 3 ? 3 : (NV <= 4 ? 2 : 1);                            // partial rows asked for before any is added
    constexpr int BIAS_PER_THREAD = (TILES * 256 + DL_THREADS - 1) / DL_THREADS;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int x_stride = (width + 31) / 32 * 32 + 8;  // 16 bytes of padding: the 16 rows fall on different banks
    bf16_t* x_hat = reinterpret_cast<bf16_t*>(lds);                                          // [16][x_stride]
    float* up_part = reinterpret_cast<float*>(lds + (size_t)DL_TOKENS * x_stride * 2);        // [KSPLIT][TILES][4][64]
    bf16_t* hidden = reinterpret_cast<bf16_t*>(up_part + DL_KSPLIT * TILES * 256);            // [16][H_STRIDE]
    f32x4* stage = reinterpret_cast<f32x4*>(hidden + DL_TOKENS * H_STRIDE);                   // [16 waves][stage_pieces]

    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int slice = blockIdx.x, token0 = blockIdx.y * tokens_per_block;
    const int n_pieces = width / 4;
    const int row16 = lane % 16, quad = lane / 16;
    const int n_steps = (width + 31) / 32;
    const int steps_per_unit = (n_steps + DL_KSPLIT - 1) / DL_KSPLIT;

    // ---- the pending sums and the norm. With T tokens in this block (rounded up to a power of
    // two), wave w works for token w % T and takes the partial rows w / T, w / T + 16 / T, ...
    // A wave's loads complete in the order they were issued: the first partial rows are asked for
    // first, then the first pieces of both matrices, which stay in flight through all that follows
    // until the products need them.
    const int tokens_here = min(tokens_per_block, n_tokens - token0);
    int t2 = 1;
    while (t2 < tokens_here) t2 *= 2;
    if (stage_pieces < n_pieces) t2 = DL_TOKENS;  // no room to share a token's sums among waves
    const int waves_per_token = __builtin_amdgcn_readfirstlane(DL_WAVES >> (31 - __builtin_clz(t2)));
    // t2 is a power of two; the scalar unit has no division, and a quotient computed by the vector
    // unit would drag every address below into vector registers
    const int local = wave & (t2 - 1), sub = __builtin_amdgcn_readfirstlane(wave >> (31 - __builtin_clz(t2)));
    const int token = token0 + local;
    const bool live = token < n_tokens;
    const int safe_token = live ? token : n_tokens - 1;
    // all of a round's loads are asked for before any is used, with no branch between them; the
    // bias comes from a row of zeros' worth of the base if there is none (and is then not added)
    f32x4 row[NV], bias_piece[NV];
    const float* base_row = in.base + (size_t)safe_token * width;
    const float* bias_row = in.bias ? in.bias : base_row;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        int piece = min(lane + WAVE * j, n_pieces - 1);
        row[j] = load16<f32x4>(base_row, 16 * piece);
        bias_piece[j] = load16<f32x4>(bias_row, 16 * piece);
    }
    f32x4 part[ROWS_AT_ONCE][NV];
    auto ask_for_partial_rows = [&](int s0) {
#pragma unroll
        for (int u = 0; u < ROWS_AT_ONCE; u++) {
            int s = max(0, min(s0 + waves_per_token * u, in.n_partials - 1));
            // the row's address is the same in every lane (a scalar), the lanes differ by a 32-bit offset
            const int partial_index = __builtin_amdgcn_readfirstlane(s * in.rows + safe_token);  // partial rows number fewer than 2^31
            const float* partial_row = (in.n_partials ? in.partials : in.base) + (size_t)partial_index * width;
#pragma unroll
            for (int j = 0; j < NV; j++) part[u][j] = load16<f32x4>(partial_row, 16 * min(lane + WAVE * j, n_pieces - 1));
        }
    };
    auto add_partial_rows = [&](int s0) {
#pragma unroll
        for (int u = 0; u < ROWS_AT_ONCE; u++) {
            // a row that does not count was asked for again (a finite one): times zero, not a branch,
            // which would make the compiler wait for every load under way
            const float counts = s0 + waves_per_token * u < in.n_partials ? 1.0f : 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++) row[j] += part[u][j] * counts;
        }
    };
    const int round_stride = waves_per_token * ROWS_AT_ONCE;
    ask_for_partial_rows(sub);
    const float bias_counts = in.bias ? 1.0f : 0.0f, base_counts = sub == 0 ? 1.0f : 0.0f;
#pragma unroll
    for (int j = 0; j < NV; j++) row[j] = (row[j] + bias_piece[j] * bias_counts) * base_counts;
    // the up matrix: behind the partial rows in the order of the loads, so that the sums do not wait for it
    int up_at[UP_UNITS], up_part_of[UP_UNITS], up_tile[UP_UNITS];
    Vec16 up_piece[UP_UNITS][UP_ROUND];
    float up_bias[BIAS_PER_THREAD];
    auto ask_for_up_matrix = [&]() {
#pragma unroll
        for (int u = 0; u < UP_UNITS; u++) {
            int unit = min(wave + DL_WAVES * u, TILES * DL_KSPLIT - 1);
            up_tile[u] = unit % TILES, up_part_of[u] = unit / TILES;
            up_at[u] = min(slice * (U / 16) + up_tile[u], (inner + 15) / 16 - 1);  // row tile of w_up; beyond the last: zeros come out below
#pragma unroll
            for (int j = 0; j < UP_ROUND; j++)
                up_piece[u][j] = load16<Vec16>(w_up + packed_offset<bf16_t>(up_at[u], min(up_part_of[u] + DL_KSPLIT * j, n_steps - 1), n_steps, 0), lane * 16);
        }
        // and the bias of the hidden units this thread will finish, while nothing waits for it
#pragma unroll
        for (int i = 0; i < BIAS_PER_THREAD; i++) {
            const int index = tid + DL_THREADS * i, tile = index / 256, r = (index / WAVE) % 4, l = index % WAVE;
            const int h = slice * U + tile * 16 + 4 * (l / 16) + r;
            up_bias[i] = (b_up ? b_up : gamma)[b_up && h < inner ? h : 0];
        }
    };
    if (sub + round_stride >= in.n_partials) {  // one round of partial rows: the same for the whole wave
        ask_for_up_matrix();
        add_partial_rows(sub);
    } else {
        add_partial_rows(sub);
        keep_order();
        ask_for_partial_rows(sub + round_stride);
        ask_for_up_matrix();
        add_partial_rows(sub + round_stride);
        for (int s0 = sub + 2 * round_stride; s0 < in.n_partials; s0 += round_stride) {  // many partial rows and few waves a token
            ask_for_partial_rows(s0);
            add_partial_rows(s0);
        }
    }
    // the down matrix is needed last: asked for now, it has the norm and the up product to arrive in
    keep_order();
    const int down_tiles = (width + 15) / 16, down_k_steps = packed_k_steps<bf16_t>(inner);
    Vec16 down_piece[DOWN_GROUP][K_STEPS_DOWN];
#pragma unroll
    for (int g = 0; g < DOWN_GROUP; g++) {
        int out_tile = min(wave + DL_WAVES * g, down_tiles - 1);
#pragma unroll
        for (int s = 0; s < K_STEPS_DOWN; s++)  // chunks beyond the hidden units: read again, met by zeros of the hidden row
            down_piece[g][s] = load16<Vec16>(w_down + packed_offset<bf16_t>(out_tile, min(slice * K_STEPS_DOWN + s, down_k_steps - 1), down_k_steps, 0), lane * 16);
    }
    {
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
                    for (int j = 0; j < UP_ROUND; j++)
                        up_piece[u][j] = load16<Vec16>(w_up + packed_offset<bf16_t>(up_at[u], min(up_part_of[u] + DL_KSPLIT * (i0 + j), n_steps - 1), n_steps, 0), lane * 16);
            }
#pragma unroll
            for (int u = 0; u < UP_UNITS; u++)
#pragma unroll
                for (int j = 0; j < UP_ROUND; j++) {
                    int step = up_part_of[u] + DL_KSPLIT * (i0 + j);
                    Vec16 w = mask16(up_piece[u][j], step < n_steps);
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
    lds_barrier();
    // acc[r] of lane l in tile t is (token l % 16, hidden unit 16 t + 4 (l / 16) + r)
#pragma unroll
    for (int i = 0; i < BIAS_PER_THREAD; i++) {
        const int index = tid + DL_THREADS * i;
        if (index >= TILES * 256) break;
        const int tile = index / 256, r = (index / WAVE) % 4, l = index % WAVE;
        float value = 0.0f;
#pragma unroll
        for (int p = 0; p < DL_KSPLIT; p++) value += up_part[((p * TILES + tile) * 4 + r) * WAVE + l];
        const int unit = tile * 16 + 4 * (l / 16) + r, h = slice * U + unit;
        if (h < inner) {
            if (b_up) value += up_bias[i];
            if (epilogue == MLLM_EPI_GELU_TANH) value = gelu_tanh_for_bf16(value);
            else if (epilogue == MLLM_EPI_GELU_ERF) value = gelu_erf_for_bf16(value);
        } else {
            value = 0.0f;
        }
        hidden[(l % 16) * H_STRIDE + unit] = static_cast<bf16_t>(value);
    }
    lds_barrier();

    // ---- this slice's share of the down product: rows of w_down in tiles of 16, columns slice*U ..
    {
        const int token = token0 + row16;
        for (int tile0 = wave; tile0 < down_tiles; tile0 += DL_WAVES * DOWN_GROUP) {
            if (tile0 != wave) {  // wider than the rows asked for at the start cover
#pragma unroll
                for (int g = 0; g < DOWN_GROUP; g++) {
                    int out_tile = min(tile0 + DL_WAVES * g, down_tiles - 1);
#pragma unroll
                    for (int s = 0; s < K_STEPS_DOWN; s++)
                        down_piece[g][s] = load16<Vec16>(w_down + packed_offset<bf16_t>(out_tile, min(slice * K_STEPS_DOWN + s, down_k_steps - 1), down_k_steps, 0), lane * 16);
                }
            }
#pragma unroll
            for (int g = 0; g < DOWN_GROUP; g++) {
                int tile = tile0 + DL_WAVES * g;
                f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int s = 0; s < K_STEPS_DOWN; s++) {
                    bf16x8 x = *reinterpret_cast<const bf16x8*>(hidden + row16 * H_STRIDE + s * 32 + quad * 8);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&down_piece[g][s]), x, acc, 0, 0, 0);
                }
                int out_col = tile * 16 + 4 * quad;
                if (row16 < tokens_here && out_col < width)
                    *reinterpret_cast<f32x4*>(partial_out + ((size_t)slice * n_tokens + token) * width + out_col) = acc;
            }
        }
    }
}

// Four columns of a pending row with their sums taken: eight partial rows asked for at a time.
__device__ __forceinline__ f32x4 pending_piece(const PendingSum& in, int row_index, int width, int piece) {
    f32x4 value = load4(in.base + (size_t)row_index * width + 4 * piece);
    if (in.bias) value += load4(in.bias + 4 * piece);
    for (int s0 = 0; s0 < in.n_partials; s0 += 8) {
        f32x4 part[8];
#pragma unroll
        for (int u = 0; u < 8; u++)
            part[u] = load4(in.partials + ((size_t)min(s0 + u, in.n_partials - 1) * in.rows + row_index) * width + 4 * piece);
#pragma unroll
        for (int u = 0; u < 8; u++) value += part[u] * (s0 + u < in.n_partials ? 1.0f : 0.0f);
    }
    return value;
}

// The share of group `group` of `n_groups` in those four columns: the partial rows group, group + n_groups, ..., and with
// group 0 the base row and the bias.
__device__ __forceinline__ f32x4 pending_piece_share(const PendingSum& in, int row_index, int width, int piece, int group, int n_groups) {
    f32x4 value = {0.0f, 0.0f, 0.0f, 0.0f};
    if (group == 0) {
        value = load4(in.base + (size_t)row_index * width + 4 * piece);
        if (in.bias) value += load4(in.bias + 4 * piece);
    }
    for (int s0 = group; s0 < in.n_partials; s0 += 8 * n_groups) {
        f32x4 part[8];
#pragma unroll
        for (int u = 0; u < 8; u++)
            part[u] = load4(in.partials + ((size_t)min(s0 + u * n_groups, in.n_partials - 1) * in.rows + row_index) * width + 4 * piece);
#pragma unroll
        for (int u = 0; u < 8; u++) value += part[u] * (s0 + u * n_groups < in.n_partials ? 1.0f : 0.0f);
    }
    return value;
}

// out = base + bias + the partial rows: the pending stream as plain rows, for whatever does not
// take it pending. grid (pieces of 256 x 4 columns, rows).
__global__ __launch_bounds__(256) void pending_sum_kernel(PendingSum in, float* __restrict__ out, int width) {
    const int piece = blockIdx.x * 256 + threadIdx.x, row_index = blockIdx.y;
    if (piece * 4 >= width) return;
    *reinterpret_cast<f32x4*>(out + (size_t)row_index * width + 4 * piece) = pending_piece(in, row_index, width, piece);
}

// Row LayerNorm of pending rows (the sums are taken on the way in): a block a row, the row kept in LDS; row_index, if
// given, names the pending row of each output row. Centred, in 32-bit, like the norm of plain rows (elementwise.hip).
// GROUPS > 1 (a row of many partial rows, few of them in a launch: the rows a decode step's last layer leaves for the
// final norm): the block's threads in so many groups of `group_lanes`, each of which adds up every GROUPS-th partial row,
// all asked for at once; their shares meet in LDS, in a fixed order.
template <typename OutT, int GROUPS>
__global__ __launch_bounds__(GROUPS == 1 ? 256 : 1024) void pending_layernorm_kernel(
    PendingSum in, const int* __restrict__ row_index, const float* __restrict__ gamma, const float* __restrict__ beta,
    OutT* __restrict__ out, float* __restrict__ summed, int width, float eps, int packed_out, int group_lanes) {
    constexpr int THREADS = GROUPS == 1 ? 256 : 1024, WAVES = THREADS / WAVE;
    extern __shared__ f32x4 row_pieces[];  // width / 4, and behind them GROUPS x width / 4 for the groups' shares
    __shared__ float red[2][WAVES];
    const int tid = threadIdx.x, n_pieces = width / 4;
    const int source = row_index ? row_index[blockIdx.x] : blockIdx.x;
    if constexpr (GROUPS > 1) {
        const int group = tid / group_lanes, piece = tid % group_lanes;
        if (group < GROUPS && piece < n_pieces)
            row_pieces[(1 + group) * n_pieces + piece] = pending_piece_share(in, source, width, piece, group, GROUPS);
        __syncthreads();
    }
    float sum = 0.0f;
    for (int piece = tid; piece < n_pieces; piece += THREADS) {
        f32x4 value;
        if constexpr (GROUPS > 1) {
            value = row_pieces[n_pieces + piece];
#pragma unroll
            for (int g = 1; g < GROUPS; g++) value += row_pieces[(1 + g) * n_pieces + piece];
        } else {
            value = pending_piece(in, source, width, piece);
        }
        row_pieces[piece] = value;
        if (summed) *reinterpret_cast<f32x4*>(summed + (size_t)blockIdx.x * width + 4 * piece) = value;  // the row with its sums taken
        sum += (value[0] + value[1]) + (value[2] + value[3]);
    }
    sum = wave_total(sum);
    if (tid % WAVE == 0) red[0][tid / WAVE] = sum;
    __syncthreads();
    const float n = (float)width;
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; w += 4) total += (red[0][w] + red[0][w + 1]) + (red[0][w + 2] + red[0][w + 3]);
    const float mean = total / n;
    float squares = 0.0f;
    for (int piece = tid; piece < n_pieces; piece += THREADS) {
        f32x4 d = row_pieces[piece] - mean;
        squares += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
    }
    squares = wave_total(squares);
    if (tid % WAVE == 0) red[1][tid / WAVE] = squares;
    __syncthreads();
    total = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; w += 4) total += (red[1][w] + red[1][w + 1]) + (red[1][w + 2] + red[1][w + 3]);
    const float inverse_stddev = 1.0f / sqrtf(total / n + eps);
    for (int piece = tid; piece < n_pieces; piece += THREADS) {
        f32x4 y = (row_pieces[piece] - mean) * inverse_stddev * load4(gamma + 4 * piece) + load4(beta + 4 * piece);
        // four consecutive columns lie together in the packed layout too (inside one 16-byte piece)
        OutT* at = out + (packed_out ? packed_element<OutT>(blockIdx.x, 4 * piece, width) : (size_t)blockIdx.x * width + 4 * piece);
        if constexpr (sizeof(OutT) == 2) store_bf16x4(at, y);
        else *reinterpret_cast<f32x4*>(at) = y;
    }
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
    // Few tokens a block: more waves share a token's pending sums (one round of loads instead of
    // several, each a trip to memory) and more blocks pull at the matrices; many tokens a block: the
    // matrices are read fewer times.
    const int tokens_per_block = stage_pieces == 0 ? DL_TOKENS : (n_tokens <= 4 ? 1 : (n_tokens <= 8 ? 2 : (n_tokens <= 16 ? 4 : (n_tokens <= 64 ? 8 : DL_TOKENS))));
    dim3 grid((inner + U - 1) / U, (n_tokens + tokens_per_block - 1) / tokens_per_block);
    mllm_count_kernel(MLLM_K_DECODE_MLP_HALF);
    decode_mlp_half_kernel<NV, U><<<grid, DL_THREADS, lds, stream>>>(in, summed, gamma, beta, eps, w_up, b_up, w_down, partial_out,
                                                                      n_tokens, width, inner, epilogue, stage_pieces, tokens_per_block);
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

// Up to how many rows the two layer kernels beat the kernels run one by one, for a layer of this
// width (0: never). A property of the kernels, measured on MI355X: every (token, head) block pulls
// its own copy of the partial rows and of its head's matrices through one compute unit, which grows
// with the width, while what the fusion saves (five kernel boundaries a layer) does not. Up to 768
// columns the fused kernels win up to 16 rows (by 2 % at 1 row, 11 % at 8, 12 % at 16, and lose by
// 4 % at 32); at 1,024 columns they lose at every row count (1.10 against 0.96 ms a step at 1 row).
MLLM_API int mllm_decode_layer_rows(int width) {
    if (!mllm_decode_layer_supported(width, 0, 0, 0)) return 0;
    return width <= 768 ? 16 : 0;
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
        mllm_count_kernel(MLLM_K_DECODE_ATTENTION_HALF);                                                                \
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
    MLLM_REQUIRE(n_tokens >= 0 && n_tokens <= 65535 * 4, "decode_mlp_half: %d tokens", n_tokens);
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
    mllm_count_kernel(MLLM_K_PENDING_SUM);
    pending_sum_kernel<<<grid, 256, 0, stream>>>(in, out, width);
    return mllm_check_launch("pending_sum");
}


// LayerNorm of pending rows; row_index (or null) names the pending row of each of the n_rows output rows.
// summed (or null): [n_rows, width], also gets each of those rows with its sums taken, not normalised.
MLLM_API int mllm_pending_layernorm(const float* base, const float* partials, const float* pending_bias, int n_partials,
                                    int pending_rows, const int* row_index, const float* gamma, const float* beta, void* out,
                                    float* summed, int n_rows, int width, float eps, int out_dtype, int packed_out,
                                    hipStream_t stream) {
    MLLM_REQUIRE(base != nullptr && out != nullptr, "pending_layernorm: no rows");
    MLLM_REQUIRE(n_partials >= 0 && (n_partials == 0 || partials != nullptr), "pending_layernorm: %d partial rows without memory", n_partials);
    MLLM_REQUIRE(width > 0 && width % 4 == 0 && width <= 32768, "pending_layernorm: width %d is not a multiple of 4 up to 32768", width);
    MLLM_REQUIRE(n_rows >= 0 && pending_rows >= 0 && eps > 0.0f, "pending_layernorm: bad sizes");
    if (n_rows == 0) return 0;
    PendingSum in{base, partials, pending_bias, n_partials, pending_rows};
    mllm_count_kernel(MLLM_K_PENDING_LAYERNORM);
    // Many partial rows to a row and few rows (the final norm of a decode step behind the feed-forward half's 48 slices): four
    // groups of threads take every fourth partial row each. Where the rows are many the compute units are busy as it is.
    const int group_lanes = (width / 4 + WAVE - 1) / WAVE * WAVE;
    const bool grouped = n_partials >= 16 && n_rows <= 64 && 4 * group_lanes <= 1024;
#define MLLM_PENDING_NORM(OutT)                                                                                              \
    if (grouped)                                                                                                             \
        pending_layernorm_kernel<OutT, 4><<<n_rows, 1024, (size_t)width * 4 * 5, stream>>>(in, row_index, gamma, beta, (OutT*)out, summed, width, eps, packed_out, group_lanes); \
    else                                                                                                                     \
        pending_layernorm_kernel<OutT, 1><<<n_rows, 256, (size_t)width * 4, stream>>>(in, row_index, gamma, beta, (OutT*)out, summed, width, eps, packed_out, group_lanes);
    if (out_dtype == MLLM_F32) {
        MLLM_PENDING_NORM(float)
    } else if (out_dtype == MLLM_BF16) {
        MLLM_PENDING_NORM(bf16_t)
    } else {
        MLLM_REQUIRE(false, "pending_layernorm: unknown output dtype %d", out_dtype);
    }
#undef MLLM_PENDING_NORM
    return mllm_check_launch("pending_layernorm");
}
