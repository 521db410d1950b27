// The tiled bfloat16 product for many rows (prompt portions): out[M,N] = act(A[M,K] . W[N,K]^T + bias) (+ residual),
// W in the packed layout, K a multiple of 64. Included by gemm.hip (which defines CacheScatter).
//
// What the kernel is built around, each measured on MI355X:
//  * Operands go from memory to LDS directly (global_load_lds_dwordx4: a wave's load lands as 1 KiB
//    of consecutive LDS in lane order), one or two tiles of K ahead of the products, and cost no
//    registers. Which bytes a lane asks for is therefore what lays the tile out in LDS. A chunk of
//    the packed W is taken as it lies. For the row-major A, four lanes read the 64 bytes a row has in
//    a chunk, so that a quarter wave touches 4 cache lines (a lane per row touched 16, and the
//    lookups in the vector cache, not the bytes, bounded the kernel: 27 -> 17 us at 2,048 x 2,304 x
//    768); a row's four pieces lie in LDS rotated by the row (piece ^ (row / 4) % 4), so that the
//    sixteen lanes of a fragment read fall on sixteen different groups of banks.
//  * A wave owns 64 x 64 outputs or more: at 32 x 32 every matrix instruction needs two fragment
//    reads of its own and the LDS, not the matrix cores, sets the pace.
//  * W is the first operand of the matrix instruction: a lane then holds four consecutive columns
//    of one row, and the epilogue, which goes through LDS once more, stores whole rows of a wave's
//    tile in 16-byte pieces (stored as the accumulators lie, the same tile costs 6 us of an 18 us
//    product).
//  * One barrier a tile. Before it a wave waits for its own fragment reads of the tile that is
//    ending: the loads issued right after the barrier overwrite that tile's stage, and a fragment
//    read still queued in the LDS unit would see the new tile (found as a wrong row in one product
//    out of thousands).
#pragma once

#include <type_traits>

namespace stream {

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt with only the vector-memory counter set: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

template <int N>
__device__ __forceinline__ void wait_lgkmcnt() {
    // only the counter of LDS and scalar-memory operations (as a builtin, so that the compiler counts on it too)
    __builtin_amdgcn_s_waitcnt(0xF | (0x3 << 14) | (0x7 << 4) | ((N & 0xF) << 8));
}

template <typename OutT>
__device__ __forceinline__ void put4(OutT* at, f32x4 v);
template <>
__device__ __forceinline__ void put4<float>(float* at, f32x4 v) {
    *reinterpret_cast<f32x4*>(at) = v;
}
template <>
__device__ __forceinline__ void put4<bf16_t>(bf16_t* at, f32x4 v) {
    bf16x4 o;
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = static_cast<bf16_t>(v[e]);
    *reinterpret_cast<bf16x4*>(at) = o;
}

// grid (N tiles, M tiles, blocks along K). gridDim.z > 1: each block takes k_per_block of K (a multiple
// of 64) and leaves a partial product in matrix blockIdx.z of `out` (float, no bias / epilogue / residual).
// WAVES_K = 2: two waves share a tile of outputs and take half of every tile of K each; their sums meet in LDS at the end.
template <typename OutT, int BM, int BN, int WAVES_M, int WAVES_N, int WAVES_K, int STAGES>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N * WAVES_K) void gemm_stream_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias, const float* __restrict__ residual,
    OutT* __restrict__ out, int M, int N, int K, int epilogue, CacheScatter scatter, int k_per_block) {
    constexpr int NW = WAVES_M * WAVES_N * WAVES_K;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, FM = WM / 32, FN = WN / 32;
    constexpr int BK = 64, KS = BK / 16 / WAVES_K;           // steps of 16 along K a wave takes of a tile
    constexpr int OWN = FM / WAVES_K;                        // slabs of 32 rows of its tile a wave finishes
    constexpr int A_LOADS = BM / 16 * 2, W_LOADS = BN / 16 * 2, LOADS = A_LOADS + W_LOADS;  // loads of 1 KiB a tile of K
    static_assert(WAVES_K == 1 || WAVES_K == 2, "a tile of K is taken whole or in halves");
    static_assert(FM >= 1 && FN >= 1 && FM % WAVES_K == 0, "the waves that share a tile finish equal parts of it");
    static_assert(A_LOADS % NW == 0 && W_LOADS % NW == 0, "every wave issues the same loads of A and of W");
    constexpr int A_LPW = A_LOADS / NW, LPW = LOADS / NW;
    static_assert(LPW * (STAGES - 1) < 64, "the loads in flight must fit the counter");
    constexpr int STAGE_BYTES = (BM + BN) * 128;
    constexpr int OUT_VEC = 16 / (int)sizeof(OutT);          // columns in a 16-byte piece of the output
    constexpr int SLAB_ROW = WN * (int)sizeof(OutT) + 16;    // a row of a wave's tile in LDS, padded by one piece
    constexpr int PIECES = WN / OUT_VEC;
    constexpr int SHARED_SUMS = WAVES_K == 1 ? 0 : NW * FN * OWN * 4096;  // what the waves that share a tile hand each other
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int wave_k = wave / (WAVES_M * WAVES_N), wave_m = wave / WAVES_N % WAVES_M, wave_n = wave % WAVES_N;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int k_begin = blockIdx.z * k_per_block, k_end = min(K, k_begin + k_per_block);
    const int k_steps = K / 32, n_tiles = (k_end - k_begin) / BK;
    const int w_row_tiles = (N + 15) / 16;
    out += (size_t)blockIdx.z * M * N;

    // This wave's loads of a tile: load q = wave + NW * i of the stage, the first A_LPW of them from A. An address is a
    // base that all lanes share, which moves on with the tile, and a lane's own 32-bit offset.
    const unsigned char* base[LPW];
    unsigned lane_offset[LPW];
#pragma unroll
    for (int i = 0; i < LPW; i++) {
        const int q = wave + NW * i;
        if (i < A_LPW) {
            const int rt = q / 2, kc = q % 2;
            const int r16 = lane / 4, piece = (lane % 4) ^ ((r16 >> 2) & 3);
            const int row = min(m0 + rt * 16 + r16, M - 1);  // beyond the last row: that row again, never stored
            base[i] = reinterpret_cast<const unsigned char*>(A + k_begin + kc * 32);
            lane_offset[i] = ((unsigned)row * (unsigned)K + piece * 8) * 2;
        } else {
            const int qw = q - A_LOADS, rt = qw / 2, kc = qw % 2;
            const int row_tile = min(n0 / 16 + rt, w_row_tiles - 1);
            base[i] = reinterpret_cast<const unsigned char*>(W + packed_offset<bf16_t>(row_tile, k_begin / 32 + kc, k_steps, 0));
            lane_offset[i] = lane * 16;
        }
    }
    auto issue_load = [&](int tile, int stage, int i) {
        const int t = min(tile, n_tiles - 1);  // beyond the end: the last tile again, never used (the count of loads in flight stays the same)
        const unsigned char* p = base[i] + (size_t)t * (i < A_LPW ? BK * 2 : 2 * 1024) + lane_offset[i];
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)p,
                                         (void __attribute__((address_space(3)))*)(lds + stage * STAGE_BYTES + (wave + NW * i) * 1024), 16, 0, 0);
    };
    auto issue = [&](int tile, int stage) {
#pragma unroll
        for (int i = 0; i < LPW; i++) issue_load(tile, stage, i);
    };

    // How a wave's rows leave: 32 rows of its tile at a time pass through LDS and are stored in 16-byte pieces of whole
    // rows, ROWS_A_STEP rows with every store (a power of two, so that a step's place is a constant; with 12 or 24 pieces
    // a row some lanes idle). A lane keeps its piece and its row within the step for the whole tile.
    constexpr int ROWS_A_STEP = PIECES > 32 ? 1 : PIECES > 16 ? 2 : PIECES > 8 ? 4 : PIECES > 4 ? 8 : 16;
    constexpr int ROW_STEPS = 32 / ROWS_A_STEP;
    static_assert(ROWS_A_STEP * PIECES <= WAVE, "a step's pieces fit a wave");
    const int n_wave = n0 + wave_n * WN, own0 = wave_k * OWN;
    const int lane_row = lane / PIECES, lane_piece = lane % PIECES;
    const int m_lane = m0 + wave_m * WM + own0 * 32 + lane_row, n_lane = n_wave + lane_piece * OUT_VEC;
    // rows from the lane's first one to the end of the matrix; none for a lane that idles or whose columns lie outside
    const int rows_left = lane_row < ROWS_A_STEP && n_lane < N ? M - m_lane : 0;

    // What the epilogue adds is asked for now and arrives while the products run: asked for where it is used, every
    // block would wait for it at the end, with nothing left to hide the trip behind.
    f32x4 early_bias[FN][4];
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int n = n_wave + j * 32 + 8 * g + 4 * (lane / 32);  // N is a multiple of 8: four columns are inside or outside together
            early_bias[j][g] = bias && n < N ? *reinterpret_cast<const f32x4*>(bias + n) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    constexpr bool WITH_RESIDUAL = sizeof(OutT) == 4, CAN_SCATTER = sizeof(OutT) == 2;
    f32x4 early_residual[WITH_RESIDUAL ? OWN : 1][WITH_RESIDUAL ? ROW_STEPS : 1];
    if constexpr (WITH_RESIDUAL) {
        const float* residual_lane = residual + (size_t)m_lane * N + n_lane;
#pragma unroll
        for (int i = 0; i < OWN; i++)
#pragma unroll
            for (int r = 0; r < ROW_STEPS; r++) {
                const int row = i * 32 + r * ROWS_A_STEP;
                early_residual[i][r] = residual && row < rows_left ? *reinterpret_cast<const f32x4*>(residual_lane + (size_t)row * N) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
    }
    int early_slot[CAN_SCATTER ? OWN : 1][CAN_SCATTER ? ROW_STEPS : 1];  // the cache slots of the lane's rows (a fused q/k/v projection)
    if constexpr (CAN_SCATTER) {
        if (scatter.enabled) {
#pragma unroll
            for (int i = 0; i < OWN; i++)
#pragma unroll
                for (int r = 0; r < ROW_STEPS; r++) {
                    const int row = i * 32 + r * ROWS_A_STEP;
                    early_slot[i][r] = row < rows_left ? scatter.slots[m_lane + row] : -1;
                }
        }
    }

    f32x16 acc[FN][FM];
    if (n_tiles > 0) {
#pragma unroll
        for (int s = 0; s < STAGES - 1; s++) issue(s, s);
    }
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[j][i][v] = 0.0f;
    if (n_tiles > 0) {

        // A 32 x 16 fragment: lane l holds row l % 32, k (l / 32) * 8 .. + 8. W: chunk [piece][row]; A: chunk [row][piece rotated].
        const int w_frag0 = BM * 128 + (wave_n * WN / 16) * 2048 + ((lane % 32) / 16) * 2048 + (lane / 32) * 256 + (lane % 16) * 16;
        const int a_row0 = (wave_m * WM / 16) * 2048 + ((lane % 32) / 16) * 2048 + (lane % 16) * 64, a_turn = ((lane % 16) >> 2) & 3;
        const int kk0 = wave_k * KS;
        bf16x8 a[2][FM], w[2][FN];
        auto read_frags = [&](int set, const unsigned char* stage, int kk) {
#pragma unroll
            for (int i = 0; i < FM; i++)
                a[set][i] = *reinterpret_cast<const bf16x8*>(stage + a_row0 + i * 4096 + (kk / 2) * 1024 + ((((kk % 2) * 2 + lane / 32) ^ a_turn) * 16));
#pragma unroll
            for (int j = 0; j < FN; j++) w[set][j] = *reinterpret_cast<const bf16x8*>(stage + w_frag0 + j * 4096 + (kk / 2) * 1024 + (kk % 2) * 512);
        };
        // The products of step s of a tile, and between them the step's share of the loads of the tile STAGES - 1 ahead:
        // a compute unit takes a load of 1 KiB every 16 cycles or so, and a wave that issues all of a tile's loads at
        // once stands still until the unit has taken them, its matrix core with it.
        auto step_loads = [](int s) { return (s * LPW + KS - 1) / KS; };  // loads 'step_loads(s) .. step_loads(s + 1)' go with step s
        auto products = [&](int set, int s, int load_tile, int load_stage) {
#pragma unroll
            for (int j = 0; j < FN; j++)
#pragma unroll
                for (int i = 0; i < FM; i++) {
                    acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w[set][j], a[set][i], acc[j][i], 0, 0, 0);
                    constexpr int PER_STEP = FM * FN;
                    const int first = step_loads(s), count = step_loads(s + 1) - first, slot = j * FM + i;
                    // the step's loads spread over its products: after product 'slot' come loads slot*count/PER_STEP .. (slot+1)*count/PER_STEP
#pragma unroll
                    for (int l = slot * count / PER_STEP; l < (slot + 1) * count / PER_STEP; l++) issue_load(load_tile, load_stage, first + l);
                    __builtin_amdgcn_sched_barrier(0);
                }
        };
        // In flight when a tile ends: the whole tiles between the next one and the one being asked for, and of that one
        // what the steps before the last have issued.
        constexpr int IN_FLIGHT_AT_END = (STAGES - 3) * LPW + (KS - 1) * LPW / KS + ((KS - 1) * LPW % KS ? 1 : 0);
        static_assert(STAGES >= 3, "a tile's loads are spread over the tile before the one before it");
        wait_vmcnt<LPW*(STAGES - 2)>();
        wait_lgkmcnt<0>();  // kernel arguments still on their way would make every wait for fragments in the loop a wait for all of them
        asm volatile("s_barrier" ::: "memory");
        read_frags(0, lds, kk0);
        // The order of a step is kept as written (the compiler otherwise gathers the reads of a whole tile in front of the
        // barrier and the products behind it): the fragments of the next step are asked for, then this step's products
        // are issued, and the reads travel while the matrix cores work. A step begins with the wait for its own
        // fragments, asked for a step ago: with loads into LDS under way the compiler can only wait for every LDS
        // operation at once, and left to place that wait itself it puts it behind the reads of the next step.
        for (int t = 0; t < n_tiles; t++) {
            const unsigned char* stage = lds + (t % STAGES) * STAGE_BYTES;
            const int load_tile = t + STAGES - 1, load_stage = (t + STAGES - 1) % STAGES;  // the stage of tile t - 1, which every wave has left
#pragma unroll
            for (int s = 0; s + 1 < KS; s++) {
                wait_lgkmcnt<0>();
                __builtin_amdgcn_sched_barrier(0);
                read_frags((s + 1) % 2, stage, kk0 + s + 1);
                __builtin_amdgcn_sched_barrier(0);
                products(s % 2, s, load_tile, load_stage);
            }
            // the next tile has landed in every wave, and every wave has its last fragments of this one
            wait_vmcnt<IN_FLIGHT_AT_END>();
            wait_lgkmcnt<0>();
            asm volatile("s_barrier" ::: "memory");
            read_frags(KS % 2, lds + ((t + 1) % STAGES) * STAGE_BYTES, kk0);
            __builtin_amdgcn_sched_barrier(0);
            products((KS - 1) % 2, KS - 1, load_tile, load_stage);
        }
    }

    // acc[j][i][v] is row m0 + wave_m*WM + i*32 + lane%32, column n0 + wave_n*WN + j*32 + 8*(v/4) + 4*(lane/32) + v%4.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // no load is under way, no wave still reads the stages
    if constexpr (WAVES_K == 2) {
        // The two waves of a tile hand each other the slabs they do not finish, as the accumulators lie (a lane's four
        // values side by side: no bank conflicts), and add what they are handed to the slabs they do finish.
        f32x4* mine = reinterpret_cast<f32x4*>(lds + wave * (FN * OWN * 4096));
        const f32x4* theirs = reinterpret_cast<const f32x4*>(lds + (wave ^ (WAVES_M * WAVES_N)) * (FN * OWN * 4096));
        static_assert((WAVES_M * WAVES_N & (WAVES_M * WAVES_N - 1)) == 0, "the partner's index differs in one bit");
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int i = 0; i < OWN; i++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    f32x4 value;
#pragma unroll
                    for (int e = 0; e < 4; e++) value[e] = wave_k == 0 ? acc[j][OWN + i][4 * g + e] : acc[j][i][4 * g + e];
                    mine[((j * OWN + i) * 4 + g) * WAVE + lane] = value;
                }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int i = 0; i < OWN; i++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const f32x4 value = theirs[((j * OWN + i) * 4 + g) * WAVE + lane];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        // kept at index i whichever half the wave finishes: indices stay constants, registers stay registers
                        const float sum = (wave_k == 0 ? acc[j][i][4 * g + e] : acc[j][OWN + i][4 * g + e]) + value[e];
                        acc[j][i][4 * g + e] = sum;
                    }
                }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    // Through LDS: 32 rows of the wave's tile at a time, written as the accumulators lie, read back and stored row by row.
    // The kind of epilogue is a constant inside 'leave' (as a run-time value every group of four accumulators
    // carried its own branches, and a lone wave on its SIMD pays every instruction in full).
    unsigned char* slab = lds + SHARED_SUMS + wave * (32 * SLAB_ROW);
    unsigned char* slab_write = slab + (lane % 32) * SLAB_ROW + 4 * (lane / 32) * (int)sizeof(OutT);
    const unsigned char* slab_read = slab + min(lane_row, ROWS_A_STEP - 1) * SLAB_ROW + lane_piece * 16;  // (an idling lane reads inside the slab too)
    auto leave = [&](auto kind, auto scattered) {
        constexpr int KIND = decltype(kind)::value;
        constexpr bool SCATTERED = decltype(scattered)::value;
        // where a lane's piece goes: q columns to out [M, q_width], key and value columns into the cache page at the
        // row's slot (a piece lies inside one head: the head size is a multiple of 8)
        OutT* out_lane = out + (size_t)m_lane * (SCATTERED ? scatter.q_width : N) + n_lane;
        bool to_cache = false;
        OutT* pages = nullptr;
        int kv_head = 0;
        if constexpr (SCATTERED) {
            to_cache = n_lane >= scatter.q_width;
            int c = n_lane - scatter.q_width;
            pages = (OutT*)(c < scatter.kv_width ? scatter.k_pages : scatter.v_pages);
            if (c >= scatter.kv_width) c -= scatter.kv_width;
            kv_head = c / scatter.head_size;
            pages += c % scatter.head_size;
        }
#pragma unroll
        for (int i = 0; i < OWN; i++) {
#pragma unroll
            for (int j = 0; j < FN; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    f32x4 value;
#pragma unroll
                    for (int e = 0; e < 4; e++) value[e] = acc[j][i][4 * g + e];
                    value += early_bias[j][g];
                    if constexpr (KIND == MLLM_EPI_GELU_TANH) {
#pragma unroll
                        for (int e = 0; e < 4; e++) value[e] = sizeof(OutT) == 2 ? gelu_tanh_for_bf16(value[e]) : gelu_tanh(value[e]);
                    } else if constexpr (KIND == MLLM_EPI_GELU_ERF) {
#pragma unroll
                        for (int e = 0; e < 4; e++) value[e] = sizeof(OutT) == 2 ? gelu_erf_for_bf16(value[e]) : gelu_erf(value[e]);
                    }
                    put4<OutT>(reinterpret_cast<OutT*>(slab_write) + j * 32 + 8 * g, value);
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int r = 0; r < ROW_STEPS; r++) {
                const int row = i * 32 + r * ROWS_A_STEP;
                Vec16 v = *reinterpret_cast<const Vec16*>(slab_read + r * ROWS_A_STEP * SLAB_ROW);
                if (row >= rows_left) continue;
                if constexpr (SCATTERED) {
                    if (to_cache) {
                        const int slot = early_slot[i][r];
                        if (slot < 0) continue;
                        const int page = slot >> scatter.page_shift, offset = slot & ((1 << scatter.page_shift) - 1);
                        *reinterpret_cast<Vec16*>(pages + ((((size_t)page * scatter.n_kv_heads + kv_head) << scatter.page_shift) + offset) * scatter.head_size) = v;
                    } else {
                        *reinterpret_cast<Vec16*>(out_lane + (size_t)row * scatter.q_width) = v;
                    }
                } else {
                    if constexpr (WITH_RESIDUAL) {
                        f32x4 sum = *reinterpret_cast<f32x4*>(&v);
                        sum = early_residual[i][r] + sum;   // zeros where there is no residual
                        v = *reinterpret_cast<Vec16*>(&sum);
                    }
                    *reinterpret_cast<Vec16*>(out_lane + (size_t)row * N) = v;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
    };
    using std::integral_constant;
    if constexpr (CAN_SCATTER) {
        if (scatter.enabled) {
            leave(integral_constant<int, MLLM_EPI_NONE>{}, integral_constant<bool, true>{});  // (a q/k/v projection has no activation)
            return;
        }
    }
    if (epilogue == MLLM_EPI_GELU_TANH) leave(integral_constant<int, MLLM_EPI_GELU_TANH>{}, integral_constant<bool, false>{});
    else if (epilogue == MLLM_EPI_GELU_ERF) leave(integral_constant<int, MLLM_EPI_GELU_ERF>{}, integral_constant<bool, false>{});
    else leave(integral_constant<int, MLLM_EPI_NONE>{}, integral_constant<bool, false>{});
}

template <typename OutT, int BM, int BN, int WAVES_M, int WAVES_N, int WAVES_K, int STAGES>
void launch(const bf16_t* a, const bf16_t* w, const float* bias, const float* residual, OutT* o, int M, int N, int K, int epilogue,
           hipStream_t stream, CacheScatter scatter, int k_blocks) {
    // the stages of the loop, or what the epilogue passes through LDS (the sums that waves sharing a tile hand each other,
    // then 32 rows of every wave's tile, padded), whichever is more
    constexpr int NW = WAVES_M * WAVES_N * WAVES_K;
    constexpr int SHARED_SUMS = WAVES_K == 1 ? 0 : NW * (BN / WAVES_N / 32) * (BM / WAVES_M / 32 / WAVES_K) * 4096;
    constexpr int SLAB_BYTES = SHARED_SUMS + NW * 32 * (BN / WAVES_N * (int)sizeof(OutT) + 16);
    constexpr int LDS_BYTES = STAGES * (BM + BN) * 128 > SLAB_BYTES ? STAGES * (BM + BN) * 128 : SLAB_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "a block's LDS");
    static bool raised = false;  // per instantiation: the limit on dynamic LDS is a property of the kernel
    if (!raised && LDS_BYTES > 64 * 1024) {
        // (if this fails the launch below fails too, and the entry point reports that)
        raised = hipFuncSetAttribute((const void*)gemm_stream_kernel<OutT, BM, BN, WAVES_M, WAVES_N, WAVES_K, STAGES>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) == hipSuccess;
    }
    const int k_per_block = k_blocks == 1 ? K : ceil_div(ceil_div(K, k_blocks), 64) * 64;
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM), k_blocks);
    gemm_stream_kernel<OutT, BM, BN, WAVES_M, WAVES_N, WAVES_K, STAGES><<<grid, 64 * NW, LDS_BYTES, stream>>>(
        a, w, bias, residual, o, M, N, K, epilogue, scatter, k_per_block);
}

// Whether the product takes this kernel: bfloat16 with a packed W, whole tiles of K, whole 16-byte pieces of output
// columns, enough rows to fill tiles of 128, an A whose bytes a 32-bit offset reaches; a fused q/k/v projection only
// where a piece stays inside one head.
inline bool takes(int M, int N, int K, bool packed, const CacheScatter& scatter, size_t out_element) {
    if (!packed || K % 64 != 0 || K < 64 || N % 8 != 0 || M < 192 || ceil_div(M, 128) > 65535) return false;
    if ((long long)M * K * 2 >= (1LL << 32)) return false;
    if (scatter.enabled && (out_element != 2 || scatter.head_size % 8 != 0 || scatter.q_width % 8 != 0 || scatter.kv_width % 8 != 0)) return false;
    return true;
}

template <typename OutT>
void dispatch(const bf16_t* a, const bf16_t* w, const float* bias, const float* residual, OutT* o, int M, int N, int K, int epilogue,
             hipStream_t stream, CacheScatter scatter, int k_blocks) {
    static const int variant = getenv("MLLM_GEMM_VARIANT") ? atoi(getenv("MLLM_GEMM_VARIANT")) : 0;
#define MLLM_STREAM(BM, BN, WM_, WN_, WK_, ST) launch<OutT, BM, BN, WM_, WN_, WK_, ST>(a, w, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks)
    switch (variant) {
        case 1: MLLM_STREAM(128, 192, 2, 2, 1, 3); return;
        case 2: MLLM_STREAM(128, 128, 2, 2, 1, 3); return;
        case 3: MLLM_STREAM(128, 64, 2, 1, 2, 3); return;
        case 4: MLLM_STREAM(256, 128, 4, 2, 1, 3); return;
        case 5: MLLM_STREAM(128, 128, 2, 2, 1, 4); return;
        case 6: MLLM_STREAM(128, 64, 2, 1, 2, 4); return;
        case 7: MLLM_STREAM(128, 64, 2, 2, 1, 3); return;
        case 8: MLLM_STREAM(128, 128, 4, 2, 1, 3); return;
        case 9: MLLM_STREAM(128, 64, 2, 1, 2, 5); return;
        case 10: if constexpr (sizeof(OutT) == 2) { MLLM_STREAM(128, 192, 2, 2, 2, 3); return; } break;
        case 12: MLLM_STREAM(128, 128, 2, 2, 2, 3); return;
        default: break;
    }
    if (ceil_div(M, 128) * ceil_div(N, 192) * k_blocks >= 160) MLLM_STREAM(128, 192, 2, 2, 1, 3);
    else if (K / k_blocks >= 1536) MLLM_STREAM(128, 64, 2, 1, 2, 4);
    else MLLM_STREAM(128, 64, 2, 2, 1, 3);
#undef MLLM_STREAM
}

}  // namespace stream
