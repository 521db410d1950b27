// The tiled bfloat16 product for many rows (prompt portions): out[M,N] = act(A[M,K] . W[N,K]^T + bias) (+ residual),
// W in the packed layout, K a multiple of 64. Included by gemm.hip (which defines CacheScatter).
//
// What the kernel is built around, each measured on MI355X:
//  * Operands go from memory to LDS directly (global_load_lds_dwordx4: a wave's load lands as 1 KiB
//    of consecutive LDS in lane order) and cost no registers. Which bytes a lane asks for is therefore
//    what lays the tile out in LDS. A chunk of the packed W is taken as it lies. For the row-major A,
//    eight lanes read the 128 bytes a row has in a tile of K, one whole cache line (the vector cache
//    works by lines, not bytes: a lane per row touched 64 lines with a load, four lanes per 64 bytes
//    of a row touched every line twice: 18.3 -> 18.0 us at 2,048 x 768 x 3,072); a row's eight pieces lie in LDS rotated by the row
//    (piece ^ (row / 2) % 8), so that the sixteen lanes of a fragment read fall on sixteen different
//    groups of banks.
//  * A block has a compute unit to itself and a wave a SIMD: whatever a wave waits for, its matrix
//    core waits for too. So a wave owns 64 x 64 outputs or more (at 64 x 32 the fragment reads, not
//    the products, set the pace); fragments are asked for two steps of K before their products; a
//    tile's loads from memory go out a few at a time between the products of earlier tiles (a compute
//    unit takes a load of 1 KiB every 16 cycles or so: a wave that issues a whole tile's loads at
//    once stands still meanwhile); and the order of all this is pinned (sched_barrier), because left
//    alone the compiler gathers a tile's reads in front of the barrier and its products behind it.
//  * With loads into LDS under way the compiler can only wait for all LDS operations at once before
//    the first use of any value read from LDS. The fragment reads are therefore inline assembly the
//    compiler does not see through, with the wave's own counted waits.
//  * The blocks of one XCD take the tiles of one rectangle of the output: the eight L2 caches then
//    each fetch a part of A and W once (taking tiles in turn, every XCD reads nearly all of both:
//    21.4 -> 18.3 us for 2,048 x 768 x 3,072).
//  * W is the first operand of the matrix instruction: a lane then holds four consecutive columns
//    of one row, and the epilogue, which goes through LDS once more, stores whole rows of a wave's
//    tile in 16-byte pieces (stored as the accumulators lie, the same tile costs 6 us of an 18 us
//    product). A lone wave pays every instruction of the epilogue in full: the kind of epilogue is a
//    compile-time constant there, and a lane's place in the rows is a constant of the lane.
//  * One barrier a tile. Before it a wave waits for its own fragment reads of the tile that is
//    ending: the loads issued right after the barrier overwrite that tile's stage, and a fragment
//    read still queued in the LDS unit would see the new tile (found as a wrong row in one product
//    out of thousands).
#pragma once

#include <type_traits>
#include <utility>

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

typedef int i32x4 __attribute__((ext_vector_type(4)));

template <typename F, int... I>
__device__ __forceinline__ void static_for_each(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant in its body
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_each(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

// A fragment read the compiler does not know to be one: with loads into LDS under way it can only wait for every LDS
// operation at once, before the first use of anything read from LDS, which ends all reading ahead. The value is in the
// register once a wait of the wave's own (fragments_landed) has passed; until then nothing may read the register.
template <int OFFSET>
__device__ __forceinline__ void ask_fragment(i32x4& to, unsigned address) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(to) : "v"(address), "n"(OFFSET));
}
// waits until at most IN_FLIGHT of the wave's LDS operations are under way (they complete in order; a scalar load,
// which counts there too and completes out of order, must not be under way: the loop has none, which a test of the
// compiled code checks); the fragments named are only read after it
template <int IN_FLIGHT>
__device__ __forceinline__ void fragments_landed(i32x4& first) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(first) : "n"(IN_FLIGHT));
}
__device__ __forceinline__ void and_this_one(i32x4& fragment) { asm volatile("" : "+v"(fragment)); }
__device__ __forceinline__ void still_written(const i32x4& fragment) { asm volatile("" : : "v"(fragment)); }

// Eight rectangles of 'wide' x 'high' tiles, 'across' of them side by side along N, cover the tiles of the output.
struct XcdTiles {
    int across, wide, high;
};
// the split of the eight rectangles (1 x 8, 2 x 4, 4 x 2 or 8 x 1) whose rectangle needs the fewest rows of A and W together
inline XcdTiles place_tiles(int tiles_m, int tiles_n, int bm, int bn) {
    XcdTiles best{1, tiles_n, ceil_div(tiles_m, 8)};
    long best_rows = -1;
    for (int across = 1; across <= 8; across *= 2) {
        const int wide = ceil_div(tiles_n, across), high = ceil_div(tiles_m, 8 / across);
        const long rows = (long)wide * bn + (long)high * bm;
        if (best_rows < 0 || rows < best_rows) best = XcdTiles{across, wide, high}, best_rows = rows;
    }
    return best;
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

// grid: one row of blocks, placed by 'places' (tiles and blocks along K). More than one block along K: each block takes k_per_block of K (a multiple
// of 64) and leaves a partial product in matrix 'block_k' of `out` (float, no bias / epilogue / residual).
// WAVES_K = 2: two waves share a tile of outputs and take half of every tile of K each; their sums meet in LDS at the end.
template <typename OutT, int BM, int BN, int WAVES_M, int WAVES_N, int WAVES_K, int STAGES>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N * WAVES_K) void gemm_stream_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias, const float* __restrict__ residual,
    OutT* __restrict__ out, int M, int N, int K, int epilogue, CacheScatter scatter, int k_per_block, XcdTiles places) {
    constexpr int NW = WAVES_M * WAVES_N * WAVES_K;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, FM = WM / 32, FN = WN / 32;
    constexpr int BK = 64, KS = BK / 16 / WAVES_K;           // steps of 16 along K a wave takes of a tile
    constexpr int OWN = FM / WAVES_K;                        // slabs of 32 rows of its tile a wave finishes
    constexpr int A_LOADS = BM / 8, W_LOADS = BN / 16 * 2, LOADS = A_LOADS + W_LOADS;  // loads of 1 KiB a tile of K
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
    // Blocks go round the eight XCDs in turn, each with an L2 of its own: the blocks of one XCD take the tiles of one
    // rectangle of the output, so that the rows of A and of W an XCD reads are few and each is fetched into its L2 once.
    const int xcd = blockIdx.x % 8, in_xcd = blockIdx.x / 8;
    const int block_k = in_xcd / (places.wide * places.high), in_rectangle = in_xcd % (places.wide * places.high);
    const int tile_m = (xcd / places.across) * places.high + in_rectangle / places.wide;
    const int tile_n = (xcd % places.across) * places.wide + in_rectangle % places.wide;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    if (m0 >= M || n0 >= N) return;  // (the rectangles cover more than the matrix; the whole block leaves)
    const int k_begin = block_k * k_per_block, k_end = min(K, k_begin + k_per_block);
    const int k_steps = K / 32, n_tiles = (k_end - k_begin) / BK;
    const int w_row_tiles = (N + 15) / 16;
    out += (size_t)block_k * M * N;

    // This wave's loads of a tile: load q = wave + NW * i of the stage, the first A_LPW of them from A. An address is a
    // base that all lanes share, which moves on with the tile, and a lane's own 32-bit offset.
    const unsigned char* base[LPW];
    unsigned lane_offset[LPW];
#pragma unroll
    for (int i = 0; i < LPW; i++) {
        const int q = wave + NW * i;
        if (i < A_LPW) {
            // eight rows of 128 bytes: eight lanes take the eight pieces of a row (a whole cache line), turned by the row
            const int in_tile = q * 8 + lane / 8, piece = (lane % 8) ^ ((in_tile >> 1) & 7);
            const int row = min(m0 + in_tile, M - 1);  // beyond the last row: that row again, never stored
            base[i] = reinterpret_cast<const unsigned char*>(A + k_begin);
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

        // A 32 x 16 fragment: lane l holds row l % 32, k (l / 32) * 8 .. + 8. W: chunk [piece][row]; A: rows of 128 bytes, a
        // row's eight pieces turned by the row (piece ^ (row / 2) % 8: the sixteen rows of a quarter wave's read then fall
        // on sixteen different groups of banks).
        const int w_frag0 = BM * 128 + (wave_n * WN / 16) * 2048 + ((lane % 32) / 16) * 2048 + (lane / 32) * 256 + (lane % 16) * 16;
        const int a_row0 = (wave_m * WM + lane % 32) * 128, a_turn = (lane >> 1) & 7;
        // Fragments are asked for two steps before their products (four sets of registers): a step's reads come from all
        // waves at once, and the LDS takes longer over them than one step's products last. A turn of the loop is four
        // steps: one tile, or two where two waves share the tile's steps. Step g of a turn: wait for set g; then its products,
        // and between them the reads of step g + 2 and the step's share of the loads of a tile further on.
        constexpr int SETS = 4, TILES_A_TURN = SETS / KS, FRAGMENTS = FM + FN, PRODUCTS = FM * FN;
        i32x4 a[SETS][FM], w[SETS][FN];
        const int kk0 = wave_k * KS;
        unsigned a_lane[KS];  // step s of the wave's steps of a tile: pieces 2 (kk0 + s) and 2 (kk0 + s) + 1 of the row
#pragma unroll
        for (int step = 0; step < KS; step++) a_lane[step] = a_row0 + (((2 * (kk0 + step) + lane / 32) ^ a_turn) * 16);
        const unsigned w_lane = w_frag0 + wave_k * (KS / 2) * 1024;
        auto ask = [&](auto set, auto step, auto fragment, unsigned stage_offset) {  // fragment 'fragment' of step 'step' of a tile
            constexpr int SET = decltype(set)::value, S = decltype(step)::value, F = decltype(fragment)::value;
            if constexpr (F < FM) ask_fragment<F * 4096>(a[SET][F], a_lane[S] + stage_offset);
            else ask_fragment<(F - FM) * 4096 + (S / 2) * 1024 + (S % 2) * 512>(w[SET][F - FM], w_lane + stage_offset);
        };
        // The loads of tile u + STAGES go into the stage of tile u, between the barrier in tile u (which every wave passes
        // with its reads of tile u done) and the barrier in tile u + 1: KS steps, each with its share.
        // loads share(e) .. share(e + 1) go with step e after the barrier; with two stages all of them at once, behind the
        // barrier that frees their stage: they have one tile's time to land, and none of it to spare
        auto share = [](int e) { return STAGES == 2 ? (e >= 1 ? LPW : 0) : (e * LPW + KS - 1) / KS; };
        auto stage_of = [](int tile) { return (tile % STAGES) * STAGE_BYTES; };

        // before the loop: what the turns before the first would have asked for
        constexpr int EARLY = (KS >= 2 ? 2 : KS);
#pragma unroll
        for (int i = 0; i < LPW; i++)
            if (i < share(EARLY)) issue_load(STAGES - 1, STAGES - 1, i);
        wait_vmcnt<LPW*(STAGES - 2) + share(EARLY)>();
        wait_lgkmcnt<0>();  // (kernel arguments)
        asm volatile("s_barrier" ::: "memory");
        static_for<2>([&](auto g) {
            constexpr int G = decltype(g)::value;
            static_for<FRAGMENTS>([&](auto f) { ask(g, std::integral_constant<int, G % KS>{}, f, stage_of(G / KS)); });
        });
        __builtin_amdgcn_sched_barrier(0);
        for (int t = 0; t < n_tiles; t += TILES_A_TURN) {
            static_for<SETS>([&](auto g) {
                constexpr int G = decltype(g)::value, S = G % KS;
                const int tile = t + G / KS;
                if (TILES_A_TURN > 1 && tile >= n_tiles) return;  // an odd count of tiles: the turn's second half falls away
                if constexpr (S == KS - 2) {
                    // the next tile has landed in every wave, and every wave has all its fragments of this one
                    wait_vmcnt<LPW*(STAGES - 2)>();
                    fragments_landed<0>(a[G][0]);
                    asm volatile("s_barrier" ::: "memory");
                } else {
                    fragments_landed<FRAGMENTS>(a[G][0]);  // the reads of the step after this one may still travel
                }
                static_for<FM>([&](auto i) { if constexpr (decltype(i)::value > 0) and_this_one(a[G][decltype(i)::value]); });
                static_for<FN>([&](auto j) { and_this_one(w[G][decltype(j)::value]); });
                __builtin_amdgcn_sched_barrier(0);
                constexpr int NEXT = G + 2, NEXT_SET = NEXT % SETS, NEXT_STEP = NEXT % KS;
                const unsigned next_stage = stage_of(t + NEXT / KS);
                // after the barrier of tile u: tile u + STAGES into the stage of tile u; before it: the rest of the tile before
                constexpr int E = S >= KS - 2 ? S - (KS - 2) : S + 2;
                const int load_into = S >= KS - 2 ? tile : tile - 1 + STAGES;  // (as a tile whose stage it is)
                const int load_tile = S >= KS - 2 ? tile + STAGES : tile - 1 + STAGES;
                static_for<PRODUCTS>([&](auto p) {
                    constexpr int P = decltype(p)::value, J = P / FM, I = P % FM;
                    acc[J][I] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8*>(&w[G][J]), *reinterpret_cast<bf16x8*>(&a[G][I]), acc[J][I], 0, 0, 0);
                    static_for<(P + 1) * FRAGMENTS / PRODUCTS - P * FRAGMENTS / PRODUCTS>([&](auto f) {
                        ask(std::integral_constant<int, NEXT_SET>{}, std::integral_constant<int, NEXT_STEP>{},
                            std::integral_constant<int, P * FRAGMENTS / PRODUCTS + decltype(f)::value>{}, next_stage);
                    });
                    constexpr int COUNT = share(E + 1) - share(E);
                    static_for<(P + 1) * COUNT / PRODUCTS - P * COUNT / PRODUCTS>([&](auto l) {
                        issue_load(load_tile, load_into % STAGES, share(E) + P * COUNT / PRODUCTS + decltype(l)::value);
                    });
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        }
        // the fragments asked for last are never used, but on their way into registers that must not be given away yet
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        static_for<SETS>([&](auto g) {
            static_for<FM>([&](auto i) { still_written(a[decltype(g)::value][decltype(i)::value]); });
            static_for<FN>([&](auto j) { still_written(w[decltype(g)::value][decltype(j)::value]); });
        });
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
    // 'where' the wave's columns go: 0 rows of out [M, N]; a fused q/k/v projection: 1 all of them q columns (rows of out
    // [M, q_width]), 2 all of them key columns or all of them value columns (into the cache pages), 3 some of each.
    auto leave = [&](auto kind, auto where) {
        constexpr int KIND = decltype(kind)::value, WHERE = decltype(where)::value;
        constexpr bool SCATTERED = WHERE != 0;
        // where a lane's piece goes: q columns to out [M, q_width], key and value columns into the cache page at the
        // row's slot (a piece lies inside one head: the head size is a multiple of 8)
        const int row_stride = SCATTERED ? scatter.q_width : N;
        OutT* out_lane = out + (size_t)m_lane * row_stride + n_lane;
        // A piece in the cache lies at page * (bytes of a page) + ((head << page_shift) + offset) * (bytes of a row) + the
        // piece's place in the row: all but page and offset is the lane's own constant.
        bool to_cache = false;
        unsigned char* pages = nullptr;
        unsigned row_bytes = 0, page_bytes = 0;
        if constexpr (WHERE >= 2) {
            to_cache = n_lane >= scatter.q_width;
            int c = n_lane - scatter.q_width;
            pages = (unsigned char*)(c < scatter.kv_width ? scatter.k_pages : scatter.v_pages);
            if (c >= scatter.kv_width) c -= scatter.kv_width;
            row_bytes = scatter.head_size * (int)sizeof(OutT);
            page_bytes = (scatter.n_kv_heads * row_bytes) << scatter.page_shift;
            pages += (size_t)((c / scatter.head_size) << scatter.page_shift) * row_bytes + (c % scatter.head_size) * sizeof(OutT);
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
                if constexpr (WHERE >= 2) {
                    if (WHERE == 2 || to_cache) {
                        const int slot = early_slot[i][r];
                        if (slot < 0) continue;
                        const unsigned page = slot >> scatter.page_shift, offset = slot & ((1 << scatter.page_shift) - 1);
                        *reinterpret_cast<Vec16*>(pages + (size_t)page * page_bytes + offset * row_bytes) = v;
                        continue;
                    }
                }
                if constexpr (WITH_RESIDUAL && !SCATTERED) {
                    f32x4 sum = *reinterpret_cast<f32x4*>(&v);
                    sum = early_residual[i][r] + sum;   // zeros where there is no residual
                    v = *reinterpret_cast<Vec16*>(&sum);
                }
                *reinterpret_cast<Vec16*>(out_lane + (size_t)row * row_stride) = v;
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
    };
    using std::integral_constant;
    if constexpr (CAN_SCATTER) {
        if (scatter.enabled) {  // (a q/k/v projection has no activation)
            const int first = n_wave - scatter.q_width, last = min(n_wave + WN, N) - 1 - scatter.q_width;
            if (last < 0) leave(integral_constant<int, MLLM_EPI_NONE>{}, integral_constant<int, 1>{});
            else if (first >= 0 && first / scatter.kv_width == last / scatter.kv_width) leave(integral_constant<int, MLLM_EPI_NONE>{}, integral_constant<int, 2>{});
            else leave(integral_constant<int, MLLM_EPI_NONE>{}, integral_constant<int, 3>{});
            return;
        }
    }
    if (epilogue == MLLM_EPI_GELU_TANH) leave(integral_constant<int, MLLM_EPI_GELU_TANH>{}, integral_constant<int, 0>{});
    else if (epilogue == MLLM_EPI_GELU_ERF) leave(integral_constant<int, MLLM_EPI_GELU_ERF>{}, integral_constant<int, 0>{});
    else leave(integral_constant<int, MLLM_EPI_NONE>{}, integral_constant<int, 0>{});
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
    const XcdTiles places = place_tiles(ceil_div(M, BM), ceil_div(N, BN), BM, BN);
    mllm_count_kernel(MLLM_K_GEMM_STREAM);
    gemm_stream_kernel<OutT, BM, BN, WAVES_M, WAVES_N, WAVES_K, STAGES><<<8 * places.wide * places.high * k_blocks, 64 * NW, LDS_BYTES, stream>>>(
        a, w, bias, residual, o, M, N, K, epilogue, scatter, k_per_block, places);
}

// Whether the product takes this kernel: bfloat16 with a packed W, whole tiles of K, whole 16-byte pieces of output
// columns, more rows than the kernel for few rows takes (from 65 rows on this one is the faster, half-empty tile or not),
// an A whose bytes a 32-bit offset reaches; a fused q/k/v projection only
// where a piece stays inside one head.
inline bool takes(int M, int N, int K, bool packed, const CacheScatter& scatter, size_t out_element) {
    if (!packed || K % 64 != 0 || K < 64 || N % 8 != 0 || M <= 64 || ceil_div(M, 128) > 65535) return false;
    if ((long long)M * K * 2 >= (1LL << 32)) return false;
    if (scatter.enabled && (out_element != 2 || scatter.head_size % 8 != 0 || scatter.q_width % 8 != 0 || scatter.kv_width % 8 != 0)) return false;
    if (scatter.enabled && (((long long)scatter.n_kv_heads * scatter.head_size * 2) << scatter.page_shift) >= (1LL << 31)) return false;  // a page's bytes in 32 bits
    return true;
}

// The tile is chosen by what the busiest compute unit has to do: every block keeps a compute unit to itself (its
// stages fill most of the LDS), so the blocks run in rounds of 256, and a round costs what a tile of K costs the block
// (measured at GPT-2's three widths, 512 to 4,096 rows: 0.57 us at 128 x 192, 0.45 at 128 x 128, 0.70 at 256 x 128,
// 0.30 at 128 x 64). Wide tiles win where they still fill a round; narrow outputs take 128 x 64, with two waves
// sharing each 64 x 64 tile along K and a fourth stage where K is long.
template <typename OutT>
void dispatch(const bf16_t* a, const bf16_t* w, const float* bias, const float* residual, OutT* o, int M, int N, int K, int epilogue,
             hipStream_t stream, CacheScatter scatter, int k_blocks) {
#define MLLM_STREAM(BM, BN, WM_, WN_, WK_, ST) launch<OutT, BM, BN, WM_, WN_, WK_, ST>(a, w, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks)
    struct Choice {
        int bm, bn;
        float tile_us;
    };
    static const Choice choices[4] = {{128, 192, 0.57f}, {256, 128, 0.70f}, {128, 128, 0.45f}, {128, 64, 0.30f}};
    int best = 0;
    float best_cost = 0.0f;
    for (int c = 0; c < 4; c++) {
        const long blocks = (long)ceil_div(M, choices[c].bm) * ceil_div(N, choices[c].bn) * k_blocks;
        const float cost = (float)((blocks + 255) / 256) * choices[c].tile_us;
        if (c == 0 || cost < best_cost) best = c, best_cost = cost;  // (equal costs: the wider tile, which reads less)
    }
    // 256 x 256 (four waves of 128 x 128; the LDS holds two stages of it) brings a compute unit 40k outputs a microsecond
    // and tile of K where the others bring 30k, but only in full rounds of at least 150 blocks: from 2,048 x 6,400 on.
    // Measured against the choice among the others (whose costs above are those of smaller products: at these sizes
    // they take 1.45 times as long), on one machine in one run: 2,048 x 6,400 x 1,600 52 against 59 us (as a layer's up
    // product with its GELU 52.5 against 56.2), 8,192 x 4,096 x 1,024 74 against 85, 8,192 x 6,400 x 1,600 186 against 194;
    // but 2,048 x 4,096 x 1,024 (128 blocks) 30.7 against 23.2. (Machines of this kind differ by a tenth between them:
    // another one took 45.2 and 52.4 us for the first of these.)
    // (Only with bfloat16 out, which is what the products of that size write: with 32-bit out and a residual asked for
    // before the loop, a lane's 256 sums and 256 residual values do not fit its registers.)
    if constexpr (sizeof(OutT) == 2) {
        const long large = (long)ceil_div(M, 256) * ceil_div(N, 256), rounds = (large + 255) / 256;
        if (k_blocks == 1 && large >= 150 && large * 10 >= rounds * 256 * 7 && (float)rounds * 1.6f < best_cost * 1.45f) {
            MLLM_STREAM(256, 256, 2, 2, 1, 2);
            return;
        }
    }
    if (best == 0) MLLM_STREAM(128, 192, 2, 2, 1, 3);
    else if (best == 1) MLLM_STREAM(256, 128, 4, 2, 1, 3);
    else if (best == 2) MLLM_STREAM(128, 128, 2, 2, 1, 3);
    else if (K / k_blocks >= 1536) MLLM_STREAM(128, 64, 2, 1, 2, 4);
    else MLLM_STREAM(128, 64, 2, 2, 1, 3);
#undef MLLM_STREAM
}

}  // namespace stream
