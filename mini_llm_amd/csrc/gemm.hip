// Matrix products on the matrix cores: out[M,N] = act(A[M,K] . W[N,K]^T + bias[N]) (+ residual).
//
// W is [out, in], either row-major (rows contiguous in K: what the tied head's token table
// already is) or in the packed layout (common.h), which the weights of the layers are kept in. 32-bit inputs use the 32-bit MFMA (no reduced-precision
// matrix mode); bfloat16 inputs use the bf16 MFMA; sums are 32-bit in both. Replaces the
// reference's mult_kernel + add_bias + gelu + vector_addition (engine/src/matrixmult.cu:7-34,
// linear.cu:9-18) and its epilogue order sum -> +bias -> activation -> residual + that
// (engine/include/matvec_common.h:40-54).
#include "common.h"
#include "no_alloc.h"

#include <mutex>

namespace {

// For a fused q/k/v projection whose key and value columns go straight into the cache pages
// ([num_pages, n_kv_heads, page_size, head_size]) instead of the output matrix.
struct CacheScatter {
    void* k_pages;
    void* v_pages;
    const int* slots;  // per row: page * page_size + offset, negative = padding row
    int q_width, kv_width, n_kv_heads, head_size, page_shift;
    int enabled;
};

template <typename T>
struct Tile;
template <>
struct Tile<float> {
    static constexpr int BK = 32;   // k elements per LDS tile
    static constexpr int VEC = 4;   // elements per 16-byte vector
    static constexpr int PAD = 4;
};
template <>
struct Tile<bf16_t> {
    static constexpr int BK = 64;
    static constexpr int VEC = 8;
    static constexpr int PAD = 8;
};

}  // namespace

#include "gemm_stream.h"

namespace {

// One 16-byte piece of a row. With ALIGNED (K a multiple of VEC, so every row starts on a
// 16-byte boundary and a piece is whole or absent) the load is unconditional from a clamped
// address; whether the piece lies inside the matrix is returned in `valid` and applied later,
// when the piece goes to LDS (mask_piece). Nothing then depends on a load until the tile is
// staged, so all loads of two tiles stay in flight. Otherwise (unaligned K) the piece is gathered
// element by element, zero where the matrix ends.
// k_end: where the block's part of K ends (K itself unless several blocks share a tile along K).
template <typename T, bool ALIGNED>
__device__ __forceinline__ Vec16 load_piece(const T* __restrict__ base, int row, int n_rows, int k, int K, int k_end, bool& valid) {
    constexpr int VEC = Tile<T>::VEC;
    if constexpr (ALIGNED) {
        valid = row < n_rows && k < k_end;
        int safe_row = min(row, n_rows - 1), safe_k = min(k, K - VEC);
        return *reinterpret_cast<const Vec16*>(base + (size_t)safe_row * K + safe_k);
    } else {
        valid = true;
        Vec16 v = {{0u, 0u, 0u, 0u}};
        if (row >= n_rows || k >= k_end) return v;
        const T* p = base + (size_t)row * K + k;
        T* e = reinterpret_cast<T*>(&v);
#pragma unroll
        for (int i = 0; i < VEC; i++)
            if (k + i < k_end) e[i] = p[i];
        return v;
    }
}

__device__ __forceinline__ Vec16 mask_piece(Vec16 v, bool valid) {
    uint32_t mask = valid ? 0xffffffffu : 0u;
    return Vec16{{v.w[0] & mask, v.w[1] & mask, v.w[2] & mask, v.w[3] & mask}};
}

// Block tile BM x BN, 4 waves laid out WAVES_M x WAVES_N, each wave TM x TN tiles of 32x32.
// Tiles of A and W go memory -> registers -> LDS; the loads run two tiles ahead of the products
// (two register sets used in turn), so that one block per compute unit still hides the memory
// latency: these products are small enough that the grid often is no more than that.
// BEST: the block leaves no sums but, per row, the best (sum, column) of each of its waves (BestOfColumns).
template <typename T, typename OutT, int BM, int BN, int WAVES_M, int WAVES_N, bool ALIGNED, bool PACKED, bool BEST = false>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_kernel(const T* __restrict__ A, const T* __restrict__ W,
                                                   const float* __restrict__ bias,
                                                   const float* __restrict__ residual,
                                                   OutT* __restrict__ out, int M, int N, int K,
                                                   int epilogue, CacheScatter scatter, int k_per_block,
                                                   BestOfColumns best_out = BestOfColumns{}) {
    constexpr int BK = Tile<T>::BK, VEC = Tile<T>::VEC, PAD = Tile<T>::PAD;
    constexpr int LDK = BK + PAD;
    constexpr int TM = BM / WAVES_M / 32, TN = BN / WAVES_N / 32;
    constexpr int VPR = BK / VEC;  // 16-byte pieces per tile row
    constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    constexpr int A_PIECES = (BM * VPR + THREADS - 1) / THREADS, W_PIECES = (BN * VPR + THREADS - 1) / THREADS;
    constexpr int KC = 4 * VEC, CHUNKS_K = BK / KC;  // packed W: columns of a chunk, chunks along k in a tile
    static_assert(TM >= 1 && TN >= 1 && BN % 16 == 0 && BK % KC == 0, "tile layout");
    const int w_row_tiles = ceil_div(N, 16), w_k_steps = packed_k_steps<T>(K);

    __shared__ __attribute__((aligned(16))) T a_tiles[2][BM * LDK];  // two buffers: one is read while
    __shared__ __attribute__((aligned(16))) T w_tiles[2][BN * LDK];  // the next tile is written to the other

    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int half = lane / 32, lane32 = lane % 32;
    // The block's part of K: all of it, or, when several blocks share the tile (gridDim.z), a run
    // of k_per_block (a multiple of two LDS tiles), whose sums go to matrix blockIdx.z of `out`
    // (partial products: the caller passes no bias, residual or epilogue).
    const int k_begin = blockIdx.z * k_per_block, k_end = min(K, k_begin + k_per_block);
    out += (size_t)blockIdx.z * M * N;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // The residual rows of this lane's outputs are asked for now and arrive while the products
    // run: asked for in the epilogue, every block would wait for them at the same time, with
    // nothing left to overlap the trip with.
    float early_residual[TM][TN][16];
    float early_bias[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        int col = n0 + wave_n * TN * 32 + j * 32 + lane32;
        early_bias[j] = bias && col < N ? bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                int row = m0 + wave_m * TM * 32 + i * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                early_residual[i][j][v] = residual && row < M && col < N ? residual[(size_t)row * N + col] : 0.0f;
            }
    }

    Vec16 a_regs[2][A_PIECES], w_regs[2][W_PIECES];
    bool a_valid[2][A_PIECES], w_valid[2][W_PIECES];
    auto fetch = [&](int set, int k0) {
#pragma unroll
        for (int i = 0; i < A_PIECES; i++) {
            int piece = tid + i * THREADS;
            if (BM * VPR % THREADS == 0 || piece < BM * VPR) a_regs[set][i] = load_piece<T, ALIGNED>(A, m0 + piece / VPR, M, k0 + (piece % VPR) * VEC, K, k_end, a_valid[set][i]);
        }
#pragma unroll
        for (int i = 0; i < W_PIECES; i++) {
            int piece = tid + i * THREADS;
            if (BN * VPR % THREADS == 0 || piece < BN * VPR) {
                if constexpr (PACKED) {
                    // 64 consecutive pieces are one chunk: 1 KiB of contiguous memory
                    int chunk = piece / 64, row_tile = n0 / 16 + chunk / CHUNKS_K, k_step = k0 / KC + chunk % CHUNKS_K;
                    w_valid[set][i] = row_tile < w_row_tiles && k_step * KC < k_end;  // k_end is K or a multiple of the chunk
                    w_regs[set][i] = *reinterpret_cast<const Vec16*>(W + packed_offset<T>(min(row_tile, w_row_tiles - 1), min(k_step, w_k_steps - 1), w_k_steps, piece % 64));
                } else {
                    w_regs[set][i] = load_piece<T, ALIGNED>(W, n0 + piece / VPR, N, k0 + (piece % VPR) * VEC, K, k_end, w_valid[set][i]);
                }
            }
        }
    };
    auto stage = [&](int set) {  // register set `set` -> LDS buffer `set`
        T* a_tile = a_tiles[set];
        T* w_tile = w_tiles[set];
#pragma unroll
        for (int i = 0; i < A_PIECES; i++) {
            int piece = tid + i * THREADS;
            if (piece < BM * VPR) *reinterpret_cast<Vec16*>(&a_tile[(piece / VPR) * LDK + (piece % VPR) * VEC]) = mask_piece(a_regs[set][i], a_valid[set][i]);
        }
#pragma unroll
        for (int i = 0; i < W_PIECES; i++) {
            int piece = tid + i * THREADS;
            if (piece < BN * VPR) {
                int row = piece / VPR, k = (piece % VPR) * VEC;
                if constexpr (PACKED) {
                    int chunk = piece / 64, l = piece % 64;
                    row = (chunk / CHUNKS_K) * 16 + l % 16, k = (chunk % CHUNKS_K) * KC + (l / 16) * VEC;
                }
                *reinterpret_cast<Vec16*>(&w_tile[row * LDK + k]) = mask_piece(w_regs[set][i], w_valid[set][i]);
            }
        }
    };
    auto products = [&](int buffer) {
        const T* a_tile = a_tiles[buffer];
        const T* w_tile = w_tiles[buffer];
        if constexpr (sizeof(T) == 2) {
#pragma unroll
            for (int kk = 0; kk < BK / 16; kk++) {
                bf16x8 a[TM], b[TN];
#pragma unroll
                for (int i = 0; i < TM; i++)
                    a[i] = *reinterpret_cast<const bf16x8*>(
                        &a_tile[(wave_m * TM * 32 + i * 32 + lane32) * LDK + kk * 16 + half * 8]);
#pragma unroll
                for (int j = 0; j < TN; j++)
                    b[j] = *reinterpret_cast<const bf16x8*>(
                        &w_tile[(wave_n * TN * 32 + j * 32 + lane32) * LDK + kk * 16 + half * 8]);
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
            }
        } else {
            // A lane takes four consecutive k of its row; component c of every lane forms the
            // k pair of one 32x32x2 product, the same pairing on both operands.
#pragma unroll
            for (int kk = 0; kk < BK / 8; kk++) {
                f32x4 a[TM], b[TN];
#pragma unroll
                for (int i = 0; i < TM; i++)
                    a[i] = *reinterpret_cast<const f32x4*>(
                        &a_tile[(wave_m * TM * 32 + i * 32 + lane32) * LDK + kk * 8 + half * 4]);
#pragma unroll
                for (int j = 0; j < TN; j++)
                    b[j] = *reinterpret_cast<const f32x4*>(
                        &w_tile[(wave_n * TN * 32 + j * 32 + lane32) * LDK + kk * 8 + half * 4]);
#pragma unroll
                for (int c = 0; c < 4; c++)
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][c], b[j][c], acc[i][j], 0, 0, 0);
            }
        }
    };

    // Every fetch is unconditional (beyond K it reads a clamped address and is masked away): with
    // no branch around the loads, the wait before a tile is staged counts exactly the loads of the
    // other set that may still be in flight. One barrier a tile: while buffer b is multiplied, the
    // next tile goes into buffer 1-b, which every wave left before the barrier above.
    fetch(0, k_begin);
    fetch(1, k_begin + BK);
    stage(0);
    fetch(0, k_begin + 2 * BK);
    __syncthreads();
    for (int k0 = k_begin; k0 < k_end; k0 += 2 * BK) {
        stage(1);  // tile k0 + BK (zeros beyond K)
        fetch(1, k0 + 3 * BK);
        products(0);
        __syncthreads();
        stage(0);  // tile k0 + 2 BK
        fetch(0, k0 + 4 * BK);
        products(1);
        __syncthreads();
    }

    // A lane holds column lane%32 and rows 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 tile.
    if constexpr (BEST) {
        // Per row the best of this block's columns. The sums go to LDS as a [BM, BN] matrix (the tiles' memory: every
        // wave has left the loop behind the last barrier); then the THREADS / BM threads next to each other that share
        // a row take BN / that many columns each and settle the rest among themselves with data-parallel steps
        // inside a row of 16 lanes. (Reducing in the layout of the accumulators, where a row's 32 columns lie in 32
        // lanes, took 160 trips through the LDS crossbar a tile: the head got slower than with its logits written.)
        constexpr int SHARE = THREADS / BM, COLS = BN / SHARE;   // threads a row, columns a thread
        static_assert(SHARE >= 1 && SHARE <= 16 && (SHARE & (SHARE - 1)) == 0 && BN % SHARE == 0 && COLS % 4 == 0, "a row's threads lie in one row of 16 lanes");
        constexpr bool IN_W = sizeof(w_tiles) >= sizeof(float) * BM * BN;
        static_assert(IN_W || sizeof(a_tiles) >= sizeof(float) * BM * BN, "room for the block's sums");
        float* sums = IN_W ? reinterpret_cast<float*>(&w_tiles[0][0]) : reinterpret_cast<float*>(&a_tiles[0][0]);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int local_from = wave_m * TM * 32 + i * 32 + 8 * (v / 4);  // the same for the whole wave
                if (m0 + local_from >= M) continue;
                const int local_row = local_from + 4 * half + (v % 4);
#pragma unroll
                for (int j = 0; j < TN; j++) sums[local_row * BN + wave_n * TN * 32 + j * 32 + lane32] = acc[i][j][v] + early_bias[j];
            }
        __syncthreads();
        const int local_row = tid / SHARE, share = tid % SHARE;
        float best = -INFINITY;
        int best_index = 0x7fffffff;
        if (m0 + local_row < M) {   // (whole rows of 16 lanes go one way: SHARE divides 16)
#pragma unroll
            for (int c0 = 0; c0 < COLS; c0 += 4) {
                const f32x4 four = *reinterpret_cast<const f32x4*>(&sums[local_row * BN + share * COLS + c0]);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int col = n0 + share * COLS + c0 + e;
                    if (col < N && beats(four[e], col, best, best_index)) {
                        best = four[e];
                        best_index = col;
                    }
                }
            }
        }
        auto meet = [&](float other, int other_index) {
            if (beats(other, other_index, best, best_index)) {
                best = other;
                best_index = other_index;
            }
        };
        if constexpr (SHARE >= 2) meet(dpp_moved<0xB1>(best), __builtin_amdgcn_update_dpp(0, best_index, 0xB1, 0xf, 0xf, false));
        if constexpr (SHARE >= 4) meet(dpp_moved<0x4E>(best), __builtin_amdgcn_update_dpp(0, best_index, 0x4E, 0xf, 0xf, false));
        if constexpr (SHARE >= 8) meet(dpp_moved<0x141>(best), __builtin_amdgcn_update_dpp(0, best_index, 0x141, 0xf, 0xf, false));
        if constexpr (SHARE >= 16) meet(dpp_moved<0x140>(best), __builtin_amdgcn_update_dpp(0, best_index, 0x140, 0xf, 0xf, false));
        if (share == 0 && m0 + local_row < M) {
            size_t at = (size_t)(m0 + local_row) * best_out.per_row + blockIdx.x;
            best_out.values[at] = best;
            best_out.indices[at] = best_index;
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            int col = n0 + wave_n * TN * 32 + j * 32 + lane32;
            if (col >= N) continue;
            float b = early_bias[j];
            if (scatter.enabled) {
                // a fused q/k/v projection: the q columns go to out [M, q_width], this lane's key or
                // value column into the cache pages at the rows' slots
                OutT* pages = nullptr;
                int kv_head = 0, d = 0;
                if (col >= scatter.q_width) {
                    int c = col - scatter.q_width;
                    pages = (OutT*)(c < scatter.kv_width ? scatter.k_pages : scatter.v_pages);
                    if (c >= scatter.kv_width) c -= scatter.kv_width;
                    kv_head = c / scatter.head_size, d = c % scatter.head_size;
                }
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    int row = m0 + wave_m * TM * 32 + i * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                    if (row >= M) continue;
                    OutT value = from_float<OutT>(acc[i][j][v] + b);
                    if (pages == nullptr) {
                        out[(size_t)row * scatter.q_width + col] = value;
                    } else {
                        int slot = scatter.slots[row];
                        if (slot < 0) continue;
                        int page = slot >> scatter.page_shift, offset = slot & ((1 << scatter.page_shift) - 1);
                        pages[((((size_t)page * scatter.n_kv_heads + kv_head) << scatter.page_shift) + offset) * scatter.head_size + d] = value;
                    }
                }
                continue;
            }
#pragma unroll
            for (int v = 0; v < 16; v++) {
                int row = m0 + wave_m * TM * 32 + i * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                if (row >= M) continue;
                float value = acc[i][j][v] + b;
                if (epilogue == MLLM_EPI_GELU_TANH) value = sizeof(OutT) == 2 ? gelu_tanh_for_bf16(value) : gelu_tanh(value);
                else if (epilogue == MLLM_EPI_GELU_ERF) value = sizeof(OutT) == 2 ? gelu_erf_for_bf16(value) : gelu_erf(value);
                size_t at = (size_t)row * N + col;
                if (residual) value = early_residual[i][j][v] + value;
                out[at] = from_float<OutT>(value);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Few rows (decoding, short portions): M <= 64. The product is bound by reading W once, so the
// work is cut along N and K, not M: a block owns 16 output columns, its waves take turns along
// K, and W streams straight from memory into MFMA operands (a lane loads 16 bytes of one of the
// 16 rows; the x rows of the same k come through the cache). out^T = W . x^T, so that W is the
// 16-row operand. The waves' partial sums meet in LDS, where the epilogue runs.
// ------------------------------------------------------------------------------------------------
template <typename T, typename OutT, int MT, int KSPLIT, bool PACKED>
__global__ __launch_bounds__(64 * KSPLIT) void gemm_skinny_kernel(
    const T* __restrict__ A, const T* __restrict__ W, const float* __restrict__ bias,
    const float* __restrict__ residual, OutT* __restrict__ out, int M, int N, int K, int epilogue,
    CacheScatter scatter, int steps_per_block, int x_packed, int out_packed) {
    constexpr int VEC = Tile<T>::VEC;
    constexpr int KSTEP = 4 * VEC;  // k covered by one load of the wave: 4 lane groups x 16 bytes
    // Loads in flight per wave before any is used. At decode sizes a wave's whole share of K fits
    // in one round (768 / 4 waves = 6 steps), and the kernel waits for memory once.
    constexpr int UNROLL = MT == 1 ? 8 : 4;
    __shared__ float sums[KSPLIT][MT * 4][WAVE];

    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int row16 = lane % 16, quad = lane / 16;
    const int n0 = blockIdx.x * 16;
    const int n = n0 + row16;
    const bool n_valid = n < N;
    const T* w_row = W + (size_t)(n_valid ? n : 0) * K;

    f32x4 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) acc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // Where this lane's piece of k-step s of row tile i lies: x_base[i] + min(s * x_stride + x_lane,
    // x_limit), whether the rows of x are row-major or in the packed layout (x_packed: row tile i's
    // chunk of a k-step is then the operand as it lies in memory; from row-major rows the same load
    // touches 16 cache lines, and those loads are what a product of 48-64 rows spends most of its
    // time on). Nothing inside the loop depends on which of the two it is.
    const int n_steps = (K + KSTEP - 1) / KSTEP;
    const int x_stride = x_packed ? 64 * VEC : KSTEP;
    const int x_lane = x_packed ? lane * VEC : quad * VEC;
    const int x_limit = x_packed ? ((n_steps - 1) * 64 + lane) * VEC : K - VEC;
    const T* x_base[MT];
    bool x_valid[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) {
        int t = i * 16 + row16;
        x_valid[i] = t < M;
        // the packed matrix has (M + 15) / 16 row tiles, the kernel up to MT
        x_base[i] = x_packed ? A + (size_t)min(i, (M - 1) / 16) * n_steps * (64 * VEC) : A + (size_t)(x_valid[i] ? t : 0) * K;
    }

    // What the epilogue will want from memory for this thread's outputs (bias, residual, the cache
    // slot of a key or value row) is asked for now and arrives while the products run: asked for in
    // the epilogue it would be one more trip to memory at the end of a kernel that is a few long.
    constexpr int ITEMS = (MT * 4 * WAVE + WAVE * KSPLIT - 1) / (WAVE * KSPLIT);  // outputs a thread finishes
    constexpr bool EARLY = MT < 4;  // with four row tiles the registers are better left to the loads of x
    float early_bias[ITEMS], early_residual[ITEMS];
    int early_slot[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; j++) {
        int index = threadIdx.x + j * WAVE * KSPLIT;
        int l = index % WAVE, ir = index / WAVE;
        int token = (ir / 4) * 16 + l % 16;
        int col = n0 + 4 * (l / 16) + ir % 4;
        bool wanted = EARLY && index < MT * 4 * WAVE && token < M && col < N;
        early_bias[j] = bias && wanted ? bias[col] : 0.0f;
        early_residual[j] = residual && wanted && !scatter.enabled ? residual[(size_t)token * N + col] : 0.0f;
        early_slot[j] = scatter.enabled && wanted && col >= scatter.q_width ? scatter.slots[token] : -1;
    }

    // The block takes the k-steps first_step .. last_step-1: all of them, or, when the launch has
    // several blocks per 16 columns (gridDim.y), its part of K, whose sums then go to matrix
    // blockIdx.y of `out` (partial products; the caller passes no bias, residual or epilogue).
    // Wave w takes the steps in groups of UNROLL, every KSPLIT-th group.
    const int first_step = blockIdx.y * steps_per_block;
    const int last_step = min(n_steps, first_step + steps_per_block);
    out += (size_t)blockIdx.y * M * N;
    for (int step0 = first_step + wave * UNROLL; step0 < last_step; step0 += KSPLIT * UNROLL) {
        Vec16 w_piece[UNROLL], x_piece[UNROLL][MT];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            int k = (step0 + u) * KSTEP + quad * VEC;  // K is a multiple of VEC: a piece is whole or absent
            int safe_k = min(k, K - VEC);  // loads are unconditional, from a clamped address: no branch between them
            if constexpr (PACKED)  // a chunk of the packed layout is this wave's operand as it lies in memory
                w_piece[u] = *reinterpret_cast<const Vec16*>(W + packed_offset<T>(blockIdx.x, min(step0 + u, n_steps - 1), n_steps, lane));
            else
                w_piece[u] = *reinterpret_cast<const Vec16*>(w_row + safe_k);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                if constexpr (MT >= 4)  // measured: with four row tiles the two forms written out are faster (47 -> 54 k tokens/s at 64 rows in 32-bit), with one the common form (10.4 -> 11.9 k at 8 rows)
                    x_piece[u][i] = *reinterpret_cast<const Vec16*>(
                        x_packed ? A + packed_offset<T>(min(i, (M - 1) / 16), min(step0 + u, n_steps - 1), n_steps, lane)
                                 : A + (size_t)(x_valid[i] ? i * 16 + row16 : 0) * K + safe_k);
                else
                    x_piece[u][i] = *reinterpret_cast<const Vec16*>(x_base[i] + min((step0 + u) * x_stride + x_lane, x_limit));
            }
        }
        // what lies outside the matrices is zeroed only now, so that nothing above waits for a load
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            bool k_valid = (step0 + u) * KSTEP + quad * VEC < K && step0 + u < last_step;
            w_piece[u] = mask_piece(w_piece[u], k_valid && n_valid);
#pragma unroll
            for (int i = 0; i < MT; i++) x_piece[u][i] = mask_piece(x_piece[u][i], k_valid && x_valid[i]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            if constexpr (sizeof(T) == 2) {
                bf16x8 a = *reinterpret_cast<bf16x8*>(&w_piece[u]);
#pragma unroll
                for (int i = 0; i < MT; i++)
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, *reinterpret_cast<bf16x8*>(&x_piece[u][i]), acc[i], 0, 0, 0);
            } else {
                f32x4 a = *reinterpret_cast<f32x4*>(&w_piece[u]);
#pragma unroll
                for (int c = 0; c < 4; c++)
#pragma unroll
                    for (int i = 0; i < MT; i++)
                        acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[c], (*reinterpret_cast<f32x4*>(&x_piece[u][i]))[c], acc[i], 0, 0, 0);
            }
        }
    }

    // acc[i][r] is out[token i*16 + lane%16][column n0 + 4*(lane/16) + r]
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int r = 0; r < 4; r++) sums[wave][i * 4 + r][lane] = acc[i][r];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < ITEMS; j++) {
        int index = threadIdx.x + j * WAVE * KSPLIT;
        if (index >= MT * 4 * WAVE) continue;
        int l = index % WAVE, ir = index / WAVE;
        int token = (ir / 4) * 16 + l % 16;
        int col = n0 + 4 * (l / 16) + ir % 4;
        if (token >= M || col >= N) continue;
        float value = 0.0f;
#pragma unroll
        for (int w = 0; w < KSPLIT; w++) value += sums[w][ir][l];  // the same order for every element
        if (bias) value += EARLY ? early_bias[j] : bias[col];
        if (epilogue == MLLM_EPI_GELU_TANH) value = sizeof(OutT) == 2 ? gelu_tanh_for_bf16(value) : gelu_tanh(value);
        else if (epilogue == MLLM_EPI_GELU_ERF) value = sizeof(OutT) == 2 ? gelu_erf_for_bf16(value) : gelu_erf(value);
        if (scatter.enabled) {
            if (col < scatter.q_width) {
                out[(size_t)token * scatter.q_width + col] = from_float<OutT>(value);
            } else {
                int slot = EARLY ? early_slot[j] : scatter.slots[token];
                if (slot < 0) continue;
                int c = col - scatter.q_width;
                OutT* pages = (OutT*)(c < scatter.kv_width ? scatter.k_pages : scatter.v_pages);
                if (c >= scatter.kv_width) c -= scatter.kv_width;
                int kv_head = c / scatter.head_size, d = c % scatter.head_size;
                int page = slot >> scatter.page_shift, offset = slot & ((1 << scatter.page_shift) - 1);
                pages[((((size_t)page * scatter.n_kv_heads + kv_head) << scatter.page_shift) + offset) * scatter.head_size + d] = from_float<OutT>(value);
            }
            continue;
        }
        size_t at = (size_t)token * N + col;
        if (residual) value = (EARLY ? early_residual[j] : residual[at]) + value;
        out[out_packed ? packed_element<OutT>(token, col, N) : at] = from_float<OutT>(value);
    }
}

template <typename T, typename OutT, int MT>
void launch_skinny(const T* a, const T* w, bool packed, const float* bias, const float* residual, OutT* o, int M,
                   int N, int K, int epilogue, hipStream_t stream, CacheScatter scatter = CacheScatter{}, int k_blocks = 1,
                   int x_packed = 0, int out_packed = 0) {
    constexpr int KSTEP = 4 * Tile<T>::VEC;
    constexpr int UNROLL = MT == 1 ? 8 : 4;
    int tiles = ceil_div(N, 16), steps = ceil_div(K, KSTEP);
    int steps_per_block = k_blocks == 1 ? steps : ceil_div(ceil_div(steps, k_blocks), UNROLL) * UNROLL;
    int split = 1;  // waves per block, along K: enough waves to fill the chip, each with work to do
    while (split < 16 && tiles * k_blocks * split < 2048 && steps_per_block >= 8 * split) split *= 2;
    dim3 grid(tiles, k_blocks);
    mllm_count_kernel(MLLM_K_GEMM_SKINNY);
#define MLLM_SKINNY_CASE(SPLIT)                                                                                                   \
    if (packed) gemm_skinny_kernel<T, OutT, MT, SPLIT, true><<<grid, 64 * SPLIT, 0, stream>>>(a, w, bias, residual, o, M, N, K, epilogue, scatter, steps_per_block, x_packed, out_packed); \
    else gemm_skinny_kernel<T, OutT, MT, SPLIT, false><<<grid, 64 * SPLIT, 0, stream>>>(a, w, bias, residual, o, M, N, K, epilogue, scatter, steps_per_block, x_packed, out_packed);
    if (split == 16) { MLLM_SKINNY_CASE(16) }
    else if (split == 1) { MLLM_SKINNY_CASE(1) }
    else if (split == 2) { MLLM_SKINNY_CASE(2) }
    else if (split == 4) { MLLM_SKINNY_CASE(4) }
    else { MLLM_SKINNY_CASE(8) }
#undef MLLM_SKINNY_CASE
}

// Blocks along K that a product of few rows should be cut into, each leaving a partial product:
// when the columns alone leave most compute units idle (every block reads all rows of x, so a
// long K with few columns is slow however few bytes the matrix has) and every block still gets
// eight steps. It depends on N and K only.
template <typename T>
int skinny_k_blocks(int N, int K) {
    int tiles = ceil_div(N, 16), steps = ceil_div(K, 4 * Tile<T>::VEC);
    int k_blocks = 1;
    while (k_blocks < 8 && tiles * k_blocks < 256 && steps >= 16 * k_blocks) k_blocks *= 2;
    return k_blocks;
}

// The same for more rows (the tiled kernel, 128 x 64 tiles): only a product whose tiles leave half
// the compute units idle is cut, while the tiles of the cut product are no more than one and a
// half to a compute unit and every block keeps eight LDS tiles of K (measured: a product that
// nearly fills the chip gains less from the cut than adding the partial products up costs). Up to
// 256 rows a block may go down to four LDS tiles: the partial products are small then, and a
// 128 x 768 x 768 product takes 6.1 us in two cuts against 7.9 us whole (bfloat16; in 32-bit 8.6 us
// in four cuts against 12.6 us in two).
template <typename T>
int tiled_k_blocks(int M, int N, int K) {
    int tiles = ceil_div(M, 128) * ceil_div(N, 64);
    int k_blocks = 1;
    if (sizeof(T) == 4 && tiles > 128) {
        // In 32-bit the matrix cores set the pace, and a block has two waves on each of them: what counts is that every
        // compute unit gets the same number of blocks. 192 tiles (2,048 x 768) whole keep 192 units busy for a block's
        // time; cut in four along K they are 768 blocks, three to a unit, each a quarter as long: 128.7 -> 98.2 us at
        // K = 3,072, 35.8 -> 32.0 at K = 768; 400 tiles (2,048 x 1,600 x 6,400) in three 441 -> 379 us. The cost of a cut:
        // rounds of 256 blocks over the cuts, and 3 % for each further partial product that is written and read.
        int best = 1;
        float best_cost = 0.0f;
        for (int cuts = 1; cuts <= 8; cuts++) {
            if (cuts > 1 && K < 6 * Tile<T>::BK * cuts) break;   // three turns of the loop at least
            const float cost = (float)ceil_div(tiles * cuts, 256) / cuts * (1.0f + 0.03f * (cuts - 1));
            if (cuts == 1 || cost < best_cost) best = cuts, best_cost = cost;
        }
        return best;
    }
    if (tiles > 128) return 1;
    const int least_tiles = M <= 256 ? 4 : 8;
    while (k_blocks < 8 && tiles * k_blocks * 2 <= 384 && K >= least_tiles * Tile<T>::BK * k_blocks * 2) k_blocks *= 2;
    return k_blocks;
}

template <typename T, typename OutT, bool ALIGNED, int BM, int BN, int WAVES_M, int WAVES_N>
void launch_tile(const T* a, const T* w, bool packed, const float* bias, const float* residual, OutT* o, int M, int N,
                 int K, int epilogue, hipStream_t stream, CacheScatter scatter, int k_blocks) {
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM), k_blocks);
    constexpr int PAIR = 2 * Tile<T>::BK;  // the kernel's loop takes two LDS tiles a turn
    int k_per_block = k_blocks == 1 ? ceil_div(K, PAIR) * PAIR : ceil_div(ceil_div(K, k_blocks), PAIR) * PAIR;
    mllm_count_kernel(MLLM_K_GEMM_TILED);
    if (packed) gemm_kernel<T, OutT, BM, BN, WAVES_M, WAVES_N, ALIGNED, true><<<grid, 64 * WAVES_M * WAVES_N, 0, stream>>>(a, w, bias, residual, o, M, N, K, epilogue, scatter, k_per_block);
    else gemm_kernel<T, OutT, BM, BN, WAVES_M, WAVES_N, ALIGNED, false><<<grid, 64 * WAVES_M * WAVES_N, 0, stream>>>(a, w, bias, residual, o, M, N, K, epilogue, scatter, k_per_block);
}

template <typename T, typename OutT, bool ALIGNED>
void launch_tiled(const T* a, const T* w, bool packed, const float* bias, const float* residual, OutT* o, int M, int N,
                  int K, int epilogue, hipStream_t stream, CacheScatter scatter = CacheScatter{}, int k_blocks = 1) {
    if constexpr (sizeof(T) == 2) {  // bfloat16 with many rows and a packed W: the kernel that streams its operands straight into LDS
        if (ALIGNED && stream::takes(M, N, K, packed, scatter, sizeof(OutT))) {
            stream::dispatch<OutT>(a, w, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks);
            return;
        }
    }
    int tile = 0;
    {
        // measured on MI355X at GPT-2 sizes: many waves per block hide latency best; the large tile
        // (sixteen waves, half the traffic from the cache of the chip for the same product) from
        // about half a block a compute unit on, where it wins by 5 % (2,048 x 2,304 x 768) to 25 %
        // (8,192 x 4,096 x 1,024)
        if (M <= 32) tile = 1;
        else if (M <= 64) tile = 2;
        else if (k_blocks == 1 && M >= 192 && ceil_div(M, 256) * ceil_div(N, 128) >= (sizeof(T) == 4 ? 256 : 128)) tile = 3;  // 32-bit products are bound by the matrix cores: no compute unit may idle
        else if (ceil_div(M, 128) * ceil_div(N, 64) * k_blocks <= 128) tile = 2;  // half a block a compute unit or less: twice as many smaller blocks are 10 to 20 % faster in bfloat16 and a third faster in 32-bit (measured from 96 to 1,024 rows)
        else tile = 7;
    }
    switch (tile) {  // other shapes (128x128, 256x128 with eight waves, fewer waves) were measured and lost at every size here
        case 1: launch_tile<T, OutT, ALIGNED, 32, 128, 1, 4>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks); break;
        case 2: launch_tile<T, OutT, ALIGNED, 64, 64, 2, 2>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks); break;
        case 3: launch_tile<T, OutT, ALIGNED, 256, 128, 4, 4>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks); break;
        default: launch_tile<T, OutT, ALIGNED, 128, 64, 4, 2>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks); break;
    }
}

// Whether a product of M rows takes the kernel for few rows (which alone reads and writes rows in
// the packed layout): up to 64 rows, except for a very wide matrix (the head over the vocabulary),
// where a block of that kernel would read the rows again for every 16 columns and the tiled kernel
// with a short tile streams faster. The borders are measured on MI355X.
template <typename T>
bool takes_few_row_kernel(int M, int N, int K) {
    const bool aligned = K % Tile<T>::VEC == 0;
    const bool wide = N >= 8192;
    const int skinny_rows = !wide ? 64 : 0;  // over 50,257 columns the 32-row tile takes 40 us in 32-bit at 1 to 12 rows, this kernel 50 us
    return aligned && M <= skinny_rows;
}

template <typename T, typename OutT>
void launch_gemm(const void* A, const void* W, bool packed, const float* bias, const float* residual, void* out,
                 int M, int N, int K, int epilogue, int x_packed, int out_packed, hipStream_t stream) {
    const T* a = (const T*)A;
    const T* w = (const T*)W;
    OutT* o = (OutT*)out;
    if (takes_few_row_kernel<T>(M, N, K)) {
        if (M <= 16) launch_skinny<T, OutT, 1>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream, CacheScatter{}, 1, x_packed, out_packed);
        else if (M <= 32) launch_skinny<T, OutT, 2>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream, CacheScatter{}, 1, x_packed, out_packed);
        else launch_skinny<T, OutT, 4>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream, CacheScatter{}, 1, x_packed, out_packed);
    } else if (K % Tile<T>::VEC == 0) {
        launch_tiled<T, OutT, true>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream);
    } else {
        launch_tiled<T, OutT, false>(a, w, packed, bias, residual, o, M, N, K, epilogue, stream);
    }
}

}  // namespace

// 1 if a product of M rows with an [N, K] matrix takes rows in the packed layout (x_packed, out_packed).
MLLM_API int mllm_gemm_takes_packed_rows(int M, int N, int K, int in_dtype) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    if (in_dtype == MLLM_F32) return takes_few_row_kernel<float>(M, N, K) ? 1 : 0;
    if (in_dtype == MLLM_BF16) return takes_few_row_kernel<bf16_t>(M, N, K) ? 1 : 0;
    return 0;
}

// x_packed: A is in the packed layout of an [M, K] matrix; out_packed: out is written in the packed
// layout of an [M, N] matrix (no residual then). Both only where mllm_gemm_takes_packed_rows says so.
MLLM_API int mllm_gemm(const void* A, const void* W, int w_packed, const float* bias, const float* residual,
                       void* out, int M, int N, int K, int in_dtype, int out_dtype, int epilogue,
                       int x_packed, int out_packed, hipStream_t stream) {
    MLLM_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    MLLM_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm: unknown epilogue %d", epilogue);
    MLLM_REQUIRE(ceil_div(M, 32) <= 65535, "gemm: M=%d has too many row tiles", M);
    MLLM_REQUIRE((!x_packed && !out_packed) || mllm_gemm_takes_packed_rows(M, N, K, in_dtype),
                 "gemm: rows in the packed layout are for the kernel for few rows, which M=%d N=%d K=%d do not take", M, N, K);
    MLLM_REQUIRE(!out_packed || residual == nullptr, "gemm: a residual sum is not written in the packed layout");
    MLLM_REQUIRE(residual == nullptr || out_dtype == MLLM_F32, "gemm: a residual sum is 32-bit, the output asked for is not");
    if (M == 0) return 0;
    if (in_dtype == MLLM_F32 && out_dtype == MLLM_F32)
        launch_gemm<float, float>(A, W, w_packed != 0, bias, residual, out, M, N, K, epilogue, x_packed, out_packed, stream);
    else if (in_dtype == MLLM_BF16 && out_dtype == MLLM_BF16)
        launch_gemm<bf16_t, bf16_t>(A, W, w_packed != 0, bias, residual, out, M, N, K, epilogue, x_packed, out_packed, stream);
    else if (in_dtype == MLLM_BF16 && out_dtype == MLLM_F32)
        launch_gemm<bf16_t, float>(A, W, w_packed != 0, bias, residual, out, M, N, K, epilogue, x_packed, out_packed, stream);
    else
        MLLM_REQUIRE(false, "gemm: no kernel for input dtype %d with output dtype %d", in_dtype, out_dtype);
    return mllm_check_launch("gemm");
}

// The tile a product of M rows takes when it leaves the best of its columns instead of its sums
// (mllm_gemm_best): the tiles the plain product takes for a wide matrix at these row counts.
namespace {
struct BestTile { int bm, bn; };
BestTile best_tile(int M) {
    if (M <= 32) return {32, 128};
    if (M <= 64) return {64, 64};
    return {128, 64};
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N>
void launch_best(const T* a, const T* w, bool packed, const float* bias, int M, int N, int K, BestOfColumns best, hipStream_t stream) {
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM), 1);
    constexpr int PAIR = 2 * Tile<T>::BK;
    int k_per_block = ceil_div(K, PAIR) * PAIR;
    mllm_count_kernel(MLLM_K_GEMM_BEST);
    if (packed) gemm_kernel<T, float, BM, BN, WAVES_M, WAVES_N, true, true, true><<<grid, 64 * WAVES_M * WAVES_N, 0, stream>>>(a, w, bias, nullptr, nullptr, M, N, K, 0, CacheScatter{}, k_per_block, best);
    else gemm_kernel<T, float, BM, BN, WAVES_M, WAVES_N, true, false, true><<<grid, 64 * WAVES_M * WAVES_N, 0, stream>>>(a, w, bias, nullptr, nullptr, M, N, K, 0, CacheScatter{}, k_per_block, best);
}

template <typename T>
void launch_best_of(const void* A, const void* W, bool packed, const float* bias, int M, int N, int K, BestOfColumns best, hipStream_t stream) {
    if (M <= 32) launch_best<T, 32, 128, 1, 4>((const T*)A, (const T*)W, packed, bias, M, N, K, best, stream);
    else if (M <= 64) launch_best<T, 64, 64, 2, 2>((const T*)A, (const T*)W, packed, bias, M, N, K, best, stream);
    else launch_best<T, 128, 64, 4, 2>((const T*)A, (const T*)W, packed, bias, M, N, K, best, stream);
}
}  // namespace

// How many (value, column) pairs per row mllm_gemm_best leaves for a product of M rows with an
// [N, K] matrix; 0 where it does not take the sizes (K no whole number of 16-byte pieces).
MLLM_API int mllm_gemm_best_per_row(int M, int N, int K, int in_dtype) {
    if (M <= 0 || N <= 0 || K <= 0 || (in_dtype != MLLM_F32 && in_dtype != MLLM_BF16)) return 0;
    if (K % (in_dtype == MLLM_F32 ? 4 : 8)) return 0;
    return ceil_div(N, best_tile(M).bn);
}

// A . W^T (+ bias) whose sums are not written: per row, every block leaves the best
// (sum, column) of its columns in values / indices [M, per_row] (per_row as mllm_gemm_best_per_row
// says; every entry is written, an entry without a column holds -inf and the largest index). The
// best entry of a row by numpy's argmax rules is the row's argmax: the head of a greedy step,
// whose logits nobody reads (the reference takes the argmax on the device for the same reason:
// engine/src/argmax.cu).
MLLM_API int mllm_gemm_best(const void* A, const void* W, int w_packed, const float* bias, float* values, int* indices,
                            int per_row, int M, int N, int K, int in_dtype, hipStream_t stream) {
    MLLM_REQUIRE(M >= 0 && N > 0 && K > 0 && ceil_div(M, 32) <= 65535, "gemm_best: bad sizes M=%d N=%d K=%d", M, N, K);
    MLLM_REQUIRE(values != nullptr && indices != nullptr, "gemm_best: nowhere to leave the best columns");
    int expected = mllm_gemm_best_per_row(M, N, K, in_dtype);
    MLLM_REQUIRE(expected > 0, "gemm_best: no kernel for K=%d in dtype %d", K, in_dtype);
    MLLM_REQUIRE(per_row == expected, "gemm_best: %d entries per row were given room, the product leaves %d", per_row, expected);
    if (M == 0) return 0;
    BestOfColumns best{values, indices, per_row};
    if (in_dtype == MLLM_F32) launch_best_of<float>(A, W, w_packed != 0, bias, M, N, K, best, stream);
    else launch_best_of<bf16_t>(A, W, w_packed != 0, bias, M, N, K, best, stream);
    return mllm_check_launch("gemm_best");
}

// How many partial products mllm_gemm_split should be asked for at these sizes (1: the product is
// better left whole).
MLLM_API int mllm_gemm_split_blocks(int M, int N, int K, int in_dtype) {
    if (M <= 0 || N <= 0 || K <= 0) return 1;
    if (in_dtype == MLLM_F32) return K % 4 ? 1 : (M <= 64 ? skinny_k_blocks<float>(N, K) : tiled_k_blocks<float>(M, N, K));
    if (in_dtype == MLLM_BF16) return K % 8 ? 1 : (M <= 64 ? skinny_k_blocks<bf16_t>(N, K) : tiled_k_blocks<bf16_t>(M, N, K));
    return 1;
}

// A . W^T as k_blocks partial products over consecutive parts of K: partials [k_blocks, M, N] in
// 32-bit, whose sum (in any fixed order) is the product. For a long K with few output columns;
// whoever takes the partial products adds bias and residual.
MLLM_API int mllm_gemm_split(const void* A, const void* W, int w_packed, float* partials, int M, int N, int K,
                             int in_dtype, int k_blocks, int x_packed, hipStream_t stream) {
    MLLM_REQUIRE(!x_packed || M <= 64, "gemm_split: rows in the packed layout are for at most 64 rows, not %d", M);
    MLLM_REQUIRE(M >= 0 && N > 0 && K > 0 && ceil_div(M, 32) <= 65535, "gemm_split: bad sizes M=%d N=%d K=%d", M, N, K);
    MLLM_REQUIRE(k_blocks >= 1 && k_blocks <= 16, "gemm_split: %d partial products is not in 1..16", k_blocks);
    MLLM_REQUIRE(in_dtype == MLLM_F32 || in_dtype == MLLM_BF16, "gemm_split: unknown dtype %d", in_dtype);
    MLLM_REQUIRE(K % (in_dtype == MLLM_F32 ? 4 : 8) == 0, "gemm_split: K=%d is not a multiple of a 16-byte piece", K);
    if (M == 0) return 0;
#define MLLM_SPLIT_CASE(T)                                                                                                     \
    if (M <= 16) launch_skinny<T, float, 1>((const T*)A, (const T*)W, w_packed != 0, nullptr, nullptr, partials, M, N, K, 0, stream, CacheScatter{}, k_blocks, x_packed);      \
    else if (M <= 32) launch_skinny<T, float, 2>((const T*)A, (const T*)W, w_packed != 0, nullptr, nullptr, partials, M, N, K, 0, stream, CacheScatter{}, k_blocks, x_packed); \
    else if (M <= 64) launch_skinny<T, float, 4>((const T*)A, (const T*)W, w_packed != 0, nullptr, nullptr, partials, M, N, K, 0, stream, CacheScatter{}, k_blocks, x_packed); \
    else launch_tiled<T, float, true>((const T*)A, (const T*)W, w_packed != 0, nullptr, nullptr, partials, M, N, K, 0, stream, CacheScatter{}, k_blocks);
    if (in_dtype == MLLM_F32) { MLLM_SPLIT_CASE(float) } else { MLLM_SPLIT_CASE(bf16_t) }
#undef MLLM_SPLIT_CASE
    return mllm_check_launch("gemm_split");
}

// The fused q/k/v projection: q columns go to out_q [M, q_width], key and value columns straight
// into the cache pages at slots[row] (few rows: the skinny kernel; more: the tiled one)
// (what the reference's decode block does with its fused matvec: engine/src/transformer_block.cu:223-242).
MLLM_API int mllm_gemm_qkv_cache(const void* A, const void* W, int w_packed, const float* bias, void* out_q, void* k_pages,
                                 void* v_pages, const int* slots, int M, int K, int q_width, int kv_width,
                                 int n_kv_heads, int head_size, int page_size, int dtype, int x_packed, hipStream_t stream) {
    MLLM_REQUIRE(M >= 0 && ceil_div(M, 32) <= 65535, "gemm_qkv_cache: bad row count %d", M);
    MLLM_REQUIRE(K > 0 && q_width > 0 && kv_width == n_kv_heads * head_size && head_size > 0, "gemm_qkv_cache: bad sizes");
    MLLM_REQUIRE(page_size > 0 && (page_size & (page_size - 1)) == 0, "gemm_qkv_cache: page size %d is no power of two", page_size);
    MLLM_REQUIRE(dtype == MLLM_F32 || dtype == MLLM_BF16, "gemm_qkv_cache: unknown dtype %d", dtype);
    MLLM_REQUIRE(K % (dtype == MLLM_F32 ? 4 : 8) == 0, "gemm_qkv_cache: K=%d is not a multiple of a 16-byte piece", K);
    if (M == 0) return 0;
    CacheScatter scatter{k_pages, v_pages, slots, q_width, kv_width, n_kv_heads, head_size, 0, 1};
    while ((1 << scatter.page_shift) < page_size) scatter.page_shift++;
    int N = q_width + 2 * kv_width;
    MLLM_REQUIRE(!x_packed || mllm_gemm_takes_packed_rows(M, N, K, dtype),
                 "gemm_qkv_cache: rows in the packed layout are for the kernel for few rows, which M=%d N=%d K=%d do not take", M, N, K);
#define MLLM_QKV_CASE(T)                                                                                              \
    if (!takes_few_row_kernel<T>(M, N, K)) launch_tiled<T, T, true>((const T*)A, (const T*)W, w_packed != 0, bias, nullptr, (T*)out_q, M, N, K, 0, stream, scatter); \
    else if (M <= 16) launch_skinny<T, T, 1>((const T*)A, (const T*)W, w_packed != 0, bias, nullptr, (T*)out_q, M, N, K, 0, stream, scatter, 1, x_packed);      \
    else if (M <= 32) launch_skinny<T, T, 2>((const T*)A, (const T*)W, w_packed != 0, bias, nullptr, (T*)out_q, M, N, K, 0, stream, scatter, 1, x_packed); \
    else launch_skinny<T, T, 4>((const T*)A, (const T*)W, w_packed != 0, bias, nullptr, (T*)out_q, M, N, K, 0, stream, scatter, 1, x_packed);
    if (dtype == MLLM_F32) { MLLM_QKV_CASE(float) } else { MLLM_QKV_CASE(bf16_t) }
#undef MLLM_QKV_CASE
    return mllm_check_launch("gemm_qkv_cache");
}

// ------------------------------------------------------------------------------------------------
// The product cut along K without an allocation (no_alloc.h): the partial products go to a fixed
// array of the library instead of memory the caller brings.
// ------------------------------------------------------------------------------------------------
namespace {

constexpr size_t STATIC_SCRATCH_FLOATS = (size_t)1 << 20;  // 4 MiB
// Each GPU holds its own copy of this array at its own address. In host code the name is only a
// handle for hipGetSymbolAddress: kernels get the address that call returns, never the name.
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

constexpr int MAX_DEVICES = 64;
float* g_scratch_at[MAX_DEVICES];  // per device: the array's address there, null until looked up
std::mutex g_scratch_lock;

// The current device's array. The lookup runs once per device, with that device current.
int static_scratch(float** at) {
    int device = -1;
    hipError_t status = hipGetDevice(&device);
    MLLM_REQUIRE(status == hipSuccess, "static scratch: no current device: %s", hipGetErrorString(status));
    MLLM_REQUIRE(device >= 0 && device < MAX_DEVICES, "static scratch: device %d is beyond the %d this library keeps track of", device, MAX_DEVICES);
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (g_scratch_at[device] == nullptr) {
        void* address = nullptr;
        status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        MLLM_REQUIRE(status == hipSuccess && address != nullptr, "static scratch: the array's address on device %d is not known: %s", device,
                     hipGetErrorString(status));
        g_scratch_at[device] = static_cast<float*>(address);
    }
    *at = g_scratch_at[device];
    return 0;
}

// out = residual + bias + partials[0] + partials[1] + ..., in that order (the order of
// pending_sum_kernel, so that both give the same numbers). grid (column groups of 256, rows).
__global__ __launch_bounds__(256) void static_sum_kernel(const float* __restrict__ partials, const float* __restrict__ bias,
                                                         const float* __restrict__ residual, float* __restrict__ out, int M, int N,
                                                         int k_blocks) {
    const int col = blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    if (col >= N) return;
    const size_t at = (size_t)row * N + col;
    float value = residual ? residual[at] : 0.0f;
    if (bias) value += bias[col];
    for (int s = 0; s < k_blocks; s++) value += partials[(size_t)s * M * N + at];
    out[at] = value;
}

}  // namespace

MLLM_API long long mllm_static_scratch_bytes(void) { return (long long)(STATIC_SCRATCH_FLOATS * sizeof(float)); }

MLLM_API int mllm_static_scratch_prepare(void) {
    float* at = nullptr;
    return static_scratch(&at);
}

MLLM_API int mllm_linear_split_static(const void* A, const void* W, int w_packed, const float* bias, const float* residual,
                                      float* out, int M, int N, int K, int in_dtype, int k_blocks, hipStream_t stream) {
    MLLM_REQUIRE(A != nullptr && W != nullptr && out != nullptr, "linear_split_static: an operand is missing");
    MLLM_REQUIRE(M >= 0 && N > 0 && K > 0 && M <= 65535, "linear_split_static: bad sizes M=%d N=%d K=%d", M, N, K);
    MLLM_REQUIRE(k_blocks >= 1 && k_blocks <= 16, "linear_split_static: %d partial products is not in 1..16", k_blocks);
    MLLM_REQUIRE((size_t)k_blocks * (size_t)M * (size_t)N <= STATIC_SCRATCH_FLOATS,
                 "linear_split_static: %d partial products of %d x %d floats do not fit the library's %lld bytes of scratch memory", k_blocks, M, N,
                 mllm_static_scratch_bytes());
    if (M == 0) return 0;
    float* partials = nullptr;
    if (static_scratch(&partials)) return 1;
    if (mllm_gemm_split(A, W, w_packed, partials, M, N, K, in_dtype, k_blocks, 0, stream)) return 1;
    dim3 grid(ceil_div(N, 256), M);
    mllm_count_kernel(MLLM_K_STATIC_SUM);
    static_sum_kernel<<<grid, 256, 0, stream>>>(partials, bias, residual, out, M, N, k_blocks);
    return mllm_check_launch("linear_split_static");
}
