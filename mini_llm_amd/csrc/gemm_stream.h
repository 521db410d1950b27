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

namespace stream {

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt with only the vector-memory counter set: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
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
template <typename OutT, int BM, int BN, int WAVES_M, int WAVES_N, int STAGES>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_stream_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias, const float* __restrict__ residual,
    OutT* __restrict__ out, int M, int N, int K, int epilogue, CacheScatter scatter, int k_per_block) {
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, FM = WM / 32, FN = WN / 32;
    constexpr int BK = 64;
    constexpr int A_LOADS = BM / 16 * 2, W_LOADS = BN / 16 * 2, LOADS = A_LOADS + W_LOADS;  // loads of 1 KiB a tile of K
    static_assert(FM >= 1 && FN >= 1 && LOADS % NW == 0, "every wave issues the same number of loads");
    constexpr int LPW = LOADS / NW;
    static_assert(LPW * (STAGES - 1) < 64, "the loads in flight must fit the counter");
    constexpr int STAGE_BYTES = (BM + BN) * 128;
    constexpr int OUT_VEC = 16 / (int)sizeof(OutT);          // columns in a 16-byte piece of the output
    constexpr int SLAB_ROW = WN * (int)sizeof(OutT) + 16;    // a row of a wave's tile in LDS, padded by one piece
    constexpr int PIECES = WN / OUT_VEC;
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int k_begin = blockIdx.z * k_per_block, k_end = min(K, k_begin + k_per_block);
    const int k_steps = K / 32, n_tiles = (k_end - k_begin) / BK;
    const int w_row_tiles = (N + 15) / 16;
    out += (size_t)blockIdx.z * M * N;

    // This wave's loads of a tile: load q = wave + NW * i of the stage. src[i] is the lane's address in the block's first tile.
    const bf16_t* src[LPW];
    int dst[LPW];
#pragma unroll
    for (int i = 0; i < LPW; i++) {
        const int q = wave + NW * i;
        if (q < A_LOADS) {
            const int rt = q / 2, kc = q % 2;
            const int r16 = lane / 4, piece = (lane % 4) ^ ((r16 >> 2) & 3);
            const int row = min(m0 + rt * 16 + r16, M - 1);  // beyond the last row: that row again, never stored
            src[i] = A + (size_t)row * K + k_begin + kc * 32 + piece * 8;
            dst[i] = q * 1024;
        } else {
            const int qw = q - A_LOADS, rt = qw / 2, kc = qw % 2;
            const int row_tile = min(n0 / 16 + rt, w_row_tiles - 1);
            src[i] = W + packed_offset<bf16_t>(row_tile, k_begin / 32 + kc, k_steps, lane);
            dst[i] = BM * 128 + qw * 1024;
        }
    }
    auto issue = [&](int tile, int stage) {
        const int t = min(tile, n_tiles - 1);  // beyond the end: the last tile again, never used (the count of loads in flight stays the same)
#pragma unroll
        for (int i = 0; i < LPW; i++) {
            const int q = wave + NW * i;
            const bf16_t* p = q < A_LOADS ? src[i] + t * BK : src[i] + (size_t)t * (2 * 64 * 8);
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)p,
                                             (void __attribute__((address_space(3)))*)(lds + stage * STAGE_BYTES + dst[i]), 16, 0, 0);
        }
    };

    f32x16 acc[FN][FM];
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[j][i][v] = 0.0f;

    // What the epilogue adds is asked for now and arrives while the products run: asked for where it is used, every
    // block would wait for it at the end, with nothing left to hide the trip behind.
    constexpr int ROW_STEPS = 32 * PIECES / WAVE;  // 16-byte pieces of a 32-row slab a lane stores
    static_assert((32 * PIECES) % WAVE == 0, "the lanes of a wave share a slab's pieces evenly");
    const int n_wave = n0 + wave_n * WN;
    f32x4 early_bias[FN][4];
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int n = n_wave + j * 32 + 8 * g + 4 * (lane / 32);  // N is a multiple of 8: four columns are inside or outside together
            early_bias[j][g] = bias && n < N ? *reinterpret_cast<const f32x4*>(bias + n) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    f32x4 early_residual[sizeof(OutT) == 4 ? FM : 1][sizeof(OutT) == 4 ? ROW_STEPS : 1];
    if constexpr (sizeof(OutT) == 4) {
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int r = 0; r < ROW_STEPS; r++) {
                const int index = r * WAVE + lane, row = index / PIECES, piece = index % PIECES;
                const int m = m0 + wave_m * WM + i * 32 + row, n = n_wave + piece * OUT_VEC;
                early_residual[i][r] = residual && !scatter.enabled && m < M && n < N ? *reinterpret_cast<const f32x4*>(residual + (size_t)m * N + n)
                                                                                      : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
    }

    if (n_tiles > 0) {
#pragma unroll
        for (int s = 0; s < STAGES - 1; s++) issue(s, s);

        // A 32 x 16 fragment: lane l holds row l % 32, k (l / 32) * 8 .. + 8. W: chunk [piece][row]; A: chunk [row][piece rotated].
        const int w_frag0 = BM * 128 + (wave_n * WN / 16) * 2048 + ((lane % 32) / 16) * 2048 + (lane / 32) * 256 + (lane % 16) * 16;
        const int a_row0 = (wave_m * WM / 16) * 2048 + ((lane % 32) / 16) * 2048 + (lane % 16) * 64, a_turn = ((lane % 16) >> 2) & 3;
        bf16x8 a[2][FM], w[2][FN];
        auto read_frags = [&](int set, const unsigned char* stage, int kk) {
#pragma unroll
            for (int i = 0; i < FM; i++)
                a[set][i] = *reinterpret_cast<const bf16x8*>(stage + a_row0 + i * 4096 + (kk / 2) * 1024 + ((((kk % 2) * 2 + lane / 32) ^ a_turn) * 16));
#pragma unroll
            for (int j = 0; j < FN; j++) w[set][j] = *reinterpret_cast<const bf16x8*>(stage + w_frag0 + j * 4096 + (kk / 2) * 1024 + (kk % 2) * 512);
        };
        auto products = [&](int set) {
#pragma unroll
            for (int j = 0; j < FN; j++)
#pragma unroll
                for (int i = 0; i < FM; i++) acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w[set][j], a[set][i], acc[j][i], 0, 0, 0);
        };
        wait_vmcnt<LPW*(STAGES - 2)>();
        asm volatile("s_barrier" ::: "memory");
        issue(STAGES - 1, (STAGES - 1) % STAGES);
        read_frags(0, lds, 0);
        for (int t = 0; t < n_tiles; t++) {
            const unsigned char* stage = lds + (t % STAGES) * STAGE_BYTES;
            read_frags(1, stage, 1);
            products(0);
            read_frags(0, stage, 2);
            products(1);
            read_frags(1, stage, 3);
            products(0);
            // the next tile has landed in every wave, and every wave has its last fragments of this one
            wait_vmcnt<LPW*(STAGES - 2)>();
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            issue(t + STAGES, (t + STAGES) % STAGES);
            read_frags(0, lds + ((t + 1) % STAGES) * STAGE_BYTES, 0);
            products(1);
        }
    }

    // acc[j][i][v] is row m0 + wave_m*WM + i*32 + lane%32, column n0 + wave_n*WN + j*32 + 8*(v/4) + 4*(lane/32) + v%4.
    // Through LDS: 32 rows of the wave's tile at a time, written as the accumulators lie, read back and stored row by row.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // no load is under way, no wave still reads the stages
    unsigned char* slab = lds + wave * (32 * SLAB_ROW);
#pragma unroll
    for (int i = 0; i < FM; i++) {
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int n_local = j * 32 + 8 * g + 4 * (lane / 32);
                f32x4 value;
#pragma unroll
                for (int e = 0; e < 4; e++) value[e] = acc[j][i][4 * g + e];
                value += early_bias[j][g];
                if (epilogue == MLLM_EPI_GELU_TANH) {
#pragma unroll
                    for (int e = 0; e < 4; e++) value[e] = sizeof(OutT) == 2 ? gelu_tanh_for_bf16(value[e]) : gelu_tanh(value[e]);
                } else if (epilogue == MLLM_EPI_GELU_ERF) {
#pragma unroll
                    for (int e = 0; e < 4; e++) value[e] = sizeof(OutT) == 2 ? gelu_erf_for_bf16(value[e]) : gelu_erf(value[e]);
                }
                put4<OutT>(reinterpret_cast<OutT*>(slab + (lane % 32) * SLAB_ROW) + n_local, value);
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int r = 0; r < ROW_STEPS; r++) {
            const int index = r * WAVE + lane, row = index / PIECES, piece = index % PIECES;
            const int m = m0 + wave_m * WM + i * 32 + row, n = n_wave + piece * OUT_VEC;
            Vec16 v = *reinterpret_cast<const Vec16*>(slab + row * SLAB_ROW + piece * 16);
            if (m >= M || n >= N) continue;
            if (scatter.enabled) {
                // a fused q/k/v projection: q columns to out [M, q_width], key and value columns into the cache
                // page at the row's slot (a piece lies inside one head: the head size is a multiple of 8)
                if (n < scatter.q_width) {
                    *reinterpret_cast<Vec16*>(out + (size_t)m * scatter.q_width + n) = v;
                } else {
                    const int slot = scatter.slots[m];
                    if (slot < 0) continue;
                    int c = n - scatter.q_width;
                    OutT* pages = (OutT*)(c < scatter.kv_width ? scatter.k_pages : scatter.v_pages);
                    if (c >= scatter.kv_width) c -= scatter.kv_width;
                    const int kv_head = c / scatter.head_size, d = c % scatter.head_size;
                    const int page = slot >> scatter.page_shift, offset = slot & ((1 << scatter.page_shift) - 1);
                    *reinterpret_cast<Vec16*>(pages + ((((size_t)page * scatter.n_kv_heads + kv_head) << scatter.page_shift) + offset) * scatter.head_size + d) = v;
                }
                continue;
            }
            if constexpr (sizeof(OutT) == 4) {
                f32x4 sum = *reinterpret_cast<f32x4*>(&v);
                sum = early_residual[i][r] + sum;   // zeros where there is no residual
                v = *reinterpret_cast<Vec16*>(&sum);
            }
            *reinterpret_cast<Vec16*>(out + (size_t)m * N + n) = v;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
}

template <typename OutT, int BM, int BN, int WAVES_M, int WAVES_N, int STAGES>
void launch(const bf16_t* a, const bf16_t* w, const float* bias, const float* residual, OutT* o, int M, int N, int K, int epilogue,
           hipStream_t stream, CacheScatter scatter, int k_blocks) {
    // the stages of the loop, or the rows the epilogue passes through LDS (32 rows of every wave's tile, padded), whichever is more
    constexpr int SLAB_BYTES = WAVES_M * WAVES_N * 32 * (BN / WAVES_N * (int)sizeof(OutT) + 16);
    constexpr int LDS_BYTES = STAGES * (BM + BN) * 128 > SLAB_BYTES ? STAGES * (BM + BN) * 128 : SLAB_BYTES;
    static bool raised = false;  // per instantiation: the limit on dynamic LDS is a property of the kernel
    if (!raised && LDS_BYTES > 64 * 1024) {
        // (if this fails the launch below fails too, and the entry point reports that)
        raised = hipFuncSetAttribute((const void*)gemm_stream_kernel<OutT, BM, BN, WAVES_M, WAVES_N, STAGES>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) == hipSuccess;
    }
    const int k_per_block = k_blocks == 1 ? K : ceil_div(ceil_div(K, k_blocks), 64) * 64;
    dim3 grid(ceil_div(N, BN), ceil_div(M, BM), k_blocks);
    gemm_stream_kernel<OutT, BM, BN, WAVES_M, WAVES_N, STAGES><<<grid, 64 * WAVES_M * WAVES_N, LDS_BYTES, stream>>>(
        a, w, bias, residual, o, M, N, K, epilogue, scatter, k_per_block);
}

// Whether the product takes this kernel: bfloat16 with a packed W, whole tiles of K, whole 16-byte pieces of output
// columns, enough rows to fill tiles of 128; a fused q/k/v projection only where a piece stays inside one head.
inline bool takes(int M, int N, int K, bool packed, const CacheScatter& scatter, size_t out_element) {
    if (!packed || K % 64 != 0 || K < 64 || N % 8 != 0 || M < 192 || ceil_div(M, 128) > 65535) return false;
    if (scatter.enabled && (out_element != 2 || scatter.head_size % 8 != 0 || scatter.q_width % 8 != 0 || scatter.kv_width % 8 != 0)) return false;
    return true;
}

// Tile by the number of blocks: 128 x 128 tiles of eight waves where they give every compute unit a block, else 128 x 64
// of four waves; a long K asks for a third stage (measured at GPT-2's sizes: 2,048 rows x 2,304 / 768 / 3,072 / 768 columns).
template <typename OutT>
void dispatch(const bf16_t* a, const bf16_t* w, const float* bias, const float* residual, OutT* o, int M, int N, int K, int epilogue,
             hipStream_t stream, CacheScatter scatter, int k_blocks) {
    const int tiles_128 = ceil_div(M, 128) * ceil_div(N, 128) * k_blocks;
    if (tiles_128 >= 256) launch<OutT, 128, 128, 4, 2, 2>(a, w, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks);
    else if (K / k_blocks >= 1536) launch<OutT, 128, 64, 2, 2, 3>(a, w, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks);
    else launch<OutT, 128, 64, 2, 2, 2>(a, w, bias, residual, o, M, N, K, epilogue, stream, scatter, k_blocks);
}

}  // namespace stream
