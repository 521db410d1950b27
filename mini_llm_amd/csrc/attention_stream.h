// Prompt attention for rows of 64, 128 or 256 bytes (bfloat16 heads of 32, 64 or 128; 32-bit heads of 32 or 64)
// over pages of at least 32 keys: key and value tiles stream from the cache pages straight into LDS
// (global_load_lds_dwordx4), and a block's keys are divided among its waves. Included by attention.hip.
// The text below describes the bfloat16 kernel; what the 32-bit one does differently stands where it does it: the
// 32-bit matrix instruction (32 x 32 x 2, four to a 16-byte piece of a key), the library's expf, and values read as
// they are stored (the instruction takes single elements, so nothing has to be transposed).
//
// A block owns 64 queries of one (request, head). Each of its four waves holds all 64 queries and walks every fourth
// tile of 32 keys with softmax statistics of its own; at the end the four partial results are combined through LDS.
// So the block with the most keys, which decides the kernel's time for a causal prompt, takes a quarter of the steps
// that one wave would, no wave waits for another inside the loop (there is no barrier in it: a wave's tiles land in
// LDS that only this wave reads), and the blocks are small and many enough to fill the chip.
//
// S^T = K . Q^T and O^T = V^T . P^T run on the matrix cores (32 x 32 x 16): a lane holds one query's scores for
// sixteen of a tile's keys, so the softmax runs along registers; statistics in 32-bit, exp2 of prescaled scores, the
// accumulators rescaled only in tiles that raise some query's maximum.
//  * A tile's keys and values land in LDS as they lie in the pages, rows of head_size elements. A tile lies in one page,
//    so its page is looked up once, by the scalar unit. Rows behind the last stored key are replaced by that key's row
//    (never by what an unwritten place of the page holds) and masked by their position.
//  * V^T, the operand that needs eight consecutive keys of one column per lane, is read from those rows by the
//    transposing LDS read of this chip (ds_read_b64_tr_b16): sixteen lanes point at a block of 4 keys x 16 columns
//    and each gets the four keys of its own column.
//  * The 16-byte pieces of a row lie rotated by the row (which bytes a lane asks for decides where they land), so that
//    the sixteen lanes of a key fragment read, and the four rows of a transposing read, fall on different banks.
//  * A wave keeps two key tiles and two value tiles in flight. Before it asks for a tile into a place it has just
//    read, it waits for those reads (lgkmcnt): the load would overwrite what is still queued in the LDS unit.
#pragma once

namespace prefill_stream {

constexpr int KEYS = 32;      // keys per tile
// SPLITS (a parameter of the kernel): waves per block, 4 or 8; wave w takes tiles w, w + SPLITS, ...

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

// A 16-byte LDS read the compiler does not know to be one (see read_transposed): the value is there once
// fragments_landed has passed, and nothing may read the register before.
__device__ __forceinline__ void ask_fragment(i32x4& to, unsigned address) {
    asm volatile("ds_read_b128 %0, %1" : "=v"(to) : "v"(address));
}
__device__ __forceinline__ void fragments_landed(i32x4& first) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(first)); }
__device__ __forceinline__ void and_this_one(i32x4& fragment) { asm volatile("" : "+v"(fragment)); }

__device__ __forceinline__ unsigned lds_address(const unsigned char* p) {
    return (unsigned)(size_t)(const __attribute__((address_space(3))) unsigned char*)p;
}

// The transposing reads of a tile's values (ds_read_b64_tr_b16), written out as instructions: through the compiler's
// builtin each of them would first wait for ALL loads into LDS that are in flight (the compiler cannot tell the tile
// being read from the tiles still being loaded), which would undo the prefetching. Per 32 columns one address and
// four reads, 8 keys (8 rows) apart. The block ends with the wait for its own reads, so what it returns is valid.
template <int DT, int ROW_BYTES>
__device__ __forceinline__ void read_transposed(const unsigned (&address)[DT], short4_t (&out)[DT][4]);

template <>
__device__ __forceinline__ void read_transposed<1, 64>(const unsigned (&address)[1], short4_t (&out)[1][4]) {
    constexpr int ROW_BYTES = 64;
    asm volatile(
        "ds_read_b64_tr_b16 %0, %4 offset:%5\n\t"
        "ds_read_b64_tr_b16 %1, %4 offset:%6\n\t"
        "ds_read_b64_tr_b16 %2, %4 offset:%7\n\t"
        "ds_read_b64_tr_b16 %3, %4 offset:%8\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(out[0][0]), "=&v"(out[0][1]), "=&v"(out[0][2]), "=&v"(out[0][3])
        : "v"(address[0]), "n"(0 * 8 * ROW_BYTES), "n"(1 * 8 * ROW_BYTES), "n"(2 * 8 * ROW_BYTES), "n"(3 * 8 * ROW_BYTES)
        : "memory");
}

template <>
__device__ __forceinline__ void read_transposed<2, 128>(const unsigned (&address)[2], short4_t (&out)[2][4]) {
    constexpr int ROW_BYTES = 128;
    asm volatile(
        "ds_read_b64_tr_b16 %0, %8 offset:%10\n\t"
        "ds_read_b64_tr_b16 %1, %8 offset:%11\n\t"
        "ds_read_b64_tr_b16 %2, %8 offset:%12\n\t"
        "ds_read_b64_tr_b16 %3, %8 offset:%13\n\t"
        "ds_read_b64_tr_b16 %4, %9 offset:%10\n\t"
        "ds_read_b64_tr_b16 %5, %9 offset:%11\n\t"
        "ds_read_b64_tr_b16 %6, %9 offset:%12\n\t"
        "ds_read_b64_tr_b16 %7, %9 offset:%13\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(out[0][0]), "=&v"(out[0][1]), "=&v"(out[0][2]), "=&v"(out[0][3]), "=&v"(out[1][0]), "=&v"(out[1][1]), "=&v"(out[1][2]), "=&v"(out[1][3])
        : "v"(address[0]), "v"(address[1]), "n"(0 * 8 * ROW_BYTES), "n"(1 * 8 * ROW_BYTES), "n"(2 * 8 * ROW_BYTES), "n"(3 * 8 * ROW_BYTES)
        : "memory");
}

template <>
__device__ __forceinline__ void read_transposed<4, 256>(const unsigned (&address)[4], short4_t (&out)[4][4]) {
    constexpr int ROW_BYTES = 256;
    asm volatile(
        "ds_read_b64_tr_b16 %0, %16 offset:%20\n\t"
        "ds_read_b64_tr_b16 %1, %16 offset:%21\n\t"
        "ds_read_b64_tr_b16 %2, %16 offset:%22\n\t"
        "ds_read_b64_tr_b16 %3, %16 offset:%23\n\t"
        "ds_read_b64_tr_b16 %4, %17 offset:%20\n\t"
        "ds_read_b64_tr_b16 %5, %17 offset:%21\n\t"
        "ds_read_b64_tr_b16 %6, %17 offset:%22\n\t"
        "ds_read_b64_tr_b16 %7, %17 offset:%23\n\t"
        "ds_read_b64_tr_b16 %8, %18 offset:%20\n\t"
        "ds_read_b64_tr_b16 %9, %18 offset:%21\n\t"
        "ds_read_b64_tr_b16 %10, %18 offset:%22\n\t"
        "ds_read_b64_tr_b16 %11, %18 offset:%23\n\t"
        "ds_read_b64_tr_b16 %12, %19 offset:%20\n\t"
        "ds_read_b64_tr_b16 %13, %19 offset:%21\n\t"
        "ds_read_b64_tr_b16 %14, %19 offset:%22\n\t"
        "ds_read_b64_tr_b16 %15, %19 offset:%23\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(out[0][0]), "=&v"(out[0][1]), "=&v"(out[0][2]), "=&v"(out[0][3]), "=&v"(out[1][0]), "=&v"(out[1][1]), "=&v"(out[1][2]), "=&v"(out[1][3]), "=&v"(out[2][0]), "=&v"(out[2][1]), "=&v"(out[2][2]), "=&v"(out[2][3]), "=&v"(out[3][0]), "=&v"(out[3][1]), "=&v"(out[3][2]), "=&v"(out[3][3])
        : "v"(address[0]), "v"(address[1]), "v"(address[2]), "v"(address[3]), "n"(0 * 8 * ROW_BYTES), "n"(1 * 8 * ROW_BYTES), "n"(2 * 8 * ROW_BYTES), "n"(3 * 8 * ROW_BYTES)
        : "memory");
}

// Eight 4-byte LDS reads from one address with the offsets the 32-bit value product needs (keys 0-3 and 8-11 of a
// lane's sixteen, ROW_BYTES apart; `FROM` 0: those, 1: keys 16-19 and 24-27), as instructions, for the reason above.
// Returns when the values are in registers.
template <int ROW_BYTES, int FROM>
__device__ __forceinline__ void read_eight(unsigned address, float (&out)[8]) {
    asm volatile(
        "ds_read_b32 %0, %8 offset:%9\n\t"
        "ds_read_b32 %1, %8 offset:%10\n\t"
        "ds_read_b32 %2, %8 offset:%11\n\t"
        "ds_read_b32 %3, %8 offset:%12\n\t"
        "ds_read_b32 %4, %8 offset:%13\n\t"
        "ds_read_b32 %5, %8 offset:%14\n\t"
        "ds_read_b32 %6, %8 offset:%15\n\t"
        "ds_read_b32 %7, %8 offset:%16\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(out[0]), "=&v"(out[1]), "=&v"(out[2]), "=&v"(out[3]), "=&v"(out[4]), "=&v"(out[5]), "=&v"(out[6]), "=&v"(out[7])
        : "v"(address), "n"((16 * FROM + 0) * ROW_BYTES), "n"((16 * FROM + 1) * ROW_BYTES), "n"((16 * FROM + 2) * ROW_BYTES), "n"((16 * FROM + 3) * ROW_BYTES),
          "n"((16 * FROM + 8) * ROW_BYTES), "n"((16 * FROM + 9) * ROW_BYTES), "n"((16 * FROM + 10) * ROW_BYTES), "n"((16 * FROM + 11) * ROW_BYTES)
        : "memory");
}

template <typename T, int HD, int SPLITS>
struct Layout {
    static constexpr bool FP32 = sizeof(T) == 4;
    static constexpr int ROW_BYTES = HD * (int)sizeof(T);
    static constexpr int PPR = ROW_BYTES / 16;      // 16-byte pieces per row
    static constexpr int ROWS_PER_LOAD = 1024 / ROW_BYTES;  // rows a wave's 1 KiB load covers
    static constexpr int LOADS = KEYS / ROWS_PER_LOAD;  // loads per tile of keys (as many again for the values)
    static constexpr int TILE_BYTES = KEYS * ROW_BYTES;
    static constexpr int WAVE_BYTES = 4 * TILE_BYTES;   // two key tiles, two value tiles
    static constexpr int LDS_BYTES = SPLITS * WAVE_BYTES;
    static_assert(ROW_BYTES == 64 || ROW_BYTES == 128 || ROW_BYTES == 256, "rows of 64, 128 or 256 bytes");
    static_assert(WAVE_BYTES >= 64 * HD * 4, "a wave's partial result (of up to 64 queries) takes the place of its tiles");
    // K: sixteen consecutive keys, the same piece: their 16-byte slots must differ modulo 256 bytes.
    static __device__ __forceinline__ int k_turn(int key) { return (key / (16 / PPR)) % PPR; }
    // V: four consecutive keys, the same 64 bytes of columns: their 64-byte slots must differ modulo 256 bytes.
    // (32-bit values are read a row's 128 consecutive bytes at a time: no turn needed)
    static __device__ __forceinline__ int v_turn(int key) { return FP32 || ROW_BYTES == 64 ? 0 : (ROW_BYTES == 128 ? ((key >> 1) & 1) * 4 : (key & 3) * 4); }
};

// QUERIES: 64 queries a block (two sub-tiles of 32, both held by every wave), or 32 where that would leave compute units
// without a block: what the kernel waits for is the wave with the most tiles, and a tile of 32 queries takes it half as long.
// SPLITS: four waves a block, or eight where the portions reach far back: the kernel's time is the time of the wave with
// the most tiles (it pays every tile's chain in full), which eight waves halve; a block then has a compute unit to itself.
template <typename T, int HD, int QUERIES, int SPLITS>
__global__ __launch_bounds__(64 * SPLITS, (HD * sizeof(T) <= 128 && SPLITS == 4) ? 2 : 1) void attention_prefill_stream_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    T* __restrict__ out, int out_stride, const int* __restrict__ q_starts, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, int max_blocks, int n_heads, int n_kv_heads, int page_shift, int window, float scale) {
    typedef Layout<T, HD, SPLITS> L;
    constexpr bool FP32 = L::FP32;
    constexpr int QSUB = QUERIES / 32;
    static_assert(QUERIES == 32 || QUERIES == 64, "one or two sub-tiles of queries");
    static_assert(HD % 32 == 0, "the output is written in tiles of 32 head dimensions");
    constexpr int QSTEPS = L::PPR / 2;  // k-steps of the score product: a lane takes one 16-byte piece of its key in each
    constexpr int PIECE = 16 / (int)sizeof(T);  // elements of a 16-byte piece
    constexpr int DT = HD / 32;      // 32-row tiles of the output's head dimension
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    __shared__ float stats_lds[SPLITS][QUERIES][2];

    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int lane32 = lane % 32, half = lane / 32;
    const int request = blockIdx.x / n_heads, head = blockIdx.x % n_heads;
    const int q_first = q_starts[request];
    const int q_len = q_starts[request + 1] - q_first;
    const int tile_q0 = (gridDim.y - 1 - blockIdx.y) * QUERIES;  // the blocks with the most keys start first
    if (tile_q0 >= q_len) return;
    const int context = context_lens[request];
    if (context < 0) return;  // a padding request of a padded batch: its rows (if it has any) are nobody's, and it has no pages
    const int kv_head = head / (n_heads / n_kv_heads);
    const int* table = block_tables + (size_t)request * max_blocks;
    const int page_mask = (1 << page_shift) - 1;

    // Q^T operand, kept in registers: step s holds columns 16 s + 8 half .. + 8 of this lane's query in each sub-tile
    Vec16 q_reg[QSUB][QSTEPS];
    int q_position[QSUB];
#pragma unroll
    for (int qs = 0; qs < QSUB; qs++) {
        const int q_local = tile_q0 + qs * 32 + lane32;
        // a lane beyond the portion's end takes the portion's first row and position -1: no key is at or before it, so every
        // score of it is masked (nothing waits for the rows here: the tiles are asked for while they are still on their way)
        q_position[qs] = q_local < q_len ? context + q_local : -1;
        const T* q_row = q + (size_t)(q_first + (q_local < q_len ? q_local : 0)) * q_stride + head * HD;
#pragma unroll
        for (int s = 0; s < QSTEPS; s++) q_reg[qs][s] = *reinterpret_cast<const Vec16*>(q_row + (2 * s + half) * PIECE);
    }

    const int block_last_position = context + min(tile_q0 + QUERIES, q_len) - 1;
    const int block_first_key = window > 0 ? max(0, context + tile_q0 - window + 1) : 0;
    const int first_base = (block_first_key / KEYS) * KEYS;
    const int n_tiles = (block_last_position - first_base) / KEYS + 1;
    const int n_mine = n_tiles > wave ? (n_tiles - wave + SPLITS - 1) / SPLITS : 0;  // tiles wave, wave + SPLITS, ...

    // One half (keys or values) of this wave's i-th tile, into place i % 2. A lane asks for piece (slot ^ turn) of its
    // row, and the load puts it in the row's slot. Beyond the wave's last tile the last one is asked for again (never
    // used), so that the count of loads in flight is the same in every step.
    unsigned char* const wave_lds = lds + wave * L::WAVE_BYTES;
    auto tile_base = [&](int i) { return first_base + (wave + SPLITS * min(i, n_mine - 1)) * KEYS; };
    // a lane's place among the rows of a whole tile, in bytes: the same for every tile, so an address is a base all lanes
    // share plus this (worked out anew for every load it was a sixth of the loop's vector instructions)
    unsigned k_lane[L::LOADS], v_lane[L::LOADS];
#pragma unroll
    for (int l = 0; l < L::LOADS; l++) {
        const int row = l * L::ROWS_PER_LOAD + lane / L::PPR, slot = lane % L::PPR;
        k_lane[l] = row * L::ROW_BYTES + (slot ^ L::k_turn(row)) * 16;
        v_lane[l] = row * L::ROW_BYTES + (slot ^ L::v_turn(row)) * 16;
    }
    auto issue = [&](int i, int page, bool is_value) {  // page: the one that holds the whole tile
        const int k_base = tile_base(i);
        const int last_row = block_last_position - k_base;
        const unsigned char* base = reinterpret_cast<const unsigned char*>(
            (is_value ? v_pages : k_pages) + ((((size_t)page * n_kv_heads + kv_head) << page_shift) + (k_base & page_mask)) * HD);
        unsigned char* place = wave_lds + (is_value ? 2 * L::TILE_BYTES : 0) + (i % 2) * L::TILE_BYTES;
        if (last_row >= KEYS - 1) {
#pragma unroll
            for (int l = 0; l < L::LOADS; l++)
                __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(base + (is_value ? v_lane[l] : k_lane[l])),
                                                 (void __attribute__((address_space(3)))*)(place + l * 1024), 16, 0, 0);
        } else {  // the tile that holds the last key: the rows behind it are that key's row again
#pragma unroll
            for (int l = 0; l < L::LOADS; l++) {
                const int row = l * L::ROWS_PER_LOAD + lane / L::PPR, slot = lane % L::PPR;
                const int piece = slot ^ (is_value ? L::v_turn(row) : L::k_turn(row));
                const unsigned char* src = base + min(row, last_row) * L::ROW_BYTES + piece * 16;
                __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)src,
                                                 (void __attribute__((address_space(3)))*)(place + l * 1024), 16, 0, 0);
            }
        }
    };

    f32x16 acc_o[QSUB][DT];
    float running_max[QSUB], running_sum[QSUB];
#pragma unroll
    for (int qs = 0; qs < QSUB; qs++) {
        running_max[qs] = -INFINITY;
        running_sum[qs] = 0.0f;
#pragma unroll
        for (int i2 = 0; i2 < DT; i2++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc_o[qs][i2][v] = 0.0f;
    }
    // bfloat16: 2^x of a score prescaled by log2(e); 32-bit: the library's e^x of the scaled score. Positive either way, so
    // the scaling commutes with the maximum.
    const float score_scale = FP32 ? scale : scale * 1.4426950408889634f;
    auto weight_of = [](float x) { return FP32 ? expf(x) : __builtin_amdgcn_exp2f(x); };
    // one 16-byte piece of a key against the same piece of the queries: one product in bfloat16 (32 x 32 x 16), four in
    // 32-bit (32 x 32 x 2: component c of every lane forms the pair of one product, the same pairing on both operands)
    auto piece_product = [](const Vec16& k_piece, const Vec16& q_piece, f32x16 sums) {
        if constexpr (FP32) {
            const f32x4 k4 = *reinterpret_cast<const f32x4*>(&k_piece), q4 = *reinterpret_cast<const f32x4*>(&q_piece);
#pragma unroll
            for (int c = 0; c < 4; c++) sums = __builtin_amdgcn_mfma_f32_32x32x2f32(k4[c], q4[c], sums, 0, 0, 0);
            return sums;
        } else {
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(&k_piece), *reinterpret_cast<const bf16x8*>(&q_piece), sums, 0, 0, 0);
        }
    };

    // K fragment (32 keys x 16 columns): lane l holds key l % 32, columns 16 s + 8 (l / 32) .. + 8
    // V^T fragment by two transposing reads: the sixteen lanes of group g = l / 16 point at keys k0 + (l % 16) / 4, columns
    // 16 (g % 2) + 4 (l % 4) .. + 4 of a 32-column tile, and lane l gets keys k0 .. k0 + 3 of column 16 (g % 2) + l % 16
    const int v_key_in_read = (lane % 16) / 4, v_col = 16 * ((lane / 16) % 2) + 4 * (lane % 4);
    // The scores of a tile: S^T = K . Q^T, a key fragment serving both sub-tiles of queries. Returns with the fragments in
    // registers (their place may be loaded into again) and the products still running.
    auto scores = [&](int i, f32x16 (&s_acc)[QSUB]) {
        const unsigned char* k_tile = wave_lds + (i % 2) * L::TILE_BYTES;
#pragma unroll
        for (int qs = 0; qs < QSUB; qs++)
#pragma unroll
            for (int v = 0; v < 16; v++) s_acc[qs][v] = 0.0f;
#pragma unroll
        for (int s = 0; s < QSTEPS; s++) {
            const Vec16 k_frag = *reinterpret_cast<const Vec16*>(k_tile + lane32 * L::ROW_BYTES + (((2 * s + half) ^ L::k_turn(lane32)) * 16));
#pragma unroll
            for (int qs = 0; qs < QSUB; qs++) s_acc[qs] = piece_product(k_frag, q_reg[qs][s], s_acc[qs]);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    // A wave alone on its SIMD pays a tile's chain in full (key fragments, score products, softmax, value fragments,
    // output products: 2,860 cycles a tile, of which the softmax arithmetic is 1,350), and the wave with the most tiles
    // is what the kernel waits for. So the scores of tile i + 1 are issued before the softmax of tile i and run under it.
    // Loads, in order: K0 V0 K1 V1 K2, then with tile i: K(i+3), V(i+2); a wait that leaves the newest n tiles' worth in
    // flight has everything older. Pages are looked up a tile before their loads.
    int page_v = 0, page_k = 0;  // of tiles i + 2 and i + 3
    f32x16 s_even[QSUB], s_odd[QSUB];
    if (n_mine > 0) {
        const int page0 = table[tile_base(0) >> page_shift], page1 = table[tile_base(1) >> page_shift];
        page_v = table[tile_base(2) >> page_shift];
        page_k = table[tile_base(3) >> page_shift];
        issue(0, page0, false);
        issue(0, page0, true);
        issue(1, page1, false);
        issue(1, page1, true);
        wait_vmcnt<3 * L::LOADS>();  // in flight: V0 K1 V1
        scores(0, s_even);
        issue(2, page_v, false);
    }

    auto tile = [&](int i, f32x16 (&s_acc)[QSUB], f32x16 (&s_next)[QSUB]) {
        const int page_next = table[tile_base(i + 4) >> page_shift];
        const int k0 = first_base + (wave + SPLITS * i) * KEYS;
        const unsigned char* v_tile = wave_lds + 2 * L::TILE_BYTES + (i % 2) * L::TILE_BYTES;
        const unsigned char* k_next = wave_lds + ((i + 1) % 2) * L::TILE_BYTES;
        bf16x8 p[QSUB][2];  // the probabilities of a sub-tile of queries, as the second product's operand: keys 0-15 and 16-31 of the tile
        wait_vmcnt<2 * L::LOADS>();  // K(i+1) has landed (and V(i)); beyond the wave's last tile: that tile again, its scores never used
        // the key fragments of tile i + 1 are asked for now and travel under the first sub-tile's softmax
        i32x4 k_frag[QSTEPS];
#pragma unroll
        for (int s = 0; s < QSTEPS; s++) ask_fragment(k_frag[s], lds_address(k_next + lane32 * L::ROW_BYTES + (((2 * s + half) ^ L::k_turn(lane32)) * 16)));

        // ---- mask (only where the tile touches the diagonal, a window or the portion's end), maximum, exponentials ----
        auto softmax = [&](int qs) {
            const int sub_first_position = context + tile_q0 + qs * 32;
            const bool interior = window == 0 && tile_q0 + qs * 32 + 31 < q_len && k0 + KEYS - 1 <= sub_first_position;
            float tile_max = -INFINITY;
            if (interior) {
#pragma unroll
                for (int v = 0; v < 16; v++) tile_max = fmaxf(tile_max, s_acc[qs][v]);
            } else {
                const int first_allowed = window > 0 ? q_position[qs] - window + 1 : 0;
                const int key0 = k0 + 4 * half;
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int key = key0 + 8 * (v / 4) + (v % 4);
                    const bool allowed = (key <= q_position[qs]) & (key >= first_allowed);
                    s_acc[qs][v] = allowed ? s_acc[qs][v] : -INFINITY;
                    tile_max = fmaxf(tile_max, s_acc[qs][v]);
                }
            }
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE)) * score_scale;
            const float new_max = fmaxf(running_max[qs], tile_max);
            const float safe_max = new_max == -INFINITY ? 0.0f : new_max;  // a query with no key yet
            if (__any(new_max > running_max[qs])) {  // some query's maximum rose: what has been summed so far shrinks
                const float rescale = weight_of(running_max[qs] - safe_max);
                running_sum[qs] *= rescale;
#pragma unroll
                for (int i2 = 0; i2 < DT; i2++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc_o[qs][i2][v] *= rescale;
            }
            running_max[qs] = new_max;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float p = weight_of(__builtin_fmaf(s_acc[qs][v], score_scale, -safe_max));
                s_acc[qs][v] = p;
                running_sum[qs] += p;
            }
            if constexpr (!FP32) {
#pragma unroll
                for (int slab = 0; slab < 2; slab++)
#pragma unroll
                    for (int e = 0; e < 8; e++) p[qs][slab][e] = static_cast<bf16_t>(s_acc[qs][8 * slab + e]);
            }
        };
        softmax(0);
        __builtin_amdgcn_sched_barrier(0);
        // the scores of tile i + 1: issued here, they run under the second sub-tile's softmax and the reads of the values
        fragments_landed(k_frag[0]);
#pragma unroll
        for (int s = 1; s < QSTEPS; s++) and_this_one(k_frag[s]);
        issue(i + 3, page_k, false);  // (the fragments are in registers: their place may be loaded into)
#pragma unroll
        for (int s = 0; s < QSTEPS; s++)
#pragma unroll
            for (int qs = 0; qs < QSUB; qs++) {
                f32x16 start = s_next[qs];
                if (s == 0) {
#pragma unroll
                    for (int v = 0; v < 16; v++) start[v] = 0.0f;
                }
                s_next[qs] = piece_product(*reinterpret_cast<const Vec16*>(&k_frag[s]), q_reg[qs][s], start);
            }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int qs = 1; qs < QSUB; qs++) softmax(qs);

        // ---- O^T += V^T . P^T : two slabs of 16 keys; a lane's eight are keys 4 half .. + 4 and 8 + 4 half .. + 4 of the slab ----
        wait_vmcnt<3 * L::LOADS>();  // the newest three are K(i+2) V(i+1) K(i+3): V(i) has landed
        if constexpr (FP32) {
            // 32-bit: O^T += V^T . P^T by products of two keys: register v of the scores holds, in the lanes of half h, key
            // 8 (v / 4) + 4 h + v % 4 of the tile, so product v takes that key's values (column 32 i2 + lane % 32, read as
            // stored) against the register itself. Eight values a read, for each 32 columns.
#pragma unroll
            for (int i2 = 0; i2 < DT; i2++) {
                const unsigned address = lds_address(v_tile + (4 * half) * L::ROW_BYTES + (i2 * 32 + lane32) * 4);
                float values[8];
                read_eight<L::ROW_BYTES, 0>(address, values);
#pragma unroll
                for (int e = 0; e < 8; e++)
#pragma unroll
                    for (int qs = 0; qs < QSUB; qs++) acc_o[qs][i2] = __builtin_amdgcn_mfma_f32_32x32x2f32(values[e], s_acc[qs][e], acc_o[qs][i2], 0, 0, 0);
                read_eight<L::ROW_BYTES, 1>(address, values);
#pragma unroll
                for (int e = 0; e < 8; e++)
#pragma unroll
                    for (int qs = 0; qs < QSUB; qs++) acc_o[qs][i2] = __builtin_amdgcn_mfma_f32_32x32x2f32(values[e], s_acc[qs][8 + e], acc_o[qs][i2], 0, 0, 0);
            }
        } else {
        short4_t v_frag[DT][4];      // per 32 columns: slab 0 low keys, slab 0 high keys, slab 1 low, slab 1 high
        {
            unsigned address[DT];
#pragma unroll
            for (int i2 = 0; i2 < DT; i2++) {
                const int col = i2 * 32 + v_col;  // the four columns this lane points at: inside one 16-byte piece
                const int key_lo = 4 * half + v_key_in_read;  // keys + 8, + 16, + 24 turn their rows the same way
                address[i2] = lds_address(v_tile + key_lo * L::ROW_BYTES + (((col / 8) ^ L::v_turn(key_lo)) * 16) + (col % 8) * 2);
            }
            read_transposed<DT, L::ROW_BYTES>(address, v_frag);  // returns when the fragments are in registers
        }
#pragma unroll
        for (int slab = 0; slab < 2; slab++) {
#pragma unroll
            for (int i2 = 0; i2 < DT; i2++) {
                bf16x8 fragment;
                short4_t* halves = reinterpret_cast<short4_t*>(&fragment);
                halves[0] = v_frag[i2][2 * slab];
                halves[1] = v_frag[i2][2 * slab + 1];
#pragma unroll
                for (int qs = 0; qs < QSUB; qs++) acc_o[qs][i2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fragment, p[qs][slab], acc_o[qs][i2], 0, 0, 0);
            }
        }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        issue(i + 2, page_v, true);
        page_v = page_k;
        page_k = page_next;
    };
    for (int i = 0; i < n_mine; i += 2) {
        tile(i, s_even, s_odd);
        if (i + 1 < n_mine) tile(i + 1, s_odd, s_even);
    }
    // the loads asked for beyond the last tile land, and the last reads return, before the tiles' place is written over
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");

    // ---- the four waves' partial results, combined: each wave writes its own where its tiles lay, then finishes a share ----
    float* partial = reinterpret_cast<float*>(lds + wave * L::WAVE_BYTES);
#pragma unroll
    for (int qs = 0; qs < QSUB; qs++) {
        running_sum[qs] += __shfl_xor(running_sum[qs], 32, WAVE);
        if (half == 0) {
            stats_lds[wave][qs * 32 + lane32][0] = running_max[qs];
            stats_lds[wave][qs * 32 + lane32][1] = running_sum[qs];
        }
#pragma unroll
        for (int i2 = 0; i2 < DT; i2++)
#pragma unroll
            for (int v = 0; v < 16; v++) partial[((qs * DT + i2) * 16 + v) * WAVE + lane] = acc_o[qs][i2][v];
    }
    __syncthreads();
    for (int share = wave; share < QSUB * DT; share += SPLITS) {
        const int qs = share / DT, i2 = share % DT;
        const int q_local = tile_q0 + qs * 32 + lane32;
        if (q_local >= q_len) continue;
        float best = -INFINITY;
#pragma unroll
        for (int w = 0; w < SPLITS; w++) best = fmaxf(best, stats_lds[w][qs * 32 + lane32][0]);  // finite: a query sees at least its own key
        float weight[SPLITS], total = 0.0f;
#pragma unroll
        for (int w = 0; w < SPLITS; w++) {
            weight[w] = weight_of(stats_lds[w][qs * 32 + lane32][0] - best);  // a wave that saw no key: a weight of 0
            total += weight[w] * stats_lds[w][qs * 32 + lane32][1];
        }
        const float inverse = 1.0f / total;
        T* out_row = out + (size_t)(q_first + q_local) * out_stride + head * HD + i2 * 32;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float sum = 0.0f;
#pragma unroll
                for (int w = 0; w < SPLITS; w++)
                    sum += weight[w] * reinterpret_cast<const float*>(lds + w * L::WAVE_BYTES)[(share * 16 + 4 * g + e) * WAVE + lane];
                o[e] = sum * inverse;
            }
            if constexpr (FP32) *reinterpret_cast<f32x4*>(out_row + 8 * g + 4 * half) = f32x4{o[0], o[1], o[2], o[3]};
            else *reinterpret_cast<bf16x4*>(out_row + 8 * g + 4 * half) = bf16x4{static_cast<bf16_t>(o[0]), static_cast<bf16_t>(o[1]), static_cast<bf16_t>(o[2]), static_cast<bf16_t>(o[3])};
        }
    }
}

// Whether prompt portions with these sizes take this kernel.
template <typename T>
inline bool takes(int head_size, int page_size, int max_q_len, float scale, int q_stride, int out_stride, const void* q, const void* out) {
    const int row_bytes = head_size * (int)sizeof(T);
    if (row_bytes != 64 && row_bytes != 128 && row_bytes != 256) return false;
    if (head_size < 32) return false;    // the output's rows are tiles of 32 head dimensions
    if (page_size < KEYS) return false;  // a tile of keys lies in one page (page sizes are powers of two)
    if (max_q_len <= 64) return false;   // shorter portions: the kernel with fewer queries a block
    if (!(scale > 0.0f)) return false;   // the maximum is taken before the scaling
    // 16-byte loads of q and 8- or 16-byte stores of out
    return (q_stride * sizeof(T)) % 16 == 0 && (out_stride * sizeof(T)) % (4 * sizeof(T)) == 0 && ((size_t)q) % 16 == 0 && ((size_t)out) % (4 * sizeof(T)) == 0;
}

template <typename T, int HD, int QUERIES, int SPLITS>
void launch_queries(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out, int out_stride, const int* q_starts,
                    const int* context_lens, const int* block_tables, int max_blocks, int n_requests, int max_q_len, int n_heads, int n_kv_heads,
                    int page_shift, int window, float scale, hipStream_t stream) {
    constexpr int LDS_BYTES = Layout<T, HD, SPLITS>::LDS_BYTES;
    static bool raised = false;  // per instantiation: the limit on dynamic LDS is a property of the kernel
    if (!raised && LDS_BYTES > 60 * 1024)  // (if this fails the launch below fails too, and the entry point reports that)
        raised = hipFuncSetAttribute((const void*)attention_prefill_stream_kernel<T, HD, QUERIES, SPLITS>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) == hipSuccess;
    // x: (request, head), so that with a multiple of eight heads the blocks of one head share an XCD's L2; y: tiles of queries
    dim3 grid(n_heads * n_requests, ceil_div(max_q_len, QUERIES));
    mllm_count_kernel(MLLM_K_ATTENTION_PREFILL_STREAM);
    attention_prefill_stream_kernel<T, HD, QUERIES, SPLITS><<<grid, 64 * SPLITS, LDS_BYTES, stream>>>(
        (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, (T*)out, out_stride, q_starts, context_lens,
        block_tables, max_blocks, n_heads, n_kv_heads, page_shift, window, scale);
}

template <typename T, int HD>
void launch(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out, int out_stride, const int* q_starts,
            const int* context_lens, const int* block_tables, int max_blocks, int n_requests, int max_q_len, int max_len, int n_heads,
            int n_kv_heads, int page_shift, int window, float scale, hipStream_t stream) {
#define MLLM_STREAM_LAUNCH(QUERIES, SPLITS)                                                                                                 \
    launch_queries<T, HD, QUERIES, SPLITS>(q, q_stride, k_pages, v_pages, out, out_stride, q_starts, context_lens, block_tables, max_blocks, \
                                           n_requests, max_q_len, n_heads, n_kv_heads, page_shift, window, scale, stream)
    if constexpr (sizeof(T) == 4) {
        // 32-bit: the matrix cores are what a wave waits for (a tile of 32 keys is 96 products of 64 cycles for 32 queries),
        // so blocks of 32 queries, which the compute units take in turn, the ones with the most keys first
        // (blocks of 64 queries: 59.2 against 62.1 us for two prompts of 1,024 tokens x 12 heads of 64, 35.0 against 32.2 us for eight of 256)
        MLLM_STREAM_LAUNCH(32, 4);
    } else {
        // blocks of 64 queries where they give every compute unit a block (measured: 2 x 1,024 tokens x 12 heads 15.9 against 17.2 us),
        // else of 32 (4 x 128 tokens on 896 cached: 9.7 against 13.0 us; 512 on 7,680: 46.7 against 66.0 us)
        const bool wide = (long)n_heads * n_requests * ceil_div(max_q_len, 64) >= 256;
        // Eight waves a block where the block of the last queries has sixteen tiles of keys or more to walk (max_len: the longest
        // sequence after this step, or what bounds it; a window bounds the keys too) AND every block still finds a compute
        // unit of its own at once (eight waves' tiles leave room for one block a unit): a long context with few queries.
        // Measured, heads of 64: 512 queries on 7,680 cached keys 38.2 against 46.7 us with four waves; but two prompts of 1,024
        // tokens (384 blocks: a second round) 19.1 against 15.9 us, one of 4,096 64.8 against 57 us.
        const int reach = window > 0 ? min(max_len, window + 64) : max_len;
        const long blocks = (long)n_heads * n_requests * ceil_div(max_q_len, wide ? 64 : 32);
        bool eight = false;
        if constexpr (HD * sizeof(T) <= 128) {  // (eight waves' tiles of rows of 256 bytes do not fit a compute unit's LDS)
            eight = reach >= 16 * KEYS && blocks <= 256;
            if (wide && eight) MLLM_STREAM_LAUNCH(64, 8);
            else if (eight) MLLM_STREAM_LAUNCH(32, 8);
        }
        if (wide && !eight) MLLM_STREAM_LAUNCH(64, 4);
        else if (!eight) MLLM_STREAM_LAUNCH(32, 4);
    }
#undef MLLM_STREAM_LAUNCH
}

}  // namespace prefill_stream
