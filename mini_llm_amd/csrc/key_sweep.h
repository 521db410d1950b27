// One wave's pass over a run of cached keys of one request and head, shared by the kernels that
// decode: scores, online softmax in 32-bit and the unnormalised value sum.
//
// The rows of one head inside a page lie together, so a wave reads them as one contiguous
// stream: each lane loads 16 bytes, LPR = head bytes / 16 lanes share a row, and one load
// instruction covers RPI = 64 / LPR consecutive keys. A lane therefore holds VEC head dimensions
// (those from sub * VEC on, sub = lane % LPR) of several keys; dot products are finished with
// shuffles inside the LPR lanes, and the value sums stay per lane until merge_groups().
#pragma once

#include "common.h"

template <typename T>
struct Chunk;  // 16 bytes of a row
template <>
struct Chunk<float> {
    static constexpr int VEC = 4;
    typedef f32x4 Raw;
    static __device__ __forceinline__ float get(const Raw& r, int i) { return r[i]; }
};
template <>
struct Chunk<bf16_t> {
    static constexpr int VEC = 8;
    typedef bf16x8 Raw;
    static __device__ __forceinline__ float get(const Raw& r, int i) { return static_cast<float>(r[i]); }
};

// e^x for the softmax weights of a sweep. In 32-bit the library's expf; where keys and values are bfloat16 (eight bits
// of fraction) the hardware's 2^x of x log2(e), three instructions instead of a score of them and one unit in the last
// place of a 32-bit result: the sweep's arithmetic is what a decode step's attention waits for once its rows are there.
template <typename T>
__device__ __forceinline__ float sweep_exp(float x) {
    if constexpr (sizeof(T) == 2) return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
    else return expf(x);
}

template <typename T, int HD>
struct KeySweep {
    static constexpr int VEC = Chunk<T>::VEC;
    static constexpr int LPR = HD / VEC;      // lanes that share a row
    static constexpr int RPI = WAVE / LPR;    // rows one load instruction covers
    static constexpr int UNROLL = 8;
    static constexpr int KPI = RPI * UNROLL;  // keys per iteration
    static_assert(HD % VEC == 0 && (LPR & (LPR - 1)) == 0 && LPR <= WAVE, "head size must be a power of two");
    typedef typename Chunk<T>::Raw Raw;

    float o[VEC];         // this lane's share of sum p * v, dimensions sub * VEC ..
    float running_max;    // the same in every lane
    float running_sum;    // this lane's share until merge_groups()

    __device__ __forceinline__ void init() {
#pragma unroll
        for (int i = 0; i < VEC; i++) o[i] = 0.0f;
        running_max = -INFINITY;
        running_sum = 0.0f;
    }

    // KPI keys as loaded: converted where they are used.
    struct Fetched {
        Raw kf[UNROLL], vf[UNROLL];
    };

    // The pages of the keys base .. base+KPI-1 of the request whose block table is given, those
    // from `end` on replaced by `spare_key` (any key whose page the table holds): the first half of
    // fetch(), for a caller that wants the table's answer under way before it asks for the rows.
    __device__ __forceinline__ void look_up(int (&page)[UNROLL], const int* __restrict__ table, int page_shift,
                                            int base, int end, int spare_key, int lane) const {
        const int group = lane / LPR;
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            int key = base + u * RPI + group;
            page[u] = table[(key < end ? key : spare_key) >> page_shift];
        }
    }

    // Asks for those keys and values, given their pages. No branch between the loads: all are in
    // flight together, and nothing here waits for them. KEYS / VALUES: which of the two to ask for.
    template <bool KEYS = true, bool VALUES = true>
    __device__ __forceinline__ void fetch_rows(Fetched& f, const int (&page)[UNROLL], const T* __restrict__ k_pages,
                                               const T* __restrict__ v_pages, int kv_head, int n_kv_heads, int page_shift,
                                               int base, int end, int spare_key, int lane) const {
        const int sub = lane % LPR, group = lane / LPR;
        const int page_mask = (1 << page_shift) - 1;
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            int key = base + u * RPI + group;
            int safe_key = key < end ? key : spare_key;
            size_t row = ((((size_t)page[u] * n_kv_heads + kv_head) << page_shift) + (safe_key & page_mask));
            if constexpr (KEYS) f.kf[u] = *reinterpret_cast<const Raw*>(k_pages + row * HD + sub * VEC);
            if constexpr (VALUES) f.vf[u] = *reinterpret_cast<const Raw*>(v_pages + row * HD + sub * VEC);
        }
    }

    // Both halves at once.
    template <bool KEYS = true, bool VALUES = true>
    __device__ __forceinline__ void fetch(Fetched& f, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                                          const int* __restrict__ table, int kv_head, int n_kv_heads, int page_shift,
                                          int base, int end, int spare_key, int lane) const {
        int page[UNROLL];
        look_up(page, table, page_shift, base, end, spare_key, lane);
        fetch_rows<KEYS, VALUES>(f, page, k_pages, v_pages, kv_head, n_kv_heads, page_shift, base, end, spare_key, lane);
    }

    // Takes the fetched keys base .. min(base+KPI, end)-1 (there may be none) into the running softmax.
    // qf: the lane's VEC dimensions of the query, already scaled.
    // CLEAN_VALUES: a key that does not count may have been fetched from memory nobody has written
    // yet (the spare key of a wave without keys); its value then is replaced by zero, as not even
    // a weight of zero silences a NaN.
    template <bool CLEAN_VALUES = false>
    __device__ __forceinline__ void consume(const Fetched& f, const float (&qf)[VEC], int base, int end, int lane) {
        float dots[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            float dot = 0.0f;
#pragma unroll
            for (int i = 0; i < VEC; i++) dot += qf[i] * Chunk<T>::get(f.kf[u], i);
            dots[u] = dot;
        }
        take<CLEAN_VALUES>(f, dots, base, end, lane);
    }

    // The same for a query kept as it is stored, in bfloat16 (the lane's VEC dimensions), and the factor its scores are
    // scaled by: the products of two bfloat16 numbers are exact in 32-bit, so a dot product over pairs (v_dot2c_f32_bf16)
    // gives what the converted numbers would, in a quarter of the instructions.
    template <bool CLEAN_VALUES = false>
    __device__ __forceinline__ void consume(const Fetched& f, const Raw& q, float scale, int base, int end, int lane) {
        static_assert(sizeof(T) == 2, "a query in bfloat16 meets keys in bfloat16");
        float dots[UNROLL];
        const bf16x2* q_pairs = reinterpret_cast<const bf16x2*>(&q);
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const bf16x2* k_pairs = reinterpret_cast<const bf16x2*>(&f.kf[u]);
            float dot = 0.0f;
#pragma unroll
            for (int i = 0; i < VEC / 2; i++) dot = __builtin_amdgcn_fdot2_f32_bf16(q_pairs[i], k_pairs[i], dot, false);
            dots[u] = dot * scale;
        }
        take<CLEAN_VALUES>(f, dots, base, end, lane);
    }

    // dots: this lane's share of the scaled dot products of the fetched keys with the query.
    template <bool CLEAN_VALUES>
    __device__ __forceinline__ void take(const Fetched& f, const float (&dots)[UNROLL], int base, int end, int lane) {
        const int group = lane / LPR;
        float score[UNROLL];
        float tile_max = -INFINITY;
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            float dot = lanes_sum<LPR>(dots[u]);
            score[u] = base + u * RPI + group < end ? dot : -INFINITY;
            tile_max = fmaxf(tile_max, score[u]);
        }
        tile_max = wave_max_total(tile_max);
        float new_max = fmaxf(running_max, tile_max);
        float reference = new_max == -INFINITY ? 0.0f : new_max;  // no key so far (base >= end is allowed): nothing to rescale
        float rescale = sweep_exp<T>(running_max - reference);
        running_sum *= rescale;
#pragma unroll
        for (int i = 0; i < VEC; i++) o[i] *= rescale;
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const bool counts = base + u * RPI + group < end;
            float p = counts ? sweep_exp<T>(score[u] - reference) : 0.0f;
            running_sum += p;
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                float value = Chunk<T>::get(f.vf[u], i);
                if (CLEAN_VALUES && !counts) value = 0.0f;
                o[i] += p * value;
            }
        }
        running_max = new_max;
    }

    // Keys begin .. end-1 (begin < end).
    __device__ __forceinline__ void keys(const float (&qf)[VEC], const T* __restrict__ k_pages,
                                         const T* __restrict__ v_pages, const int* __restrict__ table,
                                         int kv_head, int n_kv_heads, int page_shift, int begin, int end, int lane) {
        for (int base = begin; base < end; base += KPI) {
            Fetched f;
            fetch(f, k_pages, v_pages, table, kv_head, n_kv_heads, page_shift, base, end, end - 1, lane);
            consume(f, qf, base, end, lane);
        }
    }

    // The same with the query as it is stored (bfloat16).
    __device__ __forceinline__ void keys(const Raw& q, float scale, const T* __restrict__ k_pages,
                                         const T* __restrict__ v_pages, const int* __restrict__ table,
                                         int kv_head, int n_kv_heads, int page_shift, int begin, int end, int lane) {
        for (int base = begin; base < end; base += KPI) {
            Fetched f;
            fetch(f, k_pages, v_pages, table, kv_head, n_kv_heads, page_shift, base, end, end - 1, lane);
            consume(f, q, scale, base, end, lane);
        }
    }

    // One more key that is not in the cache: key_row and value_row hold its HD dimensions in
    // 32-bit (LDS or memory). Counted once, by the lanes of row group 0.
    __device__ __forceinline__ void one_key(const float (&qf)[VEC], const float* key_row, const float* value_row, int lane) {
        const int sub = lane % LPR, group = lane / LPR;
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < VEC; i++) dot += qf[i] * key_row[sub * VEC + i];
        dot = lanes_sum<LPR>(dot);
        float new_max = fmaxf(running_max, dot);
        float rescale = sweep_exp<T>(running_max - new_max);
        running_sum *= rescale;
        float p = group == 0 ? sweep_exp<T>(dot - new_max) : 0.0f;
        running_sum += p;
#pragma unroll
        for (int i = 0; i < VEC; i++) o[i] = o[i] * rescale + p * value_row[sub * VEC + i];
        running_max = new_max;
    }

    // Every lane of a row group counted the same keys: the shares of the groups inside each row of
    // 16 lanes are added up (lanes LPR apart hold the same dimensions), after which the first LPR
    // lanes of a row hold that row's output and every lane of the row its sum. A no-op for rows
    // that are one group (LPR >= 16).
    __device__ __forceinline__ void merge_inside_rows() {
        if constexpr (LPR < 16) {
            running_sum = row_strided_sum<LPR>(running_sum);
#pragma unroll
            for (int i = 0; i < VEC; i++) o[i] = row_strided_sum<LPR>(o[i]);
        }
    }

    // All groups of the wave: after it every lane holds the wave's sum and lanes 0..LPR-1 its output.
    __device__ __forceinline__ void merge_groups() {
        merge_inside_rows();
#pragma unroll
        for (int offset = LPR < 16 ? 16 : LPR; offset < WAVE; offset <<= 1) {
            running_sum += __shfl_xor(running_sum, offset, WAVE);
#pragma unroll
            for (int i = 0; i < VEC; i++) o[i] += __shfl_xor(o[i], offset, WAVE);
        }
    }
};
