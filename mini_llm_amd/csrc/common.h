// Shared by every kernel file of the library: element types, conversions, wave reductions and
// the error convention of the C entry points (0 = launched, anything else = refused; the text is
// read with mllm_last_error()).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define MLLM_API extern "C" __attribute__((visibility("default")))

// Element types as the Python side names them.
enum MllmDtype : int { MLLM_F32 = 0, MLLM_BF16 = 1 };

// What a matrix product does to its sums before it stores them.
enum MllmEpilogue : int {
    MLLM_EPI_NONE = 0,       // (+ bias)
    MLLM_EPI_GELU_TANH = 1,  // gelu_new(+ bias)
    MLLM_EPI_GELU_ERF = 2,   // gelu(+ bias)
};

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int WAVE = 64;

// 16 bytes moved as one piece, whatever they hold.
struct alignas(16) Vec16 {
    uint32_t w[4];
};

// The packed layout of a weight matrix W [rows, cols]: chunks of 16 rows x 64 bytes (32 bfloat16 or
// 16 float columns), row tiles outermost, zeros beyond the matrix. Inside a chunk piece p (16
// bytes) holds row p % 16, columns (p / 16) * VEC .. of the chunk: exactly what lane p of a wave
// feeds a 16x16 MFMA as its 16-row operand. A wave therefore loads a chunk as 1 KiB of contiguous
// memory, straight into operand registers; from row-major memory the same load would touch 16
// cache lines per quarter wave, which the vector cache serves several times slower.
template <typename T>
__host__ __device__ __forceinline__ size_t packed_offset(int row_tile, int k_step, int k_steps, int lane) {
    return (((size_t)row_tile * k_steps + k_step) * 64 + lane) * (16 / sizeof(T));
}
template <typename T>
__host__ __device__ __forceinline__ int packed_k_steps(int cols) {
    return (cols * (int)sizeof(T) + 63) / 64;
}

// Where element (row, col) of a [rows, cols] matrix lies in the packed layout. Rows of activations
// are kept this way too when a product of few rows reads them next (its kernel loads whole chunks).
template <typename T>
__host__ __device__ __forceinline__ size_t packed_element(int row, int col, int cols) {
    constexpr int VEC = 16 / (int)sizeof(T), KC = 4 * VEC;
    const int in_chunk = col % KC;
    return packed_offset<T>(row / 16, col / KC, packed_k_steps<T>(cols), (in_chunk / VEC) * 16 + row % 16) + in_chunk % VEC;
}

void mllm_set_error(const char* format, ...);
int mllm_check_launch(const char* what);

// Every kernel launch is counted by kind, on the host (what the reference's launch counter is for,
// engine/include/cuda_check.h:21-41: a test can tell which kernels a step took and how many).
// Launches recorded into a graph count when they are captured, not when the graph is replayed.
enum MllmKernel : int {
    MLLM_K_EMBED = 0, MLLM_K_LAYERNORM, MLLM_K_ADD, MLLM_K_CACHE_WRITE, MLLM_K_ATTENTION_GENERAL, MLLM_K_ATTENTION_DECODE,
    MLLM_K_ATTENTION_PREFILL, MLLM_K_ATTENTION_PREFILL_STREAM, MLLM_K_PACK, MLLM_K_CONVERT, MLLM_K_DECODE_ATTENTION_HALF,
    MLLM_K_DECODE_MLP_HALF, MLLM_K_PENDING_SUM, MLLM_K_PENDING_LAYERNORM, MLLM_K_GEMM_SKINNY, MLLM_K_GEMM_TILED, MLLM_K_GEMM_STREAM,
    MLLM_K_STATIC_SUM, MLLM_K_PROBE, MLLM_K_SAMPLE, MLLM_K_GEMM_BEST, MLLM_K_CHOOSE, MLLM_K_KINDS
};
void mllm_count_kernel(MllmKernel kind);

#define MLLM_REQUIRE(condition, ...)      \
    do {                                  \
        if (!(condition)) {               \
            mllm_set_error(__VA_ARGS__);  \
            return 1;                     \
        }                                 \
    } while (0)

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return static_cast<float>(x); }

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) {
    return x;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
    return static_cast<bf16_t>(x);  // round to nearest even
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, WAVE);
    return v;
}

// The sum over a wave without a trip through the LDS crossbar: four steps between neighbours
// inside rows of 16 lanes (data-parallel primitives: a few cycles each), then the four row sums are
// read out and added. Every lane gets the result; the order of the additions is fixed.
template <int CONTROL>
__device__ __forceinline__ float dpp_moved(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CONTROL, 0xf, 0xf, false));
}
__device__ __forceinline__ float wave_total(float v) {
    v += dpp_moved<0xB1>(v);   // lanes 1,0,3,2 of each four
    v += dpp_moved<0x4E>(v);   // lanes 2,3,0,1 of each four
    v += dpp_moved<0x141>(v);  // the other four of each eight (mirrored)
    v += dpp_moved<0x140>(v);  // the other eight of each sixteen (mirrored)
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (r0 + r1) + (r2 + r3);
}

// (value, index) a comes before b: a NaN beats every number, a larger number a smaller one, and
// among equals (-0 equals +0) the smaller index wins. These are numpy.argmax's rules, which the
// reference keeps (engine/include/argmax.h:10-16, engine/src/argmax.cu:8-18). A total order: the
// best of a set does not depend on the order in which its members are compared.
__device__ __forceinline__ bool beats(float value, int index, float best, int best_index) {
    bool value_nan = value != value, best_nan = best != best;
    if (value_nan != best_nan) return value_nan;
    if (value_nan || value == best) return index < best_index;
    return value > best;
}

// Where a product leaves, instead of its sums, the best of them per row: each block writes the best
// (value, column) among its columns of a row to values/indices[row * per_row + block along N]. Whoever picks the row's best among them gets the argmax of the
// row by the rules above, and the sums themselves need not be written (a greedy step's logits).
struct BestOfColumns {
    float* values;
    int* indices;
    int per_row;
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, WAVE));
    return v;
}

// The sum over each aligned group of N neighbouring lanes (N a power of two), in every lane of the
// group: data-parallel steps inside rows of 16 lanes, the LDS crossbar only between rows.
template <int N>
__device__ __forceinline__ float lanes_sum(float v) {
    if constexpr (N >= 2) v += dpp_moved<0xB1>(v);
    if constexpr (N >= 4) v += dpp_moved<0x4E>(v);
    if constexpr (N >= 8) v += dpp_moved<0x141>(v);
    if constexpr (N >= 16) v += dpp_moved<0x140>(v);
    if constexpr (N >= 32) v += __shfl_xor(v, 16, WAVE);
    if constexpr (N >= 64) v += __shfl_xor(v, 32, WAVE);
    return v;
}

// The sum over the lanes of a row of 16 that lie STEP apart (STEP a power of two), in each of
// them: rotations of the row by STEP, 2 STEP, ...
template <int STEP>
__device__ __forceinline__ float row_strided_sum(float v) {
    if constexpr (STEP <= 1) v += dpp_moved<0x121>(v);
    if constexpr (STEP <= 2) v += dpp_moved<0x122>(v);
    if constexpr (STEP <= 4) v += dpp_moved<0x124>(v);
    if constexpr (STEP <= 8) v += dpp_moved<0x128>(v);
    return v;
}

// The maximum over a wave, in every lane: four steps inside the rows, then the four rows' maxima.
__device__ __forceinline__ float wave_max_total(float v) {
    v = fmaxf(v, dpp_moved<0xB1>(v));
    v = fmaxf(v, dpp_moved<0x4E>(v));
    v = fmaxf(v, dpp_moved<0x141>(v));
    v = fmaxf(v, dpp_moved<0x140>(v));
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// tanh form of GELU, in the reference's order of operations (engine/include/gelu_math.h:6-11).
__device__ __forceinline__ float gelu_tanh(float x) {
    const float coefficient = 0.7978845608f;
    const float cubic = 0.044715f;
    float argument = coefficient * (x + cubic * x * x * x);
    return 0.5f * x * (1.0f + tanhf(argument));
}

// exact GELU (engine/src/gelu.c:5-9).
__device__ __forceinline__ float gelu_erf(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}

// The same two functions for results that are rounded to bfloat16 (eight bits of fraction) right
// after: a dozen instructions each instead of the library's tanhf / erff, still in 32-bit.
// tanh form: 0.5 x (1 + tanh(u)) = x / (1 + e^(-2u)), with the hardware's exp2 and reciprocal
// (one unit in the last place each).
__device__ __forceinline__ float gelu_tanh_for_bf16(float x) {
    // -2 log2(e) u = x (a + b x^2) with a = -2 log2(e) sqrt(2/pi), b = 0.044715 a: seven instructions
    const float a = -2.3022081986f, b = -0.1029432396f;
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * __builtin_fmaf(x * x, b, a)));
}

// erf form: erf by the rational approximation 7.1.26 of Abramowitz and Stegun (absolute error
// below 1.5e-7, a thousandth of what the rounding to bfloat16 leaves).
__device__ __forceinline__ float gelu_erf_for_bf16(float x) {
    float z = fabsf(x) * 0.70710678118654752440f;
    float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
    float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    float erf_abs = 1.0f - poly * __builtin_amdgcn_exp2f(-1.4426950408889634f * z * z);
    return 0.5f * x * (1.0f + copysignf(erf_abs, x));
}

template <int EPI>
__device__ __forceinline__ float apply_activation(float x) {
    if constexpr (EPI == MLLM_EPI_GELU_TANH) return gelu_tanh(x);
    if constexpr (EPI == MLLM_EPI_GELU_ERF) return gelu_erf(x);
    return x;
}

__host__ __device__ static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
