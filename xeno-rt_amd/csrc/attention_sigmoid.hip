// Causal attention over the paged cache whose weights are not a softmax: the weight of a visible key is
// sigmoid(score + head_bias[h]), and the weighted values are summed as they are, with no normalisation over the keys.
// Before the sigmoid the heads' scaled scores of a (query, key) pair may be mixed with one another,
// score_h <- sum_g head_mix[h][g] * score_g (a matrix [heads][heads]); after the sum a head's output may be multiplied by
// sigmoid(gate[token][h]), one number per token and head. Grouped key/value heads, values of a width of their own, a window.
// Float32 arithmetic for either element type.
//
// A mix of the heads needs all heads' scores of a pair at once, so a workgroup owns a token with all its heads. Its
// wavefronts deal the cache blocks of the token's keys among themselves by the block's absolute number; a wavefront takes
// a block's 64 keys a lane each (scores of all heads, through LDS to the mix and the sigmoid), then its lanes change to a
// value dim each and add the block's weighted values to the head's sums in LDS. In the end the wavefronts' sums are added
// in their order. Which wavefront takes which block, and so the order of every sum, depends on the key's position alone:
// a token's output is the same bits however its request was cut into steps or batched.
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

constexpr int TOGETHER = 4;                  // query heads of one key/value head that share every load of a key or a value
constexpr int MOST_LDS = 160 * 1024;

template <typename T>
__device__ __forceinline__ void eight(const T* __restrict__ p, float (&v)[8]) {
    if constexpr (sizeof(T) == 4) {
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        struct alignas(16) Eight { T e[8]; };
        const Eight q = *reinterpret_cast<const Eight*>(p);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = to_float(q.e[e]);
    }
}

__device__ __forceinline__ float sigmoid_exact(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T, int WAVES>
__global__ void __launch_bounds__(WAVES * XRT_WAVE) attention_sigmoid_kernel(
    const T* __restrict__ q, long q_stride, int n_heads, int n_kv_heads, int head_dim, int value_dim,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int* __restrict__ block_table, int table_stride, int n_blocks,
    const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ out, float scale, int window,
    const float* __restrict__ head_mix, const float* __restrict__ head_bias, const float* __restrict__ gate, long gate_stride,
    int whole_keys, int whole_values) {
    extern __shared__ float lds[];
    float* qs = lds;                                                   // [heads][head_dim]
    float* raw = qs + n_heads * head_dim;                              // [WAVES][heads][64]: scaled scores, lane j's key
    float* wts = raw + WAVES * n_heads * XRT_WAVE;                     // [WAVES][heads][64]: the weights after mix and sigmoid
    float* sums = wts + WAVES * n_heads * XRT_WAVE;                    // [WAVES][heads][value_dim]
    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
    const long token = blockIdx.x;
    const int out_width = n_heads * value_dim;
    T* dst = out + token * out_width;
    const int slot = slots[token];
    if (slot < 0) {
        for (int i = threadIdx.x; i < out_width; i += WAVES * XRT_WAVE) dst[i] = from_float<T>(0.f);
        return;
    }
    const int pos = positions[token];
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const int group = n_heads / n_kv_heads;
    const T* q_row = q + token * q_stride;
    for (int i = threadIdx.x; i < n_heads * head_dim; i += WAVES * XRT_WAVE) qs[i] = to_float(q_row[i]);
    for (int i = threadIdx.x; i < WAVES * out_width; i += WAVES * XRT_WAVE) sums[i] = 0.f;
    __syncthreads();

    float* my_raw = raw + wave * n_heads * XRT_WAVE;
    float* my_wts = wts + wave * n_heads * XRT_WAVE;
    float* my_sums = sums + wave * out_width;
    const int* table = block_table + (long)slot * table_stride;
    const int first_block = first / XRT_BLOCK_TOKENS, last_block = pos / XRT_BLOCK_TOKENS;
    for (int b = first_block; b <= last_block; ++b) {
        if (b % WAVES != wave) continue;
        const int block = table[b];
        if (block < 0 || block >= n_blocks) continue;                  // the host never lets this happen
        const int j = b * XRT_BLOCK_TOKENS + lane;
        const bool valid = j >= first && j <= pos;
        // ---- scores: lane j's key against every head's query
        for (int kv_head = 0; kv_head < n_kv_heads; ++kv_head) {
            const long key_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * head_dim;
            for (int h0 = 0; h0 < group; h0 += TOGETHER) {
                const int n_set = min(TOGETHER, group - h0);
                const float* q_set = qs + (kv_head * group + h0) * head_dim;
                float dot[TOGETHER];
#pragma unroll
                for (int s = 0; s < TOGETHER; ++s) dot[s] = 0.f;
                if (valid) {
                    if (whole_keys) {
#pragma unroll 2
                        for (int d0 = 0; d0 < head_dim; d0 += 8) {
                            float key[8];
                            eight(k_cache + key_base + cache_key_offset(lane, d0, head_dim), key);
#pragma unroll
                            for (int s = 0; s < TOGETHER; ++s) {
                                if (s < n_set) {
                                    float of_piece = 0.f;
#pragma unroll
                                    for (int e = 0; e < 8; ++e) of_piece = fmaf(q_set[s * head_dim + d0 + e], key[e], of_piece);
                                    dot[s] += of_piece;
                                }
                            }
                        }
                    } else {
                        for (int d0 = 0; d0 < head_dim; d0 += 8) {
                            const int dims = min(8, head_dim - d0);
#pragma unroll
                            for (int s = 0; s < TOGETHER; ++s) {
                                if (s < n_set) {
                                    float of_piece = 0.f;
                                    for (int e = 0; e < dims; ++e)
                                        of_piece = fmaf(q_set[s * head_dim + d0 + e],
                                                        to_float(k_cache[key_base + cache_key_offset(lane, d0 + e, head_dim)]), of_piece);
                                    dot[s] += of_piece;
                                }
                            }
                        }
                    }
                }
#pragma unroll
                for (int s = 0; s < TOGETHER; ++s)
                    if (s < n_set) my_raw[(kv_head * group + h0 + s) * XRT_WAVE + lane] = dot[s] * scale;
            }
        }
        // ---- the heads' scores of this lane's key mixed, biased, through the sigmoid (a lane reads only what it wrote)
        for (int h = 0; h < n_heads; ++h) {
            float s = 0.f;
            if (head_mix != nullptr) {
                for (int g = 0; g < n_heads; ++g) s = fmaf(head_mix[h * n_heads + g], my_raw[g * XRT_WAVE + lane], s);
            } else {
                s = my_raw[h * XRT_WAVE + lane];
            }
            if (head_bias != nullptr) s += head_bias[h];
            my_wts[h * XRT_WAVE + lane] = valid ? sigmoid_exact(s) : 0.f;
        }
        wave_sync();
        // ---- weighted values: a lane takes a value dim, the block's tokens in their order
        const int j_begin = max(0, first - b * XRT_BLOCK_TOKENS);
        const int j_end = min(XRT_BLOCK_TOKENS - 1, pos - b * XRT_BLOCK_TOKENS);
        for (int d = lane; d < value_dim; d += XRT_WAVE) {
            for (int kv_head = 0; kv_head < n_kv_heads; ++kv_head) {
                const long value_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * value_dim;
                for (int h0 = 0; h0 < group; h0 += TOGETHER) {
                    const int n_set = min(TOGETHER, group - h0);
                    const float* w_set = my_wts + (kv_head * group + h0) * XRT_WAVE;
                    float sum[TOGETHER];
#pragma unroll
                    for (int s = 0; s < TOGETHER; ++s) sum[s] = 0.f;
                    for (int j0 = j_begin / 8 * 8; j0 <= j_end; j0 += 8) {
                        float value[8];
                        const T* piece = v_cache + value_base + cache_value_offset(d, j0, value_dim);
                        if (whole_values) {
                            eight(piece, value);                       // (what lies beyond the sequence's end is loaded and not used)
                        } else {
#pragma unroll
                            for (int e = 0; e < 8; ++e) value[e] = to_float(piece[e]);
                        }
#pragma unroll
                        for (int s = 0; s < TOGETHER; ++s) {
                            if (s < n_set) {
#pragma unroll
                                for (int e = 0; e < 8; ++e)
                                    if (j0 + e >= j_begin && j0 + e <= j_end) sum[s] = fmaf(w_set[s * XRT_WAVE + j0 + e], value[e], sum[s]);
                            }
                        }
                    }
#pragma unroll
                    for (int s = 0; s < TOGETHER; ++s)
                        if (s < n_set) my_sums[(kv_head * group + h0 + s) * value_dim + d] += sum[s];
                }
            }
        }
        wave_sync();
    }
    __syncthreads();
    for (int i = threadIdx.x; i < out_width; i += WAVES * XRT_WAVE) {
        float total = sums[i];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) total += sums[w * out_width + i];
        if (gate != nullptr) total *= sigmoid_exact(gate[token * gate_stride + i / value_dim]);
        dst[i] = from_float<T>(total);
    }
}

size_t lds_bytes(int waves, int n_heads, int head_dim, int value_dim) {
    return sizeof(float) * ((size_t)n_heads * head_dim + (size_t)2 * waves * n_heads * XRT_WAVE + (size_t)waves * n_heads * value_dim);
}

template <typename T, int WAVES>
int launch(const void* q, long q_stride, long tokens, int n_heads, int n_kv_heads, int head_dim, int value_dim, const void* k_cache,
           const void* v_cache, const int* block_table, int table_stride, int n_blocks, const int* positions, const int* slots, void* out,
           float scale, int window, const float* head_mix, const float* head_bias, const float* gate, long gate_stride, hipStream_t s) {
    const size_t bytes = lds_bytes(WAVES, n_heads, head_dim, value_dim);
    auto kernel = attention_sigmoid_kernel<T, WAVES>;
    static bool allowed = false;                                       // (once per kernel: the most LDS it may ever ask for)
    if (!allowed) {
        const hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, MOST_LDS);
        XRT_REQUIRE(status == hipSuccess, "attention (sigmoid): %d bytes of LDS were refused: %s", MOST_LDS, hipGetErrorString(status));
        allowed = true;
    }
    const int whole_keys = head_dim % 8 == 0 && (uintptr_t)k_cache % 32 == 0;
    const int whole_values = (uintptr_t)v_cache % 32 == 0;
    kernel<<<(unsigned)tokens, WAVES * XRT_WAVE, bytes, s>>>((const T*)q, q_stride, n_heads, n_kv_heads, head_dim, value_dim, (const T*)k_cache,
        (const T*)v_cache, block_table, table_stride, n_blocks, positions, slots, (T*)out, scale, window, head_mix, head_bias, gate,
        gate_stride, whole_keys, whole_values);
    XRT_LAUNCH_CHECK("attention (sigmoid)");
    return 0;
}

}  // namespace

extern "C" int xrt_attention_sigmoid(const void* q, long q_stride, int dtype, long tokens, int n_heads, int n_kv_heads, int head_dim,
                                     int value_dim, const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                                     int n_blocks, const int* positions, const int* slots, void* out, float scale, int window,
                                     const float* head_mix, const float* head_bias, const float* gate, long gate_stride, void* stream) {
    XRT_REQUIRE(tokens >= 0 && tokens < (1L << 31) && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention (sigmoid): head counts %d/%d: the first must be a multiple of the second", n_heads, n_kv_heads);
    XRT_REQUIRE(head_dim > 0 && value_dim > 0, "attention (sigmoid): head sizes %d and %d must be positive", head_dim, value_dim);
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "attention (sigmoid): unknown dtype %d", dtype);
    XRT_REQUIRE(q && k_cache && v_cache && block_table && positions && slots && out, "attention (sigmoid): null operand");
    XRT_REQUIRE(q_stride >= (long)n_heads * head_dim && (gate == nullptr || gate_stride >= n_heads), "attention (sigmoid): a row stride is shorter than its heads");
    XRT_REQUIRE(table_stride > 0 && n_blocks > 0 && window >= 0, "attention (sigmoid): empty cache or negative window");
    if (tokens == 0) return 0;
    // as many wavefronts a token as the LDS holds sums for: a model's sizes decide, never the step
    int waves = 4;
    while (waves > 1 && lds_bytes(waves, n_heads, head_dim, value_dim) > 64 * 1024) waves /= 2;
    if (lds_bytes(waves, n_heads, head_dim, value_dim) > 64 * 1024) {
        waves = 4;
        while (waves > 1 && lds_bytes(waves, n_heads, head_dim, value_dim) > MOST_LDS) waves /= 2;
    }
    XRT_REQUIRE(lds_bytes(waves, n_heads, head_dim, value_dim) <= MOST_LDS,
                "attention (sigmoid): %d heads of %d and %d dims need more LDS than a compute unit has", n_heads, head_dim, value_dim);
    hipStream_t s = (hipStream_t)stream;
#define XRT_SIGMOID(T, WAVES_)                                                                                                     \
    return launch<T, WAVES_>(q, q_stride, tokens, n_heads, n_kv_heads, head_dim, value_dim, k_cache, v_cache, block_table, table_stride, \
                             n_blocks, positions, slots, out, scale, window, head_mix, head_bias, gate, gate_stride, s)
    if (dtype == XRT_F32) {
        if (waves == 4) XRT_SIGMOID(float, 4); else if (waves == 2) XRT_SIGMOID(float, 2); else XRT_SIGMOID(float, 1);
    } else {
        if (waves == 4) XRT_SIGMOID(bf16, 4); else if (waves == 2) XRT_SIGMOID(bf16, 2); else XRT_SIGMOID(bf16, 1);
    }
#undef XRT_SIGMOID
}
