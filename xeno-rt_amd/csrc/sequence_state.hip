// Mixing along the sequence with state of fixed size per sequence, and the small operations around it:
//   xrt_short_conv          causal convolution over time on each channel (a few taps), the last taps - 1 inputs kept per sequence;
//                           also as "input plus convolution" and as the interpolation between a token and the one before it
//   xrt_linear_recurrence   per head a matrix state S [dim x vdim]: S <- diag(decay) S + k v^T, read with q before or after the
//                           update; the decay a constant per head, given per token and channel, or worked out here from a
//                           projection (two forms); then per head an RMS norm, a weight and a gate
//   xrt_add_normed          residual += scale * sum of RMS-normed rows with their gains
//   xrt_activation          tanh, silu, and the two-parameter activation xIELU, elementwise
//   xrt_rows_add            out[t] += table[ids[t]]
//   xrt_kv_store            the step's keys and values into the paged cache, values of a width of their own
// Everything that is state, a decay, a norm or a sum onto the residual stream is float32 whatever the element type of the
// activations. A sequence's tokens are worked off in their order and nothing depends on where a step begins or on which
// other sequences the step holds, so a request gives the same bits however it is cut into steps and batched.
// Sequences whose slot is negative are padding: their rows of the output are zeros and no state is touched.
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

__device__ __forceinline__ float load_as_float(const void* p, int dtype, long i) {
    return dtype == XRT_F32 ? ((const float*)p)[i] : to_float(((const bf16*)p)[i]);
}
__device__ __forceinline__ void store_from_float(void* p, int dtype, long i, float v) {
    if (dtype == XRT_F32) ((float*)p)[i] = v; else ((bf16*)p)[i] = from_float<bf16>(v);
}

__device__ __forceinline__ float silu_exact(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_exact(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// ---- short convolution -----------------------------------------------------------------------------------------

constexpr int CONV_MAX_TAPS = 8;
constexpr int CONV_SEGMENT = 64;          // tokens of a sequence that one workgroup walks
constexpr int CONV_THREADS = 256;         // channels of a workgroup

// Input `at` (counted from the step's first token of the sequence; negative: before the step) of channel c.
template <typename T>
__device__ __forceinline__ float conv_input(const T* __restrict__ x, long x_stride, int begin, int at, const float* __restrict__ state,
                                            int taps, int channels, int c) {
    if (at >= 0) return to_float(x[(long)(begin + at) * x_stride + c]);
    return state[(long)(taps - 1 + at) * channels + c];
}

// grid (sequences, segments, channel chunks). phase 0: outputs only; 1: outputs and the state (one segment per sequence);
// 2: the state only (a launch of its own after phase 0, so that no workgroup reads a state another one is writing).
template <typename T>
__global__ void __launch_bounds__(CONV_THREADS) short_conv_kernel(
    const T* __restrict__ x, long x_stride, int channels, const void* __restrict__ w, int w_dtype, int taps, int n_out, int mode,
    float* __restrict__ state, const int* __restrict__ seq_offsets, const int* __restrict__ seq_slots, T* __restrict__ out,
    long tokens, int phase) {
    const int seq = blockIdx.x, c = blockIdx.z * CONV_THREADS + threadIdx.x;
    if (c >= channels) return;
    const int begin = seq_offsets[seq], count = seq_offsets[seq + 1] - begin, slot = seq_slots[seq];
    const int first = blockIdx.y * CONV_SEGMENT, last = min(count, first + CONV_SEGMENT);
    if (first >= count && !(phase == 2 && first == 0)) return;
    if (slot < 0) {
        if (phase != 2)
            for (int o = 0; o < n_out; ++o)
                for (int t = first; t < last; ++t) out[((long)o * tokens + begin + t) * channels + c] = from_float<T>(0.f);
        return;
    }
    float* mine = state + (long)slot * (taps - 1) * channels;
    float window[CONV_MAX_TAPS - 1];
    if (phase == 2) {                                      // what the sequence's last taps - 1 inputs are after this step
#pragma unroll
        for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
            if (m < taps - 1) window[m] = conv_input(x, x_stride, begin, count - (taps - 1) + m, mine, taps, channels, c);
#pragma unroll
        for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
            if (m < taps - 1) mine[(long)m * channels + c] = window[m];
        return;
    }
#pragma unroll
    for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
        window[m] = m < taps - 1 ? conv_input(x, x_stride, begin, first - (taps - 1) + m, mine, taps, channels, c) : 0.f;
    for (int t = first; t < last; ++t) {
        const float now = to_float(x[(long)(begin + t) * x_stride + c]);
        for (int o = 0; o < n_out; ++o) {
            float y;
            if (mode == XRT_CONV_TOWARDS_LAST) {           // taps == 2: x + (the input before - x) * w
                y = fmaf(window[0] - now, load_as_float(w, w_dtype, (long)o * channels + c), now);
            } else {
                const long w_at = ((long)o * channels + c) * taps;
                y = 0.f;
#pragma unroll
                for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
                    if (m < taps - 1) y = fmaf(load_as_float(w, w_dtype, w_at + m), window[m], y);
                y = fmaf(load_as_float(w, w_dtype, w_at + taps - 1), now, y);
                if (mode == XRT_CONV_PLUS_INPUT) y += now;
            }
            out[((long)o * tokens + begin + t) * channels + c] = from_float<T>(y);
        }
#pragma unroll
        for (int m = 0; m < CONV_MAX_TAPS - 2; ++m) window[m] = window[m + 1];
        if (taps >= 2) {
#pragma unroll
            for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
                if (m == taps - 2) window[m] = now;
        }
    }
    if (phase == 1) {
#pragma unroll
        for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
            if (m < taps - 1) mine[(long)m * channels + c] = window[m];
    }
}

// ---- linear recurrence -----------------------------------------------------------------------------------------

constexpr int REC_CHUNK = 16;             // tokens whose q, k and decays are staged in LDS at a time (fewer where heads are large)

template <int DIM, bool BONUS, int THREADS>
__global__ void __launch_bounds__(THREADS) recurrence_kernel(const xrt_recurrence a, int dtype, const int* __restrict__ seq_offsets,
                                                             const int* __restrict__ seq_slots, int chunk) {
    extern __shared__ float lds[];
    constexpr int ARRAYS = BONUS ? 4 : 3;                  // q, k, decay and, with a bonus, bonus * k
    const int seq = blockIdx.x, head = blockIdx.y, j = threadIdx.x;
    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE, waves = blockDim.x / XRT_WAVE;
    const int begin = seq_offsets[seq], end = seq_offsets[seq + 1], slot = seq_slots[seq];
    const int dim = a.dim, vdim = a.vdim, heads = a.heads;
    const long out_width = (long)heads * vdim;
    if (slot < 0) {
        for (int t = begin; t < end; ++t)
            for (int c = j; c < vdim; c += blockDim.x) store_from_float(a.out, dtype, t * out_width + (long)head * vdim + c, 0.f);
        return;
    }
    float* staged = lds;                                   // [chunk][ARRAYS][dim]
    float* raw = lds + chunk * ARRAYS * dim;               // [chunk][vdim]
    const bool owner = j < vdim;
    float* kept = a.state + (((long)slot * heads + head) * dim) * vdim + j;
    float S[DIM];
#pragma unroll
    for (int i = 0; i < DIM; ++i) S[i] = owner && i < dim ? kept[(long)i * vdim] : 0.f;
    for (int t0 = begin; t0 < end; t0 += chunk) {
        const int n = min(chunk, end - t0);
        __syncthreads();                                   // the chunk before is read to its end
        for (int e = threadIdx.x; e < n * dim; e += blockDim.x) {
            const int tt = e / dim, i = e % dim;
            const long row = t0 + tt, at = (long)head * dim + i;
            const float qv = load_as_float(a.q, dtype, row * a.q_stride + at) * a.q_scale;
            const float kv = load_as_float(a.k, dtype, row * a.k_stride + at) * a.k_scale;
            float decay;
            if (a.decay_mode == XRT_DECAY_PER_HEAD) {
                decay = a.decay[head];
            } else {
                float z = a.decay[row * (long)heads * dim + at];
                if (a.decay_bias != nullptr) z += load_as_float(a.decay_bias, a.decay_bias_dtype, at);
                if (a.decay_mode == XRT_DECAY_EXP_NEG_EXP) decay = expf(-expf(z));
                else if (a.decay_mode == XRT_DECAY_SIGMOID_POWER) decay = expf(-softplus_exact(-z) * a.decay_power);   // sigmoid(z)^power
                else decay = z;
            }
            float* to = staged + (long)tt * ARRAYS * dim + i;
            to[0] = qv;
            to[dim] = kv;
            to[2 * dim] = decay;
            if constexpr (BONUS) to[3 * dim] = load_as_float(a.bonus, a.bonus_dtype, at) * kv;
        }
        float v_now = owner ? load_as_float(a.v, dtype, (long)t0 * a.v_stride + (long)head * vdim + j) : 0.f;
        __syncthreads();
        for (int tt = 0; tt < n; ++tt) {
            const float v_next = owner && tt + 1 < n ? load_as_float(a.v, dtype, (long)(t0 + tt + 1) * a.v_stride + (long)head * vdim + j) : 0.f;
            const float* sq = staged + (long)tt * ARRAYS * dim;
            const float* sk = sq + dim;
            const float* sd = sq + 2 * dim;
            float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < DIM; ++i) {
                if (i < dim) {
                    const float kv = sk[i] * v_now;
                    if constexpr (BONUS) {
                        o[i % 4] = fmaf(fmaf(sq[3 * dim + i], v_now, S[i]), sq[i], o[i % 4]);
                        S[i] = fmaf(sd[i], S[i], kv);
                    } else {
                        S[i] = fmaf(sd[i], S[i], kv);
                        o[i % 4] = fmaf(S[i], sq[i], o[i % 4]);
                    }
                }
            }
            if (owner) raw[tt * vdim + j] = (o[0] + o[1]) + (o[2] + o[3]);
            v_now = v_next;
        }
        __syncthreads();
        // the heads' outputs of the chunk: norm over vdim, weight, gate; a wavefront a token
        for (int tt = wave; tt < n; tt += waves) {
            const long row = t0 + tt;
            float inv = 1.f;
            if (a.norm) {
                float squares = 0.f;
                for (int c = lane; c < vdim; c += XRT_WAVE) squares = fmaf(raw[tt * vdim + c], raw[tt * vdim + c], squares);
                inv = 1.0f / sqrtf(wave_sum(squares) / (float)vdim + a.eps);
            }
            for (int c = lane; c < vdim; c += XRT_WAVE) {
                float value = raw[tt * vdim + c] * inv;
                if (a.norm_weight != nullptr)
                    value *= load_as_float(a.norm_weight, a.norm_weight_dtype, a.norm_weight_per_head ? (long)head * vdim + c : c);
                if (a.gate != nullptr) {
                    const float g = load_as_float(a.gate, dtype, row * a.gate_stride + (long)head * vdim + c);
                    value *= a.gate_act == XRT_GATE_SILU ? silu_exact(g) : g;
                }
                store_from_float(a.out, dtype, row * out_width + (long)head * vdim + c, value);
            }
        }
    }
    if (owner) {
#pragma unroll
        for (int i = 0; i < DIM; ++i)
            if (i < dim) kept[(long)i * vdim] = S[i];
    }
}

// ---- residual += scale * sum_n rms(x_n) * gain_n --------------------------------------------------------------

__global__ void __launch_bounds__(256) add_normed_kernel(float* __restrict__ residual, const float* __restrict__ x0, const void* __restrict__ g0,
                                                         const float* __restrict__ x1, const void* __restrict__ g1, int gain_dtype,
                                                         int width, float eps, float scale) {
    __shared__ float scratch[32];
    const long row = blockIdx.x;
    const float* in[2] = {x0, x1};
    const void* gains[2] = {g0, g1};
    float inv[2] = {0.f, 0.f};
    for (int n = 0; n < 2; ++n) {
        if (in[n] == nullptr) continue;
        float squares = 0.f;
        for (int c = threadIdx.x; c < width; c += blockDim.x) squares = fmaf(in[n][row * width + c], in[n][row * width + c], squares);
        inv[n] = 1.0f / sqrtf(block_sum(squares, scratch) / (float)width + eps);
    }
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float sum = 0.f;
        for (int n = 0; n < 2; ++n)
            if (in[n] != nullptr) sum += in[n][row * width + c] * inv[n] * load_as_float(gains[n], gain_dtype, c);
        residual[row * width + c] += scale * sum;
    }
}

// ---- activations -------------------------------------------------------------------------------------------------

__global__ void activation_kernel(const void* __restrict__ x, int x_dtype, void* __restrict__ out, int out_dtype, long count, int kind,
                                  const void* __restrict__ params, int params_dtype) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const float z = load_as_float(x, x_dtype, i);
    float y;
    if (kind == XRT_UNARY_TANH) {
        y = tanhf(z);
    } else if (kind == XRT_UNARY_SILU) {
        y = silu_exact(z);
    } else {                                               // xIELU with the numbers (p, q)
        const float p = load_as_float(params, params_dtype, 0), q = load_as_float(params, params_dtype, 1);
        if (z > 0.f) y = fmaf(softplus_exact(p) * z, z, 0.5f * z);
        else y = fmaf(0.5f + softplus_exact(q), expm1f(z) - z, 0.5f * z);
    }
    store_from_float(out, out_dtype, i, y);
}

template <typename T>
__global__ void rows_add_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out, int width, int rows) {
    const long token = blockIdx.x;
    const int id = ids[token];
    if (id < 0 || id >= rows) return;
    for (int c = threadIdx.x; c < width; c += blockDim.x) out[token * width + c] += to_float(table[(long)id * width + c]);
}

// one wavefront per (token, key/value head)
template <typename T>
__global__ void kv_store_kernel(const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride, int n_kv_heads, int head_dim,
                                int value_dim, const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ k_cache,
                                T* __restrict__ v_cache, const int* __restrict__ block_table, int table_stride, int n_blocks) {
    const int token = blockIdx.x / n_kv_heads, kv_head = blockIdx.x % n_kv_heads, lane = threadIdx.x;
    const int slot = slots[token], pos = positions[token];
    if (slot < 0) return;
    const int block = block_table[(long)slot * table_stride + pos / XRT_BLOCK_TOKENS];
    if (block < 0 || block >= n_blocks) return;
    const int within = pos % XRT_BLOCK_TOKENS;
    const long key_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * head_dim;
    const long value_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * value_dim;
    for (int e = lane; e < head_dim; e += XRT_WAVE)
        k_cache[key_base + cache_key_offset(within, e, head_dim)] = k[(long)token * k_stride + (long)kv_head * head_dim + e];
    for (int e = lane; e < value_dim; e += XRT_WAVE)
        v_cache[value_base + cache_value_offset(e, within, value_dim)] = v[(long)token * v_stride + (long)kv_head * value_dim + e];
}

}  // namespace

extern "C" int xrt_short_conv(const void* x, int dtype, long tokens, long x_stride, int channels, const void* w, int w_dtype, int taps,
                              int n_out, int mode, float* state, const int* seq_offsets, const int* seq_slots, int n_seqs, int max_count,
                              void* out, void* stream) {
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "short_conv: unknown dtype %d", dtype);
    XRT_REQUIRE(w_dtype == XRT_F32 || w_dtype == XRT_BF16, "short_conv: unknown weight dtype %d", w_dtype);
    XRT_REQUIRE(x && w && (state || taps == 1) && seq_offsets && seq_slots && out, "short_conv: null operand");
    XRT_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "short_conv: %d taps, 1 to %d are served", taps, CONV_MAX_TAPS);
    XRT_REQUIRE(mode == XRT_CONV_PLAIN || mode == XRT_CONV_PLUS_INPUT || (mode == XRT_CONV_TOWARDS_LAST && taps == 2),
                "short_conv: unknown mode %d (the interpolation towards the input before has two taps)", mode);
    XRT_REQUIRE(channels > 0 && n_out > 0 && x_stride >= channels && tokens >= 0 && n_seqs >= 0 && max_count >= 0, "short_conv: bad sizes");
    if (n_seqs == 0 || max_count == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int segments = (max_count + CONV_SEGMENT - 1) / CONV_SEGMENT;
    const int chunks = (channels + CONV_THREADS - 1) / CONV_THREADS;
    XRT_REQUIRE(segments <= 65535 && chunks <= 65535, "short_conv: a step this long is not served");
#define XRT_CONV(T, segments_, phase_)                                                                                     \
    short_conv_kernel<T><<<dim3(n_seqs, segments_, chunks), CONV_THREADS, 0, s>>>((const T*)x, x_stride, channels, w, w_dtype, taps, \
        n_out, mode, state, seq_offsets, seq_slots, (T*)out, tokens, phase_)
    if (segments == 1 || taps == 1) {                      // (one tap: no state, nothing that one workgroup writes and another reads)
        if (dtype == XRT_F32) XRT_CONV(float, segments, 1); else XRT_CONV(bf16, segments, 1);
    } else {
        if (dtype == XRT_F32) XRT_CONV(float, segments, 0); else XRT_CONV(bf16, segments, 0);
        if (dtype == XRT_F32) XRT_CONV(float, 1, 2); else XRT_CONV(bf16, 1, 2);
    }
#undef XRT_CONV
    XRT_LAUNCH_CHECK("short_conv");
    return 0;
}

extern "C" int xrt_linear_recurrence(const xrt_recurrence* args, int dtype, const int* seq_offsets, const int* seq_slots, int n_seqs,
                                     void* stream) {
    XRT_REQUIRE(args != nullptr && seq_offsets && seq_slots, "linear_recurrence: null operand");
    const xrt_recurrence a = *args;
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "linear_recurrence: unknown dtype %d", dtype);
    XRT_REQUIRE(a.q && a.k && a.v && a.state && a.out, "linear_recurrence: null operand");
    XRT_REQUIRE(a.heads > 0 && a.heads <= 65535 && a.dim > 0 && a.dim <= 256 && a.vdim > 0 && a.vdim <= 1024,
                "linear_recurrence: %d heads of %d x %d: key sizes up to 256 and value sizes up to 1024 are served", a.heads, a.dim, a.vdim);
    XRT_REQUIRE(a.decay_mode >= XRT_DECAY_PER_HEAD && a.decay_mode <= XRT_DECAY_SIGMOID_POWER && a.decay != nullptr,
                "linear_recurrence: unknown decay mode %d, or no decays", a.decay_mode);
    XRT_REQUIRE(a.q_stride >= a.heads * a.dim && a.k_stride >= a.heads * a.dim && a.v_stride >= a.heads * a.vdim &&
                (a.gate == nullptr || a.gate_stride >= a.heads * a.vdim), "linear_recurrence: a row stride is shorter than its heads");
    if (n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const bool bonus = a.bonus != nullptr;
    const int threads = (a.vdim + XRT_WAVE - 1) / XRT_WAVE * XRT_WAVE;
    const size_t per_token = (size_t)((bonus ? 4 : 3) * a.dim + a.vdim) * sizeof(float);
    const int chunk = (int)min((size_t)REC_CHUNK, (size_t)(64 * 1024) / per_token);           // (at least 5 with the largest heads)
    const size_t lds = chunk * per_token;
#define XRT_REC(DIM_, BONUS_, THREADS_) recurrence_kernel<DIM_, BONUS_, THREADS_><<<dim3(n_seqs, a.heads), threads, lds, s>>>(a, dtype, seq_offsets, seq_slots, chunk)
    // (a workgroup of few wavefronts may keep a whole column of a large state in registers)
#define XRT_REC_THREADS(DIM_, BONUS_)                                                            \
    do {                                                                                         \
        if (threads <= 128) XRT_REC(DIM_, BONUS_, 128); else if (threads <= 256) XRT_REC(DIM_, BONUS_, 256); \
        else XRT_REC(DIM_, BONUS_, 1024);                                                        \
    } while (0)
#define XRT_REC_DIM(BONUS_)                                                                      \
    do {                                                                                         \
        if (a.dim <= 32) XRT_REC_THREADS(32, BONUS_); else if (a.dim <= 64) XRT_REC_THREADS(64, BONUS_); \
        else if (a.dim <= 128) XRT_REC_THREADS(128, BONUS_); else XRT_REC_THREADS(256, BONUS_);  \
    } while (0)
    if (bonus) XRT_REC_DIM(true); else XRT_REC_DIM(false);
#undef XRT_REC_DIM
#undef XRT_REC_THREADS
#undef XRT_REC
    XRT_LAUNCH_CHECK("linear_recurrence");
    return 0;
}

extern "C" int xrt_add_normed(float* residual, const float* x0, const void* gain0, const float* x1, const void* gain1, int gain_dtype,
                              long rows, int width, float eps, float scale, void* stream) {
    XRT_REQUIRE(residual && x0 && gain0 && (x1 == nullptr) == (gain1 == nullptr), "add_normed: null operand");
    XRT_REQUIRE(gain_dtype == XRT_F32 || gain_dtype == XRT_BF16, "add_normed: unknown dtype %d", gain_dtype);
    XRT_REQUIRE(rows >= 0 && rows < (1L << 31) && width > 0, "add_normed: bad sizes");
    if (rows == 0) return 0;
    add_normed_kernel<<<(unsigned)rows, 256, 0, (hipStream_t)stream>>>(residual, x0, gain0, x1, gain1, gain_dtype, width, eps, scale);
    XRT_LAUNCH_CHECK("add_normed");
    return 0;
}

extern "C" int xrt_activation(const void* x, int x_dtype, void* out, int out_dtype, long count, int kind, const void* params,
                              int params_dtype, void* stream) {
    XRT_REQUIRE(x && out && count >= 0, "activation: null operand");
    XRT_REQUIRE((x_dtype == XRT_F32 || x_dtype == XRT_BF16) && (out_dtype == XRT_F32 || out_dtype == XRT_BF16), "activation: unknown dtype");
    XRT_REQUIRE(kind == XRT_UNARY_TANH || kind == XRT_UNARY_SILU || (kind == XRT_UNARY_XIELU && params != nullptr),
                "activation: unknown kind %d, or xIELU without its two numbers", kind);
    if (count == 0) return 0;
    const long blocks = (count + 255) / 256;
    XRT_REQUIRE(blocks < (1L << 31), "activation: too many elements");
    activation_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(x, x_dtype, out, out_dtype, count, kind, params, params_dtype);
    XRT_LAUNCH_CHECK("activation");
    return 0;
}

extern "C" int xrt_rows_add(const void* table, int dtype, const int* ids, float* out, long tokens, int width, int rows, void* stream) {
    XRT_REQUIRE(table && ids && out, "rows_add: null operand");
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "rows_add: unknown dtype %d", dtype);
    XRT_REQUIRE(tokens >= 0 && tokens < (1L << 31) && width > 0 && rows > 0, "rows_add: bad sizes");
    if (tokens == 0) return 0;
    if (dtype == XRT_F32) rows_add_kernel<float><<<(unsigned)tokens, 256, 0, (hipStream_t)stream>>>((const float*)table, ids, out, width, rows);
    else rows_add_kernel<bf16><<<(unsigned)tokens, 256, 0, (hipStream_t)stream>>>((const bf16*)table, ids, out, width, rows);
    XRT_LAUNCH_CHECK("rows_add");
    return 0;
}

extern "C" int xrt_kv_store(const void* k, long k_stride, const void* v, long v_stride, int dtype, long tokens, int n_kv_heads, int head_dim,
                            int value_dim, const int* positions, const int* slots, void* k_cache, void* v_cache, const int* block_table,
                            int table_stride, int n_blocks, void* stream) {
    XRT_REQUIRE(k && v && positions && slots && k_cache && v_cache && block_table, "kv_store: null operand");
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "kv_store: unknown dtype %d", dtype);
    XRT_REQUIRE(tokens >= 0 && n_kv_heads > 0 && head_dim > 0 && value_dim > 0 && tokens * n_kv_heads < (1L << 31), "kv_store: bad sizes");
    XRT_REQUIRE(k_stride >= (long)n_kv_heads * head_dim && v_stride >= (long)n_kv_heads * value_dim, "kv_store: a row stride is shorter than its heads");
    if (tokens == 0) return 0;
    const unsigned items = (unsigned)(tokens * n_kv_heads);
    if (dtype == XRT_F32)
        kv_store_kernel<float><<<items, XRT_WAVE, 0, (hipStream_t)stream>>>((const float*)k, k_stride, (const float*)v, v_stride, n_kv_heads, head_dim,
            value_dim, positions, slots, (float*)k_cache, (float*)v_cache, block_table, table_stride, n_blocks);
    else
        kv_store_kernel<bf16><<<items, XRT_WAVE, 0, (hipStream_t)stream>>>((const bf16*)k, k_stride, (const bf16*)v, v_stride, n_kv_heads, head_dim,
            value_dim, positions, slots, (bf16*)k_cache, (bf16*)v_cache, block_table, table_stride, n_blocks);
    XRT_LAUNCH_CHECK("kv_store");
    return 0;
}
