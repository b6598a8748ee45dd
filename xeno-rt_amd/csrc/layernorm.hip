// Layer norm over whole rows of the float32 residual stream, y = (x - mean) / sqrt(var + eps) * w + b with var the mean of
// the squared deviations, and what models put around it:
//   xrt_layernorm           the norm of (gathered) rows, into the compute dtype
//   xrt_layernorm_shift     the norm, then every row moved towards the normed row of the token before it in its sequence,
//                           h_t + (h_(t-1) - h_t) * mix; the last normed row of a sequence is its state for the next step
//   xrt_add_layernormed     residual += scale * norm(y + pre_bias): a norm after a sublayer, on its way onto the stream;
//                           the same kernel can go on to the next sublayer's norm of the row it has just written
// One workgroup per row; the row lies in LDS between the passes (mean, squared deviations, result), each thread touching
// only its own columns. All arithmetic is float32, and a row's result depends on nothing but the row (and, shifted, on the
// row before it), so it is the same bits however a step is cut or batched.
#include "xrt_hip.h"
#include "common.h"

namespace {

constexpr int NORM_THREADS = 256;

template <typename TW>
__device__ __forceinline__ float4 four(const TW* __restrict__ p) {     // four elements from a place that is a multiple of four
    if constexpr (sizeof(TW) == 4) {
        return *reinterpret_cast<const float4*>(p);
    } else {
        struct alignas(8) Four { TW e[4]; };
        const Four v = *reinterpret_cast<const Four*>(p);
        return make_float4(to_float(v.e[0]), to_float(v.e[1]), to_float(v.e[2]), to_float(v.e[3]));
    }
}

// buf[c] = layer norm of row[c] (+ add[c]) for this thread's columns: c = threadIdx.x, + 256, ..., or, where the row's
// length is a multiple of four, the quads 4 threadIdx.x, + 1024, ... (the sums a thread keeps are over other columns then,
// but which of the two it is depends on the row's length alone).
template <typename TW>
__device__ __forceinline__ void normalise(const float* __restrict__ row, const TW* __restrict__ add, const TW* __restrict__ w,
                                          const TW* __restrict__ b, float eps, int hidden, float* buf, float* scratch) {
    if (hidden % 4 == 0) {
        const int quads = hidden / 4;
        float4* buf4 = reinterpret_cast<float4*>(buf);
        float sum = 0.f;
        for (int q = threadIdx.x; q < quads; q += NORM_THREADS) {
            float4 v = *reinterpret_cast<const float4*>(row + 4 * q);
            if (add) {
                const float4 a = four(add + 4 * q);
                v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
            }
            buf4[q] = v;
            sum += (v.x + v.y) + (v.z + v.w);
        }
        const float mean = block_sum(sum, scratch) / (float)hidden;
        float squares = 0.f;
        for (int q = threadIdx.x; q < quads; q += NORM_THREADS) {
            const float4 v = buf4[q];
            const float dx = v.x - mean, dy = v.y - mean, dz = v.z - mean, dw = v.w - mean;
            squares = fmaf(dx, dx, fmaf(dy, dy, fmaf(dz, dz, fmaf(dw, dw, squares))));
        }
        const float inv = 1.0f / sqrtf(block_sum(squares, scratch) / (float)hidden + eps);
        for (int q = threadIdx.x; q < quads; q += NORM_THREADS) {
            const float4 v = buf4[q], g = four(w + 4 * q), s = four(b + 4 * q);
            buf4[q] = make_float4(fmaf((v.x - mean) * inv, g.x, s.x), fmaf((v.y - mean) * inv, g.y, s.y),
                                  fmaf((v.z - mean) * inv, g.z, s.z), fmaf((v.w - mean) * inv, g.w, s.w));
        }
        return;
    }
    float sum = 0.f;
    for (int c = threadIdx.x; c < hidden; c += NORM_THREADS) {
        const float v = row[c] + (add ? to_float(add[c]) : 0.f);
        buf[c] = v;
        sum += v;
    }
    const float mean = block_sum(sum, scratch) / (float)hidden;
    float squares = 0.f;
    for (int c = threadIdx.x; c < hidden; c += NORM_THREADS) {
        const float d = buf[c] - mean;
        squares = fmaf(d, d, squares);
    }
    const float inv = 1.0f / sqrtf(block_sum(squares, scratch) / (float)hidden + eps);
    for (int c = threadIdx.x; c < hidden; c += NORM_THREADS) buf[c] = fmaf((buf[c] - mean) * inv, to_float(w[c]), to_float(b[c]));
}

// Every thread's columns of a row, as `normalise` deals them: body(c) for each.
template <typename Body>
__device__ __forceinline__ void for_my_columns(int hidden, Body body) {
    if (hidden % 4 == 0) {
        for (int q = threadIdx.x; q < hidden / 4; q += NORM_THREADS) {
#pragma unroll
            for (int e = 0; e < 4; ++e) body(4 * q + e);
        }
    } else {
        for (int c = threadIdx.x; c < hidden; c += NORM_THREADS) body(c);
    }
}

template <typename TW, typename TO>
__global__ void __launch_bounds__(NORM_THREADS) layernorm_kernel(const float* __restrict__ x, const TW* __restrict__ w, const TW* __restrict__ b,
                                                                 float eps, TO* __restrict__ out, const int* __restrict__ rows, int hidden) {
    extern __shared__ __attribute__((aligned(16))) float buf[];
    __shared__ float scratch[32];
    const long src = rows ? rows[blockIdx.x] : blockIdx.x;
    normalise<TW>(x + src * hidden, nullptr, w, b, eps, hidden, buf, scratch);
    TO* dst = out + (long)blockIdx.x * hidden;
    for_my_columns(hidden, [&](int c) { dst[c] = from_float<TO>(buf[c]); });
}

// Row r is a token of the sequence in token_slots[r] (negative: padding, zeros out). The token before it is row r - 1 if that
// row has the same slot, else what the sequence's state holds (zeros for a sequence that starts). with_state: every
// sequence brings one token, and the row's workgroup writes the state itself once it has read it.
template <typename TW, typename TO>
__global__ void __launch_bounds__(NORM_THREADS) layernorm_shift_kernel(const float* __restrict__ x, const TW* __restrict__ w, const TW* __restrict__ b,
                                                                       const TW* __restrict__ mix, float eps, float* __restrict__ state,
                                                                       const int* __restrict__ token_slots, TO* __restrict__ out, int hidden,
                                                                       int with_state) {
    extern __shared__ __attribute__((aligned(16))) float buf[];                             // [2][hidden]: this row's norm, the one before
    __shared__ float scratch[32];
    const long r = blockIdx.x;
    const int slot = token_slots[r];
    TO* dst = out + r * hidden;
    if (slot < 0) {
        for (int c = threadIdx.x; c < hidden; c += NORM_THREADS) dst[c] = from_float<TO>(0.f);
        return;
    }
    float* here = buf;
    float* before = buf + hidden;
    normalise<TW>(x + r * hidden, nullptr, w, b, eps, hidden, here, scratch);
    const bool in_step = r > 0 && token_slots[r - 1] == slot;
    float* kept = state + (long)slot * hidden;
    if (in_step) {
        normalise<TW>(x + (r - 1) * hidden, nullptr, w, b, eps, hidden, before, scratch);
    } else {
        for_my_columns(hidden, [&](int c) { before[c] = kept[c]; });
    }
    for_my_columns(hidden, [&](int c) {
        const float h = here[c];
        dst[c] = from_float<TO>(fmaf(before[c] - h, to_float(mix[c]), h));
        if (with_state) kept[c] = h;
    });
}

// The state after a step of several tokens a sequence: the norm of each sequence's last row (a launch of its own, after
// every first token has read the old state).
template <typename TW>
__global__ void __launch_bounds__(NORM_THREADS) layernorm_state_kernel(const float* __restrict__ x, const TW* __restrict__ w, const TW* __restrict__ b,
                                                                       float eps, float* __restrict__ state, const int* __restrict__ seq_offsets,
                                                                       const int* __restrict__ seq_slots, int hidden) {
    extern __shared__ __attribute__((aligned(16))) float buf[];
    __shared__ float scratch[32];
    const int seq = blockIdx.x, slot = seq_slots[seq];
    const int begin = seq_offsets[seq], end = seq_offsets[seq + 1];
    if (slot < 0 || end <= begin) return;
    normalise<TW>(x + (long)(end - 1) * hidden, nullptr, w, b, eps, hidden, buf, scratch);
    float* kept = state + (long)slot * hidden;
    for_my_columns(hidden, [&](int c) { kept[c] = buf[c]; });
}

template <typename TW, typename TO>
__global__ void __launch_bounds__(NORM_THREADS) add_layernormed_kernel(float* __restrict__ residual, const float* __restrict__ y,
                                                                       const TW* __restrict__ pre_bias, const TW* __restrict__ w,
                                                                       const TW* __restrict__ b, float eps, float scale,
                                                                       const TW* __restrict__ next_w, const TW* __restrict__ next_b, float next_eps,
                                                                       TO* __restrict__ next_out, int hidden) {
    extern __shared__ __attribute__((aligned(16))) float buf[];
    __shared__ float scratch[32];
    const long r = blockIdx.x;
    normalise<TW>(y + r * hidden, pre_bias, w, b, eps, hidden, buf, scratch);
    float* row = residual + r * hidden;
    for_my_columns(hidden, [&](int c) { row[c] = fmaf(scale, buf[c], row[c]); });
    if (next_out == nullptr) return;
    // (every thread reads back the columns it has just written itself)
    normalise<TW>(row, nullptr, next_w, next_b, next_eps, hidden, buf, scratch);
    TO* dst = next_out + r * hidden;
    for_my_columns(hidden, [&](int c) { dst[c] = from_float<TO>(buf[c]); });
}

bool known(int dtype) { return dtype == XRT_F32 || dtype == XRT_BF16; }

}  // namespace

#define XRT_NORM_TYPES(CALL)                                                     \
    do {                                                                         \
        if (w_dtype == XRT_F32 && out_dtype == XRT_F32) CALL(float, float);      \
        else if (w_dtype == XRT_F32) CALL(float, bf16);                          \
        else if (out_dtype == XRT_F32) CALL(bf16, float);                        \
        else CALL(bf16, bf16);                                                   \
    } while (0)

extern "C" int xrt_layernorm(const float* x, const void* weight, const void* bias, int w_dtype, float eps, void* out, int out_dtype,
                             const int* rows, int n_rows, int hidden, void* stream) {
    XRT_REQUIRE(x && weight && bias && out, "layernorm: null operand");
    XRT_REQUIRE(known(w_dtype) && known(out_dtype), "layernorm: unknown dtype weight=%d out=%d", w_dtype, out_dtype);
    XRT_REQUIRE(n_rows >= 0 && hidden > 0 && hidden <= 16384, "layernorm: bad sizes rows=%d hidden=%d (rows of up to 16384)", n_rows, hidden);
    if (n_rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)hidden * sizeof(float);
#define XRT_CALL(TW, TO) layernorm_kernel<TW, TO><<<n_rows, NORM_THREADS, lds, s>>>(x, (const TW*)weight, (const TW*)bias, eps, (TO*)out, rows, hidden)
    XRT_NORM_TYPES(XRT_CALL);
#undef XRT_CALL
    XRT_LAUNCH_CHECK("layernorm");
    return 0;
}

extern "C" int xrt_layernorm_shift(const float* x, const void* weight, const void* bias, const void* mix, int w_dtype, float eps,
                                   float* state, const int* token_slots, const int* seq_offsets, const int* seq_slots, int n_seqs,
                                   int max_count, void* out, int out_dtype, int n_rows, int hidden, void* stream) {
    XRT_REQUIRE(x && weight && bias && mix && state && token_slots && seq_offsets && seq_slots && out, "layernorm_shift: null operand");
    XRT_REQUIRE(known(w_dtype) && known(out_dtype), "layernorm_shift: unknown dtype weight=%d out=%d", w_dtype, out_dtype);
    XRT_REQUIRE(n_rows >= 0 && n_seqs >= 0 && max_count >= 0 && hidden > 0 && hidden <= 8192,
                "layernorm_shift: bad sizes rows=%d hidden=%d (rows of up to 8192)", n_rows, hidden);
    if (n_rows == 0 || n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)2 * hidden * sizeof(float);
    const int with_state = max_count <= 1;
#define XRT_CALL(TW, TO)                                                                                                         \
    layernorm_shift_kernel<TW, TO><<<n_rows, NORM_THREADS, lds, s>>>(x, (const TW*)weight, (const TW*)bias, (const TW*)mix, eps, state, \
                                                                     token_slots, (TO*)out, hidden, with_state)
    XRT_NORM_TYPES(XRT_CALL);
#undef XRT_CALL
    if (!with_state) {
        if (w_dtype == XRT_F32)
            layernorm_state_kernel<float><<<n_seqs, NORM_THREADS, lds / 2, s>>>(x, (const float*)weight, (const float*)bias, eps, state, seq_offsets, seq_slots, hidden);
        else
            layernorm_state_kernel<bf16><<<n_seqs, NORM_THREADS, lds / 2, s>>>(x, (const bf16*)weight, (const bf16*)bias, eps, state, seq_offsets, seq_slots, hidden);
    }
    XRT_LAUNCH_CHECK("layernorm_shift");
    return 0;
}

extern "C" int xrt_add_layernormed(float* residual, const float* y, const void* pre_bias, const void* weight, const void* bias, int w_dtype,
                                   float eps, float scale, const void* next_weight, const void* next_bias, float next_eps, void* next_out,
                                   int out_dtype, long rows, int hidden, void* stream) {
    XRT_REQUIRE(residual && y && weight && bias, "add_layernormed: null operand");
    XRT_REQUIRE(next_out == nullptr || (next_weight && next_bias), "add_layernormed: the norm that follows needs its weight and bias");
    XRT_REQUIRE(known(w_dtype) && known(out_dtype), "add_layernormed: unknown dtype weight=%d out=%d", w_dtype, out_dtype);
    XRT_REQUIRE(rows >= 0 && rows < (1L << 31) && hidden > 0 && hidden <= 16384, "add_layernormed: bad sizes (rows of up to 16384)");
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)hidden * sizeof(float);
#define XRT_CALL(TW, TO)                                                                                                       \
    add_layernormed_kernel<TW, TO><<<(unsigned)rows, NORM_THREADS, lds, s>>>(residual, y, (const TW*)pre_bias, (const TW*)weight,  \
        (const TW*)bias, eps, scale, (const TW*)next_weight, (const TW*)next_bias, next_eps, (TO*)next_out, hidden)
    XRT_NORM_TYPES(XRT_CALL);
#undef XRT_CALL
    XRT_LAUNCH_CHECK("add_layernormed");
    return 0;
}
#undef XRT_NORM_TYPES
