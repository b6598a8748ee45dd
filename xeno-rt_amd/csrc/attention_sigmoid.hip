// Causal attention over the paged cache whose weights are not a softmax: the weight of a visible key is
// sigmoid(score + head_bias[h]), and the weighted values are summed as they are, with no normalisation over the keys.
// Before the sigmoid the heads' scaled scores of a (query, key) pair may be mixed with one another,
// score_h <- sum_g head_mix[h][g] * score_g (a matrix [heads][heads]); after the sum a head's output may be multiplied by
// sigmoid(gate[token][h]), one number per token and head. Grouped key/value heads, values of a width of their own, a window.
// Float32 arithmetic for either element type.
//
// A mix of the heads needs all heads' scores of a pair at once, so a workgroup owns a token with all its heads. Its
// wavefronts stand in teams of four; the teams deal the cache blocks of the token's keys among themselves by the block's
// absolute number, and the four wavefronts of a team work one block off together, in three passes with a barrier between:
// scores (a lane a key; a wavefront takes some query heads of one key/value head and loads that head's keys once for
// them), mix and sigmoid (a wavefront takes some heads, a lane still a key), weighted values (a lane a value dim; a
// wavefront takes some heads and adds up the block's tokens in their order). What the blocks give is added block after
// block in the order of their absolute numbers, so a token's output is the same bits however its request was cut into
// steps or batched. A step of few tokens (a decode step) would leave most of the chip idle with a workgroup a token:
// then several workgroups share a token's blocks, every block's part goes to a workspace, and a second kernel adds the
// parts in the same order, to the same bits. Loads are asked for several at a time before the first is used: one
// wavefront a block would wait out every load's whole latency, which is what this kernel's time is made of.
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

constexpr int TEAM_WAVES = 4;                // wavefronts that work one cache block off together
constexpr int MOST_TOGETHER = 4;             // query heads of one key/value head that share every load of a key or a value
constexpr int MOST_LDS = 160 * 1024;
constexpr int PIECES = XRT_BLOCK_TOKENS / 8; // pieces of eight tokens in a block's row of values

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

// eight floats from LDS at a place that is a multiple of eight floats
__device__ __forceinline__ void eight_of_lds(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

__device__ __forceinline__ float sigmoid_exact(float z) { return 1.0f / (1.0f + expf(-z)); }

// floats of LDS: the queries and the mix (padded to multiples of eight), then per team scores, weights and sums
__host__ __device__ inline size_t shared_floats(int teams, int n_heads, int head_dim, int value_dim) {
    const size_t queries = ((size_t)n_heads * head_dim + 7) / 8 * 8, mix = ((size_t)n_heads * n_heads + 7) / 8 * 8;
    const size_t sums = ((size_t)n_heads * value_dim + 7) / 8 * 8;
    return queries + mix + sums + (size_t)teams * (2 * (size_t)n_heads * XRT_WAVE + sums);
}

// SPLIT: the workgroups (token, 0 .. gridDim.y - 1) share the token's rounds of blocks and write every block's part to
// parts[token][block - first block][heads x value_dim]; else a workgroup a token, which adds the parts itself.
template <typename T, int TEAMS, bool SPLIT>
__global__ void __launch_bounds__(TEAMS * TEAM_WAVES * XRT_WAVE) attention_sigmoid_kernel(
    const T* __restrict__ q, long q_stride, int n_heads, int n_kv_heads, int head_dim, int value_dim,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int* __restrict__ block_table, int table_stride, int n_blocks,
    const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ out, float scale, int window,
    const float* __restrict__ head_mix, const float* __restrict__ head_bias, const float* __restrict__ gate, long gate_stride,
    int together, int whole_keys, int whole_values, float* __restrict__ parts, int most_blocks) {
    constexpr int THREADS = TEAMS * TEAM_WAVES * XRT_WAVE;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int out_width = n_heads * value_dim;
    const int sums_floats = (out_width + 7) / 8 * 8;
    float* qs = lds;                                                   // [heads][head_dim]
    float* mix = qs + (n_heads * head_dim + 7) / 8 * 8;                // [heads][heads]
    float* total = mix + (n_heads * n_heads + 7) / 8 * 8;             // [heads][value_dim]: the blocks' parts added up so far
    float* teams = total + sums_floats;
    const int lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE;
    const int team = wave / TEAM_WAVES, member = wave % TEAM_WAVES;
    float* raw = teams + (size_t)team * (2 * n_heads * XRT_WAVE + sums_floats);    // [heads][64]: scaled scores, lane j's key
    float* wts = raw + n_heads * XRT_WAVE;                             // [heads][64]: the weights after mix and sigmoid
    float* sums = wts + n_heads * XRT_WAVE;                            // [heads][value_dim]: what this round's block gives
    const long token = blockIdx.x;
    T* dst = out + token * out_width;
    const int slot = slots[token];
    if (slot < 0) {
        if (!SPLIT || blockIdx.y == 0)
            for (int i = threadIdx.x; i < out_width; i += THREADS) dst[i] = from_float<T>(0.f);
        return;
    }
    const int pos = positions[token];
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const int group = n_heads / n_kv_heads;
    const int sets = (group + together - 1) / together;               // sets of heads that share a key/value head's loads
    const T* q_row = q + token * q_stride;
    for (int i = threadIdx.x; i < n_heads * head_dim; i += THREADS) qs[i] = to_float(q_row[i]);
    if (head_mix != nullptr)
        for (int i = threadIdx.x; i < n_heads * n_heads; i += THREADS) mix[i] = head_mix[i];
    for (int i = threadIdx.x; i < out_width; i += THREADS) total[i] = 0.f;
    __syncthreads();

    const int* table = block_table + (long)slot * table_stride;
    const int first_block = first / XRT_BLOCK_TOKENS, last_block = pos / XRT_BLOCK_TOKENS;
    float* my_parts = SPLIT ? parts + token * most_blocks * (long)out_width : nullptr;
    for (int round = first_block / TEAMS + (SPLIT ? (int)blockIdx.y : 0); round <= last_block / TEAMS; round += SPLIT ? (int)gridDim.y : 1) {
        const int b = round * TEAMS + team;
        const bool in_range = b >= first_block && b <= last_block;
        int block = in_range ? table[b] : -1;
        if (block >= n_blocks) block = -1;                             // the host never lets this happen
        const bool active = block >= 0;
        float* part = SPLIT ? my_parts + (long)(b - first_block) * out_width : sums;
        const int j = b * XRT_BLOCK_TOKENS + lane;
        const bool valid = active && j >= first && j <= pos;
        // ---- scores: lane j's key against the queries of some heads of one key/value head
        if (active) {
            for (int item = member; item < n_kv_heads * sets; item += TEAM_WAVES) {
                const int kv_head = item / sets, h0 = item % sets * together;
                const int n_set = min(together, group - h0);
                const long key_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * head_dim;
                const float* q_set = qs + (kv_head * group + h0) * head_dim;
                float dot[MOST_TOGETHER];
#pragma unroll
                for (int s = 0; s < MOST_TOGETHER; ++s) dot[s] = 0.f;
                if (valid) {
                    if (whole_keys) {
                        for (int d0 = 0; d0 < head_dim; d0 += 32) {    // four pieces of eight dims asked for before the first is used
                            float key[4][8];
#pragma unroll
                            for (int p = 0; p < 4; ++p)
                                if (d0 + 8 * p < head_dim) eight(k_cache + key_base + cache_key_offset(lane, d0 + 8 * p, head_dim), key[p]);
#pragma unroll
                            for (int p = 0; p < 4; ++p) {
                                if (d0 + 8 * p < head_dim) {
#pragma unroll
                                    for (int s = 0; s < MOST_TOGETHER; ++s) {
                                        if (s < n_set) {
                                            float mine[8], of_piece = 0.f;
                                            eight_of_lds(q_set + s * head_dim + d0 + 8 * p, mine);
#pragma unroll
                                            for (int e = 0; e < 8; ++e) of_piece = fmaf(mine[e], key[p][e], of_piece);
                                            dot[s] += of_piece;
                                        }
                                    }
                                }
                            }
                        }
                    } else {
                        for (int d0 = 0; d0 < head_dim; d0 += 8) {
                            const int dims = min(8, head_dim - d0);
                            float key[8];
                            for (int e = 0; e < dims; ++e) key[e] = to_float(k_cache[key_base + cache_key_offset(lane, d0 + e, head_dim)]);
#pragma unroll
                            for (int s = 0; s < MOST_TOGETHER; ++s) {
                                if (s < n_set) {
                                    float of_piece = 0.f;
                                    for (int e = 0; e < dims; ++e) of_piece = fmaf(q_set[s * head_dim + d0 + e], key[e], of_piece);
                                    dot[s] += of_piece;
                                }
                            }
                        }
                    }
                }
#pragma unroll
                for (int s = 0; s < MOST_TOGETHER; ++s)
                    if (s < n_set) raw[(kv_head * group + h0 + s) * XRT_WAVE + lane] = dot[s] * scale;
            }
        }
        __syncthreads();
        // ---- the heads' scores of this lane's key mixed, biased, through the sigmoid
        if (active) {
            for (int h = member; h < n_heads; h += TEAM_WAVES) {
                float s = 0.f;
                if (head_mix != nullptr) {
                    for (int g = 0; g < n_heads; ++g) s = fmaf(mix[h * n_heads + g], raw[g * XRT_WAVE + lane], s);
                } else {
                    s = raw[h * XRT_WAVE + lane];
                }
                if (head_bias != nullptr) s += head_bias[h];
                wts[h * XRT_WAVE + lane] = valid ? sigmoid_exact(s) : 0.f;
            }
        }
        __syncthreads();
        // ---- weighted values: a lane takes a value dim of some heads of one key/value head, the block's tokens in their order
        if (active) {
            const int j_begin = max(0, first - b * XRT_BLOCK_TOKENS);
            const int j_end = min(XRT_BLOCK_TOKENS - 1, pos - b * XRT_BLOCK_TOKENS);
            const int chunks = (value_dim + XRT_WAVE - 1) / XRT_WAVE;
            for (int item = member; item < n_kv_heads * sets * chunks; item += TEAM_WAVES) {
                const int d = item % chunks * XRT_WAVE + lane;
                const int kv_head = item / chunks / sets, h0 = item / chunks % sets * together;
                const int n_set = min(together, group - h0);
                if (d >= value_dim) continue;
                const T* row = v_cache + ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * value_dim;
                const float* w_set = wts + (kv_head * group + h0) * XRT_WAVE;
                float sum[MOST_TOGETHER];
#pragma unroll
                for (int s = 0; s < MOST_TOGETHER; ++s) sum[s] = 0.f;
#pragma unroll
                for (int p0 = 0; p0 < PIECES; p0 += 4) {               // four pieces of eight tokens asked for before the first is used
                    float value[4][8];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int p = p0 + i;
                        if (8 * p + 7 >= j_begin && 8 * p <= j_end) {
                            const T* piece = row + cache_value_offset(d, 8 * p, value_dim);
                            if (whole_values) {
                                eight(piece, value[i]);
                            } else {
#pragma unroll
                                for (int e = 0; e < 8; ++e) value[i][e] = to_float(piece[e]);
                            }
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int p = p0 + i;
                        if (8 * p + 7 >= j_begin && 8 * p <= j_end) {
#pragma unroll
                            for (int e = 0; e < 8; ++e)                // (what lies before the window or beyond the sequence's end was loaded and is not used)
                                if (8 * p + e < j_begin || 8 * p + e > j_end) value[i][e] = 0.f;
#pragma unroll
                            for (int s = 0; s < MOST_TOGETHER; ++s) {
                                if (s < n_set) {
                                    float weight[8];
                                    eight_of_lds(w_set + s * XRT_WAVE + 8 * p, weight);
#pragma unroll
                                    for (int e = 0; e < 8; ++e) sum[s] = fmaf(weight[e], value[i][e], sum[s]);
                                }
                            }
                        }
                    }
                }
#pragma unroll
                for (int s = 0; s < MOST_TOGETHER; ++s)
                    if (s < n_set) part[(kv_head * group + h0 + s) * value_dim + d] = sum[s];
            }
        }
        if (in_range && !active)                                       // (a block that is not there gives nothing)
            for (int i = lane + member * XRT_WAVE; i < out_width; i += TEAM_WAVES * XRT_WAVE) part[i] = 0.f;
        // (the next block's scores are written where nobody reads now; its weights only after the barrier that follows them)
        if constexpr (!SPLIT) {
            __syncthreads();
            const float* team_sums = teams + 2 * n_heads * XRT_WAVE;
            const size_t team_stride = 2 * (size_t)n_heads * XRT_WAVE + sums_floats;
            for (int i = threadIdx.x; i < out_width; i += THREADS) {   // the round's blocks in their order (a thread its own places)
                float sum = total[i];
#pragma unroll
                for (int t = 0; t < TEAMS; ++t) {
                    const int bt = round * TEAMS + t;
                    if (bt >= first_block && bt <= last_block) sum += team_sums[t * team_stride + i];
                }
                total[i] = sum;
            }
        }
    }
    if constexpr (!SPLIT) {
        for (int i = threadIdx.x; i < out_width; i += THREADS) {       // (what the same thread added up)
            float sum = total[i];
            if (gate != nullptr) sum *= sigmoid_exact(gate[token * gate_stride + i / value_dim]);
            dst[i] = from_float<T>(sum);
        }
    }
}

// The parts of a token's blocks added in the blocks' order, times the gate.
template <typename T>
__global__ void __launch_bounds__(256) attention_sigmoid_merge_kernel(const float* __restrict__ parts, int most_blocks, int n_heads, int value_dim,
                                                                      const int* __restrict__ positions, const int* __restrict__ slots, int window,
                                                                      const float* __restrict__ gate, long gate_stride, T* __restrict__ out) {
    const long token = blockIdx.x;
    if (slots[token] < 0) return;                                      // (zeros were written already)
    const int pos = positions[token];
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const int count = pos / XRT_BLOCK_TOKENS - first / XRT_BLOCK_TOKENS + 1;
    const int out_width = n_heads * value_dim;
    const float* mine = parts + token * most_blocks * (long)out_width;
    for (int i = blockIdx.y * 256 + threadIdx.x; i < out_width; i += gridDim.y * 256) {
        float sum = 0.f;
        for (int b = 0; b < count; ++b) sum += mine[(long)b * out_width + i];
        if (gate != nullptr) sum *= sigmoid_exact(gate[token * gate_stride + i / value_dim]);
        out[token * out_width + i] = from_float<T>(sum);
    }
}

size_t lds_bytes(int teams, int n_heads, int head_dim, int value_dim) {
    return sizeof(float) * shared_floats(teams, n_heads, head_dim, value_dim);
}

// blocks that a token's keys can lie in: those of a window, or of the longest sequence
int most_blocks_of(int window, int max_context) {
    const int of_context = (max_context + XRT_BLOCK_TOKENS - 1) / XRT_BLOCK_TOKENS;
    return window > 0 ? min(of_context, (window + XRT_BLOCK_TOKENS - 2) / XRT_BLOCK_TOKENS + 1) : of_context;
}

// Workgroups that share a token's blocks: 1 where the step's tokens fill the chip by themselves (or nothing is known of the
// sequences' lengths), else as many as give the chip two workgroups a compute unit, and no more than there are rounds of blocks.
int parts_of(long tokens, int teams, int window, int max_context) {
    if (max_context <= 0 || tokens >= XRT_COMPUTE_UNITS) return 1;
    const int rounds = (most_blocks_of(window, max_context) + teams - 1) / teams + 1;
    return (int)max(1L, min((long)rounds, 2L * XRT_COMPUTE_UNITS / tokens));
}

int teams_of(int n_heads, int head_dim, int value_dim) {
    // as many teams a token as the LDS holds scores and sums for: a model's sizes decide, never the step
    // (two teams at most: eight wavefronts may have 256 registers each, sixteen would spill)
    int teams = 2;
    while (teams > 1 && lds_bytes(teams, n_heads, head_dim, value_dim) > 80 * 1024) teams /= 2;
    return teams;
}

template <typename T, int TEAMS, bool SPLIT>
int launch(const void* q, long q_stride, long tokens, int n_heads, int n_kv_heads, int head_dim, int value_dim, const void* k_cache,
           const void* v_cache, const int* block_table, int table_stride, int n_blocks, const int* positions, const int* slots, void* out,
           float scale, int window, const float* head_mix, const float* head_bias, const float* gate, long gate_stride, float* parts,
           int most_blocks, int n_parts, hipStream_t s) {
    const size_t bytes = lds_bytes(TEAMS, n_heads, head_dim, value_dim);
    auto kernel = attention_sigmoid_kernel<T, TEAMS, SPLIT>;
    static bool allowed = false;                                       // (once per kernel: the most LDS it may ever ask for)
    if (!allowed) {
        const hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, MOST_LDS);
        XRT_REQUIRE(status == hipSuccess, "attention (sigmoid): %d bytes of LDS were refused: %s", MOST_LDS, hipGetErrorString(status));
        allowed = true;
    }
    // heads of a key/value head that a wavefront takes together: as many as four, fewer where a team would otherwise have idle hands
    const int group = n_heads / n_kv_heads;
    int together = min(MOST_TOGETHER, group);
    while (together > 1 && n_kv_heads * ((group + together - 1) / together) < TEAM_WAVES) together = (together + 1) / 2;
    const int whole_keys = head_dim % 8 == 0 && (uintptr_t)k_cache % 32 == 0;
    const int whole_values = (uintptr_t)v_cache % 32 == 0;
    kernel<<<dim3((unsigned)tokens, SPLIT ? n_parts : 1), TEAMS * TEAM_WAVES * XRT_WAVE, bytes, s>>>((const T*)q, q_stride, n_heads, n_kv_heads,
        head_dim, value_dim, (const T*)k_cache, (const T*)v_cache, block_table, table_stride, n_blocks, positions, slots, (T*)out, scale, window,
        head_mix, head_bias, gate, gate_stride, together, whole_keys, whole_values, parts, most_blocks);
    if (SPLIT) {
        const int columns = max(1, min(8, (n_heads * value_dim + 255) / 256));
        attention_sigmoid_merge_kernel<T><<<dim3((unsigned)tokens, columns), 256, 0, s>>>(parts, most_blocks, n_heads, value_dim, positions, slots,
                                                                                         window, gate, gate_stride, (T*)out);
    }
    XRT_LAUNCH_CHECK("attention (sigmoid)");
    return 0;
}

}  // namespace

// floats of workspace with which a step of few tokens is shared out among more workgroups (0: none needed); max_context is
// the longest sequence after the step, 0 if unknown
extern "C" long xrt_attention_sigmoid_workspace(long tokens, int n_heads, int head_dim, int value_dim, int window, int max_context) {
    if (tokens <= 0 || n_heads <= 0 || head_dim <= 0 || value_dim <= 0) return 0;
    if (parts_of(tokens, teams_of(n_heads, head_dim, value_dim), window, max_context) <= 1) return 0;
    return tokens * most_blocks_of(window, max_context) * (long)n_heads * value_dim;
}

extern "C" int xrt_attention_sigmoid(const void* q, long q_stride, int dtype, long tokens, int n_heads, int n_kv_heads, int head_dim,
                                     int value_dim, const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                                     int n_blocks, const int* positions, const int* slots, void* out, float scale, int window,
                                     const float* head_mix, const float* head_bias, const float* gate, long gate_stride,
                                     int max_context, float* workspace, long workspace_floats, void* stream) {
    XRT_REQUIRE(tokens >= 0 && tokens < (1L << 31) && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention (sigmoid): head counts %d/%d: the first must be a multiple of the second", n_heads, n_kv_heads);
    XRT_REQUIRE(head_dim > 0 && value_dim > 0, "attention (sigmoid): head sizes %d and %d must be positive", head_dim, value_dim);
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "attention (sigmoid): unknown dtype %d", dtype);
    XRT_REQUIRE(q && k_cache && v_cache && block_table && positions && slots && out, "attention (sigmoid): null operand");
    XRT_REQUIRE(q_stride >= (long)n_heads * head_dim && (gate == nullptr || gate_stride >= n_heads), "attention (sigmoid): a row stride is shorter than its heads");
    XRT_REQUIRE(table_stride > 0 && n_blocks > 0 && window >= 0, "attention (sigmoid): empty cache or negative window");
    if (tokens == 0) return 0;
    const int teams = teams_of(n_heads, head_dim, value_dim);
    XRT_REQUIRE(lds_bytes(teams, n_heads, head_dim, value_dim) <= MOST_LDS,
                "attention (sigmoid): %d heads of %d and %d dims need more LDS than a compute unit has", n_heads, head_dim, value_dim);
    // shared out among workgroups only with a workspace that holds every block's part
    const long need = xrt_attention_sigmoid_workspace(tokens, n_heads, head_dim, value_dim, window, max_context);
    const bool split = need > 0 && workspace != nullptr && workspace_floats >= need;
    const int n_parts = split ? parts_of(tokens, teams, window, max_context) : 1;
    const int most_blocks = split ? most_blocks_of(window, max_context) : 0;
    hipStream_t s = (hipStream_t)stream;
#define XRT_SIGMOID(T, TEAMS_, SPLIT_)                                                                                                    \
    return launch<T, TEAMS_, SPLIT_>(q, q_stride, tokens, n_heads, n_kv_heads, head_dim, value_dim, k_cache, v_cache, block_table, table_stride, \
                                     n_blocks, positions, slots, out, scale, window, head_mix, head_bias, gate, gate_stride, workspace, most_blocks, \
                                     n_parts, s)
#define XRT_SIGMOID_TEAMS(T, SPLIT_) do { if (teams == 2) XRT_SIGMOID(T, 2, SPLIT_); else XRT_SIGMOID(T, 1, SPLIT_); } while (0)
    if (dtype == XRT_F32) {
        if (split) XRT_SIGMOID_TEAMS(float, true); else XRT_SIGMOID_TEAMS(float, false);
    } else {
        if (split) XRT_SIGMOID_TEAMS(bf16, true); else XRT_SIGMOID_TEAMS(bf16, false);
    }
#undef XRT_SIGMOID_TEAMS
#undef XRT_SIGMOID
    return 0;
}
