// Kernels of blocks and mixers that several designs can share: the gated delta rule with its short convolutions,
// the difference of two attention maps, and a block whose two sublayers join a 32-bit stream together under gates.
// Everything behind a projection is float32 here, whatever the type of the projections' results.
#include "common.hpp"

using namespace lsa;

namespace {

__device__ inline float sigmoid_of(float z) { return 1.f / (1.f + expf(-z)); }
__device__ inline float softplus_of(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---- a block whose sublayers' results join the stream together ---------------------------------------------------------
// x[t] += s1 * sigmoid(gates[t][:W]) * y1[t] + s2 * sigmoid(gates[t][W:]) * y2[t] (y2 may be absent), in float32 where x
// lies; then, with next_weight, normed[t] = x[t] * rsqrt(mean(x[t]^2) + eps) * next_weight.  One workgroup a token.  Rows of
// up to 256 * COLS numbers (COLS > 0): a thread issues all its loads (the stream, gates, results, scales, the next norm's
// weights) before the first store and before the sum of squares, so a row of one token waits for memory once, and keeps its
// columns in registers between the sum and the norm.  Longer rows walk their columns and read the stored row again.
constexpr int UPDATE_COLS = 16;
template <typename G, typename Y1, typename Y2, typename N, int COLS>
__global__ __launch_bounds__(256) void gated_pair_update_kernel(float* __restrict__ x, const G* __restrict__ gates, int gate_width,
                                                                const Y1* __restrict__ y1, const float* __restrict__ s1,
                                                                const Y2* __restrict__ y2, const float* __restrict__ s2,
                                                                const float* __restrict__ next_weight, float eps, N* __restrict__ normed, int width) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    float* row = x + (size_t)t * width;
    const G* g = gates + (size_t)t * gate_width;
    if constexpr (COLS > 0) {
        float xv[COLS > 0 ? COLS : 1], g1[COLS > 0 ? COLS : 1], a1[COLS > 0 ? COLS : 1], w1[COLS > 0 ? COLS : 1], g2[COLS > 0 ? COLS : 1],
            a2[COLS > 0 ? COLS : 1], w2[COLS > 0 ? COLS : 1], nw[COLS > 0 ? COLS : 1];
        // every load is of a place that is there (a column beyond the row reads the row's last one, an absent second
        // sublayer reads the first one's operands, an absent norm the first scale), so none stands under a condition
        // (the launcher makes Y2 float where there is no second sublayer, so the stream's own row can stand in)
        const Y2* second = y2 ? y2 + (size_t)t * width : reinterpret_cast<const Y2*>(row);
        const float* second_scale = y2 ? s2 : s1;
        const float* following = next_weight ? next_weight : s1;
        const int second_gate = y2 ? width : 0;
        const float counts = y2 ? 1.f : 0.f;
#pragma unroll
        for (int n = 0; n < COLS; ++n) {
            const int c = min((int)threadIdx.x + 256 * n, width - 1);
            xv[n] = row[c];
            g1[n] = (float)g[c];
            a1[n] = (float)y1[(size_t)t * width + c];
            w1[n] = s1[c];
            g2[n] = (float)g[second_gate + c];
            a2[n] = (float)second[c];
            w2[n] = second_scale[c] * counts;
            nw[n] = following[c];
        }
        float sq = 0.f;
#pragma unroll
        for (int n = 0; n < COLS; ++n) {
            xv[n] += w1[n] * sigmoid_of(g1[n]) * a1[n] + w2[n] * sigmoid_of(g2[n]) * a2[n];
            if ((int)threadIdx.x + 256 * n < width) sq += xv[n] * xv[n];
        }
#pragma unroll
        for (int n = 0; n < COLS; ++n) {
            const int c = threadIdx.x + 256 * n;
            if (c < width) row[c] = xv[n];
        }
        if (!next_weight) return;
        const float inv = rsqrtf(block_sum(sq, scratch) / (float)width + eps);
#pragma unroll
        for (int n = 0; n < COLS; ++n) {
            const int c = threadIdx.x + 256 * n;
            if (c < width) normed[(size_t)t * width + c] = (N)(xv[n] * inv * nw[n]);
        }
        return;
    }
    float sq = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) {
        float v = row[c] + s1[c] * sigmoid_of((float)g[c]) * (float)y1[(size_t)t * width + c];
        if (y2) v += s2[c] * sigmoid_of((float)g[width + c]) * (float)y2[(size_t)t * width + c];
        row[c] = v;
        sq += v * v;
    }
    if (!next_weight) return;
    const float inv = rsqrtf(block_sum(sq, scratch) / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += 256) normed[(size_t)t * width + c] = (N)(row[c] * inv * next_weight[c]);
}

// ---- differential attention: a1 - lambda a2 per head, divided by its root mean square, times a constant -------------------
// grid (tokens, heads), one wavefront.  attended [T][kv_heads][2][group][row]; out [T][kv_heads * group][value_dim].
template <typename T>
__global__ __launch_bounds__(64) void differential_heads_kernel(const T* __restrict__ attended, float lam, float keep, float eps,
                                                                T* __restrict__ out, int group, int value_dim, int row) {
    const int t = blockIdx.x, head = blockIdx.y, heads = gridDim.y, lane = threadIdx.x;
    const int g = head / group, r = head % group;
    const T* a1 = attended + (((size_t)t * (heads / group) + g) * 2 * group + r) * row;
    const T* a2 = a1 + (size_t)group * row;
    float sq = 0.f;
    for (int j = lane; j < value_dim; j += 64) {
        const float d = (float)a1[j] - lam * (float)a2[j];
        sq += d * d;
    }
    const float inv = rsqrtf(wave_sum(sq) / (float)value_dim + eps) * keep;
    T* o = out + ((size_t)t * heads + head) * value_dim;
    for (int j = lane; j < value_dim; j += 64) o[j] = (T)(((float)a1[j] - lam * (float)a2[j]) * inv);
}

// ---- the delta rule's inputs ----------------------------------------------------------------------------------------------
// grid (tokens, 2 kv_heads + 2 heads), one wavefront.  Blocks 0 .. 2 kv_heads - 1: a query or key head: causal convolution over
// the request's tokens per channel, silu, the head divided by sqrt(sum of squares + unit_eps), queries times q_scale.  The next
// `heads` blocks: a value head (convolution and silu).  The last `heads` blocks: the head's write strength sigmoid(b) and its
// decay exp(-exp(A) softplus(z + bias)), one number or one per key channel.  A token's predecessors come from the step's own
// rows where the step brings them and from state[slot][k][channel] (the request's last taps - 1 inputs, oldest first) where it
// does not; zeros before the sequence.  keep (steps of one token a row): the thread that has read a channel's state moves it on.
constexpr int MOST_DIM = 256;       // key channels of a head
template <typename T>
__global__ __launch_bounds__(64) void delta_prepare_kernel(const T* __restrict__ proj, long stride, const float* __restrict__ w, int taps,
                                                           float* state, long state_stride, const int* __restrict__ slots,
                                                           const int* __restrict__ token_row, const int* __restrict__ positions,
                                                           const int* __restrict__ row_start, float* __restrict__ out,
                                                           int kv_heads, int heads, int dim, int value_dim, float q_scale, float unit_eps, int keep,
                                                           const T* __restrict__ strength, long strength_stride, const void* __restrict__ decay,
                                                           long decay_stride, int per_channel, const float* __restrict__ decay_scale,
                                                           const float* __restrict__ decay_bias, float* __restrict__ out_strength,
                                                           float* __restrict__ out_decay) {
    const int t = blockIdx.x, block = blockIdx.y, lane = threadIdx.x;
    const int keys = kv_heads * dim, channels = 2 * keys + heads * value_dim;
    if (block >= 2 * kv_heads + heads) {
        const int head = block - 2 * kv_heads - heads;
        const float rate = expf(decay_scale[head]);
        if (per_channel) {
            const float* z = reinterpret_cast<const float*>(decay) + (size_t)t * decay_stride + (size_t)head * dim;
            for (int e = lane; e < dim; e += 64)
                out_decay[((size_t)t * heads + head) * dim + e] = expf(-rate * softplus_of(z[e] + decay_bias[head * dim + e]));
        } else if (lane == 0) {
            const float z = (float)reinterpret_cast<const T*>(decay)[(size_t)t * decay_stride + head];
            out_decay[(size_t)t * heads + head] = expf(-rate * softplus_of(z + decay_bias[head]));
        }
        if (lane == 0) out_strength[(size_t)t * heads + head] = sigmoid_of((float)strength[(size_t)t * strength_stride + head]);
        return;
    }
    const bool unit = block < 2 * kv_heads;
    const int size = unit ? dim : value_dim;
    const int base = unit ? block * dim : 2 * keys + (block - 2 * kv_heads) * value_dim;
    const int row = token_row[t], position = positions[t];
    const int first = position - (t - row_start[row]);
    const int kept = taps - 1;
    float* mine = kept ? state + (size_t)slots[row] * state_stride : nullptr;
    float held[MOST_DIM / 64];
    float sq = 0.f;
    int n = 0;
    for (int e = lane; e < size; e += 64, ++n) {
        const int c = base + e;
        float acc = 0.f;
        // both places a tap's input can come from are read, at rows that are there, and one is chosen: no load stands
        // under a condition, so a thread's loads are in flight together
        const float* kept_rows = mine ? mine : w;
#pragma unroll 4
        for (int j = 0; j < taps; ++j) {
            const int back = kept - j, place = position - back;
            const bool in_step = place >= first, from_state = !in_step && place >= 0;
            const float here = (float)proj[(size_t)(in_step ? t - back : t) * stride + c];
            const float before = kept_rows[(size_t)(from_state ? kept - (first - place) : 0) * channels + c];
            acc += w[(size_t)c * taps + j] * (in_step ? here : from_state ? before : 0.f);
        }
        acc *= sigmoid_of(acc);
        if (unit) {
            held[n] = acc;
            sq += acc * acc;
        } else {
            out[(size_t)t * channels + c] = acc;
        }
        if (keep && mine) {
            for (int k = 0; k + 1 < kept; ++k) mine[(size_t)k * channels + c] = mine[(size_t)(k + 1) * channels + c];
            mine[(size_t)(kept - 1) * channels + c] = (float)proj[(size_t)t * stride + c];
        }
    }
    if (!unit) return;
    const float inv = rsqrtf(wave_sum(sq) + unit_eps) * (block < kv_heads ? q_scale : 1.f);
    n = 0;
    for (int e = lane; e < size; e += 64, ++n) out[(size_t)t * channels + base + e] = held[n] * inv;
}

// After the step: state[slot][k] = input at position end - kept + k, from the step's rows where it brought that position, from
// the old state where it did not (k + count then indexes it), zero before the sequence.  A thread owns a channel of a row
// and goes through k upwards, so what it still has to read lies above what it has written.
template <typename T>
__global__ __launch_bounds__(256) void delta_conv_keep_kernel(const T* __restrict__ proj, long stride, float* __restrict__ state, long state_stride,
                                                              const int* __restrict__ slots, const int* __restrict__ row_start,
                                                              const int* __restrict__ row_len, const int* __restrict__ row_ctx, int kept, int channels) {
    const int row = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int count = row_len[row], end = row_ctx[row], start = row_start[row];
    if (count <= 0) return;
    const int first = end - count;
    float* mine = state + (size_t)slots[row] * state_stride;
    for (int k = 0; k < kept; ++k) {
        const int place = end - kept + k;
        float v = 0.f;
        if (place >= first) v = (float)proj[(size_t)(start + place - first) * stride + c];
        else if (place >= 0) v = mine[(size_t)(k + count) * channels + c];
        mine[(size_t)k * channels + c] = v;
    }
}

// ---- the delta rule ------------------------------------------------------------------------------------------------------------
// Per head S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, token by token.  A column of S (one value channel)
// needs only its own v and the head's q, k, g, beta, so columns run side by side.  grid (rows, heads, blocks of 16 value
// columns), four wavefronts; a wavefront has four columns, and the 16 lanes of a column share its key channels: lane part p
// keeps the channels p, p + 16, ... (DP of them) of the column in registers for the whole row, so the state is read once
// before a row's first token and written once behind its last.  What the state returns for the key, and the read-out, are
// sums over a column's 16 lanes (four adds across lanes).  Tokens go through LDS in chunks of 16: queries, keys and decays of
// the head laid out by lane part, the chunk's values and write strengths.  Every sum is formed in one order whatever the
// cut and the batch.
constexpr int PARTS = 16;           // lanes that share a column's key channels
constexpr int CHUNK = 16;           // tokens staged at a time
constexpr int BLOCK_COLUMNS = 16;   // value columns a workgroup

template <int CTRL>
__device__ inline float add_across(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// the sum over the 16 lanes of a row of lanes; every lane gets it
__device__ inline float sum_of_16(float v) {
    v = add_across<0xB1>(v);        // quad_perm [1, 0, 3, 2]
    v = add_across<0x4E>(v);        // quad_perm [2, 3, 0, 1]
    v = add_across<0x141>(v);       // row_half_mirror
    v = add_across<0x140>(v);       // row_mirror
    return v;
}

// One token of a column's walk: `S` the lane's key channels of the column, `kp`, `qp`, `gp` the token's key, query and
// decays as the lane's part reads them, `g` the head's decay where there is one a head.
template <int DP, bool PER_CHANNEL>
__device__ inline float delta_token(float (&S)[DP], const float* __restrict__ kp, const float* __restrict__ qp, const float* __restrict__ gp,
                                    float g, float beta, float v) {
    float k[DP], seen[2] = {0.f, 0.f};
#pragma unroll
    for (int i = 0; i < DP; ++i) {
        k[i] = kp[i];
        S[i] *= PER_CHANNEL ? gp[i] : g;
        seen[i & 1] += S[i] * k[i];
    }
    const float u = beta * (v - sum_of_16(seen[0] + seen[1]));
    float read[2] = {0.f, 0.f};
#pragma unroll
    for (int i = 0; i < DP; ++i) {
        S[i] += k[i] * u;
        read[i & 1] += S[i] * qp[i];
    }
    return sum_of_16(read[0] + read[1]);
}

// state[slot]: per head and block of 16 value columns a tile [dim][16], so that a workgroup's share of the state is one
// contiguous piece, read and written 16 bytes a thread and turned into the lanes' order through LDS.
template <int DP, bool PER_CHANNEL>
__global__ __launch_bounds__(256) void delta_rule_kernel(const float* __restrict__ prepared, const float* __restrict__ strength,
                                                         const float* __restrict__ decay, float* state, long state_stride,
                                                         const int* __restrict__ slots, const int* __restrict__ row_start,
                                                         const int* __restrict__ row_len, const int* __restrict__ row_ctx,
                                                         float* __restrict__ out, int heads, int kv_heads, int dim, int value_dim) {
    constexpr int PADDED = DP * PARTS;
    static_assert(CHUNK == BLOCK_COLUMNS, "the staging buffer of the queries doubles as the state's tile");
    __shared__ __align__(16) float s_q[CHUNK][PADDED], s_k[CHUNK][PADDED], s_g[PER_CHANNEL ? CHUNK : 1][PER_CHANNEL ? PADDED : 1];
    __shared__ float s_v[CHUNK][BLOCK_COLUMNS], s_beta[CHUNK], s_decay[CHUNK];
    const int row = blockIdx.x, head = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int count = row_len[row];
    if (count <= 0) return;
    const int start = row_start[row];
    const bool fresh = row_ctx[row] - count == 0;
    const int p = lane & (PARTS - 1);
    const int local = wave * 4 + (lane >> 4);
    const int column = blockIdx.z * BLOCK_COLUMNS + local;
    const bool live = column < value_dim;
    const int kv_head = head / (heads / kv_heads);
    const int keys = kv_heads * dim, channels = 2 * keys + heads * value_dim;
    float* tile = state + (size_t)slots[row] * state_stride + ((size_t)head * gridDim.z + blockIdx.z) * dim * BLOCK_COLUMNS;
    float* turned = &s_q[0][0];                     // [PADDED][16], rows beyond dim unused
    float S[DP];
    if (fresh) {
#pragma unroll
        for (int i = 0; i < DP; ++i) S[i] = 0.f;
    } else {
        for (int piece = tid; piece < dim * (BLOCK_COLUMNS / 4); piece += 256)
            reinterpret_cast<float4*>(turned)[piece] = reinterpret_cast<const float4*>(tile)[piece];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < DP; ++i) {
            const int ch = i * PARTS + p;
            S[i] = (ch < dim && live) ? turned[ch * BLOCK_COLUMNS + local] : 0.f;      // (columns beyond the values stay zero)
        }
    }
    for (int begin = 0; begin < count; begin += CHUNK) {
        const int tokens = min(CHUNK, count - begin);
        __syncthreads();
        // stage the chunk: channel ch of a token goes to [ch % 16][ch / 16], where lane part ch % 16 reads it
        for (int index = tid; index < tokens * PADDED; index += 256) {
            const int j = index / PADDED, ch = index % PADDED;
            const size_t t = (size_t)(start + begin + j);
            const int at = (ch % PARTS) * DP + ch / PARTS;
            const bool there = ch < dim;
            s_q[j][at] = there ? prepared[t * channels + kv_head * dim + ch] : 0.f;
            s_k[j][at] = there ? prepared[t * channels + keys + kv_head * dim + ch] : 0.f;
            if (PER_CHANNEL) s_g[j][at] = there ? decay[(t * heads + head) * dim + ch] : 1.f;
        }
        for (int index = tid; index < tokens * BLOCK_COLUMNS; index += 256) {
            const int j = index / BLOCK_COLUMNS, c = index % BLOCK_COLUMNS;
            const int col = blockIdx.z * BLOCK_COLUMNS + c;
            s_v[j][c] = col < value_dim ? prepared[(size_t)(start + begin + j) * channels + 2 * keys + head * value_dim + col] : 0.f;
        }
        if (tid < tokens) {
            s_beta[tid] = strength[(size_t)(start + begin + tid) * heads + head];
            if (!PER_CHANNEL) s_decay[tid] = decay[(size_t)(start + begin + tid) * heads + head];
        }
        __syncthreads();
        float* o = out + (size_t)(start + begin) * heads * value_dim + (size_t)head * value_dim + column;
        const bool writes = p == 0 && live;
        if (tokens == CHUNK) {
            // a whole chunk runs unrolled: a token's LDS loads are issued ahead of the token before it, and its read-out's
            // sum across lanes overlaps the next token's walk
            // (the read-outs wait in registers for the chunk's end: a store under a condition between two tokens would end
            // the stretch of code that the loads can move within)
            float r[CHUNK];
#pragma unroll
            for (int j = 0; j < CHUNK; ++j)
                r[j] = delta_token<DP, PER_CHANNEL>(S, &s_k[j][p * DP], &s_q[j][p * DP], PER_CHANNEL ? &s_g[j][p * DP] : nullptr,
                                                    PER_CHANNEL ? 1.f : s_decay[j], s_beta[j], s_v[j][local]);
            if (writes) {
#pragma unroll
                for (int j = 0; j < CHUNK; ++j) o[(size_t)j * heads * value_dim] = r[j];
            }
        } else {
            for (int j = 0; j < tokens; ++j) {
                const float r = delta_token<DP, PER_CHANNEL>(S, &s_k[j][p * DP], &s_q[j][p * DP], PER_CHANNEL ? &s_g[j][p * DP] : nullptr,
                                                             PER_CHANNEL ? 1.f : s_decay[j], s_beta[j], s_v[j][local]);
                if (writes) o[(size_t)j * heads * value_dim] = r;
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < DP; ++i) {
        const int ch = i * PARTS + p;
        if (ch < dim) turned[ch * BLOCK_COLUMNS + local] = S[i];
    }
    __syncthreads();
    for (int piece = tid; piece < dim * (BLOCK_COLUMNS / 4); piece += 256)
        reinterpret_cast<float4*>(tile)[piece] = reinterpret_cast<const float4*>(turned)[piece];
}

}  // namespace

LSA_EXPORT int lsa_gated_pair_update(float* x, const void* gates, int gates_code, int gate_width, const void* y1, int y1_code, const float* s1,
                                     const void* y2, int y2_code, const float* s2, const float* next_weight, float eps, void* normed,
                                     int normed_code, int n, int width, hipStream_t stream) {
    if (n <= 0) return 0;
    if (gate_width != (y2 ? 2 * width : width) || (y2 && !s2) || (next_weight && !normed)) return -1;
    if (!y2) y2_code = 0;
#define LSA_LAUNCH_R(G, Y1, Y2, N, R) gated_pair_update_kernel<G, Y1, Y2, N, R><<<n, 256, 0, stream>>>(x, (const G*)gates, gate_width, (const Y1*)y1, s1, \
        (const Y2*)y2, s2, next_weight, eps, (N*)normed, width)
#define LSA_LAUNCH(G, Y1, Y2, N) do { if (width <= 1024) LSA_LAUNCH_R(G, Y1, Y2, N, 4); else if (width <= 2048) LSA_LAUNCH_R(G, Y1, Y2, N, 8); \
                                      else if (width <= 256 * UPDATE_COLS) LSA_LAUNCH_R(G, Y1, Y2, N, UPDATE_COLS); else LSA_LAUNCH_R(G, Y1, Y2, N, 0); } while (0)
#define LSA_BY_N(G, Y1, Y2) do { if (normed_code) LSA_LAUNCH(G, Y1, Y2, bf16_t); else LSA_LAUNCH(G, Y1, Y2, float); } while (0)
#define LSA_BY_Y2(G, Y1) do { if (y2_code) LSA_BY_N(G, Y1, bf16_t); else LSA_BY_N(G, Y1, float); } while (0)
#define LSA_BY_Y1(G) do { if (y1_code) LSA_BY_Y2(G, bf16_t); else LSA_BY_Y2(G, float); } while (0)
    if (gates_code) LSA_BY_Y1(bf16_t); else LSA_BY_Y1(float);
#undef LSA_BY_Y1
#undef LSA_BY_Y2
#undef LSA_BY_N
#undef LSA_LAUNCH
#undef LSA_LAUNCH_R
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_differential_heads(int code, const void* attended, float lam, float keep, float eps, void* out, int n, int kv_heads,
                                      int group, int value_dim, int row, hipStream_t stream) {
    if (n <= 0) return 0;
    if (value_dim > row || kv_heads < 1 || group < 1) return -1;
    dim3 grid(n, kv_heads * group);
    if (code) differential_heads_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)attended, lam, keep, eps, (bf16_t*)out, group, value_dim, row);
    else differential_heads_kernel<float><<<grid, 64, 0, stream>>>((const float*)attended, lam, keep, eps, (float*)out, group, value_dim, row);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_delta_most_dim() { return MOST_DIM; }
LSA_EXPORT int lsa_delta_state_columns() { return BLOCK_COLUMNS; }

LSA_EXPORT int lsa_delta_prepare(int code, const void* proj, long stride, const float* w, int taps, float* state, long state_stride,
                                 const int* slots, const int* token_row, const int* positions, const int* row_start, float* out,
                                 int kv_heads, int heads, int dim, int value_dim, float q_scale, float unit_eps, int keep,
                                 const void* strength, long strength_stride, const void* decay, long decay_stride, int per_channel,
                                 const float* decay_scale, const float* decay_bias, float* out_strength, float* out_decay, int n,
                                 hipStream_t stream) {
    if (n <= 0) return 0;
    if (taps < 1 || dim < 1 || dim > MOST_DIM || heads < 1 || kv_heads < 1 || heads % kv_heads || (taps > 1 && (!state || !slots))) return -1;
    dim3 grid(n, 2 * kv_heads + 2 * heads);
#define LSA_LAUNCH(T) delta_prepare_kernel<T><<<grid, 64, 0, stream>>>((const T*)proj, stride, w, taps, state, state_stride, slots, token_row, positions, \
        row_start, out, kv_heads, heads, dim, value_dim, q_scale, unit_eps, keep, (const T*)strength, strength_stride, decay, decay_stride, \
        per_channel, decay_scale, decay_bias, out_strength, out_decay)
    if (code) LSA_LAUNCH(bf16_t); else LSA_LAUNCH(float);
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_delta_conv_keep(int code, const void* proj, long stride, float* state, long state_stride, const int* slots,
                                   const int* row_start, const int* row_len, const int* row_ctx, int kept, int channels, int rows,
                                   hipStream_t stream) {
    if (rows <= 0 || kept <= 0) return 0;
    dim3 grid(rows, (channels + 255) / 256);
    if (code) delta_conv_keep_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)proj, stride, state, state_stride, slots, row_start, row_len, row_ctx, kept, channels);
    else delta_conv_keep_kernel<float><<<grid, 256, 0, stream>>>((const float*)proj, stride, state, state_stride, slots, row_start, row_len, row_ctx, kept, channels);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_delta_rule(const float* prepared, const float* strength, const float* decay, int per_channel, float* state,
                              long state_stride, const int* slots, const int* row_start, const int* row_len, const int* row_ctx,
                              float* out, int rows, int heads, int kv_heads, int dim, int value_dim, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim < 1 || dim > MOST_DIM || heads < 1 || kv_heads < 1 || heads % kv_heads || value_dim < 1 || !state) return -1;
    dim3 grid(rows, heads, (value_dim + BLOCK_COLUMNS - 1) / BLOCK_COLUMNS);
    if (state_stride < (long)heads * grid.z * dim * BLOCK_COLUMNS || state_stride % 4 || ((size_t)state % 16)) return -1;
    const int parts = (dim + PARTS - 1) / PARTS;
#define LSA_LAUNCH(DP, PC) delta_rule_kernel<DP, PC><<<grid, 256, 0, stream>>>(prepared, strength, decay, state, state_stride, slots, row_start, \
        row_len, row_ctx, out, heads, kv_heads, dim, value_dim)
#define LSA_BY_DP(PC) do { if (parts <= 1) LSA_LAUNCH(1, PC); else if (parts <= 2) LSA_LAUNCH(2, PC); else if (parts <= 4) LSA_LAUNCH(4, PC); \
                           else if (parts <= 8) LSA_LAUNCH(8, PC); else LSA_LAUNCH(16, PC); } while (0)
    if (per_channel) LSA_BY_DP(true); else LSA_BY_DP(false);
#undef LSA_BY_DP
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}
