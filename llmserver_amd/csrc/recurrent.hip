// Kernels of the mixers that carry a state of fixed size from token to token: the mix of a token's row with the row
// before it, the linear recurrence S_t = diag(d_t) S_(t-1) + k_t v_t^T with its read-out, the matrix memory with
// exponential gates and a normaliser, and the per-head norm and gate behind them.  Decays, their exponentials and logarithms, the state, the sums and the norm are float32; projections
// arrive in the activations' type and are widened where they are read; a result for a 16-bit consumer is rounded once.
#include "common.hpp"

using namespace lsa;

// out[m][t] = h[t] + (before[t] - h[t]) * mu[m], before[t] = the row of the token before t in its request: a row of this
// step, the request's state for a row's first token, zeros at position 0.  grid (tokens, blocks of 256 columns): a thread
// has one column of one token, so its two loads are the only ones it waits for.  keep (only in steps of one token per
// row, where a column of a row's state is one thread's): the state becomes this token's row.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(const T* __restrict__ h, const float* __restrict__ mu, int mixes,
                                                          float* state, long state_stride, const int* __restrict__ slots,
                                                          const int* __restrict__ token_row, const int* __restrict__ positions,
                                                          const int* __restrict__ row_start, T* __restrict__ out, int n_tokens, int width,
                                                          int keep) {
    const int t = blockIdx.x;
    const int row = token_row[t];
    const bool first_of_sequence = positions[t] == 0, first_of_row = t == row_start[row];
    float* mine = state + (size_t)slots[row] * state_stride;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
        const float own = (float)h[(size_t)t * width + c];
        float before = 0.f;
        if (!first_of_sequence) before = first_of_row ? mine[c] : (float)h[(size_t)(t - 1) * width + c];
        const float difference = before - own;
        for (int m = 0; m < mixes; ++m)
            out[((size_t)m * n_tokens + t) * width + c] = (T)(own + difference * mu[(size_t)m * width + c]);
        if (keep) mine[c] = own;
    }
}

// state[slot] = the last row of every row of the step (rows without tokens keep theirs).
template <typename T>
__global__ __launch_bounds__(256) void token_shift_keep_kernel(const T* __restrict__ h, float* __restrict__ state, long state_stride,
                                                               const int* __restrict__ slots, const int* __restrict__ row_start,
                                                               const int* __restrict__ row_len, int width) {
    const int row = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int count = row_len[row];
    if (c >= width || count <= 0) return;
    state[(size_t)slots[row] * state_stride + c] = (float)h[(size_t)(row_start[row] + count - 1) * width + c];
}

// The decay of a key channel from its 32-bit logit.  mode 0: sigmoid(z)^(1 / tau) = exp(log sigmoid(z) / tau);
// mode 1: exp(-exp(z)).
__device__ __forceinline__ float decay_of(float z, int mode, float inv_tau) {
    if (mode == 0) {
        const float log_sigmoid = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
        return expf(log_sigmoid * inv_tau);
    }
    return expf(-expf(z));
}

// One token of one wavefront's DK channels: the state's update and the channels' part of the read-out.  The channels come
// from LDS four at a time (16-byte broadcast reads: every row of a chunk and every wavefront's first channel lie at
// multiples of 32 bytes); four partial sums of the read-out make its chain of dependent multiply-adds a quarter as long.
template <int DK, bool BONUS>
__device__ __forceinline__ float recurrence_token(float (&S)[DK], const float (&u)[DK], const float* q_row, const float* k_row,
                                                  const float* d_row, float value) {
    const float4* tq = reinterpret_cast<const float4*>(q_row);
    const float4* tk = reinterpret_cast<const float4*>(k_row);
    const float4* td = reinterpret_cast<const float4*>(d_row);
    float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i4 = 0; i4 < DK / 4; ++i4) {
        const float4 q4 = tq[i4], k4 = tk[i4], d4 = td[i4];
        const float qs[4] = {q4.x, q4.y, q4.z, q4.w}, ks[4] = {k4.x, k4.y, k4.z, k4.w}, ds[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int i = 4 * i4 + e;
            const float kv = ks[e] * value;
            if (BONUS) {
                o4[e] = __builtin_fmaf(__builtin_fmaf(u[i], kv, S[i]), qs[e], o4[e]);
                S[i] = __builtin_fmaf(ds[e], S[i], kv);
            } else {
                S[i] = __builtin_fmaf(ds[e], S[i], kv);
                o4[e] = __builtin_fmaf(S[i], qs[e], o4[e]);
            }
        }
    }
    return (o4[0] + o4[1]) + (o4[2] + o4[3]);
}

// grid (rows, heads, blocks of 64 value columns); a workgroup of NW wavefronts walks the row's tokens in order.
// Lane = value column; wavefront w (of up to eight) owns key channels [w * DK, (w + 1) * DK) and keeps its DK x 64 piece of the head's
// state in registers, so the state is read once before the row's first token and written once after its last one.
// The tokens go through LDS in chunks of CHUNK: queries (scaled), keys and decays of the head, widened and, for the
// decays, exponentiated once per (token, channel) by whichever thread loads them; the chunk's values of this block of
// columns; and, per wavefront, the partial read-outs of its channels, which are added up over the wavefronts when the
// chunk is through.  A wavefront reads its channels of a token from LDS as broadcasts; nothing crosses lanes.
//   BONUS false: S = d S + k v^T, then o = S^T q.      BONUS true: o = (S + (u k) v^T)^T q, then S = d S + k v^T.
// Every sum is formed in the same order whatever the step's other rows and however the sequence was cut into steps:
// the state after a token and the token's read-out are the same bits either way.
constexpr int CHUNK = 16;

template <typename T, int DK, bool BONUS>
__global__ __launch_bounds__(512) void linear_recurrence_kernel(const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
                                         const T* __restrict__ v, long v_stride, const float* __restrict__ decay,
                                         const float* __restrict__ decay_bias, int mode, float inv_tau, const float* __restrict__ bonus,
                                         float q_scale, float* state, long state_stride, const int* __restrict__ slots,
                                         const int* __restrict__ row_start, const int* __restrict__ row_len, const int* __restrict__ row_ctx,
                                         float* __restrict__ out, int heads, int dim, int value_dim) {
    extern __shared__ __align__(16) float lds[];
    const int row = blockIdx.x, head = blockIdx.y, column0 = blockIdx.z * 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int count = row_len[row];
    if (count <= 0) return;                              // (the whole workgroup: nobody waits at a barrier below)
    const int start = row_start[row], first_position = row_ctx[row] - count;
    const int padded = waves * DK;                       // channels as the wavefronts share them; those behind dim are zeros
    float* s_q = lds;                                    // [CHUNK][padded]
    float* s_k = s_q + CHUNK * padded;
    float* s_d = s_k + CHUNK * padded;
    float* s_v = s_d + CHUNK * padded;                   // [CHUNK][64]
    float* s_o = s_v + CHUNK * 64;                       // [waves][CHUNK][64]
    const int column = column0 + lane;
    const bool column_ok = column < value_dim;
    const int channel0 = wave * DK;
    float* mine = state + (size_t)slots[row] * state_stride + ((size_t)head * dim + channel0) * value_dim + column;
    float S[DK], u[DK];
#pragma unroll
    for (int i = 0; i < DK; ++i) {
        const bool ok = column_ok && channel0 + i < dim;
        S[i] = (ok && first_position > 0) ? mine[(size_t)i * value_dim] : 0.f;
        u[i] = (BONUS && channel0 + i < dim) ? bonus[(size_t)head * dim + channel0 + i] : 0.f;
    }
    const size_t key_column = (size_t)head * dim;
    for (int t0 = 0; t0 < count; t0 += CHUNK) {
        const int n = min(CHUNK, count - t0);
        __syncthreads();                                 // the chunk before has been read out of LDS
        // A thread stages PER numbers of each kind (CHUNK * padded = PER * blockDim.x): all their loads first, so that they are
        // in flight together, then the decays' exponentials and the stores.
        constexpr int PER = CHUNK * DK / 64;
        float raw_q[PER], raw_k[PER], raw_z[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = threadIdx.x + j * blockDim.x;
            const int t = i / padded, c = i - t * padded;
            raw_q[j] = 0.f; raw_k[j] = 0.f; raw_z[j] = 0.f;
            if (t < n && c < dim) {
                const size_t token = (size_t)(start + t0 + t);
                raw_q[j] = (float)q[token * q_stride + key_column + c];
                raw_k[j] = (float)k[token * k_stride + key_column + c];
                raw_z[j] = decay[token * (size_t)heads * dim + key_column + c] + (decay_bias ? decay_bias[key_column + c] : 0.f);
            }
        }
        for (int i = threadIdx.x; i < n * 64; i += blockDim.x) {
            const int t = i >> 6, c = column0 + (i & 63);
            s_v[i] = c < value_dim ? (float)v[(size_t)(start + t0 + t) * v_stride + (size_t)head * value_dim + c] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = threadIdx.x + j * blockDim.x;
            const int t = i / padded, c = i - t * padded;
            if (t >= n) continue;
            s_q[i] = raw_q[j] * q_scale;
            s_k[i] = raw_k[j];
            s_d[i] = c < dim ? decay_of(raw_z[j], mode, inv_tau) : 1.f;
        }
        __syncthreads();
        if (DK <= 16 && n == CHUNK) {
            // A whole chunk: the tokens' steps unrolled, their read-outs kept in registers and stored behind the last one, so
            // that no store to LDS stands between one token's loads and the next one's and the loads can run ahead.  (With
            // more channels a wavefront the state alone fills the registers, and running ahead would spill.)
            float kept[CHUNK];
#pragma unroll
            for (int t = 0; t < CHUNK; ++t)
                kept[t] = recurrence_token<DK, BONUS>(S, u, s_q + t * padded + channel0, s_k + t * padded + channel0,
                                                      s_d + t * padded + channel0, s_v[t * 64 + lane]);
#pragma unroll
            for (int t = 0; t < CHUNK; ++t) s_o[(wave * CHUNK + t) * 64 + lane] = kept[t];
        } else {
            for (int t = 0; t < n; ++t)
                s_o[(wave * CHUNK + t) * 64 + lane] = recurrence_token<DK, BONUS>(S, u, s_q + t * padded + channel0, s_k + t * padded + channel0,
                                                                                  s_d + t * padded + channel0, s_v[t * 64 + lane]);
        }
        __syncthreads();
        for (int i = threadIdx.x; i < n * 64; i += blockDim.x) {
            const int t = i >> 6, c = i & 63;
            if (column0 + c >= value_dim) continue;
            float total = 0.f;
            for (int w = 0; w < waves; ++w) total += s_o[(w * CHUNK + t) * 64 + c];
            out[(size_t)(start + t0 + t) * heads * value_dim + (size_t)head * value_dim + column0 + c] = total;
        }
    }
#pragma unroll
    for (int i = 0; i < DK; ++i)
        if (column_ok && channel0 + i < dim) mine[(size_t)i * value_dim] = S[i];
}

// grid (tokens, heads), one wavefront: out = x' / rms(x') * w * act(gate) over a head's value_dim numbers; x float32,
// w = weight[head * weight_stride + j] (weight_stride 0: one weight shared by the heads), gate and out of type T;
// act: gate * sigmoid(gate) (gate_kind 0) or sigmoid(gate) (1).  x' = x, or, with below [tokens][heads][2]:
// x / (max(|below[0]|, below[1]) + floor), the read-out of a matrix memory under its normaliser.
template <typename T>
__global__ __launch_bounds__(64) void heads_norm_gate_kernel(const float* __restrict__ x, const float* __restrict__ weight, int weight_stride,
                                                             float eps, const T* __restrict__ gate, long gate_stride, T* __restrict__ out,
                                                             int heads, int value_dim, int gate_kind, const float* __restrict__ below,
                                                             float floor) {
    const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* row = x + ((size_t)t * heads + head) * value_dim;
    float under = 1.f;
    if (below) {
        const float* b = below + ((size_t)t * heads + head) * 2;
        under = fmaxf(fabsf(b[0]), b[1]) + floor;
    }
    float sq = 0.f;
    for (int j = lane; j < value_dim; j += 64) {
        const float xv = below ? row[j] / under : row[j];
        sq += xv * xv;
    }
    const float inv = rsqrtf(wave_sum(sq) / (float)value_dim + eps);
    const T* g = gate + (size_t)t * gate_stride + (size_t)head * value_dim;
    const float* w = weight + (size_t)head * weight_stride;
    T* o = out + ((size_t)t * heads + head) * value_dim;
    for (int j = lane; j < value_dim; j += 64) {
        const float gv = (float)g[j];
        const float sigmoid = 1.f / (1.f + expf(-gv));
        const float xv = below ? row[j] / under : row[j];
        o[j] = (T)(xv * inv * w[j] * (gate_kind ? sigmoid : gv * sigmoid));
    }
}

// ---- a matrix memory with exponential gates --------------------------------------------------------------------------
// Per head and token: log input gate i = cap tanh(z_i / cap), log forget gate f = logsigmoid(cap tanh(z_f / cap)), a running
// maximum m_t = max(f + m_(t-1), i) (0 in front of the first token), and from them what the memory's update needs: keep = exp(f + m_(t-1) -
// m_t), take = exp(i - m_t), and exp(-m_t) for the read-out's denominator.  grid (rows, heads), eight wavefronts: the row's
// tokens 448 at a time; seven wavefronts have a thread a token for the transcendental functions, one thread of the eighth
// walks the maximum through the tokens (two dependent instructions a token), and while it walks a group the others
// prepare the group behind it and finish the group before it.  gates [T][2 heads] (inputs, then forgets), coef [T][heads][2] (keep, take),
// below [T][heads][2] (its second number is written here), top[slot][head] the maximum between steps (0 at position 0).
// run (or nullptr) [T][heads]: the sum of log keep from the first token of a token's chunk of 64 (counted from the row's
// first token of this step) up to the token itself, in 64-bit: what the chunked form of the memory forms its weights from.
constexpr int GATES_WAVES = 8;            // the first walks, the others work: seven chunks of 64 tokens at a time
__global__ __launch_bounds__(64 * GATES_WAVES) void memory_gates_kernel(const float* __restrict__ gates, float cap, float* state, long state_stride,
                                                          long top_offset, const int* __restrict__ slots, const int* __restrict__ row_start,
                                                          const int* __restrict__ row_len, const int* __restrict__ row_ctx,
                                                          float* __restrict__ coef, float* __restrict__ below, int heads,
                                                          double* __restrict__ run) {
    constexpr int GROUP = 64 * (GATES_WAVES - 1);                      // tokens at a time: a working wavefront a chunk of 64
    // two of each: while one group's maxima are walked, the group behind it is prepared and the group before it finished
    __shared__ __align__(16) float s_in[2][GROUP], s_forget[2][GROUP], s_top[2][GROUP + 8];                 // (the maximum in front of a group's token t at [3 + t], behind it at [4 + t]: sixteen bytes at a time)
    const int row = blockIdx.x, head = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    const int count = row_len[row];
    if (count <= 0) return;
    const int start = row_start[row], first_position = row_ctx[row] - count;
    float* kept = state + (size_t)slots[row] * state_stride + top_offset + head;
    const float inv_cap = 1.f / cap;
    const int groups = (count + GROUP - 1) / GROUP;
    const bool walker = tid < 64;
    const int mine = tid - 64;                                         // a worker's token of a group
    float m = 0.f;                                                     // (the walker's: the maximum so far)
    if (tid == 0) m = first_position > 0 ? *kept : 0.f;
    // what a worker keeps of its token of the group that is being walked, until the maxima are there
    float log_in = 0.f, log_forget = 0.f;
    auto prepare = [&](int g) {                                        // caps and logarithms of group g's gates
        const int n = min(GROUP, count - g * GROUP);
        log_in = 0.f; log_forget = 0.f;
        if (mine < n) {
            const size_t token = (size_t)(start + g * GROUP + mine);
            log_in = cap * tanhf(gates[token * 2 * heads + head] * inv_cap);
            const float z = cap * tanhf(gates[token * 2 * heads + heads + head] * inv_cap);
            log_forget = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
        }
        s_in[g & 1][mine] = log_in;
        s_forget[g & 1][mine] = log_forget;
    };
    auto finish = [&](int g, float li, float lf) {                     // group g's coefficients, from its maxima
        const int n = min(GROUP, count - g * GROUP);
        const size_t token = (size_t)(start + g * GROUP + mine);
        float log_keep = 0.f;
        if (mine < n) {
            const float before = s_top[g & 1][3 + mine], now = s_top[g & 1][4 + mine];
            log_keep = (lf + before) - now;
            coef[(token * heads + head) * 2] = expf(log_keep);
            coef[(token * heads + head) * 2 + 1] = expf(li - now);
            below[(token * heads + head) * 2 + 1] = expf(-now);
        }
        if (run != nullptr) {                                          // the chunk's running sum of log keep, token by token
            double total = (double)log_keep;
#pragma unroll
            for (int step = 1; step < 64; step <<= 1) {
                const double other = __shfl_up(total, step, 64);
                if (lane >= step) total += other;
            }
            if (mine < n) run[token * heads + head] = total;
        }
    };
    if (!walker) prepare(0);
    __syncthreads();
    float walked_in = 0.f, walked_forget = 0.f;                        // a worker's token of the group that is being walked
    for (int g = 0; g < groups; ++g) {
        if (walker) {
            if (tid == 0) {                                            // the walk: one thread, two dependent instructions a token
                const int n = min(GROUP, count - g * GROUP);
                const float* fs_all = s_forget[g & 1];
                const float* is_all = s_in[g & 1];
                float* tops = s_top[g & 1];
                tops[3] = m;
                int t = 0;
                for (; t + 64 <= n; t += 64) {                         // a whole chunk: all loads first, then the chain alone
                    float fs[64], is[64], ms[64];
#pragma unroll
                    for (int t4 = 0; t4 < 16; ++t4) {
                        const float4 f4 = reinterpret_cast<const float4*>(fs_all + t)[t4], i4 = reinterpret_cast<const float4*>(is_all + t)[t4];
                        fs[4 * t4] = f4.x; fs[4 * t4 + 1] = f4.y; fs[4 * t4 + 2] = f4.z; fs[4 * t4 + 3] = f4.w;
                        is[4 * t4] = i4.x; is[4 * t4 + 1] = i4.y; is[4 * t4 + 2] = i4.z; is[4 * t4 + 3] = i4.w;
                    }
#pragma unroll
                    for (int u = 0; u < 64; ++u) {
                        m = fmaxf(fs[u] + m, is[u]);
                        ms[u] = m;
                    }
#pragma unroll
                    for (int u4 = 0; u4 < 16; ++u4)
                        reinterpret_cast<float4*>(tops + 4 + t)[u4] = make_float4(ms[4 * u4], ms[4 * u4 + 1], ms[4 * u4 + 2], ms[4 * u4 + 3]);
                }
                for (; t < n; ++t) {
                    m = fmaxf(fs_all[t] + m, is_all[t]);
                    tops[4 + t] = m;
                }
            }
        } else {
            const float li = walked_in, lf = walked_forget;            // (group g - 1's, whose maxima are there)
            walked_in = log_in; walked_forget = log_forget;            // (group g's, which is being walked)
            if (g + 1 < groups) prepare(g + 1);
            if (g > 0) finish(g - 1, li, lf);
        }
        __syncthreads();
    }
    if (!walker) finish(groups - 1, walked_in, walked_forget);
    if (tid == 0) *kept = m;
}

// One token of one wavefront's DK channels of a matrix memory: S = keep S + k value (value: the token's value column times its
// take), and the channels' part of the read-out S^T q; the channels come from LDS as in recurrence_token.
template <int DK>
__device__ __forceinline__ float memory_token(float (&S)[DK], const float* q_row, const float* k_row, float keep, float value) {
    const float4* tq = reinterpret_cast<const float4*>(q_row);
    const float4* tk = reinterpret_cast<const float4*>(k_row);
    float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i4 = 0; i4 < DK / 4; ++i4) {
        const float4 q4 = tq[i4], k4 = tk[i4];
        const float qs[4] = {q4.x, q4.y, q4.z, q4.w}, ks[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int i = 4 * i4 + e;
            S[i] = __builtin_fmaf(keep, S[i], ks[e] * value);
            o4[e] = __builtin_fmaf(S[i], qs[e], o4[e]);
        }
    }
    return (o4[0] + o4[1]) + (o4[2] + o4[3]);
}

// The memory itself, laid out as linear_recurrence_kernel: grid (rows, heads, blocks of 64 columns), lane = column,
// wavefront w owns key channels [w * DK, (w + 1) * DK) and keeps its piece of the state in registers over the row's tokens.
// The columns are the head's value_dim value columns and, behind them, one more whose "value" is 1: its piece of the state
// is the normaliser n, which obeys the same recurrence with k in place of k v^T, and its read-out is n . q.  So
// out [T][heads * value_dim] gets the numerators S^T q and below [T][heads][2] (first number) gets n . q; the division is
// left to the kernel that normalises the heads.  state[slot]: the matrices [heads][dim][value_dim], then the normalisers
// [heads][dim].  Every sum is formed in the same order however the sequence was cut into steps.
template <typename T, int DK>
__global__ __launch_bounds__(512) void matrix_memory_kernel(const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
                                         const T* __restrict__ v, long v_stride, const float* __restrict__ coef, float q_scale,
                                         float* state, long state_stride, const int* __restrict__ slots,
                                         const int* __restrict__ row_start, const int* __restrict__ row_len, const int* __restrict__ row_ctx,
                                         float* __restrict__ out, float* __restrict__ below, int heads, int dim, int value_dim) {
    extern __shared__ __align__(16) float lds[];
    const int row = blockIdx.x, head = blockIdx.y, column0 = blockIdx.z * 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int count = row_len[row];
    if (count <= 0) return;                              // (the whole workgroup: nobody waits at a barrier below)
    const int start = row_start[row], first_position = row_ctx[row] - count;
    const int padded = waves * DK;                       // channels as the wavefronts share them; those behind dim are zeros
    float* s_q = lds;                                    // [CHUNK][padded]
    float* s_k = s_q + CHUNK * padded;
    float* s_v = s_k + CHUNK * padded;                   // [CHUNK][64], each value times its token's take
    float* s_keep = s_v + CHUNK * 64;                    // [CHUNK]
    float* s_o = s_keep + CHUNK;                         // [waves][CHUNK][64]
    const int column = column0 + lane;
    const bool is_value = column < value_dim, is_normaliser = column == value_dim;
    const int channel0 = wave * DK;
    float* slot = state + (size_t)slots[row] * state_stride;
    // a channel's number of this column: in the matrix, or in the normaliser behind the matrices
    float* mine = is_value ? slot + ((size_t)head * dim + channel0) * value_dim + column
                           : slot + (size_t)heads * dim * value_dim + (size_t)head * dim + channel0;
    const size_t channel_stride = is_value ? (size_t)value_dim : 1;
    float S[DK];
#pragma unroll
    for (int i = 0; i < DK; ++i) {
        const bool ok = (is_value || is_normaliser) && channel0 + i < dim;
        S[i] = (ok && first_position > 0) ? mine[(size_t)i * channel_stride] : 0.f;
    }
    const size_t key_column = (size_t)head * dim;
    for (int t0 = 0; t0 < count; t0 += CHUNK) {
        const int n = min(CHUNK, count - t0);
        __syncthreads();                                 // the chunk before has been read out of LDS
        constexpr int PER = CHUNK * DK / 64;
        float raw_q[PER], raw_k[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = threadIdx.x + j * blockDim.x;
            const int t = i / padded, c = i - t * padded;
            raw_q[j] = 0.f; raw_k[j] = 0.f;
            if (t < n && c < dim) {
                const size_t token = (size_t)(start + t0 + t);
                raw_q[j] = (float)q[token * q_stride + key_column + c];
                raw_k[j] = (float)k[token * k_stride + key_column + c];
            }
        }
        for (int i = threadIdx.x; i < n * 64; i += blockDim.x) {
            const int t = i >> 6, c = column0 + (i & 63);
            const size_t token = (size_t)(start + t0 + t);
            const float take = coef[(token * heads + head) * 2 + 1];
            const float value = c < value_dim ? (float)v[token * v_stride + (size_t)head * value_dim + c] : (c == value_dim ? 1.f : 0.f);
            s_v[i] = take * value;
        }
        if (threadIdx.x < n) s_keep[threadIdx.x] = coef[((size_t)(start + t0 + threadIdx.x) * heads + head) * 2];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = threadIdx.x + j * blockDim.x;
            if (i / padded >= n) continue;
            s_q[i] = raw_q[j] * q_scale;
            s_k[i] = raw_k[j];
        }
        __syncthreads();
        if (DK <= 16 && n == CHUNK) {
            float kept[CHUNK];
#pragma unroll
            for (int t = 0; t < CHUNK; ++t)
                kept[t] = memory_token<DK>(S, s_q + t * padded + channel0, s_k + t * padded + channel0, s_keep[t], s_v[t * 64 + lane]);
#pragma unroll
            for (int t = 0; t < CHUNK; ++t) s_o[(wave * CHUNK + t) * 64 + lane] = kept[t];
        } else {
            for (int t = 0; t < n; ++t)
                s_o[(wave * CHUNK + t) * 64 + lane] = memory_token<DK>(S, s_q + t * padded + channel0, s_k + t * padded + channel0,
                                                                       s_keep[t], s_v[t * 64 + lane]);
        }
        __syncthreads();
        for (int i = threadIdx.x; i < n * 64; i += blockDim.x) {
            const int t = i >> 6, c = column0 + (i & 63);
            if (c > value_dim) continue;
            float total = 0.f;
            for (int w = 0; w < waves; ++w) total += s_o[(w * CHUNK + t) * 64 + (i & 63)];
            const size_t token = (size_t)(start + t0 + t);
            if (c < value_dim) out[token * heads * value_dim + (size_t)head * value_dim + c] = total;
            else below[(token * heads + head) * 2] = total;
        }
    }
#pragma unroll
    for (int i = 0; i < DK; ++i)
        if ((is_value || is_normaliser) && channel0 + i < dim) mine[(size_t)i * channel_stride] = S[i];
}

// ---- the matrix memory in chunks -------------------------------------------------------------------------------------
// A row's tokens of a step in chunks of 64, counted from the row's first token of the step.  With L_t the sum of log keep
// from the chunk's first token to t, the state behind token t is e^(L_t) S_0 + sum_(j <= t) e^(L_t - L_j) take_j k_j v_j^T
// (S_0 the state in front of the chunk), and every weight is at most 1.  So (1) every chunk's own sum
// U = sum_j e^(L_last - L_j) take_j k_j v_j^T is a matrix product, all chunks at once; (2) a walk over a row's chunks,
// S <- e^(L_last) S + U, leaves the state in front of every chunk where U stood, and the row's last state in its slot; (3) a
// chunk's read-outs are two products, (scores q_t . k_j times their weights) x values and (e^(L_t) q_t) x S_0, again all
// chunks at once.  One more column behind the values, whose "value" is 1, carries the normaliser as in the scan.  All
// operands are float32 in LDS and the products run on v_mfma_f32_16x16x4_f32; a workgroup of four wavefronts forms 64 x 64
// results, a wavefront 32 x 32 of them.  An item is a (row, chunk): the grid has as many as the step could have at most,
// and a workgroup finds its row by walking the rows' lengths.
constexpr int MC = 64;                   // tokens a chunk
constexpr int MC_A = 68;                 // row length in LDS of an operand read down its rows (a lane a row)
constexpr int MC_B = 80;                 // ... of an operand read along its rows (a lane a column)

__device__ __forceinline__ bool memory_item(int item, int rows, const int* __restrict__ row_len, int& row, int& chunk) {
    int base = 0;
    for (int r = 0; r < rows; ++r) {
        const int count = row_len[r];
        const int chunks = count > 0 ? (count + MC - 1) / MC : 0;
        if (item < base + chunks) { row = r; chunk = item - base; return true; }
        base += chunks;
    }
    return false;
}

// acc += A B over inner indices [0, inner) (a multiple of 16; what lies behind an operand's end is zeros): A's (m, i) at
// a[m * MC_A + i], m counted from the wavefront's first row; B's (i, n) at b[i * b_inner + n * b_column], n counted from the
// wavefront's first column.  acc[mi][ni][e] is the result at row 16 mi + 4 (lane / 16) + e, column 16 ni + lane % 16.
// Sixteen inner indices at a time: their sixteen LDS loads are issued before the first of their sixteen products.
typedef float mc_f4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void memory_product(mc_f4 (&acc)[2][2], const float* a, const float* b, int b_inner, int b_column, int inner, int lane) {
    const int r = lane & 15, g = lane >> 4;
    const float* a0 = a + r * MC_A + g;
    const float* a1 = a0 + 16 * MC_A;
    const float* b0 = b + g * b_inner + r * b_column;
    const float* b1 = b0 + 16 * b_column;
    for (int i = 0; i < inner; i += 16) {
        float x0[4], x1[4], y0[4], y1[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            x0[u] = a0[i + 4 * u]; x1[u] = a1[i + 4 * u];
            y0[u] = b0[(i + 4 * u) * b_inner]; y1[u] = b1[(i + 4 * u) * b_inner];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(x0[u], y0[u], acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(x0[u], y1[u], acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(x1[u], y0[u], acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(x1[u], y1[u], acc[1][1], 0, 0, 0);
        }
    }
}

// A chunk's values of 64 columns from column0 on, [token][column] in LDS: zeros behind the chunk's last token and behind the
// column of ones that stands behind the values.  All of a thread's loads are issued before it stores.
template <typename T>
__device__ __forceinline__ void memory_stage_values(float* s_v, const T* __restrict__ v, long v_stride, size_t token0, int n, int head,
                                                    int value_dim, int column0, int tid) {
    T values[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        // (every load is of a place that is there, so that none stands under a condition and all are on their way together)
        const int t = min(4 * j + (tid >> 6), n - 1), c = min(column0 + (tid & 63), value_dim - 1);
        values[j] = v[(token0 + t) * v_stride + (size_t)head * value_dim + c];
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int t = 4 * j + (tid >> 6), c = column0 + (tid & 63);
        s_v[t * MC_B + (tid & 63)] = t < n ? (c < value_dim ? (float)values[j] : (c == value_dim ? 1.f : 0.f)) : 0.f;
    }
}

// (1) sums[item][head][channel][column] = sum_j e^(L_last - L_j) take_j k_j[channel] value_j[column]; grid (items, heads,
// blocks of 64 columns of value_dim + 1), 256 threads.  A = the weighted keys, read as [channel][token]; B = the values.
template <typename T>
__global__ __launch_bounds__(256) void memory_chunk_sums_kernel(const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride,
                                                                const float* __restrict__ coef, const double* __restrict__ run,
                                                                const int* __restrict__ row_start, const int* __restrict__ row_len, int rows,
                                                                float* __restrict__ sums, int heads, int dim, int value_dim) {
    __shared__ float s_k[MC * MC_A];                     // [channel][token]
    __shared__ float s_v[MC * MC_B];                     // [token][column]
    __shared__ float s_w[MC];
    int row, chunk;
    if (!memory_item(blockIdx.x, rows, row_len, row, chunk)) return;
    const int head = blockIdx.y, column0 = blockIdx.z * 64, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = min(MC, row_len[row] - chunk * MC);
    const size_t token0 = (size_t)row_start[row] + (size_t)chunk * MC;
    const int ld = value_dim + 1;
    if (tid < MC) {
        float w = 0.f;
        if (tid < n) {
            const double last = run[(token0 + n - 1) * heads + head];
            w = expf((float)(last - run[(token0 + tid) * heads + head])) * coef[((token0 + tid) * heads + head) * 2 + 1];
        }
        s_w[tid] = w;
    }
    memory_stage_values(s_v, v, v_stride, token0, n, head, value_dim, column0, tid);
    const int mt = wave >> 1, nt = wave & 1;
    const int inner = (n + 15) & ~15;
    for (int slab = 0; slab < dim; slab += 64) {
        T keys[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int t = min(4 * j + (tid >> 6), n - 1), c = min(slab + (tid & 63), dim - 1);    // (neighbouring threads read neighbouring channels of one token)
            keys[j] = k[(token0 + t) * k_stride + (size_t)head * dim + c];
        }
        __syncthreads();                                 // s_w is there; the slab before has been read
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int t = 4 * j + (tid >> 6), c = tid & 63;
            s_k[c * MC_A + t] = (t < n && slab + c < dim) ? (float)keys[j] * s_w[t] : 0.f;
        }
        __syncthreads();
        if (slab + mt * 32 >= dim || column0 + nt * 32 > value_dim) continue;
        mc_f4 acc[2][2] = {};
        memory_product(acc, s_k + mt * 32 * MC_A, s_v + nt * 32, MC_B, 1, inner, lane);
        float* base = sums + (((size_t)blockIdx.x * heads + head) * dim) * ld;
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int channel = slab + mt * 32 + 16 * mi + 4 * (lane >> 4) + e, column = column0 + nt * 32 + 16 * ni + (lane & 15);
                    if (channel < dim && column <= value_dim) base[(size_t)channel * ld + column] = acc[mi][ni][e];
                }
    }
}

// (2) grid (rows, heads, blocks of 256 numbers of a head's dim x (value_dim + 1)); a thread walks one number of the state
// through the row's chunks.  The next chunk's sum is loaded before this chunk's place is overwritten.
__global__ __launch_bounds__(256) void memory_chunk_carry_kernel(float* __restrict__ sums, const double* __restrict__ run, float* state, long state_stride,
                                                                 const int* __restrict__ slots, const int* __restrict__ row_start,
                                                                 const int* __restrict__ row_len, const int* __restrict__ row_ctx,
                                                                 int heads, int dim, int value_dim) {
    const int row = blockIdx.x, head = blockIdx.y;
    const int count = row_len[row];
    if (count <= 0) return;
    const int ld = value_dim + 1;
    const long e = (long)blockIdx.z * 256 + threadIdx.x;
    if (e >= (long)dim * ld) return;
    const int channel = (int)(e / ld), column = (int)(e - (long)channel * ld);
    int base = 0;
    for (int r = 0; r < row; ++r) base += row_len[r] > 0 ? (row_len[r] + MC - 1) / MC : 0;
    const int chunks = (count + MC - 1) / MC, start = row_start[row];
    float* slot = state + (size_t)slots[row] * state_stride;
    float* mine = column < value_dim ? slot + ((size_t)head * dim + channel) * value_dim + column
                                     : slot + (size_t)heads * dim * value_dim + (size_t)head * dim + channel;
    float S = row_ctx[row] - count > 0 ? *mine : 0.f;
    const size_t step = (size_t)heads * dim * ld;
    float* place = sums + ((size_t)base * heads + head) * dim * ld + e;
    float sum = *place;
    for (int c = 0; c < chunks; ++c) {
        const float next = c + 1 < chunks ? place[step] : 0.f;
        const size_t last = (size_t)start + min(count, (c + 1) * MC) - 1;
        const float keep = expf((float)run[last * heads + head]);
        *place = S;
        S = __builtin_fmaf(keep, S, sum);
        sum = next;
        place += step;
    }
    *mine = S;
}

// (3) out[t][head][column] = sum_(j <= t) (q_t . k_j) e^(L_t - L_j) take_j value_j[column] + e^(L_t) sum_channel q_t[channel] S_0[channel][column],
// q scaled; the column behind the values goes to below[t][head][0].  grid and workgroup as in (1).
template <typename T>
__global__ __launch_bounds__(256) void memory_chunk_read_kernel(const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
                                                                const T* __restrict__ v, long v_stride, const float* __restrict__ coef,
                                                                const double* __restrict__ run, float q_scale,
                                                                const int* __restrict__ row_start, const int* __restrict__ row_len,
                                                                const int* __restrict__ row_ctx, int rows, const float* __restrict__ sums,
                                                                float* __restrict__ out, float* __restrict__ below, int heads, int dim, int value_dim) {
    __shared__ float s_q[MC * MC_A];                     // [token][channel]
    __shared__ float s_k[MC * MC_A];                     // [token][channel]; then the weighted scores [token t][token j]
    __shared__ float s_v[MC * MC_B];                     // [token or channel][column]
    __shared__ double s_run[MC];
    __shared__ float s_take[MC], s_decay[MC];            // take_j; e^(L_t)
    int row, chunk;
    if (!memory_item(blockIdx.x, rows, row_len, row, chunk)) return;
    const int head = blockIdx.y, column0 = blockIdx.z * 64, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int count = row_len[row];
    const int n = min(MC, count - chunk * MC);
    const size_t token0 = (size_t)row_start[row] + (size_t)chunk * MC;
    const int ld = value_dim + 1;
    const bool from_zero = chunk == 0 && row_ctx[row] - count == 0;      // nothing stands in front of the sequence's first chunk
    if (tid < MC) {
        s_run[tid] = tid < n ? run[(token0 + tid) * heads + head] : 0.0;
        s_take[tid] = tid < n ? coef[((token0 + tid) * heads + head) * 2 + 1] : 0.f;
        s_decay[tid] = expf((float)s_run[tid]);
    }
    const int mt = wave >> 1, nt = wave & 1;
    // the scores of the wavefront's 32 tokens t against 32 tokens j (nothing to do where every j lies behind every t)
    mc_f4 scores[2][2] = {};
    for (int slab = 0; slab < dim; slab += 64) {
        T queries[16], keys[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int t = min(4 * j + (tid >> 6), n - 1), c = min(slab + (tid & 63), dim - 1);
            queries[j] = q[(token0 + t) * q_stride + (size_t)head * dim + c];
            keys[j] = k[(token0 + t) * k_stride + (size_t)head * dim + c];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int t = 4 * j + (tid >> 6), c = tid & 63;
            const bool there = t < n && slab + c < dim;
            s_q[t * MC_A + c] = there ? (float)queries[j] * q_scale : 0.f;
            s_k[t * MC_A + c] = there ? (float)keys[j] : 0.f;
        }
        __syncthreads();
        if (nt <= mt) memory_product(scores, s_q + mt * 32 * MC_A, s_k + nt * 32 * MC_A, 1, MC_A, min(64, (dim - slab + 15) & ~15), lane);
    }
    __syncthreads();                                     // everybody has read the keys: their place takes the weighted scores
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int t = mt * 32 + 16 * mi + 4 * (lane >> 4) + e, j = nt * 32 + 16 * ni + (lane & 15);
                float weight = 0.f;
                if (j <= t && t < n) weight = expf((float)(s_run[t] - s_run[j])) * s_take[j];
                s_k[t * MC_A + j] = scores[mi][ni][e] * weight;
            }
    memory_stage_values(s_v, v, v_stride, token0, n, head, value_dim, column0, tid);
    __syncthreads();
    const bool wanted = column0 + nt * 32 <= value_dim;  // (uniform in a wavefront)
    mc_f4 acc[2][2] = {};
    if (wanted) memory_product(acc, s_k + mt * 32 * MC_A, s_v + nt * 32, MC_B, 1, (mt + 1) * 32, lane);
    if (!from_zero) {
        const float* before = sums + (((size_t)blockIdx.x * heads + head) * dim) * ld;
        for (int slab = 0; slab < dim; slab += 64) {
            T queries[16];
            float kept[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int t = 4 * j + (tid >> 6), c = tid & 63;          // queries [token][channel] times what the chunk's state has kept
                queries[j] = q[(token0 + min(t, n - 1)) * q_stride + (size_t)head * dim + min(slab + c, dim - 1)];
                const int channel = min(slab + t, dim - 1), column = min(column0 + c, value_dim);      // the state's slab [channel][column]
                kept[j] = before[(size_t)channel * ld + column];
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int t = 4 * j + (tid >> 6), c = tid & 63;
                s_q[t * MC_A + c] = (t < n && slab + c < dim) ? (float)queries[j] * q_scale * s_decay[t] : 0.f;
                s_v[t * MC_B + c] = (slab + t < dim && column0 + c <= value_dim) ? kept[j] : 0.f;
            }
            __syncthreads();
            if (wanted) memory_product(acc, s_q + mt * 32 * MC_A, s_v + nt * 32, MC_B, 1, min(64, (dim - slab + 15) & ~15), lane);
        }
    }
    if (!wanted) return;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int t = mt * 32 + 16 * mi + 4 * (lane >> 4) + e, column = column0 + nt * 32 + 16 * ni + (lane & 15);
                if (t >= n || column > value_dim) continue;
                if (column < value_dim) out[(token0 + t) * heads * value_dim + (size_t)head * value_dim + column] = acc[mi][ni][e];
                else below[((token0 + t) * heads + head) * 2] = acc[mi][ni][e];
            }
}

template <typename T>
__global__ __launch_bounds__(256) void tanh_kernel(T* __restrict__ x, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = (T)tanhf((float)x[i]);
}

template <typename T>
__global__ __launch_bounds__(256) void scaled_sum_kernel(const T* __restrict__ x, float a, const T* __restrict__ y, float b,
                                                         T* __restrict__ out, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (T)(a * (float)x[i] + b * (float)y[i]);
}

LSA_EXPORT int lsa_token_shift(int code, const void* h, const float* mu, int mixes, float* state, long state_stride, const int* slots,
                               const int* token_row, const int* positions, const int* row_start, void* out, int n_tokens, int width,
                               int keep, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (mixes < 1 || state == nullptr || slots == nullptr) return -1;
    const dim3 grid(n_tokens, (width + 255) / 256);
#define LSA_LAUNCH(T) token_shift_kernel<T><<<grid, 256, 0, stream>>>((const T*)h, mu, mixes, state, state_stride, slots, token_row, positions, \
        row_start, (T*)out, n_tokens, width, keep)
    if (code) LSA_LAUNCH(bf16_t); else LSA_LAUNCH(float);
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_token_shift_keep(int code, const void* h, float* state, long state_stride, const int* slots, const int* row_start,
                                    const int* row_len, int rows, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    dim3 grid(rows, (width + 255) / 256);
    if (code) token_shift_keep_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)h, state, state_stride, slots, row_start, row_len, width);
    else token_shift_keep_kernel<float><<<grid, 256, 0, stream>>>((const float*)h, state, state_stride, slots, row_start, row_len, width);
    LSA_LAUNCH_CHECK();
}

// Key channels a wavefront takes: 8 for heads of up to 64 channels, 16 up to 128, 32 up to 256, 64 up to 512: at most eight
// wavefronts a workgroup, and what the tokens' chunk and the wavefronts' partial read-outs take of LDS stays below 160 KB.
constexpr int MOST_DIM = 512;
constexpr int MOST_LDS = 160 * 1024;

LSA_EXPORT int lsa_linear_recurrence_most_dim() { return MOST_DIM; }

static size_t recurrence_lds(int dim, int& dk, int& waves) {
    dk = dim <= 64 ? 8 : dim <= 128 ? 16 : dim <= 256 ? 32 : 64;
    waves = (dim + dk - 1) / dk;
    return sizeof(float) * ((size_t)3 * CHUNK * waves * dk + (size_t)CHUNK * 64 + (size_t)waves * CHUNK * 64);
}

// Once, when the library has been loaded and before any launch: lets every form of the recurrence kernel ask for more
// dynamic LDS than the default limit.  (Not part of a launch: a launch may be recorded into a graph, and a stream
// that is being captured must see launches only.)
LSA_EXPORT int lsa_recurrent_prepare() {
    hipError_t first = hipSuccess;
#define LSA_ALLOW(T, DK, B) do { \
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&linear_recurrence_kernel<T, DK, B>), \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, MOST_LDS); \
        if (e != hipSuccess && first == hipSuccess) first = e; \
    } while (0)
#define LSA_ALLOW_ALL(T) do { LSA_ALLOW(T, 8, false); LSA_ALLOW(T, 8, true); LSA_ALLOW(T, 16, false); LSA_ALLOW(T, 16, true); \
                              LSA_ALLOW(T, 32, false); LSA_ALLOW(T, 32, true); LSA_ALLOW(T, 64, false); LSA_ALLOW(T, 64, true); } while (0)
    LSA_ALLOW_ALL(float);
    LSA_ALLOW_ALL(bf16_t);
#undef LSA_ALLOW_ALL
#undef LSA_ALLOW
#define LSA_ALLOW(T, DK) do { \
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&matrix_memory_kernel<T, DK>), \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, MOST_LDS); \
        if (e != hipSuccess && first == hipSuccess) first = e; \
    } while (0)
    LSA_ALLOW(float, 8); LSA_ALLOW(float, 16); LSA_ALLOW(float, 32); LSA_ALLOW(float, 64);
    LSA_ALLOW(bf16_t, 8); LSA_ALLOW(bf16_t, 16); LSA_ALLOW(bf16_t, 32); LSA_ALLOW(bf16_t, 64);
#undef LSA_ALLOW
    (void)hipGetLastError();
    return (int)first;
}

LSA_EXPORT int lsa_linear_recurrence(int code, const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                                     const float* decay, const float* decay_bias, int mode, float tau, const float* bonus, float q_scale,
                                     float* state, long state_stride, const int* slots, const int* row_start, const int* row_len,
                                     const int* row_ctx, float* out, int rows, int heads, int dim, int value_dim, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim < 1 || dim > MOST_DIM || value_dim < 1 || heads < 1 || (mode != 0 && mode != 1) || !(tau > 0.f) || state == nullptr) return -1;
    int dk, waves;
    const size_t lds = recurrence_lds(dim, dk, waves);
    if (lds > (size_t)MOST_LDS) return -1;
    dim3 grid(rows, heads, (value_dim + 63) / 64);
#define LSA_LAUNCH(T, DK, B) \
        linear_recurrence_kernel<T, DK, B><<<grid, waves * 64, lds, stream>>>((const T*)q, q_stride, (const T*)k, k_stride, (const T*)v, v_stride, \
            decay, decay_bias, mode, 1.f / tau, bonus, q_scale, state, state_stride, slots, row_start, row_len, row_ctx, out, heads, dim, value_dim)
#define LSA_BY_DK(T, B) do { if (dk == 8) LSA_LAUNCH(T, 8, B); else if (dk == 16) LSA_LAUNCH(T, 16, B); else if (dk == 32) LSA_LAUNCH(T, 32, B); \
                             else LSA_LAUNCH(T, 64, B); } while (0)
    if (code) { if (bonus) LSA_BY_DK(bf16_t, true); else LSA_BY_DK(bf16_t, false); }
    else { if (bonus) LSA_BY_DK(float, true); else LSA_BY_DK(float, false); }
#undef LSA_BY_DK
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_heads_norm_gate(int code, const float* x, const float* weight, int weight_per_channel, float eps, const void* gate,
                                   long gate_stride, void* out, int n_tokens, int heads, int value_dim, int gate_kind, const float* below,
                                   float floor, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (gate_kind != 0 && gate_kind != 1) return -1;
    dim3 grid(n_tokens, heads);
    const int weight_stride = weight_per_channel ? value_dim : 0;
    if (code) heads_norm_gate_kernel<bf16_t><<<grid, 64, 0, stream>>>(x, weight, weight_stride, eps, (const bf16_t*)gate, gate_stride, (bf16_t*)out, heads, value_dim, gate_kind, below, floor);
    else heads_norm_gate_kernel<float><<<grid, 64, 0, stream>>>(x, weight, weight_stride, eps, (const float*)gate, gate_stride, (float*)out, heads, value_dim, gate_kind, below, floor);
    LSA_LAUNCH_CHECK();
}

// state[slot]: the matrices [heads][dim][value_dim], the normalisers [heads][dim], the maxima [heads].
LSA_EXPORT int lsa_matrix_memory(int code, const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                                 const float* gates, float cap, float q_scale, float* state, long state_stride, const int* slots,
                                 const int* row_start, const int* row_len, const int* row_ctx, float* coef, float* out, float* below,
                                 int rows, int heads, int dim, int value_dim, double* run, float* sums, int items, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim < 1 || dim > MOST_DIM || value_dim < 1 || heads < 1 || !(cap > 0.f) || state == nullptr || coef == nullptr || below == nullptr) return -1;
    if (state_stride < (long)heads * dim * value_dim + (long)heads * dim + heads) return -1;
    int dk, waves;
    recurrence_lds(dim, dk, waves);
    const size_t lds = sizeof(float) * ((size_t)2 * CHUNK * waves * dk + (size_t)CHUNK * 64 + CHUNK + (size_t)waves * CHUNK * 64);
    if (lds > (size_t)MOST_LDS) return -1;
    memory_gates_kernel<<<dim3(rows, heads), 64 * GATES_WAVES, 0, stream>>>(gates, cap, state, state_stride, (long)heads * dim * value_dim + (long)heads * dim,
                                                              slots, row_start, row_len, row_ctx, coef, below, heads, run);
    if (run != nullptr) {
        // in chunks: run [T][heads] and sums [items][heads][dim][value_dim + 1] are the caller's scratch memory; items is no
        // less than the number of chunks of 64 tokens that the rows have together
        if (sums == nullptr || items <= 0) return -1;
        const dim3 chunk_grid(items, heads, (value_dim + 1 + 63) / 64);
        const dim3 carry_grid(rows, heads, (unsigned)(((long)dim * (value_dim + 1) + 255) / 256));
#define LSA_CHUNKED(T) do { \
            memory_chunk_sums_kernel<T><<<chunk_grid, 256, 0, stream>>>((const T*)k, k_stride, (const T*)v, v_stride, coef, run, row_start, row_len, rows, \
                                                                        sums, heads, dim, value_dim); \
            memory_chunk_carry_kernel<<<carry_grid, 256, 0, stream>>>(sums, run, state, state_stride, slots, row_start, row_len, row_ctx, heads, dim, value_dim); \
            memory_chunk_read_kernel<T><<<chunk_grid, 256, 0, stream>>>((const T*)q, q_stride, (const T*)k, k_stride, (const T*)v, v_stride, coef, run, q_scale, \
                                                                        row_start, row_len, row_ctx, rows, sums, out, below, heads, dim, value_dim); \
        } while (0)
        if (code) LSA_CHUNKED(bf16_t); else LSA_CHUNKED(float);
#undef LSA_CHUNKED
        LSA_LAUNCH_CHECK();
    }
    dim3 grid(rows, heads, (value_dim + 1 + 63) / 64);
#define LSA_LAUNCH(T, DK) \
        matrix_memory_kernel<T, DK><<<grid, waves * 64, lds, stream>>>((const T*)q, q_stride, (const T*)k, k_stride, (const T*)v, v_stride, \
            coef, q_scale, state, state_stride, slots, row_start, row_len, row_ctx, out, below, heads, dim, value_dim)
#define LSA_BY_DK(T) do { if (dk == 8) LSA_LAUNCH(T, 8); else if (dk == 16) LSA_LAUNCH(T, 16); else if (dk == 32) LSA_LAUNCH(T, 32); \
                          else LSA_LAUNCH(T, 64); } while (0)
    if (code) LSA_BY_DK(bf16_t); else LSA_BY_DK(float);
#undef LSA_BY_DK
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_tanh(int code, void* x, long n, hipStream_t stream) {
    if (n <= 0) return 0;
    const int blocks = (int)((n + 255) / 256);
    if (code) tanh_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, n);
    else tanh_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, n);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_scaled_sum(int code, const void* x, float a, const void* y, float b, void* out, long n, hipStream_t stream) {
    if (n <= 0) return 0;
    const int blocks = (int)((n + 255) / 256);
    if (code) scaled_sum_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)x, a, (const bf16_t*)y, b, (bf16_t*)out, n);
    else scaled_sum_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, a, (const float*)y, b, (float*)out, n);
    LSA_LAUNCH_CHECK();
}
