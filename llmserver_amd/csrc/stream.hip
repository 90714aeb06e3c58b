// Row-wise kernels around a residual stream that is kept in float32 whatever the type of the activations:
// embedding lookup with the norm behind it, a norm of chosen rows, a short causal convolution over time with a
// per-request state, the update behind a sublayer (norm of the sublayer's result, per-channel scale, sum, and
// the weighted sum over the results of the layers so far), and several such streams side by side that sublayers read
// as a weighted sum and update all at once.  One workgroup per token row; sums of squares, rsqrt and
// every sum are 32-bit; a result for a 16-bit consumer is rounded once when it is stored.
#include "common.hpp"

using namespace lsa;

template <typename T>
__device__ inline float row_square_sum(const T* __restrict__ row, int width, float* scratch) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = (float)row[i];
        sq += v * v;
    }
    return block_sum(sq, scratch);
}

// out[t] = table[ids[t]] * rsqrt(mean(.^2) + eps) * weight.  An id outside the table gives a zero row (the host
// refuses such ids before the launch).
template <typename T>
__global__ __launch_bounds__(256) void embedding_norm_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                                             const float* __restrict__ weight, float eps, float* __restrict__ out,
                                                             int width, int vocab) {
    __shared__ float scratch[16];
    const int id = ids[blockIdx.x];
    const bool ok = id >= 0 && id < vocab;
    const T* row = table + (size_t)(ok ? id : 0) * width;
    const float sq = row_square_sum(row, width, scratch);
    const float inv = ok ? rsqrtf(sq / (float)width + eps) : 0.f;
    float* o = out + (size_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = (float)row[i] * inv * weight[i];
}

// out[i] = x[rows[i]] * rsqrt(mean(.^2) + eps) * weight (rows == nullptr: every row).
template <typename O>
__global__ __launch_bounds__(256) void norm_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                                        const float* __restrict__ weight, float eps, O* __restrict__ out, int width) {
    __shared__ float scratch[16];
    const float* row = x + (size_t)(rows ? rows[blockIdx.x] : blockIdx.x) * width;
    const float inv = rsqrtf(row_square_sum(row, width, scratch) / (float)width + eps);
    O* o = out + (size_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = (O)(row[i] * inv * weight[i]);
}

// out[t] = x[t] + sum_j w[:, j] * h(position - (taps - 1 - j)), where h(p) is the input at position p of the token's
// request: a row of this step if the step brings position p, the request's state otherwise (state[slot][k] is the
// input at position first - kept + k, `first` the position of the step's first token of the request, kept = taps - 1),
// zero before the sequence starts.
template <typename O, int V>
__global__ __launch_bounds__(256) void short_conv_kernel(const float* __restrict__ x, const float* __restrict__ w, int taps,
                                                         float* state, const int* __restrict__ slots,
                                                         const int* __restrict__ token_row, const int* __restrict__ positions,
                                                         const int* __restrict__ row_start, O* __restrict__ out, int width, int keep) {
    // V (1 or 4) neighbouring channels a thread: the rows it reads are 16-byte pieces where the width allows.
    // keep (only in steps in which every row brings one token, so that a row's state is one workgroup's): the state
    // moves on by this token here, in the thread that has just read its channels, instead of in a launch of its own.
    const int t = blockIdx.x;
    const int row = token_row[t], position = positions[t];
    const int first = position - (t - row_start[row]);
    const int kept = taps - 1;
    float* mine = state ? state + (size_t)slots[row] * kept * width : nullptr;
    for (int c = threadIdx.x * V; c < width; c += blockDim.x * V) {
        float acc[V], own[V];
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = own[v] = x[(size_t)t * width + c + v];
        for (int j = 0; j < taps; ++j) {
            const int back = kept - j, place = position - back;
            if (place < 0) continue;
            const float* src;
            if (place >= first) src = x + (size_t)(t - back) * width + c;
            else if (mine) src = mine + (size_t)(kept - (first - place)) * width + c;
            else continue;
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] += w[(size_t)(c + v) * taps + j] * src[v];
        }
#pragma unroll
        for (int v = 0; v < V; ++v) out[(size_t)t * width + c + v] = (O)acc[v];
        if (keep && mine) {
            for (int k = 0; k + 1 < kept; ++k)
#pragma unroll
                for (int v = 0; v < V; ++v) mine[(size_t)k * width + c + v] = mine[(size_t)(k + 1) * width + c + v];
#pragma unroll
            for (int v = 0; v < V; ++v) mine[(size_t)(kept - 1) * width + c + v] = own[v];
        }
    }
}

// After the step: state[slot][k] = input at position end - kept + k, from the step's rows where it brought that
// position, from the old state where it did not (k + count then indexes it), zero before the sequence.  A thread
// owns a channel of a row and goes through k upwards, so what it still has to read lies above what it has written.
__global__ __launch_bounds__(256) void short_conv_keep_kernel(const float* __restrict__ x, float* __restrict__ state,
                                                              const int* __restrict__ slots, const int* __restrict__ row_start,
                                                              const int* __restrict__ row_len, const int* __restrict__ row_ctx,
                                                              int kept, int width) {
    const int row = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int count = row_len[row], end = row_ctx[row], start = row_start[row];
    if (count <= 0) return;
    const int first = end - count;
    float* mine = state + (size_t)slots[row] * kept * width;
    for (int k = 0; k < kept; ++k) {
        const int place = end - kept + k;
        float v = 0.f;
        if (place >= first) v = x[(size_t)(start + place - first) * width + c];
        else if (place >= 0) v = mine[(size_t)(k + count) * width + c];
        mine[(size_t)k * width + c] = v;
    }
}

// s = x + y * rsqrt(mean(y^2) + eps) * weight * scale.  Without history: out = s.  With history [states][T][W]:
// history[before] = s and out = sum_{j <= before} mix[j] * history[j].  `rounded` (may be null) gets out as well.
template <typename Y, typename R, int V>
__global__ __launch_bounds__(256) void scaled_norm_add_kernel(const float* __restrict__ x, const Y* __restrict__ y,
                                                              const float* __restrict__ weight, const float* __restrict__ scale, float eps,
                                                              float* __restrict__ out, R* __restrict__ rounded, float* history,
                                                              size_t state_stride, int before, const float* __restrict__ mix, int width) {
    // V (1 or 4) neighbouring elements a thread; the first CACHE pieces of y stay in registers between the two passes.
    constexpr int CACHE = 4;
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * width;
    const Y* yr = y + base;
    const int stride = blockDim.x * V;
    float kept[CACHE][V];
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = threadIdx.x * V + k * stride;
        if (i < width) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                kept[k][v] = (float)yr[i + v];
                sq += kept[k][v] * kept[k][v];
            }
        }
    }
    for (int i = threadIdx.x * V + CACHE * stride; i < width; i += stride)
#pragma unroll
        for (int v = 0; v < V; ++v) sq += (float)yr[i + v] * (float)yr[i + v];
    const float inv = rsqrtf(block_sum(sq, scratch) / (float)width + eps);
    auto finish = [&](int i, const float (&yv)[V]) {
        float s[V], total[V];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            s[v] = x[base + i + v] + yv[v] * inv * weight[i + v] * (scale ? scale[i + v] : 1.f);
            total[v] = 0.f;
        }
        if (history) {
            for (int j = 0; j < before; ++j) {
                const float m = mix[j];
                const float* h = history + (size_t)j * state_stride + base + i;
#pragma unroll
                for (int v = 0; v < V; ++v) total[v] += m * h[v];
            }
            const float m = mix[before];
#pragma unroll
            for (int v = 0; v < V; ++v) {
                history[(size_t)before * state_stride + base + i + v] = s[v];
                s[v] = total[v] + m * s[v];
            }
        }
#pragma unroll
        for (int v = 0; v < V; ++v) {
            out[base + i + v] = s[v];
            if (rounded) rounded[base + i + v] = (R)s[v];
        }
    };
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = threadIdx.x * V + k * stride;
        if (i < width) finish(i, kept[k]);
    }
    for (int i = threadIdx.x * V + CACHE * stride; i < width; i += stride) {
        float yv[V];
#pragma unroll
        for (int v = 0; v < V; ++v) yv[v] = (float)yr[i + v];
        finish(i, yv);
    }
}

// out[c][t] = table[ids[t]] * scale, widened to float32, for each of `copies` equal copies (several residual streams start
// alike); an id outside the table gives a zero row.
template <typename T>
__global__ __launch_bounds__(256) void embedding_wide_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                                             float* __restrict__ out, int width, int vocab, float scale, int copies,
                                                             size_t copy_stride) {
    const int id = ids[blockIdx.x];
    const bool ok = id >= 0 && id < vocab;
    const T* row = table + (size_t)(ok ? id : 0) * width;
    float* o = out + (size_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float value = ok ? (float)row[i] * scale : 0.f;
        for (int c = 0; c < copies; ++c) o[(size_t)c * copy_stride + i] = value;
    }
}

// ---- several residual streams x [S][T][W], float32 ------------------------------------------------------------------------
constexpr int MOST_STREAMS = 8;
constexpr int STREAM_CACHE = 8;           // elements of a row a thread keeps between the two passes (rows of up to 2,048 are read once; sixteen gained nothing at 4,096 and cost a prompt a little)

// The kernels below take the number of streams as a template parameter: the small per-stream arrays then live in registers
// (indexed by a run-time count they would go to scratch memory, and a row of one token would wait for that).
// out[i] = rmsnorm(sum_s read[s] * x[s][rows[i]]) * weight (rows == nullptr: every row).
template <typename O, int S>
__global__ __launch_bounds__(256) void streams_read_kernel(const float* __restrict__ x, size_t stream_stride,
                                                           const float* __restrict__ read, const int* __restrict__ rows,
                                                           const float* __restrict__ weight, float eps, O* __restrict__ out, int width) {
    __shared__ float scratch[16];
    const float* row = x + (size_t)(rows ? rows[blockIdx.x] : blockIdx.x) * width;
    float r[S];
#pragma unroll
    for (int s = 0; s < S; ++s) r[s] = read[s];
    auto summed = [&](int i) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < S; ++s) u += r[s] * row[(size_t)s * stream_stride + i];
        return u;
    };
    float kept[STREAM_CACHE], weights[STREAM_CACHE];
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < STREAM_CACHE; ++k) {
        const int i = threadIdx.x + k * 256;
        const float u = summed(min(i, width - 1));       // (a load of a place that is there stands under no condition)
        weights[k] = weight[min(i, width - 1)];          // (asked for now: behind the sum of squares nothing waits for memory)
        kept[k] = i < width ? u : 0.f;
        sq += kept[k] * kept[k];
    }
    for (int i = threadIdx.x + STREAM_CACHE * 256; i < width; i += 256) {
        const float u = summed(i);
        sq += u * u;
    }
    const float inv = rsqrtf(block_sum(sq, scratch) / (float)width + eps);
    O* o = out + (size_t)blockIdx.x * width;
#pragma unroll
    for (int k = 0; k < STREAM_CACHE; ++k) {
        const int i = threadIdx.x + k * 256;
        if (i < width) o[i] = (O)(kept[k] * inv * weights[k]);
    }
    for (int i = threadIdx.x + STREAM_CACHE * 256; i < width; i += 256) o[i] = (O)(summed(i) * inv * weight[i]);
}

// Every new stream from the streams as they stood before the update, stored where they lie: x[t] <- sum_s mix[s][t] * x[s] + write[t] * y, and, where next_read
// is given, normed = rmsnorm(sum_t next_read[t] * x[t]) * next_weight: what the next sublayer reads, in the same pass (the
// row of sums stays in registers between the two passes; wider rows are formed again from the streams just written, by the
// thread that wrote them).  One workgroup a token row.
template <typename Y, typename R, int S>
__global__ __launch_bounds__(256) void streams_update_kernel(float* __restrict__ x, size_t stream_stride, const Y* __restrict__ y,
                                                             const float* __restrict__ mix, const float* __restrict__ write,
                                                             const float* __restrict__ next_read, const float* __restrict__ next_weight,
                                                             float next_eps, R* __restrict__ normed, int width) {
    __shared__ float scratch[16];
    float m[S][S], w[S], r[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int t = 0; t < S; ++t) m[s][t] = mix[s * S + t];
        w[s] = write[s];
        r[s] = next_read ? next_read[s] : 0.f;
    }
    float* row = x + (size_t)blockIdx.x * width;
    const Y* yr = y + (size_t)blockIdx.x * width;
    // one column of all streams: the new streams are written, what the next sublayer reads of them is returned
    auto updated = [&](int i) {
        float old[S];
#pragma unroll
        for (int s = 0; s < S; ++s) old[s] = row[(size_t)s * stream_stride + i];
        const float update = (float)yr[i];
        float u = 0.f;
#pragma unroll
        for (int t = 0; t < S; ++t) {
            float fresh = 0.f;
#pragma unroll
            for (int s = 0; s < S; ++s) fresh += m[s][t] * old[s];
            fresh += w[t] * update;
            row[(size_t)t * stream_stride + i] = fresh;
            u += r[t] * fresh;
        }
        return u;
    };
    // the first STREAM_CACHE columns of a thread: every load is issued before the first store (a store to the streams would
    // otherwise hold back the loads behind it, and a row of one token would wait for memory once a column), and every load
    // is of a place that is there, so that none stands under a condition
    float kept[STREAM_CACHE], olds[STREAM_CACHE][S], updates[STREAM_CACHE], weights[STREAM_CACHE];
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < STREAM_CACHE; ++k) {
        const int i = min((int)threadIdx.x + k * 256, width - 1);
#pragma unroll
        for (int s = 0; s < S; ++s) olds[k][s] = row[(size_t)s * stream_stride + i];
        updates[k] = (float)yr[i];
        weights[k] = next_read ? next_weight[i] : 0.f;    // (asked for now: behind the sum of squares nothing waits for memory)
    }
#pragma unroll
    for (int k = 0; k < STREAM_CACHE; ++k) {
        const int i = threadIdx.x + k * 256;
        float u = 0.f;
        if (i < width) {
#pragma unroll
            for (int t = 0; t < S; ++t) {
                float fresh = 0.f;
#pragma unroll
                for (int s = 0; s < S; ++s) fresh += m[s][t] * olds[k][s];
                fresh += w[t] * updates[k];
                row[(size_t)t * stream_stride + i] = fresh;
                u += r[t] * fresh;
            }
        }
        kept[k] = u;
        sq += u * u;
    }
    for (int i = threadIdx.x + STREAM_CACHE * 256; i < width; i += 256) {
        const float u = updated(i);
        sq += u * u;
    }
    if (!next_read) return;                              // (the whole workgroup)
    const float inv = rsqrtf(block_sum(sq, scratch) / (float)width + next_eps);
    R* o = normed + (size_t)blockIdx.x * width;
#pragma unroll
    for (int k = 0; k < STREAM_CACHE; ++k) {
        const int i = threadIdx.x + k * 256;
        if (i < width) o[i] = (R)(kept[k] * inv * weights[k]);
    }
    for (int i = threadIdx.x + STREAM_CACHE * 256; i < width; i += 256) {
        float u = 0.f;
#pragma unroll
        for (int t = 0; t < S; ++t) u += r[t] * row[(size_t)t * stream_stride + i];
        o[i] = (R)(u * inv * next_weight[i]);
    }
}

// s = x + u * rsqrt(mean(u^2) + eps) * weight with u = y, or a * y + b * y2 where y2 is given; out = s; and where
// next_weight is given, normed = s * rsqrt(mean(s^2) + next_eps) * next_weight: the norm behind a sublayer, the sum with
// the stream and the norm in front of the next sublayer in one pass (the row stays in registers between the two sums
// of squares; rows wider than 256 * V * CACHE elements are read again).
template <typename Y, typename R, int V>
__global__ __launch_bounds__(256) void norm_add_norm_kernel(const float* __restrict__ x, const Y* __restrict__ y, const Y* __restrict__ y2,
                                                            float a, float b, const float* __restrict__ weight, float eps,
                                                            float* __restrict__ out, const float* __restrict__ next_weight, float next_eps,
                                                            R* __restrict__ normed, int width) {
    constexpr int CACHE = 4;
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * width;
    const int stride = blockDim.x * V;
    auto update = [&](int i, float (&u)[V]) {
#pragma unroll
        for (int v = 0; v < V; ++v) u[v] = y2 ? a * (float)y[base + i + v] + b * (float)y2[base + i + v] : (float)y[base + i + v];
    };
    float kept[CACHE][V];
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = threadIdx.x * V + k * stride;
        if (i < width) {
            update(i, kept[k]);
#pragma unroll
            for (int v = 0; v < V; ++v) sq += kept[k][v] * kept[k][v];
        }
    }
    for (int i = threadIdx.x * V + CACHE * stride; i < width; i += stride) {
        float u[V];
        update(i, u);
#pragma unroll
        for (int v = 0; v < V; ++v) sq += u[v] * u[v];
    }
    const float inv = rsqrtf(block_sum(sq, scratch) / (float)width + eps);
    float sq2 = 0.f;
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = threadIdx.x * V + k * stride;
        if (i < width) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const float s = x[base + i + v] + kept[k][v] * inv * weight[i + v];
                kept[k][v] = s;
                out[base + i + v] = s;
                sq2 += s * s;
            }
        }
    }
    for (int i = threadIdx.x * V + CACHE * stride; i < width; i += stride) {
        float u[V];
        update(i, u);
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float s = x[base + i + v] + u[v] * inv * weight[i + v];
            out[base + i + v] = s;
            sq2 += s * s;
        }
    }
    if (!next_weight) return;
    const float inv2 = rsqrtf(block_sum(sq2, scratch) / (float)width + next_eps);
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = threadIdx.x * V + k * stride;
        if (i < width) {
#pragma unroll
            for (int v = 0; v < V; ++v) normed[base + i + v] = (R)(kept[k][v] * inv2 * next_weight[i + v]);
        }
    }
    for (int i = threadIdx.x * V + CACHE * stride; i < width; i += stride)         // (its own writes of a moment ago)
#pragma unroll
        for (int v = 0; v < V; ++v) normed[base + i + v] = (R)(out[base + i + v] * inv2 * next_weight[i + v]);
}

LSA_EXPORT int lsa_embedding_wide(int table_code, const void* table, const int* ids, float* out, int n, int width, int vocab,
                                  float scale, int copies, hipStream_t stream) {
    if (n <= 0) return 0;
    if (copies < 1) return -1;
    const size_t copy_stride = (size_t)n * width;
    if (table_code) embedding_wide_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)table, ids, out, width, vocab, scale, copies, copy_stride);
    else embedding_wide_kernel<float><<<n, 256, 0, stream>>>((const float*)table, ids, out, width, vocab, scale, copies, copy_stride);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_most_streams() { return MOST_STREAMS; }

// x [streams][n_tokens][width]; out [n_out][width].
LSA_EXPORT int lsa_streams_read(const float* x, int streams, int n_tokens, const float* read, const int* rows, const float* weight, float eps,
                                void* out, int out_code, int n_out, int width, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (streams < 1 || streams > MOST_STREAMS) return -1;
    const size_t stream_stride = (size_t)n_tokens * width;
#define LSA_LAUNCH(O, S) streams_read_kernel<O, S><<<n_out, 256, 0, stream>>>(x, stream_stride, read, rows, weight, eps, (O*)out, width)
#define LSA_BY_STREAMS(O) switch (streams) { case 1: LSA_LAUNCH(O, 1); break; case 2: LSA_LAUNCH(O, 2); break; case 3: LSA_LAUNCH(O, 3); break; \
        case 4: LSA_LAUNCH(O, 4); break; case 5: LSA_LAUNCH(O, 5); break; case 6: LSA_LAUNCH(O, 6); break; case 7: LSA_LAUNCH(O, 7); break; \
        default: LSA_LAUNCH(O, 8); }
    if (out_code) LSA_BY_STREAMS(bf16_t) else LSA_BY_STREAMS(float)
#undef LSA_BY_STREAMS
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_streams_update(float* x, int streams, int n_tokens, const void* y, int y_code, const float* mix, const float* write,
                                  const float* next_read, const float* next_weight, float next_eps, void* normed, int normed_code, int width,
                                  hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (streams < 1 || streams > MOST_STREAMS || (next_read != nullptr && (normed == nullptr || next_weight == nullptr))) return -1;
    const size_t stream_stride = (size_t)n_tokens * width;
#define LSA_LAUNCH_S(Y, R, S) streams_update_kernel<Y, R, S><<<n_tokens, 256, 0, stream>>>(x, stream_stride, (const Y*)y, mix, write, next_read, \
                                                                                          next_weight, next_eps, (R*)normed, width)
#define LSA_LAUNCH(Y, R) switch (streams) { case 1: LSA_LAUNCH_S(Y, R, 1); break; case 2: LSA_LAUNCH_S(Y, R, 2); break; case 3: LSA_LAUNCH_S(Y, R, 3); break; \
        case 4: LSA_LAUNCH_S(Y, R, 4); break; case 5: LSA_LAUNCH_S(Y, R, 5); break; case 6: LSA_LAUNCH_S(Y, R, 6); break; \
        case 7: LSA_LAUNCH_S(Y, R, 7); break; default: LSA_LAUNCH_S(Y, R, 8); }
    if (y_code && normed_code) LSA_LAUNCH(bf16_t, bf16_t)
    else if (y_code) LSA_LAUNCH(bf16_t, float)
    else if (normed_code) LSA_LAUNCH(float, bf16_t)
    else LSA_LAUNCH(float, float)
#undef LSA_LAUNCH
#undef LSA_LAUNCH_S
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_norm_add_norm(const float* x, const void* y, const void* y2, int y_code, float a, float b, const float* weight, float eps,
                                 float* out, const float* next_weight, float next_eps, void* normed, int normed_code, int n, int width,
                                 hipStream_t stream) {
    if (n <= 0) return 0;
    if (next_weight != nullptr && normed == nullptr) return -1;
#define LSA_LAUNCH_V(Y, R, V) norm_add_norm_kernel<Y, R, V><<<n, 256, 0, stream>>>(x, (const Y*)y, (const Y*)y2, a, b, weight, eps, out, next_weight, \
                                                                                next_eps, (R*)normed, width)
#define LSA_LAUNCH(Y, R) do { if (width % 4 == 0) LSA_LAUNCH_V(Y, R, 4); else LSA_LAUNCH_V(Y, R, 1); } while (0)
    if (y_code && normed_code) LSA_LAUNCH(bf16_t, bf16_t);
    else if (y_code) LSA_LAUNCH(bf16_t, float);
    else if (normed_code) LSA_LAUNCH(float, bf16_t);
    else LSA_LAUNCH(float, float);
#undef LSA_LAUNCH
#undef LSA_LAUNCH_V
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_embedding_norm(int table_code, const void* table, const int* ids, const float* weight, float eps, float* out,
                                  int n, int width, int vocab, hipStream_t stream) {
    if (n <= 0) return 0;
    if (table_code) embedding_norm_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)table, ids, weight, eps, out, width, vocab);
    else embedding_norm_kernel<float><<<n, 256, 0, stream>>>((const float*)table, ids, weight, eps, out, width, vocab);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_norm_rows(const float* x, const int* rows, const float* weight, float eps, void* out, int out_code, int n_out,
                             int width, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (out_code) norm_rows_kernel<bf16_t><<<n_out, 256, 0, stream>>>(x, rows, weight, eps, (bf16_t*)out, width);
    else norm_rows_kernel<float><<<n_out, 256, 0, stream>>>(x, rows, weight, eps, (float*)out, width);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_short_conv(const float* x, const float* w, int taps, float* state, const int* slots, const int* token_row,
                              const int* positions, const int* row_start, void* out, int out_code, int n, int width, int keep,
                              hipStream_t stream) {
    if (n <= 0) return 0;
    if (taps < 1 || (taps > 1 && (state == nullptr || slots == nullptr))) return -1;
#define LSA_LAUNCH(O, V) short_conv_kernel<O, V><<<n, 256, 0, stream>>>(x, w, taps, state, slots, token_row, positions, row_start, (O*)out, width, keep)
    if (width % 4 == 0) { if (out_code) LSA_LAUNCH(bf16_t, 4); else LSA_LAUNCH(float, 4); }
    else { if (out_code) LSA_LAUNCH(bf16_t, 1); else LSA_LAUNCH(float, 1); }
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_short_conv_keep(const float* x, float* state, const int* slots, const int* row_start, const int* row_len,
                                   const int* row_ctx, int kept, int rows, int width, hipStream_t stream) {
    if (rows <= 0 || kept <= 0) return 0;
    short_conv_keep_kernel<<<dim3(rows, (width + 255) / 256), 256, 0, stream>>>(x, state, slots, row_start, row_len, row_ctx, kept, width);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_scaled_norm_add(const float* x, const void* y, int y_code, const float* weight, const float* scale, float eps,
                                   float* out, void* rounded, int rounded_code, float* history, long state_stride, int before,
                                   const float* mix, int n, int width, hipStream_t stream) {
    if (n <= 0) return 0;
    if (history != nullptr && (mix == nullptr || before < 0)) return -1;
#define LSA_LAUNCH_V(Y, R, V) scaled_norm_add_kernel<Y, R, V><<<n, 256, 0, stream>>>(x, (const Y*)y, weight, scale, eps, out, (R*)rounded, history, \
                                                                                  (size_t)state_stride, before, mix, width)
#define LSA_LAUNCH(Y, R) do { if (width % 4 == 0) LSA_LAUNCH_V(Y, R, 4); else LSA_LAUNCH_V(Y, R, 1); } while (0)
    if (y_code && rounded_code) LSA_LAUNCH(bf16_t, bf16_t);
    else if (y_code) LSA_LAUNCH(bf16_t, float);
    else if (rounded_code) LSA_LAUNCH(float, bf16_t);
    else LSA_LAUNCH(float, float);
#undef LSA_LAUNCH
#undef LSA_LAUNCH_V
    LSA_LAUNCH_CHECK();
}
