// Around attention over a shared low-rank latent: one row [latent, rotated key part, zeros] per token is the token's
// key and, transposed, its value in a paged cache with one key-value head; a query head's row is
// [its query mapped into the latent, its rotated part, zeros].  Rotation turns neighbouring dimensions (2i, 2i+1)
// together by the token's angle i; norm, rotation and sigmoid are 32-bit, every result is rounded once.
#include "common.hpp"

using namespace lsa;

// The rotated value of element e of a vector whose first 2 * pairs elements turn; cs = the token's [cos.., sin..].
template <typename T>
__device__ inline float turned(const T* __restrict__ v, int e, const float* __restrict__ cs, int pairs) {
    const int pair = e >> 1;
    if (pair >= pairs) return (float)v[e];
    const float u = (float)v[2 * pair], w = (float)v[2 * pair + 1], c = cs[pair], s = cs[pairs + pair];
    return (e & 1) ? w * c + u * s : u * c - w * s;
}

// grid (tokens, heads + 1, pieces of 64 of a row).  proj row: heads x [dim plain, rot_dim rotated] query dimensions, then
// the token's `rank` latent dimensions and its rot_dim rotated key dimensions.  Workgroups (t, h < heads, piece) assemble
// head h's query row [U_h^T q_h, rotate(p_h), zeros], 64 elements each; the first part comes from `q_latent`
// [heads][tokens][rank] (a batched product made before) or, where `up_keys` [heads][dim][rank] is given (steps of few tokens,
// where that product would be a launch of its own for a few thousand multiplications), is multiplied here: a lane owns an
// element, the workgroup's wavefronts share the rows of the matrix between them and add their sums up in LDS.
// Workgroup (t, heads, 0) writes the token's cache row.
template <typename T>
__global__ void latent_prepare_kernel(
    const T* __restrict__ proj, long proj_stride, const T* __restrict__ q_latent, const T* __restrict__ up_keys,
    const float* __restrict__ norm_weight, float eps,
    const float* __restrict__ cos_sin, int pairs, T* __restrict__ keys, T* __restrict__ values, const int* __restrict__ table,
    int table_stride, const int* __restrict__ token_row, const int* __restrict__ positions, int page_size, T* __restrict__ out_q,
    int heads, int dim, int rot_dim, int rank, int row_width, int write_cache, int n_tokens) {
    __shared__ float scratch[16];
    __shared__ float partial[4][64];
    const int t = blockIdx.x, head = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const T* mine = proj + (size_t)t * proj_stride;
    const float* cs = cos_sin + (size_t)t * 2 * pairs;
    const int per_head = dim + rot_dim;
    if (head < heads) {
        const T* qh = mine + head * per_head;
        if (!up_keys) {                 // nothing to multiply: one workgroup assembles the whole row
            for (int e = threadIdx.x; e < row_width; e += blockDim.x) {
                float v = 0.f;
                if (e < rank) v = (float)q_latent[((size_t)head * n_tokens + t) * rank + e];
                else if (e < rank + rot_dim) v = turned(qh + dim, e - rank, cs, pairs);
                out_q[((size_t)t * heads + head) * row_width + e] = (T)v;
            }
            return;
        }
        const int e = blockIdx.z * 64 + lane;
        float v = 0.f;
        if (e < rank) {
            const int share = (dim + waves - 1) / waves, d0 = wave * share, d1 = min(dim, d0 + share);
            const T* u = up_keys + (size_t)head * dim * rank + e;
            int d = d0;
            for (; d + 8 <= d1; d += 8) {                   // eight rows of the matrix under way at a time
                float w[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) w[k] = (float)u[(size_t)(d + k) * rank];
#pragma unroll
                for (int k = 0; k < 8; ++k) v += (float)qh[d + k] * w[k];
            }
            for (; d < d1; ++d) v += (float)qh[d] * (float)u[(size_t)d * rank];
        }
        partial[wave][lane] = v;
        __syncthreads();
        if (wave) return;
        v = 0.f;
        for (int w = 0; w < waves; ++w) v += partial[w][lane];
        if (e >= row_width) return;
        if (e >= rank) v = e < rank + rot_dim ? turned(qh + dim, e - rank, cs, pairs) : 0.f;
        out_q[((size_t)t * heads + head) * row_width + e] = (T)v;
        return;
    }
    if (!write_cache || blockIdx.z) return;
    const T* down = mine + (size_t)heads * per_head;
    float sq = 0.f;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) {
        const float v = (float)down[i];
        sq += v * v;
    }
    const float inv = rsqrtf(block_sum(sq, scratch) / (float)rank + eps);
    const int position = positions[t];
    const int page = table[(size_t)token_row[t] * table_stride + position / page_size], slot = position % page_size;
    if (page < 0) return;
    T* key = keys + ((size_t)page * page_size + slot) * row_width;
    T* value = values + (size_t)page * row_width * page_size + slot;
    for (int e = threadIdx.x; e < row_width; e += blockDim.x) {
        float v = 0.f;
        if (e < rank) v = (float)down[e] * inv * norm_weight[e];
        else if (e < rank + rot_dim) v = turned(down + rank, e - rank, cs, pairs);
        key[e] = (T)v;
        value[(size_t)e * page_size] = (T)v;
    }
}

// grid (tokens, heads, pieces of 64 of a head's values): out[t][h * v + j] = y_h[t][j] * sigmoid(proj[t][gate_column + h])
// (gate_column < 0: no gate), where y_h[t] comes from `y` [heads][tokens][v] (a batched product made before) or, where
// `up_values` [heads][rank][v] is given, is the head's weighted latent sum `mixed[t][h][0 .. rank)` (rows of row_width) times
// that matrix, multiplied here as in the kernel above.
template <typename T>
__global__ void gate_heads_kernel(const T* __restrict__ y, const T* __restrict__ mixed, const T* __restrict__ up_values,
                                  int rank, int row_width, const T* __restrict__ proj, long proj_stride,
                                  int gate_column, T* __restrict__ out, int heads, int v, int n_tokens, int per_channel) {
    // (per_channel: the gate of channel i of a head stands at column gate_column + head * v + i, not at gate_column + head)
    __shared__ float partial[4][64];
    const int t = blockIdx.x, head = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int j = blockIdx.z * 64 + lane;
    float value = 0.f;
    if (up_values) {
        if (j < v) {
            const T* row = mixed + ((size_t)t * heads + head) * row_width;
            const int share = (rank + waves - 1) / waves, r0 = wave * share, r1 = min(rank, r0 + share);
            const T* u = up_values + (size_t)head * rank * v + j;
            int r = r0;
            for (; r + 8 <= r1; r += 8) {
                float w[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) w[k] = (float)u[(size_t)(r + k) * v];
#pragma unroll
                for (int k = 0; k < 8; ++k) value += (float)row[r + k] * w[k];
            }
            for (; r < r1; ++r) value += (float)row[r] * (float)u[(size_t)r * v];
        }
        partial[wave][lane] = value;
        __syncthreads();
        if (wave) return;
        value = 0.f;
        for (int w = 0; w < waves; ++w) value += partial[w][lane];
    } else {                            // nothing to multiply: one workgroup gates the head's whole row
        float g = 1.f;
        if (gate_column >= 0 && !per_channel) g = 1.f / (1.f + expf(-(float)proj[(size_t)t * proj_stride + gate_column + head]));
        for (int i = threadIdx.x; i < v; i += blockDim.x) {
            if (gate_column >= 0 && per_channel) g = 1.f / (1.f + expf(-(float)proj[(size_t)t * proj_stride + gate_column + (size_t)head * v + i]));
            out[((size_t)t * heads + head) * v + i] = (T)((float)y[((size_t)head * n_tokens + t) * v + i] * g);
        }
        return;
    }
    if (j >= v) return;
    float g = 1.f;
    if (gate_column >= 0) g = 1.f / (1.f + expf(-(float)proj[(size_t)t * proj_stride + gate_column + (per_channel ? (size_t)head * v + j : (size_t)head)]));
    out[((size_t)t * heads + head) * v + j] = (T)(value * g);
}

LSA_EXPORT int lsa_latent_prepare(int code, const void* proj, long proj_stride, const void* q_latent, const void* up_keys,
                                  const float* norm_weight, float eps,
                                  const float* cos_sin, int pairs, void* keys, void* values, const int* table, int table_stride,
                                  const int* token_row, const int* positions, int page_size, void* out_q, int heads, int dim, int rot_dim,
                                  int rank, int row_width, int write_cache, int n_tokens, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (rank + rot_dim > row_width || 2 * pairs > rot_dim || page_size <= 0 || (q_latent == nullptr) == (up_keys == nullptr)) return -1;
    // (256 threads where the product is made here and for the cache row's norm; the copy alone needs a wavefront a piece)
    dim3 grid(n_tokens, heads + 1, up_keys ? (row_width + 63) / 64 : 1);
#define LSA_LAUNCH(T) latent_prepare_kernel<T><<<grid, 256, 0, stream>>>((const T*)proj, proj_stride, (const T*)q_latent, (const T*)up_keys, \
        norm_weight, eps, cos_sin, pairs, (T*)keys, (T*)values, table, table_stride, token_row, positions, page_size, (T*)out_q, heads, dim, \
        rot_dim, rank, row_width, write_cache, n_tokens)
    if (code) LSA_LAUNCH(bf16_t); else LSA_LAUNCH(float);
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_gate_heads(int code, const void* y, const void* mixed, const void* up_values, int rank, int row_width, const void* proj,
                              long proj_stride, int gate_column, void* out, int heads, int v, int n_tokens, int per_channel,
                              hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if ((y == nullptr) == (up_values == nullptr) || (up_values != nullptr && (mixed == nullptr || rank > row_width))) return -1;
    dim3 grid(n_tokens, heads, up_values ? (v + 63) / 64 : 1);
#define LSA_LAUNCH(T) gate_heads_kernel<T><<<grid, up_values ? 256 : 64, 0, stream>>>((const T*)y, (const T*)mixed, (const T*)up_values, rank, row_width, \
        (const T*)proj, proj_stride, gate_column, (T*)out, heads, v, n_tokens, per_channel)
    if (code) LSA_LAUNCH(bf16_t); else LSA_LAUNCH(float);
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}
