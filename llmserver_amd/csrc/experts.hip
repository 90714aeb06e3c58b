// Routed experts for a flat batch of tokens.  The router's logits, the choice of the `top` largest and their softmax
// are 32-bit.  The experts' products pick every (token, chosen expert) pair's matrices on the device from the list
// the router wrote: a pair streams its expert's gate and up rows against the token's row and applies silu(gate) * up;
// a token's output row is the weighted sum over its pairs of the expert's down rows against the pair's hidden row.
// Sums are 32-bit; the hidden row is rounded once to the activations' type; the output is float32.
#include "common.hpp"

using namespace lsa;

constexpr float NEG_INF = -__builtin_huge_valf();

// The experts' activation.  limit <= 0: silu(gate) * up.  limit > 0: the clamped form g * sigmoid(1.702 g) * (u + 1) with
// g = min(gate, limit), u = clamp(up, -limit, limit).
__device__ __forceinline__ float gated_activation(float g, float u, float limit) {
    if (limit > 0.f) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        return g / (1.f + expf(-1.702f * g)) * (u + 1.f);
    }
    return g / (1.f + expf(-g)) * u;
}

// Dot product of a weight row with a vector in LDS, a wavefront wide: 16-byte pieces where the length allows.
template <typename T>
__device__ inline float wave_dot(const T* __restrict__ w, const T* x_lds, int n, int lane) {
    constexpr int V = Elem<T>::kVec;
    float acc = 0.f;
    if (n % V == 0 && ((reinterpret_cast<size_t>(w) | reinterpret_cast<size_t>(x_lds)) & 15) == 0) {
        for (int i = lane * V; i < n; i += 64 * V) {
            const Vec16<T> a = load_vec16(w + i);
            const Vec16<T> b = *reinterpret_cast<const Vec16<T>*>(x_lds + i);
#pragma unroll
            for (int k = 0; k < V; ++k) acc += (float)a.v[k] * (float)b.v[k];
        }
    } else {
        for (int i = lane; i < n; i += 64) acc += (float)w[i] * (float)x_lds[i];
    }
    return wave_sum(acc);
}

// Two rows at once against the same vector (a gate row and its up row): their loads are in flight together.
template <typename T>
__device__ inline void wave_dot2(const T* __restrict__ w0, const T* __restrict__ w1, const T* x_lds, int n, int lane, float& r0, float& r1) {
    constexpr int V = Elem<T>::kVec;
    float a0 = 0.f, a1 = 0.f;
    if (n % V == 0 && ((reinterpret_cast<size_t>(w0) | reinterpret_cast<size_t>(w1) | reinterpret_cast<size_t>(x_lds)) & 15) == 0) {
        for (int i = lane * V; i < n; i += 64 * V) {
            const Vec16<T> p = load_vec16(w0 + i);
            const Vec16<T> q = load_vec16(w1 + i);
            const Vec16<T> b = *reinterpret_cast<const Vec16<T>*>(x_lds + i);
#pragma unroll
            for (int k = 0; k < V; ++k) {
                a0 += (float)p.v[k] * (float)b.v[k];
                a1 += (float)q.v[k] * (float)b.v[k];
            }
        }
    } else {
        for (int i = lane; i < n; i += 64) {
            a0 += (float)w0[i] * (float)x_lds[i];
            a1 += (float)w1[i] * (float)x_lds[i];
        }
    }
    r0 = wave_sum(a0);
    r1 = wave_sum(a1);
}

// Router logits for steps of few tokens, where a library product would be a launch of 11 us for a few thousand
// multiplications: grid (tokens, experts / 4), a wavefront per expert, float32 throughout.
__global__ __launch_bounds__(256) void route_logits_kernel(const float* __restrict__ x, const float* __restrict__ router,
                                                           float* __restrict__ logits, int experts, int width) {
    const int lane = threadIdx.x & 63, e = blockIdx.y * 4 + (threadIdx.x >> 6), t = blockIdx.x;
    if (e >= experts) return;
    const float* r = router + (size_t)e * width;
    const float* row = x + (size_t)t * width;
    float acc = 0.f;
    if (width % 4 == 0) {
        for (int i = lane * 4; i < width; i += 256) {
            const float4 a = *reinterpret_cast<const float4*>(r + i), b = *reinterpret_cast<const float4*>(row + i);
            acc += a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
        }
    } else {
        for (int i = lane; i < width; i += 64) acc += r[i] * row[i];
    }
    acc = wave_sum(acc);
    if (lane == 0) logits[(size_t)t * experts + e] = acc;
}

// One wavefront per token: the `top` largest of the token's float32 logits (the lowest index among equal ones) and
// their softmax.  The logits themselves are a float32 matrix product made before this kernel.  A lane keeps the logits
// of experts lane, lane + 64, ... in LDS (its own entries only: nothing crosses lanes through LDS), and every lane ends
// each round with the same (best, where).
__global__ __launch_bounds__(256) void route_top_kernel(const float* __restrict__ all_logits, int experts, int top,
                                                        int* __restrict__ chosen, float* __restrict__ weights, int n_tokens,
                                                        int sigmoid_scores, int groups, int keep, const float* __restrict__ bias) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x * (blockDim.x >> 6) + wave;
    if (t >= n_tokens) return;
    // (two arrays a wavefront: the values the choice is made among, and, for sigmoid scores, the scores themselves)
    float* logits = lds + (size_t)wave * 2 * experts;
    float* scores = logits + experts;
    for (int e = lane; e < experts; e += 64) {
        float v = all_logits[(size_t)t * experts + e];
        if (bias) v += bias[e];                            // (a bias per expert joins the logits)
        if (sigmoid_scores) v = 1.f / (1.f + expf(-v));
        logits[e] = v;
        scores[e] = v;
    }
    if (sigmoid_scores && groups > 1) {
        // A group's score is the sum of its two largest scores; the `keep` best groups stay (the first of equal ones),
        // the experts of the others cannot be chosen.  Lane g (and g + 64, ...) scores group g; entries of other lanes
        // are read here (a wavefront's LDS operations complete in the order they were issued).
        __builtin_amdgcn_wave_barrier();
        const int per = experts / groups;
        {
            const int base = 0, g = lane;             // (at most 64 groups: the host refuses more)
            float mine = NEG_INF;
            if (g < groups) {
                float first = NEG_INF, second = NEG_INF;
                for (int i = 0; i < per; ++i) {
                    const float v = scores[g * per + i];
                    if (v > first) { second = first; first = v; }
                    else if (v > second) second = v;
                }
                mine = per > 1 ? first + second : first;
            }
            // rank of my group among all: groups with a larger score, or an equal one and a smaller index, come first
            int before = 0;
            for (int other = 0; other < min(64, groups - base); ++other) {
                const float theirs = __shfl(mine, other, 64);
                before += (theirs > mine || (theirs == mine && other < lane)) ? 1 : 0;
            }
            if (g < groups && before >= keep)
                for (int i = 0; i < per; ++i) logits[g * per + i] = NEG_INF;
        }
        __builtin_amdgcn_wave_barrier();
    }
    float largest = 0.f, total = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = NEG_INF;
        int where = 0x7fffffff;
        for (int e = lane; e < experts; e += 64) {
            const float v = logits[e];
            if (v > best || (v == best && e < where)) { best = v; where = e; }
        }
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) {
            const float other = __shfl_xor(best, offset, 64);
            const int other_where = __shfl_xor(where, offset, 64);
            if (other > best || (other == best && other_where < where)) { best = other; where = other_where; }
        }
        if (where >= experts) where = k < experts ? k : 0;        // (only if every logit left is NaN or -inf)
        if (k == 0) largest = best;
        const float weight = sigmoid_scores ? best : expf(best - largest);
        total += weight;
        if (lane == 0) {
            chosen[(size_t)t * top + k] = where;
            weights[(size_t)t * top + k] = weight;
        }
        if ((where & 63) == lane) logits[where] = NEG_INF;
    }
    if (lane == 0 && !sigmoid_scores)
        for (int k = 0; k < top; ++k) weights[(size_t)t * top + k] /= total;         // (its own writes)
}

// grid (pairs, blocks of hidden columns): hidden[pair][f] = silu(G[f] . x) * (U[f] . x) for the pair's expert.
template <typename T>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ gate_up,
                                                              const int* __restrict__ chosen, T* __restrict__ hidden, int top,
                                                              int inter, int width, int experts, int columns_per_block, bool in_lds,
                                                              float limit) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int pair = blockIdx.x, t = pair / top;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const T* x_lds = x + (size_t)t * width;                  // (a row too long for LDS is read where it lies)
    if (in_lds) {
        T* staged = reinterpret_cast<T*>(lds_bytes);
        for (int i = threadIdx.x; i < width; i += blockDim.x) staged[i] = x_lds[i];
        __syncthreads();
        x_lds = staged;
    }
    int expert = chosen[pair];
    expert = expert < 0 ? 0 : expert >= experts ? experts - 1 : expert;
    const T* base = gate_up + (size_t)expert * 2 * inter * width;
    const int f0 = blockIdx.y * columns_per_block, f1 = min(inter, f0 + columns_per_block);
    for (int f = f0 + wave; f < f1; f += waves) {
        float g, u;
        wave_dot2(base + (size_t)f * width, base + (size_t)(inter + f) * width, x_lds, width, lane, g, u);
        if (lane == 0) hidden[(size_t)pair * inter + f] = (T)gated_activation(g, u, limit);
    }
}

// grid (tokens, blocks of output columns): out[t][c] = sum_s weights[t][s] * (D_s[c] . hidden[t * top + s]).
// A wavefront owns a column: every lane adds up its share of all `top` dot products, weighted, and the lanes' sums meet
// once at the end; the loads of all pairs' rows are independent of one another.
template <typename T>
__global__ __launch_bounds__(256) void experts_down_kernel(const T* __restrict__ hidden, const T* __restrict__ down,
                                                           const int* __restrict__ chosen, const float* __restrict__ weights,
                                                           float* __restrict__ out, int top, int inter, int width, int experts,
                                                           int columns_per_block, bool in_lds) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    constexpr int V = Elem<T>::kVec;
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const T* h_lds = hidden + (size_t)t * top * inter;
    if (in_lds) {
        T* staged = reinterpret_cast<T*>(lds_bytes);
        for (int i = threadIdx.x; i < top * inter; i += blockDim.x) staged[i] = h_lds[i];
        __syncthreads();
        h_lds = staged;
    }
    const bool vectors = inter % V == 0 && ((reinterpret_cast<size_t>(down) | reinterpret_cast<size_t>(h_lds)) & 15) == 0;
    // the token's experts and weights, read once (a lookup per piece below would be a trip to memory each)
    constexpr int MOST = 128;
    __shared__ int expert_of[MOST];
    __shared__ float weight_of[MOST];
    for (int s = threadIdx.x; s < min(top, MOST); s += blockDim.x) {
        const int expert = chosen[(size_t)t * top + s];
        expert_of[s] = expert < 0 ? 0 : expert >= experts ? experts - 1 : expert;
        weight_of[s] = weights[(size_t)t * top + s];
    }
    __syncthreads();
    const int c0 = blockIdx.y * columns_per_block, c1 = min(width, c0 + columns_per_block);
    for (int c = c0 + wave; c < c1; c += waves) {
        float acc = 0.f;
        if (vectors && top <= MOST) {
            // The pairs' rows end to end are one long vector of top * inter / V pieces, spread over the lanes: every
            // lane is busy whatever the experts' size, and its loads do not wait for one another.
            const int pieces = inter / V, all = top * pieces;
            for (int p = lane; p < all; p += 64) {
                const int s = p / pieces, i = (p - s * pieces) * V;
                const Vec16<T> a = load_vec16(down + ((size_t)expert_of[s] * width + c) * inter + i);
                const Vec16<T> b = *reinterpret_cast<const Vec16<T>*>(h_lds + (size_t)s * inter + i);
                float part = 0.f;
#pragma unroll
                for (int k = 0; k < V; ++k) part += (float)a.v[k] * (float)b.v[k];
                acc += weight_of[s] * part;
            }
        } else {
            for (int s = 0; s < top; ++s) {
                int expert = chosen[(size_t)t * top + s];
                expert = expert < 0 ? 0 : expert >= experts ? experts - 1 : expert;
                const T* row = down + ((size_t)expert * width + c) * inter;
                const T* h = h_lds + (size_t)s * inter;
                float part = 0.f;
                for (int i = lane; i < inter; i += 64) part += (float)row[i] * (float)h[i];
                acc += weights[(size_t)t * top + s] * part;
            }
        }
        acc = wave_sum(acc);
        if (lane == 0) out[(size_t)t * width + c] = acc;
    }
}

LSA_EXPORT int lsa_route_logits(const float* x, const float* router, float* logits, int n, int experts, int width, hipStream_t stream) {
    if (n <= 0) return 0;
    route_logits_kernel<<<dim3(n, (experts + 3) / 4), 256, 0, stream>>>(x, router, logits, experts, width);
    LSA_LAUNCH_CHECK();
}

// sigmoid_scores: the choice is made among sigmoid(logits), which are the weights as they are; groups > 1: only the
// experts of the `keep` best of `groups` equal groups of neighbours can be chosen (at most 64 groups).
LSA_EXPORT int lsa_route_top(const float* logits, int experts, int top, int* chosen, float* weights, int n, int sigmoid_scores,
                             int groups, int keep, const float* bias, hipStream_t stream) {
    if (n <= 0) return 0;
    if (top < 1 || top > experts || (size_t)experts * 32 > 60000) return -1;
    if (groups > 1 && (!sigmoid_scores || groups > 64 || experts % groups || keep < 1 || keep > groups || top > keep * (experts / groups))) return -1;
    route_top_kernel<<<(n + 3) / 4, 256, (size_t)experts * 8 * sizeof(float), stream>>>(logits, experts, top, chosen, weights, n,
                                                                                       sigmoid_scores, groups, keep, bias);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_experts_gate_up(int code, const void* x, const void* gate_up, const int* chosen, void* hidden, int n, int top,
                                   int inter, int width, int experts, float limit, hipStream_t stream) {
    if (n <= 0) return 0;
    size_t lds = (size_t)width * (code ? 2 : 4);
    const bool in_lds = lds <= 64000;
    if (!in_lds) lds = 0;
    const int columns = 16;
    dim3 grid(n * top, (inter + columns - 1) / columns);
    if (code) experts_gate_up_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)x, (const bf16_t*)gate_up, chosen, (bf16_t*)hidden, top, inter, width, experts, columns, in_lds, limit);
    else experts_gate_up_kernel<float><<<grid, 256, lds, stream>>>((const float*)x, (const float*)gate_up, chosen, (float*)hidden, top, inter, width, experts, columns, in_lds, limit);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_experts_down(int code, const void* hidden, const void* down, const int* chosen, const float* weights, float* out,
                                int n, int top, int inter, int width, int experts, hipStream_t stream) {
    if (n <= 0) return 0;
    // (a block takes four columns: staging the token's hidden rows in LDS would cost as much as it reads of the weights)
    const size_t lds = 0;
    const bool in_lds = false;
    const int columns = 4;
    dim3 grid(n, (width + columns - 1) / columns);
    if (code) experts_down_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)hidden, (const bf16_t*)down, chosen, weights, out, top, inter, width, experts, columns, in_lds);
    else experts_down_kernel<float><<<grid, 256, lds, stream>>>((const float*)hidden, (const float*)down, chosen, weights, out, top, inter, width, experts, columns, in_lds);
    LSA_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------------------------------------
// Many tokens (portions of prompts, large batches): the pairs are sorted by expert, each expert's pairs padded to whole
// tiles of TILE_M rows, and one MFMA product per tile multiplies the tile's rows with its expert's matrix, so an expert's
// weights are read once per tile of 64 pairs instead of once per pair.  bfloat16 only (the float32 path keeps the
// kernels above).
//
// sort: one workgroup.  sorted[i] = pair at padded place i (-1: padding), tile_expert[j] = expert of tile j (-1: no tile).
// The order of an expert's pairs among themselves is whatever the atomics give; every pair's row is computed on its
// own, so the results do not depend on it.
constexpr int TILE_M = 64;

__global__ __launch_bounds__(1024) void experts_sort_kernel(const int* __restrict__ chosen, int n_pairs, int experts,
                                                            int* __restrict__ sorted, int* __restrict__ tile_expert, int max_tiles) {
    extern __shared__ int lds_ints[];
    int* counts = lds_ints;
    int* offsets = lds_ints + experts;
    for (int e = threadIdx.x; e < experts; e += blockDim.x) counts[e] = 0;
    for (int i = threadIdx.x; i < max_tiles * TILE_M; i += blockDim.x) sorted[i] = -1;
    for (int j = threadIdx.x; j < max_tiles; j += blockDim.x) tile_expert[j] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = chosen[p];
        if (e >= 0 && e < experts) atomicAdd(&counts[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int running = 0;
        for (int e = 0; e < experts; ++e) {
            offsets[e] = running;
            const int tiles = (counts[e] + TILE_M - 1) / TILE_M;
            for (int j = 0; j < tiles; ++j) tile_expert[running / TILE_M + j] = e;
            running += tiles * TILE_M;
            counts[e] = 0;                       // from here on: how many of the expert's pairs have a place
        }
    }
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = chosen[p];
        if (e >= 0 && e < experts) sorted[offsets[e] + atomicAdd(&counts[e], 1)] = p;
    }
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// C = A . B^T for one tile of 64 sorted pairs and 128 rows of the expert's matrix (K contiguous in both).
//   GATED: B's 128 rows are 64 gate rows f0 .. f0 + 63 and their 64 up rows; the result is silu(gate) * up, 64 columns.
//   Rows of A: a[(sorted[i] / pair_div)] (pair_div = top for the tokens' rows, 1 for the pairs' hidden rows).
// Four wavefronts, each 32 rows x 16 NT columns (GATED: half of them gate columns, half their up columns): 2 x NT MFMA
// tiles of 16 x 16, k in steps of 32.  A slab of BK columns of K of both operands goes through LDS (rows padded by 16
// bytes).  NT = 4 where an expert has few pairs (its weights bound the time), 8 where it has many (every operand read
// from LDS then feeds more products, which is what bounds a tile of 4).
template <int BK, bool GATED, typename O, int NT>
__global__ __launch_bounds__(256) void experts_tile_kernel(const bf16_t* __restrict__ a, int a_stride, int pair_div,
                                                           const bf16_t* __restrict__ b, long expert_stride, int b_rows, int b_up_offset,
                                                           const int* __restrict__ sorted, const int* __restrict__ tile_expert,
                                                           O* __restrict__ out, int out_stride, int n_out, int k, float limit) {
    constexpr int ROW = BK + 8;                                    // elements of a padded row in LDS
    __shared__ __align__(16) bf16_t a_lds[TILE_M * ROW];
    constexpr int BN = 32 * NT;                                    // rows of B a block takes
    __shared__ __align__(16) bf16_t b_lds[BN * ROW];
    __shared__ int rows_of[TILE_M];
    // Workgroups go to the eight XCDs in turn by their number.  The tiles of one expert stand next to each other in the
    // list; numbered so that neighbours in the list get numbers eight apart, they run on one XCD at about the same time
    // and the expert's rows are fetched into one L2 instead of several.
    const int total = gridDim.x * gridDim.y, number = blockIdx.y * gridDim.x + blockIdx.x, share = total / 8;
    const int place = number < share * 8 ? (number % 8) * share + number / 8 : number;
    const int tile = place % gridDim.x, block_n = place / gridDim.x;
    const int expert = tile_expert[tile];
    if (expert < 0) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, quad = lane >> 4;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    if (threadIdx.x < TILE_M) rows_of[threadIdx.x] = sorted[tile * TILE_M + threadIdx.x];
    __syncthreads();
    const int n0 = block_n * (GATED ? BN / 2 : BN);                // first output column of the block
    const bf16_t* bm = b + (size_t)expert * expert_stride;
    // which rows of B the block's LDS rows are: GATED: the first half gate rows n0 + r, the second half their up rows
    auto b_row = [&](int r) {
        int row = GATED ? (r < BN / 2 ? n0 + r : b_up_offset + n0 + r - BN / 2) : n0 + r;
        const int last = GATED ? (r < BN / 2 ? n_out - 1 : b_up_offset + n_out - 1) : n_out - 1;
        return row > last ? last : row;                            // (columns beyond the matrix repeat its last row; never stored)
    };
    f32x4 acc[2][NT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int PIECES = BK / 8;                                 // 16-byte pieces of a row of a slab
    constexpr int A_LOADS = TILE_M * PIECES / 256, B_LOADS = BN * PIECES / 256;      // 16-byte loads of a thread per slab
    // A thread's pieces of a slab: the same rows and places in every slab, so their addresses are made once.  The next
    // slab's pieces travel into registers while this slab is multiplied, and go to LDS when everybody is through with it.
    const bf16_t* a_src[A_LOADS];
    const bf16_t* b_src[B_LOADS];
    int a_dst[A_LOADS], b_dst[B_LOADS];
#pragma unroll
    for (int u = 0; u < A_LOADS; ++u) {
        const int i = threadIdx.x + 256 * u, r = i / PIECES, piece = i - r * PIECES;
        const int pair = rows_of[r];
        a_src[u] = a + (size_t)(pair < 0 ? 0 : pair / pair_div) * a_stride + 8 * piece;
        a_dst[u] = r * ROW + 8 * piece;
    }
#pragma unroll
    for (int u = 0; u < B_LOADS; ++u) {
        const int i = threadIdx.x + 256 * u, r = i / PIECES, piece = i - r * PIECES;
        b_src[u] = bm + (size_t)b_row(r) * k + 8 * piece;
        b_dst[u] = r * ROW + 8 * piece;
    }
    bf16x8 a_next[A_LOADS], b_next[B_LOADS];
#pragma unroll
    for (int u = 0; u < A_LOADS; ++u) a_next[u] = *reinterpret_cast<const bf16x8*>(a_src[u]);
#pragma unroll
    for (int u = 0; u < B_LOADS; ++u) b_next[u] = *reinterpret_cast<const bf16x8*>(b_src[u]);
    for (int k0 = 0; k0 < k; k0 += BK) {
#pragma unroll
        for (int u = 0; u < A_LOADS; ++u) *reinterpret_cast<bf16x8*>(a_lds + a_dst[u]) = a_next[u];
#pragma unroll
        for (int u = 0; u < B_LOADS; ++u) *reinterpret_cast<bf16x8*>(b_lds + b_dst[u]) = b_next[u];
        __syncthreads();
        if (k0 + BK < k) {
#pragma unroll
            for (int u = 0; u < A_LOADS; ++u) a_next[u] = *reinterpret_cast<const bf16x8*>(a_src[u] + k0 + BK);
#pragma unroll
            for (int u = 0; u < B_LOADS; ++u) b_next[u] = *reinterpret_cast<const bf16x8*>(b_src[u] + k0 + BK);
        }
#pragma unroll
        for (int kk = 0; kk < BK; kk += 32) {
            bf16x8 av[2], bv[NT];
#pragma unroll
            for (int i = 0; i < 2; ++i) av[i] = *reinterpret_cast<const bf16x8*>(a_lds + (wave_m * 32 + 16 * i + col) * ROW + kk + 8 * quad);
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                // GATED: the first half of a wavefront's tiles are its gate columns, the second half their up columns
                const int r = GATED ? (j < NT / 2 ? wave_n * (BN / 4) + 16 * j : BN / 2 + wave_n * (BN / 4) + 16 * (j - NT / 2))
                                    : wave_n * (BN / 2) + 16 * j;
                bv[j] = *reinterpret_cast<const bf16x8*>(b_lds + (r + col) * ROW + kk + 8 * quad);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    // lane holds rows 4 * quad + r of each 16 x 16 tile, column col
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int pair = rows_of[wave_m * 32 + 16 * i + 4 * quad + r];
            if (pair < 0) continue;
            O* o = out + (size_t)pair * out_stride;
            if (GATED) {
#pragma unroll
                for (int j = 0; j < NT / 2; ++j) {
                    const int f = n0 + wave_n * (BN / 4) + 16 * j + col;
                    const float g = acc[i][j][r], u = acc[i][j + NT / 2][r];
                    if (f < n_out) o[f] = (O)gated_activation(g, u, limit);
                }
            } else {
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const int c = n0 + wave_n * (BN / 2) + 16 * j + col;
                    if (c < n_out) o[c] = (O)acc[i][j][r];
                }
            }
        }
}

// out[t][c] = sum_s weights[t][s] * y[t * top + s][c]
__global__ __launch_bounds__(256) void experts_combine_kernel(const float* __restrict__ y, const float* __restrict__ weights,
                                                              float* __restrict__ out, int top, int width) {
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float acc = 0.f;
        for (int s = 0; s < top; ++s) acc += weights[(size_t)t * top + s] * y[((size_t)t * top + s) * width + c];
        out[(size_t)t * width + c] = acc;
    }
}

LSA_EXPORT int lsa_experts_tile_rows() { return TILE_M; }

// Sorted, tiled products for bfloat16: hidden = silu(G x) * (U x) and y = D hidden for all pairs, then the weighted sums.
// Scratch: sorted [max_tiles * 64] and tile_expert [max_tiles] ints, y [pairs, width] floats; max_tiles >= ceil(pairs / 64) + experts.
LSA_EXPORT int lsa_experts_tiled(const void* x, const void* gate_up, const void* down, const int* chosen, const float* weights,
                                 void* hidden, float* y, float* out, int* sorted, int* tile_expert, int max_tiles, int n, int top,
                                 int inter, int width, int experts, float limit, hipStream_t stream) {
    if (n <= 0) return 0;
    const int pairs = n * top;
    if (width % 32 || inter % 32 || max_tiles < (pairs + TILE_M - 1) / TILE_M + experts || (size_t)experts * 8 > 60000) return -1;
    experts_sort_kernel<<<1, 1024, (size_t)experts * 2 * sizeof(int), stream>>>(chosen, pairs, experts, sorted, tile_expert, max_tiles);
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* gu = (const bf16_t*)gate_up;
    const bf16_t* dn = (const bf16_t*)down;
    bf16_t* hb = (bf16_t*)hidden;
    const bool many = pairs >= 16 * experts;                    // pairs to an expert: wide tiles pay
#define LSA_TILES(BK, NT) do { \
        dim3 grid1(max_tiles, (inter + 16 * NT - 1) / (16 * NT)), grid2(max_tiles, (width + 32 * NT - 1) / (32 * NT)); \
        if (!second) experts_tile_kernel<BK, true, bf16_t, NT><<<grid1, 256, 0, stream>>>(xb, width, top, gu, (long)2 * inter * width, 2 * inter, inter, sorted, tile_expert, hb, inter, inter, width, limit); \
        else experts_tile_kernel<BK, false, float, NT><<<grid2, 256, 0, stream>>>(hb, inter, 1, dn, (long)width * inter, width, 0, sorted, tile_expert, y, width, width, inter, 0.f); \
    } while (0)
    for (int pass = 0; pass < 2; ++pass) {
        const bool second = pass == 1;
        const bool wide_slab = (second ? inter : width) % 64 == 0;
        if (wide_slab && many) LSA_TILES(64, 8);
        else if (wide_slab) LSA_TILES(64, 4);
        else if (many) LSA_TILES(32, 8);
        else LSA_TILES(32, 4);
    }
#undef LSA_TILES
    experts_combine_kernel<<<n, 256, 0, stream>>>(y, weights, out, top, width);
    LSA_LAUNCH_CHECK();
}
