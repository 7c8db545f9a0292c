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

// One workgroup per token.  proj row: heads x [dim plain, rot_dim rotated] query dimensions, then the token's
// `rank` latent dimensions and its rot_dim rotated key dimensions.
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ proj, long proj_stride, const T* __restrict__ q_latent, const float* __restrict__ norm_weight, float eps,
    const float* __restrict__ cos_sin, int pairs, T* __restrict__ keys, T* __restrict__ values, const int* __restrict__ table,
    int table_stride, const int* __restrict__ token_row, const int* __restrict__ positions, int page_size, T* __restrict__ out_q,
    int heads, int dim, int rot_dim, int rank, int row_width, int write_cache, int n_tokens) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const T* mine = proj + (size_t)t * proj_stride;
    const float* cs = cos_sin + (size_t)t * 2 * pairs;
    const int per_head = dim + rot_dim;
    T* q = out_q + (size_t)t * heads * row_width;
    for (int i = threadIdx.x; i < heads * row_width; i += blockDim.x) {
        const int head = i / row_width, e = i - head * row_width;
        float v = 0.f;
        if (e < rank) v = (float)q_latent[((size_t)head * n_tokens + t) * rank + e];
        else if (e < rank + rot_dim) v = turned(mine + head * per_head + dim, e - rank, cs, pairs);
        q[i] = (T)v;
    }
    if (!write_cache) return;
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

// out[t][h * v + j] = y[h][t][j] * sigmoid(proj[t][gate_column + h])   (gate_column < 0: no gate)
template <typename T>
__global__ __launch_bounds__(256) void gate_heads_kernel(const T* __restrict__ y, const T* __restrict__ proj, long proj_stride,
                                                         int gate_column, T* __restrict__ out, int heads, int v, int n_tokens) {
    const int t = blockIdx.x;
    for (int i = threadIdx.x; i < heads * v; i += blockDim.x) {
        const int head = i / v, j = i - head * v;
        float g = 1.f;
        if (gate_column >= 0) g = 1.f / (1.f + expf(-(float)proj[(size_t)t * proj_stride + gate_column + head]));
        out[(size_t)t * heads * v + i] = (T)((float)y[((size_t)head * n_tokens + t) * v + j] * g);
    }
}

LSA_EXPORT int lsa_latent_prepare(int code, const void* proj, long proj_stride, const void* q_latent, const float* norm_weight, float eps,
                                  const float* cos_sin, int pairs, void* keys, void* values, const int* table, int table_stride,
                                  const int* token_row, const int* positions, int page_size, void* out_q, int heads, int dim, int rot_dim,
                                  int rank, int row_width, int write_cache, int n_tokens, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (rank + rot_dim > row_width || 2 * pairs > rot_dim || page_size <= 0) return -1;
#define LSA_LAUNCH(T) latent_prepare_kernel<T><<<n_tokens, 256, 0, stream>>>((const T*)proj, proj_stride, (const T*)q_latent, norm_weight, eps, \
        cos_sin, pairs, (T*)keys, (T*)values, table, table_stride, token_row, positions, page_size, (T*)out_q, heads, dim, rot_dim, rank, \
        row_width, write_cache, n_tokens)
    if (code) LSA_LAUNCH(bf16_t); else LSA_LAUNCH(float);
#undef LSA_LAUNCH
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_gate_heads(int code, const void* y, const void* proj, long proj_stride, int gate_column, void* out, int heads, int v,
                              int n_tokens, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (code) gate_heads_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)y, (const bf16_t*)proj, proj_stride, gate_column, (bf16_t*)out, heads, v, n_tokens);
    else gate_heads_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)y, (const float*)proj, proj_stride, gate_column, (float*)out, heads, v, n_tokens);
    LSA_LAUNCH_CHECK();
}
