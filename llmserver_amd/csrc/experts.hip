// Routed experts for a flat batch of tokens.  The router's logits, the choice of the `top` largest and their softmax
// are 32-bit.  The experts' products pick every (token, chosen expert) pair's matrices on the device from the list
// the router wrote: a pair streams its expert's gate and up rows against the token's row and applies silu(gate) * up;
// a token's output row is the weighted sum over its pairs of the expert's down rows against the pair's hidden row.
// Sums are 32-bit; the hidden row is rounded once to the activations' type; the output is float32.
#include "common.hpp"

using namespace lsa;

constexpr float NEG_INF = -__builtin_huge_valf();

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

// One workgroup per token: logits of all experts (a wavefront per expert in turn), then wavefront 0 picks the `top`
// largest (the lowest index among equal ones) and writes their softmax.  Dynamic LDS: a float per expert.
template <typename T>
__global__ __launch_bounds__(256) void route_kernel(const T* __restrict__ x, const float* __restrict__ router, int experts, int top,
                                                    int* __restrict__ chosen, float* __restrict__ weights, int width) {
    extern __shared__ float lds[];
    float* logits = lds;
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const T* row = x + (size_t)t * width;
    for (int e = wave; e < experts; e += waves) {
        const float* r = router + (size_t)e * width;
        float acc = 0.f;
        for (int i = lane; i < width; i += 64) acc += r[i] * (float)row[i];
        acc = wave_sum(acc);
        if (lane == 0) logits[e] = acc;
    }
    __syncthreads();
    if (wave) return;
    // Every lane ends each round with the same (best, where), so nothing crosses lanes through LDS: the lane that
    // owns an entry of `logits` (entry % 64) is the only one that reads it and the one that strikes it out.
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
        const float weight = expf(best - largest);
        total += weight;
        if (lane == 0) {
            chosen[(size_t)t * top + k] = where;
            weights[(size_t)t * top + k] = weight;
        }
        if ((where & 63) == lane) logits[where] = NEG_INF;
    }
    if (lane == 0)
        for (int k = 0; k < top; ++k) weights[(size_t)t * top + k] /= total;         // (its own writes)
}

// grid (pairs, blocks of hidden columns): hidden[pair][f] = silu(G[f] . x) * (U[f] . x) for the pair's expert.
template <typename T>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ gate_up,
                                                              const int* __restrict__ chosen, T* __restrict__ hidden, int top,
                                                              int inter, int width, int experts, int columns_per_block, bool in_lds) {
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
        if (lane == 0) hidden[(size_t)pair * inter + f] = (T)(g / (1.f + expf(-g)) * u);
    }
}

// grid (tokens, blocks of output columns): out[t][c] = sum_s weights[t][s] * (D_s[c] . hidden[t * top + s]).
template <typename T>
__global__ __launch_bounds__(256) void experts_down_kernel(const T* __restrict__ hidden, const T* __restrict__ down,
                                                           const int* __restrict__ chosen, const float* __restrict__ weights,
                                                           float* __restrict__ out, int top, int inter, int width, int experts,
                                                           int columns_per_block, bool in_lds) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const T* h_lds = hidden + (size_t)t * top * inter;
    if (in_lds) {
        T* staged = reinterpret_cast<T*>(lds_bytes);
        for (int i = threadIdx.x; i < top * inter; i += blockDim.x) staged[i] = h_lds[i];
        __syncthreads();
        h_lds = staged;
    }
    const int c0 = blockIdx.y * columns_per_block, c1 = min(width, c0 + columns_per_block);
    for (int c = c0 + wave; c < c1; c += waves) {
        float acc = 0.f;
        for (int s = 0; s < top; ++s) {
            int expert = chosen[(size_t)t * top + s];
            expert = expert < 0 ? 0 : expert >= experts ? experts - 1 : expert;
            const T* row = down + ((size_t)expert * width + c) * inter;
            acc += weights[(size_t)t * top + s] * wave_dot(row, h_lds + (size_t)s * inter, inter, lane);
        }
        if (lane == 0) out[(size_t)t * width + c] = acc;
    }
}

LSA_EXPORT int lsa_route_experts(int code, const void* x, const float* router, int experts, int top, int* chosen, float* weights,
                                 int n, int width, hipStream_t stream) {
    if (n <= 0) return 0;
    if (top < 1 || top > experts || (size_t)experts * 4 > 60000) return -1;
    const size_t lds = (size_t)experts * sizeof(float);
    if (code) route_kernel<bf16_t><<<n, 256, lds, stream>>>((const bf16_t*)x, router, experts, top, chosen, weights, width);
    else route_kernel<float><<<n, 256, lds, stream>>>((const float*)x, router, experts, top, chosen, weights, width);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_experts_gate_up(int code, const void* x, const void* gate_up, const int* chosen, void* hidden, int n, int top,
                                   int inter, int width, int experts, hipStream_t stream) {
    if (n <= 0) return 0;
    size_t lds = (size_t)width * (code ? 2 : 4);
    const bool in_lds = lds <= 64000;
    if (!in_lds) lds = 0;
    const int columns = 16;
    dim3 grid(n * top, (inter + columns - 1) / columns);
    if (code) experts_gate_up_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)x, (const bf16_t*)gate_up, chosen, (bf16_t*)hidden, top, inter, width, experts, columns, in_lds);
    else experts_gate_up_kernel<float><<<grid, 256, lds, stream>>>((const float*)x, (const float*)gate_up, chosen, (float*)hidden, top, inter, width, experts, columns, in_lds);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_experts_down(int code, const void* hidden, const void* down, const int* chosen, const float* weights, float* out,
                                int n, int top, int inter, int width, int experts, hipStream_t stream) {
    if (n <= 0) return 0;
    size_t lds = (size_t)top * inter * (code ? 2 : 4);
    const bool in_lds = lds <= 64000;
    if (!in_lds) lds = 0;
    const int columns = 16;
    dim3 grid(n, (width + columns - 1) / columns);
    if (code) experts_down_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)hidden, (const bf16_t*)down, chosen, weights, out, top, inter, width, experts, columns, in_lds);
    else experts_down_kernel<float><<<grid, 256, lds, stream>>>((const float*)hidden, (const float*)down, chosen, weights, out, top, inter, width, experts, columns, in_lds);
    LSA_LAUNCH_CHECK();
}
