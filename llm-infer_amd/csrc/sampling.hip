// Sampling from float32 logits [B, V] (tools/infer.cpp:34-106).
//   greedy     : the first maximum wins (strict >, :64-74)
//   temperature: p_i = exp((l_i - max) / T) / sum (:84-102); with r uniform in [0, 1) the
//                token is the first i with r < cumsum_i, fallback V-1 (:50-60); T <= 0 is greedy.
// r comes from a counter-based generator with a key and a counter for every
// sequence slot, so a sequence's tokens do not depend on what else is in the batch.
#include "common.h"

__host__ __device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

// uniform in [0, 1) with 24 bits, from (key, counter)
__host__ __device__ __forceinline__ float uniform01(uint64_t key, uint64_t counter) {
    const uint64_t z = mix64(mix64(key) + counter * 0x9E3779B97F4A7C15ULL);
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

extern "C" float li_uniform01(uint64_t key, uint64_t counter) { return uniform01(key, counter); }

__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, int V,
                                                      int* __restrict__ out) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float* row = logits + (int64_t)blockIdx.x * V;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = row[i];
        if (v > best || best_i == 0x7fffffff) { best = v; best_i = i; }      // ascending i: strict > keeps the first
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, WAVE);
        const int oi = __shfl_xor(best_i, o, WAVE);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) { sv[w] = best; si[w] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < nw; ++i)
            if (sv[i] > best || (sv[i] == best && si[i] < best_i)) { best = sv[i]; best_i = si[i]; }
        out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
    }
}

// state: [n_slots, 2] uint64 (key, counter); the counter advances by one per sampled token.
__global__ __launch_bounds__(1024) void sample_kernel(const float* __restrict__ logits, int V, float temperature,
                                                      const int* __restrict__ seq_slot,
                                                      unsigned long long* __restrict__ state,
                                                      const float* __restrict__ forced_r,
                                                      int* __restrict__ out) {
    __shared__ float scratch[16];
    __shared__ float sums[1024];
    __shared__ int found;
    const float* row = logits + (int64_t)blockIdx.x * V;
    const int tid = threadIdx.x, nt = blockDim.x;
    float mx = -INFINITY;
    for (int i = tid; i < V; i += nt) mx = fmaxf(mx, row[i]);
    mx = block_max(mx, scratch);
    const int chunk = (V + nt - 1) / nt;
    const int c0 = min(V, tid * chunk), c1 = min(V, c0 + chunk);
    float local = 0.f;
    for (int i = c0; i < c1; ++i) local += expf((row[i] - mx) / temperature);
    sums[tid] = local;
    if (tid == 0) found = V - 1;
    __syncthreads();
    if (tid == 0) {
        float r;
        if (forced_r) r = forced_r[blockIdx.x];
        else {
            unsigned long long* st = state + 2 * (int64_t)seq_slot[blockIdx.x];
            r = uniform01(st[0], st[1]);
            st[1] += 1;
        }
        float total = 0.f;
        for (int i = 0; i < nt; ++i) total += sums[i];
        const float target = r * total;
        float c = 0.f;
        int owner = -1;
        for (int i = 0; i < nt; ++i) {
            if (target < c + sums[i]) { owner = i; break; }
            c += sums[i];
        }
        if (owner >= 0) {
            const int b0 = min(V, owner * chunk), b1 = min(V, b0 + chunk);
            int pick = b1 - 1;
            for (int i = b0; i < b1; ++i) {
                c += expf((row[i] - mx) / temperature);
                if (target < c) { pick = i; break; }
            }
            found = pick;
        }
        out[blockIdx.x] = found;
    }
}

extern "C" int li_argmax(const float* logits, int n_rows, int V, int* out, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (V <= 0) return LI_BAD_ARG;
    argmax_kernel<<<n_rows, V >= 4096 ? 1024 : 256, 0, stream>>>(logits, V, out);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

extern "C" int li_sample(const float* logits, int n_rows, int V, float temperature, const int* seq_slot,
                         void* state, const float* forced_r, int* out, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (V <= 0) return LI_BAD_ARG;
    if (temperature <= 0.f) return li_argmax(logits, n_rows, V, out, stream);
    if (!forced_r && (!seq_slot || !state)) return LI_BAD_ARG;
    sample_kernel<<<n_rows, V >= 4096 ? 1024 : 256, 0, stream>>>(logits, V, temperature, seq_slot,
                                                                  (unsigned long long*)state, forced_r, out);
    LI_CHECK_LAUNCH();
    return LI_OK;
}
