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

// Greedy choice in two stages so that a few rows still use the whole chip: every workgroup finds the
// first maximum of one chunk of a row, then one workgroup per row picks among the chunks.  Ties go
// to the lowest index at every stage.
__device__ __forceinline__ void first_max_reduce(float& best, int& best_i, float* sv, int* si) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, WAVE);
        const int oi = __shfl_xor(best_i, o, WAVE);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) { sv[w] = best; si[w] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int i = 1; i < nw; ++i)
            if (sv[i] > best || (sv[i] == best && si[i] < best_i)) { best = sv[i]; best_i = si[i]; }
}

__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ logits, int V, int chunk,
                                                            float* __restrict__ part_v, int* __restrict__ part_i) {
    __shared__ float sv[4];
    __shared__ int si[4];
    const float* row = logits + (int64_t)blockIdx.x * V;
    const int lo = blockIdx.y * chunk, hi = min(V, lo + chunk);
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const float v = row[i];
        if (v > best || best_i == 0x7fffffff) { best = v; best_i = i; }      // ascending i: strict > keeps the first
    }
    first_max_reduce(best, best_i, sv, si);
    if (threadIdx.x == 0) {
        part_v[blockIdx.x * gridDim.y + blockIdx.y] = best;
        part_i[blockIdx.x * gridDim.y + blockIdx.y] = best_i;
    }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ part_v,
                                                          const int* __restrict__ part_i, int n_chunks,
                                                          int* __restrict__ out) {
    __shared__ float sv[1];
    __shared__ int si[1];
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int c = threadIdx.x; c < n_chunks; c += blockDim.x) {
        const float v = part_v[blockIdx.x * n_chunks + c];
        const int i = part_i[blockIdx.x * n_chunks + c];
        if (i != 0x7fffffff && (v > best || best_i == 0x7fffffff || (v == best && i < best_i))) { best = v; best_i = i; }
    }
    first_max_reduce(best, best_i, sv, si);
    if (threadIdx.x == 0) out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
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

// part_v, part_i: workspace of n_rows * li_argmax_chunks(V) entries each
extern "C" int li_argmax_chunks(int V) { return V <= 4096 ? 1 : (V + 4095) / 4096; }

extern "C" int li_argmax(const float* logits, int n_rows, int V, float* part_v, int* part_i, int* out,
                         hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (V <= 0 || !part_v || !part_i) return LI_BAD_ARG;
    const int n_chunks = li_argmax_chunks(V);
    const int chunk = (V + n_chunks - 1) / n_chunks;
    argmax_chunks_kernel<<<dim3(n_rows, n_chunks), 256, 0, stream>>>(logits, V, chunk, part_v, part_i);
    LI_CHECK_LAUNCH();
    argmax_final_kernel<<<n_rows, 64, 0, stream>>>(part_v, part_i, n_chunks, out);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

extern "C" int li_sample(const float* logits, int n_rows, int V, float temperature, const int* seq_slot,
                         void* state, const float* forced_r, int* out, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (V <= 0 || temperature <= 0.f) return LI_BAD_ARG;             // greedy goes through li_argmax
    if (!forced_r && (!seq_slot || !state)) return LI_BAD_ARG;
    sample_kernel<<<n_rows, V >= 4096 ? 1024 : 256, 0, stream>>>(logits, V, temperature, seq_slot,
                                                                  (unsigned long long*)state, forced_r, out);
    LI_CHECK_LAUNCH();
    return LI_OK;
}
