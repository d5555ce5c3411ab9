// Sampling from float32 logits [B, V] (tools/infer.cpp:34-106).
//   greedy     : the first maximum wins (strict >, :64-74)
//   temperature: p_i = exp((l_i - max) / T) / sum (:84-102); with r uniform in [0, 1) the
//                token is the first i with r < cumsum_i, fallback V-1 (:50-60); T <= 0 is greedy.
// r comes from a counter-based generator with a key and a counter for every
// sequence slot, so a sequence's tokens do not depend on what else is in the batch.
#include "common.h"
#include "no_alloc.h"
#include <mutex>

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

// Temperature sampling in two stages, so that a few rows still use the whole chip.
// Stage 1: a workgroup takes one chunk of a row (a multiple of 64 elements, at most 64 chunks a row),
// finds the chunk's maximum m and writes, for every 64 consecutive elements ("step"), the sum of
// exp((l - m) / T), and the chunk's sum of these, all taken in index order.
// Stage 2: one wave a row brings the chunks to the row's maximum (sum * exp((m - max) / T)), and
// finds with scans over its lanes first the chunk, then the step, then the index at which the
// cumulative sum exceeds r * total: the inverse CDF of tools/infer.cpp:50-60 up to float32 rounding
// of the sums (the exponential is the hardware's 2^x).  Where rounding lets every candidate pass,
// the last one is taken (the fallback of :60).
#define LOG2E_F 1.4426950408889634f

__device__ __forceinline__ float wave_inclusive_scan(float v, int lane) {
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const float t = __shfl_up(v, o, WAVE);
        if (lane >= o) v += t;
    }
    return v;
}

// workspace per row and chunk: [0] maximum, [1] sum, [2 .. 2 + steps) step sums; steps = chunk / 64
// (temperature_dev, if not null, holds the temperature on the device and wins: a recorded step then
// serves every temperature)
__global__ __launch_bounds__(256) void sample_chunks_kernel(const float* __restrict__ logits, int V, int chunk,
                                                            float temperature,
                                                            const float* __restrict__ temperature_dev,
                                                            float* __restrict__ ws) {
    if (temperature_dev) temperature = *temperature_dev;
    __shared__ float scratch[16];
    __shared__ float wave_tot[4];
    const float* row = logits + (int64_t)blockIdx.x * V;
    const int c0 = blockIdx.y * chunk, c1 = min(V, c0 + chunk);
    const int steps = chunk >> 6;
    float* out = ws + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * (2 + steps);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float mx = -INFINITY;
    for (int i = c0 + tid; i < c1; i += 256) mx = fmaxf(mx, row[i]);
    mx = block_max(mx, scratch);
    const float scale2 = LOG2E_F / temperature;                   // exp(d / T) = 2^(d * log2(e) / T)
    float total = 0.f;
    for (int st = wave; st < steps; st += 4) {
        const int i = c0 + st * WAVE + lane;
        float v = i < c1 ? __builtin_amdgcn_exp2f((row[i] - mx) * scale2) : 0.f;
        v = wave_sum(v);
        if (lane == 0) out[2 + st] = v;
        total += v;
    }
    if (lane == 0) wave_tot[wave] = total;
    __syncthreads();
    if (tid == 0) {
        out[0] = mx;
        out[1] = wave_tot[0] + wave_tot[1] + wave_tot[2] + wave_tot[3];
    }
}

__global__ __launch_bounds__(64) void sample_final_kernel(const float* __restrict__ logits, int V, int chunk,
                                                          int n_chunks, float temperature,
                                                          const float* __restrict__ temperature_dev,
                                                          const float* __restrict__ ws,
                                                          const int* __restrict__ seq_slot,
                                                          unsigned long long* __restrict__ state,
                                                          const float* __restrict__ forced_r,
                                                          int* __restrict__ out) {
    if (temperature_dev) temperature = *temperature_dev;
    const int lane = threadIdx.x;
    const float* row = logits + (int64_t)blockIdx.x * V;
    const int steps = chunk >> 6;
    const float* part = ws + (int64_t)blockIdx.x * n_chunks * (2 + steps);
    const float scale2 = LOG2E_F / temperature;
    float r = 0.f;
    if (lane == 0) {
        if (forced_r) r = forced_r[blockIdx.x];
        else {
            unsigned long long* st = state + 2 * (int64_t)seq_slot[blockIdx.x];
            r = uniform01(st[0], st[1]);
            st[1] += 1;
        }
    }
    r = __shfl(r, 0, WAVE);
    // the chunks, one a lane (n_chunks <= 64)
    const bool have = lane < n_chunks;
    const float m_c = have ? part[(int64_t)lane * (2 + steps)] : -INFINITY;
    const float mx = wave_max(m_c);
    const float f_c = have ? __builtin_amdgcn_exp2f((m_c - mx) * scale2) : 0.f;
    const float w_c = have ? part[(int64_t)lane * (2 + steps) + 1] * f_c : 0.f;
    float incl = wave_inclusive_scan(w_c, lane);
    const float target = r * __shfl(incl, WAVE - 1, WAVE);
    unsigned long long hit = __builtin_amdgcn_ballot_w64(have && target < incl);
    const int c = hit ? __builtin_ctzll(hit) : n_chunks - 1;
    // from here on in the chunk's own scale: sums of exp((l - m_c) / T)
    const float f_own = __shfl(f_c, c, WAVE);
    float left = (target - __shfl(incl - w_c, c, WAVE)) / f_own;      // what the chunk still has to cover
    const float* sums = part + (int64_t)c * (2 + steps) + 2;
    const int c0 = c * chunk, c1 = min(V, c0 + chunk);
    const int live_steps = (c1 - c0 + WAVE - 1) >> 6;
    int step = live_steps - 1;
    for (int base = 0; base < live_steps; base += WAVE) {
        const bool in = base + lane < live_steps;
        const float sv = in ? sums[base + lane] : 0.f;
        incl = wave_inclusive_scan(sv, lane);
        hit = __builtin_amdgcn_ballot_w64(in && left < incl);
        if (hit) {
            const int f = __builtin_ctzll(hit);
            step = base + f;
            left -= __shfl(incl - sv, f, WAVE);
            break;
        }
        if (base + WAVE < live_steps) left -= __shfl(incl, WAVE - 1, WAVE);
        else left -= __shfl(incl - sv, live_steps - 1 - base, WAVE);        // nothing hit: search the last step
    }
    const int e0 = c0 + step * WAVE, i = e0 + lane;
    const float m_own = __shfl(m_c, c, WAVE);
    const float e = i < c1 ? __builtin_amdgcn_exp2f((row[i] - m_own) * scale2) : 0.f;
    incl = wave_inclusive_scan(e, lane);
    hit = __builtin_amdgcn_ballot_w64(i < c1 && left < incl);
    const int pick = hit ? e0 + __builtin_ctzll(hit) : min(c1, e0 + WAVE) - 1;
    if (lane == 0) out[blockIdx.x] = pick;
}

// Probability of one given token of each row: softmax at temperature 1 (tools/infer.cpp:77-81; a token
// outside the vocabulary has probability 0).  Reads the chunk maxima and sums that
// sample_chunks_kernel left at temperature 1.
__global__ __launch_bounds__(64) void token_prob_kernel(const float* __restrict__ logits, int V, int chunk,
                                                        int n_chunks, const float* __restrict__ ws,
                                                        const int* __restrict__ tokens, float* __restrict__ out) {
    const int lane = threadIdx.x;
    const int steps = chunk >> 6;
    const float* part = ws + (int64_t)blockIdx.x * n_chunks * (2 + steps);
    const bool have = lane < n_chunks;
    const float m_c = have ? part[(int64_t)lane * (2 + steps)] : -INFINITY;
    const float mx = wave_max(m_c);
    const float total = wave_sum(have ? part[(int64_t)lane * (2 + steps) + 1] * __builtin_amdgcn_exp2f((m_c - mx) * LOG2E_F)
                                      : 0.f);
    if (lane == 0) {
        const int t = tokens[blockIdx.x];
        out[blockIdx.x] = (t >= 0 && t < V)
            ? __builtin_amdgcn_exp2f((logits[(int64_t)blockIdx.x * V + t] - mx) * LOG2E_F) / total : 0.f;
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

// ---------------------------------------------------------------------------
// li_argmax_static: li_argmax with its partial results in an array of the library (no_alloc.h).
// In host code the array's name is only a stand-in for the symbol; its address on a device is
// asked for once per device and that pointer is what the kernels get.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[LI_ARGMAX_STATIC_BYTES];

constexpr int MAX_DEVICES = 64;
static void* scratch_ptr[MAX_DEVICES] = {};
static std::mutex scratch_mutex;

// the array's address on the current device, or null
static void* scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> guard(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
        scratch_ptr[dev] = p;
    }
    return scratch_ptr[dev];
}

extern "C" int li_argmax_static_init(void) { return scratch_of_current_device() ? LI_OK : LI_HIP_ERROR; }

extern "C" int li_argmax_static_capacity(int V) {
    return V <= 0 ? 0 : LI_ARGMAX_STATIC_ENTRIES / li_argmax_chunks(V);
}

extern "C" int li_argmax_static(const float* logits, int n_rows, int V, int* out, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (V <= 0 || !logits || !out) return LI_BAD_ARG;
    const int n_chunks = li_argmax_chunks(V);
    if ((int64_t)n_rows * n_chunks > LI_ARGMAX_STATIC_ENTRIES) return LI_UNSUPPORTED;
    unsigned char* ptr = (unsigned char*)scratch_of_current_device();
    if (!ptr) return LI_HIP_ERROR;
    // maxima in the first half of the array, indices in the second
    float* part_v = (float*)ptr;
    int* part_i = (int*)(ptr + LI_ARGMAX_STATIC_ENTRIES * 4);
    return li_argmax(logits, n_rows, V, part_v, part_i, out, stream);
}

// chunk of a row for li_sample (a multiple of 64, at most 64 chunks) and the floats of workspace a row needs
extern "C" int li_sample_chunk(int V) {
    const int chunk = V <= 64 * 4096 ? 4096 : (V + 63) / 64;
    return (min(chunk, max(V, 1)) + 63) / 64 * 64;
}
extern "C" int li_sample_ws_floats(int V) {
    const int chunk = li_sample_chunk(V);
    return ((V + chunk - 1) / chunk) * (2 + chunk / 64);
}

// temperature_dev (may be null): one float on the device that replaces `temperature`; it must be positive
extern "C" int li_sample(const float* logits, int n_rows, int V, float temperature, const float* temperature_dev,
                         const int* seq_slot, void* state, const float* forced_r, float* ws, int* out,
                         hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (V <= 0 || (!temperature_dev && temperature <= 0.f) || !ws) return LI_BAD_ARG;      // greedy goes through li_argmax
    if (!forced_r && (!seq_slot || !state)) return LI_BAD_ARG;
    const int chunk = li_sample_chunk(V), n_chunks = (V + chunk - 1) / chunk;
    sample_chunks_kernel<<<dim3(n_rows, n_chunks), 256, 0, stream>>>(logits, V, chunk, temperature, temperature_dev, ws);
    LI_CHECK_LAUNCH();
    sample_final_kernel<<<n_rows, 64, 0, stream>>>(logits, V, chunk, n_chunks, temperature, temperature_dev, ws,
                                                   seq_slot, (unsigned long long*)state, forced_r, out);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// out[r] = softmax(logits[r])[tokens[r]]; ws as for li_sample
extern "C" int li_token_prob(const float* logits, int n_rows, int V, const int* tokens, float* ws, float* out,
                             hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (V <= 0 || !logits || !tokens || !ws || !out) return LI_BAD_ARG;
    const int chunk = li_sample_chunk(V), n_chunks = (V + chunk - 1) / chunk;
    sample_chunks_kernel<<<dim3(n_rows, n_chunks), 256, 0, stream>>>(logits, V, chunk, 1.0f, nullptr, ws);
    LI_CHECK_LAUNCH();
    token_prob_kernel<<<n_rows, 64, 0, stream>>>(logits, V, chunk, n_chunks, ws, tokens, out);
    LI_CHECK_LAUNCH();
    return LI_OK;
}
