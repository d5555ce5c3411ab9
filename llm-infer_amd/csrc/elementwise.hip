// Embedding gather, RMSNorm, rotation of q/k with the write into the paged
// cache, and the per-step bookkeeping kernel of decoding.  One kernel for each,
// every size taken at run time.
#include "common.h"

// ---------------------------------------------------------------------------
// x[t, :] = float(table[token[t], :])          (src/model/model.cpp:101-118)
// ---------------------------------------------------------------------------
template <class T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                             float* __restrict__ x, int d, int vocab) {
    const int t = blockIdx.x;
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);   // ids are checked on the host; never read outside
    const T* row = table + (int64_t)tok * d;
    float* out = x + (int64_t)t * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) out[i] = to_f32(row[i]);
}

extern "C" int li_embed(const void* table, int table_dt, const int* tokens, float* x,
                        int n_tokens, int d, int vocab, hipStream_t stream) {
    if (n_tokens <= 0) return LI_OK;
    if (d <= 0 || vocab <= 0) return LI_BAD_ARG;
    dim3 grid(n_tokens), block(256);
    if (table_dt == DT_F32) embed_kernel<float><<<grid, block, 0, stream>>>((const float*)table, tokens, x, d, vocab);
    else if (table_dt == DT_F16) embed_kernel<f16><<<grid, block, 0, stream>>>((const f16*)table, tokens, x, d, vocab);
    else if (table_dt == DT_BF16) embed_kernel<bf16><<<grid, block, 0, stream>>>((const bf16*)table, tokens, x, d, vocab);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// out[r, :] = x[row(r), :] / sqrt(mean(x^2) + eps) * w     (include/kernels_cpu.hpp:43-54)
// Sum of squares, root and scaling in float32; `rows` (may be null) picks rows.
// ---------------------------------------------------------------------------
// `row_scale` (may be null): row_scale_for(rms) of the first 16 rows, for a product that will add into these
// rows and hand them on in float16 (gemm.hip, RowsOut).
template <class TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               const int* __restrict__ rows, TO* __restrict__ out, int d, float eps,
                               float* __restrict__ row_scale) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const float* xr = x + (int64_t)(rows ? rows[r] : r) * d;
    TO* o = out + (int64_t)r * d;
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) { const float v = xr[i]; ss += v * v; }
    ss = block_sum(ss, scratch);
    const float rms = sqrtf(ss / (float)d + eps);
    if (row_scale && threadIdx.x == 0 && r < 16) row_scale[r] = row_scale_for(rms);
    for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = from_f32<TO>(xr[i] / rms * w[i]);
}

// The same for rows of up to 4 * V * blockDim.x elements (d a multiple of 4, 16-byte aligned
// pointers): the row and its weights are read once, in 16-byte pieces that stay in registers.
template <class TO, int V>
__global__ void rmsnorm_vec_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                   const int* __restrict__ rows, TO* __restrict__ out, int d, float eps,
                                   float* __restrict__ row_scale) {
    struct alignas(4 * sizeof(TO)) Out4 { TO v[4]; };
    __shared__ float scratch[16];
    const int r = blockIdx.x, n4 = d >> 2;
    const f32x4* xr = (const f32x4*)(x + (int64_t)(rows ? rows[r] : r) * d);
    const f32x4* w4 = (const f32x4*)w;
    Out4* o = (Out4*)(out + (int64_t)r * d);
    f32x4 xv[V], wv[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        xv[j] = i < n4 ? xr[i] : f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        wv[j] = i < n4 ? w4[i] : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < V; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) ss += xv[j][q] * xv[j][q];
    ss = block_sum(ss, scratch);
    const float rms = sqrtf(ss / (float)d + eps);
    if (row_scale && threadIdx.x == 0 && r < 16) row_scale[r] = row_scale_for(rms);
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        if (i < n4) {
            Out4 t;
#pragma unroll
            for (int q = 0; q < 4; ++q) t.v[q] = from_f32<TO>(xv[j][q] / rms * wv[j][q]);
            o[i] = t;
        }
    }
}

extern "C" int li_rmsnorm(const float* x, const float* w, const int* rows, void* out, int out_dt,
                          int n_rows, int d, float eps, float* row_scale, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (d <= 0) return LI_BAD_ARG;
    if (out_dt != DT_F32 && out_dt != DT_F16 && out_dt != DT_BF16) return LI_BAD_ARG;
    dim3 grid(n_rows);
    const bool vec = d % 4 == 0 && d <= 8192 && !(((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15);
    if (vec) {
        const int n4 = d / 4;
        const int threads = n4 <= 64 ? 64 : (n4 <= 256 ? 128 : (n4 <= 1024 ? 256 : 512));
        const bool two = n4 <= 2 * threads;
#define GO(TO)                                                                                             \
    do {                                                                                                   \
        if (two) rmsnorm_vec_kernel<TO, 2><<<grid, threads, 0, stream>>>(x, w, rows, (TO*)out, d, eps, row_scale); \
        else rmsnorm_vec_kernel<TO, 4><<<grid, threads, 0, stream>>>(x, w, rows, (TO*)out, d, eps, row_scale);     \
    } while (0)
        if (out_dt == DT_F32) GO(float); else if (out_dt == DT_F16) GO(f16); else GO(bf16);
#undef GO
    } else {
        dim3 block(d >= 2048 ? 512 : (d >= 512 ? 256 : 64));
        if (out_dt == DT_F32) rmsnorm_kernel<float><<<grid, block, 0, stream>>>(x, w, rows, (float*)out, d, eps, row_scale);
        else if (out_dt == DT_F16) rmsnorm_kernel<f16><<<grid, block, 0, stream>>>(x, w, rows, (f16*)out, d, eps, row_scale);
        else rmsnorm_kernel<bf16><<<grid, block, 0, stream>>>(x, w, rows, (bf16*)out, d, eps, row_scale);
    }
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Rotation of q and k by position, and the write of k and v into the cache.
//   qkv   [T, row_stride] float32: q heads, then k heads, then v heads of one token
//   q_out [T, H, hd]
//   pages: k_pages/v_pages of this layer, page = page_table[slot, pos / PAGE]
// Rotation (include/kernels_cpu.hpp:82-100): pair (a, b) <- (a cos - b sin, a sin + b cos),
// angle = pos * inv_freq[j]; adjacent pairing rotates (2j, 2j+1), half pairing
// (j, j + rotary_dim/2).  Dimensions at and beyond rotary_dim pass unchanged.
// Keys are stored after the rotation (src/model/block.cpp:141-148).
// ---------------------------------------------------------------------------
template <class T>
__global__ void rope_store_kernel(const float* __restrict__ qkv, int row_stride,
                                  const float* __restrict__ inv_freq, int rotary_dim, int half_pairing,
                                  const int* __restrict__ pos, const int* __restrict__ tok_slot,
                                  const int* __restrict__ page_table, int max_pages, int64_t page_stride,
                                  T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                  int H, int K, int hd, int kv_round) {
    const int t = blockIdx.x;
    const int p = pos[t];
    const int half = hd >> 1;
    const int n_pairs = (H + 2 * K) * half;
    const float* row = qkv + (int64_t)t * row_stride;
    int64_t page = 0;
    if (K > 0) page = page_table[(int64_t)tok_slot[t] * max_pages + p / PAGE];
    const int tp = p % PAGE;
    for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
        const int head = i / half, j = i - head * half;
        int d0, d1;
        bool rotate = false;
        if (2 * j < rotary_dim) {
            rotate = true;
            if (half_pairing) { d0 = j; d1 = j + (rotary_dim >> 1); }
            else { d0 = 2 * j; d1 = 2 * j + 1; }
        } else { d0 = 2 * j; d1 = 2 * j + 1; }
        float a = row[head * hd + d0], b = row[head * hd + d1];
        if (rotate && head < H + K) {
            float s, c;
            sincosf((float)p * inv_freq[j], &s, &c);
            const float ra = a * c - b * s, rb = a * s + b * c;
            a = ra; b = rb;
        }
        if (head >= H && kv_round != DT_F32) {
            // what goes into the cache takes a 16-bit type's values on its way (block.cpp:145-148)
            if (kv_round == DT_F16) { a = (float)(f16)a; b = (float)(f16)b; }
            else { a = (float)(bf16)a; b = (float)(bf16)b; }
        }
        if (head < H) {
            T* q = q_out + ((int64_t)t * H + head) * hd;
            q[d0] = from_f32<T>(a); q[d1] = from_f32<T>(b);
        } else if (head < H + K) {
            T* kp = k_pages + page * page_stride + (int64_t)(head - H) * k_head_elems(hd);
            kp[k_offset(tp, d0, hd)] = from_f32<T>(a); kp[k_offset(tp, d1, hd)] = from_f32<T>(b);
        } else {
            T* vp = v_pages + page * page_stride + (int64_t)(head - H - K) * v_head_elems(hd);
            vp[v_offset(tp, d0, hd)] = from_f32<T>(a); vp[v_offset(tp, d1, hd)] = from_f32<T>(b);
        }
    }
}

extern "C" int li_rope_store(const float* qkv, int row_stride, const float* inv_freq, int rotary_dim,
                             int half_pairing, const int* pos, const int* tok_slot, const int* page_table,
                             int max_pages, int64_t page_stride, void* q_out, void* k_pages, void* v_pages, int dt,
                             int n_tokens, int H, int K, int hd, int kv_round, hipStream_t stream) {
    if (n_tokens <= 0) return LI_OK;
    if (kv_round < DT_F32 || kv_round > DT_BF16) return LI_BAD_ARG;
    if (hd <= 0 || (hd & 1) || H <= 0 || K < 0 || rotary_dim < 0 || rotary_dim > hd || (rotary_dim & 1) ||
        row_stride < (H + 2 * K) * hd)
        return LI_BAD_ARG;
    if (K > 0 && (hd % 16 != 0)) return LI_UNSUPPORTED;
    dim3 grid(n_tokens), block(256);
#define LAUNCH(T)                                                                                        \
    rope_store_kernel<T><<<grid, block, 0, stream>>>(qkv, row_stride, inv_freq, rotary_dim, half_pairing, \
                                                     pos, tok_slot, page_table, max_pages, page_stride, (T*)q_out, \
                                                     (T*)k_pages, (T*)v_pages, H, K, hd, kv_round)
    if (dt == DT_F32) LAUNCH(float);
    else if (dt == DT_F16) LAUNCH(f16);
    else if (dt == DT_BF16) LAUNCH(bf16);
    else return LI_BAD_ARG;
#undef LAUNCH
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// cos and sin of pos[t] * inv_freq[j] for the tokens of a step: [T, n_freq, 2] float32.  The angles
// are the same in every layer, so a step computes them once.
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, const int* __restrict__ pos,
                                  float* __restrict__ out, int n_tokens, int n_freq) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_tokens * n_freq) return;
    const int t = i / n_freq, j = i - t * n_freq;
    float s, c;
    sincosf((float)pos[t] * inv_freq[j], &s, &c);
    out[2 * i] = c;
    out[2 * i + 1] = s;
}

extern "C" int li_rope_table(const float* inv_freq, const int* pos, float* out, int n_tokens, int n_freq,
                             hipStream_t stream) {
    if (n_tokens <= 0 || n_freq <= 0) return LI_OK;
    const int n = n_tokens * n_freq;
    rope_table_kernel<<<(n + 255) / 256, 256, 0, stream>>>(inv_freq, pos, out, n_tokens, n_freq);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Bookkeeping of one decode step, on the device so that a captured step can be
// replayed: each sequence's new token gets the position lens[slot], the
// sequence's context grows by one.  A row on `scratch_slot` is an idle row of a
// step that runs more rows than there are live sequences: position 0, a context
// of one token, and no length is changed.  With `cos_sin` (may be null) the same
// kernel fills the table of rotation angles of the step, [n, n_freq, 2] = cos and
// sin of pos * inv_freq as rope_table_kernel does, so that a step needs no
// second small kernel before its first layer.
// ---------------------------------------------------------------------------
__global__ void decode_prepare_kernel(const int* __restrict__ seq_slot, int* __restrict__ lens,
                                      int* __restrict__ pos, int* __restrict__ ctx, int n, int scratch_slot,
                                      const float* __restrict__ inv_freq, float* __restrict__ cos_sin, int n_freq) {
    // one workgroup a row: thread 0 does the bookkeeping, all threads the row's angles
    const int i = blockIdx.x;
    const int s = seq_slot[i];
    const int l = s == scratch_slot ? 0 : lens[s];
    __syncthreads();                                  // every thread has read the length before it changes
    if (threadIdx.x == 0) {
        pos[i] = l;
        ctx[i] = l + 1;
        if (s != scratch_slot) lens[s] = l + 1;
    }
    if (cos_sin)
        for (int j = threadIdx.x; j < n_freq; j += blockDim.x) {
            float sn, cs;
            sincosf((float)l * inv_freq[j], &sn, &cs);
            cos_sin[2 * ((int64_t)i * n_freq + j)] = cs;
            cos_sin[2 * ((int64_t)i * n_freq + j) + 1] = sn;
        }
}

extern "C" int li_decode_prepare(const int* seq_slot, int* lens, int* pos, int* ctx, int n, int scratch_slot,
                                 const float* inv_freq, float* cos_sin, int n_freq, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (cos_sin && (!inv_freq || n_freq <= 0)) return LI_BAD_ARG;
    decode_prepare_kernel<<<n, 64, 0, stream>>>(seq_slot, lens, pos, ctx, n, scratch_slot, inv_freq, cos_sin, n_freq);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// out[i] = act(gate[i]) * up[i] for separate gate and up rows:  gu [T, 2F] float32 with
// gate_j at column 2j and up_j at column 2j+1  ->  h [T, F].  (src/model/block.cpp:203-214)
// act: gate_activation of common.h (silu, or the reference's gelu).
template <class T>
__global__ void swiglu_kernel(const float* __restrict__ gu, T* __restrict__ h, int64_t n, int gelu) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float g = gu[2 * i], u = gu[2 * i + 1];
    h[i] = from_f32<T>(gate_activation(g, gelu != 0) * u);
}

extern "C" int li_swiglu(const float* gu, void* h, int dt, int64_t n, int gelu, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (dt == DT_F32) swiglu_kernel<float><<<grid, block, 0, stream>>>(gu, (float*)h, n, gelu);
    else if (dt == DT_F16) swiglu_kernel<f16><<<grid, block, 0, stream>>>(gu, (f16*)h, n, gelu);
    else if (dt == DT_BF16) swiglu_kernel<bf16><<<grid, block, 0, stream>>>(gu, (bf16*)h, n, gelu);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    return LI_OK;
}
