// Shared by the matrix-product sources: the epilogues, the tiled-weight layout and the split-K
// reduction.  (Included by gemm.hip and gemm_prefill.hip; every kernel here is static or inline.)
#pragma once
#include "common.h"

enum { EPI_STORE = 0, EPI_ADD = 1, EPI_SWIGLU = 2, EPI_ROPE = 3, EPI_GEGLU = 4 };

// What the EPI_ROPE epilogue needs: the columns of the product are the q heads, then the k heads,
// then the v heads of a token; q and k are rotated by the token's position (adjacent pairs), q goes
// to q_out [M, H, hd], k and v into the token's cache page.
struct RopeStore {
    const float* inv_freq;      // [rotary_dim / 2]
    const float* cos_sin;       // [M, rotary_dim / 2, 2] cos and sin of pos * inv_freq, or null
    const int* pos;             // [M] position of each row
    const int* tok_slot;        // [M] cache slot of each row
    const int* page_table;      // [slots, max_pages]
    void* q_out;
    void* k_pages;
    void* v_pages;
    int64_t page_stride;
    int rotary_dim, H, K, hd, max_pages, dt;   // dt: DT_* of q_out and the cache
};

struct Epilogue {
    void* C;        // output (unused by EPI_ROPE)
    int mode;       // EPI_*
    int out_dt;     // DT_* of C (EPI_ADD: always float32)
    int M, N;
    RopeStore rs;
};

__device__ __forceinline__ void store_one(void* C, int dt, int64_t i, float v) {
    if (dt == DT_F32) ((float*)C)[i] = v;
    else if (dt == DT_F16) ((f16*)C)[i] = (f16)v;
    else ((bf16*)C)[i] = (bf16)v;
}

// Offset of W[n, k] in the tiled order of a weight matrix (see "Tiled weights" in gemm.hip).
__host__ __device__ __forceinline__ int64_t tiled_offset(int n, int k, int K) {
    return ((((int64_t)(n >> 4) * (K >> 5) + (k >> 5)) * 64) + (((k & 31) >> 3) << 4) + (n & 15)) * 8 + (k & 7);
}

// Four consecutive elements, the first index a multiple of 4 (one aligned store).
__device__ __forceinline__ void store_four(void* C, int dt, int64_t i, const float* v) {
    if (dt == DT_F32) *(f32x4*)((float*)C + i) = f32x4{v[0], v[1], v[2], v[3]};
    else if (dt == DT_F16) *(f16x4*)((f16*)C + i) = f16x4{(f16)v[0], (f16)v[1], (f16)v[2], (f16)v[3]};
    else *(bf16x4*)((bf16*)C + i) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
}

// The EPI_ROPE epilogue in two parts, so that a kernel can fetch what it reads from memory early:
// rope_angles gives cos and sin for the pairs at d and d + 2 of a head (row m at position p), and
// rope_store4 rotates and stores.  include/kernels_cpu.hpp:82-100 and src/model/block.cpp:141-148, on
// the accumulators.  `page`: the page of the row's cache slot that holds position p (k and v heads).
__device__ __forceinline__ void rope_angles(const RopeStore& r, int m, int p, int head, int d, f32x2 (&t)[2],
                                            bool table = false) {          // table: r.cos_sin is there
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        t[j] = f32x2{1.f, 0.f};
        if (head < r.H + r.K && d + 2 * j < r.rotary_dim) {
            if (table || r.cos_sin) t[j] = *(const f32x2*)(r.cos_sin + ((int64_t)m * (r.rotary_dim >> 1) + ((d + 2 * j) >> 1)) * 2);
            else {
                float sn, cs;
                sincosf((float)p * r.inv_freq[(d + 2 * j) >> 1], &sn, &cs);
                t[j] = f32x2{cs, sn};
            }
        }
    }
}

__device__ __forceinline__ void rope_store4(const RopeStore& r, int m, int head, int d, const float* v, int p,
                                            int64_t page, const f32x2 (&t)[2]) {
    float o[4] = {v[0], v[1], v[2], v[3]};
    if (head < r.H + r.K) {
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            if (d + j < r.rotary_dim) {
                const float cs = t[j >> 1][0], sn = t[j >> 1][1];
                o[j] = v[j] * cs - v[j + 1] * sn;
                o[j + 1] = v[j] * sn + v[j + 1] * cs;
            }
        }
    }
    if (head < r.H) {
        store_four(r.q_out, r.dt, ((int64_t)m * r.H + head) * r.hd + d, o);
        return;
    }
    const int tp = p % PAGE;
    if (head < r.H + r.K) {
        // four consecutive d of a key are consecutive in the page
        store_four(r.k_pages, r.dt, page * r.page_stride + (int64_t)(head - r.H) * k_head_elems(r.hd) + k_offset(tp, d, r.hd), o);
    } else {
        const int64_t at = page * r.page_stride + (int64_t)(head - r.H - r.K) * v_head_elems(r.hd);
#pragma unroll
        for (int j = 0; j < 4; ++j) store_one(r.v_pages, r.dt, at + v_offset(tp, d + j, r.hd), o[j]);
    }
}

// v[0..3] are the results for row m and columns n..n+3 (n a multiple of 4).
__device__ __forceinline__ void epilogue4(const Epilogue& e, int m, int n, const float* v) {
    if (m >= e.M || n >= e.N) return;
    if (e.mode == EPI_ROPE) {
        const RopeStore& r = e.rs;
        const int head = n / r.hd, d = n - head * r.hd;       // the 4 columns lie in one head (hd % 16 == 0)
        const int p = r.pos[m];
        f32x2 t[2];
        rope_angles(r, m, p, head, d, t);
        const int64_t page = head < r.H ? 0 : r.page_table[(int64_t)r.tok_slot[m] * r.max_pages + p / PAGE];
        rope_store4(r, m, head, d, v, p, page, t);
        return;
    }
    if (e.mode == EPI_SWIGLU || e.mode == EPI_GEGLU) {
        // columns 2j (gate) and 2j+1 (up) give h[m, j] = act(gate) * up   (src/model/block.cpp:203-214)
        const int64_t row = (int64_t)m * (e.N >> 1);
        if (n + 3 < e.N && (e.N & 3) == 0) {
            // both values of the quad in one store (the pair's index is even, and so is N / 2)
            const float h0 = gate_activation(v[0], e.mode == EPI_GEGLU) * v[1];
            const float h1 = gate_activation(v[2], e.mode == EPI_GEGLU) * v[3];
            const int64_t at = row + (n >> 1);
            if (e.out_dt == DT_F32) *(f32x2*)((float*)e.C + at) = f32x2{h0, h1};
            else if (e.out_dt == DT_F16) *(f16x2*)((f16*)e.C + at) = f16x2{(f16)h0, (f16)h1};
            else *(bf16x2*)((bf16*)e.C + at) = bf16x2{(bf16)h0, (bf16)h1};
            return;
        }
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            if (n + j + 1 < e.N) {
                const float g = v[j], u = v[j + 1];
                store_one(e.C, e.out_dt, row + ((n + j) >> 1), gate_activation(g, e.mode == EPI_GEGLU) * u);
            }
        }
        return;
    }
    const int64_t base = (int64_t)m * e.N + n;
    const bool full = (n + 3 < e.N) && ((e.N & 3) == 0);
    if (e.mode == EPI_ADD) {
        float* c = (float*)e.C + base;
        if (full) {
            f32x4 o = *(f32x4*)c;
            o[0] += v[0]; o[1] += v[1]; o[2] += v[2]; o[3] += v[3];
            *(f32x4*)c = o;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) if (n + j < e.N) c[j] += v[j];
        }
        return;
    }
    if (full && e.out_dt == DT_F32) {
        f32x4 o = {v[0], v[1], v[2], v[3]};
        *(f32x4*)((float*)e.C + base) = o;
    } else if (full && e.out_dt == DT_F16) {
        f16x4 o = {(f16)v[0], (f16)v[1], (f16)v[2], (f16)v[3]};
        *(f16x4*)((f16*)e.C + base) = o;
    } else if (full && e.out_dt == DT_BF16) {
        bf16x4 o = {(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
        *(bf16x4*)((bf16*)e.C + base) = o;
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) if (n + j < e.N) store_one(e.C, e.out_dt, base + j, v[j]);
    }
}


// Sum of the split-K partials in ascending split order, then the epilogue.
static __global__ void splitk_reduce_kernel(const float* __restrict__ ws, int splits, Epilogue e) {
    const int64_t quads_per_row = (e.N + 3) >> 2;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= quads_per_row * e.M) return;
    const int m = (int)(i / quads_per_row), n = (int)(i % quads_per_row) * 4;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    const int64_t stride = (int64_t)e.M * e.N;
    const float* p = ws + (int64_t)m * e.N + n;
    if (n + 3 < e.N && (e.N & 3) == 0) {
        // four splits' loads in flight at a time; the sums stay in ascending split order
        int s = 0;
        for (; s + 4 <= splits; s += 4) {
            f32x4 t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = *(const f32x4*)(p + (s + u) * stride);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] += t[u][q];
        }
        for (; s < splits; ++s) {
            const f32x4 t = *(const f32x4*)(p + s * stride);
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] += t[q];
        }
    } else {
        for (int s = 0; s < splits; ++s)
#pragma unroll
            for (int q = 0; q < 4; ++q) if (n + q < e.N) v[q] += p[s * stride + q];
    }
    epilogue4(e, m, n, v);
}


// A norm split over two products of a decode step (up to 16 rows), so that no norm kernel runs between
// them.  The product that adds into the residual stream (EPI_ADD) also leaves, for the rows x it has
// just completed, (a) the sums of squares as one partial sum per workgroup and row, `ss` [blocks, 16], and
// (b) x * w * scale rounded to the 16-bit type, `xw` [M, N], w being the weight of the norm that reads
// x next (RowsOut).  The next product takes `xw` as its X and multiplies its sums by
// 1 / (scale * sqrt(mean(x^2) + eps)) from the partial sums (RowScale; gemv_tiled, and gemm_wreg's kernel of every epilogue): together  W . (x / rms * w),
// the norm of include/kernels_cpu.hpp:43-54 in another order of rounding.  `scale` keeps x * w inside
// float16's range: one power of two for each row, near 1 / (8 rms) of the row as it was when a norm was last
// taken of it (`row_scale`, written by the norm kernel or by the product that finished that norm:
// row_scale_for in common.h), so that the rounding is as fine for a model whose residual stream is of the
// order of 0.01 or 1000 as for one of the order of 1; without it the fixed `scale`.
struct RowsOut {
    float* ss;               // [gridDim.x, 16]
    void* xw;                // [M, N] in the product's 16-bit type
    const float* w;          // [N] weight of the next norm
    float scale;
    const float* row_scale;  // [16] or null
};
struct RowScale {
    const float* ss;         // [P, 16]
    int P;
    float eps;               // of the norm
    float inv_scale;         // 1 / RowsOut.scale
    const float* row_scale;  // [16] the scales RowsOut used, or null (then inv_scale)
    float* next_scale;       // [16] or null: row_scale_for(rms) of these rows, for the product that adds into them next
};

// The RMS norm that reads the rows of a residual sum next (src/model/block.cpp:127, 191): weight [N], eps, and
// where its result goes ([M, N] of out_dt).
struct NormAfter {
    const float* w;
    void* out;
    int out_dt;
    float eps;
};

// For C += X W^T with K split: the sum of the partials (ascending split order, as splitk_reduce_kernel), the
// residual sum, and the norm of the finished row, a workgroup a row.  The norm is rmsnorm_vec_kernel's, value for
// value: same pieces per thread, same order of the sum of squares, same expression.  N a multiple of 4, at most
// 4 V blockDim.x; pointers 16-byte aligned.
template <class TO, int V>
static __global__ void splitk_add_norm_kernel(const float* __restrict__ ws, int splits, float* __restrict__ C,
                                              int M, int N, const float* __restrict__ w, TO* __restrict__ out,
                                              float eps) {
    struct alignas(4 * sizeof(TO)) Out4 { TO v[4]; };
    __shared__ float scratch[16];
    const int r = blockIdx.x, n4 = N >> 2;
    f32x4* xr = (f32x4*)(C + (int64_t)r * N);
    const f32x4* w4 = (const f32x4*)w;
    Out4* o = (Out4*)(out + (int64_t)r * N);
    const int64_t stride4 = (int64_t)M * n4;
    f32x4 xv[V], wv[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        xv[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (i < n4) {
            const f32x4* p = (const f32x4*)ws + (int64_t)r * n4 + i;
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            f32x4 c = xr[i];
            // four splits' loads in flight at a time; the sums stay in ascending split order
            int s = 0;
            for (; s + 4 <= splits; s += 4) {
                f32x4 t[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) t[u] = p[(s + u) * stride4];
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int q = 0; q < 4; ++q) v[q] += t[u][q];
            }
            for (; s < splits; ++s) {
                const f32x4 t = p[s * stride4];
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] += t[q];
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) c[q] += v[q];
            xr[i] = c;
            xv[j] = c;
        }
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
    const float rms = sqrtf(ss / (float)N + eps);
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

// Whether splitk_add_norm_kernel can stand for splitk_reduce_kernel + the norm kernel.
static bool norm_after_fits(const NormAfter* na, const Epilogue& e, const float* ws) {
    return na && na->w && na->out && e.mode == EPI_ADD && e.N % 4 == 0 && e.N <= 8192 &&
           (na->out_dt == DT_F16 || na->out_dt == DT_BF16 || na->out_dt == DT_F32) &&
           !(((uintptr_t)ws | (uintptr_t)e.C | (uintptr_t)na->w | (uintptr_t)na->out) & 15);
}

static void launch_splitk_add_norm(const float* ws, int splits, const Epilogue& e, const NormAfter* na,
                                   hipStream_t stream) {
    // threads and pieces per thread as li_rmsnorm chooses them
    const int n4 = e.N / 4;
    const int threads = n4 <= 64 ? 64 : (n4 <= 256 ? 128 : (n4 <= 1024 ? 256 : 512));
    const bool two = n4 <= 2 * threads;
#define GO(TO)                                                                                                  \
    do {                                                                                                        \
        if (two) splitk_add_norm_kernel<TO, 2><<<e.M, threads, 0, stream>>>(ws, splits, (float*)e.C, e.M, e.N, na->w, (TO*)na->out, na->eps); \
        else splitk_add_norm_kernel<TO, 4><<<e.M, threads, 0, stream>>>(ws, splits, (float*)e.C, e.M, e.N, na->w, (TO*)na->out, na->eps);     \
    } while (0)
    if (na->out_dt == DT_F32) GO(float); else if (na->out_dt == DT_F16) GO(f16); else GO(bf16);
#undef GO
}

static int make_epilogue(Epilogue& e, void* C, int mode, int out_dt, int M, int N, const RopeStore* rs) {
    e.C = C; e.mode = mode; e.out_dt = out_dt; e.M = M; e.N = N;
    e.rs = RopeStore{};
    if (mode != EPI_ROPE) return LI_OK;
    if (!rs || !rs->pos || !rs->q_out || rs->hd <= 0 || rs->hd % 16 != 0 || rs->H <= 0 || rs->K < 0) return LI_BAD_ARG;
    if (N != (rs->H + 2 * rs->K) * rs->hd || rs->rotary_dim < 0 || rs->rotary_dim > rs->hd || (rs->rotary_dim & 1))
        return LI_BAD_ARG;
    if (rs->rotary_dim > 0 && !rs->inv_freq && !rs->cos_sin) return LI_BAD_ARG;
    if (rs->K > 0 && (!rs->tok_slot || !rs->page_table || !rs->k_pages || !rs->v_pages)) return LI_BAD_ARG;
    if (rs->dt < DT_F32 || rs->dt > DT_BF16) return LI_BAD_ARG;
    e.rs = *rs;
    return LI_OK;
}

static int check_common(const void* X, const void* W, const void* C, int M, int N, int K, int mode, int out_dt) {
    if (!X || !W || (!C && mode != EPI_ROPE) || M < 0 || N <= 0 || K <= 0) return LI_BAD_ARG;
    if (mode < EPI_STORE || mode > EPI_GEGLU) return LI_BAD_ARG;
    if (out_dt < DT_F32 || out_dt > DT_BF16) return LI_BAD_ARG;
    if (mode == EPI_ADD && out_dt != DT_F32) return LI_BAD_ARG;
    if ((mode == EPI_SWIGLU || mode == EPI_GEGLU) && (N & 1)) return LI_BAD_ARG;
    return LI_OK;
}

