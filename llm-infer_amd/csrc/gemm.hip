// Matrix products  C[M, N] = X[M, K] . W[N, K]^T  (both operands contiguous in K,
// the layout of the reference's matmul, include/kernels_cpu.hpp:69-80), with the
// epilogue fused (gemm_common.h): plain store, add into the float32 residual, SwiGLU on
// interleaved gate/up columns, or rotation and cache write.  This file: the products of
// decode and of short prompts, and the fallbacks; gemm_prefill.hip has the large ones.
//
//   gemm_fma    any element types and any sizes; float32 multiply-add in ascending k
//               for every output, so an output does not depend on its place in the batch.
//               It is the true 32-bit path and the fallback for K not a multiple of 8.
//   gemm_mfma   16-bit operands on the matrix cores (32x32x16), tiles staged through
//               LDS, optional split over K into a float32 workspace.
//   gemv_mfma   up to 16 rows of X (row-major W), gemv_tiled up to 64 rows (tiled W): W is
//               streamed once from HBM straight into the matrix cores' operand registers.
#include "gemm_common.h"

// ===========================================================================
// gemm_fma: 64x64 tile, 256 threads, 4x4 outputs a thread, k ascending.
// ===========================================================================
template <class TX, class TW>
__global__ __launch_bounds__(256) void gemm_fma_kernel(const TX* __restrict__ X, const TW* __restrict__ W,
                                                       int K, Epilogue e) {
    constexpr int BT = 64, BK = 16;
    __shared__ float sX[BK][BT + 4];
    __shared__ float sW[BK][BT + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * BT, n0 = blockIdx.x * BT;
    // Every sum is taken in the same order whatever the batch: FMA chains over 256 consecutive k, the
    // chains added up in ascending order (a single chain over a K of tens of thousands would lose
    // several bits more than a blocked library product does).
    float acc[4][4] = {}, total[4][4] = {};
    const int lr = tid >> 2, lk = (tid & 3) * 4;     // row of the tile and first k this thread loads
    for (int k0 = 0; k0 < K; k0 += BK) {
        if (k0 && (k0 & 255) == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) { total[i][j] += acc[i][j]; acc[i][j] = 0.f; }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            const int m = m0 + lr, n = n0 + lr;
            sX[lk + j][lr] = (m < e.M && k < K) ? to_f32(X[(int64_t)m * K + k]) : 0.f;
            sW[lk + j][lr] = (n < e.N && k < K) ? to_f32(W[(int64_t)n * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = sX[k][ty * 4 + i]; b[i] = sW[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) total[i][j] += acc[i][j];
        epilogue4(e, m0 + ty * 4 + i, n0 + tx * 4, total[i]);
    }
}

// ===========================================================================
// gemm_mfma: BN rows of W x BM rows of X per workgroup of 4 waves, BK = 64.
// W is operand A of the matrix instruction (its rows are the instruction's rows),
// X operand B, so that a lane ends with 4 consecutive columns n of one row m:
// accumulator r of a 32x32 block is n = 8*(r/4) + 4*(lane/32) + r%4, m = lane%32.
// ===========================================================================
template <class T, int BN, int BM, int WN, int WM, bool TILED>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                        int K, int k_per_split, float* __restrict__ ws,
                                                        Epilogue e) {
    typedef typename Vec<T>::v8 v8;
    constexpr int BK = 64, LD = BK + 8;
    constexpr int TN = BN / WN, TM = BM / WM;            // wave tile
    constexpr int NB = TN / 32, MB = TM / 32;            // 32x32 blocks of a wave
    constexpr int W_CHUNKS = BN * BK / 8 / 256, X_CHUNKS = BM * BK / 8 / 256;
    static_assert(WN * WM == 4 && TN % 32 == 0 && TM % 32 == 0, "tile");
    static_assert(W_CHUNKS >= 1 && X_CHUNKS >= 1, "tile too small for 256 threads");
    __shared__ __attribute__((aligned(16))) T sW[BN * LD];
    __shared__ __attribute__((aligned(16))) T sX[BM * LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, wm = wave / WN;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
    const int k_begin = blockIdx.z * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);

    f32x16 acc[NB][MB];
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

    v8 rw[W_CHUNKS], rx[X_CHUNKS];
    const int n_padded = (e.N + 15) & ~15;
    auto load_tile = [&](int k0) {
#pragma unroll
        for (int c = 0; c < W_CHUNKS; ++c) {
            const int chunk = tid + c * 256;
            // row-major: 8 threads a row; tiled: 64 threads a (16 rows x 32 k) block, as it lies in memory
            const int row = TILED ? ((chunk >> 7) << 4) + (chunk & 15) : chunk >> 3;
            const int kc = TILED ? (((chunk >> 6) & 1) << 5) + (((chunk >> 4) & 3) << 3) : (chunk & 7) * 8;
            const int n = n0 + row, k = k0 + kc;
            v8 z = {};
            if (TILED) rw[c] = (n < n_padded && k < k_end) ? *(const v8*)(W + tiled_offset(n, k, K)) : z;
            else rw[c] = (n < e.N && k < k_end) ? *(const v8*)(W + (int64_t)n * K + k) : z;
        }
#pragma unroll
        for (int c = 0; c < X_CHUNKS; ++c) {
            const int chunk = tid + c * 256, row = chunk >> 3, kc = (chunk & 7) * 8;
            const int m = m0 + row, k = k0 + kc;
            v8 z = {};
            rx[c] = (m < e.M && k < k_end) ? *(const v8*)(X + (int64_t)m * K + k) : z;
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int c = 0; c < W_CHUNKS; ++c) {
            const int chunk = tid + c * 256;
            const int row = TILED ? ((chunk >> 7) << 4) + (chunk & 15) : chunk >> 3;
            const int kc = TILED ? (((chunk >> 6) & 1) << 5) + (((chunk >> 4) & 3) << 3) : (chunk & 7) * 8;
            *(v8*)(sW + row * LD + kc) = rw[c];
        }
#pragma unroll
        for (int c = 0; c < X_CHUNKS; ++c) {
            const int chunk = tid + c * 256, row = chunk >> 3, kc = (chunk & 7) * 8;
            *(v8*)(sX + row * LD + kc) = rx[c];
        }
    };

    if (k_begin < k_end) {
        load_tile(k_begin);
        store_tile();
        __syncthreads();
        for (int k0 = k_begin; k0 < k_end; k0 += BK) {
            const bool more = k0 + BK < k_end;
            if (more) load_tile(k0 + BK);
#pragma unroll
            for (int ks = 0; ks < BK; ks += 16) {
                v8 a[NB], b[MB];
                const int kk = ks + 8 * (lane >> 5);
#pragma unroll
                for (int i = 0; i < NB; ++i) a[i] = *(const v8*)(sW + (wn * TN + i * 32 + (lane & 31)) * LD + kk);
#pragma unroll
                for (int j = 0; j < MB; ++j) b[j] = *(const v8*)(sX + (wm * TM + j * 32 + (lane & 31)) * LD + kk);
#pragma unroll
                for (int i = 0; i < NB; ++i)
#pragma unroll
                    for (int j = 0; j < MB; ++j) acc[i][j] = mfma32(a[i], b[j], acc[i][j]);
            }
            __syncthreads();
            if (more) { store_tile(); __syncthreads(); }
        }
    }

    const bool split = gridDim.z > 1;
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < MB; ++j) {
            const int m = m0 + wm * TM + j * 32 + (lane & 31);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * TN + i * 32 + 8 * g + 4 * (lane >> 5);
                float v[4] = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                if (!split) epilogue4(e, m, n, v);
                else if (m < e.M) {
                    float* p = ws + ((int64_t)blockIdx.z * e.M + m) * e.N + n;
#pragma unroll
                    for (int q = 0; q < 4; ++q) if (n + q < e.N) p[q] = v[q];
                }
            }
        }
}

// ===========================================================================
// gemv_mfma: up to 16 rows of X on the matrix cores (16x16x32), W streamed from
// global memory straight into operand A.  A wave owns NT tiles of 16 rows of W
// and one slice of K; the KW waves of a workgroup cover K and their partial
// tiles are summed through LDS in wave order.  A lane (row r = lane%16, group
// g = lane/16) loads 32 contiguous bytes of its row per 64 elements of K, so
// two back-to-back loads of a wave fetch whole 128-byte lines; X uses the same
// assignment of k to lanes, which the sum over k does not care about.
// ===========================================================================
__device__ __forceinline__ f32x4 mfma16(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

template <class T, int NT, int KW>
__global__ __launch_bounds__(64 * KW) void gemv_mfma_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                            int K, Epilogue e) {
    typedef typename Vec<T>::v8 v8;
    constexpr int U = 4;                                  // 64-element steps of K in flight
    __shared__ float part[KW][NT][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (16 * NT);
    const int steps = (K + 63) >> 6;
    const int per = (steps + KW - 1) / KW;
    const int s_begin = wave * per, s_end = min(steps, s_begin + per);
    const T* wrow[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) wrow[t] = W + (int64_t)min(n0 + 16 * t + r, e.N - 1) * K + 16 * g;
    const bool have_x = r < e.M;
    const T* xrow = X + (int64_t)(have_x ? r : 0) * K + 16 * g;
    f32x4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int s0 = s_begin; s0 < s_end; s0 += U) {
        v8 a[U][NT][2], b[U][2];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = (s0 + u) * 64;                  // this lane reads k + 16 g .. + 15
            const bool in0 = (s0 + u < s_end) && (k + 16 * g < K);
            const bool in1 = (s0 + u < s_end) && (k + 16 * g + 8 < K);
            const v8 z = {};
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                a[u][t][0] = in0 ? *(const v8*)(wrow[t] + k) : z;
                a[u][t][1] = in1 ? *(const v8*)(wrow[t] + k + 8) : z;
            }
            b[u][0] = (in0 && have_x) ? *(const v8*)(xrow + k) : z;
            b[u][1] = (in1 && have_x) ? *(const v8*)(xrow + k + 8) : z;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                acc[t] = mfma16(a[u][t][0], b[u][0], acc[t]);
                acc[t] = mfma16(a[u][t][1], b[u][1], acc[t]);
            }
    }
    if (KW > 1) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) part[wave][t][lane][q] = acc[t][q];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float v = part[0][t][lane][q];
                for (int w = 1; w < KW; ++w) v += part[w][t][lane][q];
                acc[t][q] = v;
            }
    }
    // accumulator q of a 16x16 tile: row of W n = 4 * (lane / 16) + q, row of X m = lane % 16
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        float v[4] = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
        epilogue4(e, r, n0 + 16 * t + 4 * g, v);
    }
}


// ===========================================================================
// Tiled weights.  A matrix W[N, K] (K a multiple of 32) may be kept in the order in
// which the 16x16x32 matrix instruction takes operand A:
//   [tile = n / 16][step = k / 32][lane = 16 * ((k % 32) / 8) + n % 16][k % 8]
// (rows padded to a multiple of 16).  A wave then reads each operand as one
// contiguous 1 KiB load.  gemv_tiled is gemv_mfma on that layout.
// ===========================================================================
template <class T>
__global__ void tile_weight_kernel(const T* __restrict__ W, T* __restrict__ out, int N, int K, int64_t total) {
    // one thread per 8 elements of the output
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int lane = (int)(i & 63);
    const int64_t blk = i >> 6;
    const int steps = K >> 5;
    const int step = (int)(blk % steps);
    const int tile = (int)(blk / steps);
    const int n = tile * 16 + (lane & 15), k = step * 32 + (lane >> 4) * 8;
    typedef typename Vec<T>::v8 v8;
    v8 z = {};
    *(v8*)(out + i * 8) = n < N ? *(const v8*)(W + (int64_t)n * K + k) : z;
}

template <class T, int NT, int MT, int KW>
__global__ __launch_bounds__(64 * KW) void gemv_tiled_kernel(const T* __restrict__ X, const T* __restrict__ Wt,
                                                             int K, Epilogue e, RowsOut ro, RowScale rsc) {
    // NT tiles of 16 rows of W and MT tiles of 16 rows of X per wave; W comes from HBM once, the
    // rows of X from the caches (they are few)
    typedef typename Vec<T>::v8 v8;
    constexpr int U = (NT + MT) <= 2 ? 8 : ((NT + MT) <= 4 ? 4 : 2);   // 32-element steps of K in flight
    __shared__ float part[KW][NT * MT][64][4];
    __shared__ float ss_wave[KW][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int tile0 = blockIdx.x * NT;
    const int n_tiles = (e.N + 15) >> 4;
    const int steps = K >> 5;
    const int per = (steps + KW - 1) / KW;
    const int s_begin = wave * per, s_end = min(steps, s_begin + per);
    const T* wt[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) wt[t] = Wt + ((int64_t)min(tile0 + t, n_tiles - 1) * steps * 64 + lane) * 8;
    bool have_x[MT];
    const T* xrow[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) {
        have_x[j] = 16 * j + r < e.M;
        xrow[j] = X + (int64_t)(have_x[j] ? 16 * j + r : 0) * K + 8 * g;
    }
    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < MT; ++j) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    // RowScale (rows 0..15 only): the partial sums of squares of row r are dealt to the waves, and within a
    // wave to the four lanes of the row; the loads are issued here and used after the main loop
    float ss_mine = 0.f;
    if (MT == 1 && rsc.ss) {
        // partial sum p of row r lies at ss[p * 16 + r]: the 16 lanes of a group read 64 contiguous bytes
        const float* p = rsc.ss + r;
        const int share = (rsc.P + 4 * KW - 1) / (4 * KW);
        const int lo = (wave * 4 + g) * share, hi = min(rsc.P, lo + share);
        for (int i = lo; i < hi; i += 8) {
            float v[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) v[c] = p[min(i + c, hi - 1) * 16];
#pragma unroll
            for (int c = 0; c < 8; ++c) ss_mine += (i + c < hi) ? v[c] : 0.f;
        }
    }
    for (int s0 = s_begin; s0 < s_end; s0 += U) {
        v8 a[U][NT], b[U][MT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool in = s0 + u < s_end;
            const v8 z = {};
#pragma unroll
            for (int t = 0; t < NT; ++t) a[u][t] = in ? *(const v8*)(wt[t] + (int64_t)(s0 + u) * 512) : z;
#pragma unroll
            for (int j = 0; j < MT; ++j) b[u][j] = (in && have_x[j]) ? *(const v8*)(xrow[j] + (s0 + u) * 32) : z;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int j = 0; j < MT; ++j) acc[t][j] = mfma16(a[u][t], b[u][j], acc[t][j]);
    }
    if (MT == 1 && rsc.ss) {
        ss_mine += __shfl_xor(ss_mine, 16, WAVE);
        ss_mine += __shfl_xor(ss_mine, 32, WAVE);
        if (g == 0) ss_wave[wave][r] = ss_mine;
    }
    if (KW > 1) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int j = 0; j < MT; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) part[wave][t * MT + j][lane][q] = acc[t][j][q];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int j = 0; j < MT; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float v = part[0][t * MT + j][lane][q];
                    for (int w = 1; w < KW; ++w) v += part[w][t * MT + j][lane][q];
                    acc[t][j][q] = v;
                }
    }
    if (MT == 1 && rsc.ss) {
        // this lane's row: the waves' sums in wave order, then 1 / (scale * rms)
        float ss = ss_wave[0][r];
        for (int w = 1; w < KW; ++w) ss += ss_wave[w][r];
        const float rms = sqrtf(ss / (float)K + rsc.eps);
        const float f = (rsc.row_scale ? 1.f / rsc.row_scale[r] : rsc.inv_scale) / rms;
        if (rsc.next_scale && blockIdx.x == 0 && g == 0) rsc.next_scale[r] = row_scale_for(rms);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[t][0][q] *= f;
    }
    if (ro.ss) {
        // EPI_ADD, and what RowsOut asks for (the host has checked: N a multiple of 4, at most 16 rows)
        float sq[MT];
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            sq[j] = 0.f;
            const int m = 16 * j + r;
            const float scale = ro.row_scale ? ro.row_scale[m & 15] : ro.scale;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int n = (tile0 + t) * 16 + 4 * g;
                if (m < e.M && n < e.N) {
                    float* c = (float*)e.C + (int64_t)m * e.N + n;
                    f32x4 o = *(f32x4*)c;
                    const f32x4 wv = *(const f32x4*)(ro.w + n);
                    typename Vec<T>::v4 xw;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        o[q] += acc[t][j][q];
                        sq[j] = fmaf(o[q], o[q], sq[j]);
                        xw[q] = from_f32<T>(o[q] * wv[q] * scale);
                    }
                    *(f32x4*)c = o;
                    *(typename Vec<T>::v4*)((T*)ro.xw + (int64_t)m * e.N + n) = xw;
                }
            }
            sq[j] += __shfl_xor(sq[j], 16, WAVE);
            sq[j] += __shfl_xor(sq[j], 32, WAVE);
            if (g == 0) ro.ss[(int64_t)blockIdx.x * 16 + m] = sq[j];      // (rows beyond M: zeros)
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            float v[4] = {acc[t][j][0], acc[t][j][1], acc[t][j][2], acc[t][j][3]};
            epilogue4(e, 16 * j + r, (tile0 + t) * 16 + 4 * g, v);
        }
}

// ===========================================================================
// gemm_rows: the products of 17 to 128 rows of X against a tiled weight (a decode step of a larger batch, a
// short prompt).  gemv_tiled's structure, for more rows: a workgroup owns NT tiles of 16 rows of W for the
// WHOLE of K, its KW waves take shares of K and sum their partial tiles through LDS in wave order, so every
// epilogue (residual sum, activation, rotation and cache write) is the product's own: no partial sums in
// memory, no second kernel.  W comes from HBM once, straight into operand A.  The rows of X are fetched by
// every workgroup (from L2): a wave brings its share, 64 of K at a time, into LDS of its own by
// global_load_lds in units of 8 rows x 128 bytes (whole lines; lanes that read the operand's own 16 rows x
// 64 bytes from memory fetch half lines, and that was three times slower) and reads the fragments back in
// operand order, the units placed with the exclusive-or of gemm_wreg so that the reads are free of bank
// conflicts.  No barrier in the loop: a wave waits for its own loads only, D stages of 64 of K in flight,
// by count.  A step past a wave's share takes its W from a KiB of zeros and adds nothing.
// ===========================================================================
static __device__ __attribute__((aligned(1024))) unsigned char zero_kib[1024];      // never written

template <class T, int NT, int MT, int KW, int D>
__global__ __launch_bounds__(64 * KW) void gemm_rows_kernel(const T* __restrict__ X, const T* __restrict__ Wt,
                                                            int K, int ldx, Epilogue e, RowsOut ro) {
    typedef typename Vec<T>::v8 v8;
    constexpr int UNITS = 2 * MT, STAGE = UNITS * 1024, REGION = D * STAGE;     // bytes of LDS: a stage, a wave's stages
    static_assert(REGION >= NT * MT * 1024, "a wave's partial tiles lie in its own stages");
    extern __shared__ __attribute__((aligned(1024))) unsigned char rows_smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int tile0 = blockIdx.x * NT;
    const int n_tiles = (e.N + 15) >> 4;
    const int steps = K >> 5, doubles = (steps + 1) >> 1;            // 32 and 64 of K
    const int per = (doubles + KW - 1) / KW;
    const int d_begin = wave * per, d_end = min(doubles, d_begin + per);
    const int n = d_end - d_begin;                      // this wave's steps of 64 of K (none for a short K)
    unsigned char* region = rows_smem + wave * REGION;
    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < MT; ++j) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    // What the epilogue reads from memory is fetched now, so that it has arrived when the sums are ready: the
    // tiles are dealt to the waves (tile i to wave i % KW), a lane finishes row 16 j + r, columns n .. n + 3 of
    // its tiles.  Residual sum: the four values it adds to.  Rotation: the row's position, its cache page, and
    // the angles of the quad's two pairs (from the table if there is one).
    constexpr int MINE = (NT * MT + KW - 1) / KW;
    const bool quads = (e.N & 3) == 0;
    f32x4 res[MINE];
    int row_p[MINE];
    int64_t row_page[MINE];
    f32x2 ang[MINE][2];
    if (e.mode == EPI_ADD || e.mode == EPI_ROPE) {
#pragma unroll
        for (int i = 0; i < MINE; ++i) {
            const int id = wave + i * KW, t = id / MT, j = id % MT;
            const int m = 16 * j + r, col = (tile0 + t) * 16 + 4 * g;
            res[i] = f32x4{0.f, 0.f, 0.f, 0.f};
            row_p[i] = 0;
            row_page[i] = 0;
            ang[i][0] = ang[i][1] = f32x2{1.f, 0.f};
            if (id < NT * MT && m < e.M && col < e.N) {
                if (e.mode == EPI_ADD) {
                    if (quads) res[i] = *(const f32x4*)((const float*)e.C + (int64_t)m * e.N + col);
                } else {
                    const RopeStore& rs = e.rs;
                    const int head = col / rs.hd, d = col - head * rs.hd;
                    const int pp = rs.pos[m];
                    row_p[i] = pp;
                    if (head >= rs.H) row_page[i] = rs.page_table[(int64_t)rs.tok_slot[m] * rs.max_pages + pp / PAGE];
                    if (rs.cos_sin) rope_angles(rs, m, pp, head, d, ang[i], true);
                }
            }
        }
    }
    if (n > 0) {
        // W: tile t, step s (32 of K) is 1 KiB at ((tile0 + t) steps + s) KiB, lane l its 16 bytes at 16 l; the
        // base is the wave's (scalar registers), the lane's offset never changes.
        const unsigned char* wbase[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
            wbase[t] = (const unsigned char*)Wt + (int64_t)min(tile0 + t, n_tiles - 1) * steps * 1024;
        const uint32_t woff = lane * 16;
        // X: lane 8 p + c of unit q brings chunk c ^ p (8 of K) of row 8 q + p (rows beyond M: row M - 1 again;
        // the epilogue drops them).  If K ends half way through a step of 64, the lanes of the second half
        // fetch the first half again in that step (the row ends there) and W's second half is the zeros.
        const int p = lane >> 3, chunk = (lane & 7) ^ p;
        uint32_t xoff[UNITS];
#pragma unroll
        for (int q = 0; q < UNITS; ++q) xoff[q] = ((uint32_t)min(8 * q + p, e.M - 1) * (uint32_t)ldx + 8 * chunk) * 2;
        const uint32_t odd_back = ((steps & 1) && chunk >= 4) ? 64 : 0;
        const unsigned char* xbase = (const unsigned char*)X;
        v8 a[D][2][NT];
        auto fetch = [&](int u, int i) {
            const bool in = i < n;
            const int dd = d_begin + min(i, n - 1);
            const uint32_t back = dd == doubles - 1 ? odd_back : 0;
#pragma unroll
            for (int q = 0; q < UNITS; ++q)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(xbase + (int64_t)dd * 128 + (xoff[q] - back)),
                    (__attribute__((address_space(3))) void*)(region + u * STAGE + q * 1024), 16, 0, 0);
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const int step = 2 * dd + h;
                    const unsigned char* from = (in && step < steps) ? wbase[t] + (int64_t)step * 1024
                                                                     : (const unsigned char*)zero_kib;
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(a[u][h][t]) : "v"(woff), "s"(from) : "memory");
                }
        };
        // where lane (r, g) finds row r, chunk 4 h + g of fragment 0 in a stage: unit r / 8, place
        // 8 (r % 8) + ((4 h + g) ^ r % 8); fragment j lies 2 KiB on
        const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)region +
                                  (r >> 3) * 1024 + (r & 7) * 128;
        const uint32_t lds_h0 = lds_base + (g ^ (r & 7)) * 16, lds_h1 = lds_base + ((4 + g) ^ (r & 7)) * 16;
        constexpr int PER_STAGE = UNITS + 2 * NT, AHEAD = (D - 1) * PER_STAGE;
        static_assert(AHEAD <= 63, "the wait's count");
#pragma unroll
        for (int u = 0; u < D; ++u) fetch(u, u);
        for (int i0 = 0; i0 < n; i0 += D) {
#pragma unroll
            for (int u = 0; u < D; ++u) {
                // the oldest stage in flight has landed (its rows of X in LDS, its W in registers)
                __builtin_amdgcn_s_waitcnt(0x0F70 | (AHEAD & 15) | ((AHEAD >> 4) << 14));     // vmcnt(AHEAD) only
                __builtin_amdgcn_sched_barrier(0);
                v8 b[2][MT];
#pragma unroll
                for (int j = 0; j < MT; ++j) {
                    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(b[0][j]) : "v"(lds_h0 + u * STAGE), "n"(j * 2048) : "memory");
                    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(b[1][j]) : "v"(lds_h1 + u * STAGE), "n"(j * 2048) : "memory");
                }
                __builtin_amdgcn_s_waitcnt(0xC07F);                                            // lgkmcnt(0) only
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int t = 0; t < NT; ++t)
#pragma unroll
                        for (int j = 0; j < MT; ++j) acc[t][j] = mfma16(a[u][h][t], b[h][j], acc[t][j]);
                __builtin_amdgcn_sched_barrier(0);
                fetch(u, i0 + u + D);                    // the stage is free: its fragments are in registers
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // loads past the last step are still in flight (into this wave's LDS and its ring of registers) and the
        // compiler does not know of them: wait, then name the registers, so that none of them is handed to
        // another value before the wait
        __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
        for (int u = 0; u < D; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < NT; ++t) asm volatile("" ::"v"(a[u][h][t]));
        __builtin_amdgcn_sched_barrier(0);
    }
    // the partial tiles of a wave go into its own stages (nothing is in flight into them any more)
    float* mine = (float*)region;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < MT; ++j) *(f32x4*)(mine + ((t * MT + j) * 64 + lane) * 4) = acc[t][j];
    __syncthreads();
    // each wave sums its tiles over the waves in wave order and runs the epilogue
#pragma unroll
    for (int i = 0; i < MINE; ++i) {
        const int id = wave + i * KW;
        if (id >= NT * MT) break;
        const int t = id / MT, j = id % MT;
        f32x4 v = *(const f32x4*)((const float*)rows_smem + (id * 64 + lane) * 4);
        for (int w = 1; w < KW; ++w) {
            const f32x4 pw = *(const f32x4*)((const float*)(rows_smem + w * REGION) + (id * 64 + lane) * 4);
            v[0] += pw[0]; v[1] += pw[1]; v[2] += pw[2]; v[3] += pw[3];
        }
        const int m = 16 * j + r, col = (tile0 + t) * 16 + 4 * g;
        const float vv[4] = {v[0], v[1], v[2], v[3]};
        if (e.mode == EPI_ADD && quads) {
            f32x4 o = res[i];
            o[0] += v[0]; o[1] += v[1]; o[2] += v[2]; o[3] += v[3];
            if (m < e.M && col < e.N) *(f32x4*)((float*)e.C + (int64_t)m * e.N + col) = o;
            if (NT * MT == 1 && ro.ss) {
                // RowsOut (one tile a workgroup, at most 16 rows: the host sees to it), as gemv_tiled leaves it
                float sq = 0.f;
                if (m < e.M && col < e.N) {
                    const float scale = ro.row_scale ? ro.row_scale[m] : ro.scale;
                    const f32x4 wv = *(const f32x4*)(ro.w + col);
                    typename Vec<T>::v4 xw;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        sq = fmaf(o[q], o[q], sq);
                        xw[q] = from_f32<T>(o[q] * wv[q] * scale);
                    }
                    *(typename Vec<T>::v4*)((T*)ro.xw + (int64_t)m * e.N + col) = xw;
                }
                sq += __shfl_xor(sq, 16, WAVE);
                sq += __shfl_xor(sq, 32, WAVE);
                if (g == 0) ro.ss[(int64_t)blockIdx.x * 16 + r] = sq;          // (rows beyond M: zeros)
            }
        } else if (e.mode == EPI_ROPE && e.rs.cos_sin) {
            if (m < e.M && col < e.N) {
                const int head = col / e.rs.hd;
                rope_store4(e.rs, m, head, col - head * e.rs.hd, vv, row_p[i], row_page[i], ang[i]);
            }
        } else {
            epilogue4(e, m, col, vv);
        }
    }
}

// ===========================================================================
// C interface
// ===========================================================================
extern "C" int li_gemm_fma(const void* X, int x_dt, const void* W, int w_dt, void* C, int out_dt, int mode,
                           int M, int N, int K, const RopeStore* rs, hipStream_t stream) {
    int rc = check_common(X, W, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
#define CASE(xd, TX, wd, TW)                                                                       \
    if (x_dt == xd && w_dt == wd) {                                                                \
        gemm_fma_kernel<TX, TW><<<grid, block, 0, stream>>>((const TX*)X, (const TW*)W, K, e);     \
        LI_CHECK_LAUNCH();                                                                         \
        return LI_OK;                                                                              \
    }
    CASE(DT_F32, float, DT_F32, float)
    CASE(DT_F16, f16, DT_F16, f16)
    CASE(DT_BF16, bf16, DT_BF16, bf16)
    CASE(DT_F32, float, DT_F16, f16)
    CASE(DT_F32, float, DT_BF16, bf16)
    CASE(DT_F16, f16, DT_F32, float)
    CASE(DT_BF16, bf16, DT_F32, float)
#undef CASE
    return LI_UNSUPPORTED;
}

// tile: 0 = 128x128 (W rows x X rows), 1 = 128x64, 2 = 128x32.  splits > 1 needs ws of
// splits*M*N floats.
extern "C" int li_gemm_mfma(const void* X, const void* W, int tiled, int dt, void* C, int out_dt, int mode,
                            int M, int N, int K, int tile, int splits, float* ws, const RopeStore* rs, hipStream_t stream) {
    int rc = check_common(X, W, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (K % 8 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)W & 15)) return LI_UNSUPPORTED;
    if (tiled && K % 32 != 0) return LI_UNSUPPORTED;
    if (splits < 1 || (splits > 1 && !ws)) return LI_BAD_ARG;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    int k_per_split = ((K + splits - 1) / splits + 63) / 64 * 64;
    splits = (K + k_per_split - 1) / k_per_split;
    const int bm = tile == 0 ? 128 : (tile == 1 ? 64 : 32);
    dim3 grid((N + 127) / 128, (M + bm - 1) / bm, splits), block(256);
#define GO(T, BN, BM, WN, WM, TL) \
    gemm_mfma_kernel<T, BN, BM, WN, WM, TL><<<grid, block, 0, stream>>>((const T*)X, (const T*)W, K, k_per_split, ws, e)
#define LAUNCH(T)                                                       \
    do {                                                                \
        if (tile == 0) { if (tiled) GO(T, 128, 128, 2, 2, true); else GO(T, 128, 128, 2, 2, false); } \
        else if (tile == 1) { if (tiled) GO(T, 128, 64, 2, 2, true); else GO(T, 128, 64, 2, 2, false); } \
        else if (tile == 2) { if (tiled) GO(T, 128, 32, 4, 1, true); else GO(T, 128, 32, 4, 1, false); } \
        else return LI_BAD_ARG;                                         \
    } while (0)
    if (dt == DT_F16) LAUNCH(f16); else LAUNCH(bf16);
#undef LAUNCH
#undef GO
    LI_CHECK_LAUNCH();
    if (splits > 1) {
        const int64_t quads = (int64_t)M * ((N + 3) / 4);
        splitk_reduce_kernel<<<(unsigned)((quads + 255) / 256), 256, 0, stream>>>(ws, splits, e);
        LI_CHECK_LAUNCH();
    }
    return LI_OK;
}

extern "C" int li_gemv_mfma(const void* X, const void* W, int dt, void* C, int out_dt, int mode,
                            int M, int N, int K, const RopeStore* rs, hipStream_t stream) {
    int rc = check_common(X, W, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (M > 16) return LI_BAD_ARG;
    if (K % 8 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)W & 15)) return LI_UNSUPPORTED;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    const int nt = N >= 16384 ? 2 : 1;
    const int tiles = (N + 16 * nt - 1) / (16 * nt);
    const int kw = (tiles < 1024 && K >= 2048) ? 8 : 4;
#define LAUNCH(T, NT, KW) gemv_mfma_kernel<T, NT, KW><<<tiles, 64 * KW, 0, stream>>>((const T*)X, (const T*)W, K, e)
#define PICK(T)                                          \
    do {                                                 \
        if (nt == 2 && kw == 4) LAUNCH(T, 2, 4);         \
        else if (nt == 2) LAUNCH(T, 2, 8);               \
        else if (kw == 4) LAUNCH(T, 1, 4);               \
        else LAUNCH(T, 1, 8);                            \
    } while (0)
    if (dt == DT_F16) PICK(f16); else PICK(bf16);
#undef PICK
#undef LAUNCH
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// W [N, K] row-major -> tiled order, ceil(N/16)*16 * K elements.
extern "C" int li_tile_weight(const void* W, void* out, int dt, int N, int K, hipStream_t stream) {
    if (!W || !out || N <= 0 || K <= 0 || K % 32 != 0) return LI_BAD_ARG;
    const int64_t total = (int64_t)((N + 15) / 16) * (K / 32) * 64;
    const unsigned grid = (unsigned)((total + 255) / 256);
    if (dt == DT_F16) tile_weight_kernel<f16><<<grid, 256, 0, stream>>>((const f16*)W, (f16*)out, N, K, total);
    else if (dt == DT_BF16) tile_weight_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)W, (bf16*)out, N, K, total);
    else return LI_BAD_ARG;
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ro (may be null; mode EPI_ADD, at most 16 rows): RowsOut, with li_gemv_tiled_blocks(...) partial sums a
// row.  rsc (may be null; at most 16 rows): RowScale.
static void gemv_tiled_shape(int M, int N, int K, int& nt, int& kw, int& blocks) {
    const int n_tiles = (N + 15) / 16;
    const int mt = (M + 15) / 16;
    if (nt <= 0) nt = (mt >= 2 || (M > 12 && N >= 6144)) ? 2 : 1;            // measured on MI355X (16 rows, 6,144 x 4,096: 14.5 against 16.3 us)
    if (mt >= 3) nt = 2;
    blocks = (n_tiles + nt - 1) / nt;
    if (kw <= 0) kw = (K >= 8192 || blocks < 320 || blocks > 4096) ? 8 : 4;   // measured on MI355X
    while (kw * nt * (mt == 3 ? 4 : mt) > 64) kw >>= 1;                       // the partial sums fit 64 KiB of LDS
}

// workgroups of li_gemv_tiled for this product (= partial sums a row that ss_out receives)
extern "C" int li_gemv_tiled_blocks(int M, int N, int K, int nt, int kw) {
    int blocks = 0;
    gemv_tiled_shape(M, N, K, nt, kw, blocks);
    return blocks;
}

extern "C" int li_gemv_tiled(const void* X, const void* Wt, int dt, void* C, int out_dt, int mode,
                             int M, int N, int K, int nt, int kw, const RopeStore* rs, const RowsOut* ro,
                             const RowScale* rsc, hipStream_t stream) {
    int rc = check_common(X, Wt, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (M > 64) return LI_BAD_ARG;
    if (K % 32 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)Wt & 15)) return LI_UNSUPPORTED;
    if (ro && (mode != EPI_ADD || M > 16 || (N & 3) || !ro->ss || !ro->xw || !ro->w || !(ro->scale > 0.f) ||
               (((uintptr_t)C | (uintptr_t)ro->w) & 15) || ((uintptr_t)ro->xw & 7)))
        return LI_BAD_ARG;
    if (rsc && (M > 16 || !rsc->ss || rsc->P <= 0 || !(rsc->inv_scale > 0.f))) return LI_BAD_ARG;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    const int mt = (M + 15) / 16;
    int blocks = 0;
    gemv_tiled_shape(M, N, K, nt, kw, blocks);
    if (kw < 2) return LI_BAD_ARG;
    const RowsOut no_out{};
    const RowScale no_scale{};
#define LAUNCH(T, NT, MT, KW) \
    gemv_tiled_kernel<T, NT, MT, KW><<<blocks, 64 * KW, 0, stream>>>((const T*)X, (const T*)Wt, K, e, \
                                                                     ro ? *ro : no_out, rsc ? *rsc : no_scale)
#define PICK_KW(T, NT, MT)                                \
    do {                                                  \
        if (kw == 4) LAUNCH(T, NT, MT, 4);                \
        else if (kw == 8) LAUNCH(T, NT, MT, 8);           \
        else return LI_BAD_ARG;                           \
    } while (0)
#define PICK(T)                                           \
    do {                                                  \
        if (mt == 1 && nt == 1) PICK_KW(T, 1, 1);         \
        else if (mt == 1 && nt == 2) PICK_KW(T, 2, 1);    \
        else if (mt == 2 && nt == 1) PICK_KW(T, 1, 2);    \
        else if (mt == 2 && nt == 2) PICK_KW(T, 2, 2);    \
        else if (mt <= 4 && nt == 2) PICK_KW(T, 2, 4);    \
        else return LI_BAD_ARG;                           \
    } while (0)
    if (dt == DT_F16) PICK(f16); else PICK(bf16);
#undef PICK
#undef PICK_KW
#undef LAUNCH
    LI_CHECK_LAUNCH();
    return LI_OK;
}


// Up to 128 rows of X against a tiled weight, every epilogue its own (gemm_rows).  nt: 1 or 2 tiles of 16 rows
// of W a workgroup, kw: 4 or 8 waves that share K (8: up to 64 rows of X) (0: chosen here); ldx: elements from
// one row of X to the next.  ro (or null; mode EPI_ADD, at most 16 rows, one tile a workgroup): RowsOut, with one
// partial sum a row for each of the N / 16 workgroups.
extern "C" int li_gemm_rows(const void* X, const void* Wt, int dt, void* C, int out_dt, int mode,
                            int M, int N, int K, int ldx, int nt, int kw, const RopeStore* rs, const RowsOut* ro,
                            hipStream_t stream) {
    int rc = check_common(X, Wt, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (M > 128 || ldx < K || ldx % 8 != 0) return LI_BAD_ARG;
    if (K % 32 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)Wt & 15)) return LI_UNSUPPORTED;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : (M <= 64 ? 4 : (M <= 96 ? 6 : 8)));
    const int tiles = (N + 15) / 16;
    if (nt <= 0) nt = tiles >= 1024 ? 2 : 1;          // enough workgroups for 256 CUs either way
    if (kw <= 0) kw = 4;
    if ((nt != 1 && nt != 2) || (kw != 4 && kw != 8) || (kw == 8 && mt > 4)) return LI_BAD_ARG;
    if (ro && (mode != EPI_ADD || M > 16 || nt != 1 || (N & 15) || !ro->ss || !ro->xw || !ro->w || !(ro->scale > 0.f) ||
               (((uintptr_t)C | (uintptr_t)ro->w) & 15) || ((uintptr_t)ro->xw & 7)))
        return LI_BAD_ARG;
    const RowsOut no_out{};
    const int blocks = (tiles + nt - 1) / nt;
    // stages of 64 of K a wave: what 128 KiB of LDS hold for the workgroup's waves
#define GO(T, NT, MT, KW, D)                                                                              \
    do {                                                                                                  \
        auto kfn = gemm_rows_kernel<T, NT, MT, KW, D>;                                                    \
        const size_t lds = (size_t)KW * D * 2 * MT * 1024;                                                \
        static bool allowed = false;               /* more than 64 KiB of LDS is asked for once */       \
        if (!allowed) {                                                                                   \
            if (hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
                return LI_HIP_ERROR;                                                                      \
            allowed = true;                                                                               \
        }                                                                                                 \
        kfn<<<blocks, 64 * KW, lds, stream>>>((const T*)X, (const T*)Wt, K, ldx, e, ro ? *ro : no_out);   \
    } while (0)
#define BY_MT(T, NT)                                            \
    do {                                                        \
        if (mt == 1 && kw == 4) GO(T, NT, 1, 4, 8);             \
        else if (mt == 1) GO(T, NT, 1, 8, 8);                   \
        else if (mt == 2 && kw == 4) GO(T, NT, 2, 4, 6);        \
        else if (mt == 2) GO(T, NT, 2, 8, 4);                   \
        else if (mt == 4 && kw == 4) GO(T, NT, 4, 4, 4);        \
        else if (mt == 4) GO(T, NT, 4, 8, 2);                   \
        else if (mt == 6) GO(T, NT, 6, 4, 2);                   \
        else GO(T, NT, 8, 4, 2);                                \
    } while (0)
#define PICK(T)                                   \
    do {                                          \
        if (nt == 1) BY_MT(T, 1); else BY_MT(T, 2); \
    } while (0)
    if (dt == DT_F16) PICK(f16); else PICK(bf16);
#undef PICK
#undef BY_MT
#undef GO
    LI_CHECK_LAUNCH();
    return LI_OK;
}
