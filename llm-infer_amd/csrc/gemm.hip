// Matrix products  C[M, N] = X[M, K] . W[N, K]^T  (both operands contiguous in K,
// the layout of the reference's matmul, include/kernels_cpu.hpp:69-80), with the
// epilogue fused: plain store, add into the float32 residual, or SwiGLU on
// interleaved gate/up columns.
//
//   gemm_fma   any element types and any sizes; float32 multiply-add in ascending k
//              for every output, so an output does not depend on its place in the batch.
//              It is the true 32-bit path and the fallback for K not a multiple of 8.
//   gemm_mfma  16-bit operands on the matrix cores (32x32x16), tiles staged through
//              LDS, optional split over K into a float32 workspace.
//   gemm_big   the prefill product: larger tiles, two LDS buffers, loads two tiles ahead.
//   gemv_mfma  up to 16 rows of X (row-major W), gemv_tiled up to 64 rows (tiled W): W is
//              streamed once from HBM straight into the matrix cores' operand registers.
#include "common.h"

enum { EPI_STORE = 0, EPI_ADD = 1, EPI_SWIGLU = 2, EPI_ROPE = 3 };

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

// Offset of W[n, k] in the tiled order of a weight matrix (see "Tiled weights" below).
__host__ __device__ __forceinline__ int64_t tiled_offset(int n, int k, int K) {
    return ((((int64_t)(n >> 4) * (K >> 5) + (k >> 5)) * 64) + (((k & 31) >> 3) << 4) + (n & 15)) * 8 + (k & 7);
}

// v[0..3] are the results for row m and columns n..n+3 (n a multiple of 4).
__device__ __forceinline__ void epilogue4(const Epilogue& e, int m, int n, const float* v) {
    if (m >= e.M || n >= e.N) return;
    if (e.mode == EPI_ROPE) {
        // include/kernels_cpu.hpp:82-100 and src/model/block.cpp:141-148, on the accumulators
        const RopeStore& r = e.rs;
        const int head = n / r.hd, d = n - head * r.hd;       // the 4 columns lie in one head (hd % 16 == 0)
        const int p = r.pos[m];
        float o[4] = {v[0], v[1], v[2], v[3]};
        if (head < r.H + r.K) {
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                if (d + j < r.rotary_dim) {
                    float sn, cs;
                    if (r.cos_sin) {
                        const f32x2 t = *(const f32x2*)(r.cos_sin + ((int64_t)m * (r.rotary_dim >> 1) + ((d + j) >> 1)) * 2);
                        cs = t[0]; sn = t[1];
                    } else sincosf((float)p * r.inv_freq[(d + j) >> 1], &sn, &cs);
                    o[j] = v[j] * cs - v[j + 1] * sn;
                    o[j + 1] = v[j] * sn + v[j + 1] * cs;
                }
            }
        }
        if (head < r.H) {
            const int64_t at = ((int64_t)m * r.H + head) * r.hd + d;
#pragma unroll
            for (int j = 0; j < 4; ++j) store_one(r.q_out, r.dt, at + j, o[j]);
        } else {
            const int64_t page = r.page_table[(int64_t)r.tok_slot[m] * r.max_pages + p / PAGE];
            const int tp = p % PAGE;
            if (head < r.H + r.K) {
                const int64_t at = page * r.page_stride + (int64_t)(head - r.H) * k_head_elems(r.hd);
#pragma unroll
                for (int j = 0; j < 4; ++j) store_one(r.k_pages, r.dt, at + k_offset(tp, d + j, r.hd), o[j]);
            } else {
                const int64_t at = page * r.page_stride + (int64_t)(head - r.H - r.K) * v_head_elems(r.hd);
#pragma unroll
                for (int j = 0; j < 4; ++j) store_one(r.v_pages, r.dt, at + v_offset(tp, d + j, r.hd), o[j]);
            }
        }
        return;
    }
    if (e.mode == EPI_SWIGLU) {
        // columns 2j (gate) and 2j+1 (up) give h[m, j] = silu(gate) * up   (src/model/block.cpp:209-213)
        const int64_t row = (int64_t)m * (e.N >> 1);
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            if (n + j + 1 < e.N) {
                const float g = v[j], u = v[j + 1];
                store_one(e.C, e.out_dt, row + ((n + j) >> 1), g / (1.f + expf(-g)) * u);
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
    float acc[4][4] = {};
    const int lr = tid >> 2, lk = (tid & 3) * 4;     // row of the tile and first k this thread loads
    for (int k0 = 0; k0 < K; k0 += BK) {
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
    for (int i = 0; i < 4; ++i) epilogue4(e, m0 + ty * 4 + i, n0 + tx * 4, acc[i]);
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

// Which tile a workgroup works on.  Workgroups go to the 8 XCDs in turn (workgroup L to XCD
// L % 8) and every XCD has an L2 of its own, so the tiles are numbered such that an XCD works on
// one contiguous run of them; within the run, groups of GM tiles of X go through all tiles of W
// before the next group starts.  The workgroups that are resident on an XCD together (32 or 64)
// then cover a near-square block of tiles and share its rows of X and W through that L2; with
// the tiles of X simply fastest they would share one tile of W and stream all of X past it.
__device__ __forceinline__ void tile_of_workgroup(int GM, int& bx, int& by, int& bz) {
    const int gx = gridDim.x, gy = gridDim.y;
    const int total = gx * gy * gridDim.z;
    const int L = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
    const int xcd = L & 7, per = total >> 3, rem = total & 7;
    const int id = xcd * per + min(xcd, rem) + (L >> 3);
    bz = id / (gx * gy);
    const int in_split = id - bz * gx * gy;
    const int group = in_split / (GM * gy), first = group * GM;
    const int size = min(gx - first, GM);
    const int in_group = in_split - group * GM * gy;
    bx = first + in_group % size;
    by = in_group / size;
}

// ===========================================================================
// gemm_big: the prefill product.  BN rows of W x BM rows of X per workgroup of 4
// waves (2 x 2), each wave a (BN/2) x (BM/2) tile of 32x32 blocks, BK = 64.  Two LDS
// buffers: the next tile travels global -> registers while the matrix cores work on
// the current one and is written to the other buffer afterwards, so there is one
// barrier per tile.  With 256 x 256 tiles a wave issues 16 matrix instructions for
// 8 LDS fragment reads.  W may be row-major or tiled.
// ===========================================================================
template <class T, int BN, int BM, int BK, bool TILED, bool EDGE>
__global__ __launch_bounds__(256) void gemm_big_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                       int K, int k_per_split, float* __restrict__ ws,
                                                       Epilogue e) {
    typedef typename Vec<T>::v8 v8;
    constexpr int LD = BK + 8, CPR = BK / 8;             // chunks of 8 elements per tile row
    constexpr int TN = BN / 2, TM = BM / 2;
    constexpr int NB = TN / 32, MB = TM / 32;
    constexpr int W_CHUNKS = BN * BK / 8 / 256, X_CHUNKS = BM * BK / 8 / 256;
    constexpr int BUF = (BN + BM) * LD;                  // elements of one buffer
    constexpr int KSTEPS = BK / 32;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* smem = (T*)smem_raw;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave & 1, wm = wave >> 1;
    int bx, by, bz;
    tile_of_workgroup(8, bx, by, bz);
    const int m0 = bx * BM, n0 = by * BN;
    const int n_limit = TILED ? ((e.N + 15) & ~15) : e.N;
    const int kb = bz * k_per_split, ke = min(K, kb + k_per_split);   // this workgroup's share of K

    f32x16 acc[NB][MB];
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

    // Where each of this thread's 16-byte chunks of a tile comes from and goes to.  Row-major
    // W: CPR threads a row; tiled W: 64 threads a (16 rows x 32 k) block, as it lies in memory.
    // Loads are unconditional (addresses clamped into the matrix) and masked afterwards, so that
    // the loads of two tiles can be in flight at once.
    const T* wsrc[W_CHUNKS];
    const T* xsrc[X_CHUNKS];
    int wdst[W_CHUNKS], xdst[X_CHUNKS], wkc[W_CHUNKS], xkc[X_CHUNKS];
    bool wok[W_CHUNKS], xok[X_CHUNKS];
#pragma unroll
    for (int c = 0; c < W_CHUNKS; ++c) {
        const int chunk = tid + c * 256;
        const int row = TILED ? ((chunk / (64 * KSTEPS)) << 4) + (chunk & 15) : chunk / CPR;
        wkc[c] = TILED ? (((chunk >> 6) % KSTEPS) << 5) + (((chunk >> 4) & 3) << 3) : (chunk % CPR) * 8;
        wok[c] = n0 + row < n_limit;
        const int n = min(n0 + row, n_limit - 1);
        wsrc[c] = TILED ? W + tiled_offset(n, wkc[c], K) : W + (int64_t)n * K + wkc[c];
        wdst[c] = row * LD + wkc[c];
    }
#pragma unroll
    for (int c = 0; c < X_CHUNKS; ++c) {
        const int chunk = tid + c * 256, row = chunk / CPR;
        xkc[c] = (chunk % CPR) * 8;
        xok[c] = m0 + row < e.M;
        xsrc[c] = X + (int64_t)min(m0 + row, e.M - 1) * K + xkc[c];
        xdst[c] = BN * LD + row * LD + xkc[c];
    }
    // loads are raw; the mask (rows beyond the matrix, k beyond K) is applied when the tile is
    // written to LDS, so that nothing waits for a load before then
    // (EDGE false: M, N and K are whole numbers of tiles and nothing is masked)
    auto load_tile = [&](int k0, v8 (&rw)[W_CHUNKS], v8 (&rx)[X_CHUNKS]) {
        const int64_t wstep = TILED ? (int64_t)(k0 >> 5) * 512 : k0;
#pragma unroll
        for (int c = 0; c < W_CHUNKS; ++c) {
            const bool in = !EDGE || k0 + wkc[c] < ke;
            rw[c] = *(const v8*)(wsrc[c] + (in ? wstep : 0));
        }
#pragma unroll
        for (int c = 0; c < X_CHUNKS; ++c) {
            const bool in = !EDGE || k0 + xkc[c] < ke;
            rx[c] = *(const v8*)(xsrc[c] + (in ? k0 : 0));
        }
    };
    auto store_tile = [&](T* buf, int k0, const v8 (&rw)[W_CHUNKS], const v8 (&rx)[X_CHUNKS]) {
        const v8 z = {};
#pragma unroll
        for (int c = 0; c < W_CHUNKS; ++c)
            *(v8*)(buf + wdst[c]) = (!EDGE || (wok[c] && k0 + wkc[c] < ke)) ? rw[c] : z;
#pragma unroll
        for (int c = 0; c < X_CHUNKS; ++c)
            *(v8*)(buf + xdst[c]) = (!EDGE || (xok[c] && k0 + xkc[c] < ke)) ? rx[c] : z;
    };
    auto compute = [&](const T* buf) {
        const T* sW = buf;
        const T* sX = buf + BN * LD;
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
    };

    // Tile t is computed from LDS buffer t % 2 while tile t + 1 waits in registers and the loads
    // of tile t + 2 are issued: a load has more than one tile's worth of matrix work to arrive.
    const int n_tiles = (ke - kb + BK - 1) / BK;
    v8 rw0[W_CHUNKS], rx0[X_CHUNKS], rw1[W_CHUNKS], rx1[X_CHUNKS];
    T* buf0 = smem;
    T* buf1 = smem + BUF;
    // (Loads and stores past the last tile are not branched around: they fetch the last tile again
    // and write it where nothing reads it, which keeps the count of loads in flight fixed.)
    const int k_last = kb + (n_tiles - 1) * BK;
    load_tile(kb, rw0, rx0);
    store_tile(buf0, kb, rw0, rx0);
    load_tile(min(kb + BK, k_last), rw1, rx1);
    __syncthreads();
    int t = 0;
    for (; t + 1 < n_tiles; t += 2) {
        // the scheduling barriers keep the loads at the head of each half and the LDS writes at
        // its tail; left alone the compiler sinks the loads to just before their use
        load_tile(min(kb + (t + 2) * BK, k_last), rw0, rx0);
        __builtin_amdgcn_sched_barrier(0);
        compute(buf0);
        __builtin_amdgcn_sched_barrier(0);
        store_tile(buf1, kb + (t + 1) * BK, rw1, rx1);
        __syncthreads();
        load_tile(min(kb + (t + 3) * BK, k_last), rw1, rx1);
        __builtin_amdgcn_sched_barrier(0);
        compute(buf1);
        __builtin_amdgcn_sched_barrier(0);
        store_tile(buf0, min(kb + (t + 2) * BK, k_last), rw0, rx0);
        __syncthreads();
    }
    if (t < n_tiles) compute(buf0);
    __syncthreads();
    // Epilogue through LDS: a wave lays each 32x32 block down as [row of X][32 columns] and reads it
    // back so that 8 lanes write 32 consecutive columns of one row; the loop over the block's
    // quads is not unrolled, which keeps one copy of the epilogue in the code.
    constexpr int SLD = 36;                                  // floats per staged row (padded)
    float* stage = (float*)smem_raw + wave * (32 * SLD);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < MB; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                *(f32x4*)(stage + (lane & 31) * SLD + 8 * g + 4 * (lane >> 5)) = v;
            }
            __builtin_amdgcn_wave_barrier();
            const int mb = m0 + wm * TM + j * 32, nb = n0 + wn * TN + i * 32;
#pragma unroll 1
            for (int q = lane; q < 256; q += 64) {
                const int r = q >> 3, c = (q & 7) * 4;
                const f32x4 v = *(const f32x4*)(stage + r * SLD + c);
                const float vv[4] = {v[0], v[1], v[2], v[3]};
                if (gridDim.z == 1) epilogue4(e, mb + r, nb + c, vv);
                else if (mb + r < e.M) {                 // a share of K: the partial sums go to the workspace
                    float* p = ws + ((int64_t)bz * e.M + mb + r) * e.N + nb + c;
#pragma unroll
                    for (int j = 0; j < 4; ++j) if (nb + c + j < e.N) p[j] = vv[j];
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
}

// ===========================================================================
// gemm_dma: the prefill product against a tiled W, with both operands going from global
// memory straight into LDS (global_load_lds, 16 bytes a lane): no staging registers, no
// LDS store instructions.  A load instruction of a wave fills 1 KiB of LDS in lane order,
// so a tile lies in LDS as units of 16 rows x 32 elements of K in the order of the tiled
// weight, [lane = 16*((k%32)/8) + row%16][k%8]: a unit of W is copied as it lies in
// memory, a unit of X is gathered by the lanes (16 rows, 64 contiguous bytes each).  A
// fragment of the 32x32x16 instruction is read from two such units, 16 lanes a contiguous
// 256 bytes, which is free of bank conflicts without padding.  BK = 32 (K of a tiled weight
// is a multiple of 32, so no tile is cut in K); rows beyond M or N are read from clamped
// addresses and dropped by the epilogue.  Three LDS buffers: the loads of tile t + 2 are
// issued while tile t is multiplied; one barrier per tile.
// ===========================================================================
template <class T, int BN, int BM, int WAVES, int STAGES>
__global__ __launch_bounds__(64 * WAVES) void gemm_dma_kernel(const T* __restrict__ X, const T* __restrict__ Wt,
                                                          int K, int k_per_split, float* __restrict__ ws,
                                                          Epilogue e) {
    typedef typename Vec<T>::v8 v8;
    constexpr int BK = 32;
    constexpr int TN = BN / 2, TM = BM / (WAVES / 2), NB = TN / 32, MB = TM / 32;   // 2 waves along N
    constexpr int WU = BN / 16, XU = BM / 16, UNITS = WU + XU;       // 1 KiB units of a stage
    constexpr int PER_WAVE = UNITS / WAVES;
    constexpr int STAGE = UNITS * 1024;                              // bytes
    static_assert(UNITS % WAVES == 0, "units of a stage are dealt to the waves");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // uniform: what depends on it stays scalar
    const int wn = wave & 1, wm = wave >> 1;
    int bx, by, bz;
    tile_of_workgroup(BM == 256 ? 4 : 8, bx, by, bz);
    const int m0 = bx * BM, n0 = by * BN;
    const int kb = bz * k_per_split, ke = min(K, kb + k_per_split);
    const int n_tiles = (ke - kb) / BK;
    const int w_blocks = (e.N + 15) >> 4, steps = K >> 5;

    // Where the 16 bytes of this lane come from, for each of the wave's units: a base address that
    // is the same for the whole wave and moves on by `step` bytes per tile of K, plus a 32-bit
    // offset of the lane (the host checks that X has fewer than 4 GiB).
    const unsigned char* base[PER_WAVE];
    uint32_t lane_off[PER_WAVE];
    int step[PER_WAVE];
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
        const int u = wave * PER_WAVE + i;
        if (u < WU) {
            const int blk = min(n0 / 16 + u, w_blocks - 1);
            base[i] = (const unsigned char*)(Wt + ((int64_t)blk * steps + (kb >> 5)) * 512);
            lane_off[i] = lane * 16;
            step[i] = 1024;
        } else {
            const int row = min(m0 + 16 * (u - WU) + (lane & 15), e.M - 1);
            base[i] = (const unsigned char*)(X + kb);
            lane_off[i] = ((uint32_t)row * (uint32_t)K + 8 * (lane >> 4)) * 2;
            step[i] = BK * 2;
        }
    }
    auto issue = [&](int t, int buf) {
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) {
            const int u = wave * PER_WAVE + i;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(base[i] + (int64_t)t * step[i] + lane_off[i]),
                (__attribute__((address_space(3))) void*)(smem_raw + buf * STAGE + u * 1024), 16, 0, 0);
        }
    };

    f32x16 acc[NB][MB];
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

    // byte offset of this lane's piece of a fragment within its pair of units, for k-step 0
    const int frag = ((lane & 31) >> 4) * 1024 + (16 * (lane >> 5) + (lane & 15)) * 16;
    const unsigned char* sW = smem_raw + (wn * TN / 16) * 1024 + frag;
    const unsigned char* sX = smem_raw + (WU + wm * TM / 16) * 1024 + frag;
    auto read_frags = [&](int buf, int ks, v8 (&a)[NB], v8 (&b)[MB]) {
#pragma unroll
        for (int j = 0; j < MB; ++j) b[j] = *(const v8*)(sX + buf * STAGE + j * 2048 + ks * 512);
#pragma unroll
        for (int i = 0; i < NB; ++i) a[i] = *(const v8*)(sW + buf * STAGE + i * 2048 + ks * 512);
    };
    auto multiply = [&](const v8 (&a)[NB], const v8 (&b)[MB], int lo, int hi) {
#pragma unroll
        for (int i = 0; i < NB; ++i)
            if (i >= lo && i < hi) {
#pragma unroll
                for (int j = 0; j < MB; ++j) acc[i][j] = mfma32(a[i], b[j], acc[i][j]);
            }
    };

    // The loop works in half tiles (16 of the 32 elements of K): while the matrix cores work on
    // one half, the fragments of the next are on their way from LDS.  In the middle of tile t every
    // wave has read all of it, so the barrier there both publishes tile t + 1 and frees the buffer
    // of tile t for the loads of tile t + STAGES: loads run STAGES - 1 tiles ahead.
    // (A bare s_barrier: __syncthreads would also wait for the loads still in flight.)
    // One copy of the body, the buffer a run-time offset: unrolled by the three buffers the
    // register allocator spills.  After the last tile the reads for "the next tile" fetch stale
    // data that nothing uses.
    v8 a0[NB], b0[MB], a1[NB], b1[MB];
    // waits until at most `tiles` of the tiles whose loads were issued last are still in flight
    auto wait_tiles = [&](int tiles, bool lds_too) {
        if (lds_too) {
            if (tiles <= 0) __builtin_amdgcn_s_waitcnt(0x0070);
            else if (tiles == 1) __builtin_amdgcn_s_waitcnt(0x0070 | PER_WAVE);
            else if (tiles == 2) __builtin_amdgcn_s_waitcnt(0x0070 | (2 * PER_WAVE));
            else __builtin_amdgcn_s_waitcnt(0x0070 | (3 * PER_WAVE));
        } else {
            if (tiles <= 0) __builtin_amdgcn_s_waitcnt(0x0F70);
            else if (tiles == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | PER_WAVE);
            else if (tiles == 2) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * PER_WAVE));
            else if (tiles == 3) __builtin_amdgcn_s_waitcnt(0x0F70 | (3 * PER_WAVE));
            else __builtin_amdgcn_s_waitcnt(0x0F70 | (3 * PER_WAVE));
        }
    };
    static_assert(STAGES >= 3 && STAGES <= 5 && (STAGES - 2) * PER_WAVE <= 15, "stages");
#pragma unroll
    for (int i = 0; i < STAGES; ++i)
        if (i < n_tiles) issue(i, i);
    wait_tiles(min(min(STAGES, n_tiles) - 1, 3), false);
    __builtin_amdgcn_s_barrier();
    read_frags(0, 0, a0, b0);
    int cur = 0;
#pragma unroll 1
    for (int t = 0; t < n_tiles; ++t) {
        const int nxt = cur == STAGES - 1 ? 0 : cur + 1;
        // the second half's fragments are requested between the matrix instructions of the first
        // half: requested before them, the wait the compiler places for the first half's fragments
        // (it merges the loop's entry and back edge pessimistically) would cover these reads too
        multiply(a0, b0, 0, NB / 2);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(cur, 1, a1, b1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(a0, b0, NB / 2, NB);
        __builtin_amdgcn_sched_barrier(0);
        // tile t + 1 has landed (up to STAGES - 2 later ones may be in flight); this wave's reads
        // of tile t are done
        wait_tiles(min(STAGES - 2, n_tiles - 2 - t), true);
        __builtin_amdgcn_s_barrier();
        if (t + STAGES < n_tiles) issue(t + STAGES, cur);
        multiply(a1, b1, 0, NB / 2);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(nxt, 0, a0, b0);
        __builtin_amdgcn_sched_barrier(0);
        multiply(a1, b1, NB / 2, NB);
        __builtin_amdgcn_sched_barrier(0);
        cur = nxt;
    }
    __syncthreads();
    constexpr int SLD = 36;
    float* stage = (float*)smem_raw + wave * (32 * SLD);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < MB; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                *(f32x4*)(stage + (lane & 31) * SLD + 8 * g + 4 * (lane >> 5)) = v;
            }
            __builtin_amdgcn_wave_barrier();
            const int mb = m0 + wm * TM + j * 32, nb = n0 + wn * TN + i * 32;
#pragma unroll 1
            for (int q = lane; q < 256; q += 64) {
                const int r = q >> 3, c = (q & 7) * 4;
                const f32x4 v = *(const f32x4*)(stage + r * SLD + c);
                const float vv[4] = {v[0], v[1], v[2], v[3]};
                if (gridDim.z == 1) epilogue4(e, mb + r, nb + c, vv);
                else if (mb + r < e.M) {
                    float* p = ws + ((int64_t)bz * e.M + mb + r) * e.N + nb + c;
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) if (nb + c + jj < e.N) p[jj] = vv[jj];
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
}

// Sum of the split-K partials in ascending split order, then the epilogue.
__global__ void splitk_reduce_kernel(const float* __restrict__ ws, int splits, Epilogue e) {
    const int64_t quads_per_row = (e.N + 3) >> 2;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= quads_per_row * e.M) return;
    const int m = (int)(i / quads_per_row), n = (int)(i % quads_per_row) * 4;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < splits; ++s) {
        const float* p = ws + ((int64_t)s * e.M + m) * e.N + n;
#pragma unroll
        for (int q = 0; q < 4; ++q) if (n + q < e.N) v[q] += p[q];
    }
    epilogue4(e, m, n, v);
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
                                                             int K, Epilogue e) {
    // NT tiles of 16 rows of W and MT tiles of 16 rows of X per wave; W comes from HBM once, the
    // rows of X from the caches (they are few)
    typedef typename Vec<T>::v8 v8;
    constexpr int U = (NT + MT) <= 2 ? 8 : ((NT + MT) <= 4 ? 4 : 2);   // 32-element steps of K in flight
    __shared__ float part[KW][NT * MT][64][4];
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
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            float v[4] = {acc[t][j][0], acc[t][j][1], acc[t][j][2], acc[t][j][3]};
            epilogue4(e, 16 * j + r, (tile0 + t) * 16 + 4 * g, v);
        }
}

// ===========================================================================
// gemm_stream: 17 to 128 rows of X against a tiled W.  Such a product reads W once and is
// bound by that read, but has too many rows of X to fetch them per wave: the 4 waves of a
// workgroup own different rows of W (NT tiles of 16 each) and one share of K, and the X
// slice of that share goes through LDS, 128 elements of K a stage, in the order
// [k/8][row][8] that operand B reads without bank conflicts.  W travels global ->
// registers -> operand A, two stages ahead of the matrix cores (three register sets), X
// global -> registers -> the other LDS buffer one stage ahead; one barrier a stage.  K is split over
// blockIdx.y where the rows of W alone cannot fill the chip; the partials are summed in
// split order by splitk_reduce_kernel.
// ===========================================================================
template <class T, int NT, int MT>
__global__ __launch_bounds__(256, 2) void gemm_stream_kernel(const T* __restrict__ X, const T* __restrict__ Wt,
                                                             int K, int k_per_split, float* __restrict__ ws,
                                                             Epilogue e) {
    typedef typename Vec<T>::v8 v8;
    constexpr int KC = 128, KS = KC / 32;                // elements of K and matrix steps per stage
    constexpr int MP = MT * 16 + 1;                      // rows per k/8 group, padded: conflict-free stores
    constexpr int BUF = (KC / 8) * MP;                   // 16-byte units of one buffer
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    v8* sx = (v8*)smem_raw;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n_tiles = (e.N + 15) >> 4;
    const int steps = K >> 5;
    const int tile0 = (blockIdx.x * 4 + wave) * NT;
    const int kb = blockIdx.y * k_per_split, ke = min(K, kb + k_per_split);

    const T* wt[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) wt[t] = Wt + ((int64_t)min(tile0 + t, n_tiles - 1) * steps * 64 + lane) * 8;
    // this thread's 16-byte pieces of a stage of X: column group tid % 16 of rows tid / 16 + 16 i
    const int xk8 = tid & 15, xrow0 = tid >> 4;
    const T* xp[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) xp[i] = X + (int64_t)min(xrow0 + 16 * i, e.M - 1) * K + xk8 * 8;

    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < MT; ++j) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Three register sets for W: the loads of stage s + 2 are issued before stage s is multiplied,
    // so two stages are in flight per wave.  Loads are unconditional, from addresses clamped into
    // this workgroup's share (the waits the compiler places then count exactly); what lies beyond
    // the share of K is never multiplied, rows of X beyond M are zeroed on their way into LDS.
    v8 ra[3][NT][KS], rx[MT];
    const int s_last = (ke >> 5) - 1;
    auto fetch_w = [&](int k0, v8 (&a)[NT][KS]) {
        const int s0 = k0 >> 5;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int u = 0; u < KS; ++u) a[t][u] = *(const v8*)(wt[t] + (int64_t)min(s0 + u, s_last) * 512);
    };
    auto fetch_x = [&](int k0) {
#pragma unroll
        for (int i = 0; i < MT; ++i) rx[i] = *(const v8*)(xp[i] + max(0, min(k0, K - 8 - xk8 * 8)));
    };
    auto stash = [&](int buf) {
        const v8 z = {};
#pragma unroll
        for (int i = 0; i < MT; ++i) sx[buf * BUF + xk8 * MP + xrow0 + 16 * i] = (xrow0 + 16 * i < e.M) ? rx[i] : z;
    };
    auto multiply = [&](int k0, int buf, v8 (&a)[NT][KS]) {
        const int live = min(KS, (ke - k0) >> 5);
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            if (u < live) {
                v8 b[MT];
#pragma unroll
                for (int j = 0; j < MT; ++j) b[j] = sx[buf * BUF + (4 * u + g) * MP + 16 * j + r];
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int j = 0; j < MT; ++j) acc[t][j] = mfma16(a[t][u], b[j], acc[t][j]);
            }
        }
    };

    fetch_w(kb, ra[0]);
    fetch_x(kb);
    fetch_w(kb + KC, ra[1]);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = kb; k0 < ke; k0 += 3 * KC) {
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            const int ks = k0 + d * KC;
            if (ks >= ke) break;
            fetch_x(ks + KC);
            fetch_w(ks + 2 * KC, ra[(d + 2) % 3]);
            __builtin_amdgcn_sched_barrier(0);
            multiply(ks, buf, ra[d]);
            stash(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }

    const bool split = gridDim.y > 1;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const int m = 16 * j + r, n = (tile0 + t) * 16 + 4 * g;
            float v[4] = {acc[t][j][0], acc[t][j][1], acc[t][j][2], acc[t][j][3]};
            if (!split) epilogue4(e, m, n, v);
            else if (m < e.M) {
                float* p = ws + ((int64_t)blockIdx.y * e.M + m) * e.N + n;
#pragma unroll
                for (int q = 0; q < 4; ++q) if (n + q < e.N) p[q] = v[q];
            }
        }
}

// ===========================================================================
// C interface
// ===========================================================================
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
    if (mode < EPI_STORE || mode > EPI_ROPE) return LI_BAD_ARG;
    if (out_dt < DT_F32 || out_dt > DT_BF16) return LI_BAD_ARG;
    if (mode == EPI_ADD && out_dt != DT_F32) return LI_BAD_ARG;
    if (mode == EPI_SWIGLU && (N & 1)) return LI_BAD_ARG;
    return LI_OK;
}

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

extern "C" int li_gemv_tiled(const void* X, const void* Wt, int dt, void* C, int out_dt, int mode,
                             int M, int N, int K, int nt, int kw, const RopeStore* rs, hipStream_t stream) {
    int rc = check_common(X, Wt, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (M > 64) return LI_BAD_ARG;
    if (K % 32 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)Wt & 15)) return LI_UNSUPPORTED;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    const int n_tiles = (N + 15) / 16;
    const int mt = (M + 15) / 16;
    if (nt <= 0) nt = (mt >= 2 || (M > 12 && N >= 16384)) ? 2 : 1;           // measured on MI355X
    if (mt >= 3) nt = 2;
    const int blocks = (n_tiles + nt - 1) / nt;
    if (kw <= 0) kw = (K >= 8192 || blocks < 320 || blocks > 4096) ? 8 : 4;   // measured on MI355X
    while (kw * nt * (mt == 3 ? 4 : mt) > 64) kw >>= 1;                       // the partial sums fit 64 KiB of LDS
    if (kw < 2) return LI_BAD_ARG;
#define LAUNCH(T, NT, MT, KW) \
    gemv_tiled_kernel<T, NT, MT, KW><<<blocks, 64 * KW, 0, stream>>>((const T*)X, (const T*)Wt, K, e)
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

// tile (rows of W x rows of X / depth): 0 = 128x128/64, 1 = 256x128/32
extern "C" int li_gemm_big(const void* X, const void* W, int tiled, int dt, void* C, int out_dt, int mode,
                           int M, int N, int K, int tile, int splits, float* ws, const RopeStore* rs,
                           hipStream_t stream) {
    int rc = check_common(X, W, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (K % 8 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)W & 15)) return LI_UNSUPPORTED;
    if (tiled && K % 32 != 0) return LI_UNSUPPORTED;
    if (tile < 0 || tile > 1) return LI_BAD_ARG;
    if (splits < 1 || (splits > 1 && !ws)) return LI_BAD_ARG;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    const int bn = tile ? 256 : 128, bm = 128, bk = tile ? 32 : 64;
    const size_t lds = (size_t)2 * (bn + bm) * (bk + 8) * 2;
    int k_per_split = ((K + splits - 1) / splits + bk - 1) / bk * bk;
    splits = (K + k_per_split - 1) / k_per_split;
    dim3 grid((M + bm - 1) / bm, (N + bn - 1) / bn, splits), block(256);
    const bool edge = (M % bm) || (N % bn) || (K % bk);
#define GO(T, BN, BM, BK, TL)                                                                          \
    do {                                                                                               \
        auto kfn = edge ? gemm_big_kernel<T, BN, BM, BK, TL, true> : gemm_big_kernel<T, BN, BM, BK, TL, false>; \
        if (hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
            return LI_HIP_ERROR;                                                                       \
        kfn<<<grid, block, lds, stream>>>((const T*)X, (const T*)W, K, k_per_split, ws, e);            \
    } while (0)
#define LAUNCH(T)                                                                                     \
    do {                                                                                              \
        if (tile == 0) { if (tiled) GO(T, 128, 128, 64, true); else GO(T, 128, 128, 64, false); }     \
        else { if (tiled) GO(T, 256, 128, 32, true); else GO(T, 256, 128, 32, false); }               \
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

// 17..128 rows of X, W tiled.  nt: tiles of 16 rows of W per wave (1 or 2); ws: splits * M * N floats
extern "C" int li_gemm_stream(const void* X, const void* Wt, int dt, void* C, int out_dt, int mode,
                              int M, int N, int K, int nt, int splits, float* ws, const RopeStore* rs,
                              hipStream_t stream) {
    int rc = check_common(X, Wt, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (M > 128 || (nt != 1 && nt != 2)) return LI_BAD_ARG;
    if (K % 32 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)Wt & 15)) return LI_UNSUPPORTED;
    if (splits < 1 || (splits > 1 && !ws)) return LI_BAD_ARG;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    const int mt = M <= 32 ? 2 : (M <= 64 ? 4 : 8);
    const int kc = 128;
    int k_per_split = ((K + splits - 1) / splits + kc - 1) / kc * kc;
    splits = (K + k_per_split - 1) / k_per_split;
    const int n_tiles = (N + 15) / 16;
    dim3 grid((n_tiles + 4 * nt - 1) / (4 * nt), splits), block(256);
    const size_t lds = (size_t)2 * (kc / 8) * (mt * 16 + 1) * 16;
#define GO(T, NT, MT)                                                                                  \
    do {                                                                                               \
        auto kfn = gemm_stream_kernel<T, NT, MT>;                                                      \
        if (hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
            return LI_HIP_ERROR;                                                                       \
        kfn<<<grid, block, lds, stream>>>((const T*)X, (const T*)Wt, K, k_per_split, ws, e);           \
    } while (0)
#define PICK(T)                                        \
    do {                                               \
        if (nt == 1 && mt == 2) GO(T, 1, 2);           \
        else if (nt == 1 && mt == 4) GO(T, 1, 4);      \
        else if (nt == 1) GO(T, 1, 8);                 \
        else if (mt == 2) GO(T, 2, 2);                 \
        else if (mt == 4) GO(T, 2, 4);                 \
        else GO(T, 2, 8);                              \
    } while (0)
    if (dt == DT_F16) PICK(f16); else PICK(bf16);
#undef PICK
#undef GO
    LI_CHECK_LAUNCH();
    if (splits > 1) {
        const int64_t quads = (int64_t)M * ((N + 3) / 4);
        splitk_reduce_kernel<<<(unsigned)((quads + 255) / 256), 256, 0, stream>>>(ws, splits, e);
        LI_CHECK_LAUNCH();
    }
    return LI_OK;
}

// tile: 0 = 128 x 128, 1 = 256 x 128, 2 = 256 x 256 with 8 waves (rows of W x rows of X); BK = 32; W tiled
extern "C" int li_gemm_dma(const void* X, const void* Wt, int dt, void* C, int out_dt, int mode,
                           int M, int N, int K, int tile, int splits, float* ws, const RopeStore* rs,
                           hipStream_t stream) {
    int rc = check_common(X, Wt, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (K % 32 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)Wt & 15)) return LI_UNSUPPORTED;
    if (tile < 0 || tile > 2) return LI_BAD_ARG;
    if ((int64_t)M * K * 2 >= ((int64_t)1 << 32)) return LI_UNSUPPORTED;     // 32-bit offsets into X
    if (splits < 1 || (splits > 1 && !ws)) return LI_BAD_ARG;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    const int bn = tile ? 256 : 128, bm = tile == 2 ? 256 : 128, bk = 32;
    const size_t lds = (size_t)3 * (bn + bm) / 16 * 1024;
    int k_per_split = ((K + splits - 1) / splits + bk - 1) / bk * bk;
    splits = (K + k_per_split - 1) / k_per_split;
    dim3 grid((M + bm - 1) / bm, (N + bn - 1) / bn, splits), block(tile == 2 ? 512 : 256);
#define GO(T, BN, BM, WV, ST)                                                                                \
    do {                                                                                               \
        auto kfn = gemm_dma_kernel<T, BN, BM, WV, ST>;                                                 \
        if (hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
            return LI_HIP_ERROR;                                                                       \
        kfn<<<grid, block, lds, stream>>>((const T*)X, (const T*)Wt, K, k_per_split, ws, e);           \
    } while (0)
#define LAUNCH(T)                                    \
    do {                                             \
        if (tile == 0) GO(T, 128, 128, 4, 3);        \
        else if (tile == 1) GO(T, 256, 128, 4, 3);   \
        else GO(T, 256, 256, 8, 3);                  \
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
