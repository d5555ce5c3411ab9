// The products of more than 16 rows of X: gemm_wreg against a tiled weight, gemm_big against a
// row-major one.  Epilogues, layouts and the split-K reduction are in gemm_common.h.
#include "gemm_common.h"

__device__ __forceinline__ f32x4 mfma16(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
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
        // (a chunk that lies beyond a K shorter than the tile is never used: its address is clamped too)
        const int kc = min(wkc[c], K - 8);
        wsrc[c] = TILED ? W + tiled_offset(n, kc, K) : W + (int64_t)n * K + kc;
        wdst[c] = row * LD + wkc[c];
    }
#pragma unroll
    for (int c = 0; c < X_CHUNKS; ++c) {
        const int chunk = tid + c * 256, row = chunk / CPR;
        xkc[c] = (chunk % CPR) * 8;
        xok[c] = m0 + row < e.M;
        xsrc[c] = X + (int64_t)min(m0 + row, e.M - 1) * K + min(xkc[c], K - 8);
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
// gemm_wreg: the prefill product against a tiled W with W never in LDS.  A tiled weight lies in memory
// in the order in which the 16x16x32 matrix instruction takes operand A, so a wave loads its fragments of
// W straight from global memory into a ring of registers (1 KiB contiguous a load: 8 whole lines) and only
// X goes through LDS (global_load_lds).  Four waves, each with 16 NI rows of W and all 128 rows of X of the
// tile (64 NI x 128); two workgroups (three of the narrowest tile) share a CU.  A step is 64 of K: between
// two barriers a wave issues 16 NI matrix instructions, and the LDS reads of the next fragments of X and
// the loads of W two steps ahead are issued between them, so that outside the matrix instructions a step
// has only its wait, its barrier and four loads of X.  What was measured on the way (M = 8,192, random
// float16): one barrier per 32 of K with all LDS reads before the matrix instructions 1.08 to 1.12 PFLOP/s;
// reads under the matrix instructions and 64 of K a barrier 1.11 to 1.18; X fetched as whole 128-byte
// lines instead of two half lines a row 1.23 to 1.32 (the CU's cache takes a request per line touched).
// The narrower tiles are for products whose number of tiles would otherwise leave a large part of the
// last round of workgroups empty.
// ===========================================================================
// MODE: EPI_ADD or EPI_ROPE for a kernel whose epilogue is that one alone and fetches what it reads from
// memory early (the residual a strip ahead; positions and pages once, angles a quad ahead); -1 for every
// epilogue, chosen at run time.
// The loop counts its own loads and LDS reads in flight (s_waitcnt by hand), so the compiler must add none:
// no spills (the build checks that the kernel uses no scratch memory).
// MJ: the tile's rows of X in blocks of 16 (8: 128 rows; 4: 64 rows, for products of up to 64 rows, which then
// fetch and multiply no rows that are not there).  A: how many steps ahead of their use the loads of W are
// issued (2; 4 for products of few rows, where one workgroup a CU has to keep enough of W in flight by itself:
// 8 NI KiB a wave instead of 4 NI; 3 for 65 to 128 rows, where two workgroups may share a CU).
template <class T, int NI, int MODE, int MJ = 8, int A = 2>
__global__ __launch_bounds__(256) void gemm_wreg_kernel(const T* __restrict__ X, const T* __restrict__ Wt,
                                                        int K, int k_per_split, float* __restrict__ ws, Epilogue e,
                                                        int wg_blocks, RowScale rsc) {
    typedef typename Vec<T>::v8 v8;
    // A step is 64 of K: two halves of 32, each one matrix instruction deep.
    // MJ: fragments of X (16 rows each) per wave and half step; every wave takes all the tile's rows of X
    constexpr int BN = 64 * NI, BM = 16 * MJ, XBUFS = A + 1, SLOTS = 2 * A;
    static_assert(MJ == 4 || MJ == 8, "the groups of a half are written out for 4 and 8 fragments");
    constexpr int XU = BM / 8, PER_WAVE = XU / 4;       // 1 KiB units of X per stage (8 rows x 64 of K each), and per wave
    constexpr int STAGE = XU * 1024;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave;
    int bx, by, bz;
    tile_of_workgroup(8, bx, by, bz);
    // wg_blocks: the blocks of 16 rows of W that a workgroup takes of its 4 NI (fewer: more workgroups, for a
    // product whose full tiles would leave CUs without one); a wave whose block lies beyond them fetches and
    // multiplies the workgroup's last block again and stores nothing of it
    const int m0 = bx * BM, n0 = by * 16 * wg_blocks;
    const int n_end = min(e.N, n0 + 16 * wg_blocks);
    const int kb = bz * k_per_split, ke = min(K, kb + k_per_split);
    // a share of K that is 32 more than a multiple of 64 ends with a step of one half
    const int n_halves = (ke - kb) >> 5, n_steps = (n_halves + 1) >> 1;
    const int w_blocks = (e.N + 15) >> 4, steps = K >> 5;

    // this wave's rows of W: NI blocks of 16, each a run of 1 KiB units along K
    const T* wsrc[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int blk = min(n0 / 16 + min(wn * NI + i, wg_blocks - 1), w_blocks - 1);
        wsrc[i] = Wt + (((int64_t)blk * steps + (kb >> 5)) * 64 + lane) * 8;
    }
    // This wave's share of a stage of X.  A 1 KiB unit holds 8 rows x 64 of K, so that the 8 lanes of a row
    // fetch one whole 128-byte line (16 rows x 32 of K, the operand's own order, would fetch two half
    // lines a row and pass twice as many lines through the CU's cache).  Lane 8 p + c of unit q brings
    // chunk c ^ p (8 of K) of row m0 + 8 q + p: the exclusive-or spreads the 8 rows, which lie 128 bytes
    // apart in LDS, over all banks when 16 lanes read one chunk of 16 rows as an operand.
    const unsigned char* xbase = (const unsigned char*)(X + kb);
    uint32_t xoff[PER_WAVE];
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
        const int q = wave * PER_WAVE + i, p = lane >> 3;
        const int row = min(m0 + 8 * q + p, e.M - 1);
        xoff[i] = ((uint32_t)row * (uint32_t)K + 8 * ((lane & 7) ^ p)) * 2;
    }
    // Loads past the last step of K are not branched around: they fetch the last step again (into a buffer
    // and registers that nothing reads), which keeps the count of loads in flight fixed.
    // In a last step of one half the lanes whose chunk lies in the second half fetch the first half's
    // chunk again (the row may end there); nothing reads what they bring.
    const int last = n_halves - 1;
    const uint32_t odd_back = ((n_halves & 1) && ((lane & 7) ^ (lane >> 3)) >= 4) ? 64 : 0;
    auto fill = [&](int s, int buf_off) {
        const int st = min(s, n_steps - 1);
        const int64_t at = (int64_t)st * 128;
        const uint32_t back = st == n_steps - 1 ? odd_back : 0;
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) {
            const int q = wave * PER_WAVE + i;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(xbase + at + (xoff[i] - back)),
                (__attribute__((address_space(3))) void*)(smem_raw + buf_off + q * 1024), 16, 0, 0);
        }
    };
    // The loads of W are written as instructions so that the compiler does not place waits for them (at
    // the loop's head it would wait for every load in flight); the waits are placed by hand below.
    auto fetch_w = [&](int half, v8 (&a)[NI]) {
        const int64_t at = (int64_t)min(half, last) * 512;
#pragma unroll
        for (int i = 0; i < NI; ++i)
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(a[i]) : "v"(wsrc[i] + at) : "memory");
    };

    f32x4 acc[NI][MJ];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < MJ; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Half a step: the matrix instructions on one slot of W's fragments and on the fragments of X that are
    // in b[]; as soon as the instructions that use b[j] are issued, b[j] is read again for the half after
    // this one, so the LDS reads run under the matrix instructions, and so do the loads of W, which go
    // into a slot as soon as its half is issued.  Between two barriers a wave issues 16 NI matrix
    // instructions, and outside them only the wait, the barrier and its four loads of X.
    // The LDS reads are written as instructions too, with the waits by hand: the read of b[j] is followed
    // by seven others before b[j] is used, and LDS reads complete in order, so "at most 7 in flight" is the
    // wait before every group of matrix instructions.  (Left to the compiler, each half begins with a wait
    // for all eight, the last of which has only just been issued.)
    v8 b[MJ];
    // where lane (r = lane % 16, g = lane / 16) finds row r, chunk 4 h + g (half h) of fragment 0: unit
    // r / 8, place 8 (r % 8) + ((4 h + g) ^ r % 8); fragment j lies 2 KiB on
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem_raw +
                              ((lane >> 3) & 1) * 1024 + (lane & 7) * 128;
    const uint32_t lds_lane = lds_base + ((lane >> 4) ^ (lane & 7)) * 16;
    const uint32_t lds_lane2 = lds_base + ((4 + (lane >> 4)) ^ (lane & 7)) * 16;
#define WREG_READ(J, FROM) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(b[J]) : "v"(FROM), "n"((J) * 2048));
#define WREG_GROUP(J, A, NEXT)                                                             \
    {                                                                                      \
        __builtin_amdgcn_s_waitcnt(0xC07F | ((MJ - 1) << 8));   /* lgkmcnt(MJ - 1), nothing else */ \
        __builtin_amdgcn_sched_barrier(0);                                                 \
        _Pragma("unroll") for (int i = 0; i < NI; ++i) acc[i][J] = mfma16(A[i], b[J], acc[i][J]); \
        __builtin_amdgcn_sched_barrier(0);                                                 \
        WREG_READ(J, NEXT)                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                 \
    }
#define WREG_EIGHT(F, ...) F(0, __VA_ARGS__) F(1, __VA_ARGS__) F(2, __VA_ARGS__) F(3, __VA_ARGS__) \
    if constexpr (MJ == 8) { F(4, __VA_ARGS__) F(5, __VA_ARGS__) F(6, __VA_ARGS__) F(7, __VA_ARGS__) }
#define WREG_HALF(A, NEXT)                                                                 \
    {                                                                                      \
        const uint32_t next_ = (NEXT);                                                     \
        WREG_EIGHT(WREG_GROUP, A, next_)                                                   \
    }

    // (The host gives every split of K at least one step.  Without this line the compiler builds a path
    // for no steps on which the ring's registers are written while the first loads are in flight.)
    if (n_steps <= 0) return;
    // In flight, in order: at the head of step s the loads of X of step s + A are issued, in its middle
    // those of W's first half of step s + A, at its end those of the second half.  Step s needs X of step
    // s + 1 (its second half reads ahead into it) and its own W: everything up to the loads of X of step s + 1,
    // i.e. all but the 2 NI loads that followed them in their step and the A - 2 whole steps issued since.
    v8 ring[SLOTS][NI];
    constexpr int PER_STEP = PER_WAVE + 2 * NI, AHEAD = 2 * NI + (A - 2) * PER_STEP;
    static_assert((A - 1) * PER_STEP <= 63 && AHEAD <= 63, "the waits' counts");
#pragma unroll
    for (int a = 0; a < A; ++a) {
        fill(a, a * STAGE);
        fetch_w(2 * a, ring[2 * a]);
        fetch_w(2 * a + 1, ring[2 * a + 1]);
    }
    // RowScale (MODE -1, at most 16 rows of X, K whole; the host sees to it): the partial sums of squares of row
    // tid % 16 are dealt to the 16 groups of 16 threads; they are fetched behind the first loads, and everything is
    // waited for once (the loop's counts are upper bounds and stay right with fewer loads in flight).  The groups'
    // sums lie behind the stages of X, where the epilogue finds them.
    constexpr int STRIPS_BYTES = 4 * 2 * 16 * (16 * NI + 4) * 4;
    constexpr int INFO = XBUFS * STAGE > STRIPS_BYTES ? XBUFS * STAGE : STRIPS_BYTES;     // behind the stages and the strips
    float* row_ss = (float*)(smem_raw + INFO + 2 * BM * 4);                               // [16 groups][16 rows], then [16] factors
    bool scaled = false;
    if constexpr (MODE == -1) {
        scaled = rsc.ss != nullptr;
        if (scaled) {
            const int r = tid & 15, grp = tid >> 4;
            float sum = 0.f;
            for (int p0 = grp; p0 < rsc.P; p0 += 16 * 8) {
                float v[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) v[c] = rsc.ss[min(p0 + 16 * c, rsc.P - 1) * 16 + r];
#pragma unroll
                for (int c = 0; c < 8; ++c) sum += (p0 + 16 * c < rsc.P) ? v[c] : 0.f;
            }
            row_ss[grp * 16 + r] = sum;                     // (the compiler waits for the loads it issued: all of them)
            __builtin_amdgcn_s_waitcnt(0x0070);             // vmcnt(0): the first loads too
        }
    }
    // X of step 0 has landed (and W of step 0 with it)
    if (!scaled) __builtin_amdgcn_s_waitcnt(0x0F70 | (((A - 1) * PER_STEP) & 15) | ((((A - 1) * PER_STEP) >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    WREG_EIGHT(WREG_READ, lds_lane)
    int cur = 0;                                                   // byte offset of the buffer of step s
    for (int s = 0; s < n_steps; s += A) {
#pragma unroll
        for (int u = 0; u < A; ++u) {                              // A steps a turn of the ring
            if (s + u < n_steps) {
                const int nxt = cur == (XBUFS - 1) * STAGE ? 0 : cur + STAGE;
                const int free_buf = cur == 0 ? (XBUFS - 1) * STAGE : cur - STAGE;      // of the step before this one
                // X of step s + 1 and W of step s have landed, and this wave's reads of the buffer that is filled
                // next are done (all but the MJ issued last, which read the buffer of this step); the barrier
                // publishes the one and frees the other
                __builtin_amdgcn_s_waitcnt(0x0070 | (MJ << 8) | (AHEAD & 15) | ((AHEAD >> 4) << 14));
                __builtin_amdgcn_s_barrier();
                fill(s + u + A, free_buf);
                __builtin_amdgcn_sched_barrier(0);
                WREG_HALF(ring[2 * u], lds_lane2 + cur)
                fetch_w(2 * (s + u + A), ring[2 * u]);
                __builtin_amdgcn_sched_barrier(0);
                if (2 * (s + u) + 1 < n_halves) WREG_HALF(ring[2 * u + 1], lds_lane + nxt)
                fetch_w(2 * (s + u + A) + 1, ring[2 * u + 1]);
                __builtin_amdgcn_sched_barrier(0);
                cur = nxt;
            }
        }
    }
#undef WREG_HALF
#undef WREG_EIGHT
#undef WREG_GROUP
#undef WREG_READ
    __builtin_amdgcn_s_waitcnt(0x0070);
    // Loads into the ring and reads into b[] may still be in flight here (those past the last step).  The
    // compiler does not know of them: without a use of these registers after the wait it would hand them to
    // the epilogue's values before the wait, and a load that lands late would overwrite an address.
#pragma unroll
    for (int u = 0; u < SLOTS; ++u)
#pragma unroll
        for (int i = 0; i < NI; ++i) asm volatile("" ::"v"(ring[u][i]));
#pragma unroll
    for (int j = 0; j < MJ; ++j) asm volatile("" ::"v"(b[j]));
    __builtin_amdgcn_sched_barrier(0);

    // Epilogue through LDS, a strip of 16 rows of X x 16 NI rows of W at a time: accumulator q of a 16x16
    // block is W row 4 (lane / 16) + q, X row lane % 16; read back, consecutive lanes hold consecutive
    // quads of columns of one row.  A wave has room for two strips.
    constexpr int SLD = 16 * NI + 4, QUADS = 4 * NI, STRIP = 16 * SLD;
    static_assert(STRIPS_BYTES == 4 * 2 * STRIP * 4, "the strips' size");
    int* row_pos = (int*)(smem_raw + INFO);
    int* row_page = row_pos + BM;
    if constexpr (MODE == EPI_ROPE) {
        // position and cache page of the tile's rows, once (two dependent loads a row)
        if (tid < BM) {
            const int m = min(m0 + tid, e.M - 1), p = e.rs.pos[m];
            row_pos[tid] = p;
            row_page[tid] = (e.rs.K > 0 && n0 + BN > e.rs.H * e.rs.hd)
                                ? e.rs.page_table[(int64_t)e.rs.tok_slot[m] * e.rs.max_pages + p / PAGE] : 0;
        }
    }
    if constexpr (MODE == -1) {
        if (scaled && tid < 16) {
            // this row: the groups' sums in the order of the groups, then 1 / (scale * rms)
            float ss = row_ss[tid];
            for (int grp = 1; grp < 16; ++grp) ss += row_ss[grp * 16 + tid];
            const float rms = sqrtf(ss / (float)K + rsc.eps);
            row_ss[256 + tid] = (rsc.row_scale ? 1.f / rsc.row_scale[tid] : rsc.inv_scale) / rms;
            if (rsc.next_scale && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) rsc.next_scale[tid] = row_scale_for(rms);
        }
    }
    __syncthreads();
    float* stage = (float*)smem_raw + wave * (2 * STRIP);
    const int r = lane & 15, g = lane >> 4;
    const int nb = n0 + wn * (16 * NI);                 // this wave's first column
    auto to_stage = [&](int j, int place) {
#pragma unroll
        for (int i = 0; i < NI; ++i) *(f32x4*)(stage + place * STRIP + r * SLD + 16 * i + 4 * g) = acc[i][j];
    };

    if constexpr (MODE == EPI_ADD) {
        // C += product (float32, N a multiple of 4, one split: the host sees to it).  NI quads a lane and
        // strip, in row row_of[it], from column col_of[it]; the residual of strip j + 1 is fetched before
        // strip j is added and stored.
        float* C = (float*)e.C;
        int row_of[NI], col_of[NI];
#pragma unroll
        for (int it = 0; it < NI; ++it) {
            const int q = lane + 64 * it;
            row_of[it] = q / QUADS;
            col_of[it] = nb + (q % QUADS) * 4;
        }
        f32x4 res[2][NI];
        auto fetch = [&](int j, f32x4 (&c)[NI]) {
#pragma unroll
            for (int it = 0; it < NI; ++it) {
                const int m = m0 + 16 * j + row_of[it];
                if (m < e.M && col_of[it] < n_end) c[it] = *(const f32x4*)(C + (int64_t)m * e.N + col_of[it]);
            }
        };
        fetch(0, res[0]);
#pragma unroll
        for (int j = 0; j < MJ; ++j) {
            to_stage(j, 0);
            __builtin_amdgcn_wave_barrier();
            if (j + 1 < MJ) fetch(j + 1, res[(j + 1) & 1]);
#pragma unroll
            for (int it = 0; it < NI; ++it) {
                const int m = m0 + 16 * j + row_of[it];
                if (m < e.M && col_of[it] < n_end) {
                    f32x4 o = res[j & 1][it];
                    const f32x4 v = *(const f32x4*)(stage + row_of[it] * SLD + (col_of[it] - nb));
                    o[0] += v[0]; o[1] += v[1]; o[2] += v[2]; o[3] += v[3];
                    *(f32x4*)(C + (int64_t)m * e.N + col_of[it]) = o;
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    } else {
        // Two strips a pass; the loop over their quads is not unrolled (one copy of the epilogue's code a
        // pass).  With MODE == EPI_ROPE: rotation and cache write with the table of angles (the host sees
        // to it), positions and pages from LDS, the angles of a quad fetched while the quad before it is
        // rotated and stored.
        const RopeStore& rs = e.rs;
        auto place_of = [&](int q, int& row, int& n) {      // quad q of a pass: row of the tile's strip pair, column
            const int strip = q / (16 * QUADS), qq = q - strip * (16 * QUADS);
            row = 16 * strip + qq / QUADS;
            n = nb + (qq % QUADS) * 4;
        };
#pragma unroll
        for (int jc = 0; jc < MJ; jc += 2) {
            to_stage(jc, 0);
            to_stage(jc + 1, 1);
            __builtin_amdgcn_wave_barrier();
            const int mb = m0 + 16 * jc;
            f32x2 ang[2] = {f32x2{1.f, 0.f}, f32x2{1.f, 0.f}};
            int row, n;
            place_of(lane, row, n);
            if constexpr (MODE == EPI_ROPE) {
                if (mb + row < e.M && n < n_end) rope_angles(rs, mb + row, 0, n / rs.hd, n % rs.hd, ang, true);
            }
#pragma unroll 1
            for (int q = lane; q < 2 * 16 * QUADS; q += 64) {
                const f32x4 v = *(const f32x4*)(stage + (row >> 4) * STRIP + (row & 15) * SLD + (n - nb));
                const float vv[4] = {v[0], v[1], v[2], v[3]};
                const int m = mb + row, col = n;
                if constexpr (MODE == EPI_ROPE) {
                    const f32x2 now[2] = {ang[0], ang[1]};
                    if (q + 64 < 2 * 16 * QUADS) {
                        place_of(q + 64, row, n);
                        if (mb + row < e.M && n < n_end) rope_angles(rs, mb + row, 0, n / rs.hd, n % rs.hd, ang, true);
                    }
                    if (m < e.M && col < n_end) {
                        const int head = col / rs.hd;
                        rope_store4(rs, m, head, col - head * rs.hd, vv, row_pos[m - m0], row_page[m - m0], now);
                    }
                } else {
                    if (q + 64 < 2 * 16 * QUADS) place_of(q + 64, row, n);
                    if (col >= n_end) continue;
                    if (scaled) {
                        const float f = row_ss[256 + min(m, 15)];
                        const float sv[4] = {vv[0] * f, vv[1] * f, vv[2] * f, vv[3] * f};
                        epilogue4(e, m, col, sv);
                    } else if (gridDim.z == 1) epilogue4(e, m, col, vv);
                    else if (m < e.M) {
                        float* p = ws + ((int64_t)bz * e.M + m) * e.N + col;
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) if (col + jj < e.N) p[jj] = vv[jj];
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// ===========================================================================
// C interface
// ===========================================================================
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

// tile (rows of W x rows of X): 0 = 256 x 128, 1 = 192 x 128, 2 = 128 x 128.  W tiled (K a multiple of 32),
// X below 4 GiB (the kernel addresses it with 32-bit offsets); ws: splits * M * N floats when K is split.
// `na` (or null): with K split and the residual sum as epilogue, the kernel that adds the partial sums also
// takes the norm of the finished rows; it must fit (norm_after_fits), the caller has checked the same.
// few_rows (tile 2 only): 1 = the tile has 64 rows of X, 2 = 128 rows; either way W is fetched four steps ahead
// instead of two (for products of up to 128 rows, where a workgroup has a CU to itself); 3 = 128 rows of X and W
// three steps ahead (two workgroups still fit a CU); 0 = none of these.
// wg_blocks: blocks of 16 rows of W a workgroup, from 1 to the tile's own number (0: that number); fewer make
// more workgroups of a product whose full tiles would leave CUs without one.
extern "C" int li_gemm_wreg(const void* X, const void* Wt, int dt, void* C, int out_dt, int mode,
                            int M, int N, int K, int tile, int splits, float* ws, const RopeStore* rs,
                            const NormAfter* na, int few_rows, int wg_blocks, const RowScale* rsc, hipStream_t stream) {
    int rc = check_common(X, Wt, C, M, N, K, mode, out_dt);
    if (rc) return rc;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (K % 32 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)Wt & 15)) return LI_UNSUPPORTED;
    if (tile < 0 || tile > 2 || few_rows < 0 || few_rows > 3 || (few_rows && tile != 2)) return LI_BAD_ARG;
    if ((int64_t)M * K * 2 >= ((int64_t)1 << 32)) return LI_UNSUPPORTED;
    if (splits < 1 || (splits > 1 && !ws)) return LI_BAD_ARG;
    if (M == 0) return LI_OK;
    Epilogue e;
    rc = make_epilogue(e, C, mode, out_dt, M, N, rs);
    if (rc) return rc;
    const int bn = 256 - 64 * tile, bm = few_rows == 1 ? 64 : 128, bk = 32, ahead = few_rows == 3 ? 3 : (few_rows ? 4 : 2);
    if (wg_blocks == 0) wg_blocks = bn / 16;
    if (wg_blocks < 1 || wg_blocks > bn / 16) return LI_BAD_ARG;
    int k_per_split = ((K + splits - 1) / splits + bk - 1) / bk * bk;
    splits = (K + k_per_split - 1) / k_per_split;
    if (na && !(splits > 1 && norm_after_fits(na, e, ws))) return LI_BAD_ARG;
    // rsc (or null): these rows are x * weight of a norm that the product before left unfinished (RowScale); up to
    // 16 rows, K whole, not with the epilogues that have kernels of their own
    if (rsc && (M > 16 || splits > 1 || !rsc->ss || rsc->P <= 0 || !(rsc->inv_scale > 0.f) || mode == EPI_ADD || mode == EPI_ROPE))
        return LI_BAD_ARG;
    const RowScale no_scale{};
    dim3 grid((M + bm - 1) / bm, ((N + 15) / 16 + wg_blocks - 1) / wg_blocks, splits), block(256);
    // ahead + 1 stages of X (a step is 64 of K); the epilogue stages two strips of 16 x (bn / 4 + 4) floats a wave
    // in the same LDS, and behind both lie a position and a page for each of the tile's rows
    const size_t stages = (size_t)(ahead + 1) * 2 * (bm / 16) * 1024, strips = (size_t)4 * 2 * 16 * (bn / 4 + 4) * 4;
    const size_t lds = (stages > strips ? stages : strips) + (size_t)2 * bm * 4 + (256 + 16) * 4;   // and the sums of squares of RowScale
    // the kernels of one epilogue: the residual sum into float32 with whole quads of columns; the
    // rotation with a table of angles
    const int one = splits > 1 ? -1 : (mode == EPI_ADD && N % 4 == 0) ? EPI_ADD : (mode == EPI_ROPE && e.rs.cos_sin) ? EPI_ROPE : -1;
#define GO(T, NI, MODE, MJ, A)                                                                            \
    do {                                                                                                  \
        auto kfn = gemm_wreg_kernel<T, NI, MODE, MJ, A>;                                                  \
        if (lds > 64 * 1024) {                                                                            \
            static bool allowed = false;           /* more than 64 KiB of LDS is asked for once */       \
            if (!allowed && hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
                return LI_HIP_ERROR;                                                                      \
            allowed = true;                                                                               \
        }                                                                                                 \
        kfn<<<grid, block, lds, stream>>>((const T*)X, (const T*)Wt, K, k_per_split, ws, e, wg_blocks,     \
                                          rsc ? *rsc : no_scale);                                         \
    } while (0)
#define BY_MODE(T, NI, MJ, A)                             \
    do {                                                  \
        if (one == EPI_ADD) GO(T, NI, EPI_ADD, MJ, A);    \
        else if (one == EPI_ROPE) GO(T, NI, EPI_ROPE, MJ, A); \
        else GO(T, NI, -1, MJ, A);                        \
    } while (0)
#define LAUNCH(T)                                       \
    do {                                                \
        if (tile == 0) BY_MODE(T, 4, 8, 2);             \
        else if (tile == 1) BY_MODE(T, 3, 8, 2);        \
        else if (few_rows == 1) BY_MODE(T, 2, 4, 4);    \
        else if (few_rows == 2) BY_MODE(T, 2, 8, 4);    \
        else if (few_rows == 3) BY_MODE(T, 2, 8, 3);    \
        else BY_MODE(T, 2, 8, 2);                       \
    } while (0)
    if (dt == DT_F16) LAUNCH(f16); else LAUNCH(bf16);
#undef LAUNCH
#undef BY_MODE
#undef GO
    LI_CHECK_LAUNCH();
    if (splits > 1 && na) {
        launch_splitk_add_norm(ws, splits, e, na, stream);
        LI_CHECK_LAUNCH();
    } else if (splits > 1) {
        const int64_t quads = (int64_t)M * ((N + 3) / 4);
        splitk_reduce_kernel<<<(unsigned)((quads + 255) / 256), 256, 0, stream>>>(ws, splits, e);
        LI_CHECK_LAUNCH();
    }
    return LI_OK;
}
