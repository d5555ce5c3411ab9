// Causal grouped-query attention over the paged cache, compiled for one head
// size (HEAD_DIM, a multiple of 16 up to 256).
//
// Formula (include/kernels_cpu.hpp:122-167, src/model/block.cpp:158-164): a query
// at position p of head h reads the keys 0..p of KV head h / (H/K); score =
// (q.k) * scale; softmax with the maximum subtracted; output = sum_t p_t v_t.
// With a window w only the keys p-w+1..p count.  Scores, softmax and the
// running sums are float32.
//
// 16-bit kernels: one wave owns 32 query rows.  S^T = K Q^T and O^T = V^T P^T are
// computed with the 32x32x16 matrix instruction; keys and values come from the
// cache already in operand order (common.h), so every operand is one contiguous
// load and the probabilities go from the accumulators of the first product
// straight into operand B of the second.  Pages are combined by the online
// softmax rule (state m, l, o; src/attention.cu:12-65 holds the same merge with
// o kept normalised).
//   prefill: 4 waves = 128 consecutive tokens of one sequence and one query head.
//   decode : one wave = the query heads of one KV head for one sequence and one
//            split of the context; splits are merged by a second kernel.
// float32 kernel: one workgroup per (token, head), keys in ascending order, so a
// result does not depend on how the step was cut or batched.
#include "common.h"
#include <type_traits>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size: multiple of 16, at most 256");

constexpr int HD = HEAD_DIM;
constexpr int KS = HD / 16;              // steps of the inner index for the scores
constexpr int DB = (HD + 31) / 32;       // 32-row blocks of the output's head dim
constexpr float LOG2E = 1.4426950408889634f;

struct CachePtrs {
    const void* k;            // keys of this layer: page p at k + p * page_stride (elements)
    const void* v;
    int64_t page_stride;
    const int* page_table;    // [n_slots, max_pages]
    int max_pages;
};

template <class T>
struct WaveAttn {
    typedef typename Vec<T>::v8 v8;
    v8 q[KS];
    f32x16 o[DB];
    float m, l;

    __device__ __forceinline__ void init(const T* qrow) {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            v8 z = {};
            q[s] = qrow ? *(const v8*)(qrow + 16 * s + 8 * (lane >> 5)) : z;
        }
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[b][r] = 0.f;
        m = -INFINITY;
        l = 0.f;
    }

    // The work on one page of 64 keys is cut into phases so that a kernel can keep the loads of
    // one phase in flight while the matrix cores work on another.
    __device__ __forceinline__ void load_k(const T* kpage, v8 (&kf)[2 * KS]) const {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int i = 0; i < 2 * KS; ++i) kf[i] = *(const v8*)(kpage + (i * 64 + lane) * 8);
    }
    __device__ __forceinline__ void load_v(const T* vpage, v8 (&vf)[DB * 4]) const {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int i = 0; i < DB * 4; ++i) vf[i] = *(const v8*)(vpage + (i * 64 + lane) * 8);
    }

    // Scores of the page's keys (starting at key t0) against this wave's rows, mask, running
    // maximum and sum; leaves the probabilities in s.  This lane's row sees keys lo..hi.
    __device__ __forceinline__ void scores(const v8 (&kf)[2 * KS], f32x16 (&s)[2], int t0, int lo, int hi,
                                           float scale2, bool masked = true) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[b][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) s[b] = mfma32(kf[b * KS + ks], q[ks], s[b]);
        }
        softmax_step(s, t0, lo, hi, scale2, masked);
    }

    // scale2 > 0.  A page whose keys all lie inside lo..hi for every lane of the wave (the
    // caller knows: `masked` false) skips the comparisons.
    __device__ __forceinline__ void softmax_step(f32x16 (&s)[2], int t0, int lo, int hi, float scale2,
                                                 bool masked = true) {
        const int lane = threadIdx.x & 63;
        float mx = -INFINITY;
        if (masked) {
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int t = t0 + 32 * b + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    const float v = (t >= lo && t <= hi) ? s[b][r] : -INFINITY;
                    s[b][r] = v;
                    mx = fmaxf(mx, v);
                }
        } else {
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[b][r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE)) * scale2;
        const float m_new = fmaxf(m, mx);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        // the hardware's 2^x as it is: results below the smallest normal number become 0, which
        // is what a probability that small is here
        const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
        float psum = 0.f;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = __builtin_amdgcn_exp2f(fmaf(s[b][r], scale2, -m_safe));
                s[b][r] = p;
                psum += p;
            }
        l = l * alpha + psum;
        m = m_new;
        // once the running maximum has settled no row of the wave needs rescaling
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[b][r] *= alpha;
        }
    }

    // o += V^T P^T: the probabilities go from the score accumulators into operand B as they lie.
    __device__ __forceinline__ void mix(const v8 (&vf)[DB * 4], const f32x16 (&s)[2]) {
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            v8 pf;
#pragma unroll
            for (int i = 0; i < 8; ++i) pf[i] = from_f32<T>(s[tj >> 1][8 * (tj & 1) + i]);
#pragma unroll
            for (int b = 0; b < DB; ++b) o[b] = mfma32(vf[b * 4 + tj], pf, o[b]);
        }
    }

    __device__ __forceinline__ float total() const { return l + __shfl_xor(l, 32, WAVE); }
};

// ---------------------------------------------------------------------------
// prefill.  A workgroup of 4 waves shares the pages of one KV head through LDS.  With GW query
// heads of a KV head packed into a workgroup (GW = 4, 2 or 1, the largest that divides the
// group), wave w owns head w % GW and the 32-token block w / GW of the workgroup's 128 / GW
// tokens, so every page is fetched once for up to 4 heads.
// The scores of page p+1 are computed while the probabilities of page p are:
// a wave issues its instructions in order, so a matrix instruction followed by the vector work
// of a few scores keeps both units busy, where a page's 16 matrix instructions followed by its
// softmax left each unit idle in turn.  Per step p the LDS holds the keys of page p+1 and the
// values of page p (keys travel a page ahead of the values), fetched by global_load_lds two
// steps before they are read, two buffers each, one barrier a step.  The arithmetic and its
// order are those of WaveAttn (scores, softmax_step, mix), which the decode kernel uses.
// ---------------------------------------------------------------------------
// The value is computed by this point of the program and not later: without it the compiler
// moves vector work that nothing nearby uses to where it is used, out from between the matrix
// instructions that were to cover it.
#define HERE(x) asm volatile("" : "+v"(x))

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}
// 16 bytes a lane from LDS, written as an instruction: the compiler knows of no wait it needs,
// the caller waits by count (s_waitcnt lgkmcnt) before the first use.
template <int OFFSET, class V>
__device__ __forceinline__ void lds_read16(V& to, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(to) : "v"(addr), "n"(OFFSET));
}

template <class T>
struct PrefillWave {
    typedef typename Vec<T>::v8 v8;
    v8 q[KS];
    f32x16 o[DB];
    float m, l, m_safe, alpha;

    __device__ __forceinline__ void init(const T* qrow) {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            v8 z = {};
            q[s] = qrow ? *(const v8*)(qrow + 16 * s + 8 * (lane >> 5)) : z;
        }
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[b][r] = 0.f;
        m = -INFINITY;
        l = 0.f;
        m_safe = 0.f;
        alpha = 0.f;
    }

    // n = K Q^T for the page whose fragments this lane reads at LDS address kaddr; with SOFT, between
    // its matrix instructions, the probabilities of the page before from its scores c (maximum and
    // alpha already known).  The fragment reads are written as instructions, AHEAD of their use, and
    // waited for by count: left to the compiler every other matrix instruction waited for all of them.
    template <bool SOFT>
    __device__ __forceinline__ void scores(uint32_t kaddr, f32x16 (&n)[2], const f32x16 (&c)[2], v8 (&pf)[4],
                                           float scale2) {
        constexpr int NM = 2 * KS, AHEAD = NM < 4 ? NM : 4;
        v8 kf[NM];
        static_for<0, AHEAD>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            lds_read16<((i & 1) * KS + (i >> 1)) * 1024>(kf[i], kaddr);
        });
        float psum = 0.f;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) n[b][r] = 0.f;
        static_for<0, NM>([&](auto ic) {
            constexpr int i = decltype(ic)::value, b = i & 1, ks = i >> 1, nx = i + AHEAD;
            if constexpr (nx < NM) lds_read16<((nx & 1) * KS + (nx >> 1)) * 1024>(kf[nx], kaddr);
            __builtin_amdgcn_s_waitcnt(0xC07F | ((nx < NM ? AHEAD : NM - 1 - i) << 8));   // lgkmcnt: fragment i is here
            __builtin_amdgcn_sched_barrier(0);
            n[b] = mfma32(kf[i], q[ks], n[b]);
            if (SOFT) {
#pragma unroll
                for (int e = i * 32 / NM; e < (i + 1) * 32 / NM; ++e) {
                    float p = __builtin_amdgcn_exp2f(fmaf(c[e >> 4][e & 15], scale2, -m_safe));
                    psum += p;
                    HERE(p);
                    pf[e >> 3][e & 7] = from_f32<T>(p);
                }
                HERE(psum);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if (SOFT) l = l * alpha + psum;
    }

    // The probabilities alone (the last page of a wave).
    __device__ __forceinline__ void softmax_only(const f32x16 (&c)[2], v8 (&pf)[4], float scale2) {
        float psum = 0.f;
#pragma unroll
        for (int e = 0; e < 32; ++e) {
            const float p = __builtin_amdgcn_exp2f(fmaf(c[e >> 4][e & 15], scale2, -m_safe));
            psum += p;
            pf[e >> 3][e & 7] = from_f32<T>(p);
        }
        l = l * alpha + psum;
    }

    __device__ __forceinline__ void mask(f32x16 (&n)[2], int t0, int lo, int hi) const {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int t = t0 + 32 * b + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                n[b][r] = (t >= lo && t <= hi) ? n[b][r] : -INFINITY;
            }
    }

    // The running maximum takes in a page's largest score mx; alpha is what the sums so far are
    // to be multiplied by before that page is added.
    __device__ __forceinline__ void take_max(float mx, float scale2) {
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE)) * scale2;
        const float m_new = fmaxf(m, mx);
        m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        alpha = __builtin_amdgcn_exp2f(m - m_safe);
        m = m_new;
    }

    __device__ __forceinline__ void rescale() {
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[b][r] *= alpha;
        }
    }

    // o += V^T P^T for the page whose fragments this lane reads at LDS address vaddr; with MAX, between
    // its matrix instructions, the largest of the next page's scores n.
    template <bool MAX>
    __device__ __forceinline__ void mix(uint32_t vaddr, const v8 (&pf)[4], const f32x16 (&n)[2], float scale2) {
        constexpr int NV = 4 * DB, AHEAD = 4;
        v8 vf[NV];
        static_for<0, AHEAD>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            lds_read16<((j % DB) * 4 + j / DB) * 1024>(vf[j], vaddr);
        });
        float mx = -INFINITY;
        static_for<0, NV>([&](auto jc) {
            constexpr int j = decltype(jc)::value, nx = j + AHEAD;
            if constexpr (nx < NV) lds_read16<((nx % DB) * 4 + nx / DB) * 1024>(vf[nx], vaddr);
            __builtin_amdgcn_s_waitcnt(0xC07F | ((nx < NV ? AHEAD : NV - 1 - j) << 8));
            __builtin_amdgcn_sched_barrier(0);
            o[j % DB] = mfma32(vf[j], pf[j / DB], o[j % DB]);
            if (MAX) {
#pragma unroll
                for (int e = j * 32 / NV; e < (j + 1) * 32 / NV; ++e) mx = fmaxf(mx, n[e >> 4][e & 15]);
                HERE(mx);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if (MAX) take_max(mx, scale2);
    }

    __device__ __forceinline__ float total() const { return l + __shfl_xor(l, 32, WAVE); }
};

template <class T>
__global__ __launch_bounds__(256, HD <= 128 ? 2 : 1) void attn_prefill_kernel(
    const T* __restrict__ q, T* __restrict__ out, CachePtrs c, const int* __restrict__ tile_seq,
    const int* __restrict__ tile_q0, const int* __restrict__ seq_slot, const int* __restrict__ seq_qstart,
    const int* __restrict__ seq_qlen, const int* __restrict__ seq_ctx, int H, int K, float scale, int window,
    int GW) {
    typedef typename Vec<T>::v8 v8;
    constexpr int KE = PAGE * HD, VE = PAGE * DB * 32;           // elements of a head's keys / values in a page
    constexpr int KL = KE / 512, VL = VE / 512;                  // loads of 1 KiB (a wave's) that bring them
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* smem = (T*)smem_raw;                                      // keys [2][KE], values [2][VE]

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int G = H / K, TT = 32 * (4 / GW);                     // tokens of this workgroup
    // A causal prompt's later token blocks read more pages.  Workgroups start in blockIdx order,
    // 256 at a time (one per CU); every other such round walks the token blocks backwards, so the
    // workgroups that share a CU have complementary amounts of work (measured: 15% at 2,048 tokens).
    int bx = blockIdx.x;
    if ((blockIdx.y / max(1, 256 / (int)gridDim.x)) & 1) bx = gridDim.x - 1 - bx;
    const int tile = bx / GW, sub = bx % GW;
    const int seq = tile_seq[tile];
    const int kvh = blockIdx.y / (G / GW), hc = blockIdx.y % (G / GW);
    const int h = kvh * G + hc * GW + wave % GW;
    const int qlen = seq_qlen[seq], ctx = seq_ctx[seq];
    const int q0 = tile_q0[tile] + sub * TT;
    if (q0 >= qlen) return;                                      // the same for all waves
    const int first = q0 + 32 * (wave / GW);
    const bool wave_live = first < qlen;
    const int qi = first + (lane & 31);
    const bool live = qi < qlen;
    const int base = ctx - qlen;
    const int pos = live ? base + qi : -1;
    const int64_t tok = seq_qstart[seq] + qi;
    PrefillWave<T> a;
    a.init(live ? q + (tok * H + h) * HD : nullptr);
    const int lo = (window > 0 && live) ? max(0, pos - window + 1) : 0;
    int lo_max = lo, hi_min = pos;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        lo_max = max(lo_max, __shfl_xor(lo_max, o, WAVE));
        hi_min = min(hi_min, __shfl_xor(hi_min, o, WAVE));
    }
    lo_max = __builtin_amdgcn_readfirstlane(lo_max);
    hi_min = __builtin_amdgcn_readfirstlane(hi_min);
    const int p_lo = (window > 0 ? max(0, base + q0 - window + 1) : 0) / PAGE;
    const int p_hi = (base + min(q0 + TT - 1, qlen - 1)) / PAGE;
    const int wp_lo = (window > 0 ? max(0, base + first - window + 1) : 0) / PAGE;
    const int wp_hi = wave_live ? (base + min(first + 31, qlen - 1)) / PAGE : -1;
    const int* table = c.page_table + (int64_t)seq_slot[seq] * c.max_pages;
    const T* kbase = (const T*)c.k + (int64_t)kvh * k_head_elems(HD);
    const T* vbase = (const T*)c.v + (int64_t)kvh * v_head_elems(HD);
    const float scale2 = scale * LOG2E;

    auto kbuf = [&](int p) { return smem + (p & 1) * KE; };
    auto vbuf = [&](int p) { return smem + 2 * KE + (p & 1) * VE; };
    const uint32_t lds_lane = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem_raw + lane * 16;
    auto kaddr = [&](int p) { return lds_lane + (p & 1) * (KE * 2); };            // bytes
    auto vaddr = [&](int p) { return lds_lane + 2 * (KE * 2) + (p & 1) * (VE * 2); };
    const uint32_t lane_at = lane * 16;                          // bytes
    auto bring = [&](const T* src, T* dst, int n_loads) {       // a wave takes every fourth KiB; src, dst the same for all lanes
#pragma unroll
        for (int i = 0; i < (n_loads + 3) / 4; ++i) {
            const int j = wave + 4 * i;
            if (n_loads % 4 == 0 || j < n_loads)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)((const char*)(src + j * 512) + lane_at),
                    (__attribute__((address_space(3))) void*)(dst + j * 512), 16, 0, 0);
        }
    };
    auto at_page = [&](int entry) { return (int64_t)__builtin_amdgcn_readfirstlane(entry) * c.page_stride; };
    // Step p: the keys of page p+1 and the values of page p have arrived (everyone's: wait, then
    // barrier), and nobody reads the keys of page p or the values of page p-1 any more, whose
    // buffers the loads for two steps on now fill.  The page table's entry for a step is read a
    // step before, so that it has arrived with that step's wait.
    int entry_v = table[p_lo], entry_k = table[min(p_lo + 1, p_hi)];      // of pages p+1 and p+2
    auto step = [&](int p) {
        __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0)
        __syncthreads();
        if (p + 2 <= p_hi) bring(kbase + at_page(entry_k), kbuf(p + 2), KL);
        if (p + 1 <= p_hi) bring(vbase + at_page(entry_v), vbuf(p + 1), VL);
        entry_v = entry_k;
        entry_k = table[min(p + 3, p_hi)];
    };
    auto is_masked = [&](int p) { return p * PAGE < lo_max || p * PAGE + PAGE - 1 > hi_min; };

    bring(kbase + at_page(entry_v), kbuf(p_lo), KL);
    int p = p_lo - 1;
    const int own_lo = max(p_lo, wp_lo), own_hi = min(p_hi, wp_hi);
    if (own_lo <= own_hi) {
        f32x16 sa[2], sb[2];
        v8 pf[4];
        for (; p < own_lo - 1; ++p) step(p);
        step(p);                                                 // p = own_lo - 1: the first page's scores
        a.template scores<false>(kaddr(p + 1), sa, sa, pf, scale2);
        if (is_masked(p + 1)) a.mask(sa, (p + 1) * PAGE, lo, pos);
        {
            float mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < 32; ++e) mx = fmaxf(mx, sa[e >> 4][e & 15]);
            a.take_max(mx, scale2);
        }
        ++p;
        auto both = [&](f32x16 (&cur)[2], f32x16 (&nxt)[2]) {    // page p from cur, the scores of p+1 into nxt
            step(p);
            a.template scores<true>(kaddr(p + 1), nxt, cur, pf, scale2);
            if (is_masked(p + 1)) a.mask(nxt, (p + 1) * PAGE, lo, pos);
            a.rescale();
            a.template mix<true>(vaddr(p), pf, nxt, scale2);
            ++p;
        };
        auto last = [&](f32x16 (&cur)[2]) {
            step(p);
            a.softmax_only(cur, pf, scale2);
            a.rescale();
            a.template mix<false>(vaddr(p), pf, cur, scale2);
            ++p;
        };
        // two pages a turn, so that the scores change places without copies
        if ((own_hi - p) & 1) {
            both(sa, sb);
#pragma unroll
            for (int b = 0; b < 2; ++b) sa[b] = sb[b];
        }
        while (p < own_hi) {
            both(sa, sb);
            both(sb, sa);
        }
        last(sa);
    }
    for (; p <= p_hi; ++p) step(p);
    __builtin_amdgcn_s_waitcnt(0x0F70);                          // nothing of this workgroup's is still on its way into LDS
    const float inv = 1.f / a.total();
    if (!live) return;
    T* orow = out + (tok * H + h) * HD;
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d = 32 * b + 8 * g + 4 * (lane >> 5);
            if (d < HD) {
                typename Vec<T>::v4 v = {from_f32<T>(a.o[b][4 * g] * inv), from_f32<T>(a.o[b][4 * g + 1] * inv),
                                         from_f32<T>(a.o[b][4 * g + 2] * inv), from_f32<T>(a.o[b][4 * g + 3] * inv)};
                *(typename Vec<T>::v4*)(orow + d) = v;
            }
        }
}

// ---------------------------------------------------------------------------
// decode: one new token per sequence, q [B, H, HD]
// ---------------------------------------------------------------------------
// A workgroup is W waves that take W consecutive splits of one (sequence, KV head) and merge their
// states through LDS, in wave order; the grid's z extent times W is the number of splits.  With all
// splits inside one workgroup the result is written as it is and no merge kernel runs.
template <class T, int W>
__global__ __launch_bounds__(64 * W) void attn_decode_kernel(
    const T* __restrict__ q, T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    CachePtrs c, const int* __restrict__ seq_slot, const int* __restrict__ seq_ctx, int H, int K, float scale,
    int window) {
    constexpr int OLD = 33;                                   // floats from one output dim to the next in LDS
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = blockIdx.x, G = H / K, gchunks = (G + 31) / 32;
    const int kvh = blockIdx.y / gchunks, gc = blockIdx.y % gchunks;
    const int S = gridDim.z * W, split = blockIdx.z * W + wave;
    const int grid_splits = gridDim.z, grid_split = blockIdx.z;
    const int hg = gc * 32 + (lane & 31);
    const bool live = hg < G;
    const int h = kvh * G + hg;
    const int ctx = seq_ctx[b];
    const int pos = ctx - 1;
    WaveAttn<T> a;
    a.init(live ? q + ((int64_t)b * H + h) * HD : nullptr);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int p_first = lo / PAGE, p_end = pos / PAGE + 1;
    const int per = (p_end - p_first + S - 1) / S;
    const int p0 = p_first + split * per, p1 = min(p_end, p0 + per);
    const int* table = c.page_table + (int64_t)seq_slot[b] * c.max_pages;
    const float scale2 = scale * LOG2E;
    // keys of page p+1 are loaded while the values of page p are mixed, values of page p while
    // its scores are computed
    typename WaveAttn<T>::v8 kf[2 * KS], vf[DB * 4];
    f32x16 s[2];
    const T* kbase = (const T*)c.k + (int64_t)kvh * k_head_elems(HD);
    const T* vbase = (const T*)c.v + (int64_t)kvh * v_head_elems(HD);
    if (p0 < p1) a.load_k(kbase + (int64_t)table[p0] * c.page_stride, kf);
    for (int p = p0; p < p1; ++p) {
        a.load_v(vbase + (int64_t)table[p] * c.page_stride, vf);
        a.scores(kf, s, p * PAGE, lo, live ? pos : -1, scale2, p * PAGE < lo || p * PAGE + PAGE - 1 > pos);
        if (p + 1 < p1) a.load_k(kbase + (int64_t)table[p + 1] * c.page_stride, kf);
        a.mix(vf, s);
    }
    float total = a.total();
    if (W > 1) {
        // waves 1..W-1 lay their states down as [wave - 1][dim][row] (+ m and l per row); wave 0 adds them
        // to its own in wave order:  M = max m,  o = sum o_w 2^(m_w - M),  l = sum l_w 2^(m_w - M)
        float* sm = (float*)smem_raw;
        constexpr int PER = HD * OLD + 64;
        const int row = lane & 31;
        if (wave > 0) {
            float* mine = sm + (wave - 1) * PER;
#pragma unroll
            for (int blk = 0; blk < DB; ++blk)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int d = 32 * blk + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (d < HD) mine[d * OLD + row] = a.o[blk][r];
                }
            if (lane < 32) { mine[HD * OLD + row] = a.m; mine[HD * OLD + 32 + row] = total; }
        }
        __syncthreads();
        if (wave > 0) return;
        float M = a.m;
#pragma unroll
        for (int w = 1; w < W; ++w) M = fmaxf(M, sm[(w - 1) * PER + HD * OLD + row]);
        const float f0 = (a.m == -INFINITY) ? 0.f : exp2f(a.m - M);
#pragma unroll
        for (int blk = 0; blk < DB; ++blk)
#pragma unroll
            for (int r = 0; r < 16; ++r) a.o[blk][r] *= f0;
        total *= f0;
#pragma unroll
        for (int w = 1; w < W; ++w) {
            const float* theirs = sm + (w - 1) * PER;
            const float mw = theirs[HD * OLD + row];
            const float fw = (mw == -INFINITY) ? 0.f : exp2f(mw - M);
            total += theirs[HD * OLD + 32 + row] * fw;
#pragma unroll
            for (int blk = 0; blk < DB; ++blk)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int d = 32 * blk + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (d < HD) a.o[blk][r] += theirs[d * OLD + row] * fw;
                }
        }
        a.m = M;
    }
    if (!live) return;
    if (grid_splits == 1) {
        const float inv = 1.f / total;
        T* orow = out + ((int64_t)b * H + h) * HD;
#pragma unroll
        for (int blk = 0; blk < DB; ++blk)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = 32 * blk + 8 * g + 4 * (lane >> 5);
                if (d < HD) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) orow[d + i] = from_f32<T>(a.o[blk][4 * g + i] * inv);
                }
            }
        return;
    }
    const int64_t slot = ((int64_t)b * H + h) * grid_splits + grid_split;
    float* po = part_o + slot * HD;
#pragma unroll
    for (int blk = 0; blk < DB; ++blk)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d = 32 * blk + 8 * g + 4 * (lane >> 5);
            if (d < HD) {
#pragma unroll
                for (int i = 0; i < 4; ++i) po[d + i] = a.o[blk][4 * g + i];
            }
        }
    if (lane < 32) { part_ml[slot * 2] = a.m; part_ml[slot * 2 + 1] = total; }
}

// Merge of the splits: M = max m_s, L = sum l_s 2^(m_s - M), o = sum o_s 2^(m_s - M) / L.
template <class T>
__global__ void attn_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                  T* __restrict__ out, int S) {
    __shared__ float wgt[64];                        // at most 64 splits
    __shared__ float scratch[16];
    const int64_t row = blockIdx.x;                  // (sequence, head)
    const float* ml = part_ml + row * S * 2;
    const int tid = threadIdx.x;
    const float ms = tid < S ? ml[2 * tid] : -INFINITY;
    const float M = block_max(ms, scratch);
    const float w = (tid < S && ms != -INFINITY) ? exp2f(ms - M) : 0.f;
    const float L = block_sum(tid < S ? ml[2 * tid + 1] * w : 0.f, scratch);
    if (tid < 64) wgt[tid] = w;
    __syncthreads();
    for (int d = tid; d < HD; d += blockDim.x) {
        float acc = 0.f;
        for (int s = 0; s < S; ++s) acc += part_o[(row * S + s) * HD + d] * wgt[s];
        out[row * HD + d] = from_f32<T>(acc / L);
    }
}

// ---------------------------------------------------------------------------
// float32: one workgroup of 256 threads per (token, head); chunks of 256 keys.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void attn_f32_kernel(
    const float* __restrict__ q, float* __restrict__ out, CachePtrs c, const int* __restrict__ pos_of,
    const int* __restrict__ tok_slot, int H, int K, float scale, int window) {
    __shared__ float sq[HD];
    __shared__ float sp[256];
    __shared__ float scratch[16];
    const int tid = threadIdx.x;
    const int64_t tok = blockIdx.x;
    const int h = blockIdx.y, kvh = h / (H / K);
    const int pos = pos_of[tok];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int* table = c.page_table + (int64_t)tok_slot[tok] * c.max_pages;
    for (int d = tid; d < HD; d += 256) sq[d] = q[(tok * H + h) * HD + d];
    __syncthreads();
    float m = -INFINITY, l = 0.f, o = 0.f;            // o: thread d < HD owns output dim d
    for (int t0 = lo; t0 <= pos; t0 += 256) {
        const int t = t0 + tid;
        float s = -INFINITY;
        if (t <= pos) {
            const float* kp = (const float*)c.k + (int64_t)table[t / PAGE] * c.page_stride +
                              (int64_t)kvh * k_head_elems(HD);
            float dot = 0.f;
            for (int d = 0; d < HD; ++d) dot = fmaf(sq[d], kp[k_offset(t % PAGE, d, HD)], dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, block_max(s, scratch));
        const float p = (t <= pos) ? expf(s - m_new) : 0.f;
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        __syncthreads();
        sp[tid] = p;
        __syncthreads();
        const int n = min(256, pos - t0 + 1);
        float psum = 0.f;
        for (int i = 0; i < n; ++i) psum += sp[i];
        l = l * alpha + psum;
        m = m_new;
        if (tid < HD) {
            float acc = o * alpha;
            for (int i = 0; i < n; ++i) {
                const int tt = t0 + i;
                const float* vp = (const float*)c.v + (int64_t)table[tt / PAGE] * c.page_stride +
                                  (int64_t)kvh * v_head_elems(HD);
                acc = fmaf(sp[i], vp[v_offset(tt % PAGE, tid, HD)], acc);
            }
            o = acc;
        }
        __syncthreads();
    }
    if (tid < HD) out[(tok * H + h) * HD + tid] = o / l;
}

// ---------------------------------------------------------------------------
// C interface
// ---------------------------------------------------------------------------
extern "C" int li_attn_head_dim() { return HD; }

static int check_heads(int H, int K) { return (H > 0 && K > 0 && H % K == 0) ? LI_OK : LI_BAD_ARG; }

extern "C" int li_attn_prefill(const void* q, void* out, int dt, const void* k, const void* v, int64_t page_stride,
                               const int* page_table, int max_pages, const int* tile_seq, const int* tile_q0,
                               int n_tiles, const int* seq_slot, const int* seq_qstart, const int* seq_qlen,
                               const int* seq_ctx, int H, int K, float scale, int window, hipStream_t stream) {
    if (check_heads(H, K)) return LI_BAD_ARG;
    if (n_tiles <= 0) return LI_OK;
    CachePtrs c{k, v, page_stride, page_table, max_pages};
    const int G = H / K;
    const int gw = G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1);        // query heads of a KV head per workgroup
    dim3 grid(n_tiles * gw, K * (G / gw)), block(256);
    const size_t lds = (size_t)2 * (PAGE * HD + PAGE * DB * 32) * 2;
#define GO(T)                                                                                                  \
    do {                                                                                                       \
        auto kfn = attn_prefill_kernel<T>;                                                                     \
        if (hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
            return LI_HIP_ERROR;                                                                               \
        kfn<<<grid, block, lds, stream>>>((const T*)q, (T*)out, c, tile_seq, tile_q0, seq_slot, seq_qstart,    \
                                          seq_qlen, seq_ctx, H, K, scale, window, gw);                         \
    } while (0)
    if (dt == DT_F16) GO(f16);
    else if (dt == DT_BF16) GO(bf16);
    else return LI_BAD_ARG;
#undef GO
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// How the splits of the context are dealt: waves of a workgroup (merged inside) times workgroups (merged by
// the merge kernel).  li_attn_decode_parts(splits) is the number of partial states per
// (sequence, head) that the caller's workspace must hold: part_o [B, H, parts, HD], part_ml [B, H, parts, 2]
// float32 (needed when parts > 1).
// (measured on MI355X: workgroups of several waves pay where they save the merge kernel altogether, that
// is for two and four splits; with more splits, one wave a workgroup and one merge over all of them is faster)
static int waves_per_group(int splits) { return (splits == 2 || splits == 4) ? splits : 1; }
extern "C" int li_attn_decode_parts(int splits) { return splits < 1 ? 0 : splits / waves_per_group(splits); }

template <class T, int W>
static int launch_decode(const void* q, void* out, float* part_o, float* part_ml, CachePtrs c, const int* seq_slot,
                         const int* seq_ctx, int n_seqs, int H, int K, float scale, int window, int parts,
                         hipStream_t stream) {
    const int G = H / K;
    dim3 grid(n_seqs, K * ((G + 31) / 32), parts), block(64 * W);
    const size_t lds = W > 1 ? (size_t)(W - 1) * (HD * 33 + 64) * sizeof(float) : 0;
    auto kfn = attn_decode_kernel<T, W>;
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return LI_HIP_ERROR;
    kfn<<<grid, block, lds, stream>>>((const T*)q, (T*)out, part_o, part_ml, c, seq_slot, seq_ctx, H, K, scale, window);
    LI_CHECK_LAUNCH();
    if (parts > 1) {
        attn_merge_kernel<T><<<n_seqs * H, 128, 0, stream>>>(part_o, part_ml, (T*)out, parts);
        LI_CHECK_LAUNCH();
    }
    return LI_OK;
}

extern "C" int li_attn_decode(const void* q, void* out, int dt, const void* k, const void* v, int64_t page_stride,
                              const int* page_table, int max_pages, const int* seq_slot, const int* seq_ctx,
                              int n_seqs, int H, int K, float scale, int window, int splits, float* part_o,
                              float* part_ml, hipStream_t stream) {
    if (check_heads(H, K) || splits < 1 || splits > 64) return LI_BAD_ARG;
    const int w = waves_per_group(splits), parts = splits / w;
    if (parts > 64 || (parts > 1 && (!part_o || !part_ml))) return LI_BAD_ARG;
    if (dt != DT_F16 && dt != DT_BF16) return LI_BAD_ARG;
    if (n_seqs <= 0) return LI_OK;
    CachePtrs c{k, v, page_stride, page_table, max_pages};
#define GO(T)                                                                                                      \
    (w == 4 ? launch_decode<T, 4>(q, out, part_o, part_ml, c, seq_slot, seq_ctx, n_seqs, H, K, scale, window, parts, stream) \
     : w == 2 ? launch_decode<T, 2>(q, out, part_o, part_ml, c, seq_slot, seq_ctx, n_seqs, H, K, scale, window, parts, stream) \
              : launch_decode<T, 1>(q, out, part_o, part_ml, c, seq_slot, seq_ctx, n_seqs, H, K, scale, window, parts, stream))
    return dt == DT_F16 ? GO(f16) : GO(bf16);
#undef GO
}

extern "C" int li_attn_f32(const float* q, float* out, const void* k, const void* v, int64_t page_stride,
                           const int* page_table, int max_pages, const int* pos, const int* tok_slot,
                           int n_tokens, int H, int K, float scale, int window, hipStream_t stream) {
    if (check_heads(H, K)) return LI_BAD_ARG;
    if (n_tokens <= 0) return LI_OK;
    CachePtrs c{k, v, page_stride, page_table, max_pages};
    dim3 grid(n_tokens, H), block(256);
    attn_f32_kernel<<<grid, block, 0, stream>>>(q, out, c, pos, tok_slot, H, K, scale, window);
    LI_CHECK_LAUNCH();
    return LI_OK;
}
