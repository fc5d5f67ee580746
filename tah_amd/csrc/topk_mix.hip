// Top-k softmax mix of embedding rows: the next-iteration input of a hard token, gfx950.
//
//   out[row] = sum_j softmax(top-k logits of the row)_j * embedding[index_j]
//
// One workgroup (1024 threads) per row.  The row's logits (bf16) are loaded once into registers as
// order-preserving 16-bit keys; the keys that can be among the k largest (those at or above the k-th largest
// thread maximum) are collected in LDS.  Up to 512 of them (a few more than k on anything but a flat row) are
// ranked against each other directly -- larger key first, equal keys by ascending index, ncand^2 comparisons
// spread over the workgroup -- and the k first are the selection, already in output order.  More candidates:
// the k-th largest key is found by bisection on the 16-bit key space with a block-wide count per step (no
// histogram atomics, no sort) and ties at the threshold are broken towards the lower vocabulary index by a second
// bisection on the index.  The <= k selected (index, value) pairs are
// ordered by index (so that the float sums below have one fixed order), and the mix is
// accumulated in float over bf16-rounded products, as the bf16 eager arithmetic it replaces rounds them.
#include <hip/hip_runtime.h>

#include "duo_device.h"
#include "row_keys.h"
#include "tah_duo.h"

namespace tah {
namespace {

constexpr int kMixThreads = 1024;
constexpr int kMixWaves = kMixThreads / kWave;
constexpr int kMaxTopk = 256;
constexpr int kMaxCand = 2048;  // keys that reach the lower bound of the k-th largest (two per thread)
constexpr int kPairMax = 512;   // up to this many candidates are ranked against each other directly (the usual case)
constexpr int kMaxVec = 19;  // 16-byte pieces of the row per thread: vocabularies up to 19 * 8 * 1024 = 155648

typedef float f32x4s __attribute__((ext_vector_type(4)));

struct MixParams {
    const __bf16* logits;
    const __bf16* emb;
    __bf16* out;
    bf16x8* outp;  // the rows form of the linear-layer kernels ([hidden / 32][2][64][8]) or null
    int32_t zero_disabled;
    __bf16* vals;  // the selected logits themselves, largest first ([rows, v_rs]), or null
    int32_t* idxs;  // their vocabulary indices ([rows, v_rs]), or null
    int64_t v_rs;
    const uint8_t* row_enable;
    int64_t l_rs, e_rs, o_rs;
    int32_t rows, vocab, hidden, topk;
};

// Sum of `x` over the workgroup, returned to every thread.  `red` holds kMixWaves ints; two barriers.
__device__ __forceinline__ int block_sum(int x, int* red, int wave, int lane) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m);
    __syncthreads();  // earlier readers of red are done
    if (lane == 0) red[wave] = x;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int w = 0; w < kMixWaves; ++w) t += red[w];
    return t;
}

// Largest T in [lo, hi) with count(key >= T) >= k, given count(key >= lo) >= k > count(key >= hi) (if even `lo` has
// fewer, `lo` comes back).  A 16-way search: every step counts the keys at or above fifteen thresholds spread over the
// interval, each count one ballot per wave and element slot (`pred(t, u)`: this thread's element u, u < NU, has a key
// >= t); lane i of every wave adds its wave's count for threshold i into row `round` of `tot` (zero on entry, every
// row used once), and after one barrier a ballot over that row tells which thresholds still have k keys at or above
// them.  The bounds stay in scalar registers.  Four steps for 16 bits, five for a vocabulary index; kSearchRows
// rows of `tot` per search.
constexpr int kSearchRows = 6;
template <int NU, class Pred>
__device__ __forceinline__ uint32_t search_kth(uint32_t lo, uint32_t hi, int k, int (*tot)[16], int lane, Pred pred) {
    int round = 0;
    while (hi - lo > 1 && round < kSearchRows) {
        const uint32_t step = (hi - lo + 15u) / 16u;
        auto threshold = [&](int i) { return lo + i * step < hi ? lo + i * step : hi; };  // (scalar arithmetic)
        int* t = tot[round++];
        int mine = 0;  // lane i: this wave's count for threshold i
#pragma unroll
        for (int i = 1; i < 16; ++i) {
            const uint32_t th = threshold(i);
            int c = 0;
#pragma unroll
            for (int u = 0; u < NU; ++u) c += __popcll(__ballot(pred(th, u)));
            mine = lane == i ? c : mine;
        }
        if (lane < 16 && mine != 0) atomicAdd(&t[lane], mine);
        __syncthreads();
        const unsigned long long ge = __ballot(t[lane & 15] >= k) & 0xfffeull;
        if (ge == 0ull) {
            hi = threshold(1);
        } else {
            const int i = 63 - __builtin_clzll(ge);
            const uint32_t nlo = threshold(i), nhi = i == 15 ? hi : threshold(i + 1);
            lo = nlo;
            hi = nhi;
        }
    }
    return lo;
}

// NVEC: 16-byte pieces of the row per thread, a compile-time bound (the keys must stay in registers).
template <int NVEC>
__global__ __launch_bounds__(kMixThreads) void topk_mix_kernel(const MixParams p) {
    __shared__ int red[kMixWaves];
    __shared__ int tot[3 * kSearchRows][16];
    __shared__ int sel_idx[kMaxTopk];
    __shared__ float sel_val[kMaxTopk];
    __shared__ int ord_idx[kMaxTopk];
    __shared__ __align__(16) float ord_w[kMaxTopk];
    __shared__ unsigned long long cand64[kPairMax];  // (key, -index) of a candidate as one number: larger = earlier
    __shared__ int cand_rank[kPairMax];
    __shared__ int ord_rank[kMaxTopk];
    __shared__ int n_sel;
    __shared__ uint16_t cand_key[kMaxCand];
    __shared__ int cand_idx[kMaxCand];
    __shared__ int n_cand;
    HIP_DYNAMIC_SHARED(unsigned char, dyn)  // float partial sums of the mix: [parts][hidden]

    const int row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    if (p.row_enable && !p.row_enable[row]) {  // uniform per workgroup
        if (p.zero_disabled && p.out) {
            const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int cg = tid; cg < p.hidden / 8; cg += kMixThreads) {
                *reinterpret_cast<bf16x8*>(p.out + (int64_t)row * p.o_rs + cg * 8) = z;
                if (p.outp) p.outp[((int64_t)(cg / 4) * 2 + row / 16) * 64 + (row % 16) + 16 * (cg % 4)] = z;
            }
        }
        return;
    }
    const int V = p.vocab;
    const int k = p.topk < V ? p.topk : V;
    const __bf16* lrow = p.logits + (int64_t)row * p.l_rs;
    if (tid < 3 * kSearchRows * 16) (&tot[0][0])[tid] = 0;  // the searches' counters
    if (tid < kMaxTopk) {
        ord_w[tid] = 0.f;  // (entries past the selected ones are read as zeros by the sum of four at a time)
        ord_rank[tid] = 0;
    }
    if (tid < kPairMax) cand_rank[tid] = 0;
    __syncthreads();

    // ---- the row as keys: piece j of thread t covers indices (j * 1024 + t) * 8 .. + 7 (coalesced loads) ----
    uint32_t keys[NVEC][4];  // two keys per dword, low half = even index
    // loaded four pieces at a time and turned into keys in place, with a scheduling fence per group: left
    // alone, the scheduler issues every load first and the row sits in registers twice (raw and as keys)
    constexpr int kGroup = 4;
    // A row that starts on a 16-byte boundary and has a multiple of eight entries (any real vocabulary) is loaded without
    // a branch: a piece lies inside the row or behind it as a whole, the loads of pieces behind it are sent to the row's
    // start and their keys set to 0 by a select.  With a branch around a load the compiler waits for it where the branch
    // ends, and a thread then has one load in flight instead of a group's.
    const bool whole_pieces = (reinterpret_cast<uintptr_t>(lrow) & 15) == 0 && V % 8 == 0;  // (uniform)
    if (whole_pieces) {
#pragma unroll
        for (int j0 = 0; j0 < NVEC; j0 += kGroup) {
            u32x4 w[kGroup];
#pragma unroll
            for (int j = j0; j < j0 + kGroup && j < NVEC; ++j) {
                const int i0 = (j * kMixThreads + tid) * 8;
                w[j - j0] = *reinterpret_cast<const u32x4*>(lrow + (i0 < V ? i0 : 0));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = j0; j < j0 + kGroup && j < NVEC; ++j) {
                const bool inside = (j * kMixThreads + tid) * 8 < V;
#pragma unroll
                for (int q = 0; q < 4; ++q) keys[j][q] = inside ? order_keys2(w[j - j0][q]) : 0u;  // key 0: below every real key
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
#pragma unroll
        for (int j0 = 0; j0 < NVEC; j0 += kGroup) {
#pragma unroll
            for (int j = j0; j < j0 + kGroup && j < NVEC; ++j) {
                const int i0 = (j * kMixThreads + tid) * 8;
                u32x4 w = {0u, 0u, 0u, 0u};
                if (i0 + 8 <= V && ((reinterpret_cast<uintptr_t>(lrow + i0) & 15) == 0)) {
                    w = *reinterpret_cast<const u32x4*>(lrow + i0);
                } else if (i0 < V) {
                    const uint16_t* h = reinterpret_cast<const uint16_t*>(lrow);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const uint32_t b = i0 + e < V ? h[i0 + e] : 0u;
                        w[e / 2] |= b << (16 * (e % 2));
                    }
                }
                if ((j + 1) * kMixThreads * 8 <= V) {  // (uniform) the whole piece lies inside the row, for every thread
#pragma unroll
                    for (int q = 0; q < 4; ++q) keys[j][q] = order_keys2(w[q]);
                } else {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        uint32_t lo = order_key(w[q] & 0xffffu), hi = order_key(w[q] >> 16);
                        // indices past the end get key 0 (below every real key) so that they are never selected
                        if (i0 + 2 * q >= V) lo = 0u;
                        if (i0 + 2 * q + 1 >= V) hi = 0u;
                        keys[j][q] = lo | (hi << 16);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // ---- candidates: the keys that can be among the k largest -------------------------------------------
    // The k-th largest of the 1024 thread maxima, L, is a lower bound of the k-th largest key (k <= 256 threads
    // hold a key >= L each), and on anything but a flat row only a few hundred keys reach it.  Those go to LDS
    // with their indices, and the searches below run over them (two per thread) instead of over the whole row
    // (152 per thread at the full vocabulary).  A row with more candidates than the list holds takes the
    // searches over the whole row.
    u16x2 tmax2 = {0, 0};  // the larger key per half, then the larger of the two
#pragma unroll
    for (int j = 0; j < NVEC; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) tmax2 = __builtin_elementwise_max(tmax2, __builtin_bit_cast(u16x2, keys[j][q]));
    const uint32_t tmax = tmax2.x > tmax2.y ? tmax2.x : tmax2.y;
    // count(tmax >= 1) >= k unless fewer than k threads hold an element (then L = 1), count(tmax >= 0x10000) = 0
    const uint32_t L = search_kth<1>(1u, 0x10000u, k, tot, lane, [&](uint32_t t, int) { return tmax >= t; });
    if (tid == 0) {
        n_cand = 0;
        n_sel = 0;
    }
    __syncthreads();
    if (tmax >= L) {  // (most threads hold no candidate and skip their row)
        const uint32_t below = (L - 1u) | ((L - 1u) << 16);  // key >= L  <=>  max(key, L - 1) != L - 1, two keys per dword
#pragma unroll
        for (int j = 0; j < NVEC; ++j) {
            uint32_t any = 0u;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t w = keys[j][q];
                TAH_OPAQUE1(w);
                const u16x2 m = __builtin_elementwise_max(__builtin_bit_cast(u16x2, w), __builtin_bit_cast(u16x2, below));
                any |= __builtin_bit_cast(uint32_t, m) ^ below;
            }
            if (any == 0u) continue;  // none of this piece's eight keys reaches L
            int i0 = (j * kMixThreads + tid) * 8;
            TAH_OPAQUE1(i0);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                uint32_t w = keys[j][e / 2];
                TAH_OPAQUE1(w);
                const uint32_t key = (w >> (16 * (e % 2))) & 0xffffu;
                if (key >= L) {
                    const int s_ = atomicAdd(&n_cand, 1);
                    if (s_ < kMaxCand) {
                        cand_key[s_] = (uint16_t)key;
                        cand_idx[s_] = i0 + e;
                    }
                }
            }
        }
    }
    __syncthreads();
    const int ncand = n_cand;
    const bool sorted = ncand <= kPairMax;  // (uniform) the selected entries end up in output order right away
    if (sorted) {
        // Few candidates (a few more than k on anything but a flat row): every candidate's place in the order --
        // larger key first, equal keys by ascending index -- is the number of candidates that come before it,
        // ncand^2 comparisons spread over the workgroup; the k first are the selection, already in output order.
        if (tid < ncand) cand64[tid] = ((unsigned long long)cand_key[tid] << 32) | (uint32_t)(0x7fffffff - cand_idx[tid]);
        __syncthreads();
        int cp = 64;
        while (cp < ncand) cp <<= 1;
        const int nsl = kMixThreads / cp, c = tid & (cp - 1), sl = tid / cp;
        if (c < ncand) {
            const unsigned long long mine = cand64[c];
            int r = 0;
#pragma unroll 4
            for (int i = sl; i < ncand; i += nsl) r += cand64[i] > mine ? 1 : 0;
            if (r) atomicAdd(&cand_rank[c], r);
        }
        __syncthreads();
        if (tid < ncand) {
            const int r = cand_rank[tid];
            if (r < k) {
                sel_idx[r] = cand_idx[tid];
                sel_val[r] = key_value(cand_key[tid]);
            }
        }
        if (tid == 0) n_sel = k;  // (count(key >= L) >= k)
    } else if (ncand <= kMaxCand) {
        // this thread's candidates (key 0: none)
        uint32_t ck[kMaxCand / kMixThreads];
        int ci[kMaxCand / kMixThreads];
#pragma unroll
        for (int u = 0; u < kMaxCand / kMixThreads; ++u) {
            const int c = tid + u * kMixThreads;
            ck[u] = c < ncand ? cand_key[c] : 0u;
            ci[u] = c < ncand ? cand_idx[c] : 0x7fffffff;
        }
        auto cnt_ge = [&](uint32_t t) {
            int c = 0;
#pragma unroll
            for (int u = 0; u < kMaxCand / kMixThreads; ++u) c += ck[u] >= t;
            return c;
        };
        // largest key T with count(key >= T) >= k; count(key >= L) = ncand >= k
        const uint32_t T = search_kth<kMaxCand / kMixThreads>(L, 0x10000u, k, tot + kSearchRows, lane, [&](uint32_t t, int u) { return ck[u] >= t; });
        const int n_ge = block_sum(cnt_ge(T), red, wave, lane);
        const int n_gt = block_sum(cnt_ge(T + 1), red, wave, lane);
        const int need_eq = k - n_gt;  // >= 1: that many keys == T are taken, lowest indices first
        // smallest bound M with count(key == T and index < M) >= need_eq.  More keys == T than needed is the usual
        // case on a full vocabulary (16-bit keys), so this is the same 16-way search, for the need_eq-th largest
        // of V - index over the keys == T (empty slots have key 0 < T)
        int M = V;
        if (n_ge - n_gt > need_eq)
            M = V + 1 - (int)search_kth<kMaxCand / kMixThreads>(1u, (uint32_t)V + 1u, need_eq, tot + 2 * kSearchRows, lane,
                                                                [&](uint32_t t, int u) { return ck[u] == T && (uint32_t)(V - ci[u]) >= t; });
#pragma unroll
        for (int u = 0; u < kMaxCand / kMixThreads; ++u) {
            if (ck[u] > T || (ck[u] == T && ci[u] < M)) {
                const int s_ = atomicAdd(&n_sel, 1);
                if (s_ < kMaxTopk) {
                    sel_idx[s_] = ci[u];
                    sel_val[s_] = key_value(ck[u]);
                }
            }
        }
    } else {
        auto count_ge = [&](uint32_t t) {  // elements of this thread with key >= t
            int c = 0;
#pragma unroll
            for (int j = 0; j < NVEC; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint32_t w = keys[j][q];
                    TAH_OPAQUE1(w);  // the two halves are split here, every time: hoisted out of the bisection
                                     // loop they would double the registers the row occupies
                    c += ((w & 0xffffu) >= t) + ((w >> 16) >= t);
                }
            }
            return c;
        };

        // ---- largest key T with count(key >= T) >= k: bisection, invariant count(>= lo) >= k > count(>= hi) ----
        uint32_t lo = 1u, hi = 0x10000u;  // key 0 only marks indices past the end
        int n_ge = V;                     // count(key >= lo): every real key is >= 1
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            const int cnt = block_sum(count_ge(mid), red, wave, lane);
            if (cnt >= k) { lo = mid; n_ge = cnt; }
            else hi = mid;
        }
        const uint32_t T = lo;
        const int n_gt = block_sum(count_ge(T + 1), red, wave, lane);
        const int need_eq = k - n_gt;  // >= 1: that many elements with key == T are taken, lowest indices first
        // ---- smallest index bound M with count(key == T and index < M) >= need_eq ----
        auto count_eq_below = [&](int m) {
            int c = 0;
#pragma unroll
            for (int j = 0; j < NVEC; ++j) {
                int d = m - (j * kMixThreads + tid) * 8;  // index e of this piece is below the bound iff e < d
                TAH_OPAQUE1(d);                           // (compared with constants: no per-element index registers)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint32_t w = keys[j][q];
                    TAH_OPAQUE1(w);
                    c += ((w & 0xffffu) == T) && (2 * q < d);
                    c += ((w >> 16) == T) && (2 * q + 1 < d);
                }
            }
            return c;
        };
        int mlo = 0, mhi = V;  // invariant: count(< mlo) < need_eq <= count(< mhi)
        // (the usual case needs no search: every element with key == T is taken)
        if (n_ge - n_gt > need_eq) {
            while (mhi - mlo > 1) {
                const int mid = (mlo + mhi) >> 1;
                if (block_sum(count_eq_below(mid), red, wave, lane) >= need_eq) mhi = mid;
                else mlo = mid;
            }
        }
        const int M = mhi;

        // ---- gather the k selected (index, value) pairs ----
#pragma unroll
        for (int j = 0; j < NVEC; ++j) {
            int i0 = (j * kMixThreads + tid) * 8;
            TAH_OPAQUE1(i0);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                uint32_t w = keys[j][e / 2];
                TAH_OPAQUE1(w);
                const uint32_t key = (w >> (16 * (e % 2))) & 0xffffu;
                if (key > T || (key == T && e < M - i0)) {
                    const int s = atomicAdd(&n_sel, 1);
                    if (s < kMaxTopk) {
                        sel_idx[s] = i0 + e;
                        sel_val[s] = key_value(key);
                    }
                }
            }
        }
    }
    __syncthreads();
    const int n = n_sel < kMaxTopk ? n_sel : kMaxTopk;  // == k
    if (p.vals && tid < n) {
        // largest first, equal values by ascending index: place = how many selected entries come before this one
        const float mine = sel_val[tid];
        const int mine_idx = sel_idx[tid];
        int place = sorted ? tid : 0;
        if (!sorted)
            for (int i = 0; i < n; ++i) place += (sel_val[i] > mine) || (sel_val[i] == mine && sel_idx[i] < mine_idx);
        p.vals[(int64_t)row * p.v_rs + place] = (__bf16)mine;  // (exact: the value came from a bf16)
        if (p.idxs) p.idxs[(int64_t)row * p.v_rs + place] = mine_idx;
    }
    if (!p.out) return;  // only the values were asked for (uniform)
    // order by index (all distinct): rank = number of selected entries with a smaller index
    float vmax = kNegInf;
    if (sorted) vmax = sel_val[0];
    else
        for (int i = 0; i < n; ++i) vmax = fmaxf(vmax, sel_val[i]);
    {   // rank by index among the selected, the comparisons spread over the workgroup
        int cp = 64;
        while (cp < n) cp <<= 1;
        const int nsl = kMixThreads / cp, c = tid & (cp - 1), sl = tid / cp;
        if (c < n) {
            const int mine_idx = sel_idx[c];
            int r = 0;
#pragma unroll 4
            for (int i = sl; i < n; i += nsl) r += sel_idx[i] < mine_idx ? 1 : 0;
            if (r) atomicAdd(&ord_rank[c], r);
        }
    }
    __syncthreads();
    if (tid < n) {
        const int rank = ord_rank[tid];
        ord_idx[rank] = sel_idx[tid];
        ord_w[rank] = fast_exp2((sel_val[tid] - vmax) * kLog2e);
    }
    __syncthreads();
    float denom = 0.f;  // same order in every thread and every run; four at a time, zeros past the end
    for (int i = 0; i < n; i += 4) {
        const f32x4s w4 = *reinterpret_cast<const f32x4s*>(&ord_w[i]);
        denom += w4[0];
        denom += w4[1];
        denom += w4[2];
        denom += w4[3];
    }
    const float inv = 1.0f / denom;

    // ---- mix: thread = (part, column group of 8); a part takes every parts-th selected row ----
    const int H = p.hidden, cgs = H / 8;
    float* partial = reinterpret_cast<float*>(dyn);
    const int parts = cgs >= kMixThreads ? 1 : kMixThreads / cgs;
    for (int cg0 = 0; cg0 < cgs; cg0 += kMixThreads) {
        const int part = cgs >= kMixThreads ? 0 : tid / cgs;
        const int cg = cg0 + (cgs >= kMixThreads ? tid : tid % cgs);
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (cg < cgs && part < parts) {
            // thirteen embedding rows are fetched before the first of them is used (one workgroup per token: what
            // this loop waits for is memory latency), and added in the same order as one by one
            constexpr int kAhead = 13;
            for (int i = part; i < n; i += parts * kAhead) {
                bf16x8 e[kAhead];
#pragma unroll
                for (int u = 0; u < kAhead; ++u) {
                    const int ii = i + u * parts;
                    if (ii < n) e[u] = *reinterpret_cast<const bf16x8*>(p.emb + (int64_t)ord_idx[ii] * p.e_rs + cg * 8);
                }
#pragma unroll
                for (int u = 0; u < kAhead; ++u) {
                    const int ii = i + u * parts;
                    if (ii < n) {
                        // probability rounded to bf16 (softmax output of the bf16 arithmetic), product rounded to bf16
                        const float pr = round_bf16(ord_w[ii] * inv);
#pragma unroll
                        for (int c = 0; c < 8; ++c) acc[c] += round_bf16(pr * (float)e[u][c]);
                    }
                }
            }
#pragma unroll
            for (int c = 0; c < 8; ++c) partial[(int64_t)part * H + cg * 8 + c] = acc[c];
        }
        __syncthreads();
        if (cg < cgs && part == 0) {
            bf16x8 o;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                float s = 0.f;
                for (int q = 0; q < parts; ++q) s += partial[(int64_t)q * H + cg * 8 + c];
                o[c] = (__bf16)s;
            }
            *reinterpret_cast<bf16x8*>(p.out + (int64_t)row * p.o_rs + cg * 8) = o;
            // columns 8 cg ... of row `row`: step cg / 4, lane row % 16 + 16 (cg % 4) of the packed rows form
            if (p.outp) p.outp[((int64_t)(cg / 4) * 2 + row / 16) * 64 + (row % 16) + 16 * (cg % 4)] = o;
        }
        __syncthreads();
    }
}

}  // namespace
}  // namespace tah

extern "C" int tah_topk_mix(const tah_topk_mix_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    const bool mix = a->out != nullptr;  // without `out` only values_out is produced
    if (a->rows < 0 || a->vocab <= 0 || a->topk <= 0 || (mix && a->hidden <= 0)) return TAH_E_SHAPE;
    if (a->topk > kMaxTopk || a->vocab > kMaxVec * 8 * kMixThreads || (mix && a->hidden % 8 != 0)) return TAH_E_SHAPE;
    if (a->out_packed && (!mix || a->rows > 32 || a->hidden % 32 != 0)) return TAH_E_SHAPE;
    if (a->values_out && a->values_row_stride < (a->topk < a->vocab ? a->topk : a->vocab)) return TAH_E_SHAPE;
    if (a->rows == 0) return TAH_OK;
    if (!a->logits || (!mix && !a->values_out) || (mix && !a->embedding)) return TAH_E_NULL;
    if (reinterpret_cast<uintptr_t>(a->values_out) & 1) return TAH_E_ALIGN;
    if (a->indices_out && !a->values_out) return TAH_E_NULL;
    if (reinterpret_cast<uintptr_t>(a->indices_out) & 3) return TAH_E_ALIGN;
    if (reinterpret_cast<uintptr_t>(a->out_packed) & 15) return TAH_E_ALIGN;
    if ((reinterpret_cast<uintptr_t>(a->embedding) & 15) || (reinterpret_cast<uintptr_t>(a->out) & 15) ||
        (reinterpret_cast<uintptr_t>(a->logits) & 1) || a->embedding_row_stride % 8 || a->out_row_stride % 8)
        return TAH_E_ALIGN;
    MixParams p;
    p.logits = static_cast<const __bf16*>(a->logits);
    p.emb = static_cast<const __bf16*>(a->embedding);
    p.out = static_cast<__bf16*>(a->out);
    p.outp = static_cast<bf16x8*>(a->out_packed);
    p.zero_disabled = a->zero_disabled ? 1 : 0;
    p.vals = static_cast<__bf16*>(a->values_out);
    p.idxs = a->indices_out;
    p.v_rs = a->values_row_stride;
    p.row_enable = a->row_enable;
    p.l_rs = a->logits_row_stride; p.e_rs = a->embedding_row_stride; p.o_rs = a->out_row_stride;
    p.rows = a->rows; p.vocab = a->vocab; p.hidden = a->hidden; p.topk = a->topk;
    const int cgs = mix ? a->hidden / 8 : 1;
    const int parts = cgs >= kMixThreads ? 1 : kMixThreads / cgs;
    const size_t smem = mix ? (size_t)parts * a->hidden * sizeof(float) : 0;
    if (smem > 48 * 1024) return TAH_E_SHAPE;  // (32 KiB whenever hidden < 8192)
    const int nvec = (a->vocab + 8 * kMixThreads - 1) / (8 * kMixThreads);
    const dim3 grid(a->rows), block(kMixThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (nvec <= 2) hipLaunchKernelGGL(topk_mix_kernel<2>, grid, block, smem, st, p);
    else if (nvec <= 8) hipLaunchKernelGGL(topk_mix_kernel<8>, grid, block, smem, st, p);
    else if (nvec <= 14) hipLaunchKernelGGL(topk_mix_kernel<14>, grid, block, smem, st, p);
    else hipLaunchKernelGGL(topk_mix_kernel<kMaxVec>, grid, block, smem, st, p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}
