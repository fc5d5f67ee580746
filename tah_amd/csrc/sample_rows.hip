// One token per row from temperature / min_p / top_p filtered logits, without sorting the vocabulary, gfx950.
//
// A row of bf16 logits has at most 65536 distinct values, and a token's probability depends on its value only.
// So the row is loaded once into registers as order-preserving 16-bit keys and counted into a histogram over
// the key space (LDS, 32768 keys at a time: the half nearest to the row maximum, then the far half unless its tokens
// are too light to change a float32 sum); the mass of a key is its count
// times exp((value - max) / T), a prefix sum over the keys in descending order gives the mass that precedes every
// key in the order a descending sort would put the tokens in, and both the top_p cut (the first token whose
// preceding mass exceeds top_p of the total) and the draw (the token at which the preceding kept mass passes
// u times the kept total) are located on the keys.  Tokens of equal value are told apart by vocabulary index,
// lower first, which is the order a stable descending sort leaves them in.  No pass over the row evaluates an
// exponential per token (only the optional probability output does).
//
// One workgroup of 1024 threads per row.
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>

#include "duo_device.h"
#include "row_keys.h"
#include "tah_duo.h"

namespace tah {
namespace {

constexpr int kSmpThreads = 1024;
constexpr int kSmpWaves = kSmpThreads / kWave;
constexpr int kSmpMaxVec = 19;      // 16-byte pieces of the row per thread: vocabularies up to 19 * 8 * 1024 = 155648
constexpr int kWinKeys = 32768;     // keys per histogram window
constexpr int kBinsPerThread = kWinKeys / kSmpThreads;  // 32: a thread's group of consecutive keys
constexpr int kHistWords = kWinKeys + kWinKeys / 32;    // bin b lives at word b + b / 32 (a thread's 32 bins: stride 33)
constexpr size_t kSmpSmem = (size_t)kHistWords * sizeof(uint32_t);
constexpr uint32_t kNoCut = 0x20000u;  // a distance past every key

struct SampleParams {
    const __bf16* logits;
    const __bf16* prev;
    const int32_t* add_prev;
    const uint8_t* row_enable;
    const float* uniforms;
    int64_t* tokens;
    float* probs;
    int64_t l_rs, p_rs, pr_rs;
    int32_t rows, vocab;
    float c;         // log2(e) / temperature
    float top_p;
    float min_p_l2;  // log2(min_p), -inf without the filter
};

// a + b of two packed bf16 pairs, each sum rounded to bf16 (what the eager bf16 addition gives)
__device__ __forceinline__ uint32_t add_bf16x2(uint32_t a, uint32_t b) {
    const f32x2 s = {__uint_as_float(a << 16) + __uint_as_float(b << 16),
                     __uint_as_float(a & 0xffff0000u) + __uint_as_float(b & 0xffff0000u)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(s, bf16x2e));
}

// bit e of the result: element e of the 16-byte piece (two keys per dword, low half first) equals `key`
__device__ __forceinline__ uint32_t match_mask(const uint32_t (&kv)[4], uint32_t key) {
    const uint32_t kk = key | (key << 16);
    uint32_t m = 0u;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t w = kv[q];
        TAH_OPAQUE1(w);
        const uint32_t x = w ^ kk;
        m |= ((x & 0xffffu) == 0u ? 1u : 0u) << (2 * q);
        m |= ((x >> 16) == 0u ? 1u : 0u) << (2 * q + 1);
    }
    return m;
}

template <class T>
__device__ __forceinline__ T wave_incl_scan(T x, int lane) {
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const T v = __shfl_up(x, o);
        if (lane >= o) x += v;
    }
    return x;
}

template <int NVEC, bool kProbs>
__global__ __launch_bounds__(kSmpThreads) void sample_rows_kernel(const SampleParams p) {
    __shared__ float wtot[kSmpWaves];
    __shared__ int wv[kSmpMaxVec][kSmpWaves];  // per piece and wave: tokens equal to the key looked for
    __shared__ uint32_t mini[kBinsPerThread];  // counts of one thread's group of keys, rebuilt from the row
    __shared__ int s_kmax;
    __shared__ int s_code[2];
    HIP_DYNAMIC_SHARED(unsigned char, dyn)
    uint32_t* hist = reinterpret_cast<uint32_t*>(dyn);

    const int row = blockIdx.x;
    if (p.row_enable && !p.row_enable[row]) return;  // uniform per workgroup
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int V = p.vocab;
    const __bf16* lrow = p.logits + (int64_t)row * p.l_rs;
    const __bf16* prow = (p.prev && p.add_prev && p.add_prev[row] != 0) ? p.prev + (int64_t)row * p.p_rs : nullptr;
    if (tid == 0) {
        s_kmax = 0;
        s_code[0] = 0;
        s_code[1] = 0;
    }

    // ---- the row as keys: piece j of thread t covers indices (j * 1024 + t) * 8 .. + 7 (coalesced loads) ----
    uint32_t keys[NVEC][4];  // two keys per dword, low half = even index; key 0 = past the end of the row
    auto load_piece = [&](const __bf16* base, int i0) {
        u32x4 w = {0u, 0u, 0u, 0u};
        if (i0 + 8 <= V && ((reinterpret_cast<uintptr_t>(base + i0) & 15) == 0)) {
            w = *reinterpret_cast<const u32x4*>(base + i0);
        } else if (i0 < V) {
            const uint16_t* h = reinterpret_cast<const uint16_t*>(base);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t b = i0 + e < V ? h[i0 + e] : 0u;
                w[e / 2] |= b << (16 * (e % 2));
            }
        }
        return w;
    };
    constexpr int kLoadGroup = 4;
    // Rows that start on a 16-byte boundary and have a multiple of eight entries (any real vocabulary) are loaded without
    // a branch: a piece lies inside the row or behind it as a whole, the loads of pieces behind it go to the row's start
    // and their keys become 0 by a select.  (With a branch around a load the compiler waits for it where the branch ends:
    // one load in flight per thread instead of a group's.)
    const bool whole_pieces = V % 8 == 0 && (reinterpret_cast<uintptr_t>(lrow) & 15) == 0 && (reinterpret_cast<uintptr_t>(prow) & 15) == 0;
    auto load_whole_pieces = [&](auto with_prev) __attribute__((always_inline)) {
        constexpr bool kPrev = decltype(with_prev)::value;
#pragma unroll
        for (int j0 = 0; j0 < NVEC; j0 += kLoadGroup) {
            u32x4 w[kLoadGroup], w2[kPrev ? kLoadGroup : 1];
#pragma unroll
            for (int j = j0; j < j0 + kLoadGroup && j < NVEC; ++j) {
                const int i0 = (j * kSmpThreads + tid) * 8, at = i0 < V ? i0 : 0;
                w[j - j0] = *reinterpret_cast<const u32x4*>(lrow + at);
                if constexpr (kPrev) w2[j - j0] = *reinterpret_cast<const u32x4*>(prow + at);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = j0; j < j0 + kLoadGroup && j < NVEC; ++j) {
                const bool inside = (j * kSmpThreads + tid) * 8 < V;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint32_t x = w[j - j0][q];
                    if constexpr (kPrev) x = add_bf16x2(w2[j - j0][q], x);
                    keys[j][q] = inside ? order_keys2(x) : 0u;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if (whole_pieces) {  // (uniform, and so is prow)
        if (prow) load_whole_pieces(std::true_type{});
        else load_whole_pieces(std::false_type{});
    } else
#pragma unroll
    for (int j0 = 0; j0 < NVEC; j0 += kLoadGroup) {
#pragma unroll
        for (int j = j0; j < j0 + kLoadGroup && j < NVEC; ++j) {
            const int i0 = (j * kSmpThreads + tid) * 8;
            u32x4 w = load_piece(lrow, i0);
            if (prow) {  // (uniform)
                const u32x4 w2 = load_piece(prow, i0);
#pragma unroll
                for (int q = 0; q < 4; ++q) w[q] = add_bf16x2(w2[q], w[q]);
            }
            if ((j + 1) * kSmpThreads * 8 <= V) {  // (uniform) the whole piece lies inside the row, for every thread
#pragma unroll
                for (int q = 0; q < 4; ++q) keys[j][q] = order_keys2(w[q]);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint32_t lo = order_key(w[q] & 0xffffu), hi = order_key(w[q] >> 16);
                    if (i0 + 2 * q >= V) lo = 0u;
                    if (i0 + 2 * q + 1 >= V) hi = 0u;
                    keys[j][q] = lo | (hi << 16);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- the largest key -------------------------------------------------------------------------------
    u16x2 tmax2 = {0, 0};
#pragma unroll
    for (int j = 0; j < NVEC; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) tmax2 = __builtin_elementwise_max(tmax2, __builtin_bit_cast(u16x2, keys[j][q]));
    uint32_t tmax = tmax2.x > tmax2.y ? tmax2.x : tmax2.y;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const uint32_t o = __shfl_xor(tmax, m);
        tmax = o > tmax ? o : tmax;
    }
    __syncthreads();  // s_kmax, s_code initialised
    if (lane == 0) atomicMax(&s_kmax, (int)tmax);
    __syncthreads();
    const uint32_t kmax = (uint32_t)s_kmax;  // >= 1: the row has at least one token
    const float vmax = key_value(kmax);
    // exp((value - max) / T) as a power of two, and its exponent (what min_p compares)
    auto arg_of = [&](uint32_t key) { return (key_value(key) - vmax) * p.c; };
    auto mass_of = [&](uint32_t key) { return fast_exp2(arg_of(key)); };

    // ---- min_p as a bound on the distance from the largest key: the filter keeps keys in [kthr, kmax] ----
    uint32_t kthr = 1u;
    if (p.min_p_l2 > -INFINITY) {
        uint32_t lo = 1u, hi = kmax;  // hi passes (its exponent is 0 >= log2(min_p)); smallest key that passes
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (arg_of(mid) >= p.min_p_l2) hi = mid;
            else lo = mid + 1u;
        }
        kthr = lo;
    }
    const uint32_t dmax = kmax - kthr;  // distances 0 .. dmax survive min_p

    // Histogram of the surviving tokens over the distances [wbase, wbase + 32768) from the largest key.
    auto build_hist = [&](uint32_t wbase) {
        uint32_t* mine = hist + tid * (kBinsPerThread + 1);
#pragma unroll
        for (int i = 0; i < kBinsPerThread + 1; ++i) mine[i] = 0u;  // (33 words per thread cover the padded array)
        __syncthreads();
        const uint32_t span = dmax - wbase < (uint32_t)kWinKeys - 1u ? dmax - wbase : (uint32_t)kWinKeys - 1u;  // rel <= span
        // rel = kmax - wbase - key, both halves of a dword at once in 16-bit arithmetic: keys above the window wrap to
        // 32768 and more, keys below it (and key 0, past the end of the row) stay above span as they are
        const uint32_t kb2 = ((kmax - wbase) & 0xffffu) * 0x10001u;
#pragma unroll
        for (int j = 0; j < NVEC; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t w = keys[j][q];
                TAH_OPAQUE1(w);
                const uint32_t r2 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, kb2) - __builtin_bit_cast(u16x2, w));
                const uint32_t r0 = r2 & 0xffffu, r1 = r2 >> 16;
                if (r0 <= span) atomicAdd(&hist[r0 + (r0 >> 5)], 1u);
                if (r1 <= span) atomicAdd(&hist[r1 + (r1 >> 5)], 1u);
            }
        }
        __syncthreads();
    };
    // This thread's group of 32 keys of the window: their mass, the mass of the groups before it in the window
    // (exclusive prefix in descending key order) and the window's total.
    auto scan_window = [&](uint32_t wbase, float& mass, float& excl, float& total) {
        const uint32_t* mine = hist + tid * (kBinsPerThread + 1);
        float m = 0.f;
#pragma unroll 4
        for (int i = 0; i < kBinsPerThread; ++i) {
            const uint32_t c = mine[i];
            if (c != 0u) m += (float)c * mass_of(kmax - (wbase + tid * kBinsPerThread + i));
        }
        const float incl = wave_incl_scan(m, lane);
        const float before = __shfl_up(incl, 1);
        __syncthreads();  // earlier readers of wtot are done
        if (lane == kWave - 1) wtot[wave] = incl;
        __syncthreads();
        float pre = 0.f, tot = 0.f;
#pragma unroll
        for (int w = 0; w < kSmpWaves; ++w) {
            const float t = wtot[w];
            pre += w < wave ? t : 0.f;
            tot += t;
        }
        mass = m;
        excl = pre + (lane ? before : 0.f);
        total = tot;
    };

    // The far window is needed only if its tokens can change a float32 sum: each of them weighs at most the mass of the
    // first key behind the near window, the near window weighs at least 1 (the largest token), and when all V of them
    // together stay below 2^-26 (a language model's row: the far window starts tens of e-foldings below the maximum)
    // the total is the near window's to the last bit, no far token can precede the cut, and the draw cannot reach one.
    // Otherwise the far window goes first, so that the near one (where cut and draw fall on all but flat rows) is
    // the one that stays in LDS.
    float mass1 = 0.f, excl1 = 0.f, total1 = 0.f;
    if (dmax >= (uint32_t)kWinKeys && (float)V * mass_of(kmax - (uint32_t)kWinKeys) > 1.4901161e-8f) {  // (uniform)
        build_hist(kWinKeys);
        scan_window(kWinKeys, mass1, excl1, total1);
        __syncthreads();  // the scan's reads of the histogram are done before it is cleared
    }
    float mass0, excl0, total0;
    build_hist(0u);
    scan_window(0u, mass0, excl0, total0);
    constexpr int lds_window = 0;  // which window's histogram LDS holds
    const float S = total0 + total1;  // mass of everything min_p keeps
    const float g0 = excl0, g1 = total0 + excl1;  // mass before this thread's group, window 0 / window 1

    // Counts of group `code` (window code >> 10, thread code & 1023): from the histogram in LDS, or counted again.
    auto group_counts = [&](int code) -> const uint32_t* {
        const int gt = code & (kSmpThreads - 1);
        if ((code >> 10) == lds_window) return hist + gt * (kBinsPerThread + 1);
        __syncthreads();  // earlier readers of mini are done
        if (tid < kBinsPerThread) mini[tid] = 0u;
        __syncthreads();
        const uint32_t gbase = (uint32_t)(code >> 10) * (uint32_t)kWinKeys + (uint32_t)gt * kBinsPerThread;
        const uint32_t span = dmax - gbase < (uint32_t)kBinsPerThread - 1u ? dmax - gbase : (uint32_t)kBinsPerThread - 1u;
        const uint32_t kb = kmax - gbase;  // rel = kb - key
#pragma unroll
        for (int j = 0; j < NVEC; ++j) {
            bool any = false;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t w = keys[j][q];
                TAH_OPAQUE1(w);
                any |= (kb - (w & 0xffffu)) <= span || (kb - (w >> 16)) <= span;
            }
            if (!any) continue;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t w = keys[j][q];
                TAH_OPAQUE1(w);
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t key = h ? (w >> 16) : (w & 0xffffu);
                    const uint32_t rel = kb - key;
                    if (rel <= span && key != 0u) atomicAdd(&mini[rel], 1u);
                }
            }
        }
        __syncthreads();
        return mini;
    };
    // The last group, in descending key order, that holds mass and whose preceding mass is at most `t` (and that does
    // not lie behind group `limit`): the group in which the running mass passes `t`.
    auto locate = [&](float t, int limit, int slot) {
        int code = 0;
        if (mass0 > 0.f && g0 <= t) code = tid + 1;
        if (mass1 > 0.f && g1 <= t) code = kSmpThreads + tid + 1;
        if (code > limit + 1) code = (mass0 > 0.f && g0 <= t && tid <= limit) ? tid + 1 : 0;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) {
            const int o = __shfl_xor(code, m);
            code = o > code ? o : code;
        }
        if (lane == 0 && code != 0) atomicMax(&s_code[slot], code);
        __syncthreads();
        const int got = s_code[slot];
        return got > 0 ? got - 1 : 0;
    };
    auto group_before = [&](int code) {  // mass before group `code`: its owner's value, read through LDS
        __syncthreads();
        if (tid == (code & (kSmpThreads - 1))) wtot[0] = (code >> 10) ? g1 : g0;
        __syncthreads();
        return wtot[0];
    };

    // ---- top_p: tokens at distance < dcut, and the first ncut (by index) of those at distance dcut, are kept ----
    uint32_t dcut = kNoCut;
    int ncut = 0, cut_code = 2 * kSmpThreads - 1;
    float Z = S;
    if (p.top_p < 1.f && S > 0.f) {  // (uniform)
        const float target = p.top_p * S;
        cut_code = locate(target, 2 * kSmpThreads - 1, 0);
        const uint32_t* cnt = group_counts(cut_code);
        const uint32_t gbase = (cut_code >> 10) * (uint32_t)kWinKeys + (uint32_t)(cut_code & (kSmpThreads - 1)) * kBinsPerThread;
        float A = group_before(cut_code);
        for (int i = 0; i < kBinsPerThread && dcut == kNoCut; ++i) {
            const uint32_t c = cnt[i];
            if (c == 0u) continue;
            const uint32_t d = gbase + i;
            const float e = mass_of(kmax - d);
            if (A > target) {  // every token from here on has more than top_p before it
                dcut = d;
                ncut = 0;
                Z = A;
                break;
            }
            // token j of the c equal ones has A + j e before it: kept while that is at most the target
            int kept = (int)c;
            if (e > 0.f) {
                const float q = (target - A) / e;
                if (q < (float)c) kept = (int)q + 1 < (int)c ? (int)q + 1 : (int)c;
            }
            if (kept < (int)c) {
                dcut = d;
                ncut = kept;
                Z = A + (float)kept * e;
                break;
            }
            A += (float)c * e;
        }
        if (dcut == kNoCut) {  // the whole group is kept and the next one that holds mass lies past the target
            dcut = gbase + kBinsPerThread;
            ncut = 0;
            Z = A;
        }
    }

    // Tokens equal to `key`, per piece and wave, into wv (index order = piece, then thread, then place in the piece).
    auto build_tie_table = [&](uint32_t key) {
        __syncthreads();  // earlier readers of wv are done
        if (tid < kSmpMaxVec * kSmpWaves) (&wv[0][0])[tid] = 0;
        __syncthreads();
        const uint32_t kk = key | (key << 16);
#pragma unroll
        for (int j = 0; j < NVEC; ++j) {
            // a 16-bit half of w ^ kk that is zero: a match (the usual zero-half test, exact for the lower half and
            // never silent about a match; the full mask is formed only where there may be one)
            uint32_t hit = 0u;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t w = keys[j][q];
                TAH_OPAQUE1(w);
                const uint32_t x = w ^ kk;
                hit |= (x - 0x00010001u) & ~x & 0x80008000u;
            }
            if (__ballot(hit != 0u) == 0ull) continue;
            int c = hit ? __builtin_popcount(match_mask(keys[j], key)) : 0;
            if (__ballot(c != 0) == 0ull) continue;
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) c += __shfl_xor(c, m);
            if (lane == 0) wv[j][wave] = c;
        }
        __syncthreads();
    };

    // ---- the draw: the token at which the kept mass, in the same order, passes u Z --------------------------
    if (p.tokens) {
        const float tu = p.uniforms[row] * Z;
        const int dcode = locate(tu, cut_code, 1);
        const uint32_t* cnt = group_counts(dcode);
        const uint32_t gbase = (dcode >> 10) * (uint32_t)kWinKeys + (uint32_t)(dcode & (kSmpThreads - 1)) * kBinsPerThread;
        float A = group_before(dcode);
        uint32_t du = kmax - kmax;  // distance of the drawn token's key
        int ju = 0;                 // its place among the kept tokens of that key
        bool found = false;
        for (int i = 0; i < kBinsPerThread && !found; ++i) {
            const uint32_t c = cnt[i];
            const uint32_t d = gbase + i;
            const int kept = d < dcut ? (int)c : (d == dcut ? ncut : 0);
            if (kept == 0) continue;
            const float e = mass_of(kmax - d);
            du = d;
            ju = kept - 1;  // (the last kept token, should rounding carry the target past the end)
            if (tu < A + (float)kept * e) {
                int j = e > 0.f ? (int)((tu - A) / e) : 0;
                j = j < 0 ? 0 : j;
                ju = j < kept ? j : kept - 1;
                found = true;
            }
            A += (float)kept * e;
        }
        const uint32_t keyu = kmax - du;
        build_tie_table(keyu);
        int before = 0, vstar = -1, total = 0;
#pragma unroll
        for (int j = 0; j < NVEC; ++j) {
            int t = 0;
#pragma unroll
            for (int w = 0; w < kSmpWaves; ++w) t += wv[j][w];
            if (vstar < 0 && ju < total + t) {
                vstar = j;
                before = total;
            }
            total += t;
        }
        if (vstar < 0) {  // (ju past the tokens found: cannot happen while histogram and row agree; take the last one)
#pragma unroll
            for (int j = 0; j < NVEC; ++j) {
                int t = 0;
#pragma unroll
                for (int w = 0; w < kSmpWaves; ++w) t += wv[j][w];
                if (t > 0) vstar = j;
            }
            before = 0;
            ju = 0x7fffffff;
        }
        if (vstar >= 0) {
            uint32_t mask = 0u;
#pragma unroll
            for (int j = 0; j < NVEC; ++j)
                if (j == vstar) mask = match_mask(keys[j], keyu);  // (uniform)
            const int c = __builtin_popcount(mask);
            int pre = before;
            int wave_tot = 0;
#pragma unroll
            for (int w = 0; w < kSmpWaves; ++w) {
                const int t = wv[vstar][w];
                pre += w < wave ? t : 0;
                wave_tot += t;
            }
            const int incl = wave_incl_scan(c, lane);
            const int first = pre + incl - c;  // index-order rank of this thread's first match
            int want = ju;
            if (want == 0x7fffffff) want = wave_tot - 1;  // (fallback: the piece's last match)
            if (c > 0 && want >= first && want < first + c) {
                int r = want - first;
                uint32_t m = mask;
                while (r-- > 0) m &= m - 1u;
                const int e = __builtin_ctz(m);
                p.tokens[row] = (int64_t)(vstar * kSmpThreads + tid) * 8 + e;
            }
        } else if (tid == 0) {
            p.tokens[row] = 0;
        }
    }

    // ---- optionally the distribution itself: softmax, min_p, top_p, each renormalised ------------------------
    if constexpr (kProbs) {
        float* orow = p.probs + (int64_t)row * p.pr_rs;
        const float inv = Z > 0.f ? 1.f / Z : 0.f;
        const uint32_t kcut = dcut <= dmax ? kmax - dcut : 0u;  // key of the partly kept tokens (0: none)
        if (kcut != 0u && ncut > 0) build_tie_table(kcut);
        int vbefore = 0;
#pragma unroll
        for (int j = 0; j < NVEC; ++j) {
            const int i0 = (j * kSmpThreads + tid) * 8;
            int rank = 0;
            uint32_t tmask = 0u;
            if (kcut != 0u && ncut > 0) {  // (uniform)
                tmask = match_mask(keys[j], kcut);
                const int c = __builtin_popcount(tmask);
                const int incl = wave_incl_scan(c, lane);
                int pre = vbefore, tot = 0;
#pragma unroll
                for (int w = 0; w < kSmpWaves; ++w) {
                    const int t = wv[j][w];
                    pre += w < wave ? t : 0;
                    tot += t;
                }
                rank = pre + incl - c;
                vbefore += tot;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if (i0 + e >= V) break;
                uint32_t w = keys[j][e / 2];
                TAH_OPAQUE1(w);
                const uint32_t key = (e % 2) ? (w >> 16) : (w & 0xffffu);
                const uint32_t d = kmax - key;
                bool keep = d <= dmax && d < dcut;
                if (d == dcut && d <= dmax && ncut > 0) {
                    keep = rank < ncut;
                    rank += 1;
                }
                orow[i0 + e] = keep ? mass_of(key) * inv : 0.f;
            }
        }
    }
}

}  // namespace
}  // namespace tah

extern "C" int tah_sample_rows(const tah_sample_rows_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    if (a->rows < 0 || a->vocab <= 0 || a->vocab > kSmpMaxVec * 8 * kSmpThreads) return TAH_E_SHAPE;
    if (!(a->temperature > 0.f) || !(a->top_p > 0.f) || a->min_p < 0.f || a->min_p > 1.f) return TAH_E_SHAPE;
    if (a->rows == 0) return TAH_OK;
    if (!a->logits || (!a->tokens && !a->probs) || (a->tokens && !a->uniforms)) return TAH_E_NULL;
    if (a->add_prev && !a->logits_prev) return TAH_E_NULL;
    if ((reinterpret_cast<uintptr_t>(a->logits) & 1) || (reinterpret_cast<uintptr_t>(a->logits_prev) & 1) ||
        (reinterpret_cast<uintptr_t>(a->tokens) & 7) || (reinterpret_cast<uintptr_t>(a->probs) & 3) ||
        (reinterpret_cast<uintptr_t>(a->uniforms) & 3) || (reinterpret_cast<uintptr_t>(a->add_prev) & 3))
        return TAH_E_ALIGN;
    if (a->probs && a->probs_row_stride < a->vocab) return TAH_E_SHAPE;
    SampleParams p;
    p.logits = static_cast<const __bf16*>(a->logits);
    p.prev = static_cast<const __bf16*>(a->logits_prev);
    p.add_prev = a->add_prev;
    p.row_enable = a->row_enable;
    p.uniforms = a->uniforms;
    p.tokens = a->tokens;
    p.probs = a->probs;
    p.l_rs = a->logits_row_stride; p.p_rs = a->prev_row_stride; p.pr_rs = a->probs_row_stride;
    p.rows = a->rows; p.vocab = a->vocab;
    p.c = 1.4426950408889634f / a->temperature;
    p.top_p = a->top_p;
    p.min_p_l2 = a->min_p > 0.f ? log2f(a->min_p) : -INFINITY;
    const int nvec = (a->vocab + 8 * kSmpThreads - 1) / (8 * kSmpThreads);
    const dim3 grid(a->rows), block(kSmpThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define TAH_SAMPLE_LAUNCH(N)                                                                                                  \
    do {                                                                                                                      \
        auto* kern = a->probs ? &sample_rows_kernel<N, true> : &sample_rows_kernel<N, false>;                                 \
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,              \
                                (int)kSmpSmem) != hipSuccess)                                                                 \
            return TAH_E_LAUNCH;                                                                                              \
        hipLaunchKernelGGL(kern, grid, block, kSmpSmem, st, p);                                                               \
    } while (0)
    if (nvec <= 2) TAH_SAMPLE_LAUNCH(2);
    else if (nvec <= 8) TAH_SAMPLE_LAUNCH(8);
    else TAH_SAMPLE_LAUNCH(kSmpMaxVec);
#undef TAH_SAMPLE_LAUNCH
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}
