// Duo-causal decode step against the KV cache (bandwidth-bound), gfx950.
//
// Split-K: one workgroup (4 waves) streams one chunk (1024 rows, or 256 when few rows are in play) of one kv head of
// one query's sequence, from the depth-0 slab or (depth-1 queries only) the
// depth-1 slab, for all G = Hq/Hkv query heads at once so K and V are read from
// HBM exactly once.  A wave covers 256 consecutive rows; each load instruction
// moves 1 KiB of contiguous cache (4 rows x 256 B, 16 B per lane).  Scores use
// v_dot2_f32_bf16 on the packed bf16 pairs plus a 16-lane DPP reduction; the
// online softmax runs per group of 4 rows so the accumulator is rescaled once
// per 16 rows.  Partial (max, sum, acc) triples go to a workspace and a second
// small kernel merges the chunks of each (query, head), eight chunks at a time.
// (Merging in the workgroup that finishes last would need device-scope fences,
// which cost an L2 write-back per item across the eight XCDs; a persistent grid
// striding over the items balanced worse than the hardware dispatcher.)
// A call whose (query, kv head) pairs alone fill the chip, with slabs of at most 4096 rows, skips all that: one
// workgroup per pair walks both segments and writes the finished output (duo_decode_whole_kernel).
#include <hip/hip_runtime.h>

#include <mutex>

#include "duo_device.h"
#include "tah_duo.h"

// Split-K partials of tah_duo_decode_static: device memory owned by the library (every GPU the library
// runs on holds its own copy until the process ends), for callers that cannot allocate.  In host code this
// name is only a handle for hipGetSymbolAddress; the kernels get the address that call returned.
static __device__ __align__(256) unsigned char scratch[TAH_DUO_STATIC_SCRATCH_BYTES];

namespace tah {
namespace {

constexpr int kD = 128;
constexpr int kChunk = 1024;           // rows per workgroup when there are rows enough to fill the chip
constexpr int kChunkSmall = 256;       // ... and when there are not (few sequences, short contexts): four
                                       // times the workgroups, so that enough loads are in flight
constexpr int kDecThreads = 256;     // 4 waves x (chunk / 4) rows
constexpr int kUnroll = 4;           // loads of 4 rows in flight per wave and tensor
constexpr int kPart = kD + 2;        // acc[128], m, l  (floats per partial)


struct Seg {
    const __bf16 *k, *v;
    const int32_t *pos, *start, *len;
    int64_t k_rs, k_hs, v_rs, v_hs;
    int32_t capacity;
};
struct DecParams {
    const __bf16* q;
    __bf16* o;
    __bf16* op;  // the output once more in the rows form of the linear-layer kernels ([k / 32][2][64][8]), or null
    float* lse;
    int64_t q_rs, q_hs, o_rs, o_hs;
    const int32_t *q_slot, *q_pos, *q_depth;
    int32_t depth;
    Seg c1, c2;
    float* ws;
    int32_t nq, hq, hkv, nchunk1, nchunk2;
    int32_t chunk;  // rows per workgroup (kChunk or kChunkSmall)
    int32_t whole;  // one workgroup per (query, kv head) over all rows, no partials (duo_decode_whole_kernel)
    float scale_log2e;
};

// Which chunk size a call uses: decided from sizes the host knows, the same way when the workspace is sized.
__host__ __device__ inline int chunk_rows(int nq, int hq, int capacity1) {
    const long big = (long)nq * hq * ((capacity1 + kChunk - 1) / kChunk);  // (query, head, chunk) triples at the large size
    return big < 4096 ? kChunkSmall : kChunk;
}

// One workgroup per (query, kv head) instead of split-K: when those pairs alone give every compute unit a workgroup
// and no context can be long enough for their spread to matter.
#ifndef TAH_DEC_WHOLE_MIN_PAIRS
#define TAH_DEC_WHOLE_MIN_PAIRS 256  // the CPU execution build of the tests lowers it: 256 workgroups of 1024 threads are slow there
#endif
constexpr int kWholeMinPairs = TAH_DEC_WHOLE_MIN_PAIRS, kWholeMaxCapacity = 4096;
constexpr int kWholeMaxGroup = 4;  // eight query heads per kv head do not fit the 128 registers of a 1024-thread workgroup
inline bool whole_sequence(int nq, int hq, int hkv, int capacity1) {
    return (long)nq * hkv >= kWholeMinPairs && capacity1 <= kWholeMaxCapacity && hq / hkv <= kWholeMaxGroup;
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
    return x + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
// Sum over the 16 lanes of a DPP row; every lane of the row gets the total.
__device__ __forceinline__ float row16_sum(float x) {
    x = dpp_add<0xB1>(x);   // quad_perm [1,0,3,2]
    x = dpp_add<0x4E>(x);   // quad_perm [2,3,0,1]
    x = dpp_add<0x141>(x);  // row_half_mirror
    x = dpp_add<0x140>(x);  // row_mirror
    return x;
}

// c + a.lo*b.lo + a.hi*b.hi on packed bf16 pairs (v_dot2_f32_bf16).
__device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __int_as_float((int)(w << 16)); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __int_as_float((int)(w & 0xffff0000u)); }

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;

// Visible rows of the chunk's segment for this query (0 = nothing to do).
__device__ __forceinline__ int visible_len(const DecParams& p, bool second, int slot, int qpos, int qdepth) {
    if (slot < 0) return 0;  // a query without a sequence (a finished row of a generation loop): nothing is read for it
    if (!second) {
        const int n = p.c1.len[slot];
        return qpos + 1 < n ? (qpos + 1 > 0 ? qpos + 1 : 0) : n;
    }
    return qdepth >= 1 ? p.c2.len[slot] : 0;
}

// kSub: row sub->row of the segment is not taken from memory but from sub->k / v / pos (the token the same
// workgroup is appending while it attends: what the loads return for that row is discarded).
struct SubRow {
    int row;  // -1: none in this segment
    int pos;
    u32x4 k, v;
};
// The loads of 4 U rows from r_it on (one row per 16-lane group and load; rows at or past row_end are clamped into
// the slab and flagged).
template <int U>
struct RowBlock {
    u32x4 k[U], v[U];
    int pos[U];
    bool ok[U];
};
template <int U>
__device__ __forceinline__ void load_rows(RowBlock<U>& b, const Seg& sg, bool second, const __bf16* kbase, const __bf16* vbase,
                                          const int32_t* posbase, int r_it, int row_end, int kq) {
    // all of K (and the positions) before V: a wave's loads return in order, and the scores need K only
    int rl[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int r = r_it + u * 4 + kq;
        b.ok[u] = r < row_end;
        rl[u] = b.ok[u] ? r : row_end - 1;  // keep tail loads inside the slab
        // (streaming loads: every cache row is read exactly once)
        b.k[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kbase + (int64_t)rl[u] * sg.k_rs));
        b.pos[u] = second ? posbase[rl[u]] : 0;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        b.v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vbase + (int64_t)rl[u] * sg.v_rs));
    }
}
// Scores, online softmax and the weighted sum of V for a loaded block, for the G query heads of the kv head at
// once.  m / l / acc: running maximum (log2 domain), sum and un-normalised output of this lane's row group, 8
// values of d per lane.
template <int G, int U, bool kSub = false>
__device__ __forceinline__ void attend_rows(RowBlock<U>& b, bool second, int r_it, int kq, int qpos, float scale_log2e, const u32x4 (&qv)[G],
                                            float (&m_run)[G], float (&l_run)[G], float (&acc)[G][8], const SubRow* sub = nullptr) {
    if constexpr (kSub) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool hit = r_it + u * 4 + kq == sub->row;
            b.pos[u] = hit ? sub->pos : b.pos[u];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                b.k[u][i] = hit ? sub->k[i] : b.k[u][i];
                b.v[u][i] = hit ? sub->v[i] : b.v[u][i];
            }
        }
    }
    float s[U][G];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const bool vis = b.ok[u] && (!second || b.pos[u] <= qpos);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float d = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) d = dot2_acc(b.k[u][i], qv[g][i], d);
            d = row16_sum(d) * scale_log2e;
            s[u][g] = vis ? d : kNegInf;
        }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float mx = m_run[g];
#pragma unroll
        for (int u = 0; u < U; ++u) mx = fmaxf(mx, s[u][g]);
        const float m_use = mx == kNegInf ? 0.f : mx;
        const float alpha = fast_exp2(m_run[g] - m_use);
        m_run[g] = mx;
        float pr[U], psum = 0.f;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            pr[u] = fast_exp2(s[u][g] - m_use);
            psum += pr[u];
        }
        l_run[g] = l_run[g] * alpha + psum;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] *= alpha;
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[g][2 * i] += pr[u] * bf16_lo(b.v[u][i]);
                acc[g][2 * i + 1] += pr[u] * bf16_hi(b.v[u][i]);
            }
    }
}
// Sixteen-lane groups of a wave each take one cache row per load (4 rows x 256 B = 1 KiB per instruction); U such
// loads of K and of V are in flight per wave: load, then attend.
template <int G, int U, bool kSub = false>
__device__ __forceinline__ void consume_rows(const Seg& sg, bool second, const __bf16* kbase, const __bf16* vbase, const int32_t* posbase,
                                             int r_it, int row_end, int kq, int qpos, float scale_log2e, const u32x4 (&qv)[G],
                                             float (&m_run)[G], float (&l_run)[G], float (&acc)[G][8], const SubRow* sub = nullptr) {
    RowBlock<U> b;
    load_rows<U>(b, sg, second, kbase, vbase, posbase, r_it, row_end, kq);
    attend_rows<G, U, kSub>(b, second, r_it, kq, qpos, scale_log2e, qv, m_run, l_run, acc, sub);
}

// The 16 (wave, row group) partials of a workgroup into LDS: red[16][G][kPart].
template <int G>
__device__ __forceinline__ void park_partials(float (*red)[G][kPart], int grp, int dc, const float (&m_run)[G], const float (&l_run)[G],
                                              const float (&acc)[G][8]) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int i = 0; i < 8; ++i) red[grp][g][dc * 8 + i] = acc[g][i];
        if (dc == 0) {
            red[grp][g][kD] = m_run[g];
            red[grp][g][kD + 1] = l_run[g];
        }
    }
}

// Element d of head g merged over the 16 partials: un-normalised output, sum, maximum.
template <int G>
__device__ __forceinline__ void merge16(float (*red)[G][kPart], int g, int d, float& a, float& l, float& mx) {
    mx = kNegInf;
#pragma unroll
    for (int j = 0; j < 16; ++j) mx = fmaxf(mx, red[j][g][kD]);
    const float m_use = mx == kNegInf ? 0.f : mx;
    a = 0.f;
    l = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const float w = fast_exp2(red[j][g][kD] - m_use);
        a += w * red[j][g][d];
        l += w * red[j][g][kD + 1];
    }
}

template <int G, int CH>
__global__ __launch_bounds__(kDecThreads) void duo_decode_split_kernel(const DecParams p) {
    constexpr int kRowsPerWave = CH / 4;
    HIP_DYNAMIC_SHARED(unsigned char, smem_raw)
    float (*red)[G][kPart] = reinterpret_cast<float (*)[G][kPart]>(smem_raw);  // [16][G][kPart]: one partial per (wave, row group)

    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int kq = lane / 16, dc = lane % 16;  // row within a 4-row load, 8-element d slice
    const int nslots = p.nchunk1 + p.nchunk2;
    {
        const int chunk = blockIdx.x, qi = blockIdx.y, hk = blockIdx.z;
        const bool second = chunk >= p.nchunk1;
        const int cidx = second ? chunk - p.nchunk1 : chunk;
        const int slot = p.q_slot[qi];
        const int qpos = p.q_pos[qi];
        const int qdepth = p.q_depth ? p.q_depth[qi] : p.depth;
        const int nvis = visible_len(p, second, slot, qpos, qdepth);
        const int row0 = cidx * CH;
        if (row0 >= nvis) return;  // uniform per workgroup
        const Seg& sg = second ? p.c2 : p.c1;
        const int row_end = row0 + CH < nvis ? row0 + CH : nvis;
        const int64_t base_row = sg.start[slot];
        const __bf16* kbase = sg.k + base_row * sg.k_rs + (int64_t)hk * sg.k_hs + dc * 8;
        const __bf16* vbase = sg.v + base_row * sg.v_rs + (int64_t)hk * sg.v_hs + dc * 8;
        const int32_t* posbase = second ? sg.pos + (int64_t)slot * sg.capacity : nullptr;

        // query slices: packed bf16 pairs for the dot products
        u32x4 qv[G];
#pragma unroll
        for (int g = 0; g < G; ++g)
            qv[g] = *reinterpret_cast<const u32x4*>(p.q + (int64_t)qi * p.q_rs + (int64_t)(hk * G + g) * p.q_hs + dc * 8);

        float m_run[G], l_run[G], acc[G][8];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            m_run[g] = kNegInf;
            l_run[g] = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
        }

        const int wrow0 = row0 + wave * kRowsPerWave;
        for (int it = 0; it < kRowsPerWave / (4 * kUnroll); ++it) {
            const int r_it = wrow0 + it * 4 * kUnroll;
            if (r_it >= row_end) break;  // uniform per wave
            consume_rows<G, kUnroll>(sg, second, kbase, vbase, posbase, r_it, row_end, kq, qpos, p.scale_log2e, qv, m_run, l_run, acc);
        }

        // ---- merge the 16 (wave, row group) partials of this workgroup ----------
        park_partials<G>(red, wave * 4 + kq, dc, m_run, l_run, acc);
        __syncthreads();
        for (int e = tid; e < G * kD; e += kDecThreads) {
            const int g = e / kD, d = e % kD;
            float a, l, mx;
            merge16<G>(red, g, d, a, l, mx);
            float* out = p.ws + ((int64_t)(qi * p.hq + hk * G + g) * nslots + chunk) * kPart;
            out[d] = a;
            if (d == 0) {
                out[kD] = mx;
                out[kD + 1] = l;
            }
        }

    }
}

// Element (query qi, head, d) of the finished output, row-major and, when asked for, once more in the rows form of
// the linear-layer kernels ([k / 32][2][64][8] over the [nq, hq * d] matrix the o projection multiplies).
__device__ __forceinline__ void store_output(const DecParams& p, int qi, int head, int d, float o) {
    const __bf16 ob = (__bf16)o;
    p.o[(int64_t)qi * p.o_rs + (int64_t)head * p.o_hs + d] = ob;
    if (p.op) {
        const int k = head * kD + d;
        p.op[((((int64_t)(k / 32) * 2 + qi / 16) * 64) + (qi % 16) + 16 * ((k % 32) / 8)) * 8 + k % 8] = ob;
    }
}

// The whole of a (query, kv head) in one workgroup, no partials and no merge launch: both segments one after the
// other, sixteen waves taking 16-row blocks in turn (as many loads in flight per compute unit as three split-K
// workgroups have).  For calls whose (query, kv head) pairs alone fill the chip and whose contexts are short enough
// that their spread cannot unbalance it (a generation step of 32 sequences of a few thousand tokens): one launch
// instead of two, and no partials through memory.
constexpr int kWholeWaves = 16;
constexpr int kWholeThreads = kWholeWaves * kWave;

// The four row groups of a wave (lanes 16 apart hold the same slice of d) into one partial, left in every lane.
template <int G>
__device__ __forceinline__ void combine_row_groups(float (&m_run)[G], float (&l_run)[G], float (&acc)[G][8]) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float mx = fmaxf(m_run[g], __shfl_xor(m_run[g], 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float w = fast_exp2(m_run[g] - (mx == kNegInf ? 0.f : mx));
        float l = l_run[g] * w;
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        l_run[g] = l;
        m_run[g] = mx;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float a = acc[g][i] * w;
            a += __shfl_xor(a, 16);
            a += __shfl_xor(a, 32);
            acc[g][i] = a;
        }
    }
}

template <int G>
__global__ __launch_bounds__(kWholeThreads) void duo_decode_whole_kernel(const DecParams p) {
    HIP_DYNAMIC_SHARED(unsigned char, smem_raw)
    float (*red)[G][kPart] = reinterpret_cast<float (*)[G][kPart]>(smem_raw);  // [16][G][kPart]: one partial per wave
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int kq = lane / 16, dc = lane % 16;
    const int qi = blockIdx.x, hk = blockIdx.y;
    const int slot = p.q_slot[qi];
    const int qpos = p.q_pos[qi];
    const int qdepth = p.q_depth ? p.q_depth[qi] : p.depth;
    u32x4 qv[G];
#pragma unroll
    for (int g = 0; g < G; ++g)
        qv[g] = *reinterpret_cast<const u32x4*>(p.q + (int64_t)qi * p.q_rs + (int64_t)(hk * G + g) * p.q_hs + dc * 8);
    float m_run[G], l_run[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m_run[g] = kNegInf;
        l_run[g] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
    }
    constexpr int kBlock = 4 * kUnroll;  // rows per wave and turn
    for (int seg = 0; seg < 2; ++seg) {
        const bool second = seg == 1;
        const int nvis = visible_len(p, second, slot, qpos, qdepth);
        if (nvis <= 0) continue;  // uniform per workgroup
        const Seg& sg = second ? p.c2 : p.c1;
        const int64_t base_row = sg.start[slot];
        const __bf16* kbase = sg.k + base_row * sg.k_rs + (int64_t)hk * sg.k_hs + dc * 8;
        const __bf16* vbase = sg.v + base_row * sg.v_rs + (int64_t)hk * sg.v_hs + dc * 8;
        const int32_t* posbase = second ? sg.pos + (int64_t)slot * sg.capacity : nullptr;
        for (int r_it = wave * kBlock; r_it < nvis; r_it += kWholeWaves * kBlock)
            consume_rows<G, kUnroll>(sg, second, kbase, vbase, posbase, r_it, nvis, kq, qpos, p.scale_log2e, qv, m_run, l_run, acc);
    }
    combine_row_groups<G>(m_run, l_run, acc);
    if (kq == 0) park_partials<G>(red, wave, dc, m_run, l_run, acc);
    __syncthreads();
    for (int e = tid; e < G * kD; e += kWholeThreads) {
        const int g = e / kD, d = e % kD;
        float a, l, mx;
        merge16<G>(red, g, d, a, l, mx);
        const int head = hk * G + g;
        store_output(p, qi, head, d, l > 0.f ? a / l : 0.f);
        if (p.lse && d == 0) p.lse[(int64_t)qi * p.hq + head] = l > 0.f ? (mx + fast_log2(l)) * kLn2 : kNegInf;
    }
}

// Merge the chunk partials of one (query, head): 256 threads = 8 chunk lanes x 32 threads of four
// d values, so the chunks are read eight at a time with float4 loads instead of one after another.
__global__ __launch_bounds__(256) void duo_decode_merge_kernel(const DecParams p) {
    __shared__ float mbuf[64];
    __shared__ float red4[8][kD + 4];
    const int qi = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int slot = p.q_slot[qi];
    const int qpos = p.q_pos[qi];
    const int qdepth = p.q_depth ? p.q_depth[qi] : p.depth;
    const int n1 = (visible_len(p, false, slot, qpos, qdepth) + p.chunk - 1) / p.chunk;
    const int n2 = (visible_len(p, true, slot, qpos, qdepth) + p.chunk - 1) / p.chunk;
    const int n = n1 + n2, nslots = p.nchunk1 + p.nchunk2;
    const float* part = p.ws + (int64_t)(qi * p.hq + head) * nslots * kPart;
    auto slot_of = [&](int c) { return c < n1 ? c : p.nchunk1 + (c - n1); };
    // global max over the chunk maxima (n <= a few dozen; 64 per pass)
    float mx = kNegInf;
    for (int c0 = 0; c0 < n; c0 += 64) {
        if (tid < 64) mbuf[tid] = c0 + tid < n ? part[(int64_t)slot_of(c0 + tid) * kPart + kD] : kNegInf;
        __syncthreads();
        for (int j = 0; j < 64; ++j) mx = fmaxf(mx, mbuf[j]);
        __syncthreads();
    }
    const float m_use = mx == kNegInf ? 0.f : mx;
    const int cl = tid / 32, d4 = (tid % 32) * 4;
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
    float l = 0.f;
    for (int c = cl; c < n; c += 8) {
        const float* pc = part + (int64_t)slot_of(c) * kPart;
        const float w = fast_exp2(pc[kD] - m_use);
        a[0] += w * pc[d4]; a[1] += w * pc[d4 + 1]; a[2] += w * pc[d4 + 2]; a[3] += w * pc[d4 + 3];
        l += w * pc[kD + 1];
    }
    red4[cl][d4] = a[0]; red4[cl][d4 + 1] = a[1]; red4[cl][d4 + 2] = a[2]; red4[cl][d4 + 3] = a[3];
    if (d4 == 0) red4[cl][kD] = l;
    __syncthreads();
    if (tid < kD) {
        float o = 0.f, lt = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) { o += red4[j][tid]; lt += red4[j][kD]; }
        const float inv = lt > 0.f ? 1.0f / lt : 0.f;
        store_output(p, qi, head, tid, o * inv);
        if (p.lse && tid == 0) p.lse[(int64_t)qi * p.hq + head] = lt > 0.f ? (mx + fast_log2(lt)) * kLn2 : kNegInf;
    }
}

// ---- KV append --------------------------------------------------------------
struct AppendParams {
    const __bf16 *k_new, *v_new;
    const int32_t *pos_new, *cu_new, *slot_of;
    int64_t kn_rs, kn_hs, vn_rs, vn_hs;
    __bf16 *ck, *cv;
    int32_t* cpos;
    const int32_t* start;
    int32_t* len;
    int64_t ck_rs, ck_hs, cv_rs, cv_hs;
    int32_t capacity, nseq, hkv;
    int32_t* overflow;
};

// Sequence of new row r: the b with cu_new[b] <= r < cu_new[b+1] (binary search; nseq if r is past the end).
__device__ __forceinline__ int seq_of_row(const int32_t* cu_new, int nseq, int r) {
    int lo = 0, hi = nseq;  // invariant: cu_new[lo] <= r (or lo == 0), answer in [lo, hi]
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (r >= cu_new[mid + 1]) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

// 256 threads = 8 rows per workgroup: 32 lanes move one token row, K and V of one kv head per pass
// (16 lanes x 16 bytes each).
__global__ __launch_bounds__(256) void kv_append_rows_kernel(const AppendParams a, int total_new) {
    const int r = blockIdx.x * 8 + threadIdx.x / 32, t = threadIdx.x % 32;
    if (r >= total_new) return;
    const int seq = seq_of_row(a.cu_new, a.nseq, r);
    if (seq >= a.nseq) return;
    const int slot = a.slot_of ? a.slot_of[seq] : seq;
    if (slot < 0) return;  // this sequence's rows are not cached
    const int dst = a.len[slot] + (r - a.cu_new[seq]);
    if (dst >= a.capacity) {
        if (a.overflow && t == 0) *a.overflow = 1;
        return;
    }
    const int64_t drow = (int64_t)a.start[slot] + dst;
    const int u = t % 16;
    for (int h = 0; h < a.hkv; ++h) {
        if (t < 16) {
            *reinterpret_cast<bf16x8*>(a.ck + drow * a.ck_rs + (int64_t)h * a.ck_hs + u * 8) =
                *reinterpret_cast<const bf16x8*>(a.k_new + (int64_t)r * a.kn_rs + (int64_t)h * a.kn_hs + u * 8);
        } else {
            *reinterpret_cast<bf16x8*>(a.cv + drow * a.cv_rs + (int64_t)h * a.cv_hs + u * 8) =
                *reinterpret_cast<const bf16x8*>(a.v_new + (int64_t)r * a.vn_rs + (int64_t)h * a.vn_hs + u * 8);
        }
    }
    if (a.cpos && a.pos_new && t == 0) a.cpos[(int64_t)slot * a.capacity + dst] = a.pos_new[r];
}

// Runs after the row copies on the same stream: advance the slab lengths.
__global__ void kv_append_len_kernel(const AppendParams a) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= a.nseq) return;
    const int slot = a.slot_of ? a.slot_of[b] : b;
    if (slot < 0) return;
    const int n = a.len[slot] + (a.cu_new[b + 1] - a.cu_new[b]);
    a.len[slot] = n < a.capacity ? n : a.capacity;
}

// ---- q/k RMSNorm + rotary embedding (+ append) --------------------------------
// What Qwen3Attention.forward does between the projections and the attention call
// (transformers/models/qwen3/modeling_qwen3.py: Qwen3RMSNorm.forward on the q and k heads,
// apply_rotary_pos_emb, then TaHCache.update), with the roundings of its bf16 eager arithmetic:
//   n = bf16(x * rsqrt(mean(x^2) + eps));  y = bf16(w * n)                       (per head, D = 128)
//   out[i] = bf16(bf16(y[i] * cos[i]) + bf16(rot[i] * sin[i])),  rot = (-y[64:], y[:64])
// V is only moved.  With `append`, K and V go to the token's place in
// the per-sequence slabs (as kv_append_rows_kernel does) instead of k_out / v_out.
struct PrepParams {
    const __bf16 *q, *k, *v;
    __bf16 *q_out, *k_out, *v_out;
    int64_t q_rs, q_hs, k_rs, k_hs, v_rs, v_hs, qo_rs, qo_hs, ko_rs, ko_hs, vo_rs, vo_hs;
    const __bf16 *qw, *kw, *cos, *sin;
    int64_t cs_rs;
    float eps;
    int32_t rows, hq, hkv, append;
    int32_t own_len;  // every sequence appends at most one row: the row's workgroup advances the length itself
    const __bf16* xn;  // rows whose RMS the projections still have to be divided by (input norm folded in), or nullptr
    int64_t xn_rs;
    int32_t xn_cols;
    float xn_eps;
    AppendParams a;  // destination slabs (append != 0); its k_new / v_new fields are not used
};

// Two floats rounded to bfloat16 (nearest, ties to even) and packed, lo in the low half: one
// v_cvt_pk_bf16_f32.  Going through the packed bits on purpose: a scalar cast to __bf16 and back may be
// evaluated in excess precision by the compiler, i.e. not round at all.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2e __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2e));
}
// a.lo*b.lo and a.hi*b.hi, each rounded to bf16, packed (a, b: packed bf16 pairs)
__device__ __forceinline__ uint32_t mul_bf16x2(uint32_t a, uint32_t b) {
    return pack_bf16(bf16_lo(a) * bf16_lo(b), bf16_hi(a) * bf16_hi(b));
}

// One head's 16-byte piece (lane j of the head's 16 lanes) through RMSNorm, weight and rotary embedding, with the
// roundings listed above; `sign`: 0x80008000 for the lower half of the head (j < 8), where the partner enters negated.
__device__ __forceinline__ u32x4 prep_head_piece(u32x4 xin, const u32x4& w, const u32x4& cs, const u32x4& sn, uint32_t sign, float eps) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) ss += bf16_lo(xin[i]) * bf16_lo(xin[i]) + bf16_hi(xin[i]) * bf16_hi(xin[i]);
    ss = row16_sum(ss);
    // hardware reciprocal square root (1 ulp): whether it or the order of the sum above decides
    // the last bit of a normalised value before the bf16 rounding is the same kind of difference
    const float rs = __builtin_amdgcn_rsqf(ss * (1.0f / 128.0f) + eps);
    u32x4 yn, out;
#pragma unroll
    for (int i = 0; i < 4; ++i) yn[i] = mul_bf16x2(w[i], pack_bf16(bf16_lo(xin[i]) * rs, bf16_hi(xin[i]) * rs));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // the partner's normalised values: lane j^8 of this row (row rotation by 8)
        const uint32_t pn = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)yn[i], 0x128, 0xf, 0xf, false) ^ sign;
        const uint32_t a = mul_bf16x2(yn[i], cs[i]), b = mul_bf16x2(pn, sn[i]);
        out[i] = pack_bf16(bf16_lo(a) + bf16_lo(b), bf16_hi(a) + bf16_hi(b));
    }
    return out;
}
__device__ __forceinline__ u32x4 scale_piece(u32x4 x, float f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = pack_bf16(bf16_lo(x[i]) * f, bf16_hi(x[i]) * f);
    return x;
}

// One workgroup (4 waves) per token row.  A head is handled by 16 lanes, 8 elements (16 bytes) each, so
// a wave takes 4 heads at a time and the workgroup 16: the mean of squares is a DPP reduction inside
// the row of 16 lanes, and the rotary partner of lane j's elements (+-64) sits in lane j^8 of the
// same row.
__global__ __launch_bounds__(256) void qk_prep_kernel(const PrepParams p) {
    const int r = blockIdx.x;
    const int lane = threadIdx.x % kWave;
    const int sub = threadIdx.x / 16, j = lane % 16;  // head slot 0..15 of a pass, 16-byte piece of the head
    const int items = p.hq + 2 * p.hkv;
    // the row's data first: nothing below that decides where the results go depends on it, and the
    // loads then fly while the destination is looked up
    // (one load from an address picked by selects, and a select on what it returns: with a load in each arm of a
    // branch the compiler waits for it where the arms meet, and the second pass's load would only go out after the first's
    // data is back)
    auto load_item = [&](int it) {
        const bool is_q = it < p.hq, is_k = !is_q && it < p.hq + p.hkv;
        const bool is_v = !is_q && !is_k && it < items && p.v && (p.append || p.v_out);
        const __bf16* at = p.q + (int64_t)r * p.q_rs + 8 * j;  // (a valid address for the slots without a head)
        if (is_q) at += (int64_t)it * p.q_hs;
        if (is_k) at = p.k + (int64_t)r * p.k_rs + (int64_t)(it - p.hq) * p.k_hs + 8 * j;
        if (is_v) at = p.v + (int64_t)r * p.v_rs + (int64_t)(it - p.hq - p.hkv) * p.v_hs + 8 * j;
        const u32x4 x = *reinterpret_cast<const u32x4*>(at);
        return (is_q || is_k || is_v) ? x : u32x4{0u, 0u, 0u, 0u};
    };
    constexpr int kAhead = 2;  // passes loaded up front (32 heads: the whole row at Hq = 16, Hkv = 8)
    u32x4 ahead[kAhead];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) ahead[i] = load_item(16 * i + sub);
    // input norm folded in: the factor the whole row is scaled by (1 when there is none)
    float rin = 1.0f;
    if (p.xn) {
        __shared__ float xn_part[4];
        const __bf16* xr = p.xn + (int64_t)r * p.xn_rs;
        float ss = 0.f;
        for (int c = threadIdx.x * 8; c < p.xn_cols; c += 256 * 8) {
            const u32x4 x = *reinterpret_cast<const u32x4*>(xr + c);
#pragma unroll
            for (int i = 0; i < 4; ++i) ss += bf16_lo(x[i]) * bf16_lo(x[i]) + bf16_hi(x[i]) * bf16_hi(x[i]);
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
        if (lane == 0) xn_part[threadIdx.x / kWave] = ss;
        __syncthreads();
        ss = (xn_part[0] + xn_part[1]) + (xn_part[2] + xn_part[3]);
        rin = __builtin_amdgcn_rsqf(ss / (float)p.xn_cols + p.xn_eps);
    }
    const u32x4 cs = *reinterpret_cast<const u32x4*>(p.cos + (int64_t)r * p.cs_rs + 8 * j);
    const u32x4 sn = *reinterpret_cast<const u32x4*>(p.sin + (int64_t)r * p.cs_rs + 8 * j);
    const u32x4 qw = *reinterpret_cast<const u32x4*>(p.qw + 8 * j), kw = *reinterpret_cast<const u32x4*>(p.kw + 8 * j);

    __bf16 *kdst = nullptr, *vdst = nullptr;
    int64_t kd_hs = 0, vd_hs = 0;
    if (p.append) {
        const int seq = seq_of_row(p.a.cu_new, p.a.nseq, r);
        if (seq < p.a.nseq) {
            const int slot = p.a.slot_of ? p.a.slot_of[seq] : seq;  // (may be written by an earlier kernel of the step)
            const int dst = slot < 0 ? 0 : p.a.len[slot] + (r - const_i32(p.a.cu_new, seq));
            if (p.own_len) __syncthreads();  // every wave has read the old length before thread 0 replaces it (the
                                             // branch is uniform: one row, one sequence, one slot per workgroup)
            if (slot < 0) {
                // not cached: q is still prepared, K and V of the row go nowhere
            } else if (dst >= p.a.capacity) {
                if (p.a.overflow && threadIdx.x == 0) *p.a.overflow = 1;
            } else {
                const int64_t drow = (int64_t)const_i32(p.a.start, slot) + dst;
                kdst = p.a.ck + drow * p.a.ck_rs;
                vdst = p.a.cv + drow * p.a.cv_rs;
                kd_hs = p.a.ck_hs;
                vd_hs = p.a.cv_hs;
                if (p.a.cpos && p.a.pos_new && threadIdx.x == 0) p.a.cpos[(int64_t)slot * p.a.capacity + dst] = p.a.pos_new[r];
                if (p.own_len && threadIdx.x == 0) p.a.len[slot] = dst + 1;  // nobody else reads or writes this slot's length
            }
        }
    } else {
        kdst = p.k_out + (int64_t)r * p.ko_rs;
        kd_hs = p.ko_hs;
        if (p.v_out) {
            vdst = p.v_out + (int64_t)r * p.vo_rs;
            vd_hs = p.vo_hs;
        }
    }
    const uint32_t sign = j < 8 ? 0x80008000u : 0u;  // lower half of the head: -partner * sin
    // (every lane of a wave walks the same number of passes and takes part in every lane exchange;
    // what a 16-lane row has no head for is predicated off)
    for (int pass = 0; pass * 16 < items; ++pass) {
        const int it = pass * 16 + sub;
        const bool is_q = it < p.hq, is_k = !is_q && it < p.hq + p.hkv, is_v = !is_q && !is_k && it < items;
        u32x4 xin = pass == 0 ? ahead[0] : pass == 1 ? ahead[1] : load_item(it);
        if (p.xn) xin = scale_piece(xin, rin);  // the row's input-norm factor, applied where the eager modules have a normalised projection
        if (is_v && vdst)  // a V head: moved as it is
            *reinterpret_cast<u32x4*>(vdst + (int64_t)(it - p.hq - p.hkv) * vd_hs + 8 * j) = xin;
        const int h = is_q ? it : it - p.hq;
        __bf16* y = is_q ? p.q_out + (int64_t)r * p.qo_rs + (int64_t)h * p.qo_hs
                         : (is_k && kdst ? kdst + (int64_t)h * kd_hs : nullptr);  // null: no head, or the row overflows its slab
        const u32x4 out = prep_head_piece(xin, is_q ? qw : kw, cs, sn, sign, p.eps);
        if (y) *reinterpret_cast<u32x4*>(y + 8 * j) = out;
    }
}

// ---- backward of the q/k preparation ----------------------------------------------------------------------
// out = rope(w * x * rsqrt(mean(x^2) + eps)) per head.  With g the gradient of out:
//   dyn = g cos + partner(g sin), the partner entering with the opposite sign of the forward's (+ for the lower
//         half of the head, - for the upper one: the transpose of rotate_half);
//   dw += dyn * xh, xh = x * rs (summed over rows and heads);
//   dx  = rs * (dyn w - xh * mean(dyn w xh)).
// Evaluated in float32 on the bf16 inputs (the forward's intermediate roundings are not differentiated through, as
// in any bf16 backward).  Same lane layout as the forward: 16 lanes per head, partner in lane j ^ 8.  A workgroup
// walks rows blockIdx.x, blockIdx.x + gridDim.x, ... and leaves its sums of the two weight gradients in its own row
// of dw_partial (float32 [gridDim.x, 2, 128]): no atomics, the caller adds the rows up.
struct PrepBwdParams {
    const __bf16 *q, *k, *dqo, *dko;
    __bf16 *dq, *dk;
    int64_t q_rs, q_hs, k_rs, k_hs, dqo_rs, dqo_hs, dko_rs, dko_hs, dq_rs, dq_hs, dk_rs, dk_hs;
    const __bf16 *qw, *kw, *cos, *sin;
    int64_t cs_rs;
    float eps;
    int32_t rows, hq, hkv;
    float* dw_partial;
};

__global__ __launch_bounds__(256) void qk_prep_bwd_kernel(const PrepBwdParams p) {
    __shared__ float red[2][16][128];
    const int lane = threadIdx.x % kWave;
    const int sub = threadIdx.x / 16, j = lane % 16;
    const int items = p.hq + p.hkv;
    const u32x4 qw = *reinterpret_cast<const u32x4*>(p.qw + 8 * j), kw = *reinterpret_cast<const u32x4*>(p.kw + 8 * j);
    float dwq[8], dwk[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) dwq[i] = dwk[i] = 0.f;
    const float psign = j < 8 ? 1.f : -1.f;
    for (int r = blockIdx.x; r < p.rows; r += gridDim.x) {
        const u32x4 cs = *reinterpret_cast<const u32x4*>(p.cos + (int64_t)r * p.cs_rs + 8 * j);
        const u32x4 sn = *reinterpret_cast<const u32x4*>(p.sin + (int64_t)r * p.cs_rs + 8 * j);
        // (every lane of a wave walks the same number of passes and takes part in every lane exchange)
        for (int pass = 0; pass * 16 < items; ++pass) {
            const int it = pass * 16 + sub;
            const bool is_q = it < p.hq, live = it < items;
            const int h = is_q ? it : it - p.hq;
            u32x4 xin = {0u, 0u, 0u, 0u}, gin = {0u, 0u, 0u, 0u};
            if (live) {
                xin = *reinterpret_cast<const u32x4*>(is_q ? p.q + (int64_t)r * p.q_rs + (int64_t)h * p.q_hs + 8 * j
                                                            : p.k + (int64_t)r * p.k_rs + (int64_t)h * p.k_hs + 8 * j);
                gin = *reinterpret_cast<const u32x4*>(is_q ? p.dqo + (int64_t)r * p.dqo_rs + (int64_t)h * p.dqo_hs + 8 * j
                                                            : p.dko + (int64_t)r * p.dko_rs + (int64_t)h * p.dko_hs + 8 * j);
            }
            const u32x4& w = is_q ? qw : kw;
            float x[8], g[8], u[8];
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                x[2 * i] = bf16_lo(xin[i]);
                x[2 * i + 1] = bf16_hi(xin[i]);
                g[2 * i] = bf16_lo(gin[i]);
                g[2 * i + 1] = bf16_hi(gin[i]);
                u[2 * i] = g[2 * i] * bf16_lo(sn[i]);
                u[2 * i + 1] = g[2 * i + 1] * bf16_hi(sn[i]);
                ss += x[2 * i] * x[2 * i] + x[2 * i + 1] * x[2 * i + 1];
            }
            ss = row16_sum(ss);
            const float rs = __builtin_amdgcn_rsqf(ss * (1.0f / 128.0f) + p.eps);
            float dxh[8], xh[8];
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // the partner's g sin: lane j ^ 8 of this row of 16 lanes (row rotation by 8)
                const float pu = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(u[i]), 0x128, 0xf, 0xf, false));
                const float c = (i % 2) ? bf16_hi(cs[i / 2]) : bf16_lo(cs[i / 2]);
                const float wi = (i % 2) ? bf16_hi(w[i / 2]) : bf16_lo(w[i / 2]);
                const float dyn = g[i] * c + psign * pu;
                xh[i] = x[i] * rs;
                if (is_q) dwq[i] += dyn * xh[i];
                else dwk[i] += dyn * xh[i];
                dxh[i] = dyn * wi;
                dot += dxh[i] * xh[i];
            }
            dot = row16_sum(dot) * (1.0f / 128.0f);
            u32x4 out;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                out[i] = pack_bf16(rs * (dxh[2 * i] - xh[2 * i] * dot), rs * (dxh[2 * i + 1] - xh[2 * i + 1] * dot));
            if (live) {
                __bf16* y = is_q ? p.dq + (int64_t)r * p.dq_rs + (int64_t)h * p.dq_hs : p.dk + (int64_t)r * p.dk_rs + (int64_t)h * p.dk_hs;
                *reinterpret_cast<u32x4*>(y + 8 * j) = out;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        red[0][sub][8 * j + i] = dwq[i];
        red[1][sub][8 * j + i] = dwk[i];
    }
    __syncthreads();
    const int which = threadIdx.x / 128, d = threadIdx.x % 128;
    float t = 0.f;
#pragma unroll
    for (int s_ = 0; s_ < 16; ++s_) t += red[which][s_][d];
    p.dw_partial[((int64_t)blockIdx.x * 2 + which) * 128 + d] = t;
}

// ---- q/k preparation, append and attention of a decode step in one launch --------------------------------
// What qk_prep_kernel (one row per sequence, append) followed by duo_decode_whole_kernel do, for calls the latter
// takes: the workgroup of (query, kv head) prepares the G query heads and the new K and V of its kv head itself
// (every 16-lane group of every wave repeats the few dozen operations: the prepared pieces are then where the row
// loop wants them), one group stores K and V into the slabs for the steps to come, and the row loop takes the new
// row from registers instead of reading back what is being written.  The place of the new row comes from the
// caller (append_at[], the segment's length before the call): the eight workgroups of a sequence cannot read
// len[] while one of them advances it.  Same arithmetic in the same order as the two kernels: the slabs get the
// same bits, the outputs too except where the compiler contracted a multiply-add in one kernel and not the other.
constexpr int kStepMaxGroup = 2;  // with four query heads per kv head the preparation no longer fits the 128 registers
struct StepParams {
    PrepParams prep;
    DecParams dec;
    AppendParams app[2];           // where a new row goes in the depth-0 / depth-1 segment (slabs, positions, lengths)
    const int32_t* append_at;
    const int32_t* append_depth;   // per row 0 / 1, or null: every row appends to segment `append_second`
    int32_t append_second;
};

template <int G>
__global__ __launch_bounds__(kWholeThreads) void duo_decode_step_kernel(const StepParams sp) {
    const PrepParams& pp = sp.prep;
    const DecParams& p = sp.dec;
    HIP_DYNAMIC_SHARED(unsigned char, smem_raw)
    float (*red)[G][kPart] = reinterpret_cast<float (*)[G][kPart]>(smem_raw);
    __shared__ float xn_part[kWholeWaves];
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int kq = lane / 16, dc = lane % 16;
    const int qi = blockIdx.x, hk = blockIdx.y;
    // the row's data first: the loads fly while the bookkeeping is looked up
    u32x4 xq[G];
#pragma unroll
    for (int g = 0; g < G; ++g) xq[g] = *reinterpret_cast<const u32x4*>(pp.q + (int64_t)qi * pp.q_rs + (int64_t)(hk * G + g) * pp.q_hs + 8 * dc);
    u32x4 xk = *reinterpret_cast<const u32x4*>(pp.k + (int64_t)qi * pp.k_rs + (int64_t)hk * pp.k_hs + 8 * dc);
    u32x4 xv = *reinterpret_cast<const u32x4*>(pp.v + (int64_t)qi * pp.v_rs + (int64_t)hk * pp.v_hs + 8 * dc);
    const u32x4 cs = *reinterpret_cast<const u32x4*>(pp.cos + (int64_t)qi * pp.cs_rs + 8 * dc);
    const u32x4 sn = *reinterpret_cast<const u32x4*>(pp.sin + (int64_t)qi * pp.cs_rs + 8 * dc);
    const u32x4 qw = *reinterpret_cast<const u32x4*>(pp.qw + 8 * dc), kw = *reinterpret_cast<const u32x4*>(pp.kw + 8 * dc);
    const int slot = p.q_slot[qi];
    const int qpos = p.q_pos[qi];
    const int qdepth = p.q_depth ? p.q_depth[qi] : p.depth;
    const int aslot = pp.a.slot_of ? pp.a.slot_of[qi] : qi;  // < 0: the row is not cached
    const int dst = sp.append_at[qi];
    const int pos_new = pp.a.pos_new ? pp.a.pos_new[qi] : 0;
    const int adepth = sp.append_depth ? (sp.append_depth[qi] != 0 ? 1 : 0) : sp.append_second;  // uniform per workgroup
    const AppendParams& ap = sp.app[adepth];
    const bool cached = aslot >= 0, fits = cached && dst < ap.capacity;
    // rows of a segment: with the new row where this call appends (nobody may read len[] of that segment here)
    auto visible = [&](int seg) {
        const Seg& sg = seg ? p.c2 : p.c1;
        if (slot < 0 || (seg && qdepth < 1)) return 0;  // (slot < 0: a query without a sequence)
        const int n = (seg == adepth && cached) ? (fits ? dst + 1 : (dst < ap.capacity ? dst : ap.capacity)) : sg.len[slot];
        return seg ? n : (qpos + 1 < n ? (qpos + 1 > 0 ? qpos + 1 : 0) : n);
    };
    constexpr int kBlock = 4 * kUnroll;
    // this wave's first block of cached rows goes on its way before the preparation below, which needs none of it
    const int nvis0 = visible(0);
    const int64_t base0 = slot < 0 ? 0 : p.c1.start[slot];
    const __bf16* kbase0 = p.c1.k + base0 * p.c1.k_rs + (int64_t)hk * p.c1.k_hs + dc * 8;
    const __bf16* vbase0 = p.c1.v + base0 * p.c1.v_rs + (int64_t)hk * p.c1.v_hs + dc * 8;
    RowBlock<kUnroll> first;
    const bool have_first = wave * kBlock < nvis0;  // uniform per wave
    if (have_first) load_rows<kUnroll>(first, p.c1, false, kbase0, vbase0, nullptr, wave * kBlock, nvis0, kq);
    float rin = 1.0f;
    if (pp.xn) {
        const __bf16* xr = pp.xn + (int64_t)qi * pp.xn_rs;
        float ss = 0.f;
        // summed as qk_prep_kernel's 256 threads sum it (same strides, same order), so that the factor has the same bits
        if (tid < 256)
            for (int c = tid * 8; c < pp.xn_cols; c += 256 * 8) {
                const u32x4 x = *reinterpret_cast<const u32x4*>(xr + c);
#pragma unroll
                for (int i = 0; i < 4; ++i) ss += bf16_lo(x[i]) * bf16_lo(x[i]) + bf16_hi(x[i]) * bf16_hi(x[i]);
            }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
        if (lane == 0) xn_part[wave] = ss;
        __syncthreads();
        ss = (xn_part[0] + xn_part[1]) + (xn_part[2] + xn_part[3]);
        rin = __builtin_amdgcn_rsqf(ss / (float)pp.xn_cols + pp.xn_eps);
#pragma unroll
        for (int g = 0; g < G; ++g) xq[g] = scale_piece(xq[g], rin);
        xk = scale_piece(xk, rin);
        xv = scale_piece(xv, rin);
    }
    const uint32_t sign = dc < 8 ? 0x80008000u : 0u;
    u32x4 qv[G];
#pragma unroll
    for (int g = 0; g < G; ++g) qv[g] = prep_head_piece(xq[g], qw, cs, sn, sign, pp.eps);
    SubRow sub;
    sub.k = prep_head_piece(xk, kw, cs, sn, sign, pp.eps);
    sub.v = xv;
    sub.pos = pos_new;
    if (cached && !fits && pp.a.overflow && tid == 0 && hk == 0) *pp.a.overflow = 1;
    if (fits && wave == 0 && kq == 0) {
        const int64_t drow = (int64_t)const_i32(ap.start, aslot) + dst;
        *reinterpret_cast<u32x4*>(ap.ck + drow * ap.ck_rs + (int64_t)hk * ap.ck_hs + 8 * dc) = sub.k;
        *reinterpret_cast<u32x4*>(ap.cv + drow * ap.cv_rs + (int64_t)hk * ap.cv_hs + 8 * dc) = sub.v;
        if (dc == 0 && hk == 0) {
            if (ap.cpos && pp.a.pos_new) ap.cpos[(int64_t)aslot * ap.capacity + dst] = pos_new;
            // (only this workgroup touches the length of the segment the row appends to)  A row placed anywhere but
            // at the end of its slab leaves a gap of stale rows or overwrites cached ones: reported, not repaired.
            if (ap.len[aslot] != dst && pp.a.overflow) *pp.a.overflow = 2;
            ap.len[aslot] = dst + 1;
        }
    }
    float m_run[G], l_run[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m_run[g] = kNegInf;
        l_run[g] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
    }
    // depth-0 segment: the block loaded above, then the wave's other turns
    sub.row = (adepth == 0 && fits) ? dst : -1;
    if (have_first) attend_rows<G, kUnroll, true>(first, false, wave * kBlock, kq, qpos, p.scale_log2e, qv, m_run, l_run, acc, &sub);
    for (int r_it = (wave + kWholeWaves) * kBlock; r_it < nvis0; r_it += kWholeWaves * kBlock)
        consume_rows<G, kUnroll, true>(p.c1, false, kbase0, vbase0, nullptr, r_it, nvis0, kq, qpos, p.scale_log2e, qv, m_run, l_run, acc, &sub);
    // depth-1 segment
    const int nvis1 = visible(1);
    if (nvis1 > 0) {  // uniform per workgroup
        sub.row = (adepth == 1 && fits) ? dst : -1;
        const int64_t base1 = p.c2.start[slot];
        const __bf16* kbase1 = p.c2.k + base1 * p.c2.k_rs + (int64_t)hk * p.c2.k_hs + dc * 8;
        const __bf16* vbase1 = p.c2.v + base1 * p.c2.v_rs + (int64_t)hk * p.c2.v_hs + dc * 8;
        const int32_t* posbase = p.c2.pos + (int64_t)slot * p.c2.capacity;
        for (int r_it = wave * kBlock; r_it < nvis1; r_it += kWholeWaves * kBlock)
            consume_rows<G, kUnroll, true>(p.c2, true, kbase1, vbase1, posbase, r_it, nvis1, kq, qpos, p.scale_log2e, qv, m_run, l_run, acc, &sub);
    }
    combine_row_groups<G>(m_run, l_run, acc);
    if (kq == 0) park_partials<G>(red, wave, dc, m_run, l_run, acc);
    __syncthreads();
    for (int e = tid; e < G * kD; e += kWholeThreads) {
        const int g = e / kD, d = e % kD;
        float a, l, mx;
        merge16<G>(red, g, d, a, l, mx);
        const int head = hk * G + g;
        store_output(p, qi, head, d, l > 0.f ? a / l : 0.f);
        if (p.lse && d == 0) p.lse[(int64_t)qi * p.hq + head] = l > 0.f ? (mx + fast_log2(l)) * kLn2 : kNegInf;
    }
}

Seg to_seg(const tah_kv_segment& s) {
    Seg d;
    d.k = static_cast<const __bf16*>(s.k);
    d.v = static_cast<const __bf16*>(s.v);
    d.pos = s.pos;
    d.start = s.start;
    d.len = s.len;
    d.k_rs = s.k_row_stride; d.k_hs = s.k_head_stride;
    d.v_rs = s.v_row_stride; d.v_hs = s.v_head_stride;
    d.capacity = s.capacity;
    return d;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_seg(const tah_kv_segment& s, bool need_pos) {
    if (s.capacity < 0 || s.nslots < 0) return TAH_E_SHAPE;
    if (s.capacity == 0) return TAH_OK;
    if (!s.k || !s.v || !s.start || !s.len || (need_pos && !s.pos)) return TAH_E_NULL;
    if (!aligned16(s.k) || !aligned16(s.v)) return TAH_E_ALIGN;
    if (s.k_row_stride % 8 || s.k_head_stride % 8 || s.v_row_stride % 8 || s.v_head_stride % 8) return TAH_E_ALIGN;
    return TAH_OK;
}

template <int G>
int launch_decode(const DecParams& p, hipStream_t st) {
    constexpr int kRedBytes = 16 * G * kPart * (int)sizeof(float);  // 8.3 KB per query head of the group
    if constexpr (G <= kWholeMaxGroup) {
        if (p.whole) {
            hipLaunchKernelGGL((duo_decode_whole_kernel<G>), dim3(p.nq, p.hkv), dim3(kWholeThreads), kRedBytes, st, p);
            return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
        }
    }
    const dim3 grid(p.nchunk1 + p.nchunk2, p.nq, p.hkv);
    if (p.chunk == kChunk) {
        if (kRedBytes > 64 * 1024 &&
            hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_decode_split_kernel<G, kChunk>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kRedBytes) != hipSuccess)
            return TAH_E_LAUNCH;
        hipLaunchKernelGGL((duo_decode_split_kernel<G, kChunk>), grid, dim3(kDecThreads), kRedBytes, st, p);
    } else {
        if (kRedBytes > 64 * 1024 &&
            hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_decode_split_kernel<G, kChunkSmall>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kRedBytes) != hipSuccess)
            return TAH_E_LAUNCH;
        hipLaunchKernelGGL((duo_decode_split_kernel<G, kChunkSmall>), grid, dim3(kDecThreads), kRedBytes, st, p);
    }
    hipLaunchKernelGGL(duo_decode_merge_kernel, dim3(p.nq, p.hq), dim3(256), 0, st, p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

}  // namespace
}  // namespace tah

extern "C" size_t tah_duo_decode_workspace_bytes(int32_t nq, int32_t hq, int32_t capacity1, int32_t capacity2) {
    using namespace tah;
    if (nq <= 0 || hq <= 0 || capacity1 < 0 || capacity2 < 0) return 0;
    const int ch = chunk_rows(nq, hq, capacity1);
    const size_t chunks = (size_t)(capacity1 + ch - 1) / ch + (size_t)(capacity2 + ch - 1) / ch;
    return (size_t)nq * hq * chunks * kPart * sizeof(float);
}

namespace tah {
namespace {

// Argument checks of the decode entry points and the kernels' parameters.  `fused`: the call is the second half of
// tah_duo_decode_step (no prepared q in memory, no workspace).  Returns 1 when there is nothing to do.
int dec_fill(const tah_duo_decode_args* a, DecParams& p, bool fused, void* ws, size_t ws_bytes, int too_small) {
    if (!a) return TAH_E_NULL;
    if (a->d != kD || a->nq < 0 || a->hq <= 0 || a->hkv <= 0 || a->hq % a->hkv) return TAH_E_SHAPE;
    const int g = a->hq / a->hkv;
    if (g != 1 && g != 2 && g != 4 && g != 8) return TAH_E_SHAPE;
    if (a->nq == 0) return 1;
    if (a->nq > 65535 || a->hq > 65535) return TAH_E_SHAPE;
    if (!a->o || !a->q_slot || !a->q_pos) return TAH_E_NULL;
    if (!fused) {
        if (!a->q || !ws) return TAH_E_NULL;
        if (!aligned16(a->q) || !aligned16(ws) || a->q_row_stride % 8 || a->q_head_stride % 8) return TAH_E_ALIGN;
    }
    if (a->o_packed && a->nq > 32) return TAH_E_SHAPE;
    if (!aligned16(a->o_packed)) return TAH_E_ALIGN;
    if (int rc = check_seg(a->c1, false)) return rc;
    const bool any_depth1 = a->q_depth != nullptr || a->depth >= 1;
    if (any_depth1)
        if (int rc = check_seg(a->c2, true)) return rc;
    const int cap2 = any_depth1 ? a->c2.capacity : 0;
    if (!fused && ws_bytes < tah_duo_decode_workspace_bytes(a->nq, a->hq, a->c1.capacity, cap2)) return too_small;
    p.q = static_cast<const __bf16*>(a->q);
    p.o = static_cast<__bf16*>(a->o);
    p.op = static_cast<__bf16*>(a->o_packed);
    p.lse = a->lse;
    p.q_rs = a->q_row_stride; p.q_hs = a->q_head_stride;
    p.o_rs = a->o_row_stride; p.o_hs = a->o_head_stride;
    p.q_slot = a->q_slot; p.q_pos = a->q_pos; p.q_depth = a->q_depth;
    p.depth = a->depth;
    p.c1 = to_seg(a->c1);
    p.c2 = to_seg(a->c2);
    p.ws = static_cast<float*>(ws);
    p.nq = a->nq; p.hq = a->hq; p.hkv = a->hkv;
    p.chunk = chunk_rows(a->nq, a->hq, a->c1.capacity);
    p.whole = whole_sequence(a->nq, a->hq, a->hkv, a->c1.capacity) ? 1 : 0;
    p.nchunk1 = (a->c1.capacity + p.chunk - 1) / p.chunk;
    p.nchunk2 = (cap2 + p.chunk - 1) / p.chunk;
    p.scale_log2e = a->scale * kLog2e;
    if (p.nchunk1 + p.nchunk2 == 0) return TAH_E_SHAPE;
    return TAH_OK;
}

// Shared by the two decode entry points: `ws` is the caller's workspace or the library's static scratch.
int decode_impl(const tah_duo_decode_args* a, void* ws, size_t ws_bytes, int too_small, tah_stream_t stream) {
    DecParams p;
    if (int rc = dec_fill(a, p, false, ws, ws_bytes, too_small)) return rc < 0 ? rc : TAH_OK;
    const int g = a->hq / a->hkv;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (g) {
        case 1: return launch_decode<1>(p, st);
        case 2: return launch_decode<2>(p, st);
        case 4: return launch_decode<4>(p, st);
        default: return launch_decode<8>(p, st);
    }
}

// Device address of `scratch` on the current device, looked up once per device (each GPU holds its own
// copy of the array at its own address).  Returns nullptr if the runtime refuses.
void* static_scratch_of_current_device() {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* addr[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        addr[dev] = ptr;
    }
    return addr[dev];
}

}  // namespace
}  // namespace tah

extern "C" int tah_duo_decode(const tah_duo_decode_args* a, tah_stream_t stream) {
    if (!a) return TAH_E_NULL;
    return tah::decode_impl(a, a->workspace, a->workspace_bytes, TAH_E_WORKSPACE, stream);
}

extern "C" int tah_duo_decode_static(const tah_duo_decode_args* a, tah_stream_t stream) {
    if (!a) return TAH_E_NULL;
    void* ws = tah::static_scratch_of_current_device();
    if (!ws) return TAH_E_LAUNCH;
    // No partial has to start at zero: the merge kernel reads exactly the chunks the split kernel of the
    // same call wrote, so what an earlier (larger) call left behind is never read.
    return tah::decode_impl(a, ws, TAH_DUO_STATIC_SCRATCH_BYTES, TAH_E_SCRATCH, stream);
}

namespace tah {
namespace {

// Argument checks of tah_qk_prep and its kernel parameters.  `fused`: the call is the first half of
// tah_duo_decode_step, which keeps the prepared heads in registers (q_out / k_out are not needed).
// Returns 1 when there is nothing to do.
int prep_fill(const tah_qk_prep_args* a, PrepParams& p, bool fused) {
    if (!a) return TAH_E_NULL;
    if (a->d != kD || a->rows < 0 || a->hq <= 0 || a->hkv <= 0) return TAH_E_SHAPE;
    if (a->rows == 0) return 1;
    if (!a->q || !a->k || (!fused && !a->q_out) || !a->q_weight || !a->k_weight || !a->cos || !a->sin) return TAH_E_NULL;
    if (a->append) {
        if (!a->v || !a->cu_new) return TAH_E_NULL;
        if (a->nseq <= 0 || a->cache.capacity <= 0) return TAH_E_SHAPE;
        if (int rc = check_seg(a->cache, a->pos_new != nullptr)) return rc;
    } else {
        if (!a->k_out) return TAH_E_NULL;
        if (a->v_out && !a->v) return TAH_E_NULL;
    }
    const int64_t strides[] = {a->q_row_stride, a->q_head_stride, a->k_row_stride, a->k_head_stride, a->v_row_stride,
                               a->v_head_stride, a->q_out_row_stride, a->q_out_head_stride, a->k_out_row_stride,
                               a->k_out_head_stride, a->v_out_row_stride, a->v_out_head_stride};
    for (int64_t x : strides)
        if (x % 8 != 0) return TAH_E_ALIGN;  // every access is 16 bytes wide (eight elements)
    if (a->cos_sin_row_stride % 8 != 0) return TAH_E_ALIGN;
    if (a->norm_input && (a->norm_cols <= 0 || a->norm_cols % 8 != 0 || a->norm_input_row_stride % 8 != 0)) return TAH_E_SHAPE;
    const void* ptrs[] = {a->q, a->k, a->v, a->q_out, a->k_out, a->v_out, a->q_weight, a->k_weight, a->cos, a->sin,
                          a->append ? a->cache.k : nullptr, a->append ? a->cache.v : nullptr, a->norm_input};
    for (const void* q : ptrs)
        if (q && !aligned16(q)) return TAH_E_ALIGN;
    p.q = static_cast<const __bf16*>(a->q); p.k = static_cast<const __bf16*>(a->k); p.v = static_cast<const __bf16*>(a->v);
    p.q_out = static_cast<__bf16*>(a->q_out); p.k_out = static_cast<__bf16*>(a->k_out); p.v_out = static_cast<__bf16*>(a->v_out);
    p.q_rs = a->q_row_stride; p.q_hs = a->q_head_stride; p.k_rs = a->k_row_stride; p.k_hs = a->k_head_stride;
    p.v_rs = a->v_row_stride; p.v_hs = a->v_head_stride;
    p.qo_rs = a->q_out_row_stride; p.qo_hs = a->q_out_head_stride; p.ko_rs = a->k_out_row_stride; p.ko_hs = a->k_out_head_stride;
    p.vo_rs = a->v_out_row_stride; p.vo_hs = a->v_out_head_stride;
    p.qw = static_cast<const __bf16*>(a->q_weight); p.kw = static_cast<const __bf16*>(a->k_weight);
    p.cos = static_cast<const __bf16*>(a->cos); p.sin = static_cast<const __bf16*>(a->sin);
    p.cs_rs = a->cos_sin_row_stride;
    p.eps = a->eps;
    p.rows = a->rows; p.hq = a->hq; p.hkv = a->hkv; p.append = a->append ? 1 : 0;
    p.own_len = (a->append && a->append_one_row_per_seq) ? 1 : 0;
    p.xn = static_cast<const __bf16*>(a->norm_input);
    p.xn_rs = a->norm_input_row_stride; p.xn_cols = a->norm_cols; p.xn_eps = a->norm_eps;
    p.a = AppendParams{};
    if (a->append) {
        p.a.pos_new = a->pos_new; p.a.cu_new = a->cu_new; p.a.slot_of = a->slot_of;
        p.a.ck = static_cast<__bf16*>(a->cache.k);
        p.a.cv = static_cast<__bf16*>(a->cache.v);
        p.a.cpos = a->cache.pos;
        p.a.start = a->cache.start;
        p.a.len = a->cache.len;
        p.a.ck_rs = a->cache.k_row_stride; p.a.ck_hs = a->cache.k_head_stride;
        p.a.cv_rs = a->cache.v_row_stride; p.a.cv_hs = a->cache.v_head_stride;
        p.a.capacity = a->cache.capacity; p.a.nseq = a->nseq; p.a.hkv = a->hkv;
        p.a.overflow = a->overflow;
    }
    return TAH_OK;
}

}  // namespace
}  // namespace tah

extern "C" int tah_qk_prep(const tah_qk_prep_args* a, tah_stream_t stream) {
    using namespace tah;
    PrepParams p;
    if (int rc = prep_fill(a, p, false)) return rc < 0 ? rc : TAH_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(qk_prep_kernel, dim3(a->rows), dim3(256), 0, st, p);
    if (a->append && !p.own_len) hipLaunchKernelGGL(kv_append_len_kernel, dim3((a->nseq + 63) / 64), dim3(64), 0, st, p.a);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_qk_prep_bwd(const tah_qk_prep_bwd_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    if (a->d != kD || a->rows < 0 || a->hq <= 0 || a->hkv <= 0 || a->n_partial <= 0) return TAH_E_SHAPE;
    if (!a->dw_partial) return TAH_E_NULL;
    if (reinterpret_cast<uintptr_t>(a->dw_partial) & 3) return TAH_E_ALIGN;
    if (a->rows > 0) {
        if (!a->q || !a->k || !a->dq_out || !a->dk_out || !a->dq || !a->dk || !a->q_weight || !a->k_weight || !a->cos || !a->sin)
            return TAH_E_NULL;
        for (const void* ptr : {a->q, a->k, a->dq_out, a->dk_out, (const void*)a->dq, (const void*)a->dk, a->q_weight, a->k_weight,
                                a->cos, a->sin})
            if (!aligned16(ptr)) return TAH_E_ALIGN;
        for (int64_t st : {a->q_row_stride, a->q_head_stride, a->k_row_stride, a->k_head_stride, a->dq_out_row_stride,
                           a->dq_out_head_stride, a->dk_out_row_stride, a->dk_out_head_stride, a->dq_row_stride, a->dq_head_stride,
                           a->dk_row_stride, a->dk_head_stride, a->cos_sin_row_stride})
            if (st % 8) return TAH_E_ALIGN;
    }
    PrepBwdParams p;
    p.q = static_cast<const __bf16*>(a->q); p.k = static_cast<const __bf16*>(a->k);
    p.dqo = static_cast<const __bf16*>(a->dq_out); p.dko = static_cast<const __bf16*>(a->dk_out);
    p.dq = static_cast<__bf16*>(a->dq); p.dk = static_cast<__bf16*>(a->dk);
    p.q_rs = a->q_row_stride; p.q_hs = a->q_head_stride; p.k_rs = a->k_row_stride; p.k_hs = a->k_head_stride;
    p.dqo_rs = a->dq_out_row_stride; p.dqo_hs = a->dq_out_head_stride; p.dko_rs = a->dk_out_row_stride; p.dko_hs = a->dk_out_head_stride;
    p.dq_rs = a->dq_row_stride; p.dq_hs = a->dq_head_stride; p.dk_rs = a->dk_row_stride; p.dk_hs = a->dk_head_stride;
    p.qw = static_cast<const __bf16*>(a->q_weight); p.kw = static_cast<const __bf16*>(a->k_weight);
    p.cos = static_cast<const __bf16*>(a->cos); p.sin = static_cast<const __bf16*>(a->sin);
    p.cs_rs = a->cos_sin_row_stride;
    p.eps = a->eps;
    p.rows = a->rows; p.hq = a->hq; p.hkv = a->hkv;
    p.dw_partial = a->dw_partial;
    hipLaunchKernelGGL(qk_prep_bwd_kernel, dim3(a->n_partial), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_kv_append(const tah_kv_append_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    if (a->d != kD || a->nseq < 0 || a->total_new < 0 || a->hkv <= 0 || a->hkv > 65535) return TAH_E_SHAPE;
    if (a->nseq == 0 || a->total_new == 0) return TAH_OK;
    if (!a->k_new || !a->v_new || !a->cu_new) return TAH_E_NULL;
    if (int rc = check_seg(a->cache, a->pos_new != nullptr)) return rc;
    if (a->cache.capacity == 0) return TAH_E_SHAPE;
    if (!aligned16(a->k_new) || !aligned16(a->v_new) || a->k_row_stride % 8 || a->k_head_stride % 8 ||
        a->v_row_stride % 8 || a->v_head_stride % 8)
        return TAH_E_ALIGN;
    AppendParams p;
    p.k_new = static_cast<const __bf16*>(a->k_new);
    p.v_new = static_cast<const __bf16*>(a->v_new);
    p.pos_new = a->pos_new; p.cu_new = a->cu_new; p.slot_of = a->slot_of;
    p.kn_rs = a->k_row_stride; p.kn_hs = a->k_head_stride; p.vn_rs = a->v_row_stride; p.vn_hs = a->v_head_stride;
    p.ck = static_cast<__bf16*>(a->cache.k);
    p.cv = static_cast<__bf16*>(a->cache.v);
    p.cpos = a->cache.pos;
    p.start = a->cache.start;
    p.len = a->cache.len;
    p.ck_rs = a->cache.k_row_stride; p.ck_hs = a->cache.k_head_stride;
    p.cv_rs = a->cache.v_row_stride; p.cv_hs = a->cache.v_head_stride;
    p.capacity = a->cache.capacity; p.nseq = a->nseq; p.hkv = a->hkv;
    p.overflow = a->overflow;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(kv_append_rows_kernel, dim3((a->total_new + 7) / 8), dim3(256), 0, st, p, a->total_new);
    hipLaunchKernelGGL(kv_append_len_kernel, dim3((a->nseq + 63) / 64), dim3(64), 0, st, p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

namespace tah {
namespace {
template <int G>
int launch_step(const StepParams& sp, hipStream_t st) {
    constexpr int kRedBytes = 16 * G * kPart * (int)sizeof(float);
    hipLaunchKernelGGL((duo_decode_step_kernel<G>), dim3(sp.dec.nq, sp.dec.hkv), dim3(kWholeThreads), kRedBytes, st, sp);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}
}  // namespace
}  // namespace tah

extern "C" int tah_duo_decode_step_supported(int32_t nq, int32_t hq, int32_t hkv, int32_t capacity1) {
    if (nq <= 0 || hq <= 0 || hkv <= 0 || hq % hkv) return 0;
    return tah::whole_sequence(nq, hq, hkv, capacity1) && hq / hkv <= tah::kStepMaxGroup ? 1 : 0;
}

namespace tah {
namespace {
AppendParams append_target(const tah_kv_segment& c) {
    AppendParams a{};
    a.ck = static_cast<__bf16*>(c.k);
    a.cv = static_cast<__bf16*>(c.v);
    a.cpos = c.pos;
    a.start = c.start;
    a.len = c.len;
    a.ck_rs = c.k_row_stride; a.ck_hs = c.k_head_stride; a.cv_rs = c.v_row_stride; a.cv_hs = c.v_head_stride;
    a.capacity = c.capacity;
    return a;
}
}  // namespace
}  // namespace tah

extern "C" int tah_duo_decode_step(const tah_qk_prep_args* prep, const tah_duo_decode_args* dec, const int32_t* append_at,
                                   const int32_t* append_depth, tah_stream_t stream) {
    using namespace tah;
    if (!prep || !dec) return TAH_E_NULL;
    StepParams sp;
    const int rc_p = prep_fill(prep, sp.prep, true);
    if (rc_p < 0) return rc_p;
    const int rc_d = dec_fill(dec, sp.dec, true, nullptr, 0, TAH_E_WORKSPACE);
    if (rc_d < 0) return rc_d;
    if (rc_p == 1 && rc_d == 1) return TAH_OK;
    // one row per sequence, appended to one of the two segments the queries read, in a call the one-workgroup kernel takes
    if (rc_p == 1 || rc_d == 1 || prep->rows != dec->nq || prep->hq != dec->hq || prep->hkv != dec->hkv) return TAH_E_SHAPE;
    if (!prep->append || !prep->append_one_row_per_seq || prep->nseq != prep->rows || !prep->v) return TAH_E_SHAPE;
    if (!tah_duo_decode_step_supported(dec->nq, dec->hq, dec->hkv, dec->c1.capacity)) return TAH_E_SHAPE;
    if (!append_at) return TAH_E_NULL;
    const bool have2 = dec->q_depth != nullptr || dec->depth >= 1;
    if (prep->cache.k == dec->c1.k) sp.append_second = 0;
    else if (prep->cache.k == dec->c2.k && have2) sp.append_second = 1;
    else return TAH_E_SHAPE;
    if (append_depth && !have2) return TAH_E_SHAPE;  // rows that append to the depth-1 segment need it
    sp.app[0] = append_target(dec->c1);
    sp.app[1] = have2 ? append_target(dec->c2) : AppendParams{};
    sp.append_at = append_at;
    sp.append_depth = append_depth;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return dec->hq / dec->hkv == 1 ? launch_step<1>(sp, st) : launch_step<2>(sp, st);
}
