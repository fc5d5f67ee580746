// Launch-order table of a varlen call: every tile of the query-tile kernels (forward, dQ) and of the key-tile
// kernel (dK/dV), sorted by the tile steps it will run, heaviest first.
//
// The kernels launch one workgroup per (kv head, tile) and a compute unit holds one of them at a time, so a
// call is a few hundred unequal jobs on 256 units; handed out in sequence order, the long tiles of a later
// document start when most units are already busy with short ones and the launch ends on them.  Handing the
// tiles out longest-first is the classic remedy, and with several documents in a batch it needs an order across
// documents, which depends on the sequence boundaries on the device: one 1024-thread workgroup builds it with a
// counting sort (tile steps are small integers) and the kernels read their tile from the table instead of
// deriving it from blockIdx.  Integer work, no host read-back; a table built from the call's own boundaries only
// changes the order in which tiles are started, never a result: the table is a permutation of the tile numbers, which
// the kernels turn into tiles from the call's own boundaries, so even one built from other boundaries of the same
// sizes makes them visit every tile once (in an order that is no longer the intended one).  Tiles of equal weight are
// placed in the order their threads reach the bin's counter, so the table's order among equals can differ from build to
// build; results do not depend on it.
#include <hip/hip_runtime.h>

#include "duo_device.h"
#include "tah_duo.h"

namespace tah {
namespace {

constexpr int kSchedThreads = 1024;
constexpr int kSchedMaxSeq = 4095;  // tile offsets of nseq + 1 boundaries per stream are held (and scanned) in LDS
constexpr int kSchedBins = 4096;    // tile steps are clipped to this many sort keys
constexpr int kStep = 64;           // keys (forward, dQ) or query rows (dK/dV) per tile step

struct SchedParams {
    const int32_t *cu_q1, *cu_k1, *cu_q2, *cu_k2, *pos_q2;
    int32_t nseq, group, bm;
    int32_t total_q1, total_k1, total_q2, total_k2;
    int32_t q_slots, k_slots;
    int32_t* out;
};

// exclusive scan of a[0..n) in LDS, n <= 4 * kSchedThreads, in place; returns the total
__device__ int block_exclusive_scan(int* a, int n, int* tmp) {
    const int tid = threadIdx.x;
    int v[4], sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int j = 4 * tid + i;
        v[i] = j < n ? a[j] : 0;
        sum += v[i];
    }
    tmp[tid] = sum;
    __syncthreads();
    for (int d = 1; d < kSchedThreads; d <<= 1) {  // Hillis-Steele over the per-thread sums
        const int y = tid >= d ? tmp[tid - d] : 0;
        __syncthreads();
        tmp[tid] += y;
        __syncthreads();
    }
    int run = tmp[tid] - sum;
    const int total = tmp[kSchedThreads - 1];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int j = 4 * tid + i;
        if (j < n) a[j] = run;
        run += v[i];
    }
    __syncthreads();
    return total;
}

__device__ __forceinline__ int seg_len(const int32_t* cu, int total, int b) { return total > 0 ? cu[b + 1] - cu[b] : 0; }
__device__ __forceinline__ int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Tile steps of tile i (rows i*tile .. of its segment) of sequence b in stream `second`.
template <bool kKeyTiles>
__device__ int tile_steps(const SchedParams& p, bool second, int b, int i, int tile) {
    const int lq1 = seg_len(p.cu_q1, p.total_q1, b), lk1 = seg_len(p.cu_k1, p.total_k1, b);
    const int lq2 = seg_len(p.cu_q2, p.total_q2, b), lk2 = seg_len(p.cu_k2, p.total_k2, b);
    const int off = lk1 - lq1;  // position of depth-0 query row r is r + off
    if (!kKeyTiles) {
        // query tile: depth-0 keys up to the position of its last row (+ every depth-1 key tile for depth-1 rows)
        const int lq = second ? lq2 : lq1;
        const int last_row = ((i + 1) * tile < lq ? (i + 1) * tile : lq) - 1;
        int last_pos = second ? p.pos_q2[p.cu_q2[b] + last_row] : last_row + off;
        last_pos = last_pos < lk1 - 1 ? last_pos : lk1 - 1;
        return (last_pos >= 0 ? last_pos / kStep + 1 : 0) + (second ? ceil_div(lk2, kStep) : 0);
    }
    // key tile: the query rows at or after its first key (depth-0 keys are seen by both depths' queries)
    if (second) return ceil_div(lq2, kStep);
    int first_row = i * tile - off;
    first_row = first_row > 0 ? first_row : 0;
    const int nvis = lq1 > first_row ? lq1 - first_row : 0;
    return ceil_div(nvis, kStep) + ceil_div(lq2, kStep);
}

// One sorted list: tiles of `tile` rows over segments cu_a (stream 0) and cu_b (stream 1), `slots` pairs at out.
template <bool kKeyTiles>
__device__ void build_list(const SchedParams& p, const int32_t* cu_a, int total_a, const int32_t* cu_b, int total_b,
                           int tile, int slots, int32_t* out, int* off_a, int* off_b, int* bins, int* tmp) {
    const int tid = threadIdx.x;
    for (int b = tid; b <= p.nseq; b += kSchedThreads) {
        off_a[b] = b < p.nseq ? ceil_div(seg_len(cu_a, total_a, b), tile) : 0;
        off_b[b] = b < p.nseq ? ceil_div(seg_len(cu_b, total_b, b), tile) : 0;
    }
    for (int c = tid; c < kSchedBins; c += kSchedThreads) bins[c] = 0;
    __syncthreads();
    const int n_a = block_exclusive_scan(off_a, p.nseq + 1, tmp);
    const int n_b = block_exclusive_scan(off_b, p.nseq + 1, tmp);
    const int n = n_a + n_b;

    auto locate = [&](int t, bool& second, int& b, int& i) {
        second = t >= n_a;
        const int* off = second ? off_b : off_a;
        const int local = second ? t - n_a : t;
        int lo = 0, hi = p.nseq;  // last b with off[b] <= local (sequences without tiles repeat an offset)
        while (hi - lo > 1) {
            const int mid = (lo + hi) / 2;
            if (off[mid] <= local) lo = mid; else hi = mid;
        }
        b = lo;
        i = local - off[lo];
    };
    auto sort_key = [&](bool second, int b, int i) {  // ascending key = descending tile steps
        const int steps = tile_steps<kKeyTiles>(p, second, b, i, tile);
        return kSchedBins - 1 - (steps < kSchedBins - 1 ? steps : kSchedBins - 1);
    };
    for (int t = tid; t < n; t += kSchedThreads) {
        bool second; int b, i;
        locate(t, second, b, i);
        atomicAdd(&bins[sort_key(second, b, i)], 1);
    }
    __syncthreads();
    block_exclusive_scan(bins, kSchedBins, tmp);
    for (int t = tid; t < n; t += kSchedThreads) {
        bool second; int b, i;
        locate(t, second, b, i);
        const int at = atomicAdd(&bins[sort_key(second, b, i)], 1);  // ties land in arrival order: same steps either way
        if (at < slots) {
            out[2 * at] = t;  // the tile's number in sequence order, which the kernels turn into (sequence, first row)
            out[2 * at + 1] = 0;
        }
    }
    for (int t = n + tid; t < slots; t += kSchedThreads) {  // numbers without a tile (for these boundaries) come last
        out[2 * t] = t;
        out[2 * t + 1] = 0;
    }
    __syncthreads();
}

__global__ __launch_bounds__(kSchedThreads) void schedule_build_kernel(const SchedParams p) {
    __shared__ int off_a[kSchedMaxSeq + 1], off_b[kSchedMaxSeq + 1], bins[kSchedBins], tmp[kSchedThreads];
    int32_t* q_list = p.out + kSchedHeaderWords;
    int32_t* k_list = q_list + 2 * p.q_slots;
    build_list<false>(p, p.cu_q1, p.total_q1, p.cu_q2, p.total_q2, p.bm, p.q_slots, q_list, off_a, off_b, bins, tmp);
    build_list<true>(p, p.cu_k1, p.total_k1, p.cu_k2, p.total_k2, kSchedKeyTile, p.k_slots, k_list, off_a, off_b, bins, tmp);
    if (threadIdx.x < kSchedHeaderWords) {
        int32_t h = 0;
        switch (threadIdx.x) {
            case 0: h = kSchedMagic; break;
            case kSchedNseq: h = p.nseq; break;
            case kSchedGroup: h = p.group; break;
            case kSchedTotalQ1: h = p.total_q1; break;
            case kSchedTotalQ2: h = p.total_q2; break;
            case kSchedTotalK1: h = p.total_k1; break;
            case kSchedTotalK2: h = p.total_k2; break;
            case kSchedQSlots: h = p.q_slots; break;
            case kSchedKSlots: h = p.k_slots; break;
            default: break;
        }
        p.out[threadIdx.x] = h;
    }
}

bool sched_shape_ok(int nseq, int hq, int hkv, int tq1, int tk1, int tq2, int tk2) {
    if (nseq < 0 || hq <= 0 || hkv <= 0 || hq % hkv != 0 || tq1 < 0 || tk1 < 0 || tq2 < 0 || tk2 < 0) return false;
    const int g = hq / hkv;
    return g == 1 || g == 2 || g == 4 || g == 8;
}

}  // namespace
}  // namespace tah

extern "C" size_t tah_duo_schedule_bytes(int32_t nseq, int32_t hq, int32_t hkv, int32_t total_q1, int32_t total_k1,
                                         int32_t total_q2, int32_t total_k2) {
    if (!tah::sched_shape_ok(nseq, hq, hkv, total_q1, total_k1, total_q2, total_k2)) return 0;
    const int bm = 32 * (8 / (hq / hkv));
    const size_t words = tah::kSchedHeaderWords + 2 * (size_t)tah::sched_slots(nseq, bm, total_q1, total_q2) +
                         2 * (size_t)tah::sched_slots(nseq, tah::kSchedKeyTile, total_k1, total_k2);
    return words * sizeof(int32_t);
}

extern "C" int tah_duo_schedule_build(const tah_duo_schedule_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a || !a->schedule) return TAH_E_NULL;
    if (!sched_shape_ok(a->nseq, a->hq, a->hkv, a->total_q1, a->total_k1, a->total_q2, a->total_k2)) return TAH_E_SHAPE;
    if (a->nseq > kSchedMaxSeq) return TAH_E_SHAPE;
    if ((a->total_q1 > 0 && !a->cu_q1) || (a->total_k1 > 0 && !a->cu_k1) || (a->total_q2 > 0 && (!a->cu_q2 || !a->pos_q2)) ||
        (a->total_k2 > 0 && !a->cu_k2))
        return TAH_E_NULL;
    if (a->total_q1 > 0 && !a->cu_k1) return TAH_E_NULL;  // positions of depth-0 rows count from the key segment
    if (a->schedule_bytes < tah_duo_schedule_bytes(a->nseq, a->hq, a->hkv, a->total_q1, a->total_k1, a->total_q2, a->total_k2))
        return TAH_E_WORKSPACE;
    SchedParams p;
    p.cu_q1 = a->cu_q1; p.cu_k1 = a->cu_k1; p.cu_q2 = a->cu_q2; p.cu_k2 = a->cu_k2; p.pos_q2 = a->pos_q2;
    p.nseq = a->nseq;
    p.group = a->hq / a->hkv;
    p.bm = 32 * (8 / p.group);
    p.total_q1 = a->total_q1; p.total_k1 = a->total_k1; p.total_q2 = a->total_q2; p.total_k2 = a->total_k2;
    p.q_slots = sched_slots(a->nseq, p.bm, a->total_q1, a->total_q2);
    p.k_slots = sched_slots(a->nseq, kSchedKeyTile, a->total_k1, a->total_k2);
    p.out = static_cast<int32_t*>(a->schedule);
    hipLaunchKernelGGL(schedule_build_kernel, dim3(1), dim3(kSchedThreads), 0, static_cast<hipStream_t>(stream), p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}
