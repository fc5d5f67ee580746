// Duo-causal attention backward (training), bf16 MFMA, gfx950.
//
// Three kernels, no atomics, deterministic:
//   delta     delta[h][row] = sum_d dO*O                                (fp32)
//   dq        one workgroup per query tile, same tiling as the forward:
//             S^T = K Q^T, dP^T = V dO^T, dS^T = P^T o (dP^T - delta),
//             dQ^T += K^T dS^T  (K^T operand via LDS transpose reads)
//   dkdv      one workgroup (8 waves) per 128-key tile of one kv head; loops
//             over every query tile that can see it, for all query heads of
//             the group and for both query streams (depth-0 keys collect
//             gradient from depth-0 and depth-1 queries):
//             S = Q K^T, dP = dO V^T, dV += P^T dO, dK += dS^T Q
// P is recomputed from the saved log-sum-exp.  In dkdv each lane owns one key
// (accumulator column); the workgroup's K and V tiles and the staged Q and dO
// tiles sit in LDS, the latter read both row-wise (A operand) and, through
// ds_read_b64_tr_b16, column-wise (B operand).  The 32 MFMAs of an item are
// laid out as explicit slots with their LDS reads issued two to three slots
// ahead and the exp / convert arithmetic sliced in behind the dP and dV MFMAs.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "duo_device.h"
#include "tah_duo.h"


namespace tah {
namespace {

typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kD = 128;
constexpr int kBN = 64;
constexpr int kTileBytes = kBN * kD * 2;  // one 64 x 128 bf16 tile

struct BwdStream {
    const __bf16 *q, *k, *v, *o, *d_o;
    __bf16 *dq, *dk, *dv;
    const float* lse;
    float* delta;
    const int32_t *cu_q, *cu_k, *pos_q, *pos_k;
    int64_t q_rs, q_hs, k_rs, k_hs, v_rs, v_hs, o_rs, o_hs;
    int64_t do_rs, do_hs, dq_rs, dq_hs, dk_rs, dk_hs, dv_rs, dv_hs;
    int32_t total_q, total_k;
};
struct BwdParams {
    BwdStream s1, s2;
    int32_t nseq, hq, hkv;
    float scale, scale_log2e;
    const int32_t* sched;  // launch-order table or nullptr
    // additive-mask mode only: mask[seq][head][query index][key index], strides in elements
    const void* mask;
    int64_t mask_sb, mask_sh, mask_sq, mask_sk;
    int32_t mask_f32;  // element type: 1 = float, 0 = bf16
    float inv_scale;   // 1 / scale: the mask is added to raw scores as mask / scale
    // dS exchange between the key-tile kernel and the dQ kernel that reads it back (see ds_block)
    unsigned char* ds_ws;
    int32_t ds_q1slots, ds_kt1, ds_kt;
};

// ---------------------------------------------------------------------------
// dS exchange.  With a workspace the key-tile kernel (which forms S, P, dP and dS for dK / dV anyway) also
// writes dS, and dQ = scale * dS K becomes one product that reads it back instead of a second pass that
// recomputes S and dP: 5 products per (query tile, key tile) pair instead of 7.
// The workspace is a table of 16 KiB blocks, one per (64 query rows, query head, 128 keys):
//   block = ((qslot * hq + head) * ds_kt + ktile)
//   qslot = cu_q1[seq] / 64 + seq + tile                  depth-0 query rows  (ds_q1slots slots)
//           ds_q1slots + cu_q2[seq] / 64 + seq + tile     depth-1 query rows
//   ktile = key tile inside its sequence (depth 0), ds_kt1 + key tile (depth 1)
// (cu / 64 + seq numbers the 64-row tiles of successive sequences without collisions and needs no prefix
// sum over tile counts.)  Inside a block wave w = 4 * (query half) + (32-key block) of the key-tile kernel
// owns 2 KiB: its bf16 dS registers as they are, 16 bytes (four query rows of one key, twice) per lane,
// placed so that the reader's transpose reads of one half-wave cover 256 contiguous bytes:
//   16-byte piece (a2 = register / 8, key k = lane % 32, hf = lane / 32)  ->  ((k/4)*16 + a2*8 + hf*4 + k%4) * 16
// and holds rows 16*a2 + 8*j + 4*hf + 0..3 (j = 0, 1 in the piece's two halves) of the wave's 32 query rows.
// ---------------------------------------------------------------------------
constexpr int kDsBlockBytes = 64 * 128 * 2;
constexpr int kDsWaveBytes = 2048;
__device__ __forceinline__ int ds_piece_off(int a2, int k, int hf) { return (((k >> 2) << 4) + (a2 << 3) + (hf << 2) + (k & 3)) << 4; }
inline __host__ __device__ int ds_key_slots(int total_k, int max_k) {
    const int m = (max_k > 0 && max_k < total_k) ? max_k : total_k;
    return total_k > 0 ? (m + 127) / 128 : 0;
}
inline __host__ __device__ int ds_query_slots(int total_q, int nseq) { return total_q > 0 ? total_q / 64 + nseq : 0; }


__device__ __forceinline__ float mask_value(const BwdParams& p, const unsigned char* row, int64_t k) {
    return p.mask_f32 ? reinterpret_cast<const float*>(row)[k * p.mask_sk]
                      : (float)reinterpret_cast<const __bf16*>(row)[k * p.mask_sk];
}

// ---------------------------------------------------------------------------
// delta = rowsum(dO * O): 16 lanes per (row, head), 8 elements each; behind the Hq * total_q deltas the same
// launch leaves lse * log2(e), the form in which the dK/dV kernel subtracts it from the scaled scores
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
    return x + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}

__global__ __launch_bounds__(256) void duo_bwd_delta_kernel(const BwdStream s, int hq) {
    const int64_t item = (int64_t)blockIdx.x * 16 + threadIdx.x / 16;  // (row, head) pair
    const int dc = threadIdx.x % 16;
    const int64_t total = (int64_t)s.total_q * hq;
    const int64_t it = item < total ? item : total - 1;
    const int row = (int)(it / hq), head = (int)(it % hq);
    const bf16x8 a = ld_global_16B(s.o + (int64_t)row * s.o_rs + (int64_t)head * s.o_hs + dc * 8);
    const bf16x8 b = ld_global_16B(s.d_o + (int64_t)row * s.do_rs + (int64_t)head * s.do_hs + dc * 8);
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc += (float)a[i] * (float)b[i];
    acc = dpp_add<0xB1>(acc);
    acc = dpp_add<0x4E>(acc);
    acc = dpp_add<0x141>(acc);
    acc = dpp_add<0x140>(acc);
    if (dc == 0 && item < total) {
        s.delta[(int64_t)head * s.total_q + row] = acc;
        s.delta[total + (int64_t)head * s.total_q + row] = s.lse[(int64_t)head * s.total_q + row] * kLog2e;
    }
}

// ---------------------------------------------------------------------------
// dQ kernel
// ---------------------------------------------------------------------------
constexpr int kDqThreads = 512;
constexpr int kDqStage = 2 * kTileBytes + kBN * 4;   // K tile, V tile, key positions
constexpr int kDqSmem = 2 * kDqStage + 64;

enum class Mask { kNone, kIndex, kPos };

// kDense: additive-mask mode (see the forward kernel): every key of the sequence, visibility from the mask.
template <int G, bool kDense>
__global__ __launch_bounds__(kDqThreads) TAH_WAVES_PER_EU(2, 2) void duo_bwd_dq_kernel(const BwdParams p) {
    constexpr int BM = 32 * (8 / G);
    HIP_DYNAMIC_SHARED(unsigned char, smem)
    const int tid = threadIdx.x, lane = tid % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // wave-uniform: lives in a scalar register
    const int half = lane / 32, col = lane % 32;
    const int hk = blockIdx.x;

    int seq = 0, row0 = 0, row_end = 0;
    bool second = false;
    int slot = (int)(gridDim.y - 1 - blockIdx.y);  // without a table: late (heavy) tiles of each sequence first
    // (the table's order: heaviest tile of the whole call first)
    sched_lookup(p.sched, false, p.nseq, G, p.s1.total_q, p.s2.total_q, p.s1.total_k, p.s2.total_k, (int)gridDim.y,
                 (int)blockIdx.y, slot);
    if (!(p.s1.total_q > 0 && find_tile(p.s1.cu_q, p.nseq, BM, slot, seq, row0, row_end))) {
        if (!(p.s2.total_q > 0 && find_tile(p.s2.cu_q, p.nseq, BM, slot, seq, row0, row_end))) return;
        second = true;
    }
    const BwdStream& qs = second ? p.s2 : p.s1;
    const int head = hk * G + wave % G;
    const int rblk = wave / G;
    const int k1_lo = p.s1.cu_k[seq];
    const int lk1 = p.s1.cu_k[seq + 1] - k1_lo;
    const __bf16* k1p = p.s1.k + (int64_t)k1_lo * p.s1.k_rs + (int64_t)hk * p.s1.k_hs;
    const __bf16* v1p = p.s1.v + (int64_t)k1_lo * p.s1.v_rs + (int64_t)hk * p.s1.v_hs;
    const int left1 = p.s1.total_k - k1_lo;
    int lk2 = 0, left2 = 0;
    const __bf16 *k2p = nullptr, *v2p = nullptr;
    const int32_t* pos2p = nullptr;
    if (second) {
        const int k2_lo = p.s2.cu_k[seq];
        lk2 = p.s2.cu_k[seq + 1] - k2_lo;
        k2p = p.s2.k + (int64_t)k2_lo * p.s2.k_rs + (int64_t)hk * p.s2.k_hs;
        v2p = p.s2.v + (int64_t)k2_lo * p.s2.v_rs + (int64_t)hk * p.s2.v_hs;
        pos2p = p.s2.pos_k + k2_lo;
        left2 = p.s2.total_k - k2_lo;
    }

    const int row = row0 + rblk * 32 + col;
    const bool row_ok = row < row_end;
    const int row_ld = row_ok ? row : row_end - 1;
    int qpos;
    if (second) {
        qpos = qs.pos_q[row_ld];
    } else {
        const int q_lo = qs.cu_q[seq];
        qpos = (row_ld - q_lo) + (lk1 - (qs.cu_q[seq + 1] - q_lo));
    }
    const int qlim1 = row_ok ? ((qpos < lk1 - 1 && !kDense) ? qpos : lk1 - 1) : -1;
    const int qlim2 = row_ok ? qpos : -1;
    const int wmax1 = wave_reduce_max(qlim1);
    const int wmin1 = wave_reduce_min(row_ok ? qlim1 : 0x7fffffff);
    int* bounds = reinterpret_cast<int*>(smem + 2 * kDqStage);
    if (lane == 0) bounds[wave] = wmax1;
    __syncthreads();
    int tmax1 = -1;
#pragma unroll
    for (int w = 0; w < 8; ++w) tmax1 = bounds[w] > tmax1 ? bounds[w] : tmax1;
    // same tile schedule as the forward kernel: plain / index-masked / idle depth-0 tiles, then depth-1 tiles
    // (all wave-uniform: moved to scalar registers so that the tile loops are scalar loops)
    const int n1 = __builtin_amdgcn_readfirstlane(tmax1 >= 0 ? tmax1 / kBN + 1 : 0);
    const int n2 = second ? (lk2 + kBN - 1) / kBN : 0;
    const int ntiles = n1 + n2;
    const int n_active = __builtin_amdgcn_readfirstlane(wmax1 >= 0 ? wmax1 / kBN + 1 : 0);
    int n_plain = __builtin_amdgcn_readfirstlane(wmin1 >= kBN - 1 ? (wmin1 - (kBN - 1)) / kBN + 1 : 0);
    n_plain = n_plain < n_active ? n_plain : n_active;
    if constexpr (kDense) n_plain = 0;  // the mask is read for every tile
    const unsigned char* mask_row = nullptr;  // additive-mask mode: this lane's mask row
    if constexpr (kDense) {
        const int64_t e = (int64_t)seq * p.mask_sb + (int64_t)head * p.mask_sh +
                          (int64_t)(row_ld - qs.cu_q[seq]) * p.mask_sq;
        mask_row = static_cast<const unsigned char*>(p.mask) + e * (p.mask_f32 ? 4 : 2);
    }

    bf16x8 qf[8], dof[8];
    {
        const __bf16* qrow = qs.q + (int64_t)row_ld * qs.q_rs + (int64_t)head * qs.q_hs + 8 * half;
        const __bf16* gorow = qs.d_o + (int64_t)row_ld * qs.do_rs + (int64_t)head * qs.do_hs + 8 * half;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            qf[s] = ld_global_16B(qrow + 16 * s);
            dof[s] = ld_global_16B(gorow + 16 * s);
        }
    }
    const float c = p.scale_log2e;
    float lse_c = qs.lse[(int64_t)head * qs.total_q + row_ld] * kLog2e;
    if constexpr (kDense) lse_c = lse_c == kNegInf ? -kNegInf : lse_c;  // a row that hides every key: P = 0, not exp(-inf + inf)
    const float delta = qs.delta[(int64_t)head * qs.total_q + row_ld];

    f32x16 dqacc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) dqacc[i][r] = 0.f;

    // asynchronous global -> LDS copy of one K/V tile (both row-major, swizzled), as in the forward
    // kernel: (wave-uniform pointer to the tile's first row) + (per-lane byte offset), rows past the
    // end of the array repeat its last row (finite data, masked by index)
    const int my_lrow = 8 * wave + (lane >> 4);  // second piece: 4 rows further down
    const uint32_t my_chunk0 = (uint32_t)(((lane & 15) ^ row_swizzle(my_lrow)) * 16);
    const uint32_t my_chunk1 = (uint32_t)(((lane & 15) ^ row_swizzle(my_lrow + 4)) * 16);
    auto issue_tile = [&](int it, int buf) {
        const bool s0 = it < n1;
        const int base = (s0 ? it : it - n1) * kBN;
        const int64_t krs = s0 ? p.s1.k_rs : p.s2.k_rs;
        const int64_t vrs = s0 ? p.s1.v_rs : p.s2.v_rs;
        const __bf16* kt0 = (s0 ? k1p : k2p) + (int64_t)base * krs;
        const __bf16* vt0 = (s0 ? v1p : v2p) + (int64_t)base * vrs;
        const int last = (s0 ? left1 : left2) - 1 - base;  // >= 0: a tile starts inside its segment
        unsigned char* kt = smem + buf * kDqStage;
        unsigned char* vt = kt + kTileBytes;
        const uint32_t r0 = (uint32_t)(my_lrow < last ? my_lrow : last) & 63u;
        const uint32_t r1 = (uint32_t)(my_lrow + 4 < last ? my_lrow + 4 : last) & 63u;
        const uint32_t krs2 = (uint32_t)(krs * 2) & 0xffffffu, vrs2 = (uint32_t)(vrs * 2) & 0xffffffu;
        if (!s0 && wave == 0) {  // positions of the depth-1 keys (indices past the segment repeat the last one)
            const int nleft = lk2 - base;
            async_copy_4B(pos2p + base, (uint32_t)(lane < nleft ? lane : nleft - 1) * 4u, vt + kTileBytes);
        }
        async_copy_16B(kt0, r0 * krs2 + my_chunk0, kt + (2 * wave) * 1024);
        async_copy_16B(vt0, r0 * vrs2 + my_chunk0, vt + (2 * wave) * 1024);
        async_copy_16B(kt0, r1 * krs2 + my_chunk1, kt + (2 * wave + 1) * 1024);
        async_copy_16B(vt0, r1 * vrs2 + my_chunk1, vt + (2 * wave + 1) * 1024);
    };
    auto advance = [&](int it) {
        TAH_WAIT_VMEM();
        __syncthreads();
        if (it + 1 < ntiles) issue_tile(it + 1, (it & 1) ^ 1);
    };

    int koff[8];
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) koff[s8] = rowmajor128_off(col, 2 * s8 + half);
    int toff_lo[4], toff_hi[4];  // transpose reads of K: rows 4*half + r/4 (+8), columns 32*dt + 16*grp + 4*(r%4)
    {
        const int r16 = lane & 15, grp = (lane >> 4) & 1;
        const int trow = 4 * half + (r16 >> 2);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            const int tcol = 32 * dt + 16 * grp + 4 * (r16 & 3);
            toff_lo[dt] = rowmajor128_off(trow, tcol >> 3) + (tcol & 7) * 2;
            toff_hi[dt] = rowmajor128_off(trow + 8, tcol >> 3) + (tcol & 7) * 2;
        }
    }

    auto tile = [&](int it, auto mask_tag) __attribute__((always_inline)) {
        constexpr Mask kMask = decltype(mask_tag)::value;
        const unsigned char* kt = smem + (it & 1) * kDqStage;
        const unsigned char* vt = kt + kTileBytes;
        const int* kpos = reinterpret_cast<const int*>(vt + kTileBytes);
        const int base = (it < n1 ? it : it - n1) * kBN;
        [[maybe_unused]] const int nleft = lk2 - base;  // depth-1 tiles: keys of this tile that exist
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        bf16x8 dsf[4];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            // S^T = K Q^T and dP^T = V dO^T for 32 keys x 32 queries
            f32x16 sacc = mfma32(*reinterpret_cast<const bf16x8*>(kt + koff[0] + mt * 8192), qf[0], zero);
            f32x16 dpacc = mfma32(*reinterpret_cast<const bf16x8*>(vt + koff[0] + mt * 8192), dof[0], zero);
#pragma unroll
            for (int s = 1; s < 8; ++s) {
                sacc = mfma32(*reinterpret_cast<const bf16x8*>(kt + koff[s] + mt * 8192), qf[s], sacc);
                dpacc = mfma32(*reinterpret_cast<const bf16x8*>(vt + koff[s] + mt * 8192), dof[s], dpacc);
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                bool vis = true;
                const int kl = 32 * mt + acc_row(half, r);
                if constexpr (kMask == Mask::kIndex) vis = base + kl <= qlim1;
                if constexpr (kMask == Mask::kPos) vis = kl < nleft && kpos[kl] <= qlim2;
                float sc = sacc[r];
                if constexpr (kDense) sc += mask_value(p, mask_row, vis ? base + kl : 0) * p.inv_scale;
                const float pr = vis ? fast_exp2(sc * c - lse_c) : 0.f;
                dsf[2 * mt + r / 8][r % 8] = (__bf16)(pr * (dpacc[r] - delta));
            }
        }
        // dQ^T (128 d x 32 queries) += K^T dS^T, K^T read column-wise from the row-major tile
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                const bf16x4 lo = lds_read_tr16(kt + toff_lo[dt] + st * 4096);
                const bf16x4 hi = lds_read_tr16(kt + toff_hi[dt] + st * 4096);
                dqacc[dt] = mfma32(__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7), dsf[st], dqacc[dt]);
            }
    };
    using PlainTag = std::integral_constant<Mask, Mask::kNone>;
    using IndexTag = std::integral_constant<Mask, Mask::kIndex>;
    using PosTag = std::integral_constant<Mask, Mask::kPos>;

    TAH_WAIT_VMEM();  // Q / dO fragments, lse and delta are in
    if (ntiles > 0) issue_tile(0, 0);
    int it = 0;
    for (; it < n_plain; ++it) { advance(it); tile(it, PlainTag{}); }
    for (; it < n_active; ++it) { advance(it); tile(it, IndexTag{}); }
    for (; it < n1; ++it) advance(it);
    for (; it < ntiles; ++it) { advance(it); tile(it, PosTag{}); }

    if (row_ok) {
        __bf16* drow = qs.dq + (int64_t)row * qs.dq_rs + (int64_t)head * qs.dq_hs;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                bf16x4 v4;
#pragma unroll
                for (int b = 0; b < 4; ++b) v4[b] = (__bf16)(dqacc[dt][4 * g4 + b] * p.scale);
                *reinterpret_cast<bf16x4*>(drow + 32 * dt + 8 * g4 + 4 * half) = v4;
            }
    }
}

// ---------------------------------------------------------------------------
// dK/dV kernel
// ---------------------------------------------------------------------------
constexpr int kKvThreads = 512;                           // 8 waves = 4 key blocks x 2 query halves
constexpr int kKB = 4;                                    // 32-key blocks per workgroup
constexpr int kBK = 32 * kKB;                             // keys per workgroup
static_assert(kBK == kSchedKeyTile, "the launch-order table lists key tiles of this size");
constexpr int kBQ = 64;                                   // query rows per staged tile
constexpr int kKvSlot = 2 * kTileBytes;                   // one stage: Q tile, dO tile (32 KiB)
constexpr int kKvK = 2 * kKvSlot;                         // after the two stages: this workgroup's K tile (128 x 128 bf16) ...
constexpr int kKvV = kKvK + kBK * kD * 2;                 // ... and V tile
constexpr int kKvMeta = kKvV + kBK * kD * 2;              // then per stage: lse, delta, query positions (64 dwords each)
constexpr int kKvMetaBytes = 3 * kBQ * 4;
constexpr int kKvSmem = kKvMeta + 2 * kKvMetaBytes;
constexpr int kKvRed = kKB * 128 * 64 * 4;                // final reduction: [key block][128 regs][64 lanes] f32, reuses the front
static_assert(kKvRed <= kKvSmem, "reduction buffer must fit");

// kExport: dS of every item is also written to the exchange workspace (p.ds_ws), for duo_bwd_dq_from_ds_kernel.
template <int G, bool kDense, bool kExport>
__global__ __launch_bounds__(kKvThreads) TAH_WAVES_PER_EU(2, 2) void duo_bwd_dkdv_kernel(const BwdParams p) {
    HIP_DYNAMIC_SHARED(unsigned char, smem_array)
    TAH_LDS_ZERO_BASED(smem, smem_array);
    const int tid = threadIdx.x, lane = tid % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // wave-uniform: lives in a scalar register
    const int half = lane / 32, col = lane % 32;
    const int kb = wave % kKB, qh = wave / kKB;  // 32-key block, 32-row half of the query tile
    const int hk = blockIdx.x;

    int seq = 0, key0 = 0, key_end = 0;
    bool second = false;
    int slot = (int)blockIdx.y;  // without a table: early (heavy) key tiles of each sequence first
    // (the table's order: the key tile seen by the most query rows first)
    sched_lookup(p.sched, true, p.nseq, G, p.s1.total_q, p.s2.total_q, p.s1.total_k, p.s2.total_k, (int)gridDim.y,
                 (int)blockIdx.y, slot);
    if (!(p.s1.total_k > 0 && find_tile(p.s1.cu_k, p.nseq, kBK, slot, seq, key0, key_end))) {
        if (!(p.s2.total_k > 0 && find_tile(p.s2.cu_k, p.nseq, kBK, slot, seq, key0, key_end))) return;
        second = true;
    }
    const BwdStream& ks = second ? p.s2 : p.s1;
    const int k_lo = ks.cu_k[seq];
    const int lk1 = p.s1.cu_k[seq + 1] - p.s1.cu_k[seq];
    const int q1_lo = p.s1.total_q > 0 ? p.s1.cu_q[seq] : 0;
    const int lq1 = p.s1.total_q > 0 ? p.s1.cu_q[seq + 1] - q1_lo : 0;
    const int q2_lo = p.s2.total_q > 0 ? p.s2.cu_q[seq] : 0;
    const int lq2 = p.s2.total_q > 0 ? p.s2.cu_q[seq + 1] - q2_lo : 0;
    const int off = lk1 - lq1;  // position of depth-0 query i is i + off

    // my key (accumulator column) and its position
    const int key = key0 + 32 * kb + col;
    const bool key_ok = key < key_end;
    const int key_ld = key_ok ? key : key_end - 1;
    const int kpos = key_ok ? (second ? ks.pos_k[key_ld] : key_ld - k_lo) : 0x7fffffff;

    // This workgroup's K and V rows go to LDS once (row-major, swizzled like every tile): they are the
    // B operands of S = Q K^T and dP = dO V^T, read again for every item -- keeping them in registers
    // instead would cost 64 registers per lane for the whole kernel.
    {
        const __bf16* kbase = ks.k + (int64_t)key0 * ks.k_rs + (int64_t)hk * ks.k_hs;
        const __bf16* vbase = ks.v + (int64_t)key0 * ks.v_rs + (int64_t)hk * ks.v_hs;
        const uint32_t krs2 = (uint32_t)(ks.k_rs * 2) & 0xffffffu, vrs2 = (uint32_t)(ks.v_rs * 2) & 0xffffffu;
        const int last = key_end - 1 - key0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // 32 blocks of 4 rows per tile, four per wave
            const int blk = 4 * wave + i;
            const int lrow = 4 * blk + (lane >> 4);
            const uint32_t lr = (uint32_t)(lrow < last ? lrow : last) & 127u;
            const uint32_t chunk = (uint32_t)(((lane & 15) ^ row_swizzle(lrow)) * 16);
            async_copy_16B(kbase, lr * krs2 + chunk, smem + kKvK + blk * 1024);
            async_copy_16B(vbase, lr * vrs2 + chunk, smem + kKvV + blk * 1024);
        }
    }
    // B-operand row 32*kb + col (my key) of the K tile, chunk 2s + half; V tile: + kKvV - kKvK.  The
    // swizzle XORs the chunk index, so chunk 2s + half sits at (offset of chunk `half`) ^ 32s.
    const int boff0 = kKvK + rowmajor128_off(32 * kb + col, half);

    // query tiles that can see this key tile
    const int kl0 = key0 - k_lo;  // local index of the tile's first key (depth-0 tiles: its position)
    int t1_begin = 0, nt1 = 0;
    if (!second && lq1 > 0) {
        // first depth-0 query row with position >= kl0 (additive-mask mode: every row, the mask decides)
        const int first_q = (kl0 - off > 0 && !kDense) ? kl0 - off : 0;
        t1_begin = first_q / kBQ;
        nt1 = (lq1 + kBQ - 1) / kBQ - t1_begin;
        if (nt1 < 0) nt1 = 0;
    }
    // Depth-1 query tiles: rows of a sequence come in ascending position, so the tiles that can see a depth-0
    // key tile are a suffix -- those whose last row has a position >= the tile's first key.  One lane per tile
    // looks its last row up; every wave does the same and gets the same answer.
    int t2_begin = 0;
    const int nt2_all = (lq2 + kBQ - 1) / kBQ;
    if (!second && !kDense && nt2_all > 0) {
        t2_begin = nt2_all;
        for (int t0 = 0; t0 < nt2_all; t0 += kWave) {
            const int t = t0 + lane;
            const int last = q2_lo + (t * kBQ + kBQ - 1 < lq2 - 1 ? t * kBQ + kBQ - 1 : lq2 - 1);
            const bool sees = t < nt2_all && p.s2.pos_q[last] >= kl0;
            const unsigned long long m = __builtin_amdgcn_ballot_w64(sees);
            if (m) { t2_begin = t0 + __builtin_ctzll(m); break; }
        }
    }
    const int q2_first = q2_lo + t2_begin * kBQ;  // first depth-1 query row staged by this workgroup
    const int nt2 = nt2_all - t2_begin;
    const int nitems = (nt1 + nt2) * G;
    // Depth-0 query tiles [t_vis, t_whole) (relative to t1_begin) need no mask for this wave: all 64 rows
    // exist and the first row of my half already sees the last key of my block.
    int t_whole = lq1 / kBQ - t1_begin;
    t_whole = t_whole < 0 ? 0 : (t_whole < nt1 ? t_whole : nt1);
    int t_vis = 0;
    if (!second) {
        const int need = kl0 + 32 * kb + 31 - off - 32 * qh;  // first query row that sees my last key
        t_vis = need > 0 ? (need + kBQ - 1) / kBQ - t1_begin : 0;
        t_vis = t_vis < 0 ? 0 : t_vis;
    }
    t_vis = t_vis < t_whole ? t_vis : t_whole;
    if constexpr (kDense) t_whole = t_vis = 0;  // the mask is read for every item

    f32x16 dkacc[4], dvacc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dkacc[i][r] = 0.f; dvacc[i][r] = 0.f; }
    const float c = p.scale_log2e;

    // dS exchange: my two 16-byte pieces inside the wave's 2 KiB of an item's block, and the block of item 0 of
    // each query stream (blocks of successive query tiles are hq * ds_kt blocks apart, heads ds_kt)
    [[maybe_unused]] const int ds_lane_off = ds_piece_off(0, col, half);
    [[maybe_unused]] int64_t ds_base1 = 0, ds_base2 = 0;
    if constexpr (kExport) {
        const int ktile = (second ? p.ds_kt1 : 0) + kl0 / kBK;
        const int slot1 = q1_lo / kBQ + seq + t1_begin;
        const int slot2 = p.ds_q1slots + q2_lo / kBQ + seq + t2_begin;
        ds_base1 = (((int64_t)slot1 * p.hq + hk * G) * p.ds_kt + ktile) * kDsBlockBytes + wave * kDsWaveBytes;
        ds_base2 = (((int64_t)slot2 * p.hq + hk * G) * p.ds_kt + ktile) * kDsBlockBytes + wave * kDsWaveBytes;
    }
    // An item's dS leaves at the start of the next item: a store issued where dS is complete would still be on its
    // way at the barrier that ends the item, whose wait for the staged tiles (vmcnt) counts stores as well.
    [[maybe_unused]] bf16x8 ds_keep[2] = {};

    // item = (query tile, query head): rows [r0, r_end) of stream q2s, head `head`
    auto item_rows = [&](int item, bool& q2s, int& r0, int& r_end, int& head) {
        const int t = item / G;
        head = hk * G + item % G;
        q2s = t >= nt1;
        if (!q2s) {
            r0 = q1_lo + (t1_begin + t) * kBQ;
            r_end = q1_lo + lq1;
        } else {
            r0 = q2_first + (t - nt1) * kBQ;
            r_end = q2_lo + lq2;
        }
        r_end = r0 + kBQ < r_end ? r0 + kBQ : r_end;
    };
    // Asynchronous global -> LDS copy of one item: Q and dO tiles (16 blocks of 4 rows each, two per
    // wave), then lse / delta / positions as one dword per lane (waves 0, 1, 2).  Sources are
    // (wave-uniform base of the tile) + (per-lane byte offset); rows past the end repeat the last one.
    const int my_lrow = 8 * wave + (lane >> 4);  // second piece: 4 rows further down
    const uint32_t my_chunk0 = (uint32_t)(((lane & 15) ^ row_swizzle(my_lrow)) * 16);
    const uint32_t my_chunk1 = (uint32_t)(((lane & 15) ^ row_swizzle(my_lrow + 4)) * 16);
    // The query stream that staged items come from, held in scalar registers: its fields are read from
    // the kernel arguments once per stream, not once per item (each read is a scalar-memory round trip
    // that every wave would sit through right after the barrier).
    struct ItemSrc {
        const __bf16 *q, *g;
        const float *lse, *delta;  // lse: the log2-scaled copy behind the deltas
        const int32_t* pos;
        uint32_t qrs2, grs2;
        int64_t q_hs, g_hs;
        int32_t total_q, row_lo, row_end, tile0;
    };
    auto stream_src = [&](bool q2s) {
        const BwdStream& qs = q2s ? p.s2 : p.s1;
        ItemSrc r;
        r.q = qs.q; r.g = qs.d_o; r.lse = qs.delta + (int64_t)p.hq * qs.total_q; r.delta = qs.delta; r.pos = qs.pos_q;
        r.qrs2 = (uint32_t)(qs.q_rs * 2) & 0xffffffu;
        r.grs2 = (uint32_t)(qs.do_rs * 2) & 0xffffffu;
        r.q_hs = qs.q_hs; r.g_hs = qs.do_hs;
        r.total_q = qs.total_q;
        r.row_lo = q2s ? q2_first : q1_lo + t1_begin * kBQ;
        r.row_end = q2s ? q2_lo + lq2 : q1_lo + lq1;
        r.tile0 = q2s ? nt1 : 0;
        return r;
    };
    ItemSrc src = stream_src(nt1 == 0);
    auto issue_item = [&](int item, int buf) {
        const int t = item / G, head = hk * G + item % G;
        const bool q2s = src.tile0 != 0 || nt1 == 0;
        const int r0 = src.row_lo + (t - src.tile0) * kBQ;
        const int r_end = r0 + kBQ < src.row_end ? r0 + kBQ : src.row_end;
        auto* qt = smem + buf * kKvSlot;
        auto* gt = qt + kTileBytes;
        auto* meta = TAH_LDS_CAST(float, smem + kKvMeta + buf * kKvMetaBytes);
        const int last = r_end - 1 - r0;
        const uint32_t l0 = (uint32_t)(my_lrow < last ? my_lrow : last) & 63u;
        const uint32_t l1 = (uint32_t)(my_lrow + 4 < last ? my_lrow + 4 : last) & 63u;
        const __bf16* qbase = src.q + ((int64_t)r0 * (src.qrs2 >> 1) + (int64_t)head * src.q_hs);
        const __bf16* gbase = src.g + ((int64_t)r0 * (src.grs2 >> 1) + (int64_t)head * src.g_hs);
        async_copy_16B(qbase, l0 * src.qrs2 + my_chunk0, qt + (2 * wave) * 1024);
        async_copy_16B(gbase, l0 * src.grs2 + my_chunk0, gt + (2 * wave) * 1024);
        async_copy_16B(qbase, l1 * src.qrs2 + my_chunk1, qt + (2 * wave + 1) * 1024);
        async_copy_16B(gbase, l1 * src.grs2 + my_chunk1, gt + (2 * wave + 1) * 1024);
        const uint32_t lm = (uint32_t)(lane < last ? lane : last) * 4u;
        const int64_t hrow = (int64_t)head * src.total_q + r0;
        if (wave == 0) async_copy_4B(src.lse + hrow, lm, meta);
        if (wave == 1) async_copy_4B(src.delta + hrow, lm, meta + kBQ);
        if (wave == 2 && q2s) async_copy_4B(src.pos + r0, lm, meta + 2 * kBQ);
    };
    auto advance = [&](int item) {
        TAH_WAIT_VMEM();
        __syncthreads();
        if (item + 1 == nt1 * G) src = stream_src(true);  // the next item is the first of the depth-1 stream
    };
    // this wave's 2 KiB of an item's dS block (wave-uniform), and the store of the dS kept from that item
    // Items follow one another head by head, tile by tile: the block offsets of the current and the previous item are
    // carried along (two additions per item) instead of being formed from the item number (64-bit multiplies).
    [[maybe_unused]] const int64_t ds_head_step = (int64_t)p.ds_kt * kDsBlockBytes;
    [[maybe_unused]] const int64_t ds_tile_step = (int64_t)(p.hq - (G - 1)) * p.ds_kt * kDsBlockBytes;  // last head of a tile -> first of the next
    [[maybe_unused]] int64_t ds_cur = nt1 > 0 ? ds_base1 : ds_base2, ds_prev = 0;
    [[maybe_unused]] auto ds_advance = [&](int item) __attribute__((always_inline)) {  // from `item` to `item + 1`
        ds_prev = ds_cur;
        ds_cur += (item + 1) % G != 0 ? ds_head_step : ds_tile_step;
        if (item + 1 == nt1 * G) ds_cur = ds_base2;
    };
    [[maybe_unused]] auto ds_store = [&]() __attribute__((always_inline)) {
        unsigned char* dst = p.ds_ws + ds_prev;
        // (streaming stores: 1 GB of dS per call should not push the Q / dO / K / V tiles out of the L2)
        __builtin_nontemporal_store(ds_keep[0], reinterpret_cast<bf16x8*>(dst + ds_lane_off));
        __builtin_nontemporal_store(ds_keep[1], reinterpret_cast<bf16x8*>(dst + ds_lane_off + 128));
    };

    // per-lane LDS read offsets inside a tile, computed once
    const int aoff0 = rowmajor128_off(32 * qh + col, half);  // A-operand rows 32*qh + col of the Q / dO tiles, chunk 2s + half: ^ 32s
    // transpose reads: rows 32*qh + 4*half + r/4 (+8), columns 32*dt + 16*grp + 4*(r%4); column block dt
    // sits at (offset of block 0) ^ 64dt
    int toff_lo0, toff_hi0;
    {
        const int r16 = lane & 15, grp = (lane >> 4) & 1;
        const int trow = 32 * qh + 4 * half + (r16 >> 2);
        const int tcol = 16 * grp + 4 * (r16 & 3);
        toff_lo0 = rowmajor128_off(trow, tcol >> 3) + (tcol & 7) * 2;
        toff_hi0 = rowmajor128_off(trow + 8, tcol >> 3) + (tcol & 7) * 2;
    }
    const int mrow = 32 * qh + 4 * half;  // my accumulator rows: mrow + 8*(r/4) + r%4

    // One item = 32 MFMAs per wave (S 8, dP 8, dV 8, dK 8), written as 32 slots in program order with
    // scheduling fences between them so that the order below is the order in the binary: every slot
    // first issues the LDS reads of a later slot (two slots ahead for the S / dP operand pairs, three
    // for the transpose reads of dV / dK), then its MFMA, then a slice of the vector work -- P for two
    // query rows behind each dP MFMA, dS for two rows behind each dV MFMA -- so LDS latency and the
    // exp / convert arithmetic run in the shadow of the matrix pipe.
    auto body = [&](int item, auto mask_tag, auto stage_tag) __attribute__((always_inline)) {
        constexpr bool kMasked = decltype(mask_tag)::value;
        constexpr int kStage = decltype(stage_tag)::value;  // 0 / 1: stage known at compile time; -1: item & 1
        const int stage = kStage >= 0 ? kStage : (item & 1);
        const auto* qt = smem + stage * kKvSlot;
        const auto* gt = qt + kTileBytes;
        const auto* meta = TAH_LDS_CAST(const float, smem + kKvMeta + stage * kKvMetaBytes);

        [[maybe_unused]] bool q2s = false;
        [[maybe_unused]] int nvalid = kBQ, pos0 = 0;
        [[maybe_unused]] const auto* qposs = TAH_LDS_CAST(const int, meta) + 2 * kBQ;
        [[maybe_unused]] int dense_head = 0, dense_q0 = 0;
        if constexpr (kMasked) {
            int r0, r_end, head;
            item_rows(item, q2s, r0, r_end, head);
            nvalid = r_end - r0;        // rows of the tile that exist
            pos0 = (r0 - q1_lo) + off;  // depth-0 stream: position of tile row 0
            dense_head = head;
            dense_q0 = r0 - q1_lo;      // additive-mask mode: query index of tile row 0
        }

        bf16x8 ra[3], rb[3], rt[4];  // operand rings
        f32x4 lse4[2], del4[2];      // log-sum-exp / delta of four consecutive rows, two sets in flight
        f32x16 sacc, dpacc;
        bf16x8 pfr[2], dsfr[2];
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

        // operands of slot n < 16: rows of the Q (S) or dO (dP) tile, my key's row of the K or V tile
        // (their addresses are one XOR away from two base registers: cheaper than sixteen registers
        // that stay live through the loop)
        int abase = aoff0, bbase = boff0, tlo = toff_lo0, thi = toff_hi0;
        TAH_OPAQUE2(abase, bbase);
        TAH_OPAQUE2(tlo, thi);
        // (likewise the sixteen row numbers and position addresses of the masked variants)
        [[maybe_unused]] int mrow_m = mrow, kpos_m = kpos;
        if constexpr (kMasked) TAH_OPAQUE2(mrow_m, kpos_m);
        auto load_ab = [&](int n) __attribute__((always_inline)) {
            ra[n % 3] = *TAH_LDS_CAST(const bf16x8, (n < 8 ? qt : gt) + (abase ^ (32 * (n % 8))));
            rb[n % 3] = *TAH_LDS_CAST(const bf16x8, smem + (n < 8 ? 0 : kKvV - kKvK) + (bbase ^ (32 * (n % 8))));
        };
        // B operand of tail slot m: dO columns (dV, m < 8) or Q columns (dK) of my 32 query rows
        auto load_t = [&](int m) __attribute__((always_inline)) {
            const auto* t = m < 8 ? gt : qt;
            const int st = (m % 8) / 4, dt = m % 4;
            const bf16x4 lo = lds_read_tr16(t + (tlo ^ (64 * dt)) + st * 4096);
            const bf16x4 hi = lds_read_tr16(t + (thi ^ (64 * dt)) + st * 4096);
            rt[m % 4] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        };
        // P for accumulator rows r, r + 1 (r even) from S and the saved log-sum-exp
        auto p_rows = [&](int r) __attribute__((always_inline)) {
            float pr[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int rr = r + u, j = rr / 4, b4 = rr % 4;
                const float lse = lse4[j % 2][b4];
                pr[u] = fast_exp2(sacc[rr] * c - lse);
                if constexpr (kMasked && !kDense) {
                    const int qr = mrow_m + 8 * j + b4;
                    const int qp = q2s ? qposs[qr] : pos0 + qr;
                    pr[u] = (qr < nvalid && kpos_m <= qp) ? pr[u] : 0.f;
                }
                if constexpr (kDense) {  // mask[seq][head][query][my key]
                    const int qr = mrow_m + 8 * j + b4;
                    const bool ok = qr < nvalid && key_ok;
                    const int64_t e = (int64_t)seq * p.mask_sb + (int64_t)dense_head * p.mask_sh +
                                      (int64_t)(ok ? dense_q0 + qr : 0) * p.mask_sq;
                    const float mv = mask_value(p, static_cast<const unsigned char*>(p.mask) + e * (p.mask_f32 ? 4 : 2),
                                                ok ? kl0 + 32 * kb + col : 0);
                    const float lse_row = lse == kNegInf ? -kNegInf : lse;  // all keys hidden: P = 0
                    pr[u] = ok ? fast_exp2((sacc[rr] + mv * p.inv_scale) * c - lse_row) : 0.f;
                }
            }
            const f32x2 pr2 = {pr[0], pr[1]};
            const bf16x2 pk = __builtin_convertvector(pr2, bf16x2);
            pfr[r / 8][r % 8] = pk[0];
            pfr[r / 8][r % 8 + 1] = pk[1];
        };
        // dS = P o (dP - delta) for rows r, r + 1, from the bf16 P that the dV product uses
        auto ds_rows = [&](int r) __attribute__((always_inline)) {
            const int j = r / 4, b4 = r % 4;
            const f32x2 ds2 = {(float)pfr[r / 8][r % 8] * (dpacc[r] - del4[j % 2][b4]),
                               (float)pfr[r / 8][r % 8 + 1] * (dpacc[r + 1] - del4[j % 2][b4 + 1])};
            const bf16x2 pk = __builtin_convertvector(ds2, bf16x2);
            dsfr[r / 8][r % 8] = pk[0];
            dsfr[r / 8][r % 8 + 1] = pk[1];
        };
        auto load_lse = [&](int j) __attribute__((always_inline)) {
            lse4[j % 2] = *TAH_LDS_CAST(const f32x4, meta + mrow + 8 * j);
        };
        auto load_del = [&](int j) __attribute__((always_inline)) {
            del4[j % 2] = *TAH_LDS_CAST(const f32x4, meta + kBQ + mrow + 8 * j);
        };

        load_ab(0);
        load_ab(1);
#pragma unroll
        for (int n = 0; n < 32; ++n) {
            // reads for later slots
            if (n + 2 < 16) load_ab(n + 2);
            if (n + 3 >= 16 && n + 3 < 32) load_t(n + 3 - 16);
            if (n >= 7 && n < 15 && (n - 7) % 2 == 0) load_lse((n - 7) / 2);   // rows 4j.. are used from slot 8 + 2j on
            if (n >= 15 && n < 23 && (n - 15) % 2 == 0) load_del((n - 15) / 2);
            __builtin_amdgcn_sched_barrier(0);
            // The copies of the next item (its stage is free since the barrier): a copy instruction holds
            // a wave's issue for about 80 clocks, so the two waves of a SIMD send theirs half an item apart
            // and each does it while the other has MFMAs to issue.
            if ((n == 2 && qh == 0) || (n == 18 && qh == 1)) {
                if (item + 1 < nitems) issue_item(item + 1, stage ^ 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (n < 8) {
                sacc = mfma32(ra[n % 3], rb[n % 3], n == 0 ? zero : sacc);
            } else if (n < 16) {
                dpacc = mfma32(ra[n % 3], rb[n % 3], n == 8 ? zero : dpacc);
                p_rows(2 * (n - 8));
            } else if (n < 24) {
                // dV (32 keys x 128 d) += P^T dO: needs P only, so the dS slices ride behind it
                dvacc[n % 4] = mfma32(pfr[(n - 16) / 4], rt[n % 4], dvacc[n % 4]);
                ds_rows(2 * (n - 16));
            } else {
                // dK += dS^T Q (contraction over my 32 queries)
                dkacc[n % 4] = mfma32(dsfr[(n - 24) / 4], rt[n % 4], dkacc[n % 4]);
            }
            if constexpr (kExport) {
                if (n == 0 && item > 0) ds_store();  // the previous item's dS (before this item's copies are issued)
                if (n == 31) { ds_keep[0] = dsfr[0]; ds_keep[1] = dsfr[1]; ds_advance(item); }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    using Masked = std::true_type;
    using Plain = std::false_type;
    using Stage0 = std::integral_constant<int, 0>;
    using Stage1 = std::integral_constant<int, 1>;
    using StageAny = std::integral_constant<int, -1>;

    if (nitems > 0) issue_item(0, 0);  // (the first barrier below also publishes the K and V tiles)
    // The three ranges start and end at multiples of G, so with an even G the stage of an item is
    // its parity inside the pair and the LDS offsets of both stages are compile-time constants.
    auto run = [&](int from, int to, auto mask_tag) __attribute__((always_inline)) {
        if constexpr (G % 2 == 0) {
            for (int item = from; item < to; item += 2) {
                advance(item);
                body(item, mask_tag, Stage0{});
                advance(item + 1);
                body(item + 1, mask_tag, Stage1{});
            }
        } else {
            for (int item = from; item < to; ++item) {
                advance(item);
                body(item, mask_tag, StageAny{});
            }
        }
    };
    run(0, t_vis * G, Masked{});
    run(t_vis * G, t_whole * G, Plain{});
    run(t_whole * G, nitems, Masked{});

    if constexpr (kExport) {
        if (nitems > 0) ds_store();
    }
    // ---- add the two query halves and store ---------------------------------
    TAH_WAIT_VMEM();  // no copy may still be on its way into the memory the reduction reuses
    __syncthreads();
    auto* red = TAH_LDS_CAST(float, smem);  // [key block][128 regs][64 lanes]
    if (qh == 1) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                red[(kb * 128 + dt * 16 + r) * 64 + lane] = dkacc[dt][r];
                red[(kb * 128 + 64 + dt * 16 + r) * 64 + lane] = dvacc[dt][r];
            }
    }
    __syncthreads();
    if (qh == 0) {
        // accumulator (dt, reg r, lane): key = 32*kb + acc_row(half, r), d = 32*dt + col
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int krow = key0 + 32 * kb + acc_row(half, r);
                const float dkv = (dkacc[dt][r] + red[(kb * 128 + dt * 16 + r) * 64 + lane]) * p.scale;
                const float dvv = dvacc[dt][r] + red[(kb * 128 + 64 + dt * 16 + r) * 64 + lane];
                if (krow < key_end) {
                    ks.dk[(int64_t)krow * ks.dk_rs + (int64_t)hk * ks.dk_hs + 32 * dt + col] = (__bf16)dkv;
                    ks.dv[(int64_t)krow * ks.dv_rs + (int64_t)hk * ks.dv_hs + 32 * dt + col] = (__bf16)dvv;
                }
            }
    }
}

// ---------------------------------------------------------------------------
// dQ from the exchanged dS: dQ = scale * dS K, one product per (query tile, key tile) pair
// ---------------------------------------------------------------------------
// One workgroup = the query tile of the forward / dQ kernels (256 / G rows, the G heads of one kv head), i.e.
// four units of (64 query rows, one head); waves 2u and 2u + 1 own unit u and split the head dimension.
// Per step of 64 keys the workgroup stages the K rows (row-major, swizzled, as everywhere) and every unit's
// 8 KiB of dS in LDS with asynchronous copies, three steps deep (the kernel streams dS from HBM and does one
// MFMA per 512 bytes of it, so what matters is the number of bytes on their way); a wave then forms
// dQ[64 rows x 64 d] += dS[64 x 64 keys] K[64 keys x 64 d] from transpose reads of both (dS lies key-major,
// K row-major, and both operands want the keys along a lane's registers): 16 MFMAs.
constexpr int kLqThreads = 512;
constexpr int kLqUnits = 4;
constexpr int kLqStageDs = kLqUnits * 8192;            // per unit: 64 rows x 64 keys of dS
constexpr int kLqStage = kTileBytes + kLqStageDs;      // K rows of the step + dS
constexpr int kLqStages = 3;
constexpr int kLqSmem = kLqStages * kLqStage;
constexpr int kLqCopies = 6;                           // asynchronous copies per wave and step

template <int G>
__global__ __launch_bounds__(kLqThreads) TAH_WAVES_PER_EU(2, 2) void duo_bwd_dq_from_ds_kernel(const BwdParams p) {
    static_assert(G == 1 || G == 2 || G == 4, "four (64-row tile, head) units per workgroup");
    constexpr int BM = 32 * (8 / G);
    HIP_DYNAMIC_SHARED(unsigned char, smem_array)
    TAH_LDS_ZERO_BASED(smem, smem_array);
    const int tid = threadIdx.x, lane = tid % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int half = lane / 32, col = lane % 32;
    const int hk = blockIdx.x;

    int seq = 0, row0 = 0, row_end = 0;
    bool second = false;
    int slot = (int)(gridDim.y - 1 - blockIdx.y);  // without a table: late (heavy) tiles of each sequence first
    // (the table's order: heaviest tile of the whole call first)
    sched_lookup(p.sched, false, p.nseq, G, p.s1.total_q, p.s2.total_q, p.s1.total_k, p.s2.total_k, (int)gridDim.y,
                 (int)blockIdx.y, slot);
    if (!(p.s1.total_q > 0 && find_tile(p.s1.cu_q, p.nseq, BM, slot, seq, row0, row_end))) {
        if (!(p.s2.total_q > 0 && find_tile(p.s2.cu_q, p.nseq, BM, slot, seq, row0, row_end))) return;
        second = true;
    }
    const BwdStream& qs = second ? p.s2 : p.s1;
    const int q_lo = const_i32(qs.cu_q, seq);
    const int k1_lo = const_i32(p.s1.cu_k, seq);
    const int lk1 = const_i32(p.s1.cu_k, seq + 1) - k1_lo;
    const int lq1 = p.s1.total_q > 0 ? const_i32(p.s1.cu_q, seq + 1) - const_i32(p.s1.cu_q, seq) : 0;
    const int off = lk1 - lq1;  // position of depth-0 query row i of the sequence is i + off
    const __bf16* k1p = p.s1.k + (int64_t)k1_lo * p.s1.k_rs + (int64_t)hk * p.s1.k_hs;
    const int left1 = p.s1.total_k - k1_lo;
    int lk2 = 0, left2 = 0;
    const __bf16* k2p = nullptr;
    if (second) {
        const int k2_lo = const_i32(p.s2.cu_k, seq);
        lk2 = const_i32(p.s2.cu_k, seq + 1) - k2_lo;
        k2p = p.s2.k + (int64_t)k2_lo * p.s2.k_rs + (int64_t)hk * p.s2.k_hs;
        left2 = p.s2.total_k - k2_lo;
    }

    // my unit: 64-row tile `tile` of the sequence's query rows (all wave-uniform)
    const int unit = wave / 2, dh = wave % 2;
    const int utile = unit / G, uhead = hk * G + unit % G;
    const int tile0 = (row0 - q_lo) / kBN;                 // first 64-row tile of the workgroup
    const int ntiles_wg = (row_end - row0 + kBN - 1) / kBN;  // tiles of the workgroup that exist (>= 1)
    const bool unit_ok = utile < ntiles_wg;
    // 64-key steps that hold a key visible to some row of 64-row tile t (depth-0 rows see positions <= row + off)
    // (the position of depth-1 row: pos_q, ascending inside a sequence, so a tile's last row has its largest)
    const int q_end = const_i32(qs.cu_q, seq + 1);
    auto steps_of = [&](int t) {
        int reach = 64 * t + 63 + off;  // largest position a row of the tile has
        if (second) {
            const int r = q_lo + 64 * t + 63;
            reach = const_i32(qs.pos_q, r < q_end - 1 ? r : q_end - 1);
        }
        const int last = reach < lk1 - 1 ? reach : lk1 - 1;
        return last >= 0 ? last / kBN + 1 : 0;
    };
    const int my_n1 = __builtin_amdgcn_readfirstlane(unit_ok ? steps_of(tile0 + utile) : 0);
    const int n1 = __builtin_amdgcn_readfirstlane(steps_of(tile0 + ntiles_wg - 1));  // the workgroup's last tile sees the most
    const int n2 = second ? (lk2 + kBN - 1) / kBN : 0;
    const int nsteps = n1 + n2;

    // where my unit's blocks start: (qslot, head), key tile 0.  A unit without a tile copies the first unit's
    // blocks (memory that exists; never used).
    const int qslot = (second ? p.ds_q1slots : 0) + q_lo / kBN + seq + tile0 + (unit_ok ? utile : 0);
    const unsigned char* ds_unit = p.ds_ws + (int64_t)(qslot * p.hq + uhead) * p.ds_kt * kDsBlockBytes;

    // asynchronous copies of one step: K rows as in the dQ kernel (4 rows per copy, two copies per wave), then four
    // 1 KiB pieces of my unit's dS: piece pi = 4 * dh + j covers the key-tile kernel's wave (pi / 4, 2 * hh + (pi % 4) / 2)
    const int my_lrow = 8 * wave + (lane >> 4);
    const uint32_t my_chunk0 = (uint32_t)(((lane & 15) ^ row_swizzle(my_lrow)) * 16);
    const uint32_t my_chunk1 = (uint32_t)(((lane & 15) ^ row_swizzle(my_lrow + 4)) * 16);
    auto issue_step = [&](int s, int stage) {
        const bool s0 = s < n1;
        const int ks = s0 ? s : s - n1;  // 64-key step inside its segment
        const int64_t krs = s0 ? p.s1.k_rs : p.s2.k_rs;
        const __bf16* kt0 = (s0 ? k1p : k2p) + (int64_t)ks * kBN * krs;
        const int last = (s0 ? left1 : left2) - 1 - ks * kBN;
        auto* kt = smem + stage * kLqStage;
        const uint32_t r0 = (uint32_t)(my_lrow < last ? my_lrow : last) & 63u;
        const uint32_t r1 = (uint32_t)(my_lrow + 4 < last ? my_lrow + 4 : last) & 63u;
        const uint32_t krs2 = (uint32_t)(krs * 2) & 0xffffffu;
        async_copy_16B(kt0, r0 * krs2 + my_chunk0, kt + (2 * wave) * 1024);
        async_copy_16B(kt0, r1 * krs2 + my_chunk1, kt + (2 * wave + 1) * 1024);
        const int ktile = (s0 ? 0 : p.ds_kt1) + ks / 2, hh = ks % 2;
        const unsigned char* blk = ds_unit + (int64_t)ktile * kDsBlockBytes;
        auto* dst = kt + kTileBytes + unit * 8192 + dh * 4096;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // piece pi = 4 * dh + j: query half pi / 4 = dh, key block 2 * hh + j / 2, KiB j % 2 of that wave's 2 KiB
            const uint32_t src = (uint32_t)((4 * dh + 2 * hh + j / 2) * kDsWaveBytes + (j % 2) * 1024 + lane * 16);
            async_copy_16B_stream(blk, src, dst + j * 1024);
        }
    };

    // per-lane LDS read offsets
    // dS operand (A: rows = my 32 query rows of block qb, 8 keys 16*ks4 + 8*half + 0..7): two transpose reads;
    // lane f of a 16-lane group points at the four rows 16*a2 + 4*(f%4) + 0..3 of key k0 + f/4
    const int f16 = lane & 15, a2 = (lane >> 4) & 1;
    const int ds_lane = ds_piece_off(a2, 8 * half + (f16 >> 2), f16 & 1) + 8 * ((f16 >> 1) & 1);
    // K operand (B: columns = d, same 8 keys): rows 16*ks4 + 8*half + f/4 (+4), columns 64*dh + 32*dt + 16*a2 + 4*(f%4)
    int k_lane[2][2];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int r = 8 * half + 4 * u + (f16 >> 2), cc = 64 * dh + 32 * dt + 16 * a2 + 4 * (f16 & 3);
            k_lane[dt][u] = rowmajor128_off(r, cc >> 3) + (cc & 7) * 2;
        }

    f32x16 acc[2][2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[qb][dt][r] = 0.f;

    auto compute = [&](int stage) __attribute__((always_inline)) {
        const auto* kt = smem + stage * kLqStage;
        const auto* ds = kt + kTileBytes + unit * 8192;
#pragma unroll
        for (int ks4 = 0; ks4 < 4; ++ks4) {
            bf16x8 a[2], b[2];
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                // query half qb, key block ks4 / 2 of the step: the copied piece layout is [qb][key block][2 KiB]
                const auto* w = ds + qb * 4096 + (ks4 / 2) * 2048 + (ks4 % 2) * 1024 + ds_lane;
                const bf16x4 lo = lds_read_tr16(w), hi = lds_read_tr16(w + 256);
                a[qb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int dt = 0; dt < 2; ++dt) {
                const bf16x4 lo = lds_read_tr16(kt + k_lane[dt][0] + ks4 * 4096), hi = lds_read_tr16(kt + k_lane[dt][1] + ks4 * 4096);
                b[dt] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int dt = 0; dt < 2; ++dt) acc[qb][dt] = mfma32(a[qb], b[dt], acc[qb][dt]);
        }
    };

    if (nsteps > 0) issue_step(0, 0);
    if (nsteps > 1) issue_step(1, 1);
    int stage = 0;
    for (int s = 0; s < nsteps; ++s) {
        // the copies of step s are in; those of step s + 1 (the last kLqCopies this wave issued) may still be on their way
        if (s + 1 < nsteps) TAH_WAIT_VMEM_N(kLqCopies); else TAH_WAIT_VMEM();
        __syncthreads();
        if (s + 2 < nsteps) issue_step(s + 2, stage == 0 ? 2 : stage - 1);
        if (s >= n1 ? unit_ok : s < my_n1) compute(stage);
        stage = stage == 2 ? 0 : stage + 1;
    }

    if (unit_ok) {
        // accumulator (qb, dt, reg r, lane): row 32*qb + acc_row(half, r) of my tile, d = 64*dh + 32*dt + col
        const int trow0 = row0 + utile * kBN;
        const int tend = q_end;
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = trow0 + 32 * qb + acc_row(half, r);
                if (row < tend) {
                    __bf16* drow = qs.dq + (int64_t)row * qs.dq_rs + (int64_t)uhead * qs.dq_hs + 64 * dh + col;
                    drow[0] = (__bf16)(acc[qb][0][r] * p.scale);
                    drow[32] = (__bf16)(acc[qb][1][r] * p.scale);
                }
            }
    }
}

BwdStream to_dev(const tah_duo_stream& s, const tah_duo_bwd_stream& g) {
    BwdStream d;
    d.q = static_cast<const __bf16*>(s.q);
    d.k = static_cast<const __bf16*>(s.k);
    d.v = static_cast<const __bf16*>(s.v);
    d.o = static_cast<const __bf16*>(s.o);
    d.d_o = static_cast<const __bf16*>(g.d_o);
    d.dq = static_cast<__bf16*>(g.dq);
    d.dk = static_cast<__bf16*>(g.dk);
    d.dv = static_cast<__bf16*>(g.dv);
    d.lse = s.lse;
    d.delta = g.delta;
    d.cu_q = s.cu_q; d.cu_k = s.cu_k; d.pos_q = s.pos_q; d.pos_k = s.pos_k;
    d.q_rs = s.q_row_stride; d.q_hs = s.q_head_stride;
    d.k_rs = s.k_row_stride; d.k_hs = s.k_head_stride;
    d.v_rs = s.v_row_stride; d.v_hs = s.v_head_stride;
    d.o_rs = s.o_row_stride; d.o_hs = s.o_head_stride;
    d.do_rs = g.do_row_stride; d.do_hs = g.do_head_stride;
    d.dq_rs = g.dq_row_stride; d.dq_hs = g.dq_head_stride;
    d.dk_rs = g.dk_row_stride; d.dk_hs = g.dk_head_stride;
    d.dv_rs = g.dv_row_stride; d.dv_hs = g.dv_head_stride;
    d.total_q = s.total_q;
    d.total_k = s.total_k;
    return d;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_bwd_stream(const tah_duo_stream& s, const tah_duo_bwd_stream& g, bool second) {
    if (s.total_q < 0 || s.total_k < 0) return TAH_E_SHAPE;
    if (!s.cu_q || !s.cu_k) return TAH_E_NULL;
    if (s.total_q > 0) {
        if (!s.q || !s.o || !s.lse || !g.d_o || !g.dq || !g.delta) return TAH_E_NULL;
        if (second && !s.pos_q) return TAH_E_NULL;
        if (!aligned16(s.q) || !aligned16(s.o) || !aligned16(g.d_o) || !aligned16(g.dq)) return TAH_E_ALIGN;
    }
    if (s.total_k > 0) {
        if (!s.k || !s.v || !g.dk || !g.dv) return TAH_E_NULL;
        if (second && !s.pos_k) return TAH_E_NULL;
        if (!aligned16(s.k) || !aligned16(s.v)) return TAH_E_ALIGN;
    }
    const int64_t st[] = {s.q_row_stride, s.q_head_stride, s.k_row_stride, s.k_head_stride, s.v_row_stride, s.v_head_stride,
                          s.o_row_stride, s.o_head_stride, g.do_row_stride, g.do_head_stride, g.dq_row_stride, g.dq_head_stride};
    for (int64_t x : st)
        if (x % 8 != 0) return TAH_E_ALIGN;
    // the tile copies address rows as base + row * stride with a 24-bit multiply
    for (int64_t x : {s.q_row_stride, s.k_row_stride, s.v_row_stride, g.do_row_stride})
        if (x < 0 || x >= (1 << 23)) return TAH_E_SHAPE;
    return TAH_OK;
}

template <int G, bool kDense>
int launch_bwd(const BwdParams& p, hipStream_t st) {
    constexpr int BM = 32 * (8 / G);
    for (const BwdStream* s : {&p.s1, &p.s2}) {
        if (s->total_q == 0) continue;
        const int64_t items = (int64_t)s->total_q * p.hq;
        hipLaunchKernelGGL(duo_bwd_delta_kernel, dim3((unsigned)((items + 15) / 16)), dim3(256), 0, st, *s, p.hq);
    }
    int qtiles = 0, ktiles = 0;
    if (p.s1.total_q > 0) qtiles += p.s1.total_q / BM + p.nseq;
    if (p.s2.total_q > 0) qtiles += p.s2.total_q / BM + p.nseq;
    if (p.s1.total_k > 0) ktiles += p.s1.total_k / kBK + p.nseq;
    if (p.s2.total_k > 0) ktiles += p.s2.total_k / kBK + p.nseq;
    if constexpr (!kDense && G <= 4) {
        if (p.ds_ws) {  // dS exchange: the key-tile kernel writes dS, dQ is one product that reads it back
            if (ktiles > 0) {
                if (hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_bwd_dkdv_kernel<G, false, true>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, kKvSmem) != hipSuccess)
                    return TAH_E_LAUNCH;
                hipLaunchKernelGGL((duo_bwd_dkdv_kernel<G, false, true>), dim3(p.hkv, ktiles), dim3(kKvThreads), kKvSmem, st, p);
            }
            if (qtiles > 0) {
                if (hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_bwd_dq_from_ds_kernel<G>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, kLqSmem) != hipSuccess)
                    return TAH_E_LAUNCH;
                hipLaunchKernelGGL((duo_bwd_dq_from_ds_kernel<G>), dim3(p.hkv, qtiles), dim3(kLqThreads), kLqSmem, st, p);
            }
            return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
        }
    }
    if (qtiles > 0) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_bwd_dq_kernel<G, kDense>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kDqSmem) != hipSuccess)
            return TAH_E_LAUNCH;
        hipLaunchKernelGGL((duo_bwd_dq_kernel<G, kDense>), dim3(p.hkv, qtiles), dim3(kDqThreads), kDqSmem, st, p);
    }
    if (ktiles > 0) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_bwd_dkdv_kernel<G, kDense, false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kKvSmem) != hipSuccess)
            return TAH_E_LAUNCH;
        hipLaunchKernelGGL((duo_bwd_dkdv_kernel<G, kDense, false>), dim3(p.hkv, ktiles), dim3(kKvThreads), kKvSmem, st, p);
    }
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

}  // namespace
}  // namespace tah

namespace tah {
namespace {
template <bool kDense>
int dispatch_bwd(const tah_duo_bwd_args* a, const tah_additive_mask* m, tah_stream_t stream) {
    if (!a) return TAH_E_NULL;
    const tah_duo_fwd_args& f = a->fwd;
    if (f.d != kD || f.nseq < 0 || f.hq <= 0 || f.hkv <= 0 || f.hq % f.hkv != 0) return TAH_E_SHAPE;
    const int g = f.hq / f.hkv;
    if (g != 1 && g != 2 && g != 4 && g != 8) return TAH_E_SHAPE;
    if (kDense) {
        if (!m || !m->mask) return TAH_E_NULL;
        if (f.s2.total_q != 0 || f.s2.total_k != 0 || (m->dtype != 0 && m->dtype != 1) || f.scale == 0.f) return TAH_E_SHAPE;
    }
    if (f.nseq == 0) return TAH_OK;
    if (int rc = check_bwd_stream(f.s1, a->g1, false)) return rc;
    if (int rc = check_bwd_stream(f.s2, a->g2, true)) return rc;
    BwdParams p;
    p.s1 = to_dev(f.s1, a->g1);
    p.s2 = to_dev(f.s2, a->g2);
    p.nseq = f.nseq;
    p.hq = f.hq;
    p.hkv = f.hkv;
    p.scale = f.scale;
    p.scale_log2e = f.scale * kLog2e;
    p.sched = kDense ? nullptr : static_cast<const int32_t*>(f.schedule);
    p.ds_ws = nullptr;
    p.ds_q1slots = p.ds_kt1 = p.ds_kt = 0;
    if (!kDense && a->ds_workspace && g <= 4) {
        if (reinterpret_cast<uintptr_t>(a->ds_workspace) & 15) return TAH_E_ALIGN;
        const size_t need = tah_duo_bwd_workspace_bytes(f.nseq, f.hq, f.hkv, f.s1.total_q, f.s1.total_k, f.s2.total_q, f.s2.total_k,
                                                        a->max_seqlen_k1, a->max_seqlen_k2);
        if (a->ds_workspace_bytes < need) return TAH_E_WORKSPACE;
        p.ds_ws = static_cast<unsigned char*>(a->ds_workspace);
        p.ds_q1slots = ds_query_slots(f.s1.total_q, f.nseq);
        p.ds_kt1 = ds_key_slots(f.s1.total_k, a->max_seqlen_k1);
        p.ds_kt = p.ds_kt1 + ds_key_slots(f.s2.total_k, a->max_seqlen_k2);
    }
    p.mask = nullptr;
    p.mask_sb = p.mask_sh = p.mask_sq = p.mask_sk = 0;
    p.mask_f32 = 0;
    p.inv_scale = 0.f;
    if (kDense) {
        p.mask = m->mask;
        p.mask_sb = m->seq_stride; p.mask_sh = m->head_stride; p.mask_sq = m->q_stride; p.mask_sk = m->k_stride;
        p.mask_f32 = m->dtype;
        p.inv_scale = 1.0f / f.scale;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (g) {
        case 1: return launch_bwd<1, kDense>(p, st);
        case 2: return launch_bwd<2, kDense>(p, st);
        case 4: return launch_bwd<4, kDense>(p, st);
        default: return launch_bwd<8, kDense>(p, st);
    }
}
}  // namespace
}  // namespace tah

extern "C" size_t tah_duo_bwd_workspace_bytes(int32_t nseq, int32_t hq, int32_t hkv, int32_t total_q1, int32_t total_k1,
                                              int32_t total_q2, int32_t total_k2, int32_t max_seqlen_k1, int32_t max_seqlen_k2) {
    if (nseq <= 0 || hq <= 0 || hkv <= 0 || hq % hkv != 0 || hq / hkv > 4) return 0;
    const size_t qslots = (size_t)tah::ds_query_slots(total_q1, nseq) + (size_t)tah::ds_query_slots(total_q2, nseq);
    const size_t kslots = (size_t)tah::ds_key_slots(total_k1, max_seqlen_k1) + (size_t)tah::ds_key_slots(total_k2, max_seqlen_k2);
    return qslots * (size_t)hq * kslots * (size_t)tah::kDsBlockBytes;
}

extern "C" int tah_duo_bwd_varlen(const tah_duo_bwd_args* a, tah_stream_t stream) {
    return tah::dispatch_bwd<false>(a, nullptr, stream);
}

extern "C" int tah_duo_bwd_masked(const tah_duo_bwd_args* a, const tah_additive_mask* m, tah_stream_t stream) {
    return tah::dispatch_bwd<true>(a, m, stream);
}
