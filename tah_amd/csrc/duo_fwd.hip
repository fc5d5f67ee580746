// Duo-causal attention forward (prefill / training), bf16 MFMA, gfx950.
//
// One workgroup = 8 waves = one query tile of one kv head: G = Hq/Hkv query
// heads x (256/G) query rows, wave w -> head (w % G), row block (w / G) of 32
// rows, so every K/V tile staged in LDS serves all query heads of the group.
// Per key tile of 64 keys each wave computes S^T = K Q^T (keys x queries) with
// v_mfma_f32_32x32x16_bf16, which leaves one query per lane column: the online
// softmax needs one cross-lane exchange per tile, and the bf16 probabilities
// are already in B-operand layout for O^T += V^T P^T.  K and V tiles are
// copied global -> LDS asynchronously (global_load_lds, no registers), sit
// row-major and swizzled there, and the V^T operand is read column-wise with
// ds_read_b64_tr_b16.
//
// Schedule.  A wave's work per key tile t is a vector phase X(t) (mask, online
// softmax, bf16 conversion, accumulator rescale: VALU only) and a matrix phase
// M(t) (O^T += V(t)^T P(t)^T, then S(t+1)^T = K(t+1) Q^T: MFMA + LDS reads
// only).  The two waves that share a SIMD are kept half a tile apart by the
// workgroup barriers -- while waves 0-3 run X(t), waves 4-7 run M(t-1), then
// they swap -- so the matrix pipe and the vector pipe of every SIMD are busy at
// the same time instead of taking turns.
//
// Key tiles come from the depth-0 segment (cut at the tile's largest query
// position) and, for depth-1 query tiles, from the depth-1 segment; the two-axis
// mask is evaluated per element only on tiles that straddle a query position
// (separate, mask-free instances of the vector phase handle the rest), and
// waves skip the arithmetic of tiles that lie entirely above their rows.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "duo_device.h"
#include "tah_duo.h"

namespace tah {
namespace {

constexpr int kMatrixPrio = 2;  // s_setprio of a wave while it runs its matrix phase
// Which of the two wave sets (early / late by half a tile) a wave belongs to.  Waves w and w+4 of a
// workgroup share a SIMD.
__device__ __forceinline__ int late_set(int wave) { return wave >> 2; }

constexpr int kD = 128;        // head_dim
constexpr int kBN = 64;        // keys per tile
constexpr int kThreads = 512;  // 8 waves (the 4-wave variant launches 256)
constexpr int kKBytes = kBN * kD * 2;         // 16 KiB, [key][d]
constexpr int kVBytes = kBN * kD * 2;         // 16 KiB, [key][d]
constexpr float kLazy = 8.f;                  // log2 units the row maximum may outgrow the exponent reference
constexpr int kStages = 2;                    // K ring and V ring depth
constexpr int kPosSlots = 4;                  // ring of depth-1 key positions (outlives its K tile by a phase)
constexpr int kKRing = 0;
constexpr int kVRing = kStages * kKBytes;
constexpr int kPosRing = kVRing + kStages * kVBytes;
constexpr int kBoundsOff = kPosRing + kPosSlots * kBN * 4;
constexpr int kStageOff = (kBoundsOff + 64 + 255) / 256 * 256;  // output staging: 8 KB per wave (32 rows x 256 B)
constexpr int kSmemBytes = kStageOff + 8 * 8192;
// The 4-wave variant (two workgroups per compute unit) stages its output over the K / V rings, which are dead by then.
constexpr int kSmemBytes4 = kStageOff;
static_assert(4 * 8192 <= kPosRing, "the 4-wave variant's output staging must fit the K / V rings");

struct FwdStream {
    const __bf16 *q, *k, *v;
    __bf16* o;
    float* lse;
    const int32_t *cu_q, *cu_k, *pos_q, *pos_k;
    int64_t q_rs, q_hs, k_rs, k_hs, v_rs, v_hs, o_rs, o_hs;
    int32_t total_q, total_k;
};
struct FwdParams {
    FwdStream s1, s2;
    int32_t nseq, hq, hkv;
    float scale_log2e;
    const int32_t* sched;  // launch-order table or nullptr
    // additive-mask mode only: mask[seq][head][query index][key index], strides in elements
    const void* mask;
    int64_t mask_sb, mask_sh, mask_sq, mask_sk;
    int32_t mask_f32;  // element type: 1 = float, 0 = bf16
    float inv_scale;   // 1 / scale: the mask is added to raw scores as mask / scale
};

enum class Mask { kNone, kIndex, kPos, kDense };

// kDense: additive-mask mode.  Every query attends to every key of its sequence and visibility comes
// from a dense additive mask (softmax(q k^T * scale + mask) v); only stream 1 is used.  A separate
// instantiation, so the duo-causal kernel carries none of it.
// W: waves per workgroup.  8: one workgroup per compute unit, two wave sets half a tile apart (above).  4: half the
// query tile per workgroup and two independent workgroups per compute unit -- every SIMD then holds one wave of each,
// the two drift freely against each other (the dispatcher starts them at different times and their tile counts
// differ), one workgroup's prologue, epilogue and hand-over to its successor run under the other's tile loop, and a
// workgroup needs one barrier per tile.  Each workgroup stages its own K / V tiles (twice the copies per MFMA).
template <int G, bool kDense, int W>
__global__ __launch_bounds__(64 * W) TAH_WAVES_PER_EU(2, 2) void duo_fwd_kernel(const FwdParams p) {
    static_assert(W == 8 || W == 4, "8 or 4 waves");
    static_assert(W >= G, "a workgroup holds every query head of its kv head");
    constexpr int BM = 32 * (W / G);
    constexpr int kRowsPerWave = kBN / W;       // rows of a K / V tile each wave copies
    constexpr int kPieces = kRowsPerWave / 4;   // in pieces of 4 rows (one copy instruction each)
    HIP_DYNAMIC_SHARED(unsigned char, smem)

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // wave-uniform: lives in a scalar register
    const int lane = tid % kWave;
    const int half = lane / 32;
    const int col = lane % 32;
    const int hk = blockIdx.x;

    // ---- which tile am I ---------------------------------------------------
    int seq = 0, row0 = 0, row_end = 0;
    bool second = false;
    // (the launch-order table lists tiles of 256 / G rows: a 4-wave workgroup takes one half of an entry)
    constexpr int kPerEntry = 8 / W;
    int slot;
    if (sched_lookup(p.sched, false, p.nseq, G, p.s1.total_q, p.s2.total_q, p.s1.total_k, p.s2.total_k,
                     (int)gridDim.y / kPerEntry, (int)blockIdx.y / kPerEntry, slot)) {
        // the table's order: heaviest tile of the whole call first; its tiles have kPerEntry * BM rows
        if (!(p.s1.total_q > 0 && find_tile(p.s1.cu_q, p.nseq, kPerEntry * BM, slot, seq, row0, row_end))) {
            if (!(p.s2.total_q > 0 && find_tile(p.s2.cu_q, p.nseq, kPerEntry * BM, slot, seq, row0, row_end))) return;
            second = true;
        }
        row0 += BM * ((int)blockIdx.y % kPerEntry);
        if (row0 >= row_end) return;
        row_end = row0 + BM < row_end ? row0 + BM : row_end;
    } else {
        slot = (int)(gridDim.y - 1 - blockIdx.y);  // late (heavy) tiles of each sequence first
        if (!(p.s1.total_q > 0 && find_tile(p.s1.cu_q, p.nseq, BM, slot, seq, row0, row_end))) {
            if (!(p.s2.total_q > 0 && find_tile(p.s2.cu_q, p.nseq, BM, slot, seq, row0, row_end))) return;
            second = true;
        }
    }
    const FwdStream& qs = second ? p.s2 : p.s1;

    const int head = hk * G + wave % G;
    const int rblk = wave / G;
    // depth-0 key segment of this sequence (position of a key = its local index)
    const int k1_lo = const_i32(p.s1.cu_k, seq);
    const int lk1 = const_i32(p.s1.cu_k, seq + 1) - k1_lo;
    const __bf16* k1p = p.s1.k + (int64_t)k1_lo * p.s1.k_rs + (int64_t)hk * p.s1.k_hs;
    const __bf16* v1p = p.s1.v + (int64_t)k1_lo * p.s1.v_rs + (int64_t)hk * p.s1.v_hs;
    const int left1 = p.s1.total_k - k1_lo;  // rows from the segment start to the end of the array
    // depth-1 key segment (explicit positions), only seen by depth-1 queries
    int lk2 = 0, left2 = 0;
    const __bf16 *k2p = nullptr, *v2p = nullptr;
    const int32_t* pos2p = nullptr;
    if (second) {
        const int k2_lo = const_i32(p.s2.cu_k, seq);
        lk2 = const_i32(p.s2.cu_k, seq + 1) - k2_lo;
        k2p = p.s2.k + (int64_t)k2_lo * p.s2.k_rs + (int64_t)hk * p.s2.k_hs;
        v2p = p.s2.v + (int64_t)k2_lo * p.s2.v_rs + (int64_t)hk * p.s2.v_hs;
        pos2p = p.s2.pos_k + k2_lo;
        left2 = p.s2.total_k - k2_lo;
    }

    // ---- my query row, its position, the tile's position bounds ------------
    const int row = row0 + rblk * 32 + col;
    const bool row_ok = row < row_end;
    const int row_ld = row_ok ? row : row_end - 1;  // tiles are never empty
    int qpos;
    if (second) {
        qpos = qs.pos_q[row_ld];
    } else {
        const int q_lo = const_i32(qs.cu_q, seq);
        qpos = (row_ld - q_lo) + (lk1 - (const_i32(qs.cu_q, seq + 1) - q_lo));
    }
    // last visible depth-0 key index (additive-mask mode: every key of the sequence, the mask decides)
    const int qlim1 = row_ok ? ((qpos < lk1 - 1 && !kDense) ? qpos : lk1 - 1) : -1;
    const int qlim2 = row_ok ? qpos : -1;                              // depth-1 keys: pos_k <= qlim2
    const int wmax1 = wave_reduce_max(qlim1);
    const int wmin1 = wave_reduce_min(row_ok ? qlim1 : 0x7fffffff);
    int* bounds = reinterpret_cast<int*>(smem + kBoundsOff);
    if (lane == 0) bounds[wave] = wmax1;
    __syncthreads();
    int tmax1 = -1;
#pragma unroll
    for (int w = 0; w < W; ++w) tmax1 = bounds[w] > tmax1 ? bounds[w] : tmax1;

    // Tile schedule.  All waves walk the same n1 + n2 tiles (one barrier each); what a wave does
    // with a depth-0 tile depends on where the tile lies relative to the wave's own rows:
    //   [0, n_plain)         every key visible to every row of the wave: no mask code at all
    //   [n_plain, n_active)  tile straddles a row's position: per-element index mask
    //   [n_active, n1)       tile wholly above the wave's rows: no compute
    // followed by the n2 depth-1 tiles (per-element position mask).
    // (all wave-uniform: moved to scalar registers so that the tile loops are scalar loops)
    const int n1 = __builtin_amdgcn_readfirstlane(tmax1 >= 0 ? tmax1 / kBN + 1 : 0);
    const int n2 = second ? (lk2 + kBN - 1) / kBN : 0;
    const int ntiles = n1 + n2;
    const int n_active = __builtin_amdgcn_readfirstlane(wmax1 >= 0 ? wmax1 / kBN + 1 : 0);
    int n_plain = __builtin_amdgcn_readfirstlane(wmin1 >= kBN - 1 ? (wmin1 - (kBN - 1)) / kBN + 1 : 0);
    n_plain = n_plain < n_active ? n_plain : n_active;
    if constexpr (kDense) n_plain = 0;  // the mask is read for every tile
    // additive-mask mode: this lane's mask row
    const unsigned char* mask_row = nullptr;
    if constexpr (kDense) {
        const int64_t e = (int64_t)seq * p.mask_sb + (int64_t)head * p.mask_sh +
                          (int64_t)(row_ld - qs.cu_q[seq]) * p.mask_sq;
        mask_row = static_cast<const unsigned char*>(p.mask) + e * (p.mask_f32 ? 4 : 2);
    }

    // ---- Q fragments: B operand of S^T = K Q^T ------------------------------
    bf16x8 qf[8];
    {
        const __bf16* qrow = qs.q + (int64_t)row_ld * qs.q_rs + (int64_t)head * qs.q_hs + 8 * half;
#pragma unroll
        for (int s = 0; s < 8; ++s) qf[s] = ld_global_16B(qrow + 16 * s);
    }

    f32x16 oacc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m_run = kNegInf;  // running max of raw scores
    float l_run = 0.f;      // this lane's share of the running denominator
    const float c = p.scale_log2e;

    // ---- asynchronous global -> LDS copies (no registers, no ds_write) ------------------------
    // A tile is 16 blocks of 4 rows, two per wave; lane l fills row 4*blk + l/16, physical chunk
    // l%16, i.e. fetches logical chunk (l%16) ^ row_swizzle(row) of that row.  Rows past the end
    // of the segment are clamped to the last row of the array (finite data, masked by index).
    // The source is addressed as (wave-uniform pointer to the tile's first row) + (per-lane byte
    // offset < 2^30: row strides are limited to 2^23 elements by the host-side checks).
    const int my_lrow = kRowsPerWave * wave + (lane >> 4);  // piece i: 4 * i rows further down
    uint32_t my_chunk[kPieces];
#pragma unroll
    for (int i = 0; i < kPieces; ++i) my_chunk[i] = (uint32_t)(((lane & 15) ^ row_swizzle(my_lrow + 4 * i)) * 16);
    auto issue_rows = [&](const __bf16* src, int64_t rs, int base, int left, unsigned char* dst) {
        const __bf16* tile0 = src + (int64_t)base * rs;
        const int last = left - 1 - base;  // >= 0: a tile starts inside its segment
        const uint32_t rs2 = (uint32_t)(rs * 2) & 0xffffffu;
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const uint32_t r = (uint32_t)(my_lrow + 4 * i < last ? my_lrow + 4 * i : last) & 63u;
            async_copy_16B(tile0, r * rs2 + my_chunk[i], dst + (kPieces * wave + i) * 1024);
        }
    };
    auto issue_k = [&](int it) {  // K tile `it` -> K ring, plus the positions of depth-1 keys
        unsigned char* kt = smem + kKRing + (it % kStages) * kKBytes;
        if (it < n1) {
            issue_rows(k1p, p.s1.k_rs, it * kBN, left1, kt);
        } else {
            const int base = (it - n1) * kBN;
            issue_rows(k2p, p.s2.k_rs, base, left2, kt);
            if (wave == 0) {
                int r = base + lane;
                r = r < lk2 ? r : lk2 - 1;
                async_copy_4B(pos2p + r, smem + kPosRing + (it % kPosSlots) * (kBN * 4));
            }
        }
    };
    auto issue_v = [&](int it) {
        unsigned char* vt = smem + kVRing + (it % kStages) * kVBytes;
        if (it < n1) issue_rows(v1p, p.s1.v_rs, it * kBN, left1, vt);
        else issue_rows(v2p, p.s2.v_rs, (it - n1) * kBN, left2, vt);
    };
    // start of even half-phase 2u: K(u+1) replaces K(u-1), V(u) replaces V(u-2)
    auto issue = [&](int u) {
        if (u + 1 < ntiles) issue_k(u + 1);
        if (u < ntiles) issue_v(u);
    };

    // per-lane LDS read offsets (tile-relative), computed once
    int koff[8];       // K row `col` (+32 per mt), chunk 2s + half
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) koff[s8] = rowmajor128_off(col, 2 * s8 + half);
    int voff_lo[4], voff_hi[4];  // V rows 4*half + r/4 (+8), columns 32*dt + 16*grp + 4*(r%4), +16 rows per step
    {
        const int r16 = lane & 15, grp = (lane >> 4) & 1;
        const int vrow = 4 * half + (r16 >> 2);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            const int vcol = 32 * dt + 16 * grp + 4 * (r16 & 3);
            voff_lo[dt] = rowmajor128_off(vrow, vcol >> 3) + (vcol & 7) * 2;
            voff_hi[dt] = rowmajor128_off(vrow + 8, vcol >> 3) + (vcol & 7) * 2;
        }
    }

    f32x16 sacc[2];    // S^T of the tile in flight: written by M(t-1), consumed by X(t)
    bf16x8 pfrag[4];   // its probabilities: written by X(t), consumed by M(t)

    // ---- matrix phase pieces -------------------------------------------------------------------
    auto qk = [&](int it) __attribute__((always_inline)) {  // S^T = K(it) Q^T
        const unsigned char* kt = smem + kKRing + (it % kStages) * kKBytes;
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
            sacc[mt] = mfma32(*reinterpret_cast<const bf16x8*>(kt + koff[0] + mt * 8192), qf[0], zero);
#pragma unroll
        for (int s = 1; s < 8; ++s)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                sacc[mt] = mfma32(*reinterpret_cast<const bf16x8*>(kt + koff[s] + mt * 8192), qf[s], sacc[mt]);
    };
    auto pv = [&](int it) __attribute__((always_inline)) {  // O^T (128 d x 32 queries) += V(it)^T P^T
        const unsigned char* vt = smem + kVRing + (it % kStages) * kVBytes;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                const bf16x4 lo = lds_read_tr16(vt + voff_lo[dt] + st * 4096);
                const bf16x4 hi = lds_read_tr16(vt + voff_hi[dt] + st * 4096);
                oacc[dt] = mfma32(__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7), pfrag[st], oacc[dt]);
            }
        }
    };
    // M(t): O^T += V(t)^T P(t)^T, then (kQk) S(t+1)^T = K(t+1) Q^T, as one straight-line block whose
    // LDS reads run four MFMAs ahead of their consumers.
    auto matrix = [&](int t, auto qk_tag) __attribute__((always_inline)) {
        constexpr bool kQk = decltype(qk_tag)::value;
        __builtin_amdgcn_s_setprio(kMatrixPrio);  // the matrix pipe is the scarce one: its wave issues first
        pv(t);
        if constexpr (kQk) qk(t + 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
        for (int i = 0; i < 12; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        if constexpr (kQk) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_s_setprio(0);
    };
    // is tile t+1 one this wave computes?
    auto next_active = [&](int t) { return t + 1 < n_active || (t + 1 >= n1 && t + 1 < ntiles); };

    // ---- vector phase: mask, online softmax (one query per lane column, two lanes per query) ----
    auto softmax = [&](int it, auto mask_tag) __attribute__((always_inline)) {
        constexpr Mask kMask = decltype(mask_tag)::value;
        if constexpr (kMask == Mask::kIndex) {
            const int base = it * kBN;
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    sacc[mt][r] = base + 32 * mt + acc_row(half, r) <= qlim1 ? sacc[mt][r] : kNegInf;
        } else if constexpr (kMask == Mask::kDense) {
            const int base = it * kBN;
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int kk = base + 32 * mt + acc_row(half, r);
                    const int kc = kk <= qlim1 ? kk : 0;  // (never read past the row)
                    const float mv = p.mask_f32
                                         ? reinterpret_cast<const float*>(mask_row)[(int64_t)kc * p.mask_sk]
                                         : (float)reinterpret_cast<const __bf16*>(mask_row)[(int64_t)kc * p.mask_sk];
                    sacc[mt][r] = kk <= qlim1 ? sacc[mt][r] + mv * p.inv_scale : kNegInf;
                }
        } else if constexpr (kMask == Mask::kPos) {
            const int* kpos = reinterpret_cast<const int*>(smem + kPosRing + (it % kPosSlots) * (kBN * 4));
            const int nleft = lk2 - (it - n1) * kBN;  // keys of this tile that exist
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int kk = 32 * mt + acc_row(half, r);
                    sacc[mt][r] = (kk < nleft && kpos[kk] <= qlim2) ? sacc[mt][r] : kNegInf;
                }
        }
        float mx = kNegInf;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[mt][r]);
        mx = wave_max_xor32(mx);
        // Lazy reference: the exponent reference m_run follows the true row maximum only when that
        // has grown by more than kLazy (log2 units) for some row of the wave; until then
        // probabilities may reach 2^kLazy, which fp32 sums and bf16 operands absorb, and the 64
        // accumulator multiplies are skipped.  O/l and the LSE do not depend on the reference.
        const float m_new = fmaxf(m_run, mx);
        const bool grow = (m_new - m_run) * c > kLazy;  // true for the first finite maximum (m_run = -inf)
        const int any_grow = __builtin_amdgcn_readfirstlane((int)(__builtin_amdgcn_ballot_w64(grow) != 0));  // wave-uniform, scalar
        const float m_next = any_grow ? m_new : m_run;
        const float m_use = m_next == kNegInf ? 0.f : m_next;
        const float alpha = fast_exp2((m_run - m_use) * c);  // 1 when nothing changes, 0 from -inf
        m_run = m_next;
        const float mc = m_use * c;
        float psum = 0.f;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float e = fast_exp2(sacc[mt][r] * c - mc);
                psum += e;
                pfrag[2 * mt + r / 8][r % 8] = (__bf16)e;
            }
        l_run = l_run * alpha + psum;
        f32x16* const op = oacc;  // (asm operands alone do not make a lambda capture the array)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) TAH_SCALE16_IF(op[dt], alpha, any_grow);
        // Pin the results here: without a use inside this phase the optimiser sinks the whole
        // computation to its first consumer, i.e. past the barrier into the matrix phase.
        TAH_KEEP_HERE4(pfrag[0], pfrag[1], pfrag[2], pfrag[3]);
        TAH_KEEP_HERE4(op[0], op[1], op[2], op[3]);
    };
    using PlainTag = std::integral_constant<Mask, Mask::kNone>;
    using IndexTag = std::integral_constant<Mask, kDense ? Mask::kDense : Mask::kIndex>;
    using PosTag = std::integral_constant<Mask, Mask::kPos>;

    // Workgroup timeline: half-phases h = 0 .. 2*ntiles+1, a barrier before each.  Waves of the
    // early set run S(0) at h=0, X(t) at h=2t+1 and M(t) at h=2t+2; waves of the late set run
    // everything one half-phase later.  Copies are issued at the start of every even half-phase
    // and awaited at the end of the following odd one, so a tile has two half-phases to arrive.
    // Each barrier is a scheduling fence: nothing of a vector phase may drift into a matrix phase.
#define TAH_PHASE_BARRIER()                      \
    do {                                         \
        __builtin_amdgcn_sched_barrier(0);       \
        __syncthreads();                         \
        __builtin_amdgcn_sched_barrier(0);       \
    } while (0)
    auto step_early = [&](int t, auto tag, auto qk_tag) __attribute__((always_inline)) {
        TAH_PHASE_BARRIER();
        softmax(t, tag);
        TAH_WAIT_VMEM();
        TAH_PHASE_BARRIER();
        issue(t + 1);
        matrix(t, qk_tag);
    };
    // one wave set (4-wave workgroups): the barrier that publishes the copies is the only one -- every wave has left
    // M(t-1) before it, so the ring slots the copies issued behind it overwrite are free
    auto step_single = [&](int t, auto tag, auto qk_tag) __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        softmax(t, tag);
        TAH_WAIT_VMEM();
        TAH_PHASE_BARRIER();
        issue(t + 1);
        matrix(t, qk_tag);
    };
    auto idle_single = [&](int t) __attribute__((always_inline)) {
        TAH_WAIT_VMEM();
        TAH_PHASE_BARRIER();
        issue(t + 1);
        if (next_active(t)) qk(t + 1);
    };
    auto step_late = [&](int t, auto tag, auto qk_tag) __attribute__((always_inline)) {
        TAH_WAIT_VMEM();
        TAH_PHASE_BARRIER();
        issue(t + 1);
        softmax(t, tag);
        TAH_PHASE_BARRIER();
        matrix(t, qk_tag);
    };
    auto idle_early = [&](int t) __attribute__((always_inline)) {
        TAH_PHASE_BARRIER();
        TAH_WAIT_VMEM();
        TAH_PHASE_BARRIER();
        issue(t + 1);
        if (next_active(t)) qk(t + 1);
    };
    auto idle_late = [&](int t) __attribute__((always_inline)) {
        TAH_WAIT_VMEM();
        TAH_PHASE_BARRIER();
        issue(t + 1);
        TAH_PHASE_BARRIER();
        if (next_active(t)) qk(t + 1);
    };
    using WithQk = std::true_type;
    using NoQk = std::false_type;
    // Tiles of a run whose successor is computed too take the fused PV + QK^T block; the last tile
    // of a run (at most one iteration of each second loop) takes the PV-only block.
    const int act_q = next_active(n_active - 1) ? n_active : n_active - 1;  // [0, act_q): successor active
    const int plain_q = n_plain < act_q ? n_plain : act_q;
    auto run = [&](auto late_tag) __attribute__((always_inline)) {
        constexpr bool kLate = decltype(late_tag)::value;
        auto step = [&](int t, auto tag, auto qk_tag) __attribute__((always_inline)) {
            if constexpr (W == 4) step_single(t, tag, qk_tag);
            else if constexpr (kLate) step_late(t, tag, qk_tag);
            else step_early(t, tag, qk_tag);
        };
        int t = 0;
        if constexpr (kLate) TAH_PHASE_BARRIER();  // before h = 1
        if (next_active(-1)) qk(0);
        for (; t < plain_q; ++t) step(t, PlainTag{}, WithQk{});
        for (; t < n_plain; ++t) step(t, PlainTag{}, NoQk{});
        for (; t < act_q; ++t) step(t, IndexTag{}, WithQk{});
        for (; t < n_active; ++t) step(t, IndexTag{}, NoQk{});
        for (; t < n1; ++t) {
            if constexpr (W == 4) idle_single(t);
            else if constexpr (kLate) idle_late(t);
            else idle_early(t);
        }
        for (; t < ntiles - 1; ++t) step(t, PosTag{}, WithQk{});
        for (; t < ntiles; ++t) step(t, PosTag{}, NoQk{});
        if constexpr (W == 8 && !kLate) TAH_PHASE_BARRIER();  // before h = 2*ntiles + 1
    };

    if (ntiles > 0) issue_k(0);
    TAH_WAIT_VMEM();  // K(0) and the Q fragments are in: no ordinary load stays pending across the tile loop
    if (ntiles > 0) {
        TAH_PHASE_BARRIER();  // before h = 0
        issue(0);
        if (W == 4 || late_set(wave) == 0) run(std::false_type{});
        else run(std::true_type{});
    }
    if constexpr (W == 4) {  // the output staging below overlies the rings: every wave must be done reading them
        TAH_WAIT_VMEM();
        TAH_PHASE_BARRIER();
    }
#undef TAH_PHASE_BARRIER

    // ---- epilogue -----------------------------------------------------------
    const float l_tot = wave_sum_xor32(l_run);
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    // The accumulators hold O^T (a lane owns one query row, four values of d at a time): written out
    // directly every store instruction would touch 32 rows with 8 bytes each.  The wave turns its
    // 32 x 128 tile through a private piece of LDS instead (16-byte chunks of a row XOR-swizzled by the
    // row number, so that neither side runs into bank conflicts) and stores whole rows: 4 rows x 256
    // contiguous bytes per instruction.  Nobody else reads or writes this piece: no barrier.
    unsigned char* stage = smem + (W == 4 ? 0 : kStageOff) + wave * 8192;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            bf16x4 v4;
#pragma unroll
            for (int b = 0; b < 4; ++b) v4[b] = (__bf16)(oacc[dt][4 * g4 + b] * inv);
            *reinterpret_cast<bf16x4*>(stage + col * 256 + (((4 * dt + g4) ^ (col & 15)) * 16) + half * 8) = v4;
        }
    TAH_WAVE_LDS_SYNC();  // the reads below are of other lanes' writes
    {
        const int ch = lane & 15;
        __bf16* obase = qs.o + (int64_t)head * qs.o_hs + ch * 8;
        const int tile_row0 = row0 + rblk * 32;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = 4 * i + (lane >> 4);
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(stage + r * 256 + ((ch ^ (r & 15)) * 16));
            if (tile_row0 + r < row_end) st_global_16B(obase + (int64_t)(tile_row0 + r) * qs.o_rs, v);
        }
    }
    if (row_ok && half == 0)
        qs.lse[(int64_t)head * qs.total_q + row] = l_tot > 0.f ? (m_run * c + fast_log2(l_tot)) * kLn2 : kNegInf;
}

FwdStream to_dev(const tah_duo_stream& s) {
    FwdStream d;
    d.q = static_cast<const __bf16*>(s.q);
    d.k = static_cast<const __bf16*>(s.k);
    d.v = static_cast<const __bf16*>(s.v);
    d.o = static_cast<__bf16*>(s.o);
    d.lse = s.lse;
    d.cu_q = s.cu_q;
    d.cu_k = s.cu_k;
    d.pos_q = s.pos_q;
    d.pos_k = s.pos_k;
    d.q_rs = s.q_row_stride; d.q_hs = s.q_head_stride;
    d.k_rs = s.k_row_stride; d.k_hs = s.k_head_stride;
    d.v_rs = s.v_row_stride; d.v_hs = s.v_head_stride;
    d.o_rs = s.o_row_stride; d.o_hs = s.o_head_stride;
    d.total_q = s.total_q;
    d.total_k = s.total_k;
    return d;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_stream(const tah_duo_stream& s, bool second) {
    if (s.total_q < 0 || s.total_k < 0) return TAH_E_SHAPE;
    if (s.total_q == 0) return TAH_OK;
    if (!s.q || !s.o || !s.lse || !s.cu_q || !s.cu_k) return TAH_E_NULL;
    if (s.total_k > 0 && (!s.k || !s.v)) return TAH_E_NULL;
    if (second && (!s.pos_q || (s.total_k > 0 && !s.pos_k))) return TAH_E_NULL;
    if (!aligned16(s.q) || !aligned16(s.k) || !aligned16(s.v) || !aligned16(s.o)) return TAH_E_ALIGN;
    const int64_t st[] = {s.q_row_stride, s.q_head_stride, s.k_row_stride, s.k_head_stride,
                          s.v_row_stride, s.v_head_stride, s.o_row_stride, s.o_head_stride};
    for (int64_t x : st)
        if (x % 8 != 0) return TAH_E_ALIGN;
    // the tile copies address rows as base + row * stride with a 24-bit multiply
    if (s.k_row_stride < 0 || s.v_row_stride < 0 || s.k_row_stride >= (1 << 23) || s.v_row_stride >= (1 << 23))
        return TAH_E_SHAPE;
    return TAH_OK;
}

template <int G, bool kDense>
int launch_fwd(const FwdParams& p, hipStream_t stream) {
    constexpr int BM = 32 * (8 / G);
    int tiles = 0;  // upper bound on sum_b ceil(len_b / BM), no device read needed
    if (p.s1.total_q > 0) tiles += p.s1.total_q / BM + p.nseq;
    if (p.s2.total_q > 0) tiles += p.s2.total_q / BM + p.nseq;
    // duo-causal calls with up to four query heads per kv head: 4-wave workgroups, two per compute unit (same results
    // to the bit; measured 0-5 % faster than the 8-wave form, most with several short documents)
    if constexpr (!kDense && G <= 4) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_fwd_kernel<G, kDense, 4>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes4) != hipSuccess)
            return TAH_E_LAUNCH;
        hipLaunchKernelGGL((duo_fwd_kernel<G, kDense, 4>), dim3(p.hkv, 2 * tiles), dim3(256), kSmemBytes4, stream, p);
        return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
    }
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_fwd_kernel<G, kDense, 8>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes) != hipSuccess)
        return TAH_E_LAUNCH;
    hipLaunchKernelGGL((duo_fwd_kernel<G, kDense, 8>), dim3(p.hkv, tiles), dim3(kThreads), kSmemBytes, stream, p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

template <bool kDense>
int dispatch_fwd(const tah_duo_fwd_args* a, const tah_additive_mask* m, tah_stream_t stream) {
    if (!a) return TAH_E_NULL;
    if (a->d != kD || a->nseq < 0 || a->hq <= 0 || a->hkv <= 0 || a->hq % a->hkv != 0) return TAH_E_SHAPE;
    const int g = a->hq / a->hkv;
    if (g != 1 && g != 2 && g != 4 && g != 8) return TAH_E_SHAPE;
    if (int rc = check_stream(a->s1, false)) return rc;
    if (int rc = check_stream(a->s2, true)) return rc;
    if (a->s2.total_q > 0 && (!a->s1.cu_k || (a->s1.total_k > 0 && (!a->s1.k || !a->s1.v)))) return TAH_E_NULL;
    if (kDense) {
        if (!m || !m->mask) return TAH_E_NULL;
        if (a->s2.total_q != 0 || a->s2.total_k != 0 || (m->dtype != 0 && m->dtype != 1) || a->scale == 0.f) return TAH_E_SHAPE;
    }
    if (a->nseq == 0 || (a->s1.total_q == 0 && a->s2.total_q == 0)) return TAH_OK;
    FwdParams p;
    p.s1 = to_dev(a->s1);
    p.s2 = to_dev(a->s2);
    p.nseq = a->nseq;
    p.hq = a->hq;
    p.hkv = a->hkv;
    p.scale_log2e = a->scale * kLog2e;
    p.sched = kDense ? nullptr : static_cast<const int32_t*>(a->schedule);
    p.mask = nullptr;
    p.mask_sb = p.mask_sh = p.mask_sq = p.mask_sk = 0;
    p.mask_f32 = 0;
    p.inv_scale = 0.f;
    if (kDense) {
        p.mask = m->mask;
        p.mask_sb = m->seq_stride; p.mask_sh = m->head_stride; p.mask_sq = m->q_stride; p.mask_sk = m->k_stride;
        p.mask_f32 = m->dtype;
        p.inv_scale = 1.0f / a->scale;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (g) {
        case 1: return launch_fwd<1, kDense>(p, st);
        case 2: return launch_fwd<2, kDense>(p, st);
        case 4: return launch_fwd<4, kDense>(p, st);
        default: return launch_fwd<8, kDense>(p, st);
    }
}

}  // namespace
}  // namespace tah

extern "C" int tah_duo_fwd_varlen(const tah_duo_fwd_args* a, tah_stream_t stream) {
    return tah::dispatch_fwd<false>(a, nullptr, stream);
}

extern "C" int tah_duo_fwd_masked(const tah_duo_fwd_args* a, const tah_additive_mask* m, tah_stream_t stream) {
    return tah::dispatch_fwd<true>(a, m, stream);
}
