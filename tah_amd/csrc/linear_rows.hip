// Linear layers of a decode step, gfx950: y = x W^T for at most 32 rows (one token per sequence) against a weight
// of 8 to 50 MB.  The work is streaming W from HBM once; everything here serves having all of it in flight with
// as few cache-line requests as possible:
//
//  * W is re-ordered once, when the model is loaded, into the order the matrix instruction wants it: tiles of
//    16 output columns x 32 k, each stored as the 64 16-byte operands of the 64 lanes of one
//    v_mfma_f32_16x16x32_bf16 step (lane l: column l % 16, k = 8 (l / 16) ... + 8).  A wave's load instruction
//    then reads 1 KiB that lies together, and a column tile's k steps follow each other in memory.
//  * The rows are kept in the same form ([k / 32][2 row halves][64 lanes][8]): the kernels that produce them
//    (these linear layers, the attention merge, tah_linear_pack_rows) write it, so the rows' operand is one
//    1 KiB load per step and row half as well.  Reading either operand from a row-major matrix costs one cache
//    line request per row and lane group, and those, not the bytes, bound such a kernel.
//  * One workgroup = one group of output columns over all of K; its eight waves split K and meet in LDS.  A
//    wave issues the loads of a whole chunk of steps (up to 24 KiB) before the first multiply.
//  * Epilogues: + residual (in place is fine), or the MLP's act_fn(gate) * up with the input RMSNorm's per-row
//    factor (the norm's weight is expected inside W): the sum of squares of a row comes from the operands the
//    waves load anyway.  A LayerNorm of the rows folds in the same way (the learned decider's blocks,
//    tah/model/iter_decider.py:139-152): with W' = W diag(gamma), W' LN(x) = (W' x - mean(x) W' 1) / std(x) + W beta,
//    so the kernel needs the row's sum and sum of squares, the row sums of W' and a bias that carries W beta.
//    ReLU or GELU (the exact one, nn.GELU's default) last.  Results are written row-major and/or in the packed rows
//    form for the next layer.
//
// Measured at 32 rows inside a captured step (MI355X): q|k|v 16 MB 6.0 us, o 8 MB 5.1 us, gate|up + SiLU 50 MB
// 12.3 us, down 25 MB 9.6 us, against 14 / 8.4 / 16 + 5 / 15 us for the library GEMMs and the SiLU kernel.  What
// is left besides the weight stream (7.5 TB/s once started) is about 4 us of launch, first-byte latency and
// reduction per kernel, and the rows' operand: every workgroup reads all 32 x K of it from L2, which the
// per-CU L1 fill rate (about 100 GB/s) makes 1 us per 128 KB.  Splitting K over workgroups would cut that, but
// the hand-over between workgroups (device-scope fence + counter, last one reduces) cost 7 us per split when
// tried: the fence writes back and invalidates the whole L2 of the XCD.
#include <hip/hip_runtime.h>

#include "duo_device.h"
#include "tah_duo.h"

namespace tah {
namespace {

constexpr int kLinWaves = 8;
constexpr int kLinThreads = kLinWaves * kWave;
constexpr int kLinRows = 32;    // rows per call: two 16-row halves of the MFMA's row operand
constexpr int kTileCols = 16;   // output columns of one weight tile
constexpr int kStepK = 32;      // k of one MFMA step; a tile step is 16 x 32 bf16 = 1 KiB
constexpr int kGroup24 = 24;    // gate|up: output columns per workgroup when n % 24 == 0 (256 workgroups for n = 6144)

// kPlainNorm: plain with the rows' RMSNorm factor; kPlainLayerNorm: with the rows' mean and deviation
enum Epi { kPlain = 0, kPlainNorm = 1, kGateUp16 = 2, kGateUp24 = 3, kPlainLayerNorm = 4 };

struct LinParams {
    const bf16x8* w;   // packed weight
    const bf16x8* x;   // packed rows
    const __bf16* res; // row-major residual or null
    const __bf16* bias; // [n] added to the product (rounded to bf16 first, as a GEMM's output is) or null
    const float* colsum; // kPlainLayerNorm: [n] sums of the packed weight's rows over k
    int32_t act;       // TAH_ACT_*
    __bf16* y;         // row-major result or null
    bf16x8* yp;        // packed result or null
    int64_t res_rs, y_rs;
    int32_t rows, n, k;
    float eps;
    int32_t norm;
    int32_t groups;  // column groups (workgroups per row half)
};

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }

// 16-byte unit of the packed rows form that holds row r, columns k ... k + 7 (k % 8 == 0)
__device__ __host__ __forceinline__ int64_t packed_rows_unit(int r, int k) {
    return ((int64_t)(k / kStepK) * 2 + r / 16) * 64 + (r % 16) + 16 * ((k % kStepK) / 8);
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + fast_exp2(-x * kLog2e)); }

// NC: weight tiles per workgroup (1 plain, 2 or 3 for gate|up).  CH: steps per chunk of loads.  PW: steps per wave
// when K is known at compile time (K = 32 * 8 * PW), 0: any K % 32 == 0.  NH: row halves per workgroup -- 2: all 32
// rows; 1: sixteen rows, the grid holds a workgroup per (column group, half) (or only the first half when there
// are at most 16 rows).  A layer with few column groups (n = 2048: 128) then fills the chip, and every compute
// unit pulls half of the rows' operand; the second reader of a weight tile is placed on the same XCD, whose L2 has
// it or is fetching it.
template <int NC, int CH, int EPI, int PW, int NH>
__global__ __launch_bounds__(kLinThreads) void linear_rows_kernel(const LinParams p) {
    __shared__ __align__(16) float red[kLinWaves][NC][16 * NH][kTileCols];
    __shared__ float ssq[kLinWaves][16 * NH];
    __shared__ float ssum[EPI == kPlainLayerNorm ? kLinWaves : 1][16 * NH];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int c = lane % 16, kg = lane / 16;
    int group = blockIdx.x, half = 0;
    if (NH == 1 && (int)gridDim.x == 2 * p.groups) {
        if (p.groups % 8 == 0) {  // workgroups go to the XCDs round robin: i and i + 8 share one
            group = (blockIdx.x / 16) * 8 + blockIdx.x % 8;
            half = (blockIdx.x / 8) % 2;
        } else {
            group = blockIdx.x / 2;
            half = blockIdx.x % 2;
        }
    }
    // The epilogue's own operands (residual, bias: 16 bytes each for a thread that writes results) are asked for here:
    // requested behind the reduction they would cost the kernel one trip to memory each, one after the other.
    constexpr bool kGateEpi = EPI == kGateUp16 || EPI == kGateUp24;
    constexpr int kEpiUnits = EPI == kGateUp24 ? 3 : (kGateEpi ? 2 : 2 * NC);
    bf16x8 res_early = {0, 0, 0, 0, 0, 0, 0, 0}, bias_early = {0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (!kGateEpi) {
        const bool writer = (int)threadIdx.x < 16 * NH * kEpiUnits;
        const int erow = 16 * half + (writer ? (int)threadIdx.x / kEpiUnits : 0);
        const int en0 = group * NC * kTileCols + 8 * (writer ? (int)threadIdx.x % kEpiUnits : 0);
        const bool live_row = erow < p.rows;
        // (addresses picked by selects, so that no load sits under a branch)
        const __bf16* ra = (p.res && live_row) ? p.res + (int64_t)erow * p.res_rs + en0 : reinterpret_cast<const __bf16*>(p.x);
        const __bf16* ba = p.bias ? p.bias + en0 : reinterpret_cast<const __bf16*>(p.x);
        res_early = *reinterpret_cast<const bf16x8*>(ra);
        bias_early = *reinterpret_cast<const bf16x8*>(ba);
    }
    const int steps = p.k / kStepK;
    const int per_wave = PW > 0 ? PW : (steps + kLinWaves - 1) / kLinWaves;
    int nst = steps - wave * per_wave;
    nst = nst < 0 ? 0 : (nst > per_wave ? per_wave : nst);
    const int s0 = nst > 0 ? wave * per_wave : 0;  // a wave without steps still points at valid memory
    const bf16x8* wb[NC];
#pragma unroll
    for (int t = 0; t < NC; ++t) wb[t] = p.w + ((int64_t)(group * NC + t) * steps + s0) * 64 + lane;
    const bf16x8* xb = p.x + (int64_t)s0 * 128 + 64 * half + lane;

    struct Buf {
        bf16x8 w[CH][NC], x[CH][NH];
    };
    f32x4 acc[NC][NH];
#pragma unroll
    for (int t = 0; t < NC; ++t)
#pragma unroll
        for (int h = 0; h < NH; ++h) acc[t][h] = f32x4{0.f, 0.f, 0.f, 0.f};
    float ss0 = 0.f, ss1 = 0.f, sm0 = 0.f, sm1 = 0.f;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    // Loads of chunk ch.  Without a compile-time K a step past the wave's share reads step 0 of the wave's range
    // (valid memory) and is multiplied by rows of zeros: no branch sits between the loads.
    auto issue = [&](int ch, Buf& b) __attribute__((always_inline)) {
        // the rows' operand first: it comes from L2 and is there long before the weights are, and a wave's loads
        // return in order -- behind the weight loads it would only arrive after their trip to HBM (down 11.2 -> 9.6 us)
#pragma unroll
        for (int s = 0; s < CH; ++s) {
            const int st = ch * CH + s;
            const int64_t sti = (PW > 0 || st < nst) ? st : 0;
            b.x[s][0] = xb[sti * 128];
            if constexpr (NH == 2) b.x[s][1] = xb[sti * 128 + 64];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < CH; ++s) {
            const int st = ch * CH + s;
            const int64_t sti = (PW > 0 || st < nst) ? st : 0;
#pragma unroll
            for (int t = 0; t < NC; ++t) b.w[s][t] = __builtin_nontemporal_load(wb[t] + sti * 64);
        }
    };
    auto multiply = [&](int ch, Buf& b) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < CH; ++s) {
            const bool ok = PW > 0 || ch * CH + s < nst;
            const bf16x8 a0 = ok ? b.x[s][0] : zero8, a1 = ok ? b.x[s][NH - 1] : zero8;
            if constexpr (EPI != kPlain) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float u = (float)a0[i], v = (float)a1[i];
                    ss0 += u * u;
                    ss1 += v * v;
                    if constexpr (EPI == kPlainLayerNorm) {
                        sm0 += u;
                        sm1 += v;
                    }
                }
            }
#pragma unroll
            for (int t = 0; t < NC; ++t) {
                acc[t][0] = mfma16(a0, b.w[s][t], acc[t][0]);
                if constexpr (NH == 2) acc[t][1] = mfma16(a1, b.w[s][t], acc[t][1]);
            }
        }
    };
    if constexpr (PW > 0) {
        static_assert(PW == 0 || PW % CH == 0, "chunks divide a wave's steps");
        constexpr int kChunks = PW > 0 ? PW / CH : 1;
        Buf b[2];
        issue(0, b[0]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ch = 0; ch < kChunks; ++ch) {
            if (ch + 1 < kChunks) issue(ch + 1, b[(ch + 1) % 2]);
            __builtin_amdgcn_sched_barrier(0);
            multiply(ch, b[ch % 2]);
        }
    } else {
        Buf b0, b1;
        const int nch = (nst + CH - 1) / CH;
        issue(0, b0);
        __builtin_amdgcn_sched_barrier(0);
        for (int ch = 0; ch < nch; ch += 2) {
            if (ch + 1 < nch) issue(ch + 1, b1);
            __builtin_amdgcn_sched_barrier(0);
            multiply(ch, b0);
            __builtin_amdgcn_sched_barrier(0);
            if (ch + 2 < nch) issue(ch + 2, b0);
            __builtin_amdgcn_sched_barrier(0);
            if (ch + 1 < nch) multiply(ch + 1, b1);  // never multiply a buffer that was not loaded
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- the eight K slices meet in LDS ------------------------------------------------------------------
    // accumulator (tile t, half h, register r) of lane (c, kg) is row 16 h + 4 kg + r, column c of tile t
#pragma unroll
    for (int t = 0; t < NC; ++t)
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave][t][16 * h + 4 * kg + r][c] = acc[t][h][r];
    if constexpr (EPI != kPlain) {
        // a lane's squares cover its 8 of every 32 k of rows c and 16 + c: add the four k groups
        ss0 += __shfl_xor(ss0, 16);
        ss0 += __shfl_xor(ss0, 32);
        ss1 += __shfl_xor(ss1, 16);
        ss1 += __shfl_xor(ss1, 32);
        if (kg == 0) {
            ssq[wave][c] = ss0;
            if constexpr (NH == 2) ssq[wave][16 + c] = ss1;
        }
        if constexpr (EPI == kPlainLayerNorm) {
            sm0 += __shfl_xor(sm0, 16);
            sm0 += __shfl_xor(sm0, 32);
            sm1 += __shfl_xor(sm1, 16);
            sm1 += __shfl_xor(sm1, 32);
            if (kg == 0) {
                ssum[wave][c] = sm0;
                if constexpr (NH == 2) ssum[wave][16 + c] = sm1;
            }
        }
    }
    __syncthreads();

    // ---- epilogue: one thread per (row, 8 output columns) -------------------------------------------------
    constexpr bool kGate = EPI == kGateUp16 || EPI == kGateUp24;
    constexpr int kUnits = EPI == kGateUp24 ? 3 : (kGate ? 2 : 2 * NC);  // 8-column units of output per row and workgroup
    if (threadIdx.x >= 16 * NH * kUnits) return;
    const int lrow = threadIdx.x / kUnits, unit = threadIdx.x % kUnits;  // row inside the workgroup's rows
    const int row = 16 * half + lrow;
    // where the unit's gate (or plain) and up sums sit: tile and first column inside it
    int gt = kGate ? 0 : unit / 2, gc = kGate ? 8 * unit : 8 * (unit % 2), ut = 1, uc = 8 * unit;
    if constexpr (EPI == kGateUp24) {  // tiles: gate 0-15 | gate 16-23, up 16-23 | up 0-15
        gt = unit == 2 ? 1 : 0;
        gc = unit == 1 ? 8 : 0;
        ut = unit == 2 ? 1 : 2;
        uc = unit == 0 ? 0 : 8;
    }
    float sg[8], su[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sg[i] = su[i] = 0.f;
#pragma unroll
    for (int w = 0; w < kLinWaves; ++w) {
        const f32x4 lo = *reinterpret_cast<const f32x4*>(&red[w][gt][lrow][gc]);
        const f32x4 hi = *reinterpret_cast<const f32x4*>(&red[w][gt][lrow][gc + 4]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sg[i] += lo[i];
            sg[4 + i] += hi[i];
        }
        if constexpr (kGate) {
            const f32x4 ulo = *reinterpret_cast<const f32x4*>(&red[w][ut][lrow][uc]);
            const f32x4 uhi = *reinterpret_cast<const f32x4*>(&red[w][ut][lrow][uc + 4]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                su[i] += ulo[i];
                su[4 + i] += uhi[i];
            }
        }
    }
    const int n0 = group * (EPI == kGateUp24 ? kGroup24 : (kGate ? kTileCols : NC * kTileCols)) + 8 * unit;
    const bool live = row < p.rows;
    bf16x8 out = zero8;
    if (live) {
        float rin = 1.0f;
        if constexpr (EPI != kPlain) {
            if (p.norm) {
                float ss = 0.f;
#pragma unroll
                for (int w = 0; w < kLinWaves; ++w) ss += ssq[w][lrow];
                if constexpr (EPI == kPlainLayerNorm) {
                    float sm = 0.f;
#pragma unroll
                    for (int w = 0; w < kLinWaves; ++w) sm += ssum[w][lrow];
                    const float mean = sm / (float)p.k;
                    const float var = fmaxf(ss / (float)p.k - mean * mean, 0.f);
                    rin = __builtin_amdgcn_rsqf(var + p.eps);
                    const f32x4 c0 = *reinterpret_cast<const f32x4*>(p.colsum + n0), c1 = *reinterpret_cast<const f32x4*>(p.colsum + n0 + 4);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        sg[i] -= mean * c0[i];
                        sg[4 + i] -= mean * c1[i];
                    }
                } else {
                    rin = __builtin_amdgcn_rsqf(ss / (float)p.k + p.eps);
                }
            }
        }
        if constexpr (kGate) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // the projections' own rounding to bf16, the activation's, the product's (Qwen3MLP.forward)
                const float g = (float)(__bf16)(sg[i] * rin), u = (float)(__bf16)(su[i] * rin);
                out[i] = (__bf16)((float)(__bf16)silu_f(g) * u);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) out[i] = (__bf16)(sg[i] * rin);
            if (p.bias) {
#pragma unroll
                for (int i = 0; i < 8; ++i) out[i] = (__bf16)((float)out[i] + (float)bias_early[i]);
            }
            if (p.res) {
#pragma unroll
                for (int i = 0; i < 8; ++i) out[i] = (__bf16)((float)out[i] + (float)res_early[i]);
            }
            if (p.act == TAH_ACT_RELU) {
#pragma unroll
                for (int i = 0; i < 8; ++i) out[i] = (float)out[i] > 0.f ? out[i] : (__bf16)0.f;
            } else if (p.act == TAH_ACT_GELU) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float v = (float)out[i];
                    out[i] = (__bf16)(0.5f * v * (1.0f + erff(v * 0.70710678118654752f)));
                }
            }
        }
        if (p.y) *reinterpret_cast<bf16x8*>(p.y + (int64_t)row * p.y_rs + n0) = out;
    }
    if (p.yp) {
        p.yp[packed_rows_unit(row, n0)] = out;  // rows past the last one stay zero for the next layer
        if (NH == 1 && (int)gridDim.x == p.groups) p.yp[packed_rows_unit(16 + lrow, n0)] = zero8;  // nobody computes the second half
    }
}

// ---- re-ordering -----------------------------------------------------------------------------------------
// Weight row behind column slot c of tile t of the packed order.
__device__ __host__ inline int64_t packed_weight_row(int kind, int n, int tile, int c) {
    if (kind == TAH_LINEAR_PLAIN) return (int64_t)tile * kTileCols + c;
    if (n % kGroup24 == 0) {  // groups of 24 output columns: gate 0-15 | gate 16-23, up 16-23 | up 0-15
        const int g = tile / 3, t = tile % 3;
        if (t == 0) return (int64_t)kGroup24 * g + c;
        if (t == 2) return (int64_t)n + kGroup24 * g + c;
        return c < 8 ? (int64_t)kGroup24 * g + 16 + c : (int64_t)n + kGroup24 * g + 16 + (c - 8);
    }
    const int g = tile / 2;  // groups of 16 output columns: gate | up
    return (tile % 2 ? (int64_t)n : 0) + (int64_t)kTileCols * g + c;
}

__global__ __launch_bounds__(256) void pack_weight_kernel(const __bf16* w, int64_t w_rs, bf16x8* out, int kind, int n, int k, int64_t units) {
    const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (u >= units) return;
    const int steps = k / kStepK;
    const int lane = (int)(u % 64);
    const int64_t ts = u / 64;
    const int step = (int)(ts % steps), tile = (int)(ts / steps);
    const int64_t row = packed_weight_row(kind, n, tile, lane % 16);
    out[u] = *reinterpret_cast<const bf16x8*>(w + row * w_rs + step * kStepK + 8 * (lane / 16));
}

__global__ __launch_bounds__(256) void pack_rows_kernel(const __bf16* x, int64_t x_rs, bf16x8* out, int rows, int k) {
    const int u = blockIdx.x * 256 + threadIdx.x;  // (step, half, lane)
    if (u >= k / kStepK * 128) return;
    const int lane = u % 64, half = (u / 64) % 2, step = u / 128;
    const int row = 16 * half + lane % 16;
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row < rows) v = *reinterpret_cast<const bf16x8*>(x + (int64_t)row * x_rs + step * kStepK + 8 * (lane / 16));
    out[u] = v;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Sixteen rows per workgroup when there are no more, or when the column groups alone would leave half of the
// 256 compute units idle.
constexpr int kSplitRowsBelowGroups = 129;
constexpr int kWideFromCols = 16384;  // plain layers from this many output columns on take 32 columns per workgroup

template <int NC, int CH, int EPI, int PW>
void launch(LinParams& p, int groups, hipStream_t st) {
    p.groups = groups;
    if (p.rows <= 16)
        hipLaunchKernelGGL((linear_rows_kernel<NC, CH, EPI, PW, 1>), dim3(groups), dim3(kLinThreads), 0, st, p);
    else if (groups < kSplitRowsBelowGroups)
        hipLaunchKernelGGL((linear_rows_kernel<NC, CH, EPI, PW, 1>), dim3(2 * groups), dim3(kLinThreads), 0, st, p);
    else
        hipLaunchKernelGGL((linear_rows_kernel<NC, CH, EPI, PW, 2>), dim3(groups), dim3(kLinThreads), 0, st, p);
}

}  // namespace
}  // namespace tah

extern "C" int tah_linear_pack_weight(const void* w, int64_t w_row_stride, void* packed, int32_t n, int32_t k, int32_t kind,
                                      tah_stream_t stream) {
    using namespace tah;
    if (kind != TAH_LINEAR_PLAIN && kind != TAH_LINEAR_GATE_UP) return TAH_E_SHAPE;
    if (n < 0 || k < 0 || k % kStepK != 0 || w_row_stride < k) return TAH_E_SHAPE;
    if (kind == TAH_LINEAR_PLAIN ? n % kTileCols != 0 : (n % kGroup24 != 0 && n % kTileCols != 0)) return TAH_E_SHAPE;
    if (n == 0 || k == 0) return TAH_OK;
    if (!w || !packed) return TAH_E_NULL;
    if (!aligned16(w) || !aligned16(packed) || w_row_stride % 8 != 0) return TAH_E_ALIGN;
    const int64_t total_rows = kind == TAH_LINEAR_GATE_UP ? 2 * (int64_t)n : n;
    const int64_t units = total_rows * k / 8;
    if ((units + 255) / 256 > 0x7fffffff) return TAH_E_SHAPE;
    hipLaunchKernelGGL(pack_weight_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const __bf16*>(w), w_row_stride, static_cast<bf16x8*>(packed), (int)kind, (int)n, (int)k, units);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_linear_pack_rows(const void* x, int64_t x_row_stride, void* x_packed, int32_t rows, int32_t k, tah_stream_t stream) {
    using namespace tah;
    if (rows < 0 || rows > kLinRows || k < 0 || k % kStepK != 0) return TAH_E_SHAPE;
    if (k == 0) return TAH_OK;
    if (!x_packed || (rows > 0 && !x)) return TAH_E_NULL;
    if (!aligned16(x) || !aligned16(x_packed) || (rows > 1 && x_row_stride % 8 != 0)) return TAH_E_ALIGN;
    const int units = k / kStepK * 128;
    hipLaunchKernelGGL(pack_rows_kernel, dim3((units + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const __bf16*>(x), x_row_stride, static_cast<bf16x8*>(x_packed), (int)rows, (int)k);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_linear_rows(const tah_linear_rows_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    if (a->kind != TAH_LINEAR_PLAIN && a->kind != TAH_LINEAR_GATE_UP) return TAH_E_SHAPE;
    if (a->rows < 0 || a->rows > kLinRows || a->n < 0 || a->k < 0 || a->k % kStepK != 0) return TAH_E_SHAPE;
    const bool gate_up = a->kind == TAH_LINEAR_GATE_UP;
    const bool g24 = gate_up && a->n % kGroup24 == 0;
    if (!g24 && a->n % kTileCols != 0) return TAH_E_SHAPE;
    if (a->activation != TAH_ACT_NONE && a->activation != TAH_ACT_RELU && a->activation != TAH_ACT_GELU) return TAH_E_SHAPE;
    if (a->input_norm != TAH_NORM_NONE && a->input_norm != TAH_NORM_RMS && a->input_norm != TAH_NORM_LAYER) return TAH_E_SHAPE;
    if (gate_up && (a->residual || a->bias || a->activation != TAH_ACT_NONE || a->input_norm == TAH_NORM_LAYER)) return TAH_E_SHAPE;
    if (a->input_norm == TAH_NORM_LAYER && !a->ln_colsum && a->n > 0 && a->k > 0) return TAH_E_NULL;
    if (a->out_packed && a->n % kStepK != 0) return TAH_E_SHAPE;  // the packed rows form holds whole steps of 32 columns
    if (a->n == 0 || a->k == 0 || (a->rows == 0 && !a->out_packed)) return TAH_OK;
    if (!a->w_packed || !a->x_packed || (!a->out && !a->out_packed)) return TAH_E_NULL;
    if (!aligned16(a->w_packed) || !aligned16(a->x_packed) || !aligned16(a->out) || !aligned16(a->out_packed) || !aligned16(a->residual) ||
        !aligned16(a->bias) || (a->input_norm == TAH_NORM_LAYER && !aligned16(a->ln_colsum)) ||
        (a->out && a->out_row_stride % 8 != 0) || (a->residual && a->residual_row_stride % 8 != 0))
        return TAH_E_ALIGN;
    if ((a->out && a->out_row_stride < a->n) || (a->residual && a->residual_row_stride < a->n)) return TAH_E_SHAPE;
    LinParams p{};
    p.w = static_cast<const bf16x8*>(a->w_packed);
    p.x = static_cast<const bf16x8*>(a->x_packed);
    p.res = static_cast<const __bf16*>(a->residual);
    p.bias = static_cast<const __bf16*>(a->bias);
    p.act = a->activation;
    p.colsum = a->input_norm == TAH_NORM_LAYER ? a->ln_colsum : nullptr;
    p.y = static_cast<__bf16*>(a->out);
    p.yp = static_cast<bf16x8*>(a->out_packed);
    p.res_rs = a->residual_row_stride;
    p.y_rs = a->out_row_stride;
    p.rows = a->rows;
    p.n = a->n;
    p.k = a->k;
    p.eps = a->norm_eps;
    p.norm = a->input_norm;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int steps = a->k / kStepK;
    const int pw = steps % kLinWaves == 0 ? steps / kLinWaves : 0;  // compile-time K for the sizes of the end-to-end model
    if (!gate_up && a->input_norm != TAH_NORM_LAYER && a->n >= kWideFromCols && a->n % (2 * kTileCols) == 0) {
        // an output head: two tiles per workgroup, the rows' operand is read half as often
        const int groups = a->n / (2 * kTileCols);
        if (p.norm) {
            if (pw == 8) launch<2, 2, kPlainNorm, 8>(p, groups, st);
            else launch<2, 2, kPlainNorm, 0>(p, groups, st);
        } else {
            if (pw == 8) launch<2, 2, kPlain, 8>(p, groups, st);
            else launch<2, 2, kPlain, 0>(p, groups, st);
        }
    } else if (!gate_up && a->input_norm == TAH_NORM_LAYER) {
        launch<1, 4, kPlainLayerNorm, 0>(p, a->n / kTileCols, st);
    } else if (!gate_up) {
        const int groups = a->n / kTileCols;
        if (p.norm) {
            if (pw == 8) launch<1, 8, kPlainNorm, 8>(p, groups, st);
            else launch<1, 4, kPlainNorm, 0>(p, groups, st);
        } else if (pw == 8) launch<1, 8, kPlain, 8>(p, groups, st);
        else if (pw == 24) launch<1, 8, kPlain, 24>(p, groups, st);
        else launch<1, 4, kPlain, 0>(p, groups, st);
    } else if (g24) {
        const int groups = a->n / kGroup24;
        if (pw == 8) launch<3, 4, kGateUp24, 8>(p, groups, st);
        else launch<3, 2, kGateUp24, 0>(p, groups, st);
    } else {
        const int groups = a->n / kTileCols;
        if (pw == 8) launch<2, 4, kGateUp16, 8>(p, groups, st);
        else launch<2, 2, kGateUp16, 0>(p, groups, st);
    }
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}
