// Small fused element-wise steps of a decode step, gfx950 (HBM-bound, trivially so at decode sizes: what
// they save is launches, one per fused pair per layer per latent iteration).
#include <hip/hip_runtime.h>

#include "duo_device.h"
#include "tah_duo.h"

namespace tah {
namespace {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2e __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {  // two floats -> packed bf16 pair (nearest even)
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2e));
}
__device__ __forceinline__ float lo_f(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float hi_f(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float silu(float x) { return x / (1.0f + fast_exp2(-x * kLog2e)); }

// out[r][i] = bf16(bf16(silu(gu[r][i])) * gu[r][inter + i]), eight elements per thread.  kNormed: gate and up are
// first multiplied by rsqrt(mean(xn[r]^2) + eps) and rounded to bf16 (the MLP's input norm folded in: the projection
// ran on the un-normalised row through a weight that carries the norm's weight); every workgroup of a row sums the
// row's squares for itself (a few KB from L2).
template <bool kNormed>
__global__ __launch_bounds__(256) void silu_mul_kernel(const __bf16* gu, __bf16* out, int inter, int64_t gu_rs, int64_t out_rs,
                                                       const __bf16* xn, int64_t xn_rs, int xn_cols, float xn_eps) {
    const int r = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 8;
    float rin = 1.0f;
    if constexpr (kNormed) {
        __shared__ float part[4];
        const __bf16* xr = xn + (int64_t)r * xn_rs;
        float ss = 0.f;
        for (int c = threadIdx.x * 8; c < xn_cols; c += 256 * 8) {
            const u32x4 x = *reinterpret_cast<const u32x4*>(xr + c);
#pragma unroll
            for (int q = 0; q < 4; ++q) ss += lo_f(x[q]) * lo_f(x[q]) + hi_f(x[q]) * hi_f(x[q]);
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
        if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = ss;
        __syncthreads();
        ss = (part[0] + part[1]) + (part[2] + part[3]);
        rin = __builtin_amdgcn_rsqf(ss / (float)xn_cols + xn_eps);
    }
    if (i >= inter) return;
    u32x4 g = *reinterpret_cast<const u32x4*>(gu + (int64_t)r * gu_rs + i);
    u32x4 u = *reinterpret_cast<const u32x4*>(gu + (int64_t)r * gu_rs + inter + i);
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        if constexpr (kNormed) {
            g[q] = pack2(lo_f(g[q]) * rin, hi_f(g[q]) * rin);
            u[q] = pack2(lo_f(u[q]) * rin, hi_f(u[q]) * rin);
        }
        const uint32_t s = pack2(silu(lo_f(g[q])), silu(hi_f(g[q])));  // the activation's own bf16 rounding
        o[q] = pack2(lo_f(s) * lo_f(u[q]), hi_f(s) * hi_f(u[q]));
    }
    *reinterpret_cast<u32x4*>(out + (int64_t)r * out_rs + i) = o;
}

// ---------------------------------------------------------------------------
// Greedy step: final logits of a row (first iteration, plus the second for rows that took one, summed in
// bf16 as the model's logits buffers are), their arg-max, and the generation loop's per-row bookkeeping.
// One workgroup per row; the logits are read once (16-byte loads) and never written anywhere.
// ---------------------------------------------------------------------------
constexpr int kGreedyThreads = 1024;

struct GreedyParams {
    const __bf16 *l0, *l1;
    const uint8_t* hard;
    int64_t rs0, rs1;
    int32_t vocab, eos;
    int64_t* tok;
    uint8_t* finished;
    int32_t* pos;
    int64_t* out_tokens;
    int64_t out_stride;
    const int64_t* step_idx;
    int32_t out_cols;
    int32_t* out_len;
    unsigned long long *n_hard, *n_steps;
};

__device__ __forceinline__ void take_better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) {  // ties: the lower vocabulary index
        bv = v;
        bi = i;
    }
}

// Arg-max over a row of logits a[0 .. vocab) -- of bf16(a + b) when b is given (the running sum of the iterations'
// logits lives in the model dtype) -- by the whole workgroup; the lower index among equals.  Valid in thread 0.
__device__ __forceinline__ int row_argmax(const __bf16* a, const __bf16* b, int vocab, float* wv, int* wi) {
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const bool both = b != nullptr;
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
    const int nvec = vocab / 8;
    // ten 16-byte pieces per pass, all loaded before the first is looked at (two passes over a vocabulary of 152 K):
    // 32 workgroups read 19 MB, and what a thread waits for is memory latency
    constexpr int kAhead = 10;
    for (int c0 = tid; c0 < nvec; c0 += kAhead * kGreedyThreads) {
        u32x4 x[kAhead], y[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int c = c0 + u * kGreedyThreads;
            x[u] = y[u] = u32x4{0u, 0u, 0u, 0u};
            if (c < nvec) {
                x[u] = *reinterpret_cast<const u32x4*>(a + 8 * c);
                if (both) y[u] = *reinterpret_cast<const u32x4*>(b + 8 * c);
            }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int c = c0 + u * kGreedyThreads;
            if (c >= nvec) break;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float lo = lo_f(x[u][q]), hi = hi_f(x[u][q]);
                if (both) {
                    const uint32_t s = pack2(lo + lo_f(y[u][q]), hi + hi_f(y[u][q]));
                    lo = lo_f(s);
                    hi = hi_f(s);
                }
                if (lo > bv) { bv = lo; bi = 8 * c + 2 * q; }          // indices ascend inside a thread:
                if (hi > bv) { bv = hi; bi = 8 * c + 2 * q + 1; }      // strict > keeps the first of equals
            }
        }
    }
    for (int i = nvec * 8 + tid; i < vocab; i += kGreedyThreads) {  // a tail that is not a multiple of 8
        float v = (float)a[i];
        if (both) v = (float)(__bf16)(v + (float)b[i]);
        take_better(bv, bi, v, i);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) take_better(bv, bi, __shfl_xor(bv, m), __shfl_xor(bi, m));
    if (lane == 0) {
        wv[wave] = bv;
        wi[wave] = bi;
    }
    __syncthreads();
    if (tid != 0) return 0;
    for (int w = 1; w < kGreedyThreads / kWave; ++w) take_better(bv, bi, wv[w], wi[w]);
    return bi == 0x7fffffff ? 0 : bi;
}

__global__ __launch_bounds__(kGreedyThreads) void greedy_step_kernel(const GreedyParams p) {
    __shared__ float wv[kGreedyThreads / kWave];
    __shared__ int wi[kGreedyThreads / kWave];
    const int row = blockIdx.x, tid = threadIdx.x;
    const bool active = p.finished[row] == 0;  // uniform per workgroup
    const bool both = p.l1 != nullptr && p.hard != nullptr && p.hard[row] != 0;
    int64_t nxt = 0;
    if (active) nxt = row_argmax(p.l0 + (int64_t)row * p.rs0, both ? p.l1 + (int64_t)row * p.rs1 : nullptr, p.vocab, wv, wi);
    if (tid != 0) return;
    // the loop's bookkeeping for this row (tah/model/utils.py:228-262): a row ends with its end-of-sequence token,
    // which is not part of its output; rows that have ended write zeros
    bool done = !active;
    if (active && p.eos >= 0 && nxt == p.eos) done = true;
    const int64_t column = p.step_idx[0];
    const bool room = column >= 0 && column < p.out_cols;  // a step beyond the buffer ends the row instead of writing
    if (!room) done = true;
    p.finished[row] = done ? 1 : 0;
    if (room) p.out_tokens[(int64_t)row * p.out_stride + column] = done ? 0 : nxt;
    if (!done) p.out_len[row] += 1;
    if (active) {
        p.pos[row] += 1;
        atomicAdd(p.n_steps, 1ull);
        if (p.hard != nullptr && p.hard[row] != 0) atomicAdd(p.n_hard, 1ull);
    }
    p.tok[row] = nxt;
}


// ---------------------------------------------------------------------------
// End of a tick of the generation loop in which every row advances by one latent iteration of its own token
// (rows at different iterations share a batch).  phase[row]: 0 = the row just ran the first iteration of a token,
// 1 = the second.  A row whose first iteration was called hard only moves to phase 1; every other active row gets
// its token (arg-max of the first iteration's logits, or of bf16(first + second), the first being the logits the
// previous tick left in `prev`) and the bookkeeping of greedy_step_kernel, with the row's own output column.
// ---------------------------------------------------------------------------
struct TickParams {
    const __bf16 *cur, *prev;
    int64_t rs_cur, rs_prev;
    int32_t vocab, eos, limit;
    const uint8_t* hard_now;
    int32_t* phase;
    int64_t* tok;
    uint8_t* finished;
    int32_t *pos, *out_len, *hard_len;
    int64_t* out_tokens;
    int64_t out_stride;
    unsigned long long *n_hard, *n_steps;
    const int64_t* chosen;
};

__global__ __launch_bounds__(kGreedyThreads) void greedy_tick_kernel(const TickParams p) {
    __shared__ float wv[kGreedyThreads / kWave];
    __shared__ int wi[kGreedyThreads / kWave];
    const int row = blockIdx.x, tid = threadIdx.x;
    const bool ended = p.finished[row] != 0;
    const int ph = p.phase[row];
    const bool again = ph == 0 && p.hard_now[row] != 0;
    __syncthreads();  // every thread has read the row's state before thread 0 changes it: the branches below are uniform
    if (ended) return;
    if (again) {  // the token takes a second iteration: next tick
        if (tid == 0) p.phase[row] = 1;
        return;
    }
    const bool both = ph != 0;
    const int64_t nxt = p.chosen ? p.chosen[row]  // (uniform)
                                 : row_argmax(p.cur + (int64_t)row * p.rs_cur, both ? p.prev + (int64_t)row * p.rs_prev : nullptr, p.vocab, wv, wi);
    if (tid != 0) return;
    // a row ends with its end-of-sequence token, which is not part of its output (tah/model/utils.py:228-262),
    // or when it has `limit` tokens
    bool done = p.eos >= 0 && nxt == p.eos;
    if (!done) {
        const int col = p.out_len[row];
        p.out_tokens[(int64_t)row * p.out_stride + col] = nxt;
        p.out_len[row] = col + 1;
        done = col + 1 >= p.limit;
    }
    p.finished[row] = done ? 1 : 0;
    p.pos[row] += 1;
    p.tok[row] = nxt;
    p.phase[row] = 0;
    atomicAdd(p.n_steps, 1ull);
    if (both) {
        p.hard_len[row] += 1;  // the second iteration's K/V went into the depth-1 slabs during this tick
        atomicAdd(p.n_hard, 1ull);
    }
}

// ---------------------------------------------------------------------------
// Glue of a generation step that would otherwise be a dozen element-wise launches each.
// step_begin: per row, whether it is still active, the cache slot and position it appends and attends at (-1 for
// finished rows), the rotary rows of its position, and its token's embedding row, row-major and in the rows form
// of the linear-layer kernels.  decider_tail: the second layer of the two-layer decider (width -> 1), sigmoid,
// threshold, and the same per-row bookkeeping for the second latent iteration.
// ---------------------------------------------------------------------------
struct StepBeginParams {
    const int64_t* tok;
    const int32_t* pos;
    const uint8_t* finished;
    const __bf16 *embed, *cos_table, *sin_table;
    int64_t embed_rs;
    int32_t vocab, hidden, table_rows;
    __bf16 *x, *x_packed, *cos_rows, *sin_rows;
    int64_t x_rs;
    int32_t *slot, *q_pos;
    uint8_t* active;
    // rows at their second latent iteration (phase[row] != 0) take their input from x_alt instead of the embedding
    const int32_t *phase, *hard_len;
    const __bf16* x_alt;
    int64_t x_alt_rs;
    int32_t *q_depth, *append_at;
    uint8_t* eligible;
};

__global__ __launch_bounds__(256) void step_begin_kernel(const StepBeginParams p) {
    const int row = blockIdx.x, tid = threadIdx.x;
    const bool act = p.finished[row] == 0;
    const int pos = p.pos[row];
    const int ph = p.phase ? (p.phase[row] != 0 ? 1 : 0) : 0;
    if (tid == 0) {
        p.slot[row] = act ? row : -1;
        p.q_pos[row] = act ? pos : -1;
        p.active[row] = act ? 1 : 0;
        if (p.q_depth) p.q_depth[row] = ph;
        if (p.append_at) p.append_at[row] = ph ? p.hard_len[row] : pos;
        if (p.eligible) p.eligible[row] = act && ph == 0 ? 1 : 0;
    }
    const int at = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);  // a position past the tables reads their last row
    if (tid < 16) *reinterpret_cast<u32x4*>(p.cos_rows + (int64_t)row * 128 + 8 * tid) = *reinterpret_cast<const u32x4*>(p.cos_table + (int64_t)at * 128 + 8 * tid);
    else if (tid < 32) *reinterpret_cast<u32x4*>(p.sin_rows + (int64_t)row * 128 + 8 * (tid - 16)) = *reinterpret_cast<const u32x4*>(p.sin_table + (int64_t)at * 128 + 8 * (tid - 16));
    int64_t t = p.tok[row];
    t = t < 0 ? 0 : (t >= p.vocab ? p.vocab - 1 : t);
    const __bf16* e = ph ? p.x_alt + (int64_t)row * p.x_alt_rs : p.embed + t * p.embed_rs;
    for (int c = 8 * tid; c < p.hidden; c += 8 * 256) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(e + c);
        *reinterpret_cast<u32x4*>(p.x + (int64_t)row * p.x_rs + c) = v;
        // unit (step c / 32, half row / 16, lane row % 16 + 16 ((c % 32) / 8)) of the packed rows form
        if (p.x_packed) reinterpret_cast<u32x4*>(p.x_packed)[((int64_t)(c / 32) * 2 + row / 16) * 64 + (row % 16) + 16 * ((c % 32) / 8)] = v;
    }
}

struct DeciderTailParams {
    const __bf16 *h, *w2, *b2;
    int64_t h_rs;
    int32_t width;
    float threshold;
    const uint8_t* active;
    const int32_t* pos;
    uint8_t* hard;
    int32_t *hard_i, *slot, *q_pos;
};

// One wave per row.  z = bf16(h . w2) (float32 sum), + b2 in bf16, sigmoid in float32, > threshold, and active.
__global__ __launch_bounds__(64) void decider_tail_kernel(const DeciderTailParams p) {
    const int row = blockIdx.x, lane = threadIdx.x;
    float s = 0.f;
    for (int c = 8 * lane; c < p.width; c += 8 * 64) {
        const u32x4 a = *reinterpret_cast<const u32x4*>(p.h + (int64_t)row * p.h_rs + c);
        const u32x4 b = *reinterpret_cast<const u32x4*>(p.w2 + c);
#pragma unroll
        for (int q = 0; q < 4; ++q) s += lo_f(a[q]) * lo_f(b[q]) + hi_f(a[q]) * hi_f(b[q]);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) s += __shfl_xor(s, m);
    if (lane != 0) return;
    float z = lo_f(pack2(s, 0.f));
    if (p.b2) z = lo_f(pack2(z + (float)p.b2[0], 0.f));
    const float prob = 1.0f / (1.0f + fast_exp2(-z * kLog2e));
    const bool hard = prob > p.threshold && (p.active == nullptr || p.active[row] != 0);
    p.hard[row] = hard ? 1 : 0;
    if (p.hard_i) p.hard_i[row] = hard ? 1 : 0;
    if (p.slot) p.slot[row] = hard ? row : -1;
    if (p.q_pos) p.q_pos[row] = hard ? p.pos[row] : -1;
}

}  // namespace
}  // namespace tah

extern "C" int tah_greedy_step(const tah_greedy_step_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    if (a->rows < 0 || a->vocab <= 0 || a->rows > 65535 || a->out_cols < 0 || a->out_cols > a->out_stride) return TAH_E_SHAPE;
    if (a->rows == 0) return TAH_OK;
    if (!a->logits0 || !a->tok || !a->finished || !a->pos || !a->out_tokens || !a->step_idx || !a->out_len || !a->n_hard || !a->n_steps)
        return TAH_E_NULL;
    if ((a->logits1 == nullptr) != (a->hard == nullptr)) return TAH_E_NULL;
    if ((reinterpret_cast<uintptr_t>(a->logits0) & 15) || (reinterpret_cast<uintptr_t>(a->logits1) & 15) || a->row_stride0 % 8 ||
        a->row_stride1 % 8)
        return TAH_E_ALIGN;
    GreedyParams p;
    p.l0 = static_cast<const __bf16*>(a->logits0);
    p.l1 = static_cast<const __bf16*>(a->logits1);
    p.hard = a->hard;
    p.rs0 = a->row_stride0; p.rs1 = a->row_stride1;
    p.vocab = a->vocab; p.eos = a->eos;
    p.tok = a->tok; p.finished = a->finished; p.pos = a->pos;
    p.out_tokens = a->out_tokens; p.out_stride = a->out_stride; p.step_idx = a->step_idx; p.out_len = a->out_len;
    p.out_cols = a->out_cols;
    p.n_hard = reinterpret_cast<unsigned long long*>(a->n_hard);
    p.n_steps = reinterpret_cast<unsigned long long*>(a->n_steps);
    hipLaunchKernelGGL(greedy_step_kernel, dim3(a->rows), dim3(kGreedyThreads), 0, static_cast<hipStream_t>(stream), p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_silu_mul_normed(const void* gate_up, void* out, int32_t rows, int32_t inter, int64_t gate_up_row_stride,
                                   int64_t out_row_stride, const void* norm_input, int64_t norm_input_row_stride,
                                   int32_t norm_cols, float norm_eps, tah_stream_t stream) {
    using namespace tah;
    if (rows < 0 || inter < 0 || inter % 8 != 0 || rows > 65535) return TAH_E_SHAPE;
    if (norm_input && (norm_cols <= 0 || norm_cols % 8 != 0 || norm_input_row_stride % 8 != 0)) return TAH_E_SHAPE;
    if (rows == 0 || inter == 0) return TAH_OK;
    if (!gate_up || !out) return TAH_E_NULL;
    if ((reinterpret_cast<uintptr_t>(gate_up) & 15) || (reinterpret_cast<uintptr_t>(out) & 15) || gate_up_row_stride % 8 ||
        out_row_stride % 8 || (reinterpret_cast<uintptr_t>(norm_input) & 15))
        return TAH_E_ALIGN;
    const dim3 grid((inter / 8 + 255) / 256, rows);
    const __bf16* xn = static_cast<const __bf16*>(norm_input);
    if (xn)
        hipLaunchKernelGGL(silu_mul_kernel<true>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const __bf16*>(gate_up),
                           static_cast<__bf16*>(out), inter, gate_up_row_stride, out_row_stride, xn, norm_input_row_stride, norm_cols, norm_eps);
    else
        hipLaunchKernelGGL(silu_mul_kernel<false>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const __bf16*>(gate_up),
                           static_cast<__bf16*>(out), inter, gate_up_row_stride, out_row_stride, xn, (int64_t)0, 0, 0.f);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_silu_mul(const void* gate_up, void* out, int32_t rows, int32_t inter, int64_t gate_up_row_stride,
                            int64_t out_row_stride, tah_stream_t stream) {
    return tah_silu_mul_normed(gate_up, out, rows, inter, gate_up_row_stride, out_row_stride, nullptr, 0, 0, 0.f, stream);
}

extern "C" int tah_step_begin(const tah_step_begin_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    if (a->rows < 0 || a->rows > 65535 || a->vocab <= 0 || a->hidden <= 0 || a->hidden % 8 != 0 || a->table_rows <= 0) return TAH_E_SHAPE;
    if (a->x_packed && (a->rows > 32 || a->hidden % 32 != 0)) return TAH_E_SHAPE;
    if (a->rows == 0) return TAH_OK;
    if (!a->tok || !a->pos || !a->finished || !a->embed || !a->cos_table || !a->sin_table || !a->x || !a->cos_rows || !a->sin_rows ||
        !a->slot || !a->q_pos || !a->active)
        return TAH_E_NULL;
    const void* ptrs[] = {a->embed, a->cos_table, a->sin_table, a->x, a->x_packed, a->cos_rows, a->sin_rows};
    for (const void* q : ptrs)
        if (reinterpret_cast<uintptr_t>(q) & 15) return TAH_E_ALIGN;
    if (a->embed_row_stride % 8 != 0 || a->x_row_stride % 8 != 0) return TAH_E_ALIGN;
    StepBeginParams p;
    p.tok = a->tok; p.pos = a->pos; p.finished = a->finished;
    p.embed = static_cast<const __bf16*>(a->embed);
    p.cos_table = static_cast<const __bf16*>(a->cos_table); p.sin_table = static_cast<const __bf16*>(a->sin_table);
    p.embed_rs = a->embed_row_stride; p.vocab = a->vocab; p.hidden = a->hidden; p.table_rows = a->table_rows;
    p.x = static_cast<__bf16*>(a->x); p.x_packed = static_cast<__bf16*>(a->x_packed);
    p.cos_rows = static_cast<__bf16*>(a->cos_rows); p.sin_rows = static_cast<__bf16*>(a->sin_rows);
    p.x_rs = a->x_row_stride; p.slot = a->slot; p.q_pos = a->q_pos; p.active = a->active;
    p.phase = a->phase; p.hard_len = a->hard_len; p.x_alt = static_cast<const __bf16*>(a->x_alt); p.x_alt_rs = a->x_alt_row_stride;
    p.q_depth = a->q_depth; p.append_at = a->append_at; p.eligible = a->eligible;
    if (p.phase && (!p.x_alt || (p.append_at && !p.hard_len))) return TAH_E_NULL;
    if ((reinterpret_cast<uintptr_t>(a->x_alt) & 15) || a->x_alt_row_stride % 8 != 0) return TAH_E_ALIGN;
    hipLaunchKernelGGL(step_begin_kernel, dim3(a->rows), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_decider_tail(const tah_decider_tail_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    if (a->rows < 0 || a->rows > 65535 || a->width <= 0 || a->width % 8 != 0) return TAH_E_SHAPE;
    if (a->rows == 0) return TAH_OK;
    if (!a->hidden || !a->w2 || !a->hard || (a->q_pos && !a->pos)) return TAH_E_NULL;
    if ((reinterpret_cast<uintptr_t>(a->hidden) & 15) || (reinterpret_cast<uintptr_t>(a->w2) & 15) || a->hidden_row_stride % 8 != 0) return TAH_E_ALIGN;
    DeciderTailParams p;
    p.h = static_cast<const __bf16*>(a->hidden); p.w2 = static_cast<const __bf16*>(a->w2); p.b2 = static_cast<const __bf16*>(a->b2);
    p.h_rs = a->hidden_row_stride; p.width = a->width; p.threshold = a->threshold;
    p.active = a->active; p.pos = a->pos; p.hard = a->hard; p.hard_i = a->hard_i32; p.slot = a->slot; p.q_pos = a->q_pos;
    hipLaunchKernelGGL(decider_tail_kernel, dim3(a->rows), dim3(64), 0, static_cast<hipStream_t>(stream), p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_greedy_tick(const tah_greedy_tick_args* a, tah_stream_t stream) {
    using namespace tah;
    if (!a) return TAH_E_NULL;
    if (a->rows < 0 || a->vocab <= 0 || a->rows > 65535 || a->limit < 0) return TAH_E_SHAPE;
    if (a->rows == 0) return TAH_OK;
    if ((!a->chosen && (!a->logits || !a->logits_prev)) || !a->hard_now || !a->phase || !a->tok || !a->finished || !a->pos || !a->out_tokens || !a->out_len ||
        !a->hard_len || !a->n_hard || !a->n_steps)
        return TAH_E_NULL;
    if ((reinterpret_cast<uintptr_t>(a->logits) & 15) || (reinterpret_cast<uintptr_t>(a->logits_prev) & 15) || a->row_stride % 8 ||
        a->row_stride_prev % 8)
        return TAH_E_ALIGN;
    TickParams p;
    p.cur = static_cast<const __bf16*>(a->logits); p.prev = static_cast<const __bf16*>(a->logits_prev);
    p.rs_cur = a->row_stride; p.rs_prev = a->row_stride_prev;
    p.vocab = a->vocab; p.eos = a->eos; p.limit = a->limit;
    p.hard_now = a->hard_now; p.phase = a->phase; p.tok = a->tok; p.finished = a->finished; p.pos = a->pos;
    p.out_len = a->out_len; p.hard_len = a->hard_len; p.out_tokens = a->out_tokens; p.out_stride = a->out_stride;
    p.n_hard = reinterpret_cast<unsigned long long*>(a->n_hard);
    p.n_steps = reinterpret_cast<unsigned long long*>(a->n_steps);
    p.chosen = a->chosen;
    hipLaunchKernelGGL(greedy_tick_kernel, dim3(a->rows), dim3(kGreedyThreads), 0, static_cast<hipStream_t>(stream), p);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}
