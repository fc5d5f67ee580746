// CPU execution shim for the HIP kernels in this directory tree.  TEST INFRASTRUCTURE ONLY.
//
// Compiling a kernel source with `-I tah_amd/csrc/emu` (so that this file is what
// `#include <hip/hip_runtime.h>` finds) and the host clang++ yields a library with
// the same extern "C" entry points that runs every GPU thread as an OS thread:
// one block at a time, blockDim.x threads, 64-lane waves.  `__syncthreads()` is a
// pthread barrier over the block; wave collectives (MFMA, shuffles, ballots) are
// exchanged through a per-wave mailbox guarded by a per-wave barrier.  Built with
// -fsanitize=address it bounds-checks every global and LDS access of a kernel, and
// with -fsanitize=thread it reports LDS accesses that lack a barrier.  It is never
// loaded by the product package.
//
// MFMA operand layouts modelled here (gfx950, wave64), lane l:
//   32x32x16 bf16: A[i=l%32][k=8*(l/32)+0..7], B[k=8*(l/32)+0..7][j=l%32],
//                  C/D reg r: [i = 8*(r/4) + 4*(l/32) + r%4][j = l%32]
//   16x16x32 bf16: A[i=l%16][k=8*(l/16)+0..7], B[k=8*(l/16)+0..7][j=l%16],
//                  C/D reg r: [i = 4*(l/16) + r][j = l%16]
#pragma once
#include <pthread.h>

#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <tuple>
#include <vector>

#define TAH_CPU_EMU 1
#define TAH_MUL_INPLACE(x, a) ((x) *= (a))
#define TAH_WAIT_VMEM() ((void)0)
#define TAH_WAIT_VMEM_N(n) ((void)0)
#define TAH_KEEP_HERE4(a, b, c, d) ((void)0)
#define TAH_OPAQUE2(a, b) ((void)0)
#define TAH_OPAQUE1(a) ((void)0)
#define TAH_SCALE16_IF(acc, a, cond) \
    do { if (cond) for (int tah_i_ = 0; tah_i_ < 16; ++tah_i_) (acc)[tah_i_] *= (a); } while (0)
#define TAH_ASYNC_COPY_16B(gsrc, lds_wave_base) \
    memcpy((unsigned char*)(lds_wave_base) + 16 * emu::t_lane, (const void*)(gsrc), 16)
#define TAH_ASYNC_COPY_16B_SO(sbase, voff, lds_wave_base) \
    memcpy((unsigned char*)(lds_wave_base) + 16 * emu::t_lane, (const unsigned char*)(sbase) + (voff), 16)
#define TAH_ASYNC_COPY_16B_SO_NT(sbase, voff, lds_wave_base) TAH_ASYNC_COPY_16B_SO(sbase, voff, lds_wave_base)
#define TAH_ASYNC_COPY_4B_SO(sbase, voff, lds_wave_base) \
    memcpy((unsigned char*)(lds_wave_base) + 4 * emu::t_lane, (const unsigned char*)(sbase) + (voff), 4)
#define TAH_ASYNC_COPY_4B(gsrc, lds_wave_base) \
    memcpy((unsigned char*)(lds_wave_base) + 4 * emu::t_lane, (const void*)(gsrc), 4)
#define TAH_WAVES_PER_EU(lo, hi)
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static
#define __align__(n) __attribute__((aligned(n)))

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct emu_idx { unsigned x, y, z; };

typedef int hipError_t;
typedef void* hipStream_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1 };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipPeekAtLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emu"; }
template <class F> inline hipError_t hipFuncSetAttribute(F, hipFuncAttribute, int) { return hipSuccess; }
inline hipError_t hipMemsetAsync(void* p, int v, size_t n, hipStream_t) { memset(p, v, n); return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
#define HIP_SYMBOL(x) (&(x))
inline hipError_t hipGetSymbolAddress(void** p, const void* sym) { *p = const_cast<void*>(sym); return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }

namespace emu {
constexpr int WAVE = 64;
struct WaveCtx {
    pthread_barrier_t bar;
    alignas(16) unsigned char box[WAVE][64];
};
struct BlockCtx {
    pthread_barrier_t bar;
    std::vector<WaveCtx> waves;
    unsigned char* dyn_smem = nullptr;
};
extern thread_local emu_idx t_threadIdx, t_blockIdx;
extern thread_local WaveCtx* t_wave;
extern thread_local int t_lane;
extern dim3 g_blockDim, g_gridDim;
extern BlockCtx* g_block;

#ifdef TAH_EMU_IMPL
thread_local emu_idx t_threadIdx, t_blockIdx;
thread_local WaveCtx* t_wave;
thread_local int t_lane;
dim3 g_blockDim, g_gridDim;
BlockCtx* g_block;
#endif

inline void wave_sync() { pthread_barrier_wait(&t_wave->bar); }

template <class T> inline T exchange(T v, int src) {
    static_assert(sizeof(T) <= 64, "mailbox slot too small");
    memcpy(t_wave->box[t_lane], &v, sizeof(T));
    wave_sync();
    T out;
    memcpy(&out, t_wave->box[src & (WAVE - 1)], sizeof(T));
    wave_sync();
    return out;
}

template <class K, class... Args>
void launch(K kernel, dim3 grid, dim3 block, size_t shmem, Args... args) {
    const unsigned nthr = block.x * block.y * block.z;
    if (block.y != 1 || block.z != 1) { fprintf(stderr, "emu: 1-D blocks only\n"); abort(); }
    BlockCtx ctx;
    const unsigned nwaves = (nthr + WAVE - 1) / WAVE;
    ctx.waves = std::vector<WaveCtx>(nwaves);
    pthread_barrier_init(&ctx.bar, nullptr, nthr);
    for (unsigned w = 0; w < nwaves; ++w) {
        unsigned n = (w + 1) * WAVE <= nthr ? WAVE : nthr - w * WAVE;
        pthread_barrier_init(&ctx.waves[w].bar, nullptr, n);
    }
    // exact-size allocation so that AddressSanitizer sees LDS overruns
    ctx.dyn_smem = shmem ? static_cast<unsigned char*>(aligned_alloc(16, (shmem + 15) / 16 * 16)) : nullptr;
    g_blockDim = block;
    g_gridDim = grid;
    g_block = &ctx;
    auto body = [&](unsigned tid) {
        t_threadIdx = {tid, 0, 0};
        t_wave = &ctx.waves[tid / WAVE];
        t_lane = tid % WAVE;
        for (unsigned bz = 0; bz < grid.z; ++bz)
            for (unsigned by = 0; by < grid.y; ++by)
                for (unsigned bx = 0; bx < grid.x; ++bx) {
                    t_blockIdx = {bx, by, bz};
                    pthread_barrier_wait(&ctx.bar);
                    kernel(args...);
                    pthread_barrier_wait(&ctx.bar);
                }
    };
    std::vector<std::thread> pool;
    pool.reserve(nthr);
    for (unsigned t = 0; t < nthr; ++t) pool.emplace_back(body, t);
    for (auto& th : pool) th.join();
    pthread_barrier_destroy(&ctx.bar);
    for (auto& w : ctx.waves) pthread_barrier_destroy(&w.bar);
    free(ctx.dyn_smem);
    g_block = nullptr;
}
}  // namespace emu

#define threadIdx (emu::t_threadIdx)
#define blockIdx (emu::t_blockIdx)
#define blockDim (emu::g_blockDim)
#define gridDim (emu::g_gridDim)
#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
    emu::launch(kernel, dim3(grid), dim3(block), (size_t)(shmem), ##__VA_ARGS__)
#define TAH_WAVE_LDS_SYNC() emu::wave_sync()
#define TAH_CONST_AS
#define HIP_DYNAMIC_SHARED(type, var) type* var = reinterpret_cast<type*>(emu::g_block->dyn_smem);

inline void __syncthreads() { pthread_barrier_wait(&emu::g_block->bar); }

template <class T> inline T __shfl(T v, int src, int width = 64) {
    int base = emu::t_lane & ~(width - 1);
    return emu::exchange(v, base + (src & (width - 1)));
}
template <class T> inline T __shfl_xor(T v, int mask, int width = 64) {
    (void)width;
    return emu::exchange(v, emu::t_lane ^ mask);
}
template <class T> inline T __shfl_down(T v, unsigned d, int width = 64) {
    int l = emu::t_lane, src = l + (int)d;
    if ((src & ~(width - 1)) != (l & ~(width - 1))) src = l;
    return emu::exchange(v, src);
}
template <class T> inline T __shfl_up(T v, unsigned d, int width = 64) {
    int l = emu::t_lane, src = l - (int)d;
    if (src < 0 || (src & ~(width - 1)) != (l & ~(width - 1))) src = l;
    return emu::exchange(v, src);
}
inline unsigned long long __ballot(int pred) {
    unsigned long long mine = pred ? (1ull << emu::t_lane) : 0ull, all = 0;
    memcpy(emu::t_wave->box[emu::t_lane], &mine, 8);
    emu::wave_sync();
    for (int i = 0; i < emu::WAVE; ++i) {
        unsigned long long x;
        memcpy(&x, emu::t_wave->box[i], 8);
        all |= x;
    }
    emu::wave_sync();
    return all;
}
inline int __popcll(unsigned long long x) { return __builtin_popcountll(x); }
inline int emu_readfirstlane(int v) { return emu::exchange(v, 0); }
#define __builtin_amdgcn_readfirstlane emu_readfirstlane
#define __builtin_amdgcn_ballot_w64(p) __ballot(p)

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 emu_bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float emu_f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float emu_f32x4;

inline emu_f32x16 emu_mfma_32x32x16_bf16(emu_bf16x8 a, emu_bf16x8 b, emu_f32x16 c, int, int, int) {
    struct Slot { emu_bf16x8 a, b; };
    Slot s{a, b};
    memcpy(emu::t_wave->box[emu::t_lane], &s, sizeof(s));
    emu::wave_sync();
    const int l = emu::t_lane, j = l % 32;
    emu_f32x16 d = c;
    for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r / 4) + 4 * (l / 32) + r % 4;
        float acc = 0.f;
        for (int kh = 0; kh < 2; ++kh) {
            Slot sa, sb;
            memcpy(&sa, emu::t_wave->box[i + 32 * kh], sizeof(Slot));
            memcpy(&sb, emu::t_wave->box[j + 32 * kh], sizeof(Slot));
            for (int kk = 0; kk < 8; ++kk) acc += (float)sa.a[kk] * (float)sb.b[kk];
        }
        d[r] += acc;
    }
    emu::wave_sync();
    return d;
}
inline emu_f32x4 emu_mfma_16x16x32_bf16(emu_bf16x8 a, emu_bf16x8 b, emu_f32x4 c, int, int, int) {
    struct Slot { emu_bf16x8 a, b; };
    Slot s{a, b};
    memcpy(emu::t_wave->box[emu::t_lane], &s, sizeof(s));
    emu::wave_sync();
    const int l = emu::t_lane, j = l % 16;
    emu_f32x4 d = c;
    for (int r = 0; r < 4; ++r) {
        const int i = 4 * (l / 16) + r;
        float acc = 0.f;
        for (int kq = 0; kq < 4; ++kq) {
            Slot sa, sb;
            memcpy(&sa, emu::t_wave->box[i + 16 * kq], sizeof(Slot));
            memcpy(&sb, emu::t_wave->box[j + 16 * kq], sizeof(Slot));
            for (int kk = 0; kk < 8; ++kk) acc += (float)sa.a[kk] * (float)sb.b[kk];
        }
        d[r] += acc;
    }
    emu::wave_sync();
    return d;
}
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16 emu_mfma_32x32x16_bf16
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16 emu_mfma_16x16x32_bf16

// v_dot2_f32_bf16 on the raw 32-bit pairs (4-byte bf16 vectors are not passed reliably by value on the host ABI).
inline float emu_bf16_bits(uint32_t hi16) { float f; uint32_t w = hi16 << 16; memcpy(&f, &w, 4); return f; }
inline float emu_fdot2_bits(uint32_t a, uint32_t b, float c) {
    return c + emu_bf16_bits(a & 0xffffu) * emu_bf16_bits(b & 0xffffu) + emu_bf16_bits(a >> 16) * emu_bf16_bits(b >> 16);
}
#define __builtin_amdgcn_fdot2_f32_bf16(a, b, c, clamp) \
    emu_fdot2_bits(__builtin_bit_cast(uint32_t, (a)), __builtin_bit_cast(uint32_t, (b)), (c))
inline unsigned __float_as_uint(float x) { unsigned i; memcpy(&i, &x, 4); return i; }
inline float __uint_as_float(unsigned i) { float x; memcpy(&x, &i, 4); return x; }
// v_permlane32_swap(a, b): lanes < 32 get (a[l], a[l+32]); lanes >= 32 get (b[l-32], b[l]).
struct emu_u32pair { unsigned v[2]; unsigned operator[](int i) const { return v[i]; } };
inline emu_u32pair emu_permlane32_swap(unsigned a, unsigned b, bool, bool) {
    unsigned mine[2] = {a, b};
    memcpy(emu::t_wave->box[emu::t_lane], mine, 8);
    emu::wave_sync();
    const int l = emu::t_lane;
    unsigned lo[2], hi[2];
    memcpy(lo, emu::t_wave->box[l & 31], 8);
    memcpy(hi, emu::t_wave->box[(l & 31) + 32], 8);
    emu::wave_sync();
    return l < 32 ? emu_u32pair{{lo[0], hi[0]}} : emu_u32pair{{lo[1], hi[1]}};
}
#define __builtin_amdgcn_permlane32_swap emu_permlane32_swap
inline int __float_as_int(float x) { int i; memcpy(&i, &x, 4); return i; }
inline float __int_as_float(int i) { float x; memcpy(&x, &i, 4); return x; }
// DPP lane selects used by the kernels: quad_perm, row_shl/shr/ror, row_mirror, row_half_mirror.
inline int emu_update_dpp(int old, int src, int ctrl, int, int, bool bound_ctrl) {
    const int l = emu::t_lane, row = l & ~15, i = l & 15;
    int from = -1;
    if (ctrl < 0x100) from = (l & ~3) + ((ctrl >> (2 * (l & 3))) & 3);
    else if (ctrl >= 0x101 && ctrl <= 0x10f) { int j = i + (ctrl & 15); from = j < 16 ? row + j : -1; }
    else if (ctrl >= 0x111 && ctrl <= 0x11f) { int j = i - (ctrl & 15); from = j >= 0 ? row + j : -1; }
    else if (ctrl >= 0x121 && ctrl <= 0x12f) from = row + ((i - (ctrl & 15)) & 15);  // row_ror
    else if (ctrl == 0x140) from = row + 15 - i;
    else if (ctrl == 0x141) from = row + (i & 8) + 7 - (i & 7);
    else { fprintf(stderr, "emu: unsupported dpp_ctrl 0x%x\n", ctrl); abort(); }
    const int got = emu::exchange(src, from < 0 ? l : from);
    return from < 0 ? (bound_ctrl ? 0 : old) : got;
}
#define __builtin_amdgcn_update_dpp emu_update_dpp

// ds_read_b64_tr_b16: within each group of 16 lanes, the 16 addressed 4-element rows form a flat array
// G[64] (lane-major); lane i of the group receives G[i], G[16+i], G[32+i], G[48+i].
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 emu_bf16x4;
inline uint64_t emu_ds_read_tr16_b64(const void* p) {
    uint16_t mine[4];
    memcpy(mine, p, 8);
    memcpy(emu::t_wave->box[emu::t_lane], mine, 8);
    emu::wave_sync();
    const int l = emu::t_lane, base = l & ~15, i = l & 15;
    uint16_t out[4];
    for (int t = 0; t < 4; ++t) {
        const int flat = 16 * t + i;
        memcpy(&out[t], emu::t_wave->box[base + flat / 4] + 2 * (flat % 4), 2);
    }
    emu::wave_sync();
    uint64_t r;
    memcpy(&r, out, 8);
    return r;
}
#define __builtin_amdgcn_ds_read_tr16_b64_v4bf16(p) \
    __builtin_bit_cast(emu_bf16x4, emu_ds_read_tr16_b64((const void*)(p)))

// global_load_lds: lane l copies `size` bytes from its global address to lds_base + size*l (synchronously here).
#define __builtin_amdgcn_global_load_lds(g, l, size, off, aux) \
    memcpy((unsigned char*)(void*)(l) + (off) + (size) * emu::t_lane, (const void*)(g), (size))

#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_logf(x) log2f(x)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_rsqf(x) (1.0f / sqrtf(x))
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_sched_barrier(a) ((void)0)
#define __builtin_amdgcn_s_setprio(a) ((void)0)
#define __builtin_amdgcn_s_barrier() __syncthreads()

inline int atomicAdd(int* p, int v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }
inline unsigned atomicAdd(unsigned* p, unsigned v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }
inline unsigned long long atomicAdd(unsigned long long* p, unsigned long long v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }
inline float atomicAdd(float* p, float v) {
    float old, upd;
    __atomic_load(p, &old, __ATOMIC_RELAXED);
    do { upd = old + v; } while (!__atomic_compare_exchange(p, &old, &upd, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED));
    return old;
}
inline int atomicMax(int* p, int v) {
    int old = __atomic_load_n(p, __ATOMIC_RELAXED);
    while (old < v && !__atomic_compare_exchange_n(p, &old, v, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) {}
    return old;
}
inline void __threadfence() { __atomic_thread_fence(__ATOMIC_SEQ_CST); }
