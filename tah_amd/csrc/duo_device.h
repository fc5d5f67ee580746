// Device-side helpers shared by the duo-causal attention kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tah {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

// LDS addressed through pointers that carry the LDS address space and start at LDS address 0.  A kernel that
// declares no static LDS object has its dynamic LDS at address 0; a pointer made from that integer (instead of
// the extern array's symbol, whose zero the compiler only learns after instruction selection) lets constant
// parts of an offset fold into the instructions' immediate fields -- no `v_add_u32 v, 0, v` per access -- and
// needs no generic-to-LDS conversion (a compare and a select each) where an address goes into m0.
#ifdef TAH_CPU_EMU
typedef unsigned char lds_byte;
typedef float lds_float;
typedef int lds_int;
#define TAH_LDS_ZERO_BASED(name, decl) unsigned char* const name = decl
#define TAH_LDS_CAST(T, p) (reinterpret_cast<T*>(p))
#else
typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef __attribute__((address_space(3))) float lds_float;
typedef __attribute__((address_space(3))) int lds_int;
#define TAH_LDS_ZERO_BASED(name, decl) \
    tah::lds_byte* const name = reinterpret_cast<tah::lds_byte*>(static_cast<uintptr_t>(0)); (void)decl
#define TAH_LDS_CAST(T, p) (reinterpret_cast<__attribute__((address_space(3))) T*>(p))
#endif

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegInf = -__builtin_inff();

// v_mfma_f32_32x32x16_bf16: D(32x32) += A(32x16) * B(16x32).
// lane l: A[i = l%32][k = 8*(l/32) + 0..7], B[k = 8*(l/32) + 0..7][j = l%32],
// D reg r: [i = 8*(r/4) + 4*(l/32) + r%4][j = l%32].
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Row index inside a 32-row MFMA accumulator tile held by (lane half h, reg r).
__device__ __forceinline__ constexpr int acc_row(int h, int r) { return 8 * (r / 4) + 4 * h + (r % 4); }

// x *= a with the product forced into x's own register, so that an accumulator rescaled inside a
// rarely taken branch is not copied to a second register set on the common path.
#ifndef TAH_MUL_INPLACE
#define TAH_MUL_INPLACE(x, a) asm volatile("v_mul_f32 %0, %1, %0" : "+v"(x) : "v"(a))
#endif

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

__device__ __forceinline__ bf16x8 ld_global_16B(const __bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ void st_global_16B(__bf16* p, bf16x8 v) { *reinterpret_cast<bf16x8*>(p) = v; }

// Asynchronous global -> LDS copy of 16 bytes per lane (global_load_lds_dwordx4): lane l's bytes
// land at lds_wave_base + 16*l; lds_wave_base must be wave-uniform.  Issued through inline
// assembly on purpose: the compiler then does not order later LDS reads of *other* tiles behind
// this copy (it cannot prove they do not alias and would wait for vmcnt(0) in the middle of the
// compute phase).  Completion is tracked by vmcnt: TAH_WAIT_VMEM() before the barrier that
// publishes the tile.
#ifndef TAH_ASYNC_COPY_16B
#define TAH_ASYNC_COPY_16B(gsrc, lds_wave_base)                                                                    \
    do {                                                                                                           \
        const unsigned tah_m0_ = __builtin_amdgcn_readfirstlane(                                                   \
            (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)(lds_wave_base));                        \
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"                             \
                     :                                                                                             \
                     : "s"(tah_m0_), "v"(gsrc)                                                                     \
                     : "memory");  /* m0 is reserved: the compiler reloads it before each own use */                                                                            \
    } while (0)
#endif
__device__ __forceinline__ void async_copy_16B(const void* gsrc, unsigned char* lds_wave_base) {
    TAH_ASYNC_COPY_16B(gsrc, lds_wave_base);
}
// Same copy addressed as wave-uniform base + per-lane 32-bit byte offset: the base lives in scalar
// registers and advances with scalar arithmetic, the lane offsets can be loop invariant.
#ifndef TAH_ASYNC_COPY_16B_SO
#define TAH_ASYNC_COPY_16B_SO(sbase, voff, lds_wave_base)                                                          \
    do {                                                                                                           \
        const unsigned tah_m0_ = __builtin_amdgcn_readfirstlane(                                                   \
            (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)(lds_wave_base));                        \
        const uint64_t tah_b_ = (uint64_t)(uintptr_t)(sbase);                                                      \
        /* the builtin returns int: narrow to 32 bits unsigned before widening, or bit 31 smears upward */      \
        const uint64_t tah_sb_ = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((unsigned)tah_b_) |            \
                                 ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((unsigned)(tah_b_ >> 32)) << 32); \
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"                              \
                     :                                                                                             \
                     : "s"(tah_m0_), "v"(voff), "s"(tah_sb_)                                                       \
                     : "memory");                                                                                  \
    } while (0)
#endif
__device__ __forceinline__ void async_copy_16B(const void* sbase, uint32_t voff, unsigned char* lds_wave_base) {
    TAH_ASYNC_COPY_16B_SO(sbase, voff, lds_wave_base);
}
// The same copy for data that is read once (streaming: the lines are not kept in the L2).
#ifndef TAH_ASYNC_COPY_16B_SO_NT
#define TAH_ASYNC_COPY_16B_SO_NT(sbase, voff, lds_wave_base)                                                       \
    do {                                                                                                           \
        const unsigned tah_m0_ = __builtin_amdgcn_readfirstlane(                                                   \
            (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)(lds_wave_base));                        \
        const uint64_t tah_b_ = (uint64_t)(uintptr_t)(sbase);                                                      \
        const uint64_t tah_sb_ = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((unsigned)tah_b_) |            \
                                 ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((unsigned)(tah_b_ >> 32)) << 32); \
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"                           \
                     :                                                                                             \
                     : "s"(tah_m0_), "v"(voff), "s"(tah_sb_)                                                       \
                     : "memory");                                                                                  \
    } while (0)
#endif
__device__ __forceinline__ void async_copy_16B_stream(const void* sbase, uint32_t voff, unsigned char* lds_wave_base) {
    TAH_ASYNC_COPY_16B_SO_NT(sbase, voff, lds_wave_base);
}
#ifndef TAH_CPU_EMU
__device__ __forceinline__ void async_copy_16B_stream(const void* sbase, uint32_t voff, lds_byte* lds_wave_base) {
    TAH_ASYNC_COPY_16B_SO_NT(sbase, voff, lds_wave_base);
}
#endif
// Same with 4 bytes per lane (global_load_lds_dword): lane l's dword lands at lds_wave_base + 4*l.
#ifndef TAH_ASYNC_COPY_4B
#define TAH_ASYNC_COPY_4B(gsrc, lds_wave_base)                                                                     \
    do {                                                                                                           \
        const unsigned tah_m0_ = __builtin_amdgcn_readfirstlane(                                                   \
            (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)(lds_wave_base));                        \
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"                               \
                     :                                                                                             \
                     : "s"(tah_m0_), "v"(gsrc)                                                                     \
                     : "memory");                                                                                  \
    } while (0)
#endif
__device__ __forceinline__ void async_copy_4B(const void* gsrc, void* lds_wave_base) {
    TAH_ASYNC_COPY_4B(gsrc, lds_wave_base);
}
// 4 bytes per lane from wave-uniform base + per-lane 32-bit byte offset.
#ifndef TAH_ASYNC_COPY_4B_SO
#define TAH_ASYNC_COPY_4B_SO(sbase, voff, lds_wave_base)                                                           \
    do {                                                                                                           \
        const unsigned tah_m0_ = __builtin_amdgcn_readfirstlane(                                                   \
            (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)(lds_wave_base));                        \
        const uint64_t tah_b_ = (uint64_t)(uintptr_t)(sbase);                                                      \
        const uint64_t tah_sb_ = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((unsigned)tah_b_) |            \
                                 ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((unsigned)(tah_b_ >> 32)) << 32); \
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"                                \
                     :                                                                                             \
                     : "s"(tah_m0_), "v"(voff), "s"(tah_sb_)                                                       \
                     : "memory");                                                                                  \
    } while (0)
#endif
__device__ __forceinline__ void async_copy_4B(const void* sbase, uint32_t voff, void* lds_wave_base) {
    TAH_ASYNC_COPY_4B_SO(sbase, voff, lds_wave_base);
}
#ifndef TAH_CPU_EMU
// the same copies with the destination given as an LDS-address-space pointer
__device__ __forceinline__ void async_copy_16B(const void* sbase, uint32_t voff, lds_byte* lds_wave_base) {
    TAH_ASYNC_COPY_16B_SO(sbase, voff, lds_wave_base);
}
__device__ __forceinline__ void async_copy_4B(const void* sbase, uint32_t voff, lds_float* lds_wave_base) {
    TAH_ASYNC_COPY_4B_SO(sbase, voff, lds_wave_base);
}
#endif
// acc (16 floats of an MFMA accumulator) *= a, executed only if the wave-uniform `cond` is non-zero.
// The branch lives inside the assembly so that the compiler sees one unconditional in-place update:
// a C++ `if` around accumulator updates makes it keep two copies of the accumulators.
#ifndef TAH_SCALE16_IF
#define TAH_SCALE16_IF(acc, a, cond)                                                                               \
    asm volatile(                                                                                                  \
        "s_cmp_eq_u32 %[cd], 0\n\t"                                                                                \
        "s_cbranch_scc1 .Ltah_skip_%=\n\t"                                                                         \
        "v_mul_f32 %[o0], %[al], %[o0]\n\tv_mul_f32 %[o1], %[al], %[o1]\n\t"                                       \
        "v_mul_f32 %[o2], %[al], %[o2]\n\tv_mul_f32 %[o3], %[al], %[o3]\n\t"                                       \
        "v_mul_f32 %[o4], %[al], %[o4]\n\tv_mul_f32 %[o5], %[al], %[o5]\n\t"                                       \
        "v_mul_f32 %[o6], %[al], %[o6]\n\tv_mul_f32 %[o7], %[al], %[o7]\n\t"                                       \
        "v_mul_f32 %[o8], %[al], %[o8]\n\tv_mul_f32 %[o9], %[al], %[o9]\n\t"                                       \
        "v_mul_f32 %[o10], %[al], %[o10]\n\tv_mul_f32 %[o11], %[al], %[o11]\n\t"                                   \
        "v_mul_f32 %[o12], %[al], %[o12]\n\tv_mul_f32 %[o13], %[al], %[o13]\n\t"                                   \
        "v_mul_f32 %[o14], %[al], %[o14]\n\tv_mul_f32 %[o15], %[al], %[o15]\n"                                     \
        ".Ltah_skip_%=:"                                                                                           \
        : [o0] "+v"((acc)[0]), [o1] "+v"((acc)[1]), [o2] "+v"((acc)[2]), [o3] "+v"((acc)[3]),                      \
          [o4] "+v"((acc)[4]), [o5] "+v"((acc)[5]), [o6] "+v"((acc)[6]), [o7] "+v"((acc)[7]),                      \
          [o8] "+v"((acc)[8]), [o9] "+v"((acc)[9]), [o10] "+v"((acc)[10]), [o11] "+v"((acc)[11]),                  \
          [o12] "+v"((acc)[12]), [o13] "+v"((acc)[13]), [o14] "+v"((acc)[14]), [o15] "+v"((acc)[15])               \
        : [al] "v"(a), [cd] "s"(cond)                                                                              \
        : "scc")
#endif
// Empty statement that counts as a use of four register values at this point of the program.
#ifndef TAH_KEEP_HERE4
#define TAH_KEEP_HERE4(a, b, c, d) asm volatile("" ::"v"(a), "v"(b), "v"(c), "v"(d))
#endif
// Makes two register values opaque to the optimiser at this point, so that what is derived from them
// afterwards is computed here (and not hoisted out of a loop into registers of its own).
#ifndef TAH_OPAQUE2
#define TAH_OPAQUE2(a, b) asm volatile("" : "+v"(a), "+v"(b))
#endif
#ifndef TAH_OPAQUE1
#define TAH_OPAQUE1(a) asm volatile("" : "+v"(a))
#endif
// Occupancy the kernel is written for; lets the scheduler spend registers on latency hiding.
// Between LDS writes of a wave and reads, by the same wave, of what its other lanes wrote: the lanes run
// in lockstep and the LDS serves a wave's requests in order, so all that is needed is that the compiler
// keeps the accesses in program order.
#ifndef TAH_WAVE_LDS_SYNC
#define TAH_WAVE_LDS_SYNC()                                      \
    do {                                                         \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   \
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");   \
    } while (0)
#endif
#ifndef TAH_WAVES_PER_EU
#define TAH_WAVES_PER_EU(lo, hi) __attribute__((amdgpu_waves_per_eu(lo, hi)))
#endif
#ifndef TAH_WAIT_VMEM
// s_waitcnt vmcnt(0) (expcnt/lgkmcnt untouched) as a builtin, so the compiler's own wait-count
// bookkeeping also learns that no ordinary load is pending past this point.
#define TAH_WAIT_VMEM() __builtin_amdgcn_s_waitcnt(0x0F70)
#endif
#ifndef TAH_WAIT_VMEM_N
// s_waitcnt vmcnt(n), n <= 15: all but the n most recently issued loads / asynchronous copies have landed
#define TAH_WAIT_VMEM_N(n) __builtin_amdgcn_s_waitcnt(0x0F70 | (n))
#endif

// LDS tile of R rows x 128 bf16 (256 B per row, 16 chunks of 16 B).  The chunk index is XORed
// with a 4-bit function of the row that (a) takes 16 different values over 16 consecutive rows,
// so 16 lanes reading the same logical chunk of consecutive rows (MFMA A operand, b128) touch 16
// different bank groups, and (b) moves 4 consecutive rows into 4 different aligned groups of 4
// chunks, so a transpose read (4 rows x 64 contiguous bytes per half-wave) is conflict-free too.
__device__ __forceinline__ constexpr int row_swizzle(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
__device__ __forceinline__ int rowmajor128_off(int row, int chunk) { return row * 256 + ((chunk ^ row_swizzle(row)) << 4); }

// LDS tile of R rows x 64 bf16 (128 B per row, 8 chunks of 16 B), swizzled likewise.
__device__ __forceinline__ int rowmajor64_off(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

// ds_read_b64_tr_b16: each lane supplies the LDS address of 4 consecutive bf16 (a row fragment).
// Within each group of 16 lanes the fragments form a flat array G[64] in lane order and lane i
// of the group receives G[i], G[16+i], G[32+i], G[48+i].  With lane r of the group pointing at
// element [row0 + r/4][col0 + 4*(r%4)] of a row-major tile, lane i ends up with
// [row0 + t][col0 + i] for t = 0..3: four rows of one column, i.e. a transposed fragment.
__device__ __forceinline__ bf16x4 lds_read_tr16(const unsigned char* p) {
    typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
    return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)p);
}
#ifndef TAH_CPU_EMU
__device__ __forceinline__ bf16x4 lds_read_tr16(const lds_byte* p) {
    typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
    return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)p);
}
#endif

// MFMA operand whose contraction index runs over the ROWS of a row-major [rows][128] bf16 LDS
// tile (rowmajor128_off layout): returns, for this lane, the 8 values
// tile[row16 + 8*a + 4*half + b][col32 + lane%32], a = 0..1, b = 0..3, in slot order 4*a + b --
// the slot order in which a 32x32 accumulator (lane half, reg) enumerates its rows, so that an
// accumulator converted to bf16 is directly the other operand of the same MFMA.
__device__ __forceinline__ bf16x8 lds_read_rows_as_k(const unsigned char* tile, int row16, int col32, int lane) {
    const int half = lane >> 5, r = lane & 15, grp = (lane >> 4) & 1;
    const int col = col32 + 16 * grp + 4 * (r & 3);
    const int row = row16 + 4 * half + (r >> 2);
    const bf16x4 lo = lds_read_tr16(tile + rowmajor128_off(row, col >> 3) + (col & 7) * 2);
    const bf16x4 hi = lds_read_tr16(tile + rowmajor128_off(row + 8, col >> 3) + (col & 7) * 2);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Storage slot of key `key` (0..63) inside a transposed 64-key row.  The PV
// MFMA contracts over keys; operand slot (half h, j) of 16-key step s must hold
// the same key as S^T accumulator (half h, reg 8*(s%2)+j), i.e. key
// 16s + 8*(j/4) + 4h + j%4.  Storing key 16s+8a+4h+b at slot 16s+8h+4a+b makes
// each lane's 8 operand keys one contiguous 16-byte chunk.
__device__ __forceinline__ constexpr int pv_slot(int key) {
    return (key & ~12) | ((key & 4) << 1) | ((key & 8) >> 1);
}

// max over the two lanes l and l^32 (v_permlane32_swap: no LDS traffic)
__device__ __forceinline__ float wave_max_xor32(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float wave_sum_xor32(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ int wave_reduce_max(int x) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) { int y = __shfl_xor(x, m); x = x > y ? x : y; }
    return x;
}
__device__ __forceinline__ int wave_reduce_min(int x) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) { int y = __shfl_xor(x, m); x = x < y ? x : y; }
    return x;
}

// Element i of an int32 array that no kernel of this library writes (sequence boundaries), read with
// a wave-uniform index: through the constant address space, i.e. with a scalar load when the address is
// uniform — a fraction of the latency of a vector load, which matters in the serial walk over the
// boundaries at the start of a workgroup.
#ifndef TAH_CONST_AS
#define TAH_CONST_AS __attribute__((address_space(4)))
#endif
__device__ __forceinline__ int32_t const_i32(const int32_t* a, int i) { return ((const TAH_CONST_AS int32_t*)a)[i]; }

// Locate tile `slot` among sequences whose lengths are cu[b+1]-cu[b], `bm` rows
// per tile.  On success fills seq/row0/row_end and returns true; otherwise
// subtracts the number of tiles in this stream from `slot` and returns false.
// Every lane of the wave must call it with the same arguments: the lanes take 64 sequences at a time (one pair of
// loads and a prefix sum over the lanes), so that a batch of hundreds of short sequences costs a workgroup a few
// steps and not one scalar load pair per sequence.
__device__ __forceinline__ bool find_tile(const int32_t* cu, int nseq, int bm, int& slot, int& seq, int& row0, int& row_end) {
    const int lane = (int)(threadIdx.x % kWave);
    for (int b0 = 0; b0 < nseq; b0 += kWave) {
        const int b = b0 + lane;
        int lo = 0, hi = 0;
        if (b < nseq) {
            lo = cu[b];
            hi = cu[b + 1];
        }
        const int n = (hi - lo + bm - 1) / bm;
        int incl = n;  // tiles of sequences b0 .. b
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
            const int v = __shfl_up(incl, o);
            if (lane >= o) incl += v;
        }
        const int tot = __builtin_amdgcn_readfirstlane(__shfl(incl, kWave - 1));
        if (slot < tot) {
            const int src = __builtin_ctzll(__ballot(slot < incl));  // the first sequence whose tiles reach past `slot`
            const int lo_s = __builtin_amdgcn_readfirstlane(__shfl(lo, src));
            const int hi_s = __builtin_amdgcn_readfirstlane(__shfl(hi, src));
            const int before = __builtin_amdgcn_readfirstlane(__shfl(incl - n, src));
            seq = b0 + src;
            row0 = lo_s + (slot - before) * bm;
            row_end = row0 + bm < hi_s ? row0 + bm : hi_s;
            return true;
        }
        slot -= tot;
    }
    return false;
}

// ---------------------------------------------------------------------------
// Launch-order table of a varlen call (built by tah_duo_schedule_build): the tiles of both depths sorted
// by the number of tile steps they run, heaviest first, so that a launch of few, unequal workgroups per
// compute unit ends with the light ones.  int32 words: a header, then one (x, y) pair per launch slot of
// the query-tile kernels (forward, dQ), then one pair per slot of the key-tile kernel (dK/dV).
//   x = the tile's number in the order find_tile counts them (the depth-0 stream's tiles sequence by sequence, then
//       the depth-1 stream's); y = 0 (reserved).
// Every number below the list's length appears exactly once (those past the last tile at the end), so whatever
// boundaries a call has, walking the list visits each of its tiles once: a table built for other boundaries of the
// same sizes costs the intended order, never a tile.
// ---------------------------------------------------------------------------
constexpr int32_t kSchedMagic = 0x54414853;
constexpr int kSchedHeaderWords = 16;
enum { kSchedNseq = 1, kSchedGroup, kSchedTotalQ1, kSchedTotalQ2, kSchedTotalK1, kSchedTotalK2, kSchedQSlots, kSchedKSlots };
constexpr int kSchedKeyTile = 128;  // keys per workgroup of the dK/dV kernel

// launch slots of a kernel that tiles the rows of both streams by `bm` (an upper bound on
// sum_b ceil(len_b / bm) that needs no device read)
inline __host__ __device__ int sched_slots(int nseq, int bm, int total_1, int total_2) {
    return (total_1 > 0 ? total_1 / bm + nseq : 0) + (total_2 > 0 ? total_2 / bm + nseq : 0);
}

// The tile number that launch slot `idx` takes from the table, if the table was built for this call's sizes and this
// kernel's grid (true); otherwise the caller keeps its own order (false).
__device__ __forceinline__ bool sched_lookup(const int32_t* sched, bool key_tiles, int nseq, int group, int total_q1,
                                             int total_q2, int total_k1, int total_k2, int slots, int idx, int& slot) {
    if (!sched) return false;
    if (const_i32(sched, 0) != kSchedMagic || const_i32(sched, kSchedNseq) != nseq || const_i32(sched, kSchedGroup) != group ||
        const_i32(sched, kSchedTotalQ1) != total_q1 || const_i32(sched, kSchedTotalQ2) != total_q2 ||
        const_i32(sched, kSchedTotalK1) != total_k1 || const_i32(sched, kSchedTotalK2) != total_k2 ||
        const_i32(sched, key_tiles ? kSchedKSlots : kSchedQSlots) != slots)
        return false;
    const int base = kSchedHeaderWords + (key_tiles ? 2 * const_i32(sched, kSchedQSlots) : 0);
    const int x = const_i32(sched, base + 2 * idx);
    if (x < 0 || x >= slots) return false;  // (not a table this library wrote)
    slot = x;
    return true;
}

}  // namespace tah
