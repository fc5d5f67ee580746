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

// out[r][i] = bf16(bf16(silu(gu[r][i])) * gu[r][inter + i]), eight elements per thread
__global__ __launch_bounds__(256) void silu_mul_kernel(const __bf16* gu, __bf16* out, int inter, int64_t gu_rs, int64_t out_rs) {
    const int r = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= inter) return;
    const u32x4 g = *reinterpret_cast<const u32x4*>(gu + (int64_t)r * gu_rs + i);
    const u32x4 u = *reinterpret_cast<const u32x4*>(gu + (int64_t)r * gu_rs + inter + i);
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t s = pack2(silu(lo_f(g[q])), silu(hi_f(g[q])));  // the activation's own bf16 rounding
        o[q] = pack2(lo_f(s) * lo_f(u[q]), hi_f(s) * hi_f(u[q]));
    }
    *reinterpret_cast<u32x4*>(out + (int64_t)r * out_rs + i) = o;
}

}  // namespace
}  // namespace tah

extern "C" int tah_silu_mul(const void* gate_up, void* out, int32_t rows, int32_t inter, int64_t gate_up_row_stride,
                            int64_t out_row_stride, tah_stream_t stream) {
    using namespace tah;
    if (rows < 0 || inter < 0 || inter % 8 != 0 || rows > 65535) return TAH_E_SHAPE;
    if (rows == 0 || inter == 0) return TAH_OK;
    if (!gate_up || !out) return TAH_E_NULL;
    if ((reinterpret_cast<uintptr_t>(gate_up) & 15) || (reinterpret_cast<uintptr_t>(out) & 15) || gate_up_row_stride % 8 ||
        out_row_stride % 8)
        return TAH_E_ALIGN;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((inter / 8 + 255) / 256, rows), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const __bf16*>(gate_up), static_cast<__bf16*>(out), inter, gate_up_row_stride, out_row_stride);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}
