// Hard-token index build and row gather/scatter (integer / byte work, exact).
//
// The index build is a single-workgroup stream compaction: 1024 threads, each
// owning 16 consecutive mask bytes per pass, a wave-shuffle + LDS block scan per
// pass, and a running carry.  Row-major order of the True entries is the packing
// order the model's forward loop uses for iteration-2 rows.
#include <hip/hip_runtime.h>

#include "duo_device.h"
#include "tah_duo.h"

namespace tah {
namespace {

constexpr int kScanThreads = 1024;
constexpr int kPerThread = 16;

__global__ __launch_bounds__(kScanThreads) void hard_index_kernel(const uint8_t* mask, int B, int S, int32_t* pos_out,
                                                                  int32_t* flat_out, int32_t* seq_out, int32_t* cu_out) {
    __shared__ int wave_tot[kScanThreads / kWave];
    __shared__ int carry_s;
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int64_t total = (int64_t)B * S;
    if (tid == 0) carry_s = 0;
    // a mask without columns has no element (b, 0) to carry a row's boundary: every boundary is 0
    if (S == 0)
        for (int b = tid; b < B; b += kScanThreads) cu_out[b] = 0;
    __syncthreads();
    for (int64_t chunk = 0; chunk < total; chunk += (int64_t)kScanThreads * kPerThread) {
        const int64_t f0 = chunk + (int64_t)tid * kPerThread;
        uint8_t m[kPerThread];
        int cnt = 0;
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            m[i] = (f0 + i < total) ? mask[f0 + i] : 0;
            cnt += m[i] != 0;
        }
        // inclusive scan of cnt across the wave, then across waves
        int inc = cnt;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const int y = __shfl_up(inc, d);
            if (lane >= d) inc += y;
        }
        if (lane == kWave - 1) wave_tot[wave] = inc;
        __syncthreads();
        int wave_off = 0;
        for (int w = 0; w < wave; ++w) wave_off += wave_tot[w];
        int chunk_total = 0;
        for (int w = 0; w < kScanThreads / kWave; ++w) chunk_total += wave_tot[w];
        const int carry = carry_s;
        int run = carry + wave_off + inc - cnt;  // True entries before flat index f0
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const int64_t f = f0 + i;
            if (f < total) {
                const int b = (int)(f / S), s = (int)(f - (int64_t)b * S);
                if (s == 0) cu_out[b] = run;
                if (m[i]) {
                    if (pos_out) pos_out[run] = s;
                    if (flat_out) flat_out[run] = (int32_t)f;
                    if (seq_out) seq_out[run] = b;
                    ++run;
                }
            }
        }
        __syncthreads();
        if (tid == 0) carry_s = carry + chunk_total;
        __syncthreads();
    }
    if (tid == 0) cu_out[B] = carry_s;
}

__global__ void pad_rows_kernel(const int32_t* cu, const int32_t* seq_of, int n, const int32_t* n_dev, int width,
                                int32_t* out, int32_t* overflow) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (n_dev && *n_dev < n) n = *n_dev;
    if (r < n) {
        const int b = seq_of[r];
        const int rank = r - cu[b];
        out[r] = rank < width ? b * width + rank : -1;  // an entry that does not fit its row is dropped by the copy
        if (rank >= width && overflow) *overflow = 1;
    }
}

template <typename V>
__global__ void rows_copy_kernel(const unsigned char* src, const int32_t* src_rows, unsigned char* dst,
                                 const int32_t* dst_rows, const uint8_t* dst_enable, int n, const int32_t* n_dev,
                                 int vec_per_row, int64_t src_stride, int64_t dst_stride, int row_base) {
    const int r = blockIdx.y;
    if (r >= n || (n_dev && row_base + r >= *n_dev)) return;
    const int64_t sr = src_rows ? src_rows[r] : row_base + r;
    const int64_t dr = dst_rows ? dst_rows[r] : row_base + r;
    if (sr < 0 || dr < 0) return;  // dropped entry (see pad_rows_kernel)
    if (dst_enable && !dst_enable[dr]) return;
    const V* s = reinterpret_cast<const V*>(src + sr * src_stride);
    V* d = reinterpret_cast<V*>(dst + dr * dst_stride);
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < vec_per_row; i += gridDim.x * blockDim.x) d[i] = s[i];
}

struct alignas(16) V16 { uint32_t x[4]; };

template <typename V>
int launch_copy(const void* src, const int32_t* src_rows, void* dst, const int32_t* dst_rows, const uint8_t* dst_enable, int n,
                const int32_t* n_dev, int64_t row_bytes, int64_t src_stride, int64_t dst_stride, hipStream_t st) {
    const int vec = (int)(row_bytes / (int64_t)sizeof(V));
    int gx = (vec + 255) / 256;
    gx = gx < 1 ? 1 : (gx > 64 ? 64 : gx);
    for (int r0 = 0; r0 < n; r0 += 65535) {  // grid.y limit
        const int nr = n - r0 < 65535 ? n - r0 : 65535;
        hipLaunchKernelGGL(rows_copy_kernel<V>, dim3(gx, nr), dim3(256), 0, st, static_cast<const unsigned char*>(src),
                           src_rows ? src_rows + r0 : nullptr, static_cast<unsigned char*>(dst),
                           dst_rows ? dst_rows + r0 : nullptr, dst_enable, nr, n_dev, vec, src_stride, dst_stride, r0);
    }
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

}  // namespace
}  // namespace tah

extern "C" int tah_hard_index_build(const uint8_t* mask, int32_t B, int32_t S, int32_t* pos_out, int32_t* flat_out,
                                    int32_t* seq_out, int32_t* cu_out, tah_stream_t stream) {
    using namespace tah;
    if (B < 0 || S < 0) return TAH_E_SHAPE;
    if (!cu_out || (!mask && (int64_t)B * S > 0)) return TAH_E_NULL;
    if ((int64_t)B * S >= (int64_t)1 << 31) return TAH_E_SHAPE;
    hipLaunchKernelGGL(hard_index_kernel, dim3(1), dim3(kScanThreads), 0, static_cast<hipStream_t>(stream), mask, B, S,
                       pos_out, flat_out, seq_out, cu_out);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_pad_rows_build(const int32_t* cu, const int32_t* seq_of, int32_t n, const int32_t* n_dev, int32_t width,
                                  int32_t* out, int32_t* overflow, tah_stream_t stream) {
    using namespace tah;
    if (n < 0 || width < 0) return TAH_E_SHAPE;
    if (n == 0) return TAH_OK;
    if (!cu || !seq_of || !out) return TAH_E_NULL;
    hipLaunchKernelGGL(pad_rows_kernel, dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), cu, seq_of, n,
                       n_dev, width, out, overflow);
    return hipGetLastError() == hipSuccess ? TAH_OK : TAH_E_LAUNCH;
}

extern "C" int tah_rows_copy(const void* src, const int32_t* src_rows, void* dst, const int32_t* dst_rows,
                             const uint8_t* dst_enable, int32_t n, const int32_t* n_dev, int64_t row_bytes,
                             int64_t src_stride_bytes, int64_t dst_stride_bytes, tah_stream_t stream) {
    using namespace tah;
    if (n < 0 || row_bytes < 0) return TAH_E_SHAPE;
    if (n == 0 || row_bytes == 0) return TAH_OK;
    if (!src || !dst) return TAH_E_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uintptr_t bits = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | (uintptr_t)row_bytes |
                           (uintptr_t)src_stride_bytes | (uintptr_t)dst_stride_bytes;
    if (bits % 16 == 0) return launch_copy<V16>(src, src_rows, dst, dst_rows, dst_enable, n, n_dev, row_bytes, src_stride_bytes, dst_stride_bytes, st);
    if (bits % 8 == 0) return launch_copy<uint64_t>(src, src_rows, dst, dst_rows, dst_enable, n, n_dev, row_bytes, src_stride_bytes, dst_stride_bytes, st);
    if (bits % 4 == 0) return launch_copy<uint32_t>(src, src_rows, dst, dst_rows, dst_enable, n, n_dev, row_bytes, src_stride_bytes, dst_stride_bytes, st);
    if (bits % 2 == 0) return launch_copy<uint16_t>(src, src_rows, dst, dst_rows, dst_enable, n, n_dev, row_bytes, src_stride_bytes, dst_stride_bytes, st);
    return launch_copy<uint8_t>(src, src_rows, dst, dst_rows, dst_enable, n, n_dev, row_bytes, src_stride_bytes, dst_stride_bytes, st);
}

extern "C" int tah_duo_abi_version(void) { return TAH_DUO_ABI_VERSION; }

extern "C" const char* tah_duo_error_string(int code) {
    switch (code) {
        case TAH_OK: return "ok";
        case TAH_E_NULL: return "a required pointer is NULL";
        case TAH_E_SHAPE: return "unsupported shape (head_dim must be 128, Hq/Hkv in {1,2,4,8}, sizes >= 0)";
        case TAH_E_ALIGN: return "pointers must be 16-byte aligned and strides multiples of 8 elements";
        case TAH_E_LAUNCH: return "HIP launch failed";
        case TAH_E_WORKSPACE: return "workspace too small";
        case TAH_E_SCRATCH: return "the call needs more split-K scratch than tah_duo_decode_static holds (TAH_DUO_STATIC_SCRATCH_BYTES)";
        default: return "unknown error";
    }
}
