// 128x128 block weight dequantizer: e4m3fn bytes * fp32 block scale -> bf16 (or fp32).
//
// Restates weight_dequant_kernel
// (/root/reference/triton_kernels/deepseekv3/offical_kernel.py:31-43): one fp32
// multiply per element, rounded once (RNE) to the output type.
//
// Pure streaming, no LDS and no reuse: every lane loads 8 consecutive e4m3fn
// bytes (one 8-byte load), expands them with v_cvt_pk_f32_fp8, multiplies by the
// scale of its 128x128 block (one scalar-ish load per lane, same address for 16
// neighbouring lanes, L1/L2 resident) and writes 8 bf16 as one 16-byte store, so
// a wave's store instruction covers 1 KiB of contiguous output.  All tile accesses are
// non-temporal (no cache allocation for data touched once).  Each wave walks
// kWdRows rows of a 512-column stripe to keep several loads in flight.
//
// HBM traffic per element: 1 B in + 2 B out (+ 4 B per 16384 elements of scale).
#include "common.h"

namespace mdy {

constexpr int kWdRows = 2;           // rows per wave (independent loads in flight)
constexpr int kWdWaves = 4;          // waves per block
constexpr int kWdCols = 64 * 8;      // columns per wave pass

template <typename OUT, bool VEC>
__global__ __launch_bounds__(256) void weight_dequant_kernel(const uint8_t* __restrict__ x, const float* __restrict__ s,
                                                              OUT* __restrict__ y, int N, int K, int sK, int bshift) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = blockIdx.x * kWdCols + lane * 8;
    const int row0 = (block_row() * kWdWaves + wave) * kWdRows;
    if (col >= K) return;

    uint2 raw[kWdRows];
    float sc[kWdRows];
#pragma unroll
    for (int r = 0; r < kWdRows; ++r) {
        const int row = row0 + r;
        raw[r] = make_uint2(0u, 0u);
        sc[r] = 0.0f;
        if (row < N) {
            const uint8_t* p = x + (int64_t)row * K + col;
            if (VEC) {
                raw[r] = load_nt8(p);
            } else {
                uint32_t w[2] = {0u, 0u};
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (col + i < K) w[i >> 2] |= (uint32_t)p[i] << ((i & 3) * 8);
                raw[r] = make_uint2(w[0], w[1]);
            }
            sc[r] = s[(int64_t)(row >> bshift) * sK + (col >> bshift)];      // bshift = log2(block size), 7 for 128x128 blocks
        }
    }
#pragma unroll
    for (int r = 0; r < kWdRows; ++r) {
        const int row = row0 + r;
        if (row >= N) continue;
        floatx2 a = __builtin_amdgcn_cvt_pk_f32_fp8(raw[r].x, false);
        floatx2 b = __builtin_amdgcn_cvt_pk_f32_fp8(raw[r].x, true);
        floatx2 c = __builtin_amdgcn_cvt_pk_f32_fp8(raw[r].y, false);
        floatx2 d = __builtin_amdgcn_cvt_pk_f32_fp8(raw[r].y, true);
        float f[8] = {a.x * sc[r], a.y * sc[r], b.x * sc[r], b.y * sc[r],
                      c.x * sc[r], c.y * sc[r], d.x * sc[r], d.y * sc[r]};
        OUT* q = y + (int64_t)row * K + col;
        if (sizeof(OUT) == 2) {
            if (VEC) {
                uint4 o = make_uint4(pack2_bf16(f[0], f[1]), pack2_bf16(f[2], f[3]), pack2_bf16(f[4], f[5]),
                                     pack2_bf16(f[6], f[7]));
                store_nt16(q, o);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (col + i < K) reinterpret_cast<uint16_t*>(q)[i] = (uint16_t)(pack2_bf16(f[i], 0.0f) & 0xFFFFu);
            }
        } else {
            if (VEC) {
                store_nt16(q, make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])));
                store_nt16(q + 4, make_uint4(__float_as_uint(f[4]), __float_as_uint(f[5]), __float_as_uint(f[6]), __float_as_uint(f[7])));
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (col + i < K) reinterpret_cast<float*>(q)[i] = f[i];
            }
        }
    }
}

// block_size: the edge of the square scale blocks, a power of two from 8 up (128 in the DeepSeek-V3 format; the
// reference's weight_dequant takes any block_size, offical_kernel.py:46-53)
int launch_weight_dequant(const void* x, const float* s, void* y, int64_t N, int64_t K, int block_size, int out_dtype,
                          hipStream_t stream) {
    if (N == 0 || K == 0) return 0;
    dim3 grid, block(256);
    if (!grid_rows((K + kWdCols - 1) / kWdCols, (N + kWdRows * kWdWaves - 1) / (kWdRows * kWdWaves), grid)) return kErrTooManyBlocks;
    int bshift = 0;
    while ((1 << bshift) < block_size) ++bshift;
    const int sK = (int)((K + block_size - 1) / block_size);
    const bool vec = (K % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 7) == 0) &&
                     ((reinterpret_cast<uintptr_t>(y) & 15) == 0);
    const uint8_t* xp = static_cast<const uint8_t*>(x);
    if (out_dtype == 0) {
        uint16_t* yp = static_cast<uint16_t*>(y);
        if (vec)
            hipLaunchKernelGGL((weight_dequant_kernel<uint16_t, true>), grid, block, 0, stream, xp, s, yp, (int)N, (int)K, sK, bshift);
        else
            hipLaunchKernelGGL((weight_dequant_kernel<uint16_t, false>), grid, block, 0, stream, xp, s, yp, (int)N, (int)K, sK, bshift);
    } else {
        float* yp = static_cast<float*>(y);
        if (vec)
            hipLaunchKernelGGL((weight_dequant_kernel<float, true>), grid, block, 0, stream, xp, s, yp, (int)N, (int)K, sK, bshift);
        else
            hipLaunchKernelGGL((weight_dequant_kernel<float, false>), grid, block, 0, stream, xp, s, yp, (int)N, (int)K, sK, bshift);
    }
    return (int)hipGetLastError();
}

}  // namespace mdy
