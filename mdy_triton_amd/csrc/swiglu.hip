// SwiGLU activation, alone or fused with the 1x128 activation quantizer that feeds the
// down-projection GEMM:  act[m, n] = bf16( silu(gate[m, n]) * up[m, n] ),  gate/up = the two
// halves of a row of x[M, 2N] ("up-gate": up first; "gate-up": gate first).
//
// Restates _fused_silu_fwdv2 / silu_fwd and _fused_silu_bwd_dupgatev2 / silu_bwd
// (/root/reference/triton_kernels/deepseekv3/fp8_kernel.py:315-344, 384-402 and :346-382, 404-421;
// the same kernels are at triton_kernels/megatron_patchs/swiglu.py:6-36), and the sequence
// act = silu_fwd(up_gate); qact, sact = act_quant(act) of Fp8MLP (fp8_kernel.py:447-450, 500-515).
//
// The fused kernel rounds the product to bf16 exactly where the unfused sequence does and
// quantizes THAT value, so its (bytes, scales) are those of act_quant applied to its own bf16
// output; the bf16 tensor itself (302 MB read + 151 MB written + 151 MB read again at the MLP-down
// shape) is only written when the caller asks for it (training keeps it for the backward pass).
//
// Layout of the work as in the activation quantizer: 16 lanes own one 128-column group, each lane
// loads 8 up and 8 gate values (two 16-byte non-temporal loads), absmax by DPP inside the 16-lane
// row, one 8-byte store of e4m3fn per lane.  sigmoid = 1 / (1 + 2^(-g*log2 e)) on the hardware
// exp2 / rcp units (about 1 ulp each in fp32, far below the bf16 rounding that follows).
//
// HBM traffic per output element: 4 B in, 1 B out, 4/128 B scale (+ 2 B when act is written).
#include "common.h"

namespace mdy {

constexpr int kSgRowsPerWave = 2;
constexpr int kSgWaves = 4;
constexpr int kSgRowsPerBlock = kSgRowsPerWave * kSgWaves;

__device__ __forceinline__ float sg_sigmoid(float g) {
    // 2^(-g * log2(e)); for g << 0 the exponential overflows to +inf and the reciprocal gives 0
    const float e = __builtin_amdgcn_exp2f(-1.44269504088896340736f * g);
    return __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ void unpack8(const uint4& r, float (&f)[8]) {
    f[0] = bf16_lo(r.x); f[1] = bf16_hi(r.x); f[2] = bf16_lo(r.y); f[3] = bf16_hi(r.y);
    f[4] = bf16_lo(r.z); f[5] = bf16_hi(r.z); f[6] = bf16_lo(r.w); f[7] = bf16_hi(r.w);
}

__device__ __forceinline__ uint4 load8_bf16(const uint16_t* p, int col, int N, bool vec) {
    if (vec) return load_nt16(p);
    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i)
        if (col + i < N) w[i >> 1] |= (uint32_t)p[i] << ((i & 1) * 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// Block = 8 rows x 512 columns, 256 threads; blocks arranged by grid_rows, or (by_xcd, with row-major scales)
// as grid (8, column chunks, slabs of 8 row blocks) so that all column chunks of a row block run on one XCD and
// the 16-byte pieces of its scale lines meet in one L2 (see act_quant_kernel).
// QUANT: write e4m3fn + scales; act may be null.  !QUANT: act only.
template <int MODE, bool QUANT, bool VEC>
__global__ __launch_bounds__(256) void swiglu_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ act,
                                                     uint8_t* __restrict__ y, float* __restrict__ s, int M, int N,
                                                     int64_t x_row_stride, int up_off, int gate_off, int PM, int PN,
                                                     int64_t s_row_stride, int64_t s_col_stride, int by_xcd) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = (by_xcd ? blockIdx.y : blockIdx.x) * 512 + lane * 8;
    const int row_block = by_xcd ? (int)((blockIdx.z << 3) + blockIdx.x) : block_row();
    const int row0 = row_block * kSgRowsPerBlock + wave * kSgRowsPerWave;

    uint4 ru[kSgRowsPerWave], rg[kSgRowsPerWave];
#pragma unroll
    for (int r = 0; r < kSgRowsPerWave; ++r) {
        const int row = row0 + r;
        ru[r] = rg[r] = make_uint4(0u, 0u, 0u, 0u);
        if (row < M && col < N) {
            const uint16_t* p = x + (int64_t)row * x_row_stride + col;
            ru[r] = load8_bf16(p + up_off, col, N, VEC);
            rg[r] = load8_bf16(p + gate_off, col, N, VEC);
        }
    }
#pragma unroll
    for (int r = 0; r < kSgRowsPerWave; ++r) {
        const int row = row0 + r;
        float u[8], g[8], f[8];
        unpack8(ru[r], u);
        unpack8(rg[r], g);
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            const float a0 = (g[i] * sg_sigmoid(g[i])) * u[i];
            const float a1 = (g[i + 1] * sg_sigmoid(g[i + 1])) * u[i + 1];
            w[i >> 1] = pack2_bf16(a0, a1);
            f[i] = bf16_lo(w[i >> 1]);          // the value the unfused sequence would quantize
            f[i + 1] = bf16_hi(w[i >> 1]);
        }
        if (act != nullptr && row < M && col < N) {
            uint16_t* q = act + (int64_t)row * N + col;
            if (VEC) {
                store_nt16(q, make_uint4(w[0], w[1], w[2], w[3]));
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (col + i < N) q[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
            }
        }
        if (QUANT) {
            float m = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i += 2) m = fmaxf(fmaxf(fabsf(f[i]), fabsf(f[i + 1])), m);
            const float amax = row16_max(m);
            float sc;
            const uint2 packed = quantize8<MODE>(f, amax, sc);
            if (row < PM && col < PN) {
                store_nt8(y + (int64_t)row * PN + col, packed);
                if ((lane & 15) == 0) s[(int64_t)row * s_row_stride + (int64_t)(col >> 7) * s_col_stride] = sc;
            }
        }
    }
}

// dx[m, up] = silu(gate) * dy ; dx[m, gate] = (sig + silu*(1 - sig)) * up * dy   (fp8_kernel.py:346-382)
template <bool VEC>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ dy,
                                                         uint16_t* __restrict__ dx, int M, int N, int64_t x_row_stride,
                                                         int up_off, int gate_off) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = blockIdx.x * 512 + lane * 8;
    const int row0 = block_row() * kSgRowsPerBlock + wave * kSgRowsPerWave;
#pragma unroll
    for (int r = 0; r < kSgRowsPerWave; ++r) {
        const int row = row0 + r;
        if (row >= M || col >= N) continue;
        const uint16_t* p = x + (int64_t)row * x_row_stride + col;
        float u[8], g[8], d[8];
        unpack8(load8_bf16(p + up_off, col, N, VEC), u);
        unpack8(load8_bf16(p + gate_off, col, N, VEC), g);
        unpack8(load8_bf16(dy + (int64_t)row * N + col, col, N, VEC), d);
        uint32_t wu[4], wg[4];
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            float du[2], dg[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const float sig = sg_sigmoid(g[i + e]);
                const float a = sig * g[i + e];
                du[e] = a * d[i + e];
                const float dact = u[i + e] * d[i + e];
                dg[e] = (sig + a * (1.0f - sig)) * dact;
            }
            wu[i >> 1] = pack2_bf16(du[0], du[1]);
            wg[i >> 1] = pack2_bf16(dg[0], dg[1]);
        }
        uint16_t* q = dx + (int64_t)row * 2 * N + col;
        if (VEC) {
            store_nt16(q + up_off, make_uint4(wu[0], wu[1], wu[2], wu[3]));
            store_nt16(q + gate_off, make_uint4(wg[0], wg[1], wg[2], wg[3]));
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (col + i < N) {
                    q[up_off + i] = (uint16_t)(wu[i >> 1] >> ((i & 1) * 16));
                    q[gate_off + i] = (uint16_t)(wg[i >> 1] >> ((i & 1) * 16));
                }
        }
    }
}

int launch_swiglu(const void* x, void* act, void* y, float* s, int64_t M, int64_t N, int64_t x_row_stride,
                  int gate_first, int64_t PM, int64_t PN, int64_t s_row_stride, int64_t s_col_stride, int mode,
                  hipStream_t stream) {
    const bool quant = y != nullptr;
    const int64_t rows = quant ? PM : M, cols = quant ? PN : N;
    if (rows == 0 || cols == 0) return 0;
    const int up_off = gate_first ? (int)N : 0, gate_off = gate_first ? 0 : (int)N;
    const bool vec = (N % 8 == 0) && (x_row_stride % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) &&
                     (act == nullptr || (reinterpret_cast<uintptr_t>(act) & 15) == 0);
    const int by_xcd = (quant && s_col_stride == 1) ? 1 : 0;    // row-major scales
    const int64_t chunks = (cols + 511) / 512;
    if (chunks > 65535) return kErrTooManyBlocks;
    const int64_t slab_rows = (int64_t)kSgRowsPerBlock * 8;                  // rows per grid.z step
    const int64_t rows_per_launch = by_xcd ? slab_rows * 65535 : rows;      // grid.z takes 65535 slabs
    for (int64_t r0 = 0; r0 < rows; r0 += rows_per_launch) {
        const int64_t n_rows = rows - r0 < rows_per_launch ? rows - r0 : rows_per_launch;
        const int64_t m = M - r0 < 0 ? 0 : (M - r0 < n_rows ? M - r0 : n_rows);
        dim3 grid(8, (unsigned)chunks, (unsigned)((n_rows + slab_rows - 1) / slab_rows)), block(256);
        if (!by_xcd && !grid_rows(chunks, (n_rows + kSgRowsPerBlock - 1) / kSgRowsPerBlock, grid)) return kErrTooManyBlocks;
        const uint16_t* xp = static_cast<const uint16_t*>(x) + r0 * x_row_stride;
        uint16_t* ap = act ? static_cast<uint16_t*>(act) + r0 * N : nullptr;
        uint8_t* yp = quant ? static_cast<uint8_t*>(y) + r0 * PN : nullptr;
        float* sp = quant ? s + r0 * s_row_stride : nullptr;
        const int pm = quant ? (int)n_rows : 0;
#define MDY_SG(MODE, QUANT, VEC)                                                                                     \
    hipLaunchKernelGGL((swiglu_kernel<MODE, QUANT, VEC>), grid, block, 0, stream, xp, ap, yp, sp, (int)m, (int)N,      \
                       x_row_stride, up_off, gate_off, pm, (int)PN, s_row_stride, s_col_stride, by_xcd)
        if (!quant) {
            if (vec) MDY_SG(0, false, true); else MDY_SG(0, false, false);
        } else if (mode == 0) {
            if (vec) MDY_SG(0, true, true); else MDY_SG(0, true, false);
        } else {
            if (vec) MDY_SG(1, true, true); else MDY_SG(1, true, false);
        }
#undef MDY_SG
    }
    return (int)hipGetLastError();
}

int launch_swiglu_bwd(const void* x, const void* dy, void* dx, int64_t M, int64_t N, int64_t x_row_stride,
                      int gate_first, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    dim3 grid;
    if (!grid_rows((N + 511) / 512, (M + kSgRowsPerBlock - 1) / kSgRowsPerBlock, grid)) return kErrTooManyBlocks;
    const int up_off = gate_first ? (int)N : 0, gate_off = gate_first ? 0 : (int)N;
    const bool vec = (N % 8 == 0) && (x_row_stride % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) &&
                     ((reinterpret_cast<uintptr_t>(dy) & 15) == 0) && ((reinterpret_cast<uintptr_t>(dx) & 15) == 0);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const uint16_t* dyp = static_cast<const uint16_t*>(dy);
    uint16_t* dxp = static_cast<uint16_t*>(dx);
    if (vec)
        hipLaunchKernelGGL((swiglu_bwd_kernel<true>), grid, dim3(256), 0, stream, xp, dyp, dxp, (int)M, (int)N, x_row_stride, up_off, gate_off);
    else
        hipLaunchKernelGGL((swiglu_bwd_kernel<false>), grid, dim3(256), 0, stream, xp, dyp, dxp, (int)M, (int)N, x_row_stride, up_off, gate_off);
    return (int)hipGetLastError();
}

}  // namespace mdy
