// 128x128 block weight quantizer: bf16 -> e4m3fn bytes + one fp32 scale per block,
// optionally also the transposed copy (for the backward GEMMs).
//
// Restates _quant_weight_kernel
// (/root/reference/triton_kernels/dpsk_fp8linear/fp8.py:171-203; clamp + eps dialect)
// and _weight_quant_block_kernel
// (/root/reference/triton_kernels/deepseekv3/fp8_kernel.py:88-122; plain amax/448).
//
// One 512-thread block per 128x128 tile.  Thread t owns columns (t%16)*8..+7 of
// rows (t/16)*4 + i, i = 0..3: four 16-byte loads kept in registers (the tile is
// read from HBM exactly once), absmax reduced inside the wave with __shfl_xor,
// the eight wave results combined through LDS.
// The quotient is the same reciprocal + 2-FMA form as the activation quantizer.
// The transposed copy goes through a padded LDS tile: a thread's 4 consecutive rows of one column are 4
// consecutive bytes of a transposed row (4-byte LDS writes, 8-byte reads).
//
// HBM traffic per element: 2 B in + 1 B out (+ 1 B for the transposed copy).
#include "common.h"

namespace mdy {

// XT: input type (0 bf16, 1 fp16, 2 fp32); the reciprocal quotient is proven for bf16 inputs, other types divide.
template <int MODE, bool VEC, int XT>
__global__ __launch_bounds__(512) void weight_quant_kernel(const void* __restrict__ w, uint8_t* __restrict__ y,
                                                            float* __restrict__ s, uint8_t* __restrict__ y_t,
                                                            float* __restrict__ s_t, int N, int K, int64_t w_row_stride,
                                                            int64_t w_col_stride, int PN, int PK) {
    constexpr int RPT = 4;             // rows per thread
    constexpr int NRG = 128 / RPT;     // row groups of RPT consecutive rows, 16 threads (8 columns each) per group
    constexpr int WAVES = NRG / 4;
    __shared__ float wave_max[WAVES];
    __shared__ __attribute__((aligned(16))) uint8_t tile[128][128 + 8];   // [k][n], transposed

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = t >> 6;
    const int bn = block_row();  // block row (along N)
    const int bk = blockIdx.x;   // block column (along K)
    if (bn >= (PN >> 7)) return;
    const int c0 = bk * 128 + (t & 15) * 8;
    const int rbase = bn * 128 + (t >> 4) * RPT;

    float f[RPT][8];
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        load_row8_f32<XT, VEC>(w, rbase + i, c0, N, K, w_row_stride, w_col_stride, f[i]);
#pragma unroll
        for (int j = 0; j < 4; ++j) m = fmaxf(fmaxf(fabsf(f[i][2 * j]), fabsf(f[i][2 * j + 1])), m);
    }
    // wave-wide max, then across the waves
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (lane == 0) wave_max[wave] = m;
    __syncthreads();
    float amax = wave_max[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) amax = fmaxf(amax, wave_max[w]);

    const float sc = group_scale<MODE>(amax);
    const bool fast = XT == 0 && group_is_fast<MODE>(amax);
    const float r = 1.0f / sc;
    if (t == 0) {
        if (s) s[(int64_t)bn * (PK >> 7) + bk] = sc;
        if (s_t) s_t[(int64_t)bk * (PN >> 7) + bn] = sc;
    }
    uint32_t qlo[RPT], qhi[RPT];   // row i of the quantized bytes: columns 0..3 | 4..7
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const uint2 o = quantize8_scaled<MODE>(f[i], sc, r, fast);
        const int row = rbase + i;  // < PN because PN % 128 == 0
        if (y) store_nt8(y + (int64_t)row * PK + c0, o);      // NULL: only the transposed copy is wanted
        qlo[i] = o.x;
        qhi[i] = o.y;
    }
    if (y_t) {
        // column j of the thread's RPT x 8 bytes = RPT consecutive bytes of row (t%16)*8 + j of the transposed tile
        const int cl = (t & 15) * 8, rg = t >> 4;
        uint32_t c_lo[4], c_hi[4];
        transpose4x4_bytes(qlo, c_lo);
        transpose4x4_bytes(qhi, c_hi);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<uint32_t*>(&tile[cl + j][rg * 4]) = c_lo[j];
            *reinterpret_cast<uint32_t*>(&tile[cl + 4 + j][rg * 4]) = c_hi[j];
        }
        __syncthreads();
        // y_t[k][n]: thread owns output columns (t%16)*8..+7 (n) of output rows t/16 + NRG*i (k)
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const int kk = rg + NRG * i;
            // cached store: neighbouring tiles complete the rows of y_t in L2 (1-7 % faster than non-temporal here)
            *reinterpret_cast<uint2*>(y_t + (int64_t)(bk * 128 + kk) * PN + bn * 128 + cl) =
                *reinterpret_cast<const uint2*>(&tile[kk][cl]);
        }
    }
}

int launch_weight_quant(const void* w, int w_dtype, void* y, float* s, void* y_t, float* s_t, int64_t N, int64_t K,
                        int64_t w_row_stride, int64_t w_col_stride, int64_t PN, int64_t PK, int mode,
                        hipStream_t stream) {
    if (PN == 0 || PK == 0) return 0;
    dim3 grid;
    if (!grid_rows(PK / 128, PN / 128, grid)) return kErrTooManyBlocks;
    // 512 threads per tile: 4 rows per thread, 56 VGPRs, 8 waves per SIMD (256 threads with 8 rows each need 89
    // VGPRs and measured 1-5 % slower at every size tried)
    dim3 block(512);
    const bool vec = rows_vectorizable(w, K, w_row_stride, w_col_stride, xt_size(w_dtype));
    uint8_t* yp = static_cast<uint8_t*>(y);
    uint8_t* ytp = static_cast<uint8_t*>(y_t);
#define MDY_WQ(MODE, VEC, XT)                                                                                      \
    hipLaunchKernelGGL((weight_quant_kernel<MODE, VEC, XT>), grid, block, 0, stream, w, yp, s, ytp, s_t, (int)N, \
                       (int)K, w_row_stride, w_col_stride, (int)PN, (int)PK)
#define MDY_WQ_V(MODE, XT) do { if (vec) MDY_WQ(MODE, true, XT); else MDY_WQ(MODE, false, XT); } while (0)
#define MDY_WQ_X(MODE) do { if (w_dtype == 0) MDY_WQ_V(MODE, 0); else if (w_dtype == 1) MDY_WQ_V(MODE, 1); else MDY_WQ_V(MODE, 2); } while (0)
    if (mode == 0) MDY_WQ_X(0); else if (mode == 1) MDY_WQ_X(1); else MDY_WQ_X(2);
#undef MDY_WQ_X
#undef MDY_WQ_V
#undef MDY_WQ
    return (int)hipGetLastError();
}

}  // namespace mdy
