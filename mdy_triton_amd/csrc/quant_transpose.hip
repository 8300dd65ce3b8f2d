// Training-time quantizer: one pass over a bf16 matrix produces
//   (1) the row-wise 1x128 quantization y[PM,PK] with scales s[kb*s_kb_stride + m]      (as the forward quantizer), and
//   (2) the quantized TRANSPOSE y_t[PK,PM], scaled either per 128x1 column group (t_mode 0) or per
//       128x128 block (t_mode 1),
// in the DeepLinear dialect (MODE 1: scale = (min(amax,1e4) + 1e-8) / 448, saturating cast) or, per column group only,
// in the official dialect (MODE 0: scale = amax / 448, no clamp, no eps: act_quant_block(x) and
// act_quant_block(x, transpose=True) of /root/reference/triton_kernels/deepseekv3/fp8_kernel.py:14-87 in one pass).
//
// Restates _quant_grad_output_kernel (/root/reference/triton_kernels/dpsk_fp8linear/fp8.py:13-44;
// t_mode 0: second half at :40-44 quantizes along axis 0 and stores ST[off_n + pid_m*PN]) and the
// training branch of _quant_input_kernel (fp8.py:115-120; t_mode 1: one scale per 128x128 tile, the
// max of the rows' clamped+eps maxima, stored ST[pid_n*num_programs(0) + pid_m]).
//
// One 256-thread block per 128x128 tile, the tile stays in registers (read once).  Thread t owns
// columns (t%16)*8..+7 of the 8 consecutive rows (t/16)*8 + i: row maxima by DPP inside 16-lane rows, column maxima by
// a per-thread max over its 8 rows followed by an LDS reduction over the 16 row groups.  Quotients
// use the reciprocal + 2-FMA form (bit-identical to IEEE division for every finite amax in this
// dialect); groups whose amax exceeds the 1e4 clamp or is not finite divide plainly and clamp.
// Because a thread's rows are consecutive, its 8 bytes of one column are 8 consecutive bytes of a row of the
// transposed tile: the transpose goes through a padded LDS tile with 8-byte writes and 8-byte reads, and both
// outputs are written row-contiguously.
#include "common.h"

namespace mdy {

// x / s.  FAST (the group's amax lies where the reciprocal form is proven bit-identical to IEEE division and,
// in the DeepLinear dialect, amax <= 1e4, so |x/s| <= 448 needs no clamp) uses the reciprocal form; otherwise an
// IEEE division, saturated at +-448 in the DeepLinear dialect (NaN kept).
template <int MODE, bool FAST>
__device__ __forceinline__ float qt_quot(float x, float s, float r) {
    if (FAST) return fast_quotient(x, s, r);
    return sat_for_mode<MODE>(x / s);
}

// Scale layouts: row scale of row m, K group kb at s[kb * s_kb_stride + m * s_m_stride]; column-group scale of
// column k, row group a at s_t[a * st_a_stride + k * st_k_stride] (TMODE 0) / block scale at s_t[kb * (PM/128) + a]
// (TMODE 1).  y may be null (MODE 0 callers that only want the transposed copy): the row-wise outputs are skipped.
// XT: input type (0 bf16, 1 fp16, 2 fp32); the reciprocal quotient is proven for bf16 inputs only, other types divide.
template <int MODE, int TMODE, bool VEC, int RPT, int XT>
__global__ __launch_bounds__(2048 / RPT) void quant_transpose_kernel(const void* __restrict__ x, uint8_t* __restrict__ y,
                                                               float* __restrict__ s, uint8_t* __restrict__ y_t,
                                                               float* __restrict__ s_t, int M, int K,
                                                               int64_t x_row_stride, int64_t x_col_stride, int PM,
                                                               int PK, int64_t s_kb_stride, int64_t s_m_stride,
                                                               int64_t st_a_stride, int64_t st_k_stride) {
    constexpr int NRG = 128 / RPT;        // row groups of RPT consecutive rows; 16 threads (8 columns each) per group
    constexpr int WAVES = NRG / 4;
    __shared__ float col_part[WAVES][128];  // per wave (4 row groups) partial column maxima
    __shared__ __attribute__((aligned(16))) float col_amax[128];
    __shared__ __attribute__((aligned(16))) float col_sc[128];   // per column: scale of the transposed copy ...
    __shared__ __attribute__((aligned(16))) float col_rc[128];   // ... and its reciprocal, computed once per column
    __shared__ float row_sc[128];         // the tile's 128 row scales, written out as one contiguous run
    __shared__ float blk_part[WAVES];
    __shared__ __attribute__((aligned(16))) uint8_t tile[128][128 + 8];   // [k][m], transposed

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int bm = block_row(), bk = blockIdx.x;
    if (bm >= (PM >> 7)) return;
    const int cl = (t & 15) * 8;          // first local column of this thread
    const int rg = t >> 4;                // row group 0..NRG-1
    const int c0 = bk * 128 + cl;

    float f[RPT][8];
    float rmax[RPT];
    float cmax[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) cmax[j] = 0.0f;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        load_row8_f32<XT, VEC>(x, bm * 128 + rg * RPT + i, c0, M, K, x_row_stride, x_col_stride, f[i]);
        float m = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            m = fmaxf(fmaxf(fabsf(f[i][2 * j]), fabsf(f[i][2 * j + 1])), m);
            cmax[2 * j] = fmaxf(cmax[2 * j], fabsf(f[i][2 * j]));
            cmax[2 * j + 1] = fmaxf(cmax[2 * j + 1], fabsf(f[i][2 * j + 1]));
        }
        rmax[i] = row16_max(m);
    }

    // ---- (1) row-wise quantization straight from registers
#pragma unroll
    for (int i = 0; i < (y != nullptr ? RPT : 0); ++i) {
        const int row = bm * 128 + rg * RPT + i;    // < PM
        const float sc = group_scale<MODE>(rmax[i]);
        const float r = 1.0f / sc;
        float q[8];
        if (XT == 0 && group_is_fast<MODE>(rmax[i])) {
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = qt_quot<MODE, true>(f[i][j], sc, r);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = qt_quot<MODE, false>(f[i][j], sc, r);
        }
        store_nt8(y + (int64_t)row * PK + c0, make_uint2(pack4_fp8<MODE>(q[0], q[1], q[2], q[3]), pack4_fp8<MODE>(q[4], q[5], q[6], q[7])));
        if ((t & 15) == 0) row_sc[rg * RPT + i] = sc;
    }

    // ---- (2) scales of the transposed copy
    float tamax[8];   // amax that scales this thread's 8 columns in the transposed copy
    float tsc[8], tr[8];
    if (TMODE == 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            // the 4 row groups of a wave hold the same columns in lanes 16 apart: fold them before going to LDS
            float m = fmaxf(cmax[j], __shfl_xor(cmax[j], 16, 64));
            m = fmaxf(m, __shfl_xor(m, 32, 64));
            if (lane < 16) col_part[wave][cl + j] = m;
        }
        __syncthreads();
        if (t < 128) {
            float m = 0.0f;
#pragma unroll
            for (int g = 0; g < WAVES; ++g) m = fmaxf(m, col_part[g][t]);
            const float sc = group_scale<MODE>(m);
            col_amax[t] = m;
            col_sc[t] = sc;
            col_rc[t] = 1.0f / sc;
            s_t[(int64_t)bm * st_a_stride + (int64_t)(bk * 128 + t) * st_k_stride] = sc;
            if (y != nullptr) s[(int64_t)bk * s_kb_stride + (int64_t)(bm * 128 + t) * s_m_stride] = row_sc[t];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            tamax[j] = col_amax[cl + j];
            tsc[j] = col_sc[cl + j];
            tr[j] = col_rc[cl + j];
        }
    } else {
        float m = 0.0f;
#pragma unroll
        for (int i = 0; i < RPT; ++i) m = fmaxf(m, rmax[i]);
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
        if (lane == 0) blk_part[wave] = m;
        __syncthreads();
        float bmax = blk_part[0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) bmax = fmaxf(bmax, blk_part[w]);
        if (t == 0) s_t[(int64_t)bk * (PM >> 7) + bm] = group_scale<MODE>(bmax);
        if (t < 128 && y != nullptr) s[(int64_t)bk * s_kb_stride + (int64_t)(bm * 128 + t) * s_m_stride] = row_sc[t];
        const float bsc = group_scale<MODE>(bmax), brc = 1.0f / bsc;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            tamax[j] = bmax;
            tsc[j] = bsc;
            tr[j] = brc;
        }
    }
    bool tfast = XT == 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) tfast = tfast && group_is_fast<MODE>(tamax[j]);
    uint32_t qlo[RPT], qhi[RPT];   // row i of the transposed copy's bytes: columns 0..3 | 4..7
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        float q[8];
        if (tfast) {
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = qt_quot<MODE, true>(f[i][j], tsc[j], tr[j]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = qt_quot<MODE, false>(f[i][j], tsc[j], tr[j]);
        }
        qlo[i] = pack4_fp8<MODE>(q[0], q[1], q[2], q[3]);
        qhi[i] = pack4_fp8<MODE>(q[4], q[5], q[6], q[7]);
    }
    // column j of the thread's RPT x 8 bytes = RPT consecutive bytes of row cl+j of the transposed tile
    if (RPT == 8) {
        uint32_t tb[8][2];   // [column j][rows 0..3 | 4..7]
        uint32_t lo8[8], hi8[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) { lo8[i] = qlo[i % RPT]; hi8[i] = qhi[i % RPT]; }
        transpose8x8_bytes(lo8, hi8, tb);
#pragma unroll
        for (int j = 0; j < 8; ++j) *reinterpret_cast<uint2*>(&tile[cl + j][rg * 8]) = make_uint2(tb[j][0], tb[j][1]);
    } else {
        const uint32_t rl[4] = {qlo[0], qlo[1 % RPT], qlo[2 % RPT], qlo[3 % RPT]};
        const uint32_t rh[4] = {qhi[0], qhi[1 % RPT], qhi[2 % RPT], qhi[3 % RPT]};
        uint32_t c_lo[4], c_hi[4];
        transpose4x4_bytes(rl, c_lo);
        transpose4x4_bytes(rh, c_hi);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<uint32_t*>(&tile[cl + j][rg * 4]) = c_lo[j];
            *reinterpret_cast<uint32_t*>(&tile[cl + 4 + j][rg * 4]) = c_hi[j];
        }
    }
    __syncthreads();
    // y_t[k][m]: thread owns output columns (t%16)*8..+7 (m) of output rows t/16 + NRG*i (k)
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int kk = rg + NRG * i;
        const uint2 v = *reinterpret_cast<const uint2*>(&tile[kk][cl]);
        // plain (cached) store: the 128-byte pieces that neighbouring tiles write into the same rows of y_t are merged
        // in L2 before they go to memory (non-temporal stores measured 6-10 % slower here; y keeps them)
        *reinterpret_cast<uint2*>(y_t + (int64_t)(bk * 128 + kk) * PM + bm * 128 + cl) = v;
    }
}

// Shared launcher.  mode: dialect (0 official, column groups only; 1 DeepLinear); t_mode: 0 per column group, 1 per
// 128x128 block.
static int launch_qt(int mode, const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                     int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int64_t s_kb_stride,
                     int64_t s_m_stride, int64_t st_a_stride, int64_t st_k_stride, int t_mode, hipStream_t stream) {
    if (PM == 0 || PK == 0) return 0;
    dim3 grid;
    if (!grid_rows(PK / 128, PM / 128, grid)) return kErrTooManyBlocks;
    // 512 threads (4 rows each) when there are few tiles per CU: more waves to hide the load and store latency
    const bool wide = (PK / 128) * (PM / 128) < 256 * 24;
    dim3 block(wide ? 512 : 256);
    const bool vec = rows_vectorizable(x, K, x_row_stride, x_col_stride, xt_size(x_dtype));
    uint8_t* yp = static_cast<uint8_t*>(y);
    uint8_t* ytp = static_cast<uint8_t*>(y_t);
#define MDY_QT(MODE, TM, VEC, XT)                                                                                         \
    do {                                                                                                                  \
        if (wide)                                                                                                         \
            hipLaunchKernelGGL((quant_transpose_kernel<MODE, TM, VEC, 4, XT>), grid, block, 0, stream, x, yp, s, ytp, s_t, \
                               (int)M, (int)K, x_row_stride, x_col_stride, (int)PM, (int)PK, s_kb_stride, s_m_stride,     \
                               st_a_stride, st_k_stride);                                                                 \
        else                                                                                                              \
            hipLaunchKernelGGL((quant_transpose_kernel<MODE, TM, VEC, 8, XT>), grid, block, 0, stream, x, yp, s, ytp, s_t, \
                               (int)M, (int)K, x_row_stride, x_col_stride, (int)PM, (int)PK, s_kb_stride, s_m_stride,     \
                               st_a_stride, st_k_stride);                                                                 \
    } while (0)
#define MDY_QT_V(MODE, TM, XT) do { if (vec) MDY_QT(MODE, TM, true, XT); else MDY_QT(MODE, TM, false, XT); } while (0)
#define MDY_QT_X(MODE, TM) do { if (x_dtype == 0) MDY_QT_V(MODE, TM, 0); else if (x_dtype == 1) MDY_QT_V(MODE, TM, 1); else MDY_QT_V(MODE, TM, 2); } while (0)
    if (mode == 0) MDY_QT_X(0, 0);
    else if (mode == 2) MDY_QT_X(2, 0);
    else if (t_mode == 0) MDY_QT_X(1, 0);
    else MDY_QT_X(1, 1);
#undef MDY_QT_X
#undef MDY_QT_V
#undef MDY_QT
    return (int)hipGetLastError();
}

int launch_quant_transpose(const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                           int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int64_t s_kb_stride,
                           int t_mode, hipStream_t stream) {
    // DeepLinear layouts: row scales [PK/128][s_kb_stride >= PM], column-group scales [PM/128][PK]
    return launch_qt(1, x, x_dtype, y, s, y_t, s_t, M, K, x_row_stride, x_col_stride, PM, PK, s_kb_stride, 1, PK, 1, t_mode, stream);
}

int launch_act_quant_transpose(const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                               int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int mode, hipStream_t stream) {
    // official layouts, both row-major: s [PM][PK/128], s_t [PK][PM/128]; mode 0 (e4m3fn) or 2 (e5m2)
    return launch_qt(mode == 2 ? 2 : 0, x, x_dtype, y, s, y_t, s_t, M, K, x_row_stride, x_col_stride, PM, PK, 1, PK / 128, 1, PM / 128, 0, stream);
}

}  // namespace mdy
