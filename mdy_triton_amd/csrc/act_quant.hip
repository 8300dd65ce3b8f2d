// Per-token 1x128 activation quantizer: bf16 -> e4m3fn bytes + one fp32 scale per group.
//
// Restates the arithmetic of act_quant_kernel
// (/root/reference/triton_kernels/deepseekv3/offical_kernel.py:9-18) and of
// _quant_input_kernel's forward half
// (/root/reference/triton_kernels/dpsk_fp8linear/fp8.py:104-113) for wave64:
//
//   * 16 lanes own one 128-element group: one 16-byte load (8 bf16) per lane, so a
//     wave covers 512 contiguous elements of a row per load instruction;
//   * absmax by v_max3_f32 on the unpacked values, then a 4-step DPP butterfly
//     inside the 16-lane row (no LDS, no barrier);
//   * scale = amax / 448 and r = 1 / scale with IEEE division once per group; each
//     element is x*r corrected by two FMAs (bit-identical to x / scale, proven
//     exhaustively over bf16 x bf16); groups whose amax is tiny, above 1e4
//     (DeepLinear dialect, needs the saturating cast) or non-finite divide plainly;
//   * loads and stores are non-temporal (every byte is touched once);
//   * v_cvt_pk_fp8_f32 x4 -> one 8-byte store per lane; lane 0 of the row stores
//     the scale at a caller-given (row, column) stride so that both the row-major
//     [M, K/128] layout and the column-major padded [K/128][PM] layout come out
//     of the same kernel.
//
// HBM traffic per element: 2 B in, 1 B out, 4/128 B scale = 3.03125 B.
#include "common.h"

namespace mdy {

constexpr int kAqRowsPerWave = 2;
constexpr int kAqWaves = 4;
constexpr int kAqRowsPerBlock = kAqRowsPerWave * kAqWaves;  // 8 rows x 512 columns per block

// 8 bf16 of row `row` from column `col` on, zeros outside the M x K matrix
template <bool VEC>
__device__ __forceinline__ uint4 load8(const uint16_t* __restrict__ x, int row, int col, int M, int K, int64_t x_row_stride) {
    if (row >= M || col >= K) return make_uint4(0u, 0u, 0u, 0u);
    const uint16_t* p = x + (int64_t)row * x_row_stride + col;
    if (VEC) return load_nt16(p);  // K % 8 == 0: all 8 columns in range
    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i)
        if (col + i < K) w[i >> 1] |= (uint32_t)p[i] << ((i & 1) * 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// The same 8 values as fp32 for an input of type XT (0 bf16, 1 fp16, 2 fp32), zeros outside the M x K matrix.
// The reference kernels load with .to(tl.float32), so every input type is quantized from its exact fp32 value.
template <int XT, bool VEC>
__device__ __forceinline__ void load8_f32(const void* __restrict__ x, int row, int col, int M, int K, int64_t x_row_stride,
                                          float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = 0.0f;
    if (row >= M || col >= K) return;
    if (XT == 0) {
        const uint4 v = load8<VEC>(static_cast<const uint16_t*>(x), row, col, M, K, x_row_stride);
        f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x); f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
        f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z); f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
    } else if (XT == 1) {
        const _Float16* p = static_cast<const _Float16*>(x) + (int64_t)row * x_row_stride + col;
        if (VEC) {
            const uint4 v = load_nt16(p);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0xFFFFu));
                f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] >> 16));
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (col + i < K) f[i] = (float)p[i];
        }
    } else {
        const float* p = static_cast<const float*>(x) + (int64_t)row * x_row_stride + col;
        if (VEC) {
            const uint4 a = load_nt16(p), b = load_nt16(p + 4);
            f[0] = __uint_as_float(a.x); f[1] = __uint_as_float(a.y); f[2] = __uint_as_float(a.z); f[3] = __uint_as_float(a.w);
            f[4] = __uint_as_float(b.x); f[5] = __uint_as_float(b.y); f[6] = __uint_as_float(b.z); f[7] = __uint_as_float(b.w);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (col + i < K) f[i] = p[i];
        }
    }
}
// absmax of a quantization group of `lanes` consecutive lanes x 8 values (lanes a power of two, 1..64)
__device__ __forceinline__ float group_max8(const float (&f)[8], int lanes) {
    float m = 0.0f;
    m = fmaxf(fmaxf(fabsf(f[0]), fabsf(f[1])), m);
    m = fmaxf(fmaxf(fabsf(f[2]), fabsf(f[3])), m);
    m = fmaxf(fmaxf(fabsf(f[4]), fabsf(f[5])), m);
    m = fmaxf(fmaxf(fabsf(f[6]), fabsf(f[7])), m);
    if (lanes == 16) return row16_max(m);
    for (int off = 1; off < lanes; off <<= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    return m;
}

// the lane's 8 values as fp32 and the absmax of its 128-element group (16 lanes)
__device__ __forceinline__ float unpack8_group_max(const uint4& raw, float (&f)[8]) {
    f[0] = bf16_lo(raw.x); f[1] = bf16_hi(raw.x);
    f[2] = bf16_lo(raw.y); f[3] = bf16_hi(raw.y);
    f[4] = bf16_lo(raw.z); f[5] = bf16_hi(raw.z);
    f[6] = bf16_lo(raw.w); f[7] = bf16_hi(raw.w);
    float m = 0.0f;
    m = fmaxf(fmaxf(fabsf(f[0]), fabsf(f[1])), m);
    m = fmaxf(fmaxf(fabsf(f[2]), fabsf(f[3])), m);
    m = fmaxf(fmaxf(fabsf(f[4]), fabsf(f[5])), m);
    m = fmaxf(fmaxf(fabsf(f[6]), fabsf(f[7])), m);
    return row16_max(m);
}

// Block = 8 rows x 512 columns, 256 threads.  Two block arrangements:
//   by_xcd = 0: grid_rows(column chunks, row blocks);
//   by_xcd = 1: grid (8, column chunks, slabs of 8 row blocks).  Consecutive workgroup ids go to consecutive
//     XCDs, so with 8 as the fastest grid dimension blockIdx.x IS the XCD and all column chunks of row block
//     z * 8 + x run on one XCD.  With row-major scales their scale stores are 16-byte pieces of the same
//     128-byte lines; pieces written through different XCDs' L2s reach memory as partial lines, which costs
//     1-3 % of the kernel from cold caches and 4-7 % back to back.  Column-major scales (a line = 32 rows of one
//     K group) gain nothing from any such grouping and keep the plain arrangement.
template <int MODE, bool VEC>
__global__ __launch_bounds__(256) void act_quant_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ y,
                                                         float* __restrict__ s, int M, int K, int64_t x_row_stride,
                                                         int PM, int PK, int64_t s_row_stride, int64_t s_col_stride, int by_xcd) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = (by_xcd ? blockIdx.y : blockIdx.x) * 512 + lane * 8;  // first of this lane's 8 columns
    const int row_block = by_xcd ? (int)((blockIdx.z << 3) + blockIdx.x) : block_row();
    // the last slab may reach past the rows: rows >= PM are dropped below (leaving here instead, before the
    // loads are issued, measured 3 % slower)
    const int row0 = row_block * kAqRowsPerBlock + wave * kAqRowsPerWave;
    const bool col_in_out = col < PK;  // PK % 128 == 0, so whole 16-lane rows agree

    uint4 raw[kAqRowsPerWave];
#pragma unroll
    for (int r = 0; r < kAqRowsPerWave; ++r) {
        const int row = row0 + r;
        raw[r] = load8<VEC>(x, row, col, M, K, x_row_stride);
    }

#pragma unroll
    for (int r = 0; r < kAqRowsPerWave; ++r) {
        const int row = row0 + r;
        float f[8];
        const float amax = unpack8_group_max(raw[r], f);
        float scale;
        const uint2 packed = quantize8<MODE>(f, amax, scale);
        if (row < PM && col_in_out) {
            store_nt8(y + (int64_t)row * PK + col, packed);
            if ((lane & 15) == 0) s[(int64_t)row * s_row_stride + (int64_t)(col >> 7) * s_col_stride] = scale;
        }
    }
}

// Column-major scales (s_row_stride == 1): block = 32 rows x 512 columns, 8 waves x 4 rows.  The 32 x 4 scales of
// the block are staged in LDS and leave as four full 128-byte lines (32 consecutive rows of one K group each)
// instead of 4-byte pieces from every row's own store.
template <int MODE, bool VEC>
__global__ __launch_bounds__(512) void act_quant_cm_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ y,
                                                            float* __restrict__ s, int M, int K, int64_t x_row_stride,
                                                            int PM, int PK, int64_t s_col_stride) {
    constexpr int R = 4;
    __shared__ float lds_sc[4][32];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = blockIdx.x * 512 + lane * 8;
    const int rb0 = block_row() * 32;
    const int row0 = rb0 + wave * R;
    const bool col_in_out = col < PK;
    uint4 raw[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = row0 + r;
        raw[r] = load8<VEC>(x, row, col, M, K, x_row_stride);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = row0 + r;
        float f[8];
        const float amax = unpack8_group_max(raw[r], f);
        float scale;
        const uint2 packed = quantize8<MODE>(f, amax, scale);
        if (row < PM && col_in_out) store_nt8(y + (int64_t)row * PK + col, packed);
        if ((lane & 15) == 0) lds_sc[lane >> 4][wave * R + r] = scale;
    }
    __syncthreads();
    if (threadIdx.x < 128) {
        const int g = threadIdx.x >> 5, rr = threadIdx.x & 31;
        const int row = rb0 + rr, c = blockIdx.x * 512 + g * 128;
        if (row < PM && c < PK) s[(int64_t)(c >> 7) * s_col_stride + row] = lds_sc[g][rr];
    }
}

// The general form of the quantizer: fp16 / fp32 inputs, and group widths other than 128 (8 x a power of two lanes, up
// to 512 elements: the reference's act_quant takes any block_size, offical_kernel.py:21-27).  The same block shape as
// act_quant_kernel (8 rows x 512 columns, plain arrangement), the quotient by IEEE division (the reciprocal form is
// proven for bf16 inputs only, and only the 128-wide bf16 case is tuned).
template <int MODE, int XT, bool VEC>
__global__ __launch_bounds__(256) void act_quant_typed_kernel(const void* __restrict__ x, uint8_t* __restrict__ y,
                                                               float* __restrict__ s, int M, int K, int64_t x_row_stride,
                                                               int PM, int PK, int64_t s_row_stride, int64_t s_col_stride,
                                                               int group_lanes, int group_shift) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = blockIdx.x * 512 + lane * 8;
    const int row0 = block_row() * kAqRowsPerBlock + wave * kAqRowsPerWave;
    float f[kAqRowsPerWave][8];
#pragma unroll
    for (int r = 0; r < kAqRowsPerWave; ++r) load8_f32<XT, VEC>(x, row0 + r, col, M, K, x_row_stride, f[r]);
#pragma unroll
    for (int r = 0; r < kAqRowsPerWave; ++r) {
        const int row = row0 + r;
        const float amax = group_max8(f[r], group_lanes);
        const float sc = group_scale<MODE>(amax);
        const uint2 packed = quantize8_scaled<MODE>(f[r], sc, 0.0f, false);
        if (row < PM && col < PK) {
            store_nt8(y + (int64_t)row * PK + col, packed);
            if ((lane & (group_lanes - 1)) == 0) s[(int64_t)row * s_row_stride + (int64_t)(col >> group_shift) * s_col_stride] = sc;
        }
    }
}

// x_dtype: 0 bf16, 1 fp16, 2 fp32; block_size: 8 x a power of two, 8..512.  bf16 with block_size 128 is launch_act_quant.
int launch_act_quant_typed(const void* x, int x_dtype, int block_size, void* y, float* s, int64_t M, int64_t K,
                           int64_t x_row_stride, int64_t PM, int64_t PK, int64_t s_row_stride, int64_t s_col_stride, int mode,
                           hipStream_t stream) {
    if (x_dtype == 0 && block_size == 128 && mode != 2)
        return launch_act_quant(x, y, s, M, K, x_row_stride, PM, PK, s_row_stride, s_col_stride, mode, stream);
    if (PM == 0 || PK == 0) return 0;
    const int esz = x_dtype == 2 ? 4 : 2;
    const bool vec = (K % 8 == 0) && ((x_row_stride * esz) % 16 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    const int lanes = block_size / 8;
    int shift = 0;
    while ((1 << shift) < block_size) ++shift;
    dim3 grid;
    if (!grid_rows((PK + 511) / 512, (PM + kAqRowsPerBlock - 1) / kAqRowsPerBlock, grid)) return kErrTooManyBlocks;
    uint8_t* yp = static_cast<uint8_t*>(y);
#define MDY_AQT(MODE, XT, VEC)                                                                                         \
    hipLaunchKernelGGL((act_quant_typed_kernel<MODE, XT, VEC>), grid, dim3(256), 0, stream, x, yp, s, (int)M, (int)K, \
                       x_row_stride, (int)PM, (int)PK, s_row_stride, s_col_stride, lanes, shift)
#define MDY_AQT_V(MODE, XT) do { if (vec) MDY_AQT(MODE, XT, true); else MDY_AQT(MODE, XT, false); } while (0)
#define MDY_AQT_X(MODE) do { if (x_dtype == 0) MDY_AQT_V(MODE, 0); else if (x_dtype == 1) MDY_AQT_V(MODE, 1); else MDY_AQT_V(MODE, 2); } while (0)
    if (mode == 0) MDY_AQT_X(0); else if (mode == 1) MDY_AQT_X(1); else MDY_AQT_X(2);
#undef MDY_AQT_X
#undef MDY_AQT_V
#undef MDY_AQT
    return (int)hipGetLastError();
}

int launch_act_quant(const void* x, void* y, float* s, int64_t M, int64_t K, int64_t x_row_stride, int64_t PM,
                     int64_t PK, int64_t s_row_stride, int64_t s_col_stride, int mode, hipStream_t stream) {
    if (PM == 0 || PK == 0) return 0;
    const bool vec = (K % 8 == 0) && (x_row_stride % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    // column-major scales of a large matrix: 32-row blocks that write whole scale lines (16384x7168: 61.5 -> 58 us;
    // below ~64 M elements the 256-thread blocks are as fast or faster)
    if (s_row_stride == 1 && s_col_stride != 1 && PM * PK >= ((int64_t)1 << 26)) {
        dim3 grid, block(512);
        if (!grid_rows((PK + 511) / 512, (PM + 31) / 32, grid)) return kErrTooManyBlocks;
        const uint16_t* xp = static_cast<const uint16_t*>(x);
        uint8_t* yp = static_cast<uint8_t*>(y);
#define MDY_CM(MODE, VEC)                                                                                          \
    hipLaunchKernelGGL((act_quant_cm_kernel<MODE, VEC>), grid, block, 0, stream, xp, yp, s, (int)M, (int)K, x_row_stride, \
                       (int)PM, (int)PK, s_col_stride)
        if (mode == 0) {
            if (vec) MDY_CM(0, true); else MDY_CM(0, false);
        } else {
            if (vec) MDY_CM(1, true); else MDY_CM(1, false);
        }
#undef MDY_CM
        return (int)hipGetLastError();
    }
    const int by_xcd = s_col_stride == 1 ? 1 : 0;      // row-major scales
    const int64_t chunks = (PK + 511) / 512;
    if (chunks > 65535) return kErrTooManyBlocks;
    const int64_t slab_rows = (int64_t)kAqRowsPerBlock * 8;                  // rows per grid.z step
    const int64_t rows_per_launch = by_xcd ? slab_rows * 65535 : PM;        // grid.z takes 65535 slabs
    for (int64_t r0 = 0; r0 < PM; r0 += rows_per_launch) {
        const int64_t pm = PM - r0 < rows_per_launch ? PM - r0 : rows_per_launch;
        const int64_t m = M - r0 < 0 ? 0 : (M - r0 < pm ? M - r0 : pm);
        dim3 grid(8, (unsigned)chunks, (unsigned)((pm + slab_rows - 1) / slab_rows)), block(256);
        if (!by_xcd && !grid_rows(chunks, (pm + kAqRowsPerBlock - 1) / kAqRowsPerBlock, grid)) return kErrTooManyBlocks;
        const uint16_t* xp = static_cast<const uint16_t*>(x) + r0 * x_row_stride;
        uint8_t* yp = static_cast<uint8_t*>(y) + r0 * PK;
        float* sp = s + r0 * s_row_stride;
#define MDY_AQ(MODE, VEC)                                                                                       \
    hipLaunchKernelGGL((act_quant_kernel<MODE, VEC>), grid, block, 0, stream, xp, yp, sp, (int)m, (int)K,       \
                       x_row_stride, (int)pm, (int)PK, s_row_stride, s_col_stride, by_xcd)
        if (mode == 0) {
            if (vec) MDY_AQ(0, true); else MDY_AQ(0, false);
        } else {
            if (vec) MDY_AQ(1, true); else MDY_AQ(1, false);
        }
#undef MDY_AQ
    }
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// diagnostics
// ---------------------------------------------------------------------------
__global__ void cast_f32_to_e4m3_kernel(const float* __restrict__ x, uint8_t* __restrict__ y, int64_t n, int saturate) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = x[i];
    if (saturate) {
        float c = __builtin_amdgcn_fmed3f(v, -kFp8Max, kFp8Max);
        v = (v != v) ? v : c;
    }
    y[i] = (uint8_t)(pack4_e4m3(v, 0.0f, 0.0f, 0.0f) & 0xFFu);
}

__global__ void cast_f32_to_e5m2_kernel(const float* __restrict__ x, uint8_t* __restrict__ y, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    y[i] = (uint8_t)(pack4_e5m2(x[i], 0.0f, 0.0f, 0.0f) & 0xFFu);
}

int launch_cast_f32_to_e5m2(const float* x, void* y, int64_t n, hipStream_t stream) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(cast_f32_to_e5m2_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x,
                       static_cast<uint8_t*>(y), n);
    return (int)hipGetLastError();
}

int launch_cast_f32_to_e4m3(const float* x, void* y, int64_t n, int saturate, hipStream_t stream) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(cast_f32_to_e4m3_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x,
                       static_cast<uint8_t*>(y), n, saturate);
    return (int)hipGetLastError();
}

// One block per amax bit pattern; threads stride over x patterns 0..amax (both signs).
// Groups that the quantizers would divide plainly are counted in out[3] and skipped.
template <int MODE>
__global__ __launch_bounds__(256) void quotient_selfcheck_kernel(unsigned long long* out, int amax_lo) {
    const uint32_t ai = (uint32_t)amax_lo + blockIdx.x;
    const float amax = bf16_one((uint16_t)ai);
    const float s = group_scale<MODE>(amax);
    const bool fast = group_is_fast<MODE>(amax);      // the quantizers' own criterion
    const float r = 1.0f / s;
    unsigned long long pairs = 0, f32_bad = 0, fp8_bad = 0, plain = 0;
    for (uint32_t t = threadIdx.x; t < 2 * (ai + 1); t += blockDim.x) {
        const uint32_t xi = (t >> 1) | ((t & 1) << 15);
        const float x = bf16_one((uint16_t)xi);
        ++pairs;
        if (!fast) {
            ++plain;
            continue;
        }
        const float ref = x / s;
        const float q = fast_quotient(x, s, r);
        const uint32_t bref = pack4_e4m3(ref, 0.f, 0.f, 0.f) & 0xFF;
        const uint32_t bq = pack4_e4m3(q, 0.f, 0.f, 0.f) & 0xFF;
        if (__float_as_uint(ref) != __float_as_uint(q) && !(ref != ref && q != q)) ++f32_bad;
        if (bref != bq) ++fp8_bad;
    }
    atomicAdd(&out[0], pairs);
    atomicAdd(&out[1], f32_bad);
    atomicAdd(&out[2], fp8_bad);
    atomicAdd(&out[3], plain);
}

__global__ void zero4_kernel(unsigned long long* out) {
    if (threadIdx.x < 4) out[threadIdx.x] = 0ull;
}

int launch_quotient_selfcheck(uint64_t* out, int amax_lo, int amax_hi, int mode, hipStream_t stream) {
    unsigned long long* o = reinterpret_cast<unsigned long long*>(out);
    hipLaunchKernelGGL(zero4_kernel, dim3(1), dim3(64), 0, stream, o);
    if (amax_hi <= amax_lo) return (int)hipGetLastError();
    dim3 grid((unsigned)(amax_hi - amax_lo)), block(256);
    if (mode == 0)
        hipLaunchKernelGGL(quotient_selfcheck_kernel<0>, grid, block, 0, stream, o, amax_lo);
    else
        hipLaunchKernelGGL(quotient_selfcheck_kernel<1>, grid, block, 0, stream, o, amax_lo);
    return (int)hipGetLastError();
}

}  // namespace mdy
