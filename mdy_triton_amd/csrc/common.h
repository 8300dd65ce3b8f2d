// Shared device helpers and host-side launch declarations for libmdyfp8.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mdy {

typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr float kFp8Max = 448.0f;        // largest e4m3fn value
constexpr float kBf8Max = 57344.0f;      // largest e5m2 value
// Quantizer dialects (the MODE template parameter): 0 official (s = amax / 448, e4m3fn), 1 DeepLinear (clamp 1e4 + eps
// 1e-8, saturating e4m3fn cast), 2 official with e5m2 bytes (s = amax / 57344: the default fp8 dtype of
// /root/reference/triton_kernels/deepseekv3/fp8_kernel.py:62,124 is torch.float8_e5m2).
constexpr int kGroup = 128;  // quantization group / block edge

// Smallest biased exponent of amax for which the reciprocal + 2-FMA quotient is
// proven (exhaustively over all bf16 pairs) to give the same e4m3fn byte as IEEE
// division in the official dialect; below it s = amax/448 is subnormal or the
// residual underflows.  The DeepLinear dialect (eps keeps s normal) is clean for
// every finite amax.
constexpr uint32_t kFastQuotientMinExp = 23;

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
__device__ __forceinline__ float bf16_one(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// Scale of one quantization group from its absmax (fp32, IEEE division).
template <int MODE>
__device__ __forceinline__ float group_scale(float amax) {
    if (MODE == 0) return amax / kFp8Max;
    if (MODE == 2) return amax / kBf8Max;
    // clamp(amax, 0, 1e4) + 1e-8, NaN kept (fminf would drop it)
    float c = amax > 1e4f ? 1e4f : amax;
    return (c + 1e-8f) / kFp8Max;
}

// True when the fast quotient may be used for a group with this absmax.
template <int MODE>
__device__ __forceinline__ bool fast_quotient_ok(float amax) {
    uint32_t b = __float_as_uint(amax);
    if (MODE == 2) return false;            // the exhaustive proof covers e4m3fn bytes only
    if (MODE == 0) return b >= (kFastQuotientMinExp << 23) && b < 0x7F800000u;
    return b < 0x7F800000u;
}

// x / s through r = RN(1/s): q0 = x*r, e = fma(q0, s, -x), q = fma(-e, r, q0).
// The residual is kept negated so that x = -0 gives q = -0.
__device__ __forceinline__ float fast_quotient(float x, float s, float r) {
    float q0 = x * r;
    float e = __builtin_fmaf(q0, s, -x);
    return __builtin_fmaf(-e, r, q0);
}

template <int MODE>
__device__ __forceinline__ float sat_for_mode(float q) {
    // v_med3_f32 returns a non-NaN operand for a NaN input, so keep NaN by hand.
    if (MODE != 1) return q;
    float c = __builtin_amdgcn_fmed3f(q, -kFp8Max, kFp8Max);
    return q != q ? q : c;
}

// four fp32 -> four e4m3fn bytes (RNE) packed little-endian into one dword
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
    return (uint32_t)w;
}

// four fp32 -> four e5m2 bytes (RNE) packed little-endian into one dword
__device__ __forceinline__ uint32_t pack4_e5m2(float a, float b, float c, float d) {
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, w, true);
    return (uint32_t)w;
}
template <int MODE>
__device__ __forceinline__ uint32_t pack4_fp8(float a, float b, float c, float d) {
    return MODE == 2 ? pack4_e5m2(a, b, c, d) : pack4_e4m3(a, b, c, d);
}

// One lane's 8 values of a 128-element group with absmax `amax` -> 8 e4m3fn bytes and the group's scale: the
// reciprocal + 2-FMA quotient where it is proven bit-identical to IEEE division, plain division elsewhere.
template <int MODE>
__device__ __forceinline__ uint2 quantize8_scaled(const float (&f)[8], float s, float r, bool fast) {
    float q[8];
    if (fast) {
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = fast_quotient(f[i], s, r);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = sat_for_mode<MODE>(f[i] / s);
    }
    uint2 out;
    out.x = pack4_fp8<MODE>(q[0], q[1], q[2], q[3]);
    out.y = pack4_fp8<MODE>(q[4], q[5], q[6], q[7]);
    return out;
}
// True when a group with this absmax may take the reciprocal form in its dialect (the DeepLinear dialect also
// needs |x / s| <= 448 without the saturating clamp, i.e. an absmax within the 1e4 clamp).
template <int MODE>
__device__ __forceinline__ bool group_is_fast(float amax) {
    return MODE == 0 ? fast_quotient_ok<0>(amax) : MODE == 2 ? false : (amax <= 1e4f);
}
template <int MODE>
__device__ __forceinline__ uint2 quantize8(const float (&f)[8], float amax, float& scale_out) {
    const float s = group_scale<MODE>(amax);
    scale_out = s;
    return quantize8_scaled<MODE>(f, s, 1.0f / s, group_is_fast<MODE>(amax));
}

// 4x4 byte transpose with v_perm_b32: r[i] holds bytes (i,0..3); on return c[j] holds bytes (0..3, j).
__device__ __forceinline__ void transpose4x4_bytes(const uint32_t (&r)[4], uint32_t (&c)[4]) {
    // __builtin_amdgcn_perm(s0, s1, sel): result byte k = byte sel[k] of {s1: 0..3, s0: 4..7}
    const uint32_t t0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);   // r0.b0 r1.b0 r0.b1 r1.b1
    const uint32_t t1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);   // r0.b2 r1.b2 r0.b3 r1.b3
    const uint32_t t2 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
    c[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    c[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    c[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    c[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}
// 8 rows x 8 columns of bytes: row i = (lo[i], hi[i]); column j comes back as tb[j][0] (rows 0..3), tb[j][1] (rows 4..7)
__device__ __forceinline__ void transpose8x8_bytes(const uint32_t (&lo)[8], const uint32_t (&hi)[8], uint32_t (&tb)[8][2]) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const uint32_t rl[4] = {lo[4 * half], lo[4 * half + 1], lo[4 * half + 2], lo[4 * half + 3]};
        const uint32_t rh[4] = {hi[4 * half], hi[4 * half + 1], hi[4 * half + 2], hi[4 * half + 3]};
        uint32_t cl[4], ch[4];
        transpose4x4_bytes(rl, cl);
        transpose4x4_bytes(rh, ch);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            tb[j][half] = cl[j];
            tb[4 + j][half] = ch[j];
        }
    }
}

// max over the 16 lanes of a DPP row (one 128-element quantization group: 16 lanes x 8 values)
__device__ __forceinline__ float row16_max(float v) {
    // butterfly over the 16 lanes of a DPP row: xor 1, xor 2 (quad_perm), then
    // row_half_mirror (lane -> 7-lane inside each 8) and row_mirror (lane -> 15-lane)
    int i = __float_as_int(v);
    i = __float_as_int(fmaxf(__int_as_float(i), __int_as_float(__builtin_amdgcn_mov_dpp(i, 0xB1, 0xF, 0xF, true))));   // quad_perm [1,0,3,2]
    i = __float_as_int(fmaxf(__int_as_float(i), __int_as_float(__builtin_amdgcn_mov_dpp(i, 0x4E, 0xF, 0xF, true))));   // quad_perm [2,3,0,1]
    i = __float_as_int(fmaxf(__int_as_float(i), __int_as_float(__builtin_amdgcn_mov_dpp(i, 0x141, 0xF, 0xF, true))));  // row_half_mirror
    i = __float_as_int(fmaxf(__int_as_float(i), __int_as_float(__builtin_amdgcn_mov_dpp(i, 0x140, 0xF, 0xF, true))));  // row_mirror
    return __int_as_float(i);
}

// Streaming (non-temporal) vector accesses: the quantizers and the dequantizer touch every
// byte exactly once, so they bypass cache allocation; measured 1.25-1.5x over plain accesses.
typedef unsigned uintx4_t __attribute__((ext_vector_type(4)));
typedef unsigned uintx2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 load_nt16(const void* p) {
    const uintx4_t v = __builtin_nontemporal_load(static_cast<const uintx4_t*>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint2 load_nt8(const void* p) {
    const uintx2_t v = __builtin_nontemporal_load(static_cast<const uintx2_t*>(p));
    return make_uint2(v[0], v[1]);
}
__device__ __forceinline__ void store_nt16(void* p, const uint4& v) {
    const uintx4_t u = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(u, static_cast<uintx4_t*>(p));
}
__device__ __forceinline__ void store_nt8(void* p, const uint2& v) {
    const uintx2_t u = {v.x, v.y};
    __builtin_nontemporal_store(u, static_cast<uintx2_t*>(p));
}

// 8 values of row `row`, columns c0 .. c0+7, of an [N, K] matrix of type XT (0 bf16, 1 fp16, 2 fp32; element (n, k) at
// base[n * rs + k * cs]) as fp32, zeros outside the matrix.  VEC: cs == 1, all 8 columns in range, 16-byte aligned rows.
// The reference kernels load with .to(tl.float32): every input type is quantized from its exact fp32 value.
template <int XT, bool VEC>
__device__ __forceinline__ void load_row8_f32(const void* __restrict__ base, int row, int c0, int N, int K, int64_t rs, int64_t cs,
                                              float (&f)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = 0.0f;
    if (row >= N || c0 >= K) return;
    if (XT == 0) {
        const uint16_t* p = static_cast<const uint16_t*>(base) + (int64_t)row * rs;
        if (VEC) {
            const uint4 v = load_nt16(p + c0);
            f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x); f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
            f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z); f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (c0 + j < K) f[j] = bf16_one(p[(int64_t)(c0 + j) * cs]);
        }
    } else if (XT == 1) {
        const _Float16* p = static_cast<const _Float16*>(base) + (int64_t)row * rs;
        if (VEC) {
            const uint4 v = load_nt16(p + c0);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                f[2 * j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] & 0xFFFFu));
                f[2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] >> 16));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (c0 + j < K) f[j] = (float)p[(int64_t)(c0 + j) * cs];
        }
    } else {
        const float* p = static_cast<const float*>(base) + (int64_t)row * rs;
        if (VEC) {
            const uint4 a = load_nt16(p + c0), b = load_nt16(p + c0 + 4);
            f[0] = __uint_as_float(a.x); f[1] = __uint_as_float(a.y); f[2] = __uint_as_float(a.z); f[3] = __uint_as_float(a.w);
            f[4] = __uint_as_float(b.x); f[5] = __uint_as_float(b.y); f[6] = __uint_as_float(b.z); f[7] = __uint_as_float(b.w);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (c0 + j < K) f[j] = p[(int64_t)(c0 + j) * cs];
        }
    }
}
// true when the vector form of load_row8_f32 applies to a matrix of element size esz
inline bool rows_vectorizable(const void* base, int64_t K, int64_t rs, int64_t cs, int esz) {
    return cs == 1 && K % 8 == 0 && (rs * esz) % 16 == 0 && (reinterpret_cast<uintptr_t>(base) & 15) == 0;
}
inline int xt_size(int xt) { return xt == 2 ? 4 : 2; }

__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
    floatx2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    return __builtin_bit_cast(uint32_t, h);
}

// Blocks that tile a matrix, nx wide and ny high (x fastest): grid.y takes at most 65535 blocks and a token
// dimension can need more, so the block rows beyond kGridRowChunk continue in grid.z.  The last z slice may
// reach past ny: kernels drop block rows >= ny.  (A 1-D grid with a division per block measured 3-7 % slower
// for the row quantizers, whose blocks live for one load.)
constexpr int kGridRowChunk = 32768;
__device__ __forceinline__ int block_row() { return (int)(blockIdx.y + blockIdx.z * kGridRowChunk); }
// false when the blocks do not fit
inline bool grid_rows(int64_t nx, int64_t ny, dim3& grid) {
    if (nx <= 0 || ny <= 0 || nx > 0x7FFFFFFF || ny > (int64_t)65535 * kGridRowChunk) return false;
    grid = dim3((unsigned)nx, (unsigned)(ny < kGridRowChunk ? ny : kGridRowChunk), (unsigned)((ny + kGridRowChunk - 1) / kGridRowChunk));
    return true;
}
constexpr int kErrTooManyBlocks = 9;   // hipErrorInvalidConfiguration

// ---------------------------------------------------------------------------
// host-side launchers (defined one per .hip file); all return hipError_t as int
// ---------------------------------------------------------------------------
int launch_act_quant(const void* x, void* y, float* s, int64_t M, int64_t K, int64_t x_row_stride,
                     int64_t PM, int64_t PK, int64_t s_row_stride, int64_t s_col_stride, int mode,
                     hipStream_t stream);
int launch_act_quant_typed(const void* x, int x_dtype, int block_size, void* y, float* s, int64_t M, int64_t K,
                           int64_t x_row_stride, int64_t PM, int64_t PK, int64_t s_row_stride, int64_t s_col_stride, int mode,
                           hipStream_t stream);
int launch_weight_quant(const void* w, int w_dtype, void* y, float* s, void* y_t, float* s_t, int64_t N, int64_t K,
                        int64_t w_row_stride, int64_t w_col_stride, int64_t PN, int64_t PK, int mode,
                        hipStream_t stream);
int launch_quant_transpose(const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                           int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int64_t s_kb_stride,
                           int t_mode, hipStream_t stream);
int launch_act_quant_transpose(const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                               int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int mode, hipStream_t stream);
int launch_fp8_gemm_nt_rowscaled(const void* a, const float* a_s, int64_t as_rs, int64_t as_cs, const void* b,
                                 const float* b_s, int64_t bs_rs, int64_t bs_cs, void* c, int64_t M, int64_t N, int64_t K,
                                 int fmt, int out_dtype, hipStream_t stream);
int launch_swiglu(const void* x, void* act, void* y, float* s, int64_t M, int64_t N, int64_t x_row_stride,
                  int gate_first, int64_t PM, int64_t PN, int64_t s_row_stride, int64_t s_col_stride, int mode,
                  hipStream_t stream);
int launch_swiglu_bwd(const void* x, const void* dy, void* dx, int64_t M, int64_t N, int64_t x_row_stride,
                      int gate_first, hipStream_t stream);
int launch_weight_dequant(const void* x, const float* s, void* y, int64_t N, int64_t K, int block_size, int out_dtype,
                          hipStream_t stream);
int launch_fp8_gemm_nt(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                       const void* b, const float* b_s, void* c, const void* bias, int64_t M, int64_t N,
                       int64_t K, int out_dtype, hipStream_t stream);
int launch_fp8_gemm_nt_e5m2(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                            const void* b, const float* b_s, void* c, const void* bias, int64_t M, int64_t N,
                            int64_t K, int out_dtype, hipStream_t stream);
int64_t fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int launch_fp8_gemm_nt_ws(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                          const void* b, const float* b_s, void* c, const void* bias, int64_t M, int64_t N,
                          int64_t K, int out_dtype, void* workspace, int64_t workspace_bytes, hipStream_t stream);
int fp8_gemm_path(const void* a, const void* b, int64_t as_rs, int64_t as_cs, int64_t M, int64_t N, int64_t K,
                  int with_workspace);
// static device scratch of the no-allocation GEMM entry point (defined in fp8_gemm.hip)
constexpr int64_t kStaticScratchBytes = (int64_t)32 << 20;
int static_scratch_ptr(void** out);
int launch_fp8_gemm_nt_static(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                              const void* b, const float* b_s, void* c, const void* bias, int64_t M, int64_t N,
                              int64_t K, int out_dtype, hipStream_t stream);
int launch_fp8_grouped_gemm_nt(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                               const void* b, const float* b_s, void* c, const void* bias, const int64_t* m_splits,
                               int64_t G, int64_t M, int64_t N, int64_t K, int out_dtype, hipStream_t stream);
int launch_group_pad(const void* x, void* y, const int64_t* m_splits, int64_t G, int64_t row_bytes, int64_t multiple,
                     int unpad, hipStream_t stream);
int launch_add_grad(void* x, const void* y, int64_t n, int x_dtype, int y_dtype, hipStream_t stream);
int launch_add_bias(void* x, const void* b, int b_dtype, int64_t M, int64_t N, hipStream_t stream);
int launch_cast_f32_to_e4m3(const float* x, void* y, int64_t n, int saturate, hipStream_t stream);
int launch_cast_f32_to_e5m2(const float* x, void* y, int64_t n, hipStream_t stream);
int launch_quotient_selfcheck(uint64_t* out, int amax_lo, int amax_hi, int mode, hipStream_t stream);

}  // namespace mdy
