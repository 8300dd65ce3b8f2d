// extern "C" entry points of libmdyfp8.so: argument validation + dispatch.
// Declarations and the reference interface each one replaces: include/mdy_fp8.h.
#include "../../include/mdy_fp8.h"

#include <cstdarg>
#include <cstdio>

#include "common.h"

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int launched(int hip_err, const char* what) {
    if (hip_err == 0) return 0;
    return fail(hip_err, "%s: launch failed: %s", what, hipGetErrorString(static_cast<hipError_t>(hip_err)));
}

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

constexpr int64_t kMaxDim = (int64_t)1 << 30;  // kernels index rows/columns with 32-bit ints

// The kernels are built for gfx950 only; refuse to launch elsewhere instead of
// letting the runtime fail with a missing code object.
int check_device() {
    static thread_local int cached_dev = -1;
    static thread_local int cached_ok = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(MDY_E_DEVICE, "no HIP device is current");
    if (dev != cached_dev) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return fail(MDY_E_DEVICE, "cannot query device %d", dev);
        cached_ok = (__builtin_strncmp(prop.gcnArchName, "gfx950", 6) == 0);
        cached_dev = dev;
        if (!cached_ok) return fail(MDY_E_DEVICE, "device %d is %s, this library is built for gfx950", dev, prop.gcnArchName);
    }
    if (!cached_ok) return fail(MDY_E_DEVICE, "device %d is not gfx950", dev);
    return 0;
}

}  // namespace

extern "C" {

int mdy_fp8_abi_version(void) { return MDY_FP8_ABI_VERSION; }

const char* mdy_fp8_last_error(void) { return g_err; }

int mdy_act_quant(const void* x, void* y, float* s, int64_t M, int64_t K, int64_t x_row_stride, int64_t PM,
                  int64_t PK, int64_t s_row_stride, int64_t s_col_stride, int mode, void* stream) {
    if (mode != MDY_QUANT_OFFICIAL && mode != MDY_QUANT_DEEPLINEAR) return fail(MDY_E_DTYPE, "act_quant: unknown mode %d", mode);
    if (M < 0 || K < 0 || PM < M || PK < K || PM > kMaxDim || PK > kMaxDim)
        return fail(MDY_E_SHAPE, "act_quant: need 0 <= M <= PM, 0 <= K <= PK (M=%lld K=%lld PM=%lld PK=%lld)",
                    (long long)M, (long long)K, (long long)PM, (long long)PK);
    if (PK % 128 != 0) return fail(MDY_E_SHAPE, "act_quant: PK=%lld is not a multiple of 128", (long long)PK);
    if (PM == 0 || PK == 0) return 0;
    if (!y || !s || (!x && M > 0 && K > 0)) return fail(MDY_E_NULL, "act_quant: null pointer");
    // rows may overlap only as a broadcast (stride 0, an expanded tensor); a single row has no stride to speak of
    if (M > 1 && x_row_stride != 0 && x_row_stride < K)
        return fail(MDY_E_SHAPE, "act_quant: x_row_stride=%lld < K=%lld (and not 0)", (long long)x_row_stride, (long long)K);
    if (!aligned(y, 8)) return fail(MDY_E_ALIGN, "act_quant: y must be 8-byte aligned");
    if (!aligned(x, 2) || !aligned(s, 4)) return fail(MDY_E_ALIGN, "act_quant: x/s misaligned for their element type");
    if (int e = check_device()) return e;
    return launched(mdy::launch_act_quant(x, y, s, M, K, x_row_stride, PM, PK, s_row_stride, s_col_stride, mode,
                                          static_cast<hipStream_t>(stream)),
                    "act_quant");
}

static bool block_size_ok(int64_t bs, int64_t lo, int64_t hi) { return bs >= lo && bs <= hi && (bs & (bs - 1)) == 0; }

int mdy_act_quant_typed(const void* x, int x_dtype, int block_size, void* y, float* s, int64_t M, int64_t K, int64_t x_row_stride,
                        int64_t PM, int64_t PK, int64_t s_row_stride, int64_t s_col_stride, int mode, void* stream) {
    if (x_dtype == MDY_XT_BF16 && block_size == 128 && mode != MDY_QUANT_OFFICIAL_E5M2)
        return mdy_act_quant(x, y, s, M, K, x_row_stride, PM, PK, s_row_stride, s_col_stride, mode, stream);
    if (x_dtype != MDY_XT_BF16 && x_dtype != MDY_XT_F16 && x_dtype != MDY_XT_F32) return fail(MDY_E_DTYPE, "act_quant_typed: unknown x_dtype %d", x_dtype);
    if (mode != MDY_QUANT_OFFICIAL && mode != MDY_QUANT_DEEPLINEAR && mode != MDY_QUANT_OFFICIAL_E5M2) return fail(MDY_E_DTYPE, "act_quant_typed: unknown mode %d", mode);
    if (!block_size_ok(block_size, 8, 512)) return fail(MDY_E_SHAPE, "act_quant_typed: block_size=%d must be a power of two from 8 to 512", block_size);
    if (M < 0 || K < 0 || PM < M || PK < K || PM > kMaxDim || PK > kMaxDim)
        return fail(MDY_E_SHAPE, "act_quant_typed: need 0 <= M <= PM, 0 <= K <= PK");
    if (PK % block_size != 0) return fail(MDY_E_SHAPE, "act_quant_typed: PK=%lld is not a multiple of block_size=%d", (long long)PK, block_size);
    if (PM == 0 || PK == 0) return 0;
    if (!y || !s || (!x && M > 0 && K > 0)) return fail(MDY_E_NULL, "act_quant_typed: null pointer");
    if (M > 1 && x_row_stride != 0 && x_row_stride < K) return fail(MDY_E_SHAPE, "act_quant_typed: x_row_stride < K (and not 0)");
    if (!aligned(y, 8) || !aligned(s, 4) || !aligned(x, x_dtype == MDY_XT_F32 ? 4 : 2))
        return fail(MDY_E_ALIGN, "act_quant_typed: y must be 8-byte aligned, x and s aligned for their element type");
    if (int e = check_device()) return e;
    return launched(mdy::launch_act_quant_typed(x, x_dtype, block_size, y, s, M, K, x_row_stride, PM, PK, s_row_stride, s_col_stride,
                                                mode, static_cast<hipStream_t>(stream)),
                    "act_quant_typed");
}

int mdy_weight_quant_typed(const void* w, int w_dtype, void* y, float* s, void* y_t, float* s_t, int64_t N, int64_t K,
                           int64_t w_row_stride, int64_t w_col_stride, int64_t PN, int64_t PK, int mode, void* stream) {
    if (w_dtype != MDY_XT_BF16 && w_dtype != MDY_XT_F16 && w_dtype != MDY_XT_F32) return fail(MDY_E_DTYPE, "weight_quant: unknown w_dtype %d", w_dtype);
    if (mode != MDY_QUANT_OFFICIAL && mode != MDY_QUANT_DEEPLINEAR && mode != MDY_QUANT_OFFICIAL_E5M2) return fail(MDY_E_DTYPE, "weight_quant: unknown mode %d", mode);
    if (N < 0 || K < 0 || PN < N || PK < K || PN > kMaxDim || PK > kMaxDim)
        return fail(MDY_E_SHAPE, "weight_quant: need 0 <= N <= PN, 0 <= K <= PK");
    if (PN % 128 != 0 || PK % 128 != 0) return fail(MDY_E_SHAPE, "weight_quant: PN=%lld, PK=%lld must be multiples of 128", (long long)PN, (long long)PK);
    if ((y_t == nullptr) != (s_t == nullptr)) return fail(MDY_E_NULL, "weight_quant: y_t and s_t must be given together");
    if ((y == nullptr) != (s == nullptr)) return fail(MDY_E_NULL, "weight_quant: y and s must be given together");
    if (PN == 0 || PK == 0) return 0;
    if ((!y && !y_t) || (!w && N > 0 && K > 0)) return fail(MDY_E_NULL, "weight_quant: null pointer");
    if ((y && !aligned(y, 8)) || (y_t && !aligned(y_t, 8))) return fail(MDY_E_ALIGN, "weight_quant: y / y_t must be 8-byte aligned");
    if (int e = check_device()) return e;
    return launched(mdy::launch_weight_quant(w, w_dtype, y, s, y_t, s_t, N, K, w_row_stride, w_col_stride, PN, PK, mode,
                                             static_cast<hipStream_t>(stream)),
                    "weight_quant");
}

int mdy_weight_quant(const void* w, void* y, float* s, void* y_t, float* s_t, int64_t N, int64_t K,
                     int64_t w_row_stride, int64_t w_col_stride, int64_t PN, int64_t PK, int mode, void* stream) {
    return mdy_weight_quant_typed(w, MDY_XT_BF16, y, s, y_t, s_t, N, K, w_row_stride, w_col_stride, PN, PK, mode, stream);
}

int mdy_quant_transpose_typed(const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                              int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int64_t s_kb_stride, int t_mode,
                              void* stream) {
    if (x_dtype != MDY_XT_BF16 && x_dtype != MDY_XT_F16 && x_dtype != MDY_XT_F32) return fail(MDY_E_DTYPE, "quant_transpose: unknown x_dtype %d", x_dtype);
    if (t_mode != MDY_T_COLUMN && t_mode != MDY_T_BLOCK) return fail(MDY_E_DTYPE, "quant_transpose: unknown t_mode %d", t_mode);
    if (M < 0 || K < 0 || PM < M || PK < K || PM > kMaxDim || PK > kMaxDim)
        return fail(MDY_E_SHAPE, "quant_transpose: need 0 <= M <= PM, 0 <= K <= PK");
    if (PM % 128 != 0 || PK % 128 != 0) return fail(MDY_E_SHAPE, "quant_transpose: PM=%lld, PK=%lld must be multiples of 128", (long long)PM, (long long)PK);
    if (s_kb_stride < PM) return fail(MDY_E_SHAPE, "quant_transpose: s_kb_stride=%lld < PM=%lld", (long long)s_kb_stride, (long long)PM);
    if (PM == 0 || PK == 0) return 0;
    if (!y || !s || !y_t || !s_t || (!x && M > 0 && K > 0)) return fail(MDY_E_NULL, "quant_transpose: null pointer");
    if (!aligned(y, 8) || !aligned(y_t, 8)) return fail(MDY_E_ALIGN, "quant_transpose: y / y_t must be 8-byte aligned");
    if (!aligned(x, x_dtype == MDY_XT_F32 ? 4 : 2) || !aligned(s, 4) || !aligned(s_t, 4)) return fail(MDY_E_ALIGN, "quant_transpose: x/s/s_t misaligned for their element type");
    if (int e = check_device()) return e;
    return launched(mdy::launch_quant_transpose(x, x_dtype, y, s, y_t, s_t, M, K, x_row_stride, x_col_stride, PM, PK, s_kb_stride,
                                                t_mode, static_cast<hipStream_t>(stream)),
                    "quant_transpose");
}

int mdy_quant_transpose(const void* x, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                        int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int64_t s_kb_stride, int t_mode,
                        void* stream) {
    return mdy_quant_transpose_typed(x, MDY_XT_BF16, y, s, y_t, s_t, M, K, x_row_stride, x_col_stride, PM, PK, s_kb_stride, t_mode,
                                     stream);
}

int mdy_act_quant_transpose(const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                            int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int mode, void* stream) {
    if (mode != MDY_QUANT_OFFICIAL && mode != MDY_QUANT_OFFICIAL_E5M2) return fail(MDY_E_DTYPE, "act_quant_transpose: mode must be MDY_QUANT_OFFICIAL or MDY_QUANT_OFFICIAL_E5M2");
    if (x_dtype != MDY_XT_BF16 && x_dtype != MDY_XT_F16 && x_dtype != MDY_XT_F32) return fail(MDY_E_DTYPE, "act_quant_transpose: unknown x_dtype %d", x_dtype);
    if (M < 0 || K < 0 || PM < M || PK < K || PM > kMaxDim || PK > kMaxDim)
        return fail(MDY_E_SHAPE, "act_quant_transpose: need 0 <= M <= PM, 0 <= K <= PK");
    if (PM % 128 != 0 || PK % 128 != 0) return fail(MDY_E_SHAPE, "act_quant_transpose: PM=%lld, PK=%lld must be multiples of 128", (long long)PM, (long long)PK);
    if ((y == nullptr) != (s == nullptr)) return fail(MDY_E_NULL, "act_quant_transpose: y and s must be given together");
    if (PM == 0 || PK == 0) return 0;
    if (!y_t || !s_t || (!x && M > 0 && K > 0)) return fail(MDY_E_NULL, "act_quant_transpose: null pointer");
    if ((y && !aligned(y, 8)) || !aligned(y_t, 8)) return fail(MDY_E_ALIGN, "act_quant_transpose: y / y_t must be 8-byte aligned");
    if (!aligned(x, x_dtype == MDY_XT_F32 ? 4 : 2) || (s && !aligned(s, 4)) || !aligned(s_t, 4)) return fail(MDY_E_ALIGN, "act_quant_transpose: x/s/s_t misaligned for their element type");
    if (int e = check_device()) return e;
    return launched(mdy::launch_act_quant_transpose(x, x_dtype, y, s, y_t, s_t, M, K, x_row_stride, x_col_stride, PM, PK, mode,
                                                    static_cast<hipStream_t>(stream)),
                    "act_quant_transpose");
}

int mdy_fp8_gemm_nt_rowscaled(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                              const float* b_s, int64_t bs_row_stride, int64_t bs_col_stride, void* c, int64_t M, int64_t N,
                              int64_t K, int fmt, int out_dtype, void* stream) {
    if (fmt != MDY_FMT_E4M3 && fmt != MDY_FMT_E5M2) return fail(MDY_E_DTYPE, "fp8_gemm_nt_rowscaled: unknown operand format %d", fmt);
    if (out_dtype != MDY_DT_BF16 && out_dtype != MDY_DT_F32) return fail(MDY_E_DTYPE, "fp8_gemm_nt_rowscaled: unknown out_dtype %d", out_dtype);
    if (M < 0 || N < 0 || K < 128 || K % 128 != 0 || M > kMaxDim || N > kMaxDim || K > (1 << 20))
        return fail(MDY_E_SHAPE, "fp8_gemm_nt_rowscaled: needs K a multiple of 128 up to 2^20 (M=%lld N=%lld K=%lld)", (long long)M,
                    (long long)N, (long long)K);
    if (M == 0 || N == 0) return 0;
    if (!a || !a_s || !b || !b_s || !c) return fail(MDY_E_NULL, "fp8_gemm_nt_rowscaled: null pointer");
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(c, out_dtype == MDY_DT_BF16 ? 2 : 4) || !aligned(a_s, 4) || !aligned(b_s, 4))
        return fail(MDY_E_ALIGN, "fp8_gemm_nt_rowscaled: a and b must be 16-byte aligned, c and the scales aligned for their type");
    if (int e = check_device()) return e;
    const int rc = mdy::launch_fp8_gemm_nt_rowscaled(a, a_s, as_row_stride, as_col_stride, b, b_s, bs_row_stride, bs_col_stride, c,
                                                     M, N, K, fmt, out_dtype, static_cast<hipStream_t>(stream));
    if (rc == -1) return fail(MDY_E_SHAPE, "fp8_gemm_nt_rowscaled: scale strides must be non-negative and span less than 2^31 bytes");
    return launched(rc, "fp8_gemm_nt_rowscaled");
}

int mdy_swiglu(const void* x, void* act, void* y, float* s, int64_t M, int64_t N, int64_t x_row_stride, int gate_first,
               int64_t PM, int64_t PN, int64_t s_row_stride, int64_t s_col_stride, int mode, void* stream) {
    if (M < 0 || N < 0 || M > kMaxDim || 2 * N > kMaxDim) return fail(MDY_E_SHAPE, "swiglu: bad shape M=%lld N=%lld", (long long)M, (long long)N);
    if (!act && !y) return fail(MDY_E_NULL, "swiglu: neither act nor y given");
    if (y) {
        if (mode != MDY_QUANT_OFFICIAL && mode != MDY_QUANT_DEEPLINEAR) return fail(MDY_E_DTYPE, "swiglu: unknown mode %d", mode);
        if (PM < M || PN < N || PM > kMaxDim || PN > kMaxDim) return fail(MDY_E_SHAPE, "swiglu: need M <= PM, N <= PN");
        if (PN % 128 != 0) return fail(MDY_E_SHAPE, "swiglu: PN=%lld is not a multiple of 128", (long long)PN);
        if (PM == 0 || PN == 0) return 0;
        if (!s) return fail(MDY_E_NULL, "swiglu: y given without s");
        if (!aligned(y, 8) || !aligned(s, 4)) return fail(MDY_E_ALIGN, "swiglu: y must be 8-byte, s 4-byte aligned");
    } else {
        if (M == 0 || N == 0) return 0;
    }
    if (!x && M > 0 && N > 0) return fail(MDY_E_NULL, "swiglu: null x");
    if (M > 0 && x_row_stride < 2 * N) return fail(MDY_E_SHAPE, "swiglu: x_row_stride=%lld < 2N=%lld", (long long)x_row_stride, (long long)(2 * N));
    if (!aligned(x, 2) || (act && !aligned(act, 2))) return fail(MDY_E_ALIGN, "swiglu: x/act misaligned for bf16");
    if (int e = check_device()) return e;
    return launched(mdy::launch_swiglu(x, act, y, s, M, N, x_row_stride, gate_first != 0, PM, PN, s_row_stride, s_col_stride,
                                       mode, static_cast<hipStream_t>(stream)),
                    "swiglu");
}

int mdy_swiglu_bwd(const void* x, const void* dy, void* dx, int64_t M, int64_t N, int64_t x_row_stride, int gate_first,
                   void* stream) {
    if (M < 0 || N < 0 || M > kMaxDim || 2 * N > kMaxDim) return fail(MDY_E_SHAPE, "swiglu_bwd: bad shape");
    if (M == 0 || N == 0) return 0;
    if (!x || !dy || !dx) return fail(MDY_E_NULL, "swiglu_bwd: null pointer");
    if (x_row_stride < 2 * N) return fail(MDY_E_SHAPE, "swiglu_bwd: x_row_stride < 2N");
    if (!aligned(x, 2) || !aligned(dy, 2) || !aligned(dx, 2)) return fail(MDY_E_ALIGN, "swiglu_bwd: misaligned pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_swiglu_bwd(x, dy, dx, M, N, x_row_stride, gate_first != 0, static_cast<hipStream_t>(stream)),
                    "swiglu_bwd");
}

int mdy_weight_dequant_block(const void* x, const float* s, void* y, int64_t N, int64_t K, int block_size, int out_dtype,
                             void* stream) {
    if (out_dtype != MDY_DT_BF16 && out_dtype != MDY_DT_F32) return fail(MDY_E_DTYPE, "weight_dequant: unknown out_dtype %d", out_dtype);
    if (!block_size_ok(block_size, 8, 1 << 20)) return fail(MDY_E_SHAPE, "weight_dequant: block_size=%d must be a power of two >= 8", block_size);
    if (N < 0 || K < 0 || N > kMaxDim || K > kMaxDim) return fail(MDY_E_SHAPE, "weight_dequant: bad shape");
    if (N == 0 || K == 0) return 0;
    if (!x || !s || !y) return fail(MDY_E_NULL, "weight_dequant: null pointer");
    if (!aligned(y, out_dtype == MDY_DT_BF16 ? 2 : 4) || !aligned(s, 4)) return fail(MDY_E_ALIGN, "weight_dequant: misaligned pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_weight_dequant(x, s, y, N, K, block_size, out_dtype, static_cast<hipStream_t>(stream)), "weight_dequant");
}

int mdy_weight_dequant(const void* x, const float* s, void* y, int64_t N, int64_t K, int out_dtype, void* stream) {
    return mdy_weight_dequant_block(x, s, y, N, K, 128, out_dtype, stream);
}

int mdy_fp8_gemm_nt(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                    const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                    void* stream) {
    if (out_dtype != MDY_DT_BF16 && out_dtype != MDY_DT_F32) return fail(MDY_E_DTYPE, "fp8_gemm_nt: unknown out_dtype %d", out_dtype);
    if (M < 0 || N < 0 || K < 1 || M > kMaxDim || N > kMaxDim || K > kMaxDim)
        return fail(MDY_E_SHAPE, "fp8_gemm_nt: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    if (M == 0 || N == 0) return 0;
    if (!a || !a_s || !b || !b_s || !c) return fail(MDY_E_NULL, "fp8_gemm_nt: null pointer");
    if (!aligned(c, out_dtype == MDY_DT_BF16 ? 2 : 4) || !aligned(a_s, 4) || !aligned(b_s, 4) || (bias && !aligned(bias, 2)))
        return fail(MDY_E_ALIGN, "fp8_gemm_nt: misaligned pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_fp8_gemm_nt(a, a_s, as_row_stride, as_col_stride, b, b_s, c, bias, M, N, K, out_dtype,
                                            static_cast<hipStream_t>(stream)),
                    "fp8_gemm_nt");
}

int mdy_fp8_gemm_nt_e5m2(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                         const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                         void* stream) {
    if (out_dtype != MDY_DT_BF16 && out_dtype != MDY_DT_F32) return fail(MDY_E_DTYPE, "fp8_gemm_nt_e5m2: unknown out_dtype %d", out_dtype);
    if (M < 0 || N < 0 || K < 1 || M > kMaxDim || N > kMaxDim || K > kMaxDim)
        return fail(MDY_E_SHAPE, "fp8_gemm_nt_e5m2: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    if (M == 0 || N == 0) return 0;
    if (!a || !a_s || !b || !b_s || !c) return fail(MDY_E_NULL, "fp8_gemm_nt_e5m2: null pointer");
    if (!aligned(c, out_dtype == MDY_DT_BF16 ? 2 : 4) || !aligned(a_s, 4) || !aligned(b_s, 4) || (bias && !aligned(bias, 2)))
        return fail(MDY_E_ALIGN, "fp8_gemm_nt_e5m2: misaligned pointer");
    if (int e = check_device()) return e;
    const int rc = mdy::launch_fp8_gemm_nt_e5m2(a, a_s, as_row_stride, as_col_stride, b, b_s, c, bias, M, N, K, out_dtype,
                                                static_cast<hipStream_t>(stream));
    if (rc == -1)
        return fail(MDY_E_SHAPE, "fp8_gemm_nt_e5m2: needs K a multiple of 128 up to 65536, 16-byte aligned a and b, activation scales within 2^31 bytes "
                    "(other e5m2 problems: mdy_fp8_gemm_nt_rowscaled with the weight scales expanded to one per row)");
    return launched(rc, "fp8_gemm_nt_e5m2");
}

int64_t mdy_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K < 1 || M > kMaxDim || N > kMaxDim || K > kMaxDim) return 0;
    return mdy::fp8_gemm_workspace_bytes(M, N, K);
}

int mdy_fp8_gemm_nt_ws(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                       const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                       void* workspace, int64_t workspace_bytes, void* stream) {
    if (out_dtype != MDY_DT_BF16 && out_dtype != MDY_DT_F32) return fail(MDY_E_DTYPE, "fp8_gemm_nt_ws: unknown out_dtype %d", out_dtype);
    if (M < 0 || N < 0 || K < 1 || M > kMaxDim || N > kMaxDim || K > kMaxDim)
        return fail(MDY_E_SHAPE, "fp8_gemm_nt_ws: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    if (workspace_bytes < 0) return fail(MDY_E_SHAPE, "fp8_gemm_nt_ws: workspace_bytes < 0");
    if (M == 0 || N == 0) return 0;
    if (!a || !a_s || !b || !b_s || !c) return fail(MDY_E_NULL, "fp8_gemm_nt_ws: null pointer");
    if (!aligned(c, out_dtype == MDY_DT_BF16 ? 2 : 4) || !aligned(a_s, 4) || !aligned(b_s, 4) || (bias && !aligned(bias, 2)))
        return fail(MDY_E_ALIGN, "fp8_gemm_nt_ws: misaligned pointer");
    if (workspace && !aligned(workspace, 16)) return fail(MDY_E_ALIGN, "fp8_gemm_nt_ws: workspace must be 16-byte aligned");
    if (int e = check_device()) return e;
    return launched(mdy::launch_fp8_gemm_nt_ws(a, a_s, as_row_stride, as_col_stride, b, b_s, c, bias, M, N, K, out_dtype,
                                               workspace, workspace_bytes, static_cast<hipStream_t>(stream)),
                    "fp8_gemm_nt_ws");
}

int mdy_fp8_gemm_path(const void* a, const void* b, int64_t as_row_stride, int64_t as_col_stride, int64_t M, int64_t N,
                      int64_t K, int with_workspace) {
    if (M < 1 || N < 1 || K < 1 || M > kMaxDim || N > kMaxDim || K > kMaxDim)
        return fail(MDY_E_SHAPE, "fp8_gemm_path: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    return mdy::fp8_gemm_path(a, b, as_row_stride, as_col_stride, M, N, K, with_workspace);
}

int64_t mdy_fp8_gemm_static_workspace_bytes(void) { return mdy::kStaticScratchBytes; }

int mdy_fp8_gemm_static_workspace_init(void) {
    if (int e = check_device()) return e;
    void* p = nullptr;
    return launched(mdy::static_scratch_ptr(&p), "fp8_gemm_static_workspace_init");
}

int mdy_fp8_gemm_nt_static_ws(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                              const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                              void* stream) {
    if (out_dtype != MDY_DT_BF16 && out_dtype != MDY_DT_F32) return fail(MDY_E_DTYPE, "fp8_gemm_nt_static_ws: unknown out_dtype %d", out_dtype);
    if (M < 0 || N < 0 || K < 1 || M > kMaxDim || N > kMaxDim || K > kMaxDim)
        return fail(MDY_E_SHAPE, "fp8_gemm_nt_static_ws: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    if (M == 0 || N == 0) return 0;
    if (!a || !a_s || !b || !b_s || !c) return fail(MDY_E_NULL, "fp8_gemm_nt_static_ws: null pointer");
    if (!aligned(c, out_dtype == MDY_DT_BF16 ? 2 : 4) || !aligned(a_s, 4) || !aligned(b_s, 4) || (bias && !aligned(bias, 2)))
        return fail(MDY_E_ALIGN, "fp8_gemm_nt_static_ws: misaligned pointer");
    const int64_t need = mdy::fp8_gemm_workspace_bytes(M, N, K);
    if (need > mdy::kStaticScratchBytes)
        return fail(MDY_E_SHAPE, "fp8_gemm_nt_static_ws: M=%lld N=%lld K=%lld needs %lld bytes of scratch, the static buffer holds %lld; "
                    "use mdy_fp8_gemm_nt_ws with a caller-owned workspace (or mdy_fp8_gemm_nt)",
                    (long long)M, (long long)N, (long long)K, (long long)need, (long long)mdy::kStaticScratchBytes);
    if (int e = check_device()) return e;
    return launched(mdy::launch_fp8_gemm_nt_static(a, a_s, as_row_stride, as_col_stride, b, b_s, c, bias, M, N, K, out_dtype,
                                                   static_cast<hipStream_t>(stream)),
                    "fp8_gemm_nt_static_ws");
}

int mdy_fp8_grouped_gemm_nt(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                            const float* b_s, void* c, const void* bias, const int64_t* m_splits, int64_t G, int64_t N,
                            int64_t K, int out_dtype, void* stream) {
    if (out_dtype != MDY_DT_BF16 && out_dtype != MDY_DT_F32) return fail(MDY_E_DTYPE, "fp8_grouped_gemm_nt: unknown out_dtype %d", out_dtype);
    if (G < 0 || G > (1 << 20) || N < 0 || K < 1 || N > kMaxDim || K > kMaxDim)
        return fail(MDY_E_SHAPE, "fp8_grouped_gemm_nt: bad shape G=%lld N=%lld K=%lld", (long long)G, (long long)N, (long long)K);
    if (G == 0 || N == 0) return 0;
    if (!m_splits) return fail(MDY_E_NULL, "fp8_grouped_gemm_nt: null m_splits");
    int64_t M = 0;
    for (int64_t g = 0; g < G; ++g) {
        if (m_splits[g] < 0 || m_splits[g] > kMaxDim) return fail(MDY_E_SHAPE, "fp8_grouped_gemm_nt: m_splits[%lld]=%lld", (long long)g, (long long)m_splits[g]);
        M += m_splits[g];
    }
    if (M > kMaxDim) return fail(MDY_E_SHAPE, "fp8_grouped_gemm_nt: too many rows (%lld)", (long long)M);
    if (M == 0) return 0;
    if (!a || !a_s || !b || !b_s || !c) return fail(MDY_E_NULL, "fp8_grouped_gemm_nt: null pointer");
    if (!aligned(c, out_dtype == MDY_DT_BF16 ? 2 : 4) || !aligned(a_s, 4) || !aligned(b_s, 4) || (bias && !aligned(bias, 2)))
        return fail(MDY_E_ALIGN, "fp8_grouped_gemm_nt: misaligned pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_fp8_grouped_gemm_nt(a, a_s, as_row_stride, as_col_stride, b, b_s, c, bias, m_splits, G, M, N, K,
                                                    out_dtype, static_cast<hipStream_t>(stream)),
                    "fp8_grouped_gemm_nt");
}

int mdy_group_pad_rows(const void* x, void* y, const int64_t* m_splits, int64_t G, int64_t row_bytes, int64_t multiple,
                       int unpad, void* stream) {
    if (G < 0 || G > (1 << 20) || row_bytes < 0 || row_bytes > ((int64_t)1 << 32) || multiple < 1 || multiple > (1 << 20))
        return fail(MDY_E_SHAPE, "group_pad_rows: bad G=%lld / row_bytes=%lld / multiple=%lld", (long long)G, (long long)row_bytes,
                    (long long)multiple);
    if (G == 0 || row_bytes == 0) return 0;
    if (!m_splits) return fail(MDY_E_NULL, "group_pad_rows: null m_splits");
    int64_t rows = 0, padded = 0;
    for (int64_t g = 0; g < G; ++g) {
        if (m_splits[g] < 0 || m_splits[g] > kMaxDim) return fail(MDY_E_SHAPE, "group_pad_rows: m_splits[%lld]=%lld", (long long)g, (long long)m_splits[g]);
        rows += m_splits[g];
        padded += (m_splits[g] + multiple - 1) / multiple * multiple;
    }
    if (padded > ((int64_t)1 << 36)) return fail(MDY_E_SHAPE, "group_pad_rows: too many rows (%lld)", (long long)padded);
    if ((unpad ? rows : padded) == 0) return 0;
    if (!y || (!x && (unpad ? padded : rows) > 0)) return fail(MDY_E_NULL, "group_pad_rows: null pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_group_pad(x, y, m_splits, G, row_bytes, multiple, unpad, static_cast<hipStream_t>(stream)),
                    "group_pad_rows");
}

int mdy_add_bias_typed(void* x, const void* b, int b_dtype, int64_t M, int64_t N, void* stream) {
    if (b_dtype != MDY_XT_BF16 && b_dtype != MDY_XT_F16 && b_dtype != MDY_XT_F32) return fail(MDY_E_DTYPE, "add_bias: unknown b_dtype %d", b_dtype);
    if (M < 0 || N < 0 || M > kMaxDim || N > kMaxDim) return fail(MDY_E_SHAPE, "add_bias: bad shape");
    if (M == 0 || N == 0) return 0;
    if (!x || !b) return fail(MDY_E_NULL, "add_bias: null pointer");
    if (!aligned(x, 2) || !aligned(b, b_dtype == MDY_XT_F32 ? 4 : 2)) return fail(MDY_E_ALIGN, "add_bias: misaligned pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_add_bias(x, b, b_dtype, M, N, static_cast<hipStream_t>(stream)), "add_bias");
}

int mdy_add_bias(void* x, const void* b, int64_t M, int64_t N, void* stream) {
    return mdy_add_bias_typed(x, b, MDY_XT_BF16, M, N, stream);
}

int mdy_add_grad(void* x, const void* y, int64_t n, int x_dtype, int y_dtype, void* stream) {
    if ((x_dtype != MDY_DT_BF16 && x_dtype != MDY_DT_F32) || (y_dtype != MDY_DT_BF16 && y_dtype != MDY_DT_F32))
        return fail(MDY_E_DTYPE, "add_grad: dtypes must be MDY_DT_BF16 or MDY_DT_F32");
    if (n < 0) return fail(MDY_E_SHAPE, "add_grad: n < 0");
    if (n == 0) return 0;
    if (!x || !y) return fail(MDY_E_NULL, "add_grad: null pointer");
    if (!aligned(x, x_dtype == MDY_DT_BF16 ? 2 : 4) || !aligned(y, y_dtype == MDY_DT_BF16 ? 2 : 4))
        return fail(MDY_E_ALIGN, "add_grad: misaligned pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_add_grad(x, y, n, x_dtype, y_dtype, static_cast<hipStream_t>(stream)), "add_grad");
}

int mdy_cast_f32_to_e4m3(const float* x, void* y, int64_t n, int saturate, void* stream) {
    if (n < 0) return fail(MDY_E_SHAPE, "cast_f32_to_e4m3: n < 0");
    if (n == 0) return 0;
    if (!x || !y) return fail(MDY_E_NULL, "cast_f32_to_e4m3: null pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_cast_f32_to_e4m3(x, y, n, saturate, static_cast<hipStream_t>(stream)), "cast_f32_to_e4m3");
}

int mdy_cast_f32_to_e5m2(const float* x, void* y, int64_t n, void* stream) {
    if (n < 0) return fail(MDY_E_SHAPE, "cast_f32_to_e5m2: n < 0");
    if (n == 0) return 0;
    if (!x || !y) return fail(MDY_E_NULL, "cast_f32_to_e5m2: null pointer");
    if (int e = check_device()) return e;
    return launched(mdy::launch_cast_f32_to_e5m2(x, y, n, static_cast<hipStream_t>(stream)), "cast_f32_to_e5m2");
}

int mdy_quotient_selfcheck(uint64_t* out, int amax_lo, int amax_hi, int mode, void* stream) {
    if (!out) return fail(MDY_E_NULL, "quotient_selfcheck: null pointer");
    if (amax_lo < 0 || amax_hi > 0x7F80 || amax_lo > amax_hi) return fail(MDY_E_SHAPE, "quotient_selfcheck: range must lie in [0, 0x7F80]");
    if (mode != 0 && mode != 1) return fail(MDY_E_DTYPE, "quotient_selfcheck: unknown mode");
    if (int e = check_device()) return e;
    return launched(mdy::launch_quotient_selfcheck(out, amax_lo, amax_hi, mode, static_cast<hipStream_t>(stream)), "quotient_selfcheck");
}

}  // extern "C"
