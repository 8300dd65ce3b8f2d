// In-place row-broadcast bias add on a bf16 matrix:
//   x[m, n] = bf16( fp32(x[m, n]) + fp32(b[n]) )
// Restates _add_bias_kernel (/root/reference/triton_kernels/dpsk_fp8linear/fp8.py:283-295).
// Streaming kernel: 8 bf16 (16 bytes) per lane, bias slice re-read from L2.
// The GEMM entry point folds the same add into its epilogue; this kernel is for
// callers that use add_bias on its own.
#include "common.h"

namespace mdy {

// BT: type of the bias (0 bf16, 1 fp16, 2 fp32; the reference loads it with .to(tl.float32), fp8.py:291); VEC: whole
// 16-byte pieces of x, and of a bf16 bias.
template <bool VEC, int BT>
__global__ __launch_bounds__(256) void add_bias_kernel(uint16_t* __restrict__ x, const void* __restrict__ bv, int M,
                                                        int N) {
    const int col = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (col >= N) return;
    float bias[8];
    if (VEC && BT == 0) {
        const uint4 v = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(bv) + col);
        bias[0] = bf16_lo(v.x); bias[1] = bf16_hi(v.x); bias[2] = bf16_lo(v.y); bias[3] = bf16_hi(v.y);
        bias[4] = bf16_lo(v.z); bias[5] = bf16_hi(v.z); bias[6] = bf16_lo(v.w); bias[7] = bf16_hi(v.w);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            bias[i] = 0.0f;
            if (col + i < N)
                bias[i] = BT == 0 ? bf16_one(static_cast<const uint16_t*>(bv)[col + i])
                        : BT == 1 ? (float)static_cast<const _Float16*>(bv)[col + i] : static_cast<const float*>(bv)[col + i];
        }
    }
    for (int row = blockIdx.y; row < M; row += gridDim.y) {
        uint16_t* p = x + (int64_t)row * N + col;
        if (VEC) {
            uint4 v = *reinterpret_cast<const uint4*>(p);
            v.x = pack2_bf16(bf16_lo(v.x) + bias[0], bf16_hi(v.x) + bias[1]);
            v.y = pack2_bf16(bf16_lo(v.y) + bias[2], bf16_hi(v.y) + bias[3]);
            v.z = pack2_bf16(bf16_lo(v.z) + bias[4], bf16_hi(v.z) + bias[5]);
            v.w = pack2_bf16(bf16_lo(v.w) + bias[6], bf16_hi(v.w) + bias[7]);
            *reinterpret_cast<uint4*>(p) = v;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (col + i < N) p[i] = (uint16_t)(pack2_bf16(bf16_one(p[i]) + bias[i], 0.0f) & 0xFFFFu);
        }
    }
}

int launch_add_bias(void* x, const void* b, int b_dtype, int64_t M, int64_t N, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    const unsigned gy = (unsigned)(M < 4096 ? M : 4096);
    dim3 grid((unsigned)((N + 2047) / 2048), gy);
    const bool vec = (N % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) &&
                     ((reinterpret_cast<uintptr_t>(b) & 15) == 0);
    uint16_t* xp = static_cast<uint16_t*>(x);
#define MDY_AB(VEC, BT) hipLaunchKernelGGL((add_bias_kernel<VEC, BT>), grid, dim3(256), 0, stream, xp, b, (int)M, (int)N)
    if (b_dtype == 0) { if (vec) MDY_AB(true, 0); else MDY_AB(false, 0); }
    else if (b_dtype == 1) { if (vec) MDY_AB(true, 1); else MDY_AB(false, 1); }
    else { if (vec) MDY_AB(true, 2); else MDY_AB(false, 2); }
#undef MDY_AB
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// In-place gradient accumulation x = T(fp32(x) + fp32(y)) over flat tensors of n elements, x fp32 or bf16, y fp32 or
// bf16.  Restates _add_grad_kernel (/root/reference/triton_kernels/megatron_patchs/add_kernel.py:41-62), which the
// Megatron patch uses to add a bf16 weight gradient into the fp32 main_grad buffer.  Streaming, 8 elements per lane.
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float grad_load(const T* p, int64_t i);
template <>
__device__ __forceinline__ float grad_load<float>(const float* p, int64_t i) { return p[i]; }
template <>
__device__ __forceinline__ float grad_load<uint16_t>(const uint16_t* p, int64_t i) { return bf16_one(p[i]); }
__device__ __forceinline__ void grad_store(float* p, int64_t i, float v) { p[i] = v; }
__device__ __forceinline__ void grad_store(uint16_t* p, int64_t i, float v) { p[i] = (uint16_t)(pack2_bf16(v, 0.0f) & 0xFFFFu); }

template <typename TX, typename TY>
__global__ __launch_bounds__(256) void add_grad_kernel(TX* __restrict__ x, const TY* __restrict__ y, int64_t n) {
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        if (i0 + j < n) grad_store(x, i0 + j, grad_load<TX>(x, i0 + j) + grad_load<TY>(y, i0 + j));
}

// dtype codes: 0 bf16, 1 fp32
int launch_add_grad(void* x, const void* y, int64_t n, int x_dtype, int y_dtype, hipStream_t stream) {
    if (n == 0) return 0;
    const int64_t blocks = (n + 2047) / 2048;
    if (blocks > 0x7FFFFFFF) return kErrTooManyBlocks;
    dim3 grid((unsigned)blocks), block(256);
    if (x_dtype == 1 && y_dtype == 0)
        hipLaunchKernelGGL((add_grad_kernel<float, uint16_t>), grid, block, 0, stream, static_cast<float*>(x), static_cast<const uint16_t*>(y), n);
    else if (x_dtype == 1)
        hipLaunchKernelGGL((add_grad_kernel<float, float>), grid, block, 0, stream, static_cast<float*>(x), static_cast<const float*>(y), n);
    else if (y_dtype == 0)
        hipLaunchKernelGGL((add_grad_kernel<uint16_t, uint16_t>), grid, block, 0, stream, static_cast<uint16_t*>(x), static_cast<const uint16_t*>(y), n);
    else
        hipLaunchKernelGGL((add_grad_kernel<uint16_t, float>), grid, block, 0, stream, static_cast<uint16_t*>(x), static_cast<const float*>(y), n);
    return (int)hipGetLastError();
}

}  // namespace mdy
