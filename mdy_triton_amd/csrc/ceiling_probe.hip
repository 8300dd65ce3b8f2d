// Ceiling probes: what the memory system and the matrix cores give the access patterns of this library's kernels when
// the arithmetic is taken out.  Built into libmdyfp8_probe.so, which only `bench.py --ceilings` loads; not part of
// libmdyfp8.so, no declaration in include/mdy_fp8.h, no counterpart in the reference.
//   copy_aq      the loads and stores of act_quant_kernel (16-byte non-temporal loads of bf16 rows, 8 rows x 512 columns per
//                workgroup on the same XCD-grouped grid, 8-byte non-temporal stores, one 4-byte scale store per 16 lanes);
//                the quantization is replaced by "keep the high byte of every bf16"
//   copy_wd      the loads and stores of weight_dequant_kernel (8 bytes in, 16 bytes out per lane, 2 rows per wave in
//                flight, one scale load per lane); the conversion is replaced by a byte spread
//   mfma_loop    a register-resident loop of v_mfma_f32_16x16x128_f8f6f4 only (8 + 4 operand fragments per wave, 32 MFMAs
//                per iteration, no memory access): accumulating in place, or starting from zero and folded into an fp32
//                accumulator with 4 v_fma_f32 per MFMA as the block-scaled GEMM has to
//   load_pattern the operand loads of a small-M GEMM (16 weight rows and 16 activation rows per workgroup) as MFMA fragments
//                straight from memory, as whole 128-byte lines, and as whole rows
//   empty        a kernel that does nothing (the launch floor inside a replayed graph)
#include <cstdint>

#include "common.h"

namespace mdy {

typedef int probe_intx8 __attribute__((ext_vector_type(8)));
typedef float probe_floatx4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void copy_aq_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ y, float* __restrict__ s,
                                                       int M, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = blockIdx.y * 512 + lane * 8;
    const int row0 = ((int)((blockIdx.z << 3) + blockIdx.x)) * 8 + wave * 2;
    uint4 raw[2];
#pragma unroll
    for (int r = 0; r < 2; ++r)
        raw[r] = (row0 + r < M && col < K) ? load_nt16(x + (int64_t)(row0 + r) * K + col) : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int row = row0 + r;
        // high bytes of the eight bf16 values
        const uint32_t lo = __builtin_amdgcn_perm(raw[r].y, raw[r].x, 0x07050301u);
        const uint32_t hi = __builtin_amdgcn_perm(raw[r].w, raw[r].z, 0x07050301u);
        if (row < M && col < K) {
            store_nt8(y + (int64_t)row * K + col, make_uint2(lo, hi));
            if ((lane & 15) == 0) s[(int64_t)row * (K >> 7) + (col >> 7)] = __uint_as_float(lo & 0x3F800000u);
        }
    }
}

__global__ __launch_bounds__(256) void copy_wd_kernel(const uint8_t* __restrict__ x, const float* __restrict__ s,
                                                       uint16_t* __restrict__ y, int N, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = blockIdx.x * 512 + lane * 8;
    const int row0 = (block_row() * 4 + wave) * 2;
    if (col >= K) return;
    uint2 raw[2];
    float sc[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int row = row0 + r;
        raw[r] = make_uint2(0u, 0u);
        sc[r] = 0.0f;
        if (row < N) {
            raw[r] = load_nt8(x + (int64_t)row * K + col);
            sc[r] = s[(int64_t)(row >> 7) * (K >> 7) + (col >> 7)];
        }
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int row = row0 + r;
        if (row >= N) continue;
        const uint32_t t = __float_as_uint(sc[r]) & 0x01010101u;
        // every byte becomes the high byte of a 16-bit value
        const uint4 o = make_uint4(__builtin_amdgcn_perm(raw[r].x, t, 0x05010400u), __builtin_amdgcn_perm(raw[r].x, t, 0x07030602u),
                                   __builtin_amdgcn_perm(raw[r].y, t, 0x05010400u), __builtin_amdgcn_perm(raw[r].y, t, 0x07030602u));
        store_nt16(y + (int64_t)row * K + col, o);
    }
}

// FOLD = false: 32 accumulating MFMAs per iteration.  FOLD = true: every MFMA starts from zero and its four results are
// folded into the accumulator by four v_fma_f32 four MFMAs later, as in the GEMM's K loop.
template <bool FOLD>
__global__ __launch_bounds__(512) void mfma_loop_kernel(const uint32_t* __restrict__ seed, float* __restrict__ out, int iters, float sc) {
    probe_intx8 fa[8], fb[4];
    const uint32_t s0 = seed[threadIdx.x & 63];           // 0 everywhere: constant operand bytes; else hashed per lane
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) fa[i][e] = s0 == 0 ? 0x38383838 : (int)((s0 + (uint32_t)(i * 8 + e) * 2654435761u) * 2246822519u);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) fb[i][e] = s0 == 0 ? 0x38383838 : (int)((s0 * 40503u + (uint32_t)(i * 8 + e) * 2246822519u) * 2654435761u);
    if (s0 != 0) {      // no NaN / Inf patterns: clear the top exponent bit of every byte
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e) fa[i][e] &= 0xBFBFBFBF;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e) fb[i][e] &= 0xBFBFBFBF;
    }
    probe_floatx4 acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = probe_floatx4{0.f, 0.f, 0.f, 0.f};
    const probe_floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
        probe_floatx4 p[5];
#pragma unroll
        for (int t = 0; t < 32 + 4; ++t) {
            if (t < 32) {
                const int i = t >> 2, j = t & 3;
                if (FOLD) p[t % 5] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa[i], zero, 0, 0, 0, 0, 0, 0);
                else acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa[i], acc[i][j], 0, 0, 0, 0, 0, 0);
            }
            if (FOLD && t >= 4) {
                const int u = t - 4, i = u >> 2, j = u & 3;
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][j][e] = __builtin_fmaf(p[u % 5][e], sc, acc[i][j][e]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("" : "+v"(fa[0]));      // keep the loop body from being hoisted
    }
    float r = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) r += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    out[blockIdx.x * 512 + threadIdx.x] = r;
}

// The same work per iteration (32 x 16x16x128 = 16 x 32x32x64) with v_mfma_f32_32x32x64_f8f6f4, which reads half the operand
// bytes from the register file per multiply-add: 2 x 2 output tiles of 32x32, each with operands for 128 of K (two MFMAs),
// two passes over them per iteration.  FOLD: the first MFMA of a pair starts from zero, the second accumulates onto it, and
// 16 v_fma_f32 fold the pair's results (4 per 32768 multiply-adds, as with the 16x16x128 form).
typedef float probe_floatx16 __attribute__((ext_vector_type(16)));
template <bool FOLD>
__global__ __launch_bounds__(512) void mfma32_loop_kernel(const uint32_t* __restrict__ seed, float* __restrict__ out, int iters, float sc) {
    probe_intx8 fa[2][2], fb[2][2];
    const uint32_t s0 = seed[threadIdx.x & 63];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            fa[i >> 1][i & 1][e] = s0 == 0 ? 0x38383838 : (int)(((s0 + (uint32_t)(i * 8 + e) * 2654435761u) * 2246822519u) & 0xBFBFBFBFu);
            fb[i >> 1][i & 1][e] = s0 == 0 ? 0x38383838 : (int)(((s0 * 40503u + (uint32_t)(i * 8 + e) * 2246822519u) * 2654435761u) & 0xBFBFBFBFu);
        }
    probe_floatx16 acc[2][2], zero;
#pragma unroll
    for (int e = 0; e < 16; ++e) zero[e] = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = zero;
    for (int it = 0; it < iters; ++it) {
        probe_floatx16 p[2];
#pragma unroll
        for (int t = 0; t < 8 + 1; ++t) {
            if (t < 8) {
                const int i = (t >> 1) & 1, j = t & 1;
                asm volatile("" : "+v"(fb[j][0]));      // the second pass is not the first one's common subexpression
                if (FOLD) {
                    p[t % 2] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j][0], fa[i][0], zero, 0, 0, 0, 0, 0, 0);
                    p[t % 2] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j][1], fa[i][1], p[t % 2], 0, 0, 0, 0, 0, 0);
                } else {
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j][0], fa[i][0], acc[i][j], 0, 0, 0, 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j][1], fa[i][1], acc[i][j], 0, 0, 0, 0, 0, 0);
                }
            }
            if (FOLD && t >= 1) {
                const int u = t - 1, i = (u >> 1) & 1, j = u & 1;
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = __builtin_fmaf(p[u % 2][e], sc, acc[i][j][e]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("" : "+v"(fa[0][0]));
    }
    float r = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) r += acc[i][j][e];
    out[blockIdx.x * 512 + threadIdx.x] = r;
}

// Load patterns of a small-M GEMM's operands with the arithmetic taken out: a workgroup of 8 waves owns 16 weight rows
// (b: [N, K] bytes) and re-reads 16 activation rows (a: [16, K] bytes); wave w takes the K blocks w, w + 8, .. and issues
// all of its loads (up to 8 K blocks) before it folds them into one word that is never stored.
//   PATTERN 0  MFMA fragments straight from memory: lane (r, q) = (lane % 16, lane / 16) loads the two 16-byte halves of
//              bytes [32 q, 32 q + 32) of row r's K block - per instruction 16 lines, 64 bytes of each
//   PATTERN 1  whole lines: lane l loads piece l % 8 of row l / 8 (and of row 8 + l / 8) of the K block - per instruction 8
//              lines, all 128 bytes of each
//   PATTERN 2  whole rows: wave w reads weight rows 2 w, 2 w + 1 and activation rows 2 w, 2 w + 1 end to end, 1 KB per
//              instruction (K <= 8192)
template <int PATTERN>
__global__ __launch_bounds__(512) void load_pattern_kernel(const uint8_t* __restrict__ b, const uint8_t* __restrict__ a,
                                                            uint32_t* __restrict__ out, int N, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * 16, KB = K >> 7;
    uint4 v[8][4];
    uint32_t x = 0;
    if (PATTERN == 2) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (i * 1024 + lane * 16 < K) {
                v[i][0] = *reinterpret_cast<const uint4*>(b + (size_t)(n0 + 2 * wave) * K + i * 1024 + lane * 16);
                v[i][1] = *reinterpret_cast<const uint4*>(b + (size_t)(n0 + 2 * wave + 1) * K + i * 1024 + lane * 16);
                v[i][2] = *reinterpret_cast<const uint4*>(a + (size_t)(2 * wave) * K + i * 1024 + lane * 16);
                v[i][3] = *reinterpret_cast<const uint4*>(a + (size_t)(2 * wave + 1) * K + i * 1024 + lane * 16);
            }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (i * 1024 + lane * 16 < K)
#pragma unroll
                for (int t = 0; t < 4; ++t) x ^= v[i][t].x ^ v[i][t].y ^ v[i][t].z ^ v[i][t].w;
    } else {
        const int row = PATTERN == 0 ? (lane & 15) : (lane >> 3);
        const int o0 = PATTERN == 0 ? (lane >> 4) * 32 : (lane & 7) * 16;
        const int second_row = PATTERN == 0 ? 0 : 8, second_off = PATTERN == 0 ? 16 : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int kb = wave + 8 * u;
            if (kb < KB) {
                v[u][0] = *reinterpret_cast<const uint4*>(b + (size_t)(n0 + row) * K + kb * 128 + o0);
                v[u][1] = *reinterpret_cast<const uint4*>(b + (size_t)(n0 + row + second_row) * K + kb * 128 + o0 + second_off);
                v[u][2] = *reinterpret_cast<const uint4*>(a + (size_t)row * K + kb * 128 + o0);
                v[u][3] = *reinterpret_cast<const uint4*>(a + (size_t)(row + second_row) * K + kb * 128 + o0 + second_off);
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (wave + 8 * u < KB)
#pragma unroll
                for (int t = 0; t < 4; ++t) x ^= v[u][t].x ^ v[u][t].y ^ v[u][t].z ^ v[u][t].w;
    }
    if (x == 0x12345678u) out[blockIdx.x] = x;      // keeps the loads; practically never taken
}

__global__ void empty_kernel() {}

}  // namespace mdy

// All entry points return 0 or a hipError_t; -2 for bad arguments.  Pointers are device memory.
extern "C" int mdy_probe_copy_aq(const void* x, void* y, float* s, int64_t M, int64_t K, void* stream) {
    if (!x || !y || !s || M < 1 || K < 512 || K % 512 != 0 || M % 64 != 0) return -2;
    dim3 grid(8, (unsigned)(K / 512), (unsigned)(M / 64)), block(256);
    hipLaunchKernelGGL(mdy::copy_aq_kernel, grid, block, 0, static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x),
                       static_cast<uint8_t*>(y), s, (int)M, (int)K);
    return (int)hipGetLastError();
}

extern "C" int mdy_probe_copy_wd(const void* x, const float* s, void* y, int64_t N, int64_t K, void* stream) {
    if (!x || !y || !s || N < 1 || K < 512 || K % 512 != 0 || N % 8 != 0) return -2;
    dim3 grid, block(256);
    if (!mdy::grid_rows(K / 512, N / 8, grid)) return -2;
    hipLaunchKernelGGL(mdy::copy_wd_kernel, grid, block, 0, static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(x), s,
                       static_cast<uint16_t*>(y), (int)N, (int)K);
    return (int)hipGetLastError();
}

// fold: bit 0 = fold every MFMA's result with v_fma_f32, bit 1 = 32x32x64 instead of 16x16x128 MFMAs
// seed: 64 uint32 (all zero: constant operand bytes 0x38 = 1.0; otherwise per-lane hash seeds); out: workgroups * 512 floats
extern "C" int mdy_probe_mfma_loop(int fold, const void* seed, float* out, int workgroups, int iters, void* stream) {
    if (!seed || !out || workgroups < 1 || iters < 1 || fold < 0 || fold > 3) return -2;
    if (fold & 2) {
        if (fold & 1)
            hipLaunchKernelGGL(mdy::mfma32_loop_kernel<true>, dim3((unsigned)workgroups), dim3(512), 0, static_cast<hipStream_t>(stream),
                               static_cast<const uint32_t*>(seed), out, iters, 1.0f);
        else
            hipLaunchKernelGGL(mdy::mfma32_loop_kernel<false>, dim3((unsigned)workgroups), dim3(512), 0, static_cast<hipStream_t>(stream),
                               static_cast<const uint32_t*>(seed), out, iters, 1.0f);
    } else if (fold)
        hipLaunchKernelGGL(mdy::mfma_loop_kernel<true>, dim3((unsigned)workgroups), dim3(512), 0, static_cast<hipStream_t>(stream),
                           static_cast<const uint32_t*>(seed), out, iters, 1.0f);
    else
        hipLaunchKernelGGL(mdy::mfma_loop_kernel<false>, dim3((unsigned)workgroups), dim3(512), 0, static_cast<hipStream_t>(stream),
                           static_cast<const uint32_t*>(seed), out, iters, 1.0f);
    return (int)hipGetLastError();
}

// b: N x K bytes, a: 16 x K bytes, out: N / 16 words; N % 16 == 0, K % 128 == 0, K <= 8192; pattern 0, 1 or 2
extern "C" int mdy_probe_load_pattern(int pattern, const void* b, const void* a, void* out, int64_t N, int64_t K, void* stream) {
    if (!b || !a || !out || N < 16 || N % 16 != 0 || K < 128 || K % 128 != 0 || K > 8192 || pattern < 0 || pattern > 2) return -2;
    dim3 grid((unsigned)(N / 16)), block(512);
    const uint8_t* bp = static_cast<const uint8_t*>(b);
    const uint8_t* ap = static_cast<const uint8_t*>(a);
    uint32_t* op = static_cast<uint32_t*>(out);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (pattern == 0) hipLaunchKernelGGL(mdy::load_pattern_kernel<0>, grid, block, 0, st, bp, ap, op, (int)N, (int)K);
    else if (pattern == 1) hipLaunchKernelGGL(mdy::load_pattern_kernel<1>, grid, block, 0, st, bp, ap, op, (int)N, (int)K);
    else hipLaunchKernelGGL(mdy::load_pattern_kernel<2>, grid, block, 0, st, bp, ap, op, (int)N, (int)K);
    return (int)hipGetLastError();
}

extern "C" int mdy_probe_empty(void* stream) {
    hipLaunchKernelGGL(mdy::empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream));
    return (int)hipGetLastError();
}
