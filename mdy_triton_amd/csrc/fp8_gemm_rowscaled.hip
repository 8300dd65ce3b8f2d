// Block-scaled FP8 GEMM, NT layout, with 1x128 scales on BOTH operands:
//   c[m,n] = sum_kb (sum_{k in kb} a[m,k] b[n,k]) * a_s[m,kb] * b_s[n,kb]
//
// Restates the have_w=False branch of _fp8_matmul_kernel
// (/root/reference/triton_kernels/deepseekv3/fp8_kernel.py:190-205; launcher fp8_matmul :214-252), which the
// reference's Fp8Linear uses for its weight gradient dw = dy^T . x with both operands quantized along the token
// dimension (fp8_matmul_bwd, :254-257).
//
// The combined scale differs for each of a lane's four results of an MFMA (four consecutive n of one m), so the
// fold is 4 multiplies + 4 FMAs per MFMA instead of 4 FMAs.  Two kernels: the scheduled tile body of fp8_gemm_tile.h in its
// row-scaled-weight form (128x256 tiles; the 256x256 tile has no registers left for the per-column scales) for problems
// that fill the CUs, and a plain loop (128x128 tile, four waves of 64x64, the K block's two panels and two scale vectors
// copied global -> LDS by `buffer_load ... lds`, double buffered, one barrier per K block) for the rest.  K % 128 == 0 (the callers contract over a padded token count).
#include "fp8_gemm_tile.h"

namespace mdy {

// FMT: byte format of both operands, 0 e4m3fn, 1 e5m2 (the MFMA's cbsz / blgp operand-format fields).
template <typename OUT, int FMT>
__global__ __launch_bounds__(256) void fp8_gemm_rowscaled_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, int bs_rs, int bs_cs, uint32_t bs_bytes,
    OUT* __restrict__ c, int M, int N, int K, int tiles_n) {
    constexpr int BM = 128, BN = 128;
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a[2][BM * 128];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_b[2][BN * 128];
    __shared__ __attribute__((aligned(256))) float lds_sa[2][BM];
    __shared__ __attribute__((aligned(256))) float lds_sb[2][BN];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    const int KB = K >> 7;

    // ---- copies: 4 waves x 8 rows per instruction, 4 instructions per panel; rows past M / N read zero
    const intx4 ra = make_rsrc(a + (size_t)m0 * K, (uint32_t)min(BM, M - m0) * (uint32_t)K);
    const intx4 rb = make_rsrc(b + (size_t)n0 * K, (uint32_t)min(BN, N - n0) * (uint32_t)K);
    const intx4 rsa = make_rsrc(a_s, as_bytes), rsb = make_rsrc(b_s, bs_bytes);
    const int prow = wave * 8 + (lane >> 3);
    const int voff = prow * K + (((lane & 7) ^ swz(prow)) << 4);
    // scale vectors: waves 0, 1 copy the 128 activation scales of the K block, waves 2, 3 the 128 weight-row scales
    const bool sc_a = wave < 2;
    const int sc_row = (wave & 1) * 64 + lane;
    const intx4 rsc = sc_a ? rsa : rsb;
    const int sc_voff = sc_a ? min(m0 + sc_row, M - 1) * as_rs * 4 : min(n0 + sc_row, N - 1) * bs_rs * 4;
    const int sc_kstep = (sc_a ? as_cs : bs_cs) * 4;
    const uint32_t la = lds_addr(&lds_a[0][0]) + wave * 1024, lb = lds_addr(&lds_b[0][0]) + wave * 1024;
    const uint32_t lsc = (sc_a ? lds_addr(&lds_sa[0][0]) : lds_addr(&lds_sb[0][0])) + (wave & 1) * 256;
    auto copy_block = [&](int kb, int buf) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            dma16(ra, voff, p * 32 * K + kb * 128, la + buf * (BM * 128) + p * 32 * 128);
            dma16(rb, voff, p * 32 * K + kb * 128, lb + buf * (BN * 128) + p * 32 * 128);
        }
        dma4(rsc, sc_voff, kb * sc_kstep, lsc + buf * 512);
    };

    // ---- fragments: lane -> row lane%16 and the 32-byte K slice lane/16 of a 16-row sub-tile
    const int frow = lane & 15, fk = lane >> 4;
    const int a_rd0 = (wm * 64 + frow) * 128 + (((2 * fk) ^ swz(frow)) << 4);
    const int a_rd1 = (wm * 64 + frow) * 128 + (((2 * fk + 1) ^ swz(frow)) << 4);
    const int b_rd0 = (wn * 64 + frow) * 128 + (((2 * fk) ^ swz(frow)) << 4);
    const int b_rd1 = (wn * 64 + frow) * 128 + (((2 * fk + 1) ^ swz(frow)) << 4);
    auto frag = [&](const uint8_t* base, int rd0, int rd1, int idx) {
        const intx4 lo = *reinterpret_cast<const intx4*>(base + rd0 + idx * 2048);
        const intx4 hi = *reinterpret_cast<const intx4*>(base + rd1 + idx * 2048);
        return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    copy_block(0, 0);
    for (int kb = 0; kb < KB; ++kb) {
        const int buf = kb & 1;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();     // K block kb is in LDS, and every wave has finished reading the other buffer
        if (kb + 1 < KB) copy_block(kb + 1, buf ^ 1);
        intx8 fb[4];
        floatx4 sbv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            fb[j] = frag(lds_b[buf], b_rd0, b_rd1, j);
            sbv[j] = *reinterpret_cast<const floatx4*>(&lds_sb[buf][wn * 64 + j * 16 + 4 * fk]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const intx8 fa = frag(lds_a[buf], a_rd0, a_rd1, i);
            const float sa = lds_sa[buf][wm * 64 + i * 16 + frow];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                const floatx4 p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa, zero, FMT, FMT, 0, 0, 0, 0);
                acc[i][j][0] = __builtin_fmaf(p[0], sa * sbv[j][0], acc[i][j][0]);
                acc[i][j][1] = __builtin_fmaf(p[1], sa * sbv[j][1], acc[i][j][1]);
                acc[i][j][2] = __builtin_fmaf(p[2], sa * sbv[j][2], acc[i][j][2]);
                acc[i][j][3] = __builtin_fmaf(p[3], sa * sbv[j][3], acc[i][j][3]);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    const bool vec_ok = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + wm * 64 + i * 16 + frow;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + wn * 64 + j * 16 + 4 * fk;
            const float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
            store4<OUT>(c, N, m, n, M, N, v, vec_ok);
        }
    }
}

// The scheduled tile body of fp8_gemm_tile.h in its row-scaled-weight form, 128x256 tiles (8 waves of 64x64, ring of three
// K blocks): for problems that give every CU a tile.  Smaller problems run the plain kernel above, two workgroups per CU.
template <typename OUT, int FMT>
__global__ __launch_bounds__(512) void fp8_gemm_rowscaled_tile_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, int bs_rs, int bs_cs, uint32_t bs_bytes,
    OUT* __restrict__ c, int M, int N, int K, int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(1024))) uint8_t pool[TileLds<128, 256, 8, 3>::bytes];
    const int ntiles = tiles_m * tiles_n;
    int tm, tn;
    const Duty duty = tile_of(xcd_contiguous(blockIdx.x, ntiles), tiles_m, tiles_n, tm, tn);
    fp8_gemm_tile<128, 256, 2, 4, 3, OUT, 0, 0, 0, FMT, true>(a, a_s, as_rs, as_cs, as_bytes, b, b_s, c, nullptr, tm * 128, M, M,
                                                              tn * 256, N, K, N, duty, 0, K >> 7, pool, bs_rs, bs_cs, bs_bytes);
}

// returns hipError_t, or -1 when the operands do not qualify (K % 128 != 0, misaligned, scale extents >= 2^31 bytes)
int launch_fp8_gemm_nt_rowscaled(const void* a, const float* a_s, int64_t as_rs, int64_t as_cs, const void* b,
                                 const float* b_s, int64_t bs_rs, int64_t bs_cs, void* c, int64_t M, int64_t N, int64_t K,
                                 int fmt, int out_dtype, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    const int64_t KB = K / 128;
    const int64_t a_ext = ((M - 1) * as_rs + (KB - 1) * as_cs + 1) * 4, b_ext = ((N - 1) * bs_rs + (KB - 1) * bs_cs + 1) * 4;
    if (K % 128 != 0 || K > (1 << 20) || as_rs < 0 || as_cs < 0 || bs_rs < 0 || bs_cs < 0 || a_ext >= ((int64_t)1 << 31) ||
        b_ext >= ((int64_t)1 << 31) || ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) != 0 ||
        128 * K >= ((int64_t)1 << 31))
        return -1;
    // 128x256 tiles of the scheduled body once they fill the CUs (and K fits its weight-scale staging)
    const int64_t big_m = (M + 127) / 128, big_n = (N + 255) / 256;
    if (big_m * big_n >= 200 && K <= (1 << 16) && big_m * big_n <= 0x7FFFFFFF) {
#define MDY_RST(OUT_T, FMT)                                                                                              \
    hipLaunchKernelGGL((fp8_gemm_rowscaled_tile_kernel<OUT_T, FMT>), dim3((unsigned)(big_m * big_n)), dim3(512), 0, stream, \
                       static_cast<const uint8_t*>(a), a_s, (int)as_rs, (int)as_cs, (uint32_t)a_ext,                      \
                       static_cast<const uint8_t*>(b), b_s, (int)bs_rs, (int)bs_cs, (uint32_t)b_ext, static_cast<OUT_T*>(c), \
                       (int)M, (int)N, (int)K, (int)big_m, (int)big_n)
        if (out_dtype == 0) { if (fmt == 0) MDY_RST(uint16_t, 0); else MDY_RST(uint16_t, 1); }
        else { if (fmt == 0) MDY_RST(float, 0); else MDY_RST(float, 1); }
#undef MDY_RST
        return (int)hipGetLastError();
    }
    const int tiles_m = (int)((M + 127) / 128), tiles_n = (int)((N + 127) / 128);
    if ((int64_t)tiles_m * tiles_n > 0x7FFFFFFF) return kErrTooManyBlocks;
    dim3 grid((unsigned)(tiles_m * tiles_n)), block(256);
#define MDY_RS(OUT_T, FMT)                                                                                                 \
    hipLaunchKernelGGL((fp8_gemm_rowscaled_kernel<OUT_T, FMT>), grid, block, 0, stream, static_cast<const uint8_t*>(a), a_s, \
                       (int)as_rs, (int)as_cs, (uint32_t)a_ext, static_cast<const uint8_t*>(b), b_s, (int)bs_rs, (int)bs_cs, \
                       (uint32_t)b_ext, static_cast<OUT_T*>(c), (int)M, (int)N, (int)K, tiles_n)
    if (out_dtype == 0) { if (fmt == 0) MDY_RS(uint16_t, 0); else MDY_RS(uint16_t, 1); }
    else { if (fmt == 0) MDY_RS(float, 0); else MDY_RS(float, 1); }
#undef MDY_RS
    return (int)hipGetLastError();
}

}  // namespace mdy
