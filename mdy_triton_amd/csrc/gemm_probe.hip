// Timing probe of the MFMA tile kernel: one tile configuration with parts of its K loop switched off.
// It exists so that the cost of each part (global->LDS copies, LDS fragment reads, the FMA fold of the block
// scales, the pre-touches) can be measured on the product's own code, with the product's own operands, and the
// power / clock readings taken while it runs; the results of a probe with anything switched off are NOT a GEMM.
// No counterpart in the reference.  Built into libmdyfp8_probe.so, which only `bench.py --ablation` loads: it is not
// part of libmdyfp8.so and has no declaration in include/mdy_fp8.h.
#include "fp8_gemm_tile.h"

namespace mdy {

template <int BM, int BN, int WGM, int WGN, int STAGES, int GAP, int ABL>
static int probe_launch(const uint8_t* a, const float* a_s, int as_rs, int as_cs, uint32_t as_bytes, const uint8_t* b,
                        const float* b_s, uint16_t* c, int M, int N, int K, int max_wgs, hipStream_t stream) {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int wgs = (BM * BN >= 256 * 256 && tiles_m * tiles_n > max_wgs) ? max_wgs : tiles_m * tiles_n;
    hipLaunchKernelGGL((fp8_gemm_mfma_kernel<BM, BN, WGM, WGN, STAGES, uint16_t, GAP, 0, ABL>), dim3((unsigned)wgs),
                       dim3(WGM * WGN * 64), 0, stream, a, a_s, as_rs, as_cs, as_bytes, b, b_s, c,
                       static_cast<const uint16_t*>(nullptr), M, N, K, N, tiles_m, tiles_n, 1);
    return (int)hipGetLastError();
}

// tile: 0 = 256x256 (ring of 2 K blocks), 1 = 128x256 (ring of 3).  ablation: bit set of
// 1 no copies in the loop, 2 no LDS reads, 4 no FMA fold, 8 no pre-touches; the combinations built are
// 0, 8, 1, 2, 4, 3, 5, 7 (0 and 8 give the exact GEMM result).  Returns -1 for a combination that is not built.
static int launch_fp8_gemm_probe(int tile, int ablation, const void* a, const float* a_s, int64_t as_rs, int64_t as_cs,
                          const void* b, const float* b_s, void* c, int64_t M, int64_t N, int64_t K, hipStream_t stream) {
    const int KB = (int)(K / 128);
    const int64_t as_extent = ((M - 1) * as_rs + (int64_t)(KB - 1) * as_cs + 1) * 4;
    int cus = 256;
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
    }
#define MDY_PROBE(BM, BN, ST, GAP, ABL)                                                                            \
    return probe_launch<BM, BN, 2, 4, ST, GAP, ABL>(static_cast<const uint8_t*>(a), a_s, (int)as_rs, (int)as_cs,   \
                                                    (uint32_t)as_extent, static_cast<const uint8_t*>(b), b_s,      \
                                                    static_cast<uint16_t*>(c), (int)M, (int)N, (int)K, cus, stream)
#define MDY_PROBE_TILE(BM, BN, ST, GAP)                  \
    switch (ablation) {                                  \
        case 0: MDY_PROBE(BM, BN, ST, GAP, 0);           \
        case 8: MDY_PROBE(BM, BN, ST, GAP, 8);           \
        case 1: MDY_PROBE(BM, BN, ST, GAP, 1);           \
        case 2: MDY_PROBE(BM, BN, ST, GAP, 2);           \
        case 4: MDY_PROBE(BM, BN, ST, GAP, 4);           \
        case 3: MDY_PROBE(BM, BN, ST, GAP, 3);           \
        case 5: MDY_PROBE(BM, BN, ST, GAP, 5);           \
        case 7: MDY_PROBE(BM, BN, ST, GAP, 7);           \
        default: return -1;                              \
    }
    if (tile == 0) { MDY_PROBE_TILE(256, 256, 2, 0) }
    if (tile == 1) { MDY_PROBE_TILE(128, 256, 3, 0) }
#undef MDY_PROBE_TILE
#undef MDY_PROBE
    return -1;
}

// The product's 256x256 kernel with another shape of the block of tiles that an XCD runs at a time (GM tile rows x
// 32 / GM tile columns; the product uses 4 x 8) and the pre-touches on or off: the exact GEMM result every time.
static int launch_fp8_gemm_order_probe(int gm, int pretouch, const void* a, const float* a_s, int64_t as_rs, int64_t as_cs,
                                       const void* b, const float* b_s, void* c, int64_t M, int64_t N, int64_t K, hipStream_t stream) {
    const int KB = (int)(K / 128);
    const int64_t as_extent = ((M - 1) * as_rs + (int64_t)(KB - 1) * as_cs + 1) * 4;
    int cus = 256, dev = 0;
    if (hipGetDevice(&dev) == hipSuccess) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
    }
    const int tiles_m = (int)((M + 255) / 256), tiles_n = (int)((N + 255) / 256);
    const int wgs = tiles_m * tiles_n > cus ? cus : tiles_m * tiles_n;
#define MDY_ORDER(GM)                                                                                                   \
    hipLaunchKernelGGL((fp8_gemm_mfma_kernel<256, 256, 2, 4, 2, uint16_t, 0, 0, 0, 0, GM>), dim3((unsigned)wgs), dim3(512), 0, stream, \
                       static_cast<const uint8_t*>(a), a_s, (int)as_rs, (int)as_cs, (uint32_t)as_extent,                  \
                       static_cast<const uint8_t*>(b), b_s, static_cast<uint16_t*>(c), static_cast<const uint16_t*>(nullptr), \
                       (int)M, (int)N, (int)K, (int)N, tiles_m, tiles_n, pretouch)
    if (gm == 2) MDY_ORDER(2);
    else if (gm == 4) MDY_ORDER(4);
    else if (gm == 8) MDY_ORDER(8);
    else return -1;
#undef MDY_ORDER
    return (int)hipGetLastError();
}

}  // namespace mdy

// Entry point of the probe library.  K % 128 == 0, K <= 65536, N % 4 == 0, a / b / c 16-byte aligned, activation scales
// within 2^31 bytes; returns 0, a hipError_t, -1 for a tile / ablation pair that is not built, -2 for bad arguments.
extern "C" int mdy_fp8_gemm_order_probe(int gm, int pretouch, const void* a, const float* a_s, int64_t as_row_stride,
                                        int64_t as_col_stride, const void* b, const float* b_s, void* c, int64_t M, int64_t N,
                                        int64_t K, void* stream) {
    if (M < 1 || N < 1 || K < 128 || K % 128 != 0 || K > 65536 || N % 4 != 0 || !a || !a_s || !b || !b_s || !c) return -2;
    if (((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15) != 0) return -2;
    if (as_row_stride < 0 || as_col_stride < 0 ||
        ((M - 1) * as_row_stride + (K / 128 - 1) * as_col_stride + 1) * 4 >= ((int64_t)1 << 31))
        return -2;
    return mdy::launch_fp8_gemm_order_probe(gm, pretouch, a, a_s, as_row_stride, as_col_stride, b, b_s, c, M, N, K,
                                            static_cast<hipStream_t>(stream));
}

extern "C" int mdy_fp8_gemm_probe(int tile, int ablation, const void* a, const float* a_s, int64_t as_row_stride,
                                  int64_t as_col_stride, const void* b, const float* b_s, void* c, int64_t M, int64_t N,
                                  int64_t K, void* stream) {
    if (M < 1 || N < 1 || K < 128 || K % 128 != 0 || K > 65536 || N % 4 != 0 || !a || !a_s || !b || !b_s || !c) return -2;
    if (((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15) != 0) return -2;
    if (as_row_stride < 0 || as_col_stride < 0 ||
        ((M - 1) * as_row_stride + (K / 128 - 1) * as_col_stride + 1) * 4 >= ((int64_t)1 << 31))
        return -2;
    return mdy::launch_fp8_gemm_probe(tile, ablation, a, a_s, as_row_stride, as_col_stride, b, b_s, c, M, N, K,
                                      static_cast<hipStream_t>(stream));
}
