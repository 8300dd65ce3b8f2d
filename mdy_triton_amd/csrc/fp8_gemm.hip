// Block-scaled FP8 GEMM, NT layout, for gfx950 MFMA:
//   c[m,n] = sum_kb (sum_{k in kb} a[m,k] b[n,k]) * a_s[m,kb] * b_s[n/128,kb] (+ bias[n])
//
// Restates fp8_gemm_kernel
// (/root/reference/triton_kernels/deepseekv3/offical_kernel.py:61-97) and the contract
// of the DeepGEMM call in /root/reference/triton_kernels/dpsk_fp8linear/fp8.py:307-311.
//
// Main kernel (K % 128 == 0):
//   * one workgroup owns a BM x BN tile of C; per 128-wide K block the A and B
//     panels (BM x 128 and BN x 128 bytes) and the BM activation scales are
//     copied global -> LDS by `buffer_load ... lds` (no registers involved) into
//     a ring of 2..8 K blocks, one barrier per K block.  The buffer descriptors
//     cover exactly the rows of the tile, so rows past M or N read as zero;
//   * LDS rows are 128 bytes; the eight 16-byte chunks of a row are XOR-swizzled
//     with (row & 7) ^ (row>>3 & 1): each DMA lane fetches the permuted chunk,
//     the ds_read_b128 fragment reads are bank-conflict free;
//   * v_mfma_f32_16x16x128_f8f6f4 consumes a whole 128-deep scale block per
//     instruction.  The B rows go in as the MFMA "A" operand and the A rows as
//     its "B" operand, so a lane ends up with 4 consecutive n of one m: the
//     per-block scale a_s[m,kb]*b_s[n/128,kb] is ONE value per lane and
//     sub-tile, and the epilogue stores 8 contiguous bytes per lane;
//   * each MFMA starts from C = 0 and writes plain VGPRs; its 4 results are folded
//     into the fp32 master accumulator with v_fma_f32 a few MFMAs later (the
//     promotion the reference does at offical_kernel.py:86), so the VALU work
//     runs in the shadow of the matrix pipe;
//   * the smaller fragment set of the wave tile is held in registers for the
//     whole K block, the other one is streamed through a two-deep register queue;
//   * workgroup ids are remapped so that the 32 workgroups that share an XCD's L2
//     cover a compact 4 x 8 block of tiles.
// Tile sizes from 64x64 to 256x256 share that body; the host picks by tile count, and with a
// workspace also splits K (fp8_gemm_splitk_kernel + splitk_reduce_kernel).  The 128x192 tile (mid-size
// shapes whose 128x256 tiles would leave a quarter of the CUs idle) runs a second body with producer and
// consumer waves (fp8_gemm_tile_ws in fp8_gemm_tile.h).
// Small-M kernel (M <= 64): weight streaming in whole 128-byte lines, one workgroup of 8 waves per 8, 16 or 32
// columns, the waves split K and reduce through LDS (with a workspace also over slabs of K for 33..64 rows against
// a narrow weight).  Strip kernel: 17..64 rows against many 128-column strips.  Scalar kernel: any other
// shape/alignment.
#include <cstdlib>
#include <mutex>

#include "fp8_gemm_tile.h"

namespace mdy {

// ---------------------------------------------------------------------------
// Split-K: shapes whose tiles do not fill the CUs (few rows against a long K) are cut along K as well.
// Workgroup (ks, tile) accumulates K blocks ks*kb_per .. of its tile and stores the fp32 partial sums
// into slab ks of a caller-provided workspace [ksplit][M][N]; splitk_reduce_kernel then adds the slabs in
// slab order (so the result does not depend on scheduling), adds the bias and converts.
// ---------------------------------------------------------------------------
template <int BM, int BN, int WGM, int WGN, int STAGES>
__global__ __launch_bounds__(WGM* WGN * 64) void fp8_gemm_splitk_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, float* __restrict__ ws, int M, int N, int K,
    int tiles_m, int tiles_n, int ksplit, int kb_per) {
    __shared__ __attribute__((aligned(1024))) uint8_t pool[TileLds<BM, BN, WGM * WGN, STAGES>::bytes];
    const int ntiles = tiles_m * tiles_n;
    // slab-major order: the workgroups that share an XCD work on the same K range, so they share its A rows
    const int pid = xcd_contiguous(blockIdx.x, ntiles * ksplit);
    const int ks = __builtin_amdgcn_readfirstlane(pid / ntiles);
    int tm, tn;
    const Duty duty = tile_of(pid - ks * ntiles, tiles_m, tiles_n, tm, tn);
    const int kb0 = ks * kb_per, kb1 = min(K >> 7, kb0 + kb_per);
    fp8_gemm_tile<BM, BN, WGM, WGN, STAGES, float>(a, a_s, as_rs, as_cs, as_bytes, b, b_s, ws + (size_t)ks * M * N, nullptr,
                                                   tm * BM, M, M, tn * BN, N, K, N, duty, kb0, kb1, pool);
}

// The same on the producer / consumer tile (128x128 and 128x64 tiles, 4 consumer + 4 producer waves): against the one-body
// tile, after a cache flush / back to back, results identical: 512x4096x7168 42.6 -> 36.5 / 32.1 -> 29.4 us, 256x7168x18432
// 89.9 -> 74.1 / 57.9 -> 53.2 us, 128x2112x7168 20.4 -> 19.2 / 15.6 -> 14.4 us, 96x4096x7168 25.3 -> 24.4 / 17.3 -> 15.4 us.
template <int BM, int BN, int STAGES>
__global__ __launch_bounds__(512) void fp8_gemm_splitk_ws_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, float* __restrict__ ws, int M, int N, int K,
    int tiles_m, int tiles_n, int ksplit, int kb_per) {
    constexpr bool HOLD_A = BM / 2 <= BN / 2;
    __shared__ __attribute__((aligned(1024)))
    uint8_t pool[TileLdsWs<BM, BN, 8, HOLD_A ? STAGES - 1 : STAGES, HOLD_A ? STAGES : STAGES - 1, STAGES - 1>::bytes];
    const int ntiles = tiles_m * tiles_n;
    const int pid = xcd_contiguous(blockIdx.x, ntiles * ksplit);
    const int ks = __builtin_amdgcn_readfirstlane(pid / ntiles);
    int tm, tn;
    const Duty duty = tile_of(pid - ks * ntiles, tiles_m, tiles_n, tm, tn);
    const int kb0 = ks * kb_per, kb1 = min(K >> 7, kb0 + kb_per);
    fp8_gemm_tile_ws<BM, BN, 2, 2, 4, STAGES, float>(a, a_s, as_rs, as_cs, as_bytes, b, b_s, ws + (size_t)ks * M * N, nullptr, tm * BM, M, M,
                                                     tn * BN, N, K, N, duty, kb0, kb1, pool);
}

template <typename OUT, bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, OUT* __restrict__ c,
                                                            const uint16_t* __restrict__ bias, int64_t MN, int N,
                                                            int ksplit) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * (VEC ? 4 : 1);
    if (i >= MN) return;
    if (VEC) {   // N % 4 == 0: the 4 elements lie in one row
        float4 s = *reinterpret_cast<const float4*>(ws + i);
        for (int k0 = 1; k0 < ksplit; k0 += 4) {      // four slabs' loads in flight; added in slab order
            float4 v[4];
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) v[kk] = *reinterpret_cast<const float4*>(ws + (int64_t)min(k0 + kk, ksplit - 1) * MN + i);
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
                if (k0 + kk < ksplit) { s.x += v[kk].x; s.y += v[kk].y; s.z += v[kk].z; s.w += v[kk].w; }
        }
        if (bias != nullptr) {
            const int n = (int)(i % N);
            s.x += bf16_one(bias[n]); s.y += bf16_one(bias[n + 1]); s.z += bf16_one(bias[n + 2]); s.w += bf16_one(bias[n + 3]);
        }
        if (sizeof(OUT) == 2)
            *reinterpret_cast<uint2*>(c + i) = make_uint2(pack2_bf16(s.x, s.y), pack2_bf16(s.z, s.w));
        else
            *reinterpret_cast<float4*>(c + i) = s;
    } else {
        float s = ws[i];
        for (int k = 1; k < ksplit; ++k) s += ws[(int64_t)k * MN + i];
        if (bias != nullptr) s += bf16_one(bias[i % N]);
        if (sizeof(OUT) == 2)
            reinterpret_cast<uint16_t*>(c)[i] = (uint16_t)(pack2_bf16(s, 0.0f) & 0xFFFFu);
        else
            reinterpret_cast<float*>(c)[i] = s;
    }
}

// ---------------------------------------------------------------------------
// Grouped (mixture-of-experts) GEMM: rows row_start[g] .. row_start[g+1] of a are multiplied with
// expert g's weight b[g] ([N, K], scales b_s[g]); c has the rows of a.  The table travels as a kernel
// argument; a workgroup finds its group by binary search over the tile prefix sums.  Tiles never
// straddle two groups: each group is tiled from its own first row, short last tiles read zeros and
// store only their own rows.
// ---------------------------------------------------------------------------
constexpr int kMaxGroups = 256;
struct GroupTable {
    int n_groups;
    int row_start[kMaxGroups + 1];   // first row of group g; [n_groups] = total rows
    int tile_start[kMaxGroups + 1];  // tile rows (of BM) before group g
};

// Tile rows are 256 rows high; a group's last tile row, when it holds at most 128 rows, runs as a 128x256 tile
// (ring of 3 K blocks in the LDS the 256x256 tile's ring of 2 would take).
template <typename OUT>
__global__ __launch_bounds__(512) void fp8_grouped_gemm_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, OUT* __restrict__ c,
    const uint16_t* __restrict__ bias, int N, int K, int tiles_n, const GroupTable tbl) {
    constexpr int kBig = TileLds<256, 256, 8, 2>::bytes, kSmall = TileLds<128, 256, 8, 3>::bytes;
    __shared__ __attribute__((aligned(1024))) uint8_t pool[kBig > kSmall ? kBig : kSmall];
    const int G = tbl.n_groups;
    const int pid = xcd_contiguous(blockIdx.x, tbl.tile_start[G] * tiles_n);
    const int trow = pid / tiles_n;               // position in units of whole tile rows
    int lo = 0, hi = G - 1;                       // last g with tile_start[g] <= trow (empty groups skipped)
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (tbl.tile_start[mid] <= trow) lo = mid; else hi = mid - 1;
    }
    // everything derived from the table is wave-uniform; say so (the copies need scalar descriptors)
    const int g = __builtin_amdgcn_readfirstlane(lo);
    const int tiles_m = __builtin_amdgcn_readfirstlane(tbl.tile_start[g + 1] - tbl.tile_start[g]);
    int tm, tn;
    Duty duty = tile_of(pid - tbl.tile_start[g] * tiles_n, tiles_m, tiles_n, tm, tn);
    duty.a_duty = __builtin_amdgcn_readfirstlane(duty.a_duty);
    duty.b_duty = __builtin_amdgcn_readfirstlane(duty.b_duty);
    duty.a_sh = __builtin_amdgcn_readfirstlane(duty.a_sh);
    duty.b_sh = __builtin_amdgcn_readfirstlane(duty.b_sh);
    const int KB = K >> 7, NB = (N + 127) >> 7;
    const int r0 = __builtin_amdgcn_readfirstlane(tbl.row_start[g]), r1 = __builtin_amdgcn_readfirstlane(tbl.row_start[g + 1]);
    const int m0 = __builtin_amdgcn_readfirstlane(r0 + tm * 256);
    const int m_total = __builtin_amdgcn_readfirstlane(tbl.row_start[G]);
    const int n0 = __builtin_amdgcn_readfirstlane(tn * 256);
    const uint8_t* bg = b + (size_t)g * N * K;
    const float* bsg = b_s + (size_t)g * NB * KB;
    const uint16_t* biasg = bias ? bias + (size_t)g * N : nullptr;
    if (r1 - m0 <= 128)
        fp8_gemm_tile<128, 256, 2, 4, 3, OUT>(a, a_s, as_rs, as_cs, as_bytes, bg, bsg, c, biasg, m0, r1, m_total, n0, N, K, N, duty, 0, KB, pool);
    else
        fp8_gemm_tile<256, 256, 2, 4, 2, OUT>(a, a_s, as_rs, as_cs, as_bytes, bg, bsg, c, biasg, m0, r1, m_total, n0, N, K, N, duty, 0, KB, pool);
}

constexpr int kSmWaves = 8;      // waves per workgroup of the small-M kernels

// ---------------------------------------------------------------------------
// Small-M kernel with whole-line loads (up to 16*MT rows; decode and routed-expert shapes): pure weight streaming, one
// workgroup of 8 waves per 16*NC output columns, the waves share out the K blocks and their partial sums are reduced
// through LDS.  An MFMA operand wants lane (r, q) to hold 32 bytes of row r, so fragment loads straight from global
// memory touch, per instruction, 16 rows x 4 pieces of 16 bytes: 64 of every 128-byte line, the line's other half by the
// next instruction.  Measured on loads alone (M=16, N=2048, K=7168, replayed graph): 8.5 us per call that way, 3.4 us
// when every load instruction covers whole lines (8 rows x the 128 bytes of one K block: lane l has piece l & 7 of
// row l >> 3).  So here a wave loads its K blocks that way, UF blocks before the first use, and turns a block into
// fragments through LDS that only this wave touches - two 16-byte writes and two 16-byte reads per 16 rows, pieces
// XOR-swizzled by the row so that both fall on all banks - which needs no barrier: every wave runs on as its own
// loads arrive (and, with two LDS tiles per wave, block u+1 on its way through LDS while the MFMAs of block u run).  Wave w owns the K blocks
// [w per, (w+1) per), per = ceil(KB / 8): no branch depends on the block, so the waits the compiler places count
// exactly; a block beyond the wave's range is a re-read of the last valid one whose product is replaced by zero.
// ---------------------------------------------------------------------------
template <int MT, int NC, int UF, typename OUT, int FMT, bool HALF = false, int WK = kSmWaves>
__device__ __forceinline__ void smallm_lines_body(const uint8_t* __restrict__ a, const float* __restrict__ a_s, int64_t as_rs, int64_t as_cs,
                                                  const uint8_t* __restrict__ b, const float* __restrict__ b_s, OUT* __restrict__ c,
                                                  const uint16_t* __restrict__ bias, int M, int N, int K, int kb_lo = 0,
                                                  int kb_hi = -1) {
    constexpr int SUB = NC * MT, TILES = NC + MT;      // (column group, row sub-tile) pairs; 16-row operand tiles per K block
    // WK waves share out the K blocks of one set of columns; with a short K (fewer blocks than waves) the 8 waves form
    // 8 / WK such sets side by side instead of idling
    constexpr int SETS = kSmWaves / WK;
    static_assert(SUB <= WK && SETS * WK == kSmWaves, "one wave of a set reduces one (column group, row sub-tile) pair");
    constexpr int SV = (UF + 3) / 4;                    // activation-scale loads per row sub-tile and pass
    // LDS regions and fragment sets per wave: two (block u + 1 on its way through LDS while the MFMAs of block u run) where
    // one workgroup per CU is all there is (16 rows x 16 columns against a long K: M=16 N=2048 K=7168 5.4 us against 7.2 with
    // one); one elsewhere, so that two or three workgroups fit a CU's LDS (M=16 N=24576 K=1536 10.0 -> 8.3 us, N=129280
    // K=7168 165 -> 154 us; 17..32 rows: 10.0 -> 9.6 us at N=2048 K=7168)
    constexpr int NBUF = (MT == 1 && NC == 1) ? 2 : 1;
    __shared__ __attribute__((aligned(16))) uint8_t lds[kSmWaves][NBUF][TILES * 2048];
    __shared__ float red[kSmWaves][SUB][64][4];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int frow = lane & 15, fk = lane >> 4;
    const int r8 = lane >> 3, pc = lane & 7;
    // HALF: 8 weight columns per workgroup (the other half of the MFMA's 16 rows stays unused): twice the workgroups for a
    // narrow weight
    static_assert(!HALF || NC == 1, "half a column group per workgroup: one group");
    constexpr int BT = HALF ? 1 : 2 * NC;              // 8-row weight loads per K block
    const int set = wave / WK, wk = wave % WK;
    const int n0 = (blockIdx.x * SETS + set) * (HALF ? 8 : 16 * NC);
    const int KB = K >> 7, NB = (N + 127) >> 7;
    const int k_hi = kb_hi < 0 ? KB : kb_hi;                                     // the workgroup's K blocks: [kb_lo, k_hi)
    const int per = (k_hi - kb_lo + WK - 1) / WK;
    const int k_begin = min(kb_lo + wk * per, k_hi), k_end = min(k_begin + per, k_hi);      // this wave's K blocks
    // global: lane l loads piece l & 7 of row 8 t + (l >> 3) for t = 0, 1 of every 16-row tile
    const uint8_t* bld[BT];
    const uint8_t* ald[2 * MT];
#pragma unroll
    for (int t = 0; t < BT; ++t) bld[t] = b + (int64_t)min(n0 + 8 * t + r8, N - 1) * K + pc * 16;
#pragma unroll
    for (int t = 0; t < 2 * MT; ++t) ald[t] = a + (int64_t)min(8 * t + r8, M - 1) * K + pc * 16;
    const float* bsp[NC];
    const float* asp[MT];
#pragma unroll
    for (int j = 0; j < NC; ++j) bsp[j] = b_s + (int64_t)min((n0 + 16 * j) >> 7, NB - 1) * KB;
#pragma unroll
    for (int i = 0; i < MT; ++i) asp[i] = a_s + (int64_t)min(i * 16 + frow, M - 1) * as_rs;
    // LDS: piece p of row r of a tile at r * 128 + ((p ^ (r & 7)) * 16)
    const int wr_off = r8 * 128 + ((pc ^ r8) << 4);                                 // + 1024 for the rows 8 .. 15
    const int rd_lo = frow * 128 + (((2 * fk) ^ (frow & 7)) << 4), rd_hi = frow * 128 + (((2 * fk + 1) ^ (frow & 7)) << 4);

    floatx4 acc[NC][MT];
#pragma unroll
    for (int j = 0; j < NC; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[j][i] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (int kp = k_begin; kp < k_end; kp += UF) {      // uniform in the wave
        intx4 vb[UF][BT], va[UF][2 * MT];      // plain vectors: a struct type here ends up in scratch memory
        float sb[UF][NC], sraw[SV][MT];
#pragma unroll
        for (int u = 0; u < UF; ++u) {
            const int kb = min(kp + u, k_end - 1);
#pragma unroll
            for (int t = 0; t < BT; ++t) vb[u][t] = __builtin_nontemporal_load(reinterpret_cast<const intx4*>(bld[t] + (int64_t)kb * 128));
#pragma unroll
            for (int t = 0; t < 2 * MT; ++t) va[u][t] = *reinterpret_cast<const intx4*>(ald[t] + (int64_t)kb * 128);
#pragma unroll
            for (int j = 0; j < NC; ++j) sb[u][j] = bsp[j][kb];
        }
        // the activation scales: one load per lane and K block of its row touches 16 lines for 64 bytes (UF of them cost
        // 1.5 us per call), so the 4 lanes of a row each load another block's scale and hand it over when it is needed
#pragma unroll
        for (int v = 0; v < SV; ++v) {
            const int kb = min(kp + fk + 4 * v, k_end - 1);
#pragma unroll
            for (int i = 0; i < MT; ++i) sraw[v][i] = asp[i][(int64_t)kb * as_cs];
        }
        intx8 fa[NBUF][MT], fb[NBUF][NC];
        auto through_lds = [&](int u) {      // block u of the pass: registers -> this wave's LDS -> fragments
            uint8_t* buf = lds[wave][u % NBUF];
#pragma unroll
            for (int t = 0; t < BT; ++t) *reinterpret_cast<intx4*>(buf + t * 1024 + wr_off) = vb[u][t];
#pragma unroll
            for (int t = 0; t < 2 * MT; ++t) *reinterpret_cast<intx4*>(buf + (2 * NC + t) * 1024 + wr_off) = va[u][t];
#pragma unroll
            for (int j = 0; j < NC; ++j) {
                const intx4 lo = *reinterpret_cast<const intx4*>(buf + j * 2048 + rd_lo), hi = *reinterpret_cast<const intx4*>(buf + j * 2048 + rd_hi);
                fb[u % NBUF][j] = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const uint8_t* src = buf + (NC + i) * 2048;
                const intx4 lo = *reinterpret_cast<const intx4*>(src + rd_lo), hi = *reinterpret_cast<const intx4*>(src + rd_hi);
                fa[u % NBUF][i] = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
        };
        if (NBUF == 2) through_lds(0);
#pragma unroll
        for (int u = 0; u < UF; ++u) {
            if (NBUF == 1) through_lds(u);
            else if (u + 1 < UF) through_lds(u + 1);
            const bool valid = kp + u < k_end;      // uniform in the wave
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const float sa = __int_as_float(__builtin_amdgcn_ds_bpermute((frow + 16 * (u & 3)) << 2, __float_as_int(sraw[u >> 2][i])));
#pragma unroll
                for (int j = 0; j < NC; ++j) {
                    floatx4 p = mfma_block<FMT>(fb[u % NBUF][j], fa[u % NBUF][i]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) p[e] = valid ? p[e] : 0.0f;
                    fold(acc[j][i], p, sa * sb[u][j]);
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < NC; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][j * MT + i][lane][e] = acc[j][i][e];
    __syncthreads();
    if (wk < SUB) {
        // wave (j, i) of a set reduces column group j, row sub-tile i (fixed order, so results do not depend on timing)
        const int j = wk / MT, i = wk % MT;
        const bool vec_ok = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float t = 0.0f;
#pragma unroll
            for (int w = 0; w < WK; ++w) t += red[set * WK + w][wk][lane][e];
            v[e] = t;
        }
        const int m = i * 16 + frow, n = n0 + 16 * j + 4 * fk;
        if (bias != nullptr) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < N) v[e] += bf16_one(bias[n + e]);
        }
        if (!HALF || fk < 2) store4<OUT>(c, N, m, n, M, N, v, vec_ok);      // HALF: columns 8 .. 15 of the tile belong to the next workgroup
    }
}

template <int MT, int NC, int UF, typename OUT, int FMT>
__global__ __launch_bounds__(kSmWaves * 64) void fp8_gemm_smallm_lines_kernel(const uint8_t* __restrict__ a, const float* __restrict__ a_s,
                                                                               int64_t as_rs, int64_t as_cs, const uint8_t* __restrict__ b,
                                                                               const float* __restrict__ b_s, OUT* __restrict__ c,
                                                                               const uint16_t* __restrict__ bias, int M, int N, int K) {
    smallm_lines_body<MT, NC, UF, OUT, FMT>(a, a_s, as_rs, as_cs, b, b_s, c, bias, M, N, K);
}

// 33..64 rows against a narrow weight and a long K: K is cut into slabs as well (grid row = slab), workgroup (32 columns, slab)
// writes the fp32 partial sums of its K blocks into slab blockIdx.y of a workspace [slabs][M][N], and splitk_reduce_kernel adds
// the slabs in slab order.
template <int UF>
__global__ __launch_bounds__(kSmWaves * 64) void fp8_gemm_smallm_lines_slab_kernel(const uint8_t* __restrict__ a, const float* __restrict__ a_s,
                                                                                    int64_t as_rs, int64_t as_cs, const uint8_t* __restrict__ b,
                                                                                    const float* __restrict__ b_s, float* __restrict__ ws, int M,
                                                                                    int N, int K, int kb_per) {
    const int kb_lo = blockIdx.y * kb_per;
    smallm_lines_body<4, 2, UF, float, 0>(a, a_s, as_rs, as_cs, b, b_s, ws + (size_t)blockIdx.y * M * N, nullptr, M, N, K, kb_lo,
                                          min(K >> 7, kb_lo + kb_per));
}

// up to 16 rows, 32 columns per workgroup, registers held to 128 per lane so that two workgroups share a CU
template <int UF, typename OUT, int FMT>
__global__ __launch_bounds__(kSmWaves * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void fp8_gemm_smallm_lines_occ2_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int64_t as_rs, int64_t as_cs, const uint8_t* __restrict__ b,
    const float* __restrict__ b_s, OUT* __restrict__ c, const uint16_t* __restrict__ bias, int M, int N, int K) {
    smallm_lines_body<1, 2, UF, OUT, FMT>(a, a_s, as_rs, as_cs, b, b_s, c, bias, M, N, K);
}

// up to 16 rows against a short K (1..4 K blocks): WK waves per set of 16 * NC columns, 8 / WK sets per workgroup
template <int NC, int UF, int WK, typename OUT, int FMT>
__global__ __launch_bounds__(kSmWaves * 64) void fp8_gemm_smallm_lines_shortk_kernel(const uint8_t* __restrict__ a,
                                                                                      const float* __restrict__ a_s, int64_t as_rs,
                                                                                      int64_t as_cs, const uint8_t* __restrict__ b,
                                                                                      const float* __restrict__ b_s, OUT* __restrict__ c,
                                                                                      const uint16_t* __restrict__ bias, int M, int N, int K) {
    smallm_lines_body<1, NC, UF, OUT, FMT, false, WK>(a, a_s, as_rs, as_cs, b, b_s, c, bias, M, N, K);
}

// up to 16 rows against a narrow weight: 8 columns per workgroup
template <int UF, typename OUT, int FMT>
__global__ __launch_bounds__(kSmWaves * 64) void fp8_gemm_smallm_lines_half_kernel(const uint8_t* __restrict__ a, const float* __restrict__ a_s,
                                                                                    int64_t as_rs, int64_t as_cs, const uint8_t* __restrict__ b,
                                                                                    const float* __restrict__ b_s, OUT* __restrict__ c,
                                                                                    const uint16_t* __restrict__ bias, int M, int N, int K) {
    smallm_lines_body<1, 1, UF, OUT, FMT, true>(a, a_s, as_rs, as_cs, b, b_s, c, bias, M, N, K);
}

// The same for a grouped GEMM whose groups have at most 16*MT rows each (routed experts at decode): blockIdx.y is the group,
// its rows, weight, weight scales, bias and output rows are the operands of an ordinary small-M GEMM.
struct GroupRows {
    int row_start[kMaxGroups + 1];   // first row of group g; [G] = total rows
};

template <int MT, int NC, int UF, typename OUT>
__global__ __launch_bounds__(kSmWaves * 64) void fp8_grouped_lines_kernel(const uint8_t* __restrict__ a, const float* __restrict__ a_s,
                                                                           int64_t as_rs, int64_t as_cs, const uint8_t* __restrict__ b,
                                                                           const float* __restrict__ b_s, OUT* __restrict__ c,
                                                                           const uint16_t* __restrict__ bias, int N, int K,
                                                                           const GroupRows rows) {
    const int g = blockIdx.y;
    const int r0 = __builtin_amdgcn_readfirstlane(rows.row_start[g]);
    const int M = __builtin_amdgcn_readfirstlane(rows.row_start[g + 1]) - r0;
    if (M <= 0) return;      // uniform in the workgroup
    const int KB = K >> 7, NB = (N + 127) >> 7;
    smallm_lines_body<MT, NC, UF, OUT, 0>(a + (size_t)r0 * K, a_s + (int64_t)r0 * as_rs, as_rs, as_cs, b + (size_t)g * N * K,
                                          b_s + (size_t)g * NB * KB, c + (size_t)r0 * N, bias ? bias + (size_t)g * N : nullptr, M, N, K);
}

// ---------------------------------------------------------------------------
// Row-vector kernel: written for up to 4 rows, used for one (single-token decode against a long K: see gemv_pays).  No
// matrix cores: a weight row against one activation row is a
// dot product, and what bounds it is how many weight bytes every CU has in flight.  A wave owns R weight rows and
// issues all of their loads up front (16 bytes per lane, 1 KB per load and row: K = 7168 -> 7 KB per row in flight), a
// workgroup of 8 waves covers 8 R consecutive rows, so N = 2048 still gives 256 workgroups where the 16-column MFMA
// kernel gives 128 (M = 1, N = 2048, K = 7168: 6.9 -> 4.9 us per call in a replayed graph).  The activation rows and
// their scales are staged in LDS once per workgroup.  Per 16-byte piece a lane converts its bytes to fp32, takes the
// dot product with the matching activation bytes and folds it with a_s[m,kb] * b_s[n/128,kb] (the piece lies in one K
// block); the 64 partial sums of a row are added across the wave at the end.  The sum of a K block is thus formed
// in eight scaled parts instead of one - the same value in exact arithmetic, another rounding (as with the K split).
// ---------------------------------------------------------------------------
constexpr int kGemvMaxK = 16384;     // MR rows x K bytes of activations in LDS
constexpr int kGemvPieces = 8;       // 16-byte pieces per lane and batch over the wave's R rows (R x JB = 8: 8 KB in flight)

template <int FMT>
__device__ __forceinline__ void fp8x4_to_f32(uint32_t w, float (&f)[4]) {
    floatx2 lo, hi;
    if (FMT == 0) {
        lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
        hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    } else {
        lo = __builtin_amdgcn_cvt_pk_f32_bf8((int)w, false);
        hi = __builtin_amdgcn_cvt_pk_f32_bf8((int)w, true);
    }
    f[0] = lo.x; f[1] = lo.y; f[2] = hi.x; f[3] = hi.y;
}

template <int MR, int R, typename OUT, int FMT>
__global__ __launch_bounds__(512) void fp8_gemv_kernel(const uint8_t* __restrict__ a, const float* __restrict__ a_s, int64_t as_rs,
                                                        int64_t as_cs, const uint8_t* __restrict__ b, const float* __restrict__ b_s,
                                                        OUT* __restrict__ c, const uint16_t* __restrict__ bias, int N, int K) {
    __shared__ __attribute__((aligned(16))) uint8_t lds_x[MR * kGemvMaxK];
    __shared__ float lds_sa[MR * (kGemvMaxK / 128)];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int KB = K >> 7, NB = (N + 127) >> 7;
    // the activation rows (16 bytes per thread and step) and their scales
    for (int m = 0; m < MR; ++m) {
        for (int off = tid * 16; off < K; off += 512 * 16)
            *reinterpret_cast<uint4*>(lds_x + m * K + off) = *reinterpret_cast<const uint4*>(a + (int64_t)m * K + off);
        for (int kb = tid; kb < KB; kb += 512) lds_sa[m * KB + kb] = a_s[(int64_t)m * as_rs + (int64_t)kb * as_cs];
    }
    const int n0 = (blockIdx.x * 8 + wave) * R;
    float acc[MR][R];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
    const int pieces = K >> 4;                       // 16-byte pieces of a row; piece p of this lane: p = j * 64 + lane
    bool staged = false;
    constexpr int JB = kGemvPieces / R;
    for (int j0 = 0; j0 * 64 < pieces; j0 += JB) {
        uint4 w[R][JB];
        float sb[R][JB];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int n = min(n0 + r, N - 1);
            const uint8_t* row = b + (int64_t)n * K;
            const float* srow = b_s + (int64_t)min(n >> 7, NB - 1) * KB;
#pragma unroll
            for (int j = 0; j < JB; ++j) {
                const int p = (j0 + j) * 64 + lane;
                const bool ok = p < pieces;
                w[r][j] = ok ? load_nt16(row + (int64_t)p * 16) : make_uint4(0u, 0u, 0u, 0u);
                sb[r][j] = ok ? srow[p >> 3] : 0.0f;
            }
        }
        if (!staged) {      // the weight loads are in flight: now wait for the activation rows
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int j = 0; j < JB; ++j) {
            const int p = (j0 + j) * 64 + lane;
            if (p < pieces) {
                const int kb = p >> 3;
                float wf[R][16];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint32_t ww[4] = {w[r][j].x, w[r][j].y, w[r][j].z, w[r][j].w};
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float f4[4];
                        fp8x4_to_f32<FMT>(ww[q], f4);
                        wf[r][4 * q] = f4[0]; wf[r][4 * q + 1] = f4[1]; wf[r][4 * q + 2] = f4[2]; wf[r][4 * q + 3] = f4[3];
                    }
                }
#pragma unroll
                for (int m = 0; m < MR; ++m) {
                    const uint4 xv = *reinterpret_cast<const uint4*>(lds_x + m * K + p * 16);
                    const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
                    float xf[16];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float f4[4];
                        fp8x4_to_f32<FMT>(xw[q], f4);
                        xf[4 * q] = f4[0]; xf[4 * q + 1] = f4[1]; xf[4 * q + 2] = f4[2]; xf[4 * q + 3] = f4[3];
                    }
                    const float sa = lds_sa[m * KB + kb];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        float d = 0.0f;
#pragma unroll
                        for (int e = 0; e < 16; ++e) d = __builtin_fmaf(wf[r][e], xf[e], d);
                        acc[m][r] = __builtin_fmaf(d, sa * sb[r][j], acc[m][r]);
                    }
                }
            }
        }
    }
    if (!staged) __syncthreads();
    // add the 64 partial sums of every (m, r) across the wave; lane 0 stores
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float v = acc[m][r];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
            const int n = n0 + r;
            if (lane == 0 && n < N) {
                if (bias != nullptr) v += bf16_one(bias[n]);
                if (sizeof(OUT) == 2)
                    reinterpret_cast<uint16_t*>(c)[(int64_t)m * N + n] = (uint16_t)(pack2_bf16(v, 0.0f) & 0xFFFFu);
                else
                    reinterpret_cast<float*>(c)[(int64_t)m * N + n] = v;
            }
        }
}

// ---------------------------------------------------------------------------
// Strip kernel: few rows (<= 16*MT <= 64 per group) against a weight that is wide enough to give every CU
// work without splitting K (many column strips: a vocabulary-sized N, or many experts).  One workgroup = 8
// waves = 128 weight columns of one group, wave w streams rows n0+16w .. +15 of the weight (each row is read
// once, in whole 128-byte lines: 8 rows x one K block per instruction, turned into MFMA fragments through a
// 2 KB tile of LDS that only this wave touches, as in the whole-line small-M kernel; the loads of step s+1
// are issued before the wait for step s), while the activation rows of the step (<= 64 rows x 512 bytes) and
// their scales are copied into LDS ONCE per workgroup and shared by the 8 waves - in the small-M kernels every
// 16 or 32 columns re-read them.  grid = (ceil(N/128), groups).
// ---------------------------------------------------------------------------
constexpr int kStripKC = 4;   // K blocks per step; the 64-row variant takes 2 (59 KB of LDS instead of 92, two workgroups per CU)

template <int MT, typename OUT, int FMT = 0, int KC_ = kStripKC>
__global__ __launch_bounds__(512) void fp8_gemm_strip_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, OUT* __restrict__ c,
    const uint16_t* __restrict__ bias, int N, int K, const GroupTable tbl) {
    constexpr int ROWS = MT * 16, KC = KC_;
    constexpr int CPW = KC * MT / 4;      // activation copy instructions (8 rows x one K block) per wave and step
    static_assert(CPW * 4 == KC * MT, "the step's copies divide evenly among the 8 waves");
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a[2][KC][ROWS * 128];
    __shared__ __attribute__((aligned(256))) float lds_sa[2][KC][64];
    __shared__ __attribute__((aligned(256))) float lds_bs[512];
    __shared__ __attribute__((aligned(256))) uint8_t lds_dummy[8 * 1024];
    __shared__ __attribute__((aligned(16))) uint8_t lds_bt[8][2048];      // a wave's weight tile on its way to fragments

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = blockIdx.y;
    const int r0 = __builtin_amdgcn_readfirstlane(tbl.row_start[g]);
    const int r1 = __builtin_amdgcn_readfirstlane(tbl.row_start[g + 1]);
    const int m_total = __builtin_amdgcn_readfirstlane(tbl.row_start[tbl.n_groups]);
    const int rows = r1 - r0;                  // <= ROWS
    if (rows <= 0) return;
    const int n0 = blockIdx.x * 128;
    const int KB = K >> 7, NB = (N + 127) >> 7;
    const int steps = (KB + KC - 1) / KC;
    const uint8_t* bg = b + (size_t)g * N * K;

    // ---- copies: activation rows (8 rows x 128 bytes per instruction) and their scales (one row per lane)
    const intx4 ra = make_rsrc(a + (size_t)r0 * K, (uint32_t)rows * (uint32_t)K);
    intx4 rs = make_rsrc(a_s, as_bytes);
    if (wave >= KC) rs[2] = 0;
    const int prow = lane >> 3;
    // a wave's instructions all land on row groups of the same parity (j / KC = wave / KC + (8 / KC) t): one swizzle per wave
    const int voff = prow * K + (((lane & 7) ^ swz(((wave / KC) & 1) * 8 + prow)) << 4);
    const int s_voff = min(r0 + min(lane, rows - 1), m_total - 1) * as_rs * 4;
    const uint32_t la0 = lds_addr(&lds_a[0][0][0]);
    const uint32_t ls0 = wave < KC ? lds_addr(&lds_sa[0][wave][0]) : lds_addr(&lds_dummy[0]) + wave * 1024;
    const uint32_t ls_buf = wave < KC ? KC * 64 * 4 : 0;
    auto copy_step = [&](int step, int buf) {
        // instruction j of the step: K block j % KC, row group j / KC (8 rows); wave w takes j = w, w + 8, ...
#pragma unroll
        for (int t = 0; t < CPW; ++t) {
            const int j = wave + 8 * t, kc = j % KC, rg = j / KC;
            dma16(ra, voff, rg * 8 * K + (step * KC + kc) * 128, la0 + (buf * KC + kc) * (ROWS * 128) + rg * 1024);
        }
        dma4(rs, s_voff, min(step * KC + wave, KB - 1) * as_cs * 4, ls0 + buf * ls_buf);
    };

    // ---- weight rows in whole lines: lane l loads piece l & 7 of row 8 t + (l >> 3), t = 0, 1, of every K block
    const int frow = lane & 15, fk = lane >> 4;
    const int r8 = lane >> 3, pc = lane & 7;
    const uint8_t* bld0 = bg + (size_t)min(n0 + wave * 16 + r8, N - 1) * K + pc * 16;
    const uint8_t* bld1 = bg + (size_t)min(n0 + wave * 16 + 8 + r8, N - 1) * K + pc * 16;
    // Two register sets, filled by loads the compiler does not count (like the copies into LDS): the waits are the
    // explicit vmcnt below, so the loads of step s+1 stay in flight across the wait for step s.
    intx4 bset0[KC][2], bset1[KC][2];
    auto load_b = [&](int step, intx4 (&v)[KC][2]) {
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) {
            const int kb = min(step * KC + kc, KB - 1);      // the clamped duplicates are never used
            asm volatile("global_load_dwordx4 %0, %1, off nt" : "=&v"(v[kc][0]) : "v"(bld0 + (size_t)kb * 128) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off nt" : "=&v"(v[kc][1]) : "v"(bld1 + (size_t)kb * 128) : "memory");
        }
    };
    // the wave's LDS tile: piece p of row r at r * 128 + ((p ^ (r & 7)) * 16)
    uint8_t* bt = lds_bt[wave];
    const int bt_wr = r8 * 128 + ((pc ^ r8) << 4);
    const int bt_lo = frow * 128 + (((2 * fk) ^ (frow & 7)) << 4), bt_hi = frow * 128 + (((2 * fk + 1) ^ (frow & 7)) << 4);
    const int a_rd0 = frow * 128 + (((2 * fk) ^ swz(frow)) << 4);
    const int a_rd1 = frow * 128 + (((2 * fk + 1) ^ swz(frow)) << 4);

    floatx4 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

    if (wave == 0) {
        const intx4 rbs = make_rsrc(b_s + ((size_t)g * NB + min(n0 >> 7, NB - 1)) * KB, (uint32_t)KB * 4u);
        for (int cc = 0; cc < KB; cc += 64) dma4(rbs, lane * 4, cc * 4, lds_addr(&lds_bs[cc]));
    }
    auto run_step = [&](int step, intx4 (&cur)[KC][2], intx4 (&nxt)[KC][2]) {
        const int buf = step & 1;
        // the next step's weight rows, then wait for all but those: this step's weights and copies.  No load whose
        // registers are never read is issued: the compiler would hand such registers to other values while the load is
        // still on its way.
        if (step + 1 < steps) {
            load_b(step + 1, nxt);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * KC) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __builtin_amdgcn_s_barrier();                   // the step's activation rows are in LDS; buffer buf^1 is free
        asm volatile("" ::: "memory");
        if (step + 1 < steps) copy_step(step + 1, buf ^ 1);
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) {
            const int kb = step * KC + kc;
            if (kb < KB) {
                const float sb = lds_bs[kb];
                *reinterpret_cast<intx4*>(bt + bt_wr) = cur[kc][0];
                *reinterpret_cast<intx4*>(bt + 1024 + bt_wr) = cur[kc][1];
                const intx4 wlo = *reinterpret_cast<const intx4*>(bt + bt_lo), whi = *reinterpret_cast<const intx4*>(bt + bt_hi);
                const intx8 fb = intx8{wlo[0], wlo[1], wlo[2], wlo[3], whi[0], whi[1], whi[2], whi[3]};
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    const uint8_t* la = &lds_a[buf][kc][i * 2048];
                    const intx4 lo = *reinterpret_cast<const intx4*>(la + a_rd0);
                    const intx4 hi = *reinterpret_cast<const intx4*>(la + a_rd1);
                    const intx8 fa = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    const float sc = lds_sa[buf][kc][i * 16 + frow] * sb;
                    const floatx4 p = mfma_block<FMT>(fb, fa);
                    fold(acc[i], p, sc);
                }
            }
        }
    };
    copy_step(0, 0);
    load_b(0, bset0);
    int step = 0;
    for (; step + 1 < steps; step += 2) {      // unrolled by two: the register sets swap without moves
        run_step(step, bset0, bset1);
        run_step(step + 1, bset1, bset0);
    }
    if (step < steps) run_step(step, bset0, bset1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    const bool vec_ok = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
    const uint16_t* gbias = bias ? bias + (size_t)g * N : nullptr;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = r0 + i * 16 + frow, n = n0 + wave * 16 + 4 * fk;
        float v[4] = {acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
        if (gbias != nullptr) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < N) v[e] += bf16_one(gbias[n + e]);
        }
        store4<OUT>(c, N, m, n, r1, N, v, vec_ok);
    }
}

// ---------------------------------------------------------------------------
// Scalar kernel: any M, N, K, any alignment (K tail reads as zero, like the masked
// loads at offical_kernel.py:82-83).  One thread per output element.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float e4m3_to_f32(uint8_t v) {
    floatx2 f = __builtin_amdgcn_cvt_pk_f32_fp8((int)v, false);
    return f.x;
}

template <typename OUT>
__global__ __launch_bounds__(256) void fp8_gemm_scalar_kernel(const uint8_t* __restrict__ a,
                                                               const float* __restrict__ a_s, int64_t as_rs,
                                                               int64_t as_cs, const uint8_t* __restrict__ b,
                                                               const float* __restrict__ b_s, OUT* __restrict__ c,
                                                               const uint16_t* __restrict__ bias, int M, int N, int K) {
    const int n = blockIdx.x * 16 + (threadIdx.x & 15);
    const int m = block_row() * 16 + (threadIdx.x >> 4);
    if (m >= M || n >= N) return;
    const int KB = (K + 127) >> 7;
    float acc = 0.0f;
    for (int kb = 0; kb < KB; ++kb) {
        float p = 0.0f;
        const int k1 = min(K, (kb + 1) * 128);
        for (int k = kb * 128; k < k1; ++k)
            p = __builtin_fmaf(e4m3_to_f32(a[(int64_t)m * K + k]), e4m3_to_f32(b[(int64_t)n * K + k]), p);
        const float sc = a_s[(int64_t)m * as_rs + (int64_t)kb * as_cs] * b_s[(int64_t)(n >> 7) * KB + kb];
        acc = __builtin_fmaf(p, sc, acc);
    }
    if (bias != nullptr) acc += bf16_one(bias[n]);
    if (sizeof(OUT) == 2)
        reinterpret_cast<uint16_t*>(c)[(int64_t)m * N + n] = (uint16_t)(pack2_bf16(acc, 0.0f) & 0xFFFFu);
    else
        reinterpret_cast<float*>(c)[(int64_t)m * N + n] = acc;
}

// Compute units of the current device (workgroups of the big tile that run at once, one per CU): read from the
// device properties once per device and thread, 256 on a full MI355X, fewer on a partitioned part.
static int cu_count() {
    static thread_local int cached_dev = -1, cached_cus = 256;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return cached_cus;
    if (dev != cached_dev) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) cached_cus = cus;
        cached_dev = dev;
    }
    return cached_cus;
}

// Pre-touches of the shared A / B panels (fp8_gemm_tile.h): a workgroup loads one dword of every line of its share of a
// panel a few K blocks ahead so that the panel copies of all sharers hit in L2.  Measured both ways in one process:
// a GEMM alone after a cache flush is 4-5 % faster with them, a step of act_quant + GEMM repeated back to back 1.7 %
// faster (C3: 468 -> 460 us); only one and the same GEMM relaunched without anything in between, at the board's power
// limit, is 1.5 % slower (397 -> 391 us for 1024 tiles).  On by default; MDY_FP8_PRETOUCH=0 in the environment
// (read once per process) turns them off for the dense tile kernels.
static bool pretouch_enabled() {
    static const bool on = [] {
        const char* e = getenv("MDY_FP8_PRETOUCH");
        return e == nullptr || e[0] != '0';
    }();
    return on;
}

template <int BM, int BN, int WGM, int WGN, int STAGES, typename OUT, int FMT = 0>
static int launch_mfma(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, uint32_t as_bytes,
                       const uint8_t* b, const float* b_s, OUT* c, const uint16_t* bias, int M, int N, int K,
                       int ldc, hipStream_t stream) {
    const int cus = cu_count();
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    // the 256x256 tile fills a CU's LDS: one workgroup per CU that walks its tiles itself
    const int wgs = (BM * BN >= 256 * 256 && tiles_m * tiles_n > cus) ? cus : tiles_m * tiles_n;
    dim3 grid((unsigned)wgs), block(WGM * WGN * 64);
    hipLaunchKernelGGL((fp8_gemm_mfma_kernel<BM, BN, WGM, WGN, STAGES, OUT, 0, 0, 0, FMT>), grid, block, 0, stream, a, a_s, (int)as_rs,
                       (int)as_cs, as_bytes, b, b_s, c, bias, M, N, K, ldc, tiles_m, tiles_n, pretouch_enabled() ? 1 : 0);
    return (int)hipGetLastError();
}


// How many 256-wide tile columns the 256x256 kernel should take when the tile count is not a
// multiple of the CU count: if the last, partly filled round holds at most half a round of
// tiles, those columns are better cut into 128x256 tiles (twice as many workgroups, each ~0.6x
// the time), which fills the machine for one short round instead of half-filling a long one.
// Returns tiles_n when no split pays.
static int main_tile_columns(int tiles_m, int tiles_n) {
    const int cus = cu_count();
    const long total = (long)tiles_m * tiles_n;
    const long full_rounds = total / cus;
    if (full_rounds < 1 || total % cus == 0) return tiles_n;
    const int cols_main = (int)(full_rounds * cus / tiles_m);
    if (cols_main <= 0 || cols_main >= tiles_n) return tiles_n;
    const long rounds_main = ((long)cols_main * tiles_m + cus - 1) / cus;
    const long rem_small = 2L * (tiles_n - cols_main) * tiles_m;
    const double cost_split = (double)rounds_main + 0.6 * (double)((rem_small + cus - 1) / cus);
    const double cost_plain = (double)((total + cus - 1) / cus);
    return cost_split < cost_plain - 0.05 ? cols_main : tiles_n;
}

// 256x256 tiles (one workgroup per CU) when they fill most of the CUs, or when 128x128 tiles (two workgroups
// per CU) would need a second round: 144..199 tiles of 256x256 measured 20-26 % faster than 577..796 of 128x128.
static bool big_tiles_pay(int64_t M, int64_t N) {
    const int cus = cu_count();
    const int64_t t256 = ((M + 255) / 256) * ((N + 255) / 256);
    const int64_t t128 = ((M + 127) / 128) * ((N + 127) / 128);
    return t256 >= 200 || t128 > 2 * cus;
}

// Tile and ring depth for the shapes that do not take 256x256 tiles:
//   0: 128x128, 2 K blocks in LDS (two workgroups share a CU)   3: 64x64, 8 K blocks
//   4: 128x256, 3 K blocks, 8 waves                             5: 256x128, 3 K blocks, 8 waves
//   1: 128x128, 2: 128x64, 6: 128x192 - one workgroup per CU of 4 consumer + 4 producer waves (fp8_gemm_tile_ws), 2 or 3
//      K blocks in flight.  Against the same tiles on the one-body kernel (4 waves, ring of 4 / 6; 8 waves, ring of 3),
//      relaunched back to back / after a cache flush, row-major scales: 2048x2048x7168 46.6 -> 38.5 / 56.5 -> 53.0 us,
//      2048x2048x256 8.0 -> 7.2 / 11.0 -> 10.4 us, 2048x1024x7168 34.3 -> 29.7 / 47.2 -> 44.2 us, 1000x1090x1664
//      13.0 -> 10.2 / 18.0 -> 16.2 us, 4096x1536x7168 59.5 -> 49.7 / 63.6 -> 63.2 us (column-major scales 54.8 -> 47.3 /
//      61.7 -> 57.8 us).
// Measured rule: the smallest tile that still gives every workgroup a CU of its own (the time of these
// shapes goes with the bytes each CU has to pull, not with its MFMAs), and the ring as deep as LDS allows.
// Between 257 and 512 tiles of 128x128 that is a 128x256 tile (else, if those are too many, 256x128), one per CU,
// rather than two 128x128 workgroups per CU: 4096x1536x7168 77 -> 70 us, 8192x1024x7168 91 -> 75 us,
// 1100x6000x16384 178 -> 140 us (K <= 512: 4-6 % slower, so short K keeps the 128x128 tiles).
static int few_tiles_config(int M, int N, int K) {
    const int cus = cu_count();
    const long rows128 = (M + 127) / 128, rows64 = (M + 63) / 64, rows256 = (M + 255) / 256;
    const long cols128 = (N + 127) / 128, cols64 = (N + 63) / 64, cols256 = (N + 255) / 256;
    if (rows64 * cols64 <= cus) return 3;
    if (rows128 * cols64 <= cus) return 2;
    if (rows128 * cols128 <= cus) return 1;
    if (K < 1024) return 0;    // a handful of K blocks: two short workgroups per CU hide each other's prologue and epilogue
    const long wide = rows128 * cols256, tall = rows256 * cols128;
    // more 128x256 tiles than 3/4 of the CUs and 128x192 tiles still one per CU: the smaller tile puts the idle CUs to
    // work (4096x1536x7168: 256 tiles of 128x192 instead of 192 of 128x256), and its wave tiles are small enough for
    // the producer / consumer kernel (measured at that shape, same process, relaunched back to back: 59.5 -> 49.7 us
    // with row-major scales, 54.8 -> 47.3 us with column-major ones; after a cache flush 61.7 -> 57.8 us)
    if (wide <= cus && rows128 * ((N + 191) / 192) <= cus && rows128 * ((N + 191) / 192) > wide) return 6;
    if (wide <= cus) return 4;    // also when it pads more than the tall tile: 12800x384x7168 82 against 95 us
    if (tall <= cus) return 5;
    return 0;
}

template <typename OUT, int FMT = 0>
static int launch_strip(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, uint32_t as_bytes,
                        const uint8_t* b, const float* b_s, OUT* c, const uint16_t* bias, const int64_t* m_splits, int G,
                        int max_rows, int N, int K, hipStream_t stream) {
    GroupTable tbl;
    tbl.n_groups = G;
    int row = 0;
    for (int g = 0; g < G; ++g) {
        tbl.row_start[g] = row;
        tbl.tile_start[g] = 0;
        row += (int)m_splits[g];
    }
    for (int g = G; g <= kMaxGroups; ++g) { tbl.row_start[g] = row; tbl.tile_start[g] = 0; }
    dim3 grid((unsigned)((N + 127) / 128), (unsigned)G), block(512);
#define MDY_STRIP(MT)                                                                                              \
    hipLaunchKernelGGL((fp8_gemm_strip_kernel<MT, OUT, FMT>), grid, block, 0, stream, a, a_s, (int)as_rs, (int)as_cs, as_bytes, b, \
                       b_s, c, bias, N, K, tbl)
    if (max_rows <= 16) MDY_STRIP(1);
    else if (max_rows <= 32) MDY_STRIP(2);
    else if (max_rows <= 48) MDY_STRIP(3);
    else      // 49..64 rows: 2 K blocks per step, so that two workgroups fit a CU's LDS (32 groups x 64 rows, N=4096, K=7168
              // 201 -> 174..193 us; 64 x 56 rows, N=4096, K=2048 127 -> 109 us; M=64, N=36864 79 -> 71 us)
        hipLaunchKernelGGL((fp8_gemm_strip_kernel<4, OUT, FMT, 2>), grid, block, 0, stream, a, a_s, (int)as_rs, (int)as_cs, as_bytes, b, b_s,
                           c, bias, N, K, tbl);
#undef MDY_STRIP
    return (int)hipGetLastError();
}

// The row-vector kernel: one row against a long K that fits its LDS staging (K % 128 == 0, 16-byte aligned operands: the
// caller checks).  With 2..4 rows, and with one row and a K of up to 4096, the whole-line MFMA kernel is ahead (per call
// in a replayed graph: M=4 N=2048 K=7168 9.3 us here, 5.5 there; M=2 N=7168 K=2048 7.3 against 3.9; M=1 N=7168 K=2048
// 5.4 against 3.8; M=1 N=4096 K=4096 5.0 against 4.4; but M=1 N=2048 K=7168 4.0 against 5.0, N=18432 24.5 against 26.6).
static bool gemv_pays(int64_t M, int64_t K) { return M == 1 && K > 4096 && K <= kGemvMaxK; }

// The whole-line small-M kernel (K % 128 == 0, 16-byte aligned operands: the caller checks): up to 16 rows always, up to
// 24 unless there are 200 strips of 128 columns (then the strip kernel), up to 32 unless the weight is very wide, up to 64
// for a middling N.  Measured per call in a replayed graph, K=7168 unless noted: M=32 N=16384 31.3 us here, 34.9 us on
// 128x128 tiles; N=18432 42.0 against 34.8 us; M=16 N=129280 165 against 184 us on strips; M=8 N=32768 42.5 against 59 us;
// M=24 N=32768 K=2048 19.1 against 17.4 us on strips; M=64 N=7168 K=2048 6.6 against 8.7 us on 64x64 tiles, N=12800 K=2048
// 11.7 against 8.9 us, N=4096 17.1 against 24.8 us on the fragment-loading kernel, N=2048 16.2 against 15.5 us.
static bool lines_pays(int64_t M, int64_t N) {
    const int64_t strips = (N + 127) / 128;
    return (M <= 16 || (M <= 24 && strips < 200) || (M <= 32 && strips < 136) || (M <= 64 && N >= 3200 && strips < 100));
}

// the strip kernel: few rows (per group) and enough 128-column strips to fill the CUs without splitting K
static bool strip_pays(int64_t max_rows, int64_t strips) { return max_rows > 4 && max_rows <= 64 && strips >= 200; }

// Up to 64 rows (K % 128 == 0, aligned operands: the caller checks; big_ok: the scales also fit the tile kernels'
// 32-bit addressing).  FMT: operand byte format, 0 e4m3fn, 1 e5m2.
template <typename OUT, int FMT>
static int dispatch_small(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, int64_t as_extent, bool big_ok,
                          const uint8_t* b, const float* b_s, OUT* c, const uint16_t* bias, int M, int N, int K, hipStream_t stream) {
    if (gemv_pays(M, K)) {
        dim3 grid((unsigned)((N + 7) / 8)), block(512);      // one weight row per wave
        hipLaunchKernelGGL((fp8_gemv_kernel<1, 1, OUT, FMT>), grid, block, 0, stream, a, a_s, as_rs, as_cs, b, b_s, c, bias, N, K);
        return (int)hipGetLastError();
    }
    // up to 24 rows, and up to 32 unless the weight is very wide, run the whole-line kernel (measured, K=7168: M=32 N=16384
    // 31.3 us there, 34.9 us on 128x128 tiles; N=18432 42.0 against 34.8 us; M=32 N=129280 240 against 206 us on strips;
    // M=16 N=129280 161 against 182 us on strips; M=24 N=25600 K=4096 28.3 against 34.6 us)
    const bool lines = lines_pays(M, N);
    if (!lines && M <= 64 && big_ok && strip_pays(M, (N + 127) / 128)) {
        const int64_t one = M;
        return launch_strip<OUT, FMT>(a, a_s, as_rs, as_cs, (uint32_t)as_extent, b, b_s, c, bias, &one, 1, M, N, K, stream);
    }
    // 32..64 rows against a wide weight: the whole-line kernel re-reads the activation rows in every one of its N/16 or
    // N/32 workgroups, and from 32 rows on that traffic costs more than the empty rows of an MFMA tile (see lines_pays).
    // (128..199 tiles of 128x128, one per CU, on the producer / consumer body: against the one-body tile, back to back, M=64
    // N=18432 K=7168 36.1 -> 28.2 us, M=48 N=16384 K=2048 13.5 -> 10.7 us, M=64 N=24576 K=1536 12.6 -> 10.5 us; 2-3 % after a flush)
    if (!lines && M >= 32 && M <= 64 && big_ok && (N + 127) / 128 >= 128) {
        const int tiles_n = (N + 127) / 128;
        hipLaunchKernelGGL((fp8_gemm_ws_kernel<128, 128, 2, 2, 4, 4, OUT, FMT>), dim3((unsigned)tiles_n), dim3(512), 0, stream, a, a_s,
                           (int)as_rs, (int)as_cs, (uint32_t)as_extent, b, b_s, c, bias, M, N, K, N, 1, tiles_n, pretouch_enabled() ? 1 : 0);
        return (int)hipGetLastError();
    }
    if (!lines && M >= 32 && M <= 64 && big_ok && (N + 63) / 64 >= 100)
        return launch_mfma<64, 64, 2, 2, 8, OUT, FMT>(a, a_s, as_rs, as_cs, (uint32_t)as_extent, b, b_s, c, bias, M, N, K, N, stream);
    {      // everything else, and what lines_pays prefers: the whole-line kernel
        // 32 columns per workgroup when that still leaves ~200 workgroups (loads alone, M=16: N=7168, K=2048 2.9 -> 2.5 us
        // per call; N=2048, K=7168 3.4 -> 4.1 us); the K blocks of a wave in passes of up to 8 (up to 16 rows, and up to 32 with 16
        // columns per workgroup: M=20 N=2048 K=5120 9.5 -> 6.3 us, M=24 N=4096 K=7168 10.0 -> 8.3 us against passes of 4), 4
        // (33..64 rows, 16 columns: M=64 N=5120 K=4096 17.3 -> 15.2 us against passes of 2) or 2
        const bool wide = (N + 31) / 32 >= 200;
        const int per = (K / 128 + kSmWaves - 1) / kSmWaves, cap = M <= 16 ? 8 : M <= 32 ? (wide ? 4 : 8) : (wide ? 2 : 4);
        int uf = per;
        if (per > cap) {
            uf = cap;
            for (int d = cap; d > cap / 2; --d)
                if (per % d == 0) { uf = d; break; }
        }
        dim3 grid((unsigned)(wide ? (N + 31) / 32 : (N + 15) / 16));
#define MDY_LINES(MT, NC, UF)                                                                                                       \
    hipLaunchKernelGGL((fp8_gemm_smallm_lines_kernel<MT, NC, UF, OUT, FMT>), grid, dim3(kSmWaves * 64), 0, stream, a, a_s, as_rs, as_cs, b, \
                       b_s, c, bias, M, N, K)
#define MDY_LINES_UF4(MT, NC)                         \
    switch (uf) {                                     \
        case 1: MDY_LINES(MT, NC, 1); break;          \
        case 2: MDY_LINES(MT, NC, 2); break;          \
        case 3: MDY_LINES(MT, NC, 3); break;          \
        default: MDY_LINES(MT, NC, 4); break;         \
    }
#define MDY_LINES_UF8(MT, NC)                         \
    switch (uf) {                                     \
        case 5: MDY_LINES(MT, NC, 5); break;          \
        case 6: MDY_LINES(MT, NC, 6); break;          \
        case 7: MDY_LINES(MT, NC, 7); break;          \
        case 8: MDY_LINES(MT, NC, 8); break;          \
        default: MDY_LINES_UF4(MT, NC)                \
    }
        // a short K (1..4 K blocks) against a large weight: fewer waves along K, 2, 4 or 8 sets of columns per workgroup
        // instead of idle waves (per call in a replayed graph: M=16 N=32768 K=512 7.0 -> 5.0 us, M=4 N=129280 K=512 27.3 -> 18.7;
        // small weights lose 0.2 us: N=7168 K=512 2.9 -> 3.1; 12 K blocks as 4 waves x 3: no gain)
        const int KBs = K / 128;
        if (M <= 16 && KBs <= 4 && (int64_t)N * K >= (8 << 20)) {
            const int wk = KBs == 1 ? 1 : KBs == 2 ? 2 : 4;
            const int nc = (wide && wk >= 2) ? 2 : 1, sets = 8 / wk;
            grid = dim3((unsigned)((N + 16 * nc * sets - 1) / (16 * nc * sets)));
#define MDY_SK(NC, WK)                                                                                                              \
    hipLaunchKernelGGL((fp8_gemm_smallm_lines_shortk_kernel<NC, 1, WK, OUT, FMT>), grid, dim3(kSmWaves * 64), 0, stream, a, a_s, as_rs, \
                       as_cs, b, b_s, c, bias, M, N, K)
            if (wk == 1) MDY_SK(1, 1);
            else if (wk == 2 && nc == 2) MDY_SK(2, 2);
            else if (wk == 2) MDY_SK(1, 2);
            else if (nc == 2) MDY_SK(2, 4);
            else MDY_SK(1, 4);
#undef MDY_SK
            return (int)hipGetLastError();
        }
        // a narrow weight (fewer than 100 groups of 16 columns): 8 columns per workgroup, twice the workgroups (per call in
        // a replayed graph: M=16 N=1584 K=4096 4.6 -> 3.8 us, M=16 N=1024 K=8192 7.2 -> 6.3, M=4 N=1536 K=7168 5.3 -> 4.8,
        // M=16 N=576 K=7168 6.0 -> 5.8; N=2048 and wider: no gain)
        if (M <= 16 && (N + 15) / 16 < 100) {
            grid = dim3((unsigned)((N + 7) / 8));
#define MDY_HALF(UF)                                                                                                                \
    hipLaunchKernelGGL((fp8_gemm_smallm_lines_half_kernel<UF, OUT, FMT>), grid, dim3(kSmWaves * 64), 0, stream, a, a_s, as_rs, as_cs, b, \
                       b_s, c, bias, M, N, K)
            switch (uf) {
                case 1: MDY_HALF(1); break;
                case 2: MDY_HALF(2); break;
                case 3: MDY_HALF(3); break;
                case 4: MDY_HALF(4); break;
                case 5: MDY_HALF(5); break;
                case 6: MDY_HALF(6); break;
                case 7: MDY_HALF(7); break;
                default: MDY_HALF(8); break;
            }
#undef MDY_HALF
        } else if (M <= 16 && wide && (uf == 4 || uf == 5)) {
            // passes of 4 or 5 K blocks need 129..138 registers: held to 128, two workgroups share a CU (M=16 N=24576 K=4096
            // 21.7 -> 19.5 us, M=8 N=32768 K=5120 28.5 -> 26.1; deeper passes would spill: N=16384 K=7168 21.8 -> 30.4 us)
            if (uf == 4)
                hipLaunchKernelGGL((fp8_gemm_smallm_lines_occ2_kernel<4, OUT, FMT>), grid, dim3(kSmWaves * 64), 0, stream, a, a_s, as_rs,
                                   as_cs, b, b_s, c, bias, M, N, K);
            else
                hipLaunchKernelGGL((fp8_gemm_smallm_lines_occ2_kernel<5, OUT, FMT>), grid, dim3(kSmWaves * 64), 0, stream, a, a_s, as_rs,
                                   as_cs, b, b_s, c, bias, M, N, K);
        } else if (M <= 16 && wide) {
            MDY_LINES_UF8(1, 2)
        } else if (M <= 16) {
            MDY_LINES_UF8(1, 1)
        } else if (M <= 32 && wide) {
            MDY_LINES_UF4(2, 2)
        } else if (M <= 32) {
            MDY_LINES_UF8(2, 1)
        } else if (wide) {
            if (uf == 1) MDY_LINES(4, 2, 1);
            else MDY_LINES(4, 2, 2);
        } else {
            MDY_LINES_UF4(4, 1)
        }
#undef MDY_LINES_UF8
#undef MDY_LINES_UF4
#undef MDY_LINES
        return (int)hipGetLastError();
    }
    return -1;   // not reached: every M <= 64 ends in the whole-line kernel above
}

// The MFMA tile kernels for more than 64 rows (K % 128 == 0, aligned operands, scales within 2^31 bytes: the caller
// checks).  FMT: operand byte format, 0 e4m3fn, 1 e5m2.
template <typename OUT, int FMT>
static int dispatch_tiles(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, int64_t as_extent, const uint8_t* b,
                          const float* b_s, OUT* c, const uint16_t* bias, int M, int N, int K, hipStream_t stream) {
    const int KB = K / 128;
    if (big_tiles_pay(M, N)) {
        const int tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
        const int cols_main = main_tile_columns(tiles_m, tiles_n);
        const int n_main = cols_main < tiles_n ? cols_main * 256 : N;
        int rc = launch_mfma<256, 256, 2, 4, 2, OUT, FMT>(a, a_s, as_rs, as_cs, (uint32_t)as_extent, b, b_s, c, bias, M, n_main, K, N,
                                                       stream);
        if (rc != 0 || n_main == N) return rc;
        // remaining columns as 128x256 tiles (LDS has room for a ring of 3 K blocks there: 1-2 % of the whole
        // call); n_main is a multiple of 256, so every pointer below keeps its alignment
        return launch_mfma<128, 256, 2, 4, 3, OUT, FMT>(a, a_s, as_rs, as_cs, (uint32_t)as_extent, b + (size_t)n_main * K,
                                                     b_s + (size_t)(n_main >> 7) * KB, c + n_main,
                                                     bias ? bias + n_main : nullptr, M, N - n_main, K, N, stream);
    }
    // Fewer tiles than that: the workgroups no longer fill the CUs, every K block's copy latency shows, and
    // the time goes with K.  Use the LDS that the missing co-resident workgroups leave free for a deeper ring of
    // K blocks in flight, and smaller tiles when even 128x128 tiles leave most CUs idle.
#define MDY_FEW(BM_, BN_, WGM_, WGN_, ST_)                                                                            \
    return launch_mfma<BM_, BN_, WGM_, WGN_, ST_, OUT, FMT>(a, a_s, as_rs, as_cs, (uint32_t)as_extent, b, b_s, c, bias, M, N, K, N, stream)
    switch (few_tiles_config(M, N, K)) {
#define MDY_WS(BM_, BN_, ST_)                                                                                          \
    {                                                                                                                  \
        const int tiles_m = (M + BM_ - 1) / BM_, tiles_n = (N + BN_ - 1) / BN_;                                        \
        hipLaunchKernelGGL((fp8_gemm_ws_kernel<BM_, BN_, 2, 2, 4, ST_, OUT, FMT>), dim3((unsigned)(tiles_m * tiles_n)), dim3(512), 0, \
                           stream, a, a_s, (int)as_rs, (int)as_cs, (uint32_t)as_extent, b, b_s, c, bias, M, N, K, N, tiles_m, \
                           tiles_n, pretouch_enabled() ? 1 : 0);                                                       \
        return (int)hipGetLastError();                                                                                 \
    }
        case 1: MDY_WS(128, 128, 4)
        case 2: MDY_WS(128, 64, 5)
        case 6: MDY_WS(128, 192, 4)
#undef MDY_WS
        case 3: MDY_FEW(64, 64, 2, 2, 8);
        case 4: MDY_FEW(128, 256, 2, 4, 3);
        case 5: MDY_FEW(256, 128, 2, 4, 3);
        default: MDY_FEW(128, 128, 2, 2, 2);
    }
#undef MDY_FEW
}

template <typename OUT>
static int dispatch(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, const uint8_t* b,
                    const float* b_s, OUT* c, const uint16_t* bias, int M, int N, int K, hipStream_t stream) {
    const int KB = (K + 127) / 128;
    // byte extent of the activation scales as the MFMA kernel addresses them
    const int64_t as_extent = ((int64_t)(M - 1) * as_rs + (int64_t)(KB - 1) * as_cs + 1) * 4;
    const bool mfma_ok = (K % 128 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15) == 0) &&
                         ((reinterpret_cast<uintptr_t>(b) & 15) == 0);
    const bool big_ok = mfma_ok && K <= (1 << 16) && as_rs >= 0 && as_cs >= 0 && as_extent < ((int64_t)1 << 31);
    if (!mfma_ok || (M > 64 && !big_ok)) {
        dim3 grid;
        if (!grid_rows((N + 15) / 16, (M + 15) / 16, grid)) return kErrTooManyBlocks;
        hipLaunchKernelGGL((fp8_gemm_scalar_kernel<OUT>), grid, dim3(256), 0, stream, a, a_s, as_rs, as_cs, b, b_s, c,
                           bias, M, N, K);
        return (int)hipGetLastError();
    }
    if (M <= 64) return dispatch_small<OUT, 0>(a, a_s, as_rs, as_cs, as_extent, big_ok, b, b_s, c, bias, M, N, K, stream);
    return dispatch_tiles<OUT, 0>(a, a_s, as_rs, as_cs, as_extent, b, b_s, c, bias, M, N, K, stream);
}

// ---- split-K plan: which tile, how many K slices; ksplit == 1 means "do not split"
struct SplitPlan {
    int config;     // 1: 128x128 tiles, 2: 128x64 (producer / consumer kernel)   3: 64x64 (ring of 8)   4: whole-line kernel, 32 columns
    int ksplit;     // slabs of the workspace
    int kb_per;     // K blocks per slab
};

static SplitPlan plan_split(int64_t M, int64_t N, int64_t K) {
    const int cus = cu_count();
    SplitPlan p{0, 1, 0};
    // up to 32 rows the weight-streaming kernel is as fast; below 32 K blocks the second pass costs more than
    // the split gains
    if (M <= 32 || K % 128 != 0 || K > (1 << 16) || M > (1 << 20)) return p;
    const int KB = (int)(K / 128);
    if (big_tiles_pay(M, N) || KB < 32) return p;
    if (M <= 64 && strip_pays(M, (N + 127) / 128)) return p;
    // up to 32 K blocks the whole-line kernel is as fast without the second pass (M=64 N=6400 K=4096: 10.6 against 12.9 us)
    if (lines_pays(M, N) && KB <= 32) return p;
    // 33..64 rows against a weight so narrow that its groups of 32 columns leave three quarters of the CUs idle: the
    // whole-line kernel over slabs of K (per call in a replayed graph: M=64 N=2048 K=7168 11.3 -> 9.5 us, M=40 11.4 -> 8.9 us,
    // M=64 N=1536 K=7168 11.0 -> 9.2 us against 64x64 tiles; N=4096: 12.9 against 12.8 us, so wider weights keep the tiles)
    if (M <= 64) {
        const long strips = (N + 31) / 32;
        long ks = cus / strips;
        if (ks > KB / 8) ks = KB / 8;
        if (ks > 8) ks = 8;
        if (strips * 4 <= cus && ks >= 2) {
            p.config = 4;
            p.kb_per = (int)((KB + ks - 1) / ks);
            p.ksplit = (KB + p.kb_per - 1) / p.kb_per;
            return p;
        }
        // up to 32 K blocks the whole-line kernel in one launch is ahead of tiles over slabs of K (M=64 N=3072 K=4096: 8.7
        // against 10.5 us)
        if (KB <= 32) return p;
    }
    // the largest tile that, cut into slabs of at least 8 K blocks, still yields a workgroup for most CUs
    const long rows128 = (M + 127) / 128, rows64 = (M + 63) / 64;
    const long cols128 = (N + 127) / 128, cols64 = (N + 63) / 64;
    const long tiles[4] = {0, rows128 * cols128, rows128 * cols64, rows64 * cols64};
    for (int cfg = 1; cfg <= 3; ++cfg) {
        if (cfg != 3 && M <= 64) continue;                       // 128-row tiles would be half empty
        long ks = cus / tiles[cfg];
        if (ks > KB / 8) ks = KB / 8;
        if (ks < 2) continue;
        if (tiles[cfg] * ks < cus * 3 / 4 && cfg != 3) continue;  // a smaller tile fills the machine better
        p.config = cfg;
        p.kb_per = (int)((KB + ks - 1) / ks);
        p.ksplit = (KB + p.kb_per - 1) / p.kb_per;
        if (p.ksplit < 2) p = SplitPlan{0, 1, 0};
        return p;
    }
    return p;
}

// Activation scales [M, K/128] row-major -> [K/128, M]: with the K-block index as the slow dimension the 64
// scales a wave copies per K block are 256 contiguous bytes instead of one dword from each of 64 cache lines
// (the tile kernels fetch every such line once per K block: +50 % line requests on top of the operand panels).
__global__ __launch_bounds__(256) void transpose_scales_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                               int M, int KB, int64_t in_row_stride) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;      // 32 x 8 threads
    const int m0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = m0 + ty + 8 * r, kb = k0 + tx;
        if (m < M && kb < KB) tile[ty + 8 * r][tx] = in[(int64_t)m * in_row_stride + kb];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int kb = k0 + ty + 8 * r, m = m0 + tx;
        if (m < M && kb < KB) out[(int64_t)kb * M + m] = tile[tx][ty + 8 * r];
    }
}

// scratch for the transposed activation scales of the shapes that run on MFMA tiles without a K split
static int64_t scale_scratch_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 64 || K % 128 != 0 || K > (1 << 16) || M > (1 << 20)) return 0;
    // the copy kernel takes ~3 us and the gain is ~3 % of the GEMM: worth it from ~200 us of GEMM on
    if ((double)M * (double)N * (double)K < 2e11) return 0;
    return ((M * (K / 128) * 4 + 255) / 256) * 256;
}

int64_t fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const SplitPlan p = plan_split(M, N, K);
    return p.ksplit > 1 ? (int64_t)p.ksplit * M * N * 4 : scale_scratch_bytes(M, N, K);
}

// returns -1 when the shape / pointers do not qualify (the caller then runs the plain path)
template <typename OUT>
static int launch_splitk(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, const uint8_t* b,
                         const float* b_s, OUT* c, const uint16_t* bias, int M, int N, int K, float* ws,
                         int64_t ws_bytes, hipStream_t stream) {
    const SplitPlan p = plan_split(M, N, K);
    if (p.ksplit < 2 || ws == nullptr || ws_bytes < (int64_t)p.ksplit * M * N * 4) return -1;
    const int KB = K / 128;
    const int64_t as_extent = ((int64_t)(M - 1) * as_rs + (int64_t)(KB - 1) * as_cs + 1) * 4;
    const bool ok = ((reinterpret_cast<uintptr_t>(a) & 15) == 0) && ((reinterpret_cast<uintptr_t>(b) & 15) == 0) &&
                    ((reinterpret_cast<uintptr_t>(ws) & 15) == 0) && as_rs >= 0 && as_cs >= 0 &&
                    as_extent < ((int64_t)1 << 31);
    if (!ok) return -1;
#define MDY_SPLIT(BM_, BN_, ST_)                                                                                      \
    {                                                                                                                 \
        const int tiles_m = (M + BM_ - 1) / BM_, tiles_n = (N + BN_ - 1) / BN_;                                       \
        hipLaunchKernelGGL((fp8_gemm_splitk_kernel<BM_, BN_, 2, 2, ST_>), dim3((unsigned)(tiles_m * tiles_n * p.ksplit)), \
                           dim3(256), 0, stream, a, a_s, (int)as_rs, (int)as_cs, (uint32_t)as_extent, b, b_s, ws, M, N, K, \
                           tiles_m, tiles_n, p.ksplit, p.kb_per);                                                     \
    }
    if (p.config == 4) {
        dim3 grid((unsigned)((N + 31) / 32), (unsigned)p.ksplit);
        if (p.kb_per <= kSmWaves)
            hipLaunchKernelGGL((fp8_gemm_smallm_lines_slab_kernel<1>), grid, dim3(kSmWaves * 64), 0, stream, a, a_s, as_rs, as_cs, b, b_s, ws,
                               M, N, K, p.kb_per);
        else
            hipLaunchKernelGGL((fp8_gemm_smallm_lines_slab_kernel<2>), grid, dim3(kSmWaves * 64), 0, stream, a, a_s, as_rs, as_cs, b, b_s, ws,
                               M, N, K, p.kb_per);
    }
#define MDY_SPLIT_WS(BM_, BN_, ST_)                                                                                   \
    {                                                                                                                 \
        const int tiles_m = (M + BM_ - 1) / BM_, tiles_n = (N + BN_ - 1) / BN_;                                       \
        hipLaunchKernelGGL((fp8_gemm_splitk_ws_kernel<BM_, BN_, ST_>), dim3((unsigned)(tiles_m * tiles_n * p.ksplit)), \
                           dim3(512), 0, stream, a, a_s, (int)as_rs, (int)as_cs, (uint32_t)as_extent, b, b_s, ws, M, N, K, \
                           tiles_m, tiles_n, p.ksplit, p.kb_per);                                                     \
    }
    else if (p.config == 1) MDY_SPLIT_WS(128, 128, 4)
    else if (p.config == 2) MDY_SPLIT_WS(128, 64, 5)
    else MDY_SPLIT(64, 64, 8)
#undef MDY_SPLIT
#undef MDY_SPLIT_WS
    int rc = (int)hipGetLastError();
    if (rc != 0) return rc;
    const int64_t MN = (int64_t)M * N;
    const bool vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
    if (vec)
        hipLaunchKernelGGL((splitk_reduce_kernel<OUT, true>), dim3((unsigned)((MN / 4 + 255) / 256)), dim3(256), 0, stream,
                           ws, c, bias, MN, N, p.ksplit);
    else
        hipLaunchKernelGGL((splitk_reduce_kernel<OUT, false>), dim3((unsigned)((MN + 255) / 256)), dim3(256), 0, stream, ws,
                           c, bias, MN, N, p.ksplit);
    return (int)hipGetLastError();
}

int launch_fp8_gemm_nt_ws(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                          const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                          void* workspace, int64_t workspace_bytes, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    int rc = -1;
    if (out_dtype == 0)
        rc = launch_splitk<uint16_t>(static_cast<const uint8_t*>(a), a_s, as_row_stride, as_col_stride,
                                     static_cast<const uint8_t*>(b), b_s, static_cast<uint16_t*>(c),
                                     static_cast<const uint16_t*>(bias), (int)M, (int)N, (int)K,
                                     static_cast<float*>(workspace), workspace_bytes, stream);
    else
        rc = launch_splitk<float>(static_cast<const uint8_t*>(a), a_s, as_row_stride, as_col_stride,
                                  static_cast<const uint8_t*>(b), b_s, static_cast<float*>(c),
                                  static_cast<const uint16_t*>(bias), (int)M, (int)N, (int)K,
                                  static_cast<float*>(workspace), workspace_bytes, stream);
    if (rc >= 0) return rc;
    // no K split: with row-major activation scales and room in the workspace, hand the tile kernels a
    // transposed copy (C3: 505 -> 491 us, C4: 487 -> 466 us for a 3 us copy kernel)
    const int64_t need = scale_scratch_bytes(M, N, K);
    if (need > 0 && workspace != nullptr && workspace_bytes >= need && as_col_stride == 1 && as_row_stride >= K / 128 &&
        as_row_stride > 1 && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
        const int KB = (int)(K / 128);
        float* ts = static_cast<float*>(workspace);
        hipLaunchKernelGGL(transpose_scales_kernel, dim3((unsigned)((M + 31) / 32), (unsigned)((KB + 31) / 32)), dim3(256), 0,
                           stream, a_s, ts, (int)M, KB, as_row_stride);
        rc = (int)hipGetLastError();
        if (rc != 0) return rc;
        return launch_fp8_gemm_nt(a, ts, 1, M, b, b_s, c, bias, M, N, K, out_dtype, stream);
    }
    return launch_fp8_gemm_nt(a, a_s, as_row_stride, as_col_stride, b, b_s, c, bias, M, N, K, out_dtype, stream);
}

// Which kernel family a call would run (the same tests as dispatch() / launch_splitk(), no launch):
//   0 scalar (one thread per output element)   1 small-M weight streaming   2 strip   3 MFMA tiles
//   4 MFMA tiles split along K (needs the workspace)
int fp8_gemm_path(const void* a, const void* b, int64_t as_rs, int64_t as_cs, int64_t M, int64_t N, int64_t K,
                  int with_workspace) {
    const int64_t KB = (K + 127) / 128;
    const int64_t as_extent = ((M - 1) * as_rs + (KB - 1) * as_cs + 1) * 4;
    const bool mfma_ok = (K % 128 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15) == 0) &&
                         ((reinterpret_cast<uintptr_t>(b) & 15) == 0);
    const bool big_ok = mfma_ok && K <= (1 << 16) && as_rs >= 0 && as_cs >= 0 && as_extent < ((int64_t)1 << 31);
    if (with_workspace && big_ok && plan_split(M, N, K).ksplit > 1) return 4;
    if (!mfma_ok || (M > 64 && !big_ok)) return 0;
    if (lines_pays(M, N)) return 1;
    if (M <= 64 && big_ok && strip_pays(M, (N + 127) / 128)) return 2;
    if (M >= 32 && M <= 64 && big_ok && ((N + 127) / 128 >= 128 || (N + 63) / 64 >= 100)) return 3;
    if (M <= 64) return 1;
    return 3;
}

// ---------------------------------------------------------------------------
// The workspace call for callers that cannot allocate (HIP graph capture, serving loops, harnesses that forbid
// hipMalloc): the scratch memory is a file-scope device array of kStaticScratchBytes that every GPU the library
// runs on holds until the process ends.  In host code the array's name is only a stand-in: its device address
// is resolved once per device with hipGetSymbolAddress (each GPU has its own copy at its own address) and that
// pointer, never the name, goes to the kernels.  Nothing has to start at zero: the K-split kernels write every
// element of the slabs they use before the reduction reads them, and the scale transposition writes all of its
// output.  All calls on one GPU share the array, so calls that overlap in time on one GPU race.
// ---------------------------------------------------------------------------
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the current device; resolves it on the first call per device
int static_scratch_ptr(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

int launch_fp8_gemm_nt_static(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                              const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                              hipStream_t stream) {
    void* ws = nullptr;
    const int rc = static_scratch_ptr(&ws);
    if (rc != 0) return rc;
    return launch_fp8_gemm_nt_ws(a, a_s, as_row_stride, as_col_stride, b, b_s, c, bias, M, N, K, out_dtype, ws,
                                 kStaticScratchBytes, stream);
}

// The MFMA kernels on e5m2 operands: the tile, weight-streaming and strip kernels (the K split and the grouped GEMM are
// e4m3fn only).  Returns -1 when the operands do not qualify (K % 128 != 0, K > 65536, unaligned, scales beyond 2^31 bytes).
int launch_fp8_gemm_nt_e5m2(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                            const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                            hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    const int64_t KB = K / 128;
    const int64_t as_extent = ((M - 1) * as_row_stride + (KB - 1) * as_col_stride + 1) * 4;
    const bool ok = K % 128 == 0 && K <= (1 << 16) && as_row_stride >= 0 && as_col_stride >= 0 &&
                    as_extent < ((int64_t)1 << 31) &&
                    ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0;
    if (!ok) return -1;
    const uint8_t* ap = static_cast<const uint8_t*>(a);
    const uint8_t* bp = static_cast<const uint8_t*>(b);
    const uint16_t* biasp = static_cast<const uint16_t*>(bias);
    if (M <= 64) {
        if (out_dtype == 0)
            return dispatch_small<uint16_t, 1>(ap, a_s, as_row_stride, as_col_stride, as_extent, true, bp, b_s, static_cast<uint16_t*>(c),
                                               biasp, (int)M, (int)N, (int)K, stream);
        return dispatch_small<float, 1>(ap, a_s, as_row_stride, as_col_stride, as_extent, true, bp, b_s, static_cast<float*>(c), biasp,
                                        (int)M, (int)N, (int)K, stream);
    }
    if (out_dtype == 0)
        return dispatch_tiles<uint16_t, 1>(ap, a_s, as_row_stride, as_col_stride, as_extent, bp, b_s, static_cast<uint16_t*>(c), biasp,
                                           (int)M, (int)N, (int)K, stream);
    return dispatch_tiles<float, 1>(ap, a_s, as_row_stride, as_col_stride, as_extent, bp, b_s, static_cast<float*>(c), biasp, (int)M,
                                    (int)N, (int)K, stream);
}

int launch_fp8_gemm_nt(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                       const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                       hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    const uint8_t* ap = static_cast<const uint8_t*>(a);
    const uint8_t* bp = static_cast<const uint8_t*>(b);
    const uint16_t* biasp = static_cast<const uint16_t*>(bias);
    if (out_dtype == 0)
        return dispatch<uint16_t>(ap, a_s, as_row_stride, as_col_stride, bp, b_s, static_cast<uint16_t*>(c), biasp,
                                  (int)M, (int)N, (int)K, stream);
    return dispatch<float>(ap, a_s, as_row_stride, as_col_stride, bp, b_s, static_cast<float*>(c), biasp, (int)M,
                           (int)N, (int)K, stream);
}

template <typename OUT>
static int launch_grouped(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, uint32_t as_bytes,
                          const uint8_t* b, const float* b_s, OUT* c, const uint16_t* bias, const int64_t* m_splits,
                          int G, int N, int K, hipStream_t stream) {
    GroupTable tbl;
    tbl.n_groups = G;
    int row = 0, trow = 0;
    for (int g = 0; g < G; ++g) {
        tbl.row_start[g] = row;
        tbl.tile_start[g] = trow;
        row += (int)m_splits[g];
        trow += ((int)m_splits[g] + 255) / 256;
    }
    for (int g = G; g <= kMaxGroups; ++g) { tbl.row_start[g] = row; tbl.tile_start[g] = trow; }
    if (trow == 0) return 0;
    const int tiles_n = (N + 255) / 256;
    dim3 grid((unsigned)(trow * tiles_n)), block(512);
    hipLaunchKernelGGL((fp8_grouped_gemm_kernel<OUT>), grid, block, 0, stream, a, a_s, (int)as_rs, (int)as_cs, as_bytes, b, b_s,
                       c, bias, N, K, tiles_n, tbl);
    return (int)hipGetLastError();
}

// Groups of at most 64 rows each on the whole-line small-M kernel, one grid row per group (32 weight columns per workgroup).
template <typename OUT>
static int launch_grouped_lines(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, const uint8_t* b, const float* b_s,
                                OUT* c, const uint16_t* bias, const int64_t* m_splits, int G, int max_rows, int N, int K,
                                hipStream_t stream) {
    GroupRows rows;
    int row = 0;
    for (int g = 0; g < G; ++g) {
        rows.row_start[g] = row;
        row += (int)m_splits[g];
    }
    for (int g = G; g <= kMaxGroups; ++g) rows.row_start[g] = row;
    const int per = (K / 128 + kSmWaves - 1) / kSmWaves, cap = max_rows <= 16 ? 8 : max_rows <= 32 ? 4 : 2;
    int uf = per;
    if (per > cap) {
        uf = cap;
        for (int d = cap; d > cap / 2; --d)
            if (per % d == 0) { uf = d; break; }
    }
    dim3 grid((unsigned)((N + 31) / 32), (unsigned)G), block(kSmWaves * 64);
#define MDY_GL(MT, UF)                                                                                                             \
    hipLaunchKernelGGL((fp8_grouped_lines_kernel<MT, 2, UF, OUT>), grid, block, 0, stream, a, a_s, as_rs, as_cs, b, b_s, c, bias, N, K, rows)
    if (max_rows <= 16) {
        if (uf <= 1) MDY_GL(1, 1);
        else if (uf <= 2) MDY_GL(1, 2);
        else if (uf <= 4) MDY_GL(1, 4);
        else if (uf <= 7) MDY_GL(1, 7);
        else MDY_GL(1, 8);
    } else if (max_rows <= 32) {
        if (uf <= 1) MDY_GL(2, 1);
        else if (uf <= 2) MDY_GL(2, 2);
        else MDY_GL(2, 4);
    } else {
        if (uf <= 1) MDY_GL(4, 1);
        else MDY_GL(4, 2);
    }
#undef MDY_GL
    return (int)hipGetLastError();
}

template <typename OUT>
static int dispatch_grouped(const uint8_t* a, const float* a_s, int64_t as_rs, int64_t as_cs, const uint8_t* b,
                            const float* b_s, OUT* c, const uint16_t* bias, const int64_t* m_splits, int G, int64_t M,
                            int N, int K, hipStream_t stream) {
    const int KB = (K + 127) / 128, NB = (N + 127) / 128;
    const int64_t as_extent = ((M - 1) * as_rs + (int64_t)(KB - 1) * as_cs + 1) * 4;
    const bool tiled_ok = (K % 128 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15) == 0) &&
                          ((reinterpret_cast<uintptr_t>(b) & 15) == 0) && K <= (1 << 16) && as_rs >= 0 && as_cs >= 0 &&
                          as_extent < ((int64_t)1 << 31) && G <= kMaxGroups;
    if (tiled_ok) {
        int64_t max_rows = 0;
        for (int g = 0; g < G; ++g) max_rows = m_splits[g] > max_rows ? m_splits[g] : max_rows;
        // few rows per group (routed experts at decode): the whole-line small-M kernel up to 16 rows, and up to 64 when
        // there are too few strips for the strip kernel (per call in a replayed graph, strip or tile kernel -> here:
        // 32 groups x 16 rows, N=4096, K=7168 191 -> 176 us = 5.3 TB/s of weights; 64 x 2 rows 323 -> 279 us = 6.7 TB/s;
        // 8 x 4 rows, N=2048 43 -> 21 us; 4 x 16 rows, N=2048 42 -> 13 us; 16 x 24 rows, N=1536, K=4096 28.7 -> 26.5 us; but
        // 32 x 24 rows 201 us on strips, 230 us here; 32 x 40 rows 168 against 288 us; 32 x 64 rows 200 against 324 us)
        const bool strips = strip_pays(max_rows, (int64_t)G * ((N + 127) / 128));
        if (max_rows <= 16 || (max_rows <= 64 && !strips))
            return launch_grouped_lines<OUT>(a, a_s, as_rs, as_cs, b, b_s, c, bias, m_splits, G, (int)max_rows, N, K, stream);
        if (strips)
            return launch_strip<OUT>(a, a_s, as_rs, as_cs, (uint32_t)as_extent, b, b_s, c, bias, m_splits, G, (int)max_rows, N, K,
                                     stream);
        return launch_grouped<OUT>(a, a_s, as_rs, as_cs, (uint32_t)as_extent, b, b_s, c, bias, m_splits, G, N, K, stream);
    }
    // any other shape / alignment: one dense call per group
    int64_t row = 0;
    for (int g = 0; g < G; ++g) {
        const int64_t mg = m_splits[g];
        if (mg > 0) {
            int rc = dispatch<OUT>(a + row * K, a_s + row * as_rs, as_rs, as_cs, b + (size_t)g * N * K,
                                   b_s + (size_t)g * NB * KB, c + row * N, bias ? bias + (size_t)g * N : nullptr, (int)mg, N, K,
                                   stream);
            if (rc != 0) return rc;
        }
        row += mg;
    }
    return 0;
}

int launch_fp8_grouped_gemm_nt(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                               const void* b, const float* b_s, void* c, const void* bias, const int64_t* m_splits,
                               int64_t G, int64_t M, int64_t N, int64_t K, int out_dtype, hipStream_t stream) {
    if (M == 0 || N == 0 || G == 0) return 0;
    const uint8_t* ap = static_cast<const uint8_t*>(a);
    const uint8_t* bp = static_cast<const uint8_t*>(b);
    const uint16_t* biasp = static_cast<const uint16_t*>(bias);
    if (out_dtype == 0)
        return dispatch_grouped<uint16_t>(ap, a_s, as_row_stride, as_col_stride, bp, b_s, static_cast<uint16_t*>(c), biasp,
                                          m_splits, (int)G, M, (int)N, (int)K, stream);
    return dispatch_grouped<float>(ap, a_s, as_row_stride, as_col_stride, bp, b_s, static_cast<float*>(c), biasp, m_splits,
                                   (int)G, M, (int)N, (int)K, stream);
}

}  // namespace mdy
