// The MFMA tile body of the block-scaled FP8 GEMM and the kernel that walks tiles with it (gfx950 only).
// Shared by fp8_gemm.hip (the product kernels) and gemm_probe.hip (the timing probe that switches parts of the
// K loop off); the description of the kernels is at the top of fp8_gemm.hip.  Two bodies: fp8_gemm_tile (every wave
// does everything; the large tiles) and fp8_gemm_tile_ws (producer / consumer waves; 128x192 tiles).
#pragma once
#include "common.h"

namespace mdy {

// chunk swizzle of an LDS row; depends on row bits 0..3 only so that rows 16 apart share it
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// One 128-deep scale block of a 16x16 sub-tile, from zero: v_mfma_f32_16x16x128_f8f6f4 with e4m3 operands and unit
// hardware scales.  The weight rows go in as the MFMA's rows and the activation rows as its columns, so a lane's
// four results are four consecutive n of one m.
// FMT: byte format of both operands, 0 e4m3fn, 1 e5m2 (the instruction's cbsz / blgp fields).
template <int FMT = 0>
__device__ __forceinline__ floatx4 mfma_block(const intx8& weight_rows, const intx8& act_rows) {
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(weight_rows, act_rows, zero, FMT, FMT, 0, 0, 0, 0);
}

// The promotion of one K block (offical_kernel.py:86): acc += (MFMA result of the block) * (its combined scale).
__device__ __forceinline__ void fold(floatx4& acc, const floatx4& p, float sc) {
    acc[0] = __builtin_fmaf(p[0], sc, acc[0]);
    acc[1] = __builtin_fmaf(p[1], sc, acc[1]);
    acc[2] = __builtin_fmaf(p[2], sc, acc[2]);
    acc[3] = __builtin_fmaf(p[3], sc, acc[3]);
}

template <typename OUT>
__device__ __forceinline__ void store4(OUT* c, int64_t ldc, int m, int n, int M, int N, const float (&v)[4], bool vec_ok) {
    if (m >= M || n >= N) return;
    OUT* p = c + (int64_t)m * ldc + n;
    if (vec_ok && n + 3 < N) {
        // plain (cached) stores: the 8-byte pieces of a line written by different instructions are
        // merged in L2; non-temporal stores measured ~5 % slower here
        if (sizeof(OUT) == 2) {
            *reinterpret_cast<uint2*>(p) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
        } else {
            *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (n + i < N) {
                if (sizeof(OUT) == 2)
                    reinterpret_cast<uint16_t*>(p)[i] = (uint16_t)(pack2_bf16(v[i], 0.0f) & 0xFFFFu);
                else
                    reinterpret_cast<float*>(p)[i] = v[i];
            }
        }
    }
}

// raw buffer descriptor: base, byte range, no stride, no swizzle
__device__ __forceinline__ intx4 make_rsrc(const void* base, uint32_t bytes) {
    const uint64_t p = reinterpret_cast<uint64_t>(base);
    intx4 r;
    r[0] = (int)(uint32_t)p;
    r[1] = (int)((uint32_t)(p >> 32) & 0xFFFFu);
    r[2] = (int)bytes;
    r[3] = 0x00020000;
    return r;
}
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const void*)p);
}
// 64 lanes x 16 bytes, global (descriptor base + voff + soff) -> LDS (lds + lane*16).
// Issued as inline asm so that the copy stays asynchronous: the kernel waits for it
// with an explicit s_waitcnt vmcnt + barrier once per K block, nowhere else.
// rsrc, soff and lds must be wave-uniform.
__device__ __forceinline__ void dma16(const intx4& rsrc, int voff, int soff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
                 :: "v"(voff), "s"(rsrc), "s"(soff), "s"(lds) : "memory");
}
__device__ __forceinline__ void dma4(const intx4& rsrc, int voff, int soff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dword %0, %1, %2 offen lds"
                 :: "v"(voff), "s"(rsrc), "s"(soff), "s"(lds) : "memory");
}

// Shares of the panel pre-touches: the A panel of a tile row is cut into 2^a_sh shares among the tiles of
// that row that run side by side, the B panel of a tile column into 2^b_sh shares among its tile rows.
// In the producer/consumer kernel a touch covers kTouchBurst CONSECUTIVE lines (K blocks) of a row at a time: a K
// block's copy needs one 128-byte line from each of a panel's rows, rows that lie K bytes apart - for memory that is
// one isolated line per DRAM page and K block.  Touching 4 lines (512 contiguous bytes) of a row every 4th K block
// instead of one line every K block asks memory for the same bytes in a quarter of the places.  Measured one launch
// after a cache flush (operands cold, caches full of dirty lines), same process, row-major scales: 4096x1536x7168
// 63.5 -> 57.2 us, 2048x2048x7168 52.7 -> 44.2 us, 2048x1024x7168 44.6 -> 34.4 us, 1024x4096x7168 54.0 -> 44.8 us;
// bursts of 2 / 8 / 16 lines are 1.5 / 1.4 / 4.3 us slower than 4 at the first shape; touching single lines further
// ahead (5 or 8 K blocks instead of 2) changes nothing; relaunched back to back (operands in the caches) all tie.
// The one-body kernel (hundreds of tiles, many workgroups on every panel) keeps single-line touches: bursts made
// 4096x18432x7168 472 -> 491 us and 4096x7168x18432 455 -> 468 us back to back.
constexpr int kTouchBurstLog = 2, kTouchBurst = 1 << kTouchBurstLog;
// a byte offset beyond every descriptor of these kernels (their ranges stay below 2^31): such a lane accesses nothing
constexpr int kOutOfRange = 0x7ffffff0;
struct Duty {
    int a_duty, a_sh, b_duty, b_sh;
};

// LDS of one tile workgroup, carved out of a pool that the kernel declares: the ring of A and B panels, the ring of activation scales, the tile's weight
// scales for all K blocks, and a dummy area for copies that must go nowhere.
template <int BM, int BN, int WAVES, int STAGES>
struct TileLds {
    static constexpr int NBS = (BN + 127) / 128;
    static constexpr int a_off = 0;
    static constexpr int b_off = a_off + STAGES * BM * 128;
    static constexpr int s_off = b_off + STAGES * BN * 128;
    static constexpr int bs_off = s_off + (STAGES * BM * 4 + 255) / 256 * 256;
    static constexpr int dummy_off = bs_off + NBS * 512 * 4;
    static constexpr int bytes = dummy_off + WAVES * 512;
};

// LDS of a wave-specialized tile workgroup: separate ring depths for the a panels, the b panels and the activation scales.
template <int BM, int BN, int WAVES, int SA, int SB, int SS>
struct TileLdsWs {
    static constexpr int NBS = (BN + 127) / 128;
    static constexpr int BSROW = 512;
    static constexpr int a_off = 0;
    static constexpr int b_off = a_off + SA * BM * 128;
    static constexpr int s_off = b_off + SB * BN * 128;
    static constexpr int bs_off = s_off + (SS * BM * 4 + 255) / 256 * 256;
    static constexpr int dummy_off = bs_off + NBS * BSROW * 4;
    static constexpr int bytes = dummy_off + WAVES * 512;
};

// One BM x BN tile of C: WGM x WGN waves, each wave (BM/WGM) x (BN/WGN).
//   rows m0 .. min(m0+BM, m_end) of a (m_end = end of the matrix, or of the expert group the tile belongs to),
//   columns n0 .. of b / b_s / bias (already offset to the group's weight), K % 128 == 0, K <= 65536,
//   K blocks kb0 .. kb1-1 of them (all of them except in the split-K kernel).
// as_bytes = byte size of the addressed part of a_s (host computed, < 2^31); m_total = rows of a_s.
// duty: which share of the A / B panel lines this workgroup pre-touches for the workgroups that copy the same
// panels (those with the same tile row / tile column), and into how many shares the panels are cut.
//
// Schedule of one K block (NT = TI*TJ MFMA slots, each followed DEPTH slots later by its 4 FMAs):
//   slots 0..      the last copies of K block kb+1 (those that did not fit into the tail below), one per GAP
//                  slots, then one "duty touch" load for K block kb+3;
//   slot TB        = first MFMA of the last streamed fragment: every LDS read of this K block has been
//                  consumed, so the wave waits for its copies of kb+1 and meets the others at THE barrier
//                  of the K block; behind it buffer `cur` is free and buffer `cur^1` is complete;
//   slots TB..     while the last MFMAs and FMAs of kb still run: reload the held fragments, the first
//                  streamed fragment and the scales from buffer cur^1, and issue the first copies of kb+2
//                  into buffer cur, one per GAP slots.
// So the LDS latency after the barrier and the issue time of the copies sit in the shadow of the matrix
// pipe instead of in front of the first MFMA of the next K block.
// BROW_: the weight operand carries one scale per ROW and K block (b_s[n * bs_rs + kb * bs_cs], bs_bytes long) instead of
// one per 128x128 block: the scales of the tile's BN rows travel through LDS per K block like the activation scales
// (copied by the waves behind the activation-scale waves), a lane keeps the four scales of its four columns of every
// sub-tile, and the fold multiplies them in: 4 multiplies + 4 FMAs per MFMA instead of 4 FMAs.
template <int BM, int BN, int WGM, int WGN, int STAGES, typename OUT, int GAP_ = 0, int TD_ = 0, int ABL_ = 0, int FMT_ = 0,
          bool BROW_ = false>
__device__ __forceinline__ void fp8_gemm_tile(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, OUT* __restrict__ c,
    const uint16_t* __restrict__ bias, int m0, int m_end, int m_total, int n0, int N, int K, int ldc, const Duty duty,
    int kb0, int kb1, uint8_t* __restrict__ pool, int bs_rs = 0, int bs_cs = 0, uint32_t bs_bytes = 0) {
    // ABL_ switches parts of the K loop off for the timing probe (mdy_fp8_gemm_probe); the product uses 0.
    //   1: no global->LDS copies in the loop (the ring is filled once and replayed)   2: no LDS fragment / scale reads
    //   4: no FMA fold (the MFMAs accumulate in place, no block scales)                8: no pre-touches
    constexpr bool NO_COPY = (ABL_ & 1) != 0, NO_LDS = (ABL_ & 2) != 0, NO_FOLD = (ABL_ & 4) != 0;
    constexpr bool NO_TOUCH = (ABL_ & 8) != 0 || NO_COPY;
    constexpr int WAVES = WGM * WGN;
    constexpr int WM = BM / WGM, WN = BN / WGN, TI = WM / 16, TJ = WN / 16;
    constexpr int PASS_ROWS = WAVES * 8;  // rows copied by one DMA instruction of every wave
    constexpr int A_PASSES = BM / PASS_ROWS, B_PASSES = BN / PASS_ROWS;
    constexpr int S_WAVES = BM / 64;      // waves that also copy the activation scales
    constexpr int DEPTH = 4;              // MFMAs in flight before their results are folded
    static_assert(BM % PASS_ROWS == 0 && BN % PASS_ROWS == 0 && PASS_ROWS % 16 == 0, "tile/threads mismatch");
    // A wave's WN columns lie in one 128-column weight-scale block when WN divides 128 (tiles then start on multiples
    // of WN); the 192-wide tile (WN = 48, tiles start on multiples of 64) can straddle two: its 16-column sub-tiles never
    // do, so such a wave keeps two combined scales per row and each sub-tile takes the one of its block.
    constexpr bool STRADDLE = (128 % WN) != 0;
    static_assert(WN <= 128 && (!STRADDLE || BN == 192) && S_WAVES <= WAVES && WAVES >= 2, "weight-scale blocks per wave column");
    constexpr bool HOLD_A = TI <= TJ;
    constexpr int NH = HOLD_A ? TI : TJ, NS = HOLD_A ? TJ : TI;
    constexpr int NT = TI * TJ;
    constexpr int NDMA = 1 + A_PASSES + B_PASSES;       // copies per K block and wave: scales, A passes, B passes
    constexpr int TB = NT - NH;                         // slot of the barrier
    constexpr int NSLOT = NT + DEPTH;                   // slots of a K block (the last DEPTH hold FMAs only)
    // Copy j of a K block goes out in slot TB+1 + GAP*j, counted on from the barrier of the block two before it
    // and running over into the first slots of the next block.  With 8 waves one copy per slot and wave is
    // twice what the CU's address unit takes (64 lanes x 16 bytes = 16 clocks each, a slot is 64 clocks for
    // the two waves of a SIMD): the waves then queue on the copy instruction and their MFMAs behind it wait.
    // Measured: 256x256 tiles 1-5 % faster with every second slot; 128x256 and 128x192 tiles 2-7 % at 4096x1536x7168.
    constexpr int GAP = GAP_ > 0 ? GAP_ : (WAVES >= 8 && NT >= 12) ? 2 : 1;
    constexpr int TAIL = (NSLOT - TB - 1 + GAP - 1) / GAP;   // copies that still fit behind the barrier
    constexpr int FIRST = TAIL < NDMA ? TAIL : NDMA;         // copies of K block kb+2 issued in the tail of kb
    constexpr int TOUCH = FIRST < NDMA ? TB + 1 + GAP * (NDMA - 1) - NSLOT + 1 : 0;   // slot after the last copy
    constexpr int TD = TD_ > 0 ? TD_ : STAGES + 1;      // duty touches run this many K blocks ahead (in front of the copies)
    // loads younger than the last copy of K block kb+1 when the wave waits for it in K block kb: the copies of
    // blocks kb+2 .. kb+STAGES-1 and one touch per K block since (loads complete in order, so vmcnt(YOUNGER)
    // means "block kb+1 has landed")
    constexpr int YOUNGER = (STAGES - 2) * NDMA + STAGES - 1;
    static_assert(STAGES >= 2 && YOUNGER <= 63, "vmcnt is a 6-bit counter");
    static_assert(NS % 2 == 0 && NS >= 2, "the first streamed fragment of the next K block reuses queue slot 0");
    static_assert(TOUCH < TB, "not enough slots in front of the barrier");

    using L = TileLds<BM, BN, WAVES, STAGES>;
    constexpr int NBS = L::NBS;
    uint8_t(*lds_a)[BM * 128] = reinterpret_cast<uint8_t(*)[BM * 128]>(pool + L::a_off);     // [STAGES]
    uint8_t(*lds_b)[BN * 128] = reinterpret_cast<uint8_t(*)[BN * 128]>(pool + L::b_off);     // [STAGES]
    float(*lds_s)[BM] = reinterpret_cast<float(*)[BM]>(pool + L::s_off);                      // [STAGES]
    float(*lds_bs)[512] = reinterpret_cast<float(*)[512]>(pool + L::bs_off);                  // [NBS] weight scales, all K blocks
    uint8_t* lds_dummy = pool + L::dummy_off;                                                 // target of copies that must go nowhere

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int M = m_end;
    const int KB = K >> 7;

    // ---- DMA.  What depends on the tile: the descriptors (limited to the rows of the tile, so that the M and N
    // tails read 0), the rows whose scales a lane copies, and the share of the panels this workgroup pre-touches.
    struct TileAddr {
        intx4 ra, rb, rt;
        int s_voff, touch_off, n0;
    };
    const int prow = wave * 8 + (lane >> 3);                          // row inside a pass
    const int voff = prow * K + (((lane & 7) ^ swz(prow)) << 4);      // permuted chunk of that row
    // scale copies: waves 0 .. S_WAVES-1 copy 64 activation scales of the K block each; with BROW_ the next BN / 64 waves
    // copy 64 weight-row scales each (into the area that otherwise holds the weight's block scales); the rest copy nothing
    constexpr int SB_WAVES = BROW_ ? BN / 64 : 0;
    static_assert(S_WAVES + SB_WAVES <= WAVES && (!BROW_ || STAGES * BN * 4 <= L::NBS * 512 * 4), "waves / LDS for the weight-row scales");
    const bool sb_wave = BROW_ && wave >= S_WAVES && wave < S_WAVES + SB_WAVES;
    float* lds_sbr = reinterpret_cast<float*>(pool + L::bs_off);     // BROW_: [STAGES][BN] weight-row scales
    intx4 rs = sb_wave ? make_rsrc(b_s, bs_bytes) : make_rsrc(a_s, as_bytes);
    if (wave >= S_WAVES && !sb_wave) rs[2] = 0;                       // these waves copy no scales: always out of range
    const int sc_cs = sb_wave ? bs_cs : as_cs;
    const uint32_t sc_bytes = sb_wave ? bs_bytes : as_bytes;
    const uint32_t ld_base = lds_addr(&lds_dummy[0]) + wave * 512;
    const uint32_t la_base = lds_addr(&lds_a[0][0]) + wave * 1024;
    const uint32_t lb_base = lds_addr(&lds_b[0][0]) + wave * 1024;
    const uint32_t ls_base = wave < S_WAVES ? lds_addr(&lds_s[0][0]) + wave * 256
                             : sb_wave ? lds_addr(lds_sbr) + (wave - S_WAVES) * 256 : ld_base;
    const uint32_t ls_buf = wave < S_WAVES ? BM * 4 : sb_wave ? BN * 4 : 0;
    // duty touch: the even waves load one dword of every line of this workgroup's share of the B panel (64
    // rows per wave), the odd waves of the A panel, TD K blocks ahead, into the dummy area: the lines are in L2
    // when this workgroup and its neighbours copy them.  Waves beyond the share run the same instruction on an
    // empty descriptor.
    const bool touch_b = (wave & 1) == 0;
    const int t_idx = (wave >> 1) * 64 + lane;
    auto tile_addr = [&](int tm0, int tn0, const Duty& d) {
        TileAddr t;
        t.ra = make_rsrc(a + (size_t)tm0 * K, (uint32_t)min(BM, M - tm0) * (uint32_t)K);
        t.rb = make_rsrc(b + (size_t)tn0 * K, (uint32_t)min(BN, N - tn0) * (uint32_t)K);
        t.s_voff = sb_wave ? min(tn0 + (wave - S_WAVES) * 64 + lane, N - 1) * bs_rs * 4
                           : min(tm0 + (wave % S_WAVES) * 64 + lane, m_total - 1) * as_rs * 4;
        const int share = touch_b ? (BN >> d.b_sh) : (BM >> d.a_sh);      // rows of the share
        t.rt = touch_b ? t.rb : t.ra;
        // nobody to share with: touching one's own lines ahead of the copy only adds requests (measured)
        if ((wave >> 1) * 64 >= share || (touch_b ? d.b_sh : d.a_sh) == 0) t.rt[2] = 0;
        t.touch_off = ((touch_b ? d.b_duty : d.a_duty) * share + t_idx % share) * K;
        t.n0 = tn0;
        return t;
    };
    const TileAddr me = tile_addr(m0, n0, duty);

    // copy i (0: scales, then the A passes, then the B passes) of K block kb into buffer buf.  Past the last K
    // block the offsets run beyond the descriptors: no memory access, zeros into a buffer nobody reads any more.
    auto issue = [&](const TileAddr& t, int i, int kb, int buf) {
        const bool more = kb < kb1;
        if (i == 0)
            dma4(rs, t.s_voff, more ? kb * sc_cs * 4 : (int)sc_bytes, ls_base + buf * ls_buf);
        else if (i <= A_PASSES)
            dma16(t.ra, voff, (i - 1) * PASS_ROWS * K + (more ? kb * 128 : t.ra[2]), la_base + buf * (BM * 128) + (i - 1) * PASS_ROWS * 128);
        else
            dma16(t.rb, voff, (i - 1 - A_PASSES) * PASS_ROWS * K + (more ? kb * 128 : t.rb[2]),
                  lb_base + buf * (BN * 128) + (i - 1 - A_PASSES) * PASS_ROWS * 128);
    };
    auto touch = [&](const TileAddr& t, int kb) { dma4(t.rt, t.touch_off, kb < kb1 ? kb * 128 : t.rt[2], ld_base + 256); };
    // The start of a tile: its weight scales, then the copies in the order the K loop keeps up: for every K block its
    // first FIRST copies, the rest, one touch; K blocks 0 .. STAGES-2 whole and the first copies of block STAGES-1.
    auto prologue = [&](const TileAddr& t) {
        if (!BROW_ && wave < NBS) {
            const int nb = min((t.n0 >> 7) + wave, ((N + 127) >> 7) - 1);
            const intx4 rbs = make_rsrc(b_s + (size_t)nb * KB, (uint32_t)KB * 4u);
            for (int cc = 0; cc < KB; cc += 64) dma4(rbs, lane * 4, cc * 4, lds_addr(&lds_bs[wave][cc]));
        }
#pragma unroll
        for (int blk = 0; blk < STAGES - 1; ++blk) {
#pragma unroll
            for (int i = 0; i < NDMA; ++i) issue(t, i, kb0 + blk, blk);
            if (!NO_TOUCH) touch(t, kb0 + blk + 1 + TD - STAGES);
            else touch(t, 1 << 20);      // same load count for the waits below: a copy of nothing
        }
#pragma unroll
        for (int i = 0; i < FIRST; ++i) issue(t, i, kb0 + STAGES - 1, STAGES - 1);
        if (NO_COPY) {     // probe: the whole ring up front, nothing is copied later
#pragma unroll
            for (int i = FIRST; i < NDMA; ++i) issue(t, i, kb0 + STAGES - 1, STAGES - 1);
        }
    };

    // ---- fragment reads: lane -> row (lane%16) and the 32-byte K slice (lane/16) of a 16-row sub-tile
    const int frow = lane & 15, fk = lane >> 4;
    const int a_rd0 = (wm * WM + frow) * 128 + (((2 * fk) ^ swz(frow)) << 4);
    const int a_rd1 = (wm * WM + frow) * 128 + (((2 * fk + 1) ^ swz(frow)) << 4);
    const int b_rd0 = (wn * WN + frow) * 128 + (((2 * fk) ^ swz(frow)) << 4);
    const int b_rd1 = (wn * WN + frow) * 128 + (((2 * fk + 1) ^ swz(frow)) << 4);
    const int h0 = HOLD_A ? a_rd0 : b_rd0, h1 = HOLD_A ? a_rd1 : b_rd1;   // held operand
    const int x0 = HOLD_A ? b_rd0 : a_rd0, x1 = HOLD_A ? b_rd1 : a_rd1;   // streamed operand
    const int s_rd = wm * WM + frow;
    const int bs_col = (n0 & 127) + wn * WN;                        // first column of the wave inside the tile's first scale block
    const float* my_bs = lds_bs[bs_col >> 7];
    const float* my_bs_hi = lds_bs[(bs_col + WN - 1) >> 7];         // STRADDLE: the block of the wave's last columns
    const int jsplit = STRADDLE ? min(TJ, (128 - (bs_col & 127)) >> 4) : TJ;   // sub-tiles j < jsplit lie in the first block

    floatx4 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    auto read_frag = [&](const uint8_t* base, int rd0, int rd1, int idx) {
        const intx4 lo = *reinterpret_cast<const intx4*>(base + rd0 + idx * 2048);
        const intx4 hi = *reinterpret_cast<const intx4*>(base + rd1 + idx * 2048);
        return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    // ---- prologue, wait for block 0, load the registers of step 0
    prologue(me);
    if (NO_COPY) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * (NDMA + 1) + 1 + FIRST) : "memory");
    __syncthreads();
    intx8 fh[NH], fx[2];
    float sc[TI], sc_hi[STRADDLE ? TI : 1];
    floatx4 sbv[BROW_ ? TJ : 1];                 // BROW_: the weight-row scales of this lane's four columns of every sub-tile
    const float* sbr_lane = lds_sbr + wn * WN + 4 * fk;
    if (BROW_) {
#pragma unroll
        for (int j = 0; j < TJ; ++j) sbv[j] = *reinterpret_cast<const floatx4*>(sbr_lane + j * 16);
    }
#pragma unroll
    for (int h = 0; h < NH; ++h) fh[h] = read_frag(HOLD_A ? lds_a[0] : lds_b[0], h0, h1, h);
    {
        const float sb = BROW_ ? 1.0f : my_bs[kb0], sb_hi = BROW_ ? 1.0f : my_bs_hi[kb0];
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const float sa = lds_s[0][s_rd + i * 16];
            sc[i] = sa * sb;
            if (STRADDLE) sc_hi[i] = sa * sb_hi;
        }
    }
    fx[0] = read_frag(HOLD_A ? lds_b[0] : lds_a[0], x0, x1, 0);

    int cur = 0;                                             // buffer of K block kb: kb % STAGES
    for (int kb = kb0; kb < kb1; ++kb) {
        const int nxt = cur + 1 == STAGES ? 0 : cur + 1;     // buffer of K block kb+1
        const int last = cur == 0 ? STAGES - 1 : cur - 1;    // buffer of K block kb+STAGES-1
        const uint8_t* lx = HOLD_A ? lds_b[cur] : lds_a[cur];            // streamed operand of this K block
        const uint8_t* lh_n = HOLD_A ? lds_a[nxt] : lds_b[nxt];          // operands and scales of the next one
        const uint8_t* lx_n = HOLD_A ? lds_b[nxt] : lds_a[nxt];
        const float* ls_n = lds_s[nxt];
        float sc_n[TI], sc_hi_n[STRADDLE ? TI : 1];
        floatx4 sbv_n[BROW_ ? TJ : 1];
        floatx4 p[DEPTH + 1];
#pragma unroll
        for (int t = 0; t < NT + DEPTH; ++t) {
            if (t < NT) {
                const int si = t / NH, h = t % NH;
                if (h == 0 && si + 1 < NS) {
                    if (!NO_LDS) fx[(si + 1) & 1] = read_frag(lx, x0, x1, si + 1);
                    else asm volatile("" : "+v"(fx[(si + 1) & 1]));      // probe: keep the operand opaque to the optimizer
                }
                const intx8 fa_ = HOLD_A ? fh[h] : fx[si & 1];
                const intx8 fb_ = HOLD_A ? fx[si & 1] : fh[h];
                if (!NO_FOLD) {
                    p[t % (DEPTH + 1)] = mfma_block<FMT_>(fb_, fa_);
                } else {
                    floatx4& d = acc[HOLD_A ? h : si][HOLD_A ? si : h];
                    d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb_, fa_, d, FMT_, FMT_, 0, 0, 0, 0);
                }
                if (t == TB) {
                    // K block kb+1 has landed once only the younger loads are left in flight
                    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(YOUNGER) : "memory");
                    __syncthreads();
                    if (!NO_LDS) {
                        fx[0] = read_frag(lx_n, x0, x1, 0);      // queue slot 0 was last used by streamed fragment NS-2
                        const float sb = BROW_ ? 1.0f : my_bs[min(kb + 1, KB - 1)], sb_hi = BROW_ ? 1.0f : my_bs_hi[min(kb + 1, KB - 1)];
                        if (BROW_) {
#pragma unroll
                            for (int j = 0; j < TJ; ++j) sbv_n[j] = *reinterpret_cast<const floatx4*>(sbr_lane + nxt * BN + j * 16);
                        }
#pragma unroll
                        for (int i = 0; i < TI; ++i) {
                            const float sa = ls_n[s_rd + i * 16];
                            sc_n[i] = sa * sb;
                            if (STRADDLE) sc_hi_n[i] = sa * sb_hi;
                        }
                    } else {
                        asm volatile("" : "+v"(fx[0]));
#pragma unroll
                        for (int i = 0; i < TI; ++i) {
                            sc_n[i] = sc[i];
                            if (STRADDLE) sc_hi_n[i] = sc_hi[i];
                        }
                    }
                }
                if (t >= TB) {
                    if (!NO_LDS) fh[h] = read_frag(lh_n, h0, h1, h);   // fh[h] had its last use just above
                    else asm volatile("" : "+v"(fh[h]));
                }
            }
            if (t >= DEPTH && !NO_FOLD) {
                const int u = t - DEPTH, si = u / NH, h = u % NH;
                const int i = HOLD_A ? h : si, j = HOLD_A ? si : h;
                const floatx4 q = p[u % (DEPTH + 1)];
                if (BROW_) {
                    acc[i][j][0] = __builtin_fmaf(q[0], sc[i] * sbv[j][0], acc[i][j][0]);
                    acc[i][j][1] = __builtin_fmaf(q[1], sc[i] * sbv[j][1], acc[i][j][1]);
                    acc[i][j][2] = __builtin_fmaf(q[2], sc[i] * sbv[j][2], acc[i][j][2]);
                    acc[i][j][3] = __builtin_fmaf(q[3], sc[i] * sbv[j][3], acc[i][j][3]);
                } else {
                    fold(acc[i][j], q, (STRADDLE && j >= jsplit) ? sc_hi[i] : sc[i]);
                }
            }
            if (!NO_COPY) {
#pragma unroll
                for (int j = 0; j < NDMA; ++j) {
                    const int v = TB + 1 + GAP * j;
                    if (v < NSLOT && v == t) issue(me, j, kb + STAGES, cur);                    // behind the barrier: buffer cur is free
                    if (v >= NSLOT && v - NSLOT == t) issue(me, j, kb + STAGES - 1, last);      // the rest of the block started in kb-1
                }
            }
            if (t == TOUCH && !NO_TOUCH) touch(me, kb + TD);
            __builtin_amdgcn_sched_barrier(0);  // keep the MFMA / FMA / ds_read / copy interleaving as written
        }
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            sc[i] = sc_n[i];
            if (STRADDLE) sc_hi[i] = sc_hi_n[i];
        }
        if (BROW_) {
#pragma unroll
            for (int j = 0; j < TJ; ++j) sbv[j] = sbv_n[j];
        }
        cur = nxt;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing may still be writing LDS when the wave ends

    // ---- epilogue: lane holds c[m][n..n+3], m = .. + lane%16, n = .. + 4*(lane/16)
    const bool vec_ok = (ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const int m = m0 + wm * WM + i * 16 + frow;
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const int n = n0 + wn * WN + j * 16 + 4 * fk;
            float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
            if (bias != nullptr) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) v[e] += bf16_one(bias[n + e]);
            }
            store4<OUT>(c, ldc, m, n, M, N, v, vec_ok);
        }
    }
}

// Tile order shared by the kernels below: consecutive workgroup ids land on different XCDs (8 of
// them); give each XCD a contiguous run of tiles, walked in groups of 4 tile rows.
__device__ __forceinline__ int xcd_contiguous(int pid, int ntiles) {
    return (ntiles % 8 == 0) ? (pid & 7) * (ntiles >> 3) + (pid >> 3) : pid;
}
// GM: tile rows per group; the 32 workgroups that an XCD runs at a time then cover a GM x (32 / GM) block of tiles
// (4 x 8 in the product; the probe library also builds 2 x 16 and 8 x 4 to measure their fabric traffic and energy).
template <int GM = 4>
__device__ __forceinline__ Duty tile_of(int local, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int group = local / (GM * tiles_n);
    const int first_m = group * GM;
    const int gsz = min(tiles_m - first_m, GM);
    const int in_group = (local % (GM * tiles_n)) % gsz;
    tm = first_m + in_group;
    tn = (local % (GM * tiles_n)) / gsz;
    // the workgroups of an XCD run a gsz x (up to 32 / GM) block of tiles at a time
    Duty d;
    d.b_sh = gsz >= 8 ? 3 : gsz >= 4 ? 2 : gsz >= 2 ? 1 : 0;
    constexpr int COLS = 32 / GM;
    d.a_sh = (tiles_n >= 16 && COLS >= 16) ? 4 : (tiles_n >= 8 && COLS >= 8) ? 3 : (tiles_n >= 4 && COLS >= 4) ? 2 : tiles_n >= 2 ? 1 : 0;
    d.b_duty = in_group & ((1 << d.b_sh) - 1);
    d.a_duty = tn & ((1 << d.a_sh) - 1);
    return d;
}

// The tile with SPECIALIZED waves and the barrier of a K block EARLY in the block, for small wave tiles.
// In fp8_gemm_tile every wave copies, reads fragments, issues MFMAs and folds, and the one barrier of a K block sits in
// front of its last streamed fragment: behind it every wave reloads the held fragments, the first streamed fragment and the
// scales of the next block from LDS with only NH MFMAs left to cover that latency, and every buffer_load ... lds stays at
// the head of its (in-order) wave until the CU's address unit takes it, holding back the MFMAs queued behind it.  With a
// 256x256 tile both are a small part of a K block; with 64x96 wave tiles on a 128x192 tile, in-kernel clocks at
// 4096x1536x7168 showed 560-730 of ~1700 clocks per K block behind the barrier for 4 of 12 MFMAs, 40 clocks per MFMA slot
// without a copy near it and 60 with one every second slot.  Here:
//   * the first WGM x WGN waves ("consumers") run the MFMAs, the LDS reads and the fold and never touch global memory in the
//     K loop; PW further waves ("producers") do nothing but the global->LDS copies and the pre-touches (small wave tiles
//     leave registers for the second set of waves: all waves of a workgroup get the same allocation);
//   * the barrier of block kb is at slot E, a few MFMAs into the block.  For a consumer it says "I have left block kb-1";
//     a producer first waits for its own copies of block kb+1.  Behind it the consumers read block kb+1's held fragments,
//     first streamed fragment and scales from LDS into a SECOND set of registers, spread over the slots (block kb+1 then
//     starts on registers loaded a dozen slots earlier; the K loop is unrolled by two so that the sets swap without
//     moves), and the producers copy block kb+STAGES-1 and touch the lines of a later block;
//   * the held operand of block kb is read during block kb-1, the streamed operand during block kb itself: the held
//     operand's buffer is free one block earlier, so its ring is one buffer shorter (STAGES-1) than the streamed operand's
//     (STAGES) for the same STAGES-2 blocks in flight.  The activation scales follow the held operand;
//   * on the 192-wide tile a wave's columns can straddle two 128-column blocks of weight scales: the combined scale is
//     kept per row and 32-column group (multiplies once per block instead of a select per MFMA).
// Swizzle, fragment layout, fold, epilogue and pre-touch shares are fp8_gemm_tile's.
template <int BM, int BN, int WGM, int WGN, int PW, int STAGES, typename OUT, int FMT_ = 0, int E_ = 2>
__device__ __forceinline__ void fp8_gemm_tile_ws(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, OUT* __restrict__ c,
    const uint16_t* __restrict__ bias, int m0, int m_end, int m_total, int n0, int N, int K, int ldc, const Duty duty,
    int kb0, int kb1, uint8_t* __restrict__ pool) {
    constexpr int CW = WGM * WGN;                       // consumer waves
    constexpr int WM = BM / WGM, WN = BN / WGN, TI = WM / 16, TJ = WN / 16;
    constexpr int PASS_ROWS = PW * 8;                   // rows copied by one instruction of every producer
    constexpr int A_PASSES = BM / PASS_ROWS, B_PASSES = BN / PASS_ROWS;
    constexpr int S_WAVES = BM / 64;                    // producers that also copy the activation scales
    constexpr int DEPTH = 4;
    static_assert(BM % PASS_ROWS == 0 && BN % PASS_ROWS == 0 && PASS_ROWS % 16 == 0, "tile/threads mismatch");
    constexpr bool STRADDLE = (128 % WN) != 0;
    static_assert(WN <= 128 && (!STRADDLE || BN == 192) && S_WAVES <= PW && PW >= 2, "weight-scale blocks per wave column");
    constexpr bool HOLD_A = TI <= TJ;
    constexpr int NH = HOLD_A ? TI : TJ, NS = HOLD_A ? TJ : TI;
    constexpr int NT = TI * TJ;
    constexpr int SC = 1;                               // scale copies per K block and producer
    constexpr int NDMA = SC + A_PASSES + B_PASSES;
    constexpr int E = E_;
    constexpr int TDA = 2;
    static_assert(STAGES >= 4 && (STAGES - 2) * (NDMA + 1) + 1 <= 63, "streamed ring of at least 4 K blocks; vmcnt is a 6-bit counter");
    constexpr int SA = HOLD_A ? STAGES - 1 : STAGES, SB = HOLD_A ? STAGES : STAGES - 1;   // ring depths of a and b
    constexpr int SS = STAGES - 1;                                                        // ring depth of the activation scales
    // loads younger than the last copy of block kb+1 at the barrier of block kb: the touch behind those copies and the
    // copies + touches of blocks kb+2 .. kb+STAGES-2
    constexpr int YOUNGER = (STAGES - 3) * (NDMA + 1) + 1;
    static_assert(NS % 2 == 0 && NS >= 2, "the first streamed fragment of the next K block reuses queue slot 0");
    constexpr int PWIN = NT - 2 - (E + 1);
    static_assert(E >= 0 && E < NT - NH && PWIN >= NH, "barrier slot");

    using L = TileLdsWs<BM, BN, CW + PW, SA, SB, SS>;
    constexpr int NBS = L::NBS;
    uint8_t(*lds_a)[BM * 128] = reinterpret_cast<uint8_t(*)[BM * 128]>(pool + L::a_off);
    uint8_t(*lds_b)[BN * 128] = reinterpret_cast<uint8_t(*)[BN * 128]>(pool + L::b_off);
    float(*lds_s)[BM] = reinterpret_cast<float(*)[BM]>(pool + L::s_off);
    float(*lds_bs)[L::BSROW] = reinterpret_cast<float(*)[L::BSROW]>(pool + L::bs_off);
    uint8_t* lds_dummy = pool + L::dummy_off;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = m_end;
    const int KB = K >> 7;

    if (wave >= CW) {
        // ------------------------------------------------------------------ producer
        const int pw = wave - CW;
        const int prow = pw * 8 + (lane >> 3);
        const int voff = prow * K + (((lane & 7) ^ swz(prow)) << 4);
        intx4 rs = make_rsrc(a_s, as_bytes);
        if (pw >= S_WAVES) rs[2] = 0;
        const uint32_t ld_base = lds_addr(&lds_dummy[0]) + wave * 512;
        const uint32_t la_base = lds_addr(&lds_a[0][0]) + pw * 1024;
        const uint32_t lb_base = lds_addr(&lds_b[0][0]) + pw * 1024;
        const uint32_t ls_base = pw < S_WAVES ? lds_addr(&lds_s[0][0]) + pw * 256 : ld_base;
        const uint32_t ls_buf = pw < S_WAVES ? BM * 4 : 0;
        const intx4 ra = make_rsrc(a + (size_t)m0 * K, (uint32_t)min(BM, M - m0) * (uint32_t)K);
        const intx4 rb = make_rsrc(b + (size_t)n0 * K, (uint32_t)min(BN, N - n0) * (uint32_t)K);
        const int s_voff = min(m0 + (pw % S_WAVES) * 64 + lane, m_total - 1) * as_rs * 4;
        const bool touch_b = (pw & 1) == 0;
        const int t_idx = (pw >> 1) * 64 + lane;
        const int share = touch_b ? (BN >> duty.b_sh) : (BM >> duty.a_sh);
        intx4 rt = touch_b ? rb : ra;
        if ((touch_b ? duty.b_sh : duty.a_sh) == 0) rt[2] = 0;
        const int touch_row0 = (touch_b ? duty.b_duty : duty.a_duty) * share;
        constexpr int TOUCH_LANES = (PW / 2) * 64;
        auto issue = [&](int i, int kb, int bufa, int bufb, int bufs) {
            const bool more = kb < kb1;
            if (i < SC)
                dma4(rs, s_voff, more ? kb * as_cs * 4 : (int)as_bytes, ls_base + bufs * ls_buf);
            else if (i < SC + A_PASSES)
                dma16(ra, voff, (i - SC) * PASS_ROWS * K + (more ? kb * 128 : ra[2]), la_base + bufa * (BM * 128) + (i - SC) * PASS_ROWS * 128);
            else
                dma16(rb, voff, (i - SC - A_PASSES) * PASS_ROWS * K + (more ? kb * 128 : rb[2]),
                      lb_base + bufb * (BN * 128) + (i - SC - A_PASSES) * PASS_ROWS * 128);
        };
        auto touch = [&](int kbp) {      // kTouchBurst consecutive lines of a row at a time (see kTouchBurst)
            const int j = kbp & (kTouchBurst - 1), base = kbp - j;
            const int q = j * TOUCH_LANES + t_idx, row = q >> kTouchBurstLog, line = q & (kTouchBurst - 1);
            const bool ok = row < share && base + line < kb1;
            dma4(rt, ok ? (touch_row0 + row) * K + (base + line) * 128 : kOutOfRange, 0, ld_base + 256);
        };

        if (pw < NBS) {
            const int nb = min((n0 >> 7) + pw, ((N + 127) >> 7) - 1);
            const intx4 rbs = make_rsrc(b_s + (size_t)nb * KB, (uint32_t)KB * 4u);
            for (int cc = 0; cc < KB; cc += 64) dma4(rbs, lane * 4, cc * 4, lds_addr(&lds_bs[pw][cc]));
        }
#pragma unroll
        for (int blk = 0; blk < STAGES - 1; ++blk) {
#pragma unroll
            for (int i = 0; i < NDMA; ++i) issue(i, kb0 + blk, blk % SA, blk % SB, blk % SS);
            touch(kb0 + blk);                  // groups 0 .. STAGES-2 of the first burst
        }
        // the loop's first touch is of block kb0 + STAGES - 1 + TDA: the blocks in between are touched here, behind the copies,
        // so that the waits below only wait for more than they need (4096x1536x7168 after a cache flush 57.4 -> 56.1 us,
        // 2048x2048x7168 44.0 -> 43.0 us, 2048x1024x7168 34.6 -> 33.5 us)
#pragma unroll
        for (int t = 0; t < TDA; ++t) touch(kb0 + STAGES - 1 + t);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * (NDMA + 1) + 1) : "memory");    // block kb0 has landed
        __syncthreads();
        // buffers of block kb+STAGES-1 in the three rings (kb = kb0: block index STAGES-1)
        int fa = (STAGES - 1) % SA, fb = (STAGES - 1) % SB, fs = (STAGES - 1) % SS;
        for (int kb = kb0; kb < kb1; ++kb) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(YOUNGER) : "memory");   // this wave's copies of block kb+1 have landed
            __syncthreads();                                                   // every consumer has left block kb-1
#pragma unroll
            for (int i = 0; i < NDMA; ++i) issue(i, kb + STAGES - 1, fa, fb, fs);
            touch(kb + STAGES - 1 + TDA);
            fa = fa + 1 == SA ? 0 : fa + 1;
            fb = fb + 1 == SB ? 0 : fb + 1;
            fs = fs + 1 == SS ? 0 : fs + 1;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing may still be writing LDS when the wave ends
        return;
    }

    // ---------------------------------------------------------------------- consumer
    const int wm = wave / WGN, wn = wave % WGN;
    const int frow = lane & 15, fk = lane >> 4;
    const int a_rd0 = (wm * WM + frow) * 128 + (((2 * fk) ^ swz(frow)) << 4);
    const int a_rd1 = (wm * WM + frow) * 128 + (((2 * fk + 1) ^ swz(frow)) << 4);
    const int b_rd0 = (wn * WN + frow) * 128 + (((2 * fk) ^ swz(frow)) << 4);
    const int b_rd1 = (wn * WN + frow) * 128 + (((2 * fk + 1) ^ swz(frow)) << 4);
    const int h0 = HOLD_A ? a_rd0 : b_rd0, h1 = HOLD_A ? a_rd1 : b_rd1;
    const int x0 = HOLD_A ? b_rd0 : a_rd0, x1 = HOLD_A ? b_rd1 : a_rd1;
    const int s_rd = wm * WM + frow;
    const int bs_col = (n0 & 127) + wn * WN;
    // A wave's columns lie in one 128-column block of weight scales, except on the 192-wide tile (WN = 96 or 48): there
    // every group of GW columns does (GW = 32 or 16 divides the possible offsets), so the combined scale is kept per row
    // and column group: NG multiplies per row and K block instead of one select per MFMA.
    constexpr int GW = STRADDLE ? ((WN % 32 == 0) ? 32 : 16) : WN, NG = WN / GW, JPG = GW / 16;
    const float* my_bs[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) my_bs[g] = lds_bs[(bs_col + g * GW) >> 7];

    floatx4 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    auto read_frag = [&](const uint8_t* base, int rd0, int rd1, int idx) {
        const intx4 lo = *reinterpret_cast<const intx4*>(base + rd0 + idx * 2048);
        const intx4 hi = *reinterpret_cast<const intx4*>(base + rd1 + idx * 2048);
        return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    __syncthreads();                                     // block kb0, the weight scales have landed
    intx8 fh_a[NH], fh_b[NH], fx[2];
    float sc_a[TI][NG], sc_b[TI][NG];
#pragma unroll
    for (int h = 0; h < NH; ++h) fh_a[h] = read_frag(HOLD_A ? lds_a[0] : lds_b[0], h0, h1, h);
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const float sa = lds_s[0][s_rd + i * 16];
#pragma unroll
        for (int g = 0; g < NG; ++g) sc_a[i][g] = sa * my_bs[g][kb0];
    }
    fx[0] = read_frag(HOLD_A ? lds_b[0] : lds_a[0], x0, x1, 0);

    // buffers of K block kb in the ring of the held operand (and of the scales) / of the streamed operand
    int ch = 0, cx = 0;
    auto block = [&](intx8(&fh)[NH], intx8(&fhn)[NH], float(&sc)[TI][NG], float(&scn)[TI][NG], int kb) {
        const int nh = ch + 1 == STAGES - 1 ? 0 : ch + 1;     // block kb+1, held ring
        const int nx = cx + 1 == STAGES ? 0 : cx + 1;         // block kb+1, streamed ring
        const uint8_t* lx = HOLD_A ? lds_b[cx] : lds_a[cx];
        const uint8_t* lh_n = HOLD_A ? lds_a[nh] : lds_b[nh];
        const uint8_t* lx_n = HOLD_A ? lds_b[nx] : lds_a[nx];
        const float* ls_n = lds_s[nh];
        floatx4 p[DEPTH + 1];
#pragma unroll
        for (int t = 0; t < NT + DEPTH; ++t) {
            if (t < NT) {
                const int si = t / NH, h = t % NH;
                if (h == 0 && si + 1 < NS) fx[(si + 1) & 1] = read_frag(lx, x0, x1, si + 1);
                if (h == 0 && si + 1 == NS) fx[0] = read_frag(lx_n, x0, x1, 0);      // first streamed fragment of block kb+1
                const intx8 fa_ = HOLD_A ? fh[h] : fx[si & 1];
                const intx8 fb_ = HOLD_A ? fx[si & 1] : fh[h];
                p[t % (DEPTH + 1)] = mfma_block<FMT_>(fb_, fa_);
                if (t == E) __syncthreads();
                if (t == E + 1) {
                    float sbg[NG];
#pragma unroll
                    for (int g = 0; g < NG; ++g) sbg[g] = my_bs[g][min(kb + 1, KB - 1)];
#pragma unroll
                    for (int i = 0; i < TI; ++i) {
                        const float sa = ls_n[s_rd + i * 16];
#pragma unroll
                        for (int g = 0; g < NG; ++g) scn[i][g] = sa * sbg[g];
                    }
                }
#pragma unroll
                for (int hh = 0; hh < NH; ++hh)
                    if (t == E + 1 + (hh * PWIN) / NH) fhn[hh] = read_frag(lh_n, h0, h1, hh);
            }
            if (t >= DEPTH) {
                const int u = t - DEPTH, si = u / NH, h = u % NH;
                const int i = HOLD_A ? h : si, j = HOLD_A ? si : h;
                fold(acc[i][j], p[u % (DEPTH + 1)], sc[i][j / JPG]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        ch = nh;
        cx = nx;
    };
    {
        int kb = kb0;
        for (; kb + 1 < kb1; kb += 2) {
            block(fh_a, fh_b, sc_a, sc_b, kb);
            block(fh_b, fh_a, sc_b, sc_a, kb + 1);
        }
        if (kb < kb1) block(fh_a, fh_b, sc_a, sc_b, kb);     // odd number of K blocks
    }

    const bool vec_ok = (ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const int m = m0 + wm * WM + i * 16 + frow;
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const int n = n0 + wn * WN + j * 16 + 4 * fk;
            float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
            if (bias != nullptr) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) v[e] += bf16_one(bias[n + e]);
            }
            store4<OUT>(c, ldc, m, n, M, N, v, vec_ok);
        }
    }
}

// the wave-specialized tile as a kernel: one workgroup of WGM*WGN + PW waves per tile (or per several, walked in turn)
template <int BM, int BN, int WGM, int WGN, int PW, int STAGES, typename OUT, int FMT_ = 0, int E_ = 2>
__global__ __launch_bounds__((WGM * WGN + PW) * 64) void fp8_gemm_ws_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, OUT* __restrict__ c,
    const uint16_t* __restrict__ bias, int M, int N, int K, int ldc, int tiles_m, int tiles_n, int pretouch) {
    constexpr bool HOLD_A = BM / WGM <= BN / WGN;
    __shared__ __attribute__((aligned(1024)))
    uint8_t pool[TileLdsWs<BM, BN, WGM * WGN + PW, HOLD_A ? STAGES - 1 : STAGES, HOLD_A ? STAGES : STAGES - 1, STAGES - 1>::bytes];
    const int ntiles = tiles_m * tiles_n;
    for (int pid = blockIdx.x; pid < ntiles; pid += gridDim.x) {
        int tm, tn;
        Duty duty = tile_of(xcd_contiguous(pid, ntiles), tiles_m, tiles_n, tm, tn);
        if (!pretouch) duty.a_sh = duty.b_sh = 0;
        fp8_gemm_tile_ws<BM, BN, WGM, WGN, PW, STAGES, OUT, FMT_, E_>(a, a_s, as_rs, as_cs, as_bytes, b, b_s, c, bias, tm * BM, M, M,
                                                                            tn * BN, N, K, ldc, duty, 0, K >> 7, pool);
        __syncthreads();
    }
}

template <int BM, int BN, int WGM, int WGN, int STAGES, typename OUT, int GAP_ = 0, int TD_ = 0, int ABL_ = 0, int FMT_ = 0, int GM_ = 4>
__global__ __launch_bounds__(WGM* WGN * 64) void fp8_gemm_mfma_kernel(
    const uint8_t* __restrict__ a, const float* __restrict__ a_s, int as_rs, int as_cs, uint32_t as_bytes,
    const uint8_t* __restrict__ b, const float* __restrict__ b_s, OUT* __restrict__ c,
    const uint16_t* __restrict__ bias, int M, int N, int K, int ldc, int tiles_m, int tiles_n, int pretouch) {
    // The grid may be smaller than the number of tiles (one workgroup per CU for the 256x256 tile): a workgroup
    // then walks tiles blockIdx.x, blockIdx.x + gridDim.x, ... itself, which saves the ~4.5 us that pass between
    // the end of a workgroup and the start of its successor on the same CU.  Workgroup ids keep their XCD
    // (id % 8) from tile to tile when gridDim.x is a multiple of 8.
    __shared__ __attribute__((aligned(1024))) uint8_t pool[TileLds<BM, BN, WGM * WGN, STAGES>::bytes];
    const int ntiles = tiles_m * tiles_n;
    for (int pid = blockIdx.x; pid < ntiles; pid += gridDim.x) {
        int tm, tn;
        Duty duty = tile_of<GM_>(xcd_contiguous(pid, ntiles), tiles_m, tiles_n, tm, tn);
        if (!pretouch) duty.a_sh = duty.b_sh = 0;
        fp8_gemm_tile<BM, BN, WGM, WGN, STAGES, OUT, GAP_, TD_, ABL_, FMT_>(a, a_s, as_rs, as_cs, as_bytes, b, b_s, c, bias, tm * BM, M,
                                                                            M, tn * BN, N, K, ldc, duty, 0, K >> 7, pool);
        __syncthreads();   // every wave has left the tile's LDS buffers before the next tile's copies land in them
    }
}

}  // namespace mdy
