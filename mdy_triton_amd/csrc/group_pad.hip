// Row padding / unpadding of grouped (mixture-of-experts) activations.
//
// The rows of x are G consecutive groups of m_splits[g] rows; padding copies group g to a slot of
// pad(m_splits[g]) rows (the next multiple of `multiple`) and fills the slot's remaining rows with zeros,
// unpadding copies the first m_splits[g] rows of every slot back.  Restates what Fp8Padding / Fp8Unpadding
// (/root/reference/triton_kernels/megatron_patchs/dpsk_grouped_linear.py:690-902) do with TransformerEngine's
// multi_padding_fused and with torch.split / torch.cat: the padded layout is what the grouped quantizer with
// the transposed copy needs (group sizes that are multiples of 256,
// /root/reference/triton_kernels/megatron_patchs/fp8_matmul.py:227).
//
// One launch per 128 groups: the table of first rows (unpadded and padded) travels as a kernel
// argument and a wave finds the group of its destination row by binary search.  Streaming copy, 16 bytes per
// lane, non-temporal (every byte is touched once).
#include "common.h"

namespace mdy {

constexpr int kPadGroups = 128;     // the table is a kernel argument: 3 KB of the 4 KB a launch may carry
struct PadTable {
    int n_groups;
    int64_t src_start[kPadGroups + 1];   // first row of group g in the source (its [n_groups] = all source rows)
    int64_t dst_start[kPadGroups + 1];   // first row of group g in the destination
    int64_t rows[kPadGroups];            // rows of group g that hold data (the smaller of its two slot sizes)
};

// grid.x: chunks of 64 lanes x 16 bytes of a row, grid.y/z: destination rows (block_row()), 4 rows per block
template <int VEC>
__global__ __launch_bounds__(256) void group_pad_kernel(const uint8_t* __restrict__ x, uint8_t* __restrict__ y,
                                                         int64_t row_bytes, int64_t dst_rows, const PadTable tbl) {
    const int64_t row = (int64_t)block_row() * 4 + (threadIdx.x >> 6);
    const int64_t col = ((int64_t)blockIdx.x * 64 + (threadIdx.x & 63)) * VEC;
    if (row >= dst_rows || col >= row_bytes) return;
    int lo = 0, hi = tbl.n_groups - 1;     // last group whose destination slot starts at or before this row
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (tbl.dst_start[mid] <= row) lo = mid; else hi = mid - 1;
    }
    const int64_t r = row - tbl.dst_start[lo];
    const bool data = r < tbl.rows[lo];
    const uint8_t* src = x + (tbl.src_start[lo] + r) * row_bytes + col;
    uint8_t* dst = y + row * row_bytes + col;
    if (VEC == 16) {
        store_nt16(dst, data ? load_nt16(src) : make_uint4(0u, 0u, 0u, 0u));
    } else if (VEC == 2) {
        *reinterpret_cast<uint16_t*>(dst) = data ? *reinterpret_cast<const uint16_t*>(src) : (uint16_t)0;
    } else {
        *dst = data ? *src : (uint8_t)0;
    }
}

// unpad == 0: x [sum m, row_bytes] -> y [sum pad(m), row_bytes]; unpad != 0: the reverse.
int launch_group_pad(const void* x, void* y, const int64_t* m_splits, int64_t G, int64_t row_bytes, int64_t multiple,
                     int unpad, hipStream_t stream) {
    const bool a16 = row_bytes % 16 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    const bool a2 = row_bytes % 2 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 1) == 0;
    const int vec = a16 ? 16 : a2 ? 2 : 1;
    int64_t src_row = 0, dst_row = 0;
    for (int64_t g0 = 0; g0 < G; g0 += kPadGroups) {
        PadTable tbl;
        const int n = (int)(G - g0 < kPadGroups ? G - g0 : kPadGroups);
        tbl.n_groups = n;
        const int64_t src0 = src_row, dst0 = dst_row;
        for (int g = 0; g < n; ++g) {
            const int64_t m = m_splits[g0 + g], pm = (m + multiple - 1) / multiple * multiple;
            tbl.src_start[g] = src_row - src0;
            tbl.dst_start[g] = dst_row - dst0;
            tbl.rows[g] = m;
            src_row += unpad ? pm : m;
            dst_row += unpad ? m : pm;
        }
        for (int g = n; g <= kPadGroups; ++g) {
            tbl.src_start[g] = src_row - src0;
            tbl.dst_start[g] = dst_row - dst0;
            if (g < kPadGroups) tbl.rows[g] = 0;
        }
        const int64_t rows = dst_row - dst0;
        if (rows == 0 || row_bytes == 0) continue;
        dim3 grid;
        if (!grid_rows((row_bytes + 64 * vec - 1) / (64 * vec), (rows + 3) / 4, grid)) return kErrTooManyBlocks;
        const uint8_t* xp = static_cast<const uint8_t*>(x) + src0 * row_bytes;
        uint8_t* yp = static_cast<uint8_t*>(y) + dst0 * row_bytes;
        if (vec == 16) hipLaunchKernelGGL(group_pad_kernel<16>, grid, dim3(256), 0, stream, xp, yp, row_bytes, rows, tbl);
        else if (vec == 2) hipLaunchKernelGGL(group_pad_kernel<2>, grid, dim3(256), 0, stream, xp, yp, row_bytes, rows, tbl);
        else hipLaunchKernelGGL(group_pad_kernel<1>, grid, dim3(256), 0, stream, xp, yp, row_bytes, rows, tbl);
        const int rc = (int)hipGetLastError();
        if (rc != 0) return rc;
    }
    return 0;
}

}  // namespace mdy
