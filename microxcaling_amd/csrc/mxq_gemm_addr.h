// Address arithmetic of the tile copies of the two GEMM kernels (mxq_gemm.h), kept apart from the
// kernels so that it compiles for the host as well: tests/cpp/gemm_addr_check.cpp walks every
// (workgroup, tile, K step, load, wave, lane) of a set of shapes through these same functions and
// checks that each byte range read lies inside the operand it belongs to.
//
// Layout of an operand: codes (batch, rows, kbytes) uint8, row-major; scales (batch, rows, KB) uint8
// with KB = K / 32.  A "K step" is GEMM_BK = 128 bytes of codes per row: 128 elements as 8-bit codes,
// 256 as e2m1 nibbles (EPB = elements per byte = 1 or 2), i.e. 4 * EPB scale bytes per row.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MXQ_ADDR_FN __host__ __device__ __forceinline__
#else
#define MXQ_ADDR_FN inline
#endif

namespace mxq_addr {

constexpr int BK = 128;          // bytes of codes per row and K step

MXQ_ADDR_FN int imin(int a, int b) { return a < b ? a : b; }

// Which output tile a workgroup computes.  Workgroups are dealt round-robin to the 8 XCDs, each
// with its own L2, so workgroup w runs on XCD w % 8.  Give every XCD a contiguous range of
// "logical" tile numbers, and walk the tile grid in bands of 8 tile-rows: the ~32 tiles an XCD
// works on at any time then form an 8 x 4 patch that shares 8 A tiles and 4 B tiles per K step
// through that XCD's L2 instead of streaming 64 tiles from the fabric.
MXQ_ADDR_FN void tile_of_workgroup(int wg, int total, int tiles_m, int tiles_n, int* tm, int* tn) {
    constexpr int XCDS = 8, BAND = 8;
    const int q = total / XCDS, r = total % XCDS;
    const int xcd = wg % XCDS, local = wg / XCDS;
    const int logical = xcd * q + imin(xcd, r) + local;
    const int per_band = BAND * tiles_n;
    const int band = logical / per_band, in_band = logical % per_band;
    const int first_m = band * BAND;
    const int rows = imin(tiles_m - first_m, BAND);
    *tm = first_m + in_band % rows;
    *tn = in_band / rows;
}

// first scale byte of the K step that starts at byte k0 of a row of codes
MXQ_ADDR_FN int scale_byte_of(int k0, int epb) { return (k0 * epb) >> 5; }

// ---- 128 x 128 tile kernel: 256 lanes, four 16-byte pieces of A and of B per lane and K step -----
// piece j of lane tid: row of the tile and byte column inside the 128-byte K step
MXQ_ADDR_FN int small_piece_row(int tid, int j) { return (tid + j * 256) >> 3; }
MXQ_ADDR_FN int small_piece_col(int tid, int j) { return ((tid + j * 256) & 7) * 16; }
// byte offset of that piece from the operand's first byte of this batch entry, K step at byte 0;
// row0 = first row of the tile, rows = rows of the operand (rows past the edge are clamped: what they
// produce is never stored)
MXQ_ADDR_FN int64_t small_code_offset(int row0, int rows, int kbytes, int tid, int j) {
    return (int64_t)imin(row0 + small_piece_row(tid, j), rows - 1) * kbytes + small_piece_col(tid, j);
}
// lanes 0..127 fetch the scale bytes of the A rows, 128..255 those of the B rows: 4 bytes (x EPB) each
MXQ_ADDR_FN int64_t small_scale_offset(int row0, int rows, int kb, int tid) {
    return (int64_t)imin(row0 + (tid & 127), rows - 1) * kb;
}
// K step number `step` of a workgroup that owns steps kbeg .. kbeg + nk - 1 and starts its cyclic walk
// at kstart (step may be nk: the loop's last iteration fetches one step it does not use)
MXQ_ADDR_FN int small_k_byte(int kbeg, int kstart, int step, int nk) { return (kbeg + (kstart + step) % nk) * BK; }

// ---- 256 x 256 tile kernel: 512 lanes = 8 waves; wave w copies rows 32 w .. 32 w + 31 of the A tile
// and of the B tile, 8 rows per load instruction i = 0..3; lane L lands at 16-byte position L % 8 of
// row 8 i + L / 8 of its LDS image and fetches the column that belongs there ---------------------------
MXQ_ADDR_FN int large_key(int r) { return (r >> 1) & 7; }
MXQ_ADDR_FN int large_piece_row(int wave, int lane, int i) { return wave * 32 + i * 8 + (lane >> 3); }
// byte offset from the tile's first row (K step at byte 0); last_row = rows of the operand - 1 - first
// row of the tile
MXQ_ADDR_FN uint32_t large_code_offset(int wave, int lane, int i, int last_row, int kbytes) {
    const int r = large_piece_row(wave, lane, i);
    return (uint32_t)imin(r, last_row) * (uint32_t)kbytes + (uint32_t)(((lane & 7) ^ large_key(r)) * 16);
}
// the scale bytes: waves 0-3 fetch those of the 256 A rows, waves 4-7 those of the B rows, one row per lane
MXQ_ADDR_FN int large_scale_row(int wave, int lane) { return (wave & 3) * 64 + lane; }
MXQ_ADDR_FN uint32_t large_scale_offset(int wave, int lane, int rows_left, int kb) {
    return (uint32_t)imin(large_scale_row(wave, lane), rows_left - 1) * (uint32_t)kb;
}
// The tiles of an XCD walk K in step, so that the A and B panels they share are fetched into that
// XCD's L2 once (a start staggered per tile cost up to 30 % on long-K shapes, whose panels do not
// stay in L2 that long).  The eight XCDs start at eight different places of a cyclic walk, which
// spreads the slices in flight over the memory channels -- unless the last scale group of a row is
// a partial one: then everybody starts at K = 0.  gs = K steps per 16-byte scale group.
MXQ_ADDR_FN int large_kstart(int logical, int nk, int nfull, int gs) {
    return nfull != nk ? 0 : (int)(((unsigned)(logical % 8) * (unsigned)(nk / gs)) / 8u) * gs;
}
MXQ_ADDR_FN int large_kidx(int kstart, int fs, int nk) {
    const int k = kstart + fs;
    return k >= nk ? k - nk : k;
}

}  // namespace mxq_addr
