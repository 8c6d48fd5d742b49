// Address arithmetic of the GEMM kernels (mxq_gemm.h) and of the attention-score kernel
// (mxq_bmm_softmax.h), kept apart from the kernels so that it compiles for the host as well: global
// offsets of the tile copies, where each copy lands in LDS and where the fragments are read from,
// which copy instructions a K step issues in which of its groups, and which output elements a lane
// stores.  tests/cpp/gemm_addr_check.cpp walks shapes through these same functions: every global
// range inside its operand, every LDS range inside the allocation, every fragment byte the byte
// the matrix instruction expects (and landed before it is read, not overwritten while it may still
// be read), every output element written exactly once and inside the output.
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


// ---- LDS image of the 256 x 256 tile kernel ----------------------------------------------------------
// two stages of codes (A tile, then B tile: 256 rows x 128 bytes each), two scale groups (512 rows x
// 16 bytes: A rows, then B rows), two slots of scale bytes for K steps past the last whole group
// (per slot two planes of 512 rows x 4 bytes; 8-bit codes use one plane)
constexpr int L_TILE_BYTES = 256 * 128;
constexpr int L_STAGE_BYTES = 2 * L_TILE_BYTES;
constexpr int L_SCALE_OFF = 2 * L_STAGE_BYTES;
constexpr int L_SCALE_GROUP = 512 * 16;
constexpr int L_TAIL_OFF = L_SCALE_OFF + 2 * L_SCALE_GROUP;
constexpr int L_TAIL_PLANE = 512 * 4;
constexpr int L_TAIL_SLOT = 2 * L_TAIL_PLANE;
constexpr int L_LDS_BYTES = L_TAIL_OFF + 2 * L_TAIL_SLOT;
// Copy side.  A copy instruction writes lane L's bytes at (base + 16 L) or (base + 4 L).
// codes of flat step t, load instruction i of a wave (0..3: A rows 32 w + 8 i .., 4..7: B rows)
MXQ_ADDR_FN uint32_t large_lds_code_dst(int t, int wave, int i) {
    return (uint32_t)((t & 1) * L_STAGE_BYTES + (i >> 2) * L_TILE_BYTES + (wave * 32 + (i & 3) * 8) * 128);
}
// the n-th scale group a workgroup fetches (16 bytes per lane), and the scale bytes of single K step fs
// (4 bytes per lane, plane e)
MXQ_ADDR_FN uint32_t large_lds_scale_group_dst(int n, int wave) {
    return (uint32_t)(L_SCALE_OFF + (n & 1) * L_SCALE_GROUP + wave * 1024);
}
MXQ_ADDR_FN uint32_t large_lds_scale_tail_dst(int fs, int e, int wave) {
    return (uint32_t)(L_TAIL_OFF + (fs & 1) * L_TAIL_SLOT + e * L_TAIL_PLANE + wave * 256);
}
// Read side.  operand 0 = A, 1 = B; row = row of the tile; col16 = 16-byte column of the K step.
MXQ_ADDR_FN int large_lds_code_addr(int operand, int row, int col16) {       // + stage * L_STAGE_BYTES
    return operand * L_TILE_BYTES + row * 128 + ((col16 ^ large_key(row)) * 16);
}
MXQ_ADDR_FN int large_lds_scale_group_addr(int operand, int row) {           // + slot * L_SCALE_GROUP + (K step in group) * bytes per step
    return L_SCALE_OFF + operand * 4096 + row * 16;
}
MXQ_ADDR_FN int large_lds_scale_tail_addr(int operand, int row) {            // + (K step & 1) * L_TAIL_SLOT + e * L_TAIL_PLANE
    return L_TAIL_OFF + (operand * 256 + row) * 4;
}
// Row of the B tile that row fi of a 32-row MFMA fragment is.  16-bit outputs permute the rows
// (fragment row 8 q + 4 h + r = B row 16 (q / 2) + 8 h + 4 (q % 2) + r) so that the accumulator
// registers 8 j .. 8 j + 7 of a lane are 8 consecutive columns.
MXQ_ADDR_FN int large_frag_row_b(int fi, bool pair) {
    return pair ? (fi & 16) + ((fi & 4) << 1) + ((fi & 8) >> 1) + (fi & 3) : fi;
}

// ---- the K step of the 256 x 256 kernel as a schedule ------------------------------------------------
// A step runs ng groups of MFMAs.  The loads before the MFMAs of group gi read the current stage for
// gi <= barrier group; behind the MFMAs of the barrier group every wave waits for its copies and the
// workgroup meets at the one barrier of the step; after it the wave reads the next stage (operands of
// the next step's first group).  Behind the MFMAs of a group the wave issues copy instructions
// first .. first + count - 1 (0-3 A codes, 4-7 B codes, 8 scales) of the flat step `ahead` steps after
// the current one.  All nine are issued between two consecutive barriers: those of the groups behind
// the barrier first, the rest from group 0 on.  Before the first step the kernel issues the former share
// of step 1's copy itself.
MXQ_ADDR_FN constexpr int large_barrier_group(int ng) { return ng - 3; }
// `phase` (0: waves 0-3, 1: waves 4-7) lets a schedule give the two waves of a SIMD (w and w + 4) different
// places for their copy instructions; the one below does not (large_copy_by_phase() = false: the kernel
// then never asks for phase 1).  Every wave issues each of its nine loads exactly once between two
// barriers, in order.
MXQ_ADDR_FN constexpr bool large_copy_by_phase() { return false; }
MXQ_ADDR_FN constexpr int large_copy_first(int gi, int ng, int phase) {
    (void)phase;
    return gi == 0 ? 6 : gi == 1 ? 8 : gi > large_barrier_group(ng) ? (gi - large_barrier_group(ng) - 1) * 3 : 0;
}
MXQ_ADDR_FN constexpr int large_copy_count(int gi, int ng, int phase) {
    (void)phase;
    return gi == 0 ? 2 : gi == 1 ? 1 : gi > large_barrier_group(ng) ? 3 : 0;
}
MXQ_ADDR_FN constexpr int large_copy_ahead(int gi, int ng) { return gi > large_barrier_group(ng) ? 2 : 1; }
// loads of the next step that the groups behind a barrier issue (the kernel's prologue issues them itself
// for step 1)
MXQ_ADDR_FN constexpr int large_copy_behind_barrier(int ng, int phase) {
    int n = 0;
    for (int gi = large_barrier_group(ng) + 1; gi < ng; ++gi) n += large_copy_count(gi, ng, phase);
    return n;
}

// ---- output elements of a lane, 256 x 256 kernel ----------------------------------------------------------
// A 32 x 32 accumulator: lane L, register v holds C[row L % 32][fragment row 8 (v / 4) + 4 (L / 32) + v % 4]
// of the MFMA tile.  What a lane stores, relative to the tile's first row and column:
//  * 16-bit outputs, lane's own registers 8 h .. 8 h + 7: row L % 32, 8 columns from 16 h + 8 (L / 32);
//  * fp32 outputs, registers 4 q .. 4 q + 3: row L % 32, 4 columns from 8 q + 4 (L / 32);
//  * whole tiles store after an exchange between lanes L and L + 16 (piece 1 of the lower lane against
//    piece 0 of the upper one), so that four lanes hold 64 contiguous bytes of a row: piece `which`
//    (0 / 1) of a lane then is row L % 16 + 16 which, 16 bytes from byte 16 (2 (L / 16 % 2) + L / 32)
//    of the 64 (fp32: of the 16 columns 8 q .. 8 q + 15, q even).
MXQ_ADDR_FN int large_own_row(int lane) { return lane & 31; }
MXQ_ADDR_FN int large_own_col(int lane, int piece, int elems) { return 2 * elems * piece + elems * (lane >> 5); }
MXQ_ADDR_FN int large_swapped_row(int lane, int which) { return (lane & 15) + 16 * which; }
MXQ_ADDR_FN int large_swapped_col(int lane, int elems) { return elems * (2 * ((lane >> 4) & 1) + (lane >> 5)); }

// ---- attention-score kernel (mxq_bmm_softmax.h): 4 waves, a ring of B tiles per wave ------------------
constexpr int S_TILE_BYTES = 32 * 128;       // codes of a B tile
constexpr int S_RING = 3;                    // tiles per wave in LDS
constexpr int S_TILES = 16;                  // tiles per wave (4 x 16 x 32 = 2048 columns at most)
constexpr int S_LDS_BYTES = 4 * S_RING * S_TILE_BYTES;
// the i-th tile of a wave: the waves take pairs of neighbouring tiles in turn
MXQ_ADDR_FN int scores_tile_of(int wave, int i) { return 8 * (i >> 1) + 2 * wave + (i & 1); }
// copy instruction k (8 rows) of the wave's i-th tile: where it lands, what lane L fetches
MXQ_ADDR_FN uint32_t scores_lds_dst(int wave, int i, int k) {
    return (uint32_t)(wave * (S_RING * S_TILE_BYTES) + (i % S_RING) * S_TILE_BYTES + k * 1024);
}
MXQ_ADDR_FN uint32_t scores_code_offset(int lane, int k) {
    const int r = k * 8 + (lane >> 3);
    return (uint32_t)(r * 128 + (((lane & 7) ^ large_key(r)) * 16));
}
// where column col16 of tile row `row` is read from (+ the ring slot)
MXQ_ADDR_FN int scores_lds_addr(int row, int col16) { return row * 128 + ((col16 ^ large_key(row)) * 16); }
// output staging through the wave's part of the ring: piece p (16 bytes) of row r of a 32 x 64 pair of
// tiles sits at position p ^ (r & 7) of the row's 128 bytes
MXQ_ADDR_FN int scores_stage_addr(int row, int piece) { return row * 128 + ((piece ^ (row & 7)) * 16); }

}  // namespace mxq_addr
