// Host checks of the GEMM kernels and of the attention-score kernel, through the address functions the
// kernels themselves are compiled from (microxcaling_amd/csrc/mxq_gemm_addr.h).
//
// 1. Bounds of the tile copies: every (workgroup, tile, K step, load instruction, wave, lane) of a list
//    of shapes, in the order the kernels issue them; every byte range read -- 16 bytes of codes, 16 or 4
//    bytes of scales -- must lie inside the operand it belongs to: codes (batch, rows, kbytes), scales
//    (batch, rows, K / 32).
// 2. A model of the 256 x 256 kernel's LDS (model_large): the workgroup's K steps are replayed group by
//    group with LDS held as 4-byte granules that remember which operand bytes a copy put there and
//    between which two barriers it was issued.  Checked: every landing range inside the allocation and
//    inside its region; every fragment and scale read returns the bytes the matrix instruction's operand
//    layout calls for (row, K step, 16-byte column, scale byte); the copy that brought them was issued
//    before the barrier the read follows (each barrier is preceded by a wait for the wave's own copies);
//    no copy is issued into a granule that is read between the same two barriers (so no wave can still
//    want the old bytes); the operands held in registers when a group's MFMAs issue are that group's.
// 3. Output stores of the 256 x 256 kernel (stores_large): every element of the output written exactly
//    once, by the lane whose accumulator register holds it (32 x 32 accumulator layout, fragment-row
//    permutation of 16-bit outputs, the exchange between lanes L and L + 16), every 16-byte store inside
//    the output and aligned.
// 4. The attention-score kernel (model_scores): ring slots inside the wave's part of LDS, the count of
//    copies still in flight that each wait allows, slot reuse only after the slot's fragment has been
//    read and waited for, staging and stores of the quotients (every element once, inside the output).
//
//   usage: gemm_addr_check            (prints one line per shape and check; exit status 1 on the first
//                                      violation)
//          gemm_addr_check --plans    (prints which kernel and K split the rules restated here give each shape)
//
// The launch rules restated here (which kernel a shape takes, grid sizes, K splits) are those of
// mxq_capi_gemm.hip / mxq_capi_scores.hip; the loop skeletons are those of mxq_gemm.h / mxq_bmm_softmax.h.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <deque>
#include <string>
#include <vector>

#include "mxq_gemm_addr.h"

namespace {

using namespace mxq_addr;

struct Shape {
    int64_t batch;
    int M, N, K;
    bool nibbles;
    const char* what;
};

long long checked = 0;

bool inside(int64_t off, int bytes, int64_t size, const char* what, const Shape& s, int wg, int tile, int step,
            int wave, int lane) {
    ++checked;
    if (off >= 0 && off + bytes <= size) return true;
    std::printf("OUT OF BOUNDS: %s bytes [%lld, %lld) of %lld; shape %s batch=%lld M=%d N=%d K=%d nibbles=%d, "
                "workgroup %d tile %d K step %d wave %d lane %d\n",
                what, (long long)off, (long long)(off + bytes), (long long)size, s.what, (long long)s.batch, s.M,
                s.N, s.K, (int)s.nibbles, wg, tile, step, wave, lane);
    return false;
}

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- persistent 256 x 256 tile kernel (mx_gemm_nt_kernel_256p), grid = min(tiles, CUs rounded to 8) ----
bool check_large(const Shape& s, int cus) {
    const int epb = s.nibbles ? 2 : 1, sby = 4 * epb, gs = 16 / sby;
    const int kbytes = s.K / epb, kb = s.K / 32, nk = kbytes / BK, nfull = nk - nk % gs;
    const int tiles_m = (int)ceil_div(s.M, 256), tiles_n = (int)ceil_div(s.N, 256);
    const int per_batch = tiles_m * tiles_n;
    const int64_t total64 = (int64_t)per_batch * s.batch;
    const int total = (int)total64;
    const int G = total < cus ? total : cus;
    const int64_t a_size = s.batch * s.M * (int64_t)kbytes, b_size = s.batch * s.N * (int64_t)kbytes;
    const int64_t sa_size = s.batch * s.M * (int64_t)kb, sb_size = s.batch * s.N * (int64_t)kb;
    for (int wg = 0; wg < G; ++wg) {
        for (int logical = wg; logical < total; logical += G) {
            const int bz = logical / per_batch;
            int tm, tn;
            tile_of_workgroup(logical % per_batch, per_batch, tiles_m, tiles_n, &tm, &tn);
            if (tm < 0 || tm >= tiles_m || tn < 0 || tn >= tiles_n) {
                std::printf("OUT OF BOUNDS: tile (%d, %d) of (%d, %d), shape %s logical %d\n", tm, tn, tiles_m, tiles_n,
                            s.what, logical);
                return false;
            }
            const int m0 = tm * 256, n0 = tn * 256;
            const int64_t fa = bz * ((int64_t)s.M * kbytes) + (int64_t)m0 * kbytes;
            const int64_t fb = bz * ((int64_t)s.N * kbytes) + (int64_t)n0 * kbytes;
            const int64_t fsa = bz * ((int64_t)s.M * kb) + (int64_t)m0 * kb;
            const int64_t fsb = bz * ((int64_t)s.N * kb) + (int64_t)n0 * kb;
            const int kstart = large_kstart(logical, nk, nfull, gs);
            // every K step of the tile is fetched once (its first step possibly a second time, by the
            // last step of the last tile of a workgroup: same addresses)
            for (int fs = 0; fs < nk; ++fs) {
                const int k0 = large_kidx(kstart, fs, nk) * BK;
                for (int wave = 0; wave < 8; ++wave)
                    for (int lane = 0; lane < 64; ++lane) {
                        for (int i = 0; i < 4; ++i) {
                            const int64_t oa = fa + k0 + large_code_offset(wave, lane, i, s.M - 1 - m0, kbytes);
                            const int64_t ob = fb + k0 + large_code_offset(wave, lane, i, s.N - 1 - n0, kbytes);
                            if (!inside(oa, 16, a_size, "A codes", s, wg, logical, fs, wave, lane)) return false;
                            if (!inside(ob, 16, b_size, "B codes", s, wg, logical, fs, wave, lane)) return false;
                        }
                        const bool is_b = wave >= 4;
                        const int64_t base = (is_b ? fsb : fsa) + scale_byte_of(k0, epb) +
                                             large_scale_offset(wave, lane, is_b ? s.N - n0 : s.M - m0, kb);
                        const int64_t size = is_b ? sb_size : sa_size;
                        if (fs < nfull) {
                            if (fs % gs == 0 && !inside(base, 16, size, "scale group", s, wg, logical, fs, wave, lane))
                                return false;
                        } else {
                            for (int e = 0; e < epb; ++e)
                                if (!inside(base + 4 * e, 4, size, "scale tail", s, wg, logical, fs, wave, lane))
                                    return false;
                        }
                    }
            }
        }
    }
    return true;
}

// ---- 128 x 128 tile kernel (mx_gemm_nt_kernel), grid = (tiles, batch, K splits) -------------------------
bool check_small(const Shape& s, int splits) {
    const int epb = s.nibbles ? 2 : 1;
    const int kbytes = s.K / epb, kb = s.K / 32, nk_all = kbytes / BK;
    const int tiles_m = (int)ceil_div(s.M, 128), tiles_n = (int)ceil_div(s.N, 128);
    const int tiles = tiles_m * tiles_n;
    const int64_t a_size = s.M * (int64_t)kbytes, b_size = s.N * (int64_t)kbytes;   // per batch entry
    const int64_t sa_size = s.M * (int64_t)kb, sb_size = s.N * (int64_t)kb;
    const int per_split = (nk_all + splits - 1) / splits;
    for (int bx = 0; bx < tiles; ++bx) {
        int tm, tn;
        tile_of_workgroup(bx, tiles, tiles_m, tiles_n, &tm, &tn);
        if (tm < 0 || tm >= tiles_m || tn < 0 || tn >= tiles_n) {
            std::printf("OUT OF BOUNDS: tile (%d, %d) of (%d, %d), shape %s\n", tm, tn, tiles_m, tiles_n, s.what);
            return false;
        }
        const int m0 = tm * 128, n0 = tn * 128;
        for (int64_t by = 0; by < (s.batch < 3 ? s.batch : 3); ++by)          // the batch index only enters kstart
            for (int bz = 0; bz < splits; ++bz) {
                const int kbeg = bz * per_split;
                const int nk = imin(per_split, nk_all - kbeg);
                if (nk <= 0) {
                    std::printf("OUT OF BOUNDS: empty K split %d of %d, shape %s\n", bz, splits, s.what);
                    return false;
                }
                const int kstart = (int)(((unsigned)bx * 5u + (unsigned)by) % (unsigned)nk);
                for (int step = 0; step <= nk; ++step) {                       // step nk: fetched, not used
                    const int k0 = small_k_byte(kbeg, kstart, step, nk);
                    for (int tid = 0; tid < 256; ++tid) {
                        for (int j = 0; j < 4; ++j) {
                            if (!inside(small_code_offset(m0, s.M, kbytes, tid, j) + k0, 16, a_size, "A codes", s, bx,
                                        bx, step, tid >> 6, tid & 63))
                                return false;
                            if (!inside(small_code_offset(n0, s.N, kbytes, tid, j) + k0, 16, b_size, "B codes", s, bx,
                                        bx, step, tid >> 6, tid & 63))
                                return false;
                        }
                        const bool is_a = tid < 128;
                        const int64_t so = small_scale_offset(is_a ? m0 : n0, is_a ? s.M : s.N, kb, tid) +
                                           scale_byte_of(k0, epb);
                        for (int e = 0; e < epb; ++e)
                            if (!inside(so + 4 * e, 4, is_a ? sa_size : sb_size, "scales", s, bx, bx, step, tid >> 6,
                                        tid & 63))
                                return false;
                    }
                }
            }
    }
    return true;
}

// ================================================================================================
// 2. LDS model of the 256 x 256 kernel
// ================================================================================================
enum Kind { NONE = 0, A_CODES, B_CODES, A_SCALES, B_SCALES };
const char* kind_name[] = {"nothing", "A codes", "B codes", "A scales", "B scales"};

struct Granule {                 // 4 bytes of LDS
    int kind = NONE;
    int64_t off = -1;            // offset of its first byte in the operand it was copied from
    int issued = -1;             // barriers passed when the copy was issued
    int read = -1;               // barriers passed when it was last read
};

struct HalfTag { int operand, tile, h, step; };      // what a register set holds: operand 0 A / 1 B
struct ScaleTag { int operand, tile, step; };
bool same(const HalfTag& a, const HalfTag& b) { return a.operand == b.operand && a.tile == b.tile && a.h == b.h && a.step == b.step; }
bool same(const ScaleTag& a, const ScaleTag& b) { return a.operand == b.operand && a.tile == b.tile && a.step == b.step; }

struct LargeModel {
    const Shape& s;
    const bool pair;             // 16-bit outputs: permuted B fragment rows
    int epb, sby, gs, kbytes, kb, nk, nfull, tiles_m, tiles_n, per_batch, total, G, nh, qh, ng, bp;
    std::vector<Granule> lds;
    int epoch = 0;
    long long n_reads = 0, n_copies = 0;
    bool ok = true;
    // fetch side (uniform over the workgroup)
    int f_logical = 0, f_fs = 0, f_kstart = 0, f_m0 = 0, f_n0 = 0, f_bz = 0;
    int f_groups[2] = {0, 0};                        // scale groups fetched so far, per phase (waves 0-3 / 4-7)
    // compute side
    int c_groups = 0, c_slot = 0, sc_base = 0;
    bool tail = false;
    struct Where { int logical, cs; };               // tile and K step a flat step multiplies

    LargeModel(const Shape& shape, bool pair_, int cus) : s(shape), pair(pair_) {
        epb = s.nibbles ? 2 : 1;
        sby = 4 * epb;
        gs = 16 / sby;
        kbytes = s.K / epb;
        kb = s.K / 32;
        nk = kbytes / BK;
        nfull = nk - nk % gs;
        tiles_m = (int)ceil_div(s.M, 256);
        tiles_n = (int)ceil_div(s.N, 256);
        per_batch = tiles_m * tiles_n;
        total = (int)((int64_t)per_batch * s.batch);
        G = total < cus ? total : cus;
        nh = 2 * epb;
        qh = 4 / nh;
        ng = nh * 4;
        bp = large_barrier_group(ng);
        lds.assign(L_LDS_BYTES / 4, Granule());
    }

    bool bad(const char* what, int t, int gi, int wave, int lane, long long a = 0, long long b = 0) {
        std::printf("LDS MODEL: %s (%lld, %lld); shape %s M=%d N=%d K=%d nibbles=%d, flat step %d group %d wave %d lane %d, "
                    "%d barriers passed\n", what, a, b, s.what, s.M, s.N, s.K, (int)s.nibbles, t, gi, wave, lane, epoch);
        ok = false;
        return false;
    }

    void tile_origin(int logical, int* bz, int* m0, int* n0) const {
        int tm, tn;
        tile_of_workgroup(logical % per_batch, per_batch, tiles_m, tiles_n, &tm, &tn);
        *bz = logical / per_batch;
        *m0 = tm * 256;
        *n0 = tn * 256;
    }
    void fetch_tile(int logical) {
        f_logical = logical;
        tile_origin(logical, &f_bz, &f_m0, &f_n0);
        f_kstart = large_kstart(logical, nk, nfull, gs);
    }
    void fetch_advance() {
        if (++f_fs == nk) {
            f_fs = 0;
            if (f_logical + G < total) fetch_tile(f_logical + G);
        }
    }

    // lane L of a copy instruction lands `bytes` bytes at dst + bytes * L
    bool land(uint32_t dst, int bytes, int lane, int kind, int64_t off, int64_t size, int region_lo, int region_hi,
              int t, int gi, int wave) {
        const int64_t lo = (int64_t)dst + (int64_t)bytes * lane;
        if (off < 0 || off + bytes > size) return bad("copy reads outside its operand", t, gi, wave, lane, off, size);
        if (lo < region_lo || lo + bytes > region_hi || region_hi > L_LDS_BYTES)
            return bad("copy lands outside its LDS region", t, gi, wave, lane, lo, region_hi);
        for (int b = 0; b < bytes; b += 4) {
            Granule& g = lds[(lo + b) / 4];
            if (g.read == epoch) return bad("copy issued into bytes that are read between the same two barriers", t, gi, wave, lane, lo + b);
            if (g.issued == epoch) return bad("two copies into the same bytes between two barriers", t, gi, wave, lane, lo + b);
            g.kind = kind;
            g.off = off + b;
            g.issued = epoch;
            ++n_copies;
        }
        return true;
    }
    // load instruction i of the waves of a phase for flat step t, K step fs of the fetch-side tile (fetch_part)
    bool fetch_part(int t, int fs, int i, int gi, int phase) {
        const int k0 = large_kidx(f_kstart, fs, nk) * BK;
        const int64_t a_size = s.batch * s.M * (int64_t)kbytes, b_size = s.batch * s.N * (int64_t)kbytes;
        const int64_t sa_size = s.batch * s.M * (int64_t)kb, sb_size = s.batch * s.N * (int64_t)kb;
        const int64_t fa = f_bz * ((int64_t)s.M * kbytes) + (int64_t)f_m0 * kbytes;
        const int64_t fb = f_bz * ((int64_t)s.N * kbytes) + (int64_t)f_n0 * kbytes;
        for (int wave = 4 * phase; wave < 4 * phase + 4; ++wave) {
            const bool s_is_b = wave >= 4;
            const int64_t fs_base = s_is_b ? f_bz * ((int64_t)s.N * kb) + (int64_t)f_n0 * kb
                                           : f_bz * ((int64_t)s.M * kb) + (int64_t)f_m0 * kb;
            for (int lane = 0; lane < 64; ++lane) {
                const int stage_lo = (t & 1) * L_STAGE_BYTES;
                if (i < 4) {
                    if (!land(large_lds_code_dst(t, wave, i), 16, lane, A_CODES,
                              fa + k0 + large_code_offset(wave, lane, i, s.M - 1 - f_m0, kbytes), a_size, stage_lo,
                              stage_lo + L_TILE_BYTES, t, gi, wave))
                        return false;
                } else if (i < 8) {
                    if (!land(large_lds_code_dst(t, wave, i), 16, lane, B_CODES,
                              fb + k0 + large_code_offset(wave, lane, i - 4, s.N - 1 - f_n0, kbytes), b_size,
                              stage_lo + L_TILE_BYTES, stage_lo + L_STAGE_BYTES, t, gi, wave))
                        return false;
                } else {
                    const int64_t so = fs_base + scale_byte_of(k0, epb) +
                                       large_scale_offset(wave, lane, s_is_b ? s.N - f_n0 : s.M - f_m0, kb);
                    const int kind = s_is_b ? B_SCALES : A_SCALES;
                    const int64_t size = s_is_b ? sb_size : sa_size;
                    if (fs < nfull) {
                        if (fs % gs == 0) {
                            const int lo = L_SCALE_OFF + (f_groups[phase] & 1) * L_SCALE_GROUP;
                            if (!land(large_lds_scale_group_dst(f_groups[phase], wave), 16, lane, kind, so, size, lo,
                                      lo + L_SCALE_GROUP, t, gi, wave))
                                return false;
                        }
                    } else {
                        for (int e = 0; e < epb; ++e) {
                            const int lo = L_TAIL_OFF + (fs & 1) * L_TAIL_SLOT + e * L_TAIL_PLANE;
                            if (!land(large_lds_scale_tail_dst(fs, e, wave), 4, lane, kind, so + 4 * e, size, lo,
                                      lo + L_TAIL_PLANE, t, gi, wave))
                                return false;
                        }
                    }
                }
            }
        }
        if (i == 8 && fs < nfull && fs % gs == 0) ++f_groups[phase];
        return true;
    }

    bool read(int addr, int bytes, int kind, int64_t off, int t, int gi, int wave, int lane) {
        if (addr < 0 || addr + bytes > L_LDS_BYTES) return bad("read outside the LDS allocation", t, gi, wave, lane, addr);
        for (int b = 0; b < bytes; b += 4) {
            Granule& g = lds[(addr + b) / 4];
            if (g.kind != kind || g.off != off + b) {
                std::printf("  wanted %s byte %lld, LDS byte %d holds %s byte %lld\n", kind_name[kind], (long long)(off + b),
                            addr + b, kind_name[g.kind], (long long)g.off);
                return bad("a fragment read returns the wrong bytes", t, gi, wave, lane, addr + b);
            }
            if (g.issued >= epoch) return bad("read of bytes whose copy was issued after the last barrier", t, gi, wave, lane, addr + b);
            g.read = epoch;
            ++n_reads;
        }
        return true;
    }
    // the row of the tile that lane (wave, fi) reads for fragment `tile` of an operand
    int frag_row(int operand, int wave, int fi, int tile) const {
        const int wy = wave >> 1, wx = wave & 1;
        return operand == 0 ? wy * 64 + tile * 32 + fi : wx * 128 + tile * 32 + large_frag_row_b(fi, pair);
    }
    // half h of fragment `tile` of an operand out of stage `stage`, for (logical tile, K step cs) (half())
    bool read_half(int stage, int operand, int tile, int h, Where w, int t, int gi) {
        int bz, m0, n0;
        tile_origin(w.logical, &bz, &m0, &n0);
        const int k0 = large_kidx(large_kstart(w.logical, nk, nfull, gs), w.cs, nk) * BK;
        const int rows = operand == 0 ? s.M : s.N, row0 = operand == 0 ? m0 : n0;
        for (int wave = 0; wave < 8; ++wave)
            for (int lane = 0; lane < 64; ++lane) {
                const int fi = lane & 31, fg = lane >> 5;
                // the kernel: row of fragment 0 + tile * 32 rows; 16-byte columns 2 q' + fg, q' = h * qh + q
                const int lane_row = frag_row(operand, wave, fi, 0);
                const int r = frag_row(operand, wave, fi, tile);
                const int64_t row_off = (int64_t)bz * rows * kbytes + (int64_t)(row0 + imin(r, rows - 1 - row0)) * kbytes + k0;
                for (int q = 0; q < qh; ++q) {
                    const int addr = stage * L_STAGE_BYTES + large_lds_code_addr(operand, lane_row, 2 * (h * qh + q) + fg) +
                                     tile * 32 * 128;
                    // what the 32 x 32 x 64 instruction takes from lane (row, g): 8-bit codes K = 16 g .. and
                    // 32 + 16 g .. of its 64, nibbles K = 32 g .. of its 64; instruction h covers bytes 128 h / nh ..
                    const int col16 = epb == 1 ? 4 * h + 2 * q + fg : 2 * h + fg;
                    if (!read(addr, 16, operand == 0 ? A_CODES : B_CODES, row_off + 16 * col16, t, gi, wave, lane)) return false;
                }
            }
        return true;
    }
    // the scale bytes of this step for fragment `tile` (scales())
    bool read_scales(int operand, int tile, Where w, int t, int gi) {
        int bz, m0, n0;
        tile_origin(w.logical, &bz, &m0, &n0);
        const int k0 = large_kidx(large_kstart(w.logical, nk, nfull, gs), w.cs, nk) * BK;
        const int rows = operand == 0 ? s.M : s.N, row0 = operand == 0 ? m0 : n0;
        for (int wave = 0; wave < 8; ++wave)
            for (int lane = 0; lane < 64; ++lane) {
                const int fi = lane & 31;
                const int lane_row = frag_row(operand, wave, fi, 0), r = frag_row(operand, wave, fi, tile);
                const int64_t want = (int64_t)bz * rows * kb + (int64_t)(row0 + imin(r, rows - 1 - row0)) * kb + scale_byte_of(k0, epb);
                for (int e = 0; e < epb; ++e) {
                    const int addr = tail ? sc_base + large_lds_scale_tail_addr(operand, lane_row) + tile * 128 + e * L_TAIL_PLANE
                                          : sc_base + large_lds_scale_group_addr(operand, lane_row) + tile * 512 + 4 * e;
                    if (!read(addr, 4, operand == 0 ? A_SCALES : B_SCALES, want + 4 * e, t, gi, wave, lane)) return false;
                }
            }
        return true;
    }
    void scale_place(int cs) {
        tail = cs >= nfull;
        if (!tail && cs % gs == 0) c_slot = c_groups++ & 1;
        // the kernel's `sc` without the L_SCALE_OFF / L_TAIL_OFF that the per-lane offsets carry
        sc_base = tail ? (cs & 1) * L_TAIL_SLOT : c_slot * L_SCALE_GROUP + (cs % gs) * sby;
    }

    // replays workgroup wg over its first `max_tiles` tiles
    bool run(int wg, int max_tiles) {
        if (wg >= G) return true;
        std::vector<int> tiles;
        for (int l = wg; l < total && (int)tiles.size() < max_tiles; l += G) tiles.push_back(l);
        // Like the kernel, the model fetches one tile past the last one it multiplies when there is one;
        // when it stops early (max_tiles) the fetch side simply runs on into tiles nobody multiplies here.
        fetch_tile(wg);
        f_fs = 0;
        for (int phase = 0; phase < 2; ++phase)
            for (int i = 0; i < 9; ++i)
                if (!fetch_part(0, 0, i, -1, phase)) return false;
        ++epoch;                                             // s_waitcnt vmcnt(0); __syncthreads()
        fetch_advance();
        scale_place(0);
        HalfTag bfh, afh[2], late[2], bfh_n, afh_n[2];
        ScaleTag sb0, sa[2], sbv[4], sb0_n, sa_n[2];
        auto first_operands = [&](int stage, Where w, int step, HalfTag* b, ScaleTag* sb, HalfTag* a, ScaleTag* sav, int t, int gi) {
            if (!read_half(stage, 1, 0, 0, w, t, gi)) return false;
            *b = HalfTag{1, 0, 0, step};
            if (!read_scales(1, 0, w, t, gi)) return false;
            *sb = ScaleTag{1, 0, step};
            for (int ti = 0; ti < 2; ++ti) {
                if (!read_half(stage, 0, ti, 0, w, t, gi)) return false;
                a[ti] = HalfTag{0, ti, 0, step};
                if (!read_scales(0, ti, w, t, gi)) return false;
                sav[ti] = ScaleTag{0, ti, step};
            }
            return true;
        };
        if (!first_operands(0, Where{tiles[0], 0}, 0, &bfh, &sb0, afh, sa, 0, -1)) return false;
        for (int phase = 0; phase < 2; ++phase)                  // what the groups behind a barrier would have issued
            for (int i = 0; i < large_copy_behind_barrier(ng, large_copy_by_phase() ? phase : 0); ++i)
                if (!fetch_part(1, f_fs, i, -1, phase)) return false;

        int t = 0;
        for (size_t ti_ = 0; ti_ < tiles.size(); ++ti_) {
            const int logical = tiles[ti_];
            for (int cs = 0; cs < nk; ++cs, ++t) {
                const int next_cs = cs + 1 < nk ? cs + 1 : 0;
                // the tile the next flat step multiplies: the next tile of this workgroup, or, behind the
                // last one, this tile's first step once more (fetched, read, never multiplied)
                const int next_logical = next_cs != 0 ? logical : (logical + G < total ? logical + G : logical);
                const Where cur_w{logical, cs}, nxt_w{next_logical, next_cs};
                const int cur = t & 1, nxt = (t + 1) & 1;
                sbv[0] = sb0;
                for (int gi = 0; gi < ng; ++gi) {
                    const int h = gi / 4, tj = gi % 4;
                    HalfTag bfh_next = bfh, afh_next[2] = {afh[0], afh[1]};
                    if (gi < bp) {
                        const int h2 = (gi + 1) / 4, tj2 = (gi + 1) % 4;
                        if (!read_half(cur, 1, tj2, h2, cur_w, t, gi)) return false;
                        bfh_next = HalfTag{1, tj2, h2, t};
                        if (h2 == 0) {
                            if (!read_scales(1, tj2, cur_w, t, gi)) return false;
                            sbv[tj2] = ScaleTag{1, tj2, t};
                        }
                        if (tj2 == 0)
                            for (int a = 0; a < 2; ++a) {
                                if (!read_half(cur, 0, a, h2, cur_w, t, gi)) return false;
                                afh_next[a] = HalfTag{0, a, h2, t};
                            }
                    } else if (gi == bp) {
                        if (!read_half(cur, 1, 2, nh - 1, cur_w, t, gi)) return false;
                        if (!read_half(cur, 1, 3, nh - 1, cur_w, t, gi)) return false;
                        late[0] = HalfTag{1, 2, nh - 1, t};
                        late[1] = HalfTag{1, 3, nh - 1, t};
                        bfh_next = late[0];
                    } else if (gi == bp + 1) {
                        bfh_next = late[1];
                    }
                    // the MFMAs of this group: B half (tj, h) against both A halves (., h)
                    if (!same(bfh, HalfTag{1, tj, h, t})) return bad("the B registers of a group hold another fragment", t, gi, 0, 0, bfh.tile, bfh.h);
                    if (!same(sbv[tj], ScaleTag{1, tj, t})) return bad("the B scale registers of a group hold another fragment's", t, gi, 0, 0, sbv[tj].tile, sbv[tj].step);
                    for (int a = 0; a < 2; ++a) {
                        if (!same(afh[a], HalfTag{0, a, h, t})) return bad("the A registers of a group hold another fragment", t, gi, 0, 0, afh[a].tile, afh[a].h);
                        if (!same(sa[a], ScaleTag{0, a, t})) return bad("the A scale registers of a group hold another step's", t, gi, 0, 0, sa[a].tile, sa[a].step);
                    }
                    if (gi == bp) {
                        ++epoch;                             // s_waitcnt vmcnt(0) lgkmcnt(0); __syncthreads()
                        fetch_advance();
                        scale_place(next_cs);
                        if (!first_operands(nxt, nxt_w, t + 1, &bfh_n, &sb0_n, afh_n, sa_n, t, gi)) return false;
                    }
                    for (int phase = 0; phase < 2; ++phase) {
                        const int ph = large_copy_by_phase() ? phase : 0;
                        for (int i = 0; i < large_copy_count(gi, ng, ph); ++i)
                            if (!fetch_part(t + large_copy_ahead(gi, ng), f_fs, large_copy_first(gi, ng, ph) + i, gi, phase))
                                return false;
                    }
                    bfh = bfh_next;
                    afh[0] = afh_next[0];
                    afh[1] = afh_next[1];
                }
                bfh = bfh_n;
                sb0 = sb0_n;
                for (int a = 0; a < 2; ++a) {
                    afh[a] = afh_n[a];
                    sa[a] = sa_n[a];
                }
            }
        }
        return ok;
    }
};

// the model on a few workgroups of a shape: the first, one in the middle, the last, three tiles each
bool model_large(const Shape& s, int cus) {
    long long reads = 0, copies = 0;
    for (int pair = 0; pair < 2; ++pair) {
        LargeModel probe(s, pair != 0, cus);
        const int picks[4] = {0, probe.G / 2 + 1, probe.G - 1, 7};
        for (int k = 0; k < 4; ++k) {
            if (k > 0 && picks[k] == picks[k - 1]) continue;
            LargeModel m(s, pair != 0, cus);
            if (!m.run(picks[k] % probe.G, 3)) return false;
            reads += m.n_reads;
            copies += m.n_copies;
        }
    }
    std::printf("%-55s LDS model: %lld granules copied, %lld read, all as the MFMAs want them\n", s.what, copies, reads);
    return true;
}

// ================================================================================================
// 3. Output stores of the 256 x 256 kernel
// ================================================================================================
struct Coord { int m, n; };       // relative to the tile

// permlane16_swap as the epilogue uses it: `b` of the lanes 0-15 / 32-47 trades places with `a` of the
// lanes 16-31 / 48-63 (lane L with lane L + 16)
template <class T>
void swap_with_lane16(std::vector<T>& a, std::vector<T>& b) {
    for (int lane = 0; lane < 64; ++lane)
        if ((lane & 16) == 0) std::swap(b[lane], a[lane + 16]);
}

// out_bytes: 2 (bf16 / fp16) or 4; bias: a bias is added (fp32 whole tiles then store without the exchange)
bool stores_large(const Shape& s, int out_bytes, bool bias) {
    const bool pair = out_bytes == 2;
    const int tiles_m = (int)ceil_div(s.M, 256), tiles_n = (int)ceil_div(s.N, 256);
    const int per_batch = tiles_m * tiles_n;
    const int64_t total = (int64_t)per_batch * s.batch;
    const int64_t out_elems = s.batch * (int64_t)s.M * s.N;
    std::vector<int> seen_tile(per_batch, 0);
    std::vector<unsigned char> count(256 * 256);
    long long stores = 0;
    auto fail = [&](const char* what, int logical, int wave, int lane, long long a, long long b) {
        std::printf("STORES: %s (%lld, %lld); shape %s M=%d N=%d, %d-byte outputs%s, tile %d wave %d lane %d\n", what, a, b,
                    s.what, s.M, s.N, out_bytes, bias ? " with bias" : "", logical, wave, lane);
        return false;
    };
    for (int64_t logical = 0; logical < total; ++logical) {
        int tm, tn;
        tile_of_workgroup((int)(logical % per_batch), per_batch, tiles_m, tiles_n, &tm, &tn);
        const int64_t bz = logical / per_batch;
        if (bz == 0) ++seen_tile[tm * tiles_n + tn];
        const int m0 = tm * 256, n0 = tn * 256;
        const bool edge = m0 + 256 > s.M || n0 + 256 > s.N;
        if (total > 2000 && !edge && logical % 97 != 0) continue;        // whole tiles are all alike
        const int64_t cbase = bz * (int64_t)s.M * s.N;
        const bool inside = m0 + 256 <= s.M && n0 + 256 <= s.N && (s.N & 3) == 0;
        const bool inside8 = inside && (s.N & 7) == 0;
        std::fill(count.begin(), count.end(), 0);
        // one element: label = where the accumulator register's value belongs, (m, n) = where it is stored
        auto put = [&](Coord label, int m, int n, int wave, int lane) {
            if (label.m != m || label.n != n) return fail("a value is stored at another element's place", (int)logical, wave, lane, m, n);
            if (m0 + m >= s.M || n0 + n >= s.N) return fail("store outside the matrix", (int)logical, wave, lane, m0 + m, n0 + n);
            if (count[m * 256 + n]++) return fail("element stored twice", (int)logical, wave, lane, m0 + m, n0 + n);
            ++stores;
            return true;
        };
        // a 16-byte store of `elems` consecutive elements
        auto put_vec = [&](const std::vector<Coord>& labels, int m, int n, int wave, int lane) {
            const int64_t idx = cbase + (int64_t)(m0 + m) * s.N + n0 + n;
            const int elems = (int)labels.size();
            if (idx < 0 || idx + elems > out_elems) return fail("vector store outside the output", (int)logical, wave, lane, idx, out_elems);
            if ((idx * out_bytes) % 16 != 0) return fail("vector store not 16-byte aligned", (int)logical, wave, lane, idx, 0);
            for (int j = 0; j < elems; ++j)
                if (!put(labels[j], m, n + j, wave, lane)) return false;
            return true;
        };
        for (int wave = 0; wave < 8; ++wave) {
            const int wy = wave >> 1, wx = wave & 1;
            for (int ti = 0; ti < 2; ++ti)
                for (int tj = 0; tj < 4; ++tj) {
                    const int mt = wy * 64 + ti * 32, nt = wx * 128 + tj * 32;
                    // accumulator layout of the 32 x 32 x 64 instruction with the B fragment as the first
                    // operand: lane L, register v = C[A-fragment row L % 32][B-fragment row 8 (v / 4) + 4 (L / 32) + v % 4]
                    auto reg = [&](int lane, int v) {
                        const int brow = 8 * (v / 4) + 4 * (lane >> 5) + v % 4;
                        return Coord{mt + (lane & 31), nt + large_frag_row_b(brow, pair)};
                    };
                    const int elems = pair ? 8 : 4, pieces = 16 / elems;
                    const bool exchange = pair ? inside8 : (inside && !bias);
                    if (exchange) {
                        for (int q = 0; q < pieces; q += 2) {             // pieces q and q + 1 of every lane
                            std::vector<std::vector<Coord>> p0(64), p1(64);
                            for (int lane = 0; lane < 64; ++lane)
                                for (int j = 0; j < elems; ++j) {
                                    p0[lane].push_back(reg(lane, elems * q + j));
                                    p1[lane].push_back(reg(lane, elems * (q + 1) + j));
                                    // what the lane believes it holds (bias index, epilogue_pack8's n)
                                    const Coord own{mt + large_own_row(lane), nt + large_own_col(lane, q, elems) + j};
                                    if (own.m != p0[lane][j].m || own.n != p0[lane][j].n)
                                        return fail("a lane's own columns are not where its registers belong", (int)logical, wave, lane, own.m, own.n);
                                }
                            swap_with_lane16(p0, p1);
                            for (int lane = 0; lane < 64; ++lane) {
                                const int col = nt + (pair ? 0 : 8 * q) + large_swapped_col(lane, elems);
                                if (!put_vec(p0[lane], mt + large_swapped_row(lane, 0), col, wave, lane)) return false;
                                if (!put_vec(p1[lane], mt + large_swapped_row(lane, 1), col, wave, lane)) return false;
                            }
                        }
                    } else {
                        for (int lane = 0; lane < 64; ++lane)
                            for (int q = 0; q < pieces; ++q) {
                                const int m = mt + large_own_row(lane), n = nt + large_own_col(lane, q, elems);
                                std::vector<Coord> labels;
                                for (int j = 0; j < elems; ++j) labels.push_back(reg(lane, elems * q + j));
                                if (!pair && inside) {                    // store_c4 on a whole tile: one 16-byte store
                                    if (!put_vec(labels, m, n, wave, lane)) return false;
                                } else if (m0 + m < s.M) {                // element by element, guarded
                                    for (int j = 0; j < elems; ++j)
                                        if (n0 + n + j < s.N && !put(labels[j], m, n + j, wave, lane)) return false;
                                }
                            }
                    }
                }
        }
        for (int m = 0; m < 256 && m0 + m < s.M; ++m)
            for (int n = 0; n < 256 && n0 + n < s.N; ++n)
                if (count[m * 256 + n] != 1) return fail("element never stored", (int)logical, -1, -1, m0 + m, n0 + n);
    }
    for (int i = 0; i < per_batch; ++i)
        if (seen_tile[i] != 1) return fail("an output tile is not visited exactly once per batch entry", i, -1, -1, seen_tile[i], 0);
    std::printf("%-55s stores, %d-byte outputs%s: %lld elements, each once and in place\n", s.what, out_bytes,
                bias ? " + bias" : "", stores);
    return true;
}

// ================================================================================================
// 4. The attention-score kernel: (batch, M, 128) x (batch, N, 128)^T -> softmax rows (batch, M, N)
// ================================================================================================
bool model_scores(int64_t batch, int M, int N) {
    const int ntiles = N / 32;
    const int64_t b_size = batch * (int64_t)N * 128, out_elems = batch * (int64_t)M * N;
    long long granules = 0, stores = 0;
    auto fail = [&](const char* what, int wg, int wave, int lane, long long a, long long b) {
        std::printf("SCORES: %s (%lld, %lld); batch=%lld M=%d N=%d, workgroup %d wave %d lane %d\n", what, a, b,
                    (long long)batch, M, N, wg, wave, lane);
        return false;
    };
    const int strips = (int)ceil_div(M, 32);
    for (int64_t bz = 0; bz < batch; bz += (batch > 2 ? batch - 1 : 1))       // first and last batch entry
        for (int wg = 0; wg < strips; wg += (strips > 3 ? strips - 1 : 1)) { // first and last strip of rows
            const int m0 = wg * 32;
            std::vector<Granule> lds(S_LDS_BYTES / 4);
            std::vector<unsigned char> count(32 * (size_t)N, 0);
            for (int wave = 0; wave < 4; ++wave) {
                const int part_lo = wave * S_RING * S_TILE_BYTES, part_hi = part_lo + S_RING * S_TILE_BYTES;
                int my_tiles = 0;
                for (int i = 0; i < S_TILES; ++i) my_tiles += scores_tile_of(wave, i) < ntiles ? 1 : 0;
                std::deque<int> in_flight;                     // tile numbers of the copy instructions not yet waited for
                std::vector<int> landed(S_TILES, 0), slot_read_done(S_RING, 1);
                auto fetch_b = [&](int i) {
                    const int t = scores_tile_of(wave, i);
                    if (t >= ntiles) return true;
                    if (!slot_read_done[i % S_RING])
                        return fail("a ring slot is refilled before its fragment read has been waited for", wg, wave, -1, i, i % S_RING);
                    for (int k = 0; k < 4; ++k) {
                        for (int lane = 0; lane < 64; ++lane) {
                            const int64_t off = bz * (int64_t)N * 128 + (int64_t)t * S_TILE_BYTES + scores_code_offset(lane, k);
                            const int64_t lo = (int64_t)scores_lds_dst(wave, i, k) + 16 * lane;
                            if (off < 0 || off + 16 > b_size) return fail("copy reads outside B", wg, wave, lane, off, b_size);
                            if (lo < part_lo || lo + 16 > part_hi) return fail("copy lands outside the wave's ring", wg, wave, lane, lo, part_hi);
                            for (int b = 0; b < 16; b += 4) {
                                lds[(lo + b) / 4].kind = B_CODES;
                                lds[(lo + b) / 4].off = off + b;
                                lds[(lo + b) / 4].issued = i;
                                ++granules;
                            }
                        }
                        in_flight.push_back(i);
                    }
                    return true;
                };
                auto multiply = [&](int i) {
                    const int t = scores_tile_of(wave, i);
                    if (t >= ntiles) return true;
                    const int later = imin(S_RING - 1, my_tiles - 1 - i);
                    while ((int)in_flight.size() > 4 * later) {          // s_waitcnt vmcnt(4 * later): copies complete in order
                        landed[in_flight.front()]++;
                        in_flight.pop_front();
                    }
                    if (landed[i] != 4) return fail("a tile is read before its four copies have been waited for", wg, wave, -1, i, landed[i]);
                    for (int lane = 0; lane < 64; ++lane) {
                        const int fi = lane & 31, fg = lane >> 5;
                        const int brow = large_frag_row_b(fi, true);
                        for (int q = 0; q < 4; ++q) {
                            const int addr = part_lo + (i % S_RING) * S_TILE_BYTES + scores_lds_addr(brow, 2 * q + fg);
                            // two 32 x 32 x 64 instructions on 8-bit codes: lane (row, g) supplies the 16-byte
                            // columns 4 h + g and 4 h + 2 + g of the row for instruction h, in that order
                            const int64_t want = bz * (int64_t)N * 128 + (int64_t)(t * 32 + brow) * 128 + 16 * (2 * q + fg);
                            if (addr < part_lo || addr + 16 > part_hi) return fail("fragment read outside the wave's ring", wg, wave, lane, addr, part_hi);
                            for (int b = 0; b < 16; b += 4) {
                                const Granule& g = lds[(addr + b) / 4];
                                if (g.kind != B_CODES || g.off != want + b || g.issued != i)
                                    return fail("a fragment read returns the wrong bytes", wg, wave, lane, g.off, want + b);
                            }
                        }
                    }
                    slot_read_done[i % S_RING] = 0;                        // read issued; data not yet waited for
                    return true;
                };
                // the kernel's loop: the first S_RING copies, then per tile: wait for the fragment registers
                // (s_waitcnt lgkmcnt(0)), refill the slot, multiply the next tile
                for (int i = 0; i < S_RING; ++i)
                    if (!fetch_b(i)) return false;
                if (!multiply(0)) return false;
                for (int i = 0; i < S_TILES; ++i) {
                    if (i + S_RING < S_TILES) {
                        for (int k = 0; k < S_RING; ++k) slot_read_done[k] = 1;   // s_waitcnt lgkmcnt(0)
                        if (!fetch_b(i + S_RING)) return false;
                    }
                    if (i + 1 < S_TILES && !multiply(i + 1)) return false;
                }
                if (!in_flight.empty()) return fail("copies still in flight when the ring is reused for the output", wg, wave, -1, in_flight.size(), 0);
                // phase 3: pairs of tiles through the wave's part of the ring, 128-byte lines to memory
                for (int k = 0; k < S_TILES / 2; ++k) {
                    const int t0 = scores_tile_of(wave, 2 * k);
                    if (t0 >= ntiles) continue;
                    const int buf = part_lo + (k & 1) * S_TILE_BYTES;
                    std::vector<Coord> staged(S_TILE_BYTES / 16, Coord{-1, -1});     // per 16-byte piece: (row, first column)
                    for (int p = 0; p < 2; ++p)
                        for (int lane = 0; lane < 64; ++lane) {
                            const int fi = lane & 31, fg = lane >> 5;
                            // accumulator registers 0-7: columns 8 fg .. of tile p of the pair, 8-15: columns 16 + 8 fg ..
                            for (int half = 0; half < 2; ++half) {
                                const int piece = 4 * p + 2 * half + fg;
                                const int addr = buf + scores_stage_addr(fi, piece);
                                if (addr < part_lo || addr + 16 > part_hi) return fail("staging write outside the wave's ring", wg, wave, lane, addr, part_hi);
                                Coord& c = staged[(addr - buf) / 16];
                                if (c.m != -1) return fail("two lanes stage into the same 16 bytes", wg, wave, lane, addr, 0);
                                c = Coord{fi, (t0 + p) * 32 + 16 * half + 8 * fg};
                            }
                        }
                    const bool second = t0 + 1 < ntiles;
                    for (int r = 0; r < 4; ++r)
                        for (int lane = 0; lane < 64; ++lane) {
                            const int srow = lane >> 3, spiece = lane & 7, row = 8 * r + srow;
                            const int addr = buf + scores_stage_addr(row, spiece);
                            if (addr < part_lo || addr + 16 > part_hi) return fail("staging read outside the wave's ring", wg, wave, lane, addr, part_hi);
                            const Coord c = staged[(addr - buf) / 16];
                            if (!(m0 + row < M && (second || spiece < 4))) continue;
                            const int col = t0 * 32 + 8 * spiece;
                            if (c.m != row || c.n != col) return fail("a staged piece is stored at another piece's place", wg, wave, lane, c.m, c.n);
                            const int64_t idx = bz * (int64_t)M * N + (int64_t)(m0 + srow) * N + 8 * spiece + (int64_t)(8 * r) * N + t0 * 32;
                            if (idx < 0 || idx + 8 > out_elems) return fail("store outside the output", wg, wave, lane, idx, out_elems);
                            if ((idx * 2) % 16 != 0) return fail("store not 16-byte aligned", wg, wave, lane, idx, 0);
                            if (col + 8 > N) return fail("store past the end of a row", wg, wave, lane, col, N);
                            for (int j = 0; j < 8; ++j)
                                if (count[(size_t)row * N + col + j]++) return fail("element stored twice", wg, wave, lane, row, col + j);
                            stores += 8;
                        }
                }
            }
            for (int row = 0; row < 32 && m0 + row < M; ++row)
                for (int n = 0; n < N; ++n)
                    if (count[(size_t)row * N + n] != 1) return fail("element never stored", wg, -1, -1, m0 + row, n);
        }
    std::printf("scores kernel batch=%lld M=%d N=%d: %lld granules through the ring, %lld elements stored, each once\n",
                (long long)batch, M, N, granules, stores);
    return true;
}

// launch rules of mxq_capi_gemm.hip
bool takes_large(const Shape& s) {
    const int64_t total = ceil_div(s.M, 256) * ceil_div(s.N, 256) * s.batch;
    const int64_t kbytes = s.nibbles ? s.K / 2 : s.K;
    return s.M >= 512 && s.N >= 512 && s.K >= 512 && total >= 128 && total < ((int64_t)1 << 30) &&
           256 * kbytes < ((int64_t)1 << 31);
}
int k_splits(const Shape& s) {
    if (takes_large(s)) return 1;
    const int64_t tiles = ceil_div(s.M, 128) * ceil_div(s.N, 128) * s.batch;
    const int64_t nk = s.K / (s.nibbles ? 256 : 128);
    if (tiles >= 256 || nk < 4) return 1;
    int64_t splits = ceil_div(512, tiles);
    if (splits > nk / 2) splits = nk / 2;
    if (splits > 64) splits = 64;
    const int64_t per = ceil_div(nk, splits);
    return (int)ceil_div(nk, per);
}

}  // namespace

int main(int argc, char** argv) {
    const Shape shapes[] = {
        {1, 16384, 14336, 4096, false, "config 4 (MXFP8)"},
        {1, 16384, 14336, 4096, true, "config 4 (MXFP4 nibbles)"},
        {128, 2048, 2048, 128, false, "config 5 (one K step)"},
        {1, 4096, 16384, 14336, false, "weight gradient of config 4, reduced M"},
        {1, 16384, 4096, 11008, false, "K % 512 != 0 (tail scale steps)"},
        {1, 4096, 4096, 11264, true, "nibbles, K % 512 == 0"},
        {1, 4100, 4196, 1408, false, "ragged M and N, K % 512 != 0"},
        {1, 4100, 4196, 1536, true, "ragged M and N, nibbles"},
        {1, 4097, 4097, 640, false, "one row and one column past a tile edge"},
        {3, 2305, 2049, 512, false, "batched, ragged, the smallest K of the large tiles"},
        {3, 2305, 2049, 768, true, "batched, ragged, nibbles, odd number of K steps"},
        {5, 2560, 2816, 4096, false, "batched, whole tiles"},
        {1, 512, 1024, 384, false, "small tiles (GPU test shape)"},
        {1, 1030, 520, 1152, false, "small tiles, ragged"},
        {1, 70, 136, 256, false, "small tiles, less than one tile"},
        {1, 64, 8192, 8192, false, "decode shape: K split over 64 workgroups"},
        {1, 256, 8192, 8192, true, "decode shape, nibbles"},
        {1, 1, 129, 128, false, "one row"},
        {6, 200, 264, 128, false, "batched attention scores, ragged"},
        {2, 300, 257, 3328, true, "nibbles, 13 K steps, split"},
    };
    if (argc > 1 && std::string(argv[1]) == "--plans") {
        // the launch rules as restated above, one line per shape, for comparison with what the library itself
        // reports (mxq_gemm_plan, mxq_gemm_workspace_bytes): batch M N K nibbles large-tiles K-splits
        for (const Shape& s : shapes)
            std::printf("%lld %lld %lld %lld %d %d %d\n", (long long)s.batch, (long long)s.M, (long long)s.N,
                        (long long)s.K, s.nibbles ? 1 : 0, takes_large(s) ? 1 : 0, k_splits(s));
        return 0;
    }
    bool ok = true;
    // the attention-score kernel: config 5, ragged rows, an odd number of tiles, the narrowest and widest rows
    const int scores[][3] = {{128, 2048, 2048}, {3, 100, 1056}, {1, 32, 32}, {2, 33, 64}, {1, 2048, 96}, {5, 70, 2016}};
    for (const auto& c : scores) ok = ok && model_scores(c[0], c[1], c[2]);
    if (!ok) return 1;
    for (const Shape& s : shapes) {
        const long long before = checked;
        if (takes_large(s)) {
            ok = check_large(s, 256);                           // a workgroup per CU
            std::printf("%-55s 256 x 256 tiles: %lld ranges inside\n", s.what, checked - before);
            ok = ok && model_large(s, 256);
            ok = ok && stores_large(s, 2, false) && stores_large(s, 4, false) && stores_large(s, 4, true);
        }
        if (!ok) break;
        // the small-tile kernel takes any shape (it is also what a workspace-less caller of a split shape gets)
        const long long mid = checked;
        const int splits = k_splits(s);
        const bool big = (int64_t)s.M * s.N > (int64_t)8192 * 8192;     // keep the run short: large shapes unsplit only
        ok = ok && check_small(s, 1);
        if (ok && splits > 1 && !big) ok = check_small(s, splits);
        std::printf("%-55s 128 x 128 tiles (K splits 1%s): %lld ranges inside\n", s.what,
                    splits > 1 ? " and as launched" : "", checked - mid);
        if (!ok) break;
    }
    if (!ok) return 1;
    std::printf("all %lld byte ranges inside their operands\n", checked);
    return 0;
}
