// Bounds check of the GEMM kernels' tile copies, on the host.  Walks every (workgroup, tile, K step,
// load instruction, wave, lane) of a list of shapes through the address functions the kernels
// themselves use (microxcaling_amd/csrc/mxq_gemm_addr.h) in the order the kernels issue them, and
// checks that every byte range read -- 16 bytes of codes, 16 or 4 bytes of scales -- lies inside the
// operand it belongs to: codes (batch, rows, kbytes), scales (batch, rows, K / 32).
//
//   usage: gemm_addr_check            (prints one line per shape and kernel; exit status 1 on the
//                                      first range outside its operand)
//
// The launch rules restated here (which kernel a shape takes, grid sizes, K splits) are those of
// mxq_capi_gemm.hip; both kernels are checked on every shape they could be given.
#include <cstdint>
#include <cstdio>
#include <cstdlib>

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

int main() {
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
    bool ok = true;
    for (const Shape& s : shapes) {
        const long long before = checked;
        if (takes_large(s)) {
            ok = check_large(s, 256);                           // a workgroup per CU
            std::printf("%-55s 256 x 256 tiles: %lld ranges inside\n", s.what, checked - before);
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
