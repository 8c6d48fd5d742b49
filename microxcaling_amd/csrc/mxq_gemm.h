// Packed MX tensors and the scaled-MFMA GEMM that consumes them (gfx950).
//
// Packed form of a (rows, K) tensor quantized along K in blocks of 32:
//   codes  uint8 (rows, K)      one OCP 8-bit float per element: e4m3 ("fn") for the element
//                               formats fp8_e4m3 / fp6_e3m2 / fp6_e2m3 / fp4_e2m1 (all of whose
//                               values e4m3 represents exactly), e5m2 for fp8_e5m2
//   scales uint8 (rows, K/32)   E8M0: shared exponent + 127, 255 = NaN block
// codes[i][k] * 2^(scales[i][k/32] - 127) is bit-for-bit the value the fake-quantizing kernels
// return (before their final rounding to a 16-bit tensor dtype).
//
// v_mfma_scale_f32_16x16x128_f8f6f4 multiplies a 16x128 by a 128x16 tile of such codes.  Lane
// (row = lane % 16, g = lane / 16) supplies 32 codes of its row: K = 16g .. 16g+15 in its first four
// registers and K = 64+16g .. 64+16g+15 in the last four.  The E8M0 byte of K block j (32
// consecutive K) of a row is taken from the scale register of lane row + 16j -- so each lane passes
// the scale of block g, and block scaling costs nothing extra.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxq_kernels.h"

namespace {

// ================================================================================================
// quantize + pack, shared axis innermost, block size 32
// ================================================================================================
template <int DT, int RMODE, bool ZONE_ELEM, bool BF8, int UNROLL>
__global__ __launch_bounds__(TPB) void mx_pack_kernel(const u32x4* __restrict__ in,
                                                      void* __restrict__ codes_,
                                                      unsigned char* __restrict__ scales,
                                                      int64_t n_vec, MxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int LPT = 8 / PD;                            // lanes per 32-element block
    constexpr int64_t CHUNK = (int64_t)TPB * UNROLL;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.zone_row]);

    const int64_t stride = (int64_t)gridDim.x * CHUNK;
    for (int64_t base = (int64_t)blockIdx.x * CHUNK + threadIdx.x; base - threadIdx.x < n_vec;
         base += stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + j * TPB;
            v[j] = (i < n_vec) ? in[i] : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + j * TPB;
            const uint32_t um = group_max<LPT>(vec_abs_max<DT>(v[j]));
            const MxqScale sc = mxq_block_scale(um, p.emax, p.scale_emax, p.flush != 0, zone, ZS);
            uint32_t out[PD] = {};
#pragma unroll
            for (int d = 0; d < 4; ++d)
#pragma unroll
                for (int h = 0; h < PD; ++h) {
                    const float y = mxq_quant_mx_elem_unscaled<RMODE, ADT, ZONE_ELEM>(
                        Pack<DT>::get(v[j][d], h), sc, p.fmt, zone, ZS);
                    const uint32_t c = BF8 ? mxq_encode_e5m2(y) : mxq_encode_e4m3(y);
                    const int e = d * PD + h;              // element index inside the vector
                    out[e / 4] |= c << (8 * (e % 4));
                }
            if (i < n_vec) {
                if (PD == 1) reinterpret_cast<uint32_t*>(codes_)[i] = out[0];
                else reinterpret_cast<u32x2*>(codes_)[i] = u32x2{out[0], out[PD - 1]};
                if ((threadIdx.x & (LPT - 1)) == 0)
                    scales[i / LPT] = (unsigned char)mxq_encode_e8m0(sc.scale);
            }
        }
    }
}

// unpack: codes * 2^(scale-127) -> fp32 / bf16 / fp16 (for tests and for callers that want the
// fake-quantized view of a packed tensor)
template <int DT, bool BF8>
__global__ __launch_bounds__(TPB) void mx_unpack_kernel(const unsigned char* __restrict__ codes,
                                                        const unsigned char* __restrict__ scales,
                                                        void* __restrict__ out, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
        const uint32_t s = scales[i >> 5];
        const float y = BF8 ? mxq_decode_e5m2(codes[i]) : mxq_decode_e4m3(codes[i]);
        float v = y * ldexpf(1.0f, (int)s - 127);
        if (s == 255u) v = mxq_float(MXQ_QNAN_BITS);
        store_scalar<DT>(out, i, mxq_round_dt<Arith<DT>::DT_>(v));
    }
}

// ================================================================================================
// C[b] (M, N) = A[b] (M, K) x B[b] (N, K)^T on packed operands, fp32 accumulation.
// Workgroup: 256 lanes = 2 x 2 waves, tile 128 x 128 x 128; each wave owns 64 x 64 = 4 x 4 MFMA
// tiles.  A and B tiles are staged through LDS with a 144-byte row pitch, which makes the 32-byte
// per-lane fragment reads conflict free.
// ================================================================================================
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int GEMM_BM = 128, GEMM_BN = 128, GEMM_BK = 128, GEMM_PITCH = GEMM_BK + 16;

struct GemmArgs {
    const unsigned char* a;
    const unsigned char* sa;
    const unsigned char* b;
    const unsigned char* sb;
    void* c;
    const void* bias;     // optional (N), dtype of C: C = round(round(A x B^T) + bias)
    int M, N, K;
    int64_t batch_a, batch_sa, batch_b, batch_sb, batch_c;   // element strides between batches
};

// Which output tile a workgroup computes.  Workgroups are dealt round-robin to the 8 XCDs, each
// with its own L2, so workgroup w runs on XCD w % 8.  Give every XCD a contiguous range of
// "logical" tile numbers, and walk the tile grid in bands of 8 tile-rows: the ~32 tiles an XCD
// works on at any time then form an 8 x 4 patch that shares 8 A tiles and 4 B tiles per K step
// through that XCD's L2 instead of streaming 64 tiles from the fabric.
__device__ __forceinline__ void tile_of_workgroup(int wg, int total, int tiles_m, int tiles_n,
                                                  int* tm, int* tn) {
    constexpr int XCDS = 8, BAND = 8;
    const int q = total / XCDS, r = total % XCDS;
    const int xcd = wg % XCDS, local = wg / XCDS;
    const int logical = xcd * q + min(xcd, r) + local;
    const int per_band = BAND * tiles_n;
    const int band = logical / per_band, in_band = logical % per_band;
    const int first_m = band * BAND;
    const int rows = min(tiles_m - first_m, BAND);
    *tm = first_m + in_band % rows;
    *tn = in_band / rows;
}

// a lane's MFMA operand: 16 codes at p (K = 16g ..) and 16 codes at p + 64 (K = 64 + 16g ..)
__device__ __forceinline__ v8i load_frag(const unsigned char* p) {
    const u32x4 lo = *reinterpret_cast<const u32x4*>(p);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(p + 64);
    return v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
}

// The MFMAs are issued with the B fragment as the first operand, i.e. they compute 16 x 16 blocks
// of C^T: a lane then holds four *consecutive columns* n = 4 * (lane / 16) + r of one row
// m = lane % 16, which it can store with a single 8- or 16-byte access.
template <int OUT_DT>
__device__ __forceinline__ void store_c4(void* c, const void* bias, int64_t base, int m, int n,
                                         int M, int N, bool tile_inside, v4f v) {
    constexpr int ADT = Arith<OUT_DT>::DT_;
    if (bias != nullptr) {
        // what the layers do as separate tensor ops: the product is rounded to the tensor dtype,
        // the bias is added, and the sum is rounded again (by the store below)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float b = (n + r < N) ? load_scalar<OUT_DT>(bias, n + r) : 0.0f;
            const float p = (OUT_DT == MXQ_F16) ? (float)(_Float16)v[r] : mxq_round_dt<ADT>(v[r]);
            v[r] = p + b;
        }
    }
    if (tile_inside) {                                       // uniform per workgroup
        const int64_t idx = base + (int64_t)m * N + n;
        if (OUT_DT == MXQ_F32) {
            *reinterpret_cast<v4f*>(reinterpret_cast<float*>(c) + idx) = v;
        } else if (OUT_DT == MXQ_BF16) {
            *reinterpret_cast<u32x2*>(reinterpret_cast<unsigned short*>(c) + idx) =
                u32x2{Pack<MXQ_BF16>::put(v[0], v[1]), Pack<MXQ_BF16>::put(v[2], v[3])};
        } else {
            *reinterpret_cast<u32x2*>(reinterpret_cast<unsigned short*>(c) + idx) =
                u32x2{Pack<MXQ_F16>::put(v[0], v[1]), Pack<MXQ_F16>::put(v[2], v[3])};
        }
    } else if (m < M) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (n + r < N)
                store_scalar<OUT_DT>(c, base + (int64_t)m * N + n + r, mxq_round_dt<ADT>(v[r]));
    }
}

template <int CBSZ, int BLGP, int OUT_DT>
__global__ __launch_bounds__(TPB) void mx_gemm_nt_kernel(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) unsigned char As[GEMM_BM * GEMM_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char Bs[GEMM_BN * GEMM_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char sAs[GEMM_BM * 4];
    __shared__ __attribute__((aligned(16))) unsigned char sBs[GEMM_BN * 4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wy = wave >> 1, wx = wave & 1;
    int tile_m, tile_n;
    tile_of_workgroup(blockIdx.x, gridDim.x, (g.M + GEMM_BM - 1) / GEMM_BM,
                      (g.N + GEMM_BN - 1) / GEMM_BN, &tile_m, &tile_n);
    const int m0 = tile_m * GEMM_BM, n0 = tile_n * GEMM_BN;
    const int64_t bz = blockIdx.y;
    const unsigned char* A = g.a + bz * g.batch_a;
    const unsigned char* B = g.b + bz * g.batch_b;
    const unsigned char* SA = g.sa + bz * g.batch_sa;
    const unsigned char* SB = g.sb + bz * g.batch_sb;
    const int KB = g.K >> 5;                                 // scale bytes per row

    v4f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    // this lane's share of the tile copy: four 16-byte chunks of A and of B per K step
    int ld_row[4], ld_col[4];
    int64_t ga[4], gb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int c = tid + j * TPB;
        ld_row[j] = c >> 3;
        ld_col[j] = (c & 7) * 16;
        const int gm = min(m0 + ld_row[j], g.M - 1);         // rows past the edge are never stored
        const int gn = min(n0 + ld_row[j], g.N - 1);
        ga[j] = (int64_t)gm * g.K + ld_col[j];
        gb[j] = (int64_t)gn * g.K + ld_col[j];
    }
    const int srow = tid & 127;
    const bool s_is_a = tid < 128;
    const int64_t gs = s_is_a ? (int64_t)min(m0 + srow, g.M - 1) * KB
                              : (int64_t)min(n0 + srow, g.N - 1) * KB;

    const int frow = lane & 15, fg = lane >> 4;
    u32x4 va[4], vb[4];
    uint32_t sv;
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            va[j] = *reinterpret_cast<const u32x4*>(A + ga[j] + k0);
            vb[j] = *reinterpret_cast<const u32x4*>(B + gb[j] + k0);
        }
        sv = *reinterpret_cast<const uint32_t*>((s_is_a ? SA : SB) + gs + (k0 >> 5));
    };
    auto stash = [&]() {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<u32x4*>(As + ld_row[j] * GEMM_PITCH + ld_col[j]) = va[j];
            *reinterpret_cast<u32x4*>(Bs + ld_row[j] * GEMM_PITCH + ld_col[j]) = vb[j];
        }
        *reinterpret_cast<uint32_t*>((s_is_a ? sAs : sBs) + srow * 4) = sv;
    };
    // K is walked cyclically from a per-workgroup starting step (see the 256 x 256 kernel)
    const int nk = g.K / GEMM_BK;
    const int kstart = (int)((blockIdx.x * 5u + blockIdx.y) % (unsigned)nk);
    auto kof = [&](int step) { return ((kstart + step) % nk) * GEMM_BK; };
    fetch(kof(0));
    stash();
    __syncthreads();
    for (int step = 0; step < nk; ++step) {
        // next tile (the last step fetches one it does not use: no branches in the loop body, so
        // the instruction order below survives compilation); it arrives while this step computes
        fetch(kof(step + 1));
        __builtin_amdgcn_sched_barrier(0);

        v8i bf[4];
        int sb[4];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            const int n = wx * 64 + tj * 16 + frow;
            bf[tj] = load_frag(Bs + n * GEMM_PITCH + fg * 16);
            sb[tj] = sBs[n * 4 + fg];
        }
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
            const int m = wy * 64 + ti * 16 + frow;
            const v8i af = load_frag(As + m * GEMM_PITCH + fg * 16);
            const int sa = sAs[m * 4 + fg];
#pragma unroll
            for (int tj = 0; tj < 4; ++tj)
                acc[ti][tj] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    bf[tj], af, acc[ti][tj], BLGP, CBSZ, 0, sb[tj], 0, sa);
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();                                     // every wave is done with this tile
        stash();
        __syncthreads();
    }

    const int64_t cbase = bz * g.batch_c;
    const bool inside = m0 + GEMM_BM <= g.M && n0 + GEMM_BN <= g.N && (g.N & 3) == 0;
#pragma unroll
    for (int ti = 0; ti < 4; ++ti)
#pragma unroll
        for (int tj = 0; tj < 4; ++tj)
            store_c4<OUT_DT>(g.c, g.bias, cbase, m0 + wy * 64 + ti * 16 + frow, n0 + wx * 64 + tj * 16 + fg * 4,
                             g.M, g.N, inside, acc[ti][tj]);
}

// ================================================================================================
// Large-tile variant: workgroup tile 256 x 256 x 128, 2 x 2 waves, each wave 128 x 128 = 8 x 8 MFMA
// tiles (256 accumulator registers).  Per K step a wave reads 8 A and 8 B fragments from LDS for 64
// MFMAs, half the LDS traffic per flop of the 128 x 128 kernel.  LDS is double buffered
// (2 x 2 x 256 rows x 144 bytes + scales = 148 KB): the global loads of step k+1 are issued before
// the MFMAs of step k and land in the other buffer afterwards; one barrier per step.
// ================================================================================================
constexpr int G2_BM = 256, G2_BN = 256;
constexpr int G2_TILE_BYTES = G2_BM * GEMM_PITCH;                   // one operand tile
constexpr int G2_STAGE_BYTES = 2 * G2_TILE_BYTES + (G2_BM + G2_BN) * 4;
constexpr int G2_LDS_BYTES = 2 * G2_STAGE_BYTES;

// WM = waves along M (2 or 4); the workgroup has WM x 2 waves and each wave owns (256 / WM) x 128
// outputs.  WM = 4 (512 lanes) halves the accumulators per wave so that two waves fit on every
// SIMD: while one waits for LDS, memory or the barrier, the other keeps the MFMA pipe fed.
template <int CBSZ, int BLGP, int OUT_DT, int WM>
__global__ __launch_bounds__(WM * 128, 1) void mx_gemm_nt_kernel_256(GemmArgs g) {
    constexpr int NT = WM * 128;                        // lanes in the workgroup
    constexpr int TI = 16 / WM;                         // 16-row MFMA tiles per wave along M
    constexpr int CH = 2048 / NT;                       // 16-byte chunks of A (and of B) per lane
    constexpr int ROWS_PER_PASS = NT / 8;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wy = wave >> 1, wx = wave & 1;
    int tile_m, tile_n;
    tile_of_workgroup(blockIdx.x, gridDim.x, (g.M + G2_BM - 1) / G2_BM, (g.N + G2_BN - 1) / G2_BN,
                      &tile_m, &tile_n);
    const int m0 = tile_m * G2_BM, n0 = tile_n * G2_BN;
    const int64_t bz = blockIdx.y;
    const unsigned char* A = g.a + bz * g.batch_a;
    const unsigned char* B = g.b + bz * g.batch_b;
    const unsigned char* SA = g.sa + bz * g.batch_sa;
    const unsigned char* SB = g.sb + bz * g.batch_sb;
    const int KB = g.K >> 5;

    v4f acc[TI][8];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    // tile copy: 256 rows x 8 chunks of 16 bytes per operand, CH chunks of A and CH of B per lane
    // (rows c_row + ROWS_PER_PASS * j).  Rows past the edge are clamped; they are never stored.
    const int c_row = tid >> 3, c_col = (tid & 7) * 16;
    int ra[CH], rb[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        ra[j] = min(m0 + c_row + ROWS_PER_PASS * j, g.M - 1);
        rb[j] = min(n0 + c_row + ROWS_PER_PASS * j, g.N - 1);
    }
    // scales: lanes 0..255 carry a row of A, lanes 256.. (or the same lanes again) a row of B
    const int s_row = tid & 255;
    const bool two_scales = NT == 256;                  // every lane loads both
    const bool s_is_b = tid >= 256;
    const unsigned char* psa = SA + (int64_t)min(m0 + s_row, g.M - 1) * KB;
    const unsigned char* psb = SB + (int64_t)min(n0 + s_row, g.N - 1) * KB;
    const int st_off = c_row * GEMM_PITCH + c_col;

    const int frow = lane & 15, fg = lane >> 4;
    const int a_off = (wy * (TI * 16) + frow) * GEMM_PITCH + fg * 16;
    const int b_off = G2_TILE_BYTES + (wx * 128 + frow) * GEMM_PITCH + fg * 16;
    const int sa_off = 2 * G2_TILE_BYTES + (wy * (TI * 16) + frow) * 4 + fg;
    const int sb_off = 2 * G2_TILE_BYTES + G2_BM * 4 + (wx * 128 + frow) * 4 + fg;

    u32x4 va[CH], vb[CH];
    uint32_t vsa = 0, vsb = 0;
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            va[j] = *reinterpret_cast<const u32x4*>(A + (int64_t)ra[j] * g.K + (k0 + c_col));
            vb[j] = *reinterpret_cast<const u32x4*>(B + (int64_t)rb[j] * g.K + (k0 + c_col));
        }
        if (two_scales) {
            vsa = *reinterpret_cast<const uint32_t*>(psa + (k0 >> 5));
            vsb = *reinterpret_cast<const uint32_t*>(psb + (k0 >> 5));
        } else {
            vsa = *reinterpret_cast<const uint32_t*>((s_is_b ? psb : psa) + (k0 >> 5));
        }
    };
    auto stash_rows = [&](unsigned char* stage, int j) {      // chunk j of A and of B
        *reinterpret_cast<u32x4*>(stage + st_off + ROWS_PER_PASS * j * GEMM_PITCH) = va[j];
        *reinterpret_cast<u32x4*>(stage + G2_TILE_BYTES + st_off + ROWS_PER_PASS * j * GEMM_PITCH) = vb[j];
    };
    auto stash_scales = [&](unsigned char* stage) {
        if (two_scales) {
            *reinterpret_cast<uint32_t*>(stage + 2 * G2_TILE_BYTES + s_row * 4) = vsa;
            *reinterpret_cast<uint32_t*>(stage + 2 * G2_TILE_BYTES + G2_BM * 4 + s_row * 4) = vsb;
        } else {
            *reinterpret_cast<uint32_t*>(stage + 2 * G2_TILE_BYTES + (s_is_b ? G2_BM * 4 : 0) + s_row * 4) = vsa;
        }
    };

    // Every workgroup walks K cyclically from its own starting step.  Rows are K bytes apart, so
    // with K a power of two a given K slice of *every* row sits in the same L2 channel; staggering
    // the start spreads the slices in flight at any moment over all channels.
    const int nk = g.K / GEMM_BK;
    const int kstart = (int)((blockIdx.x * 5u + blockIdx.y) % (unsigned)nk);
    auto kof = [&](int step) { return ((kstart + step) % nk) * GEMM_BK; };

    fetch(kof(0));
#pragma unroll
    for (int j = 0; j < CH; ++j) stash_rows(lds, j);
    stash_scales(lds);
    __syncthreads();

    int buf = 0;
    for (int step = 0; step < nk; ++step) {
        const unsigned char* cur = lds + buf * G2_STAGE_BYTES;
        unsigned char* nxt = lds + (buf ^ 1) * G2_STAGE_BYTES;   // nobody reads it during this step
        // Fetch the next tile now; it is in flight during the MFMAs below.  The last step fetches
        // one more (unused) tile and stores it into the idle buffer: keeping the loop body free of
        // branches is what lets the instruction order below survive compilation.
        fetch(kof(step + 1));

        v8i af[TI];
        int sa[TI];
#pragma unroll
        for (int ti = 0; ti < TI; ++ti) {
            af[ti] = load_frag(cur + a_off + ti * 16 * GEMM_PITCH);
            sa[ti] = cur[sa_off + ti * 64];
        }
        __builtin_amdgcn_sched_barrier(0);                   // keep the global loads up here
        v8i bf = load_frag(cur + b_off);
        int sb = cur[sb_off];
#pragma unroll
        for (int tj = 0; tj < 8; ++tj) {
            // the next B fragment is read in the shadow of this fragment's MFMAs
            v8i bf_next = bf;
            int sb_next = sb;
            if (tj + 1 < 8) {
                bf_next = load_frag(cur + b_off + (tj + 1) * 16 * GEMM_PITCH);
                sb_next = cur[sb_off + (tj + 1) * 64];
            }
#pragma unroll
            for (int ti = 0; ti < TI; ++ti)
                acc[ti][tj] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    bf, af[ti], acc[ti][tj], BLGP, CBSZ, 0, sb, 0, sa[ti]);
            // second half of the step: the tile fetched at its top has had time to arrive; its LDS
            // writes go out in the shadow of the remaining MFMAs
            if (tj >= 4) {
#pragma unroll
                for (int j = (tj - 4) * CH / 4; j < (tj - 3) * CH / 4; ++j) stash_rows(nxt, j);
            }
            if (tj == 7) stash_scales(nxt);
            __builtin_amdgcn_sched_barrier(0);
            bf = bf_next;
            sb = sb_next;
        }
        __syncthreads();
        buf ^= 1;
    }

    const int64_t cbase = bz * g.batch_c;
    const bool inside = m0 + G2_BM <= g.M && n0 + G2_BN <= g.N && (g.N & 3) == 0;
#pragma unroll
    for (int ti = 0; ti < TI; ++ti)
#pragma unroll
        for (int tj = 0; tj < 8; ++tj)
            store_c4<OUT_DT>(g.c, g.bias, cbase, m0 + wy * (TI * 16) + ti * 16 + frow,
                             n0 + wx * 128 + tj * 16 + fg * 4, g.M, g.N, inside, acc[ti][tj]);
}

// Register-resident MFMA loop: every wave issues `iters` x 16 independent scaled MFMAs on operands
// it never reloads.  Its rate is the practical ceiling of the matrix pipes under this instruction
// (datasheet: 5 PFLOP/s dense fp8).  `sink` only keeps the compiler from deleting the loop.
__global__ __launch_bounds__(TPB) void mfma_rate_probe_kernel(int iters, float* sink) {
    v8i a = {(int)threadIdx.x, 1, 2, 3, 4, 5, 6, 7}, b = {7, 6, 5, 4, 3, 2, 1, (int)blockIdx.x};
    v4f acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[i], 0, 0, 0, 127, 0, 127);
    }
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) t += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (t == 12345.678f) sink[0] = t;
}

}  // namespace
