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
    int M, N, K;
    int64_t batch_a, batch_sa, batch_b, batch_sb, batch_c;   // element strides between batches
};

// a lane's MFMA operand: 16 codes at p (K = 16g ..) and 16 codes at p + 64 (K = 64 + 16g ..)
__device__ __forceinline__ v8i load_frag(const unsigned char* p) {
    const u32x4 lo = *reinterpret_cast<const u32x4*>(p);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(p + 64);
    return v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
}

template <int CBSZ, int BLGP, int OUT_DT>
__global__ __launch_bounds__(TPB) void mx_gemm_nt_kernel(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) unsigned char As[GEMM_BM * GEMM_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char Bs[GEMM_BN * GEMM_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char sAs[GEMM_BM * 4];
    __shared__ __attribute__((aligned(16))) unsigned char sBs[GEMM_BN * 4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wy = wave >> 1, wx = wave & 1;
    const int m0 = blockIdx.y * GEMM_BM, n0 = blockIdx.x * GEMM_BN;
    const int64_t bz = blockIdx.z;
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
    for (int k0 = 0; k0 < g.K; k0 += GEMM_BK) {
        u32x4 va[4], vb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            va[j] = *reinterpret_cast<const u32x4*>(A + ga[j] + k0);
            vb[j] = *reinterpret_cast<const u32x4*>(B + gb[j] + k0);
        }
        const uint32_t sv = *reinterpret_cast<const uint32_t*>((s_is_a ? SA : SB) + gs + (k0 >> 5));
        __syncthreads();                                     // previous step's reads are done
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<u32x4*>(As + ld_row[j] * GEMM_PITCH + ld_col[j]) = va[j];
            *reinterpret_cast<u32x4*>(Bs + ld_row[j] * GEMM_PITCH + ld_col[j]) = vb[j];
        }
        *reinterpret_cast<uint32_t*>((s_is_a ? sAs : sBs) + srow * 4) = sv;
        __syncthreads();

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
                    af, bf[tj], acc[ti][tj], CBSZ, BLGP, 0, sa, 0, sb[tj]);
        }
    }

    // D[4 * (lane / 16) + r][lane % 16] of every 16 x 16 tile
    const int64_t cbase = bz * g.batch_c;
#pragma unroll
    for (int ti = 0; ti < 4; ++ti)
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            const int n = n0 + wx * 64 + tj * 16 + frow;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + wy * 64 + ti * 16 + fg * 4 + r;
                if (m < g.M && n < g.N)
                    store_scalar<OUT_DT>(g.c, cbase + (int64_t)m * g.N + n,
                                         mxq_round_dt<Arith<OUT_DT>::DT_>(acc[ti][tj][r]));
            }
        }
}

}  // namespace
