// Packed MX tensors and the scaled-MFMA GEMM that consumes them (gfx950).
//
// Packed form of a (rows, K) tensor quantized along K in blocks of 32:
//   codes  uint8 (rows, K)      one OCP 8-bit float per element: e4m3 ("fn") for the element
//                               formats fp8_e4m3 / fp6_e3m2 / fp6_e2m3 / fp4_e2m1 (all of whose
//                               values e4m3 represents exactly), e5m2 for fp8_e5m2
//          or uint8 (rows, K/2) fp4_e2m1 elements as OCP e2m1 nibbles, the element with the lower K
//                               index in the low nibble
//   scales uint8 (rows, K/32)   E8M0: shared exponent + 127, 255 = NaN block
// codes[i][k] * 2^(scales[i][k/32] - 127) is bit-for-bit the value the fake-quantizing kernels
// return (before their final rounding to a 16-bit tensor dtype).
//
// v_mfma_scale_f32_16x16x128_f8f6f4 multiplies a 16x128 by a 128x16 tile of such codes.  Lane
// (row = lane % 16, g = lane / 16) supplies 32 8-bit codes of its row: K = 16g .. 16g+15 in its
// first four registers and K = 64+16g .. 64+16g+15 in the last four -- or 32 nibbles, K = 32g ..
// 32g+31, in four registers.  The E8M0 byte of K block j (32 consecutive K) of a row is taken
// from the scale register of lane row + 16j -- so each lane passes the scale of block g, and block
// scaling costs nothing extra.  v_mfma_scale_f32_32x32x64_f8f6f4 (the large-tile kernel) is the
// same with lane (row = lane % 32, g = lane / 32): K = 16g .. and 32+16g .., or nibbles 32g ..,
// scale of block j from lane row + 32j.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxq_gemm_addr.h"
#include "mxq_kernels.h"

namespace {

// ================================================================================================
// quantize + pack, shared axis innermost, block size 32
// ================================================================================================
// KIND of the codes (the operand format numbers of the scaled MFMA): 0 = OCP e4m3 bytes, 1 = OCP e5m2
// bytes, 2 = OCP e2m3 and 3 = OCP e3m2 6-bit codes (a little-endian bit stream: element j of a row
// in bits 6 j .. 6 j + 5, four elements in three bytes), 4 = OCP e2m1 nibbles (two per byte, the
// element with the lower K index in the low nibble)
template <int KIND>
__device__ __forceinline__ uint32_t mx_encode(float y) {
    if (KIND == 1) return mxq_encode_e5m2(y);
    if (KIND == 2) return mxq_encode_fp6<3, 1>(y);
    if (KIND == 3) return mxq_encode_fp6<2, 3>(y);
    if (KIND == 4) return mxq_encode_e2m1(y);
    return mxq_encode_e4m3(y);
}
template <int KIND>
constexpr int code_bits() { return KIND == 4 ? 4 : (KIND == 2 || KIND == 3) ? 6 : 8; }

// One element of a block as its code.  DIRECT: the element format is the format of the codes
// (fp8_e4m3 in e4m3 bytes, fp4 in nibbles, ...) and the code comes straight from the rounded
// significand (about a third fewer instructions; the pack kernels are instruction bound);
// otherwise the element is rounded to its float value, which is then encoded (fp6 / fp4 elements in
// e4m3 bytes; the round-up-zone variants).
template <int RMODE, int ADT, bool ZONE_ELEM, int KIND, bool DIRECT>
__device__ __forceinline__ uint32_t mx_code_of(float x, const MxqScale& sc, const MxParams& p,
                                               const unsigned char* zone, int zs, uint32_t max_code) {
    if constexpr (DIRECT) {
        return mxq_quant_mx_code<RMODE, ADT, code_bits<KIND>() - 1>(x, sc, p.fmt, max_code);
    } else {
        return mx_encode<KIND>(mxq_quant_mx_elem_unscaled<RMODE, ADT, ZONE_ELEM>(x, sc, p.fmt, zone, zs));
    }
}

template <int DT, int RMODE, bool ZONE_ELEM, int KIND, int UNROLL, bool DIRECT>
__global__ __launch_bounds__(TPB) void mx_pack_kernel(const u32x4* __restrict__ in,
                                                      void* __restrict__ codes_,
                                                      unsigned char* __restrict__ scales,
                                                      int64_t n_vec, MxParams p, uint32_t max_code) {
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
        if constexpr (DT == MXQ_BF16) {
            if (p.pre_nan_from != 0u) {                    // uniform: the bfloat16 quantizer first
                const unsigned short span = (unsigned short)((p.pre_nan_from >> 16) - 0x0080u);
#pragma unroll
                for (int j = 0; j < UNROLL; ++j) {
                    // plain range (normal numbers below the NaN threshold) in the whole wave: "odd
                    // significand -> + 1" on both halves of a dword at once; else element by element
                    u16x2 worst = {0, 0};
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                        worst = __builtin_elementwise_max(
                            worst, __builtin_bit_cast(u16x2, v[j][d] & 0x7FFF7FFFu) - u16x2{0x0080, 0x0080});
                    if (__all(worst[0] < span && worst[1] < span)) {
#pragma unroll
                        for (int d = 0; d < 4; ++d) v[j][d] += v[j][d] & 0x00010001u;
                    } else {
#pragma unroll
                        for (int d = 0; d < 4; ++d)
                            v[j][d] = Pack<MXQ_BF16>::put(
                                mxq_quant_bf16_to_bfloat16_nearest(Pack<MXQ_BF16>::get(v[j][d], 0), p.pre_nan_from),
                                mxq_quant_bf16_to_bfloat16_nearest(Pack<MXQ_BF16>::get(v[j][d], 1), p.pre_nan_from));
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + j * TPB;
            const uint32_t um = group_max<LPT>(vec_abs_max<DT>(v[j]));
            const MxqScale sc = mxq_block_scale(um, p.emax, p.scale_emax, p.flush != 0, zone, ZS);
            uint32_t out[PD] = {};
            uint64_t six = 0;                              // 6-bit codes: 24 (fp32 in) or 48 bits per lane
#pragma unroll
            for (int d = 0; d < 4; ++d)
#pragma unroll
                for (int h = 0; h < PD; ++h) {
                    const uint32_t c = mx_code_of<RMODE, ADT, ZONE_ELEM, KIND, DIRECT>(
                        Pack<DT>::get(v[j][d], h), sc, p, zone, ZS, max_code);
                    const int e = d * PD + h;              // element index inside the vector
                    if (code_bits<KIND>() == 6) six |= (uint64_t)c << (6 * e);
                    else if (KIND == 4) out[0] |= c << (4 * e);
                    else out[e / 4] |= c << (8 * (e % 4));
                }
            if constexpr (code_bits<KIND>() == 6) {
                // 16 elements = 12 bytes: the first of 2 (4) neighbouring lanes collects and stores them
                uint32_t w0, w1, w2;
                if (PD == 2) {
                    const uint64_t hi = __shfl_down(six, 1, 64);
                    w0 = (uint32_t)six;
                    w1 = (uint32_t)(six >> 32) | ((uint32_t)hi << 16);
                    w2 = (uint32_t)(hi >> 16);
                } else {
                    const uint32_t b0 = (uint32_t)six, b1 = (uint32_t)__shfl_down(six, 1, 64),
                                   b2 = (uint32_t)__shfl_down(six, 2, 64), b3 = (uint32_t)__shfl_down(six, 3, 64);
                    w0 = b0 | (b1 << 24);
                    w1 = (b1 >> 8) | (b2 << 16);
                    w2 = (b2 >> 16) | (b3 << 8);
                }
                if (i < n_vec && (threadIdx.x & (4 / PD - 1)) == 0) {
                    uint32_t* dst = reinterpret_cast<uint32_t*>(reinterpret_cast<unsigned char*>(codes_) + i * (3 * PD));
                    dst[0] = w0;
                    dst[1] = w1;
                    dst[2] = w2;
                }
                if (i < n_vec && (threadIdx.x & (LPT - 1)) == 0)
                    scales[i / LPT] = (unsigned char)mxq_encode_e8m0(sc.scale);
            } else if (i < n_vec) {
                if (KIND == 4) {
                    if (PD == 1) reinterpret_cast<unsigned short*>(codes_)[i] = (unsigned short)out[0];
                    else reinterpret_cast<uint32_t*>(codes_)[i] = out[0];
                } else if (PD == 1) reinterpret_cast<uint32_t*>(codes_)[i] = out[0];
                else reinterpret_cast<u32x2*>(codes_)[i] = u32x2{out[0], out[PD - 1]};
                if ((threadIdx.x & (LPT - 1)) == 0)
                    scales[i / LPT] = (unsigned char)mxq_encode_e8m0(sc.scale);
            }
        }
    }
}

// ================================================================================================
// quantize + pack + transpose: input (pre, R, C) with the shared axis = R (blocks of 32 rows, the
// second-to-last axis), output codes (pre, C, R) and scales (pre, C, R / 32) -- the K-major operand
// the GEMM wants when the contraction runs over R (gradients: x^T, grad_output^T, W^T).
// A lane keeps a 32-row x 8-byte column strip in registers (like mx_strided_tile_kernel), which
// gives, per column, the 32 codes of one block: 32 (16, 24) contiguous bytes of the output.  The
// four waves of a workgroup take four consecutive blocks of the same 64 column strips and hand
// their codes over through LDS, so that a column leaves as one 128 (64, 96) byte piece and its four
// scale bytes as one word.
// Work: blockIdx.x = (pre_i * n_tgroups + tile group) * n_cgroups + column group.
// ================================================================================================
constexpr int PACKT_TILES = TPB / 64;                   // blocks of 32 rows per workgroup
static_assert(PACKT_TILES == 4, "the scale bytes of a column's blocks travel as one 32-bit word");

template <int DT, int RMODE, bool ZONE_ELEM, int KIND, bool DIRECT>
__global__ __launch_bounds__(TPB) void mx_pack_t_kernel(const u32x2* __restrict__ in,
                                                        unsigned char* __restrict__ codes,
                                                        unsigned char* __restrict__ scales,
                                                        int64_t n_cgroups, int64_t n_tiles, int64_t pv,
                                                        MxParams p, uint32_t max_code) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int VW = Col8<DT>::VW;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int ROWS = 32;
    constexpr int NCOL = 64 * VW;                        // columns of a workgroup
    constexpr int UPT = ROWS * code_bits<KIND>() / 64;   // 8-byte units of codes per block and column
    constexpr int UPC = PACKT_TILES * UPT;               // ... per column of the workgroup
    constexpr int LDC = UPC + 1;                         // padded column pitch in LDS
    __shared__ unsigned char zone[ZONE_PAD];
    constexpr int HV = VW / 2;                           // columns of a lane per hand-over
    __shared__ u32x2 stage[(NCOL / 2) * LDC];
    __shared__ uint32_t stage_scales[NCOL];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t n_tgroups = (n_tiles + PACKT_TILES - 1) / PACKT_TILES;
    const int64_t cg = blockIdx.x % n_cgroups, rest = blockIdx.x / n_cgroups;
    const int64_t tg = rest % n_tgroups, pre_i = rest / n_tgroups;
    const int64_t c = cg * 64 + lane;                               // column strip
    const int64_t tile_i = tg * PACKT_TILES + wave;
    const bool live = c < pv && tile_i < n_tiles;
    const int64_t off0 = live ? ((pre_i * n_tiles + tile_i) * ROWS) * pv + c : 0;   // in units of 8 bytes

    u32x2 raw[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) raw[r] = live ? in[off0 + (int64_t)r * pv] : u32x2{0, 0};
    load_zone(zone, g_zone_tables[p.zone_row]);

    uint32_t um[VW];
#pragma unroll
    for (int k = 0; k < VW; ++k) um[k] = 0;
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int d = 0; d < 2; ++d)
#pragma unroll
            for (int h = 0; h < PD; ++h)
                um[d * PD + h] = max(um[d * PD + h], abs_bits(Pack<DT>::get(raw[r][d], h)));

    // hand-over in two halves (the lane's first VW / 2 columns, then the rest) so that the staging
    // area is half the size and twice as many workgroups fit a CU: consecutive lanes write
    // consecutive 8-byte units of a column
    const int64_t C = pv * VW;
    const int64_t col0 = cg * NCOL;
    const int64_t t0 = tg * PACKT_TILES;
    const int live_tiles = (n_tiles - t0 < PACKT_TILES) ? (int)(n_tiles - t0) : PACKT_TILES;
    const int live_units = live_tiles * UPT;
    const int64_t col_bytes = n_tiles * (UPT * 8);                  // bytes of codes per output column
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int kk = 0; kk < HV; ++kk) {
            const int k = half * HV + kk;
            const MxqScale sc = mxq_block_scale(um[k], p.emax, p.scale_emax, p.flush != 0, zone, ZS);
            uint32_t out[8] = {};
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const uint32_t code = mx_code_of<RMODE, ADT, ZONE_ELEM, KIND, DIRECT>(
                    Pack<DT>::get(raw[r][k / PD], k % PD), sc, p, zone, ZS, max_code);
                if (code_bits<KIND>() == 6) {
                    out[(6 * r) >> 5] |= code << ((6 * r) & 31);
                    if (((6 * r) & 31) > 26) out[((6 * r) >> 5) + 1] |= code >> (32 - ((6 * r) & 31));
                } else if (KIND == 4) out[r / 8] |= code << (4 * (r % 8));
                else out[r / 4] |= code << (8 * (r % 4));
            }
            u32x2* dst = stage + (lane * HV + kk) * LDC + wave * UPT;
#pragma unroll
            for (int u = 0; u < UPT; ++u) dst[u] = u32x2{out[2 * u], out[2 * u + 1]};
            reinterpret_cast<unsigned char*>(stage_scales)[(lane * VW + k) * PACKT_TILES + wave] =
                (unsigned char)mxq_encode_e8m0(sc.scale);
        }
        __syncthreads();
        for (int q = threadIdx.x; q < (NCOL / 2) * UPC; q += TPB) {
            const int cb = q / UPC, u = q % UPC;                    // cb = lane * HV + kk
            const int64_t col = col0 + (cb / HV) * VW + half * HV + (cb % HV);
            if (u < live_units && col < C) {
                u32x2* dst = reinterpret_cast<u32x2*>(codes + (pre_i * C + col) * col_bytes + t0 * (UPT * 8));
                dst[u] = stage[cb * LDC + u];
            }
        }
        __syncthreads();                                            // the staging area is reused
    }
    for (int cb = threadIdx.x; cb < NCOL; cb += TPB) {
        if (col0 + cb < C) {
            unsigned char* dst = scales + (pre_i * C + col0 + cb) * n_tiles + t0;
            const uint32_t word = stage_scales[cb];
            if (live_tiles == PACKT_TILES && (reinterpret_cast<uintptr_t>(dst) & 3) == 0) {
                *reinterpret_cast<uint32_t*>(dst) = word;
            } else {
                for (int t = 0; t < live_tiles; ++t) dst[t] = (unsigned char)(word >> (8 * t));
            }
        }
    }
}

// unpack: codes * 2^(scale-127) -> fp32 / bf16 / fp16 (for tests and for callers that want the
// fake-quantized view of a packed tensor)
template <int DT, int KIND>
__global__ __launch_bounds__(TPB) void mx_unpack_kernel(const unsigned char* __restrict__ codes,
                                                        const unsigned char* __restrict__ scales,
                                                        void* __restrict__ out, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
        const uint32_t s = scales[i >> 5];
        float y;
        if (code_bits<KIND>() == 6) {
            const int64_t bit = 6 * i;
            const uint32_t two = codes[bit >> 3] | ((uint32_t)codes[(bit >> 3) + ((bit & 7) > 2)] << 8);
            const uint32_t c6 = (two >> (bit & 7)) & 63u;
            y = (KIND == 2) ? mxq_decode_fp6<3, 1>(c6) : mxq_decode_fp6<2, 3>(c6);
        } else if (KIND == 4) y = mxq_decode_e2m1((codes[i >> 1] >> (4 * (i & 1))) & 15u);
        else y = (KIND == 1) ? mxq_decode_e5m2(codes[i]) : mxq_decode_e4m3(codes[i]);
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
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int GEMM_BM = 128, GEMM_BN = 128, GEMM_BK = 128, GEMM_PITCH = GEMM_BK + 16;
static_assert(GEMM_BK == mxq_addr::BK, "the address helpers assume 128-byte K steps");

struct GemmArgs {
    const unsigned char* a;
    const unsigned char* sa;
    const unsigned char* b;
    const unsigned char* sb;
    void* c;
    const void* bias;     // optional (N), dtype of C: C = round(round(A x B^T) + bias)
    uint32_t q_nan_from;  // 0: no output quantization.  Else C is bf16 and is quantized to bfloat16,
                          // round-half-away, after the product and again after the bias add (the
                          // closed form mxq_quant_bf16_to_bfloat16_nearest with this threshold)
    int M, N, K;
    int kbytes;           // bytes of codes per row: K (8-bit codes) or K / 2 (e2m1 nibbles)
    int k_splits;         // small-tile kernel: workgroups along gridDim.z share the K steps of a tile and
                          // each write an fp32 partial tile (split z of batch b at ((z * batch + b) M N)
    int64_t batch_a, batch_sa, batch_b, batch_sb, batch_c;   // strides between batches (bytes / elements of C)
};

// which output tile a workgroup computes (XCD-aware order), and the address arithmetic of the tile copies
using mxq_addr::tile_of_workgroup;

// a lane's MFMA operand: 16 codes at p (K = 16g ..) and 16 codes at p + 64 (K = 64 + 16g ..)
__device__ __forceinline__ v8i load_frag(const unsigned char* p) {
    const u32x4 lo = *reinterpret_cast<const u32x4*>(p);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(p + 64);
    return v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
}

// One K = 128 MFMA.  e2m1 operands (CBSZ = BLGP = 4) are 16 bytes per lane: the fragment a lane reads
// for a 128-byte K step (16 bytes at p, 16 at p + 64) then holds the operands of *two* MFMAs, K
// 0..127 in registers 0-3 (HALF = 0) and K 128..255 in registers 4-7 (HALF = 1).
template <int CBSZ, int BLGP, int HALF>
__device__ __forceinline__ v4f mx_mfma(const v8i& b, const v8i& a, v4f c, int sb, int sa) {
    if constexpr (CBSZ == 4) {
        const v8i b4 = {b[4 * HALF], b[4 * HALF + 1], b[4 * HALF + 2], b[4 * HALF + 3], 0, 0, 0, 0};
        const v8i a4 = {a[4 * HALF], a[4 * HALF + 1], a[4 * HALF + 2], a[4 * HALF + 3], 0, 0, 0, 0};
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b4, a4, c, 4, 4, 0, sb, 0, sa);
    } else {
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b, a, c, BLGP, CBSZ, 0, sb, 0, sa);
    }
}

// One 32 x 32 x 64 MFMA: operand registers and scale byte of MFMA h of a K step out of the four
// 16-byte reads r[0..3] of a lane (lane (i, g) reads the 16-byte columns 2 q + g, q = 0..3, of its
// row).  `sb`, `sa` hold the row's scale bytes shifted so that this lane's block comes first; op_sel
// picks byte 0 or 2.  Used by the attention-score kernel, whose K is a single step.
template <int CBSZ, int BLGP, class Frag, class Scales>
__device__ __forceinline__ v16f mx_mfma32(const Frag& b, const Frag& a, v16f c, const Scales& sb,
                                          const Scales& sa, int h) {
    if constexpr (CBSZ == 4) {
#define MXQ_MMA4(H)                                                                                       \
    __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(                                                      \
        v8i{(int)b.r[H][0], (int)b.r[H][1], (int)b.r[H][2], (int)b.r[H][3], 0, 0, 0, 0},                  \
        v8i{(int)a.r[H][0], (int)a.r[H][1], (int)a.r[H][2], (int)a.r[H][3], 0, 0, 0, 0}, c, 4, 4,          \
        ((H) & 1) * 2, sb.w[(H) >> 1], ((H) & 1) * 2, sa.w[(H) >> 1])
        return h == 0 ? MXQ_MMA4(0) : h == 1 ? MXQ_MMA4(1) : h == 2 ? MXQ_MMA4(2) : MXQ_MMA4(3);
#undef MXQ_MMA4
    } else {
#define MXQ_MMA8(H)                                                                                       \
    __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(                                                      \
        v8i{(int)b.r[2 * H][0], (int)b.r[2 * H][1], (int)b.r[2 * H][2], (int)b.r[2 * H][3],               \
            (int)b.r[2 * H + 1][0], (int)b.r[2 * H + 1][1], (int)b.r[2 * H + 1][2], (int)b.r[2 * H + 1][3]}, \
        v8i{(int)a.r[2 * H][0], (int)a.r[2 * H][1], (int)a.r[2 * H][2], (int)a.r[2 * H][3],               \
            (int)a.r[2 * H + 1][0], (int)a.r[2 * H + 1][1], (int)a.r[2 * H + 1][2], (int)a.r[2 * H + 1][3]}, \
        c, BLGP, CBSZ, (H) * 2, sb.w[0], (H) * 2, sa.w[0])
        return h == 0 ? MXQ_MMA8(0) : MXQ_MMA8(1);
#undef MXQ_MMA8
    }
}

// The same MFMA from the part of either fragment that it reads: two 16-byte pieces of a lane's row
// (8-bit codes) or one (nibbles), so that the large-tile kernel holds half fragments only.
template <class Half> struct QOF { static constexpr int Q = sizeof(Half) / 16; };
template <int CBSZ, int BLGP, class Half, class Scales>
__device__ __forceinline__ v16f mx_mfma32_half(const Half& b, const Half& a, v16f c, const Scales& sb,
                                               const Scales& sa, int h) {
    if constexpr (CBSZ == 4) {
#define MXQ_MMA4H(H)                                                                                      \
    __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(                                                      \
        v8i{(int)b.r[0][0], (int)b.r[0][1], (int)b.r[0][2], (int)b.r[0][3], 0, 0, 0, 0},                  \
        v8i{(int)a.r[0][0], (int)a.r[0][1], (int)a.r[0][2], (int)a.r[0][3], 0, 0, 0, 0}, c, 4, 4,          \
        ((H) & 1) * 2, sb.w[(H) >> 1], ((H) & 1) * 2, sa.w[(H) >> 1])
        return h == 0 ? MXQ_MMA4H(0) : h == 1 ? MXQ_MMA4H(1) : h == 2 ? MXQ_MMA4H(2) : MXQ_MMA4H(3);
#undef MXQ_MMA4H
    } else {
#define MXQ_MMA8H(H)                                                                                      \
    __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(                                                      \
        v8i{(int)b.r[0][0], (int)b.r[0][1], (int)b.r[0][2], (int)b.r[0][3],                               \
            (int)b.r[QOF<Half>::Q - 1][0], (int)b.r[QOF<Half>::Q - 1][1], (int)b.r[QOF<Half>::Q - 1][2], (int)b.r[QOF<Half>::Q - 1][3]}, \
        v8i{(int)a.r[0][0], (int)a.r[0][1], (int)a.r[0][2], (int)a.r[0][3],                               \
            (int)a.r[QOF<Half>::Q - 1][0], (int)a.r[QOF<Half>::Q - 1][1], (int)a.r[QOF<Half>::Q - 1][2], (int)a.r[QOF<Half>::Q - 1][3]}, \
        c, BLGP, CBSZ, (H) * 2, sb.w[0], (H) * 2, sa.w[0])
        return h == 0 ? MXQ_MMA8H(0) : MXQ_MMA8H(1);
#undef MXQ_MMA8H
    }
}

// Output tiles are written once and not read again by the kernel: streaming stores keep them from
// displacing the operand panels in L2 (3-5 % on the large shapes).
#define MXQ_C_STORE(ptr, val) __builtin_nontemporal_store(val, ptr)
// The MFMAs are issued with the B fragment as the first operand, i.e. they compute 16 x 16 blocks
// of C^T: a lane then holds four *consecutive columns* n = 4 * (lane / 16) + r of one row
// m = lane % 16, which it can store with a single 8- or 16-byte access.
// What the layers do as separate tensor ops after the product: round it to the tensor dtype,
// (quantize,) add the bias, round again (, quantize again).  The last rounding to the dtype is left
// to the store when nothing follows it.
template <int OUT_DT>
__device__ __forceinline__ float epilogue_value(float acc, bool has_bias, float b, uint32_t q_nan_from) {
    constexpr int ADT = Arith<OUT_DT>::DT_;
    if (!has_bias && q_nan_from == 0u) return acc;
    float p = (OUT_DT == MXQ_F16) ? (float)(_Float16)acc : mxq_round_dt<ADT>(acc);
    if (OUT_DT == MXQ_BF16 && q_nan_from != 0u) p = mxq_quant_bf16_to_bfloat16_nearest(p, q_nan_from);
    if (has_bias) {
        p += b;
        if (OUT_DT == MXQ_BF16 && q_nan_from != 0u)
            p = mxq_quant_bf16_to_bfloat16_nearest(mxq_round_dt<ADT>(p), q_nan_from);
    }
    return p;
}

template <int OUT_DT>
__device__ __forceinline__ void store_c4(void* c, const void* bias, uint32_t q_nan_from, int64_t base,
                                         int m, int n, int M, int N, bool tile_inside, v4f v) {
    constexpr int ADT = Arith<OUT_DT>::DT_;
    if (bias != nullptr || q_nan_from != 0u) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float b = (bias != nullptr && n + r < N) ? load_scalar<OUT_DT>(bias, n + r) : 0.0f;
            v[r] = epilogue_value<OUT_DT>(v[r], bias != nullptr, b, q_nan_from);
        }
    }
    if (tile_inside) {                                       // uniform per workgroup
        const int64_t idx = base + (int64_t)m * N + n;
        if (OUT_DT == MXQ_F32) {
            MXQ_C_STORE(reinterpret_cast<v4f*>(reinterpret_cast<float*>(c) + idx), v);
        } else if (OUT_DT == MXQ_BF16) {
            MXQ_C_STORE(reinterpret_cast<u32x2*>(reinterpret_cast<unsigned short*>(c) + idx),
                        (u32x2{Pack<MXQ_BF16>::put(v[0], v[1]), Pack<MXQ_BF16>::put(v[2], v[3])}));
        } else {
            MXQ_C_STORE(reinterpret_cast<u32x2*>(reinterpret_cast<unsigned short*>(c) + idx),
                        (u32x2{Pack<MXQ_F16>::put(v[0], v[1]), Pack<MXQ_F16>::put(v[2], v[3])}));
        }
    } else if (m < M) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (n + r < N)
                store_scalar<OUT_DT>(c, base + (int64_t)m * N + n + r, mxq_round_dt<ADT>(v[r]));
    }
}

// Eight consecutive columns of one row, 16-bit outputs: one 16-byte store (and bias load).
template <int OUT_DT>
__device__ __forceinline__ void store_c8(void* c, const void* bias, uint32_t q_nan_from, int64_t base,
                                         int m, int n, int M, int N, bool tile_inside, v4f lo, v4f hi) {
    constexpr int ADT = Arith<OUT_DT>::DT_;
    float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (tile_inside) {                                       // uniform per workgroup
        if (bias != nullptr) {
            const u32x4 bw = *reinterpret_cast<const u32x4*>(reinterpret_cast<const unsigned short*>(bias) + n);
#pragma unroll
            for (int r = 0; r < 8; ++r)
                v[r] = epilogue_value<OUT_DT>(v[r], true, Pack<OUT_DT>::get(bw[r >> 1], r & 1), q_nan_from);
        } else if (q_nan_from != 0u) {
#pragma unroll
            for (int r = 0; r < 8; ++r) v[r] = epilogue_value<OUT_DT>(v[r], false, 0.0f, q_nan_from);
        }
        MXQ_C_STORE(reinterpret_cast<u32x4*>(reinterpret_cast<unsigned short*>(c) + base + (int64_t)m * N + n),
                    (u32x4{Pack<OUT_DT>::put(v[0], v[1]), Pack<OUT_DT>::put(v[2], v[3]),
                           Pack<OUT_DT>::put(v[4], v[5]), Pack<OUT_DT>::put(v[6], v[7])}));
    } else if (m < M) {
#pragma unroll
        for (int r = 0; r < 8; ++r)
            if (n + r < N) {
                const float b = bias != nullptr ? load_scalar<OUT_DT>(bias, n + r) : 0.0f;
                const float x = epilogue_value<OUT_DT>(v[r], bias != nullptr, b, q_nan_from);
                store_scalar<OUT_DT>(c, base + (int64_t)m * N + n + r, mxq_round_dt<ADT>(x));
            }
    }
}

// Epilogue of eight consecutive columns n .. n + 7 of one row, packed to a 16-bit output type
// (inside tiles only: n + 7 < N, bias 16-byte aligned at n).
// With the bfloat16 quantization (q_nan_from != 0) the plain range is tried first: while every value
// the wave handles in this call -- the rounded products and, with a bias, the rounded sums -- is a
// normal number below the NaN threshold, the quantizer is "odd significand -> + 1" on both halves of a
// dword at once (convert, range check with packed 16-bit subtract / max, add: three to four
// instructions per value against a dozen per quantization, which bounded write-heavy products).
// Must be called by all lanes of a wave together.
template <int OUT_DT>
__device__ __forceinline__ u32x4 epilogue_pack8(const void* bias, uint32_t q_nan_from, int n, v4f lo, v4f hi) {
    if constexpr (OUT_DT == MXQ_BF16) {
        if (q_nan_from != 0u) {                              // uniform
            const unsigned short span = (unsigned short)((q_nan_from >> 16) - 0x0080u);
            uint32_t w[4] = {Pack<MXQ_BF16>::put(lo[0], lo[1]), Pack<MXQ_BF16>::put(lo[2], lo[3]),
                             Pack<MXQ_BF16>::put(hi[0], hi[1]), Pack<MXQ_BF16>::put(hi[2], hi[3])};
            u16x2 worst = {0, 0};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                worst = __builtin_elementwise_max(
                    worst, __builtin_bit_cast(u16x2, w[d] & 0x7FFF7FFFu) - u16x2{0x0080, 0x0080});
                w[d] += w[d] & 0x00010001u;
            }
            if (bias != nullptr) {
                const u32x4 bw = *reinterpret_cast<const u32x4*>(reinterpret_cast<const unsigned short*>(bias) + n);
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    w[d] = Pack<MXQ_BF16>::put(Pack<MXQ_BF16>::get(w[d], 0) + Pack<MXQ_BF16>::get(bw[d], 0),
                                               Pack<MXQ_BF16>::get(w[d], 1) + Pack<MXQ_BF16>::get(bw[d], 1));
                    worst = __builtin_elementwise_max(
                        worst, __builtin_bit_cast(u16x2, w[d] & 0x7FFF7FFFu) - u16x2{0x0080, 0x0080});
                    w[d] += w[d] & 0x00010001u;
                }
            }
            if (__all(worst[0] < span && worst[1] < span)) return u32x4{w[0], w[1], w[2], w[3]};
        }
    }
    float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (bias != nullptr) {
        const u32x4 bw = *reinterpret_cast<const u32x4*>(reinterpret_cast<const unsigned short*>(bias) + n);
#pragma unroll
        for (int r = 0; r < 8; ++r)
            v[r] = epilogue_value<OUT_DT>(v[r], true, Pack<OUT_DT>::get(bw[r >> 1], r & 1), q_nan_from);
    } else if (q_nan_from != 0u) {
#pragma unroll
        for (int r = 0; r < 8; ++r) v[r] = epilogue_value<OUT_DT>(v[r], false, 0.0f, q_nan_from);
    }
    return u32x4{Pack<OUT_DT>::put(v[0], v[1]), Pack<OUT_DT>::put(v[2], v[3]),
                 Pack<OUT_DT>::put(v[4], v[5]), Pack<OUT_DT>::put(v[6], v[7])};
}

// Swaps `b` of the lanes 0-15 / 32-47 of a wave with `a` of the lanes 16-31 / 48-63 (lane L with
// lane L + 16).  The large-tile kernel uses it so that the four lanes L, L + 16, L + 32, L + 48 hold
// four consecutive 16-byte pieces of one output row: a store instruction then writes 64 contiguous
// bytes per row instead of 32, half as many write requests.
__device__ __forceinline__ void swap_with_lane16(u32x4& a, u32x4& b) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const auto r = __builtin_amdgcn_permlane16_swap(a[k], b[k], false, false);
        a[k] = r[0];
        b[k] = r[1];
    }
}

// ONE_STEP: K is a single 128-byte step (attention-shaped products, head_dim 128 or 256 nibbles):
// no second fetch to wait for, no second hand-over through LDS.
template <int CBSZ, int BLGP, int OUT_DT, bool ONE_STEP = false>
__global__ __launch_bounds__(TPB) void mx_gemm_nt_kernel(GemmArgs g) {
    constexpr bool PAIR = OUT_DT != MXQ_F32;
    constexpr int EPB = (CBSZ == 4) ? 2 : 1;                 // elements per byte of codes
    constexpr int SBY = 4 * EPB;                             // scale bytes per row and 128-byte K step
    __shared__ __attribute__((aligned(16))) unsigned char As[GEMM_BM * GEMM_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char Bs[GEMM_BN * GEMM_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char sAs[GEMM_BM * SBY];
    __shared__ __attribute__((aligned(16))) unsigned char sBs[GEMM_BN * SBY];

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
        ld_row[j] = mxq_addr::small_piece_row(tid, j);
        ld_col[j] = mxq_addr::small_piece_col(tid, j);
        ga[j] = mxq_addr::small_code_offset(m0, g.M, g.kbytes, tid, j);   // rows past the edge are clamped:
        gb[j] = mxq_addr::small_code_offset(n0, g.N, g.kbytes, tid, j);   // their outputs are never stored
    }
    const int srow = tid & 127;
    const bool s_is_a = tid < 128;
    const int64_t gs = s_is_a ? mxq_addr::small_scale_offset(m0, g.M, KB, tid)
                              : mxq_addr::small_scale_offset(n0, g.N, KB, tid);

    const int frow = lane & 15, fg = lane >> 4;
    u32x4 va[4], vb[4];
    uint32_t sv[EPB];
    auto fetch = [&](int k0) {                               // k0: byte offset of the K step in a row
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            va[j] = *reinterpret_cast<const u32x4*>(A + ga[j] + k0);
            vb[j] = *reinterpret_cast<const u32x4*>(B + gb[j] + k0);
        }
#pragma unroll
        for (int e = 0; e < EPB; ++e)
            sv[e] = *reinterpret_cast<const uint32_t*>((s_is_a ? SA : SB) + gs + mxq_addr::scale_byte_of(k0, EPB) + 4 * e);
    };
    auto stash = [&]() {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<u32x4*>(As + ld_row[j] * GEMM_PITCH + ld_col[j]) = va[j];
            *reinterpret_cast<u32x4*>(Bs + ld_row[j] * GEMM_PITCH + ld_col[j]) = vb[j];
        }
#pragma unroll
        for (int e = 0; e < EPB; ++e)
            *reinterpret_cast<uint32_t*>((s_is_a ? sAs : sBs) + srow * SBY + 4 * e) = sv[e];
    };
    // this workgroup's K steps (all of them unless the tile is split over gridDim.z), walked
    // cyclically from a per-workgroup starting step
    const int nk_all = g.kbytes / GEMM_BK;
    const int per_split = (nk_all + g.k_splits - 1) / g.k_splits;
    const int kbeg = (int)blockIdx.z * per_split;
    const int nk = min(per_split, nk_all - kbeg);
    const int kstart = (int)((blockIdx.x * 5u + blockIdx.y) % (unsigned)nk);
    auto kof = [&](int step) { return mxq_addr::small_k_byte(kbeg, kstart, step, nk); };
    fetch(kof(0));
    stash();
    __syncthreads();
    for (int step = 0; step < nk; ++step) {
        // next tile (the last step fetches one it does not use: no branches in the loop body, so
        // the instruction order below survives compilation); it arrives while this step computes
        if constexpr (!ONE_STEP) fetch(kof(step + 1));
        __builtin_amdgcn_sched_barrier(0);

        v8i bf[4];
        int sb[4][EPB];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            // 16-bit outputs: fragment rows permuted so that a lane owns 8 consecutive columns per
            // fragment pair (see the 256 x 256 kernel)
            const int n = wx * 64 + (PAIR ? (tj >> 1) * 32 + (frow >> 2) * 8 + (tj & 1) * 4 + (frow & 3)
                                          : tj * 16 + frow);
            bf[tj] = load_frag(Bs + n * GEMM_PITCH + fg * 16);
#pragma unroll
            for (int e = 0; e < EPB; ++e) sb[tj][e] = sBs[n * SBY + 4 * e + fg];
        }
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
            const int m = wy * 64 + ti * 16 + frow;
            const v8i af = load_frag(As + m * GEMM_PITCH + fg * 16);
            int sa[EPB];
#pragma unroll
            for (int e = 0; e < EPB; ++e) sa[e] = sAs[m * SBY + 4 * e + fg];
#pragma unroll
            for (int tj = 0; tj < 4; ++tj)
                acc[ti][tj] = mx_mfma<CBSZ, BLGP, 0>(bf[tj], af, acc[ti][tj], sb[tj][0], sa[0]);
            if constexpr (EPB == 2) {
#pragma unroll
                for (int tj = 0; tj < 4; ++tj)
                    acc[ti][tj] = mx_mfma<CBSZ, BLGP, 1>(bf[tj], af, acc[ti][tj], sb[tj][1], sa[1]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!ONE_STEP) {
            __syncthreads();                                 // every wave is done with this tile
            stash();
            __syncthreads();
        }
    }

    const int64_t cbase = ((int64_t)blockIdx.z * gridDim.y + bz) * g.batch_c;
    const bool inside = m0 + GEMM_BM <= g.M && n0 + GEMM_BN <= g.N && (g.N & 3) == 0 &&
                        ((uintptr_t)g.c & 15) == 0;
    const bool inside8 = inside && (g.N & 7) == 0 && ((uintptr_t)g.bias & 15) == 0;
    if constexpr (PAIR) {
        if (inside8) {                                       // uniform per workgroup
            // A lane holds two 16-byte pieces of row frow of the wave's 64 columns: columns 8 fg .. and
            // 32 + 8 fg ...  Lanes frow and frow ^ 8 trade one piece each (row_ror:8 inside the 16 lanes
            // of a DPP row), after which eight lanes hold the eight pieces of one row: a store
            // instruction then writes eight full 128-byte lines instead of sixteen half lines.
            const bool low = frow < 8;
            const int ncol = n0 + wx * 64 + (low ? 0 : 32) + fg * 8;
#pragma unroll
            for (int ti = 0; ti < 4; ++ti) {
                const u32x4 p0 = epilogue_pack8<OUT_DT>(g.bias, g.q_nan_from, n0 + wx * 64 + fg * 8, acc[ti][0], acc[ti][1]);
                const u32x4 p1 = epilogue_pack8<OUT_DT>(g.bias, g.q_nan_from, n0 + wx * 64 + 32 + fg * 8, acc[ti][2], acc[ti][3]);
                const u32x4 send = low ? p1 : p0;
                u32x4 recv;
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    recv[d] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send[d], 0x128, 0xF, 0xF, false);
                const int row = m0 + wy * 64 + ti * 16 + (frow & 7);
                unsigned short* dst = reinterpret_cast<unsigned short*>(g.c) + cbase + (int64_t)row * g.N + ncol;
                MXQ_C_STORE(reinterpret_cast<u32x4*>(dst), (low ? p0 : recv));
                MXQ_C_STORE(reinterpret_cast<u32x4*>(dst + (int64_t)8 * g.N), (low ? recv : p1));
            }
            return;
        }
    }
#pragma unroll
    for (int ti = 0; ti < 4; ++ti)
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            const int m = m0 + wy * 64 + ti * 16 + frow;
            if constexpr (PAIR) {
                if (tj & 1)
                    store_c8<OUT_DT>(g.c, g.bias, g.q_nan_from, cbase, m, n0 + wx * 64 + (tj >> 1) * 32 + fg * 8,
                                     g.M, g.N, false, acc[ti][tj - 1], acc[ti][tj]);
            } else {
                store_c4<OUT_DT>(g.c, g.bias, g.q_nan_from, cbase, m, n0 + wx * 64 + tj * 16 + fg * 4, g.M, g.N,
                                 inside, acc[ti][tj]);
            }
        }
}

constexpr int G2_BM = 256, G2_BN = 256;

// Second pass of a split small-tile GEMM: C = epilogue(sum over splits, in order, of the fp32 partial
// tiles); `rows` = batch * M rows of N columns, four columns per lane.
template <int OUT_DT>
__global__ __launch_bounds__(TPB) void gemm_split_reduce_kernel(const float* __restrict__ partial, void* c,
                                                                const void* bias, uint32_t q_nan_from,
                                                                int splits, int64_t rows, int N) {
    const int groups = (N + 3) / 4;
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= rows * groups) return;
    const int64_t m = i / groups;
    const int n = (int)(i % groups) * 4;
    const bool vec = (N & 3) == 0 && ((uintptr_t)c & 15) == 0;
    const int64_t plane = rows * (int64_t)N;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    for (int z = 0; z < splits; ++z) {
        const float* p = partial + z * plane + m * N + n;
        if (vec) {
            acc += *reinterpret_cast<const v4f*>(p);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) acc[r] += p[r];
        }
    }
    store_c4<OUT_DT>(c, bias, q_nan_from, 0, (int)m, n, (int)rows, N, vec, acc);
}

// ================================================================================================
// Main GEMM kernel: persistent workgroups, tile 256 x 256 x 128 bytes of K, 512 lanes = 4 x 2 waves,
// wave tile 64 x 128 = 2 x 4 MFMA tiles of 32 x 32 (128 accumulator registers, two waves per SIMD).
// 32 x 32 x 64 MFMAs because the matrix pipes cannot be kept busy with 16 x 16 x 128 ones on 4-bit
// operands (a register-resident loop of those reaches 5-7 PFLOP/s, of 32 x 32 x 64 ones 9.2-9.5).
//
// Tile copy: global_load_lds_dwordx4 -- the memory pipe writes 16 bytes per lane straight into LDS
// (lane L of a wave lands at base + 16 L), so there are no staging registers and no ds_write
// instructions.  LDS holds two stages of codes (A 256 rows + B 256 rows, 128 bytes each, unpadded);
// the 16-byte column c of row r is kept at position c ^ ((r >> 1) & 7), which makes the 16-byte
// fragment reads of 16 consecutive rows hit 16 different bank groups, and the lanes pick their
// global address so that the linear landing order produces exactly this image.  The loads of step
// t + 1 are issued inside step t, behind its first three MFMA groups.
//
// Scales: one byte per row and 32 K, i.e. 4 bytes per row and K step, each row in a different
// cache line.  Fetching them per step would double the number of L2 requests of the kernel, so a
// lane fetches 16 bytes = 512 K of one row at a time into a two-deep ring of scale groups.  What
// is left of a row when K is not a multiple of 512 comes in per step, 4 bytes per row, into a
// two-deep ring of its own.
//
// A workgroup walks over tiles w, w + G, w + 2 G, ... (G = grid size, a multiple of 8 so that a
// workgroup stays on its XCD) in one flat sequence of K steps: the last step of a tile already
// fetches the first step of the next one, and the stores of a finished tile drain while the next
// tile computes.
// ================================================================================================
// the LDS image (mxq_gemm_addr.h)
constexpr int G3_STAGE_BYTES = mxq_addr::L_STAGE_BYTES;      // codes of A and B for one K step
constexpr int G3_SCALE_GROUP = mxq_addr::L_SCALE_GROUP;      // 512 rows x 4 K steps x 4 bytes
constexpr int G3_TAIL_PLANE = mxq_addr::L_TAIL_PLANE;        // 512 rows x 4 scale bytes
constexpr int G3_TAIL_SLOT = mxq_addr::L_TAIL_SLOT;          // one K step: one plane (8-bit) or two (nibbles)
constexpr int G3_LDS_BYTES = mxq_addr::L_LDS_BYTES;

__device__ __forceinline__ void dma16(uint32_t lds_base, uint32_t voff, const unsigned char* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(sbase) : "memory");
}
// 4 bytes per lane, lane L lands at base + 4 L
__device__ __forceinline__ void dma4(uint32_t lds_base, uint32_t voff, const unsigned char* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(sbase) : "memory");
}

template <int CBSZ, int BLGP, int OUT_DT>
__global__ __launch_bounds__(512, 1) void mx_gemm_nt_kernel_256p(GemmArgs g, int tiles_m, int tiles_n,
                                                                 int total) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wy = wave >> 1, wx = wave & 1;
    constexpr int EPB = (CBSZ == 4) ? 2 : 1;                 // elements per byte of codes
    constexpr int SBY = 4 * EPB;                             // scale bytes per row and K step
    constexpr int GS = 16 / SBY;                             // K steps covered by a 16-byte scale group
    const int KB = g.K >> 5;
    const int nk = g.kbytes / GEMM_BK;
    const int nfull = nk - nk % GS;                          // K steps whose scales come in whole groups
    const int per_batch = tiles_m * tiles_n;
    const int G = gridDim.x;

    v16f acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // The MFMAs are 32 x 32 x 64 with the B fragment as the first operand: lane L, accumulator
    // register v then holds C[m = L % 32][n = fragment row 8 (v / 4) + 4 (L / 32) + v % 4].  Which
    // rows of B make up the fragment decides which columns a lane ends up with.  fp32 outputs keep
    // fragment row i = B row i: 4 consecutive columns (16 bytes) per register quad.  For 16-bit
    // outputs fragment row i = 8 q + 4 h + r is B row 16 (q / 2) + 8 h + 4 (q % 2) + r, so that two
    // register quads of a lane are 8 consecutive columns: one 16-byte store.
    constexpr bool PAIR = OUT_DT != MXQ_F32;
    // position of 16-byte column c of row r inside its LDS row: c ^ key(r); the key takes 8
    // different values over the even rows of any 16 consecutive rows (and again over the odd ones),
    // which is what a 16-byte read by 16 lanes needs to touch every bank once

    // ---- fetch side: which tile the tile copy is working on --------------------------------------
    // Wave w brings in rows 32 w .. 32 w + 31 of A and of B, 8 rows per instruction; lane L lands at
    // position L % 8 of row 8 i + L / 8 and therefore fetches column (L % 8) ^ ((row >> 1) & 7).
    // Rows past the edge are clamped (their outputs are never stored).
    const unsigned char *fA, *fB, *fS;
    uint32_t offa[4], offb[4], offs;
    int f_kstart;
    const bool s_is_b = wave >= 4;
    auto fetch_tile = [&](int logical) {
        const int bz = logical / per_batch;
        int tm, tn;
        tile_of_workgroup(logical % per_batch, per_batch, tiles_m, tiles_n, &tm, &tn);
        const int m0 = tm * G2_BM, n0 = tn * G2_BN;
        fA = g.a + bz * g.batch_a + (int64_t)m0 * g.kbytes;
        fB = g.b + bz * g.batch_b + (int64_t)n0 * g.kbytes;
        fS = s_is_b ? g.sb + bz * g.batch_sb + (int64_t)n0 * KB : g.sa + bz * g.batch_sa + (int64_t)m0 * KB;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            offa[i] = mxq_addr::large_code_offset(wave, lane, i, g.M - 1 - m0, g.kbytes);
            offb[i] = mxq_addr::large_code_offset(wave, lane, i, g.N - 1 - n0, g.kbytes);
        }
        offs = mxq_addr::large_scale_offset(wave, lane, s_is_b ? g.N - n0 : g.M - m0, KB);
        f_kstart = mxq_addr::large_kstart(logical, nk, nfull, GS);   // the XCD's place in the cyclic K walk
    };
    int f_groups = 0;                                        // scale groups fetched so far
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;     // LDS byte address of the array (normally 0)
    // load i (0..7 codes, 8 scales) of flat step t, which is K step fs of the fetch-side tile
    auto fetch_part = [&](int t, int fs, int i) {
        const int k0 = mxq_addr::large_kidx(f_kstart, fs, nk) * GEMM_BK;
        if (i < 4) {
            dma16(lds0 + mxq_addr::large_lds_code_dst(t, wave, i), offa[i], fA + k0);
        } else if (i < 8) {
            dma16(lds0 + mxq_addr::large_lds_code_dst(t, wave, i), offb[i - 4], fB + k0);
        } else if (fs < nfull) {
            if (fs % GS == 0) {                              // a new group of GS K steps
                dma16(lds0 + mxq_addr::large_lds_scale_group_dst(f_groups, wave), offs,
                      fS + mxq_addr::scale_byte_of(k0, EPB));
                ++f_groups;
            }
        } else {                                             // past the last whole group: this step only
#pragma unroll
            for (int e = 0; e < EPB; ++e)
                dma4(lds0 + mxq_addr::large_lds_scale_tail_dst(fs, e, wave), offs,
                     fS + mxq_addr::scale_byte_of(k0, EPB) + 4 * e);
        }
    };

    // ---- compute side ---------------------------------------------------------------------------
    // A K step is 128 bytes per row: two (8-bit codes) or four (nibbles) K = 64 MFMAs per pair of
    // fragments.  Lane (i = L % 32, g = L / 32) reads the 16-byte columns 2 q + g, q = 0..3, of its
    // row: 8-bit MFMA h takes columns 4 h + g and 4 h + 2 + g (K 16 g.. and 32 + 16 g.. of its 64),
    // nibble MFMA h takes column 2 h + g (K 32 g.. of its 64).  The lane's scale is the one of block
    // g of the MFMA's two blocks, i.e. byte 2 h + g of the row's scale bytes for this step.
    constexpr int NH = 2 * EPB;                              // MFMAs per fragment pair and K step
    const int fi = lane & 31, fg = lane >> 5;
    const int a_lane = wy * 64 + fi;                                          // row of A fragment 0
    const int b_lane = wx * 128 + mxq_addr::large_frag_row_b(fi, PAIR);
    int a_addr[4], b_addr[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        a_addr[q] = mxq_addr::large_lds_code_addr(0, a_lane, 2 * q + fg);
        b_addr[q] = mxq_addr::large_lds_code_addr(1, b_lane, 2 * q + fg);
    }
    const int sa_off = mxq_addr::large_lds_scale_group_addr(0, a_lane), sa_tail = mxq_addr::large_lds_scale_tail_addr(0, a_lane);
    const int sb_off = mxq_addr::large_lds_scale_group_addr(1, b_lane), sb_tail = mxq_addr::large_lds_scale_tail_addr(1, b_lane);
    const int sshift = fg * 8;
    constexpr int QH = 4 / NH;                               // 16-byte reads of a fragment per MFMA
    struct Half { u32x4 r[QH]; };
    auto half = [&](const unsigned char* stage, const int* addr, int tile, int h) {
        Half f;
#pragma unroll
        for (int q = 0; q < QH; ++q)
            f.r[q] = *reinterpret_cast<const u32x4*>(stage + addr[h * QH + q] + tile * 32 * 128);
        return f;
    };
    struct Scales { int w[EPB]; };
    int c_groups = 0, c_slot = 0;                            // scale groups started, the one in use
    // ---- the flat sequence of K steps ---------------------------------------------------------------
    // Step t multiplies stage t & 1.  A K step is walked MFMA number by MFMA number (h = 0: the first
    // 64 bytes of K for every tile, then h = 1, ...), in NG groups of two MFMAs (one B half, both A
    // halves): a wave holds only the parts of the fragments that the current MFMAs read.  The step's one
    // barrier stands before its last two groups: by then the wave has read everything it needs from
    // this stage (the B halves of those two groups included) and the copy of the next stage has
    // landed, so right behind the barrier it reads the operands of the next step's first group, and
    // the burst of LDS reads that all eight waves make at that point runs under the MFMAs of the last
    // two groups instead of under nothing.  The same barrier frees this stage: the copy of step t + 2
    // starts behind it (six of its nine loads in the last two groups, the rest in the first two
    // groups of step t + 1), which gives it more than a step to land.
    constexpr int NG = NH * 4;
    constexpr int BP = mxq_addr::large_barrier_group(NG);    // the group behind whose MFMAs the barrier stands
    // fetch side: the K step that the copy instructions issued now belong to
    int f_logical = blockIdx.x, f_fs = 0;
    auto fetch_advance = [&]() {
        if (++f_fs == nk) {
            f_fs = 0;
            if (f_logical + G < total) {
                f_logical += G;
                fetch_tile(f_logical);
            }                                                // else: this tile's first step once more; nobody reads it
        }
    };
    // compute side: where the scale bytes of a K step sit (inside a group of 16 bytes per row, or in
    // the planes of a single step of 4 bytes per row each)
    bool tail = false;
    const unsigned char* sc = lds;
    auto scale_place = [&](int cs) {                         // once per step, in step order
        tail = cs >= nfull;
        if (!tail && cs % GS == 0) c_slot = c_groups++ & 1;
        sc = tail ? lds + (cs & 1) * G3_TAIL_SLOT : lds + c_slot * G3_SCALE_GROUP + (cs % GS) * SBY;
    };
    auto scales = [&](int in_group, int in_tail) {           // the row's scale bytes, this lane's block first
        Scales r;
#pragma unroll
        for (int e = 0; e < EPB; ++e) {
            const unsigned char* p = tail ? sc + in_tail + e * G3_TAIL_PLANE : sc + in_group + 4 * e;
            r.w[e] = (int)(*reinterpret_cast<const uint32_t*>(p) >> sshift);
        }
        return r;
    };
    // operands of the first group of the step about to run (read behind the previous step's barrier)
    Scales sa[2], sb0;
    Half afh[2], bfh;
    auto first_operands = [&](const unsigned char* stage) {
        bfh = half(stage, b_addr, 0, 0);
        sb0 = scales(sb_off, sb_tail);
#pragma unroll
        for (int ti = 0; ti < 2; ++ti) {
            afh[ti] = half(stage, a_addr, ti, 0);
            sa[ti] = scales(sa_off + ti * 512, sa_tail + ti * 128);
        }
    };
    // t: flat step number; next_cs: the K step (of its tile) that follows this one
    auto step = [&](int t, int next_cs) {
        const unsigned char* cur = lds + (t & 1) * G3_STAGE_BYTES;
        const unsigned char* nxt = lds + ((t + 1) & 1) * G3_STAGE_BYTES;
        Scales sbv[4], sa_n[2], sb0_n;
        sbv[0] = sb0;
        Half late[2], afh_n[2], bfh_n;                       // B halves of the two groups behind the barrier; the next step's
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            const int h = gi / 4, tj = gi % 4;
            Half bfh_next = bfh, afh_next[2] = {afh[0], afh[1]};    // the next group's operands are read
            if (gi < BP) {                                            // in the shadow of this group's MFMAs
                const int h2 = (gi + 1) / 4, tj2 = (gi + 1) % 4;
                bfh_next = half(cur, b_addr, tj2, h2);
                if (h2 == 0) sbv[tj2] = scales(sb_off + tj2 * 512, sb_tail + tj2 * 128);
                if (tj2 == 0) {
#pragma unroll
                    for (int ti = 0; ti < 2; ++ti) afh_next[ti] = half(cur, a_addr, ti, h2);
                }
            } else if (gi == BP) {                           // ... here those of both groups behind the barrier
                late[0] = half(cur, b_addr, 2, NH - 1);
                late[1] = half(cur, b_addr, 3, NH - 1);
                bfh_next = late[0];
            } else if (gi == BP + 1) {
                bfh_next = late[1];
            }
            // Fences for the instruction scheduler: left alone it sinks every LDS read to just above the MFMA
            // that uses it (read, wait, multiply: the read's latency in the open, group after group), and
            // it hoists the copy instructions above the MFMAs, so that every wave of the workgroup sits in
            // the memory pipe's queue at the same time with the matrix pipes idle.
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
                acc[ti][tj] = mx_mfma32_half<CBSZ, BLGP>(bfh, afh[ti], acc[ti][tj], sbv[tj], sa[ti], h);
            asm volatile("" : "+v"(acc[0][tj]), "+v"(acc[1][tj]));
            __builtin_amdgcn_sched_barrier(0);
            if (gi == BP) {
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // this wave's share of the next stage is in,
                __syncthreads();                                              // everybody's is; and this stage is free
                fetch_advance();
                scale_place(next_cs);
                bfh_n = half(nxt, b_addr, 0, 0);
                sb0_n = scales(sb_off, sb_tail);
#pragma unroll
                for (int ti = 0; ti < 2; ++ti) {
                    afh_n[ti] = half(nxt, a_addr, ti, 0);
                    sa_n[ti] = scales(sa_off + ti * 512, sa_tail + ti * 128);
                }
            }
            // this group's share of the tile copy: loads 0 .. 5 of the step after next in the two groups
            // behind the barrier, loads 6 .. 8 of what is then the next step in the first two groups
            if (!mxq_addr::large_copy_by_phase() || wave < 4) {
#pragma unroll
                for (int i = 0; i < mxq_addr::large_copy_count(gi, NG, 0); ++i)
                    fetch_part(t + mxq_addr::large_copy_ahead(gi, NG), f_fs, mxq_addr::large_copy_first(gi, NG, 0) + i);
            } else {
#pragma unroll
                for (int i = 0; i < mxq_addr::large_copy_count(gi, NG, 1); ++i)
                    fetch_part(t + mxq_addr::large_copy_ahead(gi, NG), f_fs, mxq_addr::large_copy_first(gi, NG, 1) + i);
            }
            __builtin_amdgcn_sched_barrier(0);
            bfh = bfh_next;
            afh[0] = afh_next[0];
            afh[1] = afh_next[1];
        }
        bfh = bfh_n;
        sb0 = sb0_n;
#pragma unroll
        for (int ti = 0; ti < 2; ++ti) {
            afh[ti] = afh_n[ti];
            sa[ti] = sa_n[ti];
        }
    };

    int logical = blockIdx.x;                                // tile being multiplied
    fetch_tile(logical);
#pragma unroll
    for (int i = 0; i < 9; ++i) fetch_part(0, 0, i);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    fetch_advance();
    scale_place(0);
    first_operands(lds);
    // what the two groups behind a barrier would have issued of step 1's copy
    if (!mxq_addr::large_copy_by_phase() || wave < 4) {
#pragma unroll
        for (int i = 0; i < mxq_addr::large_copy_behind_barrier(NG, 0); ++i) fetch_part(1, f_fs, i);
    } else {
#pragma unroll
        for (int i = 0; i < mxq_addr::large_copy_behind_barrier(NG, 1); ++i) fetch_part(1, f_fs, i);
    }

    int t = 0;
    while (true) {
        for (int cs = 0; cs < nk; ++cs, ++t) step(t, cs + 1 < nk ? cs + 1 : 0);
        const int next = logical + G;

        const int bz = logical / per_batch;
        int tm, tn;
        tile_of_workgroup(logical % per_batch, per_batch, tiles_m, tiles_n, &tm, &tn);
        const int m0 = tm * G2_BM, n0 = tn * G2_BN;
        const int64_t cbase = bz * g.batch_c;
        const bool inside = m0 + G2_BM <= g.M && n0 + G2_BN <= g.N && (g.N & 3) == 0 &&
                            ((uintptr_t)g.c & 15) == 0;
        const bool inside8 = inside && (g.N & 7) == 0 && ((uintptr_t)g.bias & 15) == 0;
        // Inside tiles: a lane holds the 16-byte pieces fg, 2 + fg (, 4 + fg, 6 + fg) of its row of
        // a fragment; after the exchange with lane L +- 16 it holds piece 2 * (L / 16 % 2) + fg of
        // row L % 16 and the same piece of row 16 + L % 16 (see swap_with_lane16).
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                const int mt = m0 + wy * 64 + ti * 32;
                const int nt = n0 + wx * 128 + tj * 32;
                const v16f& c = acc[ti][tj];
                if constexpr (PAIR) {
                    if (inside8) {
                        u32x4 p[2];
#pragma unroll
                        for (int h = 0; h < 2; ++h)
                            p[h] = epilogue_pack8<OUT_DT>(g.bias, g.q_nan_from, nt + mxq_addr::large_own_col(lane, h, 8),
                                                          v4f{c[8 * h], c[8 * h + 1], c[8 * h + 2], c[8 * h + 3]},
                                                          v4f{c[8 * h + 4], c[8 * h + 5], c[8 * h + 6], c[8 * h + 7]});
                        swap_with_lane16(p[0], p[1]);
                        unsigned short* out = reinterpret_cast<unsigned short*>(g.c) + cbase + nt +
                                              mxq_addr::large_swapped_col(lane, 8);
#pragma unroll
                        for (int w = 0; w < 2; ++w)
                            MXQ_C_STORE(reinterpret_cast<u32x4*>(out + (int64_t)(mt + mxq_addr::large_swapped_row(lane, w)) * g.N), p[w]);
                    } else {
#pragma unroll
                        for (int h = 0; h < 2; ++h)
                            store_c8<OUT_DT>(g.c, g.bias, g.q_nan_from, cbase, mt + mxq_addr::large_own_row(lane),
                                             nt + mxq_addr::large_own_col(lane, h, 8), g.M, g.N,
                                             false, v4f{c[8 * h], c[8 * h + 1], c[8 * h + 2], c[8 * h + 3]},
                                             v4f{c[8 * h + 4], c[8 * h + 5], c[8 * h + 6], c[8 * h + 7]});
                    }
                } else {
                    if (inside && g.bias == nullptr) {
#pragma unroll
                        for (int q = 0; q < 4; q += 2) {
                            u32x4 p[2];
#pragma unroll
                            for (int e = 0; e < 2; ++e)
#pragma unroll
                                for (int r = 0; r < 4; ++r) p[e][r] = __float_as_uint(c[4 * (q + e) + r]);
                            swap_with_lane16(p[0], p[1]);
                            float* out = reinterpret_cast<float*>(g.c) + cbase + nt + 8 * q +
                                         mxq_addr::large_swapped_col(lane, 4);
#pragma unroll
                            for (int w = 0; w < 2; ++w)
                                MXQ_C_STORE(reinterpret_cast<u32x4*>(out + (int64_t)(mt + mxq_addr::large_swapped_row(lane, w)) * g.N), p[w]);
                        }
                    } else {
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            store_c4<OUT_DT>(g.c, g.bias, g.q_nan_from, cbase, mt + mxq_addr::large_own_row(lane),
                                             nt + mxq_addr::large_own_col(lane, q, 4), g.M, g.N,
                                             inside, v4f{c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]});
                    }
                }
            }
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int tj = 0; tj < 4; ++tj)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[ti][tj][v] = 0.f;
        if (next >= total) break;
        logical = next;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // the copy ran ahead: nothing may still be landing in LDS
}

}  // namespace
