// HIP kernels for gfx950 (MI355X): MX block quantization, elementwise quantization, reductions.
// All of them are HBM-bandwidth bound: 16-byte accesses per lane, grid-sized to the chip, the
// block maximum taken with DPP lane exchanges (last axis) or held in registers (other axes), and
// non-temporal stores for the write-once output.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxq_core.h"
#include "mxq_log2_tables.h"
#include "mxq_params.h"

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// round-up zone tables in device memory: [0] fp32, [1] bf16, [2] all zero (bit-field exponents),
// [3] fp16
#define ZONE_PAD MXQ_ZONE_PAD
__device__ const unsigned char g_zone_tables[4][ZONE_PAD] = {
    {MXQ_ZONE_ROW_F32}, {MXQ_ZONE_ROW_BF16}, {0}, {MXQ_ZONE_ROW_F16}};

namespace {

constexpr int TPB = 256;                 // lanes per workgroup (4 wave64), fixed for every kernel

__device__ __forceinline__ void load_zone(unsigned char* lds, const unsigned char* src) {
    for (int i = threadIdx.x; i < ZONE_PAD / 4; i += TPB)
        reinterpret_cast<uint32_t*>(lds)[i] = reinterpret_cast<const uint32_t*>(src)[i];
    __syncthreads();
}

// ---- dtype packing ----------------------------------------------------------------------------
template <int DT> struct Pack;
template <> struct Pack<MXQ_F32> {
    static constexpr int PER_DWORD = 1;
    static __device__ __forceinline__ float get(uint32_t w, int) { return mxq_float(w); }
    static __device__ __forceinline__ uint32_t put(float lo, float) { return mxq_bits(lo); }
};
template <> struct Pack<MXQ_BF16> {
    static constexpr int PER_DWORD = 2;
    static __device__ __forceinline__ float get(uint32_t w, int half) {
        return mxq_float(half ? (w & 0xFFFF0000u) : (w << 16));
    }
    // round to nearest even and pack: one v_cvt_pk_bf16_f32 per pair
    static __device__ __forceinline__ uint32_t put(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
    }
};
template <> struct Pack<MXQ_F16> {
    static constexpr int PER_DWORD = 2;
    static __device__ __forceinline__ float get(uint32_t w, int half) {
        unsigned short h = half ? (unsigned short)(w >> 16) : (unsigned short)(w & 0xFFFFu);
        return (float)__builtin_bit_cast(_Float16, h);
    }
    static __device__ __forceinline__ uint32_t put(float lo, float hi) {   // RNE, like torch
        return (uint32_t)mxq_f16_bits(lo) | ((uint32_t)mxq_f16_bits(hi) << 16);
    }
};

template <> struct Pack<MXQ_F16OPS> : Pack<MXQ_F16> {};

// dtype whose op-by-op rounding the arithmetic follows.  MXQ_F16: an fp16 tensor computed as fp32 and
// rounded once (bit-field exponents); MXQ_F16OPS: an fp16 tensor with every op rounded to fp16.
template <int DT> struct Arith {
    static constexpr int DT_ = (DT == MXQ_BF16) ? MXQ_BF16 : (DT == MXQ_F16OPS) ? MXQ_F16OPS : MXQ_F32;
};

template <int DT>
__device__ __forceinline__ float load_scalar(const void* p, int64_t i) {
    if (DT == MXQ_F32) return reinterpret_cast<const float*>(p)[i];
    unsigned short h = reinterpret_cast<const unsigned short*>(p)[i];
    if (DT == MXQ_BF16) return mxq_float((uint32_t)h << 16);
    return (float)__builtin_bit_cast(_Float16, h);
}
template <int DT>
__device__ __forceinline__ void store_scalar(void* p, int64_t i, float v) {
    if (DT == MXQ_F32) {
        reinterpret_cast<float*>(p)[i] = v;
    } else if (DT == MXQ_BF16) {
        reinterpret_cast<unsigned short*>(p)[i] = (unsigned short)(mxq_bits(v) >> 16);
    } else {
        reinterpret_cast<unsigned short*>(p)[i] = mxq_f16_bits(v);
    }
}

__device__ __forceinline__ uint32_t abs_bits(float f) { return mxq_bits(f) & 0x7FFFFFFFu; }

// max |x| over the 16 bytes a lane holds, as an fp32-layout bit pattern.  Magnitude bit patterns
// order like unsigned integers, and Inf/NaN patterns sit above every finite one, so an integer
// max both finds the maximum and propagates Inf/NaN.  16-bit dtypes are reduced two per dword.
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
template <int DT>
__device__ __forceinline__ uint32_t vec_abs_max(const u32x4& v) {
    if (DT == MXQ_F32) {
        return max(max(v[0] & 0x7FFFFFFFu, v[1] & 0x7FFFFFFFu),
                   max(v[2] & 0x7FFFFFFFu, v[3] & 0x7FFFFFFFu));
    }
    u16x2 m = __builtin_bit_cast(u16x2, v[0] & 0x7FFF7FFFu);
#pragma unroll
    for (int d = 1; d < 4; ++d)
        m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, v[d] & 0x7FFF7FFFu));
    const unsigned short h = m[0] > m[1] ? m[0] : m[1];
    if (DT == MXQ_BF16) return (uint32_t)h << 16;
    return abs_bits((float)__builtin_bit_cast(_Float16, h));
}

// ---- lane exchange ----------------------------------------------------------------------------
// max over groups of LANES consecutive lanes (LANES in 1,2,4,8,16), result in every lane
template <int LANES>
__device__ __forceinline__ uint32_t group_max(uint32_t v) {
    if (LANES >= 2)    // quad_perm [1,0,3,2]
        v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, false));
    if (LANES >= 4)    // quad_perm [2,3,0,1]
        v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, false));
    if (LANES >= 8)    // row_half_mirror: lane i <-> 7-i inside each group of 8
        v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, false));
    if (LANES >= 16)   // row_mirror: lane i <-> 15-i inside each row of 16
        v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, false));
    return v;
}

// ================================================================================================
// MX quantization, shared axis innermost, tile = LPT lanes x 16 bytes, tile-aligned tensor.
// One lane owns 16 bytes (4 fp32 / 8 16-bit elements); LPT neighbouring lanes share a tile.
// ================================================================================================
template <int DT, int RMODE, bool ZONE_ELEM, bool LEAN, int LPT, int UNROLL>
__global__ __launch_bounds__(TPB) void mx_lastaxis_kernel(const u32x4* __restrict__ in,
                                                          u32x4* __restrict__ out, int64_t n_vec,
                                                          MxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = MxqZoneShift<ADT>::value;        // significand units of the zone table
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int64_t CHUNK = (int64_t)TPB * UNROLL;      // vectors per block and iteration
    __shared__ unsigned char zone[ZONE_PAD];

    const int64_t stride = (int64_t)gridDim.x * CHUNK;
    int64_t base = (int64_t)blockIdx.x * CHUNK + threadIdx.x;

    // first batch of loads goes out before the table copy so the two latencies overlap
    u32x4 v[UNROLL];
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
        const int64_t i = base + j * TPB;
        v[j] = (i < n_vec) ? in[i] : u32x4{0, 0, 0, 0};
    }
    load_zone(zone, g_zone_tables[p.zone_row]);

    while (true) {
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + j * TPB;
            const uint32_t um = group_max<LPT>(vec_abs_max<DT>(v[j]));
            const MxqScale sc = mxq_block_scale_dt<ADT>(um, p.emax, p.scale_emax, p.flush != 0, zone);
            u32x4 o;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                float q[2];
#pragma unroll
                for (int h = 0; h < PD; ++h)
                    q[h] = mxq_quant_mx_elem_raw<RMODE, ADT, ZONE_ELEM, LEAN>(Pack<DT>::get(v[j][d], h),
                                                                             sc, p.fmt, zone, ZS);
                o[d] = Pack<DT>::put(q[0], q[PD - 1]);
            }
            if (i < n_vec) __builtin_nontemporal_store(o, &out[i]);
        }
        base += stride;
        if (base - threadIdx.x >= n_vec) break;     // uniform per block
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + j * TPB;
            v[j] = (i < n_vec) ? in[i] : u32x4{0, 0, 0, 0};
        }
    }
}

// ================================================================================================
// MX quantization along any axis: tensor (pre, axis, post), tiles of `tile` rows of the middle
// axis.  One lane owns VW consecutive `post` positions of one tile, so a wave reads 64*VW
// contiguous elements per row.
//   mx_strided_tile_kernel  tile == ROWS exactly and axis % ROWS == 0, post % VW == 0: the tile
//                           stays in registers between the max pass and the rounding pass (one
//                           read of the input), 8-byte accesses per lane.
//   mx_strided_kernel       anything else (ragged last tile, odd sizes, VW = 1): the rounding pass
//                           re-reads the tile.
// ================================================================================================
template <int DT> struct Col8 {                      // the 8 bytes a lane owns per row
    static constexpr int VW = (DT == MXQ_F32) ? 2 : 4;
};

// SQUARE: the exponent is shared over ROWS x ROWS tiles of the last two axes (post = columns, a
// multiple of ROWS): the ROWS / VW neighbouring lanes that hold a tile's columns combine their maxima.
template <int DT, int RMODE, bool ZONE_ELEM, bool LEAN, int ROWS, bool SQUARE = false>
__global__ __launch_bounds__(TPB) void mx_strided_tile_kernel(const u32x2* __restrict__ in,
                                                              u32x2* __restrict__ out,
                                                              int64_t items, int64_t n_tiles,
                                                              int64_t pv, MxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = MxqZoneShift<ADT>::value;        // significand units of the zone table
    constexpr int VW = Col8<DT>::VW;
    constexpr int PD = Pack<DT>::PER_DWORD;
    __shared__ unsigned char zone[ZONE_PAD];

    const int64_t w = (int64_t)blockIdx.x * TPB + threadIdx.x;     // (pre_i, tile_i, column group)
    const bool live = w < items;
    const int64_t c = live ? w % pv : 0;
    const int64_t pt = live ? w / pv : 0;                           // pre_i * n_tiles + tile_i
    const int64_t off0 = pt * ROWS * pv + c;                        // in units of 8 bytes

    u32x2 raw[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) raw[r] = live ? in[off0 + (int64_t)r * pv] : u32x2{0, 0};
    load_zone(zone, g_zone_tables[p.zone_row]);

    // column maxima as fp32-layout magnitude patterns
    uint32_t um[VW];
    if (DT == MXQ_F32) {
        um[0] = um[1] = 0;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            um[0] = max(um[0], raw[r][0] & 0x7FFFFFFFu);
            um[1] = max(um[1], raw[r][1] & 0x7FFFFFFFu);
        }
    } else {
        u16x2 m0 = {0, 0}, m1 = {0, 0};
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            m0 = __builtin_elementwise_max(m0, __builtin_bit_cast(u16x2, raw[r][0] & 0x7FFF7FFFu));
            m1 = __builtin_elementwise_max(m1, __builtin_bit_cast(u16x2, raw[r][1] & 0x7FFF7FFFu));
        }
        const unsigned short h[4] = {m0[0], m0[1], m1[0], m1[1]};
#pragma unroll
        for (int k = 0; k < 4; ++k)
            um[k % VW] = (DT == MXQ_BF16) ? (uint32_t)h[k] << 16
                                          : abs_bits((float)__builtin_bit_cast(_Float16, h[k]));
    }
    if constexpr (SQUARE) {
        uint32_t m = um[0];
#pragma unroll
        for (int k = 1; k < VW; ++k) m = max(m, um[k]);
        m = group_max<ROWS / VW>(m);                 // lanes of a group are all live or all idle
#pragma unroll
        for (int k = 0; k < VW; ++k) um[k] = m;
    }
    MxqScale sc[VW];
#pragma unroll
    for (int k = 0; k < VW; ++k)
        sc[k] = mxq_block_scale_dt<ADT>(um[k], p.emax, p.scale_emax, p.flush != 0, zone);

#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        u32x2 o;
#pragma unroll
        for (int d = 0; d < 2; ++d) {
            float q[2];
#pragma unroll
            for (int h = 0; h < PD; ++h)
                q[h] = mxq_quant_mx_elem_raw<RMODE, ADT, ZONE_ELEM, LEAN>(Pack<DT>::get(raw[r][d], h),
                                                                         sc[d * PD + h], p.fmt, zone,
                                                                         ZS);
            o[d] = Pack<DT>::put(q[0], q[PD - 1]);
        }
        if (live) __builtin_nontemporal_store(o, &out[off0 + (int64_t)r * pv]);
    }
}

template <int DT, int VW> struct ColVec;     // VW elements of dtype DT
template <> struct ColVec<MXQ_F32, 1> { typedef uint32_t T; static constexpr int DW = 1; };
template <> struct ColVec<MXQ_F32, 4> { typedef u32x4 T; static constexpr int DW = 4; };
template <> struct ColVec<MXQ_BF16, 1> { typedef unsigned short T; static constexpr int DW = 1; };
template <> struct ColVec<MXQ_BF16, 8> { typedef u32x4 T; static constexpr int DW = 4; };
template <> struct ColVec<MXQ_F16, 1> { typedef unsigned short T; static constexpr int DW = 1; };
template <> struct ColVec<MXQ_F16, 8> { typedef u32x4 T; static constexpr int DW = 4; };
template <> struct ColVec<MXQ_F16OPS, 1> : ColVec<MXQ_F16, 1> {};
template <> struct ColVec<MXQ_F16OPS, 8> : ColVec<MXQ_F16, 8> {};

template <int DT, int VW>
__device__ __forceinline__ void unpack_cols(const typename ColVec<DT, VW>::T& raw, float* x) {
    if constexpr (VW == 1) {
        if (DT == MXQ_F32) x[0] = mxq_float((uint32_t)raw);
        else if (DT == MXQ_BF16) x[0] = mxq_float((uint32_t)raw << 16);
        else x[0] = (float)__builtin_bit_cast(_Float16, (unsigned short)raw);
    } else {
        constexpr int PD = Pack<DT>::PER_DWORD;
#pragma unroll
        for (int d = 0; d < ColVec<DT, VW>::DW; ++d)
#pragma unroll
            for (int h = 0; h < PD; ++h) x[d * PD + h] = Pack<DT>::get(raw[d], h);
    }
}
template <int DT, int VW>
__device__ __forceinline__ typename ColVec<DT, VW>::T pack_cols(const float* q) {
    typename ColVec<DT, VW>::T r;
    if constexpr (VW == 1) {
        if (DT == MXQ_F32) r = mxq_bits(q[0]);
        else if (DT == MXQ_BF16) r = (unsigned short)(mxq_bits(q[0]) >> 16);
        else r = mxq_f16_bits(q[0]);
    } else {
        constexpr int PD = Pack<DT>::PER_DWORD;
#pragma unroll
        for (int d = 0; d < ColVec<DT, VW>::DW; ++d) r[d] = Pack<DT>::put(q[d * PD], q[d * PD + PD - 1]);
    }
    return r;
}

template <int DT, int RMODE, bool ZONE_ELEM, bool LEAN, int VW>
__global__ __launch_bounds__(TPB) void mx_strided_kernel(const void* __restrict__ in_,
                                                         void* __restrict__ out_, int64_t pre,
                                                         int64_t axis_size, int64_t post,
                                                         int64_t tile, int64_t num_tiles,
                                                         MxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = MxqZoneShift<ADT>::value;        // significand units of the zone table
    typedef typename ColVec<DT, VW>::T V;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.zone_row]);

    const V* in = reinterpret_cast<const V*>(in_);
    V* out = reinterpret_cast<V*>(out_);
    const int64_t pv = post / VW;                       // column groups per row
    const int64_t total = pre * num_tiles * pv;
    for (int64_t w = (int64_t)blockIdx.x * TPB + threadIdx.x; w < total;
         w += (int64_t)gridDim.x * TPB) {
        const int64_t c = w % pv;
        const int64_t ti = (w / pv) % num_tiles;
        const int64_t pi = w / (pv * num_tiles);
        const int64_t row0 = ti * tile;
        const int64_t rows = (row0 + tile > axis_size) ? (axis_size - row0) : tile;
        const int64_t off0 = (pi * axis_size + row0) * pv + c;   // in units of V

        uint32_t um[VW];
#pragma unroll
        for (int k = 0; k < VW; ++k) um[k] = 0;
        for (int64_t r = 0; r < rows; ++r) {
            float x[VW];
            unpack_cols<DT, VW>(in[off0 + r * pv], x);
#pragma unroll
            for (int k = 0; k < VW; ++k) um[k] = max(um[k], abs_bits(x[k]));
        }
        MxqScale sc[VW];
#pragma unroll
        for (int k = 0; k < VW; ++k)
            sc[k] = mxq_block_scale_dt<ADT>(um[k], p.emax, p.scale_emax, p.flush != 0, zone);
        for (int64_t r = 0; r < rows; ++r) {
            float x[VW], q[VW];
            unpack_cols<DT, VW>(in[off0 + r * pv], x);
#pragma unroll
            for (int k = 0; k < VW; ++k)
                q[k] = mxq_quant_mx_elem<RMODE, ADT, ZONE_ELEM, LEAN>(x[k], sc[k], p.fmt, zone, ZS);
            out[off0 + r * pv] = pack_cols<DT, VW>(q);
        }
    }
}

// ================================================================================================
// MX quantization with the exponent shared over the blocks of two or three axes at once (tiles of
// e.g. 32 x 32 elements): one workgroup per tile, two passes over the tile (the second reads it
// from cache).  Serves the general case at any shape; the single-axis kernels above are the
// fast path.
// ================================================================================================
template <int DT, int RMODE, bool ZONE_ELEM, bool LEAN>
__global__ __launch_bounds__(TPB) void mx_axes_kernel(const void* __restrict__ in, void* __restrict__ out,
                                                      MxqAxes a, int64_t n_tiles, MxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = MxqZoneShift<ADT>::value;
    __shared__ unsigned char zone[ZONE_PAD];
    __shared__ uint32_t wave_max[TPB / 64];
    load_zone(zone, g_zone_tables[p.zone_row]);
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        int64_t base, len[3], st[3];
        mxq_axes_tile(a, tile, &base, len, st);
        const int64_t count = len[0] * len[1] * len[2], l12 = len[1] * len[2];
        const bool narrow = count < ((int64_t)1 << 31);      // 32-bit index arithmetic: far cheaper
        const uint32_t l12n = (uint32_t)l12, l2n = (uint32_t)len[2];
        auto offset = [&](int64_t e) {
            if (narrow) {
                const uint32_t en = (uint32_t)e, i0 = en / l12n, r = en - i0 * l12n, i1 = r / l2n;
                return base + i0 * st[0] + i1 * st[1] + (r - i1 * l2n) * st[2];
            }
            const int64_t i0 = e / l12, r = e % l12;
            return base + i0 * st[0] + (r / len[2]) * st[1] + (r % len[2]) * st[2];
        };
        uint32_t um = 0;
        for (int64_t e = threadIdx.x; e < count; e += TPB) um = max(um, abs_bits(load_scalar<DT>(in, offset(e))));
        for (int d = 32; d >= 1; d >>= 1) um = max(um, (uint32_t)__shfl_xor((int)um, d, 64));
        if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = um;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < TPB / 64; ++w) um = max(um, wave_max[w]);
        const MxqScale sc = mxq_block_scale_dt<ADT>(um, p.emax, p.scale_emax, p.flush != 0, zone);
        for (int64_t e = threadIdx.x; e < count; e += TPB) {
            const int64_t off = offset(e);
            store_scalar<DT>(out, off, mxq_quant_mx_elem<RMODE, ADT, ZONE_ELEM, LEAN>(load_scalar<DT>(in, off), sc,
                                                                                      p.fmt, zone, ZS));
        }
        __syncthreads();                                     // wave_max is reused by the next tile
    }
}

// ================================================================================================
// MX quantization with the block maximum supplied by the caller: element (i, k, j) uses
// max_values[i * post + j].
// ================================================================================================
template <int DT, int RMODE, bool ZONE_ELEM, bool LEAN>
__global__ __launch_bounds__(TPB) void mx_given_max_kernel(const void* __restrict__ in,
                                                           void* __restrict__ out,
                                                           const void* __restrict__ maxv,
                                                           int64_t total, int64_t axis_size,
                                                           int64_t post, MxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = MxqZoneShift<ADT>::value;        // significand units of the zone table
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.zone_row]);
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * TPB) {
        const int64_t j = i % post;
        const int64_t pi = i / (post * axis_size);
        const uint32_t um = abs_bits(load_scalar<DT>(maxv, pi * post + j));
        MxqScale sc = mxq_block_scale_dt<ADT>(um, p.emax, p.scale_emax, p.flush != 0, zone);
        float q = mxq_quant_mx_elem<RMODE, ADT, ZONE_ELEM, LEAN>(load_scalar<DT>(in, i), sc, p.fmt,
                                                                 zone, ZS);
        store_scalar<DT>(out, i, q);
    }
}

// ================================================================================================
// Elementwise quantization.  Body: 16 bytes per lane; the (< 16 byte) tail is done per element.
// ================================================================================================
template <int DT, int RMODE, bool ZONE_ELEM, bool LEAN, int UNROLL>
__global__ __launch_bounds__(TPB) void elemwise_kernel(const void* __restrict__ in_,
                                                       void* __restrict__ out_, int64_t n,
                                                       ElemParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = MxqZoneShift<ADT>::value;        // significand units of the zone table
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.zone_row]);

    const u32x4* in = reinterpret_cast<const u32x4*>(in_);
    u32x4* out = reinterpret_cast<u32x4*>(out_);
    const int64_t n_vec = n / EPV;
    const int64_t stride = (int64_t)gridDim.x * TPB * UNROLL;
    for (int64_t base = (int64_t)blockIdx.x * TPB * UNROLL + threadIdx.x;
         base - threadIdx.x < n_vec; base += stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            int64_t i = base + (int64_t)j * TPB;
            v[j] = (i < n_vec) ? in[i] : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            int64_t i = base + (int64_t)j * TPB;
            u32x4 o;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                float q[2];
#pragma unroll
                for (int h = 0; h < PD; ++h)
                    q[h] = mxq_quant_elemwise<RMODE, ADT, ZONE_ELEM, LEAN>(Pack<DT>::get(v[j][d], h), p.fmt,
                                                                           p.saturate != 0,
                                                                           p.allow_denorm != 0, zone, ZS);
                o[d] = Pack<DT>::put(q[0], q[PD - 1]);
            }
            if (i < n_vec) __builtin_nontemporal_store(o, &out[i]);
        }
    }
    // tail
    const int64_t t0 = n_vec * EPV;
    const int64_t gi = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (gi < n - t0) {
        float q = mxq_quant_elemwise<RMODE, ADT, ZONE_ELEM, LEAN>(load_scalar<DT>(in_, t0 + gi), p.fmt,
                                                                  p.saturate != 0, p.allow_denorm != 0,
                                                                  zone, ZS);
        store_scalar<DT>(out_, t0 + gi, q);
    }
}

// ================================================================================================
// Elementwise quantization of a bf16 tensor to bfloat16 with round-half-away (the vector format of
// most MX configurations, applied to every operand, product and gradient): the closed form of
// mxq_quant_bf16_to_bfloat16_nearest instead of the general rounding.  While all of a wave's values
// are normal numbers below the NaN threshold it is "odd significand -> + 1" on both halves of a dword
// at once; a wave that sees anything else goes element by element.
// ================================================================================================
template <int UNROLL>
__global__ __launch_bounds__(TPB) void elemwise_bf16_closed_kernel(const void* __restrict__ in_,
                                                                   void* __restrict__ out_, int64_t n,
                                                                   uint32_t nan_from) {
    const u32x4* in = reinterpret_cast<const u32x4*>(in_);
    u32x4* out = reinterpret_cast<u32x4*>(out_);
    const unsigned short span = (unsigned short)((nan_from >> 16) - 0x0080u);
    const int64_t n_vec = n / 8;
    const int64_t stride = (int64_t)gridDim.x * TPB * UNROLL;
    for (int64_t base = (int64_t)blockIdx.x * TPB * UNROLL + threadIdx.x; base - threadIdx.x < n_vec;
         base += stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + (int64_t)j * TPB;
            v[j] = (i < n_vec) ? in[i] : u32x4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
        }
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + (int64_t)j * TPB;
            u16x2 worst = {0, 0};
#pragma unroll
            for (int d = 0; d < 4; ++d)
                worst = __builtin_elementwise_max(
                    worst, __builtin_bit_cast(u16x2, v[j][d] & 0x7FFF7FFFu) - u16x2{0x0080, 0x0080});
            u32x4 o;
            if (__all(worst[0] < span && worst[1] < span)) {
#pragma unroll
                for (int d = 0; d < 4; ++d) o[d] = v[j][d] + (v[j][d] & 0x00010001u);
            } else {
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    o[d] = Pack<MXQ_BF16>::put(
                        mxq_quant_bf16_to_bfloat16_nearest(Pack<MXQ_BF16>::get(v[j][d], 0), nan_from),
                        mxq_quant_bf16_to_bfloat16_nearest(Pack<MXQ_BF16>::get(v[j][d], 1), nan_from));
            }
            if (i < n_vec) __builtin_nontemporal_store(o, &out[i]);
        }
    }
    const int64_t t0 = n_vec * 8;
    const int64_t gi = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (gi < n - t0)
        store_scalar<MXQ_BF16>(out_, t0 + gi, mxq_quant_bf16_to_bfloat16_nearest(load_scalar<MXQ_BF16>(in_, t0 + gi), nan_from));
}

// ================================================================================================
// round='dither' (mx/elemwise_ops.py:57-59): floor(scaled value + noise) with noise in [0, 1) drawn
// by the caller in the tensor dtype, one per element.  A training-time option off the hot path:
// one element per lane, op-by-op form of the rounding.
// ================================================================================================
template <int DT>
__global__ __launch_bounds__(TPB) void elemwise_dither_kernel(const void* __restrict__ in,
                                                              const void* __restrict__ noise,
                                                              void* __restrict__ out, int64_t n, ElemParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = MxqZoneShift<ADT>::value;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.zone_row]);
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB)
        store_scalar<DT>(out, i, mxq_quant_elemwise<MXQ_DITHER, ADT, true, false>(
                                     load_scalar<DT>(in, i), p.fmt, p.saturate != 0, p.allow_denorm != 0, zone, ZS,
                                     load_scalar<DT>(noise, i)));
}

// tensor (pre, axis, post), tiles of `tile` positions of the middle axis; a lane owns one tile at one
// `post` position
template <int DT>
__global__ __launch_bounds__(TPB) void mx_dither_kernel(const void* __restrict__ in,
                                                        const void* __restrict__ noise,
                                                        void* __restrict__ out, int64_t pre, int64_t axis_size,
                                                        int64_t post, int64_t tile, int64_t num_tiles,
                                                        MxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = MxqZoneShift<ADT>::value;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.zone_row]);
    const int64_t total = pre * num_tiles * post;
    for (int64_t w = (int64_t)blockIdx.x * TPB + threadIdx.x; w < total; w += (int64_t)gridDim.x * TPB) {
        const int64_t c = w % post;
        const int64_t ti = (w / post) % num_tiles;
        const int64_t pi = w / (post * num_tiles);
        const int64_t row0 = ti * tile;
        const int64_t rows = (row0 + tile > axis_size) ? (axis_size - row0) : tile;
        const int64_t off0 = (pi * axis_size + row0) * post + c;
        uint32_t um = 0;
        for (int64_t r = 0; r < rows; ++r) um = max(um, abs_bits(load_scalar<DT>(in, off0 + r * post)));
        const MxqScale sc = mxq_block_scale_dt<ADT>(um, p.emax, p.scale_emax, p.flush != 0, zone);
        for (int64_t r = 0; r < rows; ++r) {
            const int64_t i = off0 + r * post;
            store_scalar<DT>(out, i, mxq_quant_mx_elem<MXQ_DITHER, ADT, true, false>(
                                         load_scalar<DT>(in, i), sc, p.fmt, zone, ZS, load_scalar<DT>(noise, i)));
        }
    }
}

// ================================================================================================
// Reductions (fp32).  max propagates NaN like torch.max; sums are accumulated in a fixed order.
// ================================================================================================
struct SumOp {
    static __device__ __forceinline__ float init() { return 0.0f; }
    static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};
struct MaxOp {
    static __device__ __forceinline__ float init() { return -__builtin_inff(); }
    static __device__ __forceinline__ float apply(float a, float b) {
        return (b > a || b != b) ? b : a;          // NaN sticks once seen
    }
};

template <class OP>
__device__ __forceinline__ float wave_reduce(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = OP::apply(v, __shfl_xor(v, m, 64));
    return v;
}

// The same over the WPR consecutive waves of a workgroup that share a row: wave results combined in
// wave order through `part` (one float per wave of the workgroup).  Every wave of the workgroup
// must take part.
template <class OP, int WPR>
__device__ __forceinline__ float row_reduce(float v, float* part) {
    v = wave_reduce<OP>(v);
    if constexpr (WPR > 1) {
        const int wib = threadIdx.x >> 6;
        __syncthreads();                                     // the previous round has been read
        if ((threadIdx.x & 63) == 0) part[wib] = v;
        __syncthreads();
        const int first = wib - wib % WPR;
        v = part[first];
#pragma unroll
        for (int k = 1; k < WPR; ++k) v = OP::apply(v, part[first + k]);
    }
    return v;
}

// one block of 256 lanes per row (inner large) ...
template <class OP>
__global__ __launch_bounds__(TPB) void reduce_inner_block_kernel(const float* __restrict__ in,
                                                                 float* __restrict__ out,
                                                                 int64_t rows, int64_t inner) {
    __shared__ float part[4];
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const float* row = in + r * inner;
        float acc = OP::init();
        const bool vec_ok = (inner % 4 == 0) && ((reinterpret_cast<uintptr_t>(row) & 15) == 0);
        if (vec_ok) {
            const u32x4* rv = reinterpret_cast<const u32x4*>(row);
            for (int64_t i = threadIdx.x; i < inner / 4; i += TPB) {
                u32x4 w = rv[i];
#pragma unroll
                for (int d = 0; d < 4; ++d) acc = OP::apply(acc, mxq_float(w[d]));
            }
        } else {
            for (int64_t i = threadIdx.x; i < inner; i += TPB) acc = OP::apply(acc, row[i]);
        }
        acc = wave_reduce<OP>(acc);
        if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            float t = part[0];
            for (int wv = 1; wv < (int)(TPB >> 6); ++wv) t = OP::apply(t, part[wv]);
            out[r] = t;
        }
        __syncthreads();
    }
}

// ... or one wave per row (inner small)
template <class OP>
__global__ __launch_bounds__(TPB) void reduce_inner_wave_kernel(const float* __restrict__ in,
                                                                float* __restrict__ out,
                                                                int64_t rows, int64_t inner) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * TPB + threadIdx.x) >> 6;
    const int64_t n_waves = ((int64_t)gridDim.x * TPB) >> 6;
    for (int64_t r = wave; r < rows; r += n_waves) {
        const float* row = in + r * inner;
        float acc = OP::init();
        const bool vec_ok = (inner % 4 == 0) && ((reinterpret_cast<uintptr_t>(row) & 15) == 0);
        if (vec_ok) {
            const u32x4* rv = reinterpret_cast<const u32x4*>(row);
            for (int64_t i = lane; i < inner / 4; i += 64) {
                u32x4 w = rv[i];
#pragma unroll
                for (int d = 0; d < 4; ++d) acc = OP::apply(acc, mxq_float(w[d]));
            }
        } else {
            for (int64_t i = lane; i < inner; i += 64) acc = OP::apply(acc, row[i]);
        }
        acc = wave_reduce<OP>(acc);
        if (lane == 0) out[r] = acc;
    }
}

// outer axis: (outer, inner) -> partial (splits, inner).  VW = 4: a lane owns KG groups of 4
// consecutive columns, 1024 columns apart, so that a block reads KG * 4 KB of contiguous memory per
// row -- whole rows when inner <= 8192, and then its rows_per_split rows are one contiguous chunk.
// VW = 1: one column per lane (unaligned shapes).  Rows are accumulated in order.
template <class OP, int VW, int KG>
__global__ __launch_bounds__(TPB) void reduce_outer_kernel(const float* __restrict__ in,
                                                           float* __restrict__ partial,
                                                           int64_t outer, int64_t inner,
                                                           int64_t rows_per_split) {
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_split;
    const int64_t r1 = (r0 + rows_per_split < outer) ? r0 + rows_per_split : outer;
    if constexpr (VW == 4) {
        const int64_t pv = inner / 4;                     // column groups per row
        const int64_t cg0 = (int64_t)blockIdx.x * TPB * KG + threadIdx.x;
        float acc[KG][4];
#pragma unroll
        for (int g = 0; g < KG; ++g)
#pragma unroll
            for (int k = 0; k < 4; ++k) acc[g][k] = OP::init();
        const u32x4* p = reinterpret_cast<const u32x4*>(in);
        constexpr int RU = 16 / KG;                       // rows in flight: 16 loads (256 bytes) per lane
        int64_t r = r0;
        for (; r + RU <= r1; r += RU) {
            u32x4 w[RU][KG];
#pragma unroll
            for (int u = 0; u < RU; ++u)
#pragma unroll
                for (int g = 0; g < KG; ++g) {
                    const int64_t cg = cg0 + (int64_t)g * TPB;
                    w[u][g] = cg < pv ? p[(r + u) * pv + cg] : u32x4{0, 0, 0, 0};
                }
#pragma unroll
            for (int u = 0; u < RU; ++u)
#pragma unroll
                for (int g = 0; g < KG; ++g)
#pragma unroll
                    for (int k = 0; k < 4; ++k) acc[g][k] = OP::apply(acc[g][k], mxq_float(w[u][g][k]));
        }
        for (; r < r1; ++r) {
#pragma unroll
            for (int g = 0; g < KG; ++g) {
                const int64_t cg = cg0 + (int64_t)g * TPB;
                if (cg < pv) {
                    const u32x4 w = p[r * pv + cg];
#pragma unroll
                    for (int k = 0; k < 4; ++k) acc[g][k] = OP::apply(acc[g][k], mxq_float(w[k]));
                }
            }
        }
#pragma unroll
        for (int g = 0; g < KG; ++g) {
            const int64_t cg = cg0 + (int64_t)g * TPB;
            if (cg < pv) {
                u32x4 o;
#pragma unroll
                for (int k = 0; k < 4; ++k) o[k] = mxq_bits(acc[g][k]);
                reinterpret_cast<u32x4*>(partial + (int64_t)blockIdx.y * inner)[cg] = o;
            }
        }
    } else {
        const int64_t cg = (int64_t)blockIdx.x * TPB + threadIdx.x;
        if (cg >= inner) return;
        float acc = OP::init();
        for (int64_t r = r0; r < r1; ++r) acc = OP::apply(acc, in[r * inner + cg]);
        partial[(int64_t)blockIdx.y * inner + cg] = acc;
    }
}

// second pass: (splits, inner) -> (inner).  A block owns 64 columns; its four waves each reduce
// every fourth split (eight loads in flight), then the four partials are combined in split order.
template <class OP>
__global__ __launch_bounds__(TPB) void reduce_outer_final_kernel(const float* __restrict__ partial,
                                                                 float* __restrict__ out,
                                                                 int64_t splits, int64_t inner) {
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t c = (int64_t)blockIdx.x * 64 + lane;
    float acc = OP::init();
    if (c < inner) {
        int64_t s = wv;
        for (; s + 28 < splits; s += 32) {
            float w[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) w[u] = partial[(s + 4 * u) * inner + c];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc = OP::apply(acc, w[u]);
        }
        for (; s < splits; s += 4) acc = OP::apply(acc, partial[s * inner + c]);
    }
    part[wv][lane] = acc;
    __syncthreads();
    if (wv == 0 && c < inner) {
        float t = part[0][lane];
#pragma unroll
        for (int g = 1; g < 4; ++g) t = OP::apply(t, part[g][lane]);
        out[c] = t;
    }
}

}  // namespace
