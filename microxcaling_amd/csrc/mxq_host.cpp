// libmxq_host.so: the same scalar arithmetic as the GPU kernels (mxq_core.h), compiled for the
// host.  It serves the two CPU entry points of the reference's extension
// (quantize_mx_func_cpp, quantize_elemwise_func_cpp -- mx/cpp/funcs.cpp:23-149) for CPU tensors,
// and lets the kernel arithmetic be checked exhaustively without a GPU.  GPU tensors never come
// here: the GPU entry points live in libmxq_gfx950.so and there is no fallback between the two.
#include <stdint.h>
#include <string.h>

#include <algorithm>

#include "mxq.h"
#include "mxq_params.h"

namespace {

using namespace mxq_detail;

const unsigned char kZone[4][MXQ_ZONE_PAD] = {{MXQ_ZONE_ROW_F32}, {MXQ_ZONE_ROW_BF16}, {0}, {MXQ_ZONE_ROW_F16}};

float load_as_float(const void* p, int dtype, int64_t i) {
    if (dtype == MXQ_DTYPE_F32) return reinterpret_cast<const float*>(p)[i];
    uint16_t h = reinterpret_cast<const uint16_t*>(p)[i];
    if (dtype == MXQ_DTYPE_BF16) return mxq_float((uint32_t)h << 16);
    return (float)__builtin_bit_cast(_Float16, h);
}

void store_from_float(void* p, int dtype, int64_t i, float v) {
    if (dtype == MXQ_DTYPE_F32) {
        reinterpret_cast<float*>(p)[i] = v;
    } else if (dtype == MXQ_DTYPE_BF16) {
        reinterpret_cast<uint16_t*>(p)[i] = (uint16_t)(mxq_bits(v) >> 16);   // already bf16-exact
    } else {
        reinterpret_cast<uint16_t*>(p)[i] = __builtin_bit_cast(uint16_t, (_Float16)v);
    }
}

// element kernels selected once per call
typedef float (*MxElemFn)(float, const MxqScale&, const MxqFmt&, const unsigned char*, int, float);
typedef float (*ElemFn)(float, const MxqFmt&, bool, bool, const unsigned char*, int, float);

template <int DT, bool LEAN>
MxElemFn pick_mx(int rmode, bool ze) {
    if (rmode == MXQ_ROUND_FLOOR) return ze ? mxq_quant_mx_elem<MXQ_FLOOR, DT, true, LEAN> : mxq_quant_mx_elem<MXQ_FLOOR, DT, false, LEAN>;
    if (rmode == MXQ_ROUND_NEAREST)
        return ze ? mxq_quant_mx_elem<MXQ_NEAREST, DT, true, LEAN> : mxq_quant_mx_elem<MXQ_NEAREST, DT, false, LEAN>;
    return ze ? mxq_quant_mx_elem<MXQ_EVEN, DT, true, LEAN> : mxq_quant_mx_elem<MXQ_EVEN, DT, false, LEAN>;
}
// lean = false selects the op-by-op form, which always consults the zone table
MxElemFn pick_mx(int dtype, int flags, int rmode, bool ze, bool lean) {
    if (f16_ops(dtype, flags)) return pick_mx<MXQ_F16OPS, false>(rmode, true);
    if (dtype == MXQ_DTYPE_BF16) return lean ? pick_mx<MXQ_BF16, true>(rmode, ze) : pick_mx<MXQ_BF16, false>(rmode, true);
    return lean ? pick_mx<MXQ_F32, true>(rmode, ze) : pick_mx<MXQ_F32, false>(rmode, true);
}
template <int DT, bool LEAN>
ElemFn pick_elem(int rmode, bool ze) {
    if (rmode == MXQ_ROUND_FLOOR) return ze ? mxq_quant_elemwise<MXQ_FLOOR, DT, true, LEAN> : mxq_quant_elemwise<MXQ_FLOOR, DT, false, LEAN>;
    if (rmode == MXQ_ROUND_NEAREST) return ze ? mxq_quant_elemwise<MXQ_NEAREST, DT, true, LEAN> : mxq_quant_elemwise<MXQ_NEAREST, DT, false, LEAN>;
    return ze ? mxq_quant_elemwise<MXQ_EVEN, DT, true, LEAN> : mxq_quant_elemwise<MXQ_EVEN, DT, false, LEAN>;
}
ElemFn pick_elem(int dtype, int flags, int rmode, bool ze, bool lean) {
    if (f16_ops(dtype, flags)) return pick_elem<MXQ_F16OPS, false>(rmode, true);
    if (dtype == MXQ_DTYPE_BF16) return lean ? pick_elem<MXQ_BF16, true>(rmode, ze) : pick_elem<MXQ_BF16, false>(rmode, true);
    return lean ? pick_elem<MXQ_F32, true>(rmode, ze) : pick_elem<MXQ_F32, false>(rmode, true);
}

MxqScale block_scale(int dtype, int flags, uint32_t um, const MxParams& p, const unsigned char* zone) {
    if (f16_ops(dtype, flags)) return mxq_block_scale_f16ops(um, p.emax, p.scale_emax, zone);
    return mxq_block_scale(um, p.emax, p.scale_emax, p.flush != 0, zone, p.zshift);
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

const char* mxq_host_last_error(void) { return last_error().c_str(); }

#ifndef MXQ_BUILD_DIGEST
#define MXQ_BUILD_DIGEST "unknown"
#endif
const char* mxq_host_build_digest(void) { return MXQ_BUILD_DIGEST; }

int mxq_host_quantize_mx_by_tile(const void* in, void* out, int dtype, int64_t pre, int64_t axis_size,
                                 int64_t post, int scale_bits, int elem_ebits, int elem_mbits,
                                 float elem_max_norm, int64_t tile_size, int flush_fp32_subnorms,
                                 int rmode, int flags) {
    const char* who = "mxq_host_quantize_mx_by_tile";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, rmode, flags, &p, &ze, who);
    if (rc) return rc;
    if (pre < 0 || axis_size < 0 || post < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    int64_t total;
    if (mul_overflows(pre, axis_size, post, &total)) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
    if (total == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    const int64_t tile = (tile_size <= 0 || tile_size > axis_size) ? axis_size : tile_size;
    const unsigned char* zone = kZone[p.zone_row];
    MxElemFn fn = pick_mx(dtype, flags, rmode, ze, lean_ok(dtype, p.fmt, rmode, false) && !(flags & MXQ_HOST_FLAG_ROUND_EVERY_OP));
    for (int64_t i = 0; i < pre; ++i)
        for (int64_t k0 = 0; k0 < axis_size; k0 += tile)
            for (int64_t j = 0; j < post; ++j) {
                const int64_t k1 = std::min(k0 + tile, axis_size);
                uint32_t um = 0;
                for (int64_t k = k0; k < k1; ++k)
                    um = std::max(um, mxq_bits(load_as_float(in, dtype, (i * axis_size + k) * post + j)) & 0x7FFFFFFFu);
                MxqScale sc = block_scale(dtype, flags, um, p, zone);
                for (int64_t k = k0; k < k1; ++k) {
                    const int64_t idx = (i * axis_size + k) * post + j;
                    store_from_float(out, dtype, idx, fn(load_as_float(in, dtype, idx), sc, p.fmt, zone, p.zshift, 0.0f));
                }
            }
    return MXQ_OK;
}

int mxq_host_quantize_mx_axes(const void* in, void* out, int dtype, int n_axes, const int64_t* extents,
                              int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                              int64_t tile_size, int flush_fp32_subnorms, int rmode, int flags) {
    const char* who = "mxq_host_quantize_mx_axes";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, rmode, flags, &p, &ze, who);
    if (rc) return rc;
    MxqAxes a;
    int64_t total;
    rc = make_mx_axes(n_axes, extents, tile_size, &a, &total, who);
    if (rc) return rc;
    if (total == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    const unsigned char* zone = kZone[p.zone_row];
    MxElemFn fn = pick_mx(dtype, flags, rmode, ze, lean_ok(dtype, p.fmt, rmode, false) && !(flags & MXQ_HOST_FLAG_ROUND_EVERY_OP));
    const int64_t n_tiles = mxq_axes_tiles(a);
    for (int64_t tile = 0; tile < n_tiles; ++tile) {
        int64_t base, len[3], st[3];
        mxq_axes_tile(a, tile, &base, len, st);
        uint32_t um = 0;
        for (int64_t i = 0; i < len[0]; ++i)
            for (int64_t j = 0; j < len[1]; ++j)
                for (int64_t k = 0; k < len[2]; ++k)
                    um = std::max(um, mxq_bits(load_as_float(in, dtype, base + i * st[0] + j * st[1] + k * st[2])) & 0x7FFFFFFFu);
        MxqScale sc = block_scale(dtype, flags, um, p, zone);
        for (int64_t i = 0; i < len[0]; ++i)
            for (int64_t j = 0; j < len[1]; ++j)
                for (int64_t k = 0; k < len[2]; ++k) {
                    const int64_t idx = base + i * st[0] + j * st[1] + k * st[2];
                    store_from_float(out, dtype, idx, fn(load_as_float(in, dtype, idx), sc, p.fmt, zone, p.zshift, 0.0f));
                }
    }
    return MXQ_OK;
}

// round='dither': floor(scaled value + noise), noise[i] in [0, 1) drawn by the caller in the tensor
// dtype, one per element (mx/elemwise_ops.py:57-59)
int mxq_host_quantize_mx_dither_by_tile(const void* in, const void* noise, void* out, int dtype, int64_t pre,
                                        int64_t axis_size, int64_t post, int scale_bits, int elem_ebits,
                                        int elem_mbits, float elem_max_norm, int64_t tile_size,
                                        int flush_fp32_subnorms, int flags) {
    const char* who = "mxq_host_quantize_mx_dither_by_tile";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, MXQ_ROUND_NEAREST, flags, &p, &ze, who);
    if (rc) return rc;
    if (pre < 0 || axis_size < 0 || post < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    int64_t total;
    if (mul_overflows(pre, axis_size, post, &total)) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
    if (total == 0) return MXQ_OK;
    if (!in || !out || !noise) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    const int64_t tile = (tile_size <= 0 || tile_size > axis_size) ? axis_size : tile_size;
    const unsigned char* zone = kZone[p.zone_row];
    MxElemFn fn = f16_ops(dtype, flags)     ? mxq_quant_mx_elem<MXQ_DITHER, MXQ_F16OPS, true, false>
                  : dtype == MXQ_DTYPE_BF16 ? mxq_quant_mx_elem<MXQ_DITHER, MXQ_BF16, true, false>
                                            : mxq_quant_mx_elem<MXQ_DITHER, MXQ_F32, true, false>;
    for (int64_t i = 0; i < pre; ++i)
        for (int64_t k0 = 0; k0 < axis_size; k0 += tile)
            for (int64_t j = 0; j < post; ++j) {
                const int64_t k1 = std::min(k0 + tile, axis_size);
                uint32_t um = 0;
                for (int64_t k = k0; k < k1; ++k)
                    um = std::max(um, mxq_bits(load_as_float(in, dtype, (i * axis_size + k) * post + j)) & 0x7FFFFFFFu);
                MxqScale sc = block_scale(dtype, flags, um, p, zone);
                for (int64_t k = k0; k < k1; ++k) {
                    const int64_t idx = (i * axis_size + k) * post + j;
                    store_from_float(out, dtype, idx, fn(load_as_float(in, dtype, idx), sc, p.fmt, zone, p.zshift,
                                                         load_as_float(noise, dtype, idx)));
                }
            }
    return MXQ_OK;
}

int mxq_host_quantize_elemwise_dither(const void* in, const void* noise, void* out, int dtype, int64_t n,
                                      int bits, int exp_bits, float max_norm, int saturate_normals,
                                      int allow_denorm, int flags) {
    const char* who = "mxq_host_quantize_elemwise_dither";
    ElemParams p;
    int rc = make_elem_params(dtype, bits, exp_bits, max_norm, MXQ_ROUND_NEAREST, saturate_normals, allow_denorm,
                              flags, &p, who);
    if (rc) return rc;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!in || !out || !noise) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    const unsigned char* zone = kZone[p.zone_row];
    ElemFn fn = f16_ops(dtype, flags)     ? mxq_quant_elemwise<MXQ_DITHER, MXQ_F16OPS, true, false>
                : dtype == MXQ_DTYPE_BF16 ? mxq_quant_elemwise<MXQ_DITHER, MXQ_BF16, true, false>
                                          : mxq_quant_elemwise<MXQ_DITHER, MXQ_F32, true, false>;
    for (int64_t i = 0; i < n; ++i)
        store_from_float(out, dtype, i, fn(load_as_float(in, dtype, i), p.fmt, p.saturate != 0, p.allow_denorm != 0,
                                           zone, p.zshift, load_as_float(noise, dtype, i)));
    return MXQ_OK;
}

int mxq_host_quantize_mx_given_max(const void* in, void* out, const void* max_values, int dtype,
                                   int64_t pre, int64_t axis_size, int64_t post, int scale_bits,
                                   int elem_ebits, int elem_mbits, float elem_max_norm,
                                   int flush_fp32_subnorms, int rmode, int flags) {
    const char* who = "mxq_host_quantize_mx_given_max";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, rmode, flags, &p, &ze, who);
    if (rc) return rc;
    if (pre < 0 || axis_size < 0 || post < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    int64_t total;
    if (mul_overflows(pre, axis_size, post, &total)) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
    if (total == 0) return MXQ_OK;
    if (!in || !out || !max_values) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    const unsigned char* zone = kZone[p.zone_row];
    MxElemFn fn = pick_mx(dtype, flags, rmode, ze, lean_ok(dtype, p.fmt, rmode, false) && !(flags & MXQ_HOST_FLAG_ROUND_EVERY_OP));
    for (int64_t i = 0; i < pre; ++i)
        for (int64_t j = 0; j < post; ++j) {
            const uint32_t um = mxq_bits(load_as_float(max_values, dtype, i * post + j)) & 0x7FFFFFFFu;
            MxqScale sc = block_scale(dtype, flags, um, p, zone);
            for (int64_t k = 0; k < axis_size; ++k) {
                const int64_t idx = (i * axis_size + k) * post + j;
                store_from_float(out, dtype, idx, fn(load_as_float(in, dtype, idx), sc, p.fmt, zone, p.zshift, 0.0f));
            }
        }
    return MXQ_OK;
}

int mxq_host_quantize_elemwise(const void* in, void* out, int dtype, int64_t n, int bits, int exp_bits,
                               float max_norm, int rmode, int saturate_normals, int allow_denorm,
                               int flags) {
    const char* who = "mxq_host_quantize_elemwise";
    ElemParams p;
    int rc = make_elem_params(dtype, bits, exp_bits, max_norm, rmode, saturate_normals, allow_denorm,
                              flags, &p, who);
    if (rc) return rc;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (flags & MXQ_HOST_FLAG_CLOSED_FORM) {
        if (!(dtype == MXQ_DTYPE_BF16 && bits == 9 && exp_bits == 8 && rmode == MXQ_ROUND_NEAREST &&
              allow_denorm && !saturate_normals && p.fmt.max_bits == 0x7F7F0000u))
            return fail(MXQ_ERR_ARGUMENT, "%s: no closed form for this case", who);
        const bool nonneg = (flags & MXQ_HOST_FLAG_CLOSED_FORM_NONNEG) != 0;
        for (int64_t i = 0; i < n; ++i) {
            const float x = load_as_float(in, dtype, i);
            store_from_float(out, dtype, i, nonneg ? mxq_quant_bf16_to_bfloat16_nearest_nonneg(x)
                                                   : mxq_quant_bf16_to_bfloat16_nearest(x, p.fmt.nan_from));
        }
        return MXQ_OK;
    }
    const unsigned char* zone = kZone[p.zone_row];
    ElemFn fn = pick_elem(dtype, flags, rmode, elem_zone_matters(dtype, flags, p.fmt, rmode),
                           lean_ok(dtype, p.fmt, rmode, true) && !(flags & MXQ_HOST_FLAG_ROUND_EVERY_OP));
    for (int64_t i = 0; i < n; ++i)
        store_from_float(out, dtype, i,
                         fn(load_as_float(in, dtype, i), p.fmt, p.saturate != 0, p.allow_denorm != 0, zone, p.zshift, 0.0f));
    return MXQ_OK;
}

}  // extern "C"
#pragma GCC visibility pop
