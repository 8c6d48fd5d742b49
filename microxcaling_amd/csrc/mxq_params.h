// Host-side parameter preparation shared by the GPU entry points (mxq_capi*.hip) and the host
// build (mxq_host.cpp): argument checks, element-format constants, choice of round-up-zone table.
#pragma once
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include <string>

#include "mxq.h"
#include "mxq_core.h"
#include "mxq_log2_tables.h"

enum { ZONE_ROW_F32 = 0, ZONE_ROW_BF16 = 1, ZONE_ROW_NONE = 2, ZONE_ROW_F16 = 3 };

struct MxParams {
    MxqFmt fmt;
    int emax;         // exponent of the element format's max_norm
    int scale_emax;   // 2^(scale_bits-1) - 1
    int flush;
    int zone_row;     // which round-up-zone table
    int zshift;       // 0 for fp32 significands, 16 for bf16, 13 for fp16
    uint32_t pre_nan_from;   // mxq_pack_mx with MXQ_FLAG_PRE_BFLOAT16: NaN threshold of that quantizer, else 0
};

struct ElemParams {
    MxqFmt fmt;
    int saturate;
    int allow_denorm;
    int zone_row;
    int zshift;
    int general_only;   // chain kernels: MXQ_FLAG_GENERAL_FORM
};

namespace mxq_detail {

// host copy of the round-up-zone tables (the kernels read theirs from device memory)
static const unsigned char zone_rows[4][MXQ_ZONE_PAD] = {{MXQ_ZONE_ROW_F32}, {MXQ_ZONE_ROW_BF16}, {0}, {MXQ_ZONE_ROW_F16}};

// fp16 tensors: every op rounded to fp16 (the reference's pure-PyTorch path on such a tensor), unless
// the caller asks for bit-field exponents -- then they are widened to fp32, quantized and rounded
// back once, which is what the reference's CUDA kernels do (mx/cpp/mx.cuh:72,88).
inline bool f16_ops(int dtype, int flags) { return dtype == MXQ_DTYPE_F16 && !(flags & MXQ_FLAG_EXACT_EXPONENT); }

inline std::string& last_error() {
    static thread_local std::string s;
    return s;
}

inline int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
inline int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline bool mul_overflows(int64_t a, int64_t b, int64_t c, int64_t* out) {
    __int128 t = (__int128)a * b * c;
    if (t > (__int128)INT64_MAX) return true;
    *out = (int64_t)t;
    return false;
}

// extents: o0, s0, o1, ..., s(n-1), o(n): 2 * n_axes + 1 values.  tile_size <= 0: whole axes.
inline int make_mx_axes(int n_axes, const int64_t* extents, int64_t tile_size, MxqAxes* a, int64_t* total,
                        const char* who) {
    if (n_axes < 1 || n_axes > 3) return fail(MXQ_ERR_ARGUMENT, "%s: %d shared axes (1 to 3 supported)", who, n_axes);
    if (!extents) return fail(MXQ_ERR_ARGUMENT, "%s: null extents", who);
    for (int k = 0; k < 4; ++k) a->o[k] = 1;
    for (int k = 0; k < 3; ++k) a->s[k] = a->t[k] = a->nb[k] = 1;
    __int128 n = 1;
    for (int k = 0; k <= 2 * n_axes; ++k) {
        if (extents[k] < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
        n *= extents[k];
        if (n > (__int128)INT64_MAX) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
        if (k % 2 == 0) a->o[k / 2] = extents[k];
        else a->s[k / 2] = extents[k];
    }
    *total = (int64_t)n;
    if (*total == 0) return MXQ_OK;
    for (int k = 0; k < n_axes; ++k) {
        a->t[k] = (tile_size <= 0 || tile_size > a->s[k]) ? a->s[k] : tile_size;
        a->nb[k] = ceil_div(a->s[k], a->t[k]);
    }
    return MXQ_OK;
}

inline int make_fmt(int dtype, int flags, int ebits, int mbits, float max_norm, bool clamps, MxqFmt* fmt,
                    const char* who) {
    if (ebits < 0 || ebits > 8) return fail(MXQ_ERR_ARGUMENT, "%s: exponent bits %d outside [0, 8]", who, ebits);
    if (mbits < 2 || mbits > 24)
        return fail(MXQ_ERR_ARGUMENT, "%s: bits %d outside [2, 24] (sign + implicit one + fraction)", who, mbits);
    if (!(max_norm > 0.0f) || !(max_norm < __builtin_inff()))
        return fail(MXQ_ERR_ARGUMENT, "%s: max_norm must be positive and finite", who);
    fmt->ebits = ebits;
    fmt->t = mbits - 2;
    fmt->min_exp = ebits ? 2 - (1 << (ebits - 1)) : 0;
    // torch casts the clamp bound to the tensor dtype (65504 becomes 65536 for a bf16 tensor)
    fmt->max_bits = mxq_bits(dtype == MXQ_DTYPE_BF16 ? mxq_round_bf16(max_norm) : max_norm);
    // a clamp bound beyond the largest bf16 number: torch.clamp refuses the conversion (mx/elemwise_ops.py:154)
    if (dtype == MXQ_DTYPE_BF16 && clamps && max_norm > 3.3895313892515355e38f)
        return fail(MXQ_ERR_ARGUMENT, "%s: max_norm %g cannot be converted to bfloat16 without overflow "
                    "(the clamp of a bfloat16 tensor needs its bound in bfloat16)", who, (double)max_norm);
    if (f16_ops(dtype, flags)) {
        // a bound beyond the fp16 range: torch.clamp refuses to convert it (mx/elemwise_ops.py:154
        // raises), the comparison of the non-saturating branch (156) sees it as Inf
        fmt->max_bits = mxq_bits(mxq_round_f16(max_norm));
        if (clamps && max_norm > 65504.0f)
            return fail(MXQ_ERR_ARGUMENT, "%s: max_norm %g cannot be converted to float16 without overflow "
                        "(the clamp of a float16 tensor needs its bound in float16)", who, (double)max_norm);
    }
    fmt->min_eb = ebits ? (uint32_t)(fmt->min_exp + 127) : 127u;
    fmt->t127 = fmt->t + 127;
    // "s + 0.5" is rounded to the tensor dtype before the floor: in bf16 that turns 1 - 2^-9 into
    // 1.0, which adding 2^-9 more reproduces (all other sums keep their integer part)
    fmt->half = dtype == MXQ_DTYPE_BF16 ? 0.5f + 0.001953125f : 0.5f;
    fmt->tie_fix = dtype == MXQ_DTYPE_BF16 ? 0.5f - 0.001953125f : 0.5f - 2.98023223876953125e-8f;
    fmt->nan_from = MXQ_INF_BITS;
    fmt->bump_lo = (dtype == MXQ_DTYPE_BF16 && fmt->t >= 7) ? 128.0f : __builtin_inff();
    return MXQ_OK;
}

inline void zone_for(int dtype, int flags, int* row, int* zshift) {
    *zshift = 0;
    if (flags & MXQ_FLAG_EXACT_EXPONENT) {
        *row = ZONE_ROW_NONE;
    } else if (dtype == MXQ_DTYPE_F16) {
        *row = ZONE_ROW_F16;
        *zshift = 13;
    } else if (dtype == MXQ_DTYPE_BF16) {
        *row = ZONE_ROW_BF16;
        *zshift = 16;
    } else {
        *row = ZONE_ROW_F32;
    }
}

// May the lean element rounding be used (see mxq_round_lean)?  bf16 tensors with 7 or more
// fraction bits: the elementwise quantizer handles the one extra case of nearest mode (BUMP), floor
// mode has none, torch's emulation of even mode has too many (op-by-op form).  MX element formats
// never have more than 6 fraction bits.
// fp16 tensors evaluated op by op (f16_ops) always take the op-by-op form; callers test that first.
inline bool lean_ok(int dtype, const MxqFmt& f, int rmode, bool elementwise) {
    // Two parameter corners take the op-by-op form on every dtype.  One exponent bit: min_exp is 1, and
    // x / 2**1 underflows to zero for the smallest subnormal, which then comes out as +0 (the lean form
    // scales by 2**(t - e) in one exact step and would keep the sign).  An integer format whose max_norm
    // is 2 or more (none of the named ones): the lean form lets |x| >= 2 take its own exponent, knowing
    // that the clamp to a max_norm below 2 erases the difference.
    if (f.ebits == 1 || (f.ebits == 0 && f.max_bits >= 0x40000000u)) return false;
    // MX with an 8-bit element exponent (no named format has one): the block scale puts the maximum into
    // the top binade, where floor(log2(x)) can come out as 128 and 2**128 = inf makes the element NaN;
    // the elementwise quantizer handles that with a threshold of its own (nan_from), the lean MX form does not
    if (!elementwise && f.ebits == 8) return false;
    return dtype != MXQ_DTYPE_BF16 || f.t <= 6 || (elementwise && rmode != MXQ_ROUND_EVEN);
}

// Does the round-up zone of the *element* exponent change results?  In nearest / even modes a
// value in the zone rounds to the next power of two whichever exponent is used, as long as the
// zone is narrower than half a rounding step: count * 2^t <= 2^(22 - zshift) (largest count 88 for
// fp32; bf16 has count <= 5 while |exponent| <= 16, i.e. for formats with at most 5 exponent bits).
inline bool elem_zone_matters(int dtype, int flags, const MxqFmt& f, int rmode) {
    int row, zs;
    zone_for(dtype, flags, &row, &zs);
    if (row == ZONE_ROW_NONE || f.ebits == 0) return false;
    if (rmode == MXQ_ROUND_FLOOR) return true;
    if (row == ZONE_ROW_F32) return f.t > 15;
    return !(f.ebits <= 5 && f.t <= 3);
}

inline int make_mx_params(int dtype, int scale_bits, int ebits, int mbits, float max_norm, int flush,
                          int rmode, int flags, MxParams* p, bool* zone_elem, const char* who) {
    if (dtype < 0 || dtype > 2) return fail(MXQ_ERR_ARGUMENT, "%s: unknown dtype code %d", who, dtype);
    if (rmode < 0 || rmode > 2) return fail(MXQ_ERR_ARGUMENT, "%s: unknown rounding mode %d", who, rmode);
    if (scale_bits < 1 || scale_bits > 8)
        return fail(MXQ_ERR_ARGUMENT, "%s: scale_bits %d outside [1, 8]", who, scale_bits);
    int rc = make_fmt(dtype, flags, ebits, mbits, max_norm, true, &p->fmt, who);
    if (rc) return rc;
    // exponent of max_norm, the way the reference's kernels derive it (mx/cpp/shared_exp.cuh:33)
    int be = (int)((mxq_bits(max_norm) >> 23) & 0xFF);
    p->emax = be ? be - 127 : -126;
    p->scale_emax = (1 << (scale_bits - 1)) - 1;
    p->flush = flush ? 1 : 0;
    zone_for(dtype, flags, &p->zone_row, &p->zshift);
    p->pre_nan_from = 0u;
    *zone_elem = elem_zone_matters(dtype, flags, p->fmt, rmode);
    return MXQ_OK;
}

inline int make_elem_params(int dtype, int bits, int exp_bits, float max_norm, int rmode,
                            int saturate, int allow_denorm, int flags, ElemParams* p, const char* who) {
    if (dtype < 0 || dtype > 2) return fail(MXQ_ERR_ARGUMENT, "%s: unknown dtype code %d", who, dtype);
    if (rmode < 0 || rmode > 2) return fail(MXQ_ERR_ARGUMENT, "%s: unknown rounding mode %d", who, rmode);
    int rc = make_fmt(dtype, flags, exp_bits, bits, max_norm, saturate || exp_bits == 0, &p->fmt, who);
    if (rc) return rc;
    p->saturate = saturate ? 1 : 0;
    p->allow_denorm = allow_denorm ? 1 : 0;
    p->general_only = (flags & MXQ_FLAG_GENERAL_FORM) ? 1 : 0;
    zone_for(dtype, flags, &p->zone_row, &p->zshift);
    // the top binade's round-up zone: floor(log2|x|) = 128 there (16 for an fp16 tensor, whose top
    // binade is k = 15), and 2**that is Inf
    const uint32_t top_bits = p->zone_row == ZONE_ROW_F16 ? 0x47800000u : MXQ_INF_BITS;
    const uint32_t top_count = zone_rows[p->zone_row][p->zone_row == ZONE_ROW_F16 ? 15 + 149 : 276];
    p->fmt.nan_from = exp_bits ? top_bits - (top_count << p->zshift) : MXQ_INF_BITS;
    return MXQ_OK;
}

}  // namespace mxq_detail
