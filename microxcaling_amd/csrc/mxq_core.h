// Scalar arithmetic of MX / bfloat quantization, shared by every HIP kernel and by the host build.
//
// Parity target: the pure-PyTorch path of the reference (mx/mx_ops.py:265-292,
// mx/elemwise_ops.py:127-163), which evaluates a chain of IEEE ops in the tensor's own dtype.
// The functions below run the same IEEE fp32 operations in the same order (fp32 add / mul /
// floor are correctly rounded on gfx950 with denormals enabled, as on the CPU) and, for bf16
// tensors, round to bf16 after each op exactly where torch's CPU kernels do.  Exponents follow
// floor(log2(x)) *as evaluated in the tensor dtype*: bit-field exponent plus a table-driven
// "round-up zone" just below each power of two (see gen_log2_tables.py).
//
// Everything here is branch-light integer/fp32 code: no transcendental instruction is used
// (v_log/v_exp/v_rcp flush denormals and are not correctly rounded).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MXQ_HD __host__ __device__ __forceinline__
#else
#define MXQ_HD static inline __attribute__((always_inline))
#include <math.h>
#endif

enum MxqDtype { MXQ_F32 = 0, MXQ_F16 = 1, MXQ_BF16 = 2 };
// Not a tensor dtype of the C ABI: an fp16 tensor whose every op is rounded to fp16, the way torch's
// CPU kernels evaluate the reference's pure path on such a tensor (compute in fp32, round to fp16).
// MXQ_F16 as a template argument means "fp16 tensor, fp32 arithmetic" (the reference's CUDA kernels).
#define MXQ_F16OPS 3
enum MxqRound { MXQ_NEAREST = 0, MXQ_FLOOR = 1, MXQ_EVEN = 2 };   // mx/formats.py:12-19
// round='dither' (mx/elemwise_ops.py:57-59) is not in that enum: floor(s + u) with u in [0, 1) drawn
// by the caller, one per element.  Only the op-by-op form of the rounding knows it.
#define MXQ_DITHER 3

#define MXQ_QNAN_BITS 0x7FC00000u
#define MXQ_INF_BITS 0x7F800000u

MXQ_HD uint32_t mxq_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
MXQ_HD float mxq_float(uint32_t u) { return __builtin_bit_cast(float, u); }

// x * 2^n, exact unless the result is subnormal (then rounded to nearest even once) or overflows.
// Device: ldexpf (one v_ldexp_f32).  Host: for n in [-126, 127] a multiplication by the power of two
// built from its bit pattern -- the same correctly rounded result without a call into libm.
MXQ_HD float mxq_ldexp(float x, int n) {
#if defined(__HIP_DEVICE_COMPILE__)
    return ldexpf(x, n);
#else
    if ((unsigned)(n + 126) <= 253u) return x * mxq_float((uint32_t)(n + 127) << 23);
    return ldexpf(x, n);
#endif
}

// ---- dtype rounding ---------------------------------------------------------------------------
// fp32 -> bf16 -> fp32, round to nearest even, subnormals kept (what torch's CPU bf16 kernels do
// after every op).
MXQ_HD float mxq_round_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    __bf16 b = (__bf16)f;                       // v_cvt_pk_bf16_f32 on gfx950
    return mxq_float((uint32_t)__builtin_bit_cast(unsigned short, b) << 16);
#else
    uint32_t u = mxq_bits(f);
    if ((u & 0x7FFFFFFFu) > MXQ_INF_BITS) return mxq_float(MXQ_QNAN_BITS);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return mxq_float(u & 0xFFFF0000u);
#endif
}

// fp32 -> fp16 bits, round to nearest even, subnormals kept, overflow to Inf (v_cvt_f16_f32 on
// gfx950; the kernels run with fp16 denormals enabled), and back.
#if defined(__clang__)
// On the device the value passes through an empty asm statement first: left alone, the compiler
// fuses a preceding multiplication into v_fma_mixlo_f16 a, b, +0, and (-0) + (+0) = +0 loses the
// sign of a zero product.
MXQ_HD unsigned short mxq_f16_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm("" : "+v"(f));
#endif
    return __builtin_bit_cast(unsigned short, (_Float16)f);
}
MXQ_HD float mxq_f16_value(unsigned short h) { return (float)__builtin_bit_cast(_Float16, h); }
#else
// a host compiler without _Float16 (g++ 11 on x86): the same conversions in integer arithmetic
MXQ_HD unsigned short mxq_f16_bits(float f) {
    const uint32_t u = mxq_bits(f), sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > MXQ_INF_BITS) return (unsigned short)(sign | 0x7E00u);
    if (a >= 0x477FF000u) return (unsigned short)(sign | 0x7C00u);       // 65520 and up round to Inf
    if (a < 0x38800000u)                                                 // below 2^-14: units of 2^-24,
        return (unsigned short)(sign | (mxq_bits(mxq_float(a) + 0.5f) - 0x3F000000u));   // the ulp of [0.5, 1)
    a += 0xFFFu + ((a >> 13) & 1u);
    return (unsigned short)(sign | ((a - 0x38000000u) >> 13));
}
MXQ_HD float mxq_f16_value(unsigned short h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u;
    if (e == 0u) return mxq_float(sign | mxq_bits(mxq_ldexp((float)m, -24)));
    if (e == 31u) return mxq_float(sign | MXQ_INF_BITS | (m << 13));
    return mxq_float(sign | ((e + 112u) << 23) | (m << 13));
}
#endif
MXQ_HD float mxq_round_f16(float f) { return mxq_f16_value(mxq_f16_bits(f)); }

template <int DT>
MXQ_HD float mxq_round_dt(float f) {
    if (DT == MXQ_BF16) return mxq_round_bf16(f);
    if (DT == MXQ_F16OPS) return mxq_round_f16(f);
    return f;
}

// Shift of the round-up-zone counts for the arithmetic dtype (units of the 24-bit significand).
template <int DT> struct MxqZoneShift { static constexpr int value = DT == MXQ_BF16 ? 16 : DT == MXQ_F16OPS ? 13 : 0; };

// ---- exponent shared over the blocks of several axes ----------------------------------------------
// A contiguous tensor seen as (o[0], s[0], o[1], s[1], o[2], s[2], o[3]): up to three shared axes s
// with the products o of the axes around them; unused places have extent 1.  A tile takes t[i]
// consecutive positions of every shared axis (the last tile of an axis may be shorter) and one
// position of every other axis (mx/mx_ops.py:95-154 with several axes).
struct MxqAxes {
    int64_t o[4];
    int64_t s[3];
    int64_t t[3];       // tile extent along each shared axis
    int64_t nb[3];      // tiles along each shared axis
};
MXQ_HD int64_t mxq_axes_tiles(const MxqAxes& a) {
    return a.o[0] * a.nb[0] * a.o[1] * a.nb[1] * a.o[2] * a.nb[2] * a.o[3];
}
// tile number -> offset of its first element, its extents len[] and the element strides st[] of
// the shared axes
MXQ_HD void mxq_axes_tile(const MxqAxes& a, int64_t tile, int64_t* base, int64_t len[3], int64_t st[3]) {
    st[2] = a.o[3];
    const int64_t st_o2 = a.s[2] * st[2];
    st[1] = a.o[2] * st_o2;
    const int64_t st_o1 = a.s[1] * st[1];
    st[0] = a.o[1] * st_o1;
    const int64_t st_o0 = a.s[0] * st[0];
    int64_t r = tile;
    const int64_t i3 = r % a.o[3]; r /= a.o[3];
    const int64_t b2 = r % a.nb[2]; r /= a.nb[2];
    const int64_t i2 = r % a.o[2]; r /= a.o[2];
    const int64_t b1 = r % a.nb[1]; r /= a.nb[1];
    const int64_t i1 = r % a.o[1]; r /= a.o[1];
    const int64_t b0 = r % a.nb[0]; r /= a.nb[0];
    *base = r * st_o0 + b0 * a.t[0] * st[0] + i1 * st_o1 + b1 * a.t[1] * st[1] + i2 * st_o2 +
            b2 * a.t[2] * st[2] + i3;
    const int64_t b[3] = {b0, b1, b2};
    for (int k = 0; k < 3; ++k) {
        const int64_t left = a.s[k] - b[k] * a.t[k];
        len[k] = left < a.t[k] ? left : a.t[k];
    }
}

// ---- element format ----------------------------------------------------------------------------
struct MxqFmt {
    int ebits;          // exponent bits, 0 for integer formats
    int t;              // fraction bits kept = mbits - 2 (mbits counts sign and implicit one)
    int min_exp;        // 2 - 2^(ebits-1): exponent of the smallest normal (mx/elemwise_ops.py:139)
    uint32_t max_bits;  // bit pattern of max_norm (already rounded to the tensor dtype)
    // derived, for the lean path
    uint32_t min_eb;    // min_exp + 127, or 127 for integer formats (their exponent is fixed at 0)
    int t127;           // t + 127
    float half;         // what "+ 0.5" must add so that floor() sees the dtype-rounded sum
    float tie_fix;      // the one input of the scaled domain whose "+ 0.5" rounds up to 1.0
    uint32_t nan_from;  // elementwise only: |x| bit pattern from which floor(log2|x|) is 128
    float bump_lo;      // bf16 tensors, t >= 7: 128 (see mxq_round_lean<.., BUMP>); else +inf
};

// ---- floor(log2(x)) in the tensor dtype --------------------------------------------------------
// m: positive and finite.  zone[k+149] / zshift: see gen_log2_tables.py.
MXQ_HD int mxq_floor_log2(float m, const unsigned char* zone, int zshift) {
    int ex;
    const float fr = frexpf(m, &ex);            // m = fr * 2^ex, fr in [0.5, 1); handles subnormals
    const int k = ex - 1;
    const uint32_t gap = 0x800000u - (mxq_bits(fr) & 0x7FFFFFu);   // 2^24 - normalised significand
    return k + (gap <= ((uint32_t)zone[k + 149] << zshift) ? 1 : 0);
}

// ---- shared exponent of one block (mx/mx_ops.py:269-283) ---------------------------------------
// A block that must become NaN (Inf/NaN seen, or scale exponent overflow) gets scale = NaN; a
// block that must be flushed gets inv_scale = 0: the element code then needs no special cases.
struct MxqScale {
    float scale;      // 2^se
    float inv_scale;  // 2^-se
};

// um: max |x| of the block as an fp32-layout bit pattern (0x7F800000 and above = Inf/NaN seen).
// emax = exponent of the element format's max_norm; scale_emax = 2^(scale_bits-1) - 1.
MXQ_HD MxqScale mxq_block_scale(uint32_t um, int emax, int scale_emax, bool flush_subnorms,
                                const unsigned char* zone, int zshift) {
    const uint32_t eb = um >> 23;
    // normal maximum (also Inf/NaN, overwritten below): exponent field plus the round-up zone
    const uint32_t gap = 0x800000u - (um & 0x7FFFFFu);
    int E = (int)eb - 127 + (gap <= ((uint32_t)zone[eb + 22] << zshift) ? 1 : 0);
    if (eb == 0u)                                // rare: zero -> log2(2^-126); fp32 subnormal
        E = (um == 0u) ? -126 : mxq_floor_log2(mxq_float(um), zone, zshift);
    int se = E - emax;
    const bool nan = um >= MXQ_INF_BITS || se > scale_emax;
    se = se < -scale_emax ? -scale_emax : se;
    se = se > 127 ? 127 : se;
    MxqScale r;
    r.scale = nan ? mxq_float(MXQ_QNAN_BITS) : mxq_ldexp(1.0f, se);
    r.inv_scale = (flush_subnorms && E <= -127) ? 0.0f : mxq_ldexp(1.0f, -se);
    return r;
}

// The same for an fp16 tensor evaluated op by op in fp16.  What differs from the wide dtypes:
//  * FP32_MIN_NORMAL * (max == 0) is 0 in fp16, so an all-zero block has log2(0) = -inf and its scale
//    exponent is the lower clamp -scale_emax;
//  * 2**se is an fp16 number: Inf from se = 16 and 0 up to se = -25 (2^-25 ties to even).  Either
//    turns the whole block into NaN (x / Inf = 0 and 0 * Inf = NaN; x / 0 = Inf or NaN, the element
//    rounding returns Inf for Inf, and Inf * 0 = NaN);
//  * a nonzero fp16 maximum is at least 2^-24, so flush_fp32_subnorms only meets all-zero blocks,
//    whose elements are zeros before and after.
// um: max |x| widened to fp32 (never an fp32 subnormal).
MXQ_HD MxqScale mxq_block_scale_f16ops(uint32_t um, int emax, int scale_emax, const unsigned char* zone) {
    const uint32_t eb = um >> 23;
    const uint32_t gap = 0x800000u - (um & 0x7FFFFFu);
    const int E = (um == 0u) ? -100000 : (int)eb - 127 + (gap <= ((uint32_t)zone[eb + 22] << 13) ? 1 : 0);
    int se = E - emax;
    bool nan = um >= MXQ_INF_BITS || se > scale_emax;
    se = se < -scale_emax ? -scale_emax : se;
    nan = nan || se >= 16 || se <= -25;
    se = se < -25 ? -25 : (se > 16 ? 16 : se);
    MxqScale r;
    r.scale = nan ? mxq_float(MXQ_QNAN_BITS) : mxq_ldexp(1.0f, se);
    r.inv_scale = mxq_ldexp(1.0f, -se);
    return r;
}

template <int DT>
MXQ_HD MxqScale mxq_block_scale_dt(uint32_t um, int emax, int scale_emax, bool flush_subnorms,
                                   const unsigned char* zone) {
    if (DT == MXQ_F16OPS) return mxq_block_scale_f16ops(um, emax, scale_emax, zone);
    return mxq_block_scale(um, emax, scale_emax, flush_subnorms, zone, MxqZoneShift<DT>::value);
}

// ---- element rounding, lean form ----------------------------------------------------------------
// a: input in the tensor dtype, already divided by the block scale.  Valid for fp32 tensors with
// any t <= 22 and for bf16 tensors with t <= 6: there the only place where the dtype rounding of
// an intermediate changes a result is "s + 0.5" for s just below one half (0.5 - 2^-25 in fp32,
// which the fp32 add reproduces by itself; 0.5 - 2^-9 in bf16, reproduced by adding 2^-9 more),
// and torch's even-mode emulation equals round-half-even except for that same input.
// Inf/NaN inputs give unspecified results here; callers overwrite them.
// sign_src: a value with the sign the result must carry (+0.0 when the result must be +0).
// BUMP (bf16 tensors, nearest and floor modes, any t): with 7 or more fraction bits the scaled
// value s can be an integer in [128, 256), where bf16 has no halves: "s + 0.5" then ties to the
// even neighbour, so an odd s comes out as s + 1.  Everything else is exact: s has 8 significant
// bits, larger s are integers that "+ 0.5" leaves alone, smaller ones have room for the half.
template <int RMODE, bool ZONE, bool BUMP = false>
MXQ_HD float mxq_round_lean(float a, float sign_src, const MxqFmt& f, bool saturate,
                            const unsigned char* zone, int zshift) {
    const uint32_t ua = mxq_bits(a) & 0x7FFFFFFFu;
    uint32_t eb = (mxq_bits(a) >> 23) & 0xFFu;  // biased exponent; 0 for subnormals and zero
    if (ZONE) {                                 // eb + 22 == k + 149; rows are zero-padded past 276
        const uint32_t gap = 0x1000000u - ((ua & 0x7FFFFFu) | 0x800000u);
        eb += (gap <= ((uint32_t)zone[eb + 22] << zshift)) ? 1u : 0u;
    }
    // integer formats: min_eb = 127 pins the exponent at 0 for |a| < 2; larger |a| end above
    // max_norm with either exponent and are clamped to it
    const uint32_t ebc = eb > f.min_eb ? eb : f.min_eb;
    const int n = f.t127 - (int)ebc;
    const float s = mxq_ldexp(mxq_float(ua), n);   // exact
    float r;
    if (RMODE == MXQ_FLOOR) {
        r = floorf(s);
    } else if (RMODE == MXQ_NEAREST) {
        r = floorf(s + f.half);
        if (BUMP) {
            const float odd = r - 2.0f * floorf(r * 0.5f);
            r += (s >= f.bump_lo && s < 2.0f * f.bump_lo) ? odd : 0.0f;
        }
    } else {
        r = __builtin_rintf(s);                 // ties to even (default rounding mode)
        r = (s == f.tie_fix) ? 1.0f : r;
    }
    const float y = mxq_ldexp(r, -n);              // exact
    uint32_t uy = mxq_bits(y);
    if (saturate) uy = uy < f.max_bits ? uy : f.max_bits;
    else uy = uy > f.max_bits ? MXQ_INF_BITS : uy;
    return mxq_float(uy | (mxq_bits(sign_src) & 0x80000000u));
}

// sign(a) * r gives -0.0 when a negative value rounds to zero but +0.0 for a = +-0: a + 0.0 has
// exactly that sign.  For bf16 tensors a was first rounded to bf16, where |a| <= 2^-134 becomes
// +-0: a * 2^-16 rounds to +-0 in fp32 for exactly those values.
template <int DT>
MXQ_HD float mxq_sign_source(float a) {
    if (DT == MXQ_BF16) return a * 1.52587890625e-05f + 0.0f;
    return a + 0.0f;
}

// ---- element rounding, op-by-op form (mx/elemwise_ops.py:134-157) -------------------------------
// Rounds to the tensor dtype after every op exactly like torch's CPU kernels do.  Used for bf16
// tensors with wide element formats (t >= 7) and, on the host, to cross-check the lean form.
template <int RMODE, int DT>
MXQ_HD float mxq_round_every_op(float a, const MxqFmt& f, bool saturate, const unsigned char* zone,
                                int zshift, float noise = 0.0f) {
    const uint32_t ba = mxq_bits(a);
    const uint32_t ua = ba & 0x7FFFFFFFu;
    int e = 0;
    if (f.ebits != 0) {
        int k = (int)(ua >> 23) - 127;          // subnormal or zero: below every min_exp
        if (ua >= 0x00800000u) {
            uint32_t gap = 0x1000000u - ((ua & 0x7FFFFFu) | 0x800000u);
            k += (gap <= ((uint32_t)zone[k + 149] << zshift)) ? 1 : 0;
        }
        e = k > f.min_exp ? k : f.min_exp;
        // 2**e = inf (fp16: from 2^16) -> x / inf = 0 and 0 * inf
        if (e >= (DT == MXQ_F16OPS ? 16 : 128)) return mxq_float(MXQ_QNAN_BITS);
    }
    float s = mxq_round_dt<DT>(mxq_ldexp(mxq_float(ua), -e));  // out / 2**e
    // sign(.) is taken of this quotient: where it underflowed to zero (e = 1 and the smallest subnormal)
    // the result is +0 like for a zero input
    const bool nonzero = s != 0.0f;
    s = mxq_round_dt<DT>(mxq_ldexp(s, f.t));                   // * 2**(bits-2)
    float r;
    if (RMODE == MXQ_FLOOR) {
        r = floorf(s);
    } else if (RMODE == MXQ_NEAREST) {
        r = floorf(mxq_round_dt<DT>(s + 0.5f));
    } else if (RMODE == MXQ_DITHER) {
        r = floorf(mxq_round_dt<DT>(s + noise));
    } else {
        float d = mxq_round_dt<DT>(s - 0.5f);
        float h = d * 0.5f;
        float tie = (h == floorf(h)) ? 1.0f : 0.0f;         // (|v| - 0.5) % 2 == 0
        r = floorf(mxq_round_dt<DT>(s + 0.5f)) - tie;
    }
    float y = mxq_round_dt<DT>(mxq_ldexp(r, -f.t));
    y = mxq_round_dt<DT>(mxq_ldexp(y, e));
    uint32_t uy = mxq_bits(y) & 0x7FFFFFFFu;
    if (uy > f.max_bits) uy = (saturate || f.ebits == 0) ? f.max_bits : MXQ_INF_BITS;
    return mxq_float(uy | (nonzero ? (ba & 0x80000000u) : 0u));
}

// One element of an MX block: x / 2^se -> round -> * 2^se  (mx/mx_ops.py:285-292).  The result
// still has to be rounded to the tensor dtype (mxq_round_dt, or the packing conversion).
// LEAN: see mxq_round_lean for when it may be used.
template <int RMODE, int DT, bool ZONE, bool LEAN>
MXQ_HD float mxq_quant_mx_elem_raw(float x, const MxqScale& sc, const MxqFmt& f,
                                   const unsigned char* zone, int zshift, float noise = 0.0f) {
    const float a = x * sc.inv_scale;
    float y;
    if (LEAN) {
        // a bf16-subnormal quotient is not rounded to bf16 here: it rounds to zero in the element
        // format either way, only its sign needs the bf16 view (mxq_sign_source)
        y = mxq_round_lean<RMODE, ZONE>(a, mxq_sign_source<DT>(a), f, true, zone, zshift);
    } else {
        y = mxq_round_every_op<RMODE, DT>(mxq_round_dt<DT>(a), f, true, zone, zshift, noise);
    }
    return y * sc.scale;
}
template <int RMODE, int DT, bool ZONE, bool LEAN>
MXQ_HD float mxq_quant_mx_elem(float x, const MxqScale& sc, const MxqFmt& f,
                               const unsigned char* zone, int zshift, float noise = 0.0f) {
    return mxq_round_dt<DT>(mxq_quant_mx_elem_raw<RMODE, DT, ZONE, LEAN>(x, sc, f, zone, zshift, noise));
}

// The same element, but as (value relative to the block scale): what a packed MX tensor stores.
// Only element formats with at most 6 fraction bits exist in packed form, so the lean rounding
// always applies.
template <int RMODE, int DT, bool ZONE>
MXQ_HD float mxq_quant_mx_elem_unscaled(float x, const MxqScale& sc, const MxqFmt& f,
                                        const unsigned char* zone, int zshift) {
    const float a = x * sc.inv_scale;
    return mxq_round_lean<RMODE, ZONE>(a, mxq_sign_source<DT>(a), f, true, zone, zshift);
}

// The same element as the code of its own format, without the detour over the float value: with
// k = the rounded significand at exponent e (mxq_round_lean's r and ebc), the magnitude code is
// ((e - min_exp) << t) + k -- for subnormals (e = min_exp, k < 2^t) that is k, for normals the
// implicit one of k adds 1 to the exponent field, and a k that rounded up to 2^(t+1) carries into
// the next exponent.  Codes grow with the magnitude, so saturation is a clamp of the code at
// max_code, the code of max_norm.  SIGN_POS: bit of the sign in the code.  Not for the round-up
// zone variant (there e can exceed the exponent of the value).  NaN inputs give an arbitrary code
// (their block's scale byte says NaN).
template <int RMODE, int DT, int SIGN_POS>
MXQ_HD uint32_t mxq_quant_mx_code(float x, const MxqScale& sc, const MxqFmt& f, uint32_t max_code) {
    const float a = x * sc.inv_scale;
    const uint32_t ua = mxq_bits(a) & 0x7FFFFFFFu;
    const uint32_t eb = ua >> 23;
    const uint32_t ebc = eb > f.min_eb ? eb : f.min_eb;
    const float s = mxq_ldexp(mxq_float(ua), f.t127 - (int)ebc);   // exact
    float r;
    if (RMODE == MXQ_FLOOR) {
        r = floorf(s);
    } else if (RMODE == MXQ_NEAREST) {
        r = floorf(s + f.half);
    } else {
        r = __builtin_rintf(s);
        r = (s == f.tie_fix) ? 1.0f : r;
    }
    uint32_t mag = ((ebc - f.min_eb) << f.t) + (uint32_t)r;
    mag = mag < max_code ? mag : max_code;
    return mag | ((mxq_bits(mxq_sign_source<DT>(a)) >> 31) << SIGN_POS);
}

// max_code of the above for a format whose max_norm is one of its own values; 0 otherwise (then
// the caller rounds to the float value and encodes that)
inline uint32_t mxq_max_code(const MxqFmt& f) {
    if (f.ebits == 0 || f.t > 22) return 0u;
    const uint32_t eb = f.max_bits >> 23, frac = f.max_bits & 0x7FFFFFu;
    if (eb < f.min_eb || eb >= 255u || (frac & ((1u << (23 - f.t)) - 1u)) != 0u) return 0u;
    return ((eb - f.min_eb) << f.t) + (1u << f.t) + (frac >> (23 - f.t));
}

// OCP 8-bit float codes of a value that is exactly representable in the format (no rounding
// happens here).  e4m3 is the "fn" variant: bias 7, subnormals m * 2^-9, no infinities.
MXQ_HD uint32_t mxq_encode_e4m3(float y) {
    const uint32_t u = mxq_bits(y), ua = u & 0x7FFFFFFFu;
    const uint32_t normal = (ua >> 20) - (120u << 3);               // ((e + 7) << 3) | mantissa
    const uint32_t subnormal = (uint32_t)(mxq_float(ua) * 512.0f);  // |y| / 2^-9
    return ((u >> 24) & 0x80u) | ((ua >> 23) >= 121u ? normal : subnormal);
}
// e5m2: bias 15, subnormals m * 2^-16
MXQ_HD uint32_t mxq_encode_e5m2(float y) {
    const uint32_t u = mxq_bits(y), ua = u & 0x7FFFFFFFu;
    const uint32_t normal = (ua >> 21) - (112u << 2);
    const uint32_t subnormal = (uint32_t)(mxq_float(ua) * 65536.0f);
    return ((u >> 24) & 0x80u) | ((ua >> 23) >= 113u ? normal : subnormal);
}
MXQ_HD float mxq_decode_e4m3(uint32_t c) {
    const uint32_t e = (c >> 3) & 15u, m = c & 7u;
    const float v = e ? mxq_ldexp((float)(8u + m), (int)e - 10) : mxq_ldexp((float)m, -9);
    return (c & 0x80u) ? -v : v;
}
MXQ_HD float mxq_decode_e5m2(uint32_t c) {
    const uint32_t e = (c >> 2) & 31u, m = c & 3u;
    const float v = e ? mxq_ldexp((float)(4u + m), (int)e - 17) : mxq_ldexp((float)m, -16);
    return (c & 0x80u) ? -v : v;
}

// OCP e2m1 (fp4) code of a value that the format represents exactly: 0, 0.5, 1, 1.5, 2, 3, 4, 6
MXQ_HD uint32_t mxq_encode_e2m1(float y) {
    const uint32_t u = mxq_bits(y), ua = u & 0x7FFFFFFFu;
    const uint32_t normal = (ua >> 22) - 252u;                      // ((e + 1) << 1) | mantissa bit
    const uint32_t subnormal = (uint32_t)(mxq_float(ua) * 2.0f);    // 0 or 0.5
    return ((u >> 28) & 0x8u) | (ua >= 0x3F800000u ? normal : subnormal);
}
MXQ_HD float mxq_decode_e2m1(uint32_t c) {
    const uint32_t e = (c >> 1) & 3u, m = c & 1u;
    const float v = e ? mxq_ldexp((float)(2u + m), (int)e - 2) : 0.5f * (float)m;
    return (c & 0x8u) ? -v : v;
}

// OCP 6-bit codes of values the formats represent exactly.  e2m3: sign, 2 exponent bits (bias 1),
// 3 fraction bits -- up to 7.5 in steps of 1/8 below 1.  e3m2: 3 exponent bits (bias 3), 2 fraction
// bits -- up to 28, steps of 1/16 below 1/4.  MANT = fraction bits, BIAS = exponent bias.
template <int MANT, int BIAS>
MXQ_HD uint32_t mxq_encode_fp6(float y) {
    const uint32_t u = mxq_bits(y), ua = u & 0x7FFFFFFFu;
    const uint32_t normal = (ua >> (23 - MANT)) - ((uint32_t)(127 - BIAS) << MANT);
    const uint32_t subnormal = (uint32_t)(mxq_float(ua) * (float)(1 << (BIAS - 1 + MANT)));
    return ((u >> 26) & 0x20u) | (ua >= ((uint32_t)(128 - BIAS) << 23) ? normal : subnormal);
}
template <int MANT, int BIAS>
MXQ_HD float mxq_decode_fp6(uint32_t c) {
    const uint32_t e = (c >> MANT) & ((1u << (5 - MANT)) - 1u), m = c & ((1u << MANT) - 1u);
    const float v = e ? mxq_ldexp((float)((1u << MANT) + m), (int)e - BIAS - MANT)
                      : mxq_ldexp((float)m, 1 - BIAS - MANT);
    return (c & 0x20u) ? -v : v;
}

// E8M0 byte of a block scale: exponent + 127, 255 for a NaN block (MxqScale.scale is NaN)
MXQ_HD uint32_t mxq_encode_e8m0(float scale) {
    const uint32_t u = mxq_bits(scale);
    if (u > MXQ_INF_BITS) return 255u;
    return (u >> 23) ? (u >> 23) : 0u;            // 2^-127 is the fp32 subnormal 0x00400000 -> 0
}

// The elementwise quantizer for the commonest case, closed form: a bf16 tensor rounded to bfloat16
// (8 exponent bits, bits = 9), round-half-away, subnormals allowed, overflow to Inf.  The format
// holds every bf16 value, yet the op-by-op arithmetic is not the identity: the scaled significand
// is an integer in [128, 256) (or, in the round-up zone of the exponent, a half-integer in
// [64, 128)), and "+ 0.5" then moves an odd significand to the next even one.  Subnormals scale
// below 128 and stay.  x: already a bf16 value.
MXQ_HD float mxq_quant_bf16_to_bfloat16_nearest(float x, uint32_t nan_from) {
    const uint32_t u = mxq_bits(x), ua = u & 0x7FFFFFFFu;
    uint32_t r = u + (u & 0x10000u);                      // odd significand -> + 1 (may carry to Inf)
    r = (ua >> 23) == 0u ? (ua == 0u ? 0u : u) : r;       // subnormals stay, +-0 -> +0
    if (ua >= nan_from) r = (ua == MXQ_INF_BITS) ? u : MXQ_QNAN_BITS;
    return mxq_float(r);
}

// The same closed form for values known to be >= +0, below 2^127, or NaN / +Inf (exponentials, their
// sums and quotients): no sign of zero to fix and no top-binade zone to reach.
MXQ_HD float mxq_quant_bf16_to_bfloat16_nearest_nonneg(float x) {
    const uint32_t u = mxq_bits(x);
    return mxq_float(u + ((u - 0x00800000u) < 0x7F000000u ? (u & 0x10000u) : 0u));   // finite normals only
}

// One element of the elementwise quantizer (mx/elemwise_ops.py:127-163).
template <int RMODE, int DT, bool ZONE, bool LEAN>
MXQ_HD float mxq_quant_elemwise(float x, const MxqFmt& f, bool saturate, bool allow_denorm,
                                const unsigned char* zone, int zshift, float noise = 0.0f) {
    const uint32_t ux = mxq_bits(x) & 0x7FFFFFFFu;
    float y;
    if (LEAN) y = mxq_round_lean<RMODE, ZONE, DT == MXQ_BF16>(x, x + 0.0f, f, saturate || f.ebits == 0, zone, zshift);
    else y = mxq_round_every_op<RMODE, DT>(ux < MXQ_INF_BITS ? x : 0.0f, f, saturate, zone, zshift, noise);
    // (|A| >= min_norm) * A is +-0, and sign(+-0) is 0
    if (!allow_denorm && f.ebits > 0 && (ux >> 23) < f.min_eb) y = 0.0f;
    // exponent 128: 2**128 = inf and the value turns into 0 * inf.  +-Inf is restored after the
    // clamp (161-162); NaN propagates
    if (ux >= f.nan_from) y = (ux == MXQ_INF_BITS) ? x : mxq_float(MXQ_QNAN_BITS);
    return y;
}
