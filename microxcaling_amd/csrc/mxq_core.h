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
enum MxqRound { MXQ_NEAREST = 0, MXQ_FLOOR = 1, MXQ_EVEN = 2 };   // mx/formats.py:12-19

#define MXQ_QNAN_BITS 0x7FC00000u
#define MXQ_INF_BITS 0x7F800000u

MXQ_HD uint32_t mxq_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
MXQ_HD float mxq_float(uint32_t u) { return __builtin_bit_cast(float, u); }

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

template <int DT>
MXQ_HD float mxq_round_dt(float f) {
    if (DT == MXQ_BF16) return mxq_round_bf16(f);
    return f;
}

// ---- element format ----------------------------------------------------------------------------
struct MxqFmt {
    int ebits;          // exponent bits, 0 for integer formats
    int t;              // fraction bits kept = mbits - 2 (mbits counts sign and implicit one)
    int min_exp;        // 2 - 2^(ebits-1): exponent of the smallest normal (mx/elemwise_ops.py:139)
    uint32_t max_bits;  // bit pattern of max_norm (already rounded to the tensor dtype)
};

// ---- floor(log2(x)) in the tensor dtype --------------------------------------------------------
// ua: |x| in fp32 layout, finite and non-zero.  zone[k+149] / zshift: see gen_log2_tables.py.
MXQ_HD int mxq_floor_log2(uint32_t ua, const unsigned char* zone, int zshift) {
    int be = (int)(ua >> 23);
    uint32_t man = ua & 0x7FFFFFu;
    int k;
    uint32_t sig;
    if (be != 0) {
        k = be - 127;
        sig = man | 0x800000u;
    } else {                                    // fp32 subnormal: normalise
        int lz = __builtin_clz(man);            // man != 0
        sig = man << (lz - 8);
        k = -118 - lz;
    }
    uint32_t gap = 0x1000000u - sig;
    return k + (gap <= ((uint32_t)zone[k + 149] << zshift) ? 1 : 0);
}

// 2^n as fp32 for n in [-149, 127]
MXQ_HD float mxq_pow2(int n) {
    return mxq_float(n >= -126 ? (uint32_t)(n + 127) << 23 : 0x00400000u >> (-127 - n));
}

// ---- shared exponent of one block (mx/mx_ops.py:269-283) ---------------------------------------
struct MxqScale {
    float scale;      // 2^se
    float inv_scale;  // 2^-se
    bool nan;         // block becomes NaN: max is Inf/NaN or the scale exponent overflows
    bool flush;       // block becomes +0: max is an fp32 subnormal and flushing was requested
};

// um: max |x| of the block as an fp32-layout bit pattern (0x7F800000 and above = Inf/NaN seen).
MXQ_HD MxqScale mxq_block_scale(uint32_t um, int emax, int scale_emax, bool flush_subnorms,
                                const unsigned char* zone, int zshift) {
    MxqScale r;
    r.nan = um >= MXQ_INF_BITS;
    int E = (um == 0u || r.nan) ? -126 : mxq_floor_log2(um, zone, zshift);
    r.flush = flush_subnorms && E <= -127;
    int se = E - emax;
    if (se > scale_emax) r.nan = true;
    if (se < -scale_emax) se = -scale_emax;
    if (r.nan) se = 0;
    r.scale = mxq_pow2(se);
    r.inv_scale = mxq_pow2(-se);
    return r;
}

// ---- element rounding (mx/elemwise_ops.py:134-157) ---------------------------------------------
// a: finite input already in the tensor dtype.  Returns the quantized value before any block
// scale is re-applied.  FULL = round to the dtype after every op like torch does; !FULL drops the
// roundings that provably never change a bf16 result when t <= 6 (checked exhaustively on the
// host against the FULL variant and the torch oracle).
template <int RMODE, int DT, bool ZONE, bool FULL>
MXQ_HD float mxq_quant_finite(float a, const MxqFmt& f, bool saturate,
                              const unsigned char* zone, int zshift) {
    const uint32_t ba = mxq_bits(a);
    const uint32_t ua = ba & 0x7FFFFFFFu;
    int e = 0;
    if (f.ebits != 0) {
        int k = (int)(ua >> 23) - 127;          // subnormal or zero: below every min_exp
        if (ZONE && ua >= 0x00800000u) {
            uint32_t gap = 0x1000000u - ((ua & 0x7FFFFFu) | 0x800000u);
            k += (gap <= ((uint32_t)zone[k + 149] << zshift)) ? 1 : 0;
        }
        e = k > f.min_exp ? k : f.min_exp;
        if (e >= 128) return mxq_float(MXQ_QNAN_BITS);    // 2**128 = inf -> 0 * inf
    }
    const float mag = mxq_float(ua);
    float s;
    if (FULL) {
        s = mxq_round_dt<DT>(ldexpf(mag, -e));             // out / 2**e
        s = mxq_round_dt<DT>(ldexpf(s, f.t));              // * 2**(bits-2)
    } else {
        s = ldexpf(mag, f.t - e);
    }
    float r;
    if (RMODE == MXQ_FLOOR) {
        r = floorf(s);
    } else if (RMODE == MXQ_NEAREST) {
        r = floorf(mxq_round_dt<DT>(s + 0.5f));
    } else {
        float d = s - 0.5f;
        if (FULL) d = mxq_round_dt<DT>(d);
        float h = d * 0.5f;
        float tie = (h == floorf(h)) ? 1.0f : 0.0f;        // (|v| - 0.5) % 2 == 0
        r = floorf(mxq_round_dt<DT>(s + 0.5f)) - tie;
    }
    float y;
    if (FULL) {
        y = mxq_round_dt<DT>(ldexpf(r, -f.t));
        y = mxq_round_dt<DT>(ldexpf(y, e));
    } else {
        y = ldexpf(r, e - f.t);
    }
    uint32_t uy = mxq_bits(y) & 0x7FFFFFFFu;
    if (uy > f.max_bits) uy = (saturate || f.ebits == 0) ? f.max_bits : MXQ_INF_BITS;
    // sign(a) * r: -0.0 when a negative value rounds to zero, +0.0 for a = +-0
    return mxq_float(uy | (ua != 0u ? (ba & 0x80000000u) : 0u));
}

// One element of an MX block: x / 2^se -> round -> * 2^se  (mx/mx_ops.py:285-292).
template <int RMODE, int DT, bool ZONE, bool FULL>
MXQ_HD float mxq_quant_mx_elem(float x, const MxqScale& sc, const MxqFmt& f,
                               const unsigned char* zone, int zshift) {
    if (sc.nan) return mxq_float(MXQ_QNAN_BITS);
    if (sc.flush) return 0.0f;
    float a = mxq_round_dt<DT>(x * sc.inv_scale);
    float y = mxq_quant_finite<RMODE, DT, ZONE, FULL>(a, f, true, zone, zshift);
    return mxq_round_dt<DT>(y * sc.scale);
}

// One element of the elementwise quantizer (mx/elemwise_ops.py:127-163).
template <int RMODE, int DT, bool FULL>
MXQ_HD float mxq_quant_elemwise(float x, const MxqFmt& f, bool saturate, bool allow_denorm,
                                const unsigned char* zone, int zshift) {
    const uint32_t bx = mxq_bits(x);
    const uint32_t ux = bx & 0x7FFFFFFFu;
    if (ux > MXQ_INF_BITS) return mxq_float(MXQ_QNAN_BITS);   // NaN propagates
    if (ux == MXQ_INF_BITS) return x;                          // +-Inf restored (161-162)
    if (!allow_denorm && f.ebits > 0 && (int)(ux >> 23) - 127 < f.min_exp) {
        // (|A| >= min_norm) * A gives +-0, whose sign() is 0; but the exponent still comes from A,
        // and 2**128 = inf turns the zero into NaN for values in the top round-up zone.
        return 0.0f;
    }
    return mxq_quant_finite<RMODE, DT, true, FULL>(x, f, saturate, zone, zshift);
}
