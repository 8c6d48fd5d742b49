/* Scalar C restatement of the reference's pure-PyTorch quantization path.  TEST INFRASTRUCTURE
 * ONLY: it checks the HIP kernels and the torch oracle (mx_oracle.py); no product code links it.
 *
 * Every torch tensor op of the reference becomes one IEEE fp32 operation followed, for bf16 and
 * fp16 tensors, by a round-to-nearest-even to that dtype -- which is how torch's CPU kernels
 * evaluate ops on 16-bit tensors.  log2 is taken in double and rounded to fp32 (then to the tensor dtype), i.e. a correctly
 * rounded log2; torch's CPU log2 agrees with that on every input the tests sweep.  Nothing here
 * shares code with the kernels: exponents come from log2(), not from bit fields or tables.
 *
 * Parity status: every function here is pinned by the golden vectors written from the reference
 * itself (tests/golden/) and by the literal vectors of the reference's tests.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };
enum { RD_NEAREST = 0, RD_FLOOR = 1, RD_EVEN = 2 };     /* mx/formats.py:12-19 */

static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> fp16 bits, round to nearest even: subnormals down to 2^-24, Inf from 65520 */
static uint16_t f2h(float v) {
    uint32_t u = f2u(v), sign = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);          /* >= 2^16 (or Inf) */
    double d = fabs((double)v);
    /* units of the result: 2^(e-10) for a normal of exponent e >= -14, 2^-24 below */
    int e;
    frexp(d, &e);                                                     /* d = m * 2^e, 0.5 <= m < 1 */
    e -= 1;
    if (d == 0.0) return (uint16_t)sign;
    if (e < -14) e = -14;
    double q = ldexp(d, 10 - e);                                      /* exact: in [0, 2048) */
    double n = nearbyint(q);                                          /* ties to even (default mode) */
    uint32_t mant = (uint32_t)n;                                      /* may be 2048: carries */
    uint32_t h = (uint32_t)(e + 14) * 1024u + mant;                   /* subnormal: field 0 + mant */
    return (uint16_t)(sign | h);                                      /* 65520 and up gives 0x7C00 */
}
static float h2f(uint16_t h) {
    uint32_t e = (h >> 10) & 31u, m = h & 1023u;
    float v = e == 31u ? (m ? NAN : INFINITY) : e ? ldexpf((float)(1024u + m), (int)e - 25) : ldexpf((float)m, -24);
    return (h & 0x8000u) ? -v : v;
}

/* result of a torch op on a tensor of dtype dt */
static float R(float v, int dt) {
    if (dt == DT_F16) return h2f(f2h(v));
    if (dt != DT_BF16) return v;
    uint32_t u = f2u(v);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return u2f(0x7FC00000u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u2f(u & 0xFFFF0000u);
}

static float t_log2(float v, int dt) { return R((float)log2((double)v), dt); }
/* 2 ** e for a tensor e holding integers, NaN or +-Inf */
static float t_pow2(float e, int dt) {
    if (e != e) return e;
    if (e >= 128.0f) return INFINITY;
    if (e < -200.0f) return 0.0f;
    return R(ldexpf(1.0f, (int)e), dt);
}
static float t_sign(float v) { return (float)((v > 0.0f) - (v < 0.0f)); }
static float scalar_in(float s, int dt) { return R(s, dt); }     /* python scalar cast to the dtype */

/* mx/elemwise_ops.py:45-76 */
static float round_scaled(float v, int rmode, int dt) {
    float mag = fabsf(v);
    if (rmode == RD_FLOOR) return R(t_sign(v) * floorf(mag), dt);
    if (rmode == RD_NEAREST) return R(t_sign(v) * floorf(R(mag + 0.5f, dt)), dt);
    float d = R(mag - 0.5f, dt);
    float m = fmodf(d, 2.0f);
    if (m != 0.0f && m < 0.0f) m += 2.0f;                        /* python-style remainder */
    float tie = (m == 0.0f) ? 1.0f : 0.0f;
    return R(t_sign(v) * R(floorf(R(mag + 0.5f, dt)) - tie, dt), dt);
}

/* mx/elemwise_ops.py:127-163 */
static float elem_core(float a, int bits, int exp_bits, float max_norm, int rmode, int saturate,
                       int allow_denorm, int dt) {
    float out = a;
    if (!allow_denorm && exp_bits > 0) {
        float min_norm = ldexpf(1.0f, 2 - (1 << (exp_bits - 1)));
        out = R(((fabsf(a) >= scalar_in(min_norm, dt)) ? 1.0f : 0.0f) * a, dt);
    }
    float pe = 0.0f;
    if (exp_bits != 0) {
        float z = (a == 0.0f) ? 1.0f : 0.0f;
        pe = floorf(t_log2(R(fabsf(a) + z, dt), dt));
        float min_exp = (float)(2 - (1 << (exp_bits - 1)));
        if (pe < min_exp) pe = min_exp;                          /* clip(min=); NaN stays NaN */
        out = R(out / t_pow2(pe, dt), dt);
    }
    out = R(out * (float)(1 << (bits - 2)), dt);
    out = round_scaled(out, rmode, dt);
    out = R(out / (float)(1 << (bits - 2)), dt);
    if (exp_bits != 0) out = R(out * t_pow2(pe, dt), dt);
    float mx = scalar_in(max_norm, dt);
    if (saturate || exp_bits == 0) {
        if (out == out) out = out > mx ? mx : (out < -mx ? -mx : out);   /* clamp keeps NaN */
    } else if (fabsf(out) > mx) {
        out = t_sign(out) * INFINITY;
    }
    if (a == INFINITY) out = INFINITY;
    if (a == -INFINITY) out = -INFINITY;
    return out;
}

static float load(const void* p, int dt, int64_t i) {
    if (dt == DT_F32) return ((const float*)p)[i];
    if (dt == DT_F16) return h2f(((const uint16_t*)p)[i]);
    return u2f((uint32_t)((const uint16_t*)p)[i] << 16);
}
static void store(void* p, int dt, int64_t i, float v) {
    if (dt == DT_F32) ((float*)p)[i] = v;
    else if (dt == DT_F16) ((uint16_t*)p)[i] = f2h(v);
    else ((uint16_t*)p)[i] = (uint16_t)(f2u(R(v, DT_BF16)) >> 16);
}

void oracle_quantize_elemwise(const void* in, void* out, int dt, int64_t n, int bits, int exp_bits,
                              float max_norm, int rmode, int saturate, int allow_denorm) {
    for (int64_t i = 0; i < n; ++i)
        store(out, dt, i, elem_core(load(in, dt, i), bits, exp_bits, max_norm, rmode, saturate,
                                    allow_denorm, dt));
}

/* mx/mx_ops.py:265-292 on a (pre, axis, post) tensor, blocks of `block` along the middle axis
 * (a ragged last block is the zero-padded block of mx/mx_ops.py:114-131). */
void oracle_quantize_mx(const void* in, void* out, int dt, int64_t pre, int64_t axis, int64_t post,
                        int scale_bits, int ebits, int mbits, int emax, float max_norm,
                        int64_t block, int flush, int rmode) {
    if (block <= 0 || block > axis) block = axis;
    const float scale_emax = (float)((1 << (scale_bits - 1)) - 1);
    for (int64_t i = 0; i < pre; ++i)
        for (int64_t k0 = 0; k0 < axis; k0 += block)
            for (int64_t j = 0; j < post; ++j) {
                const int64_t k1 = k0 + block < axis ? k0 + block : axis;
                float m = 0.0f;                                   /* torch.max propagates NaN */
                for (int64_t k = k0; k < k1; ++k) {
                    float v = fabsf(load(in, dt, (i * axis + k) * post + j));
                    if (v != v || m != m) m = NAN; else if (v > m) m = v;
                }
                float z = (m == 0.0f) ? 1.0f : 0.0f;              /* mx/mx_ops.py:76-80 */
                float se = floorf(t_log2(R(m + R(ldexpf(1.0f, -126) * z, dt), dt), dt));
                float keep = (se > -127.0f) ? 1.0f : 0.0f;        /* 274-275 */
                se = R(se - (float)emax, dt);
                if (se > scale_emax) se = NAN;
                if (se < -scale_emax) se = -scale_emax;
                float p2 = t_pow2(se, dt);
                for (int64_t k = k0; k < k1; ++k) {
                    const int64_t idx = (i * axis + k) * post + j;
                    float a = load(in, dt, idx);
                    if (flush) a = R(a * keep, dt);
                    a = R(a / p2, dt);
                    a = elem_core(a, mbits, ebits, max_norm, rmode, 1, 1, dt);
                    store(out, dt, idx, R(a * p2, dt));
                }
            }
}
