// The arithmetic of the stand-in's matrix instruction, kept in a file of its own so that it can be compiled
// with optimization while the kernels around it are compiled without (they are large and compile slowly).
#include <math.h>
#include <stdint.h>

namespace emu {

static double decode8_slow(unsigned char c, int fmt) {                       // 0: e4m3 (OCP "fn"), 1: e5m2
    const int ebits = fmt == 0 ? 4 : 5, mbits = 7 - ebits, bias = fmt == 0 ? 7 : 15;
    const int e = (c >> mbits) & ((1 << ebits) - 1), m = c & ((1 << mbits) - 1);
    const double sign = (c & 0x80) ? -1.0 : 1.0;
    if (fmt == 0 && e == 15 && m == 7) return NAN;                           // S.1111.111
    if (fmt == 1 && e == 31) return m ? NAN : sign * INFINITY;
    if (e == 0) return sign * ldexp((double)m, 1 - bias - mbits);
    return sign * ldexp((double)((1 << mbits) + m), e - bias - mbits);
}

// One row (column) of an operand of v_mfma_scale_f32_*_f8f6f4 as K doubles.  regs[g]: the 8 operand registers
// of the lane of that row in group g; ktot = 32 * groups.  8-bit formats: group g holds K = 16 g .. 16 g + 15 of
// the first half of K in registers 0-3 and the same of the second half in registers 4-7; e2m1 (fmt 4): K =
// 32 g .. 32 g + 31 as nibbles (the lower K in the low nibble) in registers 0-3.
void decode_row(const void* const* regs, int groups, int fmt, double* out) {
    static double table[2][256];
    static bool ready = false;
    if (!ready) {                                                             // idempotent: a race only repeats it
        for (int f = 0; f < 2; ++f)
            for (int v = 0; v < 256; ++v) table[f][v] = decode8_slow((unsigned char)v, f);
        ready = true;
    }
    static const double mag[8] = {0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0};
    const int ktot = 32 * groups, half = ktot / 2;
    for (int k = 0; k < ktot; ++k) {
        if (fmt == 4) {
            const unsigned char* p = static_cast<const unsigned char*>(regs[k / 32]);
            const int nib = (p[(k % 32) >> 1] >> (4 * (k & 1))) & 15;
            out[k] = (nib & 8) ? -mag[nib & 7] : mag[nib & 7];
        } else if (fmt == 0 || fmt == 1) {
            const unsigned char* p = static_cast<const unsigned char*>(regs[(k % half) / 16]);
            out[k] = table[fmt][p[(k / half) * 16 + k % 16]];
        } else {
            __builtin_trap();                                                 // the 6-bit formats are not used
        }
    }
}

// sum over the K blocks of 32 of (sum of products) * 2^(sa - 127) * 2^(sb - 127); a scale byte of 255 is NaN
double scaled_dot(const double* a, const double* b, const int* scale_a, const int* scale_b, int groups) {
    double sum = 0.0;
    for (int kb = 0; kb < groups; ++kb) {
        double part = 0.0;
        for (int k = 32 * kb; k < 32 * kb + 32; ++k) part += a[k] * b[k];
        const double sa = scale_a[kb] == 255 ? NAN : ldexp(1.0, scale_a[kb] - 127);
        const double sb = scale_b[kb] == 255 ? NAN : ldexp(1.0, scale_b[kb] - 127);
        sum += part * sa * sb;
    }
    return sum;
}

}  // namespace emu
