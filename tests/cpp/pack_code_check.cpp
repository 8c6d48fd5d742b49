// Host check (compiled and run by tests/test_host_library.py): the code that the pack kernels derive
// straight from the rounded significand (mxq_quant_mx_code) equals the encoding of the rounded float
// value (mxq_quant_mx_elem_unscaled, then mxq_encode_*) for every input a block can hold -- every
// bf16 code and a random fp32 sample, under block scales 2^-126 .. 2^127 and in a flushed block.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include "mxq_params.h"
using namespace mxq_detail;

static uint32_t encode(int kind, float y) {
    switch (kind) {
        case 1: return mxq_encode_e5m2(y);
        case 2: return mxq_encode_fp6<3, 1>(y);
        case 3: return mxq_encode_fp6<2, 3>(y);
        case 4: return mxq_encode_e2m1(y);
        default: return mxq_encode_e4m3(y);
    }
}
template <int RMODE, int DT, int SP>
static long run(int kind, int ebits, int mbits, float maxn, int dtype, int rmode) {
    MxParams p; bool ze;
    if (make_mx_params(dtype, 8, ebits, mbits, maxn, 0, rmode, 0, &p, &ze, "chk")) { printf("params failed\n"); exit(1); }
    if (ze) { printf("  (zone variant, skipped) "); return 0; }
    const uint32_t mc = mxq_max_code(p.fmt);
    if (!mc) { printf("no max code\n"); exit(1); }
    const unsigned char* zone = zone_rows[p.zone_row == ZONE_ROW_NONE ? 0 : p.zone_row];
    long n = 0, bad = 0;
    std::mt19937 rng(123);
    for (int se = -130; se <= 127; se += (se > -20 && se < 20) ? 1 : 7) {
        MxqScale sc; sc.scale = ldexpf(1.0f, se); sc.inv_scale = ldexpf(1.0f, -se);
        if (se == -130) { sc.inv_scale = 0.0f; sc.scale = 1.0f; }          // flushed block
        const int count = (DT == MXQ_BF16) ? 65536 : (1 << 17);
        for (int i = 0; i < count; ++i) {
            uint32_t bits = (DT == MXQ_BF16) ? (uint32_t)i << 16 : (uint32_t)rng();
            float x = mxq_float(bits);
            if ((bits & 0x7FFFFFFFu) >= 0x7F800000u) continue;
            float a = x * sc.inv_scale;
            if (!(fabsf(a) < ldexpf(1.0f, p.emax + 1))) continue;             // not inside a block with this scale
            float y = mxq_quant_mx_elem_unscaled<RMODE, DT, false>(x, sc, p.fmt, zone, p.zshift);
            uint32_t want = encode(kind, y);
            uint32_t got = mxq_quant_mx_code<RMODE, DT, SP>(x, sc, p.fmt, mc);
            ++n;
            if (want != got && bad++ < 5) printf("\n  MISMATCH x=%a se=%d want %x got %x (y=%a)", x, se, want, got, y);
        }
    }
    if (bad) { printf("\n  %ld mismatches of %ld\n", bad, n); exit(1); }
    return n;
}
int main() {
    struct F { const char* name; int kind, ebits, mbits; float maxn; int sp; } fs[] = {
        {"e4m3", 0, 4, 5, 448.f, 7}, {"e5m2", 1, 5, 4, 57344.f, 7}, {"e2m3", 2, 2, 5, 7.5f, 5},
        {"e3m2", 3, 3, 4, 28.f, 5}, {"e2m1", 4, 2, 3, 6.f, 3}};
    for (auto& f : fs)
        for (int dt = 0; dt < 2; ++dt)
            for (int rm = 0; rm < 3; ++rm) {
                printf("%s dtype %d rmode %d: ", f.name, dt, rm); fflush(stdout);
                long n = 0;
#define CASE(R, D, S) if (rm == R && dt == (D == MXQ_BF16 ? 1 : 0) && f.sp == S) n = run<R, D, S>(f.kind, f.ebits, f.mbits, f.maxn, D == MXQ_BF16 ? MXQ_DTYPE_BF16 : MXQ_DTYPE_F32, R);
#define CASES(S) CASE(0, MXQ_F32, S) CASE(1, MXQ_F32, S) CASE(2, MXQ_F32, S) CASE(0, MXQ_BF16, S) CASE(1, MXQ_BF16, S) CASE(2, MXQ_BF16, S)
                CASES(7) CASES(5) CASES(3)
                printf("%ld inputs agree\n", n);
            }
    return 0;
}
