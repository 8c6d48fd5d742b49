// Softmax over the last axis with an elementwise quantization after every step
// (mx/softmax.py:20-54 over mx/vector_ops.py:38-130): one kernel instead of ten tensor passes.
#pragma once
#include <type_traits>

#include "mxq_kernels.h"

struct SoftmaxParams {
    ElemParams q;      // the elementwise format applied after every step
    int exp_mode;      // 0: exp(x)   1: 2^x (softmax_exp2)   2: 2^Q(x * log2(e) at bfloat16 precision)
    int use_recip;     // divide as e * Q(1 / sum) instead of e / sum (vec_use_recip)
};

namespace {

// WPR (1, 2 or 4) waves per row; a lane keeps VPL 16-byte vectors of the row in registers from the
// load to the store (vector j of lane l of the row's 64 WPR lanes is vector 64 WPR j + l), so the
// row is read once and written once.  Row reductions: shuffles inside a wave, then the waves of a
// row in order through LDS.  QMODE: SMQ_GENERIC = the elementwise quantizer with the format in p.q; SMQ_IDENT = the
// identity on values of the tensor dtype (no format configured, or bfloat16 with round-half-even on
// a bf16 tensor); SMQ_BF16 = closed form for bf16 tensor -> bfloat16, round-half-away.
// Every step rounds to the tensor dtype first, like the tensor op it stands for, then quantizes.
enum { SMQ_GENERIC = 0, SMQ_IDENT = 1, SMQ_BF16 = 2 };

template <int DT, int RMODE, int QMODE, int VPL, int WPR>
__global__ __launch_bounds__(TPB) void softmax_row_kernel(const void* __restrict__ in_,
                                                          void* __restrict__ out_, int64_t rows,
                                                          int n, SoftmaxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    constexpr int EPL = VPL * EPV;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.q.zone_row]);

    auto Qd = [&](float v) {                                 // v already is a value of the tensor dtype
        if (QMODE == SMQ_IDENT) return v;
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest(v, p.q.fmt.nan_from);
        return mxq_quant_elemwise<RMODE, ADT, true, true>(v, p.q.fmt, p.q.saturate != 0,
                                                          p.q.allow_denorm != 0, zone, ZS);
    };
    auto Q = [&](float v) { return Qd(mxq_round_dt<ADT>(v)); };
    // SMQ_BF16, values known to be +0 or normal and far from the top binade: the closed form without
    // its special cases
    auto Qplain_d = [](float v) {                            // v already is a value of the tensor dtype
        const uint32_t u = mxq_bits(v);
        return mxq_float(u + (u & 0x10000u));
    };
    auto Qplain = [&](float v) { return Qplain_d(mxq_round_dt<ADT>(v)); };

    // the quantizer for exponentials, their row sum and the quotients: all >= +0 and <= 4096 (or
    // NaN / +Inf), where the closed form needs no special cases
    auto Qp = [&](float v) {
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest_nonneg(mxq_round_dt<ADT>(v));
        return Q(v);
    };

    constexpr int LPR = 64 * WPR;                            // lanes per row
    constexpr int RPB = (TPB / 64) / WPR;                    // rows per block and iteration
    __shared__ float part[TPB / 64];
    const int wib = threadIdx.x >> 6;                        // wave in block
    const int lane = (wib % WPR) * 64 + (threadIdx.x & 63);  // lane within the row
    const int nvec_row = n / EPV;
    for (int64_t row0 = (int64_t)blockIdx.x * RPB; row0 < rows; row0 += (int64_t)gridDim.x * RPB) {
        const int64_t row = row0 + wib / WPR;
        const int nvec = row < rows ? nvec_row : 0;          // a block's spare waves go through the motions
        const u32x4* in = reinterpret_cast<const u32x4*>(in_) + row * nvec_row;
        u32x4* out = reinterpret_cast<u32x4*>(out_) + row * nvec_row;
        u32x4 raw[VPL];
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int v = j * LPR + lane;
            if (v < nvec) raw[j] = in[v];
        }
        // positions past the end of the row behave like -inf: they drop out of the maximum and
        // contribute exp(-inf) = 0 to the sum
        float x[EPL];
        float m = -__builtin_inff();
        // SMQ_BF16: the special cases of the quantizer (zero, subnormal, Inf, NaN, top binade) cost
        // more than its arithmetic, and rows of logits rarely hold any.  A wave whose inputs all lie
        // in 2^-100 <= |x| < 2^100 quantizes them with the plain closed form; if the row maximum
        // lies there too, every x - m is +0 or a normal number below 2^101 (a multiple of 2^-108),
        // and so is 1.4453125 (x - m): the plain form again.  Any other wave takes the general form.
        bool plain = QMODE == SMQ_BF16 && !p.q.general_only;
        auto in_plain_range = [](uint32_t ua) { return ua - 0x0D800000u < 0x64000000u; };   // [2^-100, 2^100)
        float lowest = __builtin_inff();                     // of this lane's quantized inputs
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const bool valid = j * LPR + lane < nvec;
#pragma unroll
            for (int d = 0; d < 4; ++d)
#pragma unroll
                for (int h = 0; h < PD; ++h) {
                    const int e = (j * 4 + d) * PD + h;
                    const float v = Pack<DT>::get(raw[j][d], h);
                    if (QMODE == SMQ_BF16) {
                        plain = plain && (!valid || in_plain_range(mxq_bits(v) & 0x7FFFFFFFu));
                        x[e] = valid ? Qplain_d(v) : -__builtin_inff();
                        lowest = fminf(lowest, valid ? x[e] : __builtin_inff());
                    } else {
                        x[e] = valid ? Qd(v) : -__builtin_inff();
                    }
                }
        }
        if (QMODE == SMQ_BF16) {
            plain = __all(plain);                            // wave-uniform from here on
            if (!plain) {
#pragma unroll
                for (int j = 0; j < VPL; ++j)
#pragma unroll
                    for (int d = 0; d < 4; ++d)
#pragma unroll
                        for (int h = 0; h < PD; ++h)
                            if (j * LPR + lane < nvec) x[(j * 4 + d) * PD + h] = Qd(Pack<DT>::get(raw[j][d], h));
            }
        }
#pragma unroll
        for (int e = 0; e < EPL; ++e) m = MaxOp::apply(m, x[e]);     // NaN sticks, like torch.max
        m = row_reduce<MaxOp, WPR>(m, part);
        // m is the same in every lane of the row; the vote makes the branch below a scalar one
        if (QMODE == SMQ_BF16) plain = __all(plain && in_plain_range(mxq_bits(m) & 0x7FFFFFFFu));

        float sum = 0.0f;
        auto exponentials = [&](auto plain_tag) {            // one loop per mode: no branch per element
            auto Qs = [&](float v) { return decltype(plain_tag)::value ? Qplain(v) : Q(v); };
            if (p.exp_mode == 0) {
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    x[e] = Qp(expf(Qs(x[e] - m)));
                    sum += x[e];
                }
            } else if (p.exp_mode == 1) {
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    x[e] = Qp(exp2f(Qs(x[e] - m)));
                    sum += x[e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    x[e] = Qp(exp2f(Qs(1.4453125f * Qs(x[e] - m))));
                    sum += x[e];
                }
            }
        };
        // Closer still: when no input of the wave lies more than 85 below the row maximum, the
        // exponentials are normal numbers (2^-123 .. 1; exactly 0 past the end of the row), and when
        // the smallest of them, divided by the row sum, is one too (checked below with a factor 2 to
        // spare), so are the quotients: their quantizer needs no special cases either, and both bf16
        // values of a pair go through it in packed form.
        auto packed = [](float a, float b) {
            const uint32_t w = Pack<MXQ_BF16>::put(a, b);
            return w + (w & 0x00010001u);
        };
        auto low_of = [](uint32_t w) { return mxq_float(w << 16); };
        auto high_of = [](uint32_t w) { return mxq_float(w & 0xFFFF0000u); };
        auto fast_exp2 = [](float v) { return __builtin_amdgcn_exp2f(v); };
        bool close = false;
        if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) close = __all(plain && lowest - m >= -85.0f);
        if (close) {
            if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) {
#pragma unroll
                for (int e = 0; e < EPL; e += 2) {
                    uint32_t dw = packed(x[e] - m, x[e + 1] - m);
                    if (p.exp_mode == 2) dw = packed(1.4453125f * low_of(dw), 1.4453125f * high_of(dw));
                    // arguments in [-85, 0] (2^x: [-123, 0]): the results are normal numbers, which the
                    // hardware exponential (v_exp_f32: about 1 ulp, flushes subnormal results only) returns
                    // without the range handling of expf / exp2f.  For e^x the fp32 product x * log2(e) in
                    // front of it is rounded at magnitudes up to 123 (half an ulp there is 2^-18), which
                    // moves the result by up to 2.6e-6 of its value -- about 45 fp32 ulps at x = -85, not
                    // the 1-2 ulps of expf, and a 1500th of the bfloat16 rounding step that follows.
                    const uint32_t ew = p.exp_mode == 0 ? packed(fast_exp2(1.44269504f * low_of(dw)), fast_exp2(1.44269504f * high_of(dw)))
                                                        : packed(fast_exp2(low_of(dw)), fast_exp2(high_of(dw)));
                    x[e] = low_of(ew);
                    x[e + 1] = high_of(ew);
                    sum += x[e];
                    sum += x[e + 1];
                }
            }
        } else if (QMODE == SMQ_BF16 && plain) {
            exponentials(std::true_type{});
        } else {
            exponentials(std::false_type{});
        }
        sum = Qp(row_reduce<SumOp, WPR>(sum, part));
        if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) {
            const float below = lowest - m;                  // +inf in a lane past the end of the row
            const float smallest = p.exp_mode == 0 ? expf(below)
                                                   : exp2f(p.exp_mode == 2 ? 1.4453125f * below : below);
            close = __all(close && mxq_bits(sum) - 0x3F800000u < 0x0A000000u &&      // 1 <= sum < 2^20
                          0.5f * smallest >= sum * 1.17549435e-38f);                 // quotients >= 2^-125
        }
        const bool recip = p.use_recip != 0;
        const float r = recip ? Qp(1.0f / sum) : 0.0f;
        // e / sum without a division per element: one refined reciprocal per row, then a product
        // and a residual correction.  For operands with 8-bit significands (the dtype-rounded
        // exponentials and sum of a bf16 tensor) this is the correctly rounded fp32 quotient,
        // checked over every pair of significands; fp32 tensors keep the division.
        const float r0 = __builtin_amdgcn_rcpf(sum);
        const float r1 = fmaf(fmaf(-sum, r0, 1.0f), r0, r0);
        auto quotient = [&](float e) {
            if (ADT != MXQ_BF16) return e / sum;
            const float q0 = e * r1;
            return fmaf(fmaf(-q0, sum, e), r1, q0);
        };

#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            u32x4 o;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                bool done = false;
                if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) {
                    if (close) {
                        const float e0 = x[(j * 4 + d) * 2], e1 = x[(j * 4 + d) * 2 + 1];
                        o[d] = recip ? packed(e0 * r, e1 * r) : packed(quotient(e0), quotient(e1));
                        done = true;
                    }
                }
                if (!done) {
                    float q[2];
#pragma unroll
                    for (int h = 0; h < PD; ++h) {
                        const float e = x[(j * 4 + d) * PD + h];
                        q[h] = Qp(recip ? e * r : quotient(e));
                    }
                    o[d] = Pack<DT>::put(q[0], q[PD - 1]);
                }
            }
            if (j * LPR + lane < nvec) __builtin_nontemporal_store(o, &out[j * LPR + lane]);
        }
    }
}

}  // namespace

// ================================================================================================
// LayerNorm / RMSNorm over the last axis with the elementwise quantizer after every step
// (mx/norm_utils.py:25-114 with axes = -1, mx/layernorm.py:100-131): one kernel instead of about
// fifteen tensor passes.  Same work mapping as the softmax kernel.  Besides the output it writes
// what the backward pass of the layer keeps: the normalized input (optional) and one statistic per
// row (LayerNorm: var + eps; RMSNorm: 1 / rms).
//   LayerNorm: mean = Q(Q(sum x) / n); d = Q(x - mean); var = Q(Q(sum Q(d d)) / n);
//              v = Q(var + eps); r = Q(1 / Q(sqrt v)); z = Q(d r); out = Q(Q(w z) + b)
//   RMSNorm:   ms = Q(Q(sum Q(x x)) / n); v = Q(ms + eps); r = Q(1 / Q(sqrt v)); z = Q(x r); same out
// weight and bias are already quantized.
// ================================================================================================
struct NormParams {
    ElemParams q;
    float eps;
    int rms;           // 1: RMSNorm
};

namespace {

template <int DT, int RMODE, int QMODE, int VPL, int WPR>
__global__ __launch_bounds__(TPB) void norm_row_kernel(const void* __restrict__ in_,
                                                       const void* __restrict__ weight_,
                                                       const void* __restrict__ bias_,
                                                       void* __restrict__ out_, void* __restrict__ znorm_,
                                                       void* __restrict__ stat_, int64_t rows, int n,
                                                       NormParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    constexpr int EPL = VPL * EPV;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.q.zone_row]);

    auto Qd = [&](float v) {                                 // v already is a value of the tensor dtype
        if (QMODE == SMQ_IDENT) return v;
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest(v, p.q.fmt.nan_from);
        return mxq_quant_elemwise<RMODE, ADT, true, true>(v, p.q.fmt, p.q.saturate != 0,
                                                          p.q.allow_denorm != 0, zone, ZS);
    };
    auto Q = [&](float v) { return Qd(mxq_round_dt<ADT>(v)); };
    // SMQ_BF16: the closed form without its special cases, for values that are normal numbers far
    // from the top binade, or zero (a -0 stays -0 here; see below where that can happen).  A wave
    // uses it for the per-element steps of a row while everything those steps see lies in a range
    // that keeps them there:
    //   inputs 2^-20 <= |x| < 2^20 (every lane of the wave), |mean| < 2^21
    //     => x - mean is +0 or at least 2^-35 in magnitude (both are multiples of 2^-35 when the
    //        mean is not negligible), its square +0 or at least 2^-70;
    //   2^-30 <= 1 / sqrt(var + eps) < 2^30 => the normalized value is +0 or within 2^-65 .. 2^51;
    //   weights 2^-20 <= |w| < 2^20, bias +0 or 2^-40 <= |b| < 2^40 (this lane's columns)
    //     => w z is normal or +-0, and w z + b is normal, +0 (exact cancellation), b or w z.  A -0
    //        product (z = +0, w < 0) gives the same sum as the +0 the general form turns it into.
    // The per-row scalars always take the general form.
    auto Qplain_d = [](float v) {
        const uint32_t u = mxq_bits(v);
        return mxq_float(u + (u & 0x10000u));
    };
    auto within = [](float v, uint32_t lo, uint32_t hi) {    // lo <= |v| < hi as bit patterns
        return (mxq_bits(v) & 0x7FFFFFFFu) - lo < hi - lo;
    };
    // the plain form on two values at once: one conversion rounds both to bf16, one add moves both
    // odd significands up (no carry leaves the low half: 0xFFFF is a NaN)
    auto plain_packed = [](float a, float b) {
        const uint32_t r = Pack<MXQ_BF16>::put(a, b);
        return r + (r & 0x00010001u);
    };
    auto low_of = [](uint32_t r) { return mxq_float(r << 16); };
    auto high_of = [](uint32_t r) { return mxq_float(r & 0xFFFF0000u); };

    constexpr int LPR = 64 * WPR;                            // lanes per row
    constexpr int RPB = (TPB / 64) / WPR;                    // rows per block and iteration
    __shared__ float part[TPB / 64];
    const int wib = threadIdx.x >> 6;                        // wave in block
    const int lane = (wib % WPR) * 64 + (threadIdx.x & 63);  // lane within the row
    const int nvec_row = n / EPV;
    const float count = (float)n;
    const u32x4* wv = reinterpret_cast<const u32x4*>(weight_);
    const u32x4* bv = reinterpret_cast<const u32x4*>(bias_);

    // this lane's columns are the same in every row: are their weights and biases in range?
    bool wb_plain = QMODE == SMQ_BF16 && !p.q.general_only;
    if (QMODE == SMQ_BF16) {
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int v = j * LPR + lane;
            if (v >= nvec_row) continue;
            const u32x4 w4 = wv[v], b4 = bv[v];
#pragma unroll
            for (int d = 0; d < 4; ++d)
#pragma unroll
                for (int h = 0; h < PD; ++h) {
                    const float w = Pack<DT>::get(w4[d], h), b = Pack<DT>::get(b4[d], h);
                    wb_plain = wb_plain && within(w, 0x35800000u, 0x49800000u) &&               // [2^-20, 2^20)
                               (mxq_bits(b) == 0u || within(b, 0x2B800000u, 0x53800000u));      // +0, [2^-40, 2^40)
                }
        }
        wb_plain = __all(wb_plain);
    }

    for (int64_t row0 = (int64_t)blockIdx.x * RPB; row0 < rows; row0 += (int64_t)gridDim.x * RPB) {
        const int64_t row = row0 + wib / WPR;
        const int nvec = row < rows ? nvec_row : 0;          // a block's spare waves go through the motions
        const u32x4* in = reinterpret_cast<const u32x4*>(in_) + row * nvec_row;
        float x[EPL];
        bool plain = QMODE == SMQ_BF16 && !p.q.general_only;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const bool valid = j * LPR + lane < nvec;
            u32x4 raw = {0, 0, 0, 0};
            if (valid) raw = in[j * LPR + lane];
#pragma unroll
            for (int d = 0; d < 4; ++d)
#pragma unroll
                for (int h = 0; h < PD; ++h) {
                    const int e = (j * 4 + d) * PD + h;
                    const float v = Pack<DT>::get(raw[d], h);
                    if (QMODE == SMQ_BF16) {
                        plain = plain && (!valid || within(v, 0x35800000u, 0x49800000u));
                        x[e] = valid ? Qplain_d(v) : 0.0f;   // zeros add nothing to the sums
                    } else {
                        x[e] = valid ? Qd(v) : 0.0f;
                    }
                }
        }
        if (QMODE == SMQ_BF16) {
            plain = __all(plain);                            // wave-uniform from here on
            if (!plain) {                                    // rare: read the row once more
#pragma unroll
                for (int j = 0; j < VPL; ++j) {
                    if (j * LPR + lane >= nvec) continue;
                    const u32x4 raw = in[j * LPR + lane];
#pragma unroll
                    for (int d = 0; d < 4; ++d)
#pragma unroll
                        for (int h = 0; h < PD; ++h) x[(j * 4 + d) * PD + h] = Qd(Pack<DT>::get(raw[d], h));
                }
            }
        }
        float sum = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) sum += p.rms ? 0.0f : x[e];
        float sq = 0.0f;
        float mean = 0.0f;
        if (!p.rms) {
            mean = Q(Q(row_reduce<SumOp, WPR>(sum, part)) / count);
            if (QMODE == SMQ_BF16) plain = __all(plain && within(mean, 0u, 0x4A000000u));    // |mean| < 2^21
        }
        auto centre_and_square = [&](auto plain_tag) {
            if constexpr (decltype(plain_tag)::value && DT == MXQ_BF16) {
                if (!p.rms) {
#pragma unroll
                    for (int j = 0; j < VPL; ++j) {
                        const bool valid = j * LPR + lane < nvec;
#pragma unroll
                        for (int k = 0; k < EPV; k += 2) {
                            const uint32_t r = plain_packed(x[j * EPV + k] - mean, x[j * EPV + k + 1] - mean);
                            x[j * EPV + k] = valid ? low_of(r) : 0.0f;
                            x[j * EPV + k + 1] = valid ? high_of(r) : 0.0f;
                        }
                    }
                }
#pragma unroll
                for (int e = 0; e < EPL; e += 2) {           // same order of additions as one by one
                    const uint32_t r = plain_packed(x[e] * x[e], x[e + 1] * x[e + 1]);
                    sq += low_of(r);
                    sq += high_of(r);
                }
            } else {
                if (!p.rms) {
#pragma unroll
                    for (int j = 0; j < VPL; ++j) {
                        const bool valid = j * LPR + lane < nvec;
#pragma unroll
                        for (int k = 0; k < EPV; ++k) x[j * EPV + k] = valid ? Q(x[j * EPV + k] - mean) : 0.0f;
                    }
                }
#pragma unroll
                for (int e = 0; e < EPL; ++e) sq += Q(x[e] * x[e]);
            }
        };
        if (QMODE == SMQ_BF16 && plain) centre_and_square(std::true_type{});
        else centre_and_square(std::false_type{});
        const float var = Q(Q(row_reduce<SumOp, WPR>(sq, part)) / count);
        const float vare = Q(var + p.eps);
        const float rinv = Q(1.0f / Q(sqrtf(vare)));
        if (lane == 0 && nvec != 0) store_scalar<DT>(stat_, row, p.rms ? rinv : vare);
        if (QMODE == SMQ_BF16)
            plain = __all(plain && wb_plain && mxq_bits(rinv) - 0x30800000u < 0x1E000000u);   // [2^-30, 2^30)

        u32x4* out = reinterpret_cast<u32x4*>(out_) + row * nvec_row;
        u32x4* zn = znorm_ ? reinterpret_cast<u32x4*>(znorm_) + row * nvec : nullptr;
        auto scale_and_shift = [&](auto plain_tag) {
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                const int v = j * LPR + lane;
                if (v >= nvec) continue;
                const u32x4 w4 = wv[v], b4 = bv[v];
                u32x4 o, z4;
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    if constexpr (decltype(plain_tag)::value && DT == MXQ_BF16) {
                        const int e = (j * 4 + d) * 2;
                        const uint32_t zr = plain_packed(x[e] * rinv, x[e + 1] * rinv);
                        const uint32_t wz = plain_packed(low_of(w4[d]) * low_of(zr), high_of(w4[d]) * high_of(zr));
                        o[d] = plain_packed(low_of(wz) + low_of(b4[d]), high_of(wz) + high_of(b4[d]));
                        z4[d] = zr;
                    } else {
                        float q[2], z[2];
#pragma unroll
                        for (int h = 0; h < PD; ++h) {
                            z[h] = Q(x[(j * 4 + d) * PD + h] * rinv);
                            q[h] = Q(Q(Pack<DT>::get(w4[d], h) * z[h]) + Pack<DT>::get(b4[d], h));
                        }
                        o[d] = Pack<DT>::put(q[0], q[PD - 1]);
                        z4[d] = Pack<DT>::put(z[0], z[PD - 1]);
                    }
                }
                __builtin_nontemporal_store(o, &out[v]);
                if (zn) __builtin_nontemporal_store(z4, &zn[v]);
            }
        };
        if (QMODE == SMQ_BF16 && plain) scale_and_shift(std::true_type{});
        else scale_and_shift(std::false_type{});
    }
}

}  // namespace

// ================================================================================================
// Activations with the elementwise quantizer after every step (mx/activations.py:237-557): one
// kernel instead of 3 to 22 tensor passes.  Elementwise, 16 bytes per lane, grid-stride.
//   logistic(y) = Q(1 / Q(Q(exp(-y)) + 1)); with vec_use_exp2: exp(t) = Q(2^Q(1.4453125 t))
//   sigmoid: logistic(q)        tanh: Q(tanh q)        silu: Q(q s), s = logistic(q)
//   gelu:    Q(q phi), phi = logistic(y), y = Q(1.703125 q)                           (first order)
//            or y = Q(1.59375 Q(Q(0.044677734375 Q(Q(q q) q)) + q))                   (cubic)
// with q = Q(input).  Besides the result it writes what the backward passes keep: the logistic
// factor (silu, gelu) and the quantized input (gelu), when the pointers are given.
// ================================================================================================
enum { ACT_SIGMOID = 0, ACT_TANH = 1, ACT_SILU = 2, ACT_GELU_FIRST_ORDER = 3, ACT_GELU = 4 };

struct ActParams {
    ElemParams q;
    int act;
    int exp_mode;      // 0: exp(x)   2: 2^Q(x * log2(e) at bfloat16 precision)  (vec_use_exp2)
};

namespace {

template <int DT, int RMODE, int QMODE>
__global__ __launch_bounds__(TPB) void activation_kernel(const void* __restrict__ in_, void* __restrict__ out_,
                                                         void* __restrict__ aux_, void* __restrict__ qin_,
                                                         int64_t n, ActParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.q.zone_row]);

    auto Qd = [&](float v) {                                 // v already is a value of the tensor dtype
        if (QMODE == SMQ_IDENT) return v;
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest(v, p.q.fmt.nan_from);
        return mxq_quant_elemwise<RMODE, ADT, true, true>(v, p.q.fmt, p.q.saturate != 0,
                                                          p.q.allow_denorm != 0, zone, ZS);
    };
    const bool via_exp2 = p.exp_mode == 2;
    // one element: result, logistic factor (silu, gelu), quantized input.
    // plain_tag (SMQ_BF16 only): the input lies in 2^-20 <= |x| < 8.  Every intermediate value of
    // the five chains is then a normal number, neither zero nor near the top binade (|arguments of
    // exp| < 50, so the exponentials lie in 4e-22 .. 3e21 and the logistic factor in 4e-22 .. 1;
    // sums add numbers of the same sign), and the closed form of the quantizer needs none of its
    // special cases, which cost four times its arithmetic.
    auto eval = [&](auto plain_tag, float x, float& aux, float& q) {
        constexpr bool PLAIN = decltype(plain_tag)::value;
        auto Qd_ = [&](float v) {
            if (PLAIN) {
                const uint32_t u = mxq_bits(v);
                return mxq_float(u + (u & 0x10000u));
            }
            return Qd(v);
        };
        auto Q = [&](float v) { return Qd_(mxq_round_dt<ADT>(v)); };
        auto logistic = [&](float y) {
            const float t = -y;
            const float e = via_exp2 ? Q(exp2f(Q(1.4453125f * t))) : Q(expf(t));
            return Q(1.0f / Q(e + 1.0f));
        };
        q = Qd_(x);
        aux = 0.0f;
        switch (p.act) {
            case ACT_SIGMOID: return logistic(q);
            case ACT_TANH: return Q(tanhf(q));
            case ACT_SILU: aux = logistic(q); return Q(q * aux);
            case ACT_GELU_FIRST_ORDER: aux = logistic(Q(1.703125f * q)); return Q(q * aux);
            default: {
                const float cube = Q(Q(q * q) * q);
                const float y = Q(1.59375f * Q(Q(0.044677734375f * cube) + q));
                aux = logistic(y);
                return Q(q * aux);
            }
        }
    };
    auto in_plain_range = [](uint32_t ua) { return ua - 0x35800000u < 0x0B800000u; };   // [2^-20, 8)
    // The plain form on the two bf16 values of a dword at once: one conversion rounds both to bf16,
    // one add moves both odd significands up (no carry leaves the low half: 0xFFFF is a NaN).
    // dword in: the pair as loaded; dwords out: result, logistic factor, quantized input.
    auto eval_pair = [&](uint32_t w, uint32_t& aux_w, uint32_t& q_w) {
        struct Pair { float a, b; };
        auto packed = [](float a, float b) {
            const uint32_t r = Pack<MXQ_BF16>::put(a, b);
            return r + (r & 0x00010001u);
        };
        auto unpack = [](uint32_t r) { return Pair{mxq_float(r << 16), mxq_float(r & 0xFFFF0000u)}; };
        auto Q2 = [&](float a, float b) { return unpack(packed(a, b)); };
        auto logistic = [&](Pair y) {                        // packed
            Pair e;
            if (via_exp2) {
                const Pair t = Q2(1.4453125f * -y.a, 1.4453125f * -y.b);
                e = Q2(exp2f(t.a), exp2f(t.b));
            } else {
                e = Q2(expf(-y.a), expf(-y.b));
            }
            const Pair s = Q2(e.a + 1.0f, e.b + 1.0f);
            // 1 / s for s with an 8-bit significand, 1 <= s < 2^72: a refined hardware reciprocal
            // and one residual correction give the correctly rounded fp32 quotient (what the
            // division of the general form gives) for a third of its instructions
            auto recip = [](float d) {
                const float r0 = __builtin_amdgcn_rcpf(d);
                const float r1 = fmaf(fmaf(-d, r0, 1.0f), r0, r0);
                return fmaf(fmaf(-r1, d, 1.0f), r1, r1);
            };
            return packed(recip(s.a), recip(s.b));
        };
        q_w = w + (w & 0x00010001u);
        const Pair q = unpack(q_w);
        aux_w = 0u;
        switch (p.act) {
            case ACT_SIGMOID: return logistic(q);
            case ACT_TANH: return packed(tanhf(q.a), tanhf(q.b));
            case ACT_SILU: {
                aux_w = logistic(q);
                const Pair s = unpack(aux_w);
                return packed(q.a * s.a, q.b * s.b);
            }
            case ACT_GELU_FIRST_ORDER: {
                aux_w = logistic(Q2(1.703125f * q.a, 1.703125f * q.b));
                const Pair s = unpack(aux_w);
                return packed(q.a * s.a, q.b * s.b);
            }
            default: {
                const Pair sq = Q2(q.a * q.a, q.b * q.b);
                const Pair cube = Q2(sq.a * q.a, sq.b * q.b);
                const Pair c = Q2(0.044677734375f * cube.a, 0.044677734375f * cube.b);
                const Pair in = Q2(c.a + q.a, c.b + q.b);
                aux_w = logistic(Q2(1.59375f * in.a, 1.59375f * in.b));
                const Pair s = unpack(aux_w);
                return packed(q.a * s.a, q.b * s.b);
            }
        }
    };

    const u32x4* in = reinterpret_cast<const u32x4*>(in_);
    u32x4* out = reinterpret_cast<u32x4*>(out_);
    u32x4* auxv = reinterpret_cast<u32x4*>(aux_);
    u32x4* qinv = reinterpret_cast<u32x4*>(qin_);
    const int64_t n_vec = n / EPV;
    const int64_t stride = (int64_t)gridDim.x * TPB;
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n_vec; i += stride) {
        const u32x4 v = in[i];
        u32x4 o, a, qv;
        auto vector = [&](auto plain_tag) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                if constexpr (decltype(plain_tag)::value && DT == MXQ_BF16) {
                    uint32_t aw, qw;
                    o[d] = eval_pair(v[d], aw, qw);
                    a[d] = aw;
                    qv[d] = qw;
                } else {
                    float r[2], ax[2], qq[2];
#pragma unroll
                    for (int h = 0; h < PD; ++h) r[h] = eval(plain_tag, Pack<DT>::get(v[d], h), ax[h], qq[h]);
                    o[d] = Pack<DT>::put(r[0], r[PD - 1]);
                    a[d] = Pack<DT>::put(ax[0], ax[PD - 1]);
                    qv[d] = Pack<DT>::put(qq[0], qq[PD - 1]);
                }
            }
        };
        bool plain = QMODE == SMQ_BF16 && !p.q.general_only;
        if (QMODE == SMQ_BF16) {
#pragma unroll
            for (int d = 0; d < 4; ++d)
#pragma unroll
                for (int h = 0; h < PD; ++h)
                    plain = plain && in_plain_range(mxq_bits(Pack<DT>::get(v[d], h)) & 0x7FFFFFFFu);
            plain = __all(plain);                            // one branch per wave
        }
        if (QMODE == SMQ_BF16 && plain) vector(std::true_type{});
        else vector(std::false_type{});
        __builtin_nontemporal_store(o, &out[i]);
        if (auxv) __builtin_nontemporal_store(a, &auxv[i]);
        if (qinv) __builtin_nontemporal_store(qv, &qinv[i]);
    }
    // tail
    const int64_t t0 = n_vec * EPV;
    const int64_t gi = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (gi < n - t0) {
        float ax, qq;
        const float r = eval(std::false_type{}, load_scalar<DT>(in_, t0 + gi), ax, qq);
        store_scalar<DT>(out_, t0 + gi, mxq_round_dt<ADT>(r));
        if (aux_) store_scalar<DT>(aux_, t0 + gi, mxq_round_dt<ADT>(ax));
        if (qin_) store_scalar<DT>(qin_, t0 + gi, qq);
    }
}

// The backward passes of the same activations (mx/activations.py:251-267, 284-297, 437-455,
// 500-557) from the tensors their forward passes saved; only exact arithmetic and the quantizer,
// so the results are those of the chain of vec_* ops bit for bit.
//   g = Q(grad_output)
//   sigmoid: d = Q(s Q(1 - s))                       s = saved output
//   tanh:    d = Q(1 - Q(t t))                       t = saved output
//   silu:    d = Q(s + Q(y Q(1 - s)))                y = saved output, s = saved sigmoid
//   gelu:    p = Q(phi Q(1 - phi)); first order: p = Q(1.703125 p);
//            cubic: p = Q(Q(1.59375 + Q(0.2138671875 Q(x x))) p);  d = Q(phi + Q(x p))
//   grad_input = Q(d g)
template <int DT, int RMODE, int QMODE>
__global__ __launch_bounds__(TPB) void activation_backward_kernel(const void* __restrict__ grad_,
                                                                  const void* __restrict__ saved_,
                                                                  const void* __restrict__ aux_,
                                                                  void* __restrict__ out_, int64_t n,
                                                                  ActParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.q.zone_row]);

    auto Qd = [&](float v) {
        if (QMODE == SMQ_IDENT) return v;
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest(v, p.q.fmt.nan_from);
        return mxq_quant_elemwise<RMODE, ADT, true, true>(v, p.q.fmt, p.q.saturate != 0,
                                                          p.q.allow_denorm != 0, zone, ZS);
    };
    auto Q = [&](float v) { return Qd(mxq_round_dt<ADT>(v)); };
    auto eval = [&](float grad, float sv, float ax) {
        const float g = Qd(grad);
        float d;
        switch (p.act) {
            case ACT_SIGMOID: d = Q(sv * Q(1.0f - sv)); break;
            case ACT_TANH: d = Q(1.0f - Q(sv * sv)); break;
            case ACT_SILU: d = Q(ax + Q(sv * Q(1.0f - ax))); break;
            default: {
                float dphi = Q(ax * Q(1.0f - ax));
                if (p.act == ACT_GELU_FIRST_ORDER) dphi = Q(1.703125f * dphi);
                else dphi = Q(Q(1.59375f + Q(0.2138671875f * Q(sv * sv))) * dphi);
                d = Q(ax + Q(sv * dphi));
            }
        }
        return Q(d * g);
    };

    const bool two = p.act >= ACT_SILU;                      // a second saved tensor

    // SMQ_BF16, plain range (see activation_kernel): a wave whose three inputs lie in
    //   grad 2^-30 <= |g| < 2^40;
    //   saved: sigmoid 2^-60 <= s <= 1; tanh 2^-20 <= |t| <= 1; silu 2^-40 <= |y| < 2^20;
    //          gelu 2^-20 <= |x| < 8;       logistic factor (silu, gelu) 2^-60 <= s <= 1
    // sees only normal numbers and zeros in its chain: 1 - s is +0 (a saturated logistic, which is
    // common) or at least 2^-8, the products are zero or stay above 2^-80, and the sum "s + ..." of
    // silu and gelu can cancel, exactly (+0) or down to one unit of its smaller term (at least
    // 2^-87, so that d g stays above 2^-117).  A zero only ever meets a product (which stays a zero of some sign) or the sum with
    // s > 0 (which ignores its sign), so the derivative d is +0 or normal; d g is then normal or
    // +-0, and adding +0.0 before the last quantization turns a -0 into the +0 the general form gives.
    // Both values of a dword go through the plain form at once (see eval_pair there).
    const uint32_t s_lo = p.act == ACT_SIGMOID ? 0x2180u : p.act == ACT_SILU ? 0x2B80u : 0x3580u;
    const uint32_t s_hi = p.act == ACT_SIGMOID ? 0x3F81u : p.act == ACT_TANH ? 0x3F81u
                        : p.act == ACT_SILU ? 0x4980u : 0x4100u;
    const uint32_t s_mask = p.act == ACT_SIGMOID ? 0xFFFFu : 0x7FFFu;   // the sigmoid must be positive
    auto halves_within = [](uint32_t w, uint32_t mask, uint32_t lo, uint32_t hi) {   // both bf16 halves
        return ((w & mask) - lo < hi - lo) && (((w >> 16) & mask) - lo < hi - lo);
    };
    auto eval_pair = [&](uint32_t gw, uint32_t sw, uint32_t aw) {
        struct Pair { float a, b; };
        auto packed = [](float a, float b) {
            const uint32_t r = Pack<MXQ_BF16>::put(a, b);
            return r + (r & 0x00010001u);
        };
        auto unpack = [](uint32_t r) { return Pair{mxq_float(r << 16), mxq_float(r & 0xFFFF0000u)}; };
        auto Q2 = [&](float a, float b) { return unpack(packed(a, b)); };
        const Pair g = unpack(gw + (gw & 0x00010001u));
        const Pair sv = unpack(sw), ax = unpack(aw);
        Pair d;
        switch (p.act) {
            case ACT_SIGMOID: {
                const Pair t = Q2(1.0f - sv.a, 1.0f - sv.b);
                d = Q2(sv.a * t.a, sv.b * t.b);
                break;
            }
            case ACT_TANH: {
                const Pair t = Q2(sv.a * sv.a, sv.b * sv.b);
                d = Q2(1.0f - t.a, 1.0f - t.b);
                break;
            }
            case ACT_SILU: {
                const Pair t = Q2(1.0f - ax.a, 1.0f - ax.b);
                const Pair u = Q2(sv.a * t.a, sv.b * t.b);
                d = Q2(ax.a + u.a, ax.b + u.b);
                break;
            }
            default: {
                const Pair t = Q2(1.0f - ax.a, 1.0f - ax.b);
                Pair dphi = Q2(ax.a * t.a, ax.b * t.b);
                if (p.act == ACT_GELU_FIRST_ORDER) {
                    dphi = Q2(1.703125f * dphi.a, 1.703125f * dphi.b);
                } else {
                    const Pair sq = Q2(sv.a * sv.a, sv.b * sv.b);
                    const Pair c = Q2(0.2138671875f * sq.a, 0.2138671875f * sq.b);
                    const Pair e = Q2(1.59375f + c.a, 1.59375f + c.b);
                    dphi = Q2(e.a * dphi.a, e.b * dphi.b);
                }
                const Pair u = Q2(sv.a * dphi.a, sv.b * dphi.b);
                d = Q2(ax.a + u.a, ax.b + u.b);
            }
        }
        return packed(d.a * g.a + 0.0f, d.b * g.b + 0.0f);
    };

    const u32x4* grad = reinterpret_cast<const u32x4*>(grad_);
    const u32x4* saved = reinterpret_cast<const u32x4*>(saved_);
    const u32x4* aux = reinterpret_cast<const u32x4*>(aux_);
    u32x4* out = reinterpret_cast<u32x4*>(out_);
    const int64_t n_vec = n / EPV;
    const int64_t stride = (int64_t)gridDim.x * TPB;
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n_vec; i += stride) {
        const u32x4 gv = grad[i], sv = saved[i];
        const u32x4 av = two ? aux[i] : u32x4{0, 0, 0, 0};
        u32x4 o;
        bool plain = false;
        if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) {
            plain = !p.q.general_only;
#pragma unroll
            for (int d = 0; d < 4; ++d)
                plain = plain && halves_within(gv[d], 0x7FFFu, 0x3080u, 0x5380u) &&
                        halves_within(sv[d], s_mask, s_lo, s_hi) &&
                        (!two || halves_within(av[d], 0xFFFFu, 0x2180u, 0x3F81u));
            plain = __all(plain);                            // one branch per wave
        }
        bool done = false;
        if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) {
            if (plain) {
#pragma unroll
                for (int d = 0; d < 4; ++d) o[d] = eval_pair(gv[d], sv[d], av[d]);
                done = true;
            }
        }
        if (!done) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                float r[2];
#pragma unroll
                for (int h = 0; h < PD; ++h)
                    r[h] = eval(Pack<DT>::get(gv[d], h), Pack<DT>::get(sv[d], h), Pack<DT>::get(av[d], h));
                o[d] = Pack<DT>::put(r[0], r[PD - 1]);
            }
        }
        __builtin_nontemporal_store(o, &out[i]);
    }
    const int64_t t0 = n_vec * EPV;
    const int64_t gi = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (gi < n - t0) {
        const float r = eval(load_scalar<DT>(grad_, t0 + gi), load_scalar<DT>(saved_, t0 + gi),
                             two ? load_scalar<DT>(aux_, t0 + gi) : 0.0f);
        store_scalar<DT>(out_, t0 + gi, mxq_round_dt<ADT>(r));
    }
}

// SoftmaxFunction.backward (mx/softmax.py:56-88) over the last axis, same work mapping as the
// forward kernel:  g = Q(grad); s = Q(sum Q(g y)); grad_input = Q(y Q(g - s)) (, Q(. * ln2) for
// softmax_exp2, with ln2 at bfloat16 precision).
template <int DT, int RMODE, int QMODE, int VPL, int WPR>
__global__ __launch_bounds__(TPB) void softmax_backward_row_kernel(const void* __restrict__ grad_,
                                                                   const void* __restrict__ y_,
                                                                   void* __restrict__ out_, int64_t rows,
                                                                   int n, SoftmaxParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    constexpr int EPL = VPL * EPV;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.q.zone_row]);

    auto Qd = [&](float v) {
        if (QMODE == SMQ_IDENT) return v;
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest(v, p.q.fmt.nan_from);
        return mxq_quant_elemwise<RMODE, ADT, true, true>(v, p.q.fmt, p.q.saturate != 0,
                                                          p.q.allow_denorm != 0, zone, ZS);
    };
    auto Q = [&](float v) { return Qd(mxq_round_dt<ADT>(v)); };

    constexpr int LPR = 64 * WPR;                            // lanes per row
    constexpr int RPB = (TPB / 64) / WPR;                    // rows per block and iteration
    __shared__ float part[TPB / 64];
    const int wib = threadIdx.x >> 6;                        // wave in block
    const int lane = (wib % WPR) * 64 + (threadIdx.x & 63);  // lane within the row
    const int nvec_row = n / EPV;
    for (int64_t row0 = (int64_t)blockIdx.x * RPB; row0 < rows; row0 += (int64_t)gridDim.x * RPB) {
        const int64_t row = row0 + wib / WPR;
        const int nvec = row < rows ? nvec_row : 0;          // a block's spare waves go through the motions
        const u32x4* gin = reinterpret_cast<const u32x4*>(grad_) + row * nvec_row;
        const u32x4* yin = reinterpret_cast<const u32x4*>(y_) + row * nvec_row;
        u32x4* out = reinterpret_cast<u32x4*>(out_) + row * nvec_row;
        float g[EPL];
        u32x4 yraw[VPL];
        float sum = 0.0f;
        // SMQ_BF16, plain range (see softmax_row_kernel): gradients 2^-30 <= |g| < 2^30 and saved
        // outputs 2^-60 <= y <= 1 in every lane of the wave, and |s| < 2^30 for the row sum, keep
        // every per-element value a normal number or +0 (g - s cancels to +0 or to no less than
        // 2^-46, and y > 0 keeps the sign of a zero): both bf16 values of a dword then go through
        // the plain form of the quantizer at once.
        bool plain = false;
        if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) plain = !p.q.general_only;
        auto plain_packed = [](float a, float b) {
            const uint32_t r = Pack<MXQ_BF16>::put(a, b);
            return r + (r & 0x00010001u);
        };
        auto low_of = [](uint32_t r) { return mxq_float(r << 16); };
        auto high_of = [](uint32_t r) { return mxq_float(r & 0xFFFF0000u); };
        auto halves_within = [](uint32_t w, uint32_t mask, uint32_t lo, uint32_t hi) {
            return ((w & mask) - lo < hi - lo) && (((w >> 16) & mask) - lo < hi - lo);
        };
        if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) {
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                const bool valid = j * LPR + lane < nvec;
                u32x4 graw = {0, 0, 0, 0};
                yraw[j] = u32x4{0, 0, 0, 0};
                if (valid) {
                    graw = gin[j * LPR + lane];
                    yraw[j] = yin[j * LPR + lane];
                }
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    plain = plain && (!valid || (halves_within(graw[d], 0x7FFFu, 0x3080u, 0x4E80u) &&
                                                 halves_within(yraw[j][d], 0xFFFFu, 0x2180u, 0x3F81u)));
                    const uint32_t gq = graw[d] + (graw[d] & 0x00010001u);
                    const int e = (j * 4 + d) * 2;
                    g[e] = valid ? low_of(gq) : 0.0f;
                    g[e + 1] = valid ? high_of(gq) : 0.0f;
                    const uint32_t prod = plain_packed(g[e] * low_of(yraw[j][d]), g[e + 1] * high_of(yraw[j][d]));
                    sum += valid ? low_of(prod) : 0.0f;
                    sum += valid ? high_of(prod) : 0.0f;
                }
            }
            plain = __all(plain);                            // wave-uniform from here on
        }
        if (!plain) {                                        // (for SMQ_BF16: rare, reads the gradient again)
            sum = 0.0f;
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                const bool valid = j * LPR + lane < nvec;
                u32x4 graw = {0, 0, 0, 0};
                yraw[j] = u32x4{0, 0, 0, 0};
                if (valid) {
                    graw = gin[j * LPR + lane];
                    yraw[j] = yin[j * LPR + lane];
                }
#pragma unroll
                for (int d = 0; d < 4; ++d)
#pragma unroll
                    for (int h = 0; h < PD; ++h) {
                        const int e = (j * 4 + d) * PD + h;
                        g[e] = valid ? Qd(Pack<DT>::get(graw[d], h)) : 0.0f;
                        sum += valid ? Q(g[e] * Pack<DT>::get(yraw[j][d], h)) : 0.0f;
                    }
            }
        }
        sum = Q(row_reduce<SumOp, WPR>(sum, part));
        if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16)
            plain = __all(plain && (mxq_bits(sum) & 0x7FFFFFFFu) < 0x4E800000u);       // |s| < 2^30, the same in every lane
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            u32x4 o;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                bool done = false;
                if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) {
                    if (plain) {
                        const int e = (j * 4 + d) * 2;
                        const uint32_t diff = plain_packed(g[e] - sum, g[e + 1] - sum);
                        uint32_t r = plain_packed(low_of(yraw[j][d]) * low_of(diff), high_of(yraw[j][d]) * high_of(diff));
                        if (p.exp_mode == 1) r = plain_packed(low_of(r) * 0.69140625f, high_of(r) * 0.69140625f);
                        o[d] = r;
                        done = true;
                    }
                }
                if (!done) {
                    float q[2];
#pragma unroll
                    for (int h = 0; h < PD; ++h) {
                        const float t = Q(Pack<DT>::get(yraw[j][d], h) * Q(g[(j * 4 + d) * PD + h] - sum));
                        q[h] = p.exp_mode == 1 ? Q(t * 0.69140625f) : t;
                    }
                    o[d] = Pack<DT>::put(q[0], q[PD - 1]);
                }
            }
            if (j * LPR + lane < nvec) __builtin_nontemporal_store(o, &out[j * LPR + lane]);
        }
    }
}

// Gradient with respect to the input of LayerNorm / RMSNorm over the last axis from what the
// forward pass saved (mx/norm_utils.py:188-258 with axes = -1, mx/layernorm.py:150-168), same work
// mapping as norm_row_kernel.  With g = Q(grad_output), d = Q(g w), n = row length:
//   LayerNorm: sd = Q(sqrt v), si = Q(1 / sd)                                 (v = saved var + eps)
//              t = Q(Q(Q(sum Q(Q(d z) sd)) / n) Q(1 / v))                     (z = saved normalized input)
//              dx = Q(Q(d si) + Q(-t z));  grad_input = Q(dx - Q(Q(sum dx) / n))
//   RMSNorm:   d1 = Q(d r), proj = Q(Q(sum Q(d1 z)) / n)                      (r = saved 1 / rms)
//              grad_input = d1 - Q(z proj), rounded to the tensor dtype only
template <int DT, int RMODE, int QMODE, int VPL, int WPR>
__global__ __launch_bounds__(TPB) void norm_backward_row_kernel(const void* __restrict__ grad_,
                                                                const void* __restrict__ weight_,
                                                                const void* __restrict__ znorm_,
                                                                const void* __restrict__ stat_,
                                                                void* __restrict__ out_, int64_t rows, int n,
                                                                NormParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    constexpr int EPL = VPL * EPV;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.q.zone_row]);

    auto Qd = [&](float v) {
        if (QMODE == SMQ_IDENT) return v;
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest(v, p.q.fmt.nan_from);
        return mxq_quant_elemwise<RMODE, ADT, true, true>(v, p.q.fmt, p.q.saturate != 0,
                                                          p.q.allow_denorm != 0, zone, ZS);
    };
    auto Q = [&](float v) { return Qd(mxq_round_dt<ADT>(v)); };

    constexpr int LPR = 64 * WPR;                            // lanes per row
    constexpr int RPB = (TPB / 64) / WPR;                    // rows per block and iteration
    __shared__ float part[TPB / 64];
    const int wib = threadIdx.x >> 6;                        // wave in block
    const int lane = (wib % WPR) * 64 + (threadIdx.x & 63);  // lane within the row
    const int nvec_row = n / EPV;
    const float count = (float)n;
    const u32x4* wv = reinterpret_cast<const u32x4*>(weight_);

    // SMQ_BF16, plain range (see norm_row_kernel).  A wave takes the plain form of the quantizer, on
    // both bf16 values of a dword at once, for the per-element steps while what they see stays in
    //   gradients 2^-30 <= |g| < 2^30, weights 2^-20 <= |w| < 2^20 (this lane's columns),
    //   normalized inputs +0 or 2^-30 <= |z| < 2^10, 2^-30 <= sd, si (r) < 2^30:
    //     g w, its products with si, with z, and that with sd are normal or zero (above 2^-110);
    //   then the row scalar t: +-0 or 2^-40 <= |t| < 2^30: t z is +-0 or above 2^-70, and
    //     d + t z is +0 (exact cancellation) or at least one unit of the smaller term;
    //   then the row mean dm: +-0 or 2^-60 <= |dm| < 2^80, likewise.
    // A zero of either sign only ever meets a row sum (which starts at +0 and is quantized in the
    // general form) or a sum with a nonzero number.  The row scalars always take the general form.
    constexpr bool CAN_PLAIN = QMODE == SMQ_BF16 && DT == MXQ_BF16;
    auto plain_packed = [](float a, float b) {
        const uint32_t r = Pack<MXQ_BF16>::put(a, b);
        return r + (r & 0x00010001u);
    };
    auto low_of = [](uint32_t r) { return mxq_float(r << 16); };
    auto high_of = [](uint32_t r) { return mxq_float(r & 0xFFFF0000u); };
    auto half_within = [](uint32_t h, uint32_t lo, uint32_t hi) { return (h & 0x7FFFu) - lo < hi - lo; };
    auto halves_within = [&](uint32_t w, uint32_t lo, uint32_t hi) {
        return half_within(w & 0xFFFFu, lo, hi) && half_within(w >> 16, lo, hi);
    };
    auto scalar_within = [](float v, uint32_t lo, uint32_t hi, bool or_zero) {
        const uint32_t ua = mxq_bits(v) & 0x7FFFFFFFu;
        return (or_zero && ua == 0u) || ua - lo < hi - lo;
    };
    bool w_plain = false;
    if constexpr (CAN_PLAIN) {
        w_plain = !p.q.general_only;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int v = j * LPR + lane;
            if (v >= nvec_row) continue;
            const u32x4 w4 = wv[v];
#pragma unroll
            for (int k = 0; k < 4; ++k) w_plain = w_plain && halves_within(w4[k], 0x3580u, 0x4980u);
        }
        w_plain = __all(w_plain);
    }

    for (int64_t row0 = (int64_t)blockIdx.x * RPB; row0 < rows; row0 += (int64_t)gridDim.x * RPB) {
        const int64_t row = row0 + wib / WPR;
        const int nvec = row < rows ? nvec_row : 0;          // a block's spare waves go through the motions
        const u32x4* gin = reinterpret_cast<const u32x4*>(grad_) + row * nvec_row;
        const u32x4* zin = reinterpret_cast<const u32x4*>(znorm_) + row * nvec_row;
        u32x4* out = reinterpret_cast<u32x4*>(out_) + row * nvec_row;
        const float stat = nvec != 0 ? load_scalar<DT>(stat_, row) : 1.0f;
        // row scalars
        const float sd = p.rms ? 0.0f : Q(sqrtf(stat));
        const float si = p.rms ? stat : Q(1.0f / sd);
        float d[EPL];                                        // Q(g w), then Q(d si)
        u32x4 zraw[VPL];
        float sum = 0.0f;
        bool plain = false;
        if constexpr (CAN_PLAIN) {
            plain = w_plain && mxq_bits(si) - 0x30800000u < 0x1E000000u &&                   // [2^-30, 2^30), positive
                    (p.rms || mxq_bits(sd) - 0x30800000u < 0x1E000000u);
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                const bool valid = j * LPR + lane < nvec;
                u32x4 graw = {0, 0, 0, 0}, wraw = {0, 0, 0, 0};
                zraw[j] = u32x4{0, 0, 0, 0};
                if (valid) {
                    graw = gin[j * LPR + lane];
                    wraw = wv[j * LPR + lane];
                    zraw[j] = zin[j * LPR + lane];
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t zw = zraw[j][k];
                    plain = plain && (!valid || (halves_within(graw[k], 0x3080u, 0x4E80u) &&
                                                 ((zw & 0xFFFFu) == 0u || half_within(zw & 0xFFFFu, 0x3080u, 0x4480u)) &&
                                                 ((zw >> 16) == 0u || half_within(zw >> 16, 0x3080u, 0x4480u))));
                    const int e = (j * 4 + k) * 2;
                    const uint32_t gq = graw[k] + (graw[k] & 0x00010001u);
                    const uint32_t dn = plain_packed(low_of(gq) * low_of(wraw[k]), high_of(gq) * high_of(wraw[k]));
                    const uint32_t dd = plain_packed(low_of(dn) * si, high_of(dn) * si);
                    d[e] = low_of(dd);
                    d[e + 1] = high_of(dd);
                    uint32_t ps;
                    if (p.rms) {
                        ps = plain_packed(d[e] * low_of(zw), d[e + 1] * high_of(zw));
                    } else {
                        const uint32_t pz = plain_packed(low_of(dn) * low_of(zw), high_of(dn) * high_of(zw));
                        ps = plain_packed(low_of(pz) * sd, high_of(pz) * sd);
                    }
                    sum += valid ? low_of(ps) : 0.0f;
                    sum += valid ? high_of(ps) : 0.0f;
                }
            }
            plain = __all(plain);                            // wave-uniform from here on
        }
        if (!plain) {                                        // (for SMQ_BF16: rare, reads the row again)
            sum = 0.0f;
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                const bool valid = j * LPR + lane < nvec;
                u32x4 graw = {0, 0, 0, 0}, wraw = {0, 0, 0, 0};
                zraw[j] = u32x4{0, 0, 0, 0};
                if (valid) {
                    graw = gin[j * LPR + lane];
                    wraw = wv[j * LPR + lane];
                    zraw[j] = zin[j * LPR + lane];
                }
#pragma unroll
                for (int k = 0; k < 4; ++k)
#pragma unroll
                    for (int h = 0; h < PD; ++h) {
                        const int e = (j * 4 + k) * PD + h;
                        const float z = Pack<DT>::get(zraw[j][k], h);
                        const float dn = Q(Qd(Pack<DT>::get(graw[k], h)) * Pack<DT>::get(wraw[k], h));
                        if (p.rms) {
                            d[e] = Q(dn * si);
                            sum += valid ? Q(d[e] * z) : 0.0f;
                        } else {
                            d[e] = Q(dn * si);
                            sum += valid ? Q(Q(dn * z) * sd) : 0.0f;
                        }
                    }
            }
        }
        float t = Q(Q(row_reduce<SumOp, WPR>(sum, part)) / count);
        if (!p.rms) t = -Q(t * Q(1.0f / stat));
        if constexpr (CAN_PLAIN) plain = __all(plain && scalar_within(t, 0x2B800000u, 0x4E800000u, true));
        float sum2 = 0.0f;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const bool valid = j * LPR + lane < nvec;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                bool done = false;
                if constexpr (CAN_PLAIN) {
                    if (plain) {
                        const int e = (j * 4 + k) * 2;
                        const uint32_t zw = zraw[j][k];
                        const uint32_t tz = plain_packed(t * low_of(zw), t * high_of(zw));
                        uint32_t nd;
                        if (p.rms) {
                            nd = Pack<MXQ_BF16>::put(d[e] - low_of(tz), d[e + 1] - high_of(tz));   // rounded only
                        } else {
                            nd = plain_packed(d[e] + low_of(tz), d[e + 1] + high_of(tz));
                        }
                        d[e] = low_of(nd);
                        d[e + 1] = high_of(nd);
                        if (!p.rms) {
                            sum2 += valid ? d[e] : 0.0f;
                            sum2 += valid ? d[e + 1] : 0.0f;
                        }
                        done = true;
                    }
                }
                if (!done) {
#pragma unroll
                    for (int h = 0; h < PD; ++h) {
                        const int e = (j * 4 + k) * PD + h;
                        const float z = Pack<DT>::get(zraw[j][k], h);
                        if (p.rms) {
                            d[e] = mxq_round_dt<ADT>(d[e] - Q(z * t));
                        } else {
                            d[e] = Q(d[e] + Q(t * z));
                            sum2 += valid ? d[e] : 0.0f;
                        }
                    }
                }
            }
        }
        const float dm = p.rms ? 0.0f : -Q(Q(row_reduce<SumOp, WPR>(sum2, part)) / count);
        if constexpr (CAN_PLAIN) plain = __all(plain && (p.rms || scalar_within(dm, 0x21800000u, 0x67800000u, true)));
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            u32x4 o;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                bool done = false;
                if constexpr (CAN_PLAIN) {
                    if (plain && !p.rms) {
                        const int e = (j * 4 + k) * 2;
                        o[k] = plain_packed(d[e] + dm, d[e + 1] + dm);
                        done = true;
                    }
                }
                if (!done) {
                    float q[2];
#pragma unroll
                    for (int h = 0; h < PD; ++h) {
                        const float v = d[(j * 4 + k) * PD + h];
                        q[h] = p.rms ? v : Q(v + dm);
                    }
                    o[k] = Pack<DT>::put(q[0], q[PD - 1]);
                }
            }
            if (j * LPR + lane < nvec) __builtin_nontemporal_store(o, &out[j * LPR + lane]);
        }
    }
}

// a op b followed by the elementwise quantizer (vec_add / vec_sub / vec_mul / vec_div / vec_recip,
// mx/vector_ops.py:38-75): one pass instead of torch's op plus a quantization pass.  The second
// operand may be a scalar, on either side.  Only correctly rounded arithmetic: bit-identical to the
// two steps.
enum { BIN_ADD = 0, BIN_SUB = 1, BIN_MUL = 2, BIN_DIV = 3 };
enum { BIN_TENSOR_TENSOR = 0, BIN_TENSOR_SCALAR = 1, BIN_SCALAR_TENSOR = 2 };

struct BinaryParams {
    ElemParams q;
    int op;
    int mode;
    float scalar;
};

template <int DT, int RMODE, int QMODE>
__global__ __launch_bounds__(TPB) void binary_kernel(const void* __restrict__ a_, const void* __restrict__ b_,
                                                     void* __restrict__ out_, int64_t n, BinaryParams p) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    constexpr int UNROLL = 2;
    __shared__ unsigned char zone[ZONE_PAD];
    load_zone(zone, g_zone_tables[p.q.zone_row]);

    auto Q = [&](float v) {
        v = mxq_round_dt<ADT>(v);
        if (QMODE == SMQ_IDENT) return v;
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest(v, p.q.fmt.nan_from);
        return mxq_quant_elemwise<RMODE, ADT, true, true>(v, p.q.fmt, p.q.saturate != 0,
                                                          p.q.allow_denorm != 0, zone, ZS);
    };
    const bool tensor_b = p.mode == BIN_TENSOR_TENSOR;
    const bool swap = p.mode == BIN_SCALAR_TENSOR;
    auto eval = [&](float x, float y) {
        if (!tensor_b) y = p.scalar;
        const float l = swap ? y : x, r = swap ? x : y;
        switch (p.op) {
            case BIN_ADD: return Q(l + r);
            case BIN_SUB: return Q(l - r);
            case BIN_MUL: return Q(l * r);
            default:
                // scalar / tensor is torch's Tensor.__rtruediv__: reciprocal(), then times the scalar
                return swap ? Q(mxq_round_dt<ADT>(1.0f / r) * l) : Q(l / r);
        }
    };

    const u32x4* a = reinterpret_cast<const u32x4*>(a_);
    const u32x4* b = reinterpret_cast<const u32x4*>(b_);
    u32x4* out = reinterpret_cast<u32x4*>(out_);
    const int64_t n_vec = n / EPV;
    const int64_t stride = (int64_t)gridDim.x * TPB * UNROLL;
    for (int64_t base = (int64_t)blockIdx.x * TPB * UNROLL + threadIdx.x; base - threadIdx.x < n_vec;
         base += stride) {
        u32x4 va[UNROLL], vb[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + (int64_t)j * TPB;
            va[j] = (i < n_vec) ? a[i] : u32x4{0, 0, 0, 0};
            vb[j] = (tensor_b && i < n_vec) ? b[i] : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t i = base + (int64_t)j * TPB;
            u32x4 o;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                float r[2];
#pragma unroll
                for (int h = 0; h < PD; ++h) r[h] = eval(Pack<DT>::get(va[j][d], h), Pack<DT>::get(vb[j][d], h));
                o[d] = Pack<DT>::put(r[0], r[PD - 1]);
            }
            if (i < n_vec) __builtin_nontemporal_store(o, &out[i]);
        }
    }
    const int64_t t0 = n_vec * EPV;
    const int64_t gi = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (gi < n - t0) {
        const float r = eval(load_scalar<DT>(a_, t0 + gi), tensor_b ? load_scalar<DT>(b_, t0 + gi) : 0.0f);
        store_scalar<DT>(out_, t0 + gi, r);
    }
}

// Gradients of the weight and the bias of LayerNorm / RMSNorm over the last axis
// (mx/layernorm.py:51-59, 148-156): with g = Q(output gradient) -- quantized here, which changes
// nothing when the caller already has -- and z = the saved normalized input, both [rows, n],
//   grad_bias[c] = Q(sum over rows of g[r, c]),  grad_weight[c] = Q(sum over rows of Q(g[r, c] z[r, c]))
// where a sum is accumulated in fp32 and rounded to the tensor dtype once, as torch.sum does.
// Two launches that read g and z once: column sums of a chunk of rows per block (fp32 partials in a
// workspace), then the partials of a column added in a fixed order and quantized.
//
// norm_param_grad_partial_kernel: grid (column groups, row chunks).  A lane owns one 16-byte vector
// of columns; the four waves of a block take every fourth row of the chunk and add their sums up
// through LDS.  partial[(chunk * 2 + k) * n + c]: k = 0 weight, 1 bias.
template <int DT, int RMODE, int QMODE>
__global__ __launch_bounds__(TPB) void norm_param_grad_partial_kernel(const void* __restrict__ grad_,
                                                                      const void* __restrict__ znorm_,
                                                                      float* __restrict__ partial,
                                                                      int64_t rows, int n,
                                                                      int64_t rows_per_chunk, ElemParams q) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int PD = Pack<DT>::PER_DWORD;
    constexpr int EPV = 4 * PD;
    constexpr int WAVES = TPB / 64;
    constexpr int UNROLL = 4;
    __shared__ unsigned char zone[ZONE_PAD];
    __shared__ float red[WAVES][2 * EPV][64];
    load_zone(zone, g_zone_tables[q.zone_row]);

    auto Qd = [&](float v) {                                 // v: a value of the tensor dtype
        if (QMODE == SMQ_IDENT) return v;
        if (QMODE == SMQ_BF16) return mxq_quant_bf16_to_bfloat16_nearest(v, q.fmt.nan_from);
        return mxq_quant_elemwise<RMODE, ADT, true, true>(v, q.fmt, q.saturate != 0, q.allow_denorm != 0,
                                                          zone, ZS);
    };
    auto Q = [&](float v) { return Qd(mxq_round_dt<ADT>(v)); };

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nvec_row = n / EPV;
    const int cv = blockIdx.x * 64 + lane;
    const bool live = cv < nvec_row;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk;
    const int64_t r1 = (r0 + rows_per_chunk < rows) ? r0 + rows_per_chunk : rows;
    const u32x4* g = reinterpret_cast<const u32x4*>(grad_) + cv;
    const u32x4* z = reinterpret_cast<const u32x4*>(znorm_) + cv;

    float acc_w[EPV], acc_b[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc_w[e] = acc_b[e] = 0.0f;

    for (int64_t r = r0 + wave; r < r1; r += WAVES * UNROLL) {
        u32x4 vg[UNROLL], vz[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const int64_t rr = r + j * WAVES;
            const bool ok = live && rr < r1;
            // rows past the chunk read as +0 (they add nothing); lanes past the row read as 1.0 so that
            // they do not spoil the wave's vote below (their sums are never stored)
            const u32x4 pad = live ? u32x4{0, 0, 0, 0} : u32x4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
            vg[j] = ok ? __builtin_nontemporal_load(&g[rr * nvec_row]) : pad;
            vz[j] = ok ? __builtin_nontemporal_load(&z[rr * nvec_row]) : pad;
        }
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            if constexpr (QMODE == SMQ_BF16 && DT == MXQ_BF16) {
                // plain range: while every gradient of the wave's row piece and every rounded product is a
                // normal number below the NaN threshold, both quantizations are "odd significand -> + 1"
                // on the two halves of a dword at once; the sums take the same values in the same order
                const unsigned short span = (unsigned short)((q.fmt.nan_from >> 16) - 0x0080u);
                u16x2 worst = {0, 0};
                uint32_t gq[4], pq[4];
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    worst = __builtin_elementwise_max(
                        worst, __builtin_bit_cast(u16x2, vg[j][d] & 0x7FFF7FFFu) - u16x2{0x0080, 0x0080});
                    gq[d] = vg[j][d] + (vg[j][d] & 0x00010001u);
                    const uint32_t pw = Pack<MXQ_BF16>::put(
                        Pack<MXQ_BF16>::get(gq[d], 0) * Pack<MXQ_BF16>::get(vz[j][d], 0),
                        Pack<MXQ_BF16>::get(gq[d], 1) * Pack<MXQ_BF16>::get(vz[j][d], 1));
                    worst = __builtin_elementwise_max(
                        worst, __builtin_bit_cast(u16x2, pw & 0x7FFF7FFFu) - u16x2{0x0080, 0x0080});
                    pq[d] = pw + (pw & 0x00010001u);
                }
                if (__all(!q.general_only && worst[0] < span && worst[1] < span)) {
#pragma unroll
                    for (int d = 0; d < 4; ++d)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            acc_w[d * 2 + h] += Pack<MXQ_BF16>::get(pq[d], h);
                            acc_b[d * 2 + h] += Pack<MXQ_BF16>::get(gq[d], h);
                        }
                    continue;
                }
            }
#pragma unroll
            for (int d = 0; d < 4; ++d)                    // rows past the chunk were read as +0
#pragma unroll
                for (int h = 0; h < PD; ++h) {
                    const float gv = Qd(Pack<DT>::get(vg[j][d], h)), zv = Pack<DT>::get(vz[j][d], h);
                    acc_w[d * PD + h] += Q(gv * zv);
                    acc_b[d * PD + h] += gv;
                }
        }
    }
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
        red[wave][e][lane] = acc_w[e];
        red[wave][EPV + e][lane] = acc_b[e];
    }
    __syncthreads();
    if (!live) return;
    // wave w adds up and stores entries k = w, w + WAVES, ... of this lane's 2 * EPV sums
    float* dst = partial + (int64_t)blockIdx.y * 2 * n + (int64_t)cv * EPV;
    for (int k = wave; k < 2 * EPV; k += WAVES) {
        float s = red[0][k][lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) s += red[w][k][lane];
        dst[(k / EPV) * (int64_t)n + (k % EPV)] = s;
    }
}

// norm_param_grad_final_kernel: one lane per (k, column) pair, 64 pairs per block; wave w adds the
// partials of its quarter of the chunks in order, the four quarter sums are added in order, the
// result is rounded to the tensor dtype and quantized.  out_w / out_b: n elements each.
template <int DT, int RMODE, int QMODE>
__global__ __launch_bounds__(TPB) void norm_param_grad_final_kernel(const float* __restrict__ partial,
                                                                    int chunks, int n,
                                                                    void* __restrict__ out_w,
                                                                    void* __restrict__ out_b, ElemParams q) {
    constexpr int ADT = Arith<DT>::DT_;
    constexpr int ZS = (ADT == MXQ_BF16) ? 16 : 0;
    constexpr int WAVES = TPB / 64;
    __shared__ unsigned char zone[ZONE_PAD];
    __shared__ float red[WAVES][64];
    load_zone(zone, g_zone_tables[q.zone_row]);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t j = (int64_t)blockIdx.x * 64 + lane;         // k * n + column
    const bool live = j < 2 * (int64_t)n;
    const int per = (chunks + WAVES - 1) / WAVES;
    const int c0 = wave * per, c1 = (c0 + per < chunks) ? c0 + per : chunks;
    float s = 0.0f;
    if (live) {
        const float* src = partial + j;
        const int64_t step = 2 * (int64_t)n;
        int c = c0;
        for (; c + 8 <= c1; c += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[(c + u) * step];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; c < c1; ++c) s += src[c * step];
    }
    red[wave][lane] = s;
    __syncthreads();
    if (wave != 0 || !live) return;
#pragma unroll
    for (int w = 1; w < WAVES; ++w) s += red[w][lane];       // +0 from a wave without chunks
    float y = mxq_round_dt<ADT>(s);
    if (QMODE == SMQ_BF16) y = mxq_quant_bf16_to_bfloat16_nearest(y, q.fmt.nan_from);
    else if (QMODE != SMQ_IDENT)
        y = mxq_quant_elemwise<RMODE, ADT, true, true>(y, q.fmt, q.saturate != 0, q.allow_denorm != 0, zone, ZS);
    if (j < n) store_scalar<DT>(out_w, j, y);
    else store_scalar<DT>(out_b, j - n, y);
}

}  // namespace
