// C ABI of libmxq_gfx950.so, continued: the attention-score kernel (packed MX product + softmax).
#include "mxq_capi_common.h"
#include "mxq_bmm_softmax.h"

namespace {

template <int CB, int BL>
void launch_scores(const BmmSoftmaxArgs& g, int64_t batch, hipStream_t s) {
    const dim3 grid((unsigned)ceil_div(g.M, BS_ROWS), (unsigned)batch);
    mx_bmm_softmax_kernel<CB, BL><<<grid, kThreads, 0, s>>>(g);
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

int mxq_bmm_softmax_mx_nt(const void* a_codes, const void* a_scales, int a_kind, const void* b_codes,
                          const void* b_scales, int b_kind, void* out, int64_t batch, int64_t M, int64_t N,
                          int64_t K, int exp2, int flags, void* hip_stream) {
    const char* who = "mxq_bmm_softmax_mx_nt";
    if ((a_kind != MXQ_CODES_E4M3 && a_kind != MXQ_CODES_E5M2) || (b_kind != MXQ_CODES_E4M3 && b_kind != MXQ_CODES_E5M2))
        return fail(MXQ_ERR_ARGUMENT, "%s: operands must be 8-bit codes (e4m3 or e5m2), got kinds %d / %d", who, a_kind, b_kind);
    if (batch < 0 || M < 0 || N < 0 || K < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (K != 128) return fail(MXQ_ERR_ARGUMENT, "%s: K must be 128 (one K step), got %lld", who, (long long)K);
    if (N % 32 != 0 || N > BS_MAX_N)
        return fail(MXQ_ERR_ARGUMENT, "%s: N must be a multiple of 32 and at most %d, got %lld", who, BS_MAX_N, (long long)N);
    if (batch == 0 || M == 0 || N == 0) return MXQ_OK;
    if (M > 0x7FFFFFFF - BS_ROWS || batch > 65535) return fail(MXQ_ERR_ARGUMENT, "%s: size too large", who);
    if (!a_codes || !a_scales || !b_codes || !b_scales || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(a_codes) || !aligned16(b_codes) || !aligned16(out) || (reinterpret_cast<uintptr_t>(a_scales) & 3) ||
        (reinterpret_cast<uintptr_t>(b_scales) & 3))
        return fail(MXQ_ERR_ARGUMENT, "%s: codes and output must be 16-byte and scales 4-byte aligned", who);
    BmmSoftmaxArgs g;
    g.a = reinterpret_cast<const unsigned char*>(a_codes);
    g.sa = reinterpret_cast<const unsigned char*>(a_scales);
    g.b = reinterpret_cast<const unsigned char*>(b_codes);
    g.sb = reinterpret_cast<const unsigned char*>(b_scales);
    g.out = out;
    g.M = (int)M;
    g.N = (int)N;
    g.exp2 = exp2 ? 1 : 0;
    g.general_only = (flags & MXQ_FLAG_GENERAL_FORM) ? 1 : 0;
    ElemParams q;                                        // bfloat16, nearest: only the NaN threshold is needed
    int rc = make_elem_params(MXQ_DTYPE_BF16, 9, 8, 3.3895313892515355e38f, MXQ_ROUND_NEAREST, 0, 1, 0, &q, who);
    if (rc) return rc;
    g.q_nan_from = q.fmt.nan_from;
    g.batch_a = M * 128; g.batch_sa = M * 4;
    g.batch_b = N * 128; g.batch_sb = N * 4;
    g.batch_c = M * N;
    hipStream_t s = (hipStream_t)hip_stream;
    if (!a_kind && !b_kind) launch_scores<0, 0>(g, batch, s);
    else if (a_kind && !b_kind) launch_scores<1, 0>(g, batch, s);
    else if (!a_kind && b_kind) launch_scores<0, 1>(g, batch, s);
    else launch_scores<1, 1>(g, batch, s);
    return check_launch(who);
}

}  // extern "C"
#pragma GCC visibility pop
