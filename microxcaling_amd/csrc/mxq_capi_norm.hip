// C ABI of libmxq_gfx950.so, continued: LayerNorm / RMSNorm row kernels, forward and backward.
#include "mxq_capi_chain.h"

#pragma GCC visibility push(default)
extern "C" {

int mxq_norm_lastdim(const void* in, const void* weight, const void* bias, void* out, void* x_norm,
                     void* row_stat, int dtype, int64_t rows, int64_t n, float eps, int rms_norm,
                     int bits, int exp_bits, float max_norm, int rmode, int allow_denorm, int flags,
                     void* hip_stream) {
    const char* who = "mxq_norm_lastdim";
    NormParams p;
    bool ident, closed;
    int rc = chain_params(dtype, bits, exp_bits, max_norm, rmode, allow_denorm, flags, &p.q, &ident, &closed, who);
    if (rc) return rc;
    p.eps = eps;
    p.rms = rms_norm ? 1 : 0;
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    if (rows < 0 || n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n > kMaxRow || n % epv != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most %lld",
                    who, (long long)n, epv, (long long)kMaxRow);
    if (rows == 0 || n == 0) return MXQ_OK;
    if (!in || !out || !weight || !bias || !row_stat) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(in) || !aligned16(out) || !aligned16(weight) || !aligned16(bias) || !aligned16(x_norm))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int64_t nvec = n / epv;
#define MXQ_NM(DT, RM, QM) MXQ_ROW_CASES(norm_row_kernel, DT, RM, QM, in, weight, bias, out, x_norm, row_stat, rows, (int)n, p)
    MXQ_CHAIN_DISPATCH(MXQ_NM);
#undef MXQ_NM
    return check_launch(who);
}

int mxq_norm_backward_lastdim(const void* grad_out, const void* weight, const void* x_norm,
                              const void* row_stat, void* grad_in, int dtype, int64_t rows, int64_t n,
                              int rms_norm, int bits, int exp_bits, float max_norm, int rmode,
                              int allow_denorm, int flags, void* hip_stream) {
    const char* who = "mxq_norm_backward_lastdim";
    NormParams p;
    bool ident, closed;
    int rc = chain_params(dtype, bits, exp_bits, max_norm, rmode, allow_denorm, flags, &p.q, &ident, &closed, who);
    if (rc) return rc;
    p.eps = 0.0f;
    p.rms = rms_norm ? 1 : 0;
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    if (rows < 0 || n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n > kMaxRow || n % epv != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most %lld",
                    who, (long long)n, epv, (long long)kMaxRow);
    if (rows == 0 || n == 0) return MXQ_OK;
    if (!grad_out || !weight || !x_norm || !row_stat || !grad_in) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(grad_out) || !aligned16(weight) || !aligned16(x_norm) || !aligned16(grad_in))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int64_t nvec = n / epv;
#define MXQ_NMB(DT, RM, QM) MXQ_ROW_CASES(norm_backward_row_kernel, DT, RM, QM, grad_out, weight, x_norm, row_stat, grad_in, rows, (int)n, p)
    MXQ_CHAIN_DISPATCH(MXQ_NMB);
#undef MXQ_NMB
    return check_launch(who);
}

}  // extern "C"
#pragma GCC visibility pop
