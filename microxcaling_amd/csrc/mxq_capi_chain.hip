// C ABI of libmxq_gfx950.so, continued: kernels that run a whole chain of "tensor op, then
// elementwise quantizer" steps -- softmax forward and backward, activations, single vector ops.
#include "mxq_capi_chain.h"

#pragma GCC visibility push(default)
extern "C" {

int mxq_softmax_lastdim(const void* in, void* out, int dtype, int64_t rows, int64_t n, int bits,
                        int exp_bits, float max_norm, int rmode, int allow_denorm, int exp_mode,
                        int use_recip, int flags, void* hip_stream) {
    const char* who = "mxq_softmax_lastdim";
    SoftmaxParams p;
    bool ident, closed;
    int rc = chain_params(dtype, bits, exp_bits, max_norm, rmode, allow_denorm, flags, &p.q, &ident, &closed, who);
    if (rc) return rc;
    if (exp_mode < 0 || exp_mode > 2) return fail(MXQ_ERR_ARGUMENT, "%s: exp_mode %d outside [0, 2]", who, exp_mode);
    p.exp_mode = exp_mode;
    p.use_recip = use_recip ? 1 : 0;
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    if (rows < 0 || n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n > kMaxRow || n % epv != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most %lld",
                    who, (long long)n, epv, (long long)kMaxRow);
    if (rows == 0 || n == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(in) || !aligned16(out))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int64_t nvec = n / epv;                       // 16-byte vectors per row, 64 lanes
#define MXQ_SM(DT, RM, QM) MXQ_ROW_CASES(softmax_row_kernel, DT, RM, QM, in, out, rows, (int)n, p)
    MXQ_CHAIN_DISPATCH(MXQ_SM);
#undef MXQ_SM
    return check_launch(who);
}

int mxq_activation_forward(const void* in, void* out, void* aux, void* q_in, int dtype, int64_t n,
                           int act, int bits, int exp_bits, float max_norm, int rmode,
                           int allow_denorm, int exp_mode, int flags, void* hip_stream) {
    const char* who = "mxq_activation_forward";
    ActParams p;
    bool ident, closed;
    int rc = chain_params(dtype, bits, exp_bits, max_norm, rmode, allow_denorm, flags, &p.q, &ident, &closed, who);
    if (rc) return rc;
    if (act < ACT_SIGMOID || act > ACT_GELU) return fail(MXQ_ERR_ARGUMENT, "%s: unknown activation %d", who, act);
    if (exp_mode != 0 && exp_mode != 2) return fail(MXQ_ERR_ARGUMENT, "%s: exp_mode %d (0 or 2)", who, exp_mode);
    p.act = act;
    p.exp_mode = exp_mode;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(in) || !aligned16(out) || !aligned16(aux) || !aligned16(q_in))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    const int grid = grid_for(ceil_div(ceil_div(n, epv), (int64_t)kThreads));
#define MXQ_ACT(DT, RM, QM) activation_kernel<DT, RM, QM><<<grid, kThreads, 0, s>>>(in, out, aux, q_in, n, p)
    MXQ_CHAIN_DISPATCH(MXQ_ACT);
#undef MXQ_ACT
    return check_launch(who);
}

int mxq_activation_backward(const void* grad_out, const void* saved, const void* aux, void* grad_in,
                            int dtype, int64_t n, int act, int bits, int exp_bits, float max_norm,
                            int rmode, int allow_denorm, int flags, void* hip_stream) {
    const char* who = "mxq_activation_backward";
    ActParams p;
    bool ident, closed;
    int rc = chain_params(dtype, bits, exp_bits, max_norm, rmode, allow_denorm, flags, &p.q, &ident, &closed, who);
    if (rc) return rc;
    if (act < ACT_SIGMOID || act > ACT_GELU) return fail(MXQ_ERR_ARGUMENT, "%s: unknown activation %d", who, act);
    p.act = act;
    p.exp_mode = 0;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!grad_out || !saved || !grad_in || (act >= ACT_SILU && !aux))
        return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(grad_out) || !aligned16(saved) || !aligned16(aux) || !aligned16(grad_in))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    const int grid = grid_for(ceil_div(ceil_div(n, epv), (int64_t)kThreads));
#define MXQ_ACTB(DT, RM, QM) \
    activation_backward_kernel<DT, RM, QM><<<grid, kThreads, 0, s>>>(grad_out, saved, aux, grad_in, n, p)
    MXQ_CHAIN_DISPATCH(MXQ_ACTB);
#undef MXQ_ACTB
    return check_launch(who);
}

int mxq_softmax_backward_lastdim(const void* grad_out, const void* y, void* grad_in, int dtype,
                                 int64_t rows, int64_t n, int bits, int exp_bits, float max_norm,
                                 int rmode, int allow_denorm, int scale_ln2, int flags, void* hip_stream) {
    const char* who = "mxq_softmax_backward_lastdim";
    SoftmaxParams p;
    bool ident, closed;
    int rc = chain_params(dtype, bits, exp_bits, max_norm, rmode, allow_denorm, flags, &p.q, &ident, &closed, who);
    if (rc) return rc;
    p.exp_mode = scale_ln2 ? 1 : 0;
    p.use_recip = 0;
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    if (rows < 0 || n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n > kMaxRow || n % epv != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most %lld",
                    who, (long long)n, epv, (long long)kMaxRow);
    if (rows == 0 || n == 0) return MXQ_OK;
    if (!grad_out || !y || !grad_in) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(grad_out) || !aligned16(y) || !aligned16(grad_in))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int64_t nvec = n / epv;
#define MXQ_SMB(DT, RM, QM) MXQ_ROW_CASES(softmax_backward_row_kernel, DT, RM, QM, grad_out, y, grad_in, rows, (int)n, p)
    MXQ_CHAIN_DISPATCH(MXQ_SMB);
#undef MXQ_SMB
    return check_launch(who);
}

int mxq_binary_elemwise(const void* a, const void* b, float scalar, int mode, void* out, int dtype,
                        int64_t n, int op, int bits, int exp_bits, float max_norm, int rmode,
                        int allow_denorm, int flags, void* hip_stream) {
    const char* who = "mxq_binary_elemwise";
    BinaryParams p;
    bool ident, closed;
    int rc = chain_params(dtype, bits, exp_bits, max_norm, rmode, allow_denorm, flags, &p.q, &ident, &closed, who);
    if (rc) return rc;
    if (op < BIN_ADD || op > BIN_DIV) return fail(MXQ_ERR_ARGUMENT, "%s: unknown operation %d", who, op);
    if (mode < BIN_TENSOR_TENSOR || mode > BIN_SCALAR_TENSOR) return fail(MXQ_ERR_ARGUMENT, "%s: unknown mode %d", who, mode);
    p.op = op;
    p.mode = mode;
    p.scalar = scalar;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!a || !out || (mode == BIN_TENSOR_TENSOR && !b)) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(a) || !aligned16(out) || (mode == BIN_TENSOR_TENSOR && !aligned16(b)))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    const int grid = grid_for(ceil_div(ceil_div(n, epv), (int64_t)kThreads * 2));
#define MXQ_BIN(DT, RM, QM) binary_kernel<DT, RM, QM><<<grid, kThreads, 0, s>>>(a, b, out, n, p)
    MXQ_CHAIN_DISPATCH(MXQ_BIN);
#undef MXQ_BIN
    return check_launch(who);
}

}  // extern "C"
#pragma GCC visibility pop
