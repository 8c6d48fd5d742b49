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


// rows of a chunk and number of chunks of the column sums: about 2048 blocks, at least 16 rows each
static void param_grad_split(int64_t rows, int64_t n, int epv, int64_t* rows_per_chunk, int64_t* chunks) {
    const int64_t groups = ceil_div(n / epv, 64);
    int64_t want = kMaxBlocks / groups;
    if (want < 1) want = 1;
    int64_t per = ceil_div(rows, want);
    if (per < 16) per = 16;
    *rows_per_chunk = per;
    *chunks = ceil_div(rows, per);
}

int64_t mxq_norm_param_grads_workspace_bytes(int dtype, int64_t rows, int64_t n) {
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    if (rows <= 0 || n <= 0 || n % epv != 0) return 0;
    int64_t per, chunks;
    param_grad_split(rows, n, epv, &per, &chunks);
    return chunks * 2 * n * (int64_t)sizeof(float);
}

int mxq_norm_param_grads(const void* grad_out, const void* x_norm, void* grad_weight, void* grad_bias,
                         void* workspace, int64_t workspace_bytes, int dtype, int64_t rows, int64_t n,
                         int bits, int exp_bits, float max_norm, int rmode, int allow_denorm, int flags,
                         void* hip_stream) {
    const char* who = "mxq_norm_param_grads";
    ElemParams q;
    bool ident, closed;
    int rc = chain_params(dtype, bits, exp_bits, max_norm, rmode, allow_denorm, flags, &q, &ident, &closed, who);
    if (rc) return rc;
    const int epv = dtype == MXQ_DTYPE_F32 ? 4 : 8;
    if (rows < 0 || n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n % epv != 0 || n > (int64_t)1 << 30)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most 2^30", who,
                    (long long)n, epv);
    if (n == 0) return MXQ_OK;
    if (rows == 0) return fail(MXQ_ERR_ARGUMENT, "%s: no rows to add up", who);
    if (!grad_out || !x_norm || !grad_weight || !grad_bias || !workspace)
        return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(grad_out) || !aligned16(x_norm) || !aligned16(workspace))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    int64_t per, chunks;
    param_grad_split(rows, n, epv, &per, &chunks);
    if (workspace_bytes < chunks * 2 * n * (int64_t)sizeof(float))
        return fail(MXQ_ERR_ARGUMENT, "%s: workspace of %lld bytes, %lld needed", who, (long long)workspace_bytes,
                    (long long)(chunks * 2 * n * (int64_t)sizeof(float)));
    hipStream_t s = (hipStream_t)hip_stream;
    const dim3 grid1((unsigned)ceil_div(n / epv, 64), (unsigned)chunks);
    const unsigned grid2 = (unsigned)ceil_div(2 * n, 64);
    float* part = static_cast<float*>(workspace);
#define MXQ_PG(DT, RM, QM)                                                                                  \
    do {                                                                                                    \
        norm_param_grad_partial_kernel<DT, RM, QM><<<grid1, kThreads, 0, s>>>(grad_out, x_norm, part, rows,  \
                                                                              (int)n, per, q);              \
        norm_param_grad_final_kernel<DT, RM, QM><<<grid2, kThreads, 0, s>>>(part, (int)chunks, (int)n,       \
                                                                            grad_weight, grad_bias, q);     \
    } while (0)
    MXQ_CHAIN_DISPATCH(MXQ_PG);
#undef MXQ_PG
    return check_launch(who);
}

}  // extern "C"
#pragma GCC visibility pop
