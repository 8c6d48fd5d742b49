// Shared by the translation units with the chain kernels (mxq_capi_chain.hip, mxq_capi_norm.hip):
// format parameters, and which kernel instance serves them.
#pragma once
#include "mxq_capi_common.h"
#include "mxq_softmax.h"

namespace {

int chain_params(int dtype, int bits, int exp_bits, float max_norm, int rmode, int allow_denorm,
                        int flags, ElemParams* q, bool* ident, bool* closed, const char* who) {
    *ident = bits == 0;
    if (dtype != MXQ_DTYPE_F32 && dtype != MXQ_DTYPE_BF16)
        return fail(MXQ_ERR_ARGUMENT, "%s: dtype code %d (fp32 and bf16 tensors only)", who, dtype);
    int rc = make_elem_params(dtype, *ident ? 9 : bits, *ident ? 8 : exp_bits, *ident ? 1.0f : max_norm,
                              *ident ? MXQ_ROUND_NEAREST : rmode, 0, allow_denorm, flags, q, who);
    if (rc) return rc;
    if (!*ident && !lean_ok(dtype, q->fmt, rmode, true))
        return fail(MXQ_ERR_ARGUMENT, "%s: round-half-even to %d fraction bits on a bf16 tensor is "
                    "only available through the separate elementwise steps", who, q->fmt.t);
    *closed = !*ident && dtype == MXQ_DTYPE_BF16 && bits == 9 && exp_bits == 8 &&
              rmode == MXQ_ROUND_NEAREST && allow_denorm && q->fmt.max_bits == 0x7F7F0000u;
    return MXQ_OK;
}
// LAUNCH(DT, RMODE, QMODE) for the instance that serves (dtype, ident, closed, rmode)
#define MXQ_CHAIN_DISPATCH(LAUNCH)                                                   \
    do {                                                                             \
        if (dtype == MXQ_DTYPE_F32) {                                                \
            if (ident) LAUNCH(MXQ_F32, MXQ_NEAREST, SMQ_IDENT);                      \
            else if (rmode == MXQ_ROUND_FLOOR) LAUNCH(MXQ_F32, MXQ_FLOOR, SMQ_GENERIC);     \
            else if (rmode == MXQ_ROUND_NEAREST) LAUNCH(MXQ_F32, MXQ_NEAREST, SMQ_GENERIC); \
            else LAUNCH(MXQ_F32, MXQ_EVEN, SMQ_GENERIC);                             \
        } else {                                                                     \
            if (ident) LAUNCH(MXQ_BF16, MXQ_NEAREST, SMQ_IDENT);                     \
            else if (closed) LAUNCH(MXQ_BF16, MXQ_NEAREST, SMQ_BF16);                \
            else if (rmode == MXQ_ROUND_FLOOR) LAUNCH(MXQ_BF16, MXQ_FLOOR, SMQ_GENERIC);     \
            else if (rmode == MXQ_ROUND_NEAREST) LAUNCH(MXQ_BF16, MXQ_NEAREST, SMQ_GENERIC); \
            else LAUNCH(MXQ_BF16, MXQ_EVEN, SMQ_GENERIC);                            \
        }                                                                            \
    } while (0)

// Which code the element format packs to: MXQ_CODES_E4M3 / _E5M2 bytes, or _E2M1 nibbles when the
// caller asks for them (MXQ_FLAG_PACK_NIBBLES, fp4 only); -1 = no packed form.
// KERNEL<DT, RM, QM, vectors per lane, waves per row> for rows of nvec 16-byte vectors: one wave per
// row up to 256 (fp32: 512) vectors, two or four waves above (64 values of a row per lane cost a
// third of the occupancy: LayerNorm on rows of 4096 bf16 values, 0.227 -> 0.192 ms with two waves)
#define MXQ_ROW_CASES(KERNEL, DT, RM, QM, ...)                                                      \
    do {                                                                                            \
        constexpr int V = (DT == MXQ_F32) ? 2 : 1;                                                  \
        const int g1 = grid_for(ceil_div(rows, 4)), g2 = grid_for(ceil_div(rows, 2)), g4 = grid_for(rows); \
        if (nvec <= 128 * V) KERNEL<DT, RM, QM, 2 * V, 1><<<g1, kThreads, 0, s>>>(__VA_ARGS__);       \
        else if (nvec <= 256 * V) KERNEL<DT, RM, QM, 4 * V, 1><<<g1, kThreads, 0, s>>>(__VA_ARGS__);  \
        else if (nvec <= 512 * V) KERNEL<DT, RM, QM, 4 * V, 2><<<g2, kThreads, 0, s>>>(__VA_ARGS__);  \
        else if (nvec <= 1024 * V) KERNEL<DT, RM, QM, 8 * V, 2><<<g2, kThreads, 0, s>>>(__VA_ARGS__); \
        else KERNEL<DT, RM, QM, 8 * V, 4><<<g4, kThreads, 0, s>>>(__VA_ARGS__);                        \
    } while (0)
constexpr int64_t kMaxRow = 16384;                           // elements in a row the row kernels hold

}  // namespace
