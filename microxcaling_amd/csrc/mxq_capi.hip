// C ABI of libmxq_gfx950.so: argument checks, kernel selection and launch geometry.
// Declarations and the reference functions each entry point replaces are in include/mxq.h.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxq.h"
#include "mxq_kernels.h"
#include "mxq_gemm.h"
#include "mxq_softmax.h"

namespace {

using namespace mxq_detail;

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MXQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MXQ_OK;
}

constexpr int kThreads = 256;
constexpr int64_t kMaxBlocks = 256 * 8;      // 256 CUs x 8 resident blocks of 256 lanes

int grid_for(int64_t work_items_per_block_iter_total) {
    int64_t g = work_items_per_block_iter_total;
    if (g < 1) g = 1;
    if (g > kMaxBlocks) g = kMaxBlocks;
    return (int)g;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int elem_size(int dtype) { return dtype == MXQ_DTYPE_F32 ? 4 : 2; }

// ---- dispatch over (dtype, rounding mode, element zone, lean) ------------------------------------
// F is a functor template: F<DT, RMODE, ZONE_ELEM, LEAN>::run(args...).  The op-by-op form always
// consults the zone table, so it exists once per rounding mode, and only bf16 tensors need it.
template <template <int, int, bool, bool> class F, int DT, typename... A>
void dispatch_round(int rmode, bool zone_elem, bool lean, A... a) {
    if (DT == MXQ_BF16 && !lean) {
        if (rmode == MXQ_ROUND_FLOOR) F<MXQ_BF16, MXQ_FLOOR, true, false>::run(a...);
        else if (rmode == MXQ_ROUND_NEAREST) F<MXQ_BF16, MXQ_NEAREST, true, false>::run(a...);
        else F<MXQ_BF16, MXQ_EVEN, true, false>::run(a...);
        return;
    }
    if (rmode == MXQ_ROUND_FLOOR) {
        if (zone_elem) F<DT, MXQ_FLOOR, true, true>::run(a...);
        else F<DT, MXQ_FLOOR, false, true>::run(a...);
    } else if (rmode == MXQ_ROUND_NEAREST) {
        if (zone_elem) F<DT, MXQ_NEAREST, true, true>::run(a...);
        else F<DT, MXQ_NEAREST, false, true>::run(a...);
    } else {
        if (zone_elem) F<DT, MXQ_EVEN, true, true>::run(a...);
        else F<DT, MXQ_EVEN, false, true>::run(a...);
    }
}
template <template <int, int, bool, bool> class F, typename... A>
void dispatch(int dtype, int rmode, bool zone_elem, bool lean, A... a) {
    if (dtype == MXQ_DTYPE_F32) dispatch_round<F, MXQ_F32>(rmode, zone_elem, lean, a...);
    else if (dtype == MXQ_DTYPE_BF16) dispatch_round<F, MXQ_BF16>(rmode, zone_elem, lean, a...);
    else dispatch_round<F, MXQ_F16>(rmode, zone_elem, lean, a...);
}

constexpr int kLastAxisUnroll = 4;

template <int DT, int RMODE, bool ZE, bool LEAN>
struct LaunchLastAxis {
    static void run(const void* in, void* out, int64_t n_vec, int lpt, MxParams p, hipStream_t s) {
        const int grid = grid_for(ceil_div(n_vec, (int64_t)kThreads * kLastAxisUnroll));
        const u32x4* i4 = reinterpret_cast<const u32x4*>(in);
        u32x4* o4 = reinterpret_cast<u32x4*>(out);
#define MXQ_CASE(L)                                                                               \
    case L:                                                                                       \
        mx_lastaxis_kernel<DT, RMODE, ZE, LEAN, L, kLastAxisUnroll><<<grid, kThreads, 0, s>>>(i4, o4, n_vec, p); \
        break;
        switch (lpt) {
            MXQ_CASE(1) MXQ_CASE(2) MXQ_CASE(4) MXQ_CASE(8) MXQ_CASE(16)
        }
#undef MXQ_CASE
    }
};

template <int DT, int RMODE, bool ZE, bool LEAN>
struct LaunchStrided {
    static void run(const void* in, void* out, int64_t pre, int64_t axis, int64_t post, int64_t tile,
                    bool aligned, MxParams p, hipStream_t s) {
        constexpr int VW8 = (DT == MXQ_F32) ? 2 : 4;        // elements in 8 bytes
        constexpr int VW16 = (DT == MXQ_F32) ? 4 : 8;       // elements in 16 bytes
        const int64_t num_tiles = ceil_div(axis, tile);
        if (aligned && tile == 32 && axis % 32 == 0 && post % VW8 == 0) {
            const int64_t pv = post / VW8;
            const int64_t items = pre * num_tiles * pv;
            const int64_t blocks = ceil_div(items, kThreads);
            if (blocks <= 0x7FFFFFFF) {
                mx_strided_tile_kernel<DT, RMODE, ZE, LEAN, 32><<<(unsigned)blocks, kThreads, 0, s>>>(
                    reinterpret_cast<const u32x2*>(in), reinterpret_cast<u32x2*>(out), items, num_tiles, pv, p);
                return;
            }
        }
        if (aligned && post % VW16 == 0) {
            const int64_t items = pre * num_tiles * (post / VW16);
            mx_strided_kernel<DT, RMODE, ZE, LEAN, VW16><<<grid_for(ceil_div(items, kThreads)), kThreads, 0, s>>>(
                in, out, pre, axis, post, tile, num_tiles, p);
        } else {
            const int64_t items = pre * num_tiles * post;
            mx_strided_kernel<DT, RMODE, ZE, LEAN, 1><<<grid_for(ceil_div(items, kThreads)), kThreads, 0, s>>>(
                in, out, pre, axis, post, tile, num_tiles, p);
        }
    }
};

template <int DT, int RMODE, bool ZE, bool LEAN>
struct LaunchGivenMax {
    static void run(const void* in, void* out, const void* maxv, int64_t total, int64_t axis,
                    int64_t post, MxParams p, hipStream_t s) {
        const int grid = grid_for(ceil_div(total, kThreads * 4));
        mx_given_max_kernel<DT, RMODE, ZE, LEAN><<<grid, kThreads, 0, s>>>(in, out, maxv, total, axis, post, p);
    }
};

constexpr int kElemUnroll = 4;

template <int DT, int RMODE, bool ZE, bool LEAN>
struct LaunchElemwise {
    static void run(const void* in, void* out, int64_t n, ElemParams p, hipStream_t s) {
        const int epv = (DT == MXQ_F32) ? 4 : 8;
        const int grid = grid_for(ceil_div(ceil_div(n, epv), (int64_t)kThreads * kElemUnroll));
        elemwise_kernel<DT, RMODE, ZE, LEAN, kElemUnroll><<<grid, kThreads, 0, s>>>(in, out, n, p);
    }
};

template <int DT, int RMODE, bool ZE, bool LEAN>
struct LaunchPack {
    static void run(const void* in, void* codes, void* scales, int64_t n_vec, int kind, MxParams p,
                    hipStream_t s) {
        const int grid = grid_for(ceil_div(n_vec, (int64_t)kThreads * 4));
        const u32x4* i4 = reinterpret_cast<const u32x4*>(in);
        unsigned char* sc = reinterpret_cast<unsigned char*>(scales);
        if (kind == 1) mx_pack_kernel<DT, RMODE, ZE, 1, 4><<<grid, kThreads, 0, s>>>(i4, codes, sc, n_vec, p);
        else if (kind == 4) mx_pack_kernel<DT, RMODE, ZE, 4, 4><<<grid, kThreads, 0, s>>>(i4, codes, sc, n_vec, p);
        else mx_pack_kernel<DT, RMODE, ZE, 0, 4><<<grid, kThreads, 0, s>>>(i4, codes, sc, n_vec, p);
    }
};

template <int DT, int RMODE, bool ZE, bool LEAN>
struct LaunchPackT {
    static void run(const void* in, void* codes, void* scales, int64_t items, int64_t n_tiles,
                    int64_t pv, int kind, MxParams p, hipStream_t s) {
        const unsigned grid = (unsigned)ceil_div(items, kThreads);
        const u32x2* i2 = reinterpret_cast<const u32x2*>(in);
        unsigned char* c = reinterpret_cast<unsigned char*>(codes);
        unsigned char* sc = reinterpret_cast<unsigned char*>(scales);
        if (kind == 1) mx_pack_t_kernel<DT, RMODE, ZE, 1><<<grid, kThreads, 0, s>>>(i2, c, sc, items, n_tiles, pv, p);
        else if (kind == 4) mx_pack_t_kernel<DT, RMODE, ZE, 4><<<grid, kThreads, 0, s>>>(i2, c, sc, items, n_tiles, pv, p);
        else mx_pack_t_kernel<DT, RMODE, ZE, 0><<<grid, kThreads, 0, s>>>(i2, c, sc, items, n_tiles, pv, p);
    }
};

template <int CB, int BL, int ODT>
int launch_gemm_dt(int64_t batch, const GemmArgs& g, hipStream_t s) {
    // large problems: persistent 256 x 256 tile kernel (144 KB of dynamic LDS, one workgroup per CU);
    // it fetches 16 scale bytes per row at a time, hence K % 512
    const int64_t tiles_m = ceil_div(g.M, G2_BM), tiles_n = ceil_div(g.N, G2_BN);
    const int64_t total = tiles_m * tiles_n * batch;
    if (g.M >= 512 && g.N >= 512 && g.K % 512 == 0 && (int64_t)256 * g.kbytes < ((int64_t)1 << 31) &&
        total < ((int64_t)1 << 30)) {
        static bool configured = false;               // raising the dynamic-LDS limit is per kernel
        static int cus = 0;
        if (!configured) {
            hipError_t e = hipFuncSetAttribute(
                reinterpret_cast<const void*>(&mx_gemm_nt_kernel_256p<CB, BL, ODT>),
                hipFuncAttributeMaxDynamicSharedMemorySize, G3_LDS_BYTES);
            int dev = 0;
            if (e == hipSuccess) e = hipGetDevice(&dev);
            if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e != hipSuccess || cus <= 0)
                return fail(MXQ_ERR_LAUNCH, "mxq_gemm_mx_nt: cannot configure the tile kernel (%d bytes of LDS): %s",
                            G3_LDS_BYTES, hipGetErrorString(e));
            cus -= cus % 8;                           // a workgroup must stay on its XCD from tile to tile
            if (cus < 8) cus = 8;
            configured = true;
        }
        const unsigned grid = (unsigned)(total < cus ? total : cus);
        mx_gemm_nt_kernel_256p<CB, BL, ODT><<<grid, 512, G3_LDS_BYTES, s>>>(g, (int)tiles_m, (int)tiles_n, (int)total);
    } else {
        dim3 grid((unsigned)(ceil_div(g.N, GEMM_BN) * ceil_div(g.M, GEMM_BM)), (unsigned)batch);
        mx_gemm_nt_kernel<CB, BL, ODT><<<grid, kThreads, 0, s>>>(g);
    }
    return MXQ_OK;
}

template <int CB, int BL>
int launch_gemm(int c_dtype, int64_t batch, const GemmArgs& g, hipStream_t s) {
    if (c_dtype == MXQ_DTYPE_F32) return launch_gemm_dt<CB, BL, MXQ_F32>(batch, g, s);
    if (c_dtype == MXQ_DTYPE_BF16) return launch_gemm_dt<CB, BL, MXQ_BF16>(batch, g, s);
    return launch_gemm_dt<CB, BL, MXQ_F16>(batch, g, s);
}

// splits of the outer axis for the two-pass outer reduction
int64_t outer_splits(int64_t outer, int64_t inner) {
    const int vw = (inner % 4 == 0) ? 4 : 1;
    const int64_t col_blocks = ceil_div(ceil_div(inner, vw), kThreads);
    int64_t s = ceil_div(2 * kMaxBlocks, col_blocks);
    const int64_t most = ceil_div(outer, 32);          // at least 32 rows per split
    if (s > most) s = most;
    if (s < 1) s = 1;
    if (s > 65535) s = 65535;
    return s;
}

template <class OP>
int reduce_inner(const float* in, float* out, int64_t rows, int64_t inner, void* stream, const char* who) {
    if (rows < 0 || inner < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (rows == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    hipStream_t s = (hipStream_t)stream;
    if (inner >= 2048) {
        const int grid = (int)(rows < 65536 ? rows : 65536);
        reduce_inner_block_kernel<OP><<<grid, kThreads, 0, s>>>(in, out, rows, inner);
    } else {
        const int grid = grid_for(ceil_div(rows, kThreads / 64));
        reduce_inner_wave_kernel<OP><<<grid, kThreads, 0, s>>>(in, out, rows, inner);
    }
    return check_launch(who);
}

template <class OP>
int reduce_outer(const float* in, float* out, void* workspace, int64_t outer, int64_t inner,
                 void* stream, const char* who) {
    if (outer < 0 || inner < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (inner == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    hipStream_t s = (hipStream_t)stream;
    const int64_t splits = outer_splits(outer, inner);
    if (splits > 1 && !workspace) return fail(MXQ_ERR_ARGUMENT, "%s: workspace required", who);
    const bool vec = (inner % 4 == 0) && aligned16(in) && aligned16(out) && (splits == 1 || aligned16(workspace));
    const int64_t rows_per_split = ceil_div(outer > 0 ? outer : 1, splits);
    float* partial = splits == 1 ? out : reinterpret_cast<float*>(workspace);
    dim3 grid((unsigned)ceil_div(ceil_div(inner, vec ? 4 : 1), kThreads), (unsigned)splits);
    if (vec) reduce_outer_kernel<OP, 4><<<grid, kThreads, 0, s>>>(in, partial, outer, inner, rows_per_split);
    else reduce_outer_kernel<OP, 1><<<grid, kThreads, 0, s>>>(in, partial, outer, inner, rows_per_split);
    int rc = check_launch(who);
    if (rc || splits == 1) return rc;
    reduce_outer_final_kernel<OP><<<(unsigned)ceil_div(inner, 64), kThreads, 0, s>>>(partial, out, splits, inner);
    return check_launch(who);
}

// shared by the chain kernels: format parameters, and which kernel instance serves them
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
int code_kind(int ebits, int mbits, int flags, const char* who) {
    const bool fp4 = ebits == 2 && mbits == 3;
    if (flags & MXQ_FLAG_PACK_NIBBLES) {
        if (!fp4) {
            fail(MXQ_ERR_ARGUMENT, "%s: 4-bit codes exist for the e2m1 format only", who);
            return -1;
        }
        return MXQ_CODES_E2M1;
    }
    if (ebits == 5 && mbits <= 4) return MXQ_CODES_E5M2;
    if (ebits >= 2 && ebits <= 4 && mbits <= 5) return MXQ_CODES_E4M3;
    fail(MXQ_ERR_ARGUMENT, "%s: element format e%dm%d has no 8-bit float code (supported: up to "
         "e4m3, and e5m2)", who, ebits, mbits - 2);
    return -1;
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

const char* mxq_last_error(void) { return last_error().c_str(); }

int mxq_version(void) { return 100; }

int mxq_quantize_mx_by_tile(const void* in, void* out, int dtype, int64_t pre, int64_t axis_size,
                            int64_t post, int scale_bits, int elem_ebits, int elem_mbits,
                            float elem_max_norm, int64_t tile_size, int flush_fp32_subnorms,
                            int rmode, int flags, void* hip_stream) {
    const char* who = "mxq_quantize_mx_by_tile";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, rmode, flags, &p, &ze, who);
    if (rc) return rc;
    if (pre < 0 || axis_size < 0 || post < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    int64_t total;
    if (mul_overflows(pre, axis_size, post, &total)) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
    if (total == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    int64_t tile = (tile_size <= 0 || tile_size > axis_size) ? axis_size : tile_size;
    hipStream_t s = (hipStream_t)hip_stream;

    const int vec_elems = 16 / elem_size(dtype);
    const bool ptr_ok = aligned16(in) && aligned16(out);
    if (post == 1 && ptr_ok && axis_size % tile == 0 && tile % vec_elems == 0) {
        const int64_t lpt = tile / vec_elems;
        if (lpt == 1 || lpt == 2 || lpt == 4 || lpt == 8 || lpt == 16) {
            dispatch<LaunchLastAxis>(dtype, rmode, ze, lean_ok(dtype, p.fmt, rmode, false), in, out, total / vec_elems, (int)lpt, p, s);
            return check_launch(who);
        }
    }
    dispatch<LaunchStrided>(dtype, rmode, ze, lean_ok(dtype, p.fmt, rmode, false), in, out, pre, axis_size, post, tile, ptr_ok, p, s);
    return check_launch(who);
}

int mxq_quantize_mx_given_max(const void* in, void* out, const void* max_values, int dtype,
                              int64_t pre, int64_t axis_size, int64_t post, int scale_bits,
                              int elem_ebits, int elem_mbits, float elem_max_norm,
                              int flush_fp32_subnorms, int rmode, int flags, void* hip_stream) {
    const char* who = "mxq_quantize_mx_given_max";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, rmode, flags, &p, &ze, who);
    if (rc) return rc;
    if (pre < 0 || axis_size < 0 || post < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    int64_t total;
    if (mul_overflows(pre, axis_size, post, &total)) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
    if (total == 0) return MXQ_OK;
    if (!in || !out || !max_values) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    dispatch<LaunchGivenMax>(dtype, rmode, ze, lean_ok(dtype, p.fmt, rmode, false), in, out, max_values, total, axis_size, post, p,
                             (hipStream_t)hip_stream);
    return check_launch(who);
}

int mxq_quantize_elemwise(const void* in, void* out, int dtype, int64_t n, int bits, int exp_bits,
                          float max_norm, int rmode, int saturate_normals, int allow_denorm,
                          int flags, void* hip_stream) {
    const char* who = "mxq_quantize_elemwise";
    ElemParams p;
    int rc = make_elem_params(dtype, bits, exp_bits, max_norm, rmode, saturate_normals, allow_denorm,
                              flags, &p, who);
    if (rc) return rc;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(in) || !aligned16(out))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    dispatch<LaunchElemwise>(dtype, rmode, elem_zone_matters(dtype, flags, p.fmt, rmode), lean_ok(dtype, p.fmt, rmode, true), in, out, n, p, (hipStream_t)hip_stream);
    return check_launch(who);
}

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
    if (n > 4096 || n % epv != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most 4096",
                    who, (long long)n, epv);
    if (rows == 0 || n == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(in) || !aligned16(out))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int grid = grid_for(ceil_div(rows, kThreads / 64));
    const int64_t nvec = n / epv;                       // 16-byte vectors per row, 64 lanes
#define MXQ_SM(DT, RM, QM)                                                                         \
    do {                                                                                           \
        constexpr int V = (DT == MXQ_F32) ? 2 : 1;                                                 \
        if (nvec <= 128 * V) softmax_row_kernel<DT, RM, QM, 2 * V><<<grid, kThreads, 0, s>>>(in, out, rows, (int)n, p);      \
        else if (nvec <= 256 * V) softmax_row_kernel<DT, RM, QM, 4 * V><<<grid, kThreads, 0, s>>>(in, out, rows, (int)n, p); \
        else softmax_row_kernel<DT, RM, QM, 8 * V><<<grid, kThreads, 0, s>>>(in, out, rows, (int)n, p);                     \
    } while (0)
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
    if (n > 4096 || n % epv != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most 4096",
                    who, (long long)n, epv);
    if (rows == 0 || n == 0) return MXQ_OK;
    if (!grad_out || !y || !grad_in) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(grad_out) || !aligned16(y) || !aligned16(grad_in))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int grid = grid_for(ceil_div(rows, kThreads / 64));
    const int64_t nvec = n / epv;
#define MXQ_SMB(DT, RM, QM)                                                                         \
    do {                                                                                            \
        constexpr int V = (DT == MXQ_F32) ? 2 : 1;                                                  \
        if (nvec <= 128 * V) softmax_backward_row_kernel<DT, RM, QM, 2 * V><<<grid, kThreads, 0, s>>>(grad_out, y, grad_in, rows, (int)n, p);      \
        else if (nvec <= 256 * V) softmax_backward_row_kernel<DT, RM, QM, 4 * V><<<grid, kThreads, 0, s>>>(grad_out, y, grad_in, rows, (int)n, p); \
        else softmax_backward_row_kernel<DT, RM, QM, 8 * V><<<grid, kThreads, 0, s>>>(grad_out, y, grad_in, rows, (int)n, p);                     \
    } while (0)
    MXQ_CHAIN_DISPATCH(MXQ_SMB);
#undef MXQ_SMB
    return check_launch(who);
}

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
    if (n > 4096 || n % epv != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most 4096",
                    who, (long long)n, epv);
    if (rows == 0 || n == 0) return MXQ_OK;
    if (!in || !out || !weight || !bias || !row_stat) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(in) || !aligned16(out) || !aligned16(weight) || !aligned16(bias) || !aligned16(x_norm))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int grid = grid_for(ceil_div(rows, kThreads / 64));
    const int64_t nvec = n / epv;
#define MXQ_NM(DT, RM, QM)                                                                         \
    do {                                                                                           \
        constexpr int V = (DT == MXQ_F32) ? 2 : 1;                                                 \
        if (nvec <= 128 * V) norm_row_kernel<DT, RM, QM, 2 * V><<<grid, kThreads, 0, s>>>(in, weight, bias, out, x_norm, row_stat, rows, (int)n, p);      \
        else if (nvec <= 256 * V) norm_row_kernel<DT, RM, QM, 4 * V><<<grid, kThreads, 0, s>>>(in, weight, bias, out, x_norm, row_stat, rows, (int)n, p); \
        else norm_row_kernel<DT, RM, QM, 8 * V><<<grid, kThreads, 0, s>>>(in, weight, bias, out, x_norm, row_stat, rows, (int)n, p);                     \
    } while (0)
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
    if (n > 4096 || n % epv != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: row length %lld must be a multiple of %d and at most 4096",
                    who, (long long)n, epv);
    if (rows == 0 || n == 0) return MXQ_OK;
    if (!grad_out || !weight || !x_norm || !row_stat || !grad_in) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(grad_out) || !aligned16(weight) || !aligned16(x_norm) || !aligned16(grad_in))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int grid = grid_for(ceil_div(rows, kThreads / 64));
    const int64_t nvec = n / epv;
#define MXQ_NMB(DT, RM, QM)                                                                        \
    do {                                                                                           \
        constexpr int V = (DT == MXQ_F32) ? 2 : 1;                                                 \
        if (nvec <= 128 * V) norm_backward_row_kernel<DT, RM, QM, 2 * V><<<grid, kThreads, 0, s>>>(grad_out, weight, x_norm, row_stat, grad_in, rows, (int)n, p);      \
        else if (nvec <= 256 * V) norm_backward_row_kernel<DT, RM, QM, 4 * V><<<grid, kThreads, 0, s>>>(grad_out, weight, x_norm, row_stat, grad_in, rows, (int)n, p); \
        else norm_backward_row_kernel<DT, RM, QM, 8 * V><<<grid, kThreads, 0, s>>>(grad_out, weight, x_norm, row_stat, grad_in, rows, (int)n, p);                     \
    } while (0)
    MXQ_CHAIN_DISPATCH(MXQ_NMB);
#undef MXQ_NMB
    return check_launch(who);
}

int mxq_pack_mx(const void* in, void* codes, void* scales, int dtype, int64_t rows, int64_t K,
                int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                int flush_fp32_subnorms, int rmode, int flags, void* hip_stream) {
    const char* who = "mxq_pack_mx";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, rmode, flags, &p, &ze, who);
    if (rc) return rc;
    const int kind = code_kind(elem_ebits, elem_mbits, flags, who);
    if (kind < 0) return MXQ_ERR_ARGUMENT;
    if (rows < 0 || K < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (K % 32 != 0) return fail(MXQ_ERR_ARGUMENT, "%s: K must be a multiple of the block size 32", who);
    int64_t total;
    if (mul_overflows(rows, K, 1, &total)) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
    if (total == 0) return MXQ_OK;
    if (!in || !codes || !scales) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(in) || !aligned16(codes))
        return fail(MXQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", who);
    dispatch<LaunchPack>(dtype, rmode, ze, true, in, codes, scales, total / (16 / elem_size(dtype)), kind,
                         p, (hipStream_t)hip_stream);
    return check_launch(who);
}

int mxq_pack_mx_t(const void* in, void* codes, void* scales, int dtype, int64_t batch, int64_t R,
                  int64_t C, int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                  int flush_fp32_subnorms, int rmode, int flags, void* hip_stream) {
    const char* who = "mxq_pack_mx_t";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, rmode, flags, &p, &ze, who);
    if (rc) return rc;
    const int kind = code_kind(elem_ebits, elem_mbits, flags, who);
    if (kind < 0) return MXQ_ERR_ARGUMENT;
    if (batch < 0 || R < 0 || C < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    const int vw = 8 / elem_size(dtype);                 // columns in the 8 bytes a lane owns
    if (R % 32 != 0 || C % vw != 0)
        return fail(MXQ_ERR_ARGUMENT, "%s: R must be a multiple of 32 and C of %d", who, vw);
    int64_t total;
    if (mul_overflows(batch, R, C, &total)) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
    if (total == 0) return MXQ_OK;
    if (!in || !codes || !scales) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if ((reinterpret_cast<uintptr_t>(in) & 7) || !aligned16(codes))
        return fail(MXQ_ERR_ARGUMENT, "%s: input must be 8-byte and codes 16-byte aligned", who);
    const int64_t n_tiles = R / 32, pv = C / vw, items = batch * n_tiles * pv;
    if (ceil_div(items, kThreads) > 0x7FFFFFFF) return fail(MXQ_ERR_ARGUMENT, "%s: tensor too large", who);
    dispatch<LaunchPackT>(dtype, rmode, ze, true, in, codes, scales, items, n_tiles, pv, kind, p,
                          (hipStream_t)hip_stream);
    return check_launch(who);
}

int mxq_unpack_mx(const void* codes, const void* scales, int code_kind, void* out, int dtype,
                  int64_t rows, int64_t K, void* hip_stream) {
    const char* who = "mxq_unpack_mx";
    if (dtype < 0 || dtype > 2) return fail(MXQ_ERR_ARGUMENT, "%s: unknown dtype code %d", who, dtype);
    if (code_kind != MXQ_CODES_E4M3 && code_kind != MXQ_CODES_E5M2 && code_kind != MXQ_CODES_E2M1)
        return fail(MXQ_ERR_ARGUMENT, "%s: unknown code kind %d", who, code_kind);
    if (rows < 0 || K < 0 || K % 32 != 0) return fail(MXQ_ERR_ARGUMENT, "%s: bad size", who);
    const int64_t n = rows * K;
    if (n == 0) return MXQ_OK;
    if (!codes || !scales || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    const unsigned char* cd = reinterpret_cast<const unsigned char*>(codes);
    const unsigned char* sc = reinterpret_cast<const unsigned char*>(scales);
    hipStream_t s = (hipStream_t)hip_stream;
    const int grid = grid_for(ceil_div(n, kThreads * 4));
#define MXQ_UNPACK(DT)                                                                       \
    if (code_kind == 1) mx_unpack_kernel<DT, 1><<<grid, kThreads, 0, s>>>(cd, sc, out, n);      \
    else if (code_kind == 4) mx_unpack_kernel<DT, 4><<<grid, kThreads, 0, s>>>(cd, sc, out, n); \
    else mx_unpack_kernel<DT, 0><<<grid, kThreads, 0, s>>>(cd, sc, out, n);
    if (dtype == MXQ_DTYPE_F32) { MXQ_UNPACK(MXQ_F32) }
    else if (dtype == MXQ_DTYPE_BF16) { MXQ_UNPACK(MXQ_BF16) }
    else { MXQ_UNPACK(MXQ_F16) }
#undef MXQ_UNPACK
    return check_launch(who);
}

int mxq_gemm_mx_nt(const void* a_codes, const void* a_scales, int a_kind, const void* b_codes,
                   const void* b_scales, int b_kind, const void* bias, void* c, int c_dtype,
                   int64_t batch, int64_t M, int64_t N, int64_t K, int epilogue_quant,
                   void* hip_stream) {
    const char* who = "mxq_gemm_mx_nt";
    if (c_dtype < 0 || c_dtype > 2) return fail(MXQ_ERR_ARGUMENT, "%s: unknown dtype code %d", who, c_dtype);
    if (epilogue_quant != 0 && (epilogue_quant != 1 || c_dtype != MXQ_DTYPE_BF16))
        return fail(MXQ_ERR_ARGUMENT, "%s: epilogue_quant must be 0, or 1 with a bf16 output", who);
    if (batch < 0 || M < 0 || N < 0 || K < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    const bool nib = a_kind == MXQ_CODES_E2M1;
    if ((a_kind != MXQ_CODES_E4M3 && a_kind != MXQ_CODES_E5M2 && a_kind != MXQ_CODES_E2M1) ||
        (b_kind != MXQ_CODES_E4M3 && b_kind != MXQ_CODES_E5M2 && b_kind != MXQ_CODES_E2M1))
        return fail(MXQ_ERR_ARGUMENT, "%s: unknown code kind %d / %d", who, a_kind, b_kind);
    if (nib != (b_kind == MXQ_CODES_E2M1))
        return fail(MXQ_ERR_ARGUMENT, "%s: e2m1 nibble codes need both operands in that form", who);
    const int kstep = nib ? 2 * GEMM_BK : GEMM_BK;      // elements in a 128-byte K step
    if (K % kstep != 0) return fail(MXQ_ERR_ARGUMENT, "%s: K must be a multiple of %d", who, kstep);
    if (batch == 0 || M == 0 || N == 0) return MXQ_OK;
    if (K == 0) return fail(MXQ_ERR_ARGUMENT, "%s: K must be positive", who);
    if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF || batch > 65535)
        return fail(MXQ_ERR_ARGUMENT, "%s: size too large", who);
    if (!a_codes || !a_scales || !b_codes || !b_scales || !c) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (!aligned16(a_codes) || !aligned16(b_codes) || (reinterpret_cast<uintptr_t>(a_scales) & 3) ||
        (reinterpret_cast<uintptr_t>(b_scales) & 3))
        return fail(MXQ_ERR_ARGUMENT, "%s: codes must be 16-byte and scales 4-byte aligned", who);
    GemmArgs g;
    g.a = reinterpret_cast<const unsigned char*>(a_codes);
    g.sa = reinterpret_cast<const unsigned char*>(a_scales);
    g.b = reinterpret_cast<const unsigned char*>(b_codes);
    g.sb = reinterpret_cast<const unsigned char*>(b_scales);
    g.c = c;
    g.bias = bias;
    g.q_nan_from = 0u;
    if (epilogue_quant) {                               // bfloat16, nearest: only the NaN threshold is needed
        ElemParams q;
        int rc = make_elem_params(MXQ_DTYPE_BF16, 9, 8, 3.3895313892515355e38f, MXQ_ROUND_NEAREST, 0, 1, 0, &q, who);
        if (rc) return rc;
        g.q_nan_from = q.fmt.nan_from;
    }
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.kbytes = (int)(nib ? K / 2 : K);
    g.batch_a = M * g.kbytes; g.batch_sa = M * (K / 32);
    g.batch_b = N * g.kbytes; g.batch_sb = N * (K / 32);
    g.batch_c = M * N;
    hipStream_t s = (hipStream_t)hip_stream;
    int rc;
    if (nib) rc = launch_gemm<4, 4>(c_dtype, batch, g, s);
    else if (!a_kind && !b_kind) rc = launch_gemm<0, 0>(c_dtype, batch, g, s);
    else if (a_kind && !b_kind) rc = launch_gemm<1, 0>(c_dtype, batch, g, s);
    else if (!a_kind && b_kind) rc = launch_gemm<0, 1>(c_dtype, batch, g, s);
    else rc = launch_gemm<1, 1>(c_dtype, batch, g, s);
    if (rc) return rc;
    return check_launch(who);
}

int mxq_probe_mfma_rate(int64_t workgroups, int iters, int code_kind, void* sink, void* hip_stream) {
    const char* who = "mxq_probe_mfma_rate";
    if (workgroups <= 0 || workgroups > 0x7FFFFFFF || iters <= 0 || !sink ||
        (code_kind != MXQ_CODES_E4M3 && code_kind != MXQ_CODES_E2M1))
        return fail(MXQ_ERR_ARGUMENT, "%s: bad argument", who);
    if (code_kind == MXQ_CODES_E2M1)
        mfma_rate_probe_kernel<4><<<(unsigned)workgroups, kThreads, 0, (hipStream_t)hip_stream>>>(
            iters, reinterpret_cast<float*>(sink));
    else
        mfma_rate_probe_kernel<0><<<(unsigned)workgroups, kThreads, 0, (hipStream_t)hip_stream>>>(
            iters, reinterpret_cast<float*>(sink));
    return check_launch(who);
}

int mxq_reduce_sum_inner(const float* in, float* out, int64_t rows, int64_t inner, void* hip_stream) {
    return reduce_inner<SumOp>(in, out, rows, inner, hip_stream, "mxq_reduce_sum_inner");
}
int mxq_reduce_max_inner(const float* in, float* out, int64_t rows, int64_t inner, void* hip_stream) {
    return reduce_inner<MaxOp>(in, out, rows, inner, hip_stream, "mxq_reduce_max_inner");
}

int64_t mxq_reduce_outer_workspace_bytes(int64_t outer, int64_t inner) {
    if (outer <= 0 || inner <= 0) return 0;
    const int64_t s = outer_splits(outer, inner);
    return s == 1 ? 0 : s * inner * (int64_t)sizeof(float);
}
int mxq_reduce_sum_outer(const float* in, float* out, void* workspace, int64_t outer, int64_t inner,
                         void* hip_stream) {
    return reduce_outer<SumOp>(in, out, workspace, outer, inner, hip_stream, "mxq_reduce_sum_outer");
}
int mxq_reduce_max_outer(const float* in, float* out, void* workspace, int64_t outer, int64_t inner,
                         void* hip_stream) {
    return reduce_outer<MaxOp>(in, out, workspace, outer, inner, hip_stream, "mxq_reduce_max_outer");
}

}  // extern "C"
#pragma GCC visibility pop
