// C ABI of libmxq_gfx950.so: argument checks, kernel selection and launch geometry.
// Declarations and the reference functions each entry point replaces are in include/mxq.h.
// This file: MX and elementwise quantization, reductions.  mxq_capi_gemm.hip: packed MX tensors and
// the GEMM.  mxq_capi_chain.hip: softmax, normalization and activation kernels.
#include <mutex>

#include "mxq_capi_common.h"

namespace {

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
struct LaunchAxes {
    static void run(const void* in, void* out, MxqAxes a, int64_t n_tiles, MxParams p, hipStream_t s) {
        // 32 x 32 tiles of the last two axes of an aligned tensor: the register-resident tile kernel,
        // the lanes of a tile sharing their maxima
        constexpr int VW8 = (DT == MXQ_F32) ? 2 : 4;
        if (a.s[2] == 1 && a.o[1] == 1 && a.o[2] == 1 && a.o[3] == 1 && a.t[0] == 32 && a.t[1] == 32 &&
            a.s[0] % 32 == 0 && a.s[1] % 32 == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 7) == 0) {
            const int64_t pv = a.s[1] / VW8, tiles_r = a.s[0] / 32;
            const int64_t items = a.o[0] * tiles_r * pv, blocks = ceil_div(items, kThreads);
            if (blocks <= 0x7FFFFFFF) {
                mx_strided_tile_kernel<DT, RMODE, ZE, LEAN, 32, true><<<(unsigned)blocks, kThreads, 0, s>>>(
                    reinterpret_cast<const u32x2*>(in), reinterpret_cast<u32x2*>(out), items, tiles_r, pv, p);
                return;
            }
        }
        const int64_t grid = n_tiles < 8 * kMaxBlocks ? n_tiles : 8 * kMaxBlocks;
        mx_axes_kernel<DT, RMODE, ZE, LEAN><<<(unsigned)grid, kThreads, 0, s>>>(in, out, a, n_tiles, p);
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
    if (vec) {
        // column groups of a row per block: as many as it takes to cover the row, up to 8 x 256
        const int64_t groups = ceil_div(inner / 4, (int64_t)kThreads);
        const int kg = groups >= 8 ? 8 : groups >= 4 ? 4 : groups >= 2 ? 2 : 1;
        dim3 grid((unsigned)ceil_div(groups, kg), (unsigned)splits);
        if (kg == 8) reduce_outer_kernel<OP, 4, 8><<<grid, kThreads, 0, s>>>(in, partial, outer, inner, rows_per_split);
        else if (kg == 4) reduce_outer_kernel<OP, 4, 4><<<grid, kThreads, 0, s>>>(in, partial, outer, inner, rows_per_split);
        else if (kg == 2) reduce_outer_kernel<OP, 4, 2><<<grid, kThreads, 0, s>>>(in, partial, outer, inner, rows_per_split);
        else reduce_outer_kernel<OP, 4, 1><<<grid, kThreads, 0, s>>>(in, partial, outer, inner, rows_per_split);
    } else {
        dim3 grid((unsigned)ceil_div(inner, kThreads), (unsigned)splits);
        reduce_outer_kernel<OP, 1, 1><<<grid, kThreads, 0, s>>>(in, partial, outer, inner, rows_per_split);
    }
    int rc = check_launch(who);
    if (rc || splits == 1) return rc;
    reduce_outer_final_kernel<OP><<<(unsigned)ceil_div(inner, 64), kThreads, 0, s>>>(partial, out, splits, inner);
    return check_launch(who);
}

// Partial results of mxq_reduce_outer_static.  In host code the array's name is only a handle: the
// address kernels can use comes from hipGetSymbolAddress, differs from GPU to GPU, and is looked up
// once per device (with that device current) on the entry point's first call there.
__attribute__((used)) static __device__ __align__(256) unsigned char scratch[MXQ_REDUCE_OUTER_STATIC_BYTES];
std::mutex scratch_mutex;
void* scratch_of_device[kMaxDevices] = {};

int scratch_on_current_device(void** ptr, const char* who) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(MXQ_ERR_LAUNCH, "%s: no usable current device (%s)", who, hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_of_device[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr)
            return fail(MXQ_ERR_LAUNCH, "%s: cannot locate the scratch array on device %d (%s)", who, dev,
                        hipGetErrorString(e));
        scratch_of_device[dev] = p;
    }
    *ptr = scratch_of_device[dev];
    return MXQ_OK;
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

const char* mxq_last_error(void) { return last_error().c_str(); }

int mxq_version(void) { return 100; }

#ifndef MXQ_BUILD_DIGEST
#define MXQ_BUILD_DIGEST "unknown"
#endif
const char* mxq_build_digest(void) { return MXQ_BUILD_DIGEST; }

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
            dispatch_any<LaunchLastAxis>(dtype, flags, rmode, ze, lean_ok(dtype, p.fmt, rmode, false), in, out, total / vec_elems, (int)lpt, p, s);
            return check_launch(who);
        }
    }
    dispatch_any<LaunchStrided>(dtype, flags, rmode, ze, lean_ok(dtype, p.fmt, rmode, false), in, out, pre, axis_size, post, tile, ptr_ok, p, s);
    return check_launch(who);
}

int mxq_quantize_mx_axes(const void* in, void* out, int dtype, int n_axes, const int64_t* extents,
                         int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                         int64_t tile_size, int flush_fp32_subnorms, int rmode, int flags,
                         void* hip_stream) {
    const char* who = "mxq_quantize_mx_axes";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, rmode, flags, &p, &ze, who);
    if (rc) return rc;
    MxqAxes a;
    int64_t total;
    rc = make_mx_axes(n_axes, extents, tile_size, &a, &total, who);
    if (rc) return rc;
    if (total == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    dispatch_any<LaunchAxes>(dtype, flags, rmode, ze, lean_ok(dtype, p.fmt, rmode, false), in, out, a, mxq_axes_tiles(a), p,
                         (hipStream_t)hip_stream);
    return check_launch(who);
}

int mxq_quantize_mx_dither_by_tile(const void* in, const void* noise, void* out, int dtype, int64_t pre,
                                   int64_t axis_size, int64_t post, int scale_bits, int elem_ebits,
                                   int elem_mbits, float elem_max_norm, int64_t tile_size,
                                   int flush_fp32_subnorms, int flags, void* hip_stream) {
    const char* who = "mxq_quantize_mx_dither_by_tile";
    MxParams p;
    bool ze;
    int rc = make_mx_params(dtype, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                            flush_fp32_subnorms, MXQ_ROUND_NEAREST, flags, &p, &ze, who);
    if (rc) return rc;
    if (pre < 0 || axis_size < 0 || post < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    int64_t total;
    if (mul_overflows(pre, axis_size, post, &total)) return fail(MXQ_ERR_ARGUMENT, "%s: size overflows int64", who);
    if (total == 0) return MXQ_OK;
    if (!in || !out || !noise) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    const int64_t tile = (tile_size <= 0 || tile_size > axis_size) ? axis_size : tile_size;
    const int64_t num_tiles = ceil_div(axis_size, tile);
    hipStream_t s = (hipStream_t)hip_stream;
    const int grid = grid_for(ceil_div(pre * num_tiles * post, kThreads));
    if (dtype == MXQ_DTYPE_F32)
        mx_dither_kernel<MXQ_F32><<<grid, kThreads, 0, s>>>(in, noise, out, pre, axis_size, post, tile, num_tiles, p);
    else if (dtype == MXQ_DTYPE_BF16)
        mx_dither_kernel<MXQ_BF16><<<grid, kThreads, 0, s>>>(in, noise, out, pre, axis_size, post, tile, num_tiles, p);
    else if (f16_ops(dtype, flags))
        mx_dither_kernel<MXQ_F16OPS><<<grid, kThreads, 0, s>>>(in, noise, out, pre, axis_size, post, tile, num_tiles, p);
    else
        mx_dither_kernel<MXQ_F16><<<grid, kThreads, 0, s>>>(in, noise, out, pre, axis_size, post, tile, num_tiles, p);
    return check_launch(who);
}

int mxq_quantize_elemwise_dither(const void* in, const void* noise, void* out, int dtype, int64_t n, int bits,
                                 int exp_bits, float max_norm, int saturate_normals, int allow_denorm,
                                 int flags, void* hip_stream) {
    const char* who = "mxq_quantize_elemwise_dither";
    ElemParams p;
    int rc = make_elem_params(dtype, bits, exp_bits, max_norm, MXQ_ROUND_NEAREST, saturate_normals, allow_denorm,
                              flags, &p, who);
    if (rc) return rc;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!in || !out || !noise) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    hipStream_t s = (hipStream_t)hip_stream;
    const int grid = grid_for(ceil_div(n, kThreads));
    if (dtype == MXQ_DTYPE_F32) elemwise_dither_kernel<MXQ_F32><<<grid, kThreads, 0, s>>>(in, noise, out, n, p);
    else if (dtype == MXQ_DTYPE_BF16) elemwise_dither_kernel<MXQ_BF16><<<grid, kThreads, 0, s>>>(in, noise, out, n, p);
    else if (f16_ops(dtype, flags)) elemwise_dither_kernel<MXQ_F16OPS><<<grid, kThreads, 0, s>>>(in, noise, out, n, p);
    else elemwise_dither_kernel<MXQ_F16><<<grid, kThreads, 0, s>>>(in, noise, out, n, p);
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
    dispatch_any<LaunchGivenMax>(dtype, flags, rmode, ze, lean_ok(dtype, p.fmt, rmode, false), in, out, max_values, total, axis_size, post, p,
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
    // bf16 tensor -> bfloat16, round-half-away, subnormals kept, overflow to Inf: the closed form
    if (dtype == MXQ_DTYPE_BF16 && bits == 9 && exp_bits == 8 && rmode == MXQ_ROUND_NEAREST && allow_denorm &&
        !saturate_normals && p.fmt.max_bits == 0x7F7F0000u &&
        !(flags & (MXQ_FLAG_EXACT_EXPONENT | MXQ_FLAG_GENERAL_FORM))) {
        const int grid = grid_for(ceil_div(ceil_div(n, 8), (int64_t)kThreads * kElemUnroll));
        elemwise_bf16_closed_kernel<kElemUnroll><<<grid, kThreads, 0, (hipStream_t)hip_stream>>>(in, out, n, p.fmt.nan_from);
        return check_launch(who);
    }
    dispatch_any<LaunchElemwise>(dtype, flags, rmode, elem_zone_matters(dtype, flags, p.fmt, rmode), lean_ok(dtype, p.fmt, rmode, true), in, out, n, p, (hipStream_t)hip_stream);
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

int mxq_reduce_outer_static(const float* in, float* out, int op, int64_t outer, int64_t inner,
                            void* hip_stream) {
    const char* who = "mxq_reduce_outer_static";
    if (op != 0 && op != 1) return fail(MXQ_ERR_ARGUMENT, "%s: op must be 0 (sum) or 1 (max)", who);
    if (outer < 0 || inner < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    const int64_t need = mxq_reduce_outer_workspace_bytes(outer, inner);
    if (need > (int64_t)MXQ_REDUCE_OUTER_STATIC_BYTES)
        return fail(MXQ_ERR_ARGUMENT, "%s: (%lld, %lld) needs %lld bytes of partial results, the built-in "
                    "scratch array holds %d; use mxq_reduce_%s_outer with a workspace", who, (long long)outer,
                    (long long)inner, (long long)need, (int)MXQ_REDUCE_OUTER_STATIC_BYTES, op ? "max" : "sum");
    void* ws = nullptr;
    if (need > 0) {
        const int rc = scratch_on_current_device(&ws, who);
        if (rc) return rc;
    }
    return op ? reduce_outer<MaxOp>(in, out, ws, outer, inner, hip_stream, who)
              : reduce_outer<SumOp>(in, out, ws, outer, inner, hip_stream, who);
}

}  // extern "C"
#pragma GCC visibility pop
