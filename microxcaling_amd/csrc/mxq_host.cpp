// libmxq_host.so: the same scalar arithmetic as the GPU kernels (mxq_core.h), compiled for the
// host.  It serves the two CPU entry points of the reference's extension
// (quantize_mx_func_cpp, quantize_elemwise_func_cpp -- mx/cpp/funcs.cpp:23-149) for CPU tensors,
// and lets the kernel arithmetic be checked exhaustively without a GPU.  GPU tensors never come
// here: the GPU entry points live in libmxq_gfx950.so and there is no fallback between the two.
// The loops are compiled around the element functions (one instantiation per dtype, rounding and form,
// chosen once per call) and large calls run on several threads; the reference's CPU entry points are
// single loops on one thread.
#include <stdint.h>
#include <string.h>

#include <stdlib.h>

#include <algorithm>
#include <thread>
#include <vector>

#include "mxq.h"
#include "mxq_params.h"

namespace {

using namespace mxq_detail;

const unsigned char kZone[4][MXQ_ZONE_PAD] = {{MXQ_ZONE_ROW_F32}, {MXQ_ZONE_ROW_BF16}, {0}, {MXQ_ZONE_ROW_F16}};

// ---- element access by tensor dtype ------------------------------------------------------------
template <int DTYPE> struct Io;
template <> struct Io<MXQ_DTYPE_F32> {
    static float load(const void* p, int64_t i) { return reinterpret_cast<const float*>(p)[i]; }
    static void store(void* p, int64_t i, float v) { reinterpret_cast<float*>(p)[i] = v; }
};
template <> struct Io<MXQ_DTYPE_BF16> {
    static float load(const void* p, int64_t i) { return mxq_float((uint32_t) reinterpret_cast<const uint16_t*>(p)[i] << 16); }
    static void store(void* p, int64_t i, float v) {
        reinterpret_cast<uint16_t*>(p)[i] = (uint16_t)(mxq_bits(v) >> 16);       // already bf16-exact
    }
};
template <> struct Io<MXQ_DTYPE_F16> {
    static float load(const void* p, int64_t i) {
        return (float)__builtin_bit_cast(_Float16, reinterpret_cast<const uint16_t*>(p)[i]);
    }
    static void store(void* p, int64_t i, float v) {
        reinterpret_cast<uint16_t*>(p)[i] = __builtin_bit_cast(uint16_t, (_Float16)v);
    }
};

// ---- the element functions as types, so that the loops below are compiled around them --------------
template <int RMODE, int DT, bool ZE, bool LEAN> struct MxElem {
    static float call(float x, const MxqScale& sc, const MxqFmt& f, const unsigned char* zone, int zs, float noise) {
        return mxq_quant_mx_elem<RMODE, DT, ZE, LEAN>(x, sc, f, zone, zs, noise);
    }
};
template <int RMODE, int DT, bool ZE, bool LEAN> struct PlainElem {
    static float call(float x, const MxqFmt& f, bool saturate, bool denorm, const unsigned char* zone, int zs, float noise) {
        return mxq_quant_elemwise<RMODE, DT, ZE, LEAN>(x, f, saturate, denorm, zone, zs, noise);
    }
};

// body(element function type, Io type), chosen once per call.  lean = false selects the op-by-op form,
// which always consults the zone table.  An fp16 tensor in exact-exponent mode is computed as fp32.
template <template <int, int, bool, bool> class E, int DT, bool LEAN, class IO, class Body>
void by_round(int rmode, bool ze, const Body& body) {
    if (rmode == MXQ_ROUND_FLOOR) {
        if (ze) body(E<MXQ_FLOOR, DT, true, LEAN>{}, IO{});
        else body(E<MXQ_FLOOR, DT, false, LEAN>{}, IO{});
    } else if (rmode == MXQ_ROUND_NEAREST) {
        if (ze) body(E<MXQ_NEAREST, DT, true, LEAN>{}, IO{});
        else body(E<MXQ_NEAREST, DT, false, LEAN>{}, IO{});
    } else {
        if (ze) body(E<MXQ_EVEN, DT, true, LEAN>{}, IO{});
        else body(E<MXQ_EVEN, DT, false, LEAN>{}, IO{});
    }
}
template <template <int, int, bool, bool> class E, class Body>
void dispatch(int dtype, int flags, int rmode, bool ze, bool lean, const Body& body) {
    if (f16_ops(dtype, flags)) by_round<E, MXQ_F16OPS, false, Io<MXQ_DTYPE_F16>>(rmode, true, body);
    else if (dtype == MXQ_DTYPE_BF16 && lean) by_round<E, MXQ_BF16, true, Io<MXQ_DTYPE_BF16>>(rmode, ze, body);
    else if (dtype == MXQ_DTYPE_BF16) by_round<E, MXQ_BF16, false, Io<MXQ_DTYPE_BF16>>(rmode, true, body);
    else if (dtype == MXQ_DTYPE_F16 && lean) by_round<E, MXQ_F32, true, Io<MXQ_DTYPE_F16>>(rmode, ze, body);
    else if (dtype == MXQ_DTYPE_F16) by_round<E, MXQ_F32, false, Io<MXQ_DTYPE_F16>>(rmode, true, body);
    else if (lean) by_round<E, MXQ_F32, true, Io<MXQ_DTYPE_F32>>(rmode, ze, body);
    else by_round<E, MXQ_F32, false, Io<MXQ_DTYPE_F32>>(rmode, true, body);
}
template <template <int, int, bool, bool> class E, class Body>
void dispatch_dither(int dtype, int flags, const Body& body) {
    if (f16_ops(dtype, flags)) body(E<MXQ_DITHER, MXQ_F16OPS, true, false>{}, Io<MXQ_DTYPE_F16>{});
    else if (dtype == MXQ_DTYPE_BF16) body(E<MXQ_DITHER, MXQ_BF16, true, false>{}, Io<MXQ_DTYPE_BF16>{});
    else if (dtype == MXQ_DTYPE_F16) body(E<MXQ_DITHER, MXQ_F32, true, false>{}, Io<MXQ_DTYPE_F16>{});
    else body(E<MXQ_DITHER, MXQ_F32, true, false>{}, Io<MXQ_DTYPE_F32>{});
}

MxqScale block_scale(int dtype, int flags, uint32_t um, const MxParams& p, const unsigned char* zone) {
    if (f16_ops(dtype, flags)) return mxq_block_scale_f16ops(um, p.emax, p.scale_emax, zone);
    return mxq_block_scale(um, p.emax, p.scale_emax, p.flush != 0, zone, p.zshift);
}

// ---- threads -------------------------------------------------------------------------------------
// body(begin, end) over the n independent work items of a call (blocks, tiles, chunks of elements), on up
// to 16 threads -- fewer when the call is small: a thread is started per 64 K elements of work.  Every item
// is computed by exactly one thread with the same arithmetic, so the result does not depend on the number of
// threads.  MXQ_HOST_THREADS in the environment, read at the first large call, sets the upper limit (1:
// everything on the calling thread).
int64_t thread_limit() {                                  // read once per process
    static const int64_t limit = [] {
        int64_t n = (int64_t)std::thread::hardware_concurrency();
        if (n > 16) n = 16;
        if (const char* env = getenv("MXQ_HOST_THREADS")) {
            const long v = strtol(env, nullptr, 10);
            if (v >= 1) n = v < 64 ? v : 64;
        }
        return n < 1 ? (int64_t)1 : n;
    }();
    return limit;
}
template <class Body>
void parallel_for(int64_t n, int64_t elements_per_item, const Body& body) {
    const int64_t per_item = elements_per_item < 1 ? 1 : elements_per_item;
    int64_t threads = n;
    if (n > 0 && per_item <= INT64_MAX / n) threads = std::min(threads, n * per_item / 65536);
    if (threads > 1) threads = std::min(threads, thread_limit());
    if (threads <= 1) {
        body((int64_t)0, n);
        return;
    }
    const int64_t per = ceil_div(n, threads);
    std::vector<std::thread> pool;
    pool.reserve((size_t)threads);
    for (int64_t t = 1; t < threads; ++t) {
        const int64_t b = t * per, e = std::min(n, b + per);
        if (b >= e) break;
        try {
            pool.emplace_back([&body, b, e] { body(b, e); });
        } catch (...) {                      // no more threads to be had: this share on the calling thread
            body(b, e);
        }
    }
    body((int64_t)0, std::min(n, per));
    for (std::thread& th : pool) th.join();
}

// ---- the loops ---------------------------------------------------------------------------------------
// tensor (pre, axis, post); one exponent per `tile` consecutive positions of the middle axis and (i, j)
template <class E, class IO, bool DITHER>
void run_by_tile(const void* in, const void* noise, void* out, int dtype, int flags, int64_t pre, int64_t axis_size,
                 int64_t post, int64_t tile, const MxParams& p, const unsigned char* zone) {
    const int64_t ntile = ceil_div(axis_size, tile);
    if (post == 1) {                                      // blocks are contiguous
        parallel_for(pre * ntile, tile, [&](int64_t begin, int64_t end) {
            for (int64_t w = begin; w < end; ++w) {
                const int64_t k0 = (w % ntile) * tile, k1 = std::min(k0 + tile, axis_size);
                const int64_t base = (w / ntile) * axis_size;
                uint32_t um = 0;
                for (int64_t k = k0; k < k1; ++k) um = std::max(um, mxq_bits(IO::load(in, base + k)) & 0x7FFFFFFFu);
                const MxqScale sc = block_scale(dtype, flags, um, p, zone);
                for (int64_t k = k0; k < k1; ++k)
                    IO::store(out, base + k, E::call(IO::load(in, base + k), sc, p.fmt, zone, p.zshift,
                                                     DITHER ? IO::load(noise, base + k) : 0.0f));
            }
        });
        return;
    }
    // blocks run down the rows of a (tile, post) panel: walk the panel row by row, one maximum per column
    parallel_for(pre * ntile, tile * post, [&](int64_t begin, int64_t end) {
        std::vector<uint32_t> um((size_t)post);
        std::vector<MxqScale> sc((size_t)post);
        for (int64_t w = begin; w < end; ++w) {
            const int64_t k0 = (w % ntile) * tile, k1 = std::min(k0 + tile, axis_size);
            const int64_t base = (w / ntile) * axis_size;
            std::fill(um.begin(), um.end(), 0u);
            for (int64_t k = k0; k < k1; ++k) {
                const int64_t row = (base + k) * post;
                for (int64_t j = 0; j < post; ++j) um[j] = std::max(um[j], mxq_bits(IO::load(in, row + j)) & 0x7FFFFFFFu);
            }
            for (int64_t j = 0; j < post; ++j) sc[j] = block_scale(dtype, flags, um[j], p, zone);
            for (int64_t k = k0; k < k1; ++k) {
                const int64_t row = (base + k) * post;
                for (int64_t j = 0; j < post; ++j)
                    IO::store(out, row + j, E::call(IO::load(in, row + j), sc[j], p.fmt, zone, p.zshift,
                                                    DITHER ? IO::load(noise, row + j) : 0.0f));
            }
        }
    });
}

template <class E, class IO>
void run_given_max(const void* in, void* out, const void* max_values, int dtype, int flags, int64_t pre,
                   int64_t axis_size, int64_t post, const MxParams& p, const unsigned char* zone) {
    parallel_for(pre, axis_size * post, [&](int64_t begin, int64_t end) {
        std::vector<MxqScale> sc((size_t)post);
        for (int64_t i = begin; i < end; ++i) {
            for (int64_t j = 0; j < post; ++j)
                sc[j] = block_scale(dtype, flags, mxq_bits(IO::load(max_values, i * post + j)) & 0x7FFFFFFFu, p, zone);
            for (int64_t k = 0; k < axis_size; ++k) {
                const int64_t row = (i * axis_size + k) * post;
                for (int64_t j = 0; j < post; ++j)
                    IO::store(out, row + j, E::call(IO::load(in, row + j), sc[j], p.fmt, zone, p.zshift, 0.0f));
            }
        }
    });
}

template <class E, class IO>
void run_axes(const void* in, void* out, int dtype, int flags, const MxqAxes& a, const MxParams& p,
              const unsigned char* zone) {
    const int64_t n_tiles = mxq_axes_tiles(a);
    parallel_for(n_tiles, a.t[0] * a.t[1] * a.t[2], [&](int64_t begin, int64_t end) {
        for (int64_t tile = begin; tile < end; ++tile) {
            int64_t base, len[3], st[3];
            mxq_axes_tile(a, tile, &base, len, st);
            uint32_t um = 0;
            for (int64_t i = 0; i < len[0]; ++i)
                for (int64_t j = 0; j < len[1]; ++j)
                    for (int64_t k = 0; k < len[2]; ++k)
                        um = std::max(um, mxq_bits(IO::load(in, base + i * st[0] + j * st[1] + k * st[2])) & 0x7FFFFFFFu);
            const MxqScale sc = block_scale(dtype, flags, um, p, zone);
            for (int64_t i = 0; i < len[0]; ++i)
                for (int64_t j = 0; j < len[1]; ++j)
                    for (int64_t k = 0; k < len[2]; ++k) {
                        const int64_t idx = base + i * st[0] + j * st[1] + k * st[2];
                        IO::store(out, idx, E::call(IO::load(in, idx), sc, p.fmt, zone, p.zshift, 0.0f));
                    }
        }
    });
}

constexpr int64_t kChunk = 4096;                          // elements per work item of the elementwise loops
template <class E, class IO, bool DITHER>
void run_elemwise(const void* in, const void* noise, void* out, int64_t n, const ElemParams& p, const unsigned char* zone) {
    parallel_for(ceil_div(n, kChunk), kChunk, [&](int64_t begin, int64_t end) {
        const int64_t last = std::min(n, end * kChunk);
        for (int64_t i = begin * kChunk; i < last; ++i)
            IO::store(out, i, E::call(IO::load(in, i), p.fmt, p.saturate != 0, p.allow_denorm != 0, zone, p.zshift,
                                      DITHER ? IO::load(noise, i) : 0.0f));
    });
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

const char* mxq_host_last_error(void) { return last_error().c_str(); }

#ifndef MXQ_BUILD_DIGEST
#define MXQ_BUILD_DIGEST "unknown"
#endif
const char* mxq_host_build_digest(void) { return MXQ_BUILD_DIGEST; }

int mxq_host_quantize_mx_by_tile(const void* in, void* out, int dtype, int64_t pre, int64_t axis_size,
                                 int64_t post, int scale_bits, int elem_ebits, int elem_mbits,
                                 float elem_max_norm, int64_t tile_size, int flush_fp32_subnorms,
                                 int rmode, int flags) {
    const char* who = "mxq_host_quantize_mx_by_tile";
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
    const int64_t tile = (tile_size <= 0 || tile_size > axis_size) ? axis_size : tile_size;
    const unsigned char* zone = kZone[p.zone_row];
    const bool lean = lean_ok(dtype, p.fmt, rmode, false) && !(flags & MXQ_HOST_FLAG_ROUND_EVERY_OP);
    dispatch<MxElem>(dtype, flags, rmode, ze, lean, [&](auto e, auto io) {
        run_by_tile<decltype(e), decltype(io), false>(in, nullptr, out, dtype, flags, pre, axis_size, post, tile, p, zone);
    });
    return MXQ_OK;
}

int mxq_host_quantize_mx_axes(const void* in, void* out, int dtype, int n_axes, const int64_t* extents,
                              int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                              int64_t tile_size, int flush_fp32_subnorms, int rmode, int flags) {
    const char* who = "mxq_host_quantize_mx_axes";
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
    const unsigned char* zone = kZone[p.zone_row];
    const bool lean = lean_ok(dtype, p.fmt, rmode, false) && !(flags & MXQ_HOST_FLAG_ROUND_EVERY_OP);
    dispatch<MxElem>(dtype, flags, rmode, ze, lean, [&](auto e, auto io) {
        run_axes<decltype(e), decltype(io)>(in, out, dtype, flags, a, p, zone);
    });
    return MXQ_OK;
}

// round='dither': floor(scaled value + noise), noise[i] in [0, 1) drawn by the caller in the tensor
// dtype, one per element (mx/elemwise_ops.py:57-59)
int mxq_host_quantize_mx_dither_by_tile(const void* in, const void* noise, void* out, int dtype, int64_t pre,
                                        int64_t axis_size, int64_t post, int scale_bits, int elem_ebits,
                                        int elem_mbits, float elem_max_norm, int64_t tile_size,
                                        int flush_fp32_subnorms, int flags) {
    const char* who = "mxq_host_quantize_mx_dither_by_tile";
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
    const unsigned char* zone = kZone[p.zone_row];
    dispatch_dither<MxElem>(dtype, flags, [&](auto e, auto io) {
        run_by_tile<decltype(e), decltype(io), true>(in, noise, out, dtype, flags, pre, axis_size, post, tile, p, zone);
    });
    return MXQ_OK;
}

int mxq_host_quantize_elemwise_dither(const void* in, const void* noise, void* out, int dtype, int64_t n,
                                      int bits, int exp_bits, float max_norm, int saturate_normals,
                                      int allow_denorm, int flags) {
    const char* who = "mxq_host_quantize_elemwise_dither";
    ElemParams p;
    int rc = make_elem_params(dtype, bits, exp_bits, max_norm, MXQ_ROUND_NEAREST, saturate_normals, allow_denorm,
                              flags, &p, who);
    if (rc) return rc;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!in || !out || !noise) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    const unsigned char* zone = kZone[p.zone_row];
    dispatch_dither<PlainElem>(dtype, flags, [&](auto e, auto io) {
        run_elemwise<decltype(e), decltype(io), true>(in, noise, out, n, p, zone);
    });
    return MXQ_OK;
}

int mxq_host_quantize_mx_given_max(const void* in, void* out, const void* max_values, int dtype,
                                   int64_t pre, int64_t axis_size, int64_t post, int scale_bits,
                                   int elem_ebits, int elem_mbits, float elem_max_norm,
                                   int flush_fp32_subnorms, int rmode, int flags) {
    const char* who = "mxq_host_quantize_mx_given_max";
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
    const unsigned char* zone = kZone[p.zone_row];
    const bool lean = lean_ok(dtype, p.fmt, rmode, false) && !(flags & MXQ_HOST_FLAG_ROUND_EVERY_OP);
    dispatch<MxElem>(dtype, flags, rmode, ze, lean, [&](auto e, auto io) {
        run_given_max<decltype(e), decltype(io)>(in, out, max_values, dtype, flags, pre, axis_size, post, p, zone);
    });
    return MXQ_OK;
}

int mxq_host_quantize_elemwise(const void* in, void* out, int dtype, int64_t n, int bits, int exp_bits,
                               float max_norm, int rmode, int saturate_normals, int allow_denorm,
                               int flags) {
    const char* who = "mxq_host_quantize_elemwise";
    ElemParams p;
    int rc = make_elem_params(dtype, bits, exp_bits, max_norm, rmode, saturate_normals, allow_denorm,
                              flags, &p, who);
    if (rc) return rc;
    if (n < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    if (n == 0) return MXQ_OK;
    if (!in || !out) return fail(MXQ_ERR_ARGUMENT, "%s: null pointer", who);
    if (flags & MXQ_HOST_FLAG_CLOSED_FORM) {
        if (!(dtype == MXQ_DTYPE_BF16 && bits == 9 && exp_bits == 8 && rmode == MXQ_ROUND_NEAREST &&
              allow_denorm && !saturate_normals && p.fmt.max_bits == 0x7F7F0000u))
            return fail(MXQ_ERR_ARGUMENT, "%s: no closed form for this case", who);
        const bool nonneg = (flags & MXQ_HOST_FLAG_CLOSED_FORM_NONNEG) != 0;
        typedef Io<MXQ_DTYPE_BF16> IO;
        for (int64_t i = 0; i < n; ++i) {
            const float x = IO::load(in, i);
            IO::store(out, i, nonneg ? mxq_quant_bf16_to_bfloat16_nearest_nonneg(x)
                                     : mxq_quant_bf16_to_bfloat16_nearest(x, p.fmt.nan_from));
        }
        return MXQ_OK;
    }
    const unsigned char* zone = kZone[p.zone_row];
    const bool lean = lean_ok(dtype, p.fmt, rmode, true) && !(flags & MXQ_HOST_FLAG_ROUND_EVERY_OP);
    dispatch<PlainElem>(dtype, flags, rmode, elem_zone_matters(dtype, flags, p.fmt, rmode), lean, [&](auto e, auto io) {
        run_elemwise<decltype(e), decltype(io), false>(in, nullptr, out, n, p, zone);
    });
    return MXQ_OK;
}

}  // extern "C"
#pragma GCC visibility pop
