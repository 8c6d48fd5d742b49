// C ABI of libmxq_gfx950.so, continued: packed MX tensors and the scaled-MFMA GEMM.
#include <mutex>

#include "mxq_capi_common.h"
#include "mxq_gemm.h"

namespace {

// max_code != 0: the element format is the format of the codes, which then come straight from the
// rounded significands (mx_code_of); the round-up-zone variants always take the generic way
template <int DT, int RMODE, bool ZE, bool LEAN>
struct LaunchPack {
    template <int KIND>
    static void one(int grid, const u32x4* in, void* codes, unsigned char* sc, int64_t n_vec, MxParams p,
                    uint32_t max_code, hipStream_t s) {
        if constexpr (!ZE) {
            if (max_code != 0u) {
                mx_pack_kernel<DT, RMODE, ZE, KIND, 4, true><<<grid, kThreads, 0, s>>>(in, codes, sc, n_vec, p, max_code);
                return;
            }
        }
        mx_pack_kernel<DT, RMODE, ZE, KIND, 4, false><<<grid, kThreads, 0, s>>>(in, codes, sc, n_vec, p, 0u);
    }
    static void run(const void* in, void* codes, void* scales, int64_t n_vec, int kind, uint32_t max_code,
                    MxParams p, hipStream_t s) {
        const int grid = grid_for(ceil_div(n_vec, (int64_t)kThreads * 4));
        const u32x4* i4 = reinterpret_cast<const u32x4*>(in);
        unsigned char* sc = reinterpret_cast<unsigned char*>(scales);
        if (kind == 1) one<1>(grid, i4, codes, sc, n_vec, p, max_code, s);
        else if (kind == 2) one<2>(grid, i4, codes, sc, n_vec, p, max_code, s);
        else if (kind == 3) one<3>(grid, i4, codes, sc, n_vec, p, max_code, s);
        else if (kind == 4) one<4>(grid, i4, codes, sc, n_vec, p, max_code, s);
        else one<0>(grid, i4, codes, sc, n_vec, p, max_code, s);
    }
};

template <int DT, int RMODE, bool ZE, bool LEAN>
struct LaunchPackT {
    template <int KIND>
    static void one(unsigned grid, const u32x2* in, unsigned char* c, unsigned char* sc, int64_t n_cgroups,
                    int64_t n_tiles, int64_t pv, MxParams p, uint32_t max_code, hipStream_t s) {
        if constexpr (!ZE) {
            if (max_code != 0u) {
                mx_pack_t_kernel<DT, RMODE, ZE, KIND, true><<<grid, kThreads, 0, s>>>(in, c, sc, n_cgroups, n_tiles, pv, p, max_code);
                return;
            }
        }
        mx_pack_t_kernel<DT, RMODE, ZE, KIND, false><<<grid, kThreads, 0, s>>>(in, c, sc, n_cgroups, n_tiles, pv, p, 0u);
    }
    static void run(const void* in, void* codes, void* scales, int64_t n_blocks, int64_t n_tiles,
                    int64_t pv, int kind, uint32_t max_code, MxParams p, hipStream_t s) {
        const unsigned grid = (unsigned)n_blocks;
        const int64_t n_cgroups = ceil_div(pv, 64);
        const u32x2* i2 = reinterpret_cast<const u32x2*>(in);
        unsigned char* c = reinterpret_cast<unsigned char*>(codes);
        unsigned char* sc = reinterpret_cast<unsigned char*>(scales);
        if (kind == 1) one<1>(grid, i2, c, sc, n_cgroups, n_tiles, pv, p, max_code, s);
        else if (kind == 2) one<2>(grid, i2, c, sc, n_cgroups, n_tiles, pv, p, max_code, s);
        else if (kind == 3) one<3>(grid, i2, c, sc, n_cgroups, n_tiles, pv, p, max_code, s);
        else if (kind == 4) one<4>(grid, i2, c, sc, n_cgroups, n_tiles, pv, p, max_code, s);
        else one<0>(grid, i2, c, sc, n_cgroups, n_tiles, pv, p, max_code, s);
    }
};

// max_code for the direct form, or 0: the element format must be the one the code kind stores
uint32_t direct_max_code(int kind, int ebits, int mbits, const MxParams& p) {
    const bool same = (kind == MXQ_CODES_E4M3 && ebits == 4 && mbits == 5) ||
                      (kind == MXQ_CODES_E5M2 && ebits == 5 && mbits == 4) ||
                      (kind == MXQ_CODES_E2M3 && ebits == 2 && mbits == 5) ||
                      (kind == MXQ_CODES_E3M2 && ebits == 3 && mbits == 4) ||
                      (kind == MXQ_CODES_E2M1 && ebits == 2 && mbits == 3);
    if (!same) return 0u;
    const uint32_t mc = mxq_max_code(p.fmt);
    const uint32_t top = (1u << (kind == MXQ_CODES_E2M1 ? 3 : kind >= MXQ_CODES_E2M3 ? 5 : 7)) - 1u;
    // e4m3 keeps its last code for NaN, e5m2 its last exponent for Inf / NaN: a max_norm beyond the
    // largest finite code means a non-standard format
    const uint32_t finite = kind == MXQ_CODES_E4M3 ? 0x7Eu : kind == MXQ_CODES_E5M2 ? 0x7Bu : top;
    return mc <= finite ? mc : 0u;
}

// The persistent 256 x 256 tile kernel serves products with enough tiles to occupy half the CUs;
// below that the small tiles, with K split, are two to five times faster (512 x 4096 x 8192: 329 ->
// 745 TFLOP/s).
constexpr int64_t kMinLargeTiles = 128;
bool large_tiles(int64_t batch, int64_t M, int64_t N, int64_t K) {
    const int64_t total = ceil_div(M, G2_BM) * ceil_div(N, G2_BN) * batch;
    return M >= 512 && N >= 512 && K >= 512 && total >= kMinLargeTiles && total < ((int64_t)1 << 30);
}

// The small-tile kernel on few tiles leaves most CUs idle (a decode-shaped product, M <= 128, has
// N / 128 of them): split the K steps of every tile over several workgroups until about two per CU
// are in flight, each with at least two steps.  1 = no split.
int gemm_k_splits(int64_t batch, int64_t M, int64_t N, int64_t K, bool nibbles) {
    if (large_tiles(batch, M, N, K)) return 1;
    const int64_t tiles = ceil_div(M, GEMM_BM) * ceil_div(N, GEMM_BN) * batch;
    const int64_t nk = K / (nibbles ? 2 * GEMM_BK : GEMM_BK);
    if (tiles >= 256 || nk < 4) return 1;
    int64_t splits = ceil_div(512, tiles);
    if (splits > nk / 2) splits = nk / 2;
    if (splits > 64) splits = 64;
    const int64_t per = ceil_div(nk, splits);
    return (int)ceil_div(nk, per);                                        // no empty split
}

template <int CB, int BL, int ODT>
int launch_gemm_dt(int64_t batch, const GemmArgs& g, void* workspace, int64_t workspace_bytes, hipStream_t s) {
    // large problems: persistent 256 x 256 tile kernel (152 KB of dynamic LDS, one workgroup per CU);
    // it fetches 16 scale bytes (512 K) per row at a time, so a row must have at least that many
    const int64_t tiles_m = ceil_div(g.M, G2_BM), tiles_n = ceil_div(g.N, G2_BN);
    const int64_t total = tiles_m * tiles_n * batch;
    if (large_tiles(batch, g.M, g.N, g.K) && (int64_t)256 * g.kbytes < ((int64_t)1 << 31)) {
        // raising the dynamic-LDS limit is per kernel and per device: done once for each (this template
        // instance, device), under a lock, and remembered with that device's CU count
        static std::mutex config_mutex;
        static int cus_of_device[kMaxDevices] = {};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
            return fail(MXQ_ERR_LAUNCH, "mxq_gemm_mx_nt: no usable current device (%s)", hipGetErrorString(e));
        int cus;
        {
            std::lock_guard<std::mutex> lock(config_mutex);
            if (cus_of_device[dev] == 0) {
                int n = 0;
                e = hipFuncSetAttribute(reinterpret_cast<const void*>(&mx_gemm_nt_kernel_256p<CB, BL, ODT>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, G3_LDS_BYTES);
                if (e == hipSuccess) e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
                if (e != hipSuccess || n <= 0)
                    return fail(MXQ_ERR_LAUNCH, "mxq_gemm_mx_nt: cannot configure the tile kernel (%d bytes of LDS): %s",
                                G3_LDS_BYTES, hipGetErrorString(e));
                n -= n % 8;                           // a workgroup must stay on its XCD from tile to tile
                cus_of_device[dev] = n < 8 ? 8 : n;
            }
            cus = cus_of_device[dev];
        }
        const unsigned grid = (unsigned)(total < cus ? total : cus);
        mx_gemm_nt_kernel_256p<CB, BL, ODT><<<grid, 512, G3_LDS_BYTES, s>>>(g, (int)tiles_m, (int)tiles_n, (int)total);
    } else {
        const int splits = gemm_k_splits(batch, g.M, g.N, g.K, CB == 4);
        const int64_t need = (int64_t)splits * batch * g.M * g.N * (int64_t)sizeof(float);
        const unsigned tiles = (unsigned)(ceil_div(g.N, GEMM_BN) * ceil_div(g.M, GEMM_BM));
        if (splits > 1 && workspace != nullptr && workspace_bytes >= need && aligned16(workspace)) {
            GemmArgs part = g;                        // fp32 partial tiles, no epilogue
            part.c = workspace;
            part.bias = nullptr;
            part.q_nan_from = 0u;
            part.k_splits = splits;
            mx_gemm_nt_kernel<CB, BL, MXQ_F32><<<dim3(tiles, (unsigned)batch, (unsigned)splits), kThreads, 0, s>>>(part);
            const int64_t rows = batch * g.M, items = rows * ceil_div(g.N, 4);
            gemm_split_reduce_kernel<ODT><<<(unsigned)ceil_div(items, kThreads), kThreads, 0, s>>>(
                reinterpret_cast<const float*>(workspace), g.c, g.bias, g.q_nan_from, splits, rows, g.N);
        } else {
            if (g.kbytes == GEMM_BK)
                mx_gemm_nt_kernel<CB, BL, ODT, true><<<dim3(tiles, (unsigned)batch), kThreads, 0, s>>>(g);
            else
                mx_gemm_nt_kernel<CB, BL, ODT><<<dim3(tiles, (unsigned)batch), kThreads, 0, s>>>(g);
        }
    }
    return MXQ_OK;
}

template <int CB, int BL>
int launch_gemm(int c_dtype, int64_t batch, const GemmArgs& g, void* ws, int64_t ws_bytes, hipStream_t s) {
    if (c_dtype == MXQ_DTYPE_F32) return launch_gemm_dt<CB, BL, MXQ_F32>(batch, g, ws, ws_bytes, s);
    if (c_dtype == MXQ_DTYPE_BF16) return launch_gemm_dt<CB, BL, MXQ_BF16>(batch, g, ws, ws_bytes, s);
    return launch_gemm_dt<CB, BL, MXQ_F16>(batch, g, ws, ws_bytes, s);
}

// splits of the outer axis for the two-pass outer reduction
int code_kind(int ebits, int mbits, int flags, const char* who) {
    const bool fp4 = ebits == 2 && mbits == 3;
    if (flags & MXQ_FLAG_PACK_SIXBIT) {
        if (ebits == 2 && mbits == 5) return MXQ_CODES_E2M3;
        if (ebits == 3 && mbits == 4) return MXQ_CODES_E3M2;
        fail(MXQ_ERR_ARGUMENT, "%s: 6-bit codes exist for the e2m3 and e3m2 formats only", who);
        return -1;
    }
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

int mxq_pack_mx(const void* in, void* codes, void* scales, int dtype, int64_t rows, int64_t K,
                int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                int flush_fp32_subnorms, int rmode, int flags, void* hip_stream) {
    const char* who = "mxq_pack_mx";
    MxParams p;
    bool ze;
    if (f16_ops(dtype, flags))
        return fail(MXQ_ERR_ARGUMENT, "%s: fp16 tensors have a packed form under MXQ_FLAG_EXACT_EXPONENT only "
                    "(the op-by-op fp16 arithmetic of the default mode has no packing kernel)", who);
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
    if (flags & MXQ_FLAG_PRE_BFLOAT16) {
        if (dtype != MXQ_DTYPE_BF16)
            return fail(MXQ_ERR_ARGUMENT, "%s: MXQ_FLAG_PRE_BFLOAT16 is for bf16 tensors", who);
        ElemParams q;
        rc = make_elem_params(dtype, 9, 8, 3.3895313892515355e38f, MXQ_ROUND_NEAREST, 0, 1, flags, &q, who);
        if (rc) return rc;
        p.pre_nan_from = q.fmt.nan_from;
    }
    dispatch<LaunchPack>(dtype, rmode, ze, true, in, codes, scales, total / (16 / elem_size(dtype)), kind,
                         direct_max_code(kind, elem_ebits, elem_mbits, p), p, (hipStream_t)hip_stream);
    return check_launch(who);
}

int mxq_pack_mx_t(const void* in, void* codes, void* scales, int dtype, int64_t batch, int64_t R,
                  int64_t C, int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                  int flush_fp32_subnorms, int rmode, int flags, void* hip_stream) {
    const char* who = "mxq_pack_mx_t";
    MxParams p;
    bool ze;
    if (f16_ops(dtype, flags))
        return fail(MXQ_ERR_ARGUMENT, "%s: fp16 tensors have a packed form under MXQ_FLAG_EXACT_EXPONENT only "
                    "(the op-by-op fp16 arithmetic of the default mode has no packing kernel)", who);
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
    const int64_t n_tiles = R / 32, pv = C / vw;
    // a workgroup: PACKT_TILES blocks of 32 rows x 64 column strips of 8 bytes
    const int64_t n_blocks = batch * ceil_div(n_tiles, PACKT_TILES) * ceil_div(pv, 64);
    if (n_blocks > 0x7FFFFFFF) return fail(MXQ_ERR_ARGUMENT, "%s: tensor too large", who);
    dispatch<LaunchPackT>(dtype, rmode, ze, true, in, codes, scales, n_blocks, n_tiles, pv, kind,
                          direct_max_code(kind, elem_ebits, elem_mbits, p), p, (hipStream_t)hip_stream);
    return check_launch(who);
}

int mxq_unpack_mx(const void* codes, const void* scales, int code_kind, void* out, int dtype,
                  int64_t rows, int64_t K, void* hip_stream) {
    const char* who = "mxq_unpack_mx";
    if (dtype < 0 || dtype > 2) return fail(MXQ_ERR_ARGUMENT, "%s: unknown dtype code %d", who, dtype);
    if (code_kind < MXQ_CODES_E4M3 || code_kind > MXQ_CODES_E2M1)
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
    else if (code_kind == 2) mx_unpack_kernel<DT, 2><<<grid, kThreads, 0, s>>>(cd, sc, out, n); \
    else if (code_kind == 3) mx_unpack_kernel<DT, 3><<<grid, kThreads, 0, s>>>(cd, sc, out, n); \
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
                   void* workspace, int64_t workspace_bytes, void* hip_stream) {
    const char* who = "mxq_gemm_mx_nt";
    if (c_dtype < 0 || c_dtype > 2) return fail(MXQ_ERR_ARGUMENT, "%s: unknown dtype code %d", who, c_dtype);
    if (epilogue_quant != 0 && (epilogue_quant != 1 || c_dtype != MXQ_DTYPE_BF16))
        return fail(MXQ_ERR_ARGUMENT, "%s: epilogue_quant must be 0, or 1 with a bf16 output", who);
    if (batch < 0 || M < 0 || N < 0 || K < 0) return fail(MXQ_ERR_ARGUMENT, "%s: negative size", who);
    const bool nib = a_kind == MXQ_CODES_E2M1;
    auto sixbit = [](int kind) { return kind == MXQ_CODES_E2M3 || kind == MXQ_CODES_E3M2; };
    if (sixbit(a_kind) || sixbit(b_kind))
        return fail(MXQ_ERR_ARGUMENT, "%s: 6-bit codes are a storage form; the GEMM takes fp6 operands as "
                    "byte codes (mxq_pack_mx without MXQ_FLAG_PACK_SIXBIT)", who);
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
    g.k_splits = 1;
    g.batch_a = M * g.kbytes; g.batch_sa = M * (K / 32);
    g.batch_b = N * g.kbytes; g.batch_sb = N * (K / 32);
    g.batch_c = M * N;
    hipStream_t s = (hipStream_t)hip_stream;
    int rc;
    if (nib) rc = launch_gemm<4, 4>(c_dtype, batch, g, workspace, workspace_bytes, s);
    else if (!a_kind && !b_kind) rc = launch_gemm<0, 0>(c_dtype, batch, g, workspace, workspace_bytes, s);
    else if (a_kind && !b_kind) rc = launch_gemm<1, 0>(c_dtype, batch, g, workspace, workspace_bytes, s);
    else if (!a_kind && b_kind) rc = launch_gemm<0, 1>(c_dtype, batch, g, workspace, workspace_bytes, s);
    else rc = launch_gemm<1, 1>(c_dtype, batch, g, workspace, workspace_bytes, s);
    if (rc) return rc;
    return check_launch(who);
}

int64_t mxq_gemm_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int a_kind) {
    if (batch <= 0 || M <= 0 || N <= 0 || K <= 0) return 0;
    const bool nib = a_kind == MXQ_CODES_E2M1;
    if (K % (nib ? 2 * GEMM_BK : GEMM_BK) != 0) return 0;
    const int splits = gemm_k_splits(batch, M, N, K, nib);
    return splits == 1 ? 0 : (int64_t)splits * batch * M * N * (int64_t)sizeof(float);
}

int mxq_gemm_plan(int64_t batch, int64_t M, int64_t N, int64_t K, int a_kind) {
    if (batch <= 0 || M <= 0 || N <= 0 || K <= 0) return -1;
    const bool nib = a_kind == MXQ_CODES_E2M1;
    if (K % (nib ? 2 * GEMM_BK : GEMM_BK) != 0) return -1;
    const int64_t kbytes = nib ? K / 2 : K;
    if (large_tiles(batch, M, N, K) && (int64_t)256 * kbytes < ((int64_t)1 << 31)) return MXQ_GEMM_PLAN_LARGE_TILES;
    if (gemm_k_splits(batch, M, N, K, nib) > 1) return MXQ_GEMM_PLAN_SPLIT_K;
    return kbytes == GEMM_BK ? MXQ_GEMM_PLAN_ONE_STEP : MXQ_GEMM_PLAN_SMALL_TILES;
}

}  // extern "C"
#pragma GCC visibility pop
