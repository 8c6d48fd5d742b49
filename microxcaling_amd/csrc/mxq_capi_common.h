// Shared by the translation units of libmxq_gfx950.so: launch checks, grid sizes and the dispatch
// over (tensor dtype, rounding mode, element zone, lean rounding).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxq.h"
#include "mxq_kernels.h"

namespace {

using namespace mxq_detail;

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MXQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MXQ_OK;
}

constexpr int kThreads = 256;
constexpr int64_t kMaxBlocks = 256 * 8;      // 256 CUs x 8 resident blocks of 256 lanes
constexpr int kMaxDevices = 64;               // per-device state is kept in tables of this size

int grid_for(int64_t work_items_per_block_iter_total) {
    int64_t g = work_items_per_block_iter_total;
    if (g < 1) g = 1;
    if (g > kMaxBlocks) g = kMaxBlocks;
    return (int)g;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

[[maybe_unused]] int elem_size(int dtype) { return dtype == MXQ_DTYPE_F32 ? 4 : 2; }

// ---- dispatch over (dtype, rounding mode, element zone, lean) ------------------------------------
// F is a functor template: F<DT, RMODE, ZONE_ELEM, LEAN>::run(args...).  The op-by-op form always
// consults the zone table, so it exists once per rounding mode (bf16 tensors with wide formats; any
// dtype for the two parameter corners of lean_ok).
template <template <int, int, bool, bool> class F, int DT, typename... A>
void dispatch_round(int rmode, bool zone_elem, bool lean, A... a) {
    if (!lean) {
        if (rmode == MXQ_ROUND_FLOOR) F<DT, MXQ_FLOOR, true, false>::run(a...);
        else if (rmode == MXQ_ROUND_NEAREST) F<DT, MXQ_NEAREST, true, false>::run(a...);
        else F<DT, MXQ_EVEN, true, false>::run(a...);
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

// The same, for the entry points that also serve fp16 tensors op by op in fp16 (f16_ops): that
// arithmetic exists in the op-by-op form only.
template <template <int, int, bool, bool> class F, typename... A>
void dispatch_any(int dtype, int flags, int rmode, bool zone_elem, bool lean, A... a) {
    if (f16_ops(dtype, flags)) {
        if (rmode == MXQ_ROUND_FLOOR) F<MXQ_F16OPS, MXQ_FLOOR, true, false>::run(a...);
        else if (rmode == MXQ_ROUND_NEAREST) F<MXQ_F16OPS, MXQ_NEAREST, true, false>::run(a...);
        else F<MXQ_F16OPS, MXQ_EVEN, true, false>::run(a...);
        return;
    }
    dispatch<F>(dtype, rmode, zone_elem, lean, a...);
}

constexpr int kLastAxisUnroll = 4;


}  // namespace
