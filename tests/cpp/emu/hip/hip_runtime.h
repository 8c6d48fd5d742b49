// A stand-in for <hip/hip_runtime.h> that lets HIP sources of this package be compiled for the host and
// executed there, for tests on machines without a GPU.  A kernel launch runs the workgroups one after
// another; the lanes of a workgroup (up to 512) are host threads, kept for the life of the process, that
// meet where the hardware's lanes exchange data or wait for each other: __syncthreads (all of them), and the
// collective instructions of a wave of 64 (DPP moves, shuffles, votes, permlane swaps, readfirstlane, the
// scaled matrix instructions).  A lane that has left the kernel counts as inactive: it no longer takes part
// in barriers, and an exchange that would read from it returns what the instruction returns for a disabled
// lane.  What is modelled is what the instructions compute, not when: a copy from memory into LDS lands at
// once (one of the orders the hardware allows), waits and scheduling hints do nothing, and the matrix
// instruction accumulates in double precision and rounds once (the hardware's own order of additions is
// not public; the tests that use it carry a tolerance).
#pragma once
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>

#include <atomic>
#include <barrier>
#include <condition_variable>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __constant__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static                    /* workgroups run one at a time */
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
typedef void* hipStream_t;
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
enum { hipFuncAttributeMaxDynamicSharedMemorySize = 8, hipDeviceAttributeMultiprocessorCount = 63 };
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "no error"; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void** p, const void* symbol) { *p = const_cast<void*>(symbol); return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, int, int) { return hipSuccess; }
// a small "device": few enough compute units that a persistent kernel gives every workgroup several tiles
inline hipError_t hipDeviceGetAttribute(int* value, int, int) { *value = 8; return hipSuccess; }

namespace emu {

constexpr int kMaxLanes = 512, kWave = 64, kMaxWaves = kMaxLanes / kWave;
constexpr size_t kDynamicLds = 160 * 1024;

struct Block {
    explicit Block(int lanes) : all(lanes) {
        for (int w = 0; w < kMaxWaves; ++w) wave[w] = std::make_unique<std::barrier<>>(kWave);
        for (auto& a : active) a.store(true);
    }
    std::barrier<> all;
    std::unique_ptr<std::barrier<>> wave[kMaxWaves];
    uint64_t slot[kMaxLanes];                // what a lane offers in an exchange
    const void* operand[kMaxLanes][2];       // ... and the operands of a matrix instruction
    int scale[kMaxLanes][2];
    std::atomic<bool> active[kMaxLanes];
};
inline Block*& block() { static Block* b = nullptr; return b; }
inline thread_local dim3 t_thread, t_block;
inline dim3 g_grid, g_blockdim;

// LDS of a launch with dynamic shared memory: mapped below 4 GB, so that the 32-bit LDS addresses the
// kernels compute from pointers (the value the hardware wants in m0) convert back to the same pointers
inline unsigned char* dynamic_lds() {
    static unsigned char* p = [] {
        void* m = mmap(nullptr, kDynamicLds, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_32BIT, -1, 0);
        if (m == MAP_FAILED) __builtin_trap();
        return static_cast<unsigned char*>(m);
    }();
    return p;
}
// a 32-bit LDS address back to a pointer: dynamic LDS as above; a static __shared__ array lies in this
// library's data, whose upper address bits are those of `anchor`
inline unsigned char* lds_pointer(uint32_t addr) {
    static unsigned char anchor;
    const uintptr_t low = reinterpret_cast<uintptr_t>(dynamic_lds());
    if (addr >= low && addr < low + kDynamicLds) return reinterpret_cast<unsigned char*>((uintptr_t)addr);
    return reinterpret_cast<unsigned char*>((reinterpret_cast<uintptr_t>(&anchor) & ~(uintptr_t)0xFFFFFFFFu) | addr);
}

// copies into LDS that have been issued and not yet carried out (see global_load_lds)
struct PendingCopy {
    unsigned char* dst;
    const unsigned char* src;
    int bytes;
};
inline std::vector<PendingCopy>& pending_copies() {
    static thread_local std::vector<PendingCopy> q;
    return q;
}
// threads that live as long as the process; a workgroup is one job for each of its lanes
class Lanes {
  public:
    static Lanes& get() {
        static Lanes* pool = new Lanes;      // never destroyed: its threads wait on it until the process ends
        return *pool;
    }
    void run(int lanes, const std::function<void(int)>& job) {
        std::unique_lock<std::mutex> lock(m_);
        job_ = &job;
        lanes_ = lanes;
        pending_ = lanes;
        ++generation_;
        start_.notify_all();
        done_.wait(lock, [&] { return pending_ == 0; });
        job_ = nullptr;
    }

  private:
    Lanes() {
        for (int t = 0; t < kMaxLanes; ++t) std::thread([this, t] { work(t); }).detach();
    }
    void work(int t) {
        uint64_t seen = 0;
        for (;;) {
            const std::function<void(int)>* job;
            {
                std::unique_lock<std::mutex> lock(m_);
                start_.wait(lock, [&] { return generation_ != seen; });
                seen = generation_;
                if (t >= lanes_) continue;                   // this launch has fewer lanes
                job = job_;
            }
            (*job)(t);
            std::lock_guard<std::mutex> lock(m_);
            if (--pending_ == 0) done_.notify_one();
        }
    }
    std::mutex m_;
    std::condition_variable start_, done_;
    const std::function<void(int)>* job_ = nullptr;
    uint64_t generation_ = 0;
    int pending_ = 0, lanes_ = 0;
};

// the workgroups of a launch one after another (dynamic_lds_bytes: as in <<<grid, block, bytes, stream>>>)
template <class Body>
void launch(dim3 grid, dim3 blockdim, size_t dynamic_lds_bytes, const Body& body) {
    static std::mutex one_launch_at_a_time;
    std::lock_guard<std::mutex> guard(one_launch_at_a_time);
    const int lanes = (int)blockdim.x;
    if (lanes < 1 || lanes > kMaxLanes || lanes % kWave != 0 || blockdim.y != 1 || blockdim.z != 1 ||
        dynamic_lds_bytes > kDynamicLds)
        __builtin_trap();
    g_grid = grid;
    g_blockdim = blockdim;
    for (unsigned bz = 0; bz < grid.z; ++bz)
        for (unsigned by = 0; by < grid.y; ++by)
            for (unsigned bx = 0; bx < grid.x; ++bx) {
                Block b(lanes);
                block() = &b;
                const std::function<void(int)> lane = [&](int t) {
                    t_thread = dim3((unsigned)t);
                    t_block = dim3(bx, by, bz);
                    body();
                    for (const PendingCopy& c : pending_copies()) memcpy(c.dst, c.src, (size_t)c.bytes);
                    pending_copies().clear();
                    b.active[t].store(false);            // leaves: no longer expected at any barrier
                    b.wave[t / kWave]->arrive_and_drop();
                    b.all.arrive_and_drop();
                };
                Lanes::get().run(lanes, lane);
                block() = nullptr;
            }
}

inline int lane_in_block() { return (int)t_thread.x; }
inline int lane_in_wave() { return (int)t_thread.x % kWave; }
inline void wave_meet() { block()->wave[lane_in_block() / kWave]->arrive_and_wait(); }

// every active lane of the wave offers `mine`; returns what lane `from` offered, or `inactive` if it has left
inline uint64_t exchange(uint64_t mine, int from, uint64_t inactive) {
    Block& b = *block();
    const int lane = lane_in_block(), w = lane / kWave;
    b.slot[lane] = mine;
    wave_meet();
    const int src = w * kWave + from;
    const uint64_t got = b.active[src].load() ? b.slot[src] : inactive;
    wave_meet();                                         // nobody overwrites a slot that is still being read
    return got;
}

// global_load_lds_dword / _dwordx4: lane L of the wave copies `bytes` bytes from base + offset to LDS address
// lds_base + bytes * L.  The hardware performs the copy some time between the instruction and the s_waitcnt
// vmcnt(n) that leaves at most n later copies outstanding; a kernel is right only if it is right for every such
// time.  Two extremes can be run: at once (default), or as late as the waits allow (MXQ_EMU_COPIES=late in the
// environment): the copy is queued and carried out by the wait that no longer tolerates it.
inline bool copies_land_late() {
    static const bool late = [] {
        const char* e = getenv("MXQ_EMU_COPIES");
        return e != nullptr && strcmp(e, "late") == 0;
    }();
    return late;
}
inline void global_load_lds(int bytes, uint32_t lds_base, uint32_t offset, const unsigned char* base) {
    unsigned char* dst = lds_pointer(lds_base + (uint32_t)(bytes * lane_in_wave()));
    if (copies_land_late()) pending_copies().push_back(PendingCopy{dst, base + offset, bytes});
    else memcpy(dst, base + offset, (size_t)bytes);
}
// s_waitcnt vmcnt(n) (n < 0: the wait does not concern vmcnt): the oldest copies until n are left, then the wave
// meets (its lanes pass a wait together, and the kernels count on that)
inline void wait_for_copies(int n) {
    std::vector<PendingCopy>& q = pending_copies();
    if (n >= 0 && (int)q.size() > n) {
        const size_t done = q.size() - (size_t)n;
        for (size_t i = 0; i < done; ++i) memcpy(q[i].dst, q[i].src, (size_t)q[i].bytes);
        q.erase(q.begin(), q.begin() + (long)done);
    }
    wave_meet();
}

// the arithmetic of the matrix instruction (emu_math.cpp)
void decode_row(const void* const* regs, int groups, int fmt, double* out);
double scaled_dot(const double* a, const double* b, const int* scale_a, const int* scale_b, int groups);

// v_mfma_scale_f32_{32x32x64,16x16x128}_f8f6f4: D = A x B + C with A (rows x K) from the first operand, B
// (K x columns) from the second, K = 64 (32 x 32) or 128 (16 x 16); formats (cbsz / blgp) 0 e4m3, 1 e5m2, 4 e2m1.
// Lane l belongs to row (column) l % DIM and to group g = l / DIM; which K values its registers hold:
// emu_math.cpp.  Its scale register (byte `opsel`) is the E8M0 scale of K block g (32 g .. 32 g + 31) of its row,
// whichever lane holds those values.  It receives column l % DIM, rows 8 (r / 4) + 4 (l / 32) + r % 4 (32 x 32,
// r = 0..15) or 4 (l / 16) + r (16 x 16, r = 0..3).
template <int DIM, class VI, class VF>
VF mfma_scale(const VI& a, const VI& b, const VF& c, int fmt_a, int fmt_b, int opsel_a, int scale_a, int opsel_b,
              int scale_b) {
    Block& blk = *block();
    const int lane = lane_in_block(), w0 = lane / kWave * kWave, l = lane % kWave;
    constexpr int GROUPS = kWave / DIM, KTOT = 32 * GROUPS, NOUT = DIM * DIM / kWave;
    blk.operand[lane][0] = &a;
    blk.operand[lane][1] = &b;
    blk.scale[lane][0] = (scale_a >> (8 * opsel_a)) & 255;
    blk.scale[lane][1] = (scale_b >> (8 * opsel_b)) & 255;
    wave_meet();
    for (int other = w0; other < w0 + kWave; ++other)
        if (!blk.active[other].load()) __builtin_trap();   // the instruction needs the whole wave
    const int j = l % DIM;
    const void* regs[GROUPS];
    double col[KTOT], row[KTOT];
    int scale_col[GROUPS], scale_row[GROUPS];
    for (int g = 0; g < GROUPS; ++g) {
        regs[g] = blk.operand[w0 + j + DIM * g][1];
        scale_col[g] = blk.scale[w0 + j + DIM * g][1];
    }
    decode_row(regs, GROUPS, fmt_b, col);
    VF d = c;
    for (int r = 0; r < NOUT; ++r) {
        const int i = DIM == 32 ? 8 * (r / 4) + 4 * (l / 32) + r % 4 : 4 * (l / 16) + r;
        for (int g = 0; g < GROUPS; ++g) {
            regs[g] = blk.operand[w0 + i + DIM * g][0];
            scale_row[g] = blk.scale[w0 + i + DIM * g][0];
        }
        decode_row(regs, GROUPS, fmt_a, row);
        d[r] = (float)((double)c[r] + scaled_dot(row, col, scale_row, scale_col, GROUPS));
    }
    wave_meet();                                          // operands stay in place until every lane has read them
    return d;
}

}  // namespace emu

#define threadIdx (emu::t_thread)
#define blockIdx (emu::t_block)
#define gridDim (emu::g_grid)
#define blockDim (emu::g_blockdim)

// the overloads HIP puts into the global namespace
inline int max(int a, int b) { return a > b ? a : b; }
inline unsigned max(unsigned a, unsigned b) { return a > b ? a : b; }
inline long max(long a, long b) { return a > b ? a : b; }
inline unsigned long max(unsigned long a, unsigned long b) { return a > b ? a : b; }
inline int min(int a, int b) { return a < b ? a : b; }
inline unsigned min(unsigned a, unsigned b) { return a < b ? a : b; }
inline long min(long a, long b) { return a < b ? a : b; }
inline unsigned long min(unsigned long a, unsigned long b) { return a < b ? a : b; }

inline unsigned __float_as_uint(float f) { return __builtin_bit_cast(unsigned, f); }
inline float __uint_as_float(unsigned u) { return __builtin_bit_cast(float, u); }

inline void __syncthreads() { emu::block()->all.arrive_and_wait(); }

// v_mov_b32_dpp with row_mask = bank_mask = 0xF: quad_perm (ctrl 0x00-0xFF), row_ror:n (0x121-0x12F),
// row_mirror (0x140), row_half_mirror (0x141); a disabled source lane leaves `old` in the destination
// (bound_ctrl false) or 0
inline int emu_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
    const int lane = emu::lane_in_wave();
    int from;
    if (ctrl >= 0 && ctrl <= 0xFF) from = (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);
    else if (ctrl >= 0x121 && ctrl <= 0x12F) from = (lane & ~15) | ((lane + (ctrl & 15)) & 15);
    else if (ctrl == 0x140) from = (lane & ~15) | (15 - (lane & 15));
    else if (ctrl == 0x141) from = (lane & ~7) | (7 - (lane & 7));
    else __builtin_trap();                                // a control this stand-in does not know
    if (row_mask != 0xF || bank_mask != 0xF) __builtin_trap();
    return (int)(uint32_t)emu::exchange((uint32_t)src, from, (uint32_t)(bound_ctrl ? 0 : old));
}
#define __builtin_amdgcn_update_dpp emu_update_dpp

template <class T>
inline T emu_shuffle(T v, int from) {
    static_assert(sizeof(T) <= 8, "exchange slot is 64 bits");
    uint64_t bits = 0;
    memcpy(&bits, &v, sizeof(T));
    const uint64_t got = (from >= 0 && from < emu::kWave) ? emu::exchange(bits, from, bits) : emu::exchange(bits, emu::lane_in_wave(), bits);
    T out;
    memcpy(&out, &got, sizeof(T));
    return out;
}
template <class T>
inline T __shfl_xor(T v, int mask, int width = 64) {
    if (width != 64) __builtin_trap();
    return emu_shuffle(v, emu::lane_in_wave() ^ mask);    // an inactive source: the lane's own value
}
template <class T>
inline T __shfl_down(T v, unsigned delta, int width = 64) {
    if (width != 64) __builtin_trap();
    return emu_shuffle(v, emu::lane_in_wave() + (int)delta);   // past the end of the wave: the lane's own value
}

inline int __all(int pred) {                               // over the lanes of the wave that are still there
    emu::Block& b = *emu::block();
    const int lane = emu::lane_in_block(), w = lane / emu::kWave;
    b.slot[lane] = pred ? 1 : 0;
    emu::wave_meet();
    int all = 1;
    for (int l = w * emu::kWave; l < (w + 1) * emu::kWave; ++l)
        if (b.active[l].load() && b.slot[l] == 0) all = 0;
    emu::wave_meet();
    return all;
}

// v_readfirstlane_b32: the value of the first lane of the wave that is still there
inline int emu_readfirstlane(int v) {
    emu::Block& b = *emu::block();
    const int lane = emu::lane_in_block(), w = lane / emu::kWave;
    b.slot[lane] = (uint32_t)v;
    emu::wave_meet();
    int got = v;
    for (int l = w * emu::kWave; l < (w + 1) * emu::kWave; ++l)
        if (b.active[l].load()) {
            got = (int)(uint32_t)b.slot[l];
            break;
        }
    emu::wave_meet();
    return got;
}
#define __builtin_amdgcn_readfirstlane emu_readfirstlane

// v_exp_f32 / v_rcp_f32: results below the smallest normal number are flushed to zero, as the instructions do
// (accuracy: the C library's instead of the hardware's 1 ulp)
inline float emu_exp2f(float x) {
    const float r = exp2f(x);
    return fabsf(r) < 1.17549435e-38f ? 0.0f : r;
}
inline float emu_rcpf(float x) {
    const float r = 1.0f / x;
    return fabsf(r) < 1.17549435e-38f ? copysignf(0.0f, r) : r;
}
#define __builtin_amdgcn_exp2f emu_exp2f
#define __builtin_amdgcn_rcpf emu_rcpf
#define __builtin_amdgcn_sched_barrier(mask) ((void)0)

// v_permlane16_swap_b32: the first operand of the lanes 16-31 / 48-63 trades places with the second operand of
// the lanes 0-15 / 32-47 (lane L + 16 with lane L)
struct emu_pair {
    unsigned v[2];
    unsigned operator[](int i) const { return v[i]; }
};
inline emu_pair emu_permlane16_swap(unsigned a, unsigned b, bool, bool) {
    const int lane = emu::lane_in_wave();
    const bool upper = (lane & 16) != 0;
    const uint64_t mine = upper ? a : b;                  // what this lane gives away
    const unsigned got = (unsigned)emu::exchange(mine, upper ? lane - 16 : lane + 16, mine);
    return upper ? emu_pair{{got, b}} : emu_pair{{a, got}};
}
#define __builtin_amdgcn_permlane16_swap emu_permlane16_swap

// (object-like macros: the kernels pass braced vectors, whose commas a function-like macro would split)
template <class VI, class VF>
inline VF emu_mfma_32x32x64(const VI& a, const VI& b, const VF& c, int cbsz, int blgp, int opsel_a, int scale_a, int opsel_b,
                            int scale_b) {
    return emu::mfma_scale<32>(a, b, c, cbsz, blgp, opsel_a, scale_a, opsel_b, scale_b);
}
template <class VI, class VF>
inline VF emu_mfma_16x16x128(const VI& a, const VI& b, const VF& c, int cbsz, int blgp, int opsel_a, int scale_a, int opsel_b,
                             int scale_b) {
    return emu::mfma_scale<16>(a, b, c, cbsz, blgp, opsel_a, scale_a, opsel_b, scale_b);
}
#define __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4 emu_mfma_32x32x64
#define __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4 emu_mfma_16x16x128
