// A stand-in for <hip/hip_runtime.h> that lets the HIP sources of this package's *quantizer* translation
// unit (mxq_kernels.h, mxq_capi.hip) be compiled for the host and executed there, for tests on machines
// without a GPU.  A kernel launch runs the workgroups one after another; the 256 lanes of a workgroup are
// 256 host threads (kept for the life of the process) that meet where the hardware's lanes exchange data or wait for each other:
// __syncthreads (all 256), and the lane exchanges of a wave of 64 (DPP, __shfl_xor, __all).  A lane that
// has left the kernel counts as inactive: it no longer takes part in barriers, and an exchange that would
// read from it returns what the instruction returns for a disabled lane.  Nothing here knows about MFMA,
// LDS copies or inline assembly: the GEMM and row kernels cannot be run this way.
#pragma once
#include <stdint.h>
#include <string.h>

#include <atomic>
#include <barrier>
#include <condition_variable>
#include <functional>
#include <mutex>
#include <thread>

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
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "no error"; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void** p, const void* symbol) { *p = const_cast<void*>(symbol); return hipSuccess; }

namespace emu {

constexpr int kLanes = 256, kWave = 64;
struct Block {
    std::barrier<> all{kLanes};
    std::barrier<> wave[kLanes / kWave] = {std::barrier<>(kWave), std::barrier<>(kWave), std::barrier<>(kWave),
                                           std::barrier<>(kWave)};
    uint64_t slot[kLanes];                   // what a lane offers in an exchange
    std::atomic<bool> active[kLanes];
};
inline Block*& block() { static Block* b = nullptr; return b; }
inline thread_local dim3 t_thread, t_block;
inline dim3 g_grid, g_blockdim;

// 256 threads that live as long as the process; a workgroup is one job for each of them
class Lanes {
  public:
    static Lanes& get() {
        static Lanes* pool = new Lanes;      // never destroyed: its threads wait on it until the process ends
        return *pool;
    }
    void run(const std::function<void(int)>& job) {
        std::unique_lock<std::mutex> lock(m_);
        job_ = &job;
        pending_ = kLanes;
        ++generation_;
        start_.notify_all();
        done_.wait(lock, [&] { return pending_ == 0; });
        job_ = nullptr;
    }

  private:
    Lanes() {
        for (int t = 0; t < kLanes; ++t) std::thread([this, t] { work(t); }).detach();
    }
    void work(int t) {
        uint64_t seen = 0;
        for (;;) {
            const std::function<void(int)>* job;
            {
                std::unique_lock<std::mutex> lock(m_);
                start_.wait(lock, [&] { return generation_ != seen; });
                seen = generation_;
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
    int pending_ = 0;
};

// the workgroups of a launch one after another, each on the 256 lane threads
template <class Body>
void launch(dim3 grid, const Body& body) {
    static std::mutex one_launch_at_a_time;
    std::lock_guard<std::mutex> guard(one_launch_at_a_time);
    g_grid = grid;
    g_blockdim = dim3(kLanes);
    for (unsigned by = 0; by < grid.y; ++by)
        for (unsigned bx = 0; bx < grid.x; ++bx) {
            Block b;
            for (auto& a : b.active) a.store(true);
            block() = &b;
            const std::function<void(int)> lane = [&](int t) {
                t_thread = dim3((unsigned)t);
                t_block = dim3(bx, by);
                body();
                b.active[t].store(false);                // leaves: no longer expected at any barrier
                b.wave[t / kWave].arrive_and_drop();
                b.all.arrive_and_drop();
            };
            Lanes::get().run(lane);
            block() = nullptr;
        }
}

// every active lane of the wave offers `mine`; returns what lane `from` offered, or `inactive` if it has left
inline uint64_t exchange(uint64_t mine, int from, uint64_t inactive) {
    Block& b = *block();
    const int lane = (int)t_thread.x, w = lane / kWave;
    b.slot[lane] = mine;
    b.wave[w].arrive_and_wait();
    const int src = w * kWave + from;
    const uint64_t got = b.active[src].load() ? b.slot[src] : inactive;
    b.wave[w].arrive_and_wait();                        // nobody overwrites a slot that is still being read
    return got;
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

inline void __syncthreads() { emu::block()->all.arrive_and_wait(); }

// v_mov_b32_dpp with row_mask = bank_mask = 0xF: quad_perm (ctrl 0x00-0xFF), row_mirror (0x140),
// row_half_mirror (0x141); a disabled source lane leaves `old` in the destination (bound_ctrl false) or 0
inline int emu_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
    const int lane = (int)emu::t_thread.x % emu::kWave;
    int from;
    if (ctrl >= 0 && ctrl <= 0xFF) from = (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);
    else if (ctrl == 0x140) from = (lane & ~15) | (15 - (lane & 15));
    else if (ctrl == 0x141) from = (lane & ~7) | (7 - (lane & 7));
    else __builtin_trap();                                // a control this stand-in does not know
    if (row_mask != 0xF || bank_mask != 0xF) __builtin_trap();
    return (int)(uint32_t)emu::exchange((uint32_t)src, from, (uint32_t)(bound_ctrl ? 0 : old));
}
#define __builtin_amdgcn_update_dpp emu_update_dpp

template <class T>
inline T __shfl_xor(T v, int mask, int width = 64) {
    if (width != 64) __builtin_trap();
    static_assert(sizeof(T) <= 8, "exchange slot is 64 bits");
    uint64_t bits = 0;
    memcpy(&bits, &v, sizeof(T));
    const int lane = (int)emu::t_thread.x % emu::kWave;
    const uint64_t got = emu::exchange(bits, lane ^ mask, bits);   // an inactive source: the lane's own value
    T out;
    memcpy(&out, &got, sizeof(T));
    return out;
}

inline int __all(int pred) {                               // over the lanes of the wave that are still there
    emu::Block& b = *emu::block();
    const int lane = (int)emu::t_thread.x, w = lane / emu::kWave;
    b.slot[lane] = pred ? 1 : 0;
    b.wave[w].arrive_and_wait();
    int all = 1;
    for (int l = w * emu::kWave; l < (w + 1) * emu::kWave; ++l)
        if (b.active[l].load() && b.slot[l] == 0) all = 0;
    b.wave[w].arrive_and_wait();
    return all;
}
