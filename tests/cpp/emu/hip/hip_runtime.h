// Stand-in for <hip/hip_runtime.h> that lets the device code of csrc/ run on the CPU, one workgroup at a time with one
// host thread per lane, so that host sanitizers see the kernel bodies.  Only what kernels.hpp and gl.hpp use is here.
//   __shared__ objects become statics (workgroups run one after the other), __syncthreads is a barrier over the
//   workgroup's threads, and the wavefront-wide operations (DPP, shuffles) are rendezvous of the 64 threads of a
//   wavefront: every lane must arrive, as the hardware operations need every lane enabled.
#pragma once
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>

#define __host__
#define __device__
#define __global__
#define __forceinline__ inline __attribute__((always_inline))
#define __shared__ static
#define __launch_bounds__(...)

struct dim3 {
    unsigned x = 1, y = 1, z = 1;
    dim3(unsigned a = 1, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {}
};
struct uint4 {
    unsigned x, y, z, w;
};

namespace emu {
constexpr int WAVE = 64, MAX_THREADS = 1024;
struct Barrier {
    std::mutex m;
    std::condition_variable cv;
    int n = 0, count = 0;
    unsigned long gen = 0;
    void reset(int parties) { n = parties, count = 0; }
    void wait()
    {
        std::unique_lock<std::mutex> lk(m);
        const unsigned long g = gen;
        if (++count == n) {
            count = 0;
            gen++;
            cv.notify_all();
        } else {
            // a lane that never arrives would be a kernel bug (an operation that needs the whole wavefront reached by a part of it)
            if (!cv.wait_for(lk, std::chrono::seconds(20), [&] { return gen != g; })) {
                fprintf(stderr, "emu: a barrier or wavefront-wide operation was not reached by every lane\n");
                abort();
            }
        }
    }
};
// what the threads of one workgroup share.  Kernels whose LDS is all dynamic (none of the __shared__ statics above) can
// have several workgroups running at once, each with a context of its own.
struct Group {
    Barrier block_barrier;
    Barrier wave_barrier[MAX_THREADS / WAVE];
    uint64_t xchg[MAX_THREADS];
    uint64_t *dyn = nullptr;  // dynamic LDS
    void reset(int threads)
    {
        block_barrier.reset(threads);
        for (int w = 0; w < threads / WAVE; w++) wave_barrier[w].reset(WAVE);
    }
};
inline Group default_group;
inline thread_local Group *group = &default_group;
inline uint64_t *dyn_lds() { return group->dyn; }
}  // namespace emu

inline thread_local dim3 threadIdx, blockIdx;
inline dim3 gridDim, blockDim;

inline void __syncthreads() { emu::group->block_barrier.wait(); }
inline unsigned long long atomicAdd(unsigned long long *p, unsigned long long v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }

namespace emu {
// value of `v` in lane `src` of the caller's wavefront (every lane of the wavefront calls this together)
inline uint64_t lane_read(uint64_t v, int src)
{
    const int t = (int)threadIdx.x, w = t / WAVE;
    Group &g = *group;
    g.xchg[t] = v;
    g.wave_barrier[w].wait();
    const uint64_t r = g.xchg[w * WAVE + src];
    g.wave_barrier[w].wait();
    return r;
}
// v_mov_b32 with a DPP control, as __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl) of gfx9:
// the controls used by the block reduction.  A lane whose row is not in row_mask keeps `old`.
inline int update_dpp(int old, int src, int ctrl, int row_mask, int /*bank_mask*/, bool bound_ctrl)
{
    const int lane = (int)threadIdx.x % WAVE, row = lane / 16, in_row = lane % 16;
    int from = -1;  // source lane, -1: none
    if (ctrl >= 0 && ctrl <= 0xFF) {
        from = (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);  // quad_perm
    } else if (ctrl == 0x140) {
        from = row * 16 + (15 - in_row);  // row_mirror
    } else if (ctrl == 0x141) {
        from = row * 16 + (in_row < 8 ? 7 - in_row : 23 - in_row);  // row_half_mirror
    } else if (ctrl == 0x142) {
        from = row >= 1 ? (row - 1) * 16 + 15 : -1;  // row_bcast:15, lane 15 of each row to the next row
    } else if (ctrl == 0x143) {
        from = row >= 2 ? 31 : -1;  // row_bcast:31, lane 31 to rows 2 and 3
    } else {
        fprintf(stderr, "emu: DPP control %#x not modelled\n", ctrl);
        abort();
    }
    const uint64_t got = lane_read((uint32_t)src, from < 0 ? lane : from);
    if (!((row_mask >> row) & 1)) return old;
    if (from < 0) return bound_ctrl ? 0 : old;
    return (int)(uint32_t)got;
}
}  // namespace emu

#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) emu::update_dpp(old, src, ctrl, rm, bm, bc)
// (uniform by construction where the kernels use it; a lane alone cannot check that here)
#define __builtin_amdgcn_readfirstlane(x) (x)
// the device's real-time counter: 100 MHz
inline uint64_t wall_clock64()
{
    return (uint64_t)(std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count() / 10);
}
#define __builtin_amdgcn_fence(order, scope) std::atomic_thread_fence(std::memory_order_seq_cst)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
// (a polling lane gives the other host threads a turn: a workgroup here is hundreds of threads on a few cores)
#define __builtin_amdgcn_s_sleep(x) std::this_thread::yield()
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __HIP_MEMORY_SCOPE_SYSTEM 0
#define __hip_atomic_load(p, order, scope) __atomic_load_n(p, __ATOMIC_SEQ_CST)
#define __hip_atomic_store(p, v, order, scope) __atomic_store_n(p, v, __ATOMIC_SEQ_CST)
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST)
template <class T>
inline T __shfl_xor(T v, int mask, int /*width*/)
{
    return (T)emu::lane_read((uint64_t)v, ((int)threadIdx.x % emu::WAVE) ^ mask);
}
template <class T>
inline T __shfl(T v, int lane, int /*width*/)
{
    return (T)emu::lane_read((uint64_t)v, lane);
}
