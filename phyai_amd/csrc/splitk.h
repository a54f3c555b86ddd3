// Cross-workgroup split-K reduction without cache-wide fences.
//
// An MI355X has eight XCDs, each with its own L2; a device-scope fence makes a
// workgroup write back / invalidate that whole L2 and costs microseconds when a
// few hundred workgroups do it.  Instead every access to data that crosses
// workgroups (partial sums, arrival counters) is a relaxed device-scope atomic:
// stores are written through to memory, loads never hit a stale L2 line, and no
// fence wider than the workgroup is issued.
//
// Why the last arriver sees every partial sum (gfx950 only; this is an argument about that
// hardware, not about the HIP memory model, under which relaxed atomics order nothing):
//  1. A relaxed agent-scope atomic store is a write-through store (sc1 set): it does not stay
//     in the issuing XCD's L2 but goes to the memory side, the coherence point of all XCDs.
//     The AMDGPU memory model's own agent-scope release on this target is "write back the L2's
//     dirty lines, then s_waitcnt vmcnt(0), then the releasing store"; nothing here is ever
//     dirty in L2, so the write-back has nothing to do and is left out.
//  2. vmcnt counts stores as well as loads on this target and a store leaves the count when
//     the memory side has acknowledged it: after wait_own_stores() (s_waitcnt vmcnt(0), an
//     asm statement with a memory clobber, so the compiler moves no access across it) every
//     store of that lane is visible device-wide.
//  3. __syncthreads() in splitk_arrive() is a workgroup-scope release + s_barrier + acquire:
//     every lane of the workgroup has passed step 2 before thread 0 goes on, and the compiler
//     keeps the counter update behind it.
//  4. Only then does thread 0 add to the tile's counter, an atomic executed at the memory side:
//     the adds of the S splits are totally ordered there, and the one that reads S - 1 was
//     issued after the partial sums of all S splits were acknowledged.
//  5. The gathering workgroup's loads are relaxed agent-scope atomic loads (sc1): they are
//     served from the memory side, never from a line its own L2 might hold, and they are issued
//     after the second barrier of splitk_arrive(), i.e. after the counter value was read.
// The same reasoning covers the reset: the gatherer stores 0 to the counter after its loads have
// returned (their values feed the epilogue), and the next call that touches the counter is a later
// kernel on the same stream or graph, ordered behind this one by the queue.
// tests/test_gpu_parity.py runs split-K shapes repeatedly against one fixed result (and under graph
// replay and from two streams) to catch a toolchain or target change that breaks an assumption.
//
// Partials are summed by the last workgroup to arrive, in split order, so the
// result does not depend on arrival order.  That workgroup also resets the
// counter, which is how the workspace header stays zero from call to call.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace phyai {

__device__ __forceinline__ void coherent_store2(float* p, float a, float b) {
    uint64_t v = (uint64_t)__float_as_uint(a) | ((uint64_t)__float_as_uint(b) << 32);
    __hip_atomic_store(reinterpret_cast<uint64_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void coherent_load2(const float* p, float& a, float& b) {
    uint64_t v = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
    a = __uint_as_float((uint32_t)v);
    b = __uint_as_float((uint32_t)(v >> 32));
}

__device__ __forceinline__ void wait_own_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// FRAG floats per thread (even), THREADS threads.  Layout of one partial:
// [FRAG/2][THREADS][2] floats, so that a wavefront's 64-bit accesses are contiguous.
// The *_part forms move CHUNK of the FRAG floats, elements e0 .. e0+CHUNK-1, so that a thread with
// a large fragment never holds more than a chunk of it outside its accumulators.
template <int FRAG, int THREADS, int CHUNK>
__device__ __forceinline__ void splitk_publish_part(float* partials, int tile, int S, int z, int e0, const float* frag) {
    float* mine = partials + ((size_t)tile * S + z) * (size_t)(FRAG * THREADS);
#pragma unroll
    for (int e = 0; e < CHUNK; e += 2)
        coherent_store2(mine + (((e0 + e) / 2) * THREADS + threadIdx.x) * 2, frag[e], frag[e + 1]);
}

template <int FRAG, int THREADS>
__device__ __forceinline__ void splitk_publish(float* partials, int tile, int S, int z, const float* frag) {
    splitk_publish_part<FRAG, THREADS, FRAG>(partials, tile, S, z, 0, frag);
    wait_own_stores();
}

// Returns true in every lane of the workgroup that arrived last.  Must be called by all
// threads, after splitk_publish (or the last splitk_publish_part and wait_own_stores).
__device__ __forceinline__ bool splitk_arrive(int* counters, int tile, int S, int* s_flag) {
    __syncthreads();
    if (threadIdx.x == 0) {
        const int old = __hip_atomic_fetch_add(counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_flag = (old == S - 1);
    }
    __syncthreads();
    return *s_flag != 0;
}

// A tile split in two, the other way round: arrive first, publish only if nobody was there.  The first of the two
// workgroups to arrive (it finds 0) writes its partial sums, waits for its stores (wait_own_stores) and then tells so
// with splitk_published(); the second (it finds 1, or 3 if the first has told already) writes nothing: it waits
// until the first has told, reads that half and adds it to the accumulators it still holds.  Half of the partial
// sums are never written.  The first workgroup runs to its end without waiting for anyone, so the second cannot
// wait for ever; its spin is bounded all the same (giving up would add a half that is not there yet: wrong
// numbers, never a hang).  The argument above carries over: the first workgroup's stores are acknowledged by the
// memory side before its second add to the counter, and the second workgroup's loads are issued after it has read
// a counter value that contains that add.
__device__ __forceinline__ int splitk_arrive_early(int* counters, int tile, int* s_flag) {
    __syncthreads();   // (nobody reads operands from LDS any more: a word of it serves as the flag)
    if (threadIdx.x == 0)
        *s_flag = __hip_atomic_fetch_add(counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    return *s_flag;
}

// All threads of the first workgroup, each after wait_own_stores().
__device__ __forceinline__ void splitk_published(int* counters, int tile) {
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_fetch_add(counters + tile, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// All threads of the second workgroup; `found` is what splitk_arrive_early returned.
__device__ __forceinline__ void splitk_await_published(int* counters, int tile, int found) {
    if (found == 1 && threadIdx.x == 0) {
        for (int spin = 0; spin < (1 << 22); ++spin) {
            if (__hip_atomic_load(counters + tile, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= 4) break;
            __builtin_amdgcn_s_sleep(8);
        }
    }
    __syncthreads();
}

// Sum of elements e0 .. e0+CHUNK-1 over the S partials of a tile, in split order.  The loads of
// two partials are in flight together: every batch of loads is a round trip to memory, and the
// round trips, not the bytes, are what the gathering workgroup waits for.
template <int FRAG, int THREADS, int CHUNK>
__device__ __forceinline__ void splitk_gather_part(const float* partials, int tile, int S, int e0, float* frag) {
    const float* all = partials + (size_t)tile * S * (size_t)(FRAG * THREADS);
#pragma unroll
    for (int e = 0; e < CHUNK; ++e) frag[e] = 0.f;
    for (int z = 0; z < S; z += 2) {
        const bool pair = z + 1 < S;   // uniform over the workgroup
        const float* p0 = all + (size_t)z * (FRAG * THREADS);
        const float* p1 = p0 + (pair ? FRAG * THREADS : 0);
        float t0[CHUNK], t1[CHUNK];
#pragma unroll
        for (int e = 0; e < CHUNK; e += 2) {
            coherent_load2(p0 + (((e0 + e) / 2) * THREADS + threadIdx.x) * 2, t0[e], t0[e + 1]);
            coherent_load2(p1 + (((e0 + e) / 2) * THREADS + threadIdx.x) * 2, t1[e], t1[e + 1]);
        }
#pragma unroll
        for (int e = 0; e < CHUNK; ++e) frag[e] += t0[e];
        if (pair) {
#pragma unroll
            for (int e = 0; e < CHUNK; ++e) frag[e] += t1[e];
        }
    }
}

// Elements e0 .. e0+CHUNK-1 of ONE split's partial (for a tile split in two, whose last arriver still holds its
// own half in registers: own + other is the sum in split order whichever half is its own, since a + b = b + a and
// the sum of the general form starts from 0 + a = a).
template <int FRAG, int THREADS, int CHUNK>
__device__ __forceinline__ void splitk_load_part(const float* partials, int tile, int S, int z, int e0, float* frag) {
    const float* one = partials + ((size_t)tile * S + z) * (size_t)(FRAG * THREADS);
#pragma unroll
    for (int e = 0; e < CHUNK; e += 2)
        coherent_load2(one + (((e0 + e) / 2) * THREADS + threadIdx.x) * 2, frag[e], frag[e + 1]);
}

// The gathering workgroup puts the tile's counter back to zero for the next call.
__device__ __forceinline__ void splitk_reset(int* counters, int tile) {
    if (threadIdx.x == 0)
        __hip_atomic_store(counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int FRAG, int THREADS>
__device__ __forceinline__ void splitk_gather(const float* partials, int* counters, int tile, int S, float* frag) {
    splitk_gather_part<FRAG, THREADS, FRAG>(partials, tile, S, 0, frag);
    splitk_reset(counters, tile);
}

}  // namespace phyai
