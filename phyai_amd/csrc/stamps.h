// Time stamps inside the GEMM kernels, for the debug build only.
//
// `make stamps` compiles the library a second time with -DPHYAI_FP8_STAMPS into
// ../lib/libphyai_fp8_stamps.so.  In that build every wavefront of the pipelined tile kernel and of the
// one-launch small-M kernel records the shader clock (s_memtime) at a few points of its life and, when it ends,
// writes them as one record of kStampSlots 64-bit words into the buffer that phyai_fp8_debug_stamps() named.
// Arithmetic and memory traffic of the kernels are otherwise unchanged (the outputs are bit-identical, which a
// test checks); the stamps cost a scalar memory instruction each and a few scalar registers, so the stamped
// kernels run a few per cent slower than the production ones.  In the normal build the macros are empty.
//
// Record layout (64-bit words): [0 .. kStampSlots - 3] shader-clock stamps, what each one marks is the kernel's
// business (see the PHYAI_STAMP lines there); [kStampSlots - 2], [kStampSlots - 1] the 100 MHz counter
// (s_memrealtime) at entry and at the end, which gives the shader clock the kernel ran at.  A stamp that a
// kernel does not take stays 0.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace phyai {
constexpr int kStampSlots = 12;
struct StampSink {
    unsigned long long* buf;   // kStampSlots words per wavefront record
    unsigned int capacity;     // records
};
}  // namespace phyai

#ifdef PHYAI_FP8_STAMPS
// one sink per translation unit (no relocatable device code); set through launch_set_stamp_sink_*()
#define PHYAI_STAMP_SINK(name) static __device__ phyai::StampSink name;
#define PHYAI_STAMP_BEGIN                                                                        \
    unsigned long long stamp_t_[phyai::kStampSlots] = {};                                        \
    stamp_t_[phyai::kStampSlots - 2] = __builtin_amdgcn_s_memrealtime();                         \
    stamp_t_[0] = __builtin_readcyclecounter();
#define PHYAI_STAMP(i) stamp_t_[i] = __builtin_readcyclecounter();
// record: this wavefront's index among all wavefronts of the launch
#define PHYAI_STAMP_END(sink, record, lane)                                                      \
    {                                                                                            \
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* the wavefront's stores are through */ \
        stamp_t_[phyai::kStampSlots - 3] = __builtin_readcyclecounter();                         \
        stamp_t_[phyai::kStampSlots - 1] = __builtin_amdgcn_s_memrealtime();                     \
        const phyai::StampSink s_ = sink;                                                        \
        if (s_.buf != nullptr && (lane) == 0 && (unsigned)(record) < s_.capacity) {              \
            _Pragma("unroll") for (int i_ = 0; i_ < phyai::kStampSlots; ++i_)                    \
                s_.buf[(size_t)(record) * phyai::kStampSlots + i_] = stamp_t_[i_];               \
        }                                                                                        \
    }
#else
#define PHYAI_STAMP_SINK(name)
#define PHYAI_STAMP_BEGIN
#define PHYAI_STAMP(i)
#define PHYAI_STAMP_END(sink, record, lane)
#endif
