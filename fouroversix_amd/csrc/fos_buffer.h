// Buffer-instruction helpers shared by the streaming quantize kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fos_device.h"

namespace fos {

// Buffer resource (V#) over [base, base + bytes): raw 32-bit byte offsets, out-of-range
// loads return zero.
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
FOS_DEVICE BufferRsrc make_rsrc(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

// Cache-policy operand of the buffer stores that write a kernel's bulk output: non-temporal.  The
// output is not read again by the kernel, and lines left dirty in L2 are written back while the next
// kernel of the stream is already reading (the pass-1 scan that followed a quantize launch took 24.4 us
// with plain stores and 22.9 us with these), and they displace what the previous kernel left there.
#ifndef FOS_ST_AUX
#define FOS_ST_AUX 2
#endif
constexpr int kStreamStore = FOS_ST_AUX;  // bit 1 = nt

// The same policy for plain global stores (use where one instruction of a wavefront writes whole lines).
FOS_DEVICE void stream_store(uint4 *dst, const uint4 &v) {
    const u32x4 w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, reinterpret_cast<u32x4 *>(dst));
}
FOS_DEVICE void stream_store(uint32_t *dst, uint32_t v) { __builtin_nontemporal_store(v, dst); }

// A wave-uniform 64-bit value, spelled so that the compiler keeps it in scalar registers (a
// descriptor it believes to differ between lanes makes every buffer access a loop over lanes).
FOS_DEVICE uint64_t uniform64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

}  // namespace fos
