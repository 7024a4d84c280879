// Asynchronous HBM -> LDS copies of gfx950 (buffer_load ... lds) and the hand-managed wait on them.
#pragma once

#include <hip/hip_runtime.h>

namespace tfcc_rocm {

typedef int lds_dma_v4i __attribute__((ext_vector_type(4)));

// Buffer descriptor in scalar registers: base, 0 stride, size in bytes, raw 32-bit format.
__device__ __forceinline__ lds_dma_v4i make_rsrc(const void* base, unsigned bytes) {
  const unsigned long long a = reinterpret_cast<unsigned long long>(base);
  lds_dma_v4i r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)a);
  r[1] = __builtin_amdgcn_readfirstlane((int)((unsigned)(a >> 32) & 0xffffu));
  r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
  r[3] = 0x00020000;
  return r;
}

// Cache-policy bits appended to the copy instructions (" sc0", " sc1", " nt" or a combination); empty = default.
#ifndef TFCC_LDS_DMA_CACHE_BITS
#define TFCC_LDS_DMA_CACHE_BITS ""
#endif

// One asynchronous 16-byte-per-lane copy HBM -> LDS.  The LDS address of lane i is ldsBase + 16*i
// (ldsBase wave-uniform, goes through M0); voffset is the lane's byte offset into the buffer.
// Inline asm on purpose: the outstanding-copy count is managed by hand (s_waitcnt vmcnt) so that
// several slabs stay in flight across iterations.
__device__ __forceinline__ void dma16(lds_dma_v4i rsrc, unsigned ldsBase, unsigned voffset) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(ldsBase), "v"(voffset), "s"(rsrc)
               : "memory", "m0");
}

// The same copy with a scalar byte offset on top of the lane's (the buffer's range check sees the lane offset
// only) and the LDS address already in a scalar register.
__device__ __forceinline__ void dma16s(lds_dma_v4i rsrc, unsigned ldsAddr, unsigned voffset, unsigned soffset) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen" TFCC_LDS_DMA_CACHE_BITS " lds"
               :
               : "s"(ldsAddr), "v"(voffset), "s"(rsrc), "s"(soffset)
               : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // s_waitcnt simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]; leave the others at max
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
}


}  // namespace tfcc_rocm
