// Direct global -> LDS loads and the wait that goes with them, shared by the int8 and fp32 tile kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

namespace lten_hip {

// One wave-wide 16-byte-per-lane load straight into LDS: lane L's bytes go to lds_addr + 16*L.
// lds_addr and base are wave-uniform; voff is the lane's byte offset from base.
__device__ __forceinline__ void async_load16(uint32_t lds_addr, const void* base, uint32_t voff)
{
	asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

// s_waitcnt vmcnt(n) only (expcnt and lgkmcnt fields left at "no wait"); n < 64.
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
	static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
	__builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// s_waitcnt vmcnt(n) lgkmcnt(0): also every LDS operation of this wavefront has completed; n = 63 leaves vmcnt alone.
template <int N>
__device__ __forceinline__ void wait_vmcnt_lgkm0()
{
	static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
	__builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (0 << 8));
}

}  // namespace lten_hip
