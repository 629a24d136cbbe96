// Direct global -> LDS loads and the wait that goes with them, shared by the int8 and fp32 tile kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

namespace lten_hip {

// One wave-wide 16-byte-per-lane load straight into LDS: lane L's bytes go to lds_addr + 16*L.
// lds_addr and base are wave-uniform; voff is the lane's byte offset from base.
// m0 is not named as a clobber: the backend treats it as a reserved register (naming it draws the warning that
// reserved registers on a clobber list are not preserved anyway), never keeps a value in it across statements and
// writes it itself immediately before each instruction of its own that reads it.
__device__ __forceinline__ void async_load16(uint32_t lds_addr, const void* base, uint32_t voff)
{
	asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

// The 4-byte form: lane L's dword goes to lds_addr + 4*L.  For operands whose rows do not start on 16-byte boundaries.
__device__ __forceinline__ void async_load4(uint32_t lds_addr, const void* base, uint32_t voff)
{
	asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

// The same for the lanes of `mask` only, without a branch: a taken branch costs a wavefront that is alone on its
// SIMD far more than the load (its MFMA stream stops while instructions are fetched again).  The execution mask is
// saved and put back inside the statement, so the compiler never sees it change; lanes that are inactive on entry
// stay out whatever `mask` says.
__device__ __forceinline__ void async_load16_masked(uint64_t mask, uint32_t lds_addr, const void* base, uint32_t voff)
{
	uint64_t saved;
	asm volatile("s_mov_b64 %0, exec\n\ts_and_b64 exec, %0, %1\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %4\n\ts_mov_b64 exec, %0"
	             : "=&s"(saved) : "s"(mask), "s"(lds_addr), "v"(voff), "s"(base) : "memory", "scc");
}

// The same with the non-temporal hint: for data that is read once (a weight stream) and should not displace what the
// caches hold.
__device__ __forceinline__ void async_load16_masked_nt(uint64_t mask, uint32_t lds_addr, const void* base, uint32_t voff)
{
	uint64_t saved;
	asm volatile("s_mov_b64 %0, exec\n\ts_and_b64 exec, %0, %1\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %4 nt\n\ts_mov_b64 exec, %0"
	             : "=&s"(saved) : "s"(mask), "s"(lds_addr), "v"(voff), "s"(base) : "memory", "scc");
}

// 16 bytes of zeros to LDS byte address lds_lane_addr (per lane) for the lanes of `mask`, without a branch; same
// handling of the execution mask.  `zero` is a register quadruple holding zeros.
typedef float lds_v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void lds_zero16_masked(uint64_t mask, uint32_t lds_lane_addr, lds_v4f zero)
{
	uint64_t saved;
	asm volatile("s_mov_b64 %0, exec\n\ts_and_b64 exec, %0, %1\n\tds_write_b128 %2, %3\n\ts_mov_b64 exec, %0"
	             : "=&s"(saved) : "s"(mask), "v"(lds_lane_addr), "v"(zero) : "memory", "scc");
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
