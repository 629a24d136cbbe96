// Shared plumbing of the C-ABI library: error reporting, the per-process stream and
// small launch helpers.  Everything here is host side.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/lten_hip.h"

namespace lten_hip {

// Thread-local message behind lten_hip_last_error(); l-ten itself prints and throws
// (l-ten/error.h:78-93), which a C ABI cannot do.
void set_error(const char* fmt, ...);
void set_kernel_name(const char* name);
hipStream_t stream();
bool capturing();  // a launch graph is being recorded: no allocation, no synchronisation

// Tuning / test switches behind lten_hip_set_option.
enum Option { OPT_QGEMM_TILE = 0, OPT_SGEMM_TILE, OPT_QSKINNY, OPT_CONV_VARIANT, OPT_QGEMM_SPLIT, OPT_COUNT };
int get_option(Option o);

// Device memory the library owns for what does not fit its entry points' workspaces (padded copies of int8 operands,
// partial sums of a reduction split over workgroups): one block per device, grown when a call needs more (never while
// a launch graph is being recorded: nullptr then, and when there is no memory), kept until the process ends.  One
// stream uses it at a time, as everything else in this library.
void* library_scratch(uint64_t bytes);
// While one of these lives, the caller promises that every row of the operands it passes to the GEMM entry points can be
// read up to its leading dimension, the last row included (BLAS only guarantees the row itself): the direct-to-LDS
// tiles then take row-contiguous operands whose row count is no multiple of 4.
struct RowsReadableToPitch {
	RowsReadableToPitch();
	~RowsReadableToPitch();
};
bool rows_readable_to_pitch();
// For a caller that keeps data in the first `bytes` of what library_scratch handed it across a call into another entry
// point of the library: while one of these lives, library_scratch hands out only what the block has behind those bytes
// and never moves it.  They nest: a callee that was itself handed the part behind a holder's bytes holds from there on.
struct LibraryScratchHold {
	explicit LibraryScratchHold(uint64_t bytes);
	~LibraryScratchHold();
	LibraryScratchHold(const LibraryScratchHold&) = delete;
	LibraryScratchHold& operator=(const LibraryScratchHold&) = delete;

private:
	bool outer_held_;
	uint64_t outer_bytes_;
};

// Looks up the current device's copy of the static scratch of lten_hip_fcq_forward_static (qgemm.hip); 0 on success.
int prepare_static_scratch();

inline uint64_t ceil_div(uint64_t a, uint64_t b) { return (a + b - 1) / b; }

}  // namespace lten_hip

#define LTEN_HIP_CHECK(expr)                                                                     \
	do {                                                                                     \
		hipError_t e_ = (expr);                                                          \
		if (e_ != hipSuccess) {                                                          \
			lten_hip::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
			return 1;                                                                \
		}                                                                                \
	} while (0)

#define LTEN_HIP_REQUIRE(cond, ...)                                                              \
	do {                                                                                     \
		if (!(cond)) {                                                                   \
			lten_hip::set_error(__VA_ARGS__);                                        \
			return 2;                                                                \
		}                                                                                \
	} while (0)

// After a kernel launch: surface launch-configuration errors immediately.
#define LTEN_HIP_LAUNCH_CHECK() LTEN_HIP_CHECK(hipGetLastError())
