// Context, memory, fill and event entry points of the C ABI (the HIP counterparts of
// l-ten/utils.cu and of gpu_fill in l-ten/math_fns.cu).
#include "common.h"

#include <cstring>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace lten_hip {

static thread_local char g_error[512] = "";
static thread_local char g_kernel[96] = "";
static hipStream_t g_stream = nullptr;
static int g_device = -1;

// Graph capture: the stream the capture runs on (the caller's, or one made here when the library is on the
// null stream, which cannot be captured) and the stream to go back to afterwards.
static hipStream_t g_capture_stream = nullptr;
static hipStream_t g_stream_before_capture = nullptr;
static bool g_capturing = false;
struct RecordedGraph {  // what a handle of lten_hip_graph_end points to
	hipGraph_t graph;
	hipGraphExec_t exec;
};

void set_error(const char* fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(g_error, sizeof(g_error), fmt, ap);
	va_end(ap);
}

void set_kernel_name(const char* name)
{
	strncpy(g_kernel, name, sizeof(g_kernel) - 1);
	g_kernel[sizeof(g_kernel) - 1] = 0;
}

hipStream_t stream() { return g_stream; }
bool capturing() { return g_capturing; }

// (work queued on the stream may still read the old block when it has to grow, hence the wait)
struct LibraryScratch {
	void* base;
	uint64_t bytes;
	bool recorded;  // a launch graph holds this block's address: it is never freed
};
static LibraryScratch g_scratch[8] = {};

static int g_rows_readable = 0;
RowsReadableToPitch::RowsReadableToPitch() { g_rows_readable++; }
RowsReadableToPitch::~RowsReadableToPitch() { g_rows_readable--; }
bool rows_readable_to_pitch() { return g_rows_readable > 0; }

static bool g_scratch_held = false;
static uint64_t g_scratch_held_bytes = 0;
LibraryScratchHold::LibraryScratchHold(uint64_t bytes) : outer_held_(g_scratch_held), outer_bytes_(g_scratch_held_bytes)
{
	g_scratch_held_bytes = (outer_held_ ? outer_bytes_ : 0) + ((bytes + 255) & ~255ull);
	g_scratch_held = true;
}
LibraryScratchHold::~LibraryScratchHold()
{
	g_scratch_held = outer_held_;
	g_scratch_held_bytes = outer_bytes_;
}

void* library_scratch(uint64_t bytes)
{
	int dev = -1;
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 8) return nullptr;
	LibraryScratch& ls = g_scratch[dev];
	// held: only what the block has left behind the holder's part, and the block stays where it is
	if (g_scratch_held) return (ls.base != nullptr && g_scratch_held_bytes + bytes <= ls.bytes) ? static_cast<char*>(ls.base) + g_scratch_held_bytes : nullptr;
	if (ls.bytes >= bytes) {
		if (capturing()) ls.recorded = true;
		return ls.base;
	}
	if (capturing()) return nullptr;
	if (ls.base != nullptr) {
		if (hipStreamSynchronize(stream()) != hipSuccess) return nullptr;
		// a block whose address a recorded graph replays stays allocated for the rest of the process; any other is freed
		if (!ls.recorded) (void)hipFree(ls.base);
		ls.base = nullptr;
		ls.bytes = 0;
		ls.recorded = false;
	}
	const uint64_t want = (bytes + (bytes >> 2) + (2u << 20)) & ~((2ull << 20) - 1);  // a quarter more, whole 2 MB pages
	void* ptr = nullptr;
	if (hipMalloc(&ptr, want) != hipSuccess) {
		(void)hipGetLastError();
		return nullptr;
	}
	ls.base = ptr;
	ls.bytes = want;
	return ls.base;
}

static int g_options[OPT_COUNT] = { 0 };
static const char* const g_option_names[OPT_COUNT] = { "qgemm_tile", "sgemm_tile", "qskinny", "conv_variant", "qgemm_split" };
int get_option(Option o) { return g_options[o]; }

// Device memory pool behind lten_hip_alloc / lten_hip_free, the counterpart of l-ten's MemoryPool for GPU buffers
// (l-ten/utils.cu:30-47 with USE_MEMORYPOOL, l-ten/memorypool.h:142-173): sizes are rounded up to a power of two (to a
// multiple of 64 MB above that), freed blocks are kept per size and handed out again, so that a layer's forward pass,
// which allocates its result tensor on every call, does not pay a hipMalloc each time.  Blocks are reused without any
// wait: safe for work issued in order on the library's stream, which is the only order this library creates, and
// lten_hip_set_stream waits for the stream it leaves, so that a block freed while work was pending there cannot be
// handed to work on the next stream before that work is done.  At most POOL_CACHE_LIMIT bytes stay cached; beyond
// that a freed block goes back to the driver, and lten_hip_pool_release returns everything cached.
constexpr uint64_t POOL_CACHE_LIMIT = 16ull << 30;
static std::mutex g_pool_mutex;
static std::map<uint64_t, std::vector<void*>> g_pool_free;  // rounded size -> cached blocks
static std::unordered_map<void*, uint64_t> g_pool_size;     // every block handed out or cached -> its rounded size, bit 0 set while cached
static uint64_t g_pool_cached = 0;

static uint64_t pool_round(uint64_t size)
{
	if (size <= 256) return 256;
	if (size > (64ull << 20)) return (size + (64ull << 20) - 1) / (64ull << 20) * (64ull << 20);
	uint64_t r = 256;
	while (r < size) r <<= 1;
	return r;
}

// Everything the pool holds (cached or handed out) comes from hipMalloc; this gives the cached part back.
static int pool_drop_cached()
{
	std::vector<void*> drop;
	{
		std::lock_guard<std::mutex> lock(g_pool_mutex);
		for (auto& kv : g_pool_free) {
			for (void* q : kv.second) { drop.push_back(q); g_pool_size.erase(q); }
			kv.second.clear();
		}
		g_pool_cached = 0;
	}
	for (void* q : drop) (void)hipFree(q);  // hipFree waits for the device: no pending work loses its memory
	return 0;
}

template <typename T>
__global__ void fill_kernel(T* p, uint64_t n, T v)
{
	uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
	uint64_t step = (uint64_t)gridDim.x * blockDim.x;
	for (; i < n; i += step) p[i] = v;
}

template <typename T>
static int fill(T* p, uint64_t n, T v)
{
	if (n == 0) return 0;
	LTEN_HIP_REQUIRE(p != nullptr, "fill: null pointer");
	uint64_t blocks = ceil_div(n, 256);
	if (blocks > 4096) blocks = 4096;
	fill_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, stream()>>>(p, n, v);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip

using namespace lten_hip;

extern "C" {

int lten_hip_init(int device)
{
	int count = 0;
	LTEN_HIP_CHECK(hipGetDeviceCount(&count));
	LTEN_HIP_REQUIRE(device >= 0 && device < count, "lten_hip_init: device %d out of range (%d devices)", device, count);
	LTEN_HIP_CHECK(hipSetDevice(device));
	hipDeviceProp_t prop;
	LTEN_HIP_CHECK(hipGetDeviceProperties(&prop, device));
	LTEN_HIP_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0,
	                 "lten_hip_init: device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
	g_device = device;
	return prepare_static_scratch();
}

const char* lten_hip_last_error(void) { return g_error; }
const char* lten_hip_last_kernel(void) { return g_kernel; }

int lten_hip_get_device(int* device)
{
	LTEN_HIP_REQUIRE(device != nullptr, "lten_hip_get_device: null pointer");
	LTEN_HIP_CHECK(hipGetDevice(device));
	return 0;
}

// What a recording cannot hold: allocation, freeing, host copies and waits.  They fail with a message of their own
// while a launch graph is being recorded (the runtime would otherwise invalidate the capture with a generic one).
#define LTEN_HIP_NOT_WHILE_RECORDING(name) \
	LTEN_HIP_REQUIRE(!capturing(), name ": not allowed between lten_hip_graph_begin and lten_hip_graph_end")

int lten_hip_set_stream(void* hip_stream)
{
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_set_stream");
	hipStream_t next = static_cast<hipStream_t>(hip_stream);
	if (next == g_stream) return 0;
	// Work still pending on the stream being left may use blocks that lten_hip_free has put back into the pool; the
	// next lten_hip_alloc could hand them to work on the new stream, which is not ordered behind it.  Waiting here
	// once keeps the pool free of per-block events.
	LTEN_HIP_CHECK(hipStreamSynchronize(g_stream));
	g_stream = next;
	return 0;
}

int lten_hip_sync(void)
{
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_sync");
	LTEN_HIP_CHECK(hipStreamSynchronize(stream()));
	return 0;
}

int lten_hip_alloc(void** device_ptr, uint64_t size, int zero_memory)
{
	LTEN_HIP_REQUIRE(device_ptr != nullptr, "lten_hip_alloc: null pointer");
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_alloc");
	*device_ptr = nullptr;
	const uint64_t rounded = pool_round(size);
	{
		std::lock_guard<std::mutex> lock(g_pool_mutex);
		auto it = g_pool_free.find(rounded);
		if (it != g_pool_free.end() && !it->second.empty()) {
			*device_ptr = it->second.back();
			it->second.pop_back();
			g_pool_cached -= rounded;
			g_pool_size[*device_ptr] = rounded;
		}
	}
	if (*device_ptr == nullptr) {
		hipError_t e = hipMalloc(device_ptr, rounded);
		if (e != hipSuccess) {
			// out of memory with blocks cached: give them back and try once more
			(void)hipGetLastError();
			pool_drop_cached();
			LTEN_HIP_CHECK(hipMalloc(device_ptr, rounded));
		}
		std::lock_guard<std::mutex> lock(g_pool_mutex);
		g_pool_size[*device_ptr] = rounded;
	}
	if (zero_memory && size) return lten_hip_zero(*device_ptr, size);  // a fill kernel, stream ordered
	return 0;
}

int lten_hip_pool_release(void)
{
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_pool_release");
	return pool_drop_cached();
}

int lten_hip_free(void* device_ptr)
{
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_free");
	if (device_ptr == nullptr) return 0;
	{
		std::lock_guard<std::mutex> lock(g_pool_mutex);
		auto it = g_pool_size.find(device_ptr);
		LTEN_HIP_REQUIRE(it == g_pool_size.end() || (it->second & 1) == 0, "lten_hip_free: %p was freed already", device_ptr);
		if (it != g_pool_size.end() && g_pool_cached + it->second <= POOL_CACHE_LIMIT) {
			g_pool_free[it->second].push_back(device_ptr);
			g_pool_cached += it->second;
			it->second |= 1;
			return 0;
		}
		if (it != g_pool_size.end()) g_pool_size.erase(it);
	}
	LTEN_HIP_CHECK(hipFree(device_ptr));  // memory that did not come from lten_hip_alloc, or a full cache
	return 0;
}

int lten_hip_zero(void* device_ptr, size_t size)
{
	if (size == 0) return 0;
	LTEN_HIP_REQUIRE(device_ptr != nullptr, "lten_hip_zero: null pointer");
	// A fill kernel rather than hipMemsetAsync, so that callers may capture this call
	// into a HIP graph.
	if ((reinterpret_cast<uintptr_t>(device_ptr) & 3) == 0 && (size & 3) == 0)
		return fill<int32_t>(static_cast<int32_t*>(device_ptr), size / 4, 0);
	return fill<uint8_t>(static_cast<uint8_t*>(device_ptr), size, 0);
}

int lten_hip_copy_to_gpu(void* device_dst, const void* host_src, size_t size)
{
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_copy_to_gpu");
	if (size == 0) return 0;
	LTEN_HIP_CHECK(hipMemcpyAsync(device_dst, host_src, size, hipMemcpyHostToDevice, stream()));
	LTEN_HIP_CHECK(hipStreamSynchronize(stream()));
	return 0;
}

int lten_hip_copy_from_gpu(void* host_dst, const void* device_src, size_t size)
{
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_copy_from_gpu");
	if (size == 0) return 0;
	LTEN_HIP_CHECK(hipMemcpyAsync(host_dst, device_src, size, hipMemcpyDeviceToHost, stream()));
	LTEN_HIP_CHECK(hipStreamSynchronize(stream()));
	return 0;
}

int lten_hip_copy_gpu_to_gpu(void* device_dst, const void* device_src, size_t size)
{
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_copy_gpu_to_gpu");
	if (size == 0) return 0;
	LTEN_HIP_CHECK(hipMemcpyAsync(device_dst, device_src, size, hipMemcpyDeviceToDevice, stream()));
	return 0;
}

int lten_hip_fill_f32(float* p, uint64_t n, float v) { return fill<float>(p, n, v); }
int lten_hip_fill_i32(int32_t* p, uint64_t n, int32_t v) { return fill<int32_t>(p, n, v); }
int lten_hip_fill_u8(uint8_t* p, uint64_t n, uint8_t v) { return fill<uint8_t>(p, n, v); }

int lten_hip_set_option(const char* name, int value)
{
	LTEN_HIP_REQUIRE(name != nullptr, "lten_hip_set_option: null name");
	for (int i = 0; i < OPT_COUNT; i++)
		if (strcmp(name, g_option_names[i]) == 0) {
			g_options[i] = value;
			return 0;
		}
	set_error("lten_hip_set_option: unknown option '%s'", name);
	return 2;
}

int lten_hip_graph_begin(void)
{
	LTEN_HIP_REQUIRE(!g_capturing, "lten_hip_graph_begin: a capture is already open");
	g_stream_before_capture = g_stream;
	if (g_stream == nullptr) {
		if (g_capture_stream == nullptr) LTEN_HIP_CHECK(hipStreamCreate(&g_capture_stream));
		LTEN_HIP_CHECK(hipStreamSynchronize(nullptr));  // earlier work on the null stream comes first
		g_stream = g_capture_stream;
	}
	hipError_t e = hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal);
	if (e != hipSuccess) {
		g_stream = g_stream_before_capture;
		set_error("lten_hip_graph_begin: %s", hipGetErrorString(e));
		return 1;
	}
	g_capturing = true;
	return 0;
}

int lten_hip_graph_end(void** graph)
{
	LTEN_HIP_REQUIRE(graph != nullptr, "lten_hip_graph_end: null pointer");
	LTEN_HIP_REQUIRE(g_capturing, "lten_hip_graph_end: no capture is open");
	*graph = nullptr;
	hipGraph_t captured = nullptr;
	const hipError_t e = hipStreamEndCapture(g_stream, &captured);
	g_stream = g_stream_before_capture;
	g_capturing = false;
	if (e != hipSuccess || captured == nullptr) {
		(void)hipGetLastError();
		set_error("lten_hip_graph_end: the capture failed (%s); only compute entry points may run between begin and end",
		          hipGetErrorString(e));
		return 1;
	}
	hipGraphExec_t exec = nullptr;
	const hipError_t ei = hipGraphInstantiate(&exec, captured, nullptr, nullptr, 0);
	if (ei != hipSuccess) {
		(void)hipGraphDestroy(captured);
		set_error("lten_hip_graph_end: hipGraphInstantiate: %s", hipGetErrorString(ei));
		return 1;
	}
	// The handle owns both objects until lten_hip_graph_destroy: the executable graph is specified to be independent
	// of the graph it was instantiated from, but nothing is gained by destroying that one early.
	*graph = new RecordedGraph{ captured, exec };
	return 0;
}

int lten_hip_graph_launch(void* graph)
{
	LTEN_HIP_REQUIRE(graph != nullptr, "lten_hip_graph_launch: null graph");
	LTEN_HIP_REQUIRE(!g_capturing, "lten_hip_graph_launch: a capture is open");
	LTEN_HIP_CHECK(hipGraphLaunch(static_cast<RecordedGraph*>(graph)->exec, stream()));
	return 0;
}

int lten_hip_graph_destroy(void* graph)
{
	if (graph == nullptr) return 0;
	RecordedGraph* g = static_cast<RecordedGraph*>(graph);
	// replays may still be running: the objects go only once the stream they were launched on is idle
	LTEN_HIP_CHECK(hipStreamSynchronize(stream()));
	const hipError_t e0 = hipGraphExecDestroy(g->exec), e1 = hipGraphDestroy(g->graph);
	delete g;
	LTEN_HIP_CHECK(e0);
	LTEN_HIP_CHECK(e1);
	return 0;
}

int lten_hip_event_create(void** event)
{
	LTEN_HIP_REQUIRE(event != nullptr, "lten_hip_event_create: null pointer");
	hipEvent_t e;
	LTEN_HIP_CHECK(hipEventCreate(&e));
	*event = e;
	return 0;
}

int lten_hip_event_record(void* event)
{
	LTEN_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), stream()));
	return 0;
}

int lten_hip_event_elapsed_ms(void* start, void* stop, float* ms)
{
	LTEN_HIP_NOT_WHILE_RECORDING("lten_hip_event_elapsed_ms");
	LTEN_HIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
	LTEN_HIP_CHECK(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
	return 0;
}

int lten_hip_event_destroy(void* event)
{
	LTEN_HIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(event)));
	return 0;
}

}  // extern "C"
